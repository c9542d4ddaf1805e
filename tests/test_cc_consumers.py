"""The two boundaries driven from outside Python.

tests/cc/muladd.cc is a framework-side consumer of include/dvm.h (the C++ graph API of the reference's include/dvm.h,
used the way its examples/cc/muladd.cc:57-75 uses it, plus late binding, dynamic shapes and the error contract); it
links libdvm.so. tests/cc/device_blob.cc drives libdvm_hip.so alone through include/dvm_hip.h with a program blob from
tests/golden/. Both are built by dvm_amd.build (g++, no HIP toolchain needed) and run here as child processes."""
import json
import os
import subprocess

import pytest

from dvm_amd import build as dvm_build

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")


def _binary(name):
    src, out, cmd = dvm_build.consumer_test_command(name)
    if not os.path.exists(out):  # normally built beforehand by dvm_amd.build.build()
        os.makedirs(os.path.dirname(out), exist_ok=True)
        subprocess.run(cmd, check=True)
    return out


def test_consumer_sources_compile_against_the_public_headers(tmp_path):
    for name in dvm_build.CONSUMER_TESTS:
        src, out, cmd = dvm_build.consumer_test_command(name)
        cmd = [str(tmp_path / name) if c == out else c for c in cmd]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr


def test_blob_fixture_is_what_the_host_compiler_emits_today():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_blob_fixture", os.path.join(GOLDEN, "make_blob_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    blob, geometry, _ = mod.build()
    with open(os.path.join(GOLDEN, "blob_muladd_fp32.bin"), "rb") as f:
        committed = f.read()
    meta = json.load(open(os.path.join(GOLDEN, "blob_muladd_fp32.json")))
    assert len(committed) == 4096 and meta["elements"] == mod.N
    assert (meta["threads"], meta["lds_bytes"]) == (geometry[1], geometry[2])
    assert blob == committed, "the bytecode changed: run python tests/golden/make_blob_fixture.py"


def test_makefile_runs_the_commands_of_the_python_build():
    # the make-style entry (DVM_ARCH=hip) compiles every source dvm_amd.build compiles, with the same flags, into the
    # same objects: compare the command lines of a dry run from scratch
    repo = os.path.dirname(HERE)
    r = subprocess.run(["make", "-n", "-B", "all", "consumers"], cwd=repo, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.splitlines() if l.startswith(("hipcc", "g++"))]
    compiled = sorted(l.split(" -c ")[1].split(" -o ")[0] + (" u4" if "-DDVM_VEC_U=4" in l else "") for l in lines if " -c " in l)
    want = sorted(os.path.relpath(s, repo) for s in dvm_build._sources("device", ".hip") + dvm_build._sources("host", ".cc"))
    want = sorted(want + ["dvm_amd/csrc/device/vm_vector.hip u4"])
    assert compiled == want
    for flag in dvm_build.HIP_FLAGS:
        assert all(flag in l for l in lines if l.startswith("hipcc") and " -c " in l), flag
    for flag in dvm_build.HOST_FLAGS:
        assert all(flag in l for l in lines if l.startswith("g++") and " -c " in l), flag
    r = subprocess.run(["make", "-n", "DVM_ARCH=gpu"], cwd=repo, capture_output=True, text=True)
    assert r.returncode != 0 and "hip" in r.stderr


@pytest.mark.gpu
def test_cpp_consumer_of_dvm_h():
    r = subprocess.run([_binary("muladd")], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and r.stdout.strip().endswith("PASS"), (r.returncode, r.stdout, r.stderr)


@pytest.mark.gpu
def test_device_layer_alone_runs_a_program_blob():
    meta = json.load(open(os.path.join(GOLDEN, "blob_muladd_fp32.json")))
    cmd = [_binary("device_blob"), os.path.join(GOLDEN, "blob_muladd_fp32.bin"), str(meta["workgroups"]), str(meta["threads"]),
           str(meta["lds_bytes"]), str(meta["elements"])]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and r.stdout.strip().endswith("PASS"), (r.returncode, r.stdout, r.stderr)
