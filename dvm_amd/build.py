"""Builds the native libraries of the package in-tree.

  dvm_amd/lib/libdvm_hip.so  device layer: HIP interpreter kernels + C ABI (include/dvm_hip.h), hipcc, gfx950
  dvm_amd/lib/libdvm.so      host library: dvm::Kernel API (include/dvm.h) + flat C ABI (include/dvm_c.h), g++

Run as `python -m dvm_amd.build` (add --force to rebuild everything).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
LIB = os.path.join(ROOT, "lib")
OBJ = os.path.join(LIB, "obj")

# The interpreter kernels branch on wave-uniform values only (every per-lane condition lives in an
# out-of-line helper), so the CFG structurizer is told to leave uniform regions alone: the
# dispatch then compiles to real scalar branches instead of a chain of predicate checks.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-mllvm", "-structurizecfg-skip-uniform-regions=true",
             "-mllvm", "-structurizecfg-relaxed-uniform-regions=true"]
HOST_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-fvisibility=hidden", "-Wall"]


def _sources(sub, ext):
    d = os.path.join(CSRC, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(ext))


def _deps():
    out = [os.path.join(CSRC, "isa_gfx950.h")]
    inc = os.path.join(os.path.dirname(ROOT), "include")
    out += [os.path.join(inc, f) for f in os.listdir(inc)]
    out += _sources("host", ".h") + _sources("device", ".h")
    return out


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), err))
    return err


def build(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    deps = _deps()
    jobs = []
    dev_objs, host_objs = [], []
    for src in _sources("device", ".hip"):
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        dev_objs.append(obj)
        if force or _stale(obj, [src] + deps):
            jobs.append(["hipcc"] + HIP_FLAGS + ["-c", src, "-o", obj])
        if os.path.basename(src) == "vm_vector.hip":
            # second build of the vector VM: four slabs per lane per instruction (kernels dvm_vm_vec_*_u4)
            obj4 = os.path.join(OBJ, "vm_vector_u4.hip.o")
            dev_objs.append(obj4)
            if force or _stale(obj4, [src] + deps):
                jobs.append(["hipcc"] + HIP_FLAGS + ["-DDVM_VEC_U=4", "-c", src, "-o", obj4])
    for src in _sources("host", ".cc"):
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        host_objs.append(obj)
        if force or _stale(obj, [src] + deps):
            jobs.append(["g++"] + HOST_FLAGS + ["-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for msg in ex.map(_run, jobs):
            if verbose and msg:
                print(msg)
    hip_so = os.path.join(LIB, "libdvm_hip.so")
    host_so = os.path.join(LIB, "libdvm.so")
    if force or _stale(hip_so, dev_objs):
        _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC"] + dev_objs + ["-o", hip_so])
    if force or _stale(host_so, host_objs):
        _run(["g++", "-shared", "-fPIC"] + host_objs + ["-o", host_so, "-ldl", "-lpthread"])
    build_consumer_tests(force)
    return hip_so, host_so


CONSUMER_TESTS = {"muladd": ["-ldvm", "-ldvm_hip"], "device_blob": ["-ldvm_hip"]}


def consumer_test_command(name):
    """g++ line for tests/cc/<name>.cc: a program outside the package that sees only include/*.h (and the bytecode
    header, for the blob test) and links the built libraries."""
    repo = os.path.dirname(ROOT)
    src = os.path.join(repo, "tests", "cc", name + ".cc")
    out = os.path.join(LIB, "tests", name)
    rocm_lib = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")
    return src, out, (["g++", "-std=c++17", "-O1", "-Wall", "-I" + os.path.join(repo, "include"), "-I" + CSRC, src, "-o", out,
                       "-L" + LIB] + CONSUMER_TESTS[name] + ["-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath-link," + rocm_lib])


def build_consumer_tests(force=False):
    os.makedirs(os.path.join(LIB, "tests"), exist_ok=True)
    for name in CONSUMER_TESTS:
        src, out, cmd = consumer_test_command(name)
        if os.path.exists(src) and (force or _stale(out, [src, os.path.join(LIB, "libdvm.so"), os.path.join(LIB, "libdvm_hip.so")] + _deps())):
            _run(cmd)


if __name__ == "__main__":
    so = build(force="--force" in sys.argv, verbose=True)
    print("built", so)
