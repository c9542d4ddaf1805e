# make-style entry for the native libraries (the same commands as `python -m dvm_amd.build`):
#   make                 dvm_amd/lib/libdvm_hip.so (device layer, hipcc, gfx950) and dvm_amd/lib/libdvm.so (host library, g++)
#   make consumers       the C++ programs of tests/cc against include/*.h and the two libraries
#   make oracle          the CPU oracle of the tests (oracle/libdvm_oracle.so)
#   make asan=1          the host library again with AddressSanitizer and UndefinedBehaviorSanitizer, into dvm_amd/lib/asan/
#                        (the reference's switch, Makefile:66-68). The host compiler writes offsets into fixed 4 KB
#                        blobs; `make asan-check` runs the CPU tests and four thousand random graphs in disassembly
#                        mode against that library (DVM_HOST_LIBRARY names it, the sanitizer runtime is preloaded).
#   make clean
# DVM_ARCH names the device layer, as in the reference's Makefile (DVM_ARCH=gpu|npu there, Makefile:3-15); the only
# one here is hip.
DVM_ARCH ?= hip
ifneq ($(DVM_ARCH),hip)
$(error DVM_ARCH=$(DVM_ARCH): this tree builds the hip (gfx950) device layer only)
endif

HIPCC ?= hipcc
CXX ?= g++
ROCM_PATH ?= /opt/rocm
GFX ?= gfx950

CSRC := dvm_amd/csrc
LIB := dvm_amd/lib
OBJ := $(LIB)/obj

# uniform regions are left to scalar branches: the interpreter loops branch on wave-uniform values only
ifneq ($(asan),)
SAN_DIR := /asan
SAN_FLAGS := -fsanitize=address,undefined -fno-sanitize-recover=undefined -fno-omit-frame-pointer -g
endif

HIP_FLAGS := --offload-arch=$(GFX) -O3 -fPIC -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
             -mllvm -structurizecfg-skip-uniform-regions=true -mllvm -structurizecfg-relaxed-uniform-regions=true
HOST_FLAGS := -std=c++17 $(if $(asan),-O1,-O2) -fPIC -fvisibility=hidden -Wall $(SAN_FLAGS)

DEV_SRC := $(sort $(wildcard $(CSRC)/device/*.hip))
HOST_SRC := $(sort $(wildcard $(CSRC)/host/*.cc))
HEADERS := $(CSRC)/isa_gfx950.h $(wildcard include/*.h) $(wildcard $(CSRC)/host/*.h) $(wildcard $(CSRC)/device/*.h)
DEV_OBJ := $(patsubst $(CSRC)/device/%.hip,$(OBJ)/%.hip.o,$(DEV_SRC)) $(OBJ)/vm_vector_u4.hip.o
HOST_OBJ := $(patsubst $(CSRC)/host/%.cc,$(OBJ)$(SAN_DIR)/%.cc.o,$(HOST_SRC))

.PHONY: all consumers oracle clean asan-check
ifneq ($(asan),)
all: $(LIB)/asan/libdvm.so
else
all: $(LIB)/libdvm_hip.so $(LIB)/libdvm.so
endif

$(OBJ):
	mkdir -p $(OBJ) $(LIB)/tests

$(OBJ)/%.hip.o: $(CSRC)/device/%.hip $(HEADERS) | $(OBJ)
	$(HIPCC) $(HIP_FLAGS) -c $< -o $@

# second build of the vector VM: four slabs per lane per instruction (kernels dvm_vm_vec_*_u4)
$(OBJ)/vm_vector_u4.hip.o: $(CSRC)/device/vm_vector.hip $(HEADERS) | $(OBJ)
	$(HIPCC) $(HIP_FLAGS) -DDVM_VEC_U=4 -c $< -o $@

$(OBJ)$(SAN_DIR)/%.cc.o: $(CSRC)/host/%.cc $(HEADERS) | $(OBJ)
	@mkdir -p $(dir $@)
	$(CXX) $(HOST_FLAGS) -c $< -o $@

$(LIB)/libdvm_hip.so: $(DEV_OBJ)
	$(HIPCC) --offload-arch=$(GFX) -shared -fPIC $(DEV_OBJ) -o $@

$(LIB)$(SAN_DIR)/libdvm.so: $(HOST_OBJ)
	@mkdir -p $(dir $@)
	$(CXX) -shared -fPIC $(SAN_FLAGS) $(HOST_OBJ) -o $@ -ldl -lpthread

# the CPU tests (the device layer is not needed for them) and the random graphs of tests/random_graphs.py, compiled in
# disassembly mode, against the sanitizer build; any report ends the run with an error
asan-check:
	$(MAKE) asan=1 all
	LD_PRELOAD="$$($(CXX) -print-file-name=libasan.so):$$($(CXX) -print-file-name=libubsan.so):$$LD_PRELOAD" \
	ASAN_OPTIONS=detect_leaks=0:abort_on_error=1 UBSAN_OPTIONS=halt_on_error=1:print_stacktrace=1 \
	DVM_HOST_LIBRARY=$(abspath $(LIB)/asan/libdvm.so) python3 -m pytest tests -q -m "not gpu" -p no:cacheprovider
	LD_PRELOAD="$$($(CXX) -print-file-name=libasan.so):$$($(CXX) -print-file-name=libubsan.so):$$LD_PRELOAD" \
	ASAN_OPTIONS=detect_leaks=0:abort_on_error=1 UBSAN_OPTIONS=halt_on_error=1:print_stacktrace=1 \
	DVM_HOST_LIBRARY=$(abspath $(LIB)/asan/libdvm.so) python3 -m tests.random_graphs --das-seeds 1000

CONSUMER_LINK := -L$(LIB) -Wl,-rpath,'$$ORIGIN/..' -Wl,-rpath-link,$(ROCM_PATH)/lib
consumers: $(LIB)/tests/muladd $(LIB)/tests/device_blob
$(LIB)/tests/muladd: tests/cc/muladd.cc $(LIB)/libdvm.so $(LIB)/libdvm_hip.so $(HEADERS)
	$(CXX) -std=c++17 -O1 -Wall -Iinclude -I$(CSRC) $< -o $@ $(CONSUMER_LINK) -ldvm -ldvm_hip
$(LIB)/tests/device_blob: tests/cc/device_blob.cc $(LIB)/libdvm_hip.so $(HEADERS)
	$(CXX) -std=c++17 -O1 -Wall -Iinclude -I$(CSRC) $< -o $@ $(CONSUMER_LINK) -ldvm_hip

oracle:
	$(MAKE) -C oracle

clean:
	rm -rf $(OBJ) $(LIB)/libdvm_hip.so $(LIB)/libdvm.so $(LIB)/tests
