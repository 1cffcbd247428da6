# Builds the TenniS reference CPU library straight from its sources where they
# lie (REF, default /root/reference) -- no cmake, nothing copied, no stand-ins.
# Outputs go only to oracle/_ref/.  This is TEST INFRASTRUCTURE (the parity
# checker and the timed CPU baseline), never part of the shipped product path.
#
# Flags mirror the reference's own haswell/OpenMP build:
#   CMakeLists.txt:8,15 (BUILDING_TENNIS, TS_DISABLE_PARALLEL), :206-213 (OpenMP),
#   :331-336 (TS_USE_SIMD/AVX/FMA), cmake/FLAGS_GCC.cmake (-O3 -std=c++11
#   -fvisibility=hidden -fPIC), cmake/tools.cmake (-mavx -mavx2 -mfma).
# Source set = CMakeLists.txt:158-173,290-316 (modules + kernels/{common,cpu}).
REF  ?= /root/reference
HERE := $(dir $(abspath $(lastword $(MAKEFILE_LIST))))
OUT  := $(HERE)_ref
OBJ  := $(OUT)/obj

MODULES := api backend board compiler core encryption engine frontend global memory module runtime utils
SRCS := $(foreach m,$(MODULES),$(shell find $(REF)/src/$(m) -name '*.cpp' 2>/dev/null)) \
        $(shell find $(REF)/src/kernels/common $(REF)/src/kernels/cpu -name '*.cpp' 2>/dev/null)
OBJS := $(patsubst $(REF)/src/%.cpp,$(OBJ)/%.o,$(SRCS))

DEFS := -DBUILDING_TENNIS -DTS_SOLUTION_DIR=\"$(REF)\" -DTS_DISABLE_PARALLEL \
        -DTS_USE_PROFILER -DTS_USE_HOOK -DTS_USE_DEBUG_API -DTS_USE_OPENMP \
        -DTS_USE_SIMD -DTS_USE_AVX -DTS_USE_FMA
CXXFLAGS := -O3 -std=c++11 -fvisibility=hidden -fPIC -fopenmp -mavx -mavx2 -mfma \
            -w -I$(REF)/include -I$(REF)/src $(DEFS)

all: lib driver
lib: $(OUT)/libtennis_ref.so
driver: $(OUT)/libref_driver.so

$(OBJ)/%.o: $(REF)/src/%.cpp
	@mkdir -p $(dir $@)
	$(CXX) $(CXXFLAGS) -c $< -o $@

$(OUT)/libtennis_ref.so: $(OBJS)
	@echo LINK $@
	@$(CXX) -shared -fopenmp -o $@ $(OBJS) -lpthread -lm

# Thin extern "C" driver (this repo's own code) over the reference's operators.
$(OUT)/libref_driver.so: $(HERE)ref_driver.cpp $(OUT)/libtennis_ref.so
	$(CXX) $(CXXFLAGS) -fvisibility=default -shared -o $@ $< -L$(OUT) -ltennis_ref -Wl,-rpath,'$$ORIGIN'

# The "hip" device backend of this repository compiled against the REAL TenniS headers and built
# INTO the library, the way TenniS builds its own device backends (src/kernels/gpu is part of
# libtennis; the base operator classes are not exported, so a backend cannot live outside it):
# libtennis_hip.so = the reference objects above + tennis_amd/backend/hip/*.cpp, and a second copy
# of the driver linked to it.  Used to run this repository's operators inside TenniS's own
# Workbench next to TenniS's CPU operators.  Needs tennis_amd/lib/libtsx_hip.so
# (python -m tennis_amd.build) and hipcc for the HIP runtime headers.
HIPCC   ?= /opt/rocm/bin/hipcc
REPO    := $(abspath $(HERE)..)
HIPDIR  := $(REPO)/tennis_amd/backend/hip
HIPOBJS := $(OBJ)/hip/hip_device.o $(OBJ)/hip/hip_ops_quantized.o $(OBJ)/hip/hip_ops_float.o $(OBJ)/hip/hip_ops_glue.o $(OBJ)/hip/hip_ops_v2.o $(OBJ)/hip/hip_ops_fused.o $(OBJ)/hip/hip_zipper_option.o
intree: $(OUT)/libtennis_hip.so $(OUT)/libref_driver_hip.so

$(OBJ)/hip/%.o: $(HIPDIR)/%.cpp $(wildcard $(HIPDIR)/*.h) $(REPO)/include/tsx_hip.h
	@mkdir -p $(dir $@)
	$(HIPCC) -x c++ -O2 -std=c++17 -fPIC -fvisibility=hidden -w -c -D__HIP_PLATFORM_AMD__ -DTSX_WITH_TENNIS $(DEFS) \
	    -mavx2 -mfma -I$(REPO)/include -I/opt/rocm/include -I$(REF)/include -I$(REF)/src $< -o $@

$(OUT)/libtennis_hip.so: $(OBJS) $(HIPOBJS) $(REPO)/tennis_amd/lib/libtsx_hip.so
	@echo LINK $@
	@$(CXX) -shared -fopenmp -Wl,-Bsymbolic -o $@ $(OBJS) $(HIPOBJS) -L$(REPO)/tennis_amd/lib -ltsx_hip \
	    -L/opt/rocm/lib -lamdhip64 -lpthread -lm -Wl,-rpath,'$$ORIGIN/../../tennis_amd/lib' -Wl,-rpath,/opt/rocm/lib

$(OUT)/libref_driver_hip.so: $(HERE)ref_driver.cpp $(OUT)/libtennis_hip.so
	$(CXX) $(CXXFLAGS) -fvisibility=default -shared -Wl,-Bsymbolic -o $@ $< -L$(OUT) -ltennis_hip -Wl,-rpath,'$$ORIGIN'

clean:
	rm -rf $(OUT)
.PHONY: all lib driver intree clean
