# TenniS with this repository's "hip" device backend built INTO it, the way TenniS builds its own device
# backends (src/kernels/gpu is part of libtennis; the base operator classes are not exported, so a backend cannot
# live outside the library):
#   libtennis_hip.so        = TenniS's sources, compiled where they lie (REF, default /root/reference; no cmake,
#                             nothing copied) + tennis_amd/backend/hip/*.cpp, linked to tennis_amd/lib/libtsx_hip.so
#   libtennis_hip_driver.so = intree_driver.cpp: extern "C" access to that library's Workbench for Python
# Both go to tennis_amd/lib/intree/.  Flags mirror the reference's haswell/OpenMP build: CMakeLists.txt:8,15
# (BUILDING_TENNIS, TS_DISABLE_PARALLEL), :206-213 (OpenMP), :331-336 (TS_USE_SIMD/AVX/FMA), cmake/FLAGS_GCC.cmake
# (-O3 -std=c++11 -fvisibility=hidden -fPIC), cmake/tools.cmake (-mavx -mavx2 -mfma); source set =
# CMakeLists.txt:158-173,290-316 (modules + kernels/{common,cpu}).  Needs tennis_amd/lib/libtsx_hip.so
# (python -m tennis_amd.build) and hipcc for the HIP runtime headers.
REF   ?= /root/reference
HIPCC ?= /opt/rocm/bin/hipcc
HERE  := $(dir $(abspath $(lastword $(MAKEFILE_LIST))))
REPO  := $(abspath $(HERE)../../..)
OUT   := $(REPO)/tennis_amd/lib/intree
OBJ   := $(OUT)/obj
HIPDIR := $(REPO)/tennis_amd/backend/hip

MODULES := api backend board compiler core encryption engine frontend global memory module runtime utils
SRCS := $(foreach m,$(MODULES),$(shell find $(REF)/src/$(m) -name '*.cpp' 2>/dev/null)) \
        $(shell find $(REF)/src/kernels/common $(REF)/src/kernels/cpu -name '*.cpp' 2>/dev/null)
OBJS := $(patsubst $(REF)/src/%.cpp,$(OBJ)/%.o,$(SRCS))
HIPOBJS := $(patsubst $(HIPDIR)/%.cpp,$(OBJ)/hip/%.o,$(wildcard $(HIPDIR)/*.cpp))

DEFS := -DBUILDING_TENNIS -DTS_SOLUTION_DIR=\"$(REF)\" -DTS_DISABLE_PARALLEL \
        -DTS_USE_PROFILER -DTS_USE_HOOK -DTS_USE_DEBUG_API -DTS_USE_OPENMP \
        -DTS_USE_SIMD -DTS_USE_AVX -DTS_USE_FMA
CXXFLAGS := -O3 -std=c++11 -fvisibility=hidden -fPIC -fopenmp -mavx -mavx2 -mfma \
            -w -I$(REF)/include -I$(REF)/src $(DEFS)

all: $(OUT)/libtennis_hip.so $(OUT)/libtennis_hip_driver.so

$(OBJ)/%.o: $(REF)/src/%.cpp
	@mkdir -p $(dir $@)
	$(CXX) $(CXXFLAGS) -c $< -o $@

$(OBJ)/hip/%.o: $(HIPDIR)/%.cpp $(wildcard $(HIPDIR)/*.h) $(REPO)/include/tsx_hip.h
	@mkdir -p $(dir $@)
	$(HIPCC) -x c++ -O2 -std=c++17 -fPIC -fvisibility=hidden -w -c -D__HIP_PLATFORM_AMD__ -DTSX_WITH_TENNIS $(DEFS) \
	    -mavx2 -mfma -I$(REPO)/include -I/opt/rocm/include -I$(REF)/include -I$(REF)/src $< -o $@

$(OUT)/libtennis_hip.so: $(OBJS) $(HIPOBJS) $(REPO)/tennis_amd/lib/libtsx_hip.so
	@echo LINK $@
	@$(CXX) -shared -fopenmp -Wl,-Bsymbolic -o $@ $(OBJS) $(HIPOBJS) -L$(REPO)/tennis_amd/lib -ltsx_hip \
	    -L/opt/rocm/lib -lamdhip64 -lpthread -lm -Wl,-rpath,'$$ORIGIN/..' -Wl,-rpath,/opt/rocm/lib

$(OUT)/libtennis_hip_driver.so: $(HERE)intree_driver.cpp $(OUT)/libtennis_hip.so
	$(CXX) $(CXXFLAGS) -fvisibility=default -shared -Wl,-Bsymbolic -o $@ $< -L$(OUT) -ltennis_hip -lpthread -Wl,-rpath,'$$ORIGIN'

clean:
	rm -rf $(OUT)
.PHONY: all clean
