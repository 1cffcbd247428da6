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

clean:
	rm -rf $(OUT)
.PHONY: all lib driver clean
