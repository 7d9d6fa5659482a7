# Builds _ref/libclpeak_ref.so from the reference's own sources, compiled where they lie (nothing is
# copied), plus ref_shim.cpp.  Only these files compile without the reference's build system; see
# ref_shim.cpp.  The kernel file is compiled once per ISA with the options its own CMakeLists uses:
# -O3 -ffast-math, LTO off, ENABLE_CPU, CLPEAK_ISA_TAG=<tag>, and the -m flags of that tag.  Run with: make -C oracle -f ref.mk   (needs the checkout at $(REF)).
REF ?= /root/reference
CXX ?= g++
CXXFLAGS := -O2 -std=c++17 -fPIC -DENABLE_CPU -I$(REF)/include -I$(REF)/src -I$(REF)/src/cpu
TUFLAGS  := -O3 -ffast-math -fno-lto -std=c++17 -fPIC -DENABLE_CPU -I$(REF)/include -I$(REF)/src/cpu

all: _ref/libclpeak_ref.so

_ref/tu_avx2.o: $(REF)/src/cpu/cpu_kernels_tu.cpp
	mkdir -p _ref
	$(CXX) $(TUFLAGS) -DCLPEAK_ISA_TAG=avx2 -mavx2 -mfma -mf16c -c $< -o $@

_ref/tu_avx512.o: $(REF)/src/cpu/cpu_kernels_tu.cpp
	mkdir -p _ref
	$(CXX) $(TUFLAGS) -DCLPEAK_ISA_TAG=avx512 -mavx512f -mavx512bw -mavx512vl -mavx512dq -c $< -o $@

_ref/libclpeak_ref.so: ref_shim.cpp $(REF)/src/common/common.cpp $(REF)/src/cpu/thread_pool.cpp _ref/tu_avx2.o _ref/tu_avx512.o
	mkdir -p _ref
	$(CXX) $(CXXFLAGS) -shared -o $@ ref_shim.cpp $(REF)/src/common/common.cpp $(REF)/src/cpu/thread_pool.cpp \
	    _ref/tu_avx2.o _ref/tu_avx512.o -lpthread

clean:
	rm -rf _ref

.PHONY: all clean
