# Builds _ref/libclpeak_ref.so from the reference's own sources, compiled where they lie (nothing is
# copied), plus ref_shim.cpp.  Only the two files below compile without the reference's build system;
# see ref_shim.cpp.  Run with: make -C oracle -f ref.mk   (needs the checkout at $(REF)).
REF ?= /root/reference
CXX ?= g++
CXXFLAGS := -O2 -std=c++17 -fPIC -DENABLE_CPU -I$(REF)/include -I$(REF)/src

all: _ref/libclpeak_ref.so

_ref/libclpeak_ref.so: ref_shim.cpp $(REF)/src/common/common.cpp $(REF)/src/cpu/thread_pool.cpp
	mkdir -p _ref
	$(CXX) $(CXXFLAGS) -shared -o $@ ref_shim.cpp $(REF)/src/common/common.cpp $(REF)/src/cpu/thread_pool.cpp -lpthread

clean:
	rm -rf _ref

.PHONY: all clean
