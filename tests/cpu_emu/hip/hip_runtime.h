// TEST INFRASTRUCTURE: a host-only stand-in for the few HIP constructs that the library's
// wave-independent kernels use, so that such a kernel (no LDS, no barriers, no cross-lane operations)
// can be compiled with g++ and run on the CPU, one thread at a time, under AddressSanitizer.  It
// checks a kernel's index arithmetic, clamps, store predicates and launch geometry against
// exactly-sized host buffers; it says nothing about timing, the memory model or the hardware.
// Never part of the library: only tests/test_cpu_emulation.py builds with it.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <algorithm>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __restrict__

struct dim3 {
	unsigned x, y, z;
	dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct float4 { float x, y, z, w; };
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }

typedef void* hipStream_t;
typedef int hipError_t;
#define hipSuccess 0
static inline hipError_t hipGetLastError() { return hipSuccess; }

namespace emu {
inline dim3 threadIdx_, blockIdx_, blockDim_, gridDim_;
inline long n_threads_run = 0;
}
#define threadIdx (emu::threadIdx_)
#define blockIdx (emu::blockIdx_)
#define blockDim (emu::blockDim_)
#define gridDim (emu::gridDim_)

using std::min;
using std::max;

// value of the wave's first active lane; the kernels built here only pass wave-uniform values
static inline int __builtin_amdgcn_readfirstlane(int x) { return x; }

template <typename K, typename... A>
static inline void emu_launch(K kernel, dim3 grid, dim3 block, A... args)
{
	emu::gridDim_ = grid;
	emu::blockDim_ = block;
	for (unsigned bz = 0; bz < grid.z; bz++)
		for (unsigned by = 0; by < grid.y; by++)
			for (unsigned bx = 0; bx < grid.x; bx++)
				for (unsigned tz = 0; tz < block.z; tz++)
					for (unsigned ty = 0; ty < block.y; ty++)
						for (unsigned tx = 0; tx < block.x; tx++) {
							emu::blockIdx_ = dim3(bx, by, bz);
							emu::threadIdx_ = dim3(tx, ty, tz);
							emu::n_threads_run++;
							kernel(args...);
						}
}
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
	emu_launch(kernel, dim3(grid), dim3(block), __VA_ARGS__)
