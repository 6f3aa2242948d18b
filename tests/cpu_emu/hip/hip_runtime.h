// TEST INFRASTRUCTURE: a host-only stand-in for the few HIP constructs that the library's simpler
// kernels use (no cross-lane operations, no inline assembly), so that such a kernel can be compiled
// with g++ and run on the CPU under AddressSanitizer: every GPU thread of a workgroup is an OS thread,
// __syncthreads() is a barrier among them, __shared__ arrays are static storage (workgroups run one
// after the other).  It checks a kernel's index arithmetic, clamps, store predicates, LDS indexing,
// barrier placement and launch geometry against exactly-sized host buffers; it says nothing about
// timing, the memory model or the hardware.  Never part of the library: only
// tests/test_cpu_emulation.py builds with it.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <algorithm>
#include <barrier>
#include <memory>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __restrict__
#define __shared__ static

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
inline thread_local dim3 threadIdx_;
inline dim3 blockIdx_, blockDim_, gridDim_;
inline long n_threads_run = 0;
inline std::unique_ptr<std::barrier<>> wg_barrier;  // the running workgroup's __syncthreads()
}
#define threadIdx (emu::threadIdx_)
#define blockIdx (emu::blockIdx_)
#define blockDim (emu::blockDim_)
#define gridDim (emu::gridDim_)

using std::min;
using std::max;

// value of the wave's first active lane; the kernels built here only pass wave-uniform values
static inline int __builtin_amdgcn_readfirstlane(int x) { return x; }
// every thread of the workgroup must reach it (a thread that has returned would hang the others, as it may on a GPU)
static inline void __syncthreads() { emu::wg_barrier->arrive_and_wait(); }

template <typename K, typename... A>
static inline void emu_launch(K kernel, dim3 grid, dim3 block, A... args)
{
	emu::gridDim_ = grid;
	emu::blockDim_ = block;
	const unsigned nt = block.x * block.y * block.z;
	const long nblocks = (long)grid.x * grid.y * grid.z;
	std::barrier<> step(nt);  // separates the workgroups: they share the static __shared__ storage
	auto worker = [&](unsigned tid) {
		emu::threadIdx_ = dim3(tid % block.x, (tid / block.x) % block.y, tid / (block.x * block.y));
		for (long bi = 0; bi < nblocks; bi++) {
			if (tid == 0) {
				emu::blockIdx_ = dim3((unsigned)(bi % grid.x), (unsigned)((bi / grid.x) % grid.y), (unsigned)(bi / ((long)grid.x * grid.y)));
				emu::wg_barrier.reset(new std::barrier<>(nt));
			}
			step.arrive_and_wait();
			kernel(args...);
			step.arrive_and_wait();
		}
	};
	std::vector<std::thread> pool;
	for (unsigned t = 0; t < nt; t++) pool.emplace_back(worker, t);
	for (auto& th : pool) th.join();
	emu::n_threads_run += (long)nt * nblocks;
}
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
	emu_launch(kernel, dim3(grid), dim3(block), __VA_ARGS__)
