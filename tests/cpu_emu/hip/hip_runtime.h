// TEST INFRASTRUCTURE: a host-only stand-in for the few HIP constructs that the library's simpler
// kernels use (inline assembly only behind the library's two helper headers, for which the runners hold
// stand-ins), so that such a kernel can be compiled
// with g++ and run on the CPU under AddressSanitizer: every GPU thread of a workgroup is an OS thread,
// __syncthreads() is a barrier among them, __shared__ arrays are static storage (workgroups run one
// after the other).  It checks a kernel's index arithmetic, clamps, store predicates, LDS indexing,
// barrier placement and launch geometry against exactly-sized host buffers; it says nothing about
// timing, the memory model or the hardware.  Lanes of a wave do not run in lockstep here: where a kernel's
// lanes hand values to each other through memory between two cross-lane operations (the radix sort of coo.hip
// does, through per-wave LDS counters), the kernel marks the point with L1_WAVE_LOCKSTEP(lanes) -- nothing on the
// GPU, a barrier among the named lanes here.  Never part of the library: only the tests build with it.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdio.h>
#include <stdint.h>
#include <string.h>
#include <algorithm>
#include <atomic>
#include <barrier>
#include <condition_variable>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __restrict__
// Statically sized __shared__ arrays become static storage.  A source that only declares the dynamic array
// (`extern __shared__ unsigned char name[];`) is built with EMU_DYNAMIC_LDS_ONLY: the declaration then names a
// global array that the test driver defines.
#ifdef EMU_DYNAMIC_LDS_ONLY
#define __shared__
#else
#define __shared__ static
#endif

struct dim3 {
	unsigned x, y, z;
	dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct float4 { float x, y, z, w; };
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
struct double2 { double x, y; };
static inline double2 make_double2(double x, double y) { return double2{x, y}; }
struct uint2 { unsigned x, y; };
struct int4 { int x, y, z, w; };
static inline int4 make_int4(int x, int y, int z, int w) { return int4{x, y, z, w}; }

typedef void* hipStream_t;
typedef int hipError_t;
#define hipSuccess 0
static inline hipError_t hipGetLastError() { return hipSuccess; }
// "device" memory is host memory and every launch has finished when it returns
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
static inline hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, hipMemcpyKind, hipStream_t)
{
	memcpy(dst, src, n);
	return hipSuccess;
}
static inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }

namespace emu {
inline thread_local dim3 threadIdx_;
inline dim3 blockIdx_, blockDim_, gridDim_;
inline long n_threads_run = 0;
inline std::unique_ptr<std::barrier<>> wg_barrier;  // the running workgroup's __syncthreads()
// Lanes of a wavefront run in lockstep on the GPU; here they are OS threads, so every cross-lane exchange is
// bracketed by a barrier among the wave's 64 threads.
inline std::vector<std::unique_ptr<std::barrier<>>> wave_barrier;
// 64 exchange slots per wave, in two planes that successive exchanges alternate between: a lane that is already
// writing its value for exchange n+1 cannot disturb a lane still reading exchange n, so one barrier per exchange is
// enough (a lane reaches exchange n+2, which reuses the plane of n, only after every lane has arrived at the barrier
// of n+1, hence finished reading n).  All lanes of a wave take part in every exchange, so their counts agree.
inline std::vector<double> wave_slots[2];
inline thread_local unsigned exchange_count = 0;  // reset at the start of every workgroup
// A runner may ask to see every launch (kernel expression as written at the launch site, grid, block, dynamic LDS
// bytes) and may set `dry`: the launch is then reported and checked against the limits of a HIP launch, not run.
inline void (*on_launch)(const char* kernel, dim3 grid, dim3 block, size_t lds) = nullptr;
inline bool dry = false;
inline unsigned char* dynamic_lds = nullptr;  // the launch's dynamically sized LDS array, exactly `lds` bytes
inline unsigned flat_tid() { return threadIdx_.x + blockDim_.x * (threadIdx_.y + blockDim_.y * threadIdx_.z); }
inline void wave_sync() { wave_barrier[flat_tid() >> 6]->arrive_and_wait(); }
// one cross-lane exchange: publish x, wait for the wave, return the plane to read the other lanes' values from
inline const std::vector<double>& exchange(double x)
{
	std::vector<double>& plane = wave_slots[exchange_count++ & 1u];
	plane[flat_tid()] = x;
	wave_sync();
	return plane;
}
// Barrier among a subset of a wave's lanes, keyed by the subset's lowest lane (disjoint subsets of one wave may
// wait at the same time): the last lane to arrive opens the gate for the others.
struct LaneGate { std::atomic<int> count{0}, generation{0}; };
inline std::unique_ptr<LaneGate[]> lane_gates;  // 64 per wave
inline void lockstep(unsigned long long lanes)
{
	const unsigned tid = flat_tid(), lane = tid & 63u;
	if (!((lanes >> lane) & 1ull)) abort();  // the caller must be one of the lanes it names
	const int n = __builtin_popcountll(lanes);
	LaneGate& g = lane_gates[(tid & ~63u) + (unsigned)__builtin_ctzll(lanes)];
	const int gen = g.generation.load();
	if (g.count.fetch_add(1) + 1 == n) {
		g.count.store(0);
		g.generation.fetch_add(1);
		g.generation.notify_all();
	} else {
		while (g.generation.load() == gen) g.generation.wait(gen);
	}
}
}
#define L1_WAVE_LOCKSTEP(lanes) emu::lockstep(lanes)
#define threadIdx (emu::threadIdx_)
#define blockIdx (emu::blockIdx_)
#define blockDim (emu::blockDim_)
#define gridDim (emu::gridDim_)

using std::min;
using std::max;

#include <string.h>
#include <stdlib.h>
static inline unsigned __float_as_uint(float x) { unsigned u; memcpy(&u, &x, 4); return u; }
static inline float __uint_as_float(unsigned u) { float x; memcpy(&x, &u, 4); return x; }
static inline int __float_as_int(float x) { int u; memcpy(&u, &x, 4); return u; }
static inline float __int_as_float(int u) { float x; memcpy(&x, &u, 4); return x; }

// value of the wave's first active lane; the kernels built here only pass wave-uniform values
static inline int __builtin_amdgcn_readfirstlane(int x) { return x; }
// Cross-lane read within the wave: every lane of the wave must call it (uniform control flow).
template <typename T>
static inline T __shfl_xor(T x, int lane_mask)
{
	const unsigned tid = emu::flat_tid(), base = tid & ~63u;
	return (T)emu::exchange((double)x)[base + ((tid ^ (unsigned)lane_mask) & 63u)];
}
template <typename T>
static inline T __shfl_xor(T x, int lane_mask, int width)
{
	if (width != 64) abort();
	return __shfl_xor(x, lane_mask);
}
// value of the lane `delta` below, or the lane's own where there is none.  Every lane of the wave must call it.
template <typename T>
static inline T __shfl_up(T x, unsigned delta, int width)
{
	if (width != 64) abort();
	const unsigned tid = emu::flat_tid();
	const std::vector<double>& plane = emu::exchange((double)x);
	return (tid & 63u) >= delta ? (T)plane[tid - delta] : x;
}
// bit l = predicate of lane l.  Every lane of the wave must call it (the emulated waves are always full or end
// with the workgroup: a lane beyond it reads as 0).
static inline unsigned long long __ballot(int pred)
{
	const unsigned tid = emu::flat_tid(), base = tid & ~63u;
	const std::vector<double>& plane = emu::exchange(pred ? 1.0 : 0.0);
	unsigned long long m = 0;
	for (unsigned l = 0; l < 64 && base + l < plane.size(); l++)
		if (plane[base + l] != 0.0) m |= 1ull << l;
	return m;
}
static inline int __popcll(unsigned long long x) { return __builtin_popcountll(x); }
// atomics on global and LDS words: the return value is the old one
static inline int atomicAdd(int* p, int v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
static inline int atomicOr(int* p, int v) { return __atomic_fetch_or(p, v, __ATOMIC_SEQ_CST); }
static inline int atomicMax(int* p, int v)
{
	int old = __atomic_load_n(p, __ATOMIC_SEQ_CST);
	while (old < v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {}
	return old;
}
// DPP row shift right by n (control 0x110 + n) with out-of-row lanes reading zero: lane l of each aligned group
// of sixteen receives the value of lane l - n of the same group.  Every lane of the wave must call it.
static inline int emu_dpp_row_shr(int src, int ctrl)
{
	const unsigned tid = emu::flat_tid(), n = (unsigned)ctrl & 15u;
	const std::vector<double>& plane = emu::exchange((double)src);
	return ((tid & 15u) >= n) ? (int)plane[tid - n] : 0;
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl) \
	(static_cast<void>(sizeof(char[((ctrl) > 0x110 && (ctrl) < 0x120 && (bound_ctrl)) ? 1 : -1])), emu_dpp_row_shr(src, ctrl))
// Raw buffer access: base + per-lane byte offset + uniform byte offset, both unsigned 32-bit; the library's
// descriptors are unbounded below 4 GiB, so an offset sum that reaches 2^32 would be dropped on the GPU: abort here.
struct __amdgpu_buffer_rsrc_t { char* base; };
static inline char* emu_buf_at(__amdgpu_buffer_rsrc_t r, int v, int s)
{
	const uint64_t off = (uint64_t)(unsigned)v + (uint64_t)(unsigned)s;
	if (off >= ((uint64_t)1 << 32)) abort();
	return r.base + off;
}
static inline unsigned emu_buf_load(__amdgpu_buffer_rsrc_t r, int v, int s) { unsigned u; memcpy(&u, emu_buf_at(r, v, s), 4); return u; }
static inline void emu_buf_store(unsigned u, __amdgpu_buffer_rsrc_t r, int v, int s) { memcpy(emu_buf_at(r, v, s), &u, 4); }
static inline void emu_buf_fadd(float x, __amdgpu_buffer_rsrc_t r, int v, int s)
{
	float y; memcpy(&y, emu_buf_at(r, v, s), 4); y += x; memcpy(emu_buf_at(r, v, s), &y, 4);
}
#define __builtin_amdgcn_make_buffer_rsrc(p, stride, num, flags) (__amdgpu_buffer_rsrc_t{(char*)(p)})
#define __builtin_amdgcn_raw_buffer_load_b32(r, v, s, aux) emu_buf_load(r, v, s)
#define __builtin_amdgcn_raw_buffer_store_b32(u, r, v, s, aux) emu_buf_store(u, r, v, s)
#define __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(x, r, v, s, aux) emu_buf_fadd(x, r, v, s)
// scheduling and wait hints have no meaning here
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#ifndef __clang__
#define __builtin_nontemporal_store(v, p) (*(p) = (v))
#define __builtin_nontemporal_load(p) (*(p))
#endif
// Memory fences order a wave's own stores before its own later loads from other lanes: lockstep lanes need
// nothing more on the GPU, OS threads need a barrier among the wave.
#define __builtin_amdgcn_fence(order, scope) emu::wave_sync()
// every thread of the workgroup must reach it (a thread that has returned would hang the others, as it may on a GPU)
static inline void __syncthreads() { emu::wg_barrier->arrive_and_wait(); }

namespace emu {
// The OS threads that play the GPU threads, kept from launch to launch (a library call is dozens of launches):
// run(nt, f) has threads 0..nt-1 execute f(thread number) and returns when all have finished.
class Pool {
	std::vector<std::thread> threads_;
	std::mutex m_;
	std::condition_variable start_, done_;
	std::function<void(unsigned)> job_;
	unsigned active_ = 0, finished_ = 0;
	long generation_ = 0;
	bool stop_ = false;
	void loop(unsigned id)
	{
		long seen = 0;
		for (;;) {
			std::function<void(unsigned)> job;
			{
				std::unique_lock<std::mutex> lk(m_);
				start_.wait(lk, [&] { return stop_ || generation_ != seen; });
				if (stop_) return;
				seen = generation_;
				if (id >= active_) continue;
				job = job_;
			}
			job(id);
			std::lock_guard<std::mutex> lk(m_);
			if (++finished_ == active_) done_.notify_all();
		}
	}

public:
	void run(unsigned nt, std::function<void(unsigned)> f)
	{
		std::unique_lock<std::mutex> lk(m_);
		// a new thread starts with seen = 0 and generation_ >= 1 below, so it picks this job up
		while (threads_.size() < nt) {
			const unsigned id = (unsigned)threads_.size();
			threads_.emplace_back([this, id] { loop(id); });
		}
		job_ = std::move(f);
		active_ = nt;
		finished_ = 0;
		generation_++;
		start_.notify_all();
		done_.wait(lk, [&] { return finished_ == active_; });
	}
	~Pool()
	{
		{
			std::lock_guard<std::mutex> lk(m_);
			stop_ = true;
		}
		start_.notify_all();
		for (auto& t : threads_) t.join();
	}
};
inline Pool& pool()
{
	static Pool p;
	return p;
}
}

template <typename K, typename... A>
static inline void emu_launch(const char* name, K kernel, dim3 grid, dim3 block, size_t lds, A... args)
{
	// what hipLaunchKernelGGL would refuse (the library reads the error after every launch; here it is fatal)
	const uint64_t nthreads = (uint64_t)block.x * block.y * block.z;
	if (!(grid.x >= 1 && grid.y >= 1 && grid.z >= 1 && grid.x <= 2147483647u && grid.y <= 65535u && grid.z <= 65535u &&
	      nthreads >= 1 && nthreads <= 1024 && lds <= 64 * 1024)) {
		fprintf(stderr, "invalid launch of %s: grid %u %u %u block %u %u %u lds %zu\n", name, grid.x, grid.y, grid.z, block.x,
		        block.y, block.z, lds);
		abort();
	}
	if (emu::on_launch) emu::on_launch(name, grid, block, lds);
	if (emu::dry) return;
	// exactly sized, so that AddressSanitizer sees an access beyond the launch's LDS size
	std::unique_ptr<unsigned char[]> lds_mem(lds ? new unsigned char[lds] : nullptr);
	emu::dynamic_lds = lds_mem.get();
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
				emu::wave_barrier.clear();
				for (unsigned w = 0; w < (nt + 63) / 64; w++)
					emu::wave_barrier.emplace_back(new std::barrier<>(std::min(64u, nt - w * 64)));
				emu::wave_slots[0].assign((nt + 63) / 64 * 64, 0.0);
				emu::wave_slots[1].assign((nt + 63) / 64 * 64, 0.0);
				emu::lane_gates.reset(new emu::LaneGate[(nt + 63) / 64 * 64]);
			}
			emu::exchange_count = 0;
			step.arrive_and_wait();
			kernel(args...);
			step.arrive_and_wait();
		}
	};
	emu::pool().run(nt, worker);  // the OS threads are kept from launch to launch
	emu::n_threads_run += (long)nt * nblocks;
}
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
	emu_launch(#kernel, kernel, dim3(grid), dim3(block), (size_t)(lds), __VA_ARGS__)
