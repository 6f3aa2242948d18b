// TEST INFRASTRUCTURE: host stand-in for csrc/sload.h, shared by the runners of the kernels that prefetch through it.
#pragma once
#include "hip/hip_runtime.h"
#include <atomic>
#include <string.h>

// Host stand-in for csrc/sload.h (the one header of the library whose inline asm issues loads), with the
// property that matters kept: the data of a prefetch arrives at the WAIT, not at the load.  sload32 poisons its
// two buffers and remembers the source; swait32 (lgkmcnt(0): everything outstanding) delivers all remembered
// loads.  A kernel that reads a buffer before its wait computes on NaNs, one that forgets the final drain leaves
// `outstanding` above zero: both show in the test.
#define L1ATTN_SLOAD_H
struct f32x16 {
	float a[16];
	float operator[](int i) const { return a[i]; }
};
namespace emu_sload {
struct Pending { f32x16 *lo, *hi; const float* p; };
inline thread_local std::vector<Pending> pending;
inline std::atomic<long> outstanding{0};
}
static inline void sload32(f32x16& lo, f32x16& hi, const float* p)
{
	for (int i = 0; i < 16; i++) lo.a[i] = hi.a[i] = NAN;
	emu_sload::pending.push_back({&lo, &hi, p});
	emu_sload::outstanding++;
}
template <int BYTES>
static inline void sload32_at(f32x16& lo, f32x16& hi, const float* p)
{
	sload32(lo, hi, p + BYTES / 4);
}
static inline void swait32(f32x16&, f32x16&)
{
	for (const auto& x : emu_sload::pending) {
		memcpy(x.lo->a, x.p, 64);
		memcpy(x.hi->a, x.p + 16, 64);
		emu_sload::outstanding--;
	}
	emu_sload::pending.clear();
}
static inline void sarrived(float&) {}
static inline void __builtin_amdgcn_sched_barrier(int) {}
