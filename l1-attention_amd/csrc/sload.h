// Scalar prefetch: 32 floats of a wave-uniform row through two 16-float SGPR groups, issued ahead of use.
//
// The compiler schedules each scalar load of a wave-uniform row only a few instructions ahead of its first use,
// so a wave sits out a scalar-cache / L2 round trip per chunk.  With these two helpers a kernel issues the load
// of chunk c+1 before the VALU work on chunk c and waits for it afterwards.  Scalar loads return out of order,
// hence the only wait is lgkmcnt(0).
//
// This is the one place in the library where inline asm issues a load.  The compiler does not know that the
// destination registers are written later than the asm statement: nothing may touch them between sload32 and
// the matching swait32.  The build verifies that on the generated code of every kernel that uses the helpers
// (build.py: check_scalar_prefetch) and rejects any other load in inline asm.
#ifndef L1ATTN_SLOAD_H
#define L1ATTN_SLOAD_H
#include <hip/hip_runtime.h>

typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void sload32(f32x16& lo, f32x16& hi, const float* p)
{
	// early-clobber outputs: the second load must still see the pointer
	asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx16 %1, %2, 0x40" : "=&s"(lo), "=&s"(hi) : "s"(p));
}
// The same load from p + BYTES (a compile-time offset inside the row: no scalar add, no second pointer).
template <int BYTES>
__device__ __forceinline__ void sload32_at(f32x16& lo, f32x16& hi, const float* p)
{
	static_assert(BYTES >= 0 && BYTES % 4 == 0 && BYTES + 0x40 < (1 << 20), "immediate offset of a scalar load");
	asm volatile("s_load_dwordx16 %0, %2, %3\n\ts_load_dwordx16 %1, %2, %4"
	             : "=&s"(lo), "=&s"(hi)
	             : "s"(p), "n"(BYTES), "n"(BYTES + 0x40));
}
__device__ __forceinline__ void swait32(f32x16& lo, f32x16& hi)
{
	asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(lo), "+s"(hi));
}
// A wave-uniform value that the compiler loads itself (an ordinary scalar load it tracks) is taken here: the
// compiler puts its wait for that load in front of this point.  Placed right after a swait32, where nothing is in
// flight, that wait costs nothing; left to the first use, it would fall between a prefetch and the work that
// covers it, and wait for the prefetch as well.
__device__ __forceinline__ void sarrived(float& x)
{
	asm volatile("" : "+s"(x));
}

#endif
