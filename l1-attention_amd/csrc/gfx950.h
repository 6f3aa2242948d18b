// The instructions this library writes by hand for gfx950, apart from the scalar prefetch of sload.h: the
// LDS-only workgroup barrier, the backward's four-pair-element steps and the fixed-point forward's SAD block.
// They are VALU and synchronisation instructions on registers the compiler allocates; none of them touches
// memory (the build rejects a load in inline asm outside sload.h).  Kept in one header so that the kernels that
// use them are otherwise plain C++: a CPU test build puts a stand-in of this header in front of it on the
// include path and runs the same kernel source on the host.
#ifndef L1ATTN_GFX950_H
#define L1ATTN_GFX950_H
#include <hip/hip_runtime.h>
#include "sload.h"

// The workgroup's dynamically sized LDS array (size given at launch).
#define L1_DYNAMIC_LDS(type, name) extern __shared__ type name[]

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global store (vmcnt(0)), which stalls the workgroup for a full HBM write round trip each time a
// barrier follows stores; here only the LDS/scalar counter is drained before the barrier.
__device__ __forceinline__ void lds_barrier()
{
	asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Eight fixed-point pair-elements of the chunk at qv[0..8) / kv[i0..i0+8) in one volatile asm block: volatile
// keeps it between the chunk's scalar prefetch and the next chunk's wait (both volatile asm), and one block per
// eight instructions keeps the compiler from padding every inline instruction with a wait state.
__device__ __forceinline__ void sad8(unsigned& au, const float* qv, const f32x16& kv, int i0)
{
#define L1_QU(i) "v"(__float_as_uint(qv[i]))
#define L1_KU(i) "s"(__float_as_uint(kv[i0 + i]))  // (a bit_cast of a vector element reads element 0)
	asm volatile("v_sad_u32 %0, %1, %9, %0\n\tv_sad_u32 %0, %2, %10, %0\n\tv_sad_u32 %0, %3, %11, %0\n\t"
	             "v_sad_u32 %0, %4, %12, %0\n\tv_sad_u32 %0, %5, %13, %0\n\tv_sad_u32 %0, %6, %14, %0\n\t"
	             "v_sad_u32 %0, %7, %15, %0\n\tv_sad_u32 %0, %8, %16, %0"
	             : "+v"(au)
	             : L1_QU(0), L1_QU(1), L1_QU(2), L1_QU(3), L1_QU(4), L1_QU(5), L1_QU(6), L1_QU(7),
	               L1_KU(0), L1_KU(1), L1_KU(2), L1_KU(3), L1_KU(4), L1_KU(5), L1_KU(6), L1_KU(7));
#undef L1_QU
#undef L1_KU
}

// sign(x) for pre-scaled differences: x is (q-k)*2^64, so every non-zero difference of
// magnitude >= 2^-64 saturates to +-1 and an exact tie stays 0.
//
// Four pair-elements of the backward pass (one src token against four dst tokens):
//   sg = sign(qc_u - kc); dq_u += sg*g_u; dk -= sg*g_u.
// One asm block so that the VALU instructions stay together: left to the compiler, the
// accumulations are sunk away from the signs and the signs spill.
__device__ __forceinline__ void pair_step4(const float* qc, float kc, const float4& g, float* dq, float& dk)
{
	float e0, e1;
	asm volatile(
	    "v_sub_f32 %0, %7, %11\n\t"
	    "v_sub_f32 %1, %8, %11\n\t"
	    "v_med3_f32 %0, %0, -1.0, 1.0\n\t"
	    "v_med3_f32 %1, %1, -1.0, 1.0\n\t"
	    "v_fmac_f32 %2, %0, %12\n\t"
	    "v_fma_f32 %6, -%0, %12, %6\n\t"
	    "v_fmac_f32 %3, %1, %13\n\t"
	    "v_fma_f32 %6, -%1, %13, %6\n\t"
	    "v_sub_f32 %0, %9, %11\n\t"
	    "v_sub_f32 %1, %10, %11\n\t"
	    "v_med3_f32 %0, %0, -1.0, 1.0\n\t"
	    "v_med3_f32 %1, %1, -1.0, 1.0\n\t"
	    "v_fmac_f32 %4, %0, %14\n\t"
	    "v_fma_f32 %6, -%0, %14, %6\n\t"
	    "v_fmac_f32 %5, %1, %15\n\t"
	    "v_fma_f32 %6, -%1, %15, %6"
	    : "=&v"(e0), "=&v"(e1), "+v"(dq[0]), "+v"(dq[1]), "+v"(dq[2]), "+v"(dq[3]), "+v"(dk)
	    : "v"(qc[0]), "v"(qc[1]), "v"(qc[2]), "v"(qc[3]), "v"(kc), "v"(g.x), "v"(g.y), "v"(g.z), "v"(g.w));
}

// The same four pair-elements on column ranks (dense_rank.hip): qc holds rq, kc holds rk (rank minus
// one half), so clamp(qc - kc, 0, 1) = hv is 1, 1/2 or 0 for q > k, q == k, q < k and sign = 2*hv - 1.
//   dq_u += hv*g_u; dk += hv*g_u
// Three instructions per pair-element; the caller turns the sums into sum(sign*g) with the row and
// column sums of g:  sum_s sign*g = 2*sum_s hv*g - sum_s g.
__device__ __forceinline__ void pair_step4_rank(const float* qc, float kc, const float4& g, float* dq, float& dk)
{
	float e0, e1;
	asm volatile(
	    "v_sub_f32_e64 %0, %7, %11 clamp\n\t"
	    "v_sub_f32_e64 %1, %8, %11 clamp\n\t"
	    "v_fmac_f32 %2, %0, %12\n\t"
	    "v_fmac_f32 %6, %0, %12\n\t"
	    "v_fmac_f32 %3, %1, %13\n\t"
	    "v_fmac_f32 %6, %1, %13\n\t"
	    "v_sub_f32_e64 %0, %9, %11 clamp\n\t"
	    "v_sub_f32_e64 %1, %10, %11 clamp\n\t"
	    "v_fmac_f32 %4, %0, %14\n\t"
	    "v_fmac_f32 %6, %0, %14\n\t"
	    "v_fmac_f32 %5, %1, %15\n\t"
	    "v_fmac_f32 %6, %1, %15"
	    : "=&v"(e0), "=&v"(e1), "+v"(dq[0]), "+v"(dq[1]), "+v"(dq[2]), "+v"(dq[3]), "+v"(dk)
	    : "v"(qc[0]), "v"(qc[1]), "v"(qc[2]), "v"(qc[3]), "v"(kc), "v"(g.x), "v"(g.y), "v"(g.z), "v"(g.w));
}

#endif
