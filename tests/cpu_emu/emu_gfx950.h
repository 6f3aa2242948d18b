// TEST INFRASTRUCTURE: host stand-in for csrc/gfx950.h, shared by the runner and the emulated library of the dense
// kernels.
#pragma once
#include "hip/hip_runtime.h"
#include "emu_sload.h"

// Stand-in for csrc/gfx950.h: what each hand-written instruction sequence computes, in plain C++.
#define L1ATTN_GFX950_H
#define L1_DYNAMIC_LDS(type, name) type* const name = reinterpret_cast<type*>(emu::dynamic_lds)
static inline void lds_barrier() { __syncthreads(); }
static inline void sad8(unsigned& au, const float* qv, const f32x16& kv, int i0)
{
	for (int i = 0; i < 8; i++) {
		const unsigned a = __float_as_uint(qv[i]), b = __float_as_uint(kv[i0 + i]);
		au += a > b ? a - b : b - a;
	}
}
static inline float emu_clamp(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }
static inline void pair_step4(const float* qc, float kc, const float4& g, float* dq, float& dk)
{
	const float gg[4] = {g.x, g.y, g.z, g.w};
	for (int i = 0; i < 4; i++) {
		const float e = emu_clamp(qc[i] - kc, -1.0f, 1.0f);
		dq[i] = fmaf(e, gg[i], dq[i]);
		dk = fmaf(-e, gg[i], dk);
	}
}
static inline void pair_step4_rank(const float* qc, float kc, const float4& g, float* dq, float& dk)
{
	const float gg[4] = {g.x, g.y, g.z, g.w};
	for (int i = 0; i < 4; i++) {
		const float e = emu_clamp(qc[i] - kc, 0.0f, 1.0f);
		dq[i] = fmaf(e, gg[i], dq[i]);
		dk = fmaf(e, gg[i], dk);
	}
}
