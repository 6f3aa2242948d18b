// Pre-passes of the experimental fixed-point dense forward (l1attn_dense_fwd_fixed_f32): q and k of every
// (batch, head) are put on a common grid so that the forward's pair-element is one v_sad_u32.
#include "fixed.h"
#include <math.h>
#include <algorithm>

namespace {

// Fixed-point forward, pre-pass 1: grid of each (batch, head) = largest |q| or |k| of the head * 2^-24
// (at least the smallest normal float), so that every value is an integer of at most 2^24 in magnitude on it.
// One workgroup per (b,h); the maximum is exact and order-independent.
__global__ __launch_bounds__(256) void fixed_absmax(const float* __restrict__ q, const float* __restrict__ k,
                                                      float* __restrict__ gq, int Tn, int H, int W)
{
	__shared__ float red[256];
	const int b = blockIdx.x / H, h = blockIdx.x % H;
	float m = 0.0f;
	for (int i = threadIdx.x; i < Tn * W; i += 256) {
		const int t = i / W, w = i - t * W;
		const int64_t off = (((int64_t)b * Tn + t) * H + h) * (int64_t)W + w;
		m = fmaxf(m, fmaxf(fabsf(q[off]), fabsf(k[off])));
	}
	red[threadIdx.x] = m;
	__syncthreads();
	for (int st = 128; st > 0; st >>= 1) {
		if ((int)threadIdx.x < st) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + st]);
		__syncthreads();
	}
	// 2^-24 of the maximum, but never below the smallest normal float (an all-zero or denormal-only head)
	if (threadIdx.x == 0) gq[blockIdx.x] = fmaxf(red[0] * 5.9604644775390625e-08f, 1.17549435e-38f);
}

// pre-pass 2: u = round(x / grid) as a two's-complement integer with the sign bit flipped (a bias of 2^31),
// which keeps the order of the values as unsigned integers: |u_q - u_k| is the distance in grid units.
__global__ __launch_bounds__(256) void fixed_quantise(const float* __restrict__ q, const float* __restrict__ k,
                                                        const float* __restrict__ gq, unsigned* __restrict__ uq,
                                                        unsigned* __restrict__ uk, int64_t n, int H, int W, int64_t TH)
{
	for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
		const int64_t row = i / W;  // (b*T + t)*H + h
		const float g = gq[(row / TH) * H + row % H];
		uq[i] = (unsigned)(int)rintf(q[i] / g) ^ 0x80000000u;
		uk[i] = (unsigned)(int)rintf(k[i] / g) ^ 0x80000000u;
	}
}

}  // namespace

int l1_launch_fixed_prepass(const float* q, const float* k, float* gq, unsigned* uq, unsigned* uk, int64_t B,
                            int64_t T, int64_t H, int64_t W, hipStream_t st)
{
	if (B * H > 2147483647LL || T * W > 2147483647LL) return L1ATTN_ERR_RANGE;
	const int64_t n = B * T * H * W;
	hipLaunchKernelGGL(fixed_absmax, dim3((unsigned)(B * H)), dim3(256), 0, st, q, k, gq, (int)T, (int)H, (int)W);
	L1_LAUNCH_CHECK();
	const dim3 qgrid((unsigned)std::min<int64_t>(l1_cdiv(n, 256), 1 << 20));
	hipLaunchKernelGGL(fixed_quantise, qgrid, dim3(256), 0, st, q, k, (const float*)gq, uq, uk, n, (int)H, (int)W, T * H);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}
