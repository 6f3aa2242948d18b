// Fused dense L1 attention for gfx950: logits, softmax over the src tokens with the
// "no-op" zero logit, and the value sum, without ever writing the [B,T,T,H] logits:
//
//   a[s]        = -1/sqrt(W) * sum_w |q[b,t,h,w] - k[b,s,h,w]|
//   vo[b,t,h,:] = sum_s exp(a[s]) * v[b,s,h,:] / (1 + sum_s exp(a[s]))
//
// This is what the reference's model code computes from the dense operator (L1Attn, a row of zero
// logits appended, softmax over dim 1, einsum 'bsdh,bshw->bdhw': example-setfind/setfind.py:128-136,
// python/l1attn_sparse.py:488-506) and what its README names as the better form ("blocked attention
// ... ala FlashAttention", README.md:21).  It also equals sparse attention over the full cartesian
// edge list.  Every logit is <= 0 and the no-op logit is 0, so the softmax needs no running maximum:
// exp(a) <= 1 and the denominator is >= 1.
//
// Tiled kernel: one wavefront per head, one lane per dst token, as in the dense forward.  A lane keeps
// its q row (W registers) and its output row (WV registers); the k and v rows of the current src token
// are wave-uniform and come through the scalar cache.  Per pair-element: v_sub, v_add |x| for the logit
// and one v_fmac for the value sum; one exp per (src, dst, head).  No LDS, no atomics; src tokens are
// summed in ascending order, so results repeat bit for bit.
#include "common.h"
#include "sload.h"
#include "xcd.h"
#include <math.h>

namespace {

template <typename T> __device__ __forceinline__ T fabs_t(T x) { return x < (T)0 ? -x : x; }
template <typename T> __device__ __forceinline__ T exp_t(T x);
template <> __device__ __forceinline__ float exp_t<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double exp_t<double>(double x) { return exp(x); }
// log(1 + x): the sum of the weights is often far below 1 (long L1 distances), where log(1 + x) formed in two
// steps would lose most of its digits
__device__ __forceinline__ float log1p_t(float x) { return log1pf(x); }
__device__ __forceinline__ double log1p_t(double x) { return log1p(x); }

// Any shape, float or double: one thread per output element (b,t,h,wv); the logit of each src token is
// recomputed by every thread of the row (W-fold redundant), which only small or odd shapes pay.
template <typename T>
__global__ __launch_bounds__(256) void fused_fwd_generic(const T* __restrict__ q, const T* __restrict__ k,
                                                           const T* __restrict__ v, T* __restrict__ vo,
                                                           T* __restrict__ lse, int64_t B, int64_t Tn, int64_t H,
                                                           int64_t W, int64_t Wv, T scale)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= B * Tn * H * Wv) return;
	const int64_t wv = idx % Wv, h = (idx / Wv) % H, t = (idx / (Wv * H)) % Tn, b = idx / (Wv * H * Tn);
	const T* qp = q + ((b * Tn + t) * H + h) * W;
	T den = 0, acc = 0;
	for (int64_t s = 0; s < Tn; s++) {
		const T* kp = k + ((b * Tn + s) * H + h) * W;
		T f = 0;
		for (int64_t w = 0; w < W; w++) f += fabs_t(qp[w] - kp[w]);
		const T p = exp_t(f * scale);
		den += p;
		acc += p * v[((b * Tn + s) * H + h) * Wv + wv];
	}
	vo[idx] = acc / ((T)1 + den);
	if (lse && wv == 0) lse[(b * Tn + t) * H + h] = log1p_t(den);
}

// grid.x = dst tiles of 64 tokens, grid.y = B * head groups; block = 64 * NH threads, wave w owns head
// hg*NH + w.  W == WV is a compile-time multiple of 16 (16, 32, 48, 64, 96: q and the output row must fit the
// registers); q, k, v, vo must be 16-byte aligned.
template <int W>
__global__ __launch_bounds__(256) void fused_fwd_f32_tile(const float* __restrict__ q, const float* __restrict__ k,
                                                            const float* __restrict__ v, float* __restrict__ vo,
                                                            float* __restrict__ lse, int Tn, int H, int n_hg, int NH,
                                                            float scale)
{
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const LogicalBlock lb = xcd_remap();
	const int b = lb.y / n_hg, hg = lb.y % n_hg;
	const int h_raw = hg * NH + wave;
	const int h = min(h_raw, H - 1);  // surplus waves of the last group redo head H-1 and store nothing
	const int t_raw = lb.x * 64 + lane;
	const int t = min(t_raw, Tn - 1);  // surplus lanes of the last tile redo token Tn-1 and store nothing
	const bool store = h_raw < H && t_raw < Tn;

	float qr[W], acc[W];
	{
		const float4* qp = reinterpret_cast<const float4*>(q + (((int64_t)b * Tn + t) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = qp[w4];
			qr[w4 * 4 + 0] = x.x; qr[w4 * 4 + 1] = x.y; qr[w4 * 4 + 2] = x.z; qr[w4 * 4 + 3] = x.w;
		}
#pragma unroll
		for (int w = 0; w < W; w++) acc[w] = 0.0f;
		// take the q row here: left alone, the compiler waits for each of its loads at the first use, inside the
		// src loop, where the sixteen waits are then issued once per src token
#pragma unroll
		for (int w = 0; w < W; w++) asm volatile("" : "+v"(qr[w]));
	}
	float den = 0.0f;
	const int64_t row = (int64_t)H * W;
	const float* kp = k + (((int64_t)b * Tn) * H + h) * (int64_t)W;  // src token 0 of this (b,h): wave-uniform
	const float* vp = v + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	for (int s = 0; s < Tn; s++) {
		float a = 0.0f;
#pragma unroll
		for (int w = 0; w < W; w++) a += fabsf(qr[w] - kp[w]);  // uniform address: scalar loads
		const float p = expf(a * scale);
		den += p;
#pragma unroll
		for (int w = 0; w < W; w++) acc[w] += p * vp[w];
		kp += row;
		vp += row;
	}
	if (store) {
		const float inv = 1.0f / (1.0f + den);
		float4* op = reinterpret_cast<float4*>(vo + (((int64_t)b * Tn + t) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++)
			op[w4] = make_float4(acc[w4 * 4 + 0] * inv, acc[w4 * 4 + 1] * inv, acc[w4 * 4 + 2] * inv,
			                     acc[w4 * 4 + 3] * inv);
		if (lse) lse[((int64_t)b * Tn + t) * H + h] = log1pf(den);
	}
}

// Software-pipelined variant of the tiled forward for W == WV a multiple of 32: the same mapping and the same
// arithmetic in the same order, but the k and v rows stream through two 32-float SGPR buffers (sload.h) as one
// sequence of chunks -- k chunks of src token s, v chunks of s, k chunks of s + 1, ... -- with the load of the
// next chunk issued before the VALU work on the current one.  A row holds an even number of chunks (2*W/32), so a
// chunk's buffer is fixed by its place in the row.  The load issued after a row's last chunk is the first k chunk
// of the next row, clamped to the last row at the end (read, never used), and drained after the loop.

// Chunk C of a src token's 2*W/32 (k chunks first, then v chunks), then the chunks after it.
// The three sweeps of the fused operator share this stream; what differs is what the second row's chunks do:
//   FUSED_FWD  xr = q row, rows = k, v:    a += |xr - k|;  p = e^{a*scale}, den += p;  yr (vo sums) += p * v
//   FUSED_DV   xr = k row, rows = q, dvo:  a += |xr - q|;  p = e^{a*scale - l};         yr (dv sums) += p * dvo
//   FUSED_DA   xr = q row, rows = k, v:    a += |xr - k|;  p (a dot product) += yr (dvo row) * v
// l (FUSED_DV): the dst token's lse, a scalar the compiler loads; `pin` names the next token's, whose load the
// caller has just issued: it is taken right after this chunk's wait, where nothing is in flight, so that the
// compiler's own wait for it never falls between a prefetch and the work that covers it.
enum { FUSED_FWD = 0, FUSED_DV = 1, FUSED_DA = 2 };
template <int W, int C, int ROLE = FUSED_FWD>
__device__ __forceinline__ void fused_pipe_chunks(const float (&xr)[W], float (&yr)[W], float& a, float& p, float& den,
                                                  float scale, f32x16& b0l, f32x16& b0h, f32x16& b1l, f32x16& b1h,
                                                  const float* krow, const float* vrow, const float* knext,
                                                  float l = 0.0f, float* pin = nullptr)
{
	constexpr int CPR = W / 32;  // chunks per k row and per v row
	f32x16& lo = (C & 1) == 0 ? b0l : b1l;  // this chunk's buffer
	f32x16& hi = (C & 1) == 0 ? b0h : b1h;
	f32x16& nl = (C & 1) == 0 ? b1l : b0l;  // the next chunk's
	f32x16& nh = (C & 1) == 0 ? b1h : b0h;
	// (the scheduler may not move the previous chunk's VALU work below this chunk's wait: the wait would then
	// come a few instructions after the load it waits for)
	__builtin_amdgcn_sched_barrier(0);
	swait32(lo, hi);
	if constexpr (ROLE == FUSED_DV && C == 0) sarrived(*pin);
	__builtin_amdgcn_sched_barrier(0);
	// the chunk after this one: the rest of the k row, then the v row, then the next token's k row
	if constexpr (C + 1 < CPR) sload32_at<(C + 1) * 128>(nl, nh, krow);
	else if constexpr (C + 1 < 2 * CPR) sload32_at<(C + 1 - CPR) * 128>(nl, nh, vrow);
	else sload32(nl, nh, knext);
	__builtin_amdgcn_sched_barrier(0);
	if constexpr (C < CPR) {
#pragma unroll
		for (int i = 0; i < 16; i++) a += fabsf(xr[C * 32 + i] - lo[i]);
#pragma unroll
		for (int i = 0; i < 16; i++) a += fabsf(xr[C * 32 + 16 + i] - hi[i]);
	} else if constexpr (ROLE == FUSED_DA) {
#pragma unroll
		for (int i = 0; i < 16; i++) p += yr[(C - CPR) * 32 + i] * lo[i];
#pragma unroll
		for (int i = 0; i < 16; i++) p += yr[(C - CPR) * 32 + 16 + i] * hi[i];
	} else {
		if constexpr (C == CPR) {
			if constexpr (ROLE == FUSED_FWD) {
				p = expf(a * scale);
				den += p;
			} else {
				p = expf(a * scale - l);
			}
		}
#pragma unroll
		for (int i = 0; i < 16; i++) yr[(C - CPR) * 32 + i] += p * lo[i];
#pragma unroll
		for (int i = 0; i < 16; i++) yr[(C - CPR) * 32 + 16 + i] += p * hi[i];
	}
	if constexpr (C + 1 < 2 * CPR)
		fused_pipe_chunks<W, C + 1, ROLE>(xr, yr, a, p, den, scale, b0l, b0h, b1l, b1h, krow, vrow, knext, l, pin);
}

template <int W>
__global__ __launch_bounds__(256) void fused_fwd_f32_pipe(const float* __restrict__ q, const float* __restrict__ k,
                                                            const float* __restrict__ v, float* __restrict__ vo,
                                                            float* __restrict__ lse, int Tn, int H, int n_hg, int NH,
                                                            float scale)
{
	static_assert(W % 32 == 0, "whole 32-float chunks");
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const LogicalBlock lb = xcd_remap();
	const int b = lb.y / n_hg, hg = lb.y % n_hg;
	const int h_raw = hg * NH + wave;
	const int h = min(h_raw, H - 1);  // surplus waves of the last group redo head H-1 and store nothing
	const int t_raw = lb.x * 64 + lane;
	const int t = min(t_raw, Tn - 1);  // surplus lanes of the last tile redo token Tn-1 and store nothing
	const bool store = h_raw < H && t_raw < Tn;

	float qr[W], acc[W];
	{
		const float4* qp = reinterpret_cast<const float4*>(q + (((int64_t)b * Tn + t) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = qp[w4];
			qr[w4 * 4 + 0] = x.x; qr[w4 * 4 + 1] = x.y; qr[w4 * 4 + 2] = x.z; qr[w4 * 4 + 3] = x.w;
		}
#pragma unroll
		for (int w = 0; w < W; w++) acc[w] = 0.0f;
		// take the q row here: left alone, the compiler waits for each of its loads at the first use, inside the
		// src loop, where the sixteen waits are then issued once per src token
#pragma unroll
		for (int w = 0; w < W; w++) asm volatile("" : "+v"(qr[w]));
	}
	float den = 0.0f;
	const int64_t row = (int64_t)H * W;
	const float* const kb = k + (((int64_t)b * Tn) * H + h) * (int64_t)W;  // src token 0 of this (b,h): wave-uniform
	const float* const vb = v + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	f32x16 b0l, b0h, b1l, b1h;
	sload32(b0l, b0h, kb);
	__builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
	for (int s = 0; s < Tn; s++) {
		float a = 0.0f, p = 0.0f;
		fused_pipe_chunks<W, 0>(qr, acc, a, p, den, scale, b0l, b0h, b1l, b1h, kb + s * row, vb + s * row,
		                        kb + min(s + 1, Tn - 1) * row);
	}
	swait32(b0l, b0h);  // drain the last prefetch before the wave ends
	if (store) {
		const float inv = 1.0f / (1.0f + den);
		float4* op = reinterpret_cast<float4*>(vo + (((int64_t)b * Tn + t) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++)
			op[w4] = make_float4(acc[w4 * 4 + 0] * inv, acc[w4 * 4 + 1] * inv, acc[w4 * 4 + 2] * inv,
			                     acc[w4 * 4 + 3] * inv);
		if (lse) lse[((int64_t)b * Tn + t) * H + h] = log1pf(den);
	}
}

// ------------------------------------------------------------------------------------------ backward
// With p[s,t] = exp(a[s,t] - lse[t]), dp[s,t] = v[s].dvo[t] and S[t] = vo[t].dvo[t] (= sum_s p*dp):
//   dA[s,t] = p * (dp - S[t])                  gradient of the logits, written in the dense layout [B,S,T,H]
//   dv[s,:] = sum_t p[s,t] * dvo[t,:]
// dq and dk then come from the dense backward on dA.  Only dA is ever held of the four [B,T,T,H] tensors
// (logits, weights and their two gradients) that the unfused composition keeps.

// any shape: one thread per dA element
template <typename T>
__global__ __launch_bounds__(256) void fused_bwd_da_generic(const T* __restrict__ dvo, const T* __restrict__ q,
                                                              const T* __restrict__ k, const T* __restrict__ v,
                                                              const T* __restrict__ vo, const T* __restrict__ lse,
                                                              T* __restrict__ dA, int64_t B, int64_t Tn, int64_t H,
                                                              int64_t W, int64_t Wv, T scale)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= B * Tn * Tn * H) return;
	const int64_t h = idx % H, t = (idx / H) % Tn, s = (idx / (H * Tn)) % Tn, b = idx / (H * Tn * Tn);
	const T* qp = q + ((b * Tn + t) * H + h) * W;
	const T* kp = k + ((b * Tn + s) * H + h) * W;
	T f = 0;
	for (int64_t w = 0; w < W; w++) f += fabs_t(qp[w] - kp[w]);
	const T* vp = v + ((b * Tn + s) * H + h) * Wv;
	const T* op = vo + ((b * Tn + t) * H + h) * Wv;
	const T* gp = dvo + ((b * Tn + t) * H + h) * Wv;
	T dp = 0, S = 0;
	for (int64_t w = 0; w < Wv; w++) { dp += vp[w] * gp[w]; S += op[w] * gp[w]; }
	dA[idx] = exp_t(f * scale - lse[(b * Tn + t) * H + h]) * (dp - S);
}

// any shape: one thread per dv element, dst tokens summed in ascending order
template <typename T>
__global__ __launch_bounds__(256) void fused_bwd_dv_generic(const T* __restrict__ dvo, const T* __restrict__ q,
                                                              const T* __restrict__ k, const T* __restrict__ lse,
                                                              T* __restrict__ dv, int64_t B, int64_t Tn, int64_t H,
                                                              int64_t W, int64_t Wv, T scale)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= B * Tn * H * Wv) return;
	const int64_t wv = idx % Wv, h = (idx / Wv) % H, s = (idx / (Wv * H)) % Tn, b = idx / (Wv * H * Tn);
	const T* kp = k + ((b * Tn + s) * H + h) * W;
	T acc = 0;
	for (int64_t t = 0; t < Tn; t++) {
		const T* qp = q + ((b * Tn + t) * H + h) * W;
		T f = 0;
		for (int64_t w = 0; w < W; w++) f += fabs_t(qp[w] - kp[w]);
		acc += exp_t(f * scale - lse[(b * Tn + t) * H + h]) * dvo[((b * Tn + t) * H + h) * Wv + wv];
	}
	dv[idx] = acc;
}

// Tiled dA: the forward's mapping (wave = head, lane = dst token t), up to eight heads per workgroup.  A lane
// keeps q[t], dvo[t] and S[t]; the k and v rows of the src token are wave-uniform.  Per pair-element v_sub,
// v_add |x|, v_fmac.  The values of DA_SJ src rows are transposed through LDS so that the workgroup stores
// runs of NH consecutive heads per (s,t) (32 bytes with eight heads) instead of 4 bytes per lane at a pitch of
// H floats.  blockDim.x = 64*NH: one element of the [64 t x NH] plane per thread and src row.
constexpr int DA_SJ = 8;    // src rows between two flushes
constexpr int DA_NH = 8;    // most heads per workgroup

template <int W>
__global__ __launch_bounds__(64 * DA_NH) void fused_bwd_da_tile(const float* __restrict__ dvo,
                                                                  const float* __restrict__ q,
                                                                  const float* __restrict__ k,
                                                                  const float* __restrict__ v,
                                                                  const float* __restrict__ vo,
                                                                  const float* __restrict__ lse,
                                                                  float* __restrict__ dA, int Tn, int H, int n_hg,
                                                                  int NH, float scale)
{
	__shared__ float tile[DA_SJ][64 * (DA_NH + 1)];  // [src row][t * (NH+1) + head]: the odd pitch spreads the banks
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const LogicalBlock lb = xcd_remap();
	const int b = lb.y / n_hg, hg = lb.y % n_hg;
	const int h = min(hg * NH + wave, H - 1);  // surplus waves of the last group redo head H-1, never stored
	const int t0 = lb.x * 64;
	const int t = min(t0 + lane, Tn - 1);      // surplus lanes of the last tile redo token Tn-1, never stored
	const int PH = NH + 1;

	float qr[W], gr[W];
	float S = 0.0f;
	{
		const int64_t off = (((int64_t)b * Tn + t) * H + h) * (int64_t)W;
		const float4* qp = reinterpret_cast<const float4*>(q + off);
		const float4* gp = reinterpret_cast<const float4*>(dvo + off);
		const float4* op = reinterpret_cast<const float4*>(vo + off);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = qp[w4], g = gp[w4], o = op[w4];
			qr[w4 * 4 + 0] = x.x; qr[w4 * 4 + 1] = x.y; qr[w4 * 4 + 2] = x.z; qr[w4 * 4 + 3] = x.w;
			gr[w4 * 4 + 0] = g.x; gr[w4 * 4 + 1] = g.y; gr[w4 * 4 + 2] = g.z; gr[w4 * 4 + 3] = g.w;
			S += o.x * g.x; S += o.y * g.y; S += o.z * g.z; S += o.w * g.w;
		}
	}
	const float l = lse[((int64_t)b * Tn + t) * H + h];
	const int64_t row = (int64_t)H * W;
	const float* kb = k + (((int64_t)b * Tn) * H + h) * (int64_t)W;  // src token 0 of this (b,h): wave-uniform
	const float* vb = v + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	// role of this thread in the flush: element (o_t, o_h) of the [64 t x NH] plane
	const int o_t = threadIdx.x / NH, o_h = threadIdx.x % NH;
	const bool o_ok = (t0 + o_t < Tn) && (hg * NH + o_h < H);
	float* const o_base = dA + (((int64_t)b * Tn) * Tn + (t0 + o_t)) * H + hg * NH + o_h;  // src token 0
	const int64_t pitch = (int64_t)Tn * H;
	for (int s0 = 0; s0 < Tn; s0 += DA_SJ) {
#pragma unroll 1
		for (int j = 0; j < DA_SJ; j++) {
			const int s = min(s0 + j, Tn - 1);  // rows past the end are computed on the last row and not stored
			const float* kp = kb + s * row;
			const float* vp = vb + s * row;
			float a = 0.0f, dp = 0.0f;
#pragma unroll
			for (int w = 0; w < W; w++) a += fabsf(qr[w] - kp[w]);
#pragma unroll
			for (int w = 0; w < W; w++) dp += gr[w] * vp[w];
			tile[j][lane * PH + wave] = expf(a * scale - l) * (dp - S);
		}
		__syncthreads();
#pragma unroll
		for (int j = 0; j < DA_SJ; j++)
			if (o_ok && s0 + j < Tn) o_base[(int64_t)(s0 + j) * pitch] = tile[j][o_t * PH + o_h];
		__syncthreads();
	}
}

// Tiled dv: wave = head, lane = src token s.  A lane keeps k[s] and its dv row; the q and dvo rows and lse of the
// dst token are wave-uniform.  Per pair-element v_sub, v_add |x|, v_fmac; dst tokens in ascending order.
template <int W>
__global__ __launch_bounds__(256) void fused_bwd_dv_tile(const float* __restrict__ dvo, const float* __restrict__ q,
                                                           const float* __restrict__ k, const float* __restrict__ lse,
                                                           float* __restrict__ dv, int Tn, int H, int n_hg, int NH,
                                                           float scale)
{
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const LogicalBlock lb = xcd_remap();
	const int b = lb.y / n_hg, hg = lb.y % n_hg;
	const int h_raw = hg * NH + wave;
	const int h = min(h_raw, H - 1);
	const int s_raw = lb.x * 64 + lane;
	const int s = min(s_raw, Tn - 1);
	const bool store = h_raw < H && s_raw < Tn;

	float kr[W], acc[W];
	{
		const float4* kp = reinterpret_cast<const float4*>(k + (((int64_t)b * Tn + s) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = kp[w4];
			kr[w4 * 4 + 0] = x.x; kr[w4 * 4 + 1] = x.y; kr[w4 * 4 + 2] = x.z; kr[w4 * 4 + 3] = x.w;
		}
#pragma unroll
		for (int w = 0; w < W; w++) acc[w] = 0.0f;
		// take the k row here rather than at its first use inside the dst loop (see fused_fwd_f32_tile)
#pragma unroll
		for (int w = 0; w < W; w++) asm volatile("" : "+v"(kr[w]));
	}
	const int64_t row = (int64_t)H * W;
	const float* qp = q + (((int64_t)b * Tn) * H + h) * (int64_t)W;    // dst token 0 of this (b,h): wave-uniform
	const float* gp = dvo + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	const float* lp = lse + ((int64_t)b * Tn) * H + h;
	for (int t = 0; t < Tn; t++) {
		float a = 0.0f;
#pragma unroll
		for (int w = 0; w < W; w++) a += fabsf(qp[w] - kr[w]);
		const float p = expf(a * scale - *lp);
#pragma unroll
		for (int w = 0; w < W; w++) acc[w] += p * gp[w];
		qp += row;
		gp += row;
		lp += H;
	}
	if (store) {
		float4* op = reinterpret_cast<float4*>(dv + (((int64_t)b * Tn + s) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++)
			op[w4] = make_float4(acc[w4 * 4 + 0], acc[w4 * 4 + 1], acc[w4 * 4 + 2], acc[w4 * 4 + 3]);
	}
}

// Software-pipelined variants of the two tiled kernels above for W a multiple of 32 (see fused_fwd_f32_pipe): the
// same mapping and the same arithmetic in the same order, the wave-uniform rows streamed through the two SGPR
// buffers of sload.h instead of being loaded where the compiler puts them.

template <int W>
__global__ __launch_bounds__(64 * DA_NH) void fused_bwd_da_pipe(const float* __restrict__ dvo,
                                                                  const float* __restrict__ q,
                                                                  const float* __restrict__ k,
                                                                  const float* __restrict__ v,
                                                                  const float* __restrict__ vo,
                                                                  const float* __restrict__ lse,
                                                                  float* __restrict__ dA, int Tn, int H, int n_hg,
                                                                  int NH, float scale)
{
	static_assert(W % 32 == 0, "whole 32-float chunks");
	__shared__ float tile[DA_SJ][64 * (DA_NH + 1)];
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const LogicalBlock lb = xcd_remap();
	const int b = lb.y / n_hg, hg = lb.y % n_hg;
	const int h = min(hg * NH + wave, H - 1);
	const int t0 = lb.x * 64;
	const int t = min(t0 + lane, Tn - 1);
	const int PH = NH + 1;

	float qr[W], gr[W];
	float S = 0.0f;
	{
		const int64_t off = (((int64_t)b * Tn + t) * H + h) * (int64_t)W;
		const float4* qp = reinterpret_cast<const float4*>(q + off);
		const float4* gp = reinterpret_cast<const float4*>(dvo + off);
		const float4* op = reinterpret_cast<const float4*>(vo + off);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = qp[w4], g = gp[w4], o = op[w4];
			qr[w4 * 4 + 0] = x.x; qr[w4 * 4 + 1] = x.y; qr[w4 * 4 + 2] = x.z; qr[w4 * 4 + 3] = x.w;
			gr[w4 * 4 + 0] = g.x; gr[w4 * 4 + 1] = g.y; gr[w4 * 4 + 2] = g.z; gr[w4 * 4 + 3] = g.w;
			S += o.x * g.x; S += o.y * g.y; S += o.z * g.z; S += o.w * g.w;
		}
	}
	float l = lse[((int64_t)b * Tn + t) * H + h];
	// take the rows, S and lse here, before the first scalar prefetch is in flight
#pragma unroll
	for (int w = 0; w < W; w++) asm volatile("" : "+v"(qr[w]), "+v"(gr[w]));
	asm volatile("" : "+v"(S), "+v"(l));
	const int64_t row = (int64_t)H * W;
	const float* const kb = k + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	const float* const vb = v + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	const int o_t = threadIdx.x / NH, o_h = threadIdx.x % NH;
	const bool o_ok = (t0 + o_t < Tn) && (hg * NH + o_h < H);
	float* const o_base = dA + (((int64_t)b * Tn) * Tn + (t0 + o_t)) * H + hg * NH + o_h;
	const int64_t pitch = (int64_t)Tn * H;
	float unused = 0.0f;
	f32x16 b0l, b0h, b1l, b1h;
	sload32(b0l, b0h, kb);
	__builtin_amdgcn_sched_barrier(0);
	for (int s0 = 0; s0 < Tn; s0 += DA_SJ) {
#pragma unroll 1
		for (int j = 0; j < DA_SJ; j++) {
			// rows past the end are computed on the last row and not stored; the row after it is the next in the stream
			const int s = min(s0 + j, Tn - 1), sn = min(s0 + j + 1, Tn - 1);
			float a = 0.0f, dp = 0.0f;
			fused_pipe_chunks<W, 0, FUSED_DA>(qr, gr, a, dp, unused, scale, b0l, b0h, b1l, b1h, kb + s * row, vb + s * row,
			                                  kb + sn * row);
			tile[j][lane * PH + wave] = expf(a * scale - l) * (dp - S);
		}
		__syncthreads();
#pragma unroll
		for (int j = 0; j < DA_SJ; j++)
			if (o_ok && s0 + j < Tn) o_base[(int64_t)(s0 + j) * pitch] = tile[j][o_t * PH + o_h];
		__syncthreads();
	}
	swait32(b0l, b0h);  // drain the last prefetch before the wave ends
}

template <int W>
__global__ __launch_bounds__(256) void fused_bwd_dv_pipe(const float* __restrict__ dvo, const float* __restrict__ q,
                                                           const float* __restrict__ k, const float* __restrict__ lse,
                                                           float* __restrict__ dv, int Tn, int H, int n_hg, int NH,
                                                           float scale)
{
	static_assert(W % 32 == 0, "whole 32-float chunks");
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const LogicalBlock lb = xcd_remap();
	const int b = lb.y / n_hg, hg = lb.y % n_hg;
	const int h_raw = hg * NH + wave;
	const int h = min(h_raw, H - 1);
	const int s_raw = lb.x * 64 + lane;
	const int s = min(s_raw, Tn - 1);
	const bool store = h_raw < H && s_raw < Tn;

	float kr[W], acc[W];
	{
		const float4* kp = reinterpret_cast<const float4*>(k + (((int64_t)b * Tn + s) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = kp[w4];
			kr[w4 * 4 + 0] = x.x; kr[w4 * 4 + 1] = x.y; kr[w4 * 4 + 2] = x.z; kr[w4 * 4 + 3] = x.w;
		}
#pragma unroll
		for (int w = 0; w < W; w++) acc[w] = 0.0f;
#pragma unroll
		for (int w = 0; w < W; w++) asm volatile("" : "+v"(kr[w]));
	}
	const int64_t row = (int64_t)H * W;
	const float* const qb = q + (((int64_t)b * Tn) * H + h) * (int64_t)W;    // dst token 0 of this (b,h): wave-uniform
	const float* const gb = dvo + (((int64_t)b * Tn) * H + h) * (int64_t)W;
	const float* const lp = lse + ((int64_t)b * Tn) * H + h;
	float unused = 0.0f;
	float l = lp[0];
	sarrived(l);  // before the first prefetch is issued
	f32x16 b0l, b0h, b1l, b1h;
	sload32(b0l, b0h, qb);
	__builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
	for (int t = 0; t < Tn; t++) {
		const int tn = min(t + 1, Tn - 1);
		float l_next = lp[(int64_t)tn * H];  // issued here, taken inside right after the first chunk's wait
		float a = 0.0f, p = 0.0f;
		fused_pipe_chunks<W, 0, FUSED_DV>(kr, acc, a, p, unused, scale, b0l, b0h, b1l, b1h, qb + t * row, gb + t * row,
		                                  qb + tn * row, l, &l_next);
		l = l_next;
	}
	swait32(b0l, b0h);  // drain the last prefetch before the wave ends
	if (store) {
		float4* op = reinterpret_cast<float4*>(dv + (((int64_t)b * Tn + s) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++)
			op[w4] = make_float4(acc[w4 * 4 + 0], acc[w4 * 4 + 1], acc[w4 * 4 + 2], acc[w4 * 4 + 3]);
	}
}

bool shape_ok(int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv)
{
	return B >= 0 && T >= 0 && H >= 0 && W >= 1 && Wv >= 1;
}

template <typename T>
int launch_generic(const T* q, const T* k, const T* v, T* vo, T* lse, int64_t B, int64_t Tn, int64_t H, int64_t W,
                   int64_t Wv, hipStream_t st)
{
	const int64_t n = B * Tn * H * Wv;
	if (n >= ((int64_t)1 << 32)) return L1ATTN_ERR_RANGE;  // one thread per output element
	const T scale = (T)(-1.0 / sqrt((double)W));
	hipLaunchKernelGGL(fused_fwd_generic<T>, dim3((unsigned)l1_cdiv(n, 256)), dim3(256), 0, st, q, k, v, vo, lse, B, Tn,
	                   H, W, Wv, scale);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

template <typename T>
int launch_bwd_generic(const T* dvo, const T* q, const T* k, const T* v, const T* vo, const T* lse, T* dA, T* dv,
                       int64_t B, int64_t Tn, int64_t H, int64_t W, int64_t Wv, hipStream_t st)
{
	const int64_t na = B * Tn * Tn * H, nv = B * Tn * H * Wv;
	if (na >= ((int64_t)1 << 32) || nv >= ((int64_t)1 << 32)) return L1ATTN_ERR_RANGE;  // one thread per element
	const T scale = (T)(-1.0 / sqrt((double)W));
	hipLaunchKernelGGL(fused_bwd_da_generic<T>, dim3((unsigned)l1_cdiv(na, 256)), dim3(256), 0, st, dvo, q, k, v, vo,
	                   lse, dA, B, Tn, H, W, Wv, scale);
	L1_LAUNCH_CHECK();
	hipLaunchKernelGGL(fused_bwd_dv_generic<T>, dim3((unsigned)l1_cdiv(nv, 256)), dim3(256), 0, st, dvo, q, k, lse, dv,
	                   B, Tn, H, W, Wv, scale);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

}  // namespace

extern "C" {

// pipe: take the software-pipelined kernel where it exists (W == Wv in {32, 64}); every other shape runs
// what l1attn_fused_fwd_f32 runs
static int fused_fwd_f32(const float* q, const float* k, const float* v, float* vo, float* lse, int64_t B, int64_t T,
                         int64_t H, int64_t W, int64_t Wv, void* stream, bool pipe)
{
	if (!shape_ok(B, T, H, W, Wv)) return L1ATTN_ERR_ARG;
	if (B * T * H == 0) return L1ATTN_OK;
	if (!q || !k || !v || !vo) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	const bool aligned = ((((uintptr_t)q) | ((uintptr_t)k) | ((uintptr_t)v) | ((uintptr_t)vo)) & 15) == 0;
	const int NH = (int)(H < 4 ? H : 4);
	const int64_t n_hg = l1_cdiv(H, NH);
	const bool tiled = aligned && W == Wv && (W == 16 || W == 32 || W == 48 || W == 64 || W == 96) && T >= 32 && T <= (1 << 30) &&
	                   B * n_hg <= 65535 && H <= 65535;
	if (!tiled) return launch_generic<float>(q, k, v, vo, lse, B, T, H, W, Wv, st);
	const float scale = (float)(-1.0 / sqrt((double)W));
	const dim3 grid((unsigned)l1_cdiv(T, 64), (unsigned)(B * n_hg), 1), block(64 * NH);
#define L1_FUSED_CASE(KERNEL, WV)                                                                                \
	hipLaunchKernelGGL(KERNEL<WV>, grid, block, 0, st, q, k, v, vo, lse, (int)T, (int)H, (int)n_hg, NH, scale)
	switch (W) {
	case 16: L1_FUSED_CASE(fused_fwd_f32_tile, 16); break;
	case 32:
		if (pipe) L1_FUSED_CASE(fused_fwd_f32_pipe, 32);
		else L1_FUSED_CASE(fused_fwd_f32_tile, 32);
		break;
	case 48: L1_FUSED_CASE(fused_fwd_f32_tile, 48); break;
	case 64:
		if (pipe) L1_FUSED_CASE(fused_fwd_f32_pipe, 64);
		else L1_FUSED_CASE(fused_fwd_f32_tile, 64);
		break;
	case 96: L1_FUSED_CASE(fused_fwd_f32_tile, 96); break;  // (pipelined, its SGPR buffers would spill)
	default: return L1ATTN_ERR_ARG;
	}
#undef L1_FUSED_CASE
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

int l1attn_fused_fwd_f32(const float* q, const float* k, const float* v, float* vo, float* lse, int64_t B, int64_t T,
                         int64_t H, int64_t W, int64_t Wv, void* stream)
{
	return fused_fwd_f32(q, k, v, vo, lse, B, T, H, W, Wv, stream, false);
}

int l1attn_fused_fwd_pipe_f32(const float* q, const float* k, const float* v, float* vo, float* lse, int64_t B,
                              int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream)
{
	return fused_fwd_f32(q, k, v, vo, lse, B, T, H, W, Wv, stream, true);
}

int l1attn_fused_fwd_f64(const double* q, const double* k, const double* v, double* vo, double* lse, int64_t B,
                         int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream)
{
	if (!shape_ok(B, T, H, W, Wv)) return L1ATTN_ERR_ARG;
	if (B * T * H == 0) return L1ATTN_OK;
	if (!q || !k || !v || !vo) return L1ATTN_ERR_ARG;
	return launch_generic<double>(q, k, v, vo, lse, B, T, H, W, Wv, (hipStream_t)stream);
}

// First stage of the fused backward: dA [B,S,T,H] (gradient of the logits) and dv from dvo and the forward's
// vo and lse.  dq and dk follow from l1attn_dense_bwd_* on dA, q, k.
// pipe: take the software-pipelined kernels where they exist (W == Wv in {32, 64}); every other shape runs what
// l1attn_fused_bwd_stage_f32 runs
static int fused_bwd_stage_f32(const float* dvo, const float* q, const float* k, const float* v, const float* vo,
                               const float* lse, float* dA, float* dv, int64_t B, int64_t T, int64_t H, int64_t W,
                               int64_t Wv, void* stream, bool pipe)
{
	if (!shape_ok(B, T, H, W, Wv)) return L1ATTN_ERR_ARG;
	if (B * T * H == 0) return L1ATTN_OK;
	if (!dvo || !q || !k || !v || !vo || !lse || !dA || !dv) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	const bool aligned = ((((uintptr_t)dvo) | ((uintptr_t)q) | ((uintptr_t)k) | ((uintptr_t)v) | ((uintptr_t)vo) |
	                       ((uintptr_t)dv)) & 15) == 0;
	const int NH = (int)(H < 4 ? H : 4);
	const int64_t n_hg = l1_cdiv(H, NH);
	const bool tiled = aligned && W == Wv && (W == 16 || W == 32 || W == 48 || W == 64 || W == 96) && T >= 32 && T <= (1 << 30) &&
	                   B * n_hg <= 65535 && H <= 65535;
	if (!tiled) return launch_bwd_generic<float>(dvo, q, k, v, vo, lse, dA, dv, B, T, H, W, Wv, st);
	const float scale = (float)(-1.0 / sqrt((double)W));
	const dim3 grid((unsigned)l1_cdiv(T, 64), (unsigned)(B * n_hg), 1), block(64 * NH);
	// the dA kernel takes up to eight heads per workgroup: longer runs of consecutive heads per store
	const int NHa = (int)(H < DA_NH ? H : DA_NH);
	const int64_t n_hga = l1_cdiv(H, NHa);
	const dim3 grida((unsigned)l1_cdiv(T, 64), (unsigned)(B * n_hga), 1), blocka(64 * NHa);
#define L1_FUSED_BWD_CASE(WV)                                                                                       \
	case WV:                                                                                                        \
		hipLaunchKernelGGL(fused_bwd_da_tile<WV>, grida, blocka, 0, st, dvo, q, k, v, vo, lse, dA, (int)T, (int)H,   \
		                   (int)n_hga, NHa, scale);                                                                 \
		hipLaunchKernelGGL(fused_bwd_dv_tile<WV>, grid, block, 0, st, dvo, q, k, lse, dv, (int)T, (int)H, (int)n_hg,  \
		                   NH, scale);                                                                              \
		break
#define L1_FUSED_BWD_PIPE_CASE(WV)                                                                                  \
	do {                                                                                                            \
		hipLaunchKernelGGL(fused_bwd_da_pipe<WV>, grida, blocka, 0, st, dvo, q, k, v, vo, lse, dA, (int)T, (int)H,   \
		                   (int)n_hga, NHa, scale);                                                                 \
		hipLaunchKernelGGL(fused_bwd_dv_pipe<WV>, grid, block, 0, st, dvo, q, k, lse, dv, (int)T, (int)H, (int)n_hg,  \
		                   NH, scale);                                                                              \
	} while (0)
	if (pipe && W == 32) L1_FUSED_BWD_PIPE_CASE(32);
	else if (pipe && W == 64) L1_FUSED_BWD_PIPE_CASE(64);
	else switch (W) {
		L1_FUSED_BWD_CASE(16);
		L1_FUSED_BWD_CASE(32);
		L1_FUSED_BWD_CASE(48);
		L1_FUSED_BWD_CASE(64);
		L1_FUSED_BWD_CASE(96);
	default: return L1ATTN_ERR_ARG;
	}
#undef L1_FUSED_BWD_CASE
#undef L1_FUSED_BWD_PIPE_CASE
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

int l1attn_fused_bwd_stage_f32(const float* dvo, const float* q, const float* k, const float* v, const float* vo,
                               const float* lse, float* dA, float* dv, int64_t B, int64_t T, int64_t H, int64_t W,
                               int64_t Wv, void* stream)
{
	return fused_bwd_stage_f32(dvo, q, k, v, vo, lse, dA, dv, B, T, H, W, Wv, stream, false);
}

int l1attn_fused_bwd_stage_pipe_f32(const float* dvo, const float* q, const float* k, const float* v, const float* vo,
                                    const float* lse, float* dA, float* dv, int64_t B, int64_t T, int64_t H, int64_t W,
                                    int64_t Wv, void* stream)
{
	return fused_bwd_stage_f32(dvo, q, k, v, vo, lse, dA, dv, B, T, H, W, Wv, stream, true);
}

int l1attn_fused_bwd_stage_f64(const double* dvo, const double* q, const double* k, const double* v, const double* vo,
                               const double* lse, double* dA, double* dv, int64_t B, int64_t T, int64_t H, int64_t W,
                               int64_t Wv, void* stream)
{
	if (!shape_ok(B, T, H, W, Wv)) return L1ATTN_ERR_ARG;
	if (B * T * H == 0) return L1ATTN_OK;
	if (!dvo || !q || !k || !v || !vo || !lse || !dA || !dv) return L1ATTN_ERR_ARG;
	return launch_bwd_generic<double>(dvo, q, k, v, vo, lse, dA, dv, B, T, H, W, Wv, (hipStream_t)stream);
}

}  // extern "C"
