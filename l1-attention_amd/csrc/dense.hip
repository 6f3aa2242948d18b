// Dense L1 attention for gfx950 (MI355X): A[b,s,t,h] = -1/sqrt(W) * sum_w |q[b,t,h,w] - k[b,s,h,w]|
// and its backward.  Replaces the kernels and launchers of the reference's
// cuda/l1attn_cuda_kernel.cu:27-685 and the dispatch in cuda/l1attn_cuda_drv.cpp:42-104.
//
// The op is a non-contraction (|a-b| does not factor), so it runs on the fp32 VALU, not on MFMA.
//
// Forward (fp32 fast path): one wavefront per head, one lane per dst token t.  A lane keeps its
// q row in registers; the k row of the current src token is wave-uniform and is read through the
// scalar cache into SGPRs, so the inner loop is two VALU instructions per pair-element
// (v_sub, v_add |x|) with no LDS or vector-memory traffic.  The workgroup (all heads of a 64-token
// dst tile) transposes each finished src row through LDS and stores [t-tile x H] contiguous runs.
//
// Backward (fp32 fast path): one lane per (h,w) column, a workgroup per dst tile of 32..88 tokens
// looping over all src tokens.  q values and dq accumulators live in registers, the dA tile is
// staged through LDS in [s][h][t] order so that a lane reads its head's four consecutive dA values
// with one broadcast ds_read_b128.  Per pair-element: v_sub, v_med3 (sign with sign(0)=0), two v_fma.
// dq is complete when the loop ends; dk is written as one partial per dst tile and summed in
// tile order by a second kernel, so the result is bitwise reproducible (no atomics).
// For T >= 2048 the pair-element takes three instructions: q and k are first replaced by
// order-preserving integer ranks per column (dense_rank.hip), on which a clamped subtraction is
// already (sign+1)/2, and the row and column sums of dA turn the accumulated sums back into
// sum(sign*dA).
//
// Generic kernels (any shape, float or double, exact comparisons) cover everything else.
#include "common.h"
#include "dense_rank.h"
#include "sload.h"
#include "gfx950.h"
#include "xcd.h"
#include "fixed.h"
#include <math.h>
#include <stdlib.h>
#include <algorithm>

namespace {

constexpr int WAVE = 64;

// ------------------------------------------------------------------------------------------
// generic kernels
// ------------------------------------------------------------------------------------------

template <typename T>
__device__ __forceinline__ T sgn_exact(T x) { return (T)((x > (T)0) - (x < (T)0)); }

template <typename T>
__device__ __forceinline__ T abs_t(T x) { return x < (T)0 ? -x : x; }

// one thread per (t,h); blockIdx.y strides over (b,s)
template <typename T>
__global__ __launch_bounds__(256) void dense_fwd_generic(const T* __restrict__ q, const T* __restrict__ k,
                                                           T* __restrict__ attn, int64_t B, int64_t Tn,
                                                           int64_t H, int64_t W, T scale)
{
	int64_t th = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (th >= Tn * H) return;
	int64_t h = th % H;
	for (int64_t bs = blockIdx.y; bs < B * Tn; bs += gridDim.y) {
		int64_t b = bs / Tn;
		const T* qp = q + (b * Tn * H + th) * W;
		const T* kp = k + (bs * H + h) * W;
		T f = 0;
		for (int64_t w = 0; w < W; w++) f += abs_t(qp[w] - kp[w]);
		attn[bs * Tn * H + th] = f * scale;
	}
}

// Short sequences (fewer tokens than the tiled kernels need): one workgroup per (b,h) keeps the T q rows and
// T k rows of the head in LDS (row pitch W+1, so that lanes with consecutive dst tokens hit different banks)
// and every thread computes whole logits.
template <typename T>
__global__ __launch_bounds__(256) void dense_fwd_small(const T* __restrict__ q, const T* __restrict__ k,
                                                         T* __restrict__ attn, int Tn, int H, int W, T scale)
{
	L1_DYNAMIC_LDS(unsigned char, small_lds);
	T* const qs = reinterpret_cast<T*>(small_lds);
	const int WP = W + 1;
	T* const ks = qs + Tn * WP;
	const int64_t b = blockIdx.x / (unsigned)H;
	const int h = (int)(blockIdx.x % (unsigned)H);
	for (int i = threadIdx.x; i < Tn * W; i += 256) {
		const int t = i / W, w = i - t * W;
		const int64_t off = ((b * Tn + t) * H + h) * (int64_t)W + w;
		qs[t * WP + w] = q[off];
		ks[t * WP + w] = k[off];
	}
	__syncthreads();
	for (int o = threadIdx.x; o < Tn * Tn; o += 256) {
		const int s = o / Tn, t = o - s * Tn;
		const T* qp = qs + t * WP;
		const T* kp = ks + s * WP;
		T f = 0;
		for (int w = 0; w < W; w++) f += abs_t(qp[w] - kp[w]);
		attn[((b * Tn + s) * Tn + t) * H + h] = f * scale;
	}
}

// one thread per dq element, src tokens summed in ascending order
template <typename T>
__global__ __launch_bounds__(256) void dense_bwd_generic_dq(const T* __restrict__ dA, const T* __restrict__ q,
                                                              const T* __restrict__ k, T* __restrict__ dq,
                                                              int64_t B, int64_t Tn, int64_t H, int64_t W, T scale)
{
	int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= B * Tn * H * W) return;
	int64_t w = idx % W, h = (idx / W) % H, t = (idx / (W * H)) % Tn, b = idx / (W * H * Tn);
	T qv = q[idx], acc = 0;
	for (int64_t s = 0; s < Tn; s++) {
		T ws = sgn_exact(qv - k[((b * Tn + s) * H + h) * W + w]) * scale;
		acc += ws * dA[((b * Tn + s) * Tn + t) * H + h];
	}
	dq[idx] = acc;
}

template <typename T>
__global__ __launch_bounds__(256) void dense_bwd_generic_dk(const T* __restrict__ dA, const T* __restrict__ q,
                                                              const T* __restrict__ k, T* __restrict__ dk,
                                                              int64_t B, int64_t Tn, int64_t H, int64_t W, T scale)
{
	int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= B * Tn * H * W) return;
	int64_t w = idx % W, h = (idx / W) % H, s = (idx / (W * H)) % Tn, b = idx / (W * H * Tn);
	T kv = k[idx], acc = 0;
	for (int64_t t = 0; t < Tn; t++) {
		T ws = sgn_exact(q[((b * Tn + t) * H + h) * W + w] - kv) * scale;
		acc -= ws * dA[((b * Tn + s) * Tn + t) * H + h];
	}
	dk[idx] = acc;
}

// ------------------------------------------------------------------------------------------
// Guard of the tiled fp32 backward that takes sign(q - k) from the scaled difference (dense_bwd_f32_fast without
// column ranks): clamp(q*2^64 - k*2^64, -1, 1) equals sign(q - k) for every pair when all magnitudes are below
// 2^63 (no overflow) and every non-zero value is at least 2^-41 in magnitude (then all values, and so all their
// differences, are whole multiples of 2^-64).  dense_bwd_sign_domain sets *flag when some value of q or k is
// outside that (NaN and infinities included); the kernel after it then recomputes dq and dk with exact
// comparisons, as the generic kernels do, and returns at once when the flag is clear.  The flag lives in the
// caller's workspace and must be zero before dense_bwd_sign_domain runs.
// ------------------------------------------------------------------------------------------

__global__ __launch_bounds__(64) void dense_bwd_clear_flag(int* __restrict__ flag)
{
	if (threadIdx.x == 0 && blockIdx.x == 0) *flag = 0;
}

__global__ __launch_bounds__(256) void dense_bwd_sign_domain(const float* __restrict__ q, const float* __restrict__ k,
                                                               int64_t n, int* __restrict__ flag)
{
	__shared__ int any_outside;
	if (threadIdx.x == 0) any_outside = 0;
	__syncthreads();
	bool outside = false;
	for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
		const float a = fabsf(q[i]), b = fabsf(k[i]);
		// !(a < 2^63) is also true for NaN
		outside |= !(a < 0x1p63f) || !(b < 0x1p63f) || (a != 0.0f && a < 0x1p-41f) || (b != 0.0f && b < 0x1p-41f);
	}
	if (outside) atomicOr(&any_outside, 1);
	__syncthreads();
	if (threadIdx.x == 0 && any_outside) atomicOr(flag, 1);
}

// blockIdx.y == 0: one thread per dq element, src tokens summed in ascending order; blockIdx.y == 1: one thread per
// dk element, dst tokens in ascending order.  The arithmetic of dense_bwd_generic_dq / _dk.
__global__ __launch_bounds__(256) void dense_bwd_exact_if_flagged(const float* __restrict__ dA, const float* __restrict__ q,
                                                                    const float* __restrict__ k, float* __restrict__ dq,
                                                                    float* __restrict__ dk, int64_t B, int64_t Tn, int64_t H,
                                                                    int64_t W, float scale, const int* __restrict__ flag)
{
	if (*flag == 0) return;
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= B * Tn * H * W) return;
	const bool for_dk = blockIdx.y != 0;
	const int64_t w = idx % W, h = (idx / W) % H, own = (idx / (W * H)) % Tn, b = idx / (W * H * Tn);
	const float mine = for_dk ? k[idx] : q[idx];
	const float* const others = for_dk ? q : k;
	float acc = 0;
	for (int64_t o = 0; o < Tn; o++) {
		const float other = others[((b * Tn + o) * H + h) * W + w];
		const float ws = sgn_exact(for_dk ? other - mine : mine - other) * scale;
		const int64_t s = for_dk ? own : o, t = for_dk ? o : own;
		const float g = dA[((b * Tn + s) * Tn + t) * H + h];
		if (for_dk) acc -= ws * g; else acc += ws * g;
	}
	(for_dk ? dk : dq)[idx] = acc;
}

// ------------------------------------------------------------------------------------------
// fp32 forward, fast path
// ------------------------------------------------------------------------------------------

constexpr int FWD_SJ = 8;  // src rows finished between two output flushes
constexpr int FWD_L2_AHEAD = 4;  // src blocks between the L2 prefetch of k rows and their use
constexpr int FWD_TILE = 1024 + 4 * WAVE;  // floats per staged src row: 64*NW outputs + one pad column per sub-tile (NH >= 4)

// grid.x = dst tiles of 64*NTS tokens, grid.y = src chunks, grid.z = B * head groups.
// block = 64 * NW threads (NW <= 16 waves) = NH heads x NTS dst sub-tiles of 64 tokens: wave w owns head
// hg*NH + w % NH and sub-tile w / NH.  Waves of the same head stream the same k rows, so the second one
// finds them in the scalar cache.
// W is a compile-time multiple of 16; q and k must be 16-byte aligned.
template <int W>
__global__ __launch_bounds__(1024) void dense_fwd_f32_fast(const float* __restrict__ q, const float* __restrict__ k,
                                                             float* __restrict__ attn, int Tn, int H, int n_hg,
                                                             int NH, int s_chunk, float scale)
{
	__shared__ float tile[FWD_SJ][FWD_TILE];
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int NW = blockDim.x >> 6, NTS = NW / NH, PH = NH + 1;
	const LogicalBlock lb = xcd_remap();
	const int b = lb.z / n_hg, hg = lb.z % n_hg;
	const int hl = wave % NH, ts = wave / NH;
	const int h = min(hg * NH + hl, H - 1);  // surplus waves of the last group redo head H-1, never stored
	const int tg0 = lb.x * NTS * WAVE;       // first dst token of the workgroup
	const int t0 = tg0 + ts * WAVE;          // first dst token of this wave
	const int t = min(t0 + lane, Tn - 1);

	float qr[W];
	{
		const float4* qp = reinterpret_cast<const float4*>(q + (((int64_t)b * Tn + t) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = qp[w4];
			qr[w4 * 4 + 0] = x.x; qr[w4 * 4 + 1] = x.y; qr[w4 * 4 + 2] = x.z; qr[w4 * 4 + 3] = x.w;
		}
	}

	// output role of this thread in the flush: element e = threadIdx.x of the [64*NTS x NH] row tile
	const int o_tl = threadIdx.x / NH, o_hh = threadIdx.x % NH;
	const bool o_ok = (tg0 + o_tl < Tn) && (hg * NH + o_hh < H);
	float* const o_base = attn + (((int64_t)b * Tn) * Tn + (tg0 + o_tl)) * H + hg * NH + o_hh;
	const int64_t o_pitch = (int64_t)Tn * H;

	const int s_begin = lb.y * s_chunk;
	const int s_end = min(Tn, s_begin + s_chunk);
	const float* const kb = k + (((int64_t)b * Tn) * H + h) * (int64_t)W;  // row 0 of this (b,h), wave-uniform
	const int64_t krow = (int64_t)H * W;
	for (int s0 = s_begin; s0 < s_end; s0 += FWD_SJ) {
		// L2 prefetch of a later src block's k rows, see dense_fwd_f32_pipe
		const float pf = kb[(int64_t)min(s0 + FWD_L2_AHEAD * FWD_SJ + (lane >> 3), Tn - 1) * krow + (lane & 7) * (W / 8)];
#pragma unroll
		for (int j = 0; j < FWD_SJ; j++) {
			const int s = min(s0 + j, Tn - 1);
			const float* kp = kb + s * krow;  // wave-uniform -> scalar loads
			float a = 0.0f;
#pragma unroll
			for (int w = 0; w < W; w++) a += fabsf(qr[w] - kp[w]);
			tile[j][(ts * WAVE + lane) * PH + hl] = a * scale;
		}
		asm volatile("" ::"v"(pf));
		lds_barrier();
#pragma unroll
		for (int j = 0; j < FWD_SJ; j++) {
			const int s = s0 + j;
			if (o_ok && s < s_end) __builtin_nontemporal_store(tile[j][o_tl * PH + o_hh], &o_base[s * o_pitch]);
		}
		lds_barrier();
	}
}

// Software-pipelined variant for W a multiple of 32.  The compiler schedules each scalar load of a
// k chunk only a few instructions ahead of its first use, so every 16 floats a wave sits out a
// scalar-cache/L2 round trip.  Here the k row streams through two 32-float SGPR buffers: the load of
// chunk c+1 is issued before the 64 VALU instructions of chunk c, so one chunk of compute (times the
// waves interleaved on the SIMD) covers the latency.  Scalar loads return out of order, hence the
// only wait used is lgkmcnt(0).
// FIXED: q and k hold biased fixed-point values (32-bit unsigned, see fixed_quantise) on a grid of gq[b*H+h]
// per (batch, head); the pair-element is then one v_sad_u32 (|a - b| + c on unsigned integers) instead of
// v_sub + v_add |x|, the sum of W <= 64 terms is exact and at most 2^31, and the logit is sum * grid * scale.

template <int W, bool FIXED = false>
__global__ __launch_bounds__(1024) void dense_fwd_f32_pipe(const float* __restrict__ q, const float* __restrict__ k,
                                                             float* __restrict__ attn, int Tn, int H, int n_hg,
                                                             int NH, int s_chunk, float scale, int V,
                                                             const float* __restrict__ gq = nullptr)
{
	// V > 1: q and k rows of width V*W are read as V consecutive heads of width W (the same memory), so
	// H counts those part-heads, NH (a multiple of V) of them share a workgroup, and the flush adds the V
	// partial sums of a head.
	static_assert(W % 32 == 0 && (FWD_SJ % 2) == 0, "chunk stream must keep buffer parity across src blocks");
	__shared__ float tile[FWD_SJ][FWD_TILE];
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int NW = blockDim.x >> 6, NTS = NW / NH, PH = NH + 1;
	const LogicalBlock lb = xcd_remap();
	const int b = lb.z / n_hg, hg = lb.z % n_hg;
	const int hl = wave % NH, ts = wave / NH;
	const int h = min(hg * NH + hl, H - 1);  // surplus waves of the last group redo head H-1, never stored
	const int tg0 = lb.x * NTS * WAVE;       // first dst token of the workgroup
	const int t0 = tg0 + ts * WAVE;          // first dst token of this wave
	const int t = min(t0 + lane, Tn - 1);

	float qr[W];
	{
		const float4* qp = reinterpret_cast<const float4*>(q + (((int64_t)b * Tn + t) * H + h) * (int64_t)W);
#pragma unroll
		for (int w4 = 0; w4 < W / 4; w4++) {
			const float4 x = qp[w4];
			qr[w4 * 4 + 0] = x.x; qr[w4 * 4 + 1] = x.y; qr[w4 * 4 + 2] = x.z; qr[w4 * 4 + 3] = x.w;
		}
	}
	const int NRH = NH / V, H_out = H / V;  // whole heads per workgroup, heads of the output
	const int o_tl = threadIdx.x / NRH, o_hh = threadIdx.x % NRH;
	const bool o_ok = (o_tl < NTS * WAVE) && (tg0 + o_tl < Tn) && (hg * NRH + o_hh < H_out);
	float* const o_base = attn + (((int64_t)b * Tn) * Tn + (tg0 + o_tl)) * H_out + hg * NRH + o_hh;
	const int64_t o_pitch = (int64_t)Tn * H_out;
	const int o_lds = o_tl * PH + o_hh * V;

	constexpr int CPR = W / 32;          // chunks per k row
	constexpr int NCH = FWD_SJ * CPR;    // chunks per src block
	const int64_t krow = (int64_t)H * W;  // floats between consecutive src rows
	const float* const kb = k + (((int64_t)b * Tn) * H + h) * (int64_t)W;  // row 0 of this (b,h), wave-uniform
	// last chunk of the last row: the running prefetch pointer is clamped to it, so rows past the end
	// of the tensor (computed but never stored) read valid memory
	const float* const k_last = kb + (int64_t)(Tn - 1) * krow + (CPR - 1) * 32;

	if constexpr (FIXED) scale *= gq[b * (H / V) + h / V];  // wave-uniform
	const int s_begin = lb.y * s_chunk;
	const int s_end = min(Tn, s_begin + s_chunk);
	f32x16 b0l, b0h, b1l, b1h;
	const float* kp = kb + (int64_t)s_begin * krow;  // chunk being prefetched
	sload32(b0l, b0h, kp);
	__builtin_amdgcn_sched_barrier(0);
	for (int s0 = s_begin; s0 < s_end; s0 += FWD_SJ) {
		// Pull the k rows of a later src block into the L2 with one vector load per wave (eight lanes per
		// row): the scalar loads below then miss the scalar cache but not the L2.  The value is not used;
		// it is taken before the flush, by which time it has long arrived.
		const float pf = kb[(int64_t)min(s0 + FWD_L2_AHEAD * FWD_SJ + (lane >> 3), Tn - 1) * krow + (lane & 7) * (W / 8)];
		float a = 0.0f;
		unsigned au = 0u;
#pragma unroll
		for (int c = 0; c < NCH; c++) {
			const int j = c / CPR, part = c % CPR;
			kp += (part == CPR - 1) ? krow - (CPR - 1) * 32 : 32;
			kp = kp < k_last ? kp : k_last;
			if ((c & 1) == 0) {
				swait32(b0l, b0h);
				__builtin_amdgcn_sched_barrier(0);
				sload32(b1l, b1h, kp);
				__builtin_amdgcn_sched_barrier(0);
				if (part == 0) { a = 0.0f; au = 0u; }
				if constexpr (FIXED) {
					sad8(au, &qr[part * 32], b0l, 0);
					sad8(au, &qr[part * 32 + 8], b0l, 8);
					sad8(au, &qr[part * 32 + 16], b0h, 0);
					sad8(au, &qr[part * 32 + 24], b0h, 8);
				} else {
#pragma unroll
					for (int i = 0; i < 16; i++) a += fabsf(qr[part * 32 + i] - b0l[i]);
#pragma unroll
					for (int i = 0; i < 16; i++) a += fabsf(qr[part * 32 + 16 + i] - b0h[i]);
				}
			} else {
				swait32(b1l, b1h);
				__builtin_amdgcn_sched_barrier(0);
				sload32(b0l, b0h, kp);
				__builtin_amdgcn_sched_barrier(0);
				if (part == 0) { a = 0.0f; au = 0u; }
				if constexpr (FIXED) {
					sad8(au, &qr[part * 32], b1l, 0);
					sad8(au, &qr[part * 32 + 8], b1l, 8);
					sad8(au, &qr[part * 32 + 16], b1h, 0);
					sad8(au, &qr[part * 32 + 24], b1h, 8);
				} else {
#pragma unroll
					for (int i = 0; i < 16; i++) a += fabsf(qr[part * 32 + i] - b1l[i]);
#pragma unroll
					for (int i = 0; i < 16; i++) a += fabsf(qr[part * 32 + 16 + i] - b1h[i]);
				}
			}
			if (part == CPR - 1) tile[j][(ts * WAVE + lane) * PH + hl] = FIXED ? (float)au * scale : a * scale;
		}
		asm volatile("" ::"v"(pf));
		lds_barrier();
#pragma unroll
		for (int j = 0; j < FWD_SJ; j++) {
			const int s = s0 + j;
			if (o_ok && s < s_end) {
				float r = tile[j][o_lds];
				for (int v = 1; v < V; v++) r += tile[j][o_lds + v];
				__builtin_nontemporal_store(r, &o_base[s * o_pitch]);
			}
		}
		lds_barrier();
	}
	swait32(b0l, b0h);  // drain the last prefetch before the wave ends
}

// ------------------------------------------------------------------------------------------
// fp32 backward, fast path
// ------------------------------------------------------------------------------------------

constexpr int BWD_SJ = 4;  // src tokens per staging step
constexpr int BWD_LDS_BATCH = 4;  // float4 reads of the staged tile issued together in the branch-free form
constexpr float BWD_PRESCALE = 18446744073709551616.0f;  // 2^64

// Raw buffer access for the branch-free step loop: a uniform base (descriptor in four SGPRs), a per-lane byte
// offset and a uniform byte offset.  Neither offset costs an instruction per access, where a flat global
// access takes a 64-bit VALU add for the address and scalar multiplies for the row.
using buf_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ buf_t make_buf(const void* base)
{
	return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);  // raw, no bounds below 4 GiB
}
__device__ __forceinline__ float buf_load(buf_t r, unsigned lane_bytes, unsigned uniform_bytes)
{
	return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_bytes, (int)uniform_bytes, 0));
}
__device__ __forceinline__ void buf_store(float v, buf_t r, unsigned lane_bytes, unsigned uniform_bytes)
{
	__builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, (int)lane_bytes, (int)uniform_bytes, 0);
}
// fp32 add in the L2, nothing returned
__device__ __forceinline__ void buf_add(float v, buf_t r, unsigned lane_bytes, unsigned uniform_bytes)
{
	__builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, r, (int)lane_bytes, (int)uniform_bytes, 0);
}

// Sum over each aligned group of 16 lanes (a DPP row); the total lands in the group's last lane.
// Lanes shifted in from outside the row read as zero.
template <int CTRL>
__device__ __forceinline__ float dpp_row_get(float x)
{
	return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_sum_to_last(float x)
{
	x += dpp_row_get<0x111>(x);  // row_shr:1
	x += dpp_row_get<0x112>(x);  // row_shr:2
	x += dpp_row_get<0x114>(x);  // row_shr:4
	x += dpp_row_get<0x118>(x);  // row_shr:8
	return x;
}

// grid.x = dst tiles of tt_rows tokens, grid.y = column chunks of blockDim.x, grid.z = batches.
// dkp: [n_ttiles][nb][T][HW] partials (or dk itself when there is a single dst tile).
//
// TT = dst tokens per workgroup: a lane keeps TT pre-scaled q values and TT dq sums in registers.
// Two families: TT 32 with up to 1024 threads (4 waves per SIMD), and TT 64..88 with up to 512
// threads (2 waves per SIMD, 256 registers each), which cuts the number of dk partials up to
// threefold; the host picks the TT that fills the chip most evenly.
// The workgroup stages dA only for the heads its columns belong to.
// PER = staged dA values per thread and step (ceil(BWD_SJ*tt_rows*heads / blockDim.x) <= PER).  The dA
// and k values of step n+1 are fetched into registers before the math of step n, so their latency
// is covered by a whole step of VALU work.
//
// RANK: q and k point to the column ranks rq and rk (rank minus one half) and the pair-elements
// take three instructions (pair_step4_rank).  The sums of g that turn sum(hv*g) into sum(sign*g)
// come from the staged tile; they are read before the step's math and added up after the math of
// its first src row, so that no wave waits for LDS: sixteen lanes per (src row, head) add up the
// TT values and store the column sum to csp [n_ttiles][nb][T][H] (the reduction kernel needs it),
// and every thread keeps the running sum over src rows of up to NR (head, dst token) slots (the
// row sums that dq needs after the loop).  dkp then holds the raw sum(hv*g) partials.
template <int TT, int MAXTHREADS, int PER, bool RANK, bool GROUPED, bool FAST, int DEEP = 0>
__global__ __launch_bounds__(MAXTHREADS) void dense_bwd_f32_fast(const float* __restrict__ dA,
                                                                   const float* __restrict__ q,
                                                                   const float* __restrict__ k,
                                                                   float* __restrict__ dq, float* __restrict__ dkp,
                                                                   float* __restrict__ csp, int Tn, int H, int W,
                                                                   float scale, int G)
{
	static_assert(!FAST || PER == BWD_SJ, "branch-free form: one staged value per thread and src row");
	constexpr int TTP = TT + 4;  // LDS row pitch: keeps 16-byte alignment for ds_read_b128
	constexpr int tt_rows = TT;
	constexpr int NR = (PER + BWD_SJ - 1) / BWD_SJ;  // (head, dst token) slots per thread, >= HB*TT / blockDim.x
	L1_DYNAMIC_LDS(float, gl);   // [BWD_SJ][HB][TTP]
	const unsigned HW = (unsigned)(H * W);
	const unsigned col0 = blockIdx.y * blockDim.x;
	const unsigned col_raw = col0 + threadIdx.x;
	// lanes past the last column shadow the chunk's first column: same inputs, same arithmetic, and
	// they store the same bits to the same addresses as the lane that owns that column
	const unsigned col = col_raw < HW ? col_raw : col0;
	const int h_lo = (int)(col0 / (unsigned)W);
	const unsigned col_end = min(HW, col0 + blockDim.x) - 1u;
	const int HB = (int)(col_end / (unsigned)W) - h_lo + 1;  // heads this workgroup touches
	const int hl = (int)(col / (unsigned)W) - h_lo;
	const int b = blockIdx.z, nb = gridDim.z;
	// wave-uniform row bases; lanes add the 32-bit column
	const float* const q_b = q + (int64_t)b * Tn * HW;
	const float* const k_b = k + (int64_t)b * Tn * HW;
	float* const dkp_b = dkp + ((int64_t)blockIdx.x * nb + b) * Tn * HW;
	// GROUPED: the workgroup takes G consecutive dst tiles one after the other and keeps one dk partial
	// for all of them: from the second tile on, a step adds to what the earlier tiles stored (same lane,
	// same address, in tile order), which cuts the partial arrays and the reduction G-fold.
	const int n_sub = GROUPED ? G : 1;
#pragma nounroll
	for (int u = 0; u < n_sub; u++) {
	const int tt = blockIdx.x * n_sub + u, t0 = tt * tt_rows;
	if (t0 >= Tn) break;
	const float* const dA_b = dA + ((int64_t)b * Tn * Tn + t0) * H + h_lo;
	float* const csp_b = RANK ? csp + ((int64_t)tt * nb + b) * Tn * H + h_lo : nullptr;

	float qc[TT], dqa[TT];
#pragma unroll
	for (int i = 0; i < TT; i++) {
		const int t = min(t0 + i, Tn - 1);
		const float v = (q_b + (int64_t)t * HW)[col];
		qc[i] = RANK ? v : v * BWD_PRESCALE;
		dqa[i] = 0.0f;
	}

	// staging roles of this thread: element e = threadIdx.x + r*blockDim.x of the [j][i][hh] step tile
	const int n_stage = BWD_SJ * tt_rows * HB;
	int st_j[PER], st_lds[PER];
	unsigned st_off[PER];  // within the step's BWD_SJ src rows of dA: below 2^31 (checked by the host)
	bool st_ok[PER];
#pragma unroll
	for (int r = 0; r < PER; r++) {
		const int e = threadIdx.x + r * blockDim.x;
		const int j = e / (tt_rows * HB), rr = e % (tt_rows * HB);
		const int i = rr / HB, hh = rr % HB;
		st_j[r] = j;
		st_ok[r] = e < n_stage && t0 + i < Tn;
		st_off[r] = ((unsigned)j * (unsigned)Tn + (unsigned)i) * (unsigned)H + (unsigned)hh;
		st_lds[r] = e < n_stage ? (j * HB + hh) * TTP + i : -1;
	}
	// RANK: row-sum slots of this thread, slot = hh*TT + i -> LDS offset hh*TTP + i of the j = 0 plane
	int rs_lds[NR];
	float rs_acc[NR];
#pragma unroll
	for (int n = 0; n < NR; n++) {
		const int slot = threadIdx.x + n * blockDim.x;
		rs_lds[n] = slot < HB * tt_rows ? (slot / tt_rows) * TTP + slot % tt_rows : -1;
		rs_acc[n] = 0.0f;
	}
	float g_pre[PER], k_pre[BWD_SJ];
	// interior tile with every staging role in use: the loads and LDS writes need no per-lane predicates.
	// FAST: the host found this to hold for every workgroup of the launch, T a multiple of BWD_SJ and no
	// idle lanes; the step loop is then compiled without a single branch around a memory access (the
	// branches of the general form cost about 4 % of the kernel).
	const bool full = FAST || (t0 + tt_rows <= Tn && n_stage == PER * (int)blockDim.x);
	// loads of the dA and k values of the step that starts at src token s0
	// FAST: running uniform pointers instead of a multiplication per row: the step being prefetched (dA, k)
	// and the step being computed (dk partial rows)
	const float* dA_pf = dA_b;
	const float* k_pf = k_b;
	float* dkp_cur = dkp_b;
	const unsigned row_bytes = HW * 4u, dA_row_bytes = (unsigned)(Tn * H) * 4u, col_bytes = col * 4u;
	const int64_t dA_step = (int64_t)BWD_SJ * Tn * H, k_step = (int64_t)BWD_SJ * HW;
	auto prefetch = [&](int s0) {
		if (FAST) {
			// PER == BWD_SJ and blockDim.x elements per src row: role r is role 0 one src row further on
			const buf_t rd = make_buf(dA_pf), rk = make_buf(k_pf);
#pragma unroll
			for (int r = 0; r < PER; r++) g_pre[r] = buf_load(rd, st_off[0] * 4u, (unsigned)r * dA_row_bytes);
#pragma unroll
			for (int j = 0; j < BWD_SJ; j++) k_pre[j] = buf_load(rk, col_bytes, (unsigned)j * row_bytes);
			return;
		}
		const float* const dA_s = dA_b + (int64_t)s0 * Tn * H;  // wave-uniform
		if (full && s0 + BWD_SJ <= Tn) {
#pragma unroll
			for (int r = 0; r < PER; r++) g_pre[r] = dA_s[st_off[r]];
		} else {
#pragma unroll
			for (int r = 0; r < PER; r++) {
				g_pre[r] = 0.0f;
				if (st_ok[r] && s0 + st_j[r] < Tn) g_pre[r] = dA_s[st_off[r]];
			}
		}
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) k_pre[j] = (k_b + (int64_t)min(s0 + j, Tn - 1) * HW)[col];
	};
	// Wait for the prefetched values.  Loads and stores share one counter and may complete out of
	// order, so a wait for a load while a store is in flight is a wait for everything.  The values
	// are therefore taken before a step's stores are issued (the loads are a whole step old by then),
	// and before the loop for the first step: otherwise each step's first use of them also waits for
	// the previous step's stores to be acknowledged.
	auto settle = [&]() {
#pragma unroll
		for (int r = 0; r < PER; r++) asm volatile("" : "+v"(g_pre[r]));
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) asm volatile("" : "+v"(k_pre[j]));
	};
	if constexpr (DEEP != 0) {
	// Two steps of prefetch distance.  With one (below), the wait at the end of a step is for the youngest
	// vector-memory operations of the wave, i.e. for everything: the loads of the next step's values and, older
	// than those, the dk stores of the step before and the column-sum store of this one.  Here two register sets
	// alternate: the set a step has just put into LDS is refilled with the values of the step after next, and
	// the wait at the end of the step is for the other set, whose loads are a whole step old; the stores issued
	// since (this step's column sums, the previous step's dk rows) and the refill stay in flight across it.
	// The step loop runs two steps per iteration, so that the sets are fixed registers.
	// DEEP == 2: the two steps of an iteration also stage their tiles in two LDS planes (the host then gives the
	// workgroup twice the LDS), and a step has one barrier instead of two.  The barrier that kept a step's LDS
	// writes behind the previous step's reads is not needed: a thread writes plane p for step n+2 only after
	// the barrier of step n+1, which every thread reaches after its reads of plane p in step n.
	static_assert(DEEP == 0 || FAST, "two-step prefetch: branch-free form only");
	float g_a[PER], k_a[BWD_SJ], g_b[PER], k_b[BWD_SJ];
	auto fetch = [&](float (&g)[PER], float (&kk)[BWD_SJ]) {
		const buf_t rd = make_buf(dA_pf), rk = make_buf(k_pf);
#pragma unroll
		for (int r = 0; r < PER; r++) g[r] = buf_load(rd, st_off[0] * 4u, (unsigned)r * dA_row_bytes);
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) kk[j] = buf_load(rk, col_bytes, (unsigned)j * row_bytes);
	};
	auto arrived = [&](float (&g)[PER], float (&kk)[BWD_SJ]) {
#pragma unroll
		for (int r = 0; r < PER; r++) asm volatile("" : "+v"(g[r]));
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) asm volatile("" : "+v"(kk[j]));
	};
	// one step: g_use / k_use hold its values (arrived); g_nxt / k_nxt are in flight for the step after it
	float* const gl_planes = gl;
	auto step = [&](const int s0, float (&g_use)[PER], float (&k_use)[BWD_SJ], float (&g_nxt)[PER], float (&k_nxt)[BWD_SJ],
	                const int plane) {
		float* const gl = gl_planes + plane * (BWD_SJ * HB * TTP);  // (hides the workgroup's array: this step's plane)
		if (DEEP != 2) lds_barrier();  // the previous step's LDS reads are done
#pragma unroll
		for (int r = 0; r < PER; r++) gl[st_lds[0] + r * HB * TTP] = g_use[r];
		float kc[BWD_SJ], dka[BWD_SJ];
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) {
			kc[j] = RANK ? k_use[j] : k_use[j] * BWD_PRESCALE;
			dka[j] = 0.0f;
		}
		lds_barrier();
		// the step after next into the set just consumed; the last two steps read rows they have read before
		const bool more = s0 + 2 * BWD_SJ < Tn;
		dA_pf += more ? dA_step : 0;
		k_pf += more ? k_step : 0;
		fetch(g_use, k_use);
		const buf_t rp = make_buf(dkp_cur);
		{
			// All dA values of this step for the lane's head, each float4 read D blocks ahead of its use, one read
			// between two blocks of math.  Every instruction of a wave takes an issue slot, an s_waitcnt too: the
			// branch-free form waits once per BL blocks instead of once per block (LDS reads return in order, so
			// blocks bi..bi+BL-1 are there once no more than the D-BL+1 reads issued after them are outstanding).
			const float4* gp0 = reinterpret_cast<const float4*>(gl + hl * TTP);
			constexpr int NI4 = TT / 4, NBLK = BWD_SJ * NI4, BL = FAST ? BWD_LDS_BATCH : 1, D = 2 * BL - 1, RING = D + 1;
			auto g_at = [&](int bi) { return gp0[((bi / NI4) * HB * TTP) / 4 + bi % NI4]; };
			float4 g_ring[RING];
#pragma unroll
			for (int d = 0; d < D; d++) g_ring[d] = g_at(d);
			// RANK: the tile values for the sums are read here and added up after the first src row's math,
			// by which time they have arrived.  Column sums: row = jj*HB + hh of the tile, sixteen lanes per
			// row (the host checks BWD_SJ*HB*16 <= blockDim.x).  Row sums: this thread's (head, dst token) slots.
			constexpr int NM = (TT / 4 + 15) / 16;
			const int cs_sub = threadIdx.x & 15, cs_row = threadIdx.x >> 4;
			float4 cs_v[NM];
			float rs_v[NR][BWD_SJ];
			if (RANK) {
				const float4* rp = reinterpret_cast<const float4*>(gl + cs_row * TTP);
#pragma unroll
				for (int m = 0; m < NM; m++) {
					cs_v[m] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
					// FAST (64-token tiles, 64*HB threads): every group of sixteen lanes has a row, every lane a float4
					if (FAST || (cs_row < BWD_SJ * HB && cs_sub + 16 * m < TT / 4)) cs_v[m] = rp[cs_sub + 16 * m];
				}
#pragma unroll
				for (int n = 0; n < NR; n++) {
#pragma unroll
					for (int jj = 0; jj < BWD_SJ; jj++) rs_v[n][jj] = (FAST || rs_lds[n] >= 0) ? gl[jj * HB * TTP + rs_lds[n]] : 0.0f;
				}
			}
#pragma unroll
			for (int bi = 0; bi < NBLK; bi++) {
				{
					const int j = bi / NI4, i4 = bi % NI4;
					if (bi + D < NBLK) g_ring[(bi + D) % RING] = g_at(bi + D);
					if (BL > 1 && bi > 0 && bi % BL == 0) {
						// s_waitcnt immediate: vmcnt and expcnt at their maxima, lgkmcnt in bits 11:8
						if (bi + BL < NBLK) __builtin_amdgcn_s_waitcnt(0xC07F | ((D - BL + 1) << 8));
						else __builtin_amdgcn_s_waitcnt(0xC07F);
					}
					__builtin_amdgcn_sched_barrier(0);
					if (RANK && j == 1 && i4 == 0) {
						// keep the loaded values opaque up to here, or the adds (and the wait for the loads)
						// are hoisted in front of the first src row's math
#pragma unroll
						for (int m = 0; m < NM; m++)
							asm volatile("" : "+v"(cs_v[m].x), "+v"(cs_v[m].y), "+v"(cs_v[m].z), "+v"(cs_v[m].w));
#pragma unroll
						for (int n = 0; n < NR; n++) {
#pragma unroll
							for (int jj = 0; jj < BWD_SJ; jj++) asm volatile("" : "+v"(rs_v[n][jj]));
						}
						float a = 0.0f;
#pragma unroll
						for (int m = 0; m < NM; m++) a += (cs_v[m].x + cs_v[m].y) + (cs_v[m].z + cs_v[m].w);
						a = row16_sum_to_last(a);
						const int jj = cs_row / HB, s = s0 + jj;
						if (cs_sub == 15 && (FAST || (cs_row < BWD_SJ * HB && s < Tn))) csp_b[(int64_t)s * H + (cs_row - jj * HB)] = a;
#pragma unroll
						for (int n = 0; n < NR; n++) rs_acc[n] += (rs_v[n][0] + rs_v[n][1]) + (rs_v[n][2] + rs_v[n][3]);
						__builtin_amdgcn_sched_barrier(0);
					}
					if (RANK) pair_step4_rank(&qc[i4 * 4], kc[j], g_ring[bi % RING], &dqa[i4 * 4], dka[j]);
					else pair_step4(&qc[i4 * 4], kc[j], g_ring[bi % RING], &dqa[i4 * 4], dka[j]);
				}
			}
		}
		arrived(g_nxt, k_nxt);
		if (!GROUPED || u == 0) {
#pragma unroll
			for (int j = 0; j < BWD_SJ; j++) buf_store(RANK ? dka[j] : dka[j] * scale, rp, col_bytes, (unsigned)j * row_bytes);
		} else {
#pragma unroll
			for (int j = 0; j < BWD_SJ; j++) buf_add(RANK ? dka[j] : dka[j] * scale, rp, col_bytes, (unsigned)j * row_bytes);
		}
		dkp_cur += (int64_t)BWD_SJ * HW;
	};
	fetch(g_a, k_a);  // step 0
	dA_pf += BWD_SJ < Tn ? dA_step : 0;
	k_pf += BWD_SJ < Tn ? k_step : 0;
	fetch(g_b, k_b);  // step 1
	arrived(g_a, k_a);
	// one barrier per dst tile where the steps have none before their LDS writes: the rank form's row sums of the
	// workgroup's previous tile are read from plane 0 after its last barrier
	if (DEEP == 2) lds_barrier();
	for (int s0 = 0; s0 < Tn; s0 += 2 * BWD_SJ) {  // (the host picks this form only for T a multiple of 2*BWD_SJ)
		step(s0, g_a, k_a, g_b, k_b, 0);
		step(s0 + BWD_SJ, g_b, k_b, g_a, k_a, DEEP == 2 ? 1 : 0);
	}
	} else {
	prefetch(0);
	settle();

	for (int s0 = 0; s0 < Tn; s0 += BWD_SJ) {
		lds_barrier();  // the previous step's LDS reads are done
		if (FAST) {
#pragma unroll
			for (int r = 0; r < PER; r++) gl[st_lds[0] + r * HB * TTP] = g_pre[r];
		} else if (full) {
#pragma unroll
			for (int r = 0; r < PER; r++) gl[st_lds[r]] = g_pre[r];
		} else {
#pragma unroll
			for (int r = 0; r < PER; r++)
				if (st_lds[r] >= 0) gl[st_lds[r]] = g_pre[r];
		}
		float kc[BWD_SJ], dka[BWD_SJ];
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) {
			kc[j] = RANK ? k_pre[j] : k_pre[j] * BWD_PRESCALE;
			dka[j] = 0.0f;
		}
		lds_barrier();
		// next step's values; FAST: the last step reads its own rows again, and nobody uses them
		if (FAST) {
			const bool more = s0 + BWD_SJ < Tn;
			dA_pf += more ? dA_step : 0;
			k_pf += more ? k_step : 0;
			prefetch(more ? s0 + BWD_SJ : s0);
		} else if (s0 + BWD_SJ < Tn) prefetch(s0 + BWD_SJ);
		// what the earlier tiles of this workgroup left in the partial rows of this step; used after the math
		float dk_old[BWD_SJ];
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) dk_old[j] = 0.0f;
		const buf_t rp = make_buf(dkp_cur);
		if (GROUPED && FAST) {
			// nothing to load: the later tiles add to the stored rows in the L2 (below)
		} else if (GROUPED && u > 0) {
#pragma unroll
			for (int j = 0; j < BWD_SJ; j++) dk_old[j] = (dkp_b + (int64_t)min(s0 + j, Tn - 1) * HW)[col];
		}
		{
			// All dA values of this step for the lane's head, each float4 read D blocks ahead of its use, one read
			// between two blocks of math.  Every instruction of a wave takes an issue slot, an s_waitcnt too: the
			// branch-free form waits once per BL blocks instead of once per block (LDS reads return in order, so
			// blocks bi..bi+BL-1 are there once no more than the D-BL+1 reads issued after them are outstanding).
			const float4* gp0 = reinterpret_cast<const float4*>(gl + hl * TTP);
			constexpr int NI4 = TT / 4, NBLK = BWD_SJ * NI4, BL = FAST ? BWD_LDS_BATCH : 1, D = 2 * BL - 1, RING = D + 1;
			auto g_at = [&](int bi) { return gp0[((bi / NI4) * HB * TTP) / 4 + bi % NI4]; };
			float4 g_ring[RING];
#pragma unroll
			for (int d = 0; d < D; d++) g_ring[d] = g_at(d);
			// RANK: the tile values for the sums are read here and added up after the first src row's math,
			// by which time they have arrived.  Column sums: row = jj*HB + hh of the tile, sixteen lanes per
			// row (the host checks BWD_SJ*HB*16 <= blockDim.x).  Row sums: this thread's (head, dst token) slots.
			constexpr int NM = (TT / 4 + 15) / 16;
			const int cs_sub = threadIdx.x & 15, cs_row = threadIdx.x >> 4;
			float4 cs_v[NM];
			float rs_v[NR][BWD_SJ];
			if (RANK) {
				const float4* rp = reinterpret_cast<const float4*>(gl + cs_row * TTP);
#pragma unroll
				for (int m = 0; m < NM; m++) {
					cs_v[m] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
					// FAST (64-token tiles, 64*HB threads): every group of sixteen lanes has a row, every lane a float4
					if (FAST || (cs_row < BWD_SJ * HB && cs_sub + 16 * m < TT / 4)) cs_v[m] = rp[cs_sub + 16 * m];
				}
#pragma unroll
				for (int n = 0; n < NR; n++) {
#pragma unroll
					for (int jj = 0; jj < BWD_SJ; jj++) rs_v[n][jj] = (FAST || rs_lds[n] >= 0) ? gl[jj * HB * TTP + rs_lds[n]] : 0.0f;
				}
			}
#pragma unroll
			for (int bi = 0; bi < NBLK; bi++) {
				{
					const int j = bi / NI4, i4 = bi % NI4;
					if (bi + D < NBLK) g_ring[(bi + D) % RING] = g_at(bi + D);
					if (BL > 1 && bi > 0 && bi % BL == 0) {
						// s_waitcnt immediate: vmcnt and expcnt at their maxima, lgkmcnt in bits 11:8
						if (bi + BL < NBLK) __builtin_amdgcn_s_waitcnt(0xC07F | ((D - BL + 1) << 8));
						else __builtin_amdgcn_s_waitcnt(0xC07F);
					}
					__builtin_amdgcn_sched_barrier(0);
					if (RANK && j == 1 && i4 == 0) {
						// keep the loaded values opaque up to here, or the adds (and the wait for the loads)
						// are hoisted in front of the first src row's math
#pragma unroll
						for (int m = 0; m < NM; m++)
							asm volatile("" : "+v"(cs_v[m].x), "+v"(cs_v[m].y), "+v"(cs_v[m].z), "+v"(cs_v[m].w));
#pragma unroll
						for (int n = 0; n < NR; n++) {
#pragma unroll
							for (int jj = 0; jj < BWD_SJ; jj++) asm volatile("" : "+v"(rs_v[n][jj]));
						}
						float a = 0.0f;
#pragma unroll
						for (int m = 0; m < NM; m++) a += (cs_v[m].x + cs_v[m].y) + (cs_v[m].z + cs_v[m].w);
						a = row16_sum_to_last(a);
						const int jj = cs_row / HB, s = s0 + jj;
						if (cs_sub == 15 && (FAST || (cs_row < BWD_SJ * HB && s < Tn))) csp_b[(int64_t)s * H + (cs_row - jj * HB)] = a;
#pragma unroll
						for (int n = 0; n < NR; n++) rs_acc[n] += (rs_v[n][0] + rs_v[n][1]) + (rs_v[n][2] + rs_v[n][3]);
						__builtin_amdgcn_sched_barrier(0);
					}
					if (RANK) pair_step4_rank(&qc[i4 * 4], kc[j], g_ring[bi % RING], &dqa[i4 * 4], dka[j]);
					else pair_step4(&qc[i4 * 4], kc[j], g_ring[bi % RING], &dqa[i4 * 4], dka[j]);
				}
			}
		}
		settle();
		if (FAST) {
			// GROUPED: the first tile stores, the others add in the L2: same lane, same address, tile order, so
			// the sums are formed in the order a load, add and store would form them (and repeat bit for bit),
			// without the load and its wait
			if (!GROUPED || u == 0) {
#pragma unroll
				for (int j = 0; j < BWD_SJ; j++) buf_store(RANK ? dka[j] : dka[j] * scale, rp, col_bytes, (unsigned)j * row_bytes);
			} else {
#pragma unroll
				for (int j = 0; j < BWD_SJ; j++) buf_add(RANK ? dka[j] : dka[j] * scale, rp, col_bytes, (unsigned)j * row_bytes);
			}
			dkp_cur += (int64_t)BWD_SJ * HW;
			continue;
		}
		// unconditional in the lane dimension: a store guarded by a per-lane predicate would let the
		// compiler sink the dk chain into the guarded block and split the four-instruction groups
#pragma unroll
		for (int j = 0; j < BWD_SJ; j++) {
			const int s = s0 + j;
			const float v = RANK ? dka[j] : dka[j] * scale;
			if (FAST || s < Tn) (dkp_b + (int64_t)s * HW)[col] = GROUPED ? dk_old[j] + v : v;
		}
	}
	}  // one or two steps of prefetch distance
	float* const dq_b = dq + (int64_t)b * Tn * HW;
	if (RANK) {
		lds_barrier();  // the last step's tile reads are done
		// exchange the row sums through the j = 0 plane of the tile: [hh][TTP]
#pragma unroll
		for (int n = 0; n < NR; n++)
			if (rs_lds[n] >= 0) gl[rs_lds[n]] = rs_acc[n];
		lds_barrier();
		const float4* rp = reinterpret_cast<const float4*>(gl + hl * TTP);
#pragma unroll
		for (int i4 = 0; i4 < TT / 4; i4++) {
			const float4 r4 = rp[i4];
			const float rr[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
			for (int u = 0; u < 4; u++) {
				const int t = t0 + i4 * 4 + u;
				if (FAST || t < Tn) (dq_b + (int64_t)t * HW)[col] = (2.0f * dqa[i4 * 4 + u] - rr[u]) * scale;
			}
		}
	} else {
#pragma unroll
		for (int i = 0; i < TT; i++) {
			const int t = t0 + i;
			if (FAST || t < Tn) (dq_b + (int64_t)t * HW)[col] = dqa[i] * scale;
		}
	}
	}  // dst tiles of the workgroup
}

// One (b, s, h) element per thread: the column sums of all dst tiles, in tile order.
__global__ __launch_bounds__(256) void dense_bwd_reduce_colsum(const float* __restrict__ csp, float* __restrict__ cs,
                                                                 int64_t n, int n_tt)
{
	const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (i >= n) return;
	float acc = csp[i];
	for (int tt = 1; tt < n_tt; tt++) acc += csp[(int64_t)tt * n + i];
	cs[i] = acc;
}

// dk[i] = sum over dst tiles, in tile order, of the partials; n = nb*T*HW elements per tile.
// VEC: n and both base pointers are multiples of 4 floats (RANK: and so is W).
// RANK: the partials are sums of hv*g; with the column sums cs [nb][T][H] of g,
//   dk = scale * (cs - 2 * sum of partials).
// AHEAD (opt-in, with the pipelined step loops): the partial arrays are read four at a time.  Left to the compiler
// the loop is one load and a wait for it per partial array, i.e. as many memory round trips in a row as there are
// partial arrays, and the kernel runs at what the occupancy can cover of that latency (4.7 of 8 TB/s measured at
// sixteen arrays).  The adds stay in tile order, so the result is the same bit for bit.
template <bool VEC, bool RANK, bool AHEAD = false>
__global__ __launch_bounds__(256) void dense_bwd_reduce_dk(const float* __restrict__ dkp, float* __restrict__ dk,
                                                             int64_t n, int n_tt, const float* __restrict__ cs,
                                                             int HW, int W, int H, float scale)
{
	if (VEC) {
		const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
		if (i >= n) return;
		float4 acc = *reinterpret_cast<const float4*>(dkp + i);
		if constexpr (AHEAD) {
			static_assert(!AHEAD || VEC, "reads ahead in the vector form only");
			int tt = 1;
			for (; tt + 3 < n_tt; tt += 4) {
				float4 p[4];
#pragma unroll
				for (int u = 0; u < 4; u++) p[u] = *reinterpret_cast<const float4*>(dkp + (int64_t)(tt + u) * n + i);
#pragma unroll
				for (int u = 0; u < 4; u++) { acc.x += p[u].x; acc.y += p[u].y; acc.z += p[u].z; acc.w += p[u].w; }
			}
			for (; tt < n_tt; tt++) {
				const float4 p = *reinterpret_cast<const float4*>(dkp + (int64_t)tt * n + i);
				acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
			}
		} else {
		for (int tt = 1; tt < n_tt; tt++) {
			const float4 p = *reinterpret_cast<const float4*>(dkp + (int64_t)tt * n + i);
			acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
		}
		}
		if (RANK) {
			const float c = cs[(i / HW) * H + (int)(i % HW) / W];
			acc.x = (c - 2.0f * acc.x) * scale; acc.y = (c - 2.0f * acc.y) * scale;
			acc.z = (c - 2.0f * acc.z) * scale; acc.w = (c - 2.0f * acc.w) * scale;
		}
		*reinterpret_cast<float4*>(dk + i) = acc;
	} else {
		const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
		if (i >= n) return;
		float acc = dkp[i];
		for (int tt = 1; tt < n_tt; tt++) acc += dkp[(int64_t)tt * n + i];
		if (RANK) acc = (cs[(i / HW) * H + (int)(i % HW) / W] - 2.0f * acc) * scale;
		dk[i] = acc;
	}
}

// qp, kp: rows of q, k copied to width WP and filled up with zeros; n = rows*WP, grid-stride
__global__ __launch_bounds__(256) void dense_pad_rows(const float* __restrict__ q, const float* __restrict__ k,
                                                        float* __restrict__ qp, float* __restrict__ kp, int64_t n, int W,
                                                        int WP)
{
	for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
		const int64_t row = i / WP;
		const int w = (int)(i - row * WP);
		qp[i] = w < W ? q[row * W + w] : 0.0f;
		kp[i] = w < W ? k[row * W + w] : 0.0f;
	}
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------

bool shape_ok(int64_t B, int64_t T, int64_t H, int64_t W)
{
	return B >= 0 && T >= 0 && H >= 0 && W >= 0;
}

template <typename T>
int launch_fwd_generic(const T* q, const T* k, T* attn, int64_t B, int64_t Tn, int64_t H, int64_t W, hipStream_t st)
{
	const T scale = (T)(-1.0 / sqrt((double)W));
	const size_t small_bytes = (size_t)2 * Tn * (W + 1) * sizeof(T);
	if (Tn <= 64 && small_bytes <= 48 * 1024 && B * H < ((int64_t)1 << 31)) {
		hipLaunchKernelGGL(dense_fwd_small<T>, dim3((unsigned)(B * H)), dim3(256), small_bytes, st, q, k, attn, (int)Tn,
		                   (int)H, (int)W, scale);
		L1_LAUNCH_CHECK();
		return L1ATTN_OK;
	}
	if (Tn * H >= ((int64_t)1 << 32)) return L1ATTN_ERR_RANGE;  // threads along x of one launch
	dim3 grid((unsigned)l1_cdiv(Tn * H, 256), (unsigned)std::min<int64_t>(B * Tn, 65535), 1);
	hipLaunchKernelGGL(dense_fwd_generic<T>, grid, dim3(256), 0, st, q, k, attn, B, Tn, H, W, scale);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

template <typename T>
int launch_bwd_generic(const T* dA, const T* q, const T* k, T* dq, T* dk, int64_t B, int64_t Tn, int64_t H,
                       int64_t W, hipStream_t st)
{
	const T scale = (T)(-1.0 / sqrt((double)W));
	const int64_t n = B * Tn * H * W;
	if (n >= ((int64_t)1 << 32)) return L1ATTN_ERR_RANGE;  // one thread per gradient element
	dim3 grid((unsigned)l1_cdiv(n, 256));
	hipLaunchKernelGGL(dense_bwd_generic_dq<T>, grid, dim3(256), 0, st, dA, q, k, dq, B, Tn, H, W, scale);
	L1_LAUNCH_CHECK();
	hipLaunchKernelGGL(dense_bwd_generic_dk<T>, grid, dim3(256), 0, st, dA, q, k, dk, B, Tn, H, W, scale);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

// heads per workgroup and dst sub-tiles per workgroup of the fast forward.  All heads of a dst tile
// in one workgroup keeps the output runs whole 64-byte lines; splitting the heads over two
// workgroups (NH 8, NTS 2, two waves sharing each k row) measured slower.
void fwd_shape(int64_t H, int64_t T, int& NH, int& NTS)
{
	(void)T;
	NH = (int)(H < 16 ? H : 16);
	NTS = 1;
}

// fast forward: W a multiple of 16 up to 128, 16-byte aligned rows, at least half a wave of tokens
bool fwd_fast_ok(const float* q, const float* k, int64_t B, int64_t T, int64_t H, int64_t W)
{
	if (W < 16 || W > 128 || (W % 16) != 0 || T < 32) return false;
	if ((((uintptr_t)q) | ((uintptr_t)k)) & 15) return false;
	if (W == 128) H *= 2;  // run as half-heads, see launch_fwd_fast()
	int NH, NTS;
	fwd_shape(H, T, NH, NTS);
	const int64_t n_hg = l1_cdiv(H, NH);
	return B * n_hg <= 65535 && T <= (1 << 30) && H <= 65535;
}

// W: width of the rows the kernels read; W_scale: width the logits are scaled by (smaller when the rows are
// zero-padded copies)
// gq != nullptr: q and k are the fixed-point copies and gq their grids (widths 32 and 64 only)
int launch_fwd_fast(const float* q, const float* k, float* attn, int64_t B, int64_t Tn, int64_t H, int64_t W,
                    int64_t W_scale, hipStream_t st, const float* gq = nullptr)
{
	// width 128 runs the pipelined width-64 kernel on half-heads (128 q registers per lane do not leave room
	// for four waves per SIMD)
	const int V = W == 128 ? 2 : 1;
	H *= V;
	W /= V;
	int NH, NTS;
	fwd_shape(H, Tn, NH, NTS);
	const int NW = NH * NTS;
	const int n_hg = (int)l1_cdiv(H, NH);
	const int n_tt = (int)l1_cdiv(Tn, WAVE * NTS);
	// split the src range so that the launch has a few thousand workgroups, in multiples of FWD_SJ
	int64_t want_chunks = l1_cdiv(2048, (int64_t)n_tt * B * n_hg);
	int64_t s_chunk = l1_cdiv(l1_cdiv(Tn, want_chunks), FWD_SJ) * FWD_SJ;
	if (s_chunk < 64) s_chunk = 64;
	int n_sc = (int)l1_cdiv(Tn, s_chunk);
	if (n_sc > 65535) { s_chunk = l1_cdiv(l1_cdiv(Tn, 65535), FWD_SJ) * FWD_SJ; n_sc = (int)l1_cdiv(Tn, s_chunk); }
	const float scale = (float)(-1.0 / sqrt((double)W_scale));
	dim3 grid(n_tt, n_sc, (unsigned)(B * n_hg)), block(64 * NW);
#define L1_FWD_CASE(KERNEL, WV)                                                                                  \
	case WV:                                                                                                     \
		hipLaunchKernelGGL(KERNEL<WV>, grid, block, 0, st, q, k, attn, (int)Tn, (int)H, n_hg, NH, (int)s_chunk,    \
		                   scale);                                                                               \
		break
#define L1_FWD_PIPE_CASE(WV)                                                                                     \
	case WV:                                                                                                     \
		hipLaunchKernelGGL((dense_fwd_f32_pipe<WV, false>), grid, block, 0, st, q, k, attn, (int)Tn, (int)H, n_hg, \
		                   NH, (int)s_chunk, scale, V, (const float*)nullptr);                                   \
		break
	if (gq) {
		if (V != 1 || (W != 32 && W != 64)) return L1ATTN_ERR_ARG;
		if (W == 32)
			hipLaunchKernelGGL((dense_fwd_f32_pipe<32, true>), grid, block, 0, st, q, k, attn, (int)Tn, (int)H, n_hg, NH,
			                   (int)s_chunk, scale, V, gq);
		else
			hipLaunchKernelGGL((dense_fwd_f32_pipe<64, true>), grid, block, 0, st, q, k, attn, (int)Tn, (int)H, n_hg, NH,
			                   (int)s_chunk, scale, V, gq);
		L1_LAUNCH_CHECK();
		return L1ATTN_OK;
	}
	switch (W) {
		L1_FWD_CASE(dense_fwd_f32_fast, 16); L1_FWD_PIPE_CASE(32);
		L1_FWD_CASE(dense_fwd_f32_fast, 48); L1_FWD_PIPE_CASE(64);
		L1_FWD_CASE(dense_fwd_f32_fast, 80); L1_FWD_PIPE_CASE(96);
		L1_FWD_CASE(dense_fwd_f32_fast, 112);
	default: return L1ATTN_ERR_ARG;
	}
#undef L1_FWD_CASE
#undef L1_FWD_PIPE_CASE
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

struct BwdPlan {
	bool fast;
	bool wide;        // TT 64..88 / 512-thread instantiation
	bool rank;        // three-instruction pair-elements on column ranks
	int threads, n_cc, n_tt, tt_rows, per;
	bool branch_free;        // every workgroup of the launch runs whole tiles and whole steps
	int deep;                // branch-free form with two steps of prefetch distance (1), and two LDS planes (2); on request
	int group, n_groups;     // consecutive dst tiles per workgroup (sharing one dk partial); workgroups along T
	size_t lds_bytes;
	size_t partial_bytes;    // partial-dk scratch for one batch (0 when a single dst tile)
	size_t rank_bytes;       // rq and rk of one batch (0 unless rank)
	size_t per_batch_bytes;  // workspace share of one batch
	size_t flag_bytes;       // head of the workspace that holds the sign-domain flag (0 with column ranks)
};

constexpr int N_CU = 256;
constexpr size_t BWD_FLAG_BYTES = 256;  // keeps what follows the flag 256-byte aligned

// loop_form: form of the branch-free step loop.  0: one step of prefetch distance (what l1attn_dense_bwd_f32
// runs); 1: two steps; 2: two steps, two LDS planes and one barrier per step.  Same sums in the same order in all
// three, so the results are bit-identical.  Shapes whose plan is not branch-free ignore it.
BwdPlan bwd_plan(int64_t B, int64_t T, int64_t H, int64_t W, int loop_form = 0)
{
	BwdPlan p{};
	const int64_t HW = H * W;
	p.fast = B >= 1 && T >= 16 && HW >= 32 && T <= (1 << 30) && B <= 65535 && HW <= (int64_t)512 * 65535 &&
	         (BWD_SJ * T + 128) * H < ((int64_t)1 << 31);  // 32-bit staging offsets
	if (!p.fast) return p;
	// wide tiles (one workgroup of up to 8 waves per CU) pay off once every CU gets its two waves per SIMD
	const int64_t wide_threads = std::min<int64_t>(512, l1_cdiv(HW, 64) * 64);
	p.wide = T >= 1024 && B * l1_cdiv(HW, wide_threads) * l1_cdiv(T, 64) * (wide_threads / 64) >= 8 * N_CU;
	int maxthreads = p.wide ? 512 : 1024;
	// narrow tiles: halve the workgroups rather than leave CUs without one
	if (!p.wide && HW >= 1024 && B * l1_cdiv(HW, 1024) * l1_cdiv(T, 32) < N_CU) maxthreads = 512;
	p.threads = (int)std::min<int64_t>(maxthreads, l1_cdiv(HW, 64) * 64);
	p.n_cc = (int)l1_cdiv(HW, p.threads);
	int64_t hb_exact = 1;  // most heads any column chunk touches
	for (int64_t cc = 0; cc < p.n_cc; cc++) {
		const int64_t c0 = cc * p.threads, c1 = std::min<int64_t>(HW, c0 + p.threads) - 1;
		hb_exact = std::max<int64_t>(hb_exact, c1 / W - c0 / W + 1);
	}
	// The rank transform costs O(T log T) per column against O(T^2) saved instructions: it pays off for
	// long sequences, and one workgroup must be able to sort a column in LDS.
	// Its column sums use sixteen lanes per (src row, head) of a step.
	p.rank = p.wide && T >= 2048 && l1_column_ranks_ok(B, T, H, W) && BWD_SJ * hb_exact * 16 <= p.threads;
	p.tt_rows = p.wide ? 88 : 32;
	p.group = 1;
	if (p.wide) {
		// Eight waves per CU at a time: one workgroup of 512 threads, two of 256.  Pick the tile height and the
		// tiles per workgroup that waste the least of the last round of workgroups; every partial array costs
		// a write in the main kernel and a read in the reduction (0.04 tile rows per array, batch and column
		// chunk, measured).
		double best = 1e30;
		const int tr_max = p.rank ? 80 : 88;  // the rank variant keeps a few more values in registers
		const int64_t slots = (int64_t)N_CU * (512 / p.threads);
		// tiles are grouped only where the branch-free step loop runs (whole 64-token tiles, whole column
		// chunks, heads of 64 columns): that is the form whose later tiles add to the partial in the L2
		const bool can_group = T % 64 == 0 && T % BWD_SJ == 0 && HW % p.threads == 0 && p.threads % W == 0 &&
		                       (int64_t)BWD_SJ * 64 * (p.threads / W) == (int64_t)4 * p.threads &&
		                       (BWD_SJ * T + 128) * H < ((int64_t)1 << 29);
		for (int tr = 64; tr <= tr_max; tr += 8) {
			for (int g = 1; g <= 8; g *= 2) {
				const int64_t ngr = l1_cdiv(l1_cdiv(T, tr), g);
				const int64_t wgs = B * p.n_cc * ngr;
				// tiles are grouped only in the 64-token instantiations (registers), see launch_bwd_fast()
				const int64_t per_tr = l1_cdiv((int64_t)BWD_SJ * tr * hb_exact, p.threads);
				if (g > 1 && (!can_group || wgs < slots || tr != 64 || per_tr > (p.rank ? 4 : 8))) continue;
				const double cost = (double)l1_cdiv(wgs, slots) * g * (tr + 1.0) + 0.04 * (double)(B * p.n_cc * ngr);
				if (cost < best) { best = cost; p.tt_rows = tr; p.group = g; }
			}
		}
	}
	p.n_tt = (int)l1_cdiv(T, p.tt_rows);
	p.n_groups = (int)l1_cdiv(p.n_tt, p.group);
	const int64_t hb_max = hb_exact;
	p.lds_bytes = (size_t)BWD_SJ * hb_max * (p.tt_rows + 4) * sizeof(float);
	p.per = (int)l1_cdiv((int64_t)BWD_SJ * p.tt_rows * hb_max, p.threads);
	if (p.lds_bytes > 64 * 1024 || p.per > 16 || (p.wide && p.per > 8)) { p.fast = false; return p; }
	// (the branch-free form addresses a step's dA rows with 32-bit byte offsets from the step's first row)
	p.branch_free = p.wide && p.tt_rows == 64 && T % 64 == 0 && T % BWD_SJ == 0 && HW % p.threads == 0 &&
	                (BWD_SJ * T + 128) * H < ((int64_t)1 << 29) &&
	                p.threads % W == 0 && (int64_t)BWD_SJ * 64 * (p.threads / W) == (int64_t)4 * p.threads;
	p.deep = (p.branch_free && T % (2 * BWD_SJ) == 0) ? loop_form : 0;
	if (p.deep == 2) p.lds_bytes *= 2;
	p.partial_bytes = p.n_tt > 1 ? (size_t)p.n_groups * T * HW * sizeof(float) : 0;
	// rq, rk [T][HW]; column sums per dst tile [n_tt][T][H] and their total [T][H]
	p.rank_bytes = p.rank ? ((size_t)2 * T * HW + (size_t)(p.n_tt + 1) * T * H) * sizeof(float) : 0;
	p.per_batch_bytes = p.partial_bytes + p.rank_bytes;
	p.flag_bytes = p.rank ? 0 : BWD_FLAG_BYTES;
	return p;
}

void launch_bwd_fast(const BwdPlan& p, dim3 grid, hipStream_t st, const float* dA, const float* q, const float* k,
                     float* dq, float* dkp, float* csp, int T, int H, int W, float scale)
{
#define L1_BWD_CASE6(TTV, MT, PERV, RANKV, GRPV, FASTV)                                                         \
	hipLaunchKernelGGL((dense_bwd_f32_fast<TTV, MT, PERV, RANKV, GRPV, FASTV>), grid, dim3(p.threads), p.lds_bytes, \
	                   st, dA, q, k, dq, dkp, csp, T, H, W, scale, p.group)
#define L1_BWD_CASE(TTV, MT, PERV, RANKV, GRPV) L1_BWD_CASE6(TTV, MT, PERV, RANKV, GRPV, false)
#define L1_BWD_CASE_DEEP(RANKV, GRPV, FORM)                                                                   \
	hipLaunchKernelGGL((dense_bwd_f32_fast<64, 512, 4, RANKV, GRPV, true, FORM>), grid, dim3(p.threads), p.lds_bytes, \
	                   st, dA, q, k, dq, dkp, csp, T, H, W, scale, p.group)
	if (p.wide && p.branch_free && p.deep == 1) {
		if (p.rank && p.group > 1) L1_BWD_CASE_DEEP(true, true, 1);
		else if (p.rank) L1_BWD_CASE_DEEP(true, false, 1);
		else if (p.group > 1) L1_BWD_CASE_DEEP(false, true, 1);
		else L1_BWD_CASE_DEEP(false, false, 1);
	} else if (p.wide && p.branch_free && p.deep == 2) {
		if (p.rank && p.group > 1) L1_BWD_CASE_DEEP(true, true, 2);
		else if (p.rank) L1_BWD_CASE_DEEP(true, false, 2);
		else if (p.group > 1) L1_BWD_CASE_DEEP(false, true, 2);
		else L1_BWD_CASE_DEEP(false, false, 2);
	} else if (p.wide && p.branch_free) {
		// bwd_plan() sets branch_free only for 64-token tiles with four staged values per thread
		if (p.rank && p.group > 1) L1_BWD_CASE6(64, 512, 4, true, true, true);
		else if (p.rank) L1_BWD_CASE6(64, 512, 4, true, false, true);
		else if (p.group > 1) L1_BWD_CASE6(64, 512, 4, false, true, true);
		else L1_BWD_CASE6(64, 512, 4, false, false, true);
	} else if (p.wide && p.rank) {
		switch (p.tt_rows) {
		case 64:
			if (p.per <= 4) L1_BWD_CASE(64, 512, 4, true, false);
			else L1_BWD_CASE(64, 512, 8, true, false);
			break;
		case 72: L1_BWD_CASE(72, 512, 8, true, false); break;
		default: L1_BWD_CASE(80, 512, 8, true, false); break;
		}
	} else if (p.wide) {
		switch (p.tt_rows) {
		case 64:
			if (p.per <= 4) L1_BWD_CASE(64, 512, 4, false, false);
			else L1_BWD_CASE(64, 512, 8, false, false);
			break;
		case 72: L1_BWD_CASE(72, 512, 8, false, false); break;
		case 80: L1_BWD_CASE(80, 512, 8, false, false); break;
		default: L1_BWD_CASE(88, 512, 8, false, false); break;
		}
	} else {
		if (p.per <= 1) L1_BWD_CASE(32, 1024, 1, false, false);
		else if (p.per <= 2) L1_BWD_CASE(32, 1024, 2, false, false);
		else if (p.per <= 4) L1_BWD_CASE(32, 1024, 4, false, false);
		else if (p.per <= 8) L1_BWD_CASE(32, 1024, 8, false, false);
		else L1_BWD_CASE(32, 1024, 16, false, false);
	}
#undef L1_BWD_CASE
#undef L1_BWD_CASE6
#undef L1_BWD_CASE_DEEP
}

}  // namespace

extern "C" {

int l1attn_dense_fwd_ws_f32(const float* q, const float* k, float* attn, int64_t B, int64_t T, int64_t H, int64_t W,
                            void* workspace, size_t workspace_bytes, void* stream);

int l1attn_dense_fwd_f32(const float* q, const float* k, float* attn, int64_t B, int64_t T, int64_t H, int64_t W,
                         void* stream)
{
	if (!shape_ok(B, T, H, W)) return L1ATTN_ERR_ARG;
	if (B * T * T * H == 0) return L1ATTN_OK;
	if (!q || !k || !attn) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	if (W < 1) return L1ATTN_ERR_ARG;
	return l1attn_dense_fwd_ws_f32(q, k, attn, B, T, H, W, nullptr, 0, stream);
}

// widths that are not a multiple of 16 run the fast kernels on zero-padded copies of q and k (|0 - 0| adds
// nothing); the copies cost O(T) against the O(T^2) of the logits
static int64_t fwd_padded_width(int64_t B, int64_t T, int64_t H, int64_t W)
{
	if (W % 16 == 0 || W > 128) return 0;
	// above 96 the pipelined half-head kernel of width 128 beats the width-112 kernel
	const int64_t WP = W > 96 ? 128 : l1_cdiv(W, 16) * 16;
	return fwd_fast_ok(nullptr, nullptr, B, T, H, WP) ? WP : 0;
}

size_t l1attn_dense_fwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W)
{
	if (!shape_ok(B, T, H, W) || B * T * H * W == 0) return 0;
	return (size_t)2 * B * T * H * fwd_padded_width(B, T, H, W) * sizeof(float);
}

int l1attn_dense_fwd_ws_f32(const float* q, const float* k, float* attn, int64_t B, int64_t T, int64_t H, int64_t W,
                            void* workspace, size_t workspace_bytes, void* stream)
{
	if (!shape_ok(B, T, H, W)) return L1ATTN_ERR_ARG;
	if (B * T * T * H == 0) return L1ATTN_OK;
	if (!q || !k || !attn) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	if (W < 1) return L1ATTN_ERR_ARG;
	if (fwd_fast_ok(q, k, B, T, H, W)) return launch_fwd_fast(q, k, attn, B, T, H, W, W, st);
	const int64_t WP = fwd_padded_width(B, T, H, W);
	const int64_t rows = B * T * H;
	if (WP > 0 && workspace && workspace_bytes >= (size_t)2 * rows * WP * sizeof(float) &&
	    (((uintptr_t)workspace) & 15) == 0 && 2 * rows * WP < ((int64_t)1 << 40)) {
		float* qp = (float*)workspace;
		float* kp = qp + rows * WP;
		const int64_t n = rows * WP;
		const dim3 grid((unsigned)std::min<int64_t>(l1_cdiv(n, 256), 1 << 20));
		hipLaunchKernelGGL(dense_pad_rows, grid, dim3(256), 0, st, q, k, qp, kp, n, (int)W, (int)WP);
		L1_LAUNCH_CHECK();
		return launch_fwd_fast(qp, kp, attn, B, T, H, WP, W, st);
	}
	return launch_fwd_generic<float>(q, k, attn, B, T, H, W, st);
}

// Fixed-point forward (experimental, fp32 in and out): workspace = grids [B*H] (padded to 256 bytes), then the
// fixed-point copies of q and k.
static size_t fixed_grid_bytes(int64_t B, int64_t H) { return l1_align_up((size_t)(B * H) * sizeof(float), 256); }

size_t l1attn_dense_fwd_fixed_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W)
{
	if (!shape_ok(B, T, H, W) || B * T * H * W == 0) return 0;
	return fixed_grid_bytes(B, H) + (size_t)2 * B * T * H * W * sizeof(float);
}

int l1attn_dense_fwd_fixed_f32(const float* q, const float* k, float* attn, int64_t B, int64_t T, int64_t H, int64_t W,
                               void* workspace, size_t workspace_bytes, void* stream)
{
	if (!shape_ok(B, T, H, W)) return L1ATTN_ERR_ARG;
	if (B * T * T * H == 0) return L1ATTN_OK;
	if (!q || !k || !attn) return L1ATTN_ERR_ARG;
	if ((W != 32 && W != 64) || !fwd_fast_ok(q, k, B, T, H, W) || B * H > 2147483647LL) return L1ATTN_ERR_ARG;
	if (!workspace || (((uintptr_t)workspace) & 15) || workspace_bytes < l1attn_dense_fwd_fixed_workspace_bytes(B, T, H, W))
		return L1ATTN_ERR_WORKSPACE;
	hipStream_t st = (hipStream_t)stream;
	float* gq = (float*)workspace;
	unsigned* uq = (unsigned*)((char*)workspace + fixed_grid_bytes(B, H));
	const int64_t n = B * T * H * W;
	unsigned* uk = uq + n;
	const int rc = l1_launch_fixed_prepass(q, k, gq, uq, uk, B, T, H, W, st);
	if (rc != L1ATTN_OK) return rc;
	return launch_fwd_fast((const float*)uq, (const float*)uk, attn, B, T, H, W, W, st, gq);
}

int l1attn_dense_fwd_f64(const double* q, const double* k, double* attn, int64_t B, int64_t T, int64_t H, int64_t W,
                         void* stream)
{
	if (!shape_ok(B, T, H, W)) return L1ATTN_ERR_ARG;
	if (B * T * T * H == 0) return L1ATTN_OK;
	if (!q || !k || !attn) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	if (W < 1) return L1ATTN_ERR_ARG;
	return launch_fwd_generic<double>(q, k, attn, B, T, H, W, st);
}

size_t l1attn_dense_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W)
{
	if (!shape_ok(B, T, H, W) || B * T * H * W == 0) return 0;
	BwdPlan p = bwd_plan(B, T, H, W);
	if (!p.fast) return 0;
	if (p.per_batch_bytes == 0) return p.flag_bytes;
	// enough batches per launch to put >= 1024 workgroups in flight, never more than B
	int64_t nb = l1_cdiv(1024, (int64_t)p.n_groups * p.n_cc);
	if (nb > B) nb = B;
	return p.flag_bytes + p.per_batch_bytes * (size_t)nb;
}

int l1attn_dense_bwd_plan_info_ex(int64_t B, int64_t T, int64_t H, int64_t W, int loop_form, int64_t* info)
{
	if (!info || !shape_ok(B, T, H, W) || loop_form < 0 || loop_form > 2) return L1ATTN_ERR_ARG;
	for (int i = 0; i < 16; i++) info[i] = 0;
	if (B * T * H * W == 0) return L1ATTN_OK;
	const BwdPlan p = bwd_plan(B, T, H, W, loop_form);
	info[0] = p.fast;
	if (!p.fast) return L1ATTN_OK;
	info[1] = p.wide; info[2] = p.rank; info[3] = p.branch_free;
	info[4] = p.threads; info[5] = p.n_cc; info[6] = p.n_tt; info[7] = p.tt_rows;
	info[8] = p.per; info[9] = p.group; info[10] = p.n_groups; info[11] = (int64_t)p.lds_bytes;
	info[12] = (int64_t)p.per_batch_bytes;
	info[13] = p.per_batch_bytes ? std::min<int64_t>(B, l1_cdiv(1024, (int64_t)p.n_groups * p.n_cc)) : B;
	info[14] = p.deep;
	info[15] = (int64_t)p.flag_bytes;
	return L1ATTN_OK;
}

int l1attn_dense_bwd_plan_info(int64_t B, int64_t T, int64_t H, int64_t W, int64_t* info)
{
	return l1attn_dense_bwd_plan_info_ex(B, T, H, W, 0, info);
}

// rank_sort: 0 = column ranks from the library block radix sort (dense_rank.hip), 1 = from the merge sort of
// rank_sort.hip; both give the same ranks
// assume_sign_range: the caller vouches that every magnitude in q and k is below 2^63 and every non-zero one at
// least 2^-41; the range check and the fix-up launch are then left out
int l1attn_dense_bwd_ex_f32(const float* d_attn, const float* q, const float* k, float* dq, float* dk, int64_t B,
                            int64_t T, int64_t H, int64_t W, int loop_form, int rank_sort, int assume_sign_range,
                            void* workspace, size_t workspace_bytes, void* stream)
{
	if (!shape_ok(B, T, H, W) || loop_form < 0 || loop_form > 2 || rank_sort < 0 || rank_sort > 1 ||
	    assume_sign_range < 0 || assume_sign_range > 1)
		return L1ATTN_ERR_ARG;
	const int64_t n = B * T * H * W;
	if (n == 0) return L1ATTN_OK;
	if (!d_attn || !q || !k || !dq || !dk) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	BwdPlan p = bwd_plan(B, T, H, W, loop_form);
	if (!p.fast) return launch_bwd_generic<float>(d_attn, q, k, dq, dk, B, T, H, W, st);
	const float scale = (float)(-1.0 / sqrt((double)W));
	const int64_t HW = H * W;
	// the head of the workspace belongs to the flag whether this call uses it or not, so that one layout serves
	// every call on a shape; a vouched call on a plan without partial arrays needs no workspace at all
	const bool uses_workspace = p.per_batch_bytes > 0 || (p.flag_bytes > 0 && !assume_sign_range);
	if (uses_workspace && (!workspace || workspace_bytes < p.flag_bytes + p.per_batch_bytes)) return L1ATTN_ERR_WORKSPACE;
	// Without column ranks the sign comes from the scaled difference: find out (on the device, without waiting)
	// whether q and k are inside the range where that is exact; the fix-up launch at the end redoes dq and dk
	// with comparisons when they are not.
	int* const flag = (p.flag_bytes && !assume_sign_range) ? (int*)workspace : nullptr;
	if (uses_workspace && p.flag_bytes) {
		workspace = (char*)workspace + p.flag_bytes;
		workspace_bytes -= p.flag_bytes;
	}
	if (flag) {
		hipLaunchKernelGGL(dense_bwd_clear_flag, dim3(1), dim3(64), 0, st, flag);
		L1_LAUNCH_CHECK();
		const dim3 dgrid((unsigned)std::min<int64_t>(l1_cdiv(n, 256 * 8), 4096));
		hipLaunchKernelGGL(dense_bwd_sign_domain, dgrid, dim3(256), 0, st, q, k, n, flag);
		L1_LAUNCH_CHECK();
	}
	const auto fix_up = [&]() -> int {
		if (!flag) return L1ATTN_OK;
		const dim3 egrid((unsigned)l1_cdiv(n, 256), 2);
		hipLaunchKernelGGL(dense_bwd_exact_if_flagged, egrid, dim3(256), 0, st, d_attn, q, k, dq, dk, B, T, H, W, scale,
		                   (const int*)flag);
		L1_LAUNCH_CHECK();
		return L1ATTN_OK;
	};
	if (p.per_batch_bytes == 0) {
		dim3 grid(1, p.n_cc, (unsigned)B);
		launch_bwd_fast(p, grid, st, d_attn, q, k, dq, dk, nullptr, (int)T, (int)H, (int)W, scale);
		L1_LAUNCH_CHECK();
		return fix_up();
	}
	int64_t nb_max = (int64_t)(workspace_bytes / p.per_batch_bytes);
	if (nb_max > B) nb_max = B;
	// workspace: [n_groups][nb_max][T][HW] dk partials, then (rank path) rq and rk [nb_max][T][HW] each, the
	// column sums per dst tile [n_tt][nb_max][T][H] and their total [nb_max][T][H]
	float* dkp = (float*)workspace;
	float* rq = dkp + (size_t)nb_max * (p.partial_bytes / sizeof(float));
	float* rk = rq + (size_t)nb_max * T * HW;
	float* csp = rk + (size_t)nb_max * T * HW;
	float* cs = csp + (size_t)p.n_tt * nb_max * T * H;
	for (int64_t b0 = 0; b0 < B; b0 += nb_max) {
		const int64_t nb = std::min<int64_t>(nb_max, B - b0);
		dim3 grid(p.n_groups, p.n_cc, (unsigned)nb);
		const float* qa = q + b0 * T * HW;
		const float* ka = k + b0 * T * HW;
		if (p.rank) {
			const int rc = rank_sort == 1 ? l1_launch_column_ranks_merge(qa, ka, rq, rk, nb, T, H, W, st)
			                           : l1_launch_column_ranks(qa, ka, rq, rk, nb, T, H, W, st);
			if (rc != L1ATTN_OK) return rc;
			qa = rq;
			ka = rk;
		}
		launch_bwd_fast(p, grid, st, d_attn + b0 * T * T * H, qa, ka, dq + b0 * T * HW, dkp, csp, (int)T, (int)H,
		                (int)W, scale);
		L1_LAUNCH_CHECK();
		const int64_t ne = nb * T * HW;
		if (p.rank) {
			const int64_t nc = nb * T * H;
			hipLaunchKernelGGL(dense_bwd_reduce_colsum, dim3((unsigned)l1_cdiv(nc, 256)), dim3(256), 0, st, csp, cs, nc,
			                   p.n_tt);
			L1_LAUNCH_CHECK();
		}
		const bool vec = ((T * HW) % 4 == 0) && ((((uintptr_t)dkp) | ((uintptr_t)dk)) & 15) == 0 &&
		                 (!p.rank || W % 4 == 0);
		const dim3 rgrid((unsigned)l1_cdiv(ne, vec ? 1024 : 256));
#define L1_REDUCE_CASE3(VECV, RANKV, AHEADV)                                                                    \
	hipLaunchKernelGGL((dense_bwd_reduce_dk<VECV, RANKV, AHEADV>), rgrid, dim3(256), 0, st, dkp, dk + b0 * T * HW, \
	                   ne, p.n_groups, cs, (int)HW, (int)W, (int)H, scale)
#define L1_REDUCE_CASE(VECV, RANKV) L1_REDUCE_CASE3(VECV, RANKV, false)
		if (vec && p.deep && p.rank) L1_REDUCE_CASE3(true, true, true);
		else if (vec && p.deep) L1_REDUCE_CASE3(true, false, true);
		else if (vec && p.rank) L1_REDUCE_CASE(true, true);
		else if (vec) L1_REDUCE_CASE(true, false);
		else if (p.rank) L1_REDUCE_CASE(false, true);
		else L1_REDUCE_CASE(false, false);
#undef L1_REDUCE_CASE
#undef L1_REDUCE_CASE3
		L1_LAUNCH_CHECK();
	}
	return fix_up();
}

int l1attn_dense_bwd_f32(const float* d_attn, const float* q, const float* k, float* dq, float* dk, int64_t B,
                         int64_t T, int64_t H, int64_t W, void* workspace, size_t workspace_bytes, void* stream)
{
	return l1attn_dense_bwd_ex_f32(d_attn, q, k, dq, dk, B, T, H, W, 0, 0, 0, workspace, workspace_bytes, stream);
}

int l1attn_dense_bwd_f64(const double* d_attn, const double* q, const double* k, double* dq, double* dk, int64_t B,
                         int64_t T, int64_t H, int64_t W, void* workspace, size_t workspace_bytes, void* stream)
{
	(void)workspace; (void)workspace_bytes;
	if (!shape_ok(B, T, H, W)) return L1ATTN_ERR_ARG;
	if (B * T * H * W == 0) return L1ATTN_OK;
	if (!d_attn || !q || !k || !dq || !dk) return L1ATTN_ERR_ARG;
	return launch_bwd_generic<double>(d_attn, q, k, dq, dk, B, T, H, W, (hipStream_t)stream);
}

}  // extern "C"
