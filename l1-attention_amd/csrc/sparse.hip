// Sparse (edge-list) L1 attention for gfx950, one-directional and bidirectional, forward and
// backward.  Replaces cuda/l1attn_sparse_cuda_kernel.cu:27-815 (nine kernels, four launchers) and
// follows the arithmetic of cpp/l1attn_sparse_drv.cpp:13-190 / cpp/l1attn_sparse_bidi_drv.cpp:15-212:
//
//   a_c = -1/sqrt(W) * sum_w |q[b,dst_c,h,w] - k[b,src_c,h,w]|
//   p_c = exp(a_c) / (1 + sum_{c' with the same dst} exp(a_c'))      (use_softmax)   or   exp(a_c)
//   vo[b,dst] += p_c * v[b,src]                  (bidi: v = vf, and also vo[b,src] += p_c * vb[b,dst])
//
// Where the reference scatters with float atomics into a [B,T,dst_mxlen,H] padded tensor and
// multiplies by an O(dst_mxlen^2) softmax Jacobian, these kernels walk the plan's dst-sorted and
// src-sorted segments: every output row is owned by one wavefront, sums run in slot order, and the
// Jacobian product is the closed form p_c*(dp_c - sum_c' p_c' dp_c').  Results are bitwise
// reproducible.  Edge weights live in slot order as P[b][slot][h] (no padding).
//
// Work item = (batch, token, head chunk) -> one wavefront.  A token's row [H*W] is contiguous; a head
// is spread over G = 2^g lanes (VEC consecutive floats per lane and chunk), so one wave holds 64/G
// heads and a row is fetched with full-width coalesced loads.  Per-head sums use xor shuffles inside
// the G-lane group.
#include "common.h"
#include "plan.h"
#include <math.h>

namespace {

// Storage types of the 16-bit forward entry points: IEEE half and bfloat16.  Rows are held in memory in
// the storage type S and converted on load and on store; every sum runs in the compute type T (float).
using f16_t = _Float16;
using bf16_t = __bf16;

// x[0..VEC) = the VEC consecutive elements at p, converted from S to T.  VEC == 4 takes one 16-byte
// (float), two 16-byte (double) or one 8-byte (16-bit types) access; p is aligned to that by the host.
template <typename T, int VEC, typename S>
__device__ __forceinline__ void ldv(const S* __restrict__ p, T (&x)[VEC])
{
	if constexpr (VEC == 4 && sizeof(S) == 4) {
		const float4 t = *reinterpret_cast<const float4*>(p);
		x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
	} else if constexpr (VEC == 4 && sizeof(S) == 8) {
		const double2 a = *reinterpret_cast<const double2*>(p);
		const double2 b = *reinterpret_cast<const double2*>(p + 2);
		x[0] = a.x; x[1] = a.y; x[2] = b.x; x[3] = b.y;
	} else if constexpr (VEC == 4 && sizeof(S) == 2) {
		const uint2 raw = *reinterpret_cast<const uint2*>(p);
		S h[4];
		__builtin_memcpy(h, &raw, 8);
#pragma unroll
		for (int i = 0; i < 4; i++) x[i] = (T)h[i];
	} else {
#pragma unroll
		for (int i = 0; i < VEC; i++) x[i] = (T)p[i];
	}
}

// the VEC consecutive elements at p = x[0..VEC), rounded to S (round to nearest even for the 16-bit types)
template <typename T, int VEC, typename S>
__device__ __forceinline__ void stv(S* __restrict__ p, const T (&x)[VEC])
{
	if constexpr (VEC == 4 && sizeof(S) == 4) {
		*reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
	} else if constexpr (VEC == 4 && sizeof(S) == 8) {
		*reinterpret_cast<double2*>(p) = make_double2(x[0], x[1]);
		*reinterpret_cast<double2*>(p + 2) = make_double2(x[2], x[3]);
	} else if constexpr (VEC == 4 && sizeof(S) == 2) {
		S h[4];
#pragma unroll
		for (int i = 0; i < 4; i++) h[i] = (S)x[i];
		uint2 raw;
		__builtin_memcpy(&raw, h, 8);
		*reinterpret_cast<uint2*>(p) = raw;
	} else {
#pragma unroll
		for (int i = 0; i < VEC; i++) p[i] = (S)x[i];
	}
}

template <typename T>
__device__ __forceinline__ T group_sum(T x, int G)
{
	for (int off = G >> 1; off > 0; off >>= 1) x += __shfl_xor(x, off);
	return x;
}

template <typename T> __device__ __forceinline__ T exp_t(T x);
template <> __device__ __forceinline__ float exp_t<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double exp_t<double>(double x) { return exp(x); }

template <typename T> __device__ __forceinline__ T abs_t(T x) { return x < (T)0 ? -x : x; }
template <typename T> __device__ __forceinline__ T sgn_t(T x) { return (T)((x > (T)0) - (x < (T)0)); }

// Orders a wave's own global stores before its later loads of the same addresses from other lanes.
// Workgroup scope is enough (the data never leaves the wave) and, unlike an agent-scope fence, does
// not write back the L2.
__device__ __forceinline__ void wave_store_load_fence()
{
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// geometry of one work item, shared by all kernels
struct Geo {
	int Tn, H, W, Wv, E;
	int log2G;     // lanes per head = 1 << log2G
	int n_hc;      // head chunks per token = ceil(H / (64 >> log2G))
	int long_on;   // 1: segments longer than PLAN_LONG_SEGMENT are left to the workgroup-per-segment launch
};

struct Lane {
	int tok, h, sub;
	bool head_ok;
	int pb, pe;    // this wave's share [pb, pe) of the segment
	int p0, p1;    // the whole segment
	int wave;
};

// Work decomposition.
//  NWV == 1: wave-per-item launch.  grid.x covers the Tn*n_hc (token, head chunk) items, four per block;
//            grid.y = batch.  Items whose segment is "long" are skipped when g.long_on.
//  NWV  > 1: workgroup-per-item launch over the plan's list of long tokens.  grid.x = capacity of the
//            list (entries beyond the count on the device exit at once), grid.y = batch, grid.z = head
//            chunk; the NWV waves take contiguous, equal shares of the segment in wave order.
template <int NWV>
__device__ __forceinline__ bool wave_item(const Geo& g, const int* __restrict__ ptr, const int* __restrict__ long_list,
                                          const int* __restrict__ n_long, Lane& L)
{
	const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
	const int lane = threadIdx.x & 63;
	int hc;
	if (NWV == 1) {
		const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave;
		if (item >= (int64_t)g.Tn * g.n_hc) return false;
		L.tok = (int)(item / g.n_hc);
		hc = (int)(item % g.n_hc);
	} else {
		if ((int)blockIdx.x >= *n_long) return false;  // uniform over the workgroup
		L.tok = long_list[blockIdx.x];
		hc = blockIdx.z;
	}
	L.p0 = ptr[L.tok];
	L.p1 = ptr[L.tok + 1];
	const int deg = L.p1 - L.p0;
	if (NWV == 1) {
		if (g.long_on && deg > PLAN_LONG_SEGMENT) return false;
		L.pb = L.p0;
		L.pe = L.p1;
	} else {
		const int share = (deg + NWV - 1) / NWV;
		L.pb = min(L.p1, L.p0 + wave * share);
		L.pe = min(L.p1, L.pb + share);
	}
	L.wave = wave;
	L.sub = lane & ((1 << g.log2G) - 1);
	L.h = hc * (64 >> g.log2G) + (lane >> g.log2G);
	L.head_ok = L.h < g.H;
	return true;
}

// Sum of x over the NWV waves of the workgroup, in wave order (bitwise reproducible), returned to
// every wave.  smem: NWV*64 elements per call site; the caller separates uses with the barriers here.
template <typename T, int NWV>
__device__ __forceinline__ T wg_sum(T x, T* smem, int wave)
{
	if (NWV == 1) return x;
	const int lane = threadIdx.x & 63;
	__syncthreads();
	smem[wave * 64 + lane] = x;
	__syncthreads();
	T s = smem[lane];
#pragma unroll
	for (int w = 1; w < NWV; w++) s += smem[w * 64 + lane];
	return s;
}

// edges in flight per wave: rows of EU edges are requested before the first is used
template <int MC> struct Unroll { static constexpr int EU = MC == 1 ? 4 : 1; };

// ---------------------------------------------------------------------------------- forward

// dst pass: logits, softmax with the "+1" denominator, value sum.  Writes vo rows and P.
// S: type of the rows in memory (v, q, k, vo); T: type of the sums and of the weights P.
template <typename T, int VEC, int MC, int NWV, typename S>
__global__ __launch_bounds__(NWV == 1 ? 256 : 64 * NWV) void sparse_fwd_dst(
    const S* __restrict__ v, const S* __restrict__ q, const S* __restrict__ k, const int* __restrict__ dst_ptr,
    const int* __restrict__ csr_src, const int* __restrict__ long_list, const int* __restrict__ n_long,
    S* __restrict__ vo, T* __restrict__ P, Geo g, int use_softmax, T scale)
{
	extern __shared__ unsigned char smem_raw[];
	T* smem = reinterpret_cast<T*>(smem_raw);
	constexpr int EU = Unroll<MC>::EU;
	Lane L;
	if (!wave_item<NWV>(g, dst_ptr, long_list, n_long, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowq = (int64_t)g.H * g.W, rowv = (int64_t)g.H * g.Wv;
	const S* qb = q + (int64_t)b * g.Tn * rowq;
	const S* kb = k + (int64_t)b * g.Tn * rowq;
	const S* vb = v + (int64_t)b * g.Tn * rowv;
	T* Pb = P + (int64_t)b * g.E * g.H;

	T qv[MC][VEC], acc[MC][VEC];
	bool okq[MC], okv[MC];
	int offq[MC], offv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		okq[m] = L.head_ok && w0 < g.W;
		okv[m] = L.head_ok && w0 < g.Wv;
		offq[m] = L.h * g.W + w0;
		offv[m] = L.h * g.Wv + w0;
#pragma unroll
		for (int i = 0; i < VEC; i++) { qv[m][i] = 0; acc[m][i] = 0; }
		if (okq[m]) ldv<T, VEC>(qb + (int64_t)L.tok * rowq + offq[m], qv[m]);
	}
	T den = 0;
	int sidx[EU];
#pragma unroll
	for (int u = 0; u < EU; u++) sidx[u] = L.pb < L.pe ? csr_src[min(L.pb + u, L.pe - 1)] : 0;
	for (int p = L.pb; p < L.pe; p += EU) {
		T kv[EU][MC][VEC], vv[EU][MC][VEC];
#pragma unroll
		for (int u = 0; u < EU; u++)
#pragma unroll
			for (int m = 0; m < MC; m++) {
#pragma unroll
				for (int i = 0; i < VEC; i++) { kv[u][m][i] = qv[m][i]; vv[u][m][i] = 0; }
				if (okq[m]) ldv<T, VEC>(kb + (int64_t)sidx[u] * rowq + offq[m], kv[u][m]);
				if (okv[m]) ldv<T, VEC>(vb + (int64_t)sidx[u] * rowv + offv[m], vv[u][m]);
			}
		// indices of the next group, clamped into this wave's share
#pragma unroll
		for (int u = 0; u < EU; u++) sidx[u] = csr_src[min(p + EU + u, L.pe - 1)];
		T d[EU];
#pragma unroll
		for (int u = 0; u < EU; u++) {
			d[u] = 0;
#pragma unroll
			for (int m = 0; m < MC; m++)
#pragma unroll
				for (int i = 0; i < VEC; i++) d[u] += abs_t(qv[m][i] - kv[u][m][i]);
		}
#pragma unroll
		for (int u = 0; u < EU; u++) d[u] = group_sum(d[u], G);
#pragma unroll
		for (int u = 0; u < EU; u++) {
			if (p + u < L.pe) {  // uniform
				const T e = exp_t(d[u] * scale);
				den += e;
#pragma unroll
				for (int m = 0; m < MC; m++)
#pragma unroll
					for (int i = 0; i < VEC; i++) acc[m][i] += e * vv[u][m][i];
				if (L.sub == 0 && L.head_ok) Pb[(int64_t)(p + u) * g.H + L.h] = e;
			}
		}
	}
	// combine the waves of a long segment in wave order
	den = wg_sum<T, NWV>(den, smem, L.wave);
#pragma unroll
	for (int m = 0; m < MC; m++)
#pragma unroll
		for (int i = 0; i < VEC; i++) acc[m][i] = wg_sum<T, NWV>(acc[m][i], smem, L.wave);
	if (use_softmax) den += (T)1;
	const T inv = use_softmax ? (T)1 / den : (T)1;
	if (L.wave == 0 || NWV == 1) {
#pragma unroll
		for (int m = 0; m < MC; m++) {
#pragma unroll
			for (int i = 0; i < VEC; i++) acc[m][i] *= inv;
			if (okv[m]) stv<T, VEC>(vo + ((int64_t)b * g.Tn + L.tok) * rowv + offv[m], acc[m]);
		}
	}
	// the weights below were stored by lane 0 of each head group: make them visible to its other lanes
	wave_store_load_fence();
	if (use_softmax && L.head_ok) {
		// normalise the stored weights of this wave's share; the G lanes of a head take every G-th slot
		for (int p = L.pb + L.sub; p < L.pe; p += G) Pb[(int64_t)p * g.H + L.h] *= inv;
	}
}

// bidi src pass: vo[b,src] += sum over the src's edges of p * vb[b,dst]   (cpp/l1attn_sparse_bidi_drv.cpp:93-96)
template <typename T, int VEC, int MC, int NWV, typename S>
__global__ __launch_bounds__(NWV == 1 ? 256 : 64 * NWV) void sparse_fwd_src(
    const S* __restrict__ vbk, const int* __restrict__ src_ptr, const int* __restrict__ csc_dst,
    const int* __restrict__ csc_slot, const int* __restrict__ long_list, const int* __restrict__ n_long,
    const T* __restrict__ P, S* __restrict__ vo, Geo g)
{
	extern __shared__ unsigned char smem_raw[];
	T* smem = reinterpret_cast<T*>(smem_raw);
	constexpr int EU = Unroll<MC>::EU;
	Lane L;
	if (!wave_item<NWV>(g, src_ptr, long_list, n_long, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowv = (int64_t)g.H * g.Wv;
	const S* vb = vbk + (int64_t)b * g.Tn * rowv;
	const T* Pb = P + (int64_t)b * g.E * g.H;
	T acc[MC][VEC];
	bool okv[MC];
	int offv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		okv[m] = L.head_ok && (m * G + L.sub) * VEC < g.Wv;
		offv[m] = L.h * g.Wv + (m * G + L.sub) * VEC;
#pragma unroll
		for (int i = 0; i < VEC; i++) acc[m][i] = 0;
	}
	int didx[EU], slot[EU];
#pragma unroll
	for (int u = 0; u < EU; u++) {
		const int e = min(L.pb + u, L.pe - 1);
		didx[u] = L.pb < L.pe ? csc_dst[e] : 0;
		slot[u] = L.pb < L.pe ? csc_slot[e] : 0;
	}
	for (int e0 = L.pb; e0 < L.pe; e0 += EU) {
		T x[EU][MC][VEC], pe[EU];
#pragma unroll
		for (int u = 0; u < EU; u++) {
			pe[u] = L.head_ok ? Pb[(int64_t)slot[u] * g.H + L.h] : (T)0;
#pragma unroll
			for (int m = 0; m < MC; m++) {
#pragma unroll
				for (int i = 0; i < VEC; i++) x[u][m][i] = 0;
				if (okv[m]) ldv<T, VEC>(vb + (int64_t)didx[u] * rowv + offv[m], x[u][m]);
			}
		}
#pragma unroll
		for (int u = 0; u < EU; u++) {
			const int e = min(e0 + EU + u, L.pe - 1);
			didx[u] = csc_dst[e];
			slot[u] = csc_slot[e];
		}
#pragma unroll
		for (int u = 0; u < EU; u++)
			if (e0 + u < L.pe)
#pragma unroll
				for (int m = 0; m < MC; m++)
#pragma unroll
					for (int i = 0; i < VEC; i++) acc[m][i] += pe[u] * x[u][m][i];
	}
#pragma unroll
	for (int m = 0; m < MC; m++)
#pragma unroll
		for (int i = 0; i < VEC; i++) acc[m][i] = wg_sum<T, NWV>(acc[m][i], smem, L.wave);
	if (L.wave == 0 || NWV == 1) {
#pragma unroll
		for (int m = 0; m < MC; m++) {
			if (okv[m]) {
				S* o = vo + ((int64_t)b * g.Tn + L.tok) * rowv + offv[m];
				T y[VEC];
				ldv<T, VEC>(o, y);
#pragma unroll
				for (int i = 0; i < VEC; i++) y[i] += acc[m][i];
				stv<T, VEC>(o, y);
			}
		}
	}
}

// --------------------------------------------------------------------------------- backward

// dst pass.  For every edge of the dst:  dp = v[src].dvo[dst] (+ vb[dst].dvo[src] for bidi);
// S = sum p*dp;  dq[dst] = scale * sum sign(q-k) * p * (dp - S)  accumulated as X - S*Y in one walk;
// bidi: dvb[dst] = sum p * dvo[src].  Leaves da = p*(dp - S) (or p*dp) per edge in DA.
// ST: type of the rows in memory (S is the softmax sum below)
template <typename T, int VEC, int MC, bool BIDI, int NWV, typename ST>
__global__ __launch_bounds__(NWV == 1 ? 256 : 64 * NWV) void sparse_bwd_dst(
    const ST* __restrict__ dvo, const ST* __restrict__ v, const ST* __restrict__ vbk, const ST* __restrict__ q,
    const ST* __restrict__ k, const int* __restrict__ dst_ptr, const int* __restrict__ csr_src,
    const int* __restrict__ long_list, const int* __restrict__ n_long, const T* __restrict__ P,
    T* __restrict__ DA, ST* __restrict__ dq, ST* __restrict__ dvb, Geo g, int use_softmax, T scale)
{
	extern __shared__ unsigned char smem_raw[];
	T* smem = reinterpret_cast<T*>(smem_raw);
	constexpr int EU = Unroll<MC>::EU;
	Lane L;
	if (!wave_item<NWV>(g, dst_ptr, long_list, n_long, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowq = (int64_t)g.H * g.W, rowv = (int64_t)g.H * g.Wv;
	const ST* qb = q + (int64_t)b * g.Tn * rowq;
	const ST* kb = k + (int64_t)b * g.Tn * rowq;
	const ST* vb_ = v + (int64_t)b * g.Tn * rowv;
	const ST* dvob = dvo + (int64_t)b * g.Tn * rowv;
	const T* Pb = P + (int64_t)b * g.E * g.H;
	T* DAb = DA + (int64_t)b * g.E * g.H;

	T qv[MC][VEC], dvod[MC][VEC], vbd[MC][VEC], X[MC][VEC], Y[MC][VEC], dvba[MC][VEC];
	bool okq[MC], okv[MC];
	int offq[MC], offv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		okq[m] = L.head_ok && w0 < g.W;
		okv[m] = L.head_ok && w0 < g.Wv;
		offq[m] = L.h * g.W + w0;
		offv[m] = L.h * g.Wv + w0;
#pragma unroll
		for (int i = 0; i < VEC; i++) { qv[m][i] = 0; dvod[m][i] = 0; vbd[m][i] = 0; X[m][i] = 0; Y[m][i] = 0; dvba[m][i] = 0; }
		if (okq[m]) ldv<T, VEC>(qb + (int64_t)L.tok * rowq + offq[m], qv[m]);
		if (okv[m]) ldv<T, VEC>(dvob + (int64_t)L.tok * rowv + offv[m], dvod[m]);
		if (BIDI && okv[m]) ldv<T, VEC>(vbk + ((int64_t)b * g.Tn + L.tok) * rowv + offv[m], vbd[m]);
	}
	T S = 0;
	int sidx[EU];
#pragma unroll
	for (int u = 0; u < EU; u++) sidx[u] = L.pb < L.pe ? csr_src[min(L.pb + u, L.pe - 1)] : 0;
	for (int p = L.pb; p < L.pe; p += EU) {
		T kv[EU][MC][VEC], vs[EU][MC][VEC], dvos[EU][MC][VEC], pe[EU];
#pragma unroll
		for (int u = 0; u < EU; u++) {
			pe[u] = L.head_ok ? Pb[(int64_t)min(p + u, L.pe - 1) * g.H + L.h] : (T)0;
#pragma unroll
			for (int m = 0; m < MC; m++) {
#pragma unroll
				for (int i = 0; i < VEC; i++) { kv[u][m][i] = qv[m][i]; vs[u][m][i] = 0; dvos[u][m][i] = 0; }
				if (okq[m]) ldv<T, VEC>(kb + (int64_t)sidx[u] * rowq + offq[m], kv[u][m]);
				if (okv[m]) ldv<T, VEC>(vb_ + (int64_t)sidx[u] * rowv + offv[m], vs[u][m]);
				if (BIDI && okv[m]) ldv<T, VEC>(dvob + (int64_t)sidx[u] * rowv + offv[m], dvos[u][m]);
			}
		}
#pragma unroll
		for (int u = 0; u < EU; u++) sidx[u] = csr_src[min(p + EU + u, L.pe - 1)];
		T dp[EU];
#pragma unroll
		for (int u = 0; u < EU; u++) {
			dp[u] = 0;
#pragma unroll
			for (int m = 0; m < MC; m++)
#pragma unroll
				for (int i = 0; i < VEC; i++) {
					dp[u] += vs[u][m][i] * dvod[m][i];
					if (BIDI) dp[u] += vbd[m][i] * dvos[u][m][i];
				}
		}
#pragma unroll
		for (int u = 0; u < EU; u++) dp[u] = group_sum(dp[u], G);
#pragma unroll
		for (int u = 0; u < EU; u++) {
			if (p + u < L.pe) {  // uniform
				const T pd = pe[u] * dp[u];
				S += pd;
#pragma unroll
				for (int m = 0; m < MC; m++)
#pragma unroll
					for (int i = 0; i < VEC; i++) {
						const T sg = sgn_t(qv[m][i] - kv[u][m][i]);
						X[m][i] += sg * pd;
						Y[m][i] += sg * pe[u];
						if (BIDI) dvba[m][i] += pe[u] * dvos[u][m][i];
					}
				if (L.sub == 0 && L.head_ok) DAb[(int64_t)(p + u) * g.H + L.h] = dp[u];
			}
		}
	}
	S = wg_sum<T, NWV>(S, smem, L.wave);
#pragma unroll
	for (int m = 0; m < MC; m++)
#pragma unroll
		for (int i = 0; i < VEC; i++) {
			X[m][i] = wg_sum<T, NWV>(X[m][i], smem, L.wave);
			if (use_softmax) Y[m][i] = wg_sum<T, NWV>(Y[m][i], smem, L.wave);
			if (BIDI) dvba[m][i] = wg_sum<T, NWV>(dvba[m][i], smem, L.wave);
		}
	if (L.wave == 0 || NWV == 1) {
#pragma unroll
		for (int m = 0; m < MC; m++) {
			T o[VEC];
#pragma unroll
			for (int i = 0; i < VEC; i++) o[i] = use_softmax ? scale * (X[m][i] - S * Y[m][i]) : scale * X[m][i];
			if (okq[m]) stv<T, VEC>(dq + ((int64_t)b * g.Tn + L.tok) * rowq + offq[m], o);
			if (BIDI && okv[m]) stv<T, VEC>(dvb + ((int64_t)b * g.Tn + L.tok) * rowv + offv[m], dvba[m]);
		}
	}
	wave_store_load_fence();  // dp values were stored by lane 0 of each head group
	if (L.head_ok) {
		for (int p = L.pb + L.sub; p < L.pe; p += G) {
			const int64_t ix = (int64_t)p * g.H + L.h;
			const T pe = Pb[ix], dp = DAb[ix];
			DAb[ix] = use_softmax ? pe * (dp - S) : pe * dp;
		}
	}
}

// src pass: dv[src] = sum p * dvo[dst];  dk[src] = -scale * sum sign(q[dst]-k[src]) * da
template <typename T, int VEC, int MC, int NWV, typename S>
__global__ __launch_bounds__(NWV == 1 ? 256 : 64 * NWV) void sparse_bwd_src(
    const S* __restrict__ dvo, const S* __restrict__ q, const S* __restrict__ k, const int* __restrict__ src_ptr,
    const int* __restrict__ csc_dst, const int* __restrict__ csc_slot, const int* __restrict__ long_list,
    const int* __restrict__ n_long, const T* __restrict__ P, const T* __restrict__ DA, S* __restrict__ dv,
    S* __restrict__ dk, Geo g, T scale)
{
	extern __shared__ unsigned char smem_raw[];
	T* smem = reinterpret_cast<T*>(smem_raw);
	constexpr int EU = Unroll<MC>::EU;
	Lane L;
	if (!wave_item<NWV>(g, src_ptr, long_list, n_long, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowq = (int64_t)g.H * g.W, rowv = (int64_t)g.H * g.Wv;
	const S* qb = q + (int64_t)b * g.Tn * rowq;
	const S* dvob = dvo + (int64_t)b * g.Tn * rowv;
	const T* Pb = P + (int64_t)b * g.E * g.H;
	const T* DAb = DA + (int64_t)b * g.E * g.H;
	T kv[MC][VEC], dva[MC][VEC], dka[MC][VEC];
	bool okq[MC], okv[MC];
	int offq[MC], offv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		okq[m] = L.head_ok && w0 < g.W;
		okv[m] = L.head_ok && w0 < g.Wv;
		offq[m] = L.h * g.W + w0;
		offv[m] = L.h * g.Wv + w0;
#pragma unroll
		for (int i = 0; i < VEC; i++) { kv[m][i] = 0; dva[m][i] = 0; dka[m][i] = 0; }
		if (okq[m]) ldv<T, VEC>(k + ((int64_t)b * g.Tn + L.tok) * rowq + offq[m], kv[m]);
	}
	int didx[EU], slot[EU];
#pragma unroll
	for (int u = 0; u < EU; u++) {
		const int e = min(L.pb + u, L.pe - 1);
		didx[u] = L.pb < L.pe ? csc_dst[e] : 0;
		slot[u] = L.pb < L.pe ? csc_slot[e] : 0;
	}
	for (int e0 = L.pb; e0 < L.pe; e0 += EU) {
		T qd[EU][MC][VEC], dd[EU][MC][VEC], pe[EU], da[EU];
#pragma unroll
		for (int u = 0; u < EU; u++) {
			const int64_t ix = (int64_t)slot[u] * g.H + L.h;
			pe[u] = L.head_ok ? Pb[ix] : (T)0;
			da[u] = L.head_ok ? DAb[ix] : (T)0;
#pragma unroll
			for (int m = 0; m < MC; m++) {
#pragma unroll
				for (int i = 0; i < VEC; i++) { qd[u][m][i] = kv[m][i]; dd[u][m][i] = 0; }
				if (okq[m]) ldv<T, VEC>(qb + (int64_t)didx[u] * rowq + offq[m], qd[u][m]);
				if (okv[m]) ldv<T, VEC>(dvob + (int64_t)didx[u] * rowv + offv[m], dd[u][m]);
			}
		}
#pragma unroll
		for (int u = 0; u < EU; u++) {
			const int e = min(e0 + EU + u, L.pe - 1);
			didx[u] = csc_dst[e];
			slot[u] = csc_slot[e];
		}
#pragma unroll
		for (int u = 0; u < EU; u++)
			if (e0 + u < L.pe)
#pragma unroll
				for (int m = 0; m < MC; m++)
#pragma unroll
					for (int i = 0; i < VEC; i++) {
						dva[m][i] += pe[u] * dd[u][m][i];
						dka[m][i] += sgn_t(qd[u][m][i] - kv[m][i]) * da[u];
					}
	}
#pragma unroll
	for (int m = 0; m < MC; m++)
#pragma unroll
		for (int i = 0; i < VEC; i++) {
			dva[m][i] = wg_sum<T, NWV>(dva[m][i], smem, L.wave);
			dka[m][i] = wg_sum<T, NWV>(dka[m][i], smem, L.wave);
		}
	if (L.wave == 0 || NWV == 1) {
#pragma unroll
		for (int m = 0; m < MC; m++) {
#pragma unroll
			for (int i = 0; i < VEC; i++) dka[m][i] *= -scale;
			if (okv[m]) stv<T, VEC>(dv + ((int64_t)b * g.Tn + L.tok) * rowv + offv[m], dva[m]);
			if (okq[m]) stv<T, VEC>(dk + ((int64_t)b * g.Tn + L.tok) * rowq + offq[m], dka[m]);
		}
	}
}

// ---------------------------------------------------------------------------------- host side

constexpr int LONG_NWV = 8;  // waves that share one long segment

struct Shape {
	int64_t B, T, H, W, Wv, E;
};

struct Cfg {
	int vec, mc;
	Geo g;
	dim3 grid, block;            // wave-per-item launch
	dim3 lgrid, lblock;          // workgroup-per-long-segment launch (only when g.long_on)
	const int *long_dst, *long_src, *n_long_dst, *n_long_src;
	const int *dst_ptr, *src_ptr, *csr_src, *csc_dst, *csc_slot;
};

int make_cfg(const Shape& s, const void* plan, const void* const* ptrs, int n_ptrs, Cfg& c)
{
	if (s.B < 0 || s.T < 0 || s.H < 0 || s.W < 1 || s.Wv < 1 || s.E < 0) return L1ATTN_ERR_ARG;
	if (s.T > (1LL << 30) || s.E > 2147483647LL - 4096 || s.B > 65535 || s.H > 32768) return L1ATTN_ERR_RANGE;
	bool aligned = true;
	for (int i = 0; i < n_ptrs; i++) aligned = aligned && ((((uintptr_t)ptrs[i]) & 15) == 0);
	c.vec = (s.W % 4 == 0 && s.Wv % 4 == 0 && aligned) ? 4 : 1;
	const int64_t wmax = s.W > s.Wv ? s.W : s.Wv;
	int64_t chunks = l1_cdiv(wmax, c.vec);
	if (chunks > 256) return L1ATTN_ERR_RANGE;
	c.mc = chunks <= 64 ? 1 : 4;
	int64_t per = l1_cdiv(chunks, c.mc);
	int lg = 0;
	while ((1 << lg) < per) lg++;
	c.g.Tn = (int)s.T; c.g.H = (int)s.H; c.g.W = (int)s.W; c.g.Wv = (int)s.Wv; c.g.E = (int)s.E;
	c.g.log2G = lg;
	c.g.n_hc = (int)l1_cdiv(s.H, 64 >> lg);
	const int64_t items = s.T * c.g.n_hc;
	if (l1_cdiv(items, 4) > 2147483647LL || c.g.n_hc > 65535) return L1ATTN_ERR_RANGE;
	c.grid = dim3((unsigned)l1_cdiv(items, 4), (unsigned)s.B, 1);
	c.block = dim3(256);
	const PlanLayout L = plan_layout(s.E, s.T);
	const int* words = (const int*)plan;
	// a list of E edges has at most E / PLAN_LONG_SEGMENT long segments: that bounds the second launch
	c.g.long_on = (c.mc == 1 && s.E > PLAN_LONG_SEGMENT) ? 1 : 0;
	c.lgrid = dim3((unsigned)L.long_cap, (unsigned)s.B, (unsigned)c.g.n_hc);
	c.lblock = dim3(64 * LONG_NWV);
	c.long_dst = words + L.long_dst;
	c.long_src = words + L.long_src;
	c.n_long_dst = words + PLAN_H_NLONG_DST;
	c.n_long_src = words + PLAN_H_NLONG_SRC;
	c.dst_ptr = words + L.dst_ptr;
	c.src_ptr = words + L.src_ptr;
	c.csr_src = words + L.csr_src;
	c.csc_dst = words + L.csc_dst;
	c.csc_slot = words + L.csc_slot;
	return L1ATTN_OK;
}

// CALL(VEC, MC, NWV, grid, block, lds_bytes)
#define DISPATCH_VM(cfg, T, CALL)                                                          \
	do {                                                                                   \
		if ((cfg).vec == 4 && (cfg).mc == 1) { CALL(4, 1, 1, (cfg).grid, (cfg).block, 0); } \
		else if ((cfg).vec == 4) { CALL(4, 4, 1, (cfg).grid, (cfg).block, 0); }            \
		else if ((cfg).mc == 1) { CALL(1, 1, 1, (cfg).grid, (cfg).block, 0); }             \
		else { CALL(1, 4, 1, (cfg).grid, (cfg).block, 0); }                                \
		if ((cfg).g.long_on) {                                                             \
			const size_t lds__ = (size_t)LONG_NWV * 64 * sizeof(T);                        \
			if ((cfg).vec == 4) { CALL(4, 1, LONG_NWV, (cfg).lgrid, (cfg).lblock, lds__); } \
			else { CALL(1, 1, LONG_NWV, (cfg).lgrid, (cfg).lblock, lds__); }               \
		}                                                                                  \
	} while (0)

template <typename T, typename S>
int sparse_fwd_impl(const S* v, const S* vbk, const S* q, const S* k, const void* plan, S* vo, T* P, Shape s,
                    int use_softmax, bool bidi, hipStream_t st)
{
	if (s.B * s.T * s.H == 0) return L1ATTN_OK;
	if (!v || !q || !k || !plan || !vo || (s.E > 0 && !P) || (bidi && !vbk)) return L1ATTN_ERR_ARG;
	const void* ptrs[] = {v, vbk, q, k, vo};
	Cfg c;
	int rc = make_cfg(s, plan, ptrs, 5, c);
	if (rc) return rc;
	const T scale = (T)(-1.0 / sqrt((double)s.W));
#define CALL(V, M, N, GRID, BLOCK, LDS)                                                                         \
	hipLaunchKernelGGL((sparse_fwd_dst<T, V, M, N, S>), GRID, BLOCK, LDS, st, v, q, k, c.dst_ptr, c.csr_src,        \
	                   c.long_dst, c.n_long_dst, vo, P, c.g, use_softmax, scale)
	DISPATCH_VM(c, T, CALL);
#undef CALL
	L1_LAUNCH_CHECK();
	if (bidi) {
#define CALL(V, M, N, GRID, BLOCK, LDS)                                                                         \
	hipLaunchKernelGGL((sparse_fwd_src<T, V, M, N, S>), GRID, BLOCK, LDS, st, vbk, c.src_ptr, c.csc_dst,            \
	                   c.csc_slot, c.long_src, c.n_long_src, (const T*)P, vo, c.g)
		DISPATCH_VM(c, T, CALL);
#undef CALL
		L1_LAUNCH_CHECK();
	}
	return L1ATTN_OK;
}

template <typename T, typename S>
int sparse_bwd_impl(const S* dvo, const S* v, const S* vbk, const S* q, const S* k, const void* plan, const T* P,
                    S* dv, S* dvb, S* dq, S* dk, T* DA, Shape s, int use_softmax, bool bidi, hipStream_t st)
{
	if (s.B * s.T * s.H == 0) return L1ATTN_OK;
	if (!dvo || !v || !q || !k || !plan || !dv || !dq || !dk || (s.E > 0 && (!P || !DA)) || (bidi && (!vbk || !dvb)))
		return L1ATTN_ERR_ARG;
	const void* ptrs[] = {dvo, v, vbk, q, k, dv, dvb, dq, dk};
	Cfg c;
	int rc = make_cfg(s, plan, ptrs, 9, c);
	if (rc) return rc;
	const T scale = (T)(-1.0 / sqrt((double)s.W));
	if (bidi) {
#define CALL(V, M, N, GRID, BLOCK, LDS)                                                                         \
	hipLaunchKernelGGL((sparse_bwd_dst<T, V, M, true, N, S>), GRID, BLOCK, LDS, st, dvo, v, vbk, q, k, c.dst_ptr,   \
	                   c.csr_src, c.long_dst, c.n_long_dst, P, DA, dq, dvb, c.g, use_softmax, scale)
		DISPATCH_VM(c, T, CALL);
#undef CALL
	} else {
#define CALL(V, M, N, GRID, BLOCK, LDS)                                                                         \
	hipLaunchKernelGGL((sparse_bwd_dst<T, V, M, false, N, S>), GRID, BLOCK, LDS, st, dvo, v, vbk, q, k, c.dst_ptr,  \
	                   c.csr_src, c.long_dst, c.n_long_dst, P, DA, dq, dvb, c.g, use_softmax, scale)
		DISPATCH_VM(c, T, CALL);
#undef CALL
	}
	L1_LAUNCH_CHECK();
#define CALL(V, M, N, GRID, BLOCK, LDS)                                                                         \
	hipLaunchKernelGGL((sparse_bwd_src<T, V, M, N, S>), GRID, BLOCK, LDS, st, dvo, q, k, c.src_ptr, c.csc_dst,      \
	                   c.csc_slot, c.long_src, c.n_long_src, P, (const T*)DA, dv, dk, c.g, scale)
	DISPATCH_VM(c, T, CALL);
#undef CALL
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

}  // namespace

extern "C" {

#define L1_SPARSE_ENTRY(SFX, TYPE)                                                                                  \
	int l1attn_sparse_fwd_##SFX(const TYPE* v, const TYPE* q, const TYPE* k, const void* plan, TYPE* vo, TYPE* P,   \
	                            int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int use_softmax, \
	                            void* stream)                                                                       \
	{                                                                                                               \
		return sparse_fwd_impl<TYPE, TYPE>(v, nullptr, q, k, plan, vo, P, Shape{B, T, H, W, Wv, E}, use_softmax, false,   \
		                             (hipStream_t)stream);                                                          \
	}                                                                                                               \
	int l1attn_sparse_bwd_##SFX(const TYPE* dvo, const TYPE* v, const TYPE* q, const TYPE* k, const void* plan,     \
	                            const TYPE* P, TYPE* dv, TYPE* dq, TYPE* dk, TYPE* DA, int64_t B, int64_t T,        \
	                            int64_t H, int64_t W, int64_t Wv, int64_t E, int use_softmax, void* stream)         \
	{                                                                                                               \
		return sparse_bwd_impl<TYPE, TYPE>(dvo, v, nullptr, q, k, plan, P, dv, nullptr, dq, dk, DA,                       \
		                             Shape{B, T, H, W, Wv, E}, use_softmax, false, (hipStream_t)stream);            \
	}                                                                                                               \
	int l1attn_sparse_bidi_fwd_##SFX(const TYPE* vf, const TYPE* vb, const TYPE* q, const TYPE* k,                  \
	                                 const void* plan, TYPE* vo, TYPE* P, int64_t B, int64_t T, int64_t H,          \
	                                 int64_t W, int64_t Wv, int64_t E, int use_softmax, void* stream)               \
	{                                                                                                               \
		return sparse_fwd_impl<TYPE, TYPE>(vf, vb, q, k, plan, vo, P, Shape{B, T, H, W, Wv, E}, use_softmax, true,        \
		                             (hipStream_t)stream);                                                          \
	}                                                                                                               \
	int l1attn_sparse_bidi_bwd_##SFX(const TYPE* dvo, const TYPE* vf, const TYPE* vb, const TYPE* q,                \
	                                 const TYPE* k, const void* plan, const TYPE* P, TYPE* dvf, TYPE* dvb,          \
	                                 TYPE* dq, TYPE* dk, TYPE* DA, int64_t B, int64_t T, int64_t H, int64_t W,      \
	                                 int64_t Wv, int64_t E, int use_softmax, void* stream)                          \
	{                                                                                                               \
		return sparse_bwd_impl<TYPE, TYPE>(dvo, vf, vb, q, k, plan, P, dvf, dvb, dq, dk, DA, Shape{B, T, H, W, Wv, E},    \
		                             use_softmax, true, (hipStream_t)stream);                                       \
	}

L1_SPARSE_ENTRY(f32, float)
L1_SPARSE_ENTRY(f64, double)

// Forward with 16-bit rows (the reference dispatches its forward kernels for Half as well,
// cuda/l1attn_sparse_cuda_kernel.cu:405-435 and :684-714, and its backward kernels for float and double
// only, :483-519): v, q, k and vo are IEEE half (f16) or bfloat16 (bf16) in memory, the logits, the
// softmax and the value sums run in fp32, the weights P are fp32.
#define L1_SPARSE_FWD16_ENTRY(SFX, STYPE)                                                                           \
	int l1attn_sparse_fwd_##SFX(const void* v, const void* q, const void* k, const void* plan, void* vo, float* P,   \
	                            int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int use_softmax, \
	                            void* stream)                                                                       \
	{                                                                                                               \
		return sparse_fwd_impl<float, STYPE>((const STYPE*)v, nullptr, (const STYPE*)q, (const STYPE*)k, plan,      \
		                                     (STYPE*)vo, P, Shape{B, T, H, W, Wv, E}, use_softmax, false,           \
		                                     (hipStream_t)stream);                                                  \
	}                                                                                                               \
	int l1attn_sparse_bidi_fwd_##SFX(const void* vf, const void* vb, const void* q, const void* k,                  \
	                                 const void* plan, void* vo, float* P, int64_t B, int64_t T, int64_t H,         \
	                                 int64_t W, int64_t Wv, int64_t E, int use_softmax, void* stream)               \
	{                                                                                                               \
		return sparse_fwd_impl<float, STYPE>((const STYPE*)vf, (const STYPE*)vb, (const STYPE*)q, (const STYPE*)k,  \
		                                     plan, (STYPE*)vo, P, Shape{B, T, H, W, Wv, E}, use_softmax, true,      \
		                                     (hipStream_t)stream);                                                  \
	}

L1_SPARSE_FWD16_ENTRY(f16, f16_t)
L1_SPARSE_FWD16_ENTRY(bf16, bf16_t)

// Backward with 16-bit rows (an addition: the reference's backward launchers take float and double only):
// dvo, v/vf, vb, q, k and the gradients dv/dvf, dvb, dq, dk are 16-bit in memory, P and DA fp32, every sum fp32,
// each gradient element rounded once on store.
#define L1_SPARSE_BWD16_ENTRY(SFX, STYPE)                                                                           \
	int l1attn_sparse_bwd_##SFX(const void* dvo, const void* v, const void* q, const void* k, const void* plan,     \
	                            const float* P, void* dv, void* dq, void* dk, float* DA, int64_t B, int64_t T,      \
	                            int64_t H, int64_t W, int64_t Wv, int64_t E, int use_softmax, void* stream)         \
	{                                                                                                               \
		return sparse_bwd_impl<float, STYPE>((const STYPE*)dvo, (const STYPE*)v, nullptr, (const STYPE*)q,          \
		                                     (const STYPE*)k, plan, P, (STYPE*)dv, nullptr, (STYPE*)dq, (STYPE*)dk, \
		                                     DA, Shape{B, T, H, W, Wv, E}, use_softmax, false, (hipStream_t)stream); \
	}                                                                                                               \
	int l1attn_sparse_bidi_bwd_##SFX(const void* dvo, const void* vf, const void* vb, const void* q, const void* k, \
	                                 const void* plan, const float* P, void* dvf, void* dvb, void* dq, void* dk,    \
	                                 float* DA, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,  \
	                                 int use_softmax, void* stream)                                                 \
	{                                                                                                               \
		return sparse_bwd_impl<float, STYPE>((const STYPE*)dvo, (const STYPE*)vf, (const STYPE*)vb,                 \
		                                     (const STYPE*)q, (const STYPE*)k, plan, P, (STYPE*)dvf, (STYPE*)dvb,   \
		                                     (STYPE*)dq, (STYPE*)dk, DA, Shape{B, T, H, W, Wv, E}, use_softmax,     \
		                                     true, (hipStream_t)stream);                                            \
	}

L1_SPARSE_BWD16_ENTRY(f16, f16_t)
L1_SPARSE_BWD16_ENTRY(bf16, bf16_t)

}  // extern "C"
