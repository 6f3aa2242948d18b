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

template <typename T, int VEC>
__device__ __forceinline__ void ldv(const T* __restrict__ p, T (&x)[VEC])
{
	if constexpr (VEC == 4 && sizeof(T) == 4) {
		const float4 t = *reinterpret_cast<const float4*>(p);
		x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
	} else if constexpr (VEC == 4 && sizeof(T) == 8) {
		const double2 a = *reinterpret_cast<const double2*>(p);
		const double2 b = *reinterpret_cast<const double2*>(p + 2);
		x[0] = a.x; x[1] = a.y; x[2] = b.x; x[3] = b.y;
	} else {
#pragma unroll
		for (int i = 0; i < VEC; i++) x[i] = p[i];
	}
}

template <typename T, int VEC>
__device__ __forceinline__ void stv(T* __restrict__ p, const T (&x)[VEC])
{
	if constexpr (VEC == 4 && sizeof(T) == 4) {
		*reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
	} else if constexpr (VEC == 4 && sizeof(T) == 8) {
		*reinterpret_cast<double2*>(p) = make_double2(x[0], x[1]);
		*reinterpret_cast<double2*>(p + 2) = make_double2(x[2], x[3]);
	} else {
#pragma unroll
		for (int i = 0; i < VEC; i++) p[i] = x[i];
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

// geometry of one work item, shared by all kernels
struct Geo {
	int Tn, H, W, Wv, E;
	int log2G;  // lanes per head = 1 << log2G
	int n_hc;   // head chunks per token = ceil(H / (64 >> log2G))
};

struct Lane {
	int tok, h, sub;
	bool head_ok;
};

__device__ __forceinline__ bool wave_item(const Geo& g, Lane& L)
{
	const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
	const int lane = threadIdx.x & 63;
	const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave;
	if (item >= (int64_t)g.Tn * g.n_hc) return false;
	L.tok = (int)(item / g.n_hc);
	const int hc = (int)(item % g.n_hc);
	L.sub = lane & ((1 << g.log2G) - 1);
	L.h = hc * (64 >> g.log2G) + (lane >> g.log2G);
	L.head_ok = L.h < g.H;
	return true;
}

// ---------------------------------------------------------------------------------- forward

// dst pass: logits, softmax with the "+1" denominator, value sum.  Writes vo rows and P.
template <typename T, int VEC, int MC>
__global__ __launch_bounds__(256) void sparse_fwd_dst(const T* __restrict__ v, const T* __restrict__ q,
                                                        const T* __restrict__ k, const int* __restrict__ dst_ptr,
                                                        const int* __restrict__ csr_src, T* __restrict__ vo,
                                                        T* __restrict__ P, Geo g, int use_softmax, T scale)
{
	Lane L;
	if (!wave_item(g, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowq = (int64_t)g.H * g.W, rowv = (int64_t)g.H * g.Wv;
	const T* qb = q + (int64_t)b * g.Tn * rowq;
	const T* kb = k + (int64_t)b * g.Tn * rowq;
	const T* vb = v + (int64_t)b * g.Tn * rowv;
	T* Pb = P + (int64_t)b * g.E * g.H;

	T qv[MC][VEC], acc[MC][VEC];
	bool okq[MC], okv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		okq[m] = L.head_ok && w0 < g.W;
		okv[m] = L.head_ok && w0 < g.Wv;
#pragma unroll
		for (int i = 0; i < VEC; i++) { qv[m][i] = 0; acc[m][i] = 0; }
		if (okq[m]) ldv<T, VEC>(qb + (int64_t)L.tok * rowq + L.h * g.W + w0, qv[m]);
	}
	const int p0 = dst_ptr[L.tok], p1 = dst_ptr[L.tok + 1];
	T den = use_softmax ? (T)1 : (T)0;
	for (int p = p0; p < p1; p++) {
		const int src = csr_src[p];
		T d = 0;
		T vv[MC][VEC];
#pragma unroll
		for (int m = 0; m < MC; m++) {
			const int w0 = (m * G + L.sub) * VEC;
			T kv[VEC];
#pragma unroll
			for (int i = 0; i < VEC; i++) { kv[i] = qv[m][i]; vv[m][i] = 0; }
			if (okq[m]) ldv<T, VEC>(kb + (int64_t)src * rowq + L.h * g.W + w0, kv);
			if (okv[m]) ldv<T, VEC>(vb + (int64_t)src * rowv + L.h * g.Wv + w0, vv[m]);
#pragma unroll
			for (int i = 0; i < VEC; i++) d += abs_t(qv[m][i] - kv[i]);
		}
		d = group_sum(d, G);
		const T e = exp_t(d * scale);
		den += e;
#pragma unroll
		for (int m = 0; m < MC; m++)
#pragma unroll
			for (int i = 0; i < VEC; i++) acc[m][i] += e * vv[m][i];
		if (L.sub == 0 && L.head_ok) Pb[(int64_t)p * g.H + L.h] = e;
	}
	const T inv = use_softmax ? (T)1 / den : (T)1;
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
#pragma unroll
		for (int i = 0; i < VEC; i++) acc[m][i] *= inv;
		if (okv[m]) stv<T, VEC>(vo + ((int64_t)b * g.Tn + L.tok) * rowv + L.h * g.Wv + w0, acc[m]);
	}
	// the weights below were stored by lane 0 of each head group: make them visible to its other lanes
	__threadfence();
	if (use_softmax && L.head_ok) {
		// normalise the stored weights; the G lanes of a head take every G-th slot
		for (int p = p0 + L.sub; p < p1; p += G) Pb[(int64_t)p * g.H + L.h] *= inv;
	}
}

// bidi src pass: vo[b,src] += sum over the src's edges of p * vb[b,dst]   (cpp/l1attn_sparse_bidi_drv.cpp:93-96)
template <typename T, int VEC, int MC>
__global__ __launch_bounds__(256) void sparse_fwd_src(const T* __restrict__ vbk, const int* __restrict__ src_ptr,
                                                        const int* __restrict__ csc_dst,
                                                        const int* __restrict__ csc_slot, const T* __restrict__ P,
                                                        T* __restrict__ vo, Geo g)
{
	Lane L;
	if (!wave_item(g, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowv = (int64_t)g.H * g.Wv;
	const T* vb = vbk + (int64_t)b * g.Tn * rowv;
	const T* Pb = P + (int64_t)b * g.E * g.H;
	T acc[MC][VEC];
	bool okv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		okv[m] = L.head_ok && (m * G + L.sub) * VEC < g.Wv;
#pragma unroll
		for (int i = 0; i < VEC; i++) acc[m][i] = 0;
	}
	const int i0 = src_ptr[L.tok], i1 = src_ptr[L.tok + 1];
	for (int e = i0; e < i1; e++) {
		const int dst = csc_dst[e], slot = csc_slot[e];
		const T pe = L.head_ok ? Pb[(int64_t)slot * g.H + L.h] : (T)0;
#pragma unroll
		for (int m = 0; m < MC; m++) {
			T x[VEC];
#pragma unroll
			for (int i = 0; i < VEC; i++) x[i] = 0;
			if (okv[m]) ldv<T, VEC>(vb + (int64_t)dst * rowv + L.h * g.Wv + (m * G + L.sub) * VEC, x);
#pragma unroll
			for (int i = 0; i < VEC; i++) acc[m][i] += pe * x[i];
		}
	}
#pragma unroll
	for (int m = 0; m < MC; m++) {
		if (okv[m]) {
			T* o = vo + ((int64_t)b * g.Tn + L.tok) * rowv + L.h * g.Wv + (m * G + L.sub) * VEC;
			T x[VEC];
			ldv<T, VEC>(o, x);
#pragma unroll
			for (int i = 0; i < VEC; i++) x[i] += acc[m][i];
			stv<T, VEC>(o, x);
		}
	}
}

// --------------------------------------------------------------------------------- backward

// dst pass.  For every edge of the dst:  dp = v[src].dvo[dst] (+ vb[dst].dvo[src] for bidi);
// S = sum p*dp;  dq[dst] = scale * sum sign(q-k) * p * (dp - S)  accumulated as X - S*Y in one walk;
// bidi: dvb[dst] = sum p * dvo[src].  Leaves da = p*(dp - S) (or p*dp) per edge in DA.
template <typename T, int VEC, int MC, bool BIDI>
__global__ __launch_bounds__(256) void sparse_bwd_dst(const T* __restrict__ dvo, const T* __restrict__ v,
                                                        const T* __restrict__ vbk, const T* __restrict__ q,
                                                        const T* __restrict__ k, const int* __restrict__ dst_ptr,
                                                        const int* __restrict__ csr_src, const T* __restrict__ P,
                                                        T* __restrict__ DA, T* __restrict__ dq,
                                                        T* __restrict__ dvb, Geo g, int use_softmax, T scale)
{
	Lane L;
	if (!wave_item(g, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowq = (int64_t)g.H * g.W, rowv = (int64_t)g.H * g.Wv;
	const T* qb = q + (int64_t)b * g.Tn * rowq;
	const T* kb = k + (int64_t)b * g.Tn * rowq;
	const T* vb_ = v + (int64_t)b * g.Tn * rowv;
	const T* dvob = dvo + (int64_t)b * g.Tn * rowv;
	const T* Pb = P + (int64_t)b * g.E * g.H;
	T* DAb = DA + (int64_t)b * g.E * g.H;

	T qv[MC][VEC], dvod[MC][VEC], vbd[MC][VEC], X[MC][VEC], Y[MC][VEC], dvba[MC][VEC];
	bool okq[MC], okv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		okq[m] = L.head_ok && w0 < g.W;
		okv[m] = L.head_ok && w0 < g.Wv;
#pragma unroll
		for (int i = 0; i < VEC; i++) { qv[m][i] = 0; dvod[m][i] = 0; vbd[m][i] = 0; X[m][i] = 0; Y[m][i] = 0; dvba[m][i] = 0; }
		if (okq[m]) ldv<T, VEC>(qb + (int64_t)L.tok * rowq + L.h * g.W + w0, qv[m]);
		if (okv[m]) ldv<T, VEC>(dvob + (int64_t)L.tok * rowv + L.h * g.Wv + w0, dvod[m]);
		if (BIDI && okv[m]) ldv<T, VEC>(vbk + ((int64_t)b * g.Tn + L.tok) * rowv + L.h * g.Wv + w0, vbd[m]);
	}
	const int p0 = dst_ptr[L.tok], p1 = dst_ptr[L.tok + 1];
	T S = 0;
	for (int p = p0; p < p1; p++) {
		const int src = csr_src[p];
		T dp = 0;
		T sg[MC][VEC], dvos[MC][VEC];
#pragma unroll
		for (int m = 0; m < MC; m++) {
			const int w0 = (m * G + L.sub) * VEC;
			T kv[VEC], vs[VEC];
#pragma unroll
			for (int i = 0; i < VEC; i++) { kv[i] = qv[m][i]; vs[i] = 0; dvos[m][i] = 0; }
			if (okq[m]) ldv<T, VEC>(kb + (int64_t)src * rowq + L.h * g.W + w0, kv);
			if (okv[m]) ldv<T, VEC>(vb_ + (int64_t)src * rowv + L.h * g.Wv + w0, vs);
			if (BIDI && okv[m]) ldv<T, VEC>(dvob + (int64_t)src * rowv + L.h * g.Wv + w0, dvos[m]);
#pragma unroll
			for (int i = 0; i < VEC; i++) {
				dp += vs[i] * dvod[m][i];
				if (BIDI) dp += vbd[m][i] * dvos[m][i];
				sg[m][i] = sgn_t(qv[m][i] - kv[i]);
			}
		}
		dp = group_sum(dp, G);
		const T pe = L.head_ok ? Pb[(int64_t)p * g.H + L.h] : (T)0;
		const T pd = pe * dp;
		S += pd;
#pragma unroll
		for (int m = 0; m < MC; m++)
#pragma unroll
			for (int i = 0; i < VEC; i++) {
				X[m][i] += sg[m][i] * pd;
				Y[m][i] += sg[m][i] * pe;
				if (BIDI) dvba[m][i] += pe * dvos[m][i];
			}
		if (L.sub == 0 && L.head_ok) DAb[(int64_t)p * g.H + L.h] = dp;
	}
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		T o[VEC];
#pragma unroll
		for (int i = 0; i < VEC; i++) o[i] = use_softmax ? scale * (X[m][i] - S * Y[m][i]) : scale * X[m][i];
		if (okq[m]) stv<T, VEC>(dq + ((int64_t)b * g.Tn + L.tok) * rowq + L.h * g.W + w0, o);
		if (BIDI && okv[m]) stv<T, VEC>(dvb + ((int64_t)b * g.Tn + L.tok) * rowv + L.h * g.Wv + w0, dvba[m]);
	}
	__threadfence();  // dp values were stored by lane 0 of each head group
	if (L.head_ok) {
		for (int p = p0 + L.sub; p < p1; p += G) {
			const int64_t ix = (int64_t)p * g.H + L.h;
			const T pe = Pb[ix], dp = DAb[ix];
			DAb[ix] = use_softmax ? pe * (dp - S) : pe * dp;
		}
	}
}

// src pass: dv[src] = sum p * dvo[dst];  dk[src] = -scale * sum sign(q[dst]-k[src]) * da
template <typename T, int VEC, int MC>
__global__ __launch_bounds__(256) void sparse_bwd_src(const T* __restrict__ dvo, const T* __restrict__ q,
                                                        const T* __restrict__ k, const int* __restrict__ src_ptr,
                                                        const int* __restrict__ csc_dst,
                                                        const int* __restrict__ csc_slot, const T* __restrict__ P,
                                                        const T* __restrict__ DA, T* __restrict__ dv,
                                                        T* __restrict__ dk, Geo g, T scale)
{
	Lane L;
	if (!wave_item(g, L)) return;
	const int b = blockIdx.y, G = 1 << g.log2G;
	const int64_t rowq = (int64_t)g.H * g.W, rowv = (int64_t)g.H * g.Wv;
	const T* qb = q + (int64_t)b * g.Tn * rowq;
	const T* dvob = dvo + (int64_t)b * g.Tn * rowv;
	const T* Pb = P + (int64_t)b * g.E * g.H;
	const T* DAb = DA + (int64_t)b * g.E * g.H;
	T kv[MC][VEC], dva[MC][VEC], dka[MC][VEC];
	bool okq[MC], okv[MC];
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
		okq[m] = L.head_ok && w0 < g.W;
		okv[m] = L.head_ok && w0 < g.Wv;
#pragma unroll
		for (int i = 0; i < VEC; i++) { kv[m][i] = 0; dva[m][i] = 0; dka[m][i] = 0; }
		if (okq[m]) ldv<T, VEC>(k + ((int64_t)b * g.Tn + L.tok) * rowq + L.h * g.W + w0, kv[m]);
	}
	const int i0 = src_ptr[L.tok], i1 = src_ptr[L.tok + 1];
	for (int e = i0; e < i1; e++) {
		const int dst = csc_dst[e], slot = csc_slot[e];
		const int64_t ix = (int64_t)slot * g.H + L.h;
		const T pe = L.head_ok ? Pb[ix] : (T)0;
		const T da = L.head_ok ? DAb[ix] : (T)0;
#pragma unroll
		for (int m = 0; m < MC; m++) {
			const int w0 = (m * G + L.sub) * VEC;
			T qd[VEC], dd[VEC];
#pragma unroll
			for (int i = 0; i < VEC; i++) { qd[i] = kv[m][i]; dd[i] = 0; }
			if (okq[m]) ldv<T, VEC>(qb + (int64_t)dst * rowq + L.h * g.W + w0, qd);
			if (okv[m]) ldv<T, VEC>(dvob + (int64_t)dst * rowv + L.h * g.Wv + w0, dd);
#pragma unroll
			for (int i = 0; i < VEC; i++) {
				dva[m][i] += pe * dd[i];
				dka[m][i] += sgn_t(qd[i] - kv[m][i]) * da;
			}
		}
	}
#pragma unroll
	for (int m = 0; m < MC; m++) {
		const int w0 = (m * G + L.sub) * VEC;
#pragma unroll
		for (int i = 0; i < VEC; i++) dka[m][i] *= -scale;
		if (okv[m]) stv<T, VEC>(dv + ((int64_t)b * g.Tn + L.tok) * rowv + L.h * g.Wv + w0, dva[m]);
		if (okq[m]) stv<T, VEC>(dk + ((int64_t)b * g.Tn + L.tok) * rowq + L.h * g.W + w0, dka[m]);
	}
}

// ---------------------------------------------------------------------------------- host side

struct Shape {
	int64_t B, T, H, W, Wv, E;
};

struct Cfg {
	int vec, mc;
	Geo g;
	dim3 grid, block;
};

int make_cfg(const Shape& s, size_t elt, const void* const* ptrs, int n_ptrs, Cfg& c)
{
	if (s.B < 0 || s.T < 0 || s.H < 0 || s.W < 1 || s.Wv < 1 || s.E < 0) return L1ATTN_ERR_ARG;
	if (s.T > (1LL << 30) || s.E > 2147483647LL - 4096 || s.B > 65535 || s.H > 32768) return L1ATTN_ERR_RANGE;
	bool aligned = true;
	for (int i = 0; i < n_ptrs; i++) aligned = aligned && ((((uintptr_t)ptrs[i]) & 15) == 0);
	c.vec = (s.W % 4 == 0 && s.Wv % 4 == 0 && aligned) ? 4 : 1;
	(void)elt;
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
	if (l1_cdiv(items, 4) > 2147483647LL) return L1ATTN_ERR_RANGE;
	c.grid = dim3((unsigned)l1_cdiv(items, 4), (unsigned)s.B, 1);
	c.block = dim3(256);
	return L1ATTN_OK;
}

#define DISPATCH_VM(cfg, CALL)                      \
	do {                                            \
		if ((cfg).vec == 4 && (cfg).mc == 1) { CALL(4, 1); } \
		else if ((cfg).vec == 4) { CALL(4, 4); }    \
		else if ((cfg).mc == 1) { CALL(1, 1); }     \
		else { CALL(1, 4); }                        \
	} while (0)

template <typename T>
int sparse_fwd_impl(const T* v, const T* vbk, const T* q, const T* k, const void* plan, T* vo, T* P, Shape s,
                    int use_softmax, bool bidi, hipStream_t st)
{
	if (s.B * s.T * s.H == 0) return L1ATTN_OK;
	if (!v || !q || !k || !plan || !vo || (s.E > 0 && !P) || (bidi && !vbk)) return L1ATTN_ERR_ARG;
	const void* ptrs[] = {v, vbk, q, k, vo};
	Cfg c;
	int rc = make_cfg(s, sizeof(T), ptrs, 5, c);
	if (rc) return rc;
	const PlanLayout L = plan_layout(s.E, s.T);
	const int* words = (const int*)plan;
	const T scale = (T)(-1.0 / sqrt((double)s.W));
#define CALL(V, M)                                                                                               \
	hipLaunchKernelGGL((sparse_fwd_dst<T, V, M>), c.grid, c.block, 0, st, v, q, k, words + L.dst_ptr,            \
	                   words + L.csr_src, vo, P, c.g, use_softmax, scale)
	DISPATCH_VM(c, CALL);
#undef CALL
	L1_LAUNCH_CHECK();
	if (bidi) {
#define CALL(V, M)                                                                                               \
	hipLaunchKernelGGL((sparse_fwd_src<T, V, M>), c.grid, c.block, 0, st, vbk, words + L.src_ptr,                \
	                   words + L.csc_dst, words + L.csc_slot, (const T*)P, vo, c.g)
		DISPATCH_VM(c, CALL);
#undef CALL
		L1_LAUNCH_CHECK();
	}
	return L1ATTN_OK;
}

template <typename T>
int sparse_bwd_impl(const T* dvo, const T* v, const T* vbk, const T* q, const T* k, const void* plan, const T* P,
                    T* dv, T* dvb, T* dq, T* dk, T* DA, Shape s, int use_softmax, bool bidi, hipStream_t st)
{
	if (s.B * s.T * s.H == 0) return L1ATTN_OK;
	if (!dvo || !v || !q || !k || !plan || !dv || !dq || !dk || (s.E > 0 && (!P || !DA)) || (bidi && (!vbk || !dvb)))
		return L1ATTN_ERR_ARG;
	const void* ptrs[] = {dvo, v, vbk, q, k, dv, dvb, dq, dk};
	Cfg c;
	int rc = make_cfg(s, sizeof(T), ptrs, 9, c);
	if (rc) return rc;
	const PlanLayout L = plan_layout(s.E, s.T);
	const int* words = (const int*)plan;
	const T scale = (T)(-1.0 / sqrt((double)s.W));
	if (bidi) {
#define CALL(V, M)                                                                                               \
	hipLaunchKernelGGL((sparse_bwd_dst<T, V, M, true>), c.grid, c.block, 0, st, dvo, v, vbk, q, k,               \
	                   words + L.dst_ptr, words + L.csr_src, P, DA, dq, dvb, c.g, use_softmax, scale)
		DISPATCH_VM(c, CALL);
#undef CALL
	} else {
#define CALL(V, M)                                                                                               \
	hipLaunchKernelGGL((sparse_bwd_dst<T, V, M, false>), c.grid, c.block, 0, st, dvo, v, vbk, q, k,              \
	                   words + L.dst_ptr, words + L.csr_src, P, DA, dq, dvb, c.g, use_softmax, scale)
		DISPATCH_VM(c, CALL);
#undef CALL
	}
	L1_LAUNCH_CHECK();
#define CALL(V, M)                                                                                               \
	hipLaunchKernelGGL((sparse_bwd_src<T, V, M>), c.grid, c.block, 0, st, dvo, q, k, words + L.src_ptr,          \
	                   words + L.csc_dst, words + L.csc_slot, P, (const T*)DA, dv, dk, c.g, scale)
	DISPATCH_VM(c, CALL);
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
		return sparse_fwd_impl<TYPE>(v, nullptr, q, k, plan, vo, P, Shape{B, T, H, W, Wv, E}, use_softmax, false,   \
		                             (hipStream_t)stream);                                                          \
	}                                                                                                               \
	int l1attn_sparse_bwd_##SFX(const TYPE* dvo, const TYPE* v, const TYPE* q, const TYPE* k, const void* plan,     \
	                            const TYPE* P, TYPE* dv, TYPE* dq, TYPE* dk, TYPE* DA, int64_t B, int64_t T,        \
	                            int64_t H, int64_t W, int64_t Wv, int64_t E, int use_softmax, void* stream)         \
	{                                                                                                               \
		return sparse_bwd_impl<TYPE>(dvo, v, nullptr, q, k, plan, P, dv, nullptr, dq, dk, DA,                       \
		                             Shape{B, T, H, W, Wv, E}, use_softmax, false, (hipStream_t)stream);            \
	}                                                                                                               \
	int l1attn_sparse_bidi_fwd_##SFX(const TYPE* vf, const TYPE* vb, const TYPE* q, const TYPE* k,                  \
	                                 const void* plan, TYPE* vo, TYPE* P, int64_t B, int64_t T, int64_t H,          \
	                                 int64_t W, int64_t Wv, int64_t E, int use_softmax, void* stream)               \
	{                                                                                                               \
		return sparse_fwd_impl<TYPE>(vf, vb, q, k, plan, vo, P, Shape{B, T, H, W, Wv, E}, use_softmax, true,        \
		                             (hipStream_t)stream);                                                          \
	}                                                                                                               \
	int l1attn_sparse_bidi_bwd_##SFX(const TYPE* dvo, const TYPE* vf, const TYPE* vb, const TYPE* q,                \
	                                 const TYPE* k, const void* plan, const TYPE* P, TYPE* dvf, TYPE* dvb,          \
	                                 TYPE* dq, TYPE* dk, TYPE* DA, int64_t B, int64_t T, int64_t H, int64_t W,      \
	                                 int64_t Wv, int64_t E, int use_softmax, void* stream)                          \
	{                                                                                                               \
		return sparse_bwd_impl<TYPE>(dvo, vf, vb, q, k, plan, P, dvf, dvb, dq, dk, DA, Shape{B, T, H, W, Wv, E},    \
		                             use_softmax, true, (hipStream_t)stream);                                       \
	}

L1_SPARSE_ENTRY(f32, float)
L1_SPARSE_ENTRY(f64, double)

}  // extern "C"
