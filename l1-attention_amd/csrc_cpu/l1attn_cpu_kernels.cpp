// Host-CPU kernels of the L1 attention operators.  This file is compiled twice into one library, once for
// the baseline x86-64 instruction set and once with AVX2 + FMA (L1CPU_NS names the copy); l1attn_cpu.cpp picks
// one at load time from what the processor reports.  Everything here is a template over the element type.
//
// Parallel decomposition, the same idea as on the GPU: every output row has exactly one owner.  The dense
// backward makes one sweep with the dst rows as owners (dq) and one with the src rows as owners (dk); the
// sparse operators walk dst-sorted segments for what is indexed by dst (softmax, vo, dq, dvb) and src-sorted
// segments for what is indexed by src (dv/dvf, dk, the reverse flow of the bidirectional forward).  No atomics,
// no per-thread partial sums: results do not depend on the number of threads.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include <omp.h>

#include "l1attn_cpu_table.h"

namespace L1CPU_NS {

constexpr int SB = 4;   // src rows sharing one pass over the dst rows in the dense forward
constexpr int RB = 8;   // rows per owner block in the dense backward

template <typename F>
static inline F l1_row(const F* __restrict__ a, const F* __restrict__ b, int64_t W)
{
	F acc = 0;
#pragma omp simd reduction(+ : acc)
	for (int64_t w = 0; w < W; w++) acc += std::fabs(a[w] - b[w]);
	return acc;
}

template <typename F>
static inline F dot_row(const F* __restrict__ a, const F* __restrict__ b, int64_t W)
{
	F acc = 0;
#pragma omp simd reduction(+ : acc)
	for (int64_t w = 0; w < W; w++) acc += a[w] * b[w];
	return acc;
}

// y[w] += g * sign(a[w] - b[w]), sign(0) = 0
template <typename F>
static inline void sign_axpy(F* __restrict__ y, const F* __restrict__ a, const F* __restrict__ b, F g, int64_t W)
{
#pragma omp simd
	for (int64_t w = 0; w < W; w++) {
		const F d = a[w] - b[w];
		y[w] += g * (F)((d > 0) - (d < 0));
	}
}

template <typename F>
static inline void axpy(F* __restrict__ y, const F* __restrict__ x, F g, int64_t W)
{
#pragma omp simd
	for (int64_t w = 0; w < W; w++) y[w] += g * x[w];
}

// ------------------------------------------------------------------------------------------ dense

template <typename F>
void dense_fwd(const F* q, const F* k, F* attn, int64_t B, int64_t T, int64_t H, int64_t W, int nt)
{
	const F scale = (F)(-1.0 / std::sqrt((double)W));
	const int64_t nsb = (T + SB - 1) / SB, row = H * W;
#pragma omp parallel for collapse(2) schedule(static) num_threads(nt)
	for (int64_t b = 0; b < B; b++)
		for (int64_t sb = 0; sb < nsb; sb++) {
			const int64_t s0 = sb * SB, ns = (T - s0 < SB) ? T - s0 : SB;
			for (int64_t t = 0; t < T; t++) {
				const F* qt = q + (b * T + t) * row;
				for (int64_t j = 0; j < ns; j++) {
					const F* ks = k + (b * T + s0 + j) * row;
					F* out = attn + ((b * T + s0 + j) * T + t) * H;
					for (int64_t h = 0; h < H; h++) out[h] = l1_row(qt + h * W, ks + h * W, W) * scale;
				}
			}
		}
}

template <typename F>
void dense_bwd(const F* dA, const F* q, const F* k, F* dq, F* dk, int64_t B, int64_t T, int64_t H, int64_t W, int nt)
{
	const F scale = (F)(-1.0 / std::sqrt((double)W));
	const int64_t nrb = (T + RB - 1) / RB, row = H * W;
	// two sweeps over (owner block, all rows of the other kind): 0 = dst rows own dq, 1 = src rows own dk
#pragma omp parallel for collapse(3) schedule(static) num_threads(nt)
	for (int sweep = 0; sweep < 2; sweep++)
		for (int64_t b = 0; b < B; b++)
			for (int64_t rb = 0; rb < nrb; rb++) {
				const int64_t r0 = rb * RB, nr = (T - r0 < RB) ? T - r0 : RB;
				F* own = (sweep == 0 ? dq : dk) + (b * T + r0) * row;
				std::memset(own, 0, sizeof(F) * nr * row);
				for (int64_t o = 0; o < T; o++) {  // the other index: src for sweep 0, dst for sweep 1
					for (int64_t j = 0; j < nr; j++) {
						const int64_t t = sweep == 0 ? r0 + j : o, s = sweep == 0 ? o : r0 + j;
						const F* g = dA + ((b * T + s) * T + t) * H;
						const F* qt = q + (b * T + t) * row;
						const F* ks = k + (b * T + s) * row;
						F* y = own + j * row;
						const F sc = sweep == 0 ? scale : -scale;
						for (int64_t h = 0; h < H; h++) sign_axpy(y + h * W, qt + h * W, ks + h * W, sc * g[h], W);
					}
				}
			}
}

// ------------------------------------------------------------------------------------------ fused
// Dense logits, softmax over src with the no-op zero logit, value sum, without the [B,T,T,H] tensor:
//   vo[b,t,h,:] = sum_s e^{a[s,t]} v[b,s,h,:] / (1 + sum_s e^{a[s,t]}),  lse = log(1 + sum_s e^{a[s,t]}).
// Every logit is <= 0 and the no-op logit is 0, so no running maximum is needed.

template <typename F>
void fused_fwd(const F* q, const F* k, const F* v, F* vo, F* lse, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv,
               int nt)
{
	const F scale = (F)(-1.0 / std::sqrt((double)W));
	const int64_t row = H * W, vrow = H * Wv;
#pragma omp parallel for collapse(2) schedule(static) num_threads(nt)
	for (int64_t b = 0; b < B; b++)
		for (int64_t t = 0; t < T; t++) {
			F* out = vo + (b * T + t) * vrow;
			std::memset(out, 0, sizeof(F) * vrow);
			for (int64_t h = 0; h < H; h++) {
				const F* qt = q + (b * T + t) * row + h * W;
				F den = 0;
				for (int64_t s = 0; s < T; s++) {
					const F p = std::exp(l1_row(qt, k + (b * T + s) * row + h * W, W) * scale);
					den += p;
					axpy(out + h * Wv, v + (b * T + s) * vrow + h * Wv, p, Wv);
				}
				const F inv = (F)1 / ((F)1 + den);
				for (int64_t w = 0; w < Wv; w++) out[h * Wv + w] *= inv;
				if (lse) lse[(b * T + t) * H + h] = std::log1p(den);
			}
		}
}

// Backward without any [T,T] tensor: with p = e^{a - lse[t]}, dp = v[s].dvo[t], S[t] = vo[t].dvo[t], the gradient of
// a logit is da = p (dp - S[t]).  One sweep with the dst rows as owners (dq), one with the src rows as owners
// (dk, dv); each recomputes the logits it needs.
template <typename F>
void fused_bwd(const F* dvo, const F* q, const F* k, const F* v, const F* vo, const F* lse, F* dq, F* dk, F* dv, int64_t B,
               int64_t T, int64_t H, int64_t W, int64_t Wv, int nt)
{
	const F scale = (F)(-1.0 / std::sqrt((double)W));
	const int64_t row = H * W, vrow = H * Wv;
	std::vector<F> Sv((size_t)B * T * H);
#pragma omp parallel for schedule(static) num_threads(nt)
	for (int64_t i = 0; i < B * T * H; i++) Sv[i] = dot_row(vo + i * Wv, dvo + i * Wv, Wv);
#pragma omp parallel for collapse(3) schedule(static) num_threads(nt)
	for (int sweep = 0; sweep < 2; sweep++)
		for (int64_t b = 0; b < B; b++)
			for (int64_t r = 0; r < T; r++) {
				F* gq = sweep == 0 ? dq + (b * T + r) * row : nullptr;
				F* gk = sweep == 1 ? dk + (b * T + r) * row : nullptr;
				F* gv = sweep == 1 ? dv + (b * T + r) * vrow : nullptr;
				if (sweep == 0) std::memset(gq, 0, sizeof(F) * row);
				else { std::memset(gk, 0, sizeof(F) * row); std::memset(gv, 0, sizeof(F) * vrow); }
				for (int64_t o = 0; o < T; o++) {
					const int64_t t = sweep == 0 ? r : o, s = sweep == 0 ? o : r;
					for (int64_t h = 0; h < H; h++) {
						const F* qt = q + (b * T + t) * row + h * W;
						const F* ks = k + (b * T + s) * row + h * W;
						const F* gt = dvo + (b * T + t) * vrow + h * Wv;
						const F p = std::exp(l1_row(qt, ks, W) * scale - lse[(b * T + t) * H + h]);
						const F da = p * (dot_row(v + (b * T + s) * vrow + h * Wv, gt, Wv) - Sv[(b * T + t) * H + h]);
						if (sweep == 0) sign_axpy(gq + h * W, qt, ks, scale * da, W);
						else {
							sign_axpy(gk + h * W, qt, ks, -scale * da, W);
							axpy(gv + h * Wv, gt, p, Wv);
						}
					}
				}
			}
}

// ----------------------------------------------------------------------------------- edge lists

// Stable counting sort of the edges by column `col` of coo: ptr[T+1], order[E] (edge ids, original order
// inside a segment).
static void segments(const int32_t* coo, int64_t stride, int64_t E, int64_t T, int col, std::vector<int64_t>& ptr,
                     std::vector<int32_t>& order)
{
	ptr.assign(T + 1, 0);
	order.resize(E);
	for (int64_t c = 0; c < E; c++) ptr[coo[c * stride + col] + 1]++;
	for (int64_t t = 0; t < T; t++) ptr[t + 1] += ptr[t];
	std::vector<int64_t> fill(ptr.begin(), ptr.end() - 1);
	for (int64_t c = 0; c < E; c++) order[fill[coo[c * stride + col]]++] = (int32_t)c;
}

template <typename F, bool BIDI>
void sparse_fwd(const F* v, const F* vb, const F* q, const F* k, const int32_t* coo, int64_t cs, F* vo, F* attn, int64_t B,
                int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t M, bool use_softmax, bool attn_zeroed, int nt)
{
	const F scale = (F)(-1.0 / std::sqrt((double)W));
	std::vector<int64_t> dptr, sptr;
	std::vector<int32_t> dord, sord;
	segments(coo, cs, E, T, 0, dptr, dord);
	if (BIDI) segments(coo, cs, E, T, 1, sptr, sord);
	const int64_t row = H * W, vrow = H * Wv;
#pragma omp parallel for collapse(2) schedule(dynamic, 16) num_threads(nt)
	for (int64_t b = 0; b < B; b++)
		for (int64_t d = 0; d < T; d++) {
			F* slots = attn + (b * T + d) * M * H;
			// the padded tensor is mostly empty slots on skewed graphs: a caller that hands over zeroed memory
			// (calloc: pages that were never touched) saves touching all of it
			if (!attn_zeroed && M > 0) std::memset(slots, 0, sizeof(F) * M * H);
			F* out = vo + (b * T + d) * vrow;
			std::memset(out, 0, sizeof(F) * vrow);
			const F* qd = q + (b * T + d) * row;
			for (int64_t h = 0; h < H; h++) {
				F den = 1;  // the no-op logit of the softmax: exp(0)
				for (int64_t e = dptr[d]; e < dptr[d + 1]; e++) {
					const int32_t* c = coo + (int64_t)dord[e] * cs;
					const F ex = std::exp(l1_row(qd + h * W, k + (b * T + c[1]) * row + h * W, W) * scale);
					slots[(int64_t)c[2] * H + h] = ex;
					den += ex;
				}
				for (int64_t e = dptr[d]; e < dptr[d + 1]; e++) {
					const int32_t* c = coo + (int64_t)dord[e] * cs;
					F& p = slots[(int64_t)c[2] * H + h];
					if (use_softmax) p = p / den;
					axpy(out + h * Wv, v + (b * T + c[1]) * vrow + h * Wv, p, Wv);
				}
			}
		}
	if (!BIDI) return;
	// reverse flow: vo[b,src] += p * vb[b,dst], the src row is the owner
#pragma omp parallel for collapse(2) schedule(dynamic, 16) num_threads(nt)
	for (int64_t b = 0; b < B; b++)
		for (int64_t s = 0; s < T; s++) {
			F* out = vo + (b * T + s) * vrow;
			for (int64_t e = sptr[s]; e < sptr[s + 1]; e++) {
				const int32_t* c = coo + (int64_t)sord[e] * cs;
				const F* slots = attn + ((b * T + c[0]) * M + c[2]) * H;
				const F* x = vb + (b * T + c[0]) * vrow;
				for (int64_t h = 0; h < H; h++) axpy(out + h * Wv, x + h * Wv, slots[h], Wv);
			}
		}
}

template <typename F, bool BIDI>
void sparse_bwd(const F* dvo, const F* v, const F* vb, const F* q, const F* k, const int32_t* coo, int64_t cs, const F* attn,
                F* dv, F* dvb, F* dq, F* dk, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t M,
                bool use_softmax, int nt)
{
	const F scale = (F)(-1.0 / std::sqrt((double)W));
	std::vector<int64_t> dptr, sptr;
	std::vector<int32_t> dord, sord;
	segments(coo, cs, E, T, 0, dptr, dord);
	segments(coo, cs, E, T, 1, sptr, sord);
	const int64_t row = H * W, vrow = H * Wv;
	std::vector<F> da((size_t)B * E * H);  // gradient of the logit of every (batch, edge, head)
	// dst rows own: the softmax Jacobian (closed form over the dst's edges), dq, dvb
#pragma omp parallel for collapse(2) schedule(dynamic, 16) num_threads(nt)
	for (int64_t b = 0; b < B; b++)
		for (int64_t d = 0; d < T; d++) {
			F* gq = dq + (b * T + d) * row;
			std::memset(gq, 0, sizeof(F) * row);
			F* gvb = BIDI ? dvb + (b * T + d) * vrow : nullptr;
			if (BIDI) std::memset(gvb, 0, sizeof(F) * vrow);
			const F* qd = q + (b * T + d) * row;
			const F* gd = dvo + (b * T + d) * vrow;
			for (int64_t h = 0; h < H; h++) {
				F S = 0;  // sum over the dst's edges of p * dp
				for (int64_t e = dptr[d]; e < dptr[d + 1]; e++) {
					const int32_t* c = coo + (int64_t)dord[e] * cs;
					const F p = attn[((b * T + d) * M + c[2]) * H + h];
					F dp = dot_row(v + (b * T + c[1]) * vrow + h * Wv, gd + h * Wv, Wv);
					if (BIDI) {
						const F* gs = dvo + (b * T + c[1]) * vrow + h * Wv;
						dp += dot_row(vb + (b * T + d) * vrow + h * Wv, gs, Wv);
						axpy(gvb + h * Wv, gs, p, Wv);
					}
					da[((size_t)b * E + dord[e]) * H + h] = dp;
					S += p * dp;
				}
				if (!use_softmax) S = 0;
				for (int64_t e = dptr[d]; e < dptr[d + 1]; e++) {
					const int32_t* c = coo + (int64_t)dord[e] * cs;
					const F p = attn[((b * T + d) * M + c[2]) * H + h];
					F& g = da[((size_t)b * E + dord[e]) * H + h];
					g = p * (g - S);
					sign_axpy(gq + h * W, qd + h * W, k + (b * T + c[1]) * row + h * W, scale * g, W);
				}
			}
		}
	// src rows own: dv (dvf) and dk
#pragma omp parallel for collapse(2) schedule(dynamic, 16) num_threads(nt)
	for (int64_t b = 0; b < B; b++)
		for (int64_t s = 0; s < T; s++) {
			F* gv = dv + (b * T + s) * vrow;
			F* gk = dk + (b * T + s) * row;
			std::memset(gv, 0, sizeof(F) * vrow);
			std::memset(gk, 0, sizeof(F) * row);
			const F* ks = k + (b * T + s) * row;
			for (int64_t e = sptr[s]; e < sptr[s + 1]; e++) {
				const int32_t* c = coo + (int64_t)sord[e] * cs;
				const F* slots = attn + ((b * T + c[0]) * M + c[2]) * H;
				const F* gd = dvo + (b * T + c[0]) * vrow;
				const F* qd = q + (b * T + c[0]) * row;
				const F* g = &da[((size_t)b * E + sord[e]) * H];
				for (int64_t h = 0; h < H; h++) {
					axpy(gv + h * Wv, gd + h * Wv, slots[h], Wv);
					sign_axpy(gk + h * W, qd + h * W, ks + h * W, -scale * g[h], W);
				}
			}
		}
}

}  // namespace L1CPU_NS

// One table per compiled copy.
#define L1CPU_CAT2(a, b) a##b
#define L1CPU_CAT(a, b) L1CPU_CAT2(a, b)
extern const L1CpuTable L1CPU_CAT(l1cpu_table_, L1CPU_NS);
const L1CpuTable L1CPU_CAT(l1cpu_table_, L1CPU_NS) = {
    L1CPU_NS::dense_fwd<float>,         L1CPU_NS::dense_fwd<double>,
    L1CPU_NS::dense_bwd<float>,         L1CPU_NS::dense_bwd<double>,
    L1CPU_NS::sparse_fwd<float, false>, L1CPU_NS::sparse_fwd<double, false>,
    L1CPU_NS::sparse_fwd<float, true>,  L1CPU_NS::sparse_fwd<double, true>,
    L1CPU_NS::sparse_bwd<float, false>, L1CPU_NS::sparse_bwd<double, false>,
    L1CPU_NS::sparse_bwd<float, true>,  L1CPU_NS::sparse_bwd<double, true>,
    L1CPU_NS::fused_fwd<float>,         L1CPU_NS::fused_fwd<double>,
    L1CPU_NS::fused_bwd<float>,         L1CPU_NS::fused_bwd<double>,
};
