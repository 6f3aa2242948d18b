// TEST INFRASTRUCTURE: runs the sparse / bidirectional forward entry points of csrc/sparse.hip, compiled for the
// host with the stand-in header next to this file (GPU threads are OS threads, cross-lane reads and fences are
// barriers among a wave's threads), for float32, float64, float16 and bfloat16 rows.  Needs a host compiler with
// _Float16 and __bf16 (ROCm's clang++).
//   run_sparse <in> <out>
// in : int64 B,T,H,W,Wv,E,use_softmax,bidi,type(0 f32,1 f64,2 f16,3 bf16),n_long_dst,n_long_src; then int32 arrays
//      dst_ptr[T+2], src_ptr[T+2], csr_src[E], csr_row[E], csc_dst[E], csc_slot[E], long_dst[n_long_dst],
//      long_src[n_long_src]; then float32 vf, vb [B,T,H,Wv], q, k [B,T,H,W]
// out: float64 vo [B,T,H,Wv], float64 P [B,E,H]
// Row buffers are allocated at their exact sizes in the storage type, so AddressSanitizer reports any access
// outside them.
#define EMU_DYNAMIC_LDS_ONLY
#include "../../l1-attention_amd/csrc/sparse.hip"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

namespace { alignas(16) unsigned char smem_raw[65536]; }  // the kernels' dynamic LDS

template <typename S>
static S* to_storage(const std::vector<float>& x)
{
	S* p = (S*)aligned_alloc(16, (x.size() * sizeof(S) + 15) / 16 * 16 + 16);
	for (size_t i = 0; i < x.size(); i++) p[i] = (S)x[i];
	return p;
}

// the backward of the storage type S (weights and scratch of type PT) on dvo and the weights just written
#define L1_EMU_BWD(SFX, S, PT)                                                                                      \
	static int backward(const int64_t* d, const void* plan, const S* dvo, const S* vf, const S* vb, const S* q,     \
	                    const S* k, const PT* P, FILE* fo)                                                          \
	{                                                                                                               \
		const int64_t B = d[0], T = d[1], H = d[2], W = d[3], Wv = d[4], E = d[5];                                  \
		const size_t nv = (size_t)(B * T * H * Wv), nq = (size_t)(B * T * H * W), ne = (size_t)(B * E * H);         \
		S* dvf = (S*)aligned_alloc(16, (nv * sizeof(S) + 15) / 16 * 16 + 16);                                       \
		S* dvb = (S*)aligned_alloc(16, (nv * sizeof(S) + 15) / 16 * 16 + 16);                                       \
		S* dq = (S*)aligned_alloc(16, (nq * sizeof(S) + 15) / 16 * 16 + 16);                                        \
		S* dk = (S*)aligned_alloc(16, (nq * sizeof(S) + 15) / 16 * 16 + 16);                                        \
		PT* DA = (PT*)aligned_alloc(16, (ne * sizeof(PT) + 15) / 16 * 16 + 16);                                     \
		for (size_t i = 0; i < nv; i++) dvb[i] = (S)0.0f;                                                           \
		const int rc = d[7] ? l1attn_sparse_bidi_bwd_##SFX(dvo, vf, vb, q, k, plan, P, dvf, dvb, dq, dk, DA, B, T,  \
		                                                   H, W, Wv, E, (int)d[6], nullptr)                         \
		                    : l1attn_sparse_bwd_##SFX(dvo, vf, q, k, plan, P, dvf, dq, dk, DA, B, T, H, W, Wv, E,    \
		                                              (int)d[6], nullptr);                                          \
		if (rc) return 30 + (rc < 0 ? -rc : rc);                                                                    \
		for (size_t i = 0; i < nv; i++) { const double x = (double)dvf[i]; fwrite(&x, 8, 1, fo); }                  \
		for (size_t i = 0; i < nv; i++) { const double x = (double)dvb[i]; fwrite(&x, 8, 1, fo); }                  \
		for (size_t i = 0; i < nq; i++) { const double x = (double)dq[i]; fwrite(&x, 8, 1, fo); }                   \
		for (size_t i = 0; i < nq; i++) { const double x = (double)dk[i]; fwrite(&x, 8, 1, fo); }                   \
		free(dvf); free(dvb); free(dq); free(dk); free(DA);                                                         \
		return 0;                                                                                                   \
	}
L1_EMU_BWD(f32, float, float)
L1_EMU_BWD(f64, double, double)
L1_EMU_BWD(f16, f16_t, float)
L1_EMU_BWD(bf16, bf16_t, float)

template <typename S, typename P, typename F>
static int run(const int64_t* d, const void* plan, const std::vector<float>& vf, const std::vector<float>& vb,
               const std::vector<float>& q, const std::vector<float>& k, const std::vector<float>& dvo, FILE* fo,
               F call)
{
	const int64_t B = d[0], T = d[1], H = d[2], Wv = d[4], E = d[5];
	S *pvf = to_storage<S>(vf), *pvb = to_storage<S>(vb), *pq = to_storage<S>(q), *pk = to_storage<S>(k);
	S* vo = (S*)aligned_alloc(16, ((size_t)(B * T * H * Wv) * sizeof(S) + 15) / 16 * 16 + 16);
	P* pw = (P*)aligned_alloc(16, ((size_t)(B * E * H) * sizeof(P) + 15) / 16 * 16 + 16);
	const int rc = call(pvf, pvb, pq, pk, plan, vo, pw);
	if (rc) return 10 + (rc < 0 ? -rc : rc);
	for (int64_t i = 0; i < B * T * H * Wv; i++) { const double x = (double)vo[i]; fwrite(&x, 8, 1, fo); }
	for (int64_t i = 0; i < B * E * H; i++) { const double x = (double)pw[i]; fwrite(&x, 8, 1, fo); }
	{
		S* pdvo = to_storage<S>(dvo);
		const int rcb = backward(d, plan, pdvo, pvf, pvb, pq, pk, (const P*)pw, fo);
		free(pdvo);
		if (rcb) return rcb;
	}
	free(pvf); free(pvb); free(pq); free(pk); free(vo); free(pw);
	return 0;
}

int main(int argc, char** argv)
{
	if (argc != 3) return 2;
	FILE* fi = fopen(argv[1], "rb");
	FILE* fo = fopen(argv[2], "wb");
	if (!fi || !fo) return 2;
	int64_t d[11];
	if (fread(d, 8, 11, fi) != 11) return 3;
	const int64_t B = d[0], T = d[1], H = d[2], W = d[3], Wv = d[4], E = d[5];
	const int sm = (int)d[6], bidi = (int)d[7], type = (int)d[8];
	const PlanLayout L = plan_layout(E, T);
	std::vector<int32_t> plan(L.total_bytes / 4, 0);
	plan[PLAN_H_MAGIC] = PLAN_MAGIC; plan[PLAN_H_E] = (int)E; plan[PLAN_H_T] = (int)T; plan[PLAN_H_E_VALID] = (int)E;
	plan[PLAN_H_NLONG_DST] = (int)d[9]; plan[PLAN_H_NLONG_SRC] = (int)d[10];
	auto rd = [&](size_t off, size_t n) { return n == 0 || fread(plan.data() + off, 4, n, fi) == n; };
	if (!rd(L.dst_ptr, T + 2) || !rd(L.src_ptr, T + 2) || !rd(L.csr_src, E) || !rd(L.csr_row, E) || !rd(L.csc_dst, E) ||
	    !rd(L.csc_slot, E) || !rd(L.long_dst, d[9]) || !rd(L.long_src, d[10]))
		return 3;
	std::vector<float> vf(B * T * H * Wv), vb(B * T * H * Wv), q(B * T * H * W), k(B * T * H * W), dvo(B * T * H * Wv);
	for (auto* x : {&vf, &vb, &q, &k, &dvo})
		if (fread(x->data(), 4, x->size(), fi) != x->size()) return 3;
	int rc;
#define CALL(SFX, S, P)                                                                                              \
	rc = run<S, P>(d, plan.data(), vf, vb, q, k, dvo, fo,                                                               \
	               [&](const S* a, const S* b, const S* qq, const S* kk, const void* pl, S* vo, P* pw) {             \
		               return bidi ? l1attn_sparse_bidi_fwd_##SFX(a, b, qq, kk, pl, vo, pw, B, T, H, W, Wv, E, sm, nullptr) \
		                           : l1attn_sparse_fwd_##SFX(a, qq, kk, pl, vo, pw, B, T, H, W, Wv, E, sm, nullptr);  \
	               })
	if (type == 0) CALL(f32, float, float);
	else if (type == 1) CALL(f64, double, double);
	else if (type == 2) CALL(f16, f16_t, float);
	else CALL(bf16, bf16_t, float);
	fclose(fi);
	fclose(fo);
	return rc;
}
