// C ABI of libl1attn_cpu.so (include/l1attn_cpu.h): argument checks, expandCoo, and the choice between the two
// compiled copies of the kernels (baseline x86-64, AVX2 + FMA) from what the processor reports.
#include <cstdlib>
#include <unordered_map>
#include <vector>

#include <omp.h>

#include "../../include/l1attn_cpu.h"
#include "l1attn_cpu_table.h"

namespace {

int g_threads = 0;  // 0: the OpenMP default

int threads()
{
	return g_threads > 0 ? g_threads : omp_get_max_threads();
}

const L1CpuTable& table()
{
	static const L1CpuTable* t = [] {
		const char* force = std::getenv("L1ATTN_CPU_ISA");  // "generic" pins the baseline copy (tests compare the two)
		if (force && force[0] == 'g') return &l1cpu_table_l1cpu_generic;
		__builtin_cpu_init();
		return (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) ? &l1cpu_table_l1cpu_avx2
		                                                                        : &l1cpu_table_l1cpu_generic;
	}();
	return *t;
}

bool bad_dims(int64_t B, int64_t T, int64_t H, int64_t W)
{
	return B < 0 || T < 0 || H < 0 || W < 1;
}

// every edge must name tokens inside [0,T) and a slot inside [0,M)
int check_coo(const int32_t* coo, int64_t cs, int64_t E, int64_t T, int64_t M)
{
	if (E < 0 || cs < 3 || M < 0 || (E > 0 && !coo)) return L1ATTN_CPU_ERR_ARG;
	for (int64_t c = 0; c < E; c++) {
		const int32_t* r = coo + c * cs;
		if (r[0] < 0 || r[0] >= T || r[1] < 0 || r[1] >= T || r[2] < 0 || r[2] >= M) return L1ATTN_CPU_ERR_INDEX;
	}
	return 0;
}

template <typename I>
int expand(const I* co, int64_t stride, int64_t E, int32_t* coo, int32_t* mxlen)
{
	// rank of each row among the earlier rows with the same key; dense counters when the keys are small
	// non-negative numbers, a hash map otherwise (the reference's dict takes any integer)
	int64_t lo = 0, hi = 0;
	for (int64_t i = 0; i < E; i++)
		for (int c = 0; c < 2; c++) {
			const int64_t x = (int64_t)co[i * stride + c];
			if (x < INT32_MIN || x > INT32_MAX) return L1ATTN_CPU_ERR_INDEX;
			lo = x < lo ? x : lo;
			hi = x > hi ? x : hi;
		}
	int32_t mx[2] = {0, 0};
	if (lo >= 0 && hi <= 4 * E + 4096) {
		std::vector<int32_t> cnt[2] = {std::vector<int32_t>(hi + 1, 0), std::vector<int32_t>(hi + 1, 0)};
		for (int64_t i = 0; i < E; i++)
			for (int c = 0; c < 2; c++) {
				const int32_t x = (int32_t)co[i * stride + c];
				const int32_t r = cnt[c][x]++;
				coo[i * 4 + c] = x;
				coo[i * 4 + 2 + c] = r;
				mx[c] = r > mx[c] ? r : mx[c];
			}
	} else {
		std::unordered_map<int32_t, int32_t> cnt[2];
		for (int64_t i = 0; i < E; i++)
			for (int c = 0; c < 2; c++) {
				const int32_t x = (int32_t)co[i * stride + c];
				const int32_t r = cnt[c][x]++;
				coo[i * 4 + c] = x;
				coo[i * 4 + 2 + c] = r;
				mx[c] = r > mx[c] ? r : mx[c];
			}
	}
	mxlen[0] = mx[0] + 1;
	mxlen[1] = mx[1] + 1;
	return 0;
}

}  // namespace

extern "C" {

int l1attn_cpu_version(void)
{
	return 100;
}

int l1attn_cpu_set_threads(int n)
{
	const int old = g_threads;
	g_threads = n > 0 ? n : 0;
	return old;
}

#define L1CPU_DENSE(SFX, F)                                                                                                  \
	int l1attn_cpu_dense_fwd_##SFX(const F* q, const F* k, F* attn, int64_t B, int64_t T, int64_t H, int64_t W)              \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W)) return L1ATTN_CPU_ERR_ARG;                                                                 \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!q || !k || !attn) return L1ATTN_CPU_ERR_ARG;                                                                    \
		table().dense_fwd_##SFX(q, k, attn, B, T, H, W, threads());                                                          \
		return 0;                                                                                                            \
	}                                                                                                                        \
	int l1attn_cpu_dense_bwd_##SFX(const F* d_attn, const F* q, const F* k, F* dq, F* dk, int64_t B, int64_t T, int64_t H,   \
	                               int64_t W)                                                                                \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W)) return L1ATTN_CPU_ERR_ARG;                                                                 \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!d_attn || !q || !k || !dq || !dk) return L1ATTN_CPU_ERR_ARG;                                                    \
		table().dense_bwd_##SFX(d_attn, q, k, dq, dk, B, T, H, W, threads());                                                \
		return 0;                                                                                                            \
	}
L1CPU_DENSE(f32, float)
L1CPU_DENSE(f64, double)

int l1attn_cpu_expand_coo(const void* co, int co_bits, int64_t co_stride, int64_t E, int32_t* coo, int32_t* mxlen)
{
	if (E < 0 || co_stride < 2 || !mxlen || (co_bits != 32 && co_bits != 64)) return L1ATTN_CPU_ERR_ARG;
	if (E > 0 && (!co || !coo)) return L1ATTN_CPU_ERR_ARG;
	return co_bits == 32 ? expand((const int32_t*)co, co_stride, E, coo, mxlen)
	                     : expand((const int64_t*)co, co_stride, E, coo, mxlen);
}

#define L1CPU_SPARSE(SFX, F)                                                                                                 \
	int l1attn_cpu_sparse_fwd_##SFX(const F* v, const F* q, const F* k, const int32_t* coo, int64_t cs, F* vo, F* attn,      \
	                                int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t M, int sm,    \
	                                int attn_zeroed)                                                                         \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W) || Wv < 1) return L1ATTN_CPU_ERR_ARG;                                                       \
		if (int rc = check_coo(coo, cs, E, T, M)) return rc;                                                                 \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!v || !q || !k || !vo || (M > 0 && !attn)) return L1ATTN_CPU_ERR_ARG;                                            \
		table().sparse_fwd_##SFX(v, nullptr, q, k, coo, cs, vo, attn, B, T, H, W, Wv, E, M, sm != 0, attn_zeroed != 0,       \
		                         threads());                                                                                 \
		return 0;                                                                                                            \
	}                                                                                                                        \
	int l1attn_cpu_sparse_bidi_fwd_##SFX(const F* vf, const F* vb, const F* q, const F* k, const int32_t* coo, int64_t cs,   \
	                                     F* vo, F* attn, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,  \
	                                     int64_t M, int sm, int attn_zeroed)                                                 \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W) || Wv < 1) return L1ATTN_CPU_ERR_ARG;                                                       \
		if (int rc = check_coo(coo, cs, E, T, M)) return rc;                                                                 \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!vf || !vb || !q || !k || !vo || (M > 0 && !attn)) return L1ATTN_CPU_ERR_ARG;                                    \
		table().bidi_fwd_##SFX(vf, vb, q, k, coo, cs, vo, attn, B, T, H, W, Wv, E, M, sm != 0, attn_zeroed != 0,             \
		                       threads());                                                                                   \
		return 0;                                                                                                            \
	}                                                                                                                        \
	int l1attn_cpu_sparse_bwd_##SFX(const F* dvo, const F* v, const F* q, const F* k, const int32_t* coo, int64_t cs,        \
	                                const F* attn, F* dv, F* dq, F* dk, int64_t B, int64_t T, int64_t H, int64_t W,          \
	                                int64_t Wv, int64_t E, int64_t M, int sm)                                                \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W) || Wv < 1) return L1ATTN_CPU_ERR_ARG;                                                       \
		if (int rc = check_coo(coo, cs, E, T, M)) return rc;                                                                 \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!dvo || !v || !q || !k || !dv || !dq || !dk || (E > 0 && !attn)) return L1ATTN_CPU_ERR_ARG;                      \
		table().sparse_bwd_##SFX(dvo, v, nullptr, q, k, coo, cs, attn, dv, nullptr, dq, dk, B, T, H, W, Wv, E, M, sm != 0,   \
		                         threads());                                                                                 \
		return 0;                                                                                                            \
	}                                                                                                                        \
	int l1attn_cpu_sparse_bidi_bwd_##SFX(const F* dvo, const F* vf, const F* vb, const F* q, const F* k, const int32_t* coo, \
	                                     int64_t cs, const F* attn, F* dvf, F* dvb, F* dq, F* dk, int64_t B, int64_t T,      \
	                                     int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t M, int sm)                     \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W) || Wv < 1) return L1ATTN_CPU_ERR_ARG;                                                       \
		if (int rc = check_coo(coo, cs, E, T, M)) return rc;                                                                 \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!dvo || !vf || !vb || !q || !k || !dvf || !dvb || !dq || !dk || (E > 0 && !attn)) return L1ATTN_CPU_ERR_ARG;     \
		table().bidi_bwd_##SFX(dvo, vf, vb, q, k, coo, cs, attn, dvf, dvb, dq, dk, B, T, H, W, Wv, E, M, sm != 0,            \
		                       threads());                                                                                   \
		return 0;                                                                                                            \
	}
L1CPU_SPARSE(f32, float)
L1CPU_SPARSE(f64, double)

#define L1CPU_FUSED(SFX, F)                                                                                                  \
	int l1attn_cpu_fused_fwd_##SFX(const F* q, const F* k, const F* v, F* vo, F* lse, int64_t B, int64_t T, int64_t H,       \
	                               int64_t W, int64_t Wv)                                                                    \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W) || Wv < 1) return L1ATTN_CPU_ERR_ARG;                                                       \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!q || !k || !v || !vo) return L1ATTN_CPU_ERR_ARG;                                                                \
		table().fused_fwd_##SFX(q, k, v, vo, lse, B, T, H, W, Wv, threads());                                                \
		return 0;                                                                                                            \
	}                                                                                                                        \
	int l1attn_cpu_fused_bwd_##SFX(const F* dvo, const F* q, const F* k, const F* v, const F* vo, const F* lse, F* dq,       \
	                               F* dk, F* dv, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv)                     \
	{                                                                                                                        \
		if (bad_dims(B, T, H, W) || Wv < 1) return L1ATTN_CPU_ERR_ARG;                                                       \
		if (B * T * H == 0) return 0;                                                                                        \
		if (!dvo || !q || !k || !v || !vo || !lse || !dq || !dk || !dv) return L1ATTN_CPU_ERR_ARG;                           \
		table().fused_bwd_##SFX(dvo, q, k, v, vo, lse, dq, dk, dv, B, T, H, W, Wv, threads());                               \
		return 0;                                                                                                            \
	}
L1CPU_FUSED(f32, float)
L1CPU_FUSED(f64, double)

}  // extern "C"
