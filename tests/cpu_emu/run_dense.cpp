// TEST INFRASTRUCTURE: runs the dense operator of csrc/dense.hip (forward, backward, fixed-point forward), compiled
// for the host with the stand-in headers next to this file, through the library's own entry points: the host
// logic that picks kernels, grids and workspace is the library's, unchanged.
//   run_dense <in> <out> <f32|f64|fixed> [wide <tt_rows> <rank 0|1> <group> [deep|deep2] | assume]
//   run_dense dims <B> <T> <H> <W>      launch geometry only, at any size: every launch the float32 forward,
//                                       backward and fixed-point forward would make is checked against the limits
//                                       of a HIP launch and printed (kernel, grid, block, LDS bytes); nothing runs
// in : int64 B,T,H,W then q,k [B,T,H,W] and dA [B,T,T,H] in the chosen type (fixed: float32)
// out: attn [B,T,T,H], dq, dk [B,T,H,W] (fixed: attn only), then int64[16] of l1attn_dense_bwd_plan_info and one
//      int64: the sign-domain flag the backward left in its workspace (-1 where the plan keeps none)
// Every buffer is malloc'ed at its exact size and every output starts as NaN, so AddressSanitizer reports an
// access outside a buffer and the caller sees an element that was never written.
//
// "wide ...": the backward runs the 512-thread tile kernels on a plan built here for the given tile height,
// rank form and tile grouping, whatever the sequence length; the library picks those kernels only from 1024
// tokens and a few thousand workgroups on, which is more than an emulation with one OS thread per GPU thread can
// walk in a test.  The launch sequence is the one of l1attn_dense_bwd_f32.
#include "hip/hip_runtime.h"

#include "emu_sload.h"

#include "emu_gfx950.h"

#include "../../l1-attention_amd/csrc/dense.hip"
#include "../../l1-attention_amd/csrc/fixed.hip"
#include <stdio.h>
#include <stdlib.h>
#include <vector>

// Column ranks by their definition, on the host (the sort kernels have their own runner):
// rk[s] = 2 #{k' < k[s]} - 1/2;  rq[t] = 2 #{k' < q[t]}, minus one unless some k' equals q[t].
bool l1_column_ranks_ok(int64_t B, int64_t T, int64_t H, int64_t W)
{
	return B >= 1 && T >= 1 && T <= L1_RANK_MAX_T && H * W >= 1 && B * H * W < ((int64_t)1 << 31);
}
int l1_launch_column_ranks(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                           int64_t W, hipStream_t)
{
	if (!l1_column_ranks_ok(B, T, H, W)) return L1ATTN_ERR_RANGE;
	if (emu::dry) return L1ATTN_OK;
	const int64_t HW = H * W;
	std::vector<float> col((size_t)T);
	for (int64_t b = 0; b < B; b++)
		for (int64_t c = 0; c < HW; c++) {
			const int64_t base = b * T * HW + c;
			for (int64_t t = 0; t < T; t++) col[(size_t)t] = k[base + t * HW];
			std::sort(col.begin(), col.end());
			for (int64_t t = 0; t < T; t++) {
				const float kv = k[base + t * HW], qv = q[base + t * HW];
				rk[base + t * HW] = (float)(2 * (std::lower_bound(col.begin(), col.end(), kv) - col.begin())) - 0.5f;
				const auto lb = std::lower_bound(col.begin(), col.end(), qv);
				const bool tie = lb != col.end() && *lb == qv;
				rq[base + t * HW] = (float)(2 * (lb - col.begin()) - (tie ? 0 : 1));
			}
		}
	return L1ATTN_OK;
}
int l1_launch_column_ranks_merge(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                                 int64_t W, hipStream_t st)
{
	return l1_launch_column_ranks(q, k, rq, rk, B, T, H, W, st);
}

// The plan of the 512-thread tile kernels for any sequence length: bwd_plan()'s arithmetic with the tile height,
// rank form and grouping given instead of chosen.  Returns fast = false where the kernels' own limits rule it out.
static BwdPlan wide_plan(int64_t B, int64_t T, int64_t H, int64_t W, int tt_rows, bool rank, int group, int deep)
{
	BwdPlan p{};
	const int64_t HW = H * W;
	if (!(B >= 1 && T >= 16 && HW >= 32 && (BWD_SJ * T + 128) * H < ((int64_t)1 << 29))) return p;
	p.fast = p.wide = true;
	p.threads = (int)std::min<int64_t>(512, l1_cdiv(HW, 64) * 64);
	p.n_cc = (int)l1_cdiv(HW, p.threads);
	int64_t hb = 1;
	for (int64_t cc = 0; cc < p.n_cc; cc++) {
		const int64_t c0 = cc * p.threads, c1 = std::min<int64_t>(HW, c0 + p.threads) - 1;
		hb = std::max<int64_t>(hb, c1 / W - c0 / W + 1);
	}
	p.rank = rank;
	if (rank && !(l1_column_ranks_ok(B, T, H, W) && BWD_SJ * hb * 16 <= p.threads && tt_rows <= 80)) p.fast = false;
	p.tt_rows = tt_rows;
	p.group = group;
	p.n_tt = (int)l1_cdiv(T, tt_rows);
	p.n_groups = (int)l1_cdiv(p.n_tt, group);
	p.lds_bytes = (size_t)BWD_SJ * hb * (tt_rows + 4) * sizeof(float);
	p.per = (int)l1_cdiv((int64_t)BWD_SJ * tt_rows * hb, p.threads);
	if (p.lds_bytes > 64 * 1024 || p.per > 8) p.fast = false;
	p.branch_free = tt_rows == 64 && T % 64 == 0 && T % BWD_SJ == 0 && HW % p.threads == 0 && p.threads % W == 0 &&
	                (int64_t)BWD_SJ * 64 * (p.threads / W) == (int64_t)4 * p.threads;
	if (group > 1 && !(p.branch_free && p.per <= (rank ? 4 : 8))) p.fast = false;  // grouped tiles: branch-free form only
	p.deep = deep;
	if (deep && !(p.branch_free && T % (2 * BWD_SJ) == 0)) p.fast = false;  // two-step prefetch: branch-free form only
	if (deep == 2) p.lds_bytes *= 2;
	p.partial_bytes = p.n_tt > 1 ? (size_t)p.n_groups * T * HW * sizeof(float) : 0;
	p.rank_bytes = rank ? ((size_t)2 * T * HW + (size_t)(p.n_tt + 1) * T * H) * sizeof(float) : 0;
	p.per_batch_bytes = p.partial_bytes + p.rank_bytes;
	return p;
}

static int run_wide(const BwdPlan& p, const float* d_attn, const float* q, const float* k, float* dq, float* dk, int64_t B,
                    int64_t T, int64_t H, int64_t W)
{
	hipStream_t st = nullptr;
	const float scale = (float)(-1.0 / sqrt((double)W));
	const int64_t HW = H * W;
	if (p.per_batch_bytes == 0) {
		launch_bwd_fast(p, dim3(1, p.n_cc, (unsigned)B), st, d_attn, q, k, dq, dk, nullptr, (int)T, (int)H, (int)W, scale);
		return 0;
	}
	const int64_t nb_max = std::min<int64_t>(B, 2);  // two batches per launch: the batch loop runs for B > 2
	void* workspace = malloc(p.per_batch_bytes * (size_t)nb_max);
	float* dkp = (float*)workspace;
	float* rq = dkp + (size_t)nb_max * (p.partial_bytes / sizeof(float));
	float* rk = rq + (size_t)nb_max * T * HW;
	float* csp = rk + (size_t)nb_max * T * HW;
	float* cs = csp + (size_t)p.n_tt * nb_max * T * H;
	for (int64_t b0 = 0; b0 < B; b0 += nb_max) {
		const int64_t nb = std::min<int64_t>(nb_max, B - b0);
		const float* qa = q + b0 * T * HW;
		const float* ka = k + b0 * T * HW;
		if (p.rank) {
			if (int rc = l1_launch_column_ranks(qa, ka, rq, rk, nb, T, H, W, st)) return rc;
			qa = rq;
			ka = rk;
		}
		launch_bwd_fast(p, dim3(p.n_groups, p.n_cc, (unsigned)nb), st, d_attn + b0 * T * T * H, qa, ka, dq + b0 * T * HW, dkp,
		                csp, (int)T, (int)H, (int)W, scale);
		const int64_t ne = nb * T * HW;
		if (p.rank) {
			const int64_t nc = nb * T * H;
			hipLaunchKernelGGL(dense_bwd_reduce_colsum, dim3((unsigned)l1_cdiv(nc, 256)), dim3(256), 0, st, csp, cs, nc, p.n_tt);
		}
		const bool vec = ((T * HW) % 4 == 0) && ((((uintptr_t)dkp) | ((uintptr_t)dk)) & 15) == 0 && (!p.rank || W % 4 == 0);
		const dim3 rgrid((unsigned)l1_cdiv(ne, vec ? 1024 : 256));
#define RUN_REDUCE3(VECV, RANKV, AHEADV)                                                                              \
	hipLaunchKernelGGL((dense_bwd_reduce_dk<VECV, RANKV, AHEADV>), rgrid, dim3(256), 0, st, dkp, dk + b0 * T * HW, ne,     \
	                   p.n_groups, cs, (int)HW, (int)W, (int)H, scale)
#define RUN_REDUCE(VECV, RANKV) RUN_REDUCE3(VECV, RANKV, false)
		if (vec && p.deep && p.rank) RUN_REDUCE3(true, true, true);
		else if (vec && p.deep) RUN_REDUCE3(true, false, true);
		else if (vec && p.rank) RUN_REDUCE(true, true);
		else if (vec) RUN_REDUCE(true, false);
		else if (p.rank) RUN_REDUCE(false, true);
		else RUN_REDUCE(false, false);
#undef RUN_REDUCE
#undef RUN_REDUCE3
	}
	free(workspace);
	return 0;
}

template <typename F>
static F* alloc_nan(size_t n)
{
	F* p = (F*)aligned_alloc(16, (n * sizeof(F) + 15) / 16 * 16);
	for (size_t i = 0; i < n; i++) p[i] = (F)NAN;
	return p;
}

template <typename F>
static int run(FILE* fi, FILE* fo, const int64_t* d, const char* mode, int argc, char** argv)
{
	const int64_t B = d[0], T = d[1], H = d[2], W = d[3];
	const size_t n = (size_t)(B * T * H * W), na = (size_t)(B * T * T * H);
	F *q = alloc_nan<F>(n), *k = alloc_nan<F>(n), *dA = alloc_nan<F>(na);
	if (fread(q, sizeof(F), n, fi) != n || fread(k, sizeof(F), n, fi) != n || fread(dA, sizeof(F), na, fi) != na) return 3;
	F *attn = alloc_nan<F>(na), *dq = alloc_nan<F>(n), *dk = alloc_nan<F>(n);
	int rc = 0;
	int64_t domain_flag = -1;  // the backward's sign-domain flag after the call; -1: the plan keeps none
	if constexpr (sizeof(F) == 8) {
		rc = l1attn_dense_fwd_f64(q, k, attn, B, T, H, W, nullptr);
		if (!rc) rc = l1attn_dense_bwd_f64(dA, q, k, dq, dk, B, T, H, W, nullptr, 0, nullptr);
	} else if (mode[1] == 'i') {  // fixed
		const size_t wb = l1attn_dense_fwd_fixed_workspace_bytes(B, T, H, W);
		void* ws = wb ? aligned_alloc(256, (wb + 255) / 256 * 256) : nullptr;
		rc = l1attn_dense_fwd_fixed_f32(q, k, attn, B, T, H, W, ws, wb, nullptr);
		free(ws);
	} else {
		const size_t wf = l1attn_dense_fwd_workspace_bytes(B, T, H, W);
		void* ws = wf ? aligned_alloc(256, (wf + 255) / 256 * 256) : nullptr;
		rc = l1attn_dense_fwd_ws_f32(q, k, attn, B, T, H, W, ws, wf, nullptr);
		free(ws);
		if (!rc && argc >= 8 && !strcmp(argv[4], "wide")) {
			const BwdPlan p = wide_plan(B, T, H, W, atoi(argv[5]), atoi(argv[6]) != 0, atoi(argv[7]),
			                            argc < 9 ? 0 : !strcmp(argv[8], "deep") ? 1 : !strcmp(argv[8], "deep2") ? 2 : 0);
			if (!p.fast) return 4;  // the kernels' limits rule this plan out
			rc = run_wide(p, dA, q, k, dq, dk, B, T, H, W);
		} else if (!rc) {
			const size_t wb = l1attn_dense_bwd_workspace_bytes(B, T, H, W);
			void* wsb = wb ? aligned_alloc(256, (wb + 255) / 256 * 256) : nullptr;
			if (wsb) memset(wsb, 0xA5, wb);  // nothing may rest on a zeroed workspace
			// "assume": the caller vouches for the sign range, the check and the fix-up are left out
			const bool assume = argc >= 5 && !strcmp(argv[4], "assume");
			rc = assume ? l1attn_dense_bwd_ex_f32(dA, q, k, dq, dk, B, T, H, W, 0, 0, 1, wsb, wb, nullptr)
			            : l1attn_dense_bwd_f32(dA, q, k, dq, dk, B, T, H, W, wsb, wb, nullptr);
			int64_t info[16];
			l1attn_dense_bwd_plan_info(B, T, H, W, info);
			if (!rc && info[15] > 0) domain_flag = *(const int*)wsb;
			free(wsb);
		}
	}
	if (rc) return 10 + (rc < 0 ? -rc : rc);
	if (emu_sload::outstanding != 0) return 9;  // a wave ended with a scalar prefetch in flight
	fwrite(attn, sizeof(F), na, fo);
	if (mode[1] != 'i') {
		fwrite(dq, sizeof(F), n, fo);
		fwrite(dk, sizeof(F), n, fo);
	}
	int64_t info[16];
	l1attn_dense_bwd_plan_info(B, T, H, W, info);
	fwrite(info, sizeof(int64_t), 16, fo);
	fwrite(&domain_flag, sizeof(int64_t), 1, fo);
	free(q); free(k); free(dA); free(attn); free(dq); free(dk);
	return 0;
}

static void print_launch(const char* kernel, dim3 g, dim3 b, size_t lds)
{
	printf("%s | %u %u %u | %u | %zu\n", kernel, g.x, g.y, g.z, b.x * b.y * b.z, lds);
}

// no memory behind the pointers: the host logic only looks at their alignment
static int dims(int64_t B, int64_t T, int64_t H, int64_t W)
{
	emu::dry = true;
	emu::on_launch = print_launch;
	float* const p = (float*)(uintptr_t)0x100000;
	const size_t wf = l1attn_dense_fwd_workspace_bytes(B, T, H, W), wb = l1attn_dense_bwd_workspace_bytes(B, T, H, W);
	printf("forward workspace %zu\n", wf);
	int rc = l1attn_dense_fwd_ws_f32(p, p, p, B, T, H, W, wf ? p : nullptr, wf, nullptr);
	printf("forward rc %d\nbackward workspace %zu\n", rc, wb);
	rc = l1attn_dense_bwd_f32(p, p, p, p, p, B, T, H, W, wb ? p : nullptr, wb, nullptr);
	printf("backward rc %d\n", rc);
	if ((W == 32 || W == 64) && T >= 32) {
		rc = l1attn_dense_fwd_fixed_f32(p, p, p, B, T, H, W, p, l1attn_dense_fwd_fixed_workspace_bytes(B, T, H, W), nullptr);
		printf("fixed rc %d\n", rc);
	}
	return 0;
}

int main(int argc, char** argv)
{
	if (argc == 6 && !strcmp(argv[1], "dims")) return dims(atoll(argv[2]), atoll(argv[3]), atoll(argv[4]), atoll(argv[5]));
	if (argc < 4) return 2;
	if (getenv("EMU_PRINT_LAUNCHES")) emu::on_launch = print_launch;  // to stdout, before the run's outputs go to <out>
	FILE* fi = fopen(argv[1], "rb");
	FILE* fo = fopen(argv[2], "wb");
	if (!fi || !fo) return 2;
	int64_t d[4];
	if (fread(d, sizeof(int64_t), 4, fi) != 4) return 3;
	const int rc = !strcmp(argv[3], "f64") ? run<double>(fi, fo, d, argv[3], argc, argv) : run<float>(fi, fo, d, argv[3], argc, argv);
	fclose(fi);
	fclose(fo);
	return rc;
}
