// TEST INFRASTRUCTURE: host stand-ins for the entry points of csrc/coo.hip and csrc/version.hip in the emulated
// library.  These functions produce what those kernels are specified to produce (the plan layout of csrc/plan.h,
// expandCoo's ranks) with plain loops, which keeps whole-operator runs on the emulated library short.  They check
// nothing about coo.hip: its kernels run from source in tests/test_cpu_emulation_coo.py (run_coo.cpp).
#include "hip/hip_runtime.h"
#include "../../l1-attention_amd/csrc/plan.h"
#include <map>
#include <vector>

extern "C" {

int l1attn_version(void) { return -1; }  // not the product library
int l1attn_probe_valu(float*, int64_t, int64_t, void*) { return L1ATTN_OK; }
int l1attn_probe_valu_op(float*, int64_t, int64_t, int op, void*) { return op >= 0 && op <= 3 ? L1ATTN_OK : L1ATTN_ERR_ARG; }

size_t l1attn_expand_coo_workspace_bytes(int64_t) { return 256; }

int l1attn_expand_coo(const void* co, int co_bits, int64_t co_stride, int64_t E, int32_t* coo, int32_t* mxlen_host,
                      void*, size_t, void*)
{
	if (E < 0 || co_stride < 2 || !mxlen_host || (co_bits != 32 && co_bits != 64)) return L1ATTN_ERR_ARG;
	mxlen_host[0] = mxlen_host[1] = 1;
	if (E == 0) return L1ATTN_OK;
	if (!co || !coo) return L1ATTN_ERR_ARG;
	std::map<int64_t, int> nd, ns;
	for (int64_t i = 0; i < E; i++) {
		const int64_t d = co_bits == 32 ? ((const int32_t*)co)[i * co_stride] : ((const int64_t*)co)[i * co_stride];
		const int64_t s = co_bits == 32 ? ((const int32_t*)co)[i * co_stride + 1] : ((const int64_t*)co)[i * co_stride + 1];
		if (d < 0 || s < 0 || d > 2147483647LL || s > 2147483647LL) return L1ATTN_ERR_INDEX;
		coo[i * 4 + 0] = (int32_t)d;
		coo[i * 4 + 1] = (int32_t)s;
		coo[i * 4 + 2] = nd[d]++;
		coo[i * 4 + 3] = ns[s]++;
		mxlen_host[0] = std::max(mxlen_host[0], coo[i * 4 + 2] + 1);
		mxlen_host[1] = std::max(mxlen_host[1], coo[i * 4 + 3] + 1);
	}
	return L1ATTN_OK;
}

size_t l1attn_sparse_plan_bytes(int64_t E, int64_t T) { return (E < 0 || T < 0) ? 0 : plan_layout(E, T).total_bytes; }
size_t l1attn_sparse_plan_workspace_bytes(int64_t, int64_t) { return 256; }

int l1attn_sparse_plan_build(const int32_t* coo, int64_t coo_stride, int64_t E, int64_t T, void* plan, size_t plan_bytes,
                             void*, size_t, void*)
{
	if (E < 0 || T < 0 || coo_stride < 2 || !plan) return L1ATTN_ERR_ARG;
	const PlanLayout L = plan_layout(E, T);
	if (plan_bytes < L.total_bytes) return L1ATTN_ERR_WORKSPACE;
	if (E > 0 && !coo) return L1ATTN_ERR_ARG;
	int* w = (int*)plan;
	for (size_t i = 0; i < L.total_bytes / 4; i++) w[i] = 0;
	// rows with an index outside [0, T) take the sentinel token T in both columns: they sort last and are dropped
	std::vector<int> dst((size_t)E), src((size_t)E);
	int bad = 0;
	for (int64_t i = 0; i < E; i++) {
		const int d = coo[i * coo_stride], s = coo[i * coo_stride + 1];
		const bool ok = d >= 0 && d < T && s >= 0 && s < T;
		dst[(size_t)i] = ok ? d : (int)T;
		src[(size_t)i] = ok ? s : (int)T;
		bad |= !ok;
	}
	auto segments = [&](const std::vector<int>& key, int* ptr, std::vector<int>& order) {  // stable counting sort
		for (int64_t i = 0; i < E; i++) ptr[key[(size_t)i] + 1]++;
		for (int64_t t = 0; t < T + 1; t++) ptr[t + 1] += ptr[t];
		std::vector<int> next(ptr, ptr + T + 1);
		order.assign((size_t)E, 0);
		for (int64_t i = 0; i < E; i++) order[(size_t)next[key[(size_t)i]]++] = (int)i;
	};
	std::vector<int> by_dst, by_src, slot_of_row((size_t)E);
	segments(dst, w + L.dst_ptr, by_dst);
	segments(src, w + L.src_ptr, by_src);
	for (int64_t p = 0; p < E; p++) {
		const int row = by_dst[(size_t)p];
		w[L.csr_src + p] = src[(size_t)row];
		w[L.csr_row + p] = row;
		slot_of_row[(size_t)row] = (int)p;
	}
	for (int64_t p = 0; p < E; p++) {
		const int row = by_src[(size_t)p];
		w[L.csc_dst + p] = dst[(size_t)row];
		w[L.csc_slot + p] = slot_of_row[(size_t)row];
	}
	int maxd = 0, maxs = 0, nld = 0, nls = 0;
	for (int64_t t = 0; t < T; t++) {
		const int dd = w[L.dst_ptr + t + 1] - w[L.dst_ptr + t], ds = w[L.src_ptr + t + 1] - w[L.src_ptr + t];
		maxd = std::max(maxd, dd);
		maxs = std::max(maxs, ds);
		if (dd > PLAN_LONG_SEGMENT) w[L.long_dst + nld++] = (int)t;
		if (ds > PLAN_LONG_SEGMENT) w[L.long_src + nls++] = (int)t;
	}
	w[PLAN_H_MAGIC] = PLAN_MAGIC; w[PLAN_H_E] = (int)E; w[PLAN_H_T] = (int)T; w[PLAN_H_BAD] = bad;
	w[PLAN_H_MAXDEG_DST] = maxd; w[PLAN_H_MAXDEG_SRC] = maxs;
	w[PLAN_H_E_VALID] = T >= 0 ? w[L.dst_ptr + T] : 0;
	w[PLAN_H_NLONG_DST] = nld; w[PLAN_H_NLONG_SRC] = nls;
	return L1ATTN_OK;
}

int l1attn_sparse_plan_check(const void* plan, int64_t E, int64_t T, int32_t* header_host, void*)
{
	if (!plan || !header_host) return L1ATTN_ERR_ARG;
	const int* w = (const int*)plan;
	for (int i = 0; i < PLAN_H_WORDS; i++) header_host[i] = w[i];
	if (w[PLAN_H_MAGIC] != PLAN_MAGIC || w[PLAN_H_E] != (int)E || w[PLAN_H_T] != (int)T) return L1ATTN_ERR_ARG;
	return w[PLAN_H_BAD] ? L1ATTN_ERR_INDEX : L1ATTN_OK;
}

}  // extern "C"
