// Column ranks for the dense backward (gfx950).
//
// The backward only needs sign(q[b,t,h,w] - k[b,s,h,w]) for every (s,t) of a column (b,h,w).  Any
// pair of maps rq, rk that keeps the order and the ties of a column gives the same signs, and maps
// onto small integers make the sign a single instruction: with rk stored minus one half,
// clamp(rq - rk, 0, 1) is 1, 1/2 or 0 for q > k, q == k, q < k, exactly.
//
// Per column: sort the T values of k, then
//   rk[s] = 2 * #{k' < k[s]} - 1/2                      (equal k share a rank)
//   rq[t] = 2 * #{k' < q[t]}      if some k' == q[t]
//           2 * #{k' < q[t]} - 1  otherwise
// so rq - (rk + 1/2) is 0 on a tie and at least 1 in magnitude otherwise.  -0 and +0 compare equal,
// as they do in q - k.  No counterpart in the reference, which evaluates sign(q-k) per element
// (cuda/l1attn_cuda_kernel.cu:206-455).
#include "common.h"
#include "dense_rank.h"
#include <rocprim/block/block_radix_sort.hpp>

namespace {

// order-preserving map of a float onto unsigned integers; both zeros map to the same key
__device__ __forceinline__ unsigned float_key(float x)
{
	if (x == 0.0f) x = 0.0f;
	const unsigned u = __float_as_uint(x);
	return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// number of entries of sorted[0, n) that are smaller than x
__device__ __forceinline__ int count_less(const unsigned* sorted, int n, unsigned x)
{
	int lo = 0;
	while (n > 0) {
		const int half = n >> 1;
		if (sorted[lo + half] < x) { lo += half + 1; n -= half + 1; }
		else n = half;
	}
	return lo;
}

// One workgroup per column.  Consecutive columns share 64-byte sectors of q and k (a column is
// strided by H*W floats), so the dispatch order is remapped to give each XCD a contiguous range of
// columns: the neighbours that need the rest of a sector run on the same L2 at about the same time.
template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void dense_column_ranks(const float* __restrict__ q, const float* __restrict__ k,
                                                             float* __restrict__ rq, float* __restrict__ rk, int Tn,
                                                             int HW, int n_col)
{
	using sort_t = rocprim::block_radix_sort<unsigned, BLOCK, ITEMS>;
	__shared__ typename sort_t::storage_type storage;
	__shared__ unsigned sorted[BLOCK * ITEMS];

	const unsigned n = gridDim.x, flat = blockIdx.x, per = n / 8u;
	const unsigned col = flat < per * 8u ? (flat % 8u) * per + flat / 8u : flat;
	if (col >= (unsigned)n_col) return;  // same for every thread of the workgroup
	const int64_t base = (int64_t)(col / (unsigned)HW) * Tn * HW + (col % (unsigned)HW);

	unsigned key[ITEMS], mine[ITEMS];
#pragma unroll
	for (int i = 0; i < ITEMS; i++) {
		const int t = (int)threadIdx.x + i * BLOCK;
		mine[i] = t < Tn ? float_key(k[base + (int64_t)t * HW]) : 0xFFFFFFFFu;  // padding sorts last
		key[i] = mine[i];
	}
	sort_t().sort(key, storage);  // thread x now holds sorted[x*ITEMS .. x*ITEMS+ITEMS)
#pragma unroll
	for (int i = 0; i < ITEMS; i++) sorted[threadIdx.x * ITEMS + i] = key[i];
	__syncthreads();
#pragma unroll
	for (int i = 0; i < ITEMS; i++) {
		const int t = (int)threadIdx.x + i * BLOCK;
		if (t < Tn) rk[base + (int64_t)t * HW] = (float)(2 * count_less(sorted, Tn, mine[i])) - 0.5f;
	}
#pragma unroll
	for (int i = 0; i < ITEMS; i++) {
		const int t = (int)threadIdx.x + i * BLOCK;
		if (t < Tn) {
			const unsigned x = float_key(q[base + (int64_t)t * HW]);
			const int lb = count_less(sorted, Tn, x);
			const bool tie = lb < Tn && sorted[lb] == x;
			rq[base + (int64_t)t * HW] = (float)(2 * lb - (tie ? 0 : 1));
		}
	}
}

constexpr int RANK_BLOCK = 512;

}  // namespace

bool l1_column_ranks_ok(int64_t B, int64_t T, int64_t H, int64_t W)
{
	return B >= 1 && T >= 1 && T <= L1_RANK_MAX_T && H * W >= 1 && B * H * W < ((int64_t)1 << 31);
}

int l1_launch_column_ranks(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                           int64_t W, hipStream_t st)
{
	if (!l1_column_ranks_ok(B, T, H, W)) return L1ATTN_ERR_RANGE;
	const int n_col = (int)(B * H * W);
	const dim3 grid((unsigned)n_col), block(RANK_BLOCK);
#define L1_RANK_CASE(ITEMS)                                                                                      \
	hipLaunchKernelGGL((dense_column_ranks<RANK_BLOCK, ITEMS>), grid, block, 0, st, q, k, rq, rk, (int)T, (int)(H * W), \
	                   n_col)
	if (T <= 1 * RANK_BLOCK) L1_RANK_CASE(1);
	else if (T <= 2 * RANK_BLOCK) L1_RANK_CASE(2);
	else if (T <= 4 * RANK_BLOCK) L1_RANK_CASE(4);
	else if (T <= 8 * RANK_BLOCK) L1_RANK_CASE(8);
	else L1_RANK_CASE(16);
#undef L1_RANK_CASE
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

extern "C" int l1attn_dense_column_ranks_f32(const float* q, const float* k, float* rq, float* rk, int64_t B,
                                             int64_t T, int64_t H, int64_t W, void* stream)
{
	if (B < 0 || T < 0 || H < 0 || W < 0) return L1ATTN_ERR_ARG;
	if (B * T * H * W == 0) return L1ATTN_OK;
	if (!q || !k || !rq || !rk) return L1ATTN_ERR_ARG;
	return l1_launch_column_ranks(q, k, rq, rk, B, T, H, W, (hipStream_t)stream);
}
