// Column ranks for the dense backward, second implementation: the column is sorted by a merge sort written for
// this kernel (registers and LDS only) instead of the library block radix sort of dense_rank.hip.  Same
// definition of the ranks, so the two produce identical rq and rk:
//   rk[s] = 2 * #{k' < k[s]} - 1/2
//   rq[t] = 2 * #{k' < q[t]}      if some k' == q[t],   2 * #{k' < q[t]} - 1 otherwise
// (see dense_rank.hip for why these make sign(q - k) one instruction in the backward).
//
// One workgroup per column (b,h,w).  A thread loads ITEMS consecutive tokens of the column's k values as
// order-preserving integer keys and sorts them in registers (odd-even transposition network); the sorted runs of
// ITEMS keys go to LDS and are merged pairwise, log2(BLOCK) rounds: in a round every thread produces the ITEMS
// consecutive outputs of its place in the merged run, which it finds by a binary search along the merge path
// (how many of the first d outputs come from the left run), then ITEMS steps of a two-way merge.  Outputs are
// held in registers until every thread has read its inputs, so the rounds work in place: BLOCK*ITEMS*4 bytes of
// LDS (16 KiB for 4096 tokens).  Keys only, so the order of equal keys does not matter.
// The searches for the ranks then run on the sorted column as in dense_rank.hip.
//
// Kept beside the library-sort kernel until both have been timed on a GPU; the backward uses this one only when
// asked to (see l1_rank_sort_choice in dense.hip).  No counterpart in the reference, which evaluates sign(q-k)
// per pair-element (cuda/l1attn_cuda_kernel.cu:206-455).
#include "common.h"
#include "dense_rank.h"

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

template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void dense_column_ranks_merge(const float* __restrict__ q, const float* __restrict__ k,
                                                                    float* __restrict__ rq, float* __restrict__ rk, int Tn,
                                                                    int HW, int n_col)
{
	constexpr int N = BLOCK * ITEMS;
	static_assert((BLOCK & (BLOCK - 1)) == 0 && (ITEMS & (ITEMS - 1)) == 0, "runs double until one is left");
	__shared__ unsigned sorted[N];

	// the same XCD-aware order of columns as dense_column_ranks: neighbours share 64-byte sectors of q and k
	const unsigned n = gridDim.x, flat = blockIdx.x, per = n / 8u;
	const unsigned col = flat < per * 8u ? (flat % 8u) * per + flat / 8u : flat;
	if (col >= (unsigned)n_col) return;  // same for every thread of the workgroup
	const int64_t base = (int64_t)(col / (unsigned)HW) * Tn * HW + (col % (unsigned)HW);
	const int out0 = (int)threadIdx.x * ITEMS;  // this thread's ITEMS consecutive places, in every round

	unsigned key[ITEMS], mine[ITEMS];
#pragma unroll
	for (int i = 0; i < ITEMS; i++) {
		const int t = out0 + i;
		mine[i] = t < Tn ? float_key(k[base + (int64_t)t * HW]) : 0xFFFFFFFFu;  // padding sorts last
		key[i] = mine[i];
	}
	// sort the thread's run in registers
#pragma unroll
	for (int r = 0; r < ITEMS; r++) {
#pragma unroll
		for (int i = r & 1; i + 1 < ITEMS; i += 2) {
			const unsigned lo = min(key[i], key[i + 1]), hi = max(key[i], key[i + 1]);
			key[i] = lo;
			key[i + 1] = hi;
		}
	}
#pragma unroll
	for (int i = 0; i < ITEMS; i++) sorted[out0 + i] = key[i];
	__syncthreads();

	for (int L = ITEMS; L < N; L *= 2) {
		const int m0 = out0 & ~(2 * L - 1);       // start of the pair of runs this thread's outputs belong to
		const unsigned* const A = sorted + m0;    // left run, L keys
		const unsigned* const Bv = A + L;         // right run, L keys
		const int d = out0 - m0;                  // outputs of the merged run before this thread's
		// merge path: i = how many of the first d outputs come from the left run
		int lo = max(0, d - L), hi = min(d, L);
		while (lo < hi) {
			const int mid = (lo + hi) >> 1;
			if (A[mid] <= Bv[d - 1 - mid]) lo = mid + 1;
			else hi = mid;
		}
		int i = lo, j = d - lo;
		unsigned a = i < L ? A[i] : 0xFFFFFFFFu, b = j < L ? Bv[j] : 0xFFFFFFFFu;
#pragma unroll
		for (int o = 0; o < ITEMS; o++) {
			const bool take_a = j >= L || (i < L && a <= b);
			key[o] = take_a ? a : b;
			if (take_a) { i++; a = i < L ? A[i] : 0xFFFFFFFFu; }
			else { j++; b = j < L ? Bv[j] : 0xFFFFFFFFu; }
		}
		__syncthreads();  // every thread has read what it needs of this round's runs
#pragma unroll
		for (int o = 0; o < ITEMS; o++) sorted[out0 + o] = key[o];
		__syncthreads();
	}

#pragma unroll
	for (int i = 0; i < ITEMS; i++) {
		const int t = out0 + i;
		if (t < Tn) rk[base + (int64_t)t * HW] = (float)(2 * count_less(sorted, Tn, mine[i])) - 0.5f;
	}
#pragma unroll
	for (int i = 0; i < ITEMS; i++) {
		const int t = out0 + i;
		if (t < Tn) {
			const unsigned x = float_key(q[base + (int64_t)t * HW]);
			const int lb = count_less(sorted, Tn, x);
			const bool tie = lb < Tn && sorted[lb] == x;
			rq[base + (int64_t)t * HW] = (float)(2 * lb - (tie ? 0 : 1));
		}
	}
}

constexpr int MERGE_BLOCK = 512;

}  // namespace

int l1_launch_column_ranks_merge(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                                 int64_t W, hipStream_t st)
{
	if (!(B >= 1 && T >= 1 && T <= L1_RANK_MAX_T && H * W >= 1 && B * H * W < ((int64_t)1 << 31))) return L1ATTN_ERR_RANGE;
	const int n_col = (int)(B * H * W);
	const dim3 grid((unsigned)n_col), block(MERGE_BLOCK);
#define L1_RANK_CASE(ITEMS)                                                                                      \
	hipLaunchKernelGGL((dense_column_ranks_merge<MERGE_BLOCK, ITEMS>), grid, block, 0, st, q, k, rq, rk, (int)T, \
	                   (int)(H * W), n_col)
	if (T <= 1 * MERGE_BLOCK) L1_RANK_CASE(1);
	else if (T <= 2 * MERGE_BLOCK) L1_RANK_CASE(2);
	else if (T <= 4 * MERGE_BLOCK) L1_RANK_CASE(4);
	else if (T <= 8 * MERGE_BLOCK) L1_RANK_CASE(8);
	else L1_RANK_CASE(16);
#undef L1_RANK_CASE
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

extern "C" int l1attn_dense_column_ranks_merge_f32(const float* q, const float* k, float* rq, float* rk, int64_t B,
                                                   int64_t T, int64_t H, int64_t W, void* stream)
{
	if (B < 0 || T < 0 || H < 0 || W < 0) return L1ATTN_ERR_ARG;
	if (B * T * H * W == 0) return L1ATTN_OK;
	if (!q || !k || !rq || !rk) return L1ATTN_ERR_ARG;
	return l1_launch_column_ranks_merge(q, k, rq, rk, B, T, H, W, (hipStream_t)stream);
}
