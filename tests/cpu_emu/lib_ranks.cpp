// TEST INFRASTRUCTURE: the column-rank entry points for the emulated library.  The merge-sort kernel
// (csrc/rank_sort.hip) runs as it is; the library-sort kernel of csrc/dense_rank.hip cannot be compiled for the host,
// so its entry points run the merge sort, which gives the same ranks by definition.
#include "hip/hip_runtime.h"
#include "../../l1-attention_amd/csrc/rank_sort.hip"

bool l1_column_ranks_ok(int64_t B, int64_t T, int64_t H, int64_t W)
{
	return B >= 1 && T >= 1 && T <= L1_RANK_MAX_T && H * W >= 1 && B * H * W < ((int64_t)1 << 31);
}
int l1_launch_column_ranks(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                           int64_t W, hipStream_t st)
{
	return l1_launch_column_ranks_merge(q, k, rq, rk, B, T, H, W, st);
}
extern "C" int l1attn_dense_column_ranks_f32(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T,
                                             int64_t H, int64_t W, void* stream)
{
	return l1attn_dense_column_ranks_merge_f32(q, k, rq, rk, B, T, H, W, stream);
}
