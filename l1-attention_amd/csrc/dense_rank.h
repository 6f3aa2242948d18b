// Column ranks of q and k for the dense backward: see dense_rank.hip.
#pragma once
#include "common.h"

constexpr int64_t L1_RANK_MAX_T = 8192;  // one workgroup sorts a whole column in LDS

bool l1_column_ranks_ok(int64_t B, int64_t T, int64_t H, int64_t W);

// rq, rk: [B,T,H,W] floats.  rk holds the rank minus one half.  Asynchronous on the stream.
int l1_launch_column_ranks(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                           int64_t W, hipStream_t st);

// The same ranks from the merge sort of rank_sort.hip (identical outputs).
int l1_launch_column_ranks_merge(const float* q, const float* k, float* rq, float* rk, int64_t B, int64_t T, int64_t H,
                                 int64_t W, hipStream_t st);
