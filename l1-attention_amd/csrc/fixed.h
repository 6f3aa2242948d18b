// Conversion of q and k to per-head fixed point for the experimental fixed-point dense forward (fixed.hip).
#pragma once
#include "common.h"

// gq [B*H]: grid of each (batch, head); uq, uk [B,T,H,W]: biased fixed-point copies of q and k.  Asynchronous.
int l1_launch_fixed_prepass(const float* q, const float* k, float* gq, unsigned* uq, unsigned* uk, int64_t B,
                            int64_t T, int64_t H, int64_t W, hipStream_t st);
