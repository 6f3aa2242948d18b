/*
 * C ABI of libl1attn_hip.so -- hand-written HIP kernels for gfx950 (MI355X) behind the
 * operator boundary of tlh24/l1-attention.  Plain pointers and sizes only; no torch types.
 *
 * Conventions
 *   - All data pointers are DEVICE pointers on the GPU that owns `stream`
 *     (a hipStream_t passed as void*; NULL = the default stream).  Tensors are contiguous,
 *     row-major, in the reference's layouts:  q,k,v,... [B,T,H,W];  attn / d_attn [B,S,T,H]
 *     with the src token S first (cuda/l1attn_cuda.py:9-15, python/l1attn.py:20-30).
 *   - The caller owns every buffer, including workspaces; the library allocates nothing and
 *     keeps no state between calls (re-entrant; calls on one stream are ordered by it).
 *   - Inputs are never written.  Outputs are fully overwritten (no zero-init needed).
 *   - Return value: 0 = launched; negative = argument error (below); positive = hipError_t.
 *     Launches are asynchronous: a kernel fault surfaces at the next synchronisation.
 *   - scale = -1/sqrt(W) is part of the operator in every reference implementation
 *     (cuda/l1attn_cuda_kernel.cu:476, cpp/l1attn_drv.cpp:22).
 */
#ifndef L1ATTN_HIP_H
#define L1ATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define L1ATTN_OK 0
#define L1ATTN_ERR_ARG (-1)       /* null pointer, negative size, W < 1, unsupported dtype code */
#define L1ATTN_ERR_WORKSPACE (-2) /* workspace missing or smaller than *_workspace_bytes() */
#define L1ATTN_ERR_RANGE (-3)     /* a size beyond what the kernels index */
#define L1ATTN_ERR_INDEX (-4)     /* edge list holds an index outside [0, T) */

/* Library version (major*10000 + minor*100 + patch). */
int l1attn_version(void);

/* ------------------------------------------------------------------------------ dense */

/*
 * attn[b,s,t,h] = -1/sqrt(W) * sum_w |q[b,t,h,w] - k[b,s,h,w]|.
 * Replaces l1attn_cuda_drv.forward(q,k) -> [attn]  (cuda/l1attn_cuda_drv.cpp:42-65,
 * kernels cuda/l1attn_cuda_kernel.cu:27-203; CPU twin cpp/l1attn_drv.cpp:13-55).
 * No layout transposes and no 32-bit index limit: attn may exceed 2^31 elements.
 */
int l1attn_dense_fwd_f32(const float* q, const float* k, float* attn,
                         int64_t B, int64_t T, int64_t H, int64_t W, void* stream);
int l1attn_dense_fwd_f64(const double* q, const double* k, double* attn,
                         int64_t B, int64_t T, int64_t H, int64_t W, void* stream);

/*
 * The f32 forward with a workspace.  Widths that are not a multiple of 16 (the reference's timing
 * sweep uses 33, 65, 97: benchmark.py:60) run the tiled kernels on zero-padded copies of q and k
 * held in `workspace` (l1attn_dense_fwd_workspace_bytes(), 0 when the shape needs none; 16-byte
 * aligned); without a workspace they take the generic kernel, as l1attn_dense_fwd_f32 does.
 * Same results either way up to fp32 summation order.
 */
size_t l1attn_dense_fwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W);
int l1attn_dense_fwd_ws_f32(const float* q, const float* k, float* attn,
                            int64_t B, int64_t T, int64_t H, int64_t W,
                            void* workspace, size_t workspace_bytes, void* stream);

/*
 * dq[b,t,h,w] =  sum_s scale*sign(q[b,t,h,w]-k[b,s,h,w]) * d_attn[b,s,t,h]
 * dk[b,s,h,w] = -sum_t scale*sign(q[b,t,h,w]-k[b,s,h,w]) * d_attn[b,s,t,h],   sign(0) = 0.
 * Replaces l1attn_cuda_drv.backward(d_attn,q,k) -> [dq,dk]  (cuda/l1attn_cuda_drv.cpp:67-104,
 * kernels cuda/l1attn_cuda_kernel.cu:206-455; CPU twin cpp/l1attn_drv.cpp:57-98).
 * d_attn is read in its native [B,S,T,H] layout.  Deterministic, unlike the reference's float
 * atomics (cuda/l1attn_cuda_kernel.cu:439, :453): dk is summed in a fixed order from partial rows,
 * each address of which is written by one lane only (where a workgroup adds several dst tiles into
 * one partial, the additions are done by the L2 in that lane's program order).  The partials are
 * held in `workspace` (device memory, 256-byte aligned, at least
 * l1attn_dense_bwd_workspace_bytes() for full speed; its fixed head, info[15] of
 * l1attn_dense_bwd_plan_info, plus any multiple of one batch's share, info[12], works: the batches
 * are then processed in several launches).  The f64 entry needs no workspace.
 * sign(): the generic f32 kernels (T < 16 or H*W < 32) and the f64 entry compare, as the reference does
 * (cpp/l1attn_drv.cpp:7-11).  The f32 tiled path takes it as clamp(q*2^64 - k*2^64, -1, 1), which equals
 * sign(q-k) for every pair while all magnitudes are below 2^63 and all non-zero ones at least 2^-41;
 * a pre-pass over q and k checks exactly that on the device (a flag in the head of the workspace), and
 * when it does not hold -- tiny values, huge ones, infinities, NaN -- one more kernel of the same call
 * recomputes dq and dk with comparisons.  The call stays asynchronous and the result is the reference's
 * for every input; only the speed differs (O(T) reads per output element in the recomputation).
 * For 2048 <= T <= 8192 (and enough work to fill the GPU) sign() is taken from the column ranks of
 * l1attn_dense_column_ranks_f32 instead, exact for all finite inputs (no pre-pass, no flag); the
 * gradient is then assembled as 2*sum(hv*d_attn) - sum(d_attn) with hv = (sign+1)/2, so an element
 * whose pairs all tie comes out as a rounding residue of the two sums (about 1e-6 of the largest
 * gradient) instead of an exact zero.
 */
size_t l1attn_dense_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W);
/*
 * No counterpart in the reference: reports how l1attn_dense_bwd_f32 tiles a shape, for tests of the host
 * logic and for tuning; computes nothing on the GPU.  info[0..15]:
 *   0 tiled path (else the generic kernels)   1 wide tiles (64..88 dst tokens, <= 512 threads)
 *   2 column ranks                            3 branch-free step loop
 *   4 threads per workgroup                   5 column chunks (workgroups across H*W)
 *   6 dst tiles                               7 dst tokens per tile
 *   8 staged d_attn values per thread, step   9 dst tiles per workgroup
 *  10 workgroups along T (= partial arrays)  11 LDS bytes per workgroup
 *  12 workspace bytes per batch              13 batches per launch with the full workspace
 *  14 form of the branch-free step loop the plan runs: 0 (always, through l1attn_dense_bwd_plan_info), or the
 *     loop_form given to l1attn_dense_bwd_plan_info_ex where the plan is branch-free
 *  15 bytes at the head of the workspace that hold the sign-domain flag (256, or 0 with column ranks)
 * Returns 0, or a negative argument error.
 */
int l1attn_dense_bwd_plan_info(int64_t B, int64_t T, int64_t H, int64_t W, int64_t* info);
int l1attn_dense_bwd_f32(const float* d_attn, const float* q, const float* k, float* dq, float* dk,
                         int64_t B, int64_t T, int64_t H, int64_t W,
                         void* workspace, size_t workspace_bytes, void* stream);
int l1attn_dense_bwd_f64(const double* d_attn, const double* q, const double* k, double* dq, double* dk,
                         int64_t B, int64_t T, int64_t H, int64_t W,
                         void* workspace, size_t workspace_bytes, void* stream);
/*
 * l1attn_dense_bwd_f32 with its internal choices as arguments; l1attn_dense_bwd_f32 is this call with
 * (0, 0, 0).  The library reads no environment variable and keeps no state between calls: a caller that wants a
 * non-default form says so here, per call.  Same workspace as l1attn_dense_bwd_f32.
 *   loop_form  step loop of the branch-free long-sequence plans: 0 one step of prefetch distance, 1 two steps,
 *              2 two steps with two LDS planes and one barrier per step.  Bit-identical results; other plans
 *              ignore it (l1attn_dense_bwd_plan_info_ex reports in info[14] what a shape runs).
 *   rank_sort  where the plan takes sign() from column ranks: 0 ranks from l1attn_dense_column_ranks_f32,
 *              1 from l1attn_dense_column_ranks_merge_f32.  Identical ranks.
 *   assume_sign_range  1: the caller vouches that every magnitude in q and k is below 2^63 and every non-zero
 *              one at least 2^-41 (ordinary activations are); the range check and the fix-up launch of the tiled
 *              path are left out, which saves one read of q and k -- about 20/T of the call, so it matters for
 *              short sequences only.  Outside the vouched range the gradient follows clamp(q*2^64 - k*2^64, -1, 1)
 *              in place of sign(q-k).  0: checked, exact for every input.
 * Other values: L1ATTN_ERR_ARG.  No counterpart in the reference; the non-zero loop_form and rank_sort exist so that
 * they can be timed against the default and are not reached by the Python operators unless the caller opts in by name.
 */
int l1attn_dense_bwd_plan_info_ex(int64_t B, int64_t T, int64_t H, int64_t W, int loop_form, int64_t* info);
int l1attn_dense_bwd_ex_f32(const float* d_attn, const float* q, const float* k, float* dq, float* dk,
                            int64_t B, int64_t T, int64_t H, int64_t W, int loop_form, int rank_sort,
                            int assume_sign_range, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Order-preserving integer ranks of q and k per column (b,h,w), the first stage of the f32
 * backward for T <= 8192: rq[b,t,h,w] - (rk[b,s,h,w] + 1/2) has the sign of q[b,t,h,w] -
 * k[b,s,h,w], is 0 exactly when they are equal (-0 == +0) and is at least 1 in magnitude
 * otherwise; rk holds its rank minus one half.  rq, rk: [B,T,H,W] floats.
 * No counterpart in the reference, which evaluates sign(q-k) per pair-element
 * (cuda/l1attn_cuda_kernel.cu:206-455); exported so that the stage can be tested on its own.
 * Returns L1ATTN_ERR_RANGE for T > 8192.
 */
int l1attn_dense_column_ranks_f32(const float* q, const float* k, float* rq, float* rk,
                                  int64_t B, int64_t T, int64_t H, int64_t W, void* stream);
/*
 * The same ranks (identical rq, rk) from a merge sort written for this library instead of the library block
 * radix sort behind l1attn_dense_column_ranks_f32.  l1attn_dense_bwd_f32 never uses it; l1attn_dense_bwd_ex_f32
 * does with rank_sort = 1.  Kept beside the other until both have been timed on a GPU.  No counterpart in the
 * reference.
 */
int l1attn_dense_column_ranks_merge_f32(const float* q, const float* k, float* rq, float* rk,
                                        int64_t B, int64_t T, int64_t H, int64_t W, void* stream);

/*
 * Experimental: the f32 forward on fixed point.  q and k of every (batch, head) are converted once to
 * 32-bit integers on a common grid g = max(|q|,|k|) * 2^-24 (caller-owned workspace of
 * l1attn_dense_fwd_fixed_workspace_bytes), the pair-element is then one v_sad_u32 (|a-b|+c) instead of a
 * subtraction and an addition, the sum over W is exact, and attn = sum * g * (-1/sqrt(W)) in fp32.
 * Inputs and output are fp32 as in l1attn_dense_fwd_f32; each input moves by at most 0.75 g (g is between
 * half and one fp32 spacing of the head's largest values), so logits differ from the fp32 kernel's by about 1e-7 of
 * the largest logit on N(0,1) or LayerNorm-scaled inputs (tolerance 1e-5).  Inputs must be finite.
 * Only W = 32 or 64, T >= 32, 16-byte aligned q and k (L1ATTN_ERR_ARG otherwise).  No counterpart in the
 * reference; not the default path of the Python operator.
 */
size_t l1attn_dense_fwd_fixed_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W);
int l1attn_dense_fwd_fixed_f32(const float* q, const float* k, float* attn,
                               int64_t B, int64_t T, int64_t H, int64_t W,
                               void* workspace, size_t workspace_bytes, void* stream);

/*
 * Fused forward: dense L1 logits, softmax over the src tokens with the no-op zero logit, value sum;
 * the [B,S,T,H] logits are never written.
 *   a[s]        = -1/sqrt(W) * sum_w |q[b,t,h,w] - k[b,s,h,w]|
 *   vo[b,t,h,:] = sum_s exp(a[s]) * v[b,s,h,:] / (1 + sum_s exp(a[s]))
 *   lse[b,t,h]  = log(1 + sum_s exp(a[s]))          (optional: lse may be NULL)
 * The reference has no single function for this; it is the composition its model code builds from
 * l1attn_cuda_drv.forward (a zero logit row appended, softmax over dim 1, 'bsdh,bshw->bdhw':
 * example-setfind/setfind.py:128-136, python/l1attn_sparse.py:488-506) and the form its README asks
 * for (README.md:21).  q,k [B,T,H,W]; v,vo [B,T,H,Wv].  Deterministic.  Backward: below.
 * f32: W == Wv in {16,32,48,64,96}, T >= 32 and 16-byte aligned pointers run the tiled kernel; every other
 * shape, and f64, a generic one (L1ATTN_ERR_RANGE when it would need 2^32 threads or more).
 */
int l1attn_fused_fwd_f32(const float* q, const float* k, const float* v, float* vo, float* lse,
                         int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream);
int l1attn_fused_fwd_f64(const double* q, const double* k, const double* v, double* vo, double* lse,
                         int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream);
/*
 * The f32 fused forward with the k and v rows streamed through a software pipeline of scalar loads (the
 * technique of the dense forward) for W == Wv in {32, 64}; every other shape runs what l1attn_fused_fwd_f32
 * runs.  Same arithmetic in the same order: results equal l1attn_fused_fwd_f32's bit for bit.  Kept as an entry of
 * its own until both have been timed on a GPU.  No counterpart in the reference.
 */
int l1attn_fused_fwd_pipe_f32(const float* q, const float* k, const float* v, float* vo, float* lse,
                              int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream);

/*
 * Backward of the fused forward, first stage.  With p[s,t] = exp(a[s,t] - lse[t]), dp[s,t] = v[s].dvo[t],
 * S[t] = vo[t].dvo[t]:   dA[b,s,t,h] = p * (dp - S[t])  (gradient of the logits, dense layout [B,S,T,H])
 * and dv[b,s,h,:] = sum_t p[s,t] * dvo[b,t,h,:].  dq and dk are then l1attn_dense_bwd_* of (dA, q, k).
 * vo and lse are the forward's outputs.  dA is the only [B,T,T,H] tensor of the whole forward + backward
 * (the unfused composition of example-setfind/setfind.py:128-136 keeps the logits, the weights and the
 * gradients of both).  Batch entries are independent: a caller that cannot hold [B,T,T,H] calls this and
 * l1attn_dense_bwd_* on slabs of batch entries (pointers advanced by whole entries, B = the slab's count) with one
 * dA buffer of the slab's size reused in stream order, as the Python driver does (1 GiB by default).
 * No counterpart in the reference.  Deterministic.  Shapes as l1attn_fused_fwd_*.
 */
int l1attn_fused_bwd_stage_f32(const float* dvo, const float* q, const float* k, const float* v,
                               const float* vo, const float* lse, float* dA, float* dv,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream);
int l1attn_fused_bwd_stage_f64(const double* dvo, const double* q, const double* k, const double* v,
                               const double* vo, const double* lse, double* dA, double* dv,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream);
/*
 * l1attn_fused_bwd_stage_f32 with the wave-uniform rows of both kernels streamed through a software pipeline of
 * scalar loads where such kernels exist (W == Wv in {32, 64}; other shapes run what l1attn_fused_bwd_stage_f32
 * runs).  Same arithmetic in the same order: bit-equal dA and dv.  No counterpart in the reference.
 */
int l1attn_fused_bwd_stage_pipe_f32(const float* dvo, const float* q, const float* k, const float* v,
                                    const float* vo, const float* lse, float* dA, float* dv,
                                    int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, void* stream);

/* -------------------------------------------------------------------------- edge lists */

/*
 * expandCoo on the GPU: for an edge list co[E, co_stride>=2] of [dst, src] rows (device memory,
 * 32- or 64-bit signed integers: co_bits = 32 | 64) writes coo int32 [E,4] (device) with
 *   coo[i] = [dst_i, src_i, #{j<i : dst_j == dst_i}, #{j<i : src_j == src_i}]
 * and mxlen_host[0..1] = {dst_mxlen, src_mxlen} = 1 + the largest rank of each kind ({1,1} for
 * E == 0).  Replaces the Python loop expandCoo (python/l1attn_sparse.py:382-427;
 * cuda/l1attn_sparse_cuda.py:58-101; cuda/l1attn_sparse_bidi_cuda.py:59-104;
 * cpp/l1attn_sparse_cpp.py:61-106).  Bit-exact (integer only).  Because two host integers are
 * returned, this call synchronises `stream` before returning.  Indices must be in
 * [0, 2^31-1]: L1ATTN_ERR_INDEX otherwise (the reference's printed "degenerate sparse head"
 * warnings are host-side diagnostics and are produced by the Python wrapper, not here).
 * workspace: device memory, >= l1attn_expand_coo_workspace_bytes(E), 256-byte aligned.
 */
size_t l1attn_expand_coo_workspace_bytes(int64_t E);
int l1attn_expand_coo(const void* co, int co_bits, int64_t co_stride, int64_t E,
                      int32_t* coo, int32_t* mxlen_host,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * Plan = the dst-sorted and src-sorted views of an edge list, built once per list and reused by
 * every forward/backward on it.  It stands in for what the reference recomputes on every call
 * through coo[:,2] (the dst_cnt slot of each edge in the padded [B,T,dst_mxlen,H] tensor,
 * cuda/l1attn_sparse_cuda_kernel.cu:50-84) and replaces the atomicAdd scatters (:179, :232,
 * :367-368, :568-569, :625-626) with segment walks.  Only columns 0 and 1 of coo are read
 * (coo int32 [E, coo_stride>=2], device); slot order inside a segment is the original row order,
 * i.e. the order of the reference's dst_cnt / src_cnt.  Rows with an index outside [0,T) are
 * dropped and flagged (the reference's behaviour is undefined there).
 * plan: device buffer of l1attn_sparse_plan_bytes(E,T) bytes, 256-byte aligned, opaque.
 * l1attn_sparse_plan_build is asynchronous; l1attn_sparse_plan_check copies the 16-word header to
 * header_host, synchronises, and returns L1ATTN_ERR_INDEX if rows were dropped
 * (header words: 1 = E, 2 = T, 3 = dropped flag, 4 = longest dst segment, 5 = longest src segment).
 */
size_t l1attn_sparse_plan_bytes(int64_t E, int64_t T);
size_t l1attn_sparse_plan_workspace_bytes(int64_t E, int64_t T);
int l1attn_sparse_plan_build(const int32_t* coo, int64_t coo_stride, int64_t E, int64_t T,
                             void* plan, size_t plan_bytes,
                             void* workspace, size_t workspace_bytes, void* stream);
int l1attn_sparse_plan_check(const void* plan, int64_t E, int64_t T, int32_t* header_host, void* stream);

/* ----------------------------------------------------------------------------- sparse */

/*
 * Sparse L1 attention over an edge list (plan from l1attn_sparse_plan_build for the same E, T):
 *   a_c = -1/sqrt(W) * sum_w |q[b,dst_c,h,w] - k[b,src_c,h,w]|
 *   p_c = exp(a_c) / (1 + sum_{c': dst_c' = dst_c} exp(a_c'))   if use_softmax, else exp(a_c)
 *   vo[b,dst,h,:] = sum_{c: dst_c = dst} p_c * v[b,src_c,h,:]        (0 for a dst without edges)
 * Replaces l1attn_sparse_cuda_drv.forward(v,q,k,coo,dst_mxlen,use_softmax) -> [vo, attn]
 * (cuda/l1attn_sparse_cuda_drv.cpp:32-46, kernels cuda/l1attn_sparse_cuda_kernel.cu:27-181,
 * launcher :373-445; CPU twin cpp/l1attn_sparse_drv.cpp:13-91).
 * q,k [B,T,H,W]; v,vo [B,T,H,Wv].  P [B,E,H] receives the edge weights p_c in plan slot order; it
 * is the saved-for-backward tensor that the reference returns as the padded `attn`
 * [B,T,dst_mxlen,H].  dst_mxlen is not needed: segments carry their own length.
 * Limits: max(W,Wv) <= 1024 when both are multiples of 4 and all pointers 16-byte aligned,
 * else <= 256 (L1ATTN_ERR_RANGE beyond).
 */
int l1attn_sparse_fwd_f32(const float* v, const float* q, const float* k, const void* plan,
                          float* vo, float* P,
                          int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                          int use_softmax, void* stream);
int l1attn_sparse_fwd_f64(const double* v, const double* q, const double* k, const void* plan,
                          double* vo, double* P,
                          int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                          int use_softmax, void* stream);

/*
 * Backward of the above: dv[b,src] = sum p_c*dvo[b,dst]; dp_c = v[b,src].dvo[b,dst];
 * da_c = p_c*(dp_c - sum_c' p_c' dp_c') (softmax) or p_c*dp_c; dq[b,dst] += scale*sign(q-k)*da_c;
 * dk[b,src] -= scale*sign(q-k)*da_c.  Replaces l1attn_sparse_cuda_drv.backward(dvo,v,q,k,coo,attn,
 * dst_mxlen,use_softmax) -> [dv,dq,dk] (cuda/l1attn_sparse_cuda_drv.cpp:48-69, kernels
 * cuda/l1attn_sparse_cuda_kernel.cu:183-370, launcher :447-531; CPU twin
 * cpp/l1attn_sparse_drv.cpp:93-190; the O(dst_mxlen^2) Jacobian loop :152-167 is evaluated in closed
 * form).  DA [B,E,H] is scratch for da_c (caller-owned, contents undefined on return).
 * Deterministic: no atomics.
 */
int l1attn_sparse_bwd_f32(const float* dvo, const float* v, const float* q, const float* k,
                          const void* plan, const float* P,
                          float* dv, float* dq, float* dk, float* DA,
                          int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                          int use_softmax, void* stream);
int l1attn_sparse_bwd_f64(const double* dvo, const double* v, const double* q, const double* k,
                          const void* plan, const double* P,
                          double* dv, double* dq, double* dk, double* DA,
                          int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                          int use_softmax, void* stream);

/*
 * Bidirectional variant: vo[b,dst] += p_c*vf[b,src] and vo[b,src] += p_c*vb[b,dst]; backward
 * dvf[b,src] += p_c*dvo[b,dst], dvb[b,dst] += p_c*dvo[b,src],
 * dp_c = vf[b,src].dvo[b,dst] + vb[b,dst].dvo[b,src]; dq, dk as above.
 * Replaces l1attn_sparse_bidi_cuda_drv.forward / .backward
 * (cuda/l1attn_sparse_bidi_cuda_drv.cpp:34-80, kernels cuda/l1attn_sparse_cuda_kernel.cu:535-649,
 * launchers :651-815; CPU twin cpp/l1attn_sparse_bidi_drv.cpp:15-212).
 */
int l1attn_sparse_bidi_fwd_f32(const float* vf, const float* vb, const float* q, const float* k,
                               const void* plan, float* vo, float* P,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                               int use_softmax, void* stream);
int l1attn_sparse_bidi_fwd_f64(const double* vf, const double* vb, const double* q, const double* k,
                               const void* plan, double* vo, double* P,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                               int use_softmax, void* stream);
int l1attn_sparse_bidi_bwd_f32(const float* dvo, const float* vf, const float* vb, const float* q,
                               const float* k, const void* plan, const float* P,
                               float* dvf, float* dvb, float* dq, float* dk, float* DA,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                               int use_softmax, void* stream);
int l1attn_sparse_bidi_bwd_f64(const double* dvo, const double* vf, const double* vb, const double* q,
                               const double* k, const void* plan, const double* P,
                               double* dvf, double* dvb, double* dq, double* dk, double* DA,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                               int use_softmax, void* stream);

/*
 * The two forwards with 16-bit rows: v/vf, vb, q, k and vo are IEEE binary16 (f16) or bfloat16
 * (bf16) in memory, 2 bytes per element, in the layouts above.  Logits, softmax and value sums run
 * in fp32; vo is rounded to nearest even once on store (bidi: once after the dst pass and once
 * after the src pass adds its sum); P [B,E,H] is fp32.  Same limits and return codes as the f32
 * entry points; 16-byte aligned pointers with W and Wv multiples of 4 take the vector path.
 * Replaces the Half instantiation of the reference's forward launchers
 * (AT_DISPATCH_FLOATING_TYPES_AND_HALF, cuda/l1attn_sparse_cuda_kernel.cu:405-435 and :684-714),
 * which computes every step in half precision.  bfloat16 is an addition, and so are the 16-bit
 * backwards below.
 */
int l1attn_sparse_fwd_f16(const void* v, const void* q, const void* k, const void* plan,
                          void* vo, float* P,
                          int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                          int use_softmax, void* stream);
int l1attn_sparse_fwd_bf16(const void* v, const void* q, const void* k, const void* plan,
                           void* vo, float* P,
                           int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                           int use_softmax, void* stream);
int l1attn_sparse_bidi_fwd_f16(const void* vf, const void* vb, const void* q, const void* k,
                               const void* plan, void* vo, float* P,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                               int use_softmax, void* stream);
int l1attn_sparse_bidi_fwd_bf16(const void* vf, const void* vb, const void* q, const void* k,
                                const void* plan, void* vo, float* P,
                                int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                                int use_softmax, void* stream);

/*
 * The two backwards with 16-bit rows: dvo, v/vf, vb, q, k and the gradients are binary16 or bfloat16 in
 * memory; P (from the 16-bit forward) and the scratch DA are fp32, every sum runs in fp32, each gradient
 * element is rounded to nearest even once on store.  No counterpart in the reference, whose backward
 * launchers dispatch float and double only (cuda/l1attn_sparse_cuda_kernel.cu:483-519, :765-803); for
 * mixed-precision training on the gather-bound path (six of the eight row gathers per edge are here).
 */
int l1attn_sparse_bwd_f16(const void* dvo, const void* v, const void* q, const void* k, const void* plan,
                          const float* P, void* dv, void* dq, void* dk, float* DA,
                          int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                          int use_softmax, void* stream);
int l1attn_sparse_bwd_bf16(const void* dvo, const void* v, const void* q, const void* k, const void* plan,
                           const float* P, void* dv, void* dq, void* dk, float* DA,
                           int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                           int use_softmax, void* stream);
int l1attn_sparse_bidi_bwd_f16(const void* dvo, const void* vf, const void* vb, const void* q, const void* k,
                               const void* plan, const float* P,
                               void* dvf, void* dvb, void* dq, void* dk, float* DA,
                               int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                               int use_softmax, void* stream);
int l1attn_sparse_bidi_bwd_bf16(const void* dvo, const void* vf, const void* vb, const void* q, const void* k,
                                const void* plan, const float* P,
                                void* dvf, void* dvb, void* dq, void* dk, float* DA,
                                int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                                int use_softmax, void* stream);

/* ------------------------------------------- measurement aids (bench.py only) */
/*
 * Not part of the operator boundary and no counterpart in the reference: nothing in the operators calls
 * these, a binding of the reference would not declare them.  They time instruction issue rates on the GPU at
 * hand so that the bench line can state what its roofline denominator means on that box.
 */
/*
 * A register-only loop of independent,
 * non-packed v_fmac_f32 (blocks workgroups of 512 threads, every wave issues iters*64 of them),
 * to time what the fp32 VALU of the GPU at hand sustains for ordinary code against the nominal
 * one instruction per SIMD every two cycles.  out: blocks*512 floats.  Asynchronous.
 */
int l1attn_probe_valu(float* out, int64_t blocks, int64_t iters, void* stream);
/*
 * The same probe for other instructions (same geometry and accounting), to learn an instruction's
 * issue rate before a kernel is built on it: op 0 = v_fmac_f32 (as above), 1 = v_sad_u32 (|a-b|+c on
 * unsigned integers in one instruction) on VGPRs, 2 = v_sad_u32 with an SGPR operand, 3 = pairs of
 * v_sub_f32 and v_add_f32 |x| (2 instructions per counted step).  No counterpart in the reference.
 */
int l1attn_probe_valu_op(float* out, int64_t blocks, int64_t iters, int op, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* L1ATTN_HIP_H */
