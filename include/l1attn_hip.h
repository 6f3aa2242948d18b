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
 * dq[b,t,h,w] =  sum_s scale*sign(q[b,t,h,w]-k[b,s,h,w]) * d_attn[b,s,t,h]
 * dk[b,s,h,w] = -sum_t scale*sign(q[b,t,h,w]-k[b,s,h,w]) * d_attn[b,s,t,h],   sign(0) = 0.
 * Replaces l1attn_cuda_drv.backward(d_attn,q,k) -> [dq,dk]  (cuda/l1attn_cuda_drv.cpp:67-104,
 * kernels cuda/l1attn_cuda_kernel.cu:206-455; CPU twin cpp/l1attn_drv.cpp:57-98).
 * d_attn is read in its native [B,S,T,H] layout.  Deterministic: no atomics; dk is summed
 * from per-dst-tile partials held in `workspace` (device memory, 256-byte aligned, at least
 * l1attn_dense_bwd_workspace_bytes() for full speed; any multiple of one batch's share works,
 * the batches are then processed in several launches).  The f64 entry needs no workspace.
 * f32 fast path: sign() is taken from (q-k)*2^64, exact for |q|,|k| < 2^63 and differences
 * that are 0 or at least 2^-64 in magnitude.
 */
size_t l1attn_dense_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t W);
int l1attn_dense_bwd_f32(const float* d_attn, const float* q, const float* k, float* dq, float* dk,
                         int64_t B, int64_t T, int64_t H, int64_t W,
                         void* workspace, size_t workspace_bytes, void* stream);
int l1attn_dense_bwd_f64(const double* d_attn, const double* q, const double* k, double* dq, double* dk,
                         int64_t B, int64_t T, int64_t H, int64_t W,
                         void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* L1ATTN_HIP_H */
