/*
 * C ABI of libl1attn_cpu.so -- the host-CPU twin of the operators, standing in for the reference's
 * three CPU extension modules (cpp/setup.py:4-16: l1attn_drv_cpp, l1attn_sparse_drv,
 * l1attn_sparse_bidi_drv).  Plain pointers and sizes only; no torch types.
 *
 * This is a separate library for tensors that live in host memory.  The GPU operators
 * (libl1attn_hip.so, include/l1attn_hip.h) never call it: a GPU tensor handed to a GPU operator is
 * computed by the HIP kernels or raises.
 *
 * Conventions
 *   - All pointers are HOST pointers to contiguous row-major tensors in the reference's layouts:
 *     q,k,v,... [B,T,H,W]; attn / d_attn of the dense operator [B,S,T,H] with the src token S first;
 *     attn of the sparse operators [B,T,dst_mxlen,H], slot r = coo[c][2] of edge c as in the reference.
 *   - The caller owns every buffer.  Inputs are never written; outputs are fully overwritten.
 *   - float32 and float64 (the reference's CPU extension is float64 only: cpp/l1attn_drv.cpp:5).
 *   - Work is split over OpenMP threads by output row, every sum is formed by one thread in a fixed order:
 *     results do not depend on the thread count and repeat bit for bit.
 *   - Return value: 0, or a negative code below.  Calls are synchronous.
 */
#ifndef L1ATTN_CPU_H
#define L1ATTN_CPU_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define L1ATTN_CPU_OK 0
#define L1ATTN_CPU_ERR_ARG (-1)   /* null pointer, negative size, W < 1 */
#define L1ATTN_CPU_ERR_INDEX (-4) /* coo holds a token outside [0,T) or a slot outside [0,dst_mxlen) */

int l1attn_cpu_version(void);
/* Threads used by the calls below: n >= 1, or 0 for the OpenMP default.  Returns the previous setting. */
int l1attn_cpu_set_threads(int n);

/*
 * attn[b,s,t,h] = -1/sqrt(W) * sum_w |q[b,t,h,w] - k[b,s,h,w]|.
 * Replaces l1attn_drv_cpp.forward(q,k) -> [attn]  (cpp/l1attn_drv.cpp:13-55).
 */
int l1attn_cpu_dense_fwd_f32(const float* q, const float* k, float* attn, int64_t B, int64_t T, int64_t H, int64_t W);
int l1attn_cpu_dense_fwd_f64(const double* q, const double* k, double* attn, int64_t B, int64_t T, int64_t H, int64_t W);

/*
 * dq[b,t,h,w] =  sum_s scale*sign(q[b,t,h,w]-k[b,s,h,w]) * d_attn[b,s,t,h]
 * dk[b,s,h,w] = -sum_t scale*sign(q[b,t,h,w]-k[b,s,h,w]) * d_attn[b,s,t,h],   sign(0) = 0.
 * Replaces l1attn_drv_cpp.backward(d_attn,q,k) -> [dq,dk]  (cpp/l1attn_drv.cpp:57-98).
 */
int l1attn_cpu_dense_bwd_f32(const float* d_attn, const float* q, const float* k, float* dq, float* dk,
                             int64_t B, int64_t T, int64_t H, int64_t W);
int l1attn_cpu_dense_bwd_f64(const double* d_attn, const double* q, const double* k, double* dq, double* dk,
                             int64_t B, int64_t T, int64_t H, int64_t W);

/*
 * expandCoo: co[E, co_stride>=2] rows of [dst, src] (32- or 64-bit signed integers, any values) ->
 * coo int32 [E,4] = [dst, src, #{j<i: dst_j==dst_i}, #{j<i: src_j==src_i}], mxlen[0..1] = 1 + the largest rank of
 * each kind ({1,1} for E == 0).  Replaces the Python loop cpp/l1attn_sparse_cpp.py:61-106
 * (python/l1attn_sparse.py:382-427).  Bit-exact.  Values that do not fit int32 are an L1ATTN_CPU_ERR_INDEX.
 */
int l1attn_cpu_expand_coo(const void* co, int co_bits, int64_t co_stride, int64_t E, int32_t* coo, int32_t* mxlen);

/*
 * Sparse forward: a_c = -1/sqrt(W) * sum_w |q[b,dst_c,h,w] - k[b,src_c,h,w]|,
 * p_c = exp(a_c) / (1 + sum over the edges of dst_c of exp(a))  (use_softmax) or exp(a_c),
 * vo[b,dst,h,:] = sum_c p_c v[b,src_c,h,:];  attn[b,dst,coo[c][2],h] = p_c, every other slot 0.
 * Replaces l1attn_sparse_drv.forward(v,q,k,coo,dst_mxlen,use_softmax) -> [vo, attn]
 * (cpp/l1attn_sparse_drv.cpp:13-91).  coo int32 [E, coo_stride>=3].  v, vo [B,T,H,Wv]: Wv may differ from W
 * (the reference's CUDA kernels allow it, cuda/l1attn_sparse_cuda_kernel.cu:385; its CPU loop does not).
 * attn_zeroed != 0: the caller hands over attn holding zeros (e.g. calloc'ed) and only the slots of the edges are
 * written; on a skewed graph the padded tensor is mostly empty slots (2 GB at 65536 tokens, dst_mxlen 2049, 4
 * heads) and clearing it would dominate the call.  attn_zeroed == 0: every slot is written.
 */
int l1attn_cpu_sparse_fwd_f32(const float* v, const float* q, const float* k, const int32_t* coo, int64_t coo_stride,
                              float* vo, float* attn, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv,
                              int64_t E, int64_t dst_mxlen, int use_softmax, int attn_zeroed);
int l1attn_cpu_sparse_fwd_f64(const double* v, const double* q, const double* k, const int32_t* coo, int64_t coo_stride,
                              double* vo, double* attn, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv,
                              int64_t E, int64_t dst_mxlen, int use_softmax, int attn_zeroed);

/*
 * Sparse backward -> dv, dq, dk.  Replaces l1attn_sparse_drv.backward(dvo,v,q,k,coo,attn,dst_mxlen,use_softmax)
 * (cpp/l1attn_sparse_drv.cpp:93-190); the softmax Jacobian product, an O(dst_mxlen^2) loop there (:152-167), is
 * evaluated as da_c = p_c * (dp_c - sum_c' p_c' dp_c') over the edges of the dst.
 */
int l1attn_cpu_sparse_bwd_f32(const float* dvo, const float* v, const float* q, const float* k, const int32_t* coo,
                              int64_t coo_stride, const float* attn, float* dv, float* dq, float* dk,
                              int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t dst_mxlen,
                              int use_softmax);
int l1attn_cpu_sparse_bwd_f64(const double* dvo, const double* v, const double* q, const double* k, const int32_t* coo,
                              int64_t coo_stride, const double* attn, double* dv, double* dq, double* dk,
                              int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t dst_mxlen,
                              int use_softmax);

/*
 * Bidirectional variant: vo[b,dst] += p_c vf[b,src], vo[b,src] += p_c vb[b,dst]; backward dvf, dvb, dq, dk with
 * dp_c = vf[b,src].dvo[b,dst] + vb[b,dst].dvo[b,src].  Replaces l1attn_sparse_bidi_drv.forward / .backward
 * (cpp/l1attn_sparse_bidi_drv.cpp:15-212).
 */
int l1attn_cpu_sparse_bidi_fwd_f32(const float* vf, const float* vb, const float* q, const float* k, const int32_t* coo,
                                   int64_t coo_stride, float* vo, float* attn, int64_t B, int64_t T, int64_t H, int64_t W,
                                   int64_t Wv, int64_t E, int64_t dst_mxlen, int use_softmax, int attn_zeroed);
int l1attn_cpu_sparse_bidi_fwd_f64(const double* vf, const double* vb, const double* q, const double* k,
                                   const int32_t* coo, int64_t coo_stride, double* vo, double* attn, int64_t B, int64_t T,
                                   int64_t H, int64_t W, int64_t Wv, int64_t E, int64_t dst_mxlen, int use_softmax,
                                   int attn_zeroed);
int l1attn_cpu_sparse_bidi_bwd_f32(const float* dvo, const float* vf, const float* vb, const float* q, const float* k,
                                   const int32_t* coo, int64_t coo_stride, const float* attn, float* dvf, float* dvb,
                                   float* dq, float* dk, int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv, int64_t E,
                                   int64_t dst_mxlen, int use_softmax);
int l1attn_cpu_sparse_bidi_bwd_f64(const double* dvo, const double* vf, const double* vb, const double* q,
                                   const double* k, const int32_t* coo, int64_t coo_stride, const double* attn,
                                   double* dvf, double* dvb, double* dq, double* dk, int64_t B, int64_t T, int64_t H,
                                   int64_t W, int64_t Wv, int64_t E, int64_t dst_mxlen, int use_softmax);

/*
 * Fused operator: dense L1 logits, softmax over the src tokens with the no-op zero logit, value sum, without the
 * [B,S,T,H] logits -- the composition of example-setfind/setfind.py:128-136 (the reference has no single function
 * for it; README.md:21 asks for it).  vo[b,t,h,:] = sum_s e^{a[s]} v[b,s,h,:] / (1 + sum_s e^{a[s]}),
 * lse[b,t,h] = log(1 + sum_s e^{a[s]}) (lse may be NULL in the forward).  The backward takes the forward's vo and
 * lse and returns dq, dk, dv; it holds no [T,T] tensor either (the logits are recomputed in two sweeps).
 * q,k [B,T,H,W]; v, vo, dvo, dv [B,T,H,Wv].  The host twin of l1attn_fused_fwd_* / l1attn_fused_bwd_stage_* of the
 * GPU library.
 */
int l1attn_cpu_fused_fwd_f32(const float* q, const float* k, const float* v, float* vo, float* lse,
                             int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv);
int l1attn_cpu_fused_fwd_f64(const double* q, const double* k, const double* v, double* vo, double* lse,
                             int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv);
int l1attn_cpu_fused_bwd_f32(const float* dvo, const float* q, const float* k, const float* v, const float* vo,
                             const float* lse, float* dq, float* dk, float* dv,
                             int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv);
int l1attn_cpu_fused_bwd_f64(const double* dvo, const double* q, const double* k, const double* v, const double* vo,
                             const double* lse, double* dq, double* dk, double* dv,
                             int64_t B, int64_t T, int64_t H, int64_t W, int64_t Wv);

#ifdef __cplusplus
}
#endif
#endif /* L1ATTN_CPU_H */
