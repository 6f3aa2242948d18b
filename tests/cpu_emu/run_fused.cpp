// TEST INFRASTRUCTURE: runs l1attn_fused_fwd_f32 / _f64 of csrc/fused.hip, compiled for the host with
// the stand-in header next to this file, on inputs read from a file, and writes vo and lse.
//   run_fused <in> <out> <f32|f64> <misalign> [pipe]      (pipe: l1attn_fused_fwd_pipe_f32 and l1attn_fused_bwd_stage_pipe_f32)
// in : int64 B,T,H,W,Wv then q,k [B,T,H,W], v [B,T,H,Wv] and dvo [B,T,H,Wv] in the chosen type
// out: vo [B,T,H,Wv], lse [B,T,H], one int64 (threads the forward ran), then the backward's first stage on
//      the forward's own vo and lse: dA [B,T,T,H], dv [B,T,H,Wv], one int64 (threads it ran)
// Buffers are malloc'ed at their exact sizes, so AddressSanitizer reports any access outside them.
// misalign = 1 offsets every buffer by one element (the library then has to take its generic kernel).
#include "hip/hip_runtime.h"

#include "emu_sload.h"

#include "../../l1-attention_amd/csrc/fused.hip"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

template <typename T>
static int run(FILE* fi, FILE* fo, const int64_t* d, bool f32, int mis, bool pipe)
{
	const int64_t B = d[0], Tn = d[1], H = d[2], W = d[3], Wv = d[4];
	const size_t nq = (size_t)(B * Tn * H * W), nv = (size_t)(B * Tn * H * Wv), nl = (size_t)(B * Tn * H);
	auto alloc = [&](size_t n) { return (T*)aligned_alloc(16, ((n + mis) * sizeof(T) + 15) / 16 * 16) + mis; };
	T *q = alloc(nq), *k = alloc(nq), *v = alloc(nv), *vo = alloc(nv), *lse = alloc(nl);
	if (fread(q, sizeof(T), nq, fi) != nq || fread(k, sizeof(T), nq, fi) != nq || fread(v, sizeof(T), nv, fi) != nv)
		return 3;
	int rc;
	if (f32 && pipe) rc = l1attn_fused_fwd_pipe_f32((const float*)q, (const float*)k, (const float*)v, (float*)vo,
	                                                (float*)lse, B, Tn, H, W, Wv, nullptr);
	else if (f32) rc = l1attn_fused_fwd_f32((const float*)q, (const float*)k, (const float*)v, (float*)vo, (float*)lse, B,
	                                        Tn, H, W, Wv, nullptr);
	else rc = l1attn_fused_fwd_f64((const double*)q, (const double*)k, (const double*)v, (double*)vo, (double*)lse,
	                               B, Tn, H, W, Wv, nullptr);
	if (rc) return 10 + (rc < 0 ? -rc : rc);
	if (emu_sload::outstanding != 0) return 9;  // a wave ended with a scalar prefetch in flight
	fwrite(vo, sizeof(T), nv, fo);
	fwrite(lse, sizeof(T), nl, fo);
	int64_t n = emu::n_threads_run;
	fwrite(&n, sizeof(n), 1, fo);
	const size_t na = (size_t)(B * Tn * Tn * H);
	T *dvo = alloc(nv), *dA = alloc(na), *dv = alloc(nv);
	if (fread(dvo, sizeof(T), nv, fi) != nv) return 3;
	emu::n_threads_run = 0;
	if (f32 && pipe) rc = l1attn_fused_bwd_stage_pipe_f32((const float*)dvo, (const float*)q, (const float*)k, (const float*)v,
	                                                      (const float*)vo, (const float*)lse, (float*)dA, (float*)dv, B, Tn,
	                                                      H, W, Wv, nullptr);
	else if (f32) rc = l1attn_fused_bwd_stage_f32((const float*)dvo, (const float*)q, (const float*)k, (const float*)v,
	                                         (const float*)vo, (const float*)lse, (float*)dA, (float*)dv, B, Tn, H, W,
	                                         Wv, nullptr);
	else rc = l1attn_fused_bwd_stage_f64((const double*)dvo, (const double*)q, (const double*)k, (const double*)v,
	                                     (const double*)vo, (const double*)lse, (double*)dA, (double*)dv, B, Tn, H, W,
	                                     Wv, nullptr);
	if (rc) return 20 + (rc < 0 ? -rc : rc);
	if (emu_sload::outstanding != 0) return 9;
	fwrite(dA, sizeof(T), na, fo);
	fwrite(dv, sizeof(T), nv, fo);
	n = emu::n_threads_run;
	fwrite(&n, sizeof(n), 1, fo);
	free(q - mis); free(k - mis); free(v - mis); free(vo - mis); free(lse - mis);
	free(dvo - mis); free(dA - mis); free(dv - mis);
	return 0;
}

int main(int argc, char** argv)
{
	if (argc != 5 && argc != 6) return 2;
	const bool pipe = argc == 6 && strcmp(argv[5], "pipe") == 0;
	FILE* fi = fopen(argv[1], "rb");
	FILE* fo = fopen(argv[2], "wb");
	if (!fi || !fo) return 2;
	int64_t d[5];
	if (fread(d, sizeof(int64_t), 5, fi) != 5) return 3;
	const bool f32 = strcmp(argv[3], "f32") == 0;
	const int mis = atoi(argv[4]);
	const int rc = f32 ? run<float>(fi, fo, d, true, mis, pipe) : run<double>(fi, fo, d, false, mis, pipe);
	fclose(fi);
	fclose(fo);
	return rc;
}
