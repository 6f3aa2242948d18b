// TEST INFRASTRUCTURE: runs the column-rank kernel of csrc/dense_rank.hip (the one the backward uses by default),
// compiled for the host with the stand-in headers next to this file: GPU threads are OS threads, and the library
// block sort it calls is the stand-in of rocprim/block/block_radix_sort.hpp here.  Everything around the sort --
// the order-preserving keys, the padding, the remapped column order, the searches and both rank formulas -- is the
// kernel's own source.
//   run_ranks_lib <in> <out>
// in : int64 B,T,H,W then q,k [B,T,H,W] float32        out: rq, rk [B,T,H,W] float32
// Buffers are malloc'ed at their exact sizes, so AddressSanitizer reports any access outside them.
#include "../../l1-attention_amd/csrc/dense_rank.hip"
#include <stdio.h>
#include <stdlib.h>

int main(int argc, char** argv)
{
	if (argc != 3) return 2;
	FILE* fi = fopen(argv[1], "rb");
	FILE* fo = fopen(argv[2], "wb");
	if (!fi || !fo) return 2;
	int64_t d[4];
	if (fread(d, sizeof(int64_t), 4, fi) != 4) return 3;
	const int64_t B = d[0], T = d[1], H = d[2], W = d[3];
	const size_t n = (size_t)(B * T * H * W);
	float* q = (float*)malloc(n * 4);
	float* k = (float*)malloc(n * 4);
	float* rq = (float*)malloc(n * 4);
	float* rk = (float*)malloc(n * 4);
	if (fread(q, 4, n, fi) != n || fread(k, 4, n, fi) != n) return 3;
	const int rc = l1attn_dense_column_ranks_f32(q, k, rq, rk, B, T, H, W, nullptr);
	if (rc) return 10 + (rc < 0 ? -rc : rc);
	fwrite(rq, 4, n, fo);
	fwrite(rk, 4, n, fo);
	fclose(fi);
	fclose(fo);
	free(q); free(k); free(rq); free(rk);
	return 0;
}
