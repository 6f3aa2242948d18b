// TEST INFRASTRUCTURE: runs the two pre-pass kernels of the fixed-point dense forward (csrc/fixed.hip), compiled
// for the host with the stand-in header next to this file.
//   run_fixed <in> <out>
// in : int64 B,T,H,W then q,k [B,T,H,W] float32        out: gq [B*H] float32, uq, uk [B,T,H,W] uint32
#include "../../l1-attention_amd/csrc/fixed.hip"
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
	const size_t n = (size_t)(B * T * H * W), ng = (size_t)(B * H);
	float* q = (float*)malloc(n * 4);
	float* k = (float*)malloc(n * 4);
	float* gq = (float*)malloc(ng * 4);
	unsigned* uq = (unsigned*)malloc(n * 4);
	unsigned* uk = (unsigned*)malloc(n * 4);
	if (fread(q, 4, n, fi) != n || fread(k, 4, n, fi) != n) return 3;
	const int rc = l1_launch_fixed_prepass(q, k, gq, uq, uk, B, T, H, W, nullptr);
	if (rc) return 10 + (rc < 0 ? -rc : rc);
	fwrite(gq, 4, ng, fo);
	fwrite(uq, 4, n, fo);
	fwrite(uk, 4, n, fo);
	fclose(fi);
	fclose(fo);
	free(q); free(k); free(gq); free(uq); free(uk);
	return 0;
}
