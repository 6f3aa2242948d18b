// TEST INFRASTRUCTURE: runs the edge-list entry points of csrc/coo.hip (l1attn_expand_coo, l1attn_sparse_plan_build,
// l1attn_sparse_plan_check) compiled for the host with the stand-in header next to this file: GPU threads are OS
// threads, ballots, shuffles and __syncthreads() are barriers, atomics are host atomics, and the one place where
// lanes hand values to each other through LDS between two cross-lane operations (L1_WAVE_LOCKSTEP in radix_scatter)
// is a barrier among the lanes it names.
//   run_coo <in> <out>
// in : int64 mode (0 expandCoo, 1 plan), bits (32 | 64), stride, E, T; then E*stride integers of `bits` bits
// out: mode 0: int32 rc, dst_mxlen, src_mxlen, then coo [E,4]
//      mode 1: int32 rc of the build, rc of the check, the 16 header words the check returned, then the plan's words
// Every buffer is allocated at its exact size (the workspace at what the library asks for) and filled with a
// pattern first, so that AddressSanitizer reports any access outside them and nothing rests on zeroed memory.
#include "../../l1-attention_amd/csrc/coo.hip"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static void* patterned(size_t bytes)
{
	void* p = aligned_alloc(256, (bytes + 255) / 256 * 256);
	memset(p, 0xA5, (bytes + 255) / 256 * 256);
	return p;
}

int main(int argc, char** argv)
{
	if (argc != 3) return 2;
	FILE* fi = fopen(argv[1], "rb");
	FILE* fo = fopen(argv[2], "wb");
	if (!fi || !fo) return 3;
	int64_t d[5];
	if (fread(d, 8, 5, fi) != 5) return 4;
	const int64_t mode = d[0], bits = d[1], stride = d[2], E = d[3], T = d[4];
	const size_t in_bytes = (size_t)(E * stride) * (size_t)(bits / 8);
	void* co = malloc(in_bytes ? in_bytes : 1);
	if (in_bytes && fread(co, 1, in_bytes, fi) != in_bytes) return 5;
	if (mode == 0) {
		const size_t wb = l1attn_expand_coo_workspace_bytes(E);
		void* ws = patterned(wb);
		int32_t* coo = (int32_t*)malloc(E ? (size_t)E * 16 : 1);
		memset(coo, 0xA5, E ? (size_t)E * 16 : 1);
		int32_t mx[2] = {-7, -7};
		const int32_t rc = l1attn_expand_coo(E ? co : nullptr, (int)bits, stride, E, E ? coo : nullptr, mx, ws, wb, nullptr);
		fwrite(&rc, 4, 1, fo);
		fwrite(mx, 4, 2, fo);
		fwrite(coo, 4, (size_t)E * 4, fo);
		free(ws);
		free(coo);
	} else {
		if (bits != 32) return 6;
		const size_t pb = l1attn_sparse_plan_bytes(E, T), wb = l1attn_sparse_plan_workspace_bytes(E, T);
		void* plan = patterned(pb);
		void* ws = patterned(wb);
		const int32_t rc = l1attn_sparse_plan_build(E ? (const int32_t*)co : nullptr, stride, E, T, plan, pb, ws, wb, nullptr);
		int32_t hdr[PLAN_H_WORDS];
		memset(hdr, 0, sizeof(hdr));
		const int32_t rc2 = rc ? 0 : l1attn_sparse_plan_check(plan, E, T, hdr, nullptr);
		fwrite(&rc, 4, 1, fo);
		fwrite(&rc2, 4, 1, fo);
		fwrite(hdr, 4, PLAN_H_WORDS, fo);
		fwrite(plan, 1, pb, fo);
		free(plan);
		free(ws);
	}
	free(co);
	fclose(fo);
	return 0;
}
