// Library identification, and a probe of what the fp32 VALU of this GPU gives to ordinary code.
#include "common.h"

extern "C" int l1attn_version(void) { return 100; }

namespace {

// Register-only loop: every wave issues `iters` x 64 independent non-packed fp32 instructions (v_fmac_f32 on four
// accumulators).  No memory traffic inside the loop; each thread stores one float at the end.
__global__ __launch_bounds__(512) void probe_valu_loop(float* __restrict__ out, int iters, float s)
{
	float a0 = threadIdx.x, a1 = a0 + 1.0f, a2 = a0 + 2.0f, a3 = a0 + 3.0f;
	const float b = s * 0.5f;
	for (int i = 0; i < iters; i++) {
#pragma unroll
		for (int u = 0; u < 16; u++)
			asm volatile("v_fmac_f32 %0, %4, %5\n\tv_fmac_f32 %1, %4, %5\n\tv_fmac_f32 %2, %4, %5\n\tv_fmac_f32 %3, %4, %5"
			             : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
			             : "v"(b), "v"(s));
	}
	out[blockIdx.x * blockDim.x + threadIdx.x] = (a0 + a1) + (a2 + a3);
}

}  // namespace

// Launches the probe: `blocks` workgroups of 512 threads (8 waves, two per SIMD when one workgroup sits on a CU),
// each wave issuing iters*64 VALU instructions.  `out` holds blocks*512 floats.  Asynchronous on the stream; the
// caller times it.  Wave-instructions issued = blocks * 8 * iters * 64.
extern "C" int l1attn_probe_valu(float* out, int64_t blocks, int64_t iters, void* stream)
{
	if (!out || blocks < 1 || blocks > 65535 || iters < 1 || iters > (1 << 24)) return L1ATTN_ERR_ARG;
	hipLaunchKernelGGL(probe_valu_loop, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, out, (int)iters, 1.0f);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}
