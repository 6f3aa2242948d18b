// Library identification, and a probe of what the fp32 VALU of this GPU gives to ordinary code.
#include "common.h"

extern "C" int l1attn_version(void) { return 10100; }  // 1.1.0: fused operator, 16-bit sparse forwards, probes

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

// The same loop for other instructions, to learn their issue rate before a kernel is built on them:
//   OP 1: v_sad_u32 (|a - b| + c on unsigned integers in one instruction), VGPR operands
//   OP 2: v_sad_u32 with the second operand in an SGPR
//   OP 3: v_sub_f32 followed by v_add_f32 with |x| (two instructions per step instead of one)
// Every wave issues iters x 64 instructions (OP 3: iters x 64 pairs).
template <int OP>
__global__ __launch_bounds__(512) void probe_op_loop(float* __restrict__ out, int iters, int s, float sf)
{
	unsigned a0 = threadIdx.x, a1 = a0 + 1, a2 = a0 + 2, a3 = a0 + 3;
	const unsigned b = threadIdx.x * 3u + 7u;
	float f0 = threadIdx.x, f1 = f0 + 1.0f, f2 = f0 + 2.0f, f3 = f0 + 3.0f, d0, d1, d2, d3;
	const float fb = (float)threadIdx.x * 0.5f;
	for (int i = 0; i < iters; i++) {
#pragma unroll
		for (int u = 0; u < 16; u++) {
			if (OP == 1)
				asm volatile("v_sad_u32 %0, %4, %5, %0\n\tv_sad_u32 %1, %4, %5, %1\n\tv_sad_u32 %2, %4, %5, %2\n\t"
				             "v_sad_u32 %3, %4, %5, %3"
				             : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
				             : "v"(b), "v"(s));
			else if (OP == 2)
				asm volatile("v_sad_u32 %0, %4, %5, %0\n\tv_sad_u32 %1, %4, %5, %1\n\tv_sad_u32 %2, %4, %5, %2\n\t"
				             "v_sad_u32 %3, %4, %5, %3"
				             : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
				             : "v"(b), "s"(s));
			else
				asm volatile("v_sub_f32 %4, %9, %8\n\tv_sub_f32 %5, %9, %8\n\tv_sub_f32 %6, %9, %8\n\t"
				             "v_sub_f32 %7, %9, %8\n\t"
				             "v_add_f32 %0, %0, |%4|\n\tv_add_f32 %1, %1, |%5|\n\tv_add_f32 %2, %2, |%6|\n\t"
				             "v_add_f32 %3, %3, |%7|"
				             : "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3), "=&v"(d0), "=&v"(d1), "=&v"(d2), "=&v"(d3)
				             : "v"(fb), "s"(sf));
		}
	}
	out[blockIdx.x * blockDim.x + threadIdx.x] =
	    OP == 3 ? (f0 + f1) + (f2 + f3) : (float)((a0 + a1) + (a2 + a3));
}

}  // namespace

// The probe for another instruction: op 0 = v_fmac_f32 (as l1attn_probe_valu), 1 = v_sad_u32 on VGPRs,
// 2 = v_sad_u32 with an SGPR operand, 3 = v_sub_f32 + v_add_f32 |x| pairs.  Same geometry and accounting.
extern "C" int l1attn_probe_valu(float* out, int64_t blocks, int64_t iters, void* stream);
extern "C" int l1attn_probe_valu_op(float* out, int64_t blocks, int64_t iters, int op, void* stream)
{
	if (!out || blocks < 1 || blocks > 65535 || iters < 1 || iters > (1 << 24) || op < 0 || op > 3) return L1ATTN_ERR_ARG;
	if (op == 0) return l1attn_probe_valu(out, blocks, iters, stream);
	const dim3 grid((unsigned)blocks), block(512);
	hipStream_t st = (hipStream_t)stream;
	if (op == 1) hipLaunchKernelGGL(probe_op_loop<1>, grid, block, 0, st, out, (int)iters, 5, 0.25f);
	else if (op == 2) hipLaunchKernelGGL(probe_op_loop<2>, grid, block, 0, st, out, (int)iters, 5, 0.25f);
	else hipLaunchKernelGGL(probe_op_loop<3>, grid, block, 0, st, out, (int)iters, 5, 0.25f);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

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
