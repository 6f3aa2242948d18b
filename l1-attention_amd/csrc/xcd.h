// Placement of workgroups on the eight XCDs of an MI355X.
#pragma once
#include <hip/hip_runtime.h>

// Workgroups are handed to the 8 XCDs round-robin in dispatch order, and each XCD has its own L2.
// This maps the flat dispatch index to a logical one such that logically consecutive workgroups
// (which share k rows) land on the same XCD: XCD x runs the logical range [x*n/8, (x+1)*n/8).
struct LogicalBlock { int x, y, z; };
__device__ __forceinline__ LogicalBlock xcd_remap()
{
	const unsigned nx = gridDim.x, ny = gridDim.y, n = nx * ny * gridDim.z;
	const unsigned flat = blockIdx.x + nx * (blockIdx.y + ny * blockIdx.z);
	const unsigned per = n / 8u;
	unsigned m = flat;
	if (flat < per * 8u) m = (flat % 8u) * per + flat / 8u;
	LogicalBlock lb;
	lb.x = (int)(m % nx);
	lb.y = (int)((m / nx) % ny);
	lb.z = (int)(m / (nx * ny));
	return lb;
}
