// Shared host-side helpers for the gfx950 L1-attention library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

// Return codes of every extern "C" entry point (mirrored in include/l1attn_hip.h).
#define L1ATTN_OK 0
#define L1ATTN_ERR_ARG (-1)        // null pointer, negative size, unsupported dtype code
#define L1ATTN_ERR_WORKSPACE (-2)  // workspace missing or too small
#define L1ATTN_ERR_RANGE (-3)      // size beyond what the kernels index (e.g. > 2^31-1 rows)
#define L1ATTN_ERR_INDEX (-4)      // edge list holds an index outside [0, T)
// positive values: hipError_t of a failed launch / runtime call

#define L1_HIP_CHECK(expr)                         \
	do {                                           \
		hipError_t e__ = (expr);                   \
		if (e__ != hipSuccess) return (int)e__;    \
	} while (0)

#define L1_LAUNCH_CHECK()                          \
	do {                                           \
		hipError_t e__ = hipGetLastError();        \
		if (e__ != hipSuccess) return (int)e__;    \
	} while (0)

static inline int64_t l1_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t l1_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
