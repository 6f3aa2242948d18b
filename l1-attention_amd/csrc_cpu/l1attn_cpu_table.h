// Function table of one compiled copy of the CPU kernels (l1attn_cpu_kernels.cpp is compiled once per
// instruction set); l1attn_cpu.cpp dispatches through the copy the processor supports.
#ifndef L1ATTN_CPU_TABLE_H
#define L1ATTN_CPU_TABLE_H
#include <cstdint>

struct L1CpuTable {
	void (*dense_fwd_f32)(const float*, const float*, float*, int64_t, int64_t, int64_t, int64_t, int);
	void (*dense_fwd_f64)(const double*, const double*, double*, int64_t, int64_t, int64_t, int64_t, int);
	void (*dense_bwd_f32)(const float*, const float*, const float*, float*, float*, int64_t, int64_t, int64_t, int64_t, int);
	void (*dense_bwd_f64)(const double*, const double*, const double*, double*, double*, int64_t, int64_t, int64_t, int64_t,
	                      int);
	void (*sparse_fwd_f32)(const float*, const float*, const float*, const float*, const int32_t*, int64_t, float*, float*,
	                       int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, bool, bool, int);
	void (*sparse_fwd_f64)(const double*, const double*, const double*, const double*, const int32_t*, int64_t, double*,
	                       double*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, bool, bool, int);
	void (*bidi_fwd_f32)(const float*, const float*, const float*, const float*, const int32_t*, int64_t, float*, float*,
	                     int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, bool, bool, int);
	void (*bidi_fwd_f64)(const double*, const double*, const double*, const double*, const int32_t*, int64_t, double*,
	                     double*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, bool, bool, int);
	void (*sparse_bwd_f32)(const float*, const float*, const float*, const float*, const float*, const int32_t*, int64_t,
	                       const float*, float*, float*, float*, float*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
	                       int64_t, bool, int);
	void (*sparse_bwd_f64)(const double*, const double*, const double*, const double*, const double*, const int32_t*, int64_t,
	                       const double*, double*, double*, double*, double*, int64_t, int64_t, int64_t, int64_t, int64_t,
	                       int64_t, int64_t, bool, int);
	void (*bidi_bwd_f32)(const float*, const float*, const float*, const float*, const float*, const int32_t*, int64_t,
	                     const float*, float*, float*, float*, float*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
	                     int64_t, bool, int);
	void (*bidi_bwd_f64)(const double*, const double*, const double*, const double*, const double*, const int32_t*, int64_t,
	                     const double*, double*, double*, double*, double*, int64_t, int64_t, int64_t, int64_t, int64_t,
	                     int64_t, int64_t, bool, int);
	void (*fused_fwd_f32)(const float*, const float*, const float*, float*, float*, int64_t, int64_t, int64_t, int64_t,
	                      int64_t, int);
	void (*fused_fwd_f64)(const double*, const double*, const double*, double*, double*, int64_t, int64_t, int64_t, int64_t,
	                      int64_t, int);
	void (*fused_bwd_f32)(const float*, const float*, const float*, const float*, const float*, const float*, float*, float*,
	                      float*, int64_t, int64_t, int64_t, int64_t, int64_t, int);
	void (*fused_bwd_f64)(const double*, const double*, const double*, const double*, const double*, const double*, double*,
	                      double*, double*, int64_t, int64_t, int64_t, int64_t, int64_t, int);
};

extern const L1CpuTable l1cpu_table_l1cpu_generic;
extern const L1CpuTable l1cpu_table_l1cpu_avx2;
#endif
