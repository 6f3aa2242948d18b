// TEST INFRASTRUCTURE: csrc/sparse.hip for the emulated library (its kernels declare their LDS as one dynamic
// array, defined here).
#define EMU_DYNAMIC_LDS_ONLY
#include "../../l1-attention_amd/csrc/sparse.hip"
namespace { alignas(16) unsigned char smem_raw[65536]; }
