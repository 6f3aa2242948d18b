// TEST INFRASTRUCTURE: the default column-rank kernel (csrc/dense_rank.hip) as it is, for the emulated library; the
// library block sort it calls is the host stand-in of rocprim/block/block_radix_sort.hpp in this folder.
#include "hip/hip_runtime.h"
#include "../../l1-attention_amd/csrc/dense_rank.hip"
