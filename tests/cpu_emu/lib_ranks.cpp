// TEST INFRASTRUCTURE: the merge-sort column-rank kernel (csrc/rank_sort.hip) as it is, for the emulated library.
#include "hip/hip_runtime.h"
#include "../../l1-attention_amd/csrc/rank_sort.hip"
