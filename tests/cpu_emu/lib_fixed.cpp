// TEST INFRASTRUCTURE: csrc/fixed.hip for the emulated library.
#include "hip/hip_runtime.h"
#include "../../l1-attention_amd/csrc/fixed.hip"
