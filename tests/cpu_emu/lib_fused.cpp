// TEST INFRASTRUCTURE: csrc/fused.hip for the emulated library.
#include "hip/hip_runtime.h"
#include "emu_sload.h"
#include "../../l1-attention_amd/csrc/fused.hip"
