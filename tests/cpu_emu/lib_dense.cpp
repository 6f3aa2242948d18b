// TEST INFRASTRUCTURE: csrc/dense.hip compiled for the host as one object of the emulated library
// (tests/test_emulated_library_cpu.py): its extern "C" entry points are the product's, the kernels run as OS threads.
#include "emu_gfx950.h"
#include "../../l1-attention_amd/csrc/dense.hip"
