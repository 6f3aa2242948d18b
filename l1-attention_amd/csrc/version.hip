// Library identification.
#include "common.h"

extern "C" int l1attn_version(void) { return 100; }
