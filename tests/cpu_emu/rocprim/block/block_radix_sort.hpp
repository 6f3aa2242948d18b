// TEST INFRASTRUCTURE: host stand-in for the one library primitive a kernel of this library uses,
// rocprim::block_radix_sort<Key, BLOCK, ITEMS>::sort(key, storage), for the CPU builds of tests/cpu_emu: every
// thread of the workgroup hands in ITEMS keys and receives the ITEMS consecutive keys of its place in the sorted
// order (thread x: positions x*ITEMS .. x*ITEMS+ITEMS-1).  The sort itself is std::sort by one thread between two
// barriers; what the tests exercise is the kernel around it.
#pragma once
#include "hip/hip_runtime.h"
#include <algorithm>

namespace rocprim {
template <class Key, unsigned BLOCK, unsigned ITEMS>
class block_radix_sort {
public:
	struct storage_type { Key keys[BLOCK * ITEMS]; };
	void sort(Key (&key)[ITEMS], storage_type& storage)
	{
		const unsigned tid = threadIdx.x;
		for (unsigned i = 0; i < ITEMS; i++) storage.keys[tid * ITEMS + i] = key[i];
		__syncthreads();
		if (tid == 0) std::sort(storage.keys, storage.keys + BLOCK * ITEMS);
		__syncthreads();
		for (unsigned i = 0; i < ITEMS; i++) key[i] = storage.keys[tid * ITEMS + i];
		__syncthreads();  // the storage may be used again
	}
};
}
