/*
 * TEST INFRASTRUCTURE, not product code.
 *
 * CPU oracle for the L1-attention hot path: a plain-C restatement of the
 * reference's CPU extension (tlh24/l1-attention, cpp/l1attn_drv.cpp,
 * cpp/l1attn_sparse_drv.cpp, cpp/l1attn_sparse_bidi_drv.cpp) and of expandCoo
 * (python/l1attn_sparse.py:382-427).  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load this library; the shipped HIP library
 * never links or calls it.
 *
 * Pinned by tests/test_oracle_pins.py against: the reference's hand-made fixtures
 * (testdense.py:20-35 one-hot tokens; python/l1attn_sparse.py:450-484 integer
 * tokens, :522-576 bidi; README.md:89 cartesian coo), closed forms evaluated in
 * fp64 with an independent vectorised formulation, autograd through that closed
 * form, finite differences, the dense<->sparse equivalence with the no-op logit,
 * permutation invariance of the edge list, an O(E^2) brute-force rank for
 * expandCoo, and (when it was built) the reference's own compiled cpp/ extension
 * under oracle/_ref.
 *
 * Build: make -C oracle   ->  oracle/liboracle.so
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define REAL double
#define FN(x) x##_f64
#define ABS fabs
#define EXP exp
#include "l1attn_oracle_impl.h"
#undef REAL
#undef FN
#undef ABS
#undef EXP

#define REAL float
#define FN(x) x##_f32
#define ABS fabsf
#define EXP expf
#include "l1attn_oracle_impl.h"
#undef REAL
#undef FN
#undef ABS
#undef EXP

/*
 * expandCoo, python/l1attn_sparse.py:382-427 (same loop in
 * cuda/l1attn_sparse_cuda.py:58-101, cuda/l1attn_sparse_bidi_cuda.py:59-104,
 * cpp/l1attn_sparse_cpp.py:61-106):  coo[i] = [dst, src, number of earlier rows with
 * the same dst, number of earlier rows with the same src]; mxlen = 1 + max rank
 * (1 for an empty list, since the maxima start at 0).  The reference's per-key dict
 * is an array here, so indices must be >= 0.
 * co: int64 [E,2].  coo: int32 [E,4].  mxlen: {dst_mxlen, src_mxlen}.
 * Returns 0, or -1 on a negative index / allocation failure.
 */
int oracle_expand_coo(const long long *co, long E, int *coo, int *mxlen)
{
	long long kmax = -1;
	for (long i = 0; i < E; i++) {
		if (co[2 * i] < 0 || co[2 * i + 1] < 0) return -1;
		if (co[2 * i] > kmax) kmax = co[2 * i];
		if (co[2 * i + 1] > kmax) kmax = co[2 * i + 1];
	}
	int *dst_cntr = (int *)malloc(sizeof(int) * (size_t)(kmax + 2));
	int *src_cntr = (int *)malloc(sizeof(int) * (size_t)(kmax + 2));
	if (!dst_cntr || !src_cntr) { free(dst_cntr); free(src_cntr); return -1; }
	for (long long i = 0; i < kmax + 2; i++) dst_cntr[i] = src_cntr[i] = -1; /* "not in dict" */
	int dst_mx = 0, src_mx = 0;
	for (long i = 0; i < E; i++) {
		long long dst = co[2 * i], src = co[2 * i + 1];
		dst_cntr[dst] += 1; /* absent -> 0, present -> +1 */
		src_cntr[src] += 1;
		coo[4 * i + 0] = (int)dst;
		coo[4 * i + 1] = (int)src;
		coo[4 * i + 2] = dst_cntr[dst];
		coo[4 * i + 3] = src_cntr[src];
		if (dst_cntr[dst] > dst_mx) dst_mx = dst_cntr[dst];
		if (src_cntr[src] > src_mx) src_mx = src_cntr[src];
	}
	free(dst_cntr);
	free(src_cntr);
	mxlen[0] = dst_mx + 1;
	mxlen[1] = src_mx + 1;
	return 0;
}

#ifdef _OPENMP
#include <omp.h>
void oracle_set_threads(int n) { omp_set_num_threads(n); }
int oracle_max_threads(void) { return omp_get_max_threads(); }
#else
void oracle_set_threads(int n) { (void)n; }
int oracle_max_threads(void) { return 1; }
#endif
