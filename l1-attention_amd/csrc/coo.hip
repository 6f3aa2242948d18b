// Edge-list preparation for sparse L1 attention on gfx950.
//
//  * l1attn_expand_coo: the reference's expandCoo (python/l1attn_sparse.py:382-427, same loop in
//    cuda/l1attn_sparse_cuda.py:58-101) on the GPU: for every edge the number of EARLIER rows
//    with the same dst / the same src, and the maximum of each +1.  The reference walks the rows
//    in Python with two dicts; here each rank comes from one stable LSD radix sort of
//    (key, row) pairs: rank = position in the sorted order - first position of the key.
//    Integer arithmetic only, so the output is bit-exact.
//  * l1attn_sparse_plan_build: the dst-sorted (CSR) and src-sorted (CSC) views of an edge list
//    that the sparse kernels walk instead of scattering with atomics
//    (cuda/l1attn_sparse_cuda_kernel.cu:148-181, :183-254, :327-370 are the scatter kernels
//    this replaces).  Rows keep their original relative order inside a segment, so slot order
//    equals the reference's dst_cnt / src_cnt order.
//
// The radix sort: 8-bit digits, tiles of 2048 rows per workgroup, per-tile digit histogram ->
// one exclusive scan over [digit][tile] -> stable scatter.  Stability inside a tile comes from
// wave-level match masks (eight ballots per 64 rows) and per-wave running digit counters in LDS;
// no atomics take part in any position, so the permutation is deterministic.
#include "common.h"
#include "plan.h"

// The lanes named in `lanes` pass this point together.  Nothing on the GPU, where a wave's lanes execute every
// instruction in lockstep; a host build that runs lanes as threads defines it as a barrier among those lanes.
#ifndef L1_WAVE_LOCKSTEP
#define L1_WAVE_LOCKSTEP(lanes) ((void)0)
#endif

namespace {

constexpr int RS_THREADS = 256;
constexpr int RS_WAVES = RS_THREADS / 64;
constexpr int RS_ITEMS = 8;
constexpr int RS_TILE = RS_THREADS * RS_ITEMS;  // 2048 rows per workgroup
constexpr int RS_BITS = 8;
constexpr int RS_DIGITS = 1 << RS_BITS;

// stats words written by the extract kernels
enum { ST_MAXKEY = 0, ST_BAD = 1, ST_MAXDEG_DST = 2, ST_MAXDEG_SRC = 3, ST_NLONG_DST = 4, ST_NLONG_SRC = 5, ST_WORDS = 8 };

// maximum over the wave's 64 lanes (every lane must call it), returned in all lanes
__device__ __forceinline__ int wave_max(int v)
{
#pragma unroll
	for (int off = 32; off >= 1; off >>= 1) {
		const int o = __shfl_xor(v, off, 64);
		v = o > v ? o : v;
	}
	return v;
}

// maximum over the workgroup (256 threads, every thread must call it), valid in thread 0
__device__ __forceinline__ int block_max_256(int v)
{
	__shared__ int wm[4];
	v = wave_max(v);
	if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = v;
	__syncthreads();
	const int a = wm[0] > wm[1] ? wm[0] : wm[1], b = wm[2] > wm[3] ? wm[2] : wm[3];
	return a > b ? a : b;
}

constexpr int ROWS_PER_THREAD = 8;  // rows per thread of the row-parallel kernels below

// Same-address atomics are served one at a time by the L2 (about 10 ns each, whatever the wave coalesces),
// so the row-parallel kernels reduce over a workgroup of 2048 rows first and issue one atomic.
template <typename IdxT>
__global__ __launch_bounds__(256) void coo_extract(const IdxT* __restrict__ co, int64_t stride, int64_t E,
                                                     int* __restrict__ dst32, int* __restrict__ src32,
                                                     int* __restrict__ coo_out, int64_t n_tok, int* __restrict__ stats)
{
	// n_tok < 0: any non-negative int32 index is valid (expandCoo); otherwise indices must be < n_tok
	// and invalid rows get the sentinel key n_tok in both columns (they sort last and are dropped).
	int key_max = 0;
	bool any_bad = false;
#pragma unroll
	for (int it = 0; it < ROWS_PER_THREAD; it++) {
		const int64_t i = ((int64_t)blockIdx.x * ROWS_PER_THREAD + it) * 256 + threadIdx.x;
		if (i < E) {
			const long long d = (long long)co[i * stride], s = (long long)co[i * stride + 1];
			const long long hi = n_tok < 0 ? 2147483647LL : (long long)n_tok - 1;
			const bool bad = d < 0 || s < 0 || d > hi || s > hi;
			int di = (int)d, si = (int)s;
			if (bad) {
				any_bad = true;
				di = si = n_tok < 0 ? 0 : (int)n_tok;
			}
			dst32[i] = di;
			src32[i] = si;
			const int m = di > si ? di : si;
			key_max = m > key_max ? m : key_max;
			if (coo_out) {
				coo_out[i * 4 + 0] = di;
				coo_out[i * 4 + 1] = si;
			}
		}
	}
	if (any_bad) atomicOr(&stats[ST_BAD], 1);
	key_max = block_max_256(key_max);
	if (threadIdx.x == 0) atomicMax(&stats[ST_MAXKEY], key_max);
}

__global__ __launch_bounds__(RS_THREADS) void radix_hist(const int* __restrict__ keys, int64_t E, int shift,
                                                           int* __restrict__ hist, int nblk)
{
	__shared__ int h[RS_DIGITS];
	h[threadIdx.x] = 0;
	__syncthreads();
	const int64_t base = (int64_t)blockIdx.x * RS_TILE;
#pragma unroll
	for (int c = 0; c < RS_ITEMS; c++) {
		const int64_t i = base + c * RS_THREADS + threadIdx.x;
		if (i < E) atomicAdd(&h[(keys[i] >> shift) & (RS_DIGITS - 1)], 1);
	}
	__syncthreads();
	hist[(int64_t)threadIdx.x * nblk + blockIdx.x] = h[threadIdx.x];
}

// Exclusive prefix sum of n ints in place, one workgroup of 1024 threads.  The array is walked in chunks of
// 8192: a thread takes eight consecutive elements (two 16-byte loads, so a wave reads 2 KiB contiguously),
// the waves combine their totals with shuffles and one pass through LDS, and the running total carries over.
// The 16-byte accesses are used when a is 16-byte aligned.
__global__ __launch_bounds__(1024) void scan_exclusive(int* __restrict__ a, int64_t n)
{
	__shared__ int wave_total[16];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const bool vec = (reinterpret_cast<uintptr_t>(a) & 15) == 0;
	int carry = 0;
	for (int64_t base = 0; base < n; base += 8192) {
		const int64_t i0 = base + (int64_t)threadIdx.x * 8;
		int v[8];
		if (vec && i0 + 8 <= n) {
			const int4 x = *reinterpret_cast<const int4*>(a + i0), y = *reinterpret_cast<const int4*>(a + i0 + 4);
			v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w; v[4] = y.x; v[5] = y.y; v[6] = y.z; v[7] = y.w;
		} else {
#pragma unroll
			for (int j = 0; j < 8; j++) v[j] = i0 + j < n ? a[i0 + j] : 0;
		}
		int total = 0;
#pragma unroll
		for (int j = 0; j < 8; j++) {  // v[j] becomes the sum of the thread's elements before j
			const int t = v[j];
			v[j] = total;
			total += t;
		}
		int incl = total;  // inclusive scan of the thread totals over the wave
#pragma unroll
		for (int off = 1; off < 64; off <<= 1) {
			const int up = __shfl_up(incl, off, 64);
			if (lane >= off) incl += up;
		}
		if (lane == 63) wave_total[wave] = incl;
		__syncthreads();
		int before = carry, all = 0;
#pragma unroll
		for (int w = 0; w < 16; w++) {
			const int t = wave_total[w];
			if (w < wave) before += t;
			all += t;
		}
		const int mine = before + incl - total;  // everything before this thread's first element
		if (vec && i0 + 8 <= n) {
			*reinterpret_cast<int4*>(a + i0) = make_int4(mine + v[0], mine + v[1], mine + v[2], mine + v[3]);
			*reinterpret_cast<int4*>(a + i0 + 4) = make_int4(mine + v[4], mine + v[5], mine + v[6], mine + v[7]);
		} else {
#pragma unroll
			for (int j = 0; j < 8; j++)
				if (i0 + j < n) a[i0 + j] = mine + v[j];
		}
		carry += all;
		__syncthreads();  // wave_total is rewritten by the next chunk
	}
}

// vals_in == nullptr means the identity permutation (first pass)
__global__ __launch_bounds__(RS_THREADS) void radix_scatter(const int* __restrict__ keys_in,
                                                              const int* __restrict__ vals_in,
                                                              int* __restrict__ keys_out, int* __restrict__ vals_out,
                                                              int64_t E, int shift, const int* __restrict__ hist,
                                                              int nblk)
{
	__shared__ int wcount[RS_WAVES][RS_DIGITS];  // rows of each digit seen so far by each wave
	__shared__ int base[RS_DIGITS];              // first output position of each digit for this tile
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
	for (int w = 0; w < RS_WAVES; w++) wcount[w][threadIdx.x] = 0;
	base[threadIdx.x] = hist[(int64_t)threadIdx.x * nblk + blockIdx.x];
	__syncthreads();

	const int64_t tile0 = (int64_t)blockIdx.x * RS_TILE + wave * (64 * RS_ITEMS);
	const unsigned long long lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
	int key[RS_ITEMS], val[RS_ITEMS], rank[RS_ITEMS];
#pragma unroll
	for (int c = 0; c < RS_ITEMS; c++) {
		const int64_t i = tile0 + c * 64 + lane;
		const bool valid = i < E;
		key[c] = valid ? keys_in[i] : 0;
		val[c] = valid ? (vals_in ? vals_in[i] : (int)i) : 0;
		const int d = (key[c] >> shift) & (RS_DIGITS - 1);
		unsigned long long m = __ballot(valid);
#pragma unroll
		for (int bit = 0; bit < RS_BITS; bit++) {
			const bool one = (d >> bit) & 1;
			const unsigned long long bm = __ballot(one);
			m &= one ? bm : ~bm;
		}
		rank[c] = -1;
		if (valid) {
			const int prev = wcount[wave][d];  // read by every lane of the digit before the leader updates it
			rank[c] = prev + __popcll(m & lt_mask);
			L1_WAVE_LOCKSTEP(m);
			if ((m & lt_mask) == 0) wcount[wave][d] = prev + __popcll(m);
		}
	}
	__syncthreads();
#pragma unroll
	for (int c = 0; c < RS_ITEMS; c++) {
		if (rank[c] >= 0) {
			const int d = (key[c] >> shift) & (RS_DIGITS - 1);
			int pos = base[d] + rank[c];
			for (int w = 0; w < wave; w++) pos += wcount[w][d];
			keys_out[pos] = key[c];
			vals_out[pos] = val[c];
		}
	}
}

__device__ __forceinline__ int lower_bound(const int* __restrict__ a, int n, int key)
{
	int lo = 0, hi = n;
	while (lo < hi) {
		const int mid = (lo + hi) >> 1;
		if (a[mid] < key) lo = mid + 1; else hi = mid;
	}
	return lo;
}

// rank of each row among the rows with its key; written to out[row*out_stride + out_col]
__global__ __launch_bounds__(256) void ranks_from_sorted(const int* __restrict__ keys_sorted,
                                                           const int* __restrict__ rows_sorted, int E,
                                                           int* __restrict__ out, int out_stride, int out_col,
                                                           int* __restrict__ maxdeg)
{
	int deg = 0;
#pragma unroll
	for (int it = 0; it < ROWS_PER_THREAD; it++) {
		const int64_t p = ((int64_t)blockIdx.x * ROWS_PER_THREAD + it) * 256 + threadIdx.x;
		if (p < E) {
			const int r = (int)p - lower_bound(keys_sorted, E, keys_sorted[p]);
			out[(int64_t)rows_sorted[p] * out_stride + out_col] = r;
			deg = r + 1 > deg ? r + 1 : deg;
		}
	}
	deg = block_max_256(deg);
	if (threadIdx.x == 0) atomicMax(maxdeg, deg);
}

__global__ __launch_bounds__(256) void segment_ptrs(const int* __restrict__ keys_sorted, int E, int n_ptr,
                                                      int* __restrict__ ptr)
{
	const int key = blockIdx.x * 256 + threadIdx.x;
	if (key < n_ptr) ptr[key] = lower_bound(keys_sorted, E, key);
}

// after the dst sort: slot p holds row rows_sorted[p]
__global__ __launch_bounds__(256) void plan_fill_csr(const int* __restrict__ rows_sorted, const int* __restrict__ src32,
                                                       int E, int* __restrict__ csr_src, int* __restrict__ csr_row,
                                                       int* __restrict__ slot_of_row)
{
	const int p = blockIdx.x * 256 + threadIdx.x;
	if (p >= E) return;
	const int row = rows_sorted[p];
	csr_src[p] = src32[row];
	csr_row[p] = row;
	slot_of_row[row] = p;
}

// after the src sort
__global__ __launch_bounds__(256) void plan_fill_csc(const int* __restrict__ rows_sorted, const int* __restrict__ dst32,
                                                       const int* __restrict__ slot_of_row, int E,
                                                       int* __restrict__ csc_dst, int* __restrict__ csc_slot)
{
	const int i = blockIdx.x * 256 + threadIdx.x;
	if (i >= E) return;
	const int row = rows_sorted[i];
	csc_dst[i] = dst32[row];
	csc_slot[i] = slot_of_row[row];
}

// longest segment of a pointer array with n_keys segments, and the list of keys whose segment is
// longer than PLAN_LONG_SEGMENT (list order is arbitrary: every entry is processed independently)
__global__ __launch_bounds__(256) void max_segment(const int* __restrict__ ptr, int n_keys, int* __restrict__ out,
                                                     int* __restrict__ long_list, int* __restrict__ n_long)
{
	const int key = blockIdx.x * 256 + threadIdx.x;
	const int deg = key < n_keys ? ptr[key + 1] - ptr[key] : 0;
	if (deg > PLAN_LONG_SEGMENT) long_list[atomicAdd(n_long, 1)] = key;
	const int wmax = wave_max(deg);
	if ((threadIdx.x & 63) == 0) atomicMax(out, wmax);
}

__global__ void fill_words(int* __restrict__ a, int n, int v)
{
	const int i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) a[i] = v;
}

__global__ void plan_header(int* __restrict__ hdr, int E, int T, const int* __restrict__ stats,
                            const int* __restrict__ dst_ptr)
{
	if (threadIdx.x == 0 && blockIdx.x == 0) {
		hdr[PLAN_H_MAGIC] = PLAN_MAGIC;
		hdr[PLAN_H_E] = E;
		hdr[PLAN_H_T] = T;
		hdr[PLAN_H_BAD] = stats[ST_BAD];
		hdr[PLAN_H_MAXDEG_DST] = stats[ST_MAXDEG_DST];
		hdr[PLAN_H_MAXDEG_SRC] = stats[ST_MAXDEG_SRC];
		hdr[PLAN_H_E_VALID] = dst_ptr[T];  // rows with the sentinel key T sort behind this position
		hdr[PLAN_H_NLONG_DST] = stats[ST_NLONG_DST];
		hdr[PLAN_H_NLONG_SRC] = stats[ST_NLONG_SRC];
	}
}

int bits_for(int64_t max_key)
{
	int b = 1;
	while (b < 31 && (1LL << b) <= max_key) b++;
	return b;
}

struct SortBufs {
	int *keys_a, *keys_b, *vals_a, *vals_b, *hist;
	int nblk;
};

size_t sort_bytes(int64_t E)
{
	const int64_t nblk = l1_cdiv(E > 0 ? E : 1, RS_TILE);
	return 4 * l1_align_up((size_t)E * 4, 256) + l1_align_up((size_t)(RS_DIGITS * nblk + 1) * 4, 256);
}

SortBufs carve_sort(char* p, int64_t E)
{
	SortBufs s;
	const size_t a = l1_align_up((size_t)E * 4, 256);
	s.keys_a = (int*)p; p += a;
	s.keys_b = (int*)p; p += a;
	s.vals_a = (int*)p; p += a;
	s.vals_b = (int*)p; p += a;
	s.hist = (int*)p;
	s.nblk = (int)l1_cdiv(E > 0 ? E : 1, RS_TILE);
	return s;
}

// Stable sort of rows 0..E-1 by keys[row].  Returns the buffers that hold the result.
int sort_rows_by_key(const int* keys, int64_t E, int key_bits, const SortBufs& s, hipStream_t st,
                     const int** keys_sorted, const int** rows_sorted)
{
	const int* kin = keys;
	const int* vin = nullptr;
	int* kout = s.keys_a;
	int* vout = s.vals_a;
	for (int shift = 0; shift < key_bits; shift += RS_BITS) {
		hipLaunchKernelGGL(radix_hist, dim3(s.nblk), dim3(RS_THREADS), 0, st, kin, E, shift, s.hist, s.nblk);
		L1_LAUNCH_CHECK();
		hipLaunchKernelGGL(scan_exclusive, dim3(1), dim3(1024), 0, st, s.hist, (int64_t)RS_DIGITS * s.nblk);
		L1_LAUNCH_CHECK();
		hipLaunchKernelGGL(radix_scatter, dim3(s.nblk), dim3(RS_THREADS), 0, st, kin, vin, kout, vout, E, shift,
		                   s.hist, s.nblk);
		L1_LAUNCH_CHECK();
		kin = kout;
		vin = vout;
		kout = (kout == s.keys_a) ? s.keys_b : s.keys_a;
		vout = (vout == s.vals_a) ? s.vals_b : s.vals_a;
	}
	*keys_sorted = kin;
	*rows_sorted = vin;
	return L1ATTN_OK;
}

constexpr int64_t MAX_EDGES = 2147483647LL - RS_TILE;

}  // namespace

extern "C" {

size_t l1attn_expand_coo_workspace_bytes(int64_t E)
{
	if (E <= 0) return 256;
	return 256 + 2 * l1_align_up((size_t)E * 4, 256) + sort_bytes(E);
}

int l1attn_expand_coo(const void* co, int co_bits, int64_t co_stride, int64_t E, int32_t* coo, int32_t* mxlen_host,
                      void* workspace, size_t workspace_bytes, void* stream)
{
	if (E < 0 || (co_bits != 32 && co_bits != 64) || co_stride < 2 || !mxlen_host) return L1ATTN_ERR_ARG;
	mxlen_host[0] = mxlen_host[1] = 1;  // the reference starts both maxima at index 0
	if (E == 0) return L1ATTN_OK;
	if (!co || !coo) return L1ATTN_ERR_ARG;
	if (E > MAX_EDGES) return L1ATTN_ERR_RANGE;
	if (!workspace || workspace_bytes < l1attn_expand_coo_workspace_bytes(E)) return L1ATTN_ERR_WORKSPACE;
	hipStream_t st = (hipStream_t)stream;
	char* p = (char*)workspace;
	int* stats = (int*)p; p += 256;
	int* dst32 = (int*)p; p += l1_align_up((size_t)E * 4, 256);
	int* src32 = (int*)p; p += l1_align_up((size_t)E * 4, 256);
	const SortBufs sb = carve_sort(p, E);
	const unsigned g256 = (unsigned)l1_cdiv(E, 256);
	const unsigned g2048 = (unsigned)l1_cdiv(E, 256 * ROWS_PER_THREAD);

	hipLaunchKernelGGL(fill_words, dim3(1), dim3(64), 0, st, stats, ST_WORDS, 0);
	L1_LAUNCH_CHECK();
	if (co_bits == 64)
		hipLaunchKernelGGL(coo_extract<long long>, dim3(g2048), dim3(256), 0, st, (const long long*)co, co_stride, E,
		                   dst32, src32, coo, (int64_t)-1, stats);
	else
		hipLaunchKernelGGL(coo_extract<int>, dim3(g2048), dim3(256), 0, st, (const int*)co, co_stride, E, dst32, src32,
		                   coo, (int64_t)-1, stats);
	L1_LAUNCH_CHECK();
	int h_stats[ST_WORDS];
	L1_HIP_CHECK(hipMemcpyAsync(h_stats, stats, sizeof(h_stats), hipMemcpyDeviceToHost, st));
	L1_HIP_CHECK(hipStreamSynchronize(st));
	if (h_stats[ST_BAD]) return L1ATTN_ERR_INDEX;
	const int bits = bits_for(h_stats[ST_MAXKEY]);

	const int *ks, *rs;
	int rc = sort_rows_by_key(dst32, E, bits, sb, st, &ks, &rs);
	if (rc) return rc;
	hipLaunchKernelGGL(ranks_from_sorted, dim3(g2048), dim3(256), 0, st, ks, rs, (int)E, coo, 4, 2,
	                   stats + ST_MAXDEG_DST);
	L1_LAUNCH_CHECK();
	rc = sort_rows_by_key(src32, E, bits, sb, st, &ks, &rs);
	if (rc) return rc;
	hipLaunchKernelGGL(ranks_from_sorted, dim3(g2048), dim3(256), 0, st, ks, rs, (int)E, coo, 4, 3,
	                   stats + ST_MAXDEG_SRC);
	L1_LAUNCH_CHECK();
	L1_HIP_CHECK(hipMemcpyAsync(h_stats, stats, sizeof(h_stats), hipMemcpyDeviceToHost, st));
	L1_HIP_CHECK(hipStreamSynchronize(st));
	mxlen_host[0] = h_stats[ST_MAXDEG_DST];
	mxlen_host[1] = h_stats[ST_MAXDEG_SRC];
	return L1ATTN_OK;
}

size_t l1attn_sparse_plan_bytes(int64_t E, int64_t T)
{
	if (E < 0 || T < 0) return 0;
	return plan_layout(E, T).total_bytes;
}

size_t l1attn_sparse_plan_workspace_bytes(int64_t E, int64_t T)
{
	(void)T;
	if (E <= 0) return 256;
	return 256 + 3 * l1_align_up((size_t)E * 4, 256) + sort_bytes(E);
}

int l1attn_sparse_plan_build(const int32_t* coo, int64_t coo_stride, int64_t E, int64_t T, void* plan,
                             size_t plan_bytes, void* workspace, size_t workspace_bytes, void* stream)
{
	if (E < 0 || T < 0 || coo_stride < 2 || !plan) return L1ATTN_ERR_ARG;
	if (E > MAX_EDGES || T > (1LL << 30)) return L1ATTN_ERR_RANGE;
	const PlanLayout L = plan_layout(E, T);
	if (plan_bytes < L.total_bytes) return L1ATTN_ERR_WORKSPACE;
	hipStream_t st = (hipStream_t)stream;
	int* words = (int*)plan;
	int* stats;
	if (E == 0) {
		// empty list: all segment pointers 0, header written from zeroed stats
		if (!workspace || workspace_bytes < 256) return L1ATTN_ERR_WORKSPACE;
		stats = (int*)workspace;
		hipLaunchKernelGGL(fill_words, dim3(1), dim3(64), 0, st, stats, ST_WORDS, 0);
		// dst_ptr and src_ptr are adjacent arrays; zero both up to the start of csr_src
		const int n = (int)(L.csr_src - L.dst_ptr);
		hipLaunchKernelGGL(fill_words, dim3((unsigned)l1_cdiv(n, 256)), dim3(256), 0, st, words + L.dst_ptr, n, 0);
		L1_LAUNCH_CHECK();
		hipLaunchKernelGGL(plan_header, dim3(1), dim3(64), 0, st, words, 0, (int)T, stats, words + L.dst_ptr);
		L1_LAUNCH_CHECK();
		return L1ATTN_OK;
	}
	if (!coo) return L1ATTN_ERR_ARG;
	if (!workspace || workspace_bytes < l1attn_sparse_plan_workspace_bytes(E, T)) return L1ATTN_ERR_WORKSPACE;
	char* p = (char*)workspace;
	stats = (int*)p; p += 256;
	const size_t ea = l1_align_up((size_t)E * 4, 256);
	int* dst32 = (int*)p; p += ea;
	int* src32 = (int*)p; p += ea;
	int* slot_of_row = (int*)p; p += ea;
	const SortBufs sb = carve_sort(p, E);
	const unsigned g256 = (unsigned)l1_cdiv(E, 256);
	const unsigned g2048 = (unsigned)l1_cdiv(E, 256 * ROWS_PER_THREAD);
	const unsigned gptr = (unsigned)l1_cdiv(T + 2, 256);
	const int bits = bits_for(T);  // keys 0..T (T = sentinel of invalid rows)

	hipLaunchKernelGGL(fill_words, dim3(1), dim3(64), 0, st, stats, ST_WORDS, 0);
	L1_LAUNCH_CHECK();
	hipLaunchKernelGGL(coo_extract<int>, dim3(g2048), dim3(256), 0, st, (const int*)coo, coo_stride, E, dst32, src32,
	                   (int*)nullptr, T, stats);
	L1_LAUNCH_CHECK();

	const int *ks, *rs;
	int rc = sort_rows_by_key(dst32, E, bits, sb, st, &ks, &rs);
	if (rc) return rc;
	hipLaunchKernelGGL(segment_ptrs, dim3(gptr), dim3(256), 0, st, ks, (int)E, (int)(T + 2), words + L.dst_ptr);
	L1_LAUNCH_CHECK();
	hipLaunchKernelGGL(plan_fill_csr, dim3(g256), dim3(256), 0, st, rs, src32, (int)E, words + L.csr_src,
	                   words + L.csr_row, slot_of_row);
	L1_LAUNCH_CHECK();
	if (T > 0) hipLaunchKernelGGL(max_segment, dim3((unsigned)l1_cdiv(T, 256)), dim3(256), 0, st, words + L.dst_ptr,
	                              (int)T, stats + ST_MAXDEG_DST, words + L.long_dst, stats + ST_NLONG_DST);
	L1_LAUNCH_CHECK();
	rc = sort_rows_by_key(src32, E, bits, sb, st, &ks, &rs);
	if (rc) return rc;
	hipLaunchKernelGGL(segment_ptrs, dim3(gptr), dim3(256), 0, st, ks, (int)E, (int)(T + 2), words + L.src_ptr);
	L1_LAUNCH_CHECK();
	if (T > 0) hipLaunchKernelGGL(max_segment, dim3((unsigned)l1_cdiv(T, 256)), dim3(256), 0, st, words + L.src_ptr,
	                              (int)T, stats + ST_MAXDEG_SRC, words + L.long_src, stats + ST_NLONG_SRC);
	L1_LAUNCH_CHECK();
	hipLaunchKernelGGL(plan_fill_csc, dim3(g256), dim3(256), 0, st, rs, dst32, slot_of_row, (int)E,
	                   words + L.csc_dst, words + L.csc_slot);
	L1_LAUNCH_CHECK();
	hipLaunchKernelGGL(plan_header, dim3(1), dim3(64), 0, st, words, (int)E, (int)T, stats, words + L.dst_ptr);
	L1_LAUNCH_CHECK();
	return L1ATTN_OK;
}

int l1attn_sparse_plan_check(const void* plan, int64_t E, int64_t T, int32_t* header_host, void* stream)
{
	// copies the 16-word header to the host and synchronises the stream: the only blocking call of the plan API
	if (!plan || !header_host) return L1ATTN_ERR_ARG;
	hipStream_t st = (hipStream_t)stream;
	L1_HIP_CHECK(hipMemcpyAsync(header_host, plan, PLAN_H_WORDS * 4, hipMemcpyDeviceToHost, st));
	L1_HIP_CHECK(hipStreamSynchronize(st));
	if (header_host[PLAN_H_MAGIC] != PLAN_MAGIC || header_host[PLAN_H_E] != (int)E || header_host[PLAN_H_T] != (int)T)
		return L1ATTN_ERR_ARG;
	if (header_host[PLAN_H_BAD]) return L1ATTN_ERR_INDEX;
	return L1ATTN_OK;
}

}  // extern "C"
