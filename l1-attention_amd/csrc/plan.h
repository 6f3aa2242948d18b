// Layout of the sparse "plan": one device buffer of int32 words that holds the dst-sorted (CSR)
// and src-sorted (CSC) views of an edge list.  Built by l1attn_sparse_plan_build (coo.hip), read by
// the kernels in sparse.hip.  Every array starts on a 256-byte boundary.
#pragma once
#include "common.h"

enum {
	PLAN_H_MAGIC = 0,
	PLAN_H_E = 1,           // rows of the edge list
	PLAN_H_T = 2,           // tokens
	PLAN_H_BAD = 3,         // 1 if a row held an index outside [0, T); such rows are dropped
	PLAN_H_MAXDEG_DST = 4,  // longest dst segment
	PLAN_H_MAXDEG_SRC = 5,  // longest src segment
	PLAN_H_E_VALID = 6,     // rows kept
	PLAN_H_NLONG_DST = 7,   // dst tokens with more than PLAN_LONG_SEGMENT edges (entries of long_dst)
	PLAN_H_NLONG_SRC = 8,   // same for src tokens
	PLAN_H_WORDS = 16
};
constexpr int PLAN_MAGIC = 0x4c314132;  // "L1A2"
// Segments longer than this are walked by a whole workgroup instead of one wavefront.
constexpr int PLAN_LONG_SEGMENT = 128;

struct PlanLayout {
	// offsets in int32 words from the start of the plan
	size_t dst_ptr;   // [T+2]  slot range of dst d is [dst_ptr[d], dst_ptr[d+1]); entry T = dropped rows
	size_t src_ptr;   // [T+2]
	size_t csr_src;   // [E]    src token of each slot (dst-sorted, original row order inside a segment)
	size_t csr_row;   // [E]    original row of each slot
	size_t csc_dst;   // [E]    dst token of each src-sorted entry
	size_t csc_slot;  // [E]    dst-sorted slot of each src-sorted entry
	size_t long_dst;  // [long_cap] dst tokens whose segment is longer than PLAN_LONG_SEGMENT (any order)
	size_t long_src;  // [long_cap]
	size_t long_cap;  // E / PLAN_LONG_SEGMENT + 1: no edge list has more long segments than that
	size_t total_bytes;
};

static inline PlanLayout plan_layout(int64_t E, int64_t T)
{
	PlanLayout L;
	size_t w = 64;  // header, padded to 256 bytes
	const size_t pa = l1_align_up((size_t)(T + 2), 64), ea = l1_align_up((size_t)(E > 0 ? E : 1), 64);
	L.dst_ptr = w; w += pa;
	L.src_ptr = w; w += pa;
	L.csr_src = w; w += ea;
	L.csr_row = w; w += ea;
	L.csc_dst = w; w += ea;
	L.csc_slot = w; w += ea;
	L.long_cap = (size_t)(E > 0 ? E : 0) / PLAN_LONG_SEGMENT + 1;
	const size_t la = l1_align_up(L.long_cap, 64);
	L.long_dst = w; w += la;
	L.long_src = w; w += la;
	L.total_bytes = w * 4;
	return L;
}
