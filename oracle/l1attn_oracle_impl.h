/*
 * TEST INFRASTRUCTURE -- body of the CPU oracle, included once per scalar type
 * by l1attn_oracle.c with REAL (float|double) and FN(name) (suffix macro) set.
 *
 * Every function restates, loop for loop, one function of the reference's CPU
 * extension (tlh24/l1-attention, cpp/), whose only scalar type is double.  The
 * float instantiation is the same loops with float accumulators.
 */

static inline REAL FN(sgn)(REAL x)
{
	/* cpp/l1attn_drv.cpp:7-11 : sign(0) == 0 */
	REAL t = x < 0 ? (REAL)-1 : (REAL)0;
	return x > 0 ? (REAL)1 : t;
}

/* ------------------------------------------------------------------ dense */

/* cpp/l1attn_drv.cpp:13-55  (loop order b,s,t,h,w; scale applied after the sum :48)
 * q,k [B,T,H,W] ; attn [B,T(src),T(dst),H] */
void FN(oracle_dense_fwd)(const REAL *q, const REAL *k, REAL *attn,
                          long B, long T, long H, long W)
{
	const REAL scale = (REAL)(-1.0 / sqrt((double)W));
	#pragma omp parallel for collapse(2) schedule(static)
	for (long b = 0; b < B; b++) {
		for (long s = 0; s < T; s++) {
			for (long t = 0; t < T; t++) {
				for (long h = 0; h < H; h++) {
					const REAL *qp = q + ((b * T + t) * H + h) * W;
					const REAL *kp = k + ((b * T + s) * H + h) * W;
					REAL f = 0;
					for (long w = 0; w < W; w++)
						f += ABS(qp[w] - kp[w]);
					f *= scale;
					attn[((b * T + s) * T + t) * H + h] = f;
				}
			}
		}
	}
}

/* cpp/l1attn_drv.cpp:57-98.  d_attn [B,S,T,H]; dq,dk [B,T,H,W] (zero-initialised here).
 * The reference nests b,s,t,h,w.  Here h is hoisted next to b so that OpenMP threads can split
 * over (b,h): outputs of different heads are disjoint, and every output element is still
 * accumulated by one thread in the reference's own (s,t) order, so the sums are unchanged. */
void FN(oracle_dense_bwd)(const REAL *d_attn, const REAL *q, const REAL *k,
                          REAL *dq, REAL *dk, long B, long T, long H, long W)
{
	const REAL scale = (REAL)(-1.0 / sqrt((double)W));
	memset(dq, 0, sizeof(REAL) * (size_t)(B * T * H * W));
	memset(dk, 0, sizeof(REAL) * (size_t)(B * T * H * W));
	#pragma omp parallel for collapse(2) schedule(static)
	for (long b = 0; b < B; b++) {
		for (long h = 0; h < H; h++) {
			for (long s = 0; s < T; s++) {
				for (long t = 0; t < T; t++) {
					REAL d_a = d_attn[((b * T + s) * T + t) * H + h];
					const REAL *qp = q + ((b * T + t) * H + h) * W;
					const REAL *kp = k + ((b * T + s) * H + h) * W;
					REAL *dqp = dq + ((b * T + t) * H + h) * W;
					REAL *dkp = dk + ((b * T + s) * H + h) * W;
					for (long w = 0; w < W; w++) {
						REAL ws = qp[w] - kp[w];
						ws = FN(sgn)(ws) * scale;
						dqp[w] += ws * d_a;
						dkp[w] -= ws * d_a;
					}
				}
			}
		}
	}
}

/* ----------------------------------------------------------------- sparse */

#define IX4(b, t, h, w, T_, H_, W_) ((((b) * (T_) + (t)) * (H_) + (h)) * (W_) + (w))

/* shared by uni and bidi: edge logits -> padded attn -> softmax (or exp).
 * cpp/l1attn_sparse_drv.cpp:38-41 (-1e12 fill), :51-62 (edge pass), :63-77 (softmax,
 * denominator starts at 1 :67).  attn [B,T,mx,H]. */
static void FN(sparse_attn_bh)(const REAL *q, const REAL *k, const int *coo, long cstride,
                               REAL *attn, long b, long h,
                               long T, long H, long W, long E, long mx, int use_softmax)
{
	const REAL scale = (REAL)(-1.0 / sqrt((double)W));
	for (long c = 0; c < E; c++) {
		long dst = coo[c * cstride + 0], src = coo[c * cstride + 1], r = coo[c * cstride + 2];
		REAL f = 0;
		for (long w = 0; w < W; w++)
			f += ABS(q[IX4(b, dst, h, w, T, H, W)] - k[IX4(b, src, h, w, T, H, W)]);
		f *= scale;
		attn[IX4(b, dst, r, h, T, mx, H)] = f;
	}
	if (use_softmax) {
		for (long d = 0; d < T; d++) {
			REAL f = 1; /* denominator bias */
			for (long r = 0; r < mx; r++)
				f += EXP(attn[IX4(b, d, r, h, T, mx, H)]);
			for (long r = 0; r < mx; r++)
				attn[IX4(b, d, r, h, T, mx, H)] = EXP(attn[IX4(b, d, r, h, T, mx, H)]) / f;
		}
	} else {
		for (long d = 0; d < T; d++)
			for (long r = 0; r < mx; r++)
				attn[IX4(b, d, r, h, T, mx, H)] = EXP(attn[IX4(b, d, r, h, T, mx, H)]);
	}
}

/* cpp/l1attn_sparse_drv.cpp:13-91.  v,q,k [B,T,H,W]; coo int32 [E,cstride>=3] rows
 * [dst,src,dst_cnt,..]; attn [B,T,mx,H] (saved for backward); vo [B,T,H,W]. */
void FN(oracle_sparse_fwd)(const REAL *v, const REAL *q, const REAL *k,
                           const int *coo, long cstride, REAL *vo, REAL *attn,
                           long B, long T, long H, long W, long E, long mx, int use_softmax)
{
	for (long i = 0; i < B * T * mx * H; i++) attn[i] = (REAL)-1e12;
	memset(vo, 0, sizeof(REAL) * (size_t)(B * T * H * W));
	#pragma omp parallel for collapse(2) schedule(static)
	for (long b = 0; b < B; b++) {
		for (long h = 0; h < H; h++) {
			FN(sparse_attn_bh)(q, k, coo, cstride, attn, b, h, T, H, W, E, mx, use_softmax);
			for (long c = 0; c < E; c++) {
				long dst = coo[c * cstride + 0], src = coo[c * cstride + 1], r = coo[c * cstride + 2];
				REAL a = attn[IX4(b, dst, r, h, T, mx, H)];
				for (long w = 0; w < W; w++)
					vo[IX4(b, dst, h, w, T, H, W)] += a * v[IX4(b, src, h, w, T, H, W)];
			}
		}
	}
}

/* softmax-Jacobian product shared by uni and bidi.
 * jac_mode 0: the reference's O(mx^2) loop, cpp/l1attn_sparse_drv.cpp:152-167.
 * jac_mode 1: the algebraically equal O(mx) closed form p_r*(dp_r - sum_q p_q dp_q),
 *             used where mx^2 is too slow; tests pin it against mode 0. */
static void FN(sparse_jac_bh)(const REAL *attn, const REAL *dattn_sm, REAL *dattn,
                              long b, long h, long T, long H, long mx,
                              int use_softmax, int jac_mode)
{
	if (use_softmax && jac_mode == 0) {
		for (long d = 0; d < T; d++)
			for (long r = 0; r < mx; r++)
				for (long qq = 0; qq < mx; qq++) {
					REAL ar = attn[IX4(b, d, r, h, T, mx, H)];
					REAL f;
					if (r == qq) f = ar * (1 - ar);
					else f = -1 * ar * attn[IX4(b, d, qq, h, T, mx, H)];
					dattn[IX4(b, d, r, h, T, mx, H)] += f * dattn_sm[IX4(b, d, qq, h, T, mx, H)];
				}
	} else if (use_softmax) {
		for (long d = 0; d < T; d++) {
			REAL s = 0;
			for (long r = 0; r < mx; r++)
				s += attn[IX4(b, d, r, h, T, mx, H)] * dattn_sm[IX4(b, d, r, h, T, mx, H)];
			for (long r = 0; r < mx; r++)
				dattn[IX4(b, d, r, h, T, mx, H)] +=
					attn[IX4(b, d, r, h, T, mx, H)] * (dattn_sm[IX4(b, d, r, h, T, mx, H)] - s);
		}
	} else {
		/* cpp/l1attn_sparse_drv.cpp:168-175 */
		for (long d = 0; d < T; d++)
			for (long r = 0; r < mx; r++)
				dattn[IX4(b, d, r, h, T, mx, H)] +=
					attn[IX4(b, d, r, h, T, mx, H)] * dattn_sm[IX4(b, d, r, h, T, mx, H)];
	}
}

/* dq/dk edge pass, cpp/l1attn_sparse_drv.cpp:176-188 */
static void FN(sparse_dqdk_bh)(const REAL *q, const REAL *k, const int *coo, long cstride,
                               const REAL *dattn, REAL *dq, REAL *dk,
                               long b, long h, long T, long H, long W, long E, long mx)
{
	const REAL scale = (REAL)(-1.0 / sqrt((double)W));
	for (long c = 0; c < E; c++) {
		long dst = coo[c * cstride + 0], src = coo[c * cstride + 1], r = coo[c * cstride + 2];
		REAL da = dattn[IX4(b, dst, r, h, T, mx, H)];
		for (long w = 0; w < W; w++) {
			REAL ws = q[IX4(b, dst, h, w, T, H, W)] - k[IX4(b, src, h, w, T, H, W)];
			ws = FN(sgn)(ws) * scale;
			dq[IX4(b, dst, h, w, T, H, W)] += ws * da;
			dk[IX4(b, src, h, w, T, H, W)] += -1 * ws * da;
		}
	}
}

/* cpp/l1attn_sparse_drv.cpp:93-190.  attn is the tensor oracle_sparse_fwd saved.
 * scratch: 2*B*T*mx*H REALs (dattn_sm, dattn), zeroed here. */
void FN(oracle_sparse_bwd)(const REAL *dvo, const REAL *v, const REAL *q, const REAL *k,
                           const int *coo, long cstride, const REAL *attn,
                           REAL *dv, REAL *dq, REAL *dk, REAL *scratch,
                           long B, long T, long H, long W, long E, long mx,
                           int use_softmax, int jac_mode)
{
	size_t n = (size_t)(B * T * H * W), na = (size_t)(B * T * mx * H);
	REAL *dattn_sm = scratch, *dattn = scratch + na;
	memset(dv, 0, sizeof(REAL) * n);
	memset(dq, 0, sizeof(REAL) * n);
	memset(dk, 0, sizeof(REAL) * n);
	memset(scratch, 0, sizeof(REAL) * 2 * na);
	#pragma omp parallel for collapse(2) schedule(static)
	for (long b = 0; b < B; b++) {
		for (long h = 0; h < H; h++) {
			for (long c = 0; c < E; c++) {
				long dst = coo[c * cstride + 0], src = coo[c * cstride + 1], r = coo[c * cstride + 2];
				REAL a = attn[IX4(b, dst, r, h, T, mx, H)];
				for (long w = 0; w < W; w++)
					dv[IX4(b, src, h, w, T, H, W)] += a * dvo[IX4(b, dst, h, w, T, H, W)];
				for (long w = 0; w < W; w++)
					dattn_sm[IX4(b, dst, r, h, T, mx, H)] +=
						v[IX4(b, src, h, w, T, H, W)] * dvo[IX4(b, dst, h, w, T, H, W)];
			}
			FN(sparse_jac_bh)(attn, dattn_sm, dattn, b, h, T, H, mx, use_softmax, jac_mode);
			FN(sparse_dqdk_bh)(q, k, coo, cstride, dattn, dq, dk, b, h, T, H, W, E, mx);
		}
	}
}

/* ------------------------------------------------------------------- bidi */

/* cpp/l1attn_sparse_bidi_drv.cpp:15-101: same attn; vo[dst] += a*vf[src] and
 * vo[src] += a*vb[dst] (:85-97). */
void FN(oracle_bidi_fwd)(const REAL *vf, const REAL *vb, const REAL *q, const REAL *k,
                         const int *coo, long cstride, REAL *vo, REAL *attn,
                         long B, long T, long H, long W, long E, long mx, int use_softmax)
{
	for (long i = 0; i < B * T * mx * H; i++) attn[i] = (REAL)-1e12;
	memset(vo, 0, sizeof(REAL) * (size_t)(B * T * H * W));
	#pragma omp parallel for collapse(2) schedule(static)
	for (long b = 0; b < B; b++) {
		for (long h = 0; h < H; h++) {
			FN(sparse_attn_bh)(q, k, coo, cstride, attn, b, h, T, H, W, E, mx, use_softmax);
			for (long c = 0; c < E; c++) {
				long dst = coo[c * cstride + 0], src = coo[c * cstride + 1], r = coo[c * cstride + 2];
				REAL a = attn[IX4(b, dst, r, h, T, mx, H)];
				for (long w = 0; w < W; w++)
					vo[IX4(b, dst, h, w, T, H, W)] += a * vf[IX4(b, src, h, w, T, H, W)];
				for (long w = 0; w < W; w++)
					vo[IX4(b, src, h, w, T, H, W)] += a * vb[IX4(b, dst, h, w, T, H, W)];
			}
		}
	}
}

/* cpp/l1attn_sparse_bidi_drv.cpp:103-212 */
void FN(oracle_bidi_bwd)(const REAL *dvo, const REAL *vf, const REAL *vb,
                         const REAL *q, const REAL *k,
                         const int *coo, long cstride, const REAL *attn,
                         REAL *dvf, REAL *dvb, REAL *dq, REAL *dk, REAL *scratch,
                         long B, long T, long H, long W, long E, long mx,
                         int use_softmax, int jac_mode)
{
	size_t n = (size_t)(B * T * H * W), na = (size_t)(B * T * mx * H);
	REAL *dattn_sm = scratch, *dattn = scratch + na;
	memset(dvf, 0, sizeof(REAL) * n);
	memset(dvb, 0, sizeof(REAL) * n);
	memset(dq, 0, sizeof(REAL) * n);
	memset(dk, 0, sizeof(REAL) * n);
	memset(scratch, 0, sizeof(REAL) * 2 * na);
	#pragma omp parallel for collapse(2) schedule(static)
	for (long b = 0; b < B; b++) {
		for (long h = 0; h < H; h++) {
			for (long c = 0; c < E; c++) {
				long dst = coo[c * cstride + 0], src = coo[c * cstride + 1], r = coo[c * cstride + 2];
				REAL a = attn[IX4(b, dst, r, h, T, mx, H)];
				for (long w = 0; w < W; w++)
					dvf[IX4(b, src, h, w, T, H, W)] += a * dvo[IX4(b, dst, h, w, T, H, W)];
				for (long w = 0; w < W; w++)
					dvb[IX4(b, dst, h, w, T, H, W)] += a * dvo[IX4(b, src, h, w, T, H, W)];
				for (long w = 0; w < W; w++)
					dattn_sm[IX4(b, dst, r, h, T, mx, H)] +=
						vf[IX4(b, src, h, w, T, H, W)] * dvo[IX4(b, dst, h, w, T, H, W)];
				for (long w = 0; w < W; w++)
					dattn_sm[IX4(b, dst, r, h, T, mx, H)] +=
						vb[IX4(b, dst, h, w, T, H, W)] * dvo[IX4(b, src, h, w, T, H, W)];
			}
			FN(sparse_jac_bh)(attn, dattn_sm, dattn, b, h, T, H, mx, use_softmax, jac_mode);
			FN(sparse_dqdk_bh)(q, k, coo, cstride, dattn, dq, dk, b, h, T, H, W, E, mx);
		}
	}
}

#undef IX4
