/*
 * dpsc_oracle.c -- CPU restatement of the sumcheck prover path.
 * TEST INFRASTRUCTURE ONLY: see dpsc_oracle.h for what this file is, what it
 * follows in the reference and which parts of parity are unpinned.
 */
#include "dpsc_oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef unsigned __int128 u128;
#define P ORC_P

/* ------------------------------------------------------------------ */
/* Goldilocks                                                          */
/* ------------------------------------------------------------------ */

uint64_t orc_gl_add(uint64_t a, uint64_t b)
{
    u128 s = (u128)a + b;
    if (s >= P) s -= P;
    return (uint64_t)s;
}

uint64_t orc_gl_sub(uint64_t a, uint64_t b) { return a >= b ? a - b : (uint64_t)((u128)a + P - b); }

uint64_t orc_gl_neg(uint64_t a) { return a ? P - a : 0; }

#ifdef ORC_FAST_REDUCE
/* Build variant used only as the timed CPU baseline: the same product reduced
 * with 2^64 = 2^32 - 1 and 2^96 = -1 instead of a 128-bit division.  The test
 * suite checks it against the plain variant. */
uint64_t orc_gl_mul(uint64_t a, uint64_t b)
{
    u128 x = (u128)a * b;
    uint64_t lo = (uint64_t)x, hi = (uint64_t)(x >> 64);
    uint64_t hh = hi >> 32, hl = hi & 0xFFFFFFFFu;
    u128 t = (u128)lo + (u128)hl * 0xFFFFFFFFu + P - hh; /* < 2^64 + 2^64 + 2^64 */
    uint64_t tl = (uint64_t)t, th = (uint64_t)(t >> 64); /* th <= 2 */
    u128 u = (u128)tl + th * 0xFFFFFFFFull;
    uint64_t r = (uint64_t)u;
    if (u >> 64) r += 0xFFFFFFFFull;
    return r >= P ? r - P : r;
}
#else
uint64_t orc_gl_mul(uint64_t a, uint64_t b) { return (uint64_t)(((u128)a * b) % P); }
#endif

uint64_t orc_gl_pow(uint64_t a, uint64_t e)
{
    uint64_t r = 1;
    while (e) {
        if (e & 1) r = orc_gl_mul(r, a);
        a = orc_gl_mul(a, a);
        e >>= 1;
    }
    return r;
}

uint64_t orc_gl_inv(uint64_t a) { return orc_gl_pow(a, P - 2); }

uint64_t orc_gl_from_i64(int64_t x)
{
    if (x >= 0) return (uint64_t)x % P;
    /* |x| computed in unsigned arithmetic so INT64_MIN is handled */
    uint64_t mag = (uint64_t)0 - (uint64_t)x;
    return orc_gl_neg(mag % P);
}

int64_t orc_gl_to_i64(uint64_t x)
{
    if (x > (P - 1) / 2) return -(int64_t)(P - x);
    return (int64_t)x;
}

/* ------------------------------------------------------------------ */
/* F_p[X]/(X^2 - 7)                                                    */
/* ------------------------------------------------------------------ */

static inline orc_e2 e2(uint64_t c0, uint64_t c1)
{
    orc_e2 r = {c0, c1};
    return r;
}
static inline orc_e2 e2_add(orc_e2 a, orc_e2 b) { return e2(orc_gl_add(a.c0, b.c0), orc_gl_add(a.c1, b.c1)); }
static inline orc_e2 e2_sub(orc_e2 a, orc_e2 b) { return e2(orc_gl_sub(a.c0, b.c0), orc_gl_sub(a.c1, b.c1)); }
static inline orc_e2 e2_mul(orc_e2 a, orc_e2 b)
{
    /* (a0 + a1 X)(b0 + b1 X) = a0 b0 + 7 a1 b1 + (a0 b1 + a1 b0) X, schoolbook */
    uint64_t c0 = orc_gl_add(orc_gl_mul(a.c0, b.c0), orc_gl_mul(ORC_W, orc_gl_mul(a.c1, b.c1)));
    uint64_t c1 = orc_gl_add(orc_gl_mul(a.c0, b.c1), orc_gl_mul(a.c1, b.c0));
    return e2(c0, c1);
}
static inline orc_e2 e2_from_u64(uint64_t x) { return e2(x % P, 0); }
static inline int e2_eq(orc_e2 a, orc_e2 b) { return a.c0 == b.c0 && a.c1 == b.c1; }
static const orc_e2 E2_ZERO = {0, 0};
static const orc_e2 E2_ONE = {1, 0};

static orc_e2 e2_inv(orc_e2 a)
{
    /* 1/(a0 + a1 X) = (a0 - a1 X)/(a0^2 - 7 a1^2) */
    uint64_t norm = orc_gl_sub(orc_gl_mul(a.c0, a.c0), orc_gl_mul(ORC_W, orc_gl_mul(a.c1, a.c1)));
    uint64_t ni = orc_gl_inv(norm);
    return e2(orc_gl_mul(a.c0, ni), orc_gl_mul(orc_gl_neg(a.c1), ni));
}

void orc_e2_add(const orc_e2 *a, const orc_e2 *b, orc_e2 *out) { *out = e2_add(*a, *b); }
void orc_e2_sub(const orc_e2 *a, const orc_e2 *b, orc_e2 *out) { *out = e2_sub(*a, *b); }
void orc_e2_mul(const orc_e2 *a, const orc_e2 *b, orc_e2 *out) { *out = e2_mul(*a, *b); }
void orc_e2_inv(const orc_e2 *a, orc_e2 *out) { *out = e2_inv(*a); }

/* ------------------------------------------------------------------ */
/* tables                                                              */
/* ------------------------------------------------------------------ */

void orc_eq_evals(const orc_e2 *point, uint32_t m, orc_e2 *out)
{
    /* Doubling from the highest variable down, so that point[j] ends up on
     * index bit j: after processing point[j..m) the table is indexed by the
     * bits j..m-1 shifted down; prepending variable j-1 interleaves. */
    out[0] = E2_ONE;
    uint64_t len = 1;
    for (uint32_t jj = m; jj-- > 0;) {
        orc_e2 r = point[jj];
        orc_e2 one_minus = e2_sub(E2_ONE, r);
        /* new[2i] = old[i]*(1-r), new[2i+1] = old[i]*r ; go backwards in place */
        for (uint64_t i = len; i-- > 0;) {
            orc_e2 v = out[i];
            out[2 * i + 1] = e2_mul(v, r);
            out[2 * i] = e2_mul(v, one_minus);
        }
        len <<= 1;
    }
}

void orc_identity_eval(const orc_e2 *r1, const orc_e2 *r2, uint32_t len, orc_e2 *out)
{
    orc_e2 acc = E2_ONE;
    for (uint32_t i = 0; i < len; i++) {
        orc_e2 a = e2_mul(r1[i], r2[i]);
        orc_e2 b = e2_mul(e2_sub(E2_ONE, r1[i]), e2_sub(E2_ONE, r2[i]));
        acc = e2_mul(acc, e2_add(a, b));
    }
    *out = acc;
}

void orc_embed_base(const uint64_t *in, uint64_t len, orc_e2 *out)
{
    for (uint64_t i = 0; i < len; i++) out[i] = e2(in[i] % P, 0);
}

void orc_embed_i64(const int64_t *in, uint64_t len, orc_e2 *out)
{
    for (uint64_t i = 0; i < len; i++) out[i] = e2(orc_gl_from_i64(in[i]), 0);
}

static void fold_low_into(const orc_e2 *src, uint64_t half, orc_e2 r, orc_e2 *dst)
{
#pragma omp parallel for schedule(static) if (half >= (1u << 14))
    for (uint64_t i = 0; i < half; i++) {
        orc_e2 lo = src[2 * i], hi = src[2 * i + 1];
        dst[i] = e2_add(lo, e2_mul(r, e2_sub(hi, lo)));
    }
}

void orc_mle_fix_low(const orc_e2 *tbl, uint32_t n, const orc_e2 *point, uint32_t k, orc_e2 *out)
{
    uint64_t len = (uint64_t)1 << n;
    orc_e2 *cur = (orc_e2 *)malloc(len * sizeof(orc_e2));
    memcpy(cur, tbl, len * sizeof(orc_e2));
    for (uint32_t j = 0; j < k; j++) {
        len >>= 1;
        /* in place is safe going upwards: dst[i] is written after src[2i], src[2i+1] are read */
        for (uint64_t i = 0; i < len; i++) {
            orc_e2 lo = cur[2 * i], hi = cur[2 * i + 1];
            cur[i] = e2_add(lo, e2_mul(point[j], e2_sub(hi, lo)));
        }
    }
    memcpy(out, cur, len * sizeof(orc_e2));
    free(cur);
}

void orc_mle_fix_high(const orc_e2 *tbl, uint32_t n, const orc_e2 *point, uint32_t k, orc_e2 *out)
{
    uint64_t len = (uint64_t)1 << n;
    orc_e2 *cur = (orc_e2 *)malloc(len * sizeof(orc_e2));
    memcpy(cur, tbl, len * sizeof(orc_e2));
    /* bind the top variable first: point[k-1] binds variable n-1 */
    for (uint32_t j = k; j-- > 0;) {
        len >>= 1;
        for (uint64_t i = 0; i < len; i++) {
            orc_e2 lo = cur[i], hi = cur[i + len];
            cur[i] = e2_add(lo, e2_mul(point[j], e2_sub(hi, lo)));
        }
    }
    memcpy(out, cur, len * sizeof(orc_e2));
    free(cur);
}

void orc_mle_evaluate(const orc_e2 *tbl, uint32_t n, const orc_e2 *point, orc_e2 *out)
{
    orc_mle_fix_low(tbl, n, point, n, out);
}

/* ------------------------------------------------------------------ */
/* BLAKE3, hash mode.  Restated from the published specification       */
/* (the reference uses the `blake3` crate through dp-crypto).          */
/* ------------------------------------------------------------------ */

static const uint32_t B3_IV[8] = {0x6A09E667u, 0xBB67AE85u, 0x3C6EF372u, 0xA54FF53Au,
                                  0x510E527Fu, 0x9B05688Cu, 0x1F83D9ABu, 0x5BE0CD19u};
static const uint8_t B3_PERM[16] = {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8};
enum { B3_CHUNK_START = 1, B3_CHUNK_END = 2, B3_PARENT = 4, B3_ROOT = 8 };

static inline uint32_t rotr32(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

static inline void b3_g(uint32_t *s, int a, int b, int c, int d, uint32_t mx, uint32_t my)
{
    s[a] = s[a] + s[b] + mx;
    s[d] = rotr32(s[d] ^ s[a], 16);
    s[c] = s[c] + s[d];
    s[b] = rotr32(s[b] ^ s[c], 12);
    s[a] = s[a] + s[b] + my;
    s[d] = rotr32(s[d] ^ s[a], 8);
    s[c] = s[c] + s[d];
    s[b] = rotr32(s[b] ^ s[c], 7);
}

static void b3_compress(const uint32_t cv[8], const uint8_t block[64], uint64_t counter,
                        uint32_t block_len, uint32_t flags, uint32_t out[16])
{
    uint32_t m[16], s[16];
    for (int i = 0; i < 16; i++)
        m[i] = (uint32_t)block[4 * i] | ((uint32_t)block[4 * i + 1] << 8) |
               ((uint32_t)block[4 * i + 2] << 16) | ((uint32_t)block[4 * i + 3] << 24);
    for (int i = 0; i < 8; i++) s[i] = cv[i];
    for (int i = 0; i < 4; i++) s[8 + i] = B3_IV[i];
    s[12] = (uint32_t)counter;
    s[13] = (uint32_t)(counter >> 32);
    s[14] = block_len;
    s[15] = flags;
    for (int r = 0; r < 7; r++) {
        b3_g(s, 0, 4, 8, 12, m[0], m[1]);
        b3_g(s, 1, 5, 9, 13, m[2], m[3]);
        b3_g(s, 2, 6, 10, 14, m[4], m[5]);
        b3_g(s, 3, 7, 11, 15, m[6], m[7]);
        b3_g(s, 0, 5, 10, 15, m[8], m[9]);
        b3_g(s, 1, 6, 11, 12, m[10], m[11]);
        b3_g(s, 2, 7, 8, 13, m[12], m[13]);
        b3_g(s, 3, 4, 9, 14, m[14], m[15]);
        if (r < 6) {
            uint32_t t[16];
            for (int i = 0; i < 16; i++) t[i] = m[B3_PERM[i]];
            memcpy(m, t, sizeof m);
        }
    }
    for (int i = 0; i < 8; i++) {
        out[i] = s[i] ^ s[i + 8];
        out[i + 8] = s[i + 8] ^ cv[i];
    }
}

/* chaining value of one chunk (<= 1024 bytes); extra flags (ROOT) go on the last block */
static void b3_chunk_cv(const uint8_t *in, size_t len, uint64_t chunk_index, uint32_t last_flags,
                        uint32_t cv_out[8])
{
    uint32_t cv[8], out[16];
    memcpy(cv, B3_IV, sizeof cv);
    size_t n_blocks = len == 0 ? 1 : (len + 63) / 64;
    for (size_t b = 0; b < n_blocks; b++) {
        uint8_t block[64] = {0};
        size_t off = b * 64;
        size_t bl = len - off < 64 ? len - off : 64;
        if (len == 0) bl = 0;
        memcpy(block, in + off, bl);
        uint32_t flags = 0;
        if (b == 0) flags |= B3_CHUNK_START;
        if (b == n_blocks - 1) flags |= B3_CHUNK_END | last_flags;
        b3_compress(cv, block, chunk_index, (uint32_t)bl, flags, out);
        memcpy(cv, out, sizeof cv);
    }
    memcpy(cv_out, cv, sizeof cv);
}

/* recursive tree: the left subtree takes the largest power-of-two number of
 * chunks that leaves at least one byte for the right subtree */
static void b3_subtree_cv(const uint8_t *in, size_t len, uint64_t chunk_index, int is_root,
                          uint32_t cv_out[8])
{
    if (len <= 1024) {
        b3_chunk_cv(in, len, chunk_index, is_root ? B3_ROOT : 0, cv_out);
        return;
    }
    size_t full_chunks = (len - 1) / 1024; /* chunks that certainly stay left of the last byte */
    size_t left_chunks = 1;
    while (left_chunks * 2 <= full_chunks) left_chunks *= 2;
    size_t left_len = left_chunks * 1024;
    uint32_t l[8], r[8], out[16];
    b3_subtree_cv(in, left_len, chunk_index, 0, l);
    b3_subtree_cv(in + left_len, len - left_len, chunk_index + left_chunks, 0, r);
    uint8_t block[64];
    for (int i = 0; i < 8; i++) {
        for (int k = 0; k < 4; k++) {
            block[4 * i + k] = (uint8_t)(l[i] >> (8 * k));
            block[32 + 4 * i + k] = (uint8_t)(r[i] >> (8 * k));
        }
    }
    b3_compress(B3_IV, block, 0, 64, B3_PARENT | (is_root ? B3_ROOT : 0), out);
    memcpy(cv_out, out, 8 * sizeof(uint32_t));
}

void orc_blake3(const uint8_t *in, size_t len, uint8_t out[32])
{
    uint32_t cv[8];
    b3_subtree_cv(in, len, 0, 1, cv);
    for (int i = 0; i < 8; i++)
        for (int k = 0; k < 4; k++) out[4 * i + k] = (uint8_t)(cv[i] >> (8 * k));
}

/* ------------------------------------------------------------------ */
/* Transcript.  Mirrors the method set the reference calls              */
/* (zkml/src/lib.rs:106-108,176-184; einsum/prove.rs:158;              */
/* logup_gkr/prover.rs:163-173,261,284-288).  The byte layout is this  */
/* repository's own (PARITY UNPINNED, the reference's is in dp-crypto): */
/*   state' = BLAKE3(state || 28 zero bytes || be32(n_rounds) || payload) */
/* ------------------------------------------------------------------ */

static void tr_absorb(orc_transcript *t, const uint8_t *payload, size_t len)
{
    uint8_t stackbuf[64 + 256];
    uint8_t *buf = len <= 256 ? stackbuf : (uint8_t *)malloc(64 + len);
    memcpy(buf, t->state, 32);
    memset(buf + 32, 0, 28);
    buf[60] = (uint8_t)(t->n_rounds >> 24);
    buf[61] = (uint8_t)(t->n_rounds >> 16);
    buf[62] = (uint8_t)(t->n_rounds >> 8);
    buf[63] = (uint8_t)(t->n_rounds);
    if (len) memcpy(buf + 64, payload, len);
    orc_blake3(buf, 64 + len, t->state);
    t->n_rounds += 1;
    if (buf != stackbuf) free(buf);
}

void orc_tr_new(orc_transcript *t, const uint8_t *label, size_t len)
{
    uint8_t padded[32] = {0};
    memcpy(padded, label, len < 32 ? len : 32);
    orc_blake3(padded, 32, t->state);
    t->n_rounds = 0;
}

void orc_tr_append_message(orc_transcript *t, const uint8_t *label, size_t len)
{
    uint8_t padded[32] = {0};
    memcpy(padded, label, len < 32 ? len : 32);
    tr_absorb(t, padded, 32);
}

void orc_tr_append_bytes(orc_transcript *t, const uint8_t *bytes, size_t len) { tr_absorb(t, bytes, len); }

void orc_tr_append_u64(orc_transcript *t, uint64_t x)
{
    uint8_t buf[32] = {0};
    for (int i = 0; i < 8; i++) buf[24 + i] = (uint8_t)(x >> (56 - 8 * i));
    tr_absorb(t, buf, 32);
}

void orc_tr_append_scalar(orc_transcript *t, const orc_e2 *x)
{
    /* big-endian c1 then big-endian c0 (the byte reversal of le(c0) || le(c1)) */
    uint8_t buf[16];
    for (int i = 0; i < 8; i++) {
        buf[i] = (uint8_t)(x->c1 >> (56 - 8 * i));
        buf[8 + i] = (uint8_t)(x->c0 >> (56 - 8 * i));
    }
    tr_absorb(t, buf, 16);
}

void orc_tr_append_scalars(orc_transcript *t, const orc_e2 *xs, size_t n)
{
    orc_tr_append_message(t, (const uint8_t *)"begin_append_vector", 19);
    for (size_t i = 0; i < n; i++) orc_tr_append_scalar(t, &xs[i]);
    orc_tr_append_message(t, (const uint8_t *)"end_append_vector", 17);
}

void orc_tr_challenge_scalar(orc_transcript *t, orc_e2 *out)
{
    tr_absorb(t, NULL, 0);
    uint64_t w0 = 0, w1 = 0;
    for (int i = 0; i < 8; i++) {
        w0 |= (uint64_t)t->state[i] << (8 * i);
        w1 |= (uint64_t)t->state[8 + i] << (8 * i);
    }
    out->c0 = w0 % P;
    out->c1 = w1 % P;
}

void orc_tr_append_and_sample(orc_transcript *t, const uint8_t *label, size_t len, orc_e2 *out)
{
    orc_tr_append_message(t, label, len);
    orc_tr_challenge_scalar(t, out);
}

/* ------------------------------------------------------------------ */
/* Sumcheck                                                            */
/* ------------------------------------------------------------------ */

uint32_t orc_terms_degree(const orc_term *terms, uint32_t n_terms)
{
    uint32_t d = 0;
    for (uint32_t i = 0; i < n_terms; i++)
        if (terms[i].n_factors > d) d = terms[i].n_factors;
    return d;
}

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_sc_round_poly(uint32_t live, uint32_t n_mles, const orc_e2 *const *tables,
                       const uint32_t *cur_nvars, const orc_term *terms, uint32_t n_terms,
                       uint32_t degree, orc_e2 *evals_out)
{
    (void)n_mles;
    uint64_t pairs = (uint64_t)1 << (live - 1);
    uint32_t npts = degree + 1;
    for (uint32_t t = 0; t < npts; t++) evals_out[t] = E2_ZERO;
    for (uint32_t ti = 0; ti < n_terms; ti++) {
        const orc_term *tm = &terms[ti];
        orc_e2 acc[ORC_MAX_FACTORS + 1];
        for (uint32_t t = 0; t < npts; t++) acc[t] = E2_ZERO;
#pragma omp parallel if (pairs >= (1u << 12))
        {
            orc_e2 local[ORC_MAX_FACTORS + 1];
            for (uint32_t t = 0; t < npts; t++) local[t] = E2_ZERO;
#pragma omp for schedule(static) nowait
            for (uint64_t i = 0; i < pairs; i++) {
                orc_e2 lo[ORC_MAX_FACTORS], dl[ORC_MAX_FACTORS];
                for (uint32_t f = 0; f < tm->n_factors; f++) {
                    uint32_t k = tm->factors[f];
                    if (cur_nvars[k] >= live) {
                        lo[f] = tables[k][2 * i];
                        dl[f] = e2_sub(tables[k][2 * i + 1], lo[f]);
                    } else {
                        /* fewer variables than the round: constant in the low ones */
                        lo[f] = tables[k][i >> (live - 1 - cur_nvars[k])];
                        dl[f] = E2_ZERO;
                    }
                }
                for (uint32_t t = 0; t < npts; t++) {
                    orc_e2 prod = E2_ONE;
                    for (uint32_t f = 0; f < tm->n_factors; f++) {
                        prod = e2_mul(prod, lo[f]);
                        lo[f] = e2_add(lo[f], dl[f]); /* value at t+1 */
                    }
                    local[t] = e2_add(local[t], prod);
                }
            }
#pragma omp critical
            for (uint32_t t = 0; t < npts; t++) acc[t] = e2_add(acc[t], local[t]);
        }
        for (uint32_t t = 0; t < npts; t++) evals_out[t] = e2_add(evals_out[t], e2_mul(tm->coeff, acc[t]));
    }
}

int orc_sc_prove(uint32_t n_vars, uint32_t n_mles, const orc_e2 *const *tables,
                 const uint32_t *mle_nvars, const orc_term *terms, uint32_t n_terms,
                 orc_transcript *tr, orc_e2 *proof_out, orc_e2 *point_out, orc_e2 *final_out)
{
    for (uint32_t k = 0; k < n_mles; k++)
        if (mle_nvars[k] > n_vars) return -1;
    for (uint32_t i = 0; i < n_terms; i++) {
        if (terms[i].n_factors > ORC_MAX_FACTORS) return -2;
        for (uint32_t f = 0; f < terms[i].n_factors; f++)
            if (terms[i].factors[f] >= n_mles) return -3;
    }
    uint32_t degree = orc_terms_degree(terms, n_terms);
    uint32_t npts = degree + 1;

    /* private copies: the caller's tables are borrowed */
    orc_e2 **cur = (orc_e2 **)calloc(n_mles ? n_mles : 1, sizeof(orc_e2 *));
    uint32_t *cur_nv = (uint32_t *)calloc(n_mles ? n_mles : 1, sizeof(uint32_t));
    for (uint32_t k = 0; k < n_mles; k++) {
        uint64_t len = (uint64_t)1 << mle_nvars[k];
        cur[k] = (orc_e2 *)malloc(len * sizeof(orc_e2));
        memcpy(cur[k], tables[k], len * sizeof(orc_e2));
        cur_nv[k] = mle_nvars[k];
    }

    orc_tr_append_u64(tr, n_vars);
    orc_tr_append_u64(tr, degree);

    for (uint32_t j = 1; j <= n_vars; j++) {
        uint32_t live = n_vars - j + 1;
        orc_e2 *msg = proof_out + (size_t)(j - 1) * npts;
        orc_sc_round_poly(live, n_mles, (const orc_e2 *const *)cur, cur_nv, terms, n_terms, degree, msg);
        orc_tr_append_scalars(tr, msg, npts);
        orc_e2 r;
        orc_tr_challenge_scalar(tr, &r);
        point_out[j - 1] = r;
        for (uint32_t k = 0; k < n_mles; k++) {
            if (cur_nv[k] == live) {
                uint64_t half = (uint64_t)1 << (live - 1);
                orc_e2 *dst = (orc_e2 *)malloc(half * sizeof(orc_e2));
                fold_low_into(cur[k], half, r, dst);
                free(cur[k]);
                cur[k] = dst;
                cur_nv[k] = live - 1;
            }
        }
    }
    for (uint32_t k = 0; k < n_mles; k++) {
        final_out[k] = cur[k][0];
        free(cur[k]);
    }
    free(cur);
    free(cur_nv);
    return 0;
}

void orc_interpolate(const orc_e2 *evals, uint32_t degree, const orc_e2 *r, orc_e2 *out)
{
    /* Lagrange over the nodes 0..degree */
    orc_e2 acc = E2_ZERO;
    for (uint32_t k = 0; k <= degree; k++) {
        orc_e2 num = E2_ONE;
        uint64_t den = 1;
        for (uint32_t m = 0; m <= degree; m++) {
            if (m == k) continue;
            num = e2_mul(num, e2_sub(*r, e2_from_u64(m)));
            den = orc_gl_mul(den, orc_gl_sub(k, m));
        }
        orc_e2 w = e2_mul(num, e2(orc_gl_inv(den), 0));
        acc = e2_add(acc, e2_mul(w, evals[k]));
    }
    *out = acc;
}

int orc_sc_verify(const orc_e2 *claimed_sum, const orc_e2 *proof, uint32_t n_vars,
                  uint32_t degree, orc_transcript *tr, orc_e2 *point_out, orc_e2 *expected_out)
{
    uint32_t npts = degree + 1;
    orc_e2 claim = *claimed_sum;
    int bad = 0;
    orc_tr_append_u64(tr, n_vars);
    orc_tr_append_u64(tr, degree);
    for (uint32_t j = 1; j <= n_vars; j++) {
        const orc_e2 *msg = proof + (size_t)(j - 1) * npts;
        if (!bad && !e2_eq(e2_add(msg[0], msg[1]), claim)) bad = (int)j;
        orc_tr_append_scalars(tr, msg, npts);
        orc_e2 r;
        orc_tr_challenge_scalar(tr, &r);
        point_out[j - 1] = r;
        orc_interpolate(msg, degree, &r, &claim);
    }
    *expected_out = claim;
    return bad;
}

/* ------------------------------------------------------------------ */
/* Einsum partial evaluation                                           */
/* ------------------------------------------------------------------ */

static uint32_t ceil_log2_u64(uint64_t x)
{
    uint32_t l = 0;
    while (((uint64_t)1 << l) < x) l++;
    return l;
}

int64_t orc_partial_eval(const int64_t *tensor, const uint64_t *padded_dims,
                         const uint64_t *unpadded_dims, uint32_t n_dims, const int32_t *kinds,
                         const orc_e2 *const *points, orc_e2 *out, uint64_t out_cap,
                         uint64_t *table_len)
{
    /* axis.rs:1148 reduce_to_shape: gather the unpadded region, row-major */
    uint64_t total = 1;
    for (uint32_t a = 0; a < n_dims; a++) total *= unpadded_dims[a];
    orc_e2 *cur = (orc_e2 *)malloc((total ? total : 1) * sizeof(orc_e2));
    {
        uint64_t idx[16] = {0};
        if (n_dims > 16) {
            free(cur);
            return -1;
        }
        for (uint64_t flat = 0; flat < total; flat++) {
            uint64_t src = 0;
            for (uint32_t a = 0; a < n_dims; a++) src = src * padded_dims[a] + idx[a];
            cur[flat] = e2(orc_gl_from_i64(tensor[src]), 0);
            for (uint32_t a = n_dims; a-- > 0;) {
                if (++idx[a] < unpadded_dims[a]) break;
                idx[a] = 0;
            }
        }
    }
    uint64_t cur_len = total;
    uint64_t chunk = 1, contraction = 1;
    /* axis.rs:1152-1214: fold over the axes from the last to the first */
    for (uint32_t a = n_dims; a-- > 0;) {
        uint64_t dim = unpadded_dims[a];
        if (kinds[a] == ORC_AXIS_OUTER) {
            uint32_t m = ceil_log2_u64(padded_dims[a]);
            orc_e2 *beta = (orc_e2 *)malloc(((uint64_t)1 << m) * sizeof(orc_e2));
            orc_eq_evals(points[a], m, beta); /* evals(point)[..size], axis.rs:1032 */
            uint64_t groups = cur_len / (chunk * dim);
            orc_e2 *next = (orc_e2 *)malloc((groups * chunk + 1) * sizeof(orc_e2));
            for (uint64_t g = 0; g < groups; g++) {
                const orc_e2 *full = cur + g * chunk * dim;
                for (uint64_t i = 0; i < chunk; i++) {
                    orc_e2 s = E2_ZERO;
                    for (uint64_t k = 0; k < dim; k++) s = e2_add(s, e2_mul(full[i + k * chunk], beta[k]));
                    next[g * chunk + i] = s;
                }
            }
            free(beta);
            free(cur);
            cur = next;
            cur_len = groups * chunk;
        } else if (kinds[a] == ORC_AXIS_STACKED) {
            chunk *= dim;
        } else {
            chunk *= dim;
            contraction *= dim;
        }
    }
    /* axis.rs:1217-1233: split into stacks, zero-pad each to a power of two */
    uint32_t nv = ceil_log2_u64(contraction);
    uint64_t tl = (uint64_t)1 << nv;
    uint64_t n_stack = contraction ? cur_len / contraction : 0;
    *table_len = tl;
    if (n_stack * tl > out_cap) {
        free(cur);
        return -2;
    }
    for (uint64_t s = 0; s < n_stack; s++) {
        for (uint64_t i = 0; i < tl; i++)
            out[s * tl + i] = i < contraction ? cur[s * contraction + i] : E2_ZERO;
    }
    free(cur);
    return (int64_t)n_stack;
}

int64_t orc_stacking_coeffs(const uint64_t *padded_dims, const uint64_t *unpadded_dims,
                            uint32_t n_dims, const int32_t *kinds, const orc_e2 *const *points,
                            orc_e2 *out, uint64_t out_cap)
{
    /* axis.rs:1046-1060: fold over reversed axes; each stacked axis b-table is the
     * new slow index: acc' = [b * a for b in beta for a in acc] */
    uint64_t len = 1;
    orc_e2 *acc = (orc_e2 *)malloc(sizeof(orc_e2));
    acc[0] = E2_ONE;
    for (uint32_t a = n_dims; a-- > 0;) {
        if (kinds[a] != ORC_AXIS_STACKED) continue;
        uint32_t m = ceil_log2_u64(padded_dims[a]);
        orc_e2 *beta = (orc_e2 *)malloc(((uint64_t)1 << m) * sizeof(orc_e2));
        orc_eq_evals(points[a], m, beta);
        uint64_t dim = unpadded_dims[a];
        orc_e2 *next = (orc_e2 *)malloc((dim * len + 1) * sizeof(orc_e2));
        for (uint64_t b = 0; b < dim; b++)
            for (uint64_t i = 0; i < len; i++) next[b * len + i] = e2_mul(acc[i], beta[b]);
        free(beta);
        free(acc);
        acc = next;
        len *= dim;
    }
    if (len > out_cap) {
        free(acc);
        return -2;
    }
    memcpy(out, acc, len * sizeof(orc_e2));
    free(acc);
    return (int64_t)len;
}

/* ------------------------------------------------------------------ */
/* LogUp-GKR                                                           */
/* ------------------------------------------------------------------ */

uint64_t orc_logup_layer_offset(uint64_t len, uint32_t k)
{
    /* layer k >= 1 has len>>k entries per array, two arrays */
    uint64_t off = 0;
    for (uint32_t j = 1; j < k; j++) off += 2 * (len >> j);
    return off;
}

uint64_t orc_logup_arena_len(uint64_t len)
{
    uint32_t top = ceil_log2_u64(len);
    /* layers 1 .. top-1: the last one has 2 entries per array (circuit.rs:82-92) */
    return orc_logup_layer_offset(len, top);
}

static orc_e2 logup_denominator(const uint64_t *const *cols, uint32_t n_cols, uint64_t i, orc_e2 c,
                                orc_e2 beta)
{
    /* circuit.rs:129-141: c + sum_k beta^k * col_k[i] */
    orc_e2 acc = c, pw = E2_ONE;
    for (uint32_t k = 0; k < n_cols; k++) {
        acc = e2_add(acc, e2_mul(pw, e2(cols[k][i] % P, 0)));
        pw = e2_mul(pw, beta);
    }
    return acc;
}

void orc_logup_build(const uint64_t *const *cols, uint32_t n_cols, const uint64_t *numer,
                     uint64_t len, const orc_e2 *c, const orc_e2 *beta, orc_e2 *arena)
{
    uint32_t top = ceil_log2_u64(len);
    if (top < 2) return; /* a 2-entry instance has only its input layer */
    uint64_t half = len >> 1;
    orc_e2 *num1 = arena, *den1 = arena + half;
    orc_e2 minus_one = e2(P - 1, 0);
#pragma omp parallel for schedule(static) if (half >= (1u << 14))
    for (uint64_t i = 0; i < half; i++) {
        orc_e2 d1 = logup_denominator(cols, n_cols, i, *c, *beta);
        orc_e2 d2 = logup_denominator(cols, n_cols, i + half, *c, *beta);
        orc_e2 n1 = numer ? e2(numer[i] % P, 0) : minus_one;
        orc_e2 n2 = numer ? e2(numer[i + half] % P, 0) : minus_one;
        /* structs.rs:48-58: n1 d2 + d1 n2 , d1 d2 */
        num1[i] = e2_add(e2_mul(n1, d2), e2_mul(d1, n2));
        den1[i] = e2_mul(d1, d2);
    }
    for (uint32_t k = 2; k < top; k++) {
        uint64_t prev_len = len >> (k - 1), cur_len = len >> k;
        const orc_e2 *pn = arena + orc_logup_layer_offset(len, k - 1), *pd = pn + prev_len;
        orc_e2 *cn = arena + orc_logup_layer_offset(len, k), *cd = cn + cur_len;
#pragma omp parallel for schedule(static) if (cur_len >= (1u << 14))
        for (uint64_t i = 0; i < cur_len; i++) {
            cn[i] = e2_add(e2_mul(pn[i], pd[i + cur_len]), e2_mul(pd[i], pn[i + cur_len]));
            cd[i] = e2_mul(pd[i], pd[i + cur_len]);
        }
    }
}

/*
 * Batched prover.  Circuit c (one per instance) has layers 0 (input, len_c
 * entries per column) .. top_c - 1 (output, 2 entries per array); its
 * num_vars is top_c - 1 (circuit.rs:67-80,564-566).
 *
 * Output stream (elements), in this order:
 *   for v = 1..total_layers:
 *        sumcheck proof of round v        v * 4 elements (degree 3)
 *        round evaluations                 n_evals(v) elements
 *   output claim evaluations              one per (multiplicity +) column per instance
 *   circuit outputs                       4 per instance (n_lo, n_hi, d_lo, d_hi)
 * followed by nothing else; the final point (total_layers + 1 elements) is
 * appended after the circuit outputs.
 */

typedef struct {
    uint32_t nv;      /* num_vars of the circuit = log2(len) - 1 */
    uint32_t n_evals; /* evaluations this circuit contributes in the last round */
    orc_e2 *arena;    /* layers 1.. */
} lg_circ;

/* MLE views of circuit `ci` at the layer with `lv` variables (lv >= 1):
 * appended to tabs/nvs; returns how many were appended. */
static uint32_t lg_layer_mles(const orc_logup_instance *in, const lg_circ *cc, uint32_t lv,
                              orc_e2 **scratch_list, uint32_t *n_scratch, const orc_e2 **tabs,
                              uint32_t *nvs)
{
    uint64_t half = (uint64_t)1 << lv;
    if (lv < cc->nv) {
        /* generic layer k with len>>k == 2*half */
        uint32_t k = 0;
        while ((in->len >> k) != 2 * half) k++;
        const orc_e2 *num = cc->arena + orc_logup_layer_offset(in->len, k);
        const orc_e2 *den = num + 2 * half;
        tabs[0] = num;
        tabs[1] = num + half;
        tabs[2] = den;
        tabs[3] = den + half;
        for (int i = 0; i < 4; i++) nvs[i] = lv;
        return 4;
    }
    /* input layer: base columns embedded, halves as separate MLEs (circuit.rs:292-410) */
    uint32_t n = 0;
    if (in->numer) {
        orc_e2 *m = (orc_e2 *)malloc(in->len * sizeof(orc_e2));
        orc_embed_base(in->numer, in->len, m);
        scratch_list[(*n_scratch)++] = m;
        tabs[n] = m;
        nvs[n++] = lv;
        tabs[n] = m + half;
        nvs[n++] = lv;
    }
    uint32_t first_col = n;
    for (uint32_t k = 0; k < in->n_cols; k++) {
        orc_e2 *m = (orc_e2 *)malloc(in->len * sizeof(orc_e2));
        orc_embed_base(in->cols[k], in->len, m);
        scratch_list[(*n_scratch)++] = m;
        tabs[first_col + k] = m; /* all low halves first ... */
        nvs[first_col + k] = lv;
        tabs[first_col + in->n_cols + k] = m + half; /* ... then all high halves */
        nvs[first_col + in->n_cols + k] = lv;
    }
    return first_col + 2 * in->n_cols;
}

static void lg_push_term(orc_term *terms, uint32_t *n_terms, orc_e2 coeff, uint32_t nf, const uint32_t *f)
{
    orc_term *t = &terms[(*n_terms)++];
    t->coeff = coeff;
    t->n_factors = nf;
    for (uint32_t i = 0; i < nf; i++) t->factors[i] = f[i];
}

/* terms of  scale * eq * ( N_lo D_hi + N_hi D_lo + lambda D_lo D_hi )  where on the
 * input layer D_x = c + sum_k beta^k col_k,x and N_x is -1 (lookup) or the
 * multiplicity half (table); expanded into monomials by hand. */
static void lg_layer_terms(const orc_logup_instance *in, int is_input, uint32_t w0, uint32_t eq_id,
                           orc_e2 scale, orc_e2 lambda, orc_term *terms, uint32_t *n_terms)
{
    if (!is_input) {
        uint32_t f1[3] = {w0 + 0, w0 + 3, eq_id}, f2[3] = {w0 + 1, w0 + 2, eq_id}, f3[3] = {w0 + 2, w0 + 3, eq_id};
        lg_push_term(terms, n_terms, scale, 3, f1);
        lg_push_term(terms, n_terms, scale, 3, f2);
        lg_push_term(terms, n_terms, e2_mul(scale, lambda), 3, f3);
        return;
    }
    uint32_t C = in->n_cols;
    orc_e2 pw[64];
    pw[0] = E2_ONE;
    for (uint32_t k = 1; k < C; k++) pw[k] = e2_mul(pw[k - 1], in->beta);
    orc_e2 c = in->c;
    if (in->numer) {
        uint32_t nlo = w0, nhi = w0 + 1, lo0 = w0 + 2, hi0 = w0 + 2 + C;
        /* N_lo * (c + sum pw_k H_k) + N_hi * (c + sum pw_k L_k) */
        {
            uint32_t f[2] = {nlo, eq_id};
            lg_push_term(terms, n_terms, e2_mul(scale, c), 2, f);
            uint32_t g[2] = {nhi, eq_id};
            lg_push_term(terms, n_terms, e2_mul(scale, c), 2, g);
        }
        for (uint32_t k = 0; k < C; k++) {
            uint32_t f[3] = {nlo, hi0 + k, eq_id};
            lg_push_term(terms, n_terms, e2_mul(scale, pw[k]), 3, f);
            uint32_t g[3] = {nhi, lo0 + k, eq_id};
            lg_push_term(terms, n_terms, e2_mul(scale, pw[k]), 3, g);
        }
        /* lambda * D_lo * D_hi */
        orc_e2 sl = e2_mul(scale, lambda);
        {
            uint32_t f[1] = {eq_id};
            lg_push_term(terms, n_terms, e2_mul(sl, e2_mul(c, c)), 1, f);
        }
        for (uint32_t k = 0; k < C; k++) {
            uint32_t f[2] = {lo0 + k, eq_id};
            lg_push_term(terms, n_terms, e2_mul(sl, e2_mul(c, pw[k])), 2, f);
            uint32_t g[2] = {hi0 + k, eq_id};
            lg_push_term(terms, n_terms, e2_mul(sl, e2_mul(c, pw[k])), 2, g);
        }
        for (uint32_t a = 0; a < C; a++)
            for (uint32_t b = 0; b < C; b++) {
                uint32_t f[3] = {lo0 + a, hi0 + b, eq_id};
                lg_push_term(terms, n_terms, e2_mul(sl, e2_mul(pw[a], pw[b])), 3, f);
            }
    } else {
        uint32_t lo0 = w0, hi0 = w0 + C;
        orc_e2 sl = e2_mul(scale, lambda);
        /* -D_hi - D_lo + lambda D_lo D_hi : constant part (lambda c^2 - 2c) */
        {
            uint32_t f[1] = {eq_id};
            orc_e2 k0 = e2_sub(e2_mul(lambda, e2_mul(c, c)), e2_add(c, c));
            lg_push_term(terms, n_terms, e2_mul(scale, k0), 1, f);
        }
        for (uint32_t k = 0; k < C; k++) {
            /* (lambda c - 1) pw_k on each of L_k, H_k */
            orc_e2 k1 = e2_mul(e2_sub(e2_mul(lambda, c), E2_ONE), pw[k]);
            uint32_t f[2] = {lo0 + k, eq_id};
            lg_push_term(terms, n_terms, e2_mul(scale, k1), 2, f);
            uint32_t g[2] = {hi0 + k, eq_id};
            lg_push_term(terms, n_terms, e2_mul(scale, k1), 2, g);
        }
        for (uint32_t a = 0; a < C; a++)
            for (uint32_t b = 0; b < C; b++) {
                uint32_t f[3] = {lo0 + a, hi0 + b, eq_id};
                lg_push_term(terms, n_terms, e2_mul(sl, e2_mul(pw[a], pw[b])), 3, f);
            }
    }
}

int64_t orc_logup_batch_prove(const orc_logup_instance *inst, uint32_t n_inst, orc_transcript *tr,
                              orc_e2 *out, uint64_t out_cap)
{
    if (n_inst == 0) return -1;
    int is_table = inst[0].numer != NULL;
    lg_circ *cc = (lg_circ *)calloc(n_inst, sizeof(lg_circ));
    uint32_t total = 0;
    for (uint32_t c = 0; c < n_inst; c++) {
        if ((inst[c].numer != NULL) != is_table) return -2; /* prover.rs:103-116 */
        uint32_t top = ceil_log2_u64(inst[c].len);
        if (((uint64_t)1 << top) != inst[c].len || top < 2) return -3;
        cc[c].nv = top - 1;
        if (c > 0 && cc[c].nv > cc[c - 1].nv) return -4; /* prover.rs:128-137 */
        if (cc[c].nv > total) total = cc[c].nv;
        cc[c].n_evals = 2 * inst[c].n_cols + (is_table ? 2 : 0);
        cc[c].arena = (orc_e2 *)malloc((orc_logup_arena_len(inst[c].len) + 1) * sizeof(orc_e2));
        orc_logup_build(inst[c].cols, inst[c].n_cols, inst[c].numer, inst[c].len, &inst[c].c, &inst[c].beta,
                        cc[c].arena);
    }
    /* circuit outputs: the last layer flat (circuit.rs:558-560): n_lo n_hi d_lo d_hi */
    orc_e2 *outputs = (orc_e2 *)malloc(4 * n_inst * sizeof(orc_e2));
    for (uint32_t c = 0; c < n_inst; c++) {
        const orc_e2 *last = cc[c].arena + orc_logup_layer_offset(inst[c].len, cc[c].nv);
        memcpy(outputs + 4 * c, last, 4 * sizeof(orc_e2));
    }
    /* prover.rs:163-166 */
    orc_e2 ninst = e2_from_u64(n_inst);
    orc_tr_append_scalars(tr, &ninst, 1);
    for (uint32_t c = 0; c < n_inst; c++) orc_tr_append_scalars(tr, outputs + 4 * c, 4);
    orc_e2 batching, alpha, lambda;
    orc_tr_append_and_sample(tr, (const uint8_t *)"initial_batching", 16, &batching);
    orc_tr_append_and_sample(tr, (const uint8_t *)"initial_alpha", 13, &alpha);
    orc_tr_append_and_sample(tr, (const uint8_t *)"initial_lambda", 14, &lambda);

    orc_e2 *point = (orc_e2 *)malloc((total + 2) * sizeof(orc_e2));
    uint32_t point_len = 1;
    point[0] = batching;

    uint32_t max_mles = 0;
    for (uint32_t c = 0; c < n_inst; c++) max_mles += cc[c].n_evals > 4 ? cc[c].n_evals : 4;
    max_mles += n_inst; /* eq tables */
    const orc_e2 **tabs = (const orc_e2 **)calloc(max_mles, sizeof(orc_e2 *));
    uint32_t *nvs = (uint32_t *)calloc(max_mles, sizeof(uint32_t));
    orc_e2 **scratch = (orc_e2 **)calloc(max_mles + n_inst, sizeof(orc_e2 *));
    size_t term_cap = 0;
    for (uint32_t c = 0; c < n_inst; c++) {
        size_t C = inst[c].n_cols;
        if (C > 64) return -7;
        term_cap += 4 + 4 * C + C * C;
    }
    if (n_inst > 1024) return -7;
    orc_term *terms = (orc_term *)calloc(term_cap, sizeof(orc_term));
    orc_e2 *prev_evals = (orc_e2 *)calloc(max_mles, sizeof(orc_e2));
    uint32_t n_prev = 0;
    orc_e2 *wit = (orc_e2 *)calloc(max_mles + 4 * n_inst, sizeof(orc_e2));
    uint64_t w = 0;
    int64_t rc = 0;
    orc_e2 *final_round = NULL;
    uint32_t n_final_round = 0;

    for (uint32_t v = 1; v <= total; v++) {
        uint32_t remaining = total - (v - 1);
        /* prover.rs:187-203: previous evaluations, then the outputs of the circuits that join now */
        uint32_t n_wit = 0;
        for (uint32_t i = 0; i < n_prev; i++) wit[n_wit++] = prev_evals[i];
        for (uint32_t c = 0; c < n_inst; c++)
            if (cc[c].nv == remaining)
                for (int i = 0; i < 4; i++) wit[n_wit++] = outputs[4 * c + i];

        /* prover.rs:214-254: sizes in decreasing order (instances are sorted that way) */
        uint32_t n_mles = 0, n_terms = 0, n_scratch = 0, layer_count = 0;
        uint32_t n_sizes = 0, size_list[64];
        for (uint32_t c = 0; c < n_inst; c++)
            if (cc[c].nv >= remaining && (n_sizes == 0 || size_list[n_sizes - 1] != cc[c].nv)) size_list[n_sizes++] = cc[c].nv;
        /* witness MLEs first (in circuit order), eq tables after them */
        uint32_t w_off[1024];
        for (uint32_t c = 0; c < n_inst; c++) {
            if (cc[c].nv < remaining) continue;
            uint32_t lv = cc[c].nv + 1 - remaining; /* variables of this circuit's layer now */
            w_off[c] = n_mles;
            n_mles += lg_layer_mles(&inst[c], &cc[c], lv, scratch, &n_scratch, tabs + n_mles, nvs + n_mles);
        }
        uint32_t witness_count = n_mles;
        orc_e2 claim = E2_ZERO;
        orc_e2 alpha_pow = E2_ONE;
        for (uint32_t s = 0; s < n_sizes; s++) {
            uint32_t size = size_list[s];
            uint32_t lv = size + 1 - remaining;
            /* eq over the last lv coordinates of the running point (prover.rs:247-249) */
            orc_e2 *eq = (orc_e2 *)malloc(((uint64_t)1 << lv) * sizeof(orc_e2));
            orc_eq_evals(point + (point_len - lv), lv, eq);
            scratch[n_scratch++] = eq;
            uint32_t eq_id = witness_count + s;
            tabs[eq_id] = eq;
            nvs[eq_id] = lv;
            n_mles = eq_id + 1;
            orc_e2 mult = e2_from_u64((uint64_t)1 << (total - size)); /* prover.rs:221-222 */
            for (uint32_t c = 0; c < n_inst; c++) {
                if (cc[c].nv != size) continue;
                int is_input = (lv == cc[c].nv);
                lg_layer_terms(&inst[c], is_input, w_off[c], eq_id, alpha_pow, lambda, terms, &n_terms);
                /* claim expression (circuit.rs:241-253):
                 * alpha^k * ( b*(n_hi - n_lo) + n_lo + lambda*( b*(d_hi - d_lo) + d_lo ) ) */
                const orc_e2 *e = wit + 4 * layer_count;
                orc_e2 nn = e2_add(e2_mul(batching, e2_sub(e[1], e[0])), e[0]);
                orc_e2 dd = e2_add(e2_mul(batching, e2_sub(e[3], e[2])), e[2]);
                orc_e2 ce = e2_mul(alpha_pow, e2_add(nn, e2_mul(lambda, dd)));
                claim = e2_add(claim, e2_mul(mult, ce));
                layer_count++;
                alpha_pow = e2_mul(alpha_pow, alpha);
            }
        }
        (void)n_wit;
        orc_tr_append_scalars(tr, &claim, 1); /* prover.rs:261 */

        orc_e2 *proof = (orc_e2 *)malloc((size_t)v * 4 * sizeof(orc_e2));
        orc_e2 *pt = (orc_e2 *)malloc(v * sizeof(orc_e2));
        orc_e2 *fin = (orc_e2 *)malloc(n_mles * sizeof(orc_e2));
        /* a sumcheck whose terms all have degree < 3 still sends 4 evaluations: the
         * batched expression always carries a degree-3 term (lambda D_lo D_hi eq) */
        rc = orc_sc_prove(v, n_mles, tabs, nvs, terms, n_terms, tr, proof, pt, fin);
        if (rc == 0 && w + (uint64_t)v * 4 + witness_count > out_cap) rc = -5;
        if (rc == 0) {
            memcpy(out + w, proof, (size_t)v * 4 * sizeof(orc_e2));
            w += (uint64_t)v * 4;
            memcpy(out + w, fin, witness_count * sizeof(orc_e2));
            w += witness_count;
            memcpy(prev_evals, fin, witness_count * sizeof(orc_e2));
            n_prev = witness_count;
            memcpy(point, pt, v * sizeof(orc_e2));
            point_len = v;
        }
        free(proof);
        free(pt);
        free(fin);
        for (uint32_t i = 0; i < n_scratch; i++) free(scratch[i]);
        if (rc != 0) break;
        /* prover.rs:284-291 */
        orc_tr_append_and_sample(tr, (const uint8_t *)"logup_batching", 14, &batching);
        if (v != total) {
            orc_tr_append_and_sample(tr, (const uint8_t *)"logup_alpha", 11, &alpha);
            orc_tr_append_and_sample(tr, (const uint8_t *)"logup_lambda", 12, &lambda);
        }
        point[point_len++] = batching;
        if (v == total) {
            final_round = prev_evals;
            n_final_round = n_prev;
        }
    }
    if (rc == 0) {
        /* prover.rs:302-330: combine low/high halves with the last batching challenge */
        uint32_t skip = 0;
        for (uint32_t c = 0; c < n_inst && rc == 0; c++) {
            const orc_e2 *ev = final_round + skip;
            skip += cc[c].n_evals;
            if (skip > n_final_round) {
                rc = -6;
                break;
            }
            uint32_t C = inst[c].n_cols;
            if (w + C + 1 > out_cap) {
                rc = -5;
                break;
            }
            if (is_table) {
                out[w++] = e2_add(e2_mul(batching, e2_sub(ev[1], ev[0])), ev[0]);
                ev += 2;
            }
            for (uint32_t k = 0; k < C; k++) out[w++] = e2_add(e2_mul(batching, e2_sub(ev[C + k], ev[k])), ev[k]);
        }
    }
    if (rc == 0) {
        if (w + 4 * (uint64_t)n_inst + point_len > out_cap) rc = -5;
    }
    if (rc == 0) {
        memcpy(out + w, outputs, 4 * (size_t)n_inst * sizeof(orc_e2));
        w += 4 * (uint64_t)n_inst;
        memcpy(out + w, point, point_len * sizeof(orc_e2));
        w += point_len;
    }
    for (uint32_t c = 0; c < n_inst; c++) free(cc[c].arena);
    free(cc);
    free(outputs);
    free(point);
    free(tabs);
    free(nvs);
    free(scratch);
    free(terms);
    free(prev_evals);
    free(wit);
    return rc == 0 ? (int64_t)w : rc;
}

/* value of  scale * eq * (N_lo D_hi + N_hi D_lo + lambda D_lo D_hi)  from final evaluations
 * (structs.rs:428-546), ev pointing at this instance's evaluations */
static orc_e2 lg_instance_eval(int is_table, int is_final, uint32_t C, orc_e2 c, orc_e2 beta, orc_e2 lambda,
                               const orc_e2 *ev, uint32_t *consumed)
{
    if (!is_final) {
        *consumed = 4;
        orc_e2 a = e2_add(e2_mul(ev[0], ev[3]), e2_mul(ev[1], ev[2]));
        return e2_add(a, e2_mul(lambda, e2_mul(ev[2], ev[3])));
    }
    orc_e2 nlo, nhi;
    const orc_e2 *cols = ev;
    if (is_table) {
        nlo = ev[0];
        nhi = ev[1];
        cols = ev + 2;
        *consumed = 2 + 2 * C;
    } else {
        nlo = nhi = e2(P - 1, 0);
        *consumed = 2 * C;
    }
    orc_e2 dlo = c, dhi = c, pw = E2_ONE;
    for (uint32_t k = 0; k < C; k++) {
        dlo = e2_add(dlo, e2_mul(pw, cols[k]));
        dhi = e2_add(dhi, e2_mul(pw, cols[C + k]));
        pw = e2_mul(pw, beta);
    }
    orc_e2 a = e2_add(e2_mul(nlo, dhi), e2_mul(nhi, dlo));
    return e2_add(a, e2_mul(lambda, e2_mul(dlo, dhi)));
}

int orc_logup_batch_verify(const uint32_t *n_cols, const uint32_t *inst_nvars,
                           const orc_e2 *cs, const orc_e2 *betas, int is_table, uint32_t n_inst,
                           const orc_e2 *stream, uint64_t stream_len, orc_transcript *tr,
                           orc_e2 *claims_out, orc_e2 *point_out)
{
    uint32_t total = 0;
    uint64_t n_claims = 0;
    for (uint32_t c = 0; c < n_inst; c++) {
        if (inst_nvars[c] > total) total = inst_nvars[c];
        n_claims += n_cols[c] + (is_table ? 1 : 0);
    }
    /* locate the pieces of the stream */
    uint64_t pos = 0;
    const orc_e2 **proofs = (const orc_e2 **)calloc(total + 1, sizeof(orc_e2 *));
    const orc_e2 **revals = (const orc_e2 **)calloc(total + 1, sizeof(orc_e2 *));
    uint32_t *n_revals = (uint32_t *)calloc(total + 1, sizeof(uint32_t));
    int rc = 0;
    for (uint32_t v = 1; v <= total && rc == 0; v++) {
        uint32_t remaining = total - (v - 1);
        uint32_t ne = 0;
        for (uint32_t c = 0; c < n_inst; c++) {
            if (inst_nvars[c] < remaining) continue;
            int is_final = (v == total);
            ne += is_final ? 2 * n_cols[c] + (is_table ? 2 : 0) : 4;
        }
        proofs[v] = stream + pos;
        pos += (uint64_t)v * 4;
        revals[v] = stream + pos;
        n_revals[v] = ne;
        pos += ne;
        if (pos > stream_len) rc = -1;
    }
    if (rc == 0 && pos + n_claims + 4 * (uint64_t)n_inst > stream_len) rc = -1;
    if (rc != 0) {
        free(proofs);
        free(revals);
        free(n_revals);
        return rc;
    }
    const orc_e2 *outputs = stream + pos + n_claims;

    /* verifier.rs:83-105 */
    orc_e2 ninst = e2_from_u64(n_inst);
    orc_tr_append_scalars(tr, &ninst, 1);
    for (uint32_t c = 0; c < n_inst; c++) orc_tr_append_scalars(tr, outputs + 4 * c, 4);
    orc_e2 batching, alpha, lambda;
    orc_tr_append_and_sample(tr, (const uint8_t *)"initial_batching", 16, &batching);
    orc_tr_append_and_sample(tr, (const uint8_t *)"initial_alpha", 13, &alpha);
    orc_tr_append_and_sample(tr, (const uint8_t *)"initial_lambda", 14, &lambda);

    orc_e2 *point = (orc_e2 *)malloc((total + 2) * sizeof(orc_e2));
    uint32_t point_len = 1;
    point[0] = batching;
    orc_e2 *wit = (orc_e2 *)malloc((n_revals[total] + 8 * (size_t)n_inst + 8) * sizeof(orc_e2));

    for (uint32_t v = 1; v <= total; v++) {
        uint32_t remaining = total - (v - 1);
        uint32_t n_wit = 0;
        if (v > 1)
            for (uint32_t i = 0; i < n_revals[v - 1]; i++) wit[n_wit++] = revals[v - 1][i];
        for (uint32_t c = 0; c < n_inst; c++)
            if (inst_nvars[c] == remaining)
                for (int i = 0; i < 4; i++) wit[n_wit++] = outputs[4 * c + i];
        /* claim (verifier.rs:138-180) */
        orc_e2 claim = E2_ZERO, alpha_pow = E2_ONE;
        uint32_t layer_count = 0;
        for (uint32_t c = 0; c < n_inst; c++) {
            if (inst_nvars[c] < remaining) continue;
            orc_e2 mult = e2_from_u64((uint64_t)1 << (total - inst_nvars[c]));
            const orc_e2 *e = wit + 4 * layer_count;
            orc_e2 nn = e2_add(e2_mul(batching, e2_sub(e[1], e[0])), e[0]);
            orc_e2 dd = e2_add(e2_mul(batching, e2_sub(e[3], e[2])), e[2]);
            claim = e2_add(claim, e2_mul(mult, e2_mul(alpha_pow, e2_add(nn, e2_mul(lambda, dd)))));
            layer_count++;
            alpha_pow = e2_mul(alpha_pow, alpha);
        }
        orc_tr_append_scalars(tr, &claim, 1);
        orc_e2 *pt = (orc_e2 *)malloc(v * sizeof(orc_e2));
        orc_e2 expected;
        int bad = orc_sc_verify(&claim, proofs[v], v, 3, tr, pt, &expected);
        orc_tr_append_and_sample(tr, (const uint8_t *)"logup_batching", 14, &batching);
        /* recompute the sumcheck's final value from the round evaluations and the
         * closed-form eq (verifier.rs:195-211) */
        orc_e2 calc = E2_ZERO;
        alpha_pow = E2_ONE;
        uint32_t off = 0;
        for (uint32_t c = 0; c < n_inst; c++) {
            if (inst_nvars[c] < remaining) continue;
            uint32_t lv = inst_nvars[c] + 1 - remaining;
            orc_e2 eqv;
            /* eq point: last lv coordinates of the previous point; evaluated at the
             * last lv coordinates of this sumcheck's point (verifier.rs:62-73,170) */
            orc_identity_eval(pt + (v - lv), point + (point_len - lv), lv, &eqv);
            uint32_t used = 0;
            orc_e2 val = lg_instance_eval(is_table, v == total, n_cols[c], cs[c], betas[c], lambda,
                                          revals[v] + off, &used);
            off += used;
            calc = e2_add(calc, e2_mul(alpha_pow, e2_mul(eqv, val)));
            alpha_pow = e2_mul(alpha_pow, alpha);
        }
        if (v != total) {
            orc_tr_append_and_sample(tr, (const uint8_t *)"logup_alpha", 11, &alpha);
            orc_tr_append_and_sample(tr, (const uint8_t *)"logup_lambda", 12, &lambda);
        }
        if (rc == 0 && (bad || !e2_eq(calc, expected))) rc = (int)v;
        memcpy(point, pt, v * sizeof(orc_e2));
        point_len = v;
        point[point_len++] = batching;
        free(pt);
    }
    /* verifier.rs:232-243 */
    uint32_t skip = 0;
    uint64_t wc = 0;
    for (uint32_t c = 0; c < n_inst; c++) {
        const orc_e2 *ev = revals[total] + skip;
        uint32_t C = n_cols[c];
        skip += 2 * C + (is_table ? 2 : 0);
        if (is_table) {
            claims_out[wc++] = e2_add(e2_mul(batching, e2_sub(ev[1], ev[0])), ev[0]);
            ev += 2;
        }
        for (uint32_t k = 0; k < C; k++) claims_out[wc++] = e2_add(e2_mul(batching, e2_sub(ev[C + k], ev[k])), ev[k]);
    }
    memcpy(point_out, point, point_len * sizeof(orc_e2));
    free(point);
    free(wit);
    free(proofs);
    free(revals);
    free(n_revals);
    return rc;
}
