/*
 * dpsc_oracle.h -- CPU restatement of the sumcheck prover path (TEST INFRASTRUCTURE ONLY).
 *
 * This library is the checker the GPU path is compared against.  It is never
 * linked into, imported by, or called from the shipped library; only the test
 * suite, the smoke check and the benchmark's cpu_baseline leg load it.
 *
 * Arithmetic: Goldilocks p = 2^64 - 2^32 + 1 and its quadratic extension
 * F_p[X]/(X^2 - 7).  Extension elements are array-of-structs {c0, c1} here (the
 * GPU library keeps them as two separate limb arrays), and every product goes
 * through unsigned __int128 (the GPU library uses 32-bit multiplies), so the
 * two implementations share no arithmetic code.
 *
 * Protocol restated from the reference's call sites (paths relative to the
 * reference checkout):
 *   - generic expression sumcheck: zkml/src/layers/hadamard.rs:93-131,
 *     zkml/src/iop/same_poly.rs:84-114, verifier contract
 *     zkml/src/layers/hadamard.rs:134-163
 *   - eq table: closed form zkml/src/poly_commit/mod.rs:184-192, usage
 *     zkml/src/layers/einsum/axis.rs:1032
 *   - einsum partial evaluation: zkml/src/layers/einsum/axis.rs:1142-1234
 *   - einsum prove: zkml/src/layers/einsum/prove.rs:46-361,
 *     expression zkml/src/layers/einsum/op_info.rs:159-199
 *   - LogUp-GKR: zkml/src/lookup/logup_gkr/circuit.rs:88-184,231-412,
 *     prover.rs:91-344, verifier.rs:77-256, structs.rs:375-547
 *
 * The sumcheck engine itself (IOPProverState::prove) lives in the un-vendored
 * dependency dp-crypto 0.1.0 @ 22e8e93 (Cargo.lock:3773-3775).  PARITY UNPINNED
 * for what only that source could fix: the round-message layout (here: d+1
 * evaluations at t = 0..d), what prove() absorbs before round 1, the transcript
 * byte encodings, and the LSB-first binding order (fixed here from the in-tree
 * call sites that use collect_raw_challenges() unreversed as a little-endian
 * evaluation point).
 */
#ifndef DPSC_ORACLE_H
#define DPSC_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_P 0xFFFFFFFF00000001ULL
#define ORC_W 7ULL /* X^2 = 7 */
#define ORC_MAX_FACTORS 8

typedef struct {
    uint64_t c0, c1;
} orc_e2;

/* ---- base field ---- */
uint64_t orc_gl_add(uint64_t a, uint64_t b);
uint64_t orc_gl_sub(uint64_t a, uint64_t b);
uint64_t orc_gl_neg(uint64_t a);
uint64_t orc_gl_mul(uint64_t a, uint64_t b);
uint64_t orc_gl_pow(uint64_t a, uint64_t e);
uint64_t orc_gl_inv(uint64_t a);
/* F::from(i64): negatives map to p - |x| (zkml/src/quantization/mod.rs:262-266) */
uint64_t orc_gl_from_i64(int64_t x);
/* inverse embedding (zkml/src/quantization/mod.rs:231-260): values above p/2 are negative */
int64_t orc_gl_to_i64(uint64_t x);

/* ---- extension field (pointer based so ctypes can call it) ---- */
void orc_e2_add(const orc_e2 *a, const orc_e2 *b, orc_e2 *out);
void orc_e2_sub(const orc_e2 *a, const orc_e2 *b, orc_e2 *out);
void orc_e2_mul(const orc_e2 *a, const orc_e2 *b, orc_e2 *out);
void orc_e2_inv(const orc_e2 *a, orc_e2 *out);

/* ---- tables ---- */
/* out[i] = prod_j (bit_j(i) ? r_j : 1 - r_j), little-endian in i; out has 2^m entries */
void orc_eq_evals(const orc_e2 *point, uint32_t m, orc_e2 *out);
/* prod_i (r1_i r2_i + (1-r1_i)(1-r2_i)) over the common prefix */
void orc_identity_eval(const orc_e2 *r1, const orc_e2 *r2, uint32_t len, orc_e2 *out);
void orc_embed_base(const uint64_t *in, uint64_t len, orc_e2 *out);
void orc_embed_i64(const int64_t *in, uint64_t len, orc_e2 *out);
/* full evaluation at a little-endian point */
void orc_mle_evaluate(const orc_e2 *tbl, uint32_t n, const orc_e2 *point, orc_e2 *out);
/* bind the k lowest variables to point[0..k): out has 2^(n-k) entries */
void orc_mle_fix_low(const orc_e2 *tbl, uint32_t n, const orc_e2 *point, uint32_t k, orc_e2 *out);
/* bind the k highest variables to point[0..k) (point[j] binds variable n-k+j) */
void orc_mle_fix_high(const orc_e2 *tbl, uint32_t n, const orc_e2 *point, uint32_t k, orc_e2 *out);

/* ---- BLAKE3 (hash mode, 32-byte output) and the transcript ---- */
void orc_blake3(const uint8_t *in, size_t len, uint8_t out[32]);

typedef struct {
    uint8_t state[32];
    uint32_t n_rounds;
} orc_transcript;

void orc_tr_new(orc_transcript *t, const uint8_t *label, size_t len);
void orc_tr_append_message(orc_transcript *t, const uint8_t *label, size_t len);
void orc_tr_append_bytes(orc_transcript *t, const uint8_t *bytes, size_t len);
void orc_tr_append_u64(orc_transcript *t, uint64_t x);
void orc_tr_append_scalar(orc_transcript *t, const orc_e2 *x);
void orc_tr_append_scalars(orc_transcript *t, const orc_e2 *xs, size_t n);
void orc_tr_challenge_scalar(orc_transcript *t, orc_e2 *out);
void orc_tr_append_and_sample(orc_transcript *t, const uint8_t *label, size_t len, orc_e2 *out);

/* ---- sumcheck ---- */
typedef struct {
    orc_e2 coeff;
    uint32_t n_factors;
    uint32_t factors[ORC_MAX_FACTORS];
} orc_term;

uint32_t orc_terms_degree(const orc_term *terms, uint32_t n_terms);

/* One round polynomial by direct summation over the current tables (no folding):
 * evals_out[t] for t = 0..degree.  tables[k] has 2^cur_nvars[k] entries; an MLE
 * with fewer than `live` variables is constant in the low live - cur_nvars[k]
 * variables. */
void orc_sc_round_poly(uint32_t live, uint32_t n_mles, const orc_e2 *const *tables,
                       const uint32_t *cur_nvars, const orc_term *terms, uint32_t n_terms,
                       uint32_t degree, orc_e2 *evals_out);

/* Full prover.  proof_out: n_vars*(degree+1) elements; point_out: n_vars;
 * final_out: n_mles.  Returns 0, or a negative value on bad arguments. */
int orc_sc_prove(uint32_t n_vars, uint32_t n_mles, const orc_e2 *const *tables,
                 const uint32_t *mle_nvars, const orc_term *terms, uint32_t n_terms,
                 orc_transcript *tr, orc_e2 *proof_out, orc_e2 *point_out, orc_e2 *final_out);

/* Verifier.  Returns 0 when every round is consistent, otherwise the 1-based
 * index of the first failing round.  point_out: n_vars; expected_out: the value
 * the caller must match against expr(final evals). */
int orc_sc_verify(const orc_e2 *claimed_sum, const orc_e2 *proof, uint32_t n_vars,
                  uint32_t degree, orc_transcript *tr, orc_e2 *point_out, orc_e2 *expected_out);

/* univariate given by evals at 0..degree, evaluated at r */
void orc_interpolate(const orc_e2 *evals, uint32_t degree, const orc_e2 *r, orc_e2 *out);

/* ---- einsum partial evaluation (axis.rs:1142-1234) ---- */
enum { ORC_AXIS_CONTRACTED = 0, ORC_AXIS_OUTER = 1, ORC_AXIS_STACKED = 2 };

/* tensor: row-major i64 with the padded dims; only the unpadded region is read.
 * points[a]: the claim-point slice of axis a (log2(padded_dims[a]) elements) for
 * Outer and Stacked axes, ignored for Contracted.  Output: n_stack tables of
 * 2^ceil_log2(contraction) entries, written consecutively to out.  Returns
 * n_stack, and the table length through *table_len. */
int64_t orc_partial_eval(const int64_t *tensor, const uint64_t *padded_dims,
                         const uint64_t *unpadded_dims, uint32_t n_dims, const int32_t *kinds,
                         const orc_e2 *const *points, orc_e2 *out, uint64_t out_cap,
                         uint64_t *table_len);

/* stacking coefficients (axis.rs:1043-1062): outer product of the stacked axes'
 * truncated eq tables; returns the count */
int64_t orc_stacking_coeffs(const uint64_t *padded_dims, const uint64_t *unpadded_dims,
                            uint32_t n_dims, const int32_t *kinds, const orc_e2 *const *points,
                            orc_e2 *out, uint64_t out_cap);

/* ---- LogUp-GKR ---- */
/* Fraction-sum tree for one instance (circuit.rs:88-184).  cols: n_cols base
 * columns of `len` entries (len a power of two >= 2); numer: multiplicities
 * (table instance) or NULL (lookup instance, numerators -1).
 * Layers above the input are written to arena as (numerator[], denominator[])
 * pairs, layer k (k >= 1) holding len >> k entries per array; arena needs
 * 2*(len-2)... entries: use orc_logup_arena_len(len). */
uint64_t orc_logup_arena_len(uint64_t len);
void orc_logup_build(const uint64_t *const *cols, uint32_t n_cols, const uint64_t *numer,
                     uint64_t len, const orc_e2 *c, const orc_e2 *beta, orc_e2 *arena);
/* offset of layer k's numerator array in the arena (denominator follows it) */
uint64_t orc_logup_layer_offset(uint64_t len, uint32_t k);

typedef struct {
    uint32_t n_cols;
    uint64_t len;
    const uint64_t *const *cols; /* n_cols pointers */
    const uint64_t *numer;       /* NULL for lookups */
    orc_e2 c, beta;
} orc_logup_instance;

/* Batched prover (prover.rs:91-344).  All instances are of one type (all
 * lookups or all tables) and ordered by non-increasing size.  Everything the
 * reference puts in LogUpBatchProof is written to a flat stream of elements:
 *   for each layer round v = 1..total: proof (v*(4) elements), then the round
 *   evaluations; then output claim evaluations; then circuit outputs.
 * The exact layout is documented at the definition.  Returns the number of
 * elements written or a negative value. */
int64_t orc_logup_batch_prove(const orc_logup_instance *inst, uint32_t n_inst, orc_transcript *tr,
                              orc_e2 *out, uint64_t out_cap);

/* Verifier twin (verifier.rs:77-256) over the same flat stream.  Returns 0 on
 * success, a positive round index on a failed check, negative on malformed
 * input.  claims_out receives the output claim evaluations recomputed from
 * the final round (one per column, plus one per multiplicity column), and
 * point_out the final point (total+1 elements). */
int orc_logup_batch_verify(const uint32_t *n_cols, const uint32_t *inst_nvars,
                           const orc_e2 *cs, const orc_e2 *betas, int is_table, uint32_t n_inst,
                           const orc_e2 *stream, uint64_t stream_len, orc_transcript *tr,
                           orc_e2 *claims_out, orc_e2 *point_out);

int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
