/*
 * dpsc_host.h -- C entry points of the host-side mirror (libdpsc_host.so).
 *
 * The mirror itself is C++ (the headers under dpsc/): transcript, expressions, the
 * prove/verify loops and the einsum and LogUp drivers, written against the C ABI
 * of libdpsumcheck.  These wrappers exist so that Python (tests, benchmark) can
 * drive the same code.  Extension elements are (c0, c1) pairs of uint64_t.
 */
#ifndef DPSC_HOST_H
#define DPSC_HOST_H

#include <stddef.h>
#include <stdint.h>

#include "../../include/dpsumcheck.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dph_transcript dph_transcript;

/* ---- Blake3Transcript ---- */
dph_transcript *dph_tr_new(const char *label);
dph_transcript *dph_tr_clone(const dph_transcript *t);
void dph_tr_free(dph_transcript *t);
void dph_tr_append_message(dph_transcript *t, const char *label);
void dph_tr_append_bytes(dph_transcript *t, const uint8_t *data, size_t len);
void dph_tr_append_u64(dph_transcript *t, uint64_t x);
void dph_tr_append_scalars(dph_transcript *t, const uint64_t *xs, size_t n);
void dph_tr_challenge_scalar(dph_transcript *t, uint64_t out[2]);
void dph_tr_append_and_sample(dph_transcript *t, const char *label, uint64_t out[2]);
void dph_tr_state(const dph_transcript *t, uint8_t state_out[32], uint32_t *n_rounds);
void dph_blake3(const uint8_t *data, size_t len, uint8_t out[32]);

/* text of the last C++ exception caught by a wrapper on this thread */
const char *dph_last_error(void);

/* ---- IOPProverState::prove over raw handles ----
 * proof_out: n_vars*(degree+1) elements, point_out: n_vars, finals_out: n_mles */
int32_t dph_sumcheck_prove(dps_ctx *ctx, uint32_t n_vars, const dps_mle *const *mles, uint32_t n_mles,
                           const dps_term *terms, uint32_t n_terms, dph_transcript *t, uint64_t *proof_out,
                           uint64_t *point_out, uint64_t *finals_out, uint32_t *degree_out);
/* the same with the value of the whole sum stated by the caller, who holds it as the claim being reduced
 * (zkml/src/layers/hadamard.rs:117-121): round 1 then takes p(1) from it, same messages */
int32_t dph_sumcheck_prove_claimed(dps_ctx *ctx, uint32_t n_vars, const dps_mle *const *mles, uint32_t n_mles,
                                   const dps_term *terms, uint32_t n_terms, const uint64_t claimed_sum[2], dph_transcript *t,
                                   uint64_t *proof_out, uint64_t *point_out, uint64_t *finals_out, uint32_t *degree_out);
/* IOPVerifierState::verify; returns 0 or DPS_ERR_INVALID when a round fails */
int32_t dph_sumcheck_verify(const uint64_t claimed_sum[2], const uint64_t *proof, uint32_t n_vars, uint32_t degree,
                            dph_transcript *t, uint64_t *point_out, uint64_t expected_out[2]);

/* ---- EinSum::prove_internal (zkml/src/layers/einsum/prove.rs:46-333) ----
 * n_ops batched operations share one LHS.  labels: 4*n_ops C strings (lhs, rhs,
 * out, bias per operation, e.g. "ik","kj","ij","j"; bias "" = the output has no
 * bias).  Tensors arrive unpadded, row-major.  biases: NULL when no output has a
 * bias, else n_ops entries (NULL where the bias labels are ""), with their shapes
 * and ranks alongside (prove.rs:191-214: every bias gives a claim of its own).
 * claim_points[r]: 2*len limbs of the claim point on output r, claim_evals 2 per op.
 * The result is written as 64-bit words:
 *   rounds, points_per_round, proof limbs..., n_evals, eval limbs...,
 *   agg_rounds (0 = none), agg proof limbs (3 points per round)...,
 *   n_claims, then per claim: point_len, point limbs..., eval limbs,
 *   n_bias_claims, then per bias claim: output index, point_len, point limbs..., eval limbs
 * Returns DPS_OK and the word count through *n_words. */
int32_t dph_einsum_prove(dps_ctx *ctx, uint32_t n_ops, const char *const *labels, const int64_t *lhs,
                         const uint64_t *lhs_shape, uint32_t lhs_rank, const int64_t *const *rhs,
                         const uint64_t *const *rhs_shapes, const uint32_t *rhs_ranks,
                         const int64_t *const *biases, const uint64_t *const *bias_shapes, const uint32_t *bias_ranks,
                         const uint64_t *const *claim_points, const uint32_t *claim_point_lens,
                         const uint64_t *claim_evals, dph_transcript *t, uint64_t *out, uint64_t out_cap,
                         uint64_t *n_words);

/* The same proof over tensors that are already on the device: raw integer
 * tensors made with dps_tensor_from_i64 / dps_tensor_from_i16 (unpadded,
 * row-major) that the caller keeps — weights across proofs, activations
 * across the layers that read them.  Nothing is uploaded per call. */
int32_t dph_einsum_prove_resident(dps_ctx *ctx, uint32_t n_ops, const char *const *labels, const dps_mle *lhs,
                                  const uint64_t *lhs_shape, uint32_t lhs_rank, const dps_mle *const *rhs,
                                  const uint64_t *const *rhs_shapes, const uint32_t *rhs_ranks,
                                  const dps_mle *const *biases, const uint64_t *const *bias_shapes, const uint32_t *bias_ranks,
                                  const uint64_t *const *claim_points, const uint32_t *claim_point_lens,
                                  const uint64_t *claim_evals, dph_transcript *t, uint64_t *out, uint64_t out_cap,
                                  uint64_t *n_words);

/* ---- new_batch_multiple_sizes_prove (zkml/src/lookup/logup_gkr/prover.rs:91-344) ----
 * Instance i has n_cols[i] base-field column tables (handles, flattened in
 * cols) and, for table instances, a multiplicity table numer[i] (numer is NULL
 * for lookups).  cs / betas: 2 limbs per instance.  The proof is written as
 * extension elements (2 words each) in this order: for every layer round v =
 * 1..total: the v*4 round-message elements, then that round's evaluations;
 * then the output claim evaluations; the 4 circuit outputs per instance; the
 * final point (total + 1 elements). */
int32_t dph_logup_batch_prove(dps_ctx *ctx, uint32_t n_inst, const uint32_t *n_cols, const dps_mle *const *cols,
                              const dps_mle *const *numer, const uint64_t *cs, const uint64_t *betas,
                              dph_transcript *t, uint64_t *out, uint64_t out_cap, uint64_t *n_elems);
/* new_verify_logup_proof_multiple_sizes (verifier.rs:77-256) over the same stream.
 * claims_out: one element per (multiplicity and) column per instance; point_out: total + 1. */
int32_t dph_logup_batch_verify(uint32_t n_inst, const uint32_t *n_cols, const uint32_t *inst_nvars, const uint64_t *cs,
                               const uint64_t *betas, int32_t is_table, const uint64_t *stream, uint64_t n_elems,
                               dph_transcript *t, uint64_t *claims_out, uint64_t *point_out);

/* Claims-batching sumcheck of the opening proof (zkml/src/poly_commit/prover.rs:140-255).
 * Polynomial p is held as chunks_per_poly[p] chunk tables (handles in `chunks`, polynomial by
 * polynomial) and has claims_per_poly[p] claims; `points` holds the claim points one after the
 * other (2 limbs per coordinate, num_vars(p) coordinates each), `evals` 2 limbs per claim.
 * Outputs: proof n_vars x 3 elements, point n_vars elements, one evaluation per chunk table. */
int32_t dph_claims_batching_prove(dps_ctx *ctx, uint32_t n_polys, const uint32_t *chunks_per_poly, const dps_mle *const *chunks,
                                  const uint32_t *claims_per_poly, const uint64_t *points, const uint64_t *evals,
                                  dph_transcript *t, uint64_t *proof_out, uint64_t *point_out, uint64_t *evals_out,
                                  uint32_t *n_vars_out);
/* Verifier twin (zkml/src/poly_commit/verifier.rs:203-340): poly_vars[p] = variables of the whole
 * polynomial.  Returns DPS_OK and the opening point when the proof verifies. */
int32_t dph_claims_batching_verify(uint32_t n_polys, const uint32_t *chunks_per_poly, const uint32_t *poly_vars,
                                   const uint32_t *claims_per_poly, const uint64_t *points, const uint64_t *evals,
                                   const uint64_t *proof, uint32_t n_vars, const uint64_t *sumcheck_evals,
                                   dph_transcript *t, uint64_t *point_out);

/* same_poly::Prover::prove (zkml/src/iop/same_poly.rs:84-114): n_claims claims (points of
 * num_vars(poly) coordinates, 2 limbs each; evals 2 limbs each) on one polynomial.
 * Outputs: proof num_vars x 3 elements, the merged claim's point and evaluation. */
int32_t dph_same_poly_prove(dps_ctx *ctx, const dps_mle *poly, uint32_t n_claims, const uint64_t *points, const uint64_t *evals,
                            dph_transcript *t, uint64_t *proof_out, uint64_t *point_out, uint64_t *eval_out);
/* same_poly::Verifier::verify (same_poly.rs:140-169); DPS_OK when the proof verifies */
int32_t dph_same_poly_verify(uint32_t num_vars, uint32_t n_claims, const uint64_t *points, const uint64_t *evals, const uint64_t *proof,
                             const uint64_t *eval, dph_transcript *t, uint64_t *point_out);

/* ---- the sumcheck linking a lookup argument to its layer ----
 * LookupInputConfig::prove_linking_sumcheck (zkml/src/lookup/operation/inputs/proving.rs:26-114) with
 * the expression of LookupVariant::build_full_sumcheck_expression (variant.rs:55-348).  The
 * configuration carries what that expression reads from the layer: */
typedef struct dph_linking_config {
    int32_t variant;        /* 0 Standard, 1 GLU, 2 Softmax, 3 Normalisation */
    int32_t normalised_sum; /* Normalisation: normalised_sum_value is Some */
    int32_t has_weight;     /* Normalisation: has_weight */
    uint32_t number_of_value_chunks, number_of_zeroing_chunks; /* ChunkingInfo */
    uint32_t table_bit_size;                                   /* Table::table_bit_size */
    int32_t table_is_signed;
    int32_t input_sign_negative; /* unsigned tables: TableSign::Negative (else Positive) */
    int64_t min_output_value, max_output_value;
    uint32_t rank;
    const uint64_t *unpadded_input_shape;
} dph_linking_config;
/* mles: the witness tables in the expression's order (per 2-D chunk its value chunks then its zeroing
 * chunks; then, GLU: one table per chunk; Normalisation: the input chunks, then the scaling tables),
 * each with the variables of the padded last two dimensions.  weight: the Normalisation weight table or
 * NULL.  Points: 2 limbs per coordinate.  Output words: rounds, points per round, the round messages,
 * n_evaluations, the evaluations of `mles` at the sumcheck point, has_weight_eval (0/1) [+ that
 * evaluation], the sumcheck point (rounds elements), n_challenges, the batching challenges. */
int32_t dph_linking_prove(dps_ctx *ctx, const dph_linking_config *cfg, const dps_mle *const *mles, uint32_t n_mles, const dps_mle *weight,
                          const uint64_t *last_claim_point, uint32_t last_claim_len, const uint64_t *logup_point, uint32_t logup_len,
                          dph_transcript *t, uint64_t *out, uint64_t out_cap, uint64_t *n_words);
/* verify_linking_sumcheck (inputs/verifying.rs:236-330) from the initial claim on: the claimed sum
 * (LookupVariant::prepare_sumcheck_verification's result) is the caller's.  DPS_OK and the sumcheck
 * point when the proof verifies. */
int32_t dph_linking_verify(const dph_linking_config *cfg, const uint64_t initial_claim[2], const uint64_t *proof, uint32_t n_rounds,
                           uint32_t points_per_round, const uint64_t *evaluations, uint32_t n_evaluations, const uint64_t *weight_eval,
                           const uint64_t *last_claim_point, uint32_t last_claim_len, const uint64_t *logup_point, uint32_t logup_len,
                           dph_transcript *t, uint64_t *point_out);

#ifdef __cplusplus
}
#endif
#endif
