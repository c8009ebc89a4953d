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
/* IOPVerifierState::verify; returns 0 or DPS_ERR_INVALID when a round fails */
int32_t dph_sumcheck_verify(const uint64_t claimed_sum[2], const uint64_t *proof, uint32_t n_vars, uint32_t degree,
                            dph_transcript *t, uint64_t *point_out, uint64_t expected_out[2]);

#ifdef __cplusplus
}
#endif
#endif
