/*
 * dpsumcheck.h -- C ABI of the MI355X sumcheck prover library (libdpsumcheck.so).
 *
 * The library replaces, for one GPU, the sumcheck engine the reference's layer
 * provers call.  That engine is a Rust generic API (crate dp-crypto, pinned in
 * the reference's Cargo.lock:3773-3775), not an FFI; every entry point below
 * names the Rust call it stands in for and a reference call site that shows the
 * contract (paths relative to the reference checkout).
 *
 * Conventions
 *   - Field: Goldilocks p = 2^64 - 2^32 + 1; extension F_p[X]/(X^2 - 7).
 *     A base element is one canonical uint64_t (< p).  An extension element
 *     crossing this ABI is two uint64_t, (c0, c1), c0 first.
 *   - Tables live in HBM.  Extension tables are structure-of-arrays: one
 *     uint64_t array of c0 limbs and one of c1 limbs.
 *   - A table of 2^n entries is the little-endian evaluation table of an
 *     n-variate multilinear polynomial: entry i sits at the point whose j-th
 *     coordinate is bit j of i.  A row-major tensor's last dimension occupies the
 *     lowest variables (zkml/src/shape.rs:475-496, zkml/src/tensor/mod.rs:1874-1897).
 *   - Sumcheck round j binds variable j-1 (lowest first); the challenges in
 *     round order are the little-endian evaluation point of the final claims
 *     (zkml/src/layers/hadamard.rs:124-129,148-149).
 *   - Every function returns a dps_status; nothing throws or aborts.  Host
 *     buffers are borrowed for the duration of the call only.  A context owns one
 *     HIP stream; calls on one context must not overlap, different contexts may be
 *     used from different threads at the same time (see dps_device_set_resident_budget
 *     for how their launches share one GPU).
 */
#ifndef DPSUMCHECK_H
#define DPSUMCHECK_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DPS_MAX_FACTORS 8 /* factor slots in a term */
#define DPS_MAX_DEGREE 6  /* largest product the kernels evaluate (reference maximum: 5, zkml/src/layers/pooling.rs:468-472) */

typedef enum dps_status {
    DPS_OK = 0,
    DPS_ERR_INVALID = 1,     /* bad argument */
    DPS_ERR_HIP = 2,         /* a HIP runtime call failed; see dps_last_error */
    DPS_ERR_OOM = 3,         /* device or host allocation failed */
    DPS_ERR_STATE = 4,       /* call out of order (e.g. round after the last round) */
    DPS_ERR_UNSUPPORTED = 5, /* degree or arity beyond the compiled kernels */
    DPS_ERR_CALLBACK = 6     /* the transcript callback returned non-zero */
} dps_status;

typedef enum dps_kind {
    DPS_BASE = 0, /* uint64_t canonical base-field entries */
    DPS_EXT2 = 1, /* two limb arrays */
    DPS_I64 = 2,  /* raw quantised int64_t entries, embedded on load (zkml/src/quantization/mod.rs:262-266) */
    DPS_I16 = 3   /* the same values stored as int16_t (quantised activations and weights fit 16 bits); a tensor
                   * input of dps_partial_eval, dps_mle_evaluate and dps_mle_fix_high only */
} dps_kind;

typedef struct dps_ctx dps_ctx;
typedef struct dps_mle dps_mle;
typedef struct dps_sc dps_sc;
typedef struct dps_logup dps_logup;

/* ---- context ---- */
int32_t dps_ctx_create(int32_t device, dps_ctx **out);
int32_t dps_ctx_destroy(dps_ctx *ctx);
/* text of the last failure on this context (never NULL) */
const char *dps_last_error(const dps_ctx *ctx);
const char *dps_status_str(int32_t status);
/* wait for everything queued on the context's stream */
int32_t dps_ctx_sync(dps_ctx *ctx);
/* Contexts on one GPU, several threads (the reference proves the chunks of a model concurrently from a thread pool,
 * zkml/src/graph/executor.rs:148, zkml/src/iop/mod.rs:268-279).  Some launches of a session stay on the GPU while the
 * host takes its turn (the resident launches of the late rounds, the launches made ahead of their round); launches of
 * that kind from different contexts share the device through a process-wide ledger, one compute unit per workgroup,
 * so that those admitted are always placed together and none waits for room another holds.  A launch that finds no
 * place is not made and its rounds run as ordinary launches: same results, bit for bit, more launches.
 * dps_device_set_resident_budget caps what all contexts of this process together may hold on `device` (compute units;
 * -1: the whole device, the default; 0: no launch ever waits on the GPU) -- for a GPU shared with other work.
 * dps_device_resident_budget reads the ledger: units held now, and the cap in force (-1 before the first context). */
int32_t dps_device_set_resident_budget(int32_t device, int32_t compute_units);
int32_t dps_device_resident_budget(int32_t device, int32_t *in_use, int32_t *budget);

/* ---- table storage: DensePolynomial::{new, new_from_smart_slice, as_view, evals}
 *      (zkml/src/tensor/mod.rs:364,390,401; zkml/src/lookup/logup_gkr/circuit.rs:262-269) ---- */
/* upload 2^n_vars canonical base elements.  Table entries (here, in dps_mle_from_ext2 and in wrapped device memory) are
 * taken as they are, not checked: an entry >= p gives undefined results (challenges, points and coefficients, which are
 * few, are checked and rejected with DPS_ERR_INVALID). */
int32_t dps_mle_from_base(dps_ctx *ctx, const uint64_t *host, uint32_t n_vars, dps_mle **out);
/* upload 2^n_vars extension elements given as two limb arrays */
int32_t dps_mle_from_ext2(dps_ctx *ctx, const uint64_t *c0, const uint64_t *c1, uint32_t n_vars, dps_mle **out);
/* Tensor<Element>::to_field_mle (zkml/src/tensor/mod.rs:328-401): embed len
 * quantised integers and zero-pad to 2^n_vars base elements, on the device */
int32_t dps_mle_from_i64(dps_ctx *ctx, const int64_t *host, uint64_t len, uint32_t n_vars, dps_mle **out);
/* upload a raw quantised tensor of any length (input of dps_partial_eval) */
int32_t dps_tensor_from_i64(dps_ctx *ctx, const int64_t *host, uint64_t len, dps_mle **out);
/* the same tensor from 16-bit storage: a quarter of the bytes on the device and over PCIe */
int32_t dps_tensor_from_i16(dps_ctx *ctx, const int16_t *host, uint64_t len, dps_mle **out);
/* Tensor<Element>::pad_next_power_of_two + to_field_mle on a tensor that is already on the
 * device (zkml/src/tensor/mod.rs:328-401, 812-990): the base-field table of the padded shape,
 * zero outside the unpadded region.  `tensor` (DPS_I64, DPS_I16 or DPS_BASE) is stored row-major
 * in its unpadded shape or in its padded one, as for dps_partial_eval.  Queued on the context's
 * stream, no wait. */
int32_t dps_mle_from_tensor(dps_ctx *ctx, const dps_mle *tensor, const uint64_t *padded_dims, const uint64_t *unpadded_dims,
                            uint32_t n_dims, dps_mle **out);
/* borrow device memory the caller owns (kind DPS_BASE / DPS_I64 / DPS_I16: d_c1 is NULL); dps_mle_free of such a
 * handle waits for the context's queued work, after which the memory is the caller's again */
int32_t dps_mle_wrap_device(dps_ctx *ctx, int32_t kind, void *d_c0, void *d_c1, uint64_t len, dps_mle **out);
/* SmartSlice::Borrowed: a window [offset, offset + 2^n_vars) sharing storage */
int32_t dps_mle_view(const dps_mle *src, uint64_t offset, uint32_t n_vars, dps_mle **out);
/* `src` read by a sumcheck as a table of n_vars variables that is 0 wherever one of
 * the added (higher) variables is 1: DensePolynomial::zero_pad_num_vars on a view
 * (zkml/src/poly_commit/prover.rs:214-226).  Nothing is copied or materialised;
 * the final evaluation dps_sc_finish returns for it is that of the padded table,
 * src(point_low) * prod (1 - point_high).  n_vars must equal the session's; the
 * handle is accepted by dps_sc_begin, dps_mle_info, dps_mle_download and dps_mle_free only. */
int32_t dps_mle_zero_pad(const dps_mle *src, uint32_t n_vars, dps_mle **out);
int32_t dps_mle_info(const dps_mle *mle, int32_t *kind, uint64_t *len);
/* copy back; c1 may be NULL for DPS_BASE / DPS_I64 / DPS_I16 (raw tensors come back as int64_t values in c0) */
int32_t dps_mle_download(const dps_mle *mle, uint64_t *c0, uint64_t *c1);
int32_t dps_mle_free(dps_mle *mle);

/* ---- poly::eq::evals (zkml/src/layers/hadamard.rs:103, zkml/src/layers/einsum/axis.rs:1032,
 *      zkml/src/lookup/logup_gkr/prover.rs:247-249): out[i] = prod_j (bit_j(i) ? r_j : 1 - r_j) ---- */
/* (Entries are materialised when something reads them: a table of more than 17 variables has only its small suffix
 * tables built here, one of at most 7 variables nothing -- a sum the host works out reads the point.) */
int32_t dps_eq_build(dps_ctx *ctx, const uint64_t *point /* 2*m */, uint32_t m, dps_mle **out);
/* `count` eq tables, table i at points[i] of m[i] coordinates (zkml/src/poly_commit/prover.rs:176-181 and
 * zkml/src/iop/same_poly.rs:88-91 build one per claim): every table of at most 2^16 entries comes out of one launch. */
int32_t dps_eq_build_many(dps_ctx *ctx, const uint64_t *const *points, const uint32_t *m, uint32_t count, dps_mle **out);

/* ---- DensePolynomial::{evaluate, fix_low_variables, fix_high_variables}
 *      (zkml/src/layers/einsum/prove.rs:208, zkml/src/tensor/mod.rs:1892, zkml/src/iop/prover.rs:448,509) ---- */
int32_t dps_mle_evaluate(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point /* 2*n */, uint32_t n, uint64_t out[2]);
/* The same evaluation for callers that cannot allocate.  No counterpart in the reference: it is for tight serving
 * loops and harnesses that forbid hipMalloc.  The call makes no hipMalloc, hipFree or host allocation and waits for
 * no stream (it returns when the value has crossed to the host, which it polls for: not a call to record under stream
 * capture); its eq tables, partial sums and ticket counter live in a file-scope device array of the library (144 KiB
 * per GPU, held until the process ends).  At most 24 variables (DPS_ERR_UNSUPPORTED beyond).  Every context on one
 * GPU shares that GPU's array: the library lets one such call at a time use it, others wait their turn.  An eq table
 * whose entries have not been read yet (dps_eq_build keeps a large one unmaterialised) is evaluated in closed form on
 * the host.  DPS_ERR_STATE while a session of the context has a launch waiting on the GPU (between its rounds):
 * ending that launch would take a stream wait. */
int32_t dps_mle_evaluate_noalloc(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point /* 2*n */, uint32_t n, uint64_t out[2]);
/* point[j] binds variable j */
int32_t dps_mle_fix_low(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point /* 2*k */, uint32_t k, dps_mle **out);
/* point[j] binds variable n-k+j */
int32_t dps_mle_fix_high(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point /* 2*k */, uint32_t k, dps_mle **out);

/* ---- FixedAxesMapping::mles_from_tensor (zkml/src/layers/einsum/axis.rs:1142-1234) ----
 * tensor: row-major, stored either with padded_dims (only the unpadded region is
 * read) or compactly with unpadded_dims -- a raw quantised tensor as the model
 * holds it, never padded or embedded by the caller; the two are told apart by
 * the table's length.
 * kinds[a]: 0 contracted, 1 outer, 2 stacked.  points[a]: 2*log2(padded_dims[a])
 * limbs for outer axes (the claim-point slice of that axis), ignored otherwise.
 * Produces prod(stacked dims) tables of 2^ceil_log2(prod(contracted dims))
 * extension entries, zero padded, written to out[0 .. *n_out). */
enum { DPS_AXIS_CONTRACTED = 0, DPS_AXIS_OUTER = 1, DPS_AXIS_STACKED = 2 };
int32_t dps_partial_eval(dps_ctx *ctx, const dps_mle *tensor, const uint64_t *padded_dims,
                         const uint64_t *unpadded_dims, uint32_t n_dims, const int32_t *kinds,
                         const uint64_t *const *points, dps_mle **out, uint32_t out_cap, uint32_t *n_out);

/* ---- VirtualPolynomialsBuilder::to_virtual_polys + IOPProverState::prove
 *      (zkml/src/layers/einsum/prove.rs:164-189, zkml/src/layers/hadamard.rs:107-129,
 *       zkml/src/lookup/logup_gkr/prover.rs:263-281) ----
 * The expression arrives flattened: sum over terms of coeff * product of tables.
 * A table with fewer than n_vars variables depends on the last (highest) ones
 * only, as the batched LogUp driver requires (prover.rs:208-249). */
typedef struct dps_term {
    uint64_t coeff[2];
    uint32_t n_factors; /* 0 .. DPS_MAX_DEGREE; 0 is a constant term */
    uint32_t factors[DPS_MAX_FACTORS];
} dps_term;

/* The tables are borrowed and never written. */
int32_t dps_sc_begin(dps_ctx *ctx, uint32_t n_vars, const dps_mle *const *mles, uint32_t n_mles,
                     const dps_term *terms, uint32_t n_terms, dps_sc **out);
int32_t dps_sc_degree(const dps_sc *sc, uint32_t *degree);
/* Optional, before round 1: the value of the whole sum, when the caller knows it (the reference's callers do: they put
 * it on the transcript before they call prove, e.g. current_claim at logup_gkr/prover.rs:257-261).  Round 1 then takes
 * p(1) = claim - p(0) instead of evaluating at 1, as every later round does with the claim it derives itself.  The
 * messages are the same bits as without the call if the claim is the true sum; with a wrong claim the proof is wrong. */
int32_t dps_sc_set_claim(dps_sc *sc, const uint64_t *claim /* 2 limbs */);
/* One round: fold with the previous round's challenge (NULL in round 1), then
 * evaluate.  evals_out receives degree+1 extension elements, p(0..degree).  Only
 * these cross to the host. */
int32_t dps_sc_round(dps_sc *sc, const uint64_t *challenge, uint64_t *evals_out);
/* After the last round: fold with the last challenge;
 * get_mle_flatten_final_evaluations (einsum/prove.rs:188): one element per table,
 * in registration order. */
int32_t dps_sc_finish(dps_sc *sc, const uint64_t *challenge, uint64_t *final_evals_out /* 2*n_mles */);
/* give a session up part-way: a kernel of it that is resident on the GPU exits, further rounds fail with
 * DPS_ERR_STATE; the handle remains to be freed */
int32_t dps_sc_abort(dps_sc *sc);
int32_t dps_sc_free(dps_sc *sc);

/* Transcript hook: absorb `n_evals` extension elements of round `round`
 * (1-based), write the squeezed challenge.  Non-zero aborts the proof. */
typedef int32_t (*dps_round_fn)(void *user, uint32_t round, const uint64_t *evals, uint32_t n_evals,
                                uint64_t *challenge_out);
/* The whole loop: proof_out n_vars*(degree+1) elements, point_out n_vars
 * elements (collect_raw_challenges, einsum/prove.rs:189), final_evals_out n_mles. */
int32_t dps_sc_prove(dps_sc *sc, dps_round_fn fn, void *user, uint64_t *proof_out, uint64_t *point_out,
                     uint64_t *final_evals_out);

/* ---- LogUpCircuit::new / LogUpLayer::next_layer (zkml/src/lookup/logup_gkr/circuit.rs:88-184,512-516) ----
 * cols: n_cols base tables of equal power-of-two length; numer: multiplicity
 * table (table instance) or NULL (lookup instance, numerators -1). */
int32_t dps_logup_build(dps_ctx *ctx, const dps_mle *const *cols, uint32_t n_cols, const dps_mle *numer,
                        const uint64_t c[2], const uint64_t beta[2], dps_logup **out);
/* number of layers including the input layer 0 */
int32_t dps_logup_num_layers(const dps_logup *lg, uint32_t *n_layers);
/* numerator and denominator tables of layer k >= 1 (views; free them with dps_mle_free).  The layers of at most 256
 * entries per array also lie in host memory (the build's last launch leaves them there; the copies of the last 8
 * trees of a context are kept): a sumcheck of at most 7 variables over such tables, or windows into them, and an
 * eq factor runs on the host from its first round, without a launch -- same messages, bit for bit. */
int32_t dps_logup_layer(const dps_logup *lg, uint32_t k, dps_mle **num, dps_mle **den);
/* LogUpCircuit::outputs (circuit.rs:558-560): n_lo, n_hi, d_lo, d_hi of the last layer */
int32_t dps_logup_outputs(const dps_logup *lg, uint64_t out[8]);
int32_t dps_logup_free(dps_logup *lg);

/* ---- measurement: the context's device memory, and HIP-event timing of the library's own launches ---- */
/* Device blocks the context has taken from the driver (hipMalloc): those handed out, those cached for reuse, and the
 * bytes of both.  Unchanged across a call means the call took nothing from the driver and gave nothing back. */
int32_t dps_ctx_pool_info(const dps_ctx *ctx, uint64_t *blocks_in_use, uint64_t *blocks_cached, uint64_t *bytes);
enum {
    DPS_K_EVAL_FIRST = 0, /* first-round evaluation of a product of full-size tables */
    DPS_K_FOLD_EVAL = 1,  /* fused fold + evaluation of a product */
    DPS_K_EVAL_TERMS = 2, /* general term evaluation */
    DPS_K_FOLD = 3,       /* stand-alone fold */
    DPS_K_EQ = 4,         /* eq table expansion */
    DPS_K_AXIS_DOT = 5,   /* partial evaluation of one axis */
    DPS_K_LOGUP = 6,      /* fraction-sum layer */
    DPS_K_FINALIZE = 7,   /* round result without an evaluation launch */
    DPS_K_TAIL = 8,       /* resident kernel running the last rounds (duration includes the host's turns) */
    DPS_K_COUNT = 9
};
/* when enabled every launch of the kernels above is bracketed by events on the
 * context's stream (adds a few microseconds per launch) */
int32_t dps_profile_enable(dps_ctx *ctx, int32_t on);
int32_t dps_profile_reset(dps_ctx *ctx);
/* per kernel class: launches, summed duration, summed algorithmic bytes, and
 * the same three for the single largest launch (by bytes) seen */
int32_t dps_profile_read(dps_ctx *ctx, int32_t kernel, uint64_t *launches, double *total_ms, double *total_bytes,
                         uint64_t *max_launches, double *max_ms, double *max_bytes);
const char *dps_kernel_name(int32_t kernel);

/* ---- arithmetic self-check: element-wise field operations on device vectors ----
 * a, b, out: n c0 limbs followed by n c1 limbs.  op: 0 add, 1 sub, 2 extension
 * product, 3 two independent base products (c0*c0, c1*c1), 4 extension times
 * base (b.c0), 5 (embed int64 a.c0, a.c1 times the 32-bit constant b.c1),
 * 6 a b + a with one reduction per limb, 7 (a.c0 b.c0 + a.c1, a.c0 b.c0 + a.c1 b.c1 + b.c0)
 * in the base field, 8 the unreduced sum 40 (a b + b a.c1 + a) + (0, 40 b.c0). */
int32_t dps_debug_field_op(dps_ctx *ctx, int32_t op, const uint64_t *a, const uint64_t *b, uint64_t n, uint64_t *out);

/* ---- bandwidth yardstick: `reps` launches of a plain device-to-device copy of
 * n_bytes (a multiple of 16); returns the average launch duration.  No
 * counterpart in the reference; it is what the evaluation kernels' bandwidth
 * and the profiler's memory counters are read against. */
int32_t dps_debug_copy(dps_ctx *ctx, uint64_t n_bytes, uint32_t reps, double *avg_ms_out);
/* the same for a launch that only reads n_bytes (what a round's first evaluation is read against) */
int32_t dps_debug_read(dps_ctx *ctx, uint64_t n_bytes, uint32_t reps, double *avg_ms_out);

#ifdef __cplusplus
}
#endif
#endif
