//! Raw declarations of the C ABI of `libdpsumcheck.so` (`include/dpsumcheck.h`), one for one: every
//! function, enum constant and struct of the header, nothing else.  The safe layer with dp-crypto's
//! names is the `dp-sumcheck` crate next to this one.
//!
//! Conventions of the ABI (the header has them in full): Goldilocks `p = 2^64 - 2^32 + 1` and its
//! extension by `X^2 = 7`; an extension element crosses as two `u64` limbs `(c0, c1)`; tables are
//! little-endian evaluation tables in device memory; every call returns a `dps_status` (0 = ok) and
//! never unwinds.  Calls on one context must not overlap; different contexts may be used from
//! different threads at the same time.
#![no_std]
#![allow(non_camel_case_types)]

use core::ffi::{c_char, c_void};

/// factor slots in a term
pub const DPS_MAX_FACTORS: usize = 8;
/// largest product the kernels evaluate
pub const DPS_MAX_DEGREE: usize = 6;

// dps_status
pub const DPS_OK: i32 = 0;
pub const DPS_ERR_INVALID: i32 = 1;
pub const DPS_ERR_HIP: i32 = 2;
pub const DPS_ERR_OOM: i32 = 3;
pub const DPS_ERR_STATE: i32 = 4;
pub const DPS_ERR_UNSUPPORTED: i32 = 5;
pub const DPS_ERR_CALLBACK: i32 = 6;

// dps_kind
pub const DPS_BASE: i32 = 0;
pub const DPS_EXT2: i32 = 1;
pub const DPS_I64: i32 = 2;
pub const DPS_I16: i32 = 3;

// axis kinds of dps_partial_eval
pub const DPS_AXIS_CONTRACTED: i32 = 0;
pub const DPS_AXIS_OUTER: i32 = 1;
pub const DPS_AXIS_STACKED: i32 = 2;

// kernel classes of dps_profile_read
pub const DPS_K_EVAL_FIRST: i32 = 0;
pub const DPS_K_FOLD_EVAL: i32 = 1;
pub const DPS_K_EVAL_TERMS: i32 = 2;
pub const DPS_K_FOLD: i32 = 3;
pub const DPS_K_EQ: i32 = 4;
pub const DPS_K_AXIS_DOT: i32 = 5;
pub const DPS_K_LOGUP: i32 = 6;
pub const DPS_K_FINALIZE: i32 = 7;
pub const DPS_K_TAIL: i32 = 8;
pub const DPS_K_COUNT: i32 = 9;

/// Opaque handles: only ever used behind a pointer.
#[repr(C)]
pub struct dps_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct dps_mle {
    _private: [u8; 0],
}
#[repr(C)]
pub struct dps_sc {
    _private: [u8; 0],
}
#[repr(C)]
pub struct dps_logup {
    _private: [u8; 0],
}

/// One term of the flattened expression: `coeff * product of tables`.
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct dps_term {
    pub coeff: [u64; 2],
    /// 0 ..= DPS_MAX_DEGREE; 0 is a constant term
    pub n_factors: u32,
    pub factors: [u32; DPS_MAX_FACTORS],
}

/// Transcript hook: absorb `n_evals` extension elements of round `round` (1-based), write the
/// squeezed challenge (two limbs).  Non-zero aborts the proof.
pub type dps_round_fn = Option<
    unsafe extern "C" fn(user: *mut c_void, round: u32, evals: *const u64, n_evals: u32, challenge_out: *mut u64) -> i32,
>;

extern "C" {
    // ---- context ----
    pub fn dps_ctx_create(device: i32, out: *mut *mut dps_ctx) -> i32;
    pub fn dps_ctx_destroy(ctx: *mut dps_ctx) -> i32;
    pub fn dps_last_error(ctx: *const dps_ctx) -> *const c_char;
    pub fn dps_status_str(status: i32) -> *const c_char;
    pub fn dps_ctx_sync(ctx: *mut dps_ctx) -> i32;
    pub fn dps_device_set_resident_budget(device: i32, compute_units: i32) -> i32;
    pub fn dps_device_resident_budget(device: i32, in_use: *mut i32, budget: *mut i32) -> i32;

    // ---- table storage ----
    pub fn dps_mle_from_base(ctx: *mut dps_ctx, host: *const u64, n_vars: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_from_ext2(ctx: *mut dps_ctx, c0: *const u64, c1: *const u64, n_vars: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_from_i64(ctx: *mut dps_ctx, host: *const i64, len: u64, n_vars: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_tensor_from_i64(ctx: *mut dps_ctx, host: *const i64, len: u64, out: *mut *mut dps_mle) -> i32;
    pub fn dps_tensor_from_i16(ctx: *mut dps_ctx, host: *const i16, len: u64, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_from_tensor(
        ctx: *mut dps_ctx,
        tensor: *const dps_mle,
        padded_dims: *const u64,
        unpadded_dims: *const u64,
        n_dims: u32,
        out: *mut *mut dps_mle,
    ) -> i32;
    pub fn dps_mle_wrap_device(ctx: *mut dps_ctx, kind: i32, d_c0: *mut c_void, d_c1: *mut c_void, len: u64, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_view(src: *const dps_mle, offset: u64, n_vars: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_zero_pad(src: *const dps_mle, n_vars: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_info(mle: *const dps_mle, kind: *mut i32, len: *mut u64) -> i32;
    pub fn dps_mle_download(mle: *const dps_mle, c0: *mut u64, c1: *mut u64) -> i32;
    pub fn dps_mle_free(mle: *mut dps_mle) -> i32;

    // ---- poly::eq::evals ----
    pub fn dps_eq_build(ctx: *mut dps_ctx, point: *const u64, m: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_eq_build_many(ctx: *mut dps_ctx, points: *const *const u64, m: *const u32, count: u32, out: *mut *mut dps_mle) -> i32;

    // ---- evaluate / fix_low / fix_high ----
    pub fn dps_mle_evaluate(ctx: *mut dps_ctx, mle: *const dps_mle, point: *const u64, n: u32, out: *mut u64) -> i32;
    pub fn dps_mle_evaluate_noalloc(ctx: *mut dps_ctx, mle: *const dps_mle, point: *const u64, n: u32, out: *mut u64) -> i32;
    pub fn dps_mle_fix_low(ctx: *mut dps_ctx, mle: *const dps_mle, point: *const u64, k: u32, out: *mut *mut dps_mle) -> i32;
    pub fn dps_mle_fix_high(ctx: *mut dps_ctx, mle: *const dps_mle, point: *const u64, k: u32, out: *mut *mut dps_mle) -> i32;

    // ---- mles_from_tensor ----
    pub fn dps_partial_eval(
        ctx: *mut dps_ctx,
        tensor: *const dps_mle,
        padded_dims: *const u64,
        unpadded_dims: *const u64,
        n_dims: u32,
        kinds: *const i32,
        points: *const *const u64,
        out: *mut *mut dps_mle,
        out_cap: u32,
        n_out: *mut u32,
    ) -> i32;

    // ---- the sumcheck session ----
    pub fn dps_sc_begin(
        ctx: *mut dps_ctx,
        n_vars: u32,
        mles: *const *const dps_mle,
        n_mles: u32,
        terms: *const dps_term,
        n_terms: u32,
        out: *mut *mut dps_sc,
    ) -> i32;
    pub fn dps_sc_degree(sc: *const dps_sc, degree: *mut u32) -> i32;
    pub fn dps_sc_set_claim(sc: *mut dps_sc, claim: *const u64) -> i32;
    pub fn dps_sc_round(sc: *mut dps_sc, challenge: *const u64, evals_out: *mut u64) -> i32;
    pub fn dps_sc_finish(sc: *mut dps_sc, challenge: *const u64, final_evals_out: *mut u64) -> i32;
    pub fn dps_sc_abort(sc: *mut dps_sc) -> i32;
    pub fn dps_sc_free(sc: *mut dps_sc) -> i32;
    pub fn dps_sc_prove(
        sc: *mut dps_sc,
        round_fn: dps_round_fn,
        user: *mut c_void,
        proof_out: *mut u64,
        point_out: *mut u64,
        final_evals_out: *mut u64,
    ) -> i32;

    // ---- LogUp fraction-sum circuit ----
    pub fn dps_logup_build(
        ctx: *mut dps_ctx,
        cols: *const *const dps_mle,
        n_cols: u32,
        numer: *const dps_mle,
        c: *const u64,
        beta: *const u64,
        out: *mut *mut dps_logup,
    ) -> i32;
    pub fn dps_logup_num_layers(lg: *const dps_logup, n_layers: *mut u32) -> i32;
    pub fn dps_logup_layer(lg: *const dps_logup, k: u32, num: *mut *mut dps_mle, den: *mut *mut dps_mle) -> i32;
    pub fn dps_logup_outputs(lg: *const dps_logup, out: *mut u64) -> i32;
    pub fn dps_logup_free(lg: *mut dps_logup) -> i32;

    // ---- measurement ----
    pub fn dps_ctx_pool_info(ctx: *const dps_ctx, blocks_in_use: *mut u64, blocks_cached: *mut u64, bytes: *mut u64) -> i32;
    pub fn dps_profile_enable(ctx: *mut dps_ctx, on: i32) -> i32;
    pub fn dps_profile_reset(ctx: *mut dps_ctx) -> i32;
    pub fn dps_profile_read(
        ctx: *mut dps_ctx,
        kernel: i32,
        launches: *mut u64,
        total_ms: *mut f64,
        total_bytes: *mut f64,
        max_launches: *mut u64,
        max_ms: *mut f64,
        max_bytes: *mut f64,
    ) -> i32;
    pub fn dps_kernel_name(kernel: i32) -> *const c_char;
    pub fn dps_debug_field_op(ctx: *mut dps_ctx, op: i32, a: *const u64, b: *const u64, n: u64, out: *mut u64) -> i32;
    pub fn dps_debug_copy(ctx: *mut dps_ctx, n_bytes: u64, reps: u32, avg_ms_out: *mut f64) -> i32;
    pub fn dps_debug_read(ctx: *mut dps_ctx, n_bytes: u64, reps: u32, avg_ms_out: *mut f64) -> i32;
}
