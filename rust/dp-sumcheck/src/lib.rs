//! The sumcheck prover API the zkml layer provers call, with dp-crypto's names, on one MI355X.
//!
//! The reference's provers (`zkml/src/layers/einsum/prove.rs:164-189`, `zkml/src/layers/hadamard.rs:107-129`,
//! `zkml/src/iop/same_poly.rs:93-112`, `zkml/src/lookup/logup_gkr/prover.rs:263-281`) do
//!
//! ```ignore
//! let mut b = VirtualPolynomialsBuilder::<F>::new(num_threads, num_vars);
//! let expr = b.lift(Either::Left(&f)) * b.lift(Either::Left(&g)) * b.lift(Either::Left(&eq));
//! let vp = b.to_virtual_polys(&[expr], &[]);
//! let (proof, state) = IOPProverState::<F>::prove(vp, transcript);
//! state.get_mle_flatten_final_evaluations(); state.collect_raw_challenges();
//! ```
//!
//! and keep doing exactly that against this crate.  Tables ([`poly::DensePolynomial`]) live in HBM; the
//! transcript stays in Rust on the host: per round the `d + 1` evaluations of the round polynomial come
//! back from the GPU, the transcript absorbs them and squeezes the challenge, which goes back.
//!
//! Field: Goldilocks `p = 2^64 - 2^32 + 1` and its extension by `X^2 = 7` ([`field::GoldilocksExt2`]); an
//! element is the pair of limbs `(c0, c1)` that crosses the C ABI.
//!
//! What this crate cannot pin against dp-crypto (its source is not vendored in the reference): the byte
//! encodings inside the transcript and in [`serialization`], and what `prove` absorbs before round 1
//! (here: the number of variables and the degree, as `u64`).  Both sit on the host side of the ABI.

pub mod context;
pub mod error;
pub mod expression;
pub mod field;
pub mod poly;
pub mod prover;
#[cfg(feature = "serde")]
pub mod serialization;
pub mod transcript;
pub mod verifier;

pub use context::Context;
pub use error::{Error, Result};
pub use expression::Expression;
pub use field::{ExtField, GoldilocksExt2};
pub use poly::DensePolynomial;
pub use prover::{
    optimal_sumcheck_threads, IOPProof, IOPProverMessage, IOPProverState, VirtualPolynomials, VirtualPolynomialsBuilder,
};
pub use transcript::Transcript;
pub use verifier::{IOPVerifierState, SubClaim, VPAuxInfo};
