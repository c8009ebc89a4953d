//! `VirtualPolynomialsBuilder` and `IOPProverState::prove` as the layer provers call them
//! (`zkml/src/layers/einsum/prove.rs:164-189`, `zkml/src/layers/hadamard.rs:107-129`,
//! `zkml/src/iop/same_poly.rs:93-112`, `zkml/src/lookup/logup_gkr/prover.rs:263-281`).
//!
//! `prove` runs the whole protocol: `dps_sc_begin` with the flattened expression, then the library's
//! round loop (`dps_sc_prove`) calling back into the caller's transcript once per round.  Round `j`
//! binds variable `j - 1`, so the challenges in round order are the little-endian evaluation point of
//! the final claims.  Tables are borrowed and never written.

use std::ffi::c_void;
use std::marker::PhantomData;
use std::ptr;

use dp_sumcheck_sys as sys;
use either::Either;

use crate::context::Context;
use crate::error::{Error, Result};
use crate::expression::Expression;
use crate::field::{from_limbs, ExtField};
use crate::poly::DensePolynomial;
use crate::transcript::Transcript;

/// The engine splits the hypercube over GPU workgroups by itself; the function exists so that call
/// sites read like the reference's (`zkml/src/layers/einsum/prove.rs:162`).
pub fn optimal_sumcheck_threads(_num_vars: usize) -> usize {
    1
}

/// One round's message: `p(0), ..., p(d)`.
#[derive(Clone, Debug, PartialEq)]
#[cfg_attr(feature = "serde", derive(serde::Serialize, serde::Deserialize))]
#[cfg_attr(feature = "serde", serde(bound = ""))]
pub struct IOPProverMessage<F: ExtField> {
    #[cfg_attr(feature = "serde", serde(with = "crate::serialization"))]
    pub evaluations: Vec<F>,
}

/// The proof as the layer proofs embed it (`einsum_sumcheck: IOPProof<F>`,
/// `zkml/src/layers/einsum/mod.rs:588-599`; `sumcheck_proofs: Vec<IOPProof<F>>`,
/// `zkml/src/lookup/logup_gkr/structs.rs:561-578`).
#[derive(Clone, Debug, PartialEq)]
#[cfg_attr(feature = "serde", derive(serde::Serialize, serde::Deserialize))]
#[cfg_attr(feature = "serde", serde(bound = ""))]
pub struct IOPProof<F: ExtField> {
    pub proofs: Vec<IOPProverMessage<F>>,
}

impl<F: ExtField> IOPProof<F> {
    /// `p_1(0) + p_1(1)`: the sum the proof is about (`zkml/src/layers/hadamard.rs:117-121`)
    pub fn extract_sum(&self) -> F {
        match self.proofs.first() {
            Some(m) if m.evaluations.len() >= 2 => m.evaluations[0] + m.evaluations[1],
            _ => F::ZERO,
        }
    }
}

/// Registered tables plus the flattened expression: what `to_virtual_polys` hands to `prove`.
pub struct VirtualPolynomials<'a, F: ExtField> {
    ctx: Context,
    num_vars: usize,
    mles: Vec<*const sys::dps_mle>,
    terms: Vec<sys::dps_term>,
    degree: usize,
    _borrow: PhantomData<&'a DensePolynomial<F>>,
}

impl<'a, F: ExtField> VirtualPolynomials<'a, F> {
    pub fn num_vars(&self) -> usize {
        self.num_vars
    }
    pub fn degree(&self) -> usize {
        self.degree
    }
}

pub struct VirtualPolynomialsBuilder<'a, F: ExtField> {
    num_vars: usize,
    mles: Vec<&'a DensePolynomial<F>>,
}

impl<'a, F: ExtField> VirtualPolynomialsBuilder<'a, F> {
    pub fn new(_num_threads: usize, num_vars: usize) -> Self {
        VirtualPolynomialsBuilder { num_vars, mles: Vec::new() }
    }

    /// Tables registered up front: `WitIn(i)` is the `i`-th of them.  Either arm is a borrow here: the
    /// engine folds into session scratch and never writes a caller's table.
    pub fn new_with_mles(
        num_threads: usize,
        num_vars: usize,
        mles: Vec<Either<&'a DensePolynomial<F>, &'a mut DensePolynomial<F>>>,
    ) -> Self {
        let mut b = Self::new(num_threads, num_vars);
        for m in mles {
            let shared: &'a DensePolynomial<F> = match m {
                Either::Left(p) => p,
                Either::Right(p) => p,
            };
            b.mles.push(shared);
        }
        b
    }

    /// Registers a table and returns its `WitIn`.
    pub fn lift(&mut self, mle: Either<&'a DensePolynomial<F>, &'a mut DensePolynomial<F>>) -> Expression<F> {
        let shared: &'a DensePolynomial<F> = match mle {
            Either::Left(p) => p,
            Either::Right(p) => p,
        };
        self.mles.push(shared);
        Expression::WitIn((self.mles.len() - 1) as u16)
    }

    /// Substitutes the challenges and flattens the expressions (their sum is proven) to monomials.
    pub fn to_virtual_polys(&self, exprs: &[Expression<F>], challenges: &[F]) -> Result<VirtualPolynomials<'a, F>> {
        let first = self.mles.first().ok_or_else(|| Error::invalid("to_virtual_polys: no tables registered"))?;
        let mut terms = Vec::new();
        let mut degree = 0usize;
        for e in exprs {
            for m in e.to_monomials(challenges) {
                if m.wits.len() > sys::DPS_MAX_FACTORS {
                    return Err(Error {
                        status: sys::DPS_ERR_UNSUPPORTED,
                        message: format!("to_virtual_polys: a product of {} tables", m.wits.len()),
                    });
                }
                let mut t = sys::dps_term { coeff: m.coeff.to_limbs(), n_factors: m.wits.len() as u32, factors: [0; sys::DPS_MAX_FACTORS] };
                for (i, w) in m.wits.iter().enumerate() {
                    t.factors[i] = *w as u32;
                }
                degree = degree.max(m.wits.len());
                terms.push(t);
            }
        }
        Ok(VirtualPolynomials {
            ctx: first.context().clone(),
            num_vars: self.num_vars,
            mles: self.mles.iter().map(|p| p.as_ptr()).collect(),
            terms,
            degree,
            _borrow: PhantomData,
        })
    }
}

/// What `prove` leaves behind: the challenges in round order and the final evaluation of every
/// registered table, in registration order (callers slice by index: `zkml/src/layers/einsum/prove.rs:186-189`).
pub struct IOPProverState<F: ExtField> {
    challenges: Vec<F>,
    final_evaluations: Vec<F>,
}

struct RoundHook<'t, F: ExtField, T: Transcript<F>> {
    transcript: &'t mut T,
    _f: PhantomData<F>,
}

// Called by the library once per round with the d + 1 evaluations; returns the challenge.
unsafe extern "C" fn round_hook<F: ExtField, T: Transcript<F>>(
    user: *mut c_void,
    _round: u32,
    evals: *const u64,
    n_evals: u32,
    challenge_out: *mut u64,
) -> i32 {
    let hook = &mut *(user as *mut RoundHook<'_, F, T>);
    let words = std::slice::from_raw_parts(evals, 2 * n_evals as usize);
    let mut msg = Vec::with_capacity(n_evals as usize);
    for p in words.chunks_exact(2) {
        match F::from_limbs(p[0], p[1]) {
            Some(x) => msg.push(x),
            None => return 1,
        }
    }
    hook.transcript.append_scalars(&msg);
    let r = hook.transcript.challenge_scalar().to_limbs();
    *challenge_out = r[0];
    *challenge_out.add(1) = r[1];
    0
}

struct Session(*mut sys::dps_sc);

impl Drop for Session {
    fn drop(&mut self) {
        unsafe {
            sys::dps_sc_free(self.0);
        }
    }
}

impl<F: ExtField> IOPProverState<F> {
    /// `IOPProverState::<F>::prove(virtual_poly, transcript)`.  dp-crypto's version is infallible by
    /// panic; this one panics too, with the library's error text (use [`IOPProverState::try_prove`]
    /// for the status).
    pub fn prove<T: Transcript<F>>(vp: VirtualPolynomials<'_, F>, transcript: &mut T) -> (IOPProof<F>, IOPProverState<F>) {
        match Self::try_prove(vp, transcript, None) {
            Ok(r) => r,
            Err(e) => panic!("sumcheck prove failed: {}", e),
        }
    }

    /// `claimed_sum`: the value of the whole sum when the caller holds it (the reference's callers put
    /// it on the transcript before they call `prove`, e.g. `zkml/src/lookup/logup_gkr/prover.rs:257-261`);
    /// round 1 then need not evaluate the polynomial at 1.  Same messages if the claim is the true sum.
    pub fn try_prove<T: Transcript<F>>(
        vp: VirtualPolynomials<'_, F>,
        transcript: &mut T,
        claimed_sum: Option<F>,
    ) -> Result<(IOPProof<F>, IOPProverState<F>)> {
        let ctx = &vp.ctx;
        let mut sc = ptr::null_mut();
        let rc = unsafe {
            sys::dps_sc_begin(
                ctx.as_ptr(),
                vp.num_vars as u32,
                vp.mles.as_ptr(),
                vp.mles.len() as u32,
                vp.terms.as_ptr(),
                vp.terms.len() as u32,
                &mut sc,
            )
        };
        ctx.check(rc, "dps_sc_begin")?;
        let session = Session(sc);
        if let Some(c) = claimed_sum {
            let limbs = c.to_limbs();
            let rc = unsafe { sys::dps_sc_set_claim(session.0, limbs.as_ptr()) };
            ctx.check(rc, "dps_sc_set_claim")?;
        }
        let mut degree = 0u32;
        unsafe {
            sys::dps_sc_degree(session.0, &mut degree);
        }
        // what prove absorbs before round 1
        transcript.append_u64(vp.num_vars as u64);
        transcript.append_u64(degree as u64);
        let npts = degree as usize + 1;
        let mut proof = vec![0u64; 2 * npts * vp.num_vars];
        let mut point = vec![0u64; 2 * vp.num_vars];
        let mut finals = vec![0u64; 2 * vp.mles.len().max(1)];
        let mut hook = RoundHook::<F, T> { transcript, _f: PhantomData };
        let rc = unsafe {
            sys::dps_sc_prove(
                session.0,
                Some(round_hook::<F, T>),
                &mut hook as *mut RoundHook<'_, F, T> as *mut c_void,
                proof.as_mut_ptr(),
                point.as_mut_ptr(),
                finals.as_mut_ptr(),
            )
        };
        ctx.check(rc, "dps_sc_prove")?;
        let proofs = proof.chunks_exact(2 * npts).map(|m| IOPProverMessage { evaluations: from_limbs::<F>(m) }).collect();
        let state = IOPProverState {
            challenges: from_limbs::<F>(&point),
            final_evaluations: from_limbs::<F>(&finals[..2 * vp.mles.len()]),
        };
        Ok((IOPProof { proofs }, state))
    }

    /// one element per registered table, in registration order
    pub fn get_mle_flatten_final_evaluations(&self) -> Vec<F> {
        self.final_evaluations.clone()
    }

    /// the challenges in round order = the little-endian point of the final claims
    pub fn collect_raw_challenges(&self) -> Vec<F> {
        self.challenges.clone()
    }
}
