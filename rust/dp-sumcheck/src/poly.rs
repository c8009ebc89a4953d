//! `DensePolynomial`: a multilinear polynomial as its little-endian evaluation table, resident in
//! HBM (entry `i` sits at the point whose `j`-th coordinate is bit `j` of `i`; a row-major tensor's
//! last dimension occupies the lowest variables, `zkml/src/shape.rs:475-496`).  Owned tables and
//! borrowed windows (`SmartSlice::Borrowed`, `zkml/src/lookup/logup_gkr/circuit.rs:262-269`) are the
//! same type: a window shares its parent's storage, which the library reference-counts.
//! [`eq::evals`] is `poly::eq::evals(&point).into_mle()`.

use std::marker::PhantomData;
use std::ptr;

use dp_sumcheck_sys as sys;

use crate::context::Context;
use crate::error::{Error, Result};
use crate::field::{from_limbs, to_limbs, ExtField};

pub struct DensePolynomial<F: ExtField> {
    ctx: Context,
    h: *mut sys::dps_mle,
    _f: PhantomData<F>,
}

impl<F: ExtField> Drop for DensePolynomial<F> {
    fn drop(&mut self) {
        unsafe {
            sys::dps_mle_free(self.h);
        }
    }
}

fn log2_strict(n: usize) -> Result<u32> {
    if n == 0 || !n.is_power_of_two() {
        return Err(Error::invalid(format!("table length {} is not a power of two", n)));
    }
    Ok(n.trailing_zeros())
}

impl<F: ExtField> DensePolynomial<F> {
    pub(crate) fn from_handle(ctx: &Context, h: *mut sys::dps_mle) -> Self {
        DensePolynomial { ctx: ctx.clone(), h, _f: PhantomData }
    }

    /// `DensePolynomial::new(Vec<F>)`: uploads the evaluations (two limb arrays on the device).
    pub fn new(ctx: &Context, evals: &[F]) -> Result<Self> {
        let n_vars = log2_strict(evals.len())?;
        let mut c0 = Vec::with_capacity(evals.len());
        let mut c1 = Vec::with_capacity(evals.len());
        for e in evals {
            let l = e.to_limbs();
            c0.push(l[0]);
            c1.push(l[1]);
        }
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_from_ext2(ctx.as_ptr(), c0.as_ptr(), c1.as_ptr(), n_vars, &mut h) };
        ctx.check(rc, "dps_mle_from_ext2")?;
        Ok(Self::from_handle(ctx, h))
    }

    /// Base-field evaluations (canonical `u64`): half the bytes, cheaper first rounds.
    pub fn from_base(ctx: &Context, evals: &[u64]) -> Result<Self> {
        let n_vars = log2_strict(evals.len())?;
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_from_base(ctx.as_ptr(), evals.as_ptr(), n_vars, &mut h) };
        ctx.check(rc, "dps_mle_from_base")?;
        Ok(Self::from_handle(ctx, h))
    }

    /// `Tensor<Element>::to_field_mle` (`zkml/src/tensor/mod.rs:328-401`): quantised integers embedded
    /// (`F::from(i64)`) and zero-padded to the next power of two, on the device.
    pub fn from_i64(ctx: &Context, values: &[i64]) -> Result<Self> {
        let n_vars = values.len().max(1).next_power_of_two().trailing_zeros();
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_from_i64(ctx.as_ptr(), values.as_ptr(), values.len() as u64, n_vars, &mut h) };
        ctx.check(rc, "dps_mle_from_i64")?;
        Ok(Self::from_handle(ctx, h))
    }

    /// `new_from_smart_slice(SmartSlice::Borrowed(&evals[offset .. offset + 2^n_vars]))`: no copy.
    pub fn view(&self, offset: u64, n_vars: u32) -> Result<Self> {
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_view(self.h, offset, n_vars, &mut h) };
        self.ctx.check(rc, "dps_mle_view")?;
        Ok(Self::from_handle(&self.ctx, h))
    }

    /// `as_view()`: a window over the whole table
    pub fn as_view(&self) -> Result<Self> {
        self.view(0, self.num_vars() as u32)
    }

    /// `zero_pad_num_vars(n)` on a view (`zkml/src/poly_commit/prover.rs:214-226`): read by a sumcheck
    /// over `n_vars` variables as 0 wherever an added (higher) variable is 1.  Nothing is materialised.
    pub fn zero_pad_num_vars(&self, n_vars: u32) -> Result<Self> {
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_zero_pad(self.h, n_vars, &mut h) };
        self.ctx.check(rc, "dps_mle_zero_pad")?;
        Ok(Self::from_handle(&self.ctx, h))
    }

    pub fn len(&self) -> usize {
        let mut len = 0u64;
        unsafe {
            sys::dps_mle_info(self.h, ptr::null_mut(), &mut len);
        }
        len as usize
    }

    pub fn is_empty(&self) -> bool {
        self.len() == 0
    }

    pub fn num_vars(&self) -> usize {
        self.len().max(1).trailing_zeros() as usize
    }

    /// `evals()`: the table copied back to the host
    pub fn evals(&self) -> Result<Vec<F>> {
        let n = self.len();
        let mut c0 = vec![0u64; n];
        let mut c1 = vec![0u64; n];
        let rc = unsafe { sys::dps_mle_download(self.h, c0.as_mut_ptr(), c1.as_mut_ptr()) };
        self.ctx.check(rc, "dps_mle_download")?;
        Ok(c0
            .iter()
            .zip(c1.iter())
            .map(|(a, b)| F::from_limbs(*a, *b).expect("the library returned a non-canonical limb"))
            .collect())
    }

    /// `evaluate(&point)`: `point[j]` binds variable `j`
    pub fn evaluate(&self, point: &[F]) -> Result<F> {
        let limbs = to_limbs(point);
        let mut out = [0u64; 2];
        let rc = unsafe { sys::dps_mle_evaluate(self.ctx.as_ptr(), self.h, limbs.as_ptr(), point.len() as u32, out.as_mut_ptr()) };
        self.ctx.check(rc, "dps_mle_evaluate")?;
        Ok(from_limbs::<F>(&out)[0])
    }

    /// `fix_high_variables(&point)`: `point[j]` binds variable `n - k + j`
    pub fn fix_high_variables(&self, point: &[F]) -> Result<Self> {
        let limbs = to_limbs(point);
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_fix_high(self.ctx.as_ptr(), self.h, limbs.as_ptr(), point.len() as u32, &mut h) };
        self.ctx.check(rc, "dps_mle_fix_high")?;
        Ok(Self::from_handle(&self.ctx, h))
    }

    /// `fix_low_variables(&point)`: `point[j]` binds variable `j`
    pub fn fix_low_variables(&self, point: &[F]) -> Result<Self> {
        let limbs = to_limbs(point);
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_mle_fix_low(self.ctx.as_ptr(), self.h, limbs.as_ptr(), point.len() as u32, &mut h) };
        self.ctx.check(rc, "dps_mle_fix_low")?;
        Ok(Self::from_handle(&self.ctx, h))
    }

    pub fn context(&self) -> &Context {
        &self.ctx
    }

    pub fn as_ptr(&self) -> *const sys::dps_mle {
        self.h
    }
}

pub mod eq {
    //! `poly::eq::evals` (`zkml/src/layers/hadamard.rs:103`, `zkml/src/layers/einsum/axis.rs:1032`,
    //! `zkml/src/lookup/logup_gkr/prover.rs:247-249`): `out[i] = prod_j (bit_j(i) ? r_j : 1 - r_j)`.
    use super::*;

    /// The table of `eq(point, .)`, built on the device.  A table of more than 17 variables is not
    /// written out until something reads its entries: a sumcheck takes the eq factor in closed form.
    pub fn evals<F: ExtField>(ctx: &Context, point: &[F]) -> Result<DensePolynomial<F>> {
        let limbs = to_limbs(point);
        let mut h = ptr::null_mut();
        let rc = unsafe { sys::dps_eq_build(ctx.as_ptr(), limbs.as_ptr(), point.len() as u32, &mut h) };
        ctx.check(rc, "dps_eq_build")?;
        Ok(DensePolynomial::from_handle(ctx, h))
    }

    /// One table per point (`zkml/src/poly_commit/prover.rs:176-181`, `zkml/src/iop/same_poly.rs:88-91`
    /// build one per claim): the small ones come out of one launch.
    pub fn evals_many<F: ExtField>(ctx: &Context, points: &[Vec<F>]) -> Result<Vec<DensePolynomial<F>>> {
        let limbs: Vec<Vec<u64>> = points.iter().map(|p| to_limbs(p)).collect();
        let ptrs: Vec<*const u64> = limbs.iter().map(|l| l.as_ptr()).collect();
        let m: Vec<u32> = points.iter().map(|p| p.len() as u32).collect();
        let mut hs: Vec<*mut sys::dps_mle> = vec![ptr::null_mut(); points.len()];
        let rc = unsafe { sys::dps_eq_build_many(ctx.as_ptr(), ptrs.as_ptr(), m.as_ptr(), points.len() as u32, hs.as_mut_ptr()) };
        ctx.check(rc, "dps_eq_build_many")?;
        Ok(hs.into_iter().map(|h| DensePolynomial::from_handle(ctx, h)).collect())
    }
}
