//! Goldilocks `p = 2^64 - 2^32 + 1` and its quadratic extension `F_p[X] / (X^2 - 7)` on the host: the
//! few elements that live above the ABI (challenges, coefficients, claims, round messages).
//! Table-sized arithmetic never runs here.

use std::ops::{Add, AddAssign, Mul, MulAssign, Neg, Sub, SubAssign};

pub const GOLDILOCKS_P: u64 = 0xFFFF_FFFF_0000_0001;
/// `X^2 = NON_RESIDUE`
pub const NON_RESIDUE: u64 = 7;

#[inline]
pub fn fp_add(a: u64, b: u64) -> u64 {
    let s = a as u128 + b as u128;
    (if s >= GOLDILOCKS_P as u128 { s - GOLDILOCKS_P as u128 } else { s }) as u64
}
#[inline]
pub fn fp_sub(a: u64, b: u64) -> u64 {
    if a >= b {
        a - b
    } else {
        a + (GOLDILOCKS_P - b)
    }
}
#[inline]
pub fn fp_neg(a: u64) -> u64 {
    if a == 0 {
        0
    } else {
        GOLDILOCKS_P - a
    }
}
#[inline]
pub fn fp_mul(a: u64, b: u64) -> u64 {
    ((a as u128 * b as u128) % GOLDILOCKS_P as u128) as u64
}
pub fn fp_pow(mut a: u64, mut e: u64) -> u64 {
    let mut r = 1u64;
    while e != 0 {
        if e & 1 == 1 {
            r = fp_mul(r, a);
        }
        a = fp_mul(a, a);
        e >>= 1;
    }
    r
}
pub fn fp_inv(a: u64) -> u64 {
    fp_pow(a, GOLDILOCKS_P - 2)
}
/// `F::from(i64)` of the reference (`zkml/src/quantization/mod.rs:262-266`): negatives map to `p - |x|`.
pub fn fp_from_i64(x: i64) -> u64 {
    if x >= 0 {
        x as u64
    } else {
        GOLDILOCKS_P - x.unsigned_abs()
    }
}

/// What the adapter needs of the field the provers are generic over: the two-limb form that crosses
/// the ABI, and ring arithmetic for the handful of elements handled on the host.
pub trait ExtField:
    Copy
    + PartialEq
    + std::fmt::Debug
    + Add<Output = Self>
    + Sub<Output = Self>
    + Mul<Output = Self>
    + Neg<Output = Self>
    + AddAssign
    + SubAssign
    + MulAssign
{
    const ZERO: Self;
    const ONE: Self;
    /// canonical limbs `(c0, c1)`, both below `p`
    fn to_limbs(&self) -> [u64; 2];
    /// `None` when a limb is not canonical
    fn from_limbs(c0: u64, c1: u64) -> Option<Self>;
    fn from_u64(x: u64) -> Self;
    fn is_zero(&self) -> bool;
    fn inverse(&self) -> Option<Self>;
    fn pow(&self, e: u64) -> Self {
        let mut r = Self::ONE;
        let mut a = *self;
        let mut e = e;
        while e != 0 {
            if e & 1 == 1 {
                r *= a;
            }
            a = a * a;
            e >>= 1;
        }
        r
    }
}

#[derive(Clone, Copy, PartialEq, Eq, Hash, Debug, Default)]
pub struct GoldilocksExt2 {
    pub c0: u64,
    pub c1: u64,
}

impl GoldilocksExt2 {
    pub const fn new(c0: u64, c1: u64) -> Self {
        GoldilocksExt2 { c0, c1 }
    }
    pub fn from_i64(x: i64) -> Self {
        GoldilocksExt2 { c0: fp_from_i64(x), c1: 0 }
    }
}

impl From<i64> for GoldilocksExt2 {
    fn from(x: i64) -> Self {
        GoldilocksExt2::from_i64(x)
    }
}

impl From<u64> for GoldilocksExt2 {
    fn from(x: u64) -> Self {
        GoldilocksExt2 { c0: x % GOLDILOCKS_P, c1: 0 }
    }
}

impl Add for GoldilocksExt2 {
    type Output = Self;
    fn add(self, o: Self) -> Self {
        GoldilocksExt2 { c0: fp_add(self.c0, o.c0), c1: fp_add(self.c1, o.c1) }
    }
}
impl Sub for GoldilocksExt2 {
    type Output = Self;
    fn sub(self, o: Self) -> Self {
        GoldilocksExt2 { c0: fp_sub(self.c0, o.c0), c1: fp_sub(self.c1, o.c1) }
    }
}
impl Neg for GoldilocksExt2 {
    type Output = Self;
    fn neg(self) -> Self {
        GoldilocksExt2 { c0: fp_neg(self.c0), c1: fp_neg(self.c1) }
    }
}
impl Mul for GoldilocksExt2 {
    type Output = Self;
    fn mul(self, o: Self) -> Self {
        // (a0 + a1 X)(b0 + b1 X) = (a0 b0 + 7 a1 b1) + (a0 b1 + a1 b0) X
        GoldilocksExt2 {
            c0: fp_add(fp_mul(self.c0, o.c0), fp_mul(NON_RESIDUE, fp_mul(self.c1, o.c1))),
            c1: fp_add(fp_mul(self.c0, o.c1), fp_mul(self.c1, o.c0)),
        }
    }
}
impl AddAssign for GoldilocksExt2 {
    fn add_assign(&mut self, o: Self) {
        *self = *self + o;
    }
}
impl SubAssign for GoldilocksExt2 {
    fn sub_assign(&mut self, o: Self) {
        *self = *self - o;
    }
}
impl MulAssign for GoldilocksExt2 {
    fn mul_assign(&mut self, o: Self) {
        *self = *self * o;
    }
}

impl ExtField for GoldilocksExt2 {
    const ZERO: Self = GoldilocksExt2 { c0: 0, c1: 0 };
    const ONE: Self = GoldilocksExt2 { c0: 1, c1: 0 };
    fn to_limbs(&self) -> [u64; 2] {
        [self.c0, self.c1]
    }
    fn from_limbs(c0: u64, c1: u64) -> Option<Self> {
        if c0 < GOLDILOCKS_P && c1 < GOLDILOCKS_P {
            Some(GoldilocksExt2 { c0, c1 })
        } else {
            None
        }
    }
    fn from_u64(x: u64) -> Self {
        GoldilocksExt2 { c0: x % GOLDILOCKS_P, c1: 0 }
    }
    fn is_zero(&self) -> bool {
        self.c0 == 0 && self.c1 == 0
    }
    fn inverse(&self) -> Option<Self> {
        if self.is_zero() {
            return None;
        }
        // 1 / (a0 + a1 X) = (a0 - a1 X) / (a0^2 - 7 a1^2)
        let norm = fp_sub(fp_mul(self.c0, self.c0), fp_mul(NON_RESIDUE, fp_mul(self.c1, self.c1)));
        let n = fp_inv(norm);
        Some(GoldilocksExt2 { c0: fp_mul(self.c0, n), c1: fp_mul(fp_neg(self.c1), n) })
    }
}

/// limbs of a slice of elements, `c0, c1` per element, as the ABI takes points and coefficients
pub(crate) fn to_limbs<F: ExtField>(xs: &[F]) -> Vec<u64> {
    let mut out = Vec::with_capacity(2 * xs.len());
    for x in xs {
        let l = x.to_limbs();
        out.push(l[0]);
        out.push(l[1]);
    }
    out
}

/// the inverse; the library only hands out canonical limbs
pub(crate) fn from_limbs<F: ExtField>(w: &[u64]) -> Vec<F> {
    w.chunks_exact(2)
        .map(|p| F::from_limbs(p[0], p[1]).expect("the library returned a non-canonical limb"))
        .collect()
}

#[cfg(test)]
mod tests {
    use super::*;

    #[test]
    fn identities() {
        let a = GoldilocksExt2::new(GOLDILOCKS_P - 1, 12345);
        let b = GoldilocksExt2::new(7, GOLDILOCKS_P - 2);
        assert_eq!(a * a.inverse().unwrap(), GoldilocksExt2::ONE);
        assert_eq!((a + b) - b, a);
        assert_eq!(a * (b + GoldilocksExt2::ONE), a * b + a);
        // X^2 = 7
        let x = GoldilocksExt2::new(0, 1);
        assert_eq!(x * x, GoldilocksExt2::new(7, 0));
        // (p - 1)^2 = 1, 2^96 = -1
        assert_eq!(fp_mul(GOLDILOCKS_P - 1, GOLDILOCKS_P - 1), 1);
        assert_eq!(fp_pow(2, 96), GOLDILOCKS_P - 1);
        assert_eq!(GoldilocksExt2::from_i64(-5).c0, GOLDILOCKS_P - 5);
    }
}
