//! The symbolic sum-of-products the provers build (`Expression::{WitIn, Constant, Challenge}` with
//! `+ - *`): `zkml/src/layers/einsum/op_info.rs:137-199`, `zkml/src/lookup/logup_gkr/circuit.rs:245-284`,
//! `zkml/src/iop/same_poly.rs:94-104`.  `Challenge(id, pow, scalar, offset)` evaluates to
//! `scalar * challenges[id]^pow + offset`.  At `to_virtual_polys` the expression is flattened to
//! monomials `coeff * product of tables`, which is what crosses the ABI (`dps_term`).

use std::collections::BTreeMap;
use std::ops::{Add, Mul, Neg, Sub};
use std::rc::Rc;

use crate::field::ExtField;

#[derive(Clone, Debug)]
pub enum Expression<F: ExtField> {
    WitIn(u16),
    Constant(F),
    Challenge(u16, usize, F, F),
    Sum(Rc<Expression<F>>, Rc<Expression<F>>),
    Product(Rc<Expression<F>>, Rc<Expression<F>>),
    Neg(Rc<Expression<F>>),
}

/// `coeff * prod tables[wits[i]]`, the table indices sorted, repeats allowed
#[derive(Clone, Debug, PartialEq)]
pub struct Monomial<F: ExtField> {
    pub coeff: F,
    pub wits: Vec<u16>,
}

impl<F: ExtField> Expression<F> {
    pub const ZERO: Expression<F> = Expression::Constant(F::ZERO);
    pub const ONE: Expression<F> = Expression::Constant(F::ONE);

    fn challenge_value(id: u16, pow: usize, scalar: F, offset: F, challenges: &[F]) -> F {
        let c = *challenges.get(id as usize).expect("Expression: challenge index out of range");
        scalar * c.pow(pow as u64) + offset
    }

    /// Flattens to monomials with the challenges substituted.  Equal products of tables are merged;
    /// monomials whose coefficient cancels to zero are dropped.
    pub fn to_monomials(&self, challenges: &[F]) -> Vec<Monomial<F>> {
        let mut raw = Vec::new();
        self.expand_into(F::ONE, challenges, &mut raw);
        let mut acc: BTreeMap<Vec<u16>, F> = BTreeMap::new();
        for m in raw {
            let e = acc.entry(m.wits).or_insert(F::ZERO);
            *e += m.coeff;
        }
        acc.into_iter().filter(|(_, c)| !c.is_zero()).map(|(wits, coeff)| Monomial { coeff, wits }).collect()
    }

    // appends scale * (this expression's monomials): a long sum costs one pass
    fn expand_into(&self, scale: F, ch: &[F], out: &mut Vec<Monomial<F>>) {
        if scale.is_zero() {
            return;
        }
        match self {
            Expression::WitIn(id) => out.push(Monomial { coeff: scale, wits: vec![*id] }),
            Expression::Constant(c) => {
                if !c.is_zero() {
                    out.push(Monomial { coeff: scale * *c, wits: Vec::new() });
                }
            }
            Expression::Challenge(id, pow, scalar, offset) => {
                let c = Self::challenge_value(*id, *pow, *scalar, *offset, ch);
                if !c.is_zero() {
                    out.push(Monomial { coeff: scale * c, wits: Vec::new() });
                }
            }
            Expression::Neg(a) => a.expand_into(-scale, ch, out),
            Expression::Sum(a, b) => {
                a.expand_into(scale, ch, out);
                b.expand_into(scale, ch, out);
            }
            Expression::Product(a, b) => {
                let mut v = Vec::new();
                let mut w = Vec::new();
                a.expand_into(F::ONE, ch, &mut v);
                b.expand_into(scale, ch, &mut w);
                out.reserve(v.len() * w.len());
                for x in &v {
                    for y in &w {
                        let coeff = x.coeff * y.coeff;
                        if coeff.is_zero() {
                            continue;
                        }
                        let mut wits = x.wits.clone();
                        wits.extend_from_slice(&y.wits);
                        wits.sort_unstable();
                        out.push(Monomial { coeff, wits });
                    }
                }
            }
        }
    }

    /// `eval_by_expr_with_instance` restricted to what the callers pass: witness evaluations and
    /// challenges (`zkml/src/lookup/logup_gkr/prover.rs:43-58`).
    pub fn evaluate(&self, wit_evals: &[F], challenges: &[F]) -> F {
        match self {
            Expression::WitIn(id) => *wit_evals.get(*id as usize).expect("Expression: witness index out of range"),
            Expression::Constant(c) => *c,
            Expression::Challenge(id, pow, scalar, offset) => Self::challenge_value(*id, *pow, *scalar, *offset, challenges),
            Expression::Neg(a) => -a.evaluate(wit_evals, challenges),
            Expression::Sum(a, b) => a.evaluate(wit_evals, challenges) + b.evaluate(wit_evals, challenges),
            Expression::Product(a, b) => a.evaluate(wit_evals, challenges) * b.evaluate(wit_evals, challenges),
        }
    }

    /// the largest number of tables in a product
    pub fn degree(&self) -> usize {
        match self {
            Expression::WitIn(_) => 1,
            Expression::Constant(_) | Expression::Challenge(..) => 0,
            Expression::Neg(a) => a.degree(),
            Expression::Sum(a, b) => a.degree().max(b.degree()),
            Expression::Product(a, b) => a.degree() + b.degree(),
        }
    }
}

impl<F: ExtField> Add for Expression<F> {
    type Output = Expression<F>;
    fn add(self, o: Self) -> Self {
        Expression::Sum(Rc::new(self), Rc::new(o))
    }
}
impl<F: ExtField> Mul for Expression<F> {
    type Output = Expression<F>;
    fn mul(self, o: Self) -> Self {
        Expression::Product(Rc::new(self), Rc::new(o))
    }
}
impl<F: ExtField> Neg for Expression<F> {
    type Output = Expression<F>;
    fn neg(self) -> Self {
        Expression::Neg(Rc::new(self))
    }
}
impl<F: ExtField> Sub for Expression<F> {
    type Output = Expression<F>;
    fn sub(self, o: Self) -> Self {
        self + (-o)
    }
}

#[cfg(test)]
mod tests {
    use super::*;
    use crate::field::GoldilocksExt2 as F;

    #[test]
    fn flattening_merges_and_cancels() {
        let w = |i| Expression::<F>::WitIn(i);
        // (w0 + w1) * w2 - w1 * w2 + 3 = w0 w2 + 3
        let e = (w(0) + w(1)) * w(2) - w(1) * w(2) + Expression::Constant(F::new(3, 0));
        let m = e.to_monomials(&[]);
        assert_eq!(m.len(), 2);
        assert_eq!(m[0], Monomial { coeff: F::new(3, 0), wits: vec![] });
        assert_eq!(m[1], Monomial { coeff: F::ONE, wits: vec![0, 2] });
        assert_eq!(e.degree(), 2);
        // Challenge(id, pow, scalar, offset) = scalar * ch^pow + offset
        let c = Expression::<F>::Challenge(0, 2, F::new(5, 0), F::new(1, 0));
        assert_eq!(c.evaluate(&[], &[F::new(3, 0)]), F::new(46, 0));
    }
}
