//! `IOPVerifierState::verify` (`zkml/src/layers/einsum/verify.rs:159-165`): host only, no GPU work.
//! Checks `p_1(0) + p_1(1) = claim`, `p_{j+1}(0) + p_{j+1}(1) = p_j(r_j)`, and returns the point and
//! the value the caller must find the expression to have there.

use crate::error::{Error, Result};
use crate::field::ExtField;
use crate::prover::IOPProof;
use crate::transcript::Transcript;

#[derive(Clone, Copy, Debug, Default, PartialEq, Eq)]
pub struct VPAuxInfo {
    pub max_degree: usize,
    pub max_num_variables: usize,
}

impl VPAuxInfo {
    /// `VPAuxInfo::from_mle_list_dimensions` (`zkml/src/util.rs:6-28`): one list of variable counts per product
    pub fn from_mle_list_dimensions(product_list: &[Vec<usize>]) -> Self {
        let mut aux = VPAuxInfo::default();
        for p in product_list {
            aux.max_degree = aux.max_degree.max(p.len());
            for v in p {
                aux.max_num_variables = aux.max_num_variables.max(*v);
            }
        }
        aux
    }
}

#[derive(Clone, Debug, PartialEq)]
pub struct SubClaim<F: ExtField> {
    pub point: Vec<F>,
    pub expected_evaluation: F,
}

/// the polynomial of degree `evals.len() - 1` through `(i, evals[i])`, at `x`
pub fn interpolate_uni<F: ExtField>(evals: &[F], x: F) -> F {
    let d = evals.len();
    let mut acc = F::ZERO;
    for k in 0..d {
        let mut num = F::ONE;
        let mut den = F::ONE;
        for m in 0..d {
            if m != k {
                num *= x - F::from_u64(m as u64);
                den *= F::from_u64(k as u64) - F::from_u64(m as u64);
            }
        }
        acc += evals[k] * num * den.inverse().expect("distinct nodes");
    }
    acc
}

pub struct IOPVerifierState;

impl IOPVerifierState {
    pub fn verify<F: ExtField, T: Transcript<F>>(
        claimed_sum: F,
        proof: &IOPProof<F>,
        aux: &VPAuxInfo,
        transcript: &mut T,
    ) -> Result<SubClaim<F>> {
        if proof.proofs.len() != aux.max_num_variables {
            return Err(Error::invalid("sumcheck verify: wrong number of rounds"));
        }
        transcript.append_u64(aux.max_num_variables as u64);
        transcript.append_u64(aux.max_degree as u64);
        let mut claim = claimed_sum;
        let mut point = Vec::with_capacity(proof.proofs.len());
        for (j, msg) in proof.proofs.iter().enumerate() {
            let ev = &msg.evaluations;
            if ev.len() != aux.max_degree + 1 {
                return Err(Error::invalid("sumcheck verify: wrong message length"));
            }
            if ev[0] + ev[1] != claim {
                return Err(Error::invalid(format!("sumcheck verify: round {} does not match the claim", j + 1)));
            }
            transcript.append_scalars(ev);
            let r = transcript.challenge_scalar();
            point.push(r);
            claim = interpolate_uni(ev, r);
        }
        Ok(SubClaim { point, expected_evaluation: claim })
    }
}

#[cfg(test)]
mod tests {
    use super::*;
    use crate::field::GoldilocksExt2 as F;

    #[test]
    fn interpolation_reproduces_a_cubic() {
        // p(x) = 2 x^3 + x + 5 at 0..3, then at 10
        let p = |x: u64| F::from_u64(2 * x * x * x + x + 5);
        let evals: Vec<F> = (0..4).map(p).collect();
        assert_eq!(interpolate_uni(&evals, F::from_u64(10)), p(10));
    }
}
