// Merging several claims (r_i, y_i) on one polynomial into a single claim:
// zkml/src/iop/same_poly.rs:56-169.  With challenges a_i the sum
//     sum_x f(x) * sum_i a_i eq(r_i, x) = sum_i a_i y_i
// is proven by sumcheck; the claim f(point) = eval at the sumcheck's point is
// what the caller carries on.
#pragma once
#include "sumcheck.hpp"

namespace dpsc {
namespace same_poly {

struct Claim {
    std::vector<F> point;
    F eval;
};

// same_poly.rs:31-43
struct Context {
    VPAuxInfo vp_info;
    explicit Context(size_t num_vars) : vp_info(from_mle_list_dimensions({{num_vars, num_vars}})) {}
};

struct Proof {
    IOPProof sumcheck;
    F eval;
};

class Prover {
public:
    // the polynomial is borrowed
    explicit Prover(const DensePolynomial &poly) : poly_(&poly) {}
    void add_claim(const Claim &claim)
    {
        if (claim.point.size() != poly_->num_vars()) throw Error(DPS_ERR_INVALID, "same_poly: claim point length does not match the polynomial");
        claims_.push_back(claim);
    }
    // same_poly.rs:84-114
    std::pair<Proof, Claim> prove(Transcript &t) const
    {
        const std::vector<F> challenges = t.read_challenges(claims_.size());
        std::vector<std::vector<F>> points;
        for (auto &c : claims_) points.push_back(c.point);
        std::vector<DensePolynomial> beta_evals = DensePolynomial::eq_many(poly_->context(), points);
        const size_t num_vars = poly_->num_vars();
        VirtualPolynomialsBuilder builder(optimal_sumcheck_threads(num_vars), num_vars);
        Expression poly_expr = builder.lift(*poly_);
        Expression sum_expr = Expression::Constant(F::zero());
        for (size_t i = 0; i < beta_evals.size(); i++)
            sum_expr = sum_expr + Expression::Challenge((uint16_t)i, 1, F::one(), F::zero()) * builder.lift(beta_evals[i]);
        auto vp = builder.to_virtual_polys({poly_expr * sum_expr}, challenges);
        // the sum the proof is about: sum_i challenge_i * claim_i (same_poly.rs:226-227)
        F claimed = F::zero();
        for (size_t i = 0; i < claims_.size(); i++) claimed += challenges[i] * claims_[i].eval;
        auto res = IOPProverState::prove(vp, t, &claimed);
        const F eval = res.second.get_mle_flatten_final_evaluations()[0];
        return {Proof{std::move(res.first), eval}, Claim{res.second.collect_raw_challenges(), eval}};
    }

private:
    const DensePolynomial *poly_;
    std::vector<Claim> claims_;
};

class Verifier {
public:
    explicit Verifier(const Context &ctx) : ctx_(&ctx) {}
    void add_claim(const Claim &claim)
    {
        if (claim.point.size() != ctx_->vp_info.max_num_variables) throw Error(DPS_ERR_INVALID, "same_poly: claim point length does not match the context");
        claims_.push_back(claim);
    }
    // same_poly.rs:140-169; throws when the proof does not verify
    Claim verify(const Proof &proof, Transcript &t) const
    {
        const std::vector<F> a = t.read_challenges(claims_.size());
        F y_res = F::zero();
        for (size_t i = 0; i < claims_.size(); i++) y_res = y_res + claims_[i].eval * a[i];
        SubClaim sub = IOPVerifierState::verify(y_res, proof.sumcheck, ctx_->vp_info, t);
        F computed = F::zero();
        for (size_t i = 0; i < claims_.size(); i++)
            computed = computed + a[i] * identity_eval(claims_[i].point.data(), sub.point.data(), std::min(claims_[i].point.size(), sub.point.size()));
        if (proof.eval * computed != sub.expected_evaluation) throw Error(DPS_ERR_INVALID, "same_poly: the evaluation does not match the sumcheck's final claim");
        return Claim{sub.point, proof.eval};
    }

private:
    const Context *ctx_;
    std::vector<Claim> claims_;
};

}  // namespace same_poly
}  // namespace dpsc
