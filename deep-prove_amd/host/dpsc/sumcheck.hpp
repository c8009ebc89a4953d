// The sumcheck prover API as the reference's layer provers call it
// (zkml/src/layers/hadamard.rs:107-129, zkml/src/layers/einsum/prove.rs:164-189,
// zkml/src/iop/same_poly.rs:93-112, zkml/src/lookup/logup_gkr/prover.rs:263-281):
//
//     VirtualPolynomialsBuilder b(num_threads, num_vars);
//     Expression e = b.lift(poly) * ...;
//     auto vp = b.to_virtual_polys({e}, challenges);
//     auto [proof, state] = IOPProverState::prove(vp, transcript);
//     state.get_mle_flatten_final_evaluations(); state.collect_raw_challenges();
//
// The tables stay on the GPU; per round only the d+1 evaluations come back and
// the transcript, which lives here on the host, returns the challenge.
#pragma once
#include <utility>

#include "expression.hpp"
#include "poly.hpp"
#include "transcript.hpp"

namespace dpsc {

struct IOPProverMessage {
    std::vector<F> evaluations;  // p(0), ..., p(d)
};

struct IOPProof {
    std::vector<IOPProverMessage> proofs;
    // IOPProof::extract_sum (zkml/src/layers/hadamard.rs:117-121)
    F extract_sum() const { return proofs.empty() ? F::zero() : proofs[0].evaluations[0] + proofs[0].evaluations[1]; }
};

struct VPAuxInfo {
    size_t max_degree = 0;
    size_t max_num_variables = 0;
};

// zkml/src/util.rs:6-28
inline VPAuxInfo from_mle_list_dimensions(const std::vector<std::vector<size_t>> &product_list)
{
    VPAuxInfo aux;
    for (auto &p : product_list) {
        aux.max_degree = std::max(aux.max_degree, p.size());
        for (auto v : p) aux.max_num_variables = std::max(aux.max_num_variables, v);
    }
    return aux;
}

// the engine splits the hypercube over GPU workgroups by itself; the argument
// only exists so that call sites read like the reference's
inline size_t optimal_sumcheck_threads(size_t) { return 1; }

class VirtualPolynomials {
public:
    const Context *ctx = nullptr;
    uint32_t num_vars = 0;
    std::vector<const dps_mle *> mles;
    std::vector<dps_term> terms;
    uint32_t degree = 0;
};

class VirtualPolynomialsBuilder {
public:
    VirtualPolynomialsBuilder(size_t /*num_threads*/, size_t num_vars) : num_vars_((uint32_t)num_vars) {}
    // new_with_mles: tables registered up front, WitIn(i) is the i-th of them
    static VirtualPolynomialsBuilder new_with_mles(size_t num_threads, size_t num_vars, const std::vector<const DensePolynomial *> &mles)
    {
        VirtualPolynomialsBuilder b(num_threads, num_vars);
        b.mles_ = mles;
        return b;
    }
    // registers a (borrowed) table and returns its WitIn
    Expression lift(const DensePolynomial &p)
    {
        mles_.push_back(&p);
        return Expression::WitIn((uint16_t)(mles_.size() - 1));
    }
    VirtualPolynomials to_virtual_polys(const std::vector<Expression> &exprs, const std::vector<F> &challenges) const
    {
        if (mles_.empty()) throw Error(DPS_ERR_INVALID, "to_virtual_polys: no tables registered");
        VirtualPolynomials vp;
        vp.ctx = &mles_[0]->context();
        vp.num_vars = num_vars_;
        for (auto *p : mles_) vp.mles.push_back(p->raw());
        for (auto &e : exprs) {
            for (auto &m : e.to_monomials(challenges)) {
                if (m.wits.size() > DPS_MAX_FACTORS) throw Error(DPS_ERR_UNSUPPORTED, "to_virtual_polys: too many factors in a product");
                dps_term t;
                memset(&t, 0, sizeof t);
                t.coeff[0] = m.coeff.c0;
                t.coeff[1] = m.coeff.c1;
                t.n_factors = (uint32_t)m.wits.size();
                for (size_t i = 0; i < m.wits.size(); i++) t.factors[i] = m.wits[i];
                vp.degree = std::max<uint32_t>(vp.degree, t.n_factors);
                vp.terms.push_back(t);
            }
        }
        return vp;
    }

private:
    uint32_t num_vars_;
    std::vector<const DensePolynomial *> mles_;
};

class IOPProverState {
public:
    // What prove() absorbs: the number of variables and the degree, then per round
    // the d+1 evaluations; the challenge of a round is squeezed right after its
    // message.  Runs the whole protocol; the returned state holds the challenges
    // and the final evaluation of every registered table.
    // `claimed_sum`: the value of the whole sum when the caller knows it (the reference's callers put it on the transcript
    // before this call); round 1 then need not evaluate the polynomial at 1.
    static std::pair<IOPProof, IOPProverState> prove(const VirtualPolynomials &vp, Transcript &transcript, const F *claimed_sum = nullptr)
    {
        const Context &ctx = *vp.ctx;
        const std::vector<const dps_mle *> &handles = vp.mles;
        dps_sc *sc = nullptr;
        ctx.check(dps_sc_begin(ctx.raw(), vp.num_vars, handles.data(), (uint32_t)handles.size(), vp.terms.data(),
                               (uint32_t)vp.terms.size(), &sc),
                  "dps_sc_begin");
        std::unique_ptr<dps_sc, int32_t (*)(dps_sc *)> guard(sc, &dps_sc_free);
        if (claimed_sum) {
            const uint64_t limbs[2] = {claimed_sum->c0, claimed_sum->c1};
            ctx.check(dps_sc_set_claim(sc, limbs), "dps_sc_set_claim");
        }
        uint32_t degree = 0;
        dps_sc_degree(sc, &degree);
        transcript.append_u64(vp.num_vars);
        transcript.append_u64(degree);
        const size_t npts = degree + 1;
        std::vector<uint64_t> proof(2 * npts * vp.num_vars), point(2 * (size_t)vp.num_vars), finals(2 * handles.size());
        ctx.check(dps_sc_prove(sc, &round_cb, &transcript, proof.data(), point.data(), finals.data()), "dps_sc_prove");
        IOPProof out;
        for (uint32_t j = 0; j < vp.num_vars; j++) out.proofs.push_back(IOPProverMessage{from_limbs(proof.data() + 2 * npts * j, npts)});
        IOPProverState st;
        st.challenges_ = from_limbs(point.data(), vp.num_vars);
        st.final_evals_ = from_limbs(finals.data(), handles.size());
        return {std::move(out), std::move(st)};
    }
    // one element per registered table, in registration order (einsum/prove.rs:188)
    const std::vector<F> &get_mle_flatten_final_evaluations() const { return final_evals_; }
    // challenges in round order = little-endian point of the final claims (einsum/prove.rs:189)
    const std::vector<F> &collect_raw_challenges() const { return challenges_; }

    // transcript hook handed to dps_sc_prove; `user` is a Transcript*
    static int32_t round_cb(void *user, uint32_t /*round*/, const uint64_t *evals, uint32_t n_evals, uint64_t *challenge_out)
    {
        Transcript *t = static_cast<Transcript *>(user);
        F msg[DPS_MAX_FACTORS + 1];
        for (uint32_t i = 0; i < n_evals; i++) msg[i] = F(evals[2 * i], evals[2 * i + 1]);
        t->append_scalars(msg, n_evals);
        F r = t->challenge_scalar();
        challenge_out[0] = r.c0;
        challenge_out[1] = r.c1;
        return 0;
    }

private:
    std::vector<F> challenges_, final_evals_;
};

struct SubClaim {
    std::vector<F> point;
    F expected_evaluation;
};

class IOPVerifierState {
public:
    // zkml/src/layers/einsum/verify.rs:159-165.  Throws when a round message does
    // not sum to the running claim.
    static SubClaim verify(const F &claimed_sum, const IOPProof &proof, const VPAuxInfo &aux, Transcript &transcript)
    {
        if (proof.proofs.size() != aux.max_num_variables) throw Error(DPS_ERR_INVALID, "sumcheck verify: wrong number of rounds");
        transcript.append_u64(aux.max_num_variables);
        transcript.append_u64(aux.max_degree);
        SubClaim sub;
        F claim = claimed_sum;
        for (size_t j = 0; j < proof.proofs.size(); j++) {
            const auto &ev = proof.proofs[j].evaluations;
            if (ev.size() != aux.max_degree + 1) throw Error(DPS_ERR_INVALID, "sumcheck verify: wrong message length");
            if (ev[0] + ev[1] != claim) throw Error(DPS_ERR_INVALID, "sumcheck verify: round " + std::to_string(j + 1) + " does not match the claim");
            transcript.append_scalars(ev);
            F r = transcript.challenge_scalar();
            sub.point.push_back(r);
            claim = interpolate_uni(ev.data(), aux.max_degree, r);
        }
        sub.expected_evaluation = claim;
        return sub;
    }
};

}  // namespace dpsc
