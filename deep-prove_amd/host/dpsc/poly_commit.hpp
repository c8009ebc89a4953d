// Claims-batching sumcheck of the opening proof: every claim (point, value) on a
// committed polynomial is reduced to one claim per committed chunk at a common
// point.  Mirrors zkml/src/poly_commit/prover.rs:140-255 (prover),
// zkml/src/poly_commit/mod.rs:31-159 (chunking, the expression) and
// zkml/src/poly_commit/verifier.rs:203-340 (verifier).
//
// A polynomial of n variables is held as 2^b chunk tables of m = n - b variables
// (chunk c = the entries whose top b index bits spell c).  For a claim at
// r = (r_1..r_n) the chunks are weighted by C_c = eq(bits(c), r_{m+1..n}) and
// share the eq table of (r_1..r_m).  The sum proven is
//     sum_x sum_claims chal^k * (sum_c C_c P_c(x)) * eq_k(x)
// over max_num_vars variables; shorter tables are read zero-padded, in place.
#pragma once
#include "sumcheck.hpp"

namespace dpsc {
namespace poly_commit {

struct Claim {
    std::vector<F> point;
    F eval;
};

// ChunkedCommitment (zkml/src/poly_commit/mod.rs:31-85); the chunk tables are borrowed
struct CommittedPoly {
    std::vector<const DensePolynomial *> chunks;
    size_t num_chunks() const { return chunks.size(); }
    size_t num_vars_for_chunk() const { return chunks[0]->num_vars(); }
    size_t num_vars() const { return num_vars_for_chunk() + DensePolynomial::log2_strict(chunks.size()); }
};

inline size_t num_batching_vars(size_t num_chunks) { return DensePolynomial::log2_strict(num_chunks); }

// mod.rs:46-58: C_c = identity_eval(r_{m+1..n}, bits_le(c))
inline std::vector<F> batching_coefficients_for_chunks(size_t num_chunks, const std::vector<F> &point)
{
    const size_t b = num_batching_vars(num_chunks);
    if (point.size() < b) throw Error(DPS_ERR_INVALID, "claim point shorter than the chunk index");
    const F *coords = point.data() + (point.size() - b);
    std::vector<F> out;
    for (size_t c = 0; c < num_chunks; c++) {
        std::vector<F> bits(b);
        for (size_t j = 0; j < b; j++) bits[j] = F((c >> j) & 1, 0);
        out.push_back(identity_eval(coords, bits.data(), b));
    }
    return out;
}

// mod.rs:64-68: the coordinates shared by all chunks
inline std::vector<F> eq_point_per_chunk(size_t num_chunks, const std::vector<F> &point)
{
    return std::vector<F>(point.begin(), point.end() - (std::ptrdiff_t)num_batching_vars(num_chunks));
}

struct ChunkedCommittedPolyInfo {
    size_t num_chunks;
    size_t num_claims;
    std::vector<std::vector<F>> batching_coefficients;  // [claim][chunk]
};

// mod.rs:95-159.  WitIn ids: all chunk tables first (in polynomial order), then one eq table per claim.
inline Expression build_sumcheck_expression(const std::vector<ChunkedCommittedPolyInfo> &infos)
{
    size_t eq_offset = 0;
    for (auto &i : infos) eq_offset += i.num_chunks;
    Expression expr = Expression::Constant(F::zero());
    size_t total_num_terms = 0, total_polys = 0;
    for (auto &info : infos) {
        for (size_t i = 0; i < info.batching_coefficients.size(); i++) {
            const auto &coeffs = info.batching_coefficients[i];
            if (coeffs.size() != info.num_chunks) throw Error(DPS_ERR_INVALID, "chunk coefficients do not match the number of chunks");
            Expression chunk_poly = Expression::Constant(F::zero());
            for (size_t c = 0; c < coeffs.size(); c++)
                chunk_poly = chunk_poly + Expression::Constant(coeffs[c]) * Expression::WitIn((uint16_t)(total_polys + c));
            expr = expr + Expression::Challenge(0, total_num_terms + i, F::one(), F::zero()) * chunk_poly *
                              Expression::WitIn((uint16_t)(total_num_terms + i + eq_offset));
        }
        total_num_terms += info.num_claims;
        total_polys += info.num_chunks;
    }
    return expr;
}

struct ClaimsBatchingProof {
    IOPProof sumcheck_proof;
    std::vector<F> sumcheck_evals;  // one per chunk table, at sumcheck_point, of the zero-padded tables
    std::vector<F> sumcheck_point;
};

// prover.rs:140-255.  polys[i] has the claims claims[i]; the caller lists the model
// commitments before the witness ones, as the reference iterates them.
inline ClaimsBatchingProof claims_batching_sumcheck(const Context &ctx, const std::vector<CommittedPoly> &polys,
                                                    const std::vector<std::vector<Claim>> &claims, Transcript &transcript)
{
    if (polys.size() != claims.size() || polys.empty()) throw Error(DPS_ERR_INVALID, "claims_batching_sumcheck: one claim list per polynomial");
    std::vector<std::vector<F>> eq_points;
    std::vector<const DensePolynomial *> committed;
    std::vector<ChunkedCommittedPolyInfo> infos;
    size_t max_num_vars = 0;
    for (size_t p = 0; p < polys.size(); p++) {
        const CommittedPoly &poly = polys[p];
        ChunkedCommittedPolyInfo info{poly.num_chunks(), claims[p].size(), {}};
        for (const Claim &cl : claims[p]) {
            if (cl.point.size() != poly.num_vars()) throw Error(DPS_ERR_INVALID, "claim point does not match the polynomial");
            transcript.append_scalars(&cl.eval, 1);
            eq_points.push_back(eq_point_per_chunk(poly.num_chunks(), cl.point));
            info.batching_coefficients.push_back(batching_coefficients_for_chunks(poly.num_chunks(), cl.point));
        }
        for (auto *c : poly.chunks) committed.push_back(c);
        max_num_vars = std::max(max_num_vars, poly.num_vars_for_chunk());
        infos.push_back(std::move(info));
    }
    // one eq table per claim (prover.rs:176-181), built together
    std::vector<DensePolynomial> eq_polys = DensePolynomial::eq_many(ctx, eq_points);
    Expression expr = build_sumcheck_expression(infos);

    // zero-padded views of every table, chunk tables first, then the eq tables
    std::vector<DensePolynomial> views;
    views.reserve(committed.size() + eq_polys.size());
    for (auto *c : committed) views.push_back(c->zero_pad_num_vars((uint32_t)max_num_vars));
    for (auto &e : eq_polys) views.push_back(e.zero_pad_num_vars((uint32_t)max_num_vars));
    std::vector<const DensePolynomial *> refs;
    for (auto &v : views) refs.push_back(&v);

    const F challenge = transcript.append_and_sample("model_batching");
    auto builder = VirtualPolynomialsBuilder::new_with_mles(optimal_sumcheck_threads(max_num_vars), max_num_vars, refs);
    auto vp = builder.to_virtual_polys({expr}, {challenge});
    auto res = IOPProverState::prove(vp, transcript);
    ClaimsBatchingProof out;
    out.sumcheck_proof = std::move(res.first);
    const auto &all = res.second.get_mle_flatten_final_evaluations();
    out.sumcheck_evals.assign(all.begin(), all.begin() + (std::ptrdiff_t)committed.size());
    out.sumcheck_point = res.second.collect_raw_challenges();
    return out;
}

// What the verifier knows of a committed polynomial
struct CommitmentShape {
    size_t num_chunks;
    size_t num_vars;  // of the whole polynomial
    size_t num_vars_for_chunk() const { return num_vars - num_batching_vars(num_chunks); }
};

// verifier.rs:203-340.  Returns the common opening point; throws when the proof does not verify.
inline std::vector<F> claims_batching_verify(const std::vector<CommitmentShape> &shapes, const std::vector<std::vector<Claim>> &claims,
                                             const IOPProof &proof, const std::vector<F> &sumcheck_evals, Transcript &transcript)
{
    if (shapes.size() != claims.size()) throw Error(DPS_ERR_INVALID, "claims_batching_verify: one claim list per polynomial");
    std::vector<std::vector<F>> eq_points;
    std::vector<F> evals;
    std::vector<ChunkedCommittedPolyInfo> infos;
    size_t max_num_vars = 0, total_chunks = 0;
    for (size_t p = 0; p < shapes.size(); p++) {
        ChunkedCommittedPolyInfo info{shapes[p].num_chunks, claims[p].size(), {}};
        for (const Claim &cl : claims[p]) {
            if (cl.point.size() != shapes[p].num_vars) throw Error(DPS_ERR_INVALID, "claim point does not match the polynomial");
            transcript.append_scalars(&cl.eval, 1);
            eq_points.push_back(eq_point_per_chunk(shapes[p].num_chunks, cl.point));
            evals.push_back(cl.eval);
            info.batching_coefficients.push_back(batching_coefficients_for_chunks(shapes[p].num_chunks, cl.point));
        }
        max_num_vars = std::max(max_num_vars, shapes[p].num_vars_for_chunk());
        total_chunks += shapes[p].num_chunks;
        infos.push_back(std::move(info));
    }
    if (sumcheck_evals.size() != total_chunks) throw Error(DPS_ERR_INVALID, "claims_batching_verify: one evaluation per chunk expected");
    Expression expr = build_sumcheck_expression(infos);
    const F challenge = transcript.append_and_sample("model_batching");
    F claimed_sum = F::zero(), chal_acc = F::one();
    for (auto &e : evals) {
        claimed_sum = claimed_sum + chal_acc * e;
        chal_acc = chal_acc * challenge;
    }
    VPAuxInfo aux;
    aux.max_degree = 2;
    aux.max_num_variables = max_num_vars;
    SubClaim sub = IOPVerifierState::verify(claimed_sum, proof, aux, transcript);
    std::vector<F> witness_evals = sumcheck_evals;
    for (auto &ep : eq_points) {
        // the eq table was zero-padded: its evaluation picks up (1 - r) for every added variable
        F v = identity_eval(sub.point.data(), ep.data(), ep.size());
        for (size_t k = ep.size(); k < sub.point.size(); k++) v = v * (F::one() - sub.point[k]);
        witness_evals.push_back(v);
    }
    if (expr.evaluate(witness_evals, {challenge}) != sub.expected_evaluation)
        throw Error(DPS_ERR_INVALID, "claims batching: the evaluations do not match the sumcheck's final claim");
    return sub.point;
}

}  // namespace poly_commit
}  // namespace dpsc
