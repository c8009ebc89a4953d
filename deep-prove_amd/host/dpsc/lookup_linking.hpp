// The sumcheck that links a lookup argument to the inputs and outputs of its layer:
// zkml/src/lookup/operation/inputs/proving.rs:26-114 (prover),
// zkml/src/lookup/operation/inputs/verifying.rs:236-330 (verifier),
// zkml/src/lookup/operation/variant.rs:55-379 (the expression of every variant),
// zkml/src/lookup/operation/variant/proving.rs:226-253 (eq tables),
// zkml/src/shape.rs:565-610 (eq point and per-chunk coefficients).
//
// A layer's tensor is cut into 2-D chunks (its last two dimensions); every chunk brings the
// tables of its value chunks and zeroing chunks, plus per-variant extras.  One sumcheck over the
// chunk's variables proves, with the claim point's leading-dimension eq values as per-chunk
// coefficients, that (a) the chunk outputs rebuilt from the looked-up pieces evaluate to the
// layer's output claim and (b) a random linear combination of the pieces evaluates, at the
// LogUp point, to what the LogUp proof claimed.  What the tables and the lookup table's
// constants are is the caller's business: this file takes the numbers the expression needs.
#pragma once
#include "sumcheck.hpp"

namespace dpsc {
namespace lookup {

enum class Variant { Standard, GLU, Softmax, Normalisation };
enum class TableSign { Positive, Negative };

// what the expression reads from ChunkingInfo and its Table (decomposer.rs:13-41)
struct ChunkingInfo {
    uint32_t number_of_value_chunks = 1;
    uint32_t number_of_zeroing_chunks = 0;
    uint32_t table_bit_size = 8;
    bool table_is_signed = true;
    int64_t min_output_value = 0, max_output_value = 0;
    TableSign input_sign = TableSign::Positive;  // unsigned tables only
};

// LookupVariant (variant.rs:19-43) without the numeric bounds, which only the range-check witnesses use
struct LookupVariant {
    Variant kind = Variant::Standard;
    bool normalised_sum = false;  // Normalisation: the mean is enforced as well
    bool has_weight = false;      // Normalisation: element-wise weight after normalising
    size_t additional_witnesses_per_chunk() const { return kind == Variant::GLU ? 1 : kind == Variant::Normalisation ? 2 : 0; }
    bool requires_normalisation() const { return kind == Variant::Softmax || kind == Variant::Normalisation; }
    // squeeze_sumcheck_challenges (variant.rs:363-379)
    std::vector<F> squeeze_sumcheck_challenges(Transcript &t) const
    {
        std::vector<F> out;
        if (requires_normalisation()) out.push_back(t.append_and_sample("normalisation"));
        if (kind == Variant::Normalisation) out.push_back(t.append_and_sample("input"));
        return out;
    }
};

struct LookupSumcheckProof {
    IOPProof sumcheck_proof;
    std::vector<F> evaluations;  // of the witness tables at the sumcheck point
    std::vector<F> sumcheck_point;
    bool has_weight_eval = false;
    F weight_eval;
};

class LookupInputConfig {
public:
    LookupInputConfig(const ChunkingInfo &ci, const LookupVariant &v, const std::vector<uint64_t> &unpadded_input_shape)
        : ci_(ci), variant_(v), shape_(unpadded_input_shape)
    {
        if (shape_.empty()) throw Error(DPS_ERR_INVALID, "LookupInputConfig: empty shape");
        for (auto d : shape_)
            if (d == 0) throw Error(DPS_ERR_INVALID, "LookupInputConfig: zero-sized dimension");
        if (ci_.number_of_value_chunks == 0) throw Error(DPS_ERR_INVALID, "LookupInputConfig: no value chunk");
    }
    size_t number_of_chunks() const
    {
        size_t n = 1;
        for (size_t i = 0; i + 2 < shape_.size(); i++) n *= shape_[i];
        return n;
    }
    size_t witnesses() const
    {
        return number_of_chunks() * (ci_.number_of_value_chunks + ci_.number_of_zeroing_chunks + variant_.additional_witnesses_per_chunk());
    }
    size_t num_vars() const
    {
        size_t v = 0;
        for (size_t i = shape_.size() >= 2 ? shape_.size() - 2 : 0; i < shape_.size(); i++) v += ceil_log2(shape_[i]);
        return v;
    }

    // Shape::compute_eq_point_and_batching_challenges: (eq point, one coefficient per chunk)
    std::pair<std::vector<F>, std::vector<F>> eq_point_and_batching_challenges(const std::vector<F> &point) const
    {
        size_t total = 0;
        for (auto d : shape_) total += ceil_log2(d);
        if (point.size() != total) throw Error(DPS_ERR_INVALID, "linking sumcheck: claim point length does not match the shape");
        // the last dimension takes the lowest variables
        std::vector<std::vector<F>> dim_points(shape_.size());
        size_t start = 0;
        for (size_t a = shape_.size(); a-- > 0;) {
            size_t l = ceil_log2(shape_[a]);
            dim_points[a].assign(point.begin() + start, point.begin() + start + l);
            start += l;
        }
        const size_t skip = shape_.size() >= 2 ? shape_.size() - 2 : 0;
        std::vector<F> eq_point, bc{F::one()};
        for (size_t i = 0; i < shape_.size(); i++) {
            if (i < skip) {
                auto ev = eq_evals_host(dim_points[i].data(), dim_points[i].size());
                std::vector<F> next;
                next.reserve(bc.size() * shape_[i]);
                for (auto &c : bc)
                    for (uint64_t k = 0; k < shape_[i]; k++) next.push_back(c * ev[k]);
                bc.swap(next);
            } else {
                eq_point.insert(eq_point.begin(), dim_points[i].begin(), dim_points[i].end());
            }
        }
        return {eq_point, bc};
    }

    // build_eq_polys' points: output, LogUp and (normalising variants) the LogUp point with its
    // final-dimension coordinates replaced by 1/2, which averages over that dimension
    std::vector<std::vector<F>> eq_points(const std::vector<F> &output_eq_point, const std::vector<F> &logup_point) const
    {
        std::vector<std::vector<F>> pts{output_eq_point, logup_point};
        if (variant_.requires_normalisation()) {
            const size_t fd = ceil_log2(shape_.back());
            if (logup_point.size() < fd) throw Error(DPS_ERR_INVALID, "linking sumcheck: LogUp point shorter than the final dimension");
            std::vector<F> np(fd, F::from_u64(2).inverse());
            np.insert(np.end(), logup_point.begin() + fd, logup_point.end());
            pts.push_back(std::move(np));
        }
        return pts;
    }

    // build_full_sumcheck_expression: challenge 0 is the sum challenge, 1 + c the coefficient of
    // chunk c, then the normalisation and input challenges.  WitIn order: per chunk its value and
    // zeroing chunks; the per-variant extras; the eq tables; the weight.
    Expression build_full_sumcheck_expression() const
    {
        using E = Expression;
        const size_t chunks = number_of_chunks();
        const uint32_t nvc = ci_.number_of_value_chunks, nz = ci_.number_of_zeroing_chunks, bits = ci_.table_bit_size;
        const size_t per_chunk = nvc + nz, total_out = chunks * per_chunk;
        const size_t total_wit = total_out + chunks * variant_.additional_witnesses_per_chunk();
        auto W = [](size_t i) { return E::WitIn((uint16_t)i); };
        auto K = [](int64_t x) { return E::Constant(F::from_i64(x)); };
        auto S = [](size_t pow) { return E::Challenge(0, pow, F::one(), F::zero()); };
        const E out_eq = W(total_wit), logup_eq = W(total_wit + 1), norm_eq = W(total_wit + 2);
        const F pow_two = F::from_i64((int64_t)1 << ceil_log2(shape_.back()));
        if (nvc * bits > 62) throw Error(DPS_ERR_UNSUPPORTED, "linking sumcheck: value wider than 62 bits");
        E full = E::ZERO();
        for (size_t c = 0; c < chunks; c++) {
            const size_t off = c * per_chunk;
            // ValueExpression::new
            E value = E::ZERO(), sum = E::ZERO();
            size_t wo, sco;
            if (nvc == 1) {
                value = W(off);
                sum = W(off) * S(1);
                wo = off + 1;
                sco = 2;
            } else {
                value = K(-((int64_t)1 << (nvc * bits - 1)));
                for (uint32_t i = 0; i < nvc; i++) {
                    value = value + K((int64_t)1 << (bits * i)) * (W(off + i) + K((int64_t)1 << (bits - 1)));
                    sum = sum + W(off + i) * S(i + 1);
                }
                wo = off + nvc;
                sco = 1 + nvc;
            }
            // build_lookup_output_expressions
            E prod = E::ONE(), clamp = E::ZERO(), sq_clamp = E::ZERO();
            if (ci_.table_is_signed) {
                for (uint32_t i = 0; i + 1 < nz; i++) {
                    prod = prod * W(wo + i);
                    sum = sum + W(wo + i) * S(sco + i);
                }
                if (nz) {
                    int64_t cmin = ci_.min_output_value, cmax = ci_.max_output_value;
                    if (nvc != 1) {
                        cmin = -((int64_t)1 << (nvc * bits - 1));
                        cmax = ((int64_t)1 << (nvc * bits - 1)) - 1;
                    }
                    // the top zeroing chunk is -1, 0 or 1: 0 keeps the value, +-1 selects the clamp
                    const E top = W(wo + nz - 1), lower = prod;
                    const E keep = E::ONE() - top * top;
                    prod = prod * keep;
                    sum = sum + top * S(sco + nz - 1);
                    const E half = E::Constant(F::from_u64(2).inverse());
                    const E hi = top * (top + E::ONE()) * half + (keep - lower * keep);
                    const E lo = top * (top - E::ONE()) * half;
                    clamp = hi * K(cmax) + lo * K(cmin);
                    if (variant_.kind == Variant::Normalisation) sq_clamp = hi * K(cmax) * K(cmax) + lo * K(cmin) * K(cmin);
                }
            } else {
                for (uint32_t i = 0; i < nz; i++) {
                    prod = prod * W(wo + i);
                    sum = sum + W(wo + i) * S(sco + i);
                }
                // with no zeroing chunk the reference's clamping term is the constant one (variant.rs:200-203)
                clamp = nz ? K(ci_.input_sign == TableSign::Positive ? ci_.max_output_value : ci_.min_output_value) : E::ONE();
            }
            const E prod_expr = clamp + prod * value;
            const E chunk_ch = E::Challenge((uint16_t)(1 + c), 1, F::one(), F::zero());
            const uint16_t norm_id = (uint16_t)(1 + chunks), input_id = (uint16_t)(2 + chunks);
            E inner = E::ZERO();
            switch (variant_.kind) {
            case Variant::Standard: inner = out_eq * prod_expr + logup_eq * sum; break;
            case Variant::GLU: inner = out_eq * prod_expr * W(total_out + c) + logup_eq * sum; break;
            case Variant::Softmax:
                inner = out_eq * prod_expr + E::Challenge(norm_id, 1, pow_two, F::zero()) * (norm_eq * prod_expr) + logup_eq * sum;
                break;
            case Variant::Normalisation: {
                const E sq_expr = sq_clamp + prod * value * value;
                const E oeq = variant_.has_weight ? out_eq * W(total_wit + 3) : out_eq;
                E output_part = oeq * prod_expr;
                if (variant_.normalised_sum) output_part = output_part + E::Challenge(norm_id, 2, pow_two, F::zero()) * (norm_eq * prod_expr);
                inner = output_part + E::Challenge(norm_id, 1, pow_two, F::zero()) * (norm_eq * sq_expr) +
                        logup_eq * (sum + E::Challenge(input_id, 1, F::one(), F::zero()) * (W(total_out + c) * W(total_out + chunks + c)));
                break;
            }
            }
            full = full + chunk_ch * inner;
        }
        return full;
    }

    // all challenges of the expression, in its order; squeezes from the transcript
    std::vector<F> batching_challenges(const std::vector<F> &per_chunk, Transcript &t) const
    {
        std::vector<F> ch{t.append_and_sample("sum")};
        ch.insert(ch.end(), per_chunk.begin(), per_chunk.end());
        auto other = variant_.squeeze_sumcheck_challenges(t);
        ch.insert(ch.end(), other.begin(), other.end());
        return ch;
    }

    // prove_linking_sumcheck; `mles` in the expression's order, the weight table last when the variant has one.
    // Returns the proof and the batching challenges.
    std::pair<LookupSumcheckProof, std::vector<F>> prove_linking_sumcheck(const std::vector<const DensePolynomial *> &mles, Transcript &transcript,
                                                                          const std::vector<F> &last_claim_point, const std::vector<F> &logup_point,
                                                                          const DensePolynomial *weight_mle) const
    {
        if (mles.size() != witnesses()) throw Error(DPS_ERR_INVALID, "linking sumcheck: expected " + std::to_string(witnesses()) + " witness tables");
        if ((weight_mle != nullptr) != (variant_.kind == Variant::Normalisation && variant_.has_weight))
            throw Error(DPS_ERR_INVALID, "linking sumcheck: a weight table goes with the weighted normalisation variant only");
        auto eb = eq_point_and_batching_challenges(last_claim_point);
        if (logup_point.size() != eb.first.size()) throw Error(DPS_ERR_INVALID, "linking sumcheck: LogUp point length does not match the chunk");
        const std::vector<F> ch = batching_challenges(eb.second, transcript);
        const Context &ctx = mles[0]->context();
        std::vector<DensePolynomial> eqs = DensePolynomial::eq_many(ctx, eq_points(eb.first, logup_point));
        std::vector<const DensePolynomial *> all(mles);
        for (auto &e : eqs) all.push_back(&e);
        if (weight_mle) all.push_back(weight_mle);
        const size_t nv = eb.first.size();
        for (auto *p : all)
            if (p->num_vars() != nv) throw Error(DPS_ERR_INVALID, "linking sumcheck: every table has the chunk's number of variables");
        auto builder = VirtualPolynomialsBuilder::new_with_mles(optimal_sumcheck_threads(nv), nv, all);
        auto vp = builder.to_virtual_polys({build_full_sumcheck_expression()}, ch);
        auto res = IOPProverState::prove(vp, transcript);
        LookupSumcheckProof proof;
        proof.sumcheck_proof = std::move(res.first);
        auto evals = res.second.get_mle_flatten_final_evaluations();
        proof.sumcheck_point = res.second.collect_raw_challenges();
        if (weight_mle) {
            proof.has_weight_eval = true;
            proof.weight_eval = evals.back();
        }
        evals.resize(mles.size());  // drops the eq tables' (and the weight's) evaluations
        proof.evaluations = std::move(evals);
        return {std::move(proof), ch};
    }

    // verify_linking_sumcheck from the initial claim on (prepare_sumcheck_verification, which reads the LogUp
    // claims, is the caller's).  Throws when the proof does not verify; returns (batching challenges, point).
    std::pair<std::vector<F>, std::vector<F>> verify_linking_sumcheck(const LookupSumcheckProof &proof, const F &initial_claim, Transcript &transcript,
                                                                      const std::vector<F> &last_claim_point, const std::vector<F> &logup_point) const
    {
        auto eb = eq_point_and_batching_challenges(last_claim_point);
        if (logup_point.size() != eb.first.size()) throw Error(DPS_ERR_INVALID, "linking sumcheck: LogUp point length does not match the chunk");
        const std::vector<F> ch = batching_challenges(eb.second, transcript);
        if (proof.evaluations.size() != witnesses()) throw Error(DPS_ERR_INVALID, "linking sumcheck: wrong number of evaluations");
        const bool weighted = variant_.kind == Variant::Normalisation && variant_.has_weight;
        if (proof.has_weight_eval != weighted) throw Error(DPS_ERR_INVALID, "linking sumcheck: weight evaluation missing or unexpected");
        const Expression expr = build_full_sumcheck_expression();
        VPAuxInfo aux;
        aux.max_num_variables = eb.first.size();
        for (auto &m : expr.to_monomials(ch)) aux.max_degree = std::max(aux.max_degree, m.wits.size());
        SubClaim sub = IOPVerifierState::verify(initial_claim, proof.sumcheck_proof, aux, transcript);
        std::vector<F> all(proof.evaluations);
        for (auto &p : eq_points(eb.first, logup_point)) all.push_back(identity_eval(p.data(), sub.point.data(), std::min(p.size(), sub.point.size())));
        if (weighted) all.push_back(proof.weight_eval);
        if (expr.evaluate(all, ch) != sub.expected_evaluation) throw Error(DPS_ERR_INVALID, "Lookup sumcheck verification failed: the expression does not match the final claim");
        return {ch, sub.point};
    }

private:
    ChunkingInfo ci_;
    LookupVariant variant_;
    std::vector<uint64_t> shape_;
};

}  // namespace lookup
}  // namespace dpsc
