// Batched LogUp-GKR fractional sumcheck, host side: the driver and its verifier
// twin, with the layer tables and every per-layer sumcheck on the GPU.
// Follows zkml/src/lookup/logup_gkr/{circuit.rs, prover.rs, verifier.rs, structs.rs}.
#pragma once
#include <map>
#include <set>

#include "sumcheck.hpp"

namespace dpsc {
namespace logup {

enum class ProofType { Lookup, Table };

struct Claim {
    std::vector<F> point;
    F eval;
};

// LogUpInput (structs.rs:140-155).  Columns are base-field tables on the GPU.
struct LogUpInput {
    ProofType type = ProofType::Lookup;
    std::vector<const DensePolynomial *> column_evals;
    const DensePolynomial *multiplicities = nullptr;  // tables only
    F constant_challenge, column_separation_challenge;
    size_t columns_per_instance = 1;  // lookups only

    static LogUpInput new_lookup(std::vector<const DensePolynomial *> cols, const F &c, const F &beta, size_t per_instance)
    {
        if (cols.empty() || per_instance == 0 || cols.size() % per_instance) throw Error(DPS_ERR_INVALID, "LogUpInput: bad column count");
        for (auto *p : cols)
            if (p->len() != cols[0]->len()) throw Error(DPS_ERR_INVALID, "All sets of evaluations should be the same length");
        LogUpInput in;
        in.type = ProofType::Lookup;
        in.column_evals = std::move(cols);
        in.constant_challenge = c;
        in.column_separation_challenge = beta;
        in.columns_per_instance = per_instance;
        return in;
    }
    static LogUpInput new_table(std::vector<const DensePolynomial *> cols, const DensePolynomial *mult, const F &c, const F &beta)
    {
        if (cols.empty() || !mult) throw Error(DPS_ERR_INVALID, "LogUpInput: no columns");
        for (auto *p : cols)
            if (p->len() != cols[0]->len()) throw Error(DPS_ERR_INVALID, "All sets of evaluations should be the same length");
        if (mult->len() != cols[0]->len()) throw Error(DPS_ERR_INVALID, "Multiplicities length was not equal to column evaluations length");
        LogUpInput in;
        in.type = ProofType::Table;
        in.column_evals = std::move(cols);
        in.multiplicities = mult;
        in.constant_challenge = c;
        in.column_separation_challenge = beta;
        in.columns_per_instance = in.column_evals.size();
        return in;
    }
};

// LogUpCircuit (circuit.rs:503-590): layer 0 is the caller's columns, the layers
// above live in one GPU arena built by dps_logup_build.
class LogUpCircuit {
public:
    LogUpCircuit(const Context &ctx, std::vector<const DensePolynomial *> cols, const DensePolynomial *mult, const F &c, const F &beta)
        : ctx_(&ctx), cols_(std::move(cols)), mult_(mult), c_(c), beta_(beta)
    {
        std::vector<const dps_mle *> hs;
        for (auto *p : cols_) hs.push_back(p->raw());
        uint64_t cc[2] = {c.c0, c.c1}, bb[2] = {beta.c0, beta.c1};
        dps_logup *h = nullptr;
        ctx.check(dps_logup_build(ctx.raw(), hs.data(), (uint32_t)hs.size(), mult ? mult->raw() : nullptr, cc, bb, &h), "dps_logup_build");
        h_.reset(h, &dps_logup_free);
        uint32_t nl = 0;
        dps_logup_num_layers(h, &nl);
        n_layers_ = nl;
    }
    // variables of the sumcheck over the input layer (circuit.rs:67-80,564-566)
    size_t num_vars() const { return n_layers_ - 1; }
    bool is_table() const { return mult_ != nullptr; }
    size_t n_cols() const { return cols_.size(); }
    const F &constant_challenge() const { return c_; }
    const F &column_separation_challenge() const { return beta_; }
    // n_lo, n_hi, d_lo, d_hi of the last layer (circuit.rs:558-560)
    std::vector<F> outputs() const
    {
        uint64_t o[8];
        ctx_->check(dps_logup_outputs(h_.get(), o), "dps_logup_outputs");
        return from_limbs(o, 4);
    }
    size_t final_eval_count() const { return 2 * cols_.size() + (mult_ ? 2 : 0); }

    struct LayerInfo {
        std::vector<DensePolynomial> mles;  // borrowed half views
        Expression sumcheck_expression = Expression::ZERO();
        Expression claim_expression = Expression::ZERO();
    };

    // layer_proving_info (circuit.rs:231-412) for the layer whose halves have `lv` variables
    LayerInfo layer_proving_info(size_t lv, size_t layer_count, uint16_t w0) const
    {
        LayerInfo li;
        const uint64_t half = uint64_t(1) << lv;
        const F one = F::one(), zero = F::zero();
        uint16_t cid = (uint16_t)(layer_count * 4);
        Expression alpha_k = Expression::Challenge(0, layer_count, one, zero);
        Expression lambda = Expression::Challenge(1, 1, one, zero);
        Expression batching = Expression::Challenge(2, 1, one, zero);
        li.claim_expression =
            alpha_k * (batching * (Expression::WitIn(cid + 1) - Expression::WitIn(cid)) + Expression::WitIn(cid) +
                       lambda * (batching * (Expression::WitIn(cid + 3) - Expression::WitIn(cid + 2)) + Expression::WitIn(cid + 2)));
        if (lv < num_vars()) {
            // generic layer k: 2 * half entries per array
            uint32_t k = (uint32_t)(num_vars() - lv);
            dps_mle *num = nullptr, *den = nullptr;
            ctx_->check(dps_logup_layer(h_.get(), k, &num, &den), "dps_logup_layer");
            DensePolynomial pn(*ctx_, num), pd(*ctx_, den);
            li.mles.push_back(pn.view(0, (uint32_t)lv));
            li.mles.push_back(pn.view(half, (uint32_t)lv));
            li.mles.push_back(pd.view(0, (uint32_t)lv));
            li.mles.push_back(pd.view(half, (uint32_t)lv));
            Expression nl = Expression::WitIn(w0), nh = Expression::WitIn(w0 + 1), dl = Expression::WitIn(w0 + 2), dh = Expression::WitIn(w0 + 3);
            li.sumcheck_expression = alpha_k * (nl * dh + nh * dl + lambda * dl * dh);
            return li;
        }
        // input layer: halves of the multiplicities (tables) and of every column
        const uint16_t C = (uint16_t)cols_.size();
        uint16_t first_col = w0;
        if (mult_) {
            li.mles.push_back(mult_->view(0, (uint32_t)lv));
            li.mles.push_back(mult_->view(half, (uint32_t)lv));
            first_col = w0 + 2;
        }
        for (auto *c : cols_) li.mles.push_back(c->view(0, (uint32_t)lv));
        for (auto *c : cols_) li.mles.push_back(c->view(half, (uint32_t)lv));
        Expression dlo = Expression::Constant(c_), dhi = Expression::Constant(c_);
        F pw = one;
        for (uint16_t i = 0; i < C; i++) {
            dlo = dlo + Expression::Constant(pw) * Expression::WitIn(first_col + i);
            dhi = dhi + Expression::Constant(pw) * Expression::WitIn(first_col + C + i);
            pw *= beta_;
        }
        if (mult_)
            li.sumcheck_expression = alpha_k * (Expression::WitIn(w0) * dhi + Expression::WitIn(w0 + 1) * dlo + lambda * dlo * dhi);
        else
            li.sumcheck_expression = alpha_k * (-dhi - dlo + lambda * dlo * dhi);
        return li;
    }

    // combine_final_evals (circuit.rs:442-500)
    std::vector<F> combine_final_evals(const F *ev, const F &batching) const
    {
        std::vector<F> out;
        const size_t C = cols_.size();
        if (mult_) {
            out.push_back(batching * (ev[1] - ev[0]) + ev[0]);
            ev += 2;
        }
        for (size_t k = 0; k < C; k++) out.push_back(batching * (ev[C + k] - ev[k]) + ev[k]);
        return out;
    }

private:
    const Context *ctx_;
    std::vector<const DensePolynomial *> cols_;
    const DensePolynomial *mult_;
    F c_, beta_;
    std::shared_ptr<dps_logup> h_;
    size_t n_layers_ = 0;
};

// LogUpBatchProof (structs.rs:561-578)
struct LogUpBatchProof {
    std::vector<IOPProof> sumcheck_proofs;
    std::vector<std::vector<F>> round_evaluations;
    std::vector<Claim> output_claims;
    std::vector<std::vector<F>> circuit_outputs;
    ProofType proof_type = ProofType::Lookup;
    std::vector<size_t> num_vars_per_instance;
    std::vector<size_t> num_denominator_columns_per_instance;

    // structs.rs:587-597
    std::pair<std::vector<F>, std::vector<F>> fractional_outputs() const
    {
        std::vector<F> n, d;
        for (auto &e : circuit_outputs) {
            n.push_back(e[0] * e[3] + e[1] * e[2]);
            d.push_back(e[2] * e[3]);
        }
        return {n, d};
    }
};

// new_batch_multiple_sizes_prove (prover.rs:91-344)
inline LogUpBatchProof new_batch_multiple_sizes_prove(const Context &ctx, const std::vector<LogUpInput> &input, Transcript &transcript)
{
    if (input.empty()) throw Error(DPS_ERR_INVALID, "No inputs provided for LogUp");
    const ProofType proof_type = input[0].type;
    std::vector<LogUpCircuit> circuits;
    for (auto &in : input) {
        if (in.type != proof_type) throw Error(DPS_ERR_INVALID, "Not all proof types matched");
        if (in.type == ProofType::Table) {
            circuits.emplace_back(ctx, in.column_evals, in.multiplicities, in.constant_challenge, in.column_separation_challenge);
        } else {
            for (size_t i = 0; i < in.column_evals.size(); i += in.columns_per_instance) {
                std::vector<const DensePolynomial *> cols(in.column_evals.begin() + i, in.column_evals.begin() + i + in.columns_per_instance);
                circuits.emplace_back(ctx, cols, nullptr, in.constant_challenge, in.column_separation_challenge);
            }
        }
    }
    const size_t num_instances = circuits.size();
    size_t total_layers = circuits[0].num_vars();
    for (size_t i = 1; i < circuits.size(); i++) {
        if (circuits[i - 1].num_vars() < circuits[i].num_vars()) throw Error(DPS_ERR_INVALID, "Circuits were not in decreasing size order");
        total_layers = std::max(total_layers, circuits[i - 1].num_vars());
    }
    if (total_layers == 0) throw Error(DPS_ERR_INVALID, "LogUp instance too small: no layer to prove");
    std::set<size_t> unique_layer_size;
    for (auto &c : circuits) unique_layer_size.insert(c.num_vars());

    LogUpBatchProof proof;
    proof.proof_type = proof_type;
    for (auto &c : circuits) proof.circuit_outputs.push_back(c.outputs());

    // prover.rs:163-173
    transcript.append_scalars(std::vector<F>{F::from_u64(num_instances)});
    for (auto &o : proof.circuit_outputs) transcript.append_scalars(o);
    F batching_challenge = transcript.append_and_sample("initial_batching");
    F alpha = transcript.append_and_sample("initial_alpha");
    F lambda = transcript.append_and_sample("initial_lambda");
    std::vector<F> sumcheck_point{batching_challenge};

    for (size_t current_layer_vars = 1; current_layer_vars <= total_layers; current_layer_vars++) {
        const size_t remaining_layers = total_layers - (current_layer_vars - 1);
        // prover.rs:187-203
        std::vector<F> wit_evals;
        if (!proof.round_evaluations.empty()) wit_evals = proof.round_evaluations.back();
        for (size_t c = 0; c < circuits.size(); c++)
            if (circuits[c].num_vars() == remaining_layers)
                wit_evals.insert(wit_evals.end(), proof.circuit_outputs[c].begin(), proof.circuit_outputs[c].end());
        if (wit_evals.empty()) throw Error(DPS_ERR_INVALID, "Proving failed: No previous evals and no evals for this number of variables");

        // prover.rs:211-254
        size_t layer_count = 0;
        uint16_t witness_offset = 0;
        const size_t point_length = sumcheck_point.size();
        std::vector<DensePolynomial> witness_mles, eq_mles;
        std::vector<Expression> sumcheck_expressions;
        Expression claim_expression = Expression::ZERO();
        for (auto it = unique_layer_size.rbegin(); it != unique_layer_size.rend(); ++it) {
            const size_t size = *it;
            if (size < remaining_layers) continue;
            Expression claim_expr_multiplier = Expression::Constant(F::from_u64(uint64_t(1) << (total_layers - size)));
            Expression sumcheck_expr = Expression::ZERO();
            const size_t current_var_count = size + 1 - remaining_layers;
            for (auto &c : circuits) {
                if (c.num_vars() != size) continue;
                auto li = c.layer_proving_info(current_var_count, layer_count, witness_offset);
                layer_count += 1;
                witness_offset += (uint16_t)li.mles.size();
                for (auto &m : li.mles) witness_mles.push_back(std::move(m));
                sumcheck_expr = sumcheck_expr + li.sumcheck_expression;
                claim_expression = claim_expression + claim_expr_multiplier * li.claim_expression;
            }
            std::vector<F> eq_point(sumcheck_point.begin() + (point_length - current_var_count), sumcheck_point.end());
            eq_mles.push_back(DensePolynomial::eq(ctx, eq_point));
            sumcheck_expressions.push_back(sumcheck_expr);
        }
        // prover.rs:257-261
        F current_claim = claim_expression.evaluate(wit_evals, {alpha, lambda, batching_challenge});
        transcript.append_scalars(std::vector<F>{current_claim});

        // prover.rs:60-68,263-275
        Expression full = Expression::ZERO();
        for (size_t i = 0; i < sumcheck_expressions.size(); i++) full = full + sumcheck_expressions[i] * Expression::WitIn((uint16_t)(witness_offset + i));
        std::vector<const DensePolynomial *> all;
        for (auto &m : witness_mles) all.push_back(&m);
        for (auto &m : eq_mles) all.push_back(&m);
        auto builder = VirtualPolynomialsBuilder::new_with_mles(optimal_sumcheck_threads(current_layer_vars), current_layer_vars, all);
        auto vp = builder.to_virtual_polys({full}, {alpha, lambda});
        auto res = IOPProverState::prove(vp, transcript, &current_claim);

        // prover.rs:278-296
        sumcheck_point = res.second.collect_raw_challenges();
        const auto &fe = res.second.get_mle_flatten_final_evaluations();
        std::vector<F> evals(fe.begin(), fe.begin() + witness_offset);
        batching_challenge = transcript.append_and_sample("logup_batching");
        if (current_layer_vars != total_layers) {
            alpha = transcript.append_and_sample("logup_alpha");
            lambda = transcript.append_and_sample("logup_lambda");
        }
        sumcheck_point.push_back(batching_challenge);
        proof.sumcheck_proofs.push_back(std::move(res.first));
        proof.round_evaluations.push_back(std::move(evals));
    }

    // prover.rs:302-330
    const size_t point_length = sumcheck_point.size();
    size_t skip = 0;
    const auto &final_round = proof.round_evaluations.back();
    for (auto &c : circuits) {
        const size_t nv = c.num_vars() + 1;
        const size_t cnt = c.final_eval_count();
        if (skip + cnt > final_round.size()) throw Error(DPS_ERR_INVALID, "Proving failed: final round evaluations too short");
        auto evals = c.combine_final_evals(final_round.data() + skip, batching_challenge);
        skip += cnt;
        for (auto &e : evals) proof.output_claims.push_back(Claim{std::vector<F>(sumcheck_point.end() - nv, sumcheck_point.end()), e});
        proof.num_vars_per_instance.push_back(c.num_vars());
        proof.num_denominator_columns_per_instance.push_back(c.n_cols());
    }
    (void)point_length;
    return proof;
}

// LogUpVerifierInstance (structs.rs:306-547)
struct LogUpVerifierInstance {
    F constant_challenge, column_separation_challenge;
    size_t num_columns = 1;
    ProofType instance_type = ProofType::Lookup;
    size_t num_vars = 0;

    size_t num_final_round_evals() const { return instance_type == ProofType::Lookup ? 2 * num_columns : 2 * (1 + num_columns); }

    // instance_expressions (structs.rs:428-546)
    void instance_expressions(size_t &layer_count, uint16_t &w0, bool is_final_round, Expression &sumcheck_expr, Expression &claim_expr) const
    {
        const F one = F::one(), zero = F::zero();
        uint16_t cid = (uint16_t)(layer_count * 4);
        Expression alpha_k = Expression::Challenge(0, layer_count, one, zero);
        Expression lambda = Expression::Challenge(1, 1, one, zero);
        Expression batching = Expression::Challenge(2, 1, one, zero);
        claim_expr = alpha_k * (batching * (Expression::WitIn(cid + 1) - Expression::WitIn(cid)) + Expression::WitIn(cid) +
                                lambda * (batching * (Expression::WitIn(cid + 3) - Expression::WitIn(cid + 2)) + Expression::WitIn(cid + 2)));
        if (!is_final_round) {
            Expression nl = Expression::WitIn(w0), nh = Expression::WitIn(w0 + 1), dl = Expression::WitIn(w0 + 2), dh = Expression::WitIn(w0 + 3);
            sumcheck_expr = alpha_k * (nl * dh + nh * dl + lambda * dl * dh);
            layer_count += 1;
            w0 += 4;
            return;
        }
        const uint16_t C = (uint16_t)num_columns;
        uint16_t first_col = instance_type == ProofType::Table ? w0 + 2 : w0;
        Expression dlo = Expression::Constant(constant_challenge), dhi = Expression::Constant(constant_challenge);
        F pw = one;
        for (uint16_t i = 0; i < C; i++) {
            dlo = dlo + Expression::Constant(pw) * Expression::WitIn(first_col + i);
            dhi = dhi + Expression::Constant(pw) * Expression::WitIn(first_col + C + i);
            pw *= column_separation_challenge;
        }
        if (instance_type == ProofType::Table)
            sumcheck_expr = alpha_k * (Expression::WitIn(w0) * dhi + Expression::WitIn(w0 + 1) * dlo + lambda * dlo * dhi);
        else
            sumcheck_expr = alpha_k * (-dhi - dlo + lambda * dlo * dhi);
        layer_count += 1;
        w0 += (uint16_t)num_final_round_evals();
    }

    // final_claim (structs.rs:375-426)
    std::vector<Claim> final_claim(const F *ev, const F &batching, const std::vector<F> &point) const
    {
        std::vector<F> sub(point.end() - (1 + num_vars), point.end());
        std::vector<Claim> out;
        if (instance_type == ProofType::Table) {
            out.push_back(Claim{sub, batching * (ev[1] - ev[0]) + ev[0]});
            ev += 2;
        }
        for (size_t k = 0; k < num_columns; k++) out.push_back(Claim{sub, batching * (ev[num_columns + k] - ev[k]) + ev[k]});
        return out;
    }
};

struct LogUpBatchVerifierClaim {
    std::vector<Claim> output_claims;
    std::vector<F> point;
    std::vector<F> numerators, denominators;
};

// new_verify_logup_proof_multiple_sizes (verifier.rs:77-256).  Throws on rejection.
inline LogUpBatchVerifierClaim new_verify_logup_proof_multiple_sizes(const LogUpBatchProof &proof, const std::vector<LogUpVerifierInstance> &instances,
                                                                     Transcript &transcript)
{
    if (proof.circuit_outputs.size() != instances.size() || proof.sumcheck_proofs.size() != proof.round_evaluations.size())
        throw Error(DPS_ERR_INVALID, "LogUp verifier: malformed proof");
    transcript.append_scalars(std::vector<F>{F::from_u64(instances.size())});
    for (auto &o : proof.circuit_outputs) {
        if (o.size() != 4) throw Error(DPS_ERR_INVALID, "LogUp verifier: malformed circuit outputs");
        transcript.append_scalars(o);
    }
    LogUpBatchVerifierClaim out;
    auto frac = proof.fractional_outputs();
    out.numerators = frac.first;
    out.denominators = frac.second;
    std::set<size_t> unique_layer_size;
    for (auto &i : instances) unique_layer_size.insert(i.num_vars);
    const size_t total_layers = proof.sumcheck_proofs.size();

    F batching_challenge = transcript.append_and_sample("initial_batching");
    F alpha = transcript.append_and_sample("initial_alpha");
    F lambda = transcript.append_and_sample("initial_lambda");
    std::vector<F> sumcheck_point{batching_challenge};

    for (size_t i = 0; i < total_layers; i++) {
        const size_t remaining_layers = total_layers - i;
        std::vector<F> wit_evals;
        if (i != 0) wit_evals = proof.round_evaluations[i - 1];
        for (size_t c = 0; c < instances.size(); c++)
            if (instances[c].num_vars == remaining_layers) wit_evals.insert(wit_evals.end(), proof.circuit_outputs[c].begin(), proof.circuit_outputs[c].end());
        if (wit_evals.empty()) throw Error(DPS_ERR_INVALID, "No previous evals and no evals for this number of variables");
        size_t layer_count = 0;
        uint16_t witness_offset = 0;
        const size_t point_length = sumcheck_point.size();
        std::vector<std::vector<F>> eq_points;
        std::vector<Expression> sumcheck_expressions;
        Expression claim_expression = Expression::ZERO();
        for (auto it = unique_layer_size.rbegin(); it != unique_layer_size.rend(); ++it) {
            const size_t size = *it;
            if (size < remaining_layers) continue;
            Expression mult = Expression::Constant(F::from_u64(uint64_t(1) << (total_layers - size)));
            Expression sumcheck_expr = Expression::ZERO();
            const size_t current_var_count = size + 1 - remaining_layers;
            for (auto &inst : instances) {
                if (inst.num_vars != size) continue;
                Expression se = Expression::ZERO(), ce = Expression::ZERO();
                inst.instance_expressions(layer_count, witness_offset, (i + 1) == total_layers, se, ce);
                sumcheck_expr = sumcheck_expr + se;
                claim_expression = claim_expression + mult * ce;
            }
            eq_points.emplace_back(sumcheck_point.begin() + (point_length - current_var_count), sumcheck_point.end());
            sumcheck_expressions.push_back(sumcheck_expr);
        }
        F current_claim = claim_expression.evaluate(wit_evals, {alpha, lambda, batching_challenge});
        transcript.append_scalars(std::vector<F>{current_claim});

        const size_t current_num_vars = i + 1;
        VPAuxInfo aux = from_mle_list_dimensions({{current_num_vars, current_num_vars, current_num_vars}});
        SubClaim sub = IOPVerifierState::verify(current_claim, proof.sumcheck_proofs[i], aux, transcript);
        batching_challenge = transcript.append_and_sample("logup_batching");

        Expression full = Expression::ZERO();
        for (size_t k = 0; k < sumcheck_expressions.size(); k++) full = full + sumcheck_expressions[k] * Expression::WitIn((uint16_t)(witness_offset + k));
        std::vector<F> full_evals = proof.round_evaluations[i];
        if (full_evals.size() != witness_offset) throw Error(DPS_ERR_INVALID, "LogUp verifier: wrong number of round evaluations");
        for (auto &ep : eq_points) full_evals.push_back(identity_eval(sub.point.data() + (sub.point.size() - ep.size()), ep.data(), ep.size()));
        F calc = full.evaluate(full_evals, {alpha, lambda});
        if ((i + 1) != total_layers) {
            alpha = transcript.append_and_sample("logup_alpha");
            lambda = transcript.append_and_sample("logup_lambda");
        }
        if (calc != sub.expected_evaluation)
            throw Error(DPS_ERR_INVALID, "LogUp Verifier error: calculated sumcheck claim does not equal this round's output claim at round " + std::to_string(i));
        sumcheck_point = sub.point;
        sumcheck_point.push_back(batching_challenge);
    }
    const auto &final_round = proof.round_evaluations.back();
    size_t skip = 0;
    for (auto &inst : instances) {
        if (skip + inst.num_final_round_evals() > final_round.size()) throw Error(DPS_ERR_INVALID, "LogUp verifier: final round evaluations too short");
        auto cl = inst.final_claim(final_round.data() + skip, batching_challenge, sumcheck_point);
        skip += inst.num_final_round_evals();
        out.output_claims.insert(out.output_claims.end(), cl.begin(), cl.end());
    }
    out.point = sumcheck_point;
    return out;
}

}  // namespace logup
}  // namespace dpsc
