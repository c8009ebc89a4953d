// Einsum / matmul proof, host side: axis classification, partial evaluation of
// the quantised inputs on the GPU, the batched degree-2 sumcheck and the input
// claims.  Follows zkml/src/layers/einsum/{axis.rs:478-580,1016-1259, prove.rs:46-361,
// op_info.rs:137-199}.  A bias added to an output gives a claim of its own: the bias tensor's
// multilinear extension at the part of the output claim's point that its axes name
// (prove.rs:191-214, axis.rs:582-637), evaluated on the GPU.  Constant tensors (weights)
// are ordinary right-hand sides here: they arrive unpadded like every tensor and are padded
// by the kernels that read them (prove.rs:66-94 pads them on the host).
#pragma once
#include <string>

#include "sumcheck.hpp"

namespace dpsc {
namespace einsum {

enum class AxisType { Contracted = DPS_AXIS_CONTRACTED, Outer = DPS_AXIS_OUTER, Stacked = DPS_AXIS_STACKED };

struct Claim {
    std::vector<F> point;
    F eval;
};

// A quantised tensor on the GPU: raw integers, row-major, stored compactly in the unpadded shape.  Padding and
// the embedding into the field happen in the kernels that read it (einsum/prove.rs:66-94 materialises a padded
// Tensor<F> instead).
struct Tensor {
    std::vector<uint64_t> padded_shape, unpadded_shape;
    DensePolynomial device;

    static Tensor with_shape(const std::vector<uint64_t> &shape, uint64_t n)
    {
        Tensor t;
        t.unpadded_shape = shape;
        for (auto d : shape) {
            uint64_t p = 1;
            while (p < d) p <<= 1;
            t.padded_shape.push_back(p);
        }
        uint64_t utotal = 1;
        for (auto d : shape) utotal *= d;
        if (n != utotal) throw Error(DPS_ERR_INVALID, "Tensor: data does not match the shape");
        return t;
    }
    // upload for the length of one proof
    static Tensor from_unpadded(const Context &ctx, const int64_t *data, uint64_t n, const std::vector<uint64_t> &shape)
    {
        Tensor t = with_shape(shape, n);
        dps_mle *h = nullptr;
        ctx.check(dps_tensor_from_i64(ctx.raw(), data, n, &h), "dps_tensor_from_i64");
        t.device = DensePolynomial(ctx, h);
        return t;
    }
    static Tensor from_unpadded(const Context &ctx, const std::vector<int64_t> &data, const std::vector<uint64_t> &shape)
    {
        return from_unpadded(ctx, data.data(), data.size(), shape);
    }
    // a tensor the caller uploaded before (dps_tensor_from_i64 / dps_tensor_from_i16, unpadded) and keeps: weights
    // stay on the device across proofs, activations go there once per layer
    static Tensor resident(const Context &ctx, const dps_mle *handle, const std::vector<uint64_t> &shape)
    {
        int32_t kind = 0;
        uint64_t len = 0;
        if (!handle || dps_mle_info(handle, &kind, &len) != DPS_OK) throw Error(DPS_ERR_INVALID, "Tensor: null handle");
        if (kind != DPS_I64 && kind != DPS_I16) throw Error(DPS_ERR_INVALID, "Tensor: the handle is not a raw integer tensor");
        Tensor t = with_shape(shape, len);
        t.device = DensePolynomial::borrowed(ctx, handle);
        return t;
    }
    // the padded tensor as a base-field table (the aggregation sumcheck's input)
    DensePolynomial padded_mle(const Context &ctx) const { return DensePolynomial::from_tensor(ctx, device, padded_shape, unpadded_shape); }
};

// Shape::split_point (zkml/src/shape.rs:475-496): the last dimension takes the lowest variables
inline std::vector<std::vector<F>> split_point(const std::vector<uint64_t> &padded_shape, const std::vector<F> &point)
{
    size_t need = 0;
    for (auto d : padded_shape) need += ceil_log2(d);
    if (point.size() != need) throw Error(DPS_ERR_INVALID, "Point length does not match shape number of variables");
    std::vector<std::vector<F>> out(padded_shape.size());
    size_t start = 0;
    for (size_t a = padded_shape.size(); a-- > 0;) {
        size_t l = ceil_log2(padded_shape[a]);
        out[a].assign(point.begin() + start, point.begin() + start + l);
        start += l;
    }
    return out;
}

struct FixedAxis {
    AxisType type = AxisType::Contracted;
    std::vector<F> point;  // empty for contracted axes
};

// One batched operation: lhs labels, rhs labels -> output labels, e.g. "ik","kj","ij"; `bias`: the labels of the bias
// tensor added to the output (a subset of the output's, "A(ij)@B(kj)->C(ik)+BIAS(k)" has "k"), empty when there is none
struct Op {
    std::string lhs, rhs, out, bias;
};

inline AxisType classify(const Op &op, char label)
{
    bool l = op.lhs.find(label) != std::string::npos, r = op.rhs.find(label) != std::string::npos, o = op.out.find(label) != std::string::npos;
    if (l && r && o) return AxisType::Stacked;
    if (l && r && !o) return AxisType::Contracted;
    if ((l != r) && o) return AxisType::Outer;
    throw Error(DPS_ERR_UNSUPPORTED, std::string("einsum axis '") + label + "' is neither stacked, contracted nor outer");
}

// bias_evaluation_point (axis.rs:582-637): the slices of the output claim's point that belong to the bias tensor's
// axes, the last axis first (it takes the lowest variables)
inline std::vector<F> bias_evaluation_point(const Op &op, const std::vector<std::vector<F>> &out_slices)
{
    std::vector<F> point;
    for (size_t a = op.bias.size(); a-- > 0;) {
        const size_t pos = op.out.find(op.bias[a]);
        if (pos == std::string::npos) throw Error(DPS_ERR_INVALID, std::string("Bias tensor has an axis '") + op.bias[a] + "' that is not present in the output tensor");
        point.insert(point.end(), out_slices[pos].begin(), out_slices[pos].end());
    }
    return point;
}

// reconstruct_full_point (prove.rs:337-361)
inline std::vector<F> reconstruct_full_point(const std::vector<FixedAxis> &fixed, const std::vector<F> &sumcheck_point, const std::vector<uint64_t> &input_shape)
{
    std::vector<F> out;
    size_t skip = 0;
    for (size_t a = fixed.size(); a-- > 0;) {
        if (fixed[a].type == AxisType::Contracted) {
            size_t l = ceil_log2(input_shape[a]);
            if (skip + l > sumcheck_point.size()) throw Error(DPS_ERR_INVALID, "reconstruct_full_point: sumcheck point too short");
            out.insert(out.end(), sumcheck_point.begin() + skip, sumcheck_point.begin() + skip + l);
            skip += l;
        } else {
            out.insert(out.end(), fixed[a].point.begin(), fixed[a].point.end());
        }
    }
    return out;
}

// mles_from_tensor (axis.rs:1142-1234) on the GPU
inline std::vector<DensePolynomial> mles_from_tensor(const Context &ctx, const std::vector<FixedAxis> &fixed, const Tensor &t)
{
    const size_t nd = t.padded_shape.size();
    std::vector<int32_t> kinds(nd);
    std::vector<std::vector<uint64_t>> limbs(nd);
    std::vector<const uint64_t *> pts(nd, nullptr);
    uint64_t stacked = 1;
    for (size_t a = 0; a < nd; a++) {
        kinds[a] = (int32_t)fixed[a].type;
        if (fixed[a].type == AxisType::Outer) {
            limbs[a] = to_limbs(fixed[a].point);
            pts[a] = limbs[a].data();
        }
        if (fixed[a].type == AxisType::Stacked) stacked *= t.unpadded_shape[a];
    }
    std::vector<dps_mle *> out(stacked, nullptr);
    uint32_t n_out = 0;
    ctx.check(dps_partial_eval(ctx.raw(), t.device.raw(), t.padded_shape.data(), t.unpadded_shape.data(), (uint32_t)nd, kinds.data(), pts.data(),
                               out.data(), (uint32_t)stacked, &n_out),
              "dps_partial_eval");
    std::vector<DensePolynomial> res;
    for (uint32_t i = 0; i < n_out; i++) res.emplace_back(ctx, out[i]);
    return res;
}

// stacking coefficients (axis.rs:1043-1062): outer product of the stacked axes' truncated eq tables
inline std::vector<F> stacking_coeffs(const std::vector<FixedAxis> &fixed, const std::vector<uint64_t> &unpadded_shape)
{
    std::vector<F> acc{F::one()};
    for (size_t a = fixed.size(); a-- > 0;) {
        if (fixed[a].type != AxisType::Stacked) continue;
        auto beta = eq_evals_host(fixed[a].point.data(), fixed[a].point.size());
        std::vector<F> next;
        for (uint64_t b = 0; b < unpadded_shape[a]; b++)
            for (auto &x : acc) next.push_back(x * beta[b]);
        acc = std::move(next);
    }
    return acc;
}

// build_einsum_expression (op_info.rs:159-199)
inline Expression build_einsum_expression(const std::vector<std::vector<F>> &coeffs)
{
    const size_t rhs_inputs = coeffs.size();
    Expression acc = Expression::ZERO();
    for (size_t i = 0; i < coeffs.size(); i++) {
        const size_t S = coeffs[i].size(), offset = i * S, rhs_offset = rhs_inputs * S + offset;
        Expression inner = Expression::Constant(coeffs[i][0]) * Expression::WitIn((uint16_t)offset) * Expression::WitIn((uint16_t)rhs_offset);
        for (size_t j = 1; j < S; j++)
            inner = Expression::Constant(coeffs[i][j]) * Expression::WitIn((uint16_t)(j + offset)) * Expression::WitIn((uint16_t)(j + rhs_offset)) + inner;
        acc = acc + Expression::Challenge(0, i, F::one(), F::zero()) * inner;
    }
    return acc;
}

struct EinSumProof {
    std::vector<F> bias_evals;  // one per output that has a bias, in output order
    IOPProof einsum_sumcheck;
    std::vector<F> einsum_evaluations;
    bool has_aggregation = false;
    IOPProof input_aggregation_sumcheck;
};

struct EinSumProofInfo {
    std::vector<Claim> claims;  // lhs first, then one per rhs
    std::vector<std::pair<size_t, Claim>> bias_claims;  // (output, claim on its bias tensor): the constant-polynomial claims of prove.rs:254-258
    EinSumProof proof;
    std::vector<F> einsum_sumcheck_point;
    std::vector<std::vector<F>> stacking_coeffs;
};

// EinSum::prove_internal (prove.rs:46-333).  ops[r] contracts the one LHS with
// rhs[r] into output r; last_claims[r] is the claim on output r; biases[r] is the
// tensor added to output r (nullptr: none; `biases` may be empty when no output has one).
inline EinSumProofInfo prove_internal(const Context &ctx, const std::vector<Op> &ops, const Tensor &lhs, const std::vector<Tensor> &rhs,
                                      const std::vector<Claim> &last_claims, Transcript &transcript, const std::vector<const Tensor *> &biases = {})
{
    const size_t R = ops.size();
    if (R == 0 || rhs.size() != R || last_claims.size() != R) throw Error(DPS_ERR_INVALID, "prove_internal: mismatched number of inputs and claims");
    if (!biases.empty() && biases.size() != R) throw Error(DPS_ERR_INVALID, "prove_internal: one bias slot per output");
    std::vector<std::vector<F>> bias_points(R);
    std::vector<std::vector<FixedAxis>> lhs_fixes(R), rhs_fixes(R);
    uint64_t contraction_size = 0, stacking_size = 0;
    for (size_t r = 0; r < R; r++) {
        const Op &op = ops[r];
        if (op.lhs.size() != lhs.padded_shape.size() || op.rhs.size() != rhs[r].padded_shape.size())
            throw Error(DPS_ERR_INVALID, "prove_internal: equation rank does not match the tensors");
        // output shape from the inputs' padded shapes, then split the claim point per output dimension
        std::vector<uint64_t> out_shape;
        for (char c : op.out) {
            size_t pl = op.lhs.find(c), pr = op.rhs.find(c);
            if (pl != std::string::npos)
                out_shape.push_back(lhs.padded_shape[pl]);
            else if (pr != std::string::npos)
                out_shape.push_back(rhs[r].padded_shape[pr]);
            else
                throw Error(DPS_ERR_INVALID, "prove_internal: output axis not found in any input tensor");
        }
        auto slices = split_point(out_shape, last_claims[r].point);
        const Tensor *bias = biases.empty() ? nullptr : biases[r];
        if ((bias != nullptr) != !op.bias.empty()) throw Error(DPS_ERR_INVALID, "prove_internal: bias labels and bias tensor do not go together");
        if (bias) {
            if (bias->padded_shape.size() != op.bias.size()) throw Error(DPS_ERR_INVALID, "prove_internal: bias rank does not match its labels");
            bias_points[r] = bias_evaluation_point(op, slices);
            size_t nv = 0;
            for (auto d : bias->padded_shape) nv += ceil_log2(d);
            if (nv != bias_points[r].size()) throw Error(DPS_ERR_INVALID, "prove_internal: bias shape does not match the output's");
        }
        auto fix = [&](const std::string &labels) {
            std::vector<FixedAxis> fa(labels.size());
            for (size_t a = 0; a < labels.size(); a++) {
                fa[a].type = classify(op, labels[a]);
                if (fa[a].type != AxisType::Contracted) fa[a].point = slices[op.out.find(labels[a])];
            }
            return fa;
        };
        lhs_fixes[r] = fix(op.lhs);
        rhs_fixes[r] = fix(op.rhs);
        uint64_t cs = 1, ss = 1;
        for (size_t a = 0; a < op.lhs.size(); a++) {
            if (lhs_fixes[r][a].type == AxisType::Contracted) cs *= lhs.unpadded_shape[a];
            if (lhs_fixes[r][a].type == AxisType::Stacked) ss *= lhs.unpadded_shape[a];
        }
        if (r == 0) {
            contraction_size = cs;
            stacking_size = ss;
        } else if (cs != contraction_size || ss != stacking_size) {
            throw Error(DPS_ERR_INVALID, "prove_internal: batched operations disagree on the contraction or stacking size");
        }
    }
    // fix_axes (axis.rs:478-500): partial evaluation on the GPU
    std::vector<std::vector<DensePolynomial>> fixed_lhs(R), fixed_rhs(R);
    EinSumProofInfo info;
    for (size_t r = 0; r < R; r++) {
        fixed_lhs[r] = mles_from_tensor(ctx, lhs_fixes[r], lhs);
        fixed_rhs[r] = mles_from_tensor(ctx, rhs_fixes[r], rhs[r]);
        info.stacking_coeffs.push_back(stacking_coeffs(lhs_fixes[r], lhs.unpadded_shape));
        if (fixed_lhs[r].size() != stacking_size || fixed_rhs[r].size() != stacking_size)
            throw Error(DPS_ERR_INVALID, "prove_internal: unexpected number of stacked tables");
    }
    F batching_challenge = transcript.append_and_sample("batching_challenge");  // prove.rs:158
    const uint32_t num_vars = ceil_log2(contraction_size);
    std::vector<const DensePolynomial *> mles;
    for (auto &v : fixed_lhs)
        for (auto &p : v) mles.push_back(&p);
    for (auto &v : fixed_rhs)
        for (auto &p : v) mles.push_back(&p);
    auto builder = VirtualPolynomialsBuilder::new_with_mles(optimal_sumcheck_threads(num_vars), num_vars, mles);
    auto vp = builder.to_virtual_polys({build_einsum_expression(info.stacking_coeffs)}, {batching_challenge});
    auto res = IOPProverState::prove(vp, transcript);  // prove.rs:184
    info.proof.einsum_sumcheck = std::move(res.first);
    info.proof.einsum_evaluations = res.second.get_mle_flatten_final_evaluations();
    info.einsum_sumcheck_point = res.second.collect_raw_challenges();
    // prove.rs:191-222: the bias tensors at their points
    for (size_t r = 0; r < R && !biases.empty(); r++) {
        if (!biases[r]) continue;
        Claim c;
        c.point = bias_points[r];
        c.eval = biases[r]->padded_mle(ctx).evaluate(c.point);
        info.proof.bias_evals.push_back(c.eval);
        info.bias_claims.emplace_back(r, std::move(c));
    }
    const auto &ev = info.proof.einsum_evaluations;
    const size_t half = ev.size() / 2;
    // prove.rs:224-253: one claim per RHS
    std::vector<Claim> rhs_claims;
    for (size_t r = 0; r < R; r++) {
        Claim c;
        c.point = reconstruct_full_point(rhs_fixes[r], info.einsum_sumcheck_point, rhs[r].padded_shape);
        c.eval = F::zero();
        for (size_t j = 0; j < stacking_size; j++) c.eval += info.stacking_coeffs[r][j] * ev[half + r * stacking_size + j];
        rhs_claims.push_back(std::move(c));
    }
    Claim lhs_claim;
    if (R > 1) {
        // prove.rs:260-302: aggregate the R claims on the LHS with a second sumcheck
        DensePolynomial input_mle = lhs.padded_mle(ctx);
        const uint32_t nv = input_mle.num_vars();
        std::vector<std::vector<F>> eq_points;
        for (size_t r = 0; r < R; r++) eq_points.push_back(reconstruct_full_point(lhs_fixes[r], info.einsum_sumcheck_point, lhs.padded_shape));
        std::vector<DensePolynomial> eq_polys = DensePolynomial::eq_many(ctx, eq_points);
        F input_batching = transcript.append_and_sample("input_batching_challenge");
        std::vector<const DensePolynomial *> am{&input_mle};
        for (auto &p : eq_polys) am.push_back(&p);
        // build_aggregation_expression (op_info.rs:137-152)
        Expression agg = Expression::ZERO();
        for (size_t i = 0; i < R; i++)
            agg = agg + Expression::WitIn(0) * Expression::WitIn((uint16_t)(i + 1)) * Expression::Challenge(0, i, F::one(), F::zero());
        auto ab = VirtualPolynomialsBuilder::new_with_mles(optimal_sumcheck_threads(nv), nv, am);
        auto avp = ab.to_virtual_polys({agg}, {input_batching});
        auto ares = IOPProverState::prove(avp, transcript);
        lhs_claim.point = ares.second.collect_raw_challenges();
        lhs_claim.eval = ares.second.get_mle_flatten_final_evaluations()[0];
        info.proof.has_aggregation = true;
        info.proof.input_aggregation_sumcheck = std::move(ares.first);
    } else {
        // prove.rs:309-316
        lhs_claim.point = reconstruct_full_point(lhs_fixes[0], info.einsum_sumcheck_point, lhs.padded_shape);
        lhs_claim.eval = F::zero();
        for (size_t j = 0; j < stacking_size; j++) lhs_claim.eval += info.stacking_coeffs[0][j] * ev[j];
    }
    info.claims.push_back(std::move(lhs_claim));
    for (auto &c : rhs_claims) info.claims.push_back(std::move(c));
    return info;
}

}  // namespace einsum
}  // namespace dpsc
