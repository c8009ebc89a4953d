// C wrappers over the C++ host mirror (see dpsc_host.h).
#include "dpsc_host.h"

#include <string>

#include "dpsc/einsum.hpp"
#include "dpsc/logup.hpp"
#include "dpsc/lookup_linking.hpp"
#include "dpsc/poly_commit.hpp"
#include "dpsc/same_poly.hpp"
#include "dpsc/sumcheck.hpp"

using namespace dpsc;

struct dph_transcript {
    Blake3Transcript t;
    explicit dph_transcript(const char *label) : t(label) {}
};

namespace {
thread_local std::string g_err;

template <class Fn>
int32_t guarded(Fn &&fn)
{
    try {
        fn();
        return DPS_OK;
    } catch (const Error &e) {
        g_err = e.what();
        return e.status;
    } catch (const std::exception &e) {
        g_err = e.what();
        return DPS_ERR_INVALID;
    }
}
}  // namespace

extern "C" {

const char *dph_last_error(void) { return g_err.c_str(); }

dph_transcript *dph_tr_new(const char *label) { return new dph_transcript(label); }
dph_transcript *dph_tr_clone(const dph_transcript *t) { return new dph_transcript(*t); }
void dph_tr_free(dph_transcript *t) { delete t; }
void dph_tr_append_message(dph_transcript *t, const char *label) { t->t.append_message(label); }
void dph_tr_append_bytes(dph_transcript *t, const uint8_t *data, size_t len) { t->t.append_bytes(data, len); }
void dph_tr_append_u64(dph_transcript *t, uint64_t x) { t->t.append_u64(x); }
void dph_tr_append_scalars(dph_transcript *t, const uint64_t *xs, size_t n)
{
    auto v = from_limbs(xs, n);
    t->t.append_scalars(v.data(), v.size());
}
void dph_tr_challenge_scalar(dph_transcript *t, uint64_t out[2])
{
    F r = t->t.challenge_scalar();
    out[0] = r.c0;
    out[1] = r.c1;
}
void dph_tr_append_and_sample(dph_transcript *t, const char *label, uint64_t out[2])
{
    F r = t->t.append_and_sample(label);
    out[0] = r.c0;
    out[1] = r.c1;
}
void dph_tr_state(const dph_transcript *t, uint8_t state_out[32], uint32_t *n_rounds)
{
    memcpy(state_out, t->t.state(), 32);
    if (n_rounds) *n_rounds = t->t.n_rounds();
}
void dph_blake3(const uint8_t *data, size_t len, uint8_t out[32]) { Blake3::hash(data, len, out); }

int32_t dph_sumcheck_prove(dps_ctx *ctx, uint32_t n_vars, const dps_mle *const *mles, uint32_t n_mles,
                           const dps_term *terms, uint32_t n_terms, dph_transcript *t, uint64_t *proof_out,
                           uint64_t *point_out, uint64_t *finals_out, uint32_t *degree_out)
{
    return dph_sumcheck_prove_claimed(ctx, n_vars, mles, n_mles, terms, n_terms, nullptr, t, proof_out, point_out, finals_out, degree_out);
}

int32_t dph_sumcheck_prove_claimed(dps_ctx *ctx, uint32_t n_vars, const dps_mle *const *mles, uint32_t n_mles,
                                   const dps_term *terms, uint32_t n_terms, const uint64_t claimed_sum[2], dph_transcript *t,
                                   uint64_t *proof_out, uint64_t *point_out, uint64_t *finals_out, uint32_t *degree_out)
{
    return guarded([&] {
        Context c(ctx);
        VirtualPolynomials vp;
        vp.ctx = &c;
        vp.num_vars = n_vars;
        vp.mles.assign(mles, mles + n_mles);
        vp.terms.assign(terms, terms + n_terms);
        F claim;
        if (claimed_sum) claim = F(claimed_sum[0], claimed_sum[1]);
        auto res = IOPProverState::prove(vp, t->t, claimed_sum ? &claim : nullptr);
        size_t npts = res.first.proofs.empty() ? 0 : res.first.proofs[0].evaluations.size();
        if (degree_out) *degree_out = npts ? (uint32_t)npts - 1 : 0;
        size_t w = 0;
        for (auto &m : res.first.proofs)
            for (auto &e : m.evaluations) {
                proof_out[w++] = e.c0;
                proof_out[w++] = e.c1;
            }
        auto &pt = res.second.collect_raw_challenges();
        for (size_t i = 0; i < pt.size(); i++) {
            point_out[2 * i] = pt[i].c0;
            point_out[2 * i + 1] = pt[i].c1;
        }
        auto &fe = res.second.get_mle_flatten_final_evaluations();
        for (size_t i = 0; i < fe.size(); i++) {
            finals_out[2 * i] = fe[i].c0;
            finals_out[2 * i + 1] = fe[i].c1;
        }
    });
}

int32_t dph_sumcheck_verify(const uint64_t claimed_sum[2], const uint64_t *proof, uint32_t n_vars, uint32_t degree,
                            dph_transcript *t, uint64_t *point_out, uint64_t expected_out[2])
{
    return guarded([&] {
        IOPProof p;
        for (uint32_t j = 0; j < n_vars; j++) p.proofs.push_back(IOPProverMessage{from_limbs(proof + 2 * (size_t)(degree + 1) * j, degree + 1)});
        VPAuxInfo aux;
        aux.max_degree = degree;
        aux.max_num_variables = n_vars;
        SubClaim sc = IOPVerifierState::verify(F(claimed_sum[0], claimed_sum[1]), p, aux, t->t);
        for (size_t i = 0; i < sc.point.size(); i++) {
            point_out[2 * i] = sc.point[i].c0;
            point_out[2 * i + 1] = sc.point[i].c1;
        }
        expected_out[0] = sc.expected_evaluation.c0;
        expected_out[1] = sc.expected_evaluation.c1;
    });
}

namespace {

// the proof and the claims as 64-bit words, in the order the header states
void write_einsum(const einsum::EinSumProofInfo &info, uint64_t *out, uint64_t out_cap, uint64_t *n_words)
{
    std::vector<uint64_t> w;
    auto put = [&](const F &x) {
        w.push_back(x.c0);
        w.push_back(x.c1);
    };
    auto put_proof = [&](const IOPProof &p) {
        w.push_back(p.proofs.size());
        w.push_back(p.proofs.empty() ? 0 : p.proofs[0].evaluations.size());
        for (auto &m : p.proofs)
            for (auto &e : m.evaluations) put(e);
    };
    put_proof(info.proof.einsum_sumcheck);
    w.push_back(info.proof.einsum_evaluations.size());
    for (auto &e : info.proof.einsum_evaluations) put(e);
    if (info.proof.has_aggregation)
        put_proof(info.proof.input_aggregation_sumcheck);
    else
        w.push_back(0);
    w.push_back(info.claims.size());
    for (auto &cl : info.claims) {
        w.push_back(cl.point.size());
        for (auto &x : cl.point) put(x);
        put(cl.eval);
    }
    w.push_back(info.bias_claims.size());
    for (auto &bc : info.bias_claims) {
        w.push_back(bc.first);
        w.push_back(bc.second.point.size());
        for (auto &x : bc.second.point) put(x);
        put(bc.second.eval);
    }
    if (w.size() > out_cap) throw Error(DPS_ERR_INVALID, "dph_einsum_prove: output buffer too small");
    memcpy(out, w.data(), w.size() * 8);
    *n_words = w.size();
}

uint64_t shape_count(const uint64_t *shape, uint32_t rank)
{
    uint64_t n = 1;
    for (uint32_t i = 0; i < rank; i++) n *= shape[i];
    return n;
}

}  // namespace

int32_t dph_einsum_prove(dps_ctx *ctx, uint32_t n_ops, const char *const *labels, const int64_t *lhs,
                         const uint64_t *lhs_shape, uint32_t lhs_rank, const int64_t *const *rhs,
                         const uint64_t *const *rhs_shapes, const uint32_t *rhs_ranks,
                         const int64_t *const *biases, const uint64_t *const *bias_shapes, const uint32_t *bias_ranks,
                         const uint64_t *const *claim_points, const uint32_t *claim_point_lens,
                         const uint64_t *claim_evals, dph_transcript *t, uint64_t *out, uint64_t out_cap,
                         uint64_t *n_words)
{
    return guarded([&] {
        Context c(ctx);
        std::vector<einsum::Op> ops;
        std::vector<einsum::Tensor> rts;
        std::vector<einsum::Claim> claims;
        std::vector<std::unique_ptr<einsum::Tensor>> bts(n_ops);
        std::vector<const einsum::Tensor *> bptr;
        einsum::Tensor lt = einsum::Tensor::from_unpadded(c, lhs, shape_count(lhs_shape, lhs_rank), std::vector<uint64_t>(lhs_shape, lhs_shape + lhs_rank));
        for (uint32_t r = 0; r < n_ops; r++) {
            ops.push_back(einsum::Op{labels[4 * r], labels[4 * r + 1], labels[4 * r + 2], labels[4 * r + 3]});
            rts.push_back(einsum::Tensor::from_unpadded(c, rhs[r], shape_count(rhs_shapes[r], rhs_ranks[r]),
                                                        std::vector<uint64_t>(rhs_shapes[r], rhs_shapes[r] + rhs_ranks[r])));
            claims.push_back(einsum::Claim{from_limbs(claim_points[r], claim_point_lens[r]), F(claim_evals[2 * r], claim_evals[2 * r + 1])});
            if (biases && biases[r])
                bts[r].reset(new einsum::Tensor(einsum::Tensor::from_unpadded(c, biases[r], shape_count(bias_shapes[r], bias_ranks[r]),
                                                                               std::vector<uint64_t>(bias_shapes[r], bias_shapes[r] + bias_ranks[r]))));
        }
        if (biases)
            for (auto &b : bts) bptr.push_back(b.get());
        write_einsum(einsum::prove_internal(c, ops, lt, rts, claims, t->t, bptr), out, out_cap, n_words);
    });
}

int32_t dph_einsum_prove_resident(dps_ctx *ctx, uint32_t n_ops, const char *const *labels, const dps_mle *lhs,
                                  const uint64_t *lhs_shape, uint32_t lhs_rank, const dps_mle *const *rhs,
                                  const uint64_t *const *rhs_shapes, const uint32_t *rhs_ranks,
                                  const dps_mle *const *biases, const uint64_t *const *bias_shapes, const uint32_t *bias_ranks,
                                  const uint64_t *const *claim_points, const uint32_t *claim_point_lens,
                                  const uint64_t *claim_evals, dph_transcript *t, uint64_t *out, uint64_t out_cap,
                                  uint64_t *n_words)
{
    return guarded([&] {
        Context c(ctx);
        std::vector<einsum::Op> ops;
        std::vector<einsum::Tensor> rts;
        std::vector<einsum::Claim> claims;
        std::vector<std::unique_ptr<einsum::Tensor>> bts(n_ops);
        std::vector<const einsum::Tensor *> bptr;
        einsum::Tensor lt = einsum::Tensor::resident(c, lhs, std::vector<uint64_t>(lhs_shape, lhs_shape + lhs_rank));
        for (uint32_t r = 0; r < n_ops; r++) {
            ops.push_back(einsum::Op{labels[4 * r], labels[4 * r + 1], labels[4 * r + 2], labels[4 * r + 3]});
            rts.push_back(einsum::Tensor::resident(c, rhs[r], std::vector<uint64_t>(rhs_shapes[r], rhs_shapes[r] + rhs_ranks[r])));
            claims.push_back(einsum::Claim{from_limbs(claim_points[r], claim_point_lens[r]), F(claim_evals[2 * r], claim_evals[2 * r + 1])});
            if (biases && biases[r])
                bts[r].reset(new einsum::Tensor(einsum::Tensor::resident(c, biases[r], std::vector<uint64_t>(bias_shapes[r], bias_shapes[r] + bias_ranks[r]))));
        }
        if (biases)
            for (auto &b : bts) bptr.push_back(b.get());
        write_einsum(einsum::prove_internal(c, ops, lt, rts, claims, t->t, bptr), out, out_cap, n_words);
    });
}

int32_t dph_logup_batch_prove(dps_ctx *ctx, uint32_t n_inst, const uint32_t *n_cols, const dps_mle *const *cols,
                              const dps_mle *const *numer, const uint64_t *cs, const uint64_t *betas,
                              dph_transcript *t, uint64_t *out, uint64_t out_cap, uint64_t *n_elems)
{
    return guarded([&] {
        Context c(ctx);
        // borrowed wrappers around the caller's handles: views share the storage and free only themselves
        std::vector<std::unique_ptr<DensePolynomial>> keep;
        auto borrow = [&](const dps_mle *h) {
            uint64_t len = 0;
            dps_mle_info(h, nullptr, &len);
            dps_mle *v = nullptr;
            c.check(dps_mle_view(h, 0, DensePolynomial::log2_strict(len), &v), "dps_mle_view");
            keep.emplace_back(new DensePolynomial(c, v));
            return keep.back().get();
        };
        std::vector<logup::LogUpInput> inputs;
        size_t k = 0;
        for (uint32_t i = 0; i < n_inst; i++) {
            std::vector<const DensePolynomial *> cl;
            for (uint32_t j = 0; j < n_cols[i]; j++) cl.push_back(borrow(cols[k++]));
            F cc(cs[2 * i], cs[2 * i + 1]), bb(betas[2 * i], betas[2 * i + 1]);
            if (numer)
                inputs.push_back(logup::LogUpInput::new_table(cl, borrow(numer[i]), cc, bb));
            else
                inputs.push_back(logup::LogUpInput::new_lookup(cl, cc, bb, n_cols[i]));
        }
        auto proof = logup::new_batch_multiple_sizes_prove(c, inputs, t->t);
        std::vector<uint64_t> w;
        auto put = [&](const F &x) {
            w.push_back(x.c0);
            w.push_back(x.c1);
        };
        for (size_t v = 0; v < proof.sumcheck_proofs.size(); v++) {
            for (auto &m : proof.sumcheck_proofs[v].proofs) {
                if (m.evaluations.size() != 4) throw Error(DPS_ERR_INVALID, "LogUp round message is not degree 3");
                for (auto &e : m.evaluations) put(e);
            }
            for (auto &e : proof.round_evaluations[v]) put(e);
        }
        for (auto &cl : proof.output_claims) put(cl.eval);
        for (auto &o : proof.circuit_outputs)
            for (auto &e : o) put(e);
        for (auto &x : proof.output_claims[0].point) put(x);
        if (w.size() > 2 * out_cap) throw Error(DPS_ERR_INVALID, "dph_logup_batch_prove: output buffer too small");
        memcpy(out, w.data(), w.size() * 8);
        *n_elems = w.size() / 2;
    });
}

int32_t dph_logup_batch_verify(uint32_t n_inst, const uint32_t *n_cols, const uint32_t *inst_nvars, const uint64_t *cs,
                               const uint64_t *betas, int32_t is_table, const uint64_t *stream, uint64_t n_elems,
                               dph_transcript *t, uint64_t *claims_out, uint64_t *point_out)
{
    return guarded([&] {
        std::vector<logup::LogUpVerifierInstance> inst(n_inst);
        size_t total = 0;
        for (uint32_t i = 0; i < n_inst; i++) {
            inst[i].constant_challenge = F(cs[2 * i], cs[2 * i + 1]);
            inst[i].column_separation_challenge = F(betas[2 * i], betas[2 * i + 1]);
            inst[i].num_columns = n_cols[i];
            inst[i].instance_type = is_table ? logup::ProofType::Table : logup::ProofType::Lookup;
            inst[i].num_vars = inst_nvars[i];
            total = std::max<size_t>(total, inst_nvars[i]);
        }
        auto all = from_limbs(stream, n_elems);
        size_t pos = 0;
        auto take = [&](size_t n) {
            if (pos + n > all.size()) throw Error(DPS_ERR_INVALID, "LogUp proof stream too short");
            std::vector<F> v(all.begin() + pos, all.begin() + pos + n);
            pos += n;
            return v;
        };
        logup::LogUpBatchProof proof;
        proof.proof_type = is_table ? logup::ProofType::Table : logup::ProofType::Lookup;
        for (size_t v = 1; v <= total; v++) {
            IOPProof p;
            for (size_t j = 0; j < v; j++) p.proofs.push_back(IOPProverMessage{take(4)});
            proof.sumcheck_proofs.push_back(std::move(p));
            const size_t remaining = total - (v - 1);
            size_t ne = 0;
            for (auto &in : inst)
                if (in.num_vars >= remaining) ne += (v == total) ? in.num_final_round_evals() : 4;
            proof.round_evaluations.push_back(take(ne));
        }
        size_t n_claims = 0;
        for (auto &in : inst) n_claims += in.num_columns + (is_table ? 1 : 0);
        take(n_claims);  // the prover's own claim evaluations are recomputed below
        for (uint32_t i = 0; i < n_inst; i++) proof.circuit_outputs.push_back(take(4));
        auto res = logup::new_verify_logup_proof_multiple_sizes(proof, inst, t->t);
        for (size_t i = 0; i < res.output_claims.size(); i++) {
            claims_out[2 * i] = res.output_claims[i].eval.c0;
            claims_out[2 * i + 1] = res.output_claims[i].eval.c1;
        }
        for (size_t i = 0; i < res.point.size(); i++) {
            point_out[2 * i] = res.point[i].c0;
            point_out[2 * i + 1] = res.point[i].c1;
        }
    });
}

namespace {

// claim lists from the flat arrays of the C interface; poly_vars[p] = variables of polynomial p
std::vector<std::vector<poly_commit::Claim>> read_claims(uint32_t n_polys, const std::vector<size_t> &poly_vars, const uint32_t *claims_per_poly,
                                                         const uint64_t *points, const uint64_t *evals)
{
    std::vector<std::vector<poly_commit::Claim>> claims(n_polys);
    size_t pw = 0, ci = 0;
    for (uint32_t p = 0; p < n_polys; p++)
        for (uint32_t k = 0; k < claims_per_poly[p]; k++) {
            poly_commit::Claim cl;
            cl.point = from_limbs(points + pw, poly_vars[p]);
            pw += 2 * poly_vars[p];
            cl.eval = F(evals[2 * ci], evals[2 * ci + 1]);
            ci++;
            claims[p].push_back(std::move(cl));
        }
    return claims;
}

}  // namespace

int32_t dph_claims_batching_prove(dps_ctx *ctx, uint32_t n_polys, const uint32_t *chunks_per_poly, const dps_mle *const *chunks,
                                  const uint32_t *claims_per_poly, const uint64_t *points, const uint64_t *evals,
                                  dph_transcript *t, uint64_t *proof_out, uint64_t *point_out, uint64_t *evals_out,
                                  uint32_t *n_vars_out)
{
    return guarded([&] {
        Context c(ctx);
        std::vector<std::unique_ptr<DensePolynomial>> keep;
        std::vector<poly_commit::CommittedPoly> polys(n_polys);
        std::vector<size_t> poly_vars(n_polys);
        size_t k = 0;
        for (uint32_t p = 0; p < n_polys; p++) {
            for (uint32_t j = 0; j < chunks_per_poly[p]; j++) {
                uint64_t len = 0;
                dps_mle_info(chunks[k], nullptr, &len);
                dps_mle *v = nullptr;
                c.check(dps_mle_view(chunks[k], 0, DensePolynomial::log2_strict(len), &v), "dps_mle_view");
                keep.emplace_back(new DensePolynomial(c, v));
                polys[p].chunks.push_back(keep.back().get());
                k++;
            }
            if (polys[p].chunks.empty()) throw Error(DPS_ERR_INVALID, "a committed polynomial needs at least one chunk");
            poly_vars[p] = polys[p].num_vars();
        }
        auto claims = read_claims(n_polys, poly_vars, claims_per_poly, points, evals);
        auto proof = poly_commit::claims_batching_sumcheck(c, polys, claims, t->t);
        size_t w = 0;
        for (auto &m : proof.sumcheck_proof.proofs) {
            if (m.evaluations.size() != 3) throw Error(DPS_ERR_INVALID, "claims batching round message is not degree 2");
            for (auto &e : m.evaluations) {
                proof_out[w++] = e.c0;
                proof_out[w++] = e.c1;
            }
        }
        for (size_t i = 0; i < proof.sumcheck_point.size(); i++) {
            point_out[2 * i] = proof.sumcheck_point[i].c0;
            point_out[2 * i + 1] = proof.sumcheck_point[i].c1;
        }
        for (size_t i = 0; i < proof.sumcheck_evals.size(); i++) {
            evals_out[2 * i] = proof.sumcheck_evals[i].c0;
            evals_out[2 * i + 1] = proof.sumcheck_evals[i].c1;
        }
        *n_vars_out = (uint32_t)proof.sumcheck_point.size();
    });
}

int32_t dph_claims_batching_verify(uint32_t n_polys, const uint32_t *chunks_per_poly, const uint32_t *poly_vars,
                                   const uint32_t *claims_per_poly, const uint64_t *points, const uint64_t *evals,
                                   const uint64_t *proof, uint32_t n_vars, const uint64_t *sumcheck_evals,
                                   dph_transcript *t, uint64_t *point_out)
{
    return guarded([&] {
        std::vector<poly_commit::CommitmentShape> shapes;
        std::vector<size_t> pv(n_polys);
        size_t total_chunks = 0;
        for (uint32_t p = 0; p < n_polys; p++) {
            shapes.push_back(poly_commit::CommitmentShape{chunks_per_poly[p], poly_vars[p]});
            pv[p] = poly_vars[p];
            total_chunks += chunks_per_poly[p];
        }
        auto claims = read_claims(n_polys, pv, claims_per_poly, points, evals);
        IOPProof pr;
        for (uint32_t j = 0; j < n_vars; j++) pr.proofs.push_back(IOPProverMessage{from_limbs(proof + 6 * (size_t)j, 3)});
        auto point = poly_commit::claims_batching_verify(shapes, claims, pr, from_limbs(sumcheck_evals, total_chunks), t->t);
        for (size_t i = 0; i < point.size(); i++) {
            point_out[2 * i] = point[i].c0;
            point_out[2 * i + 1] = point[i].c1;
        }
    });
}

int32_t dph_same_poly_prove(dps_ctx *ctx, const dps_mle *poly, uint32_t n_claims, const uint64_t *points, const uint64_t *evals,
                            dph_transcript *t, uint64_t *proof_out, uint64_t *point_out, uint64_t *eval_out)
{
    return guarded([&] {
        Context c(ctx);
        uint64_t len = 0;
        dps_mle_info(poly, nullptr, &len);
        const uint32_t nv = DensePolynomial::log2_strict(len);
        dps_mle *v = nullptr;
        c.check(dps_mle_view(poly, 0, nv, &v), "dps_mle_view");
        DensePolynomial p(c, v);
        same_poly::Prover prover(p);
        for (uint32_t i = 0; i < n_claims; i++)
            prover.add_claim(same_poly::Claim{from_limbs(points + 2 * (size_t)nv * i, nv), F(evals[2 * i], evals[2 * i + 1])});
        auto res = prover.prove(t->t);
        size_t w = 0;
        for (auto &m : res.first.sumcheck.proofs) {
            if (m.evaluations.size() != 3) throw Error(DPS_ERR_INVALID, "same_poly round message is not degree 2");
            for (auto &e : m.evaluations) {
                proof_out[w++] = e.c0;
                proof_out[w++] = e.c1;
            }
        }
        for (size_t i = 0; i < res.second.point.size(); i++) {
            point_out[2 * i] = res.second.point[i].c0;
            point_out[2 * i + 1] = res.second.point[i].c1;
        }
        eval_out[0] = res.second.eval.c0;
        eval_out[1] = res.second.eval.c1;
    });
}

int32_t dph_same_poly_verify(uint32_t num_vars, uint32_t n_claims, const uint64_t *points, const uint64_t *evals, const uint64_t *proof,
                             const uint64_t *eval, dph_transcript *t, uint64_t *point_out)
{
    return guarded([&] {
        same_poly::Context sctx(num_vars);
        same_poly::Verifier verifier(sctx);
        for (uint32_t i = 0; i < n_claims; i++)
            verifier.add_claim(same_poly::Claim{from_limbs(points + 2 * (size_t)num_vars * i, num_vars), F(evals[2 * i], evals[2 * i + 1])});
        same_poly::Proof pr;
        for (uint32_t j = 0; j < num_vars; j++) pr.sumcheck.proofs.push_back(IOPProverMessage{from_limbs(proof + 6 * (size_t)j, 3)});
        pr.eval = F(eval[0], eval[1]);
        auto claim = verifier.verify(pr, t->t);
        for (size_t i = 0; i < claim.point.size(); i++) {
            point_out[2 * i] = claim.point[i].c0;
            point_out[2 * i + 1] = claim.point[i].c1;
        }
    });
}

namespace {

lookup::LookupInputConfig linking_config(const dph_linking_config *cfg)
{
    if (!cfg || !cfg->unpadded_input_shape || cfg->rank == 0) throw Error(DPS_ERR_INVALID, "linking sumcheck: null configuration");
    if (cfg->variant < 0 || cfg->variant > 3) throw Error(DPS_ERR_INVALID, "linking sumcheck: unknown variant");
    lookup::ChunkingInfo ci;
    ci.number_of_value_chunks = cfg->number_of_value_chunks;
    ci.number_of_zeroing_chunks = cfg->number_of_zeroing_chunks;
    ci.table_bit_size = cfg->table_bit_size;
    ci.table_is_signed = cfg->table_is_signed != 0;
    ci.min_output_value = cfg->min_output_value;
    ci.max_output_value = cfg->max_output_value;
    ci.input_sign = cfg->input_sign_negative ? lookup::TableSign::Negative : lookup::TableSign::Positive;
    lookup::LookupVariant v;
    v.kind = (lookup::Variant)cfg->variant;
    v.normalised_sum = cfg->normalised_sum != 0;
    v.has_weight = cfg->has_weight != 0;
    return lookup::LookupInputConfig(ci, v, std::vector<uint64_t>(cfg->unpadded_input_shape, cfg->unpadded_input_shape + cfg->rank));
}

}  // namespace

int32_t dph_linking_prove(dps_ctx *ctx, const dph_linking_config *cfg, const dps_mle *const *mles, uint32_t n_mles, const dps_mle *weight,
                          const uint64_t *last_claim_point, uint32_t last_claim_len, const uint64_t *logup_point, uint32_t logup_len,
                          dph_transcript *t, uint64_t *out, uint64_t out_cap, uint64_t *n_words)
{
    return guarded([&] {
        Context c(ctx);
        auto config = linking_config(cfg);
        std::vector<DensePolynomial> tabs;
        tabs.reserve(n_mles + 1);
        for (uint32_t i = 0; i < n_mles; i++) tabs.push_back(DensePolynomial::borrowed(c, mles[i]));
        if (weight) tabs.push_back(DensePolynomial::borrowed(c, weight));
        std::vector<const DensePolynomial *> ptrs;
        for (uint32_t i = 0; i < n_mles; i++) ptrs.push_back(&tabs[i]);
        auto res = config.prove_linking_sumcheck(ptrs, t->t, from_limbs(last_claim_point, last_claim_len), from_limbs(logup_point, logup_len),
                                                 weight ? &tabs.back() : nullptr);
        std::vector<uint64_t> w;
        auto put = [&](const F &x) {
            w.push_back(x.c0);
            w.push_back(x.c1);
        };
        const auto &pr = res.first;
        w.push_back(pr.sumcheck_proof.proofs.size());
        w.push_back(pr.sumcheck_proof.proofs.empty() ? 0 : pr.sumcheck_proof.proofs[0].evaluations.size());
        for (auto &m : pr.sumcheck_proof.proofs)
            for (auto &e : m.evaluations) put(e);
        w.push_back(pr.evaluations.size());
        for (auto &e : pr.evaluations) put(e);
        w.push_back(pr.has_weight_eval ? 1 : 0);
        if (pr.has_weight_eval) put(pr.weight_eval);
        for (auto &x : pr.sumcheck_point) put(x);
        w.push_back(res.second.size());
        for (auto &x : res.second) put(x);
        if (w.size() > out_cap) throw Error(DPS_ERR_INVALID, "dph_linking_prove: output buffer too small");
        memcpy(out, w.data(), w.size() * 8);
        *n_words = w.size();
    });
}

int32_t dph_linking_verify(const dph_linking_config *cfg, const uint64_t initial_claim[2], const uint64_t *proof, uint32_t n_rounds,
                           uint32_t points_per_round, const uint64_t *evaluations, uint32_t n_evaluations, const uint64_t *weight_eval,
                           const uint64_t *last_claim_point, uint32_t last_claim_len, const uint64_t *logup_point, uint32_t logup_len,
                           dph_transcript *t, uint64_t *point_out)
{
    return guarded([&] {
        auto config = linking_config(cfg);
        lookup::LookupSumcheckProof pr;
        for (uint32_t j = 0; j < n_rounds; j++)
            pr.sumcheck_proof.proofs.push_back(IOPProverMessage{from_limbs(proof + 2 * (size_t)points_per_round * j, points_per_round)});
        pr.evaluations = from_limbs(evaluations, n_evaluations);
        if (weight_eval) {
            pr.has_weight_eval = true;
            pr.weight_eval = F(weight_eval[0], weight_eval[1]);
        }
        auto res = config.verify_linking_sumcheck(pr, F(initial_claim[0], initial_claim[1]), t->t, from_limbs(last_claim_point, last_claim_len),
                                                  from_limbs(logup_point, logup_len));
        for (size_t i = 0; i < res.second.size(); i++) {
            point_out[2 * i] = res.second[i].c0;
            point_out[2 * i + 1] = res.second[i].c1;
        }
    });
}

}  // extern "C"
