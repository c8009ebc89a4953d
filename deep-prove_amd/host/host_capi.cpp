// C wrappers over the C++ host mirror (see dpsc_host.h).
#include "dpsc_host.h"

#include <string>

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
    return guarded([&] {
        Context c(ctx);
        VirtualPolynomials vp;
        vp.ctx = &c;
        vp.num_vars = n_vars;
        vp.mles.assign(mles, mles + n_mles);
        vp.terms.assign(terms, terms + n_terms);
        auto res = IOPProverState::prove(vp, t->t);
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

}  // extern "C"
