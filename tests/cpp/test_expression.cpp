// CPU unit test of the host mirror's Expression: flattening to monomials agrees
// with direct evaluation, for the expressions the reference's provers build.
#include <cstdio>
#include <cstdlib>
#include <random>

#include "../../deep-prove_amd/host/dpsc/expression.hpp"

using namespace dpsc;

static std::mt19937_64 rng(42);
static F rnd() { return F(rng() % GOLDILOCKS_P, rng() % GOLDILOCKS_P); }

static F eval_monomials(const std::vector<Monomial> &ms, const std::vector<F> &w)
{
    F acc = F::zero();
    for (auto &m : ms) {
        F p = m.coeff;
        for (auto i : m.wits) p *= w[i];
        acc += p;
    }
    return acc;
}

static int check(const char *name, const Expression &e, size_t n_wits, size_t n_chal, size_t expect_degree)
{
    for (int rep = 0; rep < 5; rep++) {
        std::vector<F> w(n_wits), ch(n_chal);
        for (auto &x : w) x = rnd();
        for (auto &x : ch) x = rnd();
        auto ms = e.to_monomials(ch);
        if (eval_monomials(ms, w) != e.evaluate(w, ch)) {
            printf("FAIL %s: monomials disagree with evaluate\n", name);
            return 1;
        }
        size_t d = 0;
        for (auto &m : ms) d = std::max(d, m.wits.size());
        if (d != expect_degree) {
            printf("FAIL %s: degree %zu, expected %zu\n", name, d, expect_degree);
            return 1;
        }
    }
    printf("ok %s\n", name);
    return 0;
}

int main()
{
    int bad = 0;
    const F one = F::one(), zero = F::zero();
    // hadamard.rs:109-113: fold of Constant(1) * W0 * W1 * W2
    {
        Expression e = Expression::Constant(one);
        for (uint16_t i = 0; i < 3; i++) e = e * Expression::WitIn(i);
        bad += check("hadamard", e, 3, 0, 3);
    }
    // same_poly.rs:94-104: W0 * sum_i Challenge(i) * W_{i+1}
    {
        Expression sum = Expression::Constant(zero);
        for (uint16_t i = 0; i < 5; i++) sum = sum + Expression::Challenge(i, 1, one, zero) * Expression::WitIn(i + 1);
        bad += check("same_poly", Expression::WitIn(0) * sum, 6, 5, 2);
    }
    // op_info.rs:159-199 shape: sum_i chal^i * sum_j c_ij * W * W
    {
        Expression acc = Expression::ZERO();
        for (size_t i = 0; i < 2; i++) {
            Expression inner = Expression::Constant(rnd()) * Expression::WitIn((uint16_t)(3 * i)) * Expression::WitIn((uint16_t)(6 + 3 * i));
            for (size_t j = 1; j < 3; j++)
                inner = Expression::Constant(rnd()) * Expression::WitIn((uint16_t)(3 * i + j)) * Expression::WitIn((uint16_t)(6 + 3 * i + j)) + inner;
            acc = acc + Expression::Challenge(0, i, one, zero) * inner;
        }
        bad += check("einsum", acc, 12, 1, 2);
    }
    // circuit.rs:397-401: alpha^k * (-D_hi - D_lo + lambda * D_lo * D_hi) * eq with D = c + sum beta^i W_i
    {
        F c = rnd(), beta = rnd(), pw = one;
        Expression dlo = Expression::Constant(c), dhi = Expression::Constant(c);
        for (uint16_t i = 0; i < 2; i++) {
            dlo = dlo + Expression::Constant(pw) * Expression::WitIn(i);
            dhi = dhi + Expression::Constant(pw) * Expression::WitIn(2 + i);
            pw *= beta;
        }
        Expression e = Expression::Challenge(0, 3, one, zero) * (-dhi - dlo + Expression::Challenge(1, 1, one, zero) * dlo * dhi) * Expression::WitIn(4);
        bad += check("logup_lookup_input_layer", e, 5, 2, 3);
        // subtraction and cancellation: (W0 - W0) * W1 has no monomials
        Expression z = (Expression::WitIn(0) - Expression::WitIn(0)) * Expression::WitIn(1);
        if (!z.to_monomials({}).empty()) {
            printf("FAIL cancellation\n");
            bad++;
        }
    }
    // Challenge(id, pow, scalar, offset) = scalar * chal^pow + offset
    {
        F s = rnd(), o = rnd(), ch = rnd();
        Expression e = Expression::Challenge(0, 3, s, o);
        if (e.evaluate({}, {ch}) != s * ch * ch * ch + o) {
            printf("FAIL challenge semantics\n");
            bad++;
        }
    }
    return bad ? 1 : 0;
}
