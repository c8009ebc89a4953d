// Host-side Goldilocks / quadratic-extension arithmetic for the code that sits
// above the C ABI (transcript, expressions, claims, verifier).  Table-sized
// work never runs here: it goes through libdpsumcheck on the GPU.
#pragma once
#include <cstdint>
#include <vector>

namespace dpsc {

constexpr uint64_t GOLDILOCKS_P = 0xFFFFFFFF00000001ULL;

struct Fp {
    static uint64_t add(uint64_t a, uint64_t b)
    {
        unsigned __int128 s = (unsigned __int128)a + b;
        return (uint64_t)(s >= GOLDILOCKS_P ? s - GOLDILOCKS_P : s);
    }
    static uint64_t sub(uint64_t a, uint64_t b) { return a >= b ? a - b : a + (GOLDILOCKS_P - b); }
    static uint64_t neg(uint64_t a) { return a ? GOLDILOCKS_P - a : 0; }
    static uint64_t mul(uint64_t a, uint64_t b) { return (uint64_t)(((unsigned __int128)a * b) % GOLDILOCKS_P); }
    static uint64_t pow(uint64_t a, uint64_t e)
    {
        uint64_t r = 1;
        for (; e; e >>= 1, a = mul(a, a))
            if (e & 1) r = mul(r, a);
        return r;
    }
    static uint64_t inv(uint64_t a) { return pow(a, GOLDILOCKS_P - 2); }
    // F::from(i64) of the reference (zkml/src/quantization/mod.rs:262-266)
    static uint64_t from_i64(int64_t x) { return x >= 0 ? (uint64_t)x : GOLDILOCKS_P - ((uint64_t)0 - (uint64_t)x); }
};

// Element of F_p[X]/(X^2 - 7); the type the host mirror calls `F`.
struct F {
    uint64_t c0 = 0, c1 = 0;
    F() = default;
    F(uint64_t a, uint64_t b) : c0(a), c1(b) {}
    static F zero() { return F(0, 0); }
    static F one() { return F(1, 0); }
    static F from_u64(uint64_t x) { return F(x % GOLDILOCKS_P, 0); }
    static F from_i64(int64_t x) { return F(Fp::from_i64(x), 0); }
    F operator+(const F &o) const { return F(Fp::add(c0, o.c0), Fp::add(c1, o.c1)); }
    F operator-(const F &o) const { return F(Fp::sub(c0, o.c0), Fp::sub(c1, o.c1)); }
    F operator-() const { return F(Fp::neg(c0), Fp::neg(c1)); }
    F operator*(const F &o) const
    {
        return F(Fp::add(Fp::mul(c0, o.c0), Fp::mul(7, Fp::mul(c1, o.c1))), Fp::add(Fp::mul(c0, o.c1), Fp::mul(c1, o.c0)));
    }
    F &operator+=(const F &o) { return *this = *this + o; }
    F &operator-=(const F &o) { return *this = *this - o; }
    F &operator*=(const F &o) { return *this = *this * o; }
    bool operator==(const F &o) const { return c0 == o.c0 && c1 == o.c1; }
    bool operator!=(const F &o) const { return !(*this == o); }
    bool is_zero() const { return c0 == 0 && c1 == 0; }
    F inverse() const
    {
        uint64_t n = Fp::inv(Fp::sub(Fp::mul(c0, c0), Fp::mul(7, Fp::mul(c1, c1))));
        return F(Fp::mul(c0, n), Fp::mul(Fp::neg(c1), n));
    }
    F pow(uint64_t e) const
    {
        F r = one(), a = *this;
        for (; e; e >>= 1, a = a * a)
            if (e & 1) r = r * a;
        return r;
    }
};

// layout used when elements cross the C ABI: (c0, c1) pairs
inline std::vector<uint64_t> to_limbs(const std::vector<F> &v)
{
    std::vector<uint64_t> o(2 * v.size());
    for (size_t i = 0; i < v.size(); i++) {
        o[2 * i] = v[i].c0;
        o[2 * i + 1] = v[i].c1;
    }
    return o;
}
inline std::vector<F> from_limbs(const uint64_t *p, size_t n)
{
    std::vector<F> o(n);
    for (size_t i = 0; i < n; i++) o[i] = F(p[2 * i], p[2 * i + 1]);
    return o;
}

// poly_commit::identity_eval (zkml/src/poly_commit/mod.rs:184-192)
inline F identity_eval(const F *r1, const F *r2, size_t n)
{
    F acc = F::one();
    for (size_t i = 0; i < n; i++) acc *= r1[i] * r2[i] + (F::one() - r1[i]) * (F::one() - r2[i]);
    return acc;
}

// poly::eq::evals for the short points host code needs (stacking coefficients)
inline std::vector<F> eq_evals_host(const F *point, size_t m)
{
    std::vector<F> t(size_t(1) << m);
    t[0] = F::one();
    size_t len = 1;
    for (size_t jj = m; jj-- > 0;) {
        F r = point[jj], nr = F::one() - r;
        for (size_t i = len; i-- > 0;) {
            F v = t[i];
            t[2 * i + 1] = v * r;
            t[2 * i] = v * nr;
        }
        len <<= 1;
    }
    return t;
}

// value at r of the polynomial with the given evaluations at 0..d
inline F interpolate_uni(const F *evals, size_t d, const F &r)
{
    F acc = F::zero();
    for (size_t k = 0; k <= d; k++) {
        F num = F::one();
        uint64_t den = 1;
        for (size_t m = 0; m <= d; m++) {
            if (m == k) continue;
            num *= r - F::from_u64(m);
            den = Fp::mul(den, Fp::sub(k, m));
        }
        acc += num * F(Fp::inv(den), 0) * evals[k];
    }
    return acc;
}

}  // namespace dpsc
