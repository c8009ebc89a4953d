// Symbolic sum-of-products over registered tables, mirroring the Expression type
// the reference's provers build (WitIn / Constant / Challenge with + - *):
// zkml/src/layers/einsum/op_info.rs:137-199, zkml/src/lookup/logup_gkr/circuit.rs:245-284,
// zkml/src/iop/same_poly.rs:94-104.  Challenge(id, pow, scalar, offset) evaluates to
// scalar * challenges[id]^pow + offset.
#pragma once
#include <algorithm>
#include <map>
#include <memory>
#include <stdexcept>
#include <vector>

#include "field.hpp"

namespace dpsc {

struct Monomial {
    F coeff;
    std::vector<uint16_t> wits;  // sorted table indices, repeats allowed
};

class Expression {
public:
    enum class Kind { WitIn, Constant, Challenge, Sum, Product, Neg };

    static Expression WitIn(uint16_t id)
    {
        Expression e(Kind::WitIn);
        e.n_->id = id;
        return e;
    }
    static Expression Constant(const F &c)
    {
        Expression e(Kind::Constant);
        e.n_->scalar = c;
        return e;
    }
    static Expression Challenge(uint16_t id, size_t pow, const F &scalar, const F &offset)
    {
        Expression e(Kind::Challenge);
        e.n_->id = id;
        e.n_->pow = pow;
        e.n_->scalar = scalar;
        e.n_->offset = offset;
        return e;
    }
    static Expression ZERO() { return Constant(F::zero()); }
    static Expression ONE() { return Constant(F::one()); }

    Expression operator+(const Expression &o) const { return binary(Kind::Sum, o); }
    Expression operator*(const Expression &o) const { return binary(Kind::Product, o); }
    Expression operator-(const Expression &o) const { return *this + (-o); }
    Expression operator-() const
    {
        Expression e(Kind::Neg);
        e.n_->a = n_;
        return e;
    }

    // Flatten to monomials with the challenges substituted.  Equal products of
    // tables are merged; monomials whose coefficient cancels to zero are dropped.
    std::vector<Monomial> to_monomials(const std::vector<F> &challenges) const
    {
        std::map<std::vector<uint16_t>, F> acc;
        for (auto &m : expand(*n_, challenges)) {
            auto it = acc.find(m.wits);
            if (it == acc.end())
                acc.emplace(m.wits, m.coeff);
            else
                it->second += m.coeff;
        }
        std::vector<Monomial> out;
        for (auto &kv : acc)
            if (!kv.second.is_zero()) out.push_back(Monomial{kv.second, kv.first});
        return out;
    }

    // utils::eval_by_expr_with_instance restricted to what the callers pass:
    // witness evaluations and challenges (zkml/src/lookup/logup_gkr/prover.rs:43-58)
    F evaluate(const std::vector<F> &wit_evals, const std::vector<F> &challenges) const { return eval(*n_, wit_evals, challenges); }

    size_t degree() const
    {
        size_t d = 0;
        for (auto &m : to_monomials_symbolic()) d = std::max(d, m);
        return d;
    }

private:
    struct Node {
        Kind kind;
        uint16_t id = 0;
        size_t pow = 0;
        F scalar, offset;
        std::shared_ptr<const Node> a, b;
    };
    std::shared_ptr<Node> n_;
    explicit Expression(Kind k) : n_(std::make_shared<Node>()) { n_->kind = k; }
    Expression binary(Kind k, const Expression &o) const
    {
        Expression e(k);
        e.n_->a = n_;
        e.n_->b = o.n_;
        return e;
    }
    static F challenge_value(const Node &n, const std::vector<F> &ch)
    {
        if (n.id >= ch.size()) throw std::out_of_range("Expression: challenge index out of range");
        return n.scalar * ch[n.id].pow(n.pow) + n.offset;
    }
    static std::vector<Monomial> expand(const Node &n, const std::vector<F> &ch)
    {
        std::vector<Monomial> out;
        expand_into(n, F::one(), ch, out);
        return out;
    }
    // appends scale * (the node's monomials) to `out`: long sums (one `+` per term, as the provers build them)
    // cost one pass, not one copy of everything so far per `+`
    static void expand_into(const Node &n, const F &scale, const std::vector<F> &ch, std::vector<Monomial> &out)
    {
        if (scale.is_zero()) return;
        switch (n.kind) {
        case Kind::WitIn: out.push_back(Monomial{scale, {n.id}}); return;
        case Kind::Constant:
            if (!n.scalar.is_zero()) out.push_back(Monomial{scale * n.scalar, {}});
            return;
        case Kind::Challenge: {
            const F c = challenge_value(n, ch);
            if (!c.is_zero()) out.push_back(Monomial{scale * c, {}});
            return;
        }
        case Kind::Neg: expand_into(*n.a, -scale, ch, out); return;
        case Kind::Sum:
            expand_into(*n.a, scale, ch, out);
            expand_into(*n.b, scale, ch, out);
            return;
        case Kind::Product: {
            std::vector<Monomial> v, w;
            expand_into(*n.a, F::one(), ch, v);
            expand_into(*n.b, scale, ch, w);
            out.reserve(out.size() + v.size() * w.size());
            for (auto &x : v)
                for (auto &y : w) {
                    Monomial m{x.coeff * y.coeff, x.wits};
                    if (m.coeff.is_zero()) continue;
                    m.wits.insert(m.wits.end(), y.wits.begin(), y.wits.end());
                    std::sort(m.wits.begin(), m.wits.end());
                    out.push_back(std::move(m));
                }
            return;
        }
        }
    }
    static F eval(const Node &n, const std::vector<F> &w, const std::vector<F> &ch)
    {
        switch (n.kind) {
        case Kind::WitIn:
            if (n.id >= w.size()) throw std::out_of_range("Expression: witness index out of range");
            return w[n.id];
        case Kind::Constant: return n.scalar;
        case Kind::Challenge: return challenge_value(n, ch);
        case Kind::Neg: return -eval(*n.a, w, ch);
        case Kind::Sum: return eval(*n.a, w, ch) + eval(*n.b, w, ch);
        case Kind::Product: return eval(*n.a, w, ch) * eval(*n.b, w, ch);
        }
        return F::zero();
    }
    std::vector<size_t> to_monomials_symbolic() const
    {
        std::vector<size_t> out;
        degrees(*n_, out);
        return out;
    }
    static void degrees(const Node &n, std::vector<size_t> &out)
    {
        switch (n.kind) {
        case Kind::WitIn: out.push_back(1); break;
        case Kind::Constant:
        case Kind::Challenge: out.push_back(0); break;
        case Kind::Neg: degrees(*n.a, out); break;
        case Kind::Sum:
            degrees(*n.a, out);
            degrees(*n.b, out);
            break;
        case Kind::Product: {
            std::vector<size_t> x, y;
            degrees(*n.a, x);
            degrees(*n.b, y);
            size_t mx = 0, my = 0;
            for (auto v : x) mx = std::max(mx, v);
            for (auto v : y) my = std::max(my, v);
            out.push_back(mx + my);
            break;
        }
        }
    }
};

}  // namespace dpsc
