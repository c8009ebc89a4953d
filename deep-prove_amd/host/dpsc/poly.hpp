// RAII wrappers over the C ABI for the table types the reference's provers hold:
// DensePolynomial (owned or borrowed view, zkml/src/tensor/mod.rs:364-401,
// zkml/src/lookup/logup_gkr/circuit.rs:262-269) and poly::eq::evals.
#pragma once
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/dpsumcheck.h"
#include "field.hpp"

namespace dpsc {

struct Error : std::runtime_error {
    int32_t status;
    Error(int32_t s, const std::string &what) : std::runtime_error(what), status(s) {}
};

// One GPU context (stream, memory pool).  Shared by every table created from it.
class Context {
public:
    explicit Context(int device = 0)
    {
        int32_t rc = dps_ctx_create(device, &ctx_);
        if (rc != DPS_OK) throw Error(rc, std::string("dps_ctx_create: ") + dps_status_str(rc));
    }
    // borrow a context created elsewhere (it is not destroyed with this object)
    explicit Context(dps_ctx *borrowed) : ctx_(borrowed), owned_(false) {}
    ~Context()
    {
        if (owned_) dps_ctx_destroy(ctx_);
    }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    dps_ctx *raw() const { return ctx_; }
    void check(int32_t rc, const char *what) const
    {
        if (rc != DPS_OK) throw Error(rc, std::string(what) + ": " + dps_status_str(rc) + " (" + dps_last_error(ctx_) + ")");
    }

private:
    dps_ctx *ctx_ = nullptr;
    bool owned_ = true;
};

class DensePolynomial {
public:
    DensePolynomial() = default;
    DensePolynomial(const Context &ctx, dps_mle *h) : ctx_(&ctx), h_(h, &dps_mle_free) {}
    // a handle the caller keeps alive and frees (tensors resident on the device across proofs)
    static DensePolynomial borrowed(const Context &ctx, const dps_mle *h)
    {
        DensePolynomial p;
        p.ctx_ = &ctx;
        p.h_ = decltype(p.h_)(const_cast<dps_mle *>(h), [](dps_mle *) { return 0; });
        return p;
    }
    // pad_next_power_of_two + to_field_mle of a raw tensor that is already on the device
    static DensePolynomial from_tensor(const Context &ctx, const DensePolynomial &tensor, const std::vector<uint64_t> &padded_shape,
                                       const std::vector<uint64_t> &unpadded_shape)
    {
        dps_mle *h = nullptr;
        ctx.check(dps_mle_from_tensor(ctx.raw(), tensor.raw(), padded_shape.data(), unpadded_shape.data(), (uint32_t)padded_shape.size(), &h),
                  "dps_mle_from_tensor");
        return DensePolynomial(ctx, h);
    }

    // DensePolynomial::new(Vec<F>) for base-field evaluations
    static DensePolynomial from_base(const Context &ctx, const std::vector<uint64_t> &evals)
    {
        dps_mle *h = nullptr;
        ctx.check(dps_mle_from_base(ctx.raw(), evals.data(), log2_strict(evals.size()), &h), "dps_mle_from_base");
        return DensePolynomial(ctx, h);
    }
    static DensePolynomial from_ext(const Context &ctx, const std::vector<F> &evals)
    {
        std::vector<uint64_t> c0(evals.size()), c1(evals.size());
        for (size_t i = 0; i < evals.size(); i++) {
            c0[i] = evals[i].c0;
            c1[i] = evals[i].c1;
        }
        dps_mle *h = nullptr;
        ctx.check(dps_mle_from_ext2(ctx.raw(), c0.data(), c1.data(), log2_strict(evals.size()), &h), "dps_mle_from_ext2");
        return DensePolynomial(ctx, h);
    }
    // Tensor<Element>::to_field_mle: embed and pad to a power of two
    static DensePolynomial from_i64(const Context &ctx, const std::vector<int64_t> &v)
    {
        uint32_t nv = 0;
        while ((size_t(1) << nv) < v.size()) nv++;
        dps_mle *h = nullptr;
        ctx.check(dps_mle_from_i64(ctx.raw(), v.data(), v.size(), nv, &h), "dps_mle_from_i64");
        return DensePolynomial(ctx, h);
    }
    // poly::eq::evals(point).into_mle()
    static DensePolynomial eq(const Context &ctx, const std::vector<F> &point)
    {
        auto limbs = to_limbs(point);
        dps_mle *h = nullptr;
        ctx.check(dps_eq_build(ctx.raw(), limbs.data(), (uint32_t)point.size(), &h), "dps_eq_build");
        return DensePolynomial(ctx, h);
    }
    // several eq tables built together (one launch for all the small ones)
    static std::vector<DensePolynomial> eq_many(const Context &ctx, const std::vector<std::vector<F>> &points)
    {
        std::vector<std::vector<uint64_t>> limbs;
        std::vector<const uint64_t *> ptrs;
        std::vector<uint32_t> m;
        limbs.reserve(points.size());
        for (auto &p : points) {
            limbs.push_back(to_limbs(p));
            m.push_back((uint32_t)p.size());
        }
        for (auto &l : limbs) ptrs.push_back(l.data());
        std::vector<dps_mle *> hs(points.size(), nullptr);
        ctx.check(dps_eq_build_many(ctx.raw(), ptrs.data(), m.data(), (uint32_t)points.size(), hs.data()), "dps_eq_build_many");
        std::vector<DensePolynomial> out;
        out.reserve(hs.size());
        for (auto *h : hs) out.emplace_back(ctx, h);
        return out;
    }
    // new_from_smart_slice(SmartSlice::Borrowed(&evals[offset..offset + 2^n_vars]))
    DensePolynomial view(uint64_t offset, uint32_t n_vars) const
    {
        dps_mle *h = nullptr;
        ctx_->check(dps_mle_view(h_.get(), offset, n_vars, &h), "dps_mle_view");
        return DensePolynomial(*ctx_, h);
    }
    // as_view() + zero_pad_num_vars(n) (zkml/src/poly_commit/prover.rs:214-226): the same storage, read by a
    // sumcheck over n variables as 0 wherever an added variable is 1
    DensePolynomial zero_pad_num_vars(uint32_t n_vars) const
    {
        dps_mle *h = nullptr;
        ctx_->check(dps_mle_zero_pad(h_.get(), n_vars, &h), "dps_mle_zero_pad");
        return DensePolynomial(*ctx_, h);
    }
    uint64_t len() const
    {
        uint64_t l = 0;
        dps_mle_info(h_.get(), nullptr, &l);
        return l;
    }
    uint32_t num_vars() const { return log2_strict(len()); }
    F evaluate(const std::vector<F> &point) const
    {
        auto limbs = to_limbs(point);
        uint64_t out[2];
        ctx_->check(dps_mle_evaluate(ctx_->raw(), h_.get(), limbs.data(), (uint32_t)point.size(), out), "dps_mle_evaluate");
        return F(out[0], out[1]);
    }
    DensePolynomial fix_high_variables(const std::vector<F> &point) const
    {
        auto limbs = to_limbs(point);
        dps_mle *h = nullptr;
        ctx_->check(dps_mle_fix_high(ctx_->raw(), h_.get(), limbs.data(), (uint32_t)point.size(), &h), "dps_mle_fix_high");
        return DensePolynomial(*ctx_, h);
    }
    DensePolynomial fix_low_variables(const std::vector<F> &point) const
    {
        auto limbs = to_limbs(point);
        dps_mle *h = nullptr;
        ctx_->check(dps_mle_fix_low(ctx_->raw(), h_.get(), limbs.data(), (uint32_t)point.size(), &h), "dps_mle_fix_low");
        return DensePolynomial(*ctx_, h);
    }
    std::vector<F> evals() const
    {
        uint64_t n = len();
        std::vector<uint64_t> c0(n), c1(n);
        ctx_->check(dps_mle_download(h_.get(), c0.data(), c1.data()), "dps_mle_download");
        std::vector<F> out(n);
        for (uint64_t i = 0; i < n; i++) out[i] = F(c0[i], c1[i]);
        return out;
    }
    const dps_mle *raw() const { return h_.get(); }
    const Context &context() const { return *ctx_; }
    explicit operator bool() const { return (bool)h_; }

    static uint32_t log2_strict(uint64_t n)
    {
        uint32_t l = 0;
        while ((uint64_t(1) << l) < n) l++;
        if ((uint64_t(1) << l) != n) throw Error(DPS_ERR_INVALID, "length is not a power of two");
        return l;
    }

private:
    const Context *ctx_ = nullptr;
    std::shared_ptr<dps_mle> h_;
};

inline uint32_t ceil_log2(uint64_t n)
{
    uint32_t l = 0;
    while ((uint64_t(1) << l) < n) l++;
    return l;
}

}  // namespace dpsc
