// Fiat-Shamir transcript with the method set the reference's provers call
// (zkml/src/lib.rs:106-108,176-184; zkml/src/layers/einsum/prove.rs:158;
// zkml/src/lookup/logup_gkr/prover.rs:163-173,261,284-288).  The reference's
// Blake3Transcript byte format lives in its dp-crypto dependency and is not
// reproduced here; this one is:
//     state_0     = H(label padded with zeros to 32 bytes)
//     state_{k+1} = H(state_k || 28 zero bytes || be32(k) || payload)
// The sumcheck engine only needs the two-method Transcript interface below, so a
// host that owns the real transcript plugs it in without touching GPU code.
#pragma once
#include <string>
#include <vector>

#include "blake3.hpp"
#include "field.hpp"

namespace dpsc {

class Transcript {
public:
    virtual ~Transcript() = default;
    virtual void append_scalars(const F *xs, size_t n) = 0;
    virtual F challenge_scalar() = 0;
    virtual void append_u64(uint64_t x) = 0;
    virtual void append_message(const char *label) = 0;
    virtual void append_bytes(const uint8_t *data, size_t len) = 0;

    void append_scalars(const std::vector<F> &xs) { append_scalars(xs.data(), xs.size()); }
    F append_and_sample(const char *label)
    {
        append_message(label);
        return challenge_scalar();
    }
    // VectorTranscript::read_challenges (zkml/src/lib.rs:176-184)
    std::vector<F> read_challenges(size_t n)
    {
        std::vector<F> out(n);
        for (auto &c : out) c = challenge_scalar();
        return out;
    }
};

class Blake3Transcript final : public Transcript {
public:
    explicit Blake3Transcript(const char *label = "m2vec")
    {
        uint8_t padded[32] = {0};
        size_t n = strlen(label);
        memcpy(padded, label, n < 32 ? n : 32);
        Blake3::hash(padded, 32, state_);
        n_rounds_ = 0;
    }
    using Transcript::append_scalars;
    void append_message(const char *label) override
    {
        uint8_t padded[32] = {0};
        size_t n = strlen(label);
        memcpy(padded, label, n < 32 ? n : 32);
        absorb(padded, 32);
    }
    void append_bytes(const uint8_t *data, size_t len) override { absorb(data, len); }
    void append_u64(uint64_t x) override
    {
        uint8_t buf[32] = {0};
        for (int i = 0; i < 8; i++) buf[24 + i] = (uint8_t)(x >> (56 - 8 * i));
        absorb(buf, 32);
    }
    void append_scalar(const F &x)
    {
        uint8_t buf[16];
        for (int i = 0; i < 8; i++) {
            buf[i] = (uint8_t)(x.c1 >> (56 - 8 * i));
            buf[8 + i] = (uint8_t)(x.c0 >> (56 - 8 * i));
        }
        absorb(buf, 16);
    }
    void append_scalars(const F *xs, size_t n) override
    {
        append_message("begin_append_vector");
        for (size_t i = 0; i < n; i++) append_scalar(xs[i]);
        append_message("end_append_vector");
    }
    F challenge_scalar() override
    {
        absorb(nullptr, 0);
        uint64_t w0 = 0, w1 = 0;
        for (int i = 0; i < 8; i++) {
            w0 |= (uint64_t)state_[i] << (8 * i);
            w1 |= (uint64_t)state_[8 + i] << (8 * i);
        }
        return F(w0 % GOLDILOCKS_P, w1 % GOLDILOCKS_P);
    }
    const uint8_t *state() const { return state_; }
    uint32_t n_rounds() const { return n_rounds_; }

private:
    uint8_t state_[32];
    uint32_t n_rounds_;
    void absorb(const uint8_t *payload, size_t len)
    {
        uint8_t head[64] = {0};
        memcpy(head, state_, 32);
        head[60] = (uint8_t)(n_rounds_ >> 24);
        head[61] = (uint8_t)(n_rounds_ >> 16);
        head[62] = (uint8_t)(n_rounds_ >> 8);
        head[63] = (uint8_t)n_rounds_;
        if (len <= 64) {
            Blake3::hash_block_and(head, payload, len, state_);
        } else {
            Blake3 h;
            h.update(head, 64);
            h.update(payload, len);
            h.finalize(state_);
        }
        n_rounds_++;
    }
};

}  // namespace dpsc
