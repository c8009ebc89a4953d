// BLAKE3 in hash mode (32-byte digest), incremental.  Written from the published
// specification; the reference gets it from the `blake3` crate via dp-crypto.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#if defined(__x86_64__)
#include <immintrin.h>
#endif

namespace dpsc {

namespace blake3_detail {
// per round, where a 512-bit permute finds the sixteen message words: the first words of the column step's four G
// functions, their second words, then the same for the diagonal step
struct RoundIndex {
    alignas(64) uint32_t idx[7][16];
};
inline constexpr RoundIndex make_round_index()
{
    constexpr uint8_t S[7][16] = {
        {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8},
        {3, 4, 10, 12, 13, 2, 7, 14, 6, 5, 9, 0, 11, 15, 8, 1}, {10, 7, 12, 9, 14, 3, 13, 15, 4, 0, 11, 2, 5, 8, 1, 6},
        {12, 13, 9, 11, 15, 10, 14, 8, 7, 2, 5, 3, 0, 1, 6, 4}, {9, 14, 11, 5, 8, 12, 15, 1, 13, 3, 0, 10, 2, 6, 4, 7},
        {11, 15, 5, 0, 1, 9, 8, 6, 14, 10, 2, 12, 3, 4, 7, 13}};
    RoundIndex r{};
    for (int k = 0; k < 7; k++)
        for (int i = 0; i < 4; i++) {
            r.idx[k][i] = S[k][2 * i];           // first words of the column step's four G
            r.idx[k][4 + i] = S[k][2 * i + 1];   // their second words
            r.idx[k][8 + i] = S[k][8 + 2 * i];   // the diagonal step's
            r.idx[k][12 + i] = S[k][9 + 2 * i];
        }
    return r;
}
inline constexpr RoundIndex ROUND_INDEX = make_round_index();
}  // namespace blake3_detail

class Blake3 {
public:
    Blake3() { reset(); }
    void reset()
    {
        memcpy(cv_, IV, sizeof cv_);
        buf_len_ = 0;
        blocks_ = 0;
        chunk_ = 0;
        stack_len_ = 0;
    }
    Blake3 &update(const void *data, size_t len)
    {
        const uint8_t *p = (const uint8_t *)data;
        while (len) {
            if (chunk_len() == 1024) {
                // the current chunk is complete and more input follows: finish it as a non-root chunk
                uint32_t out[16];
                compress(cv_, buf_, chunk_, 64, flags_for_block() | CHUNK_END, out);
                push_cv(out);
                memcpy(cv_, IV, sizeof cv_);
                buf_len_ = 0;
                blocks_ = 0;
                chunk_++;
            }
            if (buf_len_ == 64) {
                uint32_t out[16];
                compress(cv_, buf_, chunk_, 64, flags_for_block(), out);
                memcpy(cv_, out, sizeof cv_);
                blocks_++;
                buf_len_ = 0;
            }
            size_t take = 64 - buf_len_;
            if (take > len) take = len;
            memcpy(buf_ + buf_len_, p, take);
            buf_len_ += take;
            p += take;
            len -= take;
        }
        return *this;
    }
    void finalize(uint8_t out[32]) const
    {
        // last block of the current chunk, then fold the stack from the top
        uint8_t block[64] = {0};
        memcpy(block, buf_, buf_len_);
        uint32_t cv[8], o[16];
        uint32_t flags = flags_for_block() | CHUNK_END;
        if (stack_len_ == 0) {
            compress(cv_, block, chunk_, (uint32_t)buf_len_, flags | ROOT, o);
        } else {
            compress(cv_, block, chunk_, (uint32_t)buf_len_, flags, o);
            memcpy(cv, o, sizeof cv);
            for (size_t i = stack_len_; i-- > 0;) {
                uint8_t parent[64];
                words_to_bytes(stack_[i], parent);
                words_to_bytes(cv, parent + 32);
                compress(IV, parent, 0, 64, PARENT | (i == 0 ? ROOT : 0u), o);
                memcpy(cv, o, sizeof cv);
            }
        }
        words_to_bytes(o, out);
    }
    static void hash(const void *data, size_t len, uint8_t out[32])
    {
        Blake3 h;
        h.update(data, len);
        h.finalize(out);
    }
    // The digest of a 64-byte block followed by at most 64 more bytes (one chunk of two blocks), without the incremental
    // hasher's buffering: the shape of every transcript step, which sits between two GPU round trips.
    static void hash_block_and(const uint8_t head[64], const uint8_t *tail, size_t tail_len, uint8_t out[32])
    {
        uint32_t cv[16], o[16];
        if (tail_len == 0) {
            compress(IV, head, 0, 64, CHUNK_START | CHUNK_END | ROOT, o);
        } else {
            uint8_t block[64] = {0};
            memcpy(block, tail, tail_len);
            compress(IV, head, 0, 64, CHUNK_START, cv);
            compress(cv, block, 0, (uint32_t)tail_len, CHUNK_END | ROOT, o);
        }
        words_to_bytes(o, out);
    }

private:
    static constexpr uint32_t CHUNK_START = 1, CHUNK_END = 2, PARENT = 4, ROOT = 8;
    static constexpr uint32_t IV[8] = {0x6A09E667u, 0xBB67AE85u, 0x3C6EF372u, 0xA54FF53Au,
                                       0x510E527Fu, 0x9B05688Cu, 0x1F83D9ABu, 0x5BE0CD19u};
    uint32_t cv_[8];
    uint8_t buf_[64];
    size_t buf_len_;
    size_t blocks_;  // blocks already compressed in the current chunk
    uint64_t chunk_;
    uint32_t stack_[54][8];
    size_t stack_len_;

    size_t chunk_len() const { return blocks_ * 64 + buf_len_; }
    uint32_t flags_for_block() const { return blocks_ == 0 ? CHUNK_START : 0u; }
    static void words_to_bytes(const uint32_t w[8], uint8_t *b)
    {
#if defined(__BYTE_ORDER__) && __BYTE_ORDER__ == __ORDER_LITTLE_ENDIAN__
        memcpy(b, w, 32);
#else
        for (int i = 0; i < 8; i++)
            for (int k = 0; k < 4; k++) b[4 * i + k] = (uint8_t)(w[i] >> (8 * k));
#endif
    }
    // Completed chunk number n (counting from 1) closes as many subtrees as n has
    // trailing zero bits: merge that many stack entries before pushing.
    void push_cv(const uint32_t out[16])
    {
        uint32_t cv[8];
        memcpy(cv, out, sizeof cv);
        uint64_t total = chunk_ + 1;
        while ((total & 1) == 0) {
            uint8_t parent[64];
            uint32_t o[16];
            words_to_bytes(stack_[stack_len_ - 1], parent);
            words_to_bytes(cv, parent + 32);
            compress(IV, parent, 0, 64, PARENT, o);
            memcpy(cv, o, sizeof cv);
            stack_len_--;
            total >>= 1;
        }
        memcpy(stack_[stack_len_++], cv, sizeof cv);
    }
    static uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
    static void g(uint32_t *s, int a, int b, int c, int d, uint32_t x, uint32_t y)
    {
        s[a] += s[b] + x;
        s[d] = rotr(s[d] ^ s[a], 16);
        s[c] += s[d];
        s[b] = rotr(s[b] ^ s[c], 12);
        s[a] += s[b] + y;
        s[d] = rotr(s[d] ^ s[a], 8);
        s[c] += s[d];
        s[b] = rotr(s[b] ^ s[c], 7);
    }
#if defined(__x86_64__)
    // The same compression with the state as four rows of four words (one G per lane, the diagonal step after rotating
    // the rows) and each round's sixteen message words picked by one 512-bit permute.  A loop over the rounds, not
    // unrolled: it runs once every few microseconds between calls into the HIP runtime, from a cold instruction cache.
    __attribute__((target("avx512f,avx512vl"))) static void compress_avx512(const uint32_t cv[8], const uint8_t block[64], uint64_t counter,
                                                                          uint32_t block_len, uint32_t flags, uint32_t out[16])
    {
        const blake3_detail::RoundIndex &ri = blake3_detail::ROUND_INDEX;
        const __m512i m = _mm512_loadu_si512(block);
        const __m128i cv_lo = _mm_loadu_si128((const __m128i *)cv), cv_hi = _mm_loadu_si128((const __m128i *)(cv + 4));
        __m128i r0 = cv_lo, r1 = cv_hi, r2 = _mm_loadu_si128((const __m128i *)IV);
        __m128i r3 = _mm_set_epi32((int)flags, (int)block_len, (int)(uint32_t)(counter >> 32), (int)(uint32_t)counter);
#define DPSC_G(mx, my)                             \
    r0 = _mm_add_epi32(_mm_add_epi32(r0, r1), mx); \
    r3 = _mm_ror_epi32(_mm_xor_si128(r3, r0), 16); \
    r2 = _mm_add_epi32(r2, r3);                    \
    r1 = _mm_ror_epi32(_mm_xor_si128(r1, r2), 12); \
    r0 = _mm_add_epi32(_mm_add_epi32(r0, r1), my); \
    r3 = _mm_ror_epi32(_mm_xor_si128(r3, r0), 8);  \
    r2 = _mm_add_epi32(r2, r3);                    \
    r1 = _mm_ror_epi32(_mm_xor_si128(r1, r2), 7);
        for (int k = 0; k < 7; k++) {
            const __m512i p = _mm512_permutexvar_epi32(_mm512_load_si512(ri.idx[k]), m);
            DPSC_G(_mm512_castsi512_si128(p), _mm512_extracti32x4_epi32(p, 1))
            // lane i of the rows now holds words i, 4 + (i + 1) % 4, 8 + (i + 2) % 4, 12 + (i + 3) % 4: the diagonals
            r1 = _mm_shuffle_epi32(r1, _MM_SHUFFLE(0, 3, 2, 1));
            r2 = _mm_shuffle_epi32(r2, _MM_SHUFFLE(1, 0, 3, 2));
            r3 = _mm_shuffle_epi32(r3, _MM_SHUFFLE(2, 1, 0, 3));
            DPSC_G(_mm512_extracti32x4_epi32(p, 2), _mm512_extracti32x4_epi32(p, 3))
            r1 = _mm_shuffle_epi32(r1, _MM_SHUFFLE(2, 1, 0, 3));
            r2 = _mm_shuffle_epi32(r2, _MM_SHUFFLE(1, 0, 3, 2));
            r3 = _mm_shuffle_epi32(r3, _MM_SHUFFLE(0, 3, 2, 1));
        }
#undef DPSC_G
        _mm_storeu_si128((__m128i *)out, _mm_xor_si128(r0, r2));
        _mm_storeu_si128((__m128i *)(out + 4), _mm_xor_si128(r1, r3));
        _mm_storeu_si128((__m128i *)(out + 8), _mm_xor_si128(r2, cv_lo));
        _mm_storeu_si128((__m128i *)(out + 12), _mm_xor_si128(r3, cv_hi));
    }
    // (DPSC_BLAKE3_PORTABLE in the environment keeps the portable loop, for the test that compares the two)
    static bool probe_avx512() { return !getenv("DPSC_BLAKE3_PORTABLE") && __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512vl"); }
    static inline const bool HAVE_AVX512 = probe_avx512();
    static bool have_avx512() { return HAVE_AVX512; }
#endif
    static void compress(const uint32_t cv[8], const uint8_t block[64], uint64_t counter, uint32_t block_len,
                         uint32_t flags, uint32_t out[16])
    {
#if defined(__x86_64__)
        if (have_avx512()) {
            compress_avx512(cv, block, counter, block_len, flags, out);
            return;
        }
#endif
        static const uint8_t SCHEDULE[7][16] = {
            {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8},
            {3, 4, 10, 12, 13, 2, 7, 14, 6, 5, 9, 0, 11, 15, 8, 1}, {10, 7, 12, 9, 14, 3, 13, 15, 4, 0, 11, 2, 5, 8, 1, 6},
            {12, 13, 9, 11, 15, 10, 14, 8, 7, 2, 5, 3, 0, 1, 6, 4}, {9, 14, 11, 5, 8, 12, 15, 1, 13, 3, 0, 10, 2, 6, 4, 7},
            {11, 15, 5, 0, 1, 9, 8, 6, 14, 10, 2, 12, 3, 4, 7, 13}};
        uint32_t m[16], s[16];
        for (int i = 0; i < 16; i++)
            m[i] = (uint32_t)block[4 * i] | ((uint32_t)block[4 * i + 1] << 8) | ((uint32_t)block[4 * i + 2] << 16) |
                   ((uint32_t)block[4 * i + 3] << 24);
        for (int i = 0; i < 8; i++) s[i] = cv[i];
        for (int i = 0; i < 4; i++) s[8 + i] = IV[i];
        s[12] = (uint32_t)counter;
        s[13] = (uint32_t)(counter >> 32);
        s[14] = block_len;
        s[15] = flags;
        for (int r = 0; r < 7; r++) {
            const uint8_t *q = SCHEDULE[r];
            g(s, 0, 4, 8, 12, m[q[0]], m[q[1]]);
            g(s, 1, 5, 9, 13, m[q[2]], m[q[3]]);
            g(s, 2, 6, 10, 14, m[q[4]], m[q[5]]);
            g(s, 3, 7, 11, 15, m[q[6]], m[q[7]]);
            g(s, 0, 5, 10, 15, m[q[8]], m[q[9]]);
            g(s, 1, 6, 11, 12, m[q[10]], m[q[11]]);
            g(s, 2, 7, 8, 13, m[q[12]], m[q[13]]);
            g(s, 3, 4, 9, 14, m[q[14]], m[q[15]]);
        }
        for (int i = 0; i < 8; i++) {
            out[i] = s[i] ^ s[i + 8];
            out[i + 8] = s[i + 8] ^ cv[i];
        }
    }
};

}  // namespace dpsc
