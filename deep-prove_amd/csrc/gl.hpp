// Goldilocks (p = 2^64 - 2^32 + 1) and its quadratic extension X^2 = 7 for gfx950.
//
// Every value handed between functions is canonical (< p).  The 64x64 product is
// formed from 32-bit multiplies (v_mad_u64_u32 / v_mul_hi_u32) and reduced with
// 2^64 = 2^32 - 1 and 2^96 = -1 (mod p); nothing here maps onto the matrix cores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gl {

typedef uint64_t u64;
typedef uint32_t u32;

constexpr u64 P = 0xFFFFFFFF00000001ULL;
constexpr u64 EPS = 0xFFFFFFFFULL;  // 2^64 mod p
constexpr u64 W = 7;                // X^2 = W

#define GL_FN __host__ __device__ __forceinline__

GL_FN u64 add(u64 a, u64 b)
{
    u64 s = a + b;
    // a + b < 2p: one conditional subtraction; on carry the true sum is s + 2^64
    return (s < a || s >= P) ? s + EPS : s;
}

GL_FN u64 sub(u64 a, u64 b)
{
    u64 d = a - b;
    return a < b ? d - EPS : d;  // wrapped by 2^64 = p + EPS
}

GL_FN u64 neg(u64 a) { return a ? P - a : 0; }

GL_FN u64 dbl(u64 a) { return add(a, a); }

// (hi * 2^64 + lo) mod p, canonical
GL_FN u64 reduce128(u64 lo, u64 hi)
{
    u32 hh = (u32)(hi >> 32), hl = (u32)hi;
    u64 t0 = lo - hh;  // 2^96 = -1
    if (lo < hh) t0 -= EPS;
    u64 t1 = ((u64)hl << 32) - hl;  // hl * (2^32 - 1)
    u64 r = t0 + t1;
    if (r < t1) r += EPS;
    return r >= P ? r - P : r;
}

GL_FN u64 mulhi64(u64 a, u64 b) { return (u64)(((unsigned __int128)a * b) >> 64); }

// the 128-bit product compiles to four v_mad_u64_u32 on the device
GL_FN u64 mul(u64 a, u64 b)
{
    unsigned __int128 p = (unsigned __int128)a * b;
    return reduce128((u64)p, (u64)(p >> 64));
}

// a * small constant (c < 2^32)
GL_FN u64 mul_small(u64 a, u32 c)
{
    u64 lo = a * (u64)c;
    u64 hi = mulhi64(a, (u64)c);  // < 2^32
    u64 t1 = (hi << 32) - hi;
    u64 r = lo + t1;
    if (r < t1) r += EPS;
    return r >= P ? r - P : r;
}

GL_FN u64 from_i64(int64_t x)
{
    // negatives map to p - |x|; |x| < 2^63 < p
    if (x >= 0) return (u64)x;
    u64 mag = (u64)0 - (u64)x;
    return P - mag;
}

GL_FN u64 canon(u64 x) { return x >= P ? x - P : x; }

struct E2 {
    u64 c0, c1;
};

GL_FN E2 e2(u64 c0, u64 c1)
{
    E2 r;
    r.c0 = c0;
    r.c1 = c1;
    return r;
}
GL_FN E2 e2_zero() { return e2(0, 0); }
GL_FN E2 e2_one() { return e2(1, 0); }
GL_FN E2 add(E2 a, E2 b) { return e2(add(a.c0, b.c0), add(a.c1, b.c1)); }
GL_FN E2 sub(E2 a, E2 b) { return e2(sub(a.c0, b.c0), sub(a.c1, b.c1)); }
GL_FN E2 neg(E2 a) { return e2(neg(a.c0), neg(a.c1)); }

// Karatsuba: three base products
GL_FN E2 mul(E2 a, E2 b)
{
    u64 v0 = mul(a.c0, b.c0);
    u64 v1 = mul(a.c1, b.c1);
    u64 v2 = mul(add(a.c0, a.c1), add(b.c0, b.c1));
    return e2(add(v0, mul_small(v1, (u32)W)), sub(sub(v2, v0), v1));
}

GL_FN E2 mul_base(E2 a, u64 b) { return e2(mul(a.c0, b), mul(a.c1, b)); }

// ---------------------------------------------------------------------------
// Products with one reduction per output limb.  The second operand carries
// w = 7 * c1 (mod p), computed once and reused, so that
//   (a0 + a1 X)(b0 + b1 X) + (c0 + c1 X) = (a0 b0 + a1 w + c0) + (a0 b1 + a1 b0 + c1) X
// is two sums of two 128-bit products plus a 64-bit term, each reduced once.
// ---------------------------------------------------------------------------
typedef unsigned __int128 u128;

struct E2P {
    u64 c0, c1, w;
};

GL_FN E2P prep(E2 b)
{
    E2P r;
    r.c0 = b.c0;
    r.c1 = b.c1;
    r.w = mul_small(b.c1, (u32)W);
    return r;
}

// (x + y + z) mod p for 128-bit x, y and 64-bit z: a 130-bit sum, reduced once
GL_FN u64 reduce_sum(u128 x, u128 y, u64 z)
{
    u128 s = x + y;
    u64 carry = s < x;  // bit 128
    u128 t = s + z;
    carry += t < s;
    u64 lo = (u64)t, hi = (u64)(t >> 64);
    // value = lo + hl 2^64 + hh 2^96 + carry 2^128, with 2^64 = 2^32 - 1, 2^96 = -1, 2^128 = -2^32
    u64 hl = (u32)hi;
    u64 sub = (hi >> 32) + (carry << 32) + hl;  // subtracted: hh + carry 2^32 + hl (from hl (2^32 - 1))
    u64 a = lo + (hl << 32);
    u64 c1 = a < lo;  // wrapped past 2^64: add 2^32 - 1
    u64 r = a - sub;
    u64 b1 = a < sub;  // wrapped below 0: subtract 2^32 - 1
    r += c1 * EPS;     // cannot wrap: a wrapped sum is below 2^64 - 2^32
    r -= b1 * EPS;     // cannot wrap: a wrapped difference is above 2^64 - 2^36
    return r >= P ? r - P : r;
}

GL_FN E2 fma(E2 a, E2P b, E2 c)
{
    u64 r0 = reduce_sum((u128)a.c0 * b.c0, (u128)a.c1 * b.w, c.c0);
    u64 r1 = reduce_sum((u128)a.c0 * b.c1, (u128)a.c1 * b.c0, c.c1);
    return e2(r0, r1);
}

GL_FN E2 mulp(E2 a, E2P b) { return fma(a, b, e2_zero()); }

GL_FN bool eq(E2 a, E2 b) { return a.c0 == b.c0 && a.c1 == b.c1; }

// ---------------------------------------------------------------------------
// Unreduced accumulation.  A long sum of products needs no reduction per term:
// the low and the high 64 bits of every 128-bit product are added into two
// 64-bit words whose carries are counted, and the whole is reduced once,
//   value = lo + cl 2^64 + (hi + ch 2^64) 2^64,   2^64 = 2^32 - 1,  2^128 = -2^32.
// Good for up to 2^32 - 1 terms.
// ---------------------------------------------------------------------------
struct Acc {
    u64 lo, hi;
    u32 cl, ch;
};

GL_FN Acc acc_zero()
{
    Acc a;
    a.lo = a.hi = 0;
    a.cl = a.ch = 0;
    return a;
}

GL_FN void acc_add64(Acc &a, u64 x)
{
    u64 s;
    a.cl += __builtin_add_overflow(a.lo, x, &s) ? 1u : 0u;
    a.lo = s;
}

GL_FN void acc_add(Acc &a, u128 p)
{
    u64 s;
    a.cl += __builtin_add_overflow(a.lo, (u64)p, &s) ? 1u : 0u;
    a.lo = s;
    a.ch += __builtin_add_overflow(a.hi, (u64)(p >> 64), &s) ? 1u : 0u;
    a.hi = s;
}

GL_FN u64 acc_reduce(const Acc &a)
{
    u64 r = reduce128(a.lo, a.hi);
    r = add(r, (u64)a.cl * EPS);      // cl (2^32 - 1) < p
    return sub(r, (u64)a.ch << 32);  // ch 2^32 < p
}

struct E2Acc {
    Acc c0, c1;
};

GL_FN E2Acc e2acc_zero()
{
    E2Acc a;
    a.c0 = acc_zero();
    a.c1 = acc_zero();
    return a;
}
// += v
GL_FN void acc_e2(E2Acc &a, E2 v)
{
    acc_add64(a.c0, v.c0);
    acc_add64(a.c1, v.c1);
}
// += x * b, b in the base field
GL_FN void acc_mul_base(E2Acc &a, E2 x, u64 b)
{
    acc_add(a.c0, (u128)x.c0 * b);
    acc_add(a.c1, (u128)x.c1 * b);
}
// += x * y, y prepared
GL_FN void acc_mul(E2Acc &a, E2 x, E2P y)
{
    acc_add(a.c0, (u128)x.c0 * y.c0);
    acc_add(a.c0, (u128)x.c1 * y.w);
    acc_add(a.c1, (u128)x.c0 * y.c1);
    acc_add(a.c1, (u128)x.c1 * y.c0);
}
GL_FN E2 acc_reduce(const E2Acc &a) { return e2(acc_reduce(a.c0), acc_reduce(a.c1)); }

}  // namespace gl
