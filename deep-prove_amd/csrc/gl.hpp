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

}  // namespace gl
