// Goldilocks (p = 2^64 - 2^32 + 1) and its quadratic extension X^2 = 7 for gfx950.
//
// Every value handed between functions is canonical (< p).  The 64x64 product is
// formed from 32-bit multiplies (v_mad_u64_u32) and reduced with 2^64 = 2^32 - 1,
// 2^96 = -1 and 2^128 = -2^32 (mod p); nothing here maps onto the matrix cores.
//
// The hot operations come in two versions with the same results, bit for bit.
// The portable one (host code, and kernels built for the CPU) is plain 64- and
// 128-bit C++.  On the GPU a kernel's time is its count of vector instructions:
// v_mad_u64_u32 issues about as fast as a 64-bit add or a 64-bit compare (4 to 5
// cycles a wavefront), so what the portable code costs there is its glue --
// 128-bit products put together from halves, overflow found by 64-bit compares
// and selects, a reduction per product.  The device versions (GL_LIMBS) work on
// 32-bit limbs: carries go from instruction to instruction (v_addc_co_u32), and a
// sum of products is gathered by v_mad_u64_u32 itself -- its 64-bit addend is the
// running sum, its carry-out is counted -- in three words by weight (1, 2^32,
// 2^64), put together and reduced once.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gl {

typedef uint64_t u64;
typedef uint32_t u32;
typedef unsigned __int128 u128;

constexpr u64 P = 0xFFFFFFFF00000001ULL;
constexpr u64 EPS = 0xFFFFFFFFULL;  // 2^64 mod p
constexpr u64 W = 7;                // X^2 = W

#define GL_FN __host__ __device__ __forceinline__
#if defined(__HIP_DEVICE_COMPILE__)
#define GL_LIMBS 1  // this pass builds GPU code
#else
#define GL_LIMBS 0
#endif

GL_FN u64 add(u64 a, u64 b)
{
    u64 s = a + b;
    // a + b < 2p: one conditional subtraction; on carry the true sum is s + 2^64
    return (s < a || s >= P) ? s + EPS : s;
}

#if GL_LIMBS
GL_FN u64 pack(u32 lo, u32 hi) { return ((u64)hi << 32) | lo; }

// l0 + 2^32 l1 + 2^64 l2 + 2^96 l3 + 2^128 l4 mod p (l4 < 2^31): (l0, l1) - (l3, l4) + l2 (2^32 - 1); canonical, or
// (CANON = false) any representative below 2^64, for values that only go into further products
template <bool CANON = true>
GL_FN u64 reduce160(u32 l0, u32 l1, u32 l2, u32 l3, u32 l4)
{
    // t = (l0, l1) - (l3, l4) as a wrapped word, b its borrow
    u32 b, c;
    const u32 t0 = __builtin_subc(l0, l3, 0u, &b);
    const u32 t1 = __builtin_subc(l1, l4, b, &b);
    // r = t + l2 (2^32 - 1) by one multiply-add (the product is at most 2^64 - 2^33 + 1), x = all ones when it carries
    u64 r, s;
    u32 x;
    asm("v_mad_u64_u32 %[r], %[s], %[l2], -1, %[t]\n\t"
        "s_nop 1\n\t"
        "v_cndmask_b32_e64 %[x], 0, -1, %[s]"
        : [r] "=v"(r), [s] "=s"(s), [x] "=v"(x)
        : [l2] "v"(l2), [t] "v"(pack(t0, t1)));
    // The value is r + (carry - borrow) 2^64 = r + (carry - borrow) EPS (mod p).  Carry alone: the wrapped word is
    // below 2^64 - 2^33, adding EPS does not wrap.  Borrow alone: t is above 2^63 as a word and nothing wrapped after
    // it, subtracting EPS stays above zero.  Both or neither: r as it is.
    u32 w;
    const u32 d0 = __builtin_subc(x, 0u - b, 0u, &w);  // (all ones or 0) - (all ones or 0) as a 64-bit word (d0, -w)
    r += pack(d0, 0u - w);
    if (!CANON) return r;
    // r >= p exactly when r + EPS wraps, and r - p is that wrapped sum
    const u32 r0 = (u32)r, r1 = (u32)(r >> 32);
    u32 s0 = __builtin_addc(r0, 0xFFFFFFFFu, 0u, &c);
    u32 s1 = __builtin_addc(r1, 0u, c, &c);
    return c ? pack(s0, s1) : r;
}

// (hi * 2^64 + lo) mod p, canonical
GL_FN u64 reduce128(u64 lo, u64 hi) { return reduce160((u32)lo, (u32)(lo >> 32), (u32)hi, (u32)(hi >> 32), 0u); }

GL_FN u64 sub(u64 a, u64 b)
{
    // the borrow of the limb-wise difference says whether p is owed
    u32 w;
    u32 d0 = __builtin_subc((u32)a, (u32)b, 0u, &w);
    u32 d1 = __builtin_subc((u32)(a >> 32), (u32)(b >> 32), w, &w);
    const u32 m = 0u - w;
    d0 = __builtin_subc(d0, m, 0u, &w);
    d1 = __builtin_subc(d1, 0u, w, &w);
    return pack(d0, d1);
}
#else
GL_FN u64 sub(u64 a, u64 b)
{
    u64 d = a - b;
    return a < b ? d - EPS : d;  // wrapped by 2^64 = p + EPS
}

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
#endif

GL_FN u64 neg(u64 a) { return a ? P - a : 0; }

GL_FN u64 dbl(u64 a) { return add(a, a); }

GL_FN u64 mulhi64(u64 a, u64 b) { return (u64)(((u128)a * b) >> 64); }

// the 128-bit product compiles to four v_mad_u64_u32 on the device
GL_FN u64 mul(u64 a, u64 b)
{
    u128 p = (u128)a * b;
    return reduce128((u64)p, (u64)(p >> 64));
}

// a b mod p as any representative below 2^64 (not canonical): for a product that only goes into further products
GL_FN u64 mul_any(u64 a, u64 b)
{
#if GL_LIMBS
    const u128 p = (u128)a * b;
    return reduce160<false>((u32)p, (u32)(p >> 32), (u32)(p >> 64), (u32)(p >> 96), 0u);
#else
    return mul(a, b);
#endif
}

// a * small constant (c < 2^32)
GL_FN u64 mul_small(u64 a, u32 c)
{
#if GL_LIMBS
    const u64 t0 = (u64)(u32)a * c;
    const u64 t1 = (u64)(u32)(a >> 32) * c + (t0 >> 32);  // a c = (t0 mod 2^32) + 2^32 t1
    return reduce160((u32)t0, (u32)t1, (u32)(t1 >> 32), 0u, 0u);
#else
    u64 lo = a * (u64)c;
    u64 hi = mulhi64(a, (u64)c);  // < 2^32
    u64 t1 = (hi << 32) - hi;
    u64 r = lo + t1;
    if (r < t1) r += EPS;
    return r >= P ? r - P : r;
#endif
}

GL_FN u64 from_i64(int64_t x)
{
    // negatives map to p - |x|; |x| < 2^63 < p
    if (x >= 0) return (u64)x;
    u64 mag = (u64)0 - (u64)x;
    return P - mag;
}

GL_FN u64 canon(u64 x) { return x >= P ? x - P : x; }

// ---------------------------------------------------------------------------
// Sums of products.  Acc gathers 64x64 products (and 64-bit terms) without
// reducing; acc_reduce gives the canonical value.  Good for 2^30 terms.
//   portable: the low and the high 64 bits of every 128-bit product are added
//     into two words whose carries are counted,
//     value = lo + cl 2^64 + (hi + ch 2^64) 2^64;
//   device: the four 32x32 products of x y go into three words by weight, each
//     added by the multiply instruction itself, carries counted,
//     value = L + 2^32 M + 2^64 H + cL 2^64 + cM 2^96 + cH 2^128.
// ---------------------------------------------------------------------------
#if GL_LIMBS
struct Acc {
    u64 L, M, H;
    u32 cL, cM, cH;
};

GL_FN Acc acc_zero()
{
    Acc a;
    a.L = a.M = a.H = 0;
    a.cL = a.cM = a.cH = 0;
    return a;
}

GL_FN void acc_add64(Acc &a, u64 x)
{
    u32 c;
    const u32 l0 = __builtin_addc((u32)a.L, (u32)x, 0u, &c);
    const u32 l1 = __builtin_addc((u32)(a.L >> 32), (u32)(x >> 32), c, &c);
    a.cL += c;
    a.L = pack(l0, l1);
}

// += x y.  A carry-out is read three instructions after the multiply that wrote it (the hardware asks for two
// instructions between a vector instruction that writes a scalar register and one that reads it).
GL_FN void acc_prod(Acc &a, u64 x, u64 y)
{
    u64 s0, s1, s2, s3;
    asm("v_mad_u64_u32 %[L], %[s0], %[xl], %[yl], %[L]\n\t"
        "v_mad_u64_u32 %[M], %[s1], %[xl], %[yh], %[M]\n\t"
        "v_mad_u64_u32 %[H], %[s2], %[xh], %[yh], %[H]\n\t"
        "v_addc_co_u32_e64 %[cL], %[s0], 0, %[cL], %[s0]\n\t"
        "v_mad_u64_u32 %[M], %[s3], %[xh], %[yl], %[M]\n\t"
        "v_addc_co_u32_e64 %[cM], %[s1], 0, %[cM], %[s1]\n\t"
        "v_addc_co_u32_e64 %[cH], %[s2], 0, %[cH], %[s2]\n\t"
        "v_addc_co_u32_e64 %[cM], %[s3], 0, %[cM], %[s3]"
        : [L] "+v"(a.L), [M] "+v"(a.M), [H] "+v"(a.H), [cL] "+v"(a.cL), [cM] "+v"(a.cM), [cH] "+v"(a.cH), [s0] "=&s"(s0),
          [s1] "=&s"(s1), [s2] "=&s"(s2), [s3] "=&s"(s3)
        : [xl] "v"((u32)x), [xh] "v"((u32)(x >> 32)), [yl] "v"((u32)y), [yh] "v"((u32)(y >> 32)));
}

// L + 2^32 M + 2^64 H + cL 2^64 + cM 2^96 + cH 2^128 (counters below 2^30), canonical
GL_FN u64 reduce_words(u64 L, u64 M, u64 H, u32 cL, u32 cM, u32 cH)
{
    u32 c;
    const u32 l0 = (u32)L;
    const u32 l1 = __builtin_addc((u32)(L >> 32), (u32)M, 0u, &c);
    u32 l2 = __builtin_addc((u32)(M >> 32), (u32)H, c, &c);
    u32 l3 = __builtin_addc((u32)(H >> 32), cM, c, &c);
    u32 l4 = cH + c;
    l2 = __builtin_addc(l2, cL, 0u, &c);
    l3 = __builtin_addc(l3, 0u, c, &c);
    l4 += c;
    return reduce160(l0, l1, l2, l3, l4);
}

GL_FN u64 acc_reduce(const Acc &a) { return reduce_words(a.L, a.M, a.H, a.cL, a.cM, a.cH); }

// x y + c, canonical (c any 64-bit word)
GL_FN u64 muladd(u64 x, u64 y, u64 c)
{
    u64 L, M, H, s0, s1, s2;
    u32 cL, cM;
    asm("v_mad_u64_u32 %[L], %[s0], %[xl], %[yl], %[c]\n\t"
        "v_mad_u64_u32 %[M], %[s2], %[xl], %[yh], 0\n\t"
        "v_mad_u64_u32 %[H], %[s2], %[xh], %[yh], 0\n\t"
        "v_mad_u64_u32 %[M], %[s1], %[xh], %[yl], %[M]\n\t"
        "v_addc_co_u32_e64 %[cL], %[s0], 0, 0, %[s0]\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32_e64 %[cM], %[s1], 0, 0, %[s1]"
        : [L] "=&v"(L), [M] "=&v"(M), [H] "=&v"(H), [cL] "=&v"(cL), [cM] "=&v"(cM), [s0] "=&s"(s0), [s1] "=&s"(s1), [s2] "=&s"(s2)
        : [xl] "v"((u32)x), [xh] "v"((u32)(x >> 32)), [yl] "v"((u32)y), [yh] "v"((u32)(y >> 32)), [c] "v"(c));
    return reduce_words(L, M, H, cL, cM, 0u);
}

// x y + z w + c, canonical
GL_FN u64 dot2(u64 x, u64 y, u64 z, u64 w, u64 c)
{
    u64 L, M, H, s0, s1, s2, s3, s4, s5;
    u32 cL, cM, cH;
    asm("v_mad_u64_u32 %[L], %[s0], %[xl], %[yl], %[c]\n\t"
        "v_mad_u64_u32 %[M], %[s5], %[xl], %[yh], 0\n\t"
        "v_mad_u64_u32 %[H], %[s5], %[xh], %[yh], 0\n\t"
        "v_mad_u64_u32 %[L], %[s1], %[zl], %[wl], %[L]\n\t"
        "v_mad_u64_u32 %[M], %[s2], %[xh], %[yl], %[M]\n\t"
        "v_mad_u64_u32 %[H], %[s3], %[zh], %[wh], %[H]\n\t"
        "v_addc_co_u32_e64 %[cL], %[s0], 0, 0, %[s0]\n\t"
        "v_mad_u64_u32 %[M], %[s4], %[zl], %[wh], %[M]\n\t"
        "v_addc_co_u32_e64 %[cL], %[s1], 0, %[cL], %[s1]\n\t"
        "v_addc_co_u32_e64 %[cM], %[s2], 0, 0, %[s2]\n\t"
        "v_mad_u64_u32 %[M], %[s5], %[zh], %[wl], %[M]\n\t"
        "v_addc_co_u32_e64 %[cH], %[s3], 0, 0, %[s3]\n\t"
        "v_addc_co_u32_e64 %[cM], %[s4], 0, %[cM], %[s4]\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32_e64 %[cM], %[s5], 0, %[cM], %[s5]"
        : [L] "=&v"(L), [M] "=&v"(M), [H] "=&v"(H), [cL] "=&v"(cL), [cM] "=&v"(cM), [cH] "=&v"(cH), [s0] "=&s"(s0), [s1] "=&s"(s1),
          [s2] "=&s"(s2), [s3] "=&s"(s3), [s4] "=&s"(s4), [s5] "=&s"(s5)
        : [xl] "v"((u32)x), [xh] "v"((u32)(x >> 32)), [yl] "v"((u32)y), [yh] "v"((u32)(y >> 32)), [zl] "v"((u32)z),
          [zh] "v"((u32)(z >> 32)), [wl] "v"((u32)w), [wh] "v"((u32)(w >> 32)), [c] "v"(c));
    return reduce_words(L, M, H, cL, cM, cH);
}
#else
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

// += x y
GL_FN void acc_prod(Acc &a, u64 x, u64 y)
{
    const u128 p = (u128)x * y;
    u64 s;
    a.cl += __builtin_add_overflow(a.lo, (u64)p, &s) ? 1u : 0u;
    a.lo = s;
    a.ch += __builtin_add_overflow(a.hi, (u64)(p >> 64), &s) ? 1u : 0u;
    a.hi = s;
}

GL_FN u64 acc_reduce(const Acc &a)
{
    u64 r = reduce128(a.lo, a.hi);
    r = add(r, (u64)a.cl * EPS);     // cl (2^32 - 1) < p
    return sub(r, (u64)a.ch << 32);  // ch 2^32 < p
}

// x y + c, canonical (c any 64-bit word)
GL_FN u64 muladd(u64 x, u64 y, u64 c)
{
    const u128 t = (u128)x * y + c;  // below 2^128
    return reduce128((u64)t, (u64)(t >> 64));
}

// x y + z w + c, canonical
GL_FN u64 dot2(u64 x, u64 y, u64 z, u64 w, u64 c)
{
    Acc a = acc_zero();
    a.lo = c;
    acc_prod(a, x, y);
    acc_prod(a, z, w);
    return acc_reduce(a);
}
#endif

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

GL_FN E2 fma(E2 a, E2P b, E2 c) { return e2(dot2(a.c0, b.c0, a.c1, b.w, c.c0), dot2(a.c0, b.c1, a.c1, b.c0, c.c1)); }

GL_FN E2 mulp(E2 a, E2P b) { return fma(a, b, e2_zero()); }

GL_FN bool eq(E2 a, E2 b) { return a.c0 == b.c0 && a.c1 == b.c1; }

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
    acc_prod(a.c0, x.c0, b);
    acc_prod(a.c1, x.c1, b);
}
// += x * y, y prepared
GL_FN void acc_mul(E2Acc &a, E2 x, E2P y)
{
    acc_prod(a.c0, x.c0, y.c0);
    acc_prod(a.c0, x.c1, y.w);
    acc_prod(a.c1, x.c0, y.c1);
    acc_prod(a.c1, x.c1, y.c0);
}
GL_FN E2 acc_reduce(const E2Acc &a) { return e2(acc_reduce(a.c0), acc_reduce(a.c1)); }

}  // namespace gl
