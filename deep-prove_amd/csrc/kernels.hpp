// HIP kernels of the sumcheck prover for gfx950 (wave64, 256 CUs in 8 XCDs).
//
// All of them are streaming kernels over structure-of-arrays limb tables; the
// bound is HBM bandwidth, so the rules are: 16-byte per-lane loads of adjacent
// table entries, every live table read once and every folded table written
// once per round, reductions finished in registers/LDS with one partial per
// workgroup, and grids sized to a few workgroups per CU.
#pragma once
#include <type_traits>
#include <utility>

#include "gl.hpp"

namespace dpk {

using gl::E2;
using gl::u32;
using gl::u64;

constexpr int BLOCK = 256;  // 4 wavefronts
constexpr int WAVE = 64;
constexpr int MAX_PTS = 8;  // evaluation points per term (degree + 1 <= 7)

// ---------------------------------------------------------------------------
// loads
// ---------------------------------------------------------------------------
struct __attribute__((aligned(16))) U64x2 {
    u64 x, y;
};

__device__ __forceinline__ U64x2 ld2(const u64 *p) { return *reinterpret_cast<const U64x2 *>(p); }
__device__ __forceinline__ void st2(u64 *p, u64 x, u64 y)
{
    U64x2 v;
    v.x = x;
    v.y = y;
    *reinterpret_cast<U64x2 *>(p) = v;
}

// Streaming store for folded tables.  Written with ordinary stores they sit in the
// memory-side cache as lines still to be written back, and that write-back then
// runs under the following launches (measured: the next proof's first round reads
// 20 % slower).  Streamed, the launch pays for its own writes; over a whole proof
// the kernels take 3 % less time.
typedef u64 u64x2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void st2_stream(u64 *p, u64 x, u64 y)
{
    u64x2v v;
    v.x = x;
    v.y = y;
    __builtin_nontemporal_store(v, reinterpret_cast<u64x2v *>(p));
}

// A table as the kernels see it.  c1 == nullptr: base-field entries in c0.
// is_i64: c0 holds raw int64 values that are embedded on load.
struct Tab {
    const u64 *c0;
    const u64 *c1;
};

__device__ __forceinline__ E2 tab_get(const u64 *c0, const u64 *c1, u64 i)
{
    return gl::e2(c0[i], c1 ? c1[i] : 0);
}

// ---------------------------------------------------------------------------
// block reduction of NP extension elements; result valid in thread 0
// ---------------------------------------------------------------------------
// Sum over the workgroup of canonical field values.  Modular additions across
// lanes would cost a shuffle pair plus a conditional subtraction per step; instead
// every value is cut into three chunks of at most 22 bits, the chunks are summed
// as plain 32-bit integers (256 threads x 2^22 < 2^31) with DPP row operations,
// and the three integer sums are recombined and reduced once.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ u32 dpp_add(u32 x)
{
    // lanes outside ROW_MASK receive 0
    return x + (u32)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, ROW_MASK, 0xF, true);
}

// after this call lane 63 holds the sum over the wavefront
__device__ __forceinline__ u32 wave_sum_u32(u32 x)
{
    x = dpp_add<0xB1, 0xF>(x);   // quad_perm [1,0,3,2]
    x = dpp_add<0x4E, 0xF>(x);   // quad_perm [2,3,0,1]
    x = dpp_add<0x141, 0xF>(x);  // row_half_mirror: the other quad of each 8 lanes
    x = dpp_add<0x140, 0xF>(x);  // row_mirror: the other half of each row of 16
    x = dpp_add<0x142, 0xA>(x);  // row_bcast:15 into rows 1 and 3
    x = dpp_add<0x143, 0xC>(x);  // row_bcast:31 into rows 2 and 3
    return x;
}

// values in, sums out (valid in thread 0 only).  lds: (BLOCK / WAVE) * 3 * NV words.
template <int NV>
__device__ __forceinline__ void block_sum(u64 (&v)[NV], u32 *lds)
{
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        u32 lo = (u32)v[i], hi = (u32)(v[i] >> 32);
        u32 c0 = wave_sum_u32(lo & 0x3FFFFFu);
        u32 c1 = wave_sum_u32((lo >> 22) | ((hi & 0xFFFu) << 10));
        u32 c2 = wave_sum_u32(hi >> 12);
        if (lane == WAVE - 1) {
            lds[(wave * NV + i) * 3 + 0] = c0;
            lds[(wave * NV + i) * 3 + 1] = c1;
            lds[(wave * NV + i) * 3 + 2] = c2;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            u64 c0 = 0, c1 = 0, c2 = 0;
#pragma unroll
            for (int w = 0; w < BLOCK / WAVE; w++) {
                c0 += lds[(w * NV + i) * 3 + 0];
                c1 += lds[(w * NV + i) * 3 + 1];
                c2 += lds[(w * NV + i) * 3 + 2];
            }
            // c0 + c1 * 2^22 + c2 * 2^44 < 2^75
            unsigned __int128 t = (unsigned __int128)c0 + ((unsigned __int128)c1 << 22) + ((unsigned __int128)c2 << 44);
            v[i] = gl::reduce128((u64)t, (u64)(t >> 64));
        }
    }
}

template <int NP>
__device__ __forceinline__ void block_reduce(E2 (&acc)[NP], u32 *lds /* (BLOCK / WAVE) * 6 * NP words */)
{
    u64 v[2 * NP];
#pragma unroll
    for (int t = 0; t < NP; t++) {
        v[2 * t] = acc[t].c0;
        v[2 * t + 1] = acc[t].c1;
    }
    block_sum<2 * NP>(v, lds);
#pragma unroll
    for (int t = 0; t < NP; t++) acc[t] = gl::e2(v[2 * t], v[2 * t + 1]);
}

// ---------------------------------------------------------------------------
// eq(r, x) table
// ---------------------------------------------------------------------------
// Small tables straight from the definition, many per launch.  Job k (blockIdx.y)
// writes 2^n_bits entries: out[i] = prod_b (bit_b(i) ? r[first + b] : 1 - r[first + b]).
constexpr int EQ_MAX_JOBS = 48;
constexpr int EQ_MAX_VARS = 34;
struct EqJob {
    u32 first, n_bits;
    u64 out_off;  // entries from the start of the output arrays; bit 63: of the second pair of arrays (s0, s1)
};
constexpr u64 EQ_JOB_SECOND = 1ull << 63;
struct EqJobs {
    u64 point[2 * EQ_MAX_VARS];  // 2 limbs per coordinate, travels in the kernel arguments
    u64 *o0, *o1;
    u64 *s0, *s1;  // a second pair of output arrays (the seeds of an expansion live apart from the table)
    EqJob job[EQ_MAX_JOBS];
};

// A table of up to EQ_DIRECT_BITS variables is the outer product of the table of its 8 lowest variables (one entry per
// thread, in a register) and the table of the others, of which a workgroup works out the rows it writes (the workgroups of
// a job, gridDim.x of them, share its rows of 256 entries).  Both are outer products themselves, of two tables of at
// most 5 variables each; the four small tables are made by one wavefront each, at the same time.  What a launch costs
// is its longest chain of field multiplications (a fifth of a microsecond each, whatever else the lane could do
// meanwhile): at most 5 for a small table, 1 for the thread's low entry and the workgroup's rows, 1 per row written.
constexpr u32 EQ_DIRECT_BITS = 17;
__global__ void __launch_bounds__(BLOCK) eq_define_kernel(EqJobs js)
{
    static_assert(BLOCK == 256 && WAVE == 64, "a row is the 8 lowest variables; four wavefronts make the four small tables");
    constexpr u32 HI_MAX = 1u << (EQ_DIRECT_BITS - 8);
    __shared__ u64 part0[4][32], part1[4][32];
    __shared__ u64 hi0[HI_MAX], hi1[HI_MAX];
    const EqJob j = js.job[blockIdx.y];
    const u32 lo_bits = j.n_bits < 8 ? j.n_bits : 8, hi_bits = j.n_bits - lo_bits, n_hi = 1u << hi_bits;
    if (blockIdx.x >= n_hi) return;  // (the whole workgroup)
    const u32 t = threadIdx.x, w = t / WAVE, lane = t % WAVE;
    // variables of the four small tables: the low 8 as la + lb, the others as ha + hb
    const u32 la = lo_bits / 2, lb = lo_bits - la, ha = hi_bits / 2, hb = hi_bits - ha;
    const u32 bits_w = w == 0 ? la : w == 1 ? lb : w == 2 ? ha : hb;
    const u32 first_w = j.first + (w == 0 ? 0 : w == 1 ? la : w == 2 ? lo_bits : lo_bits + ha);
    if (lane < (1u << bits_w)) {
        E2 v = gl::e2_one();
        for (u32 b = 0; b < bits_w; b++) {
            const E2 r = gl::e2(js.point[2 * (first_w + b)], js.point[2 * (first_w + b) + 1]);
            v = gl::mul(v, ((lane >> b) & 1) ? r : gl::sub(gl::e2_one(), r));
        }
        part0[w][lane] = v.c0;
        part1[w][lane] = v.c1;
    }
    __syncthreads();
    // the rows of this workgroup: blockIdx.x, + gridDim.x, ...
    const u32 n_rows = (n_hi - blockIdx.x + gridDim.x - 1) / gridDim.x;
    for (u32 k = t; k < n_rows; k += BLOCK) {
        const u32 h = blockIdx.x + k * gridDim.x;
        const u32 a = h & ((1u << ha) - 1), b = h >> ha;
        const E2 v = gl::mul(gl::e2(part0[2][a], part1[2][a]), gl::e2(part0[3][b], part1[3][b]));
        hi0[k] = v.c0;
        hi1[k] = v.c1;
    }
    E2 lo = gl::e2_one();
    if (t < (1u << lo_bits)) {
        const u32 a = t & ((1u << la) - 1), b = t >> la;
        lo = gl::mul(gl::e2(part0[0][a], part1[0][a]), gl::e2(part0[1][b], part1[1][b]));
    }
    __syncthreads();
    if (t >= (1u << lo_bits)) return;
    const bool second = (j.out_off & EQ_JOB_SECOND) != 0;
    u64 *o0 = (second ? js.s0 : js.o0) + (j.out_off & ~EQ_JOB_SECOND), *o1 = (second ? js.s1 : js.o1) + (j.out_off & ~EQ_JOB_SECOND);
    const gl::E2P lp = gl::prep(lo);
    for (u32 k = 0; k < n_rows; k++) {
        const u32 h = blockIdx.x + k * gridDim.x;
        const E2 v = gl::mulp(gl::e2(hi0[k], hi1[k]), lp);
        o0[((u64)h << lo_bits) | t] = v.c0;
        o1[((u64)h << lo_bits) | t] = v.c1;
    }
}

// The same for jobs of several tables at once (many small eq tables, each with its own point): descriptors and
// points lie in host-visible memory, written just before the launch.
struct EqJobM {
    u64 *o0, *o1;     // where the job's entries go
    u32 first, n_bits;
    u32 point_off;    // words from `points` to the table's point
    u32 pad;
};
__global__ void __launch_bounds__(BLOCK) eq_define_many_kernel(const EqJobM *__restrict__ jobs, const u64 *__restrict__ points)
{
    const EqJobM j = jobs[blockIdx.y];
    const u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= ((u64)1 << j.n_bits)) return;
    const u64 *pt = points + j.point_off;
    E2 acc = gl::e2_one();
    for (u32 b = 0; b < j.n_bits; b++) {
        E2 r = gl::e2(pt[2 * (j.first + b)], pt[2 * (j.first + b) + 1]);
        acc = gl::mul(acc, ((i >> b) & 1) ? r : gl::sub(gl::e2_one(), r));
    }
    j.o0[i] = acc.c0;
    j.o1[i] = acc.c1;
}

// Expansion: out[h * 2^b + l] = hi[h] * lo[l], lo has 2^b <= 256 entries.  Each
// thread keeps one lo entry in registers and walks hi entries; stores of one
// wavefront cover 512 contiguous bytes per limb array.
__global__ void __launch_bounds__(BLOCK)
eq_expand_kernel(const u64 *__restrict__ hi0, const u64 *__restrict__ hi1, u64 n_hi, const u64 *__restrict__ lo0,
                 const u64 *__restrict__ lo1, u32 b, u64 *__restrict__ o0, u64 *__restrict__ o1, u32 hi_per_block)
{
    const u32 n_lo = 1u << b;
    const u32 l = threadIdx.x & (n_lo - 1);
    const u32 sub = threadIdx.x >> b;  // several hi rows per pass when n_lo < BLOCK
    const u32 rows_per_pass = BLOCK >> b;
    E2 lo = gl::e2(lo0[l], lo1[l]);
    u64 h_begin = (u64)blockIdx.x * hi_per_block;
    u64 h_end = h_begin + hi_per_block;
    if (h_end > n_hi) h_end = n_hi;
    for (u64 h = h_begin + sub; h < h_end; h += rows_per_pass) {
        E2 v = gl::mul(gl::e2(hi0[h], hi1[h]), lo);
        u64 o = (h << b) | l;
        o0[o] = v.c0;
        o1[o] = v.c1;
    }
}

// ---------------------------------------------------------------------------
// stand-alone fold: dst[i] = src[2i] + r * (src[2i+1] - src[2i])
// ---------------------------------------------------------------------------
struct FoldDesc {
    const u64 *s0;
    const u64 *s1;  // nullptr: base-field source
    u64 *d0;
    u64 *d1;
    u64 half;  // entries written
    u64 single;  // 1: the source is one entry s of a zero-padded table (its partner is 0): dst[0] = s (1 - r)
};

__device__ __forceinline__ E2 fold1(E2 lo, E2 hi, E2 r) { return gl::add(lo, gl::mul(r, gl::sub(hi, lo))); }
// lo + (hi - lo) * r with r prepared: one reduction per output limb
__device__ __forceinline__ E2 fold1p(E2 lo, E2 hi, gl::E2P r) { return gl::fma(gl::sub(hi, lo), r, lo); }
__device__ __forceinline__ E2 fold1_base(u64 lo, u64 hi, E2 r)
{
    const u64 d = gl::sub(hi, lo);
    return gl::e2(gl::muladd(r.c0, d, lo), gl::mul(r.c1, d));
}

__device__ __forceinline__ void fold_body(const FoldDesc &d, E2 r)
{
    if (d.single) {
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            E2 v = fold1(gl::e2(d.s0[0], d.s1 ? d.s1[0] : 0), gl::e2_zero(), r);
            d.d0[0] = v.c0;
            d.d1[0] = v.c1;
        }
        return;
    }
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < d.half; i += (u64)gridDim.x * BLOCK) {
        U64x2 a = ld2(d.s0 + 2 * i);
        E2 v;
        if (d.s1) {
            U64x2 b = ld2(d.s1 + 2 * i);
            v = fold1(gl::e2(a.x, b.x), gl::e2(a.y, b.y), r);
        } else {
            v = fold1_base(a.x, a.y, r);
        }
        d.d0[i] = v.c0;
        d.d1[i] = v.c1;
    }
}

// one table per grid row, descriptors in device-visible memory
__global__ void __launch_bounds__(BLOCK) fold_kernel(const FoldDesc *__restrict__ descs, u64 r0, u64 r1)
{
    const FoldDesc d = descs[blockIdx.y];
    fold_body(d, gl::e2(r0, r1));
}

// one table, descriptor in the kernel arguments
__global__ void __launch_bounds__(BLOCK) fold_one_kernel(FoldDesc d, u64 r0, u64 r1) { fold_body(d, gl::e2(r0, r1)); }

// ---------------------------------------------------------------------------
// round result: the last workgroup of an evaluation launch sums the block
// partials of every term, scales by the term's coefficient, extends a degree-k
// term to the d+1 points of the round message (Lagrange weights over the nodes
// 0..k), adds the constant terms, and publishes the message to host-visible
// memory followed by a sequence number the host polls.
// ---------------------------------------------------------------------------
struct FinTerm {
    u64 coeff0, coeff1;
    u32 n_factors;
    u32 pad;
};

struct FinArgs {
    const u64 *partial;    // [term][block][2 * MAX_PTS]
    u32 blocks_per_term;
    u32 n_terms;
    const FinTerm *terms;
    u32 degree;
    u32 total_blocks;      // workgroups that take a ticket before the result is complete
    const u64 *lagrange;   // [k][t][i], 9*9*9
    u64 const0, const1;    // constant terms summed over the remaining hypercube
    u64 *out_dev;          // 2 * (degree + 1) limbs
    u64 *out_host;         // same, host-visible; out_host[HOST_SEQ_SLOT] receives seq
    u64 seq;
    u32 *counter;          // ticket counter, zero between launches
};
constexpr int HOST_SEQ_SLOT = 2 * MAX_PTS;
constexpr int HOST_CHK_SLOT = HOST_SEQ_SLOT + 1;
constexpr int HOST_FINALS_SLOT = HOST_SEQ_SLOT + 8;
// A second hand-off in the same 64-word area, with a sequence and a check word of its own: with its last round a
// resident kernel also publishes value and slope of the last pair of every table (4 words per table from
// HOST_FINALS_SLOT on); the final evaluations are then value + r * slope, which the host works out when the last
// challenge is drawn -- no further trip to the GPU.
constexpr int HOST_PAIRS_SEQ_SLOT = 62, HOST_PAIRS_CHK_SLOT = 63;

// Block partials cross XCDs (each XCD has its own L2).  They are written and read
// with agent-scope accesses, which go through to the coherence point, so that no
// workgroup has to write back or invalidate a whole L2: a cache-wide release or
// acquire per workgroup stalls the streaming loads of every other workgroup on
// that XCD.
__device__ __forceinline__ u64 ld_agent(const u64 *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(u64 *p, u64 v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// a value that is the same in every lane, moved to scalar registers
__device__ __forceinline__ u64 uniform64(u64 v)
{
    const u32 lo = __builtin_amdgcn_readfirstlane((u32)v), hi = __builtin_amdgcn_readfirstlane((u32)(v >> 32));
    return ((u64)hi << 32) | lo;
}
// host-visible (fine-grained pinned) memory
__device__ __forceinline__ u64 ld_sys(const u64 *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM); }
__device__ __forceinline__ void st_sys(u64 *p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM); }

__host__ __device__ __forceinline__ u64 rotl64(u64 x, u32 k)
{
    k &= 63;
    return k ? (x << k) | (x >> (64 - k)) : x;
}

// Hand `n` result words to the host (one thread calls this): the words, a check
// word and the sequence number the host polls.  Nothing waits for a store to be
// acknowledged, and the order in which the stores land does not matter: the
// host accepts the words only when  check == seq ^ xor_i rotl(word_i, i + 1).
__device__ __forceinline__ void publish_words(u64 *out_host, u32 slot0, const u64 *words, u32 n, u64 seq, int seq_slot = HOST_SEQ_SLOT,
                                              int chk_slot = HOST_CHK_SLOT)
{
    u64 chk = seq;
    for (u32 i = 0; i < n; i++) {
        const u64 w = words[i];
        chk ^= rotl64(w, i + 1);
        st_sys(out_host + slot0 + i, w);
    }
    st_sys(out_host + chk_slot, chk);
    st_sys(out_host + seq_slot, seq);
}

// Called by every thread of one workgroup once all partials are visible.
template <int NPMAX>
__device__ __forceinline__ void finalize_block(const FinArgs &fa, u32 *lds /* (BLOCK / WAVE) * 6 * MAX_PTS words */, u64 *res /* 2 * MAX_PTS */)
{
    if (threadIdx.x < 2 * MAX_PTS) res[threadIdx.x] = 0;
    __syncthreads();
    for (u32 ti = 0; ti < fa.n_terms; ti++) {
        const u32 k = fa.terms[ti].n_factors;
        E2 acc[NPMAX];
#pragma unroll
        for (int t = 0; t < NPMAX; t++) acc[t] = gl::e2_zero();
        for (u32 b = threadIdx.x; b < fa.blocks_per_term; b += BLOCK) {
            const u64 *p = fa.partial + ((u64)ti * fa.blocks_per_term + b) * 2 * MAX_PTS;
#pragma unroll
            for (int t = 0; t < NPMAX; t++) {
                if ((u32)t <= k) {
                    acc[t].c0 = gl::add(acc[t].c0, ld_agent(p + 2 * t));
                    acc[t].c1 = gl::add(acc[t].c1, ld_agent(p + 2 * t + 1));
                }
            }
        }
        block_reduce<NPMAX>(acc, lds);
        if (threadIdx.x == 0) {
            const E2 coeff = gl::e2(fa.terms[ti].coeff0, fa.terms[ti].coeff1);
            for (u32 t = 0; t <= fa.degree; t++) {
                E2 v;
                if (t <= k) {
                    v = acc[0];
#pragma unroll
                    for (int i = 1; i < NPMAX; i++)
                        if ((u32)i == t) v = acc[i];
                } else {
                    v = gl::e2_zero();
#pragma unroll
                    for (int i = 0; i < NPMAX; i++) {
                        if ((u32)i <= k) v = gl::add(v, gl::mul_base(acc[i], fa.lagrange[(k * 9 + t) * 9 + i]));
                    }
                }
                v = gl::mul(v, coeff);
                res[2 * t] = gl::add(res[2 * t], v.c0);
                res[2 * t + 1] = gl::add(res[2 * t + 1], v.c1);
            }
        }
        __syncthreads();
    }
    if (threadIdx.x <= fa.degree) {
        u32 t = threadIdx.x;
        u64 c0 = gl::add(res[2 * t], fa.const0), c1 = gl::add(res[2 * t + 1], fa.const1);
        fa.out_dev[2 * t] = c0;
        fa.out_dev[2 * t + 1] = c1;
        res[2 * t] = c0;
        res[2 * t + 1] = c1;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        *fa.counter = 0;
        publish_words(fa.out_host, 0, res, 2 * (fa.degree + 1), fa.seq);
    }
}

// Every workgroup calls this after writing its partial (thread 0 wrote it).
// Returns true in the workgroup that took the last ticket.
__device__ __forceinline__ bool take_ticket(u32 *counter, u32 total_blocks, int *flag_lds)
{
    if (threadIdx.x == 0) {
        // thread 0 wrote the partial with agent-scope stores: wait for them to be acknowledged, then take the ticket
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
        u32 t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag_lds = (t == total_blocks - 1);
    }
    __syncthreads();
    bool last = *flag_lds != 0;
    // one cache invalidation, in the last workgroup only; its loads of the partials are agent-scope as well
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return last;
}

// used when a round has no evaluation launch (a sum with constant terms only)
__global__ void __launch_bounds__(BLOCK) finalize_kernel(FinArgs fa)
{
    __shared__ u32 lds[(BLOCK / WAVE) * 6 * MAX_PTS];
    __shared__ u64 res[2 * MAX_PTS];
    finalize_block<MAX_PTS>(fa, lds, res);
}

// ---------------------------------------------------------------------------
// general term evaluation: one grid row (blockIdx.y) per term
// ---------------------------------------------------------------------------
struct FactorDesc {
    const u64 *c0;
    const u64 *c1;  // nullptr: base field
    u32 shift;      // broadcast tables: entry index = pair index >> shift
    u32 pair;       // 1: read entries 2i, 2i+1; 0: broadcast; 2: entry 0 paired with 0 (a zero-padded table down to one entry)
};

struct TermDesc {
    u32 n_factors;
    u32 pad;
    u64 n_pairs;  // pairs on which the product can be non-zero: zero-padded factors cut the range short
    FactorDesc f[DPS_MAX_FACTORS];
};

// partial sums: out[(term * gridDim.x + block) * 2 * MAX_PTS + 2 * t + limb]
template <int NF>
__device__ __forceinline__ void eval_term_body(const TermDesc &td, u64 *__restrict__ partial, u32 *lds)
{
    const u64 n_pairs = td.n_pairs;
    constexpr int NP = NF + 1;
    E2 acc[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) acc[t] = gl::e2_zero();
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < n_pairs; i += (u64)gridDim.x * BLOCK) {
        E2 cur[NF], dl[NF];
#pragma unroll
        for (int f = 0; f < NF; f++) {
            const FactorDesc &fd = td.f[f];
            if (fd.pair == 2) {
                cur[f] = tab_get(fd.c0, fd.c1, 0);
                dl[f] = gl::neg(cur[f]);
            } else if (fd.pair) {
                U64x2 a = ld2(fd.c0 + 2 * i);
                if (fd.c1) {
                    U64x2 b = ld2(fd.c1 + 2 * i);
                    cur[f] = gl::e2(a.x, b.x);
                    dl[f] = gl::e2(gl::sub(a.y, a.x), gl::sub(b.y, b.x));
                } else {
                    cur[f] = gl::e2(a.x, 0);
                    dl[f] = gl::e2(gl::sub(a.y, a.x), 0);
                }
            } else {
                cur[f] = tab_get(fd.c0, fd.c1, i >> fd.shift);
                dl[f] = gl::e2_zero();
            }
        }
#pragma unroll
        for (int t = 0; t < NP; t++) {
            E2 prod = cur[0];
#pragma unroll
            for (int f = 1; f < NF; f++) prod = gl::mul(prod, cur[f]);
            acc[t] = gl::add(acc[t], prod);
            if (t + 1 < NP) {
#pragma unroll
                for (int f = 0; f < NF; f++) cur[f] = gl::add(cur[f], dl[f]);
            }
        }
    }
    block_reduce<NP>(acc, lds);
    if (threadIdx.x == 0) {
        u64 *o = partial + ((u64)blockIdx.y * gridDim.x + blockIdx.x) * 2 * MAX_PTS;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            st_agent(o + 2 * t, acc[t].c0);
            st_agent(o + 2 * t + 1, acc[t].c1);
        }
    }
}

__global__ void __launch_bounds__(BLOCK)
eval_terms_kernel(const TermDesc *__restrict__ terms, u64 *__restrict__ partial, FinArgs fa)
{
    __shared__ u32 lds[(BLOCK / WAVE) * 6 * MAX_PTS];
    __shared__ u64 res[2 * MAX_PTS];
    __shared__ int last_flag;
    const TermDesc &td = terms[blockIdx.y];
    switch (td.n_factors) {
    case 1: eval_term_body<1>(td, partial, lds); break;
    case 2: eval_term_body<2>(td, partial, lds); break;
    case 3: eval_term_body<3>(td, partial, lds); break;
    case 4: eval_term_body<4>(td, partial, lds); break;
    case 5: eval_term_body<5>(td, partial, lds); break;
    case 6: eval_term_body<6>(td, partial, lds); break;
    default: break;
    }
    if (take_ticket(fa.counter, fa.total_blocks, &last_flag)) finalize_block<MAX_PTS>(fa, lds, res);
}

// ---------------------------------------------------------------------------
// mailbox: how a kernel that is already on the GPU is handed a challenge.  The host writes the words to fine-grained
// pinned memory, the kernel polls them with system-scope loads.  Used by the resident kernels for every round after
// their first, and by launches made ahead of their round for the first one as well.
// ---------------------------------------------------------------------------
// mailbox words; MAIL_SEQ == MAIL_ABORT_SEQ tells the kernel to exit
// MAIL_R: the challenge of the round before the one the mail starts; MAIL_RA: the one before that (read by a kernel
// that has two folds pending because its last result covered two rounds).  MAIL_SKIP1: 0 / 1, or MAIL_SKIP1_LEAVE when
// the first workgroup of a launch passes on that no mail came.
constexpr int MAIL_SEQ = 0, MAIL_CHK = 1, MAIL_R = 2, MAIL_SKIP1 = 4, MAIL_RA = 5, MAIL_WORDS = 7;
constexpr u64 MAIL_SKIP1_LEAVE = 2;
static_assert(MAIL_WORDS <= WAVE, "one wavefront reads the mailbox with one load");
constexpr u64 MAIL_ABORT_SEQ = ~(u64)0;
// A mail passed on through device memory (wait_first_mail) is written MAIL_RELAY_COPIES times, 256 bytes apart, and a
// workgroup polls the copy of its number: polls of one place are served one after the other, and with 255 workgroups on
// one copy the last of them saw the mail 2 us after the first.
constexpr u32 MAIL_RELAY_COPIES = 16, MAIL_RELAY_STRIDE = 32, MAIL_RELAY_WORDS = MAIL_RELAY_COPIES * MAIL_RELAY_STRIDE;

// check word of a mailbox: seq ^ xor over the payload words of rotl(word_i, i)
__host__ __device__ __forceinline__ u64 mail_mix(u64 w, u32 i) { return (i >= (u32)MAIL_R && i < (u32)MAIL_WORDS) ? rotl64(w, i) : 0; }

// How long a kernel waits is time, not a number of polls (a poll of host memory takes 2.5 us, one of device memory a
// fraction of that): `spin_limit` counts units of 256 ticks of the device's real-time counter (100 MHz: 2.56 us a unit;
// the host scales its figures by the counter's rate).
__device__ __forceinline__ bool wait_time_left(u64 t0, u32 spin_limit) { return wall_clock64() - t0 <= ((u64)spin_limit << 8); }

// Waits for mail number `want` and copies it to `box` (LDS).  The first wavefront
// polls: every lane loads one mailbox word, so one load instruction (one trip over
// the host link) fetches the whole mail; it is accepted when the sequence number
// matches and the check word agrees with the payload, which makes a torn read
// (the host still writing) look like no mail yet.  Returns false on abort or timeout.
__device__ __forceinline__ bool tail_wait_mail(const u64 *mail, u32 spin_limit, u64 want, u64 *box, int *ok_lds)
{
    if (threadIdx.x < WAVE) {
        const u32 l = threadIdx.x;
        int ok = 0;
        const u64 t0 = wall_clock64();
        do {
            const u64 w = l < (u32)MAIL_WORDS ? ld_sys(mail + l) : 0;
            u64 x = mail_mix(w, l);
#pragma unroll
            for (int off = WAVE / 2; off >= 1; off >>= 1) x ^= __shfl_xor(x, off, WAVE);
            const u64 seq = __shfl(w, MAIL_SEQ, WAVE), chk = __shfl(w, MAIL_CHK, WAVE);
            if (seq == MAIL_ABORT_SEQ) break;
            if (seq == want && chk == (x ^ seq)) {
                if (l < (u32)MAIL_WORDS) box[l] = w;
                ok = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(2);
            // (one lane's clock decides for the wavefront: the lanes must leave the loop together)
        } while (__shfl((int)wait_time_left(t0, spin_limit), 0, WAVE));
        if (l == 0) *ok_lds = ok;
    }
    __syncthreads();
    return *ok_lds != 0;
}

// The first mail of a launch made ahead of its round.  With few workgroups each polls the host's mailbox (relay ==
// nullptr).  With many, only the first one does (first_wg) and copies the mail to device memory (MAIL_RELAY_WORDS words:
// several copies), where the others look for it; when no mail comes it passes on a mail of this number with `reject_skip1`
// in the skip word, a value the calling variant does not accept, so that every workgroup leaves.  True: the mail is in `box`.
__device__ __forceinline__ bool wait_first_mail(const u64 *mail, u64 *relay, bool first_wg, u32 spin_limit, u64 seq, u64 reject_skip1, u64 *box,
                                                int *ok_lds)
{
    if (relay == nullptr) return tail_wait_mail(mail, spin_limit, seq, box, ok_lds);
    // (the others outlast the first workgroup, which always passes something on: their polls of device memory are quicker)
    if (!first_wg) {
        const u32 copy = (blockIdx.x + blockIdx.y * gridDim.x) & (MAIL_RELAY_COPIES - 1);
        return tail_wait_mail(relay + copy * MAIL_RELAY_STRIDE, spin_limit + spin_limit / 4 + 4000, seq, box, ok_lds);
    }
    const bool ok = tail_wait_mail(mail, spin_limit, seq, box, ok_lds);
    if (threadIdx.x < WAVE) {
        // (a copy is accepted by its check word, so the order in which the words land does not matter)
        for (u32 u = threadIdx.x; u < MAIL_RELAY_COPIES * (u32)MAIL_WORDS; u += WAVE) {
            const u32 k = u % (u32)MAIL_WORDS, copy = u / (u32)MAIL_WORDS;
            const u64 none = k == (u32)MAIL_SEQ ? seq : k == (u32)MAIL_SKIP1 ? reject_skip1 : k == (u32)MAIL_CHK ? (seq ^ mail_mix(reject_skip1, MAIL_SKIP1)) : 0;
            const u64 w = ok ? box[k] : none;
            st_sys(relay + copy * MAIL_RELAY_STRIDE + k, w);
        }
    }
    return ok;
}

// ---------------------------------------------------------------------------
// fused product kernels: one term, NF full-size tables (the first NB of them
// base-field in the source), optionally times an eq(rho, x) factor.
//
// FOLD = false: first round, the source pairs are evaluated as they are.
// FOLD = true : source quads are folded with r, the folded pair is written and
//               evaluated: every table is read once and written once per round.
// TWO         : the sources are two rounds old (base-field tables nobody has folded yet: the first two rounds were
//               one launch, pair12_kernel).  Eight source entries make a folded pair; an entry of it is the
//               combination sum_ab e_a(ra) e_b(r) x[a + 2 b] of four of them, e_0(c) = 1 - c, e_1(c) = c: four
//               products gathered unreduced and reduced once, which costs no more than one fold of a folded table.
//
// The eq factor is never folded or streamed as a table of this round's size.
// After the variables below v are bound, eq(rho, .) restricted to the remaining
// cube is  S * eq1(rho_v, x_v) * R(x')  with a scalar S, the one-variable factor
// eq1(a, b) = a b + (1 - a)(1 - b), and R = eq(rho_{v+1..}, .) a table of half this
// round's size, prepared when the eq table was built.  The kernel sums
// q(t) = sum_{x'} R(x') prod_f table_f(t, x') at t = 0..NF; the round message
// p(t) = coeff * S * eq1(rho_v, t) * q(t) at t = 0..NF+1 is formed by the host
// from the sums (q has degree NF, so q(NF+1) follows from the NF+1 sums).
//
// From round 2 on the host knows the claim p(0) + p(1); then t = 1 is skipped
// in the loop and q(1) is solved from the claim.
// ---------------------------------------------------------------------------
struct ProdArgs {
    const u64 *s0[3];
    const u64 *s1[3];
    u64 *d0[3];
    u64 *d1[3];
    const u64 *q0;  // R of this round, n_pairs entries (eq factor only)
    const u64 *q1;
    u64 n_pairs;  // pairs evaluated this round
    u64 r0, r1;   // fold challenge
    u64 ra0, ra1;  // TWO variants: the challenge of the round before that (a mail brings it as MAIL_RA)
    u32 skip1;    // 1: t = 1 is not evaluated (the launch picks the kernel variant accordingly)
    u32 two;      // 1: the sources are two rounds old (the launch picks the TWO variant)
    // A launch made before its round began (wait_first): the challenge is not in r0, r1; the kernel waits for the mail
    // with the launch's sequence number and takes it from there.
    u32 wait_first;
    u32 spin_limit;
    const u64 *mail;
    // A launch of many workgroups made ahead: only workgroup 0 polls the host's mailbox; it copies the mail to these
    // MAIL_WORDS words of device memory, where the other workgroups look for it.  nullptr: every workgroup polls the mailbox.
    u64 *relay;
    // FACT variants (rounds of at least 2^EQ_LO_BITS pairs): R is not streamed.  R(i) = hi[i >> EQ_LO_BITS] * lo[i & mask],
    // lo = eq over the EQ_LO_BITS lowest live variables, hi = R of EQ_LO_BITS rounds later.  The grid's stride is a
    // multiple of 2^EQ_LO_BITS, so a thread's pairs all have the same low part: it weights its running sums with hi only
    // (one entry per workgroup and step: scalar loads) and multiplies them by its entry of lo once, at the end.
    const u64 *lq0, *lq1, *hq0, *hq1;
};
constexpr u32 EQ_LO_BITS = 16;

// The kernels hand the host the sums q(t), t = 0..NF (q(1) left at zero when t = 1 was skipped), not the round
// message: p(t) = scale(t) q(t) + const, the extra point p(NF + 1) of a sum with an eq factor, and p(1) from the
// claim are a dozen field products, which one GPU lane takes about 2 us over and a CPU core 0.1 us, while the
// kernel of the next round cannot start before the host has drawn its challenge anyway.
struct FastFin {
    const u64 *partial;  // word k of workgroup b at partial[k * n_blocks + b]
    u32 n_blocks;
    u32 pad;
    u64 *out_host;
    u64 seq;
    u32 *counter;
    // Few workgroups: each publishes its own sums to a 64-word area of its own (slots + 64 * workgroup, laid out like
    // out_host) and the host adds them; this spares the round the ticket and the gathering, two trips through device
    // memory one after the other.  nullptr: the last workgroup gathers and publishes to out_host.
    u64 *slots;
};

// sums of the workgroups' partials, valid in thread 0
template <int NP>
__device__ __forceinline__ void gather_partials(const FastFin &ff, u32 *lds, E2 (&q)[NP])
{
#pragma unroll
    for (int t = 0; t < NP; t++) q[t] = gl::e2_zero();
    // Word k of workgroup b is at partial[k * n_blocks + b]: a wavefront's load reads 64 adjacent words.  (With a
    // workgroup's words side by side every lane touched a cache line of its own, and the gather of 768 workgroups took
    // 5 to 7 us.)  A thread issues the loads of all its workgroups before it adds: one wait, not one per workgroup.
    constexpr int AHEAD = 4;
    for (u32 b0 = threadIdx.x; b0 < ff.n_blocks; b0 += AHEAD * BLOCK) {
        u64 w[AHEAD][2 * NP];
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            const u32 b = b0 + u * BLOCK;
            const u64 *p = ff.partial + b;
#pragma unroll
            for (int k = 0; k < 2 * NP; k++) w[u][k] = b < ff.n_blocks ? ld_agent(p + (u64)k * ff.n_blocks) : 0;
        }
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
#pragma unroll
            for (int t = 0; t < NP; t++) {
                q[t].c0 = gl::add(q[t].c0, w[u][2 * t]);
                q[t].c1 = gl::add(q[t].c1, w[u][2 * t + 1]);
            }
        }
    }
    block_reduce<NP>(q, lds);
}

// sums[t] = q(t) for t = 0..NP - 1, valid in thread 0: to the host as 2 * NP words, and the ticket counter back to zero
template <int NP>
__device__ __forceinline__ void publish_sums(u64 *out_host, u64 seq, u32 *counter, const E2 (&sums)[NP])
{
    if (threadIdx.x == 0) {
        if (counter) *counter = 0;
        u64 chk = seq;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            chk ^= rotl64(sums[t].c0, 2 * t + 1) ^ rotl64(sums[t].c1, 2 * t + 2);
            st_sys(out_host + 2 * t, sums[t].c0);
            st_sys(out_host + 2 * t + 1, sums[t].c1);
        }
        st_sys(out_host + HOST_CHK_SLOT, chk);
        st_sys(out_host + HOST_SEQ_SLOT, seq);
    }
}

template <int NF, int NB, bool FOLD, bool EQ, bool SKIP1, bool FACT = false, bool TWO = false>
__global__ void __launch_bounds__(BLOCK) prod_kernel(ProdArgs a, u64 *__restrict__ partial, FastFin ff)
{
    static_assert(!FACT || EQ, "factored weights belong to the eq factor");
    static_assert(!TWO || (FOLD && NB == NF), "two folds at once: from base-field sources only");
    constexpr int NP = NF + 1;
    __shared__ u32 lds[(BLOCK / WAVE) * 6 * NP];
    __shared__ int last_flag;
    __shared__ u64 box[MAIL_WORDS];  // the mail of a launch made ahead
    __shared__ int ok_flag;
    E2 r = gl::e2(a.r0, a.r1);
    gl::E2P rp = gl::prep(r);
    // TWO: the weights of a folded entry's four sources
    E2 k2[4];
    auto set_two = [&](E2 ra, E2 rb) {
        const E2 na = gl::sub(gl::e2_one(), ra), nb = gl::sub(gl::e2_one(), rb);
        k2[0] = gl::mul(na, nb), k2[1] = gl::mul(ra, nb), k2[2] = gl::mul(na, rb), k2[3] = gl::mul(ra, rb);
    };
    if (TWO) set_two(gl::e2(a.ra0, a.ra1), r);
    // a compile-time switch: as a run-time flag the compiler evaluates t = 1 anyway and discards it
    constexpr bool skip1 = SKIP1;
    // running sums, reduced once after the loop
    gl::E2Acc lz[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) lz[t] = gl::e2acc_zero();

    // Raw operands of one loop step.  The first-round kernel has little arithmetic
    // per byte, so it loads the next step's operands before working on the
    // current ones; the fold kernels are arithmetic-bound and keep one set.
    // (Members a variant never loads -- the second limbs of base-field sources, the weights without an eq factor -- keep
    // their zeros and are never read.)
    struct Raw {
        U64x2 a0[NF] = {}, b0[NF] = {}, a1[NF] = {}, b1[NF] = {};
        U64x2 c0[TWO ? NF : 1] = {}, e0[TWO ? NF : 1] = {};  // TWO: entries 4..7 of the eight
        u64 q0 = 0, q1 = 0;
    };
    auto load_raw = [&](u64 i, Raw &w) {
#pragma unroll
        for (int f = 0; f < NF; f++) {
            if (TWO) {
                w.a0[f] = ld2(a.s0[f] + 8 * i);
                w.b0[f] = ld2(a.s0[f] + 8 * i + 2);
                w.c0[f] = ld2(a.s0[f] + 8 * i + 4);
                w.e0[f] = ld2(a.s0[f] + 8 * i + 6);
            } else if (FOLD) {
                w.a0[f] = ld2(a.s0[f] + 4 * i);
                w.b0[f] = ld2(a.s0[f] + 4 * i + 2);
                if (f >= NB) {
                    w.a1[f] = ld2(a.s1[f] + 4 * i);
                    w.b1[f] = ld2(a.s1[f] + 4 * i + 2);
                }
            } else {
                w.a0[f] = ld2(a.s0[f] + 2 * i);
                if (f >= NB) w.a1[f] = ld2(a.s1[f] + 2 * i);
            }
        }
        if (EQ) {
            if (FACT) {
                // the same entry for the whole workgroup (BLOCK divides 2^EQ_LO_BITS)
                const u32 hi = __builtin_amdgcn_readfirstlane((u32)(i >> EQ_LO_BITS));
                w.q0 = a.hq0[hi];
                w.q1 = a.hq1[hi];
            } else {
                w.q0 = a.q0[i];
                w.q1 = a.q1[i];
            }
        }
    };
    // One loop step on loaded operands, in two parts: the first uses up the operands (and folds them), the second
    // evaluates.  Between the two the fold kernels ask for the next step's operands, so that a wavefront's loads are
    // in flight while it evaluates.
    // base-field arithmetic applies only while the sources are read unfolded
    constexpr int NBE = FOLD ? 0 : NB;
    auto take = [&](u64 i, const Raw &w, E2 (&lo)[NF], E2 (&hi)[NF], E2 &rest) {
#pragma unroll
        for (int f = 0; f < NF; f++) {
            if (FOLD) {
                if (TWO) {
                    auto comb = [&](U64x2 u, U64x2 v) {
                        gl::E2Acc t = gl::e2acc_zero();
                        gl::acc_mul_base(t, k2[0], u.x);
                        gl::acc_mul_base(t, k2[1], u.y);
                        gl::acc_mul_base(t, k2[2], v.x);
                        gl::acc_mul_base(t, k2[3], v.y);
                        return gl::acc_reduce(t);
                    };
                    lo[f] = comb(w.a0[f], w.b0[f]);
                    hi[f] = comb(w.c0[f], w.e0[f]);
                } else if (f < NB) {
                    lo[f] = fold1_base(w.a0[f].x, w.a0[f].y, r);
                    hi[f] = fold1_base(w.b0[f].x, w.b0[f].y, r);
                } else {
                    lo[f] = fold1p(gl::e2(w.a0[f].x, w.a1[f].x), gl::e2(w.a0[f].y, w.a1[f].y), rp);
                    hi[f] = fold1p(gl::e2(w.b0[f].x, w.b1[f].x), gl::e2(w.b0[f].y, w.b1[f].y), rp);
                }
                st2_stream(a.d0[f] + 2 * i, lo[f].c0, hi[f].c0);
                st2_stream(a.d1[f] + 2 * i, lo[f].c1, hi[f].c1);
            } else {
                if (f < NB) {
                    lo[f] = gl::e2(w.a0[f].x, 0);
                    hi[f] = gl::e2(w.a0[f].y, 0);
                } else {
                    lo[f] = gl::e2(w.a0[f].x, w.a1[f].x);
                    hi[f] = gl::e2(w.a0[f].y, w.a1[f].y);
                }
            }
        }
        rest = EQ ? gl::e2(w.q0, w.q1) : gl::e2_one();
    };
    auto evaluate = [&](const E2 (&lo)[NF], const E2 (&hi)[NF], E2 rest) {
        const gl::E2P restp = gl::prep(rest);
        E2 dl[NF];
#pragma unroll
        for (int f = 0; f < NF; f++) dl[f] = gl::sub(hi[f], lo[f]);
        // cur holds the factors at t: lo at 0, hi at 1, then hi + (t - 1) dl
        E2 cur[NF];
#pragma unroll
        for (int f = 0; f < NF; f++) cur[f] = lo[f];
#pragma unroll
        for (int t = 0; t < NP; t++) {
            if (!(t == 1 && skip1)) {
                if (NBE > 0) {
                    u64 b = cur[0].c0;
#pragma unroll
                    for (int f = 1; f < NBE; f++) b = (NBE == NF && EQ) ? gl::mul_any(b, cur[f].c0) : gl::mul(b, cur[f].c0);
                    if (NBE == NF) {
                        if (EQ)
                            gl::acc_mul_base(lz[t], rest, b);
                        else
                            gl::acc_add64(lz[t].c0, b);
                    } else {
                        E2 prod = gl::mul_base(cur[NBE], b);
#pragma unroll
                        for (int f = NBE + 1; f < NF; f++) prod = gl::mul(prod, cur[f]);
                        if (EQ)
                            gl::acc_mul(lz[t], prod, restp);
                        else
                            gl::acc_e2(lz[t], prod);
                    }
                } else {
                    E2 prod = cur[0];
#pragma unroll
                    for (int f = 1; f < NF; f++) prod = gl::mulp(prod, gl::prep(cur[f]));
                    if (EQ)
                        gl::acc_mul(lz[t], prod, restp);
                    else
                        gl::acc_e2(lz[t], prod);
                }
            }
            if (t + 1 < NP) {
#pragma unroll
                for (int f = 0; f < NF; f++) {
                    if (t == 0) {
                        cur[f] = hi[f];
                    } else {
                        cur[f].c0 = gl::add(cur[f].c0, dl[f].c0);
                        if (f >= NBE) cur[f].c1 = gl::add(cur[f].c1, dl[f].c1);
                    }
                }
            }
        }
    };
    const u64 stride = (u64)gridDim.x * BLOCK;
    u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (FOLD) {
        Raw w;
        // TWO: from the far end back.  The launch of the first two rounds has just walked the same tables upwards: what it
        // read last is what the memory-side cache still holds.
        u64 steps = 0;
        if (TWO) {
            steps = i < a.n_pairs ? (a.n_pairs - i + stride - 1) / stride : 0;
            if (steps) i += (steps - 1) * stride;
        }
        if (i < a.n_pairs) load_raw(i, w);
        if (a.wait_first) {
            // A launch made ahead of its round waits here for its challenge, with the operands of its first step already
            // requested (they do not depend on the challenge).  It leaves when no mail comes, or when the mail asks for the
            // other way of getting p(1), which is not compiled into this variant; the host then ends the launch.
            if (!wait_first_mail(a.mail, a.relay, blockIdx.x == 0, a.spin_limit, ff.seq, SKIP1 ? 0 : 1, box, &ok_flag)) return;
            if ((box[MAIL_SKIP1] != 0) != SKIP1) return;
            // (kept in scalar registers, as the kernel argument would be)
            r = gl::e2(uniform64(box[MAIL_R]), uniform64(box[MAIL_R + 1]));
            rp = gl::prep(r);
            if (TWO) set_two(gl::e2(uniform64(box[MAIL_RA]), uniform64(box[MAIL_RA + 1])), r);
        }
        if (TWO) {
            for (; steps > 0; steps--, i -= stride) {
                E2 lo[NF], hi[NF], rest;
                take(i, w, lo, hi, rest);
                if (steps > 1) load_raw(i - stride, w);
                evaluate(lo, hi, rest);
            }
        } else {
            for (; i < a.n_pairs; i += stride) {
                E2 lo[NF], hi[NF], rest;
                take(i, w, lo, hi, rest);
                if (i + stride < a.n_pairs) load_raw(i + stride, w);
                evaluate(lo, hi, rest);
            }
        }
    } else {
        auto step = [&](u64 i, const Raw &w) {
            E2 lo[NF], hi[NF], rest;
            take(i, w, lo, hi, rest);
            evaluate(lo, hi, rest);
        };
        // two operand sets used in turn, so that a step's loads are in flight during the whole previous step
        Raw wa, wb;
        if (i < a.n_pairs) load_raw(i, wa);
        while (i < a.n_pairs) {
            if (i + stride < a.n_pairs) load_raw(i + stride, wb);
            step(i, wa);
            i += stride;
            if (i >= a.n_pairs) break;
            if (i + stride < a.n_pairs) load_raw(i + stride, wa);
            step(i, wb);
            i += stride;
        }
    }
    E2 acc[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) acc[t] = gl::acc_reduce(lz[t]);
    if (FACT) {
        // the low part of the weight, the same for all pairs of this thread
        const u64 lo = ((u64)blockIdx.x * BLOCK + threadIdx.x) & ((1u << EQ_LO_BITS) - 1);
        const gl::E2P lp = gl::prep(gl::e2(a.lq0[lo], a.lq1[lo]));
#pragma unroll
        for (int t = 0; t < NP; t++)
            if (!(t == 1 && skip1)) acc[t] = gl::mulp(acc[t], lp);
    }
    block_reduce<NP>(acc, lds);
    if (gridDim.x == 1) {
        // a single workgroup: its sums are the round's sums, no partials and no ticket
        publish_sums<NP>(ff.out_host, ff.seq, ff.counter, acc);
        return;
    }
    if (ff.slots) {
        publish_sums<NP>(ff.slots + 64 * (u64)blockIdx.x, ff.seq, nullptr, acc);
        return;
    }
    if (threadIdx.x == 0) {
        u64 *o = partial + blockIdx.x;
        const u64 total = gridDim.x;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            st_agent(o + (2 * t) * total, acc[t].c0);
            st_agent(o + (2 * t + 1) * total, acc[t].c1);
        }
    }
    if (take_ticket(ff.counter, gridDim.x, &last_flag)) {
        E2 q[NP];
        gather_partials<NP>(ff, lds, q);
        publish_sums<NP>(ff.out_host, ff.seq, ff.counter, q);
    }
}

// sums over the wavefront of canonical values (as block_sum does it: 22-bit pieces added as integers), valid in lane 63
template <int NV>
__device__ __forceinline__ void wave_sum_field(u64 (&v)[NV])
{
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const u32 lo = (u32)v[i], hi = (u32)(v[i] >> 32);
        const u64 c0 = wave_sum_u32(lo & 0x3FFFFFu);
        const u64 c1 = wave_sum_u32((lo >> 22) | ((hi & 0xFFFu) << 10));
        const u64 c2 = wave_sum_u32(hi >> 12);
        const unsigned __int128 t = (unsigned __int128)c0 + ((unsigned __int128)c1 << 22) + ((unsigned __int128)c2 << 44);
        v[i] = gl::reduce128((u64)t, (u64)(t >> 64));
    }
}

// ---------------------------------------------------------------------------
// Two rounds of eq(rho, x) f(x) g(x) from one pass over tables that are two folds behind: quad_kernel.
//
// The launch reads the state of two rounds ago (the unfolded base-field tables behind pair12_kernel, SRC_BASE, or the
// extension tables the launch of this kind before it wrote), folds it twice on the way in with the two challenges
// drawn since, writes the state S of its first round, round j, and hands over what rounds j and j + 1 need: S is not read
// again until the launch after this one folds it twice in turn.
//
// Round j + 1's tables are S[2i] + c (S[2i+1] - S[2i]) with c the challenge of round j, not drawn yet: its sums are
// polynomials of degree 2 in c, known by their values at c = 0, 1 and their leading coefficient.  Per quad (S0..S3 of f,
// T0..T3 of g), everything weighted by R(m) = eq(rho_{j+2..}, m), m the quad's index:
//   A0 = S0 T0, A1 = S1 T1, Al = (S1 - S0)(T1 - T0)       round j + 1 at t = 0 as a polynomial in c; and the even pairs of
//                                                         round j: their q(0), q(1), leading coefficient
//   B0 = S2 T2, B2 = (2 S3 - S2)(2 T3 - T2)               the odd pairs of round j at t = 0 and t = 2
//   C0 = (2 S2 - S0)(2 T2 - T0), C1 = (2 S3 - S1)(2 T3 - T1), Cl = their differences' product
//                                                         round j + 1 at t = 2 as a polynomial in c
// Round j sums over the pairs of either kind, weighted by eq1(rho_{j+1}, .): the host has q_j(0) = (1 - rho) A0 + rho B0
// and q_j(2) = (1 - rho)(2 A1 - A0 + 2 Al) + rho B2; both rounds take p(1) from their claims (the host only plans this
// launch where the eq point allows that).  Eight products and eight sums a quad where two launches of prod_kernel make
// eight as well -- and one pass over memory less: the state of round j + 1 is never written or read.
// R(m) = hi[m >> 16] lo[m & 65535] as in the FACT variants of prod_kernel; the hi weight goes onto f's four entries
// (S~ = hi S, four products a quad, the weight in scalar registers) so that the eight products need none.
// ---------------------------------------------------------------------------
// One fold of an extension table into another buffer: dst[i] = src[2i] + r (src[2i+1] - src[2i]).  The catch-up step of a
// session whose launches of two rounds each are followed by ordinary launches after all (the state in memory is then a
// fold behind what those expect).
__global__ void __launch_bounds__(BLOCK) refold_kernel(const u64 *s0, const u64 *s1, u64 *d0, u64 *d1, u64 n_out, u64 r0, u64 r1)
{
    const gl::E2P rp = gl::prep(gl::e2(r0, r1));
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < n_out; i += (u64)gridDim.x * BLOCK) {
        const U64x2 x = ld2(s0 + 2 * i), y = ld2(s1 + 2 * i);
        const E2 v = fold1p(gl::e2(x.x, y.x), gl::e2(x.y, y.y), rp);
        d0[i] = v.c0;
        d1[i] = v.c1;
    }
}

constexpr int QUAD_SUMS = 8;  // handed over in this order: A0, A1, Al, B0, B2, C0, C1, Cl
static_assert(QUAD_SUMS <= MAX_PTS, "the sums fit a workgroup's partials and the result area");

// How the work of a workgroup's step -- QUAD_STEP quads, 4 QUAD_STEP entries of S per table -- is spread over its 256
// lanes: first every lane makes two adjacent entries of S of one table (wavefronts 0 and 1 the first table's, 2 and 3 the
// second's: 8 source entries, coalesced 16-byte loads, two 16-byte stores) and leaves them in LDS; after a barrier
// wavefront w takes two of the eight products of every quad (lane = quad), reading the entries it needs from LDS, where
// entry c of quad q of a table lies at [c][q] so that a wavefront's reads are conflict-free.  Short chains of dependent
// arithmetic in many wavefronts (about 100 registers, four or five wavefronts per SIMD) instead of a lane per quad with
// 250 registers and two: the launch is bound by the latency of those chains, not by their number.  The loads of the
// next step are in flight while the products of this one are made; LDS holds two steps' entries, one barrier a step.
constexpr int QUAD_STEP = 64;
static_assert(BLOCK == 4 * QUAD_STEP && BLOCK == 4 * WAVE, "a lane per quad in each of four wavefronts");

template <bool SRC_BASE>
__global__ void __launch_bounds__(BLOCK) quad_kernel(ProdArgs a, u64 *__restrict__ partial, FastFin ff)
{
    constexpr int NS = QUAD_SUMS;
    __shared__ u64 ent[2][2][4][QUAD_STEP][2];  // [step parity][table][entry of the quad][quad][limb]
    __shared__ u64 own[2 * NS];
    __shared__ int last_flag;
    __shared__ u64 box[MAIL_WORDS];
    __shared__ int ok_flag;
    const u32 tid = threadIdx.x, lane = tid & (WAVE - 1);
    const u32 wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    // making the entries: this lane's table, and which two adjacent entries of the step's 4 QUAD_STEP
    const u32 tab = wave >> 1, pi = tid & (2 * WAVE - 1);
    const u64 *src0 = a.s0[tab], *src1 = a.s1[tab];
    u64 *dst0 = a.d0[tab], *dst1 = a.d1[tab];
    const u64 n_quads = a.n_pairs;
    const u64 stride = (u64)gridDim.x * QUAD_STEP;
    u64 m0 = (u64)blockIdx.x * QUAD_STEP;  // first quad of the step in hand
    struct Raw {
        U64x2 x[4] = {}, y[4] = {};
    };
    auto load_raw = [&](u64 first_quad, Raw &w) {
        // entries 2 pi, 2 pi + 1 of the step are made of 8 source entries
        const u64 e = 16 * first_quad + 8 * (u64)pi;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            w.x[c] = ld2(src0 + e + 2 * c);
            if (!SRC_BASE) w.y[c] = ld2(src1 + e + 2 * c);
        }
    };
    Raw raw;
    if (m0 < n_quads) load_raw(m0, raw);
    E2 ra = gl::e2(a.ra0, a.ra1), rb = gl::e2(a.r0, a.r1);
    if (a.wait_first) {
        // made ahead of its round: both challenges come by mail (the one of the round before this launch's first, and
        // the one before that); the first step's loads are on their way meanwhile
        if (!wait_first_mail(a.mail, a.relay, blockIdx.x == 0, a.spin_limit, ff.seq, 0, box, &ok_flag)) return;
        if (box[MAIL_SKIP1] != 1) return;
        rb = gl::e2(uniform64(box[MAIL_R]), uniform64(box[MAIL_R + 1]));
        ra = gl::e2(uniform64(box[MAIL_RA]), uniform64(box[MAIL_RA + 1]));
    }
    // an entry of S is sum_ab e_a(ra) e_b(rb) x[a + 2 b] over four source entries, e_0(c) = 1 - c, e_1(c) = c
    E2 k2[4];
    gl::E2P k2p[4];
    {
        const E2 na = gl::sub(gl::e2_one(), ra), nb = gl::sub(gl::e2_one(), rb);
        k2[0] = gl::mul(na, nb), k2[1] = gl::mul(ra, nb), k2[2] = gl::mul(na, rb), k2[3] = gl::mul(ra, rb);
#pragma unroll
        for (int k = 0; k < 4; k++) k2p[k] = gl::prep(k2[k]);
    }
    // sums 2 wave and 2 wave + 1, unreduced (two a lane: their registers are affordable, a reduction per product is not)
    gl::E2Acc acc0 = gl::e2acc_zero(), acc1 = gl::e2acc_zero();
    u32 parity = 0;
    for (; m0 < n_quads; m0 += stride, parity ^= 1) {
        // ---- two entries of S of this lane's table ----
        E2 v[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if (SRC_BASE) {
                gl::E2Acc t = gl::e2acc_zero();
                gl::acc_mul_base(t, k2[0], raw.x[2 * h].x);
                gl::acc_mul_base(t, k2[1], raw.x[2 * h].y);
                gl::acc_mul_base(t, k2[2], raw.x[2 * h + 1].x);
                gl::acc_mul_base(t, k2[3], raw.x[2 * h + 1].y);
                v[h] = gl::acc_reduce(t);
            } else {
                // the same combination of extension entries: sixteen products gathered unreduced and two reductions,
                // where three folds one after the other are twelve products and six reductions
                gl::E2Acc t = gl::e2acc_zero();
                gl::acc_mul(t, gl::e2(raw.x[2 * h].x, raw.y[2 * h].x), k2p[0]);
                gl::acc_mul(t, gl::e2(raw.x[2 * h].y, raw.y[2 * h].y), k2p[1]);
                gl::acc_mul(t, gl::e2(raw.x[2 * h + 1].x, raw.y[2 * h + 1].x), k2p[2]);
                gl::acc_mul(t, gl::e2(raw.x[2 * h + 1].y, raw.y[2 * h + 1].y), k2p[3]);
                v[h] = gl::acc_reduce(t);
            }
        }
        {
            const u64 e = 4 * m0 + 2 * (u64)pi;
            st2_stream(dst0 + e, v[0].c0, v[1].c0);
            st2_stream(dst1 + e, v[0].c1, v[1].c1);
        }
        // the next step's source entries, on their way while this step's products are made
        if (m0 + stride < n_quads) load_raw(m0 + stride, raw);
        if (tab == 0) {
            // the high part of the weight goes onto the first table's entries: the same for the whole workgroup's step
            const u32 hi = __builtin_amdgcn_readfirstlane((u32)(m0 >> EQ_LO_BITS));
            const gl::E2P hp = gl::prep(gl::e2(a.hq0[hi], a.hq1[hi]));
            v[0] = gl::mulp(v[0], hp);
            v[1] = gl::mulp(v[1], hp);
        }
        {
            const u32 q = pi >> 1, c = 2 * (pi & 1);
            ent[parity][tab][c][q][0] = v[0].c0;
            ent[parity][tab][c][q][1] = v[0].c1;
            ent[parity][tab][c + 1][q][0] = v[1].c0;
            ent[parity][tab][c + 1][q][1] = v[1].c1;
        }
        __syncthreads();
        // ---- two of the eight products of quad `lane` ----
        auto S = [&](int c) { return gl::e2(ent[parity][0][c][lane][0], ent[parity][0][c][lane][1]); };
        auto T = [&](int c) { return gl::e2(ent[parity][1][c][lane][0], ent[parity][1][c][lane][1]); };
        auto twice_less = [](E2 x, E2 y) { return gl::sub(gl::add(x, x), y); };  // 2 x - y
        if (m0 + lane < n_quads) {
            if (wave == 0) {
                gl::acc_mul(acc0, S(0), gl::prep(T(0)));  // A0
                gl::acc_mul(acc1, S(1), gl::prep(T(1)));  // A1
            } else if (wave == 1) {
                gl::acc_mul(acc0, gl::sub(S(1), S(0)), gl::prep(gl::sub(T(1), T(0))));  // Al
                gl::acc_mul(acc1, S(2), gl::prep(T(2)));                                // B0
            } else if (wave == 2) {
                gl::acc_mul(acc0, twice_less(S(3), S(2)), gl::prep(twice_less(T(3), T(2))));  // B2
                gl::acc_mul(acc1, twice_less(S(2), S(0)), gl::prep(twice_less(T(2), T(0))));  // C0
            } else {
                const E2 cs0 = twice_less(S(2), S(0)), cs1 = twice_less(S(3), S(1));
                const E2 ct0 = twice_less(T(2), T(0)), ct1 = twice_less(T(3), T(1));
                gl::acc_mul(acc0, cs1, gl::prep(ct1));                              // C1
                gl::acc_mul(acc1, gl::sub(cs1, cs0), gl::prep(gl::sub(ct1, ct0)));  // Cl
            }
        }
    }
    // the low part of the weight, the same for all quads of this lane (the grid's stride is a multiple of 2^EQ_LO_BITS)
    u64 w4[4];
    {
        const u64 lo = ((u64)blockIdx.x * QUAD_STEP + lane) & ((1u << EQ_LO_BITS) - 1);
        const gl::E2P lp = gl::prep(gl::e2(a.lq0[lo], a.lq1[lo]));
        const E2 s0 = gl::mulp(gl::acc_reduce(acc0), lp), s1 = gl::mulp(gl::acc_reduce(acc1), lp);
        w4[0] = s0.c0, w4[1] = s0.c1, w4[2] = s1.c0, w4[3] = s1.c1;
    }
    // the wavefront's two sums: words 4 wave .. 4 wave + 3 of the workgroup's 16
    wave_sum_field<4>(w4);
    auto publish = [&](const u64 *w) {
        if (ff.counter) *ff.counter = 0;
        publish_words(ff.out_host, 0, w, 2 * NS, ff.seq);
    };
    if (gridDim.x == 1) {
        if (lane == WAVE - 1)
#pragma unroll
            for (int k = 0; k < 4; k++) own[4 * wave + k] = w4[k];
        __syncthreads();
        if (tid == 0) publish(own);
        return;
    }
    if (lane == WAVE - 1) {
        u64 *o = partial + blockIdx.x;
        const u64 total = gridDim.x;
#pragma unroll
        for (int k = 0; k < 4; k++) st_agent(o + (u64)(4 * wave + k) * total, w4[k]);
    }
    // (every wavefront's stores acknowledged before the workgroup's ticket is taken)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (take_ticket(ff.counter, gridDim.x, &last_flag) && wave == 0) {
        // the last workgroup's first wavefront adds up the workgroups' words
        u64 sum[2 * NS];
#pragma unroll
        for (int k = 0; k < 2 * NS; k++) sum[k] = 0;
        for (u32 b = lane; b < gridDim.x; b += WAVE) {
#pragma unroll
            for (int k = 0; k < 2 * NS; k++) sum[k] = gl::add(sum[k], ld_agent(partial + (u64)k * gridDim.x + b));
        }
        wave_sum_field<2 * NS>(sum);
        if (lane == WAVE - 1) publish(sum);
    }
}

// ---------------------------------------------------------------------------
// The first two rounds of eq(rho, x) f(x) g(x), f and g in the base field, from one pass over the tables.
//
// With the lowest variable x0 bound to a challenge c, a table's value at (c, x1, x') is linear in c, so round 2's sums
// are a polynomial of degree 2 in the challenge round 1 has not drawn yet: the kernel hands over its values at c = 0, 1 and
// its leading coefficient, and the host evaluates it when the challenge is there.  All of it is base-field arithmetic on
// the entries as stored: a quad (f00, f10, f01, f11) = f[4 x' + x0 + 2 x1] and the same of g give, all weighted by
// R(x') = eq(rho_3.., x'),
//   pair x1 = 0:  f00 g00,  f10 g10,  (f10 - f00)(g10 - g00)       (round 1's q(0), q(1) and leading coefficient over the
//   pair x1 = 1:  f01 g01,  f11 g11,  (f11 - f01)(g11 - g01)        pairs of either kind: the host weights them with
//                                                                  1 - rho_2 and rho_2; and round 2 at t = 0, pair 0 alone)
//   the slopes along x1, D_a = f_a1 - f_a0, E_a likewise:  D0 E0,  D1 E1,  (D1 - D0)(E1 - E0)
// (each of the three products is a quadratic in x1 known at 0 and at 1: with its leading coefficient the host has it at
// x1 = 2, which is round 2 at t = 2: 2 (row 1) - (row 0) + 2 (row 2)).
// Nine products where round 1 alone takes six, each row the same three products of a pair of values.  A workgroup is
// three wavefronts that walk the same quads, one row each (three unreduced sums a lane, as in round 1's kernel; the
// quad comes from HBM once and twice more from the caches).  R is taken as in the FACT variants of prod_kernel:
// hi[x' >> 16], the same for a workgroup's step, weights the products; lo[x' & 0xFFFF], the same for all steps of a
// lane (the grid's stride, 64 quads a workgroup, is a multiple of 2^16), weights the sums.  Round 3 then reads the same
// tables again and folds them twice on the way in (prod_kernel's TWO variant): nothing is written for the first two rounds.
// ---------------------------------------------------------------------------
struct Pair12Args {
    const u64 *f, *g;
    u64 n_quads;
    const u64 *lq0, *lq1, *hq0, *hq1;
};
constexpr int PAIR12_BLOCK = 3 * WAVE;
constexpr int PAIR12_SUMS = 9;  // handed to the host in this order: pair 0's three, pair 1's three, the three of the slopes along x1
constexpr int PAIR12_SEQ_SLOT = 62, PAIR12_CHK_SLOT = 63;
constexpr u32 PAIR12_LEAD = 4, PAIR12_LEAD_SPINS = 1u << 16;  // steps the other rows may be ahead of row 2; polls before they go on anyway
static_assert(2 * PAIR12_SUMS <= PAIR12_SEQ_SLOT, "the sums fit the result area");

__global__ void __launch_bounds__(PAIR12_BLOCK) pair12_kernel(Pair12Args a, u64 *__restrict__ partial, FastFin ff)
{
    __shared__ int last_flag;
    __shared__ u32 row2_done;  // steps the wavefront of row 2 has behind it
    // A lane's three sums of (product) x (high weight), unreduced, their carries counted (gl::E2Acc).  Sums without carries
    // (the weight's limbs cut into 22-bit pieces, six multiply-adds per product and limb and nothing else) make the loop
    // 7 % shorter and cost 22 more registers -- 136, a few more than four wavefronts per SIMD allow.  Three per SIMD is
    // exactly what this launch's 1024 workgroups of three wavefronts fill the GPU with, with no room to spare: behind
    // a launch of a few workgroups (which every launch is that a caller makes before a proof, the eq build among them) the
    // dispatcher places some workgroups where they have to wait for others to finish, and the launch takes 105 us instead
    // of 80.  With room for a fourth wavefront it takes 86 to 90 us wherever its workgroups land.
    gl::E2Acc lz[3];
#pragma unroll
    for (int k = 0; k < 3; k++) lz[k] = gl::e2acc_zero();
    const u32 lane = threadIdx.x & (WAVE - 1);
    const u32 row = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const u64 stride = (u64)gridDim.x * WAVE;
    const u64 q0 = (u64)blockIdx.x * WAVE + lane;
    // The loop, compiled once for rows 0 and 1 (their own pair: two loads) and once for row 2 (the whole quad, and the
    // slopes along x1 made of it): a wavefront takes one or the other, no lane pays for both.
    auto run = [&](auto last_row) {
        constexpr bool ROW2 = decltype(last_row)::value;
        struct Raw {
            U64x2 f0 = {}, f1 = {}, g0 = {}, g1 = {};
            u64 h0 = 0, h1 = 0;
        };
        auto load_raw = [&](u64 q, Raw &w) {
            if (ROW2) {
                w.f0 = ld2(a.f + 4 * q);
                w.f1 = ld2(a.f + 4 * q + 2);
                w.g0 = ld2(a.g + 4 * q);
                w.g1 = ld2(a.g + 4 * q + 2);
            } else {
                w.f0 = ld2(a.f + 4 * q + 2 * row);
                w.g0 = ld2(a.g + 4 * q + 2 * row);
            }
            // the same entry for the whole workgroup (its 64 quads lie within one run of 2^16)
            const u32 hi = __builtin_amdgcn_readfirstlane((u32)(q >> EQ_LO_BITS));
            w.h0 = a.hq0[hi];
            w.h1 = a.hq1[hi];
        };
        auto step = [&](const Raw &w) {
            u64 fl = w.f0.x, fh = w.f0.y, gl_ = w.g0.x, gh = w.g0.y;
            if (ROW2) {
                // the slopes along x1, at x0 = 0 and at x0 = 1
                fl = gl::sub(w.f1.x, w.f0.x);
                fh = gl::sub(w.f1.y, w.f0.y);
                gl_ = gl::sub(w.g1.x, w.g0.x);
                gh = gl::sub(w.g1.y, w.g0.y);
            }
            const E2 H = gl::e2(w.h0, w.h1);
            gl::acc_mul_base(lz[0], H, gl::mul_any(fl, gl_));
            gl::acc_mul_base(lz[1], H, gl::mul_any(fh, gh));
            gl::acc_mul_base(lz[2], H, gl::mul_any(gl::sub(fh, fl), gl::sub(gh, gl_)));
        };
        // two operand sets used in turn, so that a step's loads are in flight during the whole previous step
        // Row 2's steps are the dearer ones: left alone the other two wavefronts run ahead of it until the lines they
        // have read are gone from the L2 when it asks for them (1.5 x the tables fetched).  So it says how far it is (a
        // word in LDS, every second step), and the others do not go more than PAIR12_LEAD steps beyond that: they sleep,
        // which leaves their SIMDs to the wavefronts that are behind.  The wait is bounded: only the traffic depends on it.
        u64 q = q0;
        u32 done = 0;  // steps of this wavefront
        Raw wa, wb;
        if (q < a.n_quads) load_raw(q, wa);
        while (q < a.n_quads) {
            if (!ROW2) {
                for (u32 spin = 0; spin < PAIR12_LEAD_SPINS && __hip_atomic_load(&row2_done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) + PAIR12_LEAD < done; spin++)
                    __builtin_amdgcn_s_sleep(2);
            }
            if (q + stride < a.n_quads) load_raw(q + stride, wb);
            step(wa);
            q += stride;
            done += 2;
            if (q < a.n_quads) {
                if (q + stride < a.n_quads) load_raw(q + stride, wa);
                step(wb);
                q += stride;
            }
            if (ROW2 && lane == 0) __hip_atomic_store(&row2_done, done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        // (a wavefront of row 2 that is through lets the others run to their end)
        if (ROW2 && lane == 0) __hip_atomic_store(&row2_done, 0x7FFFFFFFu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    if (threadIdx.x == 0) row2_done = 0;
    __syncthreads();
    if (row == 2)
        run(std::true_type{});
    else
        run(std::false_type{});
    // the low part of the weight, then the wavefront's three sums: words 6 row .. 6 row + 5 of the workgroup's 18
    const u32 lo = (u32)q0 & ((1u << EQ_LO_BITS) - 1);
    const gl::E2P lp = gl::prep(gl::e2(a.lq0[lo], a.lq1[lo]));
    u64 v[6];
#pragma unroll
    for (int k = 0; k < 3; k++) {
        const E2 x = q0 < a.n_quads ? gl::mulp(gl::acc_reduce(lz[k]), lp) : gl::e2_zero();
        v[2 * k] = x.c0, v[2 * k + 1] = x.c1;
    }
    wave_sum_field<6>(v);
    auto publish = [&](const u64 *w) {
        if (ff.counter) *ff.counter = 0;
        publish_words(ff.out_host, 0, w, 2 * PAIR12_SUMS, ff.seq, PAIR12_SEQ_SLOT, PAIR12_CHK_SLOT);
    };
    __shared__ u64 own[2 * PAIR12_SUMS];
    if (gridDim.x == 1) {
        if (lane == WAVE - 1)
#pragma unroll
            for (int k = 0; k < 6; k++) own[6 * row + k] = v[k];
        __syncthreads();
        if (threadIdx.x == 0) publish(own);
        return;
    }
    if (lane == WAVE - 1) {
        u64 *o = partial + blockIdx.x;
        const u64 total = gridDim.x;
#pragma unroll
        for (int k = 0; k < 6; k++) st_agent(o + (u64)(6 * row + k) * total, v[k]);
    }
    // (every wavefront's stores acknowledged before the workgroup's ticket is taken)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (take_ticket(ff.counter, gridDim.x, &last_flag) && row == 0) {
        // the last workgroup's first wavefront adds up the workgroups' words
        u64 s[2 * PAIR12_SUMS];
#pragma unroll
        for (int k = 0; k < 2 * PAIR12_SUMS; k++) s[k] = 0;
        for (u32 b = lane; b < gridDim.x; b += WAVE) {
#pragma unroll
            for (int k = 0; k < 2 * PAIR12_SUMS; k++) s[k] = gl::add(s[k], ld_agent(partial + (u64)k * gridDim.x + b));
        }
        wave_sum_field<2 * PAIR12_SUMS>(s);
        if (lane == WAVE - 1) publish(s);
    }
}

// ---------------------------------------------------------------------------
// slice kernel: the rounds of a product sumcheck that are latency, not bytes
//
// Once a round moves a few megabytes a launch per round is pure latency (dispatch, a wavefront's instruction stream,
// the hand-off to the host and back).  From there on the tables live in LDS: every workgroup of this launch owns a
// contiguous slice of every table -- binding the lowest variable turns entries 2i, 2i+1 into entry i, so what a
// workgroup needs in the next round is what it has just made -- and stays on the GPU, waiting for each challenge in
// the host's mailbox.  With one workgroup it runs to its last trip (the session's last round, or a few rounds before it:
// the host does those from the entries the trip leaves it); with several it runs until a workgroup is down to an entry or
// two per table, leaves them in device memory (`h0/h1`) and the first workgroup, or a launch queued behind, goes on.
//
// A trip to the host can cover two rounds.  With S the state of round j (pairs (S[2i], S[2i+1])), the tables of round
// j+1 are S[2i] + r_j (S[2i+1] - S[2i]): linear in the challenge r_j that is not known yet, so the sums of round j+1
//     q_{j+1}(t) = sum_x R_{j+1}(x) prod_f f_{j+1}(t, x)
// are a polynomial of degree NF in r_j.  Besides q_j(t) the kernel hands over that polynomial's values at r_j = 0..NF-1
// and its leading coefficient (each is the same sum over quads of S with the pair (S[4i], S[4i+2]), (S[4i+1], S[4i+3]),
// ... or the differences in place of the folded pair).  The host draws r_j from message j, evaluates the polynomial
// there, forms message j+1 and draws r_{j+1} without the GPU; the next mail carries both challenges and the kernel
// folds twice.  Same field elements as one round at a time; half the trips.
//
// Sums are added up as plain integers: a lane's canonical sums are cut into 32-bit halves and added into 64-bit
// counters, per wavefront in LDS, then per launch in device memory: one agent-scope atomic add per workgroup and counter,
// which adds the workgroup's share to the low 56 bits and one to the top byte.  The counters are never cleared during a
// launch (the host subtracts what the trip before left there; 2^10 lanes x 2^8 workgroups x 2^5 trips of 32-bit values stay
// below 2^56), so the top byte counts the adds: the workgroup whose add makes it a multiple of the number of workgroups has
// been handed, by that same atomic, the sum of everyone else's shares, and passes the total straight on to the host.  No
// ticket, no fence, no second trip through device memory.  The host recombines the halves and reduces.
// The adds to one counter are served one after the other (11 ns each, measured), and so are adds to neighbouring words:
// every counter has 256 bytes of its own, and the workgroups of a large launch add into up to SL_MAX_GROUPS sets of
// counters (workgroup w into set w mod G), each set complete with its own last add and handed to the host in an area of
// its own; the host adds the sets up.  (256 workgroups, 36 counters: the last add returned 6 us after the workgroups'
// sums were ready with one set of adjacent words, 3 us with the words apart, 1.5 us with eight sets.)
// ---------------------------------------------------------------------------
constexpr int SL_MAX_SUMS = 25;  // (NF + 1)^2 extension sums per trip at NF = 4
constexpr u32 SL_CTR_STRIDE = 32;  // 64-bit words from one counter in device memory to the next
constexpr u32 SL_MAX_GROUPS = 8;   // sets of counters (and result areas) of one launch
// A trip's result: the 4 counters of every sum (32-bit halves of both limbs, added up as integers), one word each in the
// first 4 * SL_MAX_SUMS words of the result area: the count in the low 56 bits, the trip's tag in the top byte.  A word
// is one store, so it is whole when its tag is there; the host clears the tags it has taken.
constexpr u64 SL_CTR_MASK = (1ull << 56) - 1, SL_CTR_ONE = 1ull << 56;
__host__ __device__ __forceinline__ u64 sl_tag(u64 trip_seq) { return 0x80 | (trip_seq & 0x7F); }
// With its last trip a launch that hands the session's end to the host leaves the state of that trip's first round: every
// table's entries, in an area of their own (`fin_out`: SL_FIN_MAX_WORDS words, then the trip's sequence number and a
// check word).  The host folds them with the challenges it has drawn since and does what is left: the last fold, or a
// few rounds of a handful of pairs, which cost it less than a trip costs.
constexpr int SL_GROUP_WORDS = 4 * SL_MAX_SUMS;  // a set's part of the result area
constexpr int SL_AREA_WORDS = SL_GROUP_WORDS * (int)SL_MAX_GROUPS + 32;
// (behind the sets: where the first workgroup says which mail it is waiting for and which it has had last -- read by the
// host only to say more when a result does not come)
constexpr int SL_WAITING_SLOT = SL_GROUP_WORDS * (int)SL_MAX_GROUPS, SL_HAD_SLOT = SL_WAITING_SLOT + 1;
constexpr int SL_FIN_MAX_WORDS = 1024, SL_FIN_SEQ_SLOT = SL_FIN_MAX_WORDS, SL_FIN_CHK_SLOT = SL_FIN_MAX_WORDS + 1, SL_FIN_AREA_WORDS = SL_FIN_MAX_WORDS + 2;
constexpr int SL_MAX_TRIPS = 32;
constexpr int SL_MAX_TABS = 16;   // tables of a sum of several terms (a product has at most 3)
constexpr int SL_MAX_TERMS = 24;
static_assert(2 * 4 * SL_MAX_TABS <= SL_FIN_MAX_WORDS, "the last entries of every table fit their area");
// the check word's share of word i of that area
__host__ __device__ __forceinline__ u64 sl_fin_mix(u64 word, u32 i) { return rotl64(word, (i & 31) + 1); }
// a term of a sum of several terms: coefficient (prepared: w = 7 c1) times the tables in `slot`
struct SliceTerm {
    u64 c0, c1, w;
    u32 n_factors;
    uint8_t slot[DPS_MAX_FACTORS];
    u32 pad;
};
struct SliceArgs {
    const u64 *s0[SL_MAX_TABS];
    const u64 *s1[SL_MAX_TABS];  // the tables before the folds that are pending when the launch starts: src_len entries each
                                 // (nullptr: base-field entries; only tables nothing has folded yet are)
    u64 src_len;
    u32 pend0;         // folds pending at the first trip: 0 (the launch starts with round 1), 1, or 2
    u32 n_vars, j0;    // the sum's variables; first round evaluated here (1-based)
    u32 n_trips;
    u32 dbl_mask;      // bit k: trip k covers two rounds
    // several workgroups: after their n_trips trips the tables (an entry or a few per workgroup) go to h0 / h1, the first
    // workgroup waits for all of them at the gate, takes them up with the pending folds and goes on alone for n_trips2 trips
    u32 n_trips2;
    u32 dbl_mask2;
    const u64 *eq0;    // eq storage, level 0 at entry 0 (eq factor only)
    const u64 *eq1;
    const u64 *mail;   // host mailbox
    u64 *relay;        // several workgroups: the first passes each mail on through these words of device memory
    u32 spin_limit;
    u32 finish;        // the launch's last trip is the last of the session's launches: the state of that trip's first round goes to
                       // the host (fin_out) with it; else what is left goes to h0 / h1
    u32 first_go;      // a launch that starts with round 1 (nothing pending), made when that round is due: its first trip starts
                       // without a look into the mailbox; 1: t = 1 is evaluated, 2: it comes from the claim.  0: every trip waits for its mail
    u32 groups_log;    // several workgroups: they add into 2^groups_log sets of counters (workgroup w into set w mod 2^groups_log)
    u64 *out_host;     // result area of SL_AREA_WORDS words: SL_GROUP_WORDS per set of counters
    u64 *fin_out;      // ... and the area of SL_FIN_AREA_WORDS words for the entries left with the last trip (finish)
    u64 seq0;          // sequence number of the trip that starts at round j0; the one that starts at round j has seq0 + (j - j0)
    u64 *ctr;          // several workgroups: SL_MAX_GROUPS * 4 * SL_MAX_SUMS counters in device memory, SL_CTR_STRIDE words apart, zero when the launch starts
    u32 *gate;         // ... and the count of workgroups that have left their tables in h0 / h1 (zero when the launch starts)
    u64 *h0[SL_MAX_TABS];  // where each workgroup leaves its last state (workgroup-major): for the first workgroup to go on with,
    u64 *h1[SL_MAX_TABS];  // or (a launch that ends before the last round) for the launch queued behind this one
    u64 *hw0, *hw1;        // ... and its eq weights (eq factor only; half as many entries), for the first workgroup to go on with
    // a sum of several terms (TERMS): the tables are those of all terms, the polynomial summed is sum_k coeff_k prod table
    u32 n_tabs, n_terms;
    SliceTerm terms[SL_MAX_TERMS];
};

// dynamic LDS of slice_kernel, in 64-bit words: counters per wavefront, mailbox copy, flags, the terms, then the two table buffers
// (`blk`: threads of a workgroup)
constexpr u32 SL_LDS_CTR = 0;
__host__ __device__ constexpr u32 sl_lds_box(u32 blk) { return (blk / WAVE) * 4 * SL_MAX_SUMS; }
__host__ __device__ constexpr u32 sl_lds_flags(u32 blk) { return sl_lds_box(blk) + 8; }
__host__ __device__ constexpr u32 sl_lds_terms(u32 blk) { return sl_lds_flags(blk) + 2; }
__host__ __device__ constexpr u32 sl_lds_tables(u32 blk) { return sl_lds_terms(blk) + SL_MAX_TERMS * (sizeof(SliceTerm) / 8); }
static_assert(sizeof(SliceTerm) % 8 == 0, "terms are copied as 64-bit words");
// (`eq`: the weights of the eq factor, one per pair of a table's entries, are kept like a table of half the size)
__host__ __device__ constexpr u32 sl_weights_cap(u32 cap) { return cap / 2 > 0 ? cap / 2 : 1; }
__host__ __device__ constexpr u32 slice_lds_words(u32 n_tabs, u32 cap, u32 blk, bool eq)
{
    return sl_lds_tables(blk) + n_tabs * 2 * (cap + cap / 2) + (eq ? 2 * (sl_weights_cap(cap) + sl_weights_cap(cap / 2)) : 0);
}
// A workgroup of these launches is 1024 threads: what a round costs here is the longest chain of dependent field
// multiplications in any one lane, and with more lanes each has fewer units of work behind one another.
constexpr int SL_BLOCK = 1024;
constexpr int SL_PRE = 2;  // items (table, entry) a thread of a launch made ahead asks for before it waits for its first mail

// NF: tables of the product, or with TERMS the largest number of factors of a term (the degree of the polynomial summed)
// BLK: threads of a workgroup (SL_BLOCK in the library; the kernel's CPU test runs smaller ones)
template <int NF, bool EQ, bool TERMS, int BLK = SL_BLOCK>
__global__ void __launch_bounds__(BLK) slice_kernel(SliceArgs a)
{
    constexpr int BLOCK = BLK;
    constexpr u32 SL_LDS_BOX = sl_lds_box(BLK), SL_LDS_FLAGS = sl_lds_flags(BLK), SL_LDS_TERMS = sl_lds_terms(BLK), SL_LDS_TABLES = sl_lds_tables(BLK);
    constexpr int NP = NF + 1;          // sums of the trip's first round: q(0..NF), q(1) left zero when it comes from the claim
    constexpr int NPT = NF;             // points of its second round: t = 0, 2, .., NF
    constexpr int NSMP = NF + 1;        // samples of that round's sums as a polynomial in the challenge: 0..NF-1, leading coefficient
    constexpr int NS = NP + NSMP * NPT; // extension sums per trip
    static_assert(NS <= SL_MAX_SUMS && 4 * NS <= BLK, "sums per trip fit the result area, their counters one lane each");
    extern __shared__ u64 dyn[];
    u64 *const ctr = dyn + SL_LDS_CTR;  // [wavefront][4 * SL_MAX_SUMS]
    u64 *const box = dyn + SL_LDS_BOX;
    int *const ok_flag = reinterpret_cast<int *>(dyn + SL_LDS_FLAGS);
    const SliceTerm *const lterms = reinterpret_cast<const SliceTerm *>(dyn + SL_LDS_TERMS);
    const u32 tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const u32 W = gridDim.x, wg = blockIdx.x;
    const u32 nt = TERMS ? a.n_tabs : (u32)NF;  // tables
    const u64 src_wg = a.src_len / W;             // this workgroup's share of the source
    u32 len = (u32)(src_wg >> a.pend0);           // entries per table once the pending folds are done
    const u32 cap = len;
    u32 len_log = (u32)__builtin_ctz(len);      // a workgroup's share is a power of two
    // two buffers per limb array: `cap` entries and half of that; a fold reads one and writes the other
    u64 *const buf_big = dyn + SL_LDS_TABLES, *const buf_small = buf_big + (size_t)nt * 2 * cap;
    bool in_big = true;  // where the current state is
    auto tab = [&](bool big, u32 f, int limb) -> u64 * { return big ? buf_big + (size_t)(f * 2 + limb) * cap : buf_small + (size_t)(f * 2 + limb) * (cap / 2); };
    // The weights of the eq factor, R_j(p) = eq(rho_{j+1..}, p) for the pairs p of round j, live beside the tables in the
    // same two buffers: read once when the launch starts, and from round to round the weight of a pair is the sum of the
    // weights of the two pairs it is made of (R_{j+1}(p) = R_j(2p) + R_j(2p + 1)), so a fold of the tables is an add here.
    u64 *const wts_big = buf_small + (size_t)nt * 2 * (cap / 2), *const wts_small = wts_big + 2 * sl_weights_cap(cap);
    auto wts = [&](bool big, int limb) -> u64 * { return big ? wts_big + (size_t)limb * sl_weights_cap(cap) : wts_small + (size_t)limb * sl_weights_cap(cap / 2); };
    auto weight = [&](bool big, u32 p) { return gl::e2(wts(big, 0)[p], wts(big, 1)[p]); };
    if (TERMS) {
        // the terms are read per pair and point: staged in LDS once (visible after the first wait's barrier)
        const u64 *src = reinterpret_cast<const u64 *>(a.terms);
        u64 *dst = dyn + SL_LDS_TERMS;
        for (u32 w = tid; w < a.n_terms * (u32)(sizeof(SliceTerm) / 8); w += BLOCK) dst[w] = src[w];
    }

    // lanes that share a pair (a quad) at one evaluation point split the terms among them
    const u32 p_split = TERMS ? a.n_terms : 1u;
    const u32 q_split = TERMS ? (a.n_terms * (u32)(NPT * NSMP) <= (u32)BLOCK ? a.n_terms : 1u) : 1u;
    u32 j = a.j0, pend = a.pend0;
    u64 trip_seq = a.seq0;
    u32 Wc = W;  // workgroups still at work
    for (u32 k = 0; k < a.n_trips + a.n_trips2; k++) {
        const bool regroup = k > 0 && k == a.n_trips;
        const bool dbl = ((k < a.n_trips ? a.dbl_mask >> k : a.dbl_mask2 >> (k - a.n_trips)) & 1) != 0;
        u64 src_each = src_wg;  // entries of the source a workgroup takes up (k == 0, or the first workgroup when regrouping)
        if (regroup) {
            // every workgroup leaves its entries in device memory: stores that go through to where every compute unit
            // reads (a release fence at device scope would write back the whole L2, from every wavefront of the launch:
            // 30 us at 256 workgroups), acknowledged to each lane before the workgroup is counted at the gate
            for (u32 u = tid; u < (nt << len_log); u += BLOCK) {
                const u32 f = u >> len_log, i = u & (len - 1);
                st_agent(a.h0[f] + (u64)wg * len + i, tab(in_big, f, 0)[i]);
                st_agent(a.h1[f] + (u64)wg * len + i, tab(in_big, f, 1)[i]);
            }
            if (EQ)
                for (u32 i = tid; i < (len >> 1); i += BLOCK) {
                    st_agent(a.hw0 + (u64)wg * (len >> 1) + i, wts(in_big, 0)[i]);
                    st_agent(a.hw1 + (u64)wg * (len >> 1) + i, wts(in_big, 1)[i]);
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            if (tid == 0) __hip_atomic_fetch_add(a.gate, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (wg != 0) return;
            if (tid == 0) {
                int ok = 0;
                const u64 t0 = wall_clock64();
                do {
                    if (__hip_atomic_load(a.gate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == Wc) {
                        ok = 1;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                } while (wait_time_left(t0, a.spin_limit));
                *ok_flag = ok;
            }
            __syncthreads();
            if (*ok_flag == 0) return;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            // every workgroup has made its last add: counters and gate go back to zero for the launch after this one
            for (u32 c = tid; c < SL_MAX_GROUPS * 4 * (u32)SL_MAX_SUMS; c += BLOCK) st_agent(a.ctr + (size_t)c * SL_CTR_STRIDE, 0);
            if (tid == 0) __hip_atomic_store(a.gate, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            src_each = (u64)Wc * len;
            len = (u32)(src_each >> pend);
            len_log = (u32)__builtin_ctz(len);
            Wc = 1;
            in_big = true;
        }
        trip_seq = a.seq0 + (j - a.j0);
        bool skip1;
        E2 rb_ = gl::e2_zero(), ra_ = gl::e2_zero();
        // A launch made ahead of its first round finds its sources complete (the launch before it on the stream has ended)
        // but not yet its challenges: the entries this thread will fold are asked for before it waits for the mail, so
        // that they cross from device memory during the wait (up to SL_PRE items a thread; more are loaded after the mail).
        U64x2 pre[SL_PRE][4];
        const bool have_pre = k == 0 && !a.first_go && pend >= 1 && (nt << len_log) <= (u32)(SL_PRE * BLOCK);
        if (have_pre) {
            const u64 base = (u64)wg * src_each;
#pragma unroll
            for (int sidx = 0; sidx < SL_PRE; sidx++) {
                const u32 u = tid + (u32)sidx * BLOCK;
                if (u < (nt << len_log)) {
                    const u32 f = u >> len_log, i = u & (len - 1);
                    const u64 *p0 = a.s0[f], *p1 = a.s1[f];
                    const u64 e = base + ((u64)i << pend);
                    pre[sidx][0] = ld2(p0 + e);
                    pre[sidx][2] = p1 ? ld2(p1 + e) : U64x2{0, 0};
                    if (pend == 2) {
                        pre[sidx][1] = ld2(p0 + e + 2);
                        pre[sidx][3] = ld2(p1 + e + 2);
                    }
                }
            }
        }
        if (k == 0 && a.first_go) {
            // a launch made for round 1, when it is that round's turn: nothing is pending, whether t = 1 is evaluated came
            // with the launch, and the trip over the host link that a look into the mailbox costs is saved
            skip1 = a.first_go == 2;
            __syncthreads();
        } else {
            if (wg == 0 && tid == 0) st_sys(a.out_host + SL_WAITING_SLOT, trip_seq);
            if (!wait_first_mail(a.mail, Wc > 1 ? a.relay : nullptr, wg == 0, a.spin_limit, trip_seq, MAIL_SKIP1_LEAVE, box, ok_flag)) return;
            if (wg == 0 && tid == 0) st_sys(a.out_host + SL_HAD_SLOT, trip_seq);
            if (box[MAIL_SKIP1] >= MAIL_SKIP1_LEAVE) return;
            skip1 = box[MAIL_SKIP1] != 0;
            rb_ = gl::e2(box[MAIL_R], box[MAIL_R + 1]);
            ra_ = gl::e2(box[MAIL_RA], box[MAIL_RA + 1]);
        }
        const gl::E2P rb = gl::prep(rb_), ra = gl::prep(ra_);
        // ---- the pending folds ----
        if (have_pre) {
            // (the entries asked for before the wait)
#pragma unroll
            for (int sidx = 0; sidx < SL_PRE; sidx++) {
                const u32 u = tid + (u32)sidx * BLOCK;
                if (u < (nt << len_log)) {
                    const u32 f = u >> len_log, i = u & (len - 1);
                    const U64x2 x0 = pre[sidx][0], x1 = pre[sidx][2];
                    E2 v;
                    if (pend == 1) {
                        v = a.s1[f] ? fold1p(gl::e2(x0.x, x1.x), gl::e2(x0.y, x1.y), rb) : fold1_base(x0.x, x0.y, rb_);
                    } else {
                        const U64x2 y0 = pre[sidx][1], y1 = pre[sidx][3];
                        v = fold1p(fold1p(gl::e2(x0.x, x1.x), gl::e2(x0.y, x1.y), ra), fold1p(gl::e2(y0.x, y1.x), gl::e2(y0.y, y1.y), ra), rb);
                    }
                    tab(true, f, 0)[i] = v.c0;
                    tab(true, f, 1)[i] = v.c1;
                }
            }
        } else if (k == 0 || regroup) {
            // from device memory: entry i of the state is the source's entry i (nothing pending), or is made of its entries
            // 2i, 2i+1 (one fold) or 4i..4i+3 (two)
            const u64 base = (u64)wg * src_each;
            for (u32 u = tid; u < (nt << len_log); u += BLOCK) {
                const u32 f = u >> len_log, i = u & (len - 1);
                const u64 *p0 = regroup ? a.h0[f] : a.s0[f], *p1 = regroup ? a.h1[f] : a.s1[f];
                E2 v;
                if (pend == 0) {
                    v = gl::e2(p0[base + i], p1 ? p1[base + i] : 0);
                } else if (pend == 1) {
                    const U64x2 x0 = ld2(p0 + base + 2 * (u64)i);
                    if (p1) {
                        const U64x2 x1 = ld2(p1 + base + 2 * (u64)i);
                        v = fold1p(gl::e2(x0.x, x1.x), gl::e2(x0.y, x1.y), rb);
                    } else {
                        v = fold1_base(x0.x, x0.y, rb_);
                    }
                } else {
                    const U64x2 x0 = ld2(p0 + base + 4 * (u64)i), y0 = ld2(p0 + base + 4 * (u64)i + 2);
                    const U64x2 x1 = ld2(p1 + base + 4 * (u64)i), y1 = ld2(p1 + base + 4 * (u64)i + 2);
                    v = fold1p(fold1p(gl::e2(x0.x, x1.x), gl::e2(x0.y, x1.y), ra), fold1p(gl::e2(y0.x, y1.x), gl::e2(y0.y, y1.y), ra), rb);
                }
                tab(true, f, 0)[i] = v.c0;
                tab(true, f, 1)[i] = v.c1;
            }
        } else {
            len >>= pend;
            len_log -= pend;
            for (u32 u = tid; u < (nt << len_log); u += BLOCK) {
                const u32 f = u >> len_log, i = u & (len - 1);
                const u64 *c0 = tab(in_big, f, 0), *c1 = tab(in_big, f, 1);
                E2 v;
                if (pend == 1)
                    v = fold1p(gl::e2(c0[2 * i], c1[2 * i]), gl::e2(c0[2 * i + 1], c1[2 * i + 1]), rb);
                else
                    v = fold1p(fold1p(gl::e2(c0[4 * i], c1[4 * i]), gl::e2(c0[4 * i + 1], c1[4 * i + 1]), ra),
                               fold1p(gl::e2(c0[4 * i + 2], c1[4 * i + 2]), gl::e2(c0[4 * i + 3], c1[4 * i + 3]), ra), rb);
                tab(!in_big, f, 0)[i] = v.c0;
                tab(!in_big, f, 1)[i] = v.c1;
            }
            if (EQ)
                for (u32 i = tid; i < (len >> 1); i += BLOCK) {
                    E2 v = weight(in_big, i << pend);
                    for (u32 q = 1; q < (1u << pend); q++) v = gl::add(v, weight(in_big, (i << pend) + q));
                    wts(!in_big, 0)[i] = v.c0;
                    wts(!in_big, 1)[i] = v.c1;
                }
            in_big = !in_big;
        }
        if (EQ && k == 0) {
            // the weights of round j's pairs, from the eq table's level of that round
            const u64 e0 = ((2ull << a.n_vars) - (2ull << (a.n_vars - j))) + (u64)wg * (len >> 1);
            for (u32 i = tid; i < (len >> 1); i += BLOCK) {
                wts(true, 0)[i] = a.eq0[e0 + i];
                wts(true, 1)[i] = a.eq1[e0 + i];
            }
        } else if (EQ && regroup) {
            // ... or from what the workgroups left, added up in runs of 2^pend
            for (u32 i = tid; i < (len >> 1); i += BLOCK) {
                const u64 e = (u64)i << pend;
                E2 v = gl::e2(a.hw0[e], a.hw1[e]);
                for (u32 q = 1; q < (1u << pend); q++) v = gl::add(v, gl::e2(a.hw0[e + q], a.hw1[e + q]));
                wts(true, 0)[i] = v.c0;
                wts(true, 1)[i] = v.c1;
            }
        }
        // this wavefront's counters start the trip at zero
        for (u32 c = lane; c < 4 * (u32)NS; c += WAVE) ctr[wave * 4 * SL_MAX_SUMS + c] = 0;
        __syncthreads();
        const bool big = in_big;
        // adds a lane's canonical sum into the counters of extension sum `idx`
        auto flush = [&](u32 idx, E2 v) {
            u64 *c = ctr + wave * 4 * SL_MAX_SUMS + 4 * idx;
            atomicAdd(reinterpret_cast<unsigned long long *>(c + 0), (unsigned long long)(u32)v.c0);
            atomicAdd(reinterpret_cast<unsigned long long *>(c + 1), (unsigned long long)(v.c0 >> 32));
            atomicAdd(reinterpret_cast<unsigned long long *>(c + 2), (unsigned long long)(u32)v.c1);
            atomicAdd(reinterpret_cast<unsigned long long *>(c + 3), (unsigned long long)(v.c1 >> 32));
        };
        // entry e of table f of the state
        auto ent = [&](u32 f, u32 e) { return gl::e2(tab(big, f, 0)[e], tab(big, f, 1)[e]); };
        // the polynomial summed, from its tables' values: the product of all tables, or sum_k coeff_k prod table (a table's
        // value is asked for by `val(f)`, each time a term names it: the values live in LDS, not in registers a term
        // could not index)
        // `top_only`: only the terms of NF factors (the leading coefficient in the challenge belongs to them alone)
        // `m0`, `step`: the terms m0, m0 + step, ... only (lanes that share a pair split its terms; their sums add up)
        auto poly_of = [&](auto &&val, bool top_only, u32 m0, u32 step) -> E2 {
            if (!TERMS) {
                E2 prod = val(0);
#pragma unroll
                for (u32 f = 1; f < (u32)NF; f++) prod = gl::mulp(prod, gl::prep(val(f)));
                return prod;
            }
            gl::E2Acc G = gl::e2acc_zero();
            for (u32 m = m0; m < a.n_terms; m += step) {
                const SliceTerm &tm = lterms[m];
                if (top_only && tm.n_factors < (u32)NF) continue;
                gl::E2P cp;
                cp.c0 = tm.c0;
                cp.c1 = tm.c1;
                cp.w = tm.w;
                E2 prod = gl::e2_one();
                if (tm.n_factors > 0) {
                    prod = val(tm.slot[0]);
                    for (u32 f = 1; f < tm.n_factors; f++) prod = gl::mulp(prod, gl::prep(val(tm.slot[f])));
                }
                gl::acc_mul(G, prod, cp);
            }
            return gl::acc_reduce(G);
        };
        // lo + t (hi - lo) for the small t of the evaluation points
        auto line_at = [](E2 lo, E2 hi, u32 t) {
            if (t == 0) return lo;
            const E2 d = gl::sub(hi, lo);
            E2 v = hi;
            for (u32 m = 1; m < t; m++) v = gl::add(v, d);
            return v;
        };
        // Late rounds have a pair or two per table and hundreds of lanes: a field multiplication is a chain of a hundred
        // dependent instructions, so the work of a pair is cut into units of one evaluation point (and one term) each
        // and spread over the lanes; every unit's value goes into the point's counters, where the pieces add up.
        // ---- round j: pairs of the state; units taken from the last thread down, those of the quads from the first up ----
        {
            const u32 n_pairs = len >> 1;
            const u32 rt = BLOCK - 1 - tid;
            const u32 m0 = rt % p_split, t = (rt / p_split) % (u32)NP, slot = rt / (p_split * (u32)NP), n_slots = BLOCK / (p_split * (u32)NP);
            E2 acc = gl::e2_zero();
            bool any = false;
            if (slot < n_slots && !(t == 1 && skip1)) {
                for (u32 p = slot; p < n_pairs; p += n_slots) {
                    any = true;
                    const E2 g = poly_of([&](u32 f) { return line_at(ent(f, 2 * p), ent(f, 2 * p + 1), t); }, false, m0, p_split);
                    acc = EQ ? gl::fma(g, gl::prep(weight(big, p)), acc) : gl::add(acc, g);
                }
            }
            if (any) flush(t, acc);
        }
        // ---- round j + 1 as a polynomial in the challenge of round j: quads of the state ----
        if (dbl) {
            const u32 n_quads = len >> 2;
            // a lane keeps one sample at one point (of some of the terms)
            const u32 m0 = tid % q_split, ti = (tid / q_split) % (u32)NPT, smp = (tid / (q_split * (u32)NPT)) % (u32)NSMP;
            const u32 slot = tid / (q_split * (u32)(NPT * NSMP)), n_slots = BLOCK / (q_split * (u32)(NPT * NSMP));
            const u32 t = ti == 0 ? 0 : ti + 1;  // points t = 0, 2, .., NF
            E2 acc = gl::e2_zero();
            bool any = false;
            if (slot < n_slots) {
                for (u32 u = slot; u < n_quads; u += n_slots) {
                    any = true;
                    // a table's pair of round j + 1 with the challenge of round j at this lane's sample: e0 + smp (e1 - e0) and
                    // e2 + smp (e3 - e2); for the leading coefficient the slopes e1 - e0, e3 - e2 in their place
                    auto sampled = [&](u32 f) {
                        const E2 e0 = ent(f, 4 * u), e1 = ent(f, 4 * u + 1), e2_ = ent(f, 4 * u + 2), e3 = ent(f, 4 * u + 3);
                        if (smp == (u32)NF) return line_at(gl::sub(e1, e0), gl::sub(e3, e2_), t);
                        return line_at(line_at(e0, e1, smp), line_at(e2_, e3, smp), t);
                    };
                    const E2 g = poly_of(sampled, smp == (u32)NF, m0, q_split);
                    // (the weight of a quad of round j + 1: those of its two pairs of round j)
                    acc = EQ ? gl::fma(g, gl::prep(gl::add(weight(big, 2 * u), weight(big, 2 * u + 1))), acc) : gl::add(acc, g);
                }
            }
            if (any) flush(NP + smp * NPT + ti, acc);
        }
        __syncthreads();
        // ---- hand the sums over: one counter per lane ----
        if (tid < 4 * (u32)NS && !(skip1 && tid >= 4 && tid < 8)) {
            const u32 c = tid;
            u64 v = 0;
#pragma unroll
            for (int w = 0; w < BLOCK / WAVE; w++) v += ctr[w * 4 * SL_MAX_SUMS + c];
            bool mine = true;
            u32 set = 0;
            if (Wc > 1) {
                // (the workgroups of a set: every 2^groups_log-th one)
                set = wg & ((1u << a.groups_log) - 1);
                const u64 before = __hip_atomic_fetch_add(a.ctr + (size_t)(set * (u32)SL_GROUP_WORDS + c) * SL_CTR_STRIDE, v + SL_CTR_ONE, __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT);
                mine = ((((before >> 56) + 1) & (u64)((Wc >> a.groups_log) - 1)) == 0);
                v = (before + v) & SL_CTR_MASK;
            }
            if (mine) st_sys(a.out_host + set * (u32)SL_GROUP_WORDS + c, v | (sl_tag(trip_seq) << 56));
        }
        pend = dbl ? 2 : 1;
        j += pend;
        __syncthreads();
    }
    // ---- what is left of the tables ----
    const bool big = in_big;
    if (!a.finish) {
        // to device memory, for the launch queued behind this one (which starts with this launch's pending folds)
        for (u32 i = tid; i < len; i += BLOCK) {
            for (u32 f = 0; f < nt; f++) {
                a.h0[f][(u64)wg * len + i] = tab(big, f, 0)[i];
                a.h1[f][(u64)wg * len + i] = tab(big, f, 1)[i];
            }
        }
        if (Wc > 1) {
            // Several workgroups to the end, nobody took over inside the launch: the first one waits at the gate until every
            // workgroup has made its last add, and leaves counters and gate at zero for the launch after this one.  (Clearing
            // them from the host, with a fill queued behind the launch, is a second launch and one more thing on the stream
            // between this launch and the one that goes on from its tables.)
            __syncthreads();
            if (tid == 0) __hip_atomic_fetch_add(a.gate, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (wg != 0) return;
            if (tid == 0) {
                int ok = 0;
                const u64 t0 = wall_clock64();
                do {
                    if (__hip_atomic_load(a.gate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == Wc) {
                        ok = 1;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                } while (wait_time_left(t0, a.spin_limit));
                *ok_flag = ok;
            }
            __syncthreads();
            if (*ok_flag == 0) return;  // (a workgroup gave up on the way: the host clears everything behind a failed session)
            for (u32 c = tid; c < SL_MAX_GROUPS * 4 * (u32)SL_MAX_SUMS; c += BLOCK) st_agent(a.ctr + (size_t)c * SL_CTR_STRIDE, 0);
            if (tid == 0) __hip_atomic_store(a.gate, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else if (wave == 0) {
        // to the host: entry e of table f at words 2 (f len + e), + 1 (len is a power of two)
        const u32 n_words = nt * len * 2;
        u64 x = 0;
        for (u32 w = lane; w < n_words; w += WAVE) {
            const u32 f = w >> (len_log + 1), e = (w >> 1) & (len - 1);
            const u64 word = tab(big, f, w & 1)[e];
            x ^= sl_fin_mix(word, w);
            st_sys(a.fin_out + w, word);
        }
#pragma unroll
        for (int off = WAVE / 2; off >= 1; off >>= 1) x ^= __shfl_xor(x, off, WAVE);
        if (lane == 0) {
            st_sys(a.fin_out + SL_FIN_CHK_SLOT, x ^ trip_seq);
            st_sys(a.fin_out + SL_FIN_SEQ_SLOT, trip_seq);
        }
    }
}

// ---------------------------------------------------------------------------
// fused kernel for sums of several product terms over shared tables
//
// A group is up to POLY_MAXT tables and the terms made of them.  Per pair a
// thread loads every table of the group once (folding it with the previous
// challenge on the way, and writing the folded pair when this group owns the
// table), keeps value and slope of every table in LDS (the terms pick their
// factors by index, which registers cannot do), and evaluates
//     G(t) = sum_terms coeff * prod_factors table(t)
// at t = 0..NF with the coefficients applied here, so one set of running sums
// serves all terms.  An eq factor common to all terms is taken out in closed
// form exactly as in prod_kernel (G is then the polynomial without it), and
// t = 1 is skipped when the claim is known.  Output is that of prod_kernel:
// per-workgroup sums of G(t) (times R), gathered by the last workgroup and handed to the host.
// Groups are grid rows; their partials are simply added.
// ---------------------------------------------------------------------------
constexpr int POLY_MAXT = 7;
constexpr int POLY_LDS_TERMS = 48;  // terms of a group kept in LDS; further ones are read from device memory
constexpr int POLY_RES_ROUNDS = 9;  // rounds one resident launch can run: from 256 pairs down to one
constexpr u32 POLY_PAIR = 0, POLY_PAIR_FOLD = 1, POLY_BCAST = 2;

struct PolyTab {
    const u64 *s0;
    const u64 *s1;  // nullptr: base-field source
    u64 *d0;        // POLY_PAIR_FOLD: where the folded table goes; nullptr: another group writes it
    u64 *d1;
    u32 mode;
    u32 shift;      // POLY_BCAST: entry index = pair index >> shift
};

struct PolyGroup {
    PolyTab tab[POLY_MAXT];
    u32 n_tabs;
    u32 term_begin, term_end;
    u32 op_begin, op_end;  // the same terms as a nested (Horner) program, poly_kernel only; empty: evaluate term by term
    u32 pad;
};

struct PolyTerm {
    u64 c0, c1, w;  // coefficient, prepared (w = 7 c1)
    u32 n_factors;
    uint8_t slot[DPS_MAX_FACTORS];  // table slots within the group
    u32 pad;
};
// The terms of a group in nested form: factoring the most frequent table out of the terms that contain it, again
// and again, turns sum_k c_k prod table into a tree whose every edge is one product,
//     G = c + sum_children table_child * G_child.
// The tree is walked depth first with one running value per depth:
//     ENTER d, c      acc[d] = c                          (a node with children; c = coefficient of the term ending here, or 0)
//     LEAF  d, s, c   acc[d] += table_s * c               (a child without children)
//     LEAVE d, s      acc[d - 1] += table_s * acc[d]      (back to the parent)
// and G = acc[0].  One product per edge instead of one per factor and coefficient of every term.
constexpr u32 POLY_OP_ENTER = 0, POLY_OP_LEAF = 1, POLY_OP_LEAVE = 2;
struct PolyOp {
    u64 c0, c1, w;  // coefficient, prepared (ENTER, LEAF)
    u32 code;       // kind | depth << 2 | slot << 8
    u32 pad;
};
constexpr int POLY_LDS_OPS = POLY_LDS_TERMS * 40 / 32;  // a program shares the terms' place in LDS and in the kernel arguments
static_assert(sizeof(PolyTerm) == 40 && sizeof(PolyOp) == 32, "terms and operations share storage");
static_assert(HOST_FINALS_SLOT + 4 * POLY_MAXT <= HOST_PAIRS_SEQ_SLOT && 4 * POLY_MAXT <= 6 * MAX_PTS, "last pairs of a group fit its result area");
static_assert(sizeof(PolyTerm) % 8 == 0 && sizeof(PolyGroup) % 8 == 0, "descriptors are copied as 64-bit words");

struct PolyArgs {
    const PolyGroup *groups;  // one per grid row, this round's; nullptr: the single group is in g0
    const PolyTerm *terms;    // nullptr: the terms are in t0
    const PolyOp *ops;        // poly_kernel, groups with a program: nullptr = the program is in t0 (instead of the terms)
    PolyGroup g0;
    union {
        PolyTerm t0[POLY_LDS_TERMS];
        PolyOp o0[POLY_LDS_OPS];
    };
    const u64 *q0;  // eq suffix table of this round (common eq factor only)
    const u64 *q1;
    u64 n_pairs;
    u64 r0, r1;
    // Resident rounds (poly_split_kernel, single-workgroup launches only): after round j the workgroup stays, waits
    // for the next challenge in the host's mailbox as tail_kernel does, and runs the following rounds up to
    // last_round on the tables it folded itself.  `groups` then holds one descriptor per round, starting with
    // this launch's.
    u32 j;           // this launch's round (1-based)
    u32 last_round;  // 0: exit after round j
    u32 n_vars;
    u32 spin_limit;
    const u64 *eq0;  // eq storage, level 0 at entry 0 (common eq factor only)
    const u64 *eq1;
    const u64 *mail;
    u64 seq;         // sequence number of round j; round j + k waits for mail seq + k
    u32 split_log;   // 2^split_log lanes share a pair in round j
    u32 split_cap;   // resident rounds: the share doubles as the pairs halve, up to 2^split_cap lanes
    u32 lds_state;   // resident rounds: the folded tables stay in LDS (state_off words into the dynamic LDS)
    u32 state_off;
    u32 finish;      // resident rounds: with the last round, also publish value and slope of every table's last pair
    u32 group_stride;  // resident rounds: descriptors of consecutive rounds of one group lie this many apart
    u32 wait_first;  // launched ahead of its round: the challenge of round j also arrives by mail (seq)
    u32 pad;
    u64 *relay;      // ... through these words of device memory for all workgroups but the first (see wait_first_mail); or nullptr
    // Several groups resident side by side (one workgroup each, gridDim.y of them): a workgroup cannot finish the
    // message, which is the sum over the groups, so each publishes its own sums q(t) (and later its tables' final
    // evaluations) to its 64-word slot raw_out + 64 * blockIdx.y, laid out like the main result area, and the host adds.
    u64 *raw_out;    // nullptr: a single workgroup, which publishes to the main result area
    // poly_kernel, rounds of at least 2^EQ_LO_BITS pairs whose grid stride is a multiple of that: the weights of the common eq
    // factor are not streamed (q0, q1) but taken as in the FACT variants of prod_kernel, R(i) = hi[i >> EQ_LO_BITS] * lo[i & mask]
    // -- hi per workgroup and step (scalar loads) on the running sums, lo once per thread at the end.  nullptr: streamed.
    const u64 *lq0, *lq1, *hq0, *hq1;
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <typename F, int... I>
__device__ __forceinline__ void static_for_each(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    static_for_each(f, std::make_integer_sequence<int, N>{});
}

// A node of the nested program at depth D: starts from its constant, adds table * c for every LEAF, table * (child's
// value) for every child (ENTER D + 1 ... LEAVE D + 1, walked by the next depth's function), and ends at the LEAVE of its
// own depth, which it leaves for its parent to read the table from (or at the end of the program: the root).
// `op(o)`: operation o; `table(slot)`: the slot's table at the evaluation point in hand.
template <int D, int MAXD, typename OpAt, typename TableAt>
__device__ __forceinline__ E2 poly_walk(u32 &pc, u32 n_ops, E2 acc, OpAt &&op, TableAt &&table)
{
    while (pc < n_ops) {
        const PolyOp &o = op(pc);
        const u32 code = __builtin_amdgcn_readfirstlane(o.code);
        const u32 kind = code & 3, sl = code >> 8;
        if (kind == POLY_OP_LEAF) {
            gl::E2P cp;
            cp.c0 = o.c0;
            cp.c1 = o.c1;
            cp.w = o.w;
            acc = gl::fma(table(sl), cp, acc);
            pc++;
        } else if (kind == POLY_OP_ENTER) {
            pc++;
            if constexpr (D < MAXD) {
                const E2 child = poly_walk<D + 1, MAXD>(pc, n_ops, gl::e2(o.c0, o.c1), op, table);
                // (the child stopped at its LEAVE, which names the table on the edge to it)
                const u32 edge = __builtin_amdgcn_readfirstlane(op(pc).code) >> 8;
                acc = gl::fma(child, gl::prep(table(edge)), acc);
                pc++;
            }
        } else {
            break;
        }
    }
    return acc;
}

template <int NF, bool EQ, bool SKIP1>
__global__ void __launch_bounds__(BLOCK) poly_kernel(PolyArgs a, u64 *__restrict__ partial, FastFin ff)
{
    constexpr int NP = NF + 1;
    extern __shared__ u64 dyn[];  // [n_tabs][4][BLOCK]: value c0, c1, slope c0, c1
    __shared__ u32 lds[(BLOCK / WAVE) * 6 * NP];
    __shared__ int last_flag;
    // The group's descriptors come from device memory; read from there inside the loops every use would be
    // a dependent load of its own (the small rounds are nothing but such latencies), so they are staged in LDS once.
    __shared__ PolyGroup g;
    __shared__ PolyTerm lterms[POLY_LDS_TERMS];
    const u32 tid = threadIdx.x;
    auto cur0 = [&](u32 k) -> u64 & { return dyn[(k * 4 + 0) * BLOCK + tid]; };
    auto cur1 = [&](u32 k) -> u64 & { return dyn[(k * 4 + 1) * BLOCK + tid]; };
    auto dl0 = [&](u32 k) -> u64 & { return dyn[(k * 4 + 2) * BLOCK + tid]; };
    auto dl1 = [&](u32 k) -> u64 & { return dyn[(k * 4 + 3) * BLOCK + tid]; };
    const u64 n_pairs = a.n_pairs;
    E2 r = gl::e2(a.r0, a.r1);
    const u64 *q0 = a.q0, *q1 = a.q1;
    const bool fact = EQ && a.lq0 != nullptr;
    {
        const bool inl = a.groups == nullptr;  // a single group handed over in the kernel arguments
        const u64 *src = inl ? reinterpret_cast<const u64 *>(&a.g0) : reinterpret_cast<const u64 *>(a.groups + blockIdx.y);
        u64 *dst = reinterpret_cast<u64 *>(&g);
        for (u32 w = tid; w < sizeof(PolyGroup) / 8; w += BLOCK) dst[w] = src[w];
        __syncthreads();
        const u32 nt = g.term_end - g.term_begin;
        const u32 staged = nt < (u32)POLY_LDS_TERMS ? nt : (u32)POLY_LDS_TERMS;
        const u64 *ts = inl ? reinterpret_cast<const u64 *>(a.t0) : reinterpret_cast<const u64 *>(a.terms + g.term_begin);
        u64 *td = reinterpret_cast<u64 *>(lterms);
        const u32 no = g.op_end - g.op_begin;  // at most POLY_LDS_OPS
        if (no) {
            // a program in the kernel arguments is read from there
            if (!inl) {
                const u64 *os = reinterpret_cast<const u64 *>(a.ops + g.op_begin);
                for (u32 w = tid; w < no * (sizeof(PolyOp) / 8); w += BLOCK) td[w] = os[w];
            }
        } else {
            for (u32 w = tid; w < staged * (sizeof(PolyTerm) / 8); w += BLOCK) td[w] = ts[w];
        }
        __syncthreads();
    }
    const u32 n_tabs = g.n_tabs;
    const u32 n_terms = g.term_end - g.term_begin;
    const u32 n_ops = g.op_end - g.op_begin;
    const PolyOp *lops = reinterpret_cast<const PolyOp *>(lterms);
    if (a.wait_first) {
        // launched while the previous round was still running: the challenge comes by mail
        __shared__ u64 box[MAIL_WORDS];
        __shared__ int ok_flag;
        if (!wait_first_mail(a.mail, a.relay, blockIdx.x == 0 && blockIdx.y == 0, a.spin_limit, ff.seq, SKIP1 ? 0 : 1, box, &ok_flag)) return;
        // the other way of getting p(1) is not compiled into this variant: the host ends the launch instead
        if ((box[MAIL_SKIP1] != 0) != SKIP1) return;
        r = gl::e2(uniform64(box[MAIL_R]), uniform64(box[MAIL_R + 1]));
    }
    const gl::E2P rp = gl::prep(r);

    // Few live registers matter more here than loads in flight: the loop is arithmetic, and it is the number of
    // wavefronts per SIMD that hides the latency of its dependent integer chains.  Tables are taken one at a time.
    E2 lz[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) lz[t] = gl::e2_zero();
    const bool inl = a.groups == nullptr;

    for (u64 i = (u64)blockIdx.x * BLOCK + tid; i < n_pairs; i += (u64)gridDim.x * BLOCK) {
        auto take = [&](const PolyTab &tb, u32 k) {
            E2 lo, hi;
            if (tb.mode == POLY_PAIR_FOLD) {
                const U64x2 x0 = ld2(tb.s0 + 4 * i), y0 = ld2(tb.s0 + 4 * i + 2);
                if (tb.s1) {
                    const U64x2 x1 = ld2(tb.s1 + 4 * i), y1 = ld2(tb.s1 + 4 * i + 2);
                    lo = fold1p(gl::e2(x0.x, x1.x), gl::e2(x0.y, x1.y), rp);
                    hi = fold1p(gl::e2(y0.x, y1.x), gl::e2(y0.y, y1.y), rp);
                } else {
                    lo = fold1_base(x0.x, x0.y, r);
                    hi = fold1_base(y0.x, y0.y, r);
                }
                if (tb.d0) {
                    st2_stream(tb.d0 + 2 * i, lo.c0, hi.c0);
                    st2_stream(tb.d1 + 2 * i, lo.c1, hi.c1);
                }
            } else if (tb.mode == POLY_PAIR) {
                const U64x2 x0 = ld2(tb.s0 + 2 * i);
                U64x2 x1 = U64x2{0, 0};
                if (tb.s1) x1 = ld2(tb.s1 + 2 * i);
                lo = gl::e2(x0.x, x1.x);
                hi = gl::e2(x0.y, x1.y);
            } else {
                const u64 e = i >> tb.shift;
                lo = hi = gl::e2(tb.s0[e], tb.s1 ? tb.s1[e] : 0);
            }
            const E2 d = gl::sub(hi, lo);
            cur0(k) = lo.c0;
            cur1(k) = lo.c1;
            dl0(k) = d.c0;
            dl1(k) = d.c1;
        };
        // descriptors in the kernel arguments arrive in scalar registers
        if (inl)
            for (u32 k = 0; k < n_tabs; k++) take(a.g0.tab[k], k);
        else
            for (u32 k = 0; k < n_tabs; k++) take(g.tab[k], k);
        gl::E2P restp = gl::prep(gl::e2_one());
        if (EQ) {
            if (fact) {
                // (the same entry for the whole workgroup: its pairs lie within one run of 2^EQ_LO_BITS)
                const u32 hi = __builtin_amdgcn_readfirstlane((u32)(i >> EQ_LO_BITS));
                restp = gl::prep(gl::e2(a.hq0[hi], a.hq1[hi]));
            } else {
                restp = gl::prep(gl::e2(q0[i], q1[i]));
            }
        }
        // (one copy of the body per evaluation point, t a compile-time constant in each)
        static_for<NP>([&](auto point) {
            constexpr int t = decltype(point)::value;
            if (!(t == 1 && SKIP1)) {
                E2 gsum;
                if (n_ops) {
                    // the nested program: every index below is a compile-time constant inside its case.  Read from
                    // the kernel arguments an operation arrives in scalar registers and its branches are uniform.
                    // The nested program, walked with one function per depth (poly_walk): a node's running value is a
                    // local of its depth's function, so no value is ever picked by a run-time index -- as an array
                    // indexed by the operation's depth the values lived in scratch memory (a store per depth and two
                    // dependent loads per operation, and a fifth of a gigabyte of write-backs per round), and picked
                    // by select chains they cost forty more registers.  The operations are the same for the whole
                    // wavefront: read from the kernel arguments they arrive in scalar registers, the branches are uniform.
                    auto table = [&](u32 sl) { return gl::e2(cur0(sl), cur1(sl)); };
                    u32 pc = 1;  // (operation 0 enters the root with its constant)
                    if (inl)
                        gsum = poly_walk<0, NF - 1>(pc, n_ops, gl::e2(a.o0[0].c0, a.o0[0].c1), [&](u32 o) -> const PolyOp & { return a.o0[o]; }, table);
                    else
                        gsum = poly_walk<0, NF - 1>(pc, n_ops, gl::e2(lops[0].c0, lops[0].c1), [&](u32 o) -> const PolyOp & { return lops[o]; }, table);
                } else {
                    gl::E2Acc G = gl::e2acc_zero();
                    for (u32 j = 0; j < n_terms; j++) {
                        const PolyTerm &tm = j < (u32)POLY_LDS_TERMS ? lterms[j] : a.terms[g.term_begin + j];
                        E2 prod = gl::e2_one();
                        if (tm.n_factors > 0) {
                            const u32 s0 = tm.slot[0];
                            prod = gl::e2(cur0(s0), cur1(s0));
                            for (u32 f = 1; f < tm.n_factors; f++) {
                                const u32 sl = tm.slot[f];
                                prod = gl::mulp(prod, gl::prep(gl::e2(cur0(sl), cur1(sl))));
                            }
                        }
                        gl::E2P cp;
                        cp.c0 = tm.c0;
                        cp.c1 = tm.c1;
                        cp.w = tm.w;
                        gl::acc_mul(G, prod, cp);
                    }
                    gsum = gl::acc_reduce(G);
                }
                lz[t] = EQ ? gl::fma(gsum, restp, lz[t]) : gl::add(lz[t], gsum);
            }
            if (t + 1 < NP) {
                // on to t + 1 (the slope is added even when t = 1 is skipped: t = 2 needs it twice)
                for (u32 k = 0; k < n_tabs; k++) {
                    cur0(k) = gl::add(cur0(k), dl0(k));
                    cur1(k) = gl::add(cur1(k), dl1(k));
                }
            }
        });
    }
    E2 acc[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) acc[t] = lz[t];
    if (EQ && fact) {
        // the low part of the weights: the same for all of a thread's pairs (the grid's stride is a multiple of 2^EQ_LO_BITS)
        const u32 lo = (blockIdx.x * BLOCK + tid) & ((1u << EQ_LO_BITS) - 1);
        const gl::E2P lp = gl::prep(gl::e2(a.lq0[lo], a.lq1[lo]));
#pragma unroll
        for (int t = 0; t < NP; t++) acc[t] = gl::mulp(acc[t], lp);
    }
    block_reduce<NP>(acc, lds);
    if (gridDim.x * gridDim.y == 1) {
        publish_sums<NP>(ff.out_host, ff.seq, ff.counter, acc);
        return;
    }
    if (ff.slots) {
        publish_sums<NP>(ff.slots + 64 * ((u64)blockIdx.y * gridDim.x + blockIdx.x), ff.seq, nullptr, acc);
        return;
    }
    if (tid == 0) {
        u64 *o = partial + ((u64)blockIdx.y * gridDim.x + blockIdx.x);
        const u64 total = (u64)gridDim.x * gridDim.y;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            st_agent(o + (2 * t) * total, acc[t].c0);
            st_agent(o + (2 * t + 1) * total, acc[t].c1);
        }
    }
    if (take_ticket(ff.counter, gridDim.x * gridDim.y, &last_flag)) {
        E2 q[NP];
        gather_partials<NP>(ff, lds, q);
        publish_sums<NP>(ff.out_host, ff.seq, ff.counter, q);
    }
}

// The same sum for rounds of few pairs, where a launch is one serial chain per thread: the work of a pair is
// spread over 2^split_log adjacent lanes.  First the pair's tables are divided among the lanes (each loads,
// folds and stores its tables and leaves value and slope in LDS), then the (point, term) products are: lane l
// takes every item q = point_position * n_terms + term with q = l mod 2^split_log, reading a factor at point t
// as value + t * slope.  Sums are exact in the field, so the message is the one poly_kernel computes.
// A single-workgroup launch stays resident as described at PolyArgs; with lds_state the tables it folds stay
// in LDS from one round to the next (they still go to device memory, where the final evaluations are read).
template <int NF, bool EQ, bool SKIP1>
__global__ void __launch_bounds__(BLOCK) poly_split_kernel(PolyArgs a, u64 *__restrict__ partial, FastFin ff)
{
    constexpr int NP = NF + 1;
    extern __shared__ u64 dyn[];  // [n_tabs][4][BLOCK] value c0, c1, slope c0, c1 per pair; at state_off the folded tables
    __shared__ u32 lds[(BLOCK / WAVE) * 6 * NP];
    __shared__ u64 res[6 * MAX_PTS];
    __shared__ int last_flag;
    __shared__ PolyGroup gall[POLY_RES_ROUNDS];  // the descriptors of every round this launch runs
    __shared__ PolyTerm lterms[POLY_LDS_TERMS];
    __shared__ u64 box[MAIL_WORDS];
    __shared__ int ok_flag;
    const u32 tid = threadIdx.x;
    u32 j = a.j;
    u64 n_pairs = a.n_pairs;
    E2 r = gl::e2(a.r0, a.r1);
    const u64 *q0 = a.q0, *q1 = a.q1;
    u64 cf_seq = ff.seq;  // sequence number of the round being worked on
    u32 sl = a.split_log;
    u32 in_lds = 0;  // tables (bit per slot) whose current contents this workgroup holds in LDS
    // resident rounds with lds_state: the folded tables, alternating between a buffer of 2 * BLOCK entries per limb
    // array and one of BLOCK entries (every round halves them)
    u64 *const state_a = dyn + a.state_off;
    u64 *const state_b = state_a + (size_t)POLY_MAXT * 2 * 2 * BLOCK;
    bool dst_is_a = true;
    {
        // Descriptors and terms are staged in LDS once: read where they lie (kernel arguments, device memory, or for a
        // resident launch pinned host memory) every use would be a dependent load of its own.  A resident launch has
        // a single group, whose descriptors for rounds j, j + 1, ... follow each other.
        const u32 n_rounds = a.last_round ? a.last_round - a.j + 1 : 1;
        constexpr u32 GW = sizeof(PolyGroup) / 8;
        const u64 *src = a.groups ? reinterpret_cast<const u64 *>(a.groups + blockIdx.y) : reinterpret_cast<const u64 *>(&a.g0);
        u64 *dst = reinterpret_cast<u64 *>(gall);
        for (u32 w = tid; w < n_rounds * GW; w += BLOCK) {
            const u32 rr = w / GW;
            dst[w] = src[(size_t)rr * a.group_stride * GW + (w - rr * GW)];
        }
        __syncthreads();
        const u32 nt = gall[0].term_end - gall[0].term_begin;
        const u32 staged = nt < (u32)POLY_LDS_TERMS ? nt : (u32)POLY_LDS_TERMS;
        const u64 *ts = a.terms ? reinterpret_cast<const u64 *>(a.terms + gall[0].term_begin) : reinterpret_cast<const u64 *>(a.t0);
        u64 *td = reinterpret_cast<u64 *>(lterms);
        for (u32 w = tid; w < staged * (sizeof(PolyTerm) / 8); w += BLOCK) td[w] = ts[w];
        __syncthreads();
    }
    // the challenge of a round, from the mail the host posted for it
    auto take_mail = [&](u64 seq, bool first) -> bool {
        // (only the first mail of a launch made ahead can concern several workgroups)
        const bool ok = first ? wait_first_mail(a.mail, a.relay, blockIdx.x == 0 && blockIdx.y == 0, a.spin_limit, seq, SKIP1 ? 0 : 1, box, &ok_flag)
                              : tail_wait_mail(a.mail, a.spin_limit, seq, box, &ok_flag);
        if (!ok) return false;
        // a run-time switch to evaluating t = 1 (or not) is not compiled in: the host ends the launch instead
        if ((box[MAIL_SKIP1] != 0) != SKIP1) return false;
        r = gl::e2(box[MAIL_R], box[MAIL_R + 1]);
        cf_seq = seq;
        return true;
    };
    // The eq weight of a thread's first pair of a round does not depend on the challenge: before a wait for mail it is
    // requested for the round to come, so that it is there when the mail is (rest_ahead_i: the pair it belongs to).
    E2 rest_ahead = gl::e2_one();
    u64 rest_ahead_i = ~(u64)0;
    auto request_rest = [&](const u64 *e0, const u64 *e1, u64 pairs, u32 split) {
        rest_ahead_i = ~(u64)0;
        const u64 pi = (u64)blockIdx.x * (BLOCK >> split) + (tid >> split);
        if (EQ && pi < pairs) {
            rest_ahead = gl::e2(e0[pi], e1[pi]);
            rest_ahead_i = pi;
        }
    };
    // launched while the previous round was still running: everything that depends on its challenge comes by mail
    // Likewise the entries of the first table this lane takes in its first step of a launch made ahead (a table that is
    // folded on the way in, read from device memory): four 16-byte loads that are then not waited for after the mail.
    U64x2 tab_ahead[4];
    u64 tab_ahead_i = ~(u64)0;
    if (a.wait_first) {
        request_rest(q0, q1, n_pairs, sl);
        const u32 sub0 = tid & ((1u << sl) - 1);
        const u64 pi = (u64)blockIdx.x * (BLOCK >> sl) + (tid >> sl);
        if (pi < n_pairs && sub0 < gall[0].n_tabs && gall[0].tab[sub0].mode == POLY_PAIR_FOLD) {
            const PolyTab &tb = gall[0].tab[sub0];
            tab_ahead[0] = ld2(tb.s0 + 4 * pi);
            tab_ahead[1] = ld2(tb.s0 + 4 * pi + 2);
            if (tb.s1) {
                tab_ahead[2] = ld2(tb.s1 + 4 * pi);
                tab_ahead[3] = ld2(tb.s1 + 4 * pi + 2);
            } else {
                tab_ahead[2] = tab_ahead[3] = U64x2{0, 0};
            }
            tab_ahead_i = pi;
        }
        if (!take_mail(a.seq, true)) return;
    }
  for (;;) {
    const PolyGroup &g = gall[j - a.j];
    const u32 n_tabs = g.n_tabs;
    const u32 n_terms = g.term_end - g.term_begin;
    const gl::E2P rp = gl::prep(r);
    const u32 S = 1u << sl, sub = tid & (S - 1), pib = tid >> sl, ppb = BLOCK >> sl;
    auto val = [&](u32 k, u32 c) -> u64 & { return dyn[(k * 4 + c) * BLOCK + pib]; };
    u64 *const state_dst = dst_is_a ? state_a : state_b;
    const u64 *const state_src = dst_is_a ? state_b : state_a;
    const u32 state_dst_len = dst_is_a ? 2 * BLOCK : BLOCK, state_src_len = dst_is_a ? BLOCK : 2 * BLOCK;
    // tables this round folds: with lds_state every one of them is kept in LDS, also a table another group owns
    // (only the owner writes it to device memory), so that resident groups never read each other's stores
    u32 wrote = 0;
    for (u32 k = 0; k < n_tabs; k++)
        if (g.tab[k].mode == POLY_PAIR_FOLD) wrote |= 1u << k;

    gl::E2Acc lz[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) lz[t] = gl::e2acc_zero();

    // the bounds are the same for every thread of the workgroup: the barriers inside are reached by all
    for (u64 base = (u64)blockIdx.x * ppb; base < n_pairs; base += (u64)gridDim.x * ppb) {
        const u64 i = base + pib;
        const bool active = i < n_pairs;
        // tables sub, sub + S, ... of the pair, one at a time (few live registers).  In resident rounds a folded table
        // is read from one LDS buffer and written to the other, so no lane overwrites what another still has to read.
        if (active) {
            for (u32 k = sub; k < n_tabs; k += S) {
                const PolyTab &tb = g.tab[k];
                E2 lo, hi;
                if (tb.mode == POLY_PAIR_FOLD) {
                    E2 x0, x1, y0, y1;
                    bool ext = true;
                    if ((in_lds >> k) & 1) {
                        const u64 *c0 = state_src + (size_t)(k * 2 + 0) * state_src_len, *c1 = state_src + (size_t)(k * 2 + 1) * state_src_len;
                        x0 = gl::e2(c0[4 * i], c1[4 * i]);
                        x1 = gl::e2(c0[4 * i + 1], c1[4 * i + 1]);
                        y0 = gl::e2(c0[4 * i + 2], c1[4 * i + 2]);
                        y1 = gl::e2(c0[4 * i + 3], c1[4 * i + 3]);
                    } else {
                        // (requested before the mail came: the first table of the first step of a launch made ahead)
                        const bool had = j == a.j && k == sub && i == tab_ahead_i;
                        const U64x2 p0 = had ? tab_ahead[0] : ld2(tb.s0 + 4 * i), q0v = had ? tab_ahead[1] : ld2(tb.s0 + 4 * i + 2);
                        U64x2 p1 = U64x2{0, 0}, q1v = U64x2{0, 0};
                        ext = tb.s1 != nullptr;
                        if (ext) {
                            p1 = had ? tab_ahead[2] : ld2(tb.s1 + 4 * i);
                            q1v = had ? tab_ahead[3] : ld2(tb.s1 + 4 * i + 2);
                        }
                        x0 = gl::e2(p0.x, p1.x);
                        x1 = gl::e2(p0.y, p1.y);
                        y0 = gl::e2(q0v.x, q1v.x);
                        y1 = gl::e2(q0v.y, q1v.y);
                    }
                    if (ext) {
                        lo = fold1p(x0, x1, rp);
                        hi = fold1p(y0, y1, rp);
                    } else {
                        lo = fold1_base(x0.c0, x1.c0, r);
                        hi = fold1_base(y0.c0, y1.c0, r);
                    }
                    if (tb.d0) {
                        st2_stream(tb.d0 + 2 * i, lo.c0, hi.c0);
                        st2_stream(tb.d1 + 2 * i, lo.c1, hi.c1);
                    }
                    if (a.lds_state) {
                        u64 *c0 = state_dst + (size_t)(k * 2 + 0) * state_dst_len, *c1 = state_dst + (size_t)(k * 2 + 1) * state_dst_len;
                        c0[2 * i] = lo.c0;
                        c0[2 * i + 1] = hi.c0;
                        c1[2 * i] = lo.c1;
                        c1[2 * i + 1] = hi.c1;
                    }
                } else if (tb.mode == POLY_PAIR) {
                    const U64x2 p0 = ld2(tb.s0 + 2 * i);
                    U64x2 p1 = U64x2{0, 0};
                    if (tb.s1) p1 = ld2(tb.s1 + 2 * i);
                    lo = gl::e2(p0.x, p1.x);
                    hi = gl::e2(p0.y, p1.y);
                } else {
                    const u64 e = i >> tb.shift;
                    lo = hi = gl::e2(tb.s0[e], tb.s1 ? tb.s1[e] : 0);
                }
                const E2 d = gl::sub(hi, lo);
                val(k, 0) = lo.c0;
                val(k, 1) = lo.c1;
                val(k, 2) = d.c0;
                val(k, 3) = d.c1;
            }
        }
        __syncthreads();
        if (active) {
            gl::E2P restp = gl::prep(gl::e2_one());
            if (EQ) restp = gl::prep(i == rest_ahead_i ? rest_ahead : gl::e2(q0[i], q1[i]));
            // items q = position of the point * n_terms + term; this lane's are sub, sub + S, ...  The point is a
            // run-time value, so the lanes of a wavefront run the same instructions whatever item each one holds.
            constexpr u32 NPE = SKIP1 ? NP - 1 : NP;
            u32 tpos = 0, jj = sub;
            while (jj >= n_terms && tpos < NPE) {
                jj -= n_terms;
                tpos++;
            }
            while (tpos < NPE) {
                const u32 t = (SKIP1 && tpos >= 1) ? tpos + 1 : tpos;
                auto at = [&](u32 k) {
                    const E2 d = gl::mul_base(gl::e2(val(k, 2), val(k, 3)), (u64)t);
                    return gl::add(gl::e2(val(k, 0), val(k, 1)), d);
                };
                const PolyTerm &tm = jj < (u32)POLY_LDS_TERMS ? lterms[jj] : a.terms[g.term_begin + jj];
                gl::E2P cp;
                cp.c0 = tm.c0;
                cp.c1 = tm.c1;
                cp.w = tm.w;
                E2 w = gl::e2(tm.c0, tm.c1);
                if (tm.n_factors > 0) {
                    E2 prod = at(tm.slot[0]);
                    for (u32 f = 1; f < tm.n_factors; f++) prod = gl::mulp(prod, gl::prep(at(tm.slot[f])));
                    w = gl::mulp(prod, cp);
                }
                if (EQ) w = gl::mulp(w, restp);
#pragma unroll
                for (int tt = 0; tt < NP; tt++)
                    if ((u32)tt == t) gl::acc_e2(lz[tt], w);
                jj += S;
                while (jj >= n_terms && tpos < NPE) {
                    jj -= n_terms;
                    tpos++;
                }
            }
        }
        // value and slope are overwritten by the next step
        __syncthreads();
    }
    E2 acc[NP];
#pragma unroll
    for (int t = 0; t < NP; t++) acc[t] = gl::acc_reduce(lz[t]);
    block_reduce<NP>(acc, lds);
    const bool raw = a.raw_out != nullptr;  // then gridDim.x == 1
    if (gridDim.x * gridDim.y == 1 || raw) {
        u64 *const my_out = raw ? a.raw_out + 64 * blockIdx.y : ff.out_host;
        publish_sums<NP>(my_out, cf_seq, raw ? nullptr : ff.counter, acc);
        if (a.last_round == 0) return;
        if (j >= a.last_round) {
            if (!a.finish) return;
            // with the last round: value and slope of every table's remaining pair (still in LDS, pair 0), in slot order;
            // the host folds them with the last challenge
            if (tid < n_tabs) {
#pragma unroll
                for (int k = 0; k < 4; k++) res[4 * tid + k] = dyn[(tid * 4 + k) * BLOCK];
            }
            __syncthreads();
            if (tid == 0) publish_words(my_out, HOST_FINALS_SLOT, res, 4 * n_tabs, cf_seq, HOST_PAIRS_SEQ_SLOT, HOST_PAIRS_CHK_SLOT);
            return;
        }
        // stay for the next round: its challenge arrives by mail
        j++;
        n_pairs >>= 1;
        if (sl < a.split_cap && (n_pairs << (sl + 1)) <= (u64)BLOCK) sl++;
        if (EQ) {
            const u64 off = (2ull << a.n_vars) - (2ull << (a.n_vars - j));
            q0 = a.eq0 + off;
            q1 = a.eq1 + off;
        }
        request_rest(q0, q1, n_pairs, sl);
        if (!take_mail(a.seq + (j - a.j), false)) return;
        if (a.lds_state) {
            in_lds = wrote;
            dst_is_a = !dst_is_a;
            __syncthreads();
        } else {
            // the tables this workgroup folded and stored are read back by other lanes: stores done, then no stale L1 lines
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
        continue;
    }
    if (ff.slots) {
        publish_sums<NP>(ff.slots + 64 * ((u64)blockIdx.y * gridDim.x + blockIdx.x), cf_seq, nullptr, acc);
        return;
    }
    if (tid == 0) {
        u64 *o = partial + ((u64)blockIdx.y * gridDim.x + blockIdx.x);
        const u64 total = (u64)gridDim.x * gridDim.y;
#pragma unroll
        for (int t = 0; t < NP; t++) {
            st_agent(o + (2 * t) * total, acc[t].c0);
            st_agent(o + (2 * t + 1) * total, acc[t].c1);
        }
    }
    if (take_ticket(ff.counter, gridDim.x * gridDim.y, &last_flag)) {
        E2 q[NP];
        gather_partials<NP>(ff, lds, q);
        publish_sums<NP>(ff.out_host, cf_seq, ff.counter, q);
    }
    return;
  }
}

// final evaluations: entry 0 of every table after the last fold
struct GatherDesc {
    const u64 *c0;
    const u64 *c1;
};
__global__ void gather_kernel(const GatherDesc *__restrict__ d, u32 n, u64 *__restrict__ out)
{
    u32 i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    out[2 * i] = d[i].c0[0];
    out[2 * i + 1] = d[i].c1 ? d[i].c1[0] : 0;
}

// ---------------------------------------------------------------------------
// embedding / padding of quantised integers
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(BLOCK)
embed_i64_kernel(const int64_t *__restrict__ in, u64 len, u64 padded_len, u64 *__restrict__ out)
{
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < padded_len; i += (u64)gridDim.x * BLOCK)
        out[i] = i < len ? gl::from_i64(in[i]) : 0;
}

// a raw tensor stored row-major in `src_dims` (its unpadded shape, or its padded one)
// into the base-field table of its padded shape: entry (i_0..i_{n-1}) is the
// embedded value when every i_a < unpadded_dims[a], else 0
constexpr int PAD_MAX_DIMS = 6;
struct PadTensorArgs {
    const void *in;
    int in_int;  // 8: int64, 2: int16, 0: base-field elements
    u32 n_dims;
    u64 padded_dims[PAD_MAX_DIMS], unpadded_dims[PAD_MAX_DIMS], src_strides[PAD_MAX_DIMS];
    u64 total;
    u64 *out;
};
__global__ void __launch_bounds__(BLOCK) pad_tensor_kernel(PadTensorArgs a)
{
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < a.total; i += (u64)gridDim.x * BLOCK) {
        u64 flat = i, off = 0;
        bool inside = true;
        for (int d = (int)a.n_dims - 1; d >= 0; d--) {
            u64 q = flat / a.padded_dims[d], c = flat - q * a.padded_dims[d];
            inside = inside && c < a.unpadded_dims[d];
            off += c * a.src_strides[d];
            flat = q;
        }
        u64 v = 0;
        if (inside)
            v = a.in_int == 8   ? gl::from_i64(((const int64_t *)a.in)[off])
                : a.in_int == 2 ? gl::from_i64(((const int16_t *)a.in)[off])
                                : ((const u64 *)a.in)[off];
        a.out[i] = v;
    }
}

// ---------------------------------------------------------------------------
// contraction of one tensor axis with a table beta (partial evaluation):
//   out[pre][i] = sum_k in[off_pre(pre) + k * stride_k + off_post(i)] * beta[k]
// The input is addressed through per-dimension strides so that the unpadded
// region of a padded tensor is read in place.
// ---------------------------------------------------------------------------
constexpr int AX_MAX_DIMS = 6;
struct AxisArgs {
    const u64 *in0;
    const u64 *in1;  // nullptr: base field or raw integers
    int in_int;      // 0: field elements; 8: raw int64; 2: raw int16 (embedded on load)
    const u64 *b0;
    const u64 *b1;
    u64 K, stride_k;
    u32 n_pre, n_post;
    u64 pre_dims[AX_MAX_DIMS], pre_strides[AX_MAX_DIMS];
    u64 post_dims[AX_MAX_DIMS], post_strides[AX_MAX_DIMS];
    u64 P, C;  // products of pre_dims / post_dims
    u64 k_per_slice;
    u32 n_slices;
    u64 *o0;
    u64 *o1;  // [slice][pre][i] when n_slices > 1, else [pre][i]
};

__device__ __forceinline__ u64 ax_offset(u64 flat, u32 n, const u64 *dims, const u64 *strides)
{
    u64 off = 0;
    for (int d = (int)n - 1; d >= 0; d--) {
        u64 q = flat / dims[d];
        off += (flat - q * dims[d]) * strides[d];
        flat = q;
    }
    return off;
}

__device__ __forceinline__ E2 ax_load(const AxisArgs &a, u64 off)
{
    if (a.in_int == 8) return gl::e2(gl::from_i64(((const int64_t *)a.in0)[off]), 0);
    if (a.in_int == 2) return gl::e2(gl::from_i64(((const int16_t *)a.in0)[off]), 0);
    return gl::e2(a.in0[off], a.in1 ? a.in1[off] : 0);
}

// lanes over the kept trailing index i (coalesced when the last kept dimension is contiguous)
__global__ void __launch_bounds__(BLOCK) axis_dot_col_kernel(AxisArgs a)
{
    __shared__ u64 lds[BLOCK * 2];
    const u32 lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const u64 tiles = (a.C + WAVE - 1) / WAVE;
    const u64 pre = blockIdx.x / tiles;
    const u64 i = (blockIdx.x - pre * tiles) * WAVE + lane;
    const u32 slice = blockIdx.y;
    E2 acc = gl::e2_zero();
    if (i < a.C) {
        const u64 base = ax_offset(pre, a.n_pre, a.pre_dims, a.pre_strides) + ax_offset(i, a.n_post, a.post_dims, a.post_strides);
        u64 k0 = (u64)slice * a.k_per_slice, k1 = k0 + a.k_per_slice;
        if (k1 > a.K) k1 = a.K;
        // four rows in flight per wavefront: the loop is a chain of loads otherwise (a row is 512 B per wavefront)
        constexpr u64 STEP = BLOCK / WAVE;
        auto term = [&](E2 v, E2 b) { return a.in1 ? gl::mul(v, b) : gl::mul_base(b, v.c0); };
        u64 k = k0 + wave;
        for (; k + 3 * STEP < k1; k += 4 * STEP) {
            const E2 v0 = ax_load(a, base + k * a.stride_k), v1 = ax_load(a, base + (k + STEP) * a.stride_k);
            const E2 v2 = ax_load(a, base + (k + 2 * STEP) * a.stride_k), v3 = ax_load(a, base + (k + 3 * STEP) * a.stride_k);
            const E2 b0 = gl::e2(a.b0[k], a.b1[k]), b1 = gl::e2(a.b0[k + STEP], a.b1[k + STEP]);
            const E2 b2 = gl::e2(a.b0[k + 2 * STEP], a.b1[k + 2 * STEP]), b3 = gl::e2(a.b0[k + 3 * STEP], a.b1[k + 3 * STEP]);
            acc = gl::add(acc, gl::add(gl::add(term(v0, b0), term(v1, b1)), gl::add(term(v2, b2), term(v3, b3))));
        }
        for (; k < k1; k += STEP) acc = gl::add(acc, term(ax_load(a, base + k * a.stride_k), gl::e2(a.b0[k], a.b1[k])));
    }
    lds[threadIdx.x * 2] = acc.c0;
    lds[threadIdx.x * 2 + 1] = acc.c1;
    __syncthreads();
    if (wave == 0 && i < a.C) {
#pragma unroll
        for (int w = 1; w < BLOCK / WAVE; w++) {
            acc.c0 = gl::add(acc.c0, lds[(w * WAVE + lane) * 2]);
            acc.c1 = gl::add(acc.c1, lds[(w * WAVE + lane) * 2 + 1]);
        }
        u64 o = ((u64)slice * a.P + pre) * a.C + i;
        a.o0[o] = acc.c0;
        a.o1[o] = acc.c1;
    }
}

// one workgroup per output, lanes over k (for C < 64, e.g. a row dot product)
__global__ void __launch_bounds__(BLOCK) axis_dot_row_kernel(AxisArgs a)
{
    __shared__ u32 lds[(BLOCK / WAVE) * 6];
    const u64 pre = blockIdx.x / a.C;
    const u64 i = blockIdx.x - pre * a.C;
    const u32 slice = blockIdx.y;
    const u64 base = ax_offset(pre, a.n_pre, a.pre_dims, a.pre_strides) + ax_offset(i, a.n_post, a.post_dims, a.post_strides);
    u64 k0 = (u64)slice * a.k_per_slice, k1 = k0 + a.k_per_slice;
    if (k1 > a.K) k1 = a.K;
    E2 acc[1] = {gl::e2_zero()};
    // four elements in flight per lane
    auto term = [&](E2 v, E2 b) { return a.in1 ? gl::mul(v, b) : gl::mul_base(b, v.c0); };
    u64 k = k0 + threadIdx.x;
    for (; k + 3 * BLOCK < k1; k += 4 * BLOCK) {
        const E2 v0 = ax_load(a, base + k * a.stride_k), v1 = ax_load(a, base + (k + BLOCK) * a.stride_k);
        const E2 v2 = ax_load(a, base + (k + 2 * BLOCK) * a.stride_k), v3 = ax_load(a, base + (k + 3 * BLOCK) * a.stride_k);
        const E2 b0 = gl::e2(a.b0[k], a.b1[k]), b1 = gl::e2(a.b0[k + BLOCK], a.b1[k + BLOCK]);
        const E2 b2 = gl::e2(a.b0[k + 2 * BLOCK], a.b1[k + 2 * BLOCK]), b3 = gl::e2(a.b0[k + 3 * BLOCK], a.b1[k + 3 * BLOCK]);
        acc[0] = gl::add(acc[0], gl::add(gl::add(term(v0, b0), term(v1, b1)), gl::add(term(v2, b2), term(v3, b3))));
    }
    for (; k < k1; k += BLOCK) acc[0] = gl::add(acc[0], term(ax_load(a, base + k * a.stride_k), gl::e2(a.b0[k], a.b1[k])));
    block_reduce<1>(acc, lds);
    if (threadIdx.x == 0) {
        u64 o = ((u64)slice * a.P + pre) * a.C + i;
        a.o0[o] = acc[0].c0;
        a.o1[o] = acc[0].c1;
    }
}

// ---------------------------------------------------------------------------
// evaluation of a table at a point without any memory of its own making: everything beyond the table and the two
// result words lives in one work area the caller of the kernels passes in (`ws`, WS_WORDS words)
//
//   value = sum_h eq_hi[h] * ( sum_l eq_lo[l] * table[h * 2^lo + l] ),   eq_lo over the lo lowest coordinates of the
// point, eq_hi over the others: two tables of at most 2^WS_LO_BITS entries instead of one of 2^n.  ws_eq_kernel
// writes them (and zeroes the ticket counter); ws_dot_kernel streams the table once, one row h per workgroup and
// step, a thread's eq_lo weights staying in registers across its rows, every sum unreduced until its end.
// ---------------------------------------------------------------------------
constexpr u32 WS_MAX_VARS = 24;
constexpr u32 WS_LO_BITS = 12;
constexpr u32 WS_MAX_BLOCKS = 1024;
// layout of the work area, in 64-bit words
constexpr u32 WS_OFF_COUNTER = 0;  // ticket counter (32 bits used)
constexpr u32 WS_OFF_LO0 = 32, WS_OFF_LO1 = WS_OFF_LO0 + (1u << WS_LO_BITS);
constexpr u32 WS_OFF_HI0 = WS_OFF_LO1 + (1u << WS_LO_BITS), WS_OFF_HI1 = WS_OFF_HI0 + (1u << WS_LO_BITS);
constexpr u32 WS_OFF_PARTIAL = WS_OFF_HI1 + (1u << WS_LO_BITS);  // 2 words per workgroup, word-major
constexpr u32 WS_WORDS = WS_OFF_PARTIAL + 2 * WS_MAX_BLOCKS;

struct WsPoint {
    u64 p[2 * WS_MAX_VARS];  // 2 limbs per coordinate
    u32 n, lo;               // coordinates; how many of them eq_lo covers
};

__global__ void __launch_bounds__(BLOCK) ws_eq_kernel(WsPoint pt, u64 *__restrict__ ws)
{
    const u32 i = blockIdx.x * BLOCK + threadIdx.x;
    // the ticket counter of the launch that follows starts at zero whatever an earlier call left behind
    if (i == 0) *reinterpret_cast<u32 *>(ws + WS_OFF_COUNTER) = 0;
    const u32 n_lo = 1u << pt.lo, n_hi = 1u << (pt.n - pt.lo);
    u32 first, bits, e;
    u64 *o0, *o1;
    if (i < n_lo) {
        first = 0, bits = pt.lo, e = i, o0 = ws + WS_OFF_LO0, o1 = ws + WS_OFF_LO1;
    } else if (i - n_lo < n_hi) {
        first = pt.lo, bits = pt.n - pt.lo, e = i - n_lo, o0 = ws + WS_OFF_HI0, o1 = ws + WS_OFF_HI1;
    } else {
        return;
    }
    E2 acc = gl::e2_one();
    for (u32 b = 0; b < bits; b++) {
        const E2 r = gl::e2(pt.p[2 * (first + b)], pt.p[2 * (first + b) + 1]);
        acc = gl::mul(acc, ((e >> b) & 1) ? r : gl::sub(gl::e2_one(), r));
    }
    o0[e] = acc.c0;
    o1[e] = acc.c1;
}

// KIND: 0 base-field entries, 1 extension entries, 8 raw int64, 2 raw int16.  FULL: rows of exactly 2^WS_LO_BITS entries
// (a thread's weights then sit in registers and its loads are 16 bytes wide).
template <int KIND, bool FULL>
__global__ void __launch_bounds__(BLOCK) ws_dot_kernel(const void *__restrict__ t0, const u64 *__restrict__ t1, u32 lo, u32 hi, u64 *ws, FastFin ff)
{
    __shared__ u32 lds[(BLOCK / WAVE) * 6];
    __shared__ int last_flag;
    const u64 *lo0 = ws + WS_OFF_LO0, *lo1 = ws + WS_OFF_LO1, *hi0 = ws + WS_OFF_HI0, *hi1 = ws + WS_OFF_HI1;
    const u32 rows = 1u << hi, cols = 1u << lo, tid = threadIdx.x;
    auto entry = [&](u64 i) -> E2 {
        if (KIND == 8) return gl::e2(gl::from_i64(reinterpret_cast<const int64_t *>(t0)[i]), 0);
        if (KIND == 2) return gl::e2(gl::from_i64(reinterpret_cast<const int16_t *>(t0)[i]), 0);
        if (KIND == 1) return gl::e2(reinterpret_cast<const u64 *>(t0)[i], t1[i]);
        return gl::e2(reinterpret_cast<const u64 *>(t0)[i], 0);
    };
    gl::E2Acc total = gl::e2acc_zero();
    if (FULL) {
        // columns 2 (tid + BLOCK k), 2 (tid + BLOCK k) + 1 for k = 0..STEPS-1
        constexpr int STEPS = (1 << WS_LO_BITS) / (2 * BLOCK);
        E2 w[2 * STEPS];
#pragma unroll
        for (int k = 0; k < STEPS; k++) {
            const U64x2 a = ld2(lo0 + 2 * (tid + BLOCK * k)), b = ld2(lo1 + 2 * (tid + BLOCK * k));
            w[2 * k] = gl::e2(a.x, b.x);
            w[2 * k + 1] = gl::e2(a.y, b.y);
        }
        for (u32 row = blockIdx.x; row < rows; row += gridDim.x) {
            const u64 base = (u64)row << WS_LO_BITS;
            E2 v[2 * STEPS];
#pragma unroll
            for (int k = 0; k < STEPS; k++) {
                const u64 i = base + 2 * (tid + BLOCK * k);
                if (KIND == 0 || KIND == 1) {
                    const U64x2 a = ld2(reinterpret_cast<const u64 *>(t0) + i);
                    U64x2 b = U64x2{0, 0};
                    if (KIND == 1) b = ld2(t1 + i);
                    v[2 * k] = gl::e2(a.x, b.x);
                    v[2 * k + 1] = gl::e2(a.y, b.y);
                } else {
                    v[2 * k] = entry(i);
                    v[2 * k + 1] = entry(i + 1);
                }
            }
            gl::E2Acc a = gl::e2acc_zero();
#pragma unroll
            for (int k = 0; k < 2 * STEPS; k++) {
                if (KIND == 1)
                    gl::acc_mul(a, v[k], gl::prep(w[k]));
                else
                    gl::acc_mul_base(a, w[k], v[k].c0);
            }
            gl::acc_mul(total, gl::acc_reduce(a), gl::prep(gl::e2(hi0[row], hi1[row])));
        }
    } else {
        for (u32 row = blockIdx.x; row < rows; row += gridDim.x) {
            const u64 base = (u64)row << lo;
            gl::E2Acc a = gl::e2acc_zero();
            for (u32 l = tid; l < cols; l += BLOCK) {
                const E2 wv = gl::e2(lo0[l], lo1[l]), v = entry(base + l);
                if (KIND == 1)
                    gl::acc_mul(a, v, gl::prep(wv));
                else
                    gl::acc_mul_base(a, wv, v.c0);
            }
            gl::acc_mul(total, gl::acc_reduce(a), gl::prep(gl::e2(hi0[row], hi1[row])));
        }
    }
    E2 acc[1] = {gl::acc_reduce(total)};
    block_reduce<1>(acc, lds);
    if (gridDim.x == 1) {
        publish_sums<1>(ff.out_host, ff.seq, ff.counter, acc);
        return;
    }
    if (tid == 0) {
        u64 *o = ws + WS_OFF_PARTIAL + blockIdx.x;
        st_agent(o, acc[0].c0);
        st_agent(o + gridDim.x, acc[0].c1);
    }
    if (take_ticket(ff.counter, gridDim.x, &last_flag)) {
        E2 q[1];
        gather_partials<1>(ff, lds, q);
        publish_sums<1>(ff.out_host, ff.seq, ff.counter, q);
    }
}

// sum the k-slices: out[j] = sum_s in[s * n + j]
__global__ void __launch_bounds__(BLOCK)
slice_sum_kernel(const u64 *__restrict__ i0, const u64 *__restrict__ i1, u64 n, u32 n_slices, u64 *__restrict__ o0,
                 u64 *__restrict__ o1)
{
    u64 j = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (j >= n) return;
    u64 a0 = 0, a1 = 0;
    for (u32 s = 0; s < n_slices; s++) {
        a0 = gl::add(a0, i0[(u64)s * n + j]);
        a1 = gl::add(a1, i1[(u64)s * n + j]);
    }
    o0[j] = a0;
    o1[j] = a1;
}

// copy `rows` rows of `row_len` entries into rows of `padded_len`, zero filling
__global__ void __launch_bounds__(BLOCK)
pad_rows_kernel(const u64 *__restrict__ i0, const u64 *__restrict__ i1, u64 rows, u64 row_len, u64 padded_len,
                u64 *__restrict__ o0, u64 *__restrict__ o1)
{
    u64 total = rows * padded_len;
    for (u64 j = (u64)blockIdx.x * BLOCK + threadIdx.x; j < total; j += (u64)gridDim.x * BLOCK) {
        u64 r = j / padded_len, c = j - r * padded_len;
        bool in = c < row_len;
        o0[j] = in ? i0[r * row_len + c] : 0;
        o1[j] = in ? (i1 ? i1[r * row_len + c] : 0) : 0;
    }
}

// ---------------------------------------------------------------------------
// LogUp fraction-sum layers: (n1, d1) + (n2, d2) = (n1 d2 + n2 d1, d1 d2) over the
// low/high halves of the previous layer
// ---------------------------------------------------------------------------
constexpr int LOGUP_MAX_COLS = 8;
struct LogupFirstArgs {
    const u64 *cols[LOGUP_MAX_COLS];  // base-field columns
    u32 n_cols;
    const u64 *numer;  // base-field multiplicities or nullptr (numerators -1)
    u64 c0, c1;        // constant challenge
    u64 pw[2 * LOGUP_MAX_COLS];  // powers of the column challenge
    u64 half;
    u64 *n0, *n1, *d0, *d1;
};

__global__ void __launch_bounds__(BLOCK) logup_first_kernel(LogupFirstArgs a)
{
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < a.half; i += (u64)gridDim.x * BLOCK) {
        // (the first column's power of the column challenge is 1: no product)
        E2 dlo = gl::e2(gl::add(a.c0, a.cols[0][i]), a.c1), dhi = gl::e2(gl::add(a.c0, a.cols[0][i + a.half]), a.c1);
        for (u32 k = 1; k < a.n_cols; k++) {
            E2 pw = gl::e2(a.pw[2 * k], a.pw[2 * k + 1]);
            dlo = gl::add(dlo, gl::mul_base(pw, a.cols[k][i]));
            dhi = gl::add(dhi, gl::mul_base(pw, a.cols[k][i + a.half]));
        }
        E2 num;
        if (a.numer) {
            num = gl::add(gl::mul_base(dhi, a.numer[i]), gl::mul_base(dlo, a.numer[i + a.half]));
        } else {
            num = gl::neg(gl::add(dlo, dhi));
        }
        E2 den = gl::mul(dlo, dhi);
        a.n0[i] = num.c0;
        a.n1[i] = num.c1;
        a.d0[i] = den.c0;
        a.d1[i] = den.c1;
    }
}

__global__ void __launch_bounds__(BLOCK)
logup_next_kernel(const u64 *__restrict__ pn0, const u64 *__restrict__ pn1, const u64 *__restrict__ pd0,
                  const u64 *__restrict__ pd1, u64 half, u64 *__restrict__ n0, u64 *__restrict__ n1,
                  u64 *__restrict__ d0, u64 *__restrict__ d1)
{
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < half; i += (u64)gridDim.x * BLOCK) {
        E2 nl = gl::e2(pn0[i], pn1[i]), nh = gl::e2(pn0[i + half], pn1[i + half]);
        E2 dl = gl::e2(pd0[i], pd1[i]), dh = gl::e2(pd0[i + half], pd1[i + half]);
        E2 num = gl::add(gl::mul(nl, dh), gl::mul(nh, dl));
        E2 den = gl::mul(dl, dh);
        n0[i] = num.c0;
        n1[i] = num.c1;
        d0[i] = den.c0;
        d1[i] = den.c1;
    }
}

// The levels of at most 2^LOGUP_TAIL_BITS entries of a tree, all in one launch of one workgroup: below that a level is a
// dispatch of 3 us whatever its size, and a tree has ten of them.  A level is read from LDS, where the level before left
// it (the first from device memory), and written to LDS and to the arena.  The four entries of the last level (n_lo,
// n_hi, d_lo, d_hi, what the prover puts on the transcript first) also go to the host, as a round's result does.
constexpr u32 LOGUP_TAIL_BITS = 10;
constexpr int LOGUP_TAIL_BLOCK = 1024;
// The levels of at most LOGUP_SHADOW_MAX entries per array also go to host memory (`shadow`): a sumcheck over such a
// layer is a few hundred field products, which the host does in less time than a launch takes to start, and for that
// it needs the entries.  A level of `cur` entries per array lies at word 4 (cur - 2) of the area (the levels below it
// take 4 * 2, 4 * 4, ... words): numerators' limb arrays c0 and c1, then the denominators', `cur` words each.
constexpr u32 LOGUP_SHADOW_MAX = 256;
constexpr u32 LOGUP_SHADOW_WORDS = 4 * (2 * LOGUP_SHADOW_MAX - 2);
__host__ __device__ __forceinline__ u32 logup_shadow_off(u32 cur) { return 4 * (cur - 2); }
struct LogupTailArgs {
    u64 *c0, *c1;                       // the tree's arena
    u64 off[LOGUP_TAIL_BITS + 2];       // off[0]: the level read first; off[l + 1]: level l of this launch
    u32 n_levels;
    u64 first_cur;                      // entries per array of the first level written
    u64 *out_host;                      // 8 words + check word + sequence number (slots 8 and 9)
    u64 seq;
    u64 *shadow;                        // host memory for the small levels (LOGUP_SHADOW_WORDS words), or nullptr
};
__global__ void __launch_bounds__(LOGUP_TAIL_BLOCK) logup_tail_kernel(LogupTailArgs a)
{
    constexpr u32 CAP = 1u << LOGUP_TAIL_BITS;
    // numerators (two limb arrays) and denominators (two) of a level: CAP entries each in `big`, half of that in `small`
    __shared__ u64 big[4 * CAP], small_[2 * CAP];
    u32 cur = (u32)a.first_cur;
    for (u32 l = 0; l < a.n_levels; l++, cur >>= 1) {
        const u32 prev = 2 * cur;
        const bool to_big = (l & 1) == 0;
        const u32 cap_s = to_big ? CAP / 2 : CAP, cap_d = to_big ? CAP : CAP / 2;
        const u64 *src = to_big ? small_ : big;
        u64 *dst = to_big ? big : small_;
        const u64 *g0 = a.c0 + a.off[l], *g1 = a.c1 + a.off[l];
        u64 *n0 = a.c0 + a.off[l + 1], *n1 = a.c1 + a.off[l + 1], *d0 = n0 + cur, *d1 = n1 + cur;
        for (u32 i = threadIdx.x; i < cur; i += LOGUP_TAIL_BLOCK) {
            E2 nl, nh, dl, dh;
            if (l == 0) {
                nl = gl::e2(g0[i], g1[i]), nh = gl::e2(g0[i + cur], g1[i + cur]);
                dl = gl::e2(g0[prev + i], g1[prev + i]), dh = gl::e2(g0[prev + i + cur], g1[prev + i + cur]);
            } else {
                nl = gl::e2(src[i], src[cap_s + i]), nh = gl::e2(src[i + cur], src[cap_s + i + cur]);
                dl = gl::e2(src[2 * cap_s + i], src[3 * cap_s + i]), dh = gl::e2(src[2 * cap_s + i + cur], src[3 * cap_s + i + cur]);
            }
            const E2 num = gl::add(gl::mul(nl, dh), gl::mul(nh, dl));
            const E2 den = gl::mul(dl, dh);
            n0[i] = num.c0;
            n1[i] = num.c1;
            d0[i] = den.c0;
            d1[i] = den.c1;
            dst[i] = num.c0;
            dst[cap_d + i] = num.c1;
            dst[2 * cap_d + i] = den.c0;
            dst[3 * cap_d + i] = den.c1;
            if (a.shadow && cur <= LOGUP_SHADOW_MAX) {
                u64 *sh = a.shadow + logup_shadow_off(cur);
                st_sys(sh + i, num.c0);
                st_sys(sh + cur + i, num.c1);
                st_sys(sh + 2 * cur + i, den.c0);
                st_sys(sh + 3 * cur + i, den.c1);
            }
        }
        __syncthreads();
    }
    // (the host reads the small levels once it has seen the sequence number below: every lane's stores to host memory
    // are out before the workgroup meets, and the number is written after that)
    if (a.shadow) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        // the last level: two numerators and two denominators, in the buffer written last
        const bool in_big = ((a.n_levels - 1) & 1) == 0;
        const u64 *dst = in_big ? big : small_;
        const u32 cap_d = in_big ? CAP : CAP / 2;
        const u64 w[8] = {dst[0], dst[cap_d], dst[1], dst[cap_d + 1], dst[2 * cap_d], dst[3 * cap_d], dst[2 * cap_d + 1], dst[3 * cap_d + 1]};
        publish_words(a.out_host, 0, w, 8, a.seq, 9, 8);
    }
}

// ---------------------------------------------------------------------------
// element-wise field operations on device vectors (arithmetic self-check)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(BLOCK)
field_op_kernel(int op, const u64 *__restrict__ a0, const u64 *__restrict__ a1, const u64 *__restrict__ b0,
                const u64 *__restrict__ b1, u64 n, u64 *__restrict__ o0, u64 *__restrict__ o1)
{
    u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= n) return;
    E2 a = gl::e2(a0[i], a1[i]), b = gl::e2(b0[i], b1[i]), r;
    switch (op) {
    case 0: r = gl::add(a, b); break;
    case 1: r = gl::sub(a, b); break;
    case 2: r = gl::mul(a, b); break;
    case 3: r = gl::e2(gl::mul(a.c0, b.c0), gl::mul(a.c1, b.c1)); break;  // two independent base products
    case 4: r = gl::mul_base(a, b.c0); break;
    case 5: r = gl::e2(gl::from_i64((int64_t)a.c0), gl::mul_small(a.c1, (u32)b.c1)); break;
    case 6: r = gl::fma(a, gl::prep(b), a); break;
    case 7: r = gl::e2(gl::muladd(a.c0, b.c0, a.c1), gl::dot2(a.c0, b.c0, a.c1, b.c1, b.c0)); break;
    case 8: {
        // a long unreduced sum: 40 (a b + b a.c1 + a) + (0, 40 b.c0)
        gl::E2Acc acc = gl::e2acc_zero();
        const gl::E2P bp = gl::prep(b);
        for (int k = 0; k < 40; k++) {
            gl::acc_mul(acc, a, bp);
            gl::acc_mul_base(acc, b, a.c1);
            gl::acc_e2(acc, a);
            gl::acc_add64(acc.c1, b.c0);
        }
        r = gl::acc_reduce(acc);
        break;
    }
    default: r = gl::e2_zero();
    }
    o0[i] = r.c0;
    o1[i] = r.c1;
}

// plain streaming copy, 16 bytes per lane
__global__ __launch_bounds__(BLOCK) void copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, u64 n16)
{
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < n16; i += (u64)gridDim.x * BLOCK) dst[i] = src[i];
}

// plain streaming read, 16 bytes per lane: the yardstick for launches that only read (a round's first evaluation).
// The sums keep the loads alive; one word per workgroup is written.
__global__ __launch_bounds__(BLOCK) void read_kernel(const uint4 *__restrict__ src, u64 n16, u32 *__restrict__ out)
{
    u32 acc = 0;
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < n16; i += (u64)gridDim.x * BLOCK) {
        const uint4 v = src[i];
        acc += v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) out[blockIdx.x] = acc;  // (practically never: the loads cannot be dropped, nothing is written)
}

}  // namespace dpk
