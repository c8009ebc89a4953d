// C ABI of the sumcheck prover library: contexts, table storage, sessions.
// Device code is in kernels.hpp; this file owns memory, launch geometry and the
// round protocol.  There is no CPU path: every entry point that computes
// launches kernels on the context's stream.
#include "../../include/dpsumcheck.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "kernels.hpp"

using gl::E2;
using gl::u32;
using gl::u64;

// Work area of dps_mle_evaluate_noalloc, the one entry point that allocates nothing: eq tables of the two halves of
// the point, per-workgroup partial sums and a ticket counter (dpk::WS_WORDS words, 144 KiB).  File-scope device
// memory: every GPU the library runs on holds its own copy, at its own address, until the process ends.  In host
// code the name below is only a handle for hipGetSymbolAddress; kernels are given the address that call returns.
static __device__ __align__(256) uint64_t scratch[dpk::WS_WORDS];

namespace {

// 3 workgroups per CU on 256 CUs: measured best for the streaming kernels (each workgroup pays a fixed
// reduction + ticket epilogue, so more, thinner workgroups lose more than they gain in latency hiding)
constexpr u32 MAX_BLOCKS = 768;
// areas of pinned memory for the outputs (and the small levels) of the fraction trees built last
constexpr u32 LOGUP_OUT_AREAS = 8;
constexpr size_t LOGUP_SHADOW_STRIDE = 2048;  // words per tree: dpk::LOGUP_SHADOW_WORDS rounded up
// A sum of at most this many variables over tables the host holds copies of is worked out on the host, every round of it
constexpr u32 HOST_ONLY_MAX_VARS = 7;
constexpr size_t DESC_STAGE_BYTES = 256 << 10;  // pinned staging buffer of a context for descriptor uploads
constexpr u32 PAIR12_BLOCKS = 1024;  // workgroups of the launch of the first two rounds (64 quads each: a stride of 2^16 quads)

// ---------------------------------------------------------------------------
// context
// ---------------------------------------------------------------------------
struct ProfRec {
    int kernel;
    hipEvent_t a, b;
    double bytes;
};

struct ProfStat {
    u64 launches = 0;
    double ms = 0, bytes = 0;
    u64 max_launches = 0;
    double max_ms = 0, max_bytes = 0;
};

}  // namespace

struct dps_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::string err;
    // cached device blocks, keyed by size
    std::multimap<size_t, void *> free_blocks;
    std::map<void *, size_t> live_blocks;
    u64 *d_lagrange = nullptr;  // [9][9][9]
    std::vector<u64> h_lagrange;
    u64 h_inv_den[9][9] = {};   // [d][k]: 1 / prod_{m != k, m <= d} (k - m), the Lagrange denominators over the nodes 0..d
    u32 *d_counter = nullptr;   // ticket counter of the evaluation launches; every launch leaves it at zero
    u64 *d_slice_ctr = nullptr; // sum counters of a resident launch of several workgroups (zero between trips), its ticket behind them
    u64 *h_pinned = nullptr;    // host-visible result buffer
    u64 *d_pinned = nullptr;    // device address of the same buffer
    size_t pinned_words = 0;
    double wall_clock_scale = 1.0;  // rate of the device's real-time counter / 100 MHz
    u64 logup_builds = 0;           // fraction trees built so far (their outputs rotate through a few areas of the pinned buffer)
    u64 *h_shadow = nullptr;        // host copies of those trees' small levels, one area per output area (written by the build's last launch)
    u64 *d_shadow = nullptr;        // device address of the same memory
    hipEvent_t stage_event = nullptr;  // recorded after a launch that reads the staging region of the pinned buffer
    bool stage_pending = false;
    // A session's descriptor block goes to the device through this pinned buffer (a copy from pageable memory is staged by
    // the runtime inside the call: 70 us for the 70 KB of a 17-group session); the event says when the copy has read it
    char *h_desc_stage = nullptr;
    hipEvent_t desc_event = nullptr;
    bool desc_pending = false;
    size_t res_off = 0;         // round results: h_pinned[res_off ..], sequence number at res_off + HOST_SEQ_SLOT
    u64 seq = 0;                // last sequence number handed to a launch
    struct dps_sc *tail_owner = nullptr;  // session whose tail kernel is resident on the stream
    u32 units_held = 0;         // compute units of the device's ledger that launch holds (admit_waiting_launch)
    u64 *ws = nullptr;          // this device's copy of the allocation-free entry point's work area
    bool profiling = false;
    std::vector<ProfRec> recs;
    std::vector<hipEvent_t> ev_pool;
    ProfStat stats[DPS_K_COUNT];
};

namespace {

int32_t fail(dps_ctx *ctx, int32_t code, const char *fmt, ...)
{
    if (ctx) {
        char buf[512];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        ctx->err = buf;
    }
    return code;
}

#define HIPCHK(ctx, call)                                                                                       \
    do {                                                                                                        \
        hipError_t e_ = (call);                                                                                 \
        if (e_ != hipSuccess)                                                                                   \
            return fail(ctx, e_ == hipErrorOutOfMemory ? DPS_ERR_OOM : DPS_ERR_HIP, "%s: %s (%s:%d)", #call,   \
                        hipGetErrorString(e_), __FILE__, __LINE__);                                             \
    } while (0)

#define CHK(expr)                       \
    do {                                \
        int32_t rc_ = (expr);           \
        if (rc_ != DPS_OK) return rc_;  \
    } while (0)

struct DeviceGuard {
    int prev = -1;
    bool changed = false;
    explicit DeviceGuard(int dev)
    {
        if (hipGetDevice(&prev) != hipSuccess) prev = -1;
        if (prev != dev) {
            (void)hipSetDevice(dev);
            changed = true;
        }
    }
    ~DeviceGuard()
    {
        // (nothing to restore in the usual case: a call per round that is not made)
        if (changed && prev >= 0) (void)hipSetDevice(prev);
    }
};

size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Behind the Lagrange weights: the ticket counter (and at +128 the words through which a launch's first workgroup
// passes the mail on), then the sum counters of a resident launch of several workgroups and their ticket.
constexpr size_t SLICE_CTR_WORDS = (size_t)dpk::SL_MAX_GROUPS * dpk::SL_GROUP_WORDS * dpk::SL_CTR_STRIDE;  // counters of a resident launch, each apart
constexpr size_t COUNTER_BYTES = 256 + SLICE_CTR_WORDS * 8 + 256 + (size_t)dpk::MAIL_RELAY_WORDS * 8;

// Address of `scratch` on a device, asked for once per device with that device current (every GPU has its own copy).
constexpr int WS_MAX_DEVICES = 64;
int32_t work_area_of_device(int device, u64 **out)
{
    static std::mutex mu;
    static u64 *ptr_of[WS_MAX_DEVICES] = {};
    if (device < 0 || device >= WS_MAX_DEVICES) return DPS_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr_of[device]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return DPS_ERR_HIP;
        }
        ptr_of[device] = static_cast<u64 *>(p);
    }
    *out = ptr_of[device];
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// Admission of launches that wait on the GPU.
//
// Some launches stay on the GPU while the host takes its turn: the resident launches of the late rounds (their
// workgroups hold a compute unit each from the first trip to the last, and a trip completes only when every one of them
// has added its share) and the launches made ahead of their round (they wait for the challenge by mail, the large
// ones behind their first workgroup, which passes it on).  Contexts are used from different threads, so several such
// launches can meet on one GPU; if two of them were each placed in part, neither could ever complete -- each would
// wait for workgroups that find no room while the other waits.  So every launch that waits takes its place in a
// ledger of the device first: one compute unit per workgroup (a workgroup touches one compute unit, and any workgroup
// fits an untouched one, so launches admitted together are placed together, in whatever order their workgroups
// arrive), up to the device's number of compute units.  A launch that does not get its place is not made: a round
// that would have been launched ahead is launched when its challenge is there, and a session whose resident launch
// is refused runs the same rounds as launches of their own.  The results are the same bits either way.
// Launches that wait for nothing (all others) come and go by themselves and are not counted.
// ---------------------------------------------------------------------------
struct DeviceLedger {
    std::mutex mu;
    int total = -1;  // compute units of the device (-1: not asked yet)
    int limit = -1;  // the caller's limit (dps_device_set_resident_budget; -1: none)
    int used = 0;
};
DeviceLedger &ledger_of(int device)
{
    static DeviceLedger ledgers[WS_MAX_DEVICES];
    return ledgers[device];
}

// `together`: the launch makes progress only with all of its workgroups on the GPU (refused when the device is too
// small for that); a launch whose workgroups each run to the end once the mail is there takes at most the whole budget.
bool admit_waiting_launch(dps_ctx *ctx, u32 workgroups, bool together)
{
    DeviceLedger &l = ledger_of(ctx->device);
    std::lock_guard<std::mutex> lock(l.mu);
    // (a context has one waiting launch at a time: whatever it still holds is of a launch that has ended)
    l.used -= (int)ctx->units_held;
    ctx->units_held = 0;
    const int budget = l.limit >= 0 ? std::min(l.limit, l.total) : l.total;
    int want = (int)std::min<u32>(workgroups, 1u << 20);
    if (want > budget) {
        if (together) return false;
        want = budget;
    }
    if (want <= 0 || l.used + want > budget) return false;
    l.used += want;
    ctx->units_held = (u32)want;
    return true;
}

// the context's waiting launch has had its last mail (or was told to leave and has left): its place is free again
void waiting_launch_over(dps_ctx *ctx)
{
    ctx->tail_owner = nullptr;
    if (!ctx->units_held) return;
    DeviceLedger &l = ledger_of(ctx->device);
    std::lock_guard<std::mutex> lock(l.mu);
    l.used -= (int)ctx->units_held;
    ctx->units_held = 0;
}

// A resident tail kernel blocks the stream until its session finishes.  Any other
// use of the context first makes that kernel exit (its session is then failed).
void tail_abort(dps_ctx *ctx);

int32_t pool_alloc(dps_ctx *ctx, size_t bytes, void **out)
{
    bytes = round_up(std::max<size_t>(bytes, 256), 256);
    auto it = ctx->free_blocks.lower_bound(bytes);
    if (it != ctx->free_blocks.end() && it->first <= bytes + bytes / 2 + 4096) {
        *out = it->second;
        ctx->live_blocks[it->second] = it->first;
        ctx->free_blocks.erase(it);
        return DPS_OK;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        // give cached blocks back to the driver and retry once (queued work may still use them: blocks are handed
        // back to the pool without waiting for the stream)
        (void)hipStreamSynchronize(ctx->stream);
        for (auto &kv : ctx->free_blocks) (void)hipFree(kv.second);
        ctx->free_blocks.clear();
        e = hipMalloc(&p, bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(ctx, DPS_ERR_OOM, "hipMalloc(%zu bytes): %s", bytes, hipGetErrorString(e));
        }
    }
    ctx->live_blocks[p] = bytes;
    *out = p;
    return DPS_OK;
}

void pool_free(dps_ctx *ctx, void *p)
{
    if (!p) return;
    auto it = ctx->live_blocks.find(p);
    if (it == ctx->live_blocks.end()) return;
    ctx->free_blocks.emplace(it->second, p);
    ctx->live_blocks.erase(it);
}

// A kernel's patience, as the kernels count it: units of 256 ticks of the device's real-time counter.  `units`: the figure at
// 100 MHz (2.56 us a unit); scaled by the counter's actual rate.
u32 wait_units(const dps_ctx *ctx, u32 units) { return (u32)std::min<double>(4.0e9, (double)units * ctx->wall_clock_scale); }

// profiling -----------------------------------------------------------------
hipEvent_t prof_event(dps_ctx *ctx)
{
    if (!ctx->ev_pool.empty()) {
        hipEvent_t e = ctx->ev_pool.back();
        ctx->ev_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

struct ProfScope {
    dps_ctx *ctx;
    ProfRec rec;
    bool on;
    ProfScope(dps_ctx *c, int kernel, double bytes) : ctx(c), on(c->profiling)
    {
        if (!on) return;
        rec.kernel = kernel;
        rec.bytes = bytes;
        rec.a = prof_event(ctx);
        rec.b = prof_event(ctx);
        (void)hipEventRecord(rec.a, ctx->stream);
    }
    ~ProfScope()
    {
        if (!on) return;
        (void)hipEventRecord(rec.b, ctx->stream);
        ctx->recs.push_back(rec);
    }
};

void prof_collect(dps_ctx *ctx)
{
    for (auto &r : ctx->recs) {
        float ms = 0;
        (void)hipEventSynchronize(r.b);
        (void)hipEventElapsedTime(&ms, r.a, r.b);
        ProfStat &s = ctx->stats[r.kernel];
        s.launches++;
        s.ms += ms;
        s.bytes += r.bytes;
        if (r.bytes > s.max_bytes * 1.0000001) {
            s.max_bytes = r.bytes;
            s.max_ms = ms;
            s.max_launches = 1;
        } else if (r.bytes >= s.max_bytes * 0.9999999 && s.max_launches > 0) {
            s.max_ms += ms;
            s.max_launches++;
        }
        ctx->ev_pool.push_back(r.a);
        ctx->ev_pool.push_back(r.b);
    }
    ctx->recs.clear();
}

u32 grid_for(u64 items, u32 per_block = dpk::BLOCK)
{
    u64 b = (items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return (u32)std::min<u64>(b, MAX_BLOCKS);
}

// host-side field helpers for constants (Lagrange weights, powers of two)
u64 h_pow(u64 a, u64 e)
{
    u64 r = 1;
    while (e) {
        if (e & 1) r = gl::mul(r, a);
        a = gl::mul(a, a);
        e >>= 1;
    }
    return r;
}
// a^(p - 2), p - 2 = 2^64 - 2^32 - 1: 63 squarings and 9 products along the runs of ones of the exponent (the round loop
// of a sum with an eq factor inverts one element per round)
u64 h_inv(u64 a)
{
    // base^(2^n) * tail
    auto sq_mul = [](u64 base, int n, u64 tail) {
        for (int i = 0; i < n; i++) base = gl::mul(base, base);
        return gl::mul(base, tail);
    };
    const u64 t2 = sq_mul(a, 1, a);        // 2^2 - 1
    const u64 t3 = sq_mul(t2, 1, a);       // 2^3 - 1
    const u64 t6 = sq_mul(t3, 3, t3);      // 2^6 - 1
    const u64 t12 = sq_mul(t6, 6, t6);     // 2^12 - 1
    const u64 t24 = sq_mul(t12, 12, t12);  // 2^24 - 1
    const u64 t30 = sq_mul(t24, 6, t6);    // 2^30 - 1
    const u64 t31 = sq_mul(t30, 1, a);     // 2^31 - 1
    const u64 t63 = sq_mul(t31, 32, t31);  // (2^31 - 1) 2^32 + 2^31 - 1
    return sq_mul(t63, 1, a);              // 2^64 - 2^32 - 1
}
E2 h_e2_inv(E2 a)
{
    u64 n = h_inv(gl::sub(gl::mul(a.c0, a.c0), gl::mul_small(gl::mul(a.c1, a.c1), (u32)gl::W)));
    return gl::e2(gl::mul(a.c0, n), gl::mul(gl::neg(a.c1), n));
}
// eq1(a, b) = a b + (1 - a)(1 - b)
E2 h_eq1(E2 a, E2 b)
{
    E2 one = gl::e2_one();
    return gl::add(gl::mul(a, b), gl::mul(gl::sub(one, a), gl::sub(one, b)));
}

// ---------------------------------------------------------------------------
// storage
// ---------------------------------------------------------------------------
struct Storage {
    dps_ctx *ctx = nullptr;
    u64 *c0 = nullptr;
    u64 *c1 = nullptr;
    bool owned = true;
    ~Storage()
    {
        if (owned && ctx) {
            pool_free(ctx, c0);
            pool_free(ctx, c1);
        }
    }
};

}  // namespace

// A table built by dps_eq_build remembers its point.  Behind the 2^m entries of
// eq(rho, .) the storage holds the tables eq(rho_{l..m-1}, .) for l = 1..m (2^(m-l)
// entries each, level l at entry offset 2^(m+1) - 2^(m-l+1)): the sumcheck reads
// level j in round j instead of folding the full table.
// Nothing of it is written before somebody reads it: a product or multi-term session takes the eq factor in closed
// form and reads suffix levels only (a product of 24 variables: levels 7..24 and the low tables; levels 0..6 are 2^25
// entries, half a gigabyte of writes, that it never touches), while a download, a view, an evaluation or a session
// that reads the table as an ordinary factor needs level 0.  `built` says which levels are there.
struct EqInfo {
    u32 m;
    u32 fact_levels = 0;  // levels 1..fact_levels have room for a low table behind the levels (eq_low_off)
    bool fact_built = false;  // ... and the low tables are there (built when a product session first wants them)
    u64 built = 0;        // bit l: level l is materialised
    std::vector<E2> point;
};

struct dps_mle {
    dps_ctx *ctx;
    std::shared_ptr<Storage> st;
    int32_t kind;
    u64 offset;
    u64 len;
    std::shared_ptr<EqInfo> eq;  // set on eq tables (and on views covering the whole table)
    u32 pad_vars = 0;            // > 0: read by a sumcheck as zero-padded to this many variables
    // A small level of a fraction tree: the host's copy of these entries (limb arrays), valid once the build's last launch has
    // published under sh_seq in output area sh_slot, and until the context has built LOGUP_OUT_AREAS more trees (sh_build)
    const u64 *sh0 = nullptr, *sh1 = nullptr;
    u64 sh_seq = 0, sh_build = 0;
    u32 sh_slot = 0;
    const u64 *p0() const { return st->c0 + offset; }
    const u64 *p1() const { return st->c1 ? st->c1 + offset : nullptr; }
};

namespace {

int32_t plain_ready(const dps_mle *t);

bool is_pow2(u64 x) { return x && !(x & (x - 1)); }
// raw quantised integers (not field elements): readable by the tensor kernels only
bool is_raw(int32_t kind) { return kind == DPS_I64 || kind == DPS_I16; }
int raw_bytes(int32_t kind) { return kind == DPS_I64 ? 8 : kind == DPS_I16 ? 2 : 0; }
u32 log2u(u64 x)
{
    u32 l = 0;
    while ((1ull << l) < x) l++;
    return l;
}

int32_t new_table(dps_ctx *ctx, int32_t kind, u64 len, dps_mle **out)
{
    auto st = std::make_shared<Storage>();
    st->ctx = ctx;
    void *p = nullptr;
    CHK(pool_alloc(ctx, kind == DPS_I16 ? (len * 2 + 7) / 8 * 8 : len * 8, &p));
    st->c0 = (u64 *)p;
    if (kind == DPS_EXT2) {
        CHK(pool_alloc(ctx, len * 8, &p));
        st->c1 = (u64 *)p;
    }
    dps_mle *m = new (std::nothrow) dps_mle{ctx, st, kind, 0, len, nullptr};
    if (!m) return fail(ctx, DPS_ERR_OOM, "host allocation failed");
    *out = m;
    return DPS_OK;
}

}  // namespace

// ---------------------------------------------------------------------------
// context entry points
// ---------------------------------------------------------------------------
extern "C" const char *dps_status_str(int32_t s)
{
    switch (s) {
    case DPS_OK: return "ok";
    case DPS_ERR_INVALID: return "invalid argument";
    case DPS_ERR_HIP: return "HIP runtime error";
    case DPS_ERR_OOM: return "out of memory";
    case DPS_ERR_STATE: return "call out of order";
    case DPS_ERR_UNSUPPORTED: return "unsupported degree or arity";
    case DPS_ERR_CALLBACK: return "transcript callback failed";
    default: return "unknown status";
    }
}

extern "C" const char *dps_kernel_name(int32_t k)
{
    static const char *names[DPS_K_COUNT] = {"prod_kernel<first round>", "prod_kernel<fold+eval>", "eval_terms_kernel",
                                             "fold_kernel",              "eq_expand_kernel",       "axis_dot_kernel",
                                             "logup_layer_kernel",       "finalize_kernel",        "tail_kernel"};
    return (k >= 0 && k < DPS_K_COUNT) ? names[k] : "?";
}

extern "C" const char *dps_last_error(const dps_ctx *ctx) { return ctx ? ctx->err.c_str() : "null context"; }

extern "C" int32_t dps_ctx_create(int32_t device, dps_ctx **out)
{
    if (!out) return DPS_ERR_INVALID;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) {
        (void)hipGetLastError();
        return DPS_ERR_HIP;
    }
    dps_ctx *ctx = new (std::nothrow) dps_ctx();
    if (!ctx) return DPS_ERR_OOM;
    ctx->device = device;
    DeviceGuard g(device);
    auto bail = [&](int32_t rc) {
        delete ctx;
        return rc;
    };
    if (hipStreamCreate(&ctx->stream) != hipSuccess) return bail(DPS_ERR_HIP);
    // (the context's device is current here)
    if (int32_t rc = work_area_of_device(device, &ctx->ws); rc != DPS_OK) return bail(rc);
    {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) return bail(DPS_ERR_HIP);
        DeviceLedger &l = ledger_of(device);
        std::lock_guard<std::mutex> lock(l.mu);
        l.total = cus;
    }
    // Lagrange weights: a polynomial of degree k known at 0..k, evaluated at t <= 8
    std::vector<u64> lag(9 * 9 * 9, 0);
    for (u32 k = 0; k <= 8; k++)
        for (u32 t = 0; t <= 8; t++)
            for (u32 i = 0; i <= k; i++) {
                u64 num = 1, den = 1;
                for (u32 m = 0; m <= k; m++) {
                    if (m == i) continue;
                    num = gl::mul(num, gl::sub((u64)t, (u64)m));
                    den = gl::mul(den, gl::sub((u64)i, (u64)m));
                }
                lag[(k * 9 + t) * 9 + i] = gl::mul(num, h_inv(den));
            }
    ctx->h_lagrange = lag;
    for (u32 d = 0; d <= 8; d++)
        for (u32 k = 0; k <= d; k++) {
            u64 den = 1;
            for (u32 m = 0; m <= d; m++)
                if (m != k) den = gl::mul(den, gl::sub((u64)k, (u64)m));
            ctx->h_inv_den[d][k] = h_inv(den);
        }
    const size_t lag_bytes = round_up(lag.size() * 8, 256);
    if (hipMalloc((void **)&ctx->d_lagrange, lag_bytes + COUNTER_BYTES) != hipSuccess) return bail(DPS_ERR_OOM);
    if (hipMemcpy(ctx->d_lagrange, lag.data(), lag.size() * 8, hipMemcpyHostToDevice) != hipSuccess) return bail(DPS_ERR_HIP);
    ctx->d_counter = (u32 *)((char *)ctx->d_lagrange + lag_bytes);
    ctx->d_slice_ctr = (u64 *)((char *)ctx->d_counter + 256);
    if (hipMemset(ctx->d_counter, 0, COUNTER_BYTES) != hipSuccess) return bail(DPS_ERR_HIP);
    {
        int khz = 0;
        if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device) == hipSuccess && khz > 0)
            ctx->wall_clock_scale = (double)khz / 100000.0;
        else
            (void)hipGetLastError();
    }
    ctx->pinned_words = 16384;
    if (hipEventCreateWithFlags(&ctx->stage_event, hipEventDisableTiming) != hipSuccess) return bail(DPS_ERR_HIP);
    // fine-grained host memory: a kernel's system-scope stores become visible to the polling host while the kernel runs
    if (hipHostMalloc((void **)&ctx->h_pinned, ctx->pinned_words * 8, hipHostMallocMapped | hipHostMallocCoherent) != hipSuccess) {
        (void)hipGetLastError();
        if (hipHostMalloc((void **)&ctx->h_pinned, ctx->pinned_words * 8, hipHostMallocMapped) != hipSuccess) return bail(DPS_ERR_OOM);
    }
    if (hipHostGetDevicePointer((void **)&ctx->d_pinned, ctx->h_pinned, 0) != hipSuccess) return bail(DPS_ERR_HIP);
    memset(ctx->h_pinned, 0, ctx->pinned_words * 8);
    ctx->res_off = ctx->pinned_words - 64;
    // (without this buffer descriptor blocks are uploaded from where they are)
    if (hipHostMalloc((void **)&ctx->h_desc_stage, DESC_STAGE_BYTES, hipHostMallocDefault) != hipSuccess ||
        hipEventCreateWithFlags(&ctx->desc_event, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        if (ctx->h_desc_stage) (void)hipHostFree(ctx->h_desc_stage);
        ctx->h_desc_stage = nullptr;
    }
    // (without this memory the trees' small levels are simply not copied to the host)
    if (hipHostMalloc((void **)&ctx->h_shadow, (size_t)LOGUP_OUT_AREAS * LOGUP_SHADOW_STRIDE * 8, hipHostMallocMapped | hipHostMallocCoherent) != hipSuccess ||
        hipHostGetDevicePointer((void **)&ctx->d_shadow, ctx->h_shadow, 0) != hipSuccess) {
        (void)hipGetLastError();
        if (ctx->h_shadow) (void)hipHostFree(ctx->h_shadow);
        ctx->h_shadow = ctx->d_shadow = nullptr;
    }
    *out = ctx;
    return DPS_OK;
}

extern "C" int32_t dps_ctx_destroy(dps_ctx *ctx)
{
    if (!ctx) return DPS_OK;
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    waiting_launch_over(ctx);
    prof_collect(ctx);
    for (auto e : ctx->ev_pool) (void)hipEventDestroy(e);
    if (ctx->stage_event) (void)hipEventDestroy(ctx->stage_event);
    for (auto &kv : ctx->free_blocks) (void)hipFree(kv.second);
    for (auto &kv : ctx->live_blocks) (void)hipFree(kv.first);
    if (ctx->d_lagrange) (void)hipFree(ctx->d_lagrange);
    if (ctx->h_pinned) (void)hipHostFree(ctx->h_pinned);
    if (ctx->h_shadow) (void)hipHostFree(ctx->h_shadow);
    if (ctx->h_desc_stage) (void)hipHostFree(ctx->h_desc_stage);
    if (ctx->desc_event) (void)hipEventDestroy(ctx->desc_event);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return DPS_OK;
}

extern "C" int32_t dps_device_set_resident_budget(int32_t device, int32_t compute_units)
{
    if (device < 0 || device >= WS_MAX_DEVICES || compute_units < -1) return DPS_ERR_INVALID;
    DeviceLedger &l = ledger_of(device);
    std::lock_guard<std::mutex> lock(l.mu);
    l.limit = compute_units;
    return DPS_OK;
}

extern "C" int32_t dps_device_resident_budget(int32_t device, int32_t *in_use, int32_t *budget)
{
    if (device < 0 || device >= WS_MAX_DEVICES) return DPS_ERR_INVALID;
    DeviceLedger &l = ledger_of(device);
    std::lock_guard<std::mutex> lock(l.mu);
    if (in_use) *in_use = l.used;
    // (before the first context on the device its size is not known: -1)
    if (budget) *budget = l.total < 0 ? -1 : (l.limit >= 0 ? std::min(l.limit, l.total) : l.total);
    return DPS_OK;
}

extern "C" int32_t dps_ctx_sync(dps_ctx *ctx)
{
    if (!ctx) return DPS_ERR_INVALID;
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return DPS_OK;
}

extern "C" int32_t dps_ctx_pool_info(const dps_ctx *ctx, uint64_t *blocks_in_use, uint64_t *blocks_cached, uint64_t *bytes)
{
    if (!ctx) return DPS_ERR_INVALID;
    u64 total = 0;
    for (const auto &kv : ctx->live_blocks) total += kv.second;
    for (const auto &kv : ctx->free_blocks) total += kv.first;
    if (blocks_in_use) *blocks_in_use = ctx->live_blocks.size();
    if (blocks_cached) *blocks_cached = ctx->free_blocks.size();
    if (bytes) *bytes = total;
    return DPS_OK;
}

extern "C" int32_t dps_profile_enable(dps_ctx *ctx, int32_t on)
{
    if (!ctx) return DPS_ERR_INVALID;
    ctx->profiling = on != 0;
    return DPS_OK;
}

extern "C" int32_t dps_profile_reset(dps_ctx *ctx)
{
    if (!ctx) return DPS_ERR_INVALID;
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    prof_collect(ctx);
    for (auto &s : ctx->stats) s = ProfStat();
    return DPS_OK;
}

extern "C" int32_t dps_profile_read(dps_ctx *ctx, int32_t kernel, uint64_t *launches, double *total_ms, double *total_bytes,
                                    uint64_t *max_launches, double *max_ms, double *max_bytes)
{
    if (!ctx || kernel < 0 || kernel >= DPS_K_COUNT) return DPS_ERR_INVALID;
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    prof_collect(ctx);
    const ProfStat &s = ctx->stats[kernel];
    if (launches) *launches = s.launches;
    if (total_ms) *total_ms = s.ms;
    if (total_bytes) *total_bytes = s.bytes;
    if (max_launches) *max_launches = s.max_launches;
    if (max_ms) *max_ms = s.max_ms;
    if (max_bytes) *max_bytes = s.max_bytes;
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// table storage
// ---------------------------------------------------------------------------
extern "C" int32_t dps_mle_from_base(dps_ctx *ctx, const uint64_t *host, uint32_t n_vars, dps_mle **out)
{
    if (!ctx || !host || !out || n_vars > 40) return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_base: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    u64 len = 1ull << n_vars;
    dps_mle *m = nullptr;
    CHK(new_table(ctx, DPS_BASE, len, &m));
    hipError_t e = hipMemcpyAsync(m->st->c0, host, len * 8, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        delete m;
        return fail(ctx, DPS_ERR_HIP, "upload: %s", hipGetErrorString(e));
    }
    *out = m;
    return DPS_OK;
}

extern "C" int32_t dps_mle_from_ext2(dps_ctx *ctx, const uint64_t *c0, const uint64_t *c1, uint32_t n_vars, dps_mle **out)
{
    if (!ctx || !c0 || !c1 || !out || n_vars > 40) return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_ext2: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    u64 len = 1ull << n_vars;
    dps_mle *m = nullptr;
    CHK(new_table(ctx, DPS_EXT2, len, &m));
    hipError_t e = hipMemcpyAsync(m->st->c0, c0, len * 8, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipMemcpyAsync(m->st->c1, c1, len * 8, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        delete m;
        return fail(ctx, DPS_ERR_HIP, "upload: %s", hipGetErrorString(e));
    }
    *out = m;
    return DPS_OK;
}

extern "C" int32_t dps_tensor_from_i64(dps_ctx *ctx, const int64_t *host, uint64_t len, dps_mle **out)
{
    if (!ctx || !out || (len && !host)) return fail(ctx, DPS_ERR_INVALID, "dps_tensor_from_i64: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    dps_mle *m = nullptr;
    CHK(new_table(ctx, DPS_I64, std::max<u64>(len, 1), &m));
    m->len = len;
    if (len) {
        hipError_t e = hipMemcpyAsync(m->st->c0, host, len * 8, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            delete m;
            return fail(ctx, DPS_ERR_HIP, "upload: %s", hipGetErrorString(e));
        }
    }
    *out = m;
    return DPS_OK;
}

extern "C" int32_t dps_tensor_from_i16(dps_ctx *ctx, const int16_t *host, uint64_t len, dps_mle **out)
{
    if (!ctx || !out || (len && !host)) return fail(ctx, DPS_ERR_INVALID, "dps_tensor_from_i16: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    dps_mle *m = nullptr;
    CHK(new_table(ctx, DPS_I16, std::max<u64>(len, 1), &m));
    m->len = len;
    if (len) {
        hipError_t e = hipMemcpyAsync(m->st->c0, host, len * 2, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            delete m;
            return fail(ctx, DPS_ERR_HIP, "upload: %s", hipGetErrorString(e));
        }
    }
    *out = m;
    return DPS_OK;
}

extern "C" int32_t dps_mle_from_i64(dps_ctx *ctx, const int64_t *host, uint64_t len, uint32_t n_vars, dps_mle **out)
{
    if (!ctx || !out || n_vars > 40 || len > (1ull << n_vars) || (len && !host))
        return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_i64: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    dps_mle *raw = nullptr;
    CHK(dps_tensor_from_i64(ctx, host, len, &raw));
    u64 padded = 1ull << n_vars;
    dps_mle *m = nullptr;
    int32_t rc = new_table(ctx, DPS_BASE, padded, &m);
    if (rc != DPS_OK) {
        delete raw;
        return rc;
    }
    dpk::embed_i64_kernel<<<grid_for(padded), dpk::BLOCK, 0, ctx->stream>>>((const int64_t *)raw->st->c0, len, padded, m->st->c0);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    delete raw;
    if (e != hipSuccess) {
        delete m;
        return fail(ctx, DPS_ERR_HIP, "embed: %s", hipGetErrorString(e));
    }
    *out = m;
    return DPS_OK;
}

extern "C" int32_t dps_mle_from_tensor(dps_ctx *ctx, const dps_mle *tensor, const uint64_t *padded_dims, const uint64_t *unpadded_dims,
                                       uint32_t n_dims, dps_mle **out)
{
    if (!ctx || !tensor || !padded_dims || !unpadded_dims || !out || n_dims == 0 || n_dims > dpk::PAD_MAX_DIMS)
        return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_tensor: bad argument");
    if (tensor->ctx != ctx || tensor->kind == DPS_EXT2 || tensor->pad_vars)
        return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_tensor: not a raw or base-field tensor of this context");
    u64 padded_total = 1, unpadded_total = 1;
    for (u32 a = 0; a < n_dims; a++) {
        if (!is_pow2(padded_dims[a]) || unpadded_dims[a] == 0 || unpadded_dims[a] > padded_dims[a] || padded_total > (1ull << 40) / padded_dims[a])
            return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_tensor: axis %u: sizes %llu (padded %llu)", a, (unsigned long long)unpadded_dims[a],
                        (unsigned long long)padded_dims[a]);
        padded_total *= padded_dims[a];
        unpadded_total *= unpadded_dims[a];
    }
    // stored in its padded shape, or compactly in its unpadded shape (told apart by its length)
    const bool compact = tensor->len == unpadded_total && unpadded_total != padded_total;
    if (!compact && tensor->len < padded_total) return fail(ctx, DPS_ERR_INVALID, "dps_mle_from_tensor: tensor shorter than its padded shape");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    dpk::PadTensorArgs a;
    memset(&a, 0, sizeof a);
    a.in = tensor->kind == DPS_I16 ? (const void *)tensor->st->c0 : (const void *)tensor->p0();
    a.in_int = raw_bytes(tensor->kind);
    a.n_dims = n_dims;
    u64 stride = 1;
    for (int d = (int)n_dims - 1; d >= 0; d--) {
        a.padded_dims[d] = padded_dims[d];
        a.unpadded_dims[d] = unpadded_dims[d];
        a.src_strides[d] = stride;
        stride *= compact ? unpadded_dims[d] : padded_dims[d];
    }
    a.total = padded_total;
    dps_mle *m = nullptr;
    CHK(new_table(ctx, DPS_BASE, padded_total, &m));
    a.out = m->st->c0;
    dpk::pad_tensor_kernel<<<grid_for(padded_total), dpk::BLOCK, 0, ctx->stream>>>(a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        delete m;
        return fail(ctx, DPS_ERR_HIP, "pad_tensor launch: %s", hipGetErrorString(e));
    }
    *out = m;
    return DPS_OK;
}

extern "C" int32_t dps_mle_wrap_device(dps_ctx *ctx, int32_t kind, void *d_c0, void *d_c1, uint64_t len, dps_mle **out)
{
    if (!ctx || !out || !d_c0 || kind < DPS_BASE || kind > DPS_I16 || (kind == DPS_EXT2) != (d_c1 != nullptr))
        return fail(ctx, DPS_ERR_INVALID, "dps_mle_wrap_device: bad argument");
    if (((uintptr_t)d_c0 & 15) || ((uintptr_t)d_c1 & 15)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_wrap_device: pointers must be 16-byte aligned");
    auto st = std::make_shared<Storage>();
    st->ctx = ctx;
    st->c0 = (u64 *)d_c0;
    st->c1 = (u64 *)d_c1;
    st->owned = false;
    *out = new (std::nothrow) dps_mle{ctx, st, kind, 0, len, nullptr};
    return *out ? DPS_OK : fail(ctx, DPS_ERR_OOM, "host allocation failed");
}

extern "C" int32_t dps_mle_view(const dps_mle *src, uint64_t offset, uint32_t n_vars, dps_mle **out)
{
    if (!src || !out) return DPS_ERR_INVALID;
    dps_ctx *ctx = src->ctx;
    u64 len = 1ull << n_vars;
    if (src->pad_vars) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_view: the table is a zero-padded view");
    if (src->kind == DPS_I16) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_view: no windows into int16 tensors");
    if (n_vars > 40 || offset > src->len || len > src->len - offset) return fail(ctx, DPS_ERR_INVALID, "dps_mle_view: window outside the table");
    // pair loads are 16 bytes wide
    if (n_vars >= 1 && ((src->offset + offset) & 1)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_view: offset must be even");
    // a window into an eq table shares its level 0 (a window over the whole table stays an eq table, built as its readers ask)
    if (src->eq && !(offset == 0 && len == src->len)) {
        DeviceGuard g(ctx->device);
        tail_abort(ctx);
        CHK(plain_ready(src));
    }
    *out = new (std::nothrow) dps_mle{ctx, src->st, src->kind, src->offset + offset, len, nullptr};
    if (*out && offset == 0 && len == src->len) (*out)->eq = src->eq;
    if (*out && src->sh0) {
        (*out)->sh0 = src->sh0 + offset;
        (*out)->sh1 = src->sh1 + offset;
        (*out)->sh_seq = src->sh_seq, (*out)->sh_build = src->sh_build, (*out)->sh_slot = src->sh_slot;
    }
    return *out ? DPS_OK : fail(ctx, DPS_ERR_OOM, "host allocation failed");
}

extern "C" int32_t dps_mle_zero_pad(const dps_mle *src, uint32_t n_vars, dps_mle **out)
{
    if (!src || !out) return DPS_ERR_INVALID;
    dps_ctx *ctx = src->ctx;
    if (is_raw(src->kind) || !is_pow2(src->len)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_zero_pad: not a power-of-two field table");
    if (n_vars > 40 || (1ull << n_vars) < src->len) return fail(ctx, DPS_ERR_INVALID, "dps_mle_zero_pad: %u variables are fewer than the table has", n_vars);
    if (src->eq) {
        DeviceGuard g(ctx->device);
        tail_abort(ctx);
        CHK(plain_ready(src));
    }
    *out = new (std::nothrow) dps_mle{ctx, src->st, src->kind, src->offset, src->len, nullptr, n_vars};
    return *out ? DPS_OK : fail(ctx, DPS_ERR_OOM, "host allocation failed");
}

extern "C" int32_t dps_mle_info(const dps_mle *mle, int32_t *kind, uint64_t *len)
{
    if (!mle) return DPS_ERR_INVALID;
    if (kind) *kind = mle->kind;
    if (len) *len = mle->len;
    return DPS_OK;
}

extern "C" int32_t dps_mle_download(const dps_mle *mle, uint64_t *c0, uint64_t *c1)
{
    if (!mle || !c0) return DPS_ERR_INVALID;
    dps_ctx *ctx = mle->ctx;
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    CHK(plain_ready(mle));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    if (mle->kind == DPS_I16) {
        // widened on the host: the caller's buffer holds len int64 values like a DPS_I64 tensor's
        std::vector<int16_t> tmp(mle->len);
        if (mle->len) HIPCHK(ctx, hipMemcpy(tmp.data(), mle->st->c0, mle->len * 2, hipMemcpyDeviceToHost));
        for (u64 i = 0; i < mle->len; i++) c0[i] = (u64)(int64_t)tmp[i];
        if (c1) memset(c1, 0, mle->len * 8);
        return DPS_OK;
    }
    if (mle->len) HIPCHK(ctx, hipMemcpy(c0, mle->p0(), mle->len * 8, hipMemcpyDeviceToHost));
    if (c1) {
        if (mle->kind == DPS_EXT2) {
            if (mle->len) HIPCHK(ctx, hipMemcpy(c1, mle->p1(), mle->len * 8, hipMemcpyDeviceToHost));
        } else {
            memset(c1, 0, mle->len * 8);
        }
    }
    return DPS_OK;
}

extern "C" int32_t dps_mle_free(dps_mle *mle)
{
    if (!mle) return DPS_OK;
    // No wait for the stream: when this was the last handle of its storage the block goes back to the context's pool,
    // whose next user runs on the same stream, after whatever is still queued; a session holds on to the storage of its
    // tables by itself.  Memory the caller owns is different: the caller may free or overwrite it once this returns.
    if (mle->st && !mle->st->owned) {
        DeviceGuard g(mle->ctx->device);
        tail_abort(mle->ctx);
        (void)hipStreamSynchronize(mle->ctx->stream);
    }
    delete mle;
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// eq table
// ---------------------------------------------------------------------------
namespace {

bool canonical(const u64 *v, size_t n)
{
    for (size_t i = 0; i < n; i++)
        if (v[i] >= gl::P) return false;
    return true;
}

u64 eq_level_off(u32 m, u32 l) { return (2ull << m) - (2ull << (m - l)); }
// Behind the levels: for every level l = 1..m-16 (those of at least 2^16 entries) the table eq(rho_{l..l+15}, .) of its 16 lowest
// variables.  Level l is then the product  level_{l+16}[i >> 16] * low_l[i & 65535], which the product kernels use in their
// large rounds instead of streaming level l.
u32 eq_fact_levels(u32 m) { return m > dpk::EQ_LO_BITS ? m - dpk::EQ_LO_BITS : 0; }
u32 eq_first_direct(u32 m) { return m > dpk::EQ_DIRECT_BITS ? m - dpk::EQ_DIRECT_BITS : 0; }
u64 eq_low_off(u32 m, u32 l) { return (2ull << m) + ((u64)(l - 1) << dpk::EQ_LO_BITS); }
u64 eq_storage_entries(u32 m) { return (2ull << m) + ((u64)eq_fact_levels(m) << dpk::EQ_LO_BITS); }

// Materialises the levels in `need` (bit l: level l = eq(rho_{l..m-1}, .), 2^(m-l) entries at eq_level_off) that are not
// there yet, and with `need_low` the low tables.  Levels of at most 2^16 entries come straight from the definition, in
// one launch together with the low tables and the 2^8-entry seeds eq(rho_{l..l+7}, .) the larger levels need; a larger
// level l is level l + 8 expanded by seed l (so asking for level 0 of a 24-variable table builds levels 0, 8, 16 only).
int32_t eq_ensure(dps_ctx *ctx, EqInfo &info, u64 *o0, u64 *o1, u64 need, bool need_low)
{
    const u32 m = info.m;
    const u32 first_small = eq_first_direct(m);  // levels first_small..m come straight from the definition
    need &= (2ull << m) - 1;
    u64 todo = need & ~info.built;
    // a large level needs level l + 8
    for (u32 l = 0; l < first_small; l++)
        if (((todo >> l) & 1) && !((info.built >> (l + 8)) & 1)) todo |= 1ull << (l + 8);
    const bool low = need_low && info.fact_levels && !info.fact_built;
    if (!todo && !low) return DPS_OK;
    std::vector<dpk::EqJob> jobs;
    u32 n_large = 0;
    for (u32 l = first_small; l <= m; l++)
        if ((todo >> l) & 1) jobs.push_back(dpk::EqJob{l, m - l, eq_level_off(m, l)});
    if (low)
        for (u32 l = 1; l <= info.fact_levels; l++) jobs.push_back(dpk::EqJob{l, dpk::EQ_LO_BITS, eq_low_off(m, l)});
    for (u32 l = 0; l < first_small; l++)
        if ((todo >> l) & 1) n_large++;
    // seeds live in a scratch block of their own, read by the expansions queued right behind
    void *seed_block = nullptr;
    u64 *seed0 = nullptr, *seed1 = nullptr;
    if (n_large) {
        CHK(pool_alloc(ctx, (size_t)first_small * 256 * 16, &seed_block));
        seed0 = (u64 *)seed_block;
        seed1 = seed0 + (size_t)first_small * 256;
    }
    // the seeds of the large levels to build, in the same launch
    for (u32 l = 0; l < first_small; l++)
        if ((todo >> l) & 1) jobs.push_back(dpk::EqJob{l, 8, ((u64)l * 256) | dpk::EQ_JOB_SECOND});
    int32_t rc = DPS_OK;
    auto run_jobs = [&](const std::vector<dpk::EqJob> &js_in, u64 *d0, u64 *d1) {
        for (size_t base = 0; base < js_in.size() && rc == DPS_OK; base += dpk::EQ_MAX_JOBS) {
            dpk::EqJobs js;
            memset(&js, 0, sizeof js);
            for (u32 i = 0; i < m; i++) {
                js.point[2 * i] = info.point[i].c0;
                js.point[2 * i + 1] = info.point[i].c1;
            }
            js.o0 = d0;
            js.o1 = d1;
            js.s0 = seed0;
            js.s1 = seed1;
            const u32 n = (u32)std::min<size_t>(js_in.size() - base, dpk::EQ_MAX_JOBS);
            u32 max_bits = 0;
            double entries = 0;
            for (u32 k = 0; k < n; k++) {
                js.job[k] = js_in[base + k];
                max_bits = std::max(max_bits, js.job[k].n_bits);
                entries += (double)(1ull << js.job[k].n_bits);
            }
            ProfScope ps(ctx, DPS_K_EQ, entries * 16.0);
            // up to 128 workgroups share a job's rows of 256 entries (4 rows each in the largest job)
            const u32 rows = max_bits > 8 ? 1u << (max_bits - 8) : 1;
            dpk::eq_define_kernel<<<dim3(std::min<u32>(rows, 128), n), dpk::BLOCK, 0, ctx->stream>>>(js);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "eq_define launch: %s", hipGetErrorString(e));
        }
    };
    run_jobs(jobs, o0, o1);
    if (n_large && rc == DPS_OK) {
        // highest level first: level l reads level l + 8
        for (u32 l = first_small; l-- > 0 && rc == DPS_OK;) {
            if (!((todo >> l) & 1)) continue;
            const u64 n_hi = 1ull << (m - l - 8);
            const u64 hi_off = eq_level_off(m, l + 8), out_off = eq_level_off(m, l);
            u32 blocks = (u32)std::min<u64>(n_hi, MAX_BLOCKS * 4);
            u32 per_block = (u32)((n_hi + blocks - 1) / blocks);
            blocks = (u32)((n_hi + per_block - 1) / per_block);
            ProfScope ps(ctx, DPS_K_EQ, (double)(n_hi << 8) * 16 + (double)n_hi * 16);
            dpk::eq_expand_kernel<<<blocks, dpk::BLOCK, 0, ctx->stream>>>(o0 + hi_off, o1 + hi_off, n_hi, seed0 + (size_t)l * 256, seed1 + (size_t)l * 256, 8,
                                                                         o0 + out_off, o1 + out_off, per_block);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "eq_expand launch: %s", hipGetErrorString(e));
        }
    }
    // stream order makes the block reusable by later launches on this stream
    pool_free(ctx, seed_block);
    if (rc == DPS_OK) {
        info.built |= todo;
        if (low) info.fact_built = true;
    }
    return rc;
}

// a table about to be read as ordinary entries: if it is an eq table, its level 0 has to be there
int32_t plain_ready(const dps_mle *t)
{
    if (!t || !t->eq || (t->eq->built & 1)) return DPS_OK;
    return eq_ensure(t->ctx, *t->eq, t->st->c0, t->st->c1, 1, false);
}

}  // namespace

extern "C" int32_t dps_eq_build(dps_ctx *ctx, const uint64_t *point, uint32_t m, dps_mle **out)
{
    if (!ctx || !out || (m && !point) || m > dpk::EQ_MAX_VARS) return fail(ctx, DPS_ERR_INVALID, "dps_eq_build: bad argument");
    if (!canonical(point, 2 * (size_t)m)) return fail(ctx, DPS_ERR_INVALID, "dps_eq_build: point not canonical");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    dps_mle *t = nullptr;
    CHK(new_table(ctx, DPS_EXT2, eq_storage_entries(m), &t));
    t->len = 1ull << m;
    t->eq = std::make_shared<EqInfo>();
    t->eq->m = m;
    t->eq->fact_levels = eq_fact_levels(m);
    for (u32 i = 0; i < m; i++) t->eq->point.push_back(gl::e2(point[2 * i], point[2 * i + 1]));
    // Up to 17 variables everything comes out of one launch.  Of a larger table only the levels of at most 2^17 entries
    // and the low tables are built now, in that one launch (what a product session reads, 13 MB at 24 variables); the
    // large levels wait for whoever reads them.
    // (nothing at all of a table so small that the sums over it may be the host's, which reads the point: then whoever
    // reads entries builds them)
    const u64 small = m <= HOST_ONLY_MAX_VARS ? 0 : ((2ull << m) - 1) & ~((1ull << eq_first_direct(m)) - 1);
    int32_t rc = eq_ensure(ctx, *t->eq, t->st->c0, t->st->c1, small, true);
    if (rc != DPS_OK) {
        delete t;
        return rc;
    }
    *out = t;
    return DPS_OK;
}

extern "C" int32_t dps_eq_build_many(dps_ctx *ctx, const uint64_t *const *points, const uint32_t *m, uint32_t count, dps_mle **out)
{
    if (!ctx || !out || (count && (!points || !m))) return fail(ctx, DPS_ERR_INVALID, "dps_eq_build_many: bad argument");
    for (u32 i = 0; i < count; i++) {
        out[i] = nullptr;
        if ((m[i] && !points[i]) || m[i] > dpk::EQ_MAX_VARS) return fail(ctx, DPS_ERR_INVALID, "dps_eq_build_many: bad argument (table %u)", i);
        if (!canonical(points[i], 2 * (size_t)m[i])) return fail(ctx, DPS_ERR_INVALID, "dps_eq_build_many: point %u not canonical", i);
    }
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    auto undo = [&](int32_t rc) {
        for (u32 i = 0; i < count; i++) {
            delete out[i];
            out[i] = nullptr;
        }
        return rc;
    };
    // staging region of the pinned buffer: job descriptors, then the points
    const size_t stage_lo = 1024, stage_hi = ctx->pinned_words / 2;
    std::vector<dpk::EqJobM> jobs;
    std::vector<u64> pts;
    u32 max_bits = 0;
    auto flush = [&]() -> int32_t {
        if (jobs.empty()) return DPS_OK;
        // the previous launch that read the region must be done with it
        if (ctx->stage_pending) {
            HIPCHK(ctx, hipEventSynchronize(ctx->stage_event));
            ctx->stage_pending = false;
        }
        const size_t job_words = jobs.size() * sizeof(dpk::EqJobM) / 8;
        memcpy(ctx->h_pinned + stage_lo, jobs.data(), job_words * 8);
        memcpy(ctx->h_pinned + stage_lo + job_words, pts.data(), pts.size() * 8);
        ProfScope ps(ctx, DPS_K_EQ, 0.0);
        dpk::eq_define_many_kernel<<<dim3((u32)(((1ull << max_bits) + dpk::BLOCK - 1) / dpk::BLOCK), (u32)jobs.size()), dpk::BLOCK, 0, ctx->stream>>>(
            reinterpret_cast<const dpk::EqJobM *>(ctx->d_pinned + stage_lo), ctx->d_pinned + stage_lo + job_words);
        HIPCHK(ctx, hipGetLastError());
        HIPCHK(ctx, hipEventRecord(ctx->stage_event, ctx->stream));
        ctx->stage_pending = true;
        jobs.clear();
        pts.clear();
        max_bits = 0;
        return DPS_OK;
    };
    for (u32 i = 0; i < count; i++) {
        dps_mle *t = nullptr;
        int32_t rc = new_table(ctx, DPS_EXT2, eq_storage_entries(m[i]), &t);
        if (rc != DPS_OK) return undo(rc);
        out[i] = t;
        t->len = 1ull << m[i];
        t->eq = std::make_shared<EqInfo>();
        t->eq->m = m[i];
        t->eq->fact_levels = eq_fact_levels(m[i]);  // (only tables of more than 16 variables have any: built by eq_build_dev)
        for (u32 k = 0; k < m[i]; k++) t->eq->point.push_back(gl::e2(points[i][2 * k], points[i][2 * k + 1]));
        if (m[i] > 16) {
            // large tables are built by expansion, one at a time
            const u64 small = ((2ull << m[i]) - 1) & ~((1ull << eq_first_direct(m[i])) - 1);
            rc = eq_ensure(ctx, *t->eq, t->st->c0, t->st->c1, small, true);
            if (rc != DPS_OK) return undo(rc);
            continue;
        }
        t->eq->built = (2ull << m[i]) - 1;  // every level, by the launch below
        const size_t need = ((jobs.size() + m[i] + 1) * sizeof(dpk::EqJobM)) / 8 + pts.size() + 2 * (size_t)m[i];
        if (stage_lo + need > stage_hi || jobs.size() + m[i] + 1 > 65535) {
            rc = flush();
            if (rc != DPS_OK) return undo(rc);
        }
        // every level eq(rho_{l..m-1}, .), l = 0..m, straight from the definition
        const u32 point_off = (u32)pts.size();
        pts.insert(pts.end(), points[i], points[i] + 2 * (size_t)m[i]);
        for (u32 l = 0; l <= m[i]; l++) {
            const u64 off = eq_level_off(m[i], l);
            jobs.push_back(dpk::EqJobM{t->st->c0 + off, t->st->c1 + off, l, m[i] - l, point_off, 0});
            max_bits = std::max(max_bits, m[i] - l);
        }
    }
    // the point offsets are relative to the start of the points, which follow the jobs of the same launch
    int32_t rc = flush();
    if (rc != DPS_OK) return undo(rc);
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// contraction of one axis (partial evaluation, evaluate, fix_high)
// ---------------------------------------------------------------------------
namespace {

struct AxisJob {
    const u64 *in0 = nullptr, *in1 = nullptr;
    int in_int = 0;  // bytes per raw integer entry, 0 for field elements
    const u64 *b0 = nullptr, *b1 = nullptr;
    u64 K = 1, stride_k = 1;
    std::vector<u64> pre_dims, pre_strides, post_dims, post_strides;
    u64 *o0 = nullptr, *o1 = nullptr;
};

int32_t axis_dot(dps_ctx *ctx, const AxisJob &j)
{
    dpk::AxisArgs a;
    memset(&a, 0, sizeof a);
    if (j.pre_dims.size() > dpk::AX_MAX_DIMS || j.post_dims.size() > dpk::AX_MAX_DIMS)
        return fail(ctx, DPS_ERR_UNSUPPORTED, "tensor rank above %d", dpk::AX_MAX_DIMS);
    a.in0 = j.in0;
    a.in1 = j.in1;
    a.in_int = j.in_int;
    a.b0 = j.b0;
    a.b1 = j.b1;
    a.K = j.K;
    a.stride_k = j.stride_k;
    a.n_pre = (u32)j.pre_dims.size();
    a.n_post = (u32)j.post_dims.size();
    a.P = a.C = 1;
    for (u32 d = 0; d < a.n_pre; d++) {
        a.pre_dims[d] = j.pre_dims[d];
        a.pre_strides[d] = j.pre_strides[d];
        a.P *= j.pre_dims[d];
    }
    for (u32 d = 0; d < a.n_post; d++) {
        a.post_dims[d] = j.post_dims[d];
        a.post_strides[d] = j.post_strides[d];
        a.C *= j.post_dims[d];
    }
    const u64 outputs = a.P * a.C;
    if (outputs == 0 || a.K == 0) return fail(ctx, DPS_ERR_INVALID, "empty axis contraction");
    const bool col = a.C >= 32;
    // split k over workgroups when there are too few outputs to fill the chip
    const u64 out_blocks = col ? a.P * ((a.C + dpk::WAVE - 1) / dpk::WAVE) : outputs;
    // k values one workgroup should at least own (two trips of four per wavefront, or one per lane); a few thousand workgroups
    // keep enough loads in flight to hide the latency of a launch that is a few megabytes in all
    const u64 k_unit = col ? 32 : 1024;
    u32 n_slices = 1;
    if (out_blocks < 2048 && a.K > k_unit) n_slices = (u32)std::min<u64>((a.K + k_unit - 1) / k_unit, std::max<u64>(1, 4096 / out_blocks));
    if (n_slices > 65535) n_slices = 65535;
    a.k_per_slice = (a.K + n_slices - 1) / n_slices;
    n_slices = (u32)((a.K + a.k_per_slice - 1) / a.k_per_slice);
    a.n_slices = n_slices;
    if (out_blocks > 0x7fffffffull) return fail(ctx, DPS_ERR_UNSUPPORTED, "axis contraction too large");
    void *tmp = nullptr;
    if (n_slices > 1) {
        CHK(pool_alloc(ctx, (size_t)n_slices * outputs * 16, &tmp));
        a.o0 = (u64 *)tmp;
        a.o1 = a.o0 + (size_t)n_slices * outputs;
    } else {
        a.o0 = j.o0;
        a.o1 = j.o1;
    }
    const double elem = j.in1 ? 16.0 : 8.0;
    hipError_t e;
    {
        ProfScope ps(ctx, DPS_K_AXIS_DOT, (double)outputs * (double)a.K * elem + (double)outputs * 16.0);
        if (col)
            dpk::axis_dot_col_kernel<<<dim3((u32)out_blocks, n_slices), dpk::BLOCK, 0, ctx->stream>>>(a);
        else
            dpk::axis_dot_row_kernel<<<dim3((u32)out_blocks, n_slices), dpk::BLOCK, 0, ctx->stream>>>(a);
        e = hipGetLastError();
    }
    if (e == hipSuccess && n_slices > 1) {
        dpk::slice_sum_kernel<<<(u32)((outputs + dpk::BLOCK - 1) / dpk::BLOCK), dpk::BLOCK, 0, ctx->stream>>>(
            a.o0, a.o1, outputs, n_slices, j.o0, j.o1);
        e = hipGetLastError();
    }
    pool_free(ctx, tmp);
    if (e != hipSuccess) return fail(ctx, DPS_ERR_HIP, "axis_dot launch: %s", hipGetErrorString(e));
    return DPS_OK;
}

}  // namespace

extern "C" int32_t dps_mle_evaluate(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point, uint32_t n, uint64_t out[2])
{
    if (!ctx || !mle || !out || (n && !point)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate: bad argument");
    if (mle->pad_vars) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_evaluate: the table is a zero-padded view");
    if (!is_pow2(mle->len) || (1ull << n) != mle->len) return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate: point length does not match the table");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    CHK(plain_ready(mle));
    dps_mle *eq = nullptr;
    CHK(dps_eq_build(ctx, point, n, &eq));
    if (int32_t rc_ = plain_ready(eq); rc_ != DPS_OK) {
        delete eq;
        return rc_;
    }
    AxisJob j;
    j.in0 = mle->p0();
    j.in1 = mle->p1();
    j.in_int = raw_bytes(mle->kind);
    j.b0 = eq->p0();
    j.b1 = eq->p1();
    j.K = mle->len;
    j.stride_k = 1;
    // the result lands in the second half of the pinned buffer (the first half staged the point)
    j.o0 = ctx->d_pinned + ctx->pinned_words / 2;
    j.o1 = j.o0 + 1;
    int32_t rc = axis_dot(ctx, j);
    hipError_t e = hipStreamSynchronize(ctx->stream);
    delete eq;
    if (rc != DPS_OK) return rc;
    if (e != hipSuccess) return fail(ctx, DPS_ERR_HIP, "evaluate: %s", hipGetErrorString(e));
    out[0] = ctx->h_pinned[ctx->pinned_words / 2];
    out[1] = ctx->h_pinned[ctx->pinned_words / 2 + 1];
    return DPS_OK;
}

extern "C" int32_t dps_mle_fix_high(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point, uint32_t k, dps_mle **out)
{
    if (!ctx || !mle || !out || (k && !point)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_fix_high: bad argument");
    if (mle->pad_vars) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_fix_high: the table is a zero-padded view");
    if (!is_pow2(mle->len) || (1ull << k) > mle->len) return fail(ctx, DPS_ERR_INVALID, "dps_mle_fix_high: too many variables");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    CHK(plain_ready(mle));
    dps_mle *eq = nullptr;
    CHK(dps_eq_build(ctx, point, k, &eq));
    if (int32_t rc_ = plain_ready(eq); rc_ != DPS_OK) {
        delete eq;
        return rc_;
    }
    u64 rest = mle->len >> k;
    dps_mle *res = nullptr;
    int32_t rc = new_table(ctx, DPS_EXT2, rest, &res);
    if (rc == DPS_OK) {
        AxisJob j;
        j.in0 = mle->p0();
        j.in1 = mle->p1();
        j.in_int = raw_bytes(mle->kind);
        j.b0 = eq->p0();
        j.b1 = eq->p1();
        j.K = 1ull << k;
        j.stride_k = rest;
        j.post_dims = {rest};
        j.post_strides = {1};
        j.o0 = res->st->c0;
        j.o1 = res->st->c1;
        rc = axis_dot(ctx, j);
    }
    hipError_t e = hipStreamSynchronize(ctx->stream);
    delete eq;
    if (rc == DPS_OK && e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "fix_high: %s", hipGetErrorString(e));
    if (rc != DPS_OK) {
        delete res;
        return rc;
    }
    *out = res;
    return DPS_OK;
}

extern "C" int32_t dps_mle_fix_low(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point, uint32_t k, dps_mle **out)
{
    if (!ctx || !mle || !out || (k && !point)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_fix_low: bad argument");
    if (mle->pad_vars) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_fix_low: the table is a zero-padded view");
    if (!is_pow2(mle->len) || (1ull << k) > mle->len || is_raw(mle->kind))
        return fail(ctx, DPS_ERR_INVALID, "dps_mle_fix_low: needs a power-of-two field table and k <= log2(len)");
    if (!canonical(point, 2 * (size_t)k)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_fix_low: point not canonical");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    CHK(plain_ready(mle));
    if (k == 0) return dps_mle_view(mle, 0, log2u(mle->len), out);
    // ping-pong between two buffers; the last one written becomes the result
    u64 len = mle->len;
    dps_mle *bufs[2] = {nullptr, nullptr};
    CHK(new_table(ctx, DPS_EXT2, len >> 1, &bufs[0]));
    if (k > 1) {
        int32_t rc = new_table(ctx, DPS_EXT2, len >> 2, &bufs[1]);
        if (rc != DPS_OK) {
            delete bufs[0];
            return rc;
        }
    }
    const u64 *s0 = mle->p0(), *s1 = mle->p1();
    int32_t rc = DPS_OK;
    int w = 0;
    for (u32 j = 0; j < k && rc == DPS_OK; j++) {
        len >>= 1;
        dpk::FoldDesc d{s0, s1, bufs[w]->st->c0, bufs[w]->st->c1, len};
        ProfScope ps(ctx, DPS_K_FOLD, (double)len * (s1 ? 32.0 : 16.0) + (double)len * 16.0);
        dpk::fold_one_kernel<<<grid_for(len), dpk::BLOCK, 0, ctx->stream>>>(d, point[2 * j], point[2 * j + 1]);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "fold launch: %s", hipGetErrorString(e));
        s0 = bufs[w]->st->c0;
        s1 = bufs[w]->st->c1;
        w ^= 1;
    }
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (rc == DPS_OK && e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "fix_low: %s", hipGetErrorString(e));
    dps_mle *res = bufs[w ^ 1], *other = bufs[w];
    delete other;
    if (rc != DPS_OK) {
        delete res;
        return rc;
    }
    res->len = len;
    *out = res;
    return DPS_OK;
}

namespace {

// The last step of a partial evaluation: what is left of the tensor is indexed by the stacked and contracted axes in
// their original order; like the reference (axis.rs:1222-1233) the flat result is cut into chunks of `contraction`
// entries, one table per chunk, each padded to a power of two.  `cur`: the result of the contractions so far (owned
// here), or nullptr when no outer axis was fixed (the source is then read through `dims` / `strides`).
int32_t rows_as_tables(dps_ctx *ctx, dps_mle *cur, const u64 *in0, const u64 *in1, int in_int, const std::vector<u64> &dims,
                       const std::vector<u64> &strides, u64 stacked, u64 contraction, dps_mle **out)
{
    int32_t rc = DPS_OK;
    u32 nv = log2u(contraction);
    u64 tl = 1ull << nv;
    dps_mle *all = nullptr;
    // rows that are a power of two long already: the result is the table as it stands
    const bool as_it_stands = cur && contraction == tl && cur->kind == DPS_EXT2 && cur->offset == 0 && cur->len == stacked * tl;
    if (as_it_stands) {
        all = cur;
        cur = nullptr;
    } else {
        rc = new_table(ctx, DPS_EXT2, stacked * tl, &all);
    }
    if (rc == DPS_OK && !as_it_stands) {
        if (cur) {
            dpk::pad_rows_kernel<<<grid_for(stacked * tl), dpk::BLOCK, 0, ctx->stream>>>(cur->st->c0, cur->st->c1, stacked, contraction, tl,
                                                                                    all->st->c0, all->st->c1);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "pad launch: %s", hipGetErrorString(e));
        } else {
            // no outer axis: contract a unit axis with the table {1} to copy the unpadded region
            u64 one[2] = {0, 0};
            dps_mle *unit = nullptr;
            rc = dps_eq_build(ctx, one, 0, &unit);
            if (rc == DPS_OK) rc = plain_ready(unit);
            dps_mle *flat = nullptr;
            if (rc == DPS_OK) rc = new_table(ctx, DPS_EXT2, stacked * contraction, &flat);
            if (rc == DPS_OK) {
                AxisJob j;
                j.in0 = in0;
                j.in1 = in1;
                j.in_int = in_int;
                j.b0 = unit->p0();
                j.b1 = unit->p1();
                j.K = 1;
                j.stride_k = 0;
                j.post_dims = dims;
                j.post_strides = strides;
                j.o0 = flat->st->c0;
                j.o1 = flat->st->c1;
                rc = axis_dot(ctx, j);
            }
            if (rc == DPS_OK) {
                dpk::pad_rows_kernel<<<grid_for(stacked * tl), dpk::BLOCK, 0, ctx->stream>>>(flat->st->c0, flat->st->c1, stacked, contraction,
                                                                                        tl, all->st->c0, all->st->c1);
                hipError_t e = hipGetLastError();
                if (e != hipSuccess) rc = fail(ctx, DPS_ERR_HIP, "pad launch: %s", hipGetErrorString(e));
            }
            (void)hipStreamSynchronize(ctx->stream);
            delete unit;
            delete flat;
        }
    }
    // (no wait for the stream: the blocks given back are reused in stream order, and whoever consumes the result waits)
    delete cur;
    if (rc != DPS_OK) {
        delete all;
        return rc;
    }
    for (u64 s = 0; s < stacked; s++) {
        rc = dps_mle_view(all, s * tl, nv, &out[s]);
        if (rc != DPS_OK) {
            for (u64 q = 0; q < s; q++) delete out[q];
            delete all;
            return rc;
        }
    }
    delete all;  // the views keep the storage alive
    return DPS_OK;
}

}  // namespace

extern "C" int32_t dps_partial_eval(dps_ctx *ctx, const dps_mle *tensor, const uint64_t *padded_dims,
                                    const uint64_t *unpadded_dims, uint32_t n_dims, const int32_t *kinds,
                                    const uint64_t *const *points, dps_mle **out, uint32_t out_cap, uint32_t *n_out)
{
    if (!ctx || !tensor || !padded_dims || !unpadded_dims || !kinds || !out || !n_out || n_dims == 0 || n_dims > dpk::AX_MAX_DIMS)
        return fail(ctx, DPS_ERR_INVALID, "dps_partial_eval: bad argument");
    if (tensor->pad_vars) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_partial_eval: the tensor is a zero-padded view");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    CHK(plain_ready(tensor));
    u64 padded_total = 1, contraction = 1, stacked = 1;
    for (u32 a = 0; a < n_dims; a++) {
        if (unpadded_dims[a] == 0 || unpadded_dims[a] > padded_dims[a]) return fail(ctx, DPS_ERR_INVALID, "dps_partial_eval: dimension %u", a);
        if (kinds[a] < 0 || kinds[a] > 2) return fail(ctx, DPS_ERR_INVALID, "dps_partial_eval: axis kind %u", a);
        if (kinds[a] == DPS_AXIS_OUTER && (!points || !points[a] || !is_pow2(padded_dims[a])))
            return fail(ctx, DPS_ERR_INVALID, "dps_partial_eval: outer axis %u needs a point and a power-of-two padded size", a);
        padded_total *= padded_dims[a];
        if (kinds[a] == DPS_AXIS_CONTRACTED) contraction *= unpadded_dims[a];
        if (kinds[a] == DPS_AXIS_STACKED) stacked *= unpadded_dims[a];
    }
    // the tensor is stored in its padded shape, or compactly in its unpadded shape (told apart by its length)
    u64 unpadded_total = 1;
    for (u32 a = 0; a < n_dims; a++) unpadded_total *= unpadded_dims[a];
    const bool compact = tensor->len == unpadded_total && unpadded_total != padded_total;
    if (!compact && padded_total > tensor->len) return fail(ctx, DPS_ERR_INVALID, "dps_partial_eval: tensor shorter than its padded shape");
    if (stacked > out_cap) return fail(ctx, DPS_ERR_INVALID, "dps_partial_eval: %llu tables do not fit out_cap", (unsigned long long)stacked);

    // current tensor: dims (unpadded sizes of the axes still present) and element strides
    std::vector<u64> dims(unpadded_dims, unpadded_dims + n_dims), strides(n_dims);
    std::vector<int32_t> kd(kinds, kinds + n_dims);
    std::vector<u32> orig(n_dims);
    {
        u64 s = 1;
        for (int a = (int)n_dims - 1; a >= 0; a--) {
            strides[a] = s;
            s *= compact ? unpadded_dims[a] : padded_dims[a];
            orig[a] = a;
        }
    }
    const u64 *in0 = tensor->p0(), *in1 = tensor->p1();
    int in_int = raw_bytes(tensor->kind);
    dps_mle *cur = nullptr;  // owns the intermediate
    int32_t rc = DPS_OK;
    // the reference walks the axes from the last to the first (axis.rs:1152)
    for (int a = (int)dims.size() - 1; a >= 0 && rc == DPS_OK; a--) {
        if (kd[a] != DPS_AXIS_OUTER) continue;
        u32 oa = orig[a];
        u32 m = log2u(padded_dims[oa]);
        dps_mle *beta = nullptr;
        rc = dps_eq_build(ctx, points[oa], m, &beta);
        if (rc == DPS_OK) rc = plain_ready(beta);
        if (rc != DPS_OK) {
            delete beta;
            break;
        }
        AxisJob j;
        j.in0 = in0;
        j.in1 = in1;
        j.in_int = in_int;
        j.b0 = beta->p0();
        j.b1 = beta->p1();
        j.K = dims[a];  // evals(point)[..size]
        j.stride_k = strides[a];
        u64 outputs = 1;
        for (int d = 0; d < (int)dims.size(); d++) {
            if (d == a) continue;
            (d < a ? j.pre_dims : j.post_dims).push_back(dims[d]);
            (d < a ? j.pre_strides : j.post_strides).push_back(strides[d]);
            outputs *= dims[d];
        }
        dps_mle *next = nullptr;
        rc = new_table(ctx, DPS_EXT2, outputs, &next);
        if (rc == DPS_OK) {
            j.o0 = next->st->c0;
            j.o1 = next->st->c1;
            rc = axis_dot(ctx, j);
        }
        delete beta;
        delete cur;
        cur = next;
        if (rc != DPS_OK) break;
        // the result is compact over the remaining axes
        dims.erase(dims.begin() + a);
        kd.erase(kd.begin() + a);
        orig.erase(orig.begin() + a);
        strides.assign(dims.size(), 1);
        for (int d = (int)dims.size() - 2; d >= 0; d--) strides[d] = strides[d + 1] * dims[d + 1];
        in0 = cur->st->c0;
        in1 = cur->st->c1;
        in_int = 0;
    }
    if (rc != DPS_OK) {
        delete cur;
        return rc;
    }
    CHK(rows_as_tables(ctx, cur, in0, in1, in_int, dims, strides, stacked, contraction, out));
    *n_out = (u32)stacked;
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// sumcheck session
// ---------------------------------------------------------------------------
namespace {

struct SessMle {
    const u64 *c0, *c1;  // current table
    u32 nv;              // current number of variables
    u64 *buf0[2], *buf1[2];  // ping-pong scratch, extension limbs
    int next;
    bool zpad;  // fewer variables than the sum and zero-padded: depends on the low variables, 0 where a higher one is 1
};

}  // namespace

struct dps_sc {
    dps_ctx *ctx;
    u32 n_vars, n_mles, n_terms, degree;
    u32 round;  // rounds completed
    bool finished;
    std::vector<SessMle> m;
    std::vector<std::shared_ptr<Storage>> keep;  // borrowed tables stay alive
    std::vector<dps_term> terms;                 // non-constant terms
    E2 const_sum;                                // sum of the constant terms
    // fast path: one term of distinct full-size tables, at most one of them an eq table
    bool fast;
    u32 fast_nf;        // streamed tables (the eq factor not counted)
    u32 fast_order[3];  // streamed factors sorted base-first
    int fast_eq;        // index of the eq table handled in closed form, or -1
    std::shared_ptr<EqInfo> eq_info;
    const u64 *eq_c0, *eq_c1;  // its storage (level 0 at entry 0)
    E2 fast_coeff;
    E2 eq_scalar;       // product of eq1(rho_i, r_{i+1}) over the bound variables
    E2 claim;           // p(0) + p(1) expected from the next message (valid from round 2; from round 1 with dps_sc_set_claim)
    bool have_claim;    // the caller said what the whole sum is
    std::vector<E2> last_msg;
    bool broken;        // its tail kernel was interrupted by another call on the context
    // Resident rounds of a product session (slice_kernel): from round tail_j0 on the tables live in LDS, in one launch of
    // one workgroup, or a launch of several followed by one of one.  A trip to the GPU covers one round or two.
    struct Stage {
        u32 W, j0, pend0, n_trips, dbl_mask, cap;
        u64 src_len;
        u64 *h0[dpk::SL_MAX_TABS + 1], *h1[dpk::SL_MAX_TABS + 1];  // where a stage that is not the last leaves its entries (the next stage's source)
    };
    std::vector<Stage> stages;
    std::vector<u32> slice_ids;                // the tables of the resident launches (session indices), in slot order
    std::vector<dpk::SliceTerm> slice_terms;   // sums of several terms: the terms, their tables as slots of slice_ids
    std::vector<uint8_t> round_kind;  // per round (1-based): 0 a launch of its own, 1 starts a trip, 2 starts a trip of two rounds, 3 second round of a trip,
                                      // 4 worked out on the host
    std::vector<uint8_t> round_wide;  // per round: its trip is made by several workgroups (whose counters run on from trip to trip): the sets of counters they add into
    u64 ctr_seen[dpk::SL_MAX_GROUPS * dpk::SL_GROUP_WORDS];  // ... what those counters held after the trip before
    E2 prev_chal;                     // the challenge of the call before this one
    bool pair12;                      // rounds 1 and 2 are one launch that writes nothing (pair12_kernel); round 3 folds twice on its way in
    // Launches that cover two rounds each behind that one (quad_kernel): launch k takes rounds quad_j0 + 2 k and + 1, reading
    // the state of two rounds before its first (the unfolded tables for the first launch, then what the launch before wrote)
    struct QuadStep {
        u32 j, blocks;
        const u64 *s0[2], *s1[2];
        u64 *d0[2], *d1[2];
    };
    std::vector<QuadStep> quads;      // in round order; round_kind 5 at a launch's first round, 6 at its second
    bool fast_all_base;               // every streamed table of the product is a base-field table as registered
    E2 stash[dpk::SL_MAX_SUMS];       // a trip of two rounds: the second round's sums as a polynomial in the first round's challenge
    u64 last_trip_seq;
    u32 fin_len;                      // entries per table the last trip leaves to the host: the state of its first round
    u32 fin_pend;                     // ... and the folds that state is still owed (the rounds of that trip)
    u32 host_rounds;                  // the last rounds are worked out on the host from those entries (round_kind 4)
    bool host_only = false;           // every round is: the tables were small levels of fraction trees, which the host has copies of
    std::vector<E2> host_state;       // the tables of the round in hand there, table by table
    u32 host_len;                     // entries per table in host_state (0: not taken over yet)
    bool host_fresh;                  // ... as the launch left them: the folds of its last trip are still owed
    u32 tail_j0;        // first resident round, 0 = none
    bool tail_running;
    u64 tail_seq0;
    void *scratch;      // one pool block holding every ping-pong buffer
    void *dev_block;    // descriptors, partials, per-round result
    // precomputed descriptors (device)
    std::vector<u32> fold_off, fold_cnt;            // per step j = 2..n_vars+1: all tables that fold
    std::vector<u32> fold_extra_off, fold_extra_cnt;  // same, without the fast term's tables
    std::vector<u32> term_off;                      // per round j = 1..n_vars
    dpk::FoldDesc *d_fold;
    dpk::FoldDesc *d_fold_extra;
    dpk::TermDesc *d_terms;
    dpk::FinTerm *d_fin;
    dpk::GatherDesc *d_gather;
    u64 *d_partial;
    u64 *d_result;
    u32 *d_counter;  // ticket counter of the evaluation launches, zero between rounds
    std::vector<dpk::ProdArgs> fast_args;  // per round
    std::vector<u32> fast_nb;              // base-field sources per round
    u32 max_blocks;
    // fused multi-term path: groups of at most POLY_MAXT tables, one grid row each
    bool poly;
    std::vector<std::vector<u32>> poly_tabs;  // per group: session table indices, in slot order
    std::vector<u32> poly_op_begin, poly_op_end;  // per group: its nested program in h_poly_ops
    std::vector<u32> poly_term_begin, poly_term_end;
    std::vector<int> poly_owner;              // per session table: the group that writes its fold, -1 = in no group
    u32 poly_max_tabs;                        // sizes the kernel's LDS
    u32 poly_split_cap;                       // log2 of the most lanes a pair's work is worth spreading over
    bool descs_uploaded;                      // the descriptor block is on the device (uploaded when first needed)
    bool poly_raw;                            // the resident launch has one workgroup per group; the host adds their sums
    bool wait_stays;                          // the launch waiting for mail stays for the rounds after the one it waits for
    bool wait_skip1;                          // ... and was compiled to take p(1) from the claim
    bool wait_any_skip1;                      // ... or takes p(1) either way (the tail kernel)
    bool wait_fresh;                          // ... and has not been sent a mail yet (ending it loses nothing)
    u32 wait_slots;                           // ... and publishes to this many result areas of its own (0: the main one)
    u64 pairs_seq;                            // nonzero: the last round's launch also published the tables' last pairs, under this number
    bool no_ahead;                            // a launch made ahead was in another call's way once: make no more
    std::chrono::steady_clock::time_point ahead_at;  // when the launch that has had no mail yet was made
    bool poly_finish_in_kernel;               // every table is in a group (or is the closed-form eq): the resident kernel hands over the last pairs
    dpk::PolyGroup *d_poly_groups;            // [round 1..n_vars][group]
    dpk::PolyTerm *d_poly_terms;
    std::vector<dpk::PolyGroup> h_poly_groups;  // host copies: a single group travels in the kernel arguments
    std::vector<dpk::PolyTerm> h_poly_terms;
    std::vector<dpk::PolyOp> h_poly_ops;      // nested programs of the groups (empty: term by term)
    dpk::PolyOp *d_poly_ops;
    std::vector<char> stage;                  // descriptor upload in flight (no wait at set-up)
};

namespace {

u64 *mailbox(dps_ctx *ctx) { return ctx->h_pinned + ctx->res_off - 64; }
// device memory through which the first workgroup of a large launch made ahead passes the mail on (dpk::MAIL_RELAY_WORDS
// words behind the counters of the resident launches and their gate)
u64 *mail_relay(dps_ctx *ctx) { return reinterpret_cast<u64 *>(reinterpret_cast<char *>(ctx->d_counter) + 256 + SLICE_CTR_WORDS * 8 + 256); }

// completes a mail: check word over the payload as it stands, then the sequence number the kernel waits for
void send_mail(dps_ctx *ctx, u64 seq)
{
    u64 *mb = mailbox(ctx);
    u64 chk = seq;
    for (u32 i = dpk::MAIL_R; i < (u32)dpk::MAIL_WORDS; i++) chk ^= dpk::mail_mix(mb[i], i);
    mb[dpk::MAIL_CHK] = chk;
    __atomic_store_n(mb + dpk::MAIL_SEQ, seq, __ATOMIC_RELEASE);
}

// After launches that were waiting on the GPU have been told to leave (and the stream has drained): the ticket
// counters and sum counters back to zero, whatever a launch that gave up part-way left in them, and the relayed mail
// gone -- it says "leave" under a sequence number that the launch made in its place will wait for again.
void reset_device_words(dps_ctx *ctx) { (void)hipMemsetAsync(ctx->d_counter, 0, COUNTER_BYTES, ctx->stream); }

// ... and, once the stream has drained, what such a launch published part-way: the counter words of a trip are accepted
// by a 7-bit tag, so a word nobody took must not stay for the trip that carries the same tag 128 sequence numbers later
size_t slice_area_off(const dps_ctx *ctx);
size_t slice_fin_off(const dps_ctx *ctx);
// the area of the pinned buffer for the outputs of a fraction tree (16 words each, behind the resident launches' result area)
size_t logup_out_off(const dps_ctx *ctx, u32 slot) { return slice_area_off(ctx) + dpk::SL_AREA_WORDS + 64 + 16 * (size_t)slot; }
int32_t wait_result_at(dps_ctx *ctx, size_t base_off, u64 seq, u32 slot0, u32 n, u64 *out, int seq_slot = dpk::HOST_SEQ_SLOT,
                       int chk_slot = dpk::HOST_CHK_SLOT);
void clear_resident_results(dps_ctx *ctx)
{
    for (u32 c = 0; c < dpk::SL_MAX_GROUPS * (u32)dpk::SL_GROUP_WORDS; c++) ctx->h_pinned[slice_area_off(ctx) + c] = 0;
    ctx->h_pinned[slice_fin_off(ctx) + dpk::SL_FIN_SEQ_SLOT] = 0;
}

void tail_abort(dps_ctx *ctx)
{
    dps_sc *owner = ctx->tail_owner;
    if (!owner) return;
    __atomic_store_n(mailbox(ctx) + dpk::MAIL_SEQ, dpk::MAIL_ABORT_SEQ, __ATOMIC_RELEASE);
    (void)hipStreamSynchronize(ctx->stream);
    __atomic_store_n(mailbox(ctx) + dpk::MAIL_SEQ, (u64)0, __ATOMIC_RELEASE);
    reset_device_words(ctx);
    clear_resident_results(ctx);
    owner->tail_running = false;
    // a launch that has had no mail yet has changed nothing: its session goes on with ordinary launches
    if (owner->wait_fresh)
        owner->no_ahead = true;
    else
        owner->broken = true;
    owner->wait_fresh = false;
    waiting_launch_over(ctx);
}

// result area of the resident product launches (dpk::SL_AREA_WORDS words of the pinned buffer, behind the areas of resident groups)
size_t slice_area_off(const dps_ctx *ctx) { return ctx->pinned_words / 2 + 64 + 64 * 32; }

// A workgroup of a resident launch may take most of a compute unit's LDS (it is alone there: 1024 threads); more than
// 64 KB has to be asked for, once per kernel and device.  What a launch of this kernel can have, in bytes.
constexpr u32 SLICE_LDS_DEFAULT = 64 * 1024, SLICE_LDS_LARGE = 160 * 1024;
template <int NF, bool EQ, bool TERMS>
u32 slice_lds_granted(dps_ctx *ctx)
{
    static std::atomic<int> granted[64];  // 0 not asked, 1 granted, 2 refused
    std::atomic<int> &gr = granted[ctx->device & 63];
    int v = gr.load();
    if (v == 0) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&dpk::slice_kernel<NF, EQ, TERMS>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)SLICE_LDS_LARGE);
        if (e != hipSuccess) (void)hipGetLastError();
        v = e == hipSuccess ? 1 : 2;
        gr.store(v);
    }
    return v == 1 ? SLICE_LDS_LARGE : SLICE_LDS_DEFAULT;
}

template <int NF, bool EQ, bool TERMS>
void launch_slice(dps_ctx *ctx, u32 workgroups, u32 n_tabs, u32 cap, const dpk::SliceArgs &a)
{
    dpk::slice_kernel<NF, EQ, TERMS><<<workgroups, dpk::SL_BLOCK, dpk::slice_lds_words(n_tabs, cap, dpk::SL_BLOCK, EQ) * 8, ctx->stream>>>(a);
}

// the compiled variants: a product of 1 or 2 tables times eq, of 2 or 3 without; sums of several terms up to degree 4
#define SLICE_VARIANTS(SK)                                                              \
    SK(1, true, false) SK(2, true, false) SK(2, false, false) SK(3, false, false)       \
    SK(1, true, true) SK(2, true, true) SK(3, true, true) SK(4, true, true)             \
    SK(1, false, true) SK(2, false, true) SK(3, false, true) SK(4, false, true)
int32_t launch_slice_dispatch(dps_ctx *ctx, bool terms, u32 nf, bool eq, u32 workgroups, u32 n_tabs, u32 cap, const dpk::SliceArgs &a)
{
#define SK(NF_, EQ_, T_)                                                  \
    if (terms == T_ && nf == NF_ && eq == EQ_) {                          \
        launch_slice<NF_, EQ_, T_>(ctx, workgroups, n_tabs, cap, a);      \
        return DPS_OK;                                                    \
    }
    SLICE_VARIANTS(SK)
#undef SK
    return fail(ctx, DPS_ERR_UNSUPPORTED, "no resident kernel for degree %u, eq %d, several terms %d", nf, (int)eq, (int)terms);
}
// Workgroups of a resident launch of the variant that one compute unit holds at once, with the LDS it is launched with
// (the runtime's occupancy calculation; 0: such a workgroup does not fit, or no such variant).  Asked once per
// variant, device and LDS size.
template <int NF, bool EQ, bool TERMS>
int slice_occupancy(dps_ctx *ctx, u32 n_tabs, u32 cap)
{
    static std::mutex mu;
    static std::map<std::pair<int, size_t>, int> known;
    const size_t lds = dpk::slice_lds_words(n_tabs, cap, dpk::SL_BLOCK, EQ) * 8;
    std::lock_guard<std::mutex> lock(mu);
    auto it = known.find({ctx->device, lds});
    if (it != known.end()) return it->second;
    int n = 0;
    if (lds > slice_lds_granted<NF, EQ, TERMS>(ctx) ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void *>(&dpk::slice_kernel<NF, EQ, TERMS>), (int)dpk::SL_BLOCK, lds) != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    known[{ctx->device, lds}] = n;
    return n;
}
int slice_workgroups_per_cu(dps_ctx *ctx, bool terms, u32 nf, bool eq, u32 n_tabs, u32 cap)
{
#define SK(NF_, EQ_, T_) \
    if (terms == T_ && nf == NF_ && eq == EQ_) return slice_occupancy<NF_, EQ_, T_>(ctx, n_tabs, cap);
    SLICE_VARIANTS(SK)
#undef SK
    return 0;
}
// LDS a launch of the variant can have; 0: no such variant
u32 slice_lds_limit(dps_ctx *ctx, bool terms, u32 nf, bool eq)
{
#define SK(NF_, EQ_, T_) \
    if (terms == T_ && nf == NF_ && eq == EQ_) return slice_lds_granted<NF_, EQ_, T_>(ctx);
    SLICE_VARIANTS(SK)
#undef SK
    return 0;
}

template <int NF, int NB, bool EQ>
void launch_prod(dps_ctx *ctx, bool fold, const dpk::ProdArgs &a, u32 blocks, u64 *partial, const dpk::FastFin &ff)
{
    if constexpr (EQ) {
        if constexpr (NF == 2 && NB == 2) {
            if (a.two) {
                // (planned only where the weights come factored: plan_first_two_rounds)
                if (a.skip1)
                    dpk::prod_kernel<2, 2, true, true, true, true, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
                else
                    dpk::prod_kernel<2, 2, true, true, false, true, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
                return;
            }
        }
        if (a.lq0) {
            // large round: eq weights as a product of a small low table and a later level
            if (fold && a.skip1)
                dpk::prod_kernel<NF, NB, true, true, true, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
            else if (fold)
                dpk::prod_kernel<NF, NB, true, true, false, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
            else if (a.skip1)
                dpk::prod_kernel<NF, NB, false, true, true, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
            else
                dpk::prod_kernel<NF, NB, false, true, false, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
            return;
        }
    }
    if (fold && a.skip1)
        dpk::prod_kernel<NF, NB, true, EQ, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
    else if (fold)
        dpk::prod_kernel<NF, NB, true, EQ, false><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
    else if (a.skip1)
        dpk::prod_kernel<NF, NB, false, EQ, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
    else
        dpk::prod_kernel<NF, NB, false, EQ, false><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(a, partial, ff);
}

int32_t launch_prod_dispatch(dps_ctx *ctx, u32 nf, u32 nb, bool eq, bool fold, const dpk::ProdArgs &a, u32 blocks, u64 *partial,
                             const dpk::FastFin &ff)
{
#define PK(NF_, NB_, EQ_)                                             \
    if (nf == NF_ && nb == NB_ && eq == EQ_) {                        \
        launch_prod<NF_, NB_, EQ_>(ctx, fold, a, blocks, partial, ff); \
        return DPS_OK;                                                \
    }
    PK(2, 0, false) PK(2, 1, false) PK(2, 2, false) PK(3, 0, false) PK(3, 1, false) PK(3, 2, false) PK(3, 3, false)
    PK(1, 0, true) PK(1, 1, true) PK(2, 0, true) PK(2, 1, true) PK(2, 2, true)
#undef PK
    return fail(ctx, DPS_ERR_UNSUPPORTED, "no product kernel for %u tables, %u base, eq %d", nf, nb, (int)eq);
}

template <int NF>
void launch_poly(dps_ctx *ctx, bool eq, bool skip1, const dpk::PolyArgs &a, dim3 grid, size_t lds, u64 *partial, const dpk::FastFin &ff)
{
    if (eq && skip1)
        dpk::poly_kernel<NF, true, true><<<grid, dpk::BLOCK, lds, ctx->stream>>>(a, partial, ff);
    else if (eq)
        dpk::poly_kernel<NF, true, false><<<grid, dpk::BLOCK, lds, ctx->stream>>>(a, partial, ff);
    else if (skip1)
        dpk::poly_kernel<NF, false, true><<<grid, dpk::BLOCK, lds, ctx->stream>>>(a, partial, ff);
    else
        dpk::poly_kernel<NF, false, false><<<grid, dpk::BLOCK, lds, ctx->stream>>>(a, partial, ff);
}

int32_t launch_poly_dispatch(dps_ctx *ctx, u32 nf, bool eq, bool skip1, const dpk::PolyArgs &a, dim3 grid, u32 max_tabs, u64 *partial,
                             const dpk::FastFin &ff)
{
    // value and slope of every table of a group, per thread
    const size_t lds = (size_t)std::max<u32>(max_tabs, 1) * 4 * dpk::BLOCK * 8;  // + 2.3 KB of static LDS in the kernel
    switch (nf) {
    case 1: launch_poly<1>(ctx, eq, skip1, a, grid, lds, partial, ff); break;
    case 2: launch_poly<2>(ctx, eq, skip1, a, grid, lds, partial, ff); break;
    case 3: launch_poly<3>(ctx, eq, skip1, a, grid, lds, partial, ff); break;
    case 4: launch_poly<4>(ctx, eq, skip1, a, grid, lds, partial, ff); break;
    case 5: launch_poly<5>(ctx, eq, skip1, a, grid, lds, partial, ff); break;
    case 6: launch_poly<6>(ctx, eq, skip1, a, grid, lds, partial, ff); break;
    default: return fail(ctx, DPS_ERR_UNSUPPORTED, "no fused kernel for degree %u", nf);
    }
    return DPS_OK;
}

// Several groups resident side by side publish into 64-word slots of the pinned buffer from here on
constexpr u32 POLY_RAW_MAX_GROUPS = 32;
static_assert(POLY_RAW_MAX_GROUPS == 32, "slice_area_off lies behind the result areas of the resident groups");
size_t poly_raw_off(const dps_ctx *ctx) { return ctx->pinned_words / 2 + 64; }
// a launch of this many workgroups publishes per workgroup (FastFin::slots) rather than through the last one
constexpr u32 SLOT_MAX_WORKGROUPS = 16;
static_assert(SLOT_MAX_WORKGROUPS <= POLY_RAW_MAX_GROUPS, "the per-workgroup result areas are those of the resident groups");
u32 slots_for(u32 workgroups) { return workgroups > 1 && workgroups <= SLOT_MAX_WORKGROUPS ? workgroups : 0; }

// In a launch made ahead of its round every workgroup polls the host's mailbox up to this many workgroups; in a larger
// one only the first does and passes the mail on through device memory
constexpr u32 POLY_AHEAD_MAX_WORKGROUPS = 64;
// ... and is trusted to be still waiting for its mail for this long (its own patience is several times that)
constexpr int POLY_AHEAD_PATIENCE_MS = 20;
// How long a launch made ahead waits for its mail, in units of 2.56 us (wait_units): about 150 ms, so that a caller who
// went away does not leave up to 768 waiting workgroups on the GPU for long (a resident launch waits ten seconds)
constexpr u32 AHEAD_SPIN_LIMIT = 60000;

// Rounds of at most this many pairs run on poly_split_kernel
constexpr u64 POLY_SPLIT_MAX_PAIRS = 1ull << 16;

// lanes per pair (log2) and grid of a split round: about 2^17 threads while that many items exist; a round
// that fits one workgroup takes the lanes the workgroup has when it can stay resident (a single group)
void poly_split_plan(u64 n_pairs, u32 cap, bool may_reside, u32 *split_log, u32 *blocks)
{
    u32 lp = log2u(n_pairs);
    u32 sl = (may_reside && n_pairs <= dpk::BLOCK) ? log2u(dpk::BLOCK) - lp : (lp < 17 ? 17 - lp : 0);
    sl = std::min(sl, cap);
    *split_log = sl;
    *blocks = (u32)std::max<u64>(1, (n_pairs << sl) / dpk::BLOCK);
}

// Resident launches keep the folded tables in LDS, which takes more dynamic LDS than a launch gets by default:
// asked for once per kernel and device.
template <int NF, bool EQ, bool SKIP1>
bool poly_split_state_granted(dps_ctx *ctx)
{
    static std::atomic<int> granted[64];  // 0 not asked, 1 granted, 2 refused
    std::atomic<int> &gr = granted[ctx->device & 63];
    int v = gr.load();
    if (v == 0) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&dpk::poly_split_kernel<NF, EQ, SKIP1>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)(dpk::POLY_MAXT * 10 * dpk::BLOCK * 8));
        if (e != hipSuccess) (void)hipGetLastError();
        v = e == hipSuccess ? 1 : 2;
        gr.store(v);
    }
    return v == 1;
}

template <int NF, bool EQ, bool SKIP1>
int32_t launch_poly_split_one(dps_ctx *ctx, dpk::PolyArgs &a, dim3 grid, u32 max_tabs, bool want_state, u64 *partial, const dpk::FastFin &ff)
{
    // value and slope of every table, per pair; resident launches add the folded tables themselves
    const size_t lds_vals = (size_t)std::max<u32>(max_tabs, 1) * 4 * dpk::BLOCK * 8;
    // two buffers of POLY_MAXT tables: 2 * BLOCK and BLOCK entries per limb array
    const size_t lds_state = (size_t)dpk::POLY_MAXT * 2 * 3 * dpk::BLOCK * 8;
    size_t lds = lds_vals;
    a.lds_state = 0;
    a.state_off = (u32)(lds_vals / 8);
    if (want_state && poly_split_state_granted<NF, EQ, SKIP1>(ctx)) {
        a.lds_state = 1;
        lds = lds_vals + lds_state;
    }
    // several resident groups must not read each other's stores: without the tables in LDS they cannot stay
    if (a.raw_out && !a.lds_state) return fail(ctx, DPS_ERR_HIP, "resident groups need the larger LDS allocation");
    dpk::poly_split_kernel<NF, EQ, SKIP1><<<grid, dpk::BLOCK, lds, ctx->stream>>>(a, partial, ff);
    return DPS_OK;
}

template <int NF>
int32_t launch_poly_split(dps_ctx *ctx, bool eq, bool skip1, dpk::PolyArgs &a, dim3 grid, u32 max_tabs, bool want_state, u64 *partial,
                          const dpk::FastFin &ff)
{
    if (eq && skip1) return launch_poly_split_one<NF, true, true>(ctx, a, grid, max_tabs, want_state, partial, ff);
    if (eq) return launch_poly_split_one<NF, true, false>(ctx, a, grid, max_tabs, want_state, partial, ff);
    if (skip1) return launch_poly_split_one<NF, false, true>(ctx, a, grid, max_tabs, want_state, partial, ff);
    return launch_poly_split_one<NF, false, false>(ctx, a, grid, max_tabs, want_state, partial, ff);
}

template <int NF>
bool poly_split_state_ok_nf(dps_ctx *ctx, bool eq, bool skip1)
{
    if (eq && skip1) return poly_split_state_granted<NF, true, true>(ctx);
    if (eq) return poly_split_state_granted<NF, true, false>(ctx);
    if (skip1) return poly_split_state_granted<NF, false, true>(ctx);
    return poly_split_state_granted<NF, false, false>(ctx);
}

// can a resident launch of this kernel keep its tables in LDS?
bool poly_split_state_ok(dps_ctx *ctx, u32 nf, bool eq, bool skip1)
{
    switch (nf) {
    case 1: return poly_split_state_ok_nf<1>(ctx, eq, skip1);
    case 2: return poly_split_state_ok_nf<2>(ctx, eq, skip1);
    case 3: return poly_split_state_ok_nf<3>(ctx, eq, skip1);
    case 4: return poly_split_state_ok_nf<4>(ctx, eq, skip1);
    case 5: return poly_split_state_ok_nf<5>(ctx, eq, skip1);
    case 6: return poly_split_state_ok_nf<6>(ctx, eq, skip1);
    default: return false;
    }
}

int32_t launch_poly_split_dispatch(dps_ctx *ctx, u32 nf, bool eq, bool skip1, dpk::PolyArgs &a, dim3 grid, u32 max_tabs, bool want_state,
                                   u64 *partial, const dpk::FastFin &ff)
{
    switch (nf) {
    case 1: return launch_poly_split<1>(ctx, eq, skip1, a, grid, max_tabs, want_state, partial, ff);
    case 2: return launch_poly_split<2>(ctx, eq, skip1, a, grid, max_tabs, want_state, partial, ff);
    case 3: return launch_poly_split<3>(ctx, eq, skip1, a, grid, max_tabs, want_state, partial, ff);
    case 4: return launch_poly_split<4>(ctx, eq, skip1, a, grid, max_tabs, want_state, partial, ff);
    case 5: return launch_poly_split<5>(ctx, eq, skip1, a, grid, max_tabs, want_state, partial, ff);
    case 6: return launch_poly_split<6>(ctx, eq, skip1, a, grid, max_tabs, want_state, partial, ff);
    default: return fail(ctx, DPS_ERR_UNSUPPORTED, "no fused kernel for degree %u", nf);
    }
}

u32 blocks_for_pairs(u64 n_pairs) { return grid_for(n_pairs); }
// Workgroups of a product launch (prod_kernel): one thread per pair up to MAX_BLOCKS workgroups -- and in the rounds where that
// gives a thread fewer than four pairs (2^19 pairs and fewer), four pairs a thread down to 256 workgroups: fewer partial sums
// to gather, fewer workgroups to hand the mail to, and these launches are latency by then (cfg3: 0.427 -> 0.422 ms with 512 and
// 256 workgroups in rounds 5 and 6).  The launches of sums of several terms are arithmetic and keep a thread per pair
// (with this rule cfg5 3.65 -> 3.79 ms, linking 1.01 -> 1.09).
u32 product_blocks(u64 n_pairs)
{
    const u32 full = grid_for(n_pairs), few = grid_for(n_pairs, dpk::BLOCK * 4);
    return std::min<u32>(full, std::max<u32>(few, 256));
}

}  // namespace

namespace {

// Nested (Horner) form of a group's terms: the table found in most of the remaining terms is factored out of
// them, recursively.  Appends the program to `ops`; returns its number of products.
struct HornerTerm {
    E2 coeff;
    std::vector<uint8_t> slots;  // remaining factors
};

u32 horner_build(std::vector<HornerTerm> ts, u32 depth, std::vector<dpk::PolyOp> &ops)
{
    auto make = [](u32 kind, u32 d, u32 slot, E2 c) {
        dpk::PolyOp op;
        memset(&op, 0, sizeof op);
        op.c0 = c.c0;
        op.c1 = c.c1;
        op.w = gl::mul_small(c.c1, (u32)gl::W);
        op.code = kind | d << 2 | slot << 8;
        return op;
    };
    u32 products = 0;
    // terms that end at this node were added to the node's constant by the caller
    ts.erase(std::remove_if(ts.begin(), ts.end(), [](const HornerTerm &t) { return t.slots.empty(); }), ts.end());
    while (!ts.empty()) {
        // slots are positions within a group: fewer than POLY_MAXT
        u32 count[dpk::POLY_MAXT] = {0};
        for (const HornerTerm &t : ts) {
            u32 seen = 0;
            for (uint8_t sl : t.slots)
                if (!((seen >> sl) & 1)) {
                    seen |= 1u << sl;
                    count[sl]++;
                }
        }
        u32 best = 0;
        for (u32 sl = 1; sl < (u32)dpk::POLY_MAXT; sl++)
            if (count[sl] > count[best]) best = sl;
        std::vector<HornerTerm> sub, rest;
        for (HornerTerm &t : ts) {
            auto it = std::find(t.slots.begin(), t.slots.end(), (uint8_t)best);
            if (it == t.slots.end()) {
                rest.push_back(std::move(t));
            } else {
                t.slots.erase(it);
                sub.push_back(std::move(t));
            }
        }
        E2 ends = gl::e2_zero();
        bool inner = false;
        for (const HornerTerm &t : sub) {
            if (t.slots.empty())
                ends = gl::add(ends, t.coeff);
            else
                inner = true;
        }
        if (!inner) {
            ops.push_back(make(dpk::POLY_OP_LEAF, depth, best, ends));
        } else {
            ops.push_back(make(dpk::POLY_OP_ENTER, depth + 1, 0, ends));
            products += horner_build(std::move(sub), depth + 1, ops);
            ops.push_back(make(dpk::POLY_OP_LEAVE, depth + 1, best, gl::e2_zero()));
        }
        products++;
        ts = std::move(rest);
    }
    return products;
}

// one staged upload of all descriptors; not waited for (the staging vector lives as long as the session)
int32_t ensure_descs(dps_sc *sc)
{
    if (sc->descs_uploaded || sc->stage.empty()) return DPS_OK;
    dps_ctx *ctx = sc->ctx;
    const void *from = sc->stage.data();
    const bool staged = ctx->h_desc_stage && sc->stage.size() <= DESC_STAGE_BYTES;
    if (staged) {
        // through the context's pinned buffer: the copy is then queued, not made inside the call (the buffer's previous
        // copy, of another session, has long been made; waited for all the same)
        if (ctx->desc_pending) {
            HIPCHK(ctx, hipEventSynchronize(ctx->desc_event));
            ctx->desc_pending = false;
        }
        memcpy(ctx->h_desc_stage, sc->stage.data(), sc->stage.size());
        from = ctx->h_desc_stage;
    }
    hipError_t e = hipMemcpyAsync(sc->dev_block, from, sc->stage.size(), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess && staged) {
        e = hipEventRecord(ctx->desc_event, ctx->stream);
        ctx->desc_pending = e == hipSuccess;
    }
    if (e != hipSuccess) return fail(sc->ctx, DPS_ERR_HIP, "descriptor upload: %s", hipGetErrorString(e));
    sc->descs_uploaded = true;
    return DPS_OK;
}

}  // namespace

namespace {

// Most pairs a workgroup of a resident launch can take in its first round: its LDS holds twice as many entries per table
// and half of that again.
u32 slice_pairs_per_workgroup(u32 n_tabs, bool eq, u32 lds_bytes)
{
    u32 cap = 4096;
    while (cap > 2 && dpk::slice_lds_words(n_tabs, cap, dpk::SL_BLOCK, eq) * 8 > lds_bytes) cap >>= 1;
    return cap / 2;
}
// ... and the fewest it is given when the sum is small enough for that: shorter chains of work per lane, more workgroups
// (measured with 128, 64, 32, 16: 8 products over 16 tables 0.130, 0.119, 0.114, 0.111 ms; the fraction-tree proof 3.37, 3.30,
// 3.28, 3.38 ms -- more workgroups cost little since their sums go into several sets of counters)
constexpr u32 SLICE_MIN_PAIRS = 32;
// ... and a sum that could be cut finer takes half the device at most, so that two such sums of two contexts find room
// side by side (a launch that fills the device alone sends every other context's resident rounds back to launches of their own)
constexpr u32 SLICE_SMALL_SUM_WORKGROUPS = 128;
constexpr u32 SLICE_ONE_WORKGROUP_TERM_PAIRS = 512;  // pairs x terms up to which one workgroup takes the whole sum
constexpr u32 SLICE_MAX_WORKGROUPS = 256;
// the rounds a resident launch leaves to the host: at most so many, and so many extension multiplications in all
// (measured: 2 to 6 rounds and 400 to 3000 multiplications differ by a few percent; these were the best over the benchmark configurations)
constexpr u32 HOST_TAIL_MAX_ROUNDS = 5;
constexpr u64 HOST_TAIL_MULTS = 800;

// eq * f * g over two base-field tables, large enough for the factored eq weights: rounds 1 and 2 can be one launch
// that reads the tables once and writes nothing (pair12_kernel).  `first_resident`: the first round of the resident
// launches (0: none).  Only what is known when the session is set up enters here.
bool first_two_rounds_fit(const dps_sc *sc, u32 n_mles, u32 first_resident)
{
    const u32 n = sc->n_vars;
    if (!sc->fast || sc->fast_eq < 0 || sc->fast_nf != 2 || n_mles != 3 || !sc->fast_all_base) return false;
    if (n < dpk::EQ_LO_BITS + 3 || (first_resident && first_resident <= 3)) return false;
    if (sc->eq_info->fact_levels < 3) return false;
    if (((u64)product_blocks(1ull << (n - 3)) * dpk::BLOCK) % (1ull << dpk::EQ_LO_BITS) != 0) return false;
    // (round 2's p(1) comes from the claim: its scale must not vanish at 1)
    const E2 rho2 = sc->eq_info->point[1];
    return !((rho2.c0 == 0 && rho2.c1 == 0) || (sc->fast_coeff.c0 == 0 && sc->fast_coeff.c1 == 0));
}

// Workgroups of a launch that covers two rounds (quad_kernel) over `n_quads` quads, QUAD_STEP of them a workgroup's step:
// a stride of exactly the low eq table's size (1024 workgroups: four wavefronts on every SIMD)
u32 quad_blocks(u64 n_quads) { return (u32)std::min<u64>(n_quads / dpk::QUAD_STEP, ((u64)1 << dpk::EQ_LO_BITS) / dpk::QUAD_STEP); }

// How many such launches follow the launch of the first two rounds: all of rounds 3 .. first_resident - 1 in pairs, when
// they are an even number of rounds, every one takes p(1) from its claim (no zero among those coordinates of the eq
// point) and every launch's quads still make a full stride of the factored weights.
u32 quad_launches_fit(const dps_sc *sc, u32 n_mles, u32 first_resident)
{
    const u32 n = sc->n_vars;
    if (!first_two_rounds_fit(sc, n_mles, first_resident) || first_resident < 5 || ((first_resident - 3) & 1)) return 0;
    for (u32 j = 3; j < first_resident; j++) {
        const E2 rho = sc->eq_info->point[j - 1];
        if (rho.c0 == 0 && rho.c1 == 0) return 0;
    }
    for (u32 j = 3; j < first_resident; j += 2) {
        // the launch's weights are those of round j + 1's pairs: low table of level j + 1, level j + 1 + 16
        if (j + 1 > sc->eq_info->fact_levels || n < j + 1 + dpk::EQ_LO_BITS) return 0;
    }
    return (first_resident - 3) / 2;
}

// A round of a sum of several terms with a common eq factor whose launch (poly_kernel, a thread per pair) takes the eq
// weights from the low table of its level and from the level 16 rounds later instead of streaming its own level: the
// rounds of more than 2^16 pairs, whose grid stride is a multiple of 2^16, of a table that has its low tables.
bool poly_round_weights_factored(const dps_sc *sc, u32 jj)
{
    if (!sc->poly || sc->fast_eq < 0 || !sc->eq_info || !sc->eq_info->fact_built || jj > sc->eq_info->fact_levels) return false;
    const u64 n_pairs = 1ull << (sc->n_vars - jj);
    if (n_pairs <= POLY_SPLIT_MAX_PAIRS) return false;  // (those rounds spread a pair over lanes: poly_split_kernel)
    return ((u64)blocks_for_pairs(n_pairs) * dpk::BLOCK) % (1ull << dpk::EQ_LO_BITS) == 0;
}

// Sets of counters the workgroups of a resident launch add their sums into (log2): adds to one counter are served one
// after the other, so a set is shared by no more than 32 of them and by at least 8 (the host waits for every set)
u32 slice_counter_sets_log(u32 W)
{
    u32 l = 0;
    while (l < 3 && (W >> l) > 8 && (1u << (l + 1)) <= dpk::SL_MAX_GROUPS) l++;
    return l;
}

// Passes the lanes of a workgroup make over `n_quads` quads for the second round of a trip: a lane keeps one sample at one
// point for some of the terms (slice_kernel's q_split), the lanes of a pass cover BLOCK / (q_split NF (NF + 1)) quads
u32 slice_second_round_passes(const dps_sc *sc, u32 n_quads)
{
    const u32 nf = sc->fast_nf, per_quad_pts = nf * (nf + 1);
    const u32 n_terms = sc->poly ? (u32)sc->slice_terms.size() : 1;
    const u32 q_split = n_terms * per_quad_pts <= (u32)dpk::SL_BLOCK ? n_terms : 1;
    const u32 slots = std::max<u32>(1, (u32)dpk::SL_BLOCK / (q_split * per_quad_pts));
    return (n_quads + slots - 1) / slots;
}
constexpr u32 SLICE_SECOND_ROUND_BUDGET = 10;

// Which rounds of a session are resident, in which launches, and how they pair up into trips.  `n_tabs`: tables in LDS.
// A trip covers two rounds when the second one's p(1) can come from the claim (its eq coordinate is not zero) and the
// workgroups still hold a quad each.  The first resident round is the first whose pairs fit 256 workgroups.
void plan_resident_rounds(dps_sc *sc, u32 n_tabs, u32 n_mles)
{
    const u32 n = sc->n_vars;
    const bool has_eq = sc->fast_eq >= 0;
    const u32 first_ok = 1;
    auto claim_gives_p1 = [&](u32 round) {
        if (sc->fast_coeff.c0 == 0 && sc->fast_coeff.c1 == 0) return false;
        if (!has_eq) return true;
        const E2 rho = sc->eq_info->point[round - 1];
        return !(rho.c0 == 0 && rho.c1 == 0);
    };
    const u32 lds_bytes = slice_lds_limit(sc->ctx, sc->poly, sc->fast_nf, has_eq);
    if (lds_bytes == 0) return;
    // (more pairs per workgroup would make more rounds resident, but a trip's arithmetic is a workgroup's alone: with 512
    // pairs of a 3-term sum the first trip took 75 us where a launch for the round and a trip of 128 pairs take 66)
    const u32 per_wg_max = std::min<u32>(slice_pairs_per_workgroup(n_tabs, has_eq, lds_bytes), sc->poly ? 128 : 512);
    auto pairs_of = [&](u32 round) { return (u64)1 << (n - round); };
    u32 j = first_ok;
    while (pairs_of(j) > (u64)per_wg_max * SLICE_MAX_WORKGROUPS) j++;
    // (a small sum stays with one workgroup -- 128 pairs of three terms: four workgroups were 7 us slower over the eight
    // rounds; 128 pairs of eight terms over 16 tables: four workgroups were 13 us faster)
    const u64 term_pairs = pairs_of(j) * (sc->poly ? std::max<size_t>(sc->slice_terms.size(), 1) : 1);
    const u32 per_wg = term_pairs <= SLICE_ONE_WORKGROUP_TERM_PAIRS && pairs_of(j) <= per_wg_max
                           ? (u32)pairs_of(j)
                           : (u32)std::min<u64>(per_wg_max, std::max<u64>(SLICE_MIN_PAIRS, pairs_of(j) / SLICE_SMALL_SUM_WORKGROUPS));
    sc->tail_j0 = j;
    // The last rounds are the host's: a trip costs the way to the GPU and back and a workgroup's barriers whatever it
    // carries, a round of a few pairs costs the host a microsecond.  As many rounds as stay below HOST_TAIL_MULTS
    // extension multiplications in all and whose tables fit the hand-over (the trip before them can cover two rounds:
    // four times the entries of the first host round), and never the first resident round.
    u32 host_rounds = 0;
    {
        u32 factors = 0;  // multiplications per pair and point
        if (sc->poly)
            for (const dpk::SliceTerm &t : sc->slice_terms) factors += t.n_factors + 1;
        else
            factors = sc->fast_nf;
        factors += has_eq ? 1 : 0;
        const u64 per_pair = (u64)factors * (sc->fast_nf + 1) + 2 * n_tabs;
        // (the launch keeps a trip for its single workgroup, which hands the tables over, and two rounds before it when
        // several workgroups start)
        const u32 gpu_rounds_min = pairs_of(j) > per_wg ? 3 : 1;
        while (host_rounds < HOST_TAIL_MAX_ROUNDS && host_rounds + gpu_rounds_min <= n - j && (((u64)2 << host_rounds) - 1) * per_pair <= HOST_TAIL_MULTS &&
               (u64)n_tabs * ((u64)8 << (host_rounds + 1)) <= (u64)dpk::SL_FIN_MAX_WORDS)
            host_rounds++;
    }
    const u32 n_gpu = n - host_rounds;  // the last round of a trip
    sc->host_rounds = host_rounds;
    for (u32 r = n_gpu + 1; r <= n; r++) sc->round_kind[r] = 4;
    // a launch that starts with round 1 has nothing to fold first; one behind a launch that covered two rounds
    // (quad_kernel) finds the state of two rounds ago
    u32 pend = j == 1 ? 0 : (!sc->poly && quad_launches_fit(sc, n_mles, j) ? 2 : 1);
    u64 entries = (u64)1 << (n - j + 1 + pend);  // of the tables the stage to come starts from (before its pending folds)
    auto add_stage = [&](u32 W) {
        dps_sc::Stage st;
        memset(&st, 0, sizeof st);
        st.W = W;
        st.j0 = j;
        st.pend0 = pend;
        st.src_len = entries;
        u64 len = (entries / W) >> pend;  // entries per table and workgroup in the trip's first round
        st.cap = (u32)len;
        for (;;) {
            bool dbl = len >= 4 && j + 1 <= n_gpu && claim_gives_p1(j + 1);
            // The second round's sums are (NF + 1) NF evaluations a quad where a trip of its own takes NF a pair: worth it while
            // the lanes take a workgroup's quads in a few passes (a pass is a chain of about NF + 1 dependent products), that
            // is while it costs less than the trip it saves.  Measured on the degree-4 linking sum (7 terms: two-round
            // trips from 32 entries a workgroup on, 0.83 -> 0.72 ms) and on 8 products over 16 tables (0.145 -> 0.135 ms).
            if (dbl && slice_second_round_passes(sc, (u32)(len >> 2)) * (sc->fast_nf + 1) > SLICE_SECOND_ROUND_BUDGET) dbl = false;
            if (W > 1 && j + 1 == n_gpu) dbl = false;  // the last trip is the single workgroup's
            if (dbl) st.dbl_mask |= 1u << st.n_trips;
            st.n_trips++;
            sc->round_kind[j] = dbl ? 2 : 1;
            sc->round_wide[j] = W > 1 ? (uint8_t)(1u << slice_counter_sets_log(W)) : 0;
            if (dbl) sc->round_kind[j + 1] = 3;
            pend = dbl ? 2 : 1;
            j += pend;
            // several workgroups go on while each still has a pair after the pending folds; one goes on to the last trip
            if (j > n_gpu || (W > 1 && (j == n_gpu || (len >> pend) < 2)) || st.n_trips == (u32)dpk::SL_MAX_TRIPS) break;
            len >>= pend;
        }
        entries = len * W;
        sc->fin_len = (u32)len;
        sc->fin_pend = pend;
        sc->stages.push_back(st);
    };
    if (pairs_of(j) > per_wg) add_stage((u32)(pairs_of(j) / per_wg));
    while (j <= n_gpu) add_stage(1);
}

// The session's resident launch found no place on the device (admit_waiting_launch): the rounds it would have run, and
// those the host would have worked out behind it, are launches of their own like the rounds before them.  Every
// round's launch was described at set-up whatever the plan, and the eq levels those rounds read are built.
void drop_resident_plan(dps_sc *sc)
{
    sc->stages.clear();
    sc->tail_j0 = 0;
    sc->fin_len = 0;
    sc->fin_pend = 0;
    sc->host_rounds = 0;
    // (the rounds of launches that cover two rounds, kinds 5 and 6, stay what they are)
    for (uint8_t &k : sc->round_kind)
        if (k <= 4) k = 0;
    std::fill(sc->round_wide.begin(), sc->round_wide.end(), 0);
}

}  // namespace

namespace {

// What dps_sc_begin works out for a new session, step by step: which kernels can take it, which rounds are resident, where
// every table lies in every round (the launches' descriptors), and the device block that holds descriptors, partials and
// hand-over buffers.
struct SessionSetup {
    dps_ctx *ctx;
    dps_sc *sc;
    u32 n_vars;
    const dps_mle *const *mles;
    u32 n_mles;
    std::vector<u32> nv0;  // variables of every table as registered
    // sums of several terms: the closed-form eq factor (-1: none), the degree without it, the groups of tables and the terms of each
    int eq = -1;
    u32 nf = 0;
    std::vector<std::vector<u32>> groups;
    std::vector<u32> tb, te;
    std::vector<dpk::PolyTerm> poly_terms;
    // descriptors of every round, from a dry run of the folds
    std::vector<dpk::FoldDesc> folds, folds_extra;
    std::vector<dpk::TermDesc> tdescs;
    std::vector<dpk::PolyGroup> poly_groups;  // [round][group]
    std::vector<dpk::FinTerm> fins;
    std::vector<dpk::GatherDesc> gath;
    std::vector<SessMle> sim;  // the tables as the round being described finds them
    std::vector<const u64 *> pre0, pre1;  // where a table folded in this step lay before
    std::vector<char> folded;
    size_t bytes_fold = 0, bytes_fold_x = 0, bytes_terms = 0, bytes_fin = 0, bytes_gath = 0, bytes_pg = 0, bytes_pt = 0, bytes_po = 0;

    // a zero-padded table keeps folding after it is down to one entry: both of its buffers hold at least that entry
    bool zpad_of(u32 k) const { return mles[k]->pad_vars != 0 && nv0[k] < n_vars; }
    u64 len_a(u32 k) const { return nv0[k] >= 1 ? (1ull << (nv0[k] - 1)) : (zpad_of(k) ? 1ull : 0ull); }
    u64 len_b(u32 k) const { return nv0[k] >= 2 ? (1ull << (nv0[k] - 2)) : (zpad_of(k) ? 1ull : 0ull); }
    bool in_fast(u32 k) const;

    void detect_product();
    bool closed_form_eq_factor();
    bool group_terms();
    void adopt_groups();
    void nested_programs();
    void detect_multi_term();
    int32_t plan_and_ready_tables();
    int32_t layout_scratch();
    void fold_step(u32 j);
    void poly_groups_of_round(u32 j);
    void term_descs_of_round(u32 j);
    void describe_rounds();
    int32_t plan_first_two_rounds();
    void launch_limits();
    int32_t allocate_device_block();
    int32_t stage_descriptors();
    int32_t run();
};


// tables the fused kernels fold themselves (the others fold in launches of their own)
bool SessionSetup::in_fast(u32 k) const
{
        if (sc->poly) return sc->poly_owner[k] >= 0;
        if (!sc->fast) return false;
        for (u32 f = 0; f < sc->fast_nf; f++)
            if (sc->fast_order[f] == k) return true;
        return false;
}

// One product of 2 or 3 distinct full-size tables (one of them possibly an eq table, taken in closed form): prod_kernel.
void SessionSetup::detect_product()
{
    sc->fast = false;
    sc->fast_all_base = false;
    sc->quads.clear();
    sc->broken = false;
    sc->tail_j0 = 0;
    sc->tail_running = false;
    sc->tail_seq0 = 0;
    sc->wait_stays = sc->wait_skip1 = sc->wait_any_skip1 = sc->wait_fresh = sc->no_ahead = false;
    sc->wait_slots = 0;
    sc->pairs_seq = 0;
    sc->fast_eq = -1;
    sc->eq_scalar = gl::e2_one();
    sc->claim = gl::e2_zero();
    sc->have_claim = false;
    if (sc->n_terms == 1 && sc->terms[0].n_factors >= 2 && sc->terms[0].n_factors <= 3 && n_vars >= 1) {
        const dps_term &t = sc->terms[0];
        bool ok = true;
        for (u32 f = 0; f < t.n_factors && ok; f++) {
            if (nv0[t.factors[f]] != n_vars) ok = false;
            for (u32 q = 0; q < f; q++)
                if (t.factors[q] == t.factors[f]) ok = false;
        }
        if (ok) {
            for (u32 f = 0; f < t.n_factors && sc->fast_eq < 0; f++) {
                const dps_mle *h = mles[t.factors[f]];
                if (h->eq && h->eq->m == n_vars && h->kind == DPS_EXT2) {
                    sc->fast_eq = (int)t.factors[f];
                    sc->eq_info = h->eq;
                    sc->eq_c0 = h->p0();
                    sc->eq_c1 = h->p1();
                }
            }
            u32 w = 0;
            for (u32 f = 0; f < t.n_factors; f++)
                if ((int)t.factors[f] != sc->fast_eq && mles[t.factors[f]]->kind == DPS_BASE) sc->fast_order[w++] = t.factors[f];
            for (u32 f = 0; f < t.n_factors; f++)
                if ((int)t.factors[f] != sc->fast_eq && mles[t.factors[f]]->kind != DPS_BASE) sc->fast_order[w++] = t.factors[f];
            sc->fast_nf = w;
            sc->fast_all_base = true;
            for (u32 f = 0; f < w; f++) sc->fast_all_base = sc->fast_all_base && mles[sc->fast_order[f]]->kind == DPS_BASE;
            // compiled variants: 2 or 3 streamed tables without an eq factor, 1 or 2 with one
            sc->fast = sc->fast_eq >= 0 ? (w >= 1 && w <= 2) : (w >= 2 && w <= 3);
            if (!sc->fast) sc->fast_eq = -1;
            sc->fast_coeff = gl::e2(t.coeff[0], t.coeff[1]);
        }
    }

}

// Sums of several terms (every table full-size or constant in the low variables).  True: no table stands in the way.
// An eq table that is a factor of every term exactly once comes out in closed form (`eq`).
bool SessionSetup::closed_form_eq_factor()
{
    bool ok = true;
    for (const dps_term &t : sc->terms)
        for (u32 f = 0; f < t.n_factors; f++)
            if (mles[t.factors[f]]->pad_vars && nv0[t.factors[f]] < n_vars) ok = false;
    if (ok) {
        const dps_term &t0 = sc->terms[0];
        for (u32 f = 0; f < t0.n_factors && eq < 0; f++) {
            const u32 k = t0.factors[f];
            const dps_mle *h = mles[k];
            if (!(h->eq && h->eq->m == n_vars && h->kind == DPS_EXT2 && nv0[k] == n_vars)) continue;
            bool all = true;
            u32 inner = 0;
            for (const dps_term &t : sc->terms) {
                u32 cnt = 0;
                for (u32 q = 0; q < t.n_factors; q++) cnt += t.factors[q] == k;
                if (cnt != 1) all = false;
                inner = std::max(inner, t.n_factors - 1);
            }
            if (all && inner >= 1) eq = (int)k;
        }
    }
    return ok;
}

// The terms in order, a new group whenever the tables no longer fit one (POLY_MAXT).  False: a term has too many tables.
bool SessionSetup::group_terms()
{
    nf = 0;
    for (const dps_term &t : sc->terms) nf = std::max(nf, eq >= 0 ? t.n_factors - 1 : t.n_factors);
    bool ok = nf >= 1 && nf <= 6;
    // terms in order, a new group whenever the tables no longer fit
    if (ok) {
        std::vector<u32> cur;
        u32 begin = 0;
        for (u32 ti = 0; ti < sc->n_terms && ok; ti++) {
            const dps_term &t = sc->terms[ti];
            std::vector<u32> need;
            for (u32 f = 0; f < t.n_factors; f++) {
                const u32 k = t.factors[f];
                if ((int)k == eq) continue;
                if (std::find(need.begin(), need.end(), k) == need.end()) need.push_back(k);
            }
            if (need.size() > (size_t)dpk::POLY_MAXT) {
                ok = false;
                break;
            }
            std::vector<u32> merged = cur;
            for (u32 k : need)
                if (std::find(merged.begin(), merged.end(), k) == merged.end()) merged.push_back(k);
            if (merged.size() > (size_t)dpk::POLY_MAXT) {
                groups.push_back(cur);
                tb.push_back(begin);
                te.push_back(ti);
                begin = ti;
                merged = need;
            }
            cur = merged;
        }
        if (ok) {
            groups.push_back(cur);
            tb.push_back(begin);
            te.push_back(sc->n_terms);
        }
    }
    return ok && groups.size() <= 65535;
}

// the session takes the groups: owners of the tables, the terms with their tables as slots of their group
void SessionSetup::adopt_groups()
{
    sc->poly = true;
    sc->poly_tabs = groups;
    sc->poly_term_begin = tb;
    sc->poly_term_end = te;
    sc->poly_owner.assign(n_mles, -1);
    for (size_t g = 0; g < groups.size(); g++) {
        sc->poly_max_tabs = std::max<u32>(sc->poly_max_tabs, (u32)groups[g].size());
        for (u32 k : groups[g])
            if (sc->poly_owner[k] < 0) sc->poly_owner[k] = (int)g;
    }
    sc->fast_nf = nf;
    sc->fast_coeff = gl::e2_one();
    if (eq >= 0) {
        sc->fast_eq = eq;
        sc->eq_info = mles[eq]->eq;
        sc->eq_c0 = mles[eq]->p0();
        sc->eq_c1 = mles[eq]->p1();
    }
    for (size_t g = 0; g < groups.size(); g++)
        for (u32 ti = tb[g]; ti < te[g]; ti++) {
            const dps_term &t = sc->terms[ti];
            dpk::PolyTerm pt;
            memset(&pt, 0, sizeof pt);
            pt.c0 = t.coeff[0];
            pt.c1 = t.coeff[1];
            pt.w = gl::mul_small(t.coeff[1], (u32)gl::W);
            for (u32 f = 0; f < t.n_factors; f++) {
                if ((int)t.factors[f] == eq) continue;
                const auto &gt = groups[g];
                pt.slot[pt.n_factors++] = (uint8_t)(std::find(gt.begin(), gt.end(), t.factors[f]) - gt.begin());
            }
            poly_terms.push_back(pt);
        }
}

void SessionSetup::nested_programs()
{
    // the nested form, where it saves products and fits the kernel's staging area
    sc->poly_op_begin.assign(groups.size(), 0);
    sc->poly_op_end.assign(groups.size(), 0);
    // (only the kernel of the rounds of more than 2^16 pairs runs it: a smaller sum has no use for it)
    bool use_ops = n_vars >= 1 && (1ull << (n_vars - 1)) > POLY_SPLIT_MAX_PAIRS;
    std::vector<dpk::PolyOp> all_ops;
    u32 plain = 0, nested = 0;
    for (size_t g = 0; g < groups.size() && use_ops; g++) {
        std::vector<HornerTerm> ts;
        E2 root = gl::e2_zero();
        for (u32 ti = tb[g]; ti < te[g]; ti++) {
            const dpk::PolyTerm &pt = poly_terms[ti];
            HornerTerm ht;
            ht.coeff = gl::e2(pt.c0, pt.c1);
            ht.slots.assign(pt.slot, pt.slot + pt.n_factors);
            if (ht.slots.empty()) root = gl::add(root, ht.coeff);
            plain += pt.n_factors;  // n_factors - 1 products and one for the coefficient
            ts.push_back(std::move(ht));
        }
        std::vector<dpk::PolyOp> ops;
        dpk::PolyOp enter;
        memset(&enter, 0, sizeof enter);
        enter.c0 = root.c0;
        enter.c1 = root.c1;
        enter.code = dpk::POLY_OP_ENTER;
        ops.push_back(enter);
        nested += horner_build(std::move(ts), 0, ops);
        if (ops.size() > (size_t)dpk::POLY_LDS_OPS) use_ops = false;
        sc->poly_op_begin[g] = (u32)all_ops.size();
        all_ops.insert(all_ops.end(), ops.begin(), ops.end());
        sc->poly_op_end[g] = (u32)all_ops.size();
    }
    if (use_ops && nested < plain) {
        sc->h_poly_ops = all_ops;
    } else {
        sc->poly_op_begin.assign(groups.size(), 0);
        sc->poly_op_end.assign(groups.size(), 0);
    }
}

void SessionSetup::detect_multi_term()
{
    sc->poly = false;
    sc->poly_max_tabs = 0;
    sc->d_poly_groups = nullptr;
    sc->d_poly_terms = nullptr;
    if (sc->fast || sc->n_terms < 1 || n_vars < 1) return;
    if (!closed_form_eq_factor() || !group_terms()) return;
    adopt_groups();
    nested_programs();
}

int32_t SessionSetup::plan_and_ready_tables()
{
    // the last rounds run in one resident workgroup when every registered table belongs to the term
    // (from the round of 2^8 = TAIL_PAIRS pairs on, or from round 2 in a smaller sum; the tail kernel reads extension
    // tables, which every table is once folded, so a start in round 2 needs extension tables to begin with)
    // a product with an eq factor reads the eq weights of its large rounds as products of two small tables: the low ones are
    // built now if this eq table has not served such a session before (they lie behind its levels; the table itself is not touched)
    sc->round_kind.assign(n_vars + 2, 0);
    sc->round_wide.assign(n_vars + 2, 0);
    memset(sc->ctr_seen, 0, sizeof sc->ctr_seen);
    sc->last_trip_seq = 0;
    sc->fin_len = 0;
    sc->fin_pend = 0;
    sc->host_rounds = 0;
    sc->host_len = 0;
    sc->host_fresh = false;
    sc->host_state.clear();
    sc->prev_chal = gl::e2_zero();
    sc->slice_ids.clear();
    sc->slice_terms.clear();
    if (sc->fast && n_vars >= 3 && n_mles == sc->terms[0].n_factors) {
        sc->slice_ids.assign(sc->fast_order, sc->fast_order + sc->fast_nf);
        plan_resident_rounds(sc, sc->fast_nf, n_mles);
    }
    // A sum of several terms over full-size tables (a fraction-sum layer, a claim merge, the stacked products of an
    // einsum): the same launches.  One group of tables from the first round that fits; more tables than a group holds
    // (up to SL_MAX_TABS) when every round is resident, so that the groups' own launches are never needed.
    if (sc->poly && sc->fast_nf <= 4 && sc->n_terms <= (u32)dpk::SL_MAX_TERMS) {
        std::vector<u32> ids;
        for (const auto &g : sc->poly_tabs)
            for (u32 k : g)
                if (std::find(ids.begin(), ids.end(), k) == ids.end()) ids.push_back(k);
        bool ok = n_mles == ids.size() + (sc->fast_eq >= 0 ? 1 : 0) && ids.size() <= (size_t)dpk::SL_MAX_TABS;
        for (u32 k : ids) ok = ok && nv0[k] == n_vars && !mles[k]->pad_vars;
        if (ok) {
            sc->slice_ids = ids;
            for (const dps_term &t : sc->terms) {
                dpk::SliceTerm tm;
                memset(&tm, 0, sizeof tm);
                tm.c0 = t.coeff[0], tm.c1 = t.coeff[1], tm.w = gl::mul_small(t.coeff[1], (u32)gl::W);
                for (u32 f = 0; f < t.n_factors; f++)
                    if ((int)t.factors[f] != sc->fast_eq) tm.slot[tm.n_factors++] = (uint8_t)(std::find(ids.begin(), ids.end(), t.factors[f]) - ids.begin());
                sc->slice_terms.push_back(tm);
            }
            plan_resident_rounds(sc, (u32)ids.size(), n_mles);
            if (sc->poly_tabs.size() > 1 && sc->tail_j0 != 1) {
                // several groups and not every round resident: the groups' launches take the session
                sc->stages.clear();
                sc->tail_j0 = 0;
                sc->fin_len = 0;
                sc->host_rounds = 0;
                sc->round_kind.assign(n_vars + 2, 0);
                sc->round_wide.assign(n_vars + 2, 0);
            }
        }
    }
    // A small sum over tables the host has copies of (the small levels of fraction trees): every round is the host's.
    // A launch would take longer to start than the few hundred field products take here.
    sc->host_only = false;
    if (!sc->slice_ids.empty() && n_vars >= 1 && n_vars <= HOST_ONLY_MAX_VARS) {
        bool ok = true;
        for (u32 k : sc->slice_ids) {
            const dps_mle *t = mles[k];
            ok = ok && t->sh0 && ctx->logup_builds - t->sh_build < LOGUP_OUT_AREAS && t->len == (1ull << n_vars);
        }
        if (ok) {
            // the copies are there once the builds' last launches have published (the same wait as for a tree's outputs)
            u64 seen_seq[LOGUP_OUT_AREAS] = {};
            for (u32 k : sc->slice_ids) {
                const dps_mle *t = mles[k];
                if (seen_seq[t->sh_slot] == t->sh_seq) continue;
                u64 w[8];
                if (wait_result_at(ctx, logup_out_off(ctx, t->sh_slot), t->sh_seq, 0, 8, w, 9, 8) != DPS_OK) ok = false;
                seen_seq[t->sh_slot] = t->sh_seq;
            }
        }
        if (ok) {
            const u32 len = 1u << n_vars, n_tabs = (u32)sc->slice_ids.size();
            sc->host_state.resize((size_t)len * n_tabs);
            for (u32 f = 0; f < n_tabs; f++) {
                const dps_mle *t = mles[sc->slice_ids[f]];
                for (u32 i = 0; i < len; i++) sc->host_state[(size_t)f * len + i] = gl::e2(t->sh0[i], t->sh1[i]);
            }
            sc->host_len = len;
            sc->host_fresh = false;
            sc->host_only = true;
            sc->stages.clear();
            sc->tail_j0 = 0;
            sc->fin_len = 0;
            sc->fin_pend = 0;
            sc->host_rounds = n_vars;
            sc->round_kind.assign(n_vars + 2, 4);
            std::fill(sc->round_wide.begin(), sc->round_wide.end(), 0);
            sc->pairs_seq = 1;  // (dps_sc_finish: the last entries are with the host)
            return DPS_OK;      // nothing of any table is read on the device
        }
    }
    // What this session reads of its tables: an eq table taken in closed form is read level by level -- level j in round j,
    // except in the large rounds of a product, which take the low table of level j and level j + 16 instead -- and
    // anything else as ordinary entries.  Whatever of that an eq table has not built yet is built now, on the stream.
    for (u32 k = 0; k < n_mles; k++) {
        if ((int)k == sc->fast_eq) {
            u32 first_level = 1;
            if (sc->fast) {
                first_level = sc->eq_info->fact_levels + 1;
                if (sc->tail_j0) first_level = std::min(first_level, sc->tail_j0);
            } else if (sc->poly) {
                // the large rounds of a sum of several terms read level j + 16 and the low table of level j
                while (first_level <= n_vars && poly_round_weights_factored(sc, first_level)) first_level++;
            }
            const u64 need = ((2ull << n_vars) - 1) & ~((1ull << first_level) - 1);
            CHK(eq_ensure(ctx, *sc->eq_info, const_cast<u64 *>(sc->eq_c0), const_cast<u64 *>(sc->eq_c1), need, sc->fast));
        } else {
            CHK(plain_ready(mles[k]));
        }
    }

    return DPS_OK;
}

int32_t SessionSetup::layout_scratch()
{
    // scratch: two ping-pong buffers per table, extension limbs
    size_t scratch_words = 0;
    std::vector<size_t> off_a(n_mles), off_b(n_mles);
    // a zero-padded table keeps folding after it is down to one entry: both buffers hold at least that entry
    for (u32 k = 0; k < n_mles; k++) {
        u64 la = len_a(k), lb = len_b(k);
        off_a[k] = scratch_words;
        scratch_words += round_up(2 * la, 32);
        off_b[k] = scratch_words;
        scratch_words += round_up(2 * lb, 32);
    }
    if (scratch_words) CHK(pool_alloc(ctx, scratch_words * 8, &sc->scratch));
    u64 *sbase = (u64 *)sc->scratch;
    sc->m.resize(n_mles);
    for (u32 k = 0; k < n_mles; k++) {
        SessMle &s = sc->m[k];
        s.c0 = mles[k]->p0();
        s.c1 = mles[k]->p1();
        s.nv = nv0[k];
        s.zpad = zpad_of(k);
        u64 la = len_a(k), lb = len_b(k);
        s.buf0[0] = sbase ? sbase + off_a[k] : nullptr;
        s.buf1[0] = s.buf0[0] ? s.buf0[0] + la : nullptr;
        s.buf0[1] = sbase ? sbase + off_b[k] : nullptr;
        s.buf1[1] = s.buf0[1] ? s.buf0[1] + lb : nullptr;
        s.next = 0;
    }

    return DPS_OK;
}

// Step j starts by folding, with the challenge of round j - 1, the tables that were live-sized then; the product
// kernel's arguments of round j.
void SessionSetup::fold_step(u32 j)
{
    if (j >= 2) {
        u32 prev_live = n_vars - (j - 1) + 1;
        sc->fold_off[j] = (u32)folds.size();
        sc->fold_extra_off[j] = (u32)folds_extra.size();
        if (sc->fast && j <= n_vars) {
            dpk::ProdArgs &pa = sc->fast_args[j];
            memset(&pa, 0, sizeof pa);
            u32 nb = 0;
            for (u32 f = 0; f < sc->fast_nf; f++) {
                const SessMle &s = sim[sc->fast_order[f]];
                pa.s0[f] = s.c0;
                pa.s1[f] = s.c1;
                if (!s.c1) nb++;
                pa.d0[f] = s.buf0[s.next];
                pa.d1[f] = s.buf1[s.next];
            }
            pa.n_pairs = 1ull << (n_vars - j);
            sc->fast_nb[j] = nb;
        }
        for (u32 k = 0; k < n_mles; k++) {
            SessMle &s = sim[k];
            if ((int)k == sc->fast_eq) continue;
            if (s.zpad) {
                // depends on the low variables: folds in every step, and keeps folding against 0 once it is one entry
                const bool single = s.nv == 0;
                dpk::FoldDesc d{s.c0, s.c1, s.buf0[s.next], s.buf1[s.next], single ? 1ull : 1ull << (s.nv - 1), single ? 1ull : 0ull};
                folds.push_back(d);
                folds_extra.push_back(d);
                s.c0 = d.d0;
                s.c1 = d.d1;
                if (!single) s.nv -= 1;
                s.next ^= 1;
                continue;
            }
            if (s.nv != prev_live) continue;
            dpk::FoldDesc d{s.c0, s.c1, s.buf0[s.next], s.buf1[s.next], 1ull << (s.nv - 1), 0};
            folds.push_back(d);
            if (!in_fast(k) || j == n_vars + 1) folds_extra.push_back(d);
            pre0[k] = s.c0;
            pre1[k] = s.c1;
            folded[k] = 1;
            s.c0 = d.d0;
            s.c1 = d.d1;
            s.nv -= 1;
            s.next ^= 1;
        }
        sc->fold_cnt[j] = (u32)folds.size() - sc->fold_off[j];
        sc->fold_extra_cnt[j] = (u32)folds_extra.size() - sc->fold_extra_off[j];
    } else if (sc->fast) {
        dpk::ProdArgs &pa = sc->fast_args[1];
        memset(&pa, 0, sizeof pa);
        u32 nb = 0;
        for (u32 f = 0; f < sc->fast_nf; f++) {
            const SessMle &s = sim[sc->fast_order[f]];
            pa.s0[f] = s.c0;
            pa.s1[f] = s.c1;
            if (!s.c1) nb++;
        }
        pa.n_pairs = 1ull << (n_vars - 1);
        sc->fast_nb[1] = nb;
    }
}

void SessionSetup::poly_groups_of_round(u32 j)
{
    const u32 live = n_vars - j + 1;
    for (size_t g = 0; g < sc->poly_tabs.size(); g++) {
        dpk::PolyGroup pg;
        memset(&pg, 0, sizeof pg);
        pg.n_tabs = (u32)sc->poly_tabs[g].size();
        pg.term_begin = sc->poly_term_begin[g];
        pg.term_end = sc->poly_term_end[g];
        pg.op_begin = sc->poly_op_begin[g];
        pg.op_end = sc->poly_op_end[g];
        for (u32 sl = 0; sl < pg.n_tabs; sl++) {
            const u32 k = sc->poly_tabs[g][sl];
            const SessMle &s = sim[k];
            dpk::PolyTab &tb = pg.tab[sl];
            if (folded[k]) {
                // folds with the previous challenge on the way in; the owning group writes the result
                tb.mode = dpk::POLY_PAIR_FOLD;
                tb.s0 = pre0[k];
                tb.s1 = pre1[k];
                if (sc->poly_owner[k] == (int)g) {
                    tb.d0 = const_cast<u64 *>(s.c0);
                    tb.d1 = const_cast<u64 *>(s.c1);
                }
            } else if (s.nv >= live) {
                tb.mode = dpk::POLY_PAIR;
                tb.s0 = s.c0;
                tb.s1 = s.c1;
            } else {
                tb.mode = dpk::POLY_BCAST;
                tb.s0 = s.c0;
                tb.s1 = s.c1;
                tb.shift = live - 1 - s.nv;
            }
        }
        poly_groups.push_back(pg);
    }
}

void SessionSetup::term_descs_of_round(u32 j)
{
    u32 live = n_vars - j + 1;
    sc->term_off[j] = (u32)tdescs.size();
    for (const dps_term &t : sc->terms) {
        dpk::TermDesc td;
        memset(&td, 0, sizeof td);
        td.n_factors = t.n_factors;
        td.n_pairs = 1ull << (live - 1);
        for (u32 f = 0; f < t.n_factors; f++) {
            const SessMle &s = sim[t.factors[f]];
            td.f[f].c0 = s.c0;
            td.f[f].c1 = s.c1;
            if (s.zpad) {
                // non-zero only where the higher variables are 0: the first 2^(nv-1) pairs, or entry 0 against 0
                td.f[f].pair = s.nv >= 1 ? 1 : 2;
                td.f[f].shift = 0;
                td.n_pairs = std::min<u64>(td.n_pairs, s.nv >= 1 ? 1ull << (s.nv - 1) : 1ull);
            } else if (s.nv >= live) {
                td.f[f].pair = 1;
                td.f[f].shift = 0;
            } else {
                td.f[f].pair = 0;
                td.f[f].shift = live - 1 - s.nv;
            }
        }
        tdescs.push_back(td);
    }
}

// a dry run of the rounds: every descriptor the launches will need
void SessionSetup::describe_rounds()
{
    sim = sc->m;
    sc->fold_off.assign(n_vars + 2, 0);
    sc->fold_cnt.assign(n_vars + 2, 0);
    sc->fold_extra_off.assign(n_vars + 2, 0);
    sc->fold_extra_cnt.assign(n_vars + 2, 0);
    sc->term_off.assign(n_vars + 2, 0);
    sc->fast_args.resize(n_vars + 2);
    sc->fast_nb.assign(n_vars + 2, 0);
    pre0.assign(n_mles, nullptr), pre1.assign(n_mles, nullptr);
    folded.assign(n_mles, 0);
    for (u32 j = 1; j <= n_vars + 1; j++) {
        std::fill(folded.begin(), folded.end(), 0);
        fold_step(j);
        if (j <= n_vars && sc->poly) poly_groups_of_round(j);
        if (j <= n_vars && !sc->fast && !sc->poly) term_descs_of_round(j);
    }

    for (const dps_term &t : sc->terms) fins.push_back(dpk::FinTerm{t.coeff[0], t.coeff[1], t.n_factors, 0});

    for (u32 k = 0; k < n_mles; k++) gath.push_back(dpk::GatherDesc{sim[k].c0, sim[k].c1});
}

// grid sizes the session can ask for (its partials are sized for the largest), and how a pair's work is spread in small rounds
void SessionSetup::launch_limits()
{
    sc->max_blocks = n_vars >= 1 ? blocks_for_pairs(1ull << (n_vars - 1)) : 1;
    // (the launch of the first two rounds: 18 words a workgroup where the others have at most 16)
    if (sc->pair12) sc->max_blocks = std::max<u32>(sc->max_blocks, (PAIR12_BLOCKS * 2 * dpk::PAIR12_SUMS + 2 * dpk::MAX_PTS - 1) / (2 * dpk::MAX_PTS));
    for (const dps_sc::QuadStep &q : sc->quads) sc->max_blocks = std::max<u32>(sc->max_blocks, q.blocks);
    sc->poly_split_cap = 0;
    sc->poly_finish_in_kernel = false;
    if (sc->poly) {
        // every table is in a group (or is the closed-form eq): the resident launch can publish all final evaluations
        sc->poly_finish_in_kernel = true;
        for (u32 k = 0; k < n_mles; k++)
            if (sc->poly_owner[k] < 0 && (int)k != sc->fast_eq) sc->poly_finish_in_kernel = false;
        sc->poly_raw = false;
        // items of a pair: (evaluation point, term) products; tables to fold
        u32 most_terms = 0;
        for (size_t g = 0; g < sc->poly_tabs.size(); g++) most_terms = std::max(most_terms, sc->poly_term_end[g] - sc->poly_term_begin[g]);
        const u32 items = std::max<u32>(most_terms * std::max<u32>(sc->fast_nf, 1), sc->poly_max_tabs);
        sc->poly_split_cap = std::min<u32>(4, log2u(std::max<u32>(items, 1)));
        for (u32 j = 1; j <= n_vars; j++) {
            const u64 np = 1ull << (n_vars - j);
            if (np > POLY_SPLIT_MAX_PAIRS) continue;
            u32 sl, bl;
            poly_split_plan(np, sc->poly_split_cap, sc->poly_tabs.size() <= POLY_RAW_MAX_GROUPS, &sl, &bl);
            sc->max_blocks = std::max(sc->max_blocks, bl);
        }
    }
}

int32_t SessionSetup::allocate_device_block()
{
    bytes_fold = round_up(folds.size() * sizeof(dpk::FoldDesc), 256);
    bytes_fold_x = round_up(folds_extra.size() * sizeof(dpk::FoldDesc), 256);
    bytes_terms = round_up(tdescs.size() * sizeof(dpk::TermDesc), 256);
    bytes_fin = round_up(fins.size() * sizeof(dpk::FinTerm), 256);
    bytes_gath = round_up(gath.size() * sizeof(dpk::GatherDesc), 256);
    size_t bytes_partial = round_up((size_t)std::max<u32>(sc->n_terms, 1) * sc->max_blocks * 2 * dpk::MAX_PTS * 8, 256);
    size_t bytes_result = round_up((2 * dpk::MAX_PTS + 2 * (size_t)n_mles) * 8, 256) + 256;
    bytes_pg = round_up(poly_groups.size() * sizeof(dpk::PolyGroup), 256);
    bytes_pt = round_up(poly_terms.size() * sizeof(dpk::PolyTerm), 256);
    bytes_po = round_up(sc->h_poly_ops.size() * sizeof(dpk::PolyOp), 256);
    // what a resident stage that does not run to the last round leaves for the next: two limb arrays per table
    size_t bytes_hand = 0;
    const u32 slice_tabs = (u32)sc->slice_ids.size();
    for (size_t i = 0; i + 1 < sc->stages.size(); i++) bytes_hand += round_up((size_t)sc->stages[i + 1].src_len * 8, 256) * 2 * (slice_tabs + 1);
    size_t total = bytes_fold + bytes_fold_x + bytes_terms + bytes_fin + bytes_gath + bytes_pg + bytes_pt + bytes_po + bytes_partial + bytes_result + bytes_hand;
    CHK(pool_alloc(ctx, total, &sc->dev_block));
    char *p = (char *)sc->dev_block;
    sc->d_fold = (dpk::FoldDesc *)p;
    p += bytes_fold;
    sc->d_fold_extra = (dpk::FoldDesc *)p;
    p += bytes_fold_x;
    sc->d_terms = (dpk::TermDesc *)p;
    p += bytes_terms;
    sc->d_fin = (dpk::FinTerm *)p;
    p += bytes_fin;
    sc->d_gather = (dpk::GatherDesc *)p;
    p += bytes_gath;
    sc->d_poly_groups = (dpk::PolyGroup *)p;
    p += bytes_pg;
    sc->d_poly_terms = (dpk::PolyTerm *)p;
    p += bytes_pt;
    sc->d_poly_ops = (dpk::PolyOp *)p;
    p += bytes_po;
    sc->d_partial = (u64 *)p;
    p += bytes_partial;
    sc->d_result = (u64 *)p;
    p += bytes_result;
    for (size_t i = 0; i + 1 < sc->stages.size(); i++) {
        const size_t limb = round_up((size_t)sc->stages[i + 1].src_len * 8, 256);
        for (u32 f = 0; f <= slice_tabs; f++) {
            sc->stages[i].h0[f] = (u64 *)p;
            p += limb;
            sc->stages[i].h1[f] = (u64 *)p;
            p += limb;
        }
    }
    sc->d_counter = ctx->d_counter;
    return DPS_OK;
}

int32_t SessionSetup::stage_descriptors()
{
    // one staged upload of all descriptors
    std::vector<char> &stage = sc->stage;  // lives as long as the session: the upload is not waited for
    stage.assign(bytes_fold + bytes_fold_x + bytes_terms + bytes_fin + bytes_gath + bytes_pg + bytes_pt + bytes_po, 0);
    sc->h_poly_groups = poly_groups;
    sc->h_poly_terms = poly_terms;
    char *q = stage.data();
    if (!folds.empty()) memcpy(q, folds.data(), folds.size() * sizeof(dpk::FoldDesc));
    q += bytes_fold;
    if (!folds_extra.empty()) memcpy(q, folds_extra.data(), folds_extra.size() * sizeof(dpk::FoldDesc));
    q += bytes_fold_x;
    if (!tdescs.empty()) memcpy(q, tdescs.data(), tdescs.size() * sizeof(dpk::TermDesc));
    q += bytes_terms;
    if (!fins.empty()) memcpy(q, fins.data(), fins.size() * sizeof(dpk::FinTerm));
    q += bytes_fin;
    if (!gath.empty()) memcpy(q, gath.data(), gath.size() * sizeof(dpk::GatherDesc));
    q += bytes_gath;
    if (!poly_groups.empty()) memcpy(q, poly_groups.data(), poly_groups.size() * sizeof(dpk::PolyGroup));
    q += bytes_pg;
    if (!poly_terms.empty()) memcpy(q, poly_terms.data(), poly_terms.size() * sizeof(dpk::PolyTerm));
    q += bytes_pt;
    if (!sc->h_poly_ops.empty()) memcpy(q, sc->h_poly_ops.data(), sc->h_poly_ops.size() * sizeof(dpk::PolyOp));
    // Sessions whose launches carry their descriptors themselves (a product session that ends in the resident kernel; a
    // single group of terms, inline in the kernel arguments or staged in pinned memory for the resident launch) upload
    // nothing unless a step outside that flow needs the block (ensure_descs).
    sc->descs_uploaded = false;
    const bool self_contained = (sc->fast && sc->tail_j0) || sc->tail_j0 == 1 ||
                                (sc->poly && sc->poly_tabs.size() == 1 && sc->h_poly_terms.size() <= (size_t)dpk::POLY_LDS_TERMS);
    if (!self_contained) {
        CHK(ensure_descs(sc));
    }
    return DPS_OK;
}

// eq * f * g over two base-field tables, large enough for the factored eq weights: rounds 1 and 2 are one launch that
// reads the tables once and writes nothing (pair12_kernel), and round 3 reads them again and folds twice on its way in.
int32_t SessionSetup::plan_first_two_rounds()
{
    sc->pair12 = false;
    sc->quads.clear();
    if (!first_two_rounds_fit(sc, n_mles, sc->tail_j0)) return DPS_OK;
    // (what the static test stands for; the resident launch's plan has counted on it)
    if (sc->fast_nb[1] != 2 || !sc->eq_info->fact_built) return fail(ctx, DPS_ERR_STATE, "dps_sc_begin: the eq table's low tables are missing");
    sc->pair12 = true;
    dpk::ProdArgs &p3 = sc->fast_args[3];
    for (u32 f = 0; f < 2; f++) {
        p3.s0[f] = sc->fast_args[1].s0[f];
        p3.s1[f] = nullptr;
    }
    p3.two = 1;
    sc->fast_nb[3] = 2;
    // Rounds 3 .. tail_j0 - 1 in launches of two rounds each (what the resident launch's plan counted on when it took
    // two pending folds): the first reads the unfolded tables and writes the state of round 3 where round 3 would
    // have; each later one reads what the one before wrote and writes into the table's other scratch buffer.
    const u32 n_quad = quad_launches_fit(sc, n_mles, sc->tail_j0);
    for (u32 q = 0; q < n_quad; q++) {
        dps_sc::QuadStep st;
        memset(&st, 0, sizeof st);
        st.j = 3 + 2 * q;
        st.blocks = quad_blocks(1ull << (n_vars - st.j - 1));
        for (u32 f = 0; f < 2; f++) {
            const SessMle &m = sc->m[sc->fast_order[f]];
            const int into = q & 1 ? 0 : 1;  // round 3's state lies in the smaller buffer, as it always does
            st.d0[f] = m.buf0[into];
            st.d1[f] = m.buf1[into];
            st.s0[f] = q == 0 ? sc->fast_args[1].s0[f] : sc->quads[q - 1].d0[f];
            st.s1[f] = q == 0 ? nullptr : sc->quads[q - 1].d1[f];
        }
        sc->quads.push_back(st);
        sc->round_kind[st.j] = 5;
        sc->round_kind[st.j + 1] = 6;
    }
    return DPS_OK;
}

int32_t SessionSetup::run()
{
    detect_product();
    detect_multi_term();
    CHK(plan_and_ready_tables());
    CHK(layout_scratch());
    describe_rounds();
    CHK(plan_first_two_rounds());
    launch_limits();
    CHK(allocate_device_block());
    return stage_descriptors();
}

}  // namespace

extern "C" int32_t dps_sc_begin(dps_ctx *ctx, uint32_t n_vars, const dps_mle *const *mles, uint32_t n_mles,
                                const dps_term *terms, uint32_t n_terms, dps_sc **out)
{
    if (!ctx || !out || (n_mles && !mles) || (n_terms && !terms) || n_vars > 40)
        return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    std::unique_ptr<dps_sc> sc(new (std::nothrow) dps_sc());
    if (!sc) return fail(ctx, DPS_ERR_OOM, "host allocation failed");
    sc->ctx = ctx;
    sc->n_vars = n_vars;
    sc->n_mles = n_mles;
    sc->round = 0;
    sc->finished = false;
    sc->scratch = sc->dev_block = nullptr;
    sc->const_sum = gl::e2_zero();
    sc->degree = 0;
    SessionSetup su;
    su.ctx = ctx, su.sc = sc.get(), su.n_vars = n_vars, su.mles = mles, su.n_mles = n_mles;
    std::vector<u32> &nv0 = su.nv0;
    nv0.assign(n_mles, 0);
    for (u32 k = 0; k < n_mles; k++) {
        const dps_mle *t = mles[k];
        if (!t || t->ctx != ctx) return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: table %u belongs to another context", k);
        if (is_raw(t->kind) || !is_pow2(t->len)) return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: table %u is not a power-of-two field table", k);
        nv0[k] = log2u(t->len);
        if (nv0[k] > n_vars) return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: table %u has %u variables, the sum has %u", k, nv0[k], n_vars);
        if (t->pad_vars && t->pad_vars != n_vars)
            return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: table %u is zero-padded to %u variables, the sum has %u", k, t->pad_vars, n_vars);
        sc->keep.push_back(t->st);
    }
    for (u32 i = 0; i < n_terms; i++) {
        const dps_term &t = terms[i];
        if (!canonical(t.coeff, 2)) return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: coefficient of term %u not canonical", i);
        if (t.n_factors > DPS_MAX_FACTORS) return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: term %u has %u factors", i, t.n_factors);
        if (t.n_factors > DPS_MAX_DEGREE) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_sc_begin: degree %u above %d", t.n_factors, DPS_MAX_DEGREE);
        for (u32 f = 0; f < t.n_factors; f++)
            if (t.factors[f] >= n_mles) return fail(ctx, DPS_ERR_INVALID, "dps_sc_begin: term %u names table %u", i, t.factors[f]);
        if (t.n_factors == 0) {
            sc->const_sum = gl::add(sc->const_sum, gl::e2(t.coeff[0], t.coeff[1]));
        } else {
            sc->terms.push_back(t);
            sc->degree = std::max(sc->degree, t.n_factors);
        }
    }
    sc->n_terms = (u32)sc->terms.size();

    if (const int32_t rc = su.run(); rc != DPS_OK) {
        pool_free(ctx, sc->scratch);
        pool_free(ctx, sc->dev_block);
        return rc;
    }
    *out = sc.release();
    return DPS_OK;
}

extern "C" int32_t dps_sc_set_claim(dps_sc *sc, const uint64_t *claim)
{
    if (!sc || !claim) return DPS_ERR_INVALID;
    dps_ctx *ctx = sc->ctx;
    if (sc->round != 0 || sc->finished) return fail(ctx, DPS_ERR_STATE, "dps_sc_set_claim: the session has started");
    if (!canonical(claim, 2)) return fail(ctx, DPS_ERR_INVALID, "dps_sc_set_claim: claim not canonical");
    sc->claim = gl::e2(claim[0], claim[1]);
    sc->have_claim = true;
    return DPS_OK;
}

extern "C" int32_t dps_sc_degree(const dps_sc *sc, uint32_t *degree)
{
    if (!sc || !degree) return DPS_ERR_INVALID;
    *degree = sc->degree;
    return DPS_OK;
}

namespace {

int32_t launch_folds(dps_sc *sc, u32 step, bool extra_only, const u64 *chal)
{
    dps_ctx *ctx = sc->ctx;
    u32 cnt = extra_only ? sc->fold_extra_cnt[step] : sc->fold_cnt[step];
    if (!cnt) return DPS_OK;
    CHK(ensure_descs(sc));
    const dpk::FoldDesc *d = extra_only ? sc->d_fold_extra + sc->fold_extra_off[step] : sc->d_fold + sc->fold_off[step];
    // the grid is sized for the largest table that can fold in this step; smaller (zero-padded) ones leave blocks idle
    u32 prev_live = sc->n_vars - (step - 1) + 1;
    u64 half = 1ull << (prev_live - 1);
    for (u32 base = 0; base < cnt; base += 65535) {
        u32 n = std::min<u32>(cnt - base, 65535);
        ProfScope ps(ctx, DPS_K_FOLD, (double)n * (double)half * 48.0);
        dpk::fold_kernel<<<dim3(grid_for(half), n), dpk::BLOCK, 0, ctx->stream>>>(d + base, chal[0], chal[1]);
        HIPCHK(ctx, hipGetLastError());
    }
    return DPS_OK;
}

}  // namespace

namespace {

// Wait until the launch that carries `seq` has published its `n` result words
// (at slot0 of the result area) and copy them out.  The host polls the sequence
// word; the words are accepted once the check word agrees with them, since the
// kernel's stores may land in any order.  If the result does not arrive the
// stream is queried to surface the error.
int32_t wait_result(dps_ctx *ctx, u64 seq, u32 slot0, u32 n, u64 *out) { return wait_result_at(ctx, ctx->res_off, seq, slot0, n, out); }

// the same hand-off in another 64-word area of the pinned buffer
int32_t wait_result_at(dps_ctx *ctx, size_t base_off, u64 seq, u32 slot0, u32 n, u64 *out, int seq_slot, int chk_slot)
{
    volatile u64 *base = ctx->h_pinned + base_off;
    volatile u64 *flag = base + seq_slot;
    auto take = [&]() {
        if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) != seq) return false;
        u64 chk = seq;
        for (u32 i = 0; i < n; i++) {
            out[i] = base[slot0 + i];
            chk ^= dpk::rotl64(out[i], i + 1);
        }
        return chk == base[chk_slot];
    };
    for (u64 spins = 0;; spins++) {
        if (take()) return DPS_OK;
        if ((spins & 0xFFFFF) == 0xFFFFF) {
            // about once per several milliseconds: has the stream died or finished without publishing?
            hipError_t q = hipStreamQuery(ctx->stream);
            if (q == hipSuccess) {
                if (take()) return DPS_OK;
                return fail(ctx, DPS_ERR_HIP, "round result was not published");
            }
            if (q != hipErrorNotReady) return fail(ctx, DPS_ERR_HIP, "stream error while waiting for a round: %s", hipGetErrorString(q));
        }
    }
}

// The sums of a trip of a resident launch: the four counters of each of `n_sums` sums, one word each at the start of the
// launch's result area, whole once it carries the trip's tag (dpk::sl_tag) in its top byte.  `skip1`: the counters of
// q(1) do not come (zeros are returned for them).  The tags are cleared as the words are taken, so that a word of 128
// trips ago cannot pass for this trip's.
int32_t wait_slice_sums(dps_ctx *ctx, u64 seq, u32 n_sums, bool skip1, u32 n_sets, u64 *out)
{
    volatile u64 *area = ctx->h_pinned + slice_area_off(ctx);
    const u64 tag = dpk::sl_tag(seq);
    u32 c = 0, set = 0;
    const u32 n = 4 * n_sums;
    // (set by set: `out` holds SL_GROUP_WORDS words per set)
    auto take = [&]() {
        for (; set < n_sets; set++, c = 0) {
            volatile u64 *base = area + (size_t)set * dpk::SL_GROUP_WORDS;
            u64 *o = out + (size_t)set * dpk::SL_GROUP_WORDS;
            for (; c < n; c++) {
                if (skip1 && c >= 4 && c < 8) {
                    o[c] = 0;
                    continue;
                }
                const u64 v = __atomic_load_n(base + c, __ATOMIC_ACQUIRE);
                if ((v >> 56) != tag) return false;
                o[c] = v & dpk::SL_CTR_MASK;
                base[c] = 0;
            }
        }
        return true;
    };
    for (u64 spins = 0;; spins++) {
        if (take()) return DPS_OK;
        if ((spins & 0xFFFFF) == 0xFFFFF) {
            hipError_t q = hipStreamQuery(ctx->stream);
            if (q == hipSuccess) {
                if (take()) return DPS_OK;
                // what the launch left behind, for whoever reads the message: how many workgroups had added to the first
                // counter of every set, and the number of the last mail in every copy the first workgroup passes on
                std::string left;
                {
                    std::vector<u64> words(SLICE_CTR_WORDS), relay(dpk::MAIL_RELAY_WORDS);
                    if (hipMemcpy(words.data(), ctx->d_slice_ctr, words.size() * 8, hipMemcpyDeviceToHost) == hipSuccess &&
                        hipMemcpy(relay.data(), mail_relay(ctx), relay.size() * 8, hipMemcpyDeviceToHost) == hipSuccess) {
                        left = "; adds per set:";
                        for (u32 g = 0; g < n_sets; g++) left += " " + std::to_string(words[(size_t)g * dpk::SL_GROUP_WORDS * dpk::SL_CTR_STRIDE] >> 56);
                        left += "; mail numbers passed on:";
                        for (u32 k = 0; k < dpk::MAIL_RELAY_COPIES; k++) left += " " + std::to_string(relay[(size_t)k * dpk::MAIL_RELAY_STRIDE + dpk::MAIL_SEQ]);
                        left += "; waited for " + std::to_string(seq) + ", set " + std::to_string(set) + " word " + std::to_string(c);
                        left += "; mailbox " + std::to_string(mailbox(ctx)[dpk::MAIL_SEQ]);
                        left += "; the first workgroup waited for " + std::to_string(area[dpk::SL_WAITING_SLOT]) + " and had " + std::to_string(area[dpk::SL_HAD_SLOT]);
                        left += "; tags in the area:";
                        for (u32 g = 0; g < n_sets; g++) left += " " + std::to_string(area[(size_t)g * dpk::SL_GROUP_WORDS] >> 56);
                    } else {
                        (void)hipGetLastError();
                    }
                }
                return fail(ctx, DPS_ERR_HIP, "round result was not published%s", left.c_str());
            }
            if (q != hipErrorNotReady) return fail(ctx, DPS_ERR_HIP, "stream error while waiting for a round: %s", hipGetErrorString(q));
        }
    }
}

// the area of dpk::SL_FIN_AREA_WORDS words where a resident launch leaves the tables' entries with its last trip
size_t slice_fin_off(const dps_ctx *ctx) { return ctx->pinned_words / 2 + 4096; }

// ... and those entries, `n` words published under the sequence number of that trip
int32_t wait_slice_entries(dps_ctx *ctx, u64 seq, u32 n, u64 *out)
{
    volatile u64 *base = ctx->h_pinned + slice_fin_off(ctx);
    auto take = [&]() {
        if (__atomic_load_n(base + dpk::SL_FIN_SEQ_SLOT, __ATOMIC_ACQUIRE) != seq) return false;
        u64 chk = seq;
        for (u32 i = 0; i < n; i++) {
            out[i] = base[i];
            chk ^= dpk::sl_fin_mix(out[i], i);
        }
        return chk == base[dpk::SL_FIN_CHK_SLOT];
    };
    for (u64 spins = 0;; spins++) {
        if (take()) return DPS_OK;
        if ((spins & 0xFFFFF) == 0xFFFFF) {
            hipError_t q = hipStreamQuery(ctx->stream);
            if (q == hipSuccess) {
                if (take()) return DPS_OK;
                return fail(ctx, DPS_ERR_HIP, "the tables' last entries were not published");
            }
            if (q != hipErrorNotReady) return fail(ctx, DPS_ERR_HIP, "stream error while waiting for a round: %s", hipGetErrorString(q));
        }
    }
}

// The end of a session whose resident launch has left (slice_kernel, with its last trip): the state of that trip's
// first round comes over with the trip (host_tail_load, in the same call: no other session's launch can overwrite the
// area in between), is folded with the challenges drawn since, and from then on the host holds the tables.
int32_t host_tail_load(dps_sc *sc, u64 seq)
{
    const u32 n_tabs = (u32)sc->slice_ids.size(), L = sc->fin_len;
    std::vector<u64> w(2 * (size_t)L * n_tabs);
    CHK(wait_slice_entries(sc->ctx, seq, (u32)w.size(), w.data()));
    sc->host_state.resize((size_t)L * n_tabs);
    for (size_t i = 0; i < sc->host_state.size(); i++) sc->host_state[i] = gl::e2(w[2 * i], w[2 * i + 1]);
    sc->host_len = L;
    sc->host_fresh = true;
    return DPS_OK;
}

// `r`: the challenge the call in hand brought (sc->prev_chal: the one before it)
void host_tail_advance(dps_sc *sc, E2 r)
{
    const u32 n_tabs = (u32)sc->slice_ids.size();
    auto fold_all = [&](E2 c) {
        const u32 half = sc->host_len / 2;
        for (u32 f = 0; f < n_tabs; f++) {
            const E2 *src = sc->host_state.data() + (size_t)f * sc->host_len;
            E2 *dst = sc->host_state.data() + (size_t)f * half;  // (in place: a new entry lies before the old ones still to be read)
            for (u32 i = 0; i < half; i++) {
                const E2 lo = src[2 * i], hi = src[2 * i + 1];
                dst[i] = gl::add(lo, gl::mul(c, gl::sub(hi, lo)));
            }
        }
        sc->host_len = half;
    };
    // the last trip covered two rounds: the challenge between them first
    if (sc->host_fresh && sc->fin_pend == 2) fold_all(sc->prev_chal);
    sc->host_fresh = false;
    fold_all(r);
}

// The sums q(t), t = 0 .. nf, of a round on the tables the host holds (q(1) left out when it comes from the claim):
// what slice_kernel adds up, by the definition.
void host_tail_sums(dps_sc *sc, u32 j, u32 nf, bool skip1, E2 *q)
{
    const u32 n_tabs = (u32)sc->slice_ids.size();
    const u32 len = sc->host_len, n_pairs = len / 2;
    const bool has_eq = sc->fast_eq >= 0;
    // eq(rho_{j+1..n}, x) over the pairs: variable j + 1 is the lowest bit of the pair's index
    std::vector<E2> weight(n_pairs, gl::e2_one());
    if (has_eq) {
        u32 have = 1;
        for (u32 i = j + 1; i <= sc->n_vars; i++) {
            const E2 rho = sc->eq_info->point[i - 1], one_minus = gl::sub(gl::e2_one(), rho);
            for (u32 x = 0; x < have; x++) {
                weight[x + have] = gl::mul(weight[x], rho);
                weight[x] = gl::mul(weight[x], one_minus);
            }
            have *= 2;
        }
    }
    for (u32 t = 0; t <= nf; t++) q[t] = gl::e2_zero();
    E2 val[dpk::SL_MAX_TABS];
    for (u32 p = 0; p < n_pairs; p++) {
        E2 lo[dpk::SL_MAX_TABS], d[dpk::SL_MAX_TABS];
        for (u32 f = 0; f < n_tabs; f++) {
            lo[f] = sc->host_state[(size_t)f * len + 2 * p];
            d[f] = gl::sub(sc->host_state[(size_t)f * len + 2 * p + 1], lo[f]);
            val[f] = lo[f];
        }
        for (u32 t = 0; t <= nf; t++) {
            if (t > 0)
                for (u32 f = 0; f < n_tabs; f++) val[f] = gl::add(val[f], d[f]);
            if (t == 1 && skip1) continue;
            E2 g;
            if (sc->poly) {
                g = gl::e2_zero();
                for (const dpk::SliceTerm &tm : sc->slice_terms) {
                    E2 prod = gl::e2(tm.c0, tm.c1);
                    for (u32 k = 0; k < tm.n_factors; k++) prod = gl::mul(prod, val[tm.slot[k]]);
                    g = gl::add(g, prod);
                }
            } else {
                g = val[0];
                for (u32 f = 1; f < n_tabs; f++) g = gl::mul(g, val[f]);
            }
            q[t] = gl::add(q[t], has_eq ? gl::mul(g, weight[p]) : g);
        }
    }
}

}  // namespace

namespace {

// One round of a session on the fused kernels -- a product of full-size tables, or sums of several terms over shared
// tables: what the ways a round can run have in common (the launch arguments, the mail, the message formed on the host
// from the sums a kernel hands over), and one function per way: a trip of a resident launch, a multi-term launch, a
// product launch.
struct FusedRound {
    dps_sc *sc;
    dps_ctx *ctx;
    u32 j;
    const uint64_t *challenge;
    uint64_t *evals_out;
    u64 n_pairs;
    u32 blocks;
    E2 cst;            // the constant terms' share of every evaluation
    dpk::FinArgs fa;   // (its sequence number and result area)
    dpk::ProdArgs a;
    dpk::FastFin ff;
    bool has_eq;
    u32 nf;
    E2 base_scale, s1;
    bool skip1;
    // the kernels hand over the sums q(t); the message is formed from them here (take_sums)
    struct {
        u64 scale[2 * dpk::MAX_PTS];  // p(t) = scale(t) q(t) + const, t = 0..nf
        u64 cext[2 * dpk::MAX_PTS];   // eq factor: p(nf + 1) = sum_i cext_i q(i) + k + const
        u64 k0, k1;
    } hf;
    // sums of several terms: groups of tables, and whether the single group's descriptors travel in the kernel arguments
    u32 n_groups;
    bool inline_descs;
    // What a launch for round jj looks like: the kernel, its grid, whether it stays for the later rounds.
    // Nothing here depends on a challenge, so a launch can be planned (and made) before its round begins.
    struct Plan {
        bool split, reside;
        u32 split_log, blocks;
        u64 n_pairs;
    };

    int32_t begin();
    void set_eq_weights(dpk::ProdArgs &pa, u32 jj, u32 blocks_jj) const;
    void prepare_message();
    void post_mail();
    void form_message(const E2 *q);
    int32_t take_sums(u32 n_slots);
    int32_t end_waiting_launch();
    bool admit_stages();
    int32_t launch_stages_at(u64 seq0, u32 first_go = 0);
    int32_t resident_round();
    Plan plan_round(u32 jj, bool skip1_jj) const;
    int32_t launch_round(u32 jj, const Plan &p, bool skip1_jj, bool ahead, u64 seq_jj);
    u32 slots_of(const Plan &p) const { return p.reside ? (n_groups > 1 ? n_groups : 0) : slots_for(p.blocks * n_groups); }
    int32_t multi_term_round();
    int32_t product_launch_ahead(u32 ahead = 1);
    int32_t product_round();
    int32_t first_two_rounds_launch();
    int32_t second_round_from_stash();
    const dps_sc::QuadStep *quad_at(u32 jj) const;
    int32_t launch_quad(const dps_sc::QuadStep &q, bool ahead, u64 seq_q);
    int32_t quad_first_round();
    int32_t quad_second_round();
    int32_t catch_up_after_quads();
};


// The arguments every way of running the round shares; ends a launch that waits on the GPU but cannot take this round.
int32_t FusedRound::begin()
{
    a = sc->fast_args[j];
    has_eq = sc->fast_eq >= 0;
    nf = sc->fast_nf;
    n_groups = sc->poly ? (u32)sc->poly_tabs.size() : 0;
    inline_descs = n_groups == 1 && sc->h_poly_terms.size() <= (size_t)dpk::POLY_LDS_TERMS;
    memset(&ff, 0, sizeof ff);
    memset(&hf, 0, sizeof hf);
    if (j >= 2) {
        const E2 r = gl::e2(challenge[0], challenge[1]);
        a.r0 = r.c0;
        a.r1 = r.c1;
        a.ra0 = sc->prev_chal.c0;
        a.ra1 = sc->prev_chal.c1;
        CHK(launch_folds(sc, j, true, challenge));
        if (has_eq) sc->eq_scalar = gl::mul(sc->eq_scalar, h_eq1(sc->eq_info->point[j - 2], r));
    }
    // scale(t) = coeff * S * eq1(rho_{j-1}, t).  Only whether scale(1) vanishes matters to the kernel (it then has to
    // evaluate t = 1); everything else about the message is worked out while the kernel runs (prepare_message).
    base_scale = sc->fast_coeff;
    if (has_eq) base_scale = gl::mul(base_scale, sc->eq_scalar);
    s1 = has_eq ? gl::mul(base_scale, h_eq1(sc->eq_info->point[j - 1], gl::e2_one())) : base_scale;
    skip1 = (j >= 2 || sc->have_claim) && !(s1.c0 == 0 && s1.c1 == 0);
    a.skip1 = skip1 ? 1 : 0;
    if (has_eq) set_eq_weights(a, j, blocks);
    ff.partial = sc->d_partial;
    ff.n_blocks = blocks;
    ff.out_host = fa.out_host;
    ff.seq = fa.seq;
    ff.counter = sc->d_counter;
    if (sc->tail_running && !sc->wait_any_skip1 && ((a.skip1 != 0) != sc->wait_skip1)) CHK(end_waiting_launch());
    if (sc->tail_running && sc->wait_fresh &&
        std::chrono::steady_clock::now() - sc->ahead_at > std::chrono::milliseconds(POLY_AHEAD_PATIENCE_MS))
        CHK(end_waiting_launch());
    return DPS_OK;
}

// where round jj finds its eq weights: level jj, or for the large rounds of a product (a grid whose stride is a
// multiple of the low table's size) the low table of level jj and level jj + 16
void FusedRound::set_eq_weights(dpk::ProdArgs &pa, u32 jj, u32 blocks_jj) const
{
        const u64 off = eq_level_off(sc->n_vars, jj);
        pa.q0 = sc->eq_c0 + off;
        pa.q1 = sc->eq_c1 + off;
        if (sc->fast && sc->eq_info->fact_built && jj <= sc->eq_info->fact_levels && ((u64)blocks_jj * dpk::BLOCK) % (1ull << dpk::EQ_LO_BITS) == 0) {
            const u64 lo = eq_low_off(sc->n_vars, jj), hi = eq_level_off(sc->n_vars, jj + dpk::EQ_LO_BITS);
            pa.lq0 = sc->eq_c0 + lo;
            pa.lq1 = sc->eq_c1 + lo;
            pa.hq0 = sc->eq_c0 + hi;
            pa.hq1 = sc->eq_c1 + hi;
        }
}

// scale(t), the claim and the extrapolation coefficients of this round's message: worked out while the kernel runs
void FusedRound::prepare_message()
{
        if (j >= 2) {
            // claim of this round: the previous message at the challenge (Lagrange over 0..degree)
            const E2 r = gl::e2(challenge[0], challenge[1]);
            const u32 d = sc->degree;
            E2 acc = gl::e2_zero();
            for (u32 k = 0; k <= d; k++) {
                E2 num = gl::e2_one();
                for (u32 m = 0; m <= d; m++)
                    if (m != k) num = gl::mul(num, gl::sub(r, gl::e2(m, 0)));
                acc = gl::add(acc, gl::mul(gl::mul_base(num, ctx->h_inv_den[d][k]), sc->last_msg[k]));
            }
            sc->claim = acc;
        }
        for (u32 t = 0; t <= sc->degree; t++) {
            E2 sc_t = has_eq ? gl::mul(base_scale, h_eq1(sc->eq_info->point[j - 1], gl::e2(t, 0))) : base_scale;
            hf.scale[2 * t] = sc_t.c0;
            hf.scale[2 * t + 1] = sc_t.c1;
        }
        if (has_eq) {
            // p(nf + 1) = sum_i cext_i q(i) + k + const
            const E2 s_top = gl::e2(hf.scale[2 * (nf + 1)], hf.scale[2 * (nf + 1) + 1]);
            E2 cext[dpk::MAX_PTS];
            for (u32 i = 0; i <= nf; i++) cext[i] = gl::mul_base(s_top, ctx->h_lagrange[(nf * 9 + (nf + 1)) * 9 + i]);
            if (skip1) {
                // q(1) = (claim - 2 const - scale(0) q(0)) / scale(1)
                const E2 A = gl::mul(cext[1], h_e2_inv(s1));
                cext[0] = gl::sub(cext[0], gl::mul(A, gl::e2(hf.scale[0], hf.scale[1])));
                const E2 kk = gl::mul(A, gl::sub(sc->claim, gl::add(cst, cst)));
                hf.k0 = kk.c0;
                hf.k1 = kk.c1;
                cext[1] = gl::e2_zero();
            }
            for (u32 i = 0; i <= nf; i++) {
                hf.cext[2 * i] = cext[i].c0;
                hf.cext[2 * i + 1] = cext[i].c1;
            }
        }
}

// mail for a kernel that waits on the GPU: challenge, whether t = 1 is skipped; then the sequence number it waits for
void FusedRound::post_mail()
{
        u64 *mb = mailbox(ctx);
        mb[dpk::MAIL_R] = a.r0;
        mb[dpk::MAIL_R + 1] = a.r1;
        mb[dpk::MAIL_RA] = sc->prev_chal.c0;
        mb[dpk::MAIL_RA + 1] = sc->prev_chal.c1;
        mb[dpk::MAIL_SKIP1] = a.skip1;
        send_mail(ctx, fa.seq);
}

// the message from the sums q(0..nf) (prepare_message has run): p(t) = scale(t) q(t) + const; p(1) from the claim when t = 1 was
// skipped; with an eq factor p(nf + 1) by extrapolation of q
void FusedRound::form_message(const E2 *q)
{
        const u32 np = nf + 1;
        E2 msg[dpk::MAX_PTS + 1];
        for (u32 t = 0; t < np; t++) msg[t] = gl::add(gl::mul(gl::e2(hf.scale[2 * t], hf.scale[2 * t + 1]), q[t]), cst);
        if (a.skip1) msg[1] = gl::sub(sc->claim, msg[0]);
        if (has_eq) {
            E2 e = gl::add(gl::e2(hf.k0, hf.k1), cst);
            for (u32 i = 0; i < np; i++)
                if (!(a.skip1 && i == 1)) e = gl::add(e, gl::mul(gl::e2(hf.cext[2 * i], hf.cext[2 * i + 1]), q[i]));
            msg[np] = e;
        }
        sc->last_msg.resize(sc->degree + 1);
        for (u32 t = 0; t <= sc->degree; t++) {
            evals_out[2 * t] = msg[t].c0;
            evals_out[2 * t + 1] = msg[t].c1;
            sc->last_msg[t] = msg[t];
        }
}

// Waits for the sums q(t), t = 0..nf, of this round (one set in the main result area, or n_slots sets in areas of their own --
// resident groups, or the workgroups of a small launch -- which are added) and forms the message.
int32_t FusedRound::take_sums(u32 n_slots)
{
        prepare_message();
        const u32 np = nf + 1;
        E2 q[dpk::MAX_PTS];
        u64 w[2 * dpk::MAX_PTS];
        if (n_slots) {
            for (u32 t = 0; t < np; t++) q[t] = gl::e2_zero();
            for (u32 g = 0; g < n_slots; g++) {
                CHK(wait_result_at(ctx, poly_raw_off(ctx) + 64 * (size_t)g, fa.seq, 0, 2 * np, w));
                // (the groups publish within a microsecond or two of each other, and every area read is a miss in the host's
                // caches -- the device has just written it: once the first is there the others are asked for together)
                if (g == 0)
                    for (u32 h = 1; h < n_slots; h++) {
                        const u64 *area = ctx->h_pinned + poly_raw_off(ctx) + 64 * (size_t)h;
                        __builtin_prefetch(area);
                        __builtin_prefetch(area + 8);
                    }
                for (u32 t = 0; t < np; t++) q[t] = gl::add(q[t], gl::e2(w[2 * t], w[2 * t + 1]));
            }
        } else {
            CHK(wait_result(ctx, fa.seq, 0, 2 * np, w));
            for (u32 t = 0; t < np; t++) q[t] = gl::e2(w[2 * t], w[2 * t + 1]);
        }
        form_message(q);
        return DPS_OK;
}

// A launch that takes this round may already be on the GPU, waiting for the mail: a resident one from an earlier
// round, or one made ahead during the previous round.  It cannot be used when it was compiled for the other way
// of getting p(1) (wait_any_skip1: the tail kernel, which takes either), or when it has had no mail yet and the
// caller took its time: it may have given up waiting (it polls for much longer than the limit here, so up to
// that limit it certainly has not).  Then it is ended and the round is launched normally.
int32_t FusedRound::end_waiting_launch()
{
        __atomic_store_n(mailbox(ctx) + dpk::MAIL_SEQ, dpk::MAIL_ABORT_SEQ, __ATOMIC_RELEASE);
        HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
        __atomic_store_n(mailbox(ctx) + dpk::MAIL_SEQ, (u64)0, __ATOMIC_RELEASE);
        reset_device_words(ctx);
        clear_resident_results(ctx);
        sc->tail_running = false;
        sc->wait_fresh = false;
        waiting_launch_over(ctx);
        return DPS_OK;
}

// The session's resident launches ask for their place on the device: the widest stage's workgroups, which hold a
// compute unit each and all have to be there at once.
bool FusedRound::admit_stages()
{
        u32 widest = 1;
        for (const dps_sc::Stage &st : sc->stages) {
            widest = std::max(widest, st.W);
            if (slice_workgroups_per_cu(ctx, sc->poly, sc->fast_nf, sc->fast_eq >= 0, (u32)sc->slice_ids.size(), st.cap) < 1) return false;
        }
        return admit_waiting_launch(ctx, widest, true);
}

// The launches of the resident rounds, queued one behind the other: the trip that starts at the first resident
// round has the sequence number seq0 (a round's call takes one number whether or not it makes a trip).
int32_t FusedRound::launch_stages_at(u64 seq0, u32 first_go)
{
        const u32 first = sc->tail_j0;
        // No resident launch of this context is running now: whatever an abandoned one left in the result area goes -- before
        // the launch is made, which may start its first trip at once (first_go) and publish while this thread is still here.
        memset(sc->ctr_seen, 0, sizeof sc->ctr_seen);
        for (u32 c = 0; c < dpk::SL_MAX_GROUPS * (u32)dpk::SL_GROUP_WORDS; c++) ctx->h_pinned[slice_area_off(ctx) + c] = 0;
        for (size_t si = 0; si < sc->stages.size(); si++) {
            const dps_sc::Stage &st = sc->stages[si];
            // a stage of several workgroups and the single-workgroup stage that runs to the last round are one launch:
            // the first workgroup takes the others' entries up and goes on alone
            const bool merged = st.W > 1 && si + 2 == sc->stages.size() && sc->stages[si + 1].W == 1 && sc->stages[si + 1].cap <= st.cap;
            const size_t last_si = merged ? si + 1 : si;
            dpk::SliceArgs sa;
            memset(&sa, 0, sizeof sa);
            const u32 n_tabs = (u32)sc->slice_ids.size();
            for (u32 f = 0; f < n_tabs; f++) {
                // the first stage reads what the launch of the round before it wrote (or the session's own tables)
                if (si > 0) {
                    sa.s0[f] = sc->stages[si - 1].h0[f];
                    sa.s1[f] = sc->stages[si - 1].h1[f];
                } else if (sc->poly && first == 1) {
                    sa.s0[f] = sc->m[sc->slice_ids[f]].c0;
                    sa.s1[f] = sc->m[sc->slice_ids[f]].c1;
                } else if (sc->poly) {
                    const dpk::PolyTab &tb = sc->h_poly_groups[first - 1].tab[f];
                    sa.s0[f] = tb.s0;
                    sa.s1[f] = tb.s1;
                } else if (!sc->quads.empty()) {
                    // the state of two rounds ago, as the last launch of two rounds left it
                    sa.s0[f] = sc->quads.back().d0[f];
                    sa.s1[f] = sc->quads.back().d1[f];
                } else {
                    sa.s0[f] = sc->fast_args[first].s0[f];
                    sa.s1[f] = sc->fast_args[first].s1[f];
                }
                sa.h0[f] = st.h0[f];
                sa.h1[f] = st.h1[f];
            }
            // (the eq weights of the workgroups go where one more table would)
            sa.hw0 = st.h0[n_tabs];
            sa.hw1 = st.h1[n_tabs];
            sa.n_tabs = n_tabs;
            if (sc->poly) {
                sa.n_terms = (u32)sc->slice_terms.size();
                std::copy(sc->slice_terms.begin(), sc->slice_terms.end(), sa.terms);
            }
            sa.src_len = st.src_len;
            sa.pend0 = st.pend0;
            sa.n_vars = sc->n_vars;
            sa.j0 = st.j0;
            sa.n_trips = st.n_trips;
            sa.dbl_mask = st.dbl_mask;
            if (merged) {
                sa.n_trips2 = sc->stages[si + 1].n_trips;
                sa.dbl_mask2 = sc->stages[si + 1].dbl_mask;
            }
            sa.eq0 = sc->eq_c0;
            sa.eq1 = sc->eq_c1;
            sa.mail = ctx->d_pinned + (ctx->res_off - 64);
            // (several workgroups: the first polls the host's mailbox and passes each mail on through device memory; with
            // all 256 of them polling host memory a trip took 90 us instead of 18)
            sa.relay = mail_relay(ctx);
            sa.spin_limit = wait_units(ctx, 4000000);  // ten seconds, then the kernel gives up
            sa.finish = last_si + 1 == sc->stages.size() ? 1 : 0;
            sa.first_go = si == 0 && st.pend0 == 0 && st.j0 == 1 ? first_go : 0;
            sa.out_host = ctx->d_pinned + slice_area_off(ctx);
            sa.fin_out = ctx->d_pinned + slice_fin_off(ctx);
            sa.seq0 = seq0 + (st.j0 - first);
            sa.ctr = ctx->d_slice_ctr;
            sa.gate = reinterpret_cast<u32 *>(ctx->d_slice_ctr + SLICE_CTR_WORDS);
            sa.groups_log = slice_counter_sets_log(st.W);
            ProfScope ps(ctx, DPS_K_TAIL, 0.0);
            CHK(launch_slice_dispatch(ctx, sc->poly, nf, has_eq, st.W, n_tabs, st.cap, sa));
            HIPCHK(ctx, hipGetLastError());
            si = last_si;
        }
        sc->tail_seq0 = seq0;
        sc->tail_running = true;
        sc->wait_any_skip1 = true;
        sc->wait_slots = 0;
        ctx->tail_owner = sc;
        return DPS_OK;
}

// A round among the resident ones (slice_kernel): a trip to the launch, or the second round of a trip, answered here.
int32_t FusedRound::resident_round()
{
    const u32 kind = sc->round_kind[j];
    const u32 np = nf + 1;
    E2 q[dpk::MAX_PTS];
    int32_t rc = DPS_OK;
    if (kind == 4) {
        // A round of the few pairs that are left once the launch has gone: worked out here.
        if (sc->host_len < (j == 1 ? 2u : 4u)) return fail(ctx, DPS_ERR_STATE, "dps_sc_round: the tables of the last rounds are not here");
        // (round 1 of a sum that is the host's from the start has nothing to fold)
        if (j >= 2) host_tail_advance(sc, gl::e2(challenge[0], challenge[1]));
        host_tail_sums(sc, j, nf, a.skip1 != 0, q);
        prepare_message();
        form_message(q);
    } else if (kind == 3) {
        // Second round of a trip: the kernel handed over this round's sums as a polynomial in the challenge that has
        // now been drawn (values at 0..nf-1 and the leading coefficient, per point t = 0, 2, .., nf); p(1) comes
        // from the claim.  Nothing goes to the GPU.
        const E2 r = gl::e2(challenge[0], challenge[1]);
        E2 vanish = gl::e2_one(), basis[dpk::MAX_PTS];
        for (u32 k = 0; k < nf; k++) {
            E2 num = gl::e2_one();
            for (u32 m = 0; m < nf; m++)
                if (m != k) num = gl::mul(num, gl::sub(r, gl::e2(m, 0)));
            basis[k] = gl::mul_base(num, ctx->h_inv_den[nf - 1][k]);
            vanish = gl::mul(vanish, gl::sub(r, gl::e2(k, 0)));
        }
        for (u32 t = 0; t < np; t++) q[t] = gl::e2_zero();
        for (u32 ti = 0; ti < nf; ti++) {
            E2 v = gl::mul(vanish, sc->stash[nf * nf + ti]);
            for (u32 k = 0; k < nf; k++) v = gl::add(v, gl::mul(basis[k], sc->stash[k * nf + ti]));
            q[ti == 0 ? 0 : ti + 1] = v;
        }
        prepare_message();
        form_message(q);
    } else {
        if (!sc->tail_running) {
            if (j != sc->tail_j0) return fail(ctx, DPS_ERR_STATE, "dps_sc_round: the resident launch of the last rounds is gone");
            // (a launch for round 1 needs nothing of its first mail but whether t = 1 is evaluated: it is told at once)
            CHK(launch_stages_at(fa.seq, sc->tail_j0 == 1 && j == 1 ? (a.skip1 ? 2u : 1u) : 0u));
        }
        post_mail();
        sc->wait_fresh = false;
        prepare_message();
        // sums of this round, and with a trip of two rounds those of the next
        const u32 ns = kind == 2 ? np + np * nf : np;
        u64 cnt[dpk::SL_MAX_GROUPS * dpk::SL_GROUP_WORDS];
        const u32 n_sets = sc->round_wide[j] ? sc->round_wide[j] : 1;
        rc = wait_slice_sums(ctx, fa.seq, ns, a.skip1 != 0, n_sets, cnt);
        if (rc == DPS_OK) {
            // several workgroups: the counters run on from trip to trip of the launch, and the sets of counters add up
            if (sc->round_wide[j])
                for (u32 c = 0; c < 4 * ns; c++) {
                    if (a.skip1 && c >= 4 && c < 8) continue;
                    u64 sum = 0;
                    for (u32 set = 0; set < n_sets; set++) {
                        const u64 now = cnt[set * dpk::SL_GROUP_WORDS + c];
                        sum += now - sc->ctr_seen[set * dpk::SL_GROUP_WORDS + c];
                        sc->ctr_seen[set * dpk::SL_GROUP_WORDS + c] = now;
                    }
                    cnt[c] = sum;
                }
            // limb w & 1 of sum w >> 1: counters 2w (low halves) and 2w + 1 (high halves)
            u64 w[2 * dpk::SL_MAX_SUMS];
            for (u32 i = 0; i < 2 * ns; i++) {
                const unsigned __int128 t = (unsigned __int128)cnt[2 * i] + ((unsigned __int128)cnt[2 * i + 1] << 32);
                w[i] = gl::reduce128((u64)t, (u64)(t >> 64));
            }
            for (u32 t = 0; t < np; t++) q[t] = gl::e2(w[2 * t], w[2 * t + 1]);
            for (u32 i = np; i < ns; i++) sc->stash[i - np] = gl::e2(w[2 * i], w[2 * i + 1]);
            form_message(q);
            sc->last_trip_seq = fa.seq;
            // the last trip: what is left of the tables has come with it
            if (j + (kind == 2 ? 1 : 0) == sc->n_vars - sc->host_rounds) rc = host_tail_load(sc, fa.seq);
        }
    }
    if (challenge) sc->prev_chal = gl::e2(challenge[0], challenge[1]);
    if ((kind != 4 && j == sc->n_vars - sc->host_rounds) || rc != DPS_OK) {
        // with its last trip the kernel publishes what is left of the tables and exits
        sc->tail_running = false;
        waiting_launch_over(ctx);
        if (rc == DPS_OK) sc->pairs_seq = sc->last_trip_seq;
    }
    if (rc != DPS_OK) {
        // the launch left without publishing (it gave up waiting, or the stream failed): nothing of it can be used again
        // (the wait only fails once the stream has drained, so nothing of it is still to land)
        sc->broken = true;
        reset_device_words(ctx);
        clear_resident_results(ctx);
    }
    CHK(rc);
    sc->round = j;
    return DPS_OK;
}

FusedRound::Plan FusedRound::plan_round(u32 jj, bool skip1_jj) const
{
        Plan p;
        p.n_pairs = 1ull << (sc->n_vars - jj);
        p.split = p.n_pairs <= POLY_SPLIT_MAX_PAIRS;
        p.split_log = 0;
        p.blocks = blocks_for_pairs(p.n_pairs);
        if (p.split) poly_split_plan(p.n_pairs, sc->poly_split_cap, n_groups <= POLY_RAW_MAX_GROUPS, &p.split_log, &p.blocks);
        // a single workgroup (per group) from here on: it stays for the remaining rounds
        // (several groups stay only with their tables in LDS: they must not read each other's stores)
        p.reside = p.split && n_groups <= POLY_RAW_MAX_GROUPS && p.blocks == 1 && skip1_jj && jj < sc->n_vars &&
                   sc->n_vars - jj + 1 <= (u32)dpk::POLY_RES_ROUNDS && (n_groups == 1 || poly_split_state_ok(ctx, nf, has_eq, true));
        return p;
}

// Launches the kernel of round jj.  `ahead`: round jj has not begun (its challenge is not known); the kernel
// waits for the mail of sequence number `seq_jj` and takes the challenge and the message's scalars from it.
int32_t FusedRound::launch_round(u32 jj, const Plan &p, bool skip1_jj, bool ahead, u64 seq_jj)
{
        dpk::PolyArgs pa;
        pa.groups = sc->d_poly_groups + (size_t)(jj - 1) * n_groups;
        pa.terms = sc->d_poly_terms;
        pa.ops = sc->d_poly_ops;
        if (inline_descs) {
            pa.groups = nullptr;
            pa.terms = nullptr;
            pa.ops = nullptr;
            pa.g0 = sc->h_poly_groups[jj - 1];
            if (!p.split && !sc->h_poly_ops.empty())
                memcpy(pa.o0, sc->h_poly_ops.data(), sc->h_poly_ops.size() * sizeof(dpk::PolyOp));
            else
                std::copy(sc->h_poly_terms.begin(), sc->h_poly_terms.end(), pa.t0);
        } else {
            CHK(ensure_descs(sc));
        }
        pa.q0 = pa.q1 = nullptr;
        pa.lq0 = pa.lq1 = pa.hq0 = pa.hq1 = nullptr;
        if (has_eq) {
            const u64 off = eq_level_off(sc->n_vars, jj);
            pa.q0 = sc->eq_c0 + off;
            pa.q1 = sc->eq_c1 + off;
            if (!p.split && poly_round_weights_factored(sc, jj)) {
                // not streamed: the low table of level jj and level jj + 16 (as the large rounds of a product take them)
                const u64 lo = eq_low_off(sc->n_vars, jj), hi = eq_level_off(sc->n_vars, jj + dpk::EQ_LO_BITS);
                pa.lq0 = sc->eq_c0 + lo;
                pa.lq1 = sc->eq_c1 + lo;
                pa.hq0 = sc->eq_c0 + hi;
                pa.hq1 = sc->eq_c1 + hi;
            }
        }
        pa.n_pairs = p.n_pairs;
        pa.r0 = ahead ? 0 : a.r0;
        pa.r1 = ahead ? 0 : a.r1;
        pa.j = jj;
        pa.last_round = 0;
        pa.n_vars = sc->n_vars;
        pa.spin_limit = wait_units(ctx, 4000000);
        pa.eq0 = sc->eq_c0;
        pa.eq1 = sc->eq_c1;
        pa.mail = ctx->d_pinned + (ctx->res_off - 64);
        pa.seq = seq_jj;
        pa.split_log = p.split_log;
        pa.split_cap = sc->poly_split_cap;
        pa.lds_state = pa.state_off = pa.pad = 0;
        pa.finish = sc->poly_finish_in_kernel ? 1 : 0;
        pa.group_stride = 1;
        pa.raw_out = nullptr;
        pa.wait_first = ahead ? 1 : 0;
        if (ahead && !p.reside) pa.spin_limit = wait_units(ctx, AHEAD_SPIN_LIMIT);
        // (more workgroups than should poll the host's memory: the first one polls and passes the mail on)
        pa.relay = ahead && p.blocks * n_groups > POLY_AHEAD_MAX_WORKGROUPS ? mail_relay(ctx) : nullptr;
        if (p.reside) {
            pa.last_round = sc->n_vars;
            if (n_groups > 1) {
                // one resident workgroup per group, each publishing its own sums
                CHK(ensure_descs(sc));
                pa.groups = sc->d_poly_groups + (size_t)(jj - 1) * n_groups;
                pa.group_stride = n_groups;
                pa.raw_out = ctx->d_pinned + poly_raw_off(ctx);
            } else if (inline_descs) {
                // the descriptors of the remaining rounds go through pinned memory: the kernel copies them to LDS
                // before anything else (and before it looks for mail); the area is not written again before a
                // message of this launch has arrived
                const size_t words = (size_t)(sc->n_vars - jj + 1) * sizeof(dpk::PolyGroup) / 8;
                memcpy(ctx->h_pinned, &sc->h_poly_groups[jj - 1], words * 8);
                pa.groups = reinterpret_cast<const dpk::PolyGroup *>(ctx->d_pinned);
            } else {
                pa.groups = sc->d_poly_groups + (size_t)(jj - 1);
            }
        }
        dpk::FastFin fl = ff;
        fl.seq = seq_jj;
        fl.n_blocks = p.blocks * n_groups;
        fl.slots = !p.reside && slots_for(fl.n_blocks) ? ctx->d_pinned + poly_raw_off(ctx) : nullptr;
        double pbytes = has_eq ? (double)p.n_pairs * 16.0 : 0.0;
        for (u32 k = 0; k < sc->n_mles; k++)
            if (sc->poly_owner[k] >= 0) pbytes += (double)p.n_pairs * (jj >= 2 ? 4 * 16.0 + 2 * 16.0 : 2 * 16.0);
        ProfScope ps(ctx, DPS_K_EVAL_TERMS, pbytes);
        if (p.split)
            CHK(launch_poly_split_dispatch(ctx, nf, has_eq, skip1_jj, pa, dim3(p.blocks, n_groups), sc->poly_max_tabs, p.reside, sc->d_partial, fl));
        else
            CHK(launch_poly_dispatch(ctx, nf, has_eq, skip1_jj, pa, dim3(p.blocks, n_groups), sc->poly_max_tabs, sc->d_partial, fl));
        HIPCHK(ctx, hipGetLastError());
        return DPS_OK;
}

// A round of sums of several terms over shared tables (poly_kernel / poly_split_kernel): this round's launch, or the mail for
// one that waits on the GPU; then the next round's launch behind it.
int32_t FusedRound::multi_term_round()
{
    // a launch that takes this round may already be on the GPU, waiting for the mail: a resident one from an
    // earlier round, or one made ahead during the previous round
    const bool on_gpu = sc->tail_running;
    bool stays;
    u32 slots_now;
    if (on_gpu) {
        post_mail();
        sc->wait_fresh = false;
        stays = sc->wait_stays;
        slots_now = sc->wait_slots;
    } else {
        Plan p = plan_round(j, a.skip1 != 0);
        // a launch that stays needs its place on the device (one workgroup per group, all there at once); without it
        // the round is a launch of its own
        if (p.reside && !admit_waiting_launch(ctx, std::max<u32>(n_groups, 1), true)) p.reside = false;
        CHK(launch_round(j, p, a.skip1 != 0, false, fa.seq));
        stays = p.reside;
        slots_now = slots_of(p);
        if (p.reside) {
            sc->tail_running = true;
            sc->tail_seq0 = fa.seq;
            ctx->tail_owner = sc;
            sc->poly_raw = n_groups > 1;
            sc->wait_slots = slots_now;
            sc->wait_stays = true;
            sc->wait_skip1 = true;
            sc->wait_fresh = false;
        }
    }
    if (!stays) {
        // the launch of this round ends with it
        sc->tail_running = false;
        waiting_launch_over(ctx);
        // The next round's launch is made now, behind this one: by the time this round's message has crossed to
        // the host and the challenge is drawn, it is already on the GPU looking for its mail.  Only for rounds
        // of few workgroups (every workgroup polls the mailbox), and not while launches are being timed.
        if (j < sc->n_vars && !ctx->profiling && !sc->no_ahead) {
            // p(1) comes from the claim unless the scale vanishes at 1, i.e. unless the eq point is 0 there
            bool skip1_next = true;
            if (has_eq) {
                const E2 rho = sc->eq_info->point[j];
                skip1_next = !(rho.c0 == 0 && rho.c1 == 0);
            }
            const Plan pn = plan_round(j + 1, skip1_next);
            if (sc->tail_j0 && j + 1 == sc->tail_j0) {
                // the rounds from here on are resident: their launches are queued now and wait for their first mail
                // (when the device has room for them now; else the next round asks again)
                if (admit_stages()) {
                    CHK(launch_stages_at(ctx->seq + 1));
                    sc->wait_fresh = true;
                    sc->ahead_at = std::chrono::steady_clock::now();
                }
            } else if (admit_waiting_launch(ctx, pn.blocks * std::max<u32>(n_groups, 1), pn.reside)) {
                CHK(launch_round(j + 1, pn, skip1_next, true, ctx->seq + 1));
                sc->tail_running = true;
                sc->tail_seq0 = ctx->seq + 1;
                ctx->tail_owner = sc;
                sc->wait_stays = pn.reside;
                sc->wait_skip1 = skip1_next;
                sc->wait_fresh = true;
                sc->ahead_at = std::chrono::steady_clock::now();
                sc->poly_raw = pn.reside && n_groups > 1;
                sc->wait_slots = slots_of(pn);
            }
        }
    }
    int32_t rc = take_sums(slots_now);
    if (rc != DPS_OK) {
        // a launch that left without publishing may have taken some of its tickets and written some of its tables
        sc->broken = true;
        reset_device_words(ctx);
    }
    if (stays && (rc != DPS_OK || j == sc->n_vars)) {
        // a resident launch exits after the last round; one that can finish has published the tables' last pairs with it
        sc->tail_running = false;
        waiting_launch_over(ctx);
        if (rc == DPS_OK && sc->poly_finish_in_kernel) sc->pairs_seq = fa.seq;
    }
    CHK(rc);
    sc->round = j;
    return DPS_OK;
}

// The next round's launch, made behind this round's (for the same reasons as in multi_term_round): the resident launches, or a
// product kernel, which then waits for its challenge by mail.
int32_t FusedRound::product_launch_ahead(u32 ahead)
{
    // `ahead`: 1, the round after this one; or 2 when that one is answered on the host (the second round of a launch that
    // covers two): the launch is then queued behind this round's and waits for its mail from the moment that one ends
    const u32 jn = j + ahead;
    if (jn <= sc->n_vars && !ctx->profiling && !sc->no_ahead) {
        const u64 next_seq = ctx->seq + ahead;
        const u64 pairs_n = 1ull << (sc->n_vars - jn);
        bool made = false;
        if (sc->tail_j0 && jn == sc->tail_j0) {
            // (when the device has room for the resident launches now; else the next round asks again)
            if (admit_stages()) {
                CHK(launch_stages_at(next_seq));
                made = true;
            }
        } else if (const dps_sc::QuadStep *q = quad_at(jn)) {
            // the next two rounds are one launch
            if (admit_waiting_launch(ctx, q->blocks, false)) {
                CHK(launch_quad(*q, true, next_seq));
                sc->wait_any_skip1 = false;
                sc->wait_skip1 = true;
                sc->wait_slots = 0;
                made = true;
            }
        } else if (sc->round_kind[jn] == 0 && admit_waiting_launch(ctx, product_blocks(pairs_n), false)) {
            // (more workgroups than should poll the host's memory: workgroup 0 polls and passes the mail on)
            // p(1) comes from the claim unless the scale vanishes at 1
            bool skip1_next = !(sc->fast_coeff.c0 == 0 && sc->fast_coeff.c1 == 0);
            if (has_eq) {
                const E2 rho = sc->eq_info->point[jn - 1];
                skip1_next = skip1_next && !(rho.c0 == 0 && rho.c1 == 0) && !(sc->eq_scalar.c0 == 0 && sc->eq_scalar.c1 == 0);
            }
            dpk::ProdArgs an = sc->fast_args[jn];
            if (has_eq) set_eq_weights(an, jn, product_blocks(pairs_n));
            an.r0 = an.r1 = 0;
            an.skip1 = skip1_next ? 1 : 0;
            an.wait_first = 1;
            an.spin_limit = wait_units(ctx, AHEAD_SPIN_LIMIT);
            an.mail = ctx->d_pinned + (ctx->res_off - 64);
            an.relay = product_blocks(pairs_n) > POLY_AHEAD_MAX_WORKGROUPS ? mail_relay(ctx) : nullptr;
            dpk::FastFin fn = ff;
            fn.n_blocks = product_blocks(pairs_n);
            fn.seq = next_seq;
            fn.slots = slots_for(fn.n_blocks) ? ctx->d_pinned + poly_raw_off(ctx) : nullptr;
            sc->wait_slots = slots_for(fn.n_blocks);
            CHK(launch_prod_dispatch(ctx, nf, sc->fast_nb[jn], has_eq, true, an, fn.n_blocks, sc->d_partial, fn));
            HIPCHK(ctx, hipGetLastError());
            sc->wait_any_skip1 = false;
            sc->wait_skip1 = skip1_next;
            made = true;
        }
        if (made) {
            sc->tail_running = true;
            sc->wait_fresh = true;
            sc->ahead_at = std::chrono::steady_clock::now();
            ctx->tail_owner = sc;
        }
    }

    return DPS_OK;
}

// A round of a product of full-size tables (prod_kernel).
int32_t FusedRound::product_round()
{
    u32 slots_now = sc->wait_slots;
    if (sc->tail_running) {
        // launched during the previous round
        post_mail();
        sc->wait_fresh = false;
    } else {
        slots_now = slots_for(blocks);
        ff.slots = slots_now ? ctx->d_pinned + poly_raw_off(ctx) : nullptr;
        // (in the factored form the eq weights are one entry per thread and one per workgroup and step: not counted)
        double bytes = has_eq && !a.lq0 ? (double)n_pairs * 16.0 : 0.0;
        for (u32 f = 0; f < nf; f++) {
            double eb = a.s1[f] ? 16.0 : 8.0;
            bytes += (j >= 2) ? (double)n_pairs * ((a.two ? 8 : 4) * eb + 2 * 16.0) : (double)n_pairs * 2 * eb;
        }
        ProfScope ps(ctx, j >= 2 ? DPS_K_FOLD_EVAL : DPS_K_EVAL_FIRST, bytes);
        a.wait_first = 0;
        CHK(launch_prod_dispatch(ctx, nf, sc->fast_nb[j], has_eq, j >= 2, a, blocks, sc->d_partial, ff));
        HIPCHK(ctx, hipGetLastError());
    }
    // this round's launch ends with the round
    sc->tail_running = false;
    waiting_launch_over(ctx);
    CHK(product_launch_ahead());
    if (const int32_t rc = take_sums(slots_now); rc != DPS_OK) {
        sc->broken = true;
        reset_device_words(ctx);
        return rc;
    }
    if (challenge) sc->prev_chal = gl::e2(challenge[0], challenge[1]);
    sc->round = j;
    return DPS_OK;
}

// Round 1 of a session whose first two rounds are one launch: the launch, round 1's message, and round 2's sums kept as
// a polynomial in the challenge to come.
int32_t FusedRound::first_two_rounds_launch()
{
    dpk::Pair12Args pa;
    pa.f = a.s0[0];
    pa.g = a.s0[1];
    pa.n_quads = n_pairs >> 1;
    // the weights of round 2's pairs: low table of level 2, level 2 + 16
    const u64 lo = eq_low_off(sc->n_vars, 2), hi = eq_level_off(sc->n_vars, 2 + dpk::EQ_LO_BITS);
    pa.lq0 = sc->eq_c0 + lo;
    pa.lq1 = sc->eq_c1 + lo;
    pa.hq0 = sc->eq_c0 + hi;
    pa.hq1 = sc->eq_c1 + hi;
    ff.n_blocks = PAIR12_BLOCKS;
    ff.slots = nullptr;
    {
        ProfScope ps(ctx, DPS_K_EVAL_FIRST, (double)n_pairs * 2 * 2 * 8.0);
        dpk::pair12_kernel<<<PAIR12_BLOCKS, dpk::PAIR12_BLOCK, 0, ctx->stream>>>(pa, sc->d_partial, ff);
        HIPCHK(ctx, hipGetLastError());
    }
    // round 2 needs no launch: round 3's is queued behind this one now and waits for its mail from the moment this ends
    sc->tail_running = false;
    waiting_launch_over(ctx);
    CHK(product_launch_ahead(2));
    a.skip1 = 0;  // (every point of round 1 is computed: round 2 needs them as well)
    skip1 = false;
    prepare_message();
    u64 w[2 * dpk::PAIR12_SUMS];
    if (const int32_t rc = wait_result_at(ctx, ctx->res_off, fa.seq, 0, 2 * dpk::PAIR12_SUMS, w, dpk::PAIR12_SEQ_SLOT, dpk::PAIR12_CHK_SLOT);
        rc != DPS_OK) {
        sc->broken = true;
        reset_device_words(ctx);
        return rc;
    }
    // pair 0's three (value at 0, at 1, leading coefficient of the product along x0), pair 1's, and the same three products
    // of the slopes along x1: each product is a quadratic in x1 with these as its values at 0 and 1 and its leading
    // coefficient, so at x1 = 2 (round 2 at t = 2) it is 2 v(1) - v(0) + 2 lead
    for (u32 k = 0; k < (u32)dpk::PAIR12_SUMS; k++) sc->stash[k] = gl::e2(w[2 * k], w[2 * k + 1]);
    for (u32 k = 0; k < 3; k++) {
        const E2 v0 = sc->stash[k], v1 = sc->stash[3 + k], lead = sc->stash[6 + k];
        sc->stash[6 + k] = gl::add(gl::sub(gl::add(v1, v1), v0), gl::add(lead, lead));
    }
    // round 1 sums over the pairs of either kind, weighted by eq1(rho_2, x1); its q(2) = 2 q(1) - q(0) + 2 c
    const E2 rho2 = sc->eq_info->point[1], n2 = gl::sub(gl::e2_one(), rho2);
    E2 q[3];
    for (u32 k = 0; k < 3; k++) q[k] = gl::add(gl::mul(n2, sc->stash[k]), gl::mul(rho2, sc->stash[3 + k]));
    const E2 c = q[2];
    q[2] = gl::add(gl::sub(gl::add(q[1], q[1]), q[0]), gl::add(c, c));
    form_message(q);
    sc->round = j;
    return DPS_OK;
}

// Round 2 of such a session: nothing goes to the GPU.  Each of round 2's sums q(0), q(1), q(2) is a polynomial of degree 2
// in round 1's challenge, known by its values at 0 and 1 and its leading coefficient; then round 3 is launched ahead.
int32_t FusedRound::second_round_from_stash()
{
    const E2 r = gl::e2(challenge[0], challenge[1]);
    const E2 rr = gl::mul(r, gl::sub(r, gl::e2_one()));
    E2 q[3];
    for (u32 t = 0; t < 3; t++) {
        const E2 v0 = sc->stash[3 * t], v1 = sc->stash[3 * t + 1], lead = sc->stash[3 * t + 2];
        q[t] = gl::add(gl::add(v0, gl::mul(r, gl::sub(v1, v0))), gl::mul(rr, lead));
    }
    prepare_message();
    form_message(q);
    // (round 3's launch is usually waiting already, made behind the launch of the first two rounds)
    if (!sc->tail_running) CHK(product_launch_ahead());
    sc->prev_chal = r;
    sc->round = j;
    return DPS_OK;
}

const dps_sc::QuadStep *FusedRound::quad_at(u32 jj) const
{
    for (const dps_sc::QuadStep &q : sc->quads)
        if (q.j == jj) return &q;
    return nullptr;
}

// The launch of rounds q.j and q.j + 1 (quad_kernel).  `ahead`: made before round q.j begins; it waits for the mail of
// sequence number seq_q, which brings the challenges of the two rounds before.
int32_t FusedRound::launch_quad(const dps_sc::QuadStep &q, bool ahead, u64 seq_q)
{
    dpk::ProdArgs qa;
    memset(&qa, 0, sizeof qa);
    for (u32 f = 0; f < 2; f++) {
        qa.s0[f] = q.s0[f];
        qa.s1[f] = q.s1[f];
        qa.d0[f] = q.d0[f];
        qa.d1[f] = q.d1[f];
    }
    const u64 n_quads = 1ull << (sc->n_vars - q.j - 1);
    qa.n_pairs = n_quads;
    qa.skip1 = 1;
    if (!ahead) {
        qa.r0 = a.r0, qa.r1 = a.r1;
        qa.ra0 = sc->prev_chal.c0, qa.ra1 = sc->prev_chal.c1;
    }
    qa.wait_first = ahead ? 1 : 0;
    qa.spin_limit = wait_units(ctx, AHEAD_SPIN_LIMIT);
    qa.mail = ctx->d_pinned + (ctx->res_off - 64);
    qa.relay = ahead && q.blocks > POLY_AHEAD_MAX_WORKGROUPS ? mail_relay(ctx) : nullptr;
    // the weights of round q.j + 1's pairs: low table of that level, and the level 16 rounds later
    const u64 lo = eq_low_off(sc->n_vars, q.j + 1), hi = eq_level_off(sc->n_vars, q.j + 1 + dpk::EQ_LO_BITS);
    qa.lq0 = sc->eq_c0 + lo;
    qa.lq1 = sc->eq_c1 + lo;
    qa.hq0 = sc->eq_c0 + hi;
    qa.hq1 = sc->eq_c1 + hi;
    dpk::FastFin fq = ff;
    fq.n_blocks = q.blocks;
    fq.seq = seq_q;
    fq.slots = nullptr;
    // sixteen source entries read and four written per table and quad
    const double src_bytes = q.s1[0] ? 16.0 : 8.0;
    ProfScope ps(ctx, DPS_K_FOLD_EVAL, (double)n_quads * 2 * (16 * src_bytes + 4 * 16.0));
    if (q.s1[0])
        dpk::quad_kernel<false><<<q.blocks, dpk::BLOCK, 0, ctx->stream>>>(qa, sc->d_partial, fq);
    else
        dpk::quad_kernel<true><<<q.blocks, dpk::BLOCK, 0, ctx->stream>>>(qa, sc->d_partial, fq);
    HIPCHK(ctx, hipGetLastError());
    return DPS_OK;
}

// The first round of a launch that covers two: the launch (or the mail for it), this round's message from the sums over
// the pairs of either kind, and the next round's sums kept as polynomials in the challenge to come.
int32_t FusedRound::quad_first_round()
{
    const dps_sc::QuadStep &q = *quad_at(j);
    if (sc->tail_running) {
        // (the launch's sums serve either way of getting p(1); its mail always says the one it was compiled for)
        const u32 keep = a.skip1;
        a.skip1 = 1;
        post_mail();
        a.skip1 = keep;
        sc->wait_fresh = false;
    } else {
        CHK(launch_quad(q, false, fa.seq));
    }
    // the launch ends with the round; the round after it needs no launch, so the launch after that is queued behind
    // this one now
    sc->tail_running = false;
    waiting_launch_over(ctx);
    CHK(product_launch_ahead(2));
    prepare_message();
    u64 w[2 * dpk::QUAD_SUMS];
    if (const int32_t rc = wait_result(ctx, fa.seq, 0, 2 * dpk::QUAD_SUMS, w); rc != DPS_OK) {
        sc->broken = true;
        reset_device_words(ctx);
        return rc;
    }
    E2 v[dpk::QUAD_SUMS];
    for (u32 k = 0; k < (u32)dpk::QUAD_SUMS; k++) v[k] = gl::e2(w[2 * k], w[2 * k + 1]);
    const E2 A0 = v[0], A1 = v[1], Al = v[2], B0 = v[3], B2 = v[4];
    // the even pairs' product at t = 2 from its values at 0, 1 and its leading coefficient
    const E2 A2 = gl::add(gl::sub(gl::add(A1, A1), A0), gl::add(Al, Al));
    // pairs of either kind weighted by eq1(rho, .), rho the eq point's coordinate of the variable the next round binds
    const E2 rho = sc->eq_info->point[j], nrho = gl::sub(gl::e2_one(), rho);
    E2 qs[3];
    qs[0] = gl::add(gl::mul(nrho, A0), gl::mul(rho, B0));
    qs[1] = gl::e2_zero();
    qs[2] = gl::add(gl::mul(nrho, A2), gl::mul(rho, B2));
    // the next round at t = 0 and t = 2: value at c = 0, at c = 1, leading coefficient in c
    sc->stash[0] = A0, sc->stash[1] = A1, sc->stash[2] = Al;
    sc->stash[3] = v[5], sc->stash[4] = v[6], sc->stash[5] = v[7];
    // (a.skip1 is off only when the scale has vanished, and then no q matters: the message is the constant terms')
    form_message(qs);
    if (challenge) sc->prev_chal = gl::e2(challenge[0], challenge[1]);
    sc->round = j;
    return DPS_OK;
}

// Its second round: nothing goes to the GPU but the launch after it, made ahead.
int32_t FusedRound::quad_second_round()
{
    const E2 r = gl::e2(challenge[0], challenge[1]);
    // (the launch of the rounds after this one is usually waiting already, made behind this pair's)
    if (!sc->tail_running) CHK(product_launch_ahead());
    const E2 rr = gl::mul(r, gl::sub(r, gl::e2_one()));
    E2 qs[3];
    for (u32 t = 0; t < 2; t++) {
        const E2 v0 = sc->stash[3 * t], v1 = sc->stash[3 * t + 1], lead = sc->stash[3 * t + 2];
        qs[t == 0 ? 0 : 2] = gl::add(gl::add(v0, gl::mul(r, gl::sub(v1, v0))), gl::mul(rr, lead));
    }
    qs[1] = gl::e2_zero();
    prepare_message();
    form_message(qs);
    sc->prev_chal = r;
    sc->round = j;
    return DPS_OK;
}

// The resident launch found no place on the device and the launches of two rounds each have run: the state in memory
// is two rounds old, where the ordinary launch of this round expects one fold pending.  The older of the two folds is
// made here (into the table's other buffer, and from there to where this round's launch reads).
int32_t FusedRound::catch_up_after_quads()
{
    const dps_sc::QuadStep &q = sc->quads.back();
    const u64 n_out = 1ull << (sc->n_vars - q.j);  // entries of the state of round q.j + 1
    for (u32 f = 0; f < 2; f++) {
        const SessMle &m = sc->m[sc->fast_order[f]];
        const int other = q.d0[f] == m.buf0[0] ? 1 : 0;
        u64 *t0 = m.buf0[other], *t1 = m.buf1[other];
        dpk::refold_kernel<<<grid_for(n_out), dpk::BLOCK, 0, ctx->stream>>>(q.d0[f], q.d1[f], t0, t1, n_out, sc->prev_chal.c0, sc->prev_chal.c1);
        HIPCHK(ctx, hipGetLastError());
        u64 *want0 = const_cast<u64 *>(sc->fast_args[j].s0[f]), *want1 = const_cast<u64 *>(sc->fast_args[j].s1[f]);
        if (want0 != t0) {
            HIPCHK(ctx, hipMemcpyAsync(want0, t0, n_out * 8, hipMemcpyDeviceToDevice, ctx->stream));
            HIPCHK(ctx, hipMemcpyAsync(want1, t1, n_out * 8, hipMemcpyDeviceToDevice, ctx->stream));
        }
    }
    return DPS_OK;
}

}  // namespace

extern "C" int32_t dps_sc_round(dps_sc *sc, const uint64_t *challenge, uint64_t *evals_out)
{
    if (!sc || !evals_out) return DPS_ERR_INVALID;
    dps_ctx *ctx = sc->ctx;
    if (sc->finished || sc->round >= sc->n_vars) return fail(ctx, DPS_ERR_STATE, "dps_sc_round: all %u rounds are done", sc->n_vars);
    const u32 j = sc->round + 1;
    if ((j == 1) != (challenge == nullptr)) return fail(ctx, DPS_ERR_STATE, "dps_sc_round: round %u %s a challenge", j, j == 1 ? "takes no" : "needs");
    if (challenge && !canonical(challenge, 2)) return fail(ctx, DPS_ERR_INVALID, "dps_sc_round: challenge not canonical");
    if (sc->broken) return fail(ctx, DPS_ERR_STATE, "dps_sc_round: the session was interrupted by another call on its context");
    DeviceGuard g(ctx->device);
    if (ctx->tail_owner != sc) tail_abort(ctx);
    const u32 live = sc->n_vars - j + 1;
    const u64 n_pairs = 1ull << (live - 1);
    u32 blocks = sc->fast ? product_blocks(n_pairs) : blocks_for_pairs(n_pairs);
    // constant terms: c summed over 2^(live-1) suffixes at every evaluation point
    E2 cst = gl::mul_base(sc->const_sum, h_pow(2, live - 1));
    dpk::FinArgs fa;
    memset(&fa, 0, sizeof fa);
    fa.partial = sc->d_partial;
    fa.blocks_per_term = sc->n_terms ? blocks : 0;
    fa.n_terms = sc->n_terms;
    if (!sc->fast && !sc->poly) CHK(ensure_descs(sc));
    fa.terms = sc->d_fin;
    fa.degree = sc->degree;
    fa.total_blocks = blocks * sc->n_terms;
    fa.lagrange = ctx->d_lagrange;
    fa.const0 = cst.c0;
    fa.const1 = cst.c1;
    fa.out_dev = sc->d_result;
    fa.out_host = ctx->d_pinned + ctx->res_off;
    fa.seq = ++ctx->seq;
    fa.counter = sc->d_counter;
    if (sc->n_terms == 0) {
        if (j >= 2) CHK(launch_folds(sc, j, false, challenge));
        ProfScope ps(ctx, DPS_K_FINALIZE, 0.0);
        dpk::finalize_kernel<<<1, dpk::BLOCK, 0, ctx->stream>>>(fa);
        HIPCHK(ctx, hipGetLastError());
    } else if (sc->fast || sc->poly) {
        FusedRound fr;
        memset(static_cast<void *>(&fr), 0, sizeof fr);
        fr.sc = sc, fr.ctx = ctx, fr.j = j, fr.challenge = challenge, fr.evals_out = evals_out;
        fr.n_pairs = n_pairs, fr.blocks = blocks, fr.cst = cst, fr.fa = fa;
        CHK(fr.begin());
        // the resident rounds begin here and their launch is not on the GPU yet: with no place for it on the device
        // these rounds are launches of their own
        if (sc->tail_j0 && j == sc->tail_j0 && !sc->tail_running && !fr.admit_stages()) {
            if (!sc->quads.empty()) CHK(fr.catch_up_after_quads());
            drop_resident_plan(sc);
        }
        if ((sc->tail_j0 && j >= sc->tail_j0) || sc->host_only) return fr.resident_round();
        if (sc->pair12 && j == 1) return fr.first_two_rounds_launch();
        if (sc->pair12 && j == 2) return fr.second_round_from_stash();
        if (sc->round_kind[j] == 5) return fr.quad_first_round();
        if (sc->round_kind[j] == 6) return fr.quad_second_round();
        return sc->poly ? fr.multi_term_round() : fr.product_round();
    } else {
        if (j >= 2) CHK(launch_folds(sc, j, false, challenge));
        for (u32 base = 0; base < sc->n_terms; base += 65535) {
            u32 n = std::min<u32>(sc->n_terms - base, 65535);
            ProfScope ps(ctx, DPS_K_EVAL_TERMS, 0.0);
            dpk::eval_terms_kernel<<<dim3(blocks, n), dpk::BLOCK, 0, ctx->stream>>>(
                sc->d_terms + sc->term_off[j] + base, sc->d_partial + (size_t)base * blocks * 2 * dpk::MAX_PTS, fa);
            HIPCHK(ctx, hipGetLastError());
        }
    }
    CHK(wait_result(ctx, fa.seq, 0, 2 * (sc->degree + 1), evals_out));
    sc->round = j;
    return DPS_OK;
}

extern "C" int32_t dps_sc_finish(dps_sc *sc, const uint64_t *challenge, uint64_t *final_evals_out)
{
    if (!sc || (sc->n_mles && !final_evals_out)) return DPS_ERR_INVALID;
    dps_ctx *ctx = sc->ctx;
    if (sc->finished || sc->round != sc->n_vars) return fail(ctx, DPS_ERR_STATE, "dps_sc_finish: %u of %u rounds done", sc->round, sc->n_vars);
    if (sc->n_vars >= 1 && !challenge) return fail(ctx, DPS_ERR_INVALID, "dps_sc_finish: the last challenge is missing");
    if (challenge && !canonical(challenge, 2)) return fail(ctx, DPS_ERR_INVALID, "dps_sc_finish: challenge not canonical");
    if (sc->broken) return fail(ctx, DPS_ERR_STATE, "dps_sc_finish: the session was interrupted by another call on its context");
    DeviceGuard g(ctx->device);
    if (ctx->tail_owner != sc) tail_abort(ctx);
    if (sc->pairs_seq) {
        // the resident launch published value and slope of every table's last pair with its last round: the final
        // evaluations are value + r * slope
        const E2 r = gl::e2(challenge[0], challenge[1]);
        u64 w[8 * dpk::SL_MAX_TABS];
        // the fused multi-term kernel publishes its group's tables in slot order (one area per group when several
        // groups are resident), the single-product one its factors
        if (!sc->stages.empty() || sc->host_only) {
            // the host holds the tables: the last fold leaves one entry each
            if (sc->host_len < 2) return fail(ctx, DPS_ERR_STATE, "dps_sc_finish: the tables' last entries are not here");
            host_tail_advance(sc, r);
            const u32 n_tabs = (u32)sc->slice_ids.size();
            if (sc->host_len != 1) return fail(ctx, DPS_ERR_STATE, "dps_sc_finish: %u entries left of every table", sc->host_len);
            for (u32 f = 0; f < n_tabs; f++) {
                const u32 k = sc->slice_ids[f];
                final_evals_out[2 * k] = sc->host_state[f].c0;
                final_evals_out[2 * k + 1] = sc->host_state[f].c1;
            }
        }
        const u32 n_areas = sc->poly && sc->stages.empty() && !sc->host_only ? (u32)sc->poly_tabs.size() : 0;
        for (u32 g = 0; g < n_areas; g++) {
            const u32 n_fin = sc->poly ? (u32)sc->poly_tabs[g].size() : sc->fast_nf;
            const size_t base = sc->poly_raw ? poly_raw_off(ctx) + 64 * (size_t)g : ctx->res_off;
            CHK(wait_result_at(ctx, base, sc->pairs_seq, dpk::HOST_FINALS_SLOT, 4 * n_fin, w, dpk::HOST_PAIRS_SEQ_SLOT, dpk::HOST_PAIRS_CHK_SLOT));
            for (u32 f = 0; f < n_fin; f++) {
                const u32 k = sc->poly ? sc->poly_tabs[g][f] : sc->fast_order[f];
                // a table shared by several groups is folded by each; the owner's copy counts
                if (sc->poly && sc->poly_owner[k] != (int)g) continue;
                const E2 v = gl::add(gl::e2(w[4 * f], w[4 * f + 1]), gl::mul(r, gl::e2(w[4 * f + 2], w[4 * f + 3])));
                final_evals_out[2 * k] = v.c0;
                final_evals_out[2 * k + 1] = v.c1;
            }
        }
        if (sc->fast_eq >= 0) {
            E2 v = gl::mul(sc->eq_scalar, h_eq1(sc->eq_info->point[sc->n_vars - 1], r));
            final_evals_out[2 * sc->fast_eq] = v.c0;
            final_evals_out[2 * sc->fast_eq + 1] = v.c1;
        }
        sc->finished = true;
        return DPS_OK;
    }
    if (sc->n_vars >= 1) CHK(launch_folds(sc, sc->n_vars + 1, sc->fast || sc->poly, challenge));
    if (sc->n_mles) {
        if (2 * (size_t)sc->n_mles > ctx->res_off - 64) return fail(ctx, DPS_ERR_UNSUPPORTED, "too many tables in one session");
        CHK(ensure_descs(sc));
        dpk::gather_kernel<<<(sc->n_mles + 63) / 64, 64, 0, ctx->stream>>>(sc->d_gather, sc->n_mles, ctx->d_pinned);
        HIPCHK(ctx, hipGetLastError());
    }
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    if (sc->n_mles) memcpy(final_evals_out, ctx->h_pinned, 2 * (size_t)sc->n_mles * 8);
    if (sc->fast_eq >= 0) {
        // the eq table was never folded: its value at the challenge point is the product of the one-variable factors
        E2 v = gl::mul(sc->eq_scalar, h_eq1(sc->eq_info->point[sc->n_vars - 1], gl::e2(challenge[0], challenge[1])));
        final_evals_out[2 * sc->fast_eq] = v.c0;
        final_evals_out[2 * sc->fast_eq + 1] = v.c1;
    }
    sc->finished = true;
    return DPS_OK;
}

extern "C" int32_t dps_sc_abort(dps_sc *sc)
{
    if (!sc) return DPS_ERR_INVALID;
    dps_ctx *ctx = sc->ctx;
    DeviceGuard g(ctx->device);
    if (ctx->tail_owner == sc) tail_abort(ctx);
    sc->broken = true;
    return DPS_OK;
}

extern "C" int32_t dps_sc_free(dps_sc *sc)
{
    if (!sc) return DPS_OK;
    dps_ctx *ctx = sc->ctx;
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    // a descriptor upload may still be reading the session's staging vector; the device blocks need no wait,
    // whoever gets them next uses them in stream order
    if (sc->descs_uploaded) (void)hipStreamSynchronize(ctx->stream);
    pool_free(ctx, sc->scratch);
    pool_free(ctx, sc->dev_block);
    delete sc;
    return DPS_OK;
}

extern "C" int32_t dps_sc_prove(dps_sc *sc, dps_round_fn fn, void *user, uint64_t *proof_out, uint64_t *point_out,
                                uint64_t *final_evals_out)
{
    if (!sc || !fn) return DPS_ERR_INVALID;
    dps_ctx *ctx = sc->ctx;
    if (sc->round != 0 || sc->finished) return fail(ctx, DPS_ERR_STATE, "dps_sc_prove: session already started");
    if (sc->n_vars && (!proof_out || !point_out)) return fail(ctx, DPS_ERR_INVALID, "dps_sc_prove: output buffers missing");
    const u32 npts = sc->degree + 1;
    uint64_t chal[2] = {0, 0};
    for (u32 j = 1; j <= sc->n_vars; j++) {
        uint64_t *msg = proof_out + (size_t)(j - 1) * npts * 2;
        if (const int32_t rc = dps_sc_round(sc, j == 1 ? nullptr : chal, msg); rc != DPS_OK) {
            // which round of which kind of session it was
            char where[160];
            snprintf(where, sizeof where, " [round %u of %u: %s, round kind %u, resident from %u%s%s]", j, sc->n_vars,
                     sc->fast ? "one product" : sc->poly ? "several terms" : "general", j < sc->round_kind.size() ? (u32)sc->round_kind[j] : 0u, sc->tail_j0,
                     sc->host_only ? ", on the host" : "", poly_round_weights_factored(sc, j) ? ", factored weights" : "");
            ctx->err += where;
            return rc;
        }
        if (fn(user, j, msg, npts, chal) != 0) return fail(ctx, DPS_ERR_CALLBACK, "transcript callback failed in round %u", j);
        if (!canonical(chal, 2)) return fail(ctx, DPS_ERR_CALLBACK, "transcript callback returned a non-canonical challenge in round %u", j);
        point_out[2 * (j - 1)] = chal[0];
        point_out[2 * (j - 1) + 1] = chal[1];
    }
    return dps_sc_finish(sc, sc->n_vars ? chal : nullptr, final_evals_out);
}

// ---------------------------------------------------------------------------
// DensePolynomial::evaluate for callers that must not allocate (tight serving loops, harnesses that forbid hipMalloc):
// the same value as dps_mle_evaluate, with everything beyond the table and the result kept in `scratch`.
// No hipMalloc, hipFree, stream wait or host allocation on the way; the result crosses through the context's
// pinned result area like a round message, and the call returns when it is there (the host polls for it, so this is
// not a call to make under stream capture).
// ---------------------------------------------------------------------------
namespace {

template <int KIND>
void launch_ws_dot(dps_ctx *ctx, bool full, u32 blocks, const void *t0, const u64 *t1, u32 lo, u32 hi, const dpk::FastFin &ff)
{
    if (full)
        dpk::ws_dot_kernel<KIND, true><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(t0, t1, lo, hi, ctx->ws, ff);
    else
        dpk::ws_dot_kernel<KIND, false><<<blocks, dpk::BLOCK, 0, ctx->stream>>>(t0, t1, lo, hi, ctx->ws, ff);
}

}  // namespace

extern "C" int32_t dps_mle_evaluate_noalloc(dps_ctx *ctx, const dps_mle *mle, const uint64_t *point, uint32_t n, uint64_t out[2])
{
    if (!ctx || !mle || !out || (n && !point)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate_noalloc: bad argument");
    if (mle->ctx != ctx) return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate_noalloc: the table belongs to another context");
    if (mle->pad_vars) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_evaluate_noalloc: the table is a zero-padded view");
    if (n > 40 || !is_pow2(mle->len) || (1ull << n) != mle->len)
        return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate_noalloc: point length does not match the table");
    if (n > dpk::WS_MAX_VARS)
        return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_mle_evaluate_noalloc: a table of %u variables is beyond the work area's limit of %u (use dps_mle_evaluate)", n,
                    dpk::WS_MAX_VARS);
    if (!canonical(point, 2 * (size_t)n)) return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate_noalloc: point not canonical");
    if (!ctx->ws) return fail(ctx, DPS_ERR_STATE, "dps_mle_evaluate_noalloc: the context has no work area");
    // (ending a launch that waits on the GPU for a session of this context would mean a stream wait and a memset)
    if (ctx->tail_owner) return fail(ctx, DPS_ERR_STATE, "dps_mle_evaluate_noalloc: a session of this context has a launch waiting on the GPU");
    if (mle->eq && !(mle->eq->built & 1)) {
        // An eq table whose entries nobody has read yet is not in memory (building it takes a scratch block and host
        // vectors), and need not be: the multilinear extension of eq(rho, .) at z is prod_i eq1(rho_i, z_i).
        E2 v = gl::e2_one();
        for (u32 i = 0; i < n; i++) v = gl::mul(v, h_eq1(mle->eq->point[i], gl::e2(point[2 * i], point[2 * i + 1])));
        out[0] = v.c0;
        out[1] = v.c1;
        return DPS_OK;
    }
    DeviceGuard g(ctx->device);
    // every context on a GPU shares that GPU's work area: one call at a time per device, from the first launch until the
    // result is here
    static std::mutex area_in_use[WS_MAX_DEVICES];
    std::lock_guard<std::mutex> lock(area_in_use[ctx->device]);
    dpk::WsPoint pt;
    memset(&pt, 0, sizeof pt);
    if (n) memcpy(pt.p, point, 16 * (size_t)n);
    pt.n = n;
    pt.lo = std::min<u32>(n, dpk::WS_LO_BITS);
    const u32 lo = pt.lo, hi = n - lo;
    const u32 eq_entries = (1u << lo) + (1u << hi);
    dpk::ws_eq_kernel<<<(eq_entries + dpk::BLOCK - 1) / dpk::BLOCK, dpk::BLOCK, 0, ctx->stream>>>(pt, ctx->ws);
    HIPCHK(ctx, hipGetLastError());
    const u32 blocks = std::min<u32>(1u << hi, MAX_BLOCKS);
    static_assert(MAX_BLOCKS <= dpk::WS_MAX_BLOCKS, "one partial per workgroup fits the work area");
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = ctx->ws + dpk::WS_OFF_PARTIAL;
    ff.n_blocks = blocks;
    ff.out_host = ctx->d_pinned + ctx->res_off;
    ff.seq = ++ctx->seq;
    ff.counter = reinterpret_cast<u32 *>(ctx->ws + dpk::WS_OFF_COUNTER);
    const bool full = lo == dpk::WS_LO_BITS;
    const void *t0 = mle->kind == DPS_I16 ? (const void *)mle->st->c0 : (const void *)mle->p0();
    // (no timing events here: creating one is an allocation of the runtime's)
    switch (mle->kind) {
    case DPS_BASE: launch_ws_dot<0>(ctx, full, blocks, t0, nullptr, lo, hi, ff); break;
    case DPS_EXT2: launch_ws_dot<1>(ctx, full, blocks, t0, mle->p1(), lo, hi, ff); break;
    case DPS_I64: launch_ws_dot<8>(ctx, full, blocks, t0, nullptr, lo, hi, ff); break;
    case DPS_I16: launch_ws_dot<2>(ctx, full, blocks, t0, nullptr, lo, hi, ff); break;
    default: return fail(ctx, DPS_ERR_INVALID, "dps_mle_evaluate_noalloc: unknown table kind");
    }
    HIPCHK(ctx, hipGetLastError());
    return wait_result(ctx, ff.seq, 0, 2, out);
}

// ---------------------------------------------------------------------------
// LogUp fraction-sum circuit
// ---------------------------------------------------------------------------
struct dps_logup {
    dps_ctx *ctx;
    u64 len;
    u32 n_layers;  // including the input layer
    std::shared_ptr<Storage> arena;
    std::vector<u64> layer_off;  // per layer k >= 1: offset of the numerator array; the denominator follows
    u64 out_seq = 0;             // the last launch of the build also hands the last layer's four entries to the host: under this
    u32 out_slot = 0;            // sequence number, in this one of the context's areas for them (0: it does not)
    u64 out_build = 0;           // the context's count of such builds after this one
    u32 shadow_first = 0;        // layers shadow_first.. of at most LOGUP_SHADOW_MAX entries per array also lie in host memory (0: none do)
};

static_assert(LOGUP_SHADOW_STRIDE >= dpk::LOGUP_SHADOW_WORDS, "a tree's small levels fit their area");

extern "C" int32_t dps_logup_build(dps_ctx *ctx, const dps_mle *const *cols, uint32_t n_cols, const dps_mle *numer,
                                   const uint64_t c[2], const uint64_t beta[2], dps_logup **out)
{
    if (!ctx || !cols || !out || !c || !beta || n_cols == 0) return fail(ctx, DPS_ERR_INVALID, "dps_logup_build: bad argument");
    if (n_cols > dpk::LOGUP_MAX_COLS) return fail(ctx, DPS_ERR_UNSUPPORTED, "dps_logup_build: more than %d columns", dpk::LOGUP_MAX_COLS);
    if (!canonical(c, 2) || !canonical(beta, 2)) return fail(ctx, DPS_ERR_INVALID, "dps_logup_build: challenge not canonical");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    u64 len = cols[0] ? cols[0]->len : 0;
    if (!is_pow2(len) || len < 2) return fail(ctx, DPS_ERR_INVALID, "dps_logup_build: column length must be a power of two >= 2");
    for (u32 k = 0; k < n_cols; k++)
        if (!cols[k] || cols[k]->kind != DPS_BASE || cols[k]->len != len || cols[k]->ctx != ctx || cols[k]->pad_vars)
            return fail(ctx, DPS_ERR_INVALID, "dps_logup_build: column %u is not a base table of %llu entries", k, (unsigned long long)len);
    if (numer && (numer->kind != DPS_BASE || numer->len != len)) return fail(ctx, DPS_ERR_INVALID, "dps_logup_build: multiplicity table mismatch");
    std::unique_ptr<dps_logup> lg(new (std::nothrow) dps_logup());
    if (!lg) return fail(ctx, DPS_ERR_OOM, "host allocation failed");
    lg->ctx = ctx;
    lg->len = len;
    u32 top = log2u(len);
    lg->n_layers = top;  // layers 0 .. top-1; the last has 2 entries per array
    lg->layer_off.assign(top, 0);
    u64 words = 0;
    for (u32 k = 1; k < top; k++) {
        lg->layer_off[k] = words;
        words += round_up(2 * (len >> k), 2);
    }
    auto st = std::make_shared<Storage>();
    st->ctx = ctx;
    void *p0 = nullptr, *p1 = nullptr;
    CHK(pool_alloc(ctx, std::max<u64>(words, 4) * 8, &p0));
    st->c0 = (u64 *)p0;
    CHK(pool_alloc(ctx, std::max<u64>(words, 4) * 8, &p1));
    st->c1 = (u64 *)p1;
    lg->arena = st;
    if (top >= 2) {
        dpk::LogupFirstArgs a;
        memset(&a, 0, sizeof a);
        for (u32 k = 0; k < n_cols; k++) a.cols[k] = cols[k]->p0();
        a.n_cols = n_cols;
        a.numer = numer ? numer->p0() : nullptr;
        a.c0 = c[0];
        a.c1 = c[1];
        E2 pw = gl::e2_one(), b = gl::e2(beta[0], beta[1]);
        for (u32 k = 0; k < n_cols; k++) {
            a.pw[2 * k] = pw.c0;
            a.pw[2 * k + 1] = pw.c1;
            pw = gl::mul(pw, b);
        }
        u64 half = len >> 1;
        a.half = half;
        a.n0 = st->c0 + lg->layer_off[1];
        a.n1 = st->c1 + lg->layer_off[1];
        a.d0 = a.n0 + half;
        a.d1 = a.n1 + half;
        {
            ProfScope ps(ctx, DPS_K_LOGUP, (double)len * 8.0 * (n_cols + (numer ? 1 : 0)) + (double)half * 32.0);
            dpk::logup_first_kernel<<<grid_for(half), dpk::BLOCK, 0, ctx->stream>>>(a);
            HIPCHK(ctx, hipGetLastError());
        }
        // levels of more than 2^LOGUP_TAIL_BITS entries: a launch each; the others in one launch of one workgroup
        u32 k = 2;
        for (; k < top && (len >> k) > (1ull << dpk::LOGUP_TAIL_BITS); k++) {
            u64 prev = len >> (k - 1), cur = len >> k;
            const u64 *pn0 = st->c0 + lg->layer_off[k - 1], *pn1 = st->c1 + lg->layer_off[k - 1];
            u64 *n0 = st->c0 + lg->layer_off[k], *n1 = st->c1 + lg->layer_off[k];
            ProfScope ps(ctx, DPS_K_LOGUP, (double)prev * 32.0 + (double)cur * 32.0);
            dpk::logup_next_kernel<<<grid_for(cur), dpk::BLOCK, 0, ctx->stream>>>(pn0, pn1, pn0 + prev, pn1 + prev, cur, n0, n1, n0 + cur, n1 + cur);
            HIPCHK(ctx, hipGetLastError());
        }
        if (k < top) {
            dpk::LogupTailArgs ta;
            memset(&ta, 0, sizeof ta);
            ta.c0 = st->c0;
            ta.c1 = st->c1;
            ta.n_levels = top - k;
            ta.first_cur = len >> k;
            for (u32 l = 0; l <= ta.n_levels; l++) ta.off[l] = lg->layer_off[k - 1 + l];
            lg->out_slot = (u32)(ctx->logup_builds++ % LOGUP_OUT_AREAS);
            lg->out_build = ctx->logup_builds;
            lg->out_seq = ++ctx->seq;
            ta.out_host = ctx->d_pinned + logup_out_off(ctx, lg->out_slot);
            ta.seq = lg->out_seq;
            if (ctx->d_shadow) {
                ta.shadow = ctx->d_shadow + (size_t)lg->out_slot * LOGUP_SHADOW_STRIDE;
                lg->shadow_first = k;
            }
            ProfScope ps(ctx, DPS_K_LOGUP, (double)ta.first_cur * 4 * 32.0);
            dpk::logup_tail_kernel<<<1, dpk::LOGUP_TAIL_BLOCK, 0, ctx->stream>>>(ta);
            HIPCHK(ctx, hipGetLastError());
        }
    }
    *out = lg.release();
    return DPS_OK;
}

extern "C" int32_t dps_logup_num_layers(const dps_logup *lg, uint32_t *n_layers)
{
    if (!lg || !n_layers) return DPS_ERR_INVALID;
    *n_layers = lg->n_layers;
    return DPS_OK;
}

extern "C" int32_t dps_logup_layer(const dps_logup *lg, uint32_t k, dps_mle **num, dps_mle **den)
{
    if (!lg || !num || !den) return DPS_ERR_INVALID;
    if (k < 1 || k >= lg->n_layers) return fail(lg->ctx, DPS_ERR_INVALID, "dps_logup_layer: layer %u of %u", k, lg->n_layers);
    u64 sz = lg->len >> k;
    *num = new (std::nothrow) dps_mle{lg->ctx, lg->arena, DPS_EXT2, lg->layer_off[k], sz, nullptr};
    *den = new (std::nothrow) dps_mle{lg->ctx, lg->arena, DPS_EXT2, lg->layer_off[k] + sz, sz, nullptr};
    if (!*num || !*den) return fail(lg->ctx, DPS_ERR_OOM, "host allocation failed");
    if (lg->shadow_first && k >= lg->shadow_first && sz <= dpk::LOGUP_SHADOW_MAX) {
        // the build's last launch also left this layer in host memory
        const u64 *sh = lg->ctx->h_shadow + (size_t)lg->out_slot * LOGUP_SHADOW_STRIDE + dpk::logup_shadow_off((u32)sz);
        (*num)->sh0 = sh, (*num)->sh1 = sh + sz;
        (*den)->sh0 = sh + 2 * sz, (*den)->sh1 = sh + 3 * sz;
        for (dps_mle *t : {*num, *den}) t->sh_seq = lg->out_seq, t->sh_build = lg->out_build, t->sh_slot = lg->out_slot;
    }
    return DPS_OK;
}

extern "C" int32_t dps_logup_outputs(const dps_logup *lg, uint64_t out[8])
{
    if (!lg || !out) return DPS_ERR_INVALID;
    dps_ctx *ctx = lg->ctx;
    if (lg->n_layers < 2) return fail(ctx, DPS_ERR_STATE, "dps_logup_outputs: the instance has no layer above its input");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    if (lg->out_seq) {
        // the build's last launch hands them over itself, unless a later build has taken the area since
        if (ctx->logup_builds - lg->out_build < LOGUP_OUT_AREAS && wait_result_at(ctx, logup_out_off(ctx, lg->out_slot), lg->out_seq, 0, 8, out, 9, 8) == DPS_OK)
            return DPS_OK;
    }
    u64 off = lg->layer_off[lg->n_layers - 1];
    u64 a[4], b[4];
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(a, lg->arena->c0 + off, 32, hipMemcpyDeviceToHost));
    HIPCHK(ctx, hipMemcpy(b, lg->arena->c1 + off, 32, hipMemcpyDeviceToHost));
    for (int i = 0; i < 4; i++) {
        out[2 * i] = a[i];
        out[2 * i + 1] = b[i];
    }
    return DPS_OK;
}

extern "C" int32_t dps_logup_free(dps_logup *lg)
{
    if (!lg) return DPS_OK;
    delete lg;  // (the arena goes back to the context's pool; see dps_mle_free)
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// arithmetic self-check: element-wise field operations on the device
// ---------------------------------------------------------------------------
extern "C" int32_t dps_debug_field_op(dps_ctx *ctx, int32_t op, const uint64_t *a /* 2*n: c0.., c1.. */, const uint64_t *b,
                                      uint64_t n, uint64_t *out)
{
    if (!ctx || !a || !b || !out || n == 0) return fail(ctx, DPS_ERR_INVALID, "dps_debug_field_op: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    void *p = nullptr;
    CHK(pool_alloc(ctx, 6 * n * 8, &p));
    u64 *d = (u64 *)p;
    (void)hipStreamSynchronize(ctx->stream);  // the copies below do not run on the stream; the block may have a queued user
    hipError_t e = hipMemcpy(d, a, 2 * n * 8, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(d + 2 * n, b, 2 * n * 8, hipMemcpyHostToDevice);
    if (e == hipSuccess) {
        dpk::field_op_kernel<<<(u32)((n + dpk::BLOCK - 1) / dpk::BLOCK), dpk::BLOCK, 0, ctx->stream>>>(op, d, d + n, d + 2 * n, d + 3 * n, n,
                                                                                                 d + 4 * n, d + 5 * n);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = hipMemcpy(out, d + 4 * n, 2 * n * 8, hipMemcpyDeviceToHost);
    pool_free(ctx, p);
    if (e != hipSuccess) return fail(ctx, DPS_ERR_HIP, "field op: %s", hipGetErrorString(e));
    return DPS_OK;
}

// ---------------------------------------------------------------------------
// streaming copy: the yardstick the memory counters and the evaluation kernels'
// bandwidth are read against
// ---------------------------------------------------------------------------
extern "C" int32_t dps_debug_copy(dps_ctx *ctx, uint64_t n_bytes, uint32_t reps, double *avg_ms_out)
{
    if (!ctx || n_bytes == 0 || (n_bytes & 15) || reps == 0) return fail(ctx, DPS_ERR_INVALID, "dps_debug_copy: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    void *p = nullptr;
    CHK(pool_alloc(ctx, 2 * n_bytes, &p));
    const uint4 *src = (const uint4 *)p;
    uint4 *dst = (uint4 *)((char *)p + n_bytes);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipMemsetAsync(p, 0x5a, n_bytes, ctx->stream);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const u64 n16 = n_bytes / 16;
    const u32 blocks = (u32)std::min<u64>((n16 + dpk::BLOCK - 1) / dpk::BLOCK, 8 * MAX_BLOCKS);
    if (e == hipSuccess) {
        dpk::copy_kernel<<<blocks, dpk::BLOCK, 0, ctx->stream>>>(src, dst, n16);  // untimed first touch
        e = hipEventRecord(e0, ctx->stream);
    }
    for (u32 r = 0; r < reps && e == hipSuccess; r++) {
        dpk::copy_kernel<<<blocks, dpk::BLOCK, 0, ctx->stream>>>(src, dst, n16);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipEventRecord(e1, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    pool_free(ctx, p);
    if (e != hipSuccess) return fail(ctx, DPS_ERR_HIP, "copy: %s", hipGetErrorString(e));
    if (avg_ms_out) *avg_ms_out = (double)ms / reps;
    return DPS_OK;
}

// the same for reads only: `reps` launches of a kernel that streams n_bytes in and writes nothing
extern "C" int32_t dps_debug_read(dps_ctx *ctx, uint64_t n_bytes, uint32_t reps, double *avg_ms_out)
{
    if (!ctx || n_bytes == 0 || (n_bytes & 15) || reps == 0) return fail(ctx, DPS_ERR_INVALID, "dps_debug_read: bad argument");
    DeviceGuard g(ctx->device);
    tail_abort(ctx);
    void *p = nullptr;
    CHK(pool_alloc(ctx, n_bytes + 8 * MAX_BLOCKS * 4, &p));
    const uint4 *src = (const uint4 *)p;
    u32 *sink = (u32 *)((char *)p + n_bytes);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipMemsetAsync(p, 0x5a, n_bytes, ctx->stream);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const u64 n16 = n_bytes / 16;
    const u32 blocks = (u32)std::min<u64>((n16 + dpk::BLOCK - 1) / dpk::BLOCK, 8 * MAX_BLOCKS);
    if (e == hipSuccess) {
        dpk::read_kernel<<<blocks, dpk::BLOCK, 0, ctx->stream>>>(src, n16, sink);  // untimed first touch
        e = hipEventRecord(e0, ctx->stream);
    }
    for (u32 r = 0; r < reps && e == hipSuccess; r++) {
        dpk::read_kernel<<<blocks, dpk::BLOCK, 0, ctx->stream>>>(src, n16, sink);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipEventRecord(e1, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    pool_free(ctx, p);
    if (e != hipSuccess) return fail(ctx, DPS_ERR_HIP, "read: %s", hipGetErrorString(e));
    if (avg_ms_out) *avg_ms_out = (double)ms / reps;
    return DPS_OK;
}
