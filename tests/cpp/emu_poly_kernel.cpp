// poly_kernel and poly_split_kernel (sums of several product terms over shared tables) run on the CPU through
// tests/cpp/emu/hip/hip_runtime.h: one workgroup at a time, one host thread per lane, under the host sanitizers.  These
// are the most index-heavy kernels of the library -- factor tables in LDS picked by run-time slot, the nested program
// walked with one function per depth, items of a pair spread over 1, 4 or 16 lanes, a launch that stays for the rounds
// that follow and keeps its folded tables in LDS -- and every case is compared with sums worked out by plain loops
// from the definition  G(t) = sum_terms coeff prod_factors (lo + t (hi - lo)),  weighted by the eq table where there is
// one, and with the folded tables written by plain folds.
// The nested programs are built here with the rule the library uses (the table found in most of the remaining terms is
// factored out, recursively), from terms that are also evaluated one by one: a wrong program fails the comparison.
#include <algorithm>
#include <chrono>
#include <thread>
#include <vector>

#include "dpsumcheck.h"
#include "kernels.hpp"

using gl::E2;
using gl::u32;
using gl::u64;

static u64 sm_state = 4242;
static u64 splitmix()
{
    sm_state += 0x9E3779B97F4A7C15ull;
    u64 z = sm_state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static u64 felt()
{
    for (;;) {
        const u64 v = splitmix();
        if (v < gl::P) return v;
    }
}
static E2 felt2() { return gl::e2(felt(), felt()); }

static int failures = 0;
static std::vector<u64> dyn_lds;

// a grid of gx x gy workgroups, one after the other (the kernels' static LDS is shared by whatever runs at once)
static std::vector<u32> only_blocks;  // not empty: only these workgroups (x indices) of the grid are run
template <class K, class... A>
static void launch(u32 gx, u32 gy, size_t lds_words, K kernel, A... args)
{
    gridDim = dim3(gx, gy);
    blockDim = dim3(dpk::BLOCK);
    for (u32 by = 0; by < gy; by++)
        for (u32 bx = 0; bx < gx; bx++) {
            if (!only_blocks.empty() && std::find(only_blocks.begin(), only_blocks.end(), bx) == only_blocks.end()) continue;
            dyn_lds.assign(lds_words + 16, 0xAAAAAAAAAAAAAAAAull);
            emu::default_group.reset(dpk::BLOCK);
            emu::default_group.dyn = dyn_lds.data();
            std::vector<std::thread> th;
            for (u32 t = 0; t < (u32)dpk::BLOCK; t++)
                th.emplace_back([=] {
                    threadIdx = dim3(t);
                    blockIdx = dim3(bx, by, 0);
                    kernel(args...);
                });
            for (auto &x : th) x.join();
        }
}

struct Term {
    E2 coeff;
    std::vector<u32> slots;  // table slots within the group, repeats allowed
};

// ---- the nested program of a group's terms, by the library's rule ----
struct HTerm {
    E2 coeff;
    std::vector<uint8_t> slots;
};
static dpk::PolyOp make_op(u32 kind, u32 depth, u32 slot, E2 c)
{
    dpk::PolyOp op;
    memset(&op, 0, sizeof op);
    op.c0 = c.c0, op.c1 = c.c1, op.w = gl::mul_small(c.c1, (u32)gl::W);
    op.code = kind | depth << 2 | slot << 8;
    return op;
}
static void build(std::vector<HTerm> ts, u32 depth, std::vector<dpk::PolyOp> &ops)
{
    ts.erase(std::remove_if(ts.begin(), ts.end(), [](const HTerm &t) { return t.slots.empty(); }), ts.end());
    while (!ts.empty()) {
        u32 count[dpk::POLY_MAXT] = {0};
        for (const HTerm &t : ts) {
            u32 seen = 0;
            for (uint8_t s : t.slots)
                if (!((seen >> s) & 1)) seen |= 1u << s, count[s]++;
        }
        u32 best = 0;
        for (u32 s = 1; s < (u32)dpk::POLY_MAXT; s++)
            if (count[s] > count[best]) best = s;
        std::vector<HTerm> sub, rest;
        for (HTerm &t : ts) {
            auto it = std::find(t.slots.begin(), t.slots.end(), (uint8_t)best);
            if (it == t.slots.end()) {
                rest.push_back(t);
            } else {
                t.slots.erase(it);
                sub.push_back(t);
            }
        }
        E2 ends = gl::e2_zero();
        bool inner = false;
        for (const HTerm &t : sub) {
            if (t.slots.empty())
                ends = gl::add(ends, t.coeff);
            else
                inner = true;
        }
        if (!inner) {
            ops.push_back(make_op(dpk::POLY_OP_LEAF, depth, best, ends));
        } else {
            ops.push_back(make_op(dpk::POLY_OP_ENTER, depth + 1, 0, ends));
            build(sub, depth + 1, ops);
            ops.push_back(make_op(dpk::POLY_OP_LEAVE, depth + 1, best, gl::e2_zero()));
        }
        ts = rest;
    }
}
static std::vector<dpk::PolyOp> program_of(const std::vector<Term> &terms)
{
    std::vector<HTerm> ts;
    E2 root = gl::e2_zero();
    for (const Term &t : terms) {
        HTerm h;
        h.coeff = t.coeff;
        for (u32 s : t.slots) h.slots.push_back((uint8_t)s);
        if (h.slots.empty()) root = gl::add(root, h.coeff);
        ts.push_back(h);
    }
    std::vector<dpk::PolyOp> ops;
    ops.push_back(make_op(dpk::POLY_OP_ENTER, 0, 0, root));
    build(ts, 0, ops);
    return ops;
}

static dpk::PolyTerm poly_term(const Term &t)
{
    dpk::PolyTerm pt;
    memset(&pt, 0, sizeof pt);
    pt.c0 = t.coeff.c0, pt.c1 = t.coeff.c1, pt.w = gl::mul_small(t.coeff.c1, (u32)gl::W);
    pt.n_factors = (u32)t.slots.size();
    for (size_t f = 0; f < t.slots.size(); f++) pt.slot[f] = (uint8_t)t.slots[f];
    return pt;
}

// One table of a group as a round finds it.  mode: POLY_PAIR (read as pairs), POLY_PAIR_FOLD (quads folded with r on the
// way in and, if `owned`, written), POLY_BCAST (constant in the `shift` lowest variables of the pair index).
struct Tab {
    u32 mode;
    bool base, owned;
    u32 shift;
    std::vector<u64> s0, s1, d0, d1;
    std::vector<E2> lo, hi;  // what the round evaluates, per pair (worked out here)
};
static Tab make_tab(u32 mode, bool base, bool owned, u32 shift, u64 n_pairs, E2 r)
{
    Tab t;
    t.mode = mode, t.base = base, t.owned = owned, t.shift = shift;
    const u64 n_src = mode == dpk::POLY_PAIR_FOLD ? 4 * n_pairs : mode == dpk::POLY_PAIR ? 2 * n_pairs : ((n_pairs - 1) >> shift) + 1;
    t.s0.resize(n_src + 2), t.s1.resize(base ? 0 : n_src + 2);
    for (auto &x : t.s0) x = felt();
    for (auto &x : t.s1) x = felt();
    auto at = [&](u64 k) { return gl::e2(t.s0[k], base ? 0 : t.s1[k]); };
    t.lo.resize(n_pairs), t.hi.resize(n_pairs);
    if (mode == dpk::POLY_PAIR_FOLD) {
        t.d0.assign(2 * n_pairs + 2, 0), t.d1.assign(2 * n_pairs + 2, 0);
        for (u64 i = 0; i < n_pairs; i++) {
            t.lo[i] = gl::add(at(4 * i), gl::mul(r, gl::sub(at(4 * i + 1), at(4 * i))));
            t.hi[i] = gl::add(at(4 * i + 2), gl::mul(r, gl::sub(at(4 * i + 3), at(4 * i + 2))));
        }
    } else if (mode == dpk::POLY_PAIR) {
        for (u64 i = 0; i < n_pairs; i++) t.lo[i] = at(2 * i), t.hi[i] = at(2 * i + 1);
    } else {
        for (u64 i = 0; i < n_pairs; i++) t.lo[i] = t.hi[i] = at(i >> shift);
    }
    return t;
}
static dpk::PolyTab desc_of(Tab &t)
{
    dpk::PolyTab d;
    memset(&d, 0, sizeof d);
    d.s0 = t.s0.data();
    d.s1 = t.base ? nullptr : t.s1.data();
    d.d0 = (t.mode == dpk::POLY_PAIR_FOLD && t.owned) ? t.d0.data() : nullptr;
    d.d1 = d.d0 ? t.d1.data() : nullptr;
    d.mode = t.mode;
    d.shift = t.shift;
    return d;
}

struct GroupCase {
    std::vector<Tab> tabs;
    std::vector<Term> terms;
};

// G(t) summed over the pairs by plain loops, weighted by `w` where there is an eq factor
template <int NP>
static void want_sums(const std::vector<GroupCase> &groups, u64 n_pairs, const std::vector<E2> *w, bool skip1, E2 (&want)[NP])
{
    for (int t = 0; t < NP; t++) want[t] = gl::e2_zero();
    for (const GroupCase &g : groups)
        for (u64 i = 0; i < n_pairs; i++)
            for (int t = 0; t < NP; t++) {
                if (t == 1 && skip1) continue;
                E2 G = gl::e2_zero();
                for (const Term &tm : g.terms) {
                    E2 prod = tm.coeff;
                    for (u32 s : tm.slots) prod = gl::mul(prod, gl::add(g.tabs[s].lo[i], gl::mul_base(gl::sub(g.tabs[s].hi[i], g.tabs[s].lo[i]), (u64)t)));
                    G = gl::add(G, prod);
                }
                want[t] = gl::add(want[t], w ? gl::mul(G, (*w)[i]) : G);
            }
}

static bool folds_written(const std::vector<GroupCase> &groups, u64 n_pairs)
{
    for (const GroupCase &g : groups)
        for (const Tab &t : g.tabs)
            if (t.mode == dpk::POLY_PAIR_FOLD && t.owned)
                for (u64 i = 0; i < n_pairs; i++)
                    if (t.d0[2 * i] != t.lo[i].c0 || t.d1[2 * i] != t.lo[i].c1 || t.d0[2 * i + 1] != t.hi[i].c0 || t.d1[2 * i + 1] != t.hi[i].c1) return false;
    return true;
}

// One launch of poly_kernel (split_log < 0) or of poly_split_kernel with 2^split_log lanes a pair, that exits after its
// round.  `nested`: the terms go as a nested program (poly_kernel, one group).  `inline_descs`: the single group and its
// terms travel in the kernel arguments.  `slots`: per-workgroup result areas instead of partials + ticket.
template <int NF, bool EQ, bool SKIP1>
static void run_round(const char *name, std::vector<GroupCase> groups, u64 n_pairs, E2 r, u32 gx, int split_log, bool nested, bool inline_descs, bool slots,
                      int wait = 0 /* 1: the challenge comes by mail, 2: by mail through the relay */,
                      bool fact = false /* the eq weights as products of a low and a high table (poly_kernel, stride a multiple of 2^16) */)
{
    constexpr int NP = NF + 1;
    std::vector<E2> w(n_pairs);
    std::vector<u64> q0(n_pairs), q1(n_pairs);
    for (u64 i = 0; i < n_pairs; i++) w[i] = felt2(), q0[i] = w[i].c0, q1[i] = w[i].c1;
    std::vector<u64> lq0, lq1, hq0, hq1;
    if (fact) {
        const u64 lo_n = (u64)1 << dpk::EQ_LO_BITS, hi_n = (n_pairs + lo_n - 1) / lo_n;
        lq0.resize(lo_n), lq1.resize(lo_n), hq0.resize(hi_n), hq1.resize(hi_n);
        for (u64 i = 0; i < lo_n; i++) lq0[i] = felt(), lq1[i] = felt();
        for (u64 i = 0; i < hi_n; i++) hq0[i] = felt(), hq1[i] = felt();
        for (u64 i = 0; i < n_pairs; i++) w[i] = gl::mul(gl::e2(hq0[i >> dpk::EQ_LO_BITS], hq1[i >> dpk::EQ_LO_BITS]), gl::e2(lq0[i & (lo_n - 1)], lq1[i & (lo_n - 1)]));
        // (the streamed table is not to be read)
        q0.assign(1, 0), q1.assign(1, 0);
    }
    E2 want[NP];
    want_sums<NP>(groups, n_pairs, EQ ? &w : nullptr, SKIP1, want);

    const u32 gy = (u32)groups.size();
    std::vector<dpk::PolyGroup> pg(gy);
    std::vector<dpk::PolyTerm> pt;
    std::vector<dpk::PolyOp> po;
    u32 max_tabs = 1;
    for (u32 g = 0; g < gy; g++) {
        memset(&pg[g], 0, sizeof pg[g]);
        pg[g].n_tabs = (u32)groups[g].tabs.size();
        max_tabs = std::max(max_tabs, pg[g].n_tabs);
        for (u32 k = 0; k < pg[g].n_tabs; k++) pg[g].tab[k] = desc_of(groups[g].tabs[k]);
        pg[g].term_begin = (u32)pt.size();
        for (const Term &t : groups[g].terms) pt.push_back(poly_term(t));
        pg[g].term_end = (u32)pt.size();
        if (nested) {
            const auto ops = program_of(groups[g].terms);
            pg[g].op_begin = (u32)po.size();
            po.insert(po.end(), ops.begin(), ops.end());
            pg[g].op_end = (u32)po.size();
        }
    }
    dpk::PolyArgs a;
    memset(&a, 0, sizeof a);
    if (inline_descs) {
        a.g0 = pg[0];
        if (nested)
            std::copy(po.begin(), po.end(), a.o0);
        else
            std::copy(pt.begin(), pt.end(), a.t0);
    } else {
        a.groups = pg.data();
        a.terms = pt.data();
        a.ops = po.data();
    }
    a.q0 = q0.data(), a.q1 = q1.data();
    if (fact) a.lq0 = lq0.data(), a.lq1 = lq1.data(), a.hq0 = hq0.data(), a.hq1 = hq1.data();
    a.n_pairs = n_pairs;
    a.r0 = r.c0, a.r1 = r.c1;
    a.j = 2, a.n_vars = 30;
    const u64 seq = 31;
    std::vector<u64> mail(64, 0), relay(dpk::MAIL_RELAY_WORDS, 0);
    if (wait) {
        // the mail is there before the launch (workgroups run one after the other here); the arguments hold no challenge
        a.r0 = a.r1 = 0x1234;
        a.wait_first = 1, a.mail = mail.data(), a.relay = wait == 2 ? relay.data() : nullptr, a.seq = seq, a.spin_limit = 1u << 30;
        mail[dpk::MAIL_R] = r.c0, mail[dpk::MAIL_R + 1] = r.c1, mail[dpk::MAIL_SKIP1] = SKIP1 ? 1 : 0;
        u64 chk = seq;
        for (u32 m = dpk::MAIL_R; m < (u32)dpk::MAIL_WORDS; m++) chk ^= dpk::mail_mix(mail[m], m);
        mail[dpk::MAIL_CHK] = chk, mail[dpk::MAIL_SEQ] = seq;
    }
    a.split_log = split_log < 0 ? 0 : (u32)split_log;
    a.split_cap = 4;
    a.group_stride = 1;
    const u32 n_wg = gx * gy;
    std::vector<u64> out_host(64, 0), areas(64 * (size_t)n_wg, 0), partial(2 * dpk::MAX_PTS * (size_t)n_wg + 64, 0);
    u32 counter = 0;
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = partial.data(), ff.n_blocks = n_wg, ff.out_host = out_host.data(), ff.seq = seq, ff.counter = &counter;
    ff.slots = slots ? areas.data() : nullptr;
    const size_t lds_words = (size_t)max_tabs * 4 * dpk::BLOCK;
    if (split_log < 0)
        launch(gx, gy, lds_words, dpk::poly_kernel<NF, EQ, SKIP1>, a, partial.data(), ff);
    else
        launch(gx, gy, lds_words, dpk::poly_split_kernel<NF, EQ, SKIP1>, a, partial.data(), ff);

    E2 got[NP];
    for (int t = 0; t < NP; t++) got[t] = gl::e2_zero();
    bool handed = true;
    auto take = [&](const u64 *area) {
        u64 chk = seq;
        for (int k = 0; k < 2 * NP; k++) chk ^= dpk::rotl64(area[k], k + 1);
        if (area[dpk::HOST_SEQ_SLOT] != seq || area[dpk::HOST_CHK_SLOT] != chk) handed = false;
        for (int t = 0; t < NP; t++) got[t] = gl::add(got[t], gl::e2(area[2 * t], area[2 * t + 1]));
    };
    if (slots && n_wg > 1)
        for (u32 b = 0; b < n_wg; b++) take(areas.data() + 64 * (size_t)b);
    else
        take(out_host.data());
    bool ok = handed && counter == 0 && folds_written(groups, n_pairs);
    for (int t = 0; t < NP; t++) ok = ok && gl::eq(got[t], want[t]);
    printf("%-70s NF=%d eq=%d skip1=%d pairs=%llu grid=%ux%u lanes/pair=%d nested=%d mail=%d : %s\n", name, NF, (int)EQ, (int)SKIP1, (unsigned long long)n_pairs, gx,
           gy, split_log < 0 ? 1 : 1 << split_log, (int)nested, wait, ok ? "ok" : "MISMATCH");
    for (int t = 0; t < NP; t++) printf("    q(%d) = %016llx %016llx\n", t, (unsigned long long)got[t].c0, (unsigned long long)got[t].c1);
    if (!ok) failures++;
}

// The eq weights as products of a low and a high table (poly_kernel with a grid stride of 2^16 pairs): three of the 256
// workgroups are run, each publishing to a result area of its own, and each one's sums are compared with plain loops over its
// own pairs (a workgroup's pairs: b * BLOCK + t + k * 2^16).
static void run_factored_weights(E2 r)
{
    constexpr int NF = 2, NP = 3;
    const u64 n_pairs = ((u64)1 << 16) + 300, lo_n = (u64)1 << dpk::EQ_LO_BITS;
    const u32 gx = 256;
    GroupCase g;
    for (int k = 0; k < 2; k++) g.tabs.push_back(make_tab(dpk::POLY_PAIR, true, false, 0, n_pairs, r));
    g.terms = {{felt2(), {0, 1}}, {felt2(), {1}}};
    std::vector<u64> lq0(lo_n), lq1(lo_n), hq0(2), hq1(2), q0(1, 0), q1(1, 0);
    for (u64 i = 0; i < lo_n; i++) lq0[i] = felt(), lq1[i] = felt();
    for (u64 i = 0; i < 2; i++) hq0[i] = felt(), hq1[i] = felt();
    dpk::PolyArgs a;
    memset(&a, 0, sizeof a);
    a.g0.n_tabs = 2;
    for (u32 k = 0; k < 2; k++) a.g0.tab[k] = desc_of(g.tabs[k]);
    a.g0.term_begin = 0, a.g0.term_end = 2;
    for (u32 k = 0; k < 2; k++) a.t0[k] = poly_term(g.terms[k]);
    a.q0 = q0.data(), a.q1 = q1.data();  // (the streamed table is not to be read)
    a.lq0 = lq0.data(), a.lq1 = lq1.data(), a.hq0 = hq0.data(), a.hq1 = hq1.data();
    a.n_pairs = n_pairs;
    a.r0 = r.c0, a.r1 = r.c1;
    a.j = 2, a.n_vars = 30, a.split_cap = 4, a.group_stride = 1;
    std::vector<u64> out_host(64, 0), areas(64 * (size_t)gx, 0), partial(2 * dpk::MAX_PTS * (size_t)gx + 64, 0);
    u32 counter = 0;
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = partial.data(), ff.n_blocks = gx, ff.out_host = out_host.data(), ff.seq = 77, ff.counter = &counter, ff.slots = areas.data();
    only_blocks = {0, 1, 255};
    launch(gx, 1, (size_t)2 * 4 * dpk::BLOCK, dpk::poly_kernel<NF, true, true>, a, partial.data(), ff);
    bool ok = true;
    for (u32 b : only_blocks) {
        E2 want[NP] = {gl::e2_zero(), gl::e2_zero(), gl::e2_zero()};
        for (u64 i = (u64)b * dpk::BLOCK; i < n_pairs; i += (u64)gx * dpk::BLOCK)
            for (u64 t = 0; t < (u64)dpk::BLOCK && i + t < n_pairs; t++) {
                const u64 p = i + t;
                const E2 w = gl::mul(gl::e2(hq0[p >> dpk::EQ_LO_BITS], hq1[p >> dpk::EQ_LO_BITS]), gl::e2(lq0[p & (lo_n - 1)], lq1[p & (lo_n - 1)]));
                for (int pt = 0; pt < NP; pt++) {
                    if (pt == 1) continue;
                    E2 G = gl::e2_zero();
                    for (const Term &tm : g.terms) {
                        E2 prod = tm.coeff;
                        for (u32 sl : tm.slots) prod = gl::mul(prod, gl::add(g.tabs[sl].lo[p], gl::mul_base(gl::sub(g.tabs[sl].hi[p], g.tabs[sl].lo[p]), (u64)pt)));
                        G = gl::add(G, prod);
                    }
                    want[pt] = gl::add(want[pt], gl::mul(G, w));
                }
            }
        const u64 *area = areas.data() + 64 * (size_t)b;
        u64 chk = ff.seq;
        for (int k = 0; k < 2 * NP; k++) chk ^= dpk::rotl64(area[k], k + 1);
        if (area[dpk::HOST_SEQ_SLOT] != ff.seq || area[dpk::HOST_CHK_SLOT] != chk) ok = false;
        for (int pt = 0; pt < NP; pt++) ok = ok && gl::eq(gl::e2(area[2 * pt], area[2 * pt + 1]), want[pt]);
    }
    only_blocks.clear();
    printf("%-70s pairs=%llu, workgroups 0, 1 and 255 of %u : %s\n", "eq weights as a low and a high table", (unsigned long long)n_pairs, gx, ok ? "ok" : "MISMATCH");
    if (!ok) failures++;
}

// A launch of poly_split_kernel that stays for every round down to one pair (one group, folded tables kept in LDS, the
// challenges by mail), and hands over the last pairs with its last round.  Every round's sums and the last pairs are
// compared with plain folds of reference tables.
template <int NF>
static void run_resident(const char *name, u32 n_tabs, std::vector<Term> terms, u32 log_pairs, u32 split0, u32 split_cap)
{
    constexpr int NP = NF + 1;
    const u32 n_rounds = log_pairs + 1;  // rounds j0 .. j0 + log_pairs: 2^log_pairs pairs down to one
    const u32 j0 = 5, n_vars = j0 + log_pairs;
    // reference tables: the state before round j0's fold (4 * 2^log_pairs entries)
    std::vector<std::vector<E2>> ref(n_tabs, std::vector<E2>((size_t)4 << log_pairs));
    std::vector<std::vector<u64>> s0(n_tabs), s1(n_tabs);
    std::vector<std::vector<u64>> buf0[2], buf1[2];
    for (int b = 0; b < 2; b++) buf0[b].resize(n_tabs), buf1[b].resize(n_tabs);
    for (u32 k = 0; k < n_tabs; k++) {
        for (auto &x : ref[k]) x = felt2();
        s0[k].resize(ref[k].size()), s1[k].resize(ref[k].size());
        for (size_t i = 0; i < ref[k].size(); i++) s0[k][i] = ref[k][i].c0, s1[k][i] = ref[k][i].c1;
        for (int b = 0; b < 2; b++) buf0[b][k].assign((size_t)2 << log_pairs, 0), buf1[b][k].assign((size_t)2 << log_pairs, 0);
    }
    std::vector<E2> chal(n_rounds + 1);
    for (auto &c : chal) c = felt2();
    // per-round descriptors: round j0 + i reads what round j0 + i - 1 wrote and writes to the other buffer
    std::vector<dpk::PolyGroup> pg(n_rounds);
    std::vector<dpk::PolyTerm> pt;
    for (const Term &t : terms) pt.push_back(poly_term(t));
    for (u32 i = 0; i < n_rounds; i++) {
        memset(&pg[i], 0, sizeof pg[i]);
        pg[i].n_tabs = n_tabs;
        pg[i].term_begin = 0, pg[i].term_end = (u32)pt.size();
        for (u32 k = 0; k < n_tabs; k++) {
            dpk::PolyTab &tb = pg[i].tab[k];
            tb.mode = dpk::POLY_PAIR_FOLD;
            tb.s0 = i == 0 ? s0[k].data() : buf0[(i - 1) & 1][k].data();
            tb.s1 = i == 0 ? s1[k].data() : buf1[(i - 1) & 1][k].data();
            tb.d0 = buf0[i & 1][k].data();
            tb.d1 = buf1[i & 1][k].data();
        }
    }
    dpk::PolyArgs a;
    memset(&a, 0, sizeof a);
    a.groups = pg.data();
    a.terms = pt.data();
    a.n_pairs = (u64)1 << log_pairs;
    a.r0 = chal[0].c0, a.r1 = chal[0].c1;
    a.j = j0, a.last_round = n_vars, a.n_vars = n_vars;
    a.spin_limit = 1u << 30;
    std::vector<u64> mail(64, 0), out_host(64, 0), partial(2 * dpk::MAX_PTS + 64, 0);
    a.mail = mail.data();
    a.seq = 100;
    a.split_log = split0, a.split_cap = split_cap;
    a.lds_state = 1;
    a.state_off = n_tabs * 4 * dpk::BLOCK;
    a.finish = 1;
    a.group_stride = 1;
    u32 counter = 0;
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = partial.data(), ff.n_blocks = 1, ff.out_host = out_host.data(), ff.seq = a.seq, ff.counter = &counter;
    const size_t lds_words = (size_t)n_tabs * 4 * dpk::BLOCK + (size_t)dpk::POLY_MAXT * 2 * 3 * dpk::BLOCK;

    bool ok = true;
    // the host's side: takes every round's sums as they are published, checks them, posts the next challenge
    std::thread host([&] {
        std::vector<std::vector<E2>> cur = ref;
        for (u32 i = 0; i < n_rounds; i++) {
            // fold with the challenge of the round before
            for (u32 k = 0; k < n_tabs; k++) {
                std::vector<E2> nx(cur[k].size() / 2);
                for (size_t e = 0; e < nx.size(); e++) nx[e] = gl::add(cur[k][2 * e], gl::mul(chal[i], gl::sub(cur[k][2 * e + 1], cur[k][2 * e])));
                cur[k] = nx;
            }
            const u64 np = cur[0].size() / 2;
            E2 want[NP];
            for (int t = 0; t < NP; t++) want[t] = gl::e2_zero();
            for (u64 p = 0; p < np; p++)
                for (int t = 0; t < NP; t++) {
                    if (t == 1) continue;
                    for (const Term &tm : terms) {
                        E2 prod = tm.coeff;
                        for (u32 s : tm.slots) prod = gl::mul(prod, gl::add(cur[s][2 * p], gl::mul_base(gl::sub(cur[s][2 * p + 1], cur[s][2 * p]), (u64)t)));
                        want[t] = gl::add(want[t], prod);
                    }
                }
            const u64 seq = a.seq + i;
            const auto deadline = std::chrono::steady_clock::now() + std::chrono::seconds(120);
            while (__atomic_load_n(&out_host[dpk::HOST_SEQ_SLOT], __ATOMIC_SEQ_CST) != seq && std::chrono::steady_clock::now() < deadline) std::this_thread::yield();
            u64 chk = seq;
            for (int k = 0; k < 2 * NP; k++) chk ^= dpk::rotl64(out_host[k], k + 1);
            if (out_host[dpk::HOST_SEQ_SLOT] != seq || out_host[dpk::HOST_CHK_SLOT] != chk) ok = false;
            for (int t = 0; t < NP; t++)
                if (t != 1 && !gl::eq(gl::e2(out_host[2 * t], out_host[2 * t + 1]), want[t])) ok = false;
            if (i + 1 == n_rounds) {
                // value and slope of every table's last pair came with the last round
                while (__atomic_load_n(&out_host[dpk::HOST_PAIRS_SEQ_SLOT], __ATOMIC_SEQ_CST) != seq && std::chrono::steady_clock::now() < deadline) std::this_thread::yield();
                for (u32 k = 0; k < n_tabs; k++) {
                    const u64 *w = out_host.data() + dpk::HOST_FINALS_SLOT + 4 * k;
                    const E2 d = gl::sub(cur[k][1], cur[k][0]);
                    if (w[0] != cur[k][0].c0 || w[1] != cur[k][0].c1 || w[2] != d.c0 || w[3] != d.c1) ok = false;
                }
                break;
            }
            mail[dpk::MAIL_R] = chal[i + 1].c0, mail[dpk::MAIL_R + 1] = chal[i + 1].c1;
            mail[dpk::MAIL_RA] = 0, mail[dpk::MAIL_RA + 1] = 0;
            mail[dpk::MAIL_SKIP1] = 1;
            u64 mchk = seq + 1;
            for (u32 m = dpk::MAIL_R; m < (u32)dpk::MAIL_WORDS; m++) mchk ^= dpk::mail_mix(mail[m], m);
            mail[dpk::MAIL_CHK] = mchk;
            __atomic_store_n(&mail[dpk::MAIL_SEQ], seq + 1, __ATOMIC_SEQ_CST);
        }
    });
    launch(1, 1, lds_words, dpk::poly_split_kernel<NF, false, true>, a, partial.data(), ff);
    host.join();
    printf("%-70s NF=%d tables=%u rounds=%u first share=%u : %s\n", name, NF, n_tabs, n_rounds, 1u << split0, ok ? "ok" : "MISMATCH");
    if (!ok) failures++;
}

int main()
{
    const E2 r = felt2();
    auto coeff = [] { return felt2(); };
    // ---- a fraction-sum layer: eq * (t0 t3 + t1 t2 + lambda t2 t3), folded on the way in ----
    {
        const u64 np = 700;
        GroupCase g;
        for (int k = 0; k < 4; k++) g.tabs.push_back(make_tab(dpk::POLY_PAIR_FOLD, false, true, 0, np, r));
        g.terms = {{gl::e2_one(), {0, 3}}, {gl::e2_one(), {1, 2}}, {coeff(), {2, 3}}};
        run_round<2, true, true>("layer of three terms, descriptors in the arguments", {g}, np, r, 3, -1, false, true, false);
        run_round<2, true, false>("the same, t = 1 evaluated, result areas", {g}, np, r, 2, -1, false, true, true);
        // the same sum with a pair's work spread over 1, 4 and 16 lanes
        for (int sl : {0, 2, 4}) run_round<2, true, true>("layer of three terms, lanes sharing a pair", {g}, 150, r, 2, sl, false, true, false);
        // launched ahead of its round: the challenge by mail (the first table's entries and the eq weight requested before it)
        run_round<2, true, true>("layer of three terms, launched ahead", {g}, 700, r, 3, -1, false, true, false, 1);
        run_round<2, true, true>("layer of three terms, launched ahead, mail passed on", {g}, 700, r, 3, -1, false, true, false, 2);
        run_round<2, true, true>("layer of three terms, lanes sharing a pair, launched ahead", {g}, 150, r, 2, 2, false, true, false, 1);
        run_round<2, true, true>("layer of three terms, lanes sharing a pair, ahead, mail passed on", {g}, 150, r, 3, 1, false, true, true, 2);
    }
    // ---- a linking-like expression in nested form: repeated factors, a constant, base-field and broadcast tables ----
    {
        const u64 np = 520;
        GroupCase g;
        g.tabs.push_back(make_tab(dpk::POLY_PAIR, true, false, 0, np, r));    // value chunk
        g.tabs.push_back(make_tab(dpk::POLY_PAIR, true, false, 0, np, r));    // zeroing chunk
        g.tabs.push_back(make_tab(dpk::POLY_PAIR, false, false, 0, np, r));   // eq tables as ordinary factors
        g.tabs.push_back(make_tab(dpk::POLY_PAIR, false, false, 0, np, r));
        g.tabs.push_back(make_tab(dpk::POLY_BCAST, false, false, 3, np, r));  // a table constant in the low variables
        g.terms = {{coeff(), {2, 0}}, {coeff(), {2, 0, 1}}, {coeff(), {2, 0, 1, 1}}, {coeff(), {3, 1}}, {coeff(), {3, 1, 1}}, {coeff(), {3, 4, 0}}, {coeff(), {}}};
        run_round<4, false, false>("seven monomials of degree up to 4, nested program", {g}, np, r, 3, -1, true, true, false);
        run_round<4, false, false>("the same, term by term", {g}, np, r, 3, -1, false, true, false);
        run_round<4, false, true>("the same, nested program read from memory", {g}, np, r, 2, -1, true, false, false);
        run_round<4, false, true>("the same, lanes sharing a pair", {g}, 90, r, 1, 4, false, true, true);
    }
    // ---- an opening-like shape: many groups (grid rows), a table shared by two groups and written by its owner only ----
    {
        const u64 np = 64;
        std::vector<GroupCase> groups;
        for (int gi = 0; gi < 17; gi++) {
            GroupCase g;
            const u32 nt = 2 + gi % 5;
            for (u32 k = 0; k < nt; k++) g.tabs.push_back(make_tab(dpk::POLY_PAIR_FOLD, k % 2 == 0, k != 1, 0, np, r));
            for (u32 k = 0; k + 1 < nt; k++) g.terms.push_back({coeff(), {k, k + 1}});
            groups.push_back(g);
        }
        run_round<2, false, true>("seventeen groups, ticket and gather", groups, np, r, 1, 2, false, false, false);
        run_round<2, false, true>("seventeen groups, poly_kernel", groups, np, r, 1, -1, false, false, false);
    }
    // ---- more terms than are staged in LDS (read from device memory), a full group of seven tables ----
    {
        const u64 np = 40;
        GroupCase g;
        for (int k = 0; k < 7; k++) g.tabs.push_back(make_tab(dpk::POLY_PAIR_FOLD, false, true, 0, np, r));
        for (int k = 0; k < 60; k++) g.terms.push_back({coeff(), {(u32)(k % 7), (u32)((k * 3 + 1) % 7), (u32)((k * 5 + 2) % 7)}});
        run_round<3, true, true>("sixty terms over seven tables, lanes sharing a pair", {g}, np, r, 1, 3, false, false, false);
        run_round<3, true, true>("the same, poly_kernel", {g}, np, r, 2, -1, false, false, false);
    }
    // ---- eq weights from a low and a high table: a grid of 256 workgroups (a stride of 2^16 pairs), the second step a few pairs only ----
    run_factored_weights(r);
    // ---- a launch that stays for every remaining round, folded tables in LDS, last pairs handed over ----
    run_resident<2>("resident from 64 pairs down, four lanes a pair growing to sixteen", 4, {{gl::e2_one(), {0, 3}}, {gl::e2_one(), {1, 2}}, {coeff(), {2, 3}}}, 6, 2, 4);
    run_resident<3>("resident from 16 pairs down, degree 3", 5, {{coeff(), {0, 1, 2}}, {coeff(), {3, 4}}, {coeff(), {4}}}, 4, 4, 4);
    printf("%s\n", failures ? "FAILED" : "all cases ok");
    return failures ? 1 : 0;
}
