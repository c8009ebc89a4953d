// prod_kernel (the fused fold + evaluate kernel of a product sumcheck) run on the CPU: one workgroup at a time, one host
// thread per lane, through tests/cpp/emu/hip/hip_runtime.h.  Built with the host sanitizers (address, undefined
// behaviour) and with a fill pattern for uninitialised locals (-ftrivial-auto-var-init=pattern, or =zero for a second
// opinion): a kernel body that reads something it never wrote then gives sums that differ from build to build and
// from the sums worked out here with plain loops.  tests/test_kernel_emulation.py builds and runs the quick set; the
// full set (no argument) takes a few minutes, most of it thread hand-offs.  Covers every way the kernel hands over
// its result (single workgroup, per-workgroup result areas, partials + ticket + gather), both evaluation modes, the
// eq weights streamed and taken from two small tables, a launch that waits for its challenge by mail (directly
// and through the relay), the variant that folds its sources twice on the way in, the kernel of the first two
// rounds (pair12_kernel) and the kernel that covers two rounds from sources two folds behind (quad_kernel).
#include <chrono>
#include <thread>
#include <vector>

#include "dpsumcheck.h"
#include "kernels.hpp"

using gl::E2;
using gl::u32;
using gl::u64;

static u64 sm_state = 12345;
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

template <class K, class... A>
static void launch_threads(u32 blocks, u32 threads, K kernel, A... args)
{
    gridDim = dim3(blocks);
    blockDim = dim3(threads);
    for (u32 b = 0; b < blocks; b++) {
        emu::default_group.reset(threads);
        std::vector<std::thread> th;
        for (u32 t = 0; t < threads; t++)
            th.emplace_back([=] {
                threadIdx = dim3(t);
                blockIdx = dim3(b, 0, 0);  // (indices start at zero in every dimension)
                kernel(args...);
            });
        for (auto &x : th) x.join();
    }
}
template <class K, class... A>
static void launch(u32 blocks, K kernel, A... args)
{
    launch_threads(blocks, dpk::BLOCK, kernel, args...);
}

static int failures = 0;

struct Case {
    const char *name;
    u64 n_pairs;
    u32 blocks;
    bool slots;       // per-workgroup result areas
    int wait;         // 0: challenge in the arguments, 1: by mail, every workgroup polling, 2: by mail through the relay
};

// TWO: the sources are two rounds old and are folded with `ra`, then with `r`, on the way in
template <int NF, int NB, bool FOLD, bool EQ, bool SKIP1, bool FACT, bool TWO = false>
static void run_case(const Case &c)
{
    constexpr int NP = NF + 1;
    const u64 np = c.n_pairs;
    const u64 src_len = TWO ? 8 * np : FOLD ? 4 * np : 2 * np;
    std::vector<std::vector<u64>> s0(NF), s1(NF), d0(NF), d1(NF);
    for (int f = 0; f < NF; f++) {
        s0[f].resize(src_len);
        for (auto &x : s0[f]) x = felt();
        if (f >= NB) {
            s1[f].resize(src_len);
            for (auto &x : s1[f]) x = felt();
        }
        d0[f].assign(2 * np, 0);
        d1[f].assign(2 * np, 0);
    }
    // eq weights: streamed (one per pair), or factored into a low table of 2^16 entries and a high one
    std::vector<u64> q0, q1, lq0, lq1, hq0, hq1;
    auto weight = [&](u64 i) -> E2 {
        if (!EQ) return gl::e2_one();
        if (FACT) return gl::mul(gl::e2(hq0[i >> dpk::EQ_LO_BITS], hq1[i >> dpk::EQ_LO_BITS]), gl::e2(lq0[i & 65535], lq1[i & 65535]));
        return gl::e2(q0[i], q1[i]);
    };
    if (EQ && FACT) {
        lq0.resize(65536), lq1.resize(65536);
        for (auto &x : lq0) x = felt();
        for (auto &x : lq1) x = felt();
        const u64 nh = (np + 65535) >> 16;
        hq0.resize(nh), hq1.resize(nh);
        for (auto &x : hq0) x = felt();
        for (auto &x : hq1) x = felt();
    } else if (EQ) {
        q0.resize(np), q1.resize(np);
        for (auto &x : q0) x = felt();
        for (auto &x : q1) x = felt();
    }
    const E2 r = gl::e2(felt(), felt()), ra = gl::e2(felt(), felt());

    // what the launch has to produce, by plain loops
    E2 want[NP];
    for (int t = 0; t < NP; t++) want[t] = gl::e2_zero();
    std::vector<std::vector<E2>> folded(NF, std::vector<E2>(FOLD ? 2 * np : 0));
    for (u64 i = 0; i < np; i++) {
        E2 lo[NF], hi[NF];
        for (int f = 0; f < NF; f++) {
            auto at = [&](u64 k) { return gl::e2(s0[f][k], f >= NB ? s1[f][k] : 0); };
            if (TWO) {
                auto once = [&](u64 k) { return gl::add(at(k), gl::mul(ra, gl::sub(at(k + 1), at(k)))); };
                auto twice = [&](u64 k) { return gl::add(once(k), gl::mul(r, gl::sub(once(k + 2), once(k)))); };
                lo[f] = twice(8 * i);
                hi[f] = twice(8 * i + 4);
                folded[f][2 * i] = lo[f];
                folded[f][2 * i + 1] = hi[f];
            } else if (FOLD) {
                lo[f] = gl::add(at(4 * i), gl::mul(r, gl::sub(at(4 * i + 1), at(4 * i))));
                hi[f] = gl::add(at(4 * i + 2), gl::mul(r, gl::sub(at(4 * i + 3), at(4 * i + 2))));
                folded[f][2 * i] = lo[f];
                folded[f][2 * i + 1] = hi[f];
            } else {
                lo[f] = at(2 * i);
                hi[f] = at(2 * i + 1);
            }
        }
        for (int t = 0; t < NP; t++) {
            if (t == 1 && SKIP1) continue;
            E2 prod = weight(i);
            for (int f = 0; f < NF; f++) prod = gl::mul(prod, gl::add(lo[f], gl::mul_base(gl::sub(hi[f], lo[f]), (u64)t)));
            want[t] = gl::add(want[t], prod);
        }
    }

    dpk::ProdArgs a;
    memset(&a, 0, sizeof a);
    for (int f = 0; f < NF; f++) {
        a.s0[f] = s0[f].data();
        a.s1[f] = f >= NB ? s1[f].data() : nullptr;
        a.d0[f] = d0[f].data();
        a.d1[f] = d1[f].data();
    }
    a.q0 = q0.data(), a.q1 = q1.data();
    a.lq0 = lq0.empty() ? nullptr : lq0.data(), a.lq1 = lq1.data(), a.hq0 = hq0.data(), a.hq1 = hq1.data();
    a.n_pairs = np;
    a.skip1 = SKIP1;
    std::vector<u64> mail(64, 0), relay(dpk::MAIL_RELAY_WORDS, 0), out_host(64, 0), slots(64 * 64, 0), partial(2 * NP * (size_t)c.blocks + 64, 0);
    u32 counter = 0;
    const u64 seq = 77;
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = partial.data();
    ff.n_blocks = c.blocks;
    ff.out_host = out_host.data();
    ff.seq = seq;
    ff.counter = &counter;
    ff.slots = c.slots ? slots.data() : nullptr;
    std::thread host;
    if (c.wait) {
        a.wait_first = 1;
        a.spin_limit = 1u << 30;
        a.mail = mail.data();
        a.relay = c.wait == 2 ? relay.data() : nullptr;
        // the host's side: the mail arrives while the workgroups are waiting (the first of them, run one after the other here)
        host = std::thread([&] {
            std::this_thread::sleep_for(std::chrono::milliseconds(30));
            mail[dpk::MAIL_R] = r.c0;
            mail[dpk::MAIL_R + 1] = r.c1;
            mail[dpk::MAIL_RA] = ra.c0;
            mail[dpk::MAIL_RA + 1] = ra.c1;
            mail[dpk::MAIL_SKIP1] = SKIP1;
            u64 chk = seq;
            for (u32 i = dpk::MAIL_R; i < (u32)dpk::MAIL_WORDS; i++) chk ^= dpk::mail_mix(mail[i], i);
            mail[dpk::MAIL_CHK] = chk;
            __atomic_store_n(&mail[dpk::MAIL_SEQ], seq, __ATOMIC_SEQ_CST);
        });
    } else {
        a.r0 = r.c0, a.r1 = r.c1;
        a.ra0 = ra.c0, a.ra1 = ra.c1;
    }
    a.two = TWO;
    launch(c.blocks, dpk::prod_kernel<NF, NB, FOLD, EQ, SKIP1, FACT, TWO>, a, partial.data(), ff);
    if (host.joinable()) host.join();

    E2 got[NP];
    for (int t = 0; t < NP; t++) got[t] = gl::e2_zero();
    bool handed = true;
    auto take = [&](const u64 *area) {
        u64 chk = seq;
        for (int k = 0; k < 2 * NP; k++) chk ^= dpk::rotl64(area[k], k + 1);
        if (area[dpk::HOST_SEQ_SLOT] != seq || area[dpk::HOST_CHK_SLOT] != chk) handed = false;
        for (int t = 0; t < NP; t++) got[t] = gl::add(got[t], gl::e2(area[2 * t], area[2 * t + 1]));
    };
    if (c.slots && c.blocks > 1)
        for (u32 b = 0; b < c.blocks; b++) take(slots.data() + 64 * (size_t)b);
    else
        take(out_host.data());
    bool ok = handed && counter == 0;
    for (int t = 0; t < NP; t++) ok = ok && gl::eq(got[t], want[t]);
    if (FOLD)
        for (int f = 0; f < NF && ok; f++)
            for (u64 k = 0; k < 2 * np && ok; k++) ok = d0[f][k] == folded[f][k].c0 && d1[f][k] == folded[f][k].c1;
    printf("%-58s NF=%d NB=%d fold=%d eq=%d skip1=%d fact=%d two=%d pairs=%llu workgroups=%u : %s\n", c.name, NF, NB, (int)FOLD, (int)EQ, (int)SKIP1,
           (int)FACT, (int)TWO, (unsigned long long)np, c.blocks, ok ? "ok" : "MISMATCH");
    // the sums are printed so that builds with different fills for uninitialised locals can be compared
    for (int t = 0; t < NP; t++) printf("    q(%d) = %016llx %016llx\n", t, (unsigned long long)got[t].c0, (unsigned long long)got[t].c1);
    if (!ok) failures++;
}

// pair12_kernel: the nine sums of the first two rounds of eq * f * g against plain loops over the quads.  With more than one
// step a lane the grid's stride has to be a multiple of 2^16 quads (1024 workgroups), as in the library's launches.
static void run_first_two_rounds(const char *name, u64 n_quads, u32 blocks)
{
    std::vector<u64> f(4 * n_quads), g(4 * n_quads), lq0(65536), lq1(65536), hq0((n_quads + 65535) >> 16), hq1(hq0.size());
    for (auto *v : {&f, &g, &lq0, &lq1, &hq0, &hq1})
        for (auto &x : *v) x = felt();
    E2 want[dpk::PAIR12_SUMS], want_at2[3];
    for (auto &w : want) w = gl::e2_zero();
    for (auto &w : want_at2) w = gl::e2_zero();
    for (u64 q = 0; q < n_quads; q++) {
        const E2 w = gl::mul(gl::e2(hq0[q >> 16], hq1[q >> 16]), gl::e2(lq0[q & 65535], lq1[q & 65535]));
        const u64 *a = &f[4 * q], *b = &g[4 * q];
        auto three = [&](int row, u64 fl, u64 fh, u64 gl_, u64 gh) {
            const u64 v[3] = {gl::mul(fl, gl_), gl::mul(fh, gh), gl::mul(gl::sub(fh, fl), gl::sub(gh, gl_))};
            for (int k = 0; k < 3; k++) want[3 * row + k] = gl::add(want[3 * row + k], gl::mul_base(w, v[k]));
        };
        three(0, a[0], a[1], b[0], b[1]);
        three(1, a[2], a[3], b[2], b[3]);
        // the third row: the slopes along x1 ...
        three(2, gl::sub(a[2], a[0]), gl::sub(a[3], a[1]), gl::sub(b[2], b[0]), gl::sub(b[3], b[1]));
        // ... from which the host makes round 2 at t = 2; that, by the definition, for the check below
        auto at2 = [](u64 lo, u64 hi) { return gl::sub(gl::add(hi, hi), lo); };
        const u64 fl = at2(a[0], a[2]), fh = at2(a[1], a[3]), gl_ = at2(b[0], b[2]), gh = at2(b[1], b[3]);
        const u64 v[3] = {gl::mul(fl, gl_), gl::mul(fh, gh), gl::mul(gl::sub(fh, fl), gl::sub(gh, gl_))};
        for (int k = 0; k < 3; k++) want_at2[k] = gl::add(want_at2[k], gl::mul_base(w, v[k]));
    }
    dpk::Pair12Args pa;
    pa.f = f.data(), pa.g = g.data(), pa.n_quads = n_quads;
    pa.lq0 = lq0.data(), pa.lq1 = lq1.data(), pa.hq0 = hq0.data(), pa.hq1 = hq1.data();
    std::vector<u64> out_host(64, 0), partial(2 * dpk::PAIR12_SUMS * (size_t)blocks + 64, 0);
    u32 counter = 0;
    const u64 seq = 91;
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = partial.data(), ff.n_blocks = blocks, ff.out_host = out_host.data(), ff.seq = seq, ff.counter = &counter;
    launch_threads(blocks, dpk::PAIR12_BLOCK, dpk::pair12_kernel, pa, partial.data(), ff);
    u64 chk = seq;
    for (int k = 0; k < 2 * dpk::PAIR12_SUMS; k++) chk ^= dpk::rotl64(out_host[k], k + 1);
    bool ok = out_host[dpk::PAIR12_SEQ_SLOT] == seq && out_host[dpk::PAIR12_CHK_SLOT] == chk && counter == 0;
    for (int k = 0; k < dpk::PAIR12_SUMS; k++) ok = ok && gl::eq(gl::e2(out_host[2 * k], out_host[2 * k + 1]), want[k]);
    // what the host does with the third row: 2 v(1) - v(0) + 2 lead is the product at x1 = 2
    for (int k = 0; k < 3; k++) {
        const E2 v0 = gl::e2(out_host[2 * k], out_host[2 * k + 1]), v1 = gl::e2(out_host[2 * (3 + k)], out_host[2 * (3 + k) + 1]);
        const E2 lead = gl::e2(out_host[2 * (6 + k)], out_host[2 * (6 + k) + 1]);
        ok = ok && gl::eq(gl::add(gl::sub(gl::add(v1, v1), v0), gl::add(lead, lead)), want_at2[k]);
    }
    printf("%-58s quads=%llu workgroups=%u : %s\n", name, (unsigned long long)n_quads, blocks, ok ? "ok" : "MISMATCH");
    for (int k = 0; k < dpk::PAIR12_SUMS; k++) printf("    sum %d = %016llx %016llx\n", k, (unsigned long long)out_host[2 * k], (unsigned long long)out_host[2 * k + 1]);
    if (!ok) failures++;
}

// quad_kernel: two rounds from sources that are two folds behind.  The state S it must write is worked out by folding
// the sources twice with plain loops; its eight sums are not compared with their formulas but used as the host uses
// them -- round j's q(0) and q(2) over the pairs of either kind, round j + 1's q(0) and q(2) at a random challenge -- and
// those are compared with direct sums over the pairs of S and over the pairs of S folded with that challenge.
// `wait`: as in Case.  More than one step a workgroup needs the library's stride of 2^16 quads (1024 workgroups).
template <bool SRC_BASE>
static void run_two_rounds(const char *name, u64 n_quads, u32 blocks, int wait)
{
    const u64 n_src = 16 * n_quads, n_state = 4 * n_quads;
    std::vector<u64> s0[2], s1[2], d0[2], d1[2];
    for (int f = 0; f < 2; f++) {
        s0[f].resize(n_src);
        for (auto &x : s0[f]) x = felt();
        if (!SRC_BASE) {
            s1[f].resize(n_src);
            for (auto &x : s1[f]) x = felt();
        }
        d0[f].assign(n_state, 0);
        d1[f].assign(n_state, 0);
    }
    std::vector<u64> lq0(65536), lq1(65536), hq0((n_quads + 65535) >> 16), hq1(hq0.size());
    for (auto *v : {&lq0, &lq1, &hq0, &hq1})
        for (auto &x : *v) x = felt();
    const E2 ra = gl::e2(felt(), felt()), rb = gl::e2(felt(), felt());
    // the state, by two plain folds
    std::vector<E2> S[2];
    for (int f = 0; f < 2; f++) {
        S[f].resize(n_state);
        auto at = [&](u64 k) { return gl::e2(s0[f][k], SRC_BASE ? 0 : s1[f][k]); };
        auto once = [&](u64 k) { return gl::add(at(k), gl::mul(ra, gl::sub(at(k + 1), at(k)))); };
        for (u64 e = 0; e < n_state; e++) S[f][e] = gl::add(once(4 * e), gl::mul(rb, gl::sub(once(4 * e + 2), once(4 * e))));
    }
    auto weight = [&](u64 m) { return gl::mul(gl::e2(hq0[m >> 16], hq1[m >> 16]), gl::e2(lq0[m & 65535], lq1[m & 65535])); };

    dpk::ProdArgs a;
    memset(&a, 0, sizeof a);
    for (int f = 0; f < 2; f++) {
        a.s0[f] = s0[f].data();
        a.s1[f] = SRC_BASE ? nullptr : s1[f].data();
        a.d0[f] = d0[f].data();
        a.d1[f] = d1[f].data();
    }
    a.lq0 = lq0.data(), a.lq1 = lq1.data(), a.hq0 = hq0.data(), a.hq1 = hq1.data();
    a.n_pairs = n_quads;
    a.skip1 = 1;
    std::vector<u64> mail(64, 0), relay(dpk::MAIL_RELAY_WORDS, 0), out_host(64, 0), partial(2 * dpk::QUAD_SUMS * (size_t)blocks + 64, 0);
    u32 counter = 0;
    const u64 seq = 55;
    dpk::FastFin ff;
    memset(&ff, 0, sizeof ff);
    ff.partial = partial.data(), ff.n_blocks = blocks, ff.out_host = out_host.data(), ff.seq = seq, ff.counter = &counter;
    std::thread host;
    if (wait) {
        a.wait_first = 1;
        a.spin_limit = 1u << 30;
        a.mail = mail.data();
        a.relay = wait == 2 ? relay.data() : nullptr;
        host = std::thread([&] {
            std::this_thread::sleep_for(std::chrono::milliseconds(30));
            mail[dpk::MAIL_R] = rb.c0, mail[dpk::MAIL_R + 1] = rb.c1;
            mail[dpk::MAIL_RA] = ra.c0, mail[dpk::MAIL_RA + 1] = ra.c1;
            mail[dpk::MAIL_SKIP1] = 1;
            u64 chk = seq;
            for (u32 i = dpk::MAIL_R; i < (u32)dpk::MAIL_WORDS; i++) chk ^= dpk::mail_mix(mail[i], i);
            mail[dpk::MAIL_CHK] = chk;
            __atomic_store_n(&mail[dpk::MAIL_SEQ], seq, __ATOMIC_SEQ_CST);
        });
    } else {
        a.r0 = rb.c0, a.r1 = rb.c1;
        a.ra0 = ra.c0, a.ra1 = ra.c1;
    }
    launch(blocks, dpk::quad_kernel<SRC_BASE>, a, partial.data(), ff);
    if (host.joinable()) host.join();

    u64 chk = seq;
    for (int k = 0; k < 2 * dpk::QUAD_SUMS; k++) chk ^= dpk::rotl64(out_host[k], k + 1);
    bool ok = out_host[dpk::HOST_SEQ_SLOT] == seq && out_host[dpk::HOST_CHK_SLOT] == chk && counter == 0;
    for (int f = 0; f < 2 && ok; f++)
        for (u64 e = 0; e < n_state && ok; e++) ok = d0[f][e] == S[f][e].c0 && d1[f][e] == S[f][e].c1;
    E2 v[dpk::QUAD_SUMS];
    for (int k = 0; k < dpk::QUAD_SUMS; k++) v[k] = gl::e2(out_host[2 * k], out_host[2 * k + 1]);
    const E2 A0 = v[0], A1 = v[1], Al = v[2], B0 = v[3], B2 = v[4], C0 = v[5], C1 = v[6], Cl = v[7];
    // round j: pair p of S has the weight eq1(rho, p & 1) R(p >> 1), rho any element
    const E2 rho = gl::e2(felt(), felt()), nrho = gl::sub(gl::e2_one(), rho);
    auto line = [](E2 lo, E2 hi, u64 t) { return gl::add(lo, gl::mul_base(gl::sub(hi, lo), t)); };
    E2 qj[3] = {gl::e2_zero(), gl::e2_zero(), gl::e2_zero()};
    for (u64 p = 0; p < 2 * n_quads; p++) {
        const E2 w = gl::mul(p & 1 ? rho : nrho, weight(p >> 1));
        for (u64 t = 0; t <= 2; t += 2) qj[t] = gl::add(qj[t], gl::mul(w, gl::mul(line(S[0][2 * p], S[0][2 * p + 1], t), line(S[1][2 * p], S[1][2 * p + 1], t))));
    }
    const E2 A2 = gl::add(gl::sub(gl::add(A1, A1), A0), gl::add(Al, Al));
    ok = ok && gl::eq(qj[0], gl::add(gl::mul(nrho, A0), gl::mul(rho, B0)));
    ok = ok && gl::eq(qj[2], gl::add(gl::mul(nrho, A2), gl::mul(rho, B2)));
    // round j + 1 at a challenge c: fold S with c and sum over its pairs
    const E2 c = gl::e2(felt(), felt()), cc = gl::mul(c, gl::sub(c, gl::e2_one()));
    E2 qn[3] = {gl::e2_zero(), gl::e2_zero(), gl::e2_zero()};
    for (u64 m = 0; m < n_quads; m++) {
        E2 lo[2], hi[2];
        for (int f = 0; f < 2; f++) {
            lo[f] = gl::add(S[f][4 * m], gl::mul(c, gl::sub(S[f][4 * m + 1], S[f][4 * m])));
            hi[f] = gl::add(S[f][4 * m + 2], gl::mul(c, gl::sub(S[f][4 * m + 3], S[f][4 * m + 2])));
        }
        for (u64 t = 0; t <= 2; t += 2) qn[t] = gl::add(qn[t], gl::mul(weight(m), gl::mul(line(lo[0], hi[0], t), line(lo[1], hi[1], t))));
    }
    ok = ok && gl::eq(qn[0], gl::add(gl::add(A0, gl::mul(c, gl::sub(A1, A0))), gl::mul(cc, Al)));
    ok = ok && gl::eq(qn[2], gl::add(gl::add(C0, gl::mul(c, gl::sub(C1, C0))), gl::mul(cc, Cl)));
    printf("%-58s base=%d quads=%llu workgroups=%u : %s\n", name, (int)SRC_BASE, (unsigned long long)n_quads, blocks, ok ? "ok" : "MISMATCH");
    for (int k = 0; k < dpk::QUAD_SUMS; k++) printf("    sum %d = %016llx %016llx\n", k, (unsigned long long)v[k].c0, (unsigned long long)v[k].c1);
    if (!ok) failures++;
}

int main(int argc, char **argv)
{
    // "quick": without the three-table variants and the two 256-workgroup cases (the suite's CPU run)
    const bool quick = argc > 1 && !strcmp(argv[1], "quick");
    // first round (sources read as they are), base-field and mixed sources
    run_case<2, 2, false, false, false, false>({"first round, single workgroup", 200, 1, false, 0});
    run_case<2, 2, false, false, false, false>({"first round, ragged pairs, ticket and gather", 5000, 19, false, 0});
    run_case<2, 1, false, true, false, false>({"first round with streamed eq weights, result areas", 3000, 5, true, 0});
    if (!quick) run_case<3, 1, false, false, true, false>({"first round, three tables, p(1) from the claim", 777, 2, true, 0});
    // fold + evaluate
    run_case<2, 2, true, false, true, false>({"fold of base-field sources", 4100, 18, false, 0});
    run_case<2, 0, true, false, true, false>({"fold of extension sources", 2500, 3, true, 0});
    run_case<2, 0, true, true, true, false>({"fold with streamed eq weights", 1000, 1, false, 0});
    run_case<2, 1, true, true, false, false>({"fold, mixed sources, t = 1 evaluated", 1500, 17, false, 0});
    run_case<1, 0, true, true, true, false>({"one table times eq", 900, 2, true, 0});
    if (!quick) run_case<3, 0, true, false, false, false>({"three extension tables", 600, 4, false, 0});
    // the challenge arrives by mail: every workgroup polls / the first one relays it
    run_case<2, 0, true, false, true, false>({"launch made ahead, every workgroup polls the mailbox", 1200, 3, true, 1});
    run_case<2, 2, true, false, true, false>({"launch made ahead, mail relayed by the first workgroup", 4500, 18, false, 2});
    // sources folded twice on the way in (round 3 behind the launch of the first two rounds): challenges in the arguments, by mail
    run_case<2, 2, true, false, true, false, true>({"two folds on the way in", 700, 3, false, 0});
    run_case<2, 2, true, false, true, false, true>({"two folds on the way in, ten steps a thread (walked from the far end back), ragged", 4900, 2, false, 0});
    run_case<2, 2, true, false, false, false, true>({"two folds on the way in, t = 1 evaluated, by mail", 300, 2, true, 1});
    // the first two rounds from one pass: one workgroup, several (ticket and gather by the first wavefront)
    run_first_two_rounds("first two rounds, one workgroup", 50, 1);
    run_first_two_rounds("first two rounds, ragged quads, five workgroups", 300, 5);
    // two rounds from sources two folds behind (a workgroup's step is 64 quads): one workgroup; several (ticket, gather by the
    // first wavefront); the challenges by mail, directly and through the relay
    run_two_rounds<true>("two rounds a launch, base-field sources, one workgroup", 64, 1, 0);
    run_two_rounds<true>("two rounds a launch, base-field sources, by mail", 64 * 5, 5, 1);
    run_two_rounds<false>("two rounds a launch, extension sources", 64 * 3, 3, 0);
    run_two_rounds<false>("two rounds a launch, extension sources, mail relayed", 64 * 4, 4, 2);
    // eq weights as a product of two small tables (the grid's stride is a multiple of 2^16 pairs)
    if (!quick) {
        run_two_rounds<true>("two rounds a launch, two steps in some workgroups", (1ull << 16) + 64 * 3, 1024, 0);
        run_first_two_rounds("first two rounds, two steps a lane", (1ull << 16) + 1000, 1024);
        run_case<2, 2, true, true, true, true, true>({"two folds on the way in, eq weights from two small tables", 1ull << 16, 256, false, 0});
        run_case<2, 2, false, true, false, true>({"first round, eq weights from two small tables", 3ull << 16, 256, false, 0});
        run_case<2, 2, true, true, true, true>({"fold, eq weights from two small tables", 1ull << 17, 256, false, 0});
    }
    printf("%s\n", failures ? "FAILED" : "all cases ok");
    return failures ? 1 : 0;
}
