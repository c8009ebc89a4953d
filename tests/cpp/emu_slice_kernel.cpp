// slice_kernel (the LDS-resident rounds of a product sumcheck, one or two rounds per trip to the host, one or several
// workgroups, the first of which takes the others' entries up and goes on alone) run on the CPU through tests/cpp/emu/hip/hip_runtime.h: every workgroup of a launch at once, one host
// thread per lane, and a thread that plays the host's side of the mailbox.  Every trip's sums are checked against
// sums worked out from the definitions on a reference copy of the tables: the round's q(t) by plain loops, the next
// round's sums at the sample challenges by actually folding the reference tables with 0, 1, .. and summing, the
// leading coefficient by finite differences.  Then the algebra the host relies on: the polynomial through those
// samples, evaluated at the real challenge, equals the next round's sums computed directly.  Built with the host
// sanitizers and a fill pattern for uninitialised locals by tests/test_kernel_emulation.py.
#include <chrono>
#include <memory>
#include <thread>
#include <vector>

#include "dpsumcheck.h"
#include "kernels.hpp"

using gl::E2;
using gl::u32;
using gl::u64;

static u64 sm_state = 777;
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
static u64 h_pow(u64 a, u64 e)
{
    u64 r = 1;
    while (e) {
        if (e & 1) r = gl::mul(r, a);
        a = gl::mul(a, a);
        e >>= 1;
    }
    return r;
}
static u64 h_inv(u64 a) { return h_pow(a, gl::P - 2); }

typedef std::vector<E2> Table;
static Table fold(const Table &s, E2 r)
{
    Table o(s.size() / 2);
    for (size_t i = 0; i < o.size(); i++) o[i] = gl::add(s[2 * i], gl::mul(r, gl::sub(s[2 * i + 1], s[2 * i])));
    return o;
}

// every workgroup of a launch at once
template <class K, class A>
static std::vector<std::thread> launch_all(u32 blocks, size_t lds_words, K kernel, A args, std::vector<std::unique_ptr<emu::Group>> &groups,
                                           std::vector<std::vector<u64>> &lds)
{
    gridDim = dim3(blocks);
    blockDim = dim3(dpk::BLOCK);
    std::vector<std::thread> th;
    for (u32 b = 0; b < blocks; b++) {
        groups.emplace_back(new emu::Group());
        lds.emplace_back(lds_words, 0xAAAAAAAAAAAAAAAAull);
        groups.back()->reset(dpk::BLOCK);
        groups.back()->dyn = lds.back().data();
        emu::Group *g = groups.back().get();
        for (u32 t = 0; t < (u32)dpk::BLOCK; t++)
            th.emplace_back([=] {
                emu::group = g;
                threadIdx = dim3(t);
                blockIdx = dim3(b, 0, 0);  // (indices start at zero in every dimension)
                kernel(args);
            });
    }
    return th;
}

static int failures = 0;

struct Stage {
    u32 W, j0, pend0;
    u64 src_len;
    std::vector<std::pair<u32, bool>> trips;  // first round, covers two rounds
};

struct Term {
    E2 coeff;
    std::vector<u32> tabs;
};

// A sum of n_vars variables, resident from round j0 on (j0 = 1: from the start, nothing folded yet); `wide`: workgroups of
// the first stage (1: a single stage); `single_rounds`: rounds that must start a trip of their own with t = 1 evaluated (an
// eq point with a zero coordinate there).  TERMS = false: the product of NF tables.  TERMS = true: sum_k coeff_k prod tables
// over `n_tabs` tables, NF the largest number of factors; `base_tabs` of the tables are base-field ones (j0 <= 2 only).
// `separate`: the stage of several workgroups and the single workgroup after it are two launches (as when the rounds left
// are more than one launch can run); otherwise they are one.  `host_rounds`: the last rounds are not the launch's (the
// library works them out on the host): its last trip ends before them and hands over that many more entries.
static bool g_two_behind = false;  // the first launch's sources are two folds behind its first round (as behind a launch that covered two rounds)
static bool g_first_go = false;  // launches that start with round 1 are told at once whether t = 1 is evaluated, and get no first mail
template <int NF, bool EQ, bool TERMS = false>
static void run_case(const char *name, u32 n_vars, u32 j0, u32 wide, u32 n_tabs_in, std::vector<u32> single_rounds = {}, std::vector<Term> terms = {},
                     u32 base_tabs = 0, bool separate = false, u32 host_rounds = 0)
{
    const u32 n_gpu = n_vars - host_rounds;  // the last round of a trip
    constexpr int NP = NF + 1, NPT = NF, NSMP = NF + 1, NS = NP + NSMP * NPT;
    const u32 NT = TERMS ? n_tabs_in : (u32)NF;
    if (!TERMS) {
        Term t{gl::e2_one(), {}};
        for (u32 f = 0; f < NT; f++) t.tabs.push_back(f);
        terms = {t};
    }
    const u32 first_pend = j0 == 1 ? 0 : (g_two_behind && j0 >= 3 ? 2 : 1);
    auto is_single = [&](u32 j) {
        for (u32 x : single_rounds)
            if (x == j) return true;
        return false;
    };
    // reference tables: the state before round j0's pending fold, and the challenges of every round
    std::vector<Table> ref(NT, Table((size_t)1 << (n_vars - j0 + 1 + first_pend)));
    for (u32 f = 0; f < NT; f++)
        for (auto &x : ref[f]) x = f < base_tabs ? gl::e2(felt(), 0) : felt2();
    std::vector<E2> chal(n_vars + 1);
    for (auto &c : chal) c = felt2();
    // eq storage: level l at (2 << n) - (2 << (n - l)), eq(rho_{l..n-1}, .)
    std::vector<E2> rho(n_vars);
    for (auto &x : rho) x = felt2();
    std::vector<u64> eq0((size_t)2 << n_vars, 0), eq1((size_t)2 << n_vars, 0);
    auto eq_level = [&](u32 l, u64 i) { return gl::e2(eq0[((size_t)2 << n_vars) - ((size_t)2 << (n_vars - l)) + i], eq1[((size_t)2 << n_vars) - ((size_t)2 << (n_vars - l)) + i]); };
    if (EQ)
        for (u32 l = 0; l <= n_vars; l++)
            for (u64 i = 0; i < ((u64)1 << (n_vars - l)); i++) {
                E2 v = gl::e2_one();
                for (u32 b = 0; b < n_vars - l; b++) v = gl::mul(v, ((i >> b) & 1) ? rho[l + b] : gl::sub(gl::e2_one(), rho[l + b]));
                const size_t off = ((size_t)2 << n_vars) - ((size_t)2 << (n_vars - l)) + i;
                eq0[off] = v.c0, eq1[off] = v.c1;
            }
    // the plan: stages and their trips (what the library's session planner does)
    std::vector<Stage> stages;
    {
        u32 j = j0;
        u64 entries = (u64)1 << (n_vars - j0 + 1 + first_pend);  // of the state the next stage starts from
        u32 pend = first_pend;
        if (wide > 1) {
            Stage st{wide, j, pend, entries, {}};
            u64 len_wg = (entries / wide) >> pend;
            for (;;) {
                // (the last trip is the single workgroup's, which hands the tables over)
                const bool dbl = len_wg >= 4 && j + 1 < n_gpu && !is_single(j) && !is_single(j + 1);
                st.trips.push_back({j, dbl});
                pend = dbl ? 2 : 1;
                j += pend;
                if ((len_wg >> pend) < 2 || j >= n_gpu) break;
                len_wg >>= pend;
            }
            entries = len_wg * wide;
            stages.push_back(st);
        }
        Stage st{1, j, pend, entries, {}};
        u64 len = entries >> pend;
        while (j <= n_gpu) {
            const bool dbl = len >= 4 && j + 1 <= n_gpu && !is_single(j) && !is_single(j + 1);
            st.trips.push_back({j, dbl});
            const u32 p = dbl ? 2 : 1;
            j += p;
            len >>= p;
        }
        stages.push_back(st);
    }

    std::vector<u64> mail(64, 0), relay(dpk::MAIL_RELAY_WORDS, 0), area(dpk::SL_AREA_WORDS, 0), fin(dpk::SL_FIN_AREA_WORDS, 0), gctr((size_t)dpk::SL_MAX_GROUPS * dpk::SL_GROUP_WORDS * dpk::SL_CTR_STRIDE, 0);
    u32 gate = 0;
    const u64 seq_first = 1000;
    bool ok = true;
    // device-side tables of the stage to come
    std::vector<std::vector<u64>> d0(NT), d1(NT);
    for (u32 f = 0; f < NT; f++) {
        d0[f].resize(ref[f].size()), d1[f].resize(ref[f].size());
        for (size_t i = 0; i < ref[f].size(); i++) d0[f][i] = ref[f][i].c0, d1[f][i] = ref[f][i].c1;
    }
    std::vector<Table> state = ref;  // reference state, folded as the challenges are "drawn"
    u32 folded_through = j0 - 1 - first_pend;  // the state has been folded with the challenges of rounds <= folded_through
    auto fold_to = [&](u32 round) {  // bring the reference state to the tables of `round`
        while (folded_through < round - 1) {
            folded_through++;
            for (auto &t : state) t = fold(t, chal[folded_through]);
        }
    };
    // q(t) of a round from its tables, by the definition
    auto round_sums = [&](const std::vector<Table> &tabs, u32 round, E2 *q /* NF + 1 */) {
        for (int t = 0; t <= NF; t++) q[t] = gl::e2_zero();
        for (size_t p = 0; p < tabs[0].size() / 2; p++)
            for (int t = 0; t <= NF; t++) {
                E2 g = gl::e2_zero();
                for (auto &tm : terms) {
                    E2 prod = tm.coeff;
                    for (u32 f : tm.tabs) prod = gl::mul(prod, gl::add(tabs[f][2 * p], gl::mul_base(gl::sub(tabs[f][2 * p + 1], tabs[f][2 * p]), (u64)t)));
                    g = gl::add(g, prod);
                }
                q[t] = gl::add(q[t], EQ ? gl::mul(g, eq_level(round, p)) : g);
            }
    };

    for (size_t si = 0; si < stages.size() && ok;) {
        const Stage &st = stages[si];
        const bool merged = st.W > 1 && !separate;
        const size_t last_si = merged ? si + 1 : si;
        dpk::SliceArgs a;
        memset(&a, 0, sizeof a);
        std::vector<std::vector<u64>> h0(NT), h1(NT);
        for (u32 f = 0; f < NT; f++) {
            a.s0[f] = d0[f].data();
            // a table nothing has folded yet may be a base-field one (no second limb array)
            a.s1[f] = (si == 0 && f < base_tabs) ? nullptr : d1[f].data();
            h0[f].assign(st.src_len, 0);
            h1[f].assign(st.src_len, 0);
            a.h0[f] = h0[f].data();
            a.h1[f] = h1[f].data();
        }
        // (where the workgroups leave their eq weights for the first of them)
        std::vector<u64> hw0(st.src_len, 0), hw1(st.src_len, 0);
        a.hw0 = hw0.data(), a.hw1 = hw1.data();
        a.src_len = st.src_len;
        a.pend0 = st.pend0;
        a.n_vars = n_vars;
        a.j0 = st.j0;
        a.n_trips = (u32)st.trips.size();
        for (size_t k = 0; k < st.trips.size(); k++)
            if (st.trips[k].second) a.dbl_mask |= 1u << k;
        if (merged) {
            a.n_trips2 = (u32)stages[si + 1].trips.size();
            for (size_t k = 0; k < stages[si + 1].trips.size(); k++)
                if (stages[si + 1].trips[k].second) a.dbl_mask2 |= 1u << k;
        }
        a.eq0 = eq0.data(), a.eq1 = eq1.data();
        a.mail = mail.data();
        a.relay = relay.data();
        a.spin_limit = 1u << 24;
        a.finish = last_si + 1 == stages.size();
        // a launch for round 1 told at once whether t = 1 is evaluated: its first trip gets no mail here at all
        const bool go = g_first_go && si == 0 && st.pend0 == 0 && st.j0 == 1;
        a.first_go = go ? (is_single(st.j0) ? 1 : 2) : 0;
        a.out_host = area.data();
        a.fin_out = fin.data();
        a.seq0 = seq_first + (st.j0 - j0);
        a.ctr = gctr.data();
        // (sets of counters: more of them per workgroup than the library would take, so that small launches have several)
        a.groups_log = st.W >= 8 ? 2 : st.W >= 4 ? 1 : 0;
        const u32 n_sets_wide = 1u << a.groups_log;
        a.gate = &gate;
        a.n_tabs = NT;
        a.n_terms = TERMS ? (u32)terms.size() : 0;
        for (size_t m = 0; TERMS && m < terms.size(); m++) {
            a.terms[m].c0 = terms[m].coeff.c0, a.terms[m].c1 = terms[m].coeff.c1;
            a.terms[m].w = gl::mul_small(terms[m].coeff.c1, (u32)gl::W);
            a.terms[m].n_factors = (u32)terms[m].tabs.size();
            for (size_t f = 0; f < terms[m].tabs.size(); f++) a.terms[m].slot[f] = (uint8_t)terms[m].tabs[f];
        }
        const u32 cap = (u32)((st.src_len / st.W) >> st.pend0);
        std::vector<std::unique_ptr<emu::Group>> groups;
        std::vector<std::vector<u64>> lds;
        auto threads = launch_all(st.W, dpk::slice_lds_words(NT, cap, dpk::BLOCK, EQ), dpk::slice_kernel<NF, EQ, TERMS, dpk::BLOCK>, a, groups, lds);
        // ---- the host's side ----
        std::vector<u64> seen((size_t)dpk::SL_MAX_GROUPS * dpk::SL_GROUP_WORDS, 0);  // the counters of several workgroups run on from trip to trip
        for (size_t sj = si; sj <= last_si && ok; sj++) {
            const Stage &sx = stages[sj];
            for (size_t k = 0; k < sx.trips.size() && ok; k++) {
                const u32 j = sx.trips[k].first;
                const bool dbl = sx.trips[k].second;
                const u64 seq = seq_first + (j - j0);
                const bool skip1 = !is_single(j);
                mail[dpk::MAIL_R] = j >= 1 ? chal[j - 1].c0 : 0, mail[dpk::MAIL_R + 1] = j >= 1 ? chal[j - 1].c1 : 0;
                mail[dpk::MAIL_RA] = j >= 2 ? chal[j - 2].c0 : 0, mail[dpk::MAIL_RA + 1] = j >= 2 ? chal[j - 2].c1 : 0;
                mail[dpk::MAIL_SKIP1] = skip1;
                u64 chk = seq;
                for (u32 i = dpk::MAIL_R; i < (u32)dpk::MAIL_WORDS; i++) chk ^= dpk::mail_mix(mail[i], i);
                mail[dpk::MAIL_CHK] = chk;
                if (!(go && sj == si && k == 0)) __atomic_store_n(&mail[dpk::MAIL_SEQ], seq, __ATOMIC_SEQ_CST);
                // the result: every counter of the trip's sums, tagged with the trip
                const int ns = dbl ? NS : NP;
                u64 cnt[4 * dpk::SL_MAX_SUMS] = {0};
                const auto t0 = std::chrono::steady_clock::now();
                // (several workgroups: every set of counters comes in its own part of the area, and the sets add up)
                const u32 n_sets = sx.W > 1 ? n_sets_wide : 1;
                u32 set = 0;
                for (int c = 0; c < 4 * ns && ok;) {
                    if (skip1 && c >= 4 && c < 8) {
                        cnt[c++] = 0;
                        continue;
                    }
                    const size_t at = (size_t)set * dpk::SL_GROUP_WORDS + c;
                    const u64 v = __atomic_load_n(&area[at], __ATOMIC_SEQ_CST);
                    if ((v >> 56) == dpk::sl_tag(seq)) {
                        const u64 now = v & dpk::SL_CTR_MASK;
                        if (sx.W > 1) {
                            cnt[c] += now - seen[at];
                            seen[at] = now;
                        } else {
                            cnt[c] = now;
                        }
                        area[at] = 0;
                        if (++set == n_sets) set = 0, c++;
                        continue;
                    }
                    if (std::chrono::steady_clock::now() - t0 > std::chrono::seconds(60)) {
                        printf("%s: no result for the trip of round %u (counter %d)\n", name, j, c);
                        ok = false;
                        break;
                    }
                    std::this_thread::sleep_for(std::chrono::microseconds(200));
                }
                if (!ok) break;
                auto sum_at = [&](int idx) {
                    u64 limb[2];
                    for (int l = 0; l < 2; l++) {
                        const unsigned __int128 t = (unsigned __int128)cnt[4 * idx + 2 * l] + ((unsigned __int128)cnt[4 * idx + 2 * l + 1] << 32);
                        limb[l] = gl::reduce128((u64)t, (u64)(t >> 64));
                    }
                    return gl::e2(limb[0], limb[1]);
                };
                // round j by the definition
                fold_to(j);
                E2 q[NF + 1];
                round_sums(state, j, q);
                for (int t = 0; t <= NF; t++) {
                    const E2 want = (t == 1 && skip1) ? gl::e2_zero() : q[t];
                    if (!gl::eq(sum_at(t), want)) {
                        printf("%s: round %u q(%d) differs\n", name, j, t);
                        ok = false;
                    }
                }
                if (dbl) {
                    // round j + 1 with the challenge at 0, 1, .., NF: fold the reference tables with each and sum
                    E2 c[NF + 1][NF + 1];
                    for (int s = 0; s <= NF; s++) {
                        std::vector<Table> tmp;
                        for (auto &t : state) tmp.push_back(fold(t, gl::e2((u64)s, 0)));
                        round_sums(tmp, j + 1, c[s]);
                    }
                    const int pts[4] = {0, 2, 3, 4};
                    for (int ti = 0; ti < NPT && ok; ti++) {
                        const int t = pts[ti];
                        for (int s = 0; s < NF; s++)
                            if (!gl::eq(sum_at(NP + s * NPT + ti), c[s][t])) {
                                printf("%s: round %u sample %d point %d differs\n", name, j + 1, s, t);
                                ok = false;
                            }
                        // leading coefficient = NF-th finite difference / NF!
                        E2 lead = gl::e2_zero();
                        u64 binom = 1, fact = 1;
                        for (int kk = 0; kk <= NF; kk++) {
                            const E2 term = gl::mul_base(c[kk][t], binom);
                            lead = ((NF - kk) & 1) ? gl::sub(lead, term) : gl::add(lead, term);
                            binom = binom * (u64)(NF - kk) / (u64)(kk + 1);
                        }
                        for (int kk = 2; kk <= NF; kk++) fact *= (u64)kk;
                        lead = gl::mul_base(lead, h_inv(fact));
                        if (!gl::eq(sum_at(NP + NF * NPT + ti), lead)) {
                            printf("%s: round %u leading coefficient at point %d differs\n", name, j + 1, t);
                            ok = false;
                        }
                        // what the host does with them: the polynomial at the real challenge = the round's sum computed directly
                        const E2 r = chal[j];
                        E2 val = gl::e2_zero(), vanish = gl::e2_one();
                        for (int kk = 0; kk < NF; kk++) {
                            E2 num = gl::e2_one();
                            u64 den = 1;
                            for (int m = 0; m < NF; m++)
                                if (m != kk) {
                                    num = gl::mul(num, gl::sub(r, gl::e2((u64)m, 0)));
                                    den = gl::mul(den, gl::sub((u64)kk, (u64)m));
                                }
                            val = gl::add(val, gl::mul(gl::mul_base(num, h_inv(den)), sum_at(NP + kk * NPT + ti)));
                            vanish = gl::mul(vanish, gl::sub(r, gl::e2((u64)kk, 0)));
                        }
                        val = gl::add(val, gl::mul(vanish, sum_at(NP + NF * NPT + ti)));
                        std::vector<Table> next;
                        for (auto &tb : state) next.push_back(fold(tb, r));
                        E2 q2[NF + 1];
                        round_sums(next, j + 1, q2);
                        if (!gl::eq(val, q2[t])) {
                            printf("%s: round %u point %d: interpolation at the challenge differs from the direct sum\n", name, j + 1, t);
                            ok = false;
                        }
                    }
                }
            }
        }
        if (!ok) {
            // let the launch leave: the abort sequence number, as the library does
            __atomic_store_n(&mail[dpk::MAIL_SEQ], dpk::MAIL_ABORT_SEQ, __ATOMIC_SEQ_CST);
        }
        for (auto &t : threads) t.join();
        if (!ok) break;
        if (gate != 0) ok = false, printf("%s: gate left at %u\n", name, gate);
        for (u64 c : gctr)
            if (c) ok = false, printf("%s: a counter was left at %llx\n", name, (unsigned long long)c);
        if (st.W > 1) {
            // what the workgroups left behind (for the first of them, or for the next launch) is the reference state of
            // their last trip's round
            std::vector<Table> at_last = ref;
            {
                // fold a copy of the reference from the start (the state itself may be further on already)
                u32 through = j0 - 1 - first_pend;
                while (through < st.trips.back().first - 1) {
                    through++;
                    for (auto &t : at_last) t = fold(t, chal[through]);
                }
            }
            const u64 left = at_last[0].size();
            if (left != stages[si + 1].src_len) ok = false, printf("%s: stage leaves %llu entries, the next expects %llu\n", name, (unsigned long long)left, (unsigned long long)stages[si + 1].src_len);
            for (u32 f = 0; f < NT && ok; f++) {
                d0[f].assign(left, 0), d1[f].assign(left, 0);
                for (u64 i = 0; i < left; i++) {
                    if (h0[f][i] != at_last[f][i].c0 || h1[f][i] != at_last[f][i].c1) {
                        printf("%s: handed-over entry %llu of table %u differs\n", name, (unsigned long long)i, f);
                        ok = false;
                        break;
                    }
                    d0[f][i] = h0[f][i], d1[f][i] = h1[f][i];
                }
            }
            if (stages[si + 1].pend0 != (st.trips.back().second ? 2u : 1u)) ok = false, printf("%s: pending folds disagree\n", name);
        }
        if (last_si + 1 == stages.size()) {
            // what is left of every table, published with the last trip: the state of that trip's first round
            const auto &last = stages[last_si].trips.back();
            fold_to(last.first);
            const u64 seq = seq_first + (last.first - j0);
            const u32 len_left = (u32)state[0].size();
            if (len_left != ((last.second ? 4u : 2u) << host_rounds)) ok = false, printf("%s: %u entries left\n", name, len_left);
            u64 c = seq;
            const u32 n_words = NT * len_left * 2;
            for (u32 i = 0; i < n_words; i++) c ^= dpk::sl_fin_mix(fin[i], i);
            if (fin[dpk::SL_FIN_SEQ_SLOT] != seq || fin[dpk::SL_FIN_CHK_SLOT] != c) ok = false, printf("%s: last entries not handed over\n", name);
            for (u32 f = 0; f < NT && ok; f++)
                for (u32 e = 0; e < len_left; e++)
                    if (fin[2 * (f * len_left + e)] != state[f][e].c0 || fin[2 * (f * len_left + e) + 1] != state[f][e].c1)
                        ok = false, printf("%s: last entry %u of table %u differs\n", name, e, f);
        }
        si = last_si + 1;
    }
    size_t n_trips = 0;
    for (auto &s : stages) n_trips += s.trips.size();
    printf("%-60s degree %d eq=%d n=%u from round %u, %zu stage(s), %zu trips for %u rounds : %s\n", name, NF, (int)EQ, n_vars, j0, stages.size(), n_trips,
           n_gpu - j0 + 1, ok ? "ok" : "MISMATCH");
    if (!ok) failures++;
}

int main()
{
    run_case<2, true>("two tables and eq, one workgroup, trips of two rounds", 9, 2, 1, 0);
    run_case<2, true>("odd number of rounds: the last trip covers one", 10, 2, 1, 0);
    run_case<1, true>("one table and eq", 7, 2, 1, 0);
    run_case<3, false>("three tables, no eq", 8, 3, 1, 0);
    run_case<2, false>("two tables, rounds that must go alone (t = 1 evaluated)", 9, 2, 1, 0, {4, 7});
    run_case<2, true>("four workgroups, then one", 12, 3, 4, 0);
    run_case<2, true>("two workgroups down to one entry each, rounds that must go alone", 11, 3, 2, 0, {6});
    run_case<2, true>("four workgroups and the single one as two launches", 12, 3, 4, 0, {}, {}, 0, true);
    run_case<2, true>("from round 1 (nothing folded yet)", 8, 1, 1, 0);
    // sums of several terms: a LogUp layer eq (a d + b c + lambda c d), then higher degrees, base-field tables, constants
    const Term la{felt2(), {0, 3}}, lb{felt2(), {1, 2}}, lc{felt2(), {2, 3}};
    run_case<2, true, true>("fraction-sum layer: 4 tables, 3 terms, from round 1", 7, 1, 1, 4, {}, {la, lb, lc});
    run_case<2, true, true>("the same over 4 workgroups, then one", 11, 2, 4, 4, {}, {la, lb, lc});
    run_case<3, false, true>("degree 3 without eq: repeated and single factors, a constant term", 8, 2, 1, 5, {5},
                             {Term{felt2(), {0, 1, 2}}, Term{felt2(), {3, 3, 4}}, Term{felt2(), {4}}, Term{felt2(), {}}});
    run_case<4, false, true>("degree 4, base-field tables, from round 1", 6, 1, 1, 3, {}, {Term{felt2(), {0, 0, 1, 2}}, Term{felt2(), {1, 2}}}, 2);
    run_case<2, true, true>("base-field tables folded once on the way in (from round 2)", 9, 2, 2, 3, {}, {Term{felt2(), {0, 1}}, Term{felt2(), {1, 2}}}, 2);
    // the stacked products of an einsum: 16 tables, 8 terms of two factors each, every round resident
    std::vector<Term> stacked;
    for (u32 i = 0; i < 8; i++) stacked.push_back(Term{felt2(), {2 * i, 2 * i + 1}});
    run_case<2, false, true>("16 tables, 8 products, from round 1", 8, 1, 1, 16, {}, stacked);
    run_case<2, false, true>("the same with an odd number of rounds", 7, 1, 1, 16, {}, stacked);
    // launches that leave the last rounds to the host: more entries handed over than a wavefront has lanes
    run_case<2, true>("two tables and eq, the last four rounds left out", 10, 2, 1, 0, {}, {}, 0, false, 4);
    run_case<2, true>("the same with a single round as the last trip", 9, 2, 1, 0, {}, {}, 0, false, 4);
    run_case<2, true>("four workgroups, then one, the last three rounds left out", 12, 3, 4, 0, {}, {}, 0, false, 3);
    run_case<2, false, true>("16 tables, 8 products, the last two rounds left out", 8, 1, 1, 16, {}, stacked, 0, false, 2);
    run_case<2, true, true>("fraction-sum layer over 4 workgroups, the last three rounds left out", 11, 2, 4, 4, {}, {la, lb, lc}, 0, false, 3);
    // sources two folds behind the first round: entries asked for before the first mail (few items a thread) and after it (many)
    g_two_behind = true;
    run_case<2, true>("two tables and eq from round 3, sources two folds behind", 9, 3, 1, 0);
    run_case<2, true>("the same with more entries than are asked for ahead", 11, 3, 1, 0);
    run_case<2, true>("four workgroups from round 3, sources two folds behind", 12, 3, 4, 0);
    run_case<2, false, true>("16 tables, 8 products from round 3, sources two folds behind", 8, 3, 1, 16, {}, stacked, 0, false, 2);
    g_two_behind = false;
    // launches for round 1 whose first trip starts without mail
    g_first_go = true;
    run_case<2, true>("from round 1, first trip without mail", 8, 1, 1, 0);
    run_case<2, true, true>("fraction-sum layer from round 1 over 4 workgroups, first trip without mail", 10, 1, 4, 4, {}, {la, lb, lc}, 0, false, 3);
    run_case<2, false>("two tables from round 1, t = 1 evaluated in round 1, first trip without mail", 8, 1, 1, 0, {1, 4});
    run_case<2, false, true>("16 tables, 8 products, from round 1, first trip without mail", 8, 1, 1, 16, {}, stacked, 0, false, 2);
    g_first_go = false;
    printf("%s\n", failures ? "FAILED" : "all cases ok");
    return failures ? 1 : 0;
}
