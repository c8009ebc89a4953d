#!/usr/bin/env python3
"""Benchmark of the sumcheck prover hot path on one MI355X.

Workload (the configuration the metric is quoted on): the degree-3 sumcheck of
eq(r, x) * f(x) * g(x) over n = 24 variables; f and g are 2^24 uniform
base-field values, r a uniform extension-field point.  A step is one complete
proof (session set-up, 24 rounds with the BLAKE3 transcript on the host, final
evaluations) with the tables already resident in HBM.

One JSON line is printed: the metric, the roofline of the dominant kernel from
HIP events recorded by the library around its own launches, and the CPU checker
timed on the host cores as the baseline.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
P = 0xFFFFFFFF00000001
# Counters cannot be read from inside this script: the HBM bytes of the dominant launch (rounds 3 and 4) at n = 24 (rocprofv3 FETCH_SIZE and
# WRITE_SIZE, each scaled by what the same counter reads for the library's plain copy kernel) and the vector-ALU issue
# shares of the first launch and of the dominant one are taken from the committed summaries of those runs, as "key: value" lines.
TRAFFIC_PROFILE = "profiles/quad_kernel_cfg3_n24_hbm_traffic.txt"
VALU_PROFILE = "profiles/quad_kernel_cfg3_n24_valu.txt"


def profile_value(path, key):
    """the number on the line 'key: number' of a committed profile summary, or None"""
    try:
        for line in open(os.path.join(ROOT, path)):
            if line.strip().startswith(key + ":"):
                return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def rand_base(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    v = rng.integers(0, 2**64, size=n, dtype=np.uint64)
    return np.where(v >= np.uint64(P), v - np.uint64(P), v)


def _timed(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    ts = []
    for _ in range(steps):
        t0 = time.perf_counter()
        out = fn()
        ts.append(time.perf_counter() - t0)
    return 1e3 * sum(ts) / len(ts), 1e3 * min(ts), out


def rand_i64(shape, seed):
    return np.random.Generator(np.random.PCG64(seed)).integers(-2048, 2048, size=shape, dtype=np.int64)


def other_config(args):
    """The remaining configurations, one JSON line each: a step is one complete proof of that configuration
    with its inputs resident in HBM (the einsum configurations also report the step that uploads host tensors).  The CPU leg times the checker on the same statement where it has a driver."""
    dp = importlib.import_module("deep-prove_amd")
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    orc = None
    if not args.no_cpu:
        import dpsc_oracle as orc

        orc.select(True)
    ctx = dp.Context(0)
    one = np.array([1, 0], dtype=np.uint64)
    cfg = args.config
    cpu_ms, exact, extra = None, None, {}
    if cfg == "1":
        n = 16
        f, g = rand_base(1 << n, 1), rand_base(1 << n, 2)
        mf, mg = ctx.mle_from_base(f), ctx.mle_from_base(g)
        terms = [(one, [0, 1])]
        prover = ctx.sumcheck_prover(n, [mf, mg], terms)
        run = lambda: prover(dp.Transcript(b"bench"))
        workload, metric = "cfg1: sum f*g, n=16, base field, degree 2", "sumcheck prove ms @ n=16 deg-2 base"
        if orc:
            tabs = [orc.embed_base(f), orc.embed_base(g)]
            cpu_ms, _, ref = _timed(lambda: orc.sc_prove(n, tabs, terms, orc.OracleTranscript(b"bench")), 5, 1)
            got = run()
            exact = bool(all((a == b).all() for a, b in zip(got, ref)))
    elif cfg in ("2", "4"):
        if cfg == "2":
            ops, lhs, rhs = [("ik", "kj", "ij")], rand_i64((512, 768), 11), [rand_i64((768, 3072), 12)]
            workload, metric = "cfg2: A[512x768] @ W[768x3072], partial evaluation + 10-variable degree-2 sumcheck", "einsum prove ms (gpt2 mlp up-projection)"
            nv_out = 9 + 12
        else:
            ops, lhs, rhs = [("hsd", "htd", "hst")], rand_i64((8, 512, 256), 13), [rand_i64((8, 512, 256), 14)]
            workload, metric = "cfg4: Q,K[8x512x256] 'hsd,htd->hst', partial evaluation + 8-variable sumcheck over 16 tables", "einsum prove ms (attention scores)"
            nv_out = 3 + 9 + 9
        pt = np.stack([rand_base(nv_out, 5), rand_base(nv_out, 6)], axis=-1)
        claims = [(pt, one)]  # timing only: the claimed value does not change the work
        dl, dr = dp.Tensor(ctx, lhs, 64), [dp.Tensor(ctx, x, 64) for x in rhs]
        run = lambda: dp.einsum_prove(ctx, ops, dl, dr, claims, dp.Transcript(b"bench"))
        from_host = dp.einsum_prove(ctx, ops, lhs, rhs, claims, dp.Transcript(b"bench"))
        got = run()
        exact_vs_host_path = bool((got["proof"] == from_host["proof"]).all() and (got["evaluations"] == from_host["evaluations"]).all())
        d16, r16 = dp.Tensor(ctx, lhs, 16), [dp.Tensor(ctx, x, 16) for x in rhs]
        got16 = dp.einsum_prove(ctx, ops, d16, r16, claims, dp.Transcript(b"bench"))
        exact_vs_host_path = exact_vs_host_path and bool((got16["proof"] == from_host["proof"]).all())
        extra["int16_storage_ms"] = round(_timed(lambda: dp.einsum_prove(ctx, ops, d16, r16, claims, dp.Transcript(b"bench")), args.steps, args.warmup)[0], 4)
        extra["with_upload_of_int64_host_tensors_ms"] = round(_timed(lambda: dp.einsum_prove(ctx, ops, lhs, rhs, claims, dp.Transcript(b"bench")), args.steps, args.warmup)[0], 4)
        extra["same_bits_as_host_tensor_path"] = exact_vs_host_path
        extra["note"] = "value: int64 tensors resident on the device (weights and activations uploaded once, outside the step)"
        if orc:
            # the checker's restatement of the whole driver: partial evaluations, batched sumcheck, input claims
            cpu_ms, _, (ref, _otr) = _timed(lambda: orc.einsum_prove(ops, lhs, rhs, claims, b"bench"), 1, 0)
            exact = bool((got["proof"] == ref["proof"]).all() and (got["evaluations"] == ref["evaluations"]).all()
                         and all((a[0] == b[0]).all() and (a[1] == b[1]).all() for a, b in zip(got["claims"], ref["claims"])))
    elif cfg == "5":
        log_l, log_t = 22, 16
        rng = np.random.Generator(np.random.PCG64(600))
        t_in = np.arange(1 << log_t, dtype=np.uint64)
        t_out = (t_in * np.uint64(40503) + np.uint64(17)) & np.uint64(0xFFFF)
        idx = rng.integers(0, 1 << log_t, size=1 << log_l)
        mult = np.bincount(idx, minlength=1 << log_t).astype(np.uint64)
        tr0 = dp.Transcript(b"bench")
        c, beta = tr0.append_and_sample(b"c"), tr0.append_and_sample(b"beta")
        look_cols = [t_in[idx], t_out[idx]]
        look_d = [dict(cols=[ctx.mle_from_base(x) for x in look_cols], numer=None, c=c, beta=beta)]
        tab_d = [dict(cols=[ctx.mle_from_base(t_in), ctx.mle_from_base(t_out)], numer=ctx.mle_from_base(mult), c=c, beta=beta)]

        def run():
            t = tr0.clone()
            return dp.logup_batch_prove(ctx, look_d, t), dp.logup_batch_prove(ctx, tab_d, t)

        workload = "cfg5: LogUp-GKR, 2^22 lookups (2 columns) into a 2^16-entry table with multiplicities; lookup batch + table batch"
        metric = "logup-gkr prove ms @ 2^22 lookups"
        if orc:
            def cpu():
                t = orc.OracleTranscript(b"bench")
                t.append_and_sample(b"c"), t.append_and_sample(b"beta")
                return (orc.logup_batch_prove([dict(cols=look_cols, numer=None, c=c, beta=beta)], t),
                        orc.logup_batch_prove([dict(cols=[t_in, t_out], numer=mult, c=c, beta=beta)], t))

            cpu_ms, _, ref = _timed(cpu, 1, 0)
            got = run()
            exact = bool((got[0] == ref[0]).all() and (got[1] == ref[1]).all())
    elif cfg == "linking":
        # the activation after GPT-2's MLP up-projection, [512 x 3072], through a signed 8-bit table with one zeroing chunk
        lcfg = dict(variant="standard", shape=[512, 3072], value_chunks=1, zero_chunks=1, bit_size=8, signed=True, min_out=-128, max_out=127,
                    input_sign="positive", norm_sum=False, has_weight=False)
        nv = 9 + 12
        rng = np.random.Generator(np.random.PCG64(91))
        value = rng.integers(-128, 128, size=1 << nv, dtype=np.int64)
        top = rng.integers(-1, 2, size=1 << nv, dtype=np.int64)
        lcp, lp = np.stack([rand_base(nv, 92), rand_base(nv, 93)], axis=-1), np.stack([rand_base(nv, 94), rand_base(nv, 95)], axis=-1)
        gpu = [ctx.mle_from_i64(value, nv), ctx.mle_from_i64(top, nv)]
        run = lambda: dp.linking_prove(ctx, lcfg, gpu, dp.Transcript(b"bench"), lcp, lp)
        workload = "lookup-linking sumcheck of a [512 x 3072] activation: signed 8-bit table, one value chunk + one zeroing chunk, 21 variables, degree 4"
        metric = "lookup linking prove ms"
        if orc:
            tabs = [orc.embed_i64(value), orc.embed_i64(top)]
            cpu_ms, _, ref = _timed(lambda: orc.linking_prove(lcfg, tabs, orc.OracleTranscript(b"bench"), lcp, lp), 2, 0)
            got = run()
            exact = bool((got[0] == ref[0]).all() and (got[2] == ref[2]).all())
    else:
        # the reference's test_poly_commit shape with chunks of 2^10 (zkml/src/poly_commit/mod.rs:224-409)
        rng = np.random.Generator(np.random.PCG64(77))
        sizes = [int(x) for x in rng.integers(10, 16, size=5)] + [int(x) for x in rng.integers(10, 14, size=9)]
        polys_h, polys_d, claims = [], [], []
        for i, nv in enumerate(sizes):
            full = np.stack([rand_base(1 << nv, 100 + i), rand_base(1 << nv, 200 + i)], axis=-1)
            m = min(nv, 10)
            chunks = [full[k << m:(k + 1) << m] for k in range(1 << (nv - m))]
            whole = ctx.mle_from_ext2(full)
            polys_h.append(chunks)
            polys_d.append([whole.view(k << m, m) for k in range(len(chunks))])
            cls = []
            for k in range(2 if (i < 5 and i % 2) else 1):
                pt = np.stack([rand_base(nv, 300 + 10 * i + k), rand_base(nv, 400 + 10 * i + k)], axis=-1)
                cls.append((pt, whole.evaluate(pt)))
            claims.append(cls)
        # (the call's arguments -- 132 table handles, 16 points -- are marshalled once: the step times the library, not numpy)
        prover = dp.claims_batching_prover(ctx, polys_d, claims)
        run = lambda: prover(dp.Transcript(b"bench"))
        workload = "claims-batching sumcheck of the opening proof: 14 polynomials of 10..15 variables in chunks of 2^10, 16 claims"
        metric = "claims batching prove ms"
        if orc:
            cpu_ms, _, ref = _timed(lambda: orc.claims_batching_prove(polys_h, claims, orc.OracleTranscript(b"bench")), 3, 1)
            got = run()
            exact = bool(all((a == b).all() for a, b in zip(got, ref)))
    ms, best, _ = _timed(run, args.steps, args.warmup)
    out = {"metric": metric, "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms, 4), "min_step_ms": round(best, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "u64 (Goldilocks, ext2)", "data": "synthetic", "config": {"workload": workload}}
    out.update(extra)
    if cpu_ms is not None:
        out["cpu_baseline"] = {"value": round(cpu_ms, 2), "unit": "ms", "cores": orc.num_threads(), "kind": "port",
                               "sample": "the same statement, whole; C restatement with OpenMP"}
        out["speedup_vs_cpu"] = round(cpu_ms / ms, 1)
        out["bit_exact"] = exact
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--nvars", type=int, default=24, help="variables of the sum (24 is the benchmark configuration)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true", help="benchmark configuration only: leave the other configurations out of the record")
    ap.add_argument("--config", default="3", choices=["1", "2", "3", "4", "5", "opening", "linking"],
                    help="3 (default) is the benchmark configuration; the others time the remaining configurations the same way")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    if args.config != "3":
        print(json.dumps(other_config(args)))
        return

    dp = importlib.import_module("deep-prove_amd")
    n = args.nvars
    f, g = rand_base(1 << n, 1), rand_base(1 << n, 2)
    r = np.stack([rand_base(n, 3), rand_base(n, 4)], axis=-1)
    one = np.array([1, 0], dtype=np.uint64)
    terms = [(one, [2, 0, 1])]  # eq * f * g

    ctx = dp.Context(0)
    t0 = time.perf_counter()
    mf, mg = ctx.mle_from_base(f), ctx.mle_from_base(g)
    ctx.sync()
    upload_s = time.perf_counter() - t0

    # eq table build, timed on its own
    me = ctx.eq_build(r)
    ctx.sync()
    eq_times = []
    for _ in range(5):
        t0 = time.perf_counter()
        tmp = ctx.eq_build(r)
        ctx.sync()
        eq_times.append(time.perf_counter() - t0)
        tmp.free()
    eq_ms = 1e3 * sorted(eq_times)[len(eq_times) // 2]

    # handles and terms are marshalled once; every call is still a whole proof: session, 24 rounds, final evaluations
    prover = ctx.sumcheck_prover(n, [mf, mg, me], terms)

    def prove():
        tr = dp.Transcript(b"bench")
        return prover(tr), tr

    def timed_loop(fn, steps):
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        ctx.sync()
        return 1e3 * (time.perf_counter() - t0) / steps

    for _ in range(args.warmup):
        prove()
    ctx.sync()
    per_step, proofs = [], []
    t_begin = time.perf_counter()
    for _ in range(args.steps):
        t0 = time.perf_counter()
        (proof, point, finals), tr = prove()
        per_step.append(time.perf_counter() - t0)
        proofs.append(proof)
    ctx.sync()
    total_s = time.perf_counter() - t_begin
    ms_per_step = 1e3 * total_s / args.steps
    # every step proves the same statement: all proofs must be identical
    repeatable = all((q == proofs[0]).all() for q in proofs)

    # The caller of the reference's hadamard prover holds the value of the sum (the claim it reduces, hadamard.rs:117-121);
    # stated to the engine, round 1 takes p(1) from it.  Same proof; reported beside the headline, which does not use it.
    p10 = [int(x) for x in proof[0][0]], [int(x) for x in proof[0][1]]
    claim = np.array([(p10[0][0] + p10[1][0]) % P, (p10[0][1] + p10[1][1]) % P], dtype=np.uint64)
    claimed = ctx.sumcheck_prover(n, [mf, mg, me], terms, claim=claim)
    same_with_claim = bool((claimed(dp.Transcript(b"bench"))[0] == proofs[0]).all())
    for _ in range(args.warmup):
        claimed(dp.Transcript(b"bench"))
    claimed_ms = timed_loop(lambda: claimed(dp.Transcript(b"bench")), args.steps)

    # A fresh point every step, as in the reference's flow (hadamard.rs:103-115 builds the eq table for each proof): the eq
    # build is inside the timed region.  The statement changes with the point, so these proofs are not compared.
    points = [np.stack([rand_base(n, 1000 + 2 * k), rand_base(n, 1001 + 2 * k)], axis=-1) for k in range(args.steps + 2)]

    def fresh(k):
        e = ctx.eq_build(points[k])
        out = ctx.sumcheck_prove(n, [mf, mg, e], terms, dp.Transcript(b"bench"))
        e.free()
        return out

    fresh(args.steps), fresh(args.steps + 1)
    ctx.sync()
    t0 = time.perf_counter()
    for k in range(args.steps):
        fresh(k)
    ctx.sync()
    fresh_ms = 1e3 * (time.perf_counter() - t0) / args.steps

    # same steps again with the library's HIP events on, for per-kernel durations
    ctx.profile(True)
    ctx.profile_reset()
    for _ in range(args.steps):
        prove()
    stats = ctx.profile_read()
    ctx.profile(False)

    def gbs(by, ms):
        return by / (ms * 1e-3) / 1e9 if ms > 0 else 0.0

    # plain device copy moving as many bytes as the dominant launch does (half read, half written), and a launch that
    # only reads as many bytes as round 1 does
    copy_bytes = 8 * (1 << n) * 2
    copy_ms = ctx.copy_ms(copy_bytes, 10)
    read_ms = ctx.read_ms(copy_bytes, 10)

    fe, ef = stats["fold_eval"], stats["eval_first"]
    # From 21 variables on the first two rounds are one launch that reads f and g once and writes nothing (arithmetic-bound:
    # nine base-field products a quad), and the dominant launch, by bytes, is the one of rounds 3 and 4: it reads f and g again
    # (base field), folds them twice on the way in, writes the folded tables and sums for both rounds.  Below that, round 2
    # folds and writes one round's worth.
    merged = n >= 21
    dom_ms = fe["max_ms"] / max(1, fe["max_launches"])
    dom_bytes = fe["max_bytes"]
    achieved = gbs(dom_bytes, dom_ms)
    kernel_ms = sum(s["ms"] for s in stats.values()) / args.steps
    stream_bytes = (fe["bytes"] + ef["bytes"]) / args.steps
    stream_ms = (fe["ms"] + ef["ms"]) / args.steps
    # the same launches priced as the plain algorithm streams them (eq read and folded like f and g)
    plain_round1 = float((8 + 8 + 16) * (1 << n))
    plain_round2 = float((8 + 8 + 16) * (1 << n) + 3 * 16 * (1 << (n - 1)))
    plain_round3 = float(3 * 16 * (1 << (n - 1)) + 3 * 16 * (1 << (n - 2)))
    plain_dom = plain_round3 if merged else plain_round2
    plain_first = plain_round1 + plain_round2 if merged else plain_round1
    plain_total = float(2 * (1 << n) * 32 + (1 << (n + 1)) * 16 * 3)
    first_ms = ef["ms"] / max(1, ef["launches"]) if "launches" in ef else ef["ms"] / args.steps
    roofline = {
        "bound": "hbm",
        "kernel": ("quad_kernel<true> (rounds 3 and 4 in one launch: f,g read unfolded, folded twice on the way in, written; the sums of round 3 and, as "
                   "polynomials in the challenge to come, of round 4; eq factor in closed form, its weights from two small tables)") if merged else
                  "prod_kernel<2,2,true,true,true,true> (round 2: fold f,g + evaluate; eq factor in closed form, its weights from two small tables)",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": profile_value(TRAFFIC_PROFILE, "dominant_launch_traffic_bytes") if n == 24 else None,
        "traffic_source": TRAFFIC_PROFILE if n == 24 else None,
        "algorithmic_bytes_per_launch": dom_bytes,
        "avg_launch_ms": round(dom_ms, 5),
        "plain_algorithm_bytes_per_launch": plain_dom,
        "plain_algorithm_equivalent_gbs": round(gbs(plain_dom, dom_ms), 1),
        "copy_kernel_gbs": round(gbs(2 * copy_bytes, copy_ms), 1),
        "frac_of_copy_kernel": round(achieved / gbs(2 * copy_bytes, copy_ms), 4),
        "first_launch": "pair12_kernel: rounds 1 and 2 from one pass over f and g, nothing written" if merged else "prod_kernel, round 1",
        "first_launch_ms": round(first_ms, 5),
        "first_launch_gbs": round(gbs(ef["bytes"], ef["ms"]), 1),
        "first_launch_plain_algorithm_bytes": plain_first,
        "first_launch_plain_algorithm_equivalent_gbs": round(gbs(plain_first, first_ms), 1),
        "read_kernel_gbs": round(gbs(copy_bytes, read_ms), 1),
        "first_launch_frac_of_read_kernel": round(gbs(ef["bytes"], ef["ms"]) / gbs(copy_bytes, read_ms), 4),
        "valu_issue_share_first_launch": profile_value(VALU_PROFILE, "valu_issue_share_first_launch") if n == 24 else None,
        "valu_issue_share_dominant_launch": profile_value(VALU_PROFILE, "valu_issue_share_dominant_launch") if n == 24 else None,
        "valu_source": VALU_PROFILE if n == 24 else None,
        "all_rounds_algorithmic_bytes": stream_bytes,
        "all_rounds_plain_algorithm_bytes": plain_total,
        "all_rounds_kernel_ms": round(stream_ms, 4),
        "all_rounds_gbs": round(gbs(stream_bytes, stream_ms), 1),
        "all_rounds_plain_algorithm_equivalent_gbs": round(gbs(plain_total, stream_ms), 1),
        "kernel_ms_per_proof": round(kernel_ms, 4),
    }

    element_visits = 3 * ((1 << (n + 1)) - 2)
    out = {
        "metric": "sumcheck prove ms @ n=24 deg-3 ext2" if n == 24 else f"sumcheck prove ms @ n={n} deg-3 ext2",
        "value": round(ms_per_step, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u64 (Goldilocks, ext2)",
        "data": "synthetic",
        "config": {"workload": f"cfg3: eq(r,x)*f(x)*g(x), n={n}, f,g base field, eq ext2, degree 3", "n_vars": n, "degree": 3,
                   "transcript": "BLAKE3 on the host, one round trip per round"},
        "field_elements_per_s": round(element_visits / (ms_per_step * 1e-3), 1),
        "min_step_ms": round(1e3 * min(per_step), 4),
        "eq_build_ms": round(eq_ms, 4),
        "prove_with_fresh_eq_ms": round(fresh_ms, 4),
        "prove_with_claim_ms": round(claimed_ms, 4),
        "same_proof_with_claim": same_with_claim,
        "all_steps_identical": bool(repeatable),
        "upload_s": round(upload_s, 4),
        "roofline": roofline,
    }

    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import dpsc_oracle as orc

        orc.select(True)
        tabs = [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(r)]
        reps, cpu_times = 0, []
        t_cpu0 = time.perf_counter()
        while reps < 3 and (time.perf_counter() - t_cpu0) < 20.0:
            otr = orc.OracleTranscript(b"bench")
            t0 = time.perf_counter()
            oproof, opoint, ofinals = orc.sc_prove(n, tabs, [(one, [2, 0, 1])], otr)
            cpu_times.append(time.perf_counter() - t0)
            reps += 1
        cpu_ms = 1e3 * sorted(cpu_times)[len(cpu_times) // 2]
        bit_exact = bool((oproof == proof).all() and (opoint == point).all() and (ofinals == finals).all() and otr.state() == tr.state())
        out["cpu_baseline"] = {
            "value": round(cpu_ms, 2),
            "unit": "ms",
            "cores": orc.num_threads(),
            "kind": "port",
            "sample": f"the same n={n} proof, whole, {reps} run(s), median; C restatement with OpenMP (not the reference's BN254 prover)",
        }
        out["speedup_vs_cpu"] = round(cpu_ms / ms_per_step, 1)
        out["bit_exact"] = bit_exact
        del tabs
    if n == 24 and not args.no_others:
        # The remaining configurations in the same record: a few steps each of the same measurement `--config X` makes
        # (a step = one complete proof, inputs resident in HBM), the CPU checker run once each to compare the bits.
        del prover, claimed, mf, mg, me
        others = {}
        for name, key in (("1", "cfg1"), ("2", "cfg2"), ("4", "cfg4"), ("5", "cfg5"), ("opening", "opening"), ("linking", "linking")):
            sub = argparse.Namespace(config=name, steps=5, warmup=2, no_cpu=args.no_cpu)
            res = other_config(sub)
            others[key] = {"ms": res["value"], "min_step_ms": res["min_step_ms"], "steps": sub.steps, "warmup": sub.warmup,
                           "bit_exact": res.get("bit_exact"), "workload": res["config"]["workload"]}
            if "cpu_baseline" in res:
                others[key]["cpu_port_ms"] = res["cpu_baseline"]["value"]
        out["other_configs"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
