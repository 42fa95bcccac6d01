#!/usr/bin/env python3
"""Benchmark of the sumcheck proving path on one MI355X.

A step is one whole sumcheck `prove` of the headline workload: statement (+ (* alpha t0 t1 t2) (* 3 t1)) in
eq mode over three base-field tables of 2^24 seeded uniform KoalaBear elements, F_p^4 challenges, degree-3
round messages, BLAKE3 transcript -- header absorb to last challenge, finals read back.  The tables are
resident in HBM before the timed region.  value = 3 * 2^24 table entries / time per step.

Prints one JSON line with the metric, the roofline of the dominant kernel (measured live with HIP events on
the library's stream) and the CPU oracle timed on a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FORM, TABLES, CONSTS = "(+ (* alpha t0 t1 t2) (* 3 t1))", ["t0", "t1", "t2"], ["alpha"]
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def splitmix_field(seed, count):
    """SplitMix64(seed) -> 31-bit words, rejected when >= p: the rule the library's seeded tables use."""
    P = 2130706433
    out, x, mask = [], seed, (1 << 64) - 1
    while len(out) < count:
        x = (x + 0x9E3779B97F4A7C15) & mask
        z = x
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        z ^= z >> 31
        w = z >> 33
        if w < P:
            out.append(w)
    return np.array(out, np.uint32)


def profile_entries(sa):
    lib = sa.load()
    out = []
    for i in range(lib.exh_profile_count()):
        name = C.create_string_buffer(64)
        rnd, ms, nbytes = C.c_int(), C.c_float(), C.c_uint64()
        sa.check(lib.exh_profile_entry(i, name, 64, C.byref(rnd), C.byref(ms), C.byref(nbytes)))
        out.append((name.value.decode(), rnd.value, ms.value, nbytes.value))
    return out


def cpu_baseline(sa, n_sample, d, seed):
    """The CPU oracle (a C restatement of the reference's prover, single thread) on the same statement and
    seeds at a smaller n, sized for roughly 10-30 s.  The same sample then goes through the GPU path as the
    checker of this run: the proof bytes must be the oracle's."""
    from oracle import binding as orc
    st = orc.Statement(FORM, TABLES, CONSTS)
    tables = [splitmix_field(seed * 1000 + k, 1 << n_sample) for k in range(3)]
    eq = splitmix_field(seed + 900, n_sample * d).reshape(n_sample, d)
    alpha = splitmix_field(seed + 901, d).reshape(1, d)
    t0 = time.perf_counter()
    otr = orc.Transcript("config2", d)
    orc.prove(otr, n_sample, st, tables, eq=eq, constants=alpha)
    dt = time.perf_counter() - t0
    dev = [sa.Table.upload(t) for t in tables]
    tr = sa.Transcript("config2", d)
    sa.prove(tr, n_sample, sa.Statement(FORM, TABLES, CONSTS), dev, eq=eq, constants=alpha)
    for t in dev:
        t.free()
    if tr.proof() != otr.proof():
        sys.exit(f"bench.py: the GPU proof at n={n_sample} differs from the CPU oracle's")
    return {"value": 3 * (1 << n_sample) / dt, "unit": "table entries/s", "cores": 1, "kind": "port",
            "sample": f"same statement, seeds and transcript at n={n_sample} (3*2^{n_sample} entries, "
                      f"{dt:.1f} s); the GPU proof of the same sample is byte-identical; the reference's Lisp "
                      f"prover cannot run here (no SBCL)"}


def run_sumcheck_config(sa, name, form, tables, consts, n, d, seed, steps, warmup, cpu_n):
    """A sumcheck workload other than the headline one: same timing rules, one JSON line."""
    st = sa.Statement(form, tables, consts)
    T = len(tables)
    dev = [sa.Table.random(seed * 1000 + k, 1 << n) for k in range(T)]
    eq = splitmix_field(seed + 900, n * d).reshape(n, d)
    cv = splitmix_field(seed + 901, d * max(len(consts), 1)).reshape(-1, d) if consts else None

    def step():
        tr = sa.Transcript(name, d)
        sa.prove(tr, n, st, dev, eq=eq, constants=cv)
        return tr

    for _ in range(warmup):
        step()
    sa.check(sa.load().exh_synchronize())
    t0 = time.perf_counter()
    for _ in range(steps):
        tr = step()
    sa.check(sa.load().exh_synchronize())
    dt = (time.perf_counter() - t0) / steps
    sa.check(sa.load().exh_profile_enable(1))
    for _ in range(steps):
        step()
    by_kernel = {}
    for kname, rnd, ms, nbytes in profile_entries(sa):
        k = by_kernel.setdefault((kname, rnd), [0.0, 0, nbytes])
        k[0] += ms
        k[1] += 1
    sa.check(sa.load().exh_profile_enable(0))
    (kname, kround), (ktotal, kcalls, kbytes) = max(by_kernel.items(), key=lambda kv: kv[1][0])
    avg_ms = ktotal / kcalls
    achieved = kbytes / (avg_ms * 1e-3) / 1e9
    points = max(st.degree, 1)
    out = {"metric": f"sumcheck table entries/s ({name})", "value": T * (1 << n) / dt, "unit": "table entries/s",
           "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": 1e3 * dt, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": f"u32 (Montgomery KoalaBear, F_p^{d} tower)",
           "data": "synthetic (SplitMix64-seeded uniform field elements)",
           "config": {"workload": f"sumcheck prove of {form}, eq mode, n={n}, {T} base tables, F_p^{d}",
                      "generated_kernel": st.has_generated_kernel(d), "proof_bytes": len(tr.proof()),
                      "proof_sha256": hashlib.sha256(tr.proof()).hexdigest()},
           "loop_hbm_fraction": T * (1 << n) * (8 + 8 * d) / dt / (HBM_PEAK_GBS * 1e9),
           "roofline": {"bound": "hbm", "kernel": f"{kname} (round {kround})", "achieved": achieved,
                        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                        "avg_launch_ms": avg_ms, "alg_bytes_per_launch": kbytes, "traffic": None}}
    assert len(tr.proof()) == 12 + n * (18 + 4 * points * d)
    if cpu_n > 0:
        from oracle import binding as orc
        ost = orc.Statement(form, tables, consts)
        ht = [splitmix_field(seed * 1000 + k, 1 << cpu_n) for k in range(T)]
        heq = splitmix_field(seed + 900, cpu_n * d).reshape(cpu_n, d)
        t0 = time.perf_counter()
        orc.prove(orc.Transcript(name, d), cpu_n, ost, ht, eq=heq, constants=cv)
        cdt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": T * (1 << cpu_n) / cdt, "unit": "table entries/s", "cores": 1, "kind": "port",
                               "sample": f"same statement at n={cpu_n} ({cdt:.1f} s)"}
    for t in dev:
        t.free()
    return out


def run_gkr(sa, steps, warmup, cpu_n):
    """Config 4: LogUp-GKR of 2^22 int8-range lookups into a 2^16-entry range table.  The witness tree has
    leaves (1, Z - v_i), n = 22; the table tree leaves (m_j, Z - t_j), n = 16, t_j = j - 32768, m_j the exact
    multiplicities; both roots are equal as fractions.  A step = prove-upper of both trees (fraction trees +
    every layer's sumcheck)."""
    d, nw, nt, seed = 4, 22, 16, 4
    rng = np.random.default_rng(seed)
    values = rng.integers(-128, 128, 1 << nw)
    table = np.arange(1 << nt) - 32768
    mult = np.bincount(values + 32768, minlength=1 << nt)
    z = sa.Transcript("config4-z", d).challenge()

    def leaves(num, val):
        P = sa.P
        p = np.zeros((len(num), d), np.uint32)
        p[:, 0] = np.asarray(num, np.int64) % P
        q = np.tile(z.astype(np.int64), (len(val), 1))
        q[:, 0] = (q[:, 0] - np.asarray(val, np.int64)) % P
        return p, q.astype(np.uint32)

    wit = [sa.Table.upload(a) for a in leaves(np.ones(1 << nw, np.int64), values)]
    tab = [sa.Table.upload(a) for a in leaves(mult, table)]

    def step():
        tw, tt = sa.Transcript("config4-w", d), sa.Transcript("config4-t", d)
        sa.prove_upper(tw, nw, 1, [tuple(wit)])
        sa.prove_upper(tt, nt, 1, [tuple(tab)])
        return tw, tt

    for _ in range(warmup):
        step()
    sa.check(sa.load().exh_synchronize())
    t0 = time.perf_counter()
    for _ in range(steps):
        tw, tt = step()
    sa.check(sa.load().exh_synchronize())
    dt = (time.perf_counter() - t0) / steps
    from oracle import binding as orc
    rw, rt = orc.decode_proof(tw.proof())[0], orc.decode_proof(tt.proof())[0]
    same_fraction = np.array_equal(orc.ext_mul(rw[0], rt[1]), orc.ext_mul(rt[0], rw[1]))
    # algorithmic bytes of prove-upper per tree (16 B entries): tree build 3 * 2 * 2^n * 16 - ..., layer sumchecks
    def alg(n):
        build = sum(2 * (2 << m) * 16 + 2 * (1 << m) * 16 for m in range(n))
        layers = sum(4 * (4 * (1 << l) * 16) for l in range(n - 1))
        return build + layers
    nbytes = alg(nw) + alg(nt)
    out = {"metric": "LogUp-GKR prove-upper lookups/s (config 4)", "value": (1 << nw) / dt, "unit": "lookups/s",
           "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": 1e3 * dt, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "u32 (Montgomery KoalaBear, F_p^4 tower)",
           "data": "synthetic (seeded uniform int8 lookups, exact multiplicities)",
           "config": {"workload": "LogUp-GKR: 2^22 int8-range lookups into a 2^16-entry table, witness tree n=22 + "
                                  "table tree n=16, F_p^4, prove-upper of both", "roots_equal_as_fractions": bool(same_fraction),
                      "proof_bytes": len(tw.proof()) + len(tt.proof())},
           "roofline": {"bound": "hbm", "kernel": "prove-upper (whole: tree build + 36 layer sumchecks)",
                        "achieved": nbytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS, "alg_bytes": nbytes, "traffic": None}}
    if cpu_n > 0:
        rng = np.random.default_rng(1)
        p = rng.integers(0, sa.P, (1 << cpu_n, d), dtype=np.uint32)
        q = rng.integers(1, sa.P, (1 << cpu_n, d), dtype=np.uint32)
        t0 = time.perf_counter()
        orc.gkr_prove_upper(orc.Transcript("config4-w", d), cpu_n, 1, [(p, q)])
        cdt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": (1 << cpu_n) / cdt, "unit": "lookups/s", "cores": 1, "kind": "port",
                               "sample": f"prove-upper of one tree of 2^{cpu_n} leaves ({cdt:.1f} s)"}
    return out


def run_commit(sa, steps, warmup, cpu_c):
    """Config 5 as the reference runs it: 2^24 coefficients = two columns of 2^23 (the code's domain is capped
    at 2^24 points), rate-1/2 encode to two codewords of 2^24, 2^22 BLAKE3 leaves, Merkle levels, cap of 128."""
    c, ncols = 23, 2
    cols = sa.Table.random(5005, ncols << c)

    def step():
        tr = sa.Transcript("config5", 4)
        cw, levels = sa.pcs_commit(tr, cols, ncols, c)
        cw.free(), levels.free()
        return tr

    for _ in range(warmup):
        step()
    sa.check(sa.load().exh_synchronize())
    t0 = time.perf_counter()
    for _ in range(steps):
        tr = step()
    sa.check(sa.load().exh_synchronize())
    dt = (time.perf_counter() - t0) / steps
    nleaves = 1 << (c - 1)
    nbytes = ncols * (4 << c) + ncols * (4 << (c + 1)) + ncols * (4 << (c + 1)) + 32 * nleaves + 64 * (nleaves - 1) + 32 * (nleaves - 1)
    out = {"metric": "BaseFold commit ms (config 5)", "value": 1e3 * dt, "unit": "ms", "n_gpus": 1, "steps": steps,
           "warmup": warmup, "ms_per_step": 1e3 * dt, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "u32 (Montgomery KoalaBear) + BLAKE3", "data": "synthetic (SplitMix64-seeded uniform field elements)",
           "config": {"workload": "pcs-commit: 2 columns of 2^23 coefficients -> 2 codewords of 2^24, 2^22 leaves, "
                                  "Merkle levels, cap of 128 digests", "cap_sha256": hashlib.sha256(tr.proof()).hexdigest(),
                      "leaf_hashes_per_s": nleaves / dt, "butterflies_per_s": ncols * 23 * (1 << 23) / dt},
           "roofline": {"bound": "hbm", "kernel": "encode + leaves + Merkle (whole commit)", "achieved": nbytes / dt / 1e9,
                        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS,
                        "alg_bytes": nbytes, "traffic": None}}
    if cpu_c > 0:
        from oracle import binding as orc
        hc = [splitmix_field(77 + k, 1 << cpu_c) for k in range(ncols)]
        t0 = time.perf_counter()
        orc.commit_columns(hc, cpu_c)
        cdt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": 1e3 * cdt * (1 << (c - cpu_c)), "unit": "ms", "cores": 1, "kind": "port",
                               "sample": f"commit of 2 columns of 2^{cpu_c} ({cdt:.1f} s), scaled linearly by 2^{c - cpu_c} "
                                         "(ignores the log factor of the encoder, so it flatters the CPU)"}
    return out


def run_combine(sa, steps, warmup, cpu_c):
    """combine-columns at config 5's shape: the two committed columns of 2^23 base values into the table of
    2^23 EXT8s that BaseFold opens (src/pcs.lisp:434-441)."""
    c, ncols, d = 23, 2, 8
    cols = sa.Table.random(5005, ncols << c)
    cf = splitmix_field(5006, ncols * d).reshape(ncols, d)
    lib = sa.load()

    def step():
        sa.combine_columns(cols, ncols, cf).free()

    for _ in range(warmup):
        step()
    sa.check(lib.exh_synchronize())
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    sa.check(lib.exh_synchronize())
    dt = (time.perf_counter() - t0) / steps
    sa.check(lib.exh_profile_enable(1))
    for _ in range(steps):
        step()
    entries = [e for e in profile_entries(sa) if e[0] == "combine_columns"]
    sa.check(lib.exh_profile_enable(0))
    avg_ms = sum(e[2] for e in entries) / len(entries)
    nbytes = (1 << c) * (4 * ncols + 4 * d)
    out = {"metric": "combine-columns entries/s (config 5's columns)", "value": ncols * (1 << c) / dt,
           "unit": "column entries/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": 1e3 * dt,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u32 (Montgomery KoalaBear, F_p^8)",
           "data": "synthetic (SplitMix64-seeded uniform field elements)",
           "config": {"workload": "combine-columns: 2 base columns of 2^23 with F_p^8 coefficients -> 2^23 EXT8s"},
           "roofline": {"bound": "hbm", "kernel": "combine_columns", "achieved": nbytes / (avg_ms * 1e-3) / 1e9,
                        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / (avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        "avg_launch_ms": avg_ms, "alg_bytes_per_launch": nbytes, "traffic": None}}
    if cpu_c > 0:
        from oracle import binding as orc
        hc = np.stack([splitmix_field(77 + k, 1 << cpu_c) for k in range(ncols)])
        t0 = time.perf_counter()
        orc.combine_columns(hc, cf)
        cdt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": ncols * (1 << cpu_c) / cdt, "unit": "column entries/s", "cores": 1, "kind": "port",
                               "sample": f"2 columns of 2^{cpu_c} ({cdt:.2f} s)"}
    cols.free()
    return out


# HBM bytes per launch of the dominant kernel at the headline workload, from two rocprofv3 --pmc runs of this
# file (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for the plain
# copy kernel of `--workload copy`, whose traffic is known (the summary of those runs is kept with the profiles)
MEASURED_TRAFFIC = {
    ("round_nodes_base", 24): 203495288,  # per launch of the sweep for rounds 0 and 1: the base tables read once
    ("round_fold2_base", 24): 403802364,  # round 2: 2.024e8 read (base tables) + 2.014e8 written (generation 2)
}


def run_copy(steps):
    """Calibration for the traffic counters: an elementwise kernel that reads 256 MiB and writes 256 MiB."""
    import torch
    a = torch.ones(1 << 26, dtype=torch.int32, device="cuda")
    b = torch.empty_like(a)
    for _ in range(steps):
        torch.add(a, 1, out=b)
    torch.cuda.synchronize()
    print(json.dumps({"workload": "copy", "read_bytes": a.numel() * 4, "written_bytes": b.numel() * 4, "steps": steps}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="config2", choices=["config1", "config2", "config3", "config4", "config5", "combine", "copy"],
                    help="config2 (default) is the headline; the others are the remaining configured workloads; "
                         "copy is the known-size kernel the traffic counters are calibrated on")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=24, help="variables (24 is the headline workload)")
    ap.add_argument("--cpu-n", type=int, default=22, help="variables of the CPU baseline's sample (0: skip)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus above 1 is not supported (nothing here uses a "
                 "second device)")

    if args.workload == "copy":
        run_copy(args.steps)
        return
    import sable_amd as sa
    sa.init(0)
    if args.workload == "config1":
        print(json.dumps(run_sumcheck_config(sa, "config1", "(* t0 t1)", ["t0", "t1"], [], 16, 4, 1, args.steps,
                                             args.warmup, 16 if args.cpu_n else 0)))
        return
    if args.workload == "config3":
        print(json.dumps(run_sumcheck_config(sa, "config3", "(* (+ c0 3) (- c1 c0) c2 c3)", ["c0", "c1", "c2", "c3"], [],
                                             26 if args.n == 24 else args.n, 8, 3, args.steps, args.warmup,
                                             18 if args.cpu_n else 0)))
        return
    if args.workload == "config4":
        print(json.dumps(run_gkr(sa, args.steps, args.warmup, 18 if args.cpu_n else 0)))
        return
    if args.workload == "config5":
        print(json.dumps(run_commit(sa, args.steps, args.warmup, 18 if args.cpu_n else 0)))
        return
    if args.workload == "combine":
        print(json.dumps(run_combine(sa, args.steps, args.warmup, 20 if args.cpu_n else 0)))
        return
    n, d, seed = args.n, 4, 2
    st = sa.Statement(FORM, TABLES, CONSTS)
    tables = [sa.Table.random(seed * 1000 + k, 1 << n) for k in range(3)]
    eq = splitmix_field(seed + 900, n * d).reshape(n, d)
    alpha = splitmix_field(seed + 901, d).reshape(1, d)

    def step():
        tr = sa.Transcript("config2", d)
        sa.prove(tr, n, st, tables, eq=eq, constants=alpha)
        return tr

    for _ in range(args.warmup):
        step()
    # the library runs on its own HIP stream (not torch's): exh_synchronize is the device-wide barrier
    sa.check(sa.load().exh_synchronize())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        tr = step()  # every prove ends with its finals on the host: the stream is drained
    sa.check(sa.load().exh_synchronize())
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    entries = 3 * (1 << n)
    proof = tr.proof()

    # the dominant kernel, timed live with HIP events on the library's stream over `steps` more proves
    sa.check(sa.load().exh_profile_enable(1))
    for _ in range(args.steps):
        step()
    by_kernel = {}
    for name, rnd, ms, nbytes in profile_entries(sa):
        k = by_kernel.setdefault((name, rnd), [0.0, 0, nbytes])
        k[0] += ms
        k[1] += 1
    sa.check(sa.load().exh_profile_enable(0))
    # The roofline figure is for the streaming launch (the ones that read the tables from HBM: round_*) with the
    # largest total time per prove; the launch with the largest time of all may be one of the LDS-resident ones
    # (slices, tail), which are latency-bound by construction and move a few MB: it is named beside it.
    streaming = {k: v for k, v in by_kernel.items() if k[0].startswith("round_")}
    (kname, kround), (ktotal, kcalls, kbytes) = max(streaming.items(), key=lambda kv: kv[1][0])
    (tname, tround), (ttotal, tcalls, _) = max(by_kernel.items(), key=lambda kv: kv[1][0])
    avg_ms = ktotal / kcalls
    achieved = kbytes / (avg_ms * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC.get((kname, n))
    loop_alg_bytes = 3 * (1 << n) * (8 + 8 * d)

    result = {
        "metric": "sumcheck table entries/s at n=24 deg-3", "value": entries / (elapsed / args.steps),
        "unit": "table entries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32 (Montgomery KoalaBear, F_p^4 tower; exact integers in f64 for the first sweep's products)",
        "data": "synthetic (SplitMix64-seeded uniform field elements)",
        "config": {"workload": f"sumcheck prove of {FORM}, eq mode, n={n}, three base tables of 2^{n}, F_p^4, "
                               "BLAKE3 transcript", "tables": 3, "n": n, "degree": 3, "extension": 4,
                   "proof_sha256": hashlib.sha256(proof).hexdigest(), "proof_bytes": len(proof)},
        "loop_hbm_fraction": loop_alg_bytes / (elapsed / args.steps) / (HBM_PEAK_GBS * 1e9),
        "roofline": {"bound": "hbm", "kernel": f"{kname} (round {kround})", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "avg_launch_ms": avg_ms, "launches_per_step": kcalls // args.steps,
                     "alg_bytes_per_launch": kbytes, "traffic": traffic,
                     "longest_launch": {"kernel": f"{tname} (round {tround})", "avg_launch_ms": ttotal / tcalls,
                                        "note": "LDS-resident rounds are latency-bound" if not tname.startswith("round_") else ""}},
    }
    result["cpu_baseline"] = cpu_baseline(sa, args.cpu_n, d, seed) if args.cpu_n > 0 else None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
