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


def cpu_baseline(n_sample, d, seed):
    """The CPU oracle (a C restatement of the reference's prover, single thread) on the same statement and
    seeds at a smaller n, sized for roughly 10-30 s."""
    from oracle import binding as orc
    st = orc.Statement(FORM, TABLES, CONSTS)
    tables = [splitmix_field(seed * 1000 + k, 1 << n_sample) for k in range(3)]
    eq = splitmix_field(seed + 900, n_sample * d).reshape(n_sample, d)
    alpha = splitmix_field(seed + 901, d).reshape(1, d)
    t0 = time.perf_counter()
    orc.prove(orc.Transcript("config2", d), n_sample, st, tables, eq=eq, constants=alpha)
    dt = time.perf_counter() - t0
    return {"value": 3 * (1 << n_sample) / dt, "unit": "table entries/s", "cores": 1, "kind": "port",
            "sample": f"same statement, seeds and transcript at n={n_sample} (3*2^{n_sample} entries, "
                      f"{dt:.1f} s); the reference's Lisp prover cannot run here (no SBCL)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=24, help="variables (24 is the headline workload)")
    ap.add_argument("--cpu-n", type=int, default=22, help="variables of the CPU baseline's sample (0: skip)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus above 1 is not supported (nothing here uses a "
                 "second device)")

    import sable_amd as sa
    sa.init(0)
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
    (kname, kround), (ktotal, kcalls, kbytes) = max(by_kernel.items(), key=lambda kv: kv[1][0])
    avg_ms = ktotal / kcalls
    achieved = kbytes / (avg_ms * 1e-3) / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get(f"{kname}@n{n}")
    loop_alg_bytes = 3 * (1 << n) * (8 + 8 * d)

    result = {
        "metric": "sumcheck table entries/s at n=24 deg-3", "value": entries / (elapsed / args.steps),
        "unit": "table entries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32 (Montgomery KoalaBear, F_p^4 tower)", "data": "synthetic (SplitMix64-seeded uniform field elements)",
        "config": {"workload": f"sumcheck prove of {FORM}, eq mode, n={n}, three base tables of 2^{n}, F_p^4, "
                               "BLAKE3 transcript", "tables": 3, "n": n, "degree": 3, "extension": 4,
                   "proof_sha256": hashlib.sha256(proof).hexdigest(), "proof_bytes": len(proof)},
        "loop_hbm_fraction": loop_alg_bytes / (elapsed / args.steps) / (HBM_PEAK_GBS * 1e9),
        "roofline": {"bound": "hbm", "kernel": f"{kname} (round {kround})", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "avg_launch_ms": avg_ms, "alg_bytes_per_launch": kbytes, "traffic": traffic},
    }
    result["cpu_baseline"] = cpu_baseline(args.cpu_n, d, seed) if args.cpu_n > 0 else None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
