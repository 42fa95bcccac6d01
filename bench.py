#!/usr/bin/env python3
"""Benchmark of the proving path on one MI355X.

A step is one whole sumcheck `prove` of the headline workload (config 2): statement
(+ (* alpha t0 t1 t2) (* 3 t1)) in eq mode over three base-field tables of 2^24 seeded uniform KoalaBear elements,
F_p^4 challenges, degree-3 round messages, BLAKE3 transcript -- header absorb to last challenge, finals read back.
The tables are resident in HBM before the timed region.  value = 3 * 2^24 table entries / time per step.

One JSON line: the metric; `roofline` for the streaming launch with the largest time (HIP events on the library's
stream) and `roofline_by_time` for every launch of a prove; `int32_mul`, the integer-multiply roofline;
`cpu_baseline`, the CPU oracle's threaded path on a bounded sample of the same workload (one thread and all host
threads, best of 7); `other_configs`, the other four configured workloads timed the same way in the same run.
The timed proof is checked before it is reported: the library's verifier accepts it and its SHA-256 is the one the
CPU oracle's proof of the same seeded inputs has (tests/golden/config_hashes.json).
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

from sable_amd import workloads as wl  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# The integer-multiply roofline's peak is measured by `--workload mulrate` (run_mulrate below; the issue-rate
# kernel of sable_amd/csrc/issue_rate.hip): lanes x SIMDs x compute units x clock / cycles per wavefront instruction
# of v_mad_u64_u32 with many wavefronts resident.  profiles/mulrate_kernel_stats.md holds the run this default is from.
MULRATE_DEFAULT = {"cycles_per_wave_instruction": 4.9, "clock_ghz": 2.4, "compute_units": 256}


def int32_mul_peak(rate=None):
    r = rate or MULRATE_DEFAULT
    return r["compute_units"] * 4 * 64 / r["cycles_per_wave_instruction"] * r["clock_ghz"] * 1e9


# Figures that were measured on one version of the kernels and are only reported while the kernels' sources are
# that version: HBM bytes per launch from two rocprofv3 --pmc runs (FETCH_SIZE, then WRITE_SIZE, each scaled by what
# the same counter reads for the plain copy kernel of `--workload copy`), and 32-bit integer multiply instructions
# per lane and prove from the kernels' instruction streams times their trip counts (profiles/ holds both summaries).
MEASURED = {
    "kernel_sources_sha256": "84841755ff915996f2c965a0c6de1e5fbe22a98773f07c1cce7a8c3f1a8ddc0f",
    "traffic": {("round_nodes_base", 24): 204058883, ("round_fold2_base", 24): 404005645},
    # per pair: 76 multiply-adds in the sweep (2^22 pairs of four entries), 272 multiply-adds and 96 multiplies of
    # the reductions in the extension rounds (2^21 + 2^20 + ... pairs)
    "int32_mul_per_prove": 76 * (1 << 22) + 368 * ((1 << 21) + (1 << 20) + (1 << 19) + (1 << 19)),
}
KERNEL_SOURCES = ["sumcheck_kernels.hpp", "field.hpp", "dev_transcript.hpp", "blake3.hpp", "stmtdesc.hpp"]


def kernel_sources_sha256():
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "sable_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def sha(b):
    return hashlib.sha256(bytes(b)).hexdigest()


def golden():
    with open(os.path.join(ROOT, "tests", "golden", "config_hashes.json")) as f:
        return json.load(f)


def splitmix_field(seed, count):
    """SplitMix64(seed) -> 31-bit words, kept when below p: the rule the library's seeded tables use."""
    P = wl.P
    out = np.empty(0, np.uint32)
    mask = (1 << 64) - 1
    x0 = seed
    while len(out) < count:
        m = max(64, int((count - len(out)) * 1.02) + 16)
        idx = np.arange(1, m + 1, dtype=np.uint64)
        with np.errstate(over="ignore"):
            x = (np.uint64(x0) + idx * np.uint64(0x9E3779B97F4A7C15)) & np.uint64(mask)
            z = x
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            z = z ^ (z >> np.uint64(31))
        w = (z >> np.uint64(33)).astype(np.uint32)
        out = np.concatenate([out, w[w < P]])
        x0 = int(x[-1])
    return out[:count].copy()


def profile_entries(sa):
    lib = sa.load()
    out = []
    for i in range(lib.exh_profile_count()):
        name = C.create_string_buffer(64)
        rnd, ms, nbytes = C.c_int(), C.c_float(), C.c_uint64()
        sa.check(lib.exh_profile_entry(i, name, 64, C.byref(rnd), C.byref(ms), C.byref(nbytes)))
        out.append((name.value.decode(), rnd.value, ms.value, nbytes.value))
    return out


def timed(sa, step, steps, warmup):
    """W untimed steps, then exactly K steps between two device-wide waits: seconds per step, last result."""
    out = None
    for _ in range(warmup):
        out = step()
    sa.check(sa.load().exh_synchronize())
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    sa.check(sa.load().exh_synchronize())
    return (time.perf_counter() - t0) / steps, out


def launches(sa, step, steps):
    """Every launch of `steps` more steps, timed with HIP events on the library's stream: per (kernel, round)
    [average ms, launches per step, algorithmic bytes per launch], and the same summed per kernel name."""
    sa.check(sa.load().exh_profile_enable(1))
    for _ in range(steps):
        step()
    by = {}
    for name, rnd, ms, nbytes in profile_entries(sa):
        k = by.setdefault((name, rnd), [0.0, 0, nbytes])
        k[0] += ms
        k[1] += 1
    sa.check(sa.load().exh_profile_enable(0))
    return {k: (v[0] / v[1], v[1] / steps, v[2]) for k, v in by.items()}


def by_time(by):
    total = sum(avg * per for avg, per, _ in by.values())
    rows = []
    for (name, rnd), (avg, per, nbytes) in sorted(by.items(), key=lambda kv: -kv[1][0] * kv[1][1]):
        row = {"kernel": name, "round": rnd, "avg_launch_ms": avg, "launches_per_step": per,
               "share_of_kernel_time": avg * per / total if total else 0.0, "alg_bytes_per_launch": nbytes}
        if nbytes:
            row["hbm_frac"] = nbytes / (avg * 1e-3) / 1e9 / HBM_PEAK_GBS
        rows.append(row)
    return rows


# ------------------------------------------------------------------ sumcheck configurations
def sumcheck_setup(sa, name, n=None):
    cfg = wl.SUMCHECK[name]
    n, d, T = n or cfg["n"], cfg["d"], len(cfg["tables"])
    st = sa.Statement(cfg["form"], cfg["tables"], cfg["constants"])
    dev = [sa.Table.random(wl.table_seed(cfg, k), 1 << n) for k in range(T)]
    eq = splitmix_field(wl.eq_seed(cfg), n * d).reshape(n, d)
    cv = splitmix_field(wl.constants_seed(cfg), d * len(cfg["constants"])).reshape(-1, d) if cfg["constants"] else None

    call = sa.ProveCall(n, st, dev, d, eq=eq, constants=cv)  # the arguments marshalled once, as a host would hold them

    def step():
        tr = sa.Transcript(name, d)
        chal, finals, _ = call(tr)
        return tr, finals

    return cfg, n, d, T, st, dev, eq, cv, step


def sumcheck_checked(sa, name, n, d, st, dev, eq, cv, tr, finals, gold):
    """The timed proof before it is reported: the verifier accepts it; at the configured size its digest is the
    CPU oracle's."""
    proof = tr.proof()
    claim = sa.hypercube_sum(st, n, dev, d, eq=eq, constants=cv)
    vtr = sa.Transcript(name, d, proof=proof)
    _, reduced = sa.verify(vtr, n, st, claim, eq=eq, constants=cv)
    if not (vtr.finished() and sa.check_final(reduced, st, finals, constants=cv)):
        sys.exit(f"bench.py: the verifier rejects the timed {name} proof")
    want = gold.get(name, {}).get("proof_sha256") if n == wl.SUMCHECK[name]["n"] else None
    if want is not None and sha(proof) != want:
        sys.exit(f"bench.py: the timed {name} proof differs from the CPU oracle's")
    return proof, want is not None


def run_sumcheck(sa, name, steps, warmup, gold, n=None):
    cfg, n, d, T, st, dev, eq, cv, step = sumcheck_setup(sa, name, n)
    dt, (tr, finals) = timed(sa, step, steps, warmup)
    proof, pinned = sumcheck_checked(sa, name, n, d, st, dev, eq, cv, tr, finals, gold)
    by = launches(sa, step, max(2, min(steps, 10)))
    for t in dev:
        t.free()
    streaming = {k: v for k, v in by.items() if k[0].startswith("round_")} or by
    (kname, kround), (avg_ms, per, kbytes) = max(streaming.items(), key=lambda kv: kv[1][0] * kv[1][1])
    achieved = kbytes / (avg_ms * 1e-3) / 1e9
    note = None
    if kname == "round_nodes_base":
        note = ("the launch stands for rounds 0 and 1: its algorithmic bytes are the two reads of the base tables "
                "those rounds' units take (round 0's sums, the read side of fold 1: T * 2^n * 8), shared among its "
                "passes; a pass moves one read of them, which is what `traffic` measures")
    return {"workload": f"sumcheck prove of {cfg['form']}, eq mode, n={n}, {T} base tables of 2^{n}, F_p^{d}, BLAKE3 "
                        "transcript", "n": n, "tables": T, "extension": d, "degree": st.degree,
            "ms_per_step": 1e3 * dt, "entries_per_s": T * (1 << n) / dt, "proof_bytes": len(proof),
            "proof_sha256": sha(proof), "proof_is_the_cpu_oracles": pinned, "verifier_accepts": True,
            "generated_kernel": st.has_generated_kernel(d),
            "loop_hbm_fraction": T * (1 << n) * (8 + 8 * d) / dt / (HBM_PEAK_GBS * 1e9),
            "roofline": {"bound": "hbm", "kernel": f"{kname} (round {kround})", "achieved": achieved,
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "avg_launch_ms": avg_ms,
                         "launches_per_step": per, "alg_bytes_per_launch": kbytes, "traffic": None, "note": note},
            "roofline_by_time": by_time(by)}


def run_domain(sa, steps, warmup, n=None):
    """A statement wider than the table groups' kernels (workloads.SUMCHECK["domain"]): proved in one device-driven
    session by the kernels of its direct form, which are compiled before the clock starts; the proof is verified and
    compared with the one the same library gives when it deals the statement into parts (the way the parity tests
    hold to the oracle's bytes), which is timed beside it."""
    cfg, n, d, T, st, dev, eq, cv, step = sumcheck_setup(sa, "domain", n)
    if not st.generate(d, wait=True):
        sys.exit("bench.py: the kernels of the domain statement's direct form did not compile")
    dt, (tr, finals) = timed(sa, step, steps, warmup)
    proof, _ = sumcheck_checked(sa, "domain", n, d, st, dev, eq, cv, tr, finals, {})
    by = launches(sa, step, max(2, min(steps, 5)))
    os.environ["EXACTA_HIP_NO_DIRECT"] = "1"
    try:
        dt_parts, (tr_parts, _) = timed(sa, step, max(2, steps // 4), 1)
    finally:
        del os.environ["EXACTA_HIP_NO_DIRECT"]
    if tr_parts.proof() != proof:
        sys.exit("bench.py: the direct form's proof differs from the proof in parts")
    for t in dev:
        t.free()
    nbytes = T * (1 << n) * (8 + 8 * d)
    return {"workload": f"sumcheck prove of the toy domain's leaf-layer and zerocheck statement (41 table monomials, "
                        f"degree {st.degree}), eq mode, n={n}, {T} base tables of 2^{n}, F_p^{d}, BLAKE3 transcript",
            "n": n, "tables": T, "extension": d, "degree": st.degree, "ms_per_step": 1e3 * dt,
            "ms_per_step_in_parts": 1e3 * dt_parts, "entries_per_s": T * (1 << n) / dt, "proof_bytes": len(proof),
            "proof_sha256": sha(proof), "proof_is_the_parts_paths": True, "verifier_accepts": True,
            "timed_launches_per_step": sum(per for _, per, _ in by.values()),
            "loop_hbm_fraction": nbytes / dt / (HBM_PEAK_GBS * 1e9),
            "roofline": {"bound": "hbm", "kernel": "whole round loop", "achieved": nbytes / dt / 1e9,
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS,
                         "alg_bytes": nbytes, "traffic": None},
            "roofline_by_time": by_time(by)[:8]}


# ------------------------------------------------------------------ config 4: LogUp-GKR
def run_gkr(sa, steps, warmup, gold):
    g = wl.GKR
    d, nw, nt = g["d"], g["n_witness"], g["n_table"]
    z = sa.Transcript(g["z_label"], d).challenge()
    seeded = sa.Table.random(g["seed"], 1 << nw)
    words = seeded.download()
    seeded.free()
    wit_h, tab_h = wl.gkr_leaves(np, words, z, nw, nt, d)
    wit = [sa.Table.upload(a) for a in wit_h]
    tab = [sa.Table.upload(a) for a in tab_h]

    def one_after_the_other():
        tw, tt = sa.Transcript(g["witness_label"], d), sa.Transcript(g["table_label"], d)
        sa.prove_upper(tw, nw, 1, [tuple(wit)])
        sa.prove_upper(tt, nt, 1, [tuple(tab)])
        return tw, tt

    def step():  # the two trees have a transcript each: proved side by side (exh_gkr_prove_upper_pair)
        tw, tt = sa.Transcript(g["witness_label"], d), sa.Transcript(g["table_label"], d)
        sa.prove_upper_pair((tw, nw, 1, [tuple(wit)]), (tt, nt, 1, [tuple(tab)]))
        return tw, tt

    dt_serial, _ = timed(sa, one_after_the_other, max(3, steps // 2), warmup)
    dt, (tw, tt) = timed(sa, step, steps, warmup)
    pinned = True
    for key, tr, n in (("witness", tw, nw), ("table", tt, nt)):
        vtr = sa.Transcript(g[key + "_label"], d, proof=tr.proof())
        sa.verify_upper(vtr, n, 1, 1)
        if not vtr.finished():
            sys.exit("bench.py: the verifier rejects the timed GKR proof")
        want = gold.get("config4", {}).get(key, {}).get("proof_sha256")
        if want is None:
            pinned = False
        elif sha(tr.proof()) != want:
            sys.exit(f"bench.py: the timed GKR proof ({key} tree) differs from the CPU oracle's")
    by = launches(sa, step, max(2, min(steps, 5)))
    for t in wit + tab:
        t.free()

    def alg(n):  # fraction trees (2 x 16-byte entries read per parent pair, one written) + the layers' sumchecks
        build = sum(2 * (2 << m) * 16 + 2 * (1 << m) * 16 for m in range(n))
        layers = sum(4 * (4 * (1 << l) * 16) for l in range(n - 1))
        return build + layers

    nbytes = alg(nw) + alg(nt)
    return {"workload": "LogUp-GKR: 2^22 int8-range lookups into a 2^16-entry table, witness tree n=22 + table tree "
                        "n=16, F_p^4, prove-upper of both (side by side: two host threads, two streams)",
            "ms_per_step": 1e3 * dt, "lookups_per_s": (1 << nw) / dt, "ms_per_step_one_after_the_other": 1e3 * dt_serial,
            "proof_bytes": len(tw.proof()) + len(tt.proof()), "proof_sha256": [sha(tw.proof()), sha(tt.proof())],
            "proof_is_the_cpu_oracles": pinned, "verifier_accepts": True,
            "timed_launches_per_step": sum(per for _, per, _ in by.values()),
            "roofline": {"bound": "hbm", "kernel": "prove-upper (whole: tree build + 36 layer sumchecks)",
                         "achieved": nbytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS, "alg_bytes": nbytes, "traffic": None},
            "roofline_by_time": by_time(by)[:8]}


def run_gkr_shapes(sa, steps, warmup):
    """PROVE-UPPER at the shapes a domain gives it (src/domain.lisp:346-349): several lookups proved together and
    several blocks (block weights, a sumcheck over the block index after every layer), trees of 2^14 leaves per block
    and lookup.  Each proof is checked by the library's verifier."""
    d, n, out = 4, 14, {}
    for name, k, lookups in (("one_block_three_lookups", 1, 3), ("three_blocks_one_lookup", 3, 1),
                             ("three_blocks_two_lookups", 3, 2)):
        dev = [(sa.Table.random(700 + 2 * l, k << n, d), sa.Table.random(701 + 2 * l, k << n, d))
               for l in range(lookups)]

        def step():
            tr = sa.Transcript("gkr-shapes", d)
            return tr, sa.prove_upper(tr, n, k, dev)

        dt, (tr, proved) = timed(sa, step, steps, warmup)
        vtr = sa.Transcript("gkr-shapes", d, proof=tr.proof())
        _, ri, rb, cp, cq = sa.verify_upper(vtr, n, k, lookups)
        if not (vtr.finished() and all(np.array_equal(a, b) for a, b in zip((ri, rb, cp, cq), proved))):
            sys.exit("bench.py: the library's verifier does not agree with the proved claims (%s)" % name)
        for p, q in dev:
            p.free(), q.free()
        out[name] = {"n": n, "blocks": k, "lookups": lookups, "ms_per_step": 1e3 * dt,
                     "ms_per_layer": 1e3 * dt / (n - 1), "verifier_accepts": True}
    return out


# ------------------------------------------------------------------ config 5: commitment
def run_commit(sa, steps, warmup, gold):
    cm = wl.COMMIT
    c, ncols = cm["c"], cm["ncols"]
    cols = sa.Table.random(cm["seed"], ncols << c)

    def step():
        tr = sa.Transcript(cm["label"], 4)
        cw, levels = sa.pcs_commit(tr, cols, ncols, c)
        cw.free(), levels.free()
        return tr

    dt, tr = timed(sa, step, steps, warmup)
    from_proof = tr.proof()
    cap = from_proof[-128 * 32:]
    want = gold.get("config5", {}).get("cap_sha256")
    if want is not None and sha(cap) != want:
        sys.exit("bench.py: the timed commitment's cap differs from the CPU oracle's")
    by = launches(sa, step, max(2, min(steps, 10)))
    cols.free()
    nleaves = 1 << (c - 1)
    nbytes = (ncols * (4 << c) + ncols * (4 << (c + 1)) + ncols * (4 << (c + 1)) + 32 * nleaves + 64 * (nleaves - 1)
              + 32 * (nleaves - 1))
    return {"workload": "pcs-commit: 2 columns of 2^23 coefficients -> 2 codewords of 2^24, 2^22 leaves, Merkle levels, "
                        "cap of 128 digests", "ms_per_step": 1e3 * dt, "cap_sha256": sha(cap),
            "cap_is_the_cpu_oracles": want is not None, "leaf_hashes_per_s": nleaves / dt,
            "butterflies_per_s": ncols * 23 * (1 << 23) / dt,
            "roofline": {"bound": "hbm", "kernel": "encode + leaves + Merkle (whole commit)", "achieved": nbytes / dt / 1e9,
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS,
                         "alg_bytes": nbytes, "traffic": None},
            "roofline_by_time": by_time(by)[:8]}


def run_basefold(sa, steps, warmup, gold):
    """Config 5's second half: BASEFOLD (src/pcs.lisp:581-657) of the F_p^8 combination H of the two committed
    columns at nv = 23 -- 18 fold rounds of the message table and the codeword, 8 oracle trees over the folded
    codewords (their caps through the transcript), the final table, grinding, 6 queries' openings.  Timed: the two
    combine-columns launches (H from the columns, its codeword from the committed codewords) and the prove.
    Resident before the timed region: the columns and their codewords (what PCS-COMMIT left)."""
    cm = wl.COMMIT
    c, ncols = cm["c"], cm["ncols"]
    cols = sa.Table.random(cm["seed"], ncols << c)
    cf = splitmix_field(cm["coefficient_seed"], ncols * 8).reshape(ncols, 8)
    rr = splitmix_field(cm["point_seed"], c * 8).reshape(c, 8)
    cw = sa.encode(cols, ncols, c)
    h0 = sa.combine_columns(cols, ncols, cf)
    v = sa.hypercube_sum(sa.Statement("t0", ["t0"]), c, [h0], 8, eq=rr)
    h0.free()

    def step():
        h = sa.combine_columns(cols, ncols, cf)
        cwh = sa.combine_columns(cw, ncols, cf)
        tr = sa.Transcript(cm["open_label"], 4)
        sa.basefold_prove(tr, c, rr, v, h, grind_bits=cm["grind_bits"], queries=cm["queries"], codeword=cwh)
        h.free(), cwh.free()
        return tr

    dt, tr = timed(sa, step, steps, warmup)
    proof = tr.proof()
    want = gold.get("config5", {}).get("basefold", {}).get("proof_sha256")
    if want is not None and sha(proof) != want:
        sys.exit("bench.py: the timed BaseFold proof differs from the CPU oracle's")
    by = launches(sa, step, max(2, min(steps, 5)))
    for t in (cols, cw):
        t.free()
    # algorithmic bytes: the two combinations (columns and codewords read, H and its codeword written); per round i
    # the table of 2^(23-i) EXT8s read and its fold written with the next round's sums taken in the same pass, the
    # codeword of 2^(24-i) EXT8s read and its fold written; per oracle level its codeword read, leaf digests and
    # node levels written and read
    nv, fl = c, c - 5
    ext = 32
    nbytes = ncols * (4 << c) + (ext << c) + ncols * (4 << (c + 1)) + (ext << (c + 1))
    nbytes += ext << nv  # round 0 reads H
    for i in range(fl):
        nbytes += (ext << (nv - i)) + (ext << (nv - i - 1))  # fold of the table
        if i + 1 < fl:
            nbytes += (ext << (nv + 1 - i)) + (ext << (nv - i))  # fold of the codeword
        l = i + 1
        if 2 <= l < fl and l % 2 == 0:
            leaves = (1 << (nv - i)) // 4
            nbytes += (ext << (nv - i)) + 32 * leaves + 64 * (leaves - 1) + 32 * (leaves - 1)
    total_ms = sum(avg * per for avg, per, _ in by.values())
    return {"workload": "BaseFold opening of config 5: combine-columns of the 2 committed columns (2^23) and of their "
                        "codewords (2^24) into F_p^8, then basefold at nv = 23 (18 fold rounds, 8 oracle trees, 6 queries)",
            "ms_per_step": 1e3 * dt, "proof_bytes": len(proof), "proof_sha256": sha(proof),
            "proof_is_the_cpu_oracles": want is not None, "kernel_ms_per_step": total_ms,
            "timed_launches_per_step": sum(per for _, per, _ in by.values()),
            "roofline": {"bound": "hbm", "kernel": "combine-columns x 2 + basefold (whole opening)",
                         "achieved": nbytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS, "alg_bytes": nbytes, "traffic": None},
            "roofline_by_time": by_time(by)[:10]}


def run_combine(sa, steps, warmup, ncols=2):
    """combine-columns at config 5's shape: the committed columns of 2^23 base values into the table of 2^23
    EXT8s that BaseFold opens (src/pcs.lisp:434-441)."""
    c, d = 23, 8
    cols = sa.Table.random(5005, ncols << c)
    cf = splitmix_field(5006, ncols * d).reshape(ncols, d)

    def step():
        sa.combine_columns(cols, ncols, cf).free()

    dt, _ = timed(sa, step, steps, warmup)
    by = launches(sa, step, max(2, min(steps, 10)))
    cols.free()
    nbytes = (1 << c) * (4 * ncols + 4 * d)
    total_ms = sum(avg * per for avg, per, _ in by.values())
    return {"workload": f"combine-columns: {ncols} base columns of 2^23 with F_p^8 coefficients -> 2^23 EXT8s",
            "ms_per_step": 1e3 * dt, "column_entries_per_s": ncols * (1 << c) / dt,
            "roofline": {"bound": "hbm", "kernel": "combine_columns (all launches of a call)",
                         "achieved": nbytes / (total_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": nbytes / (total_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "kernel_ms_per_call": total_ms,
                         "alg_bytes_per_call": nbytes, "traffic": None}}


# ------------------------------------------------------------------ the CPU baseline
def cpu_info():
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return model, os.cpu_count()


def cpu_baseline(sa, n_one, n_all, best_of=7):
    """The CPU oracle (a C restatement of the reference's prover: the statement as straight-line code, lines by
    addition, one reduction per four products, split eq weights; oracle/orc_fast.c) on the headline statement, seeds
    and transcript at smaller n: one thread (the reference is single-threaded) and all host threads (OpenMP over
    the HIGH blocks), best of `best_of` warm runs each.  The one-thread sample then goes through the GPU path as a
    checker of this run: the proof bytes must be the oracle's."""
    from oracle import binding as orc
    cfg = wl.SUMCHECK["config2"]
    d = cfg["d"]
    st = orc.Statement(cfg["form"], cfg["tables"], cfg["constants"])

    def inputs(n):
        tables = [orc.splitmix_field(wl.table_seed(cfg, k), 1 << n) for k in range(3)]
        eq = orc.splitmix_field(wl.eq_seed(cfg), n * d).reshape(n, d)
        alpha = orc.splitmix_field(wl.constants_seed(cfg), d).reshape(1, d)
        return tables, eq, alpha

    def best(n, threads, runs=best_of):
        tables, eq, alpha = inputs(n)
        orc.set_fast(threads)
        times = []
        for _ in range(runs + 1):  # the first run warms the caches and the allocator
            otr = orc.Transcript("config2", d)
            t0 = time.perf_counter()
            orc.prove(otr, n, st, tables, eq=eq, constants=alpha)
            times.append(time.perf_counter() - t0)
        orc.set_fast(0)
        return min(times[1:]), otr.proof(), (tables, eq, alpha)

    threads = orc.host_threads()
    one_s, proof, (tables, eq, alpha) = best(n_one, 1)
    dev = [sa.Table.upload(t) for t in tables]
    tr = sa.Transcript("config2", d)
    sa.prove(tr, n_one, sa.Statement(cfg["form"], cfg["tables"], cfg["constants"]), dev, eq=eq, constants=alpha)
    for t in dev:
        t.free()
    if tr.proof() != proof:
        sys.exit(f"bench.py: the GPU proof at n={n_one} differs from the CPU oracle's")
    all_s, _, _ = best(n_all, threads, best_of if n_all < 24 else 3)
    model, cores = cpu_info()
    return {"value": 3 * (1 << n_one) / one_s, "unit": "table entries/s", "cores": 1, "kind": "port",
            "best_of": best_of, "cpu_model": model, "host_cores": cores,
            "all_threads": {"value": 3 * (1 << n_all) / all_s, "threads": threads,
                            "sample": f"the whole workload, n={n_all}: {all_s:.3f} s per prove, best of {best_of if n_all < 24 else 3}"},
            "sample": f"same statement, seeds and transcript at n={n_one} (3*2^{n_one} entries, {one_s:.2f} s on one "
                      f"thread); the GPU proof of the same sample is byte-identical; the reference's Lisp prover "
                      f"cannot run here (no SBCL)",
            "reference_published": {
                "source": "the reference's README.md:114-149: SBCL 2.2.9, one thread, 4-vCPU Xeon 2.1 GHz VM; none at n=24",
                "3 base tables n=18 F_p^4, small values vs folding": "0.104 s vs 0.120 s = 7.6e6 / 6.6e6 table entries/s",
                "3 base tables n=18 F_p^8, split eq": "0.244 s = 3.2e6 table entries/s",
                "3 extension tables n=18 F_p^8, split eq": "0.424 s = 1.9e6 table entries/s",
                "extrapolated to config 2 (3*2^24 entries at 7.6e6/s; an extrapolation, and the constant alpha keeps the "
                "reference off its base-field kernel, so its real time is higher)": "6.6 s"}}


def run_mulrate(sa, iterations=4096):
    """Issue rates of the VALU instructions the kernels are made of (the peak the integer-multiply figure is a
    fraction of).  Per instruction: cycles per wavefront instruction and SIMD with
    8 workgroups per compute unit of 8 independent chains (issue rate), with one wavefront per SIMD and 8 chains
    (what a lone wavefront can issue), and with one wavefront per SIMD and one chain (dependent latency)."""
    lib = sa.load()
    rows = []
    clock_khz, cus = C.c_int(), C.c_int()
    for op in range(lib.exh_issue_rate_ops()):
        row = {}
        for key, chains, wg_per_cu in (("issue", 8, 8), ("lone_wave", 8, 1), ("dependent", 1, 1)):
            name = C.create_string_buffer(64)
            ms, ipw = C.c_float(), C.c_double()
            # the compute-unit count comes back from the first call; 256 on this part
            groups = wg_per_cu * (cus.value or 256)
            sa.check(lib.exh_issue_rate(op, chains, groups, iterations, name, 64, C.byref(ms), C.byref(ipw),
                                        C.byref(clock_khz), C.byref(cus)))
            groups_now = wg_per_cu * cus.value
            if groups_now != groups:  # first call on a part with another count: measure again at the right grid
                sa.check(lib.exh_issue_rate(op, chains, groups_now, iterations, name, 64, C.byref(ms), C.byref(ipw),
                                            C.byref(clock_khz), C.byref(cus)))
            waves_per_simd = wg_per_cu  # a workgroup of 256 threads puts one wavefront on each of a unit's 4 SIMDs
            cycles = ms.value * 1e-3 * clock_khz.value * 1e3 / (ipw.value * waves_per_simd)
            row["instruction"] = name.value.decode()
            row[key + "_cycles"] = round(cycles, 3)
            row[key + "_ms"] = round(ms.value, 4)
        rows.append(row)
    mad = next(r for r in rows if r["instruction"] == "v_mad_u64_u32")
    rate = {"cycles_per_wave_instruction": mad["issue_cycles"], "clock_ghz": clock_khz.value / 1e6,
            "compute_units": cus.value}
    return {"workload": "VALU issue rates: chains of one instruction, 256 threads per workgroup", "iterations": iterations,
            "clock_khz": clock_khz.value, "compute_units": cus.value, "rates": rows,
            "int32_mul_peak_per_s": int32_mul_peak(rate), "int32_mul_rate": rate}


def run_copy(steps):
    """Calibration for the traffic counters: an elementwise kernel that reads 256 MiB and writes 256 MiB."""
    import torch
    a = torch.ones(1 << 26, dtype=torch.int32, device="cuda")
    b = torch.empty_like(a)
    for _ in range(steps):
        torch.add(a, 1, out=b)
    torch.cuda.synchronize()
    print(json.dumps({"workload": "copy", "read_bytes": a.numel() * 4, "written_bytes": b.numel() * 4, "steps": steps}))


def line(metric, value, unit, higher, dtype, data, res, steps, warmup):
    out = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
           "ms_per_step": res["ms_per_step"], "higher_is_better": higher, "scaling": "weak", "vs_baseline": None,
           "dtype": dtype, "data": data, "config": {"workload": res["workload"]}}
    for k, v in res.items():
        if k in ("roofline", "roofline_by_time", "loop_hbm_fraction"):
            out[k] = v
        elif k not in ("workload", "ms_per_step"):
            out["config"][k] = v
    return out


SEEDED = "synthetic (SplitMix64-seeded uniform field elements)"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="config2",
                    choices=["config1", "config2", "config3", "config4", "config5", "basefold", "domain", "combine",
                             "combine128", "copy", "mulrate", "gkr_shapes"],
                    help="config2 (default) is the headline; the others are the remaining configured workloads; "
                         "copy is the known-size kernel the traffic counters are calibrated on")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=0, help="variables, when not the configured size")
    ap.add_argument("--cpu-n", type=int, default=20, help="variables of the one-thread CPU baseline's sample (0: skip)")
    ap.add_argument("--others", type=int, default=1, help="0: leave the other configured workloads out of the headline's line")
    args = ap.parse_args()
    sys.stdout.reconfigure(line_buffering=True)  # the line is out before the process ends, whatever ends it
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus above 1 is not supported (nothing here uses a "
                 "second device)")
    if args.workload == "copy":
        run_copy(args.steps)
        return
    # No kernels are compiled behind the bench's back: every statement here has its kernels in the library, or asks
    # for them and waits (the wide statement's direct form).  The library would otherwise start a compilation for
    # the parts of the wide statement when they are proved at n = 20, and the process would end under it.
    os.environ.setdefault("EXACTA_HIP_RTC_MIN_N", "64")
    import sable_amd as sa
    sa.init(0)
    gold = golden()
    steps, warmup, n = args.steps, args.warmup, args.n or None
    if args.workload in ("config1", "config3"):
        res = run_sumcheck(sa, args.workload, steps, warmup, gold, n)
        d = res["extension"]
        print(json.dumps(line(f"sumcheck table entries/s ({args.workload})", res["entries_per_s"], "table entries/s", True,
                              f"u32 (Montgomery KoalaBear, F_p^{d} tower)", SEEDED, res, steps, warmup)))
        return
    if args.workload == "domain":
        res = run_domain(sa, steps, warmup, n)
        print(json.dumps(line("sumcheck table entries/s (wide statement, direct form)", res["entries_per_s"],
                              "table entries/s", True, "u32 (Montgomery KoalaBear, F_p^4 tower)", SEEDED, res, steps,
                              warmup)))
        return
    if args.workload == "config4":
        res = run_gkr(sa, steps, warmup, gold)
        print(json.dumps(line("LogUp-GKR prove-upper lookups/s (config 4)", res["lookups_per_s"], "lookups/s", True,
                              "u32 (Montgomery KoalaBear, F_p^4 tower)",
                              "synthetic (seeded uniform int8 lookups, exact multiplicities)", res, steps, warmup)))
        return
    if args.workload == "gkr_shapes":
        shapes = run_gkr_shapes(sa, steps, warmup)
        blocks = shapes["three_blocks_one_lookup"]
        res = {"workload": "LogUp-GKR prove-upper at the shapes a domain gives it: 2^14 leaves per block and lookup, "
                           "one block with three lookups, three blocks with one and with two; `value` is three blocks "
                           "with one lookup", "ms_per_step": blocks["ms_per_step"], "shapes": shapes}
        print(json.dumps(line("LogUp-GKR prove-upper lookups/s (3 blocks of 2^14)", 3 * (1 << 14) / (blocks["ms_per_step"] * 1e-3),
                              "lookups/s", True, "u32 (Montgomery KoalaBear, F_p^4 tower)", SEEDED, res, steps, warmup)))
        return
    if args.workload == "config5":
        res = run_commit(sa, steps, warmup, gold)
        print(json.dumps(line("BaseFold commit ms (config 5)", res["ms_per_step"], "ms", False,
                              "u32 (Montgomery KoalaBear) + BLAKE3", SEEDED, res, steps, warmup)))
        return
    if args.workload == "basefold":
        res = run_basefold(sa, steps, warmup, gold)
        print(json.dumps(line("BaseFold opening ms (config 5, nv = 23)", res["ms_per_step"], "ms", False,
                              "u32 (Montgomery KoalaBear, F_p^8) + BLAKE3", SEEDED, res, steps, warmup)))
        return
    if args.workload == "mulrate":
        res = run_mulrate(sa)
        print(json.dumps({"metric": "int32 multiply issue peak", "value": res["int32_mul_peak_per_s"],
                          "unit": "32-bit multiplies/s (per lane)", "n_gpus": 1, "config": res}))
        return
    if args.workload in ("combine", "combine128"):
        res = run_combine(sa, steps, warmup, 128 if args.workload == "combine128" else 2)
        print(json.dumps(line("combine-columns entries/s (config 5's columns)", res["column_entries_per_s"],
                              "column entries/s", True, "u32 (Montgomery KoalaBear, F_p^8)", SEEDED, res, steps, warmup)))
        return

    # ---- the headline: config 2
    res = run_sumcheck(sa, "config2", steps, warmup, gold, n)
    current = MEASURED["kernel_sources_sha256"] == kernel_sources_sha256()
    kname = res["roofline"]["kernel"].split(" ")[0]
    res["roofline"]["traffic"] = MEASURED["traffic"].get((kname, res["n"])) if current else None
    out = line("sumcheck table entries/s at n=24 deg-3", res["entries_per_s"], "table entries/s", True,
               "u32 (Montgomery KoalaBear, F_p^4 tower; exact integers in f64 for the first sweep's products)", SEEDED,
               res, steps, warmup)
    muls = MEASURED["int32_mul_per_prove"] if current and res["n"] == 24 else None
    rate = run_mulrate(sa, 1024)["int32_mul_rate"]  # measured in this run
    peak = int32_mul_peak(rate)
    out["int32_mul"] = {"bound": "int32 multiply issue", "multiplies_per_step": muls, "peak": peak, "peak_from": rate,
                        "unit": "32-bit multiplies/s (per lane)",
                        "achieved": muls / (res["ms_per_step"] * 1e-3) if muls else None,
                        "frac": muls / (res["ms_per_step"] * 1e-3) / peak if muls else None,
                        "note": "counts are from the kernels' instruction streams and go with one version of the "
                                "sources (null when they have changed since)"}
    # one thread on a bounded sample (n = --cpu-n), all host threads at the headline's own size
    out["cpu_baseline"] = cpu_baseline(sa, args.cpu_n, 24 if res["n"] == 24 else res["n"]) if args.cpu_n > 0 else None
    if args.others and n is None:
        k = max(3, steps // 4)
        others = {}
        for name in ("config1", "config3"):
            r = run_sumcheck(sa, name, k, 2, gold)
            others[name] = {key: r[key] for key in ("workload", "ms_per_step", "entries_per_s", "proof_sha256",
                                                    "proof_is_the_cpu_oracles", "loop_hbm_fraction")}
            others[name]["roofline"] = r["roofline"]
        r = run_gkr(sa, k, 2, gold)
        others["config4"] = {key: r[key] for key in ("workload", "ms_per_step", "ms_per_step_one_after_the_other",
                                                     "lookups_per_s", "proof_sha256", "proof_is_the_cpu_oracles",
                                                     "timed_launches_per_step", "roofline")}
        others["config4"]["domain_shapes"] = run_gkr_shapes(sa, k, 2)
        r = run_commit(sa, k, 2, gold)
        others["config5"] = {key: r[key] for key in ("workload", "ms_per_step", "cap_sha256", "cap_is_the_cpu_oracles",
                                                     "roofline")}
        r = run_basefold(sa, k, 2, gold)
        others["config5"]["basefold"] = {key: r[key] for key in ("workload", "ms_per_step", "proof_sha256",
                                                                 "proof_is_the_cpu_oracles", "kernel_ms_per_step",
                                                                 "timed_launches_per_step", "roofline")}
        r = run_domain(sa, k, 2)
        others["wide_statement"] = {key: r[key] for key in ("workload", "ms_per_step", "ms_per_step_in_parts",
                                                            "entries_per_s", "proof_sha256", "proof_is_the_parts_paths",
                                                            "timed_launches_per_step", "loop_hbm_fraction", "roofline")}
        out["other_configs"] = others
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
