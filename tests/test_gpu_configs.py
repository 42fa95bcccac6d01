"""The five configured workloads at their full sizes on the GPU, through the C ABI, against the CPU oracle:
whole proofs byte for byte (a fresh oracle run on the host's cores where that takes seconds, and the committed
digests of tests/golden/config_hashes.json, which the same oracle wrote, everywhere), the library's own verifier
on every proof, and extreme inputs (all p - 1, all 0, eq points with 0 and 1 coordinates) down the default
path of the large sizes: base-field sweep, double fold, streaming rounds, LDS-resident slices, tail.
Integer work: every comparison is bit-exact.  (tests/tests.lisp:264-282, :329-395, :414-462)"""
import hashlib
import json
import os

import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc
from sable_amd import workloads as wl

pytestmark = pytest.mark.gpu
P = sa.P
HERE = os.path.dirname(os.path.abspath(__file__))


def sha(b):
    return hashlib.sha256(bytes(b)).hexdigest()


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "config_hashes.json")) as f:
        return json.load(f)


@pytest.fixture(autouse=True)
def threaded_oracle():
    orc.set_fast(orc.host_threads())
    yield
    orc.set_fast(0)


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


def test_seeded_tables_are_the_host_generators():
    for seed, count in ((1, 1), (2000, 4097), (5005, 1 << 16)):
        t = sa.Table.random(seed, count)
        assert same(t.download(), orc.splitmix_field(seed, count))
        t.free()


def sumcheck_inputs(cfg, n):
    d = cfg["d"]
    eq = orc.splitmix_field(wl.eq_seed(cfg), n * d).reshape(n, d)
    cv = orc.splitmix_field(wl.constants_seed(cfg), d * len(cfg["constants"])).reshape(-1, d) if cfg["constants"] else None
    return eq, cv


def gpu_prove(name, cfg, n, dev, eq, cv):
    st = sa.Statement(cfg["form"], cfg["tables"], cfg["constants"])
    tr = sa.Transcript(name, cfg["d"])
    chal, finals, _ = sa.prove(tr, n, st, dev, eq=eq, constants=cv)
    return st, tr.proof(), chal, finals


def oracle_prove(name, cfg, n, host, eq, cv):
    ost = orc.Statement(cfg["form"], cfg["tables"], cfg["constants"])
    otr = orc.Transcript(name, cfg["d"])
    chal, finals, _ = orc.prove(otr, n, ost, host, eq=eq, constants=cv)
    return ost, otr.proof(), chal, finals


def accepted_by_the_verifier(name, cfg, n, st, dev, proof, finals, eq, cv):
    """hypercube-sum -> verify -> check-final in the library itself (src/sumcheck.lisp:147-172)"""
    claim = sa.hypercube_sum(st, n, dev, cfg["d"], eq=eq, constants=cv)
    vtr = sa.Transcript(name, cfg["d"], proof=proof)
    _, reduced = sa.verify(vtr, n, st, claim, eq=eq, constants=cv)
    assert vtr.finished() and sa.check_final(reduced, st, finals, constants=cv)


@pytest.mark.parametrize("name", ["config1", "config2"])
def test_sumcheck_config_at_full_size_against_a_fresh_oracle_run(name, golden):
    cfg = wl.SUMCHECK[name]
    n, T = cfg["n"], len(cfg["tables"])
    eq, cv = sumcheck_inputs(cfg, n)
    dev = [sa.Table.random(wl.table_seed(cfg, k), 1 << n) for k in range(T)]
    st, proof, chal, finals = gpu_prove(name, cfg, n, dev, eq, cv)
    assert st.has_generated_kernel(cfg["d"])
    host = [orc.splitmix_field(wl.table_seed(cfg, k), 1 << n) for k in range(T)]
    _, want, ochal, ofinals = oracle_prove(name, cfg, n, host, eq, cv)
    assert proof == want, f"{name}: the GPU proof at n={n} differs from the oracle's"
    assert same(chal, ochal) and same(finals, ofinals)
    assert sha(proof) == golden[name]["proof_sha256"] and len(proof) == golden[name]["proof_bytes"]
    assert sha(np.ascontiguousarray(finals).tobytes()) == golden[name]["finals_sha256"]
    accepted_by_the_verifier(name, cfg, n, st, dev, proof, finals, eq, cv)
    for t in dev:
        t.free()


def test_config3_fp8_at_full_size_against_the_oracles_digest(golden):
    """n = 26, four base tables (1 GiB), F_p^8, the six-launch sweep: the oracle's run of this size takes a minute
    of all cores, so its digest is the committed one; the same path runs against a fresh oracle at n = 22 below."""
    name, cfg = "config3", wl.SUMCHECK["config3"]
    n = cfg["n"]
    eq, cv = sumcheck_inputs(cfg, n)
    dev = [sa.Table.random(wl.table_seed(cfg, k), 1 << n) for k in range(4)]
    st, proof, chal, finals = gpu_prove(name, cfg, n, dev, eq, cv)
    assert st.has_generated_kernel(8)
    assert len(proof) == golden[name]["proof_bytes"] == 12 + n * (18 + 4 * 4 * 8)
    assert sha(proof) == golden[name]["proof_sha256"], "config 3: the GPU proof at n=26 differs from the oracle's"
    assert sha(np.ascontiguousarray(finals).tobytes()) == golden[name]["finals_sha256"]
    accepted_by_the_verifier(name, cfg, n, st, dev, proof, finals, eq, cv)
    for t in dev:
        t.free()


@pytest.mark.parametrize("name,n", [("config3", 22), ("config2", 22), ("config2", 21), ("config1", 23)])
def test_large_default_path_against_a_fresh_oracle_run(name, n):
    """Sizes where the large-size path engages by default (several pairs per thread, 512 workgroups, the sweep
    for rounds 0 and 1, the double fold), other than the configured ones."""
    cfg = wl.SUMCHECK[name]
    T = len(cfg["tables"])
    eq, cv = sumcheck_inputs(cfg, n)
    dev = [sa.Table.random(wl.table_seed(cfg, k) + 50, 1 << n) for k in range(T)]
    host = [orc.splitmix_field(wl.table_seed(cfg, k) + 50, 1 << n) for k in range(T)]
    st, proof, chal, finals = gpu_prove(name, cfg, n, dev, eq, cv)
    _, want, ochal, ofinals = oracle_prove(name, cfg, n, host, eq, cv)
    assert proof == want and same(chal, ochal) and same(finals, ofinals)
    for t in dev:
        t.free()


EXTREME = "(* (+ t0 t1 t2 t3 -1) (- t0 t1 t2 t3))"  # two four-term linear forms, every coefficient +-1


def extreme_tables(kind, T, n, rng):
    size = 1 << n
    if kind == "max":
        return [np.full(size, P - 1, np.uint32) for _ in range(T)]
    if kind == "zero":
        return [np.zeros(size, np.uint32) for _ in range(T)]
    if kind == "first-max":  # the differences of a linear form at their largest: one table p - 1, the others 0
        return [np.full(size, P - 1 if t == 0 else 0, np.uint32) for t in range(T)]
    if kind == "alternating":  # slopes of +-(p - 1) in every pair and between pairs
        a = np.where(np.arange(size) % 2 == 0, P - 1, 0).astype(np.uint32)
        b = np.where((np.arange(size) // 2) % 2 == 0, 0, P - 1).astype(np.uint32)
        return [a if t % 2 == 0 else b for t in range(T)]
    return [rng.choice(np.array([0, 1, P - 1, P - 2, (P - 1) // 2], np.uint32), size) for _ in range(T)]


@pytest.mark.parametrize("kind", ["max", "zero", "first-max", "alternating", "mixed"])
@pytest.mark.parametrize("form,names,cnames,d,n", [
    (wl.SUMCHECK["config2"]["form"], ["t0", "t1", "t2"], ["alpha"], 4, 22),
    (wl.SUMCHECK["config3"]["form"], ["c0", "c1", "c2", "c3"], [], 8, 21),
    (EXTREME, ["t0", "t1", "t2", "t3"], [], 4, 22),
], ids=["config2", "config3", "four-term-forms"])
def test_extreme_values_down_the_default_path(kind, form, names, cnames, d, n):
    """The exact-integer double-precision products of the sweep, the 96-bit accumulators and the counted totals
    of the slices at the ends of their ranges: tables of p - 1, of 0, of the few residues next to them, with an
    eq point that has 0, 1 and p - 1 among its coordinates."""
    rng = np.random.default_rng(len(kind) + n)
    T = len(names)
    host = extreme_tables(kind, T, n, rng)
    eq = rng.integers(0, P, (n, d), dtype=np.uint32)
    eq[1] = 0
    eq[2] = [1] + [0] * (d - 1)
    eq[n - 1] = [1] + [0] * (d - 1)
    eq[n - 3] = 0
    eq[5] = P - 1
    cv = np.full((len(cnames), d), P - 1, np.uint32) if cnames else None
    st, ost = sa.Statement(form, names, cnames), orc.Statement(form, names, cnames)
    assert st.has_generated_kernel(d)
    dev = [sa.Table.upload(t) for t in host]
    tr, otr = sa.Transcript("extreme", d), orc.Transcript("extreme", d)
    got = sa.prove(tr, n, st, dev, eq=eq, constants=cv)
    want = orc.prove(otr, n, ost, host, eq=eq, constants=cv)
    assert tr.proof() == otr.proof(), f"{kind}: proof bytes differ"
    assert same(got[0], want[0]) and same(got[1], want[1])
    for t in dev:
        t.free()


@pytest.mark.parametrize("kind", ["max", "alternating", "mixed"])
def test_extreme_values_on_the_small_paths(kind, monkeypatch):
    """The same inputs at n = 13: once on the default path of that size (slices and tail only), once with the
    slices capped so that the sweep, the double fold and the streaming rounds run on small grids."""
    n, d = 13, 4
    cfg = wl.SUMCHECK["config2"]
    rng = np.random.default_rng(13)
    host = extreme_tables(kind, 3, n, rng)
    eq = rng.integers(0, P, (n, d), dtype=np.uint32)
    eq[0], eq[4] = 0, [1, 0, 0, 0]
    cv = np.full((1, d), P - 1, np.uint32)
    ost = orc.Statement(cfg["form"], cfg["tables"], cfg["constants"])
    otr = orc.Transcript("extreme-small", d)
    orc.prove(otr, n, ost, host, eq=eq, constants=cv)
    for cap in (None, "0"):
        if cap is not None:
            monkeypatch.setenv("EXACTA_HIP_MAX_SLICE_PAIRS", cap)
        st = sa.Statement(cfg["form"], cfg["tables"], cfg["constants"])
        dev = [sa.Table.upload(t) for t in host]
        tr = sa.Transcript("extreme-small", d)
        sa.prove(tr, n, st, dev, eq=eq, constants=cv)
        assert tr.proof() == otr.proof(), f"{kind}, slice cap {cap}"
        for t in dev:
            t.free()


# ------------------------------------------------------------------ config 4: LogUp-GKR
def test_gkr_config_at_full_size_against_a_fresh_oracle_run(golden):
    """prove-upper of the witness tree (2^22 leaves) and the table tree (2^16): whole proofs, the next claims and
    the verifier; the two roots are equal as fractions (the lookup argument holds)."""
    g = wl.GKR
    d = g["d"]
    z = sa.Transcript(g["z_label"], d).challenge()
    assert [int(x) for x in z] == golden["config4"]["z"]
    words = orc.splitmix_field(g["seed"], 1 << g["n_witness"])
    wit, tab = wl.gkr_leaves(np, words, z, g["n_witness"], g["n_table"], d)
    roots = []
    for key, leaves, n, label in (("witness", wit, g["n_witness"], g["witness_label"]),
                                  ("table", tab, g["n_table"], g["table_label"])):
        dev = (sa.Table.upload(leaves[0]), sa.Table.upload(leaves[1]))
        tr, otr = sa.Transcript(label, d), orc.Transcript(label, d)
        got = sa.prove_upper(tr, n, 1, [dev])
        want = orc.gkr_prove_upper(otr, n, 1, [leaves])
        assert tr.proof() == otr.proof(), f"config 4, {key} tree: proof bytes differ"
        for a, b in zip(got, want):
            assert same(a, b)
        assert sha(tr.proof()) == golden["config4"][key]["proof_sha256"]
        vtr = sa.Transcript(label, d, proof=tr.proof())
        vroots, ri, rb, cp, cq = sa.verify_upper(vtr, n, 1, 1)
        assert vtr.finished() and same(ri, got[0]) and same(cp, got[2]) and same(cq, got[3])
        roots.append(vroots[0])
        dev[0].free(), dev[1].free()
    assert same(orc.ext_mul(roots[0][0], roots[1][1]), orc.ext_mul(roots[1][0], roots[0][1]))


@pytest.mark.parametrize("n,k,lookups", [(14, 1, 1), (16, 1, 1), (15, 2, 1), (13, 3, 2), (17, 1, 2)])
def test_gkr_mid_sizes_with_block_weights(n, k, lookups):
    """Layers large enough for the streaming kernels and the grid of LDS-resident slices, with extension tables
    and block weights (K > 1 adds the top tree and the zero-padded block sumcheck)."""
    d = 4
    leaves = []
    for l in range(lookups):
        p = orc.splitmix_field(100 * n + 2 * l, (k << n) * d).reshape(-1, d)
        q = orc.splitmix_field(100 * n + 2 * l + 1, (k << n) * d).reshape(-1, d)
        leaves.append((p, q))
    dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
    tr, otr = sa.Transcript("gkr-mid", d), orc.Transcript("gkr-mid", d)
    got = sa.prove_upper(tr, n, k, dev)
    want = orc.gkr_prove_upper(otr, n, k, leaves)
    assert tr.proof() == otr.proof()
    for a, b in zip(got, want):
        assert same(a, b)
    vtr = sa.Transcript("gkr-mid", d, proof=tr.proof())
    sa.verify_upper(vtr, n, k, lookups)
    assert vtr.finished()
    for p, q in dev:
        p.free(), q.free()


# ------------------------------------------------------------------ config 5: commitment and BaseFold
def test_commit_config_at_full_size_against_a_fresh_oracle_run(golden):
    """pcs-commit of two columns of 2^23: both codewords, all 2^23 - 1 digests of the tree and the cap of 128."""
    cm = wl.COMMIT
    c, ncols = cm["c"], cm["ncols"]
    cols = sa.Table.random(cm["seed"], ncols << c)
    tr = sa.Transcript(cm["label"], 4)
    cw, levels = sa.pcs_commit(tr, cols, ncols, c)
    cap = np.frombuffer(orc.decode_proof(tr.proof())[0], np.uint8).reshape(-1, 32)
    flat = orc.splitmix_field(cm["seed"], ncols << c)
    ocw, olevels, ocap = orc.commit_columns([flat[k << c:(k + 1) << c] for k in range(ncols)], c)
    assert same(cap, ocap) and len(cap) == 128
    assert same(cw.download().reshape(ncols, -1), ocw), "codewords differ"
    dev_levels = levels.download().reshape(-1).astype("<u4").view(np.uint8).reshape(-1, 32)
    assert same(dev_levels, np.concatenate(olevels)), "Merkle levels differ"
    g = golden["config5"]
    assert sha(np.ascontiguousarray(cap).tobytes()) == g["cap_sha256"]
    assert sha(cw.download().tobytes()) == g["codewords_sha256"]
    assert sha(dev_levels.tobytes()) == g["levels_sha256"]
    for t in (cols, cw, levels):
        t.free()


def test_basefold_config_at_full_size_against_the_oracles_digest(golden):
    """BaseFold of the two columns' F_p^8 combination at nv = 23 (18 fold rounds, 8 oracle trees, 6 queries): the
    claim, the query positions and the proof's digest are the oracle's (its run takes a minute: committed)."""
    cm, g = wl.COMMIT, golden["config5"]["basefold"]
    c, ncols = cm["c"], cm["ncols"]
    cols = sa.Table.random(cm["seed"], ncols << c)
    cf = orc.splitmix_field(cm["coefficient_seed"], ncols * 8).reshape(ncols, 8)
    rr = orc.splitmix_field(cm["point_seed"], c * 8).reshape(c, 8)
    h = sa.combine_columns(cols, ncols, cf)
    v = sa.hypercube_sum(sa.Statement("t0", ["t0"]), c, [h], 8, eq=rr)
    assert [int(x) for x in v] == g["claim"]
    tr = sa.Transcript(cm["open_label"], 4)
    qs, chal, final = sa.basefold_prove(tr, c, rr, v, h, grind_bits=cm["grind_bits"], queries=cm["queries"])
    proof = tr.proof()
    assert qs == g["queries"] and len(proof) == g["proof_bytes"]
    assert sha(proof) == g["proof_sha256"], "config 5: the BaseFold proof at nv=23 differs from the oracle's"
    assert sa.basefold_verify(sa.Transcript(cm["open_label"], 4, proof=proof), c, rr, v, cm["grind_bits"],
                              cm["queries"]) == qs
    # the same opening with the table's codeword taken from the commitment (the combination of the committed
    # codewords, by the encoder's linearity) instead of eight transforms: the same bytes
    cw = sa.encode(cols, ncols, c)
    cwh = sa.combine_columns(cw, ncols, cf)
    tr2 = sa.Transcript(cm["open_label"], 4)
    qs2, _, _ = sa.basefold_prove(tr2, c, rr, v, h, grind_bits=cm["grind_bits"], queries=cm["queries"], codeword=cwh)
    assert qs2 == qs and tr2.proof() == proof, "config 5: the opening from the committed codewords differs"
    for t in (cols, h, cw, cwh):
        t.free()


@pytest.mark.parametrize("nv", [16, 19])
def test_basefold_mid_sizes_against_a_fresh_oracle_run(nv):
    h = orc.splitmix_field(700 + nv, 8 << nv).reshape(-1, 8)
    rr = orc.splitmix_field(800 + nv, nv * 8).reshape(nv, 8)
    v = orc.mle_eval(h, rr, 8)
    t = sa.Table.upload(h)
    tr, otr = sa.Transcript("bf-mid", 4), orc.Transcript("bf-mid", 4)
    got = sa.basefold_prove(tr, nv, rr, v, t)
    want = orc.basefold_prove(otr, nv, rr, v, h)
    assert tr.proof() == otr.proof()
    assert got[0] == want[0] and same(got[1], want[1]) and same(got[2], want[2])
    t.free()
