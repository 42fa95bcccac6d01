"""GPU parity for the sumcheck path: the HIP library through its C ABI against the golden whole-proof
vectors and against the CPU oracle on seeded inputs.  Integer work: every comparison is bit-exact."""
import numpy as np
import pytest

import sable_amd as sa
from conftest import launch_names
from oracle import binding as orc

pytestmark = pytest.mark.gpu
P = sa.P
hx = bytes.fromhex


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


def rand_ext(rng, shape, d):
    return rng.integers(0, P, tuple(shape) + (d,), dtype=np.uint32)


def both(form, tables, constants=()):
    return sa.Statement(form, tables, constants), orc.Statement(form, tables, constants)


def prove_both(label, d, n, form, names, host_tables, eq=None, constants=None, cnames=(), block_weights=None,
               degree=None, sc_label="sc"):
    st, ost = both(form, names, cnames)
    dev = [sa.Table.upload(t) for t in host_tables]
    tr, otr = sa.Transcript(label, d), orc.Transcript(label, d)
    got = sa.prove(tr, n, st, dev, eq=eq, constants=constants, block_weights=block_weights, degree=degree,
                   label=sc_label)
    want = orc.prove(otr, n, ost, host_tables, eq=eq, constants=constants, block_weights=block_weights,
                     degree=degree, label=sc_label)
    for t in dev:
        t.free()
    assert tr.proof() == otr.proof(), f"proof bytes differ: {form} n={n} D={d}"
    assert same(got[0], want[0]) and same(got[1], want[1])
    for a, b in zip(got[2], want[2]):
        assert same(a, b)
    return st, ost, tr.proof(), got


def test_golden_proofs_byte_for_byte(vectors):
    """tests.lisp:277-282: the prover writes the same bytes as the original prover, after the magic."""
    for v in vectors("sumcheck"):
        d, n, nt = v["d"], v["n"], len(v["tables"])
        names = [f"t{i}" for i in range(nt)]
        st = sa.Statement("(* " + " ".join(names) + ")", names)
        tables = [sa.Table.upload(np.array(t, np.uint32)) for t in v["tables"]]
        eq = np.array(v["eq_r"], np.uint32) if v["eq_r"] else None
        assert same(sa.hypercube_sum(st, n, tables, d, eq=eq), v["claim"])
        tr = sa.Transcript("sc-vec", d)
        rho, finals, _ = sa.prove(tr, n, st, tables, eq=eq)
        assert same(rho, v["rho"]) and same(finals, v["finals"])
        assert tr.proof() == b"EXACTPF1" + hx(v["proof"])[8:]
        for t in tables:
            t.free()


@pytest.mark.parametrize("n", [1, 2, 5, 9, 12, 16])
def test_config1_product_of_two_base_tables(n):
    """(* eq t0 t1): two base tables, eq mode, F_p^4; n = 16 is the full configuration."""
    rng = np.random.default_rng(1000 + n)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(2)]
    eq = rand_ext(rng, (n,), 4)
    st, ost, proof, _ = prove_both("config1", 4, n, "(* t0 t1)", ["t0", "t1"], tables, eq=eq)
    assert st.has_generated_kernel(4)
    assert len(proof) == 12 + n * (18 + 4 * 2 * 4)
    # the oracle's verifier accepts the GPU proof
    claim = orc.hypercube_sum(ost, n, tables, 4, eq=eq)
    dev = [sa.Table.upload(t) for t in tables]
    assert same(sa.hypercube_sum(st, n, dev, 4, eq=eq), claim)
    vtr = orc.Transcript("config1", 4, proof=proof)
    _, reduced = orc.verify(vtr, n, ost, claim, eq=eq)
    finals = sa.prove(sa.Transcript("config1", 4), n, st, dev, eq=eq)[1]
    assert orc.check_final(reduced, ost, finals) and vtr.finished()
    for t in dev:
        t.free()


CONFIG2 = "(+ (* alpha t0 t1 t2) (* 3 t1))"
CONFIG3 = "(* (+ c0 3) (- c1 c0) c2 c3)"


@pytest.mark.parametrize("n", [1, 3, 8, 13])
def test_config2_statement_with_a_constant(n):
    rng = np.random.default_rng(2000 + n)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    eq, alpha = rand_ext(rng, (n,), 4), rand_ext(rng, (1,), 4)
    st, ost, proof, _ = prove_both("config2", 4, n, CONFIG2, ["t0", "t1", "t2"], tables, eq=eq, constants=alpha,
                                   cnames=["alpha"])
    assert st.has_generated_kernel(4) and st.degree == 3
    assert len(proof) == 12 + n * (18 + 4 * 3 * 4)
    claim = orc.hypercube_sum(ost, n, tables, 4, eq=eq, constants=alpha)
    vtr = sa.Transcript("config2", 4, proof=proof)
    _, reduced = sa.verify(vtr, n, st, claim, eq=eq, constants=alpha)
    dev = [sa.Table.upload(t) for t in tables]
    assert same(sa.hypercube_sum(st, n, dev, 4, eq=eq, constants=alpha), claim)
    for t in dev:
        t.free()


@pytest.mark.parametrize("n", [2, 7, 11])
def test_config3_product_constraint_over_fp8(n):
    rng = np.random.default_rng(3000 + n)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(4)]
    eq = rand_ext(rng, (n,), 8)
    st, ost, proof, _ = prove_both("config3", 8, n, CONFIG3, ["c0", "c1", "c2", "c3"], tables, eq=eq)
    assert st.degree == 4 and len(proof) == 12 + n * (18 + 4 * 4 * 8)


DOMAIN_FORM = ("(+ (* A0 (+ (* m0 (- Z g1 (* BETA0 v1))) (* m1 (- Z g0 (* BETA0 v0)))))"
               " (* AL0 (- Z g0 (* BETA0 v0)) (- Z g1 (* BETA0 v1)))"
               " (* GAM0 c0) (* GETA0 c1))")
DOMAIN_TABLES = ["g0", "g1", "v0", "v1", "m0", "m1", "c0", "c1"]
DOMAIN_CONSTANTS = ["Z", "BETA0", "A0", "AL0", "GAM0", "GETA0"]


@pytest.mark.parametrize("form,names,cnames,d,base,with_eq", [
    ("(* t0 t1 t2)", ["t0", "t1", "t2"], [], 4, True, True),
    ("(* t0 t1 t2)", ["t0", "t1", "t2"], [], 8, False, False),
    ("(+ (* t0 t1 t2) (* 7 t1) -1)", ["t0", "t1", "t2"], [], 4, True, True),
    ("(+ (* t0 t1 t2) (* 7 t1) -1)", ["t0", "t1", "t2"], [], 8, True, False),
    ("(- (* alpha (expt t0 2) t1) t1)", ["t0", "t1"], ["alpha"], 4, False, True),
    ("t0", ["t0"], [], 4, True, True),
    ("(- (expt t0 3) (* t0 t1))", ["t0", "t1"], [], 8, True, True),
    ("(* t0 t1 t2 t3)", ["t0", "t1", "t2", "t3"], [], 4, False, True),
    ("(+ (* alpha t0 t1) (* 3 t1) -2)", ["t0", "t1"], ["alpha"], 4, False, False),
    # products of linear forms: kept as factors on the device, identical field elements
    ("(* (+ (* 2 t0) t1 5) (- t0 7) t2)", ["t0", "t1", "t2"], [], 4, True, True),
    ("(* (+ (* 2 t0) t1 5) (- t0 7) t2)", ["t0", "t1", "t2"], [], 8, False, True),
    ("(+ (* alpha (+ t0 1) (- t1 t0) t2) (* 3 t0) 9)", ["t0", "t1", "t2"], ["alpha"], 4, False, True),
    ("(- (* (expt (- t0 1) 2) (+ t1 t0)) (* beta (- t1 4) t0))", ["t0", "t1"], ["beta"], 4, True, False),
    ("(* (- t0) (+ t1 -3) (+ t0 t1 t2 t3 1) t3)", ["t0", "t1", "t2", "t3"], [], 8, True, True),
    # the shape of DOMAIN-STATEMENT (src/domain.lisp:95-114): a lookup with a numerator, its denominators
    # q = Z - tag - BETA0 * value at both halves, and a constraint's two halves
    (DOMAIN_FORM, DOMAIN_TABLES, DOMAIN_CONSTANTS, 8, True, True),
    (DOMAIN_FORM, DOMAIN_TABLES, DOMAIN_CONSTANTS, 4, False, True),
])
def test_any_statement_on_the_interpreter_or_generated_kernels(form, names, cnames, d, base, with_eq):
    """tests.lisp:311-395: statements that are not plain products, constants, base or extension tables."""
    n = 6
    rng = np.random.default_rng(len(form) + d)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) if base else rand_ext(rng, (1 << n,), d) for _ in names]
    eq = rand_ext(rng, (n,), d) if with_eq else None
    consts = rand_ext(rng, (len(cnames),), d) if cnames else None
    prove_both("any", d, n, form, names, tables, eq=eq, constants=consts, cnames=cnames)


def test_mixed_base_and_extension_tables():
    n, d = 5, 4
    rng = np.random.default_rng(77)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32), rand_ext(rng, (1 << n,), d)]
    prove_both("mixed", d, n, "(* t0 t1)", ["t0", "t1"], tables, eq=rand_ext(rng, (n,), d))


@pytest.mark.parametrize("K,n,d", [(3, 3, 4), (1, 4, 4), (5, 2, 8), (2, 0, 4)])
def test_block_weights(K, n, d):
    """prove with :block-weights (sumcheck.lisp:519-521, 549-550), as the GKR layers call it."""
    rng = np.random.default_rng(K * 10 + n)
    tables = [rand_ext(rng, (K << n,), d) for _ in range(2)]
    bw = rand_ext(rng, (K,), d)
    eq = rand_ext(rng, (n,), d) if n else None
    prove_both("bw", d, n, "(* t0 t1)", ["t0", "t1"], tables, eq=eq, block_weights=bw, degree=2 if n else 0,
               sc_label="gkr")


def test_round_by_round_session_matches_the_oracle_rounds():
    """The entry points an SBCL host binds: round sums and folds, one call each."""
    n, d = 7, 4
    rng = np.random.default_rng(5)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    eq, alpha = rand_ext(rng, (n,), d), rand_ext(rng, (1,), d)
    st, ost = both(CONFIG2, ["t0", "t1", "t2"], ["alpha"])
    dev = [sa.Table.upload(t) for t in tables]
    s = sa.SumcheckSession(st, d, n, dev, eq=eq, constants=alpha)
    cur = tables
    for j in range(n):
        frm, middle = j + 1, j + 1 + (n - j - 1) // 2
        low, high = orc.eq_table(eq[frm:middle], d), orc.eq_table(eq[middle:], d)
        assert same(s.round(), orc.round_sums(ost, d, 3, cur, low, high, alpha)), f"round {j}"
        r = rand_ext(rng, (), d)
        s.fold(r)
        cur = [orc.fold_flat(t, r) for t in cur]
    finals, folded = s.finish()
    assert same(finals, [t[0] for t in cur])
    with pytest.raises(sa.InvalidParameter):
        sa.SumcheckSession(st, d, n, dev[:2], eq=eq, constants=alpha)
    # one session at a time: a second begin takes the scratch arenas, the first then refuses to go on
    first = sa.SumcheckSession(st, d, n, dev, eq=eq, constants=alpha)
    second = sa.SumcheckSession(st, d, n, dev, eq=eq, constants=alpha)
    with pytest.raises(sa.InvalidParameter):
        first.round()
    assert same(second.round(), orc.round_sums(ost, d, 3, tables, orc.eq_table(eq[1:1 + (n - 1) // 2], d),
                                               orc.eq_table(eq[1 + (n - 1) // 2:], d), alpha))
    for t in dev:
        t.free()


def test_linearity_and_fold_consistency_at_scale():
    """Size-independent properties at a size the oracle does not run: the config-2 statement's round
    sums are alpha * sums(t0 t1 t2) + 3 * sums(t1), and g(0), g(2), g(3) with g(1) from the claim lie on
    one cubic whose value at r is the next round's claim (the verifier's recurrence)."""
    n, d = 20, 4
    st = sa.Statement(CONFIG2, ["t0", "t1", "t2"], ["alpha"])
    prod = sa.Statement("(* t0 t1 t2)", ["t0", "t1", "t2"])
    lin = sa.Statement("(* 1 t1)", ["t0", "t1", "t2"])
    rng = np.random.default_rng(9)
    eq, alpha = rand_ext(rng, (n,), d), rand_ext(rng, (1,), d)
    dev = [sa.Table.random(900 + k, 1 << n) for k in range(3)]
    full = sa.SumcheckSession(st, d, n, dev, eq=eq, constants=alpha)
    a = full.round()
    b = sa.SumcheckSession(prod, d, n, dev, eq=eq).round()
    c = sa.SumcheckSession(lin, d, n, dev, eq=eq, degree=3).round()
    for k in range(3):
        assert same(a[k], orc.ext_add(orc.ext_mul(alpha[0], b[k]), orc.ext_scale(c[k], 3)))
    claim = sa.hypercube_sum(st, n, dev, d, eq=eq, constants=alpha)
    tr = sa.Transcript("scale", d)
    sa.prove(tr, n, st, dev, eq=eq, constants=alpha)
    vtr = sa.Transcript("scale", d, proof=tr.proof())
    _, reduced = sa.verify(vtr, n, st, claim, eq=eq, constants=alpha)
    finals = sa.prove(sa.Transcript("scale", d), n, st, dev, eq=eq, constants=alpha)[1]
    assert sa.check_final(reduced, st, finals, constants=alpha)
    for t in dev:
        t.free()


@pytest.mark.parametrize("n", [4, 11, 17])
def test_device_loop_entry_point_from_a_host_transcript_state(n):
    """exh_sumcheck_run: the host absorbs the header, hands over its hash state, and replays the messages (every
    round in one launch, slices and last launch, streaming rounds before them)."""
    d = 4
    rng = np.random.default_rng(6 + n)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    eq, alpha = rand_ext(rng, (n,), d), rand_ext(rng, (1,), d)
    st, ost = both(CONFIG2, ["t0", "t1", "t2"], ["alpha"])
    otr = orc.Transcript("run", d)
    rho, finals, _ = orc.prove(otr, n, ost, tables, eq=eq, constants=alpha)
    want = orc.decode_proof(otr.proof())
    dev = [sa.Table.upload(t) for t in tables]
    tr = sa.Transcript("run", d)
    tr.absorb(b"sc|" + n.to_bytes(2, "little") + (3).to_bytes(2, "little") + (1).to_bytes(4, "little"))
    s = sa.SumcheckSession(st, d, n, dev, eq=eq, constants=alpha)
    msgs, chal = s.run(tr, n)
    assert same(chal, rho)
    for j in range(n):
        assert same(msgs[j], want[j])
        tr.send(msgs[j])
        assert same(tr.challenge(), chal[j])
    got_finals, _ = s.finish()
    assert same(got_finals, finals) and tr.proof() == otr.proof()
    for t in dev:
        t.free()


@pytest.mark.parametrize("form,names,cnames,d,base,with_eq,n", [
    (CONFIG3, ["c0", "c1", "c2", "c3"], [], 8, True, True, 17),
    (CONFIG2, ["t0", "t1", "t2"], ["alpha"], 4, False, True, 18),
    ("(* t0 t1)", ["t0", "t1"], [], 8, False, False, 16),
    ("(+ (* t0 t1 t2) (* 7 t1) -1)", ["t0", "t1", "t2"], [], 4, True, True, 19),
    ("(* (+ (* 5 t0) (* -3 t1) 7) (- t2 (* 2 t0)))", ["t0", "t1", "t2"], [], 4, True, True, 16),
    (DOMAIN_FORM, DOMAIN_TABLES, DOMAIN_CONSTANTS, 8, True, True, 17),  # eight columns, six constants, interpreter
])
def test_rounds_on_a_grid_of_lds_resident_slices(form, names, cnames, d, base, with_eq, n):
    """Sizes at which the rounds between the large kernels and the last workgroup run as one launch of
    many workgroups (base and extension inputs, with and without a pending fold, interpreter and generated
    kernels): the proof bytes are the oracle's."""
    rng = np.random.default_rng(n * 100 + d)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) if base else rand_ext(rng, (1 << n,), d) for _ in names]
    eq = rand_ext(rng, (n,), d) if with_eq else None
    consts = rand_ext(rng, (len(cnames),), d) if cnames else None
    prove_both("slices", d, n, form, names, tables, eq=eq, constants=consts, cnames=cnames)


@pytest.mark.parametrize("form,names,cnames,d,n", [
    (CONFIG2, ["t0", "t1", "t2"], ["alpha"], 4, 3),
    (CONFIG2, ["t0", "t1", "t2"], ["alpha"], 4, 9),
    (CONFIG2, ["t0", "t1", "t2"], ["alpha"], 4, 14),
    (CONFIG3, ["c0", "c1", "c2", "c3"], [], 8, 4),
    (CONFIG3, ["c0", "c1", "c2", "c3"], [], 8, 11),
    ("(* t0 t1)", ["t0", "t1"], [], 4, 12),
    ("(* t0 t1)", ["t0", "t1"], [], 8, 7),
    ("(* t0 t1 t2)", ["t0", "t1", "t2"], [], 8, 10),
    # linear forms with coefficients other than +-1 (a generated kernel exists for this one, too)
    ("(* (+ (* 5 t0) (* -3 t1) 7) (- t2 (* 2 t0)))", ["t0", "t1", "t2"], [], 4, 9),
    ("(* (+ (* 5 t0) (* -3 t1) 7) (- t2 (* 2 t0)))", ["t0", "t1", "t2"], [], 4, 13),
])
def test_round_one_in_the_base_field_and_the_double_fold(form, names, cnames, d, n, monkeypatch):
    """With base tables and streaming rounds 1 and 2 (forced here at small n; the headline sizes take this path
    by themselves) rounds 0 and 1 are summed from base-field products on a grid of (X0, X1) and round 2 folds
    twice at once: same proof bytes, finals and folded tables as the oracle."""
    monkeypatch.setenv("EXACTA_HIP_MAX_SLICE_PAIRS", "0")
    rng = np.random.default_rng(n * 10 + d)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in names]
    eq = rand_ext(rng, (n,), d)
    consts = rand_ext(rng, (len(cnames),), d) if cnames else None
    st, _, proof, _ = prove_both("nodes", d, n, form, names, tables, eq=eq, constants=consts, cnames=cnames)
    assert st.has_generated_kernel(d)
    # and without the eq weights
    prove_both("nodes", d, n, form, names, tables, constants=consts, cnames=cnames)
    monkeypatch.setenv("EXACTA_HIP_NO_BASE_ROUND1", "1")
    tr = sa.Transcript("nodes", d)
    dev = [sa.Table.upload(t) for t in tables]
    sa.prove(tr, n, st, dev, eq=eq, constants=consts)
    assert tr.proof() == proof
    for t in dev:
        t.free()


@pytest.mark.parametrize("K,n,d,with_eq", [(2, 8, 4, True), (4, 10, 4, False), (2, 6, 8, True)])
def test_base_field_sweep_with_block_weights(K, n, d, with_eq, monkeypatch):
    """The same opening sweep when block weights are the HIGH factor (K a power of two, base tables)."""
    monkeypatch.setenv("EXACTA_HIP_MAX_SLICE_PAIRS", "0")
    rng = np.random.default_rng(K * 100 + n)
    tables = [rng.integers(0, P, K << n, dtype=np.uint32) for _ in range(3)]
    bw = rand_ext(rng, (K,), d)
    eq = rand_ext(rng, (n,), d) if with_eq else None
    consts = rand_ext(rng, (1,), d)
    prove_both("nodes-bw", d, n, CONFIG2, ["t0", "t1", "t2"], tables, eq=eq, constants=consts, cnames=["alpha"],
               block_weights=bw)


@pytest.mark.parametrize("form,names,cnames,d,n,base", [
    (CONFIG2, ["t0", "t1", "t2"], ["alpha"], 4, 8, True),
    (CONFIG2, ["t0", "t1", "t2"], ["alpha"], 4, 3, False),
    (CONFIG3, ["c0", "c1", "c2", "c3"], [], 8, 6, True),
    ("(* t0 t1)", ["t0", "t1"], [], 8, 1, False),
    ("(* t0 t1)", ["t0", "t1"], [], 4, 9, False),
])
def test_a_small_session_builds_its_weight_tables_in_its_one_launch(form, names, cnames, d, n, base, monkeypatch):
    """A proof whose every round fits the one-workgroup launch has no set-up launch: that launch forms the eq
    weights itself in LDS (the largest such sizes for each table count here, and one round).  Same bytes as the
    oracle, and as with the set-up launch (EXACTA_HIP_NO_OWN_WEIGHTS=1); the launches differ by that one."""
    rng = np.random.default_rng(n * 31 + d)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) if base else rand_ext(rng, (1 << n,), d) for _ in names]
    eq = rand_ext(rng, (n,), d)
    consts = rand_ext(rng, (len(cnames),), d) if cnames else None
    st, _, proof, _ = prove_both("own-weights", d, n, form, names, tables, eq=eq, constants=consts, cnames=cnames)
    dev = [sa.Table.upload(t) for t in tables]
    counts = []
    for off in ("0", "1"):
        monkeypatch.setenv("EXACTA_HIP_NO_OWN_WEIGHTS", off)
        tr = sa.Transcript("own-weights", d)
        names_of = launch_names(lambda: sa.prove(tr, n, st, dev, eq=eq, constants=consts))
        assert tr.proof() == proof
        counts.append(len(names_of))
    assert counts[1] == counts[0] + 1
    for t in dev:
        t.free()


@pytest.mark.parametrize("form,names,d,n,base,with_eq", [
    ("(* t0 t1 t2)", ["t0", "t1", "t2"], 4, 17, True, True),
    ("(* t0 t1)", ["t0", "t1"], 8, 12, False, True),
    ("(* t0 t1)", ["t0", "t1"], 4, 11, False, False),
])
def test_a_session_takes_its_constants_with_the_set_up_launch_or_by_a_copy(form, names, d, n, base, with_eq, monkeypatch):
    """The constants a session stages in pinned memory reach the device with its set-up launch (weight tables, or
    ones without an eq point), which reads them where they lie; EXACTA_HIP_COPY_CONSTANTS=1 sends them with a copy
    on the stream first.  Same bytes as the oracle either way."""
    rng = np.random.default_rng(n * 17 + d)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) if base else rand_ext(rng, (1 << n,), d) for _ in names]
    eq = rand_ext(rng, (n,), d) if with_eq else None
    st, _, proof, _ = prove_both("constants", d, n, form, names, tables, eq=eq)
    dev = [sa.Table.upload(t) for t in tables]
    for copy in ("0", "1"):
        monkeypatch.setenv("EXACTA_HIP_COPY_CONSTANTS", copy)
        tr = sa.Transcript("constants", d)
        sa.prove(tr, n, st, dev, eq=eq)
        assert tr.proof() == proof, copy
    for t in dev:
        t.free()


@pytest.mark.parametrize("points,n", [(2, 7), (2, 15), (3, 14), (4, 13), (4, 19)])
def test_point_reductions_of_an_opening(points, n):
    """REDUCE-POINTS' sumcheck (src/pcs.lisp:333-373): sum_z eq(z, x) g_z(x) over extension tables, no eq weights,
    wire degree 2, label "pcs-red" -- on the kernels generated for two to four points, from one workgroup's sizes
    to streaming rounds."""
    d = 4
    rng = np.random.default_rng(points * 100 + n)
    names = [v for i in range(points) for v in ("E%d" % i, "G%d" % i)]
    form = "(+ " + " ".join("(* E%d G%d)" % (i, i) for i in range(points)) + ")"
    tables = []
    for i in range(points):
        tables += [orc.eq_table(rand_ext(rng, (n,), d), d), rand_ext(rng, (1 << n,), d)]
    st, _, _, _ = prove_both("pcs-test", d, n, form, names, tables, degree=2, sc_label="pcs-red")
    assert st.has_generated_kernel(d)


@pytest.mark.parametrize("n", [6, 19])
def test_host_replay_of_the_device_transcript(n, monkeypatch):
    """By default the host transcript takes the device transcript's final hash state; with EXACTA_HIP_REPLAY=1 it
    absorbs the logged messages itself and must draw the same challenges.  Same proof bytes, and the transcript
    goes on identically afterwards, either way."""
    rng = np.random.default_rng(77 + n)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    eq, alpha = rand_ext(rng, (n,), 4), rand_ext(rng, (1,), 4)
    st = sa.Statement(CONFIG2, ["t0", "t1", "t2"], ["alpha"])
    dev = [sa.Table.upload(t) for t in tables]
    outs = []
    for replay in ("0", "1"):
        monkeypatch.setenv("EXACTA_HIP_REPLAY", replay)
        tr = sa.Transcript("replay", 4)
        chal, finals, _ = sa.prove(tr, n, st, dev, eq=eq, constants=alpha)
        outs.append((tr.proof(), chal.copy(), finals.copy(), tr.challenge().copy(), tr.state_digest()))
    assert outs[0][0] == outs[1][0] and outs[0][4] == outs[1][4]
    for a, b in zip(outs[0][1:4], outs[1][1:4]):
        assert same(a, b)
    otr = orc.Transcript("replay", 4)
    orc.prove(otr, n, orc.Statement(CONFIG2, ["t0", "t1", "t2"], ["alpha"]), tables, eq=eq, constants=alpha)
    assert same(otr.challenge(), outs[0][3])
    for t in dev:
        t.free()


def _wide():
    from sable_amd import workloads as wl
    cfg = wl.SUMCHECK["domain"]
    return cfg["form"], cfg["tables"], cfg["constants"]


@pytest.mark.timeout(600)
@pytest.mark.parametrize("d,n,base,with_eq,K", [(4, 6, True, True, 1), (4, 12, False, True, 1), (4, 9, True, False, 1),
                                                (4, 5, True, True, 3), (8, 7, True, True, 1), (4, 18, True, True, 1)])
def test_a_wide_statement_in_direct_form(d, n, base, with_eq, K):
    """A statement of 41 table monomials over 12 tables (the toy domain's, over seeded tables): too wide for
    accumulators per table group, so its kernels evaluate the written form itself at every wire point.  The honest
    claim (summed over the statement's parts) and the proof are the oracle's, on base and extension tables, with
    and without an eq point, with block weights, and at a size whose first rounds stream from memory; the same
    proof comes out when the statement is dealt into parts instead."""
    form, names, cnames = _wide()
    st, ost = both(form, names, cnames)
    rng = np.random.default_rng(4100 + d + n)
    size = K << n
    tables = [rng.integers(0, P, size, dtype=np.uint32) if base else rand_ext(rng, (size,), d) for _ in names]
    eq = rand_ext(rng, (n,), d) if with_eq else None
    cv = rand_ext(rng, (len(cnames),), d)
    bw = rand_ext(rng, (K,), d) if K > 1 else None
    dev = [sa.Table.upload(t) for t in tables]
    assert st.generate(d, wait=True)
    if K == 1:
        assert same(sa.hypercube_sum(st, n, dev, d, eq=eq, constants=cv), orc.hypercube_sum(ost, n, tables, d, eq=eq, constants=cv))
    tr, otr = sa.Transcript("wide", d), orc.Transcript("wide", d)
    out = {}
    names = launch_names(lambda: out.setdefault("got", sa.prove(tr, n, st, dev, eq=eq, constants=cv, block_weights=bw)))
    got = out["got"]
    want = orc.prove(otr, n, ost, tables, eq=eq, constants=cv, block_weights=bw)
    assert tr.proof() == otr.proof()
    assert same(got[0], want[0]) and same(got[1], want[1])
    # one session: the few rounds that stream, then the tables in LDS (in parts: a launch per part and round)
    assert len([name for name in names if name.startswith("round_")]) < n, names
    for t in dev:
        t.free()


def test_a_wide_statement_in_parts_when_the_direct_form_is_switched_off(monkeypatch):
    form, names, cnames = _wide()
    st, ost = both(form, names, cnames)
    rng = np.random.default_rng(4200)
    d, n = 4, 8
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in names]
    eq, cv = rand_ext(rng, (n,), d), rand_ext(rng, (len(cnames),), d)
    dev = [sa.Table.upload(t) for t in tables]
    monkeypatch.setenv("EXACTA_HIP_NO_DIRECT", "1")
    tr, otr = sa.Transcript("wide", d), orc.Transcript("wide", d)
    sa.prove(tr, n, st, dev, eq=eq, constants=cv)
    orc.prove(otr, n, ost, tables, eq=eq, constants=cv)
    assert tr.proof() == otr.proof()
    for t in dev:
        t.free()


@pytest.mark.parametrize("host_rounds", [False, True])
def test_many_blocks_keep_a_tile_within_a_block(host_rounds, monkeypatch):
    """Block weights over many small blocks: a streaming launch's tile stops growing at the span of one HIGH weight
    (a block), so the grid is larger than the resident cap and -- in host-driven rounds -- so is the table of
    partial rows."""
    if host_rounds:
        monkeypatch.setenv("EXACTA_HIP_HOST_ROUNDS", "1")
    K, n, d = 600, 10, 4
    rng = np.random.default_rng(77)
    tables = [rand_ext(rng, (K << n,), d) for _ in range(2)]
    bw = rand_ext(rng, (K,), d)
    prove_both("bw-many", d, n, "(* t0 t1)", ["t0", "t1"], tables, eq=rand_ext(rng, (n,), d), block_weights=bw,
               degree=2, sc_label="gkr")


WIDE_FORMS = [
    # five-term sums are no linear forms for the kernels (four terms at most), so the products are multiplied out:
    # 25 and 50 table monomials
    ("(* (+ t0 t1 t2 t3 t4) (- t5 t6 t7 t8 t9))", 10, []),
    ("(+ (* k0 (expt (+ t0 t1 t2 t3 t4) 2) (- t5)) (* 7 (+ t5 t6 t7 t8 t9) (+ t0 t2 t4 t6 t8)) (- k1 3))", 10, ["k0", "k1"]),
]


@pytest.mark.timeout(600)
@pytest.mark.parametrize("form,nt,cnames", WIDE_FORMS)
@pytest.mark.parametrize("d,n,mixed", [(4, 7, False), (4, 11, True)])
def test_wide_forms_of_other_shapes_in_direct_form(form, nt, cnames, d, n, mixed):
    """Powers, unary minus, integer factors, a table-free term, and base tables beside extension tables."""
    names = [f"t{i}" for i in range(nt)]
    st, ost = both(form, names, cnames)
    rng = np.random.default_rng(4300 + n + nt)
    tables = [rand_ext(rng, (1 << n,), d) if (mixed and i % 3 == 0) else rng.integers(0, P, 1 << n, dtype=np.uint32)
              for i in range(nt)]
    eq = rand_ext(rng, (n,), d)
    cv = rand_ext(rng, (len(cnames),), d) if cnames else None
    dev = [sa.Table.upload(t) for t in tables]
    assert st.generate(d, wait=True)
    assert same(sa.hypercube_sum(st, n, dev, d, eq=eq, constants=cv), orc.hypercube_sum(ost, n, tables, d, eq=eq, constants=cv))
    tr, otr = sa.Transcript("wide2", d), orc.Transcript("wide2", d)
    out = {}
    names_launched = launch_names(lambda: out.setdefault("got", sa.prove(tr, n, st, dev, eq=eq, constants=cv)))
    want = orc.prove(otr, n, ost, tables, eq=eq, constants=cv)
    assert tr.proof() == otr.proof()
    assert same(out["got"][0], want[0]) and same(out["got"][1], want[1])
    assert len([name for name in names_launched if name.startswith("round_")]) < n, names_launched
    for t in dev:
        t.free()
