"""The oracle's threaded straight-line path (oracle/orc_fast.c) against its plain restatement, which the
reference's golden proofs pin: the same proof bytes, round sums and folded tables on every shape, and the
unrolled tower products against the loops of src/field.lisp:213-234 including the extreme residues."""
import itertools

import numpy as np
import pytest

from oracle import binding as orc

P = orc.P
CONFIG2 = ("(+ (* alpha t0 t1 t2) (* 3 t1))", ["t0", "t1", "t2"], ["alpha"])
CONFIG3 = ("(* (+ c0 3) (- c1 c0) c2 c3)", ["c0", "c1", "c2", "c3"], [])
GKR = ("(+ (* a p0 q1) (* a p1 q0) (* al q0 q1))", ["p0", "p1", "q0", "q1"], ["a", "al"])
ODD = ("(- (* (expt t0 3) (- t1)) (* (+ t1 2 t0) 5 k) (+))", ["t0", "t1"], ["k"])


@pytest.fixture(autouse=True)
def plain_again():
    yield
    orc.set_fast(0)


def test_unrolled_products_match_the_loops():
    rng = np.random.default_rng(5)
    edge = [0, 1, 2, P - 1, P - 2, (P - 1) // 2, (P + 1) // 2]
    for d in (4, 8):
        cases = [rng.integers(0, P, (2, d), dtype=np.uint32) for _ in range(200)]
        cases += [np.array([[x] * d, [y] * d], np.uint32) for x, y in itertools.product(edge, edge)]
        cases += [np.array([np.roll([P - 1] + [0] * (d - 1), i), np.roll([P - 1] + [0] * (d - 1), j)], np.uint32)
                  for i in range(d) for j in range(d)]
        for a, b in cases:
            assert np.array_equal(orc.ext_mul(a, b), orc.ext_mul_plain(a, b))


def test_golden_products_through_the_unrolled_code(vectors):
    for v in vectors("ext"):
        a, b = np.array(v["a"], np.uint32), np.array(v["b"], np.uint32)
        assert np.array_equal(orc.ext_mul(a, b), np.array(v["mul"], np.uint32))


def test_golden_proofs_on_the_fast_path(vectors):
    """tests.lisp:277-282 once more, with the threaded path switched on: the bytes of the original prover."""
    for threads in (1, 3):
        orc.set_fast(threads)
        for v in vectors("sumcheck"):
            d, n, nt = v["d"], v["n"], len(v["tables"])
            names = [f"t{i}" for i in range(nt)]
            st = orc.Statement("(* " + " ".join(names) + ")", names)
            tables = [np.array(t, np.uint32) for t in v["tables"]]
            eq = np.array(v["eq_r"], np.uint32) if v["eq_r"] else None
            tr = orc.Transcript("sc-vec", d)
            rho, finals, _ = orc.prove(tr, n, st, tables, eq=eq)
            assert np.array_equal(rho, np.array(v["rho"], np.uint32))
            assert tr.proof()[8:] == bytes.fromhex(v["proof"])[8:]


def prove_bytes(form, names, cnames, d, n, base, with_eq, seed, k=None):
    rng = np.random.default_rng(seed)
    blocks = k or 1
    shape = (blocks << n,) if base else (blocks << n, d)
    tables = [rng.integers(0, P, shape, dtype=np.uint32) for _ in names]
    eq = rng.integers(0, P, (n, d), dtype=np.uint32) if with_eq else None
    cv = rng.integers(0, P, (len(cnames), d), dtype=np.uint32) if cnames else None
    bw = rng.integers(0, P, (k, d), dtype=np.uint32) if k else None
    st = orc.Statement(form, names, cnames)
    tr = orc.Transcript("fast", d)
    chal, finals, folded = orc.prove(tr, n, st, tables, eq=eq, constants=cv, block_weights=bw)
    return tr.proof(), chal, finals, folded


@pytest.mark.parametrize("stmt", [CONFIG2, CONFIG3, GKR, ODD], ids=["config2", "config3", "gkr", "odd"])
@pytest.mark.parametrize("d", [4, 8])
@pytest.mark.parametrize("base,with_eq,k", [(True, True, None), (False, True, None), (True, False, None),
                                            (False, True, 3), (False, False, 2)])
def test_same_proof_as_the_plain_path(stmt, d, base, with_eq, k):
    form, names, cnames = stmt
    for n in (0, 1, 4, 9):
        orc.set_fast(0)
        want = prove_bytes(form, names, cnames, d, n, base, with_eq, 100 * n + d, k)
        for threads in (1, 5):
            orc.set_fast(threads)
            got = prove_bytes(form, names, cnames, d, n, base, with_eq, 100 * n + d, k)
            assert got[0] == want[0], (n, threads)
            assert np.array_equal(got[1], want[1]) and np.array_equal(got[2], want[2])
            for a, b in zip(got[3], want[3]):
                assert np.array_equal(a, b)


def test_written_form_and_monomials_agree_on_a_round():
    """The postfix program of the form as written and the canonical monomials are the same polynomial: one
    round's sums from each, with extreme values in the tables (all p - 1, all 0)."""
    d, points = 4, 4
    form, names, _ = CONFIG3
    st = orc.Statement(form, names)
    rng = np.random.default_rng(7)
    low, high = rng.integers(0, P, (8, d), dtype=np.uint32), rng.integers(0, P, (4, d), dtype=np.uint32)
    for fill in ("random", "max", "zero"):
        if fill == "random":
            tables = [rng.integers(0, P, 64, dtype=np.uint32) for _ in names]
        else:
            tables = [np.full(64, P - 1 if fill == "max" else 0, np.uint32) for _ in names]
        want = orc.round_sums(st, d, points, tables, low, high)
        assert np.array_equal(orc.round_sums_fast(st, d, points, tables, low, high, threads=2), want)
        lifted = [np.concatenate([t[:, None], np.zeros((64, d - 1), np.uint32)], axis=1) for t in tables]
        assert np.array_equal(orc.round_sums_fast(st, d, points, lifted, low, high, threads=3), want)


def test_splitmix_field_known_answers():
    """SplitMix64's published first outputs for seed 0 (0xe220a8397b1dcdaf, 0x6e789e6aa1b965f4,
    0x06c45d188009454f, ...), top 31 bits each, kept when below p."""
    outs = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F, 0xF88BB8A8724C81EC]
    want = [w >> 33 for w in outs if (w >> 33) < P]
    got = orc.splitmix_field(0, len(want))
    assert list(got) == want
    big = orc.splitmix_field(12345, 1 << 16)
    assert big.max() < P and len(np.unique(big)) > 65000
