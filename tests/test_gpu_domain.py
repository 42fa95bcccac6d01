"""The domain layer on the device (sable_amd/domain.py over exh_domain_leaves, exh_domain_table, exh_gkr_prove_upper
and exh_prove) against the oracle's (oracle/domain.py, after src/domain.lisp): leaves, tables and whole proofs byte
for byte on seeded domains, the verifier's acceptance and claims, and every perturbed message rejected
(tests/tests.lisp:523-575's pattern)."""
import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc
from oracle import domain as od
from sable_amd import domain as sd
from conftest import launch_names
from test_oracle_domain import CASES as ORACLE_CASES, lookup_challenges, toy_domain

pytestmark = pytest.mark.gpu
P = orc.P


def both(name, n, k, columns, constraints, lookups, merge=False):
    """The same domain for the oracle and for the device: columns as (name, kind, c, shared, data)."""
    theirs = od.Domain(name, n, [od.Column(*c) for c in columns], blocks=k, merge=merge, constraints=constraints,
                       lookups=lookups)
    mine = sd.Domain(name, n, [sd.Column(*c) for c in columns], blocks=k, merge=merge, constraints=constraints,
                     lookups=lookups)
    return theirs, mine


def products(n, k, seed, lookups=True, constraints=True, merge=False):
    """Bits A, values B and the products C = A B, one lookup of the pairs (a, b) and two constraints: the statement
    that has a kernel generated at build time for D = 4."""
    rng = np.random.default_rng(seed)
    a = rng.integers(0, 2, k << n, dtype=np.uint64)
    b = rng.integers(0, P, k << n, dtype=np.uint64)
    cols = [("a", "full", 0, False, a), ("b", "full", 0, False, b), ("c", "full", 0, False, a * b % P)]
    return both("7.products", n, k, cols, ["(* a (- a 1))", "(- c (* a b))"] if constraints else [],
                [{"tag": 5, "values": ["a", "b"]}] if lookups else [], merge)


def short(n, k, seed, merge=False):
    """One lookup of A alone and the product constraint: with the block weight in front (merged blocks) it still
    fits the round kernels' sixteen table monomials."""
    rng = np.random.default_rng(seed)
    a = rng.integers(0, 2, k << n, dtype=np.uint64)
    b = rng.integers(0, P, k << n, dtype=np.uint64)
    cols = [("a", "full", 0, False, a), ("b", "full", 0, False, b), ("c", "full", 0, False, a * b % P)]
    return both("7.short", n, k, cols, ["(- c (* a b))"], [{"tag": 5, "values": ["a"]}], merge)


def kinds(n, k, seed, merge=False, constraints=("(* s (- s 1))", "(- c (* a kb))")):
    """Every kind of column: full A and C = A KB, the per-block constant KB (:ROW n), W (:COL 2), the shared mask S
    (:COL n), a lookup with a numerator."""
    rng = np.random.default_rng(seed)
    a = rng.integers(0, P, k << n, dtype=np.uint64)
    kb = rng.integers(0, P, k, dtype=np.uint64)
    w = rng.integers(0, P, 4 * k, dtype=np.uint64)
    s = rng.integers(0, 2, 1 << n, dtype=np.uint64)
    c = a * np.repeat(kb, 1 << n) % P
    cols = [("a", "full", 0, False, a), ("c", "full", 0, False, c), ("kb", "row", n, False, kb),
            ("w", "col", 2, False, w), ("s", "col", n, True, s)]
    return both("3.kinds|3.more", n, k, cols, list(constraints),
                [{"tag": 7, "values": ["w"], "num": "(+ s 2)"}], merge)


def same_claims(xs, ys):
    return len(xs) == len(ys) and all(a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
                                      for a, b in zip(xs, ys))


def device_toy(dom):
    return sd.Domain(dom.name, dom.n, [sd.Column(c.name, c.kind, c.c, c.shared, c.data) for c in dom.columns],
                     blocks=dom.blocks, merge=dom.merge,
                     constraints=["(* a (- a 1))", "(- c (* a b))", "(* s (- s 1) m)"] if dom.constraints else [],
                     lookups=[{"tag": 5, "values": ["a", "b"]}, {"tag": 7, "values": ["c", "m", "w"], "num": "(+ s 2)"},
                              {"tag": 9, "values": ["kb"]}] if dom.lookups else [])


@pytest.mark.parametrize("d", [4, 8])
@pytest.mark.parametrize("n,k", [(4, 3), (2, 1), (9, 2)])
def test_leaves_and_tables_of_the_toy_domain(n, k, d):
    """domain-leaves and table-values of the reference's toy domain (every kind of column, three lookups)."""
    theirs = toy_domain(n=n, k=k, seed=n + k)
    mine = device_toy(theirs)
    z, betas = lookup_challenges(d, n)
    for (p, q), (wp, wq) in zip(sd.domain_leaves(mine, z, betas), od.domain_leaves(theirs, z, betas)):
        assert np.array_equal(p.download(), wp) and np.array_equal(q.download(), wq)
    for mt, tt in zip(sd.domain_tables(mine), od.domain_tables(theirs)):
        assert mt[0] == tt[0] and np.array_equal(sd.table_values(mt, k, n).download(), od.table_values(tt, k, n))


CASES = [("products", dict(n=6, k=1, seed=1)), ("products", dict(n=8, k=3, seed=2)), ("products", dict(n=12, k=2, seed=3)),
         ("products", dict(n=16, k=1, seed=4)), ("products", dict(n=5, k=4, seed=5, merge=True, lookups=False)),
         ("products", dict(n=4, k=3, seed=6, merge=True, constraints=False)), ("products", dict(n=3, k=1, seed=7, merge=True)),
         ("short", dict(n=6, k=5, seed=15, merge=True)), ("short", dict(n=9, k=2, seed=16)),
         ("products", dict(n=7, k=2, seed=8, lookups=False)), ("products", dict(n=7, k=2, seed=9, constraints=False)),
         ("products", dict(n=2, k=1, seed=10)), ("kinds", dict(n=6, k=3, seed=11)), ("kinds", dict(n=10, k=1, seed=12)),
         ("kinds", dict(n=5, k=5, seed=13, merge=True, constraints=("(- c (* a kb))",))), ("kinds", dict(n=2, k=2, seed=14))]


@pytest.mark.parametrize("d", [4, 8])
@pytest.mark.parametrize("maker,kw", CASES, ids=lambda v: v if isinstance(v, str) else "-".join("%s%s" % i for i in v.items()))
def test_proof_bytes_are_the_oracles(maker, kw, d):
    theirs, mine = globals()[maker](**kw)
    z, betas = lookup_challenges(d, kw["seed"])
    otr = orc.Transcript("dom-test", d)
    want_claims = od.prove_domain(otr, theirs, z, betas)
    tr = sa.Transcript("dom-test", d)
    claims = sd.prove_domain(tr, mine, z, betas)
    assert tr.proof() == otr.proof()
    assert same_claims(claims, want_claims)
    vtr = sa.Transcript("dom-test", d, proof=tr.proof())
    got, roots = sd.verify_domain(vtr, mine, z, betas)
    assert vtr.finished() and same_claims(got, claims)
    # a full column's claim is its multilinear extension at the claimed point (unmerged: per block)
    if not theirs.merge:
        n = theirs.n
        for (name, point, value), col in zip(claims, theirs.columns):
            if col.kind == "full":
                for b in range(theirs.blocks):
                    assert np.array_equal(value[b], orc.mle_eval(col.data[b << n:(b + 1) << n].astype(np.uint32), point, d))


def test_the_products_statement_runs_on_its_generated_kernel():
    _, mine = products(6, 1, 1)
    assert sd._compiled(mine).has_generated_kernel(4)


@pytest.mark.parametrize("merge", [False, True])
def test_rejects(merge):
    d = 4
    # a constraint that does not hold
    maker = short if merge else products
    theirs, mine = maker(5, 3, 21, merge=merge)
    broken = theirs.columns[2].data.copy()
    broken[1] = (broken[1] + 1) % P
    mine.columns[2] = sd.Column("c", data=broken)
    z, betas = lookup_challenges(d, 21)
    tr = sa.Transcript("dom-test", d)
    sd.prove_domain(tr, mine, z, betas)
    with pytest.raises(sa.VerificationFailure):
        sd.verify_domain(sa.Transcript("dom-test", d, proof=tr.proof()), mine, z, betas)
    # any changed value
    theirs, mine = maker(5, 3, 22, merge=merge)
    z, betas = lookup_challenges(d, 22)
    tr = sa.Transcript("dom-test", d)
    sd.prove_domain(tr, mine, z, betas)
    msgs = orc.decode_proof(tr.proof())
    assert len(msgs) > 20
    for i in range(len(msgs)):
        forged = [x.copy() for x in msgs]
        forged[i].reshape(-1)[0] = (int(forged[i].reshape(-1)[0]) + 1) % P
        with pytest.raises(sa.VerificationFailure):
            sd.verify_domain(sa.Transcript("dom-test", d, proof=orc.encode_messages(forged)), mine, z, betas)


@pytest.mark.parametrize("d", [4, 8])
@pytest.mark.parametrize("case", ORACLE_CASES, ids=lambda c: "-".join("%s%s" % kv for kv in c.items()))
def test_the_toy_domain_in_parts(case, d):
    """The reference's toy domain (tests/tests.lisp:487-512: every kind of column, three lookups, three
    constraints) in every shape its round-trip test takes.  Its statement expands to 41 table monomials, more than
    one kernel holds: the prover deals them into parts proved in step, and the bytes are the oracle's."""
    theirs = toy_domain(seed=d + case["n"] + case["k"], **case)
    mine = device_toy(theirs)
    z, betas = lookup_challenges(d, case["n"])
    otr = orc.Transcript("dom-test", d)
    want_claims = od.prove_domain(otr, theirs, z, betas)
    tr = sa.Transcript("dom-test", d)
    claims = sd.prove_domain(tr, mine, z, betas)
    assert tr.proof() == otr.proof() and same_claims(claims, want_claims)
    vtr = sa.Transcript("dom-test", d, proof=tr.proof())
    got, _ = sd.verify_domain(vtr, mine, z, betas)
    assert vtr.finished() and same_claims(got, claims)


def test_a_wide_statement_at_size():
    """The toy domain at n = 14 with three blocks (tables of 3 * 2^13 entries, 41 monomials in three parts)."""
    d = 4
    theirs = toy_domain(n=14, k=3, seed=77)
    mine = device_toy(theirs)
    z, betas = lookup_challenges(d, 77)
    otr = orc.Transcript("dom-test", d)
    od.prove_domain(otr, theirs, z, betas)
    tr = sa.Transcript("dom-test", d)
    sd.prove_domain(tr, mine, z, betas)
    assert tr.proof() == otr.proof()


@pytest.mark.timeout(600)
@pytest.mark.parametrize("d,n,k", [(4, 7, 2), (4, 13, 1), (8, 5, 3)])
def test_the_toy_domain_in_direct_form(d, n, k):
    """The same wide statement once its direct-form kernels are there (exh_stmt_generate compiles them: the
    written form evaluated per pair at every wire point, one accumulator per point): one device-driven session
    instead of parts proved in step, and the same bytes as the oracle's."""
    theirs = toy_domain(n=n, k=k, seed=300 + d + n)
    mine = device_toy(theirs)
    z, betas = lookup_challenges(d, n)
    otr = orc.Transcript("dom-test", d)
    want_claims = od.prove_domain(otr, theirs, z, betas)
    st = sd._compiled(mine)
    assert st.generate(d, degree=sd.domain_degree(mine), wait=True)
    tr = sa.Transcript("dom-test", d)
    out = {}
    names = launch_names(lambda: out.setdefault("claims", sd.prove_domain(tr, mine, z, betas)))
    assert tr.proof() == otr.proof() and same_claims(out["claims"], want_claims)
    # with one block everything around the zerocheck is chained on the device, so the streaming round launches
    # (named round_...) are the zerocheck's: in parts there is one per part and round, in one device-driven loop
    # only the first few rounds stream before the tables fit the workgroups' LDS
    if k == 1:
        assert len([name for name in names if name.startswith("round_")]) < n, names
    vtr = sa.Transcript("dom-test", d, proof=tr.proof())
    got, _ = sd.verify_domain(vtr, mine, z, betas)
    assert vtr.finished() and same_claims(got, out["claims"])
