"""The oracle's domain layer (oracle/domain.py, after src/domain.lisp).  Its bytes are pinned by the reference's frozen
domain cases (tests/test_oracle_frozen_cases.py); these tests hold it to what the protocol fixes, following
tests/tests.lisp:485-575: the toy domain with every kind of column, the verifier accepting the prover's proof with
the same claims, a full column's claim being its multilinear extension at the claimed point, the roots being the
sums of the leaf fractions, a broken constraint rejected and every perturbed message rejected."""
import numpy as np
import pytest

from oracle import binding as orc
from oracle import domain as od
from oracle import forms

P = orc.P


def toy_domain(n=3, k=3, merge=False, lookups=True, constraints=True, seed=5, broken=False):
    """tests.lisp:487-512: bits A, B, C = A B, a :ROW 1 shared column M, a :COL n shared mask S, a per-block
    constant KB (:ROW n), a :COL 2 column W."""
    rng = np.random.default_rng(seed)
    size = 1 << n
    a = rng.integers(0, 2, k * size, dtype=np.uint64)
    b = rng.integers(0, P, k * size, dtype=np.uint64)
    c = a * b % P
    m = rng.integers(0, P, size // 2, dtype=np.uint64)
    s = rng.integers(0, 2, size, dtype=np.uint64)
    kb = rng.integers(0, P, k, dtype=np.uint64)
    w = rng.integers(0, P, k * 4, dtype=np.uint64)
    if broken:
        c[1] = (c[1] + 1) % P
    cols = [od.Column("a", data=a), od.Column("b", data=b), od.Column("c", data=c),
            od.Column("m", "row", 1, True, m), od.Column("s", "col", n, True, s), od.Column("kb", "row", n, False, kb),
            od.Column("w", "col", 2, False, w)]
    return od.Domain("12.toy-merged" if merge else "12.toy", n, cols, blocks=k, merge=merge,
                     constraints=["(* a (- a 1))", "(- c (* a b))", "(* s (- s 1) m)"] if constraints else [],
                     lookups=[{"tag": 5, "values": ["a", "b"]}, {"tag": 7, "values": ["c", "m", "w"], "num": "(+ s 2)"},
                              {"tag": 9, "values": ["kb"]}] if lookups else [])


def lookup_challenges(d, seed):
    rng = np.random.default_rng(1000 + seed)
    return rng.integers(0, P, d, dtype=np.uint64).astype(np.uint32), rng.integers(0, P, (8, d), dtype=np.uint64).astype(np.uint32)


def proof_of(dom, d, z, betas):
    tr = orc.Transcript("dom-test", d)
    claims = od.prove_domain(tr, dom, z, betas)
    return tr.proof(), claims


def same_claims(xs, ys):
    return len(xs) == len(ys) and all(a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
                                      for a, b in zip(xs, ys))


CASES = [dict(n=3, k=3), dict(n=2, k=1), dict(n=3, k=3, merge=True), dict(n=4, k=4, merge=True),
         dict(n=3, k=2, lookups=False), dict(n=3, k=2, constraints=False), dict(n=2, k=1, merge=True),
         dict(n=4, k=5, merge=True), dict(n=3, k=5)]


@pytest.mark.parametrize("d", [4, 8])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join("%s%s" % kv for kv in c.items()))
def test_roundtrip(case, d):
    dom = toy_domain(seed=d + case["n"] + case["k"], **case)
    z, betas = lookup_challenges(d, case["n"])
    proof, proved = proof_of(dom, d, z, betas)
    tr = orc.Transcript("dom-test", d, proof=proof)
    claims, roots = od.verify_domain(tr, dom, z, betas)
    assert tr.finished() and same_claims(claims, proved)
    n, k = dom.n, dom.blocks
    for (name, point, value), col in zip(claims, dom.columns):
        if col.kind != "full":
            continue
        blocks = [orc.mle_eval(col.data[b << n:(b + 1) << n].astype(np.uint32), point[:n], d) for b in range(k)]
        if dom.merge:
            weights = orc.eq_table(point[n:], d) if k > 1 else [orc.base_to_ext(1, d)]
            want = np.zeros(d, np.uint32)
            for b in range(k):
                want = orc.ext_add(want, orc.ext_mul(weights[b], blocks[b]))
            assert np.array_equal(value, want)
        else:
            assert np.array_equal(value, np.array(blocks))
    # each lookup's root is the sum of its leaves' fractions p / q over all blocks
    for (p, q), root in zip(od.domain_leaves(dom, z, betas), roots):
        total = np.zeros(d, np.uint32)
        for pi, qi in zip(p, q):
            total = orc.ext_add(total, orc.ext_mul(pi, orc.ext_inv(qi)))
        assert np.array_equal(orc.ext_mul(total, root[1]), root[0])


def test_claims_of_the_other_column_kinds():
    """A :ROW c column's claim is the multilinear extension of its data over the variables from c on, a :COL c
    column's over the variables below c (src/domain.lisp:182-212)."""
    d, dom = 4, toy_domain(n=4, k=2, seed=11)
    z, betas = lookup_challenges(d, 11)
    _, claims = proof_of(dom, d, z, betas)
    by_name = {name: (point, value) for name, point, value in claims}
    n, k = dom.n, dom.blocks
    cols = {c.name: c for c in dom.columns}
    point, value = by_name["M"]  # :ROW 1 shared: 2^(n-1) values over variables 1..n-1
    assert len(point) == n - 1 and np.array_equal(value[0], orc.mle_eval(cols["M"].data.astype(np.uint32), point, d))
    point, value = by_name["S"]  # :COL n shared: all n variables
    assert len(point) == n and np.array_equal(value[0], orc.mle_eval(cols["S"].data.astype(np.uint32), point, d))
    point, value = by_name["KB"]  # :ROW n: one value per block, no point
    assert len(point) == 0 and np.array_equal(value[:, 0], cols["KB"].data.astype(np.uint32)) and not value[:, 1:].any()
    point, value = by_name["W"]  # :COL 2: four values per block over the first two variables
    assert len(point) == 2
    for b in range(k):
        assert np.array_equal(value[b], orc.mle_eval(cols["W"].data[4 * b:4 * b + 4].astype(np.uint32), point, d))


def test_statement_is_the_documented_sum():
    """domain-statement's value at random table and constant values against the formula of its doc string
    (src/domain.lisp:95-100), computed term by term with the field routines alone."""
    d, dom = 4, toy_domain(n=3, k=1, seed=2)
    tables = [t[0] for t in od.domain_tables(dom)]
    names = od.domain_constant_names(dom)
    st = orc.Statement(od.domain_statement(dom), tables, names)
    rng = np.random.default_rng(9)
    tv = rng.integers(0, P, (len(tables), d), dtype=np.uint64).astype(np.uint32)
    cv = rng.integers(0, P, (len(names), d), dtype=np.uint64).astype(np.uint32)
    T, Cn = dict(zip(tables, tv)), dict(zip(names, cv))
    one = orc.base_to_ext(1, d)

    def ext_form(form, half):
        """A column form at the half's tables, over the extension field."""
        if isinstance(form, int):
            return orc.base_to_ext(form % P, d)
        if isinstance(form, str):
            return T[form + "@%d" % half] if form + "@%d" % half in T else T[form]
        vals = [ext_form(a, half) for a in form[1:]]
        out = vals[0]
        for v in vals[1:]:
            out = {"+": orc.ext_add, "-": orc.ext_sub, "*": orc.ext_mul}[form[0]](out, v)
        return out

    def q(lookup, half):
        out = orc.ext_sub(Cn["%Z"], ext_form(lookup["tag"], half))
        for i, v in enumerate(lookup["values"]):
            out = orc.ext_sub(out, orc.ext_mul(Cn["%%BETA%d" % i], ext_form(v, half)))
        return out

    want = np.zeros(d, np.uint32)
    for l, lookup in enumerate(dom.lookups):
        n0, n1 = (ext_form(lookup["num"], 0), ext_form(lookup["num"], 1)) if lookup["num"] is not None else (one, one)
        q0, q1 = q(lookup, 0), q(lookup, 1)
        want = orc.ext_add(want, orc.ext_mul(Cn["%%A%d" % l], orc.ext_add(orc.ext_mul(n0, q1), orc.ext_mul(n1, q0))))
        want = orc.ext_add(want, orc.ext_mul(Cn["%%AL%d" % l], orc.ext_mul(q0, q1)))
    for i, con in enumerate(dom.constraints):
        want = orc.ext_add(want, orc.ext_mul(Cn["%%GAM%d" % i], ext_form(con, 0)))
        want = orc.ext_add(want, orc.ext_mul(Cn["%%GETA%d" % i], ext_form(con, 1)))
    assert np.array_equal(st.evaluate(tv, cv, d), want)


def test_degrees_and_tables_of_the_toy_domain():
    dom = toy_domain(n=3, k=3)
    assert [t[0] for t in od.domain_tables(dom)] == ["A@0", "A@1", "B@0", "B@1", "C@0", "C@1", "M@0", "M@1", "S@0", "S@1",
                                                      "KB", "W"]
    # q of lookup 1 has pieces of degree 1; its numerator S + 2 adds 1; the constraint S (S - 1) M has degree 3
    assert od.domain_degree(dom) == 3
    # in the block sumcheck the shared M and S do not vary: A (A - 1), C - A B give 2, plus 1 for the block weight
    assert od.domain_degree(dom, block_phase=True) == 3
    assert od.domain_degree(toy_domain(n=3, k=3, constraints=False)) == 2
    assert od.label_name("12.toy") == "toy" and od.label_name("3.oproj|3.rqo") == "oproj|rqo" and od.label_name("x.y") == "x.y"
    assert forms.form_degree(od.domain_statement(dom), {t[0] for t in od.domain_tables(dom)}) == 3


@pytest.mark.parametrize("merge", [False, True])
def test_rejects(merge):
    d = 4
    dom = toy_domain(merge=merge, seed=3, broken=True)
    z, betas = lookup_challenges(d, 3)
    with pytest.raises(orc.VerificationFailure):
        od.verify_domain(orc.Transcript("dom-test", d, proof=proof_of(dom, d, z, betas)[0]), dom, z, betas)
    dom = toy_domain(merge=merge, seed=4)
    z, betas = lookup_challenges(d, 4)
    msgs = orc.decode_proof(proof_of(dom, d, z, betas)[0])
    assert len(msgs) > 20
    for i, m in enumerate(msgs):
        forged = [x.copy() for x in msgs]
        forged[i].reshape(-1)[0] = (int(forged[i].reshape(-1)[0]) + 1) % P
        with pytest.raises(orc.VerificationFailure):
            od.verify_domain(orc.Transcript("dom-test", d, proof=orc.encode_messages(forged)), dom, z, betas)
