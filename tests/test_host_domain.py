"""The shipped library's domain layer on the CPU (sable_amd/domain.py over the C ABI's host entry points): its
statement, tables and degrees agree with the oracle's, and its verifier accepts the oracle prover's domain proofs
with the oracle verifier's claims and roots and rejects what the oracle rejects (tests/tests.lisp:523-575's pattern).
The prover needs an MI355X and is tested under -m gpu."""
import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc
from oracle import domain as od
from sable_amd import domain as sd
from test_oracle_domain import CASES, lookup_challenges, proof_of, toy_domain

P = orc.P


def mirror(dom):
    """The oracle's domain as the product's, without data (a verifier's view)."""
    text = lambda f: None if f is None else to_text(f)
    cols = [sd.Column(c.name, c.kind, c.c, c.shared) for c in dom.columns]
    return sd.Domain(dom.name, dom.n, cols, blocks=dom.blocks, merge=dom.merge,
                     constraints=[to_text(f) for f in dom.constraints],
                     lookups=[{"tag": to_text(l["tag"]), "values": [to_text(v) for v in l["values"]], "num": text(l["num"])}
                              for l in dom.lookups])


def to_text(form):
    return "(%s)" % " ".join([form[0]] + [to_text(a) for a in form[1:]]) if isinstance(form, list) else str(form)


def same_claims(xs, ys):
    return len(xs) == len(ys) and all(a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
                                      for a, b in zip(xs, ys))


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join("%s%s" % kv for kv in c.items()))
def test_statement_tables_and_degrees_agree_with_the_oracle(case):
    dom = toy_domain(**case)
    mine = mirror(dom)
    assert [t[0] for t in sd.domain_tables(mine)] == [t[0] for t in od.domain_tables(dom)]
    assert [(t[3], t[4]) for t in sd.domain_tables(mine)] == [(t[3], t[4]) for t in od.domain_tables(dom)]
    assert sd.domain_constant_names(mine) == od.domain_constant_names(dom)
    assert sd.domain_degree(mine) == od.domain_degree(dom)
    assert sd.domain_degree(mine, block_phase=True) == od.domain_degree(dom, block_phase=True)
    tables, names = [t[0] for t in od.domain_tables(dom)], od.domain_constant_names(dom)
    theirs = orc.Statement(od.domain_statement(dom), tables, names)
    ours = sa.Statement(sd.domain_statement(mine), tables, names)
    rng = np.random.default_rng(3)
    for d in (4, 8):
        tv = rng.integers(0, P, (len(tables), d), dtype=np.uint64).astype(np.uint32)
        cv = rng.integers(0, P, (len(names), d), dtype=np.uint64).astype(np.uint32)
        assert np.array_equal(sd.evaluate(ours, tv, cv, d), theirs.evaluate(tv, cv, d))


@pytest.mark.parametrize("d", [4, 8])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join("%s%s" % kv for kv in c.items()))
def test_verifier_accepts_the_oracle_provers_proofs(case, d):
    dom = toy_domain(seed=d + case["n"] + case["k"], **case)
    z, betas = lookup_challenges(d, case["n"])
    proof, proved = proof_of(dom, d, z, betas)
    want_claims, want_roots = od.verify_domain(orc.Transcript("dom-test", d, proof=proof), dom, z, betas)
    tr = sa.Transcript("dom-test", d, proof=proof)
    claims, roots = sd.verify_domain(tr, mirror(dom), z, betas)
    assert tr.finished() and same_claims(claims, want_claims) and same_claims(claims, proved)
    assert np.array_equal(roots, want_roots)


@pytest.mark.parametrize("merge", [False, True])
def test_verifier_rejects(merge):
    d = 4
    dom = toy_domain(merge=merge, seed=3, broken=True)
    z, betas = lookup_challenges(d, 3)
    with pytest.raises(sa.VerificationFailure):
        sd.verify_domain(sa.Transcript("dom-test", d, proof=proof_of(dom, d, z, betas)[0]), mirror(dom), z, betas)
    dom = toy_domain(merge=merge, seed=4)
    mine = mirror(dom)
    z, betas = lookup_challenges(d, 4)
    msgs = orc.decode_proof(proof_of(dom, d, z, betas)[0])
    for i in range(len(msgs)):
        forged = [x.copy() for x in msgs]
        forged[i].reshape(-1)[0] = (int(forged[i].reshape(-1)[0]) + 1) % P
        with pytest.raises(sa.VerificationFailure):
            sd.verify_domain(sa.Transcript("dom-test", d, proof=orc.encode_messages(forged)), mine, z, betas)
