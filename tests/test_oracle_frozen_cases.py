"""The oracle against the reference's frozen cases (tests/tests.lisp:902-925): the SHA-256 of the case files that
EXPORT-GKR-CASES, EXPORT-DOMAIN-CASES and EXPORT-PCS-CASES write -- eight PROVE-UPPER proofs (one block and
several, one to three lookups, F_p^4 and F_p^8), sixteen PROVE-DOMAIN proofs (every kind of column, merged blocks,
with and without lookups and constraints) with the verifiers' outputs, and the three commitment proofs (size
classes 5 to 10, columns split at cmax, merged sets with mixed-height trees, a segment, point reductions in batches,
BaseFold with one and two oracle levels, grinding, six queries) -- over inputs from SBCL's seeded generator
(tests/golden/sbcl_random.py).  A digest matches only if the generator, the inputs, every message of every proof,
the verifier's claims and the proof encoding are the reference's, byte for byte."""
import hashlib
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import frozen_cases as fc  # noqa: E402
from oracle import binding as orc  # noqa: E402
from oracle import domain as od  # noqa: E402


def test_the_generator_is_mt19937():
    """The first outputs of MT19937 seeded with 5489 (the published reference values)."""
    from sbcl_random import SbclRandom
    st = SbclRandom(5489)
    assert [st.chunk() for _ in range(3)] == [3499211612, 581869302, 3890346734]


def test_prove_upper_makes_the_frozen_gkr_cases():
    def prove(n, k, leaves, d):
        tr = orc.Transcript("gkr-test", d)
        orc.gkr_prove_upper(tr, n, k, leaves)
        return tr.proof()

    def verify(proof, n, k, lookups, d):
        tr = orc.Transcript("gkr-test", d, proof=proof)
        out = orc.gkr_verify_upper(tr, n, k, lookups)
        assert tr.finished()
        return out

    text = fc.gkr_cases_text(prove, verify)
    assert hashlib.sha256(text.encode()).hexdigest() == fc.GKR_SHA256


def test_prove_domain_makes_the_frozen_domain_cases():
    def prove(dom, d, z, betas):
        tr = orc.Transcript("dom-test", d)
        od.prove_domain(tr, dom, z, betas)
        return tr.proof()

    def verify(proof, dom, d, z, betas):
        tr = orc.Transcript("dom-test", d, proof=proof)
        out = od.verify_domain(tr, dom, z, betas)
        assert tr.finished()
        return out

    text = fc.domain_cases_text(od.Domain, od.Column, prove, verify)
    assert hashlib.sha256(text.encode()).hexdigest() == fc.DOMAIN_SHA256


def test_the_commitment_makes_the_frozen_pcs_cases():
    """The reference's commitment scheduler (src/pcs.lisp, prover side) restated over the oracle's primitives in
    tests/golden/pcs_cases.py: RS encoding, leaf digests chained over merged units, Merkle levels with injections and
    caps, the point reductions' sumchecks, combine-columns, the cross-unit sumcheck's dot-pairs / fold-table /
    lagrange, BaseFold over classes, grinding and the query openings."""
    import pcs_cases as pc
    assert hashlib.sha256(pc.pcs_cases_text().encode()).hexdigest() == pc.PCS_SHA256
