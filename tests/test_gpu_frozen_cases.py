"""The device's proofs against the reference's frozen cases (tests/tests.lisp:902-925), with no oracle in between:
the case files of EXPORT-GKR-CASES and EXPORT-DOMAIN-CASES rebuilt from what `exh_gkr_prove_upper`, the device's
domain prover and the library's verifiers return, over the reference's own inputs (SBCL's seeded generator,
tests/golden/sbcl_random.py), hash to the digests the reference pins."""
import hashlib
import os
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import frozen_cases as fc  # noqa: E402
import sable_amd as sa  # noqa: E402
from sable_amd import domain as sd  # noqa: E402

pytestmark = pytest.mark.gpu


def test_the_device_makes_the_frozen_gkr_cases():
    def prove(n, k, leaves, d):
        dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
        tr = sa.Transcript("gkr-test", d)
        sa.prove_upper(tr, n, k, dev)
        for p, q in dev:
            p.free(), q.free()
        return tr.proof()

    def verify(proof, n, k, lookups, d):
        tr = sa.Transcript("gkr-test", d, proof=proof)
        out = sa.verify_upper(tr, n, k, lookups)
        assert tr.finished()
        return out

    text = fc.gkr_cases_text(prove, verify)
    assert hashlib.sha256(text.encode()).hexdigest() == fc.GKR_SHA256


def test_the_device_makes_the_frozen_domain_cases():
    def prove(dom, d, z, betas):
        tr = sa.Transcript("dom-test", d)
        sd.prove_domain(tr, dom, z, betas)
        return tr.proof()

    def verify(proof, dom, d, z, betas):
        tr = sa.Transcript("dom-test", d, proof=proof)
        out = sd.verify_domain(tr, dom, z, betas)
        assert tr.finished()
        return out

    text = fc.domain_cases_text(sd.Domain, sd.Column, prove, verify)
    assert hashlib.sha256(text.encode()).hexdigest() == fc.DOMAIN_SHA256
