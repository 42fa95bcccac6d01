"""The device's proofs against the reference's frozen cases (tests/tests.lisp:902-925), with no oracle in between:
the case files of EXPORT-GKR-CASES and EXPORT-DOMAIN-CASES rebuilt from what `exh_gkr_prove_upper`, the device's
domain prover and the library's verifiers return, over the reference's own inputs (SBCL's seeded generator,
tests/golden/sbcl_random.py), hash to the digests the reference pins."""
import hashlib
import os
import sys

import numpy as np
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


def raw_table(words):
    """Words that are not field values (digests) as a device Table: allocated by the library, filled by a plain copy
    (`exh_table_upload` takes canonical values only)."""
    import ctypes as C
    words = np.ascontiguousarray(words, np.uint32)
    h = C.c_uint64()
    sa.check(sa.load().exh_table_alloc(C.c_uint64(words.size), 8, C.byref(h)))
    t = sa.Table(h.value, words.size, 8)
    hip = C.CDLL("/opt/rocm/lib/libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    assert hip.hipMemcpy(C.c_void_p(t.device_ptr()), words.ctypes.data_as(C.c_void_p), words.nbytes, 1) == 0
    return t


class DeviceBackend:
    """The commitment scheduler's primitives (tests/golden/pcs_cases.py) on the device: every array goes up, the
    library's entry point runs, the result comes down.  On the host stay the scheduler itself, the arithmetic on
    single field elements, and the one hash that chains a merged unit's leaf digest to the units before it."""
    def transcript(self, label, d):
        return sa.Transcript(label, d)

    def encode(self, columns, c):
        t = sa.Table.upload(np.concatenate(columns))
        cw = sa.encode(t, len(columns), c)
        out = cw.download().reshape(len(columns), -1)
        t.free(), cw.free()
        return [row.copy() for row in out]

    def leaf_digests(self, codewords, c, previous):
        assert len(codewords) <= 64  # (beyond 64 columns a chained digest is not a node of two digests)
        t = sa.Table.upload(np.concatenate(codewords))
        levels, _ = sa.merkle_commit(t, len(codewords), c)
        own = levels.download()[:1 << (c - 1)].copy().view(np.uint8).reshape(-1, 32)
        t.free(), levels.free()
        if previous is None:
            return own
        return np.array([np.frombuffer(sa.blake3(bytes(p) + bytes(d)), np.uint8) for p, d in zip(previous, own)], np.uint8)

    def merkle_levels(self, leaves, injections):
        as_table = lambda digests: raw_table(np.ascontiguousarray(digests, np.uint8).view(np.uint32).reshape(-1, 8))
        t = as_table(leaves)
        inj = {level: as_table(digests) for level, digests in injections.items()}
        levels = sa.merkle_levels_injected(t, inj)
        flat = levels.download().view(np.uint8).reshape(-1, 32)
        for x in [t, levels] + list(inj.values()):
            x.free()
        out, pos, n = [], 0, len(leaves)
        while n >= 1:
            out.append(flat[pos:pos + n].copy())
            pos += n
            n //= 2
        return out

    def prove_reduction(self, tr, c, form, names, tables):
        dev = [sa.Table.upload(t) for t in tables]
        st = sa.Statement(form, names)
        rho, _, _ = sa.prove(tr, c, st, dev, label="pcs-red", degree=2)
        for t in dev:
            t.free()
        st.free()
        return [r for r in rho]

    def mle_eval(self, table, point, d):
        t = sa.Table.upload(np.asarray(table, np.uint32))
        st = sa.Statement("t0", ["t0"])
        v = sa.hypercube_sum(st, len(point), [t], d, eq=np.array(point, np.uint32))
        t.free(), st.free()
        return v

    def combine_columns(self, columns, coefficients):
        t = sa.Table.upload(np.concatenate(columns))
        g = sa.combine_columns(t, len(columns), np.asarray(coefficients, np.uint32))
        out = g.download()
        t.free(), g.free()
        return out

    def eq_table(self, point, d):
        t = sa.eq_table_device(np.array(point, np.uint32), d)
        out = t.download()
        t.free()
        return out

    def scale_add(self, h, scale, column):
        tc = sa.Table.upload(np.asarray(column, np.uint32))
        th = sa.Table.upload(np.asarray(h, np.uint32)) if h is not None else None
        out = sa.scale_add(th, scale, tc)
        res = out.download()
        for x in (tc, th, out):
            if x is not None:
                x.free()
        return res

    def dot_pairs(self, e, v):
        te, tv = sa.Table.upload(np.asarray(e, np.uint32)), sa.Table.upload(np.asarray(v, np.uint32))
        out = sa.dot_pairs(te, tv)
        te.free(), tv.free()
        return out

    def fold_table(self, table, x):
        t = sa.Table.upload(np.asarray(table, np.uint32))
        f = sa.fold_table(t, x)
        out = f.download()
        t.free(), f.free()
        return out

    def basefold_classes(self, tr, nv, classes, rr, v, grind_bits, queries):
        dev = [(c, sa.Table.upload(np.asarray(h, np.uint32))) for c, h in classes]
        qs = sa.basefold_prove_classes(tr, nv, dev, rr, v, grind_bits=grind_bits, queries=queries)
        for _, t in dev:
            t.free()
        return qs

    def gather_leaves(self, codewords, c, leaves):
        t = sa.Table.upload(np.concatenate(codewords))
        rows, _ = sa.open_queries(t, len(codewords), c, None, leaves)
        t.free()
        return rows


def test_the_device_makes_the_frozen_pcs_cases():
    """The three commitment proofs of EXPORT-PCS-CASES (tests/tests.lisp:728-758) with the device's encoder, leaf
    and Merkle hashes (injected levels included), sumcheck, combine-columns, eq tables, dot-pairs, fold-table and
    BaseFold over classes under the reference's scheduler: the reference's own SHA-256."""
    import pcs_cases as pc
    assert hashlib.sha256(pc.pcs_cases_text(DeviceBackend()).encode()).hexdigest() == pc.PCS_SHA256
