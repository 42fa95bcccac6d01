"""Kernels generated at run time (exh_stmt_generate, and the compilation a first proof starts by itself): a
statement the build has no kernel for is proved on the interpreter kernel first and on its generated kernels once
they are compiled, with the oracle's bytes both times (ROUND-KERNEL compiles any statement on first use,
src/sumcheck.lisp:270-280)."""
import time

import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc

pytestmark = pytest.mark.gpu


def proof_pair(form, tables, constants, n, d, seed):
    ost = orc.Statement(form, tables, constants)
    tabs = [orc.splitmix_field(seed + k, 1 << n) for k in range(len(tables))]
    eq = orc.splitmix_field(seed + 100, n * d).reshape(n, d)
    cv = orc.splitmix_field(seed + 200, d * len(constants)).reshape(-1, d) if constants else None
    orc.set_fast(orc.host_threads())
    otr = orc.Transcript("rtc", d)
    orc.prove(otr, n, ost, tabs, eq=eq, constants=cv)
    orc.set_fast(0)
    return otr.proof(), tabs, eq, cv


def device_proof(st, tabs, eq, cv, n, d):
    dev = [sa.Table.upload(t) for t in tabs]
    tr = sa.Transcript("rtc", d)
    sa.prove(tr, n, st, dev, eq=eq, constants=cv)
    for t in dev:
        t.free()
    return tr.proof()


def test_an_unseen_statement_gets_kernels_after_its_first_proof():
    form, tables, constants, d = "(+ (* t0 t1 t2) (* 7 t0) (* c0 t1 t1) (* -2 t2))", ["t0", "t1", "t2"], ["c0"], 4
    st = sa.Statement(form, tables, constants)
    assert not st.has_generated_kernel(d)
    want, tabs, eq, cv = proof_pair(form, tables, constants, 20, d, 31)
    assert device_proof(st, tabs, eq, cv, 20, d) == want  # the interpreter kernel; starts the compilation
    deadline = time.time() + 300
    while not st.has_generated_kernel(d) and time.time() < deadline:
        time.sleep(1)
    assert st.has_generated_kernel(d)
    assert device_proof(st, tabs, eq, cv, 20, d) == want  # the generated kernels
    # a size that takes the base-field sweep, the double fold, the streaming rounds and the slices
    want, tabs, eq, cv = proof_pair(form, tables, constants, 21, d, 32)
    assert device_proof(st, tabs, eq, cv, 21, d) == want
    # and small ones (one workgroup from the start)
    for n in (1, 2, 5, 9):
        want, tabs, eq, cv = proof_pair(form, tables, constants, n, d, 33 + n)
        assert device_proof(st, tabs, eq, cv, n, d) == want


def test_generate_ahead_of_the_first_proof_d8():
    form, tables, d = "(* (- a b) (+ a (* 3 c)))", ["a", "b", "c"], 8
    st = sa.Statement(form, tables)
    assert st.generate(d, wait=True) and st.has_generated_kernel(d)
    for n in (3, 12, 18):
        want, tabs, eq, cv = proof_pair(form, tables, [], n, d, 50 + n)
        assert device_proof(st, tabs, eq, cv, n, d) == want
