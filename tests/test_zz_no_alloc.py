"""The entry point that allocates nothing: exh_dot_pairs_static against exh_dot_pairs, bit for bit, on two calls
in a row, the second on a smaller input (the static scratch array keeps the first call's partial sums), and
its refusal of sizes beyond its stated maximum."""
import ctypes as C

import numpy as np
import pytest

import sable_amd as sa

pytestmark = pytest.mark.gpu


def test_static_dot_pairs_matches_the_allocating_entry_point_twice_in_a_row():
    for length in (1 << 20, 1 << 9, 6, 1 << 14, 2):
        e, v = sa.Table.random(9000 + length, length, 8), sa.Table.random(9500 + length, length, 8)
        want = sa.dot_pairs(e, v)
        got = sa.dot_pairs_static(e, v)
        assert np.array_equal(got, want), f"length {length}"
        assert np.array_equal(sa.dot_pairs_static(e, v), want), f"length {length}, repeated"
        e.free(), v.free()


def test_static_dot_pairs_matches_the_oracle_directly():
    """Against the CPU oracle's dot-pairs itself (not only against the allocating entry point), after a larger call
    has left its partial sums in the static array."""
    from oracle import binding as orc
    big_e, big_v = sa.Table.random(9701, 1 << 16, 8), sa.Table.random(9702, 1 << 16, 8)
    sa.dot_pairs_static(big_e, big_v)
    big_e.free(), big_v.free()
    for length in (1 << 10, 6):
        e, v = sa.Table.random(9600 + length, length, 8), sa.Table.random(9650 + length, length, 8)
        he, hv = e.download().reshape(-1, 8), v.download().reshape(-1, 8)
        assert np.array_equal(sa.dot_pairs_static(e, v), orc.dot_pairs(he, hv)), f"length {length}"
        e.free(), v.free()


def test_static_dot_pairs_refuses_what_it_cannot_hold():
    lib = sa.load()
    out = np.zeros((3, 8), np.uint32)
    e = sa.Table.random(1, 6, 8)
    base = sa.Table.random(2, 48)  # base values: the wrong stride
    assert lib.exh_dot_pairs_static(C.c_uint64(e.handle), C.c_uint64(base.handle), sa._p(out)) < 0
    with pytest.raises(sa.InvalidParameter):
        sa.dot_pairs_static(e, base)
    e.free(), base.free()
    # beyond the stated maximum of 2^26 EXT8s per table (the allocating entry point takes these)
    n = ((1 << 26) + 2) * 8
    h = C.c_uint64()
    sa.check(lib.exh_table_alloc(C.c_uint64(n), 8, C.byref(h)))
    big = sa.Table(h.value, n, 8)
    with pytest.raises(sa.InvalidParameter, match="2\\^26"):
        sa.dot_pairs_static(big, big)
    big.free()
