"""GPU parity for the commitment path: Reed-Solomon encode and fold, BLAKE3 leaf digests and Merkle
levels, pcs-commit and the BaseFold loop, through the C ABI against the CPU oracle (bit-exact)."""
import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc

pytestmark = pytest.mark.gpu
P = sa.P


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


def test_rs_encode_golden_vectors(vectors):
    for v in vectors("rs-encode"):
        n = v["n"]
        msg = sa.Table.upload(np.array(v["msg"], np.uint32))
        cw = sa.encode(msg, 1, n - 1)
        assert same(cw.download(), v["cw"])
        msg.free(), cw.free()


@pytest.mark.parametrize("c,ncols", [(0, 1), (1, 2), (4, 3), (11, 2), (12, 1), (13, 2), (16, 2), (19, 1)])
def test_rs_encode_matches_the_oracle(c, ncols):
    rng = np.random.default_rng(c)
    msgs = rng.integers(0, P, (ncols, 1 << c), dtype=np.uint32)
    t = sa.Table.upload(msgs.reshape(-1))
    cw = sa.encode(t, ncols, c)
    got = cw.download().reshape(ncols, -1)
    for k in range(ncols):
        assert same(got[k], orc.rs_encode(msgs[k], c + 1)), f"column {k}"
    t.free(), cw.free()


def test_rs_encode_is_evaluation_and_full_size_roundtrip():
    """At the full size (2^23 coefficients -> 2^24 symbols) the oracle is too slow: check the codeword as
    evaluations at a few positions (position t holds f(w^bitrev(t)), rs.lisp:4-6) and that folding the
    codeword is the codeword of the folded message (rs.lisp:8-9)."""
    c = 23
    msg = sa.Table.random(5, 1 << c)
    cw = sa.encode(msg, 1, c)
    m = msg.download().astype(object)
    w = orc.root_of_unity(c + 1)
    for t in (0, 1, 2, 12345, (1 << 24) - 1):
        x = pow(w, int(format(t, "024b")[::-1], 2), P)
        # Horner in Python ints over 2^23 coefficients is slow; use numpy power sums in chunks
        xs = np.array([pow(x, i, P) for i in range(1 << 10)], dtype=object)
        step = pow(x, 1 << 10, P)
        acc, xp = 0, 1
        for i in range(0, 1 << c, 1 << 10):
            acc = (acc + xp * int(np.dot(m[i:i + (1 << 10)], xs) % P)) % P
            xp = xp * step % P
        assert int(cw.download(t, 1)[0]) == acc
    msg.free(), cw.free()


@pytest.mark.parametrize("d,n", [(8, 6), (4, 9), (8, 13)])
def test_rs_fold(d, n, vectors):
    rng = np.random.default_rng(n)
    cw = rng.integers(0, P, (1 << n, d), dtype=np.uint32)
    r = rng.integers(0, P, d, dtype=np.uint32)
    t = sa.Table.upload(cw)
    for level in (0, 1):
        m = (1 << n) >> (level + 1)
        sub = sa.Table.upload(cw[:2 * m])
        out = sa.rs_fold(sub, d, n, level, r)
        assert same(out.download(), orc.rs_fold(cw[:2 * m], orc.twiddles(n)[level], r))
        sub.free(), out.free()
    t.free()
    if d == 8 and n == 6:
        for v in vectors("rs-fold"):
            t = sa.Table.upload(np.array(v["cw"], np.uint32))
            out = sa.rs_fold(t, 8, v["n"], 0, v["r"])
            assert same(out.download(), v["res"])


@pytest.mark.parametrize("c,ncols", [(1, 1), (5, 2), (9, 3), (10, 70), (14, 2)])
def test_merkle_commit_matches_the_oracle(c, ncols):
    rng = np.random.default_rng(c + ncols)
    cols = [rng.integers(0, P, 1 << c, dtype=np.uint32) for _ in range(ncols)]
    ocw, olevels, ocap = orc.commit_columns(cols, c)
    tr, otr = sa.Transcript("commit", 4), orc.Transcript("commit", 4)
    t = sa.Table.upload(np.concatenate(cols))
    cw, levels = sa.pcs_commit(tr, t, ncols, c)
    otr.send_bytes(ocap.tobytes())
    assert tr.proof() == otr.proof()
    assert same(cw.download().reshape(ncols, -1), ocw)
    got = levels.download().reshape(-1, 8).astype("<u4").view(np.uint8).reshape(-1, 32)
    assert same(got, np.concatenate(olevels))
    for x in (t, cw, levels):
        x.free()


def test_commit_full_size_paths_open_to_the_cap():
    """Config 5's commitment at full size: two 2^23-coefficient columns -> 2^22 leaves -> cap of 128; a few
    leaves are recomputed on the host from the downloaded codeword symbols and opened against the cap."""
    c, ncols = 23, 2
    t = sa.Table.random(11, ncols << c)
    tr = sa.Transcript("commit", 4)
    cw, levels = sa.pcs_commit(tr, t, ncols, c)
    cap = np.frombuffer(orc.decode_proof(tr.proof())[0], np.uint8).reshape(-1, 32)
    nleaves = 1 << (c - 1)
    lc = orc.cap_level(nleaves)
    assert len(cap) == 128 and lc == 15
    cwlen = 1 << (c + 1)
    for leaf in (0, 1, 999999, nleaves - 1):
        rows = [cw.download(k * cwlen + 4 * leaf, 4) for k in range(ncols)]
        h = orc.leaf_digest(np.array(rows))
        path, i, start, n = [], leaf, 0, nleaves
        for _ in range(lc):
            path.append(levels.download((start + (i ^ 1)) * 8, 8).reshape(-1).astype("<u4").view(np.uint8))
            start += n
            n //= 2
            i >>= 1
        assert orc.check_path(h, np.array(path), leaf, cap)
    for x in (t, cw, levels):
        x.free()


@pytest.mark.parametrize("nv", [4, 9, 12])
def test_basefold_matches_the_oracle(nv):
    rng = np.random.default_rng(nv)
    h = rng.integers(0, P, (1 << nv, 8), dtype=np.uint32)
    rr = rng.integers(0, P, (nv, 8), dtype=np.uint32)
    v = orc.mle_eval(h, rr, 8)
    tr, otr = sa.Transcript("bf", 4), orc.Transcript("bf", 4)
    t = sa.Table.upload(h)
    got = sa.basefold_prove(tr, nv, rr, v, t)
    want = orc.basefold_prove(otr, nv, rr, v, h)
    assert tr.proof() == otr.proof()
    assert got[0] == want[0] and same(got[1], want[1]) and same(got[2], want[2])
    assert sa.basefold_verify(sa.Transcript("bf", 4, proof=tr.proof()), nv, rr, v) == got[0]
    with pytest.raises(sa.VerificationFailure):
        sa.basefold_verify(sa.Transcript("bf", 4, proof=tr.proof()), nv, rr, orc.ext_add(v, orc.base_to_ext(1, 8)))
    t.free()


@pytest.mark.parametrize("nv", [6, 11])
def test_basefold_from_the_committed_codewords_matches_the_oracle(nv):
    """The table is combine-columns of three committed columns; its codeword is handed over as the same combination
    of their committed codewords (encoding is linear) instead of being encoded again: the oracle's bytes."""
    rng = np.random.default_rng(100 + nv)
    ncols = 3
    cols = rng.integers(0, P, (ncols, 1 << nv), dtype=np.uint32)
    cf = rng.integers(0, P, (ncols, 8), dtype=np.uint32)
    rr = rng.integers(0, P, (nv, 8), dtype=np.uint32)
    h = orc.combine_columns(cols, cf)
    v = orc.mle_eval(h, rr, 8)
    otr = orc.Transcript("bf", 4)
    want = orc.basefold_prove(otr, nv, rr, v, h)
    t = sa.Table.upload(cols.reshape(-1))
    cw = sa.encode(t, ncols, nv)
    th, tcw = sa.combine_columns(t, ncols, cf), sa.combine_columns(cw, ncols, cf)
    tr = sa.Transcript("bf", 4)
    got = sa.basefold_prove(tr, nv, rr, v, th, codeword=tcw)
    assert tr.proof() == otr.proof() and got[0] == want[0]
    for x in (t, cw, th, tcw):
        x.free()


def test_basefold_round_trip_beyond_the_oracle_sizes():
    """nv = 19 (the oracle stops near 12): the claim comes from the device's hypercube sum with eq = the
    point, the prover's own round checks pass, the verifier's BaseFold side accepts the proof (rounds, final
    claim, grinding; the query openings are checked by verify-queries, tests/test_gpu_open.py) and rejects
    another claim."""
    nv = 19
    rng = np.random.default_rng(19)
    h = sa.Table.random(77, 1 << nv, 8)
    rr = rng.integers(0, P, (nv, 8), dtype=np.uint32)
    v = sa.hypercube_sum(sa.Statement("t0", ["t0"]), nv, [h], 8, eq=rr)
    tr = sa.Transcript("bf-large", 4)
    qs, chal, final = sa.basefold_prove(tr, nv, rr, v, h)
    assert len(chal) == nv - 5 and final.shape == (32, 8)
    assert sa.basefold_verify(sa.Transcript("bf-large", 4, proof=tr.proof()), nv, rr, v) == qs
    with pytest.raises(sa.VerificationFailure):
        sa.basefold_verify(sa.Transcript("bf-large", 4, proof=tr.proof()), nv, rr, orc.ext_add(v, orc.base_to_ext(1, 8)))
    h.free()


@pytest.mark.parametrize("d,ncols,length", [(8, 1, 16), (8, 2, 1 << 12), (8, 5, 1001), (4, 3, 4096), (8, 40, 512),
                                            (4, 33, 7), (8, 128, 300), (4, 70, 1 << 10), (8, 41, 3)])
def test_combine_columns_matches_the_oracle(d, ncols, length):
    """combine-columns (src/pcs.lisp:434-441): lengths that are not multiples of four included, and more than 32
    columns (the one-pass kernel that takes its coefficients from device memory, eight columns at a time)."""
    rng = np.random.default_rng(ncols * 1000 + length)
    cols = rng.integers(0, P, (ncols, length), dtype=np.uint32)
    cf = rng.integers(0, P, (ncols, d), dtype=np.uint32)
    t = sa.Table.upload(cols.reshape(-1))
    g = sa.combine_columns(t, ncols, cf)
    assert same(g.download().reshape(length, d), orc.combine_columns(cols, cf))
    g.free()
    t.free()


def test_combine_columns_feeds_basefold_at_size():
    """Two base columns of 2^19 combined into the table BaseFold opens: the claim is the same combination of the
    columns' own evaluations at the point (combine-columns is linear, as pcs.lisp:425-430 uses it), and the
    verifier accepts exactly that claim."""
    nv, ncols = 19, 2
    rng = np.random.default_rng(1434)
    cols = sa.Table.random(91, ncols << nv)
    cf = rng.integers(0, P, (ncols, 8), dtype=np.uint32)
    rr = rng.integers(0, P, (nv, 8), dtype=np.uint32)
    g = sa.combine_columns(cols, ncols, cf)
    host = cols.download().reshape(ncols, 1 << nv)
    v = np.zeros(8, np.uint32)
    for k in range(ncols):
        col = sa.Table.upload(host[k])
        y = sa.hypercube_sum(sa.Statement("t0", ["t0"]), nv, [col], 8, eq=rr)  # the column's MLE at the point
        v = orc.ext_add(v, orc.ext_mul(cf[k], y))
        col.free()
    assert same(sa.hypercube_sum(sa.Statement("t0", ["t0"]), nv, [g], 8, eq=rr), v)
    tr = sa.Transcript("bf-combined", 4)
    qs, _, _ = sa.basefold_prove(tr, nv, rr, v, g)
    assert sa.basefold_verify(sa.Transcript("bf-combined", 4, proof=tr.proof()), nv, rr, v) == qs
    g.free()
    cols.free()


@pytest.mark.parametrize("d,k", [(4, 0), (4, 1), (8, 5), (4, 12), (8, 9)])
def test_eq_table_on_the_device(d, k):
    rng = np.random.default_rng(k * 10 + d)
    r = rng.integers(0, P, (k, d), dtype=np.uint32)
    t = sa.eq_table_device(r, d)
    assert same(t.download().reshape(1 << k, d), orc.eq_table(r, d))
    t.free()


def test_reduce_points_sumcheck_from_device_tables():
    """The prover's side of reduce-points (src/pcs.lisp:333-362) from the entry points: per group of opening
    points an eq table of the point and the columns combined with the group's F_p^4 coefficients, both built on
    the device, then PROVE of (+ (* E0 G0) (* E1 G1)) with label "pcs-red" and degree 2.  Same proof bytes as the
    oracle's composition of the same steps; the claim is the combination of the columns' evaluations, and the
    verifier accepts it."""
    c, ncols, d = 12, 3, 4
    rng = np.random.default_rng(333)
    cols = rng.integers(0, P, (ncols, 1 << c), dtype=np.uint32)
    zs = [rng.integers(0, P, (c, d), dtype=np.uint32) for _ in range(2)]
    cfs = [rng.integers(0, P, (ncols, d), dtype=np.uint32) for _ in range(2)]
    form, names = "(+ (* e0 g0) (* e1 g1))", ["e0", "g0", "e1", "g1"]
    dcols = sa.Table.upload(cols.reshape(-1))
    dev, host = [], []
    for z, cf in zip(zs, cfs):
        dev += [sa.eq_table_device(z, d), sa.combine_columns(dcols, ncols, cf)]
        host += [orc.eq_table(z, d), orc.combine_columns(cols, cf)]
    tr, otr = sa.Transcript("red", d), orc.Transcript("red", d)
    st, ost = sa.Statement(form, names), orc.Statement(form, names)
    rho, finals, _ = sa.prove(tr, c, st, dev, label="pcs-red", degree=2)
    want = orc.prove(otr, c, ost, host, label="pcs-red", degree=2)
    assert tr.proof() == otr.proof() and same(rho, want[0]) and same(finals, want[1])
    claim = np.zeros(d, np.uint32)
    for z, cf in zip(zs, cfs):
        for k in range(ncols):
            lifted = np.zeros((1 << c, d), np.uint32)
            lifted[:, 0] = cols[k]
            claim = orc.ext_add(claim, orc.ext_mul(cf[k], orc.mle_eval(lifted, z, d)))
    got_rho, reduced = sa.verify(sa.Transcript("red", d, proof=tr.proof()), c, st, claim, label="pcs-red", degree=2)
    assert same(got_rho, rho)
    assert sa.check_final(reduced, st, finals)
    for t in dev:
        t.free()
    dcols.free()


@pytest.mark.parametrize("length", [2, 64, 1 << 12])
def test_dot_pairs_and_fold_table_match_the_oracle(length):
    """One class's share of a cross-rounds round (src/pcs.lisp:473-512): the three parity sums and the folds."""
    rng = np.random.default_rng(length)
    e = rng.integers(0, P, (length, 8), dtype=np.uint32)
    v = rng.integers(0, P, (length, 8), dtype=np.uint32)
    x = rng.integers(0, P, 8, dtype=np.uint32)
    te, tv = sa.Table.upload(e), sa.Table.upload(v)
    assert same(sa.dot_pairs(te, tv), orc.dot_pairs(e, v))
    fe = sa.fold_table(te, x)
    assert same(fe.download().reshape(-1, 8), orc.fold_table(e, x))
    q = rng.integers(0, P, (length, 4), dtype=np.uint32)
    x4 = rng.integers(0, P, 4, dtype=np.uint32)
    tq = sa.Table.upload(q)
    fq = sa.fold_table(tq, x4)
    assert same(fq.download().reshape(-1, 4), orc.fold_table(q, x4))
    for t in (te, tv, fe, tq, fq):
        t.free()


def test_cross_round_identity_at_size():
    """At 2^20 entries per table, beyond what the oracle runs in seconds: the round's three sums are g(0), g(1), g(2)
    of the quadratic g(X) = sum_i E_i(X) V_i(X), so after folding both tables by x the next round's g(0) + g(1) is
    g(x) by Lagrange (the check of src/pcs.lisp:502-506), and two rounds chain."""
    length = 1 << 20
    rng = np.random.default_rng(20)
    e, v = sa.Table.random(501, length, 8), sa.Table.random(502, length, 8)
    for _ in range(2):
        ev = sa.dot_pairs(e, v)
        x = rng.integers(0, P, 8, dtype=np.uint32)
        e2, v2 = sa.fold_table(e, x), sa.fold_table(v, x)
        nxt = sa.dot_pairs(e2, v2)
        assert same(orc.ext_add(nxt[0], nxt[1]), orc.lagrange(ev, x))
        e.free(), v.free()
        e, v = e2, v2
    e.free(), v.free()


@pytest.mark.parametrize("d,length", [(8, 1), (8, 1000), (4, 4096)])
def test_scale_add_builds_the_class_table(d, length):
    """src/pcs.lisp:709-716: the class's table is the sum over its units of scalar * column, from zeros."""
    rng = np.random.default_rng(709 + length)
    cols = [rng.integers(0, P, (length, d), dtype=np.uint32) for _ in range(3)]
    scs = [rng.integers(0, P, d, dtype=np.uint32) for _ in range(3)]
    want = np.zeros((length, d), np.uint32)
    h = None
    for col, sc in zip(cols, scs):
        want = orc.scale_add(want, sc, col)
        t = sa.Table.upload(col)
        nxt = sa.scale_add(h, sc, t)
        t.free()
        if h is not None:
            h.free()
        h = nxt
    assert same(h.download().reshape(length, d), want)
    h.free()


@pytest.mark.parametrize("c,ncols,count", [(1, 1, 3), (6, 5, 7), (12, 3, 40), (9, 70, 1)])
def test_open_queries_match_the_oracle(c, ncols, count):
    """src/pcs.lisp:721-734: the queried leaves' rows and their paths, as the prover records them."""
    rng = np.random.default_rng(c * 100 + ncols)
    cols = [rng.integers(0, P, 1 << c, dtype=np.uint32) for _ in range(ncols)]
    ocw, olevels, ocap = orc.commit_columns(cols, c)
    nleaves = 1 << (c - 1)
    idx = rng.integers(0, nleaves, count).astype(np.uint64)
    idx[0], idx[-1] = 0, nleaves - 1
    want_leaves, want_paths = orc.open_queries(ocw, c, olevels, idx)
    t = sa.Table.upload(np.concatenate(cols))
    cw = sa.encode(t, ncols, c)
    levels, cap = sa.merkle_commit(cw, ncols, c)
    got_leaves, got_paths = sa.open_queries(cw, ncols, c, levels, idx)
    assert same(got_leaves, want_leaves)
    assert got_paths.shape == want_paths.shape and same(got_paths, want_paths)
    only_leaves, none = sa.open_queries(cw, ncols, c, None, idx)
    assert same(only_leaves, want_leaves) and none.shape == (count, 0, 32)
    empty = sa.open_queries(cw, ncols, c, levels, np.zeros(0, np.uint64))
    assert empty[0].shape == (0, ncols, 4)
    with pytest.raises(sa.ExactaError):
        sa.open_queries(cw, ncols, c, levels, np.array([nleaves], np.uint64))
    for x in (t, cw, levels):
        x.free()


def test_open_queries_full_size_open_to_the_cap():
    """Config 5's commitment: 64 queried leaves of the 2^22-leaf tree, each hashed and walked up its path to the cap."""
    c, ncols = 23, 2
    t = sa.Table.random(12, ncols << c)
    cw = sa.encode(t, ncols, c)
    levels, cap = sa.merkle_commit(cw, ncols, c)
    nleaves = 1 << (c - 1)
    idx = np.random.default_rng(5).integers(0, nleaves, 64).astype(np.uint64)
    leaves, paths = sa.open_queries(cw, ncols, c, levels, idx)
    assert paths.shape == (64, orc.cap_level(nleaves), 32)
    for q, l in enumerate(int(x) for x in idx):
        assert orc.check_path(orc.leaf_digest(leaves[q]), paths[q], l, cap)
    assert not orc.check_path(orc.leaf_digest(leaves[0]), paths[1], int(idx[0]), cap)
    for x in (t, cw, levels):
        x.free()
