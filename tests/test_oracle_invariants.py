"""The oracle where no golden bytes exist: invariants the reference's own suite uses
(tests/tests.lisp:311-462, 694-720) and brute force from the definitions on tiny inputs."""
import numpy as np
import pytest

import pyfield as pf
from oracle import binding as orc
from oracle import forms

P = orc.P


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


def rand_ext(rng, shape, d):
    return rng.integers(0, P, tuple(shape) + (d,), dtype=np.uint32)


CONFIG2 = "(+ (* alpha t0 t1 t2) (* 3 t1))"


# ------------------------------------------------------------------ sumcheck
@pytest.mark.parametrize("d", [4, 8])
def test_sumcheck_base_tables_equal_lifted(d):
    """tests.lisp:329-346: base tables and their lift give the same proof, byte for byte."""
    n = 4
    rng = np.random.default_rng(d)
    st = orc.Statement("(+ (* t0 t1 t2) (* 7 t1))", ["t0", "t1", "t2"])
    base = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    lifted = [np.concatenate([b[:, None], np.zeros((1 << n, d - 1), np.uint32)], axis=1) for b in base]
    eq = rand_ext(rng, (n,), d)

    def proof(tables):
        tr = orc.Transcript("base", d)
        rho, finals, _ = orc.prove(tr, n, st, tables, eq=eq)
        return rho.tolist(), finals.tolist(), tr.proof()

    assert proof(base) == proof(lifted)
    assert same(orc.hypercube_sum(st, n, base, d, eq=eq), orc.hypercube_sum(st, n, lifted, d, eq=eq))


@pytest.mark.parametrize("d,with_eq", [(4, True), (4, False), (8, True)])
def test_round_messages_from_the_definition(d, with_eq):
    """Every round message recomputed from g_j(X) = sum_x w_j(x) F(line_X) with an independent
    pure-Python field: config 2's statement (a constant, a non-product term), base tables."""
    n = 3
    rng = np.random.default_rng(100 + d)
    form = forms.read_form(CONFIG2)
    st = orc.Statement(CONFIG2, ["t0", "t1", "t2"], ["alpha"])
    assert st.degree == 3
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    alpha = rand_ext(rng, (), d)
    eq = rand_ext(rng, (n,), d) if with_eq else None
    tr = orc.Transcript("def", d)
    rho, finals, _ = orc.prove(tr, n, st, tables, eq=eq, constants=[alpha])
    msgs = tr.messages()
    cur = [[pf.lift(int(v), d) for v in t] for t in tables]
    claim = orc.hypercube_sum(st, n, tables, d, eq=eq, constants=[alpha])
    for j in range(n):
        pairs = len(cur[0]) // 2
        w = pf.eq_table([list(map(int, e)) for e in eq[j + 1:]], d) if with_eq else [pf.lift(1, d)] * pairs
        g = {}
        for X in (0, 1, 2, 3):
            acc = pf.lift(0, d)
            for i in range(pairs):
                vals = {"ALPHA": list(map(int, alpha))}
                for t in range(3):
                    lo, hi = cur[t][2 * i], cur[t][2 * i + 1]
                    vals[f"T{t}"] = pf.add(lo, pf.scale(pf.sub(hi, lo), X))
                acc = pf.add(acc, pf.mul(w[i], pf.evaluate(form, vals, d)))
            g[X] = acc
        assert msgs[j].tolist() == [g[0], g[2], g[3]]
        # claim_j = (1 - r_j) g(0) + r_j g(1) in eq mode, g(0) + g(1) otherwise
        if with_eq:
            rj = list(map(int, eq[j]))
            expect = pf.add(pf.mul(pf.sub(pf.lift(1, d), rj), g[0]), pf.mul(rj, g[1]))
        else:
            expect = pf.add(g[0], g[1])
        assert same(claim, expect)
        r = list(map(int, rho[j]))
        claim = orc.lagrange([g[0], g[1], g[2], g[3]], r)
        cur = [[pf.add(t[2 * i], pf.mul(r, pf.sub(t[2 * i + 1], t[2 * i]))) for i in range(pairs)] for t in cur]
    assert same(finals, [t[0] for t in cur])


def test_round_sums_are_linear_in_the_statement():
    """sums(alpha t0 t1 t2 + 3 t1) = alpha sums(t0 t1 t2) + 3 sums(t1): ties the statement with a constant
    to product statements, which the golden whole-proof vectors pin."""
    d, n = 4, 5
    rng = np.random.default_rng(5)
    tables = [rng.integers(0, P, 1 << n, dtype=np.uint32) for _ in range(3)]
    alpha = rand_ext(rng, (), d)
    eq = rand_ext(rng, (n,), d)
    low, high = orc.eq_table(eq[1:3], d), orc.eq_table(eq[3:], d)
    full = orc.round_sums(orc.Statement(CONFIG2, ["t0", "t1", "t2"], ["alpha"]), d, 3, tables, low, high, [alpha])
    prod = orc.round_sums(orc.Statement("(* t0 t1 t2)", ["t0", "t1", "t2"]), d, 3, tables, low, high)
    lin = orc.round_sums(orc.Statement("t1", ["t0", "t1", "t2"]), d, 3, tables, low, high)
    for k in range(3):
        assert same(full[k], orc.ext_add(orc.ext_mul(alpha, prod[k]), orc.ext_scale(lin[k], 3)))
    # split weights: LOW[l] HIGH[h] is the eq table's entry (the eq tables themselves are vector-pinned)
    whole = orc.eq_table(eq[1:], d)
    for h in range(len(high)):
        for l in range(len(low)):
            assert same(whole[h * len(low) + l], orc.ext_mul(low[l], high[h]))


@pytest.mark.parametrize("d", [4, 8])
def test_sumcheck_of_any_statement(d):
    """tests.lisp:311-327: a statement that is not a plain product, with a constant; prover and verifier."""
    n = 3
    rng = np.random.default_rng(3)
    st = orc.Statement("(+ (* alpha t0 t1) (* 3 t1) -2)", ["t0", "t1"], ["alpha"])
    assert st.degree == 2
    alpha = rand_ext(rng, (), d)
    tables = [rand_ext(rng, (1 << n,), d) for _ in range(2)]
    claim = orc.hypercube_sum(st, n, tables, d, constants=[alpha])
    prover = orc.Transcript("any", d)
    _, finals, _ = orc.prove(prover, n, st, tables, constants=[alpha])
    verifier = orc.Transcript("any", d, proof=prover.proof())
    _, reduced = orc.verify(verifier, n, st, claim, constants=[alpha])
    assert orc.check_final(reduced, st, finals, constants=[alpha])
    with pytest.raises(orc.VerificationFailure):
        orc.check_final(orc.ext_add(reduced, orc.base_to_ext(1, d)), st, finals, constants=[alpha])


def test_sumcheck_block_weights_equal_flat_statement():
    """With block weights the rounds prove sum_b bw_b sum_x eq(r,x) F(tables(x,b)) (sumcheck.lisp:519-521):
    claim_0 recovered from the first message equals that sum."""
    d, n, K = 4, 3, 3
    rng = np.random.default_rng(8)
    st = orc.Statement("(* t0 t1)", ["t0", "t1"])
    tables = [rand_ext(rng, (K << n,), d) for _ in range(2)]
    bw = rand_ext(rng, (K,), d)
    eq = rand_ext(rng, (n,), d)
    total = np.zeros(d, np.uint32)
    for b in range(K):
        blk = [t[b << n:(b + 1) << n] for t in tables]
        total = orc.ext_add(total, orc.ext_mul(bw[b], orc.hypercube_sum(st, n, blk, d, eq=eq)))
    prover = orc.Transcript("bw", d)
    _, finals, folded = orc.prove(prover, n, st, tables, eq=eq, block_weights=bw)
    verifier = orc.Transcript("bw", d, proof=prover.proof())
    _, reduced = orc.verify(verifier, n, st, total, eq=eq, blocks=K)
    acc = np.zeros(d, np.uint32)
    for b in range(K):
        acc = orc.ext_add(acc, orc.ext_mul(bw[b], orc.ext_mul(folded[0][b], folded[1][b])))
    assert same(reduced, acc)
    assert same(finals[0], folded[0][0])


# ------------------------------------------------------------------ LogUp-GKR (tests.lisp:399-462)
def random_leaves(rng, lookups, n, k, d):
    out = []
    for _ in range(lookups):
        p = rand_ext(rng, (k << n,), d)
        q = rand_ext(rng, (k << n,), d)
        q[:, 0] |= 1
        out.append((p, q))
    return out


GKR_CASES = [(3, 1, 1, 4), (3, 3, 2, 4), (2, 4, 1, 8), (4, 5, 2, 4), (1, 2, 1, 4), (1, 1, 2, 8), (2, 2, 3, 4)]


@pytest.mark.parametrize("n,k,lookups,d", GKR_CASES)
def test_gkr_roundtrip(n, k, lookups, d):
    rng = np.random.default_rng(n + k + lookups + d)
    leaves = random_leaves(rng, lookups, n, k, d)
    prover = orc.Transcript("gkr-test", d)
    outputs = orc.gkr_prove_upper(prover, n, k, leaves)
    verifier = orc.Transcript("gkr-test", d, proof=prover.proof())
    roots, ri, rb, cp, cq = orc.gkr_verify_upper(verifier, n, k, lookups)
    assert verifier.finished()
    for a, b in zip((ri, rb, cp, cq), outputs):
        assert same(a, b)
    for (p, q), root in zip(leaves, roots):
        # LogUp: each root is the sum of its leaf fractions
        total = np.zeros(d, np.uint32)
        for a, b in zip(p, q):
            total = orc.ext_add(total, orc.ext_mul(a, orc.ext_inv(b)))
        assert same(orc.ext_mul(root[0], orc.ext_inv(root[1])), total)
    # the claims are on the leaves' parents: sum_{b<K} eq(rb, b) parent_b(ri)
    weights = orc.eq_table(rb, d) if len(rb) else [orc.base_to_ext(1, d)]
    size = 1 << (n - 1)
    for (p, q), claim_p, claim_q in zip(leaves, cp, cq):
        pp, qq = orc.gkr_reduce_layer(p, q, k, n - 1)
        for values, claim in ((pp, claim_p), (qq, claim_q)):
            acc = np.zeros(d, np.uint32)
            for b in range(k):
                acc = orc.ext_add(acc, orc.ext_mul(weights[b], orc.mle_eval(values[b * size:(b + 1) * size], ri, d)))
            assert same(claim, acc)


def test_gkr_reduce_layer_from_the_definition():
    d, k, m = 4, 2, 2
    rng = np.random.default_rng(2)
    p, q = rand_ext(rng, (k << (m + 1),), d), rand_ext(rng, (k << (m + 1),), d)
    pp, qq = orc.gkr_reduce_layer(p, q, k, m)
    for b in range(k):
        for x in range(1 << m):
            c0, c1 = b * (2 << m) + x, b * (2 << m) + x + (1 << m)
            P0, Q0, P1, Q1 = (list(map(int, v)) for v in (p[c0], q[c0], p[c1], q[c1]))
            assert pp[b * (1 << m) + x].tolist() == pf.add(pf.mul(P0, Q1), pf.mul(P1, Q0))
            assert qq[b * (1 << m) + x].tolist() == pf.mul(Q0, Q1)


def test_gkr_rejects_forgeries():
    n, k, lookups, d = 3, 3, 2, 4
    rng = np.random.default_rng(9)
    leaves = random_leaves(rng, lookups, n, k, d)
    prover = orc.Transcript("gkr-test", d)
    orc.gkr_prove_upper(prover, n, k, leaves)
    msgs = prover.messages()
    orc.gkr_verify_upper(orc.Transcript("gkr-test", d, proof=orc.encode_messages(msgs)), n, k, lookups)
    for i, m in enumerate(msgs):
        if isinstance(m, bytes):
            continue
        forged = [x if isinstance(x, bytes) else x.copy() for x in msgs]
        forged[i].reshape(-1)[0] = (int(forged[i].reshape(-1)[0]) + 1) % P
        with pytest.raises(orc.VerificationFailure):
            orc.gkr_verify_upper(orc.Transcript("gkr-test", d, proof=orc.encode_messages(forged)), n, k, lookups)


# ------------------------------------------------------------------ commitment
def test_rs_fold_commutes_with_encode():
    """rs.lisp:8-9: the folded codeword is the codeword of (1 - r) m_even + r m_odd."""
    n = 6
    rng = np.random.default_rng(4)
    m = rng.integers(0, P, 1 << (n - 1), dtype=np.uint32)
    r = int(rng.integers(0, P))
    folded = orc.rs_fold(orc.rs_encode(m, n), orc.twiddles(n)[0], [r])
    msg = [(int(a) * (1 - r) + int(b) * r) % P for a, b in zip(m[0::2], m[1::2])]
    assert same(folded, orc.rs_encode(msg, n - 1))
    # the twiddle levels: level l+1 is the twiddles of the half-size domain
    assert all(same(a, b) for a, b in zip(orc.twiddles(n)[1:], orc.twiddles(n - 1)))


def test_leaf_digest_chunks_and_chain():
    rng = np.random.default_rng(6)
    rows = rng.integers(0, P, (150, 4), dtype=np.uint32)
    chunk = lambda r: orc.blake3(np.asarray(r, "<u4").tobytes())
    h = chunk(rows[:64])
    h = orc.blake3(h + chunk(rows[64:128]))
    h = orc.blake3(h + chunk(rows[128:]))
    assert orc.leaf_digest(rows) == h
    assert orc.leaf_digest(rows[64:], previous=chunk(rows[:64])) == h
    assert orc.node(h, h) == orc.blake3(h + h)
    assert [orc.cap_level(x) for x in (1, 2, 128, 256, 1 << 22)] == [0, 0, 0, 1, 15]


def test_commit_columns_paths_open_to_the_cap():
    c, ncols = 9, 3
    rng = np.random.default_rng(10)
    cols = [rng.integers(0, P, 1 << c, dtype=np.uint32) for _ in range(ncols)]
    cw, levels, cap = orc.commit_columns(cols, c)
    assert all(same(cw[k], orc.rs_encode(cols[k], c + 1)) for k in range(ncols))
    nleaves = 1 << (c - 1)
    lc = orc.cap_level(nleaves)
    assert len(cap) == nleaves >> lc == 128 and same(cap, levels[lc])
    for leaf in (0, 1, 77, nleaves - 1):
        rows = [[int(cw[k][4 * leaf + s]) for s in range(4)] for k in range(ncols)]
        h = orc.leaf_digest(rows)
        assert h == bytes(levels[0][leaf])
        path, i = [], leaf
        for level in levels[:lc]:
            path.append(level[i ^ 1])
            i >>= 1
        assert orc.check_path(h, np.array(path, np.uint8).reshape(-1, 32), leaf, cap)
        bad = bytes([h[0] ^ 1]) + h[1:]
        assert not orc.check_path(bad, np.array(path, np.uint8).reshape(-1, 32), leaf, cap)


@pytest.mark.parametrize("nv", [4, 9])
def test_basefold_roundtrip(nv):
    rng = np.random.default_rng(nv)
    h = rand_ext(rng, (1 << nv,), 8)
    rr = rand_ext(rng, (nv,), 8)
    v = orc.mle_eval(h, rr, 8)
    prover = orc.Transcript("bf", 4)
    qs, chal, final = orc.basefold_prove(prover, nv, rr, v, h)
    # pcs.lisp:645: the final table is the message folded at the challenges
    t = h
    for x in chal:
        t = orc.fold_table(t, x)
    assert same(t, final)
    proof = prover.proof()
    verifier = orc.Transcript("bf", 4, proof=proof)
    assert orc.basefold_verify(verifier, nv, rr, v) == qs
    with pytest.raises(orc.VerificationFailure):
        orc.basefold_verify(orc.Transcript("bf", 4, proof=proof), nv, rr, orc.ext_add(v, orc.base_to_ext(1, 8)))
    msgs = orc.decode_proof(proof)
    fl = max(0, nv - 5)
    for i in range(fl + 1):  # every absorbed field message, perturbed, is rejected
        forged = [x if isinstance(x, bytes) else x.copy() for x in msgs]
        k = [j for j, x in enumerate(forged) if not isinstance(x, bytes)][i]
        forged[k].reshape(-1)[0] = (int(forged[k].reshape(-1)[0]) + 1) % P
        with pytest.raises(orc.VerificationFailure):
            orc.basefold_verify(orc.Transcript("bf", 4, proof=orc.encode_messages(forged)), nv, rr, v)


def test_combine_columns_from_the_definition():
    """combine-columns (src/pcs.lisp:434-441) against an independent big-integer evaluation of
    g[x] = sum_k coefficient_k * column_k[x], coordinate by coordinate; unit coefficients give back a column
    embedded in the extension; the map is linear in the coefficients."""
    rng = np.random.default_rng(434)
    for d, ncols, length in ((8, 1, 5), (8, 3, 17), (4, 6, 32)):
        cols = rng.integers(0, P, (ncols, length), dtype=np.uint32)
        cf = rng.integers(0, P, (ncols, d), dtype=np.uint32)
        got = orc.combine_columns(cols, cf)
        want = [[sum(int(cf[k][c]) * int(cols[k][x]) for k in range(ncols)) % P for c in range(d)] for x in range(length)]
        assert got.tolist() == want
        unit = np.zeros((ncols, d), np.uint32)
        unit[ncols - 1, 0] = 1
        only = orc.combine_columns(cols, unit)
        assert only[:, 0].tolist() == cols[ncols - 1].tolist() and not only[:, 1:].any()
        cf2 = rng.integers(0, P, (ncols, d), dtype=np.uint32)
        both = orc.combine_columns(cols, ((cf.astype(np.uint64) + cf2) % P).astype(np.uint32))
        apart = (got.astype(np.uint64) + orc.combine_columns(cols, cf2)) % P
        assert both.tolist() == apart.tolist()


def test_dot_pairs_and_fold_table_from_the_definition():
    """dot-pairs (src/pcs.lisp:473-483) and fold-table (src/field.lisp:365-370) against the independent
    pure-Python field: the three picks (even, odd, 2 odd - even) and entry + r (next - entry)."""
    rng = np.random.default_rng(473)
    for length in (2, 6):
        e = rng.integers(0, P, (length, 8), dtype=np.uint32)
        v = rng.integers(0, P, (length, 8), dtype=np.uint32)
        picks = [lambda t, i: t[i], lambda t, i: t[i + 1],
                 lambda t, i: pf.sub(pf.scale(t[i + 1], 2), t[i])]
        el, vl = [list(map(int, row)) for row in e], [list(map(int, row)) for row in v]
        want = []
        for pick in picks:
            total = [0] * 8
            for i in range(0, length, 2):
                total = pf.add(total, pf.mul(pick(el, i), pick(vl, i)))
            want.append(total)
        assert orc.dot_pairs(e, v).tolist() == want
        r = [int(x) for x in rng.integers(0, P, 8, dtype=np.uint32)]
        folded = [pf.add(el[i], pf.mul(r, pf.sub(el[i + 1], el[i]))) for i in range(0, length, 2)]
        assert orc.fold_table(e, np.array(r, np.uint32)).tolist() == folded


def test_scale_add_from_the_definition():
    rng = np.random.default_rng(709)
    h = rng.integers(0, P, (5, 8), dtype=np.uint32)
    col = rng.integers(0, P, (5, 8), dtype=np.uint32)
    sc = rng.integers(0, P, 8, dtype=np.uint32)
    want = [pf.add(list(map(int, h[x])), pf.mul(list(map(int, sc)), list(map(int, col[x])))) for x in range(5)]
    assert orc.scale_add(h, sc, col).tolist() == want


@pytest.mark.parametrize("c,ncols", [(1, 1), (4, 3), (10, 2)])
def test_open_queries_from_the_definition(c, ncols):
    """src/pcs.lisp:721-734: the opened leaves are symbols 4l..4l+3 of every codeword (:275-277), the paths the
    siblings up to the cap level (:79-84): numpy indexing, and every opening hashes up to the committed cap."""
    rng = np.random.default_rng(721 + c)
    cols = [rng.integers(0, pf.P, 1 << c, dtype=np.uint32) for _ in range(ncols)]
    cw, levels, cap = orc.commit_columns(cols, c)
    nleaves = 1 << (c - 1)
    idx = np.concatenate([[0, nleaves - 1], rng.integers(0, nleaves, 9)]).astype(np.uint64)
    leaves, paths = orc.open_queries(cw, c, levels, idx)
    depth = orc.cap_level(nleaves)
    assert leaves.shape == (len(idx), ncols, 4) and paths.shape == (len(idx), depth, 32)
    for q, l in enumerate(int(x) for x in idx):
        assert np.array_equal(leaves[q], cw[:, 4 * l:4 * l + 4])
        for lev in range(depth):
            assert np.array_equal(paths[q, lev], levels[lev][(l >> lev) ^ 1])
        assert orc.check_path(orc.leaf_digest(leaves[q]), paths[q], l, cap)
        if depth:  # a path of another leaf does not open this one
            other = (q + 1) % len(idx)
            if (int(idx[other]) >> 1) != (l >> 1):
                assert not orc.check_path(orc.leaf_digest(leaves[q]), paths[other], l, cap)
    no_paths = orc.open_queries(cw, c, None, idx)
    assert np.array_equal(no_paths[0], leaves) and no_paths[1].shape == (len(idx), 0, 32)
