"""GPU parity for LogUp-GKR: layer reductions and prove-upper through the C ABI against the CPU oracle
(bit-exact), with the reference's semantic checks (tests/tests.lisp:414-462)."""
import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc

pytestmark = pytest.mark.gpu
P = sa.P


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


def random_leaves(rng, lookups, n, k, d):
    out = []
    for _ in range(lookups):
        p = rng.integers(0, P, (k << n, d), dtype=np.uint32)
        q = rng.integers(0, P, (k << n, d), dtype=np.uint32)
        q[:, 0] |= 1
        out.append((p, q))
    return out


@pytest.mark.parametrize("d,k,m", [(4, 1, 0), (4, 1, 9), (8, 3, 4), (4, 5, 11)])
def test_reduce_layer(d, k, m):
    rng = np.random.default_rng(m + k)
    p = rng.integers(0, P, (k << (m + 1), d), dtype=np.uint32)
    q = rng.integers(0, P, (k << (m + 1), d), dtype=np.uint32)
    tp, tq = sa.Table.upload(p), sa.Table.upload(q)
    op, oq = sa.gkr_reduce_layer(tp, tq, d, k, m)
    wp, wq = orc.gkr_reduce_layer(p, q, k, m)
    assert same(op.download(), wp) and same(oq.download(), wq)
    for t in (tp, tq, op, oq):
        t.free()


CASES = [(3, 1, 1, 4), (3, 3, 2, 4), (2, 4, 1, 8), (4, 5, 2, 4), (1, 2, 1, 4), (1, 1, 2, 8), (2, 2, 3, 4),
         (10, 1, 1, 4), (6, 1, 2, 8),
         # several blocks at sizes where the layers' sumchecks run on the device-driven loop, the top tree on the
         # chain and the folded tables stay on the device for the sumcheck over the block index
         (9, 3, 1, 4), (8, 2, 2, 4), (7, 6, 1, 8), (11, 4, 3, 4),
         # one block: the layers chained on the device (up to twelve base challenges per layer), from the smallest
         # tree that chains to one whose upper layers take the grid of slices
         (2, 1, 1, 4), (5, 1, 2, 4), (7, 1, 1, 8), (13, 1, 1, 4), (12, 1, 2, 4), (6, 1, 3, 4), (11, 1, 3, 4),
         # statements of many tables in F_p^8: few pairs fit the one-workgroup launch, and the rounds just above it
         # go to two workgroups' slices
         (9, 1, 3, 8), (10, 1, 2, 8), (8, 3, 2, 8)]


@pytest.mark.parametrize("n,k,lookups,d", CASES)
def test_prove_upper_matches_the_oracle(n, k, lookups, d):
    rng = np.random.default_rng(n + k + lookups + d)
    leaves = random_leaves(rng, lookups, n, k, d)
    dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
    tr, otr = sa.Transcript("gkr-test", d), orc.Transcript("gkr-test", d)
    got = sa.prove_upper(tr, n, k, dev)
    want = orc.gkr_prove_upper(otr, n, k, leaves)
    assert tr.proof() == otr.proof()
    for a, b in zip(got, want):
        assert same(a, b)
    # the library's verifier accepts, and agrees with the prover's outputs
    vtr = sa.Transcript("gkr-test", d, proof=tr.proof())
    roots, ri, rb, cp, cq = sa.verify_upper(vtr, n, k, lookups)
    assert vtr.finished()
    for a, b in zip((ri, rb, cp, cq), got):
        assert same(a, b)
    # LogUp: each root is the sum of its leaf fractions
    for (p, q), root in zip(leaves, roots):
        total = np.zeros(d, np.uint32)
        for a, b in zip(p[:64], q[:64]) if n > 8 else zip(p, q):
            total = orc.ext_add(total, orc.ext_mul(a, orc.ext_inv(b)))
        if n <= 8:
            assert same(orc.ext_mul(root[0], orc.ext_inv(root[1])), total)
    for p, q in dev:
        p.free(), q.free()


@pytest.mark.parametrize("n,k,lookups,d", [(12, 3, 1, 4), (11, 5, 2, 4), (10, 3, 3, 4), (10, 6, 1, 8), (9, 12, 1, 4)])
def test_several_blocks_on_the_grid_of_slices_and_on_the_streaming_rounds(n, k, lookups, d, monkeypatch):
    """Tables of K 2^m entries (K not a power of two) take the grid of LDS-resident slices with a multiple of K's odd
    part of workgroups; with the switch they stay on the streaming rounds.  Both are the oracle's proof."""
    rng = np.random.default_rng(7 * n + k)
    leaves = random_leaves(rng, lookups, n, k, d)
    dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
    otr = orc.Transcript("gkr-blocks", d)
    want = orc.gkr_prove_upper(otr, n, k, leaves)
    # (and with the older ways of moving a layer's constants and logs: a copy on the stream before the set-up launch,
    # the folded tables fetched with the logs)
    for switches in ({}, {"EXACTA_HIP_NO_BLOCK_SLICES": "1"}, {"EXACTA_HIP_COPY_CONSTANTS": "1"},
                     {"EXACTA_HIP_FETCH_FINALS": "1"}):
        for name in ("EXACTA_HIP_NO_BLOCK_SLICES", "EXACTA_HIP_COPY_CONSTANTS", "EXACTA_HIP_FETCH_FINALS"):
            monkeypatch.setenv(name, switches.get(name, "0"))
        tr = sa.Transcript("gkr-blocks", d)
        got = sa.prove_upper(tr, n, k, dev)
        assert tr.proof() == otr.proof(), switches
        for a, b in zip(got, want):
            assert same(a, b)
    for p, q in dev:
        p.free(), q.free()


@pytest.mark.parametrize("n,lookups,d", [(9, 1, 4), (6, 2, 4), (8, 1, 8), (7, 3, 4)])
def test_the_chained_layers_and_the_host_driven_layers_send_the_same_bytes(n, lookups, d, monkeypatch):
    rng = np.random.default_rng(100 + n)
    leaves = random_leaves(rng, lookups, n, 1, d)
    dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
    chained = sa.Transcript("gkr-test", d)
    got = sa.prove_upper(chained, n, 1, dev)
    monkeypatch.setenv("EXACTA_HIP_NO_GKR_CHAIN", "1")
    driven = sa.Transcript("gkr-test", d)
    want = sa.prove_upper(driven, n, 1, dev)
    assert chained.proof() == driven.proof() and chained.state_digest() == driven.state_digest()
    for a, b in zip(got, want):
        assert same(a, b)
    for p, q in dev:
        p.free(), q.free()


# two trees side by side (a second host thread, stream and workspace): each proof's bytes, outputs and final
# transcript state are those of the call on its own; pairs of different sizes, both chained, one host-driven
# (several blocks), both large enough for the grids of slices that must share the device
PAIRS = [((13, 1, 1, 4), (9, 1, 1, 4)), ((16, 1, 1, 4), (15, 1, 2, 4)), ((6, 3, 2, 4), (12, 1, 1, 4)),
         ((7, 1, 1, 8), (3, 1, 1, 4)), ((17, 1, 1, 4), (17, 1, 1, 4))]


@pytest.mark.parametrize("first,second", PAIRS)
def test_two_trees_side_by_side_are_the_two_single_calls(first, second):
    rng = np.random.default_rng(sum(first) + 3 * sum(second))
    calls, alone = [], []
    for which, (n, k, lookups, d) in enumerate((first, second)):
        leaves = random_leaves(rng, lookups, n, k, d)
        dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
        label = "tree-%d" % which
        tr = sa.Transcript(label, d)
        alone.append((tr, sa.prove_upper(tr, n, k, dev)))
        calls.append((sa.Transcript(label, d), n, k, dev))
    for _ in range(2):  # (the second time with the side context's buffers already there)
        fresh = [(sa.Transcript("tree-%d" % which, c[0].degree),) + c[1:] for which, c in enumerate(calls)]
        outs = sa.prove_upper_pair(fresh[0], fresh[1])
        for (tr, want), call, got in zip(alone, fresh, outs):
            assert call[0].proof() == tr.proof()
            for a, b in zip(got, want):
                assert same(a, b)
    # the transcripts go on identically after the proofs
    a = sa.Transcript("tree-0", calls[0][0].degree)
    b = sa.Transcript("tree-0", calls[0][0].degree)
    sa.prove_upper(a, *calls[0][1:])
    sa.prove_upper_pair((b,) + calls[0][1:], (sa.Transcript("tree-1", calls[1][0].degree),) + calls[1][1:])
    assert same(a.challenge(), b.challenge())
    for c in calls:
        for p, q in c[3]:
            p.free(), q.free()


def test_a_pair_needs_two_transcripts():
    rng = np.random.default_rng(5)
    leaves = random_leaves(rng, 1, 3, 1, 4)
    dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
    tr = sa.Transcript("gkr-test", 4)
    with pytest.raises(sa.ExactaError):
        sa.prove_upper_pair((tr, 3, 1, dev), (tr, 3, 1, dev))


def test_verify_upper_rejects_forgeries():
    n, k, lookups, d = 3, 3, 2, 4
    rng = np.random.default_rng(9)
    leaves = random_leaves(rng, lookups, n, k, d)
    dev = [(sa.Table.upload(p), sa.Table.upload(q)) for p, q in leaves]
    tr = sa.Transcript("gkr-test", d)
    sa.prove_upper(tr, n, k, dev)
    msgs = orc.decode_proof(tr.proof())
    for i, m in enumerate(msgs):
        if isinstance(m, bytes):
            continue
        forged = [x if isinstance(x, bytes) else x.copy() for x in msgs]
        forged[i].reshape(-1)[0] = (int(forged[i].reshape(-1)[0]) + 1) % P
        with pytest.raises(sa.VerificationFailure):
            sa.verify_upper(sa.Transcript("gkr-test", d, proof=orc.encode_messages(forged)), n, k, lookups)


def test_logup_lookup_argument_small():
    """A lookup argument of the configured shape, small: 2^10 lookups of int8-range values into a 2^8-entry
    range table with exact multiplicities; the witness and table trees' root fractions are equal."""
    d, nw, nt = 4, 10, 8
    rng = np.random.default_rng(4)
    values = rng.integers(-128, 128, 1 << nw)
    table = np.arange(-128, 128)
    mult = np.array([(values == t).sum() for t in table])
    tr = sa.Transcript("logup", d)
    z = tr.challenge()
    lift = lambda x: np.concatenate([np.asarray(x, np.int64)[:, None] % P, np.zeros((len(x), d - 1), np.int64)], 1)
    zq = lambda v: (z.astype(np.int64)[None, :] - lift(v)) % P
    wit = (lift(np.ones(1 << nw, np.int64)).astype(np.uint32), zq(values).astype(np.uint32))
    tab = (lift(mult).astype(np.uint32), zq(table).astype(np.uint32))
    roots = []
    for (p, q), n in ((wit, nw), (tab, nt)):
        dev = (sa.Table.upload(p), sa.Table.upload(q))
        t = sa.Transcript("logup-tree", d)
        sa.prove_upper(t, n, 1, [dev])
        r = orc.decode_proof(t.proof())[0]
        roots.append(orc.ext_mul(r[0], orc.ext_inv(r[1])))
        dev[0].free(), dev[1].free()
    assert same(roots[0], roots[1])
