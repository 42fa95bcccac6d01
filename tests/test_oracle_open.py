"""The oracle's final opening over several size classes (oracle/orc_open.c): BaseFold with classes joining at later
levels, open-queries, verify-queries and Merkle trees of mixed height (src/pcs.lisp:64-95, 581-657, 721-843).
Its BaseFold over classes and its trees with injections are pinned by the reference's frozen commitment cases
(tests/test_oracle_frozen_cases.py); the opening as a whole and the verifier are held here to what the protocol
itself fixes: the verifier accepts the prover's proof, rejects every perturbed opening, and the
single-class case is the one-class prover byte for byte."""
import numpy as np
import pytest

from oracle import binding as orc

P = orc.P


def committed_class(c, ncols, seed):
    flat = orc.splitmix_field(seed, ncols << c)
    cols = [flat[k << c:(k + 1) << c] for k in range(ncols)]
    cw, levels, cap = orc.commit_columns(cols, c)
    coef = orc.splitmix_field(seed + 1, ncols * 8).reshape(ncols, 8)
    h = orc.combine_columns(np.stack(cols), coef)
    return {"c": c, "ncols": ncols, "codewords": cw, "levels": levels, "cap": cap, "coef": coef, "h": h}


def opening(classes, seed=1, queries=5):
    nv = max(c for c, _ in classes)
    keys = [committed_class(c, ncols, 100 * seed + c) for c, ncols in sorted(classes)]
    rr = orc.splitmix_field(seed + 7, nv * 8).reshape(nv, 8)
    v = np.zeros(8, np.uint32)
    for key in keys:  # the claim: sum_c H_c at the last c coordinates of the point
        v = orc.ext_add(v, orc.mle_eval(key["h"], rr[nv - key["c"]:], 8))
    tr = orc.Transcript("open", 4)
    qs = orc.pcs_open(tr, nv, keys, rr, v, queries=queries)
    return nv, keys, rr, v, tr.proof(), qs


@pytest.mark.parametrize("classes", [[(7, 2)], [(9, 1)], [(6, 2), (8, 1), (9, 3)], [(5, 1), (10, 2)], [(8, 70), (9, 1)],
                                     [(5, 1), (6, 1), (7, 1), (8, 1)]])
def test_verifier_accepts_the_opening(classes):
    nv, keys, rr, v, proof, qs = opening(classes)
    assert len(qs) == 5 and all(q < 1 << (nv - 1) for q in qs)
    vtr = orc.Transcript("open", 4, proof=proof)
    assert orc.pcs_verify_opening(vtr, nv, keys, rr, v, queries=5) and vtr.finished()
    with pytest.raises(orc.VerificationFailure):
        orc.pcs_verify_opening(orc.Transcript("open", 4, proof=proof), nv, keys, rr, orc.ext_add(v, orc.base_to_ext(1, 8)),
                               queries=5)


def test_single_class_is_the_one_class_prover():
    """With one class of size nv the loop is orc_basefold_prove's, message for message, before the keys' openings."""
    nv, keys, rr, v, proof, qs = opening([(9, 2)])
    otr = orc.Transcript("open", 4)
    want_qs, _, _ = orc.basefold_prove(otr, nv, rr, v, keys[0]["h"], queries=5)
    one = orc.decode_proof(otr.proof())
    many = orc.decode_proof(proof)
    assert qs == want_qs and len(many) == len(one) + 2
    for a, b in zip(one, many):
        assert (a == b) if isinstance(a, bytes) else np.array_equal(a, b)


def test_every_perturbed_message_is_rejected():
    """tests.lisp:444-462's pattern on the opening: one word or byte of any message changed, and the verifier
    rejects (a sumcheck round, an oracle cap, the final table, the nonce, an opened symbol, a path byte)."""
    nv, keys, rr, v, proof, qs = opening([(6, 2), (9, 2)], seed=3)
    msgs = orc.decode_proof(proof)
    hit = 0
    for i, m in enumerate(msgs):
        forged = [x if isinstance(x, bytes) else x.copy() for x in msgs]
        if isinstance(m, bytes):
            if not m:
                continue
            b = bytearray(m)
            b[len(b) // 2] ^= 1
            forged[i] = bytes(b)
        else:
            flat = forged[i].reshape(-1)
            flat[len(flat) // 2] = (int(flat[len(flat) // 2]) + 1) % P
        with pytest.raises((orc.VerificationFailure, orc.OracleError)):
            orc.pcs_verify_opening(orc.Transcript("open", 4, proof=orc.encode_messages(forged)), nv, keys, rr, v, queries=5)
        hit += 1
    assert hit >= 10
    # and a wrong committed cap, or wrong coefficients, on the verifier's side
    bad = [dict(k) for k in keys]
    bad[0]["cap"] = keys[0]["cap"] ^ 1  # every cap entry: the queries reach only a few of them
    with pytest.raises(orc.VerificationFailure):
        orc.pcs_verify_opening(orc.Transcript("open", 4, proof=proof), nv, bad, rr, v, queries=5)
    bad = [dict(k) for k in keys]
    bad[1]["coef"] = keys[1]["coef"].copy()
    bad[1]["coef"][0, 0] = (int(bad[1]["coef"][0, 0]) + 1) % P
    with pytest.raises(orc.VerificationFailure):
        orc.pcs_verify_opening(orc.Transcript("open", 4, proof=proof), nv, bad, rr, v, queries=5)


def python_levels(leaves, injections):
    """merkle-levels by its definition (src/pcs.lisp:64-77) on top of the hash alone."""
    level, levels, l = [bytes(x) for x in leaves], [], 1
    while True:
        levels.append(level)
        if len(level) == 1:
            return levels
        level = [orc.blake3(level[i] + level[i + 1]) for i in range(0, len(level), 2)]
        if l in injections:
            level = [orc.blake3(a + bytes(b)) for a, b in zip(level, injections[l])]
        l += 1


@pytest.mark.parametrize("height,inject_at", [(4, [1]), (6, [1, 3]), (5, [5]), (3, [])])
def test_mixed_height_trees_against_the_definition(height, inject_at):
    rng = np.random.default_rng(height)
    n = 1 << height
    leaves = rng.integers(0, 256, (n, 32), dtype=np.uint8)
    injections = {l: rng.integers(0, 256, (n >> l, 32), dtype=np.uint8) for l in inject_at}
    got = orc.merkle_levels_injected(leaves, injections)
    want = python_levels(leaves, injections)
    assert len(got) == len(want) == height + 1
    for a, b in zip(got, want):
        assert [bytes(x) for x in a] == b
    # every leaf's path checks against the root with the digests injected along it, and not without them
    for i in (0, 1, n // 2, n - 1):
        path, idx = [], i
        for l in range(height):
            path.append(got[l][idx ^ 1])
            idx >>= 1
        at = {l: injections[l][i >> l] for l in inject_at}
        assert orc.check_path_injected(leaves[i], np.array(path).reshape(-1, 32), i, got[-1], at)
        if inject_at:
            assert not orc.check_path_injected(leaves[i], np.array(path).reshape(-1, 32), i, got[-1], {})
