"""GPU parity for the final opening over several size classes: combine-columns, BaseFold with classes joining at
later levels, open-queries, and on the host verify-queries; Merkle trees of mixed height.  Through the C ABI
against the CPU oracle, bit for bit, with the forgery checks of tests/tests.lisp:444-462 on the opening."""
import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc

pytestmark = pytest.mark.gpu
P = sa.P


def committed(c, ncols, seed):
    """One class committed on both sides: (device key, oracle key)."""
    cols = sa.Table.random(seed, ncols << c)
    tr = sa.Transcript("open-commit", 4)
    cw, levels = sa.pcs_commit(tr, cols, ncols, c)
    cap = np.frombuffer(orc.decode_proof(tr.proof())[0], np.uint8).reshape(-1, 32)
    coef = orc.splitmix_field(seed + 1, ncols * 8).reshape(ncols, 8)
    flat = orc.splitmix_field(seed, ncols << c)
    host_cols = [flat[k << c:(k + 1) << c] for k in range(ncols)]
    ocw, olevels, ocap = orc.commit_columns(host_cols, c)
    assert np.array_equal(cap, ocap)
    h = orc.combine_columns(np.stack(host_cols), coef)
    dev = {"c": c, "ncols": ncols, "columns": cols, "codewords": cw, "levels": levels, "coef": coef, "cap": cap}
    host = {"c": c, "ncols": ncols, "codewords": ocw, "levels": olevels, "cap": ocap, "coef": coef, "h": h}
    return dev, host


def free(keys):
    for k in keys:
        for name in ("columns", "codewords", "levels"):
            k[name].free()


@pytest.mark.parametrize("classes", [[(9, 2)], [(6, 2), (8, 1), (9, 3)], [(5, 1), (10, 2)], [(8, 70), (9, 1)],
                                     [(5, 1), (6, 1), (7, 1), (8, 1)], [(10, 2), (13, 1), (14, 2)], [(12, 3), (17, 2)]])
def test_opening_matches_the_oracle_and_verifies(classes):
    nv = max(c for c, _ in classes)
    both = [committed(c, ncols, 300 + 10 * c + ncols) for c, ncols in sorted(classes)]
    dev, host = [d for d, _ in both], [h for _, h in both]
    rr = orc.splitmix_field(17 + nv, nv * 8).reshape(nv, 8)
    v = np.zeros(8, np.uint32)
    for key in host:
        v = orc.ext_add(v, orc.mle_eval(key["h"], rr[nv - key["c"]:], 8))
    tr, otr = sa.Transcript("open", 4), orc.Transcript("open", 4)
    qs = sa.pcs_open(tr, nv, dev, rr, v, queries=7)
    want = orc.pcs_open(otr, nv, host, rr, v, queries=7)
    assert qs == want
    assert tr.proof() == otr.proof(), "opening: proof bytes differ from the oracle's"
    # both verifiers accept it, and reject another claim
    vtr = sa.Transcript("open", 4, proof=tr.proof())
    assert sa.pcs_verify_opening(vtr, nv, dev, rr, v, queries=7) and vtr.finished()
    assert orc.pcs_verify_opening(orc.Transcript("open", 4, proof=tr.proof()), nv, host, rr, v, queries=7)
    with pytest.raises(sa.VerificationFailure):
        sa.pcs_verify_opening(sa.Transcript("open", 4, proof=tr.proof()), nv, dev, rr, orc.ext_add(v, orc.base_to_ext(1, 8)),
                              queries=7)
    free(dev)


def test_verify_queries_rejects_every_perturbed_message():
    classes = [(6, 2), (9, 2)]
    nv = 9
    both = [committed(c, ncols, 500 + c) for c, ncols in classes]
    dev, host = [d for d, _ in both], [h for _, h in both]
    rr = orc.splitmix_field(91, nv * 8).reshape(nv, 8)
    v = np.zeros(8, np.uint32)
    for key in host:
        v = orc.ext_add(v, orc.mle_eval(key["h"], rr[nv - key["c"]:], 8))
    tr = sa.Transcript("open", 4)
    sa.pcs_open(tr, nv, dev, rr, v, queries=5)
    msgs = orc.decode_proof(tr.proof())
    hit = 0
    for i, m in enumerate(msgs):
        forged = [x if isinstance(x, bytes) else x.copy() for x in msgs]
        if isinstance(m, bytes):
            if not m:
                continue
            b = bytearray(m)
            b[len(b) // 2] ^= 1  # one path byte, cap byte or nonce bit
            forged[i] = bytes(b)
        else:
            flat = forged[i].reshape(-1)
            flat[len(flat) // 2] = (int(flat[len(flat) // 2]) + 1) % P  # one opened symbol or message word
        with pytest.raises(sa.ExactaError):
            sa.pcs_verify_opening(sa.Transcript("open", 4, proof=orc.encode_messages(forged)), nv, dev, rr, v, queries=5)
        hit += 1
    assert hit >= 10
    bad = [dict(k) for k in dev]
    bad[0]["cap"] = dev[0]["cap"] ^ 1
    with pytest.raises(sa.VerificationFailure):
        sa.pcs_verify_opening(sa.Transcript("open", 4, proof=tr.proof()), nv, bad, rr, v, queries=5)
    bad = [dict(k) for k in dev]
    bad[1]["coef"] = dev[1]["coef"].copy()
    bad[1]["coef"][0, 0] = (int(bad[1]["coef"][0, 0]) + 1) % P
    with pytest.raises(sa.VerificationFailure):
        sa.pcs_verify_opening(sa.Transcript("open", 4, proof=tr.proof()), nv, bad, rr, v, queries=5)
    free(dev)


def test_opening_at_the_configured_size_verifies():
    """nv = 23 with a second class of 2^19: the device's opening is accepted by the host's verify-queries (the
    oracle's prover of this size takes minutes; its verifier takes the device's proof in a second)."""
    classes = [(19, 1), (23, 2)]
    nv = 23
    dev = []
    for c, ncols in classes:
        cols = sa.Table.random(900 + c, ncols << c)
        t = sa.Transcript("open-commit", 4)
        cw, levels = sa.pcs_commit(t, cols, ncols, c)
        cap = np.frombuffer(orc.decode_proof(t.proof())[0], np.uint8).reshape(-1, 32)
        dev.append({"c": c, "ncols": ncols, "columns": cols, "codewords": cw, "levels": levels, "cap": cap,
                    "coef": orc.splitmix_field(901 + c, ncols * 8).reshape(ncols, 8)})
    rr = orc.splitmix_field(77, nv * 8).reshape(nv, 8)
    v = np.zeros(8, np.uint32)
    for key in dev:  # the claim from the device's own combined columns
        g = sa.combine_columns(key["columns"], key["ncols"], key["coef"])
        v = orc.ext_add(v, sa.hypercube_sum(sa.Statement("t0", ["t0"]), key["c"], [g], 8, eq=rr[nv - key["c"]:]))
        g.free()
    tr = sa.Transcript("open", 4)
    qs = sa.pcs_open(tr, nv, dev, rr, v, queries=6)
    assert len(qs) == 6
    vtr = sa.Transcript("open", 4, proof=tr.proof())
    assert sa.pcs_verify_opening(vtr, nv, dev, rr, v, queries=6) and vtr.finished()
    host = [{"c": k["c"], "ncols": k["ncols"], "cap": k["cap"], "coef": k["coef"]} for k in dev]
    assert orc.pcs_verify_opening(orc.Transcript("open", 4, proof=tr.proof()), nv, host, rr, v, queries=6)
    free(dev)


@pytest.mark.parametrize("height,inject_at", [(4, [1]), (6, [1, 3]), (5, [5]), (3, []), (13, [1, 2])])
def test_mixed_height_trees(height, inject_at):
    """merkle-levels with injections on the device against the oracle; every level, and paths that check only with
    the injected digests along them."""
    rng = np.random.default_rng(height)
    n = 1 << height
    # (digests whose words are below p, so that they upload as table values: any 32 bytes hash alike)
    digests = lambda count: (rng.integers(0, 1 << 30, (count, 8), dtype=np.uint32)).astype("<u4").view(np.uint8).reshape(count, 32)
    leaves = digests(n)
    inj = [digests(n >> l) for l in inject_at]
    as_table = lambda d: sa.Table.upload(np.ascontiguousarray(d).view("<u4").reshape(-1, 8))
    tl, ti = as_table(leaves), [as_table(d) for d in inj]
    levels = sa.merkle_levels_injected(tl, dict(zip(inject_at, ti)))
    want = np.concatenate(orc.merkle_levels_injected(leaves, dict(zip(inject_at, inj))))
    got = levels.download().reshape(-1).astype("<u4").view(np.uint8).reshape(-1, 32)
    assert np.array_equal(got, want)
    root = got[-1:]
    for i in (0, n - 1, n // 3):
        path, idx, start, cnt = [], i, 0, n
        for l in range(height):
            path.append(got[start + (idx ^ 1)])
            start += cnt
            cnt //= 2
            idx >>= 1
        at = {l: d[i >> l] for l, d in zip(inject_at, inj)}
        assert sa.check_path(leaves[i], np.array(path).reshape(-1, 32), i, root, at)
        assert orc.check_path_injected(leaves[i], np.array(path).reshape(-1, 32), i, root, at)
        if inject_at:
            assert not sa.check_path(leaves[i], np.array(path).reshape(-1, 32), i, root)
    for t in [tl, levels] + ti:
        t.free()
