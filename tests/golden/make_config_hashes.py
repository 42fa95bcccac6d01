#!/usr/bin/env python3
"""Writes tests/golden/config_hashes.json: the CPU oracle's proofs of the five configured workloads at their full
sizes, as SHA-256 digests.

The oracle (oracle/, a C restatement of the reference's CPU prover, pinned by the reference's golden vectors) runs
here on its threaded path, which tests/test_oracle_fast.py holds to the plain path's bytes.  The GPU tests compare
the device's proofs of the same seeded inputs with these digests, and where the host has the minutes also with a
fresh oracle run.  Needs no GPU and about 64 GiB of memory at most (config 3: four tables of 2^26).

    python tests/golden/make_config_hashes.py [config1 config2 ...]
"""
import hashlib
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import binding as orc  # noqa: E402
from sable_amd import workloads as wl  # noqa: E402

OUT = os.path.join(HERE, "config_hashes.json")


def sha(b):
    return hashlib.sha256(bytes(b)).hexdigest()


def sumcheck(name, n=None):
    cfg = wl.SUMCHECK[name]
    n, d = n or cfg["n"], cfg["d"]
    st = orc.Statement(cfg["form"], cfg["tables"], cfg["constants"])
    tables = [orc.splitmix_field(wl.table_seed(cfg, k), 1 << n) for k in range(len(cfg["tables"]))]
    eq = orc.splitmix_field(wl.eq_seed(cfg), n * d).reshape(n, d)
    cv = orc.splitmix_field(wl.constants_seed(cfg), d * len(cfg["constants"])).reshape(-1, d) if cfg["constants"] else None
    tr = orc.Transcript(name, d)
    chal, finals, _ = orc.prove(tr, n, st, tables, eq=eq, constants=cv)
    proof = tr.proof()
    return {"n": n, "d": d, "proof_bytes": len(proof), "proof_sha256": sha(proof),
            "finals_sha256": sha(np.ascontiguousarray(finals).tobytes())}


def gkr():
    g = wl.GKR
    d = g["d"]
    z = orc.Transcript(g["z_label"], d).challenge()
    words = orc.splitmix_field(g["seed"], 1 << g["n_witness"])
    wit, tab = wl.gkr_leaves(np, words, z, g["n_witness"], g["n_table"], d)
    out = {"z": [int(x) for x in z]}
    for key, leaves, n, label in (("witness", wit, g["n_witness"], g["witness_label"]),
                                  ("table", tab, g["n_table"], g["table_label"])):
        tr = orc.Transcript(label, d)
        ri, rb, cp, cq = orc.gkr_prove_upper(tr, n, 1, [leaves])
        proof = tr.proof()
        out[key] = {"n": n, "proof_bytes": len(proof), "proof_sha256": sha(proof),
                    "claims_sha256": sha(np.concatenate([ri.reshape(-1), cp.reshape(-1), cq.reshape(-1)]).tobytes())}
    return out


def commit():
    cm = wl.COMMIT
    c, ncols = cm["c"], cm["ncols"]
    flat = orc.splitmix_field(cm["seed"], ncols << c)
    cols = [flat[k << c:(k + 1) << c] for k in range(ncols)]
    codewords, levels, cap = orc.commit_columns(cols, c)
    out = {"c": c, "ncols": ncols, "cap_rows": len(cap), "cap_sha256": sha(np.ascontiguousarray(cap).tobytes()),
           "codewords_sha256": sha(np.ascontiguousarray(codewords).tobytes()),
           "levels_sha256": sha(np.concatenate(levels).tobytes())}
    cf = orc.splitmix_field(cm["coefficient_seed"], ncols * 8).reshape(ncols, 8)
    rr = orc.splitmix_field(cm["point_seed"], c * 8).reshape(c, 8)
    h = orc.combine_columns(np.stack(cols), cf)
    v = orc.mle_eval(h, rr, 8)
    tr = orc.Transcript(cm["open_label"], 4)
    qs, chal, final = orc.basefold_prove(tr, c, rr, v, h, grind_bits=cm["grind_bits"], queries=cm["queries"])
    proof = tr.proof()
    out["basefold"] = {"nv": c, "claim": [int(x) for x in v], "queries": [int(q) for q in qs], "proof_bytes": len(proof),
                       "proof_sha256": sha(proof)}
    return out


def main():
    which = sys.argv[1:] or ["config1", "config2", "config3", "config4", "config5"]
    orc.set_fast(orc.host_threads())
    data = {}
    if os.path.exists(OUT):
        with open(OUT) as f:
            data = json.load(f)
    for name in which:
        t0 = time.perf_counter()
        data[name] = sumcheck(name) if name in wl.SUMCHECK else gkr() if name == "config4" else commit()
        print(f"{name}: {time.perf_counter() - t0:.1f} s", flush=True)
        with open(OUT, "w") as f:
            json.dump(data, f, indent=1, sort_keys=True)
            f.write("\n")


if __name__ == "__main__":
    main()
