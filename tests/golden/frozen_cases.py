"""The case files behind the reference's *FROZEN-CASES* (tests/tests.lisp:902-925), rebuilt as text: the inputs
from SBCL's seeded generator (sbcl_random.py), the proofs from whichever prover is handed in (the oracle's or the
device's), the JSON laid out as EXPORT-GKR-CASES (tests/tests.lisp:464-483) and EXPORT-DOMAIN-CASES
(tests/tests.lisp:587-624) write it.  The reference pins the SHA-256 of each file; its removed C++ and Python
verifiers accepted exactly these proofs."""
import numpy as np

from sbcl_random import SbclRandom

P = 2130706433
# tests/tests.lisp:903-904
GKR_SHA256 = "100cba9c4c818c1d2bb79467fe807ed3f7f7054274b5331cb7c22f78bd538320"
DOMAIN_SHA256 = "7a53788916a303f668251d4e05b22085efcb4d57813bc58a0f93e7f214cbcf12"


def _ints(a):
    return "[" + ",".join(str(int(v)) for v in np.asarray(a).reshape(-1)) + "]"


def _exts(es):
    return "[" + ",".join(_ints(e) for e in es) + "]"


# ------------------------------------------------------------------ LogUp-GKR
GKR_CASES = [(3, 1, 1, 4), (3, 3, 2, 4), (2, 4, 1, 8), (4, 5, 2, 4), (1, 2, 1, 4), (1, 1, 2, 8), (2, 2, 3, 4), (5, 6, 2, 8)]


def random_leaves(lookups, n, k, d, state):
    """RANDOM-LEAVES (tests/tests.lisp:399-406): per lookup the numerators, then the (nonzero) denominators."""
    def ext(nonzero=False):
        while True:
            e = [state.random(P) for _ in range(d)]
            if not (nonzero and not any(e)):
                return e
    return [(np.array([ext() for _ in range(k << n)], np.uint32), np.array([ext(True) for _ in range(k << n)], np.uint32))
            for _ in range(lookups)]


def gkr_cases_text(prove, verify):
    """prove(n, k, leaves, d) -> proof bytes of PROVE-UPPER on a transcript labelled "gkr-test";
    verify(proof, n, k, lookups, d) -> (roots, ri, rb, cp, cq) of VERIFY-UPPER."""
    out = ["[\n"]
    for i, (n, k, lookups, d) in enumerate(GKR_CASES):
        leaves = random_leaves(lookups, n, k, d, SbclRandom(7 * (n + k + lookups + d)))
        proof = prove(n, k, leaves, d)
        roots, ri, rb, cp, cq = verify(proof, n, k, lookups, d)
        out.append('{"n": %d, "K": %d, "L": %d, "D": %d, "label": "gkr-test", "proof": "%s", "roots": %s, "ri": %s, '
                   '"rb": %s, "cp": %s, "cq": %s}%s\n' % (n, k, lookups, d, proof.hex(), _ints(roots), _ints(ri), _ints(rb),
                                                          _ints(cp), _ints(cq), "," if i + 1 < len(GKR_CASES) else ""))
    out.append("]\n")
    return "".join(out)


# ------------------------------------------------------------------ domains
DOMAIN_CASES = [dict(n=3, k=3), dict(n=2, k=1), dict(n=3, k=3, merge=True), dict(n=4, k=4, merge=True),
                dict(n=3, k=2, lookups=False), dict(n=3, k=2, constraints=False), dict(n=4, k=5, merge=True), dict(n=3, k=5)]
_CONSTRAINTS = '[["*","a",["-","a",1]],["-","c",["*","a","b"]],["*","s",["-","s",1],"m"]]'
_LOOKUPS = ('{"tag": 5, "values": ["a","b"], "num": null},{"tag": 7, "values": ["c","m","w"], "num": ["+","s",2]},'
            '{"tag": 9, "values": ["kb"], "num": null}')


def toy_domain(Domain, Column, state, n=3, k=3, merge=False, lookups=True, constraints=True):
    """TOY-DOMAIN (tests/tests.lisp:487-512), its columns drawn in the reference's order."""
    size = 1 << n
    a = np.array([state.random(2) for _ in range(k * size)], np.uint64)
    b = np.array([state.random(P) for _ in range(k * size)], np.uint64)
    c = a * b % P
    m = np.array([state.random(P) for _ in range(size // 2)], np.uint64)
    s = np.array([state.random(2) for _ in range(size)], np.uint64)
    kb = np.array([state.random(P) for _ in range(k)], np.uint64)
    w = np.array([state.random(P) for _ in range(4 * k)], np.uint64)
    cols = [Column("a", data=a), Column("b", data=b), Column("c", data=c), Column("m", "row", 1, True, m),
            Column("s", "col", n, True, s), Column("kb", "row", n, False, kb), Column("w", "col", 2, False, w)]
    return Domain("12.toy-merged" if merge else "12.toy", n, cols, blocks=k, merge=merge,
                  constraints=["(* a (- a 1))", "(- c (* a b))", "(* s (- s 1) m)"] if constraints else [],
                  lookups=[{"tag": 5, "values": ["a", "b"]}, {"tag": 7, "values": ["c", "m", "w"], "num": "(+ s 2)"},
                           {"tag": 9, "values": ["kb"]}] if lookups else [])


def domain_cases_text(Domain, Column, prove, verify):
    """prove(domain, d, z, betas) -> proof bytes of PROVE-DOMAIN on a transcript labelled "dom-test";
    verify(proof, domain, d, z, betas) -> (claims, roots) of VERIFY-DOMAIN."""
    out = ["[\n"]
    for i, case in enumerate(DOMAIN_CASES):
        for d in (4, 8):
            state = SbclRandom(d + 3 * case["n"] + case["k"])
            dom = toy_domain(Domain, Column, state, **case)
            z = np.array([state.random(P) for _ in range(d)], np.uint32)  # LOOKUP-CHALLENGES, tests/tests.lisp:514-516
            betas = np.array([[state.random(P) for _ in range(d)] for _ in range(8)], np.uint32)
            proof = prove(dom, d, z, betas)
            claims, roots = verify(proof, dom, d, z, betas)
            columns = ",".join('{"name": "%s", "kind": "%s", "c": %d, "shared": %s}'
                               % (col.name.lower(), col.kind, col.c, "true" if col.shared else "false") for col in dom.columns)
            claimed = ",".join('"%s": {"point": %s, "value": %s}'
                               % (name.lower(), _exts(point), _exts([value]) if np.asarray(value).ndim == 1 else _exts(value))
                               for name, point, value in claims)
            out.append('{"name": "%s", "n": %d, "K": %d, "merge": %s, "D": %d, "label": "dom-test", "columns": [%s], '
                       '"constraints": %s, "lookups": [%s], "Z": %s, "beta": %s, "proof": "%s", "roots": [%s], '
                       '"claims": {%s}}%s\n'
                       % (dom.name, case["n"], case["k"], "true" if case.get("merge") else "false", d, columns,
                          _CONSTRAINTS if case.get("constraints", True) else "[]",
                          _LOOKUPS if case.get("lookups", True) else "", _ints(z), _exts(betas), proof.hex(),
                          ",".join("[%s,%s]" % (_ints(p), _ints(q)) for p, q in roots), claimed,
                          "," if (i + 1 < len(DOMAIN_CASES) or d != 8) else ""))
    out.append("]\n")
    return "".join(out)
