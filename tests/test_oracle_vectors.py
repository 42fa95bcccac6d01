"""The CPU oracle against the reference's golden vectors (known-answer tests written by Sable's
original Python implementation; the reference's own suite checks the same vectors in
tests/tests.lisp:45-282)."""
import numpy as np
import pytest

from oracle import binding as orc
from oracle import forms

P = orc.P
hx = bytes.fromhex


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


# ------------------------------------------------------------------ field (tests.lisp:45-82)
def test_field_tower(vectors):
    assert P - 1 == (1 << 24) * 127
    assert orc.fpow(3, (P - 1) // 2) == P - 1          # 3 is a non-residue
    z = np.zeros(8, np.uint32); z[4] = 1               # z^8 = 3 (check-tower, field.lisp:379-387)
    acc = orc.base_to_ext(1, 8)
    for _ in range(8):
        acc = orc.ext_mul(acc, z)
    assert same(acc, orc.base_to_ext(3, 8))
    for v in vectors("pow"):
        assert orc.fpow(v["a"], v["e"]) == v["res"]
    for v in vectors("ext"):
        a, b = v["a"], v["b"]
        assert same(orc.ext_add(a, b), v["add"])
        assert same(orc.ext_sub(a, b), v["sub"])
        assert same(orc.ext_mul(a, b), v["mul"])
        assert same(orc.ext_inv(a), v["inv"])
        assert same(orc.ext_eq1(a, b), v["eq1"])


def test_field_multilinear(vectors):
    for v in vectors("lagrange"):
        assert same(orc.lagrange(v["vals"], v["x"]), v["res"])
    for v in vectors("eq"):
        d = v["d"]
        a = np.array(v["a"], np.uint32).reshape(-1, d)
        b = np.array(v["b"], np.uint32).reshape(-1, d)
        assert same(orc.ext_eq(a, b, d), v["res"])
    for v in vectors("mle"):
        d = v["d"]
        r = np.array(v["r"], np.uint32).reshape(-1, d)
        assert same(orc.eq_table(r, d), v["eqtab"])
        assert same(orc.mle_eval(np.array(v["base"], np.uint32), r, d), v["base_res"])
        assert same(orc.mle_eval(np.array(v["ext"], np.uint32).reshape(-1, d), r, d), v["ext_res"])


def test_field_inverse_of_zero():
    with pytest.raises(orc.OracleError):
        orc.finv(0)
    with pytest.raises(orc.OracleError):
        orc.ext_inv(np.zeros(8, np.uint32))
    rng = np.random.default_rng(7)
    for d in (4, 8):
        a = rng.integers(0, P, d, dtype=np.uint32)
        assert same(orc.ext_mul(a, orc.ext_inv(a)), orc.base_to_ext(1, d))


def test_ext_mul_is_polynomial_multiplication():
    """Independent of the vectors: tower order is the bit-reversed power basis of F_p[w]/(w^D - 3)."""
    rng = np.random.default_rng(1)
    for d in (4, 8):
        bits = d.bit_length() - 1
        rev = [int(format(i, f"0{bits}b")[::-1], 2) for i in range(d)]
        for _ in range(20):
            a = [int(x) for x in rng.integers(0, P, d)]
            b = [int(x) for x in rng.integers(0, P, d)]
            pa = [a[rev[e]] for e in range(d)]
            pb = [b[rev[e]] for e in range(d)]
            c = [0] * d
            for i in range(d):
                for j in range(d):
                    if i + j < d:
                        c[i + j] = (c[i + j] + pa[i] * pb[j]) % P
                    else:
                        c[i + j - d] = (c[i + j - d] + 3 * pa[i] * pb[j]) % P
            assert same(orc.ext_mul(a, b), [c[rev[i]] for i in range(d)])


# ------------------------------------------------------------------ forms (tests.lisp:104-138)
def test_forms_against_python(vectors):
    form = forms.read_form("(- (+ (* (+ c0 3) (- c1 c0) c2) 7) (expt c0 2))")
    names = ["C0", "C1", "C2"]
    values = {"C0": 11, "C1": P - 5, "C2": 1 << 30}
    for v in vectors("poly"):
        expected = sorted(((tuple(names[i] for i in ids), c) for ids, c in v["terms"]),
                          key=lambda t: (len(t[0]), t[0]))
        assert forms.expand(form) == expected
        total = 0
        for m, c in forms.expand(form):
            term = c
            for name in m:
                term = term * values[name] % P
            total = (total + term) % P
        assert total == v["eval"] == forms.evaluate_base(form, values)
        assert forms.form_degree(form) == v["degree"]
        assert forms.form_variables(form) == [names[i] for i in v["vars"]]
        assert forms.constant_term(form) == v["const"]


def test_forms_as_data():
    assert forms.expand(forms.read_form("(* (+ a 1) (- a 1))")) == [((), P - 1), (("A", "A"), 1)]
    assert forms.expand(forms.read_form("(- (* 2 x) x x)")) == []
    assert forms.form_degree(forms.read_form("(* (+ alpha t0) t1 t1)"), ["T0", "T1"]) == 3
    with pytest.raises(ValueError):
        forms.expand(forms.read_form("(/ a b)"))


# ------------------------------------------------------------------ hashes and transcript (tests.lisp:142-184)
def test_blake3_standard(vectors):
    for v in vectors("blake3"):
        data = hx(v["input"])
        assert orc.blake3(data) == hx(v["digest"])
        assert orc.blake3(data, 131) == hx(v["xof"])


def test_blake3_sequential(vectors):
    for v in vectors("b3s"):
        s = orc.B3S.new()
        for c in v["chunks"]:
            s.update(hx(c))
        assert s.digest(32) == hx(v["digest"])
        assert s.digest(200) == hx(v["xof"])


def test_transcript_replay(vectors):
    for v in vectors("transcript"):
        tr = orc.Transcript(hx(v["label"]), 8)
        for op in v["ops"]:
            kind, args = op[0], op[1:]
            if kind == "absorb":
                tr.absorb(hx(args[0]))
            elif kind == "absorb-ext":
                tr.absorb(np.array(args[0], np.uint32).astype("<u4").tobytes())
            elif kind == "challenge-base":
                assert same(tr.challenge_base(args[0]), args[1])
            elif kind == "challenge":
                assert same(tr.challenge(args[0]), args[1])
            elif kind == "challenge-bits":
                assert tr.challenge_bits(args[0], args[1]) == args[2]
            elif kind == "digest":
                assert tr.state_digest() == hx(args[0])
            else:
                raise AssertionError(f"unknown transcript op {kind}")
    for v in vectors("grind"):
        assert orc.check_grind(hx(v["base"]), v["nonce"], v["bits"]) == bool(v["ok"])


def test_transcript_grind_roundtrip():
    p = orc.Transcript("pow", 4)
    nonce = p.grind(6)
    v = orc.Transcript("pow", 4, proof=p.proof())
    assert v.verify_grind(6) == nonce and v.finished()
    with pytest.raises(orc.OracleError):
        orc.Transcript("x", 5)


# ------------------------------------------------------------------ proof bytes (tests.lisp:210-236)
def as_written(octets):
    return b"EXACTPF1" + octets[8:] if octets[:8] == b"SABLEPF1" else octets


def test_proofio_roundtrip(vectors):
    for v in vectors("proofio"):
        raw = hx(v["bytes"])
        parsed = orc.decode_proof(raw)
        assert len(parsed) == len(v["msgs"])
        for m, spec in zip(parsed, v["msgs"]):
            if spec[0] == "bytes":
                assert m == hx(spec[1])
            else:
                assert list(m.shape) == spec[1]
                assert same(m.reshape(-1), spec[2])
        assert orc.encode_messages(parsed) == as_written(raw)


def test_proofio_rejects_malformed(vectors):
    reasons = {"magic": "magic", "truncated": "truncated", "trailing": "trailing", "tag": "tag",
               "range": "range", "rank": "rank", "huge": "truncated"}
    for v in vectors("proofio-bad"):
        with pytest.raises(orc.MalformedProof) as e:
            orc.decode_proof(hx(v["bytes"]))
        assert e.value.reason == reasons[v["why"]]


# ------------------------------------------------------------------ Reed-Solomon (tests.lisp:240-251)
def test_reed_solomon(vectors):
    for v in vectors("rs-encode"):
        n = v["n"]
        assert orc.root_of_unity(n) == v["root"]
        assert same(orc.domain_points(n), v["points"])
        tw = orc.twiddles(n)
        assert len(tw) == len(v["tw"])
        for a, b in zip(tw, v["tw"]):
            assert same(a, b)
        assert same(orc.rs_encode(v["msg"], n), v["cw"])
        assert same(orc.rs_brute_eval(v["msg"], n), v["cw"])
    for v in vectors("rs-fold"):
        out = orc.rs_fold(np.array(v["cw"], np.uint32), orc.twiddles(v["n"])[0], v["r"])
        assert same(out, v["res"])
    with pytest.raises(orc.OracleError):
        orc.root_of_unity(30)


# ------------------------------------------------------------------ sumcheck (tests.lisp:255-282)
def sumcheck_case(v):
    d, nt = v["d"], len(v["tables"])
    names = [f"T{i}" for i in range(nt)]
    st = orc.Statement(["*"] + names, names)
    return dict(d=d, n=v["n"], st=st, claim=np.array(v["claim"], np.uint32), proof=hx(v["proof"]),
                rho=v["rho"], reduced=v["reduced"],
                eq=np.array(v["eq_r"], np.uint32) if v["eq_r"] else None,
                tables=[np.array(t, np.uint32) for t in v["tables"]],
                finals=np.array(v["finals"], np.uint32))


def test_sumcheck_against_python(vectors):
    for v in vectors("sumcheck"):
        c = sumcheck_case(v)
        # the verifier on the Python prover's proof
        tr = orc.Transcript("sc-vec", c["d"], proof=c["proof"])
        vrho, vreduced = orc.verify(tr, c["n"], c["st"], c["claim"], eq=c["eq"])
        assert same(vrho, c["rho"]) and same(vreduced, c["reduced"])
        assert orc.check_final(vreduced, c["st"], c["finals"])
        assert tr.finished()
        # the prover writes the same bytes as the Python prover, after the magic
        tr = orc.Transcript("sc-vec", c["d"])
        assert same(orc.hypercube_sum(c["st"], c["n"], c["tables"], c["d"], eq=c["eq"]), c["claim"])
        prho, pfinals, _ = orc.prove(tr, c["n"], c["st"], c["tables"], eq=c["eq"])
        assert same(prho, c["rho"]) and same(pfinals, c["finals"])
        assert tr.proof() == as_written(c["proof"])


def test_sumcheck_rejects_forgeries(vectors):
    c = sumcheck_case(vectors("sumcheck")[0])

    def run(proof, claim=c["claim"]):
        tr = orc.Transcript("sc-vec", c["d"], proof=proof)
        _, reduced = orc.verify(tr, c["n"], c["st"], claim)
        return orc.check_final(reduced, c["st"], c["finals"])

    assert run(c["proof"])
    with pytest.raises(orc.VerificationFailure):
        run(c["proof"], orc.ext_add(c["claim"], orc.base_to_ext(1, c["d"])))
    for j in range(c["n"]):
        msgs = orc.decode_proof(c["proof"])
        msgs[j][0, 1] = (int(msgs[j][0, 1]) + 1) % P
        with pytest.raises(orc.VerificationFailure):
            run(orc.encode_messages(msgs))
    msgs = orc.decode_proof(c["proof"])
    msgs[0] = np.zeros((1, c["d"]), np.uint32)
    with pytest.raises(orc.MessageShapeError):
        run(orc.encode_messages(msgs))
    msgs[0] = bytes(4)
    with pytest.raises(orc.MessageShapeError):
        run(orc.encode_messages(msgs))
    with pytest.raises(orc.TranscriptExhausted):
        run(orc.encode_messages(orc.decode_proof(c["proof"])[:c["n"] - 1]))
