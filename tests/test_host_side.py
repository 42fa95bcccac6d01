"""The shipped library's host side, on the CPU: the C-ABI library loads and exports every symbol the
headers declare, and its transcript / proof bytes / forms / verifier agree with the reference's golden
vectors.  No device entry point is called (they need an MI355X and fail loudly without one)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import sable_amd as sa
from oracle import binding as orc
from oracle import forms as oforms

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
hx = bytes.fromhex


def same(a, b):
    return np.array_equal(np.asarray(a, np.uint64), np.asarray(b, np.uint64))


def test_library_exports_every_declared_symbol():
    lib = sa.load()
    declared = set()
    for header in ("exacta_hip.h", "exacta_host.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        declared |= set(re.findall(r"\b(exh_[a-z0-9_]+)\s*\(", text))
    assert len(declared) > 40
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared but not exported"


def test_device_entry_points_fail_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(sa.DeviceError):
        sa.init()
    h = C.c_uint64()
    buf = np.zeros(4, np.uint32)
    assert sa.load().exh_table_upload(buf.ctypes.data_as(sa.u32p), C.c_uint64(4), 1, C.byref(h)) == sa.lib.E_DEVICE


def test_blake3_and_transcript_vectors(vectors):
    for v in vectors("blake3"):
        data = hx(v["input"])
        assert sa.blake3(data) == hx(v["digest"])
        assert sa.blake3(data, 131) == hx(v["xof"])
    for v in vectors("transcript"):
        tr = sa.Transcript(hx(v["label"]), 8)
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
    p = sa.Transcript("pow", 4)
    nonce = p.grind(6)
    v = sa.Transcript("pow", 4, proof=p.proof())
    assert v.verify_grind(6) == nonce and v.finished()
    with pytest.raises(sa.InvalidParameter):
        sa.Transcript("x", 5)


def test_proof_bytes_vectors(vectors):
    for v in vectors("proofio"):
        raw = hx(v["bytes"])
        tr = sa.Transcript("", 4, proof=raw)
        assert tr.proof() == b"EXACTPF1" + raw[8:]
    reasons = {"magic": "magic", "truncated": "truncated", "trailing": "trailing-bytes", "tag": "unknown-tag",
               "range": "value-range", "rank": "rank", "huge": "truncated"}
    for v in vectors("proofio-bad"):
        with pytest.raises(sa.MalformedProof) as e:
            sa.Transcript("", 4, proof=hx(v["bytes"]))
        assert e.value.reason == reasons[v["why"]]


def test_field_helpers_vectors(vectors):
    for v in vectors("ext"):
        assert same(sa.ext_mul(v["a"], v["b"]), v["mul"])
        assert same(sa.ext_inv(v["a"]), v["inv"])
    for v in vectors("mle"):
        assert same(sa.eq_table(np.array(v["r"], np.uint32).reshape(-1, v["d"]), v["d"]), v["eqtab"])
    with pytest.raises(sa.FieldDivisionByZero):
        sa.ext_inv(np.zeros(8, np.uint32))


def test_verifier_on_the_golden_proofs(vectors):
    """tests.lisp:264-276: verify + check-final on the original prover's proofs."""
    for v in vectors("sumcheck"):
        d, nt = v["d"], len(v["tables"])
        names = [f"t{i}" for i in range(nt)]
        st = sa.Statement("(* " + " ".join(names) + ")", names)
        assert st.degree == nt
        tr = sa.Transcript("sc-vec", d, proof=hx(v["proof"]))
        eq = np.array(v["eq_r"], np.uint32) if v["eq_r"] else None
        rho, reduced = sa.verify(tr, v["n"], st, v["claim"], eq=eq)
        assert same(rho, v["rho"]) and same(reduced, v["reduced"])
        assert sa.check_final(reduced, st, v["finals"]) and tr.finished()
        with pytest.raises(sa.VerificationFailure):
            sa.check_final(orc.ext_add(reduced, orc.base_to_ext(1, d)), st, v["finals"])


def test_verifier_rejects_forgeries(vectors):
    """tests.lisp:284-309."""
    v = vectors("sumcheck")[0]
    d, n = v["d"], v["n"]
    st = sa.Statement("(* t0 t1)", ["t0", "t1"])
    proof = hx(v["proof"])

    def run(proof, claim=v["claim"]):
        tr = sa.Transcript("sc-vec", d, proof=proof)
        _, reduced = sa.verify(tr, n, st, claim)
        return sa.check_final(reduced, st, v["finals"])

    assert run(proof)
    with pytest.raises(sa.VerificationFailure):
        run(proof, orc.ext_add(v["claim"], orc.base_to_ext(1, d)))
    for j in range(n):
        msgs = orc.decode_proof(proof)
        msgs[j][0, 1] = (int(msgs[j][0, 1]) + 1) % sa.P
        with pytest.raises(sa.VerificationFailure):
            run(orc.encode_messages(msgs))
    msgs = orc.decode_proof(proof)
    msgs[0] = np.zeros((1, d), np.uint32)
    with pytest.raises(sa.MessageShapeError):
        run(orc.encode_messages(msgs))
    with pytest.raises(sa.TranscriptExhausted):
        run(orc.encode_messages(orc.decode_proof(proof)[:n - 1]))


def test_statement_compile_matches_expand():
    st = sa.Statement("(- (+ (* (+ c0 3) (- c1 c0) c2) 7) (expt c0 2))", ["c0", "c1", "c2"])
    assert st.degree == 3 == oforms.form_degree(oforms.read_form(st.form))
    assert sa.Statement("(* (+ alpha t0) t1 t1)", ["t0", "t1"], ["alpha"]).degree == 3
    with pytest.raises(sa.InvalidParameter):
        sa.Statement("(/ a b)", ["a", "b"])
    with pytest.raises(sa.InvalidParameter):
        sa.Statement("(* a b)", ["a"])
    # check-final evaluates the statement: compare with the oracle's evaluation on random values
    rng = np.random.default_rng(0)
    d = 4
    form = "(+ (* alpha t0 t1 t2) (* 3 t1) -2)"
    st = sa.Statement(form, ["t0", "t1", "t2"], ["alpha"])
    ost = orc.Statement(form, ["t0", "t1", "t2"], ["alpha"])
    tv = rng.integers(0, sa.P, (3, d), dtype=np.uint32)
    cv = rng.integers(0, sa.P, (1, d), dtype=np.uint32)
    assert sa.check_final(ost.evaluate(tv, cv, d), st, tv, constants=cv)
    # a product of linear forms keeps its written shape for the kernels (the generated kernel of the F_p^8
    # configuration is registered under that shape) and evaluates to the same field element
    form = "(* (+ c0 3) (- c1 c0) c2 c3)"
    names = ["c0", "c1", "c2", "c3"]
    st, ost = sa.Statement(form, names), orc.Statement(form, names)
    assert st.has_generated_kernel(8) and not st.has_generated_kernel(4)
    for form, names, cnames in [(form, names, []),
                                ("(- (* (expt (- t0 1) 2) (+ t1 t0)) (* beta (- t1 4) t0))", ["t0", "t1"], ["beta"])]:
        st, ost = sa.Statement(form, names, cnames), orc.Statement(form, names, cnames)
        tv = rng.integers(0, sa.P, (len(names), 8), dtype=np.uint32)
        cv = rng.integers(0, sa.P, (max(len(cnames), 1), 8), dtype=np.uint32)
        assert sa.check_final(ost.evaluate(tv, cv, 8), st, tv, constants=cv if cnames else None)


def test_gkr_layer_statements_have_build_time_kernels():
    """LAYER-STATEMENT (src/gkr.lisp:30-41) for one to three lookups, and (* bw statement) for the sumcheck over the
    block index, as the library forms them: each has kernels generated at build time for F_p^4 (a statement without
    them runs on the interpreter kernels, several times slower)."""
    for lookups in (1, 2, 3):
        tables, constants, terms = [], [], []
        for l in range(lookups):
            tables += ["P0-%d" % l, "P1-%d" % l, "Q0-%d" % l, "Q1-%d" % l]
            constants += ["A%d" % l, "AL%d" % l]
            terms += ["(* A%d P0-%d Q1-%d)" % (l, l, l), "(* A%d P1-%d Q0-%d)" % (l, l, l), "(* AL%d Q0-%d Q1-%d)" % (l, l, l)]
        form = "(+ " + " ".join(terms) + ")"
        assert sa.Statement(form, tables, constants).has_generated_kernel(4), lookups
        assert sa.Statement("(* BW " + form + ")", ["BW"] + tables, constants).has_generated_kernel(4), lookups


def test_point_reduction_statements_have_build_time_kernels():
    """REDUCE-POINTS' statement (src/pcs.lisp:344-347) for one to four points, as an opening forms it."""
    for points in (1, 2, 3, 4):
        names = [n for i in range(points) for n in ("E%d" % i, "G%d" % i)]
        form = "(+ " + " ".join("(* E%d G%d)" % (i, i) for i in range(points)) + ")"
        assert sa.Statement(form, names).has_generated_kernel(4), points


def test_the_bench_constants_go_with_the_present_kernel_sources():
    """bench.py reports measured traffic and multiply counts only for the version of the kernels they were measured
    on: the stamp has to be renewed (with the figures) when the kernels' sources change."""
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert bench.MEASURED["kernel_sources_sha256"] == bench.kernel_sources_sha256()
