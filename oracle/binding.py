"""ctypes binding of the CPU oracle (oracle/liborc.so).  TEST INFRASTRUCTURE ONLY: imported by
tests/, the smoke check and the benchmark's cpu_baseline leg; never by the shipped library.

All field data are numpy uint32 arrays of canonical residues; an EXT is a row of D words.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from . import forms

P = 2130706433
HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liborc.so")

OK, E_PARAM, E_DIVZERO, E_SHAPE, E_EXHAUSTED, E_REJECT, E_MALFORMED = 0, -1, -2, -3, -4, -5, -6
MALFORMED_REASONS = {1: "magic", 2: "truncated", 3: "trailing", 4: "tag", 5: "range", 6: "rank", 7: "dimension"}


class OracleError(Exception):
    def __init__(self, status, what=""):
        self.status = status
        super().__init__(f"oracle status {status} {what}")


class VerificationFailure(OracleError):
    pass


class MessageShapeError(OracleError):
    pass


class TranscriptExhausted(OracleError):
    pass


class MalformedProof(OracleError):
    def __init__(self, status, reason):
        super().__init__(status, reason)
        self.reason = reason


def build():
    subprocess.check_call(["make", "-s", "-C", HERE])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _declare(_lib)
    return _lib


u32p = C.POINTER(C.c_uint32)
u8p = C.POINTER(C.c_uint8)
u64p = C.POINTER(C.c_uint64)
i32p = C.POINTER(C.c_int32)


class Stmt(C.Structure):
    _fields_ = [("T", C.c_int), ("C", C.c_int), ("nterms", C.c_int), ("coeff", u32p), ("start", i32p),
                ("vars", i32p), ("nops", C.c_int), ("ops", i32p), ("args", i32p)]


class Msg(C.Structure):
    _fields_ = [("kind", C.c_int), ("rank", C.c_int), ("dims", C.c_uint64 * 8), ("count", C.c_uint64),
                ("bytes", u8p), ("vals", u32p)]


def _declare(l):
    l.orc_fadd.restype = l.orc_fsub.restype = l.orc_fmul.restype = l.orc_fpow.restype = C.c_uint32
    l.orc_fadd.argtypes = l.orc_fsub.argtypes = l.orc_fmul.argtypes = [C.c_uint32, C.c_uint32]
    l.orc_fpow.argtypes = [C.c_uint32, C.c_uint64]
    l.orc_tr_new.restype = C.c_void_p
    l.orc_tr_new.argtypes = [C.c_char_p, C.c_uint64, C.c_int]
    l.orc_tr_new_verifier.restype = C.c_void_p
    l.orc_tr_new_verifier.argtypes = [C.c_char_p, C.c_uint64, C.c_int, C.c_char_p, C.c_uint64, C.POINTER(C.c_int)]
    l.orc_tr_free.argtypes = [C.c_void_p]
    l.orc_tr_message.restype = C.POINTER(Msg)
    l.orc_tr_message.argtypes = [C.c_void_p, C.c_uint64]
    l.orc_tr_message_count.restype = C.c_uint64
    l.orc_tr_message_count.argtypes = [C.c_void_p]
    l.orc_tr_encode_proof.restype = C.c_uint64
    l.orc_tr_encode_proof.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
    l.orc_tr_grind.restype = C.c_uint64
    l.orc_tr_grind.argtypes = [C.c_void_p, C.c_int]
    l.orc_twiddles_size.restype = C.c_uint64
    l.orc_commit_columns.restype = C.c_uint64
    for name in ("orc_tr_absorb", "orc_tr_send", "orc_tr_record", "orc_tr_send_bytes", "orc_tr_record_bytes",
                 "orc_tr_squeeze", "orc_tr_challenge_base", "orc_tr_challenge", "orc_tr_challenges",
                 "orc_tr_challenge_bits", "orc_tr_verify_grind", "orc_tr_state_digest", "orc_tr_finished",
                 "orc_tr_degree"):
        getattr(l, name).argtypes = None


def _u32(a):
    if isinstance(a, np.ndarray) and a.dtype == np.uint32 and a.flags.c_contiguous and a.size > (1 << 16):
        return a  # a large table already in the wire type (its values are residues by construction)
    a = np.asarray(a, dtype=np.uint64)
    out = np.empty(a.shape, np.uint32)  # keeps rank 0 (ascontiguousarray would not)
    out[...] = a % P
    return out


def _p(a):
    return a.ctypes.data_as(u32p) if a is not None else None


def _check(status, what=""):
    if status == OK:
        return
    if status == E_REJECT:
        raise VerificationFailure(status, what)
    if status == E_SHAPE:
        raise MessageShapeError(status, what)
    if status == E_EXHAUSTED:
        raise TranscriptExhausted(status, what)
    if status == E_MALFORMED:
        raise MalformedProof(status, MALFORMED_REASONS.get(lib().orc_malformed_reason(), "?"))
    raise OracleError(status, what)


# ------------------------------------------------------------------ field
def fadd(a, b): return lib().orc_fadd(a % P, b % P)
def fsub(a, b): return lib().orc_fsub(a % P, b % P)
def fmul(a, b): return lib().orc_fmul(a % P, b % P)
def fpow(a, e): return lib().orc_fpow(a % P, e)


def finv(a):
    out = C.c_uint32()
    _check(lib().orc_finv(C.c_uint32(a % P), C.byref(out)), "finv")
    return out.value


def _ext2(name, a, b):
    a, b = _u32(a), _u32(b)
    out = np.zeros_like(a)
    getattr(lib(), name)(len(a), _p(a), _p(b), _p(out))
    return out


def ext_add(a, b): return _ext2("orc_ext_add", a, b)
def ext_sub(a, b): return _ext2("orc_ext_sub", a, b)
def ext_mul(a, b): return _ext2("orc_ext_mul", a, b)
def ext_eq1(a, b): return _ext2("orc_ext_eq1", a, b)


def ext_scale(a, s):
    a = _u32(a)
    out = np.zeros_like(a)
    lib().orc_ext_scale(len(a), _p(a), C.c_uint32(s % P), _p(out))
    return out


def ext_inv(a):
    a = _u32(a)
    out = np.zeros_like(a)
    _check(lib().orc_ext_inv(len(a), _p(a), _p(out)), "ext-inv")
    return out


def ext_eq(as_, bs, d):
    as_, bs = _u32(as_).reshape(-1, d), _u32(bs).reshape(-1, d)
    out = np.zeros(d, np.uint32)
    lib().orc_ext_eq(d, len(as_), _p(as_), _p(bs), _p(out))
    return out


def base_to_ext(x, d):
    out = np.zeros(d, np.uint32)
    out[0] = x % P
    return out


def lagrange(values, x):
    values, x = _u32(values), _u32(x)
    out = np.zeros_like(x)
    lib().orc_lagrange(len(x), len(values), _p(values), _p(x), _p(out))
    return out


def eq_table(r, d):
    r = _u32(r).reshape(-1, d)
    out = np.zeros((1 << len(r), d), np.uint32)
    lib().orc_eq_table(d, len(r), _p(r), _p(out))
    return out


def fold_table(table, r):
    table, r = _u32(table), _u32(r)
    out = np.zeros((len(table) // 2, len(r)), np.uint32)
    lib().orc_fold_table(len(r), C.c_uint64(len(table)), _p(table), _p(r), _p(out))
    return out


def mle_eval(values, r, d):
    values = _u32(values)
    r = _u32(r).reshape(-1, d)
    assert len(values) == 1 << len(r)
    out = np.zeros(d, np.uint32)
    lib().orc_mle_eval(d, len(r), _p(values), 1 if values.ndim == 1 else d, _p(r), _p(out))
    return out


# ------------------------------------------------------------------ hashes
def blake3(data, n=32):
    out = (C.c_uint8 * n)()
    lib().orc_blake3_hash(C.c_char_p(bytes(data)), C.c_uint64(len(data)), out, C.c_uint64(n))
    return bytes(out)


class B3S(C.Structure):
    _fields_ = [("cv", C.c_uint32 * 8), ("block", C.c_uint8 * 64), ("used", C.c_uint32), ("counter", C.c_uint64)]

    @classmethod
    def new(cls, data=b""):
        s = cls()
        lib().orc_b3s_init(C.byref(s))
        return s.update(data)

    def update(self, data):
        lib().orc_b3s_update(C.byref(self), C.c_char_p(bytes(data)), C.c_uint64(len(data)))
        return self

    def digest(self, n=32):
        out = (C.c_uint8 * n)()
        lib().orc_b3s_digest(C.byref(self), out, C.c_uint64(n))
        return bytes(out)


# ------------------------------------------------------------------ transcript
def _label(label):
    return label.encode() if isinstance(label, str) else bytes(label)


class Transcript:
    """make-transcript (src/transcript.lisp:75-84): a prover transcript, or with `proof` a verifier
    transcript replaying the proof's messages."""

    def __init__(self, label, degree, proof=None):
        label = _label(label)
        if proof is None:
            self.h = lib().orc_tr_new(label, len(label), degree)
            if not self.h:
                raise OracleError(E_PARAM, "degree")
        else:
            st = C.c_int()
            self.h = lib().orc_tr_new_verifier(label, len(label), degree, bytes(proof), len(proof), C.byref(st))
            if not self.h:
                _check(st.value, "decode-proof")
        self.h = C.c_void_p(self.h)
        self.degree = degree

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_tr_free(self.h)
            self.h = None

    def absorb(self, data):
        data = _label(data)
        lib().orc_tr_absorb(self.h, C.c_char_p(data), C.c_uint64(len(data)))

    def _field(self, fn, value, shape):
        if value is not None:
            a = _u32(value)
            dims = (C.c_uint64 * 8)(*a.shape)
            _check(fn(self.h, _p(a), a.ndim, dims, None))
            return a
        if shape is None:
            raise ValueError("a verifier passes the shape it expects")
        out = np.zeros(shape, np.uint32)
        dims = (C.c_uint64 * 8)(*shape)
        _check(fn(self.h, None, len(shape), dims, _p(out)))
        return out

    def send(self, value=None, shape=None): return self._field(lib().orc_tr_send, value, shape)
    def record(self, value=None, shape=None): return self._field(lib().orc_tr_record, value, shape)

    def _bytes(self, fn, value, length):
        if value is not None:
            value = bytes(value)
            _check(fn(self.h, C.c_char_p(value), C.c_int64(len(value)), None, C.c_uint64(0), None))
            return value
        n = C.c_uint64()
        cap = 1 << 24
        out = (C.c_uint8 * cap)()
        _check(fn(self.h, None, C.c_int64(-1 if length is None else length), out, C.c_uint64(cap), C.byref(n)))
        return bytes(out[:n.value])

    def send_bytes(self, value=None, length=None): return self._bytes(lib().orc_tr_send_bytes, value, length)
    def record_bytes(self, value=None, length=None): return self._bytes(lib().orc_tr_record_bytes, value, length)

    def challenge_base(self, k):
        out = np.zeros(k, np.uint32)
        lib().orc_tr_challenge_base(self.h, k, _p(out))
        return out

    def challenge(self, degree=None):
        return self.challenge_base(degree or self.degree)

    def challenges(self, k, degree=None):
        d = degree or self.degree
        return self.challenge_base(d * k).reshape(k, d)

    def challenge_bits(self, nbits, k):
        out = np.zeros(k, np.uint64)
        lib().orc_tr_challenge_bits(self.h, nbits, k, out.ctypes.data_as(u64p))
        return [int(x) for x in out]

    def grind(self, bits): return lib().orc_tr_grind(self.h, bits)

    def verify_grind(self, bits):
        nonce = C.c_uint64()
        _check(lib().orc_tr_verify_grind(self.h, bits, C.byref(nonce)), "proof-of-work")
        return nonce.value

    def state_digest(self):
        out = (C.c_uint8 * 32)()
        lib().orc_tr_state_digest(self.h, out)
        return bytes(out)

    def finished(self): return bool(lib().orc_tr_finished(self.h))

    def messages(self):
        out = []
        for i in range(lib().orc_tr_message_count(self.h)):
            m = lib().orc_tr_message(self.h, i).contents
            if m.kind == 0:
                out.append(bytes(m.bytes[:m.count]))
            else:
                shape = tuple(m.dims[k] for k in range(m.rank))
                out.append(np.ctypeslib.as_array(m.vals, shape=(m.count,)).copy().reshape(shape)
                           if m.count else np.zeros(shape, np.uint32))
        return out

    def proof(self):
        n = lib().orc_tr_encode_proof(self.h, None, 0)
        out = (C.c_uint8 * n)()
        lib().orc_tr_encode_proof(self.h, out, n)
        return bytes(out)


def check_grind(base, nonce, bits):
    return bool(lib().orc_check_grind(C.c_char_p(bytes(base)), C.c_uint64(nonce), bits))


def encode_messages(messages):
    """encode-proof (src/proofio.lisp:45-49) of a list of bytes / arrays."""
    tr = Transcript("", 4)
    for m in messages:
        if isinstance(m, (bytes, bytearray)):
            tr.record_bytes(m)
        else:
            tr.record(m)
    return tr.proof()


def decode_proof(proof):
    return Transcript("", 4, proof=proof).messages()


# ------------------------------------------------------------------ Reed-Solomon
def root_of_unity(k):
    out = C.c_uint32()
    _check(lib().orc_root_of_unity(k, C.byref(out)), "root-of-unity")
    return out.value


def twiddles(n):
    flat = np.zeros(lib().orc_twiddles_size(n), np.uint32)
    lib().orc_twiddles(n, _p(flat))
    levels, pos, length = [], 0, 1 << (n - 1)
    for _ in range(max(1, n - 1)):
        levels.append(flat[pos:pos + length].copy())
        pos += length
        length //= 2
    return levels


def domain_points(n):
    out = np.zeros(1 << n, np.uint32)
    lib().orc_domain_points(n, _p(out))
    return out


def rs_encode(message, n):
    m = _u32(message)
    assert len(m) == 1 << (n - 1)
    out = np.zeros(1 << n, np.uint32)
    _check(lib().orc_rs_encode(_p(m), n, _p(out)), "encode")
    return out


def rs_brute_eval(message, n):
    m = _u32(message)
    out = np.zeros(1 << n, np.uint32)
    lib().orc_rs_brute_eval(_p(m), n, _p(out))
    return out


def rs_fold(codeword, twiddle_level, r):
    cw, tw, r = _u32(codeword), _u32(twiddle_level), _u32(r)
    d = 1 if cw.ndim == 1 else cw.shape[1]
    m = len(cw) // 2
    out = np.zeros((m, d) if d > 1 else m, np.uint32)
    lib().orc_rs_fold(d, C.c_uint64(m), _p(cw), _p(tw), _p(r), _p(out))
    return out


def dot_pairs(e, v):
    """dot-pairs (src/pcs.lisp:473-483) of two tables of EXT8s for the parities 0, 1, 2: (3, 8)."""
    e, v = _u32(e), _u32(v)
    out = np.zeros((3, 8), np.uint32)
    for parity in range(3):
        lib().orc_dot_pairs(_p(e), _p(v), C.c_uint64(len(e)), parity, _p(out[parity]))
    return out


def scale_add(h, scale, column):
    """h + scale * column over extension tables (src/pcs.lisp:709-716): a new array."""
    h, scale, column = _u32(h).copy(), _u32(scale), _u32(column)
    lib().orc_scale_add(len(scale), C.c_uint64(len(h)), _p(scale), _p(column), _p(h))
    return h


def open_queries(codewords, c, levels, leaves):
    """open-queries' data for one (unit, class) (src/pcs.lisp:721-734): codewords (ncols, 2^(c+1)); levels: the
    bytes of all levels, leaves first, or None -> (leaves (Q, ncols, 4), paths (Q, depth, 32) bytes)."""
    cw = _u32(codewords)
    ncols = cw.shape[0]
    idx = np.ascontiguousarray(leaves, np.uint64)
    depth = cap_level(1 << (c - 1)) if levels is not None else 0
    out = np.zeros((len(idx), ncols, 4), np.uint32)
    paths = np.zeros((len(idx), depth, 32), np.uint8)
    lv = None
    if levels is not None:  # a list of levels (as commit_columns returns them) or their bytes
        lv = (np.concatenate([np.ascontiguousarray(l, np.uint8).reshape(-1) for l in levels])
              if isinstance(levels, (list, tuple)) else np.frombuffer(bytes(levels), np.uint8).copy())
    got = lib().orc_open_queries(_p(cw), ncols, c, lv.ctypes.data_as(C.c_void_p) if lv is not None else None,
                                 idx.ctypes.data_as(C.c_void_p), len(idx), _p(out), paths.ctypes.data_as(C.c_void_p))
    assert got == depth
    return out, paths


def combine_columns(columns, coefficients):
    """combine-columns (src/pcs.lisp:434-441): columns (ncols, len) base values, coefficients (ncols, D)."""
    cols, cf = _u32(columns), _u32(coefficients)
    ncols, length = cols.shape
    d = cf.shape[1]
    out = np.zeros((length, d), np.uint32)
    lib().orc_combine_columns(d, ncols, C.c_uint64(length), _p(cols), _p(cf), _p(out))
    return out


# ------------------------------------------------------------------ statements and sumcheck
def _postfix(form, index, n_tables):
    """The form as written, as the postfix program of orc.h's orc_stmt: what ARITHMETIC-FORM emits
    (src/forms.lisp:113-141), n-ary chains reduced left to right, (expt b k) as k - 1 products of b."""
    ops, args = [], []

    def emit(op, arg=0):
        ops.append(op)
        args.append(arg)

    def chain(op, arguments, empty):
        if not arguments:
            emit(2, empty)
            return
        walk(arguments[0])
        for a in arguments[1:]:
            walk(a)
            emit(op)

    def walk(f):
        if isinstance(f, bool):
            raise ValueError("malformed form")
        if isinstance(f, int):
            emit(2, f % P)
        elif isinstance(f, str):
            v = index[f.upper()]
            emit(0, v) if v < n_tables else emit(1, v - n_tables)
        elif isinstance(f, (list, tuple)) and f:
            op, arguments = f[0], list(f[1:])
            if op == "+":
                chain(3, arguments, 0)
            elif op == "*":
                chain(5, arguments, 1)
            elif op == "-":
                if not arguments:
                    raise ValueError("malformed form")
                if len(arguments) == 1:
                    walk(arguments[0])
                    emit(6)
                else:
                    chain(4, arguments, 0)
            elif op in ("expt", "EXPT"):
                base, k = arguments
                if not isinstance(k, int) or k < 0:
                    raise ValueError("malformed form")
                chain(5, [base] * k, 1)
            else:
                raise ValueError("malformed form")
        else:
            raise ValueError("malformed form: %r" % (f,))

    walk(form)
    return ops, args


def set_fast(threads):
    """threads > 0: orc_sumcheck_prove (and the provers built on it) run the threaded straight-line path of
    orc_fast.c; 0: the plain restatement (the default, the one the golden proofs pin).  Same bytes either way."""
    lib().orc_set_fast(int(threads))


def host_threads():
    return lib().orc_host_threads()


def splitmix_field(seed, count):
    """The seeded synthetic field elements of the benchmarks (exh_table_random's rule) on the host."""
    out = np.empty(count, np.uint32)
    lib().orc_splitmix_field(C.c_uint64(seed), C.c_uint64(count), _p(out))
    return out


def ext_mul_plain(a, b):
    a, b = _u32(a), _u32(b)
    out = np.zeros_like(a)
    lib().orc_ext_mul_plain(len(a), _p(a), _p(b), _p(out))
    return out


def round_sums_fast(st, d, points, tables, low, high, constants=None, threads=1):
    arrs, strides, ptrs = _tables(tables, d)
    low, high = _u32(low).reshape(-1, d), _u32(high).reshape(-1, d)
    ca = _u32(constants).reshape(-1, d) if constants is not None and len(constants) else np.zeros((1, d), np.uint32)
    out = np.zeros((points, d), np.uint32)
    _check(lib().orc_round_sums_fast(C.byref(st.c), d, points, C.c_uint64(len(low)), C.c_uint64(len(high)), ptrs,
                                     strides.ctypes.data_as(i32p), _p(low), _p(high), _p(ca), threads, _p(out)))
    return out


class Statement:
    """A statement form with its table and constant variables fixed: the oracle's monomial IR."""

    def __init__(self, form, tables, constants=()):
        self.form = forms.read_form(form) if isinstance(form, str) and form.strip().startswith("(") else (
            form.upper() if isinstance(form, str) else form)
        self.tables = [t.upper() for t in tables]
        self.constants = [c.upper() for c in constants]
        index = {v: i for i, v in enumerate(self.tables + self.constants)}
        terms = forms.expand(self.form)
        coeff, start, vs = [], [0], []
        for m, c in terms:
            coeff.append(c)
            vs.extend(index[v] for v in m)
            start.append(len(vs))
        self._coeff = np.array(coeff, np.uint32)
        self._start = np.array(start, np.int32)
        self._vars = np.array(vs if vs else [0], np.int32)
        ops, args = _postfix(self.form, index, len(self.tables))
        self._ops, self._args = np.array(ops, np.int32), np.array(args, np.int32)
        self.c = Stmt(len(self.tables), len(self.constants), len(coeff), _p(self._coeff),
                      self._start.ctypes.data_as(i32p), self._vars.ctypes.data_as(i32p), len(ops),
                      self._ops.ctypes.data_as(i32p), self._args.ctypes.data_as(i32p))
        self.degree = lib().orc_stmt_degree(C.byref(self.c))

    def evaluate(self, table_values, constants, d):
        tv = _u32(table_values).reshape(-1, d)
        cv = _u32(constants).reshape(-1, d) if len(self.constants) else np.zeros((1, d), np.uint32)
        out = np.zeros(d, np.uint32)
        lib().orc_stmt_eval(C.byref(self.c), d, _p(tv), _p(cv), _p(out))
        return out


def _tables(tables, d):
    arrs = [_u32(t) for t in tables]
    strides = np.array([1 if a.ndim == 1 else d for a in arrs], np.int32)
    ptrs = (u32p * len(arrs))(*[_p(a) for a in arrs])
    return arrs, strides, ptrs


def hypercube_sum(st, n, tables, d, eq=None, constants=None):
    arrs, strides, ptrs = _tables(tables, d)
    eqa = _u32(eq).reshape(-1, d) if eq is not None else None
    ca = _u32(constants).reshape(-1, d) if constants is not None and len(constants) else np.zeros((1, d), np.uint32)
    out = np.zeros(d, np.uint32)
    lib().orc_hypercube_sum(C.byref(st.c), n, d, ptrs, strides.ctypes.data_as(i32p), _p(eqa), _p(ca), _p(out))
    return out


def prove(tr, n, st, tables, eq=None, constants=None, label="sc", block_weights=None, degree=None):
    """prove (src/sumcheck.lisp:512-571): returns (challenges (n,D), finals (T,D), folded [T x (K,D)])."""
    d = tr.degree
    arrs, strides, ptrs = _tables(tables, d)
    eqa = _u32(eq).reshape(-1, d) if eq is not None else None
    ca = _u32(constants).reshape(-1, d) if constants is not None and len(constants) else np.zeros((1, d), np.uint32)
    bw = _u32(block_weights).reshape(-1, d) if block_weights is not None else None
    K = len(bw) if bw is not None else 1
    for a, s in zip(arrs, strides):
        assert a.size == (K << n) * s, "table size"
    chal = np.zeros((n, d), np.uint32)
    finals = np.zeros((len(arrs), d), np.uint32)
    folded = [np.zeros((K, d), np.uint32) for _ in arrs]
    fptrs = (u32p * len(arrs))(*[_p(a) for a in folded])
    label = _label(label)
    _check(lib().orc_sumcheck_prove(tr.h, n, C.byref(st.c), ptrs, strides.ctypes.data_as(i32p), _p(eqa), _p(ca),
                                    C.c_char_p(label), C.c_uint64(len(label)), _p(bw), K,
                                    -1 if degree is None else degree, _p(chal), _p(finals), fptrs), "prove")
    return chal, finals, folded


def verify(tr, n, st, claim, eq=None, constants=None, blocks=1, label="sc", degree=None):
    """verify (src/sumcheck.lisp:147-163): returns (challenges, reduced claim)."""
    d = tr.degree
    eqa = _u32(eq).reshape(-1, d) if eq is not None else None
    ca = _u32(constants).reshape(-1, d) if constants is not None and len(constants) else np.zeros((1, d), np.uint32)
    claim = _u32(claim)
    chal = np.zeros((n, d), np.uint32)
    reduced = np.zeros(d, np.uint32)
    label = _label(label)
    _check(lib().orc_sumcheck_verify(tr.h, n, C.byref(st.c), _p(claim), _p(eqa), _p(ca), blocks, C.c_char_p(label),
                                     C.c_uint64(len(label)), -1 if degree is None else degree, _p(chal),
                                     _p(reduced)), "verify")
    return chal, reduced


def check_final(reduced, st, finals, constants=None):
    d = len(reduced)
    ca = _u32(constants).reshape(-1, d) if constants is not None and len(constants) else np.zeros((1, d), np.uint32)
    f = _u32(finals).reshape(-1, d)
    r = _u32(reduced)
    _check(lib().orc_check_final(C.byref(st.c), d, _p(r), _p(f), _p(ca)), "sumcheck-final")
    return True


def round_sums(st, d, points, tables, low, high, constants=None):
    arrs, strides, ptrs = _tables(tables, d)
    low, high = _u32(low).reshape(-1, d), _u32(high).reshape(-1, d)
    ca = _u32(constants).reshape(-1, d) if constants is not None and len(constants) else np.zeros((1, d), np.uint32)
    out = np.zeros((points, d), np.uint32)
    lib().orc_round_sums(C.byref(st.c), d, points, C.c_uint64(len(low)), C.c_uint64(len(high)), ptrs,
                         strides.ctypes.data_as(i32p), _p(low), _p(high), _p(ca), _p(out))
    return out


def fold_flat(entries, r):
    e, r = _u32(entries), _u32(r)
    d = len(r)
    stride = 1 if e.ndim == 1 else d
    n = e.size // stride
    out = np.zeros((n // 2, d), np.uint32)
    lib().orc_fold_flat(d, C.c_uint64(n), _p(e), stride, _p(r), _p(out))
    return out


# ------------------------------------------------------------------ GKR
def _block_bits(k):
    return (k - 1).bit_length()


def gkr_prove_upper(tr, n, k, leaves, label="gkr"):
    """prove-upper (src/gkr.lisp:215-272).  leaves: per lookup (p, q), arrays (K*2^n, D)."""
    d = tr.degree
    flat = []
    for p, q in leaves:
        flat += [_u32(p).reshape(-1, d), _u32(q).reshape(-1, d)]
    ptrs = (u32p * len(flat))(*[_p(a) for a in flat])
    L, lk = len(leaves), _block_bits(k)
    ri = np.zeros((max(n - 1, 0), d), np.uint32)
    rb = np.zeros((lk, d), np.uint32)
    cp, cq = np.zeros((L, d), np.uint32), np.zeros((L, d), np.uint32)
    label = _label(label)
    _check(lib().orc_gkr_prove_upper(tr.h, n, k, L, ptrs, C.c_char_p(label), C.c_uint64(len(label)), _p(ri), _p(rb),
                                     _p(cp), _p(cq)), "prove-upper")
    return ri, rb, cp, cq


def gkr_verify_upper(tr, n, k, lookups, label="gkr"):
    d = tr.degree
    lk = _block_bits(k)
    roots = np.zeros((lookups, 2, d), np.uint32)
    ri = np.zeros((max(n - 1, 0), d), np.uint32)
    rb = np.zeros((lk, d), np.uint32)
    cp, cq = np.zeros((lookups, d), np.uint32), np.zeros((lookups, d), np.uint32)
    label = _label(label)
    _check(lib().orc_gkr_verify_upper(tr.h, n, k, lookups, C.c_char_p(label), C.c_uint64(len(label)), _p(roots),
                                      _p(ri), _p(rb), _p(cp), _p(cq)), "verify-upper")
    return roots, ri, rb, cp, cq


def gkr_reduce_layer(p, q, k, m):
    p, q = _u32(p), _u32(q)
    d = p.shape[1]
    pp, qq = np.zeros((k << m, d), np.uint32), np.zeros((k << m, d), np.uint32)
    lib().orc_gkr_reduce_layer(d, k, m, _p(p), _p(q), _p(pp), _p(qq))
    return pp, qq


# ------------------------------------------------------------------ commitment
def leaf_digest(rows, previous=None):
    rows = _u32(rows).reshape(-1, 4)
    out = (C.c_uint8 * 32)()
    lib().orc_leaf_digest(_p(rows), C.c_uint64(len(rows)), C.c_char_p(previous) if previous else None, out)
    return bytes(out)


def node(left, right):
    out = (C.c_uint8 * 32)()
    lib().orc_node(C.c_char_p(left), C.c_char_p(right), out)
    return bytes(out)


def cap_level(leaves): return lib().orc_cap_level(C.c_uint64(leaves))


def merkle_levels(leaves):
    """leaves: (n, 32) uint8 -> list of levels, leaves first."""
    leaves = np.ascontiguousarray(leaves, np.uint8).reshape(-1, 32)
    n = len(leaves)
    out = np.zeros((2 * n - 1, 32), np.uint8)
    lib().orc_merkle_levels(leaves.ctypes.data_as(u8p), C.c_uint64(n), out.ctypes.data_as(u8p))
    levels, pos = [], 0
    while n >= 1:
        levels.append(out[pos:pos + n].copy())
        pos += n
        n //= 2
    return levels


def check_path(h, path, i, cap):
    path = np.ascontiguousarray(path, np.uint8).reshape(-1, 32)
    cap = np.ascontiguousarray(cap, np.uint8).reshape(-1, 32)
    return bool(lib().orc_check_path(C.c_char_p(bytes(h)), path.ctypes.data_as(u8p), len(path), C.c_uint64(i),
                                     cap.ctypes.data_as(u8p)))


def commit_columns(columns, c):
    """pcs-commit of one class (src/pcs.lisp:279-304): returns (codewords, levels, cap)."""
    cols = [_u32(col) for col in columns]
    for col in cols:
        assert len(col) == 1 << c
    ptrs = (u32p * len(cols))(*[_p(a) for a in cols])
    cw = np.zeros((len(cols), 1 << (c + 1)), np.uint32)
    nleaves = 1 << (c - 1)
    levels = np.zeros((2 * nleaves - 1, 32), np.uint8)
    cap = np.zeros((nleaves, 32), np.uint8)
    rows = lib().orc_commit_columns(ptrs, len(cols), c, _p(cw), levels.ctypes.data_as(u8p), cap.ctypes.data_as(u8p))
    out_levels, pos, n = [], 0, nleaves
    while n >= 1:
        out_levels.append(levels[pos:pos + n].copy())
        pos += n
        n //= 2
    return cw, out_levels, cap[:rows].copy()


def basefold_prove(tr, nv, rr, v, h, grind_bits=4, queries=6):
    rr, v, h = _u32(rr).reshape(-1, 8), _u32(v), _u32(h).reshape(-1, 8)
    assert len(h) == 1 << nv and len(rr) == nv
    fl = max(0, nv - 5)
    qs = np.zeros(queries, np.uint64)
    chal = np.zeros((max(fl, 1), 8), np.uint32)
    final = np.zeros((1 << (nv - fl), 8), np.uint32)
    _check(lib().orc_basefold_prove(tr.h, nv, _p(rr), _p(v), _p(h), grind_bits, queries, qs.ctypes.data_as(u64p),
                                    _p(chal), _p(final)), "basefold")
    return [int(q) for q in qs], chal[:fl], final


def basefold_verify(tr, nv, rr, v, grind_bits=4, queries=6):
    rr, v = _u32(rr).reshape(-1, 8), _u32(v)
    qs = np.zeros(queries, np.uint64)
    _check(lib().orc_basefold_verify(tr.h, nv, _p(rr), _p(v), grind_bits, queries, qs.ctypes.data_as(u64p)),
           "basefold")
    return [int(q) for q in qs]


# ------------------------------------------------------------------ the opening over several classes (orc_open.c)
class OpenKey(C.Structure):
    _fields_ = [("c", C.c_int32), ("ncols", C.c_int32), ("codewords", u32p), ("levels", u8p), ("cap", u8p),
                ("coef", u32p), ("h", u32p)]


def merkle_levels_injected(leaves, injections):
    """merkle-levels with injections (src/pcs.lisp:64-77): injections = {level: digests}; a list of levels."""
    lv = np.ascontiguousarray(leaves, np.uint8).reshape(-1, 32)
    n = len(lv)
    levels = sorted(injections)
    arrs = [np.ascontiguousarray(injections[l], np.uint8).reshape(-1, 32) for l in levels]
    ptrs = (u8p * max(len(arrs), 1))(*[a.ctypes.data_as(u8p) for a in arrs])
    lvl = np.array(levels if levels else [0], np.int32)
    out = np.zeros((2 * n - 1, 32), np.uint8)
    lib().orc_merkle_levels_injected(lv.ctypes.data_as(u8p), C.c_uint64(n), len(arrs), lvl.ctypes.data_as(i32p), ptrs,
                                     out.ctypes.data_as(u8p))
    res, pos = [], 0
    while n >= 1:
        res.append(out[pos:pos + n].copy())
        pos += n
        n //= 2
    return res


def check_path_injected(h, path, i, cap, injected_at):
    """check-path with injected-at (src/pcs.lisp:86-95): injected_at = {level: digest}."""
    h = np.frombuffer(bytes(h), np.uint8).copy()
    p = np.ascontiguousarray(path, np.uint8).reshape(-1, 32)
    capa = np.ascontiguousarray(cap, np.uint8).reshape(-1, 32)
    levels = sorted(injected_at)
    lvl = np.array(levels if levels else [0], np.int32)
    dig = np.array([np.frombuffer(bytes(injected_at[l]), np.uint8) for l in levels], np.uint8).reshape(-1, 32) \
        if levels else np.zeros((1, 32), np.uint8)
    return bool(lib().orc_check_path_injected(h.ctypes.data_as(u8p), p.ctypes.data_as(u8p), len(p), C.c_uint64(i),
                                              capa.ctypes.data_as(u8p), len(levels), lvl.ctypes.data_as(i32p),
                                              dig.ctypes.data_as(u8p)))


def _open_keys(keys, prover):
    """keys: dicts with c, ncols, coef (ncols, 8) and, for the prover, codewords (ncols, 2^(c+1)), levels (list of
    (n, 32) arrays), h (2^c, 8); for the verifier, cap (rows, 32)."""
    arr = (OpenKey * len(keys))()
    keep = []
    for k, key in enumerate(keys):
        coef = _u32(key["coef"]).reshape(-1, 8)
        keep.append(coef)
        arr[k].c, arr[k].ncols, arr[k].coef = key["c"], key["ncols"], _p(coef)
        if prover:
            cw = np.ascontiguousarray(key["codewords"], np.uint32)
            lv = np.ascontiguousarray(np.concatenate(key["levels"]), np.uint8)
            h = _u32(key["h"]).reshape(-1, 8)
            keep += [cw, lv, h]
            arr[k].codewords, arr[k].levels, arr[k].h = _p(cw), lv.ctypes.data_as(u8p), _p(h)
        else:
            cap = np.ascontiguousarray(key["cap"], np.uint8)
            keep.append(cap)
            arr[k].cap = cap.ctypes.data_as(u8p)
    return arr, keep


def pcs_open(tr, nv, keys, rr, v, grind_bits=4, queries=6):
    arr, keep = _open_keys(keys, True)
    rr, v = _u32(rr).reshape(-1, 8), _u32(v)
    qs = np.zeros(queries, np.uint64)
    _check(lib().orc_pcs_open(tr.h, nv, len(keys), arr, _p(rr), _p(v), grind_bits, queries,
                              qs.ctypes.data_as(u64p)), "pcs-open")
    return [int(q) for q in qs]


def pcs_verify_opening(tr, nv, keys, rr, v, grind_bits=4, queries=6):
    arr, keep = _open_keys(keys, False)
    rr, v = _u32(rr).reshape(-1, 8), _u32(v)
    _check(lib().orc_pcs_verify_opening(tr.h, nv, len(keys), arr, _p(rr), _p(v), grind_bits, queries), "pcs")
    return True


def basefold_classes(tr, nv, classes, rr, v, grind_bits=4, queries=6):
    """basefold (src/pcs.lisp:581-657) alone over the classes' combined columns: classes = [(c, h (2^c, 8)), ...]
    in ascending c, the largest being nv.  Returns the query positions."""
    arr = (OpenKey * len(classes))()
    keep = []
    for k, (c, h) in enumerate(classes):
        h = _u32(h).reshape(-1, 8)
        assert len(h) == 1 << c
        keep.append(h)
        arr[k].c, arr[k].ncols, arr[k].h = c, 0, _p(h)
    rr, v = _u32(rr).reshape(-1, 8), _u32(v)
    qs = np.zeros(queries, np.uint64)
    _check(lib().orc_basefold_classes(tr.h, nv, len(classes), arr, _p(rr), _p(v), grind_bits, queries,
                                      qs.ctypes.data_as(u64p)), "basefold")
    return [int(q) for q in qs]
