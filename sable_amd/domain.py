"""Domains over the HIP library: the host side of the reference's src/domain.lisp, with the columns resident in HBM.

make_domain, domain_tables, domain_statement, domain_degree, prove_domain and verify_domain keep the reference's
names and argument meaning.  The prover's heavy parts run on the device: the leaves of every lookup's fraction tree
(exh_domain_leaves), the sumcheck's tables (exh_domain_table), the LogUp-GKR above the leaves (exh_gkr_prove_upper)
and the leaf-layer/zerocheck sumcheck (exh_prove) on a kernel for the domain's statement.  The verifier is host
arithmetic over the library's transcript, VERIFY and EVALUATE.

Forms are the reference's s-expressions as text, e.g. "(- c (* a b))"; a lookup is a dict with "tag", "values"
and optionally "num".
"""
import ctypes as C

import numpy as np

import sable_amd as sa
from sable_amd import lib as _lib
from sable_amd import load, check, _p, _u32, _bytes

KINDS = {"full": 0, "row": 1, "col": 2}


# ------------------------------------------------------------------ forms as text
def _tokens(text):
    return str(text).replace("(", " ( ").replace(")", " ) ").split()


def _rename(text, mapping):
    """The form with each variable that `mapping` names replaced (SUBLIS on the reference's form)."""
    out = []
    for tok in _tokens(text):
        out.append(mapping.get(tok.upper(), tok.upper()))
    return " ".join(out).replace("( ", "(").replace(" )", ")")


def _variables(text):
    ops = {"+", "-", "*", "EXPT"}
    toks, out, after_open = _tokens(text), set(), False
    for tok in toks:
        if tok == "(":
            after_open = True
            continue
        if tok == ")":
            after_open = False
            continue
        if after_open and tok.upper() in ops:
            after_open = False
            continue
        after_open = False
        if not tok.lstrip("+-").isdigit():
            out.add(tok.upper())
    return out


# ------------------------------------------------------------------ the domain (src/domain.lisp:29-51)
class Column:
    """A column: `data` a device Table of base values (the prover's; None for the verifier), or an array to upload."""

    def __init__(self, name, kind="full", c=0, shared=False, data=None):
        if kind not in KINDS:
            raise sa.InvalidParameter(_lib.E_PARAM, "kind: full, row or col")
        self.name, self.kind, self.shared = name.upper(), kind, bool(shared)
        self.c = 0 if kind == "full" else int(c)
        if data is not None and not isinstance(data, sa.Table):
            data = sa.Table.upload(np.ascontiguousarray(_u32(np.asarray(data))))
        self.data = data

    def c_struct(self, keep):
        name = self.name.encode()
        keep.append(name)
        return _DomainColumn(name, KINDS[self.kind], self.c, int(self.shared), self.data.handle)


class _DomainColumn(C.Structure):
    _fields_ = [("name", C.c_char_p), ("kind", C.c_int32), ("c", C.c_int32), ("shared", C.c_int32),
                ("data", C.c_uint64)]


class Domain:
    def __init__(self, name, n, columns, blocks=1, merge=False, constraints=(), lookups=()):
        if not (isinstance(n, int) and n >= 2):
            raise sa.InvalidParameter(_lib.E_PARAM, "n: at least 2")
        for col in columns:
            if col.shared and col.kind == "full":
                raise sa.InvalidParameter(_lib.E_PARAM, "shared: NIL for a :FULL column")
            if col.name.startswith("%"):
                raise sa.InvalidParameter(_lib.E_PARAM, "a column's name may not begin with %")
        self.name, self.n, self.blocks, self.merge = name, n, int(blocks), bool(merge)
        self.columns = list(columns)
        self.constraints = [str(f) for f in constraints]
        self.lookups = [{"tag": str(l["tag"]), "values": [str(v) for v in l["values"]],
                         "num": None if l.get("num") is None else str(l["num"])} for l in lookups]
        self._statements, self._degrees = {}, {}


make_domain = Domain


# ------------------------------------------------------------------ the tables of the sumcheck (:55-79)
def domain_tables(dom):
    """[(symbol, column, half, kind, c)] in the proof's order (DOMAIN-TABLES)."""
    n, out = dom.n, []
    for col in dom.columns:
        two = col.kind == "full" or (col.kind == "row" and col.c < n) or (col.kind == "col" and col.c == n)
        if two:
            kind, c = ("col", n - 1) if col.kind == "col" else (col.kind, col.c)
            out += [("%s@%d" % (col.name, h), col, h, kind, c) for h in (0, 1)]
        else:
            out.append((col.name, col, None, col.kind, n - 1 if col.kind == "row" else col.c))
    return out


def at_half(form, dom, half):
    return _rename(form, {col.name: sym for sym, col, h, _, _ in domain_tables(dom) if h == half})


# ------------------------------------------------------------------ the statement (:83-114)
def _arity(dom):
    return max([1] + [len(l["values"]) for l in dom.lookups])


def _denominator(lookup, dom, half):
    betas = " ".join("(* %%BETA%d %s)" % (i, at_half(v, dom, half)) for i, v in enumerate(lookup["values"]))
    return "(- %%Z %s %s)" % (at_half(lookup["tag"], dom, half), betas)


def domain_statement(dom):
    """DOMAIN-STATEMENT as text.  The constants carry a % so that no column's name meets them."""
    terms = []
    for l, lookup in enumerate(dom.lookups):
        q0, q1, num = _denominator(lookup, dom, 0), _denominator(lookup, dom, 1), lookup["num"]
        inner = "(+ (* %s %s) (* %s %s))" % (at_half(num, dom, 0), q1, at_half(num, dom, 1), q0) if num is not None \
            else "(+ %s %s)" % (q0, q1)
        terms += ["(* %%A%d %s)" % (l, inner), "(* %%AL%d %s %s)" % (l, q0, q1)]
    for i, con in enumerate(dom.constraints):
        terms += ["(* %%GAM%d %s)" % (i, at_half(con, dom, 0)), "(* %%GETA%d %s)" % (i, at_half(con, dom, 1))]
    return "(+ %s)" % " ".join(terms)


def domain_constant_names(dom):
    names = ["%Z"] + ["%%BETA%d" % i for i in range(_arity(dom))]
    for l in range(max(1, len(dom.lookups))):
        names += ["%%A%d" % l, "%%AL%d" % l]
    for i in range(max(1, len(dom.constraints))):
        names += ["%%GAM%d" % i, "%%GETA%d" % i]
    return names


def _compiled(dom, block_phase=False):
    """The domain's statement compiled once per domain (and once more with the block weight in front)."""
    if block_phase not in dom._statements:
        form, tables = domain_statement(dom), [t[0] for t in domain_tables(dom)]
        if block_phase:
            form, tables = "(* BW %s)" % form, ["BW"] + tables
        dom._statements[block_phase] = sa.Statement(form, tables, domain_constant_names(dom))
    return dom._statements[block_phase]


def _monomials(form, variables):
    """The largest number of the given variables in one monomial of the form's expansion: the library's EXPAND
    with those variables as the tables and the others as constants, whose STATEMENT-DEGREE is that count."""
    counted = [v for v in sorted(_variables(form)) if v in variables]
    if not counted:
        return 0
    others = [v for v in sorted(_variables(form)) if v not in variables]
    st = sa.Statement(str(form), counted, others)
    degree = st.degree
    st.free()
    return degree


def domain_degree(dom, block_phase=False):
    """DOMAIN-DEGREE (:116-155): the header degree of the statement's round polynomials."""
    if block_phase in dom._degrees:
        return dom._degrees[block_phase]
    n = dom.n
    tables = {sym: (col, kind, c) for sym, col, _, kind, c in domain_tables(dom)}
    rounds = ["block"] if block_phase else list(range(n - 1))

    def varying(rnd):
        out = set()
        for sym, (col, kind, c) in tables.items():
            if rnd == "block":
                v = not col.shared
            else:
                v = True if kind == "full" else (rnd < c if kind == "col" else rnd >= c)
            if v:
                out.add(sym)
        return out

    sets = [varying(rnd) for rnd in rounds]

    def piece(form):
        return max([0] + [_monomials(form, s) for s in sets])

    def q(lookup, half):
        return max([piece(at_half(lookup["tag"], dom, half))] + [piece(at_half(v, dom, half)) for v in lookup["values"]])

    best = 0
    for lookup in dom.lookups:
        q0, q1, num = q(lookup, 0), q(lookup, 1), lookup["num"]
        if num is not None:
            best = max(best, piece(at_half(num, dom, 0)) + q1, piece(at_half(num, dom, 1)) + q0, q0 + q1)
        else:
            best = max(best, q0 + q1)
    for con in dom.constraints:
        best = max(best, piece(at_half(con, dom, 0)), piece(at_half(con, dom, 1)))
    dom._degrees[block_phase] = best + 1 if block_phase else best
    return dom._degrees[block_phase]


# ------------------------------------------------------------------ field helpers on canonical residues
def _add(a, b):
    return ((a.astype(np.uint64) + b) % sa.P).astype(np.uint32)


def _sub(a, b):
    return ((a.astype(np.uint64) + sa.P - b) % sa.P).astype(np.uint32)


def _fold_pair(lo, hi, r):
    return _add(lo, sa.ext_mul(r, _sub(hi, lo)))


def _constants(dom, z, betas, as_, lam, gams, eta):
    out = [_u32(z)] + [_u32(betas[i]) for i in range(_arity(dom))]
    for a in as_:
        out += [a, sa.ext_mul(a, lam)]
    for g in gams:
        out += [g, sa.ext_mul(g, eta)]
    return np.array(out, np.uint32)


def _challenges(tr, dom):
    as_ = tr.challenges(max(1, len(dom.lookups)))
    lam = tr.challenge()
    gams = tr.challenges(max(1, len(dom.constraints)))
    return as_, lam, gams, tr.challenge()


def _block_weights(rb, k, d):
    if len(rb) == 0:
        one = np.zeros((1, d), np.uint32)
        one[0, 0] = 1
        return one
    return sa.eq_table(rb, d)[:k]


def label_name(name):
    """LABEL-NAME (src/transcript.lisp:219-230)."""
    def strip(seg):
        k = 0
        while k < len(seg) and seg[k] in "0123456789":
            k += 1
        return seg[k + 1:] if 0 < k < len(seg) and seg[k] == "." else seg
    return "|".join(strip(seg) for seg in name.split("|"))


def domain_claims(dom, rho, rb, tt, finals):
    """DOMAIN-CLAIMS (:182-212): [(name, point, value)]."""
    n, tables, d = dom.n, domain_tables(dom), len(tt)
    full = list(rho) + [tt]
    claims = []
    for col in dom.columns:
        halves = [t for t in tables if t[1] is col]
        f0, f1 = finals[halves[0][0]], finals[halves[-1][0]]
        if len(halves) > 1:
            point = full[col.c:] if col.kind == "row" else full
            value = _fold_pair(f0, f1, tt) if f0.ndim == 1 else np.array([_fold_pair(a, b, tt) for a, b in zip(f0, f1)])
        else:
            point = list(rho[:min(col.c, n - 1)]) if col.kind == "col" else []
            value = f0
        if dom.merge and not col.shared:
            point = list(point) + list(rb)
        claims.append((col.name, np.array(point, np.uint32).reshape(-1, d), value))
    return claims


# ------------------------------------------------------------------ verifier (:229-284)
def verify_domain(tr, dom, z, betas, label="dom"):
    """VERIFY-DOMAIN: (claims, roots); raises VerificationFailure."""
    d, n, k = tr.degree, dom.n, dom.blocks
    lk, lookups, tables = sa._block_bits(k), len(dom.lookups), domain_tables(dom)
    st = _compiled(dom)
    tr.absorb(_bytes(label) + label_name(dom.name).encode())
    roots = np.zeros((0, 2, d), np.uint32)
    if lookups:
        roots, r, rb, cp, cq = sa.verify_upper(tr, n, k, lookups)
    else:
        r, rb = tr.challenges(n - 1), tr.challenges(lk)
    as_, lam, gams, eta = _challenges(tr, dom)
    constants = _constants(dom, z, betas, as_, lam, gams, eta)
    claim = np.zeros(d, np.uint32)
    for l in range(lookups):  # LAYER-CLAIM (src/gkr.lisp:53-55)
        claim = _add(claim, sa.ext_mul(as_[l], _add(cp[l], sa.ext_mul(lam, cq[l]))))
    bw = _block_weights(rb, k, d)
    rho, reduced = sa.verify(tr, n - 1, st, claim, eq=r, constants=constants, blocks=k, label=label,
                             degree=domain_degree(dom))
    if dom.merge:
        rbn = np.zeros((0, d), np.uint32)
        if lk:
            rbn, reduced = sa.verify(tr, lk, _compiled(dom, True), reduced, constants=constants,
                                     label=_bytes(label) + b"-blk", degree=domain_degree(dom, block_phase=True))
        finals = {sym: tr.send(shape=(1, d))[0] for sym, *_ in tables}
        weight = bw[0]
        if k > 1:
            weight, e = np.zeros(d, np.uint32), sa.eq_table(rbn, d)
            for b in range(k):
                weight = _add(weight, sa.ext_mul(bw[b], e[b]))
        value = evaluate(st, np.array([finals[sym] for sym, *_ in tables]), constants, d)
        if not np.array_equal(reduced, sa.ext_mul(weight, value)):
            raise sa.VerificationFailure(_lib.E_REJECT, _reject(dom))
        return domain_claims(dom, rho, rbn, tr.challenge(), finals), roots
    finals = {sym: tr.send(shape=(1 if col.shared else k, d)) for sym, col, *_ in tables}
    total = np.zeros(d, np.uint32)
    for b in range(k):
        at = np.array([finals[sym][b if len(finals[sym]) > 1 else 0] for sym, *_ in tables])
        total = _add(total, sa.ext_mul(bw[b], evaluate(st, at, constants, d)))
    if not np.array_equal(reduced, total):
        raise sa.VerificationFailure(_lib.E_REJECT, _reject(dom))
    return domain_claims(dom, rho, [], tr.challenge(), finals), roots


def _reject(dom):
    return "verification-failure: domain %s: leaf/zerocheck sumcheck failed" % dom.name


def evaluate(st, table_values, constants, d):
    """EVALUATE of a compiled statement at table values (T, D) and constants."""
    tv, cv = np.ascontiguousarray(_u32(table_values).reshape(-1, d)), sa._consts(constants, d)
    out = np.zeros(d, np.uint32)
    check(load().exh_stmt_evaluate(C.c_uint64(st.handle), d, _p(tv), _p(cv), _p(out)))
    return out


# ------------------------------------------------------------------ prover (:288-372)
def _c_columns(dom):
    keep = []
    arr = (_DomainColumn * len(dom.columns))(*[col.c_struct(keep) for col in dom.columns])
    return arr, keep


def domain_leaves(dom, z, betas):
    """DOMAIN-LEAVES on the device: per lookup (p, q), Tables of K 2^n EXTs of the degree of z."""
    z, d = _u32(z), len(z)
    betas = np.ascontiguousarray(_u32(betas).reshape(-1, d))
    arr, keep = _c_columns(dom)
    out = []
    for lookup in dom.lookups:
        vals = (C.c_char_p * max(1, len(lookup["values"])))(*[v.encode() for v in lookup["values"]])
        hp, hq = C.c_uint64(), C.c_uint64()
        check(load().exh_domain_leaves(d, dom.n, dom.blocks, arr, len(dom.columns), lookup["tag"].encode(), vals,
                                       len(lookup["values"]), None if lookup["num"] is None else lookup["num"].encode(),
                                       _p(z), _p(betas), C.byref(hp), C.byref(hq)))
        words = (dom.blocks << dom.n) * d
        out.append((sa.Table(hp.value, words, d), sa.Table(hq.value, words, d)))
    return out


def table_values(table, k, n):
    """TABLE-VALUES on the device: the Table of K 2^(n-1) base values of one sumcheck table."""
    _, col, half, _, _ = table
    keep = []
    cs = col.c_struct(keep)
    h = C.c_uint64()
    check(load().exh_domain_table(C.byref(cs), -1 if half is None else half, n, k, C.byref(h)))
    return sa.Table(h.value, k << (n - 1), 1)


def prove_domain(tr, dom, z, betas, label="dom"):
    """PROVE-DOMAIN: the column claims, as verify_domain returns them."""
    d, n, k = tr.degree, dom.n, dom.blocks
    lk, lookups, tables = sa._block_bits(k), len(dom.lookups), domain_tables(dom)
    st = _compiled(dom)
    tr.absorb(_bytes(label) + label_name(dom.name).encode())
    if lookups:
        leaves = domain_leaves(dom, z, betas)
        r, rb, cp, cq = sa.prove_upper(tr, n, k, leaves)
        for p, q in leaves:
            p.free(), q.free()
    else:
        r, rb = tr.challenges(n - 1), tr.challenges(lk)
    as_, lam, gams, eta = _challenges(tr, dom)
    constants = _constants(dom, z, betas, as_, lam, gams, eta)
    bw = _block_weights(rb, k, d)
    device_tables = [table_values(t, k, n) for t in tables]
    rho, finals, folded = sa.prove(tr, n - 1, st, device_tables, eq=r, constants=constants, label=label,
                                   block_weights=bw, degree=domain_degree(dom))
    for t in device_tables:
        t.free()
    if dom.merge:
        rbn = np.zeros((0, d), np.uint32)
        if lk:
            def padded(values, shared):
                fill = values[:1] if shared else np.zeros((1, d), np.uint32)
                return sa.Table.upload(np.concatenate([values] + [fill] * ((1 << lk) - k)))
            block_tables = [padded(bw, False)] + [padded(f, t[1].shared) for f, t in zip(folded, tables)]
            rbn, finals, _ = sa.prove(tr, lk, _compiled(dom, True), block_tables, constants=constants,
                                      label=_bytes(label) + b"-blk", degree=domain_degree(dom, block_phase=True))
            finals = finals[1:]
            for t in block_tables:
                t.free()
        named = {t[0]: f for t, f in zip(tables, finals)}
        for sym, *_ in tables:
            tr.send(named[sym].reshape(1, d))
        return domain_claims(dom, rho, rbn, tr.challenge(), named)
    named = {t[0]: (f[:1] if t[1].shared else f) for t, f in zip(tables, folded)}
    for sym, *_ in tables:
        tr.send(named[sym])
    return domain_claims(dom, rho, [], tr.challenge(), named)
