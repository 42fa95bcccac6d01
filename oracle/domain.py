"""Domains -- the leaf layer and zerocheck caller of the proving path, restated from the reference's
src/domain.lisp (test oracle: only tests, the smoke check and the bench's CPU baseline may use this file).

A domain is K blocks of 2^n elements with base-field columns, constraints (forms over the column names that
vanish everywhere) and lookups (tag, values, numerator forms).  Its proof is one batched LogUp-GKR down to layer
n-1 (oracle gkr_prove_upper), one sumcheck over the halves of the columns that proves the trees' leaf layer and
the zerocheck (oracle prove), and a fresh point that turns the halves' finals into column claims.

The sumcheck underneath is pinned by the reference's golden vectors.  This layer is pinned by the reference's
frozen domain cases (tests/tests.lisp:587-624, digest at :904): the sixteen proofs of EXPORT-DOMAIN-CASES, made here
over the reference's own inputs (SBCL's seeded generator restated in tests/golden/sbcl_random.py), with the
verifier's claims and roots, hash to the SHA-256 the reference holds (tests/test_oracle_frozen_cases.py).  Beside
that, what the protocol fixes: the verifier accepts the prover's proof, its claims are the columns' multilinear
extensions at the claimed points, the roots are the sums of the leaf fractions, a broken constraint and every
perturbed message are rejected (tests/test_oracle_domain.py, after tests/tests.lisp:485-575), and the statement's
value at random points equals the formula in the doc string of domain-statement (src/domain.lisp:95-114).

Forms are nested lists as in oracle/forms.py: an int, an upper-case name, or [op, arg...].
"""
import numpy as np

from . import binding as orc
from . import forms

P = orc.P


# ------------------------------------------------------------------ the domain (src/domain.lisp:29-51)
class Column:
    def __init__(self, name, kind="full", c=0, shared=False, data=None):
        self.name, self.kind, self.shared = name.upper(), kind, bool(shared)
        self.c = 0 if kind == "full" else c
        self.data = None if data is None else np.asarray(data, np.uint64) % P


class Domain:
    def __init__(self, name, n, columns, blocks=1, merge=False, constraints=(), lookups=()):
        """columns: Column objects; constraints: forms; lookups: dicts with "tag", "values" and optionally "num"."""
        if not (isinstance(n, int) and n >= 2):
            raise ValueError("n: at least 2")
        for col in columns:
            if col.shared and col.kind == "full":
                raise ValueError("shared: NIL for a :FULL column")
        self.name, self.n, self.blocks, self.merge = name, n, blocks, bool(merge)
        self.columns = list(columns)
        self.constraints = [normal(f) for f in constraints]
        self.lookups = [{"tag": normal(l["tag"]), "values": [normal(v) for v in l["values"]],
                         "num": normal(l["num"]) if l.get("num") is not None else None} for l in lookups]


def normal(form):
    """A form given as text or as nested lists, as nested lists with upper-case names."""
    if isinstance(form, str):
        return forms.read_form(form) if form.strip().startswith("(") else (
            int(form) if form.strip().lstrip("+-").isdigit() else form.strip().upper())
    if isinstance(form, (list, tuple)):
        return [form[0] if i == 0 else normal(a) for i, a in enumerate(form)]
    return form


def sublis(form, mapping):
    if isinstance(form, str):
        return mapping.get(form, form)
    if isinstance(form, list):
        return [form[0]] + [sublis(a, mapping) for a in form[1:]]
    return form


# ------------------------------------------------------------------ the tables of the sumcheck (:55-79)
def half_symbol(name, half):
    return "%s@%d" % (name, half)


def domain_tables(dom):
    """(symbol, column, half, kind, c) in the proof's order: two tables (halves 0 and 1) for a column that depends
    on the top in-block variable, one (half None) for a column that does not."""
    n, out = dom.n, []
    for col in dom.columns:
        if col.kind == "full" or (col.kind == "row" and col.c < n):
            out += [(half_symbol(col.name, h), col, h, col.kind, col.c) for h in (0, 1)]
        elif col.kind == "col" and col.c == n:
            out += [(half_symbol(col.name, h), col, h, "col", n - 1) for h in (0, 1)]
        elif col.kind == "row":
            out.append((col.name, col, None, "row", n - 1))
        else:
            out.append((col.name, col, None, "col", col.c))
    return out


def at_half(form, dom, half):
    return sublis(form, {col.name: sym for sym, col, h, _, _ in domain_tables(dom) if h == half})


# ------------------------------------------------------------------ the statement (:83-114)
def constant_symbol(name, i=None):
    # the reference interns these in its own package; here a prefix no column name may carry keeps them apart
    return "%" + name + ("" if i is None else str(i))


def arity(dom):
    return max([1] + [len(l["values"]) for l in dom.lookups])


def denominator_form(lookup, dom, half):
    return ["-", constant_symbol("Z"), at_half(lookup["tag"], dom, half)] + [
        ["*", constant_symbol("BETA", i), at_half(v, dom, half)] for i, v in enumerate(lookup["values"])]


def domain_statement(dom):
    """sum_l a_l (N_l(0) q_l(1) + N_l(1) q_l(0)) + a_l lambda q_l(0) q_l(1) + sum_i gamma_i C_i(0) + gamma_i eta C_i(1)"""
    terms = []
    for l, lookup in enumerate(dom.lookups):
        q0, q1, num = denominator_form(lookup, dom, 0), denominator_form(lookup, dom, 1), lookup["num"]
        inner = ["+", ["*", at_half(num, dom, 0), q1], ["*", at_half(num, dom, 1), q0]] if num is not None else ["+", q0, q1]
        terms += [["*", constant_symbol("A", l), inner], ["*", constant_symbol("AL", l), q0, q1]]
    for i, con in enumerate(dom.constraints):
        terms += [["*", constant_symbol("GAM", i), at_half(con, dom, 0)],
                  ["*", constant_symbol("GETA", i), at_half(con, dom, 1)]]
    return ["+"] + terms


def domain_constant_names(dom):
    names = [constant_symbol("Z")] + [constant_symbol("BETA", i) for i in range(arity(dom))]
    for l in range(max(1, len(dom.lookups))):
        names += [constant_symbol("A", l), constant_symbol("AL", l)]
    for i in range(max(1, len(dom.constraints))):
        names += [constant_symbol("GAM", i), constant_symbol("GETA", i)]
    return names


def domain_constants(dom, z, betas, as_, lam, gams, eta):
    """The constants' values in domain_constant_names' order (:158-168)."""
    out = [z] + [betas[i] for i in range(arity(dom))]
    for a in as_:
        out += [a, orc.ext_mul(a, lam)]
    for g in gams:
        out += [g, orc.ext_mul(g, eta)]
    return np.array(out, np.uint32)


def domain_challenges(tr, dom):
    as_ = tr.challenges(max(1, len(dom.lookups)))
    lam = tr.challenge()
    gams = tr.challenges(max(1, len(dom.constraints)))
    eta = tr.challenge()
    return as_, lam, gams, eta


def domain_degree(dom, block_phase=False):
    """The header degree (:116-155): per polynomial piece only the tables that vary in a round count, maximised over
    the rounds; products add, sums take the maximum; the block sumcheck counts non-shared tables, plus 1."""
    n = dom.n
    tables = {sym: (col, kind, c) for sym, col, _, kind, c in domain_tables(dom)}
    rounds = ["block"] if block_phase else list(range(n - 1))

    def varies(sym, rnd):
        col, kind, c = tables[sym]
        if rnd == "block":
            return not col.shared
        return True if kind == "full" else (rnd < c if kind == "col" else rnd >= c)

    def piece(form):
        return max([0] + [max([0] + [sum(1 for v in mono if varies(v, rnd)) for mono, _ in forms.expand(form)])
                          for rnd in rounds])

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
    return best + 1 if block_phase else best


# ------------------------------------------------------------------ claims (:182-212)
def fold_pair(lo, hi, r):
    return orc.ext_add(lo, orc.ext_mul(r, orc.ext_sub(hi, lo)))


def domain_claims(dom, rho, rb, tt, finals):
    """Per column (name, point, value): finals maps a table symbol to its value(s) -- (D,) merged, (rows, D) else."""
    n, tables = dom.n, domain_tables(dom)
    full = list(rho) + [tt]
    claims = []
    for col in dom.columns:
        halves = [t for t in tables if t[1] is col]
        f0, f1 = finals[halves[0][0]], finals[halves[-1][0]]
        if len(halves) > 1:
            point = full[col.c:] if col.kind == "row" else full
            value = fold_pair(f0, f1, tt) if f0.ndim == 1 else np.array([fold_pair(a, b, tt) for a, b in zip(f0, f1)])
        else:
            point = list(rho[:min(col.c, n - 1)]) if col.kind == "col" else []
            value = f0
        if dom.merge and not col.shared:
            point = list(point) + list(rb)
        claims.append((col.name, np.array(point, np.uint32).reshape(-1, len(tt)), value))
    return claims


# ------------------------------------------------------------------ verifier (:229-284)
def label_name(name):
    """label-name (src/transcript.lisp:219-230): "12.mo" -> "mo", "3.oproj|3.rqo" -> "oproj|rqo"."""
    def strip(seg):
        k = 0
        while k < len(seg) and seg[k].isdigit() and seg[k].isascii():
            k += 1
        return seg[k + 1:] if 0 < k < len(seg) and seg[k] == "." else seg
    return "|".join(strip(seg) for seg in name.split("|"))


def layer_claim(as_, lam, cp, cq):
    out = np.zeros(len(lam), np.uint32)
    for a, p, q in zip(as_, cp, cq):
        out = orc.ext_add(out, orc.ext_mul(a, orc.ext_add(p, orc.ext_mul(lam, q))))
    return out


def block_weights(rb, k, d):
    return orc.base_to_ext(1, d).reshape(1, d) if len(rb) == 0 else orc.eq_table(rb, d)[:k]


def _statement(dom, extra_table=None):
    form, tables = domain_statement(dom), [t[0] for t in domain_tables(dom)]
    if extra_table:
        form, tables = ["*", extra_table, form], [extra_table] + tables
    return orc.Statement(form, tables, domain_constant_names(dom))


def verify_domain(tr, dom, z, betas, label="dom"):
    """verify-domain: (claims, roots); raises VerificationFailure."""
    d, n, k = tr.degree, dom.n, dom.blocks
    lk, lookups, tables = orc._block_bits(k), len(dom.lookups), domain_tables(dom)
    st = _statement(dom)
    tr.absorb(orc._label(label) + label_name(dom.name).encode())
    roots = np.zeros((0, 2, d), np.uint32)
    if lookups:
        roots, r, rb, cp, cq = orc.gkr_verify_upper(tr, n, k, lookups)
    else:
        r, rb = tr.challenges(n - 1), tr.challenges(lk)
    as_, lam, gams, eta = domain_challenges(tr, dom)
    constants = domain_constants(dom, z, betas, as_, lam, gams, eta)
    claim = layer_claim(as_, lam, cp, cq) if lookups else np.zeros(d, np.uint32)
    bw = block_weights(rb, k, d)
    rho, reduced = orc.verify(tr, n - 1, st, claim, eq=r, constants=constants, blocks=k, label=label,
                              degree=domain_degree(dom))
    if dom.merge:
        rbn = np.zeros((0, d), np.uint32)
        if lk:
            rbn, reduced = orc.verify(tr, lk, _statement(dom, "BW"), reduced, constants=constants,
                                      label=orc._label(label) + b"-blk", degree=domain_degree(dom, block_phase=True))
        finals = {sym: tr.send(shape=(1, d))[0] for sym, *_ in tables}
        weight = bw[0]
        if k > 1:
            weight, e = np.zeros(d, np.uint32), orc.eq_table(rbn, d)
            for b in range(k):
                weight = orc.ext_add(weight, orc.ext_mul(bw[b], e[b]))
        value = st.evaluate(np.array([finals[sym] for sym, *_ in tables]), constants, d)
        if not np.array_equal(reduced, orc.ext_mul(weight, value)):
            raise orc.VerificationFailure(orc.E_REJECT, "domain: leaf/zerocheck sumcheck failed")
        return domain_claims(dom, rho, rbn, tr.challenge(), finals), roots
    finals = {sym: tr.send(shape=(1 if col.shared else k, d)) for sym, col, *_ in tables}
    total = np.zeros(d, np.uint32)
    for b in range(k):
        at = np.array([finals[sym][b if len(finals[sym]) > 1 else 0] for sym, *_ in tables])
        total = orc.ext_add(total, orc.ext_mul(bw[b], st.evaluate(at, constants, d)))
    if not np.array_equal(reduced, total):
        raise orc.VerificationFailure(orc.E_REJECT, "domain: leaf/zerocheck sumcheck failed")
    return domain_claims(dom, rho, [], tr.challenge(), finals), roots


# ------------------------------------------------------------------ prover (:288-372)
def column_values(col, b, n):
    """The column in block b at every in-block index x < 2^n (column-value, :288-296)."""
    x, c = np.arange(1 << n), col.c
    if col.kind == "full":
        return col.data[(0 if col.shared else b << n) + x]
    if col.kind == "row":
        return col.data[(0 if col.shared else b << (n - c)) + (x >> c)]
    return col.data[(0 if col.shared else b << c) + (x & ((1 << c) - 1))]


def evaluate_base(form, values):
    """A form over arrays of base values, by direct recursion."""
    if isinstance(form, int):
        return np.uint64(form % P)
    if isinstance(form, str):
        return values[form]
    op, args = form[0], [evaluate_base(a, values) for a in form[1:]]
    if op == "+":
        out = np.uint64(0)
        for a in args:
            out = (out + a) % P
        return out
    if op == "*":
        out = np.uint64(1)
        for a in args:
            out = out * a % P
        return out
    if op == "-":
        if len(args) == 1:
            return (P - args[0]) % P
        out = args[0]
        for a in args[1:]:
            out = (out + P - a) % P
        return out
    if op in ("expt", "EXPT"):
        base, out = evaluate_base(form[1], values), np.uint64(1)
        for _ in range(form[2]):
            out = out * base % P
        return out
    raise ValueError("malformed form")


def domain_leaves(dom, z, betas):
    """Per lookup (p, q), each (K 2^n, D): p the numerator (1 if absent), q = Z - tag - sum_i beta_i v_i (:298-319)."""
    d, n, k = len(z), dom.n, dom.blocks
    z, betas = np.asarray(z, np.uint64), np.asarray(betas, np.uint64).reshape(-1, d)
    out = []
    for lookup in dom.lookups:
        p, q = np.zeros((k << n, d), np.uint64), np.zeros((k << n, d), np.uint64)
        for b in range(k):
            values = {col.name: column_values(col, b, n) for col in dom.columns}
            rows = slice(b << n, (b + 1) << n)
            p[rows, 0] = evaluate_base(lookup["num"], values) if lookup["num"] is not None else 1
            acc = np.broadcast_to(z, (1 << n, d)).copy()
            acc[:, 0] = (acc[:, 0] + P - evaluate_base(lookup["tag"], values)) % P
            for beta, v in zip(betas, lookup["values"]):
                vv = np.broadcast_to(evaluate_base(v, values), (1 << n,)).astype(np.uint64)
                acc = (acc + P - (vv[:, None] * beta[None, :]) % P) % P
            q[rows] = acc
        out.append((p.astype(np.uint32), q.astype(np.uint32)))
    return out


def table_values(table, k, n):
    """A sumcheck table: the column at its half's points, K blocks of 2^(n-1) base values (:321-331)."""
    _, col, half, _, _ = table
    h = 1 << (n - 1)
    lo = half * h if half else 0
    return np.concatenate([column_values(col, b, n)[lo:lo + h] for b in range(k)]).astype(np.uint32)


def prove_domain(tr, dom, z, betas, label="dom"):
    """prove-domain: the column claims, as verify_domain returns them."""
    d, n, k = tr.degree, dom.n, dom.blocks
    lk, lookups, tables = orc._block_bits(k), len(dom.lookups), domain_tables(dom)
    st = _statement(dom)
    tr.absorb(orc._label(label) + label_name(dom.name).encode())
    if lookups:
        r, rb, cp, cq = orc.gkr_prove_upper(tr, n, k, domain_leaves(dom, z, betas))
    else:
        r, rb = tr.challenges(n - 1), tr.challenges(lk)
    as_, lam, gams, eta = domain_challenges(tr, dom)
    constants = domain_constants(dom, z, betas, as_, lam, gams, eta)
    bw = block_weights(rb, k, d)
    rho, finals, folded = orc.prove(tr, n - 1, st, [table_values(t, k, n) for t in tables], eq=r, constants=constants,
                                    label=label, block_weights=bw, degree=domain_degree(dom))
    if dom.merge:
        rbn = np.zeros((0, d), np.uint32)
        if lk:
            def padded(values, shared):
                fill = values[:1] if shared else np.zeros((1, d), np.uint32)
                return np.concatenate([values] + [fill] * ((1 << lk) - k))
            rbn, finals, _ = orc.prove(tr, lk, _statement(dom, "BW"),
                                       [padded(bw, False)] + [padded(f, t[1].shared) for f, t in zip(folded, tables)],
                                       constants=constants, label=orc._label(label) + b"-blk",
                                       degree=domain_degree(dom, block_phase=True))
            finals = finals[1:]
        named = {t[0]: f for t, f in zip(tables, finals)}
        for sym, *_ in tables:
            tr.send(named[sym].reshape(1, d))
        return domain_claims(dom, rho, rbn, tr.challenge(), named)
    named = {t[0]: (f[:1] if t[1].shared else f) for t, f in zip(tables, folded)}
    for sym, *_ in tables:
        tr.send(named[sym])
    return domain_claims(dom, rho, [], tr.challenge(), named)
