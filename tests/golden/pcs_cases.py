"""The commitment proofs behind the reference's frozen PCS cases (tests/tests.lisp:627-758, digest at :905),
rebuilt: the prover side of src/pcs.lisp's scheduler -- units and size classes (:105-178), merge sets and
mixed-height trees (:218-269), PCS-COMMIT (:279-304), PCS-OPEN with its point reductions (:319-432), PCS-SEGMENT and
the cross-unit sumcheck (:445-567), PCS-FINISH and OPEN-QUERIES (:669-734) -- written over the oracle's primitives
(encoding, leaf digests, Merkle levels with injections, sumcheck, BaseFold over classes, transcript).  Test
infrastructure: it exists to hold those primitives to the reference's bytes."""
import numpy as np

from oracle import binding as orc
from oracle.domain import label_name
from sbcl_random import SbclRandom

P = 2130706433
CMIN, CAPLOG = 5, 7
PCS_SHA256 = "6ade2c3e6acad8ce06eea085b01b9534d625ff4476f7d970a2b3376949378d37"  # tests/tests.lisp:905

SCENARIOS = [  # tests/tests.lisp:630-645
    dict(cmax=9, seed=21, merge=["12.g1", "12.g2"], segment=["12.g1", "12.g2"],
         units=[("w", [("wa", 2, 9), ("wb", 1, 6), ("wc", 1, 3)]), ("12.g1", [("x", 3, 8), ("y", 1, 9)]),
                ("12.g2", [("z", 2, 7), ("u", 1, 9)]), ("big", [("v", 2, 10)])]),
    dict(cmax=10, seed=22, merge=["3.a", "3.b"], segment=None,
         units=[("w2", [("p", 1, 10), ("q", 6, 5)]), ("3.a", [("r", 2, 10)]), ("3.b", [("s", 1, 8), ("t", 4, 6)])]),
    dict(cmax=9, seed=23, merge=None, segment=["7.a", "7.b"], max_points=2,
         units=[("7.a", [("e", 1, 9), ("f", 2, 9), ("g", 1, 9)]), ("7.b", [("h", 3, 7)])]),
]


def ext(values, d):
    return np.array(list(values) + [0] * (d - len(values)), np.uint32)


def zero(d):
    return np.zeros(d, np.uint32)


def one(d):
    return ext([1], d)


def embed(a, d=8):
    return ext(list(a), d)


def ext_sum(items, d):
    acc = zero(d)
    for e in items:
        acc = orc.ext_add(acc, e)
    return acc


class OracleBackend:
    """The primitives the scheduler stands on, over host arrays: the oracle's here; tests/test_gpu_frozen_cases.py
    has the device's behind the same names.  (The arithmetic on single field elements around them -- claims,
    Lagrange interpolation of three values, eq of two points -- is the oracle's in both.)"""
    def transcript(self, label, d):
        return orc.Transcript(label, d)

    def encode(self, columns, c):
        return [orc.rs_encode(column, c + 1) for column in columns]

    def leaf_digests(self, codewords, c, previous):
        digests = np.zeros((1 << (c - 1), 32), np.uint8)
        for l in range(1 << (c - 1)):
            rows = np.array([cw[4 * l:4 * l + 4] for cw in codewords], np.uint32)
            digests[l] = np.frombuffer(orc.leaf_digest(rows, None if previous is None else bytes(previous[l])), np.uint8)
        return digests

    def merkle_levels(self, leaves, injections):
        return orc.merkle_levels_injected(leaves, injections)

    def prove_reduction(self, tr, c, form, names, tables):
        rho, _, _ = orc.prove(tr, c, orc.Statement(form, names), tables, label="pcs-red", degree=2)
        return [r for r in rho]

    def mle_eval(self, table, point, d):
        return orc.mle_eval(table, np.array(point), d)

    def combine_columns(self, columns, coefficients):
        return orc.combine_columns(np.array(columns), coefficients)

    def eq_table(self, point, d):
        return orc.eq_table(np.array(point), d)

    def scale_add(self, h, scale, column):
        column = np.asarray(column, np.uint32)
        return orc.scale_add(np.zeros_like(column) if h is None else h, scale, column)

    def dot_pairs(self, e, v):
        return orc.dot_pairs(e, v)

    def fold_table(self, table, x):
        return orc.fold_table(table, x)

    def basefold_classes(self, tr, nv, classes, rr, v, grind_bits, queries):
        return orc.basefold_classes(tr, nv, classes, rr, v, grind_bits=grind_bits, queries=queries)

    def gather_leaves(self, codewords, c, leaves):
        return np.array([[cw[4 * l:4 * l + 4] for cw in codewords] for l in leaves], np.uint32)


# ------------------------------------------------------------------ inputs (tests/tests.lisp:647-668)
def pcs_data(units, state):
    return {tensor: np.array([state.random(P) for _ in range(k << c0)], np.uint32)
            for _, items in units for tensor, k, c0 in items}


def pcs_claims(units, data, state):
    out = []
    for name, items in units:
        claims = []
        for tensor, k, c0 in items:
            values = data[tensor]
            for p in range(2):
                point = [ext([state.random(P) for _ in range(4)], 4) for _ in range(c0)]
                for _ in range(2 if p == 0 else 1):
                    coefficients = [(b, ext([state.random(P) for _ in range(4)], 4)) for b in range(k)]
                    value = ext_sum([orc.ext_mul(w, orc.mle_eval(values[b << c0:(b + 1) << c0], np.array(point), 4))
                                     for b, w in coefficients], 4)
                    claims.append((tensor, point, coefficients, value))
        out.append((name, claims))
    return out


# ------------------------------------------------------------------ units (src/pcs.lisp:105-178)
def class_of_size(c0, cmax):
    return min(max(c0, CMIN), cmax)


class Unit:
    def __init__(self, name, items, cmax):
        self.name, self.items, self.tensors = name, items, {}
        classes = {}
        for tensor, k, c0 in items:
            for b in range(k):
                for j in range(1 << max(0, c0 - cmax)):
                    classes.setdefault(class_of_size(c0, cmax), []).append((tensor, b, j))
        self.classes = sorted(classes.items())
        self.info = {tensor: (k, c0) for tensor, k, c0 in items}

    def members(self, c):
        return dict(self.classes)[c]

    def columns(self, c, cmax):
        cols = []
        for tensor, b, j in self.members(c):
            _, c0 = self.info[tensor]
            length = 1 << min(c0, cmax)
            offset = (b << c0) + j * length
            column = np.zeros(1 << c, np.uint32)
            column[:length] = self.tensors[tensor][offset:offset + length]
            cols.append(column)
        return cols


def class_claims(unit, claims, cmax):
    out = {}
    for tensor, point, coefficients, value in claims:
        _, c0 = unit.info[tensor]
        c = class_of_size(c0, cmax)
        columns = unit.members(c)
        index = lambda b, j: columns.index((tensor, b, j))
        if c0 > cmax:
            hi = point[cmax:]
            cd = []
            for b, w in coefficients:
                for j in range(1 << (c0 - cmax)):
                    cf = w
                    for bit, x in enumerate(hi):  # (reduce #'ext* factors :initial-value w)
                        cf = orc.ext_mul(cf, x if (j >> bit) & 1 else orc.ext_sub(one(4), x))
                    cd.append((index(b, j), cf))
            claim = (point[:cmax], cd, value)
        else:
            claim = (point + [zero(4) for _ in range(c - c0)], [(index(b, 0), w) for b, w in coefficients], value)
        out.setdefault(c, []).append(claim)
    return out


def by_point(claims):
    groups = []
    for z, columns, value in claims:
        for g in groups:
            if len(g[0]) == len(z) and all(np.array_equal(a, b) for a, b in zip(g[0], z)):
                g[1].append((columns, value))
                break
        else:
            groups.append((z, [(columns, value)]))
    return groups


# ------------------------------------------------------------------ the commitment object (src/pcs.lisp:190-304)
def cap_level(leaves):
    return max(0, leaves.bit_length() - 1 - CAPLOG)


class Uc:
    def __init__(self, unit, c, rho, alpha, y, ncols):
        self.unit, self.c, self.rho, self.alpha, self.y, self.ncols = unit, c, rho, alpha, y, ncols
        self.column = self.lam = self.sc = None


class Pu:
    def __init__(self, c, rho, y):
        self.c, self.rho, self.y = c, rho, y
        self.column = self.lam = self.sc = None


class Pcs:
    def __init__(self, tr, cmax, queries, grind, max_points=64, backend=None):
        self.tr, self.cmax, self.queries, self.grind, self.max_reduction_points = tr, cmax, queries, grind, max_points
        self.b = backend or OracleBackend()
        self.units, self.order, self.ucs = {}, [], {}
        self.msets, self.mset_of, self.seg_decl, self.seg_of, self.segs = [], {}, [], {}, []
        self.states, self.codewords, self.trees = {}, {}, {}

    def declare(self, name, items):
        self.units[name] = Unit(name, items, self.cmax)
        self.order.append(name)

    def nv(self):
        return max(c for u in self.units.values() for c, _ in u.classes)

    def merge(self, names):
        sid = len(self.msets)
        self.msets.append(names)
        for name in names:
            self.mset_of[name] = sid

    def segment_decl(self, names):
        i = len(self.seg_decl)
        self.seg_decl.append(names)
        for name in names:
            self.seg_of[name] = i

    def set_id(self, name):
        return self.mset_of[name] if name in self.mset_of else ("unit", name)

    def set_members(self, sid):
        return [sid[1]] if isinstance(sid, tuple) else self.msets[sid]

    def set_classes(self, sid):
        return sorted({c for name in self.set_members(sid) for c, _ in self.units[name].classes})

    def set_mixed(self, sid):
        classes = self.set_classes(sid)
        cm = classes[-1]
        lc = cap_level(1 << (cm - 1))
        return cm, [c for c in classes if cm - c <= lc]

    def set_trees(self, sid):
        _, mixed = self.set_mixed(sid)
        return [("mixed", sid)] + [("single", sid, c) for c in self.set_classes(sid) if c not in mixed]

    def tree_class(self, tid):
        return self.set_mixed(tid[1])[0] if tid[0] == "mixed" else tid[2]

    def tree_levels(self, tid):
        if tid[0] == "single":
            return self.b.merkle_levels(self.states[(tid[1], tid[2])], {})
        sid = tid[1]
        cm, mixed = self.set_mixed(sid)
        return self.b.merkle_levels(self.states[(sid, cm)], {cm - c: self.states[(sid, c)] for c in mixed if c != cm})

    def commit(self, name, tensors):
        unit, sid = self.units[name], self.set_id(name)
        unit.tensors = tensors
        for c, _ in unit.classes:
            codewords = self.b.encode(unit.columns(c, self.cmax), c)
            self.codewords[(name, c)] = codewords
            self.states[(sid, c)] = self.b.leaf_digests(codewords, c, self.states.get((sid, c)))
        if name == self.set_members(sid)[-1]:
            for tid in self.set_trees(sid):
                levels = self.tree_levels(tid)
                self.trees[tid] = levels
                cap = levels[cap_level(1 << (self.tree_class(tid) - 1))]
                self.tr.send_bytes(bytes(np.ascontiguousarray(cap, np.uint8).tobytes()))

    # -------------------------------------------------------------- opening (src/pcs.lisp:319-432)
    def combine(self, group):
        betas = self.tr.challenges(len(group))
        columns, claim = {}, zero(4)
        for (cd, value), beta in zip(group, betas):
            claim = orc.ext_add(claim, orc.ext_mul(beta, value))
            for k, coefficient in cd:
                columns[k] = orc.ext_add(columns.get(k, zero(4)), orc.ext_mul(beta, coefficient))
        return sorted(columns.items()), claim

    def reduce_points(self, c, groups, columns):
        combined = []
        for z, members in groups:
            comb, _ = self.combine(members)
            combined.append((z, comb))
        names, tables = [], []
        for i, (z, comb) in enumerate(combined):
            # g[x] = sum_k (ext-scale cf (aref column_k x)): combine-columns at F_p^4
            g = self.b.combine_columns([columns[k] for k, _ in comb], np.array([cf for _, cf in comb], np.uint32))
            names += ["E%d" % i, "G%d" % i]
            tables += [self.b.eq_table(z, 4), g]
        form = "(+ " + " ".join("(* E%d G%d)" % (i, i) for i in range(len(combined))) + ")"
        return self.b.prove_reduction(self.tr, c, form, names, tables)

    def max_points(self, c):
        return max(2, min(self.max_reduction_points, (8 << 30) // (2 * (1 << c) * 4 * 4)))

    def open(self, name, claims):
        unit = self.units[name]
        by_class = class_claims(unit, claims, self.cmax)
        self.tr.absorb(b"pcs-open|" + label_name(name).encode())
        for c, members in unit.classes:
            ncols = len(members)
            columns = unit.columns(c, self.cmax)
            groups = by_point(by_class.get(c, []))

            def receive(keys, rho):
                values = [(k, self.b.mle_eval(columns[k], rho, 4)) for k in keys]
                self.tr.send(np.array([v for _, v in values], np.uint32).reshape(len(keys), 4))
                return values

            while len(groups) > self.max_points(c):
                step, reduced = self.max_points(c), []
                for at in range(0, len(groups), step):
                    batch = groups[at:at + step]
                    r = self.reduce_points(c, batch, columns)
                    keys = sorted({k for _, cl in batch for cd, _ in cl for k, _ in cd})
                    values = receive(keys, r)
                    reduced.append((r, [([(k, one(4))], v) for k, v in values]))
                groups = reduced
            rho = self.reduce_points(c, groups, columns) if groups else [r for r in self.tr.challenges(c)]
            values = receive(list(range(ncols)), rho)
            alpha = self.tr.challenges(ncols, 8)
            y = ext_sum([orc.ext_mul(a, embed(v)) for a, (_, v) in zip(alpha, values)], 8)
            uc = Uc(unit, c, rho, alpha, y, ncols)
            uc.column = self.b.combine_columns(columns, alpha)
            self.ucs[(name, c)] = uc

    # -------------------------------------------------------------- the cross-unit sumcheck (src/pcs.lisp:445-516)
    def lam_scaled(self, lam, y, c, nv):
        return orc.ext_scale(orc.ext_mul(lam, y), orc.fpow(2, nv - c))

    def class_state(self, us, nv):
        states = []
        for c in sorted({u.c for u in us}):
            members = [u for u in us if u.c == c]
            const = ext_sum([self.lam_scaled(u.lam, u.y, c, nv) for u in members], 8)
            # (e * lambda per entry of eq-table: lambda times the table)
            e = np.concatenate([self.b.scale_add(None, u.lam, self.b.eq_table([embed(x) for x in u.rho], 8)) for u in members])
            v = np.concatenate([np.asarray(u.column, np.uint32).reshape(-1, 8) for u in members])
            states.append({"c": c, "const": const, "e": e, "v": v})
        return states

    def cross_rounds(self, states, nv, claim):
        inverse_2, r = orc.finv(2), []
        for j in range(nv):
            ev = [zero(8), zero(8), zero(8)]
            for s in states:
                if j < nv - s["c"]:
                    ev = [orc.ext_add(e, orc.ext_scale(s["const"], inverse_2)) for e in ev]
                else:
                    dp = self.b.dot_pairs(s["e"], s["v"])
                    ev = [orc.ext_add(e, dp[parity]) for parity, e in enumerate(ev)]
            self.tr.send(np.array(ev, np.uint32))
            assert np.array_equal(orc.ext_add(ev[0], ev[1]), claim), "cross-unit sumcheck round %d" % j
            x = self.tr.challenge(8)
            r.append(x)
            claim = orc.lagrange(np.array(ev), x)
            for s in states:
                if j < nv - s["c"]:
                    s["const"] = orc.ext_scale(s["const"], inverse_2)
                else:
                    s["e"], s["v"] = self.b.fold_table(s["e"], x), self.b.fold_table(s["v"], x)
        return r, claim

    def segment(self, i):
        nv, names = self.nv(), self.seg_decl[i]
        keys = [(name, c) for name in names for c, _ in self.units[name].classes]
        ucs = [self.ucs[k] for k in keys]
        self.tr.absorb(b"pcs-seg")
        for uc, lam in zip(ucs, self.tr.challenges(len(ucs), 8)):
            uc.lam = lam
        classes = sorted({u.c for u in ucs})
        states = self.class_state(ucs, nv)
        claim = ext_sum([self.lam_scaled(u.lam, u.y, u.c, nv) for u in ucs], 8)
        r, claim = self.cross_rounds(states, nv, claim)
        coefficients = [orc.ext_mul(u.lam, orc.ext_eq(np.array([embed(x) for x in u.rho]), np.array(r[nv - u.c:]), 8))
                        for u in ucs]
        ys = [ext_sum([orc.ext_mul(e, self.b.mle_eval(u.column, r[nv - c:], 8))
                       for u, e in zip(ucs, coefficients) if u.c == c], 8) for c in classes]
        self.tr.send(np.array(ys, np.uint32).reshape(len(classes), 8))
        assert np.array_equal(ext_sum(ys, 8), claim), "segment reduction"
        pus = []
        for c, y in zip(classes, ys):
            pu = Pu(c, r[nv - c:], y)
            h = None
            for u, e in zip(ucs, coefficients):
                if u.c == c:
                    h = self.b.scale_add(h, e, u.column)
            pu.column = h
            pus.append(pu)
        self.segs.append({"keys": keys, "coefficients": dict(zip(keys, coefficients)), "pus": pus})

    # -------------------------------------------------------------- finish (src/pcs.lisp:669-734)
    def finish(self):
        nv = self.nv()
        keys = [(name, c) for name in self.order for c, _ in self.units[name].classes]
        gkeys = [k for k in keys if k[0] not in self.seg_of]
        members = [self.ucs[k] for k in gkeys] + [pu for seg in self.segs for pu in seg["pus"]]
        self.tr.absorb(b"pcs-finish")
        for u, lam in zip(members, self.tr.challenges(len(members), 8)):
            u.lam = lam
        classes = sorted({u.c for u in members})
        claim = ext_sum([self.lam_scaled(u.lam, u.y, u.c, nv) for u in members], 8)
        rr, v = self.cross_rounds(self.class_state(members, nv), nv, claim)
        for u in members:
            u.sc = orc.ext_mul(u.lam, orc.ext_eq(np.array([embed(x) for x in u.rho]), np.array(rr[nv - u.c:]), 8))
        h = []
        for c in classes:
            hc = None
            for u in members:
                if u.c == c:
                    hc = self.b.scale_add(hc, u.sc, u.column)
            h.append((c, hc))
        qs = self.b.basefold_classes(self.tr, nv, h, np.array(rr), v, self.grind, self.queries)
        self.open_queries(keys, qs, nv)

    def open_queries(self, keys, qs, nv):
        last = {}
        for k in keys:
            last[self.set_id(k[0])] = k
        for name, c in keys:
            codewords = self.codewords[(name, c)]
            self.tr.record(self.b.gather_leaves(codewords, c, [q >> (nv - c) for q in qs]))
            if last[self.set_id(name)] == (name, c):
                for tid in self.set_trees(self.set_id(name)):
                    tc, levels = self.tree_class(tid), self.trees[tid]
                    lc = cap_level(1 << (tc - 1))
                    octets = b""
                    for q in qs:
                        i = q >> (nv - tc)
                        for level in levels[:lc]:
                            octets += bytes(np.ascontiguousarray(level[i ^ 1], np.uint8).tobytes())
                            i >>= 1
                    self.tr.record_bytes(octets)


def pcs_proof(scenario, backend=None):
    """PCS-PROOF (tests/tests.lisp:688-696): the claims and the proof bytes."""
    backend = backend or OracleBackend()
    state = SbclRandom(scenario["seed"])
    data = pcs_data(scenario["units"], state)
    claims = pcs_claims(scenario["units"], data, state)
    tr = backend.transcript("pcs-test", 4)
    pcs = Pcs(tr, scenario["cmax"], 6, 4, scenario.get("max_points", 64), backend)
    for name, items in scenario["units"]:
        pcs.declare(name, items)
    if scenario["merge"]:
        pcs.merge(scenario["merge"])
    if scenario["segment"]:
        pcs.segment_decl(scenario["segment"])
    for name, items in scenario["units"]:
        pcs.commit(name, {tensor: data[tensor] for tensor, _, _ in items})
    for name, unit_claims in claims:
        pcs.open(name, unit_claims)
        if scenario["segment"] and name == scenario["segment"][-1]:
            pcs.segment(0)
    pcs.finish()
    return claims, tr.proof()


def _ints(a):
    return "[" + ",".join(str(int(v)) for v in np.asarray(a).reshape(-1)) + "]"


def _exts(es):
    return "[" + ",".join(_ints(e) for e in es) + "]"


def pcs_cases_text(backend=None):
    """EXPORT-PCS-CASES (tests/tests.lisp:728-758)."""
    out = ["[\n"]
    for i, sc in enumerate(SCENARIOS):
        claims, proof = pcs_proof(sc, backend)
        units = ",".join('{"name": "%s", "items": [%s]}' % (name, ",".join('["%s", %d, %d]' % item for item in items))
                         for name, items in sc["units"])
        claimed = ",".join('{"unit": "%s", "claims": [%s]}' % (name, ",".join(
            '{"tensor": "%s", "point": %s, "coefficients": {%s}, "value": %s}'
            % (tensor, _exts(point), ",".join('"%d": %s' % (b, _ints(w)) for b, w in coefficients), _ints(value))
            for tensor, point, coefficients, value in unit_claims)) for name, unit_claims in claims)
        out.append('{"label": "pcs-test", "cmax": %d, "max_points": %d, "queries": 6, "grind": 4, "units": [%s], '
                   '"merge": [%s], "segment": [%s], "claims": [%s], "proof": "%s"}%s\n'
                   % (sc["cmax"], sc.get("max_points", 64), units, ",".join('"%s"' % m for m in (sc["merge"] or [])),
                      ",".join('"%s"' % m for m in (sc["segment"] or [])), claimed, proof.hex(),
                      "," if i + 1 < len(SCENARIOS) else ""))
    out.append("]\n")
    return "".join(out)
