"""Statement forms as data, restated from the reference's src/forms.lisp:28-109 (test oracle).

A form is an int, a variable name (str), or a list [op, arg...] with op in '+', '-', '*', 'expt'.
`read_form` parses the s-expression text the reference writes, e.g. "(+ (* alpha t0 t1 t2) (* 3 t1))".
`expand` gives the canonical sum of monomials: a list of (monomial, coefficient) with each monomial a
sorted tuple of variable names, like terms merged, zero terms dropped, in graded order
(src/forms.lisp:57-78).  Variable names compare as upper-case strings, as Lisp symbol names do.
"""
P = 2130706433


def read_form(text):
    tokens = text.replace("(", " ( ").replace(")", " ) ").split()
    pos = 0

    def parse():
        nonlocal pos
        tok = tokens[pos]
        pos += 1
        if tok == "(":
            out = []
            while tokens[pos] != ")":
                out.append(parse())
            pos += 1
            return out
        if tok == ")":
            raise ValueError("unbalanced form")
        try:
            return int(tok)
        except ValueError:
            return tok.upper()

    form = parse()
    if pos != len(tokens):
        raise ValueError("trailing tokens in form")
    return form


def _monomial_key(m):
    return (len(m), m)


def _collect(terms):
    table = {}
    for m, c in terms:
        table[m] = (table.get(m, 0) + c) % P
    return sorted(((m, c) for m, c in table.items() if c), key=lambda t: _monomial_key(t[0]))


def expand(form):
    if isinstance(form, bool):
        raise ValueError("malformed form")
    if isinstance(form, int):
        return _collect([((), form % P)])
    if isinstance(form, str):
        return [((form.upper(),), 1)]
    if isinstance(form, (list, tuple)) and form:
        op, args = form[0], list(form[1:])
        if op == "+":
            return _collect([t for a in args for t in expand(a)])
        if op == "-":
            if not args:
                raise ValueError("malformed form")
            first = expand(args[0])
            if len(args) == 1:
                return [(m, (-c) % P) for m, c in first]
            rest = [(m, (-c) % P) for a in args[1:] for m, c in expand(a)]
            return _collect(first + rest)
        if op == "*":
            acc = expand(1)
            for a in args:
                b = expand(a)
                acc = _collect([(tuple(sorted(m1 + m2)), c1 * c2 % P) for m1, c1 in acc for m2, c2 in b])
            return acc
        if op in ("expt", "EXPT"):
            base, k = args
            if not isinstance(k, int) or k < 0:
                raise ValueError("malformed form")
            return expand(["*"] + [base] * k)
    raise ValueError("malformed form: %r" % (form,))


def form_variables(form):
    return sorted({v for m, _ in expand(form) for v in m})


def form_degree(form, variables=None):
    best = 0
    for m, _ in expand(form):
        d = len(m) if variables is None else sum(1 for v in m if v in variables)
        best = max(best, d)
    return best


def constant_term(form):
    for m, c in expand(form):
        if m == ():
            return c
    return 0


def evaluate_base(form, values):
    """The form over F_p by direct recursion (not through expand): a cross-check of expand."""
    if isinstance(form, int):
        return form % P
    if isinstance(form, str):
        return values[form.upper()] % P
    op, args = form[0], form[1:]
    vals = [evaluate_base(a, values) for a in args]
    if op == "+":
        return sum(vals) % P
    if op == "*":
        out = 1
        for v in vals:
            out = out * v % P
        return out
    if op == "-":
        return (-vals[0]) % P if len(vals) == 1 else (vals[0] - sum(vals[1:])) % P
    if op in ("expt", "EXPT"):
        return pow(evaluate_base(args[0], values), args[1], P)
    raise ValueError("malformed form")
