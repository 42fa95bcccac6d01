"""A tiny pure-Python model of F_p[w]/(w^D - 3) in tower order, written from the mathematics
(polynomial multiplication, bit-reversed coordinates), independent of the C oracle: tests use it for
brute-force checks on small cases."""
P = 2130706433


def _rev(d):
    bits = d.bit_length() - 1
    return [int(format(i, f"0{bits}b")[::-1], 2) if bits else 0 for i in range(d)]


def add(a, b): return [(x + y) % P for x, y in zip(a, b)]
def sub(a, b): return [(x - y) % P for x, y in zip(a, b)]
def scale(a, s): return [x * s % P for x in a]
def lift(v, d): return [v % P] + [0] * (d - 1)


def mul(a, b):
    d = len(a)
    rev = _rev(d)
    pa, pb = [a[rev[e]] for e in range(d)], [b[rev[e]] for e in range(d)]
    c = [0] * d
    for i in range(d):
        for j in range(d):
            k = i + j
            if k < d:
                c[k] = (c[k] + pa[i] * pb[j]) % P
            else:
                c[k - d] = (c[k - d] + 3 * pa[i] * pb[j]) % P
    return [c[rev[i]] for i in range(d)]


def eq_table(r, d):
    """eq(r, x) for x in {0,1}^k, bit b of x paired with r[b], from the definition."""
    one = lift(1, d)
    out = []
    for x in range(1 << len(r)):
        e = one
        for b, rb in enumerate(r):
            e = mul(e, rb if (x >> b) & 1 else sub(one, rb))
        out.append(e)
    return out


def evaluate(form, values, d):
    """A form (nested list) over F_p^D by direct recursion."""
    if isinstance(form, int):
        return lift(form, d)
    if isinstance(form, str):
        return values[form.upper()]
    op, args = form[0], [evaluate(a, values, d) for a in form[1:]] if form[0] not in ("expt", "EXPT") else None
    if op == "+":
        out = lift(0, d)
        for a in args:
            out = add(out, a)
        return out
    if op == "*":
        out = lift(1, d)
        for a in args:
            out = mul(out, a)
        return out
    if op == "-":
        if len(args) == 1:
            return sub(lift(0, d), args[0])
        out = args[0]
        for a in args[1:]:
            out = sub(out, a)
        return out
    base, k = evaluate(form[1], values, d), form[2]
    out = lift(1, d)
    for _ in range(k):
        out = mul(out, base)
    return out
