#!/usr/bin/env python3
"""Convert the reference's golden-vector data file (tests/vectors.sexp, 103 vectors written by
Sable's original Python implementation) into tests/golden/vectors.json.

The input is a data file: one s-expression holding plists of integers, strings and nested lists.
This script only reads that data (it executes nothing from the reference) and re-emits it as JSON:

    (:kind :key value ...)  ->  {"kind": "kind", "key": value, ...}
    (a b c) -> [a, b, c]     () -> []     nil -> null     t -> true     "..." -> string

Run in the build container only (the reference tree does not travel):

    python tests/golden/make_vectors.py [/root/reference/tests/vectors.sexp]
"""
import json
import os
import sys


def tokenize(text):
    i, n = 0, len(text)
    while i < n:
        c = text[i]
        if c == ";":
            while i < n and text[i] != "\n":
                i += 1
        elif c.isspace():
            i += 1
        elif c in "()":
            yield c
            i += 1
        elif c == '"':
            j = text.index('"', i + 1)
            yield ("str", text[i + 1:j])
            i = j + 1
        else:
            j = i
            while j < n and not text[j].isspace() and text[j] not in "()":
                j += 1
            yield ("atom", text[i:j])
            i = j


def parse(tokens):
    stack = [[]]
    for tok in tokens:
        if tok == "(":
            stack.append([])
        elif tok == ")":
            done = stack.pop()
            stack[-1].append(done)
        else:
            kind, value = tok
            if kind == "str":
                stack[-1].append(value)
            elif value.startswith(":"):
                stack[-1].append({"kw": value[1:]})
            elif value.lower() == "nil":
                stack[-1].append(None)
            elif value.lower() == "t":
                stack[-1].append(True)
            else:
                stack[-1].append(int(value))
    assert len(stack) == 1 and len(stack[0]) == 1
    return stack[0][0]


def vector(form):
    out = {"kind": form[0]["kw"]}
    rest = form[1:]
    assert len(rest) % 2 == 0
    for k, v in zip(rest[0::2], rest[1::2]):
        out[k["kw"].replace("-", "_")] = v
    return out


def main():
    src = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/tests/vectors.sexp"
    with open(src) as f:
        forms = parse(tokenize(f.read()))
    vectors = [vector(form) for form in forms]
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.json")
    with open(dst, "w") as f:
        f.write("[\n")
        f.write(",\n".join(json.dumps(v, separators=(",", ":")) for v in vectors))
        f.write("\n]\n")
    print(f"{len(vectors)} vectors -> {dst}")


if __name__ == "__main__":
    main()
