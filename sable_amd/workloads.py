"""The five configured workloads as data: statements, sizes, seeds and transcript labels.

Nothing here computes; the benchmark, the parity tests and the script that writes the full-size fixtures all
read their shapes from this one place, so that a proof hash means the same inputs everywhere.  Synthetic field
elements come from SplitMix64(seed): each output's top 31 bits, kept when below p (the rule of the
transcript's own challenges, src/transcript.lisp:159-164) -- `Table.random` on the device side.
"""

P = 2130706433

# sumcheck configurations: table k is seeded with seed * 1000 + k, the eq point with seed + 900 (n * D
# elements), the constants with seed + 901
SUMCHECK = {
    "config1": dict(form="(* t0 t1)", tables=["t0", "t1"], constants=[], n=16, d=4, seed=1),
    "config2": dict(form="(+ (* alpha t0 t1 t2) (* 3 t1))", tables=["t0", "t1", "t2"], constants=["alpha"], n=24, d=4,
                    seed=2),
    "config3": dict(form="(* (+ c0 3) (- c1 c0) c2 c3)", tables=["c0", "c1", "c2", "c3"], constants=[], n=26, d=8,
                    seed=3),
    # A statement wider than the table groups' kernels hold: the leaf-layer and zerocheck statement of the
    # reference's toy domain (tests/tests.lisp:487-512 through src/domain.lisp:95-114: three lookups, three
    # constraints, every kind of column; 41 table monomials), over seeded tables instead of a witness -- the
    # prover's work does not depend on the constraints holding.
    "domain": dict(
        form="(+ (* %A0 (+ (- %Z 5 (* %BETA0 A@0) (* %BETA1 B@0)) (- %Z 5 (* %BETA0 A@1) (* %BETA1 B@1))))"
             " (* %AL0 (- %Z 5 (* %BETA0 A@0) (* %BETA1 B@0)) (- %Z 5 (* %BETA0 A@1) (* %BETA1 B@1)))"
             " (* %A1 (+ (* (+ S@0 2) (- %Z 7 (* %BETA0 C@1) (* %BETA1 M@1) (* %BETA2 W)))"
             " (* (+ S@1 2) (- %Z 7 (* %BETA0 C@0) (* %BETA1 M@0) (* %BETA2 W)))))"
             " (* %AL1 (- %Z 7 (* %BETA0 C@0) (* %BETA1 M@0) (* %BETA2 W)) (- %Z 7 (* %BETA0 C@1) (* %BETA1 M@1) (* %BETA2 W)))"
             " (* %A2 (+ (- %Z 9 (* %BETA0 KB)) (- %Z 9 (* %BETA0 KB)))) (* %AL2 (- %Z 9 (* %BETA0 KB)) (- %Z 9 (* %BETA0 KB)))"
             " (* %GAM0 (* A@0 (- A@0 1))) (* %GETA0 (* A@1 (- A@1 1))) (* %GAM1 (- C@0 (* A@0 B@0)))"
             " (* %GETA1 (- C@1 (* A@1 B@1))) (* %GAM2 (* S@0 (- S@0 1) M@0)) (* %GETA2 (* S@1 (- S@1 1) M@1)))",
        tables=["A@0", "A@1", "B@0", "B@1", "C@0", "C@1", "M@0", "M@1", "S@0", "S@1", "W", "KB"],
        constants=["%Z", "%BETA0", "%BETA1", "%BETA2", "%A0", "%AL0", "%A1", "%AL1", "%A2", "%AL2", "%GAM0", "%GETA0",
                   "%GAM1", "%GETA1", "%GAM2", "%GETA2"],
        n=20, d=4, seed=7),
}


def table_seed(cfg, k):
    return cfg["seed"] * 1000 + k


def eq_seed(cfg):
    return cfg["seed"] + 900


def constants_seed(cfg):
    return cfg["seed"] + 901


# config 4, LogUp-GKR: 2^22 lookups of int8-range values into the 2^16-entry range table t_j = j - 32768 with
# exact multiplicities.  Lookup i is (w_i & 255) - 128 with w the field elements of seed 4004; Z is the first
# challenge of a transcript labelled "config4-z"; the witness tree (leaves 1 / (Z - v_i), n = 22) is proved on a
# transcript labelled "config4-w", the table tree (leaves m_j / (Z - t_j), n = 16) on "config4-t".
GKR = dict(d=4, n_witness=22, n_table=16, seed=4004, z_label="config4-z", witness_label="config4-w",
           table_label="config4-t")


def gkr_leaves(np, words, z, n_witness, n_table, d=4):
    """Host arrays of the two trees' leaves, ((p, q) witness, (p, q) table), from the seeded words and Z."""
    values = (words[: 1 << n_witness].astype(np.int64) & 255) - 128
    half = 1 << (n_table - 1)
    table = np.arange(1 << n_table, dtype=np.int64) - half
    mult = np.bincount(values + half, minlength=1 << n_table)

    def leaves(num, val):
        p = np.zeros((len(num), d), np.uint32)
        p[:, 0] = np.asarray(num, np.int64) % P
        q = np.tile(np.asarray(z, np.int64), (len(val), 1))
        q[:, 0] = (q[:, 0] - np.asarray(val, np.int64)) % P
        return p, q.astype(np.uint32)

    return leaves(np.ones(1 << n_witness, np.int64), values), leaves(mult, table)


# config 5, commitment: 2^24 coefficients as two columns of 2^23 (one seeded run of 2^24 elements), encoded to
# two codewords of 2^24, 2^22 leaves, cap of 128; then BaseFold of the columns' F_p^8 combination (coefficients
# seeded 5006) at the point seeded 5007, on a transcript labelled "config5-bf".
COMMIT = dict(c=23, ncols=2, seed=5005, label="config5", coefficient_seed=5006, point_seed=5007, open_label="config5-bf",
              grind_bits=4, queries=6)
