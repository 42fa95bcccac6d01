"""SBCL's pseudo-random numbers for a seeded state, as the reference's own tests draw their inputs:
`(sb-ext:seed-random-state k)` followed by `(random bound state)` (tests/tests.lisp:399-406, 487-512 and the
exporters behind *FROZEN-CASES*, tests/tests.lisp:902-925).

SBCL is the reference's compiler, not part of its sources (README.md:114-149 names SBCL 2.2.9); what is restated
here is its published generator (src/code/target-random.lisp): MT19937 with the standard seeding recurrence for an
integer seed below 2^32 (`init-random-state`), 32-bit tempered chunks (`random-chunk`), and for an integer bound the
accept-reject loop over the chunk's low `integer-length (bound - 1)` bits (`%random-fixnum`).  Nothing pins this
file by itself; the frozen digests do: a proof of the oracle over inputs drawn here hashes to the reference's own
SHA-256 only if generator, inputs, protocol and wire format all agree (tests/test_oracle_frozen_cases.py)."""


class SbclRandom:
    def __init__(self, seed):
        if not 0 <= seed < 1 << 32:
            raise ValueError("integer seeds below 2^32 only")
        s, mt = seed, [0] * 624
        mt[0] = s
        for i in range(1, 624):
            s = (1812433253 * (s ^ (s >> 30)) + i) & 0xFFFFFFFF
            mt[i] = s
        self.mt, self.k = mt, 624

    def _update(self):
        mt = self.mt
        for i in range(624):
            y = (mt[i] & 0x80000000) | (mt[(i + 1) % 624] & 0x7FFFFFFF)
            mt[i] = mt[(i + 397) % 624] ^ (y >> 1) ^ (0x9908B0DF if y & 1 else 0)
        self.k = 0

    def chunk(self):
        if self.k == 624:
            self._update()
        y = self.mt[self.k]
        self.k += 1
        y ^= y >> 11
        y ^= (y << 7) & 0x9D2C5680
        y ^= (y << 15) & 0xEFC60000
        y ^= y >> 18
        return y & 0xFFFFFFFF

    def random(self, bound):
        """(random bound state) for an integer 1 <= bound <= 2^32."""
        if bound == 1:
            return 0
        mask = (1 << (bound - 1).bit_length()) - 1
        while True:
            v = self.chunk() & mask
            if v < bound:
                return v
