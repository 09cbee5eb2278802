"""Philox-4x64-10 in plain Python integers.

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  The reference draws its random inputs from the
backend's NumPy-compatible `random` module (delayrepay/random.py:6-13) and has no
generator of its own; the device generator of this repository (`random.device`) is
specified as "the stream of `numpy.random.Philox`", so NumPy is the oracle for it.
This file restates the algorithm NumPy implements (Salmon, Moraes, Dror, Shaw:
"Parallel random numbers: as easy as 1, 2, 3", SC'11, section 3.2; multipliers and
Weyl constants of the 4x64 variant) independently of both NumPy and the kernel text, so
that the tests can tell a wrong constant or a transposed word from a matching pair of
mistakes.  Pinned in tests/test_oracle.py against NumPy's generator and against the
paper's known-answer vectors for the all-zero and all-ones inputs.
"""
M64 = (1 << 64) - 1
MUL0, MUL1 = 0xD2E7470EE14C6C93, 0xCA5A826395121157
WEYL0, WEYL1 = 0x9E3779B97F4A7C15, 0xBB67AE8584CAA73B


def block(counter, key, rounds=10):
    """The four 64-bit outputs for a 256-bit `counter` and a 128-bit `key` (integers)."""
    x = [(counter >> (64 * i)) & M64 for i in range(4)]
    k0, k1 = key & M64, (key >> 64) & M64
    for _ in range(rounds):
        p0 = MUL0 * x[0]
        p1 = MUL1 * x[2]
        x = [(p1 >> 64) ^ x[1] ^ k0, p1 & M64, (p0 >> 64) ^ x[3] ^ k1, p0 & M64]
        k0 = (k0 + WEYL0) & M64
        k1 = (k1 + WEYL1) & M64
    return x


def stream(key, counter, n, skip=0):
    """Outputs skip .. skip+n-1 of the stream NumPy's `Philox(key=key, counter=counter)`
    produces: NumPy steps the counter before it makes a block, so output 0 is word 0 of
    the block at counter + 1."""
    out = []
    for r in range(skip, skip + n):
        out.append(block((counter + 1 + r // 4) % (1 << 256), key)[r % 4])
    return out


def doubles(words):
    """Doubles in [0, 1) from raw outputs: the top 53 bits scaled by 2^-53."""
    return [(w >> 11) * (1.0 / 9007199254740992.0) for w in words]
