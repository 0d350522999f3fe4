"""CPU oracle for ``TritonHub.Layers.Dropout``, forward + backward (TEST INFRASTRUCTURE ONLY).

numpy restatement of the reference's ``TritonHub/Layers/dropout.py``; imported by ``tests/`` only.

The kernel (dropout.py:12-23, the backward :56-67 is the same function of ``dout``) works on the flattened tensor:
``rand_p = tl.rand(seed, cols)``; ``y = where(rand_p < p, 0, x / (1 - p))``, with ``cols`` the flat element index,
``p`` a float32 scalar, ``1 - p`` and the quotient in float32 (float64 storage: float64 quotient by the float32
``1 - p``), rounded to the storage type on store.  ``p == 0`` or eval mode return the input, ``p == 1`` zeros
(dropout.py:29-32).

``tl.rand`` is not part of the reference: it is Triton's (``triton/language/random.py``; setup.py:14 of the reference
requires ``triton`` without a version, this image holds 3.6.0).  Its published algorithm, restated here:
  * ``randint(seed, offset)``: the first of the four output words of Philox-4x32 with 10 rounds (Salmon, Moraes, Dror,
    Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11; multipliers 0xD2511F53 / 0xCD9E8D57, key increments
    0x9E3779B9 / 0xBB67AE85), counter = (offset, 0, 0, 0) for 32-bit offsets -- (low word, high word, 0, 0) for 64-bit
    ones -- and key = (low word of seed, high word of seed);
  * ``rand``: that word as int32 ``v``, folded to non-negative (``v < 0 ? -v - 1 : v``), converted to float32 and
    multiplied by float32(4.6566127342e-10): a float32 in [0, 1).

Pinned in tests/test_dropout_oracle_pins.py: ``philox4x32_10`` against the known-answer vectors of the Random123
distribution (kat_vectors), ``randint`` / ``rand`` bit for bit against tests/golden/dropout_golden.npz (written by
tests/golden/make_dropout_golden.py, which runs ``tl.randint`` / ``tl.rand`` of Triton 3.6.0 in its CPU interpreter),
and the keep rate against the binomial bound.
"""
import numpy as np

ROUND_A, ROUND_B = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
KEY_A, KEY_B = 0x9E3779B9, 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)
RAND_SCALE = np.float32(4.6566127342e-10)


def philox4x32_10(counter, key, rounds=10):
    """counter: four uint32 arrays (or scalars), key: two Python ints -> four uint32 arrays."""
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint64) & MASK32 for c in counter)
    c0, c1, c2, c3 = np.broadcast_arrays(c0, c1, c2, c3)
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(rounds):
        pa = ROUND_A * c0                       # 32 x 32 -> 64 bit products, exact in uint64
        pb = ROUND_B * c2
        c0, c1, c2, c3 = ((pb >> np.uint64(32)) ^ c1 ^ np.uint64(k0), pb & MASK32,
                          (pa >> np.uint64(32)) ^ c3 ^ np.uint64(k1), pa & MASK32)
        k0 = (k0 + KEY_A) & 0xFFFFFFFF
        k1 = (k1 + KEY_B) & 0xFFFFFFFF
    return tuple(c.astype(np.uint32) for c in (c0, c1, c2, c3))


def randint(seed, offsets):
    """tl.randint(seed, offsets): int32.  `offsets`: integer array; values of 2^32 and more use the 64-bit form."""
    off = np.asarray(offsets, dtype=np.uint64)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    zero = np.zeros_like(off)
    word, _, _, _ = philox4x32_10((off & MASK32, off >> np.uint64(32), zero, zero), (seed & 0xFFFFFFFF, seed >> 32))
    return word.view(np.int32)


def rand(seed, offsets):
    """tl.rand(seed, offsets): float32 in [0, 1)."""
    v = randint(seed, offsets).astype(np.int64)
    v = np.where(v < 0, -v - 1, v)
    return v.astype(np.float32) * RAND_SCALE           # int -> float32 rounds to nearest even, as sitofp does


def dropout(x, p, seed, first_offset=0):
    """The kernel on a tensor in its storage type (numpy float32 / float64, or float32 holding 16-bit values whose
    result the caller rounds): x flattened in row-major order, element i uses offset first_offset + i."""
    x = np.asarray(x)
    p32 = np.float32(p)
    keep_div = np.float32(1.0) - p32
    flat = x.reshape(-1)
    r = rand(seed, np.arange(flat.size, dtype=np.uint64) + np.uint64(first_offset))
    if flat.dtype == np.float64:
        q = flat / np.float64(keep_div)
    else:
        q = flat.astype(np.float32) / keep_div
    return np.where(r < p32, np.zeros_like(q), q).reshape(x.shape)
