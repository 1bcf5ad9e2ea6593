"""Restatement of rand 0.9 `StdRng::seed_from_u64` + `random::<f32>()`.

The reference's seeded mat-mul tests (candle-core/tests/quantized_tests.rs:928-948) draw
their operands from `StdRng::seed_from_u64(314159265358979)`.  rand 0.9 is not vendored in
the reference tree, so its published algorithm is restated here:
  * rand_core 0.9 `SeedableRng::seed_from_u64`: a PCG32 stream (multiplier
    6364136223846793005, increment 11634580027462260723) expands the u64 into the 32-byte seed;
  * `StdRng` = ChaCha12 (rand_chacha 0.9), 64-bit block counter starting at 0, stream 0,
    output words consumed in order;
  * `StandardUniform` for f32: `(next_u32() >> 8) as f32 * 2^-24`.
The restatement is validated by the reference's own *dense* expected values
(quantized_tests.rs:1108-1110: [1.262, 1.513, -0.208, 1.702]), which depend on nothing else.
"""
import numpy as np

M64 = (1 << 64) - 1


def _pcg32_seed(state):
    out = []
    for _ in range(8):
        state = (state * 6364136223846793005 + 11634580027462260723) & M64
        xorshifted = (((state >> 18) ^ state) >> 27) & 0xFFFFFFFF
        rot = state >> 59
        x = ((xorshifted >> rot) | (xorshifted << ((32 - rot) & 31))) & 0xFFFFFFFF
        out.append(x)
    return out  # eight little-endian u32 words = the 32-byte key


def _rotl(x, n):
    return ((x << np.uint32(n)) | (x >> np.uint32(32 - n)))


def _chacha_blocks(key_words, first_block, nblocks, rounds=12):
    """Vectorised over blocks; returns uint32 array [nblocks, 16]."""
    ctr = np.arange(first_block, first_block + nblocks, dtype=np.uint64)
    s = np.zeros((16, nblocks), dtype=np.uint32)
    s[0], s[1], s[2], s[3] = 0x61707865, 0x3320646E, 0x79622D32, 0x6B206574
    for i in range(8):
        s[4 + i] = key_words[i]
    s[12] = (ctr & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    s[13] = (ctr >> np.uint64(32)).astype(np.uint32)
    x = s.copy()

    def qr(a, b, c, d):
        x[a] += x[b]; x[d] = _rotl(x[d] ^ x[a], 16)
        x[c] += x[d]; x[b] = _rotl(x[b] ^ x[c], 12)
        x[a] += x[b]; x[d] = _rotl(x[d] ^ x[a], 8)
        x[c] += x[d]; x[b] = _rotl(x[b] ^ x[c], 7)

    with np.errstate(over="ignore"):
        for _ in range(rounds // 2):
            qr(0, 4, 8, 12); qr(1, 5, 9, 13); qr(2, 6, 10, 14); qr(3, 7, 11, 15)
            qr(0, 5, 10, 15); qr(1, 6, 11, 12); qr(2, 7, 8, 13); qr(3, 4, 9, 14)
        x += s
    return x.T.copy()


def std_rng_f32(seed, n):
    """First n values of `rng.random::<f32>()` for `StdRng::seed_from_u64(seed)`."""
    key = _pcg32_seed(seed)
    nblocks = (n + 15) // 16
    words = _chacha_blocks(key, 0, nblocks).reshape(-1)[:n]
    return (words >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / (1 << 24))
