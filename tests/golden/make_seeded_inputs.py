"""Regenerates tests/golden/seeded_m11_k512_n21.npz.

The reference's seeded full-path tests (candle-core/tests/quantized_tests.rs:874-894)
draw their inputs from rand 0.8.5's `StdRng::seed_from_u64(314159265358979)`:
m*k values for lhs, then n*k for rhs, each `rng.gen::<f32>() - 0.5`.  This script
restates that generator (rand_core 0.6 `seed_from_u64` = PCG32 key expansion;
`StdRng` = ChaCha with 12 rounds, 64-bit block counter, stream 0; `gen::<f32>()` =
`(next_u32() >> 8) * 2^-24`) and writes the inputs as a fixture.  The generator is
self-validated: f32 `lhs @ rhs.T` at flat indices [0, 77, 154, 230] must round to
[1.262, 1.513, -0.208, 1.702] (quantized_tests.rs:1008).

Run:  python tests/golden/make_seeded_inputs.py
"""
import os

import numpy as np

M64 = (1 << 64) - 1
M32 = (1 << 32) - 1


def seed_from_u64(state: int) -> bytes:
    key = b""
    for _ in range(8):
        state = (state * 6364136223846793005 + 11634580027462260723) & M64
        xorshifted = (((state >> 18) ^ state) >> 27) & M32
        rot = state >> 59
        x = ((xorshifted >> rot) | (xorshifted << ((32 - rot) & 31))) & M32
        key += x.to_bytes(4, "little")
    return key


def rotl(v, n):
    return ((v << n) & M32) | (v >> (32 - n))


def chacha_block(key_words, counter: int, rounds: int = 12):
    st = [0x61707865, 0x3320646E, 0x79622D32, 0x6B206574] + list(key_words) + [
        counter & M32, (counter >> 32) & M32, 0, 0]
    w = list(st)

    def qr(a, b, c, d):
        w[a] = (w[a] + w[b]) & M32; w[d] = rotl(w[d] ^ w[a], 16)
        w[c] = (w[c] + w[d]) & M32; w[b] = rotl(w[b] ^ w[c], 12)
        w[a] = (w[a] + w[b]) & M32; w[d] = rotl(w[d] ^ w[a], 8)
        w[c] = (w[c] + w[d]) & M32; w[b] = rotl(w[b] ^ w[c], 7)

    for _ in range(rounds // 2):
        qr(0, 4, 8, 12); qr(1, 5, 9, 13); qr(2, 6, 10, 14); qr(3, 7, 11, 15)
        qr(0, 5, 10, 15); qr(1, 6, 11, 12); qr(2, 7, 8, 13); qr(3, 4, 9, 14)
    return [(w[i] + st[i]) & M32 for i in range(16)]


def std_rng_f32(seed: int, count: int) -> np.ndarray:
    key = seed_from_u64(seed)
    kw = [int.from_bytes(key[4 * i:4 * i + 4], "little") for i in range(8)]
    out = np.empty(count, dtype=np.float32)
    i, ctr = 0, 0
    while i < count:
        for word in chacha_block(kw, ctr):
            if i >= count:
                break
            out[i] = np.float32(word >> 8) * np.float32(2.0 ** -24)
            i += 1
        ctr += 1
    return out


def main():
    m, k, n = 11, 512, 21
    vals = std_rng_f32(314159265358979, m * k + n * k) - np.float32(0.5)
    lhs = vals[: m * k].reshape(m, k)
    rhs = vals[m * k:].reshape(n, k)
    mm = (lhs.astype(np.float64) @ rhs.astype(np.float64).T).astype(np.float32).ravel()
    spot = [round(float(mm[i]), 3) for i in (0, m * n // 3, m * n * 2 // 3, m * n - 1)]
    assert spot == [1.262, 1.513, -0.208, 1.702], spot
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "seeded_m11_k512_n21.npz")
    np.savez_compressed(out, lhs=lhs, rhs=rhs)
    print("wrote", out, spot)


if __name__ == "__main__":
    main()
