"""Writes tests/golden/sq5_kat.json: known-answer vectors for the Squirrel5 noise.

The reference (Clyde013/randumb) ships no tests or golden vectors, so these answers are
derived here from the closed form with nothing but Python's arbitrary-precision integers
(explicit ``& 0xFFFFFFFF`` after every step) and ``struct`` for the fp32 rounding - no NumPy,
no oracle module, no reference code.  The constants and step order restate
src/rten_cpp/RandumbTensor.py:140-163 and src/rten_cpp/csrc/cuda/rten.cu:13-47.

Run:  python tests/golden/make_sq5_kat.py
"""
import json
import os
import random
import struct

M32 = 0xFFFFFFFF
N1, N2, N3, N4, N5 = 0xD2A80A3F, 0xA884F197, 0x6C736F4B, 0xB79F3ABB, 0x1B56C4F5
PRIME = 198491317


def mangle(idx, seed):
    b = idx & M32
    b = (b * N1) & M32
    b = (b + seed) & M32
    b ^= b >> 9
    b = (b + N2) & M32
    b ^= b >> 11
    b = (b * N3) & M32
    b ^= b >> 13
    b = (b + N4) & M32
    b ^= b >> 15
    b = (b * N5) & M32
    b ^= b >> 17
    return b


def to_f32(bits):
    """int32(bits) rounded to fp32 (nearest even, via struct) times 2**-31 (exact)."""
    s = bits - (1 << 32) if bits >> 31 else bits
    f = struct.unpack("<f", struct.pack("<f", float(s)))[0]  # float(s) is exact in fp64; pack rounds RNE
    return f * 2.0 ** -31


def main():
    rng = random.Random(20250607)
    one_d = [(0, 0), (1, 0), (0, 1337), (1, 1337), (2, 1337), (198491317, 1337), (0xFFFFFFFF, 1337),
             (12345678, 42), (0x80000000, 7), (0x7FFFFFFF, 2 ** 31 - 1), (3, 0xFFFFFFFF)]
    one_d += [(rng.getrandbits(32), rng.getrandbits(31)) for _ in range(40)]
    two_d = [(1, 0, 1337), (3, 5, 1337), (767, 255, 0), (2359295, 255, 47), (58720255, 1023, 11),
             (0, 0, 0), (4095, 15, 1337), (21, 63, 1338)]
    two_d += [(rng.getrandbits(26), rng.getrandbits(10), rng.getrandbits(31)) for _ in range(40)]
    out = {"one_d": [], "two_d": []}
    for idx, seed in one_d:
        b = mangle(idx, seed)
        out["one_d"].append({"idx": idx, "seed": seed, "bits": b, "f32_hex": to_f32(b).hex()})
    for n, m, seed in two_d:
        a = (PRIME * n + m) & M32
        b = mangle(a, seed)
        out["two_d"].append({"n": n, "m": m, "seed": seed, "addr": a, "bits": b, "f32_hex": to_f32(b).hex()})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sq5_kat.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path, len(out["one_d"]), len(out["two_d"]))


if __name__ == "__main__":
    main()
