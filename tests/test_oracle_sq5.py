"""Pins the oracle's Squirrel5 noise: known answers, three spellings, edge cases.

Restates nothing from the oracle: the known-answer table was derived separately with
big-int Python (tests/golden/make_sq5_kat.py) and a second table is quoted from the
written structural analysis of the reference (values derived there by hand from
src/rten_cpp/RandumbTensor.py:140-163).
"""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "sq5_kat.json")

# (idx, seed) -> (bits, float) and (n, m, seed) -> (addr, bits, float), from the analysis document.
ANALYSIS_1D = [
    (0, 0, 0x16791E00, 0.17557120323181152),
    (1, 0, 0xC895CB1D, -0.4329286813735962),
    (0, 1337, 0x9F42372D, -0.7557917833328247),
    (1, 1337, 0x77EA941E, 0.9368462562561035),
    (2, 1337, 0xF520803C, -0.08494564890861511),
    (198491317, 1337, 0xB0083F71, -0.6247482895851135),
    (0xFFFFFFFF, 1337, 0x1646088D, 0.17401224374771118),
    (12345678, 42, 0x432DC9A2, 0.5248348116874695),
]
ANALYSIS_2D = [
    (1, 0, 1337, 0x0BD4BCB5, 0xB0083F71, -0.6247482895851135),
    (3, 5, 1337, 0x237E3624, 0xD52296C6, -0.3348819315433502),
    (767, 255, 0, 0x7261634A, 0x880D8622, -0.9370872974395752),
    (2359295, 255, 47, 0x7D9F444A, 0x17C0668C, 0.18555909395217896),
]


def test_known_answers_from_analysis(oracle):
    L = oracle.lib()
    for idx, seed, bits, f in ANALYSIS_1D:
        assert oracle.sq5_u32_py(idx, seed) == bits
        assert L.rdbo_sq5_u32(idx, seed) == bits
        assert int(oracle.sq5_u32_np(np.array([idx], dtype=np.uint32), seed)[0]) == bits
        assert np.float32(L.rdbo_sq5_f32(idx, seed)) == np.float32(f)
        assert np.float32(oracle.u32_to_f32_py(bits)) == np.float32(f)
    for n, m, seed, addr, bits, f in ANALYSIS_2D:
        assert oracle.mix2d_py(n, m) == addr
        assert L.rdbo_sq5_u32(addr, seed) == bits
        assert np.float32(L.rdbo_noise_at(n, m, seed)) == np.float32(f)
        assert oracle.noise_2d_np([n], [m], seed)[0, 0] == np.float32(f)


def test_golden_fixture(oracle):
    L = oracle.lib()
    with open(GOLD) as fh:
        gold = json.load(fh)
    assert len(gold["one_d"]) >= 40 and len(gold["two_d"]) >= 40
    for e in gold["one_d"]:
        f = np.float32(float.fromhex(e["f32_hex"]))
        assert L.rdbo_sq5_u32(e["idx"], e["seed"]) == e["bits"]
        assert oracle.sq5_u32_py(e["idx"], e["seed"]) == e["bits"]
        assert np.float32(L.rdbo_sq5_f32(e["idx"], e["seed"])) == f
        assert oracle.noise_1d_np(np.array([e["idx"]], dtype=np.uint32), e["seed"])[0] == f
    for e in gold["two_d"]:
        f = np.float32(float.fromhex(e["f32_hex"]))
        assert oracle.mix2d_py(e["n"], e["m"]) == e["addr"]
        assert np.float32(L.rdbo_noise_at(e["n"], e["m"], e["seed"])) == f
        assert oracle.noise_2d_np([e["n"]], [e["m"]], e["seed"])[0, 0] == f


def test_three_spellings_agree_on_a_million_indices(oracle):
    rng = np.random.default_rng(1234)
    N = 1_000_000
    for seed in (0, 1337, 2**31 - 1, 0xFFFFFFFF):
        # C (through the 1-D fill) vs NumPy on a contiguous range ...
        c = oracle.noise_1d(N, seed)
        n = oracle.noise_1d_np(np.arange(N, dtype=np.uint32), seed)
        assert np.array_equal(c.view(np.uint32), n.view(np.uint32))
    # ... and on random 32-bit indices including the wrap-around region, against big-int Python
    idx = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    idx[:4] = [0, 1, 0xFFFFFFFF, 0x80000000]
    bits_np = oracle.sq5_u32_np(idx, 1337)
    L = oracle.lib()
    for i in range(0, idx.size, 7):
        b = oracle.sq5_u32_py(int(idx[i]), 1337)
        assert b == int(bits_np[i]) == L.rdbo_sq5_u32(int(idx[i]), 1337)


def test_2d_fill_matches_numpy_and_wraps(oracle):
    # rows large enough that PRIME*n wraps 2**32 many times
    N, M, seed = 3000, 70, 47
    c = oracle.noise_2d(N, M, seed)
    n = oracle.noise_2d_np(np.arange(N), np.arange(M), seed)
    assert np.array_equal(c.view(np.uint32), n.view(np.uint32))
    big_rows = np.array([58_720_255, 2**31 - 1, 2**32 - 1, 21_000_000], dtype=np.uint64)
    t = oracle.noise_2d_np(big_rows, np.arange(5), seed)
    for r, row in enumerate(big_rows):
        for m in range(5):
            assert np.float32(oracle.noise_py(int(row), m, seed)) == t[r, m]


def test_float_edge_cases(oracle):
    # int32 min -> exactly -1; int32 max rounds up to 2**31 in fp32 -> exactly +1; 0 -> 0
    assert oracle.u32_to_f32_py(0x80000000) == -1.0
    assert oracle.u32_to_f32_py(0x7FFFFFFF) == 1.0
    assert oracle.u32_to_f32_py(0) == 0.0
    f = oracle.u32_to_f32_np(np.array([0x80000000, 0x7FFFFFFF, 0, 0x7FFFFF80, 0x7FFFFFBF, 0x7FFFFFC0],
                                      dtype=np.uint32))
    assert f[0] == -1.0 and f[1] == 1.0 and f[2] == 0.0
    # ties-to-even at the 24-bit boundary: 0x7FFFFFC0 is halfway between 0x7FFFFF80 and 2**31
    assert f[3] == np.float32(0x7FFFFF80) * np.float32(2.0**-31)
    assert f[4] == f[3] and f[5] == 1.0
    # the scale the reference writes, 1/0x7FFFFFFF, is 2**-31 once rounded to fp32
    assert np.float32(1.0 / 0x7FFFFFFF) == np.float32(2.0**-31)
    # whole range stays inside [-1, 1]
    x = oracle.noise_1d(200000, 5)
    assert x.min() >= -1.0 and x.max() <= 1.0
    assert abs(float(x.mean())) < 0.01 and abs(float(x.var()) - 1.0 / 3.0) < 0.01
