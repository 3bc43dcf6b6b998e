"""Pins the oracle's scalar arithmetic: bf16 rounding, scale constants, the canonical dot."""
import ctypes

import numpy as np
import torch

from oracle import hip12 as O
from oracle import literal


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 50,
                        np.array([0.0, -0.0, 1.0, 3.3635857, 0.29730177, 65504.0, 1e-30, -32000.0,
                                  1.00390625, 1.01171875], dtype=np.float32)])
    got = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    ref = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    L = O.lib()
    for val in x[:200]:
        assert L.hipo_round_bf16(ctypes.c_float(float(val))) == float(torch.tensor(val).to(torch.bfloat16))


def test_scale_constants():
    # bf16, HID=128: the two rounded constants multiply to 0.9973, not 1
    cq, ck = O.scale_constants(128, "bf16")
    assert cq == 3.359375 and ck == 0.296875
    cq, ck = O.scale_constants(64, "bf16")
    assert cq == float(torch.tensor(64.0 ** 0.25).to(torch.bfloat16))
    assert ck == float(torch.tensor(64.0 ** -0.25).to(torch.bfloat16))
    cq, ck = O.scale_constants(64, "f32")
    s = np.float32(8.0)
    ss = np.sqrt(s, dtype=np.float32)
    assert cq == float(np.float32(s / ss)) and ck == float(np.float32(np.float32(1.0) / ss))
    assert abs(cq * ck - 1.0) < 1e-6


def test_canonical_dot():
    rng = np.random.default_rng(1)
    L = O.lib()
    for hid in (16, 64, 128, 256):
        for _ in range(50):
            a = rng.standard_normal(hid).astype(np.float32)
            b = rng.standard_normal(hid).astype(np.float32)
            got = L.hipo_dot(a.ctypes.data, b.ctypes.data, hid)
            lit = float(literal.dot_canonical(a, b))
            assert got == lit  # same order -> same bits
            assert abs(got - float(np.dot(a.astype(np.float64), b.astype(np.float64)))) < 1e-4
    # small integers: every partial sum is exact, so any order gives the exact answer
    a = rng.integers(-8, 8, 128).astype(np.float32)
    b = rng.integers(-8, 8, 128).astype(np.float32)
    assert L.hipo_dot(a.ctypes.data, b.ctypes.data, 128) == float(np.dot(a.astype(np.int64), b.astype(np.int64)))
    # order sensitivity: a transposed-operand / wrong-segment bug changes this value
    a = np.zeros(128, np.float32); b = np.ones(128, np.float32)
    a[0] = 1e8; a[8] = 1.0; a[1] = -1e8
    assert L.hipo_dot(a.ctypes.data, b.ctypes.data, 128) == 1.0
