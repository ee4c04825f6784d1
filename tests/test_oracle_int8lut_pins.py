"""Pins of the oracle's restatement of the reference's int8-LUT variant (oracle/hlq_oracle.py: lut_int8,
gemv_int8lut_f64, gemv_int8lut_chain_uniform).

The reference has no caller, test or fixture for that variant, so the functions are pinned by what the
arithmetic fixes: a scalar re-derivation with Python floats and the struct module's fp16 rounding, invariances
(power-of-two scaling, negation), the cases where int8 tables lose nothing (then the exact oracle must come out),
and closed forms.  None of these retypes the oracle's formulas.
"""
import struct

import numpy as np
import pytest

from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O


def f16(v: float) -> float:
    """Round a Python float to fp16 (IEEE round-to-nearest-even) with the struct module."""
    return struct.unpack("<e", struct.pack("<e", v))[0]


def rne(v: float) -> int:
    return int(round(v))            # Python rounds halves to even


def test_lut_int8_against_scalar_python():
    x = (np.random.default_rng(1).standard_normal(64) * 2).astype(np.float16)
    q, sc = O.lut_int8(x, 32)
    assert q.shape == (16, 16) and q.dtype == np.int8 and sc.shape == (2,) and sc.dtype == np.float16
    for g in range(2):
        entries = []
        for c in range(8):
            a = [float(v) for v in x[32 * g + 4 * c:32 * g + 4 * c + 4]]
            row = []
            for m in range(16):
                t = 0.0
                for i in range(4):
                    if m >> i & 1:
                        t = f16(t + a[i])              # the sum of two fp16 values is exact in a double
                row.append(t)
            entries.append(row)
        top = max(abs(t) for row in entries for t in row)
        s = f16(float(np.float32(top) / np.float32(127.0)))
        assert float(sc[g]) == s
        for c in range(8):
            for m in range(16):
                want = max(-128, min(127, rne(f16(float(np.float32(entries[c][m]) / np.float32(s))))))
                assert int(q[8 * g + c, m]) == want, (g, c, m)


def test_lut_int8_properties():
    r = np.random.default_rng(2)
    x = r.standard_normal(512).astype(np.float16)
    x[128:256] = 0                                     # a group of zeros
    x[256:384] = 0
    x[300] = np.float16(-3.5)                          # a group with a single non-zero activation
    q, sc = O.lut_int8(x, 128)
    assert np.all(q[:, 0] == 0)                        # the empty subset
    per_group = np.abs(q.astype(np.int32)).reshape(4, -1).max(1)
    assert per_group.tolist() == [127, 0, 127, 127] and float(sc[1]) == 0.0
    assert set(np.unique(q[64:96])) == {-127, 0}       # one activation: every entry is 0 or the extreme
    # what the tables stand for is within half a step (plus the quotient's fp16 rounding) of the fp16 tables
    lut = O.lut_float(x).astype(np.float64)
    step = np.repeat(sc.astype(np.float64), 32)[:, None]
    assert np.all(np.abs(q * step - lut) <= 0.5 * step + 2.0 ** -9 * np.abs(lut) + 1e-12)
    # scaling by a power of two moves the scales and leaves the entries; negation flips them
    q2, sc2 = O.lut_int8((x.astype(np.float32) * 4).astype(np.float16), 128)
    assert np.array_equal(q2, q) and np.array_equal(sc2.astype(np.float32), sc.astype(np.float32) * 4)
    qn, scn = O.lut_int8(-x, 128)
    assert np.array_equal(qn, -q) and np.array_equal(scn, sc)


def lossless_case(seed, k=256, n=64, bits=2, group=128):
    """Integer activations whose largest subset sum per group is exactly 127: scale 1, entries = sums."""
    r = np.random.default_rng(seed)
    x = r.integers(-3, 4, k).astype(np.float16)
    for g in range(k // group):
        x[g * group:g * group + 4] = [100, 27, 0, 0]   # subset sums up to 127, every other chunk at most 12
    wq = O.pack_planes(r.integers(0, 2, (bits, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // group), 0.25 * 2 ** b) for b in range(bits)]).astype(np.float16)
    wz = np.full((n, k // group), -0.5, np.float16)
    return x, wq, ws, wz


def test_int8_tables_that_lose_nothing_give_the_exact_oracle():
    x, wq, ws, wz = lossless_case(3)
    q, sc = O.lut_int8(x, 128)
    assert np.all(sc == np.float16(1.0)) and np.array_equal(q.astype(np.float64), O.lut_float(x).astype(np.float64))
    want = O.gemv_f64(x, wq, ws, wz, 128)
    assert np.array_equal(O.gemv_int8lut_f64(x, wq, ws, wz, 128), want)
    # the reference's op order on the same weights read as its uniform format (zero point 0): exact as well,
    # every intermediate being a small multiple of 1/4
    z0 = np.zeros_like(wz)
    chain = O.gemv_int8lut_chain_uniform(x, wq, ws[0], 128)
    assert np.array_equal(chain.astype(np.float64), O.gemv_f64(x, wq, ws, z0, 128))


def test_gemv_int8lut_closed_forms():
    L = make_layer(256, 64, bits=2, group=64, seed=5)
    x = L.x[0]
    q, sc = O.lut_int8(x, 64)
    zeros = np.zeros_like(L.w_quant)
    xs = x.astype(np.float64).reshape(-1, 64).sum(-1)
    # no bit set: the zero term alone, which does not go through the tables
    assert np.allclose(O.gemv_int8lut_f64(x, zeros, L.w_scale, L.w_zero, 64), (L.w_zero.astype(np.float64) * xs).sum(-1), rtol=0, atol=1e-12)
    # every bit set: entry 15 of every chunk
    ones = np.full_like(L.w_quant, 0xFF)
    full = (q[:, 15].astype(np.float64).reshape(-1, 16).sum(-1) * sc.astype(np.float64))
    want = (L.w_zero.astype(np.float64) * xs).sum(-1) + (L.w_scale.astype(np.float64) * full[None, None, :]).sum((0, 2))
    assert np.allclose(O.gemv_int8lut_f64(x, ones, L.w_scale, L.w_zero, 64), want, rtol=0, atol=1e-9)
    # a single set bit at (plane 1, column 7, k = 70): the entry of that one activation times its scales
    one = np.zeros_like(L.w_quant)
    one[1, 7, 70 // 8] = 1 << (70 % 8)
    y = O.gemv_int8lut_f64(x, one, L.w_scale, np.zeros_like(L.w_zero), 64)
    assert np.count_nonzero(y) <= 1
    assert y[7] == float(L.w_scale[1, 7, 1]) * float(sc[1]) * int(q[70 // 4, 1 << (70 % 4)])


@pytest.mark.parametrize("bits,group", [(2, 128), (3, 64)])
def test_int8_tables_cost_accuracy_but_stay_near(bits, group):
    """Seven-bit tables: each looked-up entry is off by at most half a step of its group, so the result is off by
    at most sum_b |s_b| * step / 2 per chunk -- far inside that in practice."""
    L = make_layer(1024, 96, bits=bits, group=group, seed=7)
    exact = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group)
    y = O.gemv_int8lut_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group)
    _, sc = O.lut_int8(L.x[0], group)
    bound = (np.abs(L.w_scale.astype(np.float64)) * (sc.astype(np.float64) * (0.5 + 2.0 ** -4) * (group // 4))[None, None, :]).sum((0, 2))
    assert np.all(np.abs(y - exact) <= bound)
    assert np.sqrt(np.mean((y - exact) ** 2)) <= 0.1 * np.sqrt(np.mean(exact ** 2))
    assert not np.array_equal(y, exact)


def test_chain_uniform_close_to_exact_evaluation():
    L = make_layer(512, 64, bits=3, group=128, seed=9)
    ws = np.stack([L.w_scale[0].astype(np.float32) * 2 ** b for b in range(3)]).astype(np.float16)
    z0 = np.zeros_like(L.w_zero)
    ref = O.gemv_int8lut_f64(L.x[0], L.w_quant, ws, z0, 128)
    chain = O.gemv_int8lut_chain_uniform(L.x[0], L.w_quant, L.w_scale[0], 128)
    assert chain.dtype == np.float16
    assert np.max(np.abs(chain.astype(np.float64) - ref)) <= 2e-2 * np.sqrt(np.mean(ref ** 2))
