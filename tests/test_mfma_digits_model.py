"""CPU model of the activation digits of the matrix-core GEMV engine (build_pair in elutq_amd/csrc/hlq_gemv_mfma.hip):
an integer |xi| <= 2^18 is split as xi = 343 hi + lo and each part gives balanced base-7 digits in -3..3 by fp16
arithmetic -- q = fma(X, fp16(1/7), 1536) - 1536, digit = fma(q, -7, X).  Exhaustive over every integer the kernel can
meet: the digits are in range (fp4 e2m1 holds -3..3 exactly) and sum(d_t 7^t) is the integer itself, so the only loss
of the engine's operand is the rounding of x * scale to an integer.  The fused multiply-add rounds once: modelled as an
exact float64 product and sum followed by one rounding to fp16.
"""
import numpy as np

TERMS, SPLIT, XBITS = 7, 3, 18


def fma16(a, b, c):
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float16)


def digits_of_part(X, nd):
    c7, big, m7 = np.float16(1.0 / 7.0), np.float16(1536.0), np.float16(-7.0)
    out = []
    X = X.astype(np.float16)
    for _ in range(nd - 1):
        q = (fma16(X, np.full_like(X, c7), np.full_like(X, big)) - big).astype(np.float16)
        out.append(fma16(q, np.full_like(X, m7), X))
        X = q
    out.append(X)
    return out


def test_every_integer_of_the_fixed_point_range_has_exact_digits():
    xi = np.arange(-(1 << XBITS), (1 << XBITS) + 1, dtype=np.int64)
    xf = xi.astype(np.float32)
    hi = np.rint(xf * np.float32(1.0 / 343.0)).astype(np.float32)
    lo = (xf - np.float32(343.0) * hi).astype(np.float32)              # exact: |343 hi| < 2^19
    assert np.max(np.abs(lo)) <= 171 and np.max(np.abs(hi)) <= 765     # both below 2048: exact in fp16
    d = digits_of_part(lo, SPLIT) + digits_of_part(hi, TERMS - SPLIT)
    assert len(d) == TERMS
    total = np.zeros_like(xi)
    for t, dt in enumerate(d):
        di = dt.astype(np.int64)
        assert np.array_equal(di.astype(np.float16), dt)               # integers
        assert di.min() >= -3 and di.max() <= 3, t
        total += di * 7 ** t
    assert np.array_equal(total, xi)


def test_the_scale_puts_the_largest_activation_of_a_half_unit_below_the_range():
    """scale = 2^(126 + XBITS - eb) for amax in [2^(eb-127), 2^(eb-126)): amax * scale in [2^(XBITS-1), 2^XBITS)."""
    r = np.random.default_rng(0)
    amax = np.abs(np.concatenate([r.standard_normal(4096) * 10.0 ** r.integers(-6, 5, 4096),
                                  [65504.0, 2.0 ** -24, 6.1e-5, 1.0, 0.99999]])).astype(np.float16).astype(np.float32)
    amax = amax[amax > 0]
    eb = (amax.view(np.uint32) >> 23) & 0xFF
    scale = ((253 + XBITS - eb).astype(np.uint32) << 23).view(np.float32)
    inv = ((eb + 1 - XBITS).astype(np.uint32) << 23).view(np.float32)
    v = amax.astype(np.float64) * scale
    assert np.all(v >= 2.0 ** (XBITS - 1)) and np.all(v < 2.0 ** XBITS)
    assert np.array_equal(scale.astype(np.float64) * inv, np.ones(len(amax)))
