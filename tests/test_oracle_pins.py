"""Pins of the CPU oracle (oracle/hlq_oracle.py, oracle/lut_gemv_ref.c).

The reference ships no tests, golden vectors or fixtures for this path, so each oracle
function is pinned by what the mathematics fixes: library routines it must reduce to,
closed forms, brute force on tiny inputs, and exactness on integer-valued inputs where
every fp16 operation is exact.  None of these retypes the oracle's own formula.
"""
import itertools

import numpy as np
import pytest

from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O


def rng(seed=0):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------ a1 packing
def test_pack_hand_vectors():
    bits = np.zeros((1, 1, 8), np.uint8)
    bits[0, 0, 0] = 1
    assert O.pack_planes(bits)[0, 0, 0] == 0x01          # k=0 is the least significant bit
    bits[:] = 0
    bits[0, 0, 7] = 1
    assert O.pack_planes(bits)[0, 0, 0] == 0x80
    bits[:] = 0
    bits[0, 0, [1, 4]] = 1
    assert O.pack_planes(bits)[0, 0, 0] == 0x12


def test_pack_equals_numpy_packbits_little():
    planes = rng(1).integers(0, 2, (2, 32, 64), dtype=np.uint8)
    want = np.packbits(planes, axis=-1, bitorder="little")
    got = O.pack_planes(planes)
    assert got.dtype == np.uint8 and got.shape == (2, 32, 8)
    assert np.array_equal(got, want)
    assert np.array_equal(O.unpack_planes(got), planes)


def test_pack_brute_force_triple_loop():
    planes = rng(2).integers(0, 2, (3, 5, 16), dtype=np.uint8)
    got = O.pack_planes(planes)
    for b, n, i in itertools.product(range(3), range(5), range(2)):
        v = 0
        for j in range(8):
            v |= int(planes[b, n, 8 * i + j]) << j
        assert got[b, n, i] == v


# ------------------------------------------------------------------ a2 export layout
def test_export_arrays_shapes_and_byte_counts():
    n, k, b, g = 64, 256, 3, 64
    r = rng(3)
    q = r.integers(0, 2, (n, k, b), dtype=np.uint8)
    s = r.uniform(0.01, 0.02, (n, k // g, b)).astype(np.float32)
    z = r.uniform(-0.02, -0.01, (n, k // g, 1)).astype(np.float32)
    wq, ws, wz = O.export_arrays(q, s, z)
    assert wq.shape == (b, n, k // 8) and ws.shape == (b, n, k // g) and wz.shape == (n, k // g)
    cfg = O.weight_config(k, n, b, False)
    assert cfg["weight_data_len"] == wq.nbytes == k * n * b // 8
    # element [b][n][g] of the scale file is scale[n][g][b] of the quantizer tensor
    assert ws[2, 5, 1] == np.float16(s[5, 1, 2]) and wz[7, 3] == np.float16(z[7, 3, 0])
    # plane b, row n, byte i, bit j is q[n, 8i+j, b]
    assert (wq[1, 9, 4] >> 3) & 1 == q[9, 35, 1]
    assert "groupsize" not in cfg and O.weight_config(k, n, b, True, 64)["groupsize"] == 64


@pytest.mark.parametrize("bits,group,bpw", [(2, 128, 2.375), (2, 64, 2.75), (3, 128, 3.5)])
def test_bits_per_weight_matches_readme(bits, group, bpw):
    # README.md:34,37,42 of the reference quotes 2.37 / 2.75 / 3.5 bits per weight
    L = make_layer(256, 64, bits=bits, group=group, seed=0)
    total_bits = 8 * (L.w_quant.nbytes + L.w_scale.nbytes + L.w_zero.nbytes)
    assert total_bits / (L.k * L.n) == pytest.approx(bpw)
    assert bpw == bits + 16 * (bits + 1) / group


# ------------------------------------------------------------------ a4 dequant / matmul
def test_dequantize_equals_einsum():
    L = make_layer(256, 96, bits=3, group=64, seed=4)
    planes = np.unpackbits(L.w_quant, axis=-1, bitorder="little").astype(np.float64)   # [B,N,K]
    s = L.w_scale.astype(np.float64)
    z = L.w_zero.astype(np.float64)
    want = np.einsum("bngj,bng->ngj", planes.reshape(3, 96, 4, 64), s) + z[:, :, None]
    got = O.dequantize(L.w_quant, L.w_scale, L.w_zero, 64)
    assert np.array_equal(got, want.reshape(96, 256))


def test_gemv_closed_forms():
    L = make_layer(256, 64, bits=2, group=128, seed=5)
    x = L.x[0].astype(np.float64)
    xs = x.reshape(2, 128).sum(1)
    z = L.w_zero.astype(np.float64)
    s = L.w_scale.astype(np.float64)
    zero_planes = np.zeros_like(L.w_quant)
    one_planes = np.full_like(L.w_quant, 0xFF)
    np.testing.assert_allclose(O.gemv_f64(L.x[0], zero_planes, L.w_scale, L.w_zero, 128), z @ xs, rtol=1e-12)
    np.testing.assert_allclose(O.gemv_f64(L.x[0], one_planes, L.w_scale, L.w_zero, 128),
                               (s.sum(0) + z) @ xs, rtol=1e-12)
    # unit-vector activation picks one column of W
    e = np.zeros(256, np.float16)
    e[130] = 1
    w = O.dequantize(L.w_quant, L.w_scale, L.w_zero, 128)
    assert np.array_equal(O.gemv_f64(e, L.w_quant, L.w_scale, L.w_zero, 128), w[:, 130])
    # a single set bit: y_n = s*x_k + zero fold
    single = np.zeros_like(L.w_quant)
    single[1, 7, 200 // 8] = 1 << (200 % 8)
    y = O.gemv_f64(L.x[0], single, L.w_scale, L.w_zero, 128)
    want = z @ xs
    want[7] += s[1, 7, 1] * x[200]
    np.testing.assert_allclose(y, want, rtol=1e-12)


def test_gemv_linearity_and_column_permutation():
    L = make_layer(256, 64, bits=2, group=64, seed=6)
    x1, x2 = L.x[0], make_layer(256, 64, seed=7).x[0]
    f = lambda x: O.gemv_f64(x, L.w_quant, L.w_scale, L.w_zero, 64)
    np.testing.assert_allclose(f(x1) + f(x2), O.dequantize(L.w_quant, L.w_scale, L.w_zero, 64)
                               @ (x1.astype(np.float64) + x2.astype(np.float64)), rtol=1e-10, atol=1e-12)
    perm = rng(8).permutation(64)
    yp = O.gemv_f64(x1, L.w_quant[:, perm], L.w_scale[:, perm], L.w_zero[perm], 64)
    assert np.array_equal(yp, f(x1)[perm])


# ------------------------------------------------------------------ a7 loader permutation
@pytest.mark.parametrize("threads", [1, 2, 4])
def test_rearrange_is_the_index_formula_and_bijective(threads, lutref):
    n, k, bits, g = 64 * threads, 128, 2, 64
    L = make_layer(k, n, bits=bits, group=g, seed=9)
    # tag every byte / half with its own flat index so the permutation is visible
    tag_q = (np.arange(L.w_quant.size) % 251).astype(np.uint8).reshape(L.w_quant.shape)
    tag_s = np.arange(L.w_scale.size, dtype=np.uint16).view(np.float16).reshape(L.w_scale.shape)
    tag_z = np.arange(L.w_zero.size, dtype=np.uint16).view(np.float16).reshape(L.w_zero.shape)
    wq, ws, wz = O.rearrange_reference(tag_q, tag_s, tag_z, g, threads)
    rw = lutref.RefWeight(tag_q, tag_s, tag_z, g, threads)
    assert np.array_equal(wq, rw.weight) and np.array_equal(ws.view(np.uint16), rw.scale.view(np.uint16))
    assert np.array_equal(wz.view(np.uint16), rw.zero.view(np.uint16))
    # brute-force the documented layout [thread][bit][tile][K/8][32]
    chunk = n // threads
    idx = 0
    for t in range(threads):
        for b in range(bits):
            for tile in range(chunk // 32):
                for kb in range(k // 8):
                    for r in range(32):
                        assert wq[idx] == tag_q[b, t * chunk + tile * 32 + r, kb]
                        idx += 1
    assert idx == wq.size
    # scales and zeros are bijections of their inputs
    assert sorted(ws.view(np.uint16).tolist()) == list(range(tag_s.size))
    assert sorted(wz.view(np.uint16).tolist()) == list(range(tag_z.size))
    # zeros: [tile][g][32]
    assert wz.view(np.uint16)[1 * (k // g) * 32 + 1 * 32 + 5] == tag_z.view(np.uint16)[32 + 5, 1]


# ------------------------------------------------------------------ a8 LUT
def test_lut_brute_force(lutref):
    x = make_layer(128, 64, seed=10).x[0][:64]
    lut_py = O.lut_float(x)
    lut_c = lutref.lut(x)
    assert np.array_equal(lut_py.view(np.uint16), lut_c.view(np.uint16))
    for c in range(16):
        for m in range(16):
            acc = np.float16(0)
            for i in range(4):
                if m & (1 << i):
                    acc = np.float16(acc + x[4 * c + i])     # numpy rounds every fp16 add
            assert lut_py[c, m] == acc
    assert np.all(lut_py[:, 0] == 0) and np.array_equal(lut_py[:, 1], x[0::4]) and np.array_equal(lut_py[:, 8], x[3::4])


# ------------------------------------------------------------------ a9-a12 fp16 chain
@pytest.mark.parametrize("bits,group", [(2, 128), (3, 128), (2, 64), (4, 128)])
def test_fp16_chain_python_equals_c(bits, group, lutref):
    L = make_layer(512, 128, bits=bits, group=group, seed=11, bias=True)
    for fused in (True, False):
        want = O.gemv_fp16_chain(L.x[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias, fused)
        for threads in (1, 2, 4):
            got = lutref.RefWeight(L.w_quant, L.w_scale, L.w_zero, group, threads, L.bias).gemv(L.x[0], fused)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_fp16_chain_exact_on_integer_inputs(lutref):
    """x in {-2..2}, scales powers of two, zeros small integers/4: every fp16 operation of
    the chain is exact, so it must equal the float64 result bit for bit."""
    r = rng(12)
    k, n, bits, g = 256, 64, 2, 128
    x = r.integers(-2, 3, k).astype(np.float16)
    planes = r.integers(0, 2, (bits, n, k), dtype=np.uint8)
    wq = O.pack_planes(planes)
    ws = np.stack([np.full((n, k // g), 0.25, np.float16), np.full((n, k // g), 0.5, np.float16)])
    wz = (r.integers(-3, 1, (n, k // g)) / 4).astype(np.float16)
    y64 = O.gemv_f64(x, wq, ws, wz, g)
    assert np.all(np.abs(y64) < 1024)
    for fused in (True, False):
        y = O.gemv_fp16_chain(x, wq, ws, wz, g, fused=fused)
        assert np.array_equal(y.astype(np.float64), y64)
        yc = lutref.RefWeight(wq, ws, wz, g, 2).gemv(x, fused)
        assert np.array_equal(yc.astype(np.float64), y64)
    assert np.array_equal(lutref.RefWeight(wq, ws, wz, g, 2).gemv_fast(x).astype(np.float64), y64)


def test_fp16_chain_close_to_f64_and_gemm_is_row_loop(lutref):
    L = make_layer(1024, 128, bits=2, group=128, m=3, seed=13)
    y64 = O.gemm_f64(L.x, L.w_quant, L.w_scale, L.w_zero, 128)
    rw = lutref.RefWeight(L.w_quant, L.w_scale, L.w_zero, 128, 4)
    ym = rw.gemm(L.x)
    for i in range(3):
        assert np.array_equal(ym[i].view(np.uint16), rw.gemv(L.x[i]).view(np.uint16))
    # the reference's all-fp16 chain sits within ~1e-2 of rms(y) of the exact result
    assert np.max(np.abs(ym.astype(np.float64) - y64)) / np.sqrt(np.mean(y64 ** 2)) < 2e-2
    fast = np.stack([rw.gemv_fast(r) for r in L.x])
    assert O.rel_err(fast, y64) < 5e-2
    # the NumPy row loop is the C one bit for bit (two implementations, 1 and 4 threads, both mac forms)
    for fused in (True, False):
        yr = O.gemm_rows(L.x, L.w_quant, L.w_scale, L.w_zero, 128, fused=fused)
        assert yr.shape == (3, 128) and yr.dtype == np.float16
        for threads in (1, 4):
            yc = lutref.RefWeight(L.w_quant, L.w_scale, L.w_zero, 128, threads).gemm(L.x, fused)
            assert np.array_equal(yr.view(np.uint16), yc.view(np.uint16))


def test_gemm_rows_exact_on_integer_inputs():
    """Rows of small integers against power-of-two scales: every fp16 operation of the row loop is
    exact, so it equals the float64 dequantize-then-matmul bit for bit, row by row, bias included."""
    r = rng(21)
    m, k, n, bits, g = 5, 256, 96, 3, 64
    x = r.integers(-2, 3, (m, k)).astype(np.float16)
    wq = O.pack_planes(r.integers(0, 2, (bits, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // g), 2.0 ** (b - 3), np.float16) for b in range(bits)])
    wz = (r.integers(-3, 1, (n, k // g)) / 4).astype(np.float16)
    bias = r.integers(-4, 5, n).astype(np.float16)
    y64 = O.gemm_f64(x, wq, ws, wz, g, bias)
    assert np.all(np.abs(y64) < 1024)
    assert np.array_equal(O.gemm_rows(x, wq, ws, wz, g, bias).astype(np.float64), y64)
    # a permutation of the rows permutes the result: rows do not see each other
    perm = r.permutation(m)
    assert np.array_equal(O.gemm_rows(x[perm], wq, ws, wz, g, bias), O.gemm_rows(x, wq, ws, wz, g, bias)[perm])


def test_rel_err_metric():
    ref = np.array([1.0, -2.0, 0.0, 4.0])
    assert O.rel_err(ref, ref) == 0
    y = ref + np.array([0.01, 0, 0, 0])
    assert O.rel_err(y, ref) == pytest.approx(0.01)
    rms = np.sqrt(np.mean(ref ** 2))
    y = ref + np.array([0, 0, 0.001, 0])
    assert O.rel_err(y, ref) == pytest.approx(0.001 / (0.05 * rms))
