"""Pins of the oracle's block-sparse extra plane (use_sparse layers).

The reference has a consumer of this format (loader, rearrangement, kernel) but no producer,
no tests and no fixtures, so the restatement is pinned by the cases in which a sparse layer
must coincide with something already pinned: blocks on every (tile, group) pair are one more
dense plane -- bit for bit through the fp16 chain, because the operation order is then the
same; no blocks are the base layer; a single bit is a single scale.  The loader's permutation
is checked by brute force over its index expressions, and the NumPy and C restatements
(independent code) must agree bit for bit for every thread count.
"""
import numpy as np
import pytest

from elutq_amd.synth import make_layer, make_sparse_plane
from oracle import hlq_oracle as O


def full_cover(layer, plane_index):
    """The SparsePlane that lists plane `plane_index` of a dense layer block by block."""
    bits = O.unpack_planes(layer.w_quant)[plane_index]                  # [N, K]
    n, k, g = layer.n, layer.k, layer.group
    blk_bits, blk_scale, mask = [], [], []
    for t in range(n // 32):
        for gi in range(k // g):
            blk_bits.append(bits[32 * t:32 * t + 32, g * gi:g * gi + g])
            blk_scale.append(layer.w_scale[plane_index, 32 * t:32 * t + 32, gi])
            mask.append((32 * t, g * gi))
    return O.SparsePlane(np.stack(blk_bits), np.stack(blk_scale), np.array(mask, np.uint32), g)


@pytest.mark.parametrize("bits,group", [(2, 128), (3, 64)])
def test_blocks_everywhere_equal_one_more_dense_plane(bits, group):
    L = make_layer(256, 64, bits, group, seed=3, bias=True)
    sp = full_cover(L, bits - 1)
    base = (L.w_quant[:bits - 1], L.w_scale[:bits - 1], L.w_zero)
    x = L.x[0]
    assert np.array_equal(O.dequantize_sparse(*base, sp), O.dequantize(L.w_quant, L.w_scale, L.w_zero, group))
    for fused in (True, False):
        want = O.gemv_fp16_chain(x, L.w_quant, L.w_scale, L.w_zero, group, L.bias, fused)
        got = O.gemv_sparse_fp16_chain(x, *base, sp, L.bias, fused)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_no_blocks_is_the_base_layer():
    L = make_layer(256, 64, 2, 128, seed=4)
    sp = O.SparsePlane(np.zeros((0, 32, 128), np.uint8), np.zeros((0, 32), np.float16), np.zeros((0, 2), np.uint32), 128)
    want = O.gemv_fp16_chain(L.x[0], L.w_quant, L.w_scale, L.w_zero, 128)
    got = O.gemv_sparse_fp16_chain(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert np.array_equal(O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp),
                          O.dequantize(L.w_quant, L.w_scale, L.w_zero, 128))


def test_single_bit_single_scale():
    k, n, g = 256, 96, 64
    wq = np.zeros((1, n, k // 8), np.uint8)
    ws = np.zeros((1, n, k // g), np.float16)
    wz = np.zeros((n, k // g), np.float16)
    bits = np.zeros((1, 32, g), np.uint8)
    bits[0, 5, 9] = 1
    scale = np.zeros((1, 32), np.float16)
    scale[0, 5] = 0.375
    sp = O.SparsePlane(bits, scale, np.array([[64, 128]], np.uint32), g)
    w = O.dequantize_sparse(wq, ws, wz, sp)
    want = np.zeros((n, k))
    want[64 + 5, 128 + 9] = 0.375
    assert np.array_equal(w, want)
    x = np.zeros(k, np.float16)
    x[128 + 9] = 2.0
    y = O.gemv_sparse_fp16_chain(x, wq, ws, wz, sp)
    assert y[69] == np.float16(0.75) and np.count_nonzero(y) == 1


def test_dequantize_sparse_brute_force():
    L = make_layer(256, 64, 2, 64, seed=5)
    bits, scale, mask = make_sparse_plane(256, 64, 64, 0.5, seed=6)
    sp = O.SparsePlane(bits, scale, mask, 64)
    w = O.dequantize(L.w_quant, L.w_scale, L.w_zero, 64)
    for i in range(mask.shape[0]):
        for ch in range(32):
            for j in range(64):
                if bits[i, ch, j]:
                    w[int(mask[i, 0]) + ch, int(mask[i, 1]) + j] += float(scale[i, ch])
    assert np.array_equal(O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp), w)


def test_sparse_export_payloads_and_config():
    L = make_layer(256, 64, 2, 128, seed=7)
    bits, scale, mask = make_sparse_plane(256, 64, 128, 0.5, seed=8)
    sp = O.SparsePlane(bits, scale, mask, 128)
    wq, ws, mk = O.sparse_export_arrays(L.w_quant, L.w_scale, sp)
    nblk = mask.shape[0]
    cfg = O.sparse_weight_config(256, 64, 2, False, sp)
    # sizes the loader allocates and reads (parameters.cpp:36-63)
    assert len(wq) == cfg["weight_data_len"] == 256 * 64 * 2 // 8 + nblk * 32 * 128 // 8
    assert len(ws) == 2 * (2 * 256 * 64 // 128 + cfg["sparse_mask_len"] // 2 * 32)
    assert len(mk) == 4 * cfg["sparse_mask_len"] and cfg["sparse_mask_len"] == 2 * nblk
    assert cfg["use_sparse"] is True and cfg["base_bit"] == 2
    # block i, channel ch, byte j sits where the rearrangement reads it (kernal.cpp:582)
    tail = np.frombuffer(wq, np.uint8)[256 * 64 * 2 // 8:]
    for i in (0, nblk - 1):
        for ch in (0, 17, 31):
            for j in (0, 15):
                byte = tail[2 * i * 2 * 128 + ch * 128 // 8 + j]
                assert byte == np.packbits(bits[i, ch, 8 * j:8 * j + 8], bitorder="little")[0]


def test_rearrange_sparse_brute_force_and_bijective():
    L = make_layer(128, 64, 2, 64, seed=9)
    bits, scale, mask = make_sparse_plane(128, 64, 64, 0.6, seed=10)
    sp = O.SparsePlane(bits, scale, mask, 64)
    n, k, g, base = 64, 128, 64, 2
    # tag every byte with its own index so the permutation itself is visible
    tag = np.arange(base * n * k // 8 + mask.shape[0] * 32 * g // 8)
    wq_tag = (tag % 251).astype(np.uint8)
    dense = wq_tag[:base * n * k // 8].reshape(base, n, k // 8)
    blocks = wq_tag[base * n * k // 8:].reshape(-1, 32, g // 8)
    sp_tag = O.SparsePlane(O.unpack_planes(blocks), scale, mask, g)
    got_w, got_s, got_z = O.rearrange_sparse_reference(dense, L.w_scale, L.w_zero, sp_tag)
    want = []
    for b in range(base):
        for i in range(0, n, 32):
            for j in range(k // 8):
                for c in range(32):
                    want.append(dense[b, i + c, j])
    for i in range(mask.shape[0]):
        for j in range(g // 8):
            for c in range(32):
                want.append(blocks[i, c, j])
    assert np.array_equal(got_w, np.array(want, np.uint8))
    assert got_w.size == wq_tag.size and sorted(got_w.tolist()) == sorted(wq_tag.tolist())
    assert np.array_equal(got_s[-scale.size:], scale.reshape(-1))       # block scales stay in place
    assert got_z.size == L.w_zero.size


@pytest.mark.parametrize("group,threads", [(128, 1), (128, 2), (64, 4)])
def test_numpy_chain_equals_c_restatement(lutref, group, threads):
    k, n = 512, 128
    L = make_layer(k, n, 2, group, seed=11, bias=True)
    bits, scale, mask = make_sparse_plane(k, n, group, 0.4, seed=12)
    sp = O.SparsePlane(bits, scale, mask, group)
    wq, ws, mk = O.sparse_export_arrays(L.w_quant, L.w_scale, sp)
    ref = lutref.RefSparseWeight(wq, ws, L.w_zero, mk, k, n, 2, group, L.bias)
    # the C loader's output equals the NumPy one
    rw, rs, rz = O.rearrange_sparse_reference(L.w_quant, L.w_scale, L.w_zero, sp)
    assert np.array_equal(ref.weight, rw) and np.array_equal(ref.scale.view(np.uint16), rs.view(np.uint16))
    assert np.array_equal(ref.zero.view(np.uint16), rz.view(np.uint16))
    for fused in (True, False):
        want = O.gemv_sparse_fp16_chain(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp, L.bias, fused)
        got = ref.gemv(L.x[0], threads, fused)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_chain_exact_on_integer_inputs(lutref):
    """Integer activations and power-of-two scales: every fp16 operation is exact, so the chain
    must equal the float64 product bit for bit."""
    k, n, g = 256, 64, 128
    r = np.random.default_rng(13)
    planes = r.integers(0, 2, (2, n, k), dtype=np.uint8)
    wq = O.pack_planes(planes)
    ws = np.stack([np.full((n, k // g), 0.5), np.full((n, k // g), 1.0)]).astype(np.float16)
    wz = np.full((n, k // g), -0.5, np.float16)
    bits, _, mask = make_sparse_plane(k, n, g, 0.5, seed=14)
    scale = np.full((mask.shape[0], 32), 2.0, np.float16)
    sp = O.SparsePlane(bits, scale, mask, g)
    x = r.integers(-2, 3, k).astype(np.float16)
    want = O.gemv_sparse_f64(x, wq, ws, wz, sp)
    got = O.gemv_sparse_fp16_chain(x, wq, ws, wz, sp)
    assert np.array_equal(got.astype(np.float64), want)
    wqb, wsb, mk = O.sparse_export_arrays(wq, ws, sp)
    assert np.array_equal(lutref.RefSparseWeight(wqb, wsb, wz, mk, k, n, 2, g).gemv(x, 2).astype(np.float64), want)


def test_chain_close_to_float64():
    k, n, g = 512, 64, 128
    L = make_layer(k, n, 2, g, seed=15)
    bits, scale, mask = make_sparse_plane(k, n, g, 0.3, seed=16)
    sp = O.SparsePlane(bits, scale, mask, g)
    want = O.gemv_sparse_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp)
    got = O.gemv_sparse_fp16_chain(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp)
    rms = np.sqrt(np.mean(want ** 2))
    assert np.max(np.abs(got.astype(np.float64) - want)) < 2e-2 * rms
