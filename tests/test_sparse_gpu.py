"""GPU parity of layers with a block-sparse extra plane (use_sparse exports), through the C ABI.

Same bars as the dense path: rel_err <= 1e-2 against the float64 oracle
(max_i |y_i - ref_i| / max(|ref_i|, 0.05 rms(ref))), max|y - y_ref| <= 2e-2 rms against the
restatement of the reference's all-fp16 chain, bit-exact where the arithmetic is exact.
"""
import os

import numpy as np
import pytest
import torch

from elutq_amd import _lib
from elutq_amd.export_io import SparseBlocks, write_export_dir
from elutq_amd.hlq_linear import GemvGroup, HLQLinear
from elutq_amd.repack import repack_tree
from elutq_amd.synth import make_layer, make_sparse_plane, pack_bits_lsb_first
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(params=["inline", "own_launch"], autouse=True)
def plane_launch(request, monkeypatch):
    """Every test runs twice: with the plane's blocks looked up inside the dense batch-1 launch (where the block list
    fits the inline form and the layer has at most three dense planes), and with the plane as a launch of its own."""
    monkeypatch.setattr(HLQLinear, "use_sparse_inline", request.param == "inline")
    return request.param


def build(k, n, bits, group, density, seed, dev, m=1, bias=True, mode="blocks"):
    """mode "blocks": the plane in its file form (the block kernels); "dense": written out as one more plane."""
    L = make_layer(k, n, bits, group, m=m, seed=seed, bias=bias)
    b, s, mk = make_sparse_plane(k, n, group, density, seed=seed + 100)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, L.bias, dev,
                                       SparseBlocks(pack_bits_lsb_first(b), s, mk), sparse_mode=mode)
    assert (mod.sparse_count > 0) == (mode == "blocks" and mk.shape[0] > 0)
    return L, O.SparsePlane(b, s, mk, group), mod


def run(mod, x, dev):
    y = mod(torch.from_numpy(np.ascontiguousarray(x)).to(dev))
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("k,n,bits,group,density", [
    (256, 64, 2, 128, 0.5), (512, 128, 2, 128, 0.3), (1024, 256, 3, 64, 0.2), (1024, 192, 1, 64, 1.0),
    (2048, 512, 2, 128, 0.05), (384, 96, 4, 128, 0.5), (704, 128, 2, 64, 0.3),
    (4096, 64, 2, 64, 1.0), (8192, 32, 2, 128, 0.9),          # 64 / ~58 blocks on a tile: more than one round of the plane kernel's waves
])
def test_gemv_matches_oracle(cuda, lutref, k, n, bits, group, density):
    L, sp, mod = build(k, n, bits, group, density, k + n, cuda)
    print(f"sparse gemv K={k} N={n} w{bits}g{group} blocks={mod.sparse_count}", flush=True)
    y = run(mod, L.x, cuda)[0]
    ref = O.gemv_sparse_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp, L.bias)
    assert y.shape == (n,) and y.dtype == np.float16
    assert O.rel_err(y, ref) <= TOL
    # the plane's fp32 term joins the dense fp32 sum before the one rounding to fp16
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
    wq, ws, mk = O.sparse_export_arrays(L.w_quant, L.w_scale, sp)
    chain = lutref.RefSparseWeight(wq, ws, L.w_zero, mk, k, n, bits, group, L.bias).gemv(L.x[0], 2 if n % 64 == 0 else 1)
    assert np.max(np.abs(y.astype(np.float64) - chain.astype(np.float64))) <= 2e-2 * np.sqrt(np.mean(ref ** 2))


@pytest.mark.parametrize("m", [2, 5, 33, 64, 70])
def test_gemm_matches_oracle_and_rows_equal_gemv(cuda, m):
    k, n, group = 512, 192, 128
    L, sp, mod = build(k, n, 2, group, 0.4, 7 + m, cuda, m=m)
    print(f"sparse gemm M={m} blocks={mod.sparse_count}", flush=True)
    y = run(mod, L.x, cuda)
    w = O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp)
    ref = L.x.astype(np.float64) @ w.T + L.bias.astype(np.float64)
    assert y.shape == (m, n)
    assert O.rel_err(y, ref) <= TOL
    # the reference defines m > 1 as one GEMV per row (arm_gemm.cpp:380-385)
    y0 = run(mod, L.x[m - 1:m], cuda)[0]
    assert np.max(np.abs(y[m - 1].astype(np.float64) - y0.astype(np.float64))) <= 2.0 ** -9 * max(1.0, np.max(np.abs(ref)))


@pytest.mark.parametrize("group,m", [(128, 1), (64, 1), (128, 9)])
def test_bit_exact_on_integer_inputs(cuda, group, m):
    """Integer activations, power-of-two scales: every product and sum is exact in fp32 and the result
    is representable in fp16, so the GPU must return the float64 result itself."""
    k, n = 512, 128
    r = np.random.default_rng(group + m)
    wq = O.pack_planes(r.integers(0, 2, (2, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // group), 0.5), np.full((n, k // group), 1.0)]).astype(np.float16)
    wz = np.full((n, k // group), -0.5, np.float16)
    b, _, mk = make_sparse_plane(k, n, group, 0.5, seed=group)
    s = np.full((mk.shape[0], 32), 2.0, np.float16)
    sp = O.SparsePlane(b, s, mk, group)
    mod = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda, SparseBlocks(sp.packed, s, mk), sparse_mode="blocks")
    auto = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda, SparseBlocks(sp.packed, s, mk))
    assert mod.sparse_count > 0 and auto.sparse_count == 0 and auto.bits == 3
    x = r.integers(-2, 3, (m, k)).astype(np.float16)
    y = run(mod, x, cuda)
    want = x.astype(np.float64) @ O.dequantize_sparse(wq, ws, wz, sp).T
    assert np.array_equal(y.astype(np.float64), want)
    assert np.array_equal(run(auto, x, cuda).astype(np.float64), want)       # the dense form: the same bits


def test_blocks_everywhere_equal_one_more_dense_plane(cuda):
    """A sparse plane that lists every (tile, group) pair is a dense plane: both layers dequantize to
    the same W and, on inputs where the arithmetic is exact, return the same bits."""
    k, n, group = 512, 128, 128
    L = make_layer(k, n, 3, group, seed=31)
    bits = O.unpack_planes(L.w_quant)[2]
    blk, sc, mk = [], [], []
    for t in range(n // 32):
        for g in range(k // group):
            blk.append(bits[32 * t:32 * t + 32, group * g:group * g + group])
            sc.append(L.w_scale[2, 32 * t:32 * t + 32, g])
            mk.append((32 * t, group * g))
    sp = SparseBlocks(pack_bits_lsb_first(np.stack(blk)), np.stack(sc), np.array(mk, np.uint32))
    dense = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, cuda)
    sparse = HLQLinear.from_export_arrays(L.w_quant[:2], L.w_scale[:2], L.w_zero, group, None, cuda, sp, sparse_mode="blocks")
    again = HLQLinear.from_export_arrays(L.w_quant[:2], L.w_scale[:2], L.w_zero, group, None, cuda, sp)
    # written out densely, the full cover IS the three-plane layer: the same buffers
    assert again.bits == 3 and torch.equal(again.planes, dense.planes) and torch.equal(again.scales, dense.scales)
    wd, wsp = dense.dequantize().float().cpu().numpy(), sparse.dequantize().float().cpu().numpy()
    ref = O.dequantize(L.w_quant, L.w_scale, L.w_zero, group)
    assert np.max(np.abs(wd - ref)) <= 2.0 ** -11 * np.max(np.abs(ref))
    assert np.max(np.abs(wsp - ref)) <= 2.0 ** -9 * np.max(np.abs(ref))       # two roundings instead of one
    yd, ys = run(dense, L.x, cuda)[0], run(sparse, L.x, cuda)[0]
    want = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group)
    assert O.rel_err(yd, want) <= TOL and O.rel_err(ys, want) <= TOL


def test_unaligned_and_overlapping_blocks(cuda):
    """k starts need only be multiples of 4, and blocks may overlap or repeat: each adds its own term."""
    k, n, group = 384, 64, 64
    L = make_layer(k, n, 2, group, seed=41)
    r = np.random.default_rng(42)
    mk = np.array([[0, 4], [0, 36], [0, 36], [32, 316], [32, 0]], np.uint32)
    b = r.integers(0, 2, (5, 32, group), dtype=np.uint8)
    s = r.uniform(0.02, 0.08, (5, 32)).astype(np.float16)
    sp = O.SparsePlane(b, s, mk, group)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, cuda, SparseBlocks(sp.packed, s, mk))
    assert mod.sparse_count == 5          # off the group grid and repeated: stays in block form whatever the mode
    with pytest.raises(ValueError):
        HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, cuda, SparseBlocks(sp.packed, s, mk),
                                     sparse_mode="dense")
    y = run(mod, L.x, cuda)[0]
    assert O.rel_err(y, O.gemv_sparse_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp)) <= TOL
    w = mod.dequantize().float().cpu().numpy()
    ref = O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp)
    assert np.max(np.abs(w - ref)) <= 2.0 ** -9 * np.max(np.abs(ref))


def test_ragged_n(cuda):
    """N = 100: the block on channels 96..127 only contributes to channels 96..99."""
    k, n, npad, group = 256, 100, 128, 128
    L = make_layer(k, npad, 2, group, seed=51, bias=True)
    b, s, mk = make_sparse_plane(k, npad, group, 1.0, seed=52)
    sp = O.SparsePlane(b, s, mk, group)
    sb = SparseBlocks(sp.packed, s, mk)
    mod = HLQLinear.from_export_arrays(L.w_quant[:, :n], L.w_scale[:, :n], L.w_zero[:n], group, L.bias[:n], cuda, sb,
                                       sparse_mode="blocks")
    dense = HLQLinear.from_export_arrays(L.w_quant[:, :n], L.w_scale[:, :n], L.w_zero[:n], group, L.bias[:n], cuda, sb)
    x = np.concatenate([L.x, -L.x, 0.5 * L.x])
    assert dense.sparse_count == 0 and O.rel_err(run(dense, x, cuda), (x.astype(np.float64) @ O.dequantize_sparse(
        L.w_quant, L.w_scale, L.w_zero, sp).T + L.bias.astype(np.float64))[:, :n]) <= TOL
    y = run(mod, x, cuda)
    ref = (x.astype(np.float64) @ O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp).T + L.bias.astype(np.float64))[:, :n]
    assert y.shape == (3, n) and O.rel_err(y, ref) <= TOL
    assert O.rel_err(run(mod, L.x, cuda)[0], ref[0]) <= TOL


def test_export_dir_and_repacked_dir_load_the_same_layer(cuda, tmp_path):
    k, n, group = 512, 128, 128
    L, sp, mod = build(k, n, 2, group, 0.3, 61, cuda)
    src, dst = str(tmp_path / "src"), str(tmp_path / "dst")
    d = os.path.join(src, "0", "mlp.gate_proj")
    write_export_dir(d, L.w_quant, L.w_scale, L.w_zero, L.bias, sparse=SparseBlocks(sp.packed, sp.scale, sp.mask))
    assert repack_tree(src, dst, sparse_mode="blocks") == 1
    y = run(mod, L.x, cuda)
    for path in (d, os.path.join(dst, "0", "mlp.gate_proj")):
        other = HLQLinear.from_export_dir(path, cuda, sparse_mode="blocks")
        assert other.sparse_count == mod.sparse_count and "sparse_blocks" in repr(other)
        assert np.array_equal(run(other, L.x, cuda).view(np.uint16), y.view(np.uint16))
    # the default of loader and CLI: one more dense plane, from either tree form, the same bits
    dst2 = str(tmp_path / "dst_dense")
    assert repack_tree(src, dst2) == 1
    a, b = HLQLinear.from_export_dir(d, cuda), HLQLinear.from_export_dir(os.path.join(dst2, "0", "mlp.gate_proj"), cuda)
    assert a.sparse_count == 0 and b.sparse_count == 0 and a.bits == b.bits == 3
    ya = run(a, L.x, cuda)
    assert np.array_equal(ya.view(np.uint16), run(b, L.x, cuda).view(np.uint16))
    assert O.rel_err(ya[0], O.gemv_sparse_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp, L.bias)) <= TOL


def test_full_size_layer(cuda):
    """q_proj of LLaMA-3-8B (4096 x 4096, w2g128) with a tenth of its blocks present."""
    k = n = 4096
    L, sp, mod = build(k, n, 2, 128, 0.1, 71, cuda, bias=False)
    print(f"sparse gemv 4096x4096 blocks={mod.sparse_count}", flush=True)
    y = run(mod, L.x, cuda)[0]
    assert O.rel_err(y, O.gemv_sparse_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp)) <= TOL
    y2 = run(mod, L.x, cuda)[0]
    assert np.array_equal(y.view(np.uint16), y2.view(np.uint16))          # run-to-run determinism
    ym = run(mod, -L.x, cuda)[0]
    assert np.array_equal((-ym).view(np.uint16), y.view(np.uint16))       # y(-x) = -y(x) exactly


@pytest.mark.parametrize("k,n,bits,group,density", [(512, 128, 2, 128, 0.3), (1024, 256, 3, 64, 0.2), (4096, 4096, 2, 128, 0.1),
                                                     (832, 128, 2, 64, 0.3)])
def test_dense_form_matches_oracle(cuda, k, n, bits, group, density):
    """The default way to hold the plane on this GPU: one more dense plane, every dense kernel as it is."""
    L, sp, mod = build(k, n, bits, group, density, k + n + 1, cuda, m=3, mode="dense")
    assert mod.bits == bits + 1
    y = run(mod, L.x, cuda)
    ref = L.x.astype(np.float64) @ O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp).T + L.bias.astype(np.float64)
    assert O.rel_err(y, ref) <= TOL
    assert O.rel_err(run(mod, L.x[:1], cuda)[0], ref[0]) <= TOL
    w = mod.dequantize().float().cpu().numpy()
    wref = O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, sp)
    assert np.max(np.abs(w - wref)) <= 2.0 ** -11 * np.max(np.abs(wref))


def _fused_case(k, n, bits, group, density, seed, dev):
    L, sp, mod = build(k, n, bits, group, density, seed, dev)
    g = torch.Generator(device=dev).manual_seed(seed)
    res = torch.randn(1, n, generator=g, device=dev).half()
    out = torch.full((1, n), float("nan"), dtype=torch.float16, device=dev)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=dev)
    return L, sp, mod, g, res, out, ws


FUSED_SHAPES = [(4096, 64, 2, 64, 1.0), (1024, 256, 2, 128, 0.3), (512, 96, 3, 64, 0.5), (4096, 1024, 2, 128, 0.1), (1088, 160, 2, 64, 0.4),
                (4096, 4096, 2, 128, 0.05)]


@pytest.mark.parametrize("k,n,bits,group,density", FUSED_SHAPES)
@pytest.mark.parametrize("ksplit,waves", [(0, 0), (1, 4), (2, 16), (_lib.GEMV_NARROW16, 0), (_lib.GEMV_NARROW32, 0),
                                          (_lib.GEMV_WIDE, 0)])
def test_fused_rmsnorm_prologue_and_residual(cuda, plane_launch, k, n, bits, group, density, ksplit, waves):
    """The layer inside a decode step: RMSNorm in front (formed by both launches, the plane's and the dense one's),
    bias, the plane's fp32 term and the residual behind, one rounding."""
    L, sp, mod, g, res, out, ws = _fused_case(k, n, bits, group, density, k + n + 3, cuda)
    print(f"sparse fused gemv K={k} N={n} w{bits}g{group} ksplit={ksplit} waves={waves} blocks={mod.sparse_count}", flush=True)
    mod.ksplit, mod.waves = ksplit, waves
    x = (torch.randn(1, k, generator=g, device=cuda) * 3).half()
    w = (1 + 0.1 * torch.randn(k, generator=g, device=cuda)).half()
    eps = 1e-5
    mod.gemv_fused(x, out, ws, prologue=1, norm_weight=w, eps=eps, residual=res)
    xf = x.float()
    h = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).half()
    ref = (O.gemv_sparse_f64(h.cpu().numpy()[0], L.w_quant, L.w_scale, L.w_zero, sp, L.bias)
           + res.cpu().numpy()[0].astype(np.float64))
    y = out.cpu().numpy()[0]
    assert O.rel_err(y, ref) <= TOL
    # against the unfused calls on the normalised input (1 / rms is summed in another order there: h may differ
    # in the last fp16 bit of a few elements)
    unfused = mod(h).float() + res.float()
    assert float((out.float() - unfused).abs().max()) <= 2e-2 * float(unfused.abs().max())
    # no prologue, no residual: the same bits as the plain entry point (which launches the library's own shape)
    mod.gemv_fused(h, out, ws)
    if (ksplit, waves) == (0, 0):
        assert torch.equal(out, mod(h))
    else:
        assert float((out.float() - mod(h).float()).abs().max()) <= 2.0 ** -9 * float(unfused.abs().max())
    assert int(ws[:65536].count_nonzero()) == 0        # the head of the workspace is left zero-filled


@pytest.mark.parametrize("k,n,bits,group,density", [(1024, 256, 2, 128, 0.3), (1536, 192, 4, 64, 0.2), (960, 96, 2, 64, 0.5),
                                                     (14336, 4096, 2, 128, 0.02)])
@pytest.mark.parametrize("ksplit", [0, _lib.GEMV_NARROW32, _lib.GEMV_WIDE])
def test_fused_silu_mul_prologue(cuda, plane_launch, k, n, bits, group, density, ksplit):
    import torch.nn.functional as F
    if ksplit == _lib.GEMV_NARROW32 and k > 8192:
        pytest.skip("the narrow-tile kernel holds the tables of at most 8192 activations")
    L, sp, mod, g, res, out, ws = _fused_case(k, n, bits, group, density, k + n + 5, cuda)
    print(f"sparse fused silu gemv K={k} N={n} w{bits}g{group} ksplit={ksplit} blocks={mod.sparse_count}", flush=True)
    mod.ksplit = ksplit
    gu = torch.randn(1, 2 * k, generator=g, device=cuda).half()
    mod.gemv_fused(gu, out, ws, prologue=2, residual=res)
    act = (F.silu(gu[:, :k].float()) * gu[:, k:].float()).half()
    ref = (O.gemv_sparse_f64(act.cpu().numpy()[0], L.w_quant, L.w_scale, L.w_zero, sp, L.bias)
           + res.cpu().numpy()[0].astype(np.float64))
    assert O.rel_err(out.cpu().numpy()[0], ref) <= TOL


def test_fused_wide_layer_runs_of_column_blocks(cuda):
    """gate|up of LLaMA-3-8B with a sparse plane: more column blocks than compute units, so the dense launch
    walks runs of them; the plane's term and the RMSNorm go through the same launch pair."""
    k, n = 4096, 28672
    L, sp, mod, g, res, out, ws = _fused_case(k, n, 2, 128, 0.05, 91, cuda)
    x = (torch.randn(1, k, generator=g, device=cuda) * 2).half()
    w = (1 + 0.1 * torch.randn(k, generator=g, device=cuda)).half()
    mod.gemv_fused(x, out, ws, prologue=1, norm_weight=w, eps=1e-5)
    xf = x.float()
    h = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()).half()
    # the oracle on 128 sampled channel tiles (4096 columns), the plane's blocks on those tiles renumbered
    tiles = np.sort(np.random.default_rng(n).choice(n // 32, 128, replace=False))
    tiles[0], tiles[-1] = 0, n // 32 - 1
    idx = (tiles[:, None] * 32 + np.arange(32)[None, :]).reshape(-1)
    pos = {int(t): i for i, t in enumerate(tiles)}
    keep = [i for i, c in enumerate(sp.mask[:, 0]) if int(c) // 32 in pos]
    sub_mask = np.array([[pos[int(sp.mask[i, 0]) // 32] * 32, sp.mask[i, 1]] for i in keep], np.uint32)
    sub = O.SparsePlane(sp.bits[keep], sp.scale[keep], sub_mask, 128)
    assert len(keep) > 100
    ref = O.gemv_sparse_f64(h.cpu().numpy()[0], L.w_quant[:, idx], L.w_scale[:, idx], L.w_zero[idx], sub, L.bias[idx])
    y = out.cpu().numpy()[0]
    assert O.rel_err(y[idx], ref) <= TOL
    # without the plane the result differs: the blocks do take part
    dense = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, 128, L.bias, cuda)
    yd = torch.empty_like(out)
    dense.gemv_fused(x, yd, ws, prologue=1, norm_weight=w, eps=1e-5)
    assert not torch.equal(yd, out)


def test_fused_integer_inputs_bit_exact(cuda):
    """SiLU(gate) * up with gate = 0 is 0, and a unit norm weight on inputs whose mean square is 1 - eps leaves
    integers: exact arithmetic in both launches, so the result is the float64 one."""
    k, n, group = 512, 128, 128
    r = np.random.default_rng(5)
    wq = O.pack_planes(r.integers(0, 2, (2, n, k), dtype=np.uint8))
    ws_ = np.stack([np.full((n, k // group), 0.5), np.full((n, k // group), 1.0)]).astype(np.float16)
    wz = np.full((n, k // group), -0.5, np.float16)
    b, _, mk = make_sparse_plane(k, n, group, 0.5, seed=6)
    s = np.full((mk.shape[0], 32), 2.0, np.float16)
    sp = O.SparsePlane(b, s, mk, group)
    mod = HLQLinear.from_export_arrays(wq, ws_, wz, group, None, cuda, SparseBlocks(sp.packed, s, mk), sparse_mode="blocks")
    x = r.choice(np.array([-1.0, 1.0], np.float16), (1, k))          # mean square exactly 1
    xd = torch.from_numpy(x).to(cuda)
    out = torch.empty(1, n, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    one = torch.ones(k, dtype=torch.float16, device=cuda)
    mod.gemv_fused(xd, out, ws, prologue=1, norm_weight=one, eps=0.0)
    want = x.astype(np.float64) @ O.dequantize_sparse(wq, ws_, wz, sp).T
    assert np.array_equal(out.cpu().numpy().astype(np.float64), want)


def test_fused_refuses_slices_and_group_refuses_sparse(cuda, plane_launch):
    if plane_launch == "inline":
        pytest.skip("a plane looked up inside the dense launch takes part in handed-over slices: test_inline_*")
    L, sp, mod = build(256, 64, 2, 128, 0.5, 81, cuda)
    x = torch.from_numpy(L.x).to(cuda)
    out = torch.empty(1, 64, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    sl = torch.zeros(4, 256, dtype=torch.float32, device=cuda)
    with pytest.raises(ValueError):
        mod.gemv_fused(x, out, ws, prologue=1, norm_weight=torch.ones(256, dtype=torch.float16, device=cuda), slices_in=sl)
    with pytest.raises(ValueError):
        mod.gemv_fused(x, out, ws, slices_out=torch.zeros(4, 64, dtype=torch.float32, device=cuda))
    with pytest.raises(_lib.ElutqError):                 # the dense part's workspace alone is too small
        mod.gemv_fused(x, out, ws[:mod._ws_bytes])
    with pytest.raises(NotImplementedError):
        GemvGroup([mod], [x], [out])


# ---- the inline form: blocks looked up inside the dense launch ---------------------------------------------------------

def test_inline_form_exists_where_the_blocks_allow_it(cuda, plane_launch):
    L, sp, mod = build(512, 128, 2, 128, 0.3, 5, cuda)
    assert mod.sparse_inline is not None
    four = build(384, 96, 4, 128, 0.5, 6, cuda)[2]                       # the plane would be a fifth: no instance
    assert four.sparse_inline is None
    # off the grid of the groups / two blocks on one cell: the form cannot hold them, the layer keeps its own launch
    k, n, group = 384, 64, 64
    L2 = make_layer(k, n, 2, group, seed=41)
    r = np.random.default_rng(1)
    for mk in (np.array([[0, 4]], np.uint32), np.array([[0, 64], [0, 64]], np.uint32)):
        b = r.integers(0, 2, (len(mk), 32, group), dtype=np.uint8)
        s = r.uniform(0.02, 0.08, (len(mk), 32)).astype(np.float16)
        m2 = HLQLinear.from_export_arrays(L2.w_quant, L2.w_scale, L2.w_zero, group, None, cuda,
                                          SparseBlocks(O.SparsePlane(b, s, mk, group).packed, s, mk), sparse_mode="blocks")
        assert m2.sparse_count == len(mk) and m2.sparse_inline is None
        y = run(m2, L2.x, cuda)[0]
        assert O.rel_err(y, O.gemv_sparse_f64(L2.x[0], L2.w_quant, L2.w_scale, L2.w_zero, O.SparsePlane(b, s, mk, group))) <= TOL


@pytest.mark.parametrize("k,n,bits,group,density", [(512, 128, 2, 128, 0.3), (1024, 256, 3, 64, 0.2), (4096, 4096, 2, 128, 0.1),
                                                     (14336, 4096, 2, 128, 0.1), (4096, 14336, 2, 64, 0.1), (8128, 192, 1, 64, 0.5)])
def test_inline_and_own_launch_agree(cuda, monkeypatch, k, n, bits, group, density):
    """The two ways of running the plane add the same terms in fp32 before the one rounding: results within one fp16
    step of each other, and both within the oracle's bar."""
    L, sp, mod = build(k, n, bits, group, density, k + n + 9, cuda, bias=False)
    assert mod.sparse_inline is not None
    monkeypatch.setattr(HLQLinear, "use_sparse_inline", True)
    yi = run(mod, L.x, cuda)[0]
    monkeypatch.setattr(HLQLinear, "use_sparse_inline", False)
    yo = run(mod, L.x, cuda)[0]
    ref = O.gemv_sparse_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, sp)
    assert O.rel_err(yi, ref) <= TOL and O.rel_err(yo, ref) <= TOL
    assert np.max(np.abs(yi.astype(np.float64) - yo.astype(np.float64))) <= 2.0 ** -9 * max(1.0, np.max(np.abs(ref)))


def test_inline_plane_with_handed_over_slices(cuda, monkeypatch):
    """down -> q|k|v of a decode step with a plane on both layers: the producer leaves its K slices unsummed (the
    blocks' terms are part of each slice's sum), the consumer adds them up in its RMSNorm prologue."""
    monkeypatch.setattr(HLQLinear, "use_sparse_inline", True)
    kd, hid, nq = 14336, 4096, 6144
    Ld, spd, down = build(kd, hid, 2, 128, 0.05, 301, cuda, bias=False)
    Lq, spq, qkv = build(hid, nq, 2, 128, 0.1, 302, cuda, bias=False)
    down.ksplit = _lib.GEMV_WIDE
    qkv.ksplit, qkv.waves = 2, 16
    g = torch.Generator(device=cuda).manual_seed(7)
    gu = torch.randn(1, 2 * kd, generator=g, device=cuda).half()
    res = torch.randn(1, hid, generator=g, device=cuda).half()
    w = (1 + 0.1 * torch.randn(hid, generator=g, device=cuda)).half()
    ws = torch.zeros(max(down.workspace_bytes, qkv.workspace_bytes), dtype=torch.uint8, device=cuda)
    # the producer summing for itself
    x1 = torch.empty(1, hid, dtype=torch.float16, device=cuda)
    down.gemv_fused(gu, x1, ws, prologue=2, residual=res)
    y1 = torch.empty(1, nq, dtype=torch.float16, device=cuda)
    qkv.gemv_fused(x1, y1, ws, prologue=1, norm_weight=w, eps=1e-5)
    # the slices handed over
    assert down.slices >= 2
    sl = torch.zeros(down.slices, hid, dtype=torch.float32, device=cuda)
    dummy = torch.empty(1, hid, dtype=torch.float16, device=cuda)
    down.gemv_fused(gu, dummy, ws, prologue=2, slices_out=sl)
    y2 = torch.empty(1, nq, dtype=torch.float16, device=cuda)
    x2 = torch.empty(1, hid, dtype=torch.float16, device=cuda)
    qkv.gemv_fused(res, y2, ws, prologue=1, norm_weight=w, eps=1e-5, slices_in=sl, x_out=x2)
    assert torch.equal(x1, x2) and torch.equal(y1, y2)
    import torch.nn.functional as F
    act = (F.silu(gu[:, :kd].float()) * gu[:, kd:].float()).half()
    ref = O.gemv_sparse_f64(act.cpu().numpy()[0], Ld.w_quant, Ld.w_scale, Ld.w_zero, spd) + res.cpu().numpy()[0].astype(np.float64)
    assert O.rel_err(x1.cpu().numpy()[0], ref) <= TOL
