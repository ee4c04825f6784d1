"""CPU-only tests of the host side: the C-ABI library loads and exports every symbol the
header declares, the host repack is a bijection with the documented layout, the export
directory reader/writer round-trips, and argument checks return the documented codes.
No GPU compute is called here."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

from elutq_amd import _lib
from elutq_amd.export_io import read_export_dir, write_export_dir
from elutq_amd.hlq_linear import repack_export_arrays, unpack_to_export_arrays
from elutq_amd.synth import algorithmic_bytes, make_layer

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "elutq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(elutq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = header_symbols()
    assert "elutq_hlq_gemv_f16" in names and "elutq_hlq_repack_host" in names and len(names) >= 12
    L = _lib.lib()
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/elutq_hip.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes table and header disagree"
    assert L.elutq_version() >= 100
    assert L.elutq_status_string(0) == b"ok"
    assert b"group" in L.elutq_status_string(-4)


def test_size_queries_and_argument_errors():
    L = _lib.lib()
    assert L.elutq_hlq_planes_bytes(4096, 4096, 2) == 4096 * 4096 * 2 // 8
    assert L.elutq_hlq_scales_bytes(4096, 4096, 2, 128) == 2 * 2 * 4096 * 32
    assert L.elutq_hlq_zeros_bytes(4096, 4096, 128) == 2 * 4096 * 32
    # columns are padded to 64, an odd number of groups to an even one
    assert L.elutq_hlq_planes_bytes(384, 70, 3) == 128 * 3 * 3 * 16 * 8 // 8
    assert L.elutq_hlq_zeros_bytes(384, 70, 128) == 128 * 2 * 4
    assert L.elutq_hlq_planes_bytes(100, 64, 2) == 0          # K % 64
    # K may end half way through the last unit of 128 at group 64 (the reference asks for K % groupsize == 0 only,
    # arm_gemm.cpp:249): the unit is stored whole
    assert L.elutq_hlq_planes_bytes(320, 64, 2) == 64 * 3 * 2 * 16
    assert L.elutq_hlq_scales_bytes(320, 64, 2, 64) == 64 * 3 * 2 * 4 and L.elutq_hlq_scales_bytes(320, 64, 2, 128) == 0
    assert L.elutq_hlq_zeros_bytes(320, 64, 64) == 64 * 3 * 4 and L.elutq_hlq_workspace_bytes(320, 64, 2, 64, 1) >= 64 * 1024
    assert L.elutq_hlq_workspace_bytes(4096, 4096, 2, 32, 1) == 0
    assert L.elutq_hlq_workspace_bytes(4096, 4096, 2, 128, 1) >= 64 * 1024
    one = ctypes.c_void_p(1)
    g = lambda K, N, b, G: L.elutq_hlq_gemv_f16(one, one, one, None, one, one, K, N, b, G, None, 0, None)
    assert g(4096, 64, 5, 128) == -3
    assert g(4096, 64, 2, 32) == -4
    assert g(4000, 64, 2, 128) == -2
    assert g(4096, 0, 2, 128) == -2
    assert g(320, 64, 2, 128) == -2 and g(64, 64, 2, 64) == -2 and g(352, 64, 2, 64) == -2
    assert L.elutq_hlq_gemv_f16(None, one, one, None, one, one, 4096, 64, 2, 128, None, 0, None) == -1
    assert L.elutq_hlq_gemm_f16(one, one, one, None, one, one, 0, 4096, 64, 2, 128, None, 0, None) == -2
    assert L.elutq_hlq_repack_host(None, None, None, 128, 64, 2, 128, None, None, None) == -1
    with pytest.raises(_lib.ElutqError, match="group must be 64 or 128"):
        _lib.check(-4, "t")
    # K slices of a batch-1 launch: none where the column blocks fill the chip, up to four where they do not,
    # the caller's count when given, 0 for what no launch accepts
    assert L.elutq_hlq_gemv_slices(4096, 14336, 2, 128, 0, 0) == 1
    assert L.elutq_hlq_gemv_slices(4096, 4096, 2, 128, 0, 0) == 1
    assert L.elutq_hlq_gemv_slices(14336, 4096, 2, 128, 0, 0) == 4
    assert L.elutq_hlq_gemv_slices(4096, 1024, 2, 128, 0, 0) == 4
    assert L.elutq_hlq_gemv_slices(4096, 6144, 2, 128, 2, 16) == 2
    assert L.elutq_hlq_gemv_slices(256, 64, 2, 128, 0, 0) == 2          # never more slices than units
    assert L.elutq_hlq_gemv_slices(4096, 4096, 2, 128, 33, 0) == 0
    assert L.elutq_hlq_gemv_slices(4000, 4096, 2, 128, 0, 0) == 0
    # entry points that take handed-over slices check their arguments before any launch
    assert L.elutq_decode_rope_attn_sliced_f16(None, 2, 2048, one, one, one, one, 4, 2, 128, 64, 10000.0, 1, None, 0, None) == -1
    assert L.elutq_decode_rope_attn_sliced_f16(one, 5, 2048, one, one, one, one, 4, 2, 128, 64, 10000.0, 1, None, 0, None) == -7
    assert L.elutq_decode_rope_attn_sliced_f16(one, 2, 100, one, one, one, one, 4, 2, 128, 64, 10000.0, 1, None, 0, None) == -7
    assert L.elutq_decode_rope_attn_sliced_f16(one, 2, 2048, one, one, one, one, 4, 2, 64, 64, 10000.0, 1, None, 0, None) == -7
    f = _lib.GemvFusion(0, 0.0, None, None, None, ctypes.c_void_p(1), 2, None)
    fused = lambda fus, ks=0: L.elutq_hlq_gemv_fused_f16(one, one, one, None, one, one, 4096, 64, 2, 128, one, 1 << 20, None,
                                                         ctypes.byref(fus), ks, 0)
    assert fused(f) == -7                                               # slices come with the RMSNorm prologue only
    assert fused(_lib.GemvFusion(1, 1e-5, one, None, None, one, 5, None)) == -7      # at most four
    assert fused(_lib.GemvFusion(1, 1e-5, one, None, None, one, 2, one)) == -7       # x_out may not be x itself
    wide = L.elutq_hlq_gemv_fused_f16(one, one, one, None, one, one, 4096, 28672, 2, 128, one, 1 << 20, None,
                                      ctypes.byref(_lib.GemvFusion(1, 1e-5, one, None, None, one, 2, None)), 0, 0)
    assert wide == -7                                                   # a consumer has one tile per compute unit at most
    assert fused(_lib.GemvFusion(0, 0.0, None, one, one, None, 0, None), 4) == -7    # the consumer adds the residual
    assert fused(_lib.GemvFusion(0, 0.0, None, None, one, None, 0, None), 1) == -7   # one slice: nothing to hand over
    # the buffers of handed-over slices come with their sizes: a producer's S x N floats, a consumer's n_slices_in x K
    GF = _lib.GemvFusion
    assert fused(GF(1, 1e-5, one, None, None, one, 2, None, 0, 2 * 4096 * 4 - 1)) == -5
    assert fused(GF(1, 1e-5, one, None, None, one, 2, None, 0, 0)) == -5
    assert fused(GF(0, 0.0, None, None, one, None, 0, None, 4 * 64 * 4 - 1, 0), 4) == -5
    assert fused(GF(0, 0.0, None, None, one, None, 0, None, 0, 0), 2) == -5
    # the query a caller decides with before it lets a producer leave its slices unsummed: the launch's own limits
    acc = L.elutq_hlq_gemv_accepts_slices
    assert acc(4096, 6144, 2, 128, 2, 16, 4) == 1                       # LLaMA-3-8B q|k|v in two K slices: 192 tiles
    assert acc(4096, 6144, 2, 128, 0, 0, 4) == 1
    assert acc(4096, 28672, 2, 128, 0, 0, 2) == 0                       # more tiles than compute units (what `wide` is refused for)
    assert acc(8192, 10240, 2, 128, 2, 16, 4) == 0                      # a q|k|v of 160 column blocks in two slices: 320 tiles
    assert acc(8192, 10240, 2, 128, 1, 16, 4) == 1
    assert acc(4096, 6144, 2, 128, 2, 16, 5) == 0 and acc(4096, 6144, 2, 128, 2, 16, 0) == 0
    assert acc(4000, 6144, 2, 128, 0, 0, 2) == 0


def test_decoder_defers_down_only_where_the_next_qkv_takes_the_slices():
    """A decode step must never meet a launch that refuses handed-over slices: the decision is the library's
    query, taken per layer when the decoder is built (here replayed on shapes, no GPU needed)."""
    L = _lib.lib()
    # LLaMA-3-8B: down 14336 -> 4096 in four slices, q|k|v 4096 -> 6144 in two slices: taken
    n_d = L.elutq_hlq_gemv_slices(14336, 4096, 2, 128, 0, 0)
    assert n_d == 4 and L.elutq_hlq_gemv_accepts_slices(4096, 6144, 2, 128, 2, 16, n_d) == 1
    # a model with hidden 8192 and 64 + 2 x 8 heads of 128: q|k|v has 160 column blocks; in two K slices that is
    # 320 tiles for 256 compute units -> the launch walks runs of column blocks and takes no slices, so
    # down (16384 -> 8192, sliced) must sum for itself
    n_d = L.elutq_hlq_gemv_slices(16384, 8192, 2, 128, 0, 0)
    assert 2 <= n_d <= 4
    assert L.elutq_hlq_gemv_accepts_slices(8192, 10240, 2, 128, 2, 16, n_d) == 0


@pytest.mark.parametrize("k,n,bits,group", [(256, 64, 2, 128), (384, 70, 3, 128), (128, 1, 1, 64),
                                             (512, 200, 4, 64), (1024, 128, 2, 64), (192, 70, 2, 64), (1088, 64, 3, 64)])
def test_repack_roundtrip_and_layout(k, n, bits, group):
    L = make_layer(k, n, bits=bits, group=group, seed=3)
    planes, scales, zeros = repack_export_arrays(L.w_quant, L.w_scale, L.w_zero, group)
    wq, ws, wz = unpack_to_export_arrays(planes, scales, zeros, k, n, bits, group)
    assert np.array_equal(wq, L.w_quant)
    assert np.array_equal(ws.view(np.uint16), L.w_scale.view(np.uint16))
    assert np.array_equal(wz.view(np.uint16), L.w_zero.view(np.uint16))
    # documented layout, checked independently of the library's inverse:
    ncb, U, NG = (n + 63) // 64, (k + 127) // 128, k // group
    NT = (NG + 1) // 2
    p = planes.view(np.uint32).reshape(ncb, U, bits, 64, 4)
    rot = lambda v, r: ((int(v) >> r) | (int(v) << (32 - r))) & 0xFFFFFFFF
    rs = np.random.default_rng(0)
    for _ in range(80):
        col, u, b, d, i = rs.integers(n), rs.integers(U), rs.integers(bits), rs.integers(4), rs.integers(32)
        kk = u * 128 + d * 32 + i
        want = (L.w_quant[b, col, kk // 8] >> (kk % 8)) & 1 if kk < k else 0      # past K: zero bits
        natural = rot(p[col // 64, u, b, col % 64, d], 2)          # undo the rotate-left by 2
        assert (natural >> i) & 1 == want
    s = scales.view(np.uint16).reshape(ncb, NT, bits, 64, 2)
    z = zeros.view(np.uint16).reshape(ncb, NT, 64, 2)
    for _ in range(50):
        col, g, b = rs.integers(n), rs.integers(NG), rs.integers(bits)
        assert s[col // 64, g // 2, b, col % 64, g % 2] == L.w_scale.view(np.uint16)[b, col, g]
        assert z[col // 64, g // 2, col % 64, g % 2] == L.w_zero.view(np.uint16)[col, g]
    # padding columns are zero
    if n % 64:
        assert not p[-1, :, :, n % 64:, :].any() and not s[-1, :, :, n % 64:, :].any()


def test_repack_rejects_bad_shapes():
    L = make_layer(256, 64, seed=1)
    with pytest.raises(ValueError):
        repack_export_arrays(L.w_quant, L.w_scale, L.w_zero, 64)       # wrong group for these scales
    with pytest.raises(ValueError):
        repack_export_arrays(L.w_quant[:, :, :8], L.w_scale[:, :, :1], L.w_zero[:, :1], 64)   # K = 64


def test_export_dir_roundtrip(tmp_path):
    L = make_layer(256, 96, bits=3, group=64, seed=5, bias=True)
    d = tmp_path / "0" / "self_attn.q_proj"
    write_export_dir(str(d), L.w_quant, L.w_scale, L.w_zero, L.bias)
    cfg = json.load(open(d / "weight_config.json"))
    assert cfg == {"weight_data_len": 256 * 96 * 3 // 8, "base_bit": 3, "use_sparse": False,
                   "in_channel": 256, "out_channel": 96, "has_bias": True}       # no groupsize key
    assert os.path.getsize(d / "w_quant.bin") == 256 * 96 * 3 // 8
    assert os.path.getsize(d / "w_scale.bin") == 2 * 3 * 96 * 4
    assert os.path.getsize(d / "w_zero.bin") == 2 * 96 * 4
    e = read_export_dir(str(d))                      # group derived from the w_zero.bin size
    assert (e.k, e.n, e.bits, e.group) == (256, 96, 3, 64)
    assert np.array_equal(e.w_quant, L.w_quant) and np.array_equal(e.w_scale, L.w_scale)
    assert np.array_equal(e.w_zero, L.w_zero) and np.array_equal(e.bias, L.bias)
    write_export_dir(str(d), L.w_quant, L.w_scale, L.w_zero, None, groupsize=64)
    assert read_export_dir(str(d)).group == 64 and read_export_dir(str(d)).bias is None
    # truncated file -> error, not garbage
    with open(d / "w_scale.bin", "r+b") as f:
        f.truncate(10)
    with pytest.raises(ValueError):
        read_export_dir(str(d))


def test_algorithmic_bytes_table():
    assert algorithmic_bytes(4096, 4096, 2, 128) == 4_997_120
    assert algorithmic_bytes(4096, 1024, 2, 128) == 1_255_424
    assert algorithmic_bytes(4096, 14336, 2, 128) == 17_469_440
    assert algorithmic_bytes(14336, 4096, 2, 128) == 17_469_440
    assert algorithmic_bytes(4096, 4096, 3, 128) == 7_356_416
    assert algorithmic_bytes(4096, 4096, 2, 64) == 5_783_552


def test_bench_refuses_more_than_one_gpu():
    """The path needs no collective and every figure is for one GPU: `bench.py --gpus N`, N > 1, says so
    and exits with status 2 before it touches a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""


@pytest.mark.parametrize("k,n,group", [(512, 128, 128), (768, 96, 64), (448, 64, 64), (1024, 100, 128)])
def test_sparse_inline_form_holds_every_block_where_the_kernel_looks(k, n, group):
    """elutq_hlq_sparse_inline_host against a bit-by-bit reconstruction: per (column block, unit) a record, in it lane n's
    plane bits at the dense planes' positions (dword d = k 32d..32d+31 of the unit, rotated left by 2) and the fp16
    scales of the unit's two 64-k halves; zero wherever no block lies."""
    from elutq_amd.hlq_linear import sparse_inline
    from elutq_amd.synth import make_sparse_plane, pack_bits_lsb_first
    npad = (n + 31) // 32 * 32
    bits, scale, mask = make_sparse_plane(k // group * group, npad, group, 0.4, seed=k + n)
    keep = mask[:, 0] < n
    bits, scale, mask = bits[keep], scale[keep], mask[keep]
    form = sparse_inline(mask, pack_bits_lsb_first(bits), scale, k, n, group)
    assert form is not None
    U, ncb = (k + 127) // 128, (n + 63) // 64
    head = form[:32].view(np.int32)
    assert head[0] == 0x53504c31 and list(head[1:6]) == [k, n, group, U, ncb]
    cells = form[32:32 + 4 * ncb * U].view(np.int32).reshape(ncb, U)
    recs_off = (32 + 4 * ncb * U + 255) // 256 * 256
    nrec = int(head[6])
    assert form.size == recs_off + 1280 * nrec
    recs = form[recs_off:].reshape(nrec, 1280)
    # the plane as a dense [npad64, U * 128] bit matrix and a per-(channel, 64-k half) scale matrix
    want_bits = np.zeros((ncb * 64, U * 128), np.uint8)
    want_scale = np.zeros((ncb * 64, U * 2), np.float16)
    for b, s, (c, k0) in zip(bits, scale, mask):
        want_bits[c:c + 32, k0:k0 + group] = b
        for h in range(k0 // 64, (k0 + group) // 64):
            want_scale[c:c + 32, h] = s
    used = set()
    for cb in range(ncb):
        for u in range(U):
            blk = want_bits[64 * cb:64 * cb + 64, 128 * u:128 * u + 128]
            sc = want_scale[64 * cb:64 * cb + 64, 2 * u:2 * u + 2]
            c = cells[cb, u]
            if c < 0:
                assert not blk.any() and not sc.any()
                continue
            assert 0 <= c < nrec and c not in used
            used.add(int(c))
            w = recs[c, :1024].view(np.uint32).reshape(64, 4)
            w = (w >> 2) | (w << 30)                                    # rotation undone
            got = ((w[:, :, None] >> np.arange(32, dtype=np.uint32)) & 1).astype(np.uint8).reshape(64, 128)
            assert np.array_equal(got, blk)
            got_sc = recs[c, 1024:].view(np.float16).reshape(64, 2)
            assert np.array_equal(got_sc, sc)
    assert len(used) == nrec
    # what the form cannot hold comes back as None: a block off the grid of the groups, two blocks on one cell
    one = pack_bits_lsb_first(bits[:1])
    assert sparse_inline(np.array([[0, 4]], np.uint32), one, scale[:1], k, n, group) is None
    two = pack_bits_lsb_first(bits[[0, 0]])
    assert sparse_inline(np.array([[0, 0], [0, 0]], np.uint32), two, scale[[0, 0]], k, n, group) is None


def test_inline_sparse_call_checks_the_size_of_the_form():
    """A form smaller than the layer's cell table is refused before anything is launched (no GPU needed for the
    refusal: the argument checks come first)."""
    L = _lib.lib()
    one = ctypes.c_void_p(256)          # never dereferenced
    need = 32 + 4 * (4096 // 64) * (4096 // 128)
    rc = L.elutq_hlq_sparse_gemv_inline_f16(one, one, one, None, one, need - 1, one, one, 4096, 4096, 2, 128, one, 1 << 20,
                                            None, None, 0, 0)
    assert rc == -5, rc                 # ELUTQ_ERR_WORKSPACE
    rc = L.elutq_hlq_sparse_gemv_inline_f16(one, one, one, None, one, 1 << 20, one, one, 4096, 4096, 4, 128, one, 1 << 20,
                                            None, None, 0, 0)
    assert rc == -3, rc                 # ELUTQ_ERR_BITS: the plane would be a fifth
