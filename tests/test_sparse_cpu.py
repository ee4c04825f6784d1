"""Host side of the block-sparse extra plane: the export files of a use_sparse layer, the index
the kernels read, and the repack CLI.  No GPU."""
import json
import os

import numpy as np
import pytest

from elutq_amd import _lib
from elutq_amd.export_io import (SparseBlocks, densify_sparse, read_export_dir, read_repacked_dir, read_repacked_sparse,
                                 write_export_dir)
from elutq_amd.hlq_linear import sparse_index, unpack_to_export_arrays
from elutq_amd.repack import repack_tree
from elutq_amd.synth import make_layer, make_sparse_plane, pack_bits_lsb_first
from oracle import hlq_oracle as O


def sparse_layer(k, n, bits, group, density, seed):
    L = make_layer(k, n, bits, group, seed=seed, bias=True)
    b, s, m = make_sparse_plane(k, n, group, density, seed=seed + 100)
    return L, b, s, m, SparseBlocks(pack_bits_lsb_first(b), s, m)


def test_export_files_are_what_the_reference_loader_reads(tmp_path):
    """Byte for byte the payloads the oracle derives from the loader's offsets and sizes."""
    L, b, s, m, sp = sparse_layer(256, 96, 2, 64, 0.5, 1)
    d = str(tmp_path / "0" / "mlp.up_proj")
    write_export_dir(d, L.w_quant, L.w_scale, L.w_zero, L.bias, sparse=sp)
    osp = O.SparsePlane(b, s, m, 64)
    wq, ws, mk = O.sparse_export_arrays(L.w_quant, L.w_scale, osp)
    assert open(os.path.join(d, "w_quant.bin"), "rb").read() == wq
    assert open(os.path.join(d, "w_scale.bin"), "rb").read() == ws
    assert open(os.path.join(d, "weight_mask.bin"), "rb").read() == mk
    assert json.load(open(os.path.join(d, "weight_config.json"))) == O.sparse_weight_config(256, 96, 2, True, osp)
    e = read_export_dir(d)
    assert (e.k, e.n, e.bits, e.group) == (256, 96, 2, 64)
    assert np.array_equal(e.w_quant, L.w_quant) and np.array_equal(e.w_scale, L.w_scale)
    assert np.array_equal(e.sparse.blocks, sp.blocks) and np.array_equal(e.sparse.scale, s)
    assert np.array_equal(e.sparse.mask, m)
    with open(os.path.join(d, "weight_mask.bin"), "r+b") as f:
        f.truncate(8)
    with pytest.raises(ValueError):
        read_export_dir(d)


def test_index_is_a_row_pointer_over_channel_tiles():
    k, n, g = 512, 160, 128
    _, _, mask = make_sparse_plane(k, n, g, 0.5, seed=3)
    idx = sparse_index(mask, k, n, g)
    tiles, nblk, head = n // 32, mask.shape[0], 16
    assert idx.dtype == np.int32 and idx.size == tiles + 1 + nblk + tiles * head
    counts = np.bincount(mask[:, 0] // 32, minlength=tiles)
    ptr = np.concatenate([[0], np.cumsum(counts)])
    assert np.array_equal(idx[:tiles + 1], ptr)
    assert np.array_equal(idx[tiles + 1:tiles + 1 + nblk], mask[:, 1].astype(np.int32))
    # behind it, per tile, the k starts of its first 16 blocks once more (-1: no such block)
    h = idx[tiles + 1 + nblk:].reshape(tiles, head)
    for t in range(tiles):
        want = mask[ptr[t]:ptr[t + 1], 1].astype(np.int32)[:head]
        assert np.array_equal(h[t, :want.size], want) and np.all(h[t, want.size:] == -1)
    # ragged N: the last tile is partial
    assert sparse_index(np.array([[96, 0]], np.uint32), 128, 100, 128).tolist() == [0, 0, 0, 0, 1, 0] + [-1] * 48 + [0] + [-1] * 15
    assert sparse_index(np.zeros((0, 2), np.uint32), 128, 64, 64).tolist() == [0, 0, 0] + [-1] * 32
    # more blocks on a tile than the head holds: the first 16 there, all of them in the list
    many = np.array([[0, 4 * i] for i in range(20)], np.uint32)
    idx = sparse_index(many, 256, 32, 128)
    assert idx[:2].tolist() == [0, 20] and idx[2:22].tolist() == [4 * i for i in range(20)] and idx[22:].tolist() == [4 * i for i in range(16)]


@pytest.mark.parametrize("mask", [
    [32, 0, 64],              # odd length
    [16, 0],                  # channel start not a multiple of 32
    [128, 0],                 # channel start beyond N
    [0, 2],                   # k start not a multiple of 4
    [0, 192],                 # block ends beyond K
    [64, 0, 32, 0],           # descending channel starts
])
def test_index_rejects_malformed_lists(mask):
    with pytest.raises(_lib.ElutqError) as e:
        sparse_index(np.array(mask, np.uint32), 256, 128, 128)
    assert e.value.status == -8 and "sparse" in str(e.value)


def test_dense_form_of_the_plane_is_the_same_weight():
    """One more dense plane with scale 0 where no block exists dequantizes to exactly the sparse layer's W;
    planes that do not fit that form are reported as such."""
    L, b, s, m, sp = sparse_layer(384, 96, 2, 128, 0.5, 7)
    wq, ws = densify_sparse(L.w_quant, L.w_scale, sp, 128)
    assert wq.shape == (3, 96, 48) and ws.shape == (3, 96, 3) and ws.dtype == np.float16
    assert np.array_equal(wq[:2], L.w_quant) and np.array_equal(ws[:2], L.w_scale)
    assert np.array_equal(O.dequantize(wq, ws, L.w_zero, 128), O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, O.SparsePlane(b, s, m, 128)))
    # ragged N: the rows of the last tile beyond N are dropped
    wq2, ws2 = densify_sparse(L.w_quant[:, :70], L.w_scale[:, :70], sp, 128)
    assert np.array_equal(wq2[2], wq[2, :70]) and np.array_equal(ws2[2], ws[2, :70])
    one = SparseBlocks(sp.blocks[:1], s[:1], np.array([[0, 0]], np.uint32))
    assert densify_sparse(L.w_quant, L.w_scale, SparseBlocks(sp.blocks[:1], s[:1], np.array([[0, 4]], np.uint32)), 128) is None
    assert densify_sparse(L.w_quant, L.w_scale, SparseBlocks(sp.blocks[:2], s[:2], np.array([[32, 128], [32, 128]], np.uint32)), 128) is None
    assert densify_sparse(np.zeros((4, 96, 48), np.uint8), np.zeros((4, 96, 3), np.float16), one, 128) is None
    assert densify_sparse(L.w_quant, L.w_scale, one, 128) is not None


def test_repack_cli_and_the_sparse_plane(tmp_path):
    L, b, s, m, sp = sparse_layer(256, 64, 2, 128, 0.5, 5)
    src = str(tmp_path / "src")
    write_export_dir(os.path.join(src, "0", "mlp.down_proj"), L.w_quant, L.w_scale, L.w_zero, L.bias, sparse=sp)
    write_export_dir(os.path.join(src, "0", "mlp.up_proj"), L.w_quant, L.w_scale, L.w_zero)
    # default: the plane becomes a third dense plane
    dst = str(tmp_path / "dst")
    assert repack_tree(src, dst) == 2
    k, n, bits, group, planes, scales, zeros, bias = read_repacked_dir(os.path.join(dst, "0", "mlp.down_proj"))
    assert (k, n, bits, group) == (256, 64, 3, 128) and read_repacked_sparse(os.path.join(dst, "0", "mlp.down_proj")) is None
    wq, ws, wz = unpack_to_export_arrays(planes, scales, zeros, k, n, bits, group)
    assert np.array_equal(O.dequantize(wq, ws, wz, 128), O.dequantize_sparse(L.w_quant, L.w_scale, L.w_zero, O.SparsePlane(b, s, m, 128)))
    # "blocks": the file form is kept beside the two dense planes
    dst = str(tmp_path / "dst_blocks")
    assert repack_tree(src, dst, sparse_mode="blocks") == 2
    assert read_repacked_dir(os.path.join(dst, "0", "mlp.down_proj"))[2] == 2
    got = read_repacked_sparse(os.path.join(dst, "0", "mlp.down_proj"))
    assert np.array_equal(got.blocks, sp.blocks) and np.array_equal(got.scale, s) and np.array_equal(got.mask, m)
    assert read_repacked_sparse(os.path.join(dst, "0", "mlp.up_proj")) is None
    # a malformed list stops the repack instead of producing a tree that faults later
    bad = SparseBlocks(sp.blocks[:1], s[:1], np.array([[0, 130]], np.uint32))
    write_export_dir(os.path.join(src, "1", "mlp.up_proj"), L.w_quant, L.w_scale, L.w_zero, sparse=bad)
    with pytest.raises(_lib.ElutqError):
        repack_tree(src, str(tmp_path / "dst2"))
