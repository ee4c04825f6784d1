"""CPU oracle for the HLQ bit-serial LUT GEMV/GEMM path.  TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy, what the reference (Nkniexin/ELUTQ) computes on
the path "packed --export files -> loader repack -> LUT GEMV/GEMM".  It is the
checker the HIP kernels are compared with; nothing in the shipped package may
import it (only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg).

Reference lines each function follows (paths relative to the reference root):

  pack_planes / unpack_planes   GPTQ/HLQ.py:239-251   (Pack_T_MAC_Weight, LSB-first)
  export_arrays                 GPTQ/HLQ.py:207-236   (w_zero / w_scale / w_quant files)
  weight_config                 GPTQ/HLQ.py:175-193   (weight_config.json keys)
  dequantize                    GPTQ/quant.py:176-183 (W = sum_b q_b*s_b + z)
  rearrange_reference           C++/ops/src/arm/arm_t_mac_kernal.cpp:472-552
  lut_float                     C++/ops/src/arm/arm_t_mac_kernal.cpp:95-138
  gemv_fp16_chain               C++/ops/src/arm/arm_gemm.cpp:248-308 +
                                C++/ops/src/arm/arm_t_mac_kernal.cpp:364-469
  gemm_rows                     C++/ops/src/arm/arm_gemm.cpp:362-387
  lut_int8                      C++/ops/src/arm/arm_t_mac_kernal.cpp:15-93  (int8 LUT, absmax/127 per group)
  gemv_int8lut_f64              the HLQ sum evaluated exactly on those int8 tables
  gemv_int8lut_chain_uniform    C++/ops/src/arm/arm_gemv.cpp:4-34 +
                                C++/ops/src/arm/arm_t_mac_kernal.cpp:258-362 (no caller in the reference)
  sparse_export_arrays          C++/ops/src/arm/parameters.cpp:19-64 (what the loader reads)
  rearrange_sparse_reference    C++/ops/src/arm/arm_t_mac_kernal.cpp:554-647
  dequantize_sparse             C++/ops/src/arm/arm_t_mac_kernal.cpp:678-788 (which weights a block adds to)
  gemv_sparse_fp16_chain        C++/ops/src/arm/arm_gemm.cpp:725-808 +
                                C++/ops/src/arm/arm_t_mac_kernal.cpp:678-788

Parity pins (tests/test_oracle_*.py): the reference ships no tests, golden
vectors or fixtures for this path, so every function is pinned by mathematics:
pack_planes against numpy.packbits(bitorder="little") and hand vectors;
dequantize/gemv against an independent einsum in float64 and the closed forms
(all-zero planes, all-one planes, unit-vector activations, single set bit);
rearrange_reference by bijectivity and by brute-force index enumeration on tiny
shapes; lut_float by brute force over the 16 subsets; gemv_fp16_chain against
the C restatement (oracle/lut_gemv_ref.c, an independent implementation that
indexes the rearranged buffers the way the reference kernel does) bit-for-bit,
and against integer-only inputs where every fp16 operation is exact so the
chain must equal the float64 result bit-for-bit.  The sparse extra plane has no
producer in the reference (its exporter always writes use_sparse = false), so its
format is the one the C++ loader and kernel consume; it is pinned by the cases
that reduce to the dense path (blocks on every tile and group == one more dense
plane, bit for bit; no blocks == the base layer), by brute force over the
loader's index expressions, and by the C restatement bit for bit.  The int8-LUT
variant has no caller either: lut_int8 and the two GEMVs on its tables are pinned
(tests/test_oracle_int8lut_pins.py) by a scalar re-derivation with Python floats,
by invariance under power-of-two scaling and negation, by the cases where int8
tables lose nothing (the exact oracle must come out) and by closed forms; the
byte interleave of its update kernel is not restated, so the variant's WEIGHT
ARRANGEMENT is "parity unpinned" (no loader, exporter or fixture holds one).
"""
from __future__ import annotations

import numpy as np

__all__ = [
    "pack_planes", "unpack_planes", "export_arrays", "weight_config",
    "dequantize", "gemv_f64", "gemm_f64", "rearrange_reference",
    "lut_float", "gemv_fp16_chain", "gemm_rows", "rel_err",
    "SparsePlane", "sparse_export_arrays", "sparse_weight_config", "rearrange_sparse_reference",
    "dequantize_sparse", "gemv_sparse_f64", "gemv_sparse_fp16_chain",
]


# --------------------------------------------------------------------------- #
# a1: bit-plane packing (GPTQ/HLQ.py:239-251)
# --------------------------------------------------------------------------- #
def pack_planes(planes: np.ndarray) -> np.ndarray:
    """uint8 0/1 planes [B, N, K] -> uint8 [B, N, K/8]; bit j of byte i is
    planes[b, n, 8*i + j] (LSB first), exactly the triple loop of
    Pack_T_MAC_Weight."""
    planes = np.asarray(planes)
    assert planes.ndim == 3 and planes.shape[2] % 8 == 0
    b, n, k = planes.shape
    p = planes.astype(np.uint8).reshape(b, n, k // 8, 8)
    out = np.zeros((b, n, k // 8), dtype=np.uint8)
    for j in range(8):
        out |= (p[..., j] & 1) << j
    return out


def unpack_planes(packed: np.ndarray) -> np.ndarray:
    """Inverse of pack_planes: uint8 [B, N, K/8] -> uint8 0/1 [B, N, K]."""
    packed = np.asarray(packed, dtype=np.uint8)
    b, n, k8 = packed.shape
    out = np.zeros((b, n, k8, 8), dtype=np.uint8)
    for j in range(8):
        out[..., j] = (packed >> j) & 1
    return out.reshape(b, n, k8 * 8)


# --------------------------------------------------------------------------- #
# a2: on-disk arrays (GPTQ/HLQ.py:207-236) and json (GPTQ/HLQ.py:175-193)
# --------------------------------------------------------------------------- #
def export_arrays(q: np.ndarray, scale: np.ndarray, zero: np.ndarray):
    """Quantizer-side tensors -> the three file payloads.

    q     uint8 [N, K, B]    (0/1; quant.py:204)
    scale float [N, K/G, B]  (quant.py:205)
    zero  float [N, K/G, 1]  (quant.py:206)

    returns (w_quant uint8 [B,N,K/8], w_scale fp16 [B,N,K/G], w_zero fp16 [N,K/G])
    whose .tobytes() are the contents of w_quant.bin / w_scale.bin / w_zero.bin.
    """
    q = np.asarray(q)
    scale = np.asarray(scale)
    zero = np.asarray(zero)
    assert q.ndim == 3 and scale.ndim == 3 and zero.ndim == 3
    w_zero = zero.astype(np.float16)[..., 0].copy()                    # [N, K/G]   (no permute)
    w_scale = np.ascontiguousarray(scale.astype(np.float16).transpose(2, 0, 1))  # [B, N, K/G]
    planes = np.ascontiguousarray(q.astype(np.uint8).transpose(2, 0, 1))         # [B, N, K]
    w_quant = pack_planes(planes)
    return w_quant, w_scale, w_zero


def weight_config(k: int, n: int, bits: int, has_bias: bool, groupsize: int | None = None) -> dict:
    """Keys written at GPTQ/HLQ.py:177-193.  The exporter never writes
    'groupsize' although the loader reads it (parameters.cpp:17); pass
    groupsize to add it the way a fixed exporter would."""
    cfg = {
        "weight_data_len": int(k * n * bits // 8),
        "base_bit": int(bits),
        "use_sparse": False,
        "in_channel": int(k),
        "out_channel": int(n),
        "has_bias": bool(has_bias),
    }
    if groupsize is not None:
        cfg["groupsize"] = int(groupsize)
    return cfg


# --------------------------------------------------------------------------- #
# a4: dequantize (GPTQ/quant.py:176-183) and the float64 matmul oracle
# --------------------------------------------------------------------------- #
def dequantize(w_quant: np.ndarray, w_scale: np.ndarray, w_zero: np.ndarray, group: int,
               dtype=np.float64) -> np.ndarray:
    """Export arrays -> dense W [N, K]:  W[n,k] = sum_b bit_b[n,k]*s[b,n,k//G] + z[n,k//G]."""
    planes = unpack_planes(w_quant).astype(dtype)           # [B, N, K]
    b, n, k = planes.shape
    assert k % group == 0
    s = np.repeat(np.asarray(w_scale).astype(dtype), group, axis=2)     # [B, N, K]
    z = np.repeat(np.asarray(w_zero).astype(dtype), group, axis=1)      # [N, K]
    return (planes * s).sum(axis=0) + z


def gemv_f64(x, w_quant, w_scale, w_zero, group, bias=None) -> np.ndarray:
    """y[n] = sum_k x[k] W[n,k] (+ bias) in float64 from fp16-valued inputs."""
    w = dequantize(w_quant, w_scale, w_zero, group, np.float64)
    y = w @ np.asarray(x).astype(np.float64).reshape(-1)
    if bias is not None:
        y = y + np.asarray(bias).astype(np.float64)
    return y


def gemm_f64(x, w_quant, w_scale, w_zero, group, bias=None) -> np.ndarray:
    """x [M, K] -> y [M, N] in float64."""
    w = dequantize(w_quant, w_scale, w_zero, group, np.float64)
    y = np.asarray(x).astype(np.float64) @ w.T
    if bias is not None:
        y = y + np.asarray(bias).astype(np.float64)[None, :]
    return y


# --------------------------------------------------------------------------- #
# a7: the loader's permutation (arm_t_mac_kernal.cpp:472-552)
# --------------------------------------------------------------------------- #
def rearrange_reference(w_quant, w_scale, w_zero, group: int, n_thread: int):
    """Returns flat (weight u8, scale f16, zero f16) in the reference's run-time
    layout: planes [thread][bit][tile32][K/8][32], scales [thread][bit][tile32][g][32],
    zeros [tile32][g][32]."""
    w_quant = np.asarray(w_quant, dtype=np.uint8)
    w_scale = np.asarray(w_scale, dtype=np.float16)
    w_zero = np.asarray(w_zero, dtype=np.float16)
    bits, n, k8 = w_quant.shape
    ng = w_zero.shape[1]
    assert w_scale.shape == (bits, n, ng) and ng * group == k8 * 8
    chunk = (n + n_thread - 1) // n_thread
    wq, ws = [], []
    for t in range(n_thread):
        start, end = t * chunk, min((t + 1) * chunk, n)
        if start >= end:
            continue
        assert (end - start) % 32 == 0, "reference requires 32-channel tiles per thread chunk"
        for b in range(bits):
            blk = w_quant[b, start:end].reshape(-1, 32, k8)        # [tile, r, kb]
            wq.append(blk.transpose(0, 2, 1).reshape(-1))          # [tile, kb, r]
    for t in range(n_thread):
        start, end = t * chunk, min((t + 1) * chunk, n)
        if start >= end:
            continue
        for b in range(bits):
            blk = w_scale[b, start:end].reshape(-1, 32, ng)
            ws.append(blk.transpose(0, 2, 1).reshape(-1))
    wz = w_zero.reshape(-1, 32, ng).transpose(0, 2, 1).reshape(-1)
    return np.concatenate(wq), np.concatenate(ws), np.ascontiguousarray(wz)


# --------------------------------------------------------------------------- #
# a8: fp16 LUT (arm_t_mac_kernal.cpp:95-138)
# --------------------------------------------------------------------------- #
def lut_float(x: np.ndarray) -> np.ndarray:
    """x fp16 [K] -> fp16 [K/4, 16]; LUT[c][m] = sequential fp16 sum of x[4c+i]
    over the set bits i of m in ascending i (temp[g] += activation[i+..])."""
    x = np.asarray(x, dtype=np.float16).reshape(-1, 4)
    lut = np.zeros((x.shape[0], 16), dtype=np.float16)
    for m in range(16):
        acc = np.zeros(x.shape[0], dtype=np.float16)
        for i in range(4):
            if m >> i & 1:
                acc = (acc.astype(np.float32) + x[:, i].astype(np.float32)).astype(np.float16)
        lut[:, m] = acc
    return lut


def _h(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


def _mac16(acc, a, b, fused):
    """fp16 acc + a*b: one rounding if fused (fmla), two otherwise."""
    if fused:
        return (acc.astype(np.float64) + a.astype(np.float64) * b.astype(np.float64)).astype(np.float16)
    prod = (a.astype(np.float32) * b.astype(np.float32)).astype(np.float16)
    return (acc.astype(np.float32) + prod.astype(np.float32)).astype(np.float16)


# --------------------------------------------------------------------------- #
# a9/a10: the live fp16 GEMV chain (arm_gemm.cpp:248-308, kernal.cpp:364-469)
# --------------------------------------------------------------------------- #
def gemv_fp16_chain(x, w_quant, w_scale, w_zero, group, bias=None, fused=True) -> np.ndarray:
    """Follows the reference op for op with every fp16 rounding point:
       xs[g]  sequential fp16 sum of the group's activations
       y[n]   sequential over g of fp16 (y + xs[g]*z[n,g])
       per plane: acc_g sequential fp16 sum of LUT[lo nibble] then LUT[hi nibble] per byte;
                  c = acc_0*s_0, then c += acc_g*s_g;  y = fp16(y + c)
       y += bias.
    'fused' selects fmla (one rounding per multiply-add), which is what
    -O3 -ffp-contract=fast yields for `v += a*b` on float16x8_t."""
    x = np.asarray(x, dtype=np.float16).reshape(-1)
    w_quant = np.asarray(w_quant, dtype=np.uint8)
    w_scale = np.asarray(w_scale, dtype=np.float16)
    w_zero = np.asarray(w_zero, dtype=np.float16)
    bits, n, k8 = w_quant.shape
    k = k8 * 8
    ng = k // group
    xs = np.zeros(ng, dtype=np.float16)
    for g in range(ng):
        a = np.float16(0)
        for j in range(group):
            a = np.float16(np.float32(a) + np.float32(x[g * group + j]))
        xs[g] = a
    y = np.zeros(n, dtype=np.float16)
    for g in range(ng):
        y = _mac16(y, np.full(n, xs[g], dtype=np.float16), w_zero[:, g], fused)
    lut = lut_float(x)
    for b in range(bits):
        c = None
        for g in range(ng):
            acc = np.zeros(n, dtype=np.float16)
            for l in range(0, group, 8):
                byte = w_quant[b, :, (g * group + l) // 8]
                c0 = (g * group + l) // 4
                acc = _h(acc.astype(np.float32) + lut[c0, byte & 15].astype(np.float32))
                acc = _h(acc.astype(np.float32) + lut[c0 + 1, byte >> 4].astype(np.float32))
            if g == 0:
                c = _h(acc.astype(np.float32) * w_scale[b, :, 0].astype(np.float32))
            else:
                c = _mac16(c, acc, w_scale[b, :, g], fused)
        y = _h(y.astype(np.float32) + c.astype(np.float32))
    if bias is not None:
        y = _h(y.astype(np.float32) + np.asarray(bias, dtype=np.float16).astype(np.float32))
    return y


def gemm_rows(x, w_quant, w_scale, w_zero, group, bias=None, fused=True) -> np.ndarray:
    """m > 1 in the reference is a row loop over the GEMV (arm_gemm.cpp:380-385)."""
    x = np.asarray(x, dtype=np.float16)
    return np.stack([gemv_fp16_chain(r, w_quant, w_scale, w_zero, group, bias, fused) for r in x])


# --------------------------------------------------------------------------- #
# a14: the int8-LUT variant (arm_gemv.cpp:4-34; arm_t_mac_kernal.cpp:15-93 and 258-362).
# Nothing in the reference calls it and its exporter writes no weights for it (one scale per
# (channel, group) shared by all planes, planes weighted 2^order, no zero point).  What it
# defines on its own is the quantization of the tables, which is what lut_int8 restates; the
# update kernel's byte interleave (low nibbles to channels 0..15 of a tile, high nibbles to
# channels 16..31, :296-318) is not restated: no loader or exporter produces that arrangement.
# --------------------------------------------------------------------------- #
def lut_int8(x, actk: int):
    """x fp16 [K] -> (q int8 [K/4, 16], scale fp16 [K/actk]).  Per group of `actk` activations
    (arm_t_mac_kernal.cpp:22-48): the fp16 subset sums of lut_float, scale = fp16(max|entry| / 127)
    (:50), q = saturate_int8(round-to-nearest-even(fp16(entry / scale))) (:59-90; a NaN quotient,
    0 / 0 in a group of zeros, converts to 0, an infinite one saturates).
    One deliberate difference: the reference's quantizing loop runs `for k < Actk; k += 16` over a group's
    4 * Actk table entries (:52-58), i.e. it converts only the first Actk of them and leaves the rest of
    its output unwritten; here every entry of the group is converted with the group's scale.  The reference
    definition with that loop bound corrected, in other words: parity with the reference is unpinned beyond
    the first Actk entries of a group (nothing in the reference calls, loads or tests the variant)."""
    lut = lut_float(x)
    per = actk // 4
    ng = lut.shape[0] // per
    assert actk % 4 == 0 and ng * per == lut.shape[0]
    scale = np.zeros(ng, dtype=np.float16)
    q = np.zeros(lut.shape, dtype=np.int8)
    for g in range(ng):
        t = lut[g * per:(g + 1) * per]
        m = np.max(np.abs(t))
        s = (np.float32(m) / np.float32(127.0)).astype(np.float16)
        scale[g] = s
        with np.errstate(divide="ignore", invalid="ignore"):
            d = (t.astype(np.float32) / np.float32(s)).astype(np.float16)
        r = np.rint(d.astype(np.float32))
        r = np.where(np.isnan(r), np.float32(0), r)
        q[g * per:(g + 1) * per] = np.clip(r, -128, 127).astype(np.int8)
    return q, scale


def _nibbles(w_quant) -> np.ndarray:
    """uint8 [bits, N, K/8] -> table index per chunk of 4 activations, uint8 [bits, N, K/4]
    (low nibble = the byte's first four k, arm_t_mac_kernal.cpp:302-305)."""
    w = np.asarray(w_quant, dtype=np.uint8)
    return np.stack([w & 15, w >> 4], axis=-1).reshape(w.shape[0], w.shape[1], -1)


def gemv_int8lut_f64(x, w_quant, w_scale, w_zero, group, bias=None) -> np.ndarray:
    """The HLQ sum with the tables quantized by lut_int8, everything else exact:
    y[n] = sum_g ( z[n,g] * sum_{k in g} x[k] + sum_b s[b,n,g] * scale[g] * sum_{chunks c in g} q[c, nibble_b(n, c)] )."""
    x = np.asarray(x, dtype=np.float16).reshape(-1)
    q, sc = lut_int8(x, group)
    idx = _nibbles(w_quant)
    bits, n, k4 = idx.shape
    ng = k4 * 4 // group
    looked = np.take_along_axis(np.broadcast_to(q.astype(np.int64)[None, None], (bits, n, k4, 16)),
                                idx[..., None].astype(np.int64), axis=-1)[..., 0]
    isum = looked.reshape(bits, n, ng, group // 4).sum(-1)
    xs = x.astype(np.float64).reshape(ng, group).sum(-1)
    y = (np.asarray(w_zero, dtype=np.float64) * xs[None, :]).sum(-1)
    y = y + (np.asarray(w_scale, dtype=np.float64) * sc.astype(np.float64)[None, None, :] * isum).sum((0, 2))
    return y if bias is None else y + np.asarray(bias).astype(np.float64)


def gemv_int8lut_chain_uniform(x, w_quant, w_scale, actk: int) -> np.ndarray:
    """arm_gemv (arm_gemv.cpp:4-34) on uniformly quantized planes, op for op in fp16 as
    t_mac_g4_int8_update_impl (:258-362) orders them, every channel reading every chunk:
    per plane `order`, per group: int16 sum of the looked-up int8 entries, converted to fp16;
    c = (v * lut_scale) * w_scale for the first group, c += (v * lut_scale) * w_scale after it (:341-352);
    out = c for plane 0, out += c * 2^order after it (:356-367).  w_scale fp16 [N, K/actk]."""
    x = np.asarray(x, dtype=np.float16).reshape(-1)
    q, sc = lut_int8(x, actk)
    idx = _nibbles(w_quant)
    bits, n, k4 = idx.shape
    ng = k4 * 4 // actk
    w_scale = np.asarray(w_scale, dtype=np.float16)
    out = np.zeros(n, dtype=np.float16)
    for order in range(bits):
        c = None
        for g in range(ng):
            cs = slice(g * actk // 4, (g + 1) * actk // 4)
            acc = np.take_along_axis(np.broadcast_to(q[cs].astype(np.int16)[None], (n, actk // 4, 16)),
                                     idx[order][:, cs, None].astype(np.int64), axis=-1)[..., 0].sum(-1, dtype=np.int16)
            v = acc.astype(np.float16)
            t = _h(_h(v.astype(np.float32) * np.float32(sc[g])).astype(np.float32) * w_scale[:, g].astype(np.float32))
            c = t if g == 0 else _h(c.astype(np.float32) + t.astype(np.float32))
        out = c if order == 0 else _h(out.astype(np.float32) + _h(c.astype(np.float32) * np.float32(1 << order)).astype(np.float32))
    return out


# --------------------------------------------------------------------------- #
# Block-sparse extra plane (use_sparse = true): parameters.cpp:19-64,
# arm_t_mac_kernal.cpp:554-647 and 678-788, arm_gemm.cpp:683-868.
#
# Beside `base_bit` dense planes the layer holds one more plane that exists only
# on listed blocks of 32 output channels x G input channels.  weight_mask.bin is
# a list of uint32 pairs (channel start, k start), grouped by channel start in
# ascending order (the thread split at arm_gemm.cpp:840-846 relies on that).
# Block i's bits follow the dense planes in w_quant.bin as uint8 [32][G/8]
# (LSB-first along K like every plane), its 32 fp16 scales follow the dense
# scales in w_scale.bin; there is no zero term for the extra plane.
# --------------------------------------------------------------------------- #
class SparsePlane:
    """bits uint8 0/1 [nblk, 32, G]; scale fp16 [nblk, 32]; mask uint32 [nblk, 2] = (channel start, k start)."""

    def __init__(self, bits, scale, mask, group: int):
        self.bits = np.asarray(bits, dtype=np.uint8)
        self.scale = np.asarray(scale, dtype=np.float16)
        self.mask = np.asarray(mask, dtype=np.uint32).reshape(-1, 2)
        self.group = int(group)
        nblk = self.mask.shape[0]
        assert self.bits.shape == (nblk, 32, group) and self.scale.shape == (nblk, 32)
        assert np.all(np.diff(self.mask[:, 0].astype(np.int64)) >= 0), "blocks must be grouped by ascending channel start"

    @property
    def packed(self) -> np.ndarray:
        """uint8 [nblk, 32, G/8], the bytes that follow the dense planes in w_quant.bin."""
        return pack_planes(self.bits) if self.bits.size else np.zeros((0, 32, self.group // 8), np.uint8)


def sparse_export_arrays(w_quant, w_scale, sp: SparsePlane):
    """-> (w_quant.bin bytes, w_scale.bin bytes, weight_mask.bin bytes) of a sparse layer:
    the dense payloads (export_arrays) with the block data appended (parameters.cpp:36-64)."""
    wq = np.ascontiguousarray(w_quant, dtype=np.uint8).tobytes() + sp.packed.tobytes()
    ws = np.ascontiguousarray(w_scale, dtype=np.float16).tobytes() + sp.scale.tobytes()
    return wq, ws, np.ascontiguousarray(sp.mask, dtype=np.uint32).tobytes()


def sparse_weight_config(k: int, n: int, base_bits: int, has_bias: bool, sp: SparsePlane, groupsize: int | None = None) -> dict:
    """Keys the loader reads for a sparse layer (parameters.cpp:17-27); weight_data_len is what
    the rearrangement checks: K*N*base_bit/8 + mask_len*2*G (arm_t_mac_kernal.cpp:594)."""
    cfg = weight_config(k, n, base_bits, has_bias, groupsize)
    mask_len = int(sp.mask.size)
    cfg["use_sparse"] = True
    cfg["sparse_mask_len"] = mask_len
    cfg["weight_data_len"] = int(k * n * base_bits // 8 + mask_len * 2 * sp.group)
    return cfg


def rearrange_sparse_reference(w_quant, w_scale, w_zero, sp: SparsePlane):
    """Flat (weight u8, scale f16, zero f16) as t_mac_g4_rearrange_weight_sparse_impl leaves them:
    dense planes [bit][tile32][K/8][32] (no thread dimension), then every block as [G/8][32];
    dense scales [bit][tile32][g][32] followed by the block scales untouched; zeros [tile32][g][32]."""
    wq, ws, wz = rearrange_reference(w_quant, w_scale, w_zero, sp.group, 1)
    blocks = sp.packed.transpose(0, 2, 1).reshape(-1)
    return np.concatenate([wq, blocks]), np.concatenate([ws, sp.scale.reshape(-1)]), wz


def dequantize_sparse(w_quant, w_scale, w_zero, sp: SparsePlane, dtype=np.float64) -> np.ndarray:
    """Dense W [N, K] of a sparse layer: the base planes' W plus, on every block,
    scale[blk, ch] where the block's bit is set."""
    w = dequantize(w_quant, w_scale, w_zero, sp.group, dtype)
    for i, (c0, k0) in enumerate(sp.mask.astype(np.int64)):
        w[c0:c0 + 32, k0:k0 + sp.group] += sp.bits[i].astype(dtype) * sp.scale[i].astype(dtype)[:, None]
    return w


def gemv_sparse_f64(x, w_quant, w_scale, w_zero, sp: SparsePlane, bias=None) -> np.ndarray:
    y = dequantize_sparse(w_quant, w_scale, w_zero, sp) @ np.asarray(x).astype(np.float64).reshape(-1)
    return y if bias is None else y + np.asarray(bias).astype(np.float64)


def gemv_sparse_fp16_chain(x, w_quant, w_scale, w_zero, sp: SparsePlane, bias=None, fused=True) -> np.ndarray:
    """The reference's op order for a sparse layer (arm_gemm.cpp:725-808): zero fold and dense
    planes exactly as in gemv_fp16_chain, then the extra plane as the last one
    (arm_t_mac_kernal.cpp:678-788): per block acc = sequential fp16 sum of LUT[lo] then LUT[hi]
    per byte; over a run of blocks with the same channel start c = acc*s for the first,
    c += acc*s afterwards; out[channels] = fp16(out + c) once per run; bias last."""
    x = np.asarray(x, dtype=np.float16).reshape(-1)
    y = gemv_fp16_chain(x, w_quant, w_scale, w_zero, sp.group, None, fused)
    lut = lut_float(x)
    packed = sp.packed
    nblk = sp.mask.shape[0]
    c = None
    for i in range(nblk):
        c0, k0 = int(sp.mask[i, 0]), int(sp.mask[i, 1])
        acc = np.zeros(32, dtype=np.float16)
        for l in range(0, sp.group, 8):
            byte = packed[i, :, l // 8]
            t = (k0 + l) // 4
            acc = _h(acc.astype(np.float32) + lut[t, byte & 15].astype(np.float32))
            acc = _h(acc.astype(np.float32) + lut[t + 1, byte >> 4].astype(np.float32))
        if i == 0 or c0 != int(sp.mask[i - 1, 0]):
            c = _h(acc.astype(np.float32) * sp.scale[i].astype(np.float32))
        else:
            c = _mac16(c, acc, sp.scale[i], fused)
        if i == nblk - 1 or c0 != int(sp.mask[i + 1, 0]):
            y[c0:c0 + 32] = _h(y[c0:c0 + 32].astype(np.float32) + c.astype(np.float32))
    if bias is not None:
        y = _h(y.astype(np.float32) + np.asarray(bias, dtype=np.float16).astype(np.float32))
    return y


# --------------------------------------------------------------------------- #
# tolerance metric used by every parity test
# --------------------------------------------------------------------------- #
def rel_err(y, ref, floor_frac: float = 0.05) -> float:
    """max_i |y_i - ref_i| / max(|ref_i|, floor_frac * rms(ref)).

    The floor keeps outputs that cross zero from dominating: without it a
    correctly rounded fp16 result next to 0 has unbounded relative error."""
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    den = np.maximum(np.abs(ref), max(floor_frac * rms, 1e-30))
    return float(np.max(np.abs(y - ref) / den)) if ref.size else 0.0
