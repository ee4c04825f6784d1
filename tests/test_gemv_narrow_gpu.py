"""The narrow-tile GEMV kernel (ksplit = ELUTQ_GEMV_NARROW16 / NARROW32: a workgroup owns 16 / 32 columns over
all of K) at the shapes the other GEMV tests do not reach: K up to 8192 (two rounds per wave), unit counts that
leave unit lanes and whole waves without work, ragged N, every plane count and group size; and its limits.
Bar as for the wide-tile kernel: rel_err <= 1e-2 against the float64 oracle, 2^-10 absolute (one fp16 rounding),
bit-exact on integer-valued inputs."""
import numpy as np
import pytest
import torch

from elutq_amd import _lib
from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu
NARROW = [_lib.GEMV_NARROW16, _lib.GEMV_NARROW32]


def to_mod(L, dev, ksplit):
    m = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, dev)
    m.ksplit = ksplit
    return m


def run(m, x, dev):
    y = m(torch.from_numpy(np.ascontiguousarray(x)).to(dev))
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("k,n,bits,group", [
    (8192, 128, 2, 128),     # 64 units: sixteen waves, two rounds at 32 columns
    (6400, 64, 2, 128),      # 50 units: the last wave's unit lanes partly idle
    (4224, 96, 2, 64),       # 33 units: one unit into the second round / ninth wave
    (4096, 256, 3, 128), (4096, 200, 4, 64), (5120, 70, 1, 128), (8192, 65, 3, 64), (640, 17, 2, 64),
    (4160, 96, 2, 64), (8128, 64, 2, 64), (448, 40, 4, 64),       # K ends half way through the last unit of 128
])
@pytest.mark.parametrize("ksplit", NARROW)
def test_narrow_matches_oracle(cuda, k, n, bits, group, ksplit):
    L = make_layer(k, n, bits=bits, group=group, seed=k + n + bits, bias=(n % 2 == 0))
    y = run(to_mod(L, cuda, ksplit), L.x, cuda)[0]
    ref = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias)
    assert O.rel_err(y, ref) <= 1e-2
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))


@pytest.mark.parametrize("k,bits,group", [(4224, 2, 128), (8192, 3, 64), (2176, 4, 128)])
@pytest.mark.parametrize("ksplit", NARROW)
def test_narrow_exact_sums_on_integer_inputs(cuda, k, bits, group, ksplit):
    """x in {-2..2}, power-of-two scales, quarter-integer zeros: every partial sum is an exact fp32 value whichever
    lanes and waves add it up, so the output is the float64 result rounded once to fp16, bit for bit.  (The
    768-k case of test_gemv_gpu.py, whose sums also fit fp16, compares these kernels with the reference's
    fp16 chain as well.)"""
    r = np.random.default_rng(k + bits)
    n = 80
    x = r.integers(-2, 3, (1, k)).astype(np.float16)
    wq = O.pack_planes(r.integers(0, 2, (bits, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // group), 2.0 ** (b - 4), np.float16) for b in range(bits)])
    wz = (r.integers(-3, 1, (n, k // group)) / 4).astype(np.float16)
    m = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda)
    m.ksplit = ksplit
    y = run(m, x, cuda)[0]
    assert np.array_equal(y, O.gemv_f64(x[0], wq, ws, wz, group).astype(np.float16))


def test_library_choice_and_limits(cuda):
    L = _lib.lib()
    # up to 64 / 128 column blocks the library's own launch is the narrow one: the same bits as naming it
    for n, ks in ((4096, _lib.GEMV_NARROW16), (6144, _lib.GEMV_NARROW32)):
        Lr = make_layer(512, n, bits=2, group=128, seed=n)
        assert np.array_equal(run(to_mod(Lr, cuda, 0), Lr.x, cuda), run(to_mod(Lr, cuda, ks), Lr.x, cuda))
    # tables of all of K in one workgroup: K <= 8192
    big = make_layer(8320, 64, bits=2, group=128, seed=1)
    for ks in NARROW:
        with pytest.raises(_lib.ElutqError):
            run(to_mod(big, cuda, ks), big.x, cuda)
    assert np.all(np.isfinite(run(to_mod(big, cuda, 0), big.x, cuda)))            # the library falls back to wide tiles
    # a wave count goes with K slices only
    m = to_mod(make_layer(512, 64, bits=2, group=128, seed=2), cuda, _lib.GEMV_NARROW16)
    m.waves = 8
    with pytest.raises(_lib.ElutqError):
        m(torch.zeros(1, 512, dtype=torch.float16, device=cuda))
    # no K slices to hand over
    m.waves = 0
    ws = torch.zeros(m.workspace_bytes, dtype=torch.uint8, device=cuda)
    with pytest.raises(_lib.ElutqError):
        m.gemv_fused(torch.zeros(1, 512, dtype=torch.float16, device=cuda), torch.zeros(1, 64, dtype=torch.float16, device=cuda),
                     ws, slices_out=torch.zeros(4, 64, dtype=torch.float32, device=cuda))
    assert L.elutq_hlq_gemv_slices(512, 64, 2, 128, _lib.GEMV_NARROW16, 0) == 1
    assert L.elutq_hlq_gemv_slices(512, 64, 2, 128, _lib.GEMV_WIDE, 0) == L.elutq_hlq_gemv_slices(512, 64, 2, 128, 0, 0) >= 2
