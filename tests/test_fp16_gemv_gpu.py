"""Dense fp16 GEMV (elutq_fp16_gemv_f16: the bit == 16 branch of the reference's arm_gemm, the unquantized lm_head
of a decode step) against the float64 product of the same fp16 inputs -- a matrix-vector product needs no oracle of
its own, NumPy's is the textbook one -- and against the unfused RMSNorm.  Tolerance: the sum is formed in fp32 and
rounded once, so |y - ref| <= 2^-10 max(1, |ref|) (one fp16 rounding plus fp32 summation error); rel_err <= 1e-2 as
for every other kernel here."""
import numpy as np
import pytest
import torch

from elutq_amd import _lib
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu


def run(w, x, bias=None, norm_w=None, eps=0.0):
    L = _lib.lib()
    n, k = w.shape
    y = torch.full((n,), float("nan"), dtype=torch.float16, device=w.device)
    rc = L.elutq_fp16_gemv_f16(w.data_ptr(), bias.data_ptr() if bias is not None else None, x.data_ptr(), y.data_ptr(), k, n,
                               norm_w.data_ptr() if norm_w is not None else None, eps, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "elutq_fp16_gemv_f16")
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("k,n", [(4096, 1000), (512, 1), (8, 3), (520, 257), (5120, 64), (8192, 130), (4104, 33), (32768, 5)])
@pytest.mark.parametrize("bias", [False, True])
def test_matches_float64_product(cuda, k, n, bias):
    g = torch.Generator(device=cuda).manual_seed(k + n)
    w = (torch.randn(n, k, generator=g, device=cuda) * 0.05).half()
    x = torch.randn(k, generator=g, device=cuda).half()
    b = torch.randn(n, generator=g, device=cuda).half() if bias else None
    y = run(w, x, b)
    ref = w.cpu().numpy().astype(np.float64) @ x.cpu().numpy().astype(np.float64)
    if bias:
        ref = ref + b.cpu().numpy().astype(np.float64)
    assert y.dtype == np.float16 and y.shape == (n,)
    assert O.rel_err(y, ref) <= 1e-2
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))


def test_exact_on_integer_inputs_and_unit_vectors(cuda):
    r = np.random.default_rng(3)
    k, n = 1536, 100
    w = torch.from_numpy(r.integers(-3, 4, (n, k)).astype(np.float16)).to(cuda)
    x = torch.from_numpy(r.integers(-2, 3, k).astype(np.float16)).to(cuda)
    ref = w.cpu().numpy().astype(np.float64) @ x.cpu().numpy().astype(np.float64)
    assert np.array_equal(run(w, x).astype(np.float64), ref)          # every partial sum is an exact fp32 integer
    for kk in (0, 7, 8, 511, 512, 1535):
        e = torch.zeros(k, dtype=torch.float16, device=cuda)
        e[kk] = 1
        assert np.array_equal(run(w, e), w[:, kk].cpu().numpy())       # x = e_k returns column k


def test_rmsnorm_prologue_equals_the_unfused_operator(cuda):
    """x <- fp16(x * rstd * weight) exactly as elutq_decode_rmsnorm_f16 stores it: the same bits as norm, then GEMV."""
    L = _lib.lib()
    g = torch.Generator(device=cuda).manual_seed(9)
    k, n = 4096, 3000
    w = (torch.randn(n, k, generator=g, device=cuda) * 0.03).half()
    x = (torch.randn(k, generator=g, device=cuda) * 2).half()
    nw = (1 + 0.1 * torch.randn(k, generator=g, device=cuda)).half()
    fused = run(w, x, norm_w=nw, eps=1e-5)
    xn = torch.empty_like(x)
    _lib.check(L.elutq_decode_rmsnorm_f16(x.data_ptr(), nw.data_ptr(), xn.data_ptr(), k, 1e-5,
                                          torch.cuda.current_stream().cuda_stream), "elutq_decode_rmsnorm_f16")
    assert np.array_equal(fused, run(w, xn))
    xf = x.float()
    h = (xf * torch.rsqrt(xf.pow(2).mean() + 1e-5) * nw.float()).half()
    ref = w.cpu().numpy().astype(np.float64) @ h.cpu().numpy().astype(np.float64)
    assert O.rel_err(fused, ref) <= 1e-2


def test_lm_head_size_sampled_rows_and_limits(cuda):
    """128256 x 4096 (the LLaMA-3-8B lm_head): 2048 sampled rows against float64, run-to-run determinism."""
    L = _lib.lib()
    g = torch.Generator(device=cuda).manual_seed(1)
    n, k = 128256, 4096
    w = (torch.randn(n, k, generator=g, device=cuda) * 0.02).half()
    x = torch.randn(k, generator=g, device=cuda).half()
    y = run(w, x)
    idx = np.sort(np.random.default_rng(0).choice(n, 2048, replace=False))
    idx[:2], idx[-2:] = (0, 1), (n - 2, n - 1)
    ref = w[torch.from_numpy(idx).to(cuda)].cpu().numpy().astype(np.float64) @ x.cpu().numpy().astype(np.float64)
    assert np.max(np.abs(y[idx].astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
    assert np.array_equal(y, run(w, x))
    st = torch.cuda.current_stream().cuda_stream
    one = torch.zeros(64, dtype=torch.float16, device=cuda)
    assert L.elutq_fp16_gemv_f16(w.data_ptr(), None, x.data_ptr(), one.data_ptr(), 12, 4, None, 0.0, st) == -2      # K % 8
    assert L.elutq_fp16_gemv_f16(w.data_ptr(), None, x.data_ptr(), one.data_ptr(), 32776, 4, None, 0.0, st) == -2   # K > 32768
    assert L.elutq_fp16_gemv_f16(w.data_ptr() + 2, None, x.data_ptr(), one.data_ptr(), 64, 4, None, 0.0, st) == -2  # alignment
    assert L.elutq_fp16_gemv_f16(None, None, x.data_ptr(), one.data_ptr(), 64, 4, None, 0.0, st) == -1
