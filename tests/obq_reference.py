"""A textbook restatement of GPTQ / OBQ error compensation, written to pin elutq_amd.hlq_quantize.gptq_hlq
(the counterpart of HLQ.fasterquant, GPTQ/HLQ.py:108-153) by brute force on small inputs.  It shares nothing with the
implementation under test but the injected group quantizer: no Cholesky factor, no blocked update -- the inverse
Hessian of the columns not yet quantized is kept explicitly in float64 and one column at a time is eliminated from it:

    q_i        the group's quantization (made when the group starts, from the weights as compensated so far) at column i
    e          = (w_i - q_i) / Hinv[i, i]
    W[:, j]   -= e * Hinv[i, j]                  for every later column j
    Hinv      -= Hinv[:, i] Hinv[i, :] / Hinv[i, i]      (column i leaves the problem)

(Frantar et al., "GPTQ", eq. 2-3 with the quantization order fixed.)  The rows of the Cholesky factor the reference
uses are these rows Hinv[i, i:] divided by sqrt(Hinv[i, i]), which is why the two must agree."""
import numpy as np


def uniform_group_quantizer(w1, bits, group, iters=0):
    """A min / max grid per row: simple, deterministic, the same function for both implementations.  Takes and returns
    what quantize_groups does (w_q, codes, scales, zeros); codes / scales / zeros only in shape."""
    import torch
    w = w1.double()
    lo, hi = w.min(dim=1, keepdim=True).values, w.max(dim=1, keepdim=True).values
    step = (hi - lo).clamp_min(1e-12) / (2 ** bits - 1)
    lev = torch.round((w - lo) / step).clamp(0, 2 ** bits - 1)
    wq = (lo + lev * step).to(w1.dtype)
    rows, cols = w1.shape
    codes = torch.stack([(lev.long() >> b) & 1 for b in range(bits)], dim=2).to(torch.uint8)
    scales = torch.stack([step[:, 0] * 2.0 ** b for b in range(bits)], dim=1).reshape(rows, 1, bits).float()
    return wq, codes, scales, lo.reshape(rows, 1, 1).float()


def obq_reference(weight, hessian, bits, group, percdamp=0.01, actorder=False, quantizer=uniform_group_quantizer):
    """weight [N, K], hessian [K, K] (NumPy) -> w_q [N, K] float64."""
    import torch
    w = np.array(weight, dtype=np.float64)
    h = np.array(hessian, dtype=np.float64)
    n, k = w.shape
    dead = np.diag(h) == 0
    h[dead, dead] = 1
    w[:, dead] = 0
    if actorder:
        perm = np.argsort(-np.diag(h), kind="stable")
        w, h = w[:, perm], h[perm][:, perm]
    h = h + np.eye(k) * (percdamp * np.mean(np.diag(h)))
    hinv = np.linalg.inv(h)
    wq = np.zeros_like(w)
    for c0 in range(0, k, group):
        c1 = min(c0 + group, k)
        q1 = quantizer(torch.from_numpy(w[:, c0:c1].copy()), bits, c1 - c0)[0].double().numpy()
        for i in range(c0, c1):
            e = (w[:, i] - q1[:, i - c0]) / hinv[i, i]
            w[:, i + 1:] -= np.outer(e, hinv[i, i + 1:])
            wq[:, i] = q1[:, i - c0]
            hinv = hinv - np.outer(hinv[:, i], hinv[i, :]) / hinv[i, i]
            hinv[i, :] = 0
            hinv[:, i] = 0
            hinv[i, i] = 1                      # (keeps later divisions defined; column i is never read again)
    if actorder:
        wq = wq[:, np.argsort(perm, kind="stable")]
    return wq


def correlated_problem(seed, n, k, m=96):
    r = np.random.default_rng(seed)
    mix = r.standard_normal((k, k)) / np.sqrt(k) + np.eye(k)
    x = r.standard_normal((m, k)) @ mix
    w = r.standard_normal((n, k)) * 0.05
    return w, 2.0 / m * x.T @ x
