"""CPU baseline of the benchmark: the per-expert quantize -> dequantize -> fp32 matmul loop.

TEST / MEASUREMENT INFRASTRUCTURE ONLY.  This is the scheme of the reference's own test
oracle (fp8_gmm/test.py:209-214: for each expert ``matmul(a[start:end] * a_scale_inv,
b[i].t() * b_scale_inv)``) extended to the six GEMMs of an MLP step, written with
multi-threaded torch CPU ops so that it uses all host cores.  The fp8 round trip is
``clamp(+-max).to(float8).float()``, which the test-suite pins to the oracle's bytes.
"""
import time

import torch

_MAX = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}


def _qdq(x, dtype):
    """Per-tensor scaled fp8 round trip: returns (dequantised fp32 without the scale, scale_inv)."""
    xf = x.float()
    amax = xf.abs().max().clamp_min(1e-30)
    scale = _MAX[dtype] / amax
    q = (xf * scale).clamp(-_MAX[dtype], _MAX[dtype]).to(dtype)
    return q.float(), 1.0 / scale


def mlp_step_sample(tokens, hidden, ffn, seed=0):
    """One expert's MLP forward + backward (6 GEMMs) in the quantize-dequantize-fp32 scheme.

    Returns (seconds, flops).  flops = 6 * 2 * tokens * hidden * ffn.
    """
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(ffn, hidden, generator=g) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(hidden, ffn, generator=g) * 0.02).to(torch.bfloat16)
    dy = (torch.randn(tokens, hidden, generator=g) * 1e-2).to(torch.bfloat16)
    e4, e5 = torch.float8_e4m3fn, torch.float8_e5m2

    t0 = time.perf_counter()
    xq, xs = _qdq(x, e4)
    w1q, w1s = _qdq(w1, e4)
    w2q, w2s = _qdq(w2, e4)
    pre = (torch.matmul(xq, w1q.t()) * (xs * w1s)).to(torch.bfloat16)                      # fc1
    act = torch.nn.functional.gelu(pre.float(), approximate="tanh")
    aq, as_ = _qdq(act, e4)
    out = (torch.matmul(aq, w2q.t()) * (as_ * w2s)).to(torch.bfloat16)                     # fc2
    dq, ds = _qdq(dy, e5)
    dw2 = (torch.matmul(dq.t(), aq) * (ds * as_)).to(torch.bfloat16)                       # fc2 wgrad
    dact = (torch.matmul(dq, w2q) * (ds * w2s)).to(torch.bfloat16)                         # fc2 dgrad
    p = pre.float()
    t = torch.tanh(0.79788456 * p * (1 + 0.044715 * p * p))
    dgelu = 0.5 * p * ((1 - t * t) * (0.79788456 + 0.1070322243 * p * p)) + 0.5 * (1 + t)
    dpq, dps = _qdq(dact.float() * dgelu, e5)
    dx = (torch.matmul(dpq, w1q) * (dps * w1s)).to(torch.bfloat16)                         # fc1 dgrad
    dw1 = (torch.matmul(dpq.t(), xq) * (dps * xs)).to(torch.bfloat16)                      # fc1 wgrad
    dt = time.perf_counter() - t0
    assert out.shape == (tokens, hidden) and dx.shape == x.shape and dw1.shape == w1.shape and dw2.shape == w2.shape
    return dt, 6 * 2 * tokens * hidden * ffn


def mlp_step_grouped(sizes, hidden, ffn, seed=0):
    """The grouped step as the reference's test oracle walks it: a loop over the experts, each on its own row
    slice with its own weights (fp8_gmm/test.py:209-214), 6 GEMMs per expert.  Every expert quantises its weights
    inside the timed region, as the step casts them on every pass.  The weights' values are drawn once and shared
    (only their cost matters here).  Returns (seconds, flops) with flops = 6 * 2 * sum(sizes) * hidden * ffn."""
    g = torch.Generator().manual_seed(seed)
    tokens = int(sum(sizes))
    x = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(ffn, hidden, generator=g) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(hidden, ffn, generator=g) * 0.02).to(torch.bfloat16)
    dy = (torch.randn(tokens, hidden, generator=g) * 1e-2).to(torch.bfloat16)
    e4, e5 = torch.float8_e4m3fn, torch.float8_e5m2
    t0 = time.perf_counter()
    start = 0
    for rows in sizes:
        xs_, dys = x[start: start + rows], dy[start: start + rows]
        start += rows
        w1q, w1s = _qdq(w1, e4)
        w2q, w2s = _qdq(w2, e4)
        if rows == 0:
            continue
        xq, xs = _qdq(xs_, e4)
        pre = (torch.matmul(xq, w1q.t()) * (xs * w1s)).to(torch.bfloat16)
        act = torch.nn.functional.gelu(pre.float(), approximate="tanh")
        aq, as_ = _qdq(act, e4)
        out = (torch.matmul(aq, w2q.t()) * (as_ * w2s)).to(torch.bfloat16)
        dq, ds = _qdq(dys, e5)
        dw2 = (torch.matmul(dq.t(), aq) * (ds * as_)).to(torch.bfloat16)
        dact = (torch.matmul(dq, w2q) * (ds * w2s)).to(torch.bfloat16)
        p = pre.float()
        t = torch.tanh(0.79788456 * p * (1 + 0.044715 * p * p))
        dgelu = 0.5 * p * ((1 - t * t) * (0.79788456 + 0.1070322243 * p * p)) + 0.5 * (1 + t)
        dpq, dps = _qdq(dact.float() * dgelu, e5)
        dx = (torch.matmul(dpq, w1q) * (dps * w1s)).to(torch.bfloat16)
        dw1 = (torch.matmul(dpq.t(), xq) * (dps * xs)).to(torch.bfloat16)
        assert out.shape == (rows, hidden) and dx.shape == (rows, hidden) and dw1.shape == w1.shape and dw2.shape == w2.shape
    dt = time.perf_counter() - t0
    return dt, 6 * 2 * tokens * hidden * ffn
