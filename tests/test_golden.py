"""Committed golden fixtures (tests/golden/golden_small.npz, written by tests/golden/make_golden.py).

CPU:  the oracle still reproduces the committed bytes (guards the oracle against silent edits).
GPU:  the HIP entry points reproduce the same committed bytes - fp8 bytes, padded layouts and amax
      bit for bit; GEMM outputs within 1e-2 of the committed result.
"""
import os

import numpy as np
import pytest
import torch

from helpers import assert_bytes_equal, assert_gemm_close, assert_scalar_bits_equal
from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))
G = np.load(os.path.join(HERE, "golden", "golden_small.npz"))
SHAPES = [(137, 72), (59, 40), (16, 128), (1, 33), (45, 1)]
E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2
DTYPES = [("e4m3", E4M3), ("e5m2", E5M2)]


def bf16(name, shape):
    return torch.from_numpy(G[name].view(np.int16).copy()).view(torch.bfloat16).reshape(shape)


def fp8(name, dtype, shape=None):
    t = torch.from_numpy(G[name].copy()).view(dtype)
    return t.reshape(shape) if shape is not None else t


def f32(name):
    return torch.from_numpy(G[name].copy())


def _run_pointwise(backend, to_dev):
    """Runs the four multi-tensor entry points over all fixture tensors in ONE call each per dtype."""
    results = {}
    for tag, dt in DTYPES:
        xs = [to_dev(bf16(f"x{i}", s)) for i, s in enumerate(SHAPES)]
        pres = [to_dev(bf16(f"pre{i}", s)) for i, s in enumerate(SHAPES)]
        scales = [to_dev(f32(f"scale{i}")) for i in range(len(SHAPES))]
        tshapes = [(n, (m + 15) // 16 * 16) for m, n in SHAPES]
        dev = xs[0].device
        q = [torch.empty(s, dtype=dt, device=dev) for s in SHAPES]
        qa = [torch.zeros(1, device=dev) for _ in SHAPES]
        backend.multi_quantize(xs, q, scales, qa)
        o = [torch.empty(s, dtype=dt, device=dev) for s in SHAPES]
        t = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dt) for ts in tshapes]
        ca = [torch.zeros(1, device=dev) for _ in SHAPES]
        backend.multi_cast_transpose(xs, o, t, scales, ca)
        t2 = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dt) for ts in tshapes]
        backend.multi_transpose(o, t2)
        xs0 = [x.nan_to_num(0.0, 0.0, 0.0) for x in xs]
        do = [torch.empty(s, dtype=dt, device=dev) for s in SHAPES]
        dt_ = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dt) for ts in tshapes]
        da = [torch.zeros(1, device=dev) for _ in SHAPES]
        backend.multi_cast_transpose_dgelu(xs0, pres, do, dt_, scales, da)
        results[tag] = dict(q=q, qa=qa, o=o, t=t, ca=ca, t2=t2, do=do, dt=dt_, da=da)
    return results


def _check_pointwise(results):
    for tag, _ in DTYPES:
        r = results[tag]
        for i in range(len(SHAPES)):
            for key, name in (("q", "quant"), ("o", "ct_out"), ("t", "ct_t"), ("t2", "tr_t"), ("do", "dg_out"),
                              ("dt", "dg_t")):
                golden = torch.from_numpy(G[f"{name}_{tag}_{i}"].copy())
                assert_bytes_equal(r[key][i], golden.reshape(r[key][i].shape), f"{name}_{tag}_{i}")
            for key, name in (("qa", "quant_amax"), ("ca", "ct_amax"), ("da", "dg_amax")):
                assert_scalar_bits_equal(r[key][i], f32(f"{name}_{tag}_{i}"), f"{name}_{tag}_{i}")


def test_oracle_reproduces_golden_pointwise():
    _check_pointwise(_run_pointwise(ref, lambda t: t))


def test_oracle_reproduces_golden_gemm():
    sizes = G["gemm_sizes"].tolist()
    m, k, n, e = sum(sizes), 64, 48, len(sizes)
    a, a5, b = fp8("gemm_a", E4M3, (m, k)), fp8("gemm_a5", E5M2, (m, k)), fp8("gemm_b", E4M3, (e, n, k))
    sa, sb = list(f32("gemm_sa")), list(f32("gemm_sb"))
    c = torch.zeros(m, n, dtype=torch.bfloat16)
    ref.fp8_gmm(a, b, sizes, sa, sb, c, naive=True)
    assert torch.equal(c.view(torch.int16), bf16("gemm_c", (m, n)).view(torch.int16))
    c5 = torch.zeros(m, n, dtype=torch.bfloat16)
    ref.fp8_gmm(a5, b, sizes, sa, sb, c5, naive=True)
    assert torch.equal(c5.view(torch.int16), bf16("gemm_c5", (m, n)).view(torch.int16))


@pytest.mark.gpu
def test_hip_reproduces_golden_pointwise(dev):
    from fp8_gmm_amd import backend

    _check_pointwise(_run_pointwise(backend, lambda t: t.to(dev)))


@pytest.mark.gpu
def test_hip_reproduces_golden_gemm(dev):
    from fp8_gmm_amd import backend

    sizes = G["gemm_sizes"].tolist()
    m, k, n, e = sum(sizes), 64, 48, len(sizes)
    a, a5, b = fp8("gemm_a", E4M3, (m, k)), fp8("gemm_a5", E5M2, (m, k)), fp8("gemm_b", E4M3, (e, n, k))
    sa, sb, cs = f32("gemm_sa").to(dev), f32("gemm_sb").to(dev), f32("gemm_cs").to(dev)
    gs = torch.tensor(sizes)
    c = backend.fp8_gmm(a.to(dev), b.to(dev), gs, sa, sb)
    assert_gemm_close(c, bf16("gemm_c", (m, n)).float(), 1e-2, "fwd")
    c5 = backend.fp8_gmm(a5.to(dev), b.to(dev), gs, sa, sb, backward=True)
    assert_gemm_close(c5, bf16("gemm_c5", (m, n)).float(), 1e-2, "bwd e5m2")
    cg = torch.empty(m, n, dtype=E4M3, device=dev)
    pre = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    am = torch.zeros(e, device=dev)
    backend.fp8_gmm(a.to(dev), b.to(dev), gs, sa, sb, cg, E4M3, pre, cs, am)
    assert_gemm_close(pre, bf16("gemm_gelu_pre", (m, n)).float(), 1e-2, "pre_gelu")
    gold = fp8("gemm_gelu_c", E4M3, (m, n))
    ia, ib = cg.cpu().view(torch.uint8).to(torch.int32), gold.view(torch.uint8).to(torch.int32)
    assert ((ia & 0x7F) - (ib & 0x7F)).abs().max() <= 1, "fp8 GELU output more than one code step from the fixture"
    assert torch.allclose(am.cpu(), f32("gemm_gelu_amax"), rtol=1e-4, atol=0)   # accumulation order, hardware exp2 / rcp
