"""Writes tests/golden/golden_small.npz: seeded inputs and the oracle's outputs for every entry point.

The reference holds no golden vectors, test fixtures or known-answer files of its own (its tests use
unseeded random tensors), so these fixtures come from the CPU oracle after it has been pinned against
PyTorch, closed forms and hand-computed bytes (tests/test_oracle_pins.py).  They freeze that state:
the oracle (CPU) and the HIP kernels (GPU) are both checked against the same committed bytes.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ref  # noqa: E402

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2
SHAPES = [(137, 72), (59, 40), (16, 128), (1, 33), (45, 1)]
PAD = 16


def u8(t):
    return t.contiguous().view(torch.uint8).numpy().copy()


def u16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def main():
    g = torch.Generator().manual_seed(20240601)
    out = {}
    for idx, (m, n) in enumerate(SHAPES):
        mp = (m + PAD - 1) // PAD * PAD
        x = torch.randn(m, n, generator=g).to(torch.bfloat16)
        pre = (torch.randn(m, n, generator=g) * 2).to(torch.bfloat16)
        if idx == 0:  # a few outliers and specials
            x[0, 0], x[1, 1], x[2, 2], x[3, 3] = 200.0, -200.0, float("inf"), float("nan")
        scale = torch.tensor([[3.25, 0.017, 448.0 / 4.1, -1.5, 1.0][idx]], dtype=torch.float32)
        out[f"x{idx}"], out[f"pre{idx}"], out[f"scale{idx}"] = u16(x), u16(pre), scale.numpy()
        for tag, dt in (("e4m3", E4M3), ("e5m2", E5M2)):
            q, a = torch.empty(m, n, dtype=dt), torch.zeros(1)
            ref.multi_quantize([x], [q], [scale], [a])
            out[f"quant_{tag}_{idx}"], out[f"quant_amax_{tag}_{idx}"] = u8(q), a.numpy()
            o, t, a = torch.empty(m, n, dtype=dt), torch.empty(n, mp, dtype=dt), torch.zeros(1)
            ref.multi_cast_transpose([x], [o], [t], [scale], [a])
            out[f"ct_out_{tag}_{idx}"], out[f"ct_t_{tag}_{idx}"], out[f"ct_amax_{tag}_{idx}"] = u8(o), u8(t), a.numpy()
            t2 = torch.empty(n, mp, dtype=dt)
            ref.multi_transpose([o], [t2])
            out[f"tr_t_{tag}_{idx}"] = u8(t2)
            o, t, a = torch.empty(m, n, dtype=dt), torch.empty(n, mp, dtype=dt), torch.zeros(1)
            ref.multi_cast_transpose_dgelu([x.nan_to_num(0.0, 0.0, 0.0)], [pre], [o], [t], [scale], [a])
            out[f"dg_out_{tag}_{idx}"], out[f"dg_t_{tag}_{idx}"], out[f"dg_amax_{tag}_{idx}"] = u8(o), u8(t), a.numpy()
    # grouped GEMM at the tiny configuration: E=4, K=256, N=512 is too big for a fixture; use K=64, N=48
    sizes = [37, 0, 21, 6]
    e, k, n = len(sizes), 64, 48
    a = ref.f32_to_fp8(torch.randn(sum(sizes), k, generator=g), E4M3)
    a5 = ref.f32_to_fp8(torch.randn(sum(sizes), k, generator=g) * 0.01 * 4096, E5M2)
    b = ref.f32_to_fp8(torch.randn(e, n, k, generator=g), E4M3)
    sa = [torch.tensor(0.5 + 0.25 * i) for i in range(e)]
    sb = [torch.tensor(0.03 * (i + 1)) for i in range(e)]
    c = torch.zeros(sum(sizes), n, dtype=torch.bfloat16)
    ref.fp8_gmm(a, b, sizes, sa, sb, c, naive=True)
    c5 = torch.zeros(sum(sizes), n, dtype=torch.bfloat16)
    ref.fp8_gmm(a5, b, sizes, sa, sb, c5, naive=True)
    cs = [torch.tensor([2.0 + i]) for i in range(e)]
    am = [torch.zeros(1) for _ in range(e)]
    cg, pre = torch.zeros(sum(sizes), n, dtype=E4M3), torch.zeros(sum(sizes), n, dtype=torch.bfloat16)
    ref.fp8_gmm(a, b, sizes, sa, sb, cg, E4M3, pre, cs, am, naive=True)
    out.update(gemm_sizes=np.array(sizes), gemm_a=u8(a), gemm_a5=u8(a5), gemm_b=u8(b),
               gemm_sa=np.array([float(s) for s in sa], dtype=np.float32),
               gemm_sb=np.array([float(s) for s in sb], dtype=np.float32), gemm_c=u16(c), gemm_c5=u16(c5),
               gemm_cs=np.array([float(s) for s in cs], dtype=np.float32), gemm_gelu_c=u8(cg), gemm_gelu_pre=u16(pre),
               gemm_gelu_amax=np.array([float(x) for x in am], dtype=np.float32))
    path = os.path.join(HERE, "golden_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
