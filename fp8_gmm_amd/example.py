"""The reference's benchmark recipe as a runnable module: ``python -m fp8_gmm_amd.example``.

One routed MoE layer, forward + backward, timed for four kinds of experts on the same sizes and the same procedure as
the reference's script (fp8_gmm/example.py:134-204: 16384 tokens, hidden 4096, inner 6400, 16 experts, top-2; 4
warm-up and 16 timed steps with fresh random inputs, wall clock between two device synchronisations):

* ``bf16``: the layer without FP8 (the reference's ``Bf16Module``, example.py:35-69, whose experts run on
  megablocks' bf16 grouped GEMM).  Here the experts are one vendor bf16 GEMM per expert on its row slice, the
  routing operators the same as for the other three;
* ``fp8-linear``: two ``GroupedLinear`` with a GELU between them, ``cutlass=False``;
* ``fp8-linear-cutlass``: the same with ``cutlass=True`` (the reference's CUTLASS data flow: an unscaled grouped GEMM
  followed by ``multi_scale_mul``);
* ``fp8-mlp``: one ``GroupedMlp``.

Prints one line per kind, as the reference's script does.
"""
import argparse
import math
import time

import numpy as np
import torch

from .fp8 import DelayedScaling, Format, fp8_autocast
from .moe import Fp8LinearModule, Fp8MlpModule, _RoutedModule


class _SlicedLinear(torch.autograd.Function):
    """``y[rows of expert i] = x[rows of expert i] @ w[i]^T`` with one bf16 GEMM per expert, and its two gradients."""

    @staticmethod
    def forward(ctx, x, w, sizes):
        ctx.save_for_backward(x, w)
        ctx.sizes = sizes
        y = torch.empty(x.shape[0], w.shape[1], dtype=x.dtype, device=x.device)
        row = 0
        for i, m in enumerate(sizes):
            if m:
                torch.matmul(x[row: row + m], w[i].t(), out=y[row: row + m])
            row += m
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dy = dy.contiguous()
        dx = torch.empty_like(x)
        dw = torch.zeros_like(w)
        row = 0
        for i, m in enumerate(ctx.sizes):
            if m:
                torch.matmul(dy[row: row + m], w[i], out=dx[row: row + m])
                torch.matmul(dy[row: row + m].t(), x[row: row + m], out=dw[i])
            row += m
        return dx, dw, None


class Bf16Module(_RoutedModule):
    """The routed layer in bf16: experts ``gelu(x w1^T) w2^T`` with weights ``[E, inner, hidden]`` and
    ``[E, hidden, inner]``, initialised like the reference's (uniform in +-1/sqrt(fan-in), example.py:44-47)."""

    def __init__(self, n_embd, n_inner, n_experts, top_k, dtype=torch.bfloat16, device="cuda"):
        super().__init__(n_embd, n_inner, n_experts, top_k, dtype, device)
        w1 = torch.empty(n_experts, n_inner, n_embd, dtype=dtype, device=device)
        w2 = torch.empty(n_experts, n_embd, n_inner, dtype=dtype, device=device)
        torch.nn.init.uniform_(w1, -math.sqrt(1.0 / n_embd), math.sqrt(1.0 / n_embd))
        torch.nn.init.uniform_(w2, -math.sqrt(1.0 / n_inner), math.sqrt(1.0 / n_inner))
        self.w1, self.w2 = torch.nn.Parameter(w1), torch.nn.Parameter(w2)
        self.act = torch.nn.GELU()

    def experts(self, x, batch_sizes):
        sizes = [int(v) for v in batch_sizes.tolist()]
        return _SlicedLinear.apply(self.act(_SlicedLinear.apply(x, self.w1, sizes)), self.w2, sizes)


KINDS = {
    "bf16": ("Bf16Module", lambda a: Bf16Module(a.hidden, a.inner, a.experts, a.top_k)),
    "fp8-linear": ("Fp8LinearModule", lambda a: Fp8LinearModule(a.hidden, a.inner, a.experts, a.top_k, cutlass=False)),
    "fp8-linear-cutlass": ("Fp8LinearModule cutlass", lambda a: Fp8LinearModule(a.hidden, a.inner, a.experts, a.top_k,
                                                                                cutlass=True)),
    "fp8-mlp": ("Fp8MlpModule", lambda a: Fp8MlpModule(a.hidden, a.inner, a.experts, a.top_k)),
}


def run(kind, args):
    """Milliseconds per forward + backward step of one kind of layer."""
    model = KINDS[kind][1](args)
    fp8_recipe = DelayedScaling(margin=0, interval=1, fp8_format=Format.HYBRID)
    dtype = torch.bfloat16

    def step():
        x = torch.randn(args.tokens, args.hidden, dtype=dtype, device="cuda", requires_grad=True)
        with fp8_autocast(enabled=kind != "bf16", fp8_recipe=fp8_recipe):
            out = model(x)
        out.backward(torch.randn(*out.size(), dtype=dtype, device="cuda"))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - start) * 1e3 / args.steps
    del model
    torch.cuda.empty_cache()
    return ms


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--tokens", type=int, default=16384)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--inner", type=int, default=6400)
    ap.add_argument("--experts", type=int, default=16)
    ap.add_argument("--top-k", type=int, default=2, dest="top_k")
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--steps", type=int, default=16)
    ap.add_argument("--kinds", nargs="*", default=list(KINDS), choices=list(KINDS))
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("fp8_gmm_amd.example: needs a GPU")
    torch.manual_seed(0)
    np.random.seed(0)
    times = {}
    for kind in args.kinds:
        times[kind] = run(kind, args)
        print(f"{KINDS[kind][0]} run: {times[kind]:.3f} ms", flush=True)
    return times


if __name__ == "__main__":
    main()
