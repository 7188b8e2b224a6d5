"""The reference's native module ``fp8_gmm_backend`` (csrc/ops.cu:9-16) as served by fp8_gmm_amd/compat: the six
pybind names, called the way the reference's own Python layer and tests call them (fp8_gmm/backend.py:9-22,78-82,
fp8_gmm/test.py:36-134,170-229), against the CPU oracle - bytes, padded layouts and amax bit-exact, GEMM
results within 1e-2."""
import importlib
import sys

import pytest
import torch

from helpers import (REFERENCE_SHAPES, assert_bytes_equal, assert_gemm_close, assert_scalar_bits_equal, gen,
                     randn_bf16, transpose_shapes)
from oracle import ref

pytestmark = pytest.mark.gpu

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2


@pytest.fixture(scope="module")
def shim():
    """Imported under its top-level name, as the reference's `import fp8_gmm_backend as backend` would find it."""
    import fp8_gmm_amd.compat

    sys.path.insert(0, fp8_gmm_amd.compat.__path__[0])
    try:
        mod = importlib.import_module("fp8_gmm_backend")
    finally:
        sys.path.pop(0)
    assert {"fp8_gmm", "multi_quantize", "multi_scale_mul", "multi_pad_transpose", "multi_pad_cast_transpose",
            "multi_pad_cast_transpose_dgelu"} <= set(dir(mod))
    return mod


def _inputs(g, std=1.0):
    return [randn_bf16(s, g, std) for s in REFERENCE_SHAPES]


def _scales(g, n):
    # the reference's tests draw the scales from randn: negative ones included (fp8_gmm/test.py:40)
    return [torch.randn(1, generator=g) for _ in range(n)]


@pytest.mark.parametrize("dtype", [E4M3, E5M2])
def test_multi_quantize(dev, shim, dtype):
    g = gen(11)
    xs, scales = _inputs(g), _scales(g, len(REFERENCE_SHAPES))
    want = [torch.empty(x.shape, dtype=dtype) for x in xs]
    want_amax = [torch.zeros(1) for _ in xs]
    ref.multi_quantize(xs, want, scales, want_amax)
    outs = [torch.empty(x.shape, dtype=dtype, device=dev) for x in xs]
    amaxes = [torch.zeros(1, device=dev) for _ in xs]
    shim.multi_quantize([x.to(dev) for x in xs], outs, [s.to(dev) for s in scales], amaxes)
    for i in range(len(xs)):
        assert_bytes_equal(outs[i], want[i], f"tensor {i}")
        assert_scalar_bits_equal(amaxes[i], want_amax[i], f"amax {i}")


@pytest.mark.parametrize("dtype", [E4M3, E5M2])
@pytest.mark.parametrize("padded", [False, True])
def test_multi_pad_transpose(dev, shim, dtype, padded):
    g = gen(12)
    xs = [ref.f32_to_fp8(randn_bf16(s, g).float(), dtype) for s in REFERENCE_SHAPES]
    t_shapes = transpose_shapes(REFERENCE_SHAPES, padded)
    want = [torch.empty(s, dtype=dtype) for s in t_shapes]
    ref.multi_transpose(xs, want)
    outs = [torch.full(s, 0x55, dtype=torch.uint8, device=dev).view(dtype) for s in t_shapes]
    shim.multi_pad_transpose([x.to(dev) for x in xs], outs)
    for i in range(len(xs)):
        assert_bytes_equal(outs[i], want[i], f"tensor {i}")


@pytest.mark.parametrize("dtype", [E4M3, E5M2])
@pytest.mark.parametrize("padded", [False, True])
@pytest.mark.parametrize("dgelu", [False, True])
def test_multi_pad_cast_transpose(dev, shim, dtype, padded, dgelu):
    g = gen(13)
    xs, scales = _inputs(g), _scales(g, len(REFERENCE_SHAPES))
    pres = _inputs(g, 2.0)
    t_shapes = transpose_shapes(REFERENCE_SHAPES, padded)
    want = [torch.empty(x.shape, dtype=dtype) for x in xs]
    want_t = [torch.empty(s, dtype=dtype) for s in t_shapes]
    want_amax = [torch.zeros(1) for _ in xs]
    outs = [torch.empty(x.shape, dtype=dtype, device=dev) for x in xs]
    outs_t = [torch.full(s, 0x55, dtype=torch.uint8, device=dev).view(dtype) for s in t_shapes]
    amaxes = [torch.zeros(1, device=dev) for _ in xs]
    d = lambda ts: [t.to(dev) for t in ts]   # noqa: E731
    if dgelu:
        ref.multi_cast_transpose_dgelu(xs, pres, want, want_t, scales, want_amax)
        shim.multi_pad_cast_transpose_dgelu(d(xs), d(pres), outs, outs_t, d(scales), amaxes)
    else:
        ref.multi_cast_transpose(xs, want, want_t, scales, want_amax)
        shim.multi_pad_cast_transpose(d(xs), outs, outs_t, d(scales), amaxes)
    for i in range(len(xs)):
        assert_bytes_equal(outs[i], want[i], f"tensor {i}")
        assert_bytes_equal(outs_t[i], want_t[i], f"transposed tensor {i}")
        assert_scalar_bits_equal(amaxes[i], want_amax[i], f"amax {i}")


@pytest.mark.parametrize("a_dtype", [E4M3, E5M2])
def test_fp8_gmm_then_scale_mul(dev, shim, a_dtype):
    """The reference's CUTLASS data flow (fp8_gmm/backend.py:78-82) on its own test case (fp8_gmm/test.py:170-229:
    groups [16, 32, 16], k = 32, n = 64): unscaled grouped GEMM to bf16, then the in-place product with the two
    scale_inv per group.  A second case adds a group without rows, which the extension cannot take."""
    for sizes, k, n in (([16, 32, 16], 32, 64), ([16, 0, 33, 16], 32, 64)):
        g = gen(14)
        e, m = len(sizes), sum(sizes)
        a = ref.f32_to_fp8(randn_bf16((m, k), g).float(), a_dtype)
        b = ref.f32_to_fp8(randn_bf16((e, n, k), g).float(), E4M3)
        sa = [torch.rand(1, generator=g) + 0.5 for _ in range(e)]
        sb = [torch.rand(1, generator=g) + 0.5 for _ in range(e)]
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        shim.fp8_gmm(a.to(dev), b.to(dev), c, torch.tensor(sizes, dtype=torch.int64))
        unscaled = ref.fp32_matmul_reference(a, b, sizes, [torch.ones(1)] * e, [torch.ones(1)] * e)
        assert_gemm_close(c, unscaled, 1e-2, "unscaled GEMM")
        bounds = [0]
        for s in sizes:
            bounds.append(bounds[-1] + s)
        slices = [c[bounds[i]: bounds[i + 1]] for i in range(e)]
        # the oracle's statement of the second step, on the GPU's own bf16 values: bit-exact
        want = [s.cpu().clone() for s in slices]
        ref.multi_scale_mul(want, sa, sb)
        shim.multi_scale_mul(slices, [t.to(dev) for t in sa], [t.to(dev) for t in sb])
        for i in range(e):
            assert torch.equal(slices[i].cpu().view(torch.int16), want[i].view(torch.int16)), f"group {i}"
        scaled = ref.fp32_matmul_reference(a, b, sizes, sa, sb)
        assert_gemm_close(c, scaled, 2e-2, "scaled result (two roundings)")


def test_fp8_gmm_argument_checks(dev, shim):
    a = torch.zeros(32, 32, dtype=E4M3, device=dev)
    b = torch.zeros(2, 64, 32, dtype=E4M3, device=dev)
    c = torch.zeros(32, 64, dtype=torch.bfloat16, device=dev)
    sizes = torch.tensor([16, 16], dtype=torch.int64)
    shim.fp8_gmm(a, b, c, sizes)
    with pytest.raises(RuntimeError):
        shim.fp8_gmm(a, b.view(E5M2), c, sizes)                      # b must be e4m3 (csrc/fp8_gmm.cu:179)
    with pytest.raises(RuntimeError):
        shim.fp8_gmm(a, b, c.float(), sizes)                         # c must be bf16
    with pytest.raises(RuntimeError):
        shim.fp8_gmm(a, b, c, sizes.to(torch.int32))                 # int64 batch sizes
    with pytest.raises(RuntimeError):
        shim.fp8_gmm(a, b, c, torch.tensor([16, 8], dtype=torch.int64))   # must sum to the rows of a
    with pytest.raises(RuntimeError):
        shim.fp8_gmm(a, b[:, :, :16], c, sizes)                      # contiguous, matching k
