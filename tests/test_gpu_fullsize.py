"""Parity at the full size of the headline workload (E = 8, 4096 -> 14336, 16384 tokens, ragged split).

The CPU oracle cannot finish these sizes in seconds, so the checks are properties that do not depend on size:
  * GEMMs on operands from {0, +-0.25 .. +-2}: every partial sum is exact in fp32, whatever the order, so the
    result must equal a plain fp32 matmul of the dequantised operands bit for bit (here torch's, on the GPU);
    this for the forward, data-gradient and weight-gradient shapes, on transposed copies and in place;
  * a sample of rows of each result against the CPU oracle;
  * cast + transpose: the transposed copy is the transpose of the row-major copy plus zero padding, the
    row-major copy equals what the quantize kernel writes, amax equals max|x|, sampled rows equal the oracle's
    bytes, and casting the dequantised bytes again returns the same bytes;
  * the whole GroupedMlp step against an fp32 autograd model of the same layer (cosine similarity).
"""
import pytest
import torch

from helpers import assert_bytes_equal, gen
from oracle import ref

pytestmark = pytest.mark.gpu

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2
SIZES = [1439, 3146, 3993, 1820, 909, 3499, 669, 909]   # bench.py's config-2 split
HIDDEN, FFN = 4096, 14336
VALS = torch.tensor([0.0, 0.5, -0.5, 1.0, -1.0, 2.0, -2.0, 0.25])


def _backend():
    from fp8_gmm_amd import backend

    return backend


def _exact_fp8(shape, dtype, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    idx = torch.randint(0, 8, shape, generator=g, device=dev)
    return VALS.to(dev)[idx].to(dtype)


def _bounds(sizes):
    b = [0]
    for s in sizes:
        b.append(b[-1] + s)
    return b


@pytest.mark.parametrize("a_dtype,k,n", [(E4M3, HIDDEN, FFN), (E4M3, FFN, HIDDEN), (E5M2, FFN, HIDDEN)])
def test_grouped_gemm_full_size_exact(dev, a_dtype, k, n):
    """fc1 forward, fc2 forward and fc1 dgrad shapes (3808 resp. 1088 tiles, the latter with tiles shared
    along K): bit-equal to the fp32 matmul, and a row sample equal to the oracle."""
    backend = _backend()
    m_total, e = sum(SIZES), len(SIZES)
    a = _exact_fp8((m_total, k), a_dtype, dev, 1)
    b = _exact_fp8((e, n, k), E4M3, dev, 2)
    sa = torch.full((e,), 0.5, device=dev)
    sb = torch.full((e,), 0.25, device=dev)
    c = backend.fp8_gmm(a, b, torch.tensor(SIZES), sa, sb, backward=(a_dtype == E5M2))
    bounds = _bounds(SIZES)
    for i in range(e):
        rows = slice(bounds[i], bounds[i + 1])
        want = ((a[rows].float() @ b[i].float().t()) * 0.125).to(torch.bfloat16)
        assert torch.equal(c[rows].view(torch.int16), want.view(torch.int16)), f"expert {i}"
    # a few rows per expert against the CPU oracle (first, last, one inside)
    a_cpu, b_cpu, c_cpu = a.cpu(), b.cpu(), c.cpu()
    for i in range(e):
        for r in (bounds[i], bounds[i] + SIZES[i] // 2, bounds[i + 1] - 1):
            want = torch.empty(1, n, dtype=torch.bfloat16)
            ref.cublas_fp8_gemm(a_cpu[r: r + 1], b_cpu[i], want, torch.tensor(0.5), torch.tensor(0.25))
            assert torch.equal(c_cpu[r: r + 1].view(torch.int16), want.view(torch.int16)), f"expert {i} row {r}"


def test_wgrad_full_size_exact(dev):
    """fc1 weight gradient: dW[i][F, H] = dY_i^T [F, Mpad_i] . X_i^T [H, Mpad_i]^T, contraction over each expert's
    padded token count (K differs per problem: 768 .. 4096)."""
    backend = _backend()
    pads = [(s + 127) // 128 * 128 for s in SIZES]
    g_t = [_exact_fp8((FFN, p), E5M2, dev, 10 + i) for i, p in enumerate(pads)]
    x_t = [_exact_fp8((HIDDEN, p), E4M3, dev, 30 + i) for i, p in enumerate(pads)]
    dw = torch.empty(len(SIZES), FFN, HIDDEN, dtype=torch.bfloat16, device=dev)
    ones = torch.ones(len(SIZES), device=dev)
    backend.grouped_gemm(g_t, x_t, list(dw.unbind(0)), ones, ones)
    for i in range(len(SIZES)):
        want = (g_t[i].float() @ x_t[i].float().t()).to(torch.bfloat16)
        assert torch.equal(dw[i].view(torch.int16), want.view(torch.int16)), f"expert {i}"


@pytest.mark.parametrize("dtype", [E4M3, E5M2])
def test_cast_transpose_full_size_properties(dev, dtype):
    backend = _backend()
    g = torch.Generator(device=dev).manual_seed(5)
    bounds = _bounds(SIZES)
    pads = [(s + 127) // 128 * 128 for s in SIZES]
    x = torch.randn(sum(SIZES), HIDDEN, generator=g, device=dev).to(torch.bfloat16)
    x[17, 33] = 200.0   # outliers: saturation and amax
    x[bounds[3] + 5, 4000] = -1000.0
    w = (torch.randn(2, FFN, HIDDEN, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    ins = [x[bounds[i]: bounds[i + 1]] for i in range(len(SIZES))] + list(w.unbind(0))
    scales = [torch.tensor([s], device=dev) for s in ([3.0, 0.5, 1.0, 7.25, 100.0, 1.0, 0.125, 2.0] + [3000.0, 1.0])]
    outs = [torch.empty(t.shape, dtype=dtype, device=dev) for t in ins]
    t_cols = pads + [FFN, FFN]
    touts = [torch.full((t.shape[1], c), 0x55, dtype=torch.uint8, device=dev).view(dtype) for t, c in zip(ins, t_cols)]
    amaxes = torch.zeros(len(ins), device=dev)
    backend.multi_cast_transpose(ins, outs, touts, scales, amaxes)
    q_outs = [torch.empty(t.shape, dtype=dtype, device=dev) for t in ins]
    q_amaxes = torch.zeros(len(ins), device=dev)
    backend.multi_quantize(ins, q_outs, scales, q_amaxes)
    for i, t in enumerate(ins):
        rows = t.shape[0]
        o8, t8 = outs[i].view(torch.uint8), touts[i].view(torch.uint8)
        assert torch.equal(t8[:, :rows], o8.t()), f"tensor {i}: transposed copy is not the transpose"
        assert int(t8[:, rows:].max().item() if t_cols[i] > rows else 0) == 0, f"tensor {i}: padding not zero"
        assert torch.equal(q_outs[i].view(torch.uint8), o8), f"tensor {i}: quantize and cast+transpose disagree"
        assert amaxes[i].item() == t.float().abs().max().item() == q_amaxes[i].item(), f"tensor {i}: amax"
        # sampled rows against the oracle's bytes
        for r in (0, rows // 3, rows - 1):
            want = ref.f32_to_fp8((t[r: r + 1].float().cpu() * scales[i].item()).contiguous(), dtype)
            assert_bytes_equal(outs[i][r: r + 1], want, f"tensor {i} row {r}")
    # round trip: fp8 -> bf16 is exact, so casting the dequantised values with scale 1 returns the same bytes
    deq = [o.to(torch.bfloat16) for o in outs[:3]]
    again = [torch.empty(o.shape, dtype=dtype, device=dev) for o in outs[:3]]
    backend.multi_quantize(deq, again, [torch.ones(1, device=dev)] * 3, torch.zeros(3, device=dev))
    for i in range(3):
        assert torch.equal(again[i].view(torch.uint8), outs[i].view(torch.uint8)), f"round trip {i}"


def test_grouped_mlp_full_size_step(dev):
    """Two training steps of the config-2 layer; the second (real scales) against an fp32 autograd model."""
    import fp8_gmm_amd as pkg

    e = len(SIZES)
    g = torch.Generator(device=dev).manual_seed(9)
    module = pkg.GroupedMlp(HIDDEN, FFN, e, torch.bfloat16, device=dev)
    x = torch.randn(sum(SIZES), HIDDEN, generator=g, device=dev).to(torch.bfloat16)
    dy = (torch.randn(sum(SIZES), HIDDEN, generator=g, device=dev) * 1e-2).to(torch.bfloat16)
    gs = torch.tensor(SIZES)
    for _ in range(2):
        xd = x.clone().requires_grad_()
        module.zero_grad()
        with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=2)):
            out = module(xd, gs)
        out.backward(dy)
    bounds = _bounds(SIZES)

    def cos(a, b):
        a, b = a.detach().float().flatten(), b.detach().float().flatten()
        return (torch.dot(a, b) / (a.norm() * b.norm())).item()

    # expert by expert, to bound the fp32 model's memory
    for i in range(e):
        rows = slice(bounds[i], bounds[i + 1])
        xr = x[rows].float().requires_grad_()
        w1 = module.fc1_weight.data[i].float().requires_grad_()
        w2 = module.fc2_weight.data[i].float().requires_grad_()
        ref_out = torch.nn.functional.gelu(xr @ w1.t(), approximate="tanh") @ w2.t()
        ref_out.backward(dy[rows].float())
        assert cos(out[rows], ref_out) > 0.995, f"expert {i} output"
        assert cos(xd.grad[rows], xr.grad) > 0.99, f"expert {i} grad_input"
        assert cos(module.fc1_weight.grad[i], w1.grad) > 0.99, f"expert {i} fc1 grad"
        assert cos(module.fc2_weight.grad[i], w2.grad) > 0.99, f"expert {i} fc2 grad"
    assert torch.isfinite(out.float()).all() and torch.isfinite(module.fc1_weight.grad.float()).all()


def test_cast_pad_bandwidth_configuration_full_size(dev):
    """Config 5 at its real size: 8 tensors [M_i, 4096], M_i in [1, 8191], pad to 128, +-200 outliers, e4m3 with
    scale 448 / amax.  Size-independent checks: transposed copy = transpose + zero padding, amax = max|x| (the
    outliers), nothing saturates wrongly (dequantised outliers are exactly +-448 / scale), sampled rows equal
    the oracle's bytes."""
    import numpy as np

    backend = _backend()
    rng = np.random.default_rng(1005)
    rows = [int(v) for v in rng.integers(1, 8192, size=8)] + [1, 127, 129]
    cols, pad = 4096, 128
    g = torch.Generator(device=dev).manual_seed(1005)
    ins, outs, touts, scales = [], [], [], []
    for m in rows:
        x = torch.randn(m, cols, generator=g, device=dev)
        hit = torch.rand(m, cols, generator=g, device=dev) < 1e-3
        x = torch.where(hit, torch.where(torch.rand(m, cols, generator=g, device=dev) < 0.5, -200.0, 200.0), x)
        x[0, 0] = 200.0
        ins.append(x.to(torch.bfloat16))
        outs.append(torch.full((m, cols), 0x55, dtype=torch.uint8, device=dev).view(E4M3))
        touts.append(torch.full((cols, (m + pad - 1) // pad * pad), 0x55, dtype=torch.uint8, device=dev).view(E4M3))
        scales.append((448.0 / ins[-1].float().abs().max()).reshape(1))
    amaxes = torch.zeros(len(rows), device=dev)
    backend.multi_cast_transpose(ins, outs, touts, scales, amaxes)
    for i, m in enumerate(rows):
        o8, t8 = outs[i].view(torch.uint8), touts[i].view(torch.uint8)
        assert torch.equal(t8[:, :m], o8.t()), f"tensor {i}"
        if t8.shape[1] > m:
            assert int(t8[:, m:].max()) == 0, f"tensor {i}: padding"
        assert amaxes[i].item() == 200.0
        assert outs[i][0, 0].float().item() == 448.0       # the outlier lands exactly on the largest finite value
        for r in (0, m // 2, m - 1):
            want = ref.f32_to_fp8((ins[i][r: r + 1].float().cpu() * scales[i].item()).contiguous(), E4M3)
            assert_bytes_equal(outs[i][r: r + 1], want, f"tensor {i} row {r}")


@pytest.mark.parametrize("k,n", [(FFN, HIDDEN), (HIDDEN, FFN)])
def test_dgrad_in_place_full_size_exact(dev, k, n):
    """Data-gradient shapes with the weight read in place (b[i] is [k, n]): bit-equal to the fp32 matmul."""
    backend = _backend()
    e = len(SIZES)
    a = _exact_fp8((sum(SIZES), k), E5M2, dev, 3)
    b = _exact_fp8((e, k, n), E4M3, dev, 4)
    sa = torch.full((e,), 0.5, device=dev)
    sb = torch.full((e,), 0.25, device=dev)
    c = backend.fp8_gmm(a, b, torch.tensor(SIZES), sa, sb, backward=True, b_transposed=True)
    bounds = _bounds(SIZES)
    for i in range(e):
        rows = slice(bounds[i], bounds[i + 1])
        want = ((a[rows].float() @ b[i].float()) * 0.125).to(torch.bfloat16)
        assert torch.equal(c[rows].view(torch.int16), want.view(torch.int16)), f"expert {i}"


def test_wgrad_in_place_full_size_exact(dev):
    """fc1 weight gradient on the row-major slices, dW[i] = dY_i^T . X_i, contraction over the expert's own
    (unpadded, ragged) row count: bit-equal to the fp32 matmul."""
    backend = _backend()
    e, bounds = len(SIZES), _bounds(SIZES)
    dy = _exact_fp8((sum(SIZES), FFN), E5M2, dev, 5)
    x = _exact_fp8((sum(SIZES), HIDDEN), E4M3, dev, 6)
    dw = torch.empty(e, FFN, HIDDEN, dtype=torch.bfloat16, device=dev)
    ones = torch.ones(e, device=dev)
    backend.grouped_gemm([dy[bounds[i]: bounds[i + 1]] for i in range(e)],
                         [x[bounds[i]: bounds[i + 1]] for i in range(e)], list(dw.unbind(0)), ones, ones,
                         transposed=True)
    for i in range(e):
        rows = slice(bounds[i], bounds[i + 1])
        want = (dy[rows].float().t() @ x[rows].float()).to(torch.bfloat16)
        assert torch.equal(dw[i].view(torch.int16), want.view(torch.int16)), f"expert {i}"
