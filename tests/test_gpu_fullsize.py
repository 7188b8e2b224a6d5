"""Parity at the full size of the benchmark workloads: the headline one (config 2: E = 8, 4096 -> 14336, 16384
tokens, ragged split) and the two the reference itself cannot run - config 3 (GroupedLinear, E = 64, 2048 -> 1408,
24576 tokens split by Zipf popularity: experts with no rows and with fewer than 16, amax history 16; the reference
asserts `0 not in group_sizes`, fp8_gmm/grouped_linear.py:205) and config 4 (GroupedMlp, E = 128, 2048 -> 768,
65536 tokens: 384 tensors in one cast launch where the reference stops at 64, csrc/multi_pad_fusion.cu:512).

The CPU oracle cannot finish these sizes in seconds, so the checks are properties that do not depend on size:
  * GEMMs on operands from {0, +-0.25 .. +-2}: every partial sum is exact in fp32, whatever the order, so the
    result must equal a plain fp32 matmul of the dequantised operands bit for bit (here torch's, on the GPU);
    this for the forward, data-gradient and weight-gradient shapes, on transposed copies and in place;
  * a sample of rows of each result against the CPU oracle;
  * cast + transpose: the transposed copy is the transpose of the row-major copy plus zero padding, the
    row-major copy equals what the quantize kernel writes, amax equals max|x|, sampled rows equal the oracle's
    bytes, and casting the dequantised bytes again returns the same bytes;
  * the whole module steps: sampled experts against the CPU oracle stage by stage (helpers.check_*_against_oracle),
    and the scaling state (scale, scale_inv, amax history) bit for bit against the oracle's update rule fed with
    max|x| of the tensors that were cast.
"""
import pytest
import torch

import numpy as np

from helpers import (assert_bytes_equal, assert_scalar_bits_equal, check_linear_expert_against_oracle,
                     check_mlp_expert_against_oracle, gen)
from oracle import modules as orc
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
    """Two training steps of the config-2 layer; the second (real scales) against the CPU oracle on two experts
    (the smallest and a ragged mid-sized one), stage by stage."""
    import fp8_gmm_amd as pkg

    e = len(SIZES)
    g = torch.Generator(device=dev).manual_seed(9)
    module = pkg.GroupedMlp(HIDDEN, FFN, e, torch.bfloat16, device=dev)
    module.fc1_weight.data.normal_(0, 0.02, generator=g)
    module.fc2_weight.data.normal_(0, 0.02, generator=g)
    x = torch.randn(sum(SIZES), HIDDEN, generator=g, device=dev).to(torch.bfloat16)
    dy = (torch.randn(sum(SIZES), HIDDEN, generator=g, device=dev) * 1e-2).to(torch.bfloat16)
    gs = torch.tensor(SIZES)
    captured = {}
    module.capture_intermediates(captured)
    for _ in range(2):
        xd = x.clone().requires_grad_()
        module.zero_grad()
        with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=2)):
            out = module(xd, gs)
        out.backward(dy)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(module.fc1_weight.grad.float()).all()
    for i in (6, 4):   # 669 and 909 rows: what the CPU oracle finishes in seconds at these feature counts
        check_mlp_expert_against_oracle(module, captured, i, SIZES, x, dy, out, xd.grad, 1e-2, "config 2")


def _bench_splits(kind, experts, tokens, seed):
    """The split bench.py draws for its workloads (its own function: same generator, same seed, and for the Zipf
    workload the same empty and tiny expert)."""
    import importlib.util
    import os

    spec = importlib.util.spec_from_file_location(
        "bench_for_splits", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    return bench.splits(kind, experts, tokens, seed)


def _slice_amax(t, bounds):
    """max|t[rows of expert i]| per expert, exactly (0 for an expert without rows)."""
    a = t.float().abs().amax(dim=1)
    out = torch.zeros(len(bounds) - 1)
    for i in range(len(bounds) - 1):
        if bounds[i + 1] > bounds[i]:
            out[i] = a[bounds[i]: bounds[i + 1]].max().item()
    return out


def test_config3_grouped_linear_seventeen_steps(dev):
    """Config 3 at its real size, 18 training steps with an amax history of 16: after every step scale, scale_inv
    and the whole amax history must equal, bit for bit, the oracle's delayed-scaling rule applied to max|x| of each
    tensor that was cast (the history wraps once); experts without rows leave their amax at zero, keep their
    scale and get a zero weight gradient; on the last step four experts - the largest, a mid-sized one, the
    smallest ones with rows - are checked against the CPU oracle."""
    import fp8_gmm_amd as pkg

    e, k, n, tokens, hist, steps = 64, 2048, 1408, 24576, 16, 18
    sizes = _bench_splits("zipf", e, tokens, 1003)
    assert sum(sizes) == tokens and len(sizes) == e
    # this workload is defined by having an expert without rows and one with fewer than 16
    assert sum(sizes) == tokens and 0 in sizes and any(0 < s < 16 for s in sizes)
    bounds = _bounds(sizes)
    g = torch.Generator(device=dev).manual_seed(1003)
    module = pkg.GroupedLinear(k, n, e, torch.bfloat16, device=dev)
    module.weight_tensor.data.normal_(0, 0.02, generator=g)
    fp8_recipe = pkg.DelayedScaling(amax_history_len=hist)
    fwd, bwd = orc.Meta(3 * e, hist), orc.Meta(2 * e, hist)
    w_amax = module.weight_tensor.detach().float().abs().amax(dim=(1, 2)).cpu()
    gs = torch.tensor(sizes)
    xs = [3 * i for i in range(e)]
    ws = [3 * i + 1 for i in range(e)]
    for step in range(steps):
        x = (torch.randn(tokens, k, generator=g, device=dev) * (1.0 + 0.25 * step)).to(torch.bfloat16)
        dy = (torch.randn(tokens, n, generator=g, device=dev) * 1e-2 / (1.0 + step)).to(torch.bfloat16)
        if step > 0:
            fwd.update(448.0)
            bwd.update(57344.0)
        fwd.amax_history[0][xs] = _slice_amax(x, bounds)
        fwd.amax_history[0][ws] = w_amax
        bwd.amax_history[0][[2 * i for i in range(e)]] = _slice_amax(dy, bounds)
        xd = x.clone().requires_grad_()
        module.weight_tensor.grad = None
        with pkg.fp8_autocast(fp8_recipe=fp8_recipe):
            out = module(xd, gs)
        out.backward(dy)
        gm = module.fp8_meta
        for name, got, want in (("fwd", gm["scaling_fwd"], fwd), ("bwd", gm["scaling_bwd"], bwd)):
            assert_scalar_bits_equal(got.scale, want.scale, f"step {step} {name} scale")
            assert_scalar_bits_equal(got.scale_inv, want.scale_inv, f"step {step} {name} scale_inv")
            assert_scalar_bits_equal(got.amax_history, want.amax_history, f"step {step} {name} amax history")
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    grad_w = module.weight_tensor.grad
    for i, s in enumerate(sizes):
        if s == 0:
            assert not grad_w[i].any(), f"expert {i} has no rows: its weight gradient must be zero"
            assert gm["scaling_fwd"].scale[3 * i].item() == 1.0    # never saw an amax: still the initial scale
    live = [i for i in np.argsort(sizes) if sizes[i] > 0]
    for i in (int(np.argmax(sizes)), int(live[len(live) // 2]), int(live[0]), int(live[1])):
        check_linear_expert_against_oracle(module, i, sizes, x, dy, out, xd.grad, 1e-2, "config 3")


@pytest.mark.parametrize("a_dtype,form", [(E4M3, "fwd"), (E5M2, "dgrad"), (E5M2, "wgrad")])
def test_config3_gemms_exact(dev, a_dtype, form):
    """The three GEMMs of config 3 (64 problems; N = 1408 is 5.5 tiles wide, rows from 0 to thousands per expert)
    on operands whose every partial sum is exact: bit-equal to the fp32 matmul."""
    backend = _backend()
    e, k, n = 64, 2048, 1408
    sizes = _bench_splits("zipf", e, 24576, 1003)
    sizes[3] += sizes[-1]
    sizes[-1] = 0
    bounds = _bounds(sizes)
    x = _exact_fp8((sum(sizes), k), E4M3, dev, 41)
    w = _exact_fp8((e, n, k), E4M3, dev, 42)
    dy = _exact_fp8((sum(sizes), n), E5M2, dev, 43)
    sa = torch.full((e,), 0.5, device=dev)
    sb = torch.full((e,), 0.25, device=dev)
    if form == "fwd":
        c = backend.fp8_gmm(x, w, torch.tensor(sizes), sa, sb)
        for i in range(e):
            rows = slice(bounds[i], bounds[i + 1])
            want = ((x[rows].float() @ w[i].float().t()) * 0.125).to(torch.bfloat16)
            assert torch.equal(c[rows].view(torch.int16), want.view(torch.int16)), f"expert {i} ({sizes[i]} rows)"
    elif form == "dgrad":
        c = backend.fp8_gmm(dy, w, torch.tensor(sizes), sa, sb, backward=True, b_transposed=True)
        for i in range(e):
            rows = slice(bounds[i], bounds[i + 1])
            want = ((dy[rows].float() @ w[i].float()) * 0.125).to(torch.bfloat16)
            assert torch.equal(c[rows].view(torch.int16), want.view(torch.int16)), f"expert {i} ({sizes[i]} rows)"
    else:
        dw = torch.full((e, n, k), float("nan"), dtype=torch.bfloat16, device=dev)
        backend.grouped_gemm(backend.TensorBatch.rows_of(dy, bounds), backend.TensorBatch.rows_of(x, bounds),
                             backend.TensorBatch.stack_of(dw), sa, sb, transposed=True)
        for i in range(e):
            rows = slice(bounds[i], bounds[i + 1])
            want = ((dy[rows].float().t() @ x[rows].float()) * 0.125).to(torch.bfloat16)
            assert torch.equal(dw[i].view(torch.int16), want.view(torch.int16)), f"expert {i} ({sizes[i]} rows)"


def test_config4_grouped_mlp_many_experts(dev):
    """Config 4 at its real size: 128 experts, 384 tensors in the forward cast launch, 128-problem tables in all
    six GEMMs.  Two steps; after the second, scales of the directly cast tensors bit-exact against the oracle's
    rule, and four experts (smallest, largest, first, last) against the CPU oracle stage by stage."""
    import fp8_gmm_amd as pkg

    e, h, f, tokens = 128, 2048, 768, 65536
    sizes = _bench_splits("uniform", e, tokens, 1004)
    bounds = _bounds(sizes)
    g = torch.Generator(device=dev).manual_seed(1004)
    module = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)
    module.fc1_weight.data.normal_(0, 0.02, generator=g)
    module.fc2_weight.data.normal_(0, 0.02, generator=g)
    x = torch.randn(tokens, h, generator=g, device=dev).to(torch.bfloat16)
    dy = (torch.randn(tokens, h, generator=g, device=dev) * 1e-2).to(torch.bfloat16)
    gs = torch.tensor(sizes)
    captured = {}
    module.capture_intermediates(captured)
    for _ in range(2):
        xd = x.clone().requires_grad_()
        module.zero_grad()
        with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=4)):
            out = module(xd, gs)
        out.backward(dy)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    # second step ran with scale = 448 / amax of the first: the rule, from max|x| of what was cast
    gm = module.fp8_meta
    want = orc.Meta(6 * e, 4)
    want.amax_history[0][[3 * i for i in range(e)]] = _slice_amax(x, bounds)
    want.amax_history[0][[3 * i + 1 for i in range(e)]] = module.fc1_weight.detach().float().abs().amax(dim=(1, 2)).cpu()
    want.amax_history[0][[3 * (e + i) + 1 for i in range(e)]] = \
        module.fc2_weight.detach().float().abs().amax(dim=(1, 2)).cpu()
    want.update(448.0)
    direct = [3 * i for i in range(e)] + [3 * i + 1 for i in range(e)] + [3 * (e + i) + 1 for i in range(e)]
    assert_scalar_bits_equal(gm["scaling_fwd"].scale[direct], want.scale[direct], "forward scales of cast tensors")
    want_b = orc.Meta(4 * e, 4)
    want_b.amax_history[0][[2 * i for i in range(e)]] = _slice_amax(dy, bounds)
    want_b.update(57344.0)
    g1 = [2 * i for i in range(e)]
    assert_scalar_bits_equal(gm["scaling_bwd"].scale[g1], want_b.scale[g1], "grad_out scales")
    for i in (int(np.argmin(sizes)), int(np.argmax(sizes)), 0, e - 1):
        check_mlp_expert_against_oracle(module, captured, i, sizes, x, dy, out, xd.grad, 1e-2, "config 4")


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
