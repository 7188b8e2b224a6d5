"""GroupedLinear / GroupedMlp forward + backward on the GPU against the CPU oracle's restatement.

The reference has no module-level test at all (its test file stops at the backend entry
points); these tests run the autograd modules for several steps of delayed scaling and
compare outputs, gradients and the recorded scaling state.
"""
import pytest
import torch

from helpers import (assert_close_multistage, assert_gemm_close, assert_scalar_bits_equal,
                     check_mlp_expert_against_oracle, gen, randn_bf16)
from oracle import modules as orc

pytestmark = pytest.mark.gpu


def _pkg():
    import fp8_gmm_amd

    return fp8_gmm_amd


def _sync_meta(oracle_meta, gpu_meta):
    oracle_meta.scale = gpu_meta.scale.detach().cpu().clone()
    oracle_meta.scale_inv = gpu_meta.scale_inv.detach().cpu().clone()
    oracle_meta.amax_history = gpu_meta.amax_history.detach().cpu().clone()


def _check_amax(gpu_meta, oracle_meta, exact_slots, approx_slots, what):
    g = gpu_meta.amax_history[0].detach().cpu()
    o = oracle_meta.amax_history[0]
    if exact_slots:
        assert_scalar_bits_equal(g[exact_slots], o[exact_slots], f"{what} amax (cast of given tensors)")
    if approx_slots:
        assert torch.allclose(g[approx_slots], o[approx_slots], rtol=2e-2, atol=0), f"{what} amax (derived tensors)"


LINEAR_CASES = {
    "config1": ([137, 401, 59, 403], 256, 512),
    "zero-rows": ([0, 48, 0, 5, 130], 128, 192),
    "aligned": ([32, 64, 16], 64, 128),
}


@pytest.mark.parametrize("case", list(LINEAR_CASES))
@pytest.mark.parametrize("cutlass", [False, True])
def test_grouped_linear_fwd_bwd(dev, case, cutlass):
    pkg = _pkg()
    sizes, k, n = LINEAR_CASES[case]
    e, m, hist = len(sizes), sum(sizes), 4
    g = gen(1001)
    w = randn_bf16((e, n, k), g, 0.02)
    module = pkg.GroupedLinear(k, n, e, torch.bfloat16, device=dev, cutlass=cutlass)
    module.weight_tensor.data.copy_(w)
    fp8_recipe = pkg.DelayedScaling(amax_history_len=hist)
    fwd, bwd = orc.Meta(3 * e, hist), orc.Meta(2 * e, hist)
    tol = 2e-2 if cutlass else 1e-2  # the two-rounding path rounds the bf16 result twice
    for step in range(3):
        x = randn_bf16((m, k), g)
        dy = randn_bf16((m, n), g, 1e-2)
        if step > 0:
            fwd.update(448.0)
            bwd.update(57344.0)
        o = orc.grouped_linear_step(x, w, sizes, dy, fwd, bwd)
        xd = x.to(dev).requires_grad_()
        module.weight_tensor.grad = None
        with pkg.fp8_autocast(enabled=True, fp8_recipe=fp8_recipe):
            out = module(xd, torch.tensor(sizes, dtype=torch.int64))
        out.backward(dy.to(dev))
        torch.cuda.synchronize()
        gm = module.fp8_meta
        assert_scalar_bits_equal(gm["scaling_fwd"].scale, fwd.scale, f"step {step} fwd scale")
        assert_scalar_bits_equal(gm["scaling_bwd"].scale, bwd.scale, f"step {step} bwd scale")
        assert_scalar_bits_equal(gm["scaling_fwd"].amax_history, fwd.amax_history, f"step {step} fwd amax history")
        assert_scalar_bits_equal(gm["scaling_bwd"].amax_history, bwd.amax_history, f"step {step} bwd amax history")
        assert_gemm_close(out, o["out"].float(), tol, f"step {step} out")
        assert_gemm_close(xd.grad, o["grad_input"].float(), tol, f"step {step} grad_input")
        assert_gemm_close(module.weight_tensor.grad, o["grad_weight"].float(), tol, f"step {step} grad_weight")
        for i, s in enumerate(sizes):
            if s == 0:
                assert not module.weight_tensor.grad[i].any(), "an expert without tokens has a zero weight gradient"


def test_grouped_linear_inference_and_frozen_weight(dev):
    """no_grad forward (cast-only path, multi_quantize) and a frozen weight (no wgrad, no padding)."""
    pkg = _pkg()
    sizes, k, n = [137, 401, 59, 403], 256, 512
    e, m = len(sizes), sum(sizes)
    g = gen(1002)
    w = randn_bf16((e, n, k), g, 0.02)
    x = randn_bf16((m, k), g)
    dy = randn_bf16((m, n), g, 1e-2)
    fwd, bwd = orc.Meta(3 * e, 1), orc.Meta(2 * e, 1)
    o = orc.grouped_linear_step(x, w, sizes, dy, fwd, bwd)
    module = pkg.GroupedLinear(k, n, e, torch.bfloat16, device=dev)
    module.weight_tensor.data.copy_(w)
    gs = torch.tensor(sizes)
    with torch.no_grad(), pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=1)):
        out = module(x.to(dev), gs)
    assert_gemm_close(out, o["out"].float(), 1e-2, "no_grad out")
    module.weight_tensor.requires_grad_(False)
    xd = x.to(dev).requires_grad_()
    with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=1)):
        out = module(xd, gs)
    out.backward(dy.to(dev))
    assert module.weight_tensor.grad is None
    # a no_grad pass does not count as a training step, so this first training pass still runs with
    # the initial scales: same oracle result
    assert_gemm_close(out, o["out"].float(), 1e-2, "frozen-weight out")
    assert_gemm_close(xd.grad, o["grad_input"].float(), 1e-2, "frozen-weight grad_input")
    assert_scalar_bits_equal(module.fp8_meta["scaling_fwd"].amax_history[0], fwd.amax_history[0], "fwd amax")


MLP_CASES = {
    "small": ([137, 401, 59, 403], 256, 512),
    "zero-rows": ([0, 48, 0, 5, 130], 128, 384),
}


@pytest.mark.parametrize("case", list(MLP_CASES))
def test_grouped_mlp_fwd_bwd(dev, case):
    pkg = _pkg()
    sizes, h, f = MLP_CASES[case]
    e, m, hist = len(sizes), sum(sizes), 3
    g = gen(2001)
    w1 = randn_bf16((e, f, h), g, 0.02)
    w2 = randn_bf16((e, h, f), g, 0.02)
    module = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)
    module.fc1_weight.data.copy_(w1)
    module.fc2_weight.data.copy_(w2)
    fp8_recipe = pkg.DelayedScaling(amax_history_len=hist)
    fwd, bwd = orc.Meta(3 * 2 * e, hist), orc.Meta(2 * 2 * e, hist)
    live = [i for i, s in enumerate(sizes) if s > 0]
    exact_fwd = [3 * i for i in live] + [3 * i + 1 for i in range(e)] + [3 * (e + i) + 1 for i in range(e)]
    approx_fwd = [3 * (e + i) for i in live]
    exact_bwd = [2 * i for i in live]
    approx_bwd = [2 * (e + i) for i in live]
    for step in range(3):
        x = randn_bf16((m, h), g)
        dy = randn_bf16((m, h), g, 1e-2)
        if step > 0:
            # derived amaxes (GELU output, dGELU product) depend on the accumulation order: take the
            # GPU's state so that both sides quantise with identical scales, then update both
            _sync_meta(fwd, module.fp8_meta["scaling_fwd"])
            _sync_meta(bwd, module.fp8_meta["scaling_bwd"])
            fwd.update(448.0)
            bwd.update(57344.0)
        o = orc.grouped_mlp_step(x, w1, w2, sizes, dy, fwd, bwd)
        xd = x.to(dev).requires_grad_()
        module.fc1_weight.grad = None
        module.fc2_weight.grad = None
        captured = {}
        module.capture_intermediates(captured)
        with pkg.fp8_autocast(enabled=True, fp8_recipe=fp8_recipe):
            out = module(xd, torch.tensor(sizes, dtype=torch.int64))
        out.backward(dy.to(dev))
        torch.cuda.synchronize()
        module.capture_intermediates(None)
        # stage by stage, with the oracle fed the GPU's own fp8 intermediates: every GEMM within 1e-2, the
        # directly cast bytes and amaxes bit-exact (the end-to-end comparison further down is the loose one)
        for i, rows in enumerate(sizes):
            if rows:
                check_mlp_expert_against_oracle(module, captured, i, sizes, x, dy, out, xd.grad, 1e-2, f"step {step}")
        gm = module.fp8_meta
        assert_scalar_bits_equal(gm["scaling_fwd"].scale, fwd.scale, f"step {step} fwd scale")
        assert_scalar_bits_equal(gm["scaling_bwd"].scale, bwd.scale, f"step {step} bwd scale")
        _check_amax(gm["scaling_fwd"], fwd, exact_fwd, approx_fwd, f"step {step} fwd")
        _check_amax(gm["scaling_bwd"], bwd, exact_bwd, approx_bwd, f"step {step} bwd")
        assert_close_multistage(out, o["out"], 5e-3, f"step {step} out")
        assert_close_multistage(module.fc2_weight.grad, o["grad_w2"], 5e-3, f"step {step} grad_fc2")
        assert_close_multistage(xd.grad, o["grad_input"], 1e-2, f"step {step} grad_input")
        assert_close_multistage(module.fc1_weight.grad, o["grad_w1"], 1e-2, f"step {step} grad_fc1")
        for i, s in enumerate(sizes):
            if s == 0:
                assert not module.fc1_weight.grad[i].any() and not module.fc2_weight.grad[i].any()


def test_grouped_mlp_matches_bf16_autograd(dev):
    """End-to-end sanity against plain torch autograd in fp32 (not the parity oracle): FP8 training
    noise is a few percent, so outputs and gradients must correlate strongly with the fp32 model."""
    pkg = _pkg()
    sizes, h, f = [200, 333, 91], 256, 512
    e, m = len(sizes), sum(sizes)
    g = gen(2002)
    w1 = randn_bf16((e, f, h), g, 0.05)
    w2 = randn_bf16((e, h, f), g, 0.05)
    x = randn_bf16((m, h), g)
    dy = randn_bf16((m, h), g, 1e-2)
    module = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)
    module.fc1_weight.data.copy_(w1)
    module.fc2_weight.data.copy_(w2)
    gs = torch.tensor(sizes)
    for _ in range(2):  # second pass runs with real scales
        xd = x.to(dev).requires_grad_()
        module.zero_grad()
        with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=2)):
            out = module(xd, gs)
        out.backward(dy.to(dev))
    xr = x.float().requires_grad_()
    w1r, w2r = w1.float().requires_grad_(), w2.float().requires_grad_()
    outs, start = [], 0
    for i, s in enumerate(sizes):
        hdn = torch.nn.functional.gelu(xr[start: start + s] @ w1r[i].t(), approximate="tanh")
        outs.append(hdn @ w2r[i].t())
        start += s
    ref_out = torch.cat(outs)
    ref_out.backward(dy.float())

    def cos(a, b):
        a, b = a.detach().float().cpu().flatten(), b.detach().float().flatten()
        return torch.dot(a, b) / (a.norm() * b.norm())

    assert cos(out, ref_out) > 0.995
    assert cos(xd.grad, xr.grad) > 0.99
    assert cos(module.fc1_weight.grad, w1r.grad) > 0.99
    assert cos(module.fc2_weight.grad, w2r.grad) > 0.99


@pytest.mark.parametrize("kind", ["linear", "mlp"])
def test_pad_multiple_does_not_change_results(dev, kind):
    """Padding of the transposed wgrad operands only appends zeros along the contraction: the reference's
    multiple (16) and the default here (128) must give bit-identical outputs and gradients."""
    pkg = _pkg()
    sizes, h, f = [137, 401, 0, 59, 403], 256, 512
    e, m = len(sizes), sum(sizes)
    g = gen(3001)
    x = randn_bf16((m, h), g).to(dev)
    dy = randn_bf16((m, f if kind == "linear" else h), g, 1e-2).to(dev)
    w1 = randn_bf16((e, f, h), g, 0.02).to(dev)
    w2 = randn_bf16((e, h, f), g, 0.02).to(dev)
    results = []
    for pad in (16, 128):
        if kind == "linear":
            mod = pkg.GroupedLinear(h, f, e, torch.bfloat16, device=dev, pad_multiple=pad, reference_layout=True)
            mod.weight_tensor.data.copy_(w1)
        else:
            mod = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev, pad_multiple=pad, reference_layout=True)
            mod.fc1_weight.data.copy_(w1)
            mod.fc2_weight.data.copy_(w2)
        xd = x.clone().requires_grad_()
        with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=1)):
            out = mod(xd, torch.tensor(sizes))
        out.backward(dy)
        results.append([out.detach(), xd.grad] + [p.grad for p in mod.parameters()])
    for a, b in zip(*results):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("reference_layout", [False, True], ids=["in-place", "reference-layout"])
def test_grouped_linear_reuses_cached_fp8_weights(dev, reference_layout):
    """is_first_microbatch: True casts the weights into the module's buffers, False reuses them.  The weights
    are CHANGED between the two micro-batches, so only a pass that really reuses the cached bytes (and their
    scale_inv) can match the oracle, which is handed the first pass's fp8 weights; a later True picks up the
    new weights."""
    pkg = _pkg()
    sizes, k, n = [137, 401, 59, 403], 256, 512
    e, m, hist = len(sizes), sum(sizes), 2
    g = gen(3001)
    w = randn_bf16((e, n, k), g, 0.02)
    w_changed = (w.float() * 1.5 + 0.01).to(torch.bfloat16)
    module = pkg.GroupedLinear(k, n, e, torch.bfloat16, device=dev, reference_layout=reference_layout)
    fp8_recipe = pkg.DelayedScaling(amax_history_len=hist)
    fwd, bwd = orc.Meta(3 * e, hist), orc.Meta(2 * e, hist)
    weight_slots = [3 * i + 1 for i in range(e)]
    plan = [(True, w), (True, w), (False, w_changed), (False, w_changed), (True, w_changed)]
    cached = None
    for step, (first, w_now) in enumerate(plan):
        x = randn_bf16((m, k), g)
        dy = randn_bf16((m, n), g, 1e-2)
        if step > 0:
            fwd.update(448.0, keep_scale_inv=() if first else weight_slots)
            bwd.update(57344.0)
        o = orc.grouped_linear_step(x, w_now, sizes, dy, fwd, bwd, cached=None if first else cached)
        if first:
            cached = o
        module.weight_tensor.data.copy_(w_now)
        xd = x.to(dev).requires_grad_()
        module.weight_tensor.grad = None
        with pkg.fp8_autocast(enabled=True, fp8_recipe=fp8_recipe):
            out = module(xd, torch.tensor(sizes), is_first_microbatch=first)
        out.backward(dy.to(dev))
        gm = module.fp8_meta
        assert_scalar_bits_equal(gm["scaling_fwd"].scale, fwd.scale, f"step {step} fwd scale")
        assert_scalar_bits_equal(gm["scaling_fwd"].scale_inv, fwd.scale_inv, f"step {step} fwd scale_inv")
        assert_scalar_bits_equal(gm["scaling_fwd"].amax_history, fwd.amax_history, f"step {step} fwd amax history")
        assert_scalar_bits_equal(gm["scaling_bwd"].amax_history, bwd.amax_history, f"step {step} bwd amax history")
        if not first:   # nothing was cast: the weights' amax slots received nothing
            assert not gm["scaling_fwd"].amax_history[0][weight_slots].any()
        w_fp8, w_t_fp8 = module.get_fp8_weights_scratchpad(first)
        assert torch.equal(w_fp8.cpu().view(torch.uint8), cached["w_fp8"].view(torch.uint8)), f"step {step}"
        if reference_layout:
            assert torch.equal(w_t_fp8.cpu().view(torch.uint8), cached["w_t_fp8"].view(torch.uint8)), f"step {step}"
        else:
            assert w_t_fp8 is None   # the data-gradient GEMM reads w_fp8 in place
        assert_gemm_close(out, o["out"].float(), 1e-2, f"step {step} out")
        assert_gemm_close(xd.grad, o["grad_input"].float(), 1e-2, f"step {step} grad_input")
        assert_gemm_close(module.weight_tensor.grad, o["grad_weight"].float(), 1e-2, f"step {step} grad_weight")
    assert module.get_fp8_weights_scratchpad(None) == [None, None]


def test_cached_weights_need_a_first_microbatch(dev):
    pkg = _pkg()
    module = pkg.GroupedLinear(64, 64, 2, torch.bfloat16, device=dev, reference_layout=True)
    x = torch.zeros(32, 64, dtype=torch.bfloat16, device=dev, requires_grad=True)
    with pytest.raises(RuntimeError, match="is_first_microbatch=False"):
        module(x, [16, 16], is_first_microbatch=False)
    with torch.no_grad():
        module(x, [16, 16], is_first_microbatch=True)      # casts without the transposes
        module(x, [16, 16], is_first_microbatch=False)     # enough for another pass without gradients
    with pytest.raises(RuntimeError, match="transposes"):
        module(x, [16, 16], is_first_microbatch=False)     # but not for one that needs dgrad


@pytest.mark.parametrize("frozen", [False, True], ids=["trainable", "frozen-weights"])
def test_grouped_mlp_cached_weights_equal_recast_weights(dev, frozen):
    """Once the weights' scales have settled (constant weights), reusing the cached fp8 weights must give the
    same bits as casting them again: module A runs True, True, False, False, module B casts on every pass.
    With frozen weights the backward pass takes the cast-only dGELU kernel and skips the weight gradients."""
    pkg = _pkg()
    sizes, h, f = [137, 0, 401, 59, 403], 256, 512
    e, m = len(sizes), sum(sizes)
    g = gen(3002)
    w1 = randn_bf16((e, f, h), g, 0.02).to(dev)
    w2 = randn_bf16((e, h, f), g, 0.02).to(dev)
    mods = []
    for _ in range(2):
        mod = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)
        mod.fc1_weight.data.copy_(w1)
        mod.fc2_weight.data.copy_(w2)
        if frozen:
            mod.fc1_weight.requires_grad_(False)
            mod.fc2_weight.requires_grad_(False)
        mods.append(mod)
    fp8_recipe = pkg.DelayedScaling(amax_history_len=4)
    gs = torch.tensor(sizes)
    weight_slots = [3 * i + 1 for i in range(2 * e)]
    for step, first in enumerate([True, True, False, False]):
        x = randn_bf16((m, h), g).to(dev)
        dy = randn_bf16((m, h), g, 1e-2).to(dev)
        res = []
        for mod, flag in zip(mods, (first, None)):
            xd = x.clone().requires_grad_()
            mod.zero_grad()
            with pkg.fp8_autocast(fp8_recipe=fp8_recipe):
                out = mod(xd, gs, is_first_microbatch=flag)
            out.backward(dy)
            res.append((out, xd.grad, mod.fc1_weight.grad, mod.fc2_weight.grad))
        for name, a, b in zip(("out", "grad_input", "grad_fc1", "grad_fc2"), *res):
            if a is None:
                assert b is None and frozen
                continue
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"step {step}: {name} differs"
        fa, fb = mods[0].fp8_meta["scaling_fwd"], mods[1].fp8_meta["scaling_fwd"]
        assert torch.equal(fa.scale, fb.scale) and torch.equal(fa.scale_inv, fb.scale_inv), f"step {step}"
        if first:
            assert torch.equal(fa.amax_history, fb.amax_history)
        else:
            assert not fa.amax_history[0][weight_slots].any() and fb.amax_history[0][weight_slots].all()
        assert torch.equal(mods[0].fp8_meta["scaling_bwd"].amax_history, mods[1].fp8_meta["scaling_bwd"].amax_history)


@pytest.mark.parametrize("kind", ["linear", "linear-cutlass", "mlp"])
def test_weights_cast_ahead_of_the_pass_give_the_same_bits(dev, kind):
    """``cast_weights_ahead()`` moves the scaling update and the weight casts in front of the moment the group sizes
    are known; outputs, gradients and the whole scaling state must equal those of a module that does everything
    inside ``forward``, step after step with changing weights and sizes - also with two forward passes in flight
    before their backward passes, and back on the plain path afterwards."""
    pkg = _pkg()
    e, h, f = 5, 256, 512
    g = gen(3105)
    mods = []
    for _ in range(2):
        if kind == "mlp":
            mod = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)
        else:
            mod = pkg.GroupedLinear(h, f, e, torch.bfloat16, device=dev, cutlass=kind == "linear-cutlass")
        mods.append(mod)
    mods[1].load_state_dict(mods[0].state_dict())
    params = [[p for _, p in sorted(mod.named_parameters())] for mod in mods]
    fp8_recipe = pkg.DelayedScaling(amax_history_len=3)
    out_features = h if kind == "mlp" else f
    splits = [[137, 0, 401, 59, 403], [1, 999, 0, 0, 0], [200] * 5, [64, 64, 0, 64, 808]]

    def passes(mod, ahead, batches):
        """Forward passes over all batches first, then their backward passes in reverse order."""
        outs = []
        for x, sizes, _ in batches:
            with pkg.fp8_autocast(fp8_recipe=fp8_recipe):
                if ahead:
                    assert mod.cast_weights_ahead()
                outs.append(mod(x, torch.tensor(sizes)))
        for out, (_, _, dy) in reversed(list(zip(outs, batches))):
            out.backward(dy)
        return outs

    for step, ahead in enumerate([True, True, True, False, True]):
        n = 2 if step == 2 else 1    # step 2: two passes in flight
        data = []
        for i in range(n):
            sizes = splits[(step + i) % len(splits)]
            m = sum(sizes)
            data.append((randn_bf16((m, h), g).to(dev), sizes, randn_bf16((m, out_features), g, 1e-2).to(dev)))
        res = []
        for mod, use in zip(mods, (ahead, False)):
            mod.zero_grad()
            batches = [(x.clone().requires_grad_(), sizes, dy) for x, sizes, dy in data]
            outs = passes(mod, use, batches)
            res.append(outs + [b[0].grad for b in batches] + [p.grad for _, p in sorted(mod.named_parameters())])
        for i, (a, b) in enumerate(zip(*res)):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"step {step}: result {i} differs"
        for name in ("scaling_fwd", "scaling_bwd"):
            sa, sb = mods[0].fp8_meta[name], mods[1].fp8_meta[name]
            assert torch.equal(sa.scale, sb.scale) and torch.equal(sa.scale_inv, sb.scale_inv), f"step {step} {name}"
            assert torch.equal(sa.amax_history, sb.amax_history), f"step {step} {name}"
        with torch.no_grad():   # an optimizer step: the weights change, so do their scales
            for pa, pb in zip(*params):
                pa.add_(pa.grad, alpha=-0.5)
                pb.add_(pb.grad, alpha=-0.5)
    with pytest.raises(RuntimeError, match="cast_weights_ahead"):
        mods[0].cast_weights_ahead()
        mods[0](data[0][0], torch.tensor(data[0][1]), is_first_microbatch=True)


def test_grouped_mlp_frozen_weights_against_the_oracle(dev):
    """No weight gradients: padded transposes are skipped and d(pre-GELU) goes through the cast-only dGELU
    kernel; output and grad_input must still be the oracle's."""
    pkg = _pkg()
    sizes, h, f = MLP_CASES["small"]
    e, m = len(sizes), sum(sizes)
    g = gen(3003)
    w1 = randn_bf16((e, f, h), g, 0.02)
    w2 = randn_bf16((e, h, f), g, 0.02)
    x = randn_bf16((m, h), g)
    dy = randn_bf16((m, h), g, 1e-2)
    module = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev)
    module.fc1_weight.data.copy_(w1)
    module.fc2_weight.data.copy_(w2)
    module.fc1_weight.requires_grad_(False)
    module.fc2_weight.requires_grad_(False)
    fwd, bwd = orc.Meta(3 * 2 * e, 1), orc.Meta(2 * 2 * e, 1)
    o = orc.grouped_mlp_step(x, w1, w2, sizes, dy, fwd, bwd)
    xd = x.to(dev).requires_grad_()
    with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=1)):
        out = module(xd, torch.tensor(sizes))
    out.backward(dy.to(dev))
    assert module.fc1_weight.grad is None and module.fc2_weight.grad is None
    assert_close_multistage(out, o["out"], 5e-3, "out")
    assert_close_multistage(xd.grad, o["grad_input"], 1e-2, "grad_input")
    _check_amax(module.fp8_meta["scaling_bwd"], bwd, [2 * i for i in range(e)], [2 * (e + i) for i in range(e)],
                "frozen bwd")


@pytest.mark.parametrize("kind", ["linear", "mlp"])
def test_in_place_gradient_gemms_equal_the_reference_layout(dev, kind):
    """By default no transposed fp8 copies are cast and the data- and weight-gradient GEMMs read the row-major
    tensors in place; with reference_layout=True the reference's transposed weights [E, K, N] and padded transposed
    activations / gradients are cast and used.  Same bits either way, over three steps of delayed scaling."""
    pkg = _pkg()
    sizes, h, f = [137, 0, 401, 59, 403], 256, 512
    e, m = len(sizes), sum(sizes)
    g = gen(3004)
    mods = []
    for tw in (False, True):
        if kind == "linear":
            mod = pkg.GroupedLinear(h, f, e, torch.bfloat16, device=dev, reference_layout=tw)
        else:
            mod = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev, reference_layout=tw)
        mods.append(mod)
    mods[1].load_state_dict(mods[0].state_dict())
    out_cols = f if kind == "linear" else h
    fp8_recipe = pkg.DelayedScaling(amax_history_len=2)
    for step in range(3):
        x = randn_bf16((m, h), g).to(dev)
        dy = randn_bf16((m, out_cols), g, 1e-2).to(dev)
        res = []
        for mod in mods:
            xd = x.clone().requires_grad_()
            mod.zero_grad()
            with pkg.fp8_autocast(fp8_recipe=fp8_recipe):
                out = mod(xd, torch.tensor(sizes))
            out.backward(dy)
            res.append([out, xd.grad] + [p.grad for p in mod.parameters()])
        for a, b in zip(*res):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"step {step}"
        assert torch.equal(mods[0].fp8_meta["scaling_bwd"].amax_history, mods[1].fp8_meta["scaling_bwd"].amax_history)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["linear", "mlp"])
def test_weight_gradient_on_a_transposed_gradient_copy_gives_the_same_bits(dev, kind, monkeypatch):
    """FP8GMM_WGRAD=copy: the modules cast a transposed, zero-padded copy of the gradient for the weight-gradient
    GEMM and read only the activation in place; by default they read both operands in place.  Row counts that are
    multiples of nothing, an empty expert: the same bits either way - outputs, all gradients, and the backward amax
    history - over three steps of delayed scaling."""
    pkg = _pkg()
    from fp8_gmm_amd import backend

    sizes, h, f = [137, 0, 401, 59, 403, 1], 256, 512
    e, m = len(sizes), sum(sizes)
    g = gen(3011)
    mods = []
    for _ in range(2):
        mod = (pkg.GroupedLinear if kind == "linear" else pkg.GroupedMlp)(h, f, e, torch.bfloat16, device=dev)
        mods.append(mod)
    mods[1].load_state_dict(mods[0].state_dict())
    out_cols = f if kind == "linear" else h
    fp8_recipe = pkg.DelayedScaling(amax_history_len=2)
    assert not backend.wgrad_wants_transposed_gradient(m, e)   # the default
    for step in range(3):
        x = randn_bf16((m, h), g).to(dev)
        dy = randn_bf16((m, out_cols), g, 1e-2).to(dev)
        res = []
        for mod, mode in zip(mods, ("in_place", "copy")):
            monkeypatch.setattr(backend.options, "wgrad", mode)
            xd = x.clone().requires_grad_()
            mod.zero_grad()
            with pkg.fp8_autocast(fp8_recipe=fp8_recipe):
                out = mod(xd, torch.tensor(sizes))
            out.backward(dy)
            res.append([out, xd.grad] + [p.grad for p in mod.parameters()])
        for a, b in zip(*res):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"step {step}"
        assert torch.equal(mods[0].fp8_meta["scaling_bwd"].amax_history, mods[1].fp8_meta["scaling_bwd"].amax_history)


@pytest.mark.gpu
@pytest.mark.parametrize("sizes", [[137, 0, 59, 403, 1, 700], [0, 0, 16], [300] * 9])
def test_planned_passes_equal_the_per_launch_path(dev, sizes):
    """GroupedLinear plans a whole pass with one library call (fp8gmm_plan_linear_forward / _backward).  Outputs,
    gradients, fp8 scaling state and amax history must equal, bit for bit, what the per-launch entry points give
    over three steps (ragged, empty and equal experts; with cached fp8 weights on the last step)."""
    import fp8_gmm_amd as pkg

    e, k, n = len(sizes), 256, 384
    g = torch.Generator(device=dev).manual_seed(5)
    w = (torch.randn(e, n, k, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    xs = [torch.randn(sum(sizes), k, generator=g, device=dev).to(torch.bfloat16) for _ in range(3)]
    dys = [(torch.randn(sum(sizes), n, generator=g, device=dev) * 1e-2).to(torch.bfloat16) for _ in range(3)]
    results = []
    for planned in (True, False):
        module = pkg.GroupedLinear(k, n, e, torch.bfloat16, device=dev, planned_passes=planned)
        module.weight_tensor.data.copy_(w)
        recipe = pkg.DelayedScaling(amax_history_len=2)
        trace = []
        for step, first in enumerate((None, True, False)):
            x = xs[step].clone().requires_grad_()
            module.zero_grad(set_to_none=True)
            with pkg.fp8_autocast(enabled=True, fp8_recipe=recipe):
                out = module(x, torch.tensor(sizes), is_first_microbatch=first)
            out.backward(dys[step])
            torch.cuda.synchronize()
            fwd, bwd = module.fp8_meta["scaling_fwd"], module.fp8_meta["scaling_bwd"]
            trace.append([out.detach().clone(), x.grad.clone(), module.weight_tensor.grad.clone(), fwd.scale.clone(),
                          fwd.amax_history.clone(), bwd.scale.clone(), bwd.amax_history.clone()])
        results.append(trace)
    names = ["out", "grad_input", "grad_weight", "fwd scale", "fwd amax history", "bwd scale", "bwd amax history"]
    for step, (a, b) in enumerate(zip(*results)):
        for name, ta, tb in zip(names, a, b):
            assert torch.equal(ta.view(torch.int16) if ta.dtype == torch.bfloat16 else ta,
                               tb.view(torch.int16) if tb.dtype == torch.bfloat16 else tb), f"step {step}: {name}"


@pytest.mark.gpu
def test_planned_pass_tables_are_those_of_the_per_launch_entry_points(dev, monkeypatch):
    """The tables fp8gmm_plan_linear_forward / _backward write for given buffers must be, byte for byte, the tensor
    descriptors, problem tables, work lists and shared-tile records that backend.multi_quantize / fp8_gmm /
    grouped_gemm build for the same buffers (captured here without launching anything)."""
    import ctypes

    import numpy as np

    from fp8_gmm_amd import _lib, backend

    sizes = [700, 0, 33, 1291, 5, 256]
    e, k, n, tokens = len(sizes), 512, 768, sum(sizes)
    E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
    x = torch.zeros(tokens, k, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(e, n, k, dtype=torch.bfloat16, device=dev)
    x8, w8 = torch.zeros(tokens, k, dtype=E4, device=dev), torch.zeros(e, n, k, dtype=E4, device=dev)
    y = torch.zeros(tokens, n, dtype=torch.bfloat16, device=dev)
    dy, dy8 = torch.zeros(tokens, n, dtype=torch.bfloat16, device=dev), torch.zeros(tokens, n, dtype=E5, device=dev)
    dx, dw = torch.zeros(tokens, k, dtype=torch.bfloat16, device=dev), torch.zeros(e, n, k, dtype=torch.bfloat16, device=dev)
    fs, fsi, fa = (torch.ones(3 * e, device=dev) for _ in range(3))
    bs, bsi, ba = (torch.ones(2 * e, device=dev) for _ in range(3))
    bounds = np.concatenate([[0], np.cumsum(sizes)])
    ptr = lambda t, first, stride: np.uint64(t.data_ptr() + 4 * first) + np.arange(e, dtype=np.uint64) * np.uint64(4 * stride)
    rows, stack = backend.TensorBatch.rows_of, backend.TensorBatch.stack_of

    captured = []
    monkeypatch.setattr(backend, "_flush", lambda items: captured.extend(bytes(it[0].view(np.uint8).reshape(-1)) for it in items))
    with backend.batched_uploads():
        backend.multi_quantize(rows(x, bounds) + stack(w), rows(x8, bounds) + stack(w8),
                               np.concatenate([ptr(fs, 0, 3), ptr(fs, 1, 3)]), np.concatenate([ptr(fa, 0, 3), ptr(fa, 1, 3)]))
        backend.fp8_gmm(x8, w8, sizes, ptr(fsi, 0, 3), ptr(fsi, 1, 3), c=y)
        backend.multi_quantize(rows(dy, bounds), rows(dy8, bounds), ptr(bs, 0, 2), ptr(ba, 0, 2))
        backend.grouped_gemm(rows(dy8, bounds), rows(x8, bounds), stack(dw), ptr(bsi, 0, 2), ptr(fsi, 0, 3), transposed=True)
        backend.fp8_gmm(dy8, w8, sizes, ptr(bsi, 0, 2), ptr(fsi, 1, 3), c=dx, backward=True, b_transposed=True)
    assert len(captured) == 5

    grid = _lib.gemm_grid(_lib.init(torch.cuda.current_device()))
    gs = np.asarray(sizes, dtype=np.int64)
    policy = {"auto": 0, "256": 256, "128": 128, "dual": _lib.GEMM_TILE_DUAL}[backend.options.tile]   # as backend does
    desc = _lib.LinearPass(experts=e, in_features=k, out_features=n, fwd_fmt=_lib.E4M3, bwd_fmt=_lib.E5M2, cast_weights=1,
                           dgrad=1, wgrad=1, grid=grid, stream_k=int(backend.options.stream_k), tile_policy=policy, tokens=tokens,
                           group_sizes=gs.ctypes.data, x=x.data_ptr(), x_fp8=x8.data_ptr(), w=w.data_ptr(),
                           w_fp8=w8.data_ptr(), y=y.data_ptr(), dy=dy.data_ptr(), dy_fp8=dy8.data_ptr(), dx=dx.data_ptr(),
                           dw=dw.data_ptr(), fwd_scale=fs.data_ptr(), fwd_scale_inv=fsi.data_ptr(), fwd_amax=fa.data_ptr(),
                           bwd_scale=bs.data_ptr(), bwd_scale_inv=bsi.data_ptr(), bwd_amax=ba.data_ptr())
    L = _lib.load()
    blob = np.zeros(1 << 22, dtype=np.uint8)
    want = iter(captured)
    for fn in (L.fp8gmm_plan_linear_forward, L.fp8gmm_plan_linear_backward):
        plan = _lib.PassPlan()
        # a blob that is too small reports the size the pass needs
        assert fn(ctypes.byref(desc), blob.ctypes.data, 1024, ctypes.byref(plan)) == -8
        need = plan.blob_bytes
        _lib.check(fn(ctypes.byref(desc), blob.ctypes.data, blob.nbytes, ctypes.byref(plan)))
        assert plan.blob_bytes == need
        for i in range(plan.n_launches):
            rec, ref = plan.launch[i], next(want)
            if rec.kind == _lib.PASS_CAST:
                got = bytes(blob[rec.table_offset: rec.table_offset + rec.n * 128])
                assert got == ref, "tensor descriptors differ"
            else:
                probs = bytes(blob[rec.table_offset: rec.table_offset + rec.n * 96])
                items = bytes(blob[rec.items_offset: rec.items_offset + rec.plan.rounds * rec.plan.grid * 64])
                fix = bytes(blob[rec.fixups_offset: rec.fixups_offset + rec.plan.n_fixups * 32])
                off_items = (rec.n * 96 + 127) // 128 * 128
                assert probs == ref[: rec.n * 96], "problem table differs"
                assert items == ref[off_items: off_items + len(items)], "work list differs"
                assert fix == ref[off_items + len(items):], "shared-tile records differ"


@pytest.mark.gpu
@pytest.mark.parametrize("sizes", [[137, 0, 59, 403, 1, 700], [0, 0, 16], [300] * 9])
@pytest.mark.parametrize("grads", ["both", "input", "weights"])
def test_planned_mlp_passes_equal_the_per_launch_path(dev, sizes, grads):
    """GroupedMlp plans a whole pass with one library call (fp8gmm_plan_mlp_forward / _backward).  Outputs, gradients,
    the intermediates between the kernels, fp8 scaling state and amax history must equal, bit for bit, what the
    per-launch entry points give over three steps (ragged, empty and equal experts; cached fp8 weights on the last
    step; gradients wanted for the input, the weights or both)."""
    import fp8_gmm_amd as pkg

    e, h, f = len(sizes), 256, 384
    g = torch.Generator(device=dev).manual_seed(6)
    w1 = (torch.randn(e, f, h, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn(e, h, f, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    xs = [torch.randn(sum(sizes), h, generator=g, device=dev).to(torch.bfloat16) for _ in range(3)]
    dys = [(torch.randn(sum(sizes), h, generator=g, device=dev) * 1e-2).to(torch.bfloat16) for _ in range(3)]
    results = []
    for planned in (True, False):
        module = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev, planned_passes=planned)
        module.fc1_weight.data.copy_(w1)
        module.fc2_weight.data.copy_(w2)
        for p in module.parameters():
            p.requires_grad_(grads != "input")
        cap = {}
        module.capture_intermediates(cap)
        recipe = pkg.DelayedScaling(amax_history_len=2)
        trace = []
        for step, first in enumerate((None, True, False)):
            x = xs[step].clone().requires_grad_(grads != "weights")
            module.zero_grad(set_to_none=True)
            with pkg.fp8_autocast(enabled=True, fp8_recipe=recipe):
                out = module(x, torch.tensor(sizes), is_first_microbatch=first)
            out.backward(dys[step])
            torch.cuda.synchronize()
            fwd, bwd = module.fp8_meta["scaling_fwd"], module.fp8_meta["scaling_bwd"]
            got = {"out": out.detach(), "grad_input": x.grad, "grad_fc1": module.fc1_weight.grad,
                   "grad_fc2": module.fc2_weight.grad, "fwd scale": fwd.scale, "fwd amax history": fwd.amax_history,
                   "bwd scale": bwd.scale, "bwd amax history": bwd.amax_history}
            got.update(cap)
            trace.append({k: v.clone() for k, v in got.items() if v is not None})
        results.append(trace)
    bits = {torch.bfloat16: torch.int16, torch.float8_e4m3fn: torch.uint8, torch.float8_e5m2: torch.uint8}
    for step, (a, b) in enumerate(zip(*results)):
        assert a.keys() == b.keys()
        assert {"pre_gelu_out", "gelu_out_fp8", "grad_gelu_out", "grad_pre_fp8"} <= a.keys()
        assert ("grad_input" in a) == (grads != "weights") and ("grad_fc1" in a) == (grads != "input")
        for name in a:
            ta, tb = a[name], b[name]
            assert ta.dtype == tb.dtype and ta.shape == tb.shape, name
            assert torch.equal(ta.view(bits.get(ta.dtype, ta.dtype)), tb.view(bits.get(tb.dtype, tb.dtype))), \
                f"step {step}: {name}"


@pytest.mark.gpu
def test_planned_mlp_pass_tables_are_those_of_the_per_launch_entry_points(dev, monkeypatch):
    """The tables fp8gmm_plan_mlp_forward / _backward write for given buffers must be, byte for byte, the tensor
    descriptors, problem tables, work lists and shared-tile records that backend.multi_quantize / fp8_gmm /
    grouped_gemm / multi_cast_dgelu build for the same buffers in the order GroupedMlp calls them (captured here
    without launching anything)."""
    import ctypes

    import numpy as np

    from fp8_gmm_amd import _lib, backend

    sizes = [700, 0, 33, 1291, 5, 256]
    e, h, f, tokens = len(sizes), 512, 768, sum(sizes)
    E4, E5, bf = torch.float8_e4m3fn, torch.float8_e5m2, torch.bfloat16
    z = lambda shape, dtype: torch.zeros(shape, dtype=dtype, device=dev)
    x, x8 = z((tokens, h), bf), z((tokens, h), E4)
    w1, w18, dw1 = z((e, f, h), bf), z((e, f, h), E4), z((e, f, h), bf)
    w2, w28, dw2 = z((e, h, f), bf), z((e, h, f), E4), z((e, h, f), bf)
    pre, act8, y = z((tokens, f), bf), z((tokens, f), E4), z((tokens, h), bf)
    dy, dy8, dact, dpre8, dx = z((tokens, h), bf), z((tokens, h), E5), z((tokens, f), bf), z((tokens, f), E5), z((tokens, h), bf)
    fs, fsi, fa = (torch.ones(6 * e, device=dev) for _ in range(3))
    bs, bsi, ba = (torch.ones(4 * e, device=dev) for _ in range(3))
    bounds = np.concatenate([[0], np.cumsum(sizes)])
    ptr = lambda t, first, stride: np.uint64(t.data_ptr() + 4 * first) + np.arange(e, dtype=np.uint64) * np.uint64(4 * stride)
    rows, stack = backend.TensorBatch.rows_of, backend.TensorBatch.stack_of
    g2, b2 = 3 * e, 2 * e   # first forward / backward scaling slot of the fc2 GEMMs

    captured = []
    monkeypatch.setattr(backend, "_flush", lambda items: captured.extend(bytes(it[0].view(np.uint8).reshape(-1)) for it in items))
    with backend.batched_uploads():
        # forward: casts (fc2's weights, fc1's weights, the input), fc1 with the GELU epilogue, fc2
        backend.multi_quantize(stack(w2) + stack(w1) + rows(x, bounds), stack(w28) + stack(w18) + rows(x8, bounds),
                               np.concatenate([ptr(fs, g2 + 1, 3), ptr(fs, 1, 3), ptr(fs, 0, 3)]),
                               np.concatenate([ptr(fa, g2 + 1, 3), ptr(fa, 1, 3), ptr(fa, 0, 3)]))
        backend.fp8_gmm(x8, w18, sizes, ptr(fsi, 0, 3), ptr(fsi, 1, 3), c=act8, pre_gelu_out=pre,
                        c_scales=ptr(fs, g2, 3), c_amaxes=ptr(fa, g2, 3))
        backend.fp8_gmm(act8, w28, sizes, ptr(fsi, g2, 3), ptr(fsi, g2 + 1, 3), c=y)
        # backward: cast, fc2 wgrad, fc2 dgrad, dGELU cast, fc1 dgrad, fc1 wgrad
        backend.multi_quantize(rows(dy, bounds), rows(dy8, bounds), ptr(bs, 0, 2), ptr(ba, 0, 2))
        backend.grouped_gemm(rows(dy8, bounds), rows(act8, bounds), stack(dw2), ptr(bsi, 0, 2), ptr(fsi, g2, 3), transposed=True)
        backend.fp8_gmm(dy8, w28, sizes, ptr(bsi, 0, 2), ptr(fsi, g2 + 1, 3), c=dact, backward=True, b_transposed=True)
        backend.multi_cast_dgelu(rows(dact, bounds), rows(pre, bounds), rows(dpre8, bounds), ptr(bs, b2, 2), ptr(ba, b2, 2))
        backend.fp8_gmm(dpre8, w18, sizes, ptr(bsi, b2, 2), ptr(fsi, 1, 3), c=dx, backward=True, b_transposed=True)
        backend.grouped_gemm(rows(dpre8, bounds), rows(x8, bounds), stack(dw1), ptr(bsi, b2, 2), ptr(fsi, 0, 3), transposed=True)
    assert len(captured) == 9

    grid = _lib.gemm_grid(_lib.init(torch.cuda.current_device()))
    gs = np.asarray(sizes, dtype=np.int64)
    policy = {"auto": 0, "256": 256, "128": 128, "dual": _lib.GEMM_TILE_DUAL}[backend.options.tile]   # as backend does
    desc = _lib.MlpPass(experts=e, hidden=h, ffn=f, fwd_fmt=_lib.E4M3, bwd_fmt=_lib.E5M2, cast_weights=1, dgrad=1, wgrad=1,
                        grid=grid, stream_k=int(backend.options.stream_k), tile_policy=policy, tokens=tokens,
                        group_sizes=gs.ctypes.data, x=x.data_ptr(), x_fp8=x8.data_ptr(), w1=w1.data_ptr(),
                        w1_fp8=w18.data_ptr(), w2=w2.data_ptr(), w2_fp8=w28.data_ptr(), pre=pre.data_ptr(),
                        act_fp8=act8.data_ptr(), y=y.data_ptr(), dy=dy.data_ptr(), dy_fp8=dy8.data_ptr(),
                        dact=dact.data_ptr(), dpre_fp8=dpre8.data_ptr(), dx=dx.data_ptr(), dw1=dw1.data_ptr(),
                        dw2=dw2.data_ptr(), fwd_scale=fs.data_ptr(), fwd_scale_inv=fsi.data_ptr(), fwd_amax=fa.data_ptr(),
                        bwd_scale=bs.data_ptr(), bwd_scale_inv=bsi.data_ptr(), bwd_amax=ba.data_ptr())
    L = _lib.load()
    blob = np.zeros(1 << 23, dtype=np.uint8)
    want = iter(captured)
    for fn, launches in ((L.fp8gmm_plan_mlp_forward, 3), (L.fp8gmm_plan_mlp_backward, 6)):
        plan = _lib.PassPlan()
        assert fn(ctypes.byref(desc), blob.ctypes.data, 1024, ctypes.byref(plan)) == -8
        need = plan.blob_bytes
        _lib.check(fn(ctypes.byref(desc), blob.ctypes.data, blob.nbytes, ctypes.byref(plan)))
        assert plan.blob_bytes == need and plan.n_launches == launches
        for i in range(plan.n_launches):
            rec, ref = plan.launch[i], next(want)
            if rec.kind == _lib.PASS_CAST:
                got = bytes(blob[rec.table_offset: rec.table_offset + rec.n * 128])
                assert got == ref, f"launch {i}: tensor descriptors differ"
            else:
                probs = bytes(blob[rec.table_offset: rec.table_offset + rec.n * 96])
                items = bytes(blob[rec.items_offset: rec.items_offset + rec.plan.rounds * rec.plan.grid * 64])
                fix = bytes(blob[rec.fixups_offset: rec.fixups_offset + rec.plan.n_fixups * 32])
                off_items = (rec.n * 96 + 127) // 128 * 128
                assert probs == ref[: rec.n * 96], f"launch {i}: problem table differs"
                assert items == ref[off_items: off_items + len(items)], f"launch {i}: work list differs"
                assert fix == ref[off_items + len(items):], f"launch {i}: shared-tile records differ"
    # the launch records say what each launch is
    plan = _lib.PassPlan()
    _lib.check(L.fp8gmm_plan_mlp_forward(ctypes.byref(desc), blob.ctypes.data, blob.nbytes, ctypes.byref(plan)))
    assert (plan.launch[1].out_kind, plan.launch[1].epilogue) == (_lib.E4M3, _lib.EPI_GELU)
    assert (plan.launch[2].out_kind, plan.launch[2].epilogue) == (_lib.OUT_BF16, 0)
    _lib.check(L.fp8gmm_plan_mlp_backward(ctypes.byref(desc), blob.ctypes.data, blob.nbytes, ctypes.byref(plan)))
    assert [plan.launch[i].op for i in (0, 3)] == [_lib.OP_QUANTIZE, _lib.OP_CAST_DGELU]
    assert [plan.launch[i].epilogue for i in (1, 2, 4, 5)] == [
        _lib.GEMM_A_KMAJOR | _lib.GEMM_B_KMAJOR, _lib.GEMM_B_KMAJOR, _lib.GEMM_B_KMAJOR, _lib.GEMM_A_KMAJOR | _lib.GEMM_B_KMAJOR]


@pytest.mark.gpu
def test_fused_dgelu_backward_against_the_oracle(dev):
    """GroupedMlp(fused_dgelu=True): the fc2 data-gradient GEMM forms d(pre-GELU) = fp8(v * dgelu(pre)) in its
    epilogue, from the fp32 accumulator, and the separate cast + dGELU pass is gone.  Checked against the oracle's
    step with the same fusion (oracle/modules.py, fused_dgelu=True) fed the GPU's own pre-activation and GELU bytes:
    the d(pre-GELU) bytes may sit one fp8 code step from the oracle's (another summation order under one rounding)
    on at most 1 % of the elements, their amax within 1e-3, and everything downstream within the GEMM tolerance of
    the oracle's GEMMs on the GPU's bytes.  Against the unfused module the bytes move by at most one code step (the
    unfused path rounds the GEMM result to bf16 first), and the forward pass is untouched."""
    import fp8_gmm_amd as pkg
    from helpers import _mini_meta, assert_fp8_codes_close

    sizes, h, f = [300, 0, 77, 513], 256, 512
    e, m = len(sizes), sum(sizes)
    g = torch.Generator().manual_seed(99)
    w1 = (torch.randn(e, f, h, generator=g) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn(e, h, f, generator=g) * 0.05).to(torch.bfloat16)
    x = torch.randn(m, h, generator=g).to(torch.bfloat16)
    dy = (torch.randn(m, h, generator=g) * 1e-2).to(torch.bfloat16)
    runs = {}
    for fused in (True, False):
        module = pkg.GroupedMlp(h, f, e, torch.bfloat16, device=dev, fused_dgelu=fused)
        module.fc1_weight.data.copy_(w1)
        module.fc2_weight.data.copy_(w2)
        cap = {}
        module.capture_intermediates(cap)
        recipe = pkg.DelayedScaling(amax_history_len=1)
        for _ in range(2):   # the second step runs with scales derived from real amaxes
            xd = x.to(dev).requires_grad_()
            module.zero_grad(set_to_none=True)
            with pkg.fp8_autocast(enabled=True, fp8_recipe=recipe):
                out = module(xd, torch.tensor(sizes))
            out.backward(dy.to(dev))
            torch.cuda.synchronize()
        runs[fused] = (module, cap, out.detach().cpu(), xd.grad.cpu())
    module, cap, out, gin = runs[True]
    _, cap_u, out_u, _ = runs[False]
    assert cap["grad_gelu_out"] is None, "the fused pass must not materialise the bf16 d(GELU output)"
    assert torch.equal(out.view(torch.int16), out_u.view(torch.int16)), "the forward pass must not change"
    assert_fp8_codes_close(cap["grad_pre_fp8"].cpu(), cap_u["grad_pre_fp8"].cpu(), "fused against unfused d(pre-GELU)", 0.10)

    gm = module.fp8_meta
    for i in (0, 2, 3):
        r0, r1 = sum(sizes[:i]), sum(sizes[:i + 1])
        fwd = _mini_meta(gm["scaling_fwd"], [3 * i, 3 * i + 1, 3 * i + 2, 3 * (e + i), 3 * (e + i) + 1, 3 * (e + i) + 2])
        bwd = _mini_meta(gm["scaling_bwd"], [2 * i, 2 * i + 1, 2 * (e + i), 2 * (e + i) + 1])
        given = {"pre": cap["pre_gelu_out"][r0:r1].cpu().contiguous(),
                 "gelu_fp8": cap["gelu_out_fp8"][r0:r1].cpu().contiguous()}
        o = orc.grouped_mlp_step(x[r0:r1].contiguous(), w1[i: i + 1], w2[i: i + 1], [sizes[i]], dy[r0:r1].contiguous(),
                                 fwd, bwd, given=given, fused_dgelu=True)
        got = cap["grad_pre_fp8"][r0:r1].cpu()
        assert_fp8_codes_close(got, o["own_dpre_fp8"], f"expert {i}: d(pre-GELU) against the oracle")
        gpu_amax = gm["scaling_bwd"].amax_history[0][2 * (e + i)].item()
        assert abs(gpu_amax - bwd.amax_history[0][2].item()) <= 1e-3 * gpu_amax
        # downstream of the GPU's own bytes
        o = orc.grouped_mlp_step(x[r0:r1].contiguous(), w1[i: i + 1], w2[i: i + 1], [sizes[i]], dy[r0:r1].contiguous(),
                                 _mini_meta(gm["scaling_fwd"], [3 * i, 3 * i + 1, 3 * i + 2, 3 * (e + i), 3 * (e + i) + 1,
                                                                3 * (e + i) + 2]),
                                 _mini_meta(gm["scaling_bwd"], [2 * i, 2 * i + 1, 2 * (e + i), 2 * (e + i) + 1]),
                                 given=dict(given, dpre_fp8=got.contiguous()), fused_dgelu=True)
        assert_gemm_close(gin[r0:r1], o["grad_input"].float(), 1e-2, f"expert {i} grad_input")
        assert_gemm_close(module.fc1_weight.grad[i], o["grad_w1"][0].float(), 1e-2, f"expert {i} grad_fc1")
        assert_gemm_close(module.fc2_weight.grad[i], o["grad_w2"][0].float(), 1e-2, f"expert {i} grad_fc2")
    assert not module.fc1_weight.grad[1].any() and not module.fc2_weight.grad[1].any()
