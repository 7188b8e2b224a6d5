"""Token routing on the GPU (sort / histogram / gather / scatter and their gradients) against the CPU oracle,
and the routed example layers end to end.  Integer results and copied rows are compared bit for bit; scatter's
bf16 output too (the kernel and the oracle follow the same fp32 sequence); only the per-row dot products of
scatter's weight gradient, whose summation order differs, get a tolerance (1e-5 relative to the row norms)."""
import numpy as np
import pytest
import torch

from oracle import moe as orc

pytestmark = pytest.mark.gpu


def _ops():
    from fp8_gmm_amd import moe_ops

    return moe_ops


def _ids(n, e, seed, kind="uniform"):
    rng = np.random.default_rng(seed)
    if kind == "zipf":
        p = 1.0 / np.arange(1, e + 1) ** 1.1
        return rng.choice(e, size=n, p=p / p.sum())
    if kind == "one":
        return np.full(n, e - 1)
    return rng.integers(0, e, size=n)


ROUTE_CASES = [(1, 1, "uniform"), (63, 4, "uniform"), (64, 2, "uniform"), (1000, 4, "uniform"), (1025, 7, "zipf"),
               (32768, 8, "uniform"), (24576, 64, "zipf"), (65536, 128, "uniform"), (70000, 4096, "uniform"),
               (5000, 16, "one"), (0, 8, "uniform")]


@pytest.mark.parametrize("n,e,kind", ROUTE_CASES)
def test_sort_histogram_and_bins(dev, n, e, kind):
    ops = _ops()
    ids = _ids(n, e, 100 + n, kind)
    x = torch.tensor(ids, dtype=torch.int32, device=dev)
    want_indices, want_bin_ids, want_bins, want_counts = orc.indices_and_bins(ids, e)
    indices, bin_ids, bins, counts = ops.indices_and_bins(x, max(int(np.ceil(np.log2(e))), 1), e)
    assert indices.dtype == bin_ids.dtype == bins.dtype == counts.dtype == torch.int32
    assert indices.cpu().tolist() == want_indices.tolist()
    assert bin_ids.cpu().tolist() == want_bin_ids.tolist()
    assert counts.cpu().tolist() == want_counts.tolist()
    assert bins.cpu().tolist() == want_bins.tolist()
    # the single operators give the same answers
    end_bit = max(int(np.ceil(np.log2(e))), 1)
    s_ids, s_idx = ops.sort(x, end_bit)
    assert torch.equal(s_ids, bin_ids) and torch.equal(s_idx, indices)
    assert torch.equal(ops.histogram(x, e), counts)
    assert torch.equal(ops.inclusive_cumsum(counts, 0), bins)
    _, _, inverse, _, _ = ops.route(x, e, want_inverse=True)
    assert inverse.cpu().tolist() == orc.invert(want_indices).tolist()


def test_out_of_range_ids_are_clamped(dev):
    ops = _ops()
    x = torch.tensor([5, -3, 2, 9, 0], dtype=torch.int32, device=dev)
    bin_ids, indices = ops.sort(x, 2)          # ids below 4
    assert bin_ids.cpu().tolist() == [0, 0, 2, 3, 3] and indices.cpu().tolist() == [1, 4, 2, 0, 3]
    with pytest.raises(RuntimeError):
        ops.histogram(x, 5000)
    with pytest.raises(RuntimeError):
        ops.sort(x.long())


ROW_CASES = [(1, 1, 8, 1), (37, 2, 256, 4), (128, 2, 4096, 8), (50, 1, 520, 3), (64, 8, 768, 16), (33, 3, 100, 5),
             (16, 2, 6, 2), (0, 2, 64, 4)]


@pytest.mark.parametrize("tokens,top_k,hidden,e", ROW_CASES)
def test_gather_scatter_and_their_gradients(dev, tokens, top_k, hidden, e):
    ops = _ops()
    g = torch.Generator().manual_seed(7 + tokens)
    ids = _ids(tokens * top_k, e, 200 + tokens)
    indices_cpu = orc.sort(ids)[1]
    indices = torch.tensor(indices_cpu, dtype=torch.int32, device=dev)
    x = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    y = torch.randn(tokens * top_k, hidden, generator=g).to(torch.bfloat16)
    w = torch.rand(tokens * top_k, generator=g)
    grad_rows = torch.randn(tokens * top_k, hidden, generator=g).to(torch.bfloat16)
    grad_tok = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)

    xd = x.to(dev).requires_grad_()
    got = ops.gather(xd, indices, None, None, top_k)
    assert torch.equal(got.cpu().view(torch.int16), orc.gather(x, indices_cpu, top_k).view(torch.int16))
    got.backward(grad_rows.to(dev))
    assert torch.equal(xd.grad.cpu().view(torch.int16),
                       orc.gather_backward(grad_rows, indices_cpu, top_k).view(torch.int16))

    for weights in (w, None):
        yd = y.to(dev).requires_grad_()
        wd = weights.to(dev).requires_grad_() if weights is not None else None
        out = ops.scatter(yd, indices, None, wd, None, top_k)
        assert torch.equal(out.cpu().view(torch.int16), orc.scatter(y, indices_cpu, top_k, weights).view(torch.int16))
        out.backward(grad_tok.to(dev))
        want_gx, want_gw = orc.scatter_backward(grad_tok, y, indices_cpu, top_k, weights)
        assert torch.equal(yd.grad.cpu().view(torch.int16), want_gx.view(torch.int16))
        if weights is not None and tokens:
            idx = torch.as_tensor(indices_cpu.astype(np.int64))
            bound = torch.zeros(tokens * top_k)
            bound[idx] = y.float().norm(dim=1) * grad_tok.float()[idx // top_k].norm(dim=1)
            assert ((wd.grad.cpu() - want_gw).abs() <= 1e-5 * bound + 1e-30).all()


@pytest.mark.parametrize("tokens,e,top_k,dtype", [(1, 1, 1, torch.float32), (1000, 16, 2, torch.bfloat16),
                                                   (16384, 16, 2, torch.bfloat16), (513, 64, 8, torch.float32),
                                                   (300, 200, 3, torch.bfloat16), (77, 4096, 4, torch.float32),
                                                   (0, 8, 2, torch.bfloat16)])
def test_topk_against_the_oracle(dev, tokens, e, top_k, dtype):
    """softmax + top-k in one launch: the chosen experts equal the oracle's (bf16 scores are full of equal values,
    so this also holds the rule for ties), the weights agree to a few ulp of fp32, and the gradient with respect to
    the scores agrees with the oracle's float64 chain to fp32 / bf16 rounding."""
    ops = _ops()
    rng = np.random.default_rng(900 + tokens + e)
    z = torch.from_numpy(rng.standard_normal((tokens, e)).astype(np.float32) * 2).to(dtype)
    zd = z.to(dev).requires_grad_()
    w, sel = ops.topk(zd, top_k)
    assert w.dtype == torch.float32 and sel.dtype == torch.int64 and w.shape == sel.shape == (tokens, top_k)
    want_w, want_sel = orc.topk(z.float().numpy(), top_k)
    assert (sel.cpu().numpy() == want_sel).all()
    np.testing.assert_allclose(w.detach().cpu().numpy(), want_w, rtol=4e-6, atol=1e-30)
    gw = torch.from_numpy(rng.standard_normal((tokens, top_k)).astype(np.float32))
    w.backward(gw.to(dev))
    want_g = orc.topk_backward(z.float().numpy(), want_sel, gw.numpy())
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    assert zd.grad.dtype == dtype
    np.testing.assert_allclose(zd.grad.float().cpu().numpy(), want_g, rtol=tol, atol=tol * 1e-2)


def test_topk_falls_back_to_torch_and_renormalises(dev):
    ops = _ops()
    z = torch.randn(50, 8, device=dev, dtype=torch.float64)    # not a dtype of the kernel: torch's operators
    w, sel = ops.topk(z, 2)
    tw, tsel = torch.topk(torch.softmax(z, dim=1, dtype=torch.float), 2)
    assert torch.equal(sel, tsel) and torch.equal(w, tw)
    w, _ = ops.topk(z.float(), 2, moe_renorm=True)
    assert torch.allclose(w.sum(dim=1), torch.ones(50, device=dev))


@pytest.mark.parametrize("tokens,top_k,hidden,e", [(1000, 2, 256, 4), (513, 1, 4096, 7), (300, 4, 2056, 16),
                                                    (64, 2, 100, 3)])
def test_scatter_backward_in_one_pass_equals_the_two_passes(dev, tokens, top_k, hidden, e):
    """With both gradients wanted scatter's backward pass is one launch; it must write the bits of the two
    single-purpose launches (weighted gather, per-row dot products), which run when only one gradient is wanted -
    also on rows that 16-byte accesses cannot take (hidden = 100)."""
    ops = _ops()
    rng = np.random.default_rng(40 + tokens)
    ids = torch.tensor(rng.integers(0, e, size=tokens * top_k), dtype=torch.int32, device=dev)
    indices, bin_ids, bins, _ = ops.indices_and_bins(ids, 0, e)
    x = torch.from_numpy(rng.standard_normal((tokens * top_k, hidden)).astype(np.float32)).to(torch.bfloat16).to(dev)
    w = torch.from_numpy(rng.random(tokens * top_k).astype(np.float32)).to(dev)
    g = torch.from_numpy(rng.standard_normal((tokens, hidden)).astype(np.float32)).to(torch.bfloat16).to(dev)

    def grads(need_x, need_w):
        xd, wd = x.clone().requires_grad_(need_x), w.clone().requires_grad_(need_w)
        ops.scatter(xd, indices, bin_ids, wd, bins, top_k).backward(g)
        return xd.grad, wd.grad

    both_x, both_w = grads(True, True)
    only_x, _ = grads(True, False)
    _, only_w = grads(False, True)
    assert torch.equal(both_x.view(torch.int16), only_x.view(torch.int16))
    assert torch.equal(both_w.view(torch.int32), only_w.view(torch.int32))


def test_bad_arguments_are_rejected(dev):
    ops = _ops()
    x = torch.zeros(4, 8, dtype=torch.bfloat16, device=dev)
    idx = torch.arange(8, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        ops.gather(x.float(), idx, None, None, 2)
    with pytest.raises(RuntimeError):
        ops.gather(x, idx[:5], None, None, 2)
    with pytest.raises(RuntimeError):
        ops.scatter(x, idx[:4], None, torch.ones(3, device=dev), None, 2)
    with pytest.raises(RuntimeError):
        ops.gather(x.cpu(), idx.cpu(), None, None, 2)


@pytest.mark.parametrize("kind", ["mlp", "linear"])
def test_routed_layer_forward_against_the_oracle_composition(dev, kind):
    """Fp8MlpModule / Fp8LinearModule: with the layer's own routing decisions (read back from the GPU) the output
    must be scatter(experts(gather(x))) as the CPU oracle computes it."""
    import fp8_gmm_amd as pkg
    from fp8_gmm_amd import moe
    from helpers import assert_close_multistage
    from oracle import modules as orc_mod

    tokens, h, f, e, top_k = 96, 128, 256, 5, 2
    torch.manual_seed(11)
    layer = (moe.Fp8MlpModule if kind == "mlp" else moe.Fp8LinearModule)(h, f, e, top_k, device=dev)
    x = torch.randn(tokens, h).to(torch.bfloat16)
    with torch.no_grad(), pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=1)):
        out = layer(x.to(dev))
        weights0, selected = layer.gating_network(x.to(dev)), None
        weights0, selected = pkg.moe_ops.topk(weights0, top_k)
    ids = selected.flatten().cpu().numpy()
    w = weights0.flatten().cpu()
    indices, _, _, counts = orc.indices_and_bins(ids, e)
    sizes = counts.tolist()
    xs = orc.gather(x, indices, top_k)
    if kind == "mlp":
        fwd, bwd = orc_mod.Meta(3 * 2 * e, 1), orc_mod.Meta(2 * 2 * e, 1)
        y = orc_mod.grouped_mlp_step(xs, layer.grouped_mlp.fc1_weight.detach().cpu(),
                                     layer.grouped_mlp.fc2_weight.detach().cpu(), sizes,
                                     torch.zeros(tokens * top_k, h, dtype=torch.bfloat16), fwd, bwd)["out"]
    else:
        zeros = torch.zeros(tokens * top_k, f, dtype=torch.bfloat16)
        fwd, bwd = orc_mod.Meta(3 * e, 1), orc_mod.Meta(2 * e, 1)
        mid = orc_mod.grouped_linear_step(xs, layer.grouped_linear1.weight_tensor.detach().cpu(), sizes, zeros, fwd,
                                          bwd)["out"]
        mid = torch.nn.functional.gelu(mid.float()).to(torch.bfloat16)
        fwd, bwd = orc_mod.Meta(3 * e, 1), orc_mod.Meta(2 * e, 1)
        y = orc_mod.grouped_linear_step(mid, layer.grouped_linear2.weight_tensor.detach().cpu(), sizes,
                                        torch.zeros(tokens * top_k, h, dtype=torch.bfloat16), fwd, bwd)["out"]
    want = orc.scatter(y, indices, top_k, w)
    assert_close_multistage(out, want, 1e-2, f"{kind} layer output")


def test_routed_mlp_layer_trains_like_a_dense_fp32_model(dev):
    """Forward + backward of Fp8MlpModule against an fp32 autograd model of the same routed layer (same routing
    decisions): cosine similarity of the output and of every gradient, gating weights included."""
    import fp8_gmm_amd as pkg
    from fp8_gmm_amd import moe

    tokens, h, f, e, top_k = 512, 256, 512, 8, 2
    torch.manual_seed(12)
    layer = moe.Fp8MlpModule(h, f, e, top_k, device=dev)
    x = torch.randn(tokens, h, device=dev).to(torch.bfloat16)
    dy = torch.randn(tokens, h, device=dev).to(torch.bfloat16)
    for _ in range(2):   # the second pass runs with real scales
        xd = x.clone().requires_grad_()
        layer.zero_grad()
        with pkg.fp8_autocast(fp8_recipe=pkg.DelayedScaling(amax_history_len=2)):
            out = layer(xd)
        out.backward(dy)

    xr = x.float().requires_grad_()
    gate = layer.gating_network.weight.detach().float().requires_grad_()
    w1 = layer.grouped_mlp.fc1_weight.detach().float().requires_grad_()
    w2 = layer.grouped_mlp.fc2_weight.detach().float().requires_grad_()
    logits = layer.gating_network(x).float()                  # the layer's own bf16 logits decide the routing
    _, selected = pkg.moe_ops.topk(logits, top_k)
    probs = torch.softmax(xr @ gate.t(), dim=1)
    ref = torch.zeros(tokens, h, device=dev)
    for k in range(top_k):
        ek = selected[:, k]
        hidden = torch.nn.functional.gelu(torch.einsum("th,tfh->tf", xr, w1[ek]), approximate="tanh")
        ref = ref + probs.gather(1, ek[:, None]) * torch.einsum("tf,thf->th", hidden, w2[ek])
    ref.backward(dy.float())

    def cos(a, b):
        a, b = a.detach().float().flatten(), b.detach().float().flatten()
        return (torch.dot(a, b) / (a.norm() * b.norm())).item()

    assert cos(out, ref) > 0.995
    assert cos(xd.grad, xr.grad) > 0.99
    assert cos(layer.grouped_mlp.fc1_weight.grad, w1.grad) > 0.99
    assert cos(layer.grouped_mlp.fc2_weight.grad, w2.grad) > 0.99
    assert cos(layer.gating_network.weight.grad, gate.grad) > 0.98


def test_example_bf16_layer_against_a_dense_fp32_model(dev):
    """The bf16 layer of the example recipe (one vendor GEMM per expert on its row slice, hand-written gradients)
    against an fp32 autograd model of the same routed layer with the same routing decisions."""
    import fp8_gmm_amd as pkg
    from fp8_gmm_amd import example

    tokens, h, f, e, top_k = 384, 128, 256, 6, 2
    torch.manual_seed(21)
    layer = example.Bf16Module(h, f, e, top_k, device=dev)
    x = torch.randn(tokens, h, device=dev).to(torch.bfloat16)
    dy = torch.randn(tokens, h, device=dev).to(torch.bfloat16)
    xd = x.clone().requires_grad_()
    out = layer(xd)
    out.backward(dy)

    xr = x.float().requires_grad_()
    gate = layer.gating_network.weight.detach().float().requires_grad_()
    w1 = layer.w1.detach().float().requires_grad_()
    w2 = layer.w2.detach().float().requires_grad_()
    _, selected = pkg.moe_ops.topk(layer.gating_network(x).float(), top_k)
    probs = torch.softmax(xr @ gate.t(), dim=1)
    ref = torch.zeros(tokens, h, device=dev)
    for k in range(top_k):
        ek = selected[:, k]
        hidden = torch.nn.functional.gelu(torch.einsum("th,tfh->tf", xr, w1[ek]))
        ref = ref + probs.gather(1, ek[:, None]) * torch.einsum("tf,thf->th", hidden, w2[ek])
    ref.backward(dy.float())

    def cos(a, b):
        a, b = a.detach().float().flatten(), b.detach().float().flatten()
        return (torch.dot(a, b) / (a.norm() * b.norm())).item()

    assert cos(out, ref) > 0.9995
    assert cos(xd.grad, xr.grad) > 0.999
    assert cos(layer.w1.grad, w1.grad) > 0.999
    assert cos(layer.w2.grad, w2.grad) > 0.999
    assert cos(layer.gating_network.weight.grad, gate.grad) > 0.995


def test_example_recipe_runs_every_kind_of_layer(dev, capsys):
    """``python -m fp8_gmm_amd.example`` at a small size: four timed kinds, one printed line each."""
    from fp8_gmm_amd import example

    times = example.main(["--tokens", "512", "--hidden", "256", "--inner", "512", "--experts", "8", "--warmup", "1",
                          "--steps", "2"])
    assert list(times) == list(example.KINDS) and all(t > 0 for t in times.values())
    lines = [line for line in capsys.readouterr().out.splitlines() if " run: " in line]
    assert len(lines) == 4 and lines[0].startswith("Bf16Module run: ") and lines[3].startswith("Fp8MlpModule run: ")
