"""Shared helpers of the test-suite: seeded inputs, shape lists, comparisons."""
import os

import torch

from oracle import ref

FP8_DTYPES = [torch.float8_e4m3fn, torch.float8_e5m2]

# The shape list every pointwise test of the reference runs in ONE multi-tensor call
# (fp8_gmm/test.py:10-21): aligned and unaligned tensors mixed.
REFERENCE_SHAPES = [
    (2048, 12288),
    (768, 1024),
    (256, 65536),
    (65536, 128),
    (256, 256),
    (120, 2080),
    (8, 8),
    (1, 3221),
    (2333, 1),
    (1481, 677),
]

# Smaller list with the same edge structure, for quick checks.
SMALL_SHAPES = [(256, 256), (120, 2080), (8, 8), (1, 3221), (2333, 1), (1481, 677), (17, 129), (1, 1), (128, 128)]


def padded_rows(m, pad):
    return (m + pad - 1) // pad * pad if pad else m


def transpose_shapes(shapes, padded, pad=16):
    """Shapes of the transposed outputs, as fp8_gmm/test.py:23-30 builds them."""
    return [(n, padded_rows(m, pad) if padded else m) for (m, n) in shapes]


def gen(seed):
    """The tests' random inputs: a generator seeded per call site.  FP8GMM_TEST_SEED_OFFSET (an integer, 0 by default)
    shifts every seed, to run the whole suite over other draws."""
    return torch.Generator().manual_seed(seed + int(os.environ.get("FP8GMM_TEST_SEED_OFFSET", "0")))


def randn_bf16(shape, g, std=1.0):
    return (torch.randn(shape, generator=g) * std).to(torch.bfloat16)


def bytes_of(t):
    return t.contiguous().view(torch.uint8)


def assert_bytes_equal(gpu, cpu, what=""):
    a = bytes_of(gpu.cpu())
    b = bytes_of(cpu)
    assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
    if not torch.equal(a, b):
        diff = (a != b).nonzero()
        first = tuple(diff[0].tolist())
        raise AssertionError(
            f"{what}: {diff.shape[0]} of {a.numel()} bytes differ; first at {first}: "
            f"gpu=0x{int(a[first]):02x} oracle=0x{int(b[first]):02x}"
        )


def assert_scalar_bits_equal(gpu, cpu, what=""):
    a = gpu.detach().cpu().reshape(-1).view(torch.int32)
    b = cpu.detach().reshape(-1).view(torch.int32)
    assert torch.equal(a, b), f"{what}: {gpu.detach().cpu().reshape(-1).tolist()} vs {cpu.reshape(-1).tolist()}"


def gemm_rel_err(c, ref_f32):
    """max |c - ref| / max |ref|: the GEMM acceptance metric (<= 1e-2)."""
    denom = ref_f32.abs().max().clamp_min(1e-30)
    return ((c.float() - ref_f32).abs().max() / denom).item()


def assert_gemm_close(c_gpu, ref_f32, tol=1e-2, what=""):
    """GEMM outputs vs the fp32 dequantised matmul.

    Two conditions, both stated by the north star's "max relative error <= 1e-2":
      * global:      max|c - ref| <= tol * max|ref|
      * per element: |c - ref| <= tol * |ref| + tol * rms(ref)   (bf16 rounding is 2^-9 relative;
        the rms term covers elements that cancel to near zero)
    """
    c = c_gpu.detach().float().cpu()
    assert c.shape == ref_f32.shape, f"{what}: shape {c.shape} vs {ref_f32.shape}"
    if ref_f32.numel() == 0:
        return
    assert torch.isfinite(c).all(), f"{what}: non-finite output"
    err = (c - ref_f32).abs()
    g = (err.max() / ref_f32.abs().max().clamp_min(1e-30)).item()
    assert g <= tol, f"{what}: max|err|/max|ref| = {g:.3e} > {tol}"
    rms = ref_f32.pow(2).mean().sqrt()
    bound = tol * ref_f32.abs() + tol * rms
    bad = err > bound
    assert not bad.any(), f"{what}: {int(bad.sum())} elements outside |err| <= {tol}(|ref| + rms)"


def scales_for(tensors, dtype):
    """Per-tensor scale = fp8_max / amax (fp32), scale_inv = 1 / scale, like a settled delayed-scaling state."""
    fmax = ref.FP8_MAX[dtype]
    scales, invs = [], []
    for t in tensors:
        amax = t.float().abs().max() if t.numel() else torch.tensor(0.0)
        s = torch.tensor(fmax, dtype=torch.float32) / amax if amax > 0 else torch.tensor(1.0)
        s = s.to(torch.float32).reshape(1)
        scales.append(s)
        invs.append((1.0 / s).to(torch.float32))
    return scales, invs


def assert_close_multistage(c_gpu, ref_t, fro_tol=5e-3, what=""):
    """Comparison for results that went through one or more fp8 RE-quantisations of computed values
    (GroupedMlp): the GPU and the oracle accumulate in different orders, so a value that sits on an
    fp8 rounding boundary may land one code step apart (6-12 % of that element) and move the few
    outputs it feeds by several percent of the output rms.  The orchestration is what is under test
    here (a wrong operand, scale or slot gives O(1) errors), so the bounds are:
      * relative Frobenius error <= fro_tol
      * every element within 0.02 |ref| + 0.25 rms(ref)
    Stage-exact checks of each kernel live in the backend tests.
    """
    c = c_gpu.detach().float().cpu()
    r = ref_t.float()
    assert c.shape == r.shape, f"{what}: shape {c.shape} vs {r.shape}"
    if r.numel() == 0:
        return
    assert torch.isfinite(c).all(), f"{what}: non-finite output"
    err = c - r
    fro = (err.norm() / r.norm().clamp_min(1e-30)).item()
    assert fro <= fro_tol, f"{what}: relative Frobenius error {fro:.3e} > {fro_tol}"
    rms = r.pow(2).mean().sqrt()
    bad = err.abs() > 0.02 * r.abs() + 0.25 * rms
    assert not bad.any(), f"{what}: {int(bad.sum())} elements outside 0.02|ref| + 0.25 rms"


def fp8_code_distance(a, b):
    """|difference| in fp8 code steps between two same-dtype fp8 tensors (sign-magnitude codes)."""
    ia = a.view(torch.uint8).to(torch.int32)
    ib = b.view(torch.uint8).to(torch.int32)
    sa = torch.where(ia >= 128, -(ia - 128), ia)
    sb = torch.where(ib >= 128, -(ib - 128), ib)
    return (sa - sb).abs()


def assert_fp8_codes_close(got, want, what, max_fraction_off=0.01):
    """Two fp8 tensors whose values come from contractions summed in different orders: at most one code step apart
    wherever the value is not tiny, on at most `max_fraction_off` of the elements.  A sum of thousands of terms that
    cancels to under a hundredth of the tensor's typical size carries the summation-order noise at full weight, and
    the fp8 codes are dense around zero: there the VALUES must agree to a hundredth of the typical size instead."""
    dist = fp8_code_distance(got, want)
    wv, gv = want.float(), got.float()
    rms = wv.pow(2).mean().sqrt()
    big = wv.abs() > 1e-2 * rms
    assert (dist[big] <= 1).all(), f"{what}: {int((dist[big] > 1).sum())} values more than one code step apart"
    assert ((gv - wv).abs()[~big] <= 1e-2 * rms).all(), f"{what}: small values differ by more than 1e-2 of the rms"
    off = (dist != 0).float().mean().item()
    assert off <= max_fraction_off, f"{what}: {off:.4f} of the bytes differ"


def _mini_meta(gpu_meta, slots):
    """The scaling state of `slots` of a module's GPU meta as an oracle Meta with history length 1 (amax row
    cleared: the oracle records its own)."""
    from oracle import modules as orc

    m = orc.Meta(len(slots), 1)
    m.scale = gpu_meta.scale.detach().cpu()[slots].clone()
    m.scale_inv = gpu_meta.scale_inv.detach().cpu()[slots].clone()
    return m


def check_linear_expert_against_oracle(module, i, sizes, x, dy, out, grad_input, tol=1e-2, what=""):
    """One expert of a GroupedLinear step against the CPU oracle, with the scales the GPU pass used: output,
    input gradient and weight gradient within `tol`, the amax of every directly cast tensor bit-exact.
    To be called after the step, before the next forward pass updates the scales."""
    from oracle import modules as orc

    e = len(sizes)
    r0 = sum(sizes[:i])
    r1 = r0 + sizes[i]
    gm = module.fp8_meta
    fwd = _mini_meta(gm["scaling_fwd"], [3 * i, 3 * i + 1, 3 * i + 2])
    bwd = _mini_meta(gm["scaling_bwd"], [2 * i, 2 * i + 1])
    w = module.weight_tensor.detach()[i: i + 1].cpu()
    o = orc.grouped_linear_step(x[r0:r1].cpu().contiguous(), w, [sizes[i]], dy[r0:r1].cpu().contiguous(), fwd, bwd)
    tag = f"{what} expert {i} ({sizes[i]} rows)"
    assert_gemm_close(out[r0:r1], o["out"].float(), tol, f"{tag} out")
    assert_gemm_close(grad_input[r0:r1], o["grad_input"].float(), tol, f"{tag} grad_input")
    assert_gemm_close(module.weight_tensor.grad[i], o["grad_weight"][0].float(), tol, f"{tag} grad_weight")
    g_fwd = gm["scaling_fwd"].amax_history[0].detach().cpu()
    g_bwd = gm["scaling_bwd"].amax_history[0].detach().cpu()
    assert_scalar_bits_equal(g_fwd[[3 * i, 3 * i + 1]], fwd.amax_history[0][[0, 1]], f"{tag} forward amax")
    assert_scalar_bits_equal(g_bwd[[2 * i]], bwd.amax_history[0][[0]], f"{tag} grad_out amax")
    assert e == module.num_groups


def check_mlp_expert_against_oracle(module, captured, i, sizes, x, dy, out, grad_input, tol=1e-2, what=""):
    """One expert of a GroupedMlp step against the CPU oracle, stage by stage.

    The fp8 re-quantisations inside the layer (GELU output, d(pre-GELU)) make an end-to-end comparison loose: a
    value on a rounding boundary may land one fp8 code apart and move what it feeds.  So the oracle is handed
    the GPU's own intermediates (`captured`, from GroupedMlp.capture_intermediates) at each such point, and every
    stage is held to its own bar:
      pre-GELU, d(GELU output)                     within `tol` of the oracle's own values (GEMM + bf16)
      fp8 GELU output                              at most one code step from the oracle's epilogue of the pre-GELU copy
      d(pre-GELU) fp8 bytes and its amax           bit-exact, given the GPU's bf16 inputs of that cast
      output, input and weight gradients           within `tol` of the oracle's GEMMs on the GPU's fp8 bytes
      amax of x, both weights, grad_out            bit-exact"""
    from oracle import modules as orc

    e = len(sizes)
    r0 = sum(sizes[:i])
    r1 = r0 + sizes[i]
    gm = module.fp8_meta
    fwd = _mini_meta(gm["scaling_fwd"], [3 * i, 3 * i + 1, 3 * i + 2, 3 * (e + i), 3 * (e + i) + 1, 3 * (e + i) + 2])
    bwd = _mini_meta(gm["scaling_bwd"], [2 * i, 2 * i + 1, 2 * (e + i), 2 * (e + i) + 1])
    w1 = module.fc1_weight.detach()[i: i + 1].cpu()
    w2 = module.fc2_weight.detach()[i: i + 1].cpu()
    given = {"pre": captured["pre_gelu_out"][r0:r1].cpu().contiguous(),
             "gelu_fp8": captured["gelu_out_fp8"][r0:r1].cpu().contiguous(),
             "grad_gelu": captured["grad_gelu_out"][r0:r1].cpu().contiguous(),
             "dpre_fp8": captured["grad_pre_fp8"][r0:r1].cpu().contiguous()}
    o = orc.grouped_mlp_step(x[r0:r1].cpu().contiguous(), w1, w2, [sizes[i]], dy[r0:r1].cpu().contiguous(), fwd, bwd,
                             given=given)
    tag = f"{what} expert {i} ({sizes[i]} rows)"
    assert_gemm_close(given["pre"], o["own_pre"].float(), tol, f"{tag} pre-GELU")
    # The fp8 GELU output is formed from the fp32 accumulator, of which the bf16 pre-GELU copy is a rounding: the
    # oracle's epilogue applied to that copy lands at most one code step away.  (Against the oracle's OWN
    # accumulator a value near zero can differ by several codes: a contraction of thousands of terms that cancels
    # to 1e-3 of its scale carries the summation-order noise at full weight.)
    acc = given["pre"].float().contiguous()
    from_pre = torch.empty_like(given["gelu_fp8"])
    scratch_amax = torch.zeros(1)
    ref.lib().orc_epilogue_gelu_fp8(acc.data_ptr(), acc.numel(), 1.0, 1.0, fwd.scale[3:4].data_ptr(),
                                    ref.fmt_of(from_pre.dtype), None, from_pre.data_ptr(), scratch_amax.data_ptr())
    dist = fp8_code_distance(given["gelu_fp8"], from_pre)
    if dist.max() > 1:
        at = tuple((dist == dist.max()).nonzero()[0].tolist())
        raise AssertionError(
            f"{tag}: fp8 GELU output {int(dist.max())} code steps from the oracle at {at} ({int((dist > 1).sum())} such): "
            f"gpu byte 0x{int(given['gelu_fp8'].view(torch.uint8)[at]):02x}, oracle byte "
            f"0x{int(from_pre.view(torch.uint8)[at]):02x}, pre {given['pre'][at].item()!r}, c_scale {fwd.scale[3].item()!r}")
    assert (dist != 0).float().mean() <= 0.08, f"{tag}: {(dist != 0).float().mean():.3f} of the GELU bytes differ"
    own = fp8_code_distance(given["gelu_fp8"], o["own_gelu_fp8"])
    assert (own > 1).float().mean() <= 1e-4, f"{tag}: GELU bytes far from the oracle's own"
    assert_gemm_close(out[r0:r1], o["out"].float(), tol, f"{tag} out")
    assert_gemm_close(given["grad_gelu"], o["own_grad_gelu"].float(), tol, f"{tag} d(GELU output)")
    assert_bytes_equal(given["dpre_fp8"], o["own_dpre_fp8"], f"{tag} d(pre-GELU) fp8 bytes")
    assert_gemm_close(grad_input[r0:r1], o["grad_input"].float(), tol, f"{tag} grad_input")
    assert_gemm_close(module.fc1_weight.grad[i], o["grad_w1"][0].float(), tol, f"{tag} grad_fc1")
    assert_gemm_close(module.fc2_weight.grad[i], o["grad_w2"][0].float(), tol, f"{tag} grad_fc2")
    g_fwd = gm["scaling_fwd"].amax_history[0].detach().cpu()
    g_bwd = gm["scaling_bwd"].amax_history[0].detach().cpu()
    assert_scalar_bits_equal(g_fwd[[3 * i, 3 * i + 1, 3 * (e + i) + 1]], fwd.amax_history[0][[0, 1, 4]],
                             f"{tag} amax of x, fc1 weight, fc2 weight")
    assert_scalar_bits_equal(g_bwd[[2 * i, 2 * (e + i)]], bwd.amax_history[0][[0, 2]],
                             f"{tag} amax of grad_out and d(pre-GELU)")
    assert torch.allclose(g_fwd[3 * (e + i)], fwd.amax_history[0][3], rtol=1e-3, atol=0), f"{tag} GELU amax"
