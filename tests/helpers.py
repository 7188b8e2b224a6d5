"""Shared helpers of the test-suite: seeded inputs, shape lists, comparisons."""
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
    return torch.Generator().manual_seed(seed)


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
