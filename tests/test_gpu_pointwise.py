"""GPU parity of the multi-tensor cast / pad / transpose entry points against the CPU oracle.

Mirrors the reference's ``TestBackend`` pointwise tests (fp8_gmm/test.py:36-134): the same
10-shape multi-tensor call, both fp8 dtypes, padded and unpadded transposes, random scales
(negative ones included, as ``torch.randn(1)`` gives there).  Where the reference accepts
``atol = rtol = 0.2`` against an unrounded product, these tests demand bit-exact fp8 bytes,
padded layouts and amax values against the oracle.
"""
import pytest
import torch

from helpers import (
    FP8_DTYPES,
    REFERENCE_SHAPES,
    SMALL_SHAPES,
    assert_bytes_equal,
    assert_scalar_bits_equal,
    gen,
    randn_bf16,
    transpose_shapes,
)
from oracle import ref

pytestmark = pytest.mark.gpu


def _backend():
    from fp8_gmm_amd import backend

    return backend


def _scales(n, g, positive=False):
    s = torch.randn(n, generator=g)
    if positive:
        s = s.abs() + 0.1
    return [s[i].reshape(1).clone() for i in range(n)]


def _to_dev(lst, dev):
    return [t.to(dev) for t in lst]


ALL_BF16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
EXHAUSTIVE_SCALES = [1.0, 0.5, 3.7, 448.0 / 3.1, 1e-3, 2.0**-10, 1234.5, -1.0, 57344.0 / 0.37, 2.0**20, 1e-30, 0.0]


@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_quantize_every_bf16_pattern(dev, dtype):
    """All 65 536 bf16 bit patterns (NaNs, infinities, subnormals included) times a set of scales."""
    backend = _backend()
    n = len(EXHAUSTIVE_SCALES)
    scales = [torch.tensor([s], dtype=torch.float32) for s in EXHAUSTIVE_SCALES]
    ins = [ALL_BF16.clone() for _ in range(n)]
    outs = [torch.empty(65536, dtype=dtype) for _ in range(n)]
    amaxes = [torch.zeros(1) for _ in range(n)]
    ref.multi_quantize(ins, outs, scales, amaxes)

    d_outs = [torch.empty(65536, dtype=dtype, device=dev) for _ in range(n)]
    d_amaxes = [torch.zeros(1, device=dev) for _ in range(n)]
    backend.multi_quantize(_to_dev(ins, dev), d_outs, _to_dev(scales, dev), d_amaxes)
    torch.cuda.synchronize()
    for i in range(n):
        assert_bytes_equal(d_outs[i], outs[i], f"scale {EXHAUSTIVE_SCALES[i]}")
        assert_scalar_bits_equal(d_amaxes[i], amaxes[i], f"amax, scale {EXHAUSTIVE_SCALES[i]}")


@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_cast_transpose_every_bf16_pattern(dev, dtype):
    """Same exhaustive input through the cast+transpose kernel (its own conversion code path)."""
    backend = _backend()
    x = ALL_BF16.reshape(256, 256).clone()
    for s in (1.0, 3.7, -0.25, 1e-3):
        scale = torch.tensor([s], dtype=torch.float32)
        o, t, a = torch.empty(256, 256, dtype=dtype), torch.empty(256, 256, dtype=dtype), torch.zeros(1)
        ref.multi_cast_transpose([x], [o], [t], [scale], [a])
        do = torch.empty(256, 256, dtype=dtype, device=dev)
        dt = torch.empty(256, 256, dtype=dtype, device=dev)
        da = torch.zeros(1, device=dev)
        backend.multi_cast_transpose([x.to(dev)], [do], [dt], [scale.to(dev)], [da])
        assert_bytes_equal(do, o, f"cast, scale {s}")
        assert_bytes_equal(dt, t, f"transpose, scale {s}")
        assert_scalar_bits_equal(da, a, f"amax, scale {s}")


@pytest.mark.parametrize("shapes", [SMALL_SHAPES, REFERENCE_SHAPES], ids=["small", "reference"])
@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_multi_quantize(dev, dtype, shapes):
    backend = _backend()
    g = gen(11)
    ins = [randn_bf16(s, g) for s in shapes]
    scales = _scales(len(shapes), g)
    outs = [torch.empty(s, dtype=dtype) for s in shapes]
    amaxes = [torch.zeros(1) for _ in shapes]
    amaxes[1].fill_(100.0)  # previous content larger than the data: must survive the merge
    amaxes[2].fill_(0.5)    # previous content smaller: must be replaced
    d_amaxes = _to_dev(amaxes, dev)
    ref.multi_quantize(ins, outs, scales, amaxes)
    d_outs = [torch.empty(s, dtype=dtype, device=dev) for s in shapes]
    backend.multi_quantize(_to_dev(ins, dev), d_outs, _to_dev(scales, dev), d_amaxes)
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_outs[i], outs[i], f"shape {s}")
        assert_scalar_bits_equal(d_amaxes[i], amaxes[i], f"amax {s}")


@pytest.mark.parametrize("shapes", [SMALL_SHAPES, REFERENCE_SHAPES], ids=["small", "reference"])
@pytest.mark.parametrize("padded", [True, False])
@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_multi_transpose(dev, dtype, padded, shapes):
    backend = _backend()
    g = gen(12)
    t_shapes = transpose_shapes(shapes, padded)
    ins = [randn_bf16(s, g).to(dtype) for s in shapes]
    outs = [torch.empty(ts, dtype=dtype) for ts in t_shapes]
    ref.multi_transpose(ins, outs)
    # fill with a sentinel to catch unwritten pad bytes
    d_outs = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dtype) for ts in t_shapes]
    backend.multi_transpose(_to_dev(ins, dev), d_outs)
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_outs[i], outs[i], f"shape {s}")
        # the oracle itself against the torch closed form the reference tests with (test.py:63-68)
        m = s[0]
        expect = torch.nn.functional.pad(ins[i].view(torch.uint8).t(), (0, t_shapes[i][1] - m))
        assert torch.equal(outs[i].view(torch.uint8), expect)


@pytest.mark.parametrize("shapes", [SMALL_SHAPES, REFERENCE_SHAPES], ids=["small", "reference"])
@pytest.mark.parametrize("padded", [True, False])
@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_multi_cast_transpose(dev, dtype, padded, shapes):
    backend = _backend()
    g = gen(13)
    t_shapes = transpose_shapes(shapes, padded)
    ins = [randn_bf16(s, g) for s in shapes]
    scales = _scales(len(shapes), g)
    outs = [torch.empty(s, dtype=dtype) for s in shapes]
    touts = [torch.empty(ts, dtype=dtype) for ts in t_shapes]
    amaxes = [torch.zeros(1) for _ in shapes]
    ref.multi_cast_transpose(ins, outs, touts, scales, amaxes)
    d_outs = [torch.full(s, 0x55, dtype=torch.uint8, device=dev).view(dtype) for s in shapes]
    d_touts = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dtype) for ts in t_shapes]
    d_amaxes = [torch.zeros(1, device=dev) for _ in shapes]
    backend.multi_cast_transpose(_to_dev(ins, dev), d_outs, d_touts, _to_dev(scales, dev), d_amaxes)
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_outs[i], outs[i], f"cast {s}")
        assert_bytes_equal(d_touts[i], touts[i], f"transpose {s}")
        assert_scalar_bits_equal(d_amaxes[i], amaxes[i], f"amax {s}")


@pytest.mark.parametrize("shapes", [SMALL_SHAPES, REFERENCE_SHAPES], ids=["small", "reference"])
@pytest.mark.parametrize("padded", [True, False])
@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_multi_cast_transpose_dgelu(dev, dtype, padded, shapes):
    backend = _backend()
    g = gen(14)
    t_shapes = transpose_shapes(shapes, padded)
    ins = [randn_bf16(s, g) for s in shapes]
    pres = [randn_bf16(s, g, std=2.0) for s in shapes]
    scales = _scales(len(shapes), g)
    outs = [torch.empty(s, dtype=dtype) for s in shapes]
    touts = [torch.empty(ts, dtype=dtype) for ts in t_shapes]
    amaxes = [torch.zeros(1) for _ in shapes]
    ref.multi_cast_transpose_dgelu(ins, pres, outs, touts, scales, amaxes)
    d_outs = [torch.full(s, 0x55, dtype=torch.uint8, device=dev).view(dtype) for s in shapes]
    d_touts = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dtype) for ts in t_shapes]
    d_amaxes = [torch.zeros(1, device=dev) for _ in shapes]
    backend.multi_cast_transpose_dgelu(_to_dev(ins, dev), _to_dev(pres, dev), d_outs, d_touts, _to_dev(scales, dev),
                                       d_amaxes)
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_outs[i], outs[i], f"cast {s}")
        assert_bytes_equal(d_touts[i], touts[i], f"transpose {s}")
        assert_scalar_bits_equal(d_amaxes[i], amaxes[i], f"amax {s}")


def test_dgelu_every_bf16_pattern(dev):
    """dgelu over every bf16 pre-activation value (dy = 1): the deterministic tanh must match bit for bit."""
    backend = _backend()
    dtype = torch.float8_e5m2
    pre = ALL_BF16.reshape(256, 256).clone()
    dy = torch.ones(256, 256, dtype=torch.bfloat16)
    scale = torch.tensor([100.0])
    o, t, a = torch.empty(256, 256, dtype=dtype), torch.empty(256, 256, dtype=dtype), torch.zeros(1)
    ref.multi_cast_transpose_dgelu([dy], [pre], [o], [t], [scale], [a])
    do = torch.empty(256, 256, dtype=dtype, device=dev)
    dt = torch.empty(256, 256, dtype=dtype, device=dev)
    da = torch.zeros(1, device=dev)
    backend.multi_cast_transpose_dgelu([dy.to(dev)], [pre.to(dev)], [do], [dt], [scale.to(dev)], [da])
    assert_bytes_equal(do, o, "dgelu cast")
    assert_bytes_equal(dt, t, "dgelu transpose")
    assert_scalar_bits_equal(da, a, "dgelu amax")


@pytest.mark.parametrize("dtype", FP8_DTYPES)
def test_multi_cast_dgelu_without_transpose(dev, dtype):
    """The cast-only dGELU kernel writes exactly the row-major bytes and amax of the transposing one; checked
    against the oracle and against the transposing kernel itself, on aligned, odd, tiny and multi-block shapes
    and on every bf16 pre-activation pattern."""
    backend = _backend()
    g = gen(15)
    shapes = SMALL_SHAPES + [(300, 517), (1, 70001), (0, 16)]
    ins = [randn_bf16(s, g) for s in shapes] + [torch.ones(256, 256, dtype=torch.bfloat16)]
    pres = [randn_bf16(s, g, std=2.0) for s in shapes] + [ALL_BF16.reshape(256, 256).clone()]
    shapes = shapes + [(256, 256)]
    scales = _scales(len(shapes), g)
    outs = [torch.empty(s, dtype=dtype) for s in shapes]
    amaxes = [torch.zeros(1) for _ in shapes]
    ref.multi_cast_dgelu(ins, pres, outs, scales, amaxes)
    d_outs = [torch.full(s, 0x55, dtype=torch.uint8, device=dev).view(dtype) for s in shapes]
    d_amaxes = [torch.zeros(1, device=dev) for _ in shapes]
    backend.multi_cast_dgelu(_to_dev(ins, dev), _to_dev(pres, dev), d_outs, _to_dev(scales, dev), d_amaxes)
    t_outs = [torch.empty(s, dtype=dtype, device=dev) for s in shapes]
    t_touts = [torch.empty(s[1], s[0], dtype=dtype, device=dev) for s in shapes]
    t_amaxes = [torch.zeros(1, device=dev) for _ in shapes]
    backend.multi_cast_transpose_dgelu(_to_dev(ins, dev), _to_dev(pres, dev), t_outs, t_touts, _to_dev(scales, dev),
                                       t_amaxes)
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_outs[i], outs[i], f"cast {s}")
        assert_scalar_bits_equal(d_amaxes[i], amaxes[i], f"amax {s}")
        assert torch.equal(d_outs[i].view(torch.uint8), t_outs[i].view(torch.uint8)), f"kernels disagree on {s}"
        assert_scalar_bits_equal(d_amaxes[i], t_amaxes[i].cpu(), f"kernels disagree on amax {s}")
    # misaligned views take the per-element path: same bytes
    base_x = randn_bf16((1, 4099), g).to(dev)
    base_p = randn_bf16((1, 4099), g).to(dev)
    xo, po = base_x[:, 1:], base_p[:, 1:]
    o_view = torch.empty(1, 4099, dtype=dtype, device=dev)[:, 1:]
    am = torch.zeros(1, device=dev)
    backend.multi_cast_dgelu([xo], [po], [o_view], [scales[0].to(dev)], [am])
    want, want_amax = torch.empty(1, 4098, dtype=dtype), torch.zeros(1)
    ref.multi_cast_dgelu([xo.cpu().contiguous()], [po.cpu().contiguous()], [want], [scales[0]], [want_amax])
    assert_bytes_equal(o_view, want, "misaligned cast")
    assert_scalar_bits_equal(am, want_amax, "misaligned amax")


def test_pad_multiple_128_with_outliers(dev):
    """The bandwidth configuration in small: ragged [M_i, 512] tensors, pad to 128, +-200 outliers."""
    backend = _backend()
    g = gen(15)
    dtype = torch.float8_e4m3fn
    ms = [1, 127, 128, 129, 300, 777, 1025, 31]
    ins = []
    for m in ms:
        x = torch.randn(m, 512, generator=g)
        mask = torch.rand(m, 512, generator=g) < 1e-3
        sign = torch.where(torch.rand(m, 512, generator=g) < 0.5, -1.0, 1.0)
        x = torch.where(mask, 200.0 * sign, x)
        ins.append(x.to(torch.bfloat16))
    scales = [(448.0 / x.float().abs().max()).reshape(1).float() for x in ins]
    t_shapes = transpose_shapes([tuple(x.shape) for x in ins], True, pad=128)
    outs = [torch.empty(x.shape, dtype=dtype) for x in ins]
    touts = [torch.empty(ts, dtype=dtype) for ts in t_shapes]
    amaxes = [torch.zeros(1) for _ in ins]
    ref.multi_cast_transpose(ins, outs, touts, scales, amaxes)
    d_outs = [torch.empty(x.shape, dtype=dtype, device=dev) for x in ins]
    d_touts = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dtype) for ts in t_shapes]
    d_amaxes = [torch.zeros(1, device=dev) for _ in ins]
    backend.multi_cast_transpose(_to_dev(ins, dev), d_outs, d_touts, _to_dev(scales, dev), d_amaxes)
    for i, m in enumerate(ms):
        assert_bytes_equal(d_outs[i], outs[i], f"cast M={m}")
        assert_bytes_equal(d_touts[i], touts[i], f"transpose M={m}")
        assert_scalar_bits_equal(d_amaxes[i], amaxes[i], f"amax M={m}")
        # unpad = row slice of the transposed-back layout (the padded layout round-trips)
        back = d_touts[i].cpu().view(torch.uint8).t()[:m]
        assert torch.equal(back, outs[i].view(torch.uint8))


def test_more_than_64_tensors_and_empty_ones(dev):
    """300 tensors in one call (the reference stops at 64), some with zero rows."""
    backend = _backend()
    g = gen(16)
    dtype = torch.float8_e4m3fn
    shapes = [((i * 7) % 40, 64 + 8 * (i % 5)) for i in range(300)]
    ins = [randn_bf16(s, g) for s in shapes]
    scales = _scales(300, g, positive=True)
    t_shapes = transpose_shapes(shapes, True)
    outs = [torch.empty(s, dtype=dtype) for s in shapes]
    touts = [torch.empty(ts, dtype=dtype) for ts in t_shapes]
    amaxes = [torch.zeros(1) for _ in shapes]
    ref.multi_cast_transpose(ins, outs, touts, scales, amaxes)
    d_outs = [torch.empty(s, dtype=dtype, device=dev) for s in shapes]
    d_touts = [torch.full(ts, 0x55, dtype=torch.uint8, device=dev).view(dtype) for ts in t_shapes]
    amax_flat = torch.zeros(300, device=dev)
    backend.multi_cast_transpose(_to_dev(ins, dev), d_outs, d_touts, torch.cat(scales).to(dev), amax_flat)
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_outs[i], outs[i], f"cast {i} {s}")
        assert_bytes_equal(d_touts[i], touts[i], f"transpose {i} {s}")
    assert_scalar_bits_equal(amax_flat, torch.cat(amaxes), "amax")

    q_outs = [torch.empty(s, dtype=dtype, device=dev) for s in shapes]
    q_amax = torch.zeros(300, device=dev)
    backend.multi_quantize(_to_dev(ins, dev), q_outs, torch.cat(scales).to(dev), q_amax)
    for i, s in enumerate(shapes):
        assert_bytes_equal(q_outs[i], outs[i], f"quantize {i} {s}")
    assert_scalar_bits_equal(q_amax, torch.cat(amaxes), "quantize amax")


def test_multi_scale_mul(dev):
    backend = _backend()
    g = gen(17)
    shapes = SMALL_SHAPES + [(3, 16384), (0, 8)]
    xs = [randn_bf16(s, g) for s in shapes]
    s1 = _scales(len(shapes), g)
    s2 = _scales(len(shapes), g)
    d_xs = _to_dev(xs, dev)
    ref.multi_scale_mul(xs, s1, s2)
    backend.multi_scale_mul(d_xs, _to_dev(s1, dev), _to_dev(s2, dev))
    for i, s in enumerate(shapes):
        assert_bytes_equal(d_xs[i], xs[i], f"scale_mul {s}")


def test_misaligned_views_take_the_scalar_path(dev):
    """Row slices that start at odd element offsets (not 16-byte aligned) must still be exact."""
    backend = _backend()
    g = gen(18)
    dtype = torch.float8_e4m3fn
    base = randn_bf16((50, 37), g)
    x = base[3:]  # offset 3 * 37 elements: 2-byte aligned only
    scale = torch.tensor([2.5])
    o, t, a = torch.empty(47, 37, dtype=dtype), torch.empty(37, 48, dtype=dtype), torch.zeros(1)
    ref.multi_cast_transpose([x.contiguous()], [o], [t], [scale], [a])
    d_base = base.to(dev)
    d_store = torch.empty(50 * 37 + 1, dtype=dtype, device=dev)
    do = d_store[1: 1 + 47 * 37].view(47, 37)  # 1-byte aligned output
    dt = torch.full((37, 48), 0x55, dtype=torch.uint8, device=dev).view(dtype)
    da = torch.zeros(1, device=dev)
    backend.multi_cast_transpose([d_base[3:]], [do], [dt], [scale.to(dev)], [da])
    assert_bytes_equal(do, o, "cast")
    assert_bytes_equal(dt, t, "transpose")
    assert_scalar_bits_equal(da, a, "amax")


@pytest.mark.parametrize("history_len,slots,margin,algo", [(1, 1, 0, "max"), (3, 4, 1, "max"), (16, 771, 0, "max"),
                                                          (5, 384, 2, "most_recent"), (1024, 6, 0, "max")])
def test_delayed_scaling_update_matches_the_torch_rule(dev, history_len, slots, margin, algo):
    """The fused update kernel against the torch statement of the rule (fp8.amax_and_scale_update on CPU
    tensors, itself checked against the oracle's Meta.update in the host tests): scale, scale_inv and the
    rolled history bit for bit, including columns whose amax is 0, inf, NaN or denormal."""
    from fp8_gmm_amd import fp8

    g = gen(41 + history_len + slots)
    hist = torch.rand(history_len, slots, generator=g) * 10.0 ** torch.randint(-6, 6, (1, slots), generator=g).float()
    specials = [0.0, float("inf"), float("nan"), 1e-42, 3.0e38, 448.0, 1.0]
    for j, v in enumerate(specials):
        if j < slots:
            hist[:, j] = 0.0 if v != v or v == float("inf") else v
            hist[(j * 7) % history_len, j] = v
    recipe = fp8.DelayedScaling(margin=margin, amax_history_len=history_len, amax_compute_algo=algo)
    cpu = fp8.Fp8MetaTensors(slots, history_len, torch.device("cpu"))
    gpu = fp8.Fp8MetaTensors(slots, history_len, dev)
    start_scale = torch.rand(slots, generator=g) + 0.5
    cpu.amax_history.copy_(hist), cpu.scale.copy_(start_scale)
    gpu.amax_history.copy_(hist), gpu.scale.copy_(start_scale)
    for step in range(3):
        fp8.amax_and_scale_update(cpu, 448.0, recipe)
        fp8.amax_and_scale_update(gpu, 448.0, recipe)
        for name in ("scale", "scale_inv", "amax_history"):
            a, b = getattr(gpu, name).cpu(), getattr(cpu, name)
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), f"{name} differs at step {step}"
        bump = torch.rand(slots, generator=g) * 3.0
        cpu.amax_history[0] += bump
        gpu.amax_history[0] += bump.to(dev)


def test_several_scaling_updates_in_one_launch_equal_one_launch_each(dev):
    """fp8gmm_delayed_scaling_updates: up to four directions in one kernel launch (a module's forward and backward
    state go together) must leave every tensor exactly as one launch per direction does: different history
    lengths and slot counts (more than one workgroup's worth, and none), margins, both amax rules, a kept
    scale_inv phase; a fifth update is refused."""
    from fp8_gmm_amd import fp8

    backend = _backend()
    g = gen(88)
    specs = [(16, 771, 448.0, 0, False, (3, 1)), (1, 5, 57344.0, 2, True, None), (7, 0, 448.0, 0, False, None),
             (1024, 130, 57344.0, 1, False, None)]
    single, together = [], []
    for history_len, slots, fp8_max, margin, recent, keep in specs:
        hist = torch.rand(history_len, slots, generator=g) * 10.0 ** torch.randint(-6, 6, (1, slots), generator=g).float()
        if slots > 3:
            hist[:, 0], hist[0, 1], hist[history_len // 2, 2] = 0.0, float("inf"), float("nan")
        scale, scale_inv = torch.rand(slots, generator=g) + 0.5, torch.rand(slots, generator=g) + 0.5
        for group in (single, together):
            group.append((hist.to(dev), scale.to(dev), scale_inv.to(dev), fp8_max, margin, recent, keep))
    for step in range(2):
        for args in single:
            backend.delayed_scaling_update(*args[:6], keep_scale_inv=args[6])
        backend.delayed_scaling_updates(together)
        for i, (a, b) in enumerate(zip(single, together)):
            for t, u, name in zip(a[:3], b[:3], ("amax_history", "scale", "scale_inv")):
                assert torch.equal(t.view(torch.int32), u.view(torch.int32)), f"update {i} {name} at step {step}"
        for a, b in zip(single, together):
            if a[0].shape[1]:
                bump = torch.rand(a[0].shape[1], generator=g).to(dev)
                a[0][0] += bump
                b[0][0] += bump
    with pytest.raises(RuntimeError):
        backend.delayed_scaling_updates(together + together[:1])


def test_tables_reach_the_device_through_the_staging_memory(dev, monkeypatch):
    """Tables are written into page-locked staging memory and copied by a kernel of the library (fp8gmm_upload).
    With the staging area shrunk to 2 x 8 KiB its halves are reused every few uploads: every device copy must hold
    its own table, also those made while earlier copies are still queued behind a long kernel, on two streams, and
    a table larger than a half goes through a buffer of its own."""
    import numpy as np

    backend = _backend()
    monkeypatch.setattr(backend._Staging, "HALF", 8192)
    monkeypatch.setattr(backend, "_staging", {})
    rng = np.random.default_rng(5)
    busy = torch.randn(4096, 4096, device=dev)
    side = torch.cuda.Stream(device=dev)
    copies = []
    for i in range(300):
        n = int(rng.choice([1, 16, 100, 1000, 3000, 8192, 20000]))
        table = rng.integers(0, 256, size=n, dtype=np.uint8)
        if i % 25 == 0:
            busy = busy @ busy * 1e-4      # keeps the stream busy, so that copies queue up behind it
        if i % 7 == 3:
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                copies.append((table, backend._upload(table, dev)))
        else:
            copies.append((table, backend._upload(table, dev)))
    torch.cuda.synchronize()
    for i, (table, on_device) in enumerate(copies):
        assert on_device.numel() == (len(table) + 15) // 16 * 16
        got = on_device.cpu().numpy()
        assert np.array_equal(got[: len(table)], table), f"upload {i} of {len(table)} bytes"
        assert not got[len(table):].any()
