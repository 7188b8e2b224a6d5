"""Benchmark of the FP8 grouped-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config2|config3|config4|config1|config5|example]

A step is one GroupedMlp (or GroupedLinear) forward + backward over one batch of synthetic,
HBM-resident input: casts / transposes / pads, the six (three) grouped GEMMs and the
delayed-scaling update.  Prints ONE JSON line.

  value     whole-step throughput in TFLOP/s: algorithmic GEMM flops of the step (unpadded rows,
            2 * sum_i M_i * N * K per grouped GEMM) / wall time of the step, timed over `--steps` steps
            with nothing else running (no per-kernel events)
  roofline  the dominant kernel (grouped GEMM): algorithmic flops per launch / mean launch
            duration from HIP events recorded around every launch during a second pass of
            `--steps` identical steps, against the dense FP8 MFMA peak of 5.0 PFLOP/s
  kernels   the same event timing for every kernel of the step (GB/s against 8 TB/s for the
            cast / transpose / pad kernels)
  parity    after the timed passes: sampled rows of every GEMM result of one more step against an fp32
            matmul (torch, on the GPU) of the dequantised fp8 operands, max |err| / max |ref| per result
  also      the step time of a later micro-batch that reuses the first one's fp8 weights (not the headline:
            the reference casts the weights on every pass), the step on the reference's buffers, one dense GEMM
            of the step's size next to the vendor library's, and - under `configs` - short passes of the other
            workloads (config 1, 3, 4 and 5 and the reference's example layer) with their own roofline fractions and parity gates
  hip_graph_replay  the step captured into a HIP graph once and replayed: its time with the host out of the way
  cpu_baseline  the per-expert quantize-dequantize-fp32-matmul loop (oracle/cpu_baseline.py) over
            the workload's own split, timed on this machine's host cores
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 MFMA
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (module, experts, hidden, ffn, tokens, splitter)
    "config1": ("linear", 4, 256, 512, 1000, "fixed"),
    "config2": ("mlp", 8, 4096, 14336, 16384, "dirichlet"),
    "config3": ("linear", 64, 2048, 1408, 24576, "zipf"),
    "config4": ("mlp", 128, 2048, 768, 65536, "uniform"),
    # the reference's own benchmark recipe (fp8_gmm/example.py:133): a routed layer, 16384 tokens, top-2 of 16
    # experts, router + gather + GroupedMlp + weighted scatter; `tokens` counts rows after routing
    "example": ("routed_mlp", 16, 4096, 6400, 32768, "router"),
}


def splits(kind, experts, tokens, seed):
    rng = np.random.default_rng(seed)
    if kind == "fixed":
        return [137, 401, 59, 403]
    if kind == "dirichlet":
        p = rng.dirichlet(np.ones(experts))
    elif kind == "zipf":
        p = 1.0 / np.arange(1, experts + 1) ** 1.1
        p /= p.sum()
    else:
        p = np.full(experts, 1.0 / experts)
    sizes = [int(v) for v in rng.multinomial(tokens, p)]
    if kind == "zipf":
        # the workload is defined by having an expert without rows and one with fewer than 16 (a Zipf draw of this
        # size rarely has either by itself): the two least popular experts hand their rows to the most popular one
        order = np.argsort(sizes, kind="stable")
        first, second, top = int(order[0]), int(order[1]), int(order[-1])
        sizes[top] += sizes[first] + sizes[second] - 7
        sizes[first], sizes[second] = 0, 7
    return sizes


def gemm_hbm_traffic(workload):
    """HBM bytes per grouped-GEMM launch (reads + writes) as the rocprofv3 FETCH_SIZE / WRITE_SIZE runs measured
    them: hardware counters cannot be read from inside this process, so the figure is taken from the committed
    summary of those runs (a line `gemm_hbm_bytes_per_launch: <number>` in profiles/<workload>_mlp_step_hbm_traffic.md)
    and is None when no such summary is at hand."""
    import glob
    import re

    for path in glob.glob(os.path.join(ROOT, "profiles", f"{workload}_*hbm_traffic.md")):
        m = re.search(r"gemm_hbm_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read())
        if m:
            return float(m.group(1))
    return None


def seeded_normal(shape, seed, std, dev, dtype=torch.bfloat16):
    """N(0, std) drawn on the CPU from numpy's seeded generator, then copied: the same bits on every machine."""
    rng = np.random.default_rng(seed)
    out = torch.empty(shape, dtype=dtype, device=dev)
    flat = out.view(-1)
    chunk = 1 << 26
    for start in range(0, flat.numel(), chunk):
        n = min(chunk, flat.numel() - start)
        vals = torch.from_numpy(rng.standard_normal(n, dtype=np.float32))
        flat[start: start + n] = (vals * std).to(dtype).to(dev)
    return out


def _fp8_cast(t, scale, dtype):
    fmax = 448.0 if dtype == torch.float8_e4m3fn else 57344.0
    return (t.float() * scale).clamp(-fmax, fmax).to(dtype)


def routed_parity_check(module, x, run_step):
    """One more step of the routed layer, then 64 sampled tokens of its output against an fp32 model of the same layer
    built from the module's bf16 parameters (same routing decisions; tanh-GELU): the relative rms error over the
    sampled block, which for two FP8 GEMMs in a row is a few per cent, and its cosine similarity."""
    from fp8_gmm_amd import moe_ops

    out, _ = run_step()
    torch.cuda.synchronize()
    tokens = torch.arange(0, x.shape[0], max(1, x.shape[0] // 64), device=x.device)[:64]
    with torch.no_grad():
        xs = x[tokens]
        weights, selected = moe_ops.topk(module.gating_network(xs), module.top_k)
        w1, w2 = module.grouped_mlp.fc1_weight, module.grouped_mlp.fc2_weight
        ref = torch.zeros(len(tokens), x.shape[1], device=x.device)
        for t in range(len(tokens)):
            for k in range(module.top_k):
                e = int(selected[t, k])
                hidden = torch.nn.functional.gelu(w1[e].float() @ xs[t].float(), approximate="tanh")
                ref[t] += weights[t, k] * (w2[e].float() @ hidden)
        got = out[tokens].float()
        rel_rms = ((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()).item()
        cos = (torch.dot(got.flatten(), ref.flatten()) / (got.norm() * ref.norm())).item()
    return {"rel_rms_err": round(rel_rms, 5), "cosine": round(cos, 6), "tolerance": {"rel_rms_err": 0.08, "cosine": 0.995},
            "ok": bool(rel_rms <= 0.08 and cos >= 0.995),
            "checked": "64 sampled tokens of the layer's output against an fp32 model of the routed layer on the bf16 "
                       "parameters (quantisation error included)"}


def parity_check(module, kind, x, dy, sizes, run_step):
    """One more step, then sampled rows of each GEMM result against torch's fp32 matmul of the dequantised fp8
    operands (the fp8 operands re-derived here with torch casts from the bf16 tensors and the scales the step
    used).  Returns {"max_rel_err": worst max|err| / max|ref| over the results, "per_result": {...}, "ok": bool}."""
    e = len(sizes)
    captured = {}
    if kind == "mlp":
        module.capture_intermediates(captured)
    out, xgrad = run_step()
    torch.cuda.synchronize()
    if kind == "mlp":
        module.capture_intermediates(None)
    fwd, bwd = module.fp8_meta["scaling_fwd"], module.fp8_meta["scaling_bwd"]
    s, si, sb, sbi = fwd.scale, fwd.scale_inv, bwd.scale, bwd.scale_inv
    E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
    bounds = np.concatenate([[0], np.cumsum(sizes)])
    live = [i for i in range(e) if sizes[i] > 0]
    picks = sorted({live[0], live[-1], max(live, key=lambda i: sizes[i])})
    errs = {}

    def note(name, got, ref):
        r = ((got.float() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
        errs[name] = max(errs.get(name, 0.0), r)

    for i in picks:
        r0, r1 = int(bounds[i]), int(bounds[i + 1])
        rows = torch.arange(r0, r1, max(1, (r1 - r0) // 48), device=x.device)[:64]
        if kind == "mlp":
            x1, w1s, x2, w2s, g1, g2 = 3 * i, 3 * i + 1, 3 * (e + i), 3 * (e + i) + 1, 2 * i, 2 * (e + i)
            w1 = _fp8_cast(module.fc1_weight.detach()[i], s[w1s], E4).float()
            w2 = _fp8_cast(module.fc2_weight.detach()[i], s[w2s], E4).float()
            x8 = _fp8_cast(x.detach()[r0:r1], s[x1], E4).float()
            dy8 = _fp8_cast(dy[r0:r1], sb[g1], E5).float()
            gelu8 = captured["gelu_out_fp8"][r0:r1].float()
            dpre8 = captured["grad_pre_fp8"][r0:r1].float()
            loc = rows - r0
            note("fc1 pre-activation", captured["pre_gelu_out"][rows], (x8[loc] @ w1.t()) * (si[x1] * si[w1s]))
            note("fc2 output", out[rows], (gelu8[loc] @ w2.t()) * (si[x2] * si[w2s]))
            note("fc2 dgrad", captured["grad_gelu_out"][rows], (dy8[loc] @ w2) * (sbi[g1] * si[w2s]))
            note("fc1 dgrad", xgrad[rows], (dpre8[loc] @ w1) * (sbi[g2] * si[w1s]))
            hs = torch.arange(0, w2.shape[0], max(1, w2.shape[0] // 48), device=x.device)[:64]
            note("fc2 wgrad", module.fc2_weight.grad[i][hs], (dy8[:, hs].t() @ gelu8) * (sbi[g1] * si[x2]))
            fs = torch.arange(0, w1.shape[0], max(1, w1.shape[0] // 48), device=x.device)[:64]
            note("fc1 wgrad", module.fc1_weight.grad[i][fs], (dpre8[:, fs].t() @ x8) * (sbi[g2] * si[x1]))
        else:
            xs, ws, g1 = 3 * i, 3 * i + 1, 2 * i
            w = _fp8_cast(module.weight_tensor.detach()[i], s[ws], E4).float()
            x8 = _fp8_cast(x.detach()[r0:r1], s[xs], E4).float()
            dy8 = _fp8_cast(dy[r0:r1], sb[g1], E5).float()
            loc = rows - r0
            note("output", out[rows], (x8[loc] @ w.t()) * (si[xs] * si[ws]))
            note("dgrad", xgrad[rows], (dy8[loc] @ w) * (sbi[g1] * si[ws]))
            ns = torch.arange(0, w.shape[0], max(1, w.shape[0] // 48), device=x.device)[:64]
            note("wgrad", module.weight_tensor.grad[i][ns], (dy8[:, ns].t() @ x8) * (sbi[g1] * si[xs]))
    worst = max(errs.values())
    return {"max_rel_err": float(f"{worst:.3e}"), "tolerance": 1e-2, "ok": bool(worst <= 1e-2),
            "per_result": {k: float(f"{v:.3e}") for k, v in errs.items()},
            "checked": f"64 sampled rows of experts {picks} against torch fp32 matmul of the dequantised fp8 operands"}


def sample_shader_clock(work):
    """Runs work() while a thread reads, about once per millisecond, the current shader clock (MHz, pp_dpm_sclk)
    and board power (W, hwmon power1_input) that the driver publishes in sysfs.  Returns (clock samples, power
    samples, power cap in W or None), keeping only what was read while the GPU was out of its idle state; empty
    lists where the nodes cannot be read."""
    import glob
    import re
    import threading

    clk_nodes = glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")
    pwr_nodes = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
    cap_nodes = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap")
    clocks, watts, stop = [], [], threading.Event()

    def read(node):
        try:
            with open(node) as f:
                return f.read()
        except OSError:
            return ""

    def reader():
        while not stop.is_set():
            busy = False
            for node in clk_nodes:
                m = re.search(r"(\d+)\s*Mhz\s*\*", read(node), re.IGNORECASE)
                if m and int(m.group(1)) >= 400:
                    clocks.append(int(m.group(1)))
                    busy = True
            if busy:
                for node in pwr_nodes:
                    txt = read(node).strip()
                    if txt.isdigit():
                        watts.append(int(txt) / 1e6)
            time.sleep(0.001)

    cap = None
    for node in cap_nodes:
        txt = read(node).strip()
        if txt.isdigit():
            cap = int(txt) / 1e6
    if not clk_nodes:
        return [], [], cap
    torch.cuda.synchronize()
    t = threading.Thread(target=reader, daemon=True)
    t.start()
    try:
        work()
        torch.cuda.synchronize()
    finally:
        stop.set()
        t.join()
    return clocks, watts, cap


def measure_cast_pad(args):
    """config5: the bandwidth-bound path alone - ONE multi-tensor cast + transpose + amax + pad-to-128 launch over
    8 bf16 activation tensors [M_i, 4096], M_i uniform in [1, 8191], N(0, 1) values with 0.1 % outliers at +-200.
    Returns the JSON line as a dict."""
    import fp8_gmm_amd as pkg  # noqa: F401  (loads the library)
    from fp8_gmm_amd import backend
    from fp8_gmm_amd.backend import kernel_timing

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1005)
    rows = [int(v) for v in rng.integers(1, 8192, size=8)]
    cols, pad = 4096, 128
    ins, outs, touts, scales = [], [], [], []
    for m in rows:   # drawn on the CPU from the workload's seed and copied: the same bits on every machine
        vals = rng.standard_normal((m, cols), dtype=np.float32)
        hit = rng.random((m, cols), dtype=np.float32) < 1e-3
        vals[hit] = np.where(rng.random(int(hit.sum())) < 0.5, -200.0, 200.0)
        x = torch.from_numpy(vals).to(torch.bfloat16).to(dev)
        ins.append(x)
        outs.append(torch.empty(m, cols, dtype=torch.float8_e4m3fn, device=dev))
        touts.append(torch.empty(cols, (m + pad - 1) // pad * pad, dtype=torch.float8_e4m3fn, device=dev))
        scales.append((448.0 / x.float().abs().max()).reshape(1))
    amaxes = torch.zeros(len(rows), device=dev)
    nbytes = sum(cols * (3 * m + (m + pad - 1) // pad * pad) for m in rows)

    def step():
        backend.multi_cast_transpose(ins, outs, touts, scales, amaxes)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    with kernel_timing() as timing:   # a pass of its own: the events around every launch cost the stream a few us each
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
    d = timing.summary()["multi_pad_cast_transpose"]
    replay = None if args.no_graph else graph_replay(step, args.steps)
    if replay is not None and "ms_per_step" in replay:
        replay["GB/s"] = round(nbytes / (replay["ms_per_step"] * 1e-3) / 1e9, 1)
    ach = d["work"] / (d["ms"] * 1e-3) / 1e9
    # correctness gate: the transposed copy is the padded transpose of the row-major copy, both are the bytes torch's
    # own saturating cast gives, and amax is max|x|, for every tensor
    ok = True
    for x, o, t, sc, am in zip(ins, outs, touts, scales, amaxes.tolist()):
        want = (x.float() * sc).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
        m = x.shape[0]
        ok = ok and torch.equal(o.view(torch.uint8), want) and torch.equal(t.view(torch.uint8)[:, :m], want.t()) \
            and not bool(t.view(torch.uint8)[:, m:].any()) and am == x.float().abs().max().item()
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import ref

        m = 2048
        x = ins[0][: min(m, rows[0])].cpu().contiguous() if rows[0] >= m else torch.randn(m, cols).to(torch.bfloat16)
        m = x.shape[0]
        o = torch.empty(m, cols, dtype=torch.float8_e4m3fn)
        t = torch.empty(cols, (m + pad - 1) // pad * pad, dtype=torch.float8_e4m3fn)
        a = torch.zeros(1)
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0:
            ref.multi_cast_transpose([x], [o], [t], [scales[0].cpu()], [a])
            reps += 1
        secs = time.perf_counter() - t0
        cpu = {"value": round(reps * cols * (3 * m + t.shape[1]) / secs / 1e9, 3), "unit": "GB/s", "cores": 1,
               "kind": "port", "sample": f"{reps} casts of one [{m}, {cols}] tensor by the scalar C oracle, {secs:.1f} s"}
    return {
        "metric": "cast + transpose + amax + pad GB/s, % of MI355X HBM bandwidth (8 activation tensors)",
        "value": round(nbytes / (ms_per_step * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16->fp8", "data": "synthetic",
        "config": {"workload": "config5: multi_cast_transpose over 8 x [M_i, 4096] bf16, pad 128, e4m3, "
                               "0.1 % outliers at +-200", "rows": rows, "bytes_per_step": nbytes},
        "roofline": {"kernel": "multi_pad_kernel<cast+transpose>", "bound": "hbm", "achieved": round(ach, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel_us": round(d["ms"] * 1e3, 1)},
        "wall_clock_per_call": {"us": round(ms_per_step * 1e3, 1), "GB/s": round(nbytes / (ms_per_step * 1e-3) / 1e9, 1),
                                "frac_of_hbm_peak": round(nbytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        "hip_graph_replay": replay,
        "parity": {"ok": bool(ok), "checked": "all bytes of both copies against torch's saturating e4m3 cast, zero "
                                              "padding, amax == max|x|, all 8 tensors"},
        "cpu_baseline": cpu,
    }


def dense_gemm_comparison(dev, m, n, k, reps=100):
    """[m, k] x [n, k]^T -> bf16 [m, n], e4m3 operands: TFLOP/s of the grouped kernel (one group) and of the vendor GEMM."""
    import fp8_gmm_amd.backend as backend

    def quantized(t):
        return (t * (448.0 / t.abs().max())).to(torch.float8_e4m3fn)

    a = quantized(torch.randn(m, k, device=dev))
    b = quantized(torch.randn(n, k, device=dev))
    c = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
    one = torch.ones(1, device=dev)
    sizes = torch.tensor([m])

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    flops = 2.0 * m * n * k
    out = {"shape": [m, n, k], "data": "N(0, 1) scaled to amax 448"}
    mine, vendor = [], []
    for _ in range(2):
        mine.append(timed(lambda: backend.fp8_gmm(a, b.view(1, n, k), sizes, one, one, c)))
        try:
            vendor.append(timed(lambda: torch._scaled_mm(a, b.t(), scale_a=one[0], scale_b=one[0],
                                                         out_dtype=torch.bfloat16, out=c)))
        except Exception as exc:  # the private torch entry point may change; the comparison is optional
            out["vendor_error"] = repr(exc)[:200]
    out["this_kernel_tflops"] = round(flops / min(mine) / 1e12, 1)
    if vendor:
        out["torch_scaled_mm_tflops"] = round(flops / min(vendor) / 1e12, 1)
    # The same launches on operands that toggle no bits: the board is at its power cap on random data, and what
    # the kernels gain here is what the cap costs them there.
    a.view(torch.uint8).zero_()
    b.view(torch.uint8).zero_()
    out["all_zero_operands"] = {"this_kernel_tflops": round(
        flops / timed(lambda: backend.fp8_gmm(a, b.view(1, n, k), sizes, one, one, c)) / 1e12, 1)}
    if vendor:
        try:
            out["all_zero_operands"]["torch_scaled_mm_tflops"] = round(flops / timed(
                lambda: torch._scaled_mm(a, b.t(), scale_a=one[0], scale_b=one[0], out_dtype=torch.bfloat16,
                                         out=c)) / 1e12, 1)
        except Exception as exc:
            out["vendor_error"] = repr(exc)[:200]
    return out


def measure_module(args):
    """One module workload (WORKLOADS[args.workload]): returns the JSON line as a dict."""
    import fp8_gmm_amd as pkg
    from fp8_gmm_amd.backend import kernel_timing

    kind, experts, hidden, ffn, tokens, splitter = WORKLOADS[args.workload]
    idx = int(args.workload[-1]) if args.workload[-1].isdigit() else 9
    seed = 1000 + idx
    sizes = splits(splitter, experts, tokens, seed) if splitter != "router" else None
    dev = torch.device("cuda:0")
    torch.manual_seed(seed)
    top_k = 2
    if kind == "routed_mlp":
        from fp8_gmm_amd.moe import Fp8MlpModule

        module = Fp8MlpModule(hidden, ffn, experts, top_k, device=dev)
        out_features, gemms = hidden, 6
    elif kind == "mlp":
        module = pkg.GroupedMlp(hidden, ffn, experts, torch.bfloat16, device=dev)
        module.fc1_weight.data.copy_(seeded_normal(module.fc1_weight.shape, seed + 100, 0.02, dev))
        module.fc2_weight.data.copy_(seeded_normal(module.fc2_weight.shape, seed + 200, 0.02, dev))
        out_features, gemms = hidden, 6
    else:
        module = pkg.GroupedLinear(hidden, ffn, experts, torch.bfloat16, device=dev)
        module.weight_tensor.data.copy_(seeded_normal(module.weight_tensor.shape, seed + 100, 0.02, dev))
        out_features, gemms = ffn, 3
    in_rows = tokens // top_k if kind == "routed_mlp" else tokens
    # inputs are drawn on the CPU from the workload's seed and copied, so every run sees the same bits
    x = seeded_normal((in_rows, hidden), seed + 300, 1.0, dev).requires_grad_()
    dy = seeded_normal((in_rows, out_features), seed + 400, 1e-2, dev)
    gs = torch.tensor(sizes, dtype=torch.int64) if sizes is not None else None
    fp8_recipe = pkg.DelayedScaling(amax_history_len=16)
    flops_per_gemm = 2.0 * tokens * hidden * ffn
    flops_per_step = gemms * flops_per_gemm

    def step(first=None):
        module.zero_grad(set_to_none=True)
        x.grad = None
        with pkg.fp8_autocast(enabled=True, fp8_recipe=fp8_recipe):
            out = module(x) if gs is None else module(x, gs, is_first_microbatch=first)
        out.backward(dy)
        return out, x.grad

    from fp8_gmm_amd import backend

    backend.warm_up(dev)   # library initialisation and the GEMM's workspace: not inside the timed region

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # the same steps again, with HIP events around every kernel launch: per-kernel durations
    timing = None
    if not args.no_kernel_events:
        with kernel_timing() as timing:
            for _ in range(args.steps):
                step()
            torch.cuda.synchronize()
    ms_per_step = elapsed / args.steps * 1e3
    value = flops_per_step / (ms_per_step * 1e-3) / 1e12

    roofline = None
    kernels = {}
    if timing is not None:
        summ = timing.summary()
        for name, d in summ.items():
            if name == "grouped_gemm":
                ach = flops_per_gemm / (d["ms"] * 1e-3) / 1e12
                alg_gbs = d["bytes"] / (d["ms"] * 1e-3) / 1e9
                kernels[name] = {"launches_per_step": d["launches"] / args.steps, "ms": round(d["ms"], 4),
                                 "tflops": round(ach, 1), "frac_of_mfma_peak": round(ach / FP8_PEAK_TFLOPS, 4),
                                 "algorithmic_bytes_per_launch": round(d["bytes"]),
                                 "algorithmic_GBps": round(alg_gbs, 1),
                                 "frac_of_hbm_peak": round(alg_gbs / HBM_PEAK_GBS, 4),
                                 "by_form": {form: {
                                     "launches_per_step": c["launches"] / args.steps, "ms": round(c["ms"], 4),
                                     "frac_of_mfma_peak": round(c["work"] / (c["ms"] * 1e-3) / 1e12 / FP8_PEAK_TFLOPS, 4),
                                     "frac_of_hbm_peak": round(c["bytes"] / (c["ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
                                     for form, c in sorted(d.get("forms", {}).items())}}
                traffic = gemm_hbm_traffic(args.workload)
                roofline = {"kernel": "grouped_gemm_kernel", "bound": "mfma", "achieved": round(ach, 1),
                            "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / FP8_PEAK_TFLOPS, 4),
                            "traffic": traffic,
                            "timed_over": f"a second pass of {args.steps} identical steps with HIP events around "
                                          "every launch"}
                if traffic is not None:
                    # the same launches seen from the memory side: short contractions (configs 3 and 4) move
                    # almost as many bytes per flop as the memory system can deliver
                    gbs = traffic / (d["ms"] * 1e-3) / 1e9
                    roofline["memory_side"] = {"GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
            else:
                gbs = d["work"] / (d["ms"] * 1e-3) / 1e9
                kernels[name] = {"launches_per_step": d["launches"] / args.steps, "ms": round(d["ms"], 4),
                                 "GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}

    # Shader clock under this workload, from the driver's sysfs node (what rocm-smi --showclocks prints), sampled
    # by a thread during a separate pass of 40 steps.  The 5.0 PFLOP/s MFMA peak assumes the 2.4 GHz maximum:
    # 256 CUs x 8192 flop per clock.
    clock = None
    mhz, watts, cap = ([], [], None) if args.headline_only else sample_shader_clock(
        lambda: [step() for _ in range(40)])
    if mhz and roofline is not None:
        mean = sum(mhz) / len(mhz)
        clock = {"driver_reported": {"shader_mhz_mean": round(mean, 1), "shader_mhz_min": min(mhz),
                                     "shader_mhz_max": max(mhz), "samples": len(mhz),
                                     "board_power_w_mean": round(sum(watts) / len(watts), 1) if watts else None,
                                     "board_power_w_max": max(watts) if watts else None, "board_power_cap_w": cap,
                                     "source": "pp_dpm_sclk and hwmon power1_input (sysfs), 1 ms period, over 40 "
                                               "extra steps"}}
    # Not the headline: the same step as a micro-batch after the first of an optimizer step, reusing the fp8
    # weights cast by the first (is_first_microbatch=False), which the reference stubs out.
    also = None
    if gs is not None and not args.headline_only:
        step(True)
        step(False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(False)
        torch.cuda.synchronize()
        cached_ms = (time.perf_counter() - t0) / args.steps * 1e3
        also = {"later_microbatch_with_cached_fp8_weights": {
            "ms_per_step": round(cached_ms, 4), "value": round(flops_per_step / (cached_ms * 1e-3) / 1e12, 2),
            "unit": "TFLOP/s"}}

    # ... and the same step on the reference's buffers (transposed fp8 weights, padded transposed activations and
    # gradients, written by the pad / cast / transpose kernels), which the default path no longer needs
    if gs is not None and not args.headline_only:
        ref_module = type(module)(hidden, ffn, experts, torch.bfloat16, device=dev, reference_layout=True)
        ref_module.load_state_dict(module.state_dict())
        main_module, module = module, ref_module
        try:
            for _ in range(3):
                step()
            torch.cuda.synchronize()
            with kernel_timing() as rt:
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    step()
                torch.cuda.synchronize()
                ref_ms = (time.perf_counter() - t0) / args.steps * 1e3
            ref_kernels = {name: {"launches_per_step": d["launches"] / args.steps, "ms": round(d["ms"], 4),
                                  "GBps": round(d["work"] / (d["ms"] * 1e-3) / 1e9, 1)}
                           for name, d in rt.summary().items() if name != "grouped_gemm"}
        finally:
            module = main_module
        del ref_module
        also = dict(also or {})
        also["reference_layout"] = {"ms_per_step": round(ref_ms, 4),
                                    "value": round(flops_per_step / (ref_ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                                    "kernels": ref_kernels}

    # ... and, for scale, one dense e4m3 GEMM of the step's size (all tokens as one group, tokens x ffn x hidden)
    # through this library's kernel and through the vendor library behind torch._scaled_mm, on the same Gaussian
    # operands scaled to the fp8 range, timed alternately
    if args.workload == "config2" and not args.headline_only:
        also = dict(also or {})
        also["dense_gemm_of_the_same_size"] = dense_gemm_comparison(dev, tokens, ffn, hidden)

    # the step as a HIP graph: one capture, then replays (host-bound workloads are the ones that gain)
    captured = None
    if gs is not None and not args.no_graph:
        captured = graph_replay(step, args.steps)
        if "ms_per_step" in captured:
            captured["value"] = round(flops_per_step / (captured["ms_per_step"] * 1e-3) / 1e12, 2)
            captured["unit"] = "TFLOP/s"

    # correctness gate, after everything that is timed
    parity = None
    if gs is not None and not args.no_parity:
        parity = parity_check(module, kind, x, dy, sizes, step)
    elif kind == "routed_mlp" and not args.no_parity:
        parity = routed_parity_check(module, x, step)

    cpu = None
    if not args.no_cpu_baseline:
        from oracle import cpu_baseline

        cores = torch.get_num_threads()
        cpu_baseline.mlp_step_sample(64, hidden, ffn)  # warm-up of the thread pool
        # the same per-expert loop the reference's test oracle walks, over this workload's split; for workloads
        # whose split the router decides, or with many experts, one expert's share of the tokens per expert
        cpu_sizes = sizes if sizes is not None and experts <= 16 else [tokens // 8] * 8
        secs, fl = cpu_baseline.mlp_step_grouped(cpu_sizes, hidden, ffn)
        cpu = {"value": round(fl / secs / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": f"per-expert loop over the split {cpu_sizes}: quantize -> dequantize -> fp32 matmul, "
                         f"{hidden}->{ffn} MLP fwd+bwd (6 GEMMs per expert, {fl / 1e9:.0f} GFLOP in all) incl. every "
                         f"expert's weight quantisation, {secs:.1f} s"}

    names = {"mlp": "GroupedMlp", "linear": "GroupedLinear", "routed_mlp": "Fp8MlpModule (router, gather, GroupedMlp, scatter)"}
    line = {
        "metric": f"FP8 grouped-GEMM TFLOP/s fwd+bwd, % of MI355X FP8 MFMA peak, E={experts} MoE "
                  f"{'MLP' if kind != 'linear' else 'Linear'}" + (" (routed layer)" if kind == "routed_mlp" else ""),
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "pct_of_fp8_mfma_peak": round(100.0 * value / FP8_PEAK_TFLOPS, 2),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {names[kind]} fwd+bwd, E={experts}, "
                               f"hidden={hidden}, ffn={ffn}, tokens={tokens}, split={splitter}",
                   "group_sizes": "decided by the router" if sizes is None else
                                  sizes if experts <= 16 else f"{experts} experts, min {min(sizes)} max {max(sizes)}",
                   "gemm_flops_per_step": flops_per_step},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "parity": parity,
        "kernels": kernels,
        "clock": clock,
        "hip_graph_replay": captured,
        "also": also,
    }
    return line


def graph_replay(step, steps):
    """The same step captured into a HIP graph once and replayed: what is left of the step when the host does nothing
    but start the graph (the tables of the captured launches stay in page-locked memory of their own and are copied
    again by every replay).  Returns the replay time, or the reason why the capture failed."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):   # a step on the capture's side of things first: workspaces, allocator pools
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        torch.cuda.synchronize()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        del graph
        return {"ms_per_step": round(ms, 4)}
    except Exception as exc:   # a record without this entry is still a record
        return {"error": repr(exc)[:300]}


def short_pass(args, workload):
    """A short pass of another workload for the `also.configs` record: step time, the GEMM against both roofs, the
    cast kernels against the HBM roof, and the workload's own parity gate."""
    import copy
    import gc

    a = copy.copy(args)
    a.workload = workload   # the same step and warm-up counts as the headline: these steps take 0.1 - 1.5 ms
    a.no_cpu_baseline, a.headline_only, a.copy_calibration, a.no_kernel_events = True, True, False, False
    line = measure_cast_pad(a) if workload == "config5" else measure_module(a)
    gc.collect()
    torch.cuda.empty_cache()
    keep = ("value", "unit", "ms_per_step", "steps", "config", "roofline", "kernels", "parity", "wall_clock_per_call",
            "hip_graph_replay")
    return {k: line[k] for k in keep if line.get(k) is not None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="config2", choices=sorted(WORKLOADS) + ["config5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-events", action="store_true", help="skip the second pass with per-kernel HIP events")
    ap.add_argument("--no-parity", action="store_true", help="skip the correctness gate after the timed passes")
    ap.add_argument("--no-graph", action="store_true", help="skip the pass that captures the step into a HIP graph")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the extra passes after the timed region (clock / power sampling, cached-weights "
                         "step, the HIP-graph replays, the other workloads): what a profiler should see")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 256 MiB device copy (reads 256 MiB, writes 256 MiB) so that hardware "
                         "byte counters collected around this command can be scaled against a known transfer")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); multi-GPU runs are not part of it")
    if args.headline_only:
        args.no_graph = True   # a profiler should see the timed steps, not their replays
    if args.workload == "config5":
        print(json.dumps(measure_cast_pad(args)))
        return
    line = measure_module(args)
    if args.workload == "config2" and not args.headline_only:
        # every other workload in the same record: short passes, each with its own correctness gate
        gc_configs = {}
        for w in ("config1", "config3", "config4", "config5", "example"):
            gc_configs[w] = short_pass(args, w)
        line["also"] = dict(line.get("also") or {})
        line["also"]["configs"] = gc_configs
    print(json.dumps(line))


if __name__ == "__main__":
    main()
