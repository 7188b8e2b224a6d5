"""CPU oracle of the grouped modules' forward + backward data flow.  TEST INFRASTRUCTURE ONLY.

Restates, with the byte-exact primitives of :mod:`oracle.ref`, what the reference's autograd
functions compute (fp8_gmm/grouped_linear.py:11-183, fp8_gmm/grouped_mlp.py:18-325) and the
delayed-scaling bookkeeping they rely on (slot layout fp8_gmm/utils.py:66-67,98-103).  The slot
arithmetic is written out independently of the product's ``Fp8MetaWrapper``:

    forward  tensors: 3 slots per GEMM -> slot(gemm, kind) = 3 * gemm + kind, kind 0 input, 1 weight
    backward tensors: 2 slots per GEMM -> slot(gemm)       = 2 * gemm            (grad_output)
    GroupedLinear: gemm = expert;  GroupedMlp: fc1 gemm = expert, fc2 gemm = E + expert

Parity status: the per-op arithmetic is pinned through oracle.ref; the delayed-scaling update
rule restated in :class:`Meta` comes from TransformerEngine, which is not available here
-> parity unpinned for the rule itself (the product states the same rule).
"""
import torch

from . import ref

FP8_MAX = ref.FP8_MAX


class Meta:
    """scale / scale_inv / amax history of one direction, on the CPU."""

    def __init__(self, slots, history_len):
        self.scale = torch.ones(slots, dtype=torch.float32)
        self.scale_inv = torch.ones(slots, dtype=torch.float32)
        self.amax_history = torch.zeros(history_len, slots, dtype=torch.float32)

    def update(self, fp8_max, margin=0, algo="max", keep_scale_inv=()):
        """keep_scale_inv: slots whose scale_inv stays as it is (weights whose cached fp8 copy is reused)."""
        hist = self.amax_history
        amax = hist.max(dim=0).values if algo == "max" else hist[0].clone()
        sf = (fp8_max / amax) / (2.0 ** margin)
        ok = (amax > 0) & torch.isfinite(amax)
        self.scale = torch.where(ok, sf, self.scale).to(torch.float32)
        old_inv = self.scale_inv
        self.scale_inv = (1.0 / self.scale).to(torch.float32)
        for slot in keep_scale_inv:
            self.scale_inv[slot] = old_inv[slot]
        if hist.shape[0] > 1:
            self.amax_history = torch.roll(hist, -1, 0)
        self.amax_history[0].zero_()

    def amax(self, slot):
        return self.amax_history[0][slot: slot + 1]


def _bounds(sizes, pad=None):
    out = [0]
    for s in sizes:
        out.append(out[-1] + ((s + pad - 1) // pad * pad if pad else s))
    return out


def _cast_rows(x, sizes, slots, meta, dtype, pad=16):
    """Per-expert cast (+ padded transpose) of a token-major bf16 tensor. Returns (fp8 [M, K], [fp8 [K, Mpad_i]])."""
    b = _bounds(sizes)
    out = torch.empty(x.shape, dtype=dtype)
    ts = []
    for i, s in enumerate(sizes):
        mp = (s + pad - 1) // pad * pad
        t = torch.empty(x.shape[1], mp, dtype=dtype)
        xi = x[b[i]: b[i + 1]].contiguous()
        oi = torch.empty(xi.shape, dtype=dtype)
        ref.multi_cast_transpose([xi], [oi], [t], [meta.scale[slots[i]: slots[i] + 1]], [meta.amax(slots[i])])
        out[b[i]: b[i + 1]] = oi
        ts.append(t)
    return out, ts


def _cast_weights(w, slots, meta, dtype):
    e = w.shape[0]
    out = torch.empty(w.shape, dtype=dtype)
    out_t = torch.empty(e, w.shape[2], w.shape[1], dtype=dtype)
    for i in range(e):
        ref.multi_cast_transpose([w[i].contiguous()], [out[i]], [out_t[i]], [meta.scale[slots[i]: slots[i] + 1]],
                                 [meta.amax(slots[i])])
    return out, out_t


def _gmm_bf16(a, b, sizes, a_inv, b_inv):
    c = torch.zeros(a.shape[0], b.shape[1], dtype=torch.bfloat16)
    ref.fp8_gmm(a, b, sizes, a_inv, b_inv, c)
    return c


def _wgrad(g_ts, x_ts, g_inv, x_inv):
    outs = []
    for gt, xt, gi, xi in zip(g_ts, x_ts, g_inv, x_inv):
        c = torch.zeros(gt.shape[0], xt.shape[0], dtype=torch.bfloat16)
        ref.cublas_fp8_gemm(gt, xt, c, gi, xi)
        outs.append(c)
    return torch.stack(outs)


def grouped_linear_step(x, w, sizes, dy, fwd, bwd, fwd_dtype=torch.float8_e4m3fn, bwd_dtype=torch.float8_e5m2,
                        cached=None):
    """One forward + backward of GroupedLinear with the scales currently in ``fwd`` / ``bwd``.

    Records amaxes into the metas (history row 0), returns out, grad_input, grad_weight and the fp8
    intermediates.  x [M, K] bf16, w [E, N, K] bf16, dy [M, N] bf16.  ``cached``: the result of an earlier
    step whose fp8 weights are reused instead of casting ``w`` (a micro-batch after the first).
    """
    e = len(sizes)
    xs = [3 * i for i in range(e)]
    ws = [3 * i + 1 for i in range(e)]
    gs = [2 * i for i in range(e)]
    x_fp8, x_ts = _cast_rows(x, sizes, xs, fwd, fwd_dtype)
    w_fp8, w_t_fp8 = (cached["w_fp8"], cached["w_t_fp8"]) if cached else _cast_weights(w, ws, fwd, fwd_dtype)
    out = _gmm_bf16(x_fp8, w_fp8, sizes, [fwd.scale_inv[s] for s in xs], [fwd.scale_inv[s] for s in ws])
    fwd_inv = fwd.scale_inv.clone()  # the copy the backward pass dequantises with (utils.py:77-78)
    dy_fp8, dy_ts = _cast_rows(dy, sizes, gs, bwd, bwd_dtype)
    g_inv = [bwd.scale_inv[s] for s in gs]
    grad_input = _gmm_bf16(dy_fp8, w_t_fp8, sizes, g_inv, [fwd_inv[s] for s in ws])
    grad_weight = _wgrad(dy_ts, x_ts, g_inv, [fwd_inv[s] for s in xs])
    return dict(out=out, grad_input=grad_input, grad_weight=grad_weight, x_fp8=x_fp8, x_ts=x_ts, w_fp8=w_fp8,
                w_t_fp8=w_t_fp8, dy_fp8=dy_fp8, dy_ts=dy_ts)


def grouped_mlp_step(x, w1, w2, sizes, dy, fwd, bwd, fwd_dtype=torch.float8_e4m3fn, bwd_dtype=torch.float8_e5m2,
                     cached=None, given=None, fused_dgelu=False):
    """One forward + backward of GroupedMlp. x [M, H], w1 [E, F, H], w2 [E, H, F], dy [M, H].
    ``cached``: the result of an earlier step whose fp8 weights are reused.

    ``given``: intermediates of another implementation's run of the same step (any of ``pre``, ``gelu_fp8``,
    ``grad_gelu``, ``dpre_fp8``).  A given tensor replaces this function's own from the point where it is
    produced, so that everything downstream is computed from identical bytes and can be compared GEMM by GEMM;
    this function's own values are returned beside them under ``own_*`` (the amax it records stays its own).

    ``fused_dgelu``: d(pre-GELU) is formed in the epilogue of the fc2 data-gradient GEMM, from the fp32 result
    (no bf16 d(GELU output): ``grad_gelu`` is None), as GroupedMlp(fused_dgelu=True) does."""
    given = given or {}
    e = len(sizes)
    b = _bounds(sizes)
    x1 = [3 * i for i in range(e)]
    w1s = [3 * i + 1 for i in range(e)]
    x2 = [3 * (e + i) for i in range(e)]
    w2s = [3 * (e + i) + 1 for i in range(e)]
    g1 = [2 * i for i in range(e)]
    g2 = [2 * (e + i) for i in range(e)]
    m, ffn = x.shape[0], w1.shape[1]

    x_fp8, x_ts = _cast_rows(x, sizes, x1, fwd, fwd_dtype)
    if cached:
        w1_fp8, w1_t, w2_fp8, w2_t = (cached[k] for k in ("w1_fp8", "w1_t_fp8", "w2_fp8", "w2_t_fp8"))
    else:
        w1_fp8, w1_t = _cast_weights(w1, w1s, fwd, fwd_dtype)
        w2_fp8, w2_t = _cast_weights(w2, w2s, fwd, fwd_dtype)
    pre = torch.zeros(m, ffn, dtype=torch.bfloat16)
    gelu_fp8 = torch.zeros(m, ffn, dtype=fwd_dtype)
    ref.fp8_gmm(x_fp8, w1_fp8, sizes, [fwd.scale_inv[s] for s in x1], [fwd.scale_inv[s] for s in w1s], gelu_fp8,
                fwd_dtype, pre, [fwd.scale[s: s + 1] for s in x2], [fwd.amax(s) for s in x2])
    own = dict(own_pre=pre, own_gelu_fp8=gelu_fp8)
    pre = given.get("pre", pre)
    gelu_fp8 = given.get("gelu_fp8", gelu_fp8)
    out = _gmm_bf16(gelu_fp8, w2_fp8, sizes, [fwd.scale_inv[s] for s in x2], [fwd.scale_inv[s] for s in w2s])
    fwd_inv = fwd.scale_inv.clone()

    dy_fp8, dy_ts = _cast_rows(dy, sizes, g1, bwd, bwd_dtype)
    g1_inv = [bwd.scale_inv[s] for s in g1]
    gelu_ts = []
    for i, s in enumerate(sizes):
        mp = (s + 15) // 16 * 16
        t = torch.empty(ffn, mp, dtype=fwd_dtype)
        ref.multi_transpose([gelu_fp8[b[i]: b[i + 1]].contiguous()], [t])
        gelu_ts.append(t)
    grad_w2 = _wgrad(dy_ts, gelu_ts, g1_inv, [fwd_inv[s] for s in x2])
    dpre_fp8 = torch.empty(m, ffn, dtype=bwd_dtype)
    dpre_ts = []
    if fused_dgelu:
        grad_gelu = None
        ref.fp8_gmm(dy_fp8, w2_t, sizes, g1_inv, [fwd_inv[s] for s in w2s], dpre_fp8, bwd_dtype, None,
                    [bwd.scale[s: s + 1] for s in g2], [bwd.amax(s) for s in g2], dgelu_pre=pre)
        for i, s in enumerate(sizes):
            t = torch.empty(ffn, (s + 15) // 16 * 16, dtype=bwd_dtype)
            ref.multi_transpose([dpre_fp8[b[i]: b[i + 1]].contiguous()], [t])
            dpre_ts.append(t)
    else:
        grad_gelu = _gmm_bf16(dy_fp8, w2_t, sizes, g1_inv, [fwd_inv[s] for s in w2s])
        own["own_grad_gelu"] = grad_gelu
        grad_gelu = given.get("grad_gelu", grad_gelu)
        for i, s in enumerate(sizes):
            mp = (s + 15) // 16 * 16
            t = torch.empty(ffn, mp, dtype=bwd_dtype)
            o = torch.empty(s, ffn, dtype=bwd_dtype)
            ref.multi_cast_transpose_dgelu([grad_gelu[b[i]: b[i + 1]].contiguous()], [pre[b[i]: b[i + 1]].contiguous()],
                                           [o], [t], [bwd.scale[g2[i]: g2[i] + 1]], [bwd.amax(g2[i])])
            dpre_fp8[b[i]: b[i + 1]] = o
            dpre_ts.append(t)
    own["own_dpre_fp8"] = dpre_fp8
    if "dpre_fp8" in given:
        dpre_fp8 = given["dpre_fp8"]
        dpre_ts = []
        for i, s in enumerate(sizes):
            t = torch.empty(ffn, (s + 15) // 16 * 16, dtype=bwd_dtype)
            ref.multi_transpose([dpre_fp8[b[i]: b[i + 1]].contiguous()], [t])
            dpre_ts.append(t)
    g2_inv = [bwd.scale_inv[s] for s in g2]
    grad_input = _gmm_bf16(dpre_fp8, w1_t, sizes, g2_inv, [fwd_inv[s] for s in w1s])
    grad_w1 = _wgrad(dpre_ts, x_ts, g2_inv, [fwd_inv[s] for s in x1])
    return dict(own, out=out, grad_input=grad_input, grad_w1=grad_w1, grad_w2=grad_w2, pre=pre, gelu_fp8=gelu_fp8,
                grad_gelu=grad_gelu, dpre_fp8=dpre_fp8, w1_fp8=w1_fp8, w1_t_fp8=w1_t, w2_fp8=w2_fp8, w2_t_fp8=w2_t)
