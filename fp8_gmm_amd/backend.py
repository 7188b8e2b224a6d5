"""Python entry points of the MI355X FP8 grouped-GEMM backend.

Same names, positional signatures and meaning as the reference's
``fp8_gmm/backend.py`` (``multi_quantize`` :9, ``multi_transpose`` :13,
``multi_cast_transpose`` :17, ``multi_cast_transpose_dgelu`` :21,
``cublas_fp8_gemm`` :26, ``fp8_gmm`` :58), plus ``multi_scale_mul`` (pybind name in
csrc/ops.cu:12) and ``grouped_gemm``, the list form the wgrad path uses.  Every
function validates its arguments like the reference's TORCH_CHECKs, builds a
descriptor table, has the C library plan it, uploads it through pinned memory on
the current stream and enqueues ONE kernel.  Nothing here computes on the CPU and
there is no fallback: without the HIP library the import fails.
"""
import numpy as np
import torch

from . import _lib
from ._lib import GEMM_PROBLEM, TENSOR_DESC

_lib.load()  # fail at import time, loudly, when the extension is missing

_FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)
_FMT = {torch.float8_e4m3fn: _lib.E4M3, torch.float8_e5m2: _lib.E5M2}
_OUT_KIND = {torch.bfloat16: _lib.OUT_BF16, torch.float8_e4m3fn: _lib.E4M3, torch.float8_e5m2: _lib.E5M2}


def _fail(msg):
    raise RuntimeError(msg)


class kernel_timing:
    """Context manager that brackets every kernel launch of this module with HIP events.

    The events are recorded on the stream the kernels are launched on (torch's current
    stream).  ``records`` holds ``(kernel name, algorithmic work, start event, end event)``;
    ``summary()`` synchronises and returns per-kernel launch counts, mean duration in ms and
    the algorithmic work (flops for the GEMM, bytes for the other kernels) per launch.
    """

    _active = None

    def __init__(self):
        self.records = []

    def __enter__(self):
        kernel_timing._active = self
        return self

    def __exit__(self, *exc):
        kernel_timing._active = None
        return False

    def summary(self):
        torch.cuda.synchronize()
        out = {}
        for name, work, start, end in self.records:
            d = out.setdefault(name, {"launches": 0, "ms": 0.0, "work": 0.0})
            d["launches"] += 1
            d["ms"] += start.elapsed_time(end)
            d["work"] += work
        for d in out.values():
            d["ms"] /= d["launches"]
            d["work"] /= d["launches"]
        return out


class _timed:
    def __init__(self, name, work_fn):
        self.rec = kernel_timing._active
        if self.rec is not None:
            self.name, self.work = name, float(work_fn())

    def __enter__(self):
        if self.rec is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()

    def __exit__(self, *exc):
        if self.rec is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            self.rec.records.append((self.name, self.work, self.start, end))
        return False


_OP_NAMES = {
    _lib.OP_QUANTIZE: "multi_quantize",
    _lib.OP_SCALE_MUL: "multi_scale_mul",
    _lib.OP_PAD_TRANSPOSE: "multi_pad_transpose",
    _lib.OP_PAD_CAST_TRANSPOSE: "multi_pad_cast_transpose",
    _lib.OP_PAD_CAST_TRANSPOSE_DGELU: "multi_pad_cast_transpose_dgelu",
}


def _algorithmic_bytes(op, table):
    """HBM bytes an ideal kernel moves: every input element read once, every output element written once."""
    rows = table["rows"].astype(np.int64)
    cols = table["cols"].astype(np.int64)
    rpad = table["rows_padded"].astype(np.int64)
    if op == _lib.OP_QUANTIZE:
        return int((rows * cols * 3).sum())
    if op == _lib.OP_SCALE_MUL:
        return int((rows * cols * 4).sum())
    has_out = (table["out"] != 0).astype(np.int64)
    in_bytes = {_lib.OP_PAD_TRANSPOSE: 1, _lib.OP_PAD_CAST_TRANSPOSE: 2, _lib.OP_PAD_CAST_TRANSPOSE_DGELU: 4}[op]
    return int((cols * (rows * in_bytes + rows * has_out + rpad)).sum())


def _algorithmic_flops(table):
    return int((2 * table["m"].astype(np.int64) * table["n"].astype(np.int64) * table["k"].astype(np.int64)).sum())


def _device_of(tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            _fail("fp8_gmm_amd: expected GPU tensors (the HIP path has no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            _fail("fp8_gmm_amd: all tensors of one call must live on the same device")
    return dev


def _upload(table, device):
    """Host table (numpy structured array) -> device bytes, asynchronously on the current stream."""
    host = torch.from_numpy(table.view(np.uint8).reshape(-1))
    pinned = torch.empty(host.numel(), dtype=torch.uint8, pin_memory=True)
    pinned.copy_(host)
    return pinned.to(device, non_blocking=True)


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def _scalar_ptrs(scalars, n, what):
    """Device addresses of n fp32 scalars given as a list of 0-d / 1-element tensors, a 1-D tensor, or None."""
    if scalars is None:
        return np.zeros(n, dtype=np.uint64)
    if isinstance(scalars, torch.Tensor):
        if scalars.dtype != torch.float32 or scalars.numel() != n or not scalars.is_contiguous():
            _fail(f"fp8_gmm_amd: {what} must be {n} contiguous fp32 values")
        _device_of([scalars])
        return scalars.data_ptr() + 4 * np.arange(n, dtype=np.uint64)
    if len(scalars) != n:
        _fail(f"fp8_gmm_amd: expected {n} {what}, got {len(scalars)}")
    out = np.zeros(n, dtype=np.uint64)
    for i, s in enumerate(scalars):
        if s is None:
            continue
        if s.dtype != torch.float32 or s.numel() != 1 or not s.is_cuda:
            _fail(f"fp8_gmm_amd: every entry of {what} must be a one-element fp32 GPU tensor")
        out[i] = s.data_ptr()
    return out


def _launch_multi(op, table, out_fmt, device):
    """Plan, upload and launch one multi-tensor kernel over `table`."""
    total = _lib.plan_multi_tensor(table, op)
    if total == 0:
        return
    L = _lib.load()
    dev_table = _upload(table, device)
    n = len(table)
    with torch.cuda.device(device), _timed(_OP_NAMES[op], lambda: _algorithmic_bytes(op, table)):
        s = _stream(device)
        if op == _lib.OP_QUANTIZE:
            rc = L.fp8gmm_multi_quantize(dev_table.data_ptr(), n, total, out_fmt, s)
        elif op == _lib.OP_SCALE_MUL:
            rc = L.fp8gmm_multi_scale_mul(dev_table.data_ptr(), n, total, s)
        elif op == _lib.OP_PAD_TRANSPOSE:
            rc = L.fp8gmm_multi_pad_transpose(dev_table.data_ptr(), n, total, s)
        elif op == _lib.OP_PAD_CAST_TRANSPOSE:
            rc = L.fp8gmm_multi_pad_cast_transpose(dev_table.data_ptr(), n, total, out_fmt, s)
        else:
            rc = L.fp8gmm_multi_pad_cast_transpose_dgelu(dev_table.data_ptr(), n, total, out_fmt, s)
    _lib.check(rc)


def _check_lists(n, **lists):
    for name, lst in lists.items():
        if len(lst) != n:
            _fail(f"fp8_gmm_amd: {name} has {len(lst)} entries, expected {n}")


def _common_fp8_dtype(outputs):
    dt = outputs[0].dtype
    if dt not in _FP8_DTYPES:
        _fail("fp8_gmm_amd: outputs must be float8_e4m3fn or float8_e5m2")
    for o in outputs:
        if o.dtype != dt:
            _fail("fp8_gmm_amd: all fp8 outputs of one call must share one fp8 dtype")
    return dt


# ------------------------------------------------------------------------------------------------
# multi-tensor element-wise / pad / transpose entry points
# ------------------------------------------------------------------------------------------------
def multi_quantize(inputs, outputs, scales, amaxes):
    """outputs[i] = fp8(inputs[i] * scales[i]); amaxes[i] = max(amaxes[i], max|inputs[i]|)."""
    n = len(inputs)
    if n == 0:
        return
    _check_lists(n, outputs=outputs, scales=scales, amaxes=amaxes)
    dev = _device_of(list(inputs) + list(outputs))
    dt = _common_fp8_dtype(outputs)
    table = np.zeros(n, dtype=TENSOR_DESC)
    for i, (x, o) in enumerate(zip(inputs, outputs)):
        if x.dtype != torch.bfloat16:
            _fail("fp8_gmm_amd: multi_quantize inputs must be bfloat16")
        if x.shape != o.shape:
            _fail("fp8_gmm_amd: multi_quantize input / output shapes differ")
        if not (x.is_contiguous() and o.is_contiguous()):
            _fail("fp8_gmm_amd: multi_quantize needs contiguous tensors")
        table["in"][i] = x.data_ptr()
        table["out"][i] = o.data_ptr()
        numel = x.numel()
        if numel >= 2**31:
            _fail("fp8_gmm_amd: tensors of 2^31 or more elements are not supported")
        table["rows"][i] = 1 if numel else 0
        table["cols"][i] = numel
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_QUANTIZE, table, _FMT[dt], dev)


def multi_scale_mul(inputs, scales_1, scales_2):
    """In place inputs[i] = bf16(inputs[i] * scales_1[i] * scales_2[i])."""
    n = len(inputs)
    if n == 0:
        return
    _check_lists(n, scales_1=scales_1, scales_2=scales_2)
    dev = _device_of(inputs)
    table = np.zeros(n, dtype=TENSOR_DESC)
    for i, x in enumerate(inputs):
        if x.dtype != torch.bfloat16:
            _fail("fp8_gmm_amd: multi_scale_mul inputs must be bfloat16")
        if not x.is_contiguous():
            _fail("fp8_gmm_amd: multi_scale_mul needs contiguous tensors")
        table["in"][i] = x.data_ptr()
        numel = x.numel()
        table["rows"][i] = 1 if numel else 0
        table["cols"][i] = numel
    table["scale"] = _scalar_ptrs(scales_1, n, "scales_1")
    table["in2"] = _scalar_ptrs(scales_2, n, "scales_2")
    _launch_multi(_lib.OP_SCALE_MUL, table, _lib.E4M3, dev)


def _fill_transpose_shapes(table, i, x, t):
    if x.dim() != 2 or t.dim() != 2:
        _fail("fp8_gmm_amd: transposes work on 2-D tensors")
    m, ncols = x.shape
    if t.shape[0] != ncols or t.shape[1] < m:
        _fail("fp8_gmm_amd: transposed output must be [cols, M] with M >= rows")
    if not (x.is_contiguous() and t.is_contiguous()):
        _fail("fp8_gmm_amd: transposes need contiguous tensors")
    table["rows"][i] = m
    table["cols"][i] = ncols
    table["rows_padded"][i] = t.shape[1]


def multi_transpose(inputs, outputs):
    """outputs[i][n, M] = pad(inputs[i][m, n].T): fp8 -> fp8, columns m..M-1 zero."""
    n = len(inputs)
    if n == 0:
        return
    _check_lists(n, outputs=outputs)
    dev = _device_of(list(inputs) + list(outputs))
    table = np.zeros(n, dtype=TENSOR_DESC)
    for i, (x, t) in enumerate(zip(inputs, outputs)):
        if x.dtype not in _FP8_DTYPES or x.dtype != t.dtype:
            _fail("fp8_gmm_amd: multi_transpose needs fp8 inputs and outputs of the same dtype")
        _fill_transpose_shapes(table, i, x, t)
        table["in"][i] = x.data_ptr()
        table["out_t"][i] = t.data_ptr()
    _launch_multi(_lib.OP_PAD_TRANSPOSE, table, _lib.E4M3, dev)


def multi_cast_transpose(inputs, outputs, trans_outputs, scales, amaxes):
    """outputs[i] = fp8(inputs[i] * scale); trans_outputs[i] = its zero-padded transpose; amax merged."""
    n = len(inputs)
    if n == 0:
        return
    _check_lists(n, outputs=outputs, trans_outputs=trans_outputs, scales=scales, amaxes=amaxes)
    dev = _device_of(list(inputs) + list(outputs) + list(trans_outputs))
    dt = _common_fp8_dtype(list(outputs) + list(trans_outputs))
    table = np.zeros(n, dtype=TENSOR_DESC)
    for i, (x, o, t) in enumerate(zip(inputs, outputs, trans_outputs)):
        if x.dtype != torch.bfloat16:
            _fail("fp8_gmm_amd: multi_cast_transpose inputs must be bfloat16")
        if x.shape != o.shape or not o.is_contiguous():
            _fail("fp8_gmm_amd: multi_cast_transpose input / output shapes differ or output not contiguous")
        _fill_transpose_shapes(table, i, x, t)
        table["in"][i] = x.data_ptr()
        table["out"][i] = o.data_ptr()
        table["out_t"][i] = t.data_ptr()
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_PAD_CAST_TRANSPOSE, table, _FMT[dt], dev)


def multi_cast_transpose_dgelu(inputs, gelu_inputs, outputs, trans_outputs, scales, amaxes):
    """Like multi_cast_transpose on x = inputs[i] * dgelu(gelu_inputs[i]) (tanh-GELU derivative)."""
    n = len(inputs)
    if n == 0:
        return
    _check_lists(n, gelu_inputs=gelu_inputs, outputs=outputs, trans_outputs=trans_outputs, scales=scales,
                 amaxes=amaxes)
    dev = _device_of(list(inputs) + list(gelu_inputs) + list(outputs) + list(trans_outputs))
    dt = _common_fp8_dtype(list(outputs) + list(trans_outputs))
    table = np.zeros(n, dtype=TENSOR_DESC)
    for i, (x, g, o, t) in enumerate(zip(inputs, gelu_inputs, outputs, trans_outputs)):
        if x.dtype != torch.bfloat16 or g.dtype != torch.bfloat16:
            _fail("fp8_gmm_amd: multi_cast_transpose_dgelu inputs must be bfloat16")
        if x.shape != o.shape or x.shape != g.shape or not (o.is_contiguous() and g.is_contiguous()):
            _fail("fp8_gmm_amd: multi_cast_transpose_dgelu shapes differ or tensors not contiguous")
        _fill_transpose_shapes(table, i, x, t)
        table["in"][i] = x.data_ptr()
        table["in2"][i] = g.data_ptr()
        table["out"][i] = o.data_ptr()
        table["out_t"][i] = t.data_ptr()
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_PAD_CAST_TRANSPOSE_DGELU, table, _FMT[dt], dev)


# ------------------------------------------------------------------------------------------------
# GEMMs
# ------------------------------------------------------------------------------------------------
def _launch_gemm(table, a_dtype, b_dtype, c_dtype, gelu, device):
    if a_dtype not in _FP8_DTYPES or b_dtype not in _FP8_DTYPES:
        _fail("fp8_gmm_amd: GEMM operands must be fp8")
    if a_dtype == torch.float8_e5m2 and b_dtype == torch.float8_e5m2:
        _fail("fp8_gmm_amd: e5m2 x e5m2 GEMMs are not supported")
    if c_dtype not in _OUT_KIND:
        _fail("fp8_gmm_amd: GEMM output must be bfloat16 or fp8")
    total = _lib.plan_grouped_gemm(table)
    if total == 0:
        return
    dev_table = _upload(table, device)
    with torch.cuda.device(device), _timed("grouped_gemm", lambda: _algorithmic_flops(table)):
        rc = _lib.load().fp8gmm_grouped_gemm(
            dev_table.data_ptr(), len(table), total, _FMT[a_dtype], _FMT[b_dtype], _OUT_KIND[c_dtype],
            _lib.EPI_GELU if gelu else 0, _stream(device),
        )
    _lib.check(rc)


def delayed_scaling_update(amax_history, scale, scale_inv, fp8_max, margin=0, most_recent=False):
    """In-place delayed-scaling update of one direction in ONE kernel (the rule of
    ``fp8.amax_and_scale_update``): ``amax_history`` [history, slots], ``scale`` / ``scale_inv`` [slots]."""
    for t, what in ((amax_history, "amax_history"), (scale, "scale"), (scale_inv, "scale_inv")):
        if t.dtype != torch.float32 or not t.is_contiguous():
            _fail(f"fp8_gmm_amd: {what} must be a contiguous fp32 tensor")
    if amax_history.dim() != 2 or scale.numel() != amax_history.shape[1] or scale_inv.numel() != scale.numel():
        _fail("fp8_gmm_amd: amax_history must be [history, slots] and scale / scale_inv [slots]")
    dev = _device_of([amax_history, scale, scale_inv])
    with torch.cuda.device(dev):
        rc = _lib.load().fp8gmm_delayed_scaling_update(
            amax_history.data_ptr(), scale.data_ptr(), scale_inv.data_ptr(), amax_history.shape[0],
            amax_history.shape[1], float(fp8_max), int(margin), int(bool(most_recent)), _stream(dev))
    _lib.check(rc)


def _check_2d(t, what):
    if t.dim() != 2:
        _fail(f"fp8_gmm_amd: {what} must be 2-D")
    if t.stride(1) != 1 and t.shape[1] > 1:
        _fail(f"fp8_gmm_amd: {what} must have a contiguous last dimension")
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def grouped_gemm(a_list, b_list, c_list, a_scale_invs, b_scale_invs, pre_gelu_outs=None, c_scales=None,
                 c_amaxes=None):
    """c_list[i][m, n] = epilogue(a_list[i][m, k] . b_list[i][n, k]^T) for all i in ONE launch.

    The list form of ``cublas_fp8_gemm``: the reference issues these as a Python loop of
    cuBLASLt calls (wgrad, grouped_linear.py:173-182; grouped_mlp.py:234-242,313-322).
    k may differ per entry and may be 0 (the output is then the epilogue of zero).
    """
    n = len(a_list)
    if n == 0:
        return
    _check_lists(n, b_list=b_list, c_list=c_list)
    dev = _device_of(list(a_list) + list(b_list) + list(c_list))
    a_dt, b_dt, c_dt = a_list[0].dtype, b_list[0].dtype, c_list[0].dtype
    fp8_out = c_dt in _FP8_DTYPES
    if fp8_out and c_scales is None:
        _fail("fp8_gmm_amd: an fp8 GEMM output needs c_scales")
    table = np.zeros(n, dtype=GEMM_PROBLEM)
    for i, (a, b, c) in enumerate(zip(a_list, b_list, c_list)):
        if a.dtype != a_dt or b.dtype != b_dt or c.dtype != c_dt:
            _fail("fp8_gmm_amd: all problems of one grouped GEMM must share dtypes")
        lda, ldb, ldc = _check_2d(a, "a"), _check_2d(b, "b"), _check_2d(c, "c")
        m, k = a.shape
        nn, kb = b.shape
        if k != kb or tuple(c.shape) != (m, nn):
            _fail("fp8_gmm_amd: GEMM shapes do not match: a [m, k], b [n, k], c [m, n]")
        table["a"][i], table["b"][i], table["c"][i] = a.data_ptr(), b.data_ptr(), c.data_ptr()
        table["m"][i], table["n"][i], table["k"][i] = m, nn, k
        table["lda"][i], table["ldb"][i], table["ldc"][i] = max(lda, k), max(ldb, k), max(ldc, nn)
        if pre_gelu_outs is not None:
            aux = pre_gelu_outs[i]
            if aux.dtype != torch.bfloat16 or tuple(aux.shape) != (m, nn) or _check_2d(aux, "pre_gelu_out") != ldc:
                _fail("fp8_gmm_amd: pre_gelu_out must be bf16 [m, n] with the row pitch of c")
            table["aux"][i] = aux.data_ptr()
    table["a_scale_inv"] = _scalar_ptrs(a_scale_invs, n, "a_scale_invs")
    table["b_scale_inv"] = _scalar_ptrs(b_scale_invs, n, "b_scale_invs")
    if fp8_out:
        table["c_scale"] = _scalar_ptrs(c_scales, n, "c_scales")
        table["c_amax"] = _scalar_ptrs(c_amaxes, n, "c_amaxes")
    _launch_gemm(table, a_dt, b_dt, c_dt, pre_gelu_outs is not None, dev)


def cublas_fp8_gemm(a, b, c, a_scale_inv, b_scale_inv, pre_gelu_out=None, c_scale=None, c_amax=None, backward=False):
    """c[m, n] = (a[m, k] . b[n, k]^T) * a_scale_inv * b_scale_inv, both operands K-contiguous ("TN").

    With ``pre_gelu_out`` the epilogue is GELU-aux: pre_gelu_out = bf16(result), c = gelu(result);
    an fp8 ``c`` is additionally multiplied by ``c_scale`` and its amax recorded.  ``backward``
    selected split accumulation in the reference's cuBLASLt call (backend.py:52); the MFMA
    kernel always accumulates in full fp32, so the flag changes nothing here.
    """
    if c.dtype in _FP8_DTYPES and (c_scale is None or c_amax is None):
        _fail("fp8_gmm_amd: an fp8 output needs c_scale and c_amax")
    grouped_gemm(
        [a], [b], [c], [a_scale_inv], [b_scale_inv],
        pre_gelu_outs=None if pre_gelu_out is None else [pre_gelu_out],
        c_scales=None if c_scale is None else [c_scale],
        c_amaxes=None if c_amax is None else [c_amax],
    )


def _group_sizes_list(group_sizes):
    if isinstance(group_sizes, torch.Tensor):
        if group_sizes.dim() != 1:
            _fail("fp8_gmm_amd: group_sizes must be 1-D")
        return [int(g) for g in group_sizes.tolist()]
    return [int(g) for g in group_sizes]


def fp8_gmm(a, b, group_sizes, a_scale_invs, b_scale_invs, c=None, c_dtype=torch.bfloat16, pre_gelu_out=None,
            c_scales=None, c_amaxes=None, backward=False, cutlass=False):
    """Grouped GEMM over row slices of ``a``: expert i multiplies rows
    ``[sum(group_sizes[:i]), sum(group_sizes[:i+1]))`` of ``a[tokens, k]`` with ``b[i][n, k]^T``.

    One persistent kernel launch for all experts.  ``cutlass=True`` reproduces the data
    flow of the reference's CUTLASS path (backend.py:78-82): an unscaled GEMM to bf16
    followed by ``multi_scale_mul`` (two roundings); the default applies the scales to
    the fp32 accumulator in the GEMM epilogue (one rounding), like its cuBLASLt path.
    Experts with zero rows are allowed.
    """
    sizes = _group_sizes_list(group_sizes)
    e = len(sizes)
    if a.dim() != 2 or b.dim() != 3:
        _fail("fp8_gmm_amd: fp8_gmm expects a [tokens, k] and b [experts, n, k]")
    if not (a.is_contiguous() and b.is_contiguous()):
        _fail("fp8_gmm_amd: fp8_gmm expects contiguous a and b")
    tokens, k = a.shape
    if b.shape[0] != e or b.shape[2] != k:
        _fail("fp8_gmm_amd: b must be [len(group_sizes), n, k] with k == a.shape[1]")
    if any(g < 0 for g in sizes) or sum(sizes) != tokens:
        _fail("fp8_gmm_amd: group_sizes must be non-negative and sum to a.shape[0]")
    nn = b.shape[1]
    if c is None:
        c = torch.empty(tokens, nn, device=a.device, dtype=c_dtype)
    if tuple(c.shape) != (tokens, nn) or not c.is_contiguous():
        _fail("fp8_gmm_amd: c must be a contiguous [tokens, n] tensor")
    fp8_out = c.dtype in _FP8_DTYPES
    if fp8_out and (c_scales is None or c_amaxes is None):
        _fail("fp8_gmm_amd: an fp8 output needs c_scales and c_amaxes")
    if cutlass and (c.dtype != torch.bfloat16 or pre_gelu_out is not None):
        _fail("fp8_gmm_amd: cutlass=True supports a bf16 output without GELU only")
    if pre_gelu_out is not None and (
        pre_gelu_out.dtype != torch.bfloat16 or tuple(pre_gelu_out.shape) != (tokens, nn)
        or not pre_gelu_out.is_contiguous()
    ):
        _fail("fp8_gmm_amd: pre_gelu_out must be a contiguous bf16 [tokens, n] tensor")
    dev = _device_of([a, b, c, pre_gelu_out])

    starts = np.zeros(e + 1, dtype=np.int64)
    np.cumsum(np.asarray(sizes, dtype=np.int64), out=starts[1:])
    row0 = starts[:-1].astype(np.uint64)
    table = np.zeros(e, dtype=GEMM_PROBLEM)
    table["a"] = a.data_ptr() + row0 * np.uint64(k * a.element_size())
    table["b"] = b.data_ptr() + np.arange(e, dtype=np.uint64) * np.uint64(nn * k * b.element_size())
    table["c"] = c.data_ptr() + row0 * np.uint64(nn * c.element_size())
    if pre_gelu_out is not None:
        table["aux"] = pre_gelu_out.data_ptr() + row0 * np.uint64(nn * 2)
    table["m"] = np.asarray(sizes, dtype=np.int32)
    table["n"] = nn
    table["k"] = k
    table["lda"] = k
    table["ldb"] = k
    table["ldc"] = nn
    if not cutlass:
        table["a_scale_inv"] = _scalar_ptrs(a_scale_invs, e, "a_scale_invs")
        table["b_scale_inv"] = _scalar_ptrs(b_scale_invs, e, "b_scale_invs")
    if fp8_out:
        table["c_scale"] = _scalar_ptrs(c_scales, e, "c_scales")
        table["c_amax"] = _scalar_ptrs(c_amaxes, e, "c_amaxes")
    _launch_gemm(table, a.dtype, b.dtype, c.dtype, pre_gelu_out is not None, dev)
    if cutlass:
        c_groups = [c[starts[i]: starts[i + 1]] for i in range(e)]
        multi_scale_mul(c_groups, a_scale_invs, b_scale_invs)
    return c
