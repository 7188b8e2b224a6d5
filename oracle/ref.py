"""CPU oracle, Python side.  TEST INFRASTRUCTURE ONLY.

Thin ctypes bindings over ``liboracle.so`` (built from ``fp8_oracle.c``) plus
CPU restatements of the reference's Python entry points, operating on CPU
torch tensors.  Nothing under the product package imports this module; the
tests, the smoke check and the CPU-baseline leg of the benchmark do.

Entry points mirror ``fp8_gmm/backend.py`` of the reference:

* :func:`multi_quantize`              - backend.py:9   -> csrc/multi_pointwise.cu:155
* :func:`multi_transpose`             - backend.py:13  -> csrc/multi_pad_fusion.cu:442
* :func:`multi_cast_transpose`        - backend.py:17  -> csrc/multi_pad_fusion.cu:505
* :func:`multi_cast_transpose_dgelu`  - backend.py:21  -> csrc/multi_pad_fusion.cu:587
* :func:`multi_scale_mul`             - csrc/multi_pointwise.cu:216
* :func:`cublas_fp8_gemm`             - backend.py:26
* :func:`fp8_gmm`                     - backend.py:58 (per-expert loop, fp8_gmm/test.py:209-214)
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

E4M3 = 0
E5M2 = 1

_FMT_OF = {torch.float8_e4m3fn: E4M3, torch.float8_e5m2: E5M2}
FP8_MAX = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}


def build(force=False):
    """Compile liboracle.so with gcc (a second or so)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.orc_bf16_to_f32.restype = ctypes.c_float
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_f32_to_fp8.restype = ctypes.c_uint8
        L.orc_f32_to_fp8.argtypes = [ctypes.c_float, i32]
        L.orc_fp8_to_f32.restype = ctypes.c_float
        L.orc_fp8_to_f32.argtypes = [ctypes.c_uint8, i32]
        L.orc_tanh.restype = ctypes.c_float
        L.orc_tanh.argtypes = [ctypes.c_float]
        L.orc_dgelu.restype = ctypes.c_float
        L.orc_dgelu.argtypes = [ctypes.c_float]
        L.orc_gelu.restype = ctypes.c_float
        L.orc_gelu.argtypes = [ctypes.c_float]
        for name, args in {
            "orc_fp8_to_f32_array": [vp, i64, i32, vp],
            "orc_f32_to_fp8_array": [vp, i64, i32, vp],
            "orc_f32_to_bf16_array": [vp, i64, vp],
            "orc_quantize": [vp, i64, vp, i32, vp, vp],
            "orc_scale_mul": [vp, i64, vp, vp],
            "orc_pad_transpose": [vp, i64, i64, i64, vp],
            "orc_pad_cast_transpose": [vp, i64, i64, i64, vp, i32, vp, vp, vp],
            "orc_pad_cast_transpose_dgelu": [vp, vp, i64, i64, i64, vp, i32, vp, vp, vp],
            "orc_tanh_array": [vp, i64, vp],
            "orc_dgelu_array": [vp, i64, vp],
            "orc_gelu_array": [vp, i64, vp],
            "orc_gemm_f32": [vp, i32, vp, i32, i64, i64, i64, i64, i64, vp],
            "orc_epilogue_bf16": [vp, i64, ctypes.c_float, ctypes.c_float, vp],
            "orc_epilogue_gelu_fp8": [vp, i64, ctypes.c_float, ctypes.c_float, vp, i32, vp, vp, vp],
            "orc_epilogue_dgelu_fp8": [vp, i64, ctypes.c_float, ctypes.c_float, vp, i32, vp, vp, vp],
        }.items():
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = args
        _lib = L
    return _lib


def _cpu_contig(t, dtype=None):
    assert t.device.type == "cpu", "the oracle works on CPU tensors only"
    assert t.is_contiguous(), "the oracle needs contiguous tensors (like the reference's raw data_ptr use)"
    if dtype is not None:
        assert t.dtype == dtype, f"expected {dtype}, got {t.dtype}"
    return t


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def fmt_of(dtype):
    return _FMT_OF[dtype]


# ----------------------------------------------------------------------------------------------
# element-wise helpers
# ----------------------------------------------------------------------------------------------
def f32_to_fp8(x, dtype):
    """fp32 CPU tensor -> fp8 tensor (saturating RNE)."""
    x = _cpu_contig(x.contiguous(), torch.float32)
    out = torch.empty(x.shape, dtype=dtype)
    lib().orc_f32_to_fp8_array(_ptr(x), x.numel(), fmt_of(dtype), _ptr(out))
    return out


def fp8_to_f32(x):
    x = _cpu_contig(x.contiguous())
    out = torch.empty(x.shape, dtype=torch.float32)
    lib().orc_fp8_to_f32_array(_ptr(x), x.numel(), fmt_of(x.dtype), _ptr(out))
    return out


def f32_to_bf16(x):
    x = _cpu_contig(x.contiguous(), torch.float32)
    out = torch.empty(x.shape, dtype=torch.bfloat16)
    lib().orc_f32_to_bf16_array(_ptr(x), x.numel(), _ptr(out))
    return out


def _unary(name, x):
    x = _cpu_contig(x.contiguous(), torch.float32)
    out = torch.empty_like(x)
    getattr(lib(), name)(_ptr(x), x.numel(), _ptr(out))
    return out


def tanh(x):
    return _unary("orc_tanh_array", x)


def dgelu(x):
    return _unary("orc_dgelu_array", x)


def gelu(x):
    return _unary("orc_gelu_array", x)


# ----------------------------------------------------------------------------------------------
# reference backend entry points, restated on CPU tensors
# ----------------------------------------------------------------------------------------------
def multi_quantize(inputs, outputs, scales, amaxes):
    for x, o, s, a in zip(inputs, outputs, scales, amaxes):
        _cpu_contig(x, torch.bfloat16)
        _cpu_contig(o)
        assert x.shape == o.shape
        lib().orc_quantize(_ptr(x), x.numel(), _ptr(s), fmt_of(o.dtype), _ptr(o), _ptr(a))


def multi_scale_mul(inputs, scales_1, scales_2):
    for x, s1, s2 in zip(inputs, scales_1, scales_2):
        _cpu_contig(x, torch.bfloat16)
        lib().orc_scale_mul(_ptr(x), x.numel(), _ptr(s1), _ptr(s2))


def _check_t(x, t):
    m, n = x.shape
    assert t.dim() == 2 and t.shape[0] == n and t.shape[1] >= m
    return m, n, t.shape[1]


def multi_transpose(inputs, outputs):
    for x, t in zip(inputs, outputs):
        _cpu_contig(x)
        _cpu_contig(t)
        assert x.dtype == t.dtype and x.dtype in _FMT_OF
        m, n, mpad = _check_t(x, t)
        lib().orc_pad_transpose(_ptr(x), m, n, mpad, _ptr(t))


def multi_cast_transpose(inputs, outputs, trans_outputs, scales, amaxes):
    for x, o, t, s, a in zip(inputs, outputs, trans_outputs, scales, amaxes):
        _cpu_contig(x, torch.bfloat16)
        _cpu_contig(o)
        _cpu_contig(t)
        assert o.dtype == t.dtype and x.shape == o.shape
        m, n, mpad = _check_t(x, t)
        lib().orc_pad_cast_transpose(_ptr(x), m, n, mpad, _ptr(s), fmt_of(o.dtype), _ptr(o), _ptr(t), _ptr(a))


def multi_cast_transpose_dgelu(inputs, gelu_inputs, outputs, trans_outputs, scales, amaxes):
    for x, g, o, t, s, a in zip(inputs, gelu_inputs, outputs, trans_outputs, scales, amaxes):
        _cpu_contig(x, torch.bfloat16)
        _cpu_contig(g, torch.bfloat16)
        _cpu_contig(o)
        _cpu_contig(t)
        assert o.dtype == t.dtype and x.shape == o.shape == g.shape
        m, n, mpad = _check_t(x, t)
        lib().orc_pad_cast_transpose_dgelu(
            _ptr(x), _ptr(g), m, n, mpad, _ptr(s), fmt_of(o.dtype), _ptr(o), _ptr(t), _ptr(a)
        )


def multi_cast_dgelu(inputs, gelu_inputs, outputs, scales, amaxes):
    """x = dy * dgelu(pre) cast to fp8, no transposed copy.  The reference has no such kernel and says so
    (fp8_gmm/grouped_mlp.py:252-253); it is defined as the row-major output of multi_cast_transpose_dgelu."""
    for x, g, o, s, a in zip(inputs, gelu_inputs, outputs, scales, amaxes):
        rows = x.reshape(-1, x.shape[-1]) if x.dim() > 0 and x.numel() > 0 else x.reshape(0, 1)
        t = torch.empty(rows.shape[1], rows.shape[0], dtype=o.dtype)
        multi_cast_transpose_dgelu([rows], [g.reshape(rows.shape)], [o.reshape(rows.shape)], [t], [s], [a])


def gemm_acc_naive(a, b):
    """acc[m, n] = sum_k a[m, k] b[n, k] on dequantised fp8, double accumulation in C (small sizes)."""
    _cpu_contig(a)
    _cpu_contig(b)
    m, k = a.shape
    n, kb = b.shape
    assert k == kb
    c = torch.empty(m, n, dtype=torch.float32)
    lib().orc_gemm_f32(_ptr(a), fmt_of(a.dtype), _ptr(b), fmt_of(b.dtype), m, n, k, k, k, _ptr(c))
    return c


def gemm_acc(a, b):
    """Same accumulator through torch's fp32 matmul on exactly dequantised operands (any size)."""
    if a.shape[0] == 0 or a.shape[1] == 0:
        return torch.zeros(a.shape[0], b.shape[0], dtype=torch.float32)
    return torch.matmul(fp8_to_f32(a), fp8_to_f32(b).t())


def cublas_fp8_gemm(a, b, c, a_scale_inv, b_scale_inv, pre_gelu_out=None, c_scale=None, c_amax=None,
                    backward=False, naive=False, dgelu_pre=None):
    """c[m, n] = epilogue((a[m, k] . b[n, k]^T) * a_scale_inv * b_scale_inv), see orc_epilogue_*.
    ``dgelu_pre`` (bf16 [m, n], an input): the result times dgelu(dgelu_pre) before the rounding to fp8."""
    acc = (gemm_acc_naive if naive else gemm_acc)(a.contiguous(), b.contiguous()).contiguous()
    sa, sb = float(a_scale_inv), float(b_scale_inv)
    _cpu_contig(c)
    if dgelu_pre is not None:
        assert pre_gelu_out is None and c.dtype != torch.bfloat16 and c_scale is not None and c_amax is not None
        _cpu_contig(dgelu_pre, torch.bfloat16)
        lib().orc_epilogue_dgelu_fp8(_ptr(acc), acc.numel(), sa, sb, _ptr(c_scale), fmt_of(c.dtype), _ptr(dgelu_pre),
                                     _ptr(c), _ptr(c_amax))
    elif c.dtype == torch.bfloat16:
        assert pre_gelu_out is None
        lib().orc_epilogue_bf16(_ptr(acc), acc.numel(), sa, sb, _ptr(c))
    else:
        assert c_scale is not None and c_amax is not None
        if pre_gelu_out is not None:
            _cpu_contig(pre_gelu_out, torch.bfloat16)
        lib().orc_epilogue_gelu_fp8(
            _ptr(acc), acc.numel(), sa, sb, _ptr(c_scale), fmt_of(c.dtype), _ptr(pre_gelu_out), _ptr(c), _ptr(c_amax)
        )
    return c


def fp8_gmm(a, b, group_sizes, a_scale_invs, b_scale_invs, c=None, c_dtype=torch.bfloat16, pre_gelu_out=None,
            c_scales=None, c_amaxes=None, backward=False, cutlass=False, naive=False, dgelu_pre=None):
    """Per-expert loop of the reference (fp8_gmm/backend.py:84-96; oracle form fp8_gmm/test.py:209-214)."""
    if c is None:
        c = torch.empty(a.shape[0], b.shape[1], dtype=c_dtype)
    sizes = [int(g) for g in group_sizes]
    start = 0
    for i, g in enumerate(sizes):
        end = start + g
        if g > 0:
            cublas_fp8_gemm(
                a[start:end], b[i], c[start:end], a_scale_invs[i], b_scale_invs[i],
                pre_gelu_out=pre_gelu_out[start:end] if pre_gelu_out is not None else None,
                c_scale=c_scales[i] if c_scales is not None else None,
                c_amax=c_amaxes[i] if c_amaxes is not None else None,
                backward=backward, naive=naive,
                dgelu_pre=dgelu_pre[start:end].contiguous() if dgelu_pre is not None else None,
            )
        start = end
    return c


def fp32_matmul_reference(a, b, group_sizes, a_scale_invs, b_scale_invs):
    """fp32 result (no output rounding) of the grouped GEMM: what GPU outputs are compared with."""
    out = torch.zeros(a.shape[0], b.shape[1], dtype=torch.float32)
    start = 0
    for i, g in enumerate(int(g) for g in group_sizes):
        end = start + g
        if g > 0:
            out[start:end] = gemm_acc(a[start:end].contiguous(), b[i].contiguous()) * (
                float(a_scale_invs[i]) * float(b_scale_invs[i])
            )
        start = end
    return out
