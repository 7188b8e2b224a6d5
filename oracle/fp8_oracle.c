/*
 * CPU oracle for the FP8 grouped-GEMM hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of the reference's
 * native kernels so that the HIP kernels can be checked bit for bit.  It is
 * never linked into, loaded by, or called from the product library; only the
 * test-suite, the smoke check and the CPU-baseline leg of the benchmark use it.
 *
 * Reference lines followed by each function are cited next to it
 * (paths relative to the reference checkout).
 *
 * Pinning status (what proves each function independently of this file):
 *   orc_f32_to_fp8 / orc_fp8_to_f32 : exhaustive comparison with PyTorch's CPU
 *       float8_e4m3fn / float8_e5m2 conversions (after the saturation clamp)
 *       plus hand-computed edge bytes                       -> pinned
 *   orc_f32_to_bf16                : exhaustive-ish comparison with PyTorch  -> pinned
 *   orc_quantize / amax            : torch ops (abs().max(), clamp().to())   -> pinned
 *   orc_pad_transpose layouts      : torch .t() + F.pad, brute force          -> pinned
 *   orc_tanh / orc_dgelu / orc_gelu: libm double-precision closed forms       -> pinned
 *       (to a stated absolute error; the fp32 evaluation order itself is a
 *       rule defined by this build, because the reference evaluates tanhf
 *       under --use_fast_math, which no CPU can restate bit for bit)
 *   orc_gemm                       : torch fp32/fp64 matmul on dequantised
 *       operands, identity / power-of-two invariants                          -> pinned
 *   NaN -> 0x7F (sign dropped) in orc_f32_to_fp8: follows the CUDA conversion
 *       the reference calls; nothing available here can confirm it          -> parity unpinned
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORC_E4M3 0
#define ORC_E5M2 1

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* bf16 -> fp32 is exact: the 16 bits are the top half of the fp32 word.
 * (reference: `fp32(local_input.data.elt[i])`, csrc/multi_pointwise.cu:77) */
float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> bf16, round-to-nearest-even; NaN stays NaN (quiet bit forced).
 * (reference: `bf16(fp32(x) * s1 * s2)`, csrc/multi_pointwise.cu:138) */
uint16_t orc_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/*
 * fp32 -> OCP fp8, round-to-nearest-even, saturate-to-finite.
 *   e4m3fn: 4 exponent bits (bias 7), 3 mantissa bits, max finite 448 (0x7E),
 *           no infinities, 0x7F/0xFF are NaN.
 *   e5m2  : 5 exponent bits (bias 15), 2 mantissa bits, max finite 57344 (0x7B).
 * Every |x| >= max (infinities included) gives the max finite code with the
 * sign of x; NaN gives 0x7F.  This is what `static_cast<__nv_fp8_e4m3>(float)`
 * does in the reference (csrc/multi_pointwise.cu:79, csrc/multi_pad_fusion.cu:233,379):
 * the CUDA conversion is RNE with the SATFINITE policy.
 */
uint8_t orc_f32_to_fp8(float f, int fmt) {
  const int mbits = (fmt == ORC_E4M3) ? 3 : 2;
  const int bias = (fmt == ORC_E4M3) ? 7 : 15;
  const uint32_t max_bits = (fmt == ORC_E4M3) ? 0x43e00000u /* 448 */ : 0x47600000u /* 57344 */;
  const uint8_t max_code = (fmt == ORC_E4M3) ? 0x7Eu : 0x7Bu;
  const int min_exp = 1 - bias; /* exponent of the smallest normal */

  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return 0x7Fu;           /* NaN */
  if (a >= max_bits) return sign | max_code;   /* saturate (covers +-inf) */
  if (a == 0) return sign;

  int e = (int)(a >> 23) - 127;
  uint32_t mant = a & 0x7fffffu;
  if ((a >> 23) == 0) {
    /* fp32 subnormal: far below half of the smallest fp8 subnormal */
    return sign;
  }
  uint32_t code;
  if (e >= min_exp) {
    /* normal in fp8: drop (23 - mbits) mantissa bits with RNE; a carry out of
     * the mantissa moves into the exponent field, which is the right answer */
    int drop = 23 - mbits;
    code = ((uint32_t)(e + bias) << mbits) | (mant >> drop);
    uint32_t rem = mant & ((1u << drop) - 1u);
    uint32_t half = 1u << (drop - 1);
    if (rem > half || (rem == half && (code & 1u))) code += 1u;
  } else {
    /* subnormal in fp8: quantum is 2^(min_exp - mbits); result = RNE(|x| / quantum) */
    uint32_t m24 = mant | 0x800000u;              /* 1.mant as a 24-bit integer, value m24 * 2^(e-23) */
    int shift = (min_exp - mbits) - (e - 23);     /* |x|/quantum = m24 >> shift */
    if (shift > 25) return sign;                  /* below half a quantum (m24 < 2^24) */
    code = m24 >> shift;
    uint32_t rem = m24 & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (code & 1u))) code += 1u;
  }
  return sign | (uint8_t)code;
}

/* fp8 -> fp32, exact. NaN codes give NaN, e5m2 infinities give infinities. */
float orc_fp8_to_f32(uint8_t b, int fmt) {
  const int mbits = (fmt == ORC_E4M3) ? 3 : 2;
  const int bias = (fmt == ORC_E4M3) ? 7 : 15;
  uint32_t sign = (uint32_t)(b & 0x80u) << 24;
  uint32_t mag = b & 0x7fu;
  uint32_t ef = mag >> mbits;
  uint32_t mf = mag & ((1u << mbits) - 1u);
  if (fmt == ORC_E4M3) {
    if (mag == 0x7fu) return u2f(sign | 0x7fc00000u);
  } else {
    if (ef == 31u) return u2f(sign | (mf ? 0x7fc00000u : 0x7f800000u));
  }
  float v;
  if (ef == 0) v = ldexpf((float)mf, 1 - bias - mbits);
  else v = ldexpf((float)(mf | (1u << mbits)), (int)ef - bias - mbits);
  return u2f(f2u(v) | sign);
}

void orc_fp8_to_f32_array(const uint8_t* in, int64_t n, int fmt, float* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_fp8_to_f32(in[i], fmt);
}

void orc_f32_to_fp8_array(const float* in, int64_t n, int fmt, uint8_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_fp8(in[i], fmt);
}

void orc_f32_to_bf16_array(const float* in, int64_t n, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}

/* max(|x|) that drops NaNs, like fmaxf in the reference
 * (csrc/multi_pointwise.cu:78, csrc/multi_pad_fusion.cu:236). */
static inline float amax_step(float acc, float x) {
  float ax = fabsf(x);
  return (ax > acc) ? ax : acc; /* false for NaN: NaN never enters */
}

/*
 * multi_quantize for one tensor: out = fp8(fp32(x) * scale); amax = max(amax_in, max|fp32(x)|)
 * over the UNSCALED input (reference csrc/multi_pointwise.cu:51,76-80,94-96;
 * merge with previous content: csrc/utils.cuh:183-185).
 * scale == NULL means 1 (multi_pointwise.cu:51).
 */
void orc_quantize(const uint16_t* x, int64_t n, const float* scale, int fmt, uint8_t* out, float* amax) {
  float s = scale ? *scale : 1.0f;
  float mx = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float v = orc_bf16_to_f32(x[i]);
    mx = amax_step(mx, v);
    out[i] = orc_f32_to_fp8(v * s, fmt);
  }
  if (amax) {
    /* integer atomicMax on the bit patterns of two non-negative floats */
    if ((int32_t)f2u(mx) > (int32_t)f2u(*amax)) *amax = mx;
  }
}

/* in-place x = bf16(fp32(x) * s1 * s2), left to right (csrc/multi_pointwise.cu:138). */
void orc_scale_mul(uint16_t* x, int64_t n, const float* s1, const float* s2) {
  float a = s1 ? *s1 : 1.0f, b = s2 ? *s2 : 1.0f;
  for (int64_t i = 0; i < n; ++i) x[i] = orc_f32_to_bf16(orc_bf16_to_f32(x[i]) * a * b);
}

/*
 * multi_pad_transpose for one tensor: bytes in[m][n] -> t[n][mpad];
 * t[j][i] = in[i][j] for i < m, 0x00 for m <= i < mpad
 * (reference csrc/multi_pad_fusion.cu:103-118,141-147: rows >= m are cleared
 * to fp8 zero and stored while row < padded_rows).
 */
void orc_pad_transpose(const uint8_t* in, int64_t m, int64_t n, int64_t mpad, uint8_t* t) {
  for (int64_t j = 0; j < n; ++j) {
    for (int64_t i = 0; i < m; ++i) t[j * mpad + i] = in[i * n + j];
    for (int64_t i = m; i < mpad; ++i) t[j * mpad + i] = 0;
  }
}

/*
 * multi_pad_cast_transpose for one tensor (reference csrc/multi_pad_fusion.cu:205-291):
 *   y = fp8(scale * fp32(x)); out[i][j] = y; t[j][i] = y;
 *   rows m..mpad-1 of the input read as bf16 zero, so the pad byte is
 *   fp8(scale * 0) (0x00, or 0x80 when scale is negative) (:220,231-236,276);
 *   amax over |fp32(x)| of the real rows, merged into *amax (:236,286-291).
 * out may be NULL (only the transposed copy wanted).
 */
void orc_pad_cast_transpose(const uint16_t* x, int64_t m, int64_t n, int64_t mpad, const float* scale, int fmt,
                            uint8_t* out, uint8_t* t, float* amax) {
  float s = scale ? *scale : 1.0f;
  float mx = 0.0f;
  uint8_t pad = orc_f32_to_fp8(s * 0.0f, fmt);
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t j = 0; j < n; ++j) {
      float v = orc_bf16_to_f32(x[i * n + j]);
      mx = amax_step(mx, v);
      uint8_t y = orc_f32_to_fp8(s * v, fmt);
      if (out) out[i * n + j] = y;
      t[j * mpad + i] = y;
    }
  }
  for (int64_t j = 0; j < n; ++j)
    for (int64_t i = m; i < mpad; ++i) t[j * mpad + i] = pad;
  if (amax) {
    if ((int32_t)f2u(mx) > (int32_t)f2u(*amax)) *amax = mx;
  }
}

/*
 * exp(-2a) and 1 / (1 + exp(-2a)) for a >= 0 from a fixed sequence of IEEE single-precision operations (add, mul,
 * fma, integer add / shift; no division), the sequence the HIP kernels follow (csrc/device_utils.h, det_exp_rcp),
 * so that both sides produce the same bits.  Input z = a * 2 / ln 2 >= 0:
 *   z = min(z, 125); n = rne(z) by adding 1.5 * 2^23 (adding it rounds to an integer), f = z - n in [-0.5, 0.5];
 *   q = 2^-f * 2^-n with a degree-5 minimax polynomial for 2^-f (constant term exactly 1: tanh(0) = 0), the exponent subtracted in the integer domain;
 *   r = 1 / (1 + q): quadratic first guess, two Newton steps.
 * tanh(a) = (1 - q) r.  The reference evaluates tanhf under --use_fast_math (csrc/multi_pad_fusion.cu:39-44,
 * setup.py:21), which no CPU can restate bit for bit: this order of operations is this build's rule, pinned
 * against the double-precision closed forms (tests/test_oracle_pins.py).
 */
static void orc_exp_rcp(float z, float* q_out, float* r_out) {
  z = fminf(z, 125.0f); /* NaN counts as large */
  const float magic = 12582912.0f;
  float zr = magic - z;
  float nf = zr - magic;
  float f = z + nf;
  float p = -1.3400432653725147e-3f;
  p = fmaf(p, f, 9.666378609836102e-3f);
  p = fmaf(p, f, -5.550333112478256e-2f);
  p = fmaf(p, f, 2.402234822511673e-1f);
  p = fmaf(p, f, -6.931471824645996e-1f);
  p = fmaf(p, f, 1.0f);
  float q = u2f(f2u(p) + (f2u(zr) << 23));
  float d = 1.0f + q;
  float r = fmaf(fmaf(0.3232323229312897f, q, -0.808080792427063f), q, 0.9898989796638489f);
  r = fmaf(r, fmaf(-d, r, 1.0f), r);
  r = fmaf(r, fmaf(-d, r, 1.0f), r);
  *q_out = q;
  *r_out = r;
}

float orc_tanh(float u) {
  float q, r;
  orc_exp_rcp(fabsf(u) * 2.8853900817779268f, &q, &r);
  float t = copysignf(fmaf(-q, r, r), u);
  return (u != u) ? u : t; /* the clamp above takes a NaN for a large value */
}

/*
 * Derivative of tanh-GELU, reference csrc/multi_pad_fusion.cu:39-44 (same
 * constants; python twin fp8_gmm/test.py:32-34):
 *   t = tanh(u), u = 0.79788456 c (1 + 0.044715 c^2)
 *   dgelu = 0.5 c (1 - t^2)(0.79788456 + 0.1070322243 c^2) + 0.5 (1 + t)
 * evaluated through s = 0.5 (1 + t) = 1 / (1 + exp(-2u)):  1 - t^2 = 4 s (1 - s) and s (1 - s) = q r^2, so
 *   dgelu = s + c (1.59576912 + 0.2140644486 c^2) q r^2,   s = r for c >= 0 and q r otherwise.
 * The operation order below is this build's rule (see orc_exp_rcp).  Where c^2 overflows (|c| > 1.8e19) the
 * reference's form gives NaN (0 * inf) and this one an infinity; neither is a value an activation takes.
 */
float orc_dgelu(float c) {
  float c2 = c * c;
  float w = fmaf(0.044715f, c2, 1.0f);
  float q, r;
  orc_exp_rcp(fabsf((2.3022082f * c) * w), &q, &r); /* 2.3022082 = 0.79788456 * 2 / ln 2 */
  float t1 = q * r;
  float s1 = t1 * r;
  float sig = (c >= 0.0f) ? r : t1;
  float g2 = fmaf(0.2140644486f, c2, 1.59576912f);
  return fmaf(c * g2, s1, sig);
}

/* tanh-GELU forward, the epilogue of the fc1 GEMM (the GELU-aux epilogue the
 * reference requests from cuBLASLt through fp8_gmm/backend.py:47, grouped_mlp.py:116-131). */
float orc_gelu(float v) {
  float v2 = v * v;
  float u = (0.79788456f * v) * fmaf(0.044715f, v2, 1.0f);
  float t = orc_tanh(u);
  return (0.5f * v) * (1.0f + t);
}

void orc_tanh_array(const float* in, int64_t n, float* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_tanh(in[i]);
}
void orc_dgelu_array(const float* in, int64_t n, float* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_dgelu(in[i]);
}
void orc_gelu_array(const float* in, int64_t n, float* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_gelu(in[i]);
}

/*
 * multi_pad_cast_transpose_dgelu for one tensor (reference csrc/multi_pad_fusion.cu:346-438):
 *   x = fp32(dy) * dgelu(fp32(pre));  y = fp8(scale * x);  amax over |x| (:378-382).
 *   Rows >= m read dy = pre = 0, so x = 0 * dgelu(0) = 0 and pad = fp8(scale * 0).
 */
void orc_pad_cast_transpose_dgelu(const uint16_t* dy, const uint16_t* pre, int64_t m, int64_t n, int64_t mpad,
                                  const float* scale, int fmt, uint8_t* out, uint8_t* t, float* amax) {
  float s = scale ? *scale : 1.0f;
  float mx = 0.0f;
  uint8_t pad = orc_f32_to_fp8(s * 0.0f, fmt);
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t j = 0; j < n; ++j) {
      float x = orc_bf16_to_f32(dy[i * n + j]) * orc_dgelu(orc_bf16_to_f32(pre[i * n + j]));
      mx = amax_step(mx, x);
      uint8_t y = orc_f32_to_fp8(s * x, fmt);
      if (out) out[i * n + j] = y;
      t[j * mpad + i] = y;
    }
  }
  for (int64_t j = 0; j < n; ++j)
    for (int64_t i = m; i < mpad; ++i) t[j * mpad + i] = pad;
  if (amax) {
    if ((int32_t)f2u(mx) > (int32_t)f2u(*amax)) *amax = mx;
  }
}

/*
 * One expert's GEMM on dequantised operands, the per-expert loop of the
 * reference's own test oracle (fp8_gmm/test.py:209-214) and the operand
 * convention of every GEMM in the reference (fp8_gmm/backend.py:25,57,
 * csrc/fp8_gmm.h:7-11):  A[m][k] row-major, B[n][k] row-major (K contiguous),
 *   acc[i][j] = sum_k A[i][k] * B[j][k]
 * accumulated in double and returned as fp32 (the "fp32 dequantised matmul").
 * lda / ldb are row pitches in elements.
 */
void orc_gemm_f32(const uint8_t* a, int fmt_a, const uint8_t* b, int fmt_b, int64_t m, int64_t n, int64_t k,
                  int64_t lda, int64_t ldb, float* c) {
  float lut_a[256], lut_b[256];
  for (int i = 0; i < 256; ++i) {
    lut_a[i] = orc_fp8_to_f32((uint8_t)i, fmt_a);
    lut_b[i] = orc_fp8_to_f32((uint8_t)i, fmt_b);
  }
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      double acc = 0.0;
      const uint8_t* ar = a + i * lda;
      const uint8_t* br = b + j * ldb;
      for (int64_t kk = 0; kk < k; ++kk) acc += (double)lut_a[ar[kk]] * (double)lut_b[br[kk]];
      c[i * n + j] = (float)acc;
    }
}

/*
 * GEMM epilogues (what cuBLASLt does for the reference through
 * fp8_gmm/backend.py:26-54): v = acc * (a_scale_inv * b_scale_inv);
 *   plain   : c = bf16(v)
 *   gelu-aux: pre = bf16(v); g = gelu(v); c = fp8(g * c_scale); amax = max|g|
 */
void orc_epilogue_bf16(const float* acc, int64_t n, float sa, float sb, uint16_t* c) {
  float s = sa * sb;
  for (int64_t i = 0; i < n; ++i) c[i] = orc_f32_to_bf16(acc[i] * s);
}

void orc_epilogue_gelu_fp8(const float* acc, int64_t n, float sa, float sb, const float* c_scale, int fmt,
                           uint16_t* pre, uint8_t* c, float* amax) {
  float s = sa * sb;
  float cs = c_scale ? *c_scale : 1.0f;
  float mx = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float v = acc[i] * s;
    if (pre) pre[i] = orc_f32_to_bf16(v);
    float g = orc_gelu(v);
    mx = amax_step(mx, g);
    c[i] = orc_f32_to_fp8(g * cs, fmt);
  }
  if (amax) {
    if ((int32_t)f2u(mx) > (int32_t)f2u(*amax)) *amax = mx;
  }
}

/* The data-gradient epilogue with the GELU's derivative folded in (no reference kernel: the reference forms the
 * product in a separate pass from the bf16-rounded GEMM result, fp8_gmm/grouped_mlp.py:243-287, and notes the missing
 * fusion at :252-253):  v = acc * (sa * sb);  x = v * dgelu(pre);  c = fp8(x * c_scale);  amax = max|x|.
 * dgelu is the function of the cast kernels (multi_pad_fusion.cu:39-44), v is NOT rounded to bf16 first. */
void orc_epilogue_dgelu_fp8(const float* acc, int64_t n, float sa, float sb, const float* c_scale, int fmt,
                            const uint16_t* pre, uint8_t* c, float* amax) {
  float s = sa * sb;
  float cs = c_scale ? *c_scale : 1.0f;
  float mx = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float v = acc[i] * s;
    float x = v * orc_dgelu(orc_bf16_to_f32(pre[i]));
    mx = amax_step(mx, x);
    c[i] = orc_f32_to_fp8(x * cs, fmt);
  }
  if (amax) {
    if ((int32_t)f2u(mx) > (int32_t)f2u(*amax)) *amax = mx;
  }
}
