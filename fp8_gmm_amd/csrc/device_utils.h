// Device-side helpers shared by the gfx950 kernels: bf16 / fp8 conversions, the
// deterministic tanh used by the GELU paths, wave64 reductions and the amax merge.
// Counterpart of the reference's csrc/utils.cuh, re-thought for 64-wide wavefronts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fp8gmm.h"

namespace fp8gmm {

constexpr int kWaveSize = 64;

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float bf16_lo_to_f32(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi_to_f32(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// two fp32 -> packed bf16 (element 0 in the low half), round-to-nearest-even: one v_cvt_pk_bf16_f32
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xffffu; }

template <int FMT>
struct Fp8Limits;
template <>
struct Fp8Limits<FP8GMM_E4M3> {
  static constexpr float kMax = 448.0f;
};
template <>
struct Fp8Limits<FP8GMM_E5M2> {
  static constexpr float kMax = 57344.0f;
};

// Two fp32 -> two fp8 bytes in the low (HI = false) or high (HI = true) half of `old`.
// Saturating round-to-nearest-even: |x| >= max (infinities included) -> max finite.
// The median clamps; NaN inputs are patched by the caller (fp8_nan_fix) because the
// median of (NaN, -max, max) is -max.
template <int FMT, bool HI>
__device__ __forceinline__ uint32_t cvt_pk_fp8_sat(float a, float b, uint32_t old) {
  constexpr float mx = Fp8Limits<FMT>::kMax;
  a = __builtin_amdgcn_fmed3f(a, -mx, mx);
  b = __builtin_amdgcn_fmed3f(b, -mx, mx);
  if constexpr (FMT == FP8GMM_E4M3) {
    return __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, HI);
  } else {
    return __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, HI);
  }
}

// Four scaled fp32 values -> one dword of fp8 bytes (element 0 in the low byte).
// NaN becomes 0x7F (positive canonical NaN) whatever its sign.
template <int FMT>
__device__ __forceinline__ uint32_t cvt4_fp8(float v0, float v1, float v2, float v3) {
  uint32_t w = 0;
  w = cvt_pk_fp8_sat<FMT, false>(v0, v1, w);
  w = cvt_pk_fp8_sat<FMT, true>(v2, v3, w);
  if (__builtin_expect((v0 != v0) | (v1 != v1) | (v2 != v2) | (v3 != v3), 0)) {
    if (v0 != v0) w = (w & 0xffffff00u) | 0x0000007fu;
    if (v1 != v1) w = (w & 0xffff00ffu) | 0x00007f00u;
    if (v2 != v2) w = (w & 0xff00ffffu) | 0x007f0000u;
    if (v3 != v3) w = (w & 0x00ffffffu) | 0x7f000000u;
  }
  return w;
}

template <int FMT>
__device__ __forceinline__ uint8_t cvt1_fp8(float v) {
  return (uint8_t)(cvt4_fp8<FMT>(v, 0.f, 0.f, 0.f) & 0xffu);
}

// Store through an explicit global-address-space pointer: a pointer loaded from a table is generic,
// and a generic (flat) store also counts as an LDS operation in the wait counters.
template <typename T>
__device__ __forceinline__ void global_store(void* p, T v) {
  *reinterpret_cast<__attribute__((address_space(1))) T*>(reinterpret_cast<uintptr_t>(p)) = v;
}

// The same with the streaming hint: data that is written once and read once, soon, by another launch.
template <typename T>
__device__ __forceinline__ void global_store_stream(void* p, T v) {
  __builtin_nontemporal_store(v, reinterpret_cast<__attribute__((address_space(1))) T*>(reinterpret_cast<uintptr_t>(p)));
}

// Raw buffer descriptors: offsets past `bytes` read as zero and are dropped on store, so the fast paths
// of the HBM-bound kernels need no per-lane branches and can issue all their loads back to back.
constexpr uint32_t kOobOffset = 0xffffffffu;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
}
__device__ __forceinline__ u32x2 buf_load8(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
}
// The same loads with the streaming hint, for data that is read exactly once (the inputs of the cast, pad and
// transpose kernels): the lines do not stay in L2 behind the read.  Measured on these kernels: 8 % (quantize), 5 %
// (cast + dGELU) and 20 % (pad + cast + transpose) more bandwidth than with plain loads; the hint on the stores as
// well, or on the stores alone, is worse for most of them.
__device__ __forceinline__ u32x4 buf_load16_stream(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 2);
}
__device__ __forceinline__ u32x2 buf_load8_stream(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 2);
}
__device__ __forceinline__ void buf_store16(u32x4 v, __amdgpu_buffer_rsrc_t r, uint32_t off) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)off, 0, 0);
}
__device__ __forceinline__ void buf_store8(u32x2 v, __amdgpu_buffer_rsrc_t r, uint32_t off) {
  __builtin_amdgcn_raw_buffer_store_b64(v, r, (int)off, 0, 0);
}

// max(acc, |x|) that never lets a NaN in (fmaxf semantics of the reference's amax).
// A compare + select, not v_max_f32: in IEEE mode the hardware max returns a NaN when an
// input is a signalling NaN (bf16 data can carry such patterns), which would erase `acc`.
__device__ __forceinline__ float amax_step(float acc, float x) {
  const float ax = fabsf(x);
  return (ax > acc) ? ax : acc;
}

// Wave-wide max of non-negative floats; every lane gets the result.
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWaveSize));
  return v;
}

// Merge a non-negative float into *addr with an integer atomic max on the bit
// pattern (order-free, hence deterministic).  Vector-memory atomic.
__device__ __forceinline__ void atomic_max_nonneg(float* addr, float v) {
  atomicMax(reinterpret_cast<int*>(addr), __float_as_int(v));
}

// Block-wide amax merge for blocks of NWAVES waves. `stage` is NWAVES floats of LDS.  `target` is the
// tensor's own partial-amax word (fp8gmm_tensor_desc::amax_partial), not the caller's amax slot.
template <int NWAVES>
__device__ __forceinline__ void block_amax_merge(float local, uint32_t* target, float* stage) {
  float w = wave_max(local);
  const int lane = threadIdx.x % kWaveSize;
  const int wave = threadIdx.x / kWaveSize;
  if (lane == 0) stage[wave] = w;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = stage[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) m = fmaxf(m, stage[i]);
    // amax only grows, so a value already at or above m (even a stale one) makes the atomic redundant
    float* t = reinterpret_cast<float*>(target);
    if (target != nullptr && m > 0.f && !(__builtin_nontemporal_load(t) >= m)) atomic_max_nonneg(t, m);
  }
}

// Second pass of the calls that record amax: one lane per tensor merges the tensor's partial into the
// caller's slot.  n atomics in total, against one per workgroup of the main kernel.  Run by a launch of its own
// behind the cast, or - inside a planned pass - by the first workgroup of the GEMM launch that follows the cast.
__device__ __forceinline__ void merge_amax_partials(const fp8gmm_tensor_desc* __restrict__ descs, int n, int first,
                                                    int stride) {
  for (int i = first; i < n; i += stride) {
    const float p = __builtin_bit_cast(float, descs[i].amax_partial);
    float* amax = descs[i].amax;
    if (amax != nullptr && p > 0.f) atomic_max_nonneg(amax, p);
  }
}
[[maybe_unused]] static __global__ __launch_bounds__(256) void amax_merge_kernel(const fp8gmm_tensor_desc* __restrict__ descs, int n) {
  merge_amax_partials(descs, n, blockIdx.x * blockDim.x + threadIdx.x, gridDim.x * blockDim.x);
}

// exp(-2a) and 1 / (1 + exp(-2a)) for a >= 0, from a fixed sequence of IEEE single-precision operations (add, mul,
// fma, integer add / shift: no division, no hardware approximation), so that a CPU following the same sequence
// gets the same bits.  Input z = a * 2 / ln 2 >= 0 (NaN is taken as large):
//   z = min(z, 125); n = rne(z) by adding 1.5 * 2^23, f = z - n in [-0.5, 0.5];
//   q = 2^-f * 2^-n: degree-5 minimax polynomial for 2^-f with constant term exactly 1 (1.5e-7 relative; exact at f = 0), the exponent subtracted in the integer
//   domain (the low bits of magic - z hold -n);
//   r = 1 / (1 + q): quadratic first guess on q in [0, 1] (1 % off), two Newton steps r += r (1 - d r).
// tanh(a) = (1 - q) r;  0.5 (1 + tanh(a)) = r;  0.5 (1 - tanh(a)) = q r.
// The dGELU cast is bound by vector arithmetic, not by memory: this sequence is 21 operations where a polynomial
// with one more term, an exactly rounded division and separate rounding steps took 31.
__device__ __forceinline__ void det_exp_rcp(float z, float* q_out, float* r_out) {
  z = __builtin_fminf(z, 125.0f);
  const float magic = 12582912.0f;
  const float zr = magic - z;
  const float nf = zr - magic;
  const float f = z + nf;
  float p = -1.3400432653725147e-3f;
  p = __builtin_fmaf(p, f, 9.666378609836102e-3f);
  p = __builtin_fmaf(p, f, -5.550333112478256e-2f);
  p = __builtin_fmaf(p, f, 2.402234822511673e-1f);
  p = __builtin_fmaf(p, f, -6.931471824645996e-1f);
  p = __builtin_fmaf(p, f, 1.0f);
  const float q = __uint_as_float(__float_as_uint(p) + (__float_as_uint(zr) << 23));
  const float d = 1.0f + q;
  float r = __builtin_fmaf(__builtin_fmaf(0.3232323229312897f, q, -0.808080792427063f), q, 0.9898989796638489f);
  r = __builtin_fmaf(r, __builtin_fmaf(-d, r, 1.0f), r);
  r = __builtin_fmaf(r, __builtin_fmaf(-d, r, 1.0f), r);
  *q_out = q;
  *r_out = r;
}

// |error| < 2e-7.
__device__ __forceinline__ float det_tanh(float u) {
  float q, r;
  det_exp_rcp(fabsf(u) * 2.8853900817779268f, &q, &r);
  const float t = __builtin_copysignf(__builtin_fmaf(-q, r, r), u);
  return (u != u) ? u : t;   // the clamp above takes a NaN for a large value
}

// d/dc of tanh-GELU with the constants of the reference (csrc/multi_pad_fusion.cu:39-44):
//   0.5 c (1 - t^2)(0.79788456 + 0.1070322243 c^2) + 0.5 (1 + t),  t = tanh(u),  u = 0.79788456 c (1 + 0.044715 c^2)
// With s = 0.5 (1 + t) = 1 / (1 + exp(-2u)):  1 - t^2 = 4 s (1 - s), and s (1 - s) = q r^2 for either sign of u, so
//   dgelu = s + c (1.59576912 + 0.2140644486 c^2) q r^2,   s = r for c >= 0, q r otherwise.
__device__ __forceinline__ float dgelu(float c) {
  const float c2 = c * c;
  const float w = __builtin_fmaf(0.044715f, c2, 1.0f);
  float q, r;
  det_exp_rcp(fabsf((2.3022082f * c) * w), &q, &r);   // 2.3022082 = 0.79788456 * 2 / ln 2
  const float t1 = q * r;
  const float s1 = t1 * r;
  const float sig = (c >= 0.0f) ? r : t1;
  const float g2 = __builtin_fmaf(0.2140644486f, c2, 1.59576912f);
  return __builtin_fmaf(c * g2, s1, sig);
}

__device__ __forceinline__ float gelu_tanh(float v) {
  float v2 = v * v;
  float u = (0.79788456f * v) * __builtin_fmaf(0.044715f, v2, 1.0f);
  float t = det_tanh(u);
  return (0.5f * v) * (1.0f + t);
}

// tanh-GELU for the GEMM epilogue: same formula, but tanh through the hardware exp2 / rcp
// approximations (about 1e-6 relative).  The GEMM accumulates in a different order than any CPU
// check anyway, so nothing here has to be bit-reproducible; the dGELU kernel, which is compared
// byte for byte, keeps det_tanh.
__device__ __forceinline__ float gelu_tanh_fast(float v) {
  // 0.5 (1 + tanh(u)) = 1 / (1 + exp(-2u)), u = 0.79788456 (v + 0.044715 v^3); constants carry 2 log2(e).
  const float p = __builtin_fmaf(v * v, 0.10294324f, 2.3022082f);
  const float e = __builtin_amdgcn_exp2f(-v * p);  // exp(-2u); inf for very negative v -> result -0
  return v * __builtin_amdgcn_rcpf(1.0f + e);
}

// Index of the last entry of a sorted device table whose key (read by `key(i)`) is <= x.
// Uniform across the workgroup, so it compiles to scalar loads.
template <typename KeyFn>
__device__ __forceinline__ int upper_slot(int n, int x, KeyFn key) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (key(mid) <= x) lo = mid; else hi = mid - 1;
  }
  return lo;
}

}  // namespace fp8gmm
