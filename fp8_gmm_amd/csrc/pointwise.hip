// Multi-tensor element-wise kernels for gfx950: quantize (bf16 -> fp8 + amax) and
// scale_mul (in-place bf16 *= s1 * s2).  One launch covers every tensor of the call;
// each workgroup finds its tensor by a binary search over a device-side table.
//
// Replaces csrc/multi_pointwise.cu of the reference (multi_quantize_kernel :34-97,
// multi_scale_mul_kernel :99-151).  HBM-bound: 2 B read + 1 B written per element
// (quantize), 2 B + 2 B (scale_mul); a wavefront reads 1 KB of contiguous bf16 per step
// (one 128-bit load per lane, all steps issued before the first conversion), the wave reduces amax with cross-lane shuffles and the
// workgroup issues a single integer atomic max.
#include "device_utils.h"
#include "internal.h"
#include "tiling.h"

namespace fp8gmm {
namespace {

// DGELU: the value cast is x = in * dgelu(in2) (in = gradient of the GELU output, in2 = pre-GELU activation),
// the same product, in the same order, as the transposing kernel forms.
template <int FMT, bool DGELU>
__global__ __launch_bounds__(kPwThreads) void multi_quantize_kernel(fp8gmm_tensor_desc* __restrict__ descs, int n) {
  __shared__ float stage[kPwThreads / kWaveSize];
  const int bid = blockIdx.x;
  const int t = upper_slot(n, bid, [&](int i) { return descs[i].block_begin; });
  const fp8gmm_tensor_desc d = descs[t];
  const int64_t numel = (int64_t)d.rows * d.cols;
  const int64_t base = (int64_t)(bid - d.block_begin) * kPwBlockElems;
  const uint16_t* __restrict__ in = static_cast<const uint16_t*>(d.in);
  const uint16_t* __restrict__ pre = static_cast<const uint16_t*>(d.in2);
  uint8_t* __restrict__ out = static_cast<uint8_t*>(d.out);
  const float scale = d.scale ? *d.scale : 1.f;
  const bool vec = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out) |
                     (DGELU ? reinterpret_cast<uintptr_t>(pre) : 0)) & 15) == 0 &&
                   numel * 2 < (int64_t)0xffffffff;
  float mx = 0.f;
  auto value = [&](int64_t j) {
    float x = bf16_to_f32(in[j]);
    if constexpr (DGELU) x *= dgelu(bf16_to_f32(pre[j]));
    return x;
  };

  if (vec) {
    // fast path: all loads of the workgroup's 16384 elements are issued before the first conversion
    const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, (uint32_t)(numel * 2));
    const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, (uint32_t)numel);
    const __amdgpu_buffer_rsrc_t rpre = make_rsrc(DGELU ? pre : in, (uint32_t)(numel * 2));
    u32x4 a[kPwSteps];
    u32x4 g[DGELU ? kPwSteps : 1];
    bool full[kPwSteps];
#pragma unroll
    for (int it = 0; it < kPwSteps; ++it) {
      const int64_t off = base + (int64_t)(it * kPwThreads + threadIdx.x) * kPwVec;
      full[it] = off + kPwVec <= numel;
      a[it] = buf_load16_stream(rin, full[it] ? (uint32_t)(off * 2) : kOobOffset);
      if constexpr (DGELU) g[it] = buf_load16_stream(rpre, full[it] ? (uint32_t)(off * 2) : kOobOffset);
    }
#pragma unroll
    for (int it = 0; it < kPwSteps; ++it) {
      const int64_t off = base + (int64_t)(it * kPwThreads + threadIdx.x) * kPwVec;
      const uint32_t w[4] = {a[it].x, a[it].y, a[it].z, a[it].w};
      uint32_t o[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        float x0 = bf16_lo_to_f32(w[2 * q]), x1 = bf16_hi_to_f32(w[2 * q]);
        float x2 = bf16_lo_to_f32(w[2 * q + 1]), x3 = bf16_hi_to_f32(w[2 * q + 1]);
        if constexpr (DGELU) {
          const uint32_t p[4] = {g[it].x, g[it].y, g[it].z, g[it].w};
          x0 *= dgelu(bf16_lo_to_f32(p[2 * q]));
          x1 *= dgelu(bf16_hi_to_f32(p[2 * q]));
          x2 *= dgelu(bf16_lo_to_f32(p[2 * q + 1]));
          x3 *= dgelu(bf16_hi_to_f32(p[2 * q + 1]));
        }
        mx = amax_step(amax_step(mx, x0), x1);
        mx = amax_step(amax_step(mx, x2), x3);
        o[q] = cvt4_fp8<FMT>(x0 * scale, x1 * scale, x2 * scale, x3 * scale);
      }
      buf_store8(u32x2{o[0], o[1]}, rout, full[it] ? (uint32_t)off : kOobOffset);
      if (!full[it] && off < numel) {  // the one partial group at the end of the tensor
        for (int64_t j = off; j < numel; ++j) {
          const float x = value(j);
          mx = amax_step(mx, x);
          out[j] = cvt1_fp8<FMT>(x * scale);
        }
      }
    }
  } else {
#pragma unroll 1
    for (int it = 0; it < kPwSteps; ++it) {
      const int64_t off = base + (int64_t)(it * kPwThreads + threadIdx.x) * kPwVec;
      if (off < numel) {
        const int cnt = (numel - off < kPwVec) ? (int)(numel - off) : kPwVec;
        for (int j = 0; j < cnt; ++j) {
          const float x = value(off + j);
          mx = amax_step(mx, x);
          out[off + j] = cvt1_fp8<FMT>(x * scale);
        }
      }
    }
  }
  block_amax_merge<kPwThreads / kWaveSize>(mx, d.amax != nullptr ? &descs[t].amax_partial : nullptr, stage);
}

__global__ __launch_bounds__(kPwThreads) void multi_scale_mul_kernel(const fp8gmm_tensor_desc* __restrict__ descs,
                                                                     int n) {
  const int bid = blockIdx.x;
  const int t = upper_slot(n, bid, [&](int i) { return descs[i].block_begin; });
  const fp8gmm_tensor_desc d = descs[t];
  const int64_t numel = (int64_t)d.rows * d.cols;
  const int64_t base = (int64_t)(bid - d.block_begin) * kPwBlockElems;
  // in-place: `in` is the tensor being scaled
  uint16_t* __restrict__ x = const_cast<uint16_t*>(static_cast<const uint16_t*>(d.in));
  const float s1 = d.scale ? *d.scale : 1.f;
  const float* s2p = static_cast<const float*>(d.in2);
  const float s2 = s2p ? *s2p : 1.f;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && numel * 2 < (int64_t)0xffffffff;

  if (vec) {
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, (uint32_t)(numel * 2));
    u32x4 a[kPwSteps];
    bool full[kPwSteps];
#pragma unroll
    for (int it = 0; it < kPwSteps; ++it) {
      const int64_t off = base + (int64_t)(it * kPwThreads + threadIdx.x) * kPwVec;
      full[it] = off + kPwVec <= numel;
      a[it] = buf_load16_stream(rx, full[it] ? (uint32_t)(off * 2) : kOobOffset);
    }
#pragma unroll
    for (int it = 0; it < kPwSteps; ++it) {
      const int64_t off = base + (int64_t)(it * kPwThreads + threadIdx.x) * kPwVec;
      uint32_t w[4] = {a[it].x, a[it].y, a[it].z, a[it].w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        // left to right, as the reference: (x * s1) * s2
        const float lo = bf16_lo_to_f32(w[q]) * s1 * s2;
        const float hi = bf16_hi_to_f32(w[q]) * s1 * s2;
        w[q] = pack_bf16x2(lo, hi);
      }
      buf_store16(u32x4{w[0], w[1], w[2], w[3]}, rx, full[it] ? (uint32_t)(off * 2) : kOobOffset);
      if (!full[it] && off < numel) {
        for (int64_t j = off; j < numel; ++j) x[j] = (uint16_t)f32_to_bf16_bits(bf16_to_f32(x[j]) * s1 * s2);
      }
    }
  } else {
#pragma unroll 1
    for (int it = 0; it < kPwSteps; ++it) {
      const int64_t off = base + (int64_t)(it * kPwThreads + threadIdx.x) * kPwVec;
      if (off < numel) {
        const int cnt = (numel - off < kPwVec) ? (int)(numel - off) : kPwVec;
        for (int j = 0; j < cnt; ++j) x[off + j] = (uint16_t)f32_to_bf16_bits(bf16_to_f32(x[off + j]) * s1 * s2);
      }
    }
  }
}

// Delayed-scaling update of one direction, one lane per scaling slot (columns of the [history, slots]
// amax matrix are independent, rows of a column are walked by the lane that owns it):
//   amax      = max over the history column (or its row 0)
//   scale     = (1 / amax) * fp8_max * 2^-margin   where amax is finite and > 0, else unchanged
//   scale_inv = 1 / scale, except in slots with slot % keep_period == keep_phase (keep_period > 0): those
//               keep their value, for tensors whose fp8 copy from an earlier pass is still in use
//   history   : row i <- row i + 1, last row <- old row 0, then row 0 <- 0 (a history of one row is just cleared)
// The factor is formed as reciprocal times fp8_max, which is what `fp8_max / amax` on a torch tensor
// evaluates to; the two differ in the last bit for some inputs.
__device__ __forceinline__ void delayed_scaling_update_column(float* __restrict__ history, float* __restrict__ scale,
                                                               float* __restrict__ scale_inv, int history_len, int slots,
                                                               float fp8_max, float margin_factor, int most_recent,
                                                               int keep_period, int keep_phase, int c) {
  if (c >= slots) return;
  float* col = history + c;
  const float first = col[0];
  float sc = scale[c];
  float amax = first;
  // The column is walked once, eight rows at a time: the loads of a group are issued together (one round trip to
  // memory per group, not per row - the rows are written through the same pointer they are read from, so the
  // compiler keeps loads and stores of a row-by-row loop in order), the maximum is taken, and the rows are written
  // one place up.  A group's stores end one row below its loads and the next group's loads start above them.
  constexpr int kGroup = 8;
  for (int base = 1; base < history_len; base += kGroup) {
    float v[kGroup];
#pragma unroll
    for (int j = 0; j < kGroup; ++j) v[j] = base + j < history_len ? col[(size_t)(base + j) * slots] : 0.f;
#pragma unroll
    for (int j = 0; j < kGroup; ++j) {
      if (base + j < history_len) {
        // torch.max semantics: a NaN anywhere in the column wins
        if (!most_recent) amax = (v[j] > amax || v[j] != v[j]) ? v[j] : amax;
        col[(size_t)(base + j - 1) * slots] = v[j];
      }
    }
  }
  if (amax > 0.f && amax <= 3.4028234663852886e38f) sc = ((1.0f / amax) * fp8_max) * margin_factor;
  scale[c] = sc;
  if (!(keep_period > 0 && c % keep_period == keep_phase)) scale_inv[c] = 1.0f / sc;
  if (history_len > 1) col[(size_t)(history_len - 1) * slots] = first;
  col[0] = 0.f;
}

__global__ __launch_bounds__(256) void delayed_scaling_update_kernel(float* __restrict__ history,
                                                                     float* __restrict__ scale,
                                                                     float* __restrict__ scale_inv, int history_len,
                                                                     int slots, float fp8_max, float margin_factor,
                                                                     int most_recent, int keep_period,
                                                                     int keep_phase) {
  delayed_scaling_update_column(history, scale, scale_inv, history_len, slots, fp8_max, margin_factor, most_recent,
                                keep_period, keep_phase, blockIdx.x * blockDim.x + threadIdx.x);
}

// Several directions (a module's forward and backward scaling state) in one launch: the workgroups of update u
// follow those of update u - 1.  The updates travel as a kernel argument.
struct ScalingUpdates {
  fp8gmm_scaling_update u[FP8GMM_MAX_SCALING_UPDATES];
  float margin_factor[FP8GMM_MAX_SCALING_UPDATES];
  int first_block[FP8GMM_MAX_SCALING_UPDATES + 1];
  int n;
};
__global__ __launch_bounds__(256) void delayed_scaling_updates_kernel(const ScalingUpdates all) {
  int i = 0;
  while (i + 1 < all.n && (int)blockIdx.x >= all.first_block[i + 1]) ++i;
  const fp8gmm_scaling_update& u = all.u[i];
  delayed_scaling_update_column(u.amax_history, u.scale, u.scale_inv, u.history_len, u.slots, u.fp8_max,
                                all.margin_factor[i], u.most_recent, u.keep_period, u.keep_phase,
                                ((int)blockIdx.x - all.first_block[i]) * (int)blockDim.x + (int)threadIdx.x);
}

}  // namespace
}  // namespace fp8gmm

namespace {
template <bool DGELU>
int launch_quantize(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, void* stream, bool merge = true) {
  if (n < 0 || total_blocks < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (out_fmt != FP8GMM_E4M3 && out_fmt != FP8GMM_E5M2) return FP8GMM_ERR_BAD_FORMAT;
  if (n == 0 || total_blocks == 0) return FP8GMM_OK;
  if (descs_dev == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (out_fmt == FP8GMM_E4M3)
    hipLaunchKernelGGL((fp8gmm::multi_quantize_kernel<FP8GMM_E4M3, DGELU>), dim3(total_blocks),
                       dim3(fp8gmm::kPwThreads), 0, s, descs_dev, n);
  else
    hipLaunchKernelGGL((fp8gmm::multi_quantize_kernel<FP8GMM_E5M2, DGELU>), dim3(total_blocks),
                       dim3(fp8gmm::kPwThreads), 0, s, descs_dev, n);
  if (merge) hipLaunchKernelGGL(fp8gmm::amax_merge_kernel, dim3((n + 255) / 256), dim3(256), 0, s, descs_dev, n);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}
}  // namespace

namespace fp8gmm {
int launch_cast_unmerged(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, bool dgelu, void* stream) {
  return dgelu ? launch_quantize<true>(descs_dev, n, total_blocks, out_fmt, stream, false)
               : launch_quantize<false>(descs_dev, n, total_blocks, out_fmt, stream, false);
}
}  // namespace fp8gmm

namespace fp8gmm {
// Tables travel host -> device through this kernel: it reads page-locked host memory that is mapped into the
// device's address space, 16 bytes per thread, and writes device memory.  A copy enqueued with hipMemcpyAsync runs
// as a transfer of its own whose hand-over to the next kernel of the stream took 25 - 30 us on this machine; a
// kernel of the stream hands over like any other kernel.
__global__ void __launch_bounds__(256) upload_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                     unsigned pieces) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i < pieces) dst[i] = src[i];
}
}  // namespace fp8gmm

extern "C" {

int fp8gmm_delayed_scaling_update(float* amax_history, float* scale, float* scale_inv, int history_len, int slots,
                                  float fp8_max, int margin, int most_recent, int keep_period, int keep_phase,
                                  void* stream) {
  if (history_len < 1 || slots < 0 || margin < -126 || margin > 126) return FP8GMM_ERR_BAD_ARGUMENT;
  if (keep_period < 0 || (keep_period > 0 && (keep_phase < 0 || keep_phase >= keep_period)))
    return FP8GMM_ERR_BAD_ARGUMENT;
  if (slots == 0) return FP8GMM_OK;
  if (amax_history == nullptr || scale == nullptr || scale_inv == nullptr) return FP8GMM_ERR_NULL_POINTER;
  const float margin_factor = __builtin_ldexpf(1.0f, -margin);
  hipLaunchKernelGGL(fp8gmm::delayed_scaling_update_kernel, dim3((slots + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), amax_history, scale, scale_inv, history_len, slots, fp8_max,
                     margin_factor, most_recent != 0, keep_period, keep_phase);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_delayed_scaling_updates(const fp8gmm_scaling_update* updates, int n, void* stream) {
  if (n < 0 || n > FP8GMM_MAX_SCALING_UPDATES) return FP8GMM_ERR_BAD_ARGUMENT;
  if (n == 0) return FP8GMM_OK;
  if (updates == nullptr) return FP8GMM_ERR_NULL_POINTER;
  fp8gmm::ScalingUpdates all{};
  int blocks = 0;
  for (int i = 0; i < n; ++i) {
    const fp8gmm_scaling_update& u = updates[i];
    if (u.history_len < 1 || u.slots < 0 || u.margin < -126 || u.margin > 126) return FP8GMM_ERR_BAD_ARGUMENT;
    if (u.keep_period < 0 || (u.keep_period > 0 && (u.keep_phase < 0 || u.keep_phase >= u.keep_period)))
      return FP8GMM_ERR_BAD_ARGUMENT;
    if (u.slots > 0 && (u.amax_history == nullptr || u.scale == nullptr || u.scale_inv == nullptr))
      return FP8GMM_ERR_NULL_POINTER;
    all.u[i] = u;
    all.margin_factor[i] = __builtin_ldexpf(1.0f, -u.margin);
    all.first_block[i] = blocks;
    blocks += (u.slots + 255) / 256;
  }
  all.first_block[n] = blocks;
  all.n = n;
  if (blocks == 0) return FP8GMM_OK;
  hipLaunchKernelGGL(fp8gmm::delayed_scaling_updates_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     all);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_multi_quantize(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, void* stream) {
  return launch_quantize<false>(descs_dev, n, total_blocks, out_fmt, stream);
}

int fp8gmm_multi_cast_dgelu(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, void* stream) {
  return launch_quantize<true>(descs_dev, n, total_blocks, out_fmt, stream);
}

int fp8gmm_multi_scale_mul(const fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, void* stream) {
  if (n < 0 || total_blocks < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (n == 0 || total_blocks == 0) return FP8GMM_OK;
  if (descs_dev == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipLaunchKernelGGL(fp8gmm::multi_scale_mul_kernel, dim3(total_blocks), dim3(fp8gmm::kPwThreads), 0,
                     static_cast<hipStream_t>(stream), descs_dev, n);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

void* fp8gmm_host_alloc(size_t bytes) {
  if (bytes == 0) return nullptr;
  // while a stream is being captured the runtime refuses allocations from any thread; this one is safe there (it
  // touches no stream), so the calling thread's capture mode is relaxed for its duration
  hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
  const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
  void* p = nullptr;
  const hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocDefault);
  if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return p;
}

void fp8gmm_host_free(void* p) {
  if (p == nullptr) return;
  hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
  const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
  (void)hipHostFree(p);
  if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
}

int fp8gmm_upload(void* dst_dev, const void* src_host, size_t bytes, void* stream) {
  if (bytes == 0) return FP8GMM_OK;
  if (dst_dev == nullptr || src_host == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if (((reinterpret_cast<uintptr_t>(dst_dev) | reinterpret_cast<uintptr_t>(src_host) | bytes) & 15) != 0)
    return FP8GMM_ERR_ALIGNMENT;
  if (bytes > (size_t(1) << 30)) return FP8GMM_ERR_BAD_ARGUMENT;
  const unsigned pieces = (unsigned)(bytes / 16);
  hipLaunchKernelGGL(fp8gmm::upload_kernel, dim3((pieces + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint4*>(dst_dev),
                     static_cast<const uint4*>(src_host), pieces);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

}  // extern "C"
