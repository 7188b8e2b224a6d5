// C-ABI entry points of the grouped GEMM and the kernel that completes tiles shared along K.  The main kernel
// lives in grouped_gemm_kernel.h and is instantiated per operand format / layout in gemm_variant.hip.
//
// Replaces the reference's CUTLASS grouped GEMM (csrc/fp8_gmm.cu:82-205) and its per-expert cuBLASLt loops
// (fp8_gmm/backend.py:84-96, grouped_linear.py:173-182, grouped_mlp.py:234-242,313-322) with ONE launch over
// device-side tables written by the host planner (plan.cpp).
#include "grouped_gemm_kernel.h"
#include "internal.h"

// Scratch of fp8gmm_grouped_gemm_static: the tail-balancing workspace for callers that cannot allocate one.
// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.
// In host code the name stands for the symbol, not for device memory: the per-device address is looked up once
// (scratch_for) and only that address is ever handed to a kernel.
constexpr int kStaticSlots = FP8GMM_GEMM_STATIC_SLOTS;
static __device__ __align__(256) uint8_t scratch[(size_t)kStaticSlots * FP8GMM_GEMM_SLOT_BYTES];

namespace fp8gmm {
namespace {

// Completes the tiles that the main kernel shared along K.  MT workgroups per such tile (one record of the
// fix-up list): together they add the tile's pieces, which lie in consecutive workspace slots in K order, and
// apply the epilogue.  A launch has few shared tiles (64 at most on 256 compute units), each with a megabyte of
// partial sums to read: four workgroups per tile put the whole chip to it.
// 1024 threads: thread T owns the 16-byte groups T + 1024 q of a slot, i.e. register group g = T / 256 of the
// MFMA tiles (i, j) = q of main-kernel thread T % 256: 4 consecutive columns of one row each; workgroup `part`
// of a tile takes i = part (q = part * NT .. part * NT + NT - 1).  The sums and the arithmetic are those of
// tile_epilogue's general paths, so a shared tile gets the same bits as a whole one.
constexpr int kFixupThreads = 1024;
constexpr int kFixupSplit = MT;  // workgroups per shared tile
static_assert(kFixupThreads == 4 * NTHREADS, "one register group of every MFMA tile per thread");

__global__ __launch_bounds__(kFixupThreads) void grouped_gemm_fixup_kernel(
    const fp8gmm_gemm_problem* __restrict__ probs, const fp8gmm_gemm_fixup_desc* __restrict__ fixups, int out_kind,
    int epilogue, const uint8_t* __restrict__ workspace) {
  const fp8gmm_gemm_fixup_desc fx = fixups[blockIdx.x / kFixupSplit];
  const int part = blockIdx.x % kFixupSplit;
  const fp8gmm_gemm_problem pr = probs[fx.prob];
  const int m0 = fx.m0, n0 = fx.n0;

  const int t = threadIdx.x % NTHREADS, g = threadIdx.x / NTHREADS;
  const int lane = t & 63, wave = t >> 6;
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int l32 = lane & 31, khalf = lane >> 5;

  f32x4 sum[NT];
  {
    const f32x4* first = reinterpret_cast<const f32x4*>(workspace + (size_t)fx.first_slot * kPartialBytes) +
                         (size_t)part * NT * kFixupThreads + threadIdx.x;
#pragma unroll
    for (int q = 0; q < NT; ++q) sum[q] = __builtin_nontemporal_load(first + q * kFixupThreads);
  }
  for (int w = 1; w < fx.n_pieces; ++w) {
    const f32x4* next = reinterpret_cast<const f32x4*>(workspace + (size_t)(fx.first_slot + w) * kPartialBytes) +
                        (size_t)part * NT * kFixupThreads + threadIdx.x;
    f32x4 piece[NT];
#pragma unroll
    for (int q = 0; q < NT; ++q) piece[q] = __builtin_nontemporal_load(next + q * kFixupThreads);
#pragma unroll
    for (int q = 0; q < NT; ++q) sum[q] += piece[q];
  }

  const int M = pr.m, N = pr.n;
  const float sa_inv = pr.a_scale_inv ? *pr.a_scale_inv : 1.f;
  const float sb_inv = pr.b_scale_inv ? *pr.b_scale_inv : 1.f;
  const float s = sa_inv * sb_inv;
  const bool gelu = (epilogue & FP8GMM_EPI_GELU) != 0;
  const bool dgelu_in = (epilogue & FP8GMM_EPI_DGELU) != 0 && pr.aux != nullptr;   // aux is then an input
  const int64_t ldc = pr.ldc;
  uint16_t* __restrict__ AUX = static_cast<uint16_t*>(pr.aux);
  const bool aux_ok = AUX == nullptr || (reinterpret_cast<uintptr_t>(AUX) & 7) == 0;
  const float cs = pr.c_scale ? *pr.c_scale : 1.f;
  float amax = 0.f;
#pragma unroll
  for (int q = 0; q < NT; ++q) {
    const int i = part, jj = q;
    const int m = m0 + wave_m * WM + i * 32 + l32;
    const int n = n0 + wave_n * WN + jj * 32 + g * 8 + khalf * 4;
    if (m >= M || n >= N) continue;
    float v[4], r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[e] = sum[q][e] * s;
      r[e] = gelu ? gelu_tanh_fast(v[e]) : v[e];
    }
    const int64_t off = (int64_t)m * ldc + n;
    if (dgelu_in) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) r[e] = v[e] * dgelu(bf16_to_f32(AUX[off + e]));
    }
    if (out_kind == FP8GMM_OUT_BF16) {
      uint16_t* __restrict__ C = static_cast<uint16_t*>(pr.c);
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0) && aux_ok;
      if (vec && n + 3 < N) {
        const u32x2 o = {pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
        global_store(C + off, o);
        if (gelu && AUX != nullptr) {
          const u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          global_store(AUX + off, a);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (n + e < N) {
            global_store(C + off + e, (uint16_t)f32_to_bf16_bits(r[e]));
            if (gelu && AUX != nullptr) global_store(AUX + off + e, (uint16_t)f32_to_bf16_bits(v[e]));
          }
        }
      }
    } else {
      uint8_t* __restrict__ C = static_cast<uint8_t*>(pr.c);
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 3) == 0) && aux_ok;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) amax = amax_step(amax, r[e]);
      uint32_t w;
      if (out_kind == FP8GMM_E4M3) {
        w = cvt4_fp8<FP8GMM_E4M3>(r[0] * cs, r[1] * cs, r[2] * cs, r[3] * cs);
      } else {
        w = cvt4_fp8<FP8GMM_E5M2>(r[0] * cs, r[1] * cs, r[2] * cs, r[3] * cs);
      }
      if (vec && n + 3 < N) {
        global_store(C + off, w);
        if (gelu && AUX != nullptr) {
          const u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          global_store(AUX + off, a);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (n + e < N) {
            global_store(C + off + e, (uint8_t)(w >> (8 * e)));
            if (gelu && AUX != nullptr) global_store(AUX + off + e, (uint16_t)f32_to_bf16_bits(v[e]));
          }
        }
      }
    }
  }
  if (out_kind != FP8GMM_OUT_BF16 && pr.c_amax != nullptr) {
    amax = wave_max(amax);
    if (lane == 0 && amax > 0.f && !(__builtin_nontemporal_load(pr.c_amax) >= amax)) atomic_max_nonneg(pr.c_amax, amax);
  }
}


// compute-unit count per device, looked up once (fp8gmm_init, or the first launch on the device)
std::atomic<int> g_num_cu[kMaxDevices];

int device_num_cu(int dev) {
  if (dev < 0 || dev >= kMaxDevices) return FP8GMM_ERR_NO_DEVICE;
  int cus = g_num_cu[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return FP8GMM_ERR_NO_DEVICE;
    cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    g_num_cu[dev].store(cus, std::memory_order_relaxed);
  }
  return cus;
}

// device address of `scratch` on device `dev`, which must be the current device; looked up once per device
std::atomic<uint8_t*> g_scratch[kMaxDevices];

int scratch_for(int dev, uint8_t** out) {
  if (dev < 0 || dev >= kMaxDevices) return FP8GMM_ERR_NO_DEVICE;
  uint8_t* p = g_scratch[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* addr = nullptr;
    if (hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)) != hipSuccess || addr == nullptr) {
      (void)hipGetLastError();
      return FP8GMM_ERR_NO_DEVICE;
    }
    p = static_cast<uint8_t*>(addr);
    g_scratch[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return FP8GMM_OK;
}

typedef int (*launch_fn)(const fp8gmm_gemm_problem*, const fp8gmm_gemm_item*, int, int, int, uint8_t*,
                         const fp8gmm_tensor_desc*, int, hipStream_t);

// the variant for a format / layout combination, or null when the combination does not exist
launch_fn variant_for(int a_fmt, int b_fmt, bool a_kmajor, bool b_kmajor, int tile) {
#define FP8GMM_PICK(AF, BF, AT, BT, TL)                                              \
  if (a_fmt == AF && b_fmt == BF && a_kmajor == AT && b_kmajor == BT && tile == TL) \
    return &launch_variant<AF, BF, AT, BT, TL>;
  FP8GMM_FOR_EACH_GEMM_VARIANT(FP8GMM_PICK)
#undef FP8GMM_PICK
  return nullptr;
}

int launch_checked(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                   const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt, int b_fmt,
                   int out_kind, int epilogue, void* workspace, size_t workspace_bytes, void* stream,
                   const fp8gmm_tensor_desc* merge_descs = nullptr, int merge_n = 0) {
  if (plan == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if (merge_n < 0 || (merge_n > 0 && merge_descs == nullptr)) return FP8GMM_ERR_BAD_ARGUMENT;
  if (n < 0 || plan->total_tiles < 0 || plan->rounds < 0 || plan->n_fixups < 0 || plan->n_slots < 0)
    return FP8GMM_ERR_BAD_ARGUMENT;
  if (out_kind != FP8GMM_OUT_BF16 && out_kind != FP8GMM_E4M3 && out_kind != FP8GMM_E5M2) return FP8GMM_ERR_BAD_FORMAT;
  if (epilogue & ~(FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU | FP8GMM_GEMM_A_KMAJOR | FP8GMM_GEMM_B_KMAJOR))
    return FP8GMM_ERR_BAD_ARGUMENT;
  if ((epilogue & FP8GMM_EPI_GELU) && (epilogue & FP8GMM_EPI_DGELU)) return FP8GMM_ERR_BAD_ARGUMENT;
  const bool a_kmajor = (epilogue & FP8GMM_GEMM_A_KMAJOR) != 0;
  const bool b_kmajor = (epilogue & FP8GMM_GEMM_B_KMAJOR) != 0;
  if (a_kmajor && !b_kmajor) return FP8GMM_ERR_BAD_ARGUMENT;
  if ((a_fmt != FP8GMM_E4M3 && a_fmt != FP8GMM_E5M2) || (b_fmt != FP8GMM_E4M3 && b_fmt != FP8GMM_E5M2))
    return FP8GMM_ERR_BAD_FORMAT;
  // e5m2 x e5m2 does not exist (cuBLASLt rejects it too); the contraction-major forms are the gradient GEMMs,
  // whose b is a forward tensor (weight or activation), always e4m3
  int tile = plan->tile == 0 ? kGemmTileN : plan->tile;
  if (tile != kGemmTileN && tile != FP8GMM_GEMM_SMALL_TILE) return FP8GMM_ERR_BAD_ARGUMENT;
  if (plan->tile_m != 0 && plan->tile_m != tile) {
    // the form with two sets of accumulators: bf16 results only
    if (tile != kGemmTileN || plan->tile_m != FP8GMM_GEMM_DUAL_TILE_M || out_kind != FP8GMM_OUT_BF16)
      return FP8GMM_ERR_BAD_ARGUMENT;
    tile = kTileDual;
  }
  // only the large tile is ever shared along K or has the fused epilogues
  if (tile != kGemmTileM &&
      (plan->n_slots != 0 || plan->n_fixups != 0 || (epilogue & (FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU))))
    return FP8GMM_ERR_BAD_ARGUMENT;
  const launch_fn launch = variant_for(a_fmt, b_fmt, a_kmajor, b_kmajor, tile);
  if (launch == nullptr) return FP8GMM_ERR_BAD_FORMAT;
  if (n == 0 || plan->total_tiles == 0) return merge_n > 0 ? FP8GMM_ERR_BAD_ARGUMENT : FP8GMM_OK;   // nothing would merge
  if (plan->grid <= 0 || (plan->grid % kNumXcd) != 0 || plan->rounds < 1) return FP8GMM_ERR_BAD_ARGUMENT;
  if (probs_dev == nullptr || items_dev == nullptr || (plan->n_fixups > 0 && fixups_dev == nullptr))
    return FP8GMM_ERR_NULL_POINTER;
  if (plan->n_slots > 0 && (workspace == nullptr || workspace_bytes < (size_t)plan->n_slots * kPartialBytes ||
                            (reinterpret_cast<uintptr_t>(workspace) & 255) != 0))
    return FP8GMM_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int rc = launch(probs_dev, items_dev, plan->grid, out_kind, epilogue & (FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU),
                        static_cast<uint8_t*>(workspace), merge_descs, merge_n, s);
  if (rc != FP8GMM_OK) return rc;
  if (plan->n_fixups > 0) {
    hipLaunchKernelGGL(grouped_gemm_fixup_kernel, dim3(plan->n_fixups * kFixupSplit), dim3(kFixupThreads), 0, s, probs_dev,
                       fixups_dev, out_kind, epilogue & (FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU),
                       static_cast<const uint8_t*>(workspace));
    if (hipGetLastError() != hipSuccess) return FP8GMM_ERR_LAUNCH;
  }
  return FP8GMM_OK;
}

}  // namespace

int launch_gemm_merging(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                        const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt, int b_fmt,
                        int out_kind, int epilogue, void* workspace, size_t workspace_bytes,
                        const fp8gmm_tensor_desc* merge_descs, int merge_n, void* stream) {
  return launch_checked(probs_dev, n, items_dev, fixups_dev, plan, a_fmt, b_fmt, out_kind, epilogue, workspace,
                        workspace_bytes, stream, merge_descs, merge_n);
}

}  // namespace fp8gmm

extern "C" {

void fp8gmm_gemm_tile_shape(int* tile_m, int* tile_n) {
  if (tile_m) *tile_m = fp8gmm::BM;
  if (tile_n) *tile_n = fp8gmm::BN;
}

int fp8gmm_init(int device) {
  using namespace fp8gmm;
  int current = 0;
  if (hipGetDevice(&current) != hipSuccess) return FP8GMM_ERR_NO_DEVICE;
  const int dev = device < 0 ? current : device;
  if (dev != current && hipSetDevice(dev) != hipSuccess) return FP8GMM_ERR_NO_DEVICE;
  int rc = device_num_cu(dev);
#define FP8GMM_PREPARE(AF, BF, AT, BT, TL)                  \
  if (rc > 0) {                                             \
    const int e = prepare_variant<AF, BF, AT, BT, TL>(dev); \
    if (e != FP8GMM_OK) rc = e;                             \
  }
  FP8GMM_FOR_EACH_GEMM_VARIANT(FP8GMM_PREPARE)
#undef FP8GMM_PREPARE
  if (rc > 0) {
    uint8_t* unused = nullptr;
    const int e = scratch_for(dev, &unused);
    if (e != FP8GMM_OK) rc = e;
  }
  if (dev != current) (void)hipSetDevice(current);
  return rc;
}

int fp8gmm_grouped_gemm(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                        const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt, int b_fmt,
                        int out_kind, int epilogue, void* workspace, size_t workspace_bytes, void* stream) {
  return fp8gmm::launch_checked(probs_dev, n, items_dev, fixups_dev, plan, a_fmt, b_fmt, out_kind, epilogue, workspace,
                                workspace_bytes, stream);
}

int fp8gmm_grouped_gemm_static(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                               const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt,
                               int b_fmt, int out_kind, int epilogue, void* stream) {
  using namespace fp8gmm;
  if (plan == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if (plan->n_slots > kStaticSlots) return FP8GMM_ERR_WORKSPACE;  // plan the launch with stream_k = 0, or pass a workspace
  uint8_t* ws = nullptr;
  if (plan->n_slots > 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return FP8GMM_ERR_NO_DEVICE;
    const int rc = scratch_for(dev, &ws);
    if (rc != FP8GMM_OK) return rc;
  }
  return launch_checked(probs_dev, n, items_dev, fixups_dev, plan, a_fmt, b_fmt, out_kind, epilogue, ws,
                        (size_t)kStaticSlots * FP8GMM_GEMM_SLOT_BYTES, stream);
}

}  // extern "C"
