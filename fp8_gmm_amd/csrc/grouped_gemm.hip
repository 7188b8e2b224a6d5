// Persistent FP8 grouped GEMM for gfx950 (MI355X).
//
// Replaces the reference's CUTLASS grouped GEMM (csrc/fp8_gmm.cu:82-205) and its
// per-expert cuBLASLt loops (fp8_gmm/backend.py:84-96, grouped_linear.py:173-182,
// grouped_mlp.py:234-242,313-322) with ONE launch over a device-side problem table.
//
//   c[m, n] = epilogue( sum_k a[m, k] * b[n, k] ),   a, b fp8 (K contiguous), fp32 accumulation
//
// Work decomposition
//   * the output of every problem is cut into 256 x 256 tiles; all tiles of all
//     problems form one list, walked by a persistent grid (one workgroup per CU);
//     the list is split into 8 contiguous ranges, one per XCD, so that workgroups
//     sharing an L2 work on neighbouring tiles (workgroup i runs on XCD i % 8);
//   * a workgroup is 8 wavefronts (2 along m x 4 along n); a wavefront owns a
//     128 x 64 sub-tile = 4 x 2 MFMA tiles of v_mfma_f32_32x32x64_f8f6f4;
//   * K is consumed 128 bytes per step through two LDS stages (2 x 64 KB): global
//     loads for step s+1 are issued before the MFMAs of step s and written to the
//     other stage afterwards - one barrier per step;
//   * LDS rows are 128 bytes (one K step) with the 16-byte chunks XOR-swizzled by the
//     row index so that the 16-byte fragment reads of 64 lanes spread over all banks;
//   * the weight operand (b) is fed as MFMA source 0 and the token operand (a) as
//     source 1: the accumulator layout then gives every lane 4 consecutive output
//     columns of one output row, i.e. 8-byte bf16 stores without a shuffle.
//
// Out-of-range rows / K tails are zero-filled on load, so m, n are arbitrary and k
// only has to be a multiple of 16 bytes.
#include "device_utils.h"
#include "tiling.h"

namespace fp8gmm {
namespace {

constexpr int BM = kGemmTileM;   // 256
constexpr int BN = kGemmTileN;   // 256
constexpr int BK = kGemmTileK;   // 128 bytes
constexpr int NTHREADS = 512;
constexpr int WAVES_M = 2;
constexpr int WAVES_N = 4;
constexpr int WM = BM / WAVES_M;  // 128
constexpr int WN = BN / WAVES_N;  // 64
constexpr int MT = WM / 32;       // 4 MFMA tiles along m per wave
constexpr int NT = WN / 32;       // 2 MFMA tiles along n per wave
constexpr int STAGE_BYTES = (BM + BN) * BK;  // 65536
constexpr int A_LOADS = BM * (BK / 16) / NTHREADS;  // 4 x 16-byte chunks per thread
constexpr int B_LOADS = BN * (BK / 16) / NTHREADS;  // 4
constexpr int kNumXcd = 8;

// 16-byte chunk swizzle inside a 128-byte LDS row.
__device__ __forceinline__ int swz(int row) { return row & 7; }

struct TileCoord {
  int prob;
  int m0;
  int n0;
};

template <int A_FMT, int B_FMT>
__global__ __launch_bounds__(NTHREADS) void grouped_gemm_kernel(const fp8gmm_gemm_problem* __restrict__ probs,
                                                                int nprob, int total_tiles, int out_kind,
                                                                int epilogue) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WAVES_N;  // 0..1
  const int wave_n = wave % WAVES_N;  // 0..3
  const int l32 = lane & 31;
  const int khalf = lane >> 5;  // which 32-byte half of a 64-byte MFMA K slice this lane feeds

  // ---- global -> LDS staging map: chunk (row, c) of the 128-byte-wide stage ----
  const int ld_c = tid & 7;     // 16-byte chunk in the K step
  const int ld_r = tid >> 3;    // 0..63, rows ld_r + 64 i
  const int st_off = ld_r * BK + ((ld_c ^ swz(ld_r)) << 4);  // same swizzle for rows ld_r + 64 i (64 % 8 == 0)

  // ---- LDS -> fragment map ----
  // token rows (MFMA source 1):  wave_m * 128 + mt * 32 + l32 ; weight rows (source 0): wave_n * 64 + nt * 32 + l32
  const int frag_row_off = l32 * BK;
  const int frag_swz = swz(l32);

  const int chunk = (total_tiles + kNumXcd - 1) / kNumXcd;
  const int padded_total = chunk * kNumXcd;

  for (int t = blockIdx.x; t < padded_total; t += gridDim.x) {
    // XCD-aware order: consecutive workgroup ids land on different XCDs; give each XCD a contiguous range.
    const int tile = (t % kNumXcd) * chunk + t / kNumXcd;
    if (tile >= total_tiles) continue;

    const int p = upper_slot(nprob, tile, [&](int i) { return probs[i].tile_begin; });
    const fp8gmm_gemm_problem pr = probs[p];
    const int local = tile - pr.tile_begin;
    const int tiles_m = (pr.m + BM - 1) / BM;
    const int tm = local % tiles_m;  // m fastest: neighbouring tiles share the weight slab
    const int tn = local / tiles_m;
    const int m0 = tm * BM;
    const int n0 = tn * BN;
    const int M = pr.m, N = pr.n, K = pr.k;
    const uint8_t* __restrict__ A = static_cast<const uint8_t*>(pr.a);
    const uint8_t* __restrict__ B = static_cast<const uint8_t*>(pr.b);
    const int64_t lda = pr.lda, ldb = pr.ldb;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int nk = (K + BK - 1) / BK;

    u32x4 ra[A_LOADS], rb[B_LOADS];
    const uint8_t* a_ptr[A_LOADS];
    const uint8_t* b_ptr[B_LOADS];
    bool a_ok[A_LOADS], b_ok[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = m0 + ld_r + 64 * i;
      a_ok[i] = row < M;
      a_ptr[i] = A + (int64_t)(a_ok[i] ? row : 0) * lda + ld_c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = n0 + ld_r + 64 * i;
      b_ok[i] = row < N;
      b_ptr[i] = B + (int64_t)(b_ok[i] ? row : 0) * ldb + ld_c * 16;
    }

    auto load_global = [&](int kt) {
      const int kbyte = kt * BK;
      const bool k_ok = kbyte + ld_c * 16 < K;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) {
        u32x4 v = {0u, 0u, 0u, 0u};
        if (a_ok[i] && k_ok) v = *reinterpret_cast<const u32x4*>(a_ptr[i] + kbyte);
        ra[i] = v;
      }
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i) {
        u32x4 v = {0u, 0u, 0u, 0u};
        if (b_ok[i] && k_ok) v = *reinterpret_cast<const u32x4*>(b_ptr[i] + kbyte);
        rb[i] = v;
      }
    };
    auto store_lds = [&](int stage) {
      uint8_t* sa = lds + stage * STAGE_BYTES;
      uint8_t* sb = sa + BM * BK;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) *reinterpret_cast<u32x4*>(sa + st_off + i * 64 * BK) = ra[i];
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i) *reinterpret_cast<u32x4*>(sb + st_off + i * 64 * BK) = rb[i];
    };
    auto compute = [&](int stage) {
      const uint8_t* sa = lds + stage * STAGE_BYTES + (wave_m * WM) * BK + frag_row_off;
      const uint8_t* sb = lds + stage * STAGE_BYTES + BM * BK + (wave_n * WN) * BK + frag_row_off;
#pragma unroll
      for (int ks = 0; ks < BK / 64; ++ks) {
        const int c0 = ((ks * 4 + khalf * 2) ^ frag_swz) << 4;
        const int c1 = ((ks * 4 + khalf * 2 + 1) ^ frag_swz) << 4;
        i32x8 fa[MT], fb[NT];
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const u32x4 lo = *reinterpret_cast<const u32x4*>(sa + i * 32 * BK + c0);
          const u32x4 hi = *reinterpret_cast<const u32x4*>(sa + i * 32 * BK + c1);
          fa[i] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const u32x4 lo = *reinterpret_cast<const u32x4*>(sb + j * 32 * BK + c0);
          const u32x4 hi = *reinterpret_cast<const u32x4*>(sb + j * 32 * BK + c1);
          fb[j] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
            // source 0 = weights (format B_FMT -> cbsz), source 1 = tokens (format A_FMT -> blgp)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], B_FMT, A_FMT, 0, 0,
                                                                         0, 0);
      }
    };

    if (nk > 0) {
      load_global(0);
      store_lds(0);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
      const bool more = kt + 1 < nk;
      if (more) load_global(kt + 1);
      compute(kt & 1);
      if (more) store_lds((kt + 1) & 1);
      __syncthreads();
    }

    // ---- epilogue ----
    const float sa_inv = pr.a_scale_inv ? *pr.a_scale_inv : 1.f;
    const float sb_inv = pr.b_scale_inv ? *pr.b_scale_inv : 1.f;
    const float s = sa_inv * sb_inv;
    const bool gelu = (epilogue & FP8GMM_EPI_GELU) != 0;
    const int64_t ldc = pr.ldc;
    float amax = 0.f;
    if (out_kind == FP8GMM_OUT_BF16) {
      uint16_t* __restrict__ C = static_cast<uint16_t*>(pr.c);
      uint16_t* __restrict__ AUX = static_cast<uint16_t*>(pr.aux);
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0) &&
                       (AUX == nullptr || (reinterpret_cast<uintptr_t>(AUX) & 7) == 0);
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int m = m0 + wave_m * WM + i * 32 + l32;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n0 + wave_n * WN + j * 32 + g * 8 + khalf * 4;
            if (m >= M || n >= N) continue;
            float v[4], r[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              v[q] = acc[i][j][g * 4 + q] * s;
              r[q] = gelu ? gelu_tanh(v[q]) : v[q];
            }
            const int64_t off = (int64_t)m * ldc + n;
            if (vec && n + 3 < N) {
              u32x2 o = {pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
              *reinterpret_cast<u32x2*>(C + off) = o;
              if (gelu && AUX != nullptr) {
                u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                *reinterpret_cast<u32x2*>(AUX + off) = a;
              }
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (n + q < N) {
                  C[off + q] = (uint16_t)f32_to_bf16_bits(r[q]);
                  if (gelu && AUX != nullptr) AUX[off + q] = (uint16_t)f32_to_bf16_bits(v[q]);
                }
              }
            }
          }
        }
      }
    } else {
      uint8_t* __restrict__ C = static_cast<uint8_t*>(pr.c);
      uint16_t* __restrict__ AUX = static_cast<uint16_t*>(pr.aux);
      const float cs = pr.c_scale ? *pr.c_scale : 1.f;
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 3) == 0) &&
                       (AUX == nullptr || (reinterpret_cast<uintptr_t>(AUX) & 7) == 0);
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int m = m0 + wave_m * WM + i * 32 + l32;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n0 + wave_n * WN + j * 32 + g * 8 + khalf * 4;
            if (m >= M || n >= N) continue;
            float v[4], r[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              v[q] = acc[i][j][g * 4 + q] * s;
              r[q] = gelu ? gelu_tanh(v[q]) : v[q];
              if (n + q < N) amax = amax_step(amax, r[q]);
            }
            uint32_t w;
            if (out_kind == FP8GMM_E4M3) {
              w = cvt4_fp8<FP8GMM_E4M3>(r[0] * cs, r[1] * cs, r[2] * cs, r[3] * cs);
            } else {
              w = cvt4_fp8<FP8GMM_E5M2>(r[0] * cs, r[1] * cs, r[2] * cs, r[3] * cs);
            }
            const int64_t off = (int64_t)m * ldc + n;
            if (vec && n + 3 < N) {
              *reinterpret_cast<uint32_t*>(C + off) = w;
              if (gelu && AUX != nullptr) {
                u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                *reinterpret_cast<u32x2*>(AUX + off) = a;
              }
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (n + q < N) {
                  C[off + q] = (uint8_t)(w >> (8 * q));
                  if (gelu && AUX != nullptr) AUX[off + q] = (uint16_t)f32_to_bf16_bits(v[q]);
                }
              }
            }
          }
        }
      }
      if (pr.c_amax != nullptr) {
        amax = wave_max(amax);
        if (lane == 0 && amax > 0.f) atomic_max_nonneg(pr.c_amax, amax);
      }
    }
    // all LDS reads of this tile are complete: the last main-loop barrier ordered them.
  }
}

template <int A_FMT, int B_FMT>
int launch(const fp8gmm_gemm_problem* probs_dev, int n, int total_tiles, int out_kind, int epilogue,
           hipStream_t stream) {
  static int num_cu = 0;
  static bool attr_set = false;
  const size_t lds_bytes = 2 * STAGE_BYTES;
  auto kernel = grouped_gemm_kernel<A_FMT, B_FMT>;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess)
      return FP8GMM_ERR_LAUNCH;
    attr_set = true;
  }
  if (num_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
      return FP8GMM_ERR_NO_DEVICE;
    num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  const int chunk = (total_tiles + kNumXcd - 1) / kNumXcd;
  int grid = chunk * kNumXcd;
  if (grid > num_cu) grid = num_cu;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NTHREADS), lds_bytes, stream, probs_dev, n, total_tiles, out_kind,
                     epilogue);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

}  // namespace
}  // namespace fp8gmm

extern "C" {

void fp8gmm_gemm_tile_shape(int* tile_m, int* tile_n) {
  if (tile_m) *tile_m = fp8gmm::BM;
  if (tile_n) *tile_n = fp8gmm::BN;
}

int fp8gmm_plan_grouped_gemm(fp8gmm_gemm_problem* probs, int n, int* total_tiles) {
  if (n < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (total_tiles == nullptr || (n > 0 && probs == nullptr)) return FP8GMM_ERR_NULL_POINTER;
  int64_t tiles = 0;
  for (int i = 0; i < n; ++i) {
    fp8gmm_gemm_problem& p = probs[i];
    if (p.m < 0 || p.n < 0 || p.k < 0) return FP8GMM_ERR_BAD_SHAPE;
    if (p.lda < p.k || p.ldb < p.k || p.ldc < p.n) return FP8GMM_ERR_BAD_SHAPE;
    const bool has_work = p.m > 0 && p.n > 0;
    if (has_work) {
      if (p.c == nullptr) return FP8GMM_ERR_NULL_POINTER;
      if (p.k > 0) {  // with k == 0 the operands are never read
        if (p.a == nullptr || p.b == nullptr) return FP8GMM_ERR_NULL_POINTER;
        if ((p.k & 15) || (p.lda & 15) || (p.ldb & 15)) return FP8GMM_ERR_ALIGNMENT;
        if ((reinterpret_cast<uintptr_t>(p.a) & 15) || (reinterpret_cast<uintptr_t>(p.b) & 15))
          return FP8GMM_ERR_ALIGNMENT;
      }
    }
    const int64_t tm = (p.m + fp8gmm::BM - 1) / fp8gmm::BM;
    const int64_t tn = (p.n + fp8gmm::BN - 1) / fp8gmm::BN;
    p.tile_begin = (int32_t)tiles;
    p.tiles_n = (int32_t)tn;
    tiles += tm * tn;
    if (tiles > INT32_MAX / 16) return FP8GMM_ERR_BAD_SHAPE;
  }
  *total_tiles = (int)tiles;
  return FP8GMM_OK;
}

int fp8gmm_grouped_gemm(const fp8gmm_gemm_problem* probs_dev, int n, int total_tiles, int a_fmt, int b_fmt,
                        int out_kind, int epilogue, void* stream) {
  if (n < 0 || total_tiles < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (out_kind != FP8GMM_OUT_BF16 && out_kind != FP8GMM_E4M3 && out_kind != FP8GMM_E5M2) return FP8GMM_ERR_BAD_FORMAT;
  if (epilogue & ~FP8GMM_EPI_GELU) return FP8GMM_ERR_BAD_ARGUMENT;
  if ((a_fmt != FP8GMM_E4M3 && a_fmt != FP8GMM_E5M2) || (b_fmt != FP8GMM_E4M3 && b_fmt != FP8GMM_E5M2))
    return FP8GMM_ERR_BAD_FORMAT;
  if (a_fmt == FP8GMM_E5M2 && b_fmt == FP8GMM_E5M2) return FP8GMM_ERR_BAD_FORMAT;
  if (n == 0 || total_tiles == 0) return FP8GMM_OK;
  if (probs_dev == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a_fmt == FP8GMM_E4M3 && b_fmt == FP8GMM_E4M3)
    return fp8gmm::launch<FP8GMM_E4M3, FP8GMM_E4M3>(probs_dev, n, total_tiles, out_kind, epilogue, s);
  if (a_fmt == FP8GMM_E5M2 && b_fmt == FP8GMM_E4M3)
    return fp8gmm::launch<FP8GMM_E5M2, FP8GMM_E4M3>(probs_dev, n, total_tiles, out_kind, epilogue, s);
  return fp8gmm::launch<FP8GMM_E4M3, FP8GMM_E5M2>(probs_dev, n, total_tiles, out_kind, epilogue, s);
}

}  // extern "C"
