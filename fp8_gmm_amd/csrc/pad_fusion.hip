// Multi-tensor pad + (cast) + transpose kernels for gfx950.
//
// Replaces csrc/multi_pad_fusion.cu of the reference:
//   multi_pad_transpose_kernel            (:46-153)   fp8 [m, n]  -> fp8 [n, Mpad]
//   multi_pad_cast_transpose_kernel       (:155-292)  bf16 [m, n] -> fp8 [m, n] + fp8 [n, Mpad] + amax
//   multi_pad_cast_transpose_dgelu_kernel (:294-438)  same with x = dy * dgelu(pre)
// The transposed copy is zero-padded along the token dimension (columns m..Mpad-1 hold
// fp8(scale * 0)); the row-major copy is never padded.
//
// One launch covers every tensor of the call.  A workgroup (4 wavefronts) owns a
// 128 x 128 tile:
//   * lane (rg, cg) loads 8 rows x 8 columns with one 128-bit load per row (16 lanes
//     cover 256 contiguous bytes of a row), converts, stores the row-major fp8 copy
//     with 64-bit stores (128 contiguous bytes per row per 16 lanes);
//   * the 8 x 8 byte block is transposed in registers with v_perm_b32 and written
//     to a 128 x 128-byte LDS tile (column-major, 8-byte granules XOR-swizzled by the
//     column group so that the 64 lanes of a store hit distinct banks);
//   * the tile is read back 16 bytes at a time and stored to the transposed output
//     with 128-bit stores: 8 lanes cover 128 contiguous bytes of one output row;
//   * amax: per-lane running max -> wave shuffle reduction -> one integer atomic max
//     per workgroup.
// HBM-bound: per element 2 B (bf16) or 1 B (fp8) read, 1 B + Mpad/m B written.
#include "device_utils.h"
#include "tiling.h"

namespace fp8gmm {
namespace {

constexpr int OP_TRANSPOSE = 0;
constexpr int OP_CAST = 1;
constexpr int OP_CAST_DGELU = 2;

constexpr int TM = kPtTileRows;  // 128
constexpr int TN = kPtTileCols;  // 128
constexpr int RPT = 8;           // rows per lane
constexpr int CPT = 8;           // columns per lane
static_assert((TM / RPT) * (TN / CPT) == kPtThreads, "tile / lane mapping");

// 4 x 4 byte transpose: a, b, c, d are rows (byte q = column q); outputs are columns (byte r = row r).
__device__ __forceinline__ void transpose4x4(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t& o0,
                                             uint32_t& o1, uint32_t& o2, uint32_t& o3) {
  // __builtin_amdgcn_perm(hi, lo, sel): selector bytes 0-3 pick from lo, 4-7 from hi
  const uint32_t t0 = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
  const uint32_t t1 = __builtin_amdgcn_perm(b, a, 0x07030602u);  // a2 b2 a3 b3
  const uint32_t t2 = __builtin_amdgcn_perm(d, c, 0x05010400u);  // c0 d0 c1 d1
  const uint32_t t3 = __builtin_amdgcn_perm(d, c, 0x07030602u);  // c2 d2 c3 d3
  o0 = __builtin_amdgcn_perm(t2, t0, 0x05040100u);               // a0 b0 c0 d0
  o1 = __builtin_amdgcn_perm(t2, t0, 0x07060302u);               // a1 b1 c1 d1
  o2 = __builtin_amdgcn_perm(t3, t1, 0x05040100u);               // a2 b2 c2 d2
  o3 = __builtin_amdgcn_perm(t3, t1, 0x07060302u);               // a3 b3 c3 d3
}

template <int OP, int FMT>
__global__ __launch_bounds__(kPtThreads) void multi_pad_kernel(fp8gmm_tensor_desc* __restrict__ descs, int n) {
  __shared__ __attribute__((aligned(16))) uint8_t tl[TN * TM];
  __shared__ float stage[kPtThreads / kWaveSize];

  const int bid = blockIdx.x;
  const int t = upper_slot(n, bid, [&](int i) { return descs[i].block_begin; });
  const fp8gmm_tensor_desc d = descs[t];
  const int m = d.rows;
  const int ncols = d.cols;
  const int mpad = d.rows_padded;
  const int tiles_c = (ncols + TN - 1) / TN;
  const int tile = bid - d.block_begin;
  const int r0 = (tile / tiles_c) * TM;
  const int c0 = (tile % tiles_c) * TN;

  const int tid = threadIdx.x;
  const int cg = tid & 15;  // column group: columns c0 + 8 cg .. + 7
  const int rg = tid >> 4;  // row group:    rows    r0 + 8 rg .. + 7
  const int col = c0 + CPT * cg;

  const uint8_t* __restrict__ in8 = static_cast<const uint8_t*>(d.in);
  const uint16_t* __restrict__ in16 = static_cast<const uint16_t*>(d.in);
  const uint16_t* __restrict__ pre16 = static_cast<const uint16_t*>(d.in2);
  uint8_t* __restrict__ out = static_cast<uint8_t*>(d.out);
  uint8_t* __restrict__ out_t = static_cast<uint8_t*>(d.out_t);
  float scale = 1.f;
  if constexpr (OP != OP_TRANSPOSE) scale = d.scale ? *d.scale : 1.f;

  // whole-tensor vector eligibility (uniform per workgroup)
  bool vec_in = (ncols % CPT) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0;
  if constexpr (OP == OP_TRANSPOSE) {
    vec_in = vec_in && (reinterpret_cast<uintptr_t>(in8) & 7) == 0;
  } else {
    vec_in = vec_in && (reinterpret_cast<uintptr_t>(in16) & 15) == 0;
    if constexpr (OP == OP_CAST_DGELU) vec_in = vec_in && (reinterpret_cast<uintptr_t>(pre16) & 15) == 0;
  }
  const bool vec_t = (mpad % 16) == 0 && (reinterpret_cast<uintptr_t>(out_t) & 15) == 0;

  // Descriptor path: every offset of the tensor fits 32 bits, so rows past m and columns past ncols become
  // out-of-range buffer offsets (loads return zero = the padding value, stores are dropped) and all loads
  // of the lane are issued back to back without a branch.
  constexpr int kInBytes = OP == OP_TRANSPOSE ? 1 : 2;
  const bool fast = vec_in && vec_t && (int64_t)m * ncols * kInBytes < (int64_t)0xffffffff &&
                    (int64_t)ncols * mpad < (int64_t)0xffffffff;

  float mx = 0.f;
  uint32_t y[RPT][2];  // fp8 bytes of 8 rows x 8 columns; y[i][h] byte q = column 4 h + q of row i

  if (fast) {
    const uint32_t in_bytes = (uint32_t)((int64_t)m * ncols * kInBytes);
    const __amdgpu_buffer_rsrc_t rin = make_rsrc(d.in, in_bytes);
    uint32_t eoff[RPT];  // element offset of the lane's 8 columns in row i, or out of range
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int row = r0 + RPT * rg + i;
      eoff[i] = (row < m && col < ncols) ? (uint32_t)row * (uint32_t)ncols + (uint32_t)col : kOobOffset;
    }
    if constexpr (OP == OP_TRANSPOSE) {
      u32x2 v[RPT];
#pragma unroll
      for (int i = 0; i < RPT; ++i) v[i] = buf_load8_stream(rin, eoff[i]);
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        y[i][0] = v[i].x;
        y[i][1] = v[i].y;
      }
    } else {
      u32x4 xa[RPT];
      u32x4 ga[OP == OP_CAST_DGELU ? RPT : 1];
#pragma unroll
      for (int i = 0; i < RPT; ++i) xa[i] = buf_load16_stream(rin, eoff[i] == kOobOffset ? kOobOffset : eoff[i] * 2);
      if constexpr (OP == OP_CAST_DGELU) {
        const __amdgpu_buffer_rsrc_t rpre = make_rsrc(d.in2, in_bytes);
#pragma unroll
        for (int i = 0; i < RPT; ++i) ga[i] = buf_load16_stream(rpre, eoff[i] == kOobOffset ? kOobOffset : eoff[i] * 2);
      }
      const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, out != nullptr ? in_bytes / 2 : 0u);
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        const uint32_t w[4] = {xa[i].x, xa[i].y, xa[i].z, xa[i].w};
        float x[CPT];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          x[2 * q] = bf16_lo_to_f32(w[q]);
          x[2 * q + 1] = bf16_hi_to_f32(w[q]);
        }
        if constexpr (OP == OP_CAST_DGELU) {
          const uint32_t g[4] = {ga[i].x, ga[i].y, ga[i].z, ga[i].w};
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            x[2 * q] *= dgelu(bf16_lo_to_f32(g[q]));
            x[2 * q + 1] *= dgelu(bf16_hi_to_f32(g[q]));
          }
        }
#pragma unroll
        for (int e = 0; e < CPT; ++e) mx = amax_step(mx, x[e]);
        y[i][0] = cvt4_fp8<FMT>(scale * x[0], scale * x[1], scale * x[2], scale * x[3]);
        y[i][1] = cvt4_fp8<FMT>(scale * x[4], scale * x[5], scale * x[6], scale * x[7]);
        buf_store8(u32x2{y[i][0], y[i][1]}, rout, eoff[i]);
      }
    }
  } else {
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int row = r0 + RPT * rg + i;
    const bool row_ok = row < m;
    const int64_t off = (int64_t)row * ncols + col;
    if constexpr (OP == OP_TRANSPOSE) {
      u32x2 v = {0u, 0u};
      if (row_ok) {
#pragma unroll
        for (int e = 0; e < CPT; ++e)
          if (col + e < ncols) v[e >> 2] |= (uint32_t)in8[off + e] << (8 * (e & 3));
      }
      y[i][0] = v.x;
      y[i][1] = v.y;
    } else {
      float x[CPT];
#pragma unroll
      for (int e = 0; e < CPT; ++e) x[e] = 0.f;
      if (row_ok) {
#pragma unroll
        for (int e = 0; e < CPT; ++e) {
          if (col + e < ncols) {
            x[e] = bf16_to_f32(in16[off + e]);
            if constexpr (OP == OP_CAST_DGELU) x[e] *= dgelu(bf16_to_f32(pre16[off + e]));
          }
        }
      }
#pragma unroll
      for (int e = 0; e < CPT; ++e) mx = amax_step(mx, x[e]);
      y[i][0] = cvt4_fp8<FMT>(scale * x[0], scale * x[1], scale * x[2], scale * x[3]);
      y[i][1] = cvt4_fp8<FMT>(scale * x[4], scale * x[5], scale * x[6], scale * x[7]);
      if (out != nullptr && row_ok) {
#pragma unroll
        for (int e = 0; e < CPT; ++e)
          if (col + e < ncols) out[off + e] = (uint8_t)(y[i][e >> 2] >> (8 * (e & 3)));
      }
    }
  }
  }

  // ---- 8 x 8 byte transpose in registers, then to the LDS tile ----
  // tl is column-major: row j of tl holds column c0 + j of the tile, 128 bytes = 16 granules of
  // 8 token rows; granule g of column j sits at slot g ^ ((j >> 3) & 15).
  uint32_t tc[CPT][2];  // tc[c][b]: column c of the lane, token rows 4 b .. 4 b + 3
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int b = 0; b < 2; ++b)
      transpose4x4(y[4 * b + 0][h], y[4 * b + 1][h], y[4 * b + 2][h], y[4 * b + 3][h], tc[4 * h + 0][b],
                   tc[4 * h + 1][b], tc[4 * h + 2][b], tc[4 * h + 3][b]);
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int j = CPT * cg + c;
    const int slot = rg ^ cg;  // (j >> 3) & 15 == cg
    const u32x2 v = {tc[c][0], tc[c][1]};
    *reinterpret_cast<u32x2*>(&tl[j * TM + slot * 8]) = v;
  }
  __syncthreads();

  // ---- LDS tile -> transposed output: 16 token rows of one column per lane and step ----
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(out_t, fast ? (uint32_t)((int64_t)ncols * mpad) : 0u);
#pragma unroll
  for (int q = 0; q < (TN * TM / 16) / kPtThreads; ++q) {
    const int p = tid + kPtThreads * q;
    const int j = p >> 3;       // column of the tile
    const int piece = p & 7;    // token rows 16 piece .. 16 piece + 15
    const int f = (j >> 3) & 15;
    const int slot16 = ((2 * piece) ^ f) >> 1;  // granules 2 piece, 2 piece + 1 share one 16-byte slot
    u32x4 v = *reinterpret_cast<const u32x4*>(&tl[j * TM + slot16 * 16]);
    if (f & 1) v = u32x4{v.z, v.w, v.x, v.y};   // odd swizzle: the two granules are swapped inside the slot
    const int gcol = c0 + j;
    const int grow = r0 + 16 * piece;
    const bool ok = gcol < ncols && grow < mpad;
    if (fast) {
      buf_store16(v, rt, ok ? (uint32_t)gcol * (uint32_t)mpad + (uint32_t)grow : kOobOffset);
    } else if (ok) {
      uint8_t* dst = out_t + (int64_t)gcol * mpad + grow;
      if (vec_t) {
        global_store(dst, v);
      } else {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 16; ++e)
          if (grow + e < mpad) dst[e] = (uint8_t)(w[e >> 2] >> (8 * (e & 3)));
      }
    }
  }

  if constexpr (OP != OP_TRANSPOSE)
    block_amax_merge<kPtThreads / kWaveSize>(mx, d.amax != nullptr ? &descs[t].amax_partial : nullptr, stage);
}

template <int OP>
int launch_fmt(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, hipStream_t s) {
  if (out_fmt == FP8GMM_E4M3)
    hipLaunchKernelGGL((multi_pad_kernel<OP, FP8GMM_E4M3>), dim3(total_blocks), dim3(kPtThreads), 0, s, descs_dev, n);
  else
    hipLaunchKernelGGL((multi_pad_kernel<OP, FP8GMM_E5M2>), dim3(total_blocks), dim3(kPtThreads), 0, s, descs_dev, n);
  if (OP != OP_TRANSPOSE) hipLaunchKernelGGL(amax_merge_kernel, dim3((n + 255) / 256), dim3(256), 0, s, descs_dev, n);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int check_args(const fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, bool* nothing) {
  *nothing = false;
  if (n < 0 || total_blocks < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (out_fmt != FP8GMM_E4M3 && out_fmt != FP8GMM_E5M2) return FP8GMM_ERR_BAD_FORMAT;
  if (n == 0 || total_blocks == 0) {
    *nothing = true;
    return FP8GMM_OK;
  }
  if (descs_dev == nullptr) return FP8GMM_ERR_NULL_POINTER;
  return FP8GMM_OK;
}

}  // namespace
}  // namespace fp8gmm

extern "C" {

int fp8gmm_multi_pad_transpose(const fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, void* stream) {
  bool nothing;
  const int rc = fp8gmm::check_args(descs_dev, n, total_blocks, FP8GMM_E4M3, &nothing);
  if (rc != FP8GMM_OK || nothing) return rc;
  // a pure byte shuffle: the fp8 flavour does not matter
  return fp8gmm::launch_fmt<fp8gmm::OP_TRANSPOSE>(const_cast<fp8gmm_tensor_desc*>(descs_dev), n, total_blocks,
                                                  FP8GMM_E4M3, static_cast<hipStream_t>(stream));
}

int fp8gmm_multi_pad_cast_transpose(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt,
                                    void* stream) {
  bool nothing;
  const int rc = fp8gmm::check_args(descs_dev, n, total_blocks, out_fmt, &nothing);
  if (rc != FP8GMM_OK || nothing) return rc;
  return fp8gmm::launch_fmt<fp8gmm::OP_CAST>(descs_dev, n, total_blocks, out_fmt, static_cast<hipStream_t>(stream));
}

int fp8gmm_multi_pad_cast_transpose_dgelu(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt,
                                          void* stream) {
  bool nothing;
  const int rc = fp8gmm::check_args(descs_dev, n, total_blocks, out_fmt, &nothing);
  if (rc != FP8GMM_OK || nothing) return rc;
  return fp8gmm::launch_fmt<fp8gmm::OP_CAST_DGELU>(descs_dev, n, total_blocks, out_fmt,
                                                   static_cast<hipStream_t>(stream));
}

}  // extern "C"
