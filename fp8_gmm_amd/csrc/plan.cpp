// Host-side planning for the multi-tensor kernels and library info. No GPU needed.
//
// Replaces the host halves of the reference's multi-tensor entry points, which validate
// the tensor lists and build a prefix sum of workgroups per tensor
// (csrc/multi_pointwise.cu:155-189,216-246; csrc/multi_pad_fusion.cu:442-488,505-559,587-644).
// Unlike the reference there is no aligned / unaligned split into two launches: the
// kernels pick the vector or the scalar path per tensor at run time.
#include <stdint.h>

#include "../../include/fp8gmm.h"
#include "gemm_schedule.h"
#include "tiling.h"

extern "C" {

int fp8gmm_version(void) { return FP8GMM_VERSION; }

const char* fp8gmm_status_string(int status) {
  switch (status) {
    case FP8GMM_OK: return "ok";
    case FP8GMM_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FP8GMM_ERR_BAD_SHAPE: return "bad shape (negative size, rows_padded < rows, pitch < extent or overflow)";
    case FP8GMM_ERR_BAD_FORMAT: return "unknown or unsupported fp8 format";
    case FP8GMM_ERR_ALIGNMENT: return "GEMM operand not 16-byte aligned or K / pitch not a multiple of 16";
    case FP8GMM_ERR_LAUNCH: return "HIP kernel launch failed";
    case FP8GMM_ERR_BAD_ARGUMENT: return "inconsistent scalar argument";
    case FP8GMM_ERR_NO_DEVICE: return "no usable HIP device";
    default: return "unknown fp8gmm status";
  }
}

size_t fp8gmm_sizeof_tensor_desc(void) { return sizeof(fp8gmm_tensor_desc); }
size_t fp8gmm_sizeof_gemm_problem(void) { return sizeof(fp8gmm_gemm_problem); }

int fp8gmm_plan_multi_tensor(fp8gmm_tensor_desc* descs, int n, int op, int* total_blocks) {
  if (n < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (op < FP8GMM_OP_QUANTIZE || op > FP8GMM_OP_CAST_DGELU) return FP8GMM_ERR_BAD_ARGUMENT;
  if (total_blocks == nullptr || (n > 0 && descs == nullptr)) return FP8GMM_ERR_NULL_POINTER;
  int64_t blocks = 0;
  for (int i = 0; i < n; ++i) {
    fp8gmm_tensor_desc& d = descs[i];
    if (d.rows < 0 || d.cols < 0) return FP8GMM_ERR_BAD_SHAPE;
    const int64_t numel = (int64_t)d.rows * d.cols;
    int64_t nb = 0;
    if (op == FP8GMM_OP_QUANTIZE || op == FP8GMM_OP_SCALE_MUL || op == FP8GMM_OP_CAST_DGELU) {
      if (numel > 0) {
        if (d.in == nullptr) return FP8GMM_ERR_NULL_POINTER;
        if (op != FP8GMM_OP_SCALE_MUL && d.out == nullptr) return FP8GMM_ERR_NULL_POINTER;
        if (op == FP8GMM_OP_CAST_DGELU && d.in2 == nullptr) return FP8GMM_ERR_NULL_POINTER;
      }
      nb = (numel + fp8gmm::kPwBlockElems - 1) / fp8gmm::kPwBlockElems;
    } else {
      if (d.rows_padded < d.rows) return FP8GMM_ERR_BAD_SHAPE;
      // the transposed output is [cols, rows_padded]: pad columns exist even when rows == 0
      const int64_t t_numel = (int64_t)d.cols * d.rows_padded;
      if (t_numel > 0 && d.out_t == nullptr) return FP8GMM_ERR_NULL_POINTER;
      if (numel > 0) {
        if (d.in == nullptr) return FP8GMM_ERR_NULL_POINTER;
        if (op == FP8GMM_OP_PAD_CAST_TRANSPOSE_DGELU && d.in2 == nullptr) return FP8GMM_ERR_NULL_POINTER;
      }
      const int64_t tr = ((int64_t)d.rows_padded + fp8gmm::kPtTileRows - 1) / fp8gmm::kPtTileRows;
      const int64_t tc = ((int64_t)d.cols + fp8gmm::kPtTileCols - 1) / fp8gmm::kPtTileCols;
      nb = tr * tc;
    }
    d.block_begin = (int32_t)blocks;
    d.amax_partial = 0;
    blocks += nb;
    if (blocks > INT32_MAX / 2) return FP8GMM_ERR_BAD_SHAPE;
  }
  *total_blocks = (int)blocks;
  return FP8GMM_OK;
}

int fp8gmm_gemm_schedule(const fp8gmm_gemm_problem* probs, int n, int total_tiles, int grid, int stream_k, int wg,
                         int32_t* items, int max_items) {
  using namespace fp8gmm;
  if (n < 0 || total_tiles < 0 || grid <= 0 || (grid % kNumXcd) != 0 || wg < 0 || wg >= grid || max_items < 0)
    return FP8GMM_ERR_BAD_ARGUMENT;
  if ((n > 0 && probs == nullptr) || (max_items > 0 && items == nullptr)) return FP8GMM_ERR_NULL_POINTER;
  if (n == 0 || total_tiles == 0) return 0;
  const int xcd = wg % kNumXcd, j = wg / kNumXcd;
  Sched s;
  sched_init(s, probs, n, total_tiles, xcd, grid / kNumXcd, stream_k != 0);
  Cursor c;
  cursor_init(s, j, c);
  int count = 0;
  for (; cursor_valid(s, j, c); cursor_advance(s, j, c)) {
    const Item it = cursor_item(s, xcd, j, c);
    if (count < max_items) {
      int32_t* r = items + 7 * count;
      r[0] = it.tile; r[1] = it.prob; r[2] = it.m0; r[3] = it.n0; r[4] = it.k_begin; r[5] = it.nk; r[6] = it.slot;
    }
    ++count;
  }
  return count;
}

int fp8gmm_gemm_fixup(const fp8gmm_gemm_problem* probs, int n, int total_tiles, int grid, int wg, int32_t* tile,
                      int32_t* slots, int max_slots) {
  using namespace fp8gmm;
  if (n < 0 || total_tiles < 0 || grid <= kNumXcd || (grid % kNumXcd) != 0 || wg < 0 || wg >= grid - kNumXcd ||
      max_slots < 0)
    return FP8GMM_ERR_BAD_ARGUMENT;
  if (tile == nullptr || (n > 0 && probs == nullptr) || (max_slots > 0 && slots == nullptr))
    return FP8GMM_ERR_NULL_POINTER;
  *tile = -1;
  if (n == 0 || total_tiles == 0) return 0;
  const int xcd = wg % kNumXcd, j = wg / kNumXcd + 1, wgs = grid / kNumXcd;
  Sched s;
  sched_init(s, probs, n, total_tiles, xcd, wgs, true);
  int n_following = 0;
  const int t = fixup_tile(s, j, &n_following);
  if (t < 0) return 0;
  *tile = t;
  int count = 0;
  auto put = [&](int slot) {
    if (count < max_slots) slots[count] = slot;
    ++count;
  };
  put(kSlotsPerWg * (xcd * wgs + j - 1) + 1);
  for (int q = j; q < j + n_following; ++q) put(kSlotsPerWg * (xcd * wgs + q));
  return count;
}

}  // extern "C"
