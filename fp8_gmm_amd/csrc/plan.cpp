// Host-side planning for the multi-tensor kernels and library info. No GPU needed.
//
// Replaces the host halves of the reference's multi-tensor entry points, which validate
// the tensor lists and build a prefix sum of workgroups per tensor
// (csrc/multi_pointwise.cu:155-189,216-246; csrc/multi_pad_fusion.cu:442-488,505-559,587-644).
// Unlike the reference there is no aligned / unaligned split into two launches: the
// kernels pick the vector or the scalar path per tensor at run time.
#include <stdint.h>

#include <algorithm>
#include <vector>

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
    case FP8GMM_ERR_BUFFER_TOO_SMALL: return "output array of a planning call too small (required sizes returned)";
    case FP8GMM_ERR_WORKSPACE: return "the launch needs more workspace than it was given";
    default: return "unknown fp8gmm status";
  }
}

size_t fp8gmm_sizeof_tensor_desc(void) { return sizeof(fp8gmm_tensor_desc); }
size_t fp8gmm_sizeof_gemm_problem(void) { return sizeof(fp8gmm_gemm_problem); }
size_t fp8gmm_sizeof_gemm_item(void) { return sizeof(fp8gmm_gemm_item); }

int fp8gmm_gemm_grid(int num_cu) {
  int grid = (num_cu / fp8gmm::kNumXcd) * fp8gmm::kNumXcd;
  return grid < fp8gmm::kNumXcd ? fp8gmm::kNumXcd : grid;
}

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

int fp8gmm_plan_grouped_gemm(fp8gmm_gemm_problem* probs, int n, int* total_tiles) {
  return fp8gmm_plan_grouped_gemm_layout(probs, n, 0, total_tiles);
}

int fp8gmm_plan_grouped_gemm_layout(fp8gmm_gemm_problem* probs, int n, int layout, int* total_tiles) {
  if (n < 0 || (layout & ~(FP8GMM_GEMM_A_KMAJOR | FP8GMM_GEMM_B_KMAJOR))) return FP8GMM_ERR_BAD_ARGUMENT;
  const bool a_kmajor = (layout & FP8GMM_GEMM_A_KMAJOR) != 0;
  const bool b_kmajor = (layout & FP8GMM_GEMM_B_KMAJOR) != 0;
  if (a_kmajor && !b_kmajor) return FP8GMM_ERR_BAD_ARGUMENT;  // not a combination the path uses
  if (total_tiles == nullptr || (n > 0 && probs == nullptr)) return FP8GMM_ERR_NULL_POINTER;
  int64_t tiles = 0, cost = 0;
  for (int i = 0; i < n; ++i) {
    fp8gmm_gemm_problem& p = probs[i];
    if (p.m < 0 || p.n < 0 || p.k < 0) return FP8GMM_ERR_BAD_SHAPE;
    if (p.lda < (a_kmajor ? p.m : p.k) || p.ldb < (b_kmajor ? p.n : p.k) || p.ldc < p.n) return FP8GMM_ERR_BAD_SHAPE;
    const bool has_work = p.m > 0 && p.n > 0;
    if (has_work) {
      if (p.c == nullptr) return FP8GMM_ERR_NULL_POINTER;
      if (p.k > 0) {  // with k == 0 the operands are never read
        if (p.a == nullptr || p.b == nullptr) return FP8GMM_ERR_NULL_POINTER;
        // a row-major operand is fetched in 16-byte pieces along k, a contraction-major one along its rows
        // (with b alone contraction-major any k will do: the rows of b past k read as zeros, and the 16-byte piece
        // of a that straddles k lies inside a's row pitch)
        if ((!b_kmajor && (p.k & 15)) || (p.lda & 15) || (p.ldb & 15)) return FP8GMM_ERR_ALIGNMENT;
        if ((a_kmajor && (p.m & 15)) || (b_kmajor && (p.n & 15))) return FP8GMM_ERR_ALIGNMENT;
        if ((reinterpret_cast<uintptr_t>(p.a) & 15) || (reinterpret_cast<uintptr_t>(p.b) & 15))
          return FP8GMM_ERR_ALIGNMENT;
        // the kernel addresses the rows of one tile (row-major operand) or the whole operand (contraction-major)
        // through a buffer descriptor with 32-bit byte offsets; contraction rows up to 127 past k are addressed,
        // and must fall outside the descriptor, not wrap
        if ((uint64_t)(a_kmajor ? p.k + 128 : fp8gmm::BM) * (uint64_t)p.lda > 0xffffffffull ||
            (uint64_t)(b_kmajor ? p.k + 128 : fp8gmm::BN) * (uint64_t)p.ldb > 0xffffffffull)
          return FP8GMM_ERR_BAD_SHAPE;
      }
    }
    const int64_t tm = (p.m + fp8gmm::BM - 1) / fp8gmm::BM;
    const int64_t tn = (p.n + fp8gmm::BN - 1) / fp8gmm::BN;
    p.tile_begin = (int32_t)tiles;
    p.cost_begin = (int32_t)cost;  // a tile costs ceil(k / 128) steps of the main loop (1 for k = 0)
    const int64_t steps = (p.k + 127) / 128;
    tiles += tm * tn;
    cost += tm * tn * (steps > 0 ? steps : 1);
    if (tiles > INT32_MAX / 16 || cost > INT32_MAX / 2) return FP8GMM_ERR_BAD_SHAPE;
  }
  *total_tiles = (int)tiles;
  return FP8GMM_OK;
}

// The work list of a launch: the schedule of gemm_schedule.h written out, one record per (workgroup, item), in
// the order items[r * grid + workgroup]; the slots in use are renumbered from 0 in the order the workgroups
// are walked, and the fix-up records name them by their new numbers.
// The same launch cut into 128 x 128 tiles (FP8GMM_GEMM_TILE_128) or into 128 x 256 tiles for the kernel with two
// sets of accumulators (FP8GMM_GEMM_TILE_DUAL): whole tiles only, the tile list in 8 contiguous ranges of equal
// work, the workgroups of an XCD striding through their range.
// kOverhead: what a tile costs besides its steps, in K = 128 steps: epilogue and switch of a small tile on a
// workgroup that shares its compute unit; with two sets of accumulators, the slower steps that carry the result.
static int plan_whole_tiles(const int TM, const int TN, const int kOverhead, fp8gmm_gemm_problem* probs, int n, int layout,
                            int grid, fp8gmm_gemm_item* items, int max_items, fp8gmm_gemm_plan* plan) {
  using namespace fp8gmm;
  int unused = 0;
  const int rc = fp8gmm_plan_grouped_gemm_layout(probs, n, layout, &unused);
  if (rc != FP8GMM_OK) return rc;
  const bool a_kmajor = (layout & FP8GMM_GEMM_A_KMAJOR) != 0, b_kmajor = (layout & FP8GMM_GEMM_B_KMAJOR) != 0;
  // tiles and work per problem
  std::vector<int64_t> tile_begin((size_t)n + 1, 0), work_begin((size_t)n + 1, 0);
  for (int p = 0; p < n; ++p) {
    const int64_t tiles = (int64_t)((probs[p].m + TM - 1) / TM) * ((probs[p].n + TN - 1) / TN);
    const int64_t steps = (probs[p].k + 127) / 128;
    tile_begin[p + 1] = tile_begin[p] + tiles;
    work_begin[p + 1] = work_begin[p] + tiles * ((steps > 0 ? steps : 1) + kOverhead);
    if (tile_begin[p + 1] > INT32_MAX / 16) return FP8GMM_ERR_BAD_SHAPE;
  }
  const int total_tiles = (int)tile_begin[n];
  plan->total_tiles = total_tiles;
  plan->tile = TN;
  plan->tile_m = TM == TN ? 0 : TM;
  if (total_tiles == 0) return FP8GMM_OK;
  {
    const int needed = ((total_tiles + kNumXcd - 1) / kNumXcd) * kNumXcd;
    if (grid > needed) grid = needed;
  }
  const int wgs = grid / kNumXcd;
  // XCD x takes the tiles [cut[x], cut[x + 1]): the first tile at or past x / 8 of the work
  int cut[kNumXcd + 1];
  cut[0] = 0;
  cut[kNumXcd] = total_tiles;
  {
    int p = 0;
    for (int x = 1; x < kNumXcd; ++x) {
      const int64_t target = (work_begin[n] * x + kNumXcd - 1) / kNumXcd;
      while (p < n && work_begin[p + 1] <= target) ++p;
      if (p >= n) {
        cut[x] = total_tiles;
        continue;
      }
      const int64_t per_tile = (work_begin[p + 1] - work_begin[p]) / (tile_begin[p + 1] - tile_begin[p]);
      cut[x] = (int)(tile_begin[p] + (target - work_begin[p] + per_tile - 1) / per_tile);
    }
  }
  int rounds = 0;
  for (int x = 0; x < kNumXcd; ++x) rounds = std::max(rounds, (cut[x + 1] - cut[x] + wgs - 1) / wgs);
  rounds += 1;  // every list ends with a record whose prob is -1
  plan->grid = grid;
  plan->rounds = rounds;
  if ((int64_t)rounds * grid > INT32_MAX / 64) return FP8GMM_ERR_BAD_SHAPE;
  if ((int64_t)rounds * grid > max_items) return FP8GMM_ERR_BUFFER_TOO_SMALL;
  if (items == nullptr) return FP8GMM_ERR_NULL_POINTER;
  fp8gmm_gemm_item end_record{};
  end_record.prob = -1;
  end_record.slot = -1;
  for (int i = 0; i < rounds * grid; ++i) items[i] = end_record;
  for (int x = 0; x < kNumXcd; ++x) {
    int p = 0;
    for (int t = cut[x]; t < cut[x + 1]; ++t) {
      while (tile_begin[p + 1] <= t) ++p;
      const fp8gmm_gemm_problem& pr = probs[p];
      const int local = t - cut[x];
      const int r = local / wgs, j = (local + kRoundRotation * r) % wgs;   // position in the round rotates
      fp8gmm_gemm_item& o = items[(size_t)r * grid + (size_t)j * kNumXcd + x];
      o = fp8gmm_gemm_item{};
      int m0 = 0, n0 = 0;
      tile_origin(pr.m, pr.n, (int)(t - tile_begin[p]), TM, TN, &m0, &n0);
      const int64_t rows = pr.m - m0 < TM ? pr.m - m0 : TM;
      const int64_t cols = pr.n - n0 < TN ? pr.n - n0 : TN;
      if (pr.k > 0) {
        if (!a_kmajor) {
          o.a = (uint64_t)reinterpret_cast<uintptr_t>(pr.a) + (uint64_t)m0 * (uint64_t)pr.lda;
          o.a_bytes = (uint32_t)((rows - 1) * pr.lda + ((pr.k + 15) & ~15));
        } else {
          o.a = (uint64_t)reinterpret_cast<uintptr_t>(pr.a) + (uint64_t)m0;
          o.a_bytes = (uint32_t)((int64_t)(pr.k - 1) * pr.lda + (pr.m - m0));
        }
        if (!b_kmajor) {
          o.b = (uint64_t)reinterpret_cast<uintptr_t>(pr.b) + (uint64_t)n0 * (uint64_t)pr.ldb;
          o.b_bytes = (uint32_t)((cols - 1) * pr.ldb + pr.k);
        } else {
          o.b = (uint64_t)reinterpret_cast<uintptr_t>(pr.b) + (uint64_t)n0;
          o.b_bytes = (uint32_t)((int64_t)(pr.k - 1) * pr.ldb + (pr.n - n0));
        }
      }
      o.lda = pr.lda;
      o.ldb = pr.ldb;
      o.k = pr.k;
      o.k_begin = 0;
      o.nk = (pr.k + 127) / 128;
      o.m0 = m0;
      o.n0 = n0;
      o.prob = p;
      o.slot = -1;
    }
  }
  return FP8GMM_OK;
}

int fp8gmm_plan_grouped_gemm_launch(fp8gmm_gemm_problem* probs, int n, int layout, int grid, int stream_k,
                                    fp8gmm_gemm_item* items, int max_items, fp8gmm_gemm_fixup_desc* fixups,
                                    int max_fixups, fp8gmm_gemm_plan* plan) {
  using namespace fp8gmm;
  if (plan == nullptr) return FP8GMM_ERR_NULL_POINTER;
  *plan = fp8gmm_gemm_plan{};
  if (grid <= 0 || (grid % kNumXcd) != 0 || max_items < 0 || max_fixups < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (layout & (FP8GMM_GEMM_TILE_128 | FP8GMM_GEMM_TILE_DUAL)) {
    if (layout & (FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU)) return FP8GMM_ERR_BAD_ARGUMENT;
    if ((layout & FP8GMM_GEMM_TILE_128) && (layout & FP8GMM_GEMM_TILE_DUAL)) return FP8GMM_ERR_BAD_ARGUMENT;
    const int operands = layout & ~(FP8GMM_GEMM_TILE_128 | FP8GMM_GEMM_TILE_DUAL);
    if (layout & FP8GMM_GEMM_TILE_128)
      return plan_whole_tiles(FP8GMM_GEMM_SMALL_TILE, FP8GMM_GEMM_SMALL_TILE, 3, probs, n, operands, grid, items,
                              max_items, plan);
    return plan_whole_tiles(FP8GMM_GEMM_DUAL_TILE_M, kGemmTileN, 2, probs, n, operands, grid, items, max_items, plan);
  }
  plan->tile = kGemmTileM;
  const int layout_given = layout, grid_given = grid;
  // the epilogue flags only weigh the decision to share tiles along K (completing a tile costs more with them)
  const bool gelu = (layout & (FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU)) != 0;
  layout &= ~(FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU);
  int total_tiles = 0;
  const int rc = fp8gmm_plan_grouped_gemm_layout(probs, n, layout, &total_tiles);
  if (rc != FP8GMM_OK) return rc;
  plan->total_tiles = total_tiles;
  if (total_tiles == 0) return FP8GMM_OK;
  // tail balancing can only pay when the launch has few rounds; it needs the whole grid even for few tiles
  const bool sk = stream_k != 0 && (int64_t)total_tiles <= (int64_t)kSkMaxRounds * grid && grid > kNumXcd;
  if (!sk) {
    const int needed = ((total_tiles + kNumXcd - 1) / kNumXcd) * kNumXcd;
    if (grid > needed) grid = needed;
  }
  const int wgs = grid / kNumXcd;
  const bool a_kmajor = (layout & FP8GMM_GEMM_A_KMAJOR) != 0, b_kmajor = (layout & FP8GMM_GEMM_B_KMAJOR) != 0;

  // pass 1: sizes.  The tiles that were shared along K first: the pieces of such a tile get consecutive
  // workspace slots, numbered from 0 over the launch, in K order.
  std::vector<Sched> sched(kNumXcd);
  for (int x = 0; x < kNumXcd; ++x) sched_init(sched[x], probs, n, total_tiles, x, wgs, sk, gelu ? 3 : 1);
  std::vector<int32_t> slot_map((size_t)kSlotsPerWg * grid, -1);
  std::vector<fp8gmm_gemm_fixup_desc> fix;
  int n_slots = 0;
  if (sk)
    for (int x = 0; x < kNumXcd; ++x)
      for (int j = 1; j < wgs; ++j) {
        int nf = 0;
        const int tile = fixup_tile(sched[x], j, &nf);
        if (tile < 0) continue;
        const int prob = problem_of_tile(sched[x], tile);
        fp8gmm_gemm_fixup_desc o{};
        o.prob = prob;
        tile_origin(probs[prob].m, probs[prob].n, tile - probs[prob].tile_begin, &o.m0, &o.n0);
        o.first_slot = n_slots;
        o.n_pieces = nf + 1;
        // uncompacted numbering: the piece from the tile's first K step sits in slot 2 (x wgs + j - 1) + 1,
        // the following ones in slots 2 (x wgs + q), q = j, j + 1, ...
        slot_map[kSlotsPerWg * (x * wgs + j - 1) + 1] = n_slots++;
        for (int q = j; q < j + nf; ++q) slot_map[kSlotsPerWg * (x * wgs + q)] = n_slots++;
        fix.push_back(o);
      }
  // a caller with a fixed amount of workspace (stream_k > 1 = its slots): whole tiles when sharing needs more
  if (sk && stream_k > 1 && n_slots > stream_k)
    return fp8gmm_plan_grouped_gemm_launch(probs, n, layout_given, grid_given, 0, items, max_items, fixups, max_fixups,
                                           plan);
  const int room = max_items;   // as the caller stated it
  // One pass over the schedule: the records are written as they are counted, into whatever room the caller gave;
  // a list that does not fit is only counted, and the call then reports the sizes.
  if (items == nullptr) max_items = 0;
  std::vector<int32_t> count(grid, 0);
  int rounds = 0;
  bool dangling_piece = false;
  auto write_record = [&](const Item& it, size_t index) {
    const fp8gmm_gemm_problem& p = probs[it.prob];
    fp8gmm_gemm_item o{};   // assembled in registers and stored once: stores into the list could alias anything
    const int64_t rows = p.m - it.m0 < BM ? p.m - it.m0 : BM;
    const int64_t cols = p.n - it.n0 < BN ? p.n - it.n0 : BN;
    if (p.k > 0) {
      // extents: up to the last byte of the tile's last row (row-major) / of the operand's last contraction row.
      // A row-major a whose k is not a multiple of 16 (allowed next to a contraction-major b) ends inside a
      // 16-byte piece; the bound includes the whole piece, which lies inside the row's pitch: the hardware
      // checks the range per dword, and a dword that straddled the bound would lose its valid bytes too.
      if (!a_kmajor) {
        o.a = (uint64_t)reinterpret_cast<uintptr_t>(p.a) + (uint64_t)it.m0 * (uint64_t)p.lda;
        o.a_bytes = (uint32_t)((rows - 1) * p.lda + ((p.k + 15) & ~15));
      } else {
        o.a = (uint64_t)reinterpret_cast<uintptr_t>(p.a) + (uint64_t)it.m0;
        o.a_bytes = (uint32_t)((int64_t)(p.k - 1) * p.lda + (p.m - it.m0));
      }
      if (!b_kmajor) {
        o.b = (uint64_t)reinterpret_cast<uintptr_t>(p.b) + (uint64_t)it.n0 * (uint64_t)p.ldb;
        o.b_bytes = (uint32_t)((cols - 1) * p.ldb + p.k);
      } else {
        o.b = (uint64_t)reinterpret_cast<uintptr_t>(p.b) + (uint64_t)it.n0;
        o.b_bytes = (uint32_t)((int64_t)(p.k - 1) * p.ldb + (p.n - it.n0));
      }
    }
    o.lda = p.lda;
    o.ldb = p.ldb;
    o.k = p.k;
    o.k_begin = it.k_begin;
    o.nk = it.nk;
    o.m0 = it.m0;
    o.n0 = it.n0;
    o.prob = it.prob;
    o.slot = -1;
    if (it.slot >= 0) {
      o.slot = slot_map[it.slot];
      if (o.slot < 0) dangling_piece = true;  // a partial item that no fix-up record completes
    } else if (rows <= BM / 2) {
      o.flags = FP8GMM_ITEM_HALF_HEIGHT;      // a whole tile with at most 128 valid rows
    }
    items[index] = o;
  };
  // The strided part, which holds nearly all records, round by round: record r of workgroup w sits at
  // items[r * grid + w], so this order writes the list front to back (one workgroup after the other writes a cache
  // line every 64 * grid bytes, which takes several times as long on lists of a few thousand records in fresh
  // memory).  The tiles and their order are those cursor_valid / cursor_item / cursor_advance give: a workgroup's
  // position in the round advances by kRoundRotation, modulo the workgroups of the XCD.
  struct Walk { int pos, prob; };
  std::vector<Walk> walk(grid);
  // problem and origin of every tile, filled in tile order without the divisions of tile_origin (its arithmetic,
  // walked: groups of kRasterRows rows of tiles, inside a group the row runs fastest)
  struct Where { int32_t prob, m0, n0; };
  std::vector<Where> where(items != nullptr ? total_tiles : 0);
  if (items != nullptr)
    for (int p = 0; p < n; ++p) {
      const int tiles_m = (probs[p].m + BM - 1) / BM, tiles_n = (probs[p].n + BN - 1) / BN;
      Where* w = where.data() + probs[p].tile_begin;
      for (int first = 0; first < tiles_m; first += kRasterRows) {
        const int rows = tiles_m - first < kRasterRows ? tiles_m - first : kRasterRows;
        for (int col = 0; col < tiles_n; ++col)
          for (int row = 0; row < rows; ++row) *w++ = Where{p, (first + row) * BM, col * BN};
      }
    }
  int strided_rounds = 0;
  const int rotation = kRoundRotation % wgs;   // every XCD has wgs workgroups
  for (int wg = 0; wg < grid; ++wg) {
    const Sched& sx = sched[wg % kNumXcd];
    walk[wg] = Walk{(wg / kNumXcd) % wgs, 0};
    if (sx.dp_rounds > strided_rounds) strided_rounds = sx.dp_rounds;
  }
  for (int r = 0; r < strided_rounds; ++r)
    for (int wg = 0; wg < grid; ++wg) {
      const Sched& sx = sched[wg % kNumXcd];
      if (count[wg] != r || r >= sx.dp_rounds) continue;   // this workgroup's strided part has ended
      Walk& w = walk[wg];
      const int tile = sx.range_begin + sx.wgs * r + w.pos;
      if (tile >= sx.sk_begin) continue;
      w.pos += rotation;
      if (w.pos >= wgs) w.pos -= wgs;
      count[wg] = r + 1;
      const size_t index = (size_t)r * grid + wg;
      if (index >= (size_t)max_items) continue;
      const Where& at = where[tile];
      w.prob = at.prob;
      Item it;
      it.tile = tile;
      it.prob = at.prob;
      it.m0 = at.m0;
      it.n0 = at.n0;
      it.k_begin = 0;
      it.nk = (probs[at.prob].k + 127) / 128;
      it.slot = -1;
      write_record(it, index);
    }
  // what is left: the pieces of the shared remainder
  for (int wg = 0; wg < grid; ++wg) {
    const int x = wg % kNumXcd, j = wg / kNumXcd;
    const Sched& sx = sched[x];
    Cursor c;
    cursor_init(sx, j, c);
    c.dp_i = count[wg];
    int r = count[wg], prob = walk[wg].prob;
    for (; cursor_valid(sx, j, c); cursor_advance(sx, j, c), ++r) {
      const size_t index = (size_t)r * grid + wg;
      if (index >= (size_t)max_items) continue;
      const Item it = cursor_item(sx, x, j, c, prob);
      prob = it.prob;
      write_record(it, index);
    }
    count[wg] = r;
    if (r > rounds) rounds = r;
  }
  // records without K steps repeat the height of the next record that has some (see FP8GMM_ITEM_HALF_HEIGHT)
  {
    std::vector<uint8_t> next_height(grid, 0);
    for (int r = rounds - 1; r >= 0; --r)
      for (int wg = 0; wg < grid; ++wg) {
        const size_t index = (size_t)r * grid + wg;
        if (r >= count[wg] || index >= (size_t)max_items) continue;
        fp8gmm_gemm_item& o = items[index];
        if (o.nk == 0) {
          o.flags |= next_height[wg] << 1;
        } else {
          next_height[wg] = (uint8_t)(o.flags & FP8GMM_ITEM_HALF_HEIGHT);
        }
      }
  }
  rounds += 1;  // every list ends with a record whose prob is -1
  const int n_fixups = (int)fix.size();
  plan->grid = grid;
  plan->rounds = rounds;
  plan->n_fixups = n_fixups;
  plan->n_slots = n_slots;
  if ((int64_t)rounds * grid > INT32_MAX / 64) return FP8GMM_ERR_BAD_SHAPE;
  if ((int64_t)rounds * grid > room || n_fixups > max_fixups) return FP8GMM_ERR_BUFFER_TOO_SMALL;
  if (items == nullptr || (n_fixups > 0 && fixups == nullptr)) return FP8GMM_ERR_NULL_POINTER;
  if (dangling_piece) return FP8GMM_ERR_BAD_ARGUMENT;
  for (int f = 0; f < n_fixups; ++f) fixups[f] = fix[f];
  fp8gmm_gemm_item end_record{};
  end_record.prob = -1;
  end_record.slot = -1;
  for (int r = 0; r < rounds; ++r)
    for (int wg = 0; wg < grid; ++wg)
      if (r >= count[wg]) items[(size_t)r * grid + wg] = end_record;
  return FP8GMM_OK;
}

}  // extern "C"
