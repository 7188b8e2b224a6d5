// One call that plans a whole pass of a grouped linear layer or of a grouped MLP: the tensor descriptors of its cast
// launches, the problem tables of its grouped GEMMs and their work lists, written straight into the (pinned) buffer
// that the caller uploads, plus a second call that runs one planned launch.  Host only.
//
// The reference does the equivalent host work per call in C++: CutlassFp8GroupedGemm builds the problem sizes,
// pointers and strides of every expert (csrc/fp8_gmm.cu:115-135) and MultiPadCastTranspose packs the tensor list
// into its kernel arguments (csrc/multi_pad_fusion.cu:455-502), driven by a Python loop over the experts
// (fp8_gmm/grouped_linear.py:109-188, fp8_gmm/grouped_mlp.py:60-318).  With 64 experts that loop - here: the array arithmetic that replaced it -
// costs more host time than the kernels run; from (group_sizes, base pointers, scaling-metadata bases) the whole
// pass is a few microseconds of C.
#include <stdint.h>
#include <string.h>

#include <vector>

#include "../../include/fp8gmm.h"
#include "internal.h"
#include "tiling.h"

namespace {

constexpr int64_t kLine = 128;
inline int64_t align_up(int64_t x) { return (x + kLine - 1) / kLine * kLine; }
inline uint8_t* at(void* base, int64_t bytes) { return static_cast<uint8_t*>(base) + bytes; }
inline const uint8_t* at(const void* base, int64_t bytes) { return static_cast<const uint8_t*>(base) + bytes; }

// Which tile a launch takes when the caller leaves the choice to the library: the 128 x 128 tile where the
// 256 x 256 tiles would be fewer than about half the compute units or mostly padding (see FP8GMM_GEMM_TILE_128).
bool small_tiles_pay(const fp8gmm_gemm_problem* p, int n) {
  int64_t large = 0, small = 0;
  for (int i = 0; i < n; ++i) {
    const int64_t m = p[i].m, nn = p[i].n;
    large += ((m + 255) / 256) * ((nn + 255) / 256);
    small += ((m + 127) / 128) * ((nn + 127) / 128);
  }
  return large != 0 && (large <= 160 || 2 * small <= 5 * large);
}

// ... and the form with two sets of accumulators (FP8GMM_GEMM_TILE_DUAL): a contraction of up to 2048 whose
// operands and result the 256 MB memory-side cache can largely hold, operand a row-major; what the tile boundaries
// cost such a launch is more than the form's extra operand traffic.
bool dual_tiles_pay(const fp8gmm_gemm_problem* p, int n, int layout) {
  if ((layout & FP8GMM_GEMM_A_KMAJOR) || n == 0) return false;
  int64_t bytes = 0;
  int32_t k_max = 0;
  for (int i = 0; i < n; ++i) {
    const int64_t m = p[i].m, nn = p[i].n, k = p[i].k;
    bytes += (m + nn) * k + 2 * m * nn;
    if (p[i].k > k_max) k_max = p[i].k;
  }
  return k_max <= 2048 && bytes <= ((int64_t)320 << 20);
}

struct Writer {
  void* blob;
  int64_t capacity;
  int64_t used = 0;        // bytes laid out so far (may exceed capacity: the pass is then only sized)
  bool fits = true;
  std::vector<std::vector<uint8_t>> aside;   // tables of a pass that does not fit: needed to size its work lists
  // `bytes` of the blob on their own cache lines; once the blob is full, memory on the side that is thrown away
  void* take(int64_t bytes, int64_t* offset) {
    *offset = used;
    used += align_up(bytes);
    if (blob == nullptr || used > capacity) {
      fits = false;
      aside.emplace_back((size_t)bytes + 1);
      return aside.back().data();
    }
    return at(blob, *offset);
  }
};

// the cast launch over `n` prepared descriptors
int plan_cast(Writer& w, fp8gmm_tensor_desc* descs, int n, int op, int out_fmt, fp8gmm_pass_launch* rec) {
  int total = 0;
  const int rc = fp8gmm_plan_multi_tensor(descs, n, op, &total);
  if (rc != FP8GMM_OK) return rc;
  rec->kind = total > 0 ? FP8GMM_PASS_CAST : FP8GMM_PASS_NOTHING;
  rec->op = op;
  rec->n = n;
  rec->total_blocks = total;
  rec->out_fmt = out_fmt;
  // quantize: 2 B read + 1 B written per element; with the GELU's derivative a second bf16 input
  const int64_t per_element = op == FP8GMM_OP_CAST_DGELU ? 5 : 3;
  int64_t work = 0;
  for (int i = 0; i < n; ++i) work += (int64_t)descs[i].rows * descs[i].cols * per_element;
  rec->work = (double)work;
  rec->bytes = (double)work;
  return FP8GMM_OK;
}

// a grouped GEMM over `n` prepared problems; the problems must already lie at their place in the blob
// (`epi`: FP8GMM_EPI_GELU or 0; a launch with that epilogue always takes the large tile, the only one that has it)
int plan_gemm(Writer& w, fp8gmm_gemm_problem* probs, int n, int layout, int tile_policy, int grid, int stream_k,
              int a_fmt, int b_fmt, fp8gmm_pass_launch* rec, int out_kind = FP8GMM_OUT_BF16, int epi = 0) {
  rec->op = 0;
  rec->n = n;
  rec->a_fmt = a_fmt;
  rec->b_fmt = b_fmt;
  rec->out_kind = out_kind;
  rec->epilogue = layout | epi;
  const bool small = epi == 0 && (tile_policy == 128 || (tile_policy == 0 && small_tiles_pay(probs, n)));
  const bool dual = !small && epi == 0 && out_kind == FP8GMM_OUT_BF16 &&
                    (tile_policy == FP8GMM_GEMM_TILE_DUAL || (tile_policy == 0 && dual_tiles_pay(probs, n, layout)));
  const int plan_layout = layout | epi | (small ? FP8GMM_GEMM_TILE_128 : dual ? FP8GMM_GEMM_TILE_DUAL : 0);
  const int plan_grid = small ? 2 * grid : grid;
  // room for the work list: whatever is left of the blob
  int64_t items_off = 0;
  int64_t room = w.fits ? (w.capacity - w.used) / (int64_t)sizeof(fp8gmm_gemm_item) : 0;
  if (room > INT32_MAX) room = INT32_MAX;
  if (room < 0) room = 0;
  fp8gmm_gemm_item* items = room > 0 ? reinterpret_cast<fp8gmm_gemm_item*>(at(w.blob, w.used)) : nullptr;
  // shared-tile records are few (at most one per workgroup): planned into a local array, appended afterwards
  static thread_local fp8gmm_gemm_fixup_desc fix[4096];
  int rc = fp8gmm_plan_grouped_gemm_launch(probs, n, plan_layout, plan_grid, small || dual ? 0 : stream_k, items, (int)room, fix,
                                           4096, &rec->plan);
  if (rc != FP8GMM_OK && rc != FP8GMM_ERR_BUFFER_TOO_SMALL) return rc;
  const int64_t item_bytes = (int64_t)rec->plan.rounds * rec->plan.grid * (int64_t)sizeof(fp8gmm_gemm_item);
  if (rc == FP8GMM_ERR_BUFFER_TOO_SMALL) w.fits = false;
  // the work list lies where it was planned (w.used has not moved since); when it did not fit it is only counted
  items_off = w.used;
  w.used += align_up(item_bytes);
  if (w.used > w.capacity) w.fits = false;
  int64_t fix_off = 0;
  void* fix_dst = w.take((int64_t)rec->plan.n_fixups * (int64_t)sizeof(fp8gmm_gemm_fixup_desc), &fix_off);
  if (rec->plan.n_fixups > 0) memcpy(fix_dst, fix, (size_t)rec->plan.n_fixups * sizeof(fp8gmm_gemm_fixup_desc));
  rec->items_offset = items_off;
  rec->fixups_offset = fix_off;
  rec->kind = rec->plan.total_tiles > 0 ? FP8GMM_PASS_GEMM : FP8GMM_PASS_NOTHING;
  double flops = 0, bytes = 0;
  for (int i = 0; i < n; ++i) {
    const double m = probs[i].m, nn = probs[i].n, k = probs[i].k;
    flops += 2.0 * m * nn * k;
    bytes += (m + nn) * k + m * nn * ((out_kind == FP8GMM_OUT_BF16 ? 2.0 : 1.0) + (probs[i].aux != nullptr ? 2.0 : 0.0));
  }
  rec->work = flops;
  rec->bytes = bytes;
  return FP8GMM_OK;
}

// A cast that is directly followed by a GEMM launch leaves the merge of its tensors' running maxima into the amax
// slots to that launch's first workgroup: the small launch that would do it, and the gap around it, cost a pass of
// config 3 or 4 as much as 1.5 % each.
void defer_amax_merges(fp8gmm_pass_plan* out) {
  for (int i = 0; i + 1 < out->n_launches; ++i) {
    fp8gmm_pass_launch& cast = out->launch[i];
    fp8gmm_pass_launch& next = out->launch[i + 1];
    if (cast.kind != FP8GMM_PASS_CAST || next.kind != FP8GMM_PASS_GEMM) continue;
    cast.merge_n = cast.n;
    next.merge_n = cast.n;
    next.merge_offset = cast.table_offset;
  }
}

int check_common(const fp8gmm_linear_pass* s, fp8gmm_pass_plan* out) {
  if (s == nullptr || out == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if (s->experts < 0 || s->in_features <= 0 || s->out_features <= 0 || s->grid <= 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (s->experts > 0 && s->group_sizes == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if ((s->in_features % 16) != 0 || (s->out_features % 16) != 0) return FP8GMM_ERR_ALIGNMENT;
  if (s->tile_policy != 0 && s->tile_policy != 128 && s->tile_policy != 256 && s->tile_policy != FP8GMM_GEMM_TILE_DUAL)
    return FP8GMM_ERR_BAD_ARGUMENT;
  int64_t rows = 0;
  for (int i = 0; i < s->experts; ++i) {
    if (s->group_sizes[i] < 0) return FP8GMM_ERR_BAD_SHAPE;
    rows += s->group_sizes[i];
  }
  if (rows != s->tokens) return FP8GMM_ERR_BAD_SHAPE;
  const int64_t widest = s->in_features > s->out_features ? s->in_features : s->out_features;
  if (rows * widest >= ((int64_t)1 << 31) * 64) return FP8GMM_ERR_BAD_SHAPE;
  return FP8GMM_OK;
}

}  // namespace

extern "C" {

int fp8gmm_plan_linear_forward(const fp8gmm_linear_pass* s, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out) {
  int rc = check_common(s, out);
  if (rc != FP8GMM_OK) return rc;
  memset(out, 0, sizeof(*out));
  if (s->x == nullptr || s->x_fp8 == nullptr || s->w_fp8 == nullptr || s->y == nullptr || s->fwd_scale == nullptr ||
      s->fwd_scale_inv == nullptr || s->fwd_amax == nullptr || (s->cast_weights && s->w == nullptr))
    return FP8GMM_ERR_NULL_POINTER;
  const int e = s->experts;
  const int64_t K = s->in_features, N = s->out_features;
  if (N * K >= ((int64_t)1 << 31)) return FP8GMM_ERR_BAD_SHAPE;
  Writer w{blob, (int64_t)blob_bytes};

  // ---- cast: the experts' activation slices, then (unless cached copies are reused) their weights
  const int n_cast = e + (s->cast_weights ? e : 0);
  int64_t off = 0;
  fp8gmm_tensor_desc* descs =
      static_cast<fp8gmm_tensor_desc*>(w.take((int64_t)n_cast * (int64_t)sizeof(fp8gmm_tensor_desc), &off));
  fp8gmm_pass_launch* cast = &out->launch[0];
  cast->table_offset = off;
  {
    memset(descs, 0, (size_t)n_cast * sizeof(fp8gmm_tensor_desc));
    int64_t row = 0;
    for (int i = 0; i < e; ++i) {
      const int64_t numel = s->group_sizes[i] * K;
      if (numel >= ((int64_t)1 << 31)) return FP8GMM_ERR_BAD_SHAPE;
      fp8gmm_tensor_desc& d = descs[i];
      d.in = at(s->x, row * K * 2);
      d.out = at(s->x_fp8, row * K);
      d.rows = numel > 0;
      d.cols = (int32_t)numel;
      d.scale = s->fwd_scale + 3 * i;
      d.amax = s->fwd_amax + 3 * i;
      row += s->group_sizes[i];
    }
    for (int i = 0; s->cast_weights && i < e; ++i) {
      fp8gmm_tensor_desc& d = descs[e + i];
      d.in = at(s->w, (int64_t)i * N * K * 2);
      d.out = at(s->w_fp8, (int64_t)i * N * K);
      d.rows = 1;
      d.cols = (int32_t)(N * K);
      d.scale = s->fwd_scale + 3 * i + 1;
      d.amax = s->fwd_amax + 3 * i + 1;
    }
    rc = plan_cast(w, descs, n_cast, FP8GMM_OP_QUANTIZE, s->fwd_fmt, cast);
    if (rc != FP8GMM_OK) return rc;
  }

  // ---- y[rows of expert i] = x_fp8[rows] . w_fp8[i]^T
  fp8gmm_gemm_problem* probs =
      static_cast<fp8gmm_gemm_problem*>(w.take((int64_t)e * (int64_t)sizeof(fp8gmm_gemm_problem), &off));
  fp8gmm_pass_launch* gemm = &out->launch[1];
  gemm->table_offset = off;
  {
    memset(probs, 0, (size_t)e * sizeof(fp8gmm_gemm_problem));
    int64_t row = 0;
    for (int i = 0; i < e; ++i) {
      fp8gmm_gemm_problem& p = probs[i];
      p.a = at(s->x_fp8, row * K);
      p.b = at(s->w_fp8, (int64_t)i * N * K);
      p.c = at(s->y, row * N * 2);
      p.m = (int32_t)s->group_sizes[i];
      p.n = (int32_t)N;
      p.k = (int32_t)K;
      p.lda = (int32_t)K;
      p.ldb = (int32_t)K;
      p.ldc = (int32_t)N;
      p.a_scale_inv = s->fwd_scale_inv + 3 * i;
      p.b_scale_inv = s->fwd_scale_inv + 3 * i + 1;
      row += s->group_sizes[i];
    }
    rc = plan_gemm(w, probs, e, 0, s->tile_policy, s->grid, s->stream_k, s->fwd_fmt, s->fwd_fmt, gemm);
    if (rc != FP8GMM_OK) return rc;
  }
  out->n_launches = 2;
  out->blob_bytes = w.used;
  defer_amax_merges(out);
  return w.fits ? FP8GMM_OK : FP8GMM_ERR_BUFFER_TOO_SMALL;
}

int fp8gmm_plan_linear_backward(const fp8gmm_linear_pass* s, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out) {
  int rc = check_common(s, out);
  if (rc != FP8GMM_OK) return rc;
  memset(out, 0, sizeof(*out));
  if (s->dy == nullptr || s->dy_fp8 == nullptr || s->bwd_scale == nullptr || s->bwd_scale_inv == nullptr ||
      s->bwd_amax == nullptr || s->fwd_scale_inv == nullptr)
    return FP8GMM_ERR_NULL_POINTER;
  if ((s->dgrad && (s->dx == nullptr || s->w_fp8 == nullptr)) || (s->wgrad && (s->dw == nullptr || s->x_fp8 == nullptr)))
    return FP8GMM_ERR_NULL_POINTER;
  const int e = s->experts;
  const int64_t K = s->in_features, N = s->out_features;
  Writer w{blob, (int64_t)blob_bytes};

  // ---- cast of the experts' gradient slices
  int64_t off = 0;
  fp8gmm_tensor_desc* descs = static_cast<fp8gmm_tensor_desc*>(w.take((int64_t)e * (int64_t)sizeof(fp8gmm_tensor_desc), &off));
  out->launch[0].table_offset = off;
  {
    memset(descs, 0, (size_t)e * sizeof(fp8gmm_tensor_desc));
    int64_t row = 0;
    for (int i = 0; i < e; ++i) {
      const int64_t numel = s->group_sizes[i] * N;
      if (numel >= ((int64_t)1 << 31)) return FP8GMM_ERR_BAD_SHAPE;
      fp8gmm_tensor_desc& d = descs[i];
      d.in = at(s->dy, row * N * 2);
      d.out = at(s->dy_fp8, row * N);
      d.rows = numel > 0;
      d.cols = (int32_t)numel;
      d.scale = s->bwd_scale + 2 * i;
      d.amax = s->bwd_amax + 2 * i;
      row += s->group_sizes[i];
    }
    rc = plan_cast(w, descs, e, FP8GMM_OP_QUANTIZE, s->bwd_fmt, &out->launch[0]);
    if (rc != FP8GMM_OK) return rc;
  }
  int n_launches = 1;

  // ---- dw[i] = dy_fp8[rows]^T . x_fp8[rows]: both read in place, contraction over the expert's rows.  Ahead of the
  // data gradient: its operands are the tensors the casts have just written, and a launch that reads them later, behind
  // the data gradient's pass over all the weights, finds less of them in the memory-side cache (config 3: 139 -> 126 us)
  if (s->wgrad) {
    fp8gmm_gemm_problem* probs =
        static_cast<fp8gmm_gemm_problem*>(w.take((int64_t)e * (int64_t)sizeof(fp8gmm_gemm_problem), &off));
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    rec->table_offset = off;
    {
      memset(probs, 0, (size_t)e * sizeof(fp8gmm_gemm_problem));
      int64_t row = 0;
      for (int i = 0; i < e; ++i) {
        fp8gmm_gemm_problem& p = probs[i];
        p.a = at(s->dy_fp8, row * N);
        p.b = at(s->x_fp8, row * K);
        p.c = at(s->dw, (int64_t)i * N * K * 2);
        p.m = (int32_t)N;
        p.n = (int32_t)K;
        p.k = (int32_t)s->group_sizes[i];
        p.lda = (int32_t)N;
        p.ldb = (int32_t)K;
        p.ldc = (int32_t)K;
        p.a_scale_inv = s->bwd_scale_inv + 2 * i;
        p.b_scale_inv = s->fwd_scale_inv + 3 * i;
        row += s->group_sizes[i];
      }
      rc = plan_gemm(w, probs, e, FP8GMM_GEMM_A_KMAJOR | FP8GMM_GEMM_B_KMAJOR, s->tile_policy, s->grid, s->stream_k,
                     s->bwd_fmt, s->fwd_fmt, rec);
      if (rc != FP8GMM_OK) return rc;
    }
  }
  // ---- dx[rows] = dy_fp8[rows] . w_fp8[i]: the forward weight [N, K] read in place as b[k = N][n = K]
  if (s->dgrad) {
    fp8gmm_gemm_problem* probs =
        static_cast<fp8gmm_gemm_problem*>(w.take((int64_t)e * (int64_t)sizeof(fp8gmm_gemm_problem), &off));
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    rec->table_offset = off;
    {
      memset(probs, 0, (size_t)e * sizeof(fp8gmm_gemm_problem));
      int64_t row = 0;
      for (int i = 0; i < e; ++i) {
        fp8gmm_gemm_problem& p = probs[i];
        p.a = at(s->dy_fp8, row * N);
        p.b = at(s->w_fp8, (int64_t)i * N * K);
        p.c = at(s->dx, row * K * 2);
        p.m = (int32_t)s->group_sizes[i];
        p.n = (int32_t)K;
        p.k = (int32_t)N;
        p.lda = (int32_t)N;
        p.ldb = (int32_t)K;
        p.ldc = (int32_t)K;
        p.a_scale_inv = s->bwd_scale_inv + 2 * i;
        p.b_scale_inv = s->fwd_scale_inv + 3 * i + 1;
        row += s->group_sizes[i];
      }
      rc = plan_gemm(w, probs, e, FP8GMM_GEMM_B_KMAJOR, s->tile_policy, s->grid, s->stream_k, s->bwd_fmt, s->fwd_fmt, rec);
      if (rc != FP8GMM_OK) return rc;
    }
  }

  out->n_launches = n_launches;
  out->blob_bytes = w.used;
  defer_amax_merges(out);
  return w.fits ? FP8GMM_OK : FP8GMM_ERR_BUFFER_TOO_SMALL;
}

int fp8gmm_run_planned(const void* blob_dev, const fp8gmm_pass_launch* rec, void* workspace, size_t workspace_bytes,
                       void* stream) {
  if (rec == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if (rec->kind == FP8GMM_PASS_NOTHING) return FP8GMM_OK;
  if (blob_dev == nullptr) return FP8GMM_ERR_NULL_POINTER;
  uint8_t* base = const_cast<uint8_t*>(static_cast<const uint8_t*>(blob_dev));
  if (rec->kind == FP8GMM_PASS_CAST) {
    fp8gmm_tensor_desc* descs = reinterpret_cast<fp8gmm_tensor_desc*>(base + rec->table_offset);
    switch (rec->op) {
      case FP8GMM_OP_QUANTIZE:
        if (rec->merge_n != 0)
          return fp8gmm::launch_cast_unmerged(descs, rec->n, rec->total_blocks, rec->out_fmt, false, stream);
        return fp8gmm_multi_quantize(descs, rec->n, rec->total_blocks, rec->out_fmt, stream);
      case FP8GMM_OP_CAST_DGELU:
        if (rec->merge_n != 0)
          return fp8gmm::launch_cast_unmerged(descs, rec->n, rec->total_blocks, rec->out_fmt, true, stream);
        return fp8gmm_multi_cast_dgelu(descs, rec->n, rec->total_blocks, rec->out_fmt, stream);
      default: return FP8GMM_ERR_BAD_ARGUMENT;
    }
  }
  if (rec->kind == FP8GMM_PASS_GEMM) {
    const fp8gmm_gemm_fixup_desc* fix =
        rec->plan.n_fixups > 0 ? reinterpret_cast<const fp8gmm_gemm_fixup_desc*>(base + rec->fixups_offset) : nullptr;
    return fp8gmm::launch_gemm_merging(
        reinterpret_cast<const fp8gmm_gemm_problem*>(base + rec->table_offset), rec->n,
        reinterpret_cast<const fp8gmm_gemm_item*>(base + rec->items_offset), fix, &rec->plan, rec->a_fmt, rec->b_fmt,
        rec->out_kind, rec->epilogue, workspace, workspace_bytes,
        rec->merge_n > 0 ? reinterpret_cast<const fp8gmm_tensor_desc*>(base + rec->merge_offset) : nullptr, rec->merge_n,
        stream);
  }
  return FP8GMM_ERR_BAD_ARGUMENT;
}

size_t fp8gmm_sizeof_linear_pass(void) { return sizeof(fp8gmm_linear_pass); }
size_t fp8gmm_sizeof_pass_plan(void) { return sizeof(fp8gmm_pass_plan); }

}  // extern "C"

namespace {

int check_mlp(const fp8gmm_mlp_pass* s, fp8gmm_pass_plan* out) {
  if (s == nullptr || out == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if (s->experts < 0 || s->hidden <= 0 || s->ffn <= 0 || s->grid <= 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (s->experts > 0 && s->group_sizes == nullptr) return FP8GMM_ERR_NULL_POINTER;
  if ((s->hidden % 16) != 0 || (s->ffn % 16) != 0) return FP8GMM_ERR_ALIGNMENT;
  if (s->tile_policy != 0 && s->tile_policy != 128 && s->tile_policy != 256 && s->tile_policy != FP8GMM_GEMM_TILE_DUAL)
    return FP8GMM_ERR_BAD_ARGUMENT;
  const int64_t widest = s->hidden > s->ffn ? s->hidden : s->ffn;
  int64_t rows = 0;
  for (int i = 0; i < s->experts; ++i) {
    if (s->group_sizes[i] < 0) return FP8GMM_ERR_BAD_SHAPE;
    if (s->group_sizes[i] * widest >= ((int64_t)1 << 31)) return FP8GMM_ERR_BAD_SHAPE;
    rows += s->group_sizes[i];
  }
  if (rows != s->tokens) return FP8GMM_ERR_BAD_SHAPE;
  if (rows * widest >= ((int64_t)1 << 31) * 64 || (int64_t)s->hidden * s->ffn >= ((int64_t)1 << 31))
    return FP8GMM_ERR_BAD_SHAPE;
  return FP8GMM_OK;
}

// One row-sliced tensor [tokens, cols] as `e` cast descriptors, one per expert (scaling slots `stride` apart)
void slice_descs(fp8gmm_tensor_desc* d, const fp8gmm_mlp_pass* s, const void* in, const void* in2, void* out,
                 int64_t cols, const float* scale, float* amax, int stride) {
  int64_t row = 0;
  for (int i = 0; i < s->experts; ++i) {
    const int64_t numel = s->group_sizes[i] * cols;
    d[i].in = at(in, row * cols * 2);
    if (in2 != nullptr) d[i].in2 = at(in2, row * cols * 2);
    d[i].out = at(out, row * cols);
    d[i].rows = numel > 0;
    d[i].cols = (int32_t)numel;
    d[i].scale = scale + (int64_t)stride * i;
    d[i].amax = amax + (int64_t)stride * i;
    row += s->group_sizes[i];
  }
}

// One weight stack [experts, numel] as `e` cast descriptors
void stack_descs(fp8gmm_tensor_desc* d, int e, const void* in, void* out, int64_t numel, const float* scale, float* amax) {
  for (int i = 0; i < e; ++i) {
    d[i].in = at(in, (int64_t)i * numel * 2);
    d[i].out = at(out, (int64_t)i * numel);
    d[i].rows = 1;
    d[i].cols = (int32_t)numel;
    d[i].scale = scale + 3 * (int64_t)i;
    d[i].amax = amax + 3 * (int64_t)i;
  }
}

// c[rows_i][:n] = a[rows_i][:k] . b[i]: `b` a weight stack whose expert i is n x k (kmajor: k x n, read as it lies)
void row_problems(fp8gmm_gemm_problem* p, const fp8gmm_mlp_pass* s, const void* a, const void* b, void* c, int c_bytes,
                  void* aux, int64_t n, int64_t k, bool b_kmajor, const float* a_si, int a_stride, const float* b_si,
                  const float* c_scale, float* c_amax) {
  int64_t row = 0;
  for (int i = 0; i < s->experts; ++i) {
    p[i].a = at(a, row * k);
    p[i].b = at(b, (int64_t)i * n * k);
    p[i].c = at(c, row * n * c_bytes);
    if (aux != nullptr) p[i].aux = at(aux, row * n * 2);
    p[i].m = (int32_t)s->group_sizes[i];
    p[i].n = (int32_t)n;
    p[i].k = (int32_t)k;
    p[i].lda = (int32_t)k;
    p[i].ldb = (int32_t)(b_kmajor ? n : k);
    p[i].ldc = (int32_t)n;
    p[i].a_scale_inv = a_si + (int64_t)a_stride * i;
    p[i].b_scale_inv = b_si + 3 * (int64_t)i;
    if (c_scale != nullptr) {
      p[i].c_scale = c_scale + 3 * (int64_t)i;
      p[i].c_amax = c_amax + 3 * (int64_t)i;
    }
    row += s->group_sizes[i];
  }
}

// c[i] (m x n) = a[rows_i]^T . b[rows_i]: both operands [tokens, m] / [tokens, n], contraction over the expert's rows
void weight_gradient_problems(fp8gmm_gemm_problem* p, const fp8gmm_mlp_pass* s, const void* a, const void* b, void* c,
                              int64_t m, int64_t n, const float* a_si, const float* b_si) {
  int64_t row = 0;
  for (int i = 0; i < s->experts; ++i) {
    p[i].a = at(a, row * m);
    p[i].b = at(b, row * n);
    p[i].c = at(c, (int64_t)i * m * n * 2);
    p[i].m = (int32_t)m;
    p[i].n = (int32_t)n;
    p[i].k = (int32_t)s->group_sizes[i];
    p[i].lda = (int32_t)m;
    p[i].ldb = (int32_t)n;
    p[i].ldc = (int32_t)n;
    p[i].a_scale_inv = a_si + 2 * (int64_t)i;
    p[i].b_scale_inv = b_si + 3 * (int64_t)i;
    row += s->group_sizes[i];
  }
}

template <typename T>
T* table_of(Writer& w, int n, fp8gmm_pass_launch* rec) {
  int64_t off = 0;
  T* t = static_cast<T*>(w.take((int64_t)n * (int64_t)sizeof(T), &off));
  memset(t, 0, (size_t)n * sizeof(T));
  rec->table_offset = off;
  return t;
}

}  // namespace

extern "C" {

int fp8gmm_plan_mlp_forward(const fp8gmm_mlp_pass* s, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out) {
  int rc = check_mlp(s, out);
  if (rc != FP8GMM_OK) return rc;
  memset(out, 0, sizeof(*out));
  if (s->x == nullptr || s->x_fp8 == nullptr || s->w1_fp8 == nullptr || s->w2_fp8 == nullptr || s->pre == nullptr ||
      s->act_fp8 == nullptr || s->y == nullptr || s->fwd_scale == nullptr || s->fwd_scale_inv == nullptr ||
      s->fwd_amax == nullptr || (s->cast_weights && (s->w1 == nullptr || s->w2 == nullptr)))
    return FP8GMM_ERR_NULL_POINTER;
  const int e = s->experts;
  const int64_t H = s->hidden, F = s->ffn;
  const int64_t g2 = 3 * (int64_t)e;   // first forward slot of the fc2 GEMMs
  Writer w{blob, (int64_t)blob_bytes};

  // ---- cast.  fc2's weights first and the input last: the launch walks its table in order, and what it wrote last is
  // what the memory-side cache still holds when fc1's GEMM starts reading
  {
    const int n_cast = e + (s->cast_weights ? 2 * e : 0);
    fp8gmm_pass_launch* rec = &out->launch[0];
    fp8gmm_tensor_desc* d = table_of<fp8gmm_tensor_desc>(w, n_cast, rec);
    if (s->cast_weights) {
      stack_descs(d, e, s->w2, s->w2_fp8, H * F, s->fwd_scale + g2 + 1, s->fwd_amax + g2 + 1);
      stack_descs(d + e, e, s->w1, s->w1_fp8, H * F, s->fwd_scale + 1, s->fwd_amax + 1);
    }
    slice_descs(d + (n_cast - e), s, s->x, nullptr, s->x_fp8, H, s->fwd_scale, s->fwd_amax, 3);
    rc = plan_cast(w, d, n_cast, FP8GMM_OP_QUANTIZE, s->fwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- fc1 with the GELU in its epilogue: pre (bf16) and act_fp8 = fp8(gelu(pre) * scale of fc2's input)
  {
    fp8gmm_pass_launch* rec = &out->launch[1];
    fp8gmm_gemm_problem* p = table_of<fp8gmm_gemm_problem>(w, e, rec);
    row_problems(p, s, s->x_fp8, s->w1_fp8, s->act_fp8, 1, s->pre, F, H, false, s->fwd_scale_inv, 3, s->fwd_scale_inv + 1,
                 s->fwd_scale + g2, s->fwd_amax + g2);
    rc = plan_gemm(w, p, e, 0, s->tile_policy, s->grid, s->stream_k, s->fwd_fmt, s->fwd_fmt, rec,
                   s->fwd_fmt, FP8GMM_EPI_GELU);   // an fp8 result's out_kind is its format
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- fc2
  {
    fp8gmm_pass_launch* rec = &out->launch[2];
    fp8gmm_gemm_problem* p = table_of<fp8gmm_gemm_problem>(w, e, rec);
    row_problems(p, s, s->act_fp8, s->w2_fp8, s->y, 2, nullptr, H, F, false, s->fwd_scale_inv + g2, 3,
                 s->fwd_scale_inv + g2 + 1, nullptr, nullptr);
    rc = plan_gemm(w, p, e, 0, s->tile_policy, s->grid, s->stream_k, s->fwd_fmt, s->fwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  out->n_launches = 3;
  out->blob_bytes = w.used;
  defer_amax_merges(out);
  return w.fits ? FP8GMM_OK : FP8GMM_ERR_BUFFER_TOO_SMALL;
}

int fp8gmm_plan_mlp_backward(const fp8gmm_mlp_pass* s, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out) {
  int rc = check_mlp(s, out);
  if (rc != FP8GMM_OK) return rc;
  memset(out, 0, sizeof(*out));
  if (s->dy == nullptr || s->dy_fp8 == nullptr || s->w2_fp8 == nullptr || s->pre == nullptr || s->dact == nullptr ||
      s->dpre_fp8 == nullptr || s->bwd_scale == nullptr || s->bwd_scale_inv == nullptr || s->bwd_amax == nullptr ||
      s->fwd_scale_inv == nullptr)
    return FP8GMM_ERR_NULL_POINTER;
  if ((s->dgrad && (s->dx == nullptr || s->w1_fp8 == nullptr)) ||
      (s->wgrad && (s->dw1 == nullptr || s->dw2 == nullptr || s->x_fp8 == nullptr || s->act_fp8 == nullptr)))
    return FP8GMM_ERR_NULL_POINTER;
  const int e = s->experts;
  const int64_t H = s->hidden, F = s->ffn;
  const int64_t f2 = 3 * (int64_t)e, b2 = 2 * (int64_t)e;   // first forward / backward slot of the fc2 GEMMs
  const int kmajor_both = FP8GMM_GEMM_A_KMAJOR | FP8GMM_GEMM_B_KMAJOR;
  Writer w{blob, (int64_t)blob_bytes};
  int n_launches = 0;

  // ---- cast of the gradient.  It takes the first group of backward slots although it belongs to fc2, and the
  // gradient of pre the second (fp8_gmm/grouped_mlp.py:183-184,278-279): the groups follow the order of the pass
  {
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    fp8gmm_tensor_desc* d = table_of<fp8gmm_tensor_desc>(w, e, rec);
    slice_descs(d, s, s->dy, nullptr, s->dy_fp8, H, s->bwd_scale, s->bwd_amax, 2);
    rc = plan_cast(w, d, e, FP8GMM_OP_QUANTIZE, s->bwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- dw2[i] (H x F) = dy_fp8[rows_i]^T . act_fp8[rows_i]
  if (s->wgrad) {
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    fp8gmm_gemm_problem* p = table_of<fp8gmm_gemm_problem>(w, e, rec);
    weight_gradient_problems(p, s, s->dy_fp8, s->act_fp8, s->dw2, H, F, s->bwd_scale_inv, s->fwd_scale_inv + f2);
    rc = plan_gemm(w, p, e, kmajor_both, s->tile_policy, s->grid, s->stream_k, s->bwd_fmt, s->fwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- dact[rows_i] = dy_fp8[rows_i] . w2_fp8[i]   (w2[i] is H x F: read in place as b[k = H][n = F])
  {
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    fp8gmm_gemm_problem* p = table_of<fp8gmm_gemm_problem>(w, e, rec);
    row_problems(p, s, s->dy_fp8, s->w2_fp8, s->dact, 2, nullptr, F, H, true, s->bwd_scale_inv, 2,
                 s->fwd_scale_inv + f2 + 1, nullptr, nullptr);
    rc = plan_gemm(w, p, e, FP8GMM_GEMM_B_KMAJOR, s->tile_policy, s->grid, s->stream_k, s->bwd_fmt, s->fwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- dpre_fp8 = fp8(dact * dgelu(pre))
  {
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    fp8gmm_tensor_desc* d = table_of<fp8gmm_tensor_desc>(w, e, rec);
    slice_descs(d, s, s->dact, s->pre, s->dpre_fp8, F, s->bwd_scale + b2, s->bwd_amax + b2, 2);
    rc = plan_cast(w, d, e, FP8GMM_OP_CAST_DGELU, s->bwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- dx[rows_i] = dpre_fp8[rows_i] . w1_fp8[i]   (w1[i] is F x H: b[k = F][n = H])
  if (s->dgrad) {
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    fp8gmm_gemm_problem* p = table_of<fp8gmm_gemm_problem>(w, e, rec);
    row_problems(p, s, s->dpre_fp8, s->w1_fp8, s->dx, 2, nullptr, H, F, true, s->bwd_scale_inv + b2, 2,
                 s->fwd_scale_inv + 1, nullptr, nullptr);
    rc = plan_gemm(w, p, e, FP8GMM_GEMM_B_KMAJOR, s->tile_policy, s->grid, s->stream_k, s->bwd_fmt, s->fwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  // ---- dw1[i] (F x H) = dpre_fp8[rows_i]^T . x_fp8[rows_i]
  if (s->wgrad) {
    fp8gmm_pass_launch* rec = &out->launch[n_launches++];
    fp8gmm_gemm_problem* p = table_of<fp8gmm_gemm_problem>(w, e, rec);
    weight_gradient_problems(p, s, s->dpre_fp8, s->x_fp8, s->dw1, F, H, s->bwd_scale_inv + b2, s->fwd_scale_inv);
    rc = plan_gemm(w, p, e, kmajor_both, s->tile_policy, s->grid, s->stream_k, s->bwd_fmt, s->fwd_fmt, rec);
    if (rc != FP8GMM_OK) return rc;
  }
  out->n_launches = n_launches;
  out->blob_bytes = w.used;
  defer_amax_merges(out);
  return w.fits ? FP8GMM_OK : FP8GMM_ERR_BUFFER_TOO_SMALL;
}

size_t fp8gmm_sizeof_mlp_pass(void) { return sizeof(fp8gmm_mlp_pass); }

}  // extern "C"
