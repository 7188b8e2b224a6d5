/*
 * fp8gmm - C ABI of the MI355X (gfx950) FP8 grouped-GEMM library.
 *
 * This is the boundary that replaces the reference's pybind11 module
 * `fp8_gmm_backend` (csrc/ops.cu:9-16).  Every function is `extern "C"`,
 * takes plain pointers and integers, returns an int status (0 = success,
 * negative = fp8gmm_status) and never throws, allocates, frees or synchronises:
 * scratch memory (the grouped GEMM's tail-balancing workspace, the router's
 * counters) is passed in by the caller.  fp8gmm_init is the one call that talks to
 * the runtime about anything but a launch.
 * All device work is enqueued on the HIP stream passed in (`hipStream_t`,
 * passed as `void*`; NULL = the default stream).
 *
 * Multi-tensor calls and the grouped GEMM read their work list from a table in
 * DEVICE memory (no 64-tensor limit, unlike the reference's 4 KB by-value
 * argument structs, csrc/multi_pointwise.cu:13, csrc/multi_pad_fusion.cu:14).
 * The protocol is:
 *   1. the caller fills an array of descriptors in host memory;
 *   2. `fp8gmm_plan_*` validates it, fills the scheduling fields
 *      (`block_begin` / `tile_begin`) and returns the launch size; for the GEMM
 *      it also writes the launch's work list (one record per workgroup and tile);
 *   3. the caller copies the arrays to device memory on the same stream;
 *   4. `fp8gmm_multi_*` / `fp8gmm_grouped_gemm` launches one kernel over the
 *      device copies.
 * The library never owns memory; outputs are written in place.
 */
#ifndef FP8GMM_H_
#define FP8GMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Counts the incompatible changes of this interface (a struct layout, the meaning of a field or an argument): a
 * binding compares fp8gmm_version() of the library it loaded with the value it was written against. */
#define FP8GMM_VERSION 3

/* fp8 formats (OCP): e4m3fn = torch.float8_e4m3fn, e5m2 = torch.float8_e5m2 */
#define FP8GMM_E4M3 0
#define FP8GMM_E5M2 1
/* output kind of the GEMM epilogue */
#define FP8GMM_OUT_BF16 2

typedef enum fp8gmm_status {
  FP8GMM_OK = 0,
  FP8GMM_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
  FP8GMM_ERR_BAD_SHAPE = -2,      /* negative size, rows_padded < rows, size overflow */
  FP8GMM_ERR_BAD_FORMAT = -3,     /* unknown fp8 format / unsupported format pair */
  FP8GMM_ERR_ALIGNMENT = -4,      /* GEMM operand not 16-byte aligned / K or pitch not a multiple of 16 */
  FP8GMM_ERR_LAUNCH = -5,         /* the HIP runtime rejected the launch */
  FP8GMM_ERR_BAD_ARGUMENT = -6,   /* inconsistent scalar arguments (count < 0, total mismatch, ...) */
  FP8GMM_ERR_NO_DEVICE = -7,      /* no usable gfx950 device */
  FP8GMM_ERR_BUFFER_TOO_SMALL = -8, /* an output array of a planning call cannot hold the result (sizes are returned) */
  FP8GMM_ERR_WORKSPACE = -9       /* the launch needs more workspace than it was given */
} fp8gmm_status;

/*
 * One tensor of a multi-tensor call.  `rows x cols` row-major, contiguous.
 *
 *  op                              in         in2        out             out_t                       scale / amax
 *  multi_quantize                  bf16       -          fp8 same shape  -                           read / max-merged
 *  multi_scale_mul                 bf16 (rw)  -          -               -                           scale, scale2 read
 *  multi_pad_transpose             fp8        -          -               fp8 [cols, rows_padded]     -
 *  multi_pad_cast_transpose        bf16       -          fp8 (or NULL)   fp8 [cols, rows_padded]     read / max-merged
 *  multi_pad_cast_transpose_dgelu  bf16 dy    bf16 pre   fp8 (or NULL)   fp8 [cols, rows_padded]     read / max-merged
 *  multi_cast_dgelu                bf16 dy    bf16 pre   fp8 same shape  -                           read / max-merged
 *
 * `scale` NULL means 1.0 (reference csrc/multi_pointwise.cu:51); `amax` NULL
 * means "do not record" (csrc/multi_pad_fusion.cu:290).  `amax` is merged with
 * its previous content by an integer atomic max and must hold a non-negative
 * value on entry (csrc/utils.cuh:183-185).  The workgroups of a tensor first
 * reduce into the descriptor's own `amax_partial` (one cache line per tensor:
 * the amax slots of the reference's layout sit a few bytes apart, and thousands
 * of atomics on one line serialise); a second, tiny launch of the same call
 * merges the partials into the slots.  The device table is therefore WRITTEN by
 * the calls that record amax and has to be uploaded afresh for every call.  For quantize / scale_mul, `cols`
 * may carry the whole element count with rows = 1.
 */
typedef struct fp8gmm_tensor_desc {
  const void* in;
  const void* in2;      /* dgelu: pre-GELU input; scale_mul: second scale (const float*) */
  void* out;
  void* out_t;
  const float* scale;
  float* amax;
  int32_t rows;
  int32_t cols;
  int32_t rows_padded;  /* second dimension of out_t, >= rows; ignored by ops without out_t */
  int32_t block_begin;  /* filled by fp8gmm_plan_*: first workgroup of this tensor */
  uint32_t amax_partial; /* scratch of the kernels, zeroed by fp8gmm_plan_*: running max|x| of this tensor */
  uint32_t reserved[15]; /* pads the descriptor to one 128-byte cache line */
} fp8gmm_tensor_desc;   /* 128 bytes */

/* which multi-tensor kernel a plan is for */
#define FP8GMM_OP_QUANTIZE 0
#define FP8GMM_OP_SCALE_MUL 1
#define FP8GMM_OP_PAD_TRANSPOSE 2
#define FP8GMM_OP_PAD_CAST_TRANSPOSE 3
#define FP8GMM_OP_PAD_CAST_TRANSPOSE_DGELU 4
#define FP8GMM_OP_CAST_DGELU 5

/*
 * One GEMM of a grouped launch:  c[m, n] = epilogue( a[m, k] . b[n, k]^T ).
 * Both operands are K-contiguous ("TN"), the only layout the reference uses
 * (fp8_gmm/backend.py:25,57; csrc/fp8_gmm.h:7-11).  Pitches are in elements.
 * a, b must be 16-byte aligned and k, lda, ldb multiples of 16 (the same
 * divisibility cuBLASLt demands of the reference, grouped_linear.py:68); 256 rows of an operand
 * may span at most 4 GiB (256 * lda, 256 * ldb < 2^32).
 * k == 0 is allowed and writes epilogue(0); m == 0 or n == 0 produce no work.
 *
 * Epilogue:  v = acc * (*a_scale_inv * *b_scale_inv)        (NULL scale = 1)
 *   gelu off: r = v;   gelu on: r = gelu_tanh(v) and, if aux != NULL, aux = bf16(v)
 *   out bf16: c = bf16(r)
 *   out fp8 : c = fp8_saturate(r * *c_scale), *c_amax = max(*c_amax, max|r|)
 * This is the behaviour the reference obtains from cuBLASLt through
 * fp8_gmm/backend.py:26-54 (scaled TN GEMM, optional GELU-aux epilogue and fp8
 * output with amax), and - with the scales folded in - what
 * csrc/fp8_gmm.cu:163 + MultiScaleMul compute on the CUTLASS path.
 */
typedef struct fp8gmm_gemm_problem {
  const void* a;
  const void* b;
  void* c;
  void* aux;                 /* bf16 [m, n] pre-GELU output, pitch ldc, or NULL */
  const float* a_scale_inv;
  const float* b_scale_inv;
  const float* c_scale;      /* fp8 output only */
  float* c_amax;             /* fp8 output only, may be NULL */
  int32_t m, n, k;
  int32_t lda, ldb, ldc;
  int32_t tile_begin;        /* filled by fp8gmm_plan_grouped_gemm */
  int32_t cost_begin;        /* filled by fp8gmm_plan_grouped_gemm: K = 128 steps of all earlier tiles */
} fp8gmm_gemm_problem;       /* 96 bytes */

/* flags of fp8gmm_grouped_gemm (its `epilogue` argument) */
#define FP8GMM_EPI_GELU 1
/* The derivative of the GELU folded into a data-gradient GEMM: `aux` is an INPUT, the bf16 pre-GELU activation
 * [m, n] (pitch ldc) that the forward GELU-aux epilogue wrote, and
 *   x = v * dgelu_tanh(aux);   out fp8: c = fp8_saturate(x * *c_scale), *c_amax = max(*c_amax, max|x|);   out bf16: c = bf16(x)
 * The reference forms x from the bf16-rounded v in a pass of its own (MultiPadCastTransposeDgelu,
 * csrc/multi_pad_fusion.cu:587, after the fc2 data-gradient GEMM, fp8_gmm/grouped_mlp.py:243-287) and notes the
 * missing fusion (:252-253); here v stays in fp32 until the one rounding to fp8.  Not together with
 * FP8GMM_EPI_GELU. */
#define FP8GMM_EPI_DGELU 8
/* b is stored contraction-major: b[k, n] with n contiguous and ldb >= n its row pitch, i.e.
 * c[m, n] = epilogue( a[m, k] . b[k, n] ).  This is a forward weight [N_fwd = k, K_fwd = n] as the data-gradient
 * GEMM needs it, read in place: the reference casts a transposed copy of every weight for that GEMM instead
 * (fp8_gmm/grouped_linear.py:69-74,163).  b must be e4m3, n a multiple of 16, (k + 128) * ldb < 2^32.  Plan such tables
 * with fp8gmm_plan_grouped_gemm_layout(..., FP8GMM_GEMM_B_KMAJOR, ...).  k need not be a multiple of 16 in this
 * layout: the rows of b past k read as zeros, so the columns k .. roundup(k, 16) - 1 of a (which must exist: lda is a
 * multiple of 16) only have to hold finite values - zeros, when a is a padded transposed copy.  That is the
 * weight-gradient GEMM with a transposed copy of the gradient and the activation read in place. */
#define FP8GMM_GEMM_B_KMAJOR 2
/* a is stored contraction-major as well: a[k, m] with m contiguous and lda >= m, i.e.
 * c[m, n] = epilogue( a[k, m]^T . b[k, n] ): the weight-gradient GEMM dW[N, K] = dY[M, N]^T . X[M, K] on the
 * row-major gradient and activation, without the padded transposed copies the reference casts for it
 * (fp8_gmm/grouped_linear.py:36-52,142-150).  Only together with FP8GMM_GEMM_B_KMAJOR; m and n multiples of
 * 16, k arbitrary (rows past k contribute zeros), (k + 128) * lda < 2^32. */
#define FP8GMM_GEMM_A_KMAJOR 4
/* Planning flag (fp8gmm_plan_grouped_gemm_launch's `layout` only): cut the outputs into 128 x 128 tiles instead of
 * 256 x 256 and run two workgroups per compute unit (pass a grid of 2 * fp8gmm_gemm_grid()).  For launches whose
 * contraction is short (K up to about 2048) or whose problems have few rows: a workgroup's epilogue, tile switch and
 * waits for operands then overlap the other workgroup's arithmetic, and ragged problems pad to 128 rows.  Costs
 * twice the operand traffic from L2 per flop.  Never shares tiles along K (stream_k is ignored); not available with
 * FP8GMM_EPI_GELU.  No counterpart in the reference (CUTLASS picks its tile shape at compile time,
 * csrc/fp8_gmm.cu:82-110). */
#define FP8GMM_GEMM_TILE_128 0x100
#define FP8GMM_GEMM_SMALL_TILE 128
/* Planning flag (`layout` of fp8gmm_plan_grouped_gemm_launch only): cut the outputs into tiles of 128 rows x 256
 * columns for the kernel form with two sets of accumulators per wavefront, which stores a finished tile in pieces
 * between the products of the next one (one workgroup per compute unit, the usual grid).  For launches with a short
 * contraction (up to about 2048) that fill the machine, which otherwise spend as long at their tile boundaries as in
 * their main loops; costs 1.33 x the operand traffic from L2 per flop.  bf16 results without FP8GMM_EPI_* only; never
 * shares tiles along K (stream_k is ignored).  No counterpart in the reference. */
#define FP8GMM_GEMM_TILE_DUAL 0x200
#define FP8GMM_GEMM_DUAL_TILE_M 128

/*
 * Work list of a grouped-GEMM launch, written by fp8gmm_plan_grouped_gemm_launch on the host and read by the
 * kernel: the launch has `grid` persistent workgroups (a multiple of 8; workgroup i runs on XCD i % 8), and
 * workgroup w processes the records items[r * grid + w], r = 0, 1, ..., up to the first record with
 * prob == -1.  A record is one 256 x 256 tile of one problem's c, or - for the tail tiles that the
 * workgroups of an XCD share along K - a contiguous range of K = 128 steps of one, whose fp32 partial sums go
 * to a workspace slot.  The record carries what the kernel's load stream needs (operand addresses of the
 * tile, extents for the bounds check, pitches), so that switching tiles costs it one 64-byte read.
 * No counterpart in the reference: CUTLASS's tile scheduler computes the equivalent on the device
 * (csrc/fp8_gmm.cu:73-80,146-159).
 */
typedef struct fp8gmm_gemm_item {
  uint64_t a;          /* first byte of the tile's rows of operand a (row-major: a + m0 * lda; contraction-major: a + m0) */
  uint64_t b;          /* the same for operand b and n0 */
  uint32_t a_bytes;    /* bytes addressable from `a`: reads past them deliver zeros */
  uint32_t b_bytes;
  int32_t lda, ldb;
  int32_t k;           /* contraction length of the problem */
  int32_t k_begin;     /* first K = 128 step of this record */
  int32_t nk;          /* number of K = 128 steps (0: a problem without K, only the epilogue runs) */
  int32_t m0, n0;      /* origin of the tile in c */
  int32_t prob;        /* index into the problem table; -1 ends a workgroup's list */
  int32_t slot;        /* -1: whole tile, the epilogue runs; else the workspace slot that receives the partial sums */
  int32_t flags;       /* FP8GMM_ITEM_* */
} fp8gmm_gemm_item;    /* 64 bytes */
/* The tile holds at most 128 valid rows (the last row of tiles of a ragged problem): the kernel runs it at half
 * height - its wavefronts stand on rows 64 w + 32 i, i < 2, and issue half the products; same loads, same bits.
 * Whole 256 x 256 tiles only (never a piece of a tile shared along K).  In a record without K steps (nk == 0) the
 * bit one position up repeats this flag of the workgroup's next record that has K steps: the kernel's load stream
 * skips records without K steps, and what it fetches at the end of a tile is laid out for the tile that follows. */
#define FP8GMM_ITEM_HALF_HEIGHT 1

/* One tile that was shared along K: the fix-up launch adds the partial sums of the workspace slots first_slot,
 * first_slot + 1, ..., first_slot + n_pieces - 1 (the tile's pieces in K order) and runs the epilogue. */
typedef struct fp8gmm_gemm_fixup_desc {
  int32_t prob, m0, n0;
  int32_t first_slot, n_pieces;
  int32_t reserved[3];
} fp8gmm_gemm_fixup_desc;   /* 32 bytes */

/* Sizes of a planned launch. */
typedef struct fp8gmm_gemm_plan {
  int32_t grid;        /* workgroups of the main launch */
  int32_t rounds;      /* records per workgroup, end record included: items has rounds * grid entries */
  int32_t n_fixups;    /* tiles shared along K = workgroups of the fix-up launch (0: no such launch) */
  int32_t n_slots;     /* workspace slots the launch writes: it needs n_slots * FP8GMM_GEMM_SLOT_BYTES bytes */
  int32_t total_tiles;
  int32_t tile;        /* columns of a tile: 256, or 128 when planned with FP8GMM_GEMM_TILE_128 (0 reads as 256) */
  int32_t tile_m;      /* rows of a tile where they differ from `tile`: 128 when planned with FP8GMM_GEMM_TILE_DUAL (0: as `tile`) */
  int32_t reserved;
} fp8gmm_gemm_plan;    /* 32 bytes */

#define FP8GMM_GEMM_SLOT_BYTES 262144  /* fp32 accumulators of one 256 x 256 tile */
#define FP8GMM_GEMM_STATIC_SLOTS 256   /* slots of the library's own scratch (fp8gmm_grouped_gemm_static): 64 MiB */

/* ---- library info ------------------------------------------------------------------------- */
int fp8gmm_version(void);
const char* fp8gmm_status_string(int status);
size_t fp8gmm_sizeof_tensor_desc(void);   /* lets a binding check its struct layout */
size_t fp8gmm_sizeof_gemm_problem(void);
size_t fp8gmm_sizeof_gemm_item(void);
/*
 * Once per device, before the first launch on it (with that device current or named here; -1 = the current one):
 * looks up the device's compute-unit count and lets the GEMM kernels use the whole LDS.  Returns the number of
 * compute units (> 0) or a negative status.  Launches on a device that was never initialised do this themselves
 * on their first call; calling it explicitly keeps that work out of a timed or captured region.
 */
int fp8gmm_init(int device);
/* grid of a grouped-GEMM launch on a device with `num_cu` compute units: one workgroup per unit, a multiple of 8 */
int fp8gmm_gemm_grid(int num_cu);
/* workgroup tile of the GEMM kernel (rows of c, columns of c), for callers that size grids */
void fp8gmm_gemm_tile_shape(int* tile_m, int* tile_n);

/* ---- planning (host only, no GPU needed) -------------------------------------------------- */
/* Validates `descs[0..n)` for `op` (FP8GMM_OP_*), fills block_begin, returns the launch size
 * in *total_blocks.  Replaces the host halves of MultiQuantize / MultiScaleMul /
 * MultiPad* (csrc/multi_pointwise.cu:155-189,216-246; csrc/multi_pad_fusion.cu:442-488,505-559,587-644). */
int fp8gmm_plan_multi_tensor(fp8gmm_tensor_desc* descs, int n, int op, int* total_blocks);

/* Validates `probs[0..n)`, fills tile_begin / cost_begin, returns the tile count in *total_tiles.
 * Replaces the host half of CutlassFp8GroupedGemm (csrc/fp8_gmm.cu:82-135). */
int fp8gmm_plan_grouped_gemm(fp8gmm_gemm_problem* probs, int n, int* total_tiles);
/* The same for a launch with layout flags (0, FP8GMM_GEMM_B_KMAJOR, or both KMAJOR flags): only the checks on
 * the operands differ. */
int fp8gmm_plan_grouped_gemm_layout(fp8gmm_gemm_problem* probs, int n, int layout, int* total_tiles);

/* ---- launches (descs_dev / probs_dev: DEVICE copies of planned tables) ------------------- */
/* replaces MultiQuantize, csrc/multi_pointwise.cu:155 (pybind name multi_quantize, csrc/ops.cu:11) */
int fp8gmm_multi_quantize(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, void* stream);
/* replaces MultiScaleMul, csrc/multi_pointwise.cu:216 (multi_scale_mul, csrc/ops.cu:12) */
int fp8gmm_multi_scale_mul(const fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, void* stream);
/* replaces MultiPadTranspose, csrc/multi_pad_fusion.cu:442 (multi_pad_transpose, csrc/ops.cu:13) */
int fp8gmm_multi_pad_transpose(const fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, void* stream);
/* replaces MultiPadCastTranspose, csrc/multi_pad_fusion.cu:505 (multi_pad_cast_transpose, csrc/ops.cu:14) */
int fp8gmm_multi_pad_cast_transpose(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt,
                                    void* stream);
/* replaces MultiPadCastTransposeDgelu, csrc/multi_pad_fusion.cu:587 (multi_pad_cast_transpose_dgelu, csrc/ops.cu:15) */
int fp8gmm_multi_pad_cast_transpose_dgelu(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt,
                                          void* stream);

/* x = dy * dgelu(pre) cast to fp8 WITHOUT the transposed copy: the kernel the reference says it lacks
 * ("Maybe need a new kernel for cast_dgelu only when weight requires no grad", fp8_gmm/grouped_mlp.py:252-253).
 * Same values and bytes as the `out` of fp8gmm_multi_pad_cast_transpose_dgelu. */
int fp8gmm_multi_cast_dgelu(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, void* stream);

/*
 * Validates `probs[0..n)` like fp8gmm_plan_grouped_gemm_layout, fills tile_begin / cost_begin, and writes the work
 * list of a launch with `grid` workgroups (fp8gmm_gemm_grid) into items[0 .. rounds * grid) and
 * fixups[0 .. n_fixups).  `layout` takes the launch's flags: the KMAJOR flags as for the plain plan, and
 * FP8GMM_EPI_GELU / FP8GMM_EPI_DGELU, which only weigh the decision below (completing a shared tile costs more with that epilogue).  stream_k != 0: the workgroups of an XCD share the tail tiles of their range along K when
 * the last round would otherwise be mostly idle; the launch then needs plan->n_slots workspace slots (never more
 * than 2 * grid).  stream_k > 1: the same, but with at most stream_k slots - a launch whose sharing would need more
 * is planned with whole tiles instead (callers of fp8gmm_grouped_gemm_static pass FP8GMM_GEMM_STATIC_SLOTS and never
 * see FP8GMM_ERR_WORKSPACE).  stream_k == 0: every record is a whole tile, no workspace, no fix-up launch.
 * The sizes are returned in *plan even when max_items / max_fixups are too small (FP8GMM_ERR_BUFFER_TOO_SMALL;
 * the arrays then hold the part of the list that fitted and are not to be used): call again with larger arrays.  Host only, no GPU needed.
 */
int fp8gmm_plan_grouped_gemm_launch(fp8gmm_gemm_problem* probs, int n, int layout, int grid, int stream_k,
                                    fp8gmm_gemm_item* items, int max_items, fp8gmm_gemm_fixup_desc* fixups,
                                    int max_fixups, fp8gmm_gemm_plan* plan);

/*
 * One persistent launch over all tiles of all problems (plus a small second launch when tiles were shared along K).
 * replaces Fp8GroupedGemm, csrc/fp8_gmm.cu:163 (pybind name fp8_gmm, csrc/ops.cu:10) and the
 * per-expert cuBLASLt loop of fp8_gmm/backend.py:84-96 and grouped_linear.py:173-182.
 *   probs_dev, items_dev, fixups_dev : DEVICE copies of the planned arrays (fixups_dev may be NULL when n_fixups == 0)
 *   plan         : the host struct fp8gmm_plan_grouped_gemm_launch filled
 *   a_fmt, b_fmt : FP8GMM_E4M3 / FP8GMM_E5M2 (e5m2 x e5m2 is rejected, as cuBLASLt does)
 *   out_kind     : FP8GMM_OUT_BF16, or FP8GMM_E4M3 / FP8GMM_E5M2 for an fp8 `c`
 *   epilogue     : FP8GMM_EPI_GELU or FP8GMM_EPI_DGELU, and the layout flags the table was planned with
 *   workspace    : device memory, workspace_bytes >= plan->n_slots * FP8GMM_GEMM_SLOT_BYTES, 256-byte aligned,
 *                  contents irrelevant; may be NULL when n_slots == 0.  Launches that overlap in time (different
 *                  streams) need different workspaces.  Too small: FP8GMM_ERR_WORKSPACE, nothing is launched.
 */
int fp8gmm_grouped_gemm(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                        const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt, int b_fmt,
                        int out_kind, int epilogue, void* workspace, size_t workspace_bytes, void* stream);

/*
 * fp8gmm_grouped_gemm for callers that cannot allocate a workspace (code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc).  No counterpart in the reference.  The partial sums of tiles shared along K
 * go to a scratch array that is part of the library's device image: 64 MiB (FP8GMM_GEMM_STATIC_SLOTS slots) on
 * every GPU the library runs on, held until the process ends.  The call allocates and frees nothing.  A plan
 * with more slots is refused with FP8GMM_ERR_WORKSPACE and nothing is launched (plan it with stream_k = 0, which
 * needs no slots, or call fp8gmm_grouped_gemm with a workspace).  All calls on one GPU share the array: calls
 * that overlap in time (different streams, or threads) race on it; calls on one stream are ordered and safe.
 * Nothing needs clearing between calls: a launch writes every slot before it reads it.  The device address of
 * the array is looked up by fp8gmm_init (or by the first call on a device that was never initialised).
 */
int fp8gmm_grouped_gemm_static(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                               const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt,
                               int b_fmt, int out_kind, int epilogue, void* stream);

/* ---- a whole pass of a grouped linear layer, planned by one call ---------------------------- */
/*
 * The launches of one pass of a grouped linear layer (E experts, in_features -> out_features, token-sorted rows) in
 * the default data flow: activations, gradients and weights are cast to fp8 once, row-major, and every GEMM reads
 * them in place.
 *   forward : cast x (and, unless cast_weights == 0, the weights) ; y[rows_i] = x_fp8[rows_i] . w_fp8[i]^T
 *   backward: cast dy ; dw[i] = dy_fp8[rows_i]^T . x_fp8[rows_i]  (wgrad != 0) ; dx[rows_i] = dy_fp8[rows_i] . w_fp8[i]
 *             (dgrad != 0)
 * replaces, for that data flow, the per-expert host loops of fp8_gmm/grouped_linear.py:109-188 and the argument
 * packing of csrc/fp8_gmm.cu:115-135 and csrc/multi_pad_fusion.cu:455-502.  The scaling metadata is addressed
 * through the bases of the flat fp32 arrays in TransformerEngine's slot layout, which the reference indexes in
 * fp8_gmm/utils.py:98-103: forward slots 3 i (input of expert i) and 3 i + 1 (its weight), backward slot 2 i (its
 * output gradient).  For the backward pass fwd_scale_inv is the copy of the forward scale_inv taken after the
 * forward pass.  All data pointers are device pointers that are only stored, never dereferenced, by the planner.
 */
typedef struct fp8gmm_linear_pass {
  int32_t experts, in_features, out_features;
  int32_t fwd_fmt, bwd_fmt;          /* FP8GMM_E4M3 / FP8GMM_E5M2 of forward tensors and of gradients */
  int32_t cast_weights;              /* forward: 0 when w_fp8 already holds the cast weights (cached) */
  int32_t dgrad, wgrad;              /* backward: which gradients are wanted */
  int32_t grid;                      /* fp8gmm_gemm_grid() of the device */
  int32_t stream_k;                  /* as for fp8gmm_plan_grouped_gemm_launch */
  int32_t tile_policy;               /* 0: the library chooses per launch; 256 or 128: that tile for every launch;
                                        FP8GMM_GEMM_TILE_DUAL: the 128 x 256 form for every launch that can take it */
  int32_t reserved;
  int64_t tokens;                    /* rows of x / dy: must equal the sum of group_sizes */
  const int64_t* group_sizes;        /* HOST array [experts] */
  const void* x;                     /* bf16 [tokens, in_features] */
  void* x_fp8;                       /* fp8  [tokens, in_features] */
  const void* w;                     /* bf16 [experts, out_features, in_features] */
  void* w_fp8;                       /* fp8, same shape */
  void* y;                           /* bf16 [tokens, out_features] */
  const void* dy;                    /* bf16 [tokens, out_features] */
  void* dy_fp8;                      /* fp8, same shape */
  void* dx;                          /* bf16 [tokens, in_features] */
  void* dw;                          /* bf16 [experts, out_features, in_features] */
  const float* fwd_scale;
  const float* fwd_scale_inv;
  float* fwd_amax;                   /* row 0 of the forward amax history */
  const float* bwd_scale;
  const float* bwd_scale_inv;
  float* bwd_amax;
} fp8gmm_linear_pass;

#define FP8GMM_PASS_NOTHING 0   /* a launch that turned out empty (no rows at all) */
#define FP8GMM_PASS_CAST 1
#define FP8GMM_PASS_GEMM 2
/* One launch of a planned pass; offsets are bytes from the start of the blob. */
typedef struct fp8gmm_pass_launch {
  int32_t kind;                  /* FP8GMM_PASS_* */
  int32_t op;                    /* cast: FP8GMM_OP_* */
  int32_t n;                     /* descriptors / problems */
  int32_t total_blocks;          /* cast: workgroups */
  int32_t out_fmt;               /* cast: fp8 format written */
  int32_t a_fmt, b_fmt, out_kind, epilogue;   /* GEMM: the arguments of fp8gmm_grouped_gemm */
  int32_t merge_n;               /* cast: != 0: its amax merge is left to the GEMM launch behind it, whose first
                                    workgroup runs it.  GEMM: descriptors of the cast in front whose merge it runs (0: none) */
  int64_t table_offset;          /* descriptors / problem table */
  int64_t items_offset;          /* GEMM: work list */
  int64_t fixups_offset;         /* GEMM: shared-tile records */
  int64_t merge_offset;          /* GEMM with merge_n != 0: the descriptors of that cast */
  fp8gmm_gemm_plan plan;         /* GEMM */
  double work;                   /* algorithmic flops (GEMM) or bytes (cast) of the launch */
  double bytes;                  /* algorithmic bytes: every operand read once, every result written once */
} fp8gmm_pass_launch;
typedef struct fp8gmm_pass_plan {
  int32_t n_launches;
  int32_t reserved;
  int64_t blob_bytes;            /* bytes of the blob in use: what has to be uploaded */
  fp8gmm_pass_launch launch[8];
} fp8gmm_pass_plan;
size_t fp8gmm_sizeof_linear_pass(void);
size_t fp8gmm_sizeof_pass_plan(void);
/*
 * Write every table of the pass into `blob` (host memory, preferably pinned, 128-byte aligned; blob_bytes its
 * capacity) and describe the launches in *out.  FP8GMM_ERR_BUFFER_TOO_SMALL: out->blob_bytes says how much room the
 * pass needs; call again.  The tables are those that the per-launch planning calls produce for the same tensors.
 * Host only, no GPU needed.
 */
int fp8gmm_plan_linear_forward(const fp8gmm_linear_pass* pass, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out);
int fp8gmm_plan_linear_backward(const fp8gmm_linear_pass* pass, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out);
/* Enqueue one launch of a planned pass; blob_dev is the DEVICE copy of the blob (the cast launch writes into its
 * descriptors, so every pass uploads afresh); workspace as for fp8gmm_grouped_gemm.  Run the launches of a pass in
 * their order, all of them, on one stream: a cast whose record has merge_n != 0 has left the merge of its tensors'
 * maxima into the amax slots to the GEMM launch behind it. */
int fp8gmm_run_planned(const void* blob_dev, const fp8gmm_pass_launch* launch, void* workspace, size_t workspace_bytes,
                       void* stream);

/*
 * The same for a grouped MLP (E experts, hidden -> ffn -> hidden with the tanh GELU between, token-sorted rows) in
 * its default data flow:
 *   forward : cast w2, w1 (unless cast_weights == 0) and x ;
 *             act_fp8[rows_i], pre[rows_i] = gelu epilogue of x_fp8[rows_i] . w1_fp8[i]^T (FP8GMM_EPI_GELU) ;
 *             y[rows_i] = act_fp8[rows_i] . w2_fp8[i]^T
 *   backward: cast dy ; dw2[i] = dy_fp8[rows_i]^T . act_fp8[rows_i] (wgrad != 0) ; dact[rows_i] = dy_fp8[rows_i] . w2_fp8[i] ;
 *             dpre_fp8 = fp8(dact * dgelu(pre)) (FP8GMM_OP_CAST_DGELU) ; dx[rows_i] = dpre_fp8[rows_i] . w1_fp8[i] (dgrad != 0) ;
 *             dw1[i] = dpre_fp8[rows_i]^T . x_fp8[rows_i] (wgrad != 0)
 * replaces, for that data flow, the host side of fp8_gmm/grouped_mlp.py:18-325.  Scaling slots as the reference
 * indexes them (fp8_gmm/utils.py:98-103) with 2 E GEMMs, fc1 of expert i being GEMM i and fc2 GEMM E + i: forward
 * slots 3 g (input of GEMM g), 3 g + 1 (its weight); backward slots 2 i for dy and 2 E + 2 i for the gradient of pre
 * (the reference's kGradOutputGroup1 / kGradOutputGroup2, fp8_gmm/grouped_mlp.py:183-184,278-279).  fwd_scale_inv is
 * the live array in the forward pass and the copy taken after it in the backward pass.
 */
typedef struct fp8gmm_mlp_pass {
  int32_t experts, hidden, ffn;
  int32_t fwd_fmt, bwd_fmt;
  int32_t cast_weights;              /* forward: 0 when w1_fp8 / w2_fp8 already hold the cast weights */
  int32_t dgrad, wgrad;              /* backward: gradient of the input / of the weights wanted */
  int32_t grid, stream_k, tile_policy, reserved;   /* as in fp8gmm_linear_pass */
  int64_t tokens;
  const int64_t* group_sizes;        /* HOST array [experts] */
  const void* x;                     /* bf16 [tokens, hidden] */
  void* x_fp8;                       /* fp8, same shape */
  const void* w1;                    /* bf16 [experts, ffn, hidden] */
  void* w1_fp8;
  const void* w2;                    /* bf16 [experts, hidden, ffn] */
  void* w2_fp8;
  void* pre;                         /* bf16 [tokens, ffn]: pre-GELU activation (written forward, read backward) */
  void* act_fp8;                     /* fp8  [tokens, ffn]: gelu(pre) */
  void* y;                           /* bf16 [tokens, hidden] */
  const void* dy;                    /* bf16 [tokens, hidden] */
  void* dy_fp8;
  void* dact;                        /* bf16 [tokens, ffn]: gradient of gelu(pre) */
  void* dpre_fp8;                    /* fp8  [tokens, ffn]: gradient of pre */
  void* dx;                          /* bf16 [tokens, hidden] */
  void* dw1;                         /* bf16 [experts, ffn, hidden] */
  void* dw2;                         /* bf16 [experts, hidden, ffn] */
  const float* fwd_scale;
  const float* fwd_scale_inv;
  float* fwd_amax;
  const float* bwd_scale;
  const float* bwd_scale_inv;
  float* bwd_amax;
} fp8gmm_mlp_pass;
size_t fp8gmm_sizeof_mlp_pass(void);
int fp8gmm_plan_mlp_forward(const fp8gmm_mlp_pass* pass, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out);
int fp8gmm_plan_mlp_backward(const fp8gmm_mlp_pass* pass, void* blob, size_t blob_bytes, fp8gmm_pass_plan* out);

/*
 * Delayed-scaling update of one direction, in place, for `slots` scaling factors:
 *   amax = max over the `history_len` rows of amax_history[history_len, slots] (most_recent != 0: row 0)
 *   scale = (1 / amax) * fp8_max * 2^-margin where amax is finite and > 0, else unchanged;  scale_inv = 1 / scale
 *   keep_period > 0: scale_inv of the slots with slot % keep_period == keep_phase is left as it is (the weights'
 *   slots while fp8 weights cast in an earlier micro-batch are reused: they must keep the factor they were cast with)
 *   the history moves up by one row (the last row receives the old row 0) and row 0 is cleared.
 * replaces the amax_and_scale_update of TransformerEngine's base module, which the reference's modules run
 * through `self.prepare_forward(...)` (fp8_gmm/grouped_linear.py:206, fp8_gmm/grouped_mlp.py:349).
 */
int fp8gmm_delayed_scaling_update(float* amax_history, float* scale, float* scale_inv, int history_len, int slots,
                                  float fp8_max, int margin, int most_recent, int keep_period, int keep_phase,
                                  void* stream);

/* The same for up to FP8GMM_MAX_SCALING_UPDATES directions in ONE launch (a module's forward and backward state are
 * updated at the same point, in front of a forward pass: one kernel instead of two per step).  `updates` is a HOST
 * array; its contents travel as a kernel argument. */
#define FP8GMM_MAX_SCALING_UPDATES 4
typedef struct fp8gmm_scaling_update {
  float* amax_history;   /* [history_len, slots] */
  float* scale;          /* [slots] */
  float* scale_inv;      /* [slots] */
  int32_t history_len, slots;
  float fp8_max;
  int32_t margin, most_recent, keep_period, keep_phase, reserved;
} fp8gmm_scaling_update;   /* 56 bytes */
int fp8gmm_delayed_scaling_updates(const fp8gmm_scaling_update* updates, int n, void* stream);

/*
 * Page-locked host memory that the device can read (for fp8gmm_upload's source), allocated also while a stream is
 * being captured into a graph, when the runtime refuses ordinary allocations: the tables of a captured launch are
 * read again at every replay, so they need memory that outlives the capture and is not recycled, which a staging
 * ring cannot give.  The caller keeps it unchanged and alive as long as the graph.  NULL when the allocation fails.
 * No counterpart in the reference (whose launches take their tables as kernel arguments).
 */
void* fp8gmm_host_alloc(size_t bytes);
void fp8gmm_host_free(void* p);

/*
 * Copy `bytes` of tables from page-locked host memory that the device can address (hipHostMalloc; torch's
 * pin_memory) to device memory with a kernel on `stream`: dst_dev, src_host and bytes multiples of 16, at most
 * 1 GiB.  The host memory must stay as it is until the stream has passed this point.  Every launch entry point of
 * this header reads its tables from device memory; the reference hands the same tables over as launch arguments
 * (csrc/multi_pad_fusion.cu:14-35,495-501, csrc/multi_pointwise.cu) or with one synchronous copy per array
 * (cutlass::DeviceAllocation::copy_from_host, csrc/fp8_gmm.cu:116-135).  A hipMemcpyAsync on the stream does the
 * same job; measured here its hand-over to the next kernel costs 25 - 30 us per copy, a kernel's 2 - 4.
 */
int fp8gmm_upload(void* dst_dev, const void* src_host, size_t bytes, void* stream);

/* ---- token routing around the expert layers ----------------------------------------------- */
/*
 * The reference's example MoE layers (fp8_gmm/example.py:15-32,50-59,86-94,113-119) take these steps from the
 * megablocks package, which is not part of the reference tree (no version is pinned anywhere in it); the
 * functions below implement the published meaning of megablocks.ops.sort / histogram / inclusive_cumsum /
 * gather / scatter for int32 expert ids and bf16 rows.
 *
 * fp8gmm_route_sort: stable sort of `expert_of[0..n)` (values in [0, num_experts), num_experts <= 4096; values
 * outside are clamped into the range) by expert.  Every output may be NULL:
 *   bin_ids[p]  expert of sorted position p            (ops.sort, first result)
 *   indices[p]  original position of sorted position p (ops.sort, second result)
 *   inverse[i]  sorted position of original position i (the inverse permutation)
 *   tokens_per_expert[e]  entries of expert e          (ops.histogram)
 *   bins[e]     end of expert e in sorted order        (ops.inclusive_cumsum of the histogram)
 * replaces indices_and_bins, fp8_gmm/example.py:26-32.  `workspace`: fp8gmm_route_workspace_bytes(n, num_experts)
 * bytes of device memory, contents irrelevant.
 */
size_t fp8gmm_route_workspace_bytes(int n, int num_experts);
int fp8gmm_route_sort(const int32_t* expert_of, int n, int num_experts, int32_t* bin_ids, int32_t* indices,
                      int32_t* inverse, int32_t* tokens_per_expert, int32_t* bins, void* workspace, void* stream);
/*
 * The router's choice, replacing `topk` of fp8_gmm/example.py:15-23 (softmax over the experts in fp32, then
 * torch.topk; without its moe_renorm option): probs[t, :] = softmax(scores[t, :]) and, for k < top_k (at most 8),
 * selected[t, k] = the expert with the k-th largest score of token t (the lower expert on equal scores) and
 * weights[t, k] = its probability.  scores: [tokens, num_experts] bf16 (scores_bf16 != 0) or fp32, contiguous;
 * probs: fp32 [tokens, num_experts], kept for the backward pass.
 */
int fp8gmm_route_topk(const void* scores, int scores_bf16, int tokens, int num_experts, int top_k, float* probs,
                      float* weights, int64_t* selected, void* stream);
/* grad_scores[t, j] = probs[t, j] * (g_j - sum_i g_i probs[t, i]), g = grad_weights[t, :] scattered to the selected
 * experts: the gradient of `weights` above with respect to `scores`, written as bf16 (grad_bf16 != 0) or fp32. */
int fp8gmm_route_topk_backward(const float* probs, const int64_t* selected, const float* grad_weights, int tokens,
                               int num_experts, int top_k, void* grad_scores, int grad_bf16, void* stream);
/* inverse[indices[i]] = i for a permutation `indices` of 0..n-1 (entries outside that range are skipped) */
int fp8gmm_route_invert(const int32_t* indices, int n, int32_t* inverse, void* stream);
/*
 * out[i, :] = bf16(w_i * x[indices[i] / top_k, :]) for i in [0, rows_out), w_i = weights[indices[i]] or 1 when
 * weights == NULL (then rows are copied unchanged).  x: bf16 [rows_out / top_k, hidden], out: bf16 [rows_out, hidden].
 * replaces ops.gather (fp8_gmm/example.py:52,88,115) and, with weights, the backward pass of ops.scatter.
 */
int fp8gmm_moe_gather(const void* x, const int32_t* indices, const float* weights, void* out, int rows_out,
                      int hidden, int top_k, void* stream);
/*
 * out[t, :] = bf16(sum_k w[t * top_k + k] * x[inverse[t * top_k + k], :]) for t in [0, tokens): fp32 sum over
 * k = 0 .. top_k - 1 in that order, each product rounded to fp32 before it is added; w = 1 when weights == NULL.
 * x: bf16 [tokens * top_k, hidden] in sorted order, out: bf16 [tokens, hidden].
 * replaces ops.scatter (fp8_gmm/example.py:59,94,119) and, without weights, the backward pass of ops.gather.
 */
int fp8gmm_moe_scatter(const void* x, const int32_t* inverse, const float* weights, void* out, int tokens, int hidden,
                       int top_k, void* stream);
/* grad_w[indices[i]] = < x[i, :], grad_out[indices[i] / top_k, :] > in fp32: gradient of ops.scatter with respect
 * to its weights.  x: bf16 [rows, hidden] (sorted order), grad_out: bf16 [rows / top_k, hidden], grad_w: fp32 [rows]. */
int fp8gmm_moe_scatter_wgrad(const void* x, const void* grad_out, const int32_t* indices, float* grad_w, int rows,
                             int hidden, int top_k, void* stream);
/* The whole backward pass of ops.scatter (fp8_gmm/example.py:59,94,119) in one launch: grad_x[i, :] =
 * bf16(weights[indices[i]] * grad_out[indices[i] / top_k, :]) as fp8gmm_moe_gather writes it with weights, and
 * grad_w as fp8gmm_moe_scatter_wgrad writes it, the gradient rows read once for both.  The same bits as the two
 * calls.  grad_x: bf16 [rows, hidden]. */
int fp8gmm_moe_scatter_backward(const void* x, const void* grad_out, const int32_t* indices, const float* weights,
                                void* grad_x, float* grad_w, int rows, int hidden, int top_k, void* stream);

/* ---- schedule introspection (host only, no GPU needed) ------------------------------------ */
/*
 * The work items that workgroup `wg` of a grouped-GEMM launch with `grid` workgroups (a multiple of 8)
 * processes, in order, for the HOST table `probs` (after fp8gmm_plan_grouped_gemm).  stream_k != 0:
 * as in a launch that shares the tail tiles of each XCD's range along K.  Writes up to max_items records
 * of 7 int32 - tile, problem, m0, n0, k_begin, nk, slot (k_begin / nk in steps of 128 bytes of K; slot = -1
 * when the item is a whole tile, else its position 2 * workgroup or 2 * workgroup + 1 in the launch's uncompacted
 * slot numbering; fp8gmm_plan_grouped_gemm_launch renumbers the slots in use from 0) - and returns the
 * number of items.  No counterpart in the reference (its CUTLASS scheduler is not observable); it lets the
 * schedule be checked without a GPU.
 */
int fp8gmm_gemm_schedule(const fp8gmm_gemm_problem* probs, int n, int total_tiles, int grid, int stream_k, int wg,
                         int32_t* items, int max_items);
/*
 * The tile that fix-up workgroup `wg` (0 <= wg < grid - 8) of such a launch completes (*tile, -1: none) and
 * the workspace slots whose partial sums it adds, in K order (up to max_slots); returns their number.
 */
int fp8gmm_gemm_fixup(const fp8gmm_gemm_problem* probs, int n, int total_tiles, int grid, int wg, int32_t* tile,
                      int32_t* slots, int max_slots);

#ifdef __cplusplus
}
#endif
#endif /* FP8GMM_H_ */
