// Persistent FP8 grouped GEMM for gfx950 (MI355X): the kernel template and its launcher.  Included by
// gemm_variant.hip, which is compiled once per operand format / layout combination, and by grouped_gemm.hip.
//
// Replaces the reference's CUTLASS grouped GEMM (csrc/fp8_gmm.cu:82-205) and its
// per-expert cuBLASLt loops (fp8_gmm/backend.py:84-96, grouped_linear.py:173-182,
// grouped_mlp.py:234-242,313-322) with ONE launch over a device-side problem table.
//
//   c[m, n] = epilogue( sum_k a[m, k] * b[n, k] ),   a, b fp8 (K contiguous), fp32 accumulation
//
// Work decomposition
//   * the output of every problem is cut into 256 x 256 tiles; all tiles of all problems form
//     one list walked by a persistent grid (one workgroup per CU).  The list is split into 8
//     contiguous ranges, one per XCD (workgroup i runs on XCD i % 8), so that workgroups that
//     share an L2 work on neighbouring tiles; inside a problem the m index runs fastest within
//     groups of 8 rows of tiles, so one round of an XCD's 32 workgroups is an 8 x 4 block of tiles.
//     All of that is decided on the host (gemm_schedule.h, fp8gmm_plan_grouped_gemm_launch): the kernel
//     reads its work list, one 64-byte record per tile, and does no scheduling arithmetic of its own
//     (binary searches over the problem table and integer divisions in the scalar unit cost a tile switch
//     thousands of cycles, more with every expert).
//     (Extents below are those of the default tile; the template's TILE = 128 form halves them all, see the
//     kernel.)
//   * a workgroup is 4 wavefronts (2 along m x 2 along n), one per SIMD; a wavefront owns a
//     128 x 128 sub-tile = 4 x 4 MFMA tiles of v_mfma_f32_32x32x64_f8f6f4.  Its 256 accumulators
//     live in the accumulation registers, the other 256 registers hold fragments and addresses.
//     The weight operand is MFMA source 0 and the token operand source 1: every lane then
//     holds 4 consecutive output columns of one row.
//
// Data movement
//   * operands go global -> LDS directly (`buffer_load_dwordx4 ... lds`), never through
//     registers.  Buffer descriptors bound every operand, so rows past m / n and K tails read
//     as zeros: m, n are arbitrary and k only has to be a multiple of 16.
//   * a main-loop step consumes K = 128: one 128-byte line of each of the tile's 256 token rows
//     and 256 weight rows.  LDS (all 160 KB) is a ring of five 32 KB units, a unit being the
//     256 rows x 128 B of ONE operand for one step, its eight 16-byte chunks XOR-swizzled with
//     (row >> 1) & 7 so that the 16-byte fragment reads of a wavefront are conflict-free.  Every
//     load instruction fetches 8 whole lines (two half-line requests for one line, issued apart,
//     meet in the L1 as a hit on a pending miss and stall it).
//   * at any time the ring holds the units of the step being computed, of the next step, and
//     the tokens of the step after; that step's weights replace the current tokens once the
//     step's barrier has shown that every wavefront has read them.  The token loads of step + 2
//     are issued during the low K half of a step, the weight loads during the high half, one
//     after every second MFMA.
//   * the load stream and the ring run CONTINUOUSLY across tile boundaries: while a tile's
//     epilogue stores its result, the next tile's first two steps are already in LDS.
//   * ONE s_barrier per step, between its two K = 64 halves.  The fragments of a half are read
//     from LDS during the half before it, interleaved with the MFMAs (pinned with sched_barrier).
//     With a single wavefront per SIMD nothing else fills an MFMA pipe, so whatever sits between
//     two MFMAs has to issue within the 64 cycles the first one runs: addresses are two
//     instructions per load, the load cursor advances without branches while it stays inside an
//     item, and the scheduler arithmetic of an item switch runs once per tile.
//   * epilogue: scale, convert, and - for interior bf16 tiles - a pass through the free ring unit
//     that turns the MFMA layout into whole-line stores.
#pragma once

#include <atomic>
#include <type_traits>
#include <utility>

#include "device_utils.h"
#include "tiling.h"

namespace fp8gmm {

// The result of a tile is written once and not read again by this launch: stored with the streaming hint, it does
// not push the operand slabs that neighbouring workgroups are about to re-read out of the L2, and the loads that
// follow the epilogue in the memory pipeline are not held up as long behind its stores (a dense 16384 x 14336 x
// 4096 launch: 1.14 -> 1.09 million cycles; without any stores it would be 1.06).
__device__ __forceinline__ void buf_store16_stream(u32x4 v, __amdgpu_buffer_rsrc_t r, uint32_t off) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)off, 0, 2);
}

// A buffer descriptor of a tile's result, made of values that are the same in every lane.  The compiler does not
// always know that: when it has moved the address arithmetic of a tile to the vector unit (it does, where scalar
// registers are short), a descriptor built from the outcome sits in vector registers, and every store through it
// becomes a loop that reads the four words back lane by lane - a dozen instructions and a branch per store, 32
// stores per wavefront and tile.  Reading the words back once, here, costs three instructions per tile.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_uniform_rsrc(const void* base, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uintptr_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return make_rsrc(reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo), __builtin_amdgcn_readfirstlane(bytes));
}

constexpr int kPartialBytes = FP8GMM_GEMM_SLOT_BYTES;  // one workspace slot: the fp32 accumulators of one tile
static_assert(kPartialBytes == BM * BN * 4, "a slot holds one tile of fp32 accumulators");

constexpr int BK = kGemmTileK;    // bytes of K per main-loop step: one 128-byte line of every operand row
constexpr int US = BM * BK;       // 32768 bytes per ring unit: the 256 rows of ONE operand for one step
constexpr int RING = 5;
static_assert(BM == BN, "token and weight units share one size");
constexpr int NWAVES = 4;         // one wavefront per SIMD: 256 accumulator + 256 other registers per lane
constexpr int NTHREADS = 64 * NWAVES;
constexpr int WM = 128, WN = 128;  // wavefront sub-tile
constexpr int WAVES_N = BN / WN;  // wavefronts along n: 2 (x 2 along m)
constexpr int MT = WM / 32;       // 4 MFMA tiles along m per wave
constexpr int NT = WN / 32;       // 4 MFMA tiles along n per wave
constexpr int kParts = US / 1024 / NWAVES;  // buffer_load ... lds instructions (1 KB each) per wavefront per unit: 8
constexpr int kFastStores = MT * 8;  // 16-byte stores per wavefront in the staged bf16 epilogue (8 per 32-row block)

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define FP8GMM_ALL_ACC_256 \
  "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", \
  "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", \
  "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", \
  "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63", \
  "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", \
  "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", \
  "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", \
  "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127", \
  "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", \
  "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", \
  "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", \
  "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", \
  "a192", "a193", "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", "a207", \
  "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", "a220", "a221", "a222", "a223", \
  "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", \
  "a240", "a241", "a242", "a243", "a244", "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255"
#define FP8GMM_ALL_ACC_64 \
  "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", \
  "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", \
  "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", \
  "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63"

#define FP8GMM_SB() __builtin_amdgcn_sched_barrier(0)
#define FP8GMM_WAIT_VM(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")
#define FP8GMM_WAIT_VM_LGKM(n) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(n) : "memory")
// global -> LDS: lane i's 16 bytes land at M0 + 16 i; out-of-range offsets deliver zeros
#define FP8GMM_DMA(lds_addr, voff, rsrc) \
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc))

// The accumulators of a lane are the accumulation registers a0 .. a255 (a0 .. a63 for the small tile), addressed BY
// NAME in every statement that touches them: MFMA tile (i, j) of a wavefront's sub-tile owns the 16 registers from
// 16 (NT i + j).  The compiler never sees them as values, so there is nothing for its register allocator to move,
// split or spill, whatever control flow surrounds the products (with the accumulators as ordinary values and all
// 512 registers of a lane in use, a second step body or products issued from inside the epilogue end in hundreds
// of spilled registers).  The statements are volatile and keep their order; what the compiler does not know it
// cannot protect, so: (1) nothing but these statements may use an accumulation register - every product names the
// whole file as clobbered, which keeps the compiler from parking spilled values there; (2) the waits the hardware
// needs between a product and a read of its result are this file's business: results are read tile by tile in the
// order the products were issued, never sooner than 16 products (a thousand cycles) after the last one into a tile.
template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

#define FP8GMM_ACC_READ(R) asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t[R]) : "n"(BASE + R))
#define FP8GMM_ACC_ZERO(R) asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(BASE + R))
#define FP8GMM_16_TIMES(X) X(0); X(1); X(2); X(3); X(4); X(5); X(6); X(7); X(8); X(9); X(10); X(11); X(12); X(13); X(14); X(15)
template <int BASE>
__device__ __forceinline__ f32x16 acc_tile() {   // one MFMA tile's accumulators as ordinary vector registers
  f32x16 t;
  FP8GMM_16_TIMES(FP8GMM_ACC_READ);
  return t;
}
template <int BASE>
__device__ __forceinline__ void acc_tile_clear() {
  FP8GMM_16_TIMES(FP8GMM_ACC_ZERO);
}
#undef FP8GMM_ACC_READ
#undef FP8GMM_ACC_ZERO
#undef FP8GMM_16_TIMES

// Per-problem scalars (scaling factors, the current amax) are read through the scalar unit: they are uniform,
// and a vector load would have to be waited for with vmcnt(0), i.e. together with every operand load the
// load stream has in flight for the next tile - thousands of cycles per tile when those come from HBM.
typedef __attribute__((address_space(4))) const float scalar_float;
__device__ __forceinline__ float load_scale(const float* p) {   // constant while the kernel runs; null means 1
  return p != nullptr ? *reinterpret_cast<scalar_float*>(reinterpret_cast<uintptr_t>(p)) : 1.f;
}
// The running maximum another workgroup may be raising at this moment: any value read is a lower bound of it.
__device__ __forceinline__ float peek_amax(const float* p) {
  float v;
  asm volatile("s_load_dword %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(p) : "memory");
  return v;
}
// amax only grows: once the slot holds a value at or above this wavefront's, the atomic is redundant
// (the slots of all experts share a cache line, and atomics on one line serialise)
__device__ __forceinline__ void merge_amax(float* slot, float wave_amax, int lane) {
  if (slot != nullptr && wave_amax > 0.f && !(peek_amax(slot) >= wave_amax) && lane == 0)
    atomic_max_nonneg(slot, wave_amax);
}

// Epilogue of one 256 x 256 tile whose accumulators are complete: scales, optional GELU, conversion,
// stores, amax.  Returns true when the staged bf16 path ran (exactly kFastStores stores per wavefront).
// `stage`: 32 KB of LDS that no wavefront reads or loads into until the barrier at the end of the staged path.
// `oob_zero`: accumulators of rows past m and columns past n are exactly zero (both operands row-major: what
// lies outside the tile's rows is outside the load descriptors); `oob_rows_zero`: those of rows past m are
// (operand a row-major).
//
// The staged paths store through a buffer descriptor that spans the tile's valid rows: rows past m fall outside
// it and are dropped by the hardware, lanes whose columns lie past n carry an offset beyond any descriptor.
// Edge tiles therefore run the same straight-line code as interior ones, with the same number of store
// instructions (a ragged expert's last row of tiles used to take a per-element path several times as slow,
// and the workgroups that drew those tiles set the duration of the launch).
constexpr uint32_t kMaskedOffset = 0x80000000u;  // + any row offset of a tile (< 2^30) stays out of range

// `s` = a_scale_inv * b_scale_inv and `cs` = c_scale of the problem, read by the caller ahead of time.
// TILE: 256 (the namespace's constants) or 128 (the small tile: 64 x 64 per wavefront, 16 KB of staging).
// `released(i, j)` (integral constants) is called right after MFMA tile (i, j) of the staged bf16 path has been read
// out of its accumulators: from there on they may receive the next tile's products.
// whether the plain bf16 epilogue through the staging area applies to this tile
template <int TILE>
__device__ __forceinline__ bool staged_bf16_tile(const fp8gmm_gemm_problem& pr, int m0, int n0, int out_kind,
                                                 int epilogue) {
  const int64_t ldc = pr.ldc;
  const bool interior = (m0 + TILE <= pr.m) && (n0 + TILE <= pr.n);
  const int cv = pr.n - n0 < TILE ? pr.n - n0 : TILE;
  const bool desc_ok = ((ldc & 7) == 0) && ldc < (1 << 21) && ((reinterpret_cast<uintptr_t>(pr.c) & 15) == 0);
  return out_kind == FP8GMM_OUT_BF16 && !(epilogue & (FP8GMM_EPI_GELU | FP8GMM_EPI_DGELU)) && desc_ok &&
         (interior || (cv & 7) == 0);
}
struct NothingReleased {
  template <class I, class J>
  __device__ __forceinline__ void operator()(I, J) const {}
};
// `mt`: 32-row blocks per wavefront: MT, or MT / 2 for a tile of half height, whose wavefronts stand on rows
// wave_m * 64 + 32 i.  Returns the number of stores per wavefront that the staged bf16 form left in flight (0: another form ran).
template <int TILE, class Released = NothingReleased>
__device__ __forceinline__ int tile_epilogue(const fp8gmm_gemm_problem& pr, int m0, int n0, int out_kind, int epilogue,
                                             uint8_t* stage, int mt, bool oob_zero, bool oob_rows_zero, float s, float cs,
                                             Released released = Released()) {
  constexpr int BM = TILE, BN = TILE, WN = TILE / 2, MT = TILE / 64, NT = WN / 32;
  const int WM = mt * 32;   // rows of a wavefront's sub-tile
  constexpr int kStageBytes = TILE * 32;   // per wavefront: a quarter of one ring unit
  // The lane's offsets into the staging area and the result are formed anew for every tile: computed once per
  // kernel (they do not depend on the tile) they would occupy a dozen registers all through the main loop, where
  // there are none to spare.
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int l32 = lane & 31, khalf = lane >> 5;
  const int M = pr.m, N = pr.n;
  int fast = 0;
    const bool gelu = (epilogue & FP8GMM_EPI_GELU) != 0;
    const bool dgelu_in = (epilogue & FP8GMM_EPI_DGELU) != 0 && pr.aux != nullptr;   // aux is then an INPUT
    const int64_t ldc = pr.ldc;
    float amax = 0.f;
    const bool interior = (m0 + BM <= M) && (n0 + BN <= N);
    const int rv = M - m0 < BM ? M - m0 : BM;   // valid rows and columns of this tile
    const int cv = N - n0 < BN ? N - n0 : BN;
    // 16-byte pieces of the tile's rows can be addressed with 32-bit offsets below 2^30
    const bool desc_ok = ((ldc & 7) == 0) && ldc < (1 << 21) && ((reinterpret_cast<uintptr_t>(pr.c) & 15) == 0);
    if (staged_bf16_tile<TILE>(pr, m0, n0, out_kind, epilogue)) {
      // Plain bf16 output: straight-line code with an exact store count.
      // Through LDS, so that a store instruction writes whole lines.  In the MFMA layout a lane holds 4
      // consecutive columns of one row, and a 16-byte store per lane touches 32 rows: 64 separate 32-byte
      // pieces per instruction, which the memory pipeline takes one by one.  Each wavefront stages its sub-tile
      // in units of 32 rows x 64 columns (32 x 128 B; the 16-byte chunk c of row r sits at chunk
      // c ^ ((r >> 1) & 7)) and reads a unit back row-major: 8 rows x 128 contiguous bytes per store instruction.
      // Two 4 KB staging buffers alternate, so that the read-back of one unit is under way while the next unit is
      // converted: the round trip through LDS, a third of the epilogue when exposed, hides behind the arithmetic.
      uint16_t* const C = static_cast<uint16_t*>(pr.c) + (int64_t)m0 * ldc + n0;
      const __amdgpu_buffer_rsrc_t rc = make_uniform_rsrc(C, (uint32_t)(((rv - 1) * (int)ldc + cv) * 2));
      // (the small tile's staging area holds one unit per wavefront: a wavefront's LDS operations complete in
      // order, so the read-back of a unit is done before the next unit's writes land in the same place)
      uint8_t* mine = stage + wave * kStageBytes;
      constexpr int kUnitsPerRow = NT / 2;               // units of 64 columns per 32-row block of the sub-tile
      const int wr = l32 * 128 + khalf * 8;              // + ((4 jl + g) ^ ((l32 >> 1) & 7)) * 16, jl = j & 1
      const int rrow = lane >> 3, rchunk = lane & 7;      // read-back: row 8 it + rrow, chunk rchunk
      u32x4 v[4];
      auto store_unit = [&](int i, int jj) {
        const int col = wave_n * WN + jj * 64 + rchunk * 8;
        const uint32_t lane_off = col < cv ? (uint32_t)((rrow * (int)ldc + col) * 2) : kMaskedOffset;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const uint32_t row_off = (uint32_t)((wave_m * WM + i * 32 + 8 * it) * (int)ldc * 2);  // uniform
          buf_store16_stream(v[it], rc, lane_off + row_off);
        }
      };
      static_for<MT * kUnitsPerRow>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        constexpr int i = u / kUnitsPerRow, jj = u % kUnitsPerRow;
        if (i >= mt) return;
        uint8_t* buf = mine + (kStageBytes >= 8192 ? (u & 1) * 4096 : 0);
        static_for<2>([&](auto jlc) {
          constexpr int jl = decltype(jlc)::value;
          const f32x16 t = acc_tile<16 * (NT * i + 2 * jj + jl)>();
          released(std::integral_constant<int, i>{}, std::integral_constant<int, 2 * jj + jl>{});
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const u32x2 o = {pack_bf16x2(t[4 * g + 0] * s, t[4 * g + 1] * s),
                             pack_bf16x2(t[4 * g + 2] * s, t[4 * g + 3] * s)};
            *reinterpret_cast<u32x2*>(buf + wr + (((4 * jl + g) ^ ((l32 >> 1) & 7)) << 4)) = o;
          }
        });
        // the previous unit's read-back was issued before this unit's conversion: store it now
        if (u > 0) store_unit((u - 1) / kUnitsPerRow, (u - 1) % kUnitsPerRow);
        // only this wavefront touches `mine`, and its LDS operations complete in order
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int r = 8 * it + rrow;
          v[it] = *reinterpret_cast<const u32x4*>(buf + r * 128 + ((rchunk ^ ((r >> 1) & 7)) << 4));
        }
      });
      store_unit(mt - 1, kUnitsPerRow - 1);
      __builtin_amdgcn_s_barrier();  // the staging area goes back to the operand ring
      fast = mt * kUnitsPerRow * 4;
    } else if (TILE == 256 && out_kind == FP8GMM_E4M3 && gelu && pr.aux != nullptr && desc_ok && ((ldc & 15) == 0) &&
               ((reinterpret_cast<uintptr_t>(pr.aux) & 15) == 0) && (interior || (oob_zero && (cv & 15) == 0))) {
      // The fused GELU form (e4m3 gelu(v) * c_scale, bf16 v on the side, amax of gelu(v)): both outputs go
      // through the staging area like the plain form's, one 32-row block at a time, in ONE pass over the
      // accumulators: the bf16 values are staged as they are formed (32 rows x 256 B), the fp8 bytes of the
      // block wait in 16 registers until the bf16 block has been read back, then take its place (32 rows x 128 B,
      // chunk c of row r at chunk c ^ ((r >> 1) & 7)).  Every store instruction writes whole lines: 12 per
      // block instead of 32 that touch 32 rows each.  On an edge tile the accumulators outside the problem are
      // zero (oob_zero), and gelu(0) = 0 leaves the amax alone.
      uint8_t* const C = static_cast<uint8_t*>(pr.c) + (int64_t)m0 * ldc + n0;
      uint16_t* const AUX = static_cast<uint16_t*>(pr.aux) + (int64_t)m0 * ldc + n0;
      const __amdgpu_buffer_rsrc_t rc = make_uniform_rsrc(C, (uint32_t)((rv - 1) * (int)ldc + cv));
      const __amdgpu_buffer_rsrc_t ra = make_uniform_rsrc(AUX, (uint32_t)(((rv - 1) * (int)ldc + cv) * 2));
      uint8_t* mine = stage + wave * 8192;
      const int wr = l32 * 256 + khalf * 8;   // bf16 block: + ((4 j + g) ^ (l32 & 15)) * 16
      const int wr8 = l32 * 128 + khalf * 4;  // fp8 block:  + ((2 j + g / 2) ^ ((l32 >> 1) & 7)) * 16 + (g & 1) * 8
      const int rrow = lane >> 4, rchunk = lane & 15;
      const int rrow8 = lane >> 3, rchunk8 = lane & 7;
      const int col = wave_n * WN + rchunk * 8, col8 = wave_n * WN + rchunk8 * 16;
      const uint32_t lane_off = col < cv ? (uint32_t)((rrow * (int)ldc + col) * 2) : kMaskedOffset;
      const uint32_t lane_off8 = col8 < cv ? (uint32_t)(rrow8 * (int)ldc + col8) : kMaskedOffset;
      float tile_amax = 0.f;
      static_for<MT>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (i >= mt) return;
        uint32_t f8[NT][4];
        bool any_nan = false;
        static_for<NT>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          const f32x16 t = acc_tile<16 * (NT * i + j)>();
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            float v[4], x[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = t[g * 4 + q] * s;
            const u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2*>(mine + wr + (((4 * j + g) ^ (l32 & 15)) << 4)) = a;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float r = gelu_tanh_fast(v[q]);
              // A chain of hardware max operations, pinned: written as compare + select, the compiler rebuilds
              // the 256-element reduction as a tree and keeps far more values alive than there are registers.
              // r is computed, hence never a signalling NaN, and a quiet NaN loses against the running maximum.
              asm volatile("v_max_f32 %0, %0, |%1|" : "+v"(tile_amax) : "v"(r));
              const float y = r * cs;
              any_nan |= (y != y);   // rare: dealt with once per block, below (the median turns a NaN into -max)
              x[q] = __builtin_amdgcn_fmed3f(y, -448.0f, 448.0f);
            }
            f8[j][g] = __builtin_amdgcn_cvt_pk_fp8_f32(x[2], x[3],
                                                       __builtin_amdgcn_cvt_pk_fp8_f32(x[0], x[1], 0u, false), true);
          }
        });
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(any_nan) != 0, 0)) {
          // some lane of this block saw a NaN: form the block's bytes again, with 0x7F in place of every NaN
          static_for<NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const f32x16 t = acc_tile<16 * (NT * i + j)>();
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              uint32_t nan_bytes = 0;
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const float y = gelu_tanh_fast(t[g * 4 + q] * s) * cs;
                nan_bytes |= (y != y) ? (0xffu << (8 * q)) : 0u;
              }
              f8[j][g] = (f8[j][g] & ~nan_bytes) | (0x7f7f7f7fu & nan_bytes);
            }
          });
        }
        {
          u32x4 rb[8];
#pragma unroll
          for (int it = 0; it < 8; ++it) {
            const int r = 4 * it + rrow;
            rb[it] = *reinterpret_cast<const u32x4*>(mine + r * 256 + ((rchunk ^ (r & 15)) << 4));
          }
#pragma unroll
          for (int it = 0; it < 8; ++it) {
            const uint32_t row_off = (uint32_t)((wave_m * WM + i * 32 + 4 * it) * (int)ldc * 2);
            buf_store16_stream(rb[it], ra, lane_off + row_off);
          }
        }
        // the wavefront's LDS operations complete in order: the reads above are done before these writes land
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            *reinterpret_cast<uint32_t*>(mine + wr8 + (((2 * j + (g >> 1)) ^ ((l32 >> 1) & 7)) << 4) + (g & 1) * 8) =
                f8[j][g];
        {
          u32x4 rb[4];
#pragma unroll
          for (int it = 0; it < 4; ++it) {
            const int r = 8 * it + rrow8;
            rb[it] = *reinterpret_cast<const u32x4*>(mine + r * 128 + ((rchunk8 ^ ((r >> 1) & 7)) << 4));
          }
#pragma unroll
          for (int it = 0; it < 4; ++it) {
            const uint32_t row_off = (uint32_t)((wave_m * WM + i * 32 + 8 * it) * (int)ldc);
            // plain stores, unlike the bf16 copy above: the fp8 activation is the next launch's operand, and what the
            // memory-side cache keeps of it that launch does not fetch from HBM (config 4: this launch -8 us, the
            // weight gradients that read it -4 us each)
            __builtin_amdgcn_raw_buffer_store_b128(rb[it], rc, (int)(lane_off8 + row_off), 0, 0);
          }
        }
      });
      __builtin_amdgcn_s_barrier();  // the staging area goes back to the operand ring
      merge_amax(pr.c_amax, wave_max(tile_amax), lane);
    } else if (TILE == 256 && out_kind != FP8GMM_OUT_BF16 && dgelu_in && desc_ok && ((ldc & 15) == 0) &&
               ((reinterpret_cast<uintptr_t>(pr.aux) & 7) == 0) && n0 + BN <= N && (interior || oob_rows_zero)) {
      // The data gradient with the GELU's derivative folded in: x = v * dgelu(pre), fp8(x * c_scale), amax of x.
      // `pre` (bf16, the layout of c) is read in the MFMA layout, 8 bytes per lane and piece, one 32-row block
      // ahead of the arithmetic; the fp8 bytes of a block go through the staging area (32 rows x 128 B, chunk c of
      // row r at chunk c ^ ((r >> 1) & 7)) so that every store instruction writes whole lines.  Rows past m hold
      // zero accumulators (oob_rows_zero) and read pre = 0 through the descriptor: x = 0 there, the amax is left
      // alone and the stores fall outside the result's descriptor.
      uint8_t* const C = static_cast<uint8_t*>(pr.c) + (int64_t)m0 * ldc + n0;
      const uint16_t* const PRE = static_cast<const uint16_t*>(pr.aux) + (int64_t)m0 * ldc + n0;
      const __amdgpu_buffer_rsrc_t rc = make_uniform_rsrc(C, (uint32_t)((rv - 1) * (int)ldc + cv));
      const __amdgpu_buffer_rsrc_t rp = make_uniform_rsrc(PRE, (uint32_t)(((rv - 1) * (int)ldc + cv) * 2));
      uint8_t* mine = stage + wave * 8192;
      const int wr8 = l32 * 128 + khalf * 4;  // + ((2 j + g / 2) ^ ((l32 >> 1) & 7)) * 16 + (g & 1) * 8
      const int rrow8 = lane >> 3, rchunk8 = lane & 7;
      const uint32_t lane_off8 = (uint32_t)(rrow8 * (int)ldc + wave_n * WN + rchunk8 * 16);
      const uint32_t pre_lane = (uint32_t)(((wave_m * WM + l32) * (int)ldc + wave_n * WN + khalf * 4) * 2);
      float tile_amax = 0.f;
      u32x2 pre[2][NT * 4];
      auto fetch = [&](int i, u32x2 (&dst)[NT * 4]) {
        const uint32_t row_off = (uint32_t)(i * 32 * (int)ldc * 2);
#pragma unroll
        for (int jg = 0; jg < NT * 4; ++jg) dst[jg] = buf_load8_stream(rp, pre_lane + row_off + (uint32_t)(jg * 16));
      };
      fetch(0, pre[0]);
      static_for<MT>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (i >= mt) return;
        if constexpr (i + 1 < MT) {
          if (i + 1 < mt) fetch(i + 1, pre[(i + 1) & 1]);
        }
        uint32_t f8[NT][4];
        static_for<NT>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          const f32x16 t = acc_tile<16 * (NT * i + j)>();
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const u32x2 pw = pre[i & 1][j * 4 + g];
            float x[4];
            x[0] = (t[g * 4 + 0] * s) * dgelu(bf16_lo_to_f32(pw.x));
            x[1] = (t[g * 4 + 1] * s) * dgelu(bf16_hi_to_f32(pw.x));
            x[2] = (t[g * 4 + 2] * s) * dgelu(bf16_lo_to_f32(pw.y));
            x[3] = (t[g * 4 + 3] * s) * dgelu(bf16_hi_to_f32(pw.y));
            // a pinned chain of hardware max operations, as in the GELU form: x is computed, hence never a
            // signalling NaN, and a quiet NaN loses against the running maximum
#pragma unroll
            for (int q = 0; q < 4; ++q) asm volatile("v_max_f32 %0, %0, |%1|" : "+v"(tile_amax) : "v"(x[q]));
            f8[j][g] = out_kind == FP8GMM_E4M3 ? cvt4_fp8<FP8GMM_E4M3>(x[0] * cs, x[1] * cs, x[2] * cs, x[3] * cs)
                                               : cvt4_fp8<FP8GMM_E5M2>(x[0] * cs, x[1] * cs, x[2] * cs, x[3] * cs);
          }
        });
        // only this wavefront touches `mine`, and its LDS operations complete in order
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            *reinterpret_cast<uint32_t*>(mine + wr8 + (((2 * j + (g >> 1)) ^ ((l32 >> 1) & 7)) << 4) + (g & 1) * 8) =
                f8[j][g];
        u32x4 rb[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int r = 8 * it + rrow8;
          rb[it] = *reinterpret_cast<const u32x4*>(mine + r * 128 + ((rchunk8 ^ ((r >> 1) & 7)) << 4));
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const uint32_t row_off = (uint32_t)((wave_m * WM + i * 32 + 8 * it) * (int)ldc);
          buf_store16_stream(rb[it], rc, lane_off8 + row_off);
        }
      });
      __builtin_amdgcn_s_barrier();  // the staging area goes back to the operand ring
      merge_amax(pr.c_amax, wave_max(tile_amax), lane);
    } else if (out_kind == FP8GMM_OUT_BF16) {
      uint16_t* __restrict__ C = static_cast<uint16_t*>(pr.c);
      uint16_t* __restrict__ AUX = static_cast<uint16_t*>(pr.aux);
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0) &&
                       (AUX == nullptr || (reinterpret_cast<uintptr_t>(AUX) & 7) == 0);
      static_for<MT>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (i >= mt) return;
        const int m = m0 + wave_m * WM + i * 32 + l32;
        static_for<NT>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          const f32x16 t = acc_tile<16 * (NT * i + j)>();
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n0 + wave_n * WN + j * 32 + g * 8 + khalf * 4;
            if (m >= M || n >= N) continue;
            float v[4], r[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              v[q] = t[g * 4 + q] * s;
              r[q] = gelu ? gelu_tanh_fast(v[q]) : v[q];
            }
            const int64_t off = (int64_t)m * ldc + n;
            if (dgelu_in) {
#pragma unroll
              for (int q = 0; q < 4; ++q)
                if (n + q < N) r[q] = v[q] * dgelu(bf16_to_f32(AUX[off + q]));
            }
            if (vec && n + 3 < N) {
              u32x2 o = {pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
              global_store(C + off, o);
              if (gelu && AUX != nullptr) {
                u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                global_store(AUX + off, a);
              }
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (n + q < N) {
                  global_store(C + off + q, (uint16_t)f32_to_bf16_bits(r[q]));
                  if (gelu && AUX != nullptr) global_store(AUX + off + q, (uint16_t)f32_to_bf16_bits(v[q]));
                }
              }
            }
          }
        });
      });
    } else {
      uint8_t* __restrict__ C = static_cast<uint8_t*>(pr.c);
      uint16_t* __restrict__ AUX = static_cast<uint16_t*>(pr.aux);
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 3) == 0) &&
                       (AUX == nullptr || (reinterpret_cast<uintptr_t>(AUX) & 7) == 0);
      static_for<MT>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (i >= mt) return;
        const int m = m0 + wave_m * WM + i * 32 + l32;
        static_for<NT>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          const f32x16 t = acc_tile<16 * (NT * i + j)>();
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n0 + wave_n * WN + j * 32 + g * 8 + khalf * 4;
            if (m >= M || n >= N) continue;
            float v[4], r[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              v[q] = t[g * 4 + q] * s;
              r[q] = gelu ? gelu_tanh_fast(v[q]) : v[q];
              if (dgelu_in && n + q < N) r[q] = v[q] * dgelu(bf16_to_f32(AUX[(int64_t)m * ldc + n + q]));
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
              global_store(C + off, w);
              if (gelu && AUX != nullptr) {
                u32x2 a = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                global_store(AUX + off, a);
              }
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (n + q < N) {
                  global_store(C + off + q, (uint8_t)(w >> (8 * q)));
                  if (gelu && AUX != nullptr) global_store(AUX + off + q, (uint16_t)f32_to_bf16_bits(v[q]));
                }
              }
            }
          }
        });
      });
      merge_amax(pr.c_amax, wave_max(amax), lane);
    }
    return fast;
}

// Accumulators <-> workspace slot.  Register group r4 = (i * NT + j) * 4 + g of lane t sits at
// (r4 * NTHREADS + t) * 16 bytes: every wavefront instruction moves 1 KB of contiguous memory.
// Written here and read by the fix-up launch with the streaming hint: partial sums are used once, and as ordinary
// traffic they took the place of operands in the memory-side cache that later launches of the step would have
// found there (config 3: 19 MB of them after the forward GEMM made the weight gradient, two launches later, 40 us
// slower; the same 19 MB written and read by any other kernel did the same).
template <int TILE>
__device__ __forceinline__ void partial_store(uint8_t* slot) {
  constexpr int MT = TILE / 64, NT = TILE / 64;
  float* base = reinterpret_cast<float*>(slot) + threadIdx.x * 4;
  static_for<MT * NT>([&](auto tc) {
    constexpr int ij = decltype(tc)::value;
    const f32x16 t = acc_tile<16 * ij>();
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 v = {t[4 * g + 0], t[4 * g + 1], t[4 * g + 2], t[4 * g + 3]};
      global_store_stream(base + (ij * 4 + g) * (NTHREADS * 4), v);
    }
  });
}
// The half of a work-list record (fp8gmm_gemm_item) that a side of the kernel needs, as scalar loads.
struct ItemLoad {   // bytes 0..31: what the load stream needs besides ItemTile
  uint64_t a, b;
  uint32_t a_bytes, b_bytes;
  int32_t lda, ldb;
};
struct ItemTile {   // bytes 32..63
  int32_t k, k_begin, nk, m0, n0, prob, slot, flags;
};
static_assert(sizeof(fp8gmm_gemm_item) == 64 && sizeof(ItemLoad) == 32 && sizeof(ItemTile) == 32, "record layout");
static_assert(offsetof(fp8gmm_gemm_item, k) == 32 && offsetof(fp8gmm_gemm_item, lda) == 24, "record layout");

// B_TR: operand b is stored contraction-major, b[k][n] with n contiguous and pitch ldb (the layout of a weight
// stack [N_out.., ] seen from the data-gradient GEMM), instead of b[n][k].  Its ring unit then holds 128
// contraction rows of 256 bytes; the 16-byte chunk c of row r sits at chunk c ^ 2 (r mod 8), and a fragment is
// gathered with four transposing reads (ds_read_b64_tr_b8: in a group of 16 lanes, lane 8 h + i receives byte i
// of the 8 bytes addressed by lanes 2 b + h, b = 0..7).  Everything else - schedule, MFMA order, epilogue -
// is shared, so both layouts produce the same bits.
// A_TR: the same for operand a (a[k][m], pitch lda): with both, c = a^T . b contracts over the rows of two
// row-major matrices, which is the weight-gradient GEMM on the un-transposed activations and gradients; rows
// past k read as zeros, so the contraction length needs no padding.
// TILE = 128: the small tile.  Same structure with every extent halved: 128 x 128 per workgroup, 64 x 64 = 2 x 2 MFMA
// tiles per wavefront, 16 KB ring units, 80 KB of LDS and at most 256 registers per lane, so that TWO workgroups
// share a compute unit.  It pays where the large tile leaves the machine idle: launches with fewer large tiles
// than compute units (four times as many small ones), and problems of up to 128 rows, half of whose large tiles
// would be padding - 1.1 to 1.7 times faster there.  It moves twice the operand bytes from L2 per flop: at the
// MFMA's pace that is 64 B per clock and compute unit, the L2's peak, so on launches that fill the machine with
// full tiles it is 10 - 20 % slower however short the contraction.  Which tile a launch takes is decided when it
// is planned (FP8GMM_GEMM_TILE_128); the results are the same bits either way.  No sharing along K and no fused
// GELU epilogue in this form.
template <int A_FMT, int B_FMT, bool A_TR, bool B_TR, int TILE>
__global__ __launch_bounds__(NTHREADS, TILE == 256 ? 1 : 2) void grouped_gemm_kernel(
    const fp8gmm_gemm_problem* __restrict__ probs, const fp8gmm_gemm_item* __restrict__ items, int out_kind,
    int epilogue, uint8_t* __restrict__ workspace, const fp8gmm_tensor_desc* __restrict__ merge_descs, int merge_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  // the amax merge of the cast launch in front of this one, where the pass planner has moved it here
  if (merge_n > 0 && blockIdx.x == 0) merge_amax_partials(merge_descs, merge_n, threadIdx.x, NTHREADS);
  // the tile's extents shadow the namespace's (which are those of the 256 x 256 tile)
  [[maybe_unused]] constexpr int BM = TILE;
  constexpr int BN = TILE, US = TILE * BK, WM = TILE / 2, WN = TILE / 2, MT = WM / 32, NT = WN / 32;
  constexpr int kParts = US / 1024 / NWAVES;        // 8 or 4 load instructions per wavefront and unit
  constexpr int kFastStores = MT * (NT / 2) * 4;    // stores per wavefront in the staged bf16 epilogue
  static_assert(TILE == 256 || TILE == 128, "tile sizes with a step sequence below");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: what depends on it stays in scalar registers
  const int wave_m = wave / WAVES_N;  // 0..1
  const int wave_n = wave % WAVES_N;  // 0..1
  const int l32 = lane & 31;
  const int khalf = lane >> 5;   // which 32-byte half of the 64-byte MFMA K slice this lane feeds
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);

  // DMA lane map, row-major operand: one wavefront instruction fills 8 rows x 128 B of a unit, i.e. whole
  // cache lines: lane -> row lane >> 3 of the group, slot chunk lane & 7.  Chunk c of row r is kept at chunk
  // c ^ ((r >> 1) & 7); for the rows of group wave + NWAVES j that is ((wave & 1) * 4 + (lane >> 4)) & 7, so the
  // GLOBAL chunk that has to land in slot chunk lane & 7 is a per-lane constant.
  const int drow = lane >> 3;
  const int dchunk = (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
  // fragment read map: token rows wave_m * 128 + 32 i + l32 (source 1), weight rows wave_n * 128 + 32 j + l32
  // (source 0); K half hh, lane half khalf -> chunks 4 hh + 2 khalf + {0, 1}; (row >> 1) & 7 = (l32 >> 1) & 7
  const int fsw = (l32 >> 1) & 7;
  int fc[2][2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int q = 0; q < 2; ++q) fc[hh][q] = ((4 * hh + 2 * khalf + q) ^ fsw) << 4;
  const int fa_off = (wave_m * WM + l32) * BK;
  const int fb_off = (wave_n * WN + l32) * BK;
  // contraction-major unit: 128 contraction rows x 256 B.  Fragment of K half hh: rows 64 hh + 32 khalf + b (+ 8 t
  // per read), logical chunk wave_n * 8 + 2 j + g, byte 8 h; s = lane % 16 = 2 b + h
  // (small tile: 128 contraction rows x 128 B, 8 chunks per row; rows r and r + 2 share their banks, and chunk c
  // of row r sits at chunk c ^ (r & 6))
  const int tr_b = (lane & 15) >> 1, tr_h = lane & 1, tr_g = (lane >> 4) & 1;
  constexpr int kTrPitch = BN;                         // bytes per contraction row of a unit
  const int tr_swz = TILE == 256 ? 2 * tr_b : (tr_b & 6);
  const int tr_row = (32 * khalf + tr_b) * kTrPitch + 8 * tr_h;
  int fbt_off[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) fbt_off[j] = tr_row + (((wave_n * (WN / 16) + 2 * j + tr_g) ^ tr_swz) << 4);
  int fat_off[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) fat_off[i] = tr_row + (((wave_m * (WM / 16) + 2 * i + tr_g) ^ tr_swz) << 4);
  // Tiles of half height (FP8GMM_ITEM_HALF_HEIGHT: at most 128 valid rows): the wavefronts stand two by two on
  // rows wave_m * 64 + 32 i, i < 2, and issue half the products.  Row-major tokens: the fragment addresses move
  // down by wave_m * 64 rows, a uniform amount that goes into the unit's base address (half_rows_back).
  // Contraction-major: the 16-byte chunk of fragment i is chunk wave_m * 4 + 2 i + tr_g (fat_half).
  [[maybe_unused]] const int half_rows_back = wave_m * 64 * BK;
  [[maybe_unused]] int fat_half[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
    fat_half[i] = tr_row + (((wave_m * (WM / 32) + 2 * (i & 1) + tr_g) ^ tr_swz) << 4);

  // ---- this workgroup's work list (uniform): records blockIdx.x, blockIdx.x + grid, ... up to the end record.
  // Both sides of the kernel walk it, the load side ahead of the compute side, and both read a record one item
  // before they need it, so that a tile switch never waits for memory.
  const uint8_t* const my_items = reinterpret_cast<const uint8_t*>(items + blockIdx.x);
  const size_t item_stride = (size_t)gridDim.x * sizeof(fp8gmm_gemm_item);
  auto item_load = [&](int r) { return *reinterpret_cast<const ItemLoad*>(my_items + r * item_stride); };
  auto item_tile = [&](int r) { return *reinterpret_cast<const ItemTile*>(my_items + r * item_stride + 32); };
  int r_ld = 0;                         // record the load side is in
  ItemLoad ld_next_l = item_load(0);    // ... and the record it takes next, fetched ahead
  ItemTile ld_next_t = item_tile(0);
  if (ld_next_t.prob < 0) return;

  // ---- load side: runs two steps ahead of the compute side, possibly in the next tile ----
  bool ld_live = true;  // the load cursor still points at an item
  int ld_kt = 0, ld_nk = 0, ld_kmax = 0;
  [[maybe_unused]] int ld_lda = 0, ld_ldb = 0;  // contraction-major operands only
  i32x4 rsrc_a = {0, 0, 0, 0x00020000}, rsrc_b = {0, 0, 0, 0x00020000};  // raw buffers; empty until set up
  // Addresses of the K = 128 step the load cursor points at: part j of an operand is fetched from a_k + j * a_step
  // (byte offsets into the operand's buffer, a_step uniform).  Rows past m / n are not masked: whatever they
  // deliver only reaches accumulators of rows / columns that the epilogue never stores, and the descriptor keeps
  // the access inside the operand.  The K tail is: a row-major lane whose 16-byte chunk lies past k gets an
  // out-of-range offset (zero fill); contraction rows past k are out of the descriptor's range by themselves.
  uint32_t a_base = 0, b_base = 0, a_step = 0, b_step = 0, a_k = 0, b_k = 0;
  bool k_ok = false;  // row-major operands: this lane's chunk of the step exists
  auto step_setup = [&]() {
    const uint32_t k0 = (uint32_t)ld_kt * BK;
    if constexpr (A_TR) {
      a_k = a_base + k0 * (uint32_t)ld_lda;  // k * pitch < 2^32 is checked when the table is planned
    } else {
      a_k = a_base + k0;
    }
    if constexpr (B_TR) {
      b_k = b_base + k0 * (uint32_t)ld_ldb;
    } else {
      b_k = b_base + k0;
    }
    k_ok = (int)k0 < ld_kmax;
  };
  // row-major operand: part j = rows (wave + NWAVES j) * 8 + drow of the tile.
  // contraction-major operand: one instruction fills 4 contraction rows x 256 B: part j = rows
  // (wave + NWAVES j) * 4 + lane / 16 of the unit, slot chunk lane % 16, which must receive global chunk
  // p ^ 2 (row mod 8); row mod 8 is the same for every j.
  // A record's operand addresses are those of the tile's first row / column, so these offsets depend on the
  // pitch alone.
  // (small tile: one instruction fills 8 contraction rows x 128 B; part j = rows (wave + NWAVES j) * 8 + lane / 8)
  constexpr int kTrRows = 1024 / kTrPitch;             // contraction rows per load instruction: 4 or 8
  const int krow = wave * kTrRows + lane / (kTrPitch / 16);
  const int tr_col = TILE == 256 ? ((lane & 15) ^ (2 * (krow & 7))) << 4 : ((lane & 7) ^ (krow & 6)) << 4;
  // Takes the record fetched ahead (r_ld), fetches the one after it, and sets up descriptors and offsets.
  auto load_setup = [&]() {
    for (;;) {
      const ItemLoad gl = ld_next_l;
      const ItemTile gt = ld_next_t;
      ld_live = gt.prob >= 0;
      if (!ld_live) break;
      ld_next_l = item_load(r_ld + 1);  // every list ends with an end record, so r_ld + 1 exists
      ld_next_t = item_tile(r_ld + 1);
      if (gt.nk > 0) {
        rsrc_a[0] = (int)(uint32_t)gl.a;
        rsrc_a[1] = (int)(uint32_t)(gl.a >> 32);
        rsrc_a[2] = (int)gl.a_bytes;
        rsrc_b[0] = (int)(uint32_t)gl.b;
        rsrc_b[1] = (int)(uint32_t)(gl.b >> 32);
        rsrc_b[2] = (int)gl.b_bytes;
        if constexpr (!A_TR) {
          a_base = (uint32_t)(wave * 8 + drow) * (uint32_t)gl.lda + dchunk * 16;
          a_step = NWAVES * 8 * (uint32_t)gl.lda;
        } else {
          a_base = (uint32_t)krow * (uint32_t)gl.lda + (uint32_t)tr_col;
          a_step = NWAVES * kTrRows * (uint32_t)gl.lda;
          ld_lda = gl.lda;
        }
        if constexpr (!B_TR) {
          b_base = (uint32_t)(wave * 8 + drow) * (uint32_t)gl.ldb + dchunk * 16;
          b_step = NWAVES * 8 * (uint32_t)gl.ldb;
        } else {
          b_base = (uint32_t)krow * (uint32_t)gl.ldb + (uint32_t)tr_col;
          b_step = NWAVES * kTrRows * (uint32_t)gl.ldb;
          ld_ldb = gl.ldb;
        }
        ld_kmax = gt.k - dchunk * 16;  // this lane's chunk exists iff k0 < ld_kmax
        ld_kt = gt.k_begin;
        ld_nk = gt.k_begin + gt.nk;
        step_setup();
        return;
      }
      ++r_ld;  // an item without K work needs no loads
    }
    // Past the end of the stream the loads are issued all the same, against empty descriptors (zero fill),
    // which keeps the vmcnt arithmetic uniform.
    rsrc_a[2] = 0;
    rsrc_b[2] = 0;
  };
  // One instruction of that step: part j (0..7) of the token operand into ring unit `unit`, or of the weights.
  auto dma_a = [&](int unit, int j) {
    uint32_t v = a_k + j * a_step;
    if constexpr (!A_TR) v = k_ok ? v : 0xffffffffu;
    const uint32_t l = lds_base + unit * US + (wave + NWAVES * j) * 1024;
    FP8GMM_DMA(l, v, rsrc_a);
  };
  auto dma_b = [&](int unit, int j) {
    uint32_t v = b_k + j * b_step;
    if constexpr (!B_TR) v = k_ok ? v : 0xffffffffu;
    const uint32_t l = lds_base + unit * US + (wave + NWAVES * j) * 1024;
    FP8GMM_DMA(l, v, rsrc_b);
  };
  auto dma_advance = [&]() {
    if (!ld_live) return;
    if (++ld_kt == ld_nk) {
      ++r_ld;
      load_setup();
    } else {
      step_setup();
    }
  };
  auto ring_inc = [](int x) { return x + 1 == RING ? 0 : x + 1; };

  i32x8 fa0[MT], fb0[NT], fa1[MT], fb1[NT];  // fragment double buffer: low / high K half of a step
  auto read_frag = [&](i32x8& f, const uint8_t* base, int hh) {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(base + fc[hh][0]);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(base + fc[hh][1]);
    f = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };

  typedef int i32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
  auto read_frag_tr = [&](i32x8& f, uint32_t a) {  // 4 x 8 contraction rows of the lane's column
    const i32x2 t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a));
    const i32x2 t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + 8 * kTrPitch));
    const i32x2 t2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + 16 * kTrPitch));
    const i32x2 t3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + 24 * kTrPitch));
    f = i32x8{t0.x, t0.y, t1.x, t1.y, t2.x, t2.y, t3.x, t3.y};
  };
  // Half h of such a fragment (two of its four reads): lets a step spread the reads of a fragment over two MFMAs.
  auto read_half_tr = [&](i32x8& f, uint32_t a, int h) {
    const i32x2 t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + (16 * h) * kTrPitch));
    const i32x2 t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + (16 * h + 8) * kTrPitch));
    f[4 * h + 0] = t0.x;
    f[4 * h + 1] = t0.y;
    f[4 * h + 2] = t1.x;
    f[4 * h + 3] = t1.y;
  };
  auto read_half = [&](i32x8& f, const uint8_t* base, int hh, int h) {   // row-major: one of the two 16-byte reads
    const u32x4 t = *reinterpret_cast<const u32x4*>(base + fc[hh][h]);
    f[4 * h + 0] = (int)t.x;
    f[4 * h + 1] = (int)t.y;
    f[4 * h + 2] = (int)t.z;
    f[4 * h + 3] = (int)t.w;
  };
  [[maybe_unused]] auto half_b = [&](i32x8& f, const uint8_t* unit, int j, int hh, int h) {
    if constexpr (!B_TR) {
      read_half(f, unit + fb_off + j * 32 * BK, hh, h);
    } else {
      read_half_tr(f, (uint32_t)(uintptr_t)unit + fbt_off[j] + hh * (64 * kTrPitch), h);
    }
  };
  // (token fragments: `half` = the tile they are read for is of half height)
  [[maybe_unused]] auto half_a = [&](i32x8& f, const uint8_t* unit, int i, int hh, int h, bool half = false) {
    if constexpr (!A_TR) {
      read_half(f, unit - (half ? half_rows_back : 0) + fa_off + i * 32 * BK, hh, h);
    } else {
      read_half_tr(f, (uint32_t)(uintptr_t)unit + (half ? fat_half[i] : fat_off[i]) + hh * (64 * kTrPitch), h);
    }
  };
  // weight fragment j / token fragment i, K half hh, of the unit at `unit`
  auto read_frag_b = [&](i32x8& f, const uint8_t* unit, int j, int hh) {
    if constexpr (!B_TR) {
      read_frag(f, unit + fb_off + j * 32 * BK, hh);
    } else {
      read_frag_tr(f, (uint32_t)(uintptr_t)unit + fbt_off[j] + hh * (64 * kTrPitch));
    }
  };
  auto read_frag_a = [&](i32x8& f, const uint8_t* unit, int i, int hh, bool half = false) {
    if constexpr (!A_TR) {
      read_frag(f, unit - (half ? half_rows_back : 0) + fa_off + i * 32 * BK, hh);
    } else {
      read_frag_tr(f, (uint32_t)(uintptr_t)unit + (half ? fat_half[i] : fat_off[i]) + hh * (64 * kTrPitch));
    }
  };

  // ---- fill: steps 0 and 1 of the stream into units 0..3, the first fragments into registers ----
  load_setup();
#pragma unroll
  for (int j = 0; j < kParts; ++j) dma_a(0, j);
#pragma unroll
  for (int j = 0; j < kParts; ++j) dma_b(1, j);
  dma_advance();
#pragma unroll
  for (int j = 0; j < kParts; ++j) dma_a(2, j);
#pragma unroll
  for (int j = 0; j < kParts; ++j) dma_b(3, j);
  dma_advance();
  FP8GMM_WAIT_VM(2 * kParts);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int j = 0; j < NT; ++j) read_frag_b(fb0[j], lds + US, j, 0);
  // height of the tile that a record's K steps belong to - for a record without K steps, of the next record with
  // some (the planner notes it there): the load stream skips records without K steps, so the fragments read at
  // the end of a tile are those of the next tile that has any
  auto half_height = [](const ItemTile& t) {
    return TILE == 256 && ((t.nk > 0 ? t.flags : t.flags >> 1) & FP8GMM_ITEM_HALF_HEIGHT) != 0;
  };
  ItemTile cp_next = item_tile(0);  // the compute side's next record, fetched ahead like the load side's
  bool nxt_half = half_height(cp_next);   // height of the tile whose first fragments are in fa0 / fb0
#pragma unroll
  for (int i = 0; i < MT; ++i) read_frag_a(fa0[i], lds, i, 0, nxt_half);
  int ua = 0;  // ring unit of the current step's token rows; its weight rows are in the next unit
  // vmcnt counts loads and stores in issue order.  The barrier of a step needs the next step's units, which are
  // older than the token loads issued during the low half-step: "all but the newest kParts".  Right after an
  // interior epilogue the newest operations also include that epilogue's kFastStores stores, which nothing in
  // LDS depends on: at the first barrier after it they may stay in flight.
  int relaxed = 0;   // stores of the epilogue just before that may stay in flight at the next barrier

  // The accumulation registers belong to the statements below (see acc_tile): named as clobbered once, they count
  // as used everywhere, and the compiler keeps out of them.
  if constexpr (TILE == 256) {
    asm volatile("" ::: FP8GMM_ALL_ACC_256);
  } else {
    asm volatile("" ::: FP8GMM_ALL_ACC_64);
  }
// source 0 = weights (format B_FMT -> cbsz), source 1 = tokens (format A_FMT -> blgp); MFMA tile (i, j) accumulates
// in a[16 (NT i + j) ..+15]
#if defined(__HIP_DEVICE_COMPILE__)
#define FP8GMM_MFMA(i, j, FB, FA)                                                                      \
  asm volatile("v_mfma_f32_32x32x64_f8f6f4 a[%2:%3], %0, %1, a[%2:%3] cbsz:%4 blgp:%5" ::"v"(FB), "v"(FA), \
               "n"(16 * (NT * (i) + (j))), "n"(16 * (NT * (i) + (j)) + 15), "n"(B_FMT), "n"(A_FMT))
// ... starting from zero: the first product into a tile's accumulators
#define FP8GMM_MFMA_Z(i, j, FB, FA)                                                                    \
  asm volatile("v_mfma_f32_32x32x64_f8f6f4 a[%2:%3], %0, %1, 0 cbsz:%4 blgp:%5" ::"v"(FB), "v"(FA),      \
               "n"(16 * (NT * (i) + (j))), "n"(16 * (NT * (i) + (j)) + 15), "n"(B_FMT), "n"(A_FMT))
#else  // the host pass only needs the kernel's signature (and cannot take 32-byte vectors as "v" operands)
#define FP8GMM_MFMA(i, j, FB, FA) ((void)(FB), (void)(FA))
#define FP8GMM_MFMA_Z(i, j, FB, FA) ((void)(FB), (void)(FA))
#endif
// FIRST (of the enclosing step): the first step of a tile, whose low-half products have been issued already - from
// inside the previous tile's epilogue, or by start_tile
#define FP8GMM_MF0(i, j)                                    \
  do {                                                      \
    if constexpr (!FIRST) FP8GMM_MFMA(i, j, fb0[j], fa0[i]); \
  } while (0)
#define FP8GMM_MF1(i, j) FP8GMM_MFMA(i, j, fb1[j], fa1[i])

  // The first 16 products of a tile (the low K half of its first step) start its accumulators from zero and need
  // registers only - the fragments are read a half-step ahead.  They are issued as soon as the accumulators are
  // free: from inside the previous tile's epilogue where that is the staged bf16 form, right after it otherwise.
  // Invariant at the top of the item loop: if the item has K work, those products are under way.
  // (a tile of half height has the products i < MT / 2 only)
  auto start_tile = [&fb0, &fa0](bool half, bool upper_only = false) {
    static_for<MT * NT>([&](auto tc) {
      constexpr int i = decltype(tc)::value / NT, j = decltype(tc)::value % NT;
      if ((i >= MT / 2 && half) || (i < MT / 2 && upper_only)) return;
      const i32x8 wf = fb0[j], tf = fa0[i];
      FP8GMM_MFMA_Z(i, j, wf, tf);
    });
  };
  if (cp_next.nk > 0) start_tile(nxt_half);
  // Where an epilogue cannot take the next tile's products in (every form but the staged bf16 one), it does not
  // have to carry that tile's first fragments through its arithmetic either: they are fetched again afterwards,
  // from the ring units that still hold them, which leaves the epilogue 64 more registers.
  auto refetch_first_fragments = [&](int unit_a, bool half) {
    const int unit_b = ring_inc(unit_a);
#pragma unroll
    for (int j = 0; j < NT; ++j) read_frag_b(fb0[j], lds + unit_b * US, j, 0);
#pragma unroll
    for (int i = 0; i < MT; ++i) read_frag_a(fa0[i], lds + unit_a * US, i, 0, half);
  };
  for (int r_cp = 0;; ++r_cp) {
    const ItemTile g = cp_next;
    if (g.prob < 0) break;
    cp_next = item_tile(r_cp + 1);
    // only the epilogue needs the problem's record and its scaling factors: the main loop hides the reads
    const fp8gmm_gemm_problem pr = probs[g.prob];
    const float scale_ab = load_scale(pr.a_scale_inv) * load_scale(pr.b_scale_inv);
    const float scale_c = load_scale(pr.c_scale);
    const int m0 = g.m0, n0 = g.n0;
    const bool cur_half = TILE == 256 && (g.flags & FP8GMM_ITEM_HALF_HEIGHT) != 0;   // this tile's height
    bool read_half_next = cur_half;   // height of the tile that the NEXT step belongs to

    // One K = 128 step.  `same_item`: the load cursor stays inside its current item after this step (the caller
    // knows), so advancing it is three additions; otherwise the general advance, which may switch items.
    // `half_height_tile`: the sequence for a tile of half height.  The two heights are two kinds of step, each
    // straight-line code: with both sequences inside one step behind a uniform branch, every wait for a fragment
    // after the join becomes a wait for all of them (6 % of a launch).
    auto k_step = [&](auto same_item, auto first, auto half_height_tile) {
      constexpr bool FIRST = decltype(first)::value;
      constexpr bool SAME = decltype(same_item)::value;
      constexpr bool HALF = decltype(half_height_tile)::value;
      // ring: [ua] tokens of this step, [ub] its weights, [na], [nb] the next step's, [fa] free since the
      // previous step's barrier: it receives the tokens of step + 2 during the low half-step.  The weights of
      // step + 2 go where this step's tokens are, once this step's barrier has shown that every wavefront
      // has read them.
      // The step's first MFMA needs registers only: it goes first, and the step's ring arithmetic (some thirty scalar
      // instructions) runs in its shadow instead of ahead of it.
      FP8GMM_SB(); FP8GMM_MF0(0, 0); FP8GMM_SB();
      const int ub = ring_inc(ua), na = ring_inc(ub), nb = ring_inc(na), fa = ring_inc(nb);
      // ---- low K half: fragments in fa0 / fb0; fetch the high half's from the same units.  No barrier:
      // nothing written since the last one is read here.
      if constexpr (HALF) {
        // a tile of half height: 8 products per K half, the same loads, three quarters of the fragment reads
        const uint8_t* qa = lds + ua * US;
        const uint8_t* qb = lds + ub * US;
        dma_a(fa, 0);
        half_b(fb1[0], qb, 0, 1, 0);
        half_b(fb1[0], qb, 0, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(0, 1); FP8GMM_SB();
        dma_a(fa, 1);
        half_b(fb1[1], qb, 1, 1, 0);
        half_b(fb1[1], qb, 1, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(0, 2); FP8GMM_SB();
        dma_a(fa, 2);
        half_b(fb1[2], qb, 2, 1, 0);
        half_b(fb1[2], qb, 2, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(0, 3); FP8GMM_SB();
        dma_a(fa, 3);
        half_b(fb1[3], qb, 3, 1, 0);
        half_b(fb1[3], qb, 3, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(1, 0); FP8GMM_SB();
        dma_a(fa, 4);
        half_a(fa1[0], qa, 0, 1, 0, true);
        half_a(fa1[0], qa, 0, 1, 1, true);
        FP8GMM_SB(); FP8GMM_MF0(1, 1); FP8GMM_SB();
        dma_a(fa, 5);
        half_a(fa1[1], qa, 1, 1, 0, true);
        half_a(fa1[1], qa, 1, 1, 1, true);
        FP8GMM_SB(); FP8GMM_MF0(1, 2); FP8GMM_SB();
        dma_a(fa, 6);
        dma_a(fa, 7);
        FP8GMM_SB(); FP8GMM_MF0(1, 3); FP8GMM_SB();
      } else if constexpr (TILE == 128) {
        const uint8_t* qa = lds + ua * US;
        const uint8_t* qb = lds + ub * US;
        dma_a(fa, 0);
        read_frag_b(fb1[0], qb, 0, 1);
        FP8GMM_SB(); FP8GMM_MF0(0, 1); FP8GMM_SB();
        dma_a(fa, 1);
        read_frag_b(fb1[1], qb, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(1, 0); FP8GMM_SB();
        dma_a(fa, 2);
        read_frag_a(fa1[0], qa, 0, 1);
        FP8GMM_SB(); FP8GMM_MF0(1, 1); FP8GMM_SB();
        dma_a(fa, 3);
        read_frag_a(fa1[1], qa, 1, 1);
      } else {
        // The fragment reads go out half a fragment at a time, after every MFMA.  A contraction-major operand takes 64
        // transposing reads per step and wavefront, twice the instructions of the row-major form, and a wavefront
        // issues one every 11 - 13 cycles: with whole fragments (4 reads) next to a load, or two fragments, between
        // two MFMAs the second one can be held back (worth 0.5 % of a launch against that schedule).
        const uint8_t* qa = lds + ua * US;
        const uint8_t* qb = lds + ub * US;
        dma_a(fa, 0);
        half_b(fb1[0], qb, 0, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(0, 1); FP8GMM_SB();
        half_b(fb1[0], qb, 0, 1, 1);
        half_b(fb1[1], qb, 1, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(0, 2); FP8GMM_SB();
        dma_a(fa, 1);
        half_b(fb1[1], qb, 1, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(0, 3); FP8GMM_SB();
        half_b(fb1[2], qb, 2, 1, 0);
        half_b(fb1[2], qb, 2, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(1, 0); FP8GMM_SB();
        dma_a(fa, 2);
        half_b(fb1[3], qb, 3, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(1, 1); FP8GMM_SB();
        half_b(fb1[3], qb, 3, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(1, 2); FP8GMM_SB();
        dma_a(fa, 3);
        half_a(fa1[0], qa, 0, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(1, 3); FP8GMM_SB();
        half_a(fa1[0], qa, 0, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(2, 0); FP8GMM_SB();
        dma_a(fa, 4);
        half_a(fa1[1], qa, 1, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(2, 1); FP8GMM_SB();
        half_a(fa1[1], qa, 1, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(2, 2); FP8GMM_SB();
        dma_a(fa, 5);
        half_a(fa1[2], qa, 2, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(2, 3); FP8GMM_SB();
        half_a(fa1[2], qa, 2, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(3, 0); FP8GMM_SB();
        dma_a(fa, 6);
        half_a(fa1[3], qa, 3, 1, 0);
        FP8GMM_SB(); FP8GMM_MF0(3, 1); FP8GMM_SB();
        dma_a(fa, 7);
        half_a(fa1[3], qa, 3, 1, 1);
        FP8GMM_SB(); FP8GMM_MF0(3, 2); FP8GMM_MF0(3, 3); FP8GMM_SB();
      }
      // ---- high K half: fragments in fa1 / fb1.  The barrier proves that every wavefront has read this
      // step's units (lgkmcnt(0)) and that the next step's units have landed for all of them.
      if (relaxed == kFastStores) {
        FP8GMM_WAIT_VM_LGKM(kParts + kFastStores);
      } else if (relaxed == kFastStores / 2) {
        FP8GMM_WAIT_VM_LGKM(kParts + kFastStores / 2);
      } else {
        FP8GMM_WAIT_VM_LGKM(kParts);
      }
      relaxed = 0;
      __builtin_amdgcn_s_barrier();
      if constexpr (HALF) {
        // the next step's fragments: in a step after which the load cursor may change items, all four token
        // fragments, addressed as the tile of that step wants them (a tile of full height may follow)
        const uint8_t* qa = lds + na * US;
        const uint8_t* qb = lds + nb * US;
        const bool nh = SAME ? true : read_half_next;
        FP8GMM_SB(); FP8GMM_MF1(0, 0); FP8GMM_SB();
        dma_b(ua, 0);
        half_b(fb0[0], qb, 0, 0, 0);
        half_b(fb0[0], qb, 0, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(0, 1); FP8GMM_SB();
        dma_b(ua, 1);
        half_b(fb0[1], qb, 1, 0, 0);
        half_b(fb0[1], qb, 1, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(0, 2); FP8GMM_SB();
        dma_b(ua, 2);
        half_b(fb0[2], qb, 2, 0, 0);
        half_b(fb0[2], qb, 2, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(0, 3); FP8GMM_SB();
        dma_b(ua, 3);
        half_b(fb0[3], qb, 3, 0, 0);
        half_b(fb0[3], qb, 3, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(1, 0); FP8GMM_SB();
        dma_b(ua, 4);
        half_a(fa0[0], qa, 0, 0, 0, nh);
        half_a(fa0[0], qa, 0, 0, 1, nh);
        FP8GMM_SB(); FP8GMM_MF1(1, 1); FP8GMM_SB();
        dma_b(ua, 5);
        half_a(fa0[1], qa, 1, 0, 0, nh);
        half_a(fa0[1], qa, 1, 0, 1, nh);
        FP8GMM_SB(); FP8GMM_MF1(1, 2); FP8GMM_SB();
        dma_b(ua, 6);
        if constexpr (!SAME) {
          half_a(fa0[2], qa, 2, 0, 0, nh);
          half_a(fa0[2], qa, 2, 0, 1, nh);
        }
        dma_b(ua, 7);
        if constexpr (!SAME) {
          half_a(fa0[3], qa, 3, 0, 0, nh);
          half_a(fa0[3], qa, 3, 0, 1, nh);
        }
      } else if constexpr (TILE == 128) {
        const uint8_t* qa = lds + na * US;
        const uint8_t* qb = lds + nb * US;
        FP8GMM_SB(); FP8GMM_MF1(0, 0); FP8GMM_SB();
        dma_b(ua, 0);
        read_frag_b(fb0[0], qb, 0, 0);
        FP8GMM_SB(); FP8GMM_MF1(0, 1); FP8GMM_SB();
        dma_b(ua, 1);
        read_frag_b(fb0[1], qb, 1, 0);
        FP8GMM_SB(); FP8GMM_MF1(1, 0); FP8GMM_SB();
        dma_b(ua, 2);
        read_frag_a(fa0[0], qa, 0, 0);
        FP8GMM_SB(); FP8GMM_MF1(1, 1); FP8GMM_SB();
        dma_b(ua, 3);
        read_frag_a(fa0[1], qa, 1, 0);
      } else {
        const uint8_t* qa = lds + na * US;
        const uint8_t* qb = lds + nb * US;
        // (after a step that may end its item, the next step's tile may be of half height)
        const bool nh = decltype(same_item)::value ? false : read_half_next;
        FP8GMM_SB(); FP8GMM_MF1(0, 0); FP8GMM_SB();
        dma_b(ua, 0);
        half_b(fb0[0], qb, 0, 0, 0);
        FP8GMM_SB(); FP8GMM_MF1(0, 1); FP8GMM_SB();
        half_b(fb0[0], qb, 0, 0, 1);
        half_b(fb0[1], qb, 1, 0, 0);
        FP8GMM_SB(); FP8GMM_MF1(0, 2); FP8GMM_SB();
        dma_b(ua, 1);
        half_b(fb0[1], qb, 1, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(0, 3); FP8GMM_SB();
        half_b(fb0[2], qb, 2, 0, 0);
        half_b(fb0[2], qb, 2, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(1, 0); FP8GMM_SB();
        dma_b(ua, 2);
        half_b(fb0[3], qb, 3, 0, 0);
        FP8GMM_SB(); FP8GMM_MF1(1, 1); FP8GMM_SB();
        half_b(fb0[3], qb, 3, 0, 1);
        FP8GMM_SB(); FP8GMM_MF1(1, 2); FP8GMM_SB();
        dma_b(ua, 3);
        half_a(fa0[0], qa, 0, 0, 0, nh);
        FP8GMM_SB(); FP8GMM_MF1(1, 3); FP8GMM_SB();
        half_a(fa0[0], qa, 0, 0, 1, nh);
        FP8GMM_SB(); FP8GMM_MF1(2, 0); FP8GMM_SB();
        dma_b(ua, 4);
        half_a(fa0[1], qa, 1, 0, 0, nh);
        FP8GMM_SB(); FP8GMM_MF1(2, 1); FP8GMM_SB();
        half_a(fa0[1], qa, 1, 0, 1, nh);
        FP8GMM_SB(); FP8GMM_MF1(2, 2); FP8GMM_SB();
        dma_b(ua, 5);
        half_a(fa0[2], qa, 2, 0, 0, nh);
        FP8GMM_SB(); FP8GMM_MF1(2, 3); FP8GMM_SB();
        half_a(fa0[2], qa, 2, 0, 1, nh);
        FP8GMM_SB(); FP8GMM_MF1(3, 0); FP8GMM_SB();
        dma_b(ua, 6);
        half_a(fa0[3], qa, 3, 0, 0, nh);
        FP8GMM_SB(); FP8GMM_MF1(3, 1); FP8GMM_SB();
        dma_b(ua, 7);
        half_a(fa0[3], qa, 3, 0, 1, nh);
      }
      // common to every sequence: the load cursor moves on (in the shadow of the step's last products)
      if constexpr (SAME) {
        ++ld_kt;
        step_setup();
      } else {
        dma_advance();
      }
      if constexpr (HALF) {
        FP8GMM_SB(); FP8GMM_MF1(1, 3); FP8GMM_SB();
      } else if constexpr (TILE == 256) {
        FP8GMM_SB(); FP8GMM_MF1(3, 2); FP8GMM_MF1(3, 3); FP8GMM_SB();
      }
      ua = na;
    };
    // The load cursor runs two steps ahead of this loop: while at least three steps of the item remain, its
    // next step lies in the same item.
    // The token fragments that a tile's LAST step reads belong to the next tile with K steps, and are addressed by
    // that tile's height.
    const bool after_half = half_height(cp_next);
    // One run of steps per height, one after the other, the run of the other height with no steps: as alternatives
    // behind a branch, the compiler carries the load cursor's scalar state (descriptors, LDS addresses) through the
    // join in vector registers, which the LDS-DMA statements cannot take.
    auto steps = [&](int nk, auto half_c) {
      int kt = 0;
      if (nk > 0) {
        if (nk == 1) read_half_next = after_half;
        k_step(std::false_type{}, std::true_type{}, half_c);
        kt = 1;
      }
      for (; kt + 3 < nk; ++kt) k_step(std::true_type{}, std::false_type{}, half_c);
      for (; kt < nk; ++kt) {
        if (kt == nk - 1) read_half_next = after_half;
        k_step(std::false_type{}, std::false_type{}, half_c);
      }
    };
    if (g.nk == 0) static_for<MT * NT>([&](auto tc) { acc_tile_clear<16 * decltype(tc)::value>(); });
    steps(cur_half ? 0 : g.nk, std::false_type{});
    if constexpr (TILE == 256) steps(cur_half ? g.nk : 0, std::true_type{});
    // ---- epilogue ----
    uint8_t* const stage = lds + ((ua + 4) % RING) * US;  // free until the next step's token loads
    const bool more = cp_next.prob >= 0 && cp_next.nk > 0;  // the fragments in fa0 / fb0 open another tile
    const int mt = cur_half ? MT / 2 : MT;                  // 32-row blocks of this tile per wavefront
    if (g.slot >= 0) {
      // a piece of a tile that is shared along K: leave the accumulators for the fix-up kernel
      partial_store<TILE>(workspace + (size_t)g.slot * kPartialBytes);
      relaxed = 0;
      if (more) {
        refetch_first_fragments(ua, after_half);
        start_tile(after_half);
      }
    } else if (more && staged_bf16_tile<TILE>(pr, m0, n0, out_kind, epilogue)) {
      // the next tile's first products go out as the accumulators they overwrite are read out, in the shadow of
      // the epilogue's vector arithmetic
      relaxed = tile_epilogue<TILE>(pr, m0, n0, out_kind, epilogue, stage, mt, !A_TR && !B_TR, !A_TR, scale_ab, scale_c,
                                    [&fb0, &fa0, after_half](auto ic, auto jc) {
                                      constexpr int i = decltype(ic)::value, j = decltype(jc)::value;
                                      if (i >= MT / 2 && after_half) return;
                                      const i32x8 wf = fb0[j], tf = fa0[i];
                                      FP8GMM_MFMA_Z(i, j, wf, tf);
                                    });
      // a tile of half height released the lower blocks only
      if (cur_half && !after_half) start_tile(false, true);
    } else {
      relaxed = tile_epilogue<TILE>(pr, m0, n0, out_kind, epilogue, stage, mt, !A_TR && !B_TR, !A_TR, scale_ab, scale_c);
      if (more) {
        refetch_first_fragments(ua, after_half);
        start_tile(after_half);
      }
    }
  }
  // zero-fill loads issued past the end of the stream still target this workgroup's LDS
  FP8GMM_WAIT_VM(0);
}


#undef FP8GMM_MF0
#undef FP8GMM_MF1

}  // namespace fp8gmm
#include "grouped_gemm_dual.h"
namespace fp8gmm {

// The template argument that stands for the form with two sets of accumulators (tiles of 128 x 256) wherever a tile
// size selects a kernel.
constexpr int kTileDual = FP8GMM_GEMM_DUAL_TILE_M + kGemmTileN;
static_assert(kTileDual != kGemmTileM && kTileDual != FP8GMM_GEMM_SMALL_TILE, "a code of its own");

// Per device: "the GEMM kernels may use the whole LDS" has been set for this variant.  fp8gmm_init sets it for
// every variant; a launch on a device that was never initialised sets its own.
constexpr int kMaxDevices = 64;

template <int A_FMT, int B_FMT, bool A_TR, bool B_TR, int TILE>
int prepare_variant(int dev) {
  static std::atomic<bool> attr_set[kMaxDevices];
  if (dev < 0 || dev >= kMaxDevices) return FP8GMM_ERR_NO_DEVICE;
  if (!attr_set[dev].load(std::memory_order_acquire)) {
    const void* kernel = nullptr;
    int lds_bytes = 0;
    if constexpr (TILE == kTileDual) {
      kernel = reinterpret_cast<const void*>(grouped_gemm_dual_kernel<A_FMT, B_FMT, A_TR, B_TR>);
      lds_bytes = RING * BN * BK;
    } else {
      kernel = reinterpret_cast<const void*>(grouped_gemm_kernel<A_FMT, B_FMT, A_TR, B_TR, TILE>);
      lds_bytes = RING * TILE * BK;
    }
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
      return FP8GMM_ERR_LAUNCH;
    attr_set[dev].store(true, std::memory_order_release);
  }
  return FP8GMM_OK;
}

template <int A_FMT, int B_FMT, bool A_TR, bool B_TR, int TILE>
int launch_variant(const fp8gmm_gemm_problem* probs_dev, const fp8gmm_gemm_item* items_dev, int grid, int out_kind,
                   int epilogue, uint8_t* workspace, const fp8gmm_tensor_desc* merge_descs, int merge_n,
                   hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return FP8GMM_ERR_NO_DEVICE;
  const int rc = prepare_variant<A_FMT, B_FMT, A_TR, B_TR, TILE>(dev);
  if (rc != FP8GMM_OK) return rc;
  if constexpr (TILE == kTileDual) {
    // bf16 results without a fused epilogue only (the caller has checked)
    hipLaunchKernelGGL((grouped_gemm_dual_kernel<A_FMT, B_FMT, A_TR, B_TR>), dim3(grid), dim3(NTHREADS), RING * BN * BK,
                       stream, probs_dev, items_dev, merge_descs, merge_n);
  } else {
    hipLaunchKernelGGL((grouped_gemm_kernel<A_FMT, B_FMT, A_TR, B_TR, TILE>), dim3(grid), dim3(NTHREADS),
                       RING * TILE * BK, stream, probs_dev, items_dev, out_kind, epilogue, workspace, merge_descs, merge_n);
  }
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

// One explicit instantiation per operand format / layout combination, each in its own translation unit
// (gemm_variant.hip compiled with -DFP8GMM_VARIANT_*): the kernel takes most of a minute to compile.
#define FP8GMM_FOR_EACH_GEMM_VARIANT(X)           \
  X(FP8GMM_E4M3, FP8GMM_E4M3, false, false, 256)  \
  X(FP8GMM_E5M2, FP8GMM_E4M3, false, false, 256)  \
  X(FP8GMM_E4M3, FP8GMM_E5M2, false, false, 256)  \
  X(FP8GMM_E4M3, FP8GMM_E4M3, false, true, 256)   \
  X(FP8GMM_E5M2, FP8GMM_E4M3, false, true, 256)   \
  X(FP8GMM_E4M3, FP8GMM_E4M3, true, true, 256)    \
  X(FP8GMM_E5M2, FP8GMM_E4M3, true, true, 256)    \
  X(FP8GMM_E4M3, FP8GMM_E4M3, false, false, 128)  \
  X(FP8GMM_E5M2, FP8GMM_E4M3, false, false, 128)  \
  X(FP8GMM_E4M3, FP8GMM_E5M2, false, false, 128)  \
  X(FP8GMM_E4M3, FP8GMM_E4M3, false, true, 128)   \
  X(FP8GMM_E5M2, FP8GMM_E4M3, false, true, 128)   \
  X(FP8GMM_E4M3, FP8GMM_E4M3, true, true, 128)    \
  X(FP8GMM_E5M2, FP8GMM_E4M3, true, true, 128)    \
  X(FP8GMM_E4M3, FP8GMM_E4M3, false, false, kTileDual)  \
  X(FP8GMM_E5M2, FP8GMM_E4M3, false, false, kTileDual)  \
  X(FP8GMM_E4M3, FP8GMM_E5M2, false, false, kTileDual)  \
  X(FP8GMM_E4M3, FP8GMM_E4M3, false, true, kTileDual)   \
  X(FP8GMM_E5M2, FP8GMM_E4M3, false, true, kTileDual)   \
  X(FP8GMM_E4M3, FP8GMM_E4M3, true, true, kTileDual)    \
  X(FP8GMM_E5M2, FP8GMM_E4M3, true, true, kTileDual)

#define FP8GMM_DECLARE_VARIANT(AF, BF, AT, BT, TL)                                                                     \
  extern template int prepare_variant<AF, BF, AT, BT, TL>(int);                                                        \
  extern template int launch_variant<AF, BF, AT, BT, TL>(const fp8gmm_gemm_problem*, const fp8gmm_gemm_item*, int, int, \
                                                         int, uint8_t*, const fp8gmm_tensor_desc*, int, hipStream_t);
#ifndef FP8GMM_VARIANT_INDEX
FP8GMM_FOR_EACH_GEMM_VARIANT(FP8GMM_DECLARE_VARIANT)
#endif

}  // namespace fp8gmm
