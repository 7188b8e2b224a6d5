// The grouped GEMM on tiles of 128 x 256 with TWO sets of accumulators per wavefront: while the products of one
// tile fill one set, the finished tile in the other set is scaled, converted and stored in pieces BETWEEN those
// products, and the load stream never pauses.  Included by grouped_gemm_kernel.h (whose ring, load stream, fragment
// layout and work list this kernel shares) - see there for everything that is not about the two sets.
//
// Why: with one set (grouped_gemm_kernel) a workgroup's matrix pipes idle and its ring stays full of the next tile's
// first steps through every epilogue, and all workgroups of a launch reach their epilogues together, so that the
// stores come in bursts and nothing overlaps them (a quarter to a third of a launch with a short contraction).
// Here a tile's result leaves in four pieces of eight quarters, spread over the first two steps of the next tile.
//
// The price: a wavefront's sub-tile is 64 x 128 instead of 128 x 128, so a product needs 1.5 x the fragment reads
// from LDS and 1.5 x the operand bytes through the load path (1.33 x from L2, where neighbouring tiles share).  The
// load path is what launches with a short contraction wait for most, so the form only pays where the operands come
// from the memory-side cache rather than from HBM, and never where the matrix pipes are busy (long contractions);
// which form a launch takes is decided when it is planned (FP8GMM_GEMM_TILE_DUAL).  bf16 results without a fused
// epilogue only; whole tiles only (no sharing along K).  Every tile gets the same bits as from the other forms: the
// same products in the same order into fp32 accumulators, one rounding.
//
// Layout.  Wavefront (wave_m, wave_n) owns rows wave_m * 64 + 32 i + l32 (i < 2) and columns wave_n * 128 + 32 j ..
// (j < 4) of the tile; MFMA block (i, j) of set S accumulates in a[16 (4 (i + 2 S) + j) ..+15].  LDS holds THREE
// whole steps: stage t = 16 KB of tokens (128 rows x 128 B, or 128 contraction rows x 128 B, in the layout of the
// small tile's units) followed by 32 KB of weights (the large tile's unit), 48 KB each, and behind them 4 KB per
// wavefront that stage the result pieces, 32 rows x 64 columns at a time, so that every store instruction writes
// whole 128-byte lines.  The smaller steps leave room for a longer run-up than the large tile's two and a half
// steps: a step's loads are issued two and a half to three steps before it is computed (its first half behind the
// barrier of the step three before it, which frees the stage; the rest during the low K half of the step two before
// it).  These launches wait for memory, not for the matrix pipes: what a compute unit has in flight is what it gets.
#pragma once

namespace fp8gmm {

constexpr int kDualRows = FP8GMM_GEMM_DUAL_TILE_M;   // rows of a tile of this form
constexpr int kDualStores = 4;                        // 16-byte stores per wavefront and result piece

template <int BASE>
__device__ __forceinline__ f32x4 acc_quad() {   // four consecutive accumulators as ordinary vector registers
  f32x4 t;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t[0]) : "n"(BASE + 0));
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t[1]) : "n"(BASE + 1));
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t[2]) : "n"(BASE + 2));
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t[3]) : "n"(BASE + 3));
  return t;
}

#if defined(__HIP_DEVICE_COMPILE__)
#define FP8GMM_DUAL_MFMA(S, i, j, FB, FA)                                                                 \
  asm volatile("v_mfma_f32_32x32x64_f8f6f4 a[%2:%3], %0, %1, a[%2:%3] cbsz:%4 blgp:%5" ::"v"(FB), "v"(FA), \
               "n"(16 * (4 * ((i) + 2 * (S)) + (j))), "n"(16 * (4 * ((i) + 2 * (S)) + (j)) + 15), "n"(B_FMT), \
               "n"(A_FMT))
#define FP8GMM_DUAL_MFMA_Z(S, i, j, FB, FA)                                                               \
  asm volatile("v_mfma_f32_32x32x64_f8f6f4 a[%2:%3], %0, %1, 0 cbsz:%4 blgp:%5" ::"v"(FB), "v"(FA),         \
               "n"(16 * (4 * ((i) + 2 * (S)) + (j))), "n"(16 * (4 * ((i) + 2 * (S)) + (j)) + 15), "n"(B_FMT), \
               "n"(A_FMT))
#else
#define FP8GMM_DUAL_MFMA(S, i, j, FB, FA) ((void)(FB), (void)(FA))
#define FP8GMM_DUAL_MFMA_Z(S, i, j, FB, FA) ((void)(FB), (void)(FA))
#endif

template <int A_FMT, int B_FMT, bool A_TR, bool B_TR>
__global__ __launch_bounds__(NTHREADS, 1) void grouped_gemm_dual_kernel(
    const fp8gmm_gemm_problem* __restrict__ probs, const fp8gmm_gemm_item* __restrict__ items,
    const fp8gmm_tensor_desc* __restrict__ merge_descs, int merge_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  if (merge_n > 0 && blockIdx.x == 0) merge_amax_partials(merge_descs, merge_n, threadIdx.x, NTHREADS);
  constexpr int TM = kDualRows, TN = BN;
  constexpr int kUnitA = TM * BK, kUnitB = TN * BK;   // 16 KB of tokens, 32 KB of weights
  constexpr int kStep = kUnitA + kUnitB;              // one stage of the ring: 48 KB
  constexpr int kStages = 3;
  constexpr int kPieceOffset = kStages * kStep;       // the result pieces' staging area: the last 16 KB
  constexpr int kStageBytes = 4096;                   // ... per wavefront: 32 rows x 128 B
  static_assert(kPieceOffset + NWAVES * kStageBytes == RING * BN * BK, "all of the LDS the large tile has");
  constexpr int MT = 2, NT = 4;          // MFMA blocks of a wavefront's 64 x 128 sub-tile
  constexpr int kPartsA = 4, kPartsB = 8;  // load instructions (1 KB each) per wavefront and unit

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int l32 = lane & 31;
  const int khalf = lane >> 5;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);

  // load and fragment maps: those of grouped_gemm_kernel, the token operand's with the small tile's extents
  const int drow = lane >> 3;
  const int dchunk = (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
  const int fsw = (l32 >> 1) & 7;
  int fc[2][2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int q = 0; q < 2; ++q) fc[hh][q] = ((4 * hh + 2 * khalf + q) ^ fsw) << 4;
  const int fa_off = (wave_m * 64 + l32) * BK;
  const int fb_off = (wave_n * 128 + l32) * BK;
  const int tr_b = (lane & 15) >> 1, tr_h = lane & 1, tr_g = (lane >> 4) & 1;
  constexpr int kPitchA = TM, kPitchB = TN;   // bytes per contraction row of a contraction-major unit
  int fbt_off[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
    fbt_off[j] = (32 * khalf + tr_b) * kPitchB + 8 * tr_h + (((wave_n * 8 + 2 * j + tr_g) ^ (2 * tr_b)) << 4);
  int fat_off[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
    fat_off[i] = (32 * khalf + tr_b) * kPitchA + 8 * tr_h + (((wave_m * 4 + 2 * i + tr_g) ^ (tr_b & 6)) << 4);

  // ---- work list ----
  const uint8_t* const my_items = reinterpret_cast<const uint8_t*>(items + blockIdx.x);
  const size_t item_stride = (size_t)gridDim.x * sizeof(fp8gmm_gemm_item);
  auto item_load = [&](int r) { return *reinterpret_cast<const ItemLoad*>(my_items + r * item_stride); };
  auto item_tile = [&](int r) { return *reinterpret_cast<const ItemTile*>(my_items + r * item_stride + 32); };
  int r_ld = 0;
  ItemLoad ld_next_l = item_load(0);
  ItemTile ld_next_t = item_tile(0);
  if (ld_next_t.prob < 0) return;

  // ---- load side (see grouped_gemm_kernel) ----
  bool ld_live = true;
  int ld_kt = 0, ld_nk = 0, ld_kmax = 0;
  [[maybe_unused]] int ld_lda = 0, ld_ldb = 0;
  i32x4 rsrc_a = {0, 0, 0, 0x00020000}, rsrc_b = {0, 0, 0, 0x00020000};
  uint32_t a_base = 0, b_base = 0, a_step = 0, b_step = 0, a_k = 0, b_k = 0;
  bool k_ok = false;
  auto step_setup = [&]() {
    const uint32_t k0 = (uint32_t)ld_kt * BK;
    if constexpr (A_TR) {
      a_k = a_base + k0 * (uint32_t)ld_lda;
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
  // contraction-major units: weights 4 contraction rows x 256 B per instruction, tokens 8 x 128 B
  const int krow_b = wave * 4 + lane / 16;
  const int tr_col_b = ((lane & 15) ^ (2 * (krow_b & 7))) << 4;
  const int krow_a = wave * 8 + lane / 8;
  const int tr_col_a = ((lane & 7) ^ (krow_a & 6)) << 4;
  auto load_setup = [&]() {
    for (;;) {
      const ItemLoad gl = ld_next_l;
      const ItemTile gt = ld_next_t;
      ld_live = gt.prob >= 0;
      if (!ld_live) break;
      ld_next_l = item_load(r_ld + 1);
      ld_next_t = item_tile(r_ld + 1);
      if (gt.nk > 0) {
        // (read back as lane-uniform words: with the two copies of the tile's code below, the compiler otherwise keeps
        // the record fetched ahead, and the descriptors made of it, in vector registers, which the loads cannot take)
        rsrc_a[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)gl.a);
        rsrc_a[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(gl.a >> 32));
        rsrc_a[2] = __builtin_amdgcn_readfirstlane((int)gl.a_bytes);
        rsrc_b[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)gl.b);
        rsrc_b[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(gl.b >> 32));
        rsrc_b[2] = __builtin_amdgcn_readfirstlane((int)gl.b_bytes);
        if constexpr (!A_TR) {
          a_base = (uint32_t)(wave * 8 + drow) * (uint32_t)gl.lda + dchunk * 16;
          a_step = NWAVES * 8 * (uint32_t)gl.lda;
        } else {
          a_base = (uint32_t)krow_a * (uint32_t)gl.lda + (uint32_t)tr_col_a;
          a_step = NWAVES * 8 * (uint32_t)gl.lda;
          ld_lda = gl.lda;
        }
        if constexpr (!B_TR) {
          b_base = (uint32_t)(wave * 8 + drow) * (uint32_t)gl.ldb + dchunk * 16;
          b_step = NWAVES * 8 * (uint32_t)gl.ldb;
        } else {
          b_base = (uint32_t)krow_b * (uint32_t)gl.ldb + (uint32_t)tr_col_b;
          b_step = NWAVES * 4 * (uint32_t)gl.ldb;
          ld_ldb = gl.ldb;
        }
        ld_kmax = gt.k - dchunk * 16;
        ld_kt = gt.k_begin;
        ld_nk = gt.k_begin + gt.nk;
        step_setup();
        return;
      }
      ++r_ld;
    }
    rsrc_a[2] = 0;
    rsrc_b[2] = 0;
  };
  // part j of the tokens / weights of the step the load cursor points at, into stage `stage`
  auto dma_a = [&](int stage, int j) {   // j < kPartsA
    uint32_t v = a_k + j * a_step;
    if constexpr (!A_TR) v = k_ok ? v : 0xffffffffu;
    const uint32_t l = lds_base + stage * kStep + (wave + NWAVES * j) * 1024;
    FP8GMM_DMA(l, v, rsrc_a);
  };
  auto dma_b = [&](int stage, int j) {   // j < kPartsB
    uint32_t v = b_k + j * b_step;
    if constexpr (!B_TR) v = k_ok ? v : 0xffffffffu;
    const uint32_t l = lds_base + stage * kStep + kUnitA + (wave + NWAVES * j) * 1024;
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
  auto stage_inc = [](int x) { return x + 1 == kStages ? 0 : x + 1; };

  i32x8 fa0[MT], fb0[NT], fa1[MT], fb1[NT];
  typedef int i32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
  auto read_half = [&](i32x8& f, const uint8_t* base, int hh, int h) {
    const u32x4 t = *reinterpret_cast<const u32x4*>(base + fc[hh][h]);
    f[4 * h + 0] = (int)t.x;
    f[4 * h + 1] = (int)t.y;
    f[4 * h + 2] = (int)t.z;
    f[4 * h + 3] = (int)t.w;
  };
  auto read_half_tr = [&](i32x8& f, uint32_t a, int h, int pitch) {
    const i32x2 t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + (16 * h) * pitch));
    const i32x2 t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<lds_i32x2*>(a + (16 * h + 8) * pitch));
    f[4 * h + 0] = t0.x;
    f[4 * h + 1] = t0.y;
    f[4 * h + 2] = t1.x;
    f[4 * h + 3] = t1.y;
  };
  // half h of weight fragment j / token fragment i for K half hh of the unit at `unit`
  auto half_b = [&](i32x8& f, const uint8_t* unit, int j, int hh, int h) {
    if constexpr (!B_TR) {
      read_half(f, unit + fb_off + j * 32 * BK, hh, h);
    } else {
      read_half_tr(f, (uint32_t)(uintptr_t)unit + fbt_off[j] + hh * (64 * kPitchB), h, kPitchB);
    }
  };
  auto half_a = [&](i32x8& f, const uint8_t* unit, int i, int hh, int h) {
    if constexpr (!A_TR) {
      read_half(f, unit + fa_off + i * 32 * BK, hh, h);
    } else {
      read_half_tr(f, (uint32_t)(uintptr_t)unit + fat_off[i] + hh * (64 * kPitchA), h, kPitchA);
    }
  };
  auto frag_b = [&](i32x8& f, const uint8_t* unit, int j, int hh) {
    half_b(f, unit, j, hh, 0);
    half_b(f, unit, j, hh, 1);
  };
  auto frag_a = [&](i32x8& f, const uint8_t* unit, int i, int hh) {
    half_a(f, unit, i, hh, 0);
    half_a(f, unit, i, hh, 1);
  };

  // ---- fill: steps 0 and 1 of the stream and the first half of step 2's loads; the first fragments into registers ----
  constexpr int kFirstLoads = kPartsA + 2;                 // of a step's 12 loads: the tokens and two parts of the weights
  constexpr int kLastLoads = kPartsB - 2;
  load_setup();
#pragma unroll
  for (int j = 0; j < kPartsA; ++j) dma_a(0, j);
#pragma unroll
  for (int j = 0; j < kPartsB; ++j) dma_b(0, j);
  dma_advance();
#pragma unroll
  for (int j = 0; j < kPartsA; ++j) dma_a(1, j);
#pragma unroll
  for (int j = 0; j < kPartsB; ++j) dma_b(1, j);
  dma_advance();
#pragma unroll
  for (int j = 0; j < kPartsA; ++j) dma_a(2, j);
  dma_b(2, 0);
  dma_b(2, 1);
  FP8GMM_WAIT_VM(kPartsA + kPartsB + kFirstLoads);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int j = 0; j < NT; ++j) frag_b(fb0[j], lds + kUnitA, j, 0);
#pragma unroll
  for (int i = 0; i < MT; ++i) frag_a(fa0[i], lds, i, 0);
  int cur = 0;       // stage of the current step
  int relaxed = 0;   // stores that the previous step issued (a lower bound will do): free to stay in flight at the next barrier

  asm volatile("" ::: FP8GMM_ALL_ACC_256);   // the accumulation registers belong to the statements of this file

  // ---- the finished tile that waits in the other set: where it goes ----
  bool pe_on = false;
  __amdgpu_buffer_rsrc_t pe_rc = make_rsrc(nullptr, 0);
  int pe_ldc = 0, pe_cv = 0;
  float pe_s = 1.f;
  // per-lane constants of the staged store: a lane holds 4 consecutive columns of row l32 of an MFMA block; a piece
  // (32 rows x 64 columns, two blocks) is staged as 32 rows x 128 B with 16-byte chunk c of row r at chunk
  // c ^ ((r >> 1) & 7) and read back 8 rows x 128 contiguous bytes per instruction
  const int st_wr = l32 * 128 + khalf * 8;
  const int st_rrow = lane >> 3, st_rchunk = lane & 7;
  // quarter q (0..7) of piece u (0..3) of set P: block (u / 2, 2 (u % 2) + q / 4), register group q % 4
  auto piece_quarter = [&](auto set_c, auto u_c, auto q_c, uint8_t* buf) {
    constexpr int P = decltype(set_c)::value, u = decltype(u_c)::value, q = decltype(q_c)::value;
    constexpr int i = u / 2, jj = u % 2, jl = q / 4, g = q % 4;
    const f32x4 t = acc_quad<16 * (4 * (i + 2 * P) + 2 * jj + jl) + 4 * g>();
    const u32x2 o = {pack_bf16x2(t[0] * pe_s, t[1] * pe_s), pack_bf16x2(t[2] * pe_s, t[3] * pe_s)};
    *reinterpret_cast<u32x2*>(buf + st_wr + (((4 * jl + g) ^ fsw) << 4)) = o;
  };
  auto piece_read_back = [&](u32x4 (&v)[4], const uint8_t* buf) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int r = 8 * it + st_rrow;
      v[it] = *reinterpret_cast<const u32x4*>(buf + r * 128 + ((st_rchunk ^ ((r >> 1) & 7)) << 4));
    }
  };
  auto piece_store = [&](auto u_c, const u32x4 (&v)[4]) {
    constexpr int u = decltype(u_c)::value, i = u / 2, jj = u % 2;
    const int col = wave_n * 128 + jj * 64 + st_rchunk * 8;
    const uint32_t lane_off = col < pe_cv ? (uint32_t)((st_rrow * pe_ldc + col) * 2) : kMaskedOffset;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const uint32_t row_off = (uint32_t)((wave_m * 64 + i * 32 + 8 * it) * pe_ldc * 2);  // uniform
      buf_store16_stream(v[it], pe_rc, lane_off + row_off);
    }
  };
  // pieces [U0, U1) of the waiting tile, one after the other (where no steps are left to carry them)
  auto flush = [&](auto set_c, auto u0_c, auto u1_c) {
    constexpr int U0 = decltype(u0_c)::value, U1 = decltype(u1_c)::value;
    uint8_t* buf = lds + kPieceOffset + wave * kStageBytes;
    static_for<U1 - U0>([&](auto d) {
      constexpr int u = U0 + decltype(d)::value;
      static_for<8>([&](auto qc) { piece_quarter(set_c, std::integral_constant<int, u>{}, qc, buf); });
      u32x4 v[4];
      piece_read_back(v, buf);
      piece_store(std::integral_constant<int, u>{}, v);
    });
  };

#define FP8GMM_DQ(U, Q) piece_quarter(std::integral_constant<int, 1 - S>{}, std::integral_constant<int, U>{}, \
                                      std::integral_constant<int, Q>{}, buf)
#define FP8GMM_DMF0(i, j)                                   \
  do {                                                      \
    if constexpr (FIRST) {                                  \
      FP8GMM_DUAL_MFMA_Z(S, i, j, fb0[j], fa0[i]);          \
    } else {                                                \
      FP8GMM_DUAL_MFMA(S, i, j, fb0[j], fa0[i]);            \
    }                                                       \
  } while (0)
#define FP8GMM_DMF1(i, j) FP8GMM_DUAL_MFMA(S, i, j, fb1[j], fa1[i])

  // One K = 128 step of a tile that accumulates in set S.  FIRST: the tile's first step (its low-half products start
  // from zero).  SAME: the load cursor stays inside its item after this step.  E: 0, or 1 / 2: the step carries
  // pieces 0 and 1 / 2 and 3 of the tile that waits in the other set, one in each K half: eight quarters between the
  // products, the read-back, and the four stores at the end of the half.
  auto k_step = [&](auto same_c, auto first_c, auto set_c, auto epi_c) {
    constexpr bool SAME = decltype(same_c)::value;
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr int S = decltype(set_c)::value;
    constexpr int E = decltype(epi_c)::value;
    constexpr int UL = E == 2 ? 2 : 0, UH = UL + 1;   // the pieces of the low and the high half
    FP8GMM_SB(); FP8GMM_DMF0(0, 0); FP8GMM_SB();
    const int nxt = stage_inc(cur), nn = stage_inc(nxt);
    [[maybe_unused]] uint8_t* const buf = lds + kPieceOffset + wave * kStageBytes;
    [[maybe_unused]] u32x4 pv[4];
    {
      // ---- low K half: fragments in fa0 / fb0; the high half's are read from the same stage.  The load cursor
      // points two steps ahead: the second half of that step's loads goes out (its stage was free since the
      // previous step's barrier)
      const uint8_t* qa = lds + cur * kStep;
      const uint8_t* qb = qa + kUnitA;
      dma_b(nn, 2);
      frag_b(fb1[0], qb, 0, 1);
      if constexpr (E != 0) { FP8GMM_DQ(UL, 0); FP8GMM_DQ(UL, 1); }
      FP8GMM_SB(); FP8GMM_DMF0(0, 1); FP8GMM_SB();
      dma_b(nn, 3);
      frag_b(fb1[1], qb, 1, 1);
      if constexpr (E != 0) { FP8GMM_DQ(UL, 2); }
      FP8GMM_SB(); FP8GMM_DMF0(0, 2); FP8GMM_SB();
      dma_b(nn, 4);
      frag_b(fb1[2], qb, 2, 1);
      if constexpr (E != 0) { FP8GMM_DQ(UL, 3); }
      FP8GMM_SB(); FP8GMM_DMF0(0, 3); FP8GMM_SB();
      dma_b(nn, 5);
      frag_b(fb1[3], qb, 3, 1);
      if constexpr (E != 0) { FP8GMM_DQ(UL, 4); }
      FP8GMM_SB(); FP8GMM_DMF0(1, 0); FP8GMM_SB();
      dma_b(nn, 6);
      frag_a(fa1[0], qa, 0, 1);
      if constexpr (E != 0) { FP8GMM_DQ(UL, 5); }
      FP8GMM_SB(); FP8GMM_DMF0(1, 1); FP8GMM_SB();
      dma_b(nn, 7);
      frag_a(fa1[1], qa, 1, 1);
      if constexpr (E != 0) { FP8GMM_DQ(UL, 6); FP8GMM_DQ(UL, 7); }
      FP8GMM_SB(); FP8GMM_DMF0(1, 2); FP8GMM_SB();
      if constexpr (E != 0) piece_read_back(pv, buf);
      FP8GMM_SB(); FP8GMM_DMF0(1, 3); FP8GMM_SB();
      if constexpr (E != 0) piece_store(std::integral_constant<int, UL>{}, pv);
    }
    // ---- the barrier: every wavefront has read this step's stage, and the next step's has landed.  Younger than
    // the next step's loads, and free to stay in flight: the second half of the loads of the step after it (this
    // low half's), the first half (the previous step's high half), and the stores of pieces in between
    FP8GMM_SB();
    if (relaxed != 0) {
      FP8GMM_WAIT_VM_LGKM(kFirstLoads + kLastLoads + (E != 0 ? kDualStores : 0) + 2 * kDualStores);
    } else {
      FP8GMM_WAIT_VM_LGKM(kFirstLoads + kLastLoads + (E != 0 ? kDualStores : 0));
    }
    relaxed = E != 0 ? 2 * kDualStores : 0;
    __builtin_amdgcn_s_barrier();
    {
      // ---- high K half: fragments in fa1 / fb1; the next step's low-half fragments are read from its stage.  The
      // load cursor moves on to the step three ahead, whose stage is the one this barrier has just freed
      const uint8_t* qa = lds + nxt * kStep;
      const uint8_t* qb = qa + kUnitA;
      FP8GMM_SB(); FP8GMM_DMF1(0, 0); FP8GMM_SB();
      if constexpr (SAME) {
        ++ld_kt;
        step_setup();
      } else {
        dma_advance();
      }
      dma_a(cur, 0);
      frag_b(fb0[0], qb, 0, 0);
      if constexpr (E != 0) { FP8GMM_DQ(UH, 0); FP8GMM_DQ(UH, 1); }
      FP8GMM_SB(); FP8GMM_DMF1(0, 1); FP8GMM_SB();
      dma_a(cur, 1);
      frag_b(fb0[1], qb, 1, 0);
      if constexpr (E != 0) { FP8GMM_DQ(UH, 2); }
      FP8GMM_SB(); FP8GMM_DMF1(0, 2); FP8GMM_SB();
      dma_a(cur, 2);
      frag_b(fb0[2], qb, 2, 0);
      if constexpr (E != 0) { FP8GMM_DQ(UH, 3); }
      FP8GMM_SB(); FP8GMM_DMF1(0, 3); FP8GMM_SB();
      dma_a(cur, 3);
      frag_b(fb0[3], qb, 3, 0);
      if constexpr (E != 0) { FP8GMM_DQ(UH, 4); }
      FP8GMM_SB(); FP8GMM_DMF1(1, 0); FP8GMM_SB();
      dma_b(cur, 0);
      frag_a(fa0[0], qa, 0, 0);
      if constexpr (E != 0) { FP8GMM_DQ(UH, 5); }
      FP8GMM_SB(); FP8GMM_DMF1(1, 1); FP8GMM_SB();
      dma_b(cur, 1);
      frag_a(fa0[1], qa, 1, 0);
      if constexpr (E != 0) { FP8GMM_DQ(UH, 6); FP8GMM_DQ(UH, 7); }
      FP8GMM_SB(); FP8GMM_DMF1(1, 2); FP8GMM_SB();
      if constexpr (E != 0) piece_read_back(pv, buf);
      FP8GMM_SB(); FP8GMM_DMF1(1, 3); FP8GMM_SB();
      if constexpr (E != 0) piece_store(std::integral_constant<int, UH>{}, pv);
      FP8GMM_SB();
    }
    cur = nxt;
  };

  // One tile in set S; the tile that waits (pe_on) is in the other set.  Returns false at the end of the list.
  ItemTile cp_next = item_tile(0);
  int r_cp = 0;
  auto tile = [&](auto set_c) {
    constexpr int S = decltype(set_c)::value;
    using SetC = std::integral_constant<int, S>;
    using Waiting = std::integral_constant<int, 1 - S>;
    using T = std::true_type;
    using F = std::false_type;
    using E0 = std::integral_constant<int, 0>;
    using E1 = std::integral_constant<int, 1>;
    using E2 = std::integral_constant<int, 2>;
    const ItemTile g = cp_next;
    if (g.prob < 0) return false;
    cp_next = item_tile(++r_cp);
    const fp8gmm_gemm_problem pr = probs[g.prob];
    const float scale_ab = load_scale(pr.a_scale_inv) * load_scale(pr.b_scale_inv);
    const int nk = g.nk;
    if (nk == 0) static_for<MT * NT>([&](auto tc) { acc_tile_clear<16 * (4 * 2 * S + decltype(tc)::value)>(); });
    // the steps, one run per kind and the runs one after the other (alternatives behind a branch make the compiler
    // carry the load cursor's scalar state through the join in vector registers)
    const bool carry = pe_on;
    for (int c = (nk > 0 && carry) ? 1 : 0; c > 0; --c) k_step(F{}, T{}, SetC{}, E1{});
    for (int c = (nk > 0 && !carry) ? 1 : 0; c > 0; --c) k_step(F{}, T{}, SetC{}, E0{});
    const bool same1 = 1 + 3 < nk;
    for (int c = (nk > 1 && carry && same1) ? 1 : 0; c > 0; --c) k_step(T{}, F{}, SetC{}, E2{});
    for (int c = (nk > 1 && carry && !same1) ? 1 : 0; c > 0; --c) k_step(F{}, F{}, SetC{}, E2{});
    int kt = (nk > 1 && carry) ? 2 : (nk > 0 ? 1 : 0);
    for (; kt + 3 < nk; ++kt) k_step(T{}, F{}, SetC{}, E0{});
    for (; kt < nk; ++kt) k_step(F{}, F{}, SetC{}, E0{});
    // what the steps could not carry of the waiting tile
    // (`relaxed` stays what it is: the stores of a flush only add to those in flight)
    if (carry && nk == 0) flush(Waiting{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 4>{});
    if (carry && nk == 1) flush(Waiting{}, std::integral_constant<int, 2>{}, std::integral_constant<int, 4>{});
    // ---- this tile's result: it waits in set S for the next tile's steps, if it can take the staged form
    const int m0 = g.m0, n0 = g.n0;
    const int M = pr.m, N = pr.n;
    const int ldc = pr.ldc;
    const int rv = M - m0 < TM ? M - m0 : TM;
    const int cv = N - n0 < TN ? N - n0 : TN;
    const bool desc_ok = ((ldc & 7) == 0) && ldc < (1 << 21) && ((reinterpret_cast<uintptr_t>(pr.c) & 15) == 0);
    if (desc_ok && (cv == TN || (cv & 7) == 0)) {
      uint16_t* const C = static_cast<uint16_t*>(pr.c) + (int64_t)m0 * ldc + n0;
      pe_rc = make_uniform_rsrc(C, (uint32_t)(((rv - 1) * ldc + cv) * 2));
      pe_ldc = ldc;
      pe_cv = cv;
      pe_s = scale_ab;
      pe_on = true;
    } else {
      // element by element (a pitch or base address that 16-byte stores cannot take)
      pe_on = false;
      relaxed = 0;
      uint16_t* __restrict__ C = static_cast<uint16_t*>(pr.c);
      const bool vec = ((ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0);
      static_for<MT * NT>([&](auto tc) {
        constexpr int i = decltype(tc)::value / NT, j = decltype(tc)::value % NT;
        const int m = m0 + wave_m * 64 + i * 32 + l32;
        const f32x16 t = acc_tile<16 * (4 * (i + 2 * S) + j)>();
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wave_n * 128 + j * 32 + q * 8 + khalf * 4;
          if (m >= M || n >= N) continue;
          const float r0 = t[4 * q + 0] * scale_ab, r1 = t[4 * q + 1] * scale_ab, r2 = t[4 * q + 2] * scale_ab,
                      r3 = t[4 * q + 3] * scale_ab;
          const int64_t off = (int64_t)m * ldc + n;
          if (vec && n + 3 < N) {
            const u32x2 o = {pack_bf16x2(r0, r1), pack_bf16x2(r2, r3)};
            global_store(C + off, o);
          } else {
            const float r[4] = {r0, r1, r2, r3};
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < N) global_store(C + off + e, (uint16_t)f32_to_bf16_bits(r[e]));
          }
        }
      });
    }
    return true;
  };
  for (;;) {
    if (!tile(std::integral_constant<int, 0>{})) {
      // the last tile sits in set 1
      if (pe_on) flush(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 4>{});
      break;
    }
    if (!tile(std::integral_constant<int, 1>{})) {
      if (pe_on) flush(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 4>{});
      break;
    }
  }
  // zero-fill loads issued past the end of the stream still target this workgroup's LDS
  FP8GMM_WAIT_VM(0);
}

#undef FP8GMM_DQ
#undef FP8GMM_DMF0
#undef FP8GMM_DMF1

}  // namespace fp8gmm
