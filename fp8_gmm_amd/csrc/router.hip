// Token routing around the grouped expert layers, for gfx950: group the (token, choice) pairs of a top-k
// router by expert and move rows into and out of that order.
//
// The reference's example MoE layers take these steps from the megablocks package (fp8_gmm/example.py:15-32:
// topk, ops.sort / ops.histogram / ops.inclusive_cumsum; :50-59, :86-94, :113-119: ops.gather / ops.scatter);
// megablocks is not part of the reference tree, so what is implemented here is the published meaning of those
// operators:
//   sort       stable sort of the expert ids: bin_ids = sorted ids, indices = original flat positions
//   histogram  rows per expert;  inclusive_cumsum of it = end row of every expert in sorted order
//   gather     out[i, :] = x[indices[i] / top_k, :]                       (rows into expert order)
//   scatter    out[t, :] = sum_k w[t * top_k + k] * x[pos(t, k), :]       (rows back to token order, weighted)
// where pos is the inverse of `indices`.
//
// Sorting is a counting sort in three small launches (ids are < 4096 and the list is at most a few hundred
// thousand entries): per-chunk histograms, a scan that turns them into start offsets, and a stable placement in
// which a single-wavefront workgroup walks its chunk in order.  The row movers are HBM-bound: one wavefront per
// row, 16 bytes per lane per access.
#include "device_utils.h"

namespace fp8gmm {
namespace {

constexpr int kRouteChunk = 512;        // list entries per workgroup of the counting sort
constexpr int kRouteSteps = kRouteChunk / 64;
constexpr int kRouteMaxExperts = 4096;  // size of the per-workgroup expert table in LDS (16 KB)
constexpr int kRowWaves = 4;            // wavefronts (= rows in flight) per workgroup of the row movers

__device__ __forceinline__ int clamp_expert(int e, int num_experts) {
  return e < 0 ? 0 : (e >= num_experts ? num_experts - 1 : e);
}

// counts[b][e] = entries of chunk b that go to expert e
__global__ __launch_bounds__(64) void route_count_kernel(const int32_t* __restrict__ expert_of, int n,
                                                         int num_experts, int32_t* __restrict__ counts) {
  __shared__ int32_t table[kRouteMaxExperts];
  const int lane = threadIdx.x;
  for (int e = lane; e < num_experts; e += 64) table[e] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kRouteChunk;
  int32_t ids[kRouteSteps];  // all loads of the chunk in flight at once
#pragma unroll
  for (int r = 0; r < kRouteSteps; ++r) {
    const int64_t i = base + r * 64 + lane;
    ids[r] = i < n ? expert_of[i] : -1;
  }
#pragma unroll
  for (int r = 0; r < kRouteSteps; ++r)
    if (base + r * 64 + lane < n) atomicAdd(&table[clamp_expert(ids[r], num_experts)], 1);
  __syncthreads();
  for (int e = lane; e < num_experts; e += 64) counts[(size_t)blockIdx.x * num_experts + e] = table[e];
}

// One workgroup.  counts[b][e] becomes the first sorted position of chunk b's entries for expert e;
// tokens_per_expert[e] = total of expert e, bins[e] = end of expert e in sorted order (inclusive cumsum).
__global__ __launch_bounds__(256) void route_scan_kernel(int32_t* __restrict__ counts, int chunks, int num_experts,
                                                         int32_t* __restrict__ tokens_per_expert,
                                                         int32_t* __restrict__ bins) {
  __shared__ int32_t total[kRouteMaxExperts];
  __shared__ int32_t part[256];
  const int tid = threadIdx.x;
  if (num_experts >= 256) {  // many experts: a thread per expert walks the chunks
    for (int e = tid; e < num_experts; e += 256) {
      int32_t run = 0;
      for (int b = 0; b < chunks; ++b) {
        const int32_t c = counts[(size_t)b * num_experts + e];
        counts[(size_t)b * num_experts + e] = run;  // exclusive prefix over the chunks
        run += c;
      }
      total[e] = run;
    }
  } else {  // few experts: a wavefront per expert, its lanes over 64 chunks at a time
    const int lane = tid % 64;
    for (int e = tid / 64; e < num_experts; e += 4) {
      int32_t run = 0;
      for (int b0 = 0; b0 < chunks; b0 += 64) {
        const int b = b0 + lane;
        const int32_t c = b < chunks ? counts[(size_t)b * num_experts + e] : 0;
        int32_t incl = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int32_t below = __shfl_up(incl, d, 64);
          if (lane >= d) incl += below;
        }
        if (b < chunks) counts[(size_t)b * num_experts + e] = run + incl - c;
        run += __shfl(incl, 63, 64);
      }
      if (lane == 0) total[e] = run;
    }
  }
  __syncthreads();
  // exclusive scan of the totals over the experts: thread t owns experts [t * per, (t + 1) * per)
  const int per = (num_experts + 255) / 256;
  const int lo = tid * per;
  const int hi = lo + per < num_experts ? lo + per : num_experts;
  int32_t sum = 0;
  for (int e = lo; e < hi; ++e) sum += total[e];
  part[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0;
    for (int t = 0; t < 256; ++t) {
      const int32_t s = part[t];
      part[t] = run;
      run += s;
    }
  }
  __syncthreads();
  int32_t start = part[tid];
  for (int e = lo; e < hi; ++e) {
    const int32_t cnt = total[e];
    total[e] = start;  // now: first sorted position of expert e
    if (tokens_per_expert != nullptr) tokens_per_expert[e] = cnt;
    start += cnt;
    if (bins != nullptr) bins[e] = start;
  }
  __syncthreads();
  const int64_t cells = (int64_t)chunks * num_experts;
  for (int64_t i = tid; i < cells; i += 256) counts[i] += total[i % num_experts];
}

// Stable placement: the single wavefront of a workgroup walks its chunk 64 entries at a time, in order; within
// a group of 64 an entry's rank among the entries of the same expert is the number of lower lanes that hold
// that expert.  The lanes that hold the same expert are found bit by bit of the expert id: one ballot per bit,
// ceil(log2(num_experts)) of them, whatever the number of distinct experts in the group.
__global__ __launch_bounds__(64) void route_place_kernel(const int32_t* __restrict__ expert_of, int n,
                                                         int num_experts, const int32_t* __restrict__ offsets,
                                                         int32_t* __restrict__ bin_ids,
                                                         int32_t* __restrict__ indices,
                                                         int32_t* __restrict__ inverse) {
  __shared__ int32_t next[kRouteMaxExperts];
  const int lane = threadIdx.x;
  for (int e = lane; e < num_experts; e += 64) next[e] = offsets[(size_t)blockIdx.x * num_experts + e];
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kRouteChunk;
  const uint64_t below = (1ull << lane) - 1ull;
  int bits = 0;
  while ((1 << bits) < num_experts) ++bits;
  int32_t ids[kRouteSteps];  // all loads of the chunk in flight at once
#pragma unroll
  for (int r = 0; r < kRouteSteps; ++r) {
    const int64_t i = base + r * 64 + lane;
    ids[r] = i < n ? expert_of[i] : 0;
  }
#pragma unroll
  for (int r = 0; r < kRouteSteps; ++r) {
    const int64_t i = base + r * 64 + lane;
    const bool valid = i < n;
    const int e = valid ? clamp_expert(ids[r], num_experts) : 0;
    uint64_t same = __ballot(valid);
    for (int k = 0; k < bits; ++k) {
      const bool set = (e >> k) & 1;
      const uint64_t has = __ballot(valid && set);
      same &= set ? has : ~has;
    }
    // for a valid lane `same` now marks the valid lanes with its expert
    const int pos = valid ? next[e] + __popcll(same & below) : 0;
    __syncthreads();
    if (valid && (same & below) == 0) next[e] += __popcll(same);  // the lowest lane of every expert's group
    __syncthreads();
    if (valid) {
      if (bin_ids != nullptr) bin_ids[pos] = e;
      if (indices != nullptr) indices[pos] = (int32_t)i;
      if (inverse != nullptr) inverse[i] = pos;
    }
  }
}

__global__ __launch_bounds__(256) void route_invert_kernel(const int32_t* __restrict__ indices, int n,
                                                           int32_t* __restrict__ inverse) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int32_t p = indices[i];
  if ((uint32_t)p < (uint32_t)n) inverse[p] = i;
}

__device__ __forceinline__ uint32_t scale_bf16x2(uint32_t packed, float w) {
  return pack_bf16x2(bf16_lo_to_f32(packed) * w, bf16_hi_to_f32(packed) * w);
}

// out[i, :] = w * x[src, :] with src = indices[i] / top_k and w = weights[indices[i]] (1 without weights).
// An index outside the list gives a row of zeros.
__global__ __launch_bounds__(kRowWaves * 64) void moe_gather_kernel(const uint16_t* __restrict__ x,
                                                                    const int32_t* __restrict__ indices,
                                                                    const float* __restrict__ weights,
                                                                    uint16_t* __restrict__ out, int rows_out,
                                                                    int hidden, int top_k, int vec) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kRowWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  if (row >= rows_out) return;
  const int32_t idx = indices[row];
  const bool ok = (uint32_t)idx < (uint32_t)rows_out;
  const float w = (ok && weights != nullptr) ? weights[idx] : 1.0f;
  const uint16_t* src = x + (size_t)(ok ? idx / top_k : 0) * hidden;
  uint16_t* dst = out + (size_t)row * hidden;
  if (vec) {
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(src, ok ? (uint32_t)hidden * 2u : 0u);
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(dst, (uint32_t)hidden * 2u);
    for (int c0 = 0; c0 < hidden; c0 += 64 * 8 * 4) {
      u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = buf_load16_stream(rs, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (weights != nullptr) {
          v[u].x = scale_bf16x2(v[u].x, w);
          v[u].y = scale_bf16x2(v[u].y, w);
          v[u].z = scale_bf16x2(v[u].z, w);
          v[u].w = scale_bf16x2(v[u].w, w);
        }
        buf_store16(v[u], rd, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
      }
    }
  } else {
    for (int c = lane; c < hidden; c += 64) {
      const float v = ok ? bf16_to_f32(src[c]) : 0.f;
      dst[c] = weights != nullptr ? (uint16_t)f32_to_bf16_bits(v * w) : (ok ? src[c] : (uint16_t)0);
    }
  }
}

// out[t, :] = bf16( sum over k = 0 .. top_k - 1, in that order, of w[t * top_k + k] * x[inverse[t * top_k + k], :] )
// accumulated in fp32 with separately rounded products (1 for w without weights).
__global__ __launch_bounds__(kRowWaves * 64) void moe_scatter_kernel(const uint16_t* __restrict__ x,
                                                                     const int32_t* __restrict__ inverse,
                                                                     const float* __restrict__ weights,
                                                                     uint16_t* __restrict__ out, int tokens,
                                                                     int hidden, int top_k, int vec) {
  const int lane = threadIdx.x % 64;
  const int t = blockIdx.x * kRowWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  if (t >= tokens) return;
  const int64_t rows = (int64_t)tokens * top_k;
  uint16_t* dst = out + (size_t)t * hidden;
  if (vec) {
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(dst, (uint32_t)hidden * 2u);
    constexpr int kU = 4;  // 16-byte loads in flight per lane and source row
    for (int c0 = 0; c0 < hidden; c0 += 64 * 8 * kU) {
      float acc[kU][8];
#pragma unroll
      for (int u = 0; u < kU; ++u)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[u][j] = 0.f;
#pragma unroll 2
      for (int k = 0; k < top_k; ++k) {
        const int32_t p = inverse[(size_t)t * top_k + k];
        const bool ok = (uint32_t)p < (uint32_t)rows;
        const float w = weights != nullptr ? weights[(size_t)t * top_k + k] : 1.0f;
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(x + (size_t)(ok ? p : 0) * hidden, ok ? (uint32_t)hidden * 2u : 0u);
        u32x4 v[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) v[u] = buf_load16_stream(rs, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const uint32_t q[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[u][2 * j] = acc[u][2 * j] + bf16_lo_to_f32(q[j]) * w;
            acc[u][2 * j + 1] = acc[u][2 * j + 1] + bf16_hi_to_f32(q[j]) * w;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const u32x4 o = {pack_bf16x2(acc[u][0], acc[u][1]), pack_bf16x2(acc[u][2], acc[u][3]),
                         pack_bf16x2(acc[u][4], acc[u][5]), pack_bf16x2(acc[u][6], acc[u][7])};
        buf_store16(o, rd, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
      }
    }
  } else {
    for (int c = lane; c < hidden; c += 64) {
      float acc = 0.f;
      for (int k = 0; k < top_k; ++k) {
        const int32_t p = inverse[(size_t)t * top_k + k];
        const float w = weights != nullptr ? weights[(size_t)t * top_k + k] : 1.0f;
        if ((uint32_t)p < (uint32_t)rows) acc = acc + bf16_to_f32(x[(size_t)p * hidden + c]) * w;
      }
      dst[c] = (uint16_t)f32_to_bf16_bits(acc);
    }
  }
}

// grad_w[indices[i]] = < x[i, :], grad_out[indices[i] / top_k, :] > in fp32: the gradient of scatter with respect
// to its weights.  Every position is written exactly once because `indices` is a permutation.
__global__ __launch_bounds__(kRowWaves * 64) void moe_scatter_wgrad_kernel(const uint16_t* __restrict__ x,
                                                                           const uint16_t* __restrict__ grad_out,
                                                                           const int32_t* __restrict__ indices,
                                                                           float* __restrict__ grad_w, int rows,
                                                                           int hidden, int top_k, int vec) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kRowWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  if (row >= rows) return;
  const int32_t idx = indices[row];
  if ((uint32_t)idx >= (uint32_t)rows) return;
  const uint16_t* a = x + (size_t)row * hidden;
  const uint16_t* b = grad_out + (size_t)(idx / top_k) * hidden;
  float acc = 0.f;
  if (vec) {  // 16 bytes per lane and load, four loads of each row in flight; reads past the row deliver zeros
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(a, (uint32_t)hidden * 2u);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(b, (uint32_t)hidden * 2u);
    for (int c0 = 0; c0 < hidden; c0 += 64 * 8 * 4) {
      u32x4 va[4], vb[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        va[u] = buf_load16_stream(ra, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
        vb[u] = buf_load16_stream(rb, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t pa[4] = {va[u].x, va[u].y, va[u].z, va[u].w};
        const uint32_t pb[4] = {vb[u].x, vb[u].y, vb[u].z, vb[u].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc = __builtin_fmaf(bf16_lo_to_f32(pa[q]), bf16_lo_to_f32(pb[q]), acc);
          acc = __builtin_fmaf(bf16_hi_to_f32(pa[q]), bf16_hi_to_f32(pb[q]), acc);
        }
      }
    }
  } else {
    for (int c = lane; c < hidden; c += 64) acc = __builtin_fmaf(bf16_to_f32(a[c]), bf16_to_f32(b[c]), acc);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) grad_w[idx] = acc;
}

// Both gradients of scatter in one pass over the rows: for sorted row i with idx = indices[i], token idx / top_k and
// w = weights[idx],  grad_x[i, :] = bf16(w * grad_out[token, :])  (what moe_gather_kernel writes with weights) and
// grad_w[idx] = < x[i, :], grad_out[token, :] >  (what moe_scatter_wgrad_kernel writes): the gradient row is read
// once for both.
__global__ __launch_bounds__(kRowWaves * 64) void moe_scatter_backward_kernel(const uint16_t* __restrict__ x,
                                                                              const uint16_t* __restrict__ grad_out,
                                                                              const int32_t* __restrict__ indices,
                                                                              const float* __restrict__ weights,
                                                                              uint16_t* __restrict__ grad_x,
                                                                              float* __restrict__ grad_w, int rows,
                                                                              int hidden, int top_k) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kRowWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  if (row >= rows) return;
  const int32_t idx = indices[row];
  const bool ok = (uint32_t)idx < (uint32_t)rows;
  const float w = ok ? weights[idx] : 1.0f;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(x + (size_t)row * hidden, (uint32_t)hidden * 2u);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(grad_out + (size_t)(ok ? idx / top_k : 0) * hidden,
                                              ok ? (uint32_t)hidden * 2u : 0u);   // not a row: zeros
  const __amdgpu_buffer_rsrc_t rd = make_rsrc(grad_x + (size_t)row * hidden, (uint32_t)hidden * 2u);
  float acc = 0.f;
  for (int c0 = 0; c0 < hidden; c0 += 64 * 8 * 4) {
    u32x4 va[4], vb[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      va[u] = buf_load16_stream(ra, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
      vb[u] = buf_load16_stream(rb, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t pa[4] = {va[u].x, va[u].y, va[u].z, va[u].w};
      const uint32_t pb[4] = {vb[u].x, vb[u].y, vb[u].z, vb[u].w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc = __builtin_fmaf(bf16_lo_to_f32(pa[q]), bf16_lo_to_f32(pb[q]), acc);
        acc = __builtin_fmaf(bf16_hi_to_f32(pa[q]), bf16_hi_to_f32(pb[q]), acc);
      }
      u32x4 o;
      o.x = scale_bf16x2(pb[0], w);
      o.y = scale_bf16x2(pb[1], w);
      o.z = scale_bf16x2(pb[2], w);
      o.w = scale_bf16x2(pb[3], w);
      buf_store16(o, rd, (uint32_t)(c0 + (u * 64 + lane) * 8) * 2u);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0 && ok) grad_w[idx] = acc;
}

constexpr int kTopKMax = 8;  // choices per token that the selection keeps in registers

template <bool BF16>
__device__ __forceinline__ float score_at(const void* row, int e) {
  if constexpr (BF16) return bf16_to_f32(static_cast<const uint16_t*>(row)[e]);
  return static_cast<const float*>(row)[e];
}

// One wavefront per token, its lanes over the experts.  probs[t, :] = softmax(scores[t, :]) in fp32 (max, exp of
// the differences, their sum lane by lane and then across lanes, one division per expert); the top_k choices are
// made on the scores themselves, largest first, the lower expert on equal scores, so that they do not depend on how
// an exponential rounds.
template <bool BF16>
__global__ __launch_bounds__(kRowWaves * 64) void route_topk_kernel(const void* __restrict__ scores, int tokens,
                                                                    int num_experts, int top_k,
                                                                    float* __restrict__ probs,
                                                                    float* __restrict__ weights,
                                                                    int64_t* __restrict__ selected) {
  const int lane = threadIdx.x % 64;
  const int t = blockIdx.x * kRowWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  if (t >= tokens) return;
  const void* row = static_cast<const char*>(scores) + (size_t)t * num_experts * (BF16 ? 2 : 4);
  float m = -INFINITY;
  for (int e = lane; e < num_experts; e += 64) m = fmaxf(m, score_at<BF16>(row, e));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  float sum = 0.f;
  for (int e = lane; e < num_experts; e += 64) sum += expf(score_at<BF16>(row, e) - m);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  float* p = probs + (size_t)t * num_experts;
  for (int e = lane; e < num_experts; e += 64) p[e] = expf(score_at<BF16>(row, e) - m) / sum;
  int taken[kTopKMax];  // fixed trip counts below keep it in registers
#pragma unroll
  for (int k = 0; k < kTopKMax; ++k) taken[k] = -1;
#pragma unroll
  for (int k = 0; k < kTopKMax; ++k) {
    if (k >= top_k) break;
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < num_experts; e += 64) {
      bool free_ = true;
#pragma unroll
      for (int j = 0; j < kTopKMax; ++j) free_ = free_ && taken[j] != e;
      const float v = score_at<BF16>(row, e);
      if (free_ && (at == 0x7fffffff || v > best)) {  // the first free expert of the lane, then only larger scores
        best = v;
        at = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) {
        best = ob;
        at = oa;
      }
    }
    taken[k] = at;  // the same in every lane
    if (lane == 0) {
      weights[(size_t)t * top_k + k] = expf(best - m) / sum;
      selected[(size_t)t * top_k + k] = at;
    }
  }
}

// grad_scores[t, j] = p_j * (g_j - sum_i g_i p_i) with g the gradient of the chosen weights scattered to their
// experts: the chain through the softmax for the top_k outputs of route_topk_kernel.
template <bool BF16>
__global__ __launch_bounds__(kRowWaves * 64) void route_topk_backward_kernel(const float* __restrict__ probs,
                                                                             const int64_t* __restrict__ selected,
                                                                             const float* __restrict__ grad_weights,
                                                                             int tokens, int num_experts, int top_k,
                                                                             void* __restrict__ grad_scores) {
  const int lane = threadIdx.x % 64;
  const int t = blockIdx.x * kRowWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  if (t >= tokens) return;
  const float* p = probs + (size_t)t * num_experts;
  int at[kTopKMax];
  float g[kTopKMax];
  float dot = 0.f;
#pragma unroll
  for (int k = 0; k < kTopKMax; ++k) {
    const bool used = k < top_k;
    at[k] = used ? (int)selected[(size_t)t * top_k + k] : -1;
    g[k] = used ? grad_weights[(size_t)t * top_k + k] : 0.f;
    if ((uint32_t)at[k] >= (uint32_t)num_experts) at[k] = -1, g[k] = 0.f;  // not an expert: no gradient
    if (at[k] >= 0) dot = __builtin_fmaf(g[k], p[at[k]], dot);
  }
  for (int e = lane; e < num_experts; e += 64) {
    float ge = 0.f;
#pragma unroll
    for (int k = 0; k < kTopKMax; ++k) ge += at[k] == e ? g[k] : 0.f;
    const float v = p[e] * (ge - dot);
    if constexpr (BF16) static_cast<uint16_t*>(grad_scores)[(size_t)t * num_experts + e] = (uint16_t)f32_to_bf16_bits(v);
    else static_cast<float*>(grad_scores)[(size_t)t * num_experts + e] = v;
  }
}

bool rows_vectorisable(const void* a, const void* b, int hidden) {
  return hidden % 8 == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
}

}  // namespace
}  // namespace fp8gmm

extern "C" {

size_t fp8gmm_route_workspace_bytes(int n, int num_experts) {
  if (n <= 0 || num_experts <= 0) return 0;
  const size_t chunks = ((size_t)n + fp8gmm::kRouteChunk - 1) / fp8gmm::kRouteChunk;
  return chunks * (size_t)num_experts * sizeof(int32_t);
}

int fp8gmm_route_sort(const int32_t* expert_of, int n, int num_experts, int32_t* bin_ids, int32_t* indices,
                      int32_t* inverse, int32_t* tokens_per_expert, int32_t* bins, void* workspace, void* stream) {
  using namespace fp8gmm;
  if (n < 0 || num_experts < 1 || num_experts > kRouteMaxExperts) return FP8GMM_ERR_BAD_ARGUMENT;
  if (workspace == nullptr && n > 0) return FP8GMM_ERR_NULL_POINTER;
  if (n > 0 && expert_of == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (n + kRouteChunk - 1) / kRouteChunk;
  int32_t* counts = static_cast<int32_t*>(workspace);
  if (chunks > 0)
    hipLaunchKernelGGL(route_count_kernel, dim3(chunks), dim3(64), 0, s, expert_of, n, num_experts, counts);
  // with an empty list the scan still writes the (all-zero) totals and bins
  if (chunks > 0 || tokens_per_expert != nullptr || bins != nullptr)
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(256), 0, s, counts, chunks, num_experts, tokens_per_expert,
                       bins);
  if (chunks > 0 && (bin_ids != nullptr || indices != nullptr || inverse != nullptr))
    hipLaunchKernelGGL(route_place_kernel, dim3(chunks), dim3(64), 0, s, expert_of, n, num_experts, counts, bin_ids,
                       indices, inverse);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_route_invert(const int32_t* indices, int n, int32_t* inverse, void* stream) {
  if (n < 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (n == 0) return FP8GMM_OK;
  if (indices == nullptr || inverse == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipLaunchKernelGGL(fp8gmm::route_invert_kernel, dim3((n + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), indices, n, inverse);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_route_topk(const void* scores, int scores_bf16, int tokens, int num_experts, int top_k, float* probs,
                      float* weights, int64_t* selected, void* stream) {
  using namespace fp8gmm;
  if (tokens < 0 || num_experts < 1 || top_k < 1 || top_k > kTopKMax || top_k > num_experts)
    return FP8GMM_ERR_BAD_ARGUMENT;
  if (tokens == 0) return FP8GMM_OK;
  if (scores == nullptr || probs == nullptr || weights == nullptr || selected == nullptr) return FP8GMM_ERR_NULL_POINTER;
  const dim3 grid((tokens + kRowWaves - 1) / kRowWaves), block(kRowWaves * 64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (scores_bf16)
    hipLaunchKernelGGL(route_topk_kernel<true>, grid, block, 0, s, scores, tokens, num_experts, top_k, probs, weights,
                       selected);
  else
    hipLaunchKernelGGL(route_topk_kernel<false>, grid, block, 0, s, scores, tokens, num_experts, top_k, probs, weights,
                       selected);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_route_topk_backward(const float* probs, const int64_t* selected, const float* grad_weights, int tokens,
                               int num_experts, int top_k, void* grad_scores, int grad_bf16, void* stream) {
  using namespace fp8gmm;
  if (tokens < 0 || num_experts < 1 || top_k < 1 || top_k > kTopKMax || top_k > num_experts)
    return FP8GMM_ERR_BAD_ARGUMENT;
  if (tokens == 0) return FP8GMM_OK;
  if (probs == nullptr || selected == nullptr || grad_weights == nullptr || grad_scores == nullptr)
    return FP8GMM_ERR_NULL_POINTER;
  const dim3 grid((tokens + kRowWaves - 1) / kRowWaves), block(kRowWaves * 64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (grad_bf16)
    hipLaunchKernelGGL(route_topk_backward_kernel<true>, grid, block, 0, s, probs, selected, grad_weights, tokens,
                       num_experts, top_k, grad_scores);
  else
    hipLaunchKernelGGL(route_topk_backward_kernel<false>, grid, block, 0, s, probs, selected, grad_weights, tokens,
                       num_experts, top_k, grad_scores);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_moe_gather(const void* x, const int32_t* indices, const float* weights, void* out, int rows_out,
                      int hidden, int top_k, void* stream) {
  using namespace fp8gmm;
  if (rows_out < 0 || hidden < 0 || top_k < 1 || rows_out % top_k != 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if ((int64_t)hidden * 2 > 0x7fffffff) return FP8GMM_ERR_BAD_SHAPE;
  if (rows_out == 0 || hidden == 0) return FP8GMM_OK;
  if (x == nullptr || indices == nullptr || out == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipLaunchKernelGGL(moe_gather_kernel, dim3((rows_out + kRowWaves - 1) / kRowWaves), dim3(kRowWaves * 64), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x), indices, weights,
                     static_cast<uint16_t*>(out), rows_out, hidden, top_k, (int)rows_vectorisable(x, out, hidden));
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_moe_scatter(const void* x, const int32_t* inverse, const float* weights, void* out, int tokens, int hidden,
                       int top_k, void* stream) {
  using namespace fp8gmm;
  if (tokens < 0 || hidden < 0 || top_k < 1 || (int64_t)tokens * top_k > 0x7fffffff) return FP8GMM_ERR_BAD_ARGUMENT;
  if ((int64_t)hidden * 2 > 0x7fffffff) return FP8GMM_ERR_BAD_SHAPE;
  if (tokens == 0 || hidden == 0) return FP8GMM_OK;
  if (x == nullptr || inverse == nullptr || out == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipLaunchKernelGGL(moe_scatter_kernel, dim3((tokens + kRowWaves - 1) / kRowWaves), dim3(kRowWaves * 64), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x), inverse, weights,
                     static_cast<uint16_t*>(out), tokens, hidden, top_k, (int)rows_vectorisable(x, out, hidden));
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_moe_scatter_wgrad(const void* x, const void* grad_out, const int32_t* indices, float* grad_w, int rows,
                             int hidden, int top_k, void* stream) {
  using namespace fp8gmm;
  if (rows < 0 || hidden < 0 || top_k < 1 || rows % top_k != 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if (rows == 0) return FP8GMM_OK;
  if (x == nullptr || grad_out == nullptr || indices == nullptr || grad_w == nullptr) return FP8GMM_ERR_NULL_POINTER;
  hipLaunchKernelGGL(moe_scatter_wgrad_kernel, dim3((rows + kRowWaves - 1) / kRowWaves), dim3(kRowWaves * 64), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x),
                     static_cast<const uint16_t*>(grad_out), indices, grad_w, rows, hidden, top_k,
                     (int)rows_vectorisable(x, grad_out, hidden));
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

int fp8gmm_moe_scatter_backward(const void* x, const void* grad_out, const int32_t* indices, const float* weights,
                                void* grad_x, float* grad_w, int rows, int hidden, int top_k, void* stream) {
  using namespace fp8gmm;
  if (rows < 0 || hidden < 0 || top_k < 1 || rows % top_k != 0) return FP8GMM_ERR_BAD_ARGUMENT;
  if ((int64_t)hidden * 2 > 0x7fffffff) return FP8GMM_ERR_BAD_SHAPE;
  if (rows == 0) return FP8GMM_OK;
  if (x == nullptr || grad_out == nullptr || indices == nullptr || weights == nullptr || grad_x == nullptr ||
      grad_w == nullptr)
    return FP8GMM_ERR_NULL_POINTER;
  if (!rows_vectorisable(x, grad_out, hidden) || !rows_vectorisable(grad_x, grad_x, hidden)) {
    // rows that 16-byte accesses cannot take: the two single-purpose kernels
    int rc = fp8gmm_moe_gather(grad_out, indices, weights, grad_x, rows, hidden, top_k, stream);
    if (rc != FP8GMM_OK) return rc;
    return fp8gmm_moe_scatter_wgrad(x, grad_out, indices, grad_w, rows, hidden, top_k, stream);
  }
  hipLaunchKernelGGL(moe_scatter_backward_kernel, dim3((rows + kRowWaves - 1) / kRowWaves), dim3(kRowWaves * 64), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x),
                     static_cast<const uint16_t*>(grad_out), indices, weights, static_cast<uint16_t*>(grad_x), grad_w,
                     rows, hidden, top_k);
  return hipGetLastError() == hipSuccess ? FP8GMM_OK : FP8GMM_ERR_LAUNCH;
}

}  // extern "C"
