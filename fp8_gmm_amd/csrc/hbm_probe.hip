// Plain streaming kernels that measure what the memory system of one MI355X sustains for a given mix of reads and
// writes.  They do no arithmetic worth the name, so their rate is the ceiling that the cast / transpose / pad
// kernels of the library can be priced against.  Built into its own small library (libfp8gmm_probe.so), used by
// `bench.py --workload hbm_ceiling` only; the product library does not contain or need them.
//
//   mode 0  read only       : `reads` streams of 16-byte loads, reduced to one word per thread that is never stored
//   mode 1  n reads : 1 write: `reads` input streams folded into one output stream of the same length
//   mode 2  write only      : one output stream
//
// A stream is a contiguous array of `bytes_per_stream` bytes; stream r of the input starts at src + r * bytes.
// Every workgroup walks the arrays with a grid stride, each thread moving 16 bytes per access and UNROLL accesses
// per trip (a wavefront access covers 1 KiB of consecutive addresses).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;

// BLOCKED: the UNROLL accesses of a trip cover UNROLL x 4 KiB of consecutive addresses per workgroup (a workgroup
// owns contiguous 16 KiB pieces); otherwise they are a whole grid apart (every access of the grid is one window).
template <int READS, bool WRITE, bool NT, int UNROLL, bool BLOCKED>
__global__ __launch_bounds__(kThreads) void stream_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                          int64_t vecs_per_stream, uint32_t never) {
  const int64_t stride = BLOCKED ? kThreads : (int64_t)gridDim.x * kThreads;
  const int64_t trip = (int64_t)gridDim.x * kThreads * UNROLL;
  const int64_t first = BLOCKED ? (int64_t)blockIdx.x * kThreads * UNROLL + threadIdx.x
                                : (int64_t)blockIdx.x * kThreads + threadIdx.x;
  u32x4 keep = {0, 0, 0, 0};
  for (int64_t base = first; base < vecs_per_stream; base += trip) {
    u32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      v[u] = u32x4{0, 0, 0, 0};
      const int64_t i = base + u * stride;
      if (i < vecs_per_stream) {
#pragma unroll
        for (int r = 0; r < READS; ++r) {
          const u32x4* p = src + r * vecs_per_stream + i;
          v[u] ^= NT ? __builtin_nontemporal_load(p) : *p;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t i = base + u * stride;
      if (WRITE) {
        if (i < vecs_per_stream) {
          if (READS == 0) v[u] = u32x4{(uint32_t)i, 1u, 2u, 3u};
          if (NT) __builtin_nontemporal_store(v[u], dst + i); else dst[i] = v[u];
        }
      } else {
        keep ^= v[u];
      }
    }
  }
  // `never` is a value no fold of the data produces in practice: the loads stay live, nothing is written
  if (!WRITE && (keep.x ^ keep.y ^ keep.z ^ keep.w) == never && never == 0x9e3779b9u) dst[threadIdx.x] = keep;
}

template <int READS, bool WRITE>
int launch(int nt_blocked, const void* src, void* dst, int64_t vecs, int blocks, hipStream_t stream) {
  auto s = static_cast<const u32x4*>(src);
  auto d = static_cast<u32x4*>(dst);
  const bool blocked = (nt_blocked & 2) != 0, nt = (nt_blocked & 1) != 0;
  if (blocked) {
    if (nt) stream_kernel<READS, WRITE, true, 4, true><<<blocks, kThreads, 0, stream>>>(s, d, vecs, 0x9e3779b9u);
    else stream_kernel<READS, WRITE, false, 4, true><<<blocks, kThreads, 0, stream>>>(s, d, vecs, 0x9e3779b9u);
  } else {
    if (nt) stream_kernel<READS, WRITE, true, 4, false><<<blocks, kThreads, 0, stream>>>(s, d, vecs, 0x9e3779b9u);
    else stream_kernel<READS, WRITE, false, 4, false><<<blocks, kThreads, 0, stream>>>(s, d, vecs, 0x9e3779b9u);
  }
  return (int)hipGetLastError();
}

}  // namespace

// reads: input streams (0 with write = 1: write only); write: 0 or 1; nontemporal: bit 0 = streaming hint on
// every access, bit 1 = blocked walk (see stream_kernel).
// Returns 0, a HIP error code, or -1 for a combination that is not built.
extern "C" int fp8gmm_probe_stream(int reads, int write, int nontemporal, const void* src, void* dst,
                                   int64_t bytes_per_stream, int blocks, void* stream) {
  if (bytes_per_stream <= 0 || (bytes_per_stream & 15) != 0 || blocks <= 0) return -1;
  const int64_t vecs = bytes_per_stream / 16;
  auto st = static_cast<hipStream_t>(stream);
  const int nt = nontemporal;
  if (write == 0) {
    if (reads == 1) return launch<1, false>(nt, src, dst, vecs, blocks, st);
    if (reads == 2) return launch<2, false>(nt, src, dst, vecs, blocks, st);
    return -1;
  }
  switch (reads) {
    case 0: return launch<0, true>(nt, src, dst, vecs, blocks, st);
    case 1: return launch<1, true>(nt, src, dst, vecs, blocks, st);
    case 2: return launch<2, true>(nt, src, dst, vecs, blocks, st);
    case 4: return launch<4, true>(nt, src, dst, vecs, blocks, st);
    default: return -1;
  }
}
