// Read rate of the LDS for the fragment reads of the grouped GEMM, measured in isolation: plain 16-byte reads
// (ds_read_b128, the row-major operand path), plain 8-byte reads and transposing 8-byte reads (ds_read_b64_tr_b8,
// the contraction-major operand path), at the kernel's own address patterns (conflict-free by construction).
// One workgroup per compute unit, 1, 2 or 4 wavefronts (one per SIMD); every wavefront issues 16 independent
// reads, waits for them, and repeats.  Part of libfp8gmm_probe.so, used by `bench.py --workload lds_rate` only.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
constexpr int kLdsBytes = 65536;

#define FP8GMM_READ16(instr, o0, o1, o2, o3, o4, o5, o6, o7, o8, o9, o10, o11, o12, o13, o14, o15)                   \
  asm volatile(instr " %0, %16 offset:" #o0 "\n\t" instr " %1, %16 offset:" #o1 "\n\t" instr " %2, %16 offset:" #o2   \
               "\n\t" instr " %3, %16 offset:" #o3 "\n\t" instr " %4, %16 offset:" #o4 "\n\t" instr                    \
               " %5, %16 offset:" #o5 "\n\t" instr " %6, %16 offset:" #o6 "\n\t" instr " %7, %16 offset:" #o7 "\n\t"   \
               instr " %8, %16 offset:" #o8 "\n\t" instr " %9, %16 offset:" #o9 "\n\t" instr " %10, %16 offset:" #o10  \
               "\n\t" instr " %11, %16 offset:" #o11 "\n\t" instr " %12, %16 offset:" #o12 "\n\t" instr                \
               " %13, %16 offset:" #o13 "\n\t" instr " %14, %16 offset:" #o14 "\n\t" instr " %15, %16 offset:" #o15    \
               "\n\ts_waitcnt lgkmcnt(0)"                                                                              \
               : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]),            \
                 "=&v"(x[7]), "=&v"(x[8]), "=&v"(x[9]), "=&v"(x[10]), "=&v"(x[11]), "=&v"(x[12]), "=&v"(x[13]),        \
                 "=&v"(x[14]), "=&v"(x[15])                                                                            \
               : "v"(addr)                                                                                             \
               : "memory")

// MODE 0: ds_read_b128 at the row-major fragment addresses (row l32 of a 128-byte-pitch unit, chunk swizzled with
// (row >> 1) & 7); 1: ds_read_b64 and 2: ds_read_b64_tr_b8 at the contraction-major fragment addresses (8 rows of
// a 256-byte-pitch unit per 16 lanes, chunk swizzled with 2 (row mod 8)).
template <int MODE>
__global__ __launch_bounds__(256) void lds_rate_kernel(uint32_t* __restrict__ sink, long long* __restrict__ cycles,
                                                       int iters) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  for (int i = threadIdx.x; i < kLdsBytes / 4; i += blockDim.x) reinterpret_cast<uint32_t*>(lds)[i] = i * 2654435761u;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, khalf = lane >> 5;
  uint32_t addr;
  if (MODE == 0) {
    addr = (uint32_t)(uintptr_t)lds + ((wave & 1) * 128 + l32) * 128 + (((2 * khalf) ^ ((l32 >> 1) & 7)) << 4);
  } else {
    const int tr_b = (lane & 15) >> 1, tr_h = lane & 1, tr_g = (lane >> 4) & 1;
    addr = (uint32_t)(uintptr_t)lds + (32 * khalf + tr_b) * 256 + 8 * tr_h + ((((wave & 1) * 8 + tr_g) ^ (2 * tr_b)) << 4);
  }
  uint32_t s = 0;
  __syncthreads();
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {   // largest offset 12288 + 48 + 16 bytes past row 255 of the unit: inside the 64 KiB
      u32x4 x[16];
      FP8GMM_READ16("ds_read_b128", 0, 4096, 8192, 12288, 16, 4112, 8208, 12304, 32, 4128, 8224, 12320, 48, 4144, 8240, 12336);
#pragma unroll
      for (int i = 0; i < 16; ++i) s += x[i].x;
    } else if (MODE == 1) {
      u32x2 x[16];
      FP8GMM_READ16("ds_read_b64", 0, 2048, 4096, 6144, 32, 2080, 4128, 6176, 64, 2112, 4160, 6208, 96, 2144, 4192, 6240);
#pragma unroll
      for (int i = 0; i < 16; ++i) s += x[i].x;
    } else {
      u32x2 x[16];
      FP8GMM_READ16("ds_read_b64_tr_b8", 0, 2048, 4096, 6144, 32, 2080, 4128, 6176, 64, 2112, 4160, 6208, 96, 2144, 4192, 6240);
#pragma unroll
      for (int i = 0; i < 16; ++i) s += x[i].x;
    }
  }
  const long long t1 = clock64();
  sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
}

}  // namespace

// mode 0 / 1 / 2 as above; waves: 1, 2 or 4 per workgroup; every wavefront issues iters x 16 reads.
// sink: blocks x 64 x waves uint32 (never read); cycles: blocks int64, the shader-clock cycles of each workgroup's
// loop.  Returns 0, a HIP error code, or -1 for arguments out of range.
extern "C" int fp8gmm_probe_lds(int mode, int waves, int iters, void* sink, void* cycles, int blocks, void* stream) {
  if (mode < 0 || mode > 2 || (waves != 1 && waves != 2 && waves != 4) || iters <= 0 || blocks <= 0 || sink == nullptr ||
      cycles == nullptr)
    return -1;
  auto st = static_cast<hipStream_t>(stream);
  auto sk = static_cast<uint32_t*>(sink);
  auto cy = static_cast<long long*>(cycles);
  const dim3 grid(blocks), block(64 * waves);
  if (mode == 0) lds_rate_kernel<0><<<grid, block, kLdsBytes, st>>>(sk, cy, iters);
  else if (mode == 1) lds_rate_kernel<1><<<grid, block, kLdsBytes, st>>>(sk, cy, iters);
  else lds_rate_kernel<2><<<grid, block, kLdsBytes, st>>>(sk, cy, iters);
  return (int)hipGetLastError();
}
