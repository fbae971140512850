// What this GPU sustains with nothing in the way: a stream of fp16 MFMAs on random operands (the chip runs the prefill
// kernel at its power limit, so the clock it holds under matrix load, not the nominal one, bounds that kernel on a given
// box) and a plain streaming read of a large buffer (what the memory system delivers to a kernel that does nothing else).
// Measurement aids for bench.py: built into their own library, libls_ceiling.so, which the operators never load.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ls_ceiling.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kAcc = 16;  // independent accumulators per wave: no MFMA waits for another's result

// One workgroup of four waves (one per SIMD) per CU: the LDS array below leaves no room for a second one.  Every wave
// issues iters x 16 v_mfma_f32_16x16x32_f16 on four A and four B operands read once from `operands` (random fp16
// values), the same MFMA shape and operand kind as the prefill kernel's.
__global__ __launch_bounds__(256, 1) void mfma_stream_kernel(const u32x4* __restrict__ operands, float* __restrict__ sink, int iters) {
  __shared__ char one_workgroup_per_cu[96 * 1024];
  const int lane = threadIdx.x;
  one_workgroup_per_cu[lane * 384] = (char)lane;  // (the array is used, so it is allocated: one byte per lane, read back below)
  __syncthreads();
  u32x4 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = operands[(blockIdx.x * 8 + i) % 64 * 256 + lane];
    b[i] = operands[(blockIdx.x * 8 + 4 + i) % 64 * 256 + lane];
  }
  f32x4 acc[kAcc];
#pragma unroll
  for (int j = 0; j < kAcc; j++) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    // (from inline assembly with the accumulator tied to the destination: left to itself the compiler gives every
    // result of this shape a fresh register tuple and fills the loop with register moves)
    for (int j = 0; j < kAcc; j++) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j & 3]), "v"(b[j >> 2]));
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // (the last results are complete before anything reads them)
  f32x4 s = acc[0];
#pragma unroll
  for (int j = 1; j < kAcc; j++) s += acc[j];
  const float t = s[0] + s[1] + s[2] + s[3] + (float)one_workgroup_per_cu[((lane + 1) & 255) * 384];
  if (t == 1234.5678f) sink[blockIdx.x * 256 + lane] = t;  // (keeps the arithmetic; practically never taken)
}

// Reads n16 16-byte words once, non-temporal (nothing is read twice, as in the decode gather): a wave takes 8 KB at a
// time, its eight loads side by side (a kilobyte per load instruction), the waves of the grid side by side, then the
// next 8 KB a grid's width further on.  (The pattern matters: with the eight loads of a trip a grid's width apart instead,
// 16 MB at this grid, the same read runs 8 % slower, 6.4 instead of 7.0 TB/s.)
__global__ __launch_bounds__(256) void read_stream_kernel(const u32x4* __restrict__ src, uint64_t n16, uint32_t* __restrict__ sink) {
  const uint64_t waves = (uint64_t)gridDim.x * 4, wave = ((uint64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  const uint64_t chunks = n16 / 512;  // of 8 KB
  u32x4 x = {0, 0, 0, 0};
  for (uint64_t c = wave; c < chunks; c += waves) {
    u32x4 w[8];
#pragma unroll
    for (int u = 0; u < 8; u++) w[u] = __builtin_nontemporal_load(src + c * 512 + u * 64 + lane);
#pragma unroll
    for (int u = 0; u < 8; u++) x ^= w[u];
  }
  for (uint64_t i = chunks * 512 + (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256) x ^= __builtin_nontemporal_load(src + i);
  if ((x[0] ^ x[1] ^ x[2] ^ x[3]) == 0x9e3779b9u) sink[threadIdx.x] = x[0];  // (keeps the loads; practically never taken)
}

// The same read with stores mixed in, as a split-K decode mixes its partials into its gather: in one of every `every`
// trips (spread evenly over the waves and over the launch) the wave also writes 8 KB, as sixteen rows of 512 bytes of
// which a store instruction writes a 64-byte piece each (the shape of a partial's row stores).  SYSTEM: the stores carry
// the system-scope bits (sc0 sc1: written through to memory as they are issued) instead of waiting in the L2 as dirty
// lines that are written back later.
template <bool SYSTEM>
__global__ __launch_bounds__(256) void read_with_stores_kernel(const u32x4* __restrict__ src, uint64_t n16, u32x4* __restrict__ dst, uint32_t every,
                                                               uint32_t* __restrict__ sink) {
  const uint64_t waves = (uint64_t)gridDim.x * 4, wave = ((uint64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  const uint64_t chunks = n16 / 512;  // of 8 KB: trip c of the grid's waves reads chunk c
  u32x4 x = {0, 0, 0, 0};
  for (uint64_t c = wave; c < chunks; c += waves) {
    u32x4 w[8];
#pragma unroll
    for (int u = 0; u < 8; u++) w[u] = __builtin_nontemporal_load(src + c * 512 + u * 64 + lane);
#pragma unroll
    for (int u = 0; u < 8; u++) x ^= w[u];
    // (chunk numbers scrambled, so that the trips that store are spread over the waves and over the launch)
    const uint64_t event = (c * 0x9E3779B1ull) % chunks;
    if (event % every == 0) {
      u32x4* base = dst + (event / every) * 512 + (lane & 15) * 32 + (lane >> 4);  // 8 KB = 512 x 16 B per event
#pragma unroll
      for (int u = 0; u < 8; u++) {
        // (a vector instruction may not overwrite the data of a store of more than 64 bits in the two cycles behind it)
        if (SYSTEM) asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(base + 4 * u), "v"(x) : "memory");
        else asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" : : "v"(base + 4 * u), "v"(x) : "memory");
      }
    }
  }
  for (uint64_t i = chunks * 512 + (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256) x ^= __builtin_nontemporal_load(src + i);
  if ((x[0] ^ x[1] ^ x[2] ^ x[3]) == 0x9e3779b9u) sink[threadIdx.x] = x[0];  // (keeps the loads; practically never taken)
}

}  // namespace

extern "C" int ls_ceiling_mfma_f16(const void* operands, void* sink, int iters, int workgroups, void* stream) {
  if (!operands || !sink || iters < 1 || workgroups < 1 || ((uintptr_t)operands & 15)) return -1;
  (void)hipGetLastError();  // (an earlier call of the host program may have left an error that is not this launch's)
  hipLaunchKernelGGL(mfma_stream_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, (const u32x4*)operands,
                     (float*)sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" double ls_ceiling_mfma_f16_flop(int iters, int workgroups) {
  return (double)workgroups * 4 /* waves */ * (double)iters * kAcc * (2.0 * 16 * 16 * 32);
}

extern "C" int ls_ceiling_read(const void* src, uint64_t bytes, void* sink, void* stream) {
  if (!src || !sink || bytes < 16 || ((uintptr_t)src & 15)) return -1;
  (void)hipGetLastError();  // (an earlier call of the host program may have left an error that is not this launch's)
  hipLaunchKernelGGL(read_stream_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, bytes / 16, (uint32_t*)sink);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" uint64_t ls_ceiling_read_with_stores_bytes(uint64_t bytes, uint32_t every) {
  if (every < 1) return 0;
  const uint64_t chunks = bytes / 8192;  // (events are numbered below `chunks`; every `every`-th of them stores 8 KB)
  return ((chunks + every - 1) / every + 1) * 8192;
}

extern "C" int ls_ceiling_read_with_stores(const void* src, uint64_t bytes, void* dst, uint32_t every, int system_scope, void* sink, void* stream) {
  if (!src || !dst || !sink || bytes < 16 || every < 1 || (((uintptr_t)src | (uintptr_t)dst) & 15)) return -1;
  (void)hipGetLastError();  // (an earlier call of the host program may have left an error that is not this launch's)
  if (system_scope)
    hipLaunchKernelGGL(read_with_stores_kernel<true>, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, bytes / 16, (u32x4*)dst,
                       every, (uint32_t*)sink);
  else
    hipLaunchKernelGGL(read_with_stores_kernel<false>, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, bytes / 16, (u32x4*)dst,
                       every, (uint32_t*)sink);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
