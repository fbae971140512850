// Shared device helpers for the gfx950 attention kernels (wave64 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "lsattn.h"

namespace lsattn {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));

struct F16 {};   // element tag: IEEE half
struct BF16 {};  // element tag: bfloat16

// two packed 16-bit elements -> two floats
template <typename T> __device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi);
template <> __device__ __forceinline__ void unpack2<F16>(uint32_t w, float& lo, float& hi) {
  f16x2 h = __builtin_bit_cast(f16x2, w);
  lo = (float)h[0];
  hi = (float)h[1];
}
template <> __device__ __forceinline__ void unpack2<BF16>(uint32_t w, float& lo, float& hi) {
  lo = __builtin_bit_cast(float, w << 16);
  hi = __builtin_bit_cast(float, w & 0xffff0000u);
}

// two floats -> two packed 16-bit elements, round to nearest even
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<F16>(float lo, float hi) {
  f16x2 h = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, h);
}
template <> __device__ __forceinline__ uint32_t pack2<BF16>(float lo, float hi) {
  f32x2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));  // v_cvt_pk_bf16_f32, RNE
}

// 8 packed elements (one 16-byte load) -> 8 floats
template <typename T> __device__ __forceinline__ void unpack8(const u32x4& w, float* f) {
  unpack2<T>(w[0], f[0], f[1]);
  unpack2<T>(w[1], f[2], f[3]);
  unpack2<T>(w[2], f[4], f[5]);
  unpack2<T>(w[3], f[6], f[7]);
}

template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// butterfly sum over each aligned group of 16 lanes; every lane ends with the total
__device__ __forceinline__ float sum_row16(float v) {
  v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_mov<0x141>(v);  // row_half_mirror
  v += dpp_mov<0x140>(v);  // row_mirror
  return v;
}

// exp2 that maps (-inf) - (-inf) to 0 instead of NaN
__device__ __forceinline__ float exp2_diff(float a, float b) {
  return (a == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(a - b);
}

// The launch choices of lsattn_set_tuning (0 = the library's own); defined in merge_scatter.hip.
struct Tuning {
  int prefill_rows, prefill_order, prefill_pack, decode_stage1, decode_listed;
};
Tuning tuning();

// The prefill step for head sizes 16, 32 and 64 (prefill_small.hip); `mode`: 0 fp32 partial, 1 in-place (o, m, l), 2 merge into a
// running fp32 partial.  Arguments validated by the caller.
int launch_prefill_small(const lsattn_prefill_args* a, int mode, hipStream_t st);

// check_launch reports what the launch in front of it left in the host thread's last-error slot, so every launch first
// empties that slot: an earlier runtime call of the host program may have left something there that is not this
// library's to report (hipEventQuery's "not ready", which a framework's copy engine polls with, among them).
#define LSATTN_LAUNCH_KERNEL(...)   \
  do {                              \
    (void)hipGetLastError();        \
    hipLaunchKernelGGL(__VA_ARGS__); \
  } while (0)
inline int check_launch() { return hipGetLastError() == hipSuccess ? LSATTN_OK : LSATTN_ERR_LAUNCH; }

}  // namespace lsattn
