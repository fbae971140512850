// The element-wise steps around attention in the reference's extension module, for gfx950:
//   rms_norm              (longserve_cuda_kernels/src/rms_norm.cu:10-62)
//   silu_and_mul_inplace  (longserve_cuda_kernels/src/silu_and_mul.cu:12-49)
//   rotary_emb            (longserve_cuda_kernels/src/rotary_emb.cu:10-55)
// All three are HBM-bound fp16 streams: 16 bytes per lane and access, every input byte read once.
#include "common.hip.h"

namespace lsattn {

// ---------------------------------------------------------------------------------------------------
// rms_norm: out[t, i] = half(float(x[t, i]) * float(w[i]) * inv_rms[t]),  inv_rms = rsqrt(sum x^2 / H + eps),
// the product in the reference's order (rms_norm.cu:42-45).  One wave per token row; a row of up to
// 64 * 8 * kRmsChunks elements stays in registers between the two passes, longer rows are read twice.
// ---------------------------------------------------------------------------------------------------
constexpr int kRmsChunks = 16;  // 16-byte pieces per lane held in registers: rows up to 8192 elements

__device__ __forceinline__ float wave_sum(float v) {
  v = sum_row16(v);
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

__global__ __launch_bounds__(256) void rms_norm_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ in,
                                                       const uint16_t* __restrict__ weight, int64_t num_tokens, int64_t hidden,
                                                       float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= num_tokens) return;
  const int64_t pieces = hidden / 8;  // 16-byte pieces in a row
  const u32x4* row = (const u32x4*)(in + t * hidden);
  const u32x4* wrow = (const u32x4*)weight;
  u32x4* orow = (u32x4*)(out + t * hidden);
  const bool cached = pieces <= 64 * kRmsChunks;
  u32x4 keep[kRmsChunks];
  float ss = 0.f;
  if (cached) {
#pragma unroll
    for (int c = 0; c < kRmsChunks; c++) {
      const int64_t i = lane + 64 * c;
      keep[c] = i < pieces ? row[i] : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int c = 0; c < kRmsChunks; c++) {
      float f[8];
      unpack8<F16>(keep[c], f);
#pragma unroll
      for (int e = 0; e < 8; e++) ss = __builtin_fmaf(f[e], f[e], ss);
    }
  } else {
    for (int64_t i = lane; i < pieces; i += 64) {
      float f[8];
      unpack8<F16>(row[i], f);
#pragma unroll
      for (int e = 0; e < 8; e++) ss = __builtin_fmaf(f[e], f[e], ss);
    }
  }
  ss = wave_sum(ss);
  const float inv_rms = __builtin_amdgcn_rsqf(ss / (float)hidden + eps);
  auto scale_piece = [&](const u32x4& x, const u32x4& w) {
    float a[8], b[8];
    unpack8<F16>(x, a);
    unpack8<F16>(w, b);
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = pack2<F16>(a[2 * e] * b[2 * e] * inv_rms, a[2 * e + 1] * b[2 * e + 1] * inv_rms);
    return r;
  };
  if (cached) {
#pragma unroll
    for (int c = 0; c < kRmsChunks; c++) {
      const int64_t i = lane + 64 * c;
      if (i < pieces) orow[i] = scale_piece(keep[c], wrow[i]);
    }
  } else {
    for (int64_t i = lane; i < pieces; i += 64) orow[i] = scale_piece(row[i], wrow[i]);
  }
}

// ---------------------------------------------------------------------------------------------------
// silu_and_mul_inplace: io[t, i] = half(silu(io[t, i])) * io[t, I + i] for i < I, the second half of the row untouched;
// silu in fp32, rounded to half, then a half multiply (silu_and_mul.cu:14-17, :30-33).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void silu_and_mul_kernel(uint16_t* __restrict__ io, int64_t num_tokens, int64_t inter) {
  const int64_t pieces_per_row = inter / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= num_tokens * pieces_per_row) return;
  const int64_t t = gid / pieces_per_row, i = gid % pieces_per_row;
  // (whole rows of eight halves: picking 32-bit words out of an integer vector and bit-casting them to half
  // pairs made this compiler read word 0 every time)
  f16x8* gate = (f16x8*)(io + t * 2 * inter) + i;
  const f16x8 g = *gate;
  const f16x8 u = *((const f16x8*)(io + t * 2 * inter + inter) + i);
  f16x8 r;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    const float x = (float)g[e];
    const _Float16 sl = (_Float16)(x / (1.f + __builtin_amdgcn_exp2f(-x * kLog2e)));
    r[e] = sl * u[e];  // half multiply, round to nearest even
  }
  *gate = r;
}

// ---------------------------------------------------------------------------------------------------
// rotary_emb, in place on x[t, h, :] (last dimension contiguous), in the reference's half arithmetic (rotary_emb.cu:30-33):
//   new_x1 = fma(x1, cos, -(x2 * sin)),  new_x2 = fma(x1, sin, x2 * cos)   with x1 = x[..., :D/2], x2 = x[..., D/2:],
// every product and fma rounded to half once.  A lane owns 8 elements of x1 and the matching 8 of x2.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rotary_emb_kernel(uint16_t* __restrict__ x, const uint16_t* __restrict__ cos_t,
                                                         const uint16_t* __restrict__ sin_t, int64_t stride_t, int64_t stride_h,
                                                         int64_t num_tokens, int64_t num_heads, int64_t head_dim) {
  const int64_t pieces = head_dim / 16;  // 16-byte pieces in half a head
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= num_tokens * num_heads * pieces) return;
  const int64_t c = gid % pieces;
  const int64_t h = (gid / pieces) % num_heads;
  const int64_t t = gid / (pieces * num_heads);
  uint16_t* base = x + t * stride_t + h * stride_h;
  f16x8* p1 = (f16x8*)base + c;
  f16x8* p2 = (f16x8*)(base + head_dim / 2) + c;
  const f16x8 x1 = *p1, x2 = *p2;
  const f16x8 co = *((const f16x8*)(cos_t + t * (head_dim / 2)) + c);
  const f16x8 si = *((const f16x8*)(sin_t + t * (head_dim / 2)) + c);
  const f16x8 t1 = x2 * si, t2 = x2 * co;  // rounded to half (this file is compiled without contraction)
  f16x8 n1, n2;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    n1[e] = __builtin_fmaf16(x1[e], co[e], -t1[e]);
    n2[e] = __builtin_fmaf16(x1[e], si[e], t2[e]);
  }
  *p1 = n1;
  *p2 = n2;
}

// ---------------------------------------------------------------------------------------------------
// The write-back of a step's new tokens in one launch: rotary embedding of q and of the K heads in place (the arithmetic
// of rotary_emb_kernel), every token's rotated K heads and its V heads copied to the token's slot of the KV pool, and the
// slots entered in the request table.  A unit is 32 bytes of one (token, head): the two 16-byte halves a rotary lane
// owns, or two consecutive 16-byte pieces of a V head.  Blocks past the data units do the registration, one table entry
// per lane.
// ---------------------------------------------------------------------------------------------------
struct RotaryWriteParams {
  uint16_t* q;
  int64_t q_st, q_sh, hq;
  uint16_t* kv;
  int64_t kv_st, kv_sh, hkv;
  const uint16_t* cos_t;
  const uint16_t* sin_t;
  int64_t num_tokens, head_dim;
  uint16_t* pool;
  int64_t pool_stride;  // elements per slot
  const int32_t* dest;
  int32_t* req_to_tokens;
  int64_t max_seq_len;
  const int32_t* b_req_idx;
  const int32_t* b_start_loc;
  const int32_t* b_seq_len;
  int64_t batch, data_blocks, reg_blocks_per_req;
  int32_t reg_mode;  // 0 none, 1 every token of every request (prefill), 2 the last token of every request (decode)
};

__global__ __launch_bounds__(256) void rotary_kv_write_kernel(RotaryWriteParams p) {
  if ((int64_t)blockIdx.x >= p.data_blocks) {
    const int64_t rb = (int64_t)blockIdx.x - p.data_blocks;
    if (p.reg_mode == 1) {
      const int64_t b = rb / p.reg_blocks_per_req;
      const int64_t j = (rb % p.reg_blocks_per_req) * 256 + threadIdx.x;
      if (j >= p.b_seq_len[b] || j >= p.max_seq_len) return;
      p.req_to_tokens[(int64_t)p.b_req_idx[b] * p.max_seq_len + j] = p.dest[(int64_t)p.b_start_loc[b] + j];
    } else {
      const int64_t i = rb * 256 + threadIdx.x;
      if (i >= p.batch) return;
      const int64_t pos = (int64_t)p.b_seq_len[i] - 1;
      if (pos < 0 || pos >= p.max_seq_len) return;
      p.req_to_tokens[(int64_t)p.b_req_idx[i] * p.max_seq_len + pos] = p.dest[i];
    }
    return;
  }
  const int64_t pieces = p.head_dim / 16;  // units per head
  const int64_t heads = p.hq + 2 * p.hkv;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= p.num_tokens * heads * pieces) return;
  const int64_t c = gid % pieces;
  const int64_t h = (gid / pieces) % heads;
  const int64_t t = gid / (pieces * heads);
  if (h >= p.hq + p.hkv) {
    // V head: 32 bytes to the pool
    if (!p.pool) return;
    const int64_t hv = h - p.hq;  // head index inside the token's K/V row
    const f16x8* src = (const f16x8*)(p.kv + t * p.kv_st + hv * p.kv_sh) + 2 * c;
    f16x8* dst = (f16x8*)(p.pool + (int64_t)p.dest[t] * p.pool_stride + hv * p.head_dim) + 2 * c;
    const f16x8 a = src[0], b = src[1];
    dst[0] = a;
    dst[1] = b;
    return;
  }
  const bool is_k = h >= p.hq;
  uint16_t* base = is_k ? p.kv + t * p.kv_st + (h - p.hq) * p.kv_sh : p.q + t * p.q_st + h * p.q_sh;
  f16x8* p1 = (f16x8*)base + c;
  f16x8* p2 = (f16x8*)(base + p.head_dim / 2) + c;
  const f16x8 x1 = *p1, x2 = *p2;
  const f16x8 co = *((const f16x8*)(p.cos_t + t * (p.head_dim / 2)) + c);
  const f16x8 si = *((const f16x8*)(p.sin_t + t * (p.head_dim / 2)) + c);
  const f16x8 t1 = x2 * si, t2 = x2 * co;  // rounded to half (this file is compiled without contraction)
  f16x8 n1, n2;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    n1[e] = __builtin_fmaf16(x1[e], co[e], -t1[e]);
    n2[e] = __builtin_fmaf16(x1[e], si[e], t2[e]);
  }
  *p1 = n1;
  *p2 = n2;
  if (is_k && p.pool) {
    uint16_t* prow = p.pool + (int64_t)p.dest[t] * p.pool_stride + (h - p.hq) * p.head_dim;
    *((f16x8*)prow + c) = n1;
    *((f16x8*)(prow + p.head_dim / 2) + c) = n2;
  }
}

// ---------------------------------------------------------------------------------------------------
// bf16 -> fp16 row copy, rounded toward zero (exact inside fp16's normal range, +-65504 beyond it): prepares a bf16 V
// for the prefill kernel, whose P V product runs in fp16.  One 16-byte piece per lane.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void bf16_to_f16_rows_kernel(const uint16_t* __restrict__ src, int64_t src_stride,
                                                               uint16_t* __restrict__ dst, int64_t dst_stride, int64_t n_rows,
                                                               int64_t pieces_per_row) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= n_rows * pieces_per_row) return;
  const int64_t r = gid / pieces_per_row, c = gid % pieces_per_row;
  const u32x4 w = *((const u32x4*)(src + r * src_stride) + c);
  u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float lo, hi;
    unpack2<BF16>(w[i], lo, hi);
    o[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
  *((u32x4*)(dst + r * dst_stride) + c) = o;
}

}  // namespace lsattn

using namespace lsattn;

extern "C" int lsattn_bf16_to_f16_rows(const void* src, int64_t src_stride, void* dst, int64_t dst_stride, int64_t n_rows,
                                       int64_t row_elems, void* stream) {
  if (!src || !dst || n_rows < 0 || row_elems <= 0) return LSATTN_ERR_INVALID_ARG;
  if (row_elems % 8 || src_stride % 8 || dst_stride % 8 || src_stride < row_elems || dst_stride < row_elems ||
      (((uintptr_t)src | (uintptr_t)dst) & 15))
    return LSATTN_ERR_INVALID_ARG;
  if (n_rows == 0) return LSATTN_OK;
  const int64_t blocks = (n_rows * (row_elems / 8) + 255) / 256;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(bf16_to_f16_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)src,
                     src_stride, (uint16_t*)dst, dst_stride, n_rows, row_elems / 8);
  return check_launch();
}

extern "C" int lsattn_rms_norm(void* out, const void* in, const void* weight, int64_t num_tokens, int64_t hidden_size,
                               float eps, void* stream) {
  if (!out || !in || !weight || num_tokens < 0 || hidden_size <= 0) return LSATTN_ERR_INVALID_ARG;
  if (hidden_size % 8 || (((uintptr_t)out | (uintptr_t)in | (uintptr_t)weight) & 15)) return LSATTN_ERR_INVALID_ARG;
  if (num_tokens == 0) return LSATTN_OK;
  const int64_t blocks = (num_tokens + 3) / 4;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(rms_norm_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                     (const uint16_t*)in, (const uint16_t*)weight, num_tokens, hidden_size, eps);
  return check_launch();
}

extern "C" int lsattn_silu_and_mul_inplace(void* io, int64_t num_tokens, int64_t ffn_inter_dim, void* stream) {
  if (!io || num_tokens < 0 || ffn_inter_dim <= 0) return LSATTN_ERR_INVALID_ARG;
  if (ffn_inter_dim % 8 || ((uintptr_t)io & 15)) return LSATTN_ERR_INVALID_ARG;
  if (num_tokens == 0) return LSATTN_OK;
  const int64_t blocks = (num_tokens * (ffn_inter_dim / 8) + 255) / 256;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(silu_and_mul_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)io, num_tokens,
                     ffn_inter_dim);
  return check_launch();
}

extern "C" int lsattn_rotary_emb(void* x, const void* cos, const void* sin, int64_t x_stride_t, int64_t x_stride_h,
                                 int64_t num_tokens, int64_t num_heads, int64_t head_dim, void* stream) {
  if (!x || !cos || !sin || num_tokens < 0 || num_heads <= 0 || head_dim <= 0) return LSATTN_ERR_INVALID_ARG;
  if (head_dim % 16 || x_stride_t % 8 || x_stride_h % 8 || (((uintptr_t)x | (uintptr_t)cos | (uintptr_t)sin) & 15))
    return LSATTN_ERR_INVALID_ARG;
  if (num_tokens == 0) return LSATTN_OK;
  const int64_t blocks = (num_tokens * num_heads * (head_dim / 16) + 255) / 256;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(rotary_emb_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)x,
                     (const uint16_t*)cos, (const uint16_t*)sin, x_stride_t, x_stride_h, num_tokens, num_heads, head_dim);
  return check_launch();
}

extern "C" int lsattn_rotary_kv_write(const lsattn_rotary_kv_write_args* a, void* stream) {
  if (!a || !a->q || !a->kv || !a->cos || !a->sin || a->num_tokens < 0 || a->num_q_heads <= 0 || a->num_kv_heads <= 0 ||
      a->head_dim <= 0 || a->batch < 0)
    return LSATTN_ERR_INVALID_ARG;
  if (a->head_dim % 16 || a->q_stride_t % 8 || a->q_stride_h % 8 || a->kv_stride_t % 8 || a->kv_stride_h % 8 ||
      (((uintptr_t)a->q | (uintptr_t)a->kv | (uintptr_t)a->cos | (uintptr_t)a->sin | (uintptr_t)a->pool) & 15))
    return LSATTN_ERR_INVALID_ARG;
  if (a->pool && (!a->dest_index || a->pool_slot_stride % 8 || a->pool_slot_stride < 2 * a->num_kv_heads * a->head_dim))
    return LSATTN_ERR_INVALID_ARG;
  if (a->register_mode < 0 || a->register_mode > 2) return LSATTN_ERR_INVALID_ARG;
  if (a->register_mode != 0 &&
      (!a->req_to_tokens || !a->dest_index || !a->b_req_idx || !a->b_seq_len || a->max_seq_len <= 0 ||
       (a->register_mode == 1 && (!a->b_start_loc || a->max_len_in_batch < 0 || a->max_len_in_batch > a->max_seq_len))))
    return LSATTN_ERR_INVALID_ARG;
  RotaryWriteParams p;
  p.q = (uint16_t*)a->q;
  p.q_st = a->q_stride_t;
  p.q_sh = a->q_stride_h;
  p.hq = a->num_q_heads;
  p.kv = (uint16_t*)a->kv;
  p.kv_st = a->kv_stride_t;
  p.kv_sh = a->kv_stride_h;
  p.hkv = a->num_kv_heads;
  p.cos_t = (const uint16_t*)a->cos;
  p.sin_t = (const uint16_t*)a->sin;
  p.num_tokens = a->num_tokens;
  p.head_dim = a->head_dim;
  p.pool = (uint16_t*)a->pool;
  p.pool_stride = a->pool_slot_stride;
  p.dest = a->dest_index;
  p.req_to_tokens = a->req_to_tokens;
  p.max_seq_len = a->max_seq_len;
  p.b_req_idx = a->b_req_idx;
  p.b_start_loc = a->b_start_loc;
  p.b_seq_len = a->b_seq_len;
  p.batch = a->batch;
  p.reg_mode = a->register_mode;
  const int64_t units = a->num_tokens * (a->num_q_heads + 2 * a->num_kv_heads) * (a->head_dim / 16);
  p.data_blocks = (units + 255) / 256;
  p.reg_blocks_per_req = 0;
  int64_t reg_blocks = 0;
  if (a->register_mode == 1) {
    p.reg_blocks_per_req = (a->max_len_in_batch + 255) / 256;
    reg_blocks = p.reg_blocks_per_req * a->batch;
  } else if (a->register_mode == 2) {
    reg_blocks = (a->batch + 255) / 256;
  }
  const int64_t blocks = p.data_blocks + reg_blocks;
  if (blocks == 0) return LSATTN_OK;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(rotary_kv_write_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, p);
  return check_launch();
}
