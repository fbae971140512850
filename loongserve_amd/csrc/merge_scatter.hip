// HBM-bound helpers around the attention kernels: LSE merge of separately allocated
// prefill partials, KV-pool row scatter, and prefill slot registration.
#include <atomic>

#include "common.hip.h"

namespace lsattn {

struct MergeParams {
  int32_t n;
  int64_t rows;
  const float* o[LSATTN_MAX_PARTS];
  const float* lse[LSATTN_MAX_PARTS];
  void* out;
  float* out_lse;
};

template <typename OT> __device__ __forceinline__ void put4(void* base, int64_t elem, const f32x4& v);
template <> __device__ __forceinline__ void put4<float>(void* base, int64_t elem, const f32x4& v) {
  *(f32x4*)((float*)base + elem) = v;
}
template <> __device__ __forceinline__ void put4<F16>(void* base, int64_t elem, const f32x4& v) {
  *(u32x2*)((uint16_t*)base + elem) = u32x2{pack2<F16>(v[0], v[1]), pack2<F16>(v[2], v[3])};
}
template <> __device__ __forceinline__ void put4<BF16>(void* base, int64_t elem, const f32x4& v) {
  *(u32x2*)((uint16_t*)base + elem) = u32x2{pack2<BF16>(v[0], v[1]), pack2<BF16>(v[2], v[3])};
}

// one thread per (row, 4 consecutive output elements); same recurrence as
// flash_decoding_stage2.cu:38-48 with the partials living in separate buffers
template <typename OT, int D>
__global__ __launch_bounds__(256) void lse_merge_kernel(MergeParams p) {
  constexpr int LPR = D / 4;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid / LPR;
  const int c = (int)(gid % LPR);
  if (row >= p.rows) return;
  float M = -INFINITY;
  for (int i = 0; i < p.n; i++) M = fmaxf(M, p.lse[i][row]);
  float L = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (M != -INFINITY) {
    for (int i = 0; i < p.n; i++) {
      const float w = __builtin_amdgcn_exp2f((p.lse[i][row] - M) * kLog2e);
      if (w == 0.f) continue;
      L += w;
      acc += *(const f32x4*)(p.o[i] + row * D + c * 4) * w;
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  put4<OT>(p.out, row * D + c * 4, acc * inv);
  if (c == 0) p.out_lse[row] = L > 0.f ? M + __builtin_amdgcn_logf(L) * kLn2 : -INFINITY;
}

// The partials of a step cut along the keys, joined for the rows of the sequences: one thread per (row of a sequence,
// head, 4 consecutive elements); the workgroup's 256 threads cover 8 (row, head) pairs.  MODE as the prefill kernel's
// epilogues: 0 writes (o fp32, lse), 1 folds into (o, m, l) (ring_context_flashattention_nopad.py:171-188), 2 merges into
// a running (o fp32, lse).
struct MergeCutsParams {
  const float* o_parts;
  const float* lse_parts;
  int64_t part_rows;
  int32_t n, hq;
  const int32_t* q_start;
  const int32_t* q_len;
  void* o;
  int64_t o_st, o_sh;
  float* lse;
  float* m;
  float* l;
  int64_t ml_st, ml_sh;
};
template <typename OT, int MODE> __global__ __launch_bounds__(256) void merge_cuts_kernel(MergeCutsParams p) {
  constexpr int D = 128, LPR = D / 4;
  const int b = blockIdx.y;
  const int64_t pair = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;  // (row of the sequence, head)
  const int c = threadIdx.x % LPR;
  const int64_t r = pair / p.hq;
  const int h = (int)(pair - r * p.hq);
  if (r >= p.q_len[b]) return;
  const int64_t row = (int64_t)p.q_start[b] + r;
  float M = -INFINITY;
  for (int i = 0; i < p.n; i++) M = fmaxf(M, p.lse_parts[(i * p.part_rows + row) * p.hq + h]);
  float L = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (M != -INFINITY) {
    for (int i = 0; i < p.n; i++) {
      const int64_t pr = (i * p.part_rows + row) * p.hq + h;
      const float w = __builtin_amdgcn_exp2f((p.lse_parts[pr] - M) * kLog2e);
      if (w == 0.f) continue;
      L += w;
      acc += *(const f32x4*)(p.o_parts + pr * D + c * 4) * w;
    }
  }
  // the step's partial for this row: acc / L, natural LSE = M + ln L (L >= 1 whenever any cut saw a key)
  const int64_t o_at = row * p.o_st + (int64_t)h * p.o_sh + c * 4;
  if constexpr (MODE == 0) {
    const float inv = L > 0.f ? 1.f / L : 0.f;
    put4<OT>(p.o, o_at, acc * inv);
    if (c == 0) p.lse[row * p.hq + h] = L > 0.f ? M + __builtin_amdgcn_logf(L) * kLn2 : -INFINITY;
    return;
  }
  if (!(L > 0.f)) return;  // no key in any cut: the state stays
  if constexpr (MODE == 2) {
    const float a_old = p.lse[row * p.hq + h], a_new = M + __builtin_amdgcn_logf(L) * kLn2;
    const float top = fmaxf(a_old, a_new);
    const float w_old = a_old == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((a_old - top) * kLog2e);
    const float w_new = __builtin_amdgcn_exp2f((a_new - top) * kLog2e);
    const float W = w_old + w_new;
    // (an empty row may hold anything: its old values are dropped, not multiplied by zero)
    const f32x4 old = w_old != 0.f ? *(const f32x4*)((const float*)p.o + o_at) : f32x4{0.f, 0.f, 0.f, 0.f};
    *(f32x4*)((float*)p.o + o_at) = old * (w_old / W) + acc * (w_new / (W * L));
    // (the 32 threads of a row are half a wave: the load of the old lse has returned for all of them before the one
    // store that depends on it is issued)
    if (c == 0) p.lse[row * p.hq + h] = top + __builtin_amdgcn_logf(W) * kLn2;
    return;
  }
  if constexpr (MODE == 1) {
    // the step as (m_i, l_i, acc_i) = (log2-domain LSE, 1, normalised output) into the running state
    const int64_t ml_at = row * p.ml_st + (int64_t)h * p.ml_sh;
    const float m_old = p.m[ml_at], l_old = p.l[ml_at];
    const float m_i = (M + __builtin_amdgcn_logf(L) * kLn2) * kLog2e;
    const float Mx = fmaxf(m_i, m_old);
    const float w_old = l_old * exp2_diff(m_old, Mx);
    const float w_new = __builtin_amdgcn_exp2f(m_i - Mx);
    const float Ln = w_old + w_new;
    const float inv = 1.f / Ln;
    float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
    uint16_t* optr = (uint16_t*)p.o + o_at;
    if (w_old != 0.f) {  // a row in its start state (m = -inf, l = 0) may hold anything in o
      const u32x2 old = *(const u32x2*)optr;
      unpack2<OT>(old[0], o0, o1);
      unpack2<OT>(old[1], o2, o3);
    }
    const float cn = w_new / L;
    *(u32x2*)optr = u32x2{pack2<OT>((o0 * w_old + acc[0] * cn) * inv, (o1 * w_old + acc[1] * cn) * inv),
                          pack2<OT>((o2 * w_old + acc[2] * cn) * inv, (o3 * w_old + acc[3] * cn) * inv)};
    if (c == 0) {
      p.m[ml_at] = Mx;
      p.l[ml_at] = Ln;
    }
  }
}

// dst[dest_index[i]] = src[i]; 16 bytes per lane, consecutive lanes cover one row
__global__ __launch_bounds__(256) void kv_scatter_kernel(const char* __restrict__ src, int64_t src_stride,
                                                         char* __restrict__ dst, int64_t dst_stride,
                                                         const int32_t* __restrict__ dest_index, int64_t n_rows,
                                                         int32_t chunks_per_row) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid / chunks_per_row;
  const int c = (int)(gid % chunks_per_row);
  if (row >= n_rows) return;
  const u32x4 w = *(const u32x4*)(src + row * src_stride + (int64_t)c * 16);
  *(u32x4*)(dst + (int64_t)dest_index[row] * dst_stride + (int64_t)c * 16) = w;
}

__global__ __launch_bounds__(256) void register_tokens_kernel(int32_t* __restrict__ req_to_tokens, int64_t max_seq_len,
                                                              const int32_t* __restrict__ b_req_idx,
                                                              const int32_t* __restrict__ b_start_loc,
                                                              const int32_t* __restrict__ b_seq_len,
                                                              const int32_t* __restrict__ mem_index) {
  const int64_t b = blockIdx.y;
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= b_seq_len[b]) return;
  req_to_tokens[(int64_t)b_req_idx[b] * max_seq_len + j] = mem_index[(int64_t)b_start_loc[b] + j];
}

// one new token per request: req_to_tokens[b_req_idx[i], b_seq_len[i] - 1] = mem_index[i]
template <typename IT>
__global__ __launch_bounds__(256) void register_decode_tokens_kernel(int32_t* __restrict__ req_to_tokens, int64_t max_seq_len,
                                                                     const int32_t* __restrict__ b_req_idx,
                                                                     const int32_t* __restrict__ b_seq_len,
                                                                     const IT* __restrict__ mem_index, int64_t batch) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= batch) return;
  const int64_t pos = (int64_t)b_seq_len[i] - 1;
  if (pos < 0 || pos >= max_seq_len) return;  // (the reference would write outside the row)
  req_to_tokens[(int64_t)b_req_idx[i] * max_seq_len + pos] = (int32_t)mem_index[i];
}

// ceil(x / p) for p > 0 as floor((x + p - 1) / p), also for negative x
__device__ __forceinline__ int32_t ceil_div_floor(int32_t x, int32_t p) {
  const int64_t a = (int64_t)x + p - 1;
  int64_t q = a / p;
  if ((a % p != 0) && (a < 0)) q -= 1;
  return (int32_t)q;
}

__global__ __launch_bounds__(256) void kv_ranges_kernel(const int32_t* __restrict__ idx_begin, const int32_t* __restrict__ idx_end,
                                                        const int32_t* __restrict__ first, int32_t peers, int64_t batch,
                                                        int32_t* __restrict__ range_begin, int32_t* __restrict__ range_end,
                                                        int32_t* __restrict__ new_len) {
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= batch) return;
  const int32_t rb = ceil_div_floor(idx_begin[b] - first[b], peers);
  const int32_t re = ceil_div_floor(idx_end[b] - first[b], peers);
  range_begin[b] = rb;
  range_end[b] = re;
  new_len[b] = re - rb;
}

struct CopyRegisterParams {
  const char* kv;
  int64_t kv_stride;
  char* pool;
  int64_t pool_stride;
  const int32_t* new_len;
  const int32_t* range_begin;
  const int32_t* range_end;
  const int64_t* len_sum;
  const int32_t* start_loc;
  const int32_t* cur_index;
  const int32_t* mem_index;
  const int32_t* b_req_idx;
  int32_t* req_to_tokens;
  int64_t max_seq_len, num_used, row_limit;
  int32_t chunks_per_row, should_register, rows_per_block;
};

// grid (groups of rows_per_block rows, batch); 16 bytes per lane and step, consecutive lanes cover one row.
// A workgroup past the end of its request leaves at once: the grid is sized by the longest request.
__global__ __launch_bounds__(256) void kv_copy_register_kernel(CopyRegisterParams p) {
  const int64_t b = blockIdx.y;
  int64_t n_new = p.new_len[b];
  const int64_t begin = p.range_begin[b];
  if (n_new <= 0 || begin < 0 || p.range_end[b] < 0) return;
  if (n_new > p.row_limit) n_new = p.row_limit;
  const int64_t row0 = (int64_t)blockIdx.x * p.rows_per_block;
  if (row0 >= n_new) return;
  const int64_t rows = n_new - row0 < p.rows_per_block ? n_new - row0 : p.rows_per_block;
  const int64_t mi0 = p.num_used + (b > 0 ? p.len_sum[b - 1] : 0) + row0;
  const char* src = p.kv + ((int64_t)p.start_loc[b] + begin + row0) * p.kv_stride;
  const int64_t pieces = rows * p.chunks_per_row;
  for (int64_t i = threadIdx.x; i < pieces; i += 256) {
    const int64_t r = i / p.chunks_per_row;
    const int c = (int)(i % p.chunks_per_row);
    const int32_t slot = p.mem_index[mi0 + r];
    const u32x4 w = *(const u32x4*)(src + r * p.kv_stride + (int64_t)c * 16);
    *(u32x4*)(p.pool + (int64_t)slot * p.pool_stride + (int64_t)c * 16) = w;
    if (p.should_register && c == 0) p.req_to_tokens[(int64_t)p.b_req_idx[b] * p.max_seq_len + p.cur_index[b] + row0 + r] = slot;
  }
}

struct MigrationParams {
  char* staging;
  int64_t staging_layer, staging_row;
  char* kv;
  int64_t kv_layer, kv_row;
  int64_t layers, max_seq_len;
  int32_t* req_to_tokens;
  int32_t* mem_state;
  const int32_t* alloc_mem;
  const int32_t* request_ids;
  const int32_t* num_tokens;
  const int32_t* cumsum;
  const int32_t* b_seq_len;
  int32_t chunks_per_row, rows_per_block;
};

// grid (groups of migrating tokens, batch); a workgroup moves rows_per_block tokens of one request through every layer,
// 16 bytes per lane and step
template <bool SEND> __global__ __launch_bounds__(256) void decode_migration_kernel(MigrationParams p) {
  const int64_t b = blockIdx.y;
  const int64_t n = p.num_tokens[b];
  const int64_t j0 = (int64_t)blockIdx.x * p.rows_per_block;
  if (j0 >= n) return;
  const int64_t rows = n - j0 < p.rows_per_block ? n - j0 : p.rows_per_block;
  const int64_t buf0 = (b > 0 ? p.cumsum[b - 1] : 0) + j0;
  int32_t* table = p.req_to_tokens + (int64_t)p.request_ids[b] * p.max_seq_len;
  const int64_t pos0 = SEND ? p.b_seq_len[b] - n + j0 : p.b_seq_len[b] + j0;
  const int64_t pieces = rows * p.chunks_per_row;
  for (int64_t i = threadIdx.x; i < pieces; i += 256) {
    const int64_t r = i / p.chunks_per_row;
    const int64_t c = i % p.chunks_per_row;
    int32_t slot;
    if (SEND) {
      slot = table[pos0 + r];
      if (c == 0) p.mem_state[slot] = 0;
    } else {
      slot = p.alloc_mem[buf0 + r];
      if (c == 0) table[pos0 + r] = slot;
    }
    char* kvp = p.kv + (int64_t)slot * p.kv_row + c * 16;
    char* bp = p.staging + (buf0 + r) * p.staging_row + c * 16;
    for (int64_t layer = 0; layer < p.layers; layer++) {
      if (SEND) *(u32x4*)(bp + layer * p.staging_layer) = *(const u32x4*)(kvp + layer * p.kv_layer);
      else *(u32x4*)(kvp + layer * p.kv_layer) = *(const u32x4*)(bp + layer * p.staging_layer);
    }
  }
}

template <bool SEND> static int launch_migration(const lsattn_decode_migration_args* a, hipStream_t st) {
  if (!a || !a->staging || !a->kv_cache || !a->req_to_tokens || !a->request_ids || !a->num_tokens || !a->num_tokens_cumsum ||
      !a->b_seq_len || (SEND ? !a->mem_state : !a->alloc_mem))
    return LSATTN_ERR_INVALID_ARG;
  if (a->batch < 0 || a->max_num_tokens < 0 || a->num_layers <= 0 || a->row_bytes <= 0 || a->max_seq_len <= 0)
    return LSATTN_ERR_INVALID_ARG;
  if (a->row_bytes % 16 || a->staging_row_stride_bytes % 16 || a->staging_layer_stride_bytes % 16 || a->kv_row_stride_bytes % 16 ||
      a->kv_layer_stride_bytes % 16 || (((uintptr_t)a->staging | (uintptr_t)a->kv_cache) & 15))
    return LSATTN_ERR_INVALID_ARG;
  if (a->batch == 0 || a->max_num_tokens == 0) return LSATTN_OK;
  if (a->batch > 65535) return LSATTN_ERR_INVALID_ARG;
  MigrationParams p;
  p.staging = (char*)a->staging;
  p.staging_layer = a->staging_layer_stride_bytes;
  p.staging_row = a->staging_row_stride_bytes;
  p.kv = (char*)a->kv_cache;
  p.kv_layer = a->kv_layer_stride_bytes;
  p.kv_row = a->kv_row_stride_bytes;
  p.layers = a->num_layers;
  p.max_seq_len = a->max_seq_len;
  p.req_to_tokens = a->req_to_tokens;
  p.mem_state = a->mem_state;
  p.alloc_mem = a->alloc_mem;
  p.request_ids = a->request_ids;
  p.num_tokens = a->num_tokens;
  p.cumsum = a->num_tokens_cumsum;
  p.b_seq_len = a->b_seq_len;
  const int64_t cpr = a->row_bytes / 16;
  if (cpr > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  p.chunks_per_row = (int32_t)cpr;
  p.rows_per_block = cpr >= 256 ? 1 : (int32_t)(256 / cpr);  // one 16-byte piece per lane and layer
  const int64_t blocks = (a->max_num_tokens + p.rows_per_block - 1) / p.rows_per_block;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL((decode_migration_kernel<SEND>), dim3((unsigned)blocks, (unsigned)a->batch), dim3(256), 0, st, p);
  return check_launch();
}

template <typename OT> static int launch_merge(const MergeParams& p, int D, hipStream_t st) {
  const int64_t threads = p.rows * (D / 4);
  const int64_t blocks = (threads + 255) / 256;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  switch (D) {
    case 16: LSATTN_LAUNCH_KERNEL((lse_merge_kernel<OT, 16>), dim3((unsigned)blocks), dim3(256), 0, st, p); break;
    case 32: LSATTN_LAUNCH_KERNEL((lse_merge_kernel<OT, 32>), dim3((unsigned)blocks), dim3(256), 0, st, p); break;
    case 64: LSATTN_LAUNCH_KERNEL((lse_merge_kernel<OT, 64>), dim3((unsigned)blocks), dim3(256), 0, st, p); break;
    case 128: LSATTN_LAUNCH_KERNEL((lse_merge_kernel<OT, 128>), dim3((unsigned)blocks), dim3(256), 0, st, p); break;
    default: return LSATTN_ERR_UNSUPPORTED;
  }
  return check_launch();
}

}  // namespace lsattn

using namespace lsattn;

extern "C" int lsattn_lse_merge(const lsattn_merge_args* a, void* stream) {
  if (!a || a->n_parts < 1 || a->n_parts > LSATTN_MAX_PARTS || a->rows < 0 || !a->o || !a->lse) return LSATTN_ERR_INVALID_ARG;
  MergeParams p;
  p.n = a->n_parts;
  p.rows = a->rows;
  for (int i = 0; i < LSATTN_MAX_PARTS; i++) {
    p.o[i] = i < a->n_parts ? a->o_parts[i] : nullptr;
    p.lse[i] = i < a->n_parts ? a->lse_parts[i] : nullptr;
    if (i < a->n_parts && (!p.o[i] || !p.lse[i] || ((uintptr_t)p.o[i] & 15))) return LSATTN_ERR_INVALID_ARG;
  }
  if ((uintptr_t)a->o & 15) return LSATTN_ERR_INVALID_ARG;
  p.out = a->o;
  p.out_lse = a->lse;
  if (a->rows == 0) return LSATTN_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (a->o_dtype) {
    case LSATTN_F32: return launch_merge<float>(p, a->head_dim, st);
    case LSATTN_F16: return launch_merge<F16>(p, a->head_dim, st);
    case LSATTN_BF16: return launch_merge<BF16>(p, a->head_dim, st);
    default: return LSATTN_ERR_UNSUPPORTED;
  }
}

extern "C" int lsattn_prefill_merge_cuts(const lsattn_merge_cuts_args* a, void* stream) {
  if (!a || !a->o_parts || !a->lse_parts || !a->q_b_start_loc || !a->q_b_seq_len || !a->o) return LSATTN_ERR_INVALID_ARG;
  if (a->n_parts < 1 || a->n_parts > LSATTN_MAX_KV_CUTS || a->part_rows < 0 || a->batch < 0 || a->num_q_heads <= 0 || a->max_q_len < 0)
    return LSATTN_ERR_INVALID_ARG;
  if (a->head_dim != 128) return LSATTN_ERR_UNSUPPORTED;
  if (a->mode < 0 || a->mode > 2) return LSATTN_ERR_INVALID_ARG;
  if (a->mode == 1 ? (!a->m || !a->l || (a->o_dtype != LSATTN_F16 && a->o_dtype != LSATTN_BF16)) : (!a->lse || a->o_dtype != LSATTN_F32))
    return LSATTN_ERR_INVALID_ARG;
  if (a->o_stride_t % 4 || a->o_stride_h % 4 || (((uintptr_t)a->o | (uintptr_t)a->o_parts) & 15)) return LSATTN_ERR_INVALID_ARG;
  if (a->batch == 0 || a->max_q_len == 0) return LSATTN_OK;
  if (a->batch > 65535) return LSATTN_ERR_INVALID_ARG;
  MergeCutsParams p{a->o_parts, a->lse_parts, a->part_rows, a->n_parts, a->num_q_heads, a->q_b_start_loc, a->q_b_seq_len, a->o,
                    a->o_stride_t, a->o_stride_h, a->lse, a->m, a->l, a->ml_stride_t, a->ml_stride_h};
  const int64_t pairs = (int64_t)a->max_q_len * a->num_q_heads;
  const int64_t blocks = (pairs + 7) / 8;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  const dim3 grid((unsigned)blocks, (unsigned)a->batch);
  hipStream_t st = (hipStream_t)stream;
  if (a->mode == 0) LSATTN_LAUNCH_KERNEL((merge_cuts_kernel<float, 0>), grid, dim3(256), 0, st, p);
  else if (a->mode == 2) LSATTN_LAUNCH_KERNEL((merge_cuts_kernel<float, 2>), grid, dim3(256), 0, st, p);
  else if (a->o_dtype == LSATTN_F16) LSATTN_LAUNCH_KERNEL((merge_cuts_kernel<F16, 1>), grid, dim3(256), 0, st, p);
  else LSATTN_LAUNCH_KERNEL((merge_cuts_kernel<BF16, 1>), grid, dim3(256), 0, st, p);
  return check_launch();
}

extern "C" int lsattn_kv_scatter(const void* src, int64_t src_stride_bytes, void* dst, int64_t dst_stride_bytes,
                                 const int32_t* dest_index, int64_t n_rows, int64_t row_bytes, void* stream) {
  if (!src || !dst || !dest_index || n_rows < 0 || row_bytes <= 0) return LSATTN_ERR_INVALID_ARG;
  if (row_bytes % 16 || src_stride_bytes % 16 || dst_stride_bytes % 16 || (((uintptr_t)src | (uintptr_t)dst) & 15))
    return LSATTN_ERR_INVALID_ARG;
  if (n_rows == 0) return LSATTN_OK;
  const int64_t cpr = row_bytes / 16;
  const int64_t blocks = (n_rows * cpr + 255) / 256;
  if (blocks > 0x7fffffff || cpr > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(kv_scatter_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const char*)src,
                     src_stride_bytes, (char*)dst, dst_stride_bytes, dest_index, n_rows, (int32_t)cpr);
  return check_launch();
}

extern "C" int lsattn_register_tokens(int32_t* req_to_tokens, int64_t max_seq_len, const int32_t* b_req_idx,
                                      const int32_t* b_start_loc, const int32_t* b_seq_len, const int32_t* mem_index,
                                      int64_t batch, int64_t max_len_in_batch, void* stream) {
  if (!req_to_tokens || !b_req_idx || !b_start_loc || !b_seq_len || !mem_index || batch < 0 || max_len_in_batch < 0 ||
      max_len_in_batch > max_seq_len)
    return LSATTN_ERR_INVALID_ARG;
  if (batch == 0 || max_len_in_batch == 0) return LSATTN_OK;
  if (batch > 65535) return LSATTN_ERR_INVALID_ARG;
  dim3 grid((unsigned)((max_len_in_batch + 255) / 256), (unsigned)batch);
  LSATTN_LAUNCH_KERNEL(register_tokens_kernel, grid, dim3(256), 0, (hipStream_t)stream, req_to_tokens, max_seq_len,
                     b_req_idx, b_start_loc, b_seq_len, mem_index);
  return check_launch();
}

extern "C" int lsattn_register_decode_tokens(int32_t* req_to_tokens, int64_t max_seq_len, const int32_t* b_req_idx,
                                             const int32_t* b_seq_len, const void* mem_index, int32_t mem_index_is_i64,
                                             int64_t batch, void* stream) {
  if (!req_to_tokens || !b_req_idx || !b_seq_len || !mem_index || batch < 0 || max_seq_len <= 0 ||
      (mem_index_is_i64 != 0 && mem_index_is_i64 != 1))
    return LSATTN_ERR_INVALID_ARG;
  if (batch == 0) return LSATTN_OK;
  const int64_t blocks = (batch + 255) / 256;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  if (mem_index_is_i64)
    LSATTN_LAUNCH_KERNEL(register_decode_tokens_kernel<int64_t>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       req_to_tokens, max_seq_len, b_req_idx, b_seq_len, (const int64_t*)mem_index, batch);
  else
    LSATTN_LAUNCH_KERNEL(register_decode_tokens_kernel<int32_t>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       req_to_tokens, max_seq_len, b_req_idx, b_seq_len, (const int32_t*)mem_index, batch);
  return check_launch();
}

extern "C" int lsattn_kv_ranges(const int32_t* kv_cache_index_begin, const int32_t* kv_cache_index_end,
                                const int32_t* kv_first_token_global_idx, int32_t sp_peers, int64_t batch,
                                int32_t* kv_range_begin, int32_t* kv_range_end, int32_t* new_kv_cache_len, void* stream) {
  if (!kv_cache_index_begin || !kv_cache_index_end || !kv_first_token_global_idx || !kv_range_begin || !kv_range_end ||
      !new_kv_cache_len || sp_peers < 1 || batch < 0)
    return LSATTN_ERR_INVALID_ARG;
  if (batch == 0) return LSATTN_OK;
  const int64_t blocks = (batch + 255) / 256;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL(kv_ranges_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, kv_cache_index_begin,
                     kv_cache_index_end, kv_first_token_global_idx, sp_peers, batch, kv_range_begin, kv_range_end,
                     new_kv_cache_len);
  return check_launch();
}

extern "C" int lsattn_kv_copy_register(const lsattn_kv_copy_register_args* a, void* stream) {
  if (!a || !a->kv || !a->pool || !a->new_kv_cache_len || !a->kv_range_begin || !a->kv_range_end ||
      !a->new_kv_cache_len_sum || !a->kv_b_start_loc || !a->mem_index || a->batch < 0 || a->row_bytes <= 0 ||
      a->num_used_mem_index < 0 || a->max_len_in_batch < 0)
    return LSATTN_ERR_INVALID_ARG;
  if (a->should_register && (!a->cur_kv_cache_index || !a->b_req_idx || !a->req_to_tokens || a->max_seq_len <= 0))
    return LSATTN_ERR_INVALID_ARG;
  if (a->row_bytes % 16 || a->kv_stride_bytes % 16 || a->pool_stride_bytes % 16 ||
      (((uintptr_t)a->kv | (uintptr_t)a->pool) & 15))
    return LSATTN_ERR_INVALID_ARG;
  if (a->batch == 0 || a->max_len_in_batch == 0) return LSATTN_OK;
  if (a->batch > 65535) return LSATTN_ERR_INVALID_ARG;
  CopyRegisterParams p;
  p.kv = (const char*)a->kv;
  p.kv_stride = a->kv_stride_bytes;
  p.pool = (char*)a->pool;
  p.pool_stride = a->pool_stride_bytes;
  p.new_len = a->new_kv_cache_len;
  p.range_begin = a->kv_range_begin;
  p.range_end = a->kv_range_end;
  p.len_sum = a->new_kv_cache_len_sum;
  p.start_loc = a->kv_b_start_loc;
  p.cur_index = a->cur_kv_cache_index;
  p.mem_index = a->mem_index;
  p.b_req_idx = a->b_req_idx;
  p.req_to_tokens = a->req_to_tokens;
  p.max_seq_len = a->max_seq_len;
  p.num_used = a->num_used_mem_index;
  p.row_limit = (a->max_len_in_batch + 255) / 256 * 256;  // the reference's grid: (batch, cdiv(max_len_in_batch, 256)) x 256 rows
  const int64_t cpr = a->row_bytes / 16;
  if (cpr > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  p.rows_per_block = cpr >= 4096 ? 1 : (int32_t)(4096 / cpr);  // about 64 KB per workgroup
  const int64_t blocks = (p.row_limit + p.rows_per_block - 1) / p.rows_per_block;
  if (blocks > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  p.chunks_per_row = (int32_t)cpr;
  p.should_register = a->should_register;
  LSATTN_LAUNCH_KERNEL(kv_copy_register_kernel, dim3((unsigned)blocks, (unsigned)a->batch), dim3(256), 0, (hipStream_t)stream, p);
  return check_launch();
}

extern "C" int lsattn_decode_migration_send(const lsattn_decode_migration_args* a, void* stream) {
  return launch_migration<true>(a, (hipStream_t)stream);
}
extern "C" int lsattn_decode_migration_recv(const lsattn_decode_migration_args* a, void* stream) {
  return launch_migration<false>(a, (hipStream_t)stream);
}

namespace lsattn {
static std::atomic<int32_t> g_tuning[5];
Tuning tuning() {
  Tuning t;
  t.prefill_rows = g_tuning[0].load(std::memory_order_relaxed);
  t.prefill_order = g_tuning[1].load(std::memory_order_relaxed);
  t.prefill_pack = g_tuning[2].load(std::memory_order_relaxed);
  t.decode_stage1 = g_tuning[3].load(std::memory_order_relaxed);
  t.decode_listed = g_tuning[4].load(std::memory_order_relaxed);
  return t;
}
}  // namespace lsattn

extern "C" int lsattn_set_tuning(const lsattn_tuning* t) {
  lsattn_tuning z = {};
  if (!t) t = &z;
  if (t->prefill_rows < 0 || t->prefill_rows > LSATTN_PREFILL_ROWS_HALF || t->prefill_order < 0 || t->prefill_order > LSATTN_PREFILL_ORDER_HEAD ||
      t->prefill_pack < 0 || t->prefill_pack > LSATTN_PREFILL_PACK_OFF || t->decode_stage1 < 0 || t->decode_stage1 > LSATTN_DECODE_STAGE1_SPLIT ||
      t->decode_listed < 0 || t->decode_listed > LSATTN_DECODE_LISTED_SHARES || t->reserved[0] || t->reserved[1] || t->reserved[2])
    return LSATTN_ERR_INVALID_ARG;
  const int32_t v[5] = {t->prefill_rows, t->prefill_order, t->prefill_pack, t->decode_stage1, t->decode_listed};
  for (int i = 0; i < 5; i++) lsattn::g_tuning[i].store(v[i], std::memory_order_relaxed);
  return LSATTN_OK;
}

extern "C" const char* lsattn_strerror(int code) {
  switch (code) {
    case LSATTN_OK: return "ok";
    case LSATTN_ERR_INVALID_ARG: return "invalid argument (null pointer, bad size, stride or alignment)";
    case LSATTN_ERR_UNSUPPORTED: return "unsupported head_dim, dtype or head ratio";
    case LSATTN_ERR_LAUNCH: return "kernel launch failed";
    case LSATTN_ERR_WORKSPACE: return "workspace too small";
    default: return "unknown error";
  }
}

extern "C" int lsattn_version(void) { return LSATTN_VERSION; }
