// Ring / context-parallel prefill attention step for gfx950 (MFMA, wave64).
//
// Replaces the Triton _fwd_kernel + context_attention_fwd
// (loongserve/models/llama/triton_kernel/ring_context_flashattention_nopad.py:13-284).
//
// Shape of the computation (head_dim 128):
//   * a workgroup of 4 waves owns 256 consecutive local query rows of one (sequence, q head);
//     each wave owns 64 of them and keeps their Q as MFMA B operands in registers;
//   * K/V tiles of 64 keys are staged through LDS (double buffered, XOR-swizzled 16-byte
//     chunks so that both the row-wise K reads and the transposing V reads are conflict free);
//   * scores are computed transposed, S^T = K Q^T with v_mfma_f32_32x32x16, so every lane
//     owns one query column: row max / row sum are in-lane reductions plus one
//     half-wave swap, and the fp32 S^T accumulators convert in place into the B operand
//     of O^T += V^T P^T without any cross-lane movement;
//   * V^T operands come from LDS through ds_read_b64_tr_b16 (the tile is stored row-major);
//   * causal work is skipped per wave (64 rows) and masks are applied only on tiles that
//     straddle the diagonal or the end of the KV chunk;
//   * workgroup ids are mapped so that the workgroups sharing one KV head run on one XCD
//     (ids are dealt round-robin to the 8 XCDs) and heavy (late) query tiles start first.
#include "common.hip.h"

namespace lsattn {

struct PrefillParams {
  const void* q;
  const void* k;
  const void* v;
  int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* q_first;
  const int32_t* kv_start;
  const int32_t* kv_len;
  const int32_t* kv_first;
  int32_t batch, hq, hkv, peers, nz, kv_slots;
  float scale_log2;
  void* o;
  int64_t o_st, o_sh;
  float* lse;
  float* m;
  float* l;
  int64_t ml_st, ml_sh;
};

constexpr int BM = 256;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int NWAVE = 4;

template <typename T> struct Mfma;
template <> struct Mfma<F16> {
  static __device__ __forceinline__ f32x16 run(const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mfma<BF16> {
  static __device__ __forceinline__ f32x16 run(const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// The P V product always runs on the f16 MFMA: P in [0,1] keeps 11 significant bits there
// (8 as bfloat16, which alone would cost ~1.1e-3 relative error in O).  A bfloat16 V tile is
// therefore converted to f16 while it is staged into LDS; every bfloat16 value with
// magnitude in [2^-14, 65504] is exactly representable, larger ones saturate to +-65504.
template <typename T> __device__ __forceinline__ u32x4 to_pv_operand(const u32x4& w);
template <> __device__ __forceinline__ u32x4 to_pv_operand<F16>(const u32x4& w) { return w; }
template <> __device__ __forceinline__ u32x4 to_pv_operand<BF16>(const u32x4& w) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float lo, hi;
    unpack2<BF16>(w[i], lo, hi);
    lo = __builtin_amdgcn_fmed3f(lo, -65504.f, 65504.f);
    hi = __builtin_amdgcn_fmed3f(hi, -65504.f, 65504.f);
    r[i] = pack2<F16>(lo, hi);
  }
  return r;
}

// value of the same register in the other half of the wave (lane ^ 32)
__device__ __forceinline__ float other_half(float v, int upper) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, upper ? r[0] : r[1]);
}

// physical 16-byte chunk of (row, logical chunk) inside a [64 rows][16 chunks] tile
__device__ __forceinline__ int swz(int row, int chunk) { return row * 16 + (chunk ^ (((row & 3) << 2) | ((row >> 2) & 3))); }

typedef __attribute__((address_space(3))) i16x4* lds_i16x4_ptr;

template <typename T, int MODE>  // MODE 0: partial (o fp32, lse)   MODE 1: in-place (o, m, l) update
__global__ __launch_bounds__(NWAVE * 64, 1) void prefill_kernel(PrefillParams p) {
  __shared__ u32x4 lds_k[2][BN * 16];
  __shared__ u32x4 lds_v[2][BN * 16];

  // ---- workgroup -> (sequence, q head, query tile) ----
  const int group = p.hq / p.hkv;
  int j = blockIdx.x >> 3;
  const int xcd = blockIdx.x & 7;
  const int gq = j % group;
  j /= group;
  const int zr = j % p.nz;
  j /= p.nz;
  const int slot = j % p.kv_slots;
  const int b = j / p.kv_slots;
  const int kvh = xcd + 8 * slot;
  if (kvh >= p.hkv) return;
  const int h = kvh * group + gq;
  const int z = p.nz - 1 - zr;

  const int64_t q_len = p.q_len[b];
  const int64_t m_lo = (int64_t)z * BM;
  if (m_lo >= q_len) return;
  const int64_t kv_len = p.kv_len[b];
  const int64_t q_start = p.q_start[b], kv_start = p.kv_start[b];
  const int64_t qf = p.q_first[b], kf = p.kv_first[b];
  const int64_t P = p.peers;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int qc = lane & 31, g = lane >> 5;

  // keys visible to the last valid row of the workgroup bound the tile loop
  const int64_t m_hi = (m_lo + BM < q_len ? m_lo + BM : q_len) - 1;
  int64_t n_end = 0;
  {
    const int64_t dq = qf + m_hi * P - kf;
    if (dq >= 0) n_end = dq / P + 1;
    if (n_end > kv_len) n_end = kv_len;
  }
  const int n_tiles = (int)((n_end + BN - 1) / BN);

  // ---- this wave's rows ----
  const int64_t m_w0 = m_lo + wave * 64;
  int64_t m_wlast = m_w0 + 63;
  if (m_wlast > q_len - 1) m_wlast = q_len - 1;
  const int64_t qg_wlast = qf + m_wlast * P;  // largest global position in the wave (may be < row 0 if the wave is empty)
  const int64_t qg_wfirst = qf + m_w0 * P;
  const bool wave_has_rows = m_w0 < q_len;

  // Q as B operands: qreg[qb][t] = Q[row qb*32+qc][16t + 8g .. +7]
  u32x4 qreg[2][8];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    const int64_t m = m_w0 + qb * 32 + qc;
    const bool ok = m < q_len;
    const char* src = (const char*)p.q + ((q_start + (ok ? m : 0)) * p.q_st + (int64_t)h * p.q_sh + 8 * g) * 2;
#pragma unroll
    for (int t = 0; t < 8; t++) qreg[qb][t] = ok ? *(const u32x4*)(src + t * 32) : u32x4{0, 0, 0, 0};
  }

  f32x16 oacc[4][2];
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][qb][i] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_run[2] = {0.f, 0.f};

  // ---- tile staging: thread owns 4 chunks of K and 4 of V per tile ----
  const char* kg = (const char*)p.k + (kv_start * p.k_st + (int64_t)kvh * p.k_sh) * 2;
  const char* vg = (const char*)p.v + (kv_start * p.v_st + (int64_t)kvh * p.v_sh) * 2;
  u32x4 kst[4], vst[4];
  auto load_tile = [&](int t) {
    const int64_t n0 = (int64_t)t * BN;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int cid = i * 256 + tid;
      const int r = cid >> 4, c = cid & 15;
      const bool ok = n0 + r < kv_len;
      kst[i] = ok ? *(const u32x4*)(kg + ((n0 + r) * p.k_st) * 2 + c * 16) : u32x4{0, 0, 0, 0};
      vst[i] = ok ? *(const u32x4*)(vg + ((n0 + r) * p.v_st) * 2 + c * 16) : u32x4{0, 0, 0, 0};
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int cid = i * 256 + tid;
      const int r = cid >> 4, c = cid & 15;
      lds_k[buf][swz(r, c)] = kst[i];
      lds_v[buf][swz(r, c)] = to_pv_operand<T>(vst[i]);
    }
  };

  if (n_tiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  for (int t = 0; t < n_tiles; t++) {
    const int buf = t & 1;
    if (t + 1 < n_tiles) load_tile(t + 1);

    const int64_t n0 = (int64_t)t * BN;
    const int64_t kg0 = kf + n0 * P;                 // global position of the tile's first key
    const bool active = wave_has_rows && kg0 <= qg_wlast;  // some row of the wave sees some key of the tile
    if (active) {
      const bool need_mask = !(kf + (n0 + BN - 1) * P <= qg_wfirst && n0 + BN <= kv_len);

      // ---- S^T = K Q^T ----
      f32x16 s[2][2];
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
#pragma unroll
          for (int i = 0; i < 16; i++) s[kb][qb][i] = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int t8 = 0; t8 < 8; t8++) {
          const u32x4 a = lds_k[buf][swz(kb * 32 + qc, 2 * t8 + g)];
          s[kb][0] = Mfma<T>::run(a, qreg[0][t8], s[kb][0]);
          s[kb][1] = Mfma<T>::run(a, qreg[1][t8], s[kb][1]);
        }
      }

      // ---- online softmax on the query column owned by this lane ----
      u32x4 pk[2][4];  // P^T as B operands: pk[qb][u], k-step u = kb*2 + jj
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        if (need_mask) {
          const int64_t qpos = qf + (m_w0 + qb * 32 + qc) * P;
#pragma unroll
          for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
              const int64_t n = n0 + kb * 32 + (i >> 2) * 8 + 4 * g + (i & 3);
              const bool vis = (kf + n * P <= qpos) && (n < kv_len);
              s[kb][qb][i] = vis ? s[kb][qb][i] : -INFINITY;
            }
        }
        float mx = s[0][qb][0];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[kb][qb][i]);
        mx = fmaxf(mx, other_half(mx, g));
        const float m_new = fmaxf(m_run[qb], mx * p.scale_log2);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_safe);
        m_run[qb] = m_new;
        float ps = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
          float pv[16];
#pragma unroll
          for (int i = 0; i < 16; i++) {
            pv[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][qb][i], p.scale_log2, -m_safe));
            ps += pv[i];
          }
#pragma unroll
          for (int jj = 0; jj < 2; jj++) {
            u32x4 w;
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = pack2<F16>(pv[8 * jj + 2 * e], pv[8 * jj + 2 * e + 1]);
            pk[qb][kb * 2 + jj] = w;
          }
        }
        l_run[qb] = l_run[qb] * alpha + ps;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) oacc[db][qb][i] *= alpha;
      }

      // ---- O^T += V^T P^T ----
      const int blk16 = lane >> 4;  // 16-lane block of the transposing read
      const int li = lane & 15;
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int kb = u >> 1, jj = u & 1;
        const int row_a = kb * 32 + jj * 16 + 4 * (blk16 >> 1) + (li >> 2);  // keys base + 4g + 0..3
        const int row_b = row_a + 8;                                          // keys base + 8 + 4g + 0..3
#pragma unroll
        for (int db = 0; db < 4; db++) {
          const int d_off = db * 32 + (blk16 & 1) * 16 + 4 * (li & 3);  // first of 4 consecutive elements
          const char* base = (const char*)&lds_v[buf][0];
          const char* pa = base + swz(row_a, d_off >> 3) * 16 + (d_off & 7) * 2;
          const char* pb = base + swz(row_b, d_off >> 3) * 16 + (d_off & 7) * 2;
          const i16x4 va = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)pa);
          const i16x4 vb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)pb);
          const u32x2 wa = __builtin_bit_cast(u32x2, va), wb = __builtin_bit_cast(u32x2, vb);
          const u32x4 a = {wa[0], wa[1], wb[0], wb[1]};
          oacc[db][0] = Mfma<F16>::run(a, pk[0][u], oacc[db][0]);
          oacc[db][1] = Mfma<F16>::run(a, pk[1][u], oacc[db][1]);
        }
      }
    }

    if (t + 1 < n_tiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    const int64_t m = m_w0 + qb * 32 + qc;
    const float l_tot = l_run[qb] + other_half(l_run[qb], g);
    if (m >= q_len) continue;
    const int64_t tok = q_start + m;
    if (MODE == 0) {
      const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
      float* orow = (float*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const int d = db * 32 + i4 * 8 + 4 * g;
          const f32x4 v = {oacc[db][qb][i4 * 4 + 0] * inv, oacc[db][qb][i4 * 4 + 1] * inv, oacc[db][qb][i4 * 4 + 2] * inv,
                           oacc[db][qb][i4 * 4 + 3] * inv};
          *(f32x4*)(orow + d) = v;
        }
      if (g == 0) p.lse[tok * p.hq + h] = l_tot > 0.f ? (m_run[qb] + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
    } else {
      // RING:171-188: M = max(m_i, m_old); L = l_old 2^(m_old-M) + l_i 2^(m_i-M);
      // o = (o_old l_old 2^(m_old-M) + acc 2^(m_i-M)) / L
      float* mp = p.m + tok * p.ml_st + (int64_t)h * p.ml_sh;
      float* lp = p.l + tok * p.ml_st + (int64_t)h * p.ml_sh;
      const float m_old = *mp, l_old = *lp;
      const float M = fmaxf(m_run[qb], m_old);
      if (M == -INFINITY || l_tot <= 0.f) continue;  // nothing seen in this step: state unchanged
      const float w_old = l_old * exp2_diff(m_old, M);
      const float w_new = exp2_diff(m_run[qb], M);
      const float L = w_old + l_tot * w_new;
      const float inv = 1.f / L;
      uint16_t* orow = (uint16_t*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const int d = db * 32 + i4 * 8 + 4 * g;
          u32x2* dst = (u32x2*)(orow + d);
          float o0, o1, o2, o3;
          if (w_old != 0.f) {
            const u32x2 old = *dst;
            unpack2<T>(old[0], o0, o1);
            unpack2<T>(old[1], o2, o3);
          } else {
            o0 = o1 = o2 = o3 = 0.f;
          }
          const float r0 = (o0 * w_old + oacc[db][qb][i4 * 4 + 0] * w_new) * inv;
          const float r1 = (o1 * w_old + oacc[db][qb][i4 * 4 + 1] * w_new) * inv;
          const float r2 = (o2 * w_old + oacc[db][qb][i4 * 4 + 2] * w_new) * inv;
          const float r3 = (o3 * w_old + oacc[db][qb][i4 * 4 + 3] * w_new) * inv;
          *dst = u32x2{pack2<T>(r0, r1), pack2<T>(r2, r3)};
        }
      if (g == 0) {
        *mp = M;
        *lp = L;
      }
    }
  }
}

template <typename T, int MODE> static int launch_prefill(const lsattn_prefill_args* a, hipStream_t st) {
  PrefillParams p;
  p.q = a->q;
  p.k = a->k;
  p.v = a->v;
  p.q_st = a->q_stride_t;
  p.q_sh = a->q_stride_h;
  p.k_st = a->k_stride_t;
  p.k_sh = a->k_stride_h;
  p.v_st = a->v_stride_t;
  p.v_sh = a->v_stride_h;
  p.q_start = a->q_b_start_loc;
  p.q_len = a->q_b_seq_len;
  p.q_first = a->q_first_token_global_idx;
  p.kv_start = a->kv_b_start_loc;
  p.kv_len = a->kv_b_seq_len;
  p.kv_first = a->kv_first_token_global_idx;
  p.batch = a->batch;
  p.hq = a->num_q_heads;
  p.hkv = a->num_kv_heads;
  p.peers = a->sp_peers;
  p.nz = (a->max_q_len + BM - 1) / BM;
  p.kv_slots = (a->num_kv_heads + 7) / 8;
  p.scale_log2 = a->sm_scale * kLog2e;
  p.o = a->o;
  p.o_st = a->o_stride_t;
  p.o_sh = a->o_stride_h;
  p.lse = a->lse;
  p.m = a->m;
  p.l = a->l;
  p.ml_st = a->ml_stride_t;
  p.ml_sh = a->ml_stride_h;
  const int group = a->num_q_heads / a->num_kv_heads;
  const int64_t wgs = (int64_t)8 * group * p.nz * p.kv_slots * a->batch;
  if (wgs > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  hipLaunchKernelGGL((prefill_kernel<T, MODE>), dim3((unsigned)wgs), dim3(NWAVE * 64), 0, st, p);
  return check_launch();
}

static int validate(const lsattn_prefill_args* a, int mode) {
  if (!a || !a->q || !a->k || !a->v || !a->o) return LSATTN_ERR_INVALID_ARG;
  if (!a->q_b_start_loc || !a->q_b_seq_len || !a->q_first_token_global_idx || !a->kv_b_start_loc || !a->kv_b_seq_len ||
      !a->kv_first_token_global_idx)
    return LSATTN_ERR_INVALID_ARG;
  if (a->batch < 0 || a->num_q_heads <= 0 || a->num_kv_heads <= 0 || a->sp_peers < 1 || a->max_q_len < 0)
    return LSATTN_ERR_INVALID_ARG;
  if (a->num_q_heads % a->num_kv_heads) return LSATTN_ERR_INVALID_ARG;
  if (a->head_dim != 128) return LSATTN_ERR_UNSUPPORTED;
  if (a->dtype != LSATTN_F16 && a->dtype != LSATTN_BF16) return LSATTN_ERR_UNSUPPORTED;
  // 16-byte operand loads / 8- or 16-byte output stores
  if (a->q_stride_t % 8 || a->q_stride_h % 8 || a->k_stride_t % 8 || a->k_stride_h % 8 || a->v_stride_t % 8 || a->v_stride_h % 8)
    return LSATTN_ERR_INVALID_ARG;
  if (a->o_stride_t % 4 || a->o_stride_h % 4) return LSATTN_ERR_INVALID_ARG;
  if (((uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o) & 15) return LSATTN_ERR_INVALID_ARG;
  if (mode == 0) {
    if (!a->lse || a->o_dtype != LSATTN_F32) return LSATTN_ERR_INVALID_ARG;
  } else {
    if (!a->m || !a->l || a->o_dtype != a->dtype) return LSATTN_ERR_INVALID_ARG;
  }
  return LSATTN_OK;
}

}  // namespace lsattn

using namespace lsattn;

extern "C" int lsattn_prefill_step(const lsattn_prefill_args* a, void* stream) {
  const int rc = validate(a, 0);
  if (rc != LSATTN_OK) return rc;
  if (a->batch == 0 || a->max_q_len == 0) return LSATTN_OK;
  return a->dtype == LSATTN_F16 ? launch_prefill<F16, 0>(a, (hipStream_t)stream) : launch_prefill<BF16, 0>(a, (hipStream_t)stream);
}

extern "C" int lsattn_prefill_step_merge(const lsattn_prefill_args* a, void* stream) {
  const int rc = validate(a, 1);
  if (rc != LSATTN_OK) return rc;
  if (a->batch == 0 || a->max_q_len == 0) return LSATTN_OK;
  return a->dtype == LSATTN_F16 ? launch_prefill<F16, 1>(a, (hipStream_t)stream) : launch_prefill<BF16, 1>(a, (hipStream_t)stream);
}
