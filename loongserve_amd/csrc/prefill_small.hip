// The prefill attention step for head sizes 16, 32 and 64 (the reference's Triton kernel takes them beside 128:
// loongserve/models/llama/triton_kernel/ring_context_flashattention_nopad.py:248-250), gfx950, wave64.
//
// Same arithmetic as the 128-wide kernel of prefill.hip in a plain form: no LLaMA-family model the reference serves has
// such heads, so this kernel is built to be exact and free of hidden copies, not tuned tile by tile.
//   * a workgroup of eight waves owns 128 consecutive query positions of one query head, a wave 16 of them; K and V
//     tiles of 64 keys are staged through LDS by all threads (global -> registers -> LDS, the next tile requested
//     before the present one is worked on; bfloat16 V converted to fp16 on the way), one barrier per tile;
//   * scores transposed, S^T = K Q^T with v_mfma_f32_16x16x32 (a head of 16 fills half of the contraction with
//     zeros), 32 keys per step, so a lane owns one query column: running max and sum are in-lane work plus an exchange
//     between the four lanes of a column, and the fp32 scores turn into the B operand of O^T += V^T P^T in place (P and
//     V as fp16, as in the 128-wide kernel); V^T operands through ds_read_b64_tr_b16; a wave skips the steps none of
//     its rows sees;
//   * the three epilogues of the 128-wide kernel: 0 the step's fp32 partial (O, LSE), 1 the reference's in-place
//     (o, m, l) update (ring_context_flashattention_nopad.py:171-188), 2 the LSE merge into a running fp32 (O, LSE).
#include <type_traits>

#include "common.hip.h"

namespace lsattn {
namespace {

typedef __attribute__((address_space(3))) i16x4* lds_i16x4_ptr;

template <typename T> struct MfmaS;
template <> struct MfmaS<F16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct MfmaS<BF16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// bfloat16 -> fp16, round toward zero: exact in fp16's normal range, larger magnitudes become +-65504
__device__ __forceinline__ u32x4 bf16_to_f16(const u32x4& w) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float lo, hi;
    unpack2<BF16>(w[i], lo, hi);
    r[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
  return r;
}

// lanes c, c + 16, c + 32, c + 48 hold the four parts of query column c
__device__ __forceinline__ float xor16(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
__device__ __forceinline__ float xor32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}
__device__ __forceinline__ float col_max(float v) {
  v = fmaxf(v, xor16(v));
  return fmaxf(v, xor32(v));
}
__device__ __forceinline__ float col_sum(float v) {
  v += xor16(v);
  return v + xor32(v);
}

struct SmallParams {
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
  const int32_t* o_start;
  int32_t hq, heads_per_kv, peers, v_f16;
  float scale_log2;
  void* o;
  int64_t o_st, o_sh;
  float* lse;
  float* m;
  float* l;
  int64_t ml_st, ml_sh;
};

constexpr int kWaves = 8;   // waves per workgroup
constexpr int kQB = 1;      // blocks of 16 query positions per wave: 128 positions of one head per workgroup (two blocks,
                            // which share every K and V operand read, measured no faster: the waves wait on their own chains of
                            // dependent steps, and there are half as many of them to fill the gaps)
constexpr int kRows = kWaves * kQB * 16;
constexpr int kTile = 64;   // keys per LDS tile

template <typename T, int D, int MODE>
__global__ __launch_bounds__(kWaves * 64) void prefill_small_kernel(SmallParams p) {
  constexpr int KS = D >= 32 ? D / 32 : 1;  // contraction steps of Q K^T (32 elements each; D = 16 fills half of one)
  constexpr int NDB = D / 16;               // 16-wide blocks of the head
  constexpr int CPR = D / 8;                // 16-byte chunks per K or V row
  constexpr int NCH = kTile * CPR;          // chunks per tile: at most one per thread (512 for D = 64)
  constexpr int RB = D * 2 + 16;            // bytes per row in LDS (padded: neighbouring rows start in different banks)
  constexpr int TB = kTile * RB;            // bytes per tile
  static_assert(NCH <= kWaves * 64, "one chunk per thread and tile");
  // two stages of (K tile, V tile): the next tile is written while the present one is read
  __shared__ __attribute__((aligned(16))) char lds[2 * 2 * TB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int b = blockIdx.z, h = blockIdx.y;
  const int q_len = p.q_len[b];
  const int m_wg = (int)blockIdx.x * kRows;
  if (m_wg >= q_len) return;  // (the whole workgroup: the loop below holds barriers)
  const int m0 = m_wg + wave * (kQB * 16);  // the wave's first position
  const int kv_len = p.kv_len[b], qf = p.q_first[b], kf = p.kv_first[b], P = p.peers;
  const int64_t q_start = p.q_start[b], kv_start = p.kv_start[b];
  const int64_t o_start = p.o_start ? (int64_t)p.o_start[b] : q_start;
  const int kvh = h / p.heads_per_kv;

  // keys of this KV chunk visible to global query position qpos (ring_context_flashattention_nopad.py:156-159)
  auto visible_keys = [&](int qpos) -> int {
    const int dq = qpos - kf;
    const int n = dq >= 0 ? dq / P + 1 : 0;
    return n > kv_len ? kv_len : n;
  };
  // per block qb of 16 positions: the lane's position m0 + 16 qb + c, whether it exists, the keys it sees
  bool in_range[kQB];
  int cnt[kQB];
  u32x4 qreg[kQB][KS];  // Q^T as B operands: qreg[qb][ks] = Q[position][32 ks + 8 g .. + 7]
  f32x4 oacc[kQB][NDB]; // O^T: oacc[qb][db][j] = O[position][16 db + 4 g + j]
  float m_run[kQB], l_run[kQB];  // log2-domain running max of the column; the lane's share of its running sum
#pragma unroll
  for (int qb = 0; qb < kQB; qb++) {
    const int m = m0 + 16 * qb + c;
    in_range[qb] = m < q_len;
    cnt[qb] = in_range[qb] ? visible_keys(qf + m * P) : 0;
    const char* src = (const char*)p.q + ((q_start + (in_range[qb] ? m : m_wg)) * p.q_st + (int64_t)h * p.q_sh) * 2;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const int d0 = 32 * ks + 8 * g;
      qreg[qb][ks] = d0 < D ? *(const u32x4*)(src + d0 * 2) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int db = 0; db < NDB; db++) oacc[qb][db] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
  }
  // (positions ascend: a later row sees at least as many keys)
  auto last_seen = [&](int first, int rows) -> int {  // keys the last existing position of [first, first + rows) sees; 0 if none exists
    return first < q_len ? visible_keys(qf + (first + rows - 1 < q_len ? first + rows - 1 : q_len - 1) * P) : 0;
  };
  const int cnt_wave = last_seen(m0, kQB * 16);
  const int cnt_first = m0 < q_len ? visible_keys(qf + m0 * P) : 0;
  const int cnt_wg = last_seen(m_wg, kRows);

  const char* kbase = (const char*)p.k + (kv_start * p.k_st + (int64_t)kvh * p.k_sh) * 2;
  const char* vbase = (const char*)p.v + (kv_start * p.v_st + (int64_t)kvh * p.v_sh) * 2;
  const int last_key = kv_len - 1;
  // staging: thread `tid` carries chunk `tid` of the K tile and of the V tile (row tid / CPR, 16 bytes at 8 (tid % CPR))
  const bool stager = tid < NCH;
  const int st_row = tid / CPR, st_cc = tid % CPR;
  const int st_at = st_row * RB + st_cc * 16;
  u32x4 kst = {0u, 0u, 0u, 0u}, vst = {0u, 0u, 0u, 0u};
  auto request = [&](int t) __attribute__((always_inline)) {
    if (stager) {
      const int key = t * kTile + st_row < last_key ? t * kTile + st_row : last_key;  // (rows past the end repeat the last one and are masked)
      kst = *(const u32x4*)(kbase + ((int64_t)key * p.k_st + 8 * st_cc) * 2);
      vst = *(const u32x4*)(vbase + ((int64_t)key * p.v_st + 8 * st_cc) * 2);
    }
  };
  auto deposit = [&](int stage) __attribute__((always_inline)) {
    if (stager) {
      *(u32x4*)(lds + stage * 2 * TB + st_at) = kst;
      *(u32x4*)(lds + stage * 2 * TB + TB + st_at) = (std::is_same<T, BF16>::value && !p.v_f16) ? bf16_to_f16(vst) : vst;
    }
  };
  // transposing read: lane c of a 16-lane group points at row c >> 2, columns 4 (c & 3) .. + 3 of a 4 x 16 block and
  // receives column c of it; group g takes rows 4 g .. 4 g + 3 and, sixteen rows on, 16 + 4 g .. + 3: the eight keys
  // whose scores the lane holds
  const int vread0 = (4 * g + (c >> 2)) * RB + 4 * (c & 3) * 2;
  const int kread0 = c * RB + 8 * g * 2;

  const int nt = (cnt_wg + kTile - 1) / kTile;  // the same for every wave of the workgroup
  if (nt > 0) {
    request(0);
    deposit(0);
    __syncthreads();
  }
  for (int t = 0; t < nt; t++) {
    if (t + 1 < nt) request(t + 1);
    const char* kl = lds + (t & 1) * 2 * TB;
    const char* vl = kl + TB;
#pragma unroll
    for (int half = 0; half < 2; half++) {
      const int k0 = t * kTile + 32 * half;
      if (k0 >= cnt_wave) continue;  // (wave-uniform: none of the wave's rows sees these keys)
      // S^T = K Q^T: s[qb][kb][j] = score of key k0 + 16 kb + 4 g + j for the lane's query of block qb; a K operand
      // serves both blocks
      f32x4 s[kQB][2];
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int qb = 0; qb < kQB; qb++) s[qb][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          const int d0 = 32 * ks + 8 * g;
          const u32x4 ka = d0 < D ? *(const u32x4*)(kl + (32 * half + 16 * kb) * RB + kread0 + 64 * ks) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int qb = 0; qb < kQB; qb++) s[qb][kb] = MfmaS<T>::run(ka, qreg[qb][ks], s[qb][kb]);
        }
      }
      u32x4 pk[kQB];  // P^T as B operands: the lane's eight keys are contraction slots 8 g .. 8 g + 7, the order the V^T operand uses
#pragma unroll
      for (int qb = 0; qb < kQB; qb++) {
        if (k0 + 32 > cnt_first) {  // (wave-uniform: the wave's first row, which sees the fewest keys, does not see the whole step)
#pragma unroll
          for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int j = 0; j < 4; j++) s[qb][kb][j] = k0 + 16 * kb + 4 * g + j < cnt[qb] ? s[qb][kb][j] : -INFINITY;
        }
        const float mx = fmaxf(fmaxf(fmaxf(s[qb][0][0], s[qb][0][1]), fmaxf(s[qb][0][2], s[qb][0][3])),
                               fmaxf(fmaxf(s[qb][1][0], s[qb][1][1]), fmaxf(s[qb][1][2], s[qb][1][3])));
        const float m_new = fmaxf(m_run[qb], col_max(mx) * p.scale_log2);  // (the scale is positive)
        if (__builtin_amdgcn_ballot_w64(m_new != m_run[qb]) != 0) {
          const float alpha = exp2_diff(m_run[qb], m_new);
          l_run[qb] *= alpha;
#pragma unroll
          for (int db = 0; db < NDB; db++) oacc[qb][db] *= alpha;
          m_run[qb] = m_new;
        }
        const float neg_m = m_run[qb] == -INFINITY ? 0.f : -m_run[qb];  // (a row that has seen no key yet: every P below is 0)
        float pv[8], ps = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int j = 0; j < 4; j++) {
            pv[4 * kb + j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][kb][j], p.scale_log2, neg_m));
            ps += pv[4 * kb + j];
          }
        l_run[qb] += ps;
#pragma unroll
        for (int e = 0; e < 4; e++) pk[qb][e] = pack2<F16>(pv[2 * e], pv[2 * e + 1]);
      }
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        const int at = (int)(uintptr_t)(const __attribute__((address_space(3))) char*)vl + 32 * half * RB + vread0 + db * 32;
        const i16x4 xa = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)at);
        const i16x4 xb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(at + 16 * RB));
        const u32x2 wa = __builtin_bit_cast(u32x2, xa), wb = __builtin_bit_cast(u32x2, xb);
        const u32x4 va = u32x4{wa[0], wa[1], wb[0], wb[1]};
#pragma unroll
        for (int qb = 0; qb < kQB; qb++) oacc[qb][db] = MfmaS<F16>::run(va, pk[qb], oacc[qb][db]);
      }
    }
    // the next tile into the other stage (last read one barrier ago), then everyone meets: that tile is complete and
    // this one is done with
    if (t + 1 < nt) deposit((t + 1) & 1);
    __syncthreads();
  }

  // ---- epilogues (the 128-wide kernel's), block by block of 16 positions ----
#pragma unroll
  for (int qb = 0; qb < kQB; qb++) {
    const int mb = m0 + 16 * qb;
    if (mb >= q_len) break;  // (wave-uniform: a block without positions; it only helped to stage)
    const float l_tot = col_sum(l_run[qb]);
    const bool here = in_range[qb];
    const int64_t tok = o_start + (here ? mb + c : mb);
    if (MODE == 0) {
      if (here) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        float* orow = (float*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
        for (int db = 0; db < NDB; db++) *(f32x4*)(orow + db * 16 + 4 * g) = oacc[qb][db] * inv;
        if (g == 0) p.lse[tok * p.hq + h] = l_tot > 0.f ? (m_run[qb] + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
      }
    }
    if (MODE == 1) {
      // the reference's update of (o, m, l); a row in its start state (m = -inf, l = 0) may hold anything in o
      const int64_t at = tok * p.ml_st + (int64_t)h * p.ml_sh;
      const float m_old = p.m[at], l_old = p.l[at];
      const float M = fmaxf(m_run[qb], m_old);
      const bool upd = here && M != -INFINITY && l_tot > 0.f;
      float L = 0.f;
      if (upd) {
        const float w_old = l_old * exp2_diff(m_old, M);
        const float w_new = exp2_diff(m_run[qb], M);
        L = w_old + l_tot * w_new;
        const float inv = 1.f / L;
        uint16_t* orow = (uint16_t*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
          if (w_old != 0.f) {
            const u32x2 old = *(const u32x2*)(orow + db * 16 + 4 * g);
            unpack2<T>(old[0], o0, o1);
            unpack2<T>(old[1], o2, o3);
          }
          const float r0 = (o0 * w_old + oacc[qb][db][0] * w_new) * inv, r1 = (o1 * w_old + oacc[qb][db][1] * w_new) * inv;
          const float r2 = (o2 * w_old + oacc[qb][db][2] * w_new) * inv, r3 = (o3 * w_old + oacc[qb][db][3] * w_new) * inv;
          *(u32x2*)(orow + db * 16 + 4 * g) = u32x2{pack2<T>(r0, r1), pack2<T>(r2, r3)};
        }
      }
      // (the four lanes of a column all read the old m and l above, in the same instruction as the one that writes them below)
      if (upd && g == 0) {
        p.m[at] = M;
        p.l[at] = L;
      }
    }
    if (MODE == 2) {
      // fold the step's partial into the running fp32 (O, LSE); a row that saw no key stays as it is
      const bool upd = here && l_tot > 0.f;
      const float a_old = p.lse[tok * p.hq + h] * kLog2e;
      float new_lse = 0.f;
      if (upd) {
        const float a_new = m_run[qb] + __builtin_amdgcn_logf(l_tot);
        const float top = fmaxf(a_old, a_new);
        const float w_old = exp2_diff(a_old, top);
        const float w_new = __builtin_amdgcn_exp2f(a_new - top);
        const float W = w_old + w_new;
        const float c_old = w_old / W, c_new = w_new / (W * l_tot);
        float* orow = (float*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          // an empty row (lse = -inf) may hold anything: its old values are dropped, not multiplied by zero
          const f32x4 keep = w_old != 0.f ? *(const f32x4*)(orow + db * 16 + 4 * g) : f32x4{0.f, 0.f, 0.f, 0.f};
          *(f32x4*)(orow + db * 16 + 4 * g) = keep * c_old + oacc[qb][db] * c_new;
        }
        new_lse = (top + __builtin_amdgcn_logf(W)) * kLn2;
      }
      if (upd && g == 0) p.lse[tok * p.hq + h] = new_lse;
    }
  }
}

template <typename T, int D, int MODE> int launch(const SmallParams& p, const lsattn_prefill_args* a, hipStream_t st) {
  const int64_t tiles = (a->max_q_len + kRows - 1) / kRows;  // workgroups per head and request
  if (tiles > 0x7fffffff || a->num_q_heads > 65535 || a->batch > 65535) return LSATTN_ERR_INVALID_ARG;
  LSATTN_LAUNCH_KERNEL((prefill_small_kernel<T, D, MODE>), dim3((unsigned)tiles, (unsigned)a->num_q_heads, (unsigned)a->batch),
                     dim3(kWaves * 64), 0, st, p);
  return check_launch();
}

template <typename T, int MODE> int launch_d(const SmallParams& p, const lsattn_prefill_args* a, hipStream_t st) {
  switch (a->head_dim) {
    case 16: return launch<T, 16, MODE>(p, a, st);
    case 32: return launch<T, 32, MODE>(p, a, st);
    case 64: return launch<T, 64, MODE>(p, a, st);
    default: return LSATTN_ERR_UNSUPPORTED;
  }
}

template <typename T> int launch_mode(const SmallParams& p, const lsattn_prefill_args* a, int mode, hipStream_t st) {
  switch (mode) {
    case 0: return launch_d<T, 0>(p, a, st);
    case 1: return launch_d<T, 1>(p, a, st);
    case 2: return launch_d<T, 2>(p, a, st);
    default: return LSATTN_ERR_INVALID_ARG;
  }
}

}  // namespace

// One prefill step with head_dim 16, 32 or 64 (arguments already validated; epilogue `mode` as in the 128-wide kernel).
int launch_prefill_small(const lsattn_prefill_args* a, int mode, hipStream_t st) {
  SmallParams p;
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
  p.o_start = a->o_b_start_loc;
  p.hq = (int32_t)a->num_q_heads;
  p.heads_per_kv = (int32_t)(a->num_q_heads / a->num_kv_heads);
  p.peers = (int32_t)a->sp_peers;
  p.v_f16 = a->v_is_f16;
  p.scale_log2 = a->sm_scale * kLog2e;
  p.o = a->o;
  p.o_st = a->o_stride_t;
  p.o_sh = a->o_stride_h;
  p.lse = a->lse;
  p.m = a->m;
  p.l = a->l;
  p.ml_st = a->ml_stride_t;
  p.ml_sh = a->ml_stride_h;
  return a->dtype == LSATTN_F16 ? launch_mode<F16>(p, a, mode, st) : launch_mode<BF16>(p, a, mode, st);
}

}  // namespace lsattn
