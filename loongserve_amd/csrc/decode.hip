// Token-indexed flash decoding for gfx950: stage 1 (gather + split-K partials) and
// stage 2 (LSE merge over the block axis).
//
// Stage 1 replaces flash_decoding_stage1_kernel
// (longserve_cuda_kernels/src/flash_decoding_stage1.cu:25-143).  Differences by design:
//   * one wave64 serves one KV head and up to eight query heads of its GQA group (four at a time, in
//     up to two rounds over the rows it has loaded; larger groups take several waves), so a K/V row is
//     fetched once per group instead of once per query head;
//   * a K/V row of 128 16-bit elements is read by 16 lanes x 16 bytes; a wave has four
//     such lane groups and every group keeps 8 K rows and 8 V rows in flight;
//   * each lane group runs its own online softmax; groups are merged once per block with
//     an LSE merge, and the partial is written with plain stores (no atomics), so the
//     result is deterministic;
//   * a workgroup walks several consecutive blocks, so the launch is sized for the chip
//     and not for block_seq.
#include <atomic>
#include <type_traits>

#include "common.hip.h"

namespace lsattn {

struct Stage1Params {
  float* mid_o;
  float* mid_lse;
  const void* q;
  const void* k;
  const void* v;
  int64_t k_s0, k_s1, v_s0, v_s1;
  float scale_log2;  // sm_scale * log2(e)
  const int32_t* req_to_tokens;
  const int32_t* b_req_idx;
  const int32_t* b_seqlen;
  int64_t batch, hq, hkv, num_blocks, max_seq_len, block_seq, grid_blocks;  // block_seq: tokens per partial computed
  int64_t row_mul, fine_block_seq;  // partial of coarse block i goes to row i * row_mul; rows in between are marked empty
  int64_t blk_rows, req_rows;       // rows of mid_o between consecutive blocks / requests: (batch * hq, hq) in the reference's layout
  int32_t blocks_per_wg;  // consecutive blocks walked by one workgroup
  int32_t tasks;          // hkv * (group / GT) wave tasks
  int32_t tasks_on_x;     // grid = (task groups, chunks, batch) instead of (chunks, task groups, batch)
};

constexpr int kTok = 8;  // K/V rows in flight per 16-lane group

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): loop indices that must be constant expressions
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// sum over two packed 16-bit products with fp32 accumulation (v_dot2c_f32_f16 / v_dot2c_f32_bf16)
template <typename T> __device__ __forceinline__ float dot2acc(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float dot2acc<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}
template <> __device__ __forceinline__ float dot2acc<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}
// the same as volatile inline assembly, for sequences whose instruction order is fixed by hand
template <typename T> struct Dot;
template <> struct Dot<F16> {
  static __device__ __forceinline__ void first(float& d, uint32_t a, uint32_t b) { asm volatile("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b)); }
  static __device__ __forceinline__ void next(float& d, uint32_t a, uint32_t b) { asm volatile("v_dot2c_f32_f16 %0, %1, %2" : "+v"(d) : "v"(a), "v"(b)); }
};
template <> struct Dot<BF16> {
  static __device__ __forceinline__ void first(float& d, uint32_t a, uint32_t b) { asm volatile("v_dot2_f32_bf16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b)); }
  static __device__ __forceinline__ void next(float& d, uint32_t a, uint32_t b) { asm volatile("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(d) : "v"(a), "v"(b)); }
};

// SPLIT: the NW waves of a workgroup share one task and take every NW-th batch of 32 tokens of a block; their partials
// meet in LDS.  For launches too small to fill the chip otherwise (short contexts at small batch): NW times as many rows
// in flight.
// ONCE: every K/V row is read by one wave only (at most GT query heads per KV head), so the rows are loaded
// non-temporally; otherwise the waves that take the other query heads of the group read them again and ordinary loads let
// those find the rows in L2.
template <typename T, int GT, int NW, bool SPLIT, bool ONCE, int HR>
__global__ __launch_bounds__(NW * 64) void decode_stage1_kernel(Stage1Params p) {
  constexpr int GH = GT * HR;  // query heads per task
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int grp = lane >> 4;   // which of the 4 row slots of the wave
  const int sub = lane & 15;   // 16-byte column slot: elements sub*8 .. sub*8+7
  const int jbase = (sub >> 2) * 2;  // first of the two rows whose scores this lane finishes (see the reduction)
  const int64_t b = blockIdx.z;
  // The workgroups that read the other KV heads of the same tokens are next to this one in dispatch order when the
  // task index is the fastest grid dimension: the pieces of a token's K (and V) span are then fetched close together in
  // time (measured 2 % faster on GQA 32/8, two task groups per chunk).
  const int task = SPLIT ? (int)(p.tasks_on_x ? blockIdx.x : blockIdx.y) : (int)(p.tasks_on_x ? blockIdx.x : blockIdx.y) * NW + wave;
  if (task >= p.tasks) return;  // (SPLIT: the same for every wave of the workgroup, like the block range below)
  // a task = one KV head and up to GT query heads of its group; the last task of a group whose size is not a multiple of
  // GT has fewer (nh): its spare accumulators repeat the last query head and are not written
  const int group = (int)(p.hq / p.hkv);
  const int sub_groups = (group + GH - 1) / GH;
  const int kvh = task / sub_groups;
  const int sg = task % sub_groups;
  const int qh0 = kvh * group + sg * GH;
  const int nh = group - sg * GH < GH ? group - sg * GH : GH;

  const int len = p.b_seqlen[b];  // positions inside a request are 32-bit (max_seq_len is checked on the host)
  int64_t nblk = len <= 0 ? 0 : ((int64_t)len + p.block_seq - 1) / p.block_seq;
  if (nblk > p.grid_blocks) nblk = p.grid_blocks;
  if (nblk > (p.num_blocks + p.row_mul - 1) / p.row_mul) nblk = (p.num_blocks + p.row_mul - 1) / p.row_mul;
  int64_t fine_nblk = len <= 0 ? 0 : ((int64_t)len + p.fine_block_seq - 1) / p.fine_block_seq;  // rows the request reaches
  if (fine_nblk > p.num_blocks) fine_nblk = p.num_blocks;
  // Workgroups go to the 8 XCDs round-robin in linear id order, so a fixed chunk index always lands on the same XCDs and
  // the first chunks (all that short requests have) would load some XCDs more than others; the chunk index is rotated by
  // the request index to spread them (batch 64 with lengths 4096..32768: 5.62 -> 5.9 TB/s).
  const unsigned n_chunks = p.tasks_on_x ? gridDim.y : gridDim.x;
  const unsigned chunk = ((p.tasks_on_x ? blockIdx.y : blockIdx.x) + (unsigned)b) % n_chunks;
  const int64_t blk_begin = (int64_t)chunk * p.blocks_per_wg;
  int64_t blk_end = blk_begin + p.blocks_per_wg;
  if (blk_end > nblk) blk_end = nblk;
  if (blk_begin >= blk_end) return;

  const int32_t* table = p.req_to_tokens + (int64_t)p.b_req_idx[b] * p.max_seq_len;
  const char* kbase = (const char*)p.k + ((int64_t)kvh * p.k_s1 + sub * 8) * 2;
  const char* vbase = (const char*)p.v + ((int64_t)kvh * p.v_s1 + sub * 8) * 2;
  const int64_t k_row_bytes = p.k_s0 * 2, v_row_bytes = p.v_s0 * 2;

  // q stays packed (8 elements = 4 words per head and lane); the scale is applied to the reduced dot
  u32x4 qw[GH];
#pragma unroll
  for (int h = 0; h < GH; h++) qw[h] = *(const u32x4*)((const char*)p.q + ((b * p.hq + qh0 + (h < nh ? h : nh - 1)) * 128 + sub * 8) * 2);

  for (int64_t blk = blk_begin; blk < blk_end; blk++) {
    const int t0 = (int)(blk * p.block_seq);
    const int64_t t1_64 = (int64_t)t0 + p.block_seq;
    const int t1 = t1_64 > len ? len : (int)t1_64;
    const int t_last = t1 - 1;

    float m[GH], l[GH], o[GH][8];
#pragma unroll
    for (int h = 0; h < GH; h++) {
      m[h] = -INFINITY;
      l[h] = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i++) o[h][i] = 0.f;
    }

    // Slot indices of the first batch of rows.  A row position past the block repeats the block's
    // last row (always a real slot): it is loaded like any other and dropped by the validity mask,
    // so the loop body has no divergent control flow.
    constexpr int kStep = 4 * kTok * (SPLIT ? NW : 1);
    const int it0 = t0 + (SPLIT ? wave * 4 * kTok : 0);
    int32_t slot[kTok];
#pragma unroll
    for (int j = 0; j < kTok; j++) {
      const int tok = it0 + j * 4 + grp;
      slot[j] = table[tok < t1 ? tok : t_last];
    }

    for (int it = it0; it < t1; it += kStep) {
      u32x4 kr[kTok], vr[kTok];
      // (the empty statements keep each 64-bit address next to its load instead of sixteen of them live at once)
#pragma unroll
      for (int j = 0; j < kTok; j++) {
        asm volatile("" : "+v"(slot[j]));
        kr[j] = ONCE ? __builtin_nontemporal_load((const u32x4*)(kbase + (int64_t)slot[j] * k_row_bytes))
                     : *(const u32x4*)(kbase + (int64_t)slot[j] * k_row_bytes);
      }
#pragma unroll
      for (int j = 0; j < kTok; j++) {
        asm volatile("" : "+v"(slot[j]));
        vr[j] = ONCE ? __builtin_nontemporal_load((const u32x4*)(vbase + (int64_t)slot[j] * v_row_bytes))
                     : *(const u32x4*)(vbase + (int64_t)slot[j] * v_row_bytes);
      }
      // The rows are read once: non-temporal loads.  As ordinary loads they push the block partials (which stage 2
      // reads back) out of the caches early, and the trickle of write-backs between the reads costs the gather 5 %.
      // all 16 row loads are issued before anything else happens (the scheduler would otherwise sink
      // each load next to its first use and expose its latency)
      __builtin_amdgcn_sched_barrier(0);
      // slot indices of the next batch while the rows are in flight
#pragma unroll
      for (int j = 0; j < kTok; j++) {
        const int tok = it + kStep + j * 4 + grp;
        slot[j] = table[tok < t1 ? tok : t_last];
      }
      __builtin_amdgcn_sched_barrier(0);

      // HR rounds of GT query heads each over the rows just loaded (HR = 2: groups of 5 to 8 query heads per KV head
      // fetch every row once, not once per four heads)
      static_for<HR>([&](auto hr_tag) {
        constexpr int HB = decltype(hr_tag)::value * GT;
        // Partial dots over this lane's 8 elements for the 8 rows x GT heads of the group (value index
        // v = GT*j + h), then a transposing reduction over the 16 lanes of the row group: two halving steps
        // with bank-masked DPP adds (lanes with sub bits (3,2) = (B3,B2) keep values [NV/2*B3 + NV/4*B2, +NV/4))
        // and a sum over the quad.  Every lane ends with the finished raw scores of two rows,
        // jbase = 4*B3 + 2*B2 and jbase + 1, for all GT heads: w[GT*r + h].  The softmax scale is folded
        // into the exp2 argument.
        constexpr int NV = kTok * GT;
        float u[NV / 2], w[NV / 4];
        // Everything up to the quad sums is volatile inline assembly in a fixed order: a DPP read needs two
        // wait states after the write of its source, the compiler's hazard recogniser does not look into inline
        // assembly, and it would otherwise move the dots between the DPP adds.  The first halving step of a
        // value pair (v, v + NV/2) follows the dots of the next pair, so only two partial dots are live at a time.
        float lo_prev = 0.f, hi_prev = 0.f;
  #pragma unroll
        for (int i = 0; i < NV / 2; i++) {
          const int j = i / GT, h = i % GT;
          float lo, hi;
          Dot<T>::first(lo, qw[HB + h][0], kr[j][0]);
          Dot<T>::first(hi, qw[HB + h][0], kr[j + kTok / 2][0]);
  #pragma unroll
          for (int c = 1; c < 4; c++) {
            Dot<T>::next(lo, qw[HB + h][c], kr[j][c]);
            Dot<T>::next(hi, qw[HB + h][c], kr[j + kTok / 2][c]);
          }
          if (i > 0) {
            asm volatile("v_add_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0x3" : "=v"(u[i - 1]) : "v"(lo_prev));
            asm volatile("v_add_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xc" : "+v"(u[i - 1]) : "v"(hi_prev));
          }
          lo_prev = lo;
          hi_prev = hi;
        }
        asm volatile("s_nop 1");
        asm volatile("v_add_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0x3" : "=v"(u[NV / 2 - 1]) : "v"(lo_prev));
        asm volatile("v_add_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xc" : "+v"(u[NV / 2 - 1]) : "v"(hi_prev));
        asm volatile("s_nop 1");
  #pragma unroll
        for (int i = 0; i < NV / 4; i++) asm volatile("v_add_f32_dpp %0, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5" : "=v"(w[i]) : "v"(u[i]));
        asm volatile("s_nop 1");
  #pragma unroll
        for (int i = 0; i < NV / 4; i++) asm volatile("v_add_f32_dpp %0, %1, %1 row_ror:4 row_mask:0xf bank_mask:0xa" : "+v"(w[i]) : "v"(u[i + NV / 4]));
        asm volatile("s_nop 1");
  #pragma unroll
        for (int i = 0; i < NV / 4; i++) {
          w[i] += dpp_mov<0xB1>(w[i]);  // quad_perm [1,0,3,2]
          w[i] += dpp_mov<0x4E>(w[i]);  // quad_perm [2,3,0,1]
        }
        // rows past the block only exist in its last batch and are masked there
        const bool tail = it + 4 * kTok > t1;
        if (tail) {
  #pragma unroll
          for (int r = 0; r < 2; r++) {
            const bool valid = it + (jbase + r) * 4 + grp < t1;
  #pragma unroll
            for (int h = 0; h < GT; h++) w[GT * r + h] = valid ? w[GT * r + h] : -INFINITY;
          }
        }
        float pw[2 * GT];
        float alpha[GT];
        bool grow = false;
  #pragma unroll
        for (int h = 0; h < GT; h++) {
          float mx = fmaxf(w[h], w[GT + h]);
          mx = fmaxf(mx, dpp_mov<0x124>(mx));  // row_ror:4
          mx = fmaxf(mx, dpp_mov<0x128>(mx));  // row_ror:8: now the maximum over the 8 rows, in every lane
          const float m_new = fmaxf(m[HB + h], mx * p.scale_log2);  // scale > 0
          const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
          alpha[h] = __builtin_amdgcn_exp2f(m[HB + h] - m_safe);
          grow |= m_new != m[HB + h];
          pw[h] = __builtin_amdgcn_exp2f(__builtin_fmaf(w[h], p.scale_log2, -m_safe));
          pw[GT + h] = __builtin_amdgcn_exp2f(__builtin_fmaf(w[GT + h], p.scale_log2, -m_safe));
          float ps = pw[h] + pw[GT + h];
          ps += dpp_mov<0x124>(ps);
          ps += dpp_mov<0x128>(ps);
          l[HB + h] = l[HB + h] * alpha[h] + ps;
          m[HB + h] = m_new;
        }
        // the accumulators only need rescaling when some running max moved (rare once warmed up)
        if (__builtin_amdgcn_ballot_w64(grow) != 0) {
  #pragma unroll
          for (int h = 0; h < GT; h++)
  #pragma unroll
            for (int i = 0; i < 8; i++) o[HB + h][i] *= alpha[h];
        }
        if (std::is_same<T, F16>::value) {
          // O += P V on pairs of rows: the owners pack (p[2q], p[2q+1]) to fp16 (p <= 1), row pair q is
          // broadcast from lane 4q of the group, the two V rows are interleaved element by element
          uint32_t pp[GT];
  #pragma unroll
          for (int h = 0; h < GT; h++) pp[h] = pack2<F16>(pw[h], pw[GT + h]);
          static_for<kTok / 2>([&](auto q_tag) {
            constexpr int q = decltype(q_tag)::value;
            uint32_t bq[GT];
  #pragma unroll
            for (int h = 0; h < GT; h++) bq[h] = __builtin_bit_cast(uint32_t, dpp_mov<0x150 + 4 * q>(__builtin_bit_cast(float, pp[h])));  // row_newbcast
  #pragma unroll
            for (int w4 = 0; w4 < 4; w4++) {
              const uint32_t lo = __builtin_amdgcn_perm(vr[2 * q + 1][w4], vr[2 * q][w4], 0x05040100u);
              const uint32_t hi = __builtin_amdgcn_perm(vr[2 * q + 1][w4], vr[2 * q][w4], 0x07060302u);
  #pragma unroll
              for (int h = 0; h < GT; h++) {
                o[HB + h][2 * w4] = dot2acc<F16>(bq[h], lo, o[HB + h][2 * w4]);
                o[HB + h][2 * w4 + 1] = dot2acc<F16>(bq[h], hi, o[HB + h][2 * w4 + 1]);
              }
            }
          });
        } else {
          // bf16: a bf16 P would cost ~1e-3 relative error, so P stays fp32 and is broadcast row by row
          static_for<kTok>([&](auto j_tag) {
            constexpr int j = decltype(j_tag)::value;
            float vf[8];
            unpack8<T>(vr[j], vf);
  #pragma unroll
            for (int h = 0; h < GT; h++) {
              const float pb = dpp_mov<0x150 + 4 * (j >> 1)>(pw[GT * (j & 1) + h]);  // row_newbcast
  #pragma unroll
              for (int i = 0; i < 8; i++) o[HB + h][i] = __builtin_fmaf(pb, vf[i], o[HB + h][i]);
            }
          });
        }
      });
    }

    // merge the four lane groups (and, SPLIT, the waves) and write the block's partial
    __shared__ float xw[SPLIT ? NW : 1][GH][16][10];  // per wave, head and column slot: 8 sums, running max, row sum
    auto write_partial = [&](int h, float M, float L, const float (&ov)[8]) {
      if (h >= nh) return;
      const float inv = 1.f / L;
      const int64_t row = blk * p.row_mul * p.blk_rows + b * p.req_rows + qh0 + h;
      f32x4* dst = (f32x4*)(p.mid_o + row * 128 + sub * 8);
      dst[0] = f32x4{ov[0] * inv, ov[1] * inv, ov[2] * inv, ov[3] * inv};
      dst[1] = f32x4{ov[4] * inv, ov[5] * inv, ov[6] * inv, ov[7] * inv};
      if (sub == 0) p.mid_lse[row] = (M + __builtin_amdgcn_logf(L)) * kLn2;
      // the rows of the blocks merged into this partial (row_mul <= 16: lane `sub` takes the sub-th of them)
      if (sub >= 1 && sub < p.row_mul && blk * p.row_mul + sub < fine_nblk)
        p.mid_lse[(blk * p.row_mul + sub) * p.blk_rows + b * p.req_rows + qh0 + h] = -INFINITY;
    };
#pragma unroll
    for (int h = 0; h < GH; h++) {
      float M = fmaxf(m[h], __shfl_xor(m[h], 16));
      M = fmaxf(M, __shfl_xor(M, 32));
      const float w = exp2_diff(m[h], M);  // 0 for a group (or, SPLIT, a whole wave) that saw no row
      float L = l[h] * w;
      L += __shfl_xor(L, 16);
      L += __shfl_xor(L, 32);
      float ov[8];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        float x = o[h][i] * w;
        x += __shfl_xor(x, 16);
        x += __shfl_xor(x, 32);
        ov[i] = x;
      }
      if (grp == 0) {
        if (SPLIT) {
          float* dst = xw[wave][h][sub];
#pragma unroll
          for (int i = 0; i < 8; i++) dst[i] = ov[i];
          dst[8] = M;
          dst[9] = L;
        } else {
          write_partial(h, M, L, ov);  // the block holds >= 1 row, so M is finite and L > 0
        }
      }
    }
    if (SPLIT) {
      __syncthreads();
      if (wave == 0 && grp == 0) {
#pragma unroll
        for (int h = 0; h < GH; h++) {
          float M = xw[0][h][sub][8];
#pragma unroll
          for (int w = 1; w < NW; w++) M = fmaxf(M, xw[w][h][sub][8]);
          float L = 0.f, ov[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int w = 0; w < NW; w++) {
            const float* src = xw[w][h][sub];
            const float f = exp2_diff(src[8], M);
            L += src[9] * f;
#pragma unroll
            for (int i = 0; i < 8; i++) ov[i] += src[i] * f;
          }
          write_partial(h, M, L, ov);
        }
      }
      __syncthreads();  // the next block of this workgroup writes the same LDS
    }
  }
}

// ------------------------------------------------------------------------------------
// Stage 1 for large launches (any group size): both products on the matrix pipe.
// One wave64 = one KV head, up to 16 query heads of its group (the 16 columns of a 16x16x32 MFMA) and a run of
// consecutive blocks; the waves of a workgroup are independent (no barrier) and take neighbouring KV heads over the same
// tokens, whose rows lie side by side in memory.  A batch is 32 tokens:
//   the K and V rows are loaded the way the other stage-1 kernels load them, a whole 256-byte row per 16 lanes (loading the
//     MFMA operand layout straight from memory, 16 rows x 64 bytes per instruction, ran 20 % slower), double-buffered in
//     registers so that the rows of batch j + 1 are in flight while batch j is computed;
//   at compute time the wave turns its rows into operand layout through its own 17.5 KB of LDS (rows padded to 272 and
//     288 bytes, so that the sixteen rows of a K read and the eight rows of a transposing V read fall into different banks
//     and every address is one register plus an immediate): K rows are read back as the A operand of S = K Q^T (Q^T, the B operand, stays in registers), V rows are
//     read back transposed (ds_read_b64_tr_b16) as the A operand of O^T += V^T P^T;
//   the softmax runs on the accumulators (a lane holds one query head's scores of eight tokens), and P, converted in
//     place, is the B operand of the second product.  A bfloat16 P would cost about 1e-3 relative error, so bfloat16
//     inputs multiply V by the high and by the low part of P.
// All global loads are issued from inline assembly, so that the hand-placed waits leave exactly the next batch's rows
// outstanding; tests/test_prefill_isa_hazards.py checks that no register of a load in flight is touched before its wait.
// ------------------------------------------------------------------------------------
__device__ __forceinline__ float xlane16(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
}
__device__ __forceinline__ float xlane32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}
template <typename T> struct Mfma16;
template <> struct Mfma16<F16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mfma16<BF16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

constexpr int kMfmaWaves = 4;        // waves per workgroup (independent)
constexpr int kMfmaBatch = 32;       // tokens per batch
constexpr int kMfmaKRow = 272, kMfmaVRow = 288;  // padded row lengths in LDS (bytes)
constexpr int kMfmaStage = kMfmaBatch * (kMfmaKRow + kMfmaVRow);  // LDS bytes per wave: the K rows and the V rows of one batch

// WS (small launches with fewer than four tasks): the four waves of a workgroup share one task and one block, take every
// fourth batch of its tokens and merge their partials through LDS: four times the waves of the plain shape, each short.
// One unit of work of a workgroup: request b, task group bid_t, chunk group bid_c (of n_cgroups in the grid; LISTED: the
// unit comes from a list of the units that exist, and its chunk group is taken as it is).
// RANGE: the wave's unit is blocks [r_lo, r_hi) of the request instead (r_lo < r_hi <= the request's blocks), computed into
// one partial, which goes to row r_lo; the rows of the other blocks are left alone (the merge behind it knows which rows
// hold a partial).
// The lane's eight 16-byte pieces of a partial's row, 64 bytes apart, each scaled by `inv`.  The stores carry the
// system-scope bits: such a store goes through to memory as it is issued instead of waiting in the L2 as a dirty line
// that is written back later, alone, between the reads of a gather that keeps every memory channel busy.  Measured on
// a plain streaming read of 4 GiB with 8 KB stores mixed in: 67 MB of them (1.6 % of the bytes, what config 3 writes at
// one partial per 256 tokens) take the read from 6.47 to 5.65 TB/s as ordinary stores, to 5.94 with these bits; 4 MB
// (0.1 %) to 6.28 and 6.42.  Issued from inline assembly (the compiler has no store of this kind that is not atomic);
// a vector instruction may not overwrite the data registers of a store of more than 64 bits in the two cycles behind
// it, which the compiler knows of its own stores only: hence the s_nop.
__device__ __forceinline__ void store_partial_row(float* dst, const f32x4 (&acc)[8], const float inv) {
#define LSATTN_STORE_ROW_PIECE(db)                                                                                                  \
  {                                                                                                                                \
    const f32x4 piece = acc[db] * inv;                                                                                             \
    asm volatile("global_store_dwordx4 %0, %1, off offset:%2 sc0 sc1\n\ts_nop 1" : : "v"(dst), "v"(piece), "n"(64 * db) : "memory"); \
  }
  LSATTN_STORE_ROW_PIECE(0) LSATTN_STORE_ROW_PIECE(1) LSATTN_STORE_ROW_PIECE(2) LSATTN_STORE_ROW_PIECE(3)
  LSATTN_STORE_ROW_PIECE(4) LSATTN_STORE_ROW_PIECE(5) LSATTN_STORE_ROW_PIECE(6) LSATTN_STORE_ROW_PIECE(7)
#undef LSATTN_STORE_ROW_PIECE
}

template <typename T, bool WS, bool LISTED, bool RANGE = false>
__device__ __forceinline__ void stage1_mfma_unit(const Stage1Params& p, char* lds, const int lane, const int wave, const int64_t b,
                                                 const unsigned bid_t, const unsigned bid_c, const unsigned n_cgroups,
                                                 const int64_t r_lo = 0, const int64_t r_hi = 0) {
  const int n = lane & 15, g = lane >> 4;  // query head (column) or 16-byte chunk of a row / token group or row of four
  // The waves of a workgroup: tw of them on neighbouring tasks (KV heads: their rows of a token lie side by side in memory
  // and are then fetched at about the same time), the rest on consecutive chunks of tokens.
  const int tw = WS ? 1 : (p.tasks_on_x & 7), cw = WS ? 1 : kMfmaWaves / tw;
  const int task = WS ? (int)bid_t : bid_t * tw + (wave & (tw - 1));
  if (task >= p.tasks) return;
  const int group = (int)(p.hq / p.hkv);
  const int sub_groups = (group + 15) / 16;
  const int kvh = task / sub_groups;
  const int sg = task % sub_groups;
  const int qh0 = kvh * group + sg * 16;
  const int nh = group - sg * 16 < 16 ? group - sg * 16 : 16;

  const int len = p.b_seqlen[b];
  int64_t nblk = len <= 0 ? 0 : ((int64_t)len + p.block_seq - 1) / p.block_seq;
  if (nblk > p.grid_blocks) nblk = p.grid_blocks;
  if (nblk > (p.num_blocks + p.row_mul - 1) / p.row_mul) nblk = (p.num_blocks + p.row_mul - 1) / p.row_mul;
  int64_t fine_nblk = len <= 0 ? 0 : ((int64_t)len + p.fine_block_seq - 1) / p.fine_block_seq;
  if (fine_nblk > p.num_blocks) fine_nblk = p.num_blocks;
  const unsigned n_chunks = n_cgroups * cw;
  const unsigned wave_chunk = bid_c * cw + (WS ? 0 : wave >> (tw == 4 ? 2 : tw == 2 ? 1 : 0));
  const unsigned chunk = LISTED ? wave_chunk : (wave_chunk + (unsigned)b) % n_chunks;  // (rotated by the request, as above)
  const int64_t blk_begin = RANGE ? r_lo : (int64_t)chunk * p.blocks_per_wg;  // (WS: one block per workgroup)
  int64_t blk_end = RANGE ? r_hi : blk_begin + p.blocks_per_wg;
  if (blk_end > nblk) blk_end = nblk;
  if (blk_begin >= blk_end) return;  // (WS: the same for the four waves, which meet at a barrier below)
  const int bs = (int)p.block_seq;                    // a multiple of 32 (checked on the host)
  constexpr int kStep = WS ? kMfmaWaves * kMfmaBatch : kMfmaBatch;  // tokens from one of the wave's batches to its next
  const int t_begin = (int)(blk_begin * bs) + (WS ? wave * kMfmaBatch : 0);
  const int t_end = blk_end * bs > len ? len : (int)(blk_end * bs);
  const int t_last = t_end - 1;
  const int n_batches = t_begin < t_end ? (t_end - t_begin + kStep - 1) / kStep : 0;

  const int32_t* table = p.req_to_tokens + (int64_t)p.b_req_idx[b] * p.max_seq_len;
  const char* kbase = (const char*)p.k + ((int64_t)kvh * p.k_s1) * 2 + n * 16;
  const char* vbase = (const char*)p.v + ((int64_t)kvh * p.v_s1) * 2 + n * 16;
  const int64_t k_row_bytes = p.k_s0 * 2, v_row_bytes = p.v_s0 * 2;

  // Q^T as B operands: qb[ks] = Q[head n][32 ks + 8 g .. + 7] (zero for the spare columns)
  u32x4 qb[4];
  {
    const char* qrow = (const char*)p.q + ((b * p.hq + qh0 + (n < nh ? n : 0)) * 128 + 8 * g) * 2;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) qb[ks] = n < nh ? *(const u32x4*)(qrow + ks * 64) : u32x4{0, 0, 0, 0};
  }
  char* lds_k = lds + wave * kMfmaStage;
  char* lds_v = lds_k + kMfmaBatch * kMfmaKRow;
  // the lane writes chunk n of row 4 i + g (one register + 4 i rows as immediate), reads K row n (and 16 + n), chunk
  // 4 ks + g, and V through the transposing read: lane n of a group points at row 4 g + n / 4, elements 4 (n % 4) .. + 3 of a d-block
  char* kwrite0 = lds_k + g * kMfmaKRow + n * 16;
  char* vwrite0 = lds_v + g * kMfmaVRow + n * 16;
  const char* kread0 = lds_k + n * kMfmaKRow + g * 16;
  const int vread0 = (int)(uintptr_t)(__attribute__((address_space(3))) char*)lds_v + (4 * g + (n >> 2)) * kMfmaVRow + 8 * (n & 3);
  // Slot numbers of a batch: the lane loads chunk n of the rows of tokens 4 i + g; positions past the end repeat the last
  // row.  Issued from inline assembly like the data loads (one hand-kept count of outstanding loads).
  struct Slots {
    int v[8];
  };
  auto load_slots = [&](int t0, Slots& sl) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int tok = t0 + 4 * i + g;
      const uint32_t off = (uint32_t)(tok < t_last ? tok : t_last) * 4u;  // (a row of the table is shorter than 2^31 entries)
      asm volatile("global_load_dword %0, %1, %2" : "=v"(sl.v[i]) : "v"(off), "s"(table) : "memory");
    }
  };
  // waits until at most N loads are outstanding and makes the slot numbers of `sl` usable
  auto wait_slots = [&](auto n_tag, Slots& sl) __attribute__((always_inline)) {
    constexpr int N = decltype(n_tag)::value;
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(sl.v[0]), "+v"(sl.v[1]), "+v"(sl.v[2]), "+v"(sl.v[3]), "+v"(sl.v[4]), "+v"(sl.v[5]), "+v"(sl.v[6]), "+v"(sl.v[7])
                 : "n"(N)
                 : "memory");
  };
  // the 16 row loads of a batch: K rows into kr, V rows into vr (rows are read once: non-temporal)
  auto issue = [&](const Slots& sl, u32x4 (&kr)[8], u32x4 (&vr)[8]) __attribute__((always_inline)) {
    // (the 64-bit row address is formed next to its load, in a scratch register pair that dies with it: sixteen addresses
    // formed ahead of their loads would not fit the register file beside two batches of rows)
    const uint32_t krb = (uint32_t)k_row_bytes, vrb = (uint32_t)v_row_bytes;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      uint64_t addr;
      asm volatile("v_mad_u64_u32 %1, vcc, %2, %3, %4\n\tglobal_load_dwordx4 %0, %1, off nt"
                   : "=v"(kr[i]), "=&v"(addr) : "v"(sl.v[i]), "s"(krb), "v"(kbase) : "vcc", "memory");
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      uint64_t addr;
      asm volatile("v_mad_u64_u32 %1, vcc, %2, %3, %4\n\tglobal_load_dwordx4 %0, %1, off nt"
                   : "=v"(vr[i]), "=&v"(addr) : "v"(sl.v[i]), "s"(vrb), "v"(vbase) : "vcc", "memory");
    }
  };
  // waits until at most 24 loads (the slot numbers requested last and the next batch's rows) are outstanding and makes
  // kr / vr usable
  auto wait_rows = [&](u32x4 (&kr)[8], u32x4 (&vr)[8]) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(24)"
                 : "+v"(kr[0]), "+v"(kr[1]), "+v"(kr[2]), "+v"(kr[3]), "+v"(kr[4]), "+v"(kr[5]), "+v"(kr[6]), "+v"(kr[7]), "+v"(vr[0]),
                   "+v"(vr[1]), "+v"(vr[2]), "+v"(vr[3]), "+v"(vr[4]), "+v"(vr[5]), "+v"(vr[6]), "+v"(vr[7])
                 :
                 : "memory");
  };

  f32x4 oacc[8];
  float m = -INFINITY, l = 0.f;  // running maximum (log2 domain, the same in the four lanes of a head) / the lane's part of the sum
  auto reset = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int db = 0; db < 8; db++) oacc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    m = -INFINITY;
    l = 0.f;
  };
  reset();
  auto flush = [&](int64_t blk) __attribute__((always_inline)) {
    float lt = l + xlane16(l);
    lt += xlane32(lt);
    if (n < nh) {
      const float inv = 1.f / lt;  // a block holds at least one token
      const int64_t row = blk * p.row_mul * p.blk_rows + b * p.req_rows + qh0 + n;
      float* dst = p.mid_o + row * 128 + 4 * g;
      store_partial_row(dst, oacc, inv);
      if (g == 0) p.mid_lse[row] = (m + __builtin_amdgcn_logf(lt)) * kLn2;
      if (!RANGE) {
        // the rows of the blocks merged into this partial (row_mul <= 16: lane group g takes every fourth of them)
        for (int r = 1 + g; r < p.row_mul; r += 4)
          if (blk * p.row_mul + r < fine_nblk) p.mid_lse[(blk * p.row_mul + r) * p.blk_rows + b * p.req_rows + qh0 + n] = -INFINITY;
      }
    }
  };
  // one batch whose rows have arrived in kr / vr
  auto compute = [&](int t0, const u32x4 (&kr)[8], const u32x4 (&vr)[8]) __attribute__((always_inline)) {
    // rows into operand layout through the wave's LDS (the reads of the previous batch were consumed by its MFMAs)
#pragma unroll
    for (int i = 0; i < 8; i++) {
      *(u32x4*)(kwrite0 + 4 * i * kMfmaKRow) = kr[i];
      *(u32x4*)(vwrite0 + 4 * i * kMfmaVRow) = vr[i];
    }
    f32x4 s[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      s[h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        const u32x4 ka = *(const u32x4*)(kread0 + h * 16 * kMfmaKRow + ks * 64);
        s[h] = Mfma16<T>::run(ka, qb[ks], s[h]);
      }
    }
    // s[h][r] = score of token t0 + 16 h + 4 g + r for head n
    float mx = -INFINITY;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const bool valid = t0 + 16 * h + 4 * g + r < t_end;
        s[h][r] = valid ? s[h][r] * p.scale_log2 : -INFINITY;
        mx = fmaxf(mx, s[h][r]);
      }
    mx = fmaxf(mx, xlane16(mx));
    mx = fmaxf(mx, xlane32(mx));            // over the batch's 32 tokens (at least one is valid)
    const float m_new = fmaxf(m, mx);
    const float alpha = exp2_diff(m, m_new);
    if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
#pragma unroll
      for (int db = 0; db < 8; db++) oacc[db] *= alpha;
      l *= alpha;
    }
    m = m_new;
    float pv[8];
    float ps = 0.f;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        pv[4 * h + r] = __builtin_amdgcn_exp2f(s[h][r] - m_new);
        ps += pv[4 * h + r];
      }
    l += ps;
    // P^T as B operand: the lane's eight tokens are the contraction slots 8 g .. 8 g + 7, the order the V^T operand uses
    u32x4 phi, plo;
    if (std::is_same<T, F16>::value) {
#pragma unroll
      for (int e = 0; e < 4; e++) phi[e] = pack2<F16>(pv[2 * e], pv[2 * e + 1]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        // high part: P truncated to bfloat16; low part: the rest, rounded
        const uint32_t h0 = __builtin_bit_cast(uint32_t, pv[2 * e]) & 0xffff0000u, h1 = __builtin_bit_cast(uint32_t, pv[2 * e + 1]) & 0xffff0000u;
        phi[e] = (h0 >> 16) | h1;
        plo[e] = pack2<BF16>(pv[2 * e] - __builtin_bit_cast(float, h0), pv[2 * e + 1] - __builtin_bit_cast(float, h1));
      }
    }
#pragma unroll
    for (int db = 0; db < 8; db++) {
      const i16x4 xa = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(vread0 + db * 32));
      const i16x4 xb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(vread0 + db * 32 + 16 * kMfmaVRow));
      const u32x2 wa = __builtin_bit_cast(u32x2, xa), wb = __builtin_bit_cast(u32x2, xb);
      const u32x4 va = u32x4{wa[0], wa[1], wb[0], wb[1]};
      oacc[db] = Mfma16<T>::run(va, phi, oacc[db]);
      if (!std::is_same<T, F16>::value) oacc[db] = Mfma16<T>::run(va, plo, oacc[db]);
    }
  };
  auto finish_batch = [&](int t0) __attribute__((always_inline)) {
    if (WS) return;  // (the block's partial is merged from the four waves after the loop)
    if (RANGE) {  // (one partial for the whole range)
      if (t0 + kMfmaBatch >= t_end) flush(blk_begin);
      return;
    }
    if ((t0 + kMfmaBatch - t_begin) % bs == 0 || t0 + kMfmaBatch >= t_end) {
      flush(blk_begin + (t0 - t_begin) / bs);
      reset();
    }
  };

  // Order of the loads, oldest first, when batch j is about to be computed:  rows(j) | slots(j+2) | rows(j+1).  Loads return
  // in order, so the wait for vmcnt(24) ends when rows(j) have landed and leaves the other two groups in flight (a partial's
  // stores in between count too and only make a wait longer); slots(j+1), which rows(j+1) were addressed with, were the
  // oldest group one wait earlier (that vmcnt(24), in front of an issue, is a no-op except in the first trip).
  u32x4 kr0[8], vr0[8], kr1[8], vr1[8];
  Slots s_even, s_odd;
  load_slots(t_begin, s_even);
  load_slots(t_begin + kStep, s_odd);
  wait_slots(std::integral_constant<int, 8>{}, s_even);
  issue(s_even, kr0, vr0);
  // two batches per trip, so that the register set of a batch is a compile-time choice
  for (int j = 0; j < n_batches; j += 2) {
    const int t0 = t_begin + j * kStep;
    load_slots(t0 + 2 * kStep, s_even);                     // slots(j+2): rows(j) have been addressed
    wait_slots(std::integral_constant<int, 24>{}, s_odd);   // slots(j+1) usable
    issue(s_odd, kr1, vr1);                                 // rows(j+1) (past the end: the last row again, never used)
    wait_rows(kr0, vr0);
    compute(t0, kr0, vr0);
    finish_batch(t0);
    load_slots(t0 + 3 * kStep, s_odd);                      // slots(j+3)
    wait_slots(std::integral_constant<int, 24>{}, s_even);  // slots(j+2) usable
    issue(s_even, kr0, vr0);                                // rows(j+2)
    wait_rows(kr1, vr1);
    if (j + 1 < n_batches) {
      compute(t0 + kStep, kr1, vr1);
      finish_batch(t0 + kStep);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (rows requested past the end land before the registers are given back)
  if constexpr (WS) {
    // The four partials of the block meet in LDS (each wave's own 17.5 KB: its last batch's operands have been consumed);
    // every wave then finishes two of the eight d-blocks.  A wave without a batch of its own brings m = -inf, l = 0.
    float lt = l + xlane16(l);
    lt += xlane32(lt);
    f32x4* mine = (f32x4*)(lds + wave * kMfmaStage);
#pragma unroll
    for (int db = 0; db < 8; db++) mine[db * 64 + lane] = oacc[db];
    // (as a float vector: __builtin_bit_cast applied to an element of an integer vector, bit_cast(float, v[1]), compiled to a
    // read of element 0 with this compiler)
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    *(f32x2*)(lds + wave * kMfmaStage + 8192 + lane * 8) = f32x2{m, lt};
    __syncthreads();
    float mi[kMfmaWaves], li[kMfmaWaves], M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kMfmaWaves; w++) {
      const f32x2 ml = *(const f32x2*)(lds + w * kMfmaStage + 8192 + lane * 8);
      mi[w] = ml[0];
      li[w] = ml[1];
      M = fmaxf(M, mi[w]);
    }
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < kMfmaWaves; w++) {
      mi[w] = exp2_diff(mi[w], M);  // (the weight of wave w's partial; 0 for one that saw no token)
      L += li[w] * mi[w];
    }
    if (n < nh) {
      const float inv = 1.f / L;  // a block holds at least one token
      const int64_t row = blk_begin * p.row_mul * p.blk_rows + b * p.req_rows + qh0 + n;
      float* dst = p.mid_o + row * 128 + 4 * g;
#pragma unroll
      for (int d = 0; d < 2; d++) {
        const int db = 2 * wave + d;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kMfmaWaves; w++) acc += ((const f32x4*)(lds + w * kMfmaStage))[db * 64 + lane] * mi[w];
        *(f32x4*)(dst + 16 * db) = acc * inv;
      }
      if (wave == 0) {
        if (g == 0) p.mid_lse[row] = (M + __builtin_amdgcn_logf(L)) * kLn2;
        for (int r = 1 + g; r < p.row_mul; r += 4)
          if (blk_begin * p.row_mul + r < fine_nblk) p.mid_lse[(blk_begin * p.row_mul + r) * p.blk_rows + b * p.req_rows + qh0 + n] = -INFINITY;
      }
    }
  }
}

template <typename T, bool WS>
__global__ __launch_bounds__(kMfmaWaves * 64, 2) void decode_stage1_mfma_kernel(Stage1Params p) {
  __shared__ __attribute__((aligned(1024))) char lds[kMfmaWaves * kMfmaStage];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool tasks_first = !WS && (p.tasks_on_x & 8) != 0;  // grid = (task groups, chunk groups, batch): a chunk's task groups are dispatched together
  stage1_mfma_unit<T, WS, false>(p, lds, lane, wave, blockIdx.z, tasks_first ? blockIdx.x : blockIdx.y, tasks_first ? blockIdx.y : blockIdx.x,
                                 tasks_first ? gridDim.y : gridDim.x);
}

// The plain shape over a list of the units that exist.  The grid above has a workgroup for every (chunk group, task group)
// of the longest request times the batch, and the host does not know the lengths: a batch of one long request and many
// short ones is mostly workgroups that find nothing to do (one request of 131072 tokens with 255 of 512, 256 tokens per
// partial: a million workgroups for 5000 units; starting and ending them takes three times as long as the reads).  Here
// a fixed grid of two workgroups per CU walks the units: every workgroup first numbers the units of all requests (the
// first unit of each request, a prefix sum over the batch, in LDS), then takes units blockIdx.x, blockIdx.x + gridDim.x,
// ...; the request of a unit is found by bisection.  Within a request the task groups of a chunk group are
// neighbouring units, which run at the same time on neighbouring workgroups (all KV heads of a token are fetched together).
constexpr int kListedMaxBatch = 1024;
constexpr int64_t kListedFromWorkgroups = 32768;  // launches of the plain grid from which the list is walked instead
// ... and from a quarter of that when a partial covers 1024 tokens and more (the fused call's splits): with units that long
// a skewed batch has few of them, one to a CU at best, and the plain grid's empty workgroups stand in their way (131072 +
// 63 x 2048 tokens at 2048 per partial, 8192 workgroups: 0.217 -> 0.167 ms; at 1024, 16384 workgroups: 0.207 -> 0.176);
// batches of one length lose under one percent (64 x 65536 at 1024: 2.777 -> 2.80 ms).  At 256 tokens per partial the
// list costs an even batch more than that (config 3, 16384 workgroups: 947 -> 962 us) and stays with the larger grids.
constexpr int64_t kListedFromWorkgroupsCoarse = 8192;
constexpr int64_t kListedCoarseTokens = 1024;
constexpr int64_t kCUs = 256;                     // compute units of the MI355X
constexpr int64_t kSharesMinBatch = 8;            // ... and from this many requests on (a few long requests: 4 x 131072 and 1 x 1048576 tokens measured 1 % behind the grids)
constexpr int64_t kSharesMinBlocks = 4;           // equal shares from this many blocks per worker on (an upper bound from the longest request)
template <typename T>
__global__ __launch_bounds__(kMfmaWaves * 64, 2) void decode_stage1_mfma_listed_kernel(Stage1Params p) {
  __shared__ __attribute__((aligned(1024))) char lds[kMfmaWaves * kMfmaStage];
  __shared__ uint32_t first_unit[kListedMaxBatch + 1];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tw = p.tasks_on_x & 7, cw = kMfmaWaves / tw;
  const uint32_t task_groups = (uint32_t)((p.tasks + tw - 1) / tw);
  const int batch = (int)p.batch;  // <= kListedMaxBatch (checked on the host)
  if (wave == 0) {
    const int64_t rows_avail = (p.num_blocks + p.row_mul - 1) / p.row_mul;
    uint32_t carry = 0;
    for (int b0 = 0; b0 < batch; b0 += 64) {
      const int bb = b0 + lane;
      uint32_t units = 0;
      if (bb < batch) {
        const int len = p.b_seqlen[bb];
        int64_t nblk = len <= 0 ? 0 : ((int64_t)len + p.block_seq - 1) / p.block_seq;  // (the same clamps as in the unit)
        if (nblk > p.grid_blocks) nblk = p.grid_blocks;
        if (nblk > rows_avail) nblk = rows_avail;
        const int64_t per_group = (int64_t)p.blocks_per_wg * cw;
        units = (uint32_t)((nblk + per_group - 1) / per_group) * task_groups;
      }
      uint32_t incl = units;  // inclusive prefix sum over the 64 lanes
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      if (bb < batch) first_unit[bb] = carry + incl - units;
      carry += __builtin_amdgcn_readlane(incl, 63);
    }
    if (lane == 0) first_unit[batch] = carry;
  }
  __syncthreads();
  const uint32_t total = first_unit[batch];
  for (uint32_t unit = blockIdx.x; unit < total; unit += gridDim.x) {
    // the request that holds the unit: first_unit[lo] <= unit < first_unit[hi] throughout (requests without units are skipped)
    int lo = 0, hi = batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      const uint32_t f = __builtin_amdgcn_readfirstlane(first_unit[mid]);
      if (f <= unit) lo = mid;
      else hi = mid;
    }
    const uint32_t local = unit - __builtin_amdgcn_readfirstlane(first_unit[lo]);
    const uint32_t cgroup = local / task_groups;
    stage1_mfma_unit<T, false, true>(p, lds, lane, wave, lo, local - cgroup * task_groups, cgroup, 0);
  }
}

// The plain shape with the work dealt in equal shares (the fused call, whose partials are scratch).  All blocks of all
// requests, request after request, form one line; the workgroups of a task group cut it into as many contiguous shares
// as they have waves that walk tokens, and a wave computes its share of every request it touches into ONE partial (row
// = the share's first block of that request).  Every wave gets the same number of blocks to
// within one whatever the lengths are, a request long or short costs one partial per share it touches instead of one
// per block (the partials, written while the gather saturates the memory system, cost eight times their bytes), and no
// split size has to be guessed from the longest request.  Neighbouring workgroups hold the task groups of the same
// share (all KV heads of a token are fetched at about the same time).  The merge that follows (decode_stage2_kernel with
// SHARES) works out the same shares from the lengths and visits the rows that hold a partial, nothing else.
template <typename T>
__global__ __launch_bounds__(kMfmaWaves * 64, 2) void decode_stage1_mfma_range_kernel(Stage1Params p) {
  __shared__ __attribute__((aligned(1024))) char lds[kMfmaWaves * kMfmaStage];
  __shared__ uint32_t first_block[kListedMaxBatch + 1];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tw = p.tasks_on_x & 7, cw = kMfmaWaves / tw;
  const uint32_t task_groups = (uint32_t)((p.tasks + tw - 1) / tw);
  const int batch = (int)p.batch;  // <= kListedMaxBatch (checked on the host)
  if (wave == 0) {
    uint32_t carry = 0;
    for (int b0 = 0; b0 < batch; b0 += 64) {
      const int bb = b0 + lane;
      uint32_t blocks = 0;
      if (bb < batch) {
        const int len = p.b_seqlen[bb];
        int64_t nblk = len <= 0 ? 0 : ((int64_t)len + p.block_seq - 1) / p.block_seq;  // (the same clamps as in the unit)
        if (nblk > p.grid_blocks) nblk = p.grid_blocks;
        if (nblk > p.num_blocks) nblk = p.num_blocks;
        blocks = (uint32_t)nblk;
      }
      uint32_t incl = blocks;  // inclusive prefix sum over the 64 lanes
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      if (bb < batch) first_block[bb] = carry + incl - blocks;
      carry += __builtin_amdgcn_readlane(incl, 63);
    }
    if (lane == 0) first_block[batch] = carry;
  }
  __syncthreads();
  const uint64_t total = first_block[batch];
  // the wave's share: worker v of V, over the workgroups of its task group and their waves that walk tokens
  const uint32_t tg = blockIdx.x % task_groups;
  const uint64_t V = (uint64_t)(gridDim.x / task_groups) * cw;
  const uint64_t v = (uint64_t)(blockIdx.x / task_groups) * cw + (wave / tw);
  uint32_t x = (uint32_t)(v * total / V);
  const uint32_t hi_all = (uint32_t)((v + 1) * total / V);
  if (x >= hi_all) return;
  // the request that holds block x: first_block[lo] <= x < first_block[hi] throughout (requests without blocks are skipped)
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    const uint32_t f = __builtin_amdgcn_readfirstlane(first_block[mid]);
    if (f <= x) lo = mid;
    else hi = mid;
  }
  int r = lo;
  while (x < hi_all) {
    const uint32_t r0 = __builtin_amdgcn_readfirstlane(first_block[r]), r1 = __builtin_amdgcn_readfirstlane(first_block[r + 1]);
    if (r1 > x) {
      const uint32_t end = r1 < hi_all ? r1 : hi_all;
      stage1_mfma_unit<T, false, true, true>(p, lds, lane, wave, r, tg, 0, 0, (int64_t)(x - r0), (int64_t)(end - r0));
      x = end;
    }
    r++;
  }
}

// ------------------------------------------------------------------------------------
// Stage 2: one workgroup per (request, head), the heads of a request next to each other in the grid (a request much
// longer than the others then has all its workgroups start together, wherever it stands in the batch, instead of its
// last head at the very end of the launch); SL slices of D/4 lanes walk the block axis in parallel (the reference walks
// it serially, flash_decoding_stage2.cu:38-48), then merge through LDS.
// ------------------------------------------------------------------------------------
struct Stage2Params {
  void* o;
  float* out_lse;
  const int32_t* b_seqlen;
  const float* mid_o;
  const float* mid_lse;
  int64_t batch, heads, num_seq_blocks, block_seq;
  int64_t blk_rows, req_rows;  // rows of mid_o between consecutive blocks / requests
  int64_t grid_blocks;         // (SHARES) stage 1's bound on a request's blocks, from the longest request
  int64_t shares_workers;      // (SHARES) the shares stage 1 dealt the blocks of all requests in
  uint32_t workers_mul, workers_shr;  // (SHARES) n / shares_workers = umulhi(n, mul) >> shr for n < 2^31 (mul = 0: shares_workers = 1)
};

template <typename OT> __device__ __forceinline__ void store4(void* base, int64_t elem, const f32x4& v);
template <> __device__ __forceinline__ void store4<float>(void* base, int64_t elem, const f32x4& v) {
  *(f32x4*)((float*)base + elem) = v;
}
template <> __device__ __forceinline__ void store4<F16>(void* base, int64_t elem, const f32x4& v) {
  *(u32x2*)((uint16_t*)base + elem) = u32x2{pack2<F16>(v[0], v[1]), pack2<F16>(v[2], v[3])};
}
template <> __device__ __forceinline__ void store4<BF16>(void* base, int64_t elem, const f32x4& v) {
  *(u32x2*)((uint16_t*)base + elem) = u32x2{pack2<BF16>(v[0], v[1]), pack2<BF16>(v[2], v[3])};
}

// SHARES: behind decode_stage1_mfma_range_kernel, which dealt the blocks of all requests, request after request, in
// shares_workers equal shares and left one partial per share and request, at the row of the share's first block of the
// request.  The workgroup counts the blocks in front of its request and in all (the same clamps as stage 1), lists the
// shares that begin inside its request, and visits those rows (and row 0, where the share that reaches into the
// request from the one before it, or begins with it, left its partial).
template <typename OT, int D, int NT, bool SHARES = false>
__global__ __launch_bounds__(NT) void decode_stage2_kernel(Stage2Params p) {
  constexpr int LPR = D / 4;      // lanes per row (float4 each)
  constexpr int SL = NT / LPR;    // slices walking the block axis
  const int64_t b = blockIdx.x / (uint32_t)p.heads, h = blockIdx.x % (uint32_t)p.heads;
  const int slice = threadIdx.x / LPR, c = threadIdx.x % LPR;
  auto blocks_of = [&](int64_t len) -> int64_t {
    int64_t nb = len <= 0 ? 0 : (len + p.block_seq - 1) / p.block_seq;
    if (nb > p.num_seq_blocks) nb = p.num_seq_blocks;
    if (SHARES && nb > p.grid_blocks) nb = p.grid_blocks;
    return nb;
  };
  int64_t n = blocks_of(p.b_seqlen[b]);
  // SHARES: entry i of the rows to visit is row 0 for i = 0, else the first block of share v_lo + i - 1 (its distance from
  // the request's first block); an entry whose share is empty (more shares than blocks) holds nothing
  uint64_t first = 0, total = 1, v_lo = 0;
  const uint64_t V = SHARES ? (uint64_t)p.shares_workers : 1;
  uint64_t per_share = 0;  // total / V ...
  uint32_t rest = 0;       // ... and total % V: share v begins at block v * per_share + v * rest / V (v * rest < V * V: 32 bits)
  auto share_begin = [&](uint64_t v) -> uint64_t {
    const uint32_t t = (uint32_t)v * rest;
    return v * per_share + (p.workers_mul ? __umulhi(t, p.workers_mul) >> p.workers_shr : t);
  };
  if (SHARES) {
    uint32_t pre = 0, tot = 0;
    for (int64_t i = threadIdx.x; i < p.batch; i += NT) {
      const uint32_t nb = (uint32_t)blocks_of(p.b_seqlen[i]);
      tot += nb;
      if (i < b) pre += nb;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
      pre += __shfl_xor(pre, d, 64);
      tot += __shfl_xor(tot, d, 64);
    }
    __shared__ uint32_t red[2][NT / 64];
    if ((threadIdx.x & 63) == 0) {
      red[0][threadIdx.x >> 6] = pre;
      red[1][threadIdx.x >> 6] = tot;
    }
    __syncthreads();
    pre = tot = 0;
#pragma unroll
    for (int w = 0; w < NT / 64; w++) {
      pre += red[0][w];
      tot += red[1][w];
    }
    first = pre;
    total = tot > 0 ? tot : 1;
    per_share = total / V;
    rest = (uint32_t)(total - per_share * V);
    if (n > 0) {
      v_lo = ((first + 1) * V + total - 1) / total;                        // the first share that begins behind block 0 of the request
      const uint64_t v_end = ((first + (uint64_t)n) * V + total - 1) / total;  // one past the last share that begins inside it
      n = 1 + (int64_t)(v_end > v_lo ? v_end - v_lo : 0);
    }
  }
  const int64_t row_stride = p.blk_rows;
  const int64_t row0 = b * p.req_rows + h;
  const int64_t out_row = b * p.heads + h;

  float M = -INFINITY, L = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  auto fold = [&](float lse, const f32x4& tv) {
    if (lse == -INFINITY) return;  // an empty partial contributes nothing
    const float Mn = fmaxf(M, lse);
    const float so = exp2_diff(M * kLog2e, Mn * kLog2e);
    const float sn = __builtin_amdgcn_exp2f((lse - Mn) * kLog2e);
    acc = acc * so + tv * sn;
    L = L * so + sn;
    M = Mn;
  };
  // U rows and their log-sum-exps requested together, none waiting for another: with many requests in the batch the
  // partials of one request lie batch x heads rows apart (a megabyte and more) and every load pays the full latency; a
  // long request's merge is a chain of them.  Positions past the request's last block repeat that block and are
  // dropped; an empty partial's row is loaded like any other (it may hold anything: stage 1 leaves the rows it merged
  // into another one untouched) and dropped by its log-sum-exp.
  constexpr int U = 8;  // rows a slice has in flight (sixteen measured slower: the many short requests of a batch then ask for rows they drop)
  for (int64_t i = slice; i < n; i += U * SL) {
    float lse[U];
    f32x4 tv[U];
    bool holds[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t e = i + u * SL < n ? i + u * SL : n - 1;
      int64_t blk = e;
      holds[u] = i + u * SL < n;
      if (SHARES && e > 0) {
        const uint64_t v = v_lo + (uint64_t)e - 1;
        const uint64_t x = share_begin(v);
        blk = (int64_t)(x - first);
        holds[u] = holds[u] && share_begin(v + 1) > x;  // (an empty share left nothing)
      }
      const int64_t row = blk * row_stride + row0;
      lse[u] = p.mid_lse[row];
      tv[u] = *(const f32x4*)(p.mid_o + row * D + c * 4);
    }
#pragma unroll
    for (int u = 0; u < U; u++)
      if (holds[u]) fold(lse[u], tv[u]);
  }
  __shared__ float sM[SL], sL[SL];
  __shared__ f32x4 sAcc[SL][LPR];
  if (c == 0) {
    sM[slice] = M;
    sL[slice] = L;
  }
  sAcc[slice][c] = acc;
  __syncthreads();
  if (slice == 0) {
    float Mt = -INFINITY;
#pragma unroll
    for (int s = 0; s < SL; s++) Mt = fmaxf(Mt, sM[s]);
    float Lt = 0.f;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SL; s++) {
      const float w = exp2_diff(sM[s] * kLog2e, Mt * kLog2e);
      Lt += sL[s] * w;
      a += sAcc[s][c] * w;
    }
    const float inv = Lt > 0.f ? 1.f / Lt : 0.f;
    store4<OT>(p.o, out_row * D + c * 4, a * inv);
    if (c == 0) p.out_lse[out_row] = Lt > 0.f ? Mt + __builtin_amdgcn_logf(Lt) * kLn2 : -INFINITY;
  }
}

template <typename T, int GT, int HR>
static int launch_stage1(const lsattn_decode_stage1_args* a, hipStream_t st) {
  constexpr int NW = 4;  // waves (tasks) per workgroup; 8 measured no faster
  Stage1Params p;
  p.mid_o = a->mid_o;
  p.mid_lse = a->mid_o_logexpsum;
  p.q = a->q;
  p.k = a->k;
  p.v = a->v;
  p.k_s0 = a->k_stride_0;
  p.k_s1 = a->k_stride_1;
  p.v_s0 = a->v_stride_0;
  p.v_s1 = a->v_stride_1;
  p.scale_log2 = a->sm_scale * kLog2e;
  p.req_to_tokens = a->req_to_tokens;
  p.b_req_idx = a->b_req_idx;
  p.b_seqlen = a->b_seqlen;
  p.batch = a->batch;
  p.hq = a->num_q_heads;
  p.hkv = a->num_kv_heads;
  p.num_blocks = a->num_blocks;
  p.blk_rows = a->partials_by_request ? a->num_q_heads : a->batch * a->num_q_heads;
  p.req_rows = a->partials_by_request ? a->num_blocks * a->num_q_heads : a->num_q_heads;
  p.max_seq_len = a->max_seq_len;
  p.row_mul = a->merge_blocks > 1 ? a->merge_blocks : 1;
  p.fine_block_seq = a->seq_block_size;
  p.block_seq = a->seq_block_size * p.row_mul;
  p.grid_blocks = (a->max_len_in_batch + p.block_seq - 1) / p.block_seq;  // stage1.cu:211, in partials computed
  const int group = (int)(a->num_q_heads / a->num_kv_heads);
  p.tasks = (int)a->num_kv_heads * ((group + GT * HR - 1) / (GT * HR));
  const int wgs_y = (p.tasks + NW - 1) / NW;
  // a workgroup walks consecutive blocks until it has covered at least 256 tokens (smaller units measured slower for
  // short blocks, larger ones lose to tail imbalance)
  constexpr int64_t kTokensPerWorkgroup = 256;
  int64_t per_wg = (kTokensPerWorkgroup + p.block_seq - 1) / p.block_seq;
  if (per_wg < 1) per_wg = 1;
  const int64_t rows_avail = (a->num_blocks + p.row_mul - 1) / p.row_mul;
  int64_t nblk = p.grid_blocks < rows_avail ? p.grid_blocks : rows_avail;
  if (nblk < 1) return LSATTN_OK;
  p.blocks_per_wg = (int32_t)per_wg;
  const int64_t chunks = (nblk + per_wg - 1) / per_wg;
  if (chunks > 0x7fffffff || a->batch > 65535 || wgs_y > 65535) return LSATTN_ERR_INVALID_ARG;
  // A launch of less than one workgroup per CU leaves most of the chip's load slots empty: the waves of a workgroup then
  // share one task and split each block's tokens (measured: 64 workgroups, one request of 8192 tokens with 8 KV heads,
  // 19.9 -> 10.0 us; from 256 workgroups on it gains nothing; blocks shorter than 32 tokens per wave cannot use it).
  const bool once = group <= GT * HR;
  // ... and so does a launch with fewer tasks than a workgroup has waves (one or two KV heads: the other waves would idle)
  const bool split = (chunks * wgs_y * a->batch < 256 || p.tasks < NW) && p.block_seq >= 32 * NW && p.tasks <= 65535;
  if (split) {
    p.tasks_on_x = chunks <= 65535;
    dim3 grid = p.tasks_on_x ? dim3((unsigned)p.tasks, (unsigned)chunks, (unsigned)a->batch)
                             : dim3((unsigned)chunks, (unsigned)p.tasks, (unsigned)a->batch);
    if (once) LSATTN_LAUNCH_KERNEL((decode_stage1_kernel<T, GT, NW, true, true, HR>), grid, dim3(NW * 64), 0, st, p);
    else LSATTN_LAUNCH_KERNEL((decode_stage1_kernel<T, GT, NW, true, false, HR>), grid, dim3(NW * 64), 0, st, p);
    return check_launch();
  }
  p.tasks_on_x = wgs_y <= 2 && chunks <= 65535;  // with more task groups per chunk (MHA, 32 KV heads) it measured 2 % slower
  dim3 grid = p.tasks_on_x ? dim3((unsigned)wgs_y, (unsigned)chunks, (unsigned)a->batch)
                           : dim3((unsigned)chunks, (unsigned)wgs_y, (unsigned)a->batch);
  if (once) LSATTN_LAUNCH_KERNEL((decode_stage1_kernel<T, GT, NW, false, true, HR>), grid, dim3(NW * 64), 0, st, p);
  else LSATTN_LAUNCH_KERNEL((decode_stage1_kernel<T, GT, NW, false, false, HR>), grid, dim3(NW * 64), 0, st, p);
  return check_launch();
}

// Large launches: the matrix-pipe kernel, when its conditions hold (blocks a multiple of 32 tokens, enough waves to fill
// the chip); lsattn_set_tuning forces the choice where the conditions allow it (tuning, tests).
// `shares`: deal the blocks in equal shares (decode_stage1_mfma_range_kernel) or launch nothing (*taken stays false).
template <typename T> static int launch_stage1_mfma(const lsattn_decode_stage1_args* a, hipStream_t st, bool* taken, int64_t* shares = nullptr) {
  *taken = false;
  const int group = (int)(a->num_q_heads / a->num_kv_heads);
  Stage1Params p;
  p.mid_o = a->mid_o;
  p.mid_lse = a->mid_o_logexpsum;
  p.q = a->q;
  p.k = a->k;
  p.v = a->v;
  p.k_s0 = a->k_stride_0;
  p.k_s1 = a->k_stride_1;
  p.v_s0 = a->v_stride_0;
  p.v_s1 = a->v_stride_1;
  p.scale_log2 = a->sm_scale * kLog2e;
  p.req_to_tokens = a->req_to_tokens;
  p.b_req_idx = a->b_req_idx;
  p.b_seqlen = a->b_seqlen;
  p.batch = a->batch;
  p.hq = a->num_q_heads;
  p.hkv = a->num_kv_heads;
  p.num_blocks = a->num_blocks;
  p.blk_rows = a->partials_by_request ? a->num_q_heads : a->batch * a->num_q_heads;
  p.req_rows = a->partials_by_request ? a->num_blocks * a->num_q_heads : a->num_q_heads;
  p.max_seq_len = a->max_seq_len;
  p.row_mul = a->merge_blocks > 1 ? a->merge_blocks : 1;
  p.fine_block_seq = a->seq_block_size;
  p.block_seq = a->seq_block_size * p.row_mul;
  p.grid_blocks = (a->max_len_in_batch + p.block_seq - 1) / p.block_seq;
  if (p.block_seq % kMfmaBatch || a->k_stride_0 >= (1 << 30) || a->v_stride_0 >= (1 << 30)) return LSATTN_OK;
  p.tasks = (int)a->num_kv_heads * ((group + 15) / 16);
  int64_t per_wave = (256 + p.block_seq - 1) / p.block_seq;  // a wave walks at least 256 tokens
  if (per_wave < 1) per_wave = 1;
  const int64_t rows_avail = (a->num_blocks + p.row_mul - 1) / p.row_mul;
  const int64_t nblk = p.grid_blocks < rows_avail ? p.grid_blocks : rows_avail;
  if (nblk < 1) return LSATTN_OK;
  p.blocks_per_wg = (int32_t)per_wave;
  const int64_t chunks = (nblk + per_wave - 1) / per_wave;
  const int tw = p.tasks >= 4 ? 4 : p.tasks >= 2 ? 2 : 1, cw = kMfmaWaves / tw;
  const int64_t wgs_x = (chunks + cw - 1) / cw, wgs_y = (p.tasks + tw - 1) / tw;
  if (wgs_x > 0x7fffffff || a->batch > 65535 || wgs_y > 65535) return LSATTN_OK;
  // Which shape, by the launch's size in waves of the plain shape (256 tokens x task x request; measured):
  //   groups of four and more query heads per KV head: up to 512 waves (3072 on fewer than four KV heads, where the plain
  //     shape has no neighbouring heads to put side by side) the shape whose four waves split a block (a launch of 8 to 512
  //     plain waves runs 30-45 % shorter with it than with either other kernel), above that the plain shape;
  //   smaller groups (most of an MFMA's sixteen columns idle): the plain shape from 768 waves, below that the lane kernel.
  const int64_t waves = chunks * p.tasks * a->batch;
  const bool can_split = p.block_seq % (kMfmaWaves * kMfmaBatch) == 0 && nblk <= 0x7fffffff;
  bool split_waves = group >= 4 && can_split && waves <= (p.tasks < 4 ? 3072 : 512);
  bool use = !split_waves && waves >= (group >= 4 ? 513 : 768);
  const Tuning tn = tuning();  // (lsattn_set_tuning: tuning and tests)
  if (tn.decode_stage1 == LSATTN_DECODE_STAGE1_LANE) use = split_waves = false;
  if (tn.decode_stage1 == LSATTN_DECODE_STAGE1_MFMA) use = true, split_waves = false;
  if (tn.decode_stage1 == LSATTN_DECODE_STAGE1_SPLIT && can_split) use = false, split_waves = true;
  if (shares) {
    // only where the plain shape would run, on launches with at least kSharesMinBlocks blocks of 256 tokens and more per
    // worker to deal (fewer: the grids above, whose workgroups the hardware hands out as they finish)
    const int tws = p.tasks >= 4 ? 4 : p.tasks >= 2 ? 2 : 1;
    const int64_t task_groups = (p.tasks + tws - 1) / tws;
    int64_t per_group = 2 * kCUs / task_groups;  // workgroups per task group: two workgroups per CU in all
    const bool forced = tn.decode_listed == LSATTN_DECODE_LISTED_SHARES;  // (tests: whatever the launch's size)
    if (tn.decode_listed == LSATTN_DECODE_LISTED_OFF || tn.decode_listed == LSATTN_DECODE_LISTED_ON) return LSATTN_OK;
    if (per_group < 1 || p.row_mul != 1 || a->batch > kListedMaxBatch || nblk * a->batch > 0x7fffffff) return LSATTN_OK;
    const int64_t workers = per_group * (kMfmaWaves / tws);
    if (!forced && (!use || split_waves || a->seq_block_size < 256 || a->batch < kSharesMinBatch || nblk * a->batch < kSharesMinBlocks * workers)) return LSATTN_OK;
    *taken = true;
    *shares = workers;
    p.tasks_on_x = tws;
    p.blocks_per_wg = 1;
    LSATTN_LAUNCH_KERNEL((decode_stage1_mfma_range_kernel<T>), dim3((unsigned)(per_group * task_groups)), dim3(kMfmaWaves * 64), 0, st, p);
    return check_launch();
  }
  if (split_waves) {
    *taken = true;
    p.blocks_per_wg = 1;
    p.tasks_on_x = 1;
    LSATTN_LAUNCH_KERNEL((decode_stage1_mfma_kernel<T, true>), dim3((unsigned)nblk, (unsigned)p.tasks, (unsigned)a->batch), dim3(kMfmaWaves * 64),
                       0, st, p);
    return check_launch();
  }
  if (!use) return LSATTN_OK;
  *taken = true;
  // The task groups of a chunk are dispatched one after the other (x runs fastest), so that all KV heads of a token are
  // fetched at about the same time: config 3's shape 6.03 -> 6.17 TB/s, 32 KV heads 6.0 -> 6.5.
  const bool tasks_first = wgs_y > 1 && wgs_x <= 65535;
  p.tasks_on_x = tw | (tasks_first ? 8 : 0);  // (this kernel: waves of a workgroup on neighbouring tasks; the grid's order)
  // Launches of very many workgroups walk a list of the units that exist instead (see the kernel): most of such a grid
  // is empty whenever the batch mixes long and short requests, which the host cannot see.
  // lsattn_set_tuning overrides the choice (tuning and tests).
  const int64_t wgs_total = wgs_x * wgs_y * a->batch;
  bool listed = wgs_total >= kListedFromWorkgroups || (a->seq_block_size >= kListedCoarseTokens && wgs_total >= kListedFromWorkgroupsCoarse);
  if (tn.decode_listed == LSATTN_DECODE_LISTED_OFF) listed = false;
  if (tn.decode_listed == LSATTN_DECODE_LISTED_ON) listed = true;
  if (listed && a->batch <= kListedMaxBatch && wgs_total <= 0x7fffffff) {
    const int64_t resident = 2 * kCUs;  // two workgroups of this kernel per CU
    LSATTN_LAUNCH_KERNEL((decode_stage1_mfma_listed_kernel<T>), dim3((unsigned)(wgs_total < resident ? wgs_total : resident)),
                       dim3(kMfmaWaves * 64), 0, st, p);
    return check_launch();
  }
  const dim3 grid = tasks_first ? dim3((unsigned)wgs_y, (unsigned)wgs_x, (unsigned)a->batch) : dim3((unsigned)wgs_x, (unsigned)wgs_y, (unsigned)a->batch);
  LSATTN_LAUNCH_KERNEL((decode_stage1_mfma_kernel<T, false>), grid, dim3(kMfmaWaves * 64), 0, st, p);
  return check_launch();
}

template <typename T> static int dispatch_stage1(const lsattn_decode_stage1_args* a, hipStream_t st, int64_t* shares = nullptr) {
  const int group = (int)(a->num_q_heads / a->num_kv_heads);
  if (shares) {  // (in equal shares or not at all: *shares is their number, or stays 0)
    bool taken;
    return launch_stage1_mfma<T>(a, st, &taken, shares);
  }
  {
    bool taken;
    const int rc = launch_stage1_mfma<T>(a, st, &taken);
    if (taken) return rc;
  }
  // groups of 3 and 4 take four query heads per task (3: one spare): fetching a K/V row once per group matters more than
  // the spare accumulators cost
  // groups of more than four: eight query heads per task in two rounds of four over the same rows
  if (group >= 5) return launch_stage1<T, 4, 2>(a, st);
  if (group >= 3) return launch_stage1<T, 4, 1>(a, st);
  if (group == 2) return launch_stage1<T, 2, 1>(a, st);
  return launch_stage1<T, 1, 1>(a, st);
}

}  // namespace lsattn

using namespace lsattn;

// `shares` (the fused call): launch stage 1 in equal shares if the launch is one for them (*shares: how many) or nothing.
static int decode_stage1(const lsattn_decode_stage1_args* a, void* stream, int64_t* shares) {
  if (shares) *shares = 0;
  if (!a || !a->mid_o || !a->mid_o_logexpsum || !a->q || !a->k || !a->v || !a->req_to_tokens || !a->b_req_idx ||
      !a->b_seqlen)
    return LSATTN_ERR_INVALID_ARG;
  if (a->merge_blocks < 0 || a->merge_blocks > 16 || a->seq_block_size * (a->merge_blocks > 1 ? a->merge_blocks : 1) > 0x40000000)
    return LSATTN_ERR_INVALID_ARG;
  if (a->batch < 0 || a->num_q_heads <= 0 || a->num_kv_heads <= 0 || a->num_blocks < 0 || a->seq_block_size < 1 ||
      a->max_len_in_batch < 0 || a->max_seq_len < 0 || a->max_seq_len > 0x7fffff00)  // 32-bit token positions in the kernel
    return LSATTN_ERR_INVALID_ARG;
  if (a->num_q_heads % a->num_kv_heads != 0) return LSATTN_ERR_INVALID_ARG;
  // 16-byte row loads: strides must keep every row 16-byte aligned
  if (a->k_stride_0 % 8 || a->k_stride_1 % 8 || a->v_stride_0 % 8 || a->v_stride_1 % 8) return LSATTN_ERR_INVALID_ARG;
  if (((uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->q | (uintptr_t)a->mid_o) & 15) return LSATTN_ERR_INVALID_ARG;
  if (a->head_dim != 128) return LSATTN_ERR_UNSUPPORTED;  // as flash_decoding_stage1.cu:210
  if (a->batch == 0 || a->num_blocks == 0 || a->max_len_in_batch == 0) return LSATTN_OK;
  hipStream_t st = (hipStream_t)stream;
  if (a->dtype == LSATTN_F16) return dispatch_stage1<F16>(a, st, shares);
  if (a->dtype == LSATTN_BF16) return dispatch_stage1<BF16>(a, st, shares);
  return LSATTN_ERR_UNSUPPORTED;
}

extern "C" int lsattn_decode_stage1(const lsattn_decode_stage1_args* a, void* stream) { return decode_stage1(a, stream, nullptr); }

// `live_blocks`: an upper bound of the partial rows any request has (the rows of the buffer, or fewer when the caller
// knows the longest request); it picks the shape of the merge, which decides the order of its additions.
template <typename OT> static int dispatch_stage2(const Stage2Params& p, int64_t D, dim3 grid, int64_t live_blocks, hipStream_t st) {
  if (p.shares_workers > 0) {
    if (D != 128) return LSATTN_ERR_UNSUPPORTED;
    // (a request's partials: at most one per share and one more, and no more than it has blocks)
    const int64_t most = live_blocks < p.shares_workers + 1 ? live_blocks : p.shares_workers + 1;
    if (most >= 64 && (int64_t)grid.x < 2048) LSATTN_LAUNCH_KERNEL((decode_stage2_kernel<OT, 128, 1024, true>), grid, dim3(1024), 0, st, p);
    else LSATTN_LAUNCH_KERNEL((decode_stage2_kernel<OT, 128, 256, true>), grid, dim3(256), 0, st, p);
    return check_launch();
  }
  // few (batch, head) pairs with many partials each (long contexts at small batch): 1024 threads walk the block axis in 32
  // slices instead of 8, or the merge takes a fifth of the time of the gather it follows
  const bool wide = D == 128 && live_blocks >= 64 && ((int64_t)grid.x < 2048 || (live_blocks >= 1024 && (int64_t)grid.x < 8192));
  switch (D) {
    case 32: LSATTN_LAUNCH_KERNEL((decode_stage2_kernel<OT, 32, 256>), grid, dim3(256), 0, st, p); break;
    case 64: LSATTN_LAUNCH_KERNEL((decode_stage2_kernel<OT, 64, 256>), grid, dim3(256), 0, st, p); break;
    case 128:
      if (wide) LSATTN_LAUNCH_KERNEL((decode_stage2_kernel<OT, 128, 1024>), grid, dim3(1024), 0, st, p);
      else LSATTN_LAUNCH_KERNEL((decode_stage2_kernel<OT, 128, 256>), grid, dim3(256), 0, st, p);
      break;
    default: return LSATTN_ERR_UNSUPPORTED;
  }
  return check_launch();
}

static int decode_stage2(const lsattn_decode_stage2_args* a, int64_t live_blocks, void* stream, int64_t shares_workers = 0, int64_t grid_blocks = 0) {
  if (!a || !a->o || !a->out_logexpsum || !a->b_seqlen || !a->mid_o || !a->mid_o_logexpsum) return LSATTN_ERR_INVALID_ARG;
  if (a->batch < 0 || a->num_heads <= 0 || a->num_seq_blocks < 0 || a->block_seq < 1) return LSATTN_ERR_INVALID_ARG;
  if (((uintptr_t)a->o | (uintptr_t)a->mid_o) & 15) return LSATTN_ERR_INVALID_ARG;
  if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 128) return LSATTN_ERR_UNSUPPORTED;
  if (a->batch == 0) return LSATTN_OK;
  if (a->batch * a->num_heads > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  Stage2Params p{a->o, a->out_logexpsum, a->b_seqlen, a->mid_o, a->mid_o_logexpsum,
                 a->batch, a->num_heads, a->num_seq_blocks, a->block_seq,
                 a->partials_by_request ? a->num_heads : a->batch * a->num_heads,
                 a->partials_by_request ? a->num_seq_blocks * a->num_heads : a->num_heads, grid_blocks, shares_workers, 0, 0};
  if (shares_workers > 1) {  // (shares_workers <= 2048: v * rest stays far below 2^31)
    uint32_t L = 0;
    while ((1u << L) < (uint32_t)shares_workers) L++;
    p.workers_mul = (uint32_t)((((uint64_t)1 << (31 + L)) + shares_workers - 1) / shares_workers);
    p.workers_shr = L - 1;
  }
  dim3 grid((unsigned)(a->batch * a->num_heads));
  hipStream_t st = (hipStream_t)stream;
  switch (a->o_dtype) {
    case LSATTN_F32: return dispatch_stage2<float>(p, a->head_dim, grid, live_blocks, st);
    case LSATTN_F16: return dispatch_stage2<F16>(p, a->head_dim, grid, live_blocks, st);
    case LSATTN_BF16: return dispatch_stage2<BF16>(p, a->head_dim, grid, live_blocks, st);
    default: return LSATTN_ERR_UNSUPPORTED;
  }
}

extern "C" int lsattn_decode_stage2(const lsattn_decode_stage2_args* a, void* stream) {
  return decode_stage2(a, a ? a->num_seq_blocks : 0, stream);
}

extern "C" int lsattn_decode_attention(const lsattn_decode_stage1_args* s1, const lsattn_decode_stage2_args* s2, void* stream) {
  if (!s1 || !s2) return LSATTN_ERR_INVALID_ARG;
  // the two stages must describe the same partials
  if (s1->mid_o != s2->mid_o || s1->mid_o_logexpsum != s2->mid_o_logexpsum || s1->b_seqlen != s2->b_seqlen ||
      s1->batch != s2->batch || s1->num_q_heads != s2->num_heads || s1->num_blocks != s2->num_seq_blocks ||
      s1->head_dim != s2->head_dim || s1->seq_block_size != s2->block_seq || !s1->partials_by_request != !s2->partials_by_request)
    return LSATTN_ERR_INVALID_ARG;
  // Large launches deal the tokens in equal shares (decode_stage1_mfma_range_kernel), however coarse the split asked
  // for: the partials are scratch here, and a share leaves one partial per request it touches whatever the block size.
  // The blocks the shares are counted in: 256 tokens, or the smallest multiple by a power of two whose rows the buffers hold
  // (a share's partial goes to the row of its first block).
  if (s1->merge_blocks <= 1 && s1->seq_block_size >= 256 && s1->max_len_in_batch > 0 && s1->num_blocks > 0) {
    int64_t g = 256;
    while ((s1->max_len_in_batch + g - 1) / g > s1->num_blocks) g *= 2;
    lsattn_decode_stage1_args a1 = *s1;
    a1.seq_block_size = g;
    int64_t shares = 0;
    const int rc1 = decode_stage1(&a1, stream, &shares);
    if (rc1 != LSATTN_OK) return rc1;
    if (shares > 0) {
      lsattn_decode_stage2_args a2 = *s2;
      a2.block_seq = g;
      const int64_t rows = (s1->max_len_in_batch + g - 1) / g;
      return decode_stage2(&a2, rows, stream, shares, rows);
    }
  }
  const int rc = lsattn_decode_stage1(s1, stream);
  if (rc != LSATTN_OK) return rc;
  // the merge's shape from the rows the longest request can reach, not from the rows the buffer happens to have: the
  // same call gives the same bits whatever the buffer's height (lsattn_decode_attention_static passes its own)
  int64_t live = s1->seq_block_size > 0 ? (s1->max_len_in_batch + s1->seq_block_size - 1) / s1->seq_block_size : 0;
  if (live > s2->num_seq_blocks) live = s2->num_seq_blocks;
  return decode_stage2(s2, live, stream);
}

// ------------------------------------------------------------------------------------
// lsattn_decode_attention with the split-K partials in a file-scope device array instead of caller memory, for callers
// that cannot allocate.  Every device the library runs on holds its own copy of the array at its own address; the name
// below is only the host-side handle of it, so host code uses the address hipGetSymbolAddress returns for the current
// device (looked up once per device) and nothing else.
// ------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[LSATTN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];  // zero-initialised: not looked up yet

// device address of `scratch` on the current device, or nullptr
void* scratch_on_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  // two threads that race here look the same address up twice; either store is right
  if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return nullptr;
  }
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  return ptr;
}
}  // namespace

extern "C" int lsattn_decode_attention_static(const lsattn_decode_stage1_args* s1, const lsattn_decode_stage2_args* s2,
                                              void* stream) {
  if (!s1 || !s2) return LSATTN_ERR_INVALID_ARG;
  // the partials are the library's here: the caller names none
  if (s1->mid_o || s1->mid_o_logexpsum || s2->mid_o || s2->mid_o_logexpsum) return LSATTN_ERR_INVALID_ARG;
  if (s1->b_seqlen != s2->b_seqlen || s1->batch != s2->batch || s1->num_q_heads != s2->num_heads ||
      s1->num_blocks != s2->num_seq_blocks || s1->head_dim != s2->head_dim || s1->seq_block_size != s2->block_seq)
    return LSATTN_ERR_INVALID_ARG;
  if (s1->batch < 0 || s1->num_q_heads <= 0 || s1->num_blocks < 0 || s1->seq_block_size < 1 || s1->max_len_in_batch < 0 ||
      s1->merge_blocks > 1)
    return LSATTN_ERR_INVALID_ARG;
  if (s1->head_dim != 128) return LSATTN_ERR_UNSUPPORTED;
  // Rows of partials this call can touch: stage 1 writes block i of a request only for i below both bounds, and stage 2
  // is told the same count, so it reads no row that this call has not written (the array keeps the last call's bytes).
  int64_t rows = (s1->max_len_in_batch + s1->seq_block_size - 1) / s1->seq_block_size;
  if (rows > s1->num_blocks) rows = s1->num_blocks;
  const int64_t per_row = s1->batch * s1->num_q_heads;  // (request, head) pairs per block row
  if (per_row > 0 && rows > (int64_t)LSATTN_STATIC_SCRATCH_BYTES / 4 / 129 / per_row) return LSATTN_ERR_WORKSPACE;
  if ((uint64_t)(rows * per_row * 129) * 4 > (uint64_t)LSATTN_STATIC_SCRATCH_BYTES) return LSATTN_ERR_WORKSPACE;
  // The array is laid out for as many rows as it holds for this batch, up to one per 256 tokens of the longest request:
  // the fused call below counts its equal shares in the smallest blocks whose rows it is given.
  int64_t rows_laid = (s1->max_len_in_batch + 255) / 256;
  if (per_row > 0 && rows_laid > (int64_t)LSATTN_STATIC_SCRATCH_BYTES / 4 / 129 / per_row) rows_laid = (int64_t)LSATTN_STATIC_SCRATCH_BYTES / 4 / 129 / per_row;
  if (rows_laid < rows) rows_laid = rows;
  rows = rows_laid;
  const int64_t o_floats = rows * per_row * 128;         // a multiple of 128 floats: the LSE part stays 16-byte aligned
  float* base = (float*)scratch_on_current_device();
  if (!base) return LSATTN_ERR_LAUNCH;
  lsattn_decode_stage1_args a1 = *s1;
  lsattn_decode_stage2_args a2 = *s2;
  a1.mid_o = base;
  a1.mid_o_logexpsum = base + o_floats;
  a1.num_blocks = rows;
  a1.partials_by_request = a2.partials_by_request = 1;  // (the layout is nobody's but the library's here)
  a2.mid_o = a1.mid_o;
  a2.mid_o_logexpsum = a1.mid_o_logexpsum;
  a2.num_seq_blocks = rows;
  return lsattn_decode_attention(&a1, &a2, stream);
}
