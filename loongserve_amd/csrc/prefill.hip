// Ring / context-parallel prefill attention step for gfx950 (MFMA, wave64).
//
// Replaces the Triton _fwd_kernel + context_attention_fwd
// (loongserve/models/llama/triton_kernel/ring_context_flashattention_nopad.py:13-284).
//
// Shape of the computation (head_dim 128):
//   * a workgroup of 8 waves owns 256 query rows of one sequence: consecutive local rows of one query head, or, with
//     grouped-query attention, as many rows of each of the (up to eight) query heads of a KV head; each wave owns 32 of
//     them and keeps their Q as MFMA B operands in registers; waves w and w + 4 share a SIMD.  Two smaller shapes of
//     128 rows serve small launches: SPLIT (eight waves, two per 32 rows, each taking every other 32-key step) when
//     256-row workgroups would not fill the chip, HALF (four waves, rings of two tiles, two workgroups per CU) for
//     short chunks, whose workgroups spend as long starting and ending as working;
//   * K/V tiles of 64 keys are staged through LDS (rings of four tiles, filled by global->LDS DMA,
//     XOR-swizzled 16-byte chunks so that both the row-wise K reads and the transposing V reads
//     use all 64 banks);
//   * scores are computed transposed, S^T = K Q^T with v_mfma_f32_16x16x32 (under this kernel's load the
//     chip is power-limited, and this shape sustains a clearly higher clock than 32x32x16 at the same
//     operand traffic), so every lane owns one query column of each of the wave's two 16-row blocks:
//     row max / row sum are in-lane reductions plus an exchange between the four lanes of a column,
//     and the fp32 S^T accumulators convert in place into the B operand of O^T += V^T P^T without
//     any cross-lane movement (P and V always as fp16);
//   * V^T operands come from LDS through ds_read_b64_tr_b16 (the tile is stored row-major);
//   * on this hardware an MFMA holds its own wave until it is done, and vector work of the
//     SIMD's other wave runs beside it only under conditions (no short dependent chains, no
//     dot-product instructions) and, beside MFMAs of this shape, about a third slower.  The fully visible part of the key range
//     therefore runs as alternating phases: one wave of the SIMD issues the thirty-four MFMAs of a
//     32-key step (scores, P V, and the row sums of P as a product with a matrix of ones) while the
//     other does the exponentials of its own step, a workgroup barrier ends each phase;
//   * tiles that straddle the diagonal or the end of the KV chunk run the same pipeline with a masked softmax phase
//     (scores past a row's limit become -inf, loads clamp to the chunk's last row); tiles no row of the workgroup sees
//     are not walked;
//   * workgroup ids are mapped so that the workgroups sharing one KV head run on one XCD (ids are dealt
//     round-robin to the 8 XCDs; with fewer KV heads than XCDs a head's work is dealt to several of them)
//     and heavy (late) query tiles start first.
//   * one kernel, three epilogues (MODE): 0 writes the step's fp32 partial (O, LSE) from the empty state, 1 folds the
//     step into the reference's in-place (o, m, l) state (ring_context_flashattention_nopad.py:171-188), 2 LSE-merges it
//     into a running fp32 (O, LSE); the folding ones read the old state of both row blocks of a wave at once.
#include <type_traits>

#include "common.hip.h"

namespace lsattn {

// Division of 0 <= n < 2^31 by a launch constant d >= 1 without the divide sequence (some thirty instructions each, and
// the prologue of a workgroup needs ten): n / d = umulhi(n, mul) >> shr with mul = ceil(2^(31 + L) / d), shr = L - 1,
// L = ceil(log2 d); d = 1 is mul = 0.
struct FastDiv {
  uint32_t mul, shr;
};
static FastDiv fast_div(uint32_t d) {
  if (d <= 1) return FastDiv{0, 0};
  uint32_t L = 0;
  while ((1u << L) < d) L++;
  return FastDiv{(uint32_t)((((uint64_t)1 << (31 + L)) + d - 1) / d), L - 1};
}
__device__ __forceinline__ uint32_t div_by(uint32_t n, const FastDiv& f) { return f.mul ? __umulhi(n, f.mul) >> f.shr : n; }

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
  const int32_t* o_start;  // first output row per sequence (null: q_start)
  int32_t batch, hq, hkv, peers, nz, kv_slots, slices, units_per_slice, group;
  int32_t tile_major;  // order of the workgroups in the grid: heaviest query tiles of all KV heads first
  int32_t n_first, n_second;  // the fastest and the second index of the grid: (kv_slots, units_per_slice) if tile_major, else swapped
  int32_t pack_shift, heads_per_kv;  // 1 << pack_shift query heads of a KV head side by side in a workgroup; query heads per KV head
  int32_t fold_from, fold_sum;       // (ids >> 3) from fold_from on run backwards: j -> fold_sum - j (0: the whole grid runs forwards)
  int32_t listed, rows_shift;        // the grid numbers the (request, query tile, head group) units that exist (see the kernel); log2 of a workgroup's query positions
  int32_t store_through;             // epilogue 0 writes O through to memory as the stores are issued (launches of at most two rounds; the fp16 o of epilogue 1 gains nothing from it)
  int32_t kv_cuts, kv_cut_len;       // every sequence entered kv_cuts times, entry c taking keys [c, c + 1) * kv_cut_len of its chunk
  int64_t o_cut_rows;                // and writing its rows o_cut_rows * c further down
  FastDiv d_peers, d_first, d_second, d_slices, d_group, d_cuts;
  float scale_log2;
  void* o;
  int64_t o_st, o_sh;
  float* lse;
  float* m;
  float* l;
  int64_t ml_st, ml_sh;
};

constexpr int BM = 256;   // query rows per workgroup (32 per wave)
constexpr int BN = 64;    // keys per LDS tile
constexpr int SUB = 32;   // keys per pipeline step (the contraction length of one P V MFMA)
constexpr int NWAVE = 8;  // two per SIMD
constexpr int64_t kCUs = 256;  // compute units of the MI355X (one workgroup of this kernel each)
constexpr int64_t kTileMajorBelowWorkgroups = 2048;  // 256-row workgroups in a launch below which the grid runs the heaviest tiles of all KV heads first
constexpr int64_t kListedFromWorkgroups = 4096;  // launches from which a caller's bound on the rows of all requests may shrink the grid
constexpr int kListedMaxBatch = 4096;            // (every workgroup walks the batch's lengths once)
constexpr float kLazyRescale = 8.f;  // log2 units the running max may lag before O is rescaled

template <typename T> struct Mfma;
template <> struct Mfma<F16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mfma<BF16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// The same MFMAs issued from inline assembly with the accumulator tied to the destination.  Left to itself the register
// allocator gives every 16x16 result a fresh register tuple (this shape allows any overlap of destination and
// accumulator), the accumulators then wander through the register file over the unrolled loop and the kernel spills.
// The compiler's hazard bookkeeping does not cover these: each use below is far enough from the producers and
// consumers of its operands (see the fast loop).
template <typename T> struct MfmaAsm;
template <> struct MfmaAsm<F16> {
  static __device__ __forceinline__ void acc(f32x4& c, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void first(f32x4& c, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
};
template <> struct MfmaAsm<BF16> {
  static __device__ __forceinline__ void acc(f32x4& c, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void first(f32x4& c, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
};

// The P V product always runs on the f16 MFMA: P keeps 11 significant bits there (8 as
// bfloat16, which alone would cost ~1.1e-3 relative error in O).  A bfloat16 V tile is
// therefore converted to f16 while it is staged into LDS; every bfloat16 value with
// magnitude in [2^-14, 65504] is exactly representable, larger ones saturate to +-65504.
template <typename T> __device__ __forceinline__ u32x4 to_pv_operand(const u32x4& w);
template <> __device__ __forceinline__ u32x4 to_pv_operand<F16>(const u32x4& w) { return w; }
template <> __device__ __forceinline__ u32x4 to_pv_operand<BF16>(const u32x4& w) {
  // round-toward-zero conversion: exact for every bfloat16 in fp16's normal range, and a magnitude above 65504
  // becomes +-65504 without a separate clamp
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float lo, hi;
    unpack2<BF16>(w[i], lo, hi);
    r[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
  return r;
}

// A query column of a 16x16 block lives in the four lanes c, c + 16, c + 32, c + 48: maximum / sum over them.
// ds_swizzle in bit mode (lane ^ 16 inside each half of the wave) and v_permlane32_swap (the other half) need no address
// register, so nothing of this is computed ahead of the rare branch that uses it.
__device__ __forceinline__ float lane_xor16(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // and 0x1f, or 0, xor 0x10
}
__device__ __forceinline__ float lane_xor32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // r[0] = (lower, lower), r[1] = (upper, upper)
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}
__device__ __forceinline__ float column_max(float v) {
  v = fmaxf(v, lane_xor16(v));
  return fmaxf(v, lane_xor32(v));
}
__device__ __forceinline__ float column_sum(float v) {
  v += lane_xor16(v);
  return v + lane_xor32(v);
}

// LDS: a ring of four K tiles at [0, 64K) and a ring of four V tiles at [64K, 128K); a tile is [64 rows][16 chunks of 16 bytes]
// and the chunk index is XORed with swz_k(row) / swz_v(row).
constexpr int kTileBytes = BN * 256;
constexpr int kRing = 4;  // tiles per ring
constexpr int kLdsV = kRing * kTileBytes;
constexpr int kLdsBytes = 2 * kRing * kTileBytes;
template <bool HALF> constexpr int kRingOf = HALF ? 2 : kRing;          // the four-wave shape keeps rings of two tiles
template <bool HALF> constexpr int kLdsVOf = kRingOf<HALF> * kTileBytes;  // where its V ring starts
// The XOR on the 16-byte chunk index differs between the two rings, each chosen by measurement on the read pattern of
// its operand (LDS has 64 four-byte banks; which lanes of a wide read are served together is not documented):
// sixteen K rows read with ds_read_b128 run at the rate of a linear read with row & 15 (and at half of it with the V
// ring's XOR); the transposing V reads, 32 contiguous bytes from each of eight rows per half wave, do so with the XOR
// below (and not with row & 15).  Only the low four bits of the row count, so rows 16 apart share their XOR.
__device__ __forceinline__ int swz_k(int row) { return row & 15; }
__device__ __forceinline__ int swz_v(int row) { return ((row & 7) << 1) | ((row >> 3) & 1); }

typedef __attribute__((address_space(3))) i16x4* lds_i16x4_ptr;
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;

// s_waitcnt on the vector-memory counter only (expcnt / lgkmcnt fields left at their maximum)
template <int N> __device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }

// K A-operands of one 32-key sub-tile, ka[kb][ks] = K[16 kb + lane % 16][32 ks + 8 (lane / 16) .. + 7]: 8 x 16 bytes per lane.
// koff0 is the lane's byte offset for key block 0 and k-step 0; the swizzle is an XOR on the chunk index, so k-step ks
// sits at koff0 ^ (ks << 6), key block 1 sixteen rows (4 KB) further.  lds_k_sub is the LDS byte address of the
// sub-tile (a multiple of 8 KB, so adding the offset never carries into the XORed bits).
__device__ __forceinline__ void load_k_operands(int lds_k_sub, int koff0, u32x4 (&ka)[2][4]) {
  const int base = lds_k_sub + koff0;
#pragma unroll
  for (int kb = 0; kb < 2; kb++)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) ka[kb][ks] = *(const __attribute__((address_space(3))) u32x4*)((base ^ (ks << 6)) + kb * (16 * 256));
}
// V^T A-operands of one 32-key sub-tile through transposing LDS reads: va[db] = V^T[16 db + lane % 16][the lane group's
// eight keys], which are keys 4g .. 4g+3 and 16+4g .. 16+4g+3 of the sub-tile (g = lane / 16): the keys whose scores
// the lane group holds after S^T = K Q^T.  voff0 is the lane's byte offset for d-block 0 and the first four keys;
// d-block db sits at voff0 ^ (db << 5), the second four keys sixteen rows (4 KB) further.
__device__ __forceinline__ void load_v_operands(int lds_v_sub, int voff0, u32x4 (&va)[8]) {
  const int base = lds_v_sub + voff0;
#pragma unroll
  for (int db = 0; db < 8; db++) {
    const i16x4 xa = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(base ^ (db << 5)));
    const i16x4 xb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)((base ^ (db << 5)) + 16 * 256));
    const u32x2 wa = __builtin_bit_cast(u32x2, xa), wb = __builtin_bit_cast(u32x2, xb);
    va[db] = u32x4{wa[0], wa[1], wb[0], wb[1]};
  }
}

// a wave-uniform pointer, moved to scalar registers if the compiler held it in vector registers
__device__ __forceinline__ const char* uniform_ptr(const char* ptr) {
  const uint64_t u = (uint64_t)ptr;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}

// DV: the V tiles are fp16 in memory and go straight into LDS; otherwise (bf16 V) they pass through registers and are
// converted on the way.
// SPLIT: a workgroup owns 128 query rows instead of 256: waves w and w + 4 (one SIMD) hold the same 32 rows and take the
// even and the odd 32-key sub-tiles of every tile; their partial results meet in LDS after the loop.  Half the rows per
// workgroup at the same per-wave shape: for launches with too few 256-row workgroups to fill and balance the chip.
// HALF: four waves and 128 query rows, 32 per wave and every key, with rings of two tiles (64 KB of LDS): two such
// workgroups fit a CU, and one's start-up, finish and turn-over run beside the other's tiles.  For launches whose
// workgroups are short (a few tiles each): there a workgroup that fills the CU spends as long starting and ending as working.
// A 16-byte store that goes through to memory as it is issued (system-scope bits) instead of waiting in the L2 as a dirty
// line until the end of the launch.  From inline assembly (the compiler has no such store that is not atomic); the
// s_nop keeps vector instructions off the data registers for the two cycles a store of more than 64 bits needs.
__device__ __forceinline__ void store16_through(float* addr, const f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(addr), "v"(v) : "memory");
}

template <typename T, int MODE, bool DV, bool SPLIT, bool HALF = false>
__global__ __launch_bounds__(HALF ? NWAVE * 32 : NWAVE * 64, HALF ? 2 : 1) void prefill_kernel(PrefillParams p) {
  static_assert(DV || !SPLIT, "the split variant takes fp16 V tiles only");
  static_assert(!HALF || (DV && !SPLIT), "the four-wave variant takes fp16 V tiles only and is not split");
  // (namespace-scope constants: a local one named inside the lambdas below would be captured, and a closure that holds
  // anything but references the optimiser can see through is kept in memory, with every scalar operand it feeds)
  constexpr int RING = kRingOf<HALF>;            // tiles per ring
  constexpr int LDSV = kLdsVOf<HALF>;            // the V ring behind the K ring
  // (behind the rings, for the epilogue that folds into (o, m, l): a kilobyte per wave for the old m and l of its rows)
  constexpr int kStateOff = 2 * RING * kTileBytes;
  __shared__ __attribute__((aligned(1024))) char lds[kStateOff + (MODE == 1 ? (HALF ? NWAVE / 2 : NWAVE) * 1024 : 0)];
  constexpr int BMW = SPLIT || HALF ? BM / 2 : BM;  // query rows of this workgroup

  // Workgroup ids go to the 8 XCDs round-robin.  The (query head, query tile) units of one KV head are dealt to p.slices
  // XCDs (1 when the KV heads are a multiple of 8, else as many as it takes for hkv * slices to be one), so that the
  // workgroups sharing a KV head's K/V meet in few L2s and every XCD has work whatever the head count.
  const int group = p.group;
  uint32_t j = blockIdx.x >> 3;
  const int xcd = blockIdx.x & 7;
  // A launch of the four-wave shape that fits the chip at once (two workgroups per CU) is paired up by the hardware:
  // workgroup id and id + 256 share a CU.  The second 256 then run from the lightest tile upwards, so that the heaviest
  // meets the lightest and every CU gets the same work.
  if (HALF && p.fold_from && j >= (uint32_t)p.fold_from) j = (uint32_t)p.fold_sum - j;
  // Two orders of the grid within a request, by which of the two indices runs fastest (the host sets d_first / d_second):
  // launches of a few workgroups per CU deal the heaviest query tiles of all KV heads first (under causal masking tile z
  // walks z + 1 key blocks), so that a CU that has finished a light tile of the first round takes a heavy one of the rest
  // and the last round is made of the lightest tiles; large launches take one KV head at a time per XCD, whose K/V then
  // serves all the workgroups the XCD runs.  One request after the other in both (its K/V stays in the L2s).
  const uint32_t j1 = div_by(j, p.d_first);
  const int r1 = (int)(j - j1 * p.n_first);
  int up, slot, b, cut, nz = p.nz;
  if (p.listed) {
    // The grid above is sized by the longest request times the batch (the host knows max_q_len, not the lengths): a
    // batch of one long request and many short ones is mostly workgroups without rows.  Here the grid has a workgroup
    // per unit that can exist (from an upper bound of the rows of all requests together) and a workgroup finds its
    // request by numbering the units of all requests: request b has (query heads per KV head / heads per workgroup) x
    // ceil(q_len[b] / positions per workgroup) of them, heaviest tile first.  Every wave numbers them by itself, 64
    // requests per step (an inclusive sum over the lanes); no LDS, no barrier.
    slot = r1;
    const uint32_t unit = j1;  // (KV head slots run fastest)
    const int lane_id = threadIdx.x & 63;
    uint32_t carry = 0;
    b = -1;
    up = 0;
    for (int b0 = 0; b0 < p.batch && b < 0; b0 += 64) {  // (until the unit's request is found)
      const int bb = b0 + lane_id;
      const int len = bb < p.batch ? p.q_len[bb] : 0;
      const uint32_t tiles = len > 0 ? ((uint32_t)len + (1u << p.rows_shift) - 1) >> p.rows_shift : 0;
      const uint32_t units = tiles * (uint32_t)group;
      uint32_t incl = units;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t below = __shfl_up(incl, d, 64);
        if (lane_id >= d) incl += below;
      }
      const uint32_t chunk_total = __builtin_amdgcn_readlane(incl, 63);
      if (unit < carry + chunk_total) {  // (the same for every lane)
        const uint64_t past = __builtin_amdgcn_ballot_w64(carry + incl > unit);  // lanes whose units end behind this one
        const int l0 = __builtin_amdgcn_readfirstlane(__builtin_ctzll(past));
        b = b0 + l0;
        up = (int)(unit - (carry + __builtin_amdgcn_readlane(incl, l0) - __builtin_amdgcn_readlane(units, l0)));
        nz = (int)__builtin_amdgcn_readlane(tiles, l0);
      }
      carry += chunk_total;
    }
    if (b < 0) return;  // past the last unit that exists
    cut = 0;
  } else {
    j = div_by(j1, p.d_second);
    const int r2 = (int)(j1 - j * p.n_second);
    up = p.tile_major ? r2 : r1;
    slot = p.tile_major ? r1 : r2;
    // (sequence, cut of its KV chunk): j < batch * kv_cuts for every workgroup of the grid
    b = (int)div_by(j, p.d_cuts);
    cut = (int)j - b * p.kv_cuts;
  }
  // The request's six numbers, all requested before the first of them is used (one memory latency instead of three on
  // the way to the first tile load; a workgroup's start-up is what a short launch is made of).
  const int q_len = p.q_len[b], kv_len_all = p.kv_len[b], qf = p.q_first[b], kf_all = p.kv_first[b];
  const int q_start32 = p.q_start[b], kv_start32 = p.kv_start[b];
  const int o_start32 = p.o_start ? p.o_start[b] : q_start32;
  asm volatile("" ::"s"(q_len), "s"(kv_len_all), "s"(qf), "s"(kf_all), "s"(q_start32), "s"(kv_start32), "s"(o_start32));
  // the cut's share of the chunk: keys [cut, cut + 1) * kv_cut_len, key n of the chunk at global position kv_first + n * peers
  const int key0 = cut * p.kv_cut_len;
  const int kv_rest = kv_len_all - key0;
  const int kv_len = kv_rest < 0 ? 0 : (kv_rest < p.kv_cut_len ? kv_rest : p.kv_cut_len);
  const int kf = kf_all + key0 * p.peers;
  const int64_t q_start = q_start32, kv_start = (int64_t)kv_start32 + key0, o_start = o_start32 + (int64_t)cut * p.o_cut_rows;
  const int vh = xcd + 8 * slot;  // (KV head, slice) pair: always < hkv * slices
  const int kvh = (int)div_by((uint32_t)vh, p.d_slices);
  const int u = up * p.slices + (vh - kvh * p.slices);
  if (u >= group * nz) return;
  const int zr = (int)div_by((uint32_t)u, p.d_group), gq = u - zr * group;
  const int z = nz - 1 - zr;

  // The workgroup's rows: 1 << pack_shift query heads of the KV head side by side, BMW >> pack_shift query positions of
  // each (grouped-query attention: the heads of a group read the same K/V, so a workgroup of several of them walks the
  // same tiles as one of a single head with as many rows, but its positions end sooner: a quarter of the diagonal with
  // four heads, one masked tile instead of four and a sixteenth of the scores computed for nothing).
  const int rows_wg = BMW >> p.pack_shift;  // query positions of this workgroup
  const int m_lo = z * rows_wg;
  if (m_lo >= q_len) return;
  const int P = p.peers;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int qc = lane & 15, g = lane >> 4;  // query column within a 16-row block, lane group
  const int wrow = SPLIT ? (wave & 3) : wave;  // which 32 rows of the workgroup
  const int kp = SPLIT ? (wave >> 2) : 0;      // SPLIT: parity of the sub-tiles this wave takes
  const int wph_shift = (SPLIT || HALF ? 2 : 3) - p.pack_shift;  // log2 of the 32-row groups per head
  const int h = kvh * p.heads_per_kv + (gq << p.pack_shift) + (wrow >> wph_shift);  // the wave's query head

  // keys of this KV chunk visible to global query position qpos (RING:156-159)
  auto visible_keys = [&](int qpos) -> int {
    const int dq = qpos - kf;
    const int n = dq >= 0 ? (int)div_by((uint32_t)dq, p.d_peers) + 1 : 0;
    return n > kv_len ? kv_len : n;
  };
  const int m_hi = (m_lo + rows_wg < q_len ? m_lo + rows_wg : q_len) - 1;
  const int nt = (visible_keys(qf + m_hi * P) + BN - 1) / BN;  // tiles the workgroup walks

  const int m_w0 = m_lo + (wrow & ((1 << wph_shift) - 1)) * 32;

  // The old m and l of the wave's rows (MODE 1) are asked for first of all and go straight into LDS, a float per lane:
  // they have landed when Q has (loads return in order), cost no register over the loops, and the epilogue knows without
  // a trip to memory whether a row is still in its start state (the first step of a ring, a prefill on one GPU), whose
  // old o is never read.
  if (MODE == 1) {
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const int m = m_w0 + 16 * qb + qc;
      const int64_t at = (o_start + (m < q_len ? m : 0)) * p.ml_st + (int64_t)h * p.ml_sh;
      const float* pm = p.m + at;
      const float* pl = p.l + at;
      const int dst = (int)(uintptr_t)(__attribute__((address_space(3))) char*)lds + kStateOff + wave * 1024 + qb * 256;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %2, off\n\t"
                   "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %3, off" ::"s"(dst), "s"(dst + 512), "v"(pm), "v"(pl)
                   : "m0", "memory");
    }
  }

  // Q as B operands: qreg[qb][ks] = Q[row 16 qb + qc][32 ks + 8g .. +7]; cnt[qb] = keys that row sees (0 past the end)
  u32x4 qreg[2][4];
  int cnt[2];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    const int m = m_w0 + 16 * qb + qc;
    const bool ok = m < q_len;
    const char* src = (const char*)p.q + ((q_start + (ok ? m : 0)) * p.q_st + (int64_t)h * p.q_sh + 8 * g) * 2;
#pragma unroll
    // (a row past the end holds the request's first row instead: it sees no key, cnt = 0, and is never stored; no select
    // stands between the loads and the tile loads that follow)
    for (int ks = 0; ks < 4; ks++) qreg[qb][ks] = *(const u32x4*)(src + ks * 64);
    cnt[qb] = ok ? visible_keys(qf + m * P) : 0;
  }

  // keys every row of the wave sees: sub-tiles below this need no mask (rows past the end of the sequence count as rows
  // that see nothing, so a wave that holds some masks everywhere)
  const int cnt_wave = __builtin_amdgcn_readfirstlane(m_w0 + 31 < q_len ? visible_keys(qf + m_w0 * P) : 0);
  int koff0 = qc * 256 + ((g ^ swz_k(qc)) << 4);
  int voff0;
  {
    // a transposing read hands lane c of a 16-lane group column d0 + c of the 4 x 16 block its lanes point at:
    // lane c points at row (c >> 2), columns d0 + 4 (c & 3) .. + 3
    const int row = 4 * g + (qc >> 2);
    const int d_off = 4 * (qc & 3);
    voff0 = row * 256 + (((d_off >> 3) ^ swz_v(row)) << 4) + (d_off & 7) * 2;
  }
  const int lds_base = (int)(uintptr_t)(__attribute__((address_space(3))) char*)lds;

  // staging: wave w owns rows [8w, 8w+8) of every tile, 4 rows per instruction.  The chunk bases and row strides are
  // wave-uniform and held in scalar registers.
  const char* kg = uniform_ptr((const char*)p.k + (kv_start * p.k_st + (int64_t)kvh * p.k_sh) * 2);
  const char* vg = uniform_ptr((const char*)p.v + (kv_start * p.v_st + (int64_t)kvh * p.v_sh) * 2);
  const int k_row_bytes = __builtin_amdgcn_readfirstlane((int)p.k_st * 2), v_row_bytes = __builtin_amdgcn_readfirstlane((int)p.v_st * 2);
  // staging rows of a wave: eight waves take rows [8w, 8w+8) of a tile in two instructions four rows apart; the four
  // waves of HALF take rows 4w + 16i + (0..3) in four instructions sixteen rows apart (rows sixteen apart share their
  // XOR, so one lane offset serves all four and the tile pointer moves instead)
  constexpr int NI = HALF ? 4 : 2;          // load instructions per tile and wave
  constexpr int ROW_STEP = HALF ? 16 : 4;   // rows between them
  const int st_row = (HALF ? 4 : 8) * wave + (lane >> 4);  // the lane's row of the tile in the first of its instructions
  const int last_row = kv_len - 1;
  // byte offset of the lane's 16 bytes from the tile's first row, row and swizzled chunk
  uint32_t k_lane_off[2], v_lane_off[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int r = st_row + 4 * i;
    k_lane_off[i] = (uint32_t)(r * k_row_bytes) + (((lane & 15) ^ swz_k(r)) << 4);
    v_lane_off[i] = (uint32_t)(r * v_row_bytes) + (((lane & 15) ^ swz_v(r)) << 4);
  }
  const int st_lds = lds_base + (HALF ? 4 : 8) * wave * 256;
  u32x4 vst[2];
  // All tile loads are issued from inline assembly: behind a load to LDS that the compiler sees, it waits for vmcnt(0)
  // before every later LDS read (it cannot tell which LDS bytes the load writes); the waits for these loads are the
  // explicit wait_vmem calls.  The s_nop is the wait state a write of m0 needs before an LDS-DMA load reads it.
  //
  // Tile `t` of K (of V) into ring slot S, rows past the end of the chunk replaced by its last row (they are masked
  // where they are used, and a tile that lies wholly past the end is never read): any tile index is safe.  The tile
  // pointer is scalar (a tile past the end becomes the last one), the lane's offset moves back to the last row.
  const int last_tile = last_row / BN;
  auto clamped_tile = [&](const char* base, int row_bytes, uint32_t lane_off, int i, int t, const char*& tile, uint32_t& off)
                          __attribute__((always_inline)) {
    const int tc = __builtin_amdgcn_readfirstlane(t < last_tile ? t : last_tile);
    tile = base + (int64_t)tc * BN * row_bytes;
    // rows of the tile between the lane's row, st_row + 4 i, and the last one of the chunk (the scalar part on its own,
    // so that no further per-lane values are kept across the loop)
    const int lim = __builtin_amdgcn_readfirstlane(last_row - tc * BN - ROW_STEP * i);
    int back = st_row - lim;
    back = back < 0 ? 0 : back;
    off = lane_off - (uint32_t)(back * row_bytes);
  };
  auto load_k_clamped = [&](auto slot_tag, int t) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_tag)::value;
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const char* tile;
      uint32_t off;
      clamped_tile(kg, k_row_bytes, HALF ? k_lane_off[0] + (uint32_t)(16 * i * k_row_bytes) : k_lane_off[i & 1], i, t, tile, off);
      const int dst = st_lds + S * kTileBytes + i * ROW_STEP * 256;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(tile) : "m0", "memory");
    }
  };
  auto load_v_clamped = [&](auto slot_tag, int t) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_tag)::value;
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const char* tile;
      uint32_t off;
      clamped_tile(vg, v_row_bytes, HALF ? v_lane_off[0] + (uint32_t)(16 * i * v_row_bytes) : v_lane_off[i & 1], i, t, tile, off);
      if (DV) {
        const int dst = st_lds + kLdsVOf<HALF> + S * kTileBytes + i * ROW_STEP * 256;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(tile) : "m0", "memory");
      } else {
        u32x4 w;  // into registers: see store_v_tile
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(w) : "v"(off), "s"(tile) : "memory");
        vst[i & 1] = w;
      }
    }
  };
  // (bf16 V only) the tile held in registers, converted, into ring slot S
  auto store_v_tile = [&](auto slot_tag) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_tag)::value;
    if (!DV) {
#pragma unroll
      for (int i = 0; i < 2; i++)
        *(u32x4*)(lds + kLdsVOf<HALF> + S * kTileBytes + (8 * wave + 4 * i) * 256 + lane * 16) = to_pv_operand<T>(vst[i]);
    }
  };

  // Tiles that lie wholly inside the chunk: running scalar tile pointers and the lane's 32-bit offset, K tile it + KA
  // and V tile it + VA of iteration `it` into their ring slots.
  constexpr int KA = SPLIT ? 4 : HALF ? 2 : 3, VA = SPLIT ? 3 : HALF ? 1 : 2;  // how far ahead of the tile in work the loads run
  const char* kt_run = kg;
  const char* vt_run = vg;
  auto load_tiles_fast = [&](auto r_tag) __attribute__((always_inline)) {
    constexpr int R = decltype(r_tag)::value;
    constexpr int kslot = ((R + KA) & 3) * kTileBytes, vslot = kLdsVOf<HALF> + ((R + VA) & 3) * kTileBytes;
    // one block, so that nothing is put between the loads (a wave issues an instruction every five cycles or so,
    // whatever it is)
    if (DV) {
      asm volatile(
          "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %8\n\t"
          "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %5, %8\n\t"
          "s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %6, %9\n\t"
          "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %7, %9" ::"s"(st_lds + kslot),
          "s"(st_lds + kslot + 1024), "s"(st_lds + vslot), "s"(st_lds + vslot + 1024), "v"(k_lane_off[0]), "v"(k_lane_off[1]),
          "v"(v_lane_off[0]), "v"(v_lane_off[1]), "s"(kt_run), "s"(vt_run)
          : "m0", "memory");
    } else {
      asm volatile(
          "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %4\n\t"
          "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %4" ::"s"(st_lds + kslot),
          "s"(st_lds + kslot + 1024), "v"(k_lane_off[0]), "v"(k_lane_off[1]), "s"(kt_run)
          : "m0", "memory");
    }
    kt_run += (int64_t)BN * k_row_bytes;
    if (DV) vt_run += (int64_t)BN * v_row_bytes;
  };
  // A V tile that has to be converted on its way into LDS goes through registers: loaded one iteration before it is
  // stored (three tiles ahead of its use), so the wait in front of the store is for loads a whole iteration old.
  auto load_v_regs_fast = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; i++)
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(vst[i]) : "v"(v_lane_off[i]), "s"(vt_run) : "memory");
    vt_run += (int64_t)BN * v_row_bytes;
  };

  // HALF: the four loads of K tile it + 2 into slot R (the slot of tile it, whose last operands the first MFMA phase of
  // the iteration has read) and of V tile it + 1 into slot R ^ 1, on their own: they go out at different points.
  auto load_k_fast_half = [&](auto r_tag) __attribute__((always_inline)) {
    constexpr int kslot = decltype(r_tag)::value * kTileBytes;
    const char* b1 = kt_run + 16 * (int64_t)k_row_bytes;
    const char* b2 = kt_run + 32 * (int64_t)k_row_bytes;
    const char* b3 = kt_run + 48 * (int64_t)k_row_bytes;
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %5\n\t"
        "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %6\n\t"
        "s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %7\n\t"
        "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %8" ::"s"(st_lds + kslot),
        "s"(st_lds + kslot + 16 * 256), "s"(st_lds + kslot + 32 * 256), "s"(st_lds + kslot + 48 * 256), "v"(k_lane_off[0]), "s"(kt_run),
        "s"(b1), "s"(b2), "s"(b3)
        : "m0", "memory");
    kt_run += (int64_t)BN * k_row_bytes;
  };
  auto load_v_fast_half = [&](auto r_tag) __attribute__((always_inline)) {
    constexpr int vslot = kLdsVOf<HALF> + (decltype(r_tag)::value ^ 1) * kTileBytes;
    const char* b1 = vt_run + 16 * (int64_t)v_row_bytes;
    const char* b2 = vt_run + 32 * (int64_t)v_row_bytes;
    const char* b3 = vt_run + 48 * (int64_t)v_row_bytes;
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %5\n\t"
        "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %6\n\t"
        "s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %7\n\t"
        "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %8" ::"s"(st_lds + vslot),
        "s"(st_lds + vslot + 16 * 256), "s"(st_lds + vslot + 32 * 256), "s"(st_lds + vslot + 48 * 256), "v"(v_lane_off[0]), "s"(vt_run),
        "s"(b1), "s"(b2), "s"(b3)
        : "m0", "memory");
    vt_run += (int64_t)BN * v_row_bytes;
  };

  // O^T accumulators: oacc[db][qb][r] = O[row 16 qb + qc][16 db + 4g + r]
  f32x4 oacc[8][2];
#pragma unroll
  for (int db = 0; db < 8; db++)
#pragma unroll
    for (int qb = 0; qb < 2; qb++) oacc[db][qb] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
  f32x4 s[2][2];  // s[kb][qb][r] = S[row 16 qb + qc][key 16 kb + 4g + r of the sub-tile]
  u32x4 pk[2];
  u32x4 ka[2][4], va[8];

  // Every tile goes through the same pipelined loop, and the ring slot of a tile (it & 3 == R) is a compile-time
  // constant there, so every LDS read is a fixed register plus an immediate.  A 32-key step has an MFMA phase
  // (S(i) = K(i) Q^T, then O += V(i') P(i') for the wave's previous sub-tile i', each operand register refilled for the
  // next step right behind the MFMA that consumed it) and a softmax phase (P(i)).
  // Running state, per 16-row block qb: neg_m = -m (+inf while the row has seen no key), thr_raw = (m + 2^kLazyRescale)
  // / scale, l = lacc[qb] (any element).
  int kaddr[4], vaddr[8];
  float neg_m[2] = {INFINITY, INFINITY}, thr_raw[2] = {-INFINITY, -INFINITY};
  // row sums of P on the matrix pipe: lacc[qb] += ones(16 x 32) P^T, every element of a lane's lacc[qb] is the sum of
  // its query column over all keys so far (of the fp16 P values, the ones that multiply V)
  f32x4 lacc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
  // (held in registers as an opaque value: rebuilt from constants next to the inline-assembly MFMAs it would be
  // written by vector moves the compiler cannot order against them)
  u32x4 ones = u32x4{0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  asm volatile("" : "+v"(ones));
  const float scale = p.scale_log2;
  // (wave-uniform: kept in a scalar register, the vector registers are all taken)
  float inv_scale;
  {
    const float inv = 1.f / p.scale_log2;
    asm volatile("v_readfirstlane_b32 %0, %1" : "=s"(inv_scale) : "v"(inv));
  }
  auto fphase_mfma = [&](auto par_tag, auto r_tag, auto lsum_tag) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_tag)::value;  // sub-tile i = 2it + PAR (SPLIT: the parity is in the address registers)
    constexpr int R = decltype(r_tag)::value;
    constexpr bool LSUM = decltype(lsum_tag)::value;  // the row sums of the P consumed here go through the matrix pipe
    // K operands of the wave's next sub-tile, V operands of this one
    constexpr int koff = SPLIT ? ((R + 1) & 3) * kTileBytes : (PAR ? ((R + 1) & (kRingOf<HALF> - 1)) : R) * kTileBytes + (PAR ^ 1) * (SUB * 256);
    constexpr int voff = SPLIT ? R * kTileBytes : R * kTileBytes + PAR * (SUB * 256);
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
        if (ks == 0) {
          MfmaAsm<T>::first(s[kb][0], ka[kb][ks], qreg[0][ks]);
          MfmaAsm<T>::first(s[kb][1], ka[kb][ks], qreg[1][ks]);
        } else {
          MfmaAsm<T>::acc(s[kb][0], ka[kb][ks], qreg[0][ks]);
          MfmaAsm<T>::acc(s[kb][1], ka[kb][ks], qreg[1][ks]);
        }
        ka[kb][ks] = *(const __attribute__((address_space(3))) u32x4*)(kaddr[ks] + koff + kb * (16 * 256));
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
    for (int db = 0; db < 8; db++) {
      MfmaAsm<F16>::acc(oacc[db][0], va[db], pk[0]);
      MfmaAsm<F16>::acc(oacc[db][1], va[db], pk[1]);
      const i16x4 xa = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(vaddr[db] + voff));
      const i16x4 xb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(vaddr[db] + voff + 16 * 256));
      const u32x2 wa = __builtin_bit_cast(u32x2, xa), wb = __builtin_bit_cast(u32x2, xb);
      va[db] = u32x4{wa[0], wa[1], wb[0], wb[1]};
      __builtin_amdgcn_sched_barrier(0);
    }
    if (LSUM) {
      MfmaAsm<F16>::acc(lacc[0], ones, pk[0]);
      MfmaAsm<F16>::acc(lacc[1], ones, pk[1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // P(i) = exp2(S(i) * scale - m) with the current m, and the lane's largest score of each block in mx[qb].  Sixteen
  // independent operations at a time, the levels of the maxima's trees spread between them: this wave's vector work
  // runs beside the other wave's MFMAs only without short dependent chains and without dot-product instructions
  // (those queue behind the MFMAs).
  // MASKED (tiles on the diagonal or at the end of the chunk): key n of the chunk counts for a row only if n < cnt,
  // the others' scores become -inf first; a row that has seen no key yet (neg_m = +inf) computes with m = 0.
  // MASKED iterations also return the sums of the lane's P values in fp32 (ps): a row that sees only a few keys needs its
  // row sum more exact than the fp16 P values give it.
  auto compute_p = [&](auto masked_tag, int i, float (&mx)[2], float (&ps)[2]) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    float ma[2], mb[2], t[2][8], nm[2];
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      nm[qb] = neg_m[qb];
      if (MASKED) nm[qb] = neg_m[qb] == INFINITY ? 0.f : neg_m[qb];
    }
    if (MASKED && (i + 1) * SUB > cnt_wave) {  // (wave-uniform: the wave's first row sees the fewest keys)
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        const int rel = cnt[qb] - i * SUB - 4 * g;  // keys from the lane's first one of key block 0 to the row's limit
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int r = 0; r < 4; r++) s[kb][qb][r] = (16 * kb + r < rel) ? s[kb][qb][r] : -INFINITY;
      }
    }
    if (MASKED) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        ma[qb] = fmaxf(fmaxf(s[0][qb][0], s[0][qb][1]), s[0][qb][2]);
        mb[qb] = fmaxf(fmaxf(s[0][qb][3], s[1][qb][0]), s[1][qb][1]);
      }
    }
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int r = 0; r < 4; r++) t[qb][4 * kb + r] = __builtin_fmaf(s[kb][qb][r], scale, nm[qb]);
    __builtin_amdgcn_sched_barrier(0);
    if (MASKED) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++) ma[qb] = fmaxf(fmaxf(ma[qb], s[1][qb][2]), s[1][qb][3]);
    }
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int e = 0; e < 8; e++) t[qb][e] = __builtin_amdgcn_exp2f(t[qb][e]);
    __builtin_amdgcn_sched_barrier(0);
    if (MASKED) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++) mx[qb] = fmaxf(ma[qb], mb[qb]);
    }
    if (MASKED) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
        ps[qb] = ((t[qb][0] + t[qb][1]) + (t[qb][2] + t[qb][3])) + ((t[qb][4] + t[qb][5]) + (t[qb][6] + t[qb][7]));
    }
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int e = 0; e < 4; e++) pk[qb][e] = pack2<F16>(t[qb][2 * e], t[qb][2 * e + 1]);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto fphase_softmax = [&](auto masked_tag, int i) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    float mx[2], ps[2];
    compute_p(masked_tag, i, mx, ps);
    bool over;
    if (MASKED) {
      over = (mx[0] > thr_raw[0]) | (mx[1] > thr_raw[1]);
    } else {
      // Every key counts here, so no maxima are needed to tell whether the running ones still hold: some P is 2 or more
      // (also infinite, as for the first keys a row sees, when m is still -inf) exactly if bit 14 of one of the packed
      // fp16 values, the top bit of its exponent, is set.  Six instructions instead of the eleven of the maxima.
      const uint32_t any = (pk[0][0] | pk[0][1] | pk[0][2]) | (pk[0][3] | pk[1][0] | pk[1][1]) | (pk[1][2] | pk[1][3]);
      over = (any & 0x40004000u) != 0;
    }
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(over) != 0, 0)) {
      // rare: some score is above the lazy threshold (always so for the first key a row sees); raise the running maxima
      // and redo the sub-tile (the accumulators' last MFMAs were issued before this phase's barrier and the whole of
      // compute_p lies between them and these multiplies)
      if (!MASKED) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
          mx[qb] = fmaxf(fmaxf(fmaxf(s[0][qb][0], s[0][qb][1]), fmaxf(s[0][qb][2], s[0][qb][3])),
                         fmaxf(fmaxf(s[1][qb][0], s[1][qb][1]), fmaxf(s[1][qb][2], s[1][qb][3])));
      }
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        const float m_new = fminf(neg_m[qb], -column_max(mx[qb]) * scale);  // -max(m, mx*scale)
        // (a block of rows that still has seen no key keeps neg_m = +inf: no inf - inf)
        const float al = (MASKED && m_new == neg_m[qb]) ? 1.f : __builtin_amdgcn_exp2f(m_new - neg_m[qb]);
        neg_m[qb] = m_new;
        thr_raw[qb] = (kLazyRescale - m_new) * inv_scale;
        if (MASKED) l_run[qb] *= al;
        else lacc[qb] *= al;
#pragma unroll
        for (int db = 0; db < 8; db++) oacc[db][qb] *= al;
      }
      compute_p(masked_tag, i, mx, ps);
    }
    if (MASKED) {
      l_run[0] += ps[0];
      l_run[1] += ps[1];
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // The two waves that share a SIMD (w and w + 4) run the loop half a step apart, one in its MFMA phase while the other
  // is in its softmax phase (wave priorities make no measurable difference with this MFMA shape); a workgroup barrier
  // ends every phase.
  // Not SPLIT: iteration `it` is tile `it`, sub-tiles 2it and 2it+1.  The loads of K tile it+3 and V tile it+2 go out in
  // its first softmax phase; the wait before its second MFMA phase leaves only those in flight, so a tile is complete for
  // both groups one barrier before its first read, and no read of the slot a load overwrites is still pending when the
  // load is issued.
  // SPLIT: iteration `it` is sub-tile 2it + kp of tile `it`: one MFMA phase and one softmax phase, in which K tile it+4
  // and V tile it+3 are requested.  The group of waves 4-7 runs one phase behind: the last reads of the slots these loads
  // overwrite (K tile it, V tile it-1) were issued in its MFMA phase of iteration it-1, two barriers before its loads and
  // one before those of waves 0-3.  The wait at the end of an iteration leaves that iteration's loads in flight, so
  // tile it+4 is complete for everyone after iteration it+1 of waves 4-7, one phase before waves 0-3 first read it.
  // MASKED iterations clamp the rows they load to the end of the chunk and mask the scores; the others assume that the
  // tiles they load lie inside the chunk and that every row of the workgroup sees every key of the tile.
  auto request_tiles = [&](auto r_tag, auto masked_tag, int it) __attribute__((always_inline)) {
    constexpr int R = decltype(r_tag)::value;
    if constexpr (decltype(masked_tag)::value) {
      // (tiles that lie inside the chunk take the cheaper loads here too; the running pointers advance either way)
      if (it + KA < kv_len / BN) {
        load_tiles_fast(r_tag);
      } else {
        load_k_clamped(std::integral_constant<int, (R + KA) & 3>{}, it + KA);
        if constexpr (DV) load_v_clamped(std::integral_constant<int, (R + VA) & 3>{}, it + VA);
        kt_run += (int64_t)BN * k_row_bytes;
        if (DV) vt_run += (int64_t)BN * v_row_bytes;
      }
    } else {
      load_tiles_fast(r_tag);
    }
  };
  // HALF: iteration `it` is tile `it` in ring slots R = it & 1.  V tile it+1 is requested first, into the slot of
  // tile it-1 (last read in the second MFMA phase of iteration it-1, before that iteration's closing barrier); K tile
  // it+2 behind the barrier in the middle, into the slot of tile it, whose last operands the first MFMA phase has read.
  // The wait in front of that barrier leaves the V loads just issued in flight: K tile it+1, requested half an iteration
  // earlier and read in the second MFMA phase, is then complete in every wave.  The wait in front of the closing barrier
  // leaves the K loads in flight: V tile it+1 is complete before iteration it+1 reads it.
  auto request_v_half = [&](auto r_tag, auto masked_tag, int it) __attribute__((always_inline)) {
    constexpr int R = decltype(r_tag)::value;
    if constexpr (decltype(masked_tag)::value) {
      if (it + VA < kv_len / BN) {
        load_v_fast_half(r_tag);
      } else {
        load_v_clamped(std::integral_constant<int, R ^ 1>{}, it + VA);
        vt_run += (int64_t)BN * v_row_bytes;
      }
    } else {
      load_v_fast_half(r_tag);
    }
  };
  auto request_k_half = [&](auto r_tag, auto masked_tag, int it) __attribute__((always_inline)) {
    constexpr int R = decltype(r_tag)::value;
    if constexpr (decltype(masked_tag)::value) {
      if (it + KA < kv_len / BN) {
        load_k_fast_half(r_tag);
      } else {
        load_k_clamped(std::integral_constant<int, R>{}, it + KA);
        kt_run += (int64_t)BN * k_row_bytes;
      }
    } else {
      load_k_fast_half(r_tag);
    }
  };
  auto iteration = [&](auto r_tag, auto masked_tag, int it) __attribute__((always_inline)) {
    constexpr int R = decltype(r_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value;
    if constexpr (HALF) {
      request_v_half(r_tag, masked_tag, it);
      fphase_mfma(std::integral_constant<int, 0>{}, r_tag, std::integral_constant<bool, !MASKED>{});
      wait_vmem<4>();
      __builtin_amdgcn_s_barrier();
      request_k_half(r_tag, masked_tag, it);
      fphase_softmax(masked_tag, 2 * it);
      fphase_mfma(std::integral_constant<int, 1>{}, r_tag, std::integral_constant<bool, !MASKED>{});
      fphase_softmax(masked_tag, 2 * it + 1);
      wait_vmem<4>();
      __builtin_amdgcn_s_barrier();
    } else if (SPLIT) {
      fphase_mfma(std::integral_constant<int, 0>{}, r_tag, std::integral_constant<bool, !MASKED>{});
      __builtin_amdgcn_s_barrier();
      request_tiles(r_tag, masked_tag, it);
      fphase_softmax(masked_tag, 2 * it + kp);
      wait_vmem<4>();
      __builtin_amdgcn_s_barrier();
    } else {
      fphase_mfma(std::integral_constant<int, 0>{}, r_tag, std::integral_constant<bool, !MASKED>{});
      __builtin_amdgcn_s_barrier();
      request_tiles(r_tag, masked_tag, it);
      fphase_softmax(masked_tag, 2 * it);
      __builtin_amdgcn_s_barrier();
      if (DV) wait_vmem<4>();
      fphase_mfma(std::integral_constant<int, 1>{}, r_tag, std::integral_constant<bool, !MASKED>{});
      __builtin_amdgcn_s_barrier();
      fphase_softmax(masked_tag, 2 * it + 1);
      if (!DV) {
        // everything but this iteration's two K loads has arrived: the registers hold V tile it+2, and K tile it+2
        // (loaded one iteration ago) is complete as well
        asm volatile("s_waitcnt vmcnt(2)" : "+v"(vst[0]), "+v"(vst[1]));
        store_v_tile(std::integral_constant<int, (R + 2) & 3>{});
        if (MASKED) {
          load_v_clamped(std::integral_constant<int, 0>{}, it + 3);  // (into registers: the slot is not used)
        } else {
          load_v_regs_fast();  // V tile it+3
        }
      }
      __builtin_amdgcn_s_barrier();
    }
  };

  if (nt > 0) {
    // K tiles 0 .. KA-1 and V tiles 0 .. VA-1
    load_k_clamped(std::integral_constant<int, 0>{}, 0);
    load_k_clamped(std::integral_constant<int, 1>{}, 1);
    if (!HALF) load_k_clamped(std::integral_constant<int, 2>{}, 2);
    if (SPLIT) load_k_clamped(std::integral_constant<int, 3>{}, 3);
    if (DV) {
      load_v_clamped(std::integral_constant<int, 0>{}, 0);
      if (!HALF) load_v_clamped(std::integral_constant<int, 1>{}, 1);
      if (SPLIT) load_v_clamped(std::integral_constant<int, 2>{}, 2);
    } else {
      load_v_clamped(std::integral_constant<int, 0>{}, 0);
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(vst[0]), "+v"(vst[1]));
      store_v_tile(std::integral_constant<int, 0>{});
      load_v_clamped(std::integral_constant<int, 0>{}, 1);
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(vst[0]), "+v"(vst[1]));
      store_v_tile(std::integral_constant<int, 1>{});
      load_v_clamped(std::integral_constant<int, 0>{}, 2);  // stays in registers until the end of iteration 0
    }
    // The loop's trip count is the same for every wave of the workgroup (it holds barriers).  Tiles below n_plain are
    // visible to the first row of the workgroup, hence to all of them, hold 64 keys, and the tiles requested while they
    // are worked on lie inside the chunk; the loop over them is unrolled over the four ring slots.
    int n_plain = visible_keys(qf + m_lo * P) / BN;
    if (n_plain > kv_len / BN - KA) n_plain = kv_len / BN - KA;
    if (n_plain > nt) n_plain = nt;
    n_plain = n_plain < 0 ? 0 : (n_plain & ~(kRingOf<HALF> - 1));  // (the loop is unrolled over the ring)
    const int par_off = kp * (SUB * 256);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      kaddr[ks] = ((lds_base + koff0) ^ (ks << 6)) + par_off;
      asm volatile("" : "+v"(kaddr[ks]));
    }
#pragma unroll
    for (int db = 0; db < 8; db++) {
      vaddr[db] = ((lds_base + kLdsVOf<HALF> + voff0) ^ (db << 5)) + par_off;
      asm volatile("" : "+v"(vaddr[db]));
    }
    if (DV) wait_vmem<0>();
    else wait_vmem<2>();
    __syncthreads();
    // operands of the wave's first step; its "previous" product is a V tile times a zero P
    load_k_operands(lds_base + par_off, koff0, ka);
    load_v_operands(lds_base + kLdsVOf<HALF> + par_off, voff0, va);
    pk[0] = u32x4{0, 0, 0, 0};
    pk[1] = u32x4{0, 0, 0, 0};
    kt_run = uniform_ptr(kg + (int64_t)KA * BN * k_row_bytes);
    vt_run = uniform_ptr(vg + (int64_t)(DV ? VA : 3) * BN * v_row_bytes);
    int it = 0;
    if (wave >= 4) __builtin_amdgcn_s_barrier();
    for (; it < n_plain; it += kRingOf<HALF>) {
      iteration(std::integral_constant<int, 0>{}, std::false_type{}, it);
      iteration(std::integral_constant<int, 1>{}, std::false_type{}, it + 1);
      if constexpr (!HALF) {
        iteration(std::integral_constant<int, 2>{}, std::false_type{}, it + 2);
        iteration(std::integral_constant<int, 3>{}, std::false_type{}, it + 3);
      }
    }
    // (the row sums of the last plain step's P, which the masked MFMA phases leave out; from here on the sums are kept
    // lane by lane in l_run)
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      lacc[qb] = Mfma<F16>::run(ones, pk[qb], lacc[qb]);
      l_run[qb] = g == 0 ? lacc[qb][0] : 0.f;
    }
    // The rest, with masks.  (Guarded iterations, not early exits from the unrolled body: those cost the register
    // allocation of the whole kernel.)
    for (; it < nt; it += kRingOf<HALF>) {
      iteration(std::integral_constant<int, 0>{}, std::true_type{}, it);
      if (it + 1 < nt) iteration(std::integral_constant<int, 1>{}, std::true_type{}, it + 1);
      if constexpr (!HALF) {
        if (it + 2 < nt) iteration(std::integral_constant<int, 2>{}, std::true_type{}, it + 2);
        if (it + 3 < nt) iteration(std::integral_constant<int, 3>{}, std::true_type{}, it + 3);
      }
    }
    if (wave < 4) __builtin_amdgcn_s_barrier();
    // (a V tile loaded ahead is dropped; its loads must have landed before the registers are used for anything else)
    if (!DV) asm volatile("s_waitcnt vmcnt(0)" : "+v"(vst[0]), "+v"(vst[1]));
    // the product of the wave's last step is still owed
#pragma unroll
    for (int db = 0; db < 8; db++)
#pragma unroll
      for (int qb = 0; qb < 2; qb++) oacc[db][qb] = Mfma<F16>::run(va[db], pk[qb], oacc[db][qb]);
    // (the masked iterations, of which the last one always is, keep the row sums in l_run lane by lane; the epilogues
    // add the lanes of a column up)
#pragma unroll
    for (int qb = 0; qb < 2; qb++) m_run[qb] = -neg_m[qb];
  }

  // Old state of the rows for the epilogues that fold into one.  The two waves of a split pair both need it and one of
  // them writes it: there it is read before the barrier that the writes come after.
  float st_a[2] = {0.f, 0.f}, st_b[2] = {0.f, 0.f};
  auto read_state = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const int m = m_w0 + 16 * qb + qc;
      const int64_t tok = o_start + (m < q_len ? m : 0);
      if (MODE == 1) {  // (fetched into the wave's LDS at the start)
        st_a[qb] = *(const float*)(lds + kStateOff + wave * 1024 + qb * 256 + lane * 4);
        st_b[qb] = *(const float*)(lds + kStateOff + wave * 1024 + 512 + qb * 256 + lane * 4);
      }
      if (MODE == 2) st_a[qb] = p.lse[tok * p.hq + h] * kLog2e;
    }
  };

  if (SPLIT) {
    // The partials of the even and of the odd sub-tiles meet through LDS.  Each wave of a pair keeps four of the eight
    // d-blocks (the even side 0-3, the odd side 4-7), hands the other four to its partner with its maxima and sums, and
    // finishes its half of every row: merge and stores are shared by all eight waves.
    wait_vmem<0>();  // (loads requested ahead for tiles that were never used may still be writing the rings)
    __syncthreads();
    f32x4* xout = (f32x4*)lds + (wrow * 2 + kp) * (9 * 64) + lane;         // [8 blocks + (m, m, l, l)][lane]
    const f32x4* xin = (const f32x4*)lds + (wrow * 2 + (kp ^ 1)) * (9 * 64) + lane;
    auto give = [&](auto db0_tag) __attribute__((always_inline)) {
      constexpr int DB0 = decltype(db0_tag)::value;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++) xout[(i * 2 + qb) * 64] = oacc[DB0 + i][qb];
    };
    if (kp == 0) give(std::integral_constant<int, 4>{});
    else give(std::integral_constant<int, 0>{});
    xout[8 * 64] = f32x4{m_run[0], m_run[1], l_run[0], l_run[1]};
    if (MODE != 0) read_state();
    __syncthreads();
    const f32x4 ml = xin[8 * 64];
    float w_own[2], w_in[2];
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const float m1 = ml[qb], l1 = ml[2 + qb];
      const float M = fmaxf(m_run[qb], m1);
      w_own[qb] = exp2_diff(m_run[qb], M);  // 0 for a side that saw no key
      w_in[qb] = exp2_diff(m1, M);
      // (the even side's term first on both sides: the two waves hold the same sum to the last bit)
      l_run[qb] = kp == 0 ? __builtin_fmaf(l_run[qb], w_own[qb], l1 * w_in[qb]) : __builtin_fmaf(l1, w_in[qb], l_run[qb] * w_own[qb]);
      m_run[qb] = M;
    }
    auto take = [&](auto db0_tag) __attribute__((always_inline)) {
      constexpr int DB0 = decltype(db0_tag)::value;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++) oacc[DB0 + i][qb] = oacc[DB0 + i][qb] * w_own[qb] + xin[(i * 2 + qb) * 64] * w_in[qb];
    };
    if (kp == 0) take(std::integral_constant<int, 0>{});
    else take(std::integral_constant<int, 4>{});
  } else if (MODE != 0) {
    read_state();
  }

  // ---- epilogue: d-blocks DB0 .. DB0 + NDB - 1 of the wave's rows; the per-row scalars are written by the side that holds block 0 ----
  constexpr int NDB = SPLIT ? 4 : 8;
  auto finish = [&](auto db0_tag) __attribute__((always_inline)) {
    constexpr int DB0 = decltype(db0_tag)::value;
    if (MODE == 0) {
      // the step's partial from the empty state.  THROUGH (a launch of one or two rounds: every workgroup stores as the launch
      // ends, and what the L2s hold then is written back before the launch counts as done): the stores go through to
      // memory as they are issued, 1 x 2048 tokens 46.9 -> 45.9 us.  In launches of many rounds that costs the L2's
      // joining of a line's halves while other workgroups compute (32 x 1024 tokens 398 -> 417 us): plain stores there.
      auto write_partial = [&](auto through_tag) __attribute__((always_inline)) {
        constexpr bool THROUGH = decltype(through_tag)::value;
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
          const int m = m_w0 + 16 * qb + qc;
          const float l_tot = column_sum(l_run[qb]);
          if (m < q_len) {
            const int64_t tok = o_start + m;
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            float* orow = (float*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
            for (int i = 0; i < NDB; i++) {
              if (THROUGH) store16_through(orow + (DB0 + i) * 16 + 4 * g, oacc[DB0 + i][qb] * inv);
              else *(f32x4*)(orow + (DB0 + i) * 16 + 4 * g) = oacc[DB0 + i][qb] * inv;
            }
            if (g == 0 && DB0 == 0) p.lse[tok * p.hq + h] = l_tot > 0.f ? (m_run[qb] + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
          }
        }
      };
      if (p.store_through) write_partial(std::true_type{});
      else write_partial(std::false_type{});
    }
    if (MODE == 1) {
      // the reference's update of (o, m, l) (RING:171-188).  NB row blocks at a time: all reads of their old o are in
      // flight together
      auto fold_state = [&](auto nb_tag, int qb0) __attribute__((always_inline)) {
        constexpr int NB = decltype(nb_tag)::value;
        float l_tot[NB];
        u32x2 old[NB][NDB];
        bool in_range[NB];
        bool has_old = false;  // some row of these blocks carries an earlier step's result
#pragma unroll
        for (int i = 0; i < NB; i++) {
          const int qb = qb0 + i;
          l_tot[i] = column_sum(l_run[qb]);
          in_range[i] = m_w0 + 16 * qb + qc < q_len;
          has_old |= in_range[i] && st_a[qb] != -INFINITY && st_b[qb] != 0.f;
        }
        // (the same for every lane: a wave none of whose rows has an old result does not read o at all)
        const bool read_old = __builtin_amdgcn_ballot_w64(has_old) != 0;
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
          for (int d = 0; d < NDB; d++) old[i][d] = u32x2{0u, 0u};
        if (read_old) {
#pragma unroll
          for (int i = 0; i < NB; i++) {
            const int m = m_w0 + 16 * (qb0 + i) + qc;
            const int64_t tok = o_start + (in_range[i] ? m : 0);
            const uint16_t* orow = (const uint16_t*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
            for (int d = 0; d < NDB; d++) old[i][d] = *(const u32x2*)(orow + (DB0 + d) * 16 + 4 * g);
          }
        }
#pragma unroll
        for (int i = 0; i < NB; i++) {
          const int qb = qb0 + i;
          const float m_old = st_a[qb], l_old = st_b[qb];
          const float M = fmaxf(m_run[qb], m_old);
          if (!in_range[i] || M == -INFINITY || !(l_tot[i] > 0.f)) continue;
          const int64_t tok = o_start + m_w0 + 16 * qb + qc;
          const float w_old = l_old * exp2_diff(m_old, M);
          const float w_new = exp2_diff(m_run[qb], M);
          const float L = w_old + l_tot[i] * w_new;
          const float inv = 1.f / L;
          uint16_t* orow = (uint16_t*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
          for (int d = 0; d < NDB; d++) {
            const int db = DB0 + d;
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
            if (w_old != 0.f) {  // a row in its start state (m = -inf, l = 0) may hold anything in o
              unpack2<T>(old[i][d][0], o0, o1);
              unpack2<T>(old[i][d][1], o2, o3);
            }
            const float r0 = (o0 * w_old + oacc[db][qb][0] * w_new) * inv;
            const float r1 = (o1 * w_old + oacc[db][qb][1] * w_new) * inv;
            const float r2 = (o2 * w_old + oacc[db][qb][2] * w_new) * inv;
            const float r3 = (o3 * w_old + oacc[db][qb][3] * w_new) * inv;
            *(u32x2*)(orow + db * 16 + 4 * g) = u32x2{pack2<T>(r0, r1), pack2<T>(r2, r3)};
          }
          if (g == 0 && DB0 == 0) {  // every reader of the old state has it (read_state)
            p.m[tok * p.ml_st + (int64_t)h * p.ml_sh] = M;
            p.l[tok * p.ml_st + (int64_t)h * p.ml_sh] = L;
          }
        }
      };
      if (DV) {
        fold_state(std::integral_constant<int, 2>{}, 0);
      } else {
        fold_state(std::integral_constant<int, 1>{}, 0);
        fold_state(std::integral_constant<int, 1>{}, 1);
      }
    }
    if (MODE == 2) {
      // fold this step's partial into the running fp32 (O, LSE) of each row; a row that saw no key stays as it is.
      // NB row blocks at a time: all reads of their old O are in flight together
      auto fold = [&](auto nb_tag, int qb0) __attribute__((always_inline)) {
        constexpr int NB = decltype(nb_tag)::value;
        float l_tot[NB];
        f32x4 old[NB][NDB];
        bool live[NB];
#pragma unroll
        for (int i = 0; i < NB; i++) {
          const int qb = qb0 + i;
          const int m = m_w0 + 16 * qb + qc;
          l_tot[i] = column_sum(l_run[qb]);
          live[i] = m < q_len && l_tot[i] > 0.f;
          const int64_t tok = o_start + (m < q_len ? m : 0);
          const float* orow = (const float*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
          for (int d = 0; d < NDB; d++) old[i][d] = *(const f32x4*)(orow + (DB0 + d) * 16 + 4 * g);
        }
#pragma unroll
        for (int i = 0; i < NB; i++) {
          if (!live[i]) continue;
          const int qb = qb0 + i;
          const int64_t tok = o_start + m_w0 + 16 * qb + qc;
          const float a_old = st_a[qb];
          const float a_new = m_run[qb] + __builtin_amdgcn_logf(l_tot[i]);
          const float top = fmaxf(a_old, a_new);
          const float w_old = exp2_diff(a_old, top);
          const float w_new = __builtin_amdgcn_exp2f(a_new - top);
          const float W = w_old + w_new;
          const float c_old = w_old / W, c_new = w_new / (W * l_tot[i]);
          float* orow = (float*)p.o + tok * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
          for (int d = 0; d < NDB; d++) {
            // an empty row (lse = -inf) may hold anything: its old values are dropped, not multiplied by zero
            const f32x4 keep = w_old != 0.f ? old[i][d] : f32x4{0.f, 0.f, 0.f, 0.f};
            *(f32x4*)(orow + (DB0 + d) * 16 + 4 * g) = keep * c_old + oacc[DB0 + d][qb] * c_new;
          }
          if (g == 0 && DB0 == 0) p.lse[tok * p.hq + h] = (top + __builtin_amdgcn_logf(W)) * kLn2;  // (old value: read_state)
        }
      };
      if (DV) {
        fold(std::integral_constant<int, 2>{}, 0);
      } else {
        // the variant that converts V in registers has none to spare: one block at a time
        fold(std::integral_constant<int, 1>{}, 0);
        fold(std::integral_constant<int, 1>{}, 1);
      }
    }
  };
  if constexpr (SPLIT) {
    if (kp == 1) finish(std::integral_constant<int, 4>{});
    else finish(std::integral_constant<int, 0>{});
  } else {
    finish(std::integral_constant<int, 0>{});
  }
}

// log2 of the query heads of a KV head that share a workgroup: as many as the workgroup has 32-row groups and the group
// size divides by (a power of two), unless lsattn_set_tuning asked for one head per workgroup
static int pack_shift_for(const lsattn_prefill_args* a, bool split, const Tuning& tn) {
  if (tn.prefill_pack == LSATTN_PREFILL_PACK_OFF) return 0;
  const int64_t group = a->num_q_heads / a->num_kv_heads;
  int s = 0;
  while (s < (split ? 2 : 3) && group % (2 << s) == 0) s++;
  return s;
}

template <typename T, int MODE, bool DV, bool SPLIT, bool HALF = false>
static int launch_prefill_rows(const lsattn_prefill_args* a, bool tile_major, const Tuning& tn, hipStream_t st, bool fold = false) {
  constexpr int BMW = SPLIT || HALF ? BM / 2 : BM;
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
  p.o_start = a->o_b_start_loc;
  p.batch = a->batch;
  p.hq = a->num_q_heads;
  p.hkv = a->num_kv_heads;
  p.peers = a->sp_peers;
  p.d_peers = fast_div((uint32_t)a->sp_peers);
  p.pack_shift = pack_shift_for(a, SPLIT || HALF, tn);
  p.nz = (a->max_q_len + (BMW >> p.pack_shift) - 1) / (BMW >> p.pack_shift);
  {
    int g8 = 8;  // gcd(num_kv_heads, 8)
    while (a->num_kv_heads % g8) g8 >>= 1;
    p.slices = 8 / g8;
    p.kv_slots = a->num_kv_heads / g8;  // hkv * slices / 8
  }
  p.scale_log2 = a->sm_scale * kLog2e;
  p.o = a->o;
  p.o_st = a->o_stride_t;
  p.o_sh = a->o_stride_h;
  p.lse = a->lse;
  p.m = a->m;
  p.l = a->l;
  p.ml_st = a->ml_stride_t;
  p.ml_sh = a->ml_stride_h;
  p.heads_per_kv = a->num_q_heads / a->num_kv_heads;
  const int group = p.heads_per_kv >> p.pack_shift;  // workgroups side by side over the heads of a KV head
  p.group = group;
  p.units_per_slice = (int32_t)(((int64_t)group * p.nz + p.slices - 1) / p.slices);
  p.d_group = fast_div((uint32_t)group);
  p.d_slices = fast_div((uint32_t)p.slices);
  p.kv_cuts = a->kv_cuts > 1 ? a->kv_cuts : 1;
  p.kv_cut_len = a->kv_cuts > 1 ? a->kv_cut_len : 0x7fffffff;
  p.o_cut_rows = a->kv_cuts > 1 ? a->o_cut_rows : 0;
  p.d_cuts = fast_div((uint32_t)p.kv_cuts);
  p.tile_major = tile_major || SPLIT || HALF;
  p.n_first = p.tile_major ? p.kv_slots : p.units_per_slice;
  p.n_second = p.tile_major ? p.units_per_slice : p.kv_slots;
  p.d_first = fast_div((uint32_t)p.n_first);
  p.d_second = fast_div((uint32_t)p.n_second);
  const int64_t wgs = (int64_t)8 * p.units_per_slice * p.kv_slots * a->batch * p.kv_cuts;
  if (wgs > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  p.fold_from = p.fold_sum = 0;
  p.listed = 0;
  p.rows_shift = (SPLIT || HALF ? 7 : 8) - p.pack_shift;
  // A grid of the units that can exist instead of one sized by the longest request (see the kernel), when the caller
  // bounds the rows of all requests together and that grid is at most half of the other: a skewed batch.  (One KV head
  // or slot per XCD index only, and no cuts along the keys.)
  int64_t wgs_launch = wgs;
  if (a->total_q_rows > 0 && p.slices == 1 && p.kv_cuts == 1 && a->batch <= kListedMaxBatch && wgs >= kListedFromWorkgroups) {
    const int64_t rows_wg = BMW >> p.pack_shift;
    const int64_t units_max = (int64_t)group * ((a->total_q_rows + rows_wg - 1) / rows_wg + a->batch);
    const int64_t wgs_listed = 8 * p.kv_slots * units_max;
    if (wgs_listed * 2 <= wgs) {
      p.listed = 1;
      p.n_first = p.kv_slots;
      p.d_first = fast_div((uint32_t)p.n_first);
      wgs_launch = wgs_listed;
    }
  }
  if (HALF && fold && wgs > 2 * kCUs / 2 && wgs <= 2 * kCUs) {
    p.fold_from = (int32_t)(kCUs / 8);
    p.fold_sum = p.fold_from + (int32_t)(wgs / 8) - 1;
  }
  // (a round: two four-wave workgroups per CU, one of the others.  Two rounds still gain: 16 x 256 tokens 38.0 -> 36.8 us,
  // 1 x 4096 129.0 -> 127.7; six rounds lose 1-3 %, sixteen 5 %.)
  p.store_through = MODE == 0 && wgs_launch <= 2 * (HALF ? 2 * kCUs : kCUs);
  LSATTN_LAUNCH_KERNEL((prefill_kernel<T, MODE, DV, SPLIT, HALF>), dim3((unsigned)wgs_launch), dim3(HALF ? NWAVE * 32 : NWAVE * 64), 0, st, p);
  return check_launch();
}

// Rows per workgroup and the order of the grid, both from the launch's size in 256-row workgroups (the host knows the
// batch, the head count and the longest query chunk, not the requests' lengths).
// 256 rows is the efficient shape (each staged K/V tile serves twice the rows at 1.57 us per 64 keys against 0.86 us
// for 128 rows, and a workgroup's fixed start and end cost comes once per 256 rows).  128 rows (the split variant) when
// 256-row workgroups cannot fill the chip: at most half a round of them, or at most one round whose heaviest workgroup
// walks five or more tiles of rows under the causal mask (its duration is the launch's; two rounds of 128-row
// workgroups, heaviest first, end sooner).  Above one round the 256-row shape measured faster on every shape tried
// (16 to 64 heads, 1 to 32 requests of 256 to 16384 tokens), provided the grid is in the order below.
// Grid order: launches under kTileMajorBelowWorkgroups run the heaviest tiles of all KV heads first; larger ones one KV
// head at a time per XCD (the order that keeps K/V in the L2s when every workgroup walks all keys).  With 32 KV heads
// and 4096 tokens the head-by-head order leaves a CU with tiles 9 and 16 of 16 and takes 160 us where the other takes 128.
// lsattn_set_tuning overrides both choices (tuning and tests).  The size counts workgroups as they are launched: with the query heads of a KV head side by side
// (pack_shift_for) a workgroup covers 256 >> pack_shift positions of 1 << pack_shift heads.
template <typename T, int MODE, bool DV> static int launch_prefill(const lsattn_prefill_args* a, hipStream_t st) {
  const Tuning tn = tuning();
  const int64_t nz256 = (a->max_q_len + BM - 1) / BM;
  const int ps = pack_shift_for(a, false, tn);  // (the workgroups of several heads are shorter: less padding past a short chunk)
  const int64_t cuts = a->kv_cuts > 1 ? a->kv_cuts : 1;
  // query tiles of `rows` positions over the whole batch: the longest request's times the batch, or fewer if the caller
  // bounds the rows of all requests together
  auto tiles_of = [&](int64_t rows) {
    const int64_t by_longest = a->batch * ((a->max_q_len + rows - 1) / rows);
    const int64_t by_total = a->total_q_rows > 0 ? (a->total_q_rows + rows - 1) / rows + a->batch : by_longest;
    return by_total < by_longest ? by_total : by_longest;
  };
  const int64_t wgs256 = cuts * (a->num_q_heads >> ps) * tiles_of(BM >> ps);
  bool tile_major = wgs256 < kTileMajorBelowWorkgroups;
  if (tn.prefill_order == LSATTN_PREFILL_ORDER_TILE) tile_major = true;
  if (tn.prefill_order == LSATTN_PREFILL_ORDER_HEAD) tile_major = false;
  if constexpr (!DV) {
    return launch_prefill_rows<T, MODE, false, false>(a, tile_major, tn, st);
  } else {
    bool split = wgs256 <= kCUs / 2 || (wgs256 <= kCUs && nz256 >= 5);
    // Short chunks that a 256-row workgroup pads much further than a 128-row one (100 rows of one head: 256 against 128): the
    // 128-row shapes walk the same tiles for at most four fifths of the rows (100 rows x 131072 keys in 15 cuts, MHA 32:
    // 507 -> 376 us).  Per row and tile they are 5 to 10 % behind the 256-row shape, hence the margin.
    {
      // (query positions the longest chunk is padded to; the heads side by side in a workgroup cancel out)
      const int64_t padded256 = ((a->max_q_len + (BM >> ps) - 1) / (BM >> ps)) * (BM >> ps);
      const int ph0 = pack_shift_for(a, true, tn);
      const int64_t padded128 = ((a->max_q_len + (BM / 2 >> ph0) - 1) / (BM / 2 >> ph0)) * (BM / 2 >> ph0);
      if (padded128 * 5 <= padded256 * 4) split = true;
    }
    // The four-wave shape (two workgroups per CU) for chunks of up to 1024 rows (1536 with one head per workgroup),
    // whose workgroups walk a few tiles each and spend as long starting and ending as working, from three workgroups
    // per CU on: 3 to 17 % shorter launches on batches of 4 to 32 requests of 128 to 1536 tokens.  Smaller launches keep
    // the shapes above: with at most a pair of these workgroups per CU a launch of short chunks would gain as much, but
    // one of short chunks against long K/V (which the host cannot tell apart) would run on half the CUs.  Not for
    // launches that write their rows elsewhere either (the step cut along the keys: few, long workgroups).
    const int ph = pack_shift_for(a, true, tn);
    const int64_t wgs128 = cuts * (a->num_q_heads >> ph) * tiles_of(BM / 2 >> ph);
    bool half = a->max_q_len <= (ph ? 1024 : 1536) && !a->o_b_start_loc && a->kv_cuts <= 1 && wgs128 >= 3 * kCUs;
    if (tn.prefill_rows == LSATTN_PREFILL_ROWS_128) split = true, half = false;
    if (tn.prefill_rows == LSATTN_PREFILL_ROWS_256) split = false, half = false;
    if (tn.prefill_rows == LSATTN_PREFILL_ROWS_HALF) half = true;
    // One request whose four-wave workgroups all fit the chip at once, more than one and at most two per CU (a single
    // sequence of up to 2048 tokens: 32 heads x sixteen 128-row tiles): the four-wave shape with the second half of the
    // grid running backwards (see the kernel), each CU one heavy and one light workgroup side by side, instead of the
    // split shape's two rounds.  Longer chunks keep the rules above (the pairs' work is then long against what a
    // workgroup costs besides its tiles, and the shape's rings of two tiles are the slower ones per tile).
    // (measured, one sequence, MHA 32: 2048 tokens = 512 workgroups 45.7 us against 47.1 split and 47.3 unfolded; 1792 tokens
    // = 448 39.6 against 40.5; 1536 = 384 34.2 against 33.5 and 1280 = 320 29.7 against 27.4: the fold pays from seven
    // eighths of two workgroups per CU on, below that the split shape's two rounds do)
    const bool fold = a->batch == 1 && cuts == 1 && !a->o_b_start_loc && a->max_q_len <= 2048 && wgs128 * 8 >= 7 * 2 * kCUs &&
                      wgs128 <= 2 * kCUs && tn.prefill_rows == 0;
    if (fold) return launch_prefill_rows<T, MODE, true, false, true>(a, true, tn, st, true);
    if (half) return launch_prefill_rows<T, MODE, true, false, true>(a, true, tn, st);
    return split ? launch_prefill_rows<T, MODE, true, true>(a, true, tn, st) : launch_prefill_rows<T, MODE, true, false>(a, tile_major, tn, st);
  }
}

static int validate(const lsattn_prefill_args* a, int mode) {
  if (!a || !a->q || !a->k || !a->v || !a->o) return LSATTN_ERR_INVALID_ARG;
  if (!a->q_b_start_loc || !a->q_b_seq_len || !a->q_first_token_global_idx || !a->kv_b_start_loc || !a->kv_b_seq_len ||
      !a->kv_first_token_global_idx)
    return LSATTN_ERR_INVALID_ARG;
  if (a->batch < 0 || a->num_q_heads <= 0 || a->num_kv_heads <= 0 || a->sp_peers < 1 || a->max_q_len < 0 || a->total_q_rows < 0)
    return LSATTN_ERR_INVALID_ARG;
  if (a->num_q_heads % a->num_kv_heads) return LSATTN_ERR_INVALID_ARG;
  if (a->head_dim != 128 && a->head_dim != 64 && a->head_dim != 32 && a->head_dim != 16) return LSATTN_ERR_UNSUPPORTED;
  if (a->head_dim != 128 && a->kv_cuts > 1) return LSATTN_ERR_UNSUPPORTED;  // (the cut along the keys is the 128-wide kernel's)
  if (a->dtype != LSATTN_F16 && a->dtype != LSATTN_BF16) return LSATTN_ERR_UNSUPPORTED;
  if (a->v_is_f16 != 0 && (a->v_is_f16 != 1 || a->dtype != LSATTN_BF16)) return LSATTN_ERR_INVALID_ARG;
  // the chunk cut along the keys: a multiple of the 64-key tile per cut, the cuts' outputs apart (fp32 partials only),
  // and key positions that stay within 31 bits
  if (a->kv_cuts < 0 || a->kv_cuts > LSATTN_MAX_KV_CUTS) return LSATTN_ERR_INVALID_ARG;
  if (a->kv_cuts > 1 && (mode != 0 || a->kv_cut_len < 64 || a->kv_cut_len % 64 || a->o_cut_rows <= 0 ||
                         (int64_t)a->kv_cut_len * a->kv_cuts > 0x7fffffff))
    return LSATTN_ERR_INVALID_ARG;
  // 16-byte operand loads / 8- or 16-byte output stores
  if (a->q_stride_t % 8 || a->q_stride_h % 8 || a->k_stride_t % 8 || a->k_stride_h % 8 || a->v_stride_t % 8 || a->v_stride_h % 8)
    return LSATTN_ERR_INVALID_ARG;
  if (a->o_stride_t % 4 || a->o_stride_h % 4) return LSATTN_ERR_INVALID_ARG;
  // a lane addresses the 64 rows of a K/V tile with a 32-bit byte offset from the tile's first row
  if (a->k_stride_t <= 0 || a->v_stride_t <= 0 || a->k_stride_t > (1 << 24) || a->v_stride_t > (1 << 24)) return LSATTN_ERR_INVALID_ARG;
  if (((uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o) & 15) return LSATTN_ERR_INVALID_ARG;
  if (mode == 0 || mode == 2) {
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
  if (a->head_dim != 128) return launch_prefill_small(a, 0, (hipStream_t)stream);
  if (a->dtype == LSATTN_F16) return launch_prefill<F16, 0, true>(a, (hipStream_t)stream);
  return a->v_is_f16 ? launch_prefill<BF16, 0, true>(a, (hipStream_t)stream) : launch_prefill<BF16, 0, false>(a, (hipStream_t)stream);
}

extern "C" int lsattn_prefill_step_merge(const lsattn_prefill_args* a, void* stream) {
  const int rc = validate(a, 1);
  if (rc != LSATTN_OK) return rc;
  if (a->batch == 0 || a->max_q_len == 0) return LSATTN_OK;
  if (a->head_dim != 128) return launch_prefill_small(a, 1, (hipStream_t)stream);
  if (a->dtype == LSATTN_F16) return launch_prefill<F16, 1, true>(a, (hipStream_t)stream);
  return a->v_is_f16 ? launch_prefill<BF16, 1, true>(a, (hipStream_t)stream) : launch_prefill<BF16, 1, false>(a, (hipStream_t)stream);
}

extern "C" int lsattn_prefill_step_accumulate(const lsattn_prefill_args* a, void* stream) {
  const int rc = validate(a, 2);
  if (rc != LSATTN_OK) return rc;
  if (a->batch == 0 || a->max_q_len == 0) return LSATTN_OK;
  if (a->head_dim != 128) return launch_prefill_small(a, 2, (hipStream_t)stream);
  if (a->dtype == LSATTN_F16) return launch_prefill<F16, 2, true>(a, (hipStream_t)stream);
  return a->v_is_f16 ? launch_prefill<BF16, 2, true>(a, (hipStream_t)stream) : launch_prefill<BF16, 2, false>(a, (hipStream_t)stream);
}
