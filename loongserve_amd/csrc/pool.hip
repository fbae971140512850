// Slot allocator of the KV pool for gfx950: the device-side searches and reference counting that the reference
// does with torch.nonzero over the whole pool on every call (loongserve/common/longserve_mem_manager.py:32-88).
//   take the first `need` free slots, in ascending order          (alloc, :37-40)
//   find the first run of `need` consecutive free slots           (alloc_contiguous, :50-55)
//   add / drop one reference on a list of slots and count          (add_refs :73-79, decrease_refs :82-88)
// `mem_state` is int32 per slot, 0 = free.  All of it is integer work on a few MB, bound by launch latency and
// by one pass over the state array; three short launches replace the reference's nonzero / slice / compare chains.
#include "common.hip.h"

namespace lsattn {

constexpr int kPoolThreads = 256;
constexpr int kPoolPieces = 4;                                 // 16-byte pieces per thread
constexpr int kPoolBlockSlots = kPoolThreads * 4 * kPoolPieces;  // 4096 slots per workgroup
constexpr int kPoolWaves = kPoolThreads / 64;

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Slots of one workgroup, coalesced: piece j of thread t covers slots base + 1024 j + 4 t .. + 3; the scan order of
// the (piece, thread) pairs is j-major, which is ascending slot order.  Slots past `size` read as in use.
struct PoolTile {
  int64_t base;
  i32x4 s[kPoolPieces];
  __device__ __forceinline__ void load(const int32_t* __restrict__ state, int64_t size) {
    base = (int64_t)blockIdx.x * kPoolBlockSlots;
#pragma unroll
    for (int j = 0; j < kPoolPieces; j++) {
      const int64_t p = base + j * (kPoolThreads * 4) + threadIdx.x * 4;
      if (p + 3 < size) {
        s[j] = *(const i32x4*)(state + p);
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) s[j][e] = p + e < size ? state[p + e] : 1;
      }
    }
  }
  __device__ __forceinline__ int64_t pos(int j, int e) const { return base + j * (kPoolThreads * 4) + threadIdx.x * 4 + e; }
};

__device__ __forceinline__ int wave_incl_sum(int v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(v, d);
    if (lane >= d) v += o;
  }
  return v;
}
__device__ __forceinline__ int64_t wave_incl_max(int64_t v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int64_t o = __shfl_up(v, d);
    if (lane >= d) v = o > v ? o : v;
  }
  return v;
}

// ---------------------------------------------------------------------------------------------------
// Pass 1: per workgroup of 4096 slots, the number of free slots and the position of the last slot in use (-1: none).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kPoolThreads) void pool_summarise_kernel(const int32_t* __restrict__ state, int64_t size,
                                                                      int32_t* __restrict__ blk_free,
                                                                      int64_t* __restrict__ blk_last_used) {
  __shared__ int sh_cnt[kPoolWaves];
  __shared__ int64_t sh_last[kPoolWaves];
  PoolTile t;
  t.load(state, size);
  int cnt = 0;
  int64_t last = -1;
#pragma unroll
  for (int j = 0; j < kPoolPieces; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      cnt += t.s[j][e] == 0;
      if (t.s[j][e] != 0 && t.pos(j, e) < size) last = t.pos(j, e);  // ascending within the thread's pieces
    }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    cnt += __shfl_xor(cnt, d);
    const int64_t o = __shfl_xor(last, d);
    last = o > last ? o : last;
  }
  if ((threadIdx.x & 63) == 0) {
    sh_cnt[threadIdx.x >> 6] = cnt;
    sh_last[threadIdx.x >> 6] = last;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int c = 0;
    int64_t l = -1;
    for (int w = 0; w < kPoolWaves; w++) {
      c += sh_cnt[w];
      l = sh_last[w] > l ? sh_last[w] : l;
    }
    blk_free[blockIdx.x] = c;
    blk_last_used[blockIdx.x] = l;
  }
}

// ---------------------------------------------------------------------------------------------------
// Pass 2 (one workgroup): exclusive prefix sum of the free counts and exclusive prefix maximum of the last-used
// positions over the workgroups of pass 1.  cells[0] = total free; *first_fit (when given) is preset to -1 = "no run".
// When fewer than `need` slots are free, out_index[total .. need) is filled with -1 so the result is defined.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void pool_scan_summaries_kernel(const int32_t* __restrict__ blk_free,
                                                                   const int64_t* __restrict__ blk_last_used, int64_t nb,
                                                                   int64_t* __restrict__ free_before,
                                                                   int64_t* __restrict__ last_used_before,
                                                                   int64_t* __restrict__ cells, int64_t need,
                                                                   int64_t* __restrict__ out_index,
                                                                   int64_t* __restrict__ first_fit) {
  __shared__ int64_t sh_sum[1024];
  __shared__ int64_t sh_max[1024];
  const int64_t per = (nb + 1023) / 1024;
  const int64_t b0 = (int64_t)threadIdx.x * per, b1 = b0 + per < nb ? b0 + per : nb;
  int64_t sum = 0, mx = -1;
  for (int64_t b = b0; b < b1; b++) {
    sum += blk_free[b];
    mx = blk_last_used[b] > mx ? blk_last_used[b] : mx;
  }
  sh_sum[threadIdx.x] = sum;
  sh_max[threadIdx.x] = mx;
  __syncthreads();
  // Hillis-Steele over the 1024 thread totals
  for (int d = 1; d < 1024; d <<= 1) {
    int64_t s = 0, m = -1;
    if ((int)threadIdx.x >= d) {
      s = sh_sum[threadIdx.x - d];
      m = sh_max[threadIdx.x - d];
    }
    __syncthreads();
    sh_sum[threadIdx.x] += s;
    sh_max[threadIdx.x] = m > sh_max[threadIdx.x] ? m : sh_max[threadIdx.x];
    __syncthreads();
  }
  int64_t run_sum = threadIdx.x ? sh_sum[threadIdx.x - 1] : 0;
  int64_t run_max = threadIdx.x ? sh_max[threadIdx.x - 1] : -1;
  for (int64_t b = b0; b < b1; b++) {
    free_before[b] = run_sum;
    last_used_before[b] = run_max;
    run_sum += blk_free[b];
    run_max = blk_last_used[b] > run_max ? blk_last_used[b] : run_max;
  }
  const int64_t total = sh_sum[1023];
  if (threadIdx.x == 0) {
    cells[0] = total;
    if (first_fit) *first_fit = -1;
  }
  if (out_index)
    for (int64_t i = total + threadIdx.x; i < need; i += 1024) out_index[i] = -1;
}

// ---------------------------------------------------------------------------------------------------
// Pass 3 of alloc: the free slot with rank r < need (ranks count free slots in ascending slot order) is written to
// out_index[r] and marked in use.  Workgroups whose first rank is already >= need leave at once.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kPoolThreads) void pool_take_kernel(int32_t* __restrict__ state, int64_t size,
                                                                 const int64_t* __restrict__ free_before, int64_t need,
                                                                 int64_t* __restrict__ out_index) {
  __shared__ int sh[kPoolPieces][kPoolWaves];
  const int64_t first_rank = free_before[blockIdx.x];
  if (first_rank >= need) return;
  PoolTile t;
  t.load(state, size);
  const int wave = threadIdx.x >> 6;
  int incl[kPoolPieces], mine[kPoolPieces];
#pragma unroll
  for (int j = 0; j < kPoolPieces; j++) {
    mine[j] = (t.s[j][0] == 0) + (t.s[j][1] == 0) + (t.s[j][2] == 0) + (t.s[j][3] == 0);
    incl[j] = wave_incl_sum(mine[j]);
    if ((threadIdx.x & 63) == 63) sh[j][wave] = incl[j];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kPoolPieces; j++) {
    int before = 0;  // free slots of the (piece, wave) pairs that come earlier in slot order
    for (int jj = 0; jj < kPoolPieces; jj++)
      for (int w = 0; w < kPoolWaves; w++)
        if (jj < j || (jj == j && w < wave)) before += sh[jj][w];
    int64_t rank = first_rank + before + incl[j] - mine[j];
    if (rank >= need) continue;
    i32x4 ns = t.s[j];
    bool any = false;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if (t.s[j][e] == 0 && rank < need) {
        out_index[rank++] = t.pos(j, e);
        ns[e] = 1;
        any = true;
      }
    }
    if (any) {
      const int64_t p = t.pos(j, 0);
      if (p + 3 < size) {
        *(i32x4*)(state + p) = ns;
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (p + e < size) state[p + e] = ns[e];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// Pass 3 of alloc_contiguous: with u(p) = position of the last slot in use at or before p, a run of free slots
// reaches length `need` exactly at the one p with p - u(p) == need, and starts at p - need + 1.  The smallest
// such start over the pool is the reference's can_use_index[...][0] (longserve_mem_manager.py:52-55).  The minimum is
// taken on the unsigned value, so the preset -1 stands for "none" and loses to every real start.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kPoolThreads) void pool_first_fit_kernel(const int32_t* __restrict__ state, int64_t size,
                                                                      const int64_t* __restrict__ last_used_before,
                                                                      int64_t need, int64_t* __restrict__ first_fit) {
  __shared__ int64_t sh[kPoolPieces][kPoolWaves];
  PoolTile t;
  t.load(state, size);
  const int wave = threadIdx.x >> 6;
  int64_t own[kPoolPieces], incl[kPoolPieces];
#pragma unroll
  for (int j = 0; j < kPoolPieces; j++) {
    own[j] = -1;
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (t.s[j][e] != 0) own[j] = t.pos(j, e);  // slots past the end count as in use: runs stop there
    incl[j] = wave_incl_max(own[j]);
    if ((threadIdx.x & 63) == 63) sh[j][wave] = incl[j];
  }
  __syncthreads();
  int64_t best = INT64_MAX;
#pragma unroll
  for (int j = 0; j < kPoolPieces; j++) {
    int64_t u = last_used_before[blockIdx.x];
    for (int jj = 0; jj < kPoolPieces; jj++)
      for (int w = 0; w < kPoolWaves; w++)
        if (jj < j || (jj == j && w < wave)) u = sh[jj][w] > u ? sh[jj][w] : u;
    const int64_t prev = __shfl_up(incl[j], 1);  // lanes before this one in the wave
    if ((threadIdx.x & 63) != 0) u = prev > u ? prev : u;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int64_t p = t.pos(j, e);
      if (t.s[j][e] != 0) {
        u = p;
      } else if (p - u == need && p - need + 1 < best) {
        best = p - need + 1;
      }
    }
  }
  if (best != INT64_MAX) atomicMin((unsigned long long*)first_fit, (unsigned long long)best);
}

// ---------------------------------------------------------------------------------------------------
// Reference counting on a list of slots.  torch's `mem_state[index] += d` gathers, adds and writes back, so a slot
// named k times still changes by d once; both kernels keep that: the first reads every old value, the second
// writes old + d.  counted[0] = entries whose slot is non-zero before (+1: has_used_tokens, :75) or after
// (-1: used_tokens, :85) the update; counted[1] = entries outside the pool (skipped).  Negative entries wrap
// once, as in torch indexing.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pool_refs_gather_kernel(const int32_t* __restrict__ state, int64_t size,
                                                               const int64_t* __restrict__ index, int64_t n, int delta,
                                                               int32_t* __restrict__ old_state, int64_t* __restrict__ blk_counts) {
  __shared__ int sh[2][4];
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int used = 0, bad = 0;
  if (i < n) {
    int64_t s = index[i];
    if (s < 0) s += size;
    if (s < 0 || s >= size) {
      bad = 1;
    } else {
      const int32_t o = state[s];
      old_state[i] = o;
      used = (delta > 0 ? o : o + delta) != 0;
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    used += __shfl_xor(used, d);
    bad += __shfl_xor(bad, d);
  }
  if ((threadIdx.x & 63) == 0) {
    sh[0][threadIdx.x >> 6] = used;
    sh[1][threadIdx.x >> 6] = bad;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    blk_counts[2 * blockIdx.x] = sh[0][0] + sh[0][1] + sh[0][2] + sh[0][3];
    blk_counts[2 * blockIdx.x + 1] = sh[1][0] + sh[1][1] + sh[1][2] + sh[1][3];
  }
}

__global__ __launch_bounds__(256) void pool_refs_apply_kernel(int32_t* __restrict__ state, int64_t size,
                                                              const int64_t* __restrict__ index, int64_t n, int delta,
                                                              const int32_t* __restrict__ old_state,
                                                              const int64_t* __restrict__ blk_counts, int64_t nblk,
                                                              int64_t* __restrict__ counted) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    int64_t s = index[i];
    if (s < 0) s += size;
    if (s >= 0 && s < size) state[s] = old_state[i] + delta;
  }
  if (blockIdx.x == 0) {  // the per-workgroup counts are complete: the gather launch precedes this one on the stream
    __shared__ int64_t sh[2][4];
    int64_t used = 0, bad = 0;
    for (int64_t b = threadIdx.x; b < nblk; b += 256) {
      used += blk_counts[2 * b];
      bad += blk_counts[2 * b + 1];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      used += __shfl_xor(used, d);
      bad += __shfl_xor(bad, d);
    }
    if ((threadIdx.x & 63) == 0) {
      sh[0][threadIdx.x >> 6] = used;
      sh[1][threadIdx.x >> 6] = bad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      counted[0] = sh[0][0] + sh[0][1] + sh[0][2] + sh[0][3];
      counted[1] = sh[1][0] + sh[1][1] + sh[1][2] + sh[1][3];
    }
  }
}

// Workspace layout of the searches: int64 cells[2] (cells[0] = free slots in the pool at the time of the call) | int64 free_before[nb] | int64 last_used_before[nb] |
// int64 blk_last_used[nb] | int32 blk_free[nb]
struct PoolWorkspace {
  int64_t nb;
  int64_t *cells, *free_before, *last_used_before, *blk_last_used;
  int32_t* blk_free;
};
inline int64_t pool_blocks(int64_t size) { return (size + kPoolBlockSlots - 1) / kPoolBlockSlots; }
inline size_t pool_search_bytes(int64_t size) { return (size_t)(16 + pool_blocks(size) * 28 + 15) & ~(size_t)15; }
inline PoolWorkspace pool_carve(void* ws, int64_t size) {
  PoolWorkspace w;
  w.nb = pool_blocks(size);
  w.cells = (int64_t*)ws;
  w.free_before = w.cells + 2;
  w.last_used_before = w.free_before + w.nb;
  w.blk_last_used = w.last_used_before + w.nb;
  w.blk_free = (int32_t*)(w.blk_last_used + w.nb);
  return w;
}
inline int64_t refs_blocks(int64_t n) { return (n + 255) / 256; }

}  // namespace lsattn

using namespace lsattn;

extern "C" size_t lsattn_pool_search_workspace_bytes(int64_t pool_size) { return pool_size > 0 ? pool_search_bytes(pool_size) : 0; }

extern "C" size_t lsattn_pool_refs_workspace_bytes(int64_t n) {
  return n > 0 ? (size_t)(refs_blocks(n) * 16 + ((n * 4 + 15) & ~(int64_t)15)) : 0;
}

static int pool_search_checks(const void* mem_state, int64_t size, int64_t need, const void* ws, size_t ws_bytes) {
  if (!mem_state || !ws || size <= 0 || need < 0) return LSATTN_ERR_INVALID_ARG;
  if (((uintptr_t)mem_state & 15) || ((uintptr_t)ws & 15)) return LSATTN_ERR_INVALID_ARG;
  if (ws_bytes < pool_search_bytes(size)) return LSATTN_ERR_WORKSPACE;
  if (pool_blocks(size) > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  return LSATTN_OK;
}

extern "C" int lsattn_pool_alloc(int32_t* mem_state, int64_t pool_size, int64_t need, int64_t* out_index, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  const int rc = pool_search_checks(mem_state, pool_size, need, workspace, workspace_bytes);
  if (rc != LSATTN_OK) return rc;
  if (need > 0 && !out_index) return LSATTN_ERR_INVALID_ARG;
  hipStream_t st = (hipStream_t)stream;
  const PoolWorkspace w = pool_carve(workspace, pool_size);
  LSATTN_LAUNCH_KERNEL(pool_summarise_kernel, dim3((unsigned)w.nb), dim3(kPoolThreads), 0, st, mem_state, pool_size, w.blk_free,
                     w.blk_last_used);
  LSATTN_LAUNCH_KERNEL(pool_scan_summaries_kernel, dim3(1), dim3(1024), 0, st, w.blk_free, w.blk_last_used, w.nb, w.free_before,
                     w.last_used_before, w.cells, need, out_index, (int64_t*)nullptr);
  if (need > 0)
    LSATTN_LAUNCH_KERNEL(pool_take_kernel, dim3((unsigned)w.nb), dim3(kPoolThreads), 0, st, mem_state, pool_size, w.free_before,
                       need, out_index);
  return check_launch();
}

extern "C" int lsattn_pool_find_contiguous(const int32_t* mem_state, int64_t pool_size, int64_t need, int64_t* out_start,
                                           void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = pool_search_checks(mem_state, pool_size, need, workspace, workspace_bytes);
  if (rc != LSATTN_OK) return rc;
  if (!out_start || need <= 0) return LSATTN_ERR_INVALID_ARG;
  hipStream_t st = (hipStream_t)stream;
  const PoolWorkspace w = pool_carve(workspace, pool_size);
  LSATTN_LAUNCH_KERNEL(pool_summarise_kernel, dim3((unsigned)w.nb), dim3(kPoolThreads), 0, st, mem_state, pool_size, w.blk_free,
                     w.blk_last_used);
  LSATTN_LAUNCH_KERNEL(pool_scan_summaries_kernel, dim3(1), dim3(1024), 0, st, w.blk_free, w.blk_last_used, w.nb, w.free_before,
                     w.last_used_before, w.cells, (int64_t)0, (int64_t*)nullptr, out_start);
  LSATTN_LAUNCH_KERNEL(pool_first_fit_kernel, dim3((unsigned)w.nb), dim3(kPoolThreads), 0, st, mem_state, pool_size,
                     w.last_used_before, need, out_start);
  return check_launch();
}

extern "C" int lsattn_pool_update_refs(int32_t* mem_state, int64_t pool_size, const int64_t* index, int64_t n, int delta,
                                       int64_t* counted, void* workspace, size_t workspace_bytes, void* stream) {
  if (!mem_state || pool_size <= 0 || n < 0 || (delta != 1 && delta != -1) || !counted) return LSATTN_ERR_INVALID_ARG;
  if (n > 0 && (!index || !workspace)) return LSATTN_ERR_INVALID_ARG;
  if ((uintptr_t)workspace & 15) return LSATTN_ERR_INVALID_ARG;
  if (workspace_bytes < lsattn_pool_refs_workspace_bytes(n)) return LSATTN_ERR_WORKSPACE;
  const int64_t nblk = refs_blocks(n);
  if (nblk > 0x7fffffff) return LSATTN_ERR_INVALID_ARG;
  hipStream_t st = (hipStream_t)stream;
  int64_t* blk_counts = (int64_t*)workspace;
  int32_t* old_state = (int32_t*)(blk_counts + 2 * nblk);
  if (n > 0)
    LSATTN_LAUNCH_KERNEL(pool_refs_gather_kernel, dim3((unsigned)nblk), dim3(256), 0, st, mem_state, pool_size, index, n, delta,
                       old_state, blk_counts);
  // with n == 0 one workgroup still runs, to write counted = {0, 0}
  LSATTN_LAUNCH_KERNEL(pool_refs_apply_kernel, dim3((unsigned)(nblk > 0 ? nblk : 1)), dim3(256), 0, st, mem_state, pool_size, index,
                     n, delta, old_state, blk_counts, nblk, counted);
  return check_launch();
}
