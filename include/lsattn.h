/*
 * lsattn.h -- C ABI of the MI355X (gfx950) attention hot path.
 *
 * Plain C: device pointers, sizes and element strides only; no torch, no HIP types
 * (a hipStream_t is passed as `void*`; NULL means the default stream).  Every entry point
 *   - launches asynchronously on the given stream and returns without a host sync,
 *   - allocates nothing and keeps no pointer after it returns (the caller owns every
 *     buffer, scratch included); the only state the library keeps between calls is the
 *     block of launch choices that lsattn_set_tuning stores (and the scratch array of
 *     lsattn_decode_attention_static),
 *   - returns LSATTN_OK or a negative LSATTN_ERR_* code and never aborts or throws.
 *
 * Citations name the reference interface each entry point replaces, relative to the
 * reference tree:
 *   RING  = loongserve/models/llama/triton_kernel/ring_context_flashattention_nopad.py
 *   S1CU/S1H = longserve_cuda_kernels/src/flash_decoding_stage1.{cu,h}
 *   S2CU/S2H = longserve_cuda_kernels/src/flash_decoding_stage2.{cu,h}
 *   ENTRY = longserve_cuda_kernels/src/entrypoints.cpp
 */
#ifndef LSATTN_H
#define LSATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LSATTN_OK 0
#define LSATTN_ERR_INVALID_ARG (-1) /* null pointer, negative size, bad stride            */
#define LSATTN_ERR_UNSUPPORTED (-2) /* head_dim / dtype / head ratio the kernels lack     */
#define LSATTN_ERR_LAUNCH (-3)      /* hipGetLastError() after the launch was not success */
#define LSATTN_ERR_WORKSPACE (-4)   /* the workspace passed in is smaller than required    */

/* element types of q/k/v and of `o` outputs */
#define LSATTN_F16 0
#define LSATTN_BF16 1
#define LSATTN_F32 2

#define LSATTN_MAX_PARTS 16
#define LSATTN_MAX_KV_CUTS 64 /* cuts of a KV chunk inside one prefill launch (lsattn_prefill_args.kv_cuts) */

/*
 * One ring / context-parallel prefill attention step: local Q chunk against one KV chunk.
 * Replaces context_attention_fwd + _fwd_kernel (RING:13-188, :190-284).
 *
 * q [Tq,Hq,D], k/v [Tkv,Hkv,D] with the last dimension contiguous and the token / head
 * strides given in elements (k and v are usually the two halves of one interleaved
 * [Tkv,2*Hkv,D] buffer).  The six int32 device vectors of length `batch` carry, per
 * sequence, the start row, the number of local rows and the global index of the first
 * local row for q and for the kv chunk; local row m of q has global position
 * q_first + m*sp_peers, key n has kv_first + n*sp_peers, and key n is visible to row m
 * iff kv position <= q position and n < kv_len (RING:156-159).  sp_peers = 1 with shard
 * offsets in the *_first vectors expresses contiguous sharding.
 */
typedef struct lsattn_prefill_args {
  const void* q;
  const void* k;
  const void* v;
  int64_t q_stride_t, q_stride_h;
  int64_t k_stride_t, k_stride_h;
  int64_t v_stride_t, v_stride_h;
  const int32_t* q_b_start_loc;
  const int32_t* q_b_seq_len;
  const int32_t* q_first_token_global_idx;
  const int32_t* kv_b_start_loc;
  const int32_t* kv_b_seq_len;
  const int32_t* kv_first_token_global_idx;
  int32_t batch;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;   /* 128; 16, 32 and 64 (RING:248-250) run a plainer kernel of their own, which takes no kv_cuts */
  int32_t dtype;      /* LSATTN_F16 or LSATTN_BF16 (q, k, v) */
  int32_t sp_peers;   /* logical_sp_peers_num, >= 1 */
  int32_t max_q_len;  /* max over q_b_seq_len (sizes the launch, RING:262) */
  float sm_scale;     /* natural-domain softmax scale, 1/sqrt(D) in the reference (RING:252) */
  /* outputs */
  void* o;            /* [Tq,Hq,D] */
  int64_t o_stride_t, o_stride_h;
  int32_t o_dtype;    /* step, step_accumulate: LSATTN_F32; step_merge: same as dtype */
  int32_t v_is_f16;   /* 0: v has `dtype`.  1 (dtype LSATTN_BF16 only): v already holds fp16, e.g. written by
                         lsattn_bf16_to_f16_rows: the P V product runs in fp16 either way, and a bf16 V converted
                         inside the kernel costs about 15 % of its speed */
  float* lse;         /* step, step_accumulate: [Tq,Hq] natural-log LSE, contiguous */
  float* m;           /* step_merge: [Tq,Hq] running max, log2 domain       */
  float* l;           /* step_merge: [Tq,Hq] running sum                    */
  int64_t ml_stride_t, ml_stride_h; /* strides of m and l (RING:274-275)     */
  /* Optional (NULL: q_b_start_loc, the reference's layout): per sequence, the first row of o / lse / m / l that the
   * sequence's results go to.  No counterpart in the reference: it lets one launch compute several partials of the same
   * query rows over different slices of a long KV chunk (the sequence entered once per slice, with that slice's
   * kv_b_start_loc / kv_b_seq_len / kv_first_token_global_idx and its own output rows), which lsattn_lse_merge then
   * joins: short query chunks against long KV fill the chip that way.  Zero the struct before filling it in. */
  const int32_t* o_b_start_loc;
  /* Optional (0 or 1: off), lsattn_prefill_step only; no counterpart in the reference.  kv_cuts = S in 2..LSATTN_MAX_KV_CUTS
   * enters every sequence S times into the launch: entry c attends to keys [c * kv_cut_len, (c + 1) * kv_cut_len) of the
   * sequence's KV chunk (kv_cut_len a multiple of 64) and writes the partial (o, lse) of its rows o_cut_rows * c rows
   * further down than entry 0 does, so o and lse hold S * o_cut_rows rows (o_cut_rows >= the rows of q).  A short query
   * chunk against a long KV chunk fills the chip that way (one workgroup per 128 query rows and head otherwise);
   * lsattn_prefill_merge_cuts joins the S partials.  The slices are computed in the kernel from the six vectors above:
   * nothing is prepared on the host or in other launches. */
  int32_t kv_cuts;
  int32_t kv_cut_len;
  int64_t o_cut_rows;
  /* Optional (0: unknown); no counterpart in the reference.  An upper bound of the sum of q_b_seq_len over the batch (the
   * rows of a packed q, for sequences that do not share rows).  The launch is sized by max_q_len times the batch (RING:262),
   * all the host knows; in a batch of one long request and many short ones most of those workgroups find no rows.  With
   * the bound the launch may be sized by the query tiles that can exist instead, each workgroup finding its request from
   * q_b_seq_len.  A bound below the real sum leaves the rows beyond it uncomputed. */
  int64_t total_q_rows;
} lsattn_prefill_args;

/* Partial of one step from the empty state: o = normalised fp32 output, lse = natural-log
 * log-sum-exp; rows that see no key get o = 0, lse = -inf.  Uses o (F32), lse. */
int lsattn_prefill_step(const lsattn_prefill_args* a, void* stream);

/* Drop-in for context_attention_fwd (RING:191-206): folds this step into the running
 * (o, m, l) state in place with the update of RING:171-188.  Start state is m = -inf,
 * l = 0; after any number of calls ln2*(m + log2 l) is the natural LSE over all keys
 * seen and o is the normalised output in o_dtype.  Uses o (dtype of q), m, l. */
int lsattn_prefill_step_merge(const lsattn_prefill_args* a, void* stream);

/* The step of lsattn_prefill_step folded into a running fp32 partial instead of written from the empty state:
 * (o, lse) <- LSE-merge of (o, lse) with this step's (O_i, LSE_i), in the kernel's epilogue.  It is the update of
 * RING:171-188 with the state kept as (fp32 O, natural LSE), the form the decode path and lsattn_lse_merge exchange,
 * and it saves a ring the separate merge pass over P partials.  A row with lse = -inf counts as empty, whatever its o
 * holds; a row that sees no key in this step is left untouched.  First step of a ring: lsattn_prefill_step (or start
 * from lse = -inf everywhere).  Uses o (F32), lse. */
int lsattn_prefill_step_accumulate(const lsattn_prefill_args* a, void* stream);

/*
 * Merge n normalised partials (O_i fp32 [rows,D] contiguous, LSE_i [rows]) over disjoint key
 * sets: LSE = log sum_i exp(LSE_i), O = sum_i exp(LSE_i-LSE) O_i.  Same recurrence as
 * S2CU:38-48 applied to separately allocated partials (the ring steps of one query chunk).
 */
typedef struct lsattn_merge_args {
  int32_t n_parts; /* 1..LSATTN_MAX_PARTS */
  int32_t head_dim; /* 16, 32, 64 or 128 */
  int64_t rows;    /* tokens * heads */
  const float* o_parts[LSATTN_MAX_PARTS];
  const float* lse_parts[LSATTN_MAX_PARTS];
  void* o;         /* [rows,D] contiguous */
  int32_t o_dtype; /* LSATTN_F32 / F16 / BF16 */
  int32_t reserved;
  float* lse;      /* [rows] */
} lsattn_merge_args;
int lsattn_lse_merge(const lsattn_merge_args* a, void* stream);

/*
 * Joins the partials that lsattn_prefill_step wrote with kv_cuts = n_parts (part c of row r at row c * part_rows + r of
 * o_parts [n_parts * part_rows, Hq, D] / lse_parts [n_parts * part_rows, Hq], fp32 contiguous) for the rows of the
 * sequences only (rows q_b_start_loc[b] .. + q_b_seq_len[b]; other rows of the outputs are left alone), into one of the
 * three forms the step itself can produce:
 *   mode 0: (o fp32, lse) written: the partial of the whole step, as lsattn_prefill_step without cuts;
 *   mode 1: folded into the running (o, m, l) in place by the update of RING:171-188, as lsattn_prefill_step_merge
 *           (o in o_dtype F16 / BF16; the step enters with m_i = its LSE in the log2 domain, l_i = 1);
 *   mode 2: LSE-merged into the running (o fp32, lse), as lsattn_prefill_step_accumulate.
 * Rows whose cuts all saw no key: mode 0 writes o = 0, lse = -inf; modes 1 and 2 leave the state as it is.
 * o strides in elements; lse is [rows of q, Hq] contiguous; m, l with their own strides (RING:274-275).
 * No counterpart in the reference, whose grid is one program per 128 query rows and head whatever the KV length (RING:262).
 */
typedef struct lsattn_merge_cuts_args {
  const float* o_parts;
  const float* lse_parts;
  int64_t part_rows;
  int32_t n_parts;     /* 1..LSATTN_MAX_KV_CUTS */
  int32_t mode;        /* 0, 1, 2 as above */
  int32_t batch;
  int32_t num_q_heads;
  int32_t head_dim;    /* 128 */
  int32_t max_q_len;   /* max over q_b_seq_len (sizes the launch) */
  const int32_t* q_b_start_loc;
  const int32_t* q_b_seq_len;
  void* o;
  int64_t o_stride_t, o_stride_h;
  int32_t o_dtype;     /* modes 0, 2: LSATTN_F32; mode 1: LSATTN_F16 or LSATTN_BF16 */
  int32_t reserved;
  float* lse;          /* modes 0, 2 */
  float* m;            /* mode 1 */
  float* l;            /* mode 1 */
  int64_t ml_stride_t, ml_stride_h;
} lsattn_merge_cuts_args;
int lsattn_prefill_merge_cuts(const lsattn_merge_cuts_args* a, void* stream);

/*
 * Flash-decoding stage 1 over a token-indexed KV pool.  Replaces
 * LongServe::flash_decoding_stage1 (S1H:7-27, S1CU:187-215) behind ENTRY:103-164.
 * For request b and block blk with blk*block_seq < b_seqlen[b]:
 *   mid_o[blk,b,h,:], mid_o_logexpsum[blk,b,h] = normalised partial and natural LSE of
 *   q[b,h] against pool rows req_to_tokens[b_req_idx[b], blk*BS : min((blk+1)*BS, len)].
 * Other blocks are left untouched.  Partials are written once, without atomics.
 */
typedef struct lsattn_decode_stage1_args {
  float* mid_o;            /* [num_blocks, batch, Hq, D] contiguous */
  float* mid_o_logexpsum;  /* [num_blocks, batch, Hq]               */
  const void* q;           /* [batch, Hq, D] contiguous              */
  const void* k;           /* [slots, Hkv, D], last dim contiguous   */
  const void* v;
  int64_t k_stride_0, k_stride_1; /* elements */
  int64_t v_stride_0, v_stride_1;
  float sm_scale;
  int32_t dtype;           /* LSATTN_F16 or LSATTN_BF16 */
  const int32_t* req_to_tokens; /* [max_req, max_seq_len] contiguous */
  const int32_t* b_req_idx;     /* [batch] */
  const int32_t* b_seqlen;      /* [batch] */
  int64_t batch;
  int64_t num_q_heads;
  int64_t num_kv_heads;
  int64_t num_blocks;      /* mid_o.size(0) */
  int64_t head_dim;        /* 128 */
  int64_t max_seq_len;     /* req_to_tokens.size(1) */
  int64_t seq_block_size;  /* tokens per partial, >= 1 */
  int64_t max_len_in_batch;
  int64_t merge_blocks;    /* 0 or 1: one partial per block, as the reference.  m in 2..16: one partial per m consecutive
                              blocks, written to the row of the first of them; the rows of the others (as far as the
                              request reaches) get LSE = -inf, i.e. "empty", and their mid_o is left alone.  Any LSE
                              merge over the rows (stage 2 with the same seq_block_size, or with block_seq = 1 and the
                              block count as length, longserve_model.py:514-516) gives the same result with a quarter
                              (m = 4) of the partial bytes written while the gather runs */
  int64_t partials_by_request; /* 0: mid_o is [num_blocks, batch, Hq, D], the reference's buffers (S1H:7-20).  1 (not in the
                              reference): [batch, num_blocks, Hq, D], the partials of a request side by side, for callers to
                              whom mid_o is scratch (the fused call): in a batch the rows of one request lie batch x Hq
                              rows apart in the reference's layout, a page of their own each */
} lsattn_decode_stage1_args;
int lsattn_decode_stage1(const lsattn_decode_stage1_args* a, void* stream);

/*
 * Flash-decoding stage 2: LSE-weighted merge over the block axis.  Replaces
 * LongServe::flash_decoding_stage2 (S2H:7-19, S2CU:116-132) behind ENTRY:166-221.
 * n_b = b_seqlen[b] <= 0 ? 0 : ceil(b_seqlen[b]/block_seq) rows are merged (S2CU:30);
 * n_b = 0 writes o = 0, out_logexpsum = -inf.
 */
typedef struct lsattn_decode_stage2_args {
  void* o;                 /* [batch, H, D] contiguous */
  int32_t o_dtype;         /* LSATTN_F16 / BF16 / F32  */
  int32_t reserved;
  float* out_logexpsum;    /* [batch, H] */
  const int32_t* b_seqlen; /* [batch]    */
  const float* mid_o;            /* [num_seq_blocks, batch, H, D] */
  const float* mid_o_logexpsum;  /* [num_seq_blocks, batch, H]    */
  int64_t batch;
  int64_t num_heads;
  int64_t num_seq_blocks;
  int64_t head_dim;        /* 32, 64 or 128 */
  int64_t block_seq;
  int64_t partials_by_request; /* as in lsattn_decode_stage1_args: 1 reads mid_o as [batch, num_seq_blocks, H, D] */
} lsattn_decode_stage2_args;
int lsattn_decode_stage2(const lsattn_decode_stage2_args* a, void* stream);

/*
 * Stage 1 and stage 2 over the same partials from one call: the two launches of
 * longserve_token_decode_attention_flash_decoding (FDPY:12-27) back to back on `stream`.  Both argument blocks must name
 * the same mid_o, mid_o_logexpsum, b_seqlen, batch, heads, block count, head_dim, block size and layout of the partials (else
 * LSATTN_ERR_INVALID_ARG); everything else as in the two calls it stands for.
 * mid_o and mid_o_logexpsum are scratch to this call, as they are to the reference's function (FDPY:12-27 hands neither
 * out): the call may cut the contexts otherwise than seq_block_size says.  Launches of eight and more requests with
 * enough tokens deal the blocks of all requests (256 tokens each, or the smallest multiple of that by a power of two
 * whose rows the buffers hold) in equal shares to the waves, whatever the lengths of the requests are, and leave one
 * partial per share and request; (o, out_logexpsum) are the same softmax merged from other pieces.
 */
int lsattn_decode_attention(const lsattn_decode_stage1_args* s1, const lsattn_decode_stage2_args* s2, void* stream);

/*
 * lsattn_decode_attention for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the split-K partials live in a device array inside the library instead of
 * caller memory.  It has no counterpart in the reference, whose callers allocate mid_o / mid_o_logexpsum themselves
 * (longserve_model.py:514-517).  Both argument blocks are filled as for lsattn_decode_attention, except that mid_o and
 * mid_o_logexpsum must be NULL in both; num_blocks (= num_seq_blocks) is the number of partial rows the caller would
 * have allocated, and min(num_blocks, ceil(max_len_in_batch / seq_block_size)) * batch * Hq * (D + 1) * 4 bytes must not
 * exceed LSATTN_STATIC_SCRATCH_BYTES (else LSATTN_ERR_WORKSPACE); merge_blocks must be 0 or 1.  Results are those of
 * lsattn_decode_attention: the same kernels; bit for bit whenever both calls cut the contexts alike, which they do
 * unless the launch is dealt in equal shares and the array holds fewer rows for the batch than the caller's buffers would
 * (then the shares are counted in larger blocks and the sums are added in another order).  The call allocates and frees nothing.  Each GPU has one such array (held until
 * the process ends) and every call on that GPU uses it: calls that overlap on one GPU (two streams, two threads) race;
 * calls in stream order on one stream do not.  Nothing needs clearing between calls: stage 2 reads only rows that
 * stage 1 of the same call has written.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make that call outside any stream capture.
 */
#define LSATTN_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)
int lsattn_decode_attention_static(const lsattn_decode_stage1_args* s1, const lsattn_decode_stage2_args* s2, void* stream);

/*
 * Row scatter into the KV pool: dst[dest_index[i]] = src[i] for i < n_rows, bit-exact.
 * Replaces _fwd_kernel_destindex_copy_kv
 * (loongserve/common/basemodel/triton_kernel/destindex_copy_kv.py:7-51).
 * Rows are row_bytes long (a multiple of 16, 16-byte aligned); strides are in bytes.
 */
int lsattn_kv_scatter(const void* src, int64_t src_stride_bytes, void* dst, int64_t dst_stride_bytes,
                      const int32_t* dest_index, int64_t n_rows, int64_t row_bytes, void* stream);

/*
 * Prefill registration of freshly written slots:
 *   req_to_tokens[b_req_idx[b], 0:b_seq_len[b]] = mem_index[b_start_loc[b] : +b_seq_len[b]].
 * Replaces init_req_to_token_indexes (loongserve/common/infer_utils.py:1-13), which loops
 * on the host after a device-to-host copy.
 */
int lsattn_register_tokens(int32_t* req_to_tokens, int64_t max_seq_len, const int32_t* b_req_idx,
                           const int32_t* b_start_loc, const int32_t* b_seq_len, const int32_t* mem_index,
                           int64_t batch, int64_t max_len_in_batch, void* stream);

/*
 * Decode registration of one new slot per request:
 *   req_to_tokens[b_req_idx[i], b_seq_len[i] - 1] = mem_index[i]   for i < batch.
 * Replaces copy_kv_index_to_req (loongserve/common/basemodel/triton_kernel/copy_kv_index_to_req.py:7-40, called
 * loongserve/models/llama/longserve_model.py:491, :497).  mem_index is int32, or int64 as the allocator hands it out
 * (mem_index_is_i64 = 1).  An entry whose position falls outside the row is skipped (the reference would write there).
 */
int lsattn_register_decode_tokens(int32_t* req_to_tokens, int64_t max_seq_len, const int32_t* b_req_idx,
                                  const int32_t* b_seq_len, const void* mem_index, int32_t mem_index_is_i64,
                                  int64_t batch, void* stream);

/*
 * Which locally held KV rows of each request belong to the cache-index window
 * [kv_cache_index_begin, kv_cache_index_end) when local row n holds global token
 * kv_first_token_global_idx + n * sp_peers:
 *   kv_range_begin = ceil((kv_cache_index_begin - kv_first_token_global_idx) / sp_peers)
 *   kv_range_end   = ceil((kv_cache_index_end   - kv_first_token_global_idx) / sp_peers)
 *   new_kv_cache_len = kv_range_end - kv_range_begin
 * (ceil as Python floor division of x + sp_peers - 1, the form the reference documents).
 * Replaces pre_copy_and_register_kv
 * (loongserve/models/llama/triton_kernel/copy_and_register_kv.py:6-62).
 */
int lsattn_kv_ranges(const int32_t* kv_cache_index_begin, const int32_t* kv_cache_index_end,
                     const int32_t* kv_first_token_global_idx, int32_t sp_peers, int64_t batch,
                     int32_t* kv_range_begin, int32_t* kv_range_end, int32_t* new_kv_cache_len, void* stream);

/*
 * Context migration during prefill: for every request b with new_kv_cache_len[b] > 0 and non-negative
 * range bounds, and every n < min(new_kv_cache_len[b], row_limit):
 *   slot = mem_index[num_used_mem_index + (b > 0 ? new_kv_cache_len_sum[b-1] : 0) + n]
 *   pool[slot] = kv[kv_b_start_loc[b] + kv_range_begin[b] + n]                    (bit-exact row copy)
 *   if should_register: req_to_tokens[b_req_idx[b], cur_kv_cache_index[b] + n] = slot
 * row_limit is the reference's grid bound, max_len_in_batch rounded up to a multiple of 256.
 * Replaces destindex_copy_and_register_kv
 * (loongserve/models/llama/triton_kernel/copy_and_register_kv.py:64-170; called from
 * longserve_transformer_layer_infer.py:199-215).
 * Rows are row_bytes long (a multiple of 16, 16-byte aligned); strides are in bytes.
 */
typedef struct lsattn_kv_copy_register_args {
  const void* kv;                      /* [tokens, row_bytes] source rows              */
  int64_t kv_stride_bytes;
  void* pool;                          /* [slots, row_bytes] KV pool of this layer     */
  int64_t pool_stride_bytes;
  int64_t row_bytes;
  const int32_t* new_kv_cache_len;     /* [batch] */
  const int32_t* kv_range_begin;       /* [batch] */
  const int32_t* kv_range_end;         /* [batch] */
  const int64_t* new_kv_cache_len_sum; /* [batch] inclusive prefix sum of new_kv_cache_len */
  const int32_t* kv_b_start_loc;       /* [batch] */
  const int32_t* cur_kv_cache_index;   /* [batch] (read only when should_register)     */
  const int32_t* mem_index;            /* [>= num_used_mem_index + sum] pool slots      */
  const int32_t* b_req_idx;            /* [batch] (read only when should_register)     */
  int32_t* req_to_tokens;              /* [max_req, max_seq_len] (written only when should_register) */
  int64_t max_seq_len;
  int64_t batch;
  int64_t num_used_mem_index;
  int64_t max_len_in_batch;
  int32_t should_register;
  int32_t reserved;
} lsattn_kv_copy_register_args;
int lsattn_kv_copy_register(const lsattn_kv_copy_register_args* a, void* stream);

/*
 * Decoding-stage migration of the last num_tokens[b] tokens of every request b, all layers in one launch.
 * kv_cache is [num_layers, kvcache_size, row_bytes], the staging buffer [num_layers, sum(num_tokens), row_bytes]
 * (row strides and layer strides in bytes, rows a multiple of 16 bytes, 16-byte aligned); num_tokens_cumsum is the
 * inclusive prefix sum of num_tokens (same integer type), max_num_tokens an upper bound of num_tokens[] for the launch.
 *
 * Sender, for j < num_tokens[b]:  slot = req_to_tokens[request_ids[b], b_seq_len[b] - num_tokens[b] + j];
 *   mem_state[slot] = 0;  send_buf[:, cumsum[b-1] + j] = kv_cache[:, slot]      (bit-exact)
 * Receiver, for j < num_tokens[b]:  slot = alloc_mem[cumsum[b-1] + j];
 *   req_to_tokens[request_ids[b], b_seq_len[b] + j] = slot;  kv_cache[:, slot] = recv_buf[:, cumsum[b-1] + j]
 * Replace _fwd_sender_kernel / _fwd_receiver_kernel
 * (loongserve/models/llama/triton_kernel/decoding_stage_migration.py:6-68, :100-157; called longserve_model.py:600-619).
 */
typedef struct lsattn_decode_migration_args {
  void* staging;                    /* send_buf (written) or recv_buf (read) */
  int64_t staging_layer_stride_bytes;
  int64_t staging_row_stride_bytes;
  void* kv_cache;                   /* read by the sender, written by the receiver */
  int64_t kv_layer_stride_bytes;
  int64_t kv_row_stride_bytes;
  int64_t row_bytes;
  int64_t num_layers;
  int32_t* req_to_tokens;           /* [max_req, max_seq_len] */
  int64_t max_seq_len;
  int32_t* mem_state;               /* sender only */
  const int32_t* alloc_mem;         /* receiver only: [sum(num_tokens)] */
  const int32_t* request_ids;       /* [batch] */
  const int32_t* num_tokens;        /* [batch] */
  const int32_t* num_tokens_cumsum; /* [batch] */
  const int32_t* b_seq_len;         /* [batch] */
  int64_t batch;
  int64_t max_num_tokens;
} lsattn_decode_migration_args;
int lsattn_decode_migration_send(const lsattn_decode_migration_args* a, void* stream);
int lsattn_decode_migration_recv(const lsattn_decode_migration_args* a, void* stream);

/*
 * The element-wise fp16 steps before and after attention (the rest of the reference's extension module).
 * All pointers are 16-byte aligned device pointers; sizes in elements.
 *
 * out[t, i] = half(float(in[t, i]) * float(weight[i]) * rsqrt(mean_i(in[t, i]^2) + eps)); hidden_size % 8 == 0.
 * Replaces LongServe::rms_norm (longserve_cuda_kernels/src/rms_norm.cu:10-62; binding entrypoints.cpp:15-39).
 */
int lsattn_rms_norm(void* out, const void* in, const void* weight, int64_t num_tokens, int64_t hidden_size, float eps,
                    void* stream);
/*
 * io is [num_tokens, 2 * ffn_inter_dim]: io[t, i] = half(silu(io[t, i])) * io[t, ffn_inter_dim + i] (half multiply) for
 * i < ffn_inter_dim; the second half of every row is left as it is.  ffn_inter_dim % 8 == 0.
 * Replaces LongServe::silu_and_mul_inplace (silu_and_mul.cu:12-49; binding entrypoints.cpp:41-52).
 */
int lsattn_silu_and_mul_inplace(void* io, int64_t num_tokens, int64_t ffn_inter_dim, void* stream);
/*
 * In-place rotary embedding of x[t, h, 0:head_dim] (last dimension contiguous, strides in elements, multiples of 8)
 * with cos/sin [num_tokens, head_dim/2] contiguous: x1 = x[..., :D/2], x2 = x[..., D/2:],
 *   x1' = fma(x1, cos, -(x2 * sin)),  x2' = fma(x1, sin, x2 * cos), every operation rounded to half once
 * (bit-exact with the reference's half2 arithmetic).  head_dim % 16 == 0.
 * Replaces LongServe::rotary_emb (rotary_emb.cu:10-55; binding entrypoints.cpp:54-89, called once for q and once for k).
 */
int lsattn_rotary_emb(void* x, const void* cos, const void* sin, int64_t x_stride_t, int64_t x_stride_h,
                      int64_t num_tokens, int64_t num_heads, int64_t head_dim, void* stream);

/*
 * The write-back of a step's new tokens in one launch instead of the reference's three passes over K and V:
 *   rotary embedding of q and of the K heads of kv, in place, as lsattn_rotary_emb
 *     (longserve_cuda_kernels.rotary_emb, called longserve_transformer_layer_infer.py:88-93);
 *   pool[dest_index[t]] = the token's row of kv after the rotation, K heads then V heads, bit-exact
 *     (destindex_copy_kv, longserve_transformer_layer_infer.py:377; skipped when pool is NULL);
 *   register_mode 1: req_to_tokens[b_req_idx[b], 0:b_seq_len[b]] = dest_index[b_start_loc[b] : +b_seq_len[b]]
 *     (init_req_to_token_indexes, loongserve/common/infer_utils.py:1-13);
 *   register_mode 2: req_to_tokens[b_req_idx[i], b_seq_len[i] - 1] = dest_index[i], one new token per request
 *     (copy_kv_index_to_req, longserve_model.py:491); register_mode 0: the table is left alone.
 * q [T, Hq, D] and kv [T, 2*Hkv, D] are fp16 with the last dimension contiguous (strides in elements, multiples of 8),
 * cos / sin [T, D/2] contiguous, a pool slot holds 2*Hkv*D contiguous elements, pool_slot_stride elements apart.
 * head_dim % 16 == 0.  kv stays valid for the attention step that follows (K rotated in place).
 */
typedef struct lsattn_rotary_kv_write_args {
  void* q;
  int64_t q_stride_t, q_stride_h;
  int64_t num_q_heads;
  void* kv;
  int64_t kv_stride_t, kv_stride_h;
  int64_t num_kv_heads;
  const void* cos;
  const void* sin;
  int64_t num_tokens;
  int64_t head_dim;
  void* pool;                   /* [slots, 2*Hkv*D] or NULL */
  int64_t pool_slot_stride;
  const int32_t* dest_index;    /* [num_tokens] */
  int32_t* req_to_tokens;       /* [max_req, max_seq_len] */
  int64_t max_seq_len;
  const int32_t* b_req_idx;     /* [batch] */
  const int32_t* b_start_loc;   /* [batch], register_mode 1 */
  const int32_t* b_seq_len;     /* [batch] */
  int64_t batch;
  int64_t max_len_in_batch;     /* register_mode 1: upper bound of b_seq_len[] (sizes the launch) */
  int32_t register_mode;
  int32_t reserved;
} lsattn_rotary_kv_write_args;
int lsattn_rotary_kv_write(const lsattn_rotary_kv_write_args* a, void* stream);

/*
 * Slot allocator of the KV pool.  mem_state is int32 [pool_size] on the device (16-byte aligned), 0 = free slot,
 * otherwise the slot's reference count.  The searches need a device workspace of
 * lsattn_pool_search_workspace_bytes(pool_size) bytes (16-byte aligned); nothing is allocated or kept by the library
 * and no call waits for the device.
 *
 * lsattn_pool_alloc: out_index[0:need] = the first `need` free slots in ascending order, each marked in use
 * (0 -> 1).  If fewer are free, the rest of out_index is -1; the caller compares `need` with its own count of
 * free slots first, as the reference does.  Replaces torch.nonzero(mem_state == 0)[0:need] + add_refs in
 * LongServeMemoryManager.alloc (loongserve/common/longserve_mem_manager.py:32-40).
 */
size_t lsattn_pool_search_workspace_bytes(int64_t pool_size);
int lsattn_pool_alloc(int32_t* mem_state, int64_t pool_size, int64_t need, int64_t* out_index, void* workspace,
                      size_t workspace_bytes, void* stream);
/*
 * *out_start (device) = the lowest s such that slots s .. s+need-1 are all free, or -1 if there is no such run.
 * mem_state is not changed.  Replaces the nonzero / shifted-difference search of
 * LongServeMemoryManager.alloc_contiguous (longserve_mem_manager.py:50-55); need >= 1.
 */
int lsattn_pool_find_contiguous(const int32_t* mem_state, int64_t pool_size, int64_t need, int64_t* out_start,
                                void* workspace, size_t workspace_bytes, void* stream);
/*
 * mem_state[index[i]] = old value + delta (delta = +1 or -1) for i < n; a slot listed several times still changes
 * by delta once, as `mem_state[index] += delta` does in torch.  counted (device, int64[2]):
 *   counted[0] = entries whose slot is non-zero before the update (delta = +1) or after it (delta = -1): the
 *                has_used_tokens / used_tokens of add_refs and decrease_refs (longserve_mem_manager.py:73-88);
 *   counted[1] = entries outside [-pool_size, pool_size), which are skipped (negative entries wrap once).
 * workspace: lsattn_pool_refs_workspace_bytes(n) bytes, 16-byte aligned.
 */
size_t lsattn_pool_refs_workspace_bytes(int64_t n);
int lsattn_pool_update_refs(int32_t* mem_state, int64_t pool_size, const int64_t* index, int64_t n, int delta,
                            int64_t* counted, void* workspace, size_t workspace_bytes, void* stream);

/*
 * dst[r, 0:row_elems] = fp16(src[r, 0:row_elems]) for r < n_rows, bf16 -> fp16 rounded toward zero (exact for every
 * bf16 in fp16's normal range; larger magnitudes become +-65504).  Strides in elements; row_elems, strides % 8 == 0,
 * pointers 16-byte aligned.  No counterpart in the reference (its kernels are fp16 only): prepares V for
 * lsattn_prefill_step* with v_is_f16 = 1.
 */
int lsattn_bf16_to_f16_rows(const void* src, int64_t src_stride, void* dst, int64_t dst_stride, int64_t n_rows,
                            int64_t row_elems, void* stream);

/*
 * Launch choices that the library otherwise makes from the size of a launch, forced process-wide (tuning, and tests that
 * must reach every kernel shape whatever the size of their inputs).  No counterpart in the reference.  Every field 0 means
 * "the library's choice"; a NULL argument restores that for all of them.  The block is copied; launches made after the
 * call returns see it (calls from several threads: each field is stored and read atomically, a launch may see a mix
 * while a store is under way).  The library reads no environment variable.  Returns LSATTN_ERR_INVALID_ARG for a value
 * not listed here.
 */
#define LSATTN_PREFILL_ROWS_128 1   /* eight waves, 128 query rows, two waves per 32 rows                          */
#define LSATTN_PREFILL_ROWS_256 2   /* eight waves, 256 query rows                                                */
#define LSATTN_PREFILL_ROWS_HALF 3  /* four waves, 128 query rows, two workgroups per CU                          */
#define LSATTN_PREFILL_ORDER_TILE 1 /* heaviest query tiles of all KV heads first                                  */
#define LSATTN_PREFILL_ORDER_HEAD 2 /* one KV head at a time per XCD                                               */
#define LSATTN_PREFILL_PACK_OFF 1   /* one query head per workgroup instead of the heads of a KV head side by side */
#define LSATTN_DECODE_STAGE1_LANE 1  /* the lane kernel                                                            */
#define LSATTN_DECODE_STAGE1_MFMA 2  /* the matrix-pipe kernel, one wave per block (where its conditions hold)      */
#define LSATTN_DECODE_STAGE1_SPLIT 3 /* the matrix-pipe kernel, the four waves of a workgroup on one block          */
#define LSATTN_DECODE_LISTED_OFF 1   /* stage 1's grid sized by the longest request                                */
#define LSATTN_DECODE_LISTED_ON 2    /* a fixed grid walks the list of units that exist                            */
#define LSATTN_DECODE_LISTED_SHARES 3 /* lsattn_decode_attention deals the blocks in equal shares whatever the size   */
typedef struct lsattn_tuning {
  int32_t prefill_rows;
  int32_t prefill_order;
  int32_t prefill_pack;
  int32_t decode_stage1;
  int32_t decode_listed;
  int32_t reserved[3];  /* 0 */
} lsattn_tuning;
int lsattn_set_tuning(const lsattn_tuning* t);

const char* lsattn_strerror(int code);
/* Version of this interface.  It changes whenever an argument block or an entry point changes.  The argument blocks
 * carry no size field, so a caller must be compiled against the header of the library it loads: check
 * lsattn_version() == LSATTN_VERSION once after loading and refuse to run otherwise.
 * 2 = o_b_start_loc in lsattn_prefill_args, partials_by_request in both decode argument blocks; 3 = lsattn_set_tuning,
 * kv_cuts / kv_cut_len / o_cut_rows / total_q_rows in lsattn_prefill_args, lsattn_prefill_merge_cuts. */
#define LSATTN_VERSION 3
int lsattn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* LSATTN_H */
