/*
 * ls_ceiling.h -- what one MI355X sustains with nothing in the way, measured in the run that reports a kernel's
 * fraction of it (libls_ceiling.so; loaded by bench.py only, never by the operators).  No counterpart in the reference.
 * Both calls launch asynchronously on `stream` (a hipStream_t as void*, NULL = the default stream), allocate nothing
 * and return 0, -1 (bad argument) or -3 (launch error).
 */
#ifndef LS_CEILING_H
#define LS_CEILING_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* `workgroups` workgroups of four waves, one workgroup per CU at a time (256 fill the chip once), every wave issuing
 * iters * 16 independent v_mfma_f32_16x16x32_f16 on operands read once from `operands` (at least 256 KiB of fp16 values,
 * 16-byte aligned; random values make the matrix pipe draw what it draws on real data) and nothing else.
 * sink: 4 * 256 * workgroups bytes (practically never written).  ls_ceiling_mfma_f16_flop gives the launch's flop count. */
int ls_ceiling_mfma_f16(const void* operands, void* sink, int iters, int workgroups, void* stream);
double ls_ceiling_mfma_f16_flop(int iters, int workgroups);

/* Reads `bytes` bytes at src (16-byte aligned) once, 16 bytes per lane and load, eight loads in flight per lane,
 * a wave 8 KB side by side at a time, 4096 workgroups of 256 lanes.  sink: 1024 bytes (practically never written). */
int ls_ceiling_read(const void* src, uint64_t bytes, void* sink, void* stream);

/* The same read with stores mixed in (what the partials of a split-K decode do to its gather): in one of every `every`
 * trips of a wave's loop over 8 KB of reads, spread over the waves and the launch, the wave also writes 8 KB to
 * dst (sixteen rows of 512 bytes, a store instruction a 64-byte piece of each).  every = 64: 1.6 % of the bytes, the
 * share of one fp32 partial per 256 tokens and 32 query heads on 8 KV heads.  system_scope != 0: the stores are written
 * through to memory as they are issued (sc0 sc1) instead of being written back from the L2 later.
 * dst: ls_ceiling_read_with_stores_bytes(bytes, every) bytes, 16-byte aligned. */
int ls_ceiling_read_with_stores(const void* src, uint64_t bytes, void* dst, uint32_t every, int system_scope, void* sink, void* stream);
uint64_t ls_ceiling_read_with_stores_bytes(uint64_t bytes, uint32_t every);

#ifdef __cplusplus
}
#endif
#endif /* LS_CEILING_H */
