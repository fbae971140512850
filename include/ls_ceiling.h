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
 * 4096 workgroups of 256 lanes.  sink: 1024 bytes (practically never written). */
int ls_ceiling_read(const void* src, uint64_t bytes, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LS_CEILING_H */
