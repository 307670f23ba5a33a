/* infer_kv_probe.h - C ABI of libinfer_kv_probe.so: plain streaming kernels for measurement.
 *
 * No counterpart in the reference and not part of the KV-cache path: bench.py --ceiling and
 * bench.py --counters load this library to measure what the part sustains for a read-only stream,
 * for a copy, and for the read half and the write half of a KV append on their own, with the same
 * timing method as the kernels of libinfer_kv.so.  Return codes as in infer_kv.h.
 */
#ifndef INFER_KV_PROBE_H
#define INFER_KV_PROBE_H

#include <stddef.h>
#include <stdint.h>

#include "infer_kv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A read of `bytes` in contiguous per-workgroup shares, same launch shape as the decode kernel
 * (512-thread workgroups).  `sink4` is 4 writable bytes. */
int infer_kv_probe_read(const void* src, size_t bytes, void* sink4, int workgroups, void* stream);
/* the same read with the streaming (nontemporal) hint the decode kernel puts on its V loads */
int infer_kv_probe_read_streaming(const void* src, size_t bytes, void* sink4, int workgroups, void* stream);
/* a copy as a grid-stride loop over `workgroups` workgroups of 256 threads */
int infer_kv_probe_copy(const void* src, void* dst, size_t bytes, int workgroups, void* stream);
/* a copy with one wavefront per 4 KiB and no loop (whole 4 KiB pieces only) */
int infer_kv_probe_copy_rows(const void* src, void* dst, size_t bytes, void* stream);

/* The two read streams of the decode kernel without its arithmetic: `tokens` rows of 2 KiB (8 KV heads of
 * 256 B) in each of k and v, one wavefront per KV head, 32-token steps in contiguous per-workgroup shares.
 * V is read as whole rows; K in the decode kernel's MFMA-operand pattern (16 tokens x 64 B per
 * instruction) or, with k_whole_rows, as whole rows too.  k_hint / v_hint put the streaming
 * (nontemporal) hint on the loads of that stream. */
int infer_kv_probe_read_kv_pattern(const void* k, const void* v, size_t tokens, int k_whole_rows, int k_hint,
                                   int v_hint, void* sink4, int workgroups, void* stream);

/* The two halves of infer_kv_append_bf16 for rows of 2 KiB (dkv = 1024), contiguous sources: the
 * first loads the K and V row of every row with a valid slot and stores nothing, the second stores
 * a K and a V row to the slot of every such row and loads nothing. */
int infer_kv_probe_append_read_half(const void* key, const void* value, const int32_t* slot_mapping,
                                    int64_t n_rows, int64_t num_slots, void* sink4, void* stream);
int infer_kv_probe_append_write_half(void* k_cache, void* v_cache, const int32_t* slot_mapping,
                                     int64_t n_rows, int64_t num_slots, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* INFER_KV_PROBE_H */
