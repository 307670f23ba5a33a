// Layout of the caller-provided workspace of the paged decode kernels (host side only).
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "../../include/infer_kv.h"

// Upper bound on the number of KV-split workgroups.  A caller-provided workspace is always laid out
// for it, so its offsets depend on nothing but the shape: the split and the merge launch agree on
// where every record lives whatever split count a call asks for.
#define INFER_KV_MAX_SPLIT_WG 1024

// The first pieces of every sequence have records at fixed places, [batch][KV head][this many], so that
// the merge kernel can request them before it has read how many pieces a sequence has.
#define INFER_KV_DECODE_FIRST_PIECES 4

struct DecodeWorkspace {
    size_t header_off;      // int32[64]: {spans used by the last launch, total steps, spans per workgroup and KV head} (diagnostic)
    size_t seg_first_off;   // int32[batch]: first split workgroup that touched the sequence
    size_t seg_last_off;    // int32[batch]: last one
    size_t rec_first_off;   // [batch][KV heads][INFER_KV_DECODE_FIRST_PIECES] records: pieces 0 .. 3 of every sequence
    size_t rec_off;         // [slots] records of rec_stride bytes: later pieces, one per (span position, sequence, KV head)
    size_t rec_stride;      // bytes per record, a multiple of 16
    int64_t slots_per_head; // records per KV head: split_cap + batch
    size_t total_bytes;
};

static inline size_t align_up_256(size_t x) { return (x + 255) & ~(size_t)255; }

// A partial-result record is written by one wavefront exactly as it sits in that wavefront's
// registers, so that the store is one contiguous run: for the `group` query heads n of a KV head,
//   float[4][group][8][4]  accumulator: element (g, n, t, e) is O[n][16 t + 4 g + e] (unnormalised)
//   float[group][2]        running max (log2 domain) and sum of head n
// padded to a multiple of 16 bytes.
static inline size_t decode_record_bytes(int64_t group) { return ((size_t)group * 520 + 15) & ~(size_t)15; }

// slots = num_kv_heads * (split_cap + batch): the chain of (workgroup span position s < split_cap,
// sequence b) of KV head h uses slot h * (split_cap + batch) + s + b, which is unique because
// consecutive chains along the flattened token axis advance s or b (or both) by one.  split_cap is
// INFER_KV_MAX_SPLIT_WG for a caller-provided workspace; the entry point that brings its own
// fixed-size scratch lays it out for the split count it launches.
static inline DecodeWorkspace decode_workspace_layout(int64_t batch, int64_t group, int64_t num_kv_heads,
                                                      int64_t split_cap = INFER_KV_MAX_SPLIT_WG) {
    DecodeWorkspace ws;
    ws.slots_per_head = split_cap + batch;
    const size_t slots = (size_t)num_kv_heads * (size_t)ws.slots_per_head;
    size_t off = 0;
    ws.header_off = off;      off = align_up_256(off + 64 * sizeof(int32_t));
    ws.seg_first_off = off;   off = align_up_256(off + (size_t)batch * sizeof(int32_t));
    ws.seg_last_off = off;    off = align_up_256(off + (size_t)batch * sizeof(int32_t));
    ws.rec_stride = decode_record_bytes(group);
    ws.rec_first_off = off;   off = align_up_256(off + (size_t)batch * (size_t)num_kv_heads * INFER_KV_DECODE_FIRST_PIECES * ws.rec_stride);
    ws.rec_off = off;         off = align_up_256(off + slots * ws.rec_stride);
    ws.total_bytes = off;
    return ws;
}
