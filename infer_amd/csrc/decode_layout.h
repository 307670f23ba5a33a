// Layout of the caller-provided workspace of the paged decode kernels (host side only).
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "../../include/infer_kv.h"

// Upper bound on the number of KV-split workgroups; the workspace is always laid out for it, so
// its offsets do not depend on the tuning knob.
#define INFER_KV_MAX_SPLIT_WG 1024

struct DecodeWorkspace {
    size_t header_off;      // int32[64]: {workgroups, steps per span, total steps}
    size_t seg_first_off;   // int32[batch]: first split workgroup that touched the sequence
    size_t seg_last_off;    // int32[batch]: last one
    size_t ml_off;          // float[slots][group][2]: running max (log2 domain) and sum
    size_t po_off;          // float[slots][group][128]: unnormalised accumulator
    size_t total_bytes;
};

static inline size_t align_up_256(size_t x) { return (x + 255) & ~(size_t)255; }

// slots = num_kv_heads * (INFER_KV_MAX_SPLIT_WG + batch): segment (workgroup w, sequence b) of KV
// head h uses slot h * (W + batch) + w + b, which is unique because consecutive segments along
// the flattened token axis advance w or b (or both) by one.
static inline DecodeWorkspace decode_workspace_layout(int64_t batch, int64_t group, int64_t num_kv_heads) {
    DecodeWorkspace ws;
    const size_t slots = (size_t)num_kv_heads * (size_t)(INFER_KV_MAX_SPLIT_WG + batch);
    size_t off = 0;
    ws.header_off = off;      off = align_up_256(off + 64 * sizeof(int32_t));
    ws.seg_first_off = off;   off = align_up_256(off + (size_t)batch * sizeof(int32_t));
    ws.seg_last_off = off;    off = align_up_256(off + (size_t)batch * sizeof(int32_t));
    ws.ml_off = off;          off = align_up_256(off + slots * (size_t)group * 2 * sizeof(float));
    ws.po_off = off;          off = align_up_256(off + slots * (size_t)group * 128 * sizeof(float));
    ws.total_bytes = off;
    return ws;
}
