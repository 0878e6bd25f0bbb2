// Launch parameters of the attention kernels, shared by the C ABI wrapper and the model driver.
#pragma once
#include "agpu_internal.h"

struct AttnParams {
    const float *q;  // element (b, h, i, e) at q[b*q_batch_stride + h*q_head_stride + i*q_row_stride + e]
    const float *k;  // [batch*n_heads, kv_stride, 64]
    const float *v;
    float *o;        // element (b, h, i, e) at o[b*o_batch_stride + h*o_head_stride + i*o_row_stride + e]
    int n_heads, batch, q_len, kv_len, q_offset, kv_stride, causal;
    long long q_batch_stride, q_head_stride, q_row_stride;
    long long o_batch_stride, o_head_stride, o_row_stride;
    // When non-null the kernels read the number of positions already cached from here and use
    // kv_len = *pos_dev + q_len, q_offset = *pos_dev (lets one captured launch serve every step).
    const int *pos_dev;
    // Decode kernel: fetch the first pass of K/V rows before the context length is known (hides one memory
    // round trip; reads up to 32 * waves rows whatever the length).  Set by the launcher for small launches.
    int speculate;
    // Prefill kernel: a workgroup takes query block nb-1-x and then block x (set by the launcher).
    int pair_blocks;
    // Decode kernel with the keys split over gridDim.z workgroups (set by the launcher): keys per workgroup, where
    // the partial results go, and the tickets (one per query row and head, left at zero).
    int kv_chunk;
    float *kv_partial;
    unsigned int *counters;
    int strict;  // the context's strict_sync
    // Decode kernel, q_len == 1 and batch <= 16 only: the outputs once more as the bf16 pieces of the next Linear's
    // input (row = sequence, k = head * 64 + e; layout in linear_common.h), or null.
    uint4 *px_pieces;
};

// max_kv_len bounds kv_len for launches that read it from pos_dev (sizes the key split).
int32_t agpu_attention_launch(agpu_ctx *ctx, const AttnParams &p, int max_kv_len);

// Causal prefill attention of queries 0 .. q_len - 1 over keys 0 .. kv_len - 1 (kv_len >= q_len >= 256, host values; p.k and
// p.v are not read) with K and V given as bf16 operand fragments: [batch * n_heads][tiles_cap tiles of 32 keys][768
// fragments of 16 bytes] each, in the layout attention.hip describes; agpu_attention_fragment_bytes sizes one array.
size_t agpu_attention_fragment_bytes(int heads, int kv_len);
int32_t agpu_attention_fragments_launch(agpu_ctx *ctx, const AttnParams &p, const uint4 *kfrag, const uint4 *vfrag, int tiles_cap);
