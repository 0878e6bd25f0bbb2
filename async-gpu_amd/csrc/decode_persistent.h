// One-launch-per-token decode step for a single sequence (the B = 1 greedy loop of generate_cached,
// nn/models/gpt2.rs:760-780): host-side plan and launcher of decode_persistent.hip.
#pragma once
#include "agpu_internal.h"

// What the planner needs to know about one int4 Linear of the model.
struct PkLinear {
    const uint32_t *packed;  // [K/8, stride]
    const float *scales;     // [ceil(K/group), stride]
    const float *bias;       // [N] or null
    int K, N, stride;        // N valid columns, stride = row stride of packed/scales in words
};

struct PkLayer {
    const float *ln1_g, *ln1_b, *ln2_g, *ln2_b;
    PkLinear qkv, proj, fc, fc_proj;
    float *kcache, *vcache;  // [H, n_positions, 64] of this layer, sequence 0
};

struct PkModel {
    int d, H, ff, V, P, group, n_layer;
    float eps;
    int gelu_quick, argmax_last;
    const float *wte, *wpe, *lnf_g, *lnf_b;
    PkLinear head;
    const PkLayer *layers;  // host array [n_layer]
    float *logits;          // [head.stride] row of the step's logits
    uint32_t *cur_tok, *out_tok, *next_tok;
    int *pos_dev, *step_dev;
    int out_capacity;
};

struct PkPlan {
    void *stages_dev = nullptr;   // stage table
    int n_stages = 0;
    // (value, tag) pairs: every activation vector of one step + the arg-max candidates, [1 + 8][arena_elems]: the
    // copy in memory that the producers write, then one mirror per XCD
    unsigned long long *arena = nullptr;
    size_t arena_elems = 0;
    size_t cand_off = 0;  // where the arg-max candidates start
    unsigned int *state = nullptr;  // [0] epoch of the last finished step, [1] error word (0 = none)
    int grid = 0;
    int att_per_xcd = 0;  // workgroups per XCD that only do attention
    int smax = 1;         // key ranges per head at most
    size_t lds_bytes = 0;
    int kmax = 0;         // longest input vector of a Linear: sizes the staging buffers
    int head_slots = 0;   // slots of the head's second chunk that wait in LDS (0: fetched when their turn comes)
    int spin_limit = 0;   // poll rounds a wait inside the kernel may take; 0 = the default
    int kind = 0;         // 0: every Linear spread over the device (decode_persistent.hip); 1: one tensor-parallel rank per XCD (decode_xcd.hip)
    int lin_per_xcd = 0;  // kind 1: Linear workgroups per XCD
    int touch_dist = 0;   // kind 1: how many exchanges ahead the relays touch the weights (0: not at all)
    size_t parts_elems = 0;  // kind 1: floats of one set of partial sums
    int head_tpc = 0;        // kind 1: tiles per chunk of the head stage
    float *ln_fold = nullptr;  // kind 1: the LayerNorms folded into the Linears behind them (A_n, B_n per column)
};

// Whether the persistent step can run this model (int4 head, head_dim 64, group 32, size limits).
bool agpu_pk_supported(const agpu_ctx *ctx, const PkModel &m);
int32_t agpu_pk_plan_build(agpu_ctx *ctx, const PkModel &m, PkPlan *plan);
void agpu_pk_plan_free(PkPlan *plan);
// One decode step on the context's stream.  mode 0: the real step; mode 1: the same stage chain with empty bodies
// (every wait and every tagged store, no weights, no arithmetic): the latency floor of the chain.
int32_t agpu_pk_launch(agpu_ctx *ctx, const PkModel &m, const PkPlan &plan, int mode, unsigned long long *trace = nullptr);
// The same step with the XCDs as tensor-parallel ranks (decode_xcd.hip): plan (freed by agpu_pk_plan_free) and launch.
bool agpu_xk_supported(const agpu_ctx *ctx, const PkModel &m);
int32_t agpu_xk_plan_build(agpu_ctx *ctx, const PkModel &m, PkPlan *plan);
int32_t agpu_xk_launch(agpu_ctx *ctx, const PkModel &m, const PkPlan &plan, int mode, unsigned long long *trace = nullptr);
// Launches a plan of either kind.
inline int32_t agpu_step_launch(agpu_ctx *ctx, const PkModel &m, const PkPlan &plan, int mode, unsigned long long *trace = nullptr) {
    return plan.kind == 1 ? agpu_xk_launch(ctx, m, plan, mode, trace) : agpu_pk_launch(ctx, m, plan, mode, trace);
}
// Reads and clears the error word (synchronises the stream).  0 = no error.
int32_t agpu_pk_take_error(agpu_ctx *ctx, const PkPlan &plan, unsigned int *err_out);
