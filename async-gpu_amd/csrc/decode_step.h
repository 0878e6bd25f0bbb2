// One-launch-per-token decode step for a single sequence (the B = 1 greedy loop of generate_cached,
// nn/models/gpt2.rs:760-780): host-side plan and launcher of decode_xcd.hip.
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
    void *stages_dev = nullptr;   // stage tables, one per XCD
    int n_stages = 0;
    // Every activation vector of one step, in floats: two sets (steps use them in turn) of eight mirrors (one per XCD),
    // two sets of partial sums, then the arg-max candidates
    unsigned long long *arena = nullptr;
    // The partial sums and the candidates, which cross XCDs through memory, live in device memory that no cache level
    // keeps (a hop through it is about 0.2 us shorter); `arena` holds the mirrors only.  Such memory is never freed
    // while the process runs: a plan returns it to a pool that later plans draw from.
    float *xmem = nullptr;
    size_t xmem_bytes = 0;
    size_t arena_elems = 0;  // floats of one mirror
    size_t parts_elems = 0;  // floats of one set of partial sums
    size_t cand_off = 0;     // where the arg-max candidates start (floats)
    unsigned int *state = nullptr;  // [0] number of the last finished step, [1] error word (0 = none), [2] workgroups started, [8..15] XCD of each class
    int grid = 0;
    int nr = 0;           // relay workgroups per XCD
    int att_per_xcd = 0;  // workgroups per XCD that only do attention
    int smax = 1;         // key ranges per head at most
    int lin_per_xcd = 0;  // Linear workgroups per XCD
    size_t lds_bytes = 0;
    int kmax = 0;         // longest input vector of a stage: sizes the staging buffers
    int head_slots = 0;   // how many of a workgroup's head slots wait in LDS when the head stage begins
    int head_tpc = 0;     // tiles per chunk of the head stage
    int spin_limit = 0;   // poll rounds a wait inside the kernel may take; 0 = the default
    int touch_dist = 0;   // how many exchanges ahead the relays touch the weights (0: not at all)
    float *ln_fold = nullptr;  // the LayerNorms folded into the Linears behind them (A_n, B_n per column)
};

// Whether the one-launch step can run this model (int4 head, head_dim 64, group 32, d <= 2048, vocabulary below 65536,
// a device of eight XCDs with 32 CUs each).
bool agpu_step_supported(const agpu_ctx *ctx, const PkModel &m);
int32_t agpu_step_plan_build(agpu_ctx *ctx, const PkModel &m, PkPlan *plan);
void agpu_step_plan_free(PkPlan *plan);
// One decode step on the context's stream.  mode 0: the real step; mode 1: the same stage chain with empty bodies
// (every wait and every store, no weights, no arithmetic): the latency floor of the chain.
int32_t agpu_step_launch(agpu_ctx *ctx, const PkModel &m, const PkPlan &plan, int mode, unsigned long long *trace = nullptr);
// Reads and clears the error word (synchronises the stream).  0 = no error.
int32_t agpu_step_take_error(agpu_ctx *ctx, const PkPlan &plan, unsigned int *err_out);
// Every place of the activation arena back to "not written yet" (after a step that gave up).
int32_t agpu_step_reset(agpu_ctx *ctx, const PkPlan &plan);
