// Internal launchers of elementwise.hip used by the model driver.
#pragma once
#include "agpu_internal.h"

// Token feed fused into the arg-max: the winner of row b becomes cur_tok[b] and is recorded at
// out_tok[*step_dev * rows + b]; with bump_counters (single row only) the position and step
// counters advance in the same launch.
struct ArgmaxAdvance {
    uint32_t *cur_tok;
    uint32_t *out_tok;
    int *pos_dev;
    int *step_dev;
    int delta;
    int out_capacity;
    int bump_counters;
};

int32_t agpu_argmax_rows_strided(agpu_ctx *ctx, const float *x, uint32_t *idx_out, int rows, int cols, int row_stride,
                                 int last_index, const ArgmaxAdvance *adv, float *conf_out = nullptr);
int32_t agpu_layer_norm_impl(agpu_ctx *ctx, const float *x, const float *gamma, const float *beta, float *y,
                             int rows, int d, float eps);
