/*
 * agpu_oracle.c — CPU restatement of async_gpu's quantized GPT-2 inference path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker and the timed CPU
 * baseline.  Nothing that ships (the HIP library, its host layer, the Python
 * binding) links, imports or calls it; only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg do.
 *
 * Every function cites the reference file:line (paths relative to the reference
 * checkout) whose arithmetic it restates.  Compile with -ffp-contract=off: the
 * reference's Rust never fuses a*b+c unless it asks for fma explicitly.
 *
 * Pinning status (what fixes each function besides its own formula) is listed
 * in oracle/README.md; tests/test_oracle_*.py hold the checks.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* threads                                                                  */
/* ------------------------------------------------------------------------ */

/* The reference CPU path is single threaded (nn/cpu_ref.rs, tests_inference.rs
 * have no threading).  Threads here only split independent output elements, so
 * every result is bit-identical for any thread count. */
ORC_API int orc_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
    return omp_get_max_threads();
#else
    (void)n;
    return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* int4 quantizer, unpack, dequantize                                       */
/* ------------------------------------------------------------------------ */

/* Rust f32::round: half away from zero.  roundf has exactly that rule. */
static inline float round_half_away(float v) { return roundf(v); }
/* numpy.round: half to even.  rintf under the default rounding mode. */
static inline float round_half_even(float v) { return rintf(v); }

static inline int clamp_i(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* nn/ops/quantize.rs:158-162 — nibble `index` of a word, bias 8 removed. */
ORC_API int orc_unpack_int4(uint32_t word, int index) {
    return (int)((word >> (index * 4)) & 0xFu) - 8;
}

/*
 * nn/ops/quantize.rs:102-153 (mode 0) and scripts/quantize_gpt2_int4.py:21-62
 * (mode 1).  weight_t is [K,N] row-major.  packed is [K/8,N], scales is
 * [ceil(K/g),N].
 *   mode 0: scale = max_abs/7 (1.0 when max_abs < 1e-12), q = round_half_away(v * (1/scale))
 *   mode 1: same scale rule in float32, q = round_half_even(v / scale)
 * both clamp to [-8,7] and store q+8 in nibble k%8 of word [k/8, n].
 * Returns 0, or -1 when K % 8 != 0 (the reference asserts, quantize.rs:109).
 */
ORC_API int orc_quantize_weight_int4(const float *weight_t, int K, int N, int group, int mode,
                                     uint32_t *packed, float *scales) {
    if (K % 8 != 0 || group <= 0) return -1;
    const int n_groups = (K + group - 1) / group;
    const int k_packed = K / 8;
#pragma omp parallel for schedule(static)
    for (int col = 0; col < N; ++col) {
        for (int g = 0; g < n_groups; ++g) {
            const int k0 = g * group;
            const int k1 = (k0 + group < K) ? k0 + group : K;
            float max_abs = 0.0f;
            for (int k = k0; k < k1; ++k) {
                float a = fabsf(weight_t[(size_t)k * N + col]);
                if (a > max_abs) max_abs = a;
            }
            scales[(size_t)g * N + col] = (max_abs < 1e-12f) ? 1.0f : max_abs / 7.0f;
        }
        for (int kp = 0; kp < k_packed; ++kp) {
            uint32_t word = 0;
            for (int bit = 0; bit < 8; ++bit) {
                const int k = kp * 8 + bit;
                const float v = weight_t[(size_t)k * N + col];
                const float scale = scales[(size_t)(k / group) * N + col];
                float r;
                if (mode == 0) {
                    const float inv = 1.0f / scale;
                    r = round_half_away(v * inv);
                } else {
                    r = round_half_even(v / scale);
                }
                const int q = clamp_i((int)r, -8, 7);
                word |= ((uint32_t)(q + 8) & 0xFu) << (bit * 4);
            }
            packed[(size_t)kp * N + col] = word;
        }
    }
    return 0;
}

/* nn/ops/quantize.rs:56-89 — the flat per-vector form (groups along the vector). */
ORC_API int orc_quantize_int4_per_group(const float *data, int len, int group, uint32_t *packed,
                                        float *scales) {
    if (len % 8 != 0 || group <= 0) return -1;
    const int n_groups = (len + group - 1) / group;
    memset(packed, 0, (size_t)(len / 8) * sizeof(uint32_t));
    for (int g = 0; g < n_groups; ++g) {
        const int s = g * group;
        const int e = (s + group < len) ? s + group : len;
        float max_abs = 0.0f;
        for (int i = s; i < e; ++i) {
            float a = fabsf(data[i]);
            if (a > max_abs) max_abs = a;
        }
        const float scale = (max_abs < 1e-12f) ? 1.0f : max_abs / 7.0f;
        scales[g] = scale;
        const float inv = 1.0f / scale;
        for (int i = s; i < e; ++i) {
            const int q = clamp_i((int)round_half_away(data[i] * inv), -8, 7);
            packed[i / 8] |= ((uint32_t)(q + 8) & 0xFu) << ((i % 8) * 4);
        }
    }
    return 0;
}

/* compute_gemm.rs:2882-2886 — w = (float)(nibble-8) * scale[k/g, n]; one IEEE multiply. */
ORC_API void orc_int4_dequantize(const uint32_t *packed, const float *scales, int K, int N, int group,
                                 float *w_out) {
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k) {
        const int kp = k / 8, bit = k % 8, g = k / group;
        for (int n = 0; n < N; ++n) {
            const int q = orc_unpack_int4(packed[(size_t)kp * N + n], bit);
            w_out[(size_t)k * N + n] = (float)q * scales[(size_t)g * N + n];
        }
    }
}

/* ------------------------------------------------------------------------ */
/* int4 dequant GEMM                                                        */
/* ------------------------------------------------------------------------ */

/*
 * compute_gemm.rs:2868-2900 restated literally in fp32: for each C[row,col],
 * acc = fma(a[row,k], (float)(nib-8)*scale, acc) for k ascending.  Optional
 * bias added afterwards as compute_transformer.rs:1354-1387 does (one f32 add).
 */
ORC_API void orc_int4_gemm_f32(const float *a, const uint32_t *packed, const float *scales,
                               const float *bias, float *c, int M, int N, int K, int group) {
#pragma omp parallel for schedule(static)
    for (int col = 0; col < N; ++col) {
        for (int row = 0; row < M; ++row) {
            float acc = 0.0f;
            for (int kp = 0; kp < K / 8; ++kp) {
                const uint32_t word = packed[(size_t)kp * N + col];
                for (int bit = 0; bit < 8; ++bit) {
                    const int k = kp * 8 + bit;
                    const float w = (float)((int)((word >> (bit * 4)) & 0xFu) - 8) *
                                    scales[(size_t)(k / group) * N + col];
                    acc = fmaf(a[(size_t)row * K + k], w, acc);
                }
            }
            if (bias) acc += bias[col];
            c[(size_t)row * N + col] = acc;
        }
    }
}

/*
 * Same product with f64 accumulation in the style of cpu_matmul_f64
 * (nn/cpu_ref.rs:9-21): sum += (double)a * (double)w_f32, k ascending, result
 * rounded to f32 once; bias added in f64 before the rounding.
 */
ORC_API void orc_int4_gemm_f64(const float *a, const uint32_t *packed, const float *scales,
                               const float *bias, float *c, int M, int N, int K, int group) {
#pragma omp parallel for schedule(static)
    for (int col = 0; col < N; ++col) {
        for (int row = 0; row < M; ++row) {
            double acc = 0.0;
            for (int kp = 0; kp < K / 8; ++kp) {
                const uint32_t word = packed[(size_t)kp * N + col];
                for (int bit = 0; bit < 8; ++bit) {
                    const int k = kp * 8 + bit;
                    const float w = (float)((int)((word >> (bit * 4)) & 0xFu) - 8) *
                                    scales[(size_t)(k / group) * N + col];
                    acc += (double)a[(size_t)row * K + k] * (double)w;
                }
            }
            if (bias) acc += (double)bias[col];
            c[(size_t)row * N + col] = (float)acc;
        }
    }
}

/* nn/cpu_ref.rs:9-21 — C = A[M,K] * B[K,N], f64 accumulate, f32 result. */
ORC_API void orc_matmul_f64(const float *a, const float *b, float *c, int M, int K, int N) {
#pragma omp parallel for schedule(static)
    for (int j = 0; j < N; ++j) {
        for (int i = 0; i < M; ++i) {
            double s = 0.0;
            for (int p = 0; p < K; ++p) s += (double)a[(size_t)i * K + p] * (double)b[(size_t)p * N + j];
            c[(size_t)i * N + j] = (float)s;
        }
    }
}

/* compute_transformer.rs:1354-1387 — data[i] += bias[i % n_cols]. */
ORC_API void orc_bias_add(float *data, const float *bias, int rows, int n_cols) {
    for (int r = 0; r < rows; ++r)
        for (int j = 0; j < n_cols; ++j) data[(size_t)r * n_cols + j] += bias[j];
}

/* compute_transformer.rs:1544-1606 — a += b. */
ORC_API void orc_add_inplace(float *a, const float *b, size_t n) {
    for (size_t i = 0; i < n; ++i) a[i] += b[i];
}

/* ------------------------------------------------------------------------ */
/* LayerNorm, GELU, softmax                                                 */
/* ------------------------------------------------------------------------ */

/* nn/cpu_ref.rs:27-54 — f64 two-pass mean / population variance, eps inside sqrt. */
ORC_API void orc_layer_norm_f64(const float *x, const float *gamma, const float *beta, float *y,
                                int rows, int d, float eps) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < rows; ++i) {
        const float *row = x + (size_t)i * d;
        double mean = 0.0;
        for (int j = 0; j < d; ++j) mean += (double)row[j];
        mean /= (double)d;
        double var = 0.0;
        for (int j = 0; j < d; ++j) {
            double df = (double)row[j] - mean;
            var += df * df;
        }
        var /= (double)d;
        const double inv_std = 1.0 / sqrt(var + (double)eps);
        for (int j = 0; j < d; ++j) {
            double nrm = ((double)row[j] - mean) * inv_std;
            y[(size_t)i * d + j] = (float)(nrm * (double)gamma[j] + (double)beta[j]);
        }
    }
}

/* tests_transformer.rs:84-96 — the fp32 two-pass form the kernel test compares with. */
ORC_API void orc_layer_norm_f32(const float *x, const float *gamma, const float *beta, float *y,
                                int rows, int d, float eps) {
    for (int i = 0; i < rows; ++i) {
        const float *row = x + (size_t)i * d;
        float sum = 0.0f;
        for (int j = 0; j < d; ++j) sum += row[j];
        const float mean = sum / (float)d;
        float vs = 0.0f;
        for (int j = 0; j < d; ++j) vs += (row[j] - mean) * (row[j] - mean);
        const float var = vs / (float)d;
        const float inv_std = 1.0f / sqrtf(var + eps);
        for (int j = 0; j < d; ++j) y[(size_t)i * d + j] = gamma[j] * (row[j] - mean) * inv_std + beta[j];
    }
}

/* nn/ops/norm.rs:88-237,248-400 — sum = a + b (f32 add), norm = LN(sum). */
ORC_API void orc_add_layer_norm_dual_f64(const float *a, const float *b, const float *gamma,
                                         const float *beta, float *sum_out, float *norm_out,
                                         int rows, int d, float eps) {
    for (size_t i = 0; i < (size_t)rows * d; ++i) sum_out[i] = a[i] + b[i];
    orc_layer_norm_f64(sum_out, gamma, beta, norm_out, rows, d, eps);
}

/* tests_inference.rs:3680-3685 — tanh GELU in f64. */
static inline double gelu_tanh_f64(double x) {
    const double c = 0.7978845608028654, k = 0.044715;
    const double inner = c * (x + k * x * x * x);
    return x * 0.5 * (1.0 + tanh(inner));
}

/* mode 0: tanh form (tests_inference.rs:3680-3685, nn/test_utils.rs:359-367), f64 math.
 * mode 1: x * sigmoid(1.702 x) (compute_transformer.rs:1468-1531), f64 math. */
ORC_API void orc_gelu(const float *x, float *y, size_t n, int mode) {
    for (size_t i = 0; i < n; ++i) {
        const double v = (double)x[i];
        y[i] = (float)(mode == 0 ? gelu_tanh_f64(v) : v / (1.0 + exp(-1.702 * v)));
    }
}

/* tests_transformer.rs:169-177 — the fp32 tanh form (0.797_884_6 constant). */
ORC_API void orc_gelu_tanh_f32(const float *x, float *y, size_t n) {
    const float c = 0.7978846f, k = 0.044715f;
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        const float inner = c * (v + k * v * v * v);
        y[i] = v * 0.5f * (1.0f + tanhf(inner));
    }
}

/* nn/cpu_ref.rs:111-125 — row softmax, f64 math, -inf entries give 0. */
ORC_API void orc_softmax_f64(const float *x, float *y, int rows, int cols) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < rows; ++i) {
        const float *row = x + (size_t)i * cols;
        double mx = -INFINITY;
        for (int j = 0; j < cols; ++j)
            if ((double)row[j] > mx) mx = (double)row[j];
        double s = 0.0;
        for (int j = 0; j < cols; ++j) s += exp((double)row[j] - mx);
        for (int j = 0; j < cols; ++j) y[(size_t)i * cols + j] = (float)(exp((double)row[j] - mx) / s);
    }
}

/* ------------------------------------------------------------------------ */
/* layout kernels                                                           */
/* ------------------------------------------------------------------------ */

/* compute_transformer.rs:1620-1660 — [seq,3d] -> Q,K,V [H,seq,dh]; Q cols [0,d), K [d,2d), V [2d,3d). */
ORC_API void orc_split_qkv(const float *qkv, float *q, float *k, float *v, int seq, int n_heads, int d_head) {
    const int d = n_heads * d_head;
    for (int h = 0; h < n_heads; ++h)
        for (int s = 0; s < seq; ++s)
            for (int e = 0; e < d_head; ++e) {
                const size_t o = ((size_t)h * seq + s) * d_head + e;
                const size_t i = (size_t)s * 3 * d + (size_t)h * d_head + e;
                q[o] = qkv[i];
                k[o] = qkv[i + d];
                v[o] = qkv[i + 2 * d];
            }
}

/* compute_transformer.rs:1671-1703 — [H,seq,dh] -> [seq, H*dh]. */
ORC_API void orc_concat_heads(const float *in, float *out, int seq, int n_heads, int d_head) {
    const int d = n_heads * d_head;
    for (int h = 0; h < n_heads; ++h)
        for (int s = 0; s < seq; ++s)
            for (int e = 0; e < d_head; ++e)
                out[(size_t)s * d + h * d_head + e] = in[((size_t)h * seq + s) * d_head + e];
}

/* compute_transformer.rs:1303-1344 with the offset of layers/embedding.rs:59-93 —
 * out[p,:] = wte[tok[p],:] + wpe[p+pos_offset,:] (one f32 add). */
ORC_API void orc_embedding(const uint32_t *tokens, const float *wte, const float *wpe, float *out,
                           int seq, int d, int pos_offset) {
    for (int p = 0; p < seq; ++p)
        for (int j = 0; j < d; ++j)
            out[(size_t)p * d + j] = wte[(size_t)tokens[p] * d + j] + wpe[(size_t)(p + pos_offset) * d + j];
}

/* compute_transformer.rs:1777-1812 — row 0 of src [H, src_stride, dh] -> cache[h, write_pos, :]. */
ORC_API void orc_kv_append(const float *src, float *cache, int n_heads, int src_stride, int max_seq,
                           int write_pos, int d_head) {
    for (int h = 0; h < n_heads; ++h)
        for (int e = 0; e < d_head; ++e)
            cache[((size_t)h * max_seq + write_pos) * d_head + e] = src[(size_t)h * src_stride * d_head + e];
}

/* ------------------------------------------------------------------------ */
/* attention                                                                */
/* ------------------------------------------------------------------------ */

/*
 * Multi-head attention with a KV cache, f64 math, following nn/cpu_ref.rs:130-165
 * (scores rounded to f32, softmax in f64 rounded to f32, P*V in f64) and the
 * mask / stride rules of compute_transformer.rs:1076-1112,1189:
 *   q   [H, q_len, dh], k/v [H, kv_stride, dh] (kv_len rows used), o [H, q_len, dh]
 *   key j is visible to query row i iff !causal or j <= q_offset + i.
 * With q_len == kv_len == kv_stride and q_offset == 0 this is cpu_attention_f64
 * applied per head (prefill).
 */
ORC_API void orc_attention_kv_f64(const float *q, const float *k, const float *v, float *o, int n_heads,
                                  int q_len, int kv_len, int q_offset, int kv_stride, int d_head,
                                  int causal) {
    const double scale = 1.0 / sqrt((double)d_head);
#pragma omp parallel for collapse(2) schedule(dynamic, 8)
    for (int h = 0; h < n_heads; ++h) {
        for (int i = 0; i < q_len; ++i) {
            float *scores = (float *)malloc(sizeof(float) * (size_t)kv_len);
            float *probs = (float *)malloc(sizeof(float) * (size_t)kv_len);
            const float *qi = q + ((size_t)h * q_len + i) * d_head;
            for (int j = 0; j < kv_len; ++j) {
                if (causal && j > q_offset + i) {
                    scores[j] = -INFINITY;
                } else {
                    const float *kj = k + ((size_t)h * kv_stride + j) * d_head;
                    double dot = 0.0;
                    for (int p = 0; p < d_head; ++p) dot += (double)qi[p] * (double)kj[p];
                    scores[j] = (float)(dot * scale);
                }
            }
            orc_softmax_f64(scores, probs, 1, kv_len);
            for (int e = 0; e < d_head; ++e) {
                double s = 0.0;
                for (int j = 0; j < kv_len; ++j)
                    s += (double)probs[j] * (double)v[((size_t)h * kv_stride + j) * d_head + e];
                o[((size_t)h * q_len + i) * d_head + e] = (float)s;
            }
            free(scores);
            free(probs);
        }
    }
}

/* tests_transformer.rs:512-560 — the naive all-fp32 loop the kernel tests compare with
 * (mask value -1e38, expf, probabilities normalised before P*V). */
ORC_API void orc_attention_f32_naive(const float *q, const float *k, const float *v, float *o, int n_heads,
                                     int seq, int d_head, int causal) {
    const float scale = 1.0f / sqrtf((float)d_head);
#pragma omp parallel for collapse(2) schedule(dynamic, 8)
    for (int h = 0; h < n_heads; ++h) {
        for (int i = 0; i < seq; ++i) {
            float *sc = (float *)malloc(sizeof(float) * (size_t)seq);
            const size_t base = (size_t)h * seq * d_head;
            for (int j = 0; j < seq; ++j) {
                if (causal && j > i) {
                    sc[j] = -1.0e38f;
                } else {
                    float dot = 0.0f;
                    for (int p = 0; p < d_head; ++p) dot += q[base + (size_t)i * d_head + p] * k[base + (size_t)j * d_head + p];
                    sc[j] = dot * scale;
                }
            }
            float mx = -INFINITY;
            for (int j = 0; j < seq; ++j)
                if (sc[j] > mx) mx = sc[j];
            float sum = 0.0f;
            for (int j = 0; j < seq; ++j) {
                sc[j] = expf(sc[j] - mx);
                sum += sc[j];
            }
            for (int j = 0; j < seq; ++j) sc[j] = sc[j] / sum;
            for (int e = 0; e < d_head; ++e) {
                float acc = 0.0f;
                for (int j = 0; j < seq; ++j) acc += sc[j] * v[base + (size_t)j * d_head + e];
                o[base + (size_t)i * d_head + e] = acc;
            }
            free(sc);
        }
    }
}

/* gpt2.rs:991-997 (mode 1: last maximal index, Iterator::max_by) and
 * tests_inference.rs:4504-4515 (mode 0: first maximal index, strict >). */
ORC_API uint32_t orc_argmax(const float *x, int n, int mode) {
    int best = 0;
    float bv = x[0];
    for (int i = 1; i < n; ++i) {
        if (mode == 0 ? (x[i] > bv) : (x[i] >= bv)) {
            bv = x[i];
            best = i;
        }
    }
    return (uint32_t)best;
}

/* ------------------------------------------------------------------------ */
/* full GPT-2 forward in f64 (tests_inference.rs:3577-4554)                 */
/* ------------------------------------------------------------------------ */

typedef struct {
    int K, N, group;
    float *w;    /* dequantized [K,N], (float)q*scale as the kernel forms it */
    float *bias; /* [N] or NULL */
} orc_linear;

typedef struct {
    float *ln1_g, *ln1_b, *ln2_g, *ln2_b;
    orc_linear qkv, proj, fc, fc_proj;
} orc_block;

typedef struct orc_gpt2 {
    int n_layer, n_embd, n_head, vocab, n_positions, d_head, d_ffn;
    double eps;
    float *wte, *wpe, *lnf_g, *lnf_b;
    orc_block *blocks;
    orc_linear lm_head; /* int4 tied head (K=n_embd, N=vocab) when lm_head.w != NULL */
    /* KV cache: [layer][head][n_positions][d_head] f64, kv_len rows valid */
    double *kc, *vc;
    int kv_len;
} orc_gpt2;

static float *dup_f32(const float *src, size_t n) {
    if (!src) return NULL;
    float *p = (float *)malloc(n * sizeof(float));
    memcpy(p, src, n * sizeof(float));
    return p;
}

ORC_API orc_gpt2 *orc_gpt2_create(int n_layer, int n_embd, int n_head, int vocab, int n_positions,
                                  float eps) {
    orc_gpt2 *m = (orc_gpt2 *)calloc(1, sizeof(orc_gpt2));
    m->n_layer = n_layer;
    m->n_embd = n_embd;
    m->n_head = n_head;
    m->vocab = vocab;
    m->n_positions = n_positions;
    m->d_head = n_embd / n_head;
    m->d_ffn = 4 * n_embd; /* gpt2.rs:90-92 */
    m->eps = (double)eps;
    m->blocks = (orc_block *)calloc((size_t)n_layer, sizeof(orc_block));
    return m;
}

static void free_linear(orc_linear *l) {
    free(l->w);
    free(l->bias);
    l->w = NULL;
    l->bias = NULL;
}

ORC_API void orc_gpt2_destroy(orc_gpt2 *m) {
    if (!m) return;
    for (int i = 0; i < m->n_layer; ++i) {
        orc_block *b = &m->blocks[i];
        free(b->ln1_g); free(b->ln1_b); free(b->ln2_g); free(b->ln2_b);
        free_linear(&b->qkv); free_linear(&b->proj); free_linear(&b->fc); free_linear(&b->fc_proj);
    }
    free(m->blocks);
    free(m->wte); free(m->wpe); free(m->lnf_g); free(m->lnf_b);
    free_linear(&m->lm_head);
    free(m->kc); free(m->vc);
    free(m);
}

ORC_API void orc_gpt2_set_embeddings(orc_gpt2 *m, const float *wte, const float *wpe, const float *lnf_g,
                                     const float *lnf_b) {
    m->wte = dup_f32(wte, (size_t)m->vocab * m->n_embd);
    m->wpe = dup_f32(wpe, (size_t)m->n_positions * m->n_embd);
    m->lnf_g = dup_f32(lnf_g, (size_t)m->n_embd);
    m->lnf_b = dup_f32(lnf_b, (size_t)m->n_embd);
}

ORC_API void orc_gpt2_set_layer_norms(orc_gpt2 *m, int layer, const float *ln1_g, const float *ln1_b,
                                      const float *ln2_g, const float *ln2_b) {
    orc_block *b = &m->blocks[layer];
    b->ln1_g = dup_f32(ln1_g, (size_t)m->n_embd);
    b->ln1_b = dup_f32(ln1_b, (size_t)m->n_embd);
    b->ln2_g = dup_f32(ln2_g, (size_t)m->n_embd);
    b->ln2_b = dup_f32(ln2_b, (size_t)m->n_embd);
}

/* which: 0 qkv, 1 attn proj, 2 mlp fc, 3 mlp proj; layer == -1 selects the int4 LM head. */
ORC_API int orc_gpt2_set_int4_linear(orc_gpt2 *m, int layer, int which, const uint32_t *packed,
                                     const float *scales, const float *bias, int K, int N, int group) {
    orc_linear *l;
    if (layer < 0) l = &m->lm_head;
    else {
        orc_block *b = &m->blocks[layer];
        l = which == 0 ? &b->qkv : which == 1 ? &b->proj : which == 2 ? &b->fc : &b->fc_proj;
    }
    free_linear(l);
    l->K = K; l->N = N; l->group = group;
    l->w = (float *)malloc((size_t)K * N * sizeof(float));
    orc_int4_dequantize(packed, scales, K, N, group, l->w);
    l->bias = dup_f32(bias, (size_t)N);
    return 0;
}

/* tests_inference.rs:3655-3677 — C = A*B (+bias) in f64, sum over p ascending.
 * Loop order (i,p,j) keeps each output's summation order and lets j vectorise. */
static void linear_f64(const double *a, const orc_linear *l, double *c, int M) {
    const int K = l->K, N = l->N;
#pragma omp parallel
    {
#ifdef _OPENMP
        const int nt = omp_get_num_threads(), t = omp_get_thread_num();
#else
        const int nt = 1, t = 0;
#endif
        const int chunk = (N + nt - 1) / nt;
        const int j0 = t * chunk, j1 = (j0 + chunk < N) ? j0 + chunk : N;
        for (int i = 0; i < M && j0 < j1; ++i) {
            double *ci = c + (size_t)i * N;
            for (int j = j0; j < j1; ++j) ci[j] = 0.0;
            for (int p = 0; p < K; ++p) {
                const double av = a[(size_t)i * K + p];
                const float *bp = l->w + (size_t)p * N;
                for (int j = j0; j < j1; ++j) ci[j] += av * (double)bp[j];
            }
            if (l->bias)
                for (int j = j0; j < j1; ++j) ci[j] += (double)l->bias[j];
        }
    }
}

/* tests_inference.rs:3639-3653 */
static void layer_norm_d(const double *x, const float *g, const float *b, double *y, int rows, int d,
                         double eps) {
    for (int s = 0; s < rows; ++s) {
        const double *row = x + (size_t)s * d;
        double mean = 0.0;
        for (int j = 0; j < d; ++j) mean += row[j];
        mean /= (double)d;
        double var = 0.0;
        for (int j = 0; j < d; ++j) var += (row[j] - mean) * (row[j] - mean);
        var /= (double)d;
        const double inv_std = 1.0 / sqrt(var + eps);
        for (int j = 0; j < d; ++j) y[(size_t)s * d + j] = (row[j] - mean) * inv_std * (double)g[j] + (double)b[j];
    }
}

ORC_API void orc_gpt2_reset_cache(orc_gpt2 *m) { m->kv_len = 0; }
ORC_API int orc_gpt2_cache_len(const orc_gpt2 *m) { return m->kv_len; }

typedef struct {
    double *hid, *ln, *qkv, *att, *tmp, *ffn;
} orc_work;

static void work_alloc(const orc_gpt2 *m, orc_work *w, int new_len) {
    const size_t d = (size_t)m->n_embd, n = (size_t)new_len;
    w->hid = (double *)malloc(sizeof(double) * n * d);
    w->ln = (double *)malloc(sizeof(double) * n * d);
    w->qkv = (double *)malloc(sizeof(double) * n * 3 * d);
    w->att = (double *)malloc(sizeof(double) * n * d);
    w->tmp = (double *)malloc(sizeof(double) * n * d);
    w->ffn = (double *)malloc(sizeof(double) * n * (size_t)m->d_ffn);
}

static void work_free(orc_work *w) {
    free(w->hid); free(w->ln); free(w->qkv); free(w->att); free(w->tmp); free(w->ffn);
}

static void cache_alloc(orc_gpt2 *m) {
    if (m->kc) return;
    const size_t n = (size_t)m->n_layer * m->n_head * m->n_positions * m->d_head;
    m->kc = (double *)malloc(sizeof(double) * n);
    m->vc = (double *)malloc(sizeof(double) * n);
}

/* wte[token] + wpe[position] (compute_transformer.rs:1320-1329) */
static void embed_rows(const orc_gpt2 *m, const uint32_t *tokens, int new_len, int pos0, double *hid) {
    const int d = m->n_embd;
    for (int p = 0; p < new_len; ++p)
        for (int j = 0; j < d; ++j)
            hid[(size_t)p * d + j] = (double)m->wte[(size_t)tokens[p] * d + j] + (double)m->wpe[(size_t)(pos0 + p) * d + j];
}

/* One pre-LN block on rows at positions pos0.. (tests_inference.rs:3746-3850): the K and V rows go into the
 * cache of layer L, attention runs over keys 0..pos0+s for row s. */
static void run_block(orc_gpt2 *m, int L, orc_work *w, int new_len, int pos0) {
    const int d = m->n_embd, H = m->n_head, dh = m->d_head, ff = m->d_ffn, P = m->n_positions;
    double *hid = w->hid, *ln = w->ln, *qkv = w->qkv, *att = w->att, *tmp = w->tmp, *ffn = w->ffn;
    const double scale = 1.0 / sqrt((double)dh);
    const orc_block *b = &m->blocks[L];
    layer_norm_d(hid, b->ln1_g, b->ln1_b, ln, new_len, d, m->eps);
    linear_f64(ln, &b->qkv, qkv, new_len);
    double *kc = m->kc + (size_t)L * H * P * dh, *vc = m->vc + (size_t)L * H * P * dh;
    for (int h = 0; h < H; ++h)
        for (int s = 0; s < new_len; ++s)
            for (int e = 0; e < dh; ++e) {
                kc[((size_t)h * P + pos0 + s) * dh + e] = qkv[(size_t)s * 3 * d + d + h * dh + e];
                vc[((size_t)h * P + pos0 + s) * dh + e] = qkv[(size_t)s * 3 * d + 2 * d + h * dh + e];
            }
#pragma omp parallel for collapse(2) schedule(dynamic, 4)
    for (int h = 0; h < H; ++h) {
        for (int s = 0; s < new_len; ++s) {
            const int vis = pos0 + s + 1; /* keys 0..pos0+s */
            double *sc = (double *)malloc(sizeof(double) * (size_t)vis);
            const double *qv = qkv + (size_t)s * 3 * d + h * dh;
            double mx = -INFINITY;
            for (int j = 0; j < vis; ++j) {
                const double *kj = kc + ((size_t)h * P + j) * dh;
                double dot = 0.0;
                for (int e = 0; e < dh; ++e) dot += qv[e] * kj[e];
                sc[j] = dot * scale;
                if (sc[j] > mx) mx = sc[j];
            }
            double sum = 0.0;
            for (int j = 0; j < vis; ++j) {
                sc[j] = exp(sc[j] - mx);
                sum += sc[j];
            }
            for (int j = 0; j < vis; ++j) sc[j] /= sum;
            for (int e = 0; e < dh; ++e) {
                double acc = 0.0;
                for (int j = 0; j < vis; ++j) acc += sc[j] * vc[((size_t)h * P + j) * dh + e];
                att[(size_t)s * d + h * dh + e] = acc;
            }
            free(sc);
        }
    }
    linear_f64(att, &b->proj, tmp, new_len);
    for (size_t i = 0; i < (size_t)new_len * d; ++i) hid[i] += tmp[i];
    layer_norm_d(hid, b->ln2_g, b->ln2_b, ln, new_len, d, m->eps);
    linear_f64(ln, &b->fc, ffn, new_len);
    for (size_t i = 0; i < (size_t)new_len * ff; ++i) ffn[i] = gelu_tanh_f64(ffn[i]);
    linear_f64(ffn, &b->fc_proj, tmp, new_len);
    for (size_t i = 0; i < (size_t)new_len * d; ++i) hid[i] += tmp[i];
}

/* final LayerNorm of hid into w->ln, then logits of rows r0..r0+nr-1.  LM head: the int4 head if one was set,
 * else an f64 dot with the wte rows (tests_inference.rs:4504-4510). */
static void run_head(const orc_gpt2 *m, orc_work *w, int new_len, int r0, int nr, double *logits_out) {
    const int d = m->n_embd;
    layer_norm_d(w->hid, m->lnf_g, m->lnf_b, w->ln, new_len, d, m->eps);
    if (!logits_out) return;
    if (m->lm_head.w) {
        linear_f64(w->ln + (size_t)r0 * d, &m->lm_head, logits_out, nr);
    } else {
#pragma omp parallel for schedule(static)
        for (int v = 0; v < m->vocab; ++v)
            for (int r = 0; r < nr; ++r) {
                const double *hv = w->ln + (size_t)(r0 + r) * d;
                double dot = 0.0;
                for (int j = 0; j < d; ++j) dot += hv[j] * (double)m->wte[(size_t)v * d + j];
                logits_out[(size_t)r * m->vocab + v] = dot;
            }
    }
}

/*
 * One forward over `new_len` tokens at positions kv_len .. kv_len+new_len-1,
 * attending to everything cached before them (gpt2.rs:712-734 control flow,
 * tests_inference.rs:3746-3850 arithmetic).  With an empty cache this is the
 * reference's full uncached forward.  Writes f64 logits of the rows asked for:
 *   logits_rows == 0: last row only -> logits_out[vocab]
 *   logits_rows == 1: all rows      -> logits_out[new_len, vocab]
 * hidden_out (optional, [new_len, n_embd]) receives the final-LN output.
 */
ORC_API int orc_gpt2_forward(orc_gpt2 *m, const uint32_t *tokens, int new_len, int logits_rows,
                             double *logits_out, double *hidden_out) {
    const int pos0 = m->kv_len, kv_total = pos0 + new_len;
    if (kv_total > m->n_positions || new_len <= 0) return -1;
    cache_alloc(m);
    orc_work w;
    work_alloc(m, &w, new_len);
    embed_rows(m, tokens, new_len, pos0, w.hid);
    for (int L = 0; L < m->n_layer; ++L) run_block(m, L, &w, new_len, pos0);
    m->kv_len = kv_total;
    run_head(m, &w, new_len, logits_rows ? 0 : new_len - 1, logits_rows ? new_len : 1, logits_out);
    if (hidden_out) memcpy(hidden_out, w.ln, sizeof(double) * (size_t)new_len * m->n_embd);
    work_free(&w);
    return 0;
}

static uint32_t argmax_first_d(const double *x, int n, double *margin) {
    /* tests_inference.rs:4504-4515: strict '>' keeps the first maximal index. */
    double best = -INFINITY, second = -INFINITY;
    uint32_t bi = 0;
    for (int i = 0; i < n; ++i) {
        if (x[i] > best) {
            second = best;
            best = x[i];
            bi = (uint32_t)i;
        } else if (x[i] > second) {
            second = x[i];
        }
    }
    if (margin) *margin = best - second;
    return bi;
}

/*
 * Greedy generation.  cached == 0 follows tests_inference.rs:4384-4540 (full
 * forward of the whole sequence per new token); cached != 0 follows
 * gpt2.rs:740-783 (prefill, then one token per step).  Both stop before
 * appending token `eos` when eos >= 0 (gpt2.rs:1553-1556); eos < 0 never stops.
 * tokens_out holds prompt + generated ids; margins_out (optional,
 * [max_new_tokens]) gets top1-top2 logit gaps.  Returns the total length.
 */
ORC_API int orc_gpt2_generate(orc_gpt2 *m, const uint32_t *prompt, int prompt_len, int max_new_tokens,
                              int cached, int eos, uint32_t *tokens_out, double *margins_out) {
    double *logits = (double *)malloc(sizeof(double) * (size_t)m->vocab);
    int len = prompt_len;
    memcpy(tokens_out, prompt, sizeof(uint32_t) * (size_t)prompt_len);
    orc_gpt2_reset_cache(m);
    for (int step = 0; step < max_new_tokens; ++step) {
        int rc;
        if (cached) {
            if (step == 0) rc = orc_gpt2_forward(m, tokens_out, len, 0, logits, NULL);
            else rc = orc_gpt2_forward(m, tokens_out + len - 1, 1, 0, logits, NULL);
        } else {
            orc_gpt2_reset_cache(m);
            rc = orc_gpt2_forward(m, tokens_out, len, 0, logits, NULL);
        }
        if (rc != 0) break;
        double margin;
        const uint32_t next = argmax_first_d(logits, m->vocab, &margin);
        if (margins_out) margins_out[step] = margin;
        if (eos >= 0 && next == (uint32_t)eos) break;
        tokens_out[len++] = next;
    }
    free(logits);
    return len;
}

/* ------------------------------------------------------------------------ */
/* sampling: SimpleRng, top_k_sample, generate_cached_sampling               */
/* ------------------------------------------------------------------------ */

/* SimpleRng::new / next_u64 / next_f32 (nn/models/gpt2.rs:1000-1023): xorshift64 with shifts 13, 7, 17,
 * seed 0 replaced by 0xDEADBEEFCAFE1234; next_f32 = (next_u64 >> 40) / 2^24 in [0, 1). */
ORC_API uint64_t orc_simple_rng_new(uint64_t seed) { return seed == 0 ? 0xDEADBEEFCAFE1234ull : seed; }

ORC_API float orc_simple_rng_next_f32(uint64_t *state) {
    uint64_t x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return (float)(x >> 40) / (float)(1ull << 24);
}

typedef struct { float v; int i; } orc_pair;

/* descending by value, ties in index order: what a stable sort of (index, value) pairs by
 * b.partial_cmp(a) gives (gpt2.rs:1036-1038) */
static int orc_pair_cmp(const void *a, const void *b) {
    const orc_pair *x = (const orc_pair *)a, *y = (const orc_pair *)b;
    if (x->v > y->v) return -1;
    if (x->v < y->v) return 1;
    return x->i < y->i ? -1 : (x->i > y->i ? 1 : 0);
}

/*
 * top_k_sample (gpt2.rs:1029-1058): logits / max(temperature, 1e-8) in f32, the k largest in stable
 * descending order, softmax over them in f32 (exp of the difference to the first, sequential sum, one
 * division each), then the first rank whose running sum exceeds r = rng.next_f32(); the last rank if none.
 * top_idx_out / top_val_out (optional, [k]) receive the ranked candidates.
 */
ORC_API uint32_t orc_top_k_sample(const float *logits, int n, int k, float temperature, uint64_t *rng_state,
                                  uint32_t *top_idx_out, float *top_val_out) {
    const float temp = temperature < 1e-8f ? 1e-8f : temperature;
    orc_pair *p = (orc_pair *)malloc(sizeof(orc_pair) * (size_t)n);
    for (int i = 0; i < n; ++i) {
        p[i].v = logits[i] / temp;
        p[i].i = i;
    }
    qsort(p, (size_t)n, sizeof(orc_pair), orc_pair_cmp);
    if (k > n) k = n;
    float *e = (float *)malloc(sizeof(float) * (size_t)k);
    float sum = 0.0f;
    for (int j = 0; j < k; ++j) {
        e[j] = expf(p[j].v - p[0].v);
        sum += e[j];
        if (top_idx_out) top_idx_out[j] = (uint32_t)p[j].i;
        if (top_val_out) top_val_out[j] = p[j].v;
    }
    const float r = orc_simple_rng_next_f32(rng_state);
    uint32_t pick = (uint32_t)p[k - 1].i;
    float cum = 0.0f;
    for (int j = 0; j < k; ++j) {
        cum += e[j] / sum;
        if (r < cum) {
            pick = (uint32_t)p[j].i;
            break;
        }
    }
    free(e);
    free(p);
    return pick;
}

/*
 * generate_cached_sampling (gpt2.rs:931-977): prefill, sample from the last row, then one token per step;
 * a sampled `eos` ends the sequence before it is appended (eos < 0 never stops).  The logits are rounded
 * to f32 before sampling, as the reference samples from f32 logits.  Returns the total length.
 */
ORC_API int orc_gpt2_generate_sampling(orc_gpt2 *m, const uint32_t *prompt, int prompt_len, int max_new_tokens, int top_k,
                                       float temperature, uint64_t *rng_state, int eos, uint32_t *tokens_out) {
    double *logits = (double *)malloc(sizeof(double) * (size_t)m->vocab);
    float *lf = (float *)malloc(sizeof(float) * (size_t)m->vocab);
    int len = prompt_len;
    memcpy(tokens_out, prompt, sizeof(uint32_t) * (size_t)prompt_len);
    orc_gpt2_reset_cache(m);
    for (int step = 0; step < max_new_tokens; ++step) {
        const int rc = step == 0 ? orc_gpt2_forward(m, tokens_out, len, 0, logits, NULL)
                                 : orc_gpt2_forward(m, tokens_out + len - 1, 1, 0, logits, NULL);
        if (rc != 0) break;
        for (int i = 0; i < m->vocab; ++i) lf[i] = (float)logits[i];
        const uint32_t next = orc_top_k_sample(lf, m->vocab, top_k, temperature, rng_state, NULL, NULL);
        if (eos >= 0 && next == (uint32_t)eos) break;
        tokens_out[len++] = next;
    }
    free(lf);
    free(logits);
    return len;
}

/* ------------------------------------------------------------------------ */
/* early exit: softmax_max_prob, forward_early_exit, generate_cached_early_exit */
/* ------------------------------------------------------------------------ */

/* softmax_max_prob (gpt2.rs:983-988): the largest softmax probability of a row, all in f32:
 * max by a sequential fold, sequential sum of exp(x - max), 1 / sum. */
ORC_API float orc_softmax_max_prob(const float *logits, int n) {
    float mx = -INFINITY;
    for (int i = 0; i < n; ++i) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) sum += expf(logits[i] - mx);
    return 1.0f / sum;
}

static float confidence_of(const double *logits, int n, float *scratch) {
    for (int i = 0; i < n; ++i) scratch[i] = (float)logits[i]; /* the reference probes f32 logits */
    return orc_softmax_max_prob(scratch, n);
}

/*
 * forward_early_exit (gpt2.rs:797-830): uncached forward over seq_len tokens; after every block but the last,
 * final LayerNorm + LM head on all rows and the confidence of the last row; the first layer whose confidence
 * reaches the threshold ends the forward.  logits_out [seq_len, vocab] are the logits of the layer that ended it,
 * *layers_used = 1..n_layer.  conf_out (optional, [n_layer - 1]) receives the confidences probed, -1 where no
 * probe ran.
 */
ORC_API int orc_gpt2_forward_early_exit(orc_gpt2 *m, const uint32_t *tokens, int seq_len, float threshold,
                                        double *logits_out, int *layers_used, float *conf_out) {
    if (seq_len <= 0 || seq_len > m->n_positions) return -1;
    cache_alloc(m);
    orc_gpt2_reset_cache(m);
    orc_work w;
    work_alloc(m, &w, seq_len);
    float *lf = (float *)malloc(sizeof(float) * (size_t)m->vocab);
    for (int i = 0; conf_out && i + 1 < m->n_layer; ++i) conf_out[i] = -1.0f;
    embed_rows(m, tokens, seq_len, 0, w.hid);
    int used = m->n_layer;
    for (int L = 0; L < m->n_layer; ++L) {
        run_block(m, L, &w, seq_len, 0);
        if (L + 1 < m->n_layer) {
            run_head(m, &w, seq_len, 0, seq_len, logits_out);
            const float c = confidence_of(logits_out + (size_t)(seq_len - 1) * m->vocab, m->vocab, lf);
            if (conf_out) conf_out[L] = c;
            if (c >= threshold) {
                used = L + 1;
                break;
            }
        }
    }
    if (used == m->n_layer) run_head(m, &w, seq_len, 0, seq_len, logits_out);
    *layers_used = used;
    free(lf);
    work_free(&w);
    return 0;
}

/*
 * generate_cached_early_exit (gpt2.rs:837-922): prefill with every layer, then per token the blocks run until
 * the confidence of an intermediate layer reaches the threshold; the layers skipped get zero K and V rows at
 * that position; the token is the arg-max of the logits of the last layer that ran.  A token equal to `eos`
 * ends the sequence before it is appended (eos < 0 never stops); as in the reference, the first token is produced
 * whatever max_new_tokens is.  layers_out [max(max_new_tokens, 1)] gets the layers used per step, *steps_out their
 * number; conf_out (optional, [max(max_new_tokens, 1), n_layer - 1]) the confidences probed (-1: no probe).
 * Returns the total length.
 */
ORC_API int orc_gpt2_generate_early_exit(orc_gpt2 *m, const uint32_t *prompt, int prompt_len, int max_new_tokens,
                                         float threshold, int eos, uint32_t *tokens_out, int *layers_out, int *steps_out,
                                         float *conf_out) {
    const int nl = m->n_layer, V = m->vocab, H = m->n_head, dh = m->d_head, P = m->n_positions;
    const int rows = max_new_tokens > 1 ? max_new_tokens : 1;
    double *logits = (double *)malloc(sizeof(double) * (size_t)V);
    float *lf = (float *)malloc(sizeof(float) * (size_t)V);
    int len = prompt_len, steps = 0;
    memcpy(tokens_out, prompt, sizeof(uint32_t) * (size_t)prompt_len);
    for (int i = 0; conf_out && i < rows * (nl - 1); ++i) conf_out[i] = -1.0f;
    orc_gpt2_reset_cache(m);
    *steps_out = 0;
    if (orc_gpt2_forward(m, tokens_out, prompt_len, 0, logits, NULL) != 0) {
        free(logits); free(lf);
        return len;
    }
    layers_out[steps++] = nl;
    uint32_t next = argmax_first_d(logits, V, NULL);
    if (!(eos >= 0 && next == (uint32_t)eos)) {
        tokens_out[len++] = next;
        orc_work w;
        work_alloc(m, &w, 1);
        for (int t = 1; t < max_new_tokens; ++t) {
            const int pos = m->kv_len;
            if (pos >= P) break;
            embed_rows(m, &next, 1, pos, w.hid);
            int used = nl;
            for (int L = 0; L < nl; ++L) {
                run_block(m, L, &w, 1, pos);
                if (L + 1 < nl) {
                    run_head(m, &w, 1, 0, 1, logits);
                    const float c = confidence_of(logits, V, lf);
                    if (conf_out) conf_out[(size_t)t * (nl - 1) + L] = c;
                    if (c >= threshold) {
                        for (int j = L + 1; j < nl; ++j)
                            for (int h = 0; h < H; ++h) {
                                const size_t at = (((size_t)j * H + h) * P + pos) * dh;
                                memset(m->kc + at, 0, sizeof(double) * (size_t)dh);
                                memset(m->vc + at, 0, sizeof(double) * (size_t)dh);
                            }
                        used = L + 1;
                        break;
                    }
                }
            }
            m->kv_len = pos + 1;
            layers_out[steps++] = used;
            run_head(m, &w, 1, 0, 1, logits);
            next = argmax_first_d(logits, V, NULL);
            if (eos >= 0 && next == (uint32_t)eos) break;
            tokens_out[len++] = next;
        }
        work_free(&w);
    }
    *steps_out = steps;
    free(lf);
    free(logits);
    return len;
}
