// Context, device memory and the kernel-name table of libagpu_hip.so.
#include <chrono>
#include <cstring>
#include <new>
#include <thread>

#include "agpu_internal.h"

static int32_t ctx_init(agpu_ctx *c) {
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, c->device);
    if (e != hipSuccess) return agpu_hip(c, e, "hipGetDeviceProperties");
    c->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    e = hipMalloc((void **)&c->workspace, kWorkspaceBytes);
    if (e != hipSuccess) return agpu_hip(c, e, "hipMalloc(workspace)");
    c->ws_bytes = kWorkspaceBytes;
    c->owns_workspace = true;
    e = hipMalloc((void **)&c->counters, kNumCounters * sizeof(unsigned int));
    if (e != hipSuccess) return agpu_hip(c, e, "hipMalloc(counters)");
    c->n_counters = kNumCounters;
    c->owns_counters = true;
    e = hipMemset(c->counters, 0, kNumCounters * sizeof(unsigned int));
    if (e != hipSuccess) return agpu_hip(c, e, "hipMemset(counters)");
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_ctx_create(int32_t device, agpu_ctx **out) {
    if (!out) return AGPU_ERR_NULL_POINTER;
    *out = nullptr;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int32_t)e;
    agpu_ctx *c = new (std::nothrow) agpu_ctx();
    if (!c) return AGPU_ERR_NULL_POINTER;
    c->device = device;
    e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete c;
        return (int32_t)e;
    }
    c->owns_stream = true;
    int32_t rc = ctx_init(c);
    if (rc != AGPU_OK) {
        agpu_ctx_destroy(c);
        return rc;
    }
    *out = c;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_ctx_create_on_stream(int32_t device, void *hip_stream, agpu_ctx **out) {
    if (!out) return AGPU_ERR_NULL_POINTER;
    *out = nullptr;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int32_t)e;
    agpu_ctx *c = new (std::nothrow) agpu_ctx();
    if (!c) return AGPU_ERR_NULL_POINTER;
    c->device = device;
    c->stream = (hipStream_t)hip_stream;
    c->owns_stream = false;
    int32_t rc = ctx_init(c);
    if (rc != AGPU_OK) {
        agpu_ctx_destroy(c);
        return rc;
    }
    *out = c;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_ctx_destroy(agpu_ctx *ctx) {
    if (!ctx) return AGPU_OK;
    agpu_ctx_release(ctx);
    return AGPU_OK;
}

void agpu_ctx_release(agpu_ctx *ctx) {
    if (ctx->refs.fetch_sub(1) > 1) return;  // a model still runs on this context
    (void)hipSetDevice(ctx->device);
    if (ctx->stream || !ctx->owns_stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->t0) (void)hipEventDestroy(ctx->t0);
    if (ctx->t1) (void)hipEventDestroy(ctx->t1);
    if (ctx->workspace && ctx->owns_workspace) (void)hipFree(ctx->workspace);
    if (ctx->counters && ctx->owns_counters) (void)hipFree(ctx->counters);
    if (ctx->owns_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

AGPU_EXPORT size_t agpu_ctx_workspace_bytes(const agpu_ctx *ctx) { return ctx ? ctx->ws_bytes : 0; }

AGPU_EXPORT int32_t agpu_ctx_set_workspace(agpu_ctx *ctx, void *workspace, size_t bytes) {
    AGPU_REQUIRE_CTX(ctx);
    hipError_t e = hipStreamSynchronize(ctx->stream);  // nothing in flight may still use the old scratch
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamSynchronize");
    if (!workspace) {
        // back to a scratch of the context's own
        if (ctx->owns_workspace) return AGPU_OK;
        char *own = nullptr;
        e = hipMalloc((void **)&own, kWorkspaceBytes);
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipMalloc(workspace)");
        ctx->workspace = own;
        ctx->ws_bytes = kWorkspaceBytes;
        ctx->owns_workspace = true;
        ++ctx->ws_epoch;
        return AGPU_OK;
    }
    if (bytes < kMinWorkspaceBytes || ((uintptr_t)workspace & 255u) != 0)
        return agpu_fail(ctx, AGPU_ERR_WORKSPACE, "ctx_set_workspace: need at least %zu bytes, 256-byte aligned (got %zu at %p)",
                         kMinWorkspaceBytes, bytes, workspace);
    if (ctx->owns_workspace && ctx->workspace) (void)hipFree(ctx->workspace);
    ctx->workspace = static_cast<char *>(workspace);
    ctx->ws_bytes = bytes & ~(size_t)511;  // both halves stay 256-byte aligned
    ctx->owns_workspace = false;
    ++ctx->ws_epoch;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_ctx_test_hold(agpu_ctx *ctx, int32_t ms) {
    AGPU_REQUIRE_CTX(ctx);
    std::this_thread::sleep_for(std::chrono::milliseconds(ms > 0 ? ms : 0));
    return AGPU_OK;
}

// Scratch a Linear call of this shape can use at most: the partial sums of the deepest K split any of the kernels
// would choose (one slice per 64 k) in the first half, one LayerNorm copy of x in the second.
AGPU_EXPORT size_t agpu_int4_linear_workspace_bytes(int32_t M, int32_t N, int32_t K, int32_t with_layer_norm) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const size_t slices = (size_t)(K + 63) / 64;
    const size_t rows = M <= 16 ? (size_t)M : ((size_t)M + 63) / 64 * 64, cols = ((size_t)N + 255) / 256 * 256;
    size_t partial = slices * rows * cols * sizeof(float);
    const size_t ln = with_layer_norm ? (size_t)M * K * sizeof(float) : 0;
    size_t half = partial > ln ? partial : ln;
    if (half < kMinWorkspaceBytes / 2) half = kMinWorkspaceBytes / 2;
    return 2 * ((half + 255) & ~(size_t)255);
}

AGPU_EXPORT int32_t agpu_ctx_set_strict_sync(agpu_ctx *ctx, int32_t on) {
    AGPU_REQUIRE_CTX(ctx);
    ctx->strict_sync = on ? 1 : 0;
    return AGPU_OK;
}

AGPU_EXPORT const char *agpu_last_error_string(const agpu_ctx *ctx) { return ctx ? ctx->err : "null context"; }

AGPU_EXPORT void *agpu_ctx_stream(const agpu_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

AGPU_EXPORT int32_t agpu_malloc(agpu_ctx *ctx, size_t bytes, void **out) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, out);
    *out = nullptr;
    if (bytes == 0) return AGPU_OK;
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipMalloc");
    e = hipMemsetAsync(*out, 0, bytes, ctx->stream);
    return agpu_hip(ctx, e, "hipMemsetAsync");
}

AGPU_EXPORT int32_t agpu_free(agpu_ctx *ctx, void *ptr) {
    AGPU_REQUIRE_CTX(ctx);
    if (!ptr) return AGPU_OK;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamSynchronize");
    return agpu_hip(ctx, hipFree(ptr), "hipFree");
}

AGPU_EXPORT int32_t agpu_host_alloc_mapped(agpu_ctx *ctx, size_t bytes, void **host_out, void **dev_out) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, host_out);
    AGPU_REQUIRE_PTR(ctx, dev_out);
    *host_out = *dev_out = nullptr;
    if (bytes == 0) return AGPU_OK;
    void *h = nullptr, *d = nullptr;
    hipError_t e = hipHostMalloc(&h, bytes, hipHostMallocMapped);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipHostMalloc");
    e = hipHostGetDevicePointer(&d, h, 0);
    if (e != hipSuccess) {
        (void)hipHostFree(h);
        return agpu_hip(ctx, e, "hipHostGetDevicePointer");
    }
    std::memset(h, 0, bytes);
    *host_out = h;
    *dev_out = d;
    return AGPU_OK;
}

AGPU_EXPORT int32_t agpu_host_free_mapped(agpu_ctx *ctx, void *host) {
    AGPU_REQUIRE_CTX(ctx);
    if (!host) return AGPU_OK;
    hipError_t e = hipStreamSynchronize(ctx->stream);  // a kernel may still be reading or writing the memory
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipStreamSynchronize");
    return agpu_hip(ctx, hipHostFree(host), "hipHostFree");
}

AGPU_EXPORT int32_t agpu_memcpy_h2d(agpu_ctx *ctx, void *dst, const void *src_host, size_t bytes) {
    AGPU_REQUIRE_CTX(ctx);
    if (bytes == 0) return AGPU_OK;
    AGPU_REQUIRE_PTR(ctx, dst);
    AGPU_REQUIRE_PTR(ctx, src_host);
    hipError_t e = hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipMemcpyAsync(h2d)");
    return agpu_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

AGPU_EXPORT int32_t agpu_memcpy_d2h(agpu_ctx *ctx, void *dst_host, const void *src, size_t bytes) {
    AGPU_REQUIRE_CTX(ctx);
    if (bytes == 0) return AGPU_OK;
    AGPU_REQUIRE_PTR(ctx, dst_host);
    AGPU_REQUIRE_PTR(ctx, src);
    hipError_t e = hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e != hipSuccess) return agpu_hip(ctx, e, "hipMemcpyAsync(d2h)");
    return agpu_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

AGPU_EXPORT int32_t agpu_memcpy_d2d(agpu_ctx *ctx, void *dst, const void *src, size_t bytes) {
    AGPU_REQUIRE_CTX(ctx);
    if (bytes == 0) return AGPU_OK;
    AGPU_REQUIRE_PTR(ctx, dst);
    AGPU_REQUIRE_PTR(ctx, src);
    return agpu_hip(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream),
                    "hipMemcpyAsync(d2d)");
}

AGPU_EXPORT int32_t agpu_sync(agpu_ctx *ctx) {
    AGPU_REQUIRE_CTX(ctx);
    return agpu_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

AGPU_EXPORT int32_t agpu_timer_start(agpu_ctx *ctx) {
    AGPU_REQUIRE_CTX(ctx);
    if (!ctx->t0) {
        hipError_t e = hipEventCreate(&ctx->t0);
        if (e == hipSuccess) e = hipEventCreate(&ctx->t1);
        if (e != hipSuccess) return agpu_hip(ctx, e, "hipEventCreate");
    }
    return agpu_hip(ctx, hipEventRecord(ctx->t0, ctx->stream), "hipEventRecord");
}

AGPU_EXPORT int32_t agpu_timer_stop(agpu_ctx *ctx, float *ms_out_host) {
    AGPU_REQUIRE_CTX(ctx);
    AGPU_REQUIRE_PTR(ctx, ms_out_host);
    if (!ctx->t0) return agpu_fail(ctx, AGPU_ERR_UNSUPPORTED, "timer_stop without timer_start");
    hipError_t e = hipEventRecord(ctx->t1, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(ctx->t1);
    if (e == hipSuccess) e = hipEventElapsedTime(ms_out_host, ctx->t0, ctx->t1);
    return agpu_hip(ctx, e, "timer_stop");
}

// The reference's kernel names on this path (nn/registry.rs:34-103) and the entry
// point that serves each.
static const struct {
    const char *name;
    const char *entry;
} kKernelTable[] = {
    {"int4_gemm_w4a16", "agpu_int4_linear"},
    {"bias_add", "agpu_bias_add"},
    {"layer_norm", "agpu_layer_norm"},
    {"layer_norm_v2", "agpu_layer_norm"},
    {"layer_norm_v3", "agpu_layer_norm"},
    {"layer_norm_residual", "agpu_add_layer_norm_dual"},
    {"layer_norm_residual_dual", "agpu_add_layer_norm_dual"},
    {"gelu_forward", "agpu_gelu"},
    {"gelu_forward_v2", "agpu_gelu"},
    {"elementwise_add", "agpu_add_inplace"},
    {"elementwise_add_v2", "agpu_add_inplace"},
    {"elementwise_add_v3", "agpu_add_inplace"},
    {"split_qkv", "agpu_split_qkv"},
    {"concat_heads", "agpu_concat_heads"},
    {"flash_attention", "agpu_attention"},
    {"flash_attention_v2", "agpu_attention"},
    {"flash_attn_v3", "agpu_attention"},
    {"flash_attention_kv", "agpu_attention"},
    {"kv_cache_append", "agpu_kv_append"},
    {"embedding_lookup", "agpu_embedding"},
    {"gemm_f32", "agpu_gemm_f32"},
    {"gemm_f32_v2", "agpu_gemm_f32"},
    {"gemm_f32_v3", "agpu_gemm_f32"},
};

AGPU_EXPORT int32_t agpu_kernel_lookup(const agpu_ctx *ctx, const char *name, const char **entry_point_out) {
    if (entry_point_out) *entry_point_out = nullptr;
    if (!name) return AGPU_ERR_NULL_POINTER;
    for (const auto &e : kKernelTable) {
        if (std::strcmp(e.name, name) == 0) {
            if (entry_point_out) *entry_point_out = e.entry;
            return AGPU_OK;
        }
    }
    if (ctx) {
        agpu_fail(const_cast<agpu_ctx *>(ctx), AGPU_ERR_KERNEL_NOT_FOUND, "kernel not found in registry: %s", name);
    }
    return AGPU_ERR_KERNEL_NOT_FOUND;
}
