// Internal declarations shared by the HIP translation units of libagpu_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <pthread.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/agpu.h"

#define AGPU_EXPORT extern "C" __attribute__((visibility("default")))

constexpr int kWave = 64;                                  // CDNA4 wavefront width
constexpr int kKvFragsPerTile = 4 * 3 * 2 * 32;              // 16-byte bf16 operand fragments of one (head, 32 keys) of K, and of V
constexpr size_t kWorkspaceBytes = size_t(96) << 20;       // default scratch of a context: split-K / attention partials, LayerNorm rows
constexpr size_t kMinWorkspaceBytes = size_t(1) << 20;     // smallest scratch a caller may bring
constexpr int kNumCounters = 1 << 16;                      // arrival tickets of a context (always left at zero)

struct agpu_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    int num_cus = 256;
    // Device scratch: the first half holds split-K and attention partials, the second half LayerNorm rows and, in
    // its last 8 KiB, the candidates of agpu_top_k_sample.  The context's own, or the caller's (agpu_ctx_set_workspace).
    char *workspace = nullptr;
    size_t ws_bytes = 0;
    bool owns_workspace = false;
    unsigned int *counters = nullptr;  // n_counters zeroed uint32; kernels restore zero.  The last one is the arg-max ticket.
    int n_counters = 0;
    bool owns_counters = false;
    // launch-shape overrides of the decode GEMV (agpu_int4_gemv_tune); 0 = default
    int tune_target_wgs = 0, tune_max_waves = 0, tune_rows_per_split = 256;
    int strict_sync = 0;  // agpu_ctx_set_strict_sync: split-K hand-overs with release/acquire fences (verification aid)
    unsigned long long ws_epoch = 0;   // bumped whenever the scratch moves: models drop graphs captured before
    // the one-thread-at-a-time guard: the thread inside a call, and how deep its calls are nested
    std::atomic<uintptr_t> owner{0};
    int depth = 0;
    hipEvent_t t0 = nullptr, t1 = nullptr;  // agpu_timer_*
    char err[512] = {0};
    std::atomic<int> refs{1};  // the handle itself + one per model created on the context
};

// Drops one reference; the context's resources go with the last one.
void agpu_ctx_release(agpu_ctx *ctx);

inline int32_t agpu_fail(agpu_ctx *ctx, int32_t code, const char *fmt, ...) {
    if (ctx) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
        va_end(ap);
    }
    return code;
}

inline int32_t agpu_hip(agpu_ctx *ctx, hipError_t e, const char *what) {
    if (e == hipSuccess) return AGPU_OK;
    return agpu_fail(ctx, (int32_t)e, "%s: %s", what, hipGetErrorString(e));
}

// Marks the calling thread as the one inside a call on the context; a second thread is turned away (ok == false).
// Calls nest (entry points call each other), so the same thread may enter again.
struct agpu_ctx_guard {
    agpu_ctx *c;
    bool ok;
    explicit agpu_ctx_guard(agpu_ctx *ctx) : c(ctx), ok(false) {
        const uintptr_t me = (uintptr_t)pthread_self();
        if (c->owner.load(std::memory_order_relaxed) == me) {
            ++c->depth;
            ok = true;
            return;
        }
        uintptr_t none = 0;
        ok = c->owner.compare_exchange_strong(none, me, std::memory_order_acquire);
        if (ok) c->depth = 1;
    }
    ~agpu_ctx_guard() {
        if (ok && --c->depth == 0) c->owner.store(0, std::memory_order_release);
    }
    agpu_ctx_guard(const agpu_ctx_guard &) = delete;
    agpu_ctx_guard &operator=(const agpu_ctx_guard &) = delete;
};

// First statement of every entry point that takes a context.
#define AGPU_REQUIRE_CTX(ctx)                                      \
    if (!(ctx)) return AGPU_ERR_NULL_POINTER;                      \
    agpu_ctx_guard agpu_guard_(const_cast<agpu_ctx *>(ctx));       \
    if (!agpu_guard_.ok) return AGPU_ERR_BUSY

#define AGPU_REQUIRE_PTR(ctx, p)                                                         \
    do {                                                                                 \
        if (!(p)) return agpu_fail((ctx), AGPU_ERR_NULL_POINTER, "%s: null pointer " #p, __func__); \
    } while (0)

#define AGPU_LAUNCH_CHECK(ctx, name) agpu_hip((ctx), hipGetLastError(), name)

// ---- device helpers ---------------------------------------------------------------

// Hand-over of partial results between workgroups (split K, split keys, arg-max candidates).  A workgroup writes its
// partials with relaxed agent-scope stores (write-through on gfx950), calls partials_published, takes a ticket; the
// workgroup that draws the last ticket reads every partial with relaxed agent-scope loads.  The fast form rests on a
// property of the hardware: s_waitcnt vmcnt(0) returns for a write-through store only once the store is visible to
// the whole device.  With `strict` the same steps are also expressed to the memory model, as a release fence before
// and an acquire fence after an acq_rel ticket; results must be the same bits either way.
__device__ __forceinline__ void partials_published(int strict) {
    if (strict) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}
__device__ __forceinline__ unsigned int take_ticket(unsigned int *counter, int strict) {
    if (strict) {
        const unsigned int t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        return t;
    }
    return __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Cross-lane moves as DPP modifiers of ordinary VALU instructions (a few cycles each; a ds_bpermute
// round trip through the LDS crossbar costs on the order of a hundred).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v), CTRL,
                                                                 ROW_MASK, 0xf, false));
}

// Sum / maximum over each row of 16 lanes, result in every lane of the row.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xb1, 0xf>(0.0f, v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4e, 0xf>(0.0f, v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x124, 0xf>(0.0f, v);  // row_ror:4
    v += dpp_move<0x128, 0xf>(0.0f, v);  // row_ror:8
    return v;
}

__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<0xb1, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x4e, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x124, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x128, 0xf>(v, v));
    return v;
}

// Sum / maximum over the 64 lanes, result in every lane: rows of 16 first, then row_bcast:15 into rows 1
// and 3 and row_bcast:31 into rows 2 and 3 leave the total in lane 63.  The order of additions is fixed.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += dpp_move<0x142, 0xa>(0.0f, v);
    v += dpp_move<0x143, 0xc>(0.0f, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    v = fmaxf(v, dpp_move<0x142, 0xa>(v, v));
    v = fmaxf(v, dpp_move<0x143, 0xc>(v, v));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// The same for unsigned integers (arg-max index selection).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned dpp_move_u32(unsigned old, unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp((int)old, (int)v, CTRL, ROW_MASK, 0xf, false);
}

template <bool MAX>
__device__ __forceinline__ unsigned row16_minmax_u32(unsigned v) {
    unsigned o;
    o = dpp_move_u32<0xb1, 0xf>(v, v); v = MAX ? (o > v ? o : v) : (o < v ? o : v);
    o = dpp_move_u32<0x4e, 0xf>(v, v); v = MAX ? (o > v ? o : v) : (o < v ? o : v);
    o = dpp_move_u32<0x124, 0xf>(v, v); v = MAX ? (o > v ? o : v) : (o < v ? o : v);
    o = dpp_move_u32<0x128, 0xf>(v, v); v = MAX ? (o > v ? o : v) : (o < v ? o : v);
    return v;
}

template <bool MAX>
__device__ __forceinline__ unsigned wave_minmax_u32(unsigned v) {
    v = row16_minmax_u32<MAX>(v);
    unsigned o;
    o = dpp_move_u32<0x142, 0xa>(v, v); v = MAX ? (o > v ? o : v) : (o < v ? o : v);
    o = dpp_move_u32<0x143, 0xc>(v, v); v = MAX ? (o > v ? o : v) : (o < v ? o : v);
    return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}

// tanh GELU, 0.5x(1+tanh(c(x+0.044715x^3))), accurate expf, no fast-math.
__device__ __forceinline__ float gelu_tanh_dev(float x) {
    // 0.5 * (1 + tanh(u)) == 1 / (1 + exp(-2u)): one exp and one division instead of a tanh expansion
    const float c = 0.7978845608028654f, k = 0.044715f;
    const float inner = c * (x + k * x * x * x);
    return x / (1.0f + expf(-2.0f * inner));
}

__device__ __forceinline__ float gelu_quick_dev(float x) { return x / (1.0f + expf(-1.702f * x)); }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
