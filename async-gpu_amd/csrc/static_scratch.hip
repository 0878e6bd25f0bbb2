// agpu_int4_linear for callers that cannot allocate (code under HIP graph capture, serving loops and harnesses
// that forbid hipMalloc): the same kernels, with the scratch they need in a fixed array inside the library's
// device image instead of a context's allocated workspace.
#include <cstring>
#include <mutex>

#include "linear_common.h"

namespace {

constexpr size_t kStaticWorkspaceBytes = size_t(8) << 20;  // first half: partial sums of a K split (4 MiB)
constexpr int kStaticCounters = 4096;                      // tickets of the K split, one per tile of 64 columns
constexpr size_t kStaticBytes = kStaticWorkspaceBytes + (size_t)kStaticCounters * sizeof(unsigned int);
constexpr int kMaxDevices = 16;

// One copy per GPU, at an address of that GPU's own.  In host code this name is a stand-in, never a device address:
// host code uses the pointer hipGetSymbolAddress returned.
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

struct PerDevice {
    agpu_ctx ctx;           // launch state the kernels' launchers read: stream, CU count, scratch, tickets
    unsigned char *ptr = nullptr;  // this device's copy of `scratch`
    bool ready = false;
};
PerDevice g_dev[kMaxDevices];
std::mutex g_mu;

__global__ __launch_bounds__(256) void clear_u32_kernel(unsigned int *p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

int32_t say(int32_t code, char *err_out, int32_t err_cap, const char *msg) {
    if (err_out && err_cap > 0) {
        std::strncpy(err_out, msg, (size_t)err_cap - 1);
        err_out[err_cap - 1] = '\0';
    }
    return code;
}

// Once per device, with that device current.
int32_t setup(int device, PerDevice **out, char *err_out, int32_t err_cap) {
    PerDevice &d = g_dev[device];
    if (!d.ready) {
        void *ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return say((int32_t)e, err_out, err_cap, "int4_linear_static: hipGetSymbolAddress failed");
        int cus = 0;
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
        if (e != hipSuccess) return say((int32_t)e, err_out, err_cap, "int4_linear_static: hipDeviceGetAttribute failed");
        d.ptr = static_cast<unsigned char *>(ptr);
        d.ctx.device = device;
        d.ctx.num_cus = cus > 0 ? cus : 256;
        d.ctx.workspace = reinterpret_cast<char *>(d.ptr);
        d.ctx.ws_bytes = kStaticWorkspaceBytes;
        d.ctx.owns_workspace = false;
        d.ctx.counters = reinterpret_cast<unsigned int *>(d.ptr + kStaticWorkspaceBytes);
        d.ctx.n_counters = kStaticCounters;
        d.ctx.owns_counters = false;
        d.ready = true;
    }
    *out = &d;
    return AGPU_OK;
}

}  // namespace

AGPU_EXPORT int32_t agpu_int4_linear_static(int32_t device, void *hip_stream, const float *x, const uint32_t *packed,
                                            const float *scales, const float *bias, const float *residual, float *y, int32_t M,
                                            int32_t N, int32_t K, int32_t group, uint32_t flags, char *err_out, int32_t err_cap) {
    if (device < 0 || device >= kMaxDevices) return say(AGPU_ERR_DIM_OUT_OF_RANGE, err_out, err_cap, "int4_linear_static: device out of range");
    // The tickets bound N; whether the partial sums of a shape fit the scratch depends on how its kernel splits K (many
    // shapes need none): the launchers know, and refuse with AGPU_ERR_WORKSPACE when 4 MiB do not do.
    if (N > 0 && (N + 63) / 64 > kStaticCounters - 1)
        return say(AGPU_ERR_WORKSPACE, err_out, err_cap, "int4_linear_static: N must not exceed 262080 (one ticket per 64 columns)");
    std::lock_guard<std::mutex> lock(g_mu);  // host state only: calls that overlap on the GPU still share the scratch
    int prev = -1;
    hipError_t e = hipGetDevice(&prev);
    if (e == hipSuccess && prev != device) e = hipSetDevice(device);
    if (e != hipSuccess) return say((int32_t)e, err_out, err_cap, "int4_linear_static: cannot make the device current");
    PerDevice *d = nullptr;
    int32_t rc = setup(device, &d, err_out, err_cap);
    if (rc == AGPU_OK) {
        d->ctx.stream = static_cast<hipStream_t>(hip_stream);
        d->ctx.err[0] = '\0';
        // the tickets must start at zero; a fill kernel, not a memset node, so that the call may be captured
        hipLaunchKernelGGL(clear_u32_kernel, dim3(kStaticCounters / 256), dim3(256), 0, d->ctx.stream, d->ctx.counters, kStaticCounters);
        rc = AGPU_LAUNCH_CHECK(&d->ctx, "clear_u32_kernel");
        if (rc == AGPU_OK)
            rc = agpu_ln_int4_linear_kv(&d->ctx, x, nullptr, nullptr, 0.0f, packed, scales, bias, residual, y, M, N, K, group, flags, nullptr,
                                        nullptr);
        if (rc != AGPU_OK) say(rc, err_out, err_cap, d->ctx.err);
    }
    if (prev >= 0 && prev != device) (void)hipSetDevice(prev);
    return rc;
}
