// Host-only life cycle of agpu::nn::GpuArray (include/agpu_nn.hpp): the cases of the reference's unit tests that
// need no GPU (crates/core/gpu-host/src/gpu_array.rs:434-514).  Runs on the CPU; tests/test_cpp_host.py runs it.
#include <cstdio>
#include <vector>

#include "../../include/agpu_nn.hpp"

using namespace agpu::nn;

static int g_failed = 0;
#define CHECK(cond)                                                               \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            ++g_failed;                                                           \
        }                                                                         \
    } while (0)

int main() {
    {  // from_vec_creates_host_only
        auto arr = GpuArray<float>::from_vec({1.0f, 2.0f, 3.0f});
        CHECK(arr.residency() == Residency::HostOnly);
        CHECK(arr.len() == 3 && !arr.is_empty());
    }
    {  // deref_reads_host_data: residency stays HostOnly, no device involved
        auto arr = GpuArray<uint32_t>::from_vec({10u, 20u, 30u});
        CHECK(arr.read() == (std::vector<uint32_t>{10u, 20u, 30u}));
        CHECK(arr[1] == 20u);
        CHECK(arr.residency() == Residency::HostOnly);
    }
    {  // deref_mut_marks_host_dirty
        auto arr = GpuArray<float>::from_vec({1.0f, 2.0f, 3.0f});
        arr.write()[0] = 99.0f;
        CHECK(arr.residency() == Residency::HostDirty);
        CHECK(arr[0] == 99.0f);
    }
    {  // from_slice_copies_data
        const uint8_t data[3] = {5, 10, 15};
        auto arr = GpuArray<uint8_t>::from_slice(data, 3);
        CHECK(arr.read() == (std::vector<uint8_t>{5, 10, 15}));
    }
    {  // zeroed_creates_zero_filled
        auto arr = GpuArray<float>::zeroed(100);
        CHECK(arr.len() == 100);
        bool all_zero = true;
        for (float v : arr.read()) all_zero = all_zero && v == 0.0f;
        CHECK(all_zero);
    }
    {  // empty_array
        auto arr = GpuArray<float>::from_vec({});
        CHECK(arr.is_empty() && arr.len() == 0 && arr.read().empty());
    }
    {  // size thresholds: 64 KiB, strictly below uses pinned mapped memory
        CHECK(GpuArray<float>::zeroed(100).should_use_mapped());
        CHECK(!GpuArray<float>::zeroed(16384).should_use_mapped());
        CHECK(GpuArray<float>::zeroed(16383).should_use_mapped());
    }
    {  // mark_device_dirty changes nothing before the first upload; moving keeps the state
        auto arr = GpuArray<double>::from_vec({4.0, 5.0, 6.0});
        arr.mark_device_dirty();
        CHECK(arr.residency() == Residency::HostOnly);
        arr.write()[2] = 7.0;
        GpuArray<double> moved = std::move(arr);
        CHECK(moved.residency() == Residency::HostDirty && moved[2] == 7.0 && moved.len() == 3);
        CHECK(arr.len() == 0 && arr.residency() == Residency::HostOnly);
    }
    std::printf(g_failed ? "FAILED: %d\n" : "PASSED: %d failed\n", g_failed);
    return g_failed ? 1 : 0;
}
