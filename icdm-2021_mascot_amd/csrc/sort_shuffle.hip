// Popularity sort (thrust::sort_by_key in the reference, preprocess_utils.h:87-88) and the seeded
// rating shuffle (std::random_shuffle, mf_methods.cu:38-39) on the device, both as rocPRIM stable
// LSD radix sorts.
#include "mf_host.h"
#include "mf_device.h"
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace mf {

__global__ __launch_bounds__(256) void shuffle_keys_kernel(uint64_t* __restrict__ keys, uint32_t* __restrict__ idx, uint32_t n, uint64_t base)
{
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) { keys[i] = mix64(base ^ (uint64_t)i); idx[i] = i; }
}
__global__ __launch_bounds__(256) void gather_nodes_kernel(const mf_node* __restrict__ in, mf_node* __restrict__ out, const uint32_t* __restrict__ perm, uint32_t n)
{
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t* s = reinterpret_cast<const uint32_t*>(in + perm[i]);
        uint32_t* d = reinterpret_cast<uint32_t*>(out + i);
        d[0] = s[0]; d[1] = s[1]; d[2] = s[2];
    }
}

struct DeviceBuffers {
    void* ptr[4] = {nullptr, nullptr, nullptr, nullptr};
    ~DeviceBuffers() { for (void* p : ptr) if (p) (void)hipFree(p); }
};

}  // namespace mf

using namespace mf;

extern "C" {

int mf_sort_by_count(uint32_t* cnt, uint32_t* idx, uint32_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!cnt || !idx) return invalid("mf_sort_by_count: null pointer");
    hipStream_t s = as_stream(stream);
    DeviceBuffers b;
    size_t tmp_bytes = 0;
    if (int rc = check_hip(hipMalloc(&b.ptr[0], (size_t)n * 4), "mf_sort_by_count: hipMalloc")) return rc;
    if (int rc = check_hip(hipMalloc(&b.ptr[1], (size_t)n * 4), "mf_sort_by_count: hipMalloc")) return rc;
    uint32_t* cnt_out = static_cast<uint32_t*>(b.ptr[0]);
    uint32_t* idx_out = static_cast<uint32_t*>(b.ptr[1]);
    if (int rc = check_hip(rocprim::radix_sort_pairs(nullptr, tmp_bytes, cnt, cnt_out, idx, idx_out, (size_t)n, 0, 32, s), "mf_sort_by_count: radix_sort_pairs(size)")) return rc;
    if (int rc = check_hip(hipMalloc(&b.ptr[2], tmp_bytes ? tmp_bytes : 4), "mf_sort_by_count: hipMalloc")) return rc;
    if (int rc = check_hip(rocprim::radix_sort_pairs(b.ptr[2], tmp_bytes, cnt, cnt_out, idx, idx_out, (size_t)n, 0, 32, s), "mf_sort_by_count: radix_sort_pairs")) return rc;
    if (int rc = check_hip(hipMemcpyAsync(cnt, cnt_out, (size_t)n * 4, hipMemcpyDeviceToDevice, s), "mf_sort_by_count: copy")) return rc;
    if (int rc = check_hip(hipMemcpyAsync(idx, idx_out, (size_t)n * 4, hipMemcpyDeviceToDevice, s), "mf_sort_by_count: copy")) return rc;
    return check_hip(hipStreamSynchronize(s), "mf_sort_by_count: synchronize");
}

int mf_shuffle_ratings(const mf_node* in, mf_node* out, uint32_t n, uint64_t seed, void* stream)
{
    if (n == 0) return MF_OK;
    if (!in || !out || in == out) return invalid("mf_shuffle_ratings: null or aliased buffers");
    hipStream_t s = as_stream(stream);
    DeviceBuffers b;
    DeviceBuffers b2;
    if (int rc = check_hip(hipMalloc(&b.ptr[0], (size_t)n * 8), "mf_shuffle_ratings: hipMalloc")) return rc;
    if (int rc = check_hip(hipMalloc(&b.ptr[1], (size_t)n * 8), "mf_shuffle_ratings: hipMalloc")) return rc;
    if (int rc = check_hip(hipMalloc(&b.ptr[2], (size_t)n * 4), "mf_shuffle_ratings: hipMalloc")) return rc;
    if (int rc = check_hip(hipMalloc(&b.ptr[3], (size_t)n * 4), "mf_shuffle_ratings: hipMalloc")) return rc;
    uint64_t* keys = static_cast<uint64_t*>(b.ptr[0]);
    uint64_t* keys_out = static_cast<uint64_t*>(b.ptr[1]);
    uint32_t* idx = static_cast<uint32_t*>(b.ptr[2]);
    uint32_t* perm = static_cast<uint32_t*>(b.ptr[3]);
    const uint64_t base = mix64(seed ^ 0x53485546464C4521ull);
    uint32_t grid = (n + 255) / 256; if (grid > 8192) grid = 8192;
    hipLaunchKernelGGL(shuffle_keys_kernel, dim3(grid), dim3(256), 0, s, keys, idx, n, base);
    if (int rc = launch_status("mf_shuffle_ratings: keys")) return rc;
    size_t tmp_bytes = 0;
    if (int rc = check_hip(rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys, keys_out, idx, perm, (size_t)n, 0, 64, s), "mf_shuffle_ratings: radix_sort_pairs(size)")) return rc;
    if (int rc = check_hip(hipMalloc(&b2.ptr[0], tmp_bytes ? tmp_bytes : 4), "mf_shuffle_ratings: hipMalloc")) return rc;
    if (int rc = check_hip(rocprim::radix_sort_pairs(b2.ptr[0], tmp_bytes, keys, keys_out, idx, perm, (size_t)n, 0, 64, s), "mf_shuffle_ratings: radix_sort_pairs")) return rc;
    hipLaunchKernelGGL(gather_nodes_kernel, dim3(grid), dim3(256), 0, s, in, out, perm, n);
    if (int rc = launch_status("mf_shuffle_ratings: gather")) return rc;
    return check_hip(hipStreamSynchronize(s), "mf_shuffle_ratings: synchronize");
}

}  // extern "C"
