// Popularity sort (thrust::sort_by_key in the reference, preprocess_utils.h:87-88) and the seeded
// rating shuffle (std::random_shuffle, mf_methods.cu:38-39) on the device, both as rocPRIM stable
// LSD radix sorts.
#include "mf_host.h"
#include "mf_device.h"
#include <cstring>
#include <mutex>
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

constexpr size_t kAlign = 256;
static inline size_t aligned(size_t bytes) { return (bytes + kAlign - 1) / kAlign * kAlign; }

// Workspace layout of the count sort: sorted counts, sorted ids (the radix sort's output buffers), rocPRIM's own
// temporary storage.  The size query only computes sizes; it needs a current device (rocPRIM picks its kernel
// configuration by architecture).
static int sort_layout(uint32_t n, size_t* tmp_bytes, size_t* total)
{
    size_t tmp = 0;
    uint32_t* none = nullptr;
    if (int rc = check_hip(rocprim::radix_sort_pairs(nullptr, tmp, none, none, none, none, (size_t)n, 0, 32, nullptr), "radix_sort_pairs(size)")) return rc;
    *tmp_bytes = tmp;
    *total = 2 * aligned((size_t)n * 4) + aligned(tmp ? tmp : 4);
    return MF_OK;
}
static int sort_in(uint32_t* cnt, uint32_t* idx, uint32_t n, uint8_t* ws, size_t tmp_bytes, hipStream_t s)
{
    uint32_t* cnt_out = reinterpret_cast<uint32_t*>(ws);
    uint32_t* idx_out = reinterpret_cast<uint32_t*>(ws + aligned((size_t)n * 4));
    void* tmp = ws + 2 * aligned((size_t)n * 4);
    if (int rc = check_hip(rocprim::radix_sort_pairs(tmp, tmp_bytes, cnt, cnt_out, idx, idx_out, (size_t)n, 0, 32, s), "mf_sort_by_count: radix_sort_pairs")) return rc;
    if (int rc = check_hip(hipMemcpyAsync(cnt, cnt_out, (size_t)n * 4, hipMemcpyDeviceToDevice, s), "mf_sort_by_count: copy")) return rc;
    return check_hip(hipMemcpyAsync(idx, idx_out, (size_t)n * 4, hipMemcpyDeviceToDevice, s), "mf_sort_by_count: copy");
}
// The shuffle: 64-bit keys in and out, ids in, permutation out, rocPRIM's temporary storage.
static int shuffle_layout(uint32_t n, size_t* tmp_bytes, size_t* total)
{
    size_t tmp = 0;
    uint64_t* nk = nullptr; uint32_t* nv = nullptr;
    if (int rc = check_hip(rocprim::radix_sort_pairs(nullptr, tmp, nk, nk, nv, nv, (size_t)n, 0, 64, nullptr), "radix_sort_pairs(size)")) return rc;
    *tmp_bytes = tmp;
    *total = 2 * aligned((size_t)n * 8) + 2 * aligned((size_t)n * 4) + aligned(tmp ? tmp : 4);
    return MF_OK;
}

// ---- scratch of mf_sort_by_count_static ------------------------------------------------------------------------
// Device memory that belongs to the library image: every GPU the library runs on holds its own copy from the moment
// the code object is loaded until the process ends.  20 MiB: the two output buffers of a sort of kStaticSortMax
// counts (8 MiB) and rocPRIM's temporary storage for that size (8.4 MB on gfx950 with rocPRIM 4: its own pair of
// buffers and its counters).
constexpr uint32_t kStaticSortMax = 1u << 20;
constexpr size_t kStaticScratchBytes = 20u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// The array's name is a host-side stand-in, not a device address: the address of each device's copy is asked for once,
// with that device current, and everything below uses that pointer.
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};
static int static_scratch(void** out)
{
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "mf_sort_by_count_static: hipGetDevice")) return rc;
    if (dev < 0 || dev >= kMaxDevices) return invalid("mf_sort_by_count_static: device %d is beyond the %d devices this library keeps scratch addresses for", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (int rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "mf_sort_by_count_static: hipGetSymbolAddress(scratch)")) return rc;
        if (!ptr) return invalid("mf_sort_by_count_static: the scratch array has no address on device %d", dev);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return MF_OK;
}

}  // namespace mf

using namespace mf;

extern "C" {

size_t mf_sort_by_count_workspace_bytes(uint32_t n)
{
    if (n == 0) return 0;
    size_t tmp = 0, total = 0;
    return sort_layout(n, &tmp, &total) == MF_OK ? total : 0;
}
int mf_sort_by_count_ws(uint32_t* cnt, uint32_t* idx, uint32_t n, void* workspace, size_t workspace_bytes, void* stream)
{
    if (n == 0) return MF_OK;
    if (!cnt || !idx || !workspace) return invalid("mf_sort_by_count_ws: null pointer");
    if (reinterpret_cast<uintptr_t>(workspace) % kAlign) return invalid("mf_sort_by_count_ws: the workspace must be 256-byte aligned");
    size_t tmp = 0, total = 0;
    if (int rc = sort_layout(n, &tmp, &total)) return rc;
    if (workspace_bytes < total) return invalid("mf_sort_by_count_ws: the workspace holds %zu bytes, %u counts need %zu (mf_sort_by_count_workspace_bytes)", workspace_bytes, n, total);
    return sort_in(cnt, idx, n, static_cast<uint8_t*>(workspace), tmp, as_stream(stream));
}
int mf_sort_by_count(uint32_t* cnt, uint32_t* idx, uint32_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!cnt || !idx) return invalid("mf_sort_by_count: null pointer");
    size_t tmp = 0, total = 0;
    if (int rc = sort_layout(n, &tmp, &total)) return rc;
    DeviceBuffers b;
    if (int rc = check_hip(hipMalloc(&b.ptr[0], total), "mf_sort_by_count: hipMalloc")) return rc;
    if (int rc = sort_in(cnt, idx, n, static_cast<uint8_t*>(b.ptr[0]), tmp, as_stream(stream))) return rc;
    return check_hip(hipStreamSynchronize(as_stream(stream)), "mf_sort_by_count: synchronize");      // the workspace is freed on return
}
uint32_t mf_sort_by_count_static_max(void) { return kStaticSortMax; }
int mf_sort_by_count_static(uint32_t* cnt, uint32_t* idx, uint32_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!cnt || !idx) return invalid("mf_sort_by_count_static: null pointer");
    if (n > kStaticSortMax) return invalid("mf_sort_by_count_static: %u counts, the library's own scratch holds at most %u (use mf_sort_by_count_ws with a workspace)", n, kStaticSortMax);
    size_t tmp = 0, total = 0;
    if (int rc = sort_layout(n, &tmp, &total)) return rc;
    if (total > kStaticScratchBytes) return invalid("mf_sort_by_count_static: %u counts need %zu bytes of scratch, the library's own holds %zu", n, total, kStaticScratchBytes);
    void* ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    // nothing in the scratch has to start at zero: the sort writes its output buffers before it reads them and rocPRIM
    // initialises what it keeps in its temporary storage
    return sort_in(cnt, idx, n, static_cast<uint8_t*>(ptr), tmp, as_stream(stream));
}

size_t mf_shuffle_ratings_workspace_bytes(uint32_t n)
{
    if (n == 0) return 0;
    size_t tmp = 0, total = 0;
    return shuffle_layout(n, &tmp, &total) == MF_OK ? total : 0;
}
int mf_shuffle_ratings_ws(const mf_node* in, mf_node* out, uint32_t n, uint64_t seed, void* workspace, size_t workspace_bytes, void* stream)
{
    if (n == 0) return MF_OK;
    if (!in || !out || in == out) return invalid("mf_shuffle_ratings: null or aliased buffers");
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % kAlign) return invalid("mf_shuffle_ratings_ws: the workspace must be non-null and 256-byte aligned");
    size_t tmp_bytes = 0, total = 0;
    if (int rc = shuffle_layout(n, &tmp_bytes, &total)) return rc;
    if (workspace_bytes < total) return invalid("mf_shuffle_ratings_ws: the workspace holds %zu bytes, %u ratings need %zu (mf_shuffle_ratings_workspace_bytes)", workspace_bytes, n, total);
    hipStream_t s = as_stream(stream);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    uint64_t* keys = reinterpret_cast<uint64_t*>(ws);
    uint64_t* keys_out = reinterpret_cast<uint64_t*>(ws + aligned((size_t)n * 8));
    uint32_t* idx = reinterpret_cast<uint32_t*>(ws + 2 * aligned((size_t)n * 8));
    uint32_t* perm = reinterpret_cast<uint32_t*>(ws + 2 * aligned((size_t)n * 8) + aligned((size_t)n * 4));
    void* tmp = ws + 2 * aligned((size_t)n * 8) + 2 * aligned((size_t)n * 4);
    const uint64_t base = mix64(seed ^ 0x53485546464C4521ull);
    uint32_t grid = (n + 255) / 256; if (grid > 8192) grid = 8192;
    hipLaunchKernelGGL(shuffle_keys_kernel, dim3(grid), dim3(256), 0, s, keys, idx, n, base);
    if (int rc = launch_status("mf_shuffle_ratings: keys")) return rc;
    if (int rc = check_hip(rocprim::radix_sort_pairs(tmp, tmp_bytes, keys, keys_out, idx, perm, (size_t)n, 0, 64, s), "mf_shuffle_ratings: radix_sort_pairs")) return rc;
    hipLaunchKernelGGL(gather_nodes_kernel, dim3(grid), dim3(256), 0, s, in, out, perm, n);
    return launch_status("mf_shuffle_ratings: gather");
}
int mf_shuffle_ratings(const mf_node* in, mf_node* out, uint32_t n, uint64_t seed, void* stream)
{
    if (n == 0) return MF_OK;
    if (!in || !out || in == out) return invalid("mf_shuffle_ratings: null or aliased buffers");
    size_t tmp = 0, total = 0;
    if (int rc = shuffle_layout(n, &tmp, &total)) return rc;
    DeviceBuffers b;
    if (int rc = check_hip(hipMalloc(&b.ptr[0], total), "mf_shuffle_ratings: hipMalloc")) return rc;
    if (int rc = mf_shuffle_ratings_ws(in, out, n, seed, b.ptr[0], total, stream)) return rc;
    return check_hip(hipStreamSynchronize(as_stream(stream)), "mf_shuffle_ratings: synchronize");      // the workspace is freed on return
}

}  // extern "C"
