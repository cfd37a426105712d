// Kernels around the update loop: binary16 <-> binary32 conversion, grouped-storage scatter and
// gather, the g-switching error estimate, test RMSE (dense and grouped), model init, histogram,
// re-indexing.  All are streaming, HBM-bound, grid-stride kernels.
#include "mf_host.h"
#include "mf_device.h"
#include <type_traits>
#include <cmath>
#include <vector>

namespace mf {

constexpr int kStreamBlock = 256;
static inline uint32_t stream_grid(uint64_t n, int per_thread = 1)
{
    uint64_t blocks = (n + (uint64_t)kStreamBlock * per_thread - 1) / ((uint64_t)kStreamBlock * per_thread);
    const uint64_t cap = 256ull * 32;             // 32 workgroups per CU keeps every XCD busy
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    return (uint32_t)blocks;
}

// ---- conversions (model_init.cu:85-112, precision_switching.h:1-6) -----------------------------
__global__ __launch_bounds__(kStreamBlock) void float2half_kernel(const float* __restrict__ in, uint16_t* __restrict__ out, uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t n2 = n / 2;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n2; i += stride) {
        const float2 v = reinterpret_cast<const float2*>(in)[i];
        half2_t h; h.x = (half_t)v.x; h.y = (half_t)v.y;
        reinterpret_cast<uint32_t*>(out)[i] = bits(h);
    }
    if ((n & 1) && blockIdx.x == 0 && threadIdx.x == 0) out[n - 1] = (uint16_t)bits((half_t)in[n - 1]);
}
__global__ __launch_bounds__(kStreamBlock) void half2float_kernel(const uint16_t* __restrict__ in, float* __restrict__ out, uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t n2 = n / 2;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n2; i += stride) {
        const half2_t h = from_bits<half2_t>(reinterpret_cast<const uint32_t*>(in)[i]);
        reinterpret_cast<float2*>(out)[i] = make_float2((float)h.x, (float)h.y);
    }
    if ((n & 1) && blockIdx.x == 0 && threadIdx.x == 0) out[n - 1] = (float)from_bits<half_t>(in[n - 1]);
}

// min{g : idx <= end[g]}
__device__ __forceinline__ uint32_t group_of(const uint32_t* end, uint32_t groups, uint32_t idx)
{
    uint32_t lo = 0, hi = groups - 1;
    while (lo < hi) {
        uint32_t mid = (lo + hi) >> 1;
        if (idx <= end[mid]) hi = mid; else lo = mid + 1;
    }
    return lo;
}

// ---- scatter into grouped binary16 storage (model_init.cu:30-83) ---------------------------------
template <int K>
__global__ __launch_bounds__(kBlock) void scatter_to_groups_kernel(const float* __restrict__ params, void* const* __restrict__ group_ptr,
                                                                  const uint32_t* __restrict__ group_end, const uint32_t* __restrict__ entity2group,
                                                                  const uint32_t* __restrict__ entity2sorted, uint32_t n, uint32_t groups)
{
    const int lane = threadIdx.x & 63;
    const uint32_t waves = gridDim.x * kWavesPerBlock;
    for (uint32_t e = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); e < n; e += waves) {
        const uint32_t g = entity2group[e];
        if (g >= groups) continue;
        const uint32_t first = g ? group_end[g - 1] + 1 : 0;
        const uint32_t row = entity2sorted[e] - first;
        uint16_t* dst = reinterpret_cast<uint16_t*>(group_ptr[g]) + (size_t)row * K;
        const float* src = params + (size_t)e * K;
        if constexpr (K == 128) {
            const float2 v = reinterpret_cast<const float2*>(src)[lane];
            half2_t h; h.x = (half_t)v.x; h.y = (half_t)v.y;
            reinterpret_cast<uint32_t*>(dst)[lane] = bits(h);
        } else {
            dst[lane] = (uint16_t)bits((half_t)src[lane]);
        }
    }
}

// ---- gather grouped storage into a dense fp32 matrix in sorted row order (mf_methods.cu:249-313) --
template <int K>
__global__ __launch_bounds__(kBlock) void gather_from_groups_kernel(void* const* __restrict__ group_ptr, const uint32_t* __restrict__ group_end,
                                                                   const uint8_t* __restrict__ prec, float* __restrict__ dense, uint32_t n, uint32_t groups)
{
    const int lane = threadIdx.x & 63;
    const uint32_t waves = gridDim.x * kWavesPerBlock;
    for (uint32_t row = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); row < n; row += waves) {
        const uint32_t g = group_of(group_end, groups, row);
        if (row > group_end[g]) continue;
        const uint32_t local = g ? row - group_end[g - 1] - 1 : row;
        float* dst = dense + (size_t)row * K;
        if (prec[g]) {
            const float* src = reinterpret_cast<const float*>(group_ptr[g]) + (size_t)local * K;
            for (int e = lane; e < K; e += 64) dst[e] = src[e];
        } else {
            const uint16_t* src = reinterpret_cast<const uint16_t*>(group_ptr[g]) + (size_t)local * K;
            for (int e = lane; e < K; e += 64) dst[e] = (float)from_bits<half_t>(src[e]);
        }
    }
}

// ---- per-group error (mf_methods.cu:327-379): one wavefront per group ---------------------------
__global__ __launch_bounds__(kWave) void group_error_kernel(float* __restrict__ grad_sum, const float* __restrict__ norm_sum, uint32_t norm_blocks,
                                                           const uint8_t* __restrict__ prec, const float* __restrict__ initial,
                                                           float* __restrict__ error_out, int k, uint32_t groups)
{
    const uint32_t g = blockIdx.x;
    if (g >= groups) return;
    const int lane = threadIdx.x;
    if (prec[g]) { if (lane == 0) error_out[g] = -1.f; return; }
    float acc = 0.f, nacc = 0.f;
    for (int e = lane; e < k; e += kWave) { const float v = grad_sum[(size_t)g * k + e]; acc += v * v; grad_sum[(size_t)g * k + e] = 0.f; }
    for (uint32_t b = lane; b < norm_blocks; b += kWave) nacc += norm_sum[(size_t)g * norm_blocks + b];
    acc = reduce_wave(acc, OpAdd());
    nacc = reduce_wave(nacc, OpAdd());
    if (lane == 0) error_out[g] = (acc / nacc) / initial[g];
}

// ---- test RMSE (rmse.h:26-189): wave reduction of each dot, per-wave double accumulation, LDS
// reduction across the workgroup, one double atomic per workgroup ----------------------------------
__device__ __forceinline__ void block_sum_to_global(double acc, double* out)
{
    __shared__ double part[kWavesPerBlock];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) part[w] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = 0;
        for (int i = 0; i < kWavesPerBlock; ++i) s += part[i];
        atomicAdd(out, s);
    }
}

template <int K>
__global__ __launch_bounds__(kBlock) void rmse_dense_kernel(const mf_node* __restrict__ test, uint32_t test_n, const float* __restrict__ P,
                                                           const float* __restrict__ Q, double* sum_sq)
{
    constexpr int E = K / 64;
    const int lane = threadIdx.x & 63;
    const uint32_t waves = gridDim.x * kWavesPerBlock;
    const uint32_t wid = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    double acc = 0;
    for (uint64_t base = (uint64_t)wid * kWave; base < test_n; base += (uint64_t)waves * kWave) {
        const uint64_t left = test_n - base;
        const int n = left < (uint64_t)kWave ? (int)left : kWave;
        Rating my = {0.f, 0u, 0u};
        if (lane < n) my = load_rating(test, (uint32_t)(base + lane));
        for (int j = 0; j < n; ++j) {
            const float r = bcast(my.r, j);
            const float* pp = P + (size_t)bcast(my.u, j) * K + lane;
            const float* qq = Q + (size_t)bcast(my.v, j) * K + lane;
            float d = pp[0] * qq[0];
            if constexpr (E == 2) d = d + pp[64] * qq[64];
            d = reduce_wave(d, OpAdd());
            const double err = (double)(r - d);
            acc += err * err;
        }
    }
    block_sum_to_global(acc, sum_sq);
}

template <int K>
__global__ __launch_bounds__(kBlock) void rmse_grouped_kernel(const mf_node* __restrict__ test, uint32_t test_n, void* const* __restrict__ p, void* const* __restrict__ q,
                                                             const uint32_t* __restrict__ user_end, const uint32_t* __restrict__ item_end,
                                                             const uint8_t* __restrict__ user_prec, const uint8_t* __restrict__ item_prec,
                                                             uint32_t user_groups, uint32_t item_groups, double* sum_sq)
{
    constexpr int E = K / 64;
    extern __shared__ __align__(16) uint8_t smem[];
    uint64_t* pptr_s = reinterpret_cast<uint64_t*>(smem);
    uint64_t* qptr_s = pptr_s + user_groups;
    uint32_t* uend_s = reinterpret_cast<uint32_t*>(qptr_s + item_groups);
    uint32_t* iend_s = uend_s + user_groups;
    uint8_t* uprec_s = reinterpret_cast<uint8_t*>(iend_s + item_groups);
    uint8_t* iprec_s = uprec_s + user_groups;
    for (uint32_t g = threadIdx.x; g < user_groups; g += blockDim.x) { pptr_s[g] = reinterpret_cast<uint64_t>(p[g]); uend_s[g] = user_end[g]; uprec_s[g] = user_prec[g]; }
    for (uint32_t g = threadIdx.x; g < item_groups; g += blockDim.x) { qptr_s[g] = reinterpret_cast<uint64_t>(q[g]); iend_s[g] = item_end[g]; iprec_s[g] = item_prec[g]; }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const uint32_t waves = gridDim.x * kWavesPerBlock;
    const uint32_t wid = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    double acc = 0;
    for (uint64_t base = (uint64_t)wid * kWave; base < test_n; base += (uint64_t)waves * kWave) {
        const uint64_t left = test_n - base;
        const int n = left < (uint64_t)kWave ? (int)left : kWave;
        Rating my = {0.f, 0u, 0u};
        uint64_t pptr = 0, qptr = 0; uint32_t flags = 4u;
        if (lane < n) {
            my = load_rating(test, (uint32_t)(base + lane));
            const uint32_t ug = group_of(uend_s, user_groups, my.u), ig = group_of(iend_s, item_groups, my.v);
            const bool ok = my.u <= uend_s[ug] && my.v <= iend_s[ig];
            const uint32_t urow = ug ? my.u - uend_s[ug - 1] - 1 : my.u;
            const uint32_t irow = ig ? my.v - iend_s[ig - 1] - 1 : my.v;
            const uint32_t up = uprec_s[ug] ? 1u : 0u, ip = iprec_s[ig] ? 1u : 0u;
            pptr = pptr_s[ug] + (uint64_t)urow * (K * (up ? 4u : 2u));
            qptr = qptr_s[ig] + (uint64_t)irow * (K * (ip ? 4u : 2u));
            flags = up | (ip << 1) | (ok ? 0u : 4u);
        }
        for (int j = 0; j < n; ++j) {
            const uint32_t f = bcast(flags, j);
            if (f & 4u) continue;
            const float r = bcast(my.r, j);
            const uint64_t pa = bcast(pptr, j), qa = bcast(qptr, j);
            float pv[E], qv[E];
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const int el = lane + 64 * e;
                pv[e] = (f & 1u) ? reinterpret_cast<const float*>(pa)[el] : (float)from_bits<half_t>(reinterpret_cast<const uint16_t*>(pa)[el]);
                qv[e] = (f & 2u) ? reinterpret_cast<const float*>(qa)[el] : (float)from_bits<half_t>(reinterpret_cast<const uint16_t*>(qa)[el]);
            }
            float d = pv[0] * qv[0];
            if constexpr (E == 2) d = d + pv[1] * qv[1];
            d = reduce_wave(d, OpAdd());
            const double err = (double)(r - d);
            acc += err * err;
        }
    }
    block_sum_to_global(acc, sum_sq);
}

// ---- model init (model_init.cu:19-28): N(0,1)*0.01 from counter-derived bits ----------------------
// ln x, x in (0,1], from +,-,*,/ only (identical bits on any IEEE machine).
__device__ __forceinline__ double det_log(double x)
{
    const uint64_t b = __builtin_bit_cast(uint64_t, x);
    int e = (int)((b >> 52) & 0x7ff) - 1022;
    double m = __builtin_bit_cast(double, (b & 0x000fffffffffffffull) | 0x3fe0000000000000ull);
    if (m < 0.70710678118654752440) { m = m * 2.0; e = e - 1; }
    const double s = (m - 1.0) / (m + 1.0);
    const double s2 = s * s;
    double acc = 1.0 / 21.0;
    acc = acc * s2 + 1.0 / 19.0;
    acc = acc * s2 + 1.0 / 17.0;
    acc = acc * s2 + 1.0 / 15.0;
    acc = acc * s2 + 1.0 / 13.0;
    acc = acc * s2 + 1.0 / 11.0;
    acc = acc * s2 + 1.0 / 9.0;
    acc = acc * s2 + 1.0 / 7.0;
    acc = acc * s2 + 1.0 / 5.0;
    acc = acc * s2 + 1.0 / 3.0;
    acc = acc * s2 + 1.0;
    const double lnm = (2.0 * s) * acc;
    return (double)e * 0.69314718055994530942 + lnm;
}
__device__ __forceinline__ double det_cos2pi(double t)
{
    const double t4 = t * 4.0;
    const int q = (int)t4;
    const double f = t4 - (double)q;
    const double a = f * 1.57079632679489661923;
    const double a2 = a * a;
    double c = 1.0 / 2432902008176640000.0;
    c = -1.0 / 6402373705728000.0 + a2 * c;
    c = 1.0 / 20922789888000.0 + a2 * c;
    c = -1.0 / 87178291200.0 + a2 * c;
    c = 1.0 / 479001600.0 + a2 * c;
    c = -1.0 / 3628800.0 + a2 * c;
    c = 1.0 / 40320.0 + a2 * c;
    c = -1.0 / 720.0 + a2 * c;
    c = 1.0 / 24.0 + a2 * c;
    c = -1.0 / 2.0 + a2 * c;
    c = 1.0 + a2 * c;
    double s = 1.0 / 51090942171709440000.0;
    s = -1.0 / 121645100408832000.0 + a2 * s;
    s = 1.0 / 355687428096000.0 + a2 * s;
    s = -1.0 / 1307674368000.0 + a2 * s;
    s = 1.0 / 6227020800.0 + a2 * s;
    s = -1.0 / 39916800.0 + a2 * s;
    s = 1.0 / 362880.0 + a2 * s;
    s = -1.0 / 5040.0 + a2 * s;
    s = 1.0 / 120.0 + a2 * s;
    s = -1.0 / 6.0 + a2 * s;
    s = 1.0 + a2 * s;
    s = a * s;
    switch (q & 3) { case 0: return c; case 1: return -s; case 2: return -c; default: return s; }
}
// N(0,1) from 64 bits (Box-Muller over the two 32-bit halves)
__device__ __forceinline__ double det_normal(uint64_t h)
{
    const uint32_t a = (uint32_t)(h >> 32), b = (uint32_t)h;
    const double u1 = ((double)a + 1.0) * 2.3283064365386962890625e-10;
    const double u2 = (double)b * 2.3283064365386962890625e-10;
    const double rad = __builtin_sqrt(-2.0 * det_log(u1));
    return rad * det_cos2pi(u2);
}
__global__ __launch_bounds__(kStreamBlock) void init_normal_kernel(float* __restrict__ out, uint64_t n, uint64_t base, double scale)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = (float)(det_normal(mix64(base ^ i)) * scale);
}

// ---- seeded synthetic ratings (mf_generate_ratings) ------------------------------------------------
struct SynthTables {
    const double* user_cdf; const double* item_cdf;       // cumulative Zipf weights, last entry 1.0
    const uint32_t* user_perm; const uint32_t* item_perm; // popularity rank -> id
    const float* U; const float* V;                       // [rows][rank] factors, or null (bimodal)
};
// smallest index whose cumulative weight exceeds x (x in [0,1), cdf[count-1] = 1)
__device__ __forceinline__ uint32_t cdf_rank(const double* cdf, uint32_t count, double x)
{
    uint32_t lo = 0, hi = count - 1;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (x < cdf[mid]) hi = mid; else lo = mid + 1;
    }
    return lo;
}
__global__ __launch_bounds__(kStreamBlock) void generate_ratings_kernel(mf_synth_config c, SynthTables t, uint64_t key, uint64_t first, uint64_t count,
                                                                      float inv_step, mf_node* __restrict__ out)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const uint64_t j = first + i;
        const double xu = (double)(mix64(key ^ (j * 4 + 0)) >> 11) * 1.1102230246251565404e-16;      // 53 bits in [0,1)
        const double xi = (double)(mix64(key ^ (j * 4 + 1)) >> 11) * 1.1102230246251565404e-16;
        const uint32_t u = t.user_perm[cdf_rank(t.user_cdf, c.n_users, xu)];
        const uint32_t v = t.item_perm[cdf_rank(t.item_cdf, c.n_items, xi)];
        const float nz = (float)(det_normal(mix64(key ^ (j * 4 + 2))) * (double)c.noise);
        float r;
        if (c.bimodal) {
            const double xm = (double)(mix64(key ^ (j * 4 + 3)) >> 11) * 1.1102230246251565404e-16;
            const float m = xm < 0.5 ? 20.0f : 80.0f;
            r = fminf(fmaxf(roundf(m + nz), c.lo), c.hi) * 0.04f + 1.0f;
        } else {
            float dot = 0.0f;
            for (uint32_t k = 0; k < c.rank; ++k) dot = dot + t.U[(size_t)u * c.rank + k] * t.V[(size_t)v * c.rank + k];
            const float val = (dot + c.mean) + nz;
            r = fminf(fmaxf(roundf(val * inv_step) * c.step, c.lo), c.hi);
        }
        out[i].r = r; out[i].u = u; out[i].i = v;
    }
}

// ---- preprocessing (preprocess_utils.h:6-36) ---------------------------------------------------
__global__ __launch_bounds__(kStreamBlock) void iota_kernel(uint32_t* __restrict__ a, uint32_t n)
{
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) a[i] = i;
}
// user_item_histogram (preprocess_utils.h:13-19).  With Zipf-like popularity a few counters take percents of all
// increments, and global atomics on one address serialise at the memory side.  Each workgroup therefore counts in
// an LDS table first: kHistSlots (id, count) slots per side, a slot claimed by the first id that hashes to it (two
// probes); ids that find both probes taken go to the global counter directly.  Popular ids claim their slots within
// the first few ratings, so nearly all of their increments are LDS atomics, flushed once per workgroup.
constexpr int kHistBlock = 1024;
constexpr uint32_t kHistLog = 12, kHistSlots = 1u << kHistLog;
__device__ __forceinline__ void histogram_count(uint32_t* tag, uint32_t* cnt, uint32_t id, uint32_t* global_bin)
{
    uint32_t s = (id * 2654435761u) >> (32 - kHistLog);
#pragma unroll
    for (int probe = 0; probe < 2; ++probe, s ^= 1u) {
        uint32_t t = tag[s];
        if (t == 0u) t = atomicCAS(&tag[s], 0u, id + 1u);
        if (t == 0u || t == id + 1u) { atomicAdd(&cnt[s], 1u); return; }
    }
    atomicAdd(&global_bin[id], 1u);
}
__global__ __launch_bounds__(kHistBlock) void histogram_kernel(const mf_node* __restrict__ R, uint32_t n, uint32_t per_block, uint32_t* user_bin, uint32_t* item_bin)
{
    __shared__ uint32_t tab[4 * kHistSlots];          // user tags, user counts, item tags, item counts: 64 KB
    for (uint32_t i = threadIdx.x; i < 4 * kHistSlots; i += blockDim.x) tab[i] = 0u;
    __syncthreads();
    uint32_t* utag = tab, *ucnt = tab + kHistSlots, *itag = tab + 2 * kHistSlots, *icnt = tab + 3 * kHistSlots;
    const uint64_t begin = (uint64_t)blockIdx.x * per_block;
    const uint64_t end = begin + per_block < n ? begin + per_block : n;
    for (uint64_t i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(R + i);
        histogram_count(utag, ucnt, __builtin_nontemporal_load(w + 1), user_bin);
        histogram_count(itag, icnt, __builtin_nontemporal_load(w + 2), item_bin);
    }
    __syncthreads();
    for (uint32_t s = threadIdx.x; s < kHistSlots; s += blockDim.x) {
        if (utag[s]) atomicAdd(&user_bin[utag[s] - 1u], ucnt[s]);
        if (itag[s]) atomicAdd(&item_bin[itag[s] - 1u], icnt[s]);
    }
}
__global__ __launch_bounds__(kStreamBlock) void reindex_kernel(mf_node* R, const uint32_t* __restrict__ user2sorted, const uint32_t* __restrict__ item2sorted, uint32_t n)
{
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t u = R[i].u, v = R[i].i;
        R[i].u = user2sorted[u];
        R[i].i = item2sorted[v];
    }
}

static size_t group_table_lds(uint32_t ug, uint32_t ig) { return (size_t)(ug + ig) * (8 + 4 + 1) + 16; }

}  // namespace mf

using namespace mf;

// ---- access-pattern probe ------------------------------------------------------------------------
// The memory traffic of one epoch of updates without the arithmetic: per rating the two rows are read and, where
// the hot-row tables keep the update, written back unchanged (the loaded value plus `zero`, a kernel argument the
// compiler cannot fold).  The same draw as the update kernels' thinning decides; a kept update of a hot row is a
// store here too.  What it sustains is the ceiling the memory system sets for this sequence of addresses and this
// write policy, the figure the update kernels' epoch time is compared with.
template <int BYTES, bool COH, int BYTES_Q = BYTES>       // bytes per lane and side: a row is 64 * BYTES bytes
__global__ __launch_bounds__(kBlock) void row_traffic_probe_kernel(const mf_node* R, uint32_t n, uint8_t* P, uint8_t* Q, uint32_t per_worker,
                                                                  const uint8_t* keep_u, const uint8_t* keep_v, const uint16_t* slot_u, const uint16_t* slot_v,
                                                                  uint32_t slots_u, uint32_t slots_v, uint8_t* RP, uint8_t* RQ, uint64_t key, uint32_t zero)
{
    using T = typename std::conditional<BYTES == 8, uint64_t, typename std::conditional<BYTES == 4, uint32_t, uint16_t>::type>::type;
    using TQ = typename std::conditional<BYTES_Q == 8, uint64_t, typename std::conditional<BYTES_Q == 4, uint32_t, uint16_t>::type>::type;
    constexpr int kDepth = 4;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t worker = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const uint64_t begin64 = (uint64_t)worker * per_worker;
    if (begin64 >= n) return;
    const uint32_t xcd = xcd_id();
    const uint32_t begin = (uint32_t)begin64, end = (uint64_t)begin + per_worker < n ? begin + per_worker : n;
    for (uint32_t base = begin; base < end; base += kWave) {
        uint32_t mu = 0, mv = 0, keep = 0;      // keep: bit0/bit1 write the P/Q row back, bit2/bit3 the row is this XCD's copy of a replicated row
        if (base + (uint32_t)lane < end) {
            const Rating x = load_rating(R, base + (uint32_t)lane);
            mu = x.u; mv = x.v; keep = 3u;
            if (keep_u) {
                const uint32_t rnd = (uint32_t)(mix64(key ^ (((uint64_t)(base + (uint32_t)lane) << 20) ^ (uint64_t)worker ^ 0x7468696eull)) >> 40);
                const uint32_t ku = keep_u[mu], kv = keep_v[mv];
                if (ku == kKeepReplicated || ku == kKeepReplicatedAdded) { keep |= 4u; mu = xcd * slots_u + slot_u[mu]; }
                else if (ku != 255u && (((rnd & 0xfffu) * 255u) >> 12) > ku) keep &= ~1u;
                if (kv == kKeepReplicated || kv == kKeepReplicatedAdded) { keep |= 8u; mv = xcd * slots_v + slot_v[mv]; }
                else if (kv != 255u && (((rnd >> 12) * 255u) >> 12) > kv) keep &= ~2u;
            }
        }
        const int cnt = end - base < (uint32_t)kWave ? (int)(end - base) : kWave;
        for (int j0 = 0; j0 < cnt; j0 += kDepth) {
            T a[kDepth]; TQ b[kDepth]; T* pa[kDepth]; TQ* pb[kDepth]; uint32_t kp[kDepth];
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
                const int j = j0 + d < cnt ? j0 + d : cnt - 1;
                kp[d] = j0 + d < cnt ? bcast(keep, j) : 0u;
                const uint32_t flags = bcast(keep, j);
                pa[d] = reinterpret_cast<T*>(((flags & 4u) ? RP : P) + (size_t)bcast(mu, j) * (kWave * BYTES)) + lane;
                pb[d] = reinterpret_cast<TQ*>(((flags & 8u) ? RQ : Q) + (size_t)bcast(mv, j) * (kWave * BYTES_Q)) + lane;
                a[d] = row_load(pa[d]); b[d] = row_load(pb[d]);
            }
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
                if (kp[d] & 4u) row_store<false>(pa[d], (T)(a[d] + (T)zero)); else if (kp[d] & 1u) row_store<COH>(pa[d], (T)(a[d] + (T)zero));
                if (kp[d] & 8u) row_store<false>(pb[d], (TQ)(b[d] + (TQ)zero)); else if (kp[d] & 2u) row_store<COH>(pb[d], (TQ)(b[d] + (TQ)zero));
            }
        }
    }
}

namespace {
// cumulative weights (rank+1)^-alpha, normalised by their sum; summed in rank order in double
std::vector<double> zipf_cdf(uint32_t count, float alpha)
{
    std::vector<double> cdf(count);
    double sum = 0.0;
    for (uint32_t i = 0; i < count; ++i) { sum += std::pow((double)(i + 1), -(double)alpha); cdf[i] = sum; }
    for (uint32_t i = 0; i < count; ++i) cdf[i] = cdf[i] / sum;
    return cdf;
}
// Fisher-Yates with the counter-based generator
std::vector<uint32_t> seeded_permutation(uint32_t count, uint64_t base)
{
    std::vector<uint32_t> p(count);
    for (uint32_t i = 0; i < count; ++i) p[i] = i;
    for (uint32_t i = count; i-- > 1;) { const uint32_t j = (uint32_t)(mix64(base ^ (uint64_t)i) % ((uint64_t)i + 1)); std::swap(p[i], p[j]); }
    return p;
}
}  // namespace

extern "C" {

int mf_transform_float2half(const float* in, uint16_t* out, uint64_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!in || !out) return invalid("mf_transform_float2half: null pointer");
    if ((reinterpret_cast<uintptr_t>(in) & 7) || (reinterpret_cast<uintptr_t>(out) & 3)) return invalid("mf_transform_float2half: input must be 8-byte and output 4-byte aligned");
    hipLaunchKernelGGL(float2half_kernel, dim3(stream_grid(n / 2 + 1, 4)), dim3(kStreamBlock), 0, as_stream(stream), in, out, n);
    return launch_status("mf_transform_float2half");
}
int mf_transform_half2float(const uint16_t* in, float* out, uint64_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!in || !out) return invalid("mf_transform_half2float: null pointer");
    if ((reinterpret_cast<uintptr_t>(in) & 3) || (reinterpret_cast<uintptr_t>(out) & 7)) return invalid("mf_transform_half2float: input must be 4-byte and output 8-byte aligned");
    hipLaunchKernelGGL(half2float_kernel, dim3(stream_grid(n / 2 + 1, 4)), dim3(kStreamBlock), 0, as_stream(stream), in, out, n);
    return launch_status("mf_transform_half2float");
}

int mf_cpyparams2grouped_params(const float* original_params, void* const* converted_params,
                                const uint32_t* group_end_idx, const uint32_t* entity2group,
                                const uint32_t* entity2sorted_idx, int k, uint32_t n, uint32_t group_num, void* stream)
{
    if (k != 64 && k != 128) return invalid("mf_cpyparams2grouped_params: k must be 64 or 128 (got %d)", k);
    if (n == 0) return MF_OK;
    if (!original_params || !converted_params || !group_end_idx || !entity2group || !entity2sorted_idx || group_num == 0)
        return invalid("mf_cpyparams2grouped_params: null pointer or no groups");
    const uint32_t grid = stream_grid((uint64_t)n * kWave);
    if (k == 128) hipLaunchKernelGGL(scatter_to_groups_kernel<128>, dim3(grid), dim3(kBlock), 0, as_stream(stream), original_params, converted_params, group_end_idx, entity2group, entity2sorted_idx, n, group_num);
    else hipLaunchKernelGGL(scatter_to_groups_kernel<64>, dim3(grid), dim3(kBlock), 0, as_stream(stream), original_params, converted_params, group_end_idx, entity2group, entity2sorted_idx, n, group_num);
    return launch_status("mf_cpyparams2grouped_params");
}

int mf_grouped_params2dense(void* const* group_ptr, const uint32_t* group_end_idx, const uint8_t* group_prec_info,
                            float* dense, int k, uint32_t n, uint32_t group_num, void* stream)
{
    if (k != 64 && k != 128) return invalid("mf_grouped_params2dense: k must be 64 or 128 (got %d)", k);
    if (n == 0) return MF_OK;
    if (!group_ptr || !group_end_idx || !group_prec_info || !dense || group_num == 0) return invalid("mf_grouped_params2dense: null pointer or no groups");
    const uint32_t grid = stream_grid((uint64_t)n * kWave);
    if (k == 128) hipLaunchKernelGGL(gather_from_groups_kernel<128>, dim3(grid), dim3(kBlock), 0, as_stream(stream), group_ptr, group_end_idx, group_prec_info, dense, n, group_num);
    else hipLaunchKernelGGL(gather_from_groups_kernel<64>, dim3(grid), dim3(kBlock), 0, as_stream(stream), group_ptr, group_end_idx, group_prec_info, dense, n, group_num);
    return launch_status("mf_grouped_params2dense");
}

int mf_group_error(float* grad_sum_norm, const float* norm_sum, uint32_t norm_blocks, const uint8_t* group_prec_info,
                   const float* initial_error, float* error_out, int k, uint32_t group_num, void* stream)
{
    if (k != 64 && k != 128) return invalid("mf_group_error: k must be 64 or 128 (got %d)", k);
    if (group_num == 0) return MF_OK;
    if (!grad_sum_norm || !norm_sum || !group_prec_info || !initial_error || !error_out) return invalid("mf_group_error: null pointer");
    hipLaunchKernelGGL(group_error_kernel, dim3(group_num), dim3(kWave), 0, as_stream(stream), grad_sum_norm, norm_sum, norm_blocks, group_prec_info, initial_error, error_out, k, group_num);
    return launch_status("mf_group_error");
}

int mf_test_rmse(const mf_node* test, uint32_t test_n, const float* p, const float* q, int k, double* sum_sq, void* stream)
{
    if (k != 64 && k != 128) return invalid("mf_test_rmse: k must be 64 or 128 (got %d)", k);
    if (test_n == 0) return MF_OK;
    if (!test || !p || !q || !sum_sq) return invalid("mf_test_rmse: null pointer");
    const uint32_t grid = stream_grid((uint64_t)test_n * 4);
    if (k == 128) hipLaunchKernelGGL(rmse_dense_kernel<128>, dim3(grid), dim3(kBlock), 0, as_stream(stream), test, test_n, p, q, sum_sq);
    else hipLaunchKernelGGL(rmse_dense_kernel<64>, dim3(grid), dim3(kBlock), 0, as_stream(stream), test, test_n, p, q, sum_sq);
    return launch_status("mf_test_rmse");
}

int mf_test_rmse_grouped(const mf_node* test, uint32_t test_n, void* const* p, void* const* q, int k,
                         const uint32_t* user_group_end_idx, const uint32_t* item_group_end_idx,
                         const uint8_t* user_group_prec_info, const uint8_t* item_group_prec_info,
                         uint32_t user_group_num, uint32_t item_group_num, double* sum_sq, void* stream)
{
    if (k != 64 && k != 128) return invalid("mf_test_rmse_grouped: k must be 64 or 128 (got %d)", k);
    if (test_n == 0) return MF_OK;
    if (!test || !p || !q || !sum_sq || !user_group_end_idx || !item_group_end_idx || !user_group_prec_info || !item_group_prec_info)
        return invalid("mf_test_rmse_grouped: null pointer");
    if (user_group_num == 0 || item_group_num == 0) return invalid("mf_test_rmse_grouped: at least one group per side is required");
    const size_t lds = group_table_lds(user_group_num, item_group_num);
    if (lds > 60 * 1024) return invalid("mf_test_rmse_grouped: group tables need %zu bytes of LDS", lds);
    const uint32_t grid = stream_grid((uint64_t)test_n * 4);
    if (k == 128) hipLaunchKernelGGL(rmse_grouped_kernel<128>, dim3(grid), dim3(kBlock), lds, as_stream(stream), test, test_n, p, q, user_group_end_idx, item_group_end_idx, user_group_prec_info, item_group_prec_info, user_group_num, item_group_num, sum_sq);
    else hipLaunchKernelGGL(rmse_grouped_kernel<64>, dim3(grid), dim3(kBlock), lds, as_stream(stream), test, test_n, p, q, user_group_end_idx, item_group_end_idx, user_group_prec_info, item_group_prec_info, user_group_num, item_group_num, sum_sq);
    return launch_status("mf_test_rmse_grouped");
}

int mf_init_rand_feature(float* array, uint64_t n, uint64_t seed, uint64_t stream_id, void* stream)
{
    if (n == 0) return MF_OK;
    if (!array) return invalid("mf_init_rand_feature: null pointer");
    const uint64_t base = mix64(mix64(seed ^ 0x494E49544E4F524Dull) + stream_id);
    hipLaunchKernelGGL(init_normal_kernel, dim3(stream_grid(n)), dim3(kStreamBlock), 0, as_stream(stream), array, n, base, 0.01);
    return launch_status("mf_init_rand_feature");
}

int mf_init_idx_arr(uint32_t* arr, uint32_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!arr) return invalid("mf_init_idx_arr: null pointer");
    hipLaunchKernelGGL(iota_kernel, dim3(stream_grid(n)), dim3(kStreamBlock), 0, as_stream(stream), arr, n);
    return launch_status("mf_init_idx_arr");
}

int mf_user_item_histogram(const mf_node* R, uint32_t n, uint32_t* user_bin, uint32_t* item_bin, void* stream)
{
    if (n == 0) return MF_OK;
    if (!R || !user_bin || !item_bin) return invalid("mf_user_item_histogram: null pointer");
    // one workgroup per 256k ratings (a flush costs up to 8192 global atomics), at least one per CU when n allows
    uint32_t per_block = 1u << 18;
    while (per_block > 16384u && (uint64_t)per_block * 256u > n) per_block >>= 1;
    const uint32_t blocks = (uint32_t)(((uint64_t)n + per_block - 1) / per_block);
    hipLaunchKernelGGL(histogram_kernel, dim3(blocks), dim3(kHistBlock), 0, as_stream(stream), R, n, per_block, user_bin, item_bin);
    return launch_status("mf_user_item_histogram");
}

int mf_matrix_reconst_triplet(mf_node* R, const uint32_t* user2sorted_idx, const uint32_t* item2sorted_idx, uint32_t n, void* stream)
{
    if (n == 0) return MF_OK;
    if (!R || !user2sorted_idx || !item2sorted_idx) return invalid("mf_matrix_reconst_triplet: null pointer");
    hipLaunchKernelGGL(reindex_kernel, dim3(stream_grid(n)), dim3(kStreamBlock), 0, as_stream(stream), R, user2sorted_idx, item2sorted_idx, n);
    return launch_status("mf_matrix_reconst_triplet");
}

int mf_row_traffic_probe(const mf_node* R, uint32_t n, void* p, void* q, uint32_t row_bytes, uint32_t num_workers,
                         uint64_t seed, void* stream, const mf_hogwild_options* options)
{
    return mf_row_traffic_probe_sides(R, n, p, q, row_bytes, row_bytes, num_workers, seed, stream, options);
}
int mf_row_traffic_probe_sides(const mf_node* R, uint32_t n, void* p, void* q, uint32_t row_bytes, uint32_t item_row_bytes, uint32_t num_workers,
                               uint64_t seed, void* stream, const mf_hogwild_options* options)
{
    if (n == 0) return MF_OK;
    if (!R || !p || !q) return invalid("mf_row_traffic_probe: null pointer");
    if (row_bytes != 128 && row_bytes != 256 && row_bytes != 512) return invalid("mf_row_traffic_probe: row_bytes must be 128, 256 or 512 (got %u)", row_bytes);
    if (item_row_bytes != 128 && item_row_bytes != 256 && item_row_bytes != 512) return invalid("mf_row_traffic_probe: row_bytes must be 128, 256 or 512 (got %u)", item_row_bytes);
    if (num_workers == 0) return invalid("mf_row_traffic_probe: num_workers must be positive");
    mf_hogwild_options o = {};
    if (options) o = *options;
    if ((o.user_keep == nullptr) != (o.item_keep == nullptr)) return invalid("mf_row_traffic_probe: give both keep tables or neither");
    if ((o.user_slots && (!o.user_slot || !o.user_replicas)) || (o.item_slots && (!o.item_slot || !o.item_replicas))) return invalid("mf_row_traffic_probe: replicated rows need slot tables and replica arrays");
    if ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(q)) & 7) return invalid("mf_row_traffic_probe: rows must be 8-byte aligned");
    const bool coherent = o.cached_rows == 0;
    const uint8_t* user_keep = o.user_keep; const uint8_t* item_keep = o.item_keep;
    const uint32_t per_worker = (uint32_t)(((uint64_t)n + num_workers - 1) / num_workers);
    const dim3 grid((num_workers + kWavesPerBlock - 1) / kWavesPerBlock), block(kBlock);
    uint8_t* P = static_cast<uint8_t*>(p); uint8_t* Q = static_cast<uint8_t*>(q);
    uint8_t* RP = static_cast<uint8_t*>(o.user_replicas); uint8_t* RQ = static_cast<uint8_t*>(o.item_replicas);
    const uint64_t key = mix64(seed ^ 0x70726f6265ull);
#define MF_PROBE(BYTES, COH) hipLaunchKernelGGL((row_traffic_probe_kernel<BYTES, COH>), grid, block, 0, as_stream(stream), R, n, P, Q, per_worker, user_keep, item_keep, o.user_slot, o.item_slot, o.user_slots, o.item_slots, RP, RQ, key, 0u)
#define MF_PROBE2(BP, BQ) hipLaunchKernelGGL((row_traffic_probe_kernel<BP, true, BQ>), grid, block, 0, as_stream(stream), R, n, P, Q, per_worker, user_keep, item_keep, o.user_slot, o.item_slot, o.user_slots, o.item_slots, RP, RQ, key, 0u)
    if (row_bytes != item_row_bytes) {
        // rows of different widths on the two sides: MASCOT after one side's groups have been promoted
        if (!coherent) return invalid("mf_row_traffic_probe_sides: sides of different widths are probed with device-coherent stores only");
        if (row_bytes == 256 && item_row_bytes == 512) MF_PROBE2(4, 8);
        else if (row_bytes == 512 && item_row_bytes == 256) MF_PROBE2(8, 4);
        else if (row_bytes == 128 && item_row_bytes == 256) MF_PROBE2(2, 4);
        else if (row_bytes == 256 && item_row_bytes == 128) MF_PROBE2(4, 2);
        else return invalid("mf_row_traffic_probe_sides: the wider side's rows must be twice the other's");
    }
    else if (row_bytes == 128) { if (coherent) MF_PROBE(2, true); else MF_PROBE(2, false); }
    else if (row_bytes == 256) { if (coherent) MF_PROBE(4, true); else MF_PROBE(4, false); }
    else { if (coherent) MF_PROBE(8, true); else MF_PROBE(8, false); }
#undef MF_PROBE2
#undef MF_PROBE
    return launch_status("mf_row_traffic_probe");
}

int mf_synth_baseline_config(int config, mf_synth_config* out)
{
    if (!out) return invalid("mf_synth_baseline_config: null pointer");
    //                          users    items    train       test     alpha_u alpha_i rank noise  mean  step  lo    hi   bimodal
    static const mf_synth_config table[5] = {
        {5000u, 2000u, 400000ull, 100000ull, 1.0f, 1.0f, 8u, 0.8f, 3.5f, 1.0f, 1.0f, 5.0f, 0u},
        {70000u, 10700u, 8000000ull, 2000000ull, 0.9f, 0.9f, 16u, 0.8f, 3.5f, 0.5f, 0.5f, 5.0f, 0u},
        {162000u, 59000u, 20000000ull, 5000000ull, 1.0f, 1.0f, 16u, 0.8f, 3.5f, 0.5f, 0.5f, 5.0f, 0u},
        {480000u, 17800u, 100000000ull, 1400000ull, 0.8f, 1.1f, 32u, 0.9f, 3.6f, 1.0f, 1.0f, 5.0f, 0u},
        {1000000u, 625000u, 250000000ull, 4000000ull, 1.2f, 1.2f, 0u, 15.0f, 0.0f, 1.0f, 0.0f, 100.0f, 1u},
    };
    if (config < 1 || config > 5) return invalid("mf_synth_baseline_config: configurations are numbered 1..5 (got %d)", config);
    *out = table[config - 1];
    return MF_OK;
}

static int check_synth(const char* who, const mf_synth_config* cfg)
{
    if (!cfg) return invalid("%s: null configuration", who);
    if (cfg->n_users == 0 || cfg->n_items == 0) return invalid("%s: no users or no items", who);
    if (!cfg->bimodal && (cfg->rank == 0 || cfg->rank > 1024u)) return invalid("%s: rank must be 1..1024 (got %u)", who, cfg->rank);
    if (!(cfg->step > 0.0f) || !(cfg->lo <= cfg->hi)) return invalid("%s: step must be positive and lo <= hi", who);
    return MF_OK;
}
// Workspace layout of the generator's tables: user CDF, item CDF (binary64), user permutation, item permutation
// (uint32), and unless bimodal the factors U [users][rank], V [items][rank] (binary32); every part 256-byte aligned.
struct SynthLayout { size_t ucdf, icdf, uperm, iperm, U, V, total; };
static SynthLayout synth_layout(const mf_synth_config& c)
{
    auto al = [](size_t b) { return (b + 255) / 256 * 256; };
    SynthLayout l;
    l.ucdf = 0; l.icdf = l.ucdf + al((size_t)c.n_users * 8); l.uperm = l.icdf + al((size_t)c.n_items * 8);
    l.iperm = l.uperm + al((size_t)c.n_users * 4); l.U = l.iperm + al((size_t)c.n_items * 4);
    const size_t fu = c.bimodal ? 0 : al((size_t)c.n_users * c.rank * 4), fv = c.bimodal ? 0 : al((size_t)c.n_items * c.rank * 4);
    l.V = l.U + fu; l.total = l.V + fv;
    return l;
}
static SynthTables synth_tables(const mf_synth_config& c, const void* workspace)
{
    const SynthLayout l = synth_layout(c);
    const uint8_t* ws = static_cast<const uint8_t*>(workspace);
    SynthTables t = {};
    t.user_cdf = reinterpret_cast<const double*>(ws + l.ucdf); t.item_cdf = reinterpret_cast<const double*>(ws + l.icdf);
    t.user_perm = reinterpret_cast<const uint32_t*>(ws + l.uperm); t.item_perm = reinterpret_cast<const uint32_t*>(ws + l.iperm);
    if (!c.bimodal) { t.U = reinterpret_cast<const float*>(ws + l.U); t.V = reinterpret_cast<const float*>(ws + l.V); }
    return t;
}
static uint64_t synth_key(uint64_t seed) { return mix64(seed ^ 0x53594E5448455449ull); }

size_t mf_synth_tables_bytes(const mf_synth_config* cfg)
{
    if (check_synth("mf_synth_tables_bytes", cfg)) return 0;
    return synth_layout(*cfg).total;
}
int mf_synth_build_tables(const mf_synth_config* cfg, uint64_t seed, void* workspace, size_t workspace_bytes, void* stream)
{
    if (int rc = check_synth("mf_synth_build_tables", cfg)) return rc;
    const mf_synth_config c = *cfg;
    const SynthLayout l = synth_layout(c);
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 256) return invalid("mf_synth_build_tables: the workspace must be non-null and 256-byte aligned");
    if (workspace_bytes < l.total) return invalid("mf_synth_build_tables: the workspace holds %zu bytes, the tables need %zu (mf_synth_tables_bytes)", workspace_bytes, l.total);
    hipStream_t st = as_stream(stream);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const uint64_t key = synth_key(seed);
    const std::vector<double> ucdf = zipf_cdf(c.n_users, c.user_alpha), icdf = zipf_cdf(c.n_items, c.item_alpha);
    const std::vector<uint32_t> uperm = seeded_permutation(c.n_users, mix64(key + 1)), iperm = seeded_permutation(c.n_items, mix64(key + 2));
    if (int rc = check_hip(hipMemcpyAsync(ws + l.ucdf, ucdf.data(), ucdf.size() * 8, hipMemcpyHostToDevice, st), "hipMemcpyAsync(synthetic tables)")) return rc;
    if (int rc = check_hip(hipMemcpyAsync(ws + l.icdf, icdf.data(), icdf.size() * 8, hipMemcpyHostToDevice, st), "hipMemcpyAsync(synthetic tables)")) return rc;
    if (int rc = check_hip(hipMemcpyAsync(ws + l.uperm, uperm.data(), uperm.size() * 4, hipMemcpyHostToDevice, st), "hipMemcpyAsync(synthetic tables)")) return rc;
    if (int rc = check_hip(hipMemcpyAsync(ws + l.iperm, iperm.data(), iperm.size() * 4, hipMemcpyHostToDevice, st), "hipMemcpyAsync(synthetic tables)")) return rc;
    if (!c.bimodal) {
        const uint64_t nu = (uint64_t)c.n_users * c.rank, nv = (uint64_t)c.n_items * c.rank;
        hipLaunchKernelGGL(init_normal_kernel, dim3(stream_grid(nu)), dim3(kStreamBlock), 0, st, reinterpret_cast<float*>(ws + l.U), nu, mix64(key + 3), 0.5);
        hipLaunchKernelGGL(init_normal_kernel, dim3(stream_grid(nv)), dim3(kStreamBlock), 0, st, reinterpret_cast<float*>(ws + l.V), nv, mix64(key + 4), 0.5);
        if (int rc = launch_status("mf_synth_build_tables")) return rc;
    }
    // the host-side tables above go out of scope on return: wait for their copies (the one synchronisation of the generator)
    return check_hip(hipStreamSynchronize(st), "mf_synth_build_tables: hipStreamSynchronize");
}
int mf_generate_ratings_ws(const mf_synth_config* cfg, uint64_t seed, const void* tables, uint64_t first, uint64_t count, mf_node* out, void* stream)
{
    if (int rc = check_synth("mf_generate_ratings_ws", cfg)) return rc;
    if (count == 0) return MF_OK;
    if (!out || !tables) return invalid("mf_generate_ratings_ws: null output or tables");
    const mf_synth_config c = *cfg;
    hipLaunchKernelGGL(generate_ratings_kernel, dim3(stream_grid(count)), dim3(kStreamBlock), 0, as_stream(stream), c, synth_tables(c, tables), synth_key(seed), first, count, 1.0f / c.step, out);
    return launch_status("mf_generate_ratings_ws");
}
int mf_generate_ratings(const mf_synth_config* cfg, uint64_t seed, uint64_t first, uint64_t count, mf_node* out, void* stream)
{
    if (int rc = check_synth("mf_generate_ratings", cfg)) return rc;
    if (count == 0) return MF_OK;
    if (!out) return invalid("mf_generate_ratings: null output");
    const size_t bytes = synth_layout(*cfg).total;
    void* ws = nullptr;
    if (int rc = check_hip(hipMalloc(&ws, bytes), "mf_generate_ratings: hipMalloc(tables)")) return rc;
    int rc = mf_synth_build_tables(cfg, seed, ws, bytes, stream);
    if (rc == MF_OK) rc = mf_generate_ratings_ws(cfg, seed, ws, first, count, out, stream);
    if (rc == MF_OK) rc = check_hip(hipStreamSynchronize(as_stream(stream)), "mf_generate_ratings: hipStreamSynchronize");       // the tables are freed on return
    (void)hipFree(ws);
    return rc;
}

int mf_generate_ratings_host(const mf_synth_config* cfg, uint64_t seed, uint64_t first, uint64_t count, mf_node* host_out)
{
    if (count == 0) return MF_OK;
    if (!host_out) return invalid("mf_generate_ratings_host: null output");
    void* dev = nullptr;
    if (int rc = check_hip(hipMalloc(&dev, count * sizeof(mf_node)), "mf_generate_ratings_host: hipMalloc")) return rc;
    int rc = mf_generate_ratings(cfg, seed, first, count, static_cast<mf_node*>(dev), nullptr);
    if (rc == MF_OK) rc = check_hip(hipMemcpy(host_out, dev, count * sizeof(mf_node), hipMemcpyDeviceToHost), "mf_generate_ratings_host: hipMemcpy");
    (void)hipFree(dev);
    return rc;
}

}  // extern "C"
