// Device-side building blocks shared by the gfx950 kernels: wave64 cross-lane
// reductions (DPP row rotates + v_permlane{16,32}_swap), binary16 vector types,
// the counter-based window generator and the rating-chunk loader.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/mascot_hip.h"

namespace mf {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kBlock = 256;              // 4 wavefronts per workgroup
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxBlock = 1024;          // the sampled tail of a MASCOT epoch runs 16 wavefronts per workgroup

// ---- bit casts -----------------------------------------------------------------------
__device__ __forceinline__ uint32_t bits(float x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ uint32_t bits(int x) { return (uint32_t)x; }
__device__ __forceinline__ uint32_t bits(uint32_t x) { return x; }
__device__ __forceinline__ uint32_t bits(half2_t x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ uint32_t bits(half_t x) { return (uint32_t)__builtin_bit_cast(uint16_t, x); }
template <class T> __device__ __forceinline__ T from_bits(uint32_t b);
template <> __device__ __forceinline__ float from_bits<float>(uint32_t b) { return __builtin_bit_cast(float, b); }
template <> __device__ __forceinline__ int from_bits<int>(uint32_t b) { return (int)b; }
template <> __device__ __forceinline__ uint32_t from_bits<uint32_t>(uint32_t b) { return b; }
template <> __device__ __forceinline__ half2_t from_bits<half2_t>(uint32_t b) { return __builtin_bit_cast(half2_t, b); }
template <> __device__ __forceinline__ half_t from_bits<half_t>(uint32_t b) { return __builtin_bit_cast(half_t, (uint16_t)b); }

// ---- cross-lane moves ------------------------------------------------------------------
// Value held by lane (L ^ 32).
template <class T> __device__ __forceinline__ T lane_xor32(T x)
{
    auto r = __builtin_amdgcn_permlane32_swap(bits(x), bits(x), false, false);
    // r[0] = lanes 0-31 of x replicated in both halves, r[1] = lanes 32-63 replicated.
    return from_bits<T>((threadIdx.x & 32) ? r[0] : r[1]);
}
// Value held by lane ((L + N) mod 16) of the same row of 16 lanes.
template <int N, class T> __device__ __forceinline__ T row_ror(T x)
{
    // every lane has a source lane, so no previous value is needed (mov_dpp leaves it undefined: no register to clear)
    return from_bits<T>((uint32_t)__builtin_amdgcn_mov_dpp((int)bits(x), 0x120 + N, 0xf, 0xf, true));
}

// Reduction steps: every lane ends with op(own, partner); op must be commutative.
struct OpAdd { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; } };

template <class T, class Op> __device__ __forceinline__ T step_xor32(T x, Op op)
{
    auto r = __builtin_amdgcn_permlane32_swap(bits(x), bits(x), false, false);
    return op(from_bits<T>(r[0]), from_bits<T>(r[1]));
}
template <class T, class Op> __device__ __forceinline__ T step_xor16(T x, Op op)
{
    auto r = __builtin_amdgcn_permlane16_swap(bits(x), bits(x), false, false);
    return op(from_bits<T>(r[0]), from_bits<T>(r[1]));
}
template <int N, class T, class Op> __device__ __forceinline__ T step_ror(T x, Op op) { return op(x, row_ror<N>(x)); }

// Tail shared by all layouts: the reference's shfl_down 8,4,2,1 steps inside a row of 16.
template <class T, class Op> __device__ __forceinline__ T reduce_row16(T x, Op op)
{
    x = step_ror<8>(x, op);
    x = step_ror<4>(x, op);
    x = step_ror<2>(x, op);
    x = step_ror<1>(x, op);
    return x;
}
// All 64 lanes, order 32,16,8,4,2,1.  With one element per lane (element L) this is exactly the
// reference's (m[l] + m[l+32]) followed by its 16,8,4,2,1 tree (sgd/sgd_kernel_k64.h:49-57).
template <class T, class Op> __device__ __forceinline__ T reduce_wave(T x, Op op)
{
    x = step_xor32(x, op);
    x = step_xor16(x, op);
    return reduce_row16(x, op);
}
// The reference's tree over 32 lanes when lanes L and L^32 already hold the same value.
template <class T, class Op> __device__ __forceinline__ T reduce_half_wave(T x, Op op)
{
    x = step_xor16(x, op);
    return reduce_row16(x, op);
}

__device__ __forceinline__ uint32_t bcast(uint32_t v, int lane) { return (uint32_t)__builtin_amdgcn_readlane((int)v, lane); }
__device__ __forceinline__ float bcast(float v, int lane) { return from_bits<float>(bcast(bits(v), lane)); }
__device__ __forceinline__ uint64_t bcast(uint64_t v, int lane)
{
    return (uint64_t)bcast((uint32_t)v, lane) | ((uint64_t)bcast((uint32_t)(v >> 32), lane) << 32);
}

// ---- device-coherent row accesses -----------------------------------------------------------
// MI355X has one L2 per XCD, and a row written with an ordinary store stays in the writing XCD's L2:
// the other XCDs keep reading (and training) their own copies of every hot row for as long as those stay
// cached.  Hogwild needs the opposite (the latest value any worker wrote), so with COH = true P and Q
// rows are written with agent-scope relaxed atomic stores: plain global_store instructions with the sc1
// cache policy, which write through to the memory side and drop the copies other L2s hold.  Loads stay
// ordinary cached loads (measured: agent-scope loads add a third to the epoch and change nothing in the
// convergence once the stores are coherent).
//
// The price: every store goes to the memory side, and all stores to one row serialise there.  With a row
// that takes a large share of all ratings that single row bounds the epoch; see Schedule::keep_u for what
// is done about it.  COH = false keeps ordinary write-back stores: each XCD then works on its own
// L2-resident copy of a hot row between evictions (a row that is not re-used while cached behaves the
// same either way).  The caller picks per launch (mf_hogwild_options::cached_rows).  Adding the non-temporal
// hint to the coherent stores was measured and costs a fifth of the fp32 epoch.
//
// Rows are addressed through pointers in the global address space: a pointer rebuilt from an integer (the
// per-group pointer tables) would otherwise be a generic one, and generic accesses are flat instructions
// that also count as LDS traffic, so every wait for an LDS or scalar load would wait for all row loads in flight.
#define MF_GLOBAL __attribute__((address_space(1)))
template <class T> __device__ __forceinline__ MF_GLOBAL T* global_ptr(T* p) { return (MF_GLOBAL T*)p; }
template <class T> __device__ __forceinline__ MF_GLOBAL T* global_ptr(uint64_t addr) { return (MF_GLOBAL T*)addr; }
template <class T> __device__ __forceinline__ T row_load(const T* p) { return *global_ptr(p); }
template <bool COH, class T> __device__ __forceinline__ void row_store(T* p, T v)
{
    if constexpr (COH) __hip_atomic_store(global_ptr(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *global_ptr(p) = v;
}
// Aggregated update of a hot row (Schedule::keep_u): the change is added in memory, so concurrent updates
// of the row add up instead of overwriting each other.
__device__ __forceinline__ void row_add(float* p, float d)
{
    (void)__hip_atomic_fetch_add(global_ptr(p), d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void row_add(half2_t* p, half2_t d)
{
    (void)__builtin_amdgcn_global_atomic_fadd_v2f16(global_ptr(p), d);
}

// A row seen through a buffer resource of `bytes` bytes: accesses past the end are dropped by the hardware,
// so a window of 0 bytes turns a store into a no-op without a branch.  The fp32 rules' kernels with hot-row
// code store rows this way: the store of a rating that is thinned, or whose change is added instead, is still
// issued (and dropped), every rating then issues the same number of memory instructions on the straight path
// and the compiler's counted waits (s_waitcnt vmcnt(N)) keep the look-ahead of the row loads.
typedef __amdgpu_buffer_rsrc_t row_window_t;
__device__ __forceinline__ row_window_t row_window(uint64_t row, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc((void*)row, 0, (int)bytes, 0x00020000 /* 32-bit data format, raw addressing */);
}
// COH: the sc1 cache policy of row_store's agent-scope stores
template <bool COH> __device__ __forceinline__ void window_store(row_window_t w, uint32_t byte_offset, uint32_t v)
{
    __builtin_amdgcn_raw_buffer_store_b32(v, w, (int)byte_offset, 0, COH ? 16 : 0);
}
template <bool COH> __device__ __forceinline__ void window_store(row_window_t w, uint32_t byte_offset, uint16_t v)
{
    __builtin_amdgcn_raw_buffer_store_b16(v, w, (int)byte_offset, 0, COH ? 16 : 0);
}
template <bool COH> __device__ __forceinline__ void window_store(row_window_t w, uint32_t byte_offset, uint64_t v)
{
    typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2_t, v), w, (int)byte_offset, 0, COH ? 16 : 0);
}

// Adds through a row window (row_add's instructions in their buffer form: dropped when the window is closed).
__device__ __forceinline__ void window_add(row_window_t w, uint32_t byte_offset, float d)
{
    (void)__builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(d, w, (int)byte_offset, 0, 0);
}
__device__ __forceinline__ void window_add(row_window_t w, uint32_t byte_offset, half2_t d)
{
    (void)__builtin_amdgcn_raw_ptr_buffer_atomic_fadd_v2f16(d, w, (int)byte_offset, 0, 0);
}

// ---- counter-based generator -----------------------------------------------------------
__host__ __device__ __forceinline__ uint64_t mix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// start of window `ite` of worker `wid`: the mapping of sgd/sgd_kernel.h:22-26 applied to 32
// counter-derived bits (u01 = x*2^-32 + 2^-33 in (0,1], origin = (unsigned)(u01*nnz), start = origin % nnz).
__host__ __device__ __forceinline__ uint32_t window_start_rng(uint64_t epoch_key, uint32_t wid, uint32_t ite, uint32_t nnz)
{
    uint64_t h = mix64(epoch_key ^ (((uint64_t)wid << 32) | (uint64_t)ite));
    uint32_t x = (uint32_t)(h >> 32);
    float t = (float)x * 2.3283064365386963e-10f;
    float u01 = t + 1.1641532182693481e-10f;
    float scaled = u01 * (float)nnz;
    uint32_t origin = (scaled >= 4294967296.0f) ? 0xffffffffu : (uint32_t)scaled;
    return origin % nnz;
}
__host__ __device__ __forceinline__ uint64_t window_epoch_key(uint64_t seed, uint32_t epoch)
{
    return mix64(mix64(seed ^ 0x57494E444F575321ull) + (uint64_t)epoch);
}

// ---- the Hogwild schedule shared by every update kernel ---------------------------------
struct Schedule {
    const mf_node* R;
    uint32_t nnz;
    uint32_t num_workers;
    uint32_t update_count;
    uint32_t update_vector_size;
    uint32_t range_begin, range_end;   // processed-index range [begin, end) every worker handles in this launch
    uint32_t pieces;                   // >= 1: the range of a worker is cut into this many parts, each played by a
                                       // wavefront of its own (only launches with fewer wavefronts than workers)
    uint64_t epoch_key;
    const uint32_t* window_start;   // optional [update_count][num_workers]
    // Hot rows (optional, both null = off).  keep_u[row] / keep_v[row] in 0..255; 255 = an ordinary row.
    // A row with a smaller value is a hot row: its update is carried out with probability (keep+1)/255,
    // otherwise the row is only read for the other side's update; and an update that is carried out adds
    // its change to the row in memory (row_add) instead of storing the new row.  Under last-writer-wins a
    // row with C updates in flight keeps one of them; adding keeps them all, and thinning bounds C (the
    // sum of C stale gradients is a mini-batch step C times as long) and the stores that serialise at
    // the memory side.
    const uint8_t* keep_u;
    const uint8_t* keep_v;
    // Replicated rows (optional, with the hot-row tables).  A row whose keep value is kKeepReplicated has one copy per
    // XCD: the wavefronts of XCD x read and write copy x (slot slot_u[row] of replica block x) with ordinary cached
    // accesses -- the copy lives in that XCD's L2, where the 32 CUs of the XCD race on it as the reference's
    // workers race on a row, every update carried out -- and the copies are averaged between kernel launches
    // (replica_sync_kernel).  With kKeepReplicatedAdded (rows with few updates in flight per XCD) the update is added
    // to the copy instead, so that the XCD's concurrent updates add up; the hottest rows (kKeepReplicated) use neither
    // atomics nor write-through stores, so nothing of them serialises at the memory side.
    const uint16_t* slot_u;
    const uint16_t* slot_v;
    uint32_t slots_u, slots_v;      // replica rows per XCD and side
};
constexpr uint32_t kKeepReplicated = 253u;   // keep-table value of a replicated row whose updates are stored
constexpr uint32_t kKeepReplicatedAdded = 252u;   // ... whose updates are added to this XCD's copy
constexpr uint32_t kKeepThinnedMax = 251u;   // largest keep value of a thinned row
constexpr uint32_t kReplicaRow = 0x80000000u; // Rating::ru / rv: the row is replica row (value & ~kReplicaRow) of the replica array
constexpr uint32_t kXcds = 8u;                // replica blocks: one per XCD of an MI355X

// Where the rows of one side of the model live, for the kernel that copies them to and from their per-XCD replicas:
// a dense matrix [rows][k] of elem_bytes-wide elements, or the grouped storage of the MASCOT kernel.
struct RowStorage {
    void* dense = nullptr; uint32_t elem_bytes = 4;
    void* const* group_ptr = nullptr; const uint32_t* group_end = nullptr; const uint8_t* group_prec = nullptr; uint32_t groups = 0;
};

// Index of the XCD this wavefront runs on (hardware register XCC_ID, bits 3:0).
__device__ __forceinline__ uint32_t xcd_id()
{
    return (uint32_t)__builtin_amdgcn_s_getreg(20 /* HW_REG_XCC_ID */ | (0 << 6) | (3 << 11)) & (kXcds - 1u);
}

// One lane's rating of a 64-rating chunk; the stream is read once per epoch, so bypass-style loads.
// thin: bit0/bit1 skip the P/Q update, bit2/bit3 the P/Q row is a hot row (updates are added), bit4/bit5 the P/Q row is
// a replicated row (the update goes to this XCD's copy: an ordinary cached store, or an add when bit2/bit3 is set as
// well).  ru, rv: the row to address -- u, v themselves, or kReplicaRow | index of the replica row.
struct Rating { float r; uint32_t u; uint32_t v; uint32_t thin; uint32_t ru; uint32_t rv; };
__device__ __forceinline__ Rating load_rating(const mf_node* R, uint32_t idx)
{
    const uint32_t* w = reinterpret_cast<const uint32_t*>(R + idx);
    Rating x;
    x.r = from_bits<float>(__builtin_nontemporal_load(w));
    x.u = __builtin_nontemporal_load(w + 1);
    x.v = __builtin_nontemporal_load(w + 2);
    x.thin = 0u;
    x.ru = x.u; x.rv = x.v;
    return x;
}

}  // namespace mf
