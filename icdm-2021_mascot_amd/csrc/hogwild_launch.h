// Shared by the launcher translation units (one per rule family, so that they compile in parallel): argument checks,
// the schedule and options of a call, and the launch of hogwild_kernel<Rule, HOT> for the four (k, coherence) combinations.
#pragma once
#include "mf_host.h"
#include "hogwild.h"
#include <cmath>
#include <cstring>
#include <vector>

namespace mf {

// One side's replicated rows: slot s of replica block x (x = 0..kXcds-1) is at replicas + (x * slots + s) * k * 4 bytes
// and holds a copy of row slot_row[s] in the precision the row is stored in (a binary16 row fills the first half).
struct ReplicaSide { RowStorage rows; uint8_t* replicas = nullptr; const uint32_t* slot_row = nullptr; uint32_t slots = 0; };
// merge = false: every replica := the row.  merge = true: the row and every replica := the mean of the replicas --
// of those that differ from the row (in_play = 0), or of the in_play copies the launch's workgroups could reach,
// untouched ones counting as the row itself (in_play > 0: the merge that goes with scaled steps, Call::step_scale).
int replica_sync(const ReplicaSide& user, const ReplicaSide& item, int k, bool merge, void* stream, uint32_t in_play = 0);

// A call's schedule (what the kernel gets) and the host-side part of its options.
struct Call {
    Schedule s;
    bool coherent = true;           // agent-scope row stores (mf_hogwild_options::cached_rows == 0)
    uint32_t launches = 1;          // kernel launches the call is cut into
    uint8_t* rep_u = nullptr;       // replica arrays (mf_hogwild_options::user_replicas / item_replicas)
    uint8_t* rep_v = nullptr;
    const uint32_t* slot_row_u = nullptr;
    const uint32_t* slot_row_v = nullptr;
    float step_scale = 0.f;         // mf_hogwild_options::replica_step_scale
    uint32_t resident_workers = 0;  // mf_hogwild_options::resident_workers
    bool replicated() const { return s.slots_u != 0 || s.slots_v != 0; }
};

static int check_schedule(const char* who, const void* R, uint32_t nnz, int k, uint32_t num_workers,
                          uint32_t update_count, uint32_t update_vector_size, const mf_hogwild_options* o)
{
    if (k != 64 && k != 128) return invalid("%s: k must be 64 or 128 (got %d)", who, k);
    if (!R || nnz == 0) return invalid("%s: empty rating array", who);
    if (num_workers == 0) return invalid("%s: num_workers must be positive", who);
    if ((uint64_t)update_count * update_vector_size > 0xffffffffull) return invalid("%s: update_count*update_vector_size overflows 32 bits", who);
    if ((uint64_t)nnz + update_vector_size > 0xffffffffull) return invalid("%s: nnz + update_vector_size overflows 32 bits", who);
    if (o) {
        if (o->cached_rows > 1) return invalid("%s: options.cached_rows is 0 (device-coherent row stores) or 1 (cached)", who);
        if (o->launches > 65536) return invalid("%s: options.launches is at most 65536", who);
        if ((o->user_keep == nullptr) != (o->item_keep == nullptr)) return invalid("%s: options: pass both hot-row tables or neither", who);
        const bool rep = o->user_slots || o->item_slots;
        if (rep && !o->user_keep) return invalid("%s: options: replicated rows are marked in the hot-row tables, which are missing", who);
        if (o->user_slots && (!o->user_slot || !o->user_slot_row || !o->user_replicas)) return invalid("%s: options: user_slots > 0 needs user_slot, user_slot_row and user_replicas", who);
        if (o->item_slots && (!o->item_slot || !o->item_slot_row || !o->item_replicas)) return invalid("%s: options: item_slots > 0 needs item_slot, item_slot_row and item_replicas", who);
        if (o->user_slots > 65535u || o->item_slots > 65535u) return invalid("%s: options: at most 65535 replicated rows per side", who);
        if (!(o->replica_step_scale >= 0.f) || o->replica_step_scale > 64.f) return invalid("%s: options.replica_step_scale is 0 (off) or between 1 and 64", who);
        if (rep && ((reinterpret_cast<uintptr_t>(o->user_replicas) | reinterpret_cast<uintptr_t>(o->item_replicas)) & 255u))
            return invalid("%s: options: replica arrays must be 256-byte aligned", who);
    }
    return MF_OK;
}
static Call make_call(const mf_node* R, uint32_t nnz, uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                      uint64_t seed, uint32_t epoch, const uint32_t* window_start, const mf_hogwild_options* o)
{
    Call c;
    Schedule& s = c.s;
    s.R = R; s.nnz = nnz; s.num_workers = num_workers; s.update_count = update_count;
    s.update_vector_size = update_vector_size; s.pieces = 1; s.range_begin = 0; s.range_end = update_count * update_vector_size;
    s.epoch_key = window_epoch_key(seed, epoch); s.window_start = window_start;
    s.keep_u = nullptr; s.keep_v = nullptr; s.slot_u = nullptr; s.slot_v = nullptr; s.slots_u = 0; s.slots_v = 0;
    if (o) {
        c.coherent = o->cached_rows == 0;
        c.launches = o->launches ? o->launches : 1;
        s.keep_u = o->user_keep; s.keep_v = o->item_keep;
        // a side without replicated rows keeps slots = 0; its keep table then must not hold the replicated mark
        s.slot_u = o->user_slot; s.slot_v = o->item_slot; s.slots_u = o->user_slots; s.slots_v = o->item_slots;
        c.rep_u = static_cast<uint8_t*>(o->user_replicas); c.rep_v = static_cast<uint8_t*>(o->item_replicas);
        c.slot_row_u = o->user_slot_row; c.slot_row_v = o->item_slot_row;
        c.step_scale = o->replica_step_scale;
        c.resident_workers = o->resident_workers;
    }
    return c;
}
static inline uint32_t grid_for(uint32_t num_workers) { return (num_workers + kWavesPerBlock - 1) / kWavesPerBlock; }


// What part of an epoch one call to launch() covers, in each worker's processed-rating index space.
struct Range {
    uint32_t begin = 0, end = 0;
    bool accumulate = false;      // an earlier launch of the same epoch has already run
    size_t stats_lds = 0;         // > 0: one launch of <= 256 workgroups of 16 wavefronts with this much LDS, the
                                  // rule keeping its sampled gradient sums there (MASCOT check epochs)
};
template <class P> static auto set_lds_stats(P& p, bool v) -> decltype(p.lds_stats, void()) { p.lds_stats = v; }
static void set_lds_stats(...) {}

template <class Rule, bool HOT>
static int launch_hot(const char* who, const Call& c, const typename Rule::Params& prm0, size_t lds, void* stream, Range r);
// Workgroups of `kernel` (kBlock threads, `lds` bytes of LDS of their own) that share a compute unit, and the LDS size
// to launch with so that at most `resident_workers` workers are resident on the device: the compute unit's LDS divided
// by the workgroups wanted, which leaves no room for one more.  0 = leave the launch as it is (no cap asked for, the
// cap is not below what the launch or the device keeps resident anyway, or a query failed).
static size_t lds_for_resident_cap(const void* kernel, size_t lds, uint32_t resident_workers, uint32_t num_workers)
{
    if (resident_workers == 0 || num_workers <= resident_workers) return 0;
    int blocks = 0, dev = 0, cus = 0, lds_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, kBlock, lds) != hipSuccess || hipGetDevice(&dev) != hipSuccess
        || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess
        || hipDeviceGetAttribute(&lds_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess || blocks <= 0 || cus <= 0 || lds_cu <= 0) {
        (void)hipGetLastError();
        return 0;
    }
    uint32_t want = resident_workers / (uint32_t)(kWavesPerBlock * cus);
    if (want < 1) want = 1;
    // one workgroup per compute unit is the least a launch can be held to
    if (want >= (uint32_t)blocks || num_workers <= want * (uint32_t)(kWavesPerBlock * cus)) return 0;
    const size_t padded = ((size_t)lds_cu / want) & ~(size_t)1023;
    if (padded <= lds || (size_t)(want + 1) * padded <= (size_t)lds_cu) return 0;
    int got = 0;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)padded) != hipSuccess
        || hipOccupancyMaxActiveBlocksPerMultiprocessor(&got, kernel, kBlock, padded) != hipSuccess || got != (int)want) {
        (void)hipGetLastError();
        return 0;
    }
    return padded;
}
// the kernel comes in two builds: with and without the hot-row code (Schedule::keep_u)
template <class Rule>
static int launch(const char* who, const Call& c, const typename Rule::Params& prm0, size_t lds, void* stream, Range r)
{
    return c.s.keep_u ? launch_hot<Rule, true>(who, c, prm0, lds, stream, r) : launch_hot<Rule, false>(who, c, prm0, lds, stream, r);
}
template <class Rule, bool HOT>
static int launch_hot(const char* who, const Call& c, const typename Rule::Params& prm0, size_t lds, void* stream, Range r)
{
    const Schedule& s0 = c.s;
    if (s0.update_count == 0 || s0.update_vector_size == 0 || r.begin >= r.end) return MF_OK;
    Schedule s = s0;
    typename Rule::Params prm = prm0;
    prm.rep_p = c.rep_u; prm.rep_q = c.rep_v; prm.rep_scale = 1.0f;
    // Replicated rows: every XCD's copy starts as the row, and after every kernel the row and the copies become the
    // mean of the copies (a kernel boundary is where the L2s of the XCDs are written back).
    ReplicaSide ru, rv;
    const bool replicated = HOT && c.replicated();
    // Scaled steps on replicated rows (Call::step_scale > 0): a copy sees the ratings of one XCD only, and the mean of X
    // copies moves by the X-th part of what the copies moved together, so an update of a copy takes a step that many times
    // as long (at most step_scale, the caller's bound for a stable step) and the merge is the mean over all X copies in play.
    uint32_t in_play = 0;
    auto scaled_steps = [&](uint32_t workgroups) {
        if (!replicated || !(c.step_scale > 0.f)) return;
        in_play = workgroups < kXcds ? workgroups : kXcds;
        prm.rep_scale = (in_play == kXcds || c.step_scale < (float)in_play) ? (c.step_scale < 1.f ? 1.f : c.step_scale) : (float)in_play;
    };
    if (replicated) {
        Rule::row_storage(prm, ru.rows, rv.rows);
        ru.replicas = c.rep_u; ru.slot_row = c.slot_row_u; ru.slots = s0.slots_u;
        rv.replicas = c.rep_v; rv.slot_row = c.slot_row_v; rv.slots = s0.slots_v;
        if (int rc = replica_sync(ru, rv, Rule::kK, false, stream)) return rc;
    }
    if (r.stats_lds) {
        s.range_begin = r.begin; s.range_end = r.end;
        prm.accumulate = r.accumulate;
        uint32_t blocks = (s.num_workers + 15) / 16;
        if (blocks > 256) {
            // more workers than the 4096 wavefronts of this launch: cut each worker's range into the number of
            // pieces that leaves the fewest idle wavefronts in the last pass
            blocks = 256;
            double best = 1e30;
            for (uint32_t p = 1; p <= 4; ++p) {
                const double passes = (double)(((uint64_t)s.num_workers * p + 4095) / 4096) / p;
                if (passes < best - 1e-9) { best = passes; s.pieces = p; }
            }
        }
        if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&hogwild_kernel<Rule, HOT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)r.stats_lds),
                               "hipFuncSetAttribute(MaxDynamicSharedMemorySize)")) return rc;
        set_lds_stats(prm, true);
        scaled_steps(blocks);
        hipLaunchKernelGGL((hogwild_kernel<Rule, HOT>), dim3(blocks), dim3(kMaxBlock), r.stats_lds, as_stream(stream), s, prm);
        if (int rc = launch_status(who)) return rc;
        return replicated ? replica_sync(ru, rv, Rule::kK, true, stream, in_play) : MF_OK;
    }
    // ordinary launches, cut into c.launches pieces on window boundaries
    uint32_t splits = Rule::kSplittable ? c.launches : 1;
    const uint32_t first_window = (r.begin + s0.update_vector_size - 1) / s0.update_vector_size, end_window = r.end / s0.update_vector_size;
    const uint32_t windows = end_window > first_window ? end_window - first_window : 0;
    if (splits > windows) splits = windows ? windows : 1;
    bool first = true;
    scaled_steps(grid_for(s.num_workers));
    if (const size_t padded = lds_for_resident_cap(reinterpret_cast<const void*>(&hogwild_kernel<Rule, HOT>), lds, c.resident_workers, s.num_workers)) lds = padded;
    for (uint32_t i = 0; i < splits; ++i) {
        const uint32_t b = i == 0 ? r.begin : (first_window + (uint32_t)((uint64_t)windows * i / splits)) * s0.update_vector_size;
        const uint32_t e = i + 1 == splits ? r.end : (first_window + (uint32_t)((uint64_t)windows * (i + 1) / splits)) * s0.update_vector_size;
        if (b >= e) continue;
        s.range_begin = b; s.range_end = e;
        prm.accumulate = r.accumulate || !first;
        first = false;
        hipLaunchKernelGGL((hogwild_kernel<Rule, HOT>), dim3(grid_for(s.num_workers)), dim3(kBlock), lds, as_stream(stream), s, prm);
        if (int rc = launch_status(who)) return rc;
        if (replicated) { if (int rc = replica_sync(ru, rv, Rule::kK, true, stream, in_play)) return rc; }
    }
    return MF_OK;
}

// Instantiates Rule<K, COH> for the four (k, coherence) combinations; P is the parameter pack type,
// identical across instantiations apart from the template arguments.
template <template <int, bool> class Rule, class MakeParams>
static int launch_k_coh(const char* who, int k, const Call& c, MakeParams make, size_t lds, void* stream, Range r)
{
    if (k == 128) {
        if (c.coherent) { auto a = make(typename Rule<128, true>::Params{}); return launch<Rule<128, true>>(who, c, a, lds, stream, r); }
        auto a = make(typename Rule<128, false>::Params{}); return launch<Rule<128, false>>(who, c, a, lds, stream, r);
    }
    if (c.coherent) { auto a = make(typename Rule<64, true>::Params{}); return launch<Rule<64, true>>(who, c, a, lds, stream, r); }
    auto a = make(typename Rule<64, false>::Params{}); return launch<Rule<64, false>>(who, c, a, lds, stream, r);
}
// Updates in flight during a launch of num_workers workers of Rule at this k (the build with the hot-row code and
// coherent stores, which is what a run with hot-row tables launches): resident wavefronts x ratings per wavefront.
template <template <int, bool> class Rule>
static float inflight_updates(int k, uint32_t num_workers, size_t lds, uint32_t resident_cap)
{
    int blocks = 0, dev = 0, cus = 0;
    const void* kernel = k == 128 ? reinterpret_cast<const void*>(&hogwild_kernel<Rule<128, true>, true>) : reinterpret_cast<const void*>(&hogwild_kernel<Rule<64, true>, true>);
    // a launch held to resident_cap workers runs with the LDS size that does the holding
    if (const size_t padded = lds_for_resident_cap(kernel, lds, resident_cap, num_workers)) lds = padded;
    hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, kBlock, lds);
    if (e != hipSuccess || hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || blocks <= 0 || cus <= 0) {
        (void)hipGetLastError();
        return 0.f;
    }
    const double resident = (double)blocks * kWavesPerBlock * cus;
    const double ahead = k == 128 ? Rule<128, true>::kAhead + 1 : Rule<64, true>::kAhead + 1;
    return (float)(((double)num_workers < resident ? (double)num_workers : resident) * ahead);
}
// cap: mf_hogwild_options::resident_workers of the launch (0 = none)
float inflight_sgd(int k, uint32_t num_workers, uint32_t cap);          // hogwild_launch.hip
float inflight_mpt(int k, uint32_t num_workers, uint32_t cap);
float inflight_mem_quant(int k, uint32_t num_workers, uint32_t cap);    // launch_mem_quant.hip
float inflight_muppet(int k, uint32_t num_workers, uint32_t cap);       // launch_muppet.hip
float inflight_afp(int k, uint32_t num_workers, uint32_t cap);          // launch_afp.hip
float inflight_mascot(int k, uint32_t num_workers, uint32_t user_groups, uint32_t item_groups, uint32_t cap);   // launch_mascot_binary16.hip

static Range whole_epoch(const Call& c) { Range r; r.begin = 0; r.end = c.s.range_end; return r; }

}  // namespace mf
