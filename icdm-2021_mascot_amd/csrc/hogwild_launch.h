// Shared by the launcher translation units (one per rule family, so that they compile in parallel): argument checks,
// the schedule of a call, and the launch of hogwild_kernel<Rule, HOT> for the four (k, coherence) combinations.
#pragma once
#include "mf_host.h"
#include "hogwild.h"
#include <cmath>
#include <cstring>
#include <vector>

namespace mf {

// process-wide settings, defined in hogwild_launch.hip (mf_set_hot_row_thinning, mf_set_row_coherence, mf_set_epoch_splits)
extern const uint8_t* g_keep_u;
extern const uint8_t* g_keep_v;
extern int g_row_coherence;
extern uint32_t g_epoch_splits;

static int check_schedule(const char* who, const void* R, uint32_t nnz, int k, uint32_t num_workers,
                          uint32_t update_count, uint32_t update_vector_size)
{
    if (k != 64 && k != 128) return invalid("%s: k must be 64 or 128 (got %d)", who, k);
    if (!R || nnz == 0) return invalid("%s: empty rating array", who);
    if (num_workers == 0) return invalid("%s: num_workers must be positive", who);
    if ((uint64_t)update_count * update_vector_size > 0xffffffffull) return invalid("%s: update_count*update_vector_size overflows 32 bits", who);
    if ((uint64_t)nnz + update_vector_size > 0xffffffffull) return invalid("%s: nnz + update_vector_size overflows 32 bits", who);
    (void)update_count;
    return MF_OK;
}
static Schedule make_schedule(const mf_node* R, uint32_t nnz, uint32_t num_workers, uint32_t update_count,
                              uint32_t update_vector_size, uint64_t seed, uint32_t epoch, const uint32_t* window_start)
{
    Schedule s;
    s.R = R; s.nnz = nnz; s.num_workers = num_workers; s.update_count = update_count;
    s.update_vector_size = update_vector_size; s.pieces = 1; s.range_begin = 0; s.range_end = update_count * update_vector_size; s.epoch_key = window_epoch_key(seed, epoch); s.window_start = window_start; s.keep_u = g_keep_u; s.keep_v = g_keep_v;
    return s;
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
static int launch_hot(const char* who, const Schedule& s0, const typename Rule::Params& prm0, size_t lds, void* stream, Range r);
// the kernel comes in two builds: with and without the hot-row code (Schedule::keep_u)
template <class Rule>
static int launch(const char* who, const Schedule& s0, const typename Rule::Params& prm0, size_t lds, void* stream, Range r)
{
    return s0.keep_u ? launch_hot<Rule, true>(who, s0, prm0, lds, stream, r) : launch_hot<Rule, false>(who, s0, prm0, lds, stream, r);
}
template <class Rule, bool HOT>
static int launch_hot(const char* who, const Schedule& s0, const typename Rule::Params& prm0, size_t lds, void* stream, Range r)
{
    if (s0.update_count == 0 || s0.update_vector_size == 0 || r.begin >= r.end) return MF_OK;
    Schedule s = s0;
    typename Rule::Params prm = prm0;
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
        hipLaunchKernelGGL((hogwild_kernel<Rule, HOT>), dim3(blocks), dim3(kMaxBlock), r.stats_lds, as_stream(stream), s, prm);
        return launch_status(who);
    }
    // ordinary launches, cut into g_epoch_splits pieces on window boundaries
    uint32_t splits = Rule::kSplittable ? g_epoch_splits : 1;
    const uint32_t first_window = (r.begin + s0.update_vector_size - 1) / s0.update_vector_size, end_window = r.end / s0.update_vector_size;
    const uint32_t windows = end_window > first_window ? end_window - first_window : 0;
    if (splits > windows) splits = windows ? windows : 1;
    bool first = true;
    for (uint32_t i = 0; i < splits; ++i) {
        const uint32_t b = i == 0 ? r.begin : (first_window + (uint32_t)((uint64_t)windows * i / splits)) * s0.update_vector_size;
        const uint32_t e = i + 1 == splits ? r.end : (first_window + (uint32_t)((uint64_t)windows * (i + 1) / splits)) * s0.update_vector_size;
        if (b >= e) continue;
        s.range_begin = b; s.range_end = e;
        prm.accumulate = r.accumulate || !first;
        first = false;
        hipLaunchKernelGGL((hogwild_kernel<Rule, HOT>), dim3(grid_for(s.num_workers)), dim3(kBlock), lds, as_stream(stream), s, prm);
        if (int rc = launch_status(who)) return rc;
    }
    return MF_OK;
}

// Instantiates Rule<K, COH> for the four (k, coherence) combinations; P is the parameter pack type,
// identical across instantiations apart from the template arguments.
template <template <int, bool> class Rule, class MakeParams>
static int launch_k_coh(const char* who, int k, const Schedule& s, MakeParams make, size_t lds, void* stream, Range r)
{
    const bool coh = g_row_coherence != 0;
    if (k == 128) {
        if (coh) { auto a = make(typename Rule<128, true>::Params{}); return launch<Rule<128, true>>(who, s, a, lds, stream, r); }
        auto a = make(typename Rule<128, false>::Params{}); return launch<Rule<128, false>>(who, s, a, lds, stream, r);
    }
    if (coh) { auto a = make(typename Rule<64, true>::Params{}); return launch<Rule<64, true>>(who, s, a, lds, stream, r); }
    auto a = make(typename Rule<64, false>::Params{}); return launch<Rule<64, false>>(who, s, a, lds, stream, r);
}
static Range whole_epoch(const Schedule& s) { Range r; r.begin = 0; r.end = s.range_end; return r; }

}  // namespace mf
