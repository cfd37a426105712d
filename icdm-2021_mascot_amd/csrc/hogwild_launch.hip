// extern "C" launchers of the five Hogwild update kernels.
#include "mf_host.h"
#include "rules_fp32.h"
#include "rule_mascot.h"
#include "rules_fixed_point.h"
#include <cmath>
#include <cstring>
#include <vector>

namespace mf {

// hot-row tables (device pointers, see Schedule::keep_u); null = off
static const uint8_t* g_keep_u = nullptr;
static const uint8_t* g_keep_v = nullptr;
static thread_local char g_error[512] = "";
void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}

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

// 0: ordinary write-back row stores, 1: agent-scope coherent row stores (see row_store in mf_device.h)
static int g_row_coherence = 1;
// number of consecutive kernel launches one call is cut into (each worker's windows are split evenly);
// a kernel boundary writes back and invalidates the per-XCD L2s, which is how cached row copies of
// different XCDs are reconciled during an epoch
static uint32_t g_epoch_splits = 1;

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

using namespace mf;

extern "C" {

int mf_version(void) { return 1; }
int mf_set_row_coherence(int coherent)
{
    if (coherent != 0 && coherent != 1) return invalid("mf_set_row_coherence: 0 (cached) or 1 (device-coherent)");
    g_row_coherence = coherent;
    return MF_OK;
}
int mf_get_row_coherence(void) { return g_row_coherence; }
int mf_set_epoch_splits(uint32_t splits)
{
    if (splits == 0 || splits > 65536) return invalid("mf_set_epoch_splits: between 1 and 65536");
    g_epoch_splits = splits;
    return MF_OK;
}
uint32_t mf_get_epoch_splits(void) { return g_epoch_splits; }
int mf_set_hot_row_thinning(const uint8_t* user_keep, const uint8_t* item_keep)
{
    if ((user_keep == nullptr) != (item_keep == nullptr)) return invalid("mf_set_hot_row_thinning: pass both tables or neither");
    g_keep_u = user_keep; g_keep_v = item_keep;
    return MF_OK;
}
const char* mf_last_error(void) { return g_error; }
uint32_t mf_mascot_norm_blocks(uint32_t num_workers) { return grid_for(num_workers); }

uint32_t mf_update_count(uint32_t n, uint32_t num_workers, uint32_t update_vector_size)
{
    if (num_workers == 0 || update_vector_size == 0) return 0;
    return (uint32_t)std::ceil((double)n / (double)((uint64_t)num_workers * update_vector_size));
}
uint32_t mf_first_sample_rating_idx(uint32_t e, uint32_t interval, uint32_t epochs, uint32_t update_count,
                                    uint32_t update_vector_size, float sample_ratio)
{
    const uint32_t start_idx = 5;
    const uint32_t total = update_count * update_vector_size;
    if (interval == 0) return total;
    const bool check = (e >= start_idx) && (e % interval == (start_idx % interval)) && (epochs - 1 != e);
    if (!check) return total;
    const uint32_t sample_ratings_num = (uint32_t)((float)total * sample_ratio);
    return total - sample_ratings_num;
}
float mf_lr_schedule(float lr, float decay, uint32_t e)
{
    return (float)((double)lr / (1.0 + ((double)decay * std::pow((double)e, 1.5))));
}
uint32_t mf_window_start(uint64_t seed, uint32_t epoch, uint32_t worker, uint32_t ite, uint32_t nnz)
{
    if (nnz == 0) return 0;
    return window_start_rng(window_epoch_key(seed, epoch), worker, ite, nnz);
}

int mf_single_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    if (int rc = check_schedule("mf_single_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size)) return rc;
    if (!p || !q) return invalid("mf_single_sgd_hogwild: null model pointer");
    Schedule s = make_schedule(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start);
    return launch_k_coh<SgdRule>("mf_single_sgd_hogwild", k, s, [&](auto a) { a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; return a; }, 0, stream, whole_epoch(s));
}

int mf_mem_quant_sgd_hogwild(const mf_node* R, uint32_t nnz, uint16_t* p, uint16_t* q, int k,
                             uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                             float lrate, float lambda,
                             uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    if (int rc = check_schedule("mf_mem_quant_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size)) return rc;
    if (!p || !q) return invalid("mf_mem_quant_sgd_hogwild: null model pointer");
    Schedule s = make_schedule(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start);
    return launch_k_coh<MemQuantRule>("mf_mem_quant_sgd_hogwild", k, s, [&](auto a) { a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; return a; }, 0, stream, whole_epoch(s));
}

int mf_mpt_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, uint16_t scaled_lambda_half, float scaling_factor,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    if (int rc = check_schedule("mf_mpt_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size)) return rc;
    if (!p || !q) return invalid("mf_mpt_sgd_hogwild: null model pointer");
    if (!(scaling_factor > 0)) return invalid("mf_mpt_sgd_hogwild: scaling_factor must be positive");
    Schedule s = make_schedule(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start);
    return launch_k_coh<MptRule>("mf_mpt_sgd_hogwild", k, s, [&](auto a) {
        a.p = p; a.q = q; a.lrate = lrate; a.scaled_lambda_half = scaled_lambda_half; a.scaling_factor = scaling_factor; return a; }, 0, stream, whole_epoch(s));
}

static bool muppet_precision_ok(uint8_t b) { return b == 8 || b == 12 || b == 14 || b == 16 || b == 32; }

int mf_muppet_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda, uint32_t first_sample_rating_idx,
                          float* sum_updated_val, float* sum_norms,
                          uint8_t forward_prop_precision, uint8_t backward_prop_precision,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    if (int rc = check_schedule("mf_muppet_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size)) return rc;
    if (!p || !q || !sum_updated_val || !sum_norms) return invalid("mf_muppet_sgd_hogwild: null pointer");
    if (!muppet_precision_ok(forward_prop_precision) || !muppet_precision_ok(backward_prop_precision))
        return invalid("mf_muppet_sgd_hogwild: precisions must be one of 8, 12, 14, 16, 32");
    if ((forward_prop_precision == 32) != (backward_prop_precision == 32))
        return invalid("mf_muppet_sgd_hogwild: forward and backward precision must both be 32 or both below (the backward scale reuses forward statistics)");
    Schedule s = make_schedule(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start);
    return launch_k_coh<MuppetRule>("mf_muppet_sgd_hogwild", k, s, [&](auto a) {
        a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; a.first_sample = first_sample_rating_idx;
        a.sum_updated_val = sum_updated_val; a.sum_norms = sum_norms; a.num_workers = num_workers;
        a.fwd = forward_prop_precision; a.bwd = backward_prop_precision; return a; }, 0, stream, whole_epoch(s));
}

int mf_afp_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, float lambda, int afp_epoch,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    if (int rc = check_schedule("mf_afp_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size)) return rc;
    if (!p || !q) return invalid("mf_afp_sgd_hogwild: null model pointer");
    Schedule s = make_schedule(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start);
    // afp_sgd_kernel.h:145: int initialization_threshold = (float)(update_count*update_vector_size)/10.0f
    const int init_threshold = (int)((float)(update_count * update_vector_size) / 10.0f);
    return launch_k_coh<AfpRule>("mf_afp_sgd_hogwild", k, s, [&](auto a) {
        a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; a.afp_epoch = afp_epoch; a.init_threshold = init_threshold; return a; }, 0, stream, whole_epoch(s));
}

int mf_mascot_sgd_hogwild(const mf_node* R, uint32_t nnz, void* const* p, void* const* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          const uint32_t* user_group_end_idx, const uint32_t* item_group_end_idx,
                          const uint8_t* user_group_prec_info, const uint8_t* item_group_prec_info,
                          float* grad_sum_norm_p, float* grad_sum_norm_q, float* norm_sum_p, float* norm_sum_q,
                          uint32_t first_sample_rating_idx, uint32_t user_group_num, uint32_t item_group_num,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    const char* who = "mf_mascot_sgd_hogwild";
    if (int rc = check_schedule(who, R, nnz, k, num_workers, update_count, update_vector_size)) return rc;
    if (!p || !q || !user_group_end_idx || !item_group_end_idx || !user_group_prec_info || !item_group_prec_info)
        return invalid("%s: null group table", who);
    if (!grad_sum_norm_p || !grad_sum_norm_q || !norm_sum_p || !norm_sum_q) return invalid("%s: null statistics buffer", who);
    if (user_group_num == 0 || item_group_num == 0) return invalid("%s: at least one group per side is required", who);
    if (user_group_num > 16383 || item_group_num > 16383) return invalid("%s: at most 16383 groups per side", who);
    const size_t lds = MascotRule<128, true>::lds_bytes(user_group_num, item_group_num);
    if (lds > 64 * 1024) return invalid("%s: group tables need %zu bytes of LDS (limit 65536)", who, lds);
    Schedule s = make_schedule(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start);
    auto fill = [&](auto a) {
        a.p = p; a.q = q; a.user_end = user_group_end_idx; a.item_end = item_group_end_idx;
        a.user_prec = user_group_prec_info; a.item_prec = item_group_prec_info;
        a.grad_sum_p = grad_sum_norm_p; a.grad_sum_q = grad_sum_norm_q; a.norm_sum_p = norm_sum_p; a.norm_sum_q = norm_sum_q;
        a.first_sample = first_sample_rating_idx; a.user_groups = user_group_num; a.item_groups = item_group_num;
        a.lrate = lrate; a.lambda = lambda; a.norm_stride = grid_for(num_workers); a.lds_stats = false; return a; };
    const uint32_t total = s.range_end;
    Range body = whole_epoch(s);
    if (first_sample_rating_idx >= total)                     // nothing is sampled: the kernel without the statistics code
        return launch_k_coh<MascotPlainRule>(who, k, s, fill, lds, stream, body);
    // A check epoch.  The sampled ratings [first_sample, total) run as their own launch with the gradient sums in
    // LDS when those fit (160 KB per workgroup); otherwise the whole epoch runs with the sums in global memory.
    const size_t need = lds + (size_t)(user_group_num + item_group_num) * ((size_t)k + 1) * sizeof(float);      // sums and one lock per group
    if (need > 160 * 1024) return launch_k_coh<MascotRule>(who, k, s, fill, lds, stream, body);
    body.end = first_sample_rating_idx;
    // the body still writes the (zero) norm sums of its workgroups, which the sampled launch then adds to
    if (int rc = launch_k_coh<MascotPlainRule>(who, k, s, fill, lds, stream, body)) return rc;
    Range tail;
    tail.begin = first_sample_rating_idx; tail.end = total; tail.accumulate = body.begin < body.end; tail.stats_lds = need;
    return launch_k_coh<MascotRule>(who, k, s, fill, lds, stream, tail);
}

}  // extern "C"
