// extern "C" launchers of the Hogwild update kernels: process-wide settings, closed forms of the schedule, and the
// fp32 SGD and MPT entry points (the other rules' entry points sit in launch_*.hip).
#include "hogwild_launch.h"
#include "rules_fp32.h"

namespace mf {

// hot-row tables (device pointers, see Schedule::keep_u); null = off
const uint8_t* g_keep_u = nullptr;
const uint8_t* g_keep_v = nullptr;
// 0: ordinary write-back row stores, 1: agent-scope coherent row stores (see row_store in mf_device.h)
int g_row_coherence = 1;
// number of consecutive kernel launches one call is cut into (each worker's windows are split evenly);
// a kernel boundary writes back and invalidates the per-XCD L2s, which is how cached row copies of
// different XCDs are reconciled during an epoch
uint32_t g_epoch_splits = 1;
static thread_local char g_error[512] = "";
void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}

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

}  // extern "C"
