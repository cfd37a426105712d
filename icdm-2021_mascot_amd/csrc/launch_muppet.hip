// extern "C" launcher of the MuPPET rule.
#include "hogwild_launch.h"
#include "rules_fixed_point.h"

namespace mf { float inflight_muppet(int k, uint32_t num_workers, uint32_t cap) { return inflight_updates<MuppetRule>(k, num_workers, 0, cap); } }
using namespace mf;

extern "C" {

static bool muppet_precision_ok(uint8_t b) { return b == 8 || b == 12 || b == 14 || b == 16 || b == 32; }

int mf_muppet_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                              uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                              float lrate, float lambda, uint32_t first_sample_rating_idx,
                              float* sum_updated_val, float* sum_norms,
                              uint8_t forward_prop_precision, uint8_t backward_prop_precision,
                              uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream, const mf_hogwild_options* options)
{
    if (int rc = check_schedule("mf_muppet_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size, options)) return rc;
    if (!p || !q || !sum_updated_val || !sum_norms) return invalid("mf_muppet_sgd_hogwild: null pointer");
    if (!muppet_precision_ok(forward_prop_precision) || !muppet_precision_ok(backward_prop_precision))
        return invalid("mf_muppet_sgd_hogwild: precisions must be one of 8, 12, 14, 16, 32");
    if ((forward_prop_precision == 32) != (backward_prop_precision == 32))
        return invalid("mf_muppet_sgd_hogwild: forward and backward precision must both be 32 or both below (the backward scale reuses forward statistics)");
    const Call s = make_call(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start, options);
    return launch_k_coh<MuppetRule>("mf_muppet_sgd_hogwild", k, s, [&](auto a) {
        a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; a.first_sample = first_sample_rating_idx;
        a.sum_updated_val = sum_updated_val; a.sum_norms = sum_norms; a.num_workers = num_workers;
        a.fwd = forward_prop_precision; a.bwd = backward_prop_precision; return a; }, 0, stream, whole_epoch(s));
}
int mf_muppet_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda, uint32_t first_sample_rating_idx,
                          float* sum_updated_val, float* sum_norms,
                          uint8_t forward_prop_precision, uint8_t backward_prop_precision,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    return mf_muppet_sgd_hogwild_opt(R, nnz, p, q, k, num_workers, update_count, update_vector_size, lrate, lambda, first_sample_rating_idx,
                                     sum_updated_val, sum_norms, forward_prop_precision, backward_prop_precision, seed, epoch, window_start, stream, nullptr);
}

}  // extern "C"
