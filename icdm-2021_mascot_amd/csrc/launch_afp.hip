// extern "C" launcher of the AFP rule.
#include "hogwild_launch.h"
#include "rules_fixed_point.h"

namespace mf { float inflight_afp(int k, uint32_t num_workers, uint32_t cap) { return inflight_updates<AfpRule>(k, num_workers, 0, cap); } }
using namespace mf;

extern "C" {

int mf_afp_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                           uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                           float lrate, float lambda, int afp_epoch,
                           uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream, const mf_hogwild_options* options)
{
    if (int rc = check_schedule("mf_afp_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size, options)) return rc;
    if (!p || !q) return invalid("mf_afp_sgd_hogwild: null model pointer");
    const Call s = make_call(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start, options);
    // afp_sgd_kernel.h:145: int initialization_threshold = (float)(update_count*update_vector_size)/10.0f
    const int init_threshold = (int)((float)(update_count * update_vector_size) / 10.0f);
    return launch_k_coh<AfpRule>("mf_afp_sgd_hogwild", k, s, [&](auto a) {
        a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; a.afp_epoch = afp_epoch; a.init_threshold = init_threshold; return a; }, 0, stream, whole_epoch(s));
}
int mf_afp_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, float lambda, int afp_epoch,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    return mf_afp_sgd_hogwild_opt(R, nnz, p, q, k, num_workers, update_count, update_vector_size, lrate, lambda, afp_epoch, seed, epoch, window_start, stream, nullptr);
}

}  // extern "C"
