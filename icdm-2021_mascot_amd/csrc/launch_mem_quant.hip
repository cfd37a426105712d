// extern "C" launcher of the binary16-storage rule (-v 7).
#include "hogwild_launch.h"
#include "rules_fp32.h"

namespace mf { float inflight_mem_quant(int k, uint32_t num_workers, uint32_t cap) { return inflight_updates<MemQuantRule>(k, num_workers, 0, cap); } }
using namespace mf;

extern "C" {

int mf_mem_quant_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, uint16_t* p, uint16_t* q, int k,
                                 uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                                 float lrate, float lambda,
                                 uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream, const mf_hogwild_options* options)
{
    if (int rc = check_schedule("mf_mem_quant_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size, options)) return rc;
    if (!p || !q) return invalid("mf_mem_quant_sgd_hogwild: null model pointer");
    const Call s = make_call(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start, options);
    return launch_k_coh<MemQuantRule>("mf_mem_quant_sgd_hogwild", k, s, [&](auto a) { a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; return a; }, 0, stream, whole_epoch(s));
}
int mf_mem_quant_sgd_hogwild(const mf_node* R, uint32_t nnz, uint16_t* p, uint16_t* q, int k,
                             uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                             float lrate, float lambda,
                             uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    return mf_mem_quant_sgd_hogwild_opt(R, nnz, p, q, k, num_workers, update_count, update_vector_size, lrate, lambda, seed, epoch, window_start, stream, nullptr);
}

}  // extern "C"
