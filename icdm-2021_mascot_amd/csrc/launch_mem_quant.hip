// extern "C" launcher of the binary16-storage rule (-v 7).
#include "hogwild_launch.h"
#include "rules_fp32.h"

using namespace mf;

extern "C" {

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

}  // extern "C"
