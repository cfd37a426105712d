// extern "C" launcher of the MASCOT rule; its kernels are built in launch_mascot_plain.hip and launch_mascot_sampled.hip.
#include "launch_mascot.h"

using namespace mf;

extern "C" {

int mf_mascot_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, void* const* p, void* const* q, int k,
                              uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                              float lrate, float lambda,
                              const uint32_t* user_group_end_idx, const uint32_t* item_group_end_idx,
                              const uint8_t* user_group_prec_info, const uint8_t* item_group_prec_info,
                              float* grad_sum_norm_p, float* grad_sum_norm_q, float* norm_sum_p, float* norm_sum_q,
                              uint32_t first_sample_rating_idx, uint32_t user_group_num, uint32_t item_group_num,
                              uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream, const mf_hogwild_options* options)
{
    const char* who = "mf_mascot_sgd_hogwild";
    if (int rc = check_schedule(who, R, nnz, k, num_workers, update_count, update_vector_size, options)) return rc;
    if (!p || !q || !user_group_end_idx || !item_group_end_idx || !user_group_prec_info || !item_group_prec_info)
        return invalid("%s: null group table", who);
    if (!grad_sum_norm_p || !grad_sum_norm_q || !norm_sum_p || !norm_sum_q) return invalid("%s: null statistics buffer", who);
    if (user_group_num == 0 || item_group_num == 0) return invalid("%s: at least one group per side is required", who);
    if (user_group_num > 16383 || item_group_num > 16383) return invalid("%s: at most 16383 groups per side", who);
    const size_t lds = mascot_table_lds_bytes(user_group_num, item_group_num);
    if (lds > 64 * 1024) return invalid("%s: group tables need %zu bytes of LDS (limit 65536)", who, lds);
    MascotCall c;
    c.who = who; c.k = k; c.lds = lds; c.stream = stream;
    c.c = make_call(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start, options);
    c.p = p; c.q = q; c.user_end = user_group_end_idx; c.item_end = item_group_end_idx;
    c.user_prec = user_group_prec_info; c.item_prec = item_group_prec_info;
    c.grad_sum_p = grad_sum_norm_p; c.grad_sum_q = grad_sum_norm_q; c.norm_sum_p = norm_sum_p; c.norm_sum_q = norm_sum_q;
    c.first_sample = first_sample_rating_idx; c.user_groups = user_group_num; c.item_groups = item_group_num;
    c.lrate = lrate; c.lambda = lambda; c.norm_stride = grid_for(num_workers);
    const uint32_t total = c.c.s.range_end;
    Range body = whole_epoch(c.c);
    // the unsampled part of an epoch: the kernel without the statistics code, in the build for all-binary16 runs if the
    // caller says that is what this is
    const bool binary16 = options && options->all_binary16;
    auto plain = [&](const Range& r) { return binary16 ? launch_mascot_binary16(c, r) : launch_mascot_plain(c, r); };
    if (first_sample_rating_idx >= total)                     // nothing is sampled
        return plain(body);
    // A check epoch.  The sampled ratings [first_sample, total) run as their own launch with the gradient sums in
    // LDS when those fit (160 KB per workgroup); otherwise the whole epoch runs with the sums in global memory.
    const size_t need = lds + (size_t)(user_group_num + item_group_num) * ((size_t)k + 1) * sizeof(float);      // sums and one lock per group
    if (need > 160 * 1024) return launch_mascot_sampled(c, body);
    body.end = first_sample_rating_idx;
    // the body still writes the (zero) norm sums of its workgroups, which the sampled launch then adds to
    if (int rc = plain(body)) return rc;
    Range tail;
    tail.begin = first_sample_rating_idx; tail.end = total; tail.accumulate = body.begin < body.end; tail.stats_lds = need;
    return launch_mascot_sampled(c, tail);
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
    return mf_mascot_sgd_hogwild_opt(R, nnz, p, q, k, num_workers, update_count, update_vector_size, lrate, lambda, user_group_end_idx, item_group_end_idx,
                                     user_group_prec_info, item_group_prec_info, grad_sum_norm_p, grad_sum_norm_q, norm_sum_p, norm_sum_q,
                                     first_sample_rating_idx, user_group_num, item_group_num, seed, epoch, window_start, stream, nullptr);
}

}  // extern "C"
