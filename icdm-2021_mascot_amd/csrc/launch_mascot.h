// The MASCOT launcher in four translation units: the entry point (launch_mascot.hip) and the kernels with and without
// the sampled-statistics code (launch_mascot_sampled.hip, launch_mascot_plain.hip) and for runs whose groups are all
// binary16 (launch_mascot_binary16.hip), which compile side by side.
#pragma once
#include "hogwild_launch.h"

namespace mf {

// What one mf_mascot_sgd_hogwild call carries to its launches.
struct MascotCall {
    const char* who; int k; Call c; size_t lds; void* stream;
    void* const* p; void* const* q;
    const uint32_t* user_end; const uint32_t* item_end;
    const uint8_t* user_prec; const uint8_t* item_prec;
    float* grad_sum_p; float* grad_sum_q; float* norm_sum_p; float* norm_sum_q;
    uint32_t first_sample, user_groups, item_groups;
    float lrate, lambda;
    uint32_t norm_stride;
    template <class Params> Params fill(Params a) const
    {
        a.p = p; a.q = q; a.user_end = user_end; a.item_end = item_end; a.user_prec = user_prec; a.item_prec = item_prec;
        a.grad_sum_p = grad_sum_p; a.grad_sum_q = grad_sum_q; a.norm_sum_p = norm_sum_p; a.norm_sum_q = norm_sum_q;
        a.first_sample = first_sample; a.user_groups = user_groups; a.item_groups = item_groups;
        a.lrate = lrate; a.lambda = lambda; a.norm_stride = norm_stride; a.lds_stats = false;
        return a;
    }
};
int launch_mascot_plain(const MascotCall& c, Range r);        // hogwild_kernel<MascotPlainRule<k, coh>, hot>
int launch_mascot_binary16(const MascotCall& c, Range r);     // hogwild_kernel<MascotBinary16Rule<k, coh>, hot>
int launch_mascot_sampled(const MascotCall& c, Range r);      // hogwild_kernel<MascotRule<k, coh>, hot>
size_t mascot_table_lds_bytes(uint32_t user_groups, uint32_t item_groups);

}  // namespace mf
