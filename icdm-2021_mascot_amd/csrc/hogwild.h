// The Hogwild driver loop shared by every update kernel (sgd/sgd_kernel.h:14-37 of the
// reference, redesigned for wave64):
//   * one wavefront = one worker; it walks update_count windows of update_vector_size ratings;
//   * a window is consumed in chunks of 64 ratings: one coalesced streaming load puts rating j of
//     the chunk in lane j, anything that can be computed per rating without the rows (group search,
//     row addresses) is done once, vectorised across the 64 lanes, and the per-rating loop then
//     broadcasts lane j's scalars with v_readlane;
//   * the rows of rating j+1 are requested before rating j is reduced and stored, so one rating's
//     memory latency hides behind the previous rating's arithmetic.  When consecutive ratings touch
//     the same row the freshly computed row is forwarded in registers, so a worker's own updates
//     are applied strictly in order (needed for bit-exact checks; other workers still race, that is
//     Hogwild).
#pragma once
#include "mf_device.h"

namespace mf {

template <class Rule>
__global__ __launch_bounds__(kBlock) void hogwild_kernel(Schedule s, typename Rule::Params prm)
{
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wid = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)));
    Rule rule;
    rule.init(prm, smem, lane, wid);                    // may synchronise the workgroup
    if (wid < s.num_workers) {
        uint32_t processed = 0;
        for (uint32_t ite = 0; ite < s.update_count; ++ite) {
            uint32_t start;
            if (s.window_start) start = s.window_start[(size_t)ite * s.num_workers + wid] % s.nnz;
            else start = window_start_rng(s.epoch_key, wid, ite, s.nnz);
            start = (uint32_t)__builtin_amdgcn_readfirstlane((int)start);
            for (uint32_t c = 0; c < s.update_vector_size; c += kWave) {
                const uint32_t left = s.update_vector_size - c;
                const int n = left < (uint32_t)kWave ? (int)left : kWave;
                const bool valid = lane < n;
                Rating my = {0.f, 0u, 0u};
                if (valid) {
                    uint32_t off = (c + (uint32_t)lane) % s.nnz;
                    uint32_t idx = start + off;
                    if (idx >= s.nnz || idx < start) idx -= s.nnz;
                    my = load_rating(s.R, idx);
                }
                typename Rule::Prep prep = rule.prepare(my, valid);
                typename Rule::Info ic = rule.info(my, prep, 0);
                typename Rule::Row cur, nxt;
                rule.load(cur, ic);
                for (int j = 0; j < n; ++j) {
                    const bool has_next = (j + 1) < n;
                    typename Rule::Info in = ic;
                    if (has_next) {
                        in = rule.info(my, prep, j + 1);
                        rule.load(nxt, in);
                    }
                    rule.update(cur, ic, processed);
                    if (has_next) rule.forward(nxt, in, cur, ic);
                    cur = nxt;
                    ic = in;
                    ++processed;
                }
            }
        }
    }
    rule.finish(prm, wid);                               // may synchronise the workgroup
}

}  // namespace mf
