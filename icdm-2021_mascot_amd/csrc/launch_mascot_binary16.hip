// MASCOT kernels without the sampled-statistics code and without the straight-line path for chunks of mixed precisions:
// launches of a run whose groups are all still binary16 (mf_hogwild_options::all_binary16).
#include "launch_mascot.h"
#include "rule_mascot.h"

namespace mf {

int launch_mascot_binary16(const MascotCall& c, Range r)
{
    return launch_k_coh<MascotBinary16Rule>(c.who, c.k, c.c, [&](auto a) { return c.fill(a); }, c.lds, c.stream, r);
}

// A run starts with every group in binary16, and its hot-row tables are built once: the wavefronts this build keeps
// resident are the ones to count (the build with the mixed-precision path keeps one fewer per SIMD; tables made for
// more updates in flight than there are err on the careful side).
float inflight_mascot(int k, uint32_t num_workers, uint32_t user_groups, uint32_t item_groups, uint32_t cap)
{
    return inflight_updates<MascotBinary16Rule>(k, num_workers, MascotRule<128, true>::lds_bytes(user_groups, item_groups), cap);
}

}  // namespace mf
