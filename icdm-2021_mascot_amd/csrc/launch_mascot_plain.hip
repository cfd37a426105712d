// MASCOT kernels without the sampled-statistics code (launches in which no rating is sampled).
#include "launch_mascot.h"
#include "rule_mascot.h"

namespace mf {

int launch_mascot_plain(const MascotCall& c, Range r)
{
    return launch_k_coh<MascotPlainRule>(c.who, c.k, c.c, [&](auto a) { return c.fill(a); }, c.lds, c.stream, r);
}
size_t mascot_table_lds_bytes(uint32_t user_groups, uint32_t item_groups) { return MascotRule<128, true>::lds_bytes(user_groups, item_groups); }

}  // namespace mf
