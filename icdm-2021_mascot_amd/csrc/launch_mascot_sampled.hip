// MASCOT kernels with the sampled-statistics code (the sampled part of a check epoch).
#include "launch_mascot.h"
#include "rule_mascot.h"

namespace mf {

int launch_mascot_sampled(const MascotCall& c, Range r)
{
    return launch_k_coh<MascotRule>(c.who, c.k, c.c, [&](auto a) { return c.fill(a); }, c.lds, c.stream, r);
}

}  // namespace mf
