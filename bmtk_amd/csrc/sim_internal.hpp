// Declarations shared by the two simulation drivers.
#pragma once

#include "common.hpp"

namespace bmtk {

// Whole run as one cooperative launch with state in registers and the ring in
// LDS (resident.hip).  Arguments have been validated by the caller.
int simulate_resident(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream);

}  // namespace bmtk
