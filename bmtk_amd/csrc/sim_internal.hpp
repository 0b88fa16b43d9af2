// Declarations shared by the two simulation drivers.
#pragma once

#include "common.hpp"

namespace bmtk {

constexpr int kActCap = 8192;                                   // active-row list of the resident kernel (entries)
constexpr size_t kResLdsBytes = 160u * 1024u;                   // LDS of one gfx950 compute unit
constexpr size_t kResLdsExtra = kActCap * sizeof(int) + 256u;   // the list plus the kernel's static LDS (rounded up)
// the single-workgroup form, with span elements: spike offsets and probed potentials of two steps, the items (rows to
// walk) of two steps, its static LDS (rounded up)
constexpr size_t solo_lds_extra(int span) { return (size_t)span * 4u * sizeof(float) + 10240u + 2048u; }

// Whole run as one cooperative launch with state in registers and the ring in
// LDS (resident.hip).  Arguments have been validated by the caller.
int simulate_resident(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream);

// The same for a network that fits ONE workgroup (res_groups == 1): no grid barrier, ballots handed over in LDS,
// whole synapse rows walked by a wavefront (resident_solo.hip).
int simulate_resident_solo(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream);

// Batched runs, one launch per step with the pull of a step's arrivals and the update fused (simulate_fused.hip).
int simulate_fused(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream);

}  // namespace bmtk
