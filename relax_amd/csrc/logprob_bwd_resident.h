// Launcher of the burst form of the log-prob / entropy backward (logprob_bwd_resident.hip), called from the
// dispatcher of relax_amd_logprob_entropy_bwd when rows and strides allow 16-byte accesses.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "relax_amd.h"

namespace relax_amd {

// Returns RELAX_AMD_EUNSUPPORTED (and launches nothing) when no kernel is built for this row length or element type;
// otherwise launches persistent workgroups and returns the launch status.  Same arguments and results as
// logprob_entropy_bwd_kernel.
template <typename T>
int launch_logprob_bwd_resident(const T* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                                const int32_t* token_of_row, const int64_t* targets, const float* lse,
                                const float* spx, const float* g_lp, const float* g_ent, float grad_scale,
                                const float* grad_scale_dev, float inv_t, T* dlogits, int64_t d_stride,
                                int compute_units, hipStream_t stream);

}  // namespace relax_amd
