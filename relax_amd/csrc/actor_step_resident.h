// Launcher of the register-resident fused actor step (actor_step_resident.hip), called from the dispatcher of the
// fused step when rows and strides allow 16-byte accesses.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "relax_amd.h"

namespace relax_amd {

// Returns RELAX_AMD_EUNSUPPORTED (and launches nothing) when no kernel is built for this row length or element type;
// otherwise launches one persistent workgroup per compute unit and returns the launch status.  Same arguments and
// results as actor_step_fused_kernel.
template <typename T>
int launch_actor_step_resident(const T* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                               const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                               float inv_t, const relax_amd_policy_loss_args& a, float grad_scale, float* log_prob,
                               float* entropy, float* lse, float* spx, T* dlogits, int64_t d_stride,
                               int compute_units, hipStream_t stream);

// The same for fp32 rows of 100352 .. 163840 entries, kept in the registers as their upper halves when those are all
// there is to them (actor_step_resident_wide.hip).
int launch_actor_step_resident_wide(const float* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                                    const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                                    float inv_t, const relax_amd_policy_loss_args& a, float grad_scale,
                                    float* log_prob, float* entropy, float* lse, float* spx, float* dlogits,
                                    int64_t d_stride, int compute_units, hipStream_t stream);

// The same step, same bits, with every row shared between eight one-shot 128-thread workgroups that exchange their
// waves' partial softmax sums through device memory (actor_step_split.hip); the row shapes of
// launch_actor_step_resident and launch_actor_step_resident_wide, and longer and shorter rows besides.
template <typename T>
int launch_actor_step_split(const T* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                            const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                            float inv_t, const relax_amd_policy_loss_args& a, float grad_scale, float* log_prob,
                            float* entropy, float* lse, float* spx, T* dlogits, int64_t d_stride,
                            hipStream_t stream);

}  // namespace relax_amd
