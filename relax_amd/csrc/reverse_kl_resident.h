// Launchers of the register-resident fused reverse-KL steps (reverse_kl_resident.hip, reverse_kl_split.hip), called from the dispatcher of
// the fused step when rows and strides allow 16-byte accesses.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "relax_amd.h"

namespace relax_amd {

// Returns RELAX_AMD_EUNSUPPORTED (and launches nothing) when no kernel is built for this row length or element type;
// otherwise launches one persistent workgroup per compute unit and returns the launch status.  Same arguments and
// results as reverse_kl_step_kernel.
template <typename T>
int launch_reverse_kl_resident(const T* student, const T* teacher, int64_t stride, int64_t vocab, int64_t n_rows,
                               const float* g, float grad_scale, float* kl, float* lse_s, float* lse_t, T* dstudent,
                               int compute_units, hipStream_t stream);

// The same step as one-shot workgroups, eight to a row, that hold their share of both rows in registers and exchange
// their partial sums through device memory (reverse_kl_split.hip): RELAX_AMD_EUNSUPPORTED for the same rows as above.
template <typename T>
int launch_reverse_kl_split(const T* student, const T* teacher, int64_t stride, int64_t vocab, int64_t n_rows,
                            const float* g, float grad_scale, float* kl, float* lse_s, float* lse_t, T* dstudent,
                            hipStream_t stream);

}  // namespace relax_amd
