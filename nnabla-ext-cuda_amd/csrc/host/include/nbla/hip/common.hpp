// Backend-wide helpers of the "hip" context: status-to-exception conversion
// for the C-ABI kernel layer, device selection, type mapping.  Counterpart of
// the reference's include/nbla/cuda/common.hpp:70-85 (NBLA_CUDA_CHECK) and
// src/nbla/cuda/common.cpp:20-32 (cuda_set_device).  Host C++ includes no HIP
// header: everything device-related goes through nblahip.h.
#pragma once

#include <nbla/common.hpp>
#include <nbla/exception.hpp>
#include <nbla/half.hpp>
#include <nbla/hip/defs.hpp>
#include <nblahip.h>

namespace nbla {

// Throws nbla::Exception(target_specific) for a non-zero C-ABI status.
#define NBLA_HIP_CHECK(expr)                                                           \
  do {                                                                                 \
    const int nbla_hip_status_ = (expr);                                               \
    if (nbla_hip_status_ != 0) {                                                       \
      NBLA_ERROR(::nbla::error_code::target_specific, "(%s) failed with status %d: %s", #expr, \
                 nbla_hip_status_, nblahip_error_string(nbla_hip_status_));            \
    }                                                                                  \
  } while (0)

// Same for destructors: report, never throw.
#define NBLA_HIP_FORCE_ASSERT(expr)                                                    \
  do {                                                                                 \
    const int nbla_hip_status_ = (expr);                                               \
    if (nbla_hip_status_ != 0)                                                         \
      std::fprintf(stderr, "[nbla hip] (%s) failed with status %d: %s\n", #expr,       \
                   nbla_hip_status_, nblahip_error_string(nbla_hip_status_));          \
  } while (0)

NBLA_HIP_API void hip_set_device(int device);
NBLA_HIP_API int hip_get_device();

// Storage type of the activation tensors of a type config -> C-ABI dtype code.
template <typename T> struct HipDtype;
template <> struct HipDtype<float> { static constexpr int code = NBLAHIP_F32; };
template <> struct HipDtype<Half> { static constexpr int code = NBLAHIP_F16; };

inline int hip_dtype_code(dtypes d) {
  NBLA_CHECK(d == dtypes::FLOAT || d == dtypes::HALF, error_code::type,
             "The hip backend fills and converts float32 and float16 only (other dtypes are "
             "stored and copied).");
  return d == dtypes::FLOAT ? NBLAHIP_F32 : NBLAHIP_F16;
}

} // namespace nbla
