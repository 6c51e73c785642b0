#pragma once
#include <nbla/hip/defs.hpp>
namespace nbla {
// Registers the "hip" backend, its array classes and synchronizers, and the
// normalization functions under "hip:float" and "hip:half".  Idempotent and
// thread-safe.  Counterpart of init_cuda()/init_cudnn()
// (src/nbla/cuda/init.cpp.tmpl:65-270, src/nbla/cuda/cudnn/init.cpp.tmpl:43-73).
NBLA_HIP_API void init_hip();
} // namespace nbla
