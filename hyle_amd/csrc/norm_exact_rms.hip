// RMSNorm launch shapes that cover the tensor exactly (norm_exact.h), in a file of their own so
// that they compile beside the LayerNorm ones.
#include "norm_exact.h"

namespace hyle_hip {

bool launch_norm_exact_rms(Elem type, const NormParams &p, const void *x, const void *w, void *y, hipStream_t stream) {
  return run_exact_typed<false>(type, p, Bound{x, w, nullptr, y}, stream);
}

}  // namespace hyle_hip
