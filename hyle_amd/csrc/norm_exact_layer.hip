// LayerNorm launch shapes that cover the tensor exactly (norm_exact.h), in a file of their own so
// that they compile beside the RMSNorm ones.
#include "norm_exact.h"

namespace hyle_hip {

bool launch_norm_exact_layer(Elem type, const NormParams &p, const void *x, const void *w, const void *b, void *y,
                             hipStream_t stream) {
  return run_exact_typed<true>(type, p, Bound{x, w, b, y}, stream);
}

}  // namespace hyle_hip
