// The token-granular decode kernels for 64-element head rows (see kin_token_kernel.h).
#include "kin_token_kernel.h"

namespace kin {

const void* token_kernel_small_head(bool f16, bool strided, int group, int nw, bool ldsk) {
  return token_kernel_for<kHeadDimSmall>(f16, strided, group, nw, ldsk);
}

}  // namespace kin
