// Priority order of the kernel variants (fastest first, generic last).
#include "variants.h"

namespace tvx {

const std::vector<ConvSetupFn>& ConvVariants() {
  static const std::vector<ConvSetupFn> v = {DwConv3x3Setup, DwPlanesSetup, PwConvSetup, ConvIm2colSetup, ConvBandSetup, ConvIgemmSetup, ConvIgemmF16Setup, ConvGemmSetup, ConvGenericSetup};
  return v;
}

const std::vector<FcSetupFn>& FcVariants() {
  static const std::vector<FcSetupFn> v = {FcMfmaSetup, FcGenericSetup};
  return v;
}

const std::vector<SimpleSetupFn>& PoolVariants() {
  static const std::vector<SimpleSetupFn> v = {PoolStencilSetup, PoolRowsSetup, PoolGenericSetup};
  return v;
}

}  // namespace tvx
