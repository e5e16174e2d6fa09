// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatMxfp4.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatMxfp4(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatMxfp4>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip
