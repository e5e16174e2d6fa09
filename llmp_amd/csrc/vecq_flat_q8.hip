// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatQ8.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatQ8(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ8>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip

