// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatQ4K.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatQ4K(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ4K>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip

