// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatQ50, FormatQ51.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatQ50(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ50>(a, x_type, pass, deep, stream);
}

void LaunchFlatQ51(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ51>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip
