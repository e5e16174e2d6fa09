// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatQ40, FormatIq4nl, FormatQ41.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatQ40(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ40>(a, x_type, pass, deep, stream);
}

void LaunchFlatIq4nl(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatIq4nl>(a, x_type, pass, deep, stream);
}

void LaunchFlatQ41(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ41>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip
