// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatQ8.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatQ8(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ8>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip

#ifdef LLMP_VECQ_TRACE
// The tuning build's switch for this unit's kernels (see vecq_flat_q4k.hip).
extern "C" int llmp_hip_trace_set_q8(unsigned long long* buffer) {
  return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(llmp_hip::g_trace), &buffer, sizeof(buffer)));
}
#endif
