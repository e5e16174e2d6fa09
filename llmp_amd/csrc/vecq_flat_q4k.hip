// llmp.vecq's streaming form (vecq_flat.h) instantiated for: FormatQ4K.
#include "vecq_flat.h"

namespace llmp_hip {

void LaunchFlatQ4K(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  LaunchF<FormatQ4K>(a, x_type, pass, deep, stream);
}

}  // namespace llmp_hip

#ifdef LLMP_VECQ_TRACE
// The tuning build's switch: where the waves' timestamps go (device memory, eight 64-bit words a wave), or null.
extern "C" int llmp_hip_trace_set(unsigned long long* buffer) {
  return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(llmp_hip::g_trace), &buffer, sizeof(buffer)));
}
#endif
