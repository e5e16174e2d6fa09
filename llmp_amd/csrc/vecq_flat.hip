// llmp.vecq's streaming form (vecq_flat.h): which shapes it takes, and the dispatch to the formats' translation units.
#include "vecq_flat.h"

namespace llmp_hip {

// Q4_K rows up to 64 super-blocks (32 with a GLU). Q8_0 rows of whole 256 values up to 64 units
// (32 with a GLU) whose rows, matrices and experts all start on 16-byte boundaries: the
// tiles are fetched in 16-byte chunks. The legacy 4/5-bit blocks likewise, in whole 256 values. Without a GLU, and unless `whole_rows` asks for a row
// in one tile (the block sums), longer rows in pieces, as long as their records fit.
bool FlatTakes(int type, const llmp_vecq_desc& d, bool whole_rows) {
  if (d.ncols_x < 256) return false;  // every format's unit is 256 values: no plan is made for a row without one
  const bool glu = d.g != nullptr;
  const int most = glu ? kWave / 2 : kWave;
  const bool pieces = !glu && !whole_rows;
  if (type == LLMP_TYPE_Q4_K) {
    const int units = d.ncols_x / FormatQ4K::kUnitValues;
    if (units > most) return pieces && PlanSplit<FormatQ4K>(units).lds <= kFlatLdsLimit;
    return units >= 1 && PlanFits(PlanFlat<FormatQ4K>(1, units, glu));
  }
  if (type == LLMP_TYPE_Q6_K) {
    // 210-byte blocks: matrices and experts at 16-byte boundaries and of a multiple of eight blocks (a tile's
    // last chunk then ends within its matrix); rows packed, or of a multiple of eight blocks themselves.
    const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
    const int units = d.ncols_x / FormatQ6K::kUnitValues;
    if (at % 16 != 0 || d.stride_expert % 8 != 0 || units < 1 || units > most) return false;
    if (d.stride_row != units && (units % 8 != 0 || d.stride_row % 8 != 0)) return false;
    return (static_cast<int64_t>(d.nrows) * units) % 8 == 0 && PlanFits(PlanFlat<FormatQ6K>(1, units, glu));
  }
  if (type == LLMP_TYPE_Q5_K) {
    const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
    if (at % 16 != 0) return false;
    const int units = d.ncols_x / FormatQ5K::kUnitValues;
    if (units > most) return pieces && PlanSplit<FormatQ5K>(units).lds <= kFlatLdsLimit;
    return units >= 1 && PlanFits(PlanFlat<FormatQ5K>(1, units, glu));
  }
  if (type == LLMP_TYPE_Q4_0 || type == LLMP_TYPE_Q4_1 || type == LLMP_TYPE_Q5_0 || type == LLMP_TYPE_Q5_1 ||
      type == LLMP_TYPE_IQ4_NL) {
    const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
    if (d.ncols_x % 256 != 0 || d.stride_row % 8 != 0 || d.stride_expert % 8 != 0 || at % 16 != 0) return false;
    const int units = d.ncols_x / 256;
    const auto fits = [&](auto format) {
      using F = decltype(format);
      if (units > most) return pieces && PlanSplit<F>(units).lds <= kFlatLdsLimit;
      return PlanFits(PlanFlat<F>(1, units, glu));
    };
    return type == LLMP_TYPE_Q4_0 ? fits(FormatQ40{}) : type == LLMP_TYPE_IQ4_NL ? fits(FormatIq4nl{}) : type == LLMP_TYPE_Q4_1 ? fits(FormatQ41{})
           : type == LLMP_TYPE_Q5_0 ? fits(FormatQ50{}) : fits(FormatQ51{});
  }
  if (type == LLMP_TYPE_MXFP4) {
    // A 136-byte unit: rows of an even number of units, everything on 16-byte boundaries.
    const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
    if (d.ncols_x % 512 != 0 || d.stride_row % 16 != 0 || d.stride_expert % 16 != 0 || at % 16 != 0) return false;
    const int units = d.ncols_x / 256;
    if (units > most) return pieces && PlanSplit<FormatMxfp4>(units).lds <= kFlatLdsLimit;
    return PlanFits(PlanFlat<FormatMxfp4>(1, units, glu));
  }
  if (type != LLMP_TYPE_Q8_0 || d.ncols_x % 256 != 0) return false;
  const int units = d.ncols_x / FormatQ8::kUnitValues;
  const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
  if (d.stride_row % 8 != 0 || d.stride_expert % 8 != 0 || at % 16 != 0) return false;
  if (units > most) return pieces && PlanSplit<FormatQ8>(units).lds <= kFlatLdsLimit;
  return PlanFits(PlanFlat<FormatQ8>(1, units, glu));
}

// One launcher a format, each in its own translation unit (vecq_flat_*.hip).
void LaunchFlatQ4K(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ5K(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ6K(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ40(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatIq4nl(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ41(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ50(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ51(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatMxfp4(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);
void LaunchFlatQ8(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);

void LaunchFlat(int type, const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  switch (type) {
    case LLMP_TYPE_Q4_K: LaunchFlatQ4K(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_Q5_K: LaunchFlatQ5K(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_Q6_K: LaunchFlatQ6K(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_Q4_0: LaunchFlatQ40(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_IQ4_NL: LaunchFlatIq4nl(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_Q4_1: LaunchFlatQ41(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_Q5_0: LaunchFlatQ50(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_Q5_1: LaunchFlatQ51(a, x_type, pass, deep, stream); break;
    case LLMP_TYPE_MXFP4: LaunchFlatMxfp4(a, x_type, pass, deep, stream); break;
    default: LaunchFlatQ8(a, x_type, pass, deep, stream); break;
  }
}

}  // namespace llmp_hip
