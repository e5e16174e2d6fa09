// The host side of the MI355X kernels in the reference's own C++ vocabulary: the launch
// interfaces its operator wrappers call (src/kernels/ggml/vecq.h:22-47,
// src/kernels/ggml/mxfp8_cutlass.h:26-79, src/kernels/exl3/validate.h:84-131 and
// src/kernels/exl3/linear.h:47-54, src/kernels/decode/products.h:96-109,
// src/kernels/selected_operation.h:26-35 of the reference),
// with the same names, argument meaning and error behaviour, over the C ABI of llmp_hip.h.
// Header only, C++17, no HIP or torch types: a stream is the void* the reference's
// NativeStream carries.
#ifndef LLMP_HIP_HPP_
#define LLMP_HIP_HPP_

#include <cstddef>
#include <cstdint>
#include <string>

#include "llmp_hip.h"

namespace llmp_amd {

// src/kernels/selected_operation.h:26-35: a refusal queues nothing; anything else may have
// queued work and faults the caller's launch context.
enum class KernelFailure { kNone, kRejected, kUnknown };

inline KernelFailure FromStatus(int status) {
  return status == 0 ? KernelFailure::kNone : status > 0 ? KernelFailure::kRejected : KernelFailure::kUnknown;
}
inline std::string LastError() { return llmp_hip_last_error(); }

namespace ggml {

// ggml_type values of the encodings these kernels read.
enum Type : int {
  kQ4_0 = LLMP_TYPE_Q4_0,
  kQ4_1 = LLMP_TYPE_Q4_1,
  kQ5_0 = LLMP_TYPE_Q5_0,
  kQ5_1 = LLMP_TYPE_Q5_1,
  kQ8_0 = LLMP_TYPE_Q8_0,
  kQ4_K = LLMP_TYPE_Q4_K,
  kMXFP4 = LLMP_TYPE_MXFP4,
  kIQ4_NL = LLMP_TYPE_IQ4_NL,
  kQ5_K = LLMP_TYPE_Q5_K,
  kQ6_K = LLMP_TYPE_Q6_K
};
// VecQGlu, src/kernels/ggml/llmp_ops.h:1072.
enum VecQGlu : int { kNone = LLMP_GLU_NONE, kSwiGlu = LLMP_GLU_SWIGLU, kSwiGluClamp = LLMP_GLU_SWIGLU_CLAMP, kGeGlu = LLMP_GLU_GEGLU };

// What a llmp.vecq launch reads and writes (src/kernels/ggml/vecq.h:22-41). Weight offsets
// count the weight type's blocks; activation offsets count Q8_1 blocks (36 bytes).
struct VecQDesc {
  const void* w = nullptr;
  const void* g = nullptr;
  const void* y = nullptr;
  const std::int32_t* ids = nullptr;
  float* dst = nullptr;
  int ncols_x = 0;
  int nrows = 0;
  int stride_row = 0;
  int stride_expert = 0;
  int y_token = 0;
  int y_slot = 0;
  int ids_stride = 0;
  int used = 1;
  int tokens = 1;
  int dst_token = 0;
  int dst_slot = 0;
  int glu = 0;
  float limit = 0.0f;
};

inline llmp_vecq_desc ToAbi(const VecQDesc& d) {
  return llmp_vecq_desc{d.w,      d.g,      d.y,          d.ids,  d.dst,    d.ncols_x,   d.nrows,    d.stride_row, d.stride_expert,
                        d.y_token, d.y_slot, d.ids_stride, d.used, d.tokens, d.dst_token, d.dst_slot, d.glu,        d.limit};
}

// src/kernels/ggml/vecq.h:43-47: -1 is the default choice for the shape; false for a variant
// the shape cannot take (and for any other refusal: LastError() names it).
inline int VecQVariants() { return llmp_hip_vecq_variants(); }
inline std::string VecQVariantName(int variant) {
  const char* name = llmp_hip_vecq_variant_name(variant);
  return name != nullptr ? name : "";
}
inline bool LaunchVecQ(int type, const VecQDesc& d, int variant, void* stream) {
  const llmp_vecq_desc abi = ToAbi(d);
  return llmp_hip_vecq(type, &abi, variant, stream) == 0;
}

// quantize_row_q8_1_cuda as RunQuantizeQ8 calls it (src/kernels/ggml/vecq.cu:1095-1111).
inline KernelFailure QuantizeQ8(const float* x, void* out, std::int64_t k, std::int64_t padded_k, std::int64_t rows,
                                void* stream) {
  return FromStatus(llmp_hip_q8_1_quantize(x, out, k, padded_k, k, rows, 1, rows * k, stream));
}
// src/kernels/ggml/llmp_ops.cc:2574-2576: rows are padded with zero blocks to a multiple of 512.
constexpr std::int64_t PaddedK(std::int64_t k) { return (k + 511) / 512 * 512; }

namespace mxfp8 {

// src/kernels/ggml/mxfp8_cutlass.h:28-57.
inline constexpr std::uint64_t kBlock = 32;
inline constexpr std::uint64_t kAtomRows = 128;
constexpr std::uint64_t PaddedRows(std::uint64_t rows) { return (rows + kAtomRows - 1) / kAtomRows * kAtomRows; }
constexpr std::uint64_t SwizzledScaleBytes(std::uint64_t n, std::uint64_t k) { return PaddedRows(n) * (k / kBlock); }

// src/kernels/ggml/mxfp8_cutlass.h:59-71.
struct Gemm {
  int m = 0;
  int n = 0;
  int k = 0;
  const void* a = nullptr;
  const void* a_scales = nullptr;
  const void* b = nullptr;
  const void* b_scales = nullptr;
  void* d = nullptr;
  bool bf16 = false;
  void* scratch = nullptr;
};

inline llmp_mxfp8_gemm ToAbi(const Gemm& g) {
  llmp_mxfp8_gemm abi{};
  abi.m = g.m, abi.n = g.n, abi.k = g.k;
  abi.a = g.a, abi.a_scales = g.a_scales, abi.b = g.b, abi.b_scales = g.b_scales;
  abi.d = g.d, abi.bf16 = g.bf16 ? 1 : 0, abi.scratch = g.scratch;
  return abi;
}

// src/kernels/ggml/mxfp8_cutlass.h:73-79; `sms` is the device's compute units here.
inline bool Available() { return llmp_hip_mxfp8_gemm_available() != 0; }
inline std::size_t Scratch(const Gemm& gemm, int sms) {
  const llmp_mxfp8_gemm abi = ToAbi(gemm);
  return llmp_hip_mxfp8_gemm_scratch(&abi, sms);
}
inline int Run(const Gemm& gemm, int sms, void* stream) {
  const llmp_mxfp8_gemm abi = ToAbi(gemm);
  return llmp_hip_mxfp8_gemm_run(&abi, sms, stream);
}

}  // namespace mxfp8

// The quantizing KV cache stores (src/kernels/ggml/kv_quant.h:150-192 of the reference): SetRowsQuant's
// two-dimensional case, SetRowsQuantGroup over two to sixteen of them, RopeSetRowsQuant.
namespace kv {

inline constexpr std::size_t kSetRowsQuantGroupMax = 16;  // kv_quant.h:84

using Store = llmp_set_rows_store;
using RopeStore = llmp_rope_store;

inline KernelFailure SetRowsQuant(const Store& s, void* stream) {
  return FromStatus(llmp_hip_set_rows_quant(s.type, s.x, s.x_stride, s.ids, s.index_bytes, s.destination, s.row_bytes,
                                            s.k, s.rows, stream));
}
inline KernelFailure SetRowsQuantGroup(const Store* stores, std::size_t count, void* stream) {
  return FromStatus(llmp_hip_set_rows_quant_group(static_cast<int>(count), stores, stream));
}
inline KernelFailure RopeSetRowsQuant(const RopeStore& s, void* stream) {
  return FromStatus(llmp_hip_rope_set_rows_quant(&s, stream));
}

}  // namespace kv
}  // namespace ggml

namespace decode {

// src/kernels/decode/operand.h:26-41.
enum class DecoderId : std::uint8_t {
  kBf16Dense, kF16Dense, kQ8_0Blocks, kNvfp4Split, kNvfp4Atoms, kNvfp4Interleaved, kNvfp4GgmlBlocks,
  kMxfp8Split, kMxfp8Atoms, kMxfp4Split, kMxfp4Atoms, kAffineSplit, kCount
};
// src/kernels/decode/operand.h:74-97: the C ABI's operand is that struct field for field.
using Operand = llmp_decode_operand;
static_assert(sizeof(Operand) == 64, "Operand descriptor must be 64 bytes");

// The arguments of RunVector (src/kernels/decode/products.h:96-109) once OperandOf has bound the weight.
struct Product {
  DecoderId decoder = DecoderId::kBf16Dense;
  Operand weight{};
  std::uint64_t first = 0;
  std::uint64_t outputs = 0;
  const float* x = nullptr;
  std::uint64_t rows = 0;
  std::uint64_t x_stride = 0;
  float* y = nullptr;
  std::uint64_t y_stride = 0;
};
// RunMatrix (src/kernels/decode/products.h:111-118): MatrixPath::kMma is path 0, kFma (refused here) 1.
enum class MatrixPath : std::uint8_t { kMma, kFma };
inline KernelFailure RunMatrix(const Product& p, MatrixPath path, void* stream) {
  return FromStatus(llmp_hip_decode_matrix(static_cast<int>(p.decoder), &p.weight, p.first, p.outputs, p.x, p.rows,
                                           p.x_stride, p.y, p.y_stride, static_cast<int>(path), stream));
}
inline KernelFailure RunVector(const Product& p, void* stream) {
  return FromStatus(llmp_hip_decode_vector(static_cast<int>(p.decoder), &p.weight, p.first, p.outputs, p.x, p.rows,
                                           p.x_stride, p.y, p.y_stride, stream));
}

// GluProduct and RunVectorGlu (src/kernels/decode/products.h:120-139); `glu` is ir::GluKind's value
// (src/ir/op.h:455), `limit` GluParams::limit.
struct GluProduct {
  DecoderId gate_decoder = DecoderId::kBf16Dense;
  Operand gate{};
  std::uint64_t gate_first = 0;
  DecoderId up_decoder = DecoderId::kBf16Dense;
  Operand up{};
  std::uint64_t up_first = 0;
  std::uint64_t outputs = 0;
  int glu = 0;
  float limit = 0.0f;
  const float* x = nullptr;
  std::uint64_t rows = 0;
  std::uint64_t x_stride = 0;
  float* y = nullptr;
  std::uint64_t y_stride = 0;
};
inline KernelFailure RunVectorGlu(const GluProduct& p, void* stream) {
  return FromStatus(llmp_hip_decode_vector_glu(static_cast<int>(p.gate_decoder), &p.gate, p.gate_first,
                                               static_cast<int>(p.up_decoder), &p.up, p.up_first, p.outputs, p.glu,
                                               p.limit, p.x, p.rows, p.x_stride, p.y, p.y_stride, stream));
}

// RowsGather and RunRows (src/kernels/decode/products.h:172-183).
struct RowsGather {
  DecoderId decoder = DecoderId::kBf16Dense;
  Operand weight{};
  const std::int32_t* ids = nullptr;
  std::uint64_t count = 0;
  float* out = nullptr;
  std::uint64_t out_stride = 0;
  std::int32_t* bad = nullptr;
};
inline KernelFailure RunRows(const RowsGather& g, void* stream) {
  return FromStatus(llmp_hip_decode_rows(static_cast<int>(g.decoder), &g.weight, g.ids, g.count, g.out, g.out_stride,
                                         g.bad, stream));
}

// GroupedProduct and RunGrouped (src/kernels/decode/products.h:141-170); `k` and `n` are the format's.
struct GroupedProduct {
  DecoderId decoder = DecoderId::kBf16Dense;
  std::uint32_t k = 0;
  std::uint32_t n = 0;
  const Operand* experts = nullptr;  // device memory
  std::uint64_t experts_count = 0;
  std::uint64_t first = 0;
  std::uint64_t outputs = 0;
  const std::int32_t* offsets = nullptr;
  const std::int32_t* pair_rows = nullptr;
  const std::int32_t* pair_out = nullptr;
  std::uint64_t pairs = 0;
  const float* x = nullptr;
  std::uint64_t x_rows = 0;
  std::uint64_t x_stride = 0;
  float* y = nullptr;
  std::uint64_t y_rows = 0;
  std::uint64_t y_stride = 0;
  std::uint64_t rows_hint = 0;
};
inline KernelFailure RunGrouped(const GroupedProduct& p, void* stream) {
  return FromStatus(llmp_hip_decode_grouped(static_cast<int>(p.decoder), p.experts, p.experts_count, p.k, p.n, p.first,
                                            p.outputs, p.offsets, p.pair_rows, p.pair_out, p.pairs, p.x, p.x_rows,
                                            p.x_stride, p.y, p.y_rows, p.y_stride, p.rows_hint, stream));
}

}  // namespace decode

namespace exl3 {

// src/format/encoding.h:121.
enum Codebook : int { k3Inst = LLMP_EXL3_3INST, kMcg = LLMP_EXL3_MCG, kMul1 = LLMP_EXL3_MUL1 };

// src/kernels/exl3/validate.h:84-96 (the weights) and :118-131 (LinearOperands): addresses as
// the reference carries them, uint64.
struct Weights {
  std::uint64_t trellis = 0;
  std::uint64_t suh = 0;
  std::uint64_t svh = 0;
  int k = 0;
  int n = 0;
  int bits = 0;
  int codebook = kMcg;
};
struct LinearOperands {
  Weights weights;
  std::uint64_t x = 0;      // m x k F16
  std::uint64_t a_had = 0;  // m x k F16 scratch for the transformed input
  std::uint64_t y = 0;      // m x n
  bool f32 = false;         // y in F32, else F16
  int m = 0;
};

inline llmp_exl3_linear ToAbi(const LinearOperands& o) {
  llmp_exl3_linear abi{};
  abi.weights.trellis = reinterpret_cast<const void*>(o.weights.trellis);
  abi.weights.suh = reinterpret_cast<const void*>(o.weights.suh);
  abi.weights.svh = reinterpret_cast<const void*>(o.weights.svh);
  abi.weights.k = o.weights.k, abi.weights.n = o.weights.n;
  abi.weights.bits = o.weights.bits, abi.weights.codebook = o.weights.codebook;
  abi.x = reinterpret_cast<const void*>(o.x);
  abi.a_had = reinterpret_cast<void*>(o.a_had);
  abi.y = reinterpret_cast<void*>(o.y);
  abi.f32 = o.f32 ? 1 : 0, abi.m = o.m;
  return abi;
}

// The bytes of the partial-sum area a packed linear needs (the reference's lock area,
// src/kernels/exl3/launch.h:13-36, is the caller's in the same way).
inline std::size_t ScratchBytes(const LinearOperands& o) {
  const llmp_exl3_linear abi = ToAbi(o);
  return llmp_hip_exl3_linear_scratch(&abi);
}
// PackedGemvLinear / PackedGemmLinear of src/kernels/exl3/linear.h:47-54, 1 to 16 rows.
inline KernelFailure PackedLinear(const LinearOperands& o, void* scratch, std::size_t scratch_bytes, void* stream) {
  const llmp_exl3_linear abi = ToAbi(o);
  return FromStatus(llmp_hip_exl3_linear(&abi, scratch, scratch_bytes, stream));
}

// src/kernels/exl3/validate.h:160-172 without the pointer tables (the launches carry the
// addresses): a gate and an up linear over one input, y the first's m x n rows then the second's.
struct MultiLinearOperands {
  Weights first;
  Weights second;
  std::uint64_t x = 0;      // m x k F16
  std::uint64_t a_had = 0;  // 2 x m x k F16 scratch
  std::uint64_t y = 0;      // 2 x m x n
  bool f32 = false;
  int m = 0;
};

inline llmp_exl3_multi_linear ToAbi(const MultiLinearOperands& o) {
  LinearOperands one;
  one.weights = o.first;
  llmp_exl3_multi_linear abi{};
  abi.first = ToAbi(one).weights;
  one.weights = o.second;
  abi.second = ToAbi(one).weights;
  abi.x = reinterpret_cast<const void*>(o.x);
  abi.a_had = reinterpret_cast<void*>(o.a_had);
  abi.y = reinterpret_cast<void*>(o.y);
  abi.f32 = o.f32 ? 1 : 0, abi.m = o.m;
  return abi;
}
inline std::size_t ScratchBytes(const MultiLinearOperands& o) {
  const llmp_exl3_multi_linear abi = ToAbi(o);
  return llmp_hip_exl3_multi_linear_scratch(&abi);
}
// MultiLinear of src/kernels/exl3/linear.h:51-53.
inline KernelFailure MultiLinear(const MultiLinearOperands& o, void* scratch, std::size_t scratch_bytes, void* stream) {
  const llmp_exl3_multi_linear abi = ToAbi(o);
  return FromStatus(llmp_hip_exl3_multi_linear(&abi, scratch, scratch_bytes, stream));
}

}  // namespace exl3
}  // namespace llmp_amd

#endif  // LLMP_HIP_HPP_
