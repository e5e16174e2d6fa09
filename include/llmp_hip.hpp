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
#include <utility>
#include <vector>

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

namespace moe {

// src/kernels/ggml/moe_cutlass.h:42-64: the scale atoms' offset and the grouped GEMM's operands, whose layout is
// the C ABI's field for field.
constexpr std::uint64_t SfOffset(std::uint64_t row, std::uint64_t block, std::uint64_t blocks) {
  return ((((row / 128) * (blocks / 4)) + (block / 4)) * 512) + ((row % 32) * 16) + (((row % 128) / 32) * 4) + (block % 4);
}
struct GroupedGemm {
  int groups = 0;
  int n = 0;
  int k = 0;
  const std::int32_t* offsets = nullptr;
  const std::int32_t* sf_rows = nullptr;
  const void* a = nullptr;
  const void* a_scales = nullptr;
  const void* weights = nullptr;
  std::uint64_t expert_stride = 0;
  std::uint64_t codes_offset = 0;
  std::uint64_t scales_offset = 0;
  void* d = nullptr;
  void* scratch = nullptr;
};
static_assert(sizeof(GroupedGemm) == sizeof(llmp_grouped_gemm), "GroupedGemm's layout is the C ABI's");

// moe_cutlass.h:66-76; `sms` is the device's compute units here.
inline bool GroupedGemmAvailable() { return llmp_hip_grouped_gemm_available() != 0; }
inline std::size_t GroupedGemmScratch(int groups, int sms) { return llmp_hip_grouped_gemm_scratch(groups, sms); }
inline int RunGroupedGemm(const GroupedGemm& gemm, int sms, void* stream) {
  return llmp_hip_grouped_gemm_run(reinterpret_cast<const llmp_grouped_gemm*>(&gemm), sms, stream);
}

}  // namespace moe

// The quantizing KV cache stores (src/kernels/ggml/kv_quant.h:150-192 of the reference): SetRowsQuant's
// two-dimensional case, SetRowsQuantGroup over two to sixteen of them, RopeSetRowsQuant.
namespace kv {

inline constexpr std::size_t kSetRowsQuantGroupMax = 16;  // kv_quant.h:84

using Store = llmp_set_rows_store;
using RopeStore = llmp_rope_store;

inline KernelFailure SetRowsQuant(const Store& s, void* stream) {
  return FromStatus(llmp_hip_set_rows_quant(s.type, s.x, s.x_stride, s.ids, s.index_bytes, s.destination, s.row_bytes,
                                            s.k, s.rows, s.cells, stream));
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
// PackedGemvLinear / PackedGemmLinear of src/kernels/exl3/linear.h:47-54, 1 to 65536 rows in passes of sixteen.
// UpstreamPath of src/kernels/exl3/validate.h:254-256: the packed path through 144 rows (the reconstruction paths
// it names above that are not built here; the packed path still takes those rows).
enum class LinearPath : std::uint8_t { kPacked, kReconstruct, kReconstructFused };
constexpr LinearPath UpstreamPath(int rows) {
  return rows >= 1024 ? LinearPath::kReconstructFused : rows > 144 ? LinearPath::kReconstruct : LinearPath::kPacked;
}
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
// ---------------------------------------------------------------------------------------------
// The implementation registry's entries for these kernels (src/execution/registry.h:131-195 and
// 297-356 of the reference): what each implementation computes, under the names the planner and
// its plans use (src/kernels/ggml/capabilities.cc:2486-2489 and 2881-2893,
// src/kernels/ggml/plan_step.h:201-314, src/kernels/decode/implementations.h:7-13,
// src/kernels/exl3/implementations.h:8-31). The reference's types hold spans into static tables
// and IR keys; here the same facts are plain values, so that a binding can build its
// execution::Implementation from them field by field. "C++ only": nothing of this crosses the C ABI.
namespace execution {

// registry.h:50-55.
enum class Rung : std::uint8_t { kNative = 1, kOnChipDecode = 2, kBf16Decode = 5, kPrimitive = 6 };
// registry.h:75-81.
enum DeviceFeature : std::uint32_t { kBf16Mma = 1u << 0, kInt8Mma = 1u << 1, kFp8Mma = 1u << 2, kFp4Mma = 1u << 3, kBlockScaledMma = 1u << 4 };
// The provider's architecture number of the one device this library is built for.
inline constexpr std::uint32_t kGfx950 = 950;
// registry.h:91-96.
struct ShapeRule {
  std::uint64_t min_rows = 1;
  std::uint64_t max_rows = ~std::uint64_t{0};
  std::uint64_t k_multiple = 1;
  std::uint64_t n_multiple = 1;
};
// registry.h:101-170, the fields these implementations set.
struct Capability {
  std::string op;                      // the IR operation: ir::Primitive / ir::Fused's name
  std::vector<std::string> encodings;  // operand 0 (the weight, or the stored destination): any of these
  std::uint32_t min_arch = kGfx950, max_arch = kGfx950;
  std::uint32_t needs = 0;  // DeviceFeature bits
  ShapeRule shape{};
  Rung rung = Rung::kNative;
  bool row_invariant = true;  // every row computes what its one-row launch computes, bit for bit (usable in verify plans)
  bool capturable = true;     // every entry point only queues launches with replay-invariant arguments
  std::string group;          // "ggml.mul_mat" for the members of upstream's routing
  std::vector<std::string> launches;  // the entry points (llmp_hip.h) a node of it queues, in order
};
// registry.h:322-349.
struct Implementation {
  std::string name;
  std::string source = "llmp_amd";
  std::string build = "hipcc --offload-arch=gfx950 -O3";
  std::string variant;
  std::uint32_t version = 1;
  Capability capability;
};
// registry.h:297-320, the fields a product's query sets.
struct CapabilityQuery {
  std::string op;
  std::string encoding;  // operand 0's
  std::uint64_t rows = 1, k = 0, n = 0;
  std::uint32_t arch = kGfx950;
  std::uint32_t features = kBf16Mma | kInt8Mma | kFp8Mma | kFp4Mma | kBlockScaledMma;
  bool row_invariant = false;  // required
  bool capturable = false;     // required
};

inline const char* const kDecoderNames[] = {"bf16.dense",  "f16.dense",   "q8_0.blocks", "nvfp4.split", "nvfp4.atoms", "nvfp4.interleaved",
                                            "nvfp4.ggml_blocks", "mxfp8.split", "mxfp8.atoms", "mxfp4.split", "mxfp4.atoms", "affine.split"};

inline std::vector<Implementation> Implementations() {
  std::vector<Implementation> all;
  const std::vector<std::string> blocks = {"q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q4_k", "q5_k", "q6_k", "iq4_nl", "mxfp4"};
  const auto add = [&](std::string name, std::string op, std::vector<std::string> encodings, ShapeRule shape, Rung rung,
                       std::uint32_t needs, std::vector<std::string> launches, std::string variant, std::string group = "") {
    Implementation i;
    i.name = std::move(name);
    i.variant = std::move(variant);
    i.capability.op = std::move(op);
    i.capability.encodings = std::move(encodings);
    i.capability.shape = shape;
    i.capability.rung = rung;
    i.capability.needs = needs;
    i.capability.launches = std::move(launches);
    i.capability.group = std::move(group);
    all.push_back(std::move(i));
  };
  const std::uint64_t any = ~std::uint64_t{0};
  // capabilities.cc:2881-2893 and plan_step.h:201-314: the activation quantizer and the products over its blocks.
  add("llmp.q8_1", "quantize.block32_q8_sum_f32", {"f32"}, {1, 65535, 1, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize"},
      "eight lanes a block; rows padded to 512 values");
  // The default choice of form follows the token count (a weight row a lane or the F16 matrix cores for Q4_K above one
  // token): a row's bits then differ from its one-row launch's in the last place, as upstream's multi-column kernel's
  // do, so these are not candidates of a row-invariant plan.
  const auto follows_rows = [&]() { all.back().capability.row_invariant = false; };
  add("llmp.vecq.dense", "mul_mat", blocks, {1, 16, 256, 1}, Rung::kNative, kInt8Mma, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "variant -1: a lane a unit through LDS, a weight row a lane (Q4_K, 2 to 8 tokens), matrix cores above");
  follows_rows();
  add("llmp.vecq.glu", "fused.mul_mat_glu", blocks, {1, 16, 256, 1}, Rung::kNative, kInt8Mma, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "variant -1: gate and up rows in one tile, the GLU in the row's first lane");
  follows_rows();
  // The reference's row-invariant products (docs/decisions.md D-092, src/kernels/ggml/mmvq_rows.cu): the one-token
  // launch's arithmetic for every token, the weights read once for four.
  add("llmp.mul_mat.mmvq_rows", "mul_mat", blocks, {1, 16, 256, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "variant 7 (flat pass4): passes of four tokens, each the one-token product bit for bit");
  add("llmp.mul_mat_glu.mmvq_rows", "fused.mul_mat_glu", blocks, {1, 16, 256, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "variant 7 (flat pass4) with the GLU");
  add("llmp.mul_mat_id.mmvq_rows", "mul_mat_id", blocks, {1, 128, 256, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "variant 7 (flat pass4) over up to 128 (token, slot) pairs");
  add("llmp.vecq.experts", "mul_mat_id", blocks, {1, 128, 256, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "up to 128 (token, slot) pairs; the first pair naming an expert owns it");
  add("llmp.vecq.experts_glu", "fused.mul_mat_id_glu", blocks, {1, 128, 256, 1}, Rung::kNative, 0,
      {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"}, "up to 128 (token, slot) pairs, fused GLU");
  add("llmp.vecq.grouped", "fused.grouped_mul_mat", blocks, {1, 16, 256, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "matrix g with input row g: up to 256 groups");
  add("llmp.vecq.sorted", "mul_mat_id", {"q8_0", "q4_k"}, {129, any, 256, 1}, Rung::kNative, kInt8Mma,
      {"llmp_hip_moe_route", "llmp_hip_q8_1_quantize_rows", "llmp_hip_vecq_sorted"}, "rows sorted by expert on the matrix cores");
  follows_rows();
  // Upstream's routing names (capabilities.cc:2486-2489): the same launches, members of its group.
  add("ggml.mul_mat.mmvq", "mul_mat", blocks, {1, 16, 256, 1}, Rung::kNative, 0, {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"},
      "llmp.vecq.dense's launches", "ggml.mul_mat");
  follows_rows();
  add("ggml.mul_mat_glu.mmvq_fused", "fused.mul_mat_glu", blocks, {1, 16, 256, 1}, Rung::kNative, 0,
      {"llmp_hip_q8_1_quantize", "llmp_hip_vecq"}, "llmp.vecq.glu's launches", "ggml.mul_mat");
  follows_rows();
  add("llmp.moe.router", "route.softmax_top_k", {"f32"}, {1, any, 1, 1}, Rung::kNative, 0, {"llmp_hip_moe_router"},
      "a wave a token; up to 1024 experts, 64 picks");
  add("llmp.moe.experts.cutlass", "mul_mat_id", {"nvfp4"}, {1, any, 64, 1}, Rung::kOnChipDecode, kBf16Mma,
      {"llmp_hip_moe_route", "llmp_hip_grouped_gemm_run"}, "NVFP4 operands decoded to BF16 (exact), 64 x 64 tiles walked by a fixed grid");
  add("llmp.moe.combine", "fused.moe_combine", {"f32"}, {1, any, 4, 1}, Rung::kNative, 0, {"llmp_hip_moe_combine"},
      "ordered float sum over the slots");
  // MXFP8 (plan_step.h, mxfp8_cutlass.h): the reference's names, "cutlass" included, since plans carry them.
  add("llmp.mxfp8.mul_mat_vec", "mul_mat", {"mxfp8"}, {1, 16, 32, 1}, Rung::kNative, 0, {"llmp_hip_mxfp8_gemv"}, "a wave a row");
  add("llmp.mxfp8.quantize", "quantize.mxfp8", {"f32", "bf16"}, {1, any, 128, 1}, Rung::kNative, 0, {"llmp_hip_mxfp8_quantize"},
      "codes and scale atoms");
  add("llmp.mxfp8.swizzle", "relayout.scale_atoms", {"e8m0"}, {1, any, 128, 1}, Rung::kNative, 0, {"llmp_hip_mxfp8_swizzle"}, "128 x 4 atoms");
  add("llmp.mxfp8.gemm.cutlass", "mul_mat", {"mxfp8"}, {1, any, 128, 1}, Rung::kNative, kFp8Mma | kBlockScaledMma,
      {"llmp_hip_mxfp8_swizzle", "llmp_hip_mxfp8_gemm_run"}, "v_mfma_scale_f32_16x16x128_f8f6f4, 256 x 192 tiles");
  // The decode templates (decode/implementations.h:7-13): llmp.decode.<template>.<encoding>.<layout>.
  struct Template {
    const char* name;
    const char* op;
    ShapeRule shape;
    std::uint32_t needs;
    const char* launch;
  };
  const Template templates[] = {{"vector", "mul_mat", {1, 16, 16, 1}, 0, "llmp_hip_decode_vector"},
                                {"vector_glu", "fused.mul_mat_glu", {1, 16, 16, 1}, 0, "llmp_hip_decode_vector_glu"},
                                {"matrix", "mul_mat", {1, 65535ull * 64ull, 16, 1}, kBf16Mma, "llmp_hip_decode_matrix"},
                                {"grouped", "mul_mat_id", {1, any, 16, 1}, 0, "llmp_hip_decode_grouped"},
                                {"rows", "get_rows", {1, any, 16, 1}, 0, "llmp_hip_decode_rows"}};
  for (const Template& t : templates) {
    for (int d = 0; d < 12; ++d) {
      const std::string decoder = kDecoderNames[d];
      add(std::string("llmp.decode.") + t.name + "." + decoder, t.op, {decoder.substr(0, decoder.find('.'))}, t.shape,
          d < 2 ? Rung::kNative : Rung::kOnChipDecode, t.needs, {t.launch}, std::string("decoder ") + std::to_string(d));
    }
  }
  // EXL3 (exl3/implementations.h:8-31): the packed paths and the reconstruction paths.
  add("exl3.linear.gemv", "quant_linear", {"exl3"}, {1, 8, 128, 128}, Rung::kOnChipDecode, kBf16Mma, {"llmp_hip_exl3_linear"},
      "trellis tiles as the second operand of a 16 x 16 x 16 F16 matrix instruction");
  add("exl3.linear.gemm", "quant_linear", {"exl3"}, {1, 65536, 128, 128}, Rung::kOnChipDecode, kBf16Mma, {"llmp_hip_exl3_linear"},
      "the same launches in passes of sixteen rows");
  add("exl3.multi_linear.mgemm", "quant_multi_linear", {"exl3"}, {1, 65536, 128, 128}, Rung::kOnChipDecode, kBf16Mma,
      {"llmp_hip_exl3_multi_linear"}, "gate and up in grid z, passes of sixteen rows");
  // (Upstream's choice of path by rows, UpstreamPath above; the entry point itself takes any number from one.)
  add("exl3.linear.reconstruct", "quant_linear", {"exl3"}, {145, 65536, 128, 128}, Rung::kBf16Decode, kBf16Mma,
      {"llmp_hip_exl3_linear_reconstructed"}, "input transform, rotated weights to F16 and an F16 product a slice, output transform");
  add("exl3.linear.reconstruct_fused", "quant_linear", {"exl3"}, {1024, 65536, 128, 128}, Rung::kBf16Decode, kBf16Mma,
      {"llmp_hip_exl3_linear_reconstructed"}, "the weights themselves to F16 and an F16 product a slice");
  // The quantizing KV cache stores (kv_quant.h:150-192).
  add("llmp.set_rows.quant", "set_rows", {"q8_0", "q4_0"}, {1, any, 32, 1}, Rung::kNative, 0, {"llmp_hip_set_rows_quant"}, "a thread a block");
  add("llmp.set_rows.grouped_quant", "set_rows", {"q8_0", "q4_0"}, {1, any, 32, 1}, Rung::kNative, 0, {"llmp_hip_set_rows_quant_group"},
      "two to sixteen stores a launch");
  add("llmp.rope.set_rows_quant", "fused.rope_set_rows", {"q8_0", "q4_0"}, {1, any, 32, 1}, Rung::kNative, 0,
      {"llmp_hip_rope_set_rows_quant"}, "a workgroup a token");
  // The attention that reads those caches (kv_quant.h:9-26, 146-160): not row invariant (the query rows of a pass
  // share their workgroup's online softmax tiles, each row's values its own).
  for (const char* kind : {"q8_0", "q4_0"}) {
    add(std::string("ggml.flash_attn_ext.vec_") + kind, "flash_attn_ext", {kind}, {1, any, 64, 1}, Rung::kNative, 0,
        {"llmp_hip_attn_vec_quant"}, "a lane a cell for K, a lane D / 64 values for V, the cells split over workgroups");
  }
  // One token through a routed-expert layer: the router, the experts' products, their GLU and the ordered sum fused
  // (no single counterpart in the reference: ir/decompose.cc:1080-1109 holds the five operations).
  add("llmp.moe.token", "fused.moe_ffn_token", {"q4_k"}, {1, 1, 256, 256}, Rung::kNative, 0, {"llmp_hip_moe_token"},
      "two launches: router + gate/up + GLU; down + combine");
  return all;
}

// Whether `i` computes what `q` asks (registry.h's Candidates filter: operation, operand 0's encoding, device and shape).
inline bool Computes(const Implementation& i, const CapabilityQuery& q) {
  const Capability& c = i.capability;
  if (c.op != q.op || q.arch < c.min_arch || q.arch > c.max_arch || (c.needs & ~q.features) != 0) return false;
  bool encoding = c.encodings.empty();
  for (const std::string& e : c.encodings) encoding = encoding || e == q.encoding;
  if (!encoding) return false;
  if (q.rows < c.shape.min_rows || q.rows > c.shape.max_rows) return false;
  if (q.k % c.shape.k_multiple != 0 || q.n % c.shape.n_multiple != 0) return false;
  return (!q.row_invariant || c.row_invariant) && (!q.capturable || c.capturable);
}
inline std::vector<Implementation> Candidates(const CapabilityQuery& q) {
  std::vector<Implementation> found;
  for (Implementation& i : Implementations()) {
    if (Computes(i, q)) found.push_back(std::move(i));
  }
  return found;
}

}  // namespace execution
}  // namespace llmp_amd

#endif  // LLMP_HIP_HPP_
