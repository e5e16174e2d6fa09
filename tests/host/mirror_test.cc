// The C++ host mirror (include/llmp_hip.hpp) exercised the way the reference's unit tests
// exercise its launch interfaces (tests/unit/dsv4_fast_test.cc:300-520 builds blocks, runs the
// op and compares with a scalar definition): "host" checks what needs no GPU (refusals queue
// nothing and name their reason, the layout arithmetic); "device" runs small Q8_0 and Q4_K
// products, a fused gate/up pair and the Q8_1 quantizer on the GPU and compares them with the
// CPU oracle (oracle/oracle.h: test infrastructure, linked here as the checker only).
//
// Usage: mirror_test host | device. Exit status 0 when every check holds.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstddef>
#include <cstring>
#include <set>
#include <string>
#include <vector>

#include "llmp_hip.hpp"

extern "C" {
#include "oracle.h"
}

namespace {

int g_failures = 0;

#define EXPECT(condition)                                                     \
  do {                                                                        \
    if (!(condition)) {                                                       \
      std::printf("%s:%d: EXPECT(%s) failed\n", __FILE__, __LINE__, #condition); \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

namespace hipk = llmp_amd;
using hipk::ggml::VecQDesc;

// splitmix64: seeded bytes and floats that do not depend on a library's distributions.
struct Rng {
  std::uint64_t state;
  std::uint64_t Next() {
    std::uint64_t z = (state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  float Unit() { return static_cast<float>(Next() >> 40) * (1.0f / 16777216.0f); }  // [0, 1)
  float Normal() {
    const float u = Unit() + 1e-7f, v = Unit();
    return std::sqrt(-2.0f * std::log(u)) * std::cos(6.2831853f * v);
  }
};

std::uint16_t HalfBits(float v) { return orc_f32_to_f16(v); }

// n rows of k values as Q8_0 / Q4_K blocks with plausible scales and uniform codes.
std::vector<std::uint8_t> Weights(int type, int n, int k, std::uint64_t seed) {
  Rng rng{seed};
  const int bytes = orc_block_bytes(type), elements = orc_block_elements(type);
  std::vector<std::uint8_t> w(static_cast<std::size_t>(n) * (k / elements) * bytes);
  for (std::size_t at = 0; at < w.size(); at += bytes) {
    for (int i = 0; i < bytes; ++i) w[at + i] = static_cast<std::uint8_t>(rng.Next());
    const std::uint16_t d = HalfBits(0.002f + 0.01f * rng.Unit());
    std::memcpy(&w[at], &d, 2);
    if (type == hipk::ggml::kQ4_K) {
      const std::uint16_t dmin = HalfBits(0.001f + 0.005f * rng.Unit());
      std::memcpy(&w[at + 2], &dmin, 2);
    }
  }
  return w;
}

template <typename T>
T* ToDevice(const std::vector<T>& host) {
  T* device = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&device), host.size() * sizeof(T)) != hipSuccess) return nullptr;
  if (hipMemcpy(device, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return device;
}

double WorstRelative(const std::vector<float>& got, const std::vector<float>& want) {
  double square = 0.0;
  for (float v : want) square += static_cast<double>(v) * v;
  const double floor = 1e-3 * std::sqrt(square / want.size());
  double worst = 0.0;
  for (std::size_t i = 0; i < want.size(); ++i) {
    const double error = std::fabs(static_cast<double>(got[i]) - want[i]) / std::fmax(std::fabs(want[i]), floor);
    worst = std::fmax(worst, error);
  }
  return worst;
}

void HostChecks() {
  // A refusal queues nothing and names its reason (src/kernels/ggml/vecq.h:43-47: false).
  VecQDesc d;
  EXPECT(!hipk::ggml::LaunchVecQ(hipk::ggml::kQ4_K, d, -1, nullptr));
  EXPECT(!hipk::LastError().empty());
  d.w = reinterpret_cast<const void*>(0x1000), d.y = reinterpret_cast<const void*>(0x2000);
  d.dst = reinterpret_cast<float*>(0x3000);
  d.ncols_x = 256, d.nrows = 4, d.stride_row = 1, d.y_token = 16, d.dst_token = 4;
  EXPECT(!hipk::ggml::LaunchVecQ(4, d, -1, nullptr));                          // not a type these kernels read
  EXPECT(!hipk::ggml::LaunchVecQ(hipk::ggml::kQ4_K, d, 99, nullptr));          // no such variant
  d.tokens = 17;
  EXPECT(!hipk::ggml::LaunchVecQ(hipk::ggml::kQ4_K, d, -1, nullptr));          // 1 to 16 tokens
  EXPECT(hipk::ggml::VecQVariants() >= 1);
  for (int v = 0; v < hipk::ggml::VecQVariants(); ++v) EXPECT(!hipk::ggml::VecQVariantName(v).empty());
  EXPECT(hipk::FromStatus(0) == hipk::KernelFailure::kNone);
  EXPECT(hipk::FromStatus(3) == hipk::KernelFailure::kRejected);
  EXPECT(hipk::FromStatus(-2) == hipk::KernelFailure::kUnknown);
  // Layout arithmetic of src/kernels/ggml/mxfp8_cutlass.h:33-57.
  static_assert(hipk::ggml::mxfp8::PaddedRows(1) == 128 && hipk::ggml::mxfp8::PaddedRows(129) == 256);
  static_assert(hipk::ggml::mxfp8::SwizzledScaleBytes(12288, 4096) == 12288u * 128u);
  static_assert(hipk::ggml::PaddedK(3840) == 4096 && hipk::ggml::PaddedK(512) == 512);
  hipk::ggml::mxfp8::Gemm gemm;
  EXPECT(hipk::ggml::mxfp8::Run(gemm, 256, nullptr) > 0);  // null operands: refused, nothing queued
  hipk::exl3::LinearOperands linear;
  EXPECT(hipk::exl3::PackedLinear(linear, nullptr, 0, nullptr) == hipk::KernelFailure::kRejected);
  hipk::decode::Product product;
  EXPECT(hipk::decode::RunVector(product, nullptr) == hipk::KernelFailure::kRejected);
  product.decoder = hipk::decode::DecoderId::kAffineSplit;
  EXPECT(hipk::decode::RunVector(product, nullptr) == hipk::KernelFailure::kRejected);
  EXPECT(hipk::decode::RunMatrix(product, hipk::decode::MatrixPath::kMma, nullptr) == hipk::KernelFailure::kRejected);
  hipk::decode::GluProduct glu_product;
  EXPECT(hipk::decode::RunVectorGlu(glu_product, nullptr) == hipk::KernelFailure::kRejected);
  hipk::decode::RowsGather gather;
  EXPECT(hipk::decode::RunRows(gather, nullptr) == hipk::KernelFailure::kRejected);
  hipk::decode::GroupedProduct grouped;
  EXPECT(hipk::decode::RunGrouped(grouped, nullptr) == hipk::KernelFailure::kRejected);
  // The KV cache stores: refusals without a GPU.
  hipk::ggml::kv::Store store{};
  EXPECT(hipk::ggml::kv::SetRowsQuant(store, nullptr) == hipk::KernelFailure::kRejected);
  hipk::ggml::kv::Store pair[2] = {store, store};
  EXPECT(hipk::ggml::kv::SetRowsQuantGroup(pair, 1, nullptr) == hipk::KernelFailure::kRejected);
  EXPECT(hipk::ggml::kv::SetRowsQuantGroup(pair, 2, nullptr) == hipk::KernelFailure::kRejected);
  hipk::ggml::kv::RopeStore rope{};
  EXPECT(hipk::ggml::kv::RopeSetRowsQuant(rope, nullptr) == hipk::KernelFailure::kRejected);
  EXPECT(!hipk::LastError().empty());
  hipk::exl3::MultiLinearOperands multi;
  EXPECT(hipk::exl3::MultiLinear(multi, nullptr, 0, nullptr) == hipk::KernelFailure::kRejected);
  EXPECT(hipk::exl3::ScratchBytes(multi) == 0);
}

// The registry's entries (include/llmp_hip.hpp, namespace execution) against the names the reference's planner and
// plans use and against what the entry points they list really take: a declared row limit is the entry point's own.
void RegistryChecks() {
  namespace ex = hipk::execution;
  const std::vector<ex::Implementation> all = ex::Implementations();
  std::set<std::string> names;
  for (const ex::Implementation& i : all) {
    EXPECT(names.insert(i.name).second);  // unique in a build (registry.h:323-325)
    bool well_formed = !i.name.empty();
    for (const char c : i.name) well_formed = well_formed && ((c >= 'a' && c <= 'z') || (c >= '0' && c <= '9') || c == '.' || c == '_');
    EXPECT(well_formed);
    EXPECT(!i.capability.op.empty() && !i.capability.launches.empty() && !i.variant.empty());
    EXPECT(i.capability.min_arch == ex::kGfx950 && i.capability.max_arch == ex::kGfx950);
    EXPECT(i.capability.shape.min_rows >= 1 && i.capability.shape.min_rows <= i.capability.shape.max_rows);
    for (const std::string& launch : i.capability.launches) EXPECT(launch.rfind("llmp_hip_", 0) == 0);
  }
  // The reference's names that a binding must keep (plan_step.h:201-314, capabilities.cc:2486-2489 and 2881-2893,
  // decode/implementations.h:7-13, exl3/implementations.h:8-31).
  for (const char* name : {"llmp.q8_1", "llmp.vecq.dense", "llmp.vecq.glu", "llmp.vecq.experts", "llmp.vecq.experts_glu", "llmp.vecq.grouped",
                           "ggml.mul_mat.mmvq", "ggml.mul_mat_glu.mmvq_fused", "llmp.mul_mat.mmvq_rows", "llmp.mul_mat_id.mmvq_rows", "llmp.mxfp8.mul_mat_vec", "llmp.mxfp8.quantize",
                           "llmp.mxfp8.swizzle", "llmp.mxfp8.gemm.cutlass", "llmp.moe.router", "llmp.moe.experts.cutlass", "llmp.decode.vector.nvfp4.atoms",
                           "llmp.decode.vector_glu.mxfp8.split", "llmp.decode.matrix.bf16.dense", "llmp.decode.grouped.affine.split",
                           "llmp.decode.rows.q8_0.blocks", "exl3.linear.gemv", "exl3.linear.gemm", "exl3.multi_linear.mgemm"})
    EXPECT(names.count(name) == 1);
  int decode = 0;
  for (const std::string& name : names) decode += name.rfind("llmp.decode.", 0) == 0;
  EXPECT(decode == 5 * 12);  // every built template over every decoder; matrix_fma is refused and not declared

  // Candidates: the config shapes find their implementations, and nothing outside a rule does.
  ex::CapabilityQuery q;
  q.op = "fused.mul_mat_glu", q.encoding = "q4_k", q.rows = 1, q.k = 3840, q.n = 15360, q.row_invariant = q.capturable = true;
  // A row-invariant plan (docs/decisions.md D-092 of the reference) takes the product whose every row is its one-row
  // launch bit for bit, not the default whose form follows the row count.
  std::vector<ex::Implementation> found = ex::Candidates(q);
  EXPECT(found.size() == 1 && found[0].name == "llmp.mul_mat_glu.mmvq_rows");
  q.row_invariant = false;
  found = ex::Candidates(q);
  EXPECT(found.size() == 3 && found[0].name == "llmp.vecq.glu" && found[1].name == "llmp.mul_mat_glu.mmvq_rows" &&
         found[2].name == "ggml.mul_mat_glu.mmvq_fused");
  q.rows = 17;
  EXPECT(ex::Candidates(q).empty());
  q.rows = 1, q.k = 3840 + 32;
  EXPECT(ex::Candidates(q).empty());
  q = ex::CapabilityQuery{};
  q.op = "mul_mat", q.encoding = "mxfp8", q.rows = 2048, q.k = 4096, q.n = 12288;
  found = ex::Candidates(q);
  bool gemm = false;
  for (const ex::Implementation& i : found) gemm = gemm || i.name == "llmp.mxfp8.gemm.cutlass";
  EXPECT(gemm);
  q.features = ex::kBf16Mma;  // a device without block-scaled FP8 matrix instructions
  for (const ex::Implementation& i : ex::Candidates(q)) EXPECT(i.name != "llmp.mxfp8.gemm.cutlass");
  q = ex::CapabilityQuery{};
  q.op = "quant_linear", q.encoding = "exl3", q.rows = 16, q.k = 4096, q.n = 14336;
  found = ex::Candidates(q);
  EXPECT(found.size() == 1 && found[0].name == "exl3.linear.gemm");
  q.rows = 2048;  // the packed path still computes it; the reconstruction paths are candidates from their rows on
  found = ex::Candidates(q);
  EXPECT(found.size() == 3);
  q.arch = 942;
  EXPECT(ex::Candidates(q).empty());

  // The declared row limits are the entry points' own: one row past a limit is refused by the C ABI.
  const auto rule = [&](const char* name) {
    for (const ex::Implementation& i : all)
      if (i.name == name) return i.capability.shape;
    ++g_failures;
    return ex::ShapeRule{};
  };
  alignas(16) static std::uint8_t fake[4096];
  VecQDesc d;
  d.w = fake, d.y = fake, d.dst = reinterpret_cast<float*>(fake), d.ncols_x = 256, d.nrows = 1, d.stride_row = 1, d.y_token = 16;
  d.tokens = static_cast<int>(rule("llmp.vecq.dense").max_rows) + 1, d.dst_token = 1;
  EXPECT(!hipk::ggml::LaunchVecQ(hipk::ggml::kQ4_K, d, -1, nullptr));
  EXPECT(hipk::LastError().find("tokens") != std::string::npos);
  const std::int32_t ids[1] = {0};
  d.ids = ids, d.tokens = 1, d.used = static_cast<int>(rule("llmp.vecq.experts").max_rows) + 1;
  EXPECT(!hipk::ggml::LaunchVecQ(hipk::ggml::kQ4_K, d, -1, nullptr));
  EXPECT(hipk::LastError().find("pairs") != std::string::npos || hipk::LastError().find("slots") != std::string::npos);
  hipk::exl3::LinearOperands linear;
  const std::uint64_t at = reinterpret_cast<std::uint64_t>(fake);
  linear.weights.trellis = at, linear.weights.suh = at, linear.weights.svh = at;
  linear.weights.k = 128, linear.weights.n = 128, linear.weights.bits = 4;
  linear.x = at, linear.a_had = at, linear.y = at;
  linear.m = static_cast<int>(rule("exl3.linear.gemm").max_rows) + 1;
  EXPECT(hipk::exl3::PackedLinear(linear, fake, sizeof(fake), nullptr) == hipk::KernelFailure::kRejected);
  EXPECT(hipk::LastError().find("rows") != std::string::npos);
  EXPECT(rule("llmp.mxfp8.gemm.cutlass").k_multiple == 128);
  hipk::ggml::moe::GroupedGemm grouped_gemm;
  grouped_gemm.groups = 2, grouped_gemm.n = 64, grouped_gemm.k = static_cast<int>(rule("llmp.moe.experts.cutlass").k_multiple) + 32;
  EXPECT(hipk::ggml::moe::GroupedGemmAvailable() && hipk::ggml::moe::GroupedGemmScratch(2, 256) == 0);
  EXPECT(hipk::ggml::moe::RunGroupedGemm(grouped_gemm, 256, nullptr) > 0);
  EXPECT(hipk::LastError().find("64-value") != std::string::npos);
  static_assert(hipk::ggml::moe::SfOffset(129, 5, 8) == ((1 * 2 + 1) * 512 + 1 * 16 + 0 * 4 + 1), "moe_cutlass.h:42-46");
  hipk::ggml::mxfp8::Gemm g;
  g.m = 128, g.n = 128, g.k = 128 + 32, g.a = g.a_scales = g.b = g.b_scales = fake, g.d = fake;
  EXPECT(hipk::ggml::mxfp8::Run(g, 256, nullptr) > 0);
  // The descriptor's layout is the reference's (mxfp8_cutlass.h:59-71): `bool bf16` over the C struct's one byte.
  static_assert(sizeof(hipk::ggml::mxfp8::Gemm) == sizeof(llmp_mxfp8_gemm), "Gemm's size");
  static_assert(offsetof(hipk::ggml::mxfp8::Gemm, bf16) == offsetof(llmp_mxfp8_gemm, bf16), "bf16's place");
  static_assert(offsetof(hipk::ggml::mxfp8::Gemm, scratch) == offsetof(llmp_mxfp8_gemm, scratch), "scratch's place");
  static_assert(sizeof(bool) == sizeof(static_cast<llmp_mxfp8_gemm*>(nullptr)->bf16), "one byte");
}

// One dense product on the GPU against the oracle over the same Q8_1 bytes.
void DenseProduct(int type, int n, int k, int tokens, bool glu) {
  const int elements = orc_block_elements(type);
  const std::vector<std::uint8_t> up = Weights(type, n, k, 11 + n), gate = Weights(type, n, k, 12 + n);
  Rng rng{static_cast<std::uint64_t>(13 + k)};
  std::vector<float> x(static_cast<std::size_t>(tokens) * k);
  for (float& v : x) v = rng.Normal();
  const std::int64_t padded_k = hipk::ggml::PaddedK(k);
  std::vector<std::uint8_t> q8(static_cast<std::size_t>(tokens) * (padded_k / 32) * 36);
  for (int t = 0; t < tokens; ++t)
    orc_q8_1_quantize_row(&x[static_cast<std::size_t>(t) * k], k, padded_k, &q8[static_cast<std::size_t>(t) * (padded_k / 32) * 36],
                          ORC_Q8_DEVICE);

  // The quantizer first: its blocks are the oracle's bytes.
  float* x_device = ToDevice(x);
  std::uint8_t* q8_device = nullptr;
  EXPECT(hipMalloc(reinterpret_cast<void**>(&q8_device), q8.size()) == hipSuccess);
  EXPECT(hipk::ggml::QuantizeQ8(x_device, q8_device, k, padded_k, tokens, nullptr) == hipk::KernelFailure::kNone);
  std::vector<std::uint8_t> q8_got(q8.size());
  EXPECT(hipMemcpy(q8_got.data(), q8_device, q8.size(), hipMemcpyDeviceToHost) == hipSuccess);
  EXPECT(q8_got == q8);

  std::uint8_t* up_device = ToDevice(up);
  std::uint8_t* gate_device = ToDevice(gate);
  float* dst_device = nullptr;
  EXPECT(hipMalloc(reinterpret_cast<void**>(&dst_device), static_cast<std::size_t>(tokens) * n * 4) == hipSuccess);
  VecQDesc d;
  d.w = up_device, d.g = glu ? gate_device : nullptr, d.y = q8_device, d.dst = dst_device;
  d.ncols_x = k, d.nrows = n, d.stride_row = k / elements;
  d.y_token = static_cast<int>(padded_k / 32), d.tokens = tokens, d.dst_token = n;
  d.glu = glu ? hipk::ggml::kGeGlu : hipk::ggml::kNone;
  EXPECT(hipk::ggml::LaunchVecQ(type, d, -1, nullptr));
  std::vector<float> got(static_cast<std::size_t>(tokens) * n), want(got.size());
  EXPECT(hipDeviceSynchronize() == hipSuccess);
  EXPECT(hipMemcpy(got.data(), dst_device, got.size() * 4, hipMemcpyDeviceToHost) == hipSuccess);

  orc_vecq_desc o{};
  o.w = up.data(), o.g = glu ? gate.data() : nullptr, o.y = q8.data(), o.dst = want.data();
  o.ncols_x = k, o.nrows = n, o.stride_row = d.stride_row, o.y_token = d.y_token;
  o.used = 1, o.tokens = tokens, o.dst_token = n, o.glu = glu ? ORC_GLU_GEGLU : ORC_GLU_NONE;
  EXPECT(orc_vecq(type, &o, 0, 4) == 0);
  const double worst = WorstRelative(got, want);
  std::printf("type %d %d x %d, %d tokens%s: worst relative error %.2e\n", type, n, k, tokens, glu ? ", GeGLU" : "", worst);
  EXPECT(worst <= 1e-3);  // the tolerance of the path: accumulation order only
  (void)hipFree(x_device), (void)hipFree(q8_device), (void)hipFree(up_device), (void)hipFree(gate_device), (void)hipFree(dst_device);
}

}  // namespace

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "host";
  HostChecks();
  RegistryChecks();
  if (mode == "device") {
    DenseProduct(hipk::ggml::kQ8_0, 96, 4096, 1, false);
    DenseProduct(hipk::ggml::kQ4_K, 100, 3840, 1, true);
    DenseProduct(hipk::ggml::kQ4_K, 64, 2048, 8, true);
    DenseProduct(hipk::ggml::kQ8_0, 40, 1024, 5, false);
    DenseProduct(hipk::ggml::kQ4_K, 33, 15360, 1, false);
  }
  std::printf("%s checks: %d failure(s)\n", mode.c_str(), g_failures);
  return g_failures == 0 ? 0 : 1;
}
