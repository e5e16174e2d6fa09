// The device-memory provider (include/llmp_hip_memory.h, .hpp), as the reference's tests drive its
// (tests/unit/device_memory_test.cc of the reference is the model: the shared rules over a provider whose primitives
// can be told to fail, then the real device).
//   memory_test rules    the books of llmp_amd/csrc/vmm_ledger.h on the CPU, over a backend that counts, fails and loses
//                        outcomes on request (no GPU, no HIP call)
//   memory_test host     what the C ABI refuses without a device
//   memory_test device   reservations, backing, mappings and access on the GPU: bytes written through one mapping read
//                        back through another mapping of the same backing
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstring>
#include <set>
#include <string>
#include <vector>

#include "../../llmp_amd/csrc/vmm_ledger.h"
#include "llmp_hip_memory.hpp"

namespace {

int failures = 0;
#define CHECK(cond)                                                         \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
      ++failures;                                                           \
    }                                                                       \
  } while (0)

using llmp_hip::vmm::Access;
using llmp_hip::vmm::AllocationClass;
using llmp_hip::vmm::Error;
using llmp_hip::vmm::Kind;
using llmp_hip::vmm::Status;

// A backend that keeps books of its own: address space handed out upwards from 1 << 40, handles counted up, every live
// range, handle and mapping remembered, so that a rule that let a wrong call through shows. `fail_next` makes the next
// call fail with that error once. The ledger under test sits on top of it and is reached through `->`.
class Counting final : public llmp_hip::vmm::Backend {
 public:
  static constexpr std::uint64_t kGranule = 1 << 16;
  Counting() : ledger_(this, {AllocationClass{Kind::kDevice, 0, kGranule / 2}, AllocationClass{Kind::kHost, 1, kGranule}}, kGranule) {}
  Error fail_next = Error::kOk;
  std::set<std::uint64_t> ranges, handles;
  std::vector<std::string> calls;  // what reached the backend
  std::set<std::uint64_t> mapped;  // addresses of live mappings

  // The ledger's operations under the names the checks below use.
  Status Reserve(std::uint64_t size, std::uint64_t* id) { return ledger_.Reserve(size, id); }
  Status RangeOf(std::uint64_t id, std::uint64_t* base, std::uint64_t* size) const { return ledger_.RangeOf(id, base, size); }
  Status Free(std::uint64_t id) { return ledger_.Free(id); }
  Status Create(std::size_t c, std::uint64_t size, std::uint64_t* id) { return ledger_.Create(c, size, id); }
  Status Release(std::uint64_t id) { return ledger_.Release(id); }
  Status Map(std::uint64_t r, std::uint64_t offset, std::uint64_t b) { return ledger_.Map(r, offset, b); }
  Status SetAccess(std::uint64_t r, std::uint64_t offset, std::uint64_t size, Access a) { return ledger_.SetAccess(r, offset, size, a); }
  Status Unmap(std::uint64_t r, std::uint64_t offset, std::uint64_t size) { return ledger_.Unmap(r, offset, size); }
  std::uint64_t MappedAt(std::uint64_t r, std::uint64_t offset) const { return ledger_.MappedAt(r, offset); }
  bool UndeterminedReservation(std::uint64_t id) const { return ledger_.UndeterminedReservation(id); }
  bool UndeterminedBacking(std::uint64_t id) const { return ledger_.UndeterminedBacking(id); }
  std::uint64_t UndeterminedBytes() const { return ledger_.UndeterminedBytes(); }
  std::size_t reservations() const { return ledger_.reservations(); }
  std::size_t backings() const { return ledger_.backings(); }
  std::uint64_t created_backings() const { return ledger_.created_backings(); }
  std::uint64_t released_backings() const { return ledger_.released_backings(); }

  Status ReserveSpace(std::uint64_t size, std::uint64_t* base) override {
    if (Status s = Take("reserve"); !s) return s;
    *base = next_;
    next_ += size + kGranule;
    ranges.insert(*base);
    return llmp_hip::vmm::Ok();
  }
  Status FreeSpace(std::uint64_t base, std::uint64_t) override {
    if (Status s = Take("free"); !s) return s;
    CHECK(ranges.erase(base) == 1);
    return llmp_hip::vmm::Ok();
  }
  Status CreateBlock(const AllocationClass&, std::uint64_t, std::uint64_t* handle) override {
    if (Status s = Take("create"); !s) return s;
    *handle = ++last_handle_;
    handles.insert(*handle);
    return llmp_hip::vmm::Ok();
  }
  Status ReleaseBlock(std::uint64_t handle) override {
    if (Status s = Take("release"); !s) return s;
    CHECK(handles.erase(handle) == 1);
    return llmp_hip::vmm::Ok();
  }
  Status Attach(std::uint64_t address, std::uint64_t, std::uint64_t handle) override {
    if (Status s = Take("map"); !s) return s;
    CHECK(handles.count(handle) == 1);
    CHECK(mapped.insert(address).second);
    return llmp_hip::vmm::Ok();
  }
  Status Protect(std::uint64_t, std::uint64_t, Access, bool host) override { return Take(host ? "access host" : "access device"); }
  Status Detach(std::uint64_t address, std::uint64_t size) override {
    if (Status s = Take("unmap"); !s) return s;
    for (auto at = mapped.lower_bound(address); at != mapped.end() && *at < address + size;) at = mapped.erase(at);
    return llmp_hip::vmm::Ok();
  }

 private:
  Status Take(const char* what) {
    calls.push_back(what);
    if (fail_next == Error::kOk) return llmp_hip::vmm::Ok();
    const Error e = fail_next;
    fail_next = Error::kOk;
    return Status{e, std::string(what) + " was told to fail", e == Error::kUnknown ? 999 : 0};
  }
  std::uint64_t next_ = std::uint64_t{1} << 40;
  std::uint64_t last_handle_ = 0;
  llmp_hip::vmm::Ledger ledger_;
};

void RulesChecks() {
  constexpr std::uint64_t G = Counting::kGranule;
  Counting m;
  std::uint64_t r = 0, b0 = 0, b1 = 0, b2 = 0, base = 0, size = 0;
  // Sizes: non-zero multiples of the granularity, of the class's and of the provider's.
  CHECK(m.Reserve(0, &r).error == Error::kInvalid);
  CHECK(m.Reserve(G + 1, &r).error == Error::kInvalid);
  CHECK(m.calls.empty());  // nothing reached a primitive
  CHECK(m.Reserve(8 * G, &r));
  CHECK(m.RangeOf(r, &base, &size) && size == 8 * G && base % G == 0);
  CHECK(m.Create(2, G, &b0).error == Error::kInvalid);      // no such class
  CHECK(m.Create(0, G / 2, &b0).error == Error::kInvalid);  // the class's granularity, not the provider's
  CHECK(m.Create(0, 0, &b0).error == Error::kInvalid);
  CHECK(m.Create(0, 2 * G, &b0) && m.Create(0, G, &b1) && m.Create(1, G, &b2));
  CHECK(m.backings() == 3 && m.created_backings() == 3 && m.reservations() == 1);
  // Mapping: whole, aligned, inside, into a hole, once.
  CHECK(m.Map(r, G / 2, b0).error == Error::kInvalid);
  CHECK(m.Map(r, 7 * G, b0).error == Error::kInvalid);  // runs past the end
  CHECK(m.Map(r, 2 * G, b0));
  CHECK(m.Map(r, 4 * G, b0).error == Error::kInvalid);  // already mapped
  CHECK(m.Map(r, 3 * G, b1).error == Error::kInvalid);  // overlaps b0's second granule
  CHECK(m.Map(r, G, b1));                               // the hole just before
  CHECK(m.Map(r, 4 * G, b2));                           // ... and just after
  CHECK(m.MappedAt(r, 2 * G) == b0 && m.MappedAt(r, 3 * G) == 0 && m.MappedAt(r, G) == b1 && m.MappedAt(r + 1, G) == 0);
  // Access and unmapping cover whole mappings exactly; one primitive call a run of one kind.
  m.calls.clear();
  CHECK(m.SetAccess(r, 2 * G, G, Access::kRead).error == Error::kInvalid);       // splits b0
  CHECK(m.SetAccess(r, 0, 2 * G, Access::kRead).error == Error::kInvalid);       // starts in a hole
  CHECK(m.SetAccess(r, G, 5 * G, Access::kRead).error == Error::kInvalid);       // ends in a hole
  CHECK(m.SetAccess(r, 6 * G, 4 * G, Access::kRead).error == Error::kInvalid);   // outside
  CHECK(m.calls.empty());
  CHECK(m.SetAccess(r, G, 4 * G, Access::kReadWrite));
  CHECK((m.calls == std::vector<std::string>{"access device", "access host"}));  // b1 and b0 together, then b2
  CHECK(m.Release(b0).error == Error::kInvalid && m.Free(r).error == Error::kInvalid);  // still mapped
  CHECK(m.Unmap(r, 2 * G, G).error == Error::kInvalid);
  CHECK(m.Unmap(r, G, 3 * G) && m.MappedAt(r, G) == 0 && m.MappedAt(r, 2 * G) == 0 && m.MappedAt(r, 4 * G) == b2);
  CHECK(m.Release(b0) && m.Release(b0).error == Error::kInvalid);  // a stale identity names nothing
  CHECK(m.Map(r, 0, b0).error == Error::kInvalid);
  CHECK(m.backings() == 2 && m.released_backings() == 1);
  // A known failure changes nothing and may be retried.
  m.fail_next = Error::kFailed;
  CHECK(m.Map(r, 0, b1).error == Error::kFailed && m.MappedAt(r, 0) == 0 && !m.UndeterminedBacking(b1));
  CHECK(m.Map(r, 0, b1));
  m.fail_next = Error::kOutOfMemory;
  std::uint64_t none = 7;
  CHECK(m.Create(0, G, &none).error == Error::kOutOfMemory && m.backings() == 2);
  // An unknown outcome: what it touched is undetermined, refused from then on and never retried.
  m.fail_next = Error::kUnknown;
  const Status lost = m.Unmap(r, 0, G);
  CHECK(lost.error == Error::kUnknown && lost.native == 999);
  CHECK(m.UndeterminedReservation(r) && m.UndeterminedBacking(b1) && !m.UndeterminedBacking(b2));
  CHECK(m.UndeterminedBytes() == G);
  m.calls.clear();
  CHECK(m.Unmap(r, 0, G).error == Error::kUndetermined && m.Free(r).error == Error::kUndetermined);
  CHECK(m.RangeOf(r, &base, &size).error == Error::kUndetermined && m.Release(b1).error == Error::kUndetermined);
  CHECK(m.SetAccess(r, 4 * G, G, Access::kNone).error == Error::kUndetermined && m.Map(r, 6 * G, b1).error == Error::kUndetermined);
  CHECK(m.calls.empty());
  // A create or a reserve whose outcome is unknown stays charged, with nothing to use.
  m.fail_next = Error::kUnknown;
  CHECK(m.Create(0, 3 * G, &none).error == Error::kUnknown && m.backings() == 3 && m.UndeterminedBytes() == 4 * G);
  m.fail_next = Error::kUnknown;
  CHECK(m.Reserve(G, &none).error == Error::kUnknown && m.reservations() == 2);
  // A release or a free whose outcome is unknown is not retried either.
  std::uint64_t r2 = 0, b3 = 0;
  CHECK(m.Reserve(2 * G, &r2) && m.Create(1, G, &b3));
  m.fail_next = Error::kUnknown;
  CHECK(m.Release(b3).error == Error::kUnknown && m.Release(b3).error == Error::kUndetermined);
  m.fail_next = Error::kUnknown;
  CHECK(m.Free(r2).error == Error::kUnknown && m.Free(r2).error == Error::kUndetermined);
  // Identities are never reused: a reservation made after one was freed has another name.
  std::uint64_t r3 = 0, r4 = 0;
  CHECK(m.Reserve(G, &r3) && m.Free(r3) && m.Reserve(G, &r4) && r4 != r3 && m.RangeOf(r3, &base, &size).error == Error::kInvalid);
  CHECK(m.Free(r4));
  std::printf("rules checks: %d failure(s)\n", failures);
}

using llmp_amd::providers::HipDeviceMemory;
using llmp_amd::providers::ProviderError;

void HostChecks() {
  CHECK(llmp_hip_memory_open(0, nullptr) == LLMP_PROVIDER_INVALID);
  std::uint64_t id = 0;
  CHECK(llmp_hip_memory_reserve(nullptr, 1 << 21, &id) == LLMP_PROVIDER_INVALID);
  CHECK(std::string(llmp_hip_last_error()).find("null provider") != std::string::npos);
  CHECK(llmp_hip_memory_granularity(nullptr) == 0 && llmp_hip_memory_mapped_at(nullptr, 1, 0) == 0 && llmp_hip_memory_close(nullptr) == 0);
  // No provider is opened: the device primitives are switched off in the library's default build.
  auto none = HipDeviceMemory::Open(0);
  CHECK(!none && none.error() == ProviderError::kUnsupported);
  std::printf("host checks: %d failure(s)\n", failures);
}

void DeviceChecks() {
  auto opened = HipDeviceMemory::Open(0);
  CHECK(bool(opened));
  if (!opened) {
    std::printf("device checks: %d failure(s) (%s)\n", failures, opened.detail().c_str());
    return;
  }
  HipDeviceMemory& m = **opened;
  const std::uint64_t G = m.Granularity();
  const auto classes = m.Classes();
  CHECK(classes.size() == 1 && classes[0].kind == llmp_amd::providers::BackingKind::kDevice && classes[0].granularity != 0 &&
        G % classes[0].granularity == 0 && m.ReservationAlignment() == G);
  std::printf("granularity %llu bytes\n", static_cast<unsigned long long>(G));
  CHECK(!m.Reserve(G + 4096) && !m.Create(1, G) && !m.Create(0, G / 2));
  auto r = m.Reserve(6 * G);
  auto b0 = m.Create(0, 2 * G);
  auto b1 = m.Create(0, G);
  CHECK(r && b0 && b1);
  if (!(r && b0 && b1)) {
    std::printf("device checks: %d failure(s) (%s)\n", failures, llmp_hip_last_error());
    return;
  }
  auto range = m.RangeOf(*r);
  CHECK(range && range->size == 6 * G && range->base % G == 0);
  CHECK(m.Map(*r, G, *b0) && m.Map(*r, 4 * G, *b1) && !m.Map(*r, 2 * G, *b1) && m.MappedAt(*r, G) == *b0);
  CHECK(!m.SetAccess(*r, G, G, llmp_amd::providers::Access::kReadWrite));  // splits a mapping
  CHECK(m.SetAccess(*r, G, 2 * G, llmp_amd::providers::Access::kReadWrite) && m.SetAccess(*r, 4 * G, G, llmp_amd::providers::Access::kReadWrite));
  // Bytes through the mappings: a pattern into b0 at its place, another into b1.
  std::vector<std::uint32_t> pattern(2 * G / 4), other(G / 4), back(2 * G / 4);
  for (std::size_t i = 0; i < pattern.size(); ++i) pattern[i] = static_cast<std::uint32_t>(i * 2654435761u);
  for (std::size_t i = 0; i < other.size(); ++i) other[i] = static_cast<std::uint32_t>(~i);
  void* at0 = reinterpret_cast<void*>(range->base + G);
  void* at1 = reinterpret_cast<void*>(range->base + 4 * G);
  CHECK(hipMemcpy(at0, pattern.data(), 2 * G, hipMemcpyHostToDevice) == hipSuccess);
  CHECK(hipMemcpy(at1, other.data(), G, hipMemcpyHostToDevice) == hipSuccess);
  CHECK(hipMemcpy(back.data(), at0, 2 * G, hipMemcpyDeviceToHost) == hipSuccess && back == pattern);
  // Backing outlives a mapping: unmap b0, map it elsewhere (a second reservation), and the bytes are there.
  CHECK(!m.Release(*b0) && !m.Free(*r));  // mapped
  CHECK(m.Unmap(*r, G, 2 * G) && !m.MappedAt(*r, G).has_value());
  auto r2 = m.Reserve(2 * G);
  CHECK(bool(r2));
  if (r2) {
    auto range2 = m.RangeOf(*r2);
    CHECK(m.Map(*r2, 0, *b0) && m.SetAccess(*r2, 0, 2 * G, llmp_amd::providers::Access::kReadWrite));
    std::fill(back.begin(), back.end(), 0u);
    CHECK(range2 && hipMemcpy(back.data(), reinterpret_cast<void*>(range2->base), 2 * G, hipMemcpyDeviceToHost) == hipSuccess && back == pattern);
    // The hole b0 left takes b1's sibling: a new backing of the same size, while b1 stays where it is.
    auto b2 = m.Create(0, G);
    CHECK(b2 && m.Map(*r, 2 * G, *b2) && m.SetAccess(*r, 2 * G, G, llmp_amd::providers::Access::kReadWrite));
    std::vector<std::uint32_t> small(G / 4);
    CHECK(hipMemcpy(small.data(), at1, G, hipMemcpyDeviceToHost) == hipSuccess && small == other);
    CHECK(m.Unmap(*r, 2 * G, G) && b2 && m.Release(*b2));
    CHECK(m.Unmap(*r2, 0, 2 * G) && m.Free(*r2) && !m.RangeOf(*r2));
  }
  CHECK(m.Unmap(*r, 4 * G, G) && m.Release(*b0) && m.Release(*b1) && !m.Release(*b1) && m.Free(*r));
  CHECK(m.reservations() == 0 && m.backings() == 0 && m.created_backings() == 3 && m.released_backings() == 3 && m.UndeterminedBytes() == 0);
  CHECK(hipDeviceSynchronize() == hipSuccess);
  std::printf("device checks: %d failure(s)\n", failures);
}

}  // namespace

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "rules";
  if (mode == "rules") {
    RulesChecks();
  } else if (mode == "host") {
    HostChecks();
  } else if (mode == "device") {
    DeviceChecks();
  } else {
    std::printf("usage: memory_test rules|host|device\n");
    return 2;
  }
  return failures == 0 ? 0 : 1;
}
