// The HIP device-memory provider in the reference's own C++ vocabulary (src/providers/device_memory.h:118-192 of the
// reference: DeviceMemory and VmmProvider's reads), over the C ABI of llmp_hip_memory.h. Header only, C++17 (the
// reference's std::expected becomes Expected of llmp_hip_launch.hpp), no HIP types: addresses are the device's
// virtual addresses as 64-bit numbers.
#ifndef LLMP_HIP_MEMORY_HPP_
#define LLMP_HIP_MEMORY_HPP_

#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <vector>

#include "llmp_hip_launch.hpp"
#include "llmp_hip_memory.h"

namespace llmp_amd {
namespace providers {

enum class BackingKind : std::uint8_t { kDevice, kHost };
struct AllocationClass {
  BackingKind kind = BackingKind::kDevice;
  std::uint32_t location = 0;  // the device ordinal, or the host NUMA node
  std::uint64_t granularity = 0;
};
enum class Access : std::uint8_t { kNone, kRead, kReadWrite };
using ReservationId = std::uint64_t;  // never handed out twice; 0 is none
using BackingId = std::uint64_t;
struct AddressRange {
  std::uint64_t base = 0;
  std::uint64_t size = 0;
};

// DeviceMemory for one HIP device (device_memory.h:118-157), with VmmProvider's reads (:175-192).
class HipDeviceMemory {
 public:
  // OpenDeviceMemory (src/providers/cuda/cuda_device_memory.cc:168-213).
  static Result<std::unique_ptr<HipDeviceMemory>> Open(int device) {
    llmp_hip_memory* made = nullptr;
    if (const int status = llmp_hip_memory_open(device, &made); status != 0) return Fail<std::unique_ptr<HipDeviceMemory>>(status);
    return std::unique_ptr<HipDeviceMemory>(new HipDeviceMemory(made));
  }
  HipDeviceMemory(const HipDeviceMemory&) = delete;
  HipDeviceMemory& operator=(const HipDeviceMemory&) = delete;
  // What is still the provider's when it goes is leaked, never freed under someone's feet.
  ~HipDeviceMemory() { (void)llmp_hip_memory_close(handle_); }

  std::vector<AllocationClass> Classes() const {
    std::vector<llmp_hip_allocation_class> raw(static_cast<std::size_t>(llmp_hip_memory_classes(handle_, nullptr, 0)));
    (void)llmp_hip_memory_classes(handle_, raw.data(), static_cast<int>(raw.size()));
    std::vector<AllocationClass> classes;
    for (const llmp_hip_allocation_class& c : raw)
      classes.push_back(AllocationClass{c.kind == LLMP_BACKING_HOST ? BackingKind::kHost : BackingKind::kDevice, c.location, c.granularity});
    return classes;
  }
  std::uint64_t Granularity() const { return llmp_hip_memory_granularity(handle_); }
  std::uint64_t ReservationAlignment() const { return llmp_hip_memory_reservation_alignment(handle_); }

  Result<ReservationId> Reserve(std::uint64_t size) {
    ReservationId reservation = 0;
    if (const int status = llmp_hip_memory_reserve(handle_, size, &reservation); status != 0) return Fail<ReservationId>(status);
    return reservation;
  }
  Result<AddressRange> RangeOf(ReservationId reservation) const {
    AddressRange range;
    if (const int status = llmp_hip_memory_range_of(handle_, reservation, &range.base, &range.size); status != 0) return Fail<AddressRange>(status);
    return range;
  }
  Result<Done> Free(ReservationId reservation) { return Void(llmp_hip_memory_free(handle_, reservation)); }
  Result<BackingId> Create(std::size_t allocation_class, std::uint64_t size) {
    BackingId backing = 0;
    if (const int status = llmp_hip_memory_create(handle_, allocation_class, size, &backing); status != 0) return Fail<BackingId>(status);
    return backing;
  }
  Result<Done> Release(BackingId backing) { return Void(llmp_hip_memory_release(handle_, backing)); }
  Result<Done> Map(ReservationId reservation, std::uint64_t offset, BackingId backing) {
    return Void(llmp_hip_memory_map(handle_, reservation, offset, backing));
  }
  Result<Done> SetAccess(ReservationId reservation, std::uint64_t offset, std::uint64_t size, Access access) {
    const int wanted = access == Access::kNone ? LLMP_ACCESS_NONE : access == Access::kRead ? LLMP_ACCESS_READ : LLMP_ACCESS_READ_WRITE;
    return Void(llmp_hip_memory_set_access(handle_, reservation, offset, size, wanted));
  }
  Result<Done> Unmap(ReservationId reservation, std::uint64_t offset, std::uint64_t size) {
    return Void(llmp_hip_memory_unmap(handle_, reservation, offset, size));
  }
  std::optional<BackingId> MappedAt(ReservationId reservation, std::uint64_t offset) const {
    const BackingId backing = llmp_hip_memory_mapped_at(handle_, reservation, offset);
    return backing != 0 ? std::optional<BackingId>(backing) : std::nullopt;
  }

  bool UndeterminedReservation(ReservationId reservation) const { return llmp_hip_memory_undetermined_reservation(handle_, reservation) != 0; }
  bool UndeterminedBacking(BackingId backing) const { return llmp_hip_memory_undetermined_backing(handle_, backing) != 0; }
  std::uint64_t UndeterminedBytes() const { return llmp_hip_memory_undetermined_bytes(handle_); }
  std::size_t reservations() const { return llmp_hip_memory_reservations(handle_); }
  std::size_t backings() const { return llmp_hip_memory_backings(handle_); }
  std::uint64_t created_backings() const { return llmp_hip_memory_created_backings(handle_); }
  std::uint64_t released_backings() const { return llmp_hip_memory_released_backings(handle_); }
  llmp_hip_memory* abi() const { return handle_; }

 private:
  explicit HipDeviceMemory(llmp_hip_memory* handle) : handle_(handle) {}
  template <typename T>
  static Result<T> Fail(int status) {
    return Result<T>(FromProviderStatus(status), llmp_hip_last_error());
  }
  static Result<Done> Void(int status) { return status == 0 ? Result<Done>(Done{}) : Fail<Done>(status); }
  llmp_hip_memory* handle_;
};

}  // namespace providers
}  // namespace llmp_amd

#endif  // LLMP_HIP_MEMORY_HPP_
