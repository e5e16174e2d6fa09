// The HIP device-memory provider behind include/llmp_hip_memory.h: what the reference's CudaDeviceMemory does with the
// CUDA driver (src/providers/cuda/cuda_device_memory.cc:42-144) done with HIP's virtual memory management calls, as the
// Backend of the books kept in vmm_ledger.h. Host code only.
#include <hip/hip_runtime.h>

#include <memory>
#include <numeric>
#include <string>
#include <vector>

#include "common.h"
#include "llmp_hip.h"
#include "llmp_hip_memory.h"
#include "vmm_ledger.h"

using llmp_hip::vmm::Access;
using llmp_hip::vmm::AllocationClass;
using llmp_hip::vmm::Error;
using llmp_hip::vmm::Kind;
using llmp_hip::vmm::Ledger;
using llmp_hip::vmm::Status;

namespace llmp_hip {
namespace {

// Errors the runtime reports before doing anything: the call changed nothing, and its outcome is known
// (cuda_errors.cc:17-38). Every other error leaves the outcome unknown.
bool Refused(hipError_t e) {
  switch (e) {
    case hipErrorInvalidValue:
    case hipErrorInvalidHandle:
    case hipErrorInvalidDevice:
    case hipErrorInvalidContext:
    case hipErrorNotInitialized:
    case hipErrorDeinitialized:
    case hipErrorNoDevice:
    case hipErrorNotFound:
    case hipErrorNotMapped:
    case hipErrorAlreadyMapped:
      return true;
    default:
      return false;
  }
}

Status Outcome(hipError_t e, const char* call) {
  if (e == hipSuccess) return vmm::Ok();
  (void)hipGetLastError();  // the error is this call's: not left for the next launch to find
  Error error = Error::kUnknown;
  if (e == hipErrorOutOfMemory) {
    error = Error::kOutOfMemory;
  } else if (e == hipErrorNotSupported) {
    error = Error::kUnsupported;
  } else if (Refused(e)) {
    error = Error::kFailed;
  }
  return Status{error, std::string(call) + ": " + hipGetErrorName(e) + " (" + std::to_string(static_cast<int>(e)) + ")", static_cast<int>(e)};
}

hipMemAllocationProp Properties(const AllocationClass& allocation_class) {
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = allocation_class.kind == Kind::kHost ? hipMemLocationTypeHostNuma : hipMemLocationTypeDevice;
  prop.location.id = static_cast<int>(allocation_class.location);
  return prop;
}

class HipBackend final : public vmm::Backend {
 public:
  HipBackend(int device, std::vector<AllocationClass> classes, std::uint64_t granularity)
      : device_(device), classes_(std::move(classes)), granularity_(granularity) {}

  Status ReserveSpace(std::uint64_t size, std::uint64_t* base) override {
    if (Status current = Current(); !current) return current;
    void* at = nullptr;
    if (Status reserved = Outcome(hipMemAddressReserve(&at, size, granularity_, nullptr, 0), "hipMemAddressReserve"); !reserved) return reserved;
    *base = reinterpret_cast<std::uint64_t>(at);
    return vmm::Ok();
  }
  Status FreeSpace(std::uint64_t base, std::uint64_t size) override {
    return Outcome(hipMemAddressFree(reinterpret_cast<void*>(base), size), "hipMemAddressFree");
  }
  Status CreateBlock(const AllocationClass& allocation_class, std::uint64_t size, std::uint64_t* handle) override {
    if (Status current = Current(); !current) return current;
    const hipMemAllocationProp prop = Properties(allocation_class);
    hipMemGenericAllocationHandle_t made = nullptr;
    if (Status created = Outcome(hipMemCreate(&made, size, &prop, 0), "hipMemCreate"); !created) return created;
    *handle = reinterpret_cast<std::uint64_t>(made);
    return vmm::Ok();
  }
  Status ReleaseBlock(std::uint64_t handle) override {
    return Outcome(hipMemRelease(reinterpret_cast<hipMemGenericAllocationHandle_t>(handle)), "hipMemRelease");
  }
  Status Attach(std::uint64_t address, std::uint64_t size, std::uint64_t handle) override {
    return Outcome(hipMemMap(reinterpret_cast<void*>(address), size, 0, reinterpret_cast<hipMemGenericAllocationHandle_t>(handle), 0), "hipMemMap");
  }
  Status Protect(std::uint64_t address, std::uint64_t size, Access access, bool host) override {
    hipMemAccessFlags flags = hipMemAccessFlagsProtNone;
    if (access == Access::kRead) {
      flags = hipMemAccessFlagsProtRead;
    } else if (access == Access::kReadWrite) {
      flags = hipMemAccessFlagsProtReadWrite;
    }
    // The device always; the CPU on the host node when the range holds host backing (cuda_device_memory.cc:112-123).
    std::vector<hipMemAccessDesc> descriptors;
    for (const AllocationClass& allocation_class : classes_) {
      if (allocation_class.kind == Kind::kDevice || host) {
        hipMemAccessDesc descriptor = {};
        descriptor.location = Properties(allocation_class).location;
        descriptor.flags = flags;
        descriptors.push_back(descriptor);
      }
    }
    return Outcome(hipMemSetAccess(reinterpret_cast<void*>(address), size, descriptors.data(), descriptors.size()), "hipMemSetAccess");
  }
  Status Detach(std::uint64_t address, std::uint64_t size) override {
    return Outcome(hipMemUnmap(reinterpret_cast<void*>(address), size), "hipMemUnmap");
  }

 private:
  Status Current() { return Outcome(hipSetDevice(device_), "hipSetDevice"); }
  int device_;
  std::vector<AllocationClass> classes_;
  std::uint64_t granularity_;
};

// The C ABI's return value for a status, its reason recorded for llmp_hip_last_error.
int Code(const Status& status) {
  switch (status.error) {
    case Error::kOk:
      return 0;
    case Error::kInvalid:
      return Refuse(LLMP_PROVIDER_INVALID, "%s", status.detail.c_str());
    case Error::kOutOfMemory:
      return Refuse(LLMP_PROVIDER_OUT_OF_MEMORY, "%s", status.detail.c_str());
    case Error::kUnsupported:
      return Refuse(LLMP_PROVIDER_UNSUPPORTED, "%s", status.detail.c_str());
    case Error::kFailed:
      return Refuse(LLMP_PROVIDER_FAILED, "%s", status.detail.c_str());
    case Error::kUndetermined:
      return Refuse(LLMP_PROVIDER_UNDETERMINED, "%s", status.detail.c_str());
    case Error::kUnknown:
      return Refuse(status.native > 0 ? -status.native : -static_cast<int>(hipErrorUnknown), "%s", status.detail.c_str());
  }
  return Refuse(LLMP_PROVIDER_FAILED, "%s", status.detail.c_str());
}

}  // namespace
}  // namespace llmp_hip

struct llmp_hip_memory {
  llmp_hip_memory(int device, const std::vector<AllocationClass>& classes, std::uint64_t granularity)
      : backend(device, classes, granularity), books(&backend, classes, granularity), provider(&books) {}
  llmp_hip::HipBackend backend;
  Ledger books;
  Ledger* provider;
};

using llmp_hip::Code;
using llmp_hip::Refuse;

extern "C" int llmp_hip_memory_open(int device, llmp_hip_memory** out) {
  if (out == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "memory: null result");
  *out = nullptr;
#if defined(LLMP_HIP_MEMORY_ON_DEVICE) && !defined(LLMP_HIP_MEMORY_FAULT_CAUSE_SHOWN)
#error "LLMP_HIP_MEMORY_ON_DEVICE switches on calls whose one run on an MI355X ended with the GPU faulted; define LLMP_HIP_MEMORY_FAULT_CAUSE_SHOWN as well only once that fault's cause has been shown and fixed"
#endif
#ifndef LLMP_HIP_MEMORY_ON_DEVICE
  // Switched off: the one run of these calls on an MI355X (two mappings in a reservation, access granted, host
  // copies through them) ended with the GPU faulted, before any kernel of this library ran, and the cause has not
  // been shown. Until it is, no provider is opened and no virtual memory call is made; the books of vmm_ledger.h are
  // tested on the CPU (tests/host/memory_test.cc, rules). A consumer that pages meanwhile allocates with hipMalloc and
  // copies, with no remapping.
  (void)device;
  return Refuse(LLMP_PROVIDER_UNSUPPORTED, "memory: the HIP virtual memory calls are switched off in this build");
#else
  int devices = 0;
  if (const hipError_t e = hipGetDeviceCount(&devices); e != hipSuccess || device < 0 || device >= devices) {
    (void)hipGetLastError();
    return Refuse(LLMP_PROVIDER_UNSUPPORTED, "memory: no device %d (%d visible)", device, e == hipSuccess ? devices : 0);
  }
  int vmm = 0;
  if (hipDeviceGetAttribute(&vmm, hipDeviceAttributeVirtualMemoryManagementSupported, device) != hipSuccess || vmm == 0) {
    (void)hipGetLastError();
    return Refuse(LLMP_PROVIDER_UNSUPPORTED, "memory: the device has no virtual memory management");
  }
  std::vector<AllocationClass> classes = {AllocationClass{Kind::kDevice, static_cast<std::uint32_t>(device), 0}};
  std::uint64_t common = 1;
  for (AllocationClass& allocation_class : classes) {
    const hipMemAllocationProp prop = llmp_hip::Properties(allocation_class);
    size_t granularity = 0;
    if (const Status asked = llmp_hip::Outcome(hipMemGetAllocationGranularity(&granularity, &prop, hipMemAllocationGranularityMinimum),
                                               "hipMemGetAllocationGranularity");
        !asked)
      return Code(asked);
    if (granularity == 0) return Refuse(LLMP_PROVIDER_UNSUPPORTED, "memory: a zero allocation granularity");
    allocation_class.granularity = granularity;
    common = std::lcm(common, static_cast<std::uint64_t>(granularity));
  }
  *out = new llmp_hip_memory(device, classes, common);
  return 0;
#endif
}

extern "C" int llmp_hip_memory_close(llmp_hip_memory* memory) {
  if (memory == nullptr) return 0;
  if (memory->provider->reservations() != 0 || memory->provider->backings() != 0)
    return Refuse(LLMP_PROVIDER_INVALID, "memory: %zu reservation(s) and %zu backing(s) are still the provider's",
                  memory->provider->reservations(), memory->provider->backings());
  delete memory;
  return 0;
}

extern "C" int llmp_hip_memory_classes(const llmp_hip_memory* memory, llmp_hip_allocation_class* classes, int room) {
  if (memory == nullptr) return 0;
  const std::vector<AllocationClass>& all = memory->provider->Classes();
  for (int i = 0; classes != nullptr && i < room && i < static_cast<int>(all.size()); ++i)
    classes[i] = llmp_hip_allocation_class{all[i].kind == Kind::kHost ? LLMP_BACKING_HOST : LLMP_BACKING_DEVICE, all[i].location, all[i].granularity};
  return static_cast<int>(all.size());
}

extern "C" uint64_t llmp_hip_memory_granularity(const llmp_hip_memory* memory) { return memory == nullptr ? 0 : memory->provider->Granularity(); }
extern "C" uint64_t llmp_hip_memory_reservation_alignment(const llmp_hip_memory* memory) {
  return memory == nullptr ? 0 : memory->provider->Granularity();
}

#define LLMP_MEMORY(memory)                                                           \
  if ((memory) == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "memory: null provider")

extern "C" int llmp_hip_memory_reserve(llmp_hip_memory* memory, uint64_t size, uint64_t* reservation) {
  LLMP_MEMORY(memory);
  if (reservation == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "reserve: null result");
  *reservation = 0;
  return Code(memory->provider->Reserve(size, reservation));
}
extern "C" int llmp_hip_memory_range_of(const llmp_hip_memory* memory, uint64_t reservation, uint64_t* base, uint64_t* size) {
  LLMP_MEMORY(memory);
  if (base == nullptr || size == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "range_of: null result");
  return Code(memory->provider->RangeOf(reservation, base, size));
}
extern "C" int llmp_hip_memory_free(llmp_hip_memory* memory, uint64_t reservation) {
  LLMP_MEMORY(memory);
  return Code(memory->provider->Free(reservation));
}
extern "C" int llmp_hip_memory_create(llmp_hip_memory* memory, size_t allocation_class, uint64_t size, uint64_t* backing) {
  LLMP_MEMORY(memory);
  if (backing == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "create: null result");
  *backing = 0;
  return Code(memory->provider->Create(allocation_class, size, backing));
}
extern "C" int llmp_hip_memory_release(llmp_hip_memory* memory, uint64_t backing) {
  LLMP_MEMORY(memory);
  return Code(memory->provider->Release(backing));
}
extern "C" int llmp_hip_memory_map(llmp_hip_memory* memory, uint64_t reservation, uint64_t offset, uint64_t backing) {
  LLMP_MEMORY(memory);
  return Code(memory->provider->Map(reservation, offset, backing));
}
extern "C" int llmp_hip_memory_set_access(llmp_hip_memory* memory, uint64_t reservation, uint64_t offset, uint64_t size, int access) {
  LLMP_MEMORY(memory);
  if (access != LLMP_ACCESS_NONE && access != LLMP_ACCESS_READ && access != LLMP_ACCESS_READ_WRITE)
    return Refuse(LLMP_PROVIDER_INVALID, "set_access: no such access %d", access);
  const Access wanted = access == LLMP_ACCESS_NONE ? Access::kNone : access == LLMP_ACCESS_READ ? Access::kRead : Access::kReadWrite;
  return Code(memory->provider->SetAccess(reservation, offset, size, wanted));
}
extern "C" int llmp_hip_memory_unmap(llmp_hip_memory* memory, uint64_t reservation, uint64_t offset, uint64_t size) {
  LLMP_MEMORY(memory);
  return Code(memory->provider->Unmap(reservation, offset, size));
}
extern "C" uint64_t llmp_hip_memory_mapped_at(const llmp_hip_memory* memory, uint64_t reservation, uint64_t offset) {
  return memory == nullptr ? 0 : memory->provider->MappedAt(reservation, offset);
}
extern "C" int llmp_hip_memory_undetermined_reservation(const llmp_hip_memory* memory, uint64_t reservation) {
  return memory != nullptr && memory->provider->UndeterminedReservation(reservation) ? 1 : 0;
}
extern "C" int llmp_hip_memory_undetermined_backing(const llmp_hip_memory* memory, uint64_t backing) {
  return memory != nullptr && memory->provider->UndeterminedBacking(backing) ? 1 : 0;
}
extern "C" uint64_t llmp_hip_memory_undetermined_bytes(const llmp_hip_memory* memory) {
  return memory == nullptr ? 0 : memory->provider->UndeterminedBytes();
}
extern "C" size_t llmp_hip_memory_reservations(const llmp_hip_memory* memory) { return memory == nullptr ? 0 : memory->provider->reservations(); }
extern "C" size_t llmp_hip_memory_backings(const llmp_hip_memory* memory) { return memory == nullptr ? 0 : memory->provider->backings(); }
extern "C" uint64_t llmp_hip_memory_created_backings(const llmp_hip_memory* memory) {
  return memory == nullptr ? 0 : memory->provider->created_backings();
}
extern "C" uint64_t llmp_hip_memory_released_backings(const llmp_hip_memory* memory) {
  return memory == nullptr ? 0 : memory->provider->released_backings();
}
