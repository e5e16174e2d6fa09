/*
 * C ABI of the HIP device-memory provider: explicit virtual reservations, physical backing in an
 * allocation class, and mapping with access control, as the reference's DeviceMemory gives them to
 * its paging engine (src/providers/device_memory.h:118-157) and its CUDA build implements them over
 * the driver's VMM calls (src/providers/cuda/cuda_device_memory.cc:42-215). Here the primitives are
 * hipMemAddressReserve / hipMemAddressFree, hipMemCreate / hipMemRelease, hipMemMap / hipMemUnmap and
 * hipMemSetAccess; the contract over them is the one the reference states for every implementation
 * (device_memory.h:30-45), kept by the books of llmp_amd/csrc/vmm_ledger.h:
 *   - a reservation is address space only, a non-zero multiple of the granularity;
 *   - backing is created in one allocation class, a multiple of the granularity, filled with nothing
 *     a caller may rely on;
 *   - a backing is mapped whole, at a granularity-aligned offset inside one reservation, into a hole,
 *     at most once at a time; a mapping starts with no access, until set_access grants it;
 *   - set_access and unmap take ranges that cover whole mappings exactly;
 *   - backing is released only when unmapped, a reservation freed only when nothing is mapped in it.
 * Nothing here pages on demand: touching address space whose backing is absent is a bug.
 *
 * Identities are 64-bit numbers from one counter, never handed out twice: a stale one names nothing,
 * and a reservation's never names a backing. 0 is no identity.
 *
 * Return values, as in llmp_hip_launch.h: 0 done; > 0 refused or failed with nothing changed, one
 * of LLMP_PROVIDER_* (the reference's ProviderError, device_memory.h:84-95); < 0 a primitive's
 * outcome is unknown, -(hipError_t) (ProviderError::kUnknown): the reservation and the backing it
 * touched are undetermined from then on, every later call on them returns LLMP_PROVIDER_UNDETERMINED
 * and is never retried, and their owner quarantines them. Which runtime errors are known refusals
 * follows src/providers/cuda/cuda_errors.cc:17-55: invalid value, handle, device or context, not
 * initialised, not mapped, already mapped and their like changed nothing (LLMP_PROVIDER_FAILED), out
 * of memory and not supported have codes of their own, everything else is unknown.
 * llmp_hip_last_error() (llmp_hip.h) names the reason of the calling thread's last non-zero return.
 *
 * One thread calls a provider at a time (device_memory.h:16-29): a second call that changes it
 * while one is under way aborts the process.
 */
#ifndef LLMP_HIP_MEMORY_H_
#define LLMP_HIP_MEMORY_H_

#include <stddef.h>
#include <stdint.h>

#include "llmp_hip_launch.h" /* LLMP_PROVIDER_* */

#ifdef __cplusplus
extern "C" {
#endif

typedef struct llmp_hip_memory llmp_hip_memory;

/* BackingKind and AllocationClass (device_memory.h:68-77). */
enum { LLMP_BACKING_DEVICE = 0, LLMP_BACKING_HOST = 1 };
typedef struct llmp_hip_allocation_class {
  int32_t kind;         /* LLMP_BACKING_* */
  uint32_t location;    /* the device ordinal, or the host NUMA node */
  uint64_t granularity; /* backing and offsets are multiples of it */
} llmp_hip_allocation_class;
/* Access (device_memory.h:79). */
enum { LLMP_ACCESS_NONE = 0, LLMP_ACCESS_READ = 1, LLMP_ACCESS_READ_WRITE = 2 };

/* OpenDeviceMemory (cuda_device_memory.cc:168-213): the provider of one device, LLMP_PROVIDER_UNSUPPORTED
 * where the device has no virtual memory management. One class: device-local memory. (The reference adds
 * a host class where the driver reports host-NUMA backing as mappable; HIP has no such report, and the
 * class is not offered.) In the default build this returns LLMP_PROVIDER_UNSUPPORTED for every device: the
 * primitives are compiled but switched off (llmp_amd/csrc/memory.hip says why). */
int llmp_hip_memory_open(int device, llmp_hip_memory** out);
/* Refused (LLMP_PROVIDER_INVALID) while a reservation or a backing is live. */
int llmp_hip_memory_close(llmp_hip_memory* memory);
/* Classes (:130): writes up to `room` classes, returns how many there are. */
int llmp_hip_memory_classes(const llmp_hip_memory* memory, llmp_hip_allocation_class* classes, int room);
/* Granularity and ReservationAlignment (:133-138): the granularity of reservations and offsets, a multiple
 * of every class's; every reservation's base is aligned to it. */
uint64_t llmp_hip_memory_granularity(const llmp_hip_memory* memory);
uint64_t llmp_hip_memory_reservation_alignment(const llmp_hip_memory* memory);

/* Reserve / RangeOf / Free (:140-142). */
int llmp_hip_memory_reserve(llmp_hip_memory* memory, uint64_t size, uint64_t* reservation);
int llmp_hip_memory_range_of(const llmp_hip_memory* memory, uint64_t reservation, uint64_t* base, uint64_t* size);
int llmp_hip_memory_free(llmp_hip_memory* memory, uint64_t reservation);
/* Create / Release (:144-145). */
int llmp_hip_memory_create(llmp_hip_memory* memory, size_t allocation_class, uint64_t size, uint64_t* backing);
int llmp_hip_memory_release(llmp_hip_memory* memory, uint64_t backing);
/* Map / SetAccess / Unmap (:147-155). */
int llmp_hip_memory_map(llmp_hip_memory* memory, uint64_t reservation, uint64_t offset, uint64_t backing);
int llmp_hip_memory_set_access(llmp_hip_memory* memory, uint64_t reservation, uint64_t offset, uint64_t size, int access);
int llmp_hip_memory_unmap(llmp_hip_memory* memory, uint64_t reservation, uint64_t offset, uint64_t size);
/* MappedAt (:159): the backing mapped at exactly `offset` of the reservation, or 0. */
uint64_t llmp_hip_memory_mapped_at(const llmp_hip_memory* memory, uint64_t reservation, uint64_t offset);

/* VmmProvider's reads (:175-192): whether an unknown outcome left it undetermined, the backing bytes that
 * are (their owner keeps them charged), and what is live. */
int llmp_hip_memory_undetermined_reservation(const llmp_hip_memory* memory, uint64_t reservation);
int llmp_hip_memory_undetermined_backing(const llmp_hip_memory* memory, uint64_t backing);
uint64_t llmp_hip_memory_undetermined_bytes(const llmp_hip_memory* memory);
size_t llmp_hip_memory_reservations(const llmp_hip_memory* memory);
size_t llmp_hip_memory_backings(const llmp_hip_memory* memory);
uint64_t llmp_hip_memory_created_backings(const llmp_hip_memory* memory);
uint64_t llmp_hip_memory_released_backings(const llmp_hip_memory* memory);

#ifdef __cplusplus
}
#endif

#endif /* LLMP_HIP_MEMORY_H_ */
