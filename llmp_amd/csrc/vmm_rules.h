// The rules of the device-memory provider over an implementation's primitive operations, as the reference's
// VmmProvider holds them for every implementation (src/providers/device_memory.h:160-262,
// src/providers/device_memory.cc:55-400):
//   - a reservation is address space only, a non-zero multiple of the granularity;
//   - backing is created in one allocation class, a non-zero multiple of that class's granularity and of the
//     provider's;
//   - a backing is mapped whole, at a granularity-aligned offset inside one reservation, into a hole, at most once
//     at a time;
//   - access is set, and mappings are removed, over ranges that cover whole mappings exactly;
//   - backing is released only when unmapped, a reservation freed only when nothing is mapped in it;
//   - identities are generation-checked: a stale one names nothing;
//   - a primitive whose outcome is unknown leaves the reservation and backing it touched undetermined: every later
//     call on them is refused (kUndetermined) and never retried (a retried release or free could hit a handle or a
//     range the driver has since handed to someone else).
// Plain C++ with no device types: the HIP primitives are in memory.hip, and tests/host/memory_rules_test.cc drives
// these rules on the CPU over primitives that count, fail and lose outcomes on request.
#ifndef LLMP_AMD_CSRC_VMM_RULES_H_
#define LLMP_AMD_CSRC_VMM_RULES_H_

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstdio>
#include <map>
#include <string>
#include <vector>

namespace llmp_hip {
namespace vmm {

// ProviderError of src/providers/device_memory.h:84-95, kOk added.
enum class Error { kOk, kInvalid, kOutOfMemory, kUnsupported, kFailed, kUnknown, kUndetermined };

struct Status {
  Error error = Error::kOk;
  std::string detail;
  // The runtime's own code where a primitive failed (what a negative C-ABI return carries), else 0.
  int native = 0;
  explicit operator bool() const { return error == Error::kOk; }
};

inline Status Ok() { return Status{}; }
inline Status Invalid(std::string detail) { return Status{Error::kInvalid, std::move(detail), 0}; }
inline Status RefuseUndetermined() {
  return Status{Error::kUndetermined, "undetermined after an unknown outcome: the owner must quarantine it", 0};
}

enum class Kind { kDevice, kHost };
struct AllocationClass {
  Kind kind = Kind::kDevice;
  std::uint32_t location = 0;  // the device ordinal, or the host NUMA node
  std::uint64_t granularity = 0;
};
enum class Access { kNone, kRead, kReadWrite };

// A table of values named by identities that are never reused: the low 32 bits a slot + 1, the high 32 the slot's
// generation (the reference's base::SlotTable and base::Id). 0 names nothing.
template <class T>
class Slots {
 public:
  std::uint64_t Insert(T value) {
    std::size_t slot = slots_.size();
    if (!free_.empty()) {
      slot = free_.back();
      free_.pop_back();
    } else {
      if (slots_.size() >= 0xFFFFFFFEu) return 0;
      slots_.emplace_back();
    }
    Slot& s = slots_[slot];
    s.value = std::move(value);
    s.live = true;
    ++live_;
    return (static_cast<std::uint64_t>(s.generation) << 32) | static_cast<std::uint64_t>(slot + 1);
  }
  T* Find(std::uint64_t id) {
    const std::uint64_t low = id & 0xFFFFFFFFu;
    if (low == 0 || low > slots_.size()) return nullptr;
    Slot& s = slots_[low - 1];
    return s.live && s.generation == static_cast<std::uint32_t>(id >> 32) ? &s.value : nullptr;
  }
  const T* Find(std::uint64_t id) const { return const_cast<Slots*>(this)->Find(id); }
  bool Erase(std::uint64_t id) {
    if (Find(id) == nullptr) return false;
    Slot& s = slots_[(id & 0xFFFFFFFFu) - 1];
    s.live = false;
    s.value = T();
    ++s.generation;
    free_.push_back(static_cast<std::size_t>((id & 0xFFFFFFFFu) - 1));
    --live_;
    return true;
  }
  std::size_t size() const { return live_; }
  template <class F>
  void ForEach(F&& f) const {
    for (const Slot& s : slots_)
      if (s.live) f(s.value);
  }

 private:
  struct Slot {
    T value{};
    std::uint32_t generation = 1;
    bool live = false;
  };
  std::vector<Slot> slots_;
  std::vector<std::size_t> free_;
  std::size_t live_ = 0;
};

class Rules {
 public:
  using Handle = std::uint64_t;  // the implementation's handle for a backing: an opaque number

  virtual ~Rules() = default;
  Rules(const Rules&) = delete;
  Rules& operator=(const Rules&) = delete;

  const std::vector<AllocationClass>& Classes() const { return classes_; }
  std::uint64_t Granularity() const { return granularity_; }

  // Reserve (device_memory.cc:60-87).
  Status Reserve(std::uint64_t size, std::uint64_t* reservation) {
    const Exclusive exclusive(changing_);
    if (size == 0 || !Aligned(size))
      return Invalid("a reservation of " + std::to_string(size) + " bytes is not a multiple of " + std::to_string(granularity_));
    std::uint64_t base = 0;
    if (Status reserved = DoReserve(size, &base); !reserved) {
      // The range may exist: keep it charged, with no address to use.
      if (reserved.error == Error::kUnknown) (void)reservations_.Insert(Reservation{0, size, {}, true});
      return reserved;
    }
    const std::uint64_t id = reservations_.Insert(Reservation{base, size, {}, false});
    if (id == 0) {
      const Status undone = DoFree(base, size);
      return undone ? Status{Error::kFailed, "the reservation table is full", 0}
                    : Status{undone.error, "the reservation table is full, and freeing the range failed: " + undone.detail, undone.native};
    }
    *reservation = id;
    return Ok();
  }

  // RangeOf (:112-121).
  Status RangeOf(std::uint64_t reservation, std::uint64_t* base, std::uint64_t* size) const {
    const Reservation* found = reservations_.Find(reservation);
    if (found == nullptr) return Invalid("stale or unknown reservation");
    if (found->undetermined) return RefuseUndetermined();
    *base = found->base;
    *size = found->size;
    return Ok();
  }

  // MappedAt (:123-130): the backing mapped at exactly `offset`, or 0.
  std::uint64_t MappedAt(std::uint64_t reservation, std::uint64_t offset) const {
    const Reservation* found = reservations_.Find(reservation);
    if (found == nullptr) return 0;
    const auto mapping = found->mappings.find(offset);
    return mapping != found->mappings.end() ? mapping->second.backing : 0;
  }

  // Free (:132-150).
  Status Free(std::uint64_t reservation) {
    const Exclusive exclusive(changing_);
    Reservation* found = reservations_.Find(reservation);
    if (found == nullptr) return Invalid("stale or unknown reservation");
    if (found->undetermined) return RefuseUndetermined();
    if (!found->mappings.empty()) return Invalid("the reservation still has mappings");
    if (Status freed = DoFree(found->base, found->size); !freed) {
      found->undetermined = freed.error == Error::kUnknown;
      return freed;
    }
    (void)reservations_.Erase(reservation);
    return Ok();
  }

  // Create (:152-198).
  Status Create(std::size_t allocation_class, std::uint64_t size, std::uint64_t* backing) {
    const Exclusive exclusive(changing_);
    if (allocation_class >= classes_.size()) return Invalid("no such allocation class");
    const AllocationClass& chosen = classes_[allocation_class];
    if (size == 0 || size % chosen.granularity != 0 || !Aligned(size))
      return Invalid("backing of " + std::to_string(size) + " bytes is not a multiple of the granularity");
    Handle handle = 0;
    if (Status created = DoCreate(chosen, size, &handle); !created) {
      // The backing may exist: keep it charged, with no handle to use.
      if (created.error == Error::kUnknown && backings_.Insert(Backing{allocation_class, size, 0, false, true}) != 0)
        live_backings_.fetch_add(1, std::memory_order_relaxed);
      return created;
    }
    const std::uint64_t id = backings_.Insert(Backing{allocation_class, size, handle, false, false});
    if (id == 0) {
      const Status undone = DoRelease(handle, size);
      return undone ? Status{Error::kFailed, "the backing table is full", 0}
                    : Status{undone.error, "the backing table is full, and releasing the backing failed: " + undone.detail, undone.native};
    }
    created_backings_.fetch_add(1, std::memory_order_relaxed);
    live_backings_.fetch_add(1, std::memory_order_relaxed);
    *backing = id;
    return Ok();
  }

  // Release (:200-222).
  Status Release(std::uint64_t backing) {
    const Exclusive exclusive(changing_);
    Backing* found = backings_.Find(backing);
    if (found == nullptr) return Invalid("stale or unknown backing");
    if (found->undetermined) return RefuseUndetermined();
    if (found->mapped) return Invalid("the backing is still mapped");
    if (Status released = DoRelease(found->handle, found->size); !released) {
      found->undetermined = released.error == Error::kUnknown;
      return released;
    }
    (void)backings_.Erase(backing);
    released_backings_.fetch_add(1, std::memory_order_relaxed);
    live_backings_.fetch_sub(1, std::memory_order_relaxed);
    return Ok();
  }

  // Map (:224-264).
  Status Map(std::uint64_t reservation, std::uint64_t offset, std::uint64_t backing) {
    const Exclusive exclusive(changing_);
    Reservation* place = reservations_.Find(reservation);
    Backing* found = backings_.Find(backing);
    if (place == nullptr || found == nullptr) return Invalid("stale or unknown reservation or backing");
    if (place->undetermined || found->undetermined) return RefuseUndetermined();
    if (found->mapped) return Invalid("the backing is already mapped");
    const std::uint64_t end = offset + found->size;
    if (!Aligned(offset) || end < offset || end > place->size) return Invalid("the mapping does not fit the reservation at that offset");
    // Into a hole: no mapping may overlap [offset, end).
    auto after = place->mappings.lower_bound(offset);
    if (after != place->mappings.end() && after->first < end) return Invalid("the mapping overlaps another");
    if (after != place->mappings.begin()) {
      const auto before = std::prev(after);
      if (before->first + before->second.size > offset) return Invalid("the mapping overlaps another");
    }
    if (Status mapped = DoMap(place->base + offset, found->size, found->handle); !mapped) {
      if (mapped.error == Error::kUnknown) {
        place->undetermined = true;  // the hole may hold the mapping now
        found->undetermined = true;
      }
      return mapped;
    }
    place->mappings.emplace(offset, Mapping{backing, found->size});
    found->mapped = true;
    return Ok();
  }

  // SetAccess (:293-350): one primitive call a run of mappings of the same kind (the CPU's access applies to host
  // backing only). A failure part-way leaves earlier runs changed; access is idempotent, the caller retries the
  // whole range.
  Status SetAccess(std::uint64_t reservation, std::uint64_t offset, std::uint64_t size, Access access) {
    const Exclusive exclusive(changing_);
    Reservation* place = reservations_.Find(reservation);
    if (place == nullptr) return Invalid("stale or unknown reservation");
    if (place->undetermined) return RefuseUndetermined();
    std::vector<std::uint64_t> covered;
    if (Status whole = Covered(*place, offset, size, &covered); !whole) return whole;
    const auto quarantine = [&] {
      place->undetermined = true;
      for (const std::uint64_t at : covered) backings_.Find(place->mappings.at(at).backing)->undetermined = true;
    };
    std::uint64_t run_start = offset, run_end = offset;
    bool run_host = false;
    for (const std::uint64_t at : covered) {
      const Mapping& mapping = place->mappings.at(at);
      const Backing* backing = backings_.Find(mapping.backing);
      Check(backing != nullptr, "a mapping of a released backing");
      const bool host = classes_[backing->allocation_class].kind == Kind::kHost;
      if (run_end > run_start && host != run_host) {
        if (Status set = DoSetAccess(place->base + run_start, run_end - run_start, access, run_host); !set) {
          if (set.error == Error::kUnknown) quarantine();
          return set;
        }
        run_start = run_end;
      }
      run_host = host;
      run_end = at + mapping.size;
    }
    Status set = DoSetAccess(place->base + run_start, run_end - run_start, access, run_host);
    if (!set && set.error == Error::kUnknown) quarantine();
    return set;
  }

  // Unmap (:352-385): whole mappings only.
  Status Unmap(std::uint64_t reservation, std::uint64_t offset, std::uint64_t size) {
    const Exclusive exclusive(changing_);
    Reservation* place = reservations_.Find(reservation);
    if (place == nullptr) return Invalid("stale or unknown reservation");
    if (place->undetermined) return RefuseUndetermined();
    std::vector<std::uint64_t> covered;
    if (Status whole = Covered(*place, offset, size, &covered); !whole) return whole;
    if (Status unmapped = DoUnmap(place->base + offset, size); !unmapped) {
      if (unmapped.error == Error::kUnknown) {
        place->undetermined = true;
        for (const std::uint64_t at : covered) backings_.Find(place->mappings.at(at).backing)->undetermined = true;
      }
      return unmapped;
    }
    for (const std::uint64_t at : covered) {
      Backing* backing = backings_.Find(place->mappings.at(at).backing);
      Check(backing != nullptr, "a mapping of a released backing");
      backing->mapped = false;
      place->mappings.erase(at);
    }
    return Ok();
  }

  // Whether an unknown outcome left it undetermined (:89-110), and the backing bytes that are.
  bool UndeterminedReservation(std::uint64_t reservation) const {
    const Reservation* found = reservations_.Find(reservation);
    return found != nullptr && found->undetermined;
  }
  bool UndeterminedBacking(std::uint64_t backing) const {
    const Backing* found = backings_.Find(backing);
    return found != nullptr && found->undetermined;
  }
  std::uint64_t UndeterminedBytes() const {
    std::uint64_t total = 0;
    backings_.ForEach([&](const Backing& backing) {
      if (backing.undetermined) total += backing.size;
    });
    return total;
  }

  // What is live, for tests and leak checks at shutdown (device_memory.h:183-192).
  std::size_t reservations() const { return reservations_.size(); }
  std::size_t backings() const { return live_backings_.load(std::memory_order_relaxed); }
  std::uint64_t created_backings() const { return created_backings_.load(std::memory_order_relaxed); }
  std::uint64_t released_backings() const { return released_backings_.load(std::memory_order_relaxed); }

 protected:
  // `granularity` must be a non-zero multiple of every class's granularity.
  Rules(std::vector<AllocationClass> classes, std::uint64_t granularity) : classes_(std::move(classes)), granularity_(granularity) {}

  // The primitives, called only once the rules above pass (device_memory.h:200-213).
  virtual Status DoReserve(std::uint64_t size, std::uint64_t* base) = 0;
  virtual Status DoFree(std::uint64_t base, std::uint64_t size) = 0;
  virtual Status DoCreate(const AllocationClass& allocation_class, std::uint64_t size, Handle* handle) = 0;
  virtual Status DoRelease(Handle handle, std::uint64_t size) = 0;
  virtual Status DoMap(std::uint64_t address, std::uint64_t size, Handle handle) = 0;
  virtual Status DoSetAccess(std::uint64_t address, std::uint64_t size, Access access, bool host) = 0;
  virtual Status DoUnmap(std::uint64_t address, std::uint64_t size) = 0;

 private:
  struct Mapping {
    std::uint64_t backing = 0;
    std::uint64_t size = 0;
  };
  struct Reservation {
    std::uint64_t base = 0;
    std::uint64_t size = 0;
    std::map<std::uint64_t, Mapping> mappings;  // by offset
    bool undetermined = false;
  };
  struct Backing {
    std::size_t allocation_class = 0;
    std::uint64_t size = 0;
    Handle handle = 0;
    bool mapped = false;
    bool undetermined = false;
  };

  static void Check(bool holds, const char* what) {
    if (!holds) {
      std::fprintf(stderr, "llmp_hip memory provider: %s\n", what);
      std::abort();
    }
  }
  // Held by each call that changes the provider: a second at once is fatal (one thread calls a provider at a time,
  // device_memory.h:16-29).
  class Exclusive {
   public:
    explicit Exclusive(std::atomic<bool>& changing) : changing_(changing) {
      Check(!changing_.exchange(true, std::memory_order_acquire),
            "two threads changed a memory provider at once: one thread calls it at a time");
    }
    ~Exclusive() { changing_.store(false, std::memory_order_release); }
    Exclusive(const Exclusive&) = delete;
    Exclusive& operator=(const Exclusive&) = delete;

   private:
    std::atomic<bool>& changing_;
  };

  // The mappings exactly covering [offset, offset + size), or a refusal if the range splits a mapping, leaves a
  // hole, or runs outside (device_memory.cc:266-291).
  static Status Covered(const Reservation& reservation, std::uint64_t offset, std::uint64_t size, std::vector<std::uint64_t>* covered) {
    const std::uint64_t end = offset + size;
    if (size == 0 || end < offset || end > reservation.size) return Invalid("the range runs outside the reservation");
    std::uint64_t at = offset;
    auto mapping = reservation.mappings.find(at);
    while (at < end) {
      if (mapping == reservation.mappings.end() || mapping->first != at) return Invalid("the range does not cover whole mappings");
      covered->push_back(at);
      at += mapping->second.size;
      ++mapping;
    }
    if (at != end) return Invalid("the range splits a mapping");
    return Ok();
  }
  bool Aligned(std::uint64_t value) const { return value % granularity_ == 0; }

  std::vector<AllocationClass> classes_;
  std::uint64_t granularity_;
  mutable std::atomic<bool> changing_{false};
  std::atomic<std::uint64_t> created_backings_{0};
  std::atomic<std::uint64_t> released_backings_{0};
  std::atomic<std::size_t> live_backings_{0};
  Slots<Reservation> reservations_;
  Slots<Backing> backings_;
};

}  // namespace vmm
}  // namespace llmp_hip

#endif  // LLMP_AMD_CSRC_VMM_RULES_H_
