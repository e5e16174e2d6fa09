// The books of the device-memory provider (include/llmp_hip_memory.h), kept apart from the runtime calls that move
// memory. The contract is the one the reference states for every implementation of its DeviceMemory
// (src/providers/device_memory.h:30-45, 118-157): reservations and backing in whole granules, a backing mapped whole
// into a hole at most once, access and unmapping over ranges that are whole mappings end to end, nothing released or
// freed while mapped, and an operation whose outcome the runtime cannot tell leaves what it touched lost: refused from
// then on and never tried again.
//
// How the books are kept here. Everything is counted in granules. A region (a reservation) holds its mappings as a
// vector of extents sorted by first granule, searched by bisection; a block (a backing) remembers the region it is
// attached to. Names come from one counter shared by regions and blocks, so a name is never handed out twice and a
// region's name never names a block. Every operation has the same three beats: Check (pure, refuses with nothing
// touched), one or more calls of the Backend, and Settle (commit what was done, or mark what a lost outcome may have
// changed). Plain C++, no device types: memory.hip supplies the Backend over HIP; tests/host/memory_test.cc supplies
// one that counts, fails and loses outcomes on request.
#ifndef LLMP_AMD_CSRC_VMM_LEDGER_H_
#define LLMP_AMD_CSRC_VMM_LEDGER_H_

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace llmp_hip {
namespace vmm {

// ProviderError (src/providers/device_memory.h:84-95) with a value for success.
enum class Error { kOk, kInvalid, kOutOfMemory, kUnsupported, kFailed, kUnknown, kUndetermined };

struct Status {
  Error error = Error::kOk;
  std::string detail;
  int native = 0;  // the runtime's own code where a Backend call failed, else 0
  explicit operator bool() const { return error == Error::kOk; }
  bool lost() const { return error == Error::kUnknown; }
};
inline Status Ok() { return {}; }
inline Status Misuse(const char* what) { return {Error::kInvalid, what, 0}; }
inline Status Quarantined() { return {Error::kUndetermined, "lost to an earlier unknown outcome: its owner quarantines it", 0}; }

enum class Kind { kDevice, kHost };
enum class Access { kNone, kRead, kReadWrite };
struct AllocationClass {
  Kind kind = Kind::kDevice;
  std::uint32_t location = 0;  // the device ordinal, or the host NUMA node
  std::uint64_t granularity = 0;
};

// What moves memory. Byte addresses and sizes; called only with arguments the ledger has checked.
class Backend {
 public:
  virtual ~Backend() = default;
  virtual Status ReserveSpace(std::uint64_t bytes, std::uint64_t* base) = 0;
  virtual Status FreeSpace(std::uint64_t base, std::uint64_t bytes) = 0;
  virtual Status CreateBlock(const AllocationClass& from, std::uint64_t bytes, std::uint64_t* handle) = 0;
  virtual Status ReleaseBlock(std::uint64_t handle) = 0;
  virtual Status Attach(std::uint64_t address, std::uint64_t bytes, std::uint64_t handle) = 0;
  // `cpu_too`: the range holds host backing, which the CPU of its node reads and writes as well.
  virtual Status Protect(std::uint64_t address, std::uint64_t bytes, Access access, bool cpu_too) = 0;
  virtual Status Detach(std::uint64_t address, std::uint64_t bytes) = 0;
};

class Ledger {
 public:
  // `granule`: a non-zero multiple of every class's granularity.
  Ledger(Backend* backend, std::vector<AllocationClass> classes, std::uint64_t granule)
      : backend_(backend), classes_(std::move(classes)), granule_(granule) {}
  Ledger(const Ledger&) = delete;
  Ledger& operator=(const Ledger&) = delete;

  const std::vector<AllocationClass>& Classes() const { return classes_; }
  std::uint64_t Granularity() const { return granule_; }

  Status Reserve(std::uint64_t bytes, std::uint64_t* name) {
    const Turn turn(busy_);
    if (bytes == 0 || bytes % granule_ != 0) return Misuse("a reservation is a non-zero number of whole granules");
    Region region;
    region.granules = bytes / granule_;
    const Status made = backend_->ReserveSpace(bytes, &region.base);
    if (!made && !made.lost()) return made;
    region.lost = made.lost();  // address space that may exist stays on the books, with no address to hand out
    if (region.lost) region.base = 0;
    const std::uint64_t id = next_name_++;
    regions_.emplace(id, std::move(region));
    if (made) *name = id;
    return made;
  }

  Status RangeOf(std::uint64_t name, std::uint64_t* base, std::uint64_t* bytes) const {
    const Region* region = Find(regions_, name);
    if (region == nullptr) return Misuse("no such reservation");
    if (region->lost) return Quarantined();
    *base = region->base;
    *bytes = region->granules * granule_;
    return Ok();
  }

  Status Free(std::uint64_t name) {
    const Turn turn(busy_);
    Region* region = Find(regions_, name);
    if (region == nullptr) return Misuse("no such reservation");
    if (region->lost) return Quarantined();
    if (!region->extents.empty()) return Misuse("a reservation is freed only when nothing is mapped in it");
    const Status freed = backend_->FreeSpace(region->base, region->granules * granule_);
    if (freed) {
      regions_.erase(name);
    } else {
      region->lost = freed.lost();
    }
    return freed;
  }

  Status Create(std::size_t allocation_class, std::uint64_t bytes, std::uint64_t* name) {
    const Turn turn(busy_);
    if (allocation_class >= classes_.size()) return Misuse("no such allocation class");
    const AllocationClass& from = classes_[allocation_class];
    if (bytes == 0 || bytes % granule_ != 0 || bytes % from.granularity != 0)
      return Misuse("backing is a non-zero number of whole granules, of the provider's and of its class's");
    Block block;
    block.from = allocation_class;
    block.granules = bytes / granule_;
    const Status made = backend_->CreateBlock(from, bytes, &block.handle);
    if (!made && !made.lost()) return made;
    block.lost = made.lost();  // memory that may exist stays charged, with no handle to use
    const std::uint64_t id = next_name_++;
    blocks_.emplace(id, block);
    if (made) {
      ++created_;
      *name = id;
    }
    return made;
  }

  Status Release(std::uint64_t name) {
    const Turn turn(busy_);
    Block* block = Find(blocks_, name);
    if (block == nullptr) return Misuse("no such backing");
    if (block->lost) return Quarantined();
    if (block->region != 0) return Misuse("backing is released only when unmapped");
    const Status released = backend_->ReleaseBlock(block->handle);
    if (released) {
      blocks_.erase(name);
      ++released_;
    } else {
      block->lost = released.lost();
    }
    return released;
  }

  Status Map(std::uint64_t region_name, std::uint64_t offset, std::uint64_t block_name) {
    const Turn turn(busy_);
    Region* region = Find(regions_, region_name);
    Block* block = Find(blocks_, block_name);
    if (region == nullptr || block == nullptr) return Misuse("no such reservation or backing");
    if (region->lost || block->lost) return Quarantined();
    if (block->region != 0) return Misuse("a backing is mapped at most once at a time");
    if (offset % granule_ != 0) return Misuse("a mapping starts on a granule");
    const std::uint64_t first = offset / granule_;
    if (first >= region->granules || block->granules > region->granules - first) return Misuse("the mapping runs outside the reservation");
    // The first extent that ends beyond `first` must start at or after the new mapping's end.
    const auto next = std::partition_point(region->extents.begin(), region->extents.end(),
                                           [&](const Extent& e) { return e.first + e.count <= first; });
    if (next != region->extents.end() && next->first < first + block->granules) return Misuse("the mapping would overlap another");
    const Status attached = backend_->Attach(region->base + offset, block->granules * granule_, block->handle);
    if (attached) {
      region->extents.insert(next, Extent{first, block->granules, block_name});
      block->region = region_name;
    } else if (attached.lost()) {
      region->lost = block->lost = true;
    }
    return attached;
  }

  // One Backend call for each stretch of neighbouring mappings of one kind of backing (the CPU's access goes with host
  // backing only). Access is idempotent: after a failure part-way the caller sets the whole range again.
  Status SetAccess(std::uint64_t region_name, std::uint64_t offset, std::uint64_t bytes, Access access) {
    const Turn turn(busy_);
    Region* region = Find(regions_, region_name);
    if (region == nullptr) return Misuse("no such reservation");
    if (region->lost) return Quarantined();
    std::size_t from = 0, to = 0;
    if (const Status whole = WholeMappings(*region, offset, bytes, &from, &to); !whole) return whole;
    for (std::size_t at = from; at < to;) {
      const bool host = OnHost(region->extents[at]);
      std::size_t stop = at + 1;
      while (stop < to && OnHost(region->extents[stop]) == host) ++stop;
      const std::uint64_t start = region->extents[at].first;
      const std::uint64_t end = region->extents[stop - 1].first + region->extents[stop - 1].count;
      const Status set = backend_->Protect(region->base + start * granule_, (end - start) * granule_, access, host);
      if (!set) {
        if (set.lost()) Lose(region, from, to);
        return set;
      }
      at = stop;
    }
    return Ok();
  }

  Status Unmap(std::uint64_t region_name, std::uint64_t offset, std::uint64_t bytes) {
    const Turn turn(busy_);
    Region* region = Find(regions_, region_name);
    if (region == nullptr) return Misuse("no such reservation");
    if (region->lost) return Quarantined();
    std::size_t from = 0, to = 0;
    if (const Status whole = WholeMappings(*region, offset, bytes, &from, &to); !whole) return whole;
    const Status detached = backend_->Detach(region->base + offset, bytes);
    if (detached) {
      for (std::size_t at = from; at < to; ++at) blocks_.at(region->extents[at].block).region = 0;
      region->extents.erase(region->extents.begin() + static_cast<std::ptrdiff_t>(from), region->extents.begin() + static_cast<std::ptrdiff_t>(to));
    } else if (detached.lost()) {
      Lose(region, from, to);
    }
    return detached;
  }

  // The backing whose mapping starts at exactly `offset`, or 0.
  std::uint64_t MappedAt(std::uint64_t region_name, std::uint64_t offset) const {
    const Region* region = Find(regions_, region_name);
    if (region == nullptr || offset % granule_ != 0) return 0;
    const std::size_t at = FirstAtOrAfter(*region, offset / granule_);
    return at < region->extents.size() && region->extents[at].first == offset / granule_ ? region->extents[at].block : 0;
  }

  bool UndeterminedReservation(std::uint64_t name) const {
    const Region* region = Find(regions_, name);
    return region != nullptr && region->lost;
  }
  bool UndeterminedBacking(std::uint64_t name) const {
    const Block* block = Find(blocks_, name);
    return block != nullptr && block->lost;
  }
  std::uint64_t UndeterminedBytes() const {
    std::uint64_t granules = 0;
    for (const auto& entry : blocks_)
      if (entry.second.lost) granules += entry.second.granules;
    return granules * granule_;
  }
  std::size_t reservations() const { return regions_.size(); }
  std::size_t backings() const { return blocks_.size(); }
  std::uint64_t created_backings() const { return created_; }
  std::uint64_t released_backings() const { return released_; }

 private:
  struct Extent {
    std::uint64_t first = 0, count = 0;  // granules
    std::uint64_t block = 0;             // the backing's name
  };
  struct Region {
    std::uint64_t base = 0, granules = 0;
    std::vector<Extent> extents;  // sorted by `first`, never overlapping
    bool lost = false;
  };
  struct Block {
    std::size_t from = 0;  // index of its allocation class
    std::uint64_t granules = 0, handle = 0;
    std::uint64_t region = 0;  // the reservation it is mapped in, 0 when unmapped
    bool lost = false;
  };

  // One thread calls a provider at a time (device_memory.h:16-29); a second caller while one is inside is a bug of
  // the program, reported and fatal rather than waited for.
  class Turn {
   public:
    explicit Turn(std::mutex& busy) : busy_(busy) {
      if (!busy_.try_lock()) {
        std::fprintf(stderr, "llmp_hip memory provider: entered by two threads at once\n");
        std::abort();
      }
    }
    ~Turn() { busy_.unlock(); }

   private:
    std::mutex& busy_;
  };

  template <class Table>
  static auto Find(Table& table, std::uint64_t name) -> decltype(&table.begin()->second) {
    const auto at = table.find(name);
    return at == table.end() ? nullptr : &at->second;
  }
  std::size_t FirstAtOrAfter(const Region& region, std::uint64_t granule) const {
    return static_cast<std::size_t>(std::partition_point(region.extents.begin(), region.extents.end(),
                                                         [&](const Extent& e) { return e.first < granule; }) -
                                    region.extents.begin());
  }
  bool OnHost(const Extent& extent) const { return classes_[blocks_.at(extent.block).from].kind == Kind::kHost; }
  // [offset, offset + bytes) as extents [*from, *to): refused unless they tile the range with no hole and no overhang.
  Status WholeMappings(const Region& region, std::uint64_t offset, std::uint64_t bytes, std::size_t* from, std::size_t* to) const {
    if (bytes == 0 || offset % granule_ != 0 || bytes % granule_ != 0) return Misuse("the range is not whole granules");
    const std::uint64_t first = offset / granule_, count = bytes / granule_;
    if (first >= region.granules || count > region.granules - first) return Misuse("the range runs outside the reservation");
    std::size_t at = FirstAtOrAfter(region, first);
    *from = at;
    std::uint64_t expect = first;
    while (expect < first + count) {
      if (at == region.extents.size() || region.extents[at].first != expect) return Misuse("the range does not start and continue on whole mappings");
      expect += region.extents[at++].count;
    }
    if (expect != first + count) return Misuse("the range ends inside a mapping");
    *to = at;
    return Ok();
  }
  void Lose(Region* region, std::size_t from, std::size_t to) {
    region->lost = true;
    for (std::size_t at = from; at < to; ++at) blocks_.at(region->extents[at].block).lost = true;
  }

  Backend* backend_;
  std::vector<AllocationClass> classes_;
  std::uint64_t granule_;
  std::mutex busy_;
  std::uint64_t next_name_ = 1, created_ = 0, released_ = 0;
  std::unordered_map<std::uint64_t, Region> regions_;
  std::unordered_map<std::uint64_t, Block> blocks_;
};

}  // namespace vmm
}  // namespace llmp_hip

#endif  // LLMP_AMD_CSRC_VMM_LEDGER_H_
