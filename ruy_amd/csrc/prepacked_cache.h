// The prepacked-matrix cache of a context: semantics of ruy::PrepackedCache
// (ruy/prepacked_cache.h:45-127, ruy/prepacked_cache.cc:79-127) over device
// buffers. Pure host logic with an injected allocator, so it can be unit-tested
// without a GPU.
#ifndef RUY_AMD_CSRC_PREPACKED_CACHE_H_
#define RUY_AMD_CSRC_PREPACKED_CACHE_H_

#include <cstddef>
#include <cstdint>
#include <functional>
#include <unordered_map>

namespace ruyamd {

// Shape of a packed operand: the fields of ruy::PMatLayout (ruy/mat.h:166-188).
// `rows` is the (padded) depth, `cols` the (padded) width; `kernel_*` describe
// the inner tile the consuming kernel wants.
struct PackedLayout {
  int32_t rows = 0;
  int32_t cols = 0;
  int32_t stride = 0;
  uint8_t order = 0;
  uint8_t kernel_order = 0;
  uint8_t kernel_rows = 1;
  uint8_t kernel_cols = 1;
  bool operator==(const PackedLayout& o) const {
    return rows == o.rows && cols == o.cols && stride == o.stride && order == o.order &&
           kernel_order == o.kernel_order && kernel_rows == o.kernel_rows &&
           kernel_cols == o.kernel_cols;
  }
};

// A packed operand (ruy::PEMat, ruy/mat.h:255-275): data in the kernel's
// layout plus one int32 sum per column for integer types.
struct PackedMatrix {
  void* data = nullptr;
  int32_t* sums = nullptr;
  int32_t element_size = 1;
  bool is_floating_point = false;
  PackedLayout layout;
  int32_t zero_point = 0;

  // ruy::DataBytes / ruy::SumsBytes (ruy/mat.h:341-349).
  std::ptrdiff_t DataBytes() const {
    return static_cast<std::ptrdiff_t>(layout.stride) *
           (layout.order == 0 ? layout.cols : layout.rows) * element_size;
  }
  std::ptrdiff_t SumsBytes() const {
    return is_floating_point ? 0 : static_cast<std::ptrdiff_t>(layout.cols) * 4;
  }
};

class PrepackedCache final {
 public:
  enum class Action { kGotExistingEntry, kInsertedNewEntry, kMissing };
  // kPinExisting never allocates or frees: a hit is marked so that ejection
  // passes it over from then on (its buffers may be referenced by work that
  // was recorded for later replay), a miss returns kMissing. kLookupOnly is
  // the same without the mark (for callers that may not allocate but whose
  // work has run by the time anything could be ejected).
  enum class Mode { kInsertOnMiss, kPinExisting, kLookupOnly };
  using AllocFn = std::function<void*(std::size_t)>;
  using FreeFn = std::function<void(void*)>;

  // ruy/prepacked_cache.h:45
  static constexpr std::ptrdiff_t kDefaultMaxBuffersBytes = 1 << 28;

  PrepackedCache(AllocFn alloc, FreeFn free_fn,
                 std::ptrdiff_t max_buffers_bytes = kDefaultMaxBuffersBytes)
      : alloc_(std::move(alloc)), free_(std::move(free_fn)), max_buffers_bytes_(max_buffers_bytes) {}
  ~PrepackedCache() { Clear(); }
  PrepackedCache(const PrepackedCache&) = delete;
  PrepackedCache& operator=(const PrepackedCache&) = delete;

  // Looks the (src pointer, packed layout, zero point) key up. On a hit fills
  // packed_matrix->data/sums from the entry and refreshes its timestamp. On a
  // miss allocates both buffers, ejects least-recently-used entries until the
  // new one fits or the cache is empty (an entry larger than the whole budget
  // is still kept), and inserts it; the caller must then pack into the buffers.
  // Returns kInsertedNewEntry with null data if allocation failed.
  Action Get(const void* src_data, PackedMatrix* packed_matrix, Mode mode = Mode::kInsertOnMiss);

  // Removes the entry with this key, if any, and releases its buffers: for a
  // caller that was handed a new entry and then failed to fill it, so that no
  // later Get finds buffers that were never packed. Returns whether an entry
  // was removed. (No counterpart in the reference, whose pack cannot fail.)
  bool Erase(const void* src_data, const PackedMatrix& packed_matrix);

  // Whether any entry was packed from this source pointer (whatever its layout
  // and zero point): a cheap test ahead of work that would be wasted if the
  // exact entry turned out to be missing.
  bool HasSource(const void* src_data) const;

  std::ptrdiff_t BuffersBytes() const { return buffers_bytes_; }
  int MatrixCount() const { return static_cast<int>(cache_.size()); }
  std::ptrdiff_t MaxBuffersBytes() const { return max_buffers_bytes_; }
  void Clear();
  void SetMaxBuffersBytes(std::ptrdiff_t v) {
    Clear();
    max_buffers_bytes_ = v;
  }

 private:
  struct Key {
    const void* src_data;
    PackedLayout layout;
    int32_t zero_point;
    bool operator==(const Key& o) const {
      return src_data == o.src_data && layout == o.layout && zero_point == o.zero_point;
    }
  };
  struct KeyHash {
    std::size_t operator()(const Key& k) const;
  };
  struct Entry {
    PackedMatrix packed;
    uint64_t timestamp;
    bool pinned = false;  // only Clear() releases a pinned entry
  };
  void EjectUntilRoomFor(std::ptrdiff_t new_bytes);
  bool EjectOne();  // false when only pinned entries are left

  AllocFn alloc_;
  FreeFn free_;
  std::unordered_map<Key, Entry, KeyHash> cache_;
  std::ptrdiff_t max_buffers_bytes_;
  std::ptrdiff_t buffers_bytes_ = 0;
  uint64_t timestamp_ = 0;
};

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_PREPACKED_CACHE_H_
