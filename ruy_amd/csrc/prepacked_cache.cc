#include "prepacked_cache.h"

namespace ruyamd {

std::size_t PrepackedCache::KeyHash::operator()(const Key& k) const {
  std::size_t h = reinterpret_cast<std::size_t>(k.src_data) >> 4;
  auto mix = [&h](std::size_t v) { h = h * 0x9E3779B97F4A7C15ull + v; };
  mix(static_cast<std::size_t>(k.layout.rows));
  mix(static_cast<std::size_t>(k.layout.cols));
  mix(static_cast<std::size_t>(k.layout.stride));
  mix(k.layout.order | (k.layout.kernel_order << 1) | (k.layout.kernel_rows << 8) |
      (k.layout.kernel_cols << 16));
  mix(static_cast<std::size_t>(static_cast<uint32_t>(k.zero_point)));
  return h;
}

PrepackedCache::Action PrepackedCache::Get(const void* src_data, PackedMatrix* packed_matrix, Mode mode) {
  Key key{src_data, packed_matrix->layout, packed_matrix->zero_point};
  auto it = cache_.find(key);
  if (it != cache_.end()) {
    it->second.timestamp = timestamp_++;
    if (mode == Mode::kPinExisting) it->second.pinned = true;
    *packed_matrix = it->second.packed;
    return Action::kGotExistingEntry;
  }
  if (mode != Mode::kInsertOnMiss) {
    packed_matrix->data = nullptr;
    packed_matrix->sums = nullptr;
    return Action::kMissing;
  }
  const std::ptrdiff_t data_bytes = packed_matrix->DataBytes();
  const std::ptrdiff_t sums_bytes = packed_matrix->SumsBytes();
  const std::ptrdiff_t new_bytes = data_bytes + sums_bytes;
  // Make room first: on a device the budget is real memory.
  EjectUntilRoomFor(new_bytes);
  packed_matrix->data = alloc_(static_cast<std::size_t>(data_bytes > 0 ? data_bytes : 1));
  packed_matrix->sums = nullptr;
  if (sums_bytes > 0 && packed_matrix->data) {
    packed_matrix->sums = static_cast<int32_t*>(alloc_(static_cast<std::size_t>(sums_bytes)));
    if (!packed_matrix->sums) {
      free_(packed_matrix->data);
      packed_matrix->data = nullptr;
    }
  }
  if (!packed_matrix->data) return Action::kInsertedNewEntry;  // allocation failed
  cache_.emplace(key, Entry{*packed_matrix, timestamp_++});
  buffers_bytes_ += new_bytes;
  return Action::kInsertedNewEntry;
}

bool PrepackedCache::Erase(const void* src_data, const PackedMatrix& packed_matrix) {
  auto it = cache_.find(Key{src_data, packed_matrix.layout, packed_matrix.zero_point});
  if (it == cache_.end()) return false;
  const PackedMatrix& pm = it->second.packed;
  buffers_bytes_ -= pm.DataBytes() + pm.SumsBytes();
  free_(pm.data);
  if (pm.sums) free_(pm.sums);
  cache_.erase(it);
  return true;
}

bool PrepackedCache::HasSource(const void* src_data) const {
  for (const auto& kv : cache_)
    if (kv.first.src_data == src_data) return true;
  return false;
}

void PrepackedCache::EjectUntilRoomFor(std::ptrdiff_t new_bytes) {
  while (!cache_.empty() && buffers_bytes_ + new_bytes > max_buffers_bytes_) {
    if (!EjectOne()) break;
  }
}

bool PrepackedCache::EjectOne() {
  auto oldest = cache_.end();
  for (auto it = cache_.begin(); it != cache_.end(); ++it) {
    if (it->second.pinned) continue;
    if (oldest == cache_.end() || it->second.timestamp < oldest->second.timestamp) oldest = it;
  }
  if (oldest == cache_.end()) return false;
  const PackedMatrix& pm = oldest->second.packed;
  buffers_bytes_ -= pm.DataBytes() + pm.SumsBytes();
  free_(pm.data);
  if (pm.sums) free_(pm.sums);
  cache_.erase(oldest);
  return true;
}

void PrepackedCache::Clear() {
  for (auto& kv : cache_) {
    free_(kv.second.packed.data);
    if (kv.second.packed.sums) free_(kv.second.packed.sums);
  }
  cache_.clear();
  buffers_bytes_ = 0;
}

}  // namespace ruyamd
