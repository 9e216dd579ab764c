// Host-only unit test of ruyamd::PrepackedCache with a malloc allocator.
// Mirrors the reference's known answers for the cache
// (ruy/prepacked_cache_test.cc:54-227): byte accounting 307 / 860, ejection of
// the least recently used entry, an over-budget entry is still kept, and keys
// that differ in pointer, shape, order or kernel layout are distinct.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "prepacked_cache.h"

using ruyamd::PackedMatrix;
using ruyamd::PrepackedCache;

static int g_failures = 0;
static int g_live_allocations = 0;
#define EXPECT(cond)                                                          \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::fprintf(stderr, "%s:%d: EXPECT failed: %s\n", __FILE__, __LINE__, #cond); \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

static void* CountingAlloc(std::size_t n) {
  ++g_live_allocations;
  return std::malloc(n);
}
static void CountingFree(void* p) {
  if (p) --g_live_allocations;
  std::free(p);
}

static PackedMatrix Dummy(bool is_float, int rows, int cols) {
  PackedMatrix m;
  m.element_size = is_float ? 4 : 1;
  m.is_floating_point = is_float;
  m.layout.rows = rows;
  m.layout.cols = cols;
  m.layout.stride = rows;
  m.layout.order = 0;
  m.layout.kernel_rows = 1;
  m.layout.kernel_cols = 1;
  return m;
}

static const auto kInserted = PrepackedCache::Action::kInsertedNewEntry;
static const auto kExisting = PrepackedCache::Action::kGotExistingEntry;

static void TestBasic() {
  PrepackedCache cache(CountingAlloc, CountingFree, 307);
  std::vector<std::uint8_t> data1(10 * 20), data2(5 * 3);
  PackedMatrix mat1 = Dummy(false, 10, 20);  // 200 + 20*4 = 280 bytes
  PackedMatrix mat2 = Dummy(false, 5, 3);    // 15 + 3*4 = 27 bytes
  EXPECT(cache.Get(data1.data(), &mat1) == kInserted);
  EXPECT(mat1.data != nullptr && mat1.sums != nullptr);
  EXPECT(cache.Get(data2.data(), &mat2) == kInserted);
  EXPECT(cache.MatrixCount() == 2);
  EXPECT(cache.BuffersBytes() == 307);
  PackedMatrix again = Dummy(false, 10, 20);
  EXPECT(cache.Get(data1.data(), &again) == kExisting);
  EXPECT(again.data == mat1.data && again.sums == mat1.sums);
  EXPECT(cache.Get(data2.data(), &mat2) == kExisting);
}

static void TestBasicFloat() {
  PrepackedCache cache(CountingAlloc, CountingFree, 860);
  std::vector<float> data1(10 * 20), data2(5 * 3);
  PackedMatrix mat1 = Dummy(true, 10, 20);  // 800 bytes, no sums
  PackedMatrix mat2 = Dummy(true, 5, 3);    // 60 bytes
  EXPECT(cache.Get(data1.data(), &mat1) == kInserted);
  EXPECT(mat1.sums == nullptr);
  EXPECT(cache.Get(data2.data(), &mat2) == kInserted);
  EXPECT(cache.MatrixCount() == 2);
  EXPECT(cache.BuffersBytes() == 860);
  EXPECT(cache.Get(data1.data(), &mat1) == kExisting);
  EXPECT(cache.Get(data2.data(), &mat2) == kExisting);
}

static void TestEjection() {
  PrepackedCache cache(CountingAlloc, CountingFree, 306);  // one byte short of both
  std::vector<std::uint8_t> data1(10 * 20), data2(5 * 3);
  PackedMatrix mat1 = Dummy(false, 10, 20), mat2 = Dummy(false, 5, 3);
  cache.Get(data1.data(), &mat1);
  cache.Get(data2.data(), &mat2);
  EXPECT(cache.MatrixCount() == 1);
  EXPECT(cache.BuffersBytes() == 27);
  EXPECT(cache.Get(data2.data(), &mat2) == kExisting);
  EXPECT(cache.Get(data1.data(), &mat1) == kInserted);
  EXPECT(cache.MatrixCount() == 1);
  EXPECT(cache.BuffersBytes() == 280);
  EXPECT(cache.Get(data1.data(), &mat1) == kExisting);
  EXPECT(cache.Get(data2.data(), &mat2) == kInserted);
}

static void TestEjectionOrder() {
  PrepackedCache cache(CountingAlloc, CountingFree, 1000);
  std::vector<std::uint8_t> d1(200), d2(200), d3(200), d4(200);
  PackedMatrix m1 = Dummy(false, 10, 20), m2 = m1, m3 = m1, m4 = m1;
  cache.Get(d1.data(), &m1);
  cache.Get(d2.data(), &m2);
  cache.Get(d3.data(), &m3);
  EXPECT(cache.Get(d1.data(), &m1) == kExisting);  // touch 1 and 3: 2 is the oldest
  EXPECT(cache.Get(d3.data(), &m3) == kExisting);
  cache.Get(d4.data(), &m4);
  EXPECT(cache.MatrixCount() == 3);
  EXPECT(cache.Get(d1.data(), &m1) == kExisting);
  EXPECT(cache.Get(d3.data(), &m3) == kExisting);
  EXPECT(cache.Get(d4.data(), &m4) == kExisting);
  EXPECT(cache.Get(d2.data(), &m2) == kInserted);
}

// Not in the reference: entries looked up in kPinExisting mode (their buffers
// are referenced by recorded work) survive ejection; a miss in that mode
// neither allocates nor inserts.
static void TestPinnedEntriesSurviveEjection() {
  PrepackedCache cache(CountingAlloc, CountingFree, 1000);
  std::vector<std::uint8_t> d1(200), d2(200), d3(200), d4(200), d5(200);
  PackedMatrix m1 = Dummy(false, 10, 20), m2 = m1, m3 = m1, m4 = m1, m5 = m1;
  const auto kPin = PrepackedCache::Mode::kPinExisting;
  const long allocs_before = g_live_allocations;
  EXPECT(cache.Get(d1.data(), &m1, kPin) == PrepackedCache::Action::kMissing);
  EXPECT(m1.data == nullptr && cache.MatrixCount() == 0 && g_live_allocations == allocs_before);
  m1 = Dummy(false, 10, 20);
  cache.Get(d1.data(), &m1);
  cache.Get(d2.data(), &m2);
  cache.Get(d3.data(), &m3);
  void* const pinned_data = m1.data;
  EXPECT(cache.Get(d1.data(), &m1, kPin) == kExisting);  // pin the oldest entry
  EXPECT(m1.data == pinned_data);
  cache.Get(d2.data(), &m2);
  cache.Get(d3.data(), &m3);                             // 1 is least recently used again
  cache.Get(d4.data(), &m4);                             // ejects 2, not the pinned 1
  EXPECT(cache.Get(d1.data(), &m1) == kExisting);
  EXPECT(cache.Get(d3.data(), &m3) == kExisting);
  EXPECT(cache.Get(d2.data(), &m2) == kInserted);        // ejects 4 (oldest unpinned)
  EXPECT(cache.Get(d1.data(), &m1) == kExisting && m1.data == pinned_data);
  // With only pinned entries left ejection stops, as it does on an empty cache.
  PrepackedCache small(CountingAlloc, CountingFree, 300);
  PackedMatrix a = Dummy(false, 10, 20), b = a;
  small.Get(d1.data(), &a);
  EXPECT(small.Get(d1.data(), &a, kPin) == kExisting);
  EXPECT(small.Get(d5.data(), &b) == kInserted);
  EXPECT(small.MatrixCount() == 2);
  small.Clear();  // Clear releases pinned entries too
  EXPECT(small.MatrixCount() == 0 && small.BuffersBytes() == 0);
}

static void TestOversizeEntryIsKept() {
  PrepackedCache cache(CountingAlloc, CountingFree, 100);
  std::vector<std::uint8_t> d1(200);
  PackedMatrix m1 = Dummy(false, 10, 20);
  EXPECT(cache.Get(d1.data(), &m1) == kInserted);  // 280 > 100: ejection stops at empty
  EXPECT(cache.MatrixCount() == 1);
  EXPECT(cache.Get(d1.data(), &m1) == kExisting);
}

static void TestDistinguishSubtlyDifferentMatrices() {
  PrepackedCache cache(CountingAlloc, CountingFree);
  EXPECT(cache.MaxBuffersBytes() == (1 << 28));
  std::vector<std::uint8_t> data(10 * 20 + 1);
  PackedMatrix m = Dummy(false, 10, 20);
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  EXPECT(cache.Get(data.data() + 1, &m) == kInserted);  // other source pointer
  m.layout.rows = 9;
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  m.layout.cols = 19;
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  m.layout.order = 1;
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  m.layout.kernel_rows = 2;
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  m.layout.kernel_cols = 2;
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  m.layout.kernel_order = 1;
  EXPECT(cache.Get(data.data(), &m) == kInserted);
  m.zero_point = 3;
  EXPECT(cache.Get(data.data(), &m) == kInserted);  // other zero point
  EXPECT(cache.MatrixCount() == 9);
  cache.Clear();
  EXPECT(cache.MatrixCount() == 0 && cache.BuffersBytes() == 0);
}

// A caller that got a new entry and then could not fill it (staging or the
// pack launch failed) erases it: the next Get for the same key must insert
// again instead of returning buffers that were never packed, and the byte and
// allocation accounting must be as if the entry had never existed.
static void TestEraseAfterFailedPack() {
  const int live_before = g_live_allocations;
  {
    PrepackedCache cache(CountingAlloc, CountingFree, 1000);
    std::vector<std::uint8_t> d1(200), d2(15);
    PackedMatrix m1 = Dummy(false, 10, 20), m2 = Dummy(false, 5, 3);
    EXPECT(cache.Get(d1.data(), &m1) == kInserted);
    EXPECT(cache.Get(d2.data(), &m2) == kInserted);
    EXPECT(cache.BuffersBytes() == 307 && cache.MatrixCount() == 2);
    EXPECT(cache.HasSource(d1.data()) && cache.HasSource(d2.data()));
    EXPECT(cache.Erase(d1.data(), m1));
    EXPECT(!cache.HasSource(d1.data()) && cache.HasSource(d2.data()));
    EXPECT(cache.BuffersBytes() == 27 && cache.MatrixCount() == 1);
    EXPECT(g_live_allocations == live_before + 2);  // only m2's data and sums are left
    EXPECT(!cache.Erase(d1.data(), m1));            // already gone
    PackedMatrix again = Dummy(false, 10, 20);
    EXPECT(cache.Get(d1.data(), &again) == kInserted);  // not a hit on stale buffers
    EXPECT(cache.BuffersBytes() == 307 && cache.MatrixCount() == 2);
    // A key that differs only in the zero point is a different entry.
    PackedMatrix other = Dummy(false, 5, 3);
    other.zero_point = 1;
    EXPECT(!cache.Erase(d2.data(), other));
    EXPECT(cache.MatrixCount() == 2);
    // Lookup-only mode: a hit without the ejection mark, a miss without an insert.
    PackedMatrix probe = Dummy(false, 5, 3);
    EXPECT(cache.Get(d2.data(), &probe, PrepackedCache::Mode::kLookupOnly) == kExisting);
    EXPECT(probe.data == m2.data);
    PackedMatrix absent = Dummy(false, 7, 7);
    EXPECT(cache.Get(d2.data(), &absent, PrepackedCache::Mode::kLookupOnly) == PrepackedCache::Action::kMissing);
    EXPECT(absent.data == nullptr && cache.MatrixCount() == 2);
  }
  EXPECT(g_live_allocations == live_before);
}

int main() {
  TestEraseAfterFailedPack();
  TestBasic();
  TestBasicFloat();
  TestEjection();
  TestEjectionOrder();
  TestOversizeEntryIsKept();
  TestPinnedEntriesSurviveEjection();
  TestDistinguishSubtlyDifferentMatrices();
  EXPECT(g_live_allocations == 0);  // every cache freed what it allocated
  if (g_failures) {
    std::fprintf(stderr, "%d failure(s)\n", g_failures);
    return 1;
  }
  std::printf("prepacked_cache_test: all passed\n");
  return 0;
}
