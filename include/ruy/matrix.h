// ruy::Matrix and friends for the gfx950 implementation: the same public
// surface as the reference's ruy/matrix.h (Order :29, Layout :32-50,
// CachePolicy :117-122, Matrix :132-167, MakeSimpleLayout :169-174,
// Offset/ElementPtr/Element :188-214), written for this library. A Matrix is a
// non-owning view; `data` may point to host or device memory.
#ifndef RUY_AMD_INCLUDE_RUY_MATRIX_H_
#define RUY_AMD_INCLUDE_RUY_MATRIX_H_

#include <cassert>
#include <cstddef>
#include <cstdint>
#include <type_traits>

namespace ruy {

enum class Order : std::uint8_t { kColMajor, kRowMajor };

enum class CachePolicy : std::uint8_t {
  kNeverCache,
  kCacheIfLargeSpeedup,
  kCacheIfSignificantSpeedup,
  kAlwaysCache,
};

// Shape of a matrix: rows x cols, the storage order and the stride, i.e. the
// distance in elements between the starts of consecutive columns (column-major)
// or rows (row-major).
class Layout final {
 public:
  int rows() const { return dims_[0]; }
  int cols() const { return dims_[1]; }
  int stride() const { return stride_; }
  Order order() const { return order_; }
  void set_rows(int v) { dims_[0] = v; }
  void set_cols(int v) { dims_[1] = v; }
  void set_stride(int v) { stride_ = v; }
  void set_order(Order v) { order_ = v; }

 private:
  int dims_[2] = {0, 0};
  int stride_ = 0;
  Order order_ = Order::kColMajor;
};

inline void MakeSimpleLayout(int rows, int cols, Order order, Layout* layout) {
  layout->set_rows(rows);
  layout->set_cols(cols);
  layout->set_order(order);
  layout->set_stride(order == Order::kRowMajor ? cols : rows);
}

// Element (row, col) lives `Offset` elements after the data pointer.
inline int Offset(const Layout& layout, int row, int col) {
  return layout.order() == Order::kColMajor ? row + col * layout.stride()
                                            : row * layout.stride() + col;
}

template <typename Scalar>
class Matrix final {
  static_assert(!std::is_const<Scalar>::value,
                "use Matrix<T> for inputs and outputs alike, never Matrix<const T>");

 public:
  // A pointer set from `const Scalar*` may only be read; asking for a mutable
  // pointer to it trips an assertion in debug builds.
  void set_data(Scalar* ptr) {
    data_ = ptr;
    writable_ = true;
  }
  void set_data(const Scalar* ptr) {
    data_ = ptr;
    writable_ = false;
  }
  void set_data(std::nullptr_t) { data_ = nullptr; }
  const Scalar* data() const { return data_; }
  Scalar* data() {
    assert(writable_);
    return const_cast<Scalar*>(data_);
  }

  const Layout& layout() const { return layout_; }
  Layout* mutable_layout() { return &layout_; }
  Scalar zero_point() const { return zero_point_; }
  void set_zero_point(Scalar v) { zero_point_ = v; }
  CachePolicy cache_policy() const { return cache_policy_; }
  void set_cache_policy(CachePolicy v) { cache_policy_ = v; }

 private:
  const Scalar* data_ = nullptr;
  bool writable_ = true;
  Layout layout_;
  Scalar zero_point_ = 0;
  // Anything but kNeverCache promises that equal pointers mean equal contents,
  // which lets the library keep a packed, device-resident copy between calls.
  CachePolicy cache_policy_ = CachePolicy::kNeverCache;
};

template <typename Scalar>
const Scalar* ElementPtr(const Matrix<Scalar>& m, int row, int col) {
  return m.data() + Offset(m.layout(), row, col);
}
template <typename Scalar>
Scalar* ElementPtr(Matrix<Scalar>* m, int row, int col) {
  return m->data() + Offset(m->layout(), row, col);
}
template <typename Scalar>
Scalar Element(const Matrix<Scalar>& m, int row, int col) {
  return *ElementPtr(m, row, col);
}

// Prints a host-resident matrix, one row per line.
template <typename StreamType, typename Scalar>
StreamType& operator<<(StreamType& stream, const Matrix<Scalar>& m) {
  for (int r = 0; r < m.layout().rows(); ++r) {
    for (int c = 0; c < m.layout().cols(); ++c) stream << static_cast<double>(Element(m, r, c)) << " ";
    stream << "\n";
  }
  return stream;
}

}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_MATRIX_H_
