// The dimensions of a tensor, held in place up to kInline of them. A request
// for a collective carries its tensor's shape through the op context, the
// readiness table and the wire format; with the dimensions in a std::vector
// each of those copies is a heap allocation per tensor per rank per step, and
// gradients have at most four dimensions. Shapes beyond kInline dimensions
// (the wire format allows 254) spill to a vector.
#ifndef MPIC_DIMS_H_
#define MPIC_DIMS_H_

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <utility>
#include <vector>

namespace mpic {

class Dims {
 public:
  static constexpr size_t kInline = 8;

  Dims() {}
  Dims(std::initializer_list<int64_t> l) { assign(l.begin(), l.end()); }
  Dims(const std::vector<int64_t>& v) { assign(v.data(), v.data() + v.size()); }  // NOLINT: implicit on purpose
  Dims(const int64_t* first, const int64_t* last) { assign(first, last); }
  Dims(const Dims&) = default;
  Dims& operator=(const Dims&) = default;
  // a moved-from Dims is empty
  Dims(Dims&& o) noexcept : n_(o.n_), heap_(std::move(o.heap_)) {
    std::copy(o.inline_, o.inline_ + kInline, inline_);
    o.clear();
  }
  Dims& operator=(Dims&& o) noexcept {
    if (this != &o) {
      n_ = o.n_;
      std::copy(o.inline_, o.inline_ + kInline, inline_);
      heap_ = std::move(o.heap_);
      o.clear();
    }
    return *this;
  }

  size_t size() const { return n_; }
  bool empty() const { return n_ == 0; }
  const int64_t* data() const { return n_ <= kInline ? inline_ : heap_.data(); }
  int64_t* data() { return n_ <= kInline ? inline_ : heap_.data(); }
  const int64_t* begin() const { return data(); }
  const int64_t* end() const { return data() + n_; }
  int64_t operator[](size_t i) const { return data()[i]; }
  int64_t& operator[](size_t i) { return data()[i]; }

  void clear() {
    n_ = 0;
    heap_.clear();
  }
  // Keeps the first min(size(), n) values; new ones are zero.
  void resize(size_t n) {
    if (n <= kInline) {
      if (n_ > kInline) {
        std::copy(heap_.begin(), heap_.begin() + static_cast<std::ptrdiff_t>(n), inline_);
        heap_.clear();
      } else if (n > n_) {
        std::fill(inline_ + n_, inline_ + n, 0);
      }
    } else {
      if (n_ <= kInline) heap_.assign(inline_, inline_ + n_);
      heap_.resize(n, 0);
    }
    n_ = n;
  }
  void push_back(int64_t v) {
    resize(n_ + 1);
    data()[n_ - 1] = v;
  }
  void assign(size_t n, int64_t v) {
    clear();
    resize(n);
    std::fill(data(), data() + n, v);
  }
  void assign(const int64_t* first, const int64_t* last) {
    clear();
    resize(static_cast<size_t>(last - first));
    std::copy(first, last, data());
  }

  bool operator==(const Dims& o) const { return n_ == o.n_ && std::equal(begin(), end(), o.begin()); }
  bool operator!=(const Dims& o) const { return !(*this == o); }

 private:
  size_t n_ = 0;
  int64_t inline_[kInline] = {0, 0, 0, 0, 0, 0, 0, 0};
  std::vector<int64_t> heap_;  // the dimensions when there are more than kInline
};

}  // namespace mpic
#endif  // MPIC_DIMS_H_
