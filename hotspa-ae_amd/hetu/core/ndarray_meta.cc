#include "hetu/core/ndarray_meta.h"

#include <algorithm>
#include <numeric>

namespace hetu {

int64_t NDArrayMeta::ParseAxis(int64_t axis, int64_t num_dim) {
  HT_ASSERT(axis >= -num_dim && axis < num_dim)
    << "Invalid dimension. Expected to be within [" << -num_dim << ", " << num_dim << "). Got " << axis << ".";
  return axis >= 0 ? axis : axis + num_dim;
}

// empty = all dims; negative axes wrap; result is sorted and de-duplicated
HTAxes NDArrayMeta::ParseAxes(const HTAxes axes, int64_t num_dim) {
  HTAxes ret;
  if (axes.empty()) {
    ret.resize(num_dim);
    std::iota(ret.begin(), ret.end(), 0);
    return ret;
  }
  ret.reserve(axes.size());
  for (auto a : axes) ret.push_back(ParseAxis(a, num_dim));
  std::sort(ret.begin(), ret.end());
  ret.erase(std::unique(ret.begin(), ret.end()), ret.end());
  return ret;
}

// keepdims: reduced extents become 1; otherwise they are dropped, and reducing
// every dimension gives shape {1}
HTShape NDArrayMeta::Reduce(const HTShape& shape, const HTAxes& axes, bool keepdims) {
  const int64_t num_dim = static_cast<int64_t>(shape.size());
  HTAxes parsed = ParseAxes(axes, num_dim);
  if (keepdims) {
    HTShape out = shape;
    for (auto a : parsed) out[a] = 1;
    return out;
  }
  if (static_cast<int64_t>(parsed.size()) == num_dim) return {1};
  HTShape out;
  for (int64_t i = 0; i < num_dim; ++i)
    if (!std::binary_search(parsed.begin(), parsed.end(), i)) out.push_back(shape[i]);
  return out;
}

HTShape NDArrayMeta::Broadcast(const HTShape& shape_a, const HTShape& shape_b) {
  const size_t na = shape_a.size(), nb = shape_b.size(), n = std::max(na, nb);
  HTShape out(n);
  for (size_t k = 0; k < n; ++k) {           // k counts from the last dimension
    const int64_t a = k < na ? shape_a[na - 1 - k] : 1;
    const int64_t b = k < nb ? shape_b[nb - 1 - k] : 1;
    if (a != b && a != 1 && b != 1) return HTShape();
    out[n - 1 - k] = std::max(a, b);
    if ((a == 0 || b == 0)) out[n - 1 - k] = 0;   // an empty extent stays empty
  }
  return out;
}

std::ostream& operator<<(std::ostream& os, const NDArrayMeta& meta) {
  return os << "{dtype=" << meta.dtype << ", device=" << meta.device << ", shape=" << meta.shape
            << ", stride=" << meta.stride << "}";
}

} // namespace hetu
