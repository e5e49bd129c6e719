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

std::ostream& operator<<(std::ostream& os, const NDArrayMeta& meta) {
  return os << "{dtype=" << meta.dtype << ", device=" << meta.device << ", shape=" << meta.shape
            << ", stride=" << meta.stride << "}";
}

} // namespace hetu
