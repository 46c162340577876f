// Nested brace lists as tensor literals: NestedInitList<2, Real> is what
// `{{1, 2, 3}, {4, 5, 6}}` converts to, outermost list = dimension 0, so the
// literal reads like the matrix it denotes (ginn/util/util.h:247-299).
#ifndef GINN_UTIL_UTIL_H
#define GINN_UTIL_UTIL_H

#include <vector>

#include <ginn/except.h>

namespace ginn {

template <int Rank, typename T>
struct NestedInitListImpl {
  using type = std::vector<typename NestedInitListImpl<Rank - 1, T>::type>;
};
template <typename T>
struct NestedInitListImpl<0, T> {
  using type = T;
};
template <int Rank, typename T>
using NestedInitList = typename NestedInitListImpl<Rank, T>::type;

// Extents of a nested list; every inner list of one level must have the length of the first.
template <typename Int, int Rank, typename Scalar>
std::vector<Int> shape_of(const NestedInitList<Rank, Scalar>& list) {
  std::vector<Int> shape;
  if constexpr (Rank >= 1) {
    shape.push_back(static_cast<Int>(list.size()));
    if constexpr (Rank >= 2) {
      for (const auto& inner : list)
        GINN_ASSERT(inner.size() == list.front().size(), "Inner lists have size mismatch!");
      if (!list.empty()) {
        const auto rest = shape_of<Int, Rank - 1, Scalar>(list.front());
        shape.insert(shape.end(), rest.begin(), rest.end());
      } else {
        shape.resize(static_cast<size_t>(Rank), 0);
      }
    }
  }
  return shape;
}

// Writes list[i0][i1]...[i_{Rank-1}] to dst[i0 + n0 (i1 + n1 (...))]: the column-major
// position of element (i0, i1, ...).  `stride` is the distance of this level's index.
template <int Rank, typename Scalar, typename RhsScalar, typename Int>
void store_nested(const NestedInitList<Rank, RhsScalar>& list, Scalar* dst, const std::vector<Int>& shape,
                  size_t level = 0, size_t stride = 1) {
  if constexpr (Rank == 0) {
    *dst = Scalar(list);
  } else {
    size_t i = 0;
    for (const auto& inner : list) {
      store_nested<Rank - 1, Scalar, RhsScalar, Int>(inner, dst + i * stride, shape, level + 1,
                                                     stride * static_cast<size_t>(shape[level]));
      ++i;
    }
  }
}

}  // namespace ginn

#endif  // GINN_UTIL_UTIL_H
