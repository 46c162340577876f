// argmax helpers (ginn/util/amax.h:28-66): of a host vector, of a whole tensor
// viewed as a flat vector, and along one axis of a tensor.  Device tensors are
// searched on the device; the first maximum wins, as std::max_element.
#ifndef GINN_UTIL_AMAX_H
#define GINN_UTIL_AMAX_H

#include <algorithm>
#include <vector>

#include <ginn/nonlin.h>
#include <ginn/tensor.h>

namespace ginn {

template <typename T>
size_t argmax(const std::vector<T>& v) {
  return static_cast<size_t>(std::max_element(v.begin(), v.end()) - v.begin());
}

// Positions of the maxima along axis `dim`: a tensor of the remaining axes.
template <typename Scalar>
Tensor<long long> argmax(const Tensor<Scalar>& t, Size dim) {
  Shape s = t.shape();
  GINN_ASSERT(dim >= 0 && dim < static_cast<Size>(s.size()), "Index dim is bigger than tensor rank!");
  GINN_ASSERT(s.size() <= 8, "Unsupported large rank!");
  size_t inner = 1, outer = 1;
  const size_t len = static_cast<size_t>(s[static_cast<size_t>(dim)]);
  for (Size a = 0; a < dim; ++a) inner *= static_cast<size_t>(s[static_cast<size_t>(a)]);
  for (size_t a = static_cast<size_t>(dim) + 1; a < s.size(); ++a) outer *= static_cast<size_t>(s[a]);
  s.erase(s.begin() + dim);
  Tensor<long long> out(t.dev(), s);
  if (t.dev()->kind() == GPU) {
    GINN_HIP_CALL(ginn_hip_argmax(internal::ctx_of(t), dtype_of<Scalar>(), inner, len, outer, t.data(), out.data()));
  } else {
    const Scalar* x = t.data();
    for (size_t ou = 0; ou < outer; ++ou)
      for (size_t in = 0; in < inner; ++in) {
        size_t best = 0;
        for (size_t l = 1; l < len; ++l)
          if (static_cast<float>(x[(ou * len + l) * inner + in]) > static_cast<float>(x[(ou * len + best) * inner + in]))
            best = l;
        out.v()[ou * inner + in] = static_cast<long long>(best);
      }
  }
  return out;
}

// Position of the maximum of the tensor viewed as a flat vector.
template <typename Scalar>
size_t argmax(const Tensor<Scalar>& t) {
  GINN_ASSERT(t.size() > 0, "argmax of an empty tensor");
  return static_cast<size_t>(argmax(t.reshaped({t.size()}), 0).item());
}

}  // namespace ginn

#endif  // GINN_UTIL_AMAX_H
