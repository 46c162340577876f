// Nonlinearity operators (ginn/nonlin.h:42-300): y = f(x) and
// dx (+)= f'(x, y) * dy, evaluated by libginn_hip.so.  Each operator also
// reports its device code so that AffineNode can fuse it into the product's
// epilogue.
#ifndef GINN_NONLIN_H
#define GINN_NONLIN_H

#include <memory>

#include <ginn/prod.h>

namespace ginn {

namespace internal {
inline void require_gpu(const DevPtr& dev, const char* what) {
  GINN_ASSERT(dev->kind() == GPU, std::string(what) + ": this node computes on the HIP device only "
                                                      "(move the inputs with move_to(gpu()))");
}
template <typename Scalar>
ginn_hip_ctx* ctx_of(const Tensor<Scalar>& t) {
  return hip_ctx(static_cast<int>(t.dev()->id().idx));
}
}  // namespace internal

template <typename Scalar>
class NonlinOp {
 public:
  virtual ~NonlinOp() = default;
  virtual ginn_hip_act code() const = 0;
  virtual bool backward_requires_input() const { return true; }
  virtual bool is_identity() const { return false; }

  virtual void forward(Tensor<Scalar>& y, const Tensor<Scalar>& x) const {
    y.resize(x.shape());
    if (x.dev()->kind() == CPU) {  // ginn/nonlin.h:67-300 on the host
      host::nonlin_forward<Scalar>(code(), static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(), y.data());
      return;
    }
    internal::require_gpu(x.dev(), "NonlinOp::forward");
    GINN_HIP_CALL(ginn_hip_nonlin_fwd(internal::ctx_of(x), dtype_of<Scalar>(), code(),
                                      static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(),
                                      y.data()));
  }
  // x may be an empty tensor when backward_requires_input() is false.
  virtual void backward(Tensor<Scalar>& dx, const Tensor<Scalar>& dy, const Tensor<Scalar>& x,
                        const Tensor<Scalar>& y, bool accumulate) const {
    if (dy.dev()->kind() == CPU) {
      host::nonlin_backward<Scalar>(code(), static_cast<int>(dy.rows()), static_cast<int>(dy.cols()), dy.data(),
                                   x.size() > 0 ? x.data() : nullptr, y.size() > 0 ? y.data() : nullptr, dx.data(),
                                   accumulate);
      return;
    }
    internal::require_gpu(dy.dev(), "NonlinOp::backward");
    GINN_HIP_CALL(ginn_hip_nonlin_bwd(internal::ctx_of(dy), dtype_of<Scalar>(), code(),
                                      static_cast<int>(dy.rows()), static_cast<int>(dy.cols()), dy.data(),
                                      x.size() > 0 ? x.data() : nullptr, y.size() > 0 ? y.data() : nullptr,
                                      dx.data(), accumulate ? 1 : 0));
  }
  virtual std::unique_ptr<NonlinOp<Scalar>> copy() const = 0;
};

#define GINN_DEFINE_NONLIN(Name, Code, NeedsInput, Identity)                   \
  template <typename Scalar>                                                   \
  class Name##Op : public NonlinOp<Scalar> {                                   \
   public:                                                                     \
    ginn_hip_act code() const override { return Code; }                        \
    bool backward_requires_input() const override { return NeedsInput; }       \
    bool is_identity() const override { return Identity; }                     \
    std::unique_ptr<NonlinOp<Scalar>> copy() const override {                  \
      return std::make_unique<Name##Op<Scalar>>(*this);                        \
    }                                                                          \
  }

GINN_DEFINE_NONLIN(Identity, GINN_HIP_ACT_IDENTITY, false, true);
GINN_DEFINE_NONLIN(Tanh, GINN_HIP_ACT_TANH, false, false);
GINN_DEFINE_NONLIN(Relu, GINN_HIP_ACT_RELU, false, false);
GINN_DEFINE_NONLIN(Sigmoid, GINN_HIP_ACT_SIGMOID, false, false);
GINN_DEFINE_NONLIN(Softmax, GINN_HIP_ACT_SOFTMAX, true, false);
GINN_DEFINE_NONLIN(Log, GINN_HIP_ACT_LOG, true, false);
GINN_DEFINE_NONLIN(Sqrt, GINN_HIP_ACT_SQRT, false, false);
GINN_DEFINE_NONLIN(Gelu, GINN_HIP_ACT_GELU, true, false);
GINN_DEFINE_NONLIN(Gelu2, GINN_HIP_ACT_GELU2, true, false);

#undef GINN_DEFINE_NONLIN

}  // namespace ginn

#endif  // GINN_NONLIN_H
