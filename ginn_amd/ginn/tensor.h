// Column-major tensor of the host layer.
//
// Same object model as ginn/tensor.h:64-565: {device, shape, data pointer,
// owns-memory flag}; dimension 0 is the fastest; rank-N tensors are viewed as
// matrices by folding trailing dimensions into columns (reduce()).  There are
// no Eigen views: element access on host tensors goes through v(), and device
// tensors are only touched by libginn_hip.so.
#ifndef GINN_TENSOR_H
#define GINN_TENSOR_H

#include <initializer_list>
#include <istream>
#include <numeric>
#include <ostream>
#include <type_traits>
#include <utility>

#include <ginn/dev.h>
#include <ginn/util/util.h>

namespace ginn {

template <typename ScalarType = Real>
class Tensor {
 public:
  using Scalar = ScalarType;

 private:
  DevPtr dev_ = nullptr;
  Shape shape_ = {0};
  Scalar* data_ = nullptr;
  bool owns_mem_ = true;

  void allocate(Size n) {
    GINN_ASSERT(data_ == nullptr);
    GINN_ASSERT(owns_mem_);
    if (n > 0) data_ = static_cast<Scalar*>(dev_->alloc(static_cast<size_t>(n) * sizeof(Scalar)));
  }
  void reallocate(Size n) {
    GINN_ASSERT(owns_mem_);
    if (n > 0) {
      data_ = static_cast<Scalar*>(dev_->realloc(data_, static_cast<size_t>(n) * sizeof(Scalar)));
    } else {
      release();
    }
  }
  void release() {
    GINN_ASSERT(owns_mem_);
    if (size() > 0) dev_->free(data_);
    data_ = nullptr;
  }
  void copy_from(const DevPtr& from, Scalar* src, Size n) {
    dev_->copy(*from, data_, src, static_cast<size_t>(n) * sizeof(Scalar));
  }

  ginn_hip_ctx* ctx() const { return hip_ctx(static_cast<int>(dev_->id().idx)); }

 public:
  const DevPtr& dev() const { return dev_; }
  const Shape& shape() const { return shape_; }
  Scalar* data() { return data_; }
  const Scalar* data() const { return data_; }

  static Size size(const Shape& shape) {
    Size n = 1;
    for (Size d : shape) n *= d;
    return n;
  }
  Size size() const { return size(shape_); }

  // Fold to `dim` dimensions: the last kept one absorbs all trailing ones;
  // shorter shapes are padded with 1 (ginn/tensor.h:268-282).
  static Shape reduce(const Shape& shape, Size dim) {
    const Size rank = static_cast<Size>(shape.size());
    if (dim < rank) {
      Shape out(shape.begin(), shape.begin() + dim);
      for (Size i = dim; i < rank; ++i) out[dim - 1] *= shape[i];
      return out;
    }
    Shape out(shape);
    out.resize(static_cast<size_t>(dim), 1);
    return out;
  }
  Shape shape2() const { return reduce(shape_, 2); }
  // Extents of the rank-2 fold, without building it.
  Size rows() const { return shape_.empty() ? 1 : shape_[0]; }
  Size cols() const {
    Size c = 1;
    for (size_t i = 1; i < shape_.size(); ++i) c *= shape_[i];
    return c;
  }

  // ---- construction -------------------------------------------------------
  Tensor(DevPtr dev = cpu()) : dev_(std::move(dev)) {}
  Tensor(DevPtr dev, Shape shape) : dev_(std::move(dev)), shape_(std::move(shape)) { allocate(size()); }
  Tensor(DevPtr dev, Shape shape, Scalar val) : Tensor(std::move(dev), std::move(shape)) { fill(val); }
  Tensor(Shape shape) : Tensor(cpu(), std::move(shape)) {}
  Tensor(Shape shape, const std::vector<Scalar>& val) : Tensor(std::move(shape)) {
    GINN_ASSERT(size() == static_cast<Size>(val.size()),
                "Size of Shape (" + std::to_string(size()) + ") does not match size of values (" +
                    std::to_string(val.size()) + ")!");
    std::copy(val.begin(), val.end(), data_);
  }
  Tensor(DevPtr dev, Shape shape, const std::vector<Scalar>& val) : Tensor(std::move(shape), val) {
    move_to(dev);
  }

  // Tensor literals: Tensor<Real>(NestedInitList<2, Real>{{1, 2, 3}, {4, 5, 6}}) is 2 x 3
  // (ginn/tensor.h:178-188).
  template <int Rank>
  Tensor(DevPtr dev, NestedInitList<Rank, Scalar> val) : dev_(std::move(dev)) {
    set<Rank>(val);
  }
  template <int Rank>
  Tensor(NestedInitList<Rank, Scalar> val) : dev_(cpu()) {
    set<Rank>(val);
  }

  Tensor(const Tensor& other) : dev_(other.dev_), shape_(other.shape_) {
    allocate(size());
    copy_from(other.dev_, other.data_, size());
  }
  Tensor(Tensor&& other) noexcept
      : dev_(other.dev_), shape_(other.shape_), data_(other.data_), owns_mem_(other.owns_mem_) {
    other.data_ = nullptr;
    other.shape_ = {0};
  }
  // Copy onto another device.
  Tensor(DevPtr dev, const Tensor& other) : dev_(std::move(dev)), shape_(other.shape_) {
    allocate(size());
    copy_from(other.dev_, other.data_, size());
  }
  ~Tensor() {
    if (owns_mem_ && data_) {
      try {
        release();
      } catch (...) {
      }
    }
  }

  // Assignment keeps the destination's device (ginn/tensor.h:209-228).
  Tensor& operator=(const Tensor& other) {
    if (this == &other) return *this;
    resize(other.shape_);
    copy_from(other.dev_, other.data_, size());
    return *this;
  }
  Tensor& operator=(Tensor&& other) {
    if (dev_ == other.dev_ && owns_mem_) {
      release();
      shape_ = other.shape_;
      data_ = other.data_;
      owns_mem_ = other.owns_mem_;
      other.data_ = nullptr;
      other.shape_ = {0};
    } else {
      *this = static_cast<const Tensor&>(other);
    }
    return *this;
  }

  // ---- moving between devices --------------------------------------------
  Tensor& move_to(const DevPtr& to) {
    GINN_ASSERT(owns_mem_);
    if (dev_ == to) return *this;
    Tensor from(dev_);
    from.data_ = data_;
    from.shape_ = shape_;  // frees the old storage when `from` dies
    dev_ = to;
    data_ = nullptr;
    if (size() > 0) {
      allocate(size());
      copy_from(from.dev_, from.data_, size());
    }
    return *this;
  }
  Tensor copy_to(const DevPtr& to) const { return Tensor(to, *this); }
  Tensor maybe_copy_to(const DevPtr& to) {
    if (dev_->id() == to->id()) return Tensor().map(*this);
    return copy_to(to);
  }

  // ---- shape --------------------------------------------------------------
  // Storage is reallocated only when the element count changes; device
  // reallocation discards the contents (ginn/tensor.h:247-256).
  void resize(const Shape& shape) {
    if (size() != size(shape)) {
      if (size() == 0) {
        shape_ = {0};
        allocate(size(shape));
      } else {
        reallocate(size(shape));
      }
    }
    if (shape_ != shape) shape_ = shape;
  }
  // resize({rows, cols}) that builds no Shape when nothing changes.
  void resize(Size rows, Size cols) {
    if (shape_.size() == 2 && shape_[0] == rows && shape_[1] == cols) return;
    resize(Shape{rows, cols});
  }

  // Non-owning views (ginn/tensor.h:286-325).
  Tensor& map(Tensor& other, const Shape& shape) {
    GINN_ASSERT(size(shape) == size(other.shape_));
    if (owns_mem_ && data_) release();
    dev_ = other.dev_;
    data_ = other.data_;
    shape_ = shape;
    owns_mem_ = false;
    return *this;
  }
  Tensor& map(Tensor& other) { return map(other, other.shape_); }
  Tensor& map(Tensor& other, Shape shape, Size offset) {
    GINN_ASSERT(size(shape) + offset <= size(other.shape_));
    if (owns_mem_ && data_) release();
    dev_ = other.dev_;
    data_ = other.data_ + offset;
    shape_ = std::move(shape);
    owns_mem_ = false;
    return *this;
  }
  Tensor reshaped(const Shape& shape) {
    Tensor t;
    t.map(*this, shape);
    return t;
  }
  const Tensor reshaped(const Shape& shape) const {
    Tensor t;
    t.map(const_cast<Tensor&>(*this), shape);
    return t;
  }

  // ---- host access ----------------------------------------------------------
  // Flat element access; host tensors only (m() / v() of the reference throw
  // on device tensors too, ginn/tensor.h:327-329).
  Scalar* v() {
    GINN_ASSERT(dev_->kind() == CPU, "v() can only be invoked on Cpu tensors!");
    return data_;
  }
  const Scalar* v() const {
    GINN_ASSERT(dev_->kind() == CPU, "v() can only be invoked on Cpu tensors!");
    return data_;
  }
  // Element (row, col) of the rank-2 fold.
  Scalar& at(Size r, Size c) { return v()[c * rows() + r]; }

  // Copy of the elements in storage order, from any device.
  std::vector<Scalar> vector() const {
    std::vector<Scalar> out(static_cast<size_t>(size()));
    if (size() == 0) return out;
    if constexpr (std::is_same_v<Scalar, bool>) {  // std::vector<bool> is packed: go through bytes
      std::vector<unsigned char> bytes(out.size());
      cpu()->copy(*dev_, bytes.data(), data_, bytes.size());
      for (size_t i = 0; i < out.size(); ++i) out[i] = bytes[i] != 0;
    } else {
      cpu()->copy(*dev_, out.data(), data_, out.size() * sizeof(Scalar));
    }
    return out;
  }
  Scalar item() const {
    GINN_ASSERT(size() == 1, "item() can be invoked on size 1 tensors!");
    return vector()[0];
  }

  // ---- filling --------------------------------------------------------------
  void fill(Scalar val) {
    if (size() == 0) return;
    if (dev_->kind() == CPU) {
      std::fill(data_, data_ + size(), val);
    } else if (dev_->kind() == GPU) {
      if constexpr (is_floating_point_v<Scalar>) {
        GINN_HIP_CALL(ginn_hip_fill(ctx(), dtype_of<Scalar>(), data_, static_cast<size_t>(size()),
                                    static_cast<float>(val)));
      } else {
        set(std::vector<Scalar>(static_cast<size_t>(size()), val));
      }
    } else {
      GINN_THROW("Unexpected device in Tensor::fill!");
    }
  }
  void set_zero() {
    if (size() == 0) return;
    if (dev_->kind() == CPU) {
      std::memset(static_cast<void*>(data_), 0, static_cast<size_t>(size()) * sizeof(Scalar));
    } else {
      GINN_HIP_CALL(ginn_hip_memset(ctx(), data_, 0, static_cast<size_t>(size()) * sizeof(Scalar)));
    }
  }
  void set_ones() { fill(Scalar(1)); }

  // Uniform in [-1, 1) (ginn/tensor.h:446-470).  The reference's streams come
  // from Eigen (host) and cuRAND (device); here a host tensor draws from a
  // SplitMix64 counter stream and a floating-point device tensor is filled on
  // the device from (seed, element index), the seed advancing per call; other
  // device tensors are drawn on the host and copied.
  static uint64_t& random_state() {
    static uint64_t s = 0x9e3779b97f4a7c15ull;
    return s;
  }
  static void seed(uint64_t s) { random_state() = s * 0x9e3779b97f4a7c15ull + 0x632be59bd9b4e019ull; }
  void set_random() {
    if (size() == 0) return;
    if constexpr (is_floating_point_v<Scalar>) {
      if (dev_->kind() == GPU) {
        uint64_t& s = random_state();
        s += 0x9e3779b97f4a7c15ull;
        GINN_HIP_CALL(ginn_hip_fill_uniform(ctx(), dtype_of<Scalar>(), static_cast<size_t>(size()), s, -1.f, 1.f,
                                            data_));
        return;
      }
    }
    std::vector<Scalar> host(static_cast<size_t>(size()));
    uint64_t& s = random_state();
    for (size_t i = 0; i < host.size(); ++i) {
      s += 0x9e3779b97f4a7c15ull;
      uint64_t z = s;
      z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
      z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
      z ^= z >> 31;
      const double u = static_cast<double>(z >> 11) * (1.0 / 9007199254740992.0);
      host[i] = Scalar(static_cast<float>(2.0 * u - 1.0));
    }
    set(host);
  }

  // Values in storage (column-major) order.
  void set(const std::vector<Scalar>& vals) {
    GINN_ASSERT(static_cast<Size>(vals.size()) == size());
    if (size() == 0) return;
    if constexpr (std::is_same_v<Scalar, bool>) {
      std::vector<unsigned char> bytes(vals.size());
      for (size_t i = 0; i < vals.size(); ++i) bytes[i] = vals[i] ? 1 : 0;
      dev_->copy(*cpu(), data_, bytes.data(), bytes.size());
    } else {
      dev_->copy(*cpu(), data_, const_cast<Scalar*>(vals.data()), vals.size() * sizeof(Scalar));
    }
  }

  // The first min(size(), vals.size()) elements, converted (ginn/tensor.h:472-489).
  template <typename RhsScalar, typename = std::enable_if_t<!std::is_same_v<RhsScalar, Scalar>>>
  void set(const std::vector<RhsScalar>& vals) {
    std::vector<Scalar> all = vector();
    for (size_t i = 0; i < std::min(all.size(), vals.size()); ++i) all[i] = convert<Scalar>(vals[i]);
    set(all);
  }
  // set(1, 2, 3): values in storage order (ginn/tensor.h:491-494).
  template <typename First, typename... Rest,
            typename = std::enable_if_t<std::is_arithmetic_v<First> || std::is_same_v<First, Scalar>>>
  void set(const First& first, const Rest&... rest) {
    std::vector<Scalar> all = vector();
    const std::vector<Scalar> vals{convert<Scalar>(first), convert<Scalar>(rest)...};
    for (size_t i = 0; i < std::min(all.size(), vals.size()); ++i) all[i] = vals[i];
    set(all);
  }
  // Resizes to the extents of the nested list and takes its values; element
  // (i, j, ...) is val[i][j]... (ginn/tensor.h:496-510).
  template <int Rank, typename RhsScalar = Scalar>
  void set(NestedInitList<Rank, RhsScalar> val) {
    const Shape shape = shape_of<Size, Rank, RhsScalar>(val);
    resize(shape);
    std::vector<Scalar> host(static_cast<size_t>(size()));
    if (size() > 0) store_nested<Rank, Scalar, RhsScalar, Size>(val, host.data(), shape);
    set(host);
  }

  template <typename To, typename From>
  static To convert(const From& x) {
    if constexpr (is_floating_point_v<To> && !std::is_same_v<To, float>) return To(static_cast<float>(x));
    else if constexpr (is_floating_point_v<From>) return static_cast<To>(static_cast<float>(x));
    else return static_cast<To>(x);
  }

  // this += other, elementwise, same device.
  Tensor& operator+=(const Tensor& other) {
    GINN_ASSERT(size() == other.size());
    if (size() == 0) return *this;
    if (dev_->kind() == GPU) {
      if constexpr (is_floating_point_v<Scalar>) {
        const void* src = other.data_;
        GINN_HIP_CALL(ginn_hip_add_n(ctx(), dtype_of<Scalar>(), static_cast<size_t>(size()), 1, &src, data_, 1));
      } else {
        GINN_THROW("+= on device tensors exists for floating point scalars only");
      }
    } else {
      for (Size i = 0; i < size(); ++i) data_[i] = Scalar(data_[i] + other.data_[i]);
    }
    return *this;
  }

  // Element type conversion, staged through the host.
  template <typename Other>
  Tensor<Other> cast() const {
    const std::vector<Scalar> src = vector();
    std::vector<Other> dst(src.size());
    for (size_t i = 0; i < src.size(); ++i) {
      if constexpr (is_floating_point_v<Scalar> || is_floating_point_v<Other>)
        dst[i] = Other(static_cast<float>(src[i]));
      else
        dst[i] = static_cast<Other>(src[i]);
    }
    Tensor<Other> out(dev_, shape_);
    out.set(dst);
    return out;
  }

  // Text form of ginn/tensor.h:527-564: the rank, the dimensions (each followed
  // by a blank), the elements in storage order separated by blanks, one line
  // each, at the stream's own precision.  A device tensor goes through the host.
  void save(std::ostream& out) const {
    out << shape_.size() << std::endl;
    for (Size dim : shape_) out << dim << " ";
    out << std::endl;
    const std::vector<Scalar> vals = vector();
    for (size_t i = 0; i < vals.size(); ++i) {
      if (i > 0) out << " ";
      if constexpr (is_floating_point_v<Scalar>) out << static_cast<float>(vals[i]);
      else out << vals[i];
    }
    out << std::endl;
  }

  // Reads what save() wrote: resizes to the stored shape; elements are parsed
  // as doubles and converted, and the element line has to end right after the
  // last one, as in the reference.
  void load(std::istream& in) {
    Size r = 0;
    in >> r;
    GINN_ASSERT(in.good() && r >= 0, "Tensor::load: no rank");
    Shape new_shape(static_cast<size_t>(r));
    for (Size& dim : new_shape) in >> dim;
    resize(new_shape);
    std::vector<Scalar> vals(static_cast<size_t>(size()));
    for (size_t i = 0; i < vals.size(); ++i) {
      double val = 0;
      in >> val;
      if constexpr (is_floating_point_v<Scalar>) vals[i] = Scalar(static_cast<float>(val));
      else vals[i] = static_cast<Scalar>(val);
    }
    GINN_ASSERT(!in.fail(), "Tensor::load: malformed or truncated element list");
    char end_of_line = 0;
    in.get(end_of_line);
    GINN_ASSERT(end_of_line == '\n');
    set(vals);
  }

  bool operator==(const Tensor& other) const {
    if (shape_ != other.shape_) return false;
    const auto a = vector(), b = other.vector();
    for (size_t i = 0; i < a.size(); ++i)
      if (!(static_cast<float>(a[i]) == static_cast<float>(b[i]))) return false;
    return true;
  }
};

}  // namespace ginn

#endif  // GINN_TENSOR_H
