// Devices of the host layer.
//
// Same contract as ginn/dev.h:55-75: a Device allocates, frees and copies
// memory, has a kind (CPU / GPU / NULL_DEV), an id and a precedence used by
// best_dev().  A GPU index has one context of libginn_hip.so (device index,
// stream, workspace) in place of the reference's stream + BLAS handle pair
// (ginn/dev.h:149-199), shared by all device objects of that index; PreallocGpuDevice is a bump arena in device memory
// (ginn/dev.h:214-254).  Only the GPU kinds compute; CpuDevice holds host
// staging copies of tensors.
#ifndef GINN_DEV_H
#define GINN_DEV_H

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include <ginn/def.h>

namespace ginn {

// Number of usable GPUs (ginn/dev.h:38-46).
inline int gpus() {
  int n = 0;
  if (ginn_hip_device_count(&n) != 0) return 0;
  return n;
}

enum DeviceKind { CPU, GPU, NULL_DEV };

struct DeviceId {
  const DeviceKind kind;
  const size_t idx = 0;
  bool operator==(const DeviceId& o) const { return kind == o.kind && idx == o.idx; }
};

class Device {
 public:
  virtual ~Device() = default;
  virtual void* alloc(size_t size) = 0;
  virtual void* realloc(void* data, size_t size) = 0;
  virtual void free(void* data) = 0;
  virtual DeviceKind kind() const = 0;
  virtual DeviceId id() const = 0;
  virtual short precedence() const { return 0; }

  // Copies `size` bytes from `other_data` on `other` into `data` on this device.
  void copy(const Device& other, void* data, void* other_data, size_t size);
};

using DevPtr = std::shared_ptr<Device>;

class NullDevice : public Device {
 public:
  void* alloc(size_t) override { return nullptr; }
  void* realloc(void*, size_t) override { return nullptr; }
  void free(void*) override {}
  DeviceKind kind() const override { return NULL_DEV; }
  DeviceId id() const override { return {NULL_DEV, 0}; }
  short precedence() const override { return -1; }
};

inline auto null_dev() {
  static auto dev = std::make_shared<NullDevice>();
  return dev;
}

class CpuDevice : public Device {
 public:
  void* alloc(size_t size) override { return std::malloc(size); }
  void* realloc(void* data, size_t size) override { return std::realloc(data, size); }
  void free(void* data) override { std::free(data); }
  DeviceKind kind() const override { return CPU; }
  DeviceId id() const override { return {CPU, 0}; }
};

inline auto Cpu() { return std::make_shared<CpuDevice>(); }
inline auto& cpu() {
  static auto dev = Cpu();
  return dev;
}

// Bump arena in host memory (ginn/dev.h:114-142); an allocation has to leave
// at least one byte free, as in the reference.
class PreallocCpuDevice : public Device {
  std::vector<unsigned char> storage_;
  size_t used_ = 0;

 public:
  explicit PreallocCpuDevice(size_t size) : storage_(size) {}
  void* alloc(size_t size) override {
    GINN_ASSERT(used_ + size < storage_.size(),
                "Prealloc device out of memory! Used: " + std::to_string(used_) +
                    " Attempted to allocate: " + std::to_string(size));
    void* p = storage_.data() + used_;
    used_ += size;
    return p;
  }
  void* realloc(void*, size_t) override { return nullptr; }
  void free(void*) override {}
  DeviceKind kind() const override { return CPU; }
  DeviceId id() const override { return {CPU, 0}; }
  short precedence() const override { return 1; }
  void clear() { used_ = 0; }
  size_t used() const { return used_; }
  size_t size() const { return storage_.size(); }
};

inline auto PreallocCpu(size_t size) { return std::make_shared<PreallocCpuDevice>(size); }

namespace internal {
// One context (stream, workspace) per GPU index for the whole process: every
// device object of that index -- gpu(idx), a Gpu(idx) the caller made, a
// PreallocGpu arena -- enqueues on it, so synchronising any of them waits for
// the work on that GPU's tensors.  Created on first use and kept until the
// process ends: tensors in static storage may free their memory later than
// any static destructor of this header would run.
class ContextTable {
  std::vector<ginn_hip_ctx*> ctx_;
  // A second context (stream, workspace) per GPU for work that nothing on the
  // first one's stream waits for (ginn_hip_ctx_wait_for); no memory of tensors
  // is ever allocated on it.
  std::vector<ginn_hip_ctx*> beside_;
  std::mutex mutex_;

 public:
  ContextTable() : ctx_(static_cast<size_t>(std::max(gpus(), 0)), nullptr), beside_(ctx_.size(), nullptr) {}
  ContextTable(const ContextTable&) = delete;
  ginn_hip_ctx*& at(size_t idx) {
    GINN_ASSERT(idx < ctx_.size(),
                "no GPU with index " + std::to_string(idx) + " (" + std::to_string(ctx_.size()) + " visible)");
    // Created once, whichever host threads ask first (the reference's multi-threaded
    // training makes its devices per thread, examples/mnist-dp.cu:158-172).
    if (!__atomic_load_n(&ctx_[idx], __ATOMIC_ACQUIRE)) {
      std::lock_guard<std::mutex> lock(mutex_);
      if (!ctx_[idx]) {
        ginn_hip_ctx* made = nullptr;
        GINN_HIP_CALL(ginn_hip_ctx_create(static_cast<int>(idx), 0, &made));
        __atomic_store_n(&ctx_[idx], made, __ATOMIC_RELEASE);
      }
    }
    return ctx_[idx];
  }
  ginn_hip_ctx* beside(size_t idx) {
    GINN_ASSERT(idx < beside_.size());
    std::lock_guard<std::mutex> lock(mutex_);
    if (!beside_[idx]) GINN_HIP_CALL(ginn_hip_ctx_create(static_cast<int>(idx), 0, &beside_[idx]));
    return beside_[idx];
  }
};
inline ContextTable& contexts() {
  static ContextTable* table = new ContextTable;
  return *table;
}
}  // namespace internal

// One physical GPU.  Allocations are plain device allocations; kernels, copies
// and synchronisation go to the GPU's process-wide context.
class GpuDevice : public Device {
  const size_t id_;
  ginn_hip_ctx*& ctx_;

 public:
  explicit GpuDevice(size_t id = 0) : id_(id), ctx_(internal::contexts().at(id)) {}
  GpuDevice(const GpuDevice&) = delete;
  GpuDevice& operator=(const GpuDevice&) = delete;

  void* alloc(size_t size) override {
    void* p = nullptr;
    GINN_HIP_CALL(ginn_hip_malloc(ctx_, size, &p));
    return p;
  }
  // As in the reference (ginn/dev.h:168-171) contents are not preserved.
  void* realloc(void* data, size_t size) override {
    free(data);
    return alloc(size);
  }
  void free(void* data) override { GINN_HIP_CALL(ginn_hip_free(ctx_, data)); }
  DeviceKind kind() const override { return GPU; }
  DeviceId id() const override { return {GPU, id_}; }

  ginn_hip_ctx* ctx() const { return ctx_; }
  // Context handle in the role of the reference's cublasHandle_t.
  ginn_hip_ctx*& handle() { return ctx_; }
  void* stream() const {
    void* s = nullptr;
    GINN_HIP_CALL(ginn_hip_ctx_stream(ctx_, &s));
    return s;
  }
  void synchronize() const { GINN_HIP_CALL(ginn_hip_sync(ctx_)); }
};

inline auto Gpu(size_t id) { return std::make_shared<GpuDevice>(id); }

// Process-wide device table, built on first use (ginn/dev.h:203-212).
inline auto& gpu(int idx = 0) {
  static std::vector<std::shared_ptr<GpuDevice>> devs = [] {
    std::vector<std::shared_ptr<GpuDevice>> v;
    const int n = gpus();
    for (int i = 0; i < n; ++i) v.push_back(Gpu(static_cast<size_t>(i)));
    return v;
  }();
  GINN_ASSERT(idx >= 0 && static_cast<size_t>(idx) < devs.size(),
              "gpu(" + std::to_string(idx) + "): no such device (" + std::to_string(devs.size()) + " visible)");
  return devs[static_cast<size_t>(idx)];
}

// The context that runs kernels for device index idx (role of cublas_handle(idx),
// ginn/dev.h:264).
inline ginn_hip_ctx* hip_ctx(int idx = 0) { return internal::contexts().at(static_cast<size_t>(idx)); }
inline ginn_hip_ctx*& cublas_handle(int idx = 0) { return internal::contexts().at(static_cast<size_t>(idx)); }

// Bump arena in device memory; kernels run on the context of gpu(id).
class PreallocGpuDevice : public Device {
  const size_t id_;
  ginn_hip_arena* arena_ = nullptr;

 public:
  // alignment = 1 is the reference's byte-exact bump (ginn/dev.h:236-248);
  // a larger power of two starts every block at a multiple of it.
  PreallocGpuDevice(size_t id, size_t size, size_t alignment = 1) : id_(id) {
    GINN_HIP_CALL(ginn_hip_arena_create(hip_ctx(static_cast<int>(id)), size, &arena_));
    if (alignment != 1) GINN_HIP_CALL(ginn_hip_arena_set_alignment(arena_, alignment));
  }
  explicit PreallocGpuDevice(size_t size) : PreallocGpuDevice(0, size) {}
  PreallocGpuDevice(const PreallocGpuDevice&) = delete;
  ~PreallocGpuDevice() override {
    if (arena_) ginn_hip_arena_destroy(arena_);
  }
  void* alloc(size_t size) override {
    void* p = nullptr;
    if (ginn_hip_arena_alloc(arena_, size, &p) != 0) GINN_THROW(ginn_hip_last_error());
    return p;
  }
  void* realloc(void*, size_t) override { return nullptr; }
  void free(void*) override {}
  DeviceKind kind() const override { return GPU; }
  DeviceId id() const override { return {GPU, id_}; }
  short precedence() const override { return 1; }
  void clear() { GINN_HIP_CALL(ginn_hip_arena_clear(arena_)); }
  size_t used() const {
    size_t b = 0;
    GINN_HIP_CALL(ginn_hip_arena_used(arena_, &b));
    return b;
  }
  size_t size() const {
    size_t b = 0;
    GINN_HIP_CALL(ginn_hip_arena_size(arena_, &b));
    return b;
  }
};

inline auto PreallocGpu(size_t id, size_t size) { return std::make_shared<PreallocGpuDevice>(id, size); }
inline auto PreallocGpu(size_t size) { return std::make_shared<PreallocGpuDevice>(size); }
// Not in the reference: an arena whose blocks start at multiples of `alignment` bytes.
inline auto PreallocGpuAligned(size_t id, size_t size, size_t alignment) {
  return std::make_shared<PreallocGpuDevice>(id, size, alignment);
}

// Host <-> device and device <-> device transfers (ginn/dev.h:269-343).  One
// GPU per process in this build: a copy between two different GPU indices is
// refused instead of being staged through the host.
inline void Device::copy(const Device& other, void* data, void* other_data, size_t size) {
  if (size == 0) return;
  const DeviceKind to = kind(), from = other.kind();
  if (to == CPU && from == CPU) {
    std::memcpy(data, other_data, size);
  } else if (to == CPU && from == GPU) {
    GINN_HIP_CALL(ginn_hip_memcpy_d2h(hip_ctx(static_cast<int>(other.id().idx)), data, other_data, size));
  } else if (to == GPU && from == CPU) {
    ginn_hip_ctx* ctx = hip_ctx(static_cast<int>(id().idx));
    GINN_HIP_CALL(ginn_hip_memcpy_h2d(ctx, data, other_data, size));
    // The source may be a temporary of the caller: finish the copy before returning.
    GINN_HIP_CALL(ginn_hip_sync(ctx));
  } else if (to == GPU && from == GPU) {
    GINN_ASSERT(id().idx == other.id().idx, "copies between different GPUs are not part of this build");
    GINN_HIP_CALL(ginn_hip_memcpy_d2d(hip_ctx(static_cast<int>(id().idx)), data, other_data, size));
  } else {
    GINN_THROW("Unexpected device in Device::copy()!");
  }
}

// Device of highest precedence among the inputs (ginn/dev.h:346-359).
template <typename NodeType>
auto best_dev(const std::vector<NodeType>& ins) {
  GINN_ASSERT(!ins.empty());
  auto best = std::max_element(ins.begin(), ins.end(), [](const auto& a, const auto& b) {
    return a->dev()->precedence() < b->dev()->precedence();
  });
  return (*best)->dev();
}

}  // namespace ginn

#endif  // GINN_DEV_H
