// Context, memory, arena and timing entry points of libginn_hip.so.
#include <cstring>
#include <new>
#include <string>

#include <algorithm>
#include <cstdlib>
#include <iterator>

#include <vector>

#include "common.h"

namespace ginn_hip {

namespace {
thread_local std::string g_last_error;
}

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

void clear_error() { g_last_error.clear(); }

namespace {

constexpr size_t kDefaultWorkspace = 64ull << 20;
constexpr size_t kHostStaging = 1ull << 20;

__global__ void fill_bytes_kernel(uint8_t* __restrict__ dst, uint32_t word,
                                  size_t bytes) {
  // Head and tail are written byte-wise, the 16-byte aligned body as uint4.
  const size_t tid = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
  size_t head = (16 - (addr & 15)) & 15;
  if (head > bytes) head = bytes;
  const size_t body = (bytes - head) / 16;
  const size_t tail_start = head + body * 16;
  const uint8_t b = static_cast<uint8_t>(word & 0xff);
  for (size_t i = tid; i < head; i += nthreads) dst[i] = b;
  uint4* body_ptr = reinterpret_cast<uint4*>(dst + head);
  const uint4 w4 = make_uint4(word, word, word, word);
  for (size_t i = tid; i < body; i += nthreads) body_ptr[i] = w4;
  for (size_t i = tail_start + tid; i < bytes; i += nthreads) dst[i] = b;
}

int create_ctx(int device, hipStream_t stream, bool own_stream,
               size_t workspace_bytes, ginn_hip_ctx** out) {
  GH_CHECK_ARG(out != nullptr, "ginn_hip_ctx_create: ctx is NULL");
  int count = 0;
  GH_HIP(hipGetDeviceCount(&count));
  GH_CHECK_ARG(device >= 0 && device < count,
               "ginn_hip_ctx_create: device %d out of range (%d visible)",
               device, count);
  GH_HIP(hipSetDevice(device));
  noalloc_prepare(device);
  ginn_hip_ctx* ctx = new (std::nothrow) ginn_hip_ctx();
  if (!ctx) return fail(kOutOfMemory, "ginn_hip_ctx_create: host allocation failed");
  ctx->device = device;
  ctx->owns_stream = own_stream;
  ctx->stream = stream;
  hipError_t e = hipSuccess;
  if (own_stream) {
    // Default priority on purpose: mixed stream priorities are not used.
    e = hipStreamCreate(&ctx->stream);
  }
  if (e == hipSuccess) {
    ctx->workspace_bytes = workspace_bytes ? workspace_bytes : kDefaultWorkspace;
    e = hipMalloc(&ctx->workspace, ctx->workspace_bytes);
  }
  if (e == hipSuccess) {
    ctx->host_staging_bytes = kHostStaging;
    e = hipHostMalloc(&ctx->host_staging, ctx->host_staging_bytes, hipHostMallocDefault);
  }
  if (e == hipSuccess) e = hipEventCreateWithFlags(&ctx->staging_event, hipEventDisableTiming);
  for (int i = 0; i < 64 && e == hipSuccess; ++i) e = hipEventCreate(&ctx->events[i]);
  if (e == hipSuccess) {
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e == hipSuccess) ctx->num_cus = prop.multiProcessorCount;
  }
  if (e != hipSuccess) {
    int rc = fail(kHipError, "ginn_hip_ctx_create: %s", hipGetErrorString(e));
    ginn_hip_ctx_destroy(ctx);
    // ginn_hip_ctx_destroy clears nothing in the error slot on success paths
    // only; restore the creation failure for the caller.
    return rc;
  }
  *out = ctx;
  return kOk;
}

}  // namespace

int stage_to_workspace(ginn_hip_ctx* ctx, size_t offset, const void* host_src,
                       size_t bytes) {
  GH_CHECK_ARG(offset + bytes <= ctx->workspace_bytes,
               "workspace too small: need %zu bytes at offset %zu, have %zu",
               bytes, offset, ctx->workspace_bytes);
  GH_CHECK_ARG(bytes <= ctx->host_staging_bytes,
               "table of %zu bytes exceeds the %zu-byte staging buffer", bytes,
               ctx->host_staging_bytes);
  // Ring of pinned memory.  When the cursor wraps, wait for the copies that
  // still read the old contents.
  size_t aligned = (bytes + 63) & ~size_t(63);
  if (ctx->host_staging_used + aligned > ctx->host_staging_bytes) {
    GH_HIP(hipEventRecord(ctx->staging_event, ctx->stream));
    GH_HIP(hipEventSynchronize(ctx->staging_event));
    ctx->host_staging_used = 0;
  }
  char* slot = static_cast<char*>(ctx->host_staging) + ctx->host_staging_used;
  ctx->host_staging_used += aligned;
  memcpy(slot, host_src, bytes);
  GH_HIP(hipMemcpyAsync(static_cast<char*>(ctx->workspace) + offset, slot, bytes,
                        hipMemcpyHostToDevice, ctx->stream));
  return kOk;
}

}  // namespace ginn_hip

namespace {
// Block sizes of the pool: powers of two from 256 B to 2 MiB, multiples of 2 MiB above.
size_t pool_block_size(size_t bytes) {
  constexpr size_t kLarge = size_t(2) << 20;
  if (bytes > kLarge) return (bytes + kLarge - 1) / kLarge * kLarge;
  size_t b = 256;
  while (b < bytes) b <<= 1;
  return b;
}
constexpr size_t kSlabBytes = size_t(2) << 20;
constexpr size_t kSlabMaxBlock = size_t(64) << 10;

// The slab that ptr was cut from, or end().
std::map<uintptr_t, ginn_hip_slab>::iterator slab_of(ginn_hip_pool& pool, const void* ptr) {
  const uintptr_t at = reinterpret_cast<uintptr_t>(ptr);
  auto it = pool.slabs.upper_bound(at);
  if (it == pool.slabs.begin()) return pool.slabs.end();
  --it;
  return at < it->first + kSlabBytes ? it : pool.slabs.end();
}

// Gives a slab without live blocks back to the driver (its cached blocks have
// been taken off the free lists by the caller, or are taken off here).
void pool_release_slab(ginn_hip_pool& pool, std::map<uintptr_t, ginn_hip_slab>::iterator slab) {
  const uintptr_t base = slab->first;
  const ginn_hip_slab s = slab->second;
  auto list = pool.free_blocks.find(s.block);
  if (list != pool.free_blocks.end()) {
    auto& v = list->second;
    const size_t before = v.size();
    v.erase(std::remove_if(v.begin(), v.end(),
                           [&](void* p) {
                             const uintptr_t at = reinterpret_cast<uintptr_t>(p);
                             return at >= base && at < base + kSlabBytes;
                           }),
            v.end());
    pool.cached_bytes -= (before - v.size()) * s.block;
  }
  for (size_t off = 0; off < s.carved; off += s.block) pool.block_size.erase(reinterpret_cast<void*>(base + off));
  auto open = pool.open_slab.find(s.block);
  if (open != pool.open_slab.end() && open->second == base) pool.open_slab.erase(open);
  (void)hipFree(reinterpret_cast<void*>(base));
  pool.slabs.erase(slab);
}

// Gives every cached block that can go back to the driver: blocks of their
// own, and slabs none of whose blocks is in use.  The caller holds the pool's mutex.
void pool_release_cached(ginn_hip_pool& pool) {
  for (auto& [size, blocks] : pool.free_blocks) {
    std::vector<void*> kept;
    for (void* p : blocks) {
      if (slab_of(pool, p) != pool.slabs.end()) {
        kept.push_back(p);
        continue;
      }
      (void)hipFree(p);
      pool.block_size.erase(p);
      pool.cached_bytes -= size;
    }
    blocks.swap(kept);
  }
  for (auto it = pool.slabs.begin(); it != pool.slabs.end();) {
    auto next = std::next(it);
    if (it->second.live == 0) pool_release_slab(pool, it);
    it = next;
  }
}
}  // namespace

using namespace ginn_hip;

extern "C" {

const char* ginn_hip_last_error(void) { return g_last_error.c_str(); }

const char* ginn_hip_version(void) { return "0.1"; }

int ginn_hip_device_count(int* count) {
  GH_CHECK_ARG(count != nullptr, "ginn_hip_device_count: count is NULL");
  int c = 0;
  hipError_t e = hipGetDeviceCount(&c);
  if (e != hipSuccess) {
    // As ginn::gpus() does (ginn/dev.h:41-43): no usable runtime means zero.
    (void)hipGetLastError();
    c = 0;
  }
  *count = c;
  return kOk;
}

int ginn_hip_ctx_create(int device, size_t workspace_bytes, ginn_hip_ctx** ctx) {
  return create_ctx(device, nullptr, true, workspace_bytes, ctx);
}

int ginn_hip_ctx_create_on_stream(int device, void* stream,
                                  size_t workspace_bytes, ginn_hip_ctx** ctx) {
  return create_ctx(device, static_cast<hipStream_t>(stream), false,
                    workspace_bytes, ctx);
}

int ginn_hip_ctx_destroy(ginn_hip_ctx* ctx) {
  if (!ctx) return kOk;
  // Like ~GpuDevice (ginn/dev.h:194-198) teardown swallows runtime errors.
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& ev : ctx->events)
    if (ev) (void)hipEventDestroy(ev);
  if (ctx->staging_event) (void)hipEventDestroy(ctx->staging_event);
  if (ctx->order_event) (void)hipEventDestroy(ctx->order_event);
  if (ctx->host_staging) (void)hipHostFree(ctx->host_staging);
  if (ctx->workspace) (void)hipFree(ctx->workspace);
  if (ctx->folds.arena) (void)hipFree(ctx->folds.arena);
  pool_release_cached(ctx->pool);
  for (auto& slab : ctx->pool.slabs) (void)hipFree(reinterpret_cast<void*>(slab.first));  // blocks never released
  if (ctx->owns_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
  return kOk;
}

int ginn_hip_ctx_device(const ginn_hip_ctx* ctx, int* device) {
  GH_CHECK_ARG(ctx && device, "ginn_hip_ctx_device: NULL argument");
  *device = ctx->device;
  return kOk;
}

int ginn_hip_ctx_stream(const ginn_hip_ctx* ctx, void** stream) {
  GH_CHECK_ARG(ctx && stream, "ginn_hip_ctx_stream: NULL argument");
  *stream = ctx->stream;
  return kOk;
}

int ginn_hip_sync(ginn_hip_ctx* ctx) {
  GH_CHECK_ARG(ctx, "ginn_hip_sync: ctx is NULL");
  if (int rc = ginn_hip_flush_folds(ctx)) return rc;  // postponed folds belong to what the caller waits for
  GH_HIP(hipStreamSynchronize(ctx->stream));
  return kOk;
}

int ginn_hip_malloc(ginn_hip_ctx* ctx, size_t bytes, void** ptr) {
  GH_CHECK_ARG(ctx && ptr, "ginn_hip_malloc: NULL argument");
  *ptr = nullptr;
  if (bytes == 0) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  ginn_hip_pool& pool = ctx->pool;
  std::lock_guard<std::mutex> lock(pool.mutex);
  const size_t block = pool.enabled ? pool_block_size(bytes) : bytes;
  if (pool.enabled) {
    auto it = pool.free_blocks.find(block);
    if (it != pool.free_blocks.end() && !it->second.empty()) {
      *ptr = it->second.back();
      it->second.pop_back();
      pool.cached_bytes -= block;
      auto slab = slab_of(pool, *ptr);
      if (slab != pool.slabs.end()) ++slab->second.live;
      return kOk;
    }
    if (block <= kSlabMaxBlock) {
      // Cut the next block of this size class's slab; a new slab when it is used up.
      auto open = pool.open_slab.find(block);
      auto slab = open == pool.open_slab.end() ? pool.slabs.end() : pool.slabs.find(open->second);
      if (slab == pool.slabs.end() || slab->second.carved + block > kSlabBytes) {
        void* base = nullptr;
        if (hipMalloc(&base, kSlabBytes) == hipSuccess) {
          ginn_hip_slab fresh;
          fresh.block = block;
          slab = pool.slabs.emplace(reinterpret_cast<uintptr_t>(base), fresh).first;
          pool.open_slab[block] = slab->first;
        } else {
          (void)hipGetLastError();  // no room for a slab: a block of its own below
          slab = pool.slabs.end();
        }
      }
      if (slab != pool.slabs.end()) {
        *ptr = reinterpret_cast<void*>(slab->first + slab->second.carved);
        slab->second.carved += block;
        ++slab->second.live;
        pool.block_size[*ptr] = block;
        return kOk;
      }
    }
  }
  hipError_t e = hipMalloc(ptr, block);
  if (e == hipErrorOutOfMemory && pool.cached_bytes > 0) {
    // The cache holds what the driver lacks: give it back and ask again.
    (void)hipGetLastError();
    pool_release_cached(pool);
    e = hipMalloc(ptr, block);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *ptr = nullptr;
    return fail(e == hipErrorOutOfMemory ? kOutOfMemory : kHipError,
                "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
  }
  if (pool.enabled) pool.block_size[*ptr] = block;
  return kOk;
}

int ginn_hip_free(ginn_hip_ctx* ctx, void* ptr) {
  GH_CHECK_ARG(ctx, "ginn_hip_free: ctx is NULL");
  if (!ptr) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  ginn_hip_pool& pool = ctx->pool;
  std::lock_guard<std::mutex> lock(pool.mutex);
  auto it = pool.block_size.find(ptr);
  if (it != pool.block_size.end()) {
    const size_t block = it->second;
    const bool keep = pool.enabled && pool.cached_bytes + block <= pool.limit_bytes;
    auto slab = slab_of(pool, ptr);
    if (slab != pool.slabs.end()) {
      // Part of a slab: it waits on the free list, or the slab goes when this was its last block in use.
      --slab->second.live;
      if (!keep && slab->second.live == 0) {
        pool_release_slab(pool, slab);
      } else {
        pool.free_blocks[block].push_back(ptr);
        pool.cached_bytes += block;
      }
      return kOk;
    }
    if (keep) {
      pool.free_blocks[block].push_back(ptr);
      pool.cached_bytes += block;
      return kOk;
    }
    pool.block_size.erase(it);
  }
  GH_HIP(hipFree(ptr));
  return kOk;
}

int ginn_hip_pool_configure(ginn_hip_ctx* ctx, int enabled, size_t limit_bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_pool_configure: ctx is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  ginn_hip_pool& pool = ctx->pool;
  std::lock_guard<std::mutex> lock(pool.mutex);
  pool.enabled = enabled != 0;
  pool.limit_bytes = limit_bytes;
  if (!pool.enabled || pool.cached_bytes > pool.limit_bytes) {
    GH_HIP(hipStreamSynchronize(ctx->stream));
    pool_release_cached(pool);
  }
  return kOk;
}

int ginn_hip_gemm_temp_budget(ginn_hip_ctx* ctx, size_t bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm_temp_budget: ctx is NULL");
  std::lock_guard<std::mutex> lock(ctx->mutex);
  ctx->gemm_temp_budget = bytes;
  return kOk;
}

int ginn_hip_pool_trim(ginn_hip_ctx* ctx) {
  GH_CHECK_ARG(ctx, "ginn_hip_pool_trim: ctx is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  GH_HIP(hipStreamSynchronize(ctx->stream));
  std::lock_guard<std::mutex> lock(ctx->pool.mutex);
  pool_release_cached(ctx->pool);
  return kOk;
}

int ginn_hip_pool_stats(ginn_hip_ctx* ctx, size_t* cached_bytes, size_t* blocks) {
  GH_CHECK_ARG(ctx && cached_bytes && blocks, "ginn_hip_pool_stats: NULL argument");
  std::lock_guard<std::mutex> lock(ctx->pool.mutex);
  *cached_bytes = ctx->pool.cached_bytes;
  *blocks = ctx->pool.block_size.size();
  return kOk;
}

int ginn_hip_memcpy_h2d(ginn_hip_ctx* ctx, void* dst, const void* host_src,
                        size_t bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_memcpy_h2d: ctx is NULL");
  if (bytes == 0) return kOk;
  GH_CHECK_ARG(dst && host_src, "ginn_hip_memcpy_h2d: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  GH_HIP(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, ctx->stream));
  return kOk;
}

int ginn_hip_memcpy_d2h(ginn_hip_ctx* ctx, void* host_dst, const void* src,
                        size_t bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_memcpy_d2h: ctx is NULL");
  if (bytes == 0) return kOk;
  GH_CHECK_ARG(host_dst && src, "ginn_hip_memcpy_d2h: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  GH_HIP(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  GH_HIP(hipStreamSynchronize(ctx->stream));
  return kOk;
}

int ginn_hip_memcpy_d2d(ginn_hip_ctx* ctx, void* dst, const void* src,
                        size_t bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_memcpy_d2d: ctx is NULL");
  if (bytes == 0) return kOk;
  GH_CHECK_ARG(dst && src, "ginn_hip_memcpy_d2d: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  GH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return kOk;
}

int ginn_hip_memset(ginn_hip_ctx* ctx, void* dst, int byte_value, size_t bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_memset: ctx is NULL");
  if (bytes == 0) return kOk;
  GH_CHECK_ARG(dst, "ginn_hip_memset: dst is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  const uint32_t b = static_cast<uint32_t>(byte_value) & 0xffu;
  const uint32_t word = b | (b << 8) | (b << 16) | (b << 24);
  size_t blocks = (bytes / 16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  const size_t max_blocks = static_cast<size_t>(ctx->num_cus) * 8;
  if (blocks > max_blocks) blocks = max_blocks;
  fill_bytes_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx->stream>>>(
      static_cast<uint8_t*>(dst), word, bytes);
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_arena_create(ginn_hip_ctx* ctx, size_t bytes, ginn_hip_arena** arena) {
  GH_CHECK_ARG(ctx && arena, "ginn_hip_arena_create: NULL argument");
  GH_CHECK_ARG(bytes > 0, "ginn_hip_arena_create: size must be positive");
  ginn_hip_arena* a = new (std::nothrow) ginn_hip_arena();
  if (!a) return fail(kOutOfMemory, "ginn_hip_arena_create: host allocation failed");
  a->ctx = ctx;
  a->size = bytes;
  void* p = nullptr;
  int rc = ginn_hip_malloc(ctx, bytes, &p);
  if (rc != kOk) {
    delete a;
    return rc;
  }
  a->base = static_cast<char*>(p);
  *arena = a;
  return kOk;
}

int ginn_hip_arena_destroy(ginn_hip_arena* arena) {
  if (!arena) return kOk;
  (void)hipSetDevice(arena->ctx->device);
  if (arena->base) (void)ginn_hip_free(arena->ctx, arena->base);  // it came from ginn_hip_malloc
  delete arena;
  return kOk;
}

int ginn_hip_arena_alloc(ginn_hip_arena* arena, size_t bytes, void** ptr) {
  GH_CHECK_ARG(arena && ptr, "ginn_hip_arena_alloc: NULL argument");
  // Byte-exact bump with the strict '<' of PreallocGpuDevice::alloc
  // (ginn/dev.h:238-241) unless the caller asked for aligned blocks.
  const size_t al = arena->alignment;
  const size_t start = al > 1 ? (arena->used + al - 1) / al * al : arena->used;
  if (!(start + bytes < arena->size)) {
    *ptr = nullptr;
    return fail(kOutOfMemory,
                "Prealloc device out of memory! Used: %zu Attempted to allocate: %zu",
                arena->used, bytes);
  }
  *ptr = arena->base + start;
  arena->used = start + bytes;
  return kOk;
}

int ginn_hip_arena_set_alignment(ginn_hip_arena* arena, size_t alignment) {
  GH_CHECK_ARG(arena, "ginn_hip_arena_set_alignment: arena is NULL");
  GH_CHECK_ARG(alignment >= 1 && alignment <= 4096 && (alignment & (alignment - 1)) == 0,
               "ginn_hip_arena_set_alignment: %zu is not a power of two in 1..4096", alignment);
  arena->alignment = alignment;
  return kOk;
}

int ginn_hip_arena_clear(ginn_hip_arena* arena) {
  GH_CHECK_ARG(arena, "ginn_hip_arena_clear: arena is NULL");
  arena->used = 0;
  return kOk;
}

int ginn_hip_arena_used(const ginn_hip_arena* arena, size_t* bytes) {
  GH_CHECK_ARG(arena && bytes, "ginn_hip_arena_used: NULL argument");
  *bytes = arena->used;
  return kOk;
}

int ginn_hip_arena_size(const ginn_hip_arena* arena, size_t* bytes) {
  GH_CHECK_ARG(arena && bytes, "ginn_hip_arena_size: NULL argument");
  *bytes = arena->size;
  return kOk;
}

int ginn_hip_ctx_wait_for(ginn_hip_ctx* waiter, ginn_hip_ctx* signaler, int* ordered) {
  GH_CHECK_ARG(waiter && signaler && ordered, "ginn_hip_ctx_wait_for: NULL argument");
  GH_CHECK_ARG(waiter->device == signaler->device, "ginn_hip_ctx_wait_for: contexts of devices %d and %d",
               waiter->device, signaler->device);
  *ordered = 0;
  if (waiter == signaler || waiter->stream == signaler->stream) {
    *ordered = 1;  // one stream: already in order
    return kOk;
  }
  GH_HIP(hipSetDevice(signaler->device));
  for (ginn_hip_ctx* c : {waiter, signaler}) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    GH_HIP(hipStreamIsCapturing(c->stream, &status));
    if (status != hipStreamCaptureStatusNone) return kOk;
  }
  {
    std::lock_guard<std::mutex> lock(signaler->mutex);
    if (!signaler->order_event) GH_HIP(hipEventCreateWithFlags(&signaler->order_event, hipEventDisableTiming));
    // The wait below refers to this record; a later record by another host thread does not change it.
    GH_HIP(hipEventRecord(signaler->order_event, signaler->stream));
    GH_HIP(hipStreamWaitEvent(waiter->stream, signaler->order_event, 0));
  }
  *ordered = 1;
  return kOk;
}

int ginn_hip_capture_begin(ginn_hip_ctx* ctx) {
  GH_CHECK_ARG(ctx, "ginn_hip_capture_begin: ctx is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  GH_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
  return kOk;
}

int ginn_hip_capture_end(ginn_hip_ctx* ctx, ginn_hip_graph** graph) {
  GH_CHECK_ARG(ctx && graph, "ginn_hip_capture_end: NULL argument");
  *graph = nullptr;
  GH_HIP(hipSetDevice(ctx->device));
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g);
  if (e != hipSuccess || !g) {
    (void)hipGetLastError();
    return fail(kHipError, "ginn_hip_capture_end: the capture failed (%s): something that cannot be recorded ran "
                           "on the stream", hipGetErrorString(e));
  }
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    (void)hipGraphDestroy(g);
    return fail(kHipError, "ginn_hip_capture_end: hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  ginn_hip_graph* out = new (std::nothrow) ginn_hip_graph();
  if (!out) {
    (void)hipGraphExecDestroy(exec);
    (void)hipGraphDestroy(g);
    return fail(kOutOfMemory, "ginn_hip_capture_end: host allocation failed");
  }
  out->ctx = ctx;
  out->graph = g;
  out->exec = exec;
  *graph = out;
  return kOk;
}

int ginn_hip_graph_launch(ginn_hip_graph* graph) {
  GH_CHECK_ARG(graph && graph->exec, "ginn_hip_graph_launch: graph is NULL");
  GH_HIP(hipSetDevice(graph->ctx->device));
  GH_HIP(hipGraphLaunch(graph->exec, graph->ctx->stream));
  return kOk;
}

int ginn_hip_graph_kernel_count(ginn_hip_graph* graph, size_t* kernels) {
  GH_CHECK_ARG(graph && graph->graph && kernels, "ginn_hip_graph_kernel_count: NULL argument");
  *kernels = 0;
  size_t n = 0;
  GH_HIP(hipGraphGetNodes(graph->graph, nullptr, &n));
  std::vector<hipGraphNode_t> nodes(n);
  if (n) GH_HIP(hipGraphGetNodes(graph->graph, nodes.data(), &n));
  for (size_t i = 0; i < n; ++i) {
    hipGraphNodeType type;
    GH_HIP(hipGraphNodeGetType(nodes[i], &type));
    if (type == hipGraphNodeTypeKernel) ++*kernels;
  }
  return kOk;
}

int ginn_hip_graph_destroy(ginn_hip_graph* graph) {
  if (!graph) return kOk;
  (void)hipSetDevice(graph->ctx->device);
  if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
  if (graph->graph) (void)hipGraphDestroy(graph->graph);
  delete graph;
  return kOk;
}

int ginn_hip_event_record(ginn_hip_ctx* ctx, int slot) {
  GH_CHECK_ARG(ctx, "ginn_hip_event_record: ctx is NULL");
  GH_CHECK_ARG(slot >= 0 && slot < 64, "ginn_hip_event_record: slot %d out of range", slot);
  GH_HIP(hipEventRecord(ctx->events[slot], ctx->stream));
  return kOk;
}

int ginn_hip_event_elapsed_ms(ginn_hip_ctx* ctx, int start, int stop, float* ms) {
  GH_CHECK_ARG(ctx && ms, "ginn_hip_event_elapsed_ms: NULL argument");
  GH_CHECK_ARG(start >= 0 && start < 64 && stop >= 0 && stop < 64,
               "ginn_hip_event_elapsed_ms: slot out of range");
  GH_HIP(hipEventSynchronize(ctx->events[stop]));
  GH_HIP(hipEventElapsedTime(ms, ctx->events[start], ctx->events[stop]));
  return kOk;
}

}  // extern "C"
