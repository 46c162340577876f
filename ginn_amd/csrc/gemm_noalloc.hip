// ginn_hip_gemm_noalloc: the product entry point for callers that cannot
// allocate (HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc).  Same kernels as ginn_hip_gemm; what differs is where the
// split-K partial sums live: not in a context's hipMalloc'ed workspace but in
// a file-scope device array that exists once per GPU for the life of the
// process.  Nothing here allocates or frees device or pinned memory.
#include "common.h"

namespace ginn_hip {

namespace {

constexpr size_t kScratchBytes = 16u << 20;  // 16 MiB per GPU
// Largest output (elements): two fp32 partial copies of it fit the scratch, so
// every split-K plan of the launchers has room for at least two splits.
constexpr long long kMaxOutputElements = static_cast<long long>(kScratchBytes / (2 * sizeof(float)));
constexpr int kMaxDevices = 64;

// The scratch.  In host code this name is only a handle for
// hipGetSymbolAddress: it is never passed to a kernel or a runtime call.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

struct DeviceState {
  std::mutex mutex;        // orders host threads that use this GPU's scratch
  bool ready = false;
  void* scratch_ptr = nullptr;  // this GPU's copy of `scratch`, from hipGetSymbolAddress
  int num_cus = 256;
};
DeviceState g_state[kMaxDevices];

// With `device` current: looks up this GPU's address of the array, once.
int prepare_locked(int device, DeviceState& st) {
  if (st.ready) return kOk;
  void* ptr = nullptr;
  GH_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return fail(kHipError, "ginn_hip_gemm_noalloc: no device address for the scratch array on GPU %d", device);
  int cus = 0;
  GH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  st.scratch_ptr = ptr;
  st.num_cus = cus > 0 ? cus : 256;
  st.ready = true;
  return kOk;
}

}  // namespace

// Called by context creation (the library's set-up call), with the device
// current, so that a later first use inside a stream capture has nothing left
// to look up.  Failures surface at the entry point itself.
void noalloc_prepare(int device) {
  if (device < 0 || device >= kMaxDevices) return;
  DeviceState& st = g_state[device];
  std::lock_guard<std::mutex> lock(st.mutex);
  (void)prepare_locked(device, st);
}

}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" int ginn_hip_gemm_noalloc(int device, void* stream, ginn_hip_dtype dtype, ginn_hip_op op_a,
                                     ginn_hip_op op_b, int m, int n, int k, const void* A, int lda, const void* B,
                                     int ldb, float beta, void* C, int ldc) {
  GH_CHECK_ARG(device >= 0 && device < kMaxDevices, "ginn_hip_gemm_noalloc: device %d out of range", device);
  GH_CHECK_ARG(m >= 0 && n >= 0 && k >= 0, "ginn_hip_gemm_noalloc: negative dimension (m=%d n=%d k=%d)", m, n, k);
  GH_CHECK_ARG(static_cast<long long>(m) * n <= kMaxOutputElements,
               "ginn_hip_gemm_noalloc: output of %d x %d elements exceeds the %lld elements that the %zu-byte "
               "per-GPU scratch array is sized for; use ginn_hip_gemm with a context",
               m, n, kMaxOutputElements, kScratchBytes);
  if (m == 0 || n == 0) return kOk;  // an empty product touches nothing, as in ginn_hip_gemm
  int count = 0;
  GH_HIP(hipGetDeviceCount(&count));
  GH_CHECK_ARG(device < count, "ginn_hip_gemm_noalloc: device %d out of range (%d visible)", device, count);
  GH_HIP(hipSetDevice(device));
  DeviceState& st = g_state[device];
  std::lock_guard<std::mutex> lock(st.mutex);
  if (int rc = prepare_locked(device, st)) return rc;
  // A context on the stack: the launchers read device, stream, workspace and
  // CU count from it; it owns nothing.  The partial sums of a split-K plan are
  // written in full before the fold reads them, so the array's old contents
  // never matter and nothing has to be cleared between calls.
  ginn_hip_ctx local;
  local.device = device;
  local.stream = static_cast<hipStream_t>(stream);
  local.workspace = st.scratch_ptr;
  local.workspace_bytes = kScratchBytes;
  local.num_cus = st.num_cus;
  local.may_allocate = false;
  GemmArgs a{};
  a.dtype = dtype;
  a.op_a = op_a;
  a.op_b = op_b;
  a.m = m;
  a.n = n;
  a.k = k;
  a.A = A;
  a.lda = lda;
  a.B = B;
  a.ldb = ldb;
  a.beta = beta;
  a.C = C;
  a.ldc = ldc;
  a.batch = 1;
  return launch_gemm(&local, a);
}
