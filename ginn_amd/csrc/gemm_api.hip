// Matrix-product entry points: argument checks in the manner of a BLAS,
// kernel selection, and the AffineNode forward composition.
#include <vector>

#include "common.h"

namespace ginn_hip {

namespace {

int check_gemm_args(const char* who, const GemmArgs& a) {
  GH_CHECK_ARG(dtype_valid(a.dtype), "%s: unknown dtype %d", who, a.dtype);
  GH_CHECK_ARG(a.op_a == GINN_HIP_OP_N || a.op_a == GINN_HIP_OP_T, "%s: bad op_a %d", who, a.op_a);
  GH_CHECK_ARG(a.op_b == GINN_HIP_OP_N || a.op_b == GINN_HIP_OP_T, "%s: bad op_b %d", who, a.op_b);
  GH_CHECK_ARG(a.m >= 0 && a.n >= 0 && a.k >= 0, "%s: negative dimension (m=%d n=%d k=%d)", who, a.m, a.n, a.k);
  GH_CHECK_ARG(a.batch >= 0, "%s: negative batch %d", who, a.batch);
  if (!a.acols) {
    const int a_rows = a.op_a == GINN_HIP_OP_N ? a.m : a.k;
    GH_CHECK_ARG(a.lda >= (a_rows > 1 ? a_rows : 1), "%s: lda=%d smaller than the %d rows of A", who, a.lda, a_rows);
  }
  if (!a.bcols) {
    const int b_rows = a.op_b == GINN_HIP_OP_N ? a.k : a.n;
    GH_CHECK_ARG(a.ldb >= (b_rows > 1 ? b_rows : 1), "%s: ldb=%d smaller than the %d rows of B", who, a.ldb, b_rows);
  }
  if (!a.ccols)
    GH_CHECK_ARG(a.ldc >= (a.m > 1 ? a.m : 1), "%s: ldc=%d smaller than m=%d", who, a.ldc, a.m);
  if (a.m == 0 || a.n == 0 || a.batch == 0) return kOk;
  GH_CHECK_ARG(a.ccols || a.C != nullptr, "%s: C is NULL", who);
  if (a.k > 0) {
    GH_CHECK_ARG(a.acols || a.A != nullptr, "%s: A is NULL", who);
    GH_CHECK_ARG(a.bcols || a.B != nullptr, "%s: B is NULL", who);
  }
  if (a.batch > 1) {
    GH_CHECK_ARG(a.stride_a >= 0 && a.stride_b >= 0 && a.stride_c >= 0, "%s: negative stride", who);
  }
  return kOk;
}

// A leading dimension or pointer that rules out 16-byte accesses -- an odd row count as the leading
// dimension of a column-major operand is enough -- leaves a product on the any-shape kernel's element
// loads: 20 x slower than its aligned neighbour for a large one (fp16 4095 x 4097 x 4099: 2.6-2.9 ms
// against 0.11 ms for 4096^3).  A large product is therefore computed on copies with padded leading
// dimensions (blocks from the context's pool, released after the calls: reuse is ordered on the stream):
// the operands that need it are copied in, the output (and the kept pre-activation) copied in when beta
// reads it and copied back afterwards.  Not while the stream is being captured (the pool may have to
// allocate) and not for the entry point that must not allocate.
int launch_gemm_realigned(ginn_hip_ctx* ctx, const GemmArgs& a) {
  if (a.batch != 1 || a.acols || a.bcols || a.ccols || !ctx->may_allocate) return kUnsupported;
  const size_t es = dtype_size(a.dtype);
  const int per16 = static_cast<int>(16 / es);
  auto bad = [&](const void* ptr, int ld) { return reinterpret_cast<uintptr_t>(ptr) % 16 != 0 || ld % per16 != 0; };
  bool fix_a = bad(a.A, a.lda), fix_b = bad(a.B, a.ldb);
  bool fix_c = bad(a.C, a.ldc) || (a.pre && bad(a.pre, a.ldc));
  const bool fix_bias = a.bias && reinterpret_cast<uintptr_t>(a.bias) % 16 != 0;
  if (!fix_a && !fix_b && !fix_c && !fix_bias) return kUnsupported;
  // From where the copies pay (measured, any-shape kernel alone -> on copies, us): fp32 1001 x 1003 x 1005
  // 115 -> 56, 515 x 2049 x 515 75 -> 47, but 801 x 803 x 805 54 -> 62; fp16 with one operand to copy
  // 1024 x 1024 x 1001 73 -> 20, with all three 1501 x 1503 x 1505 181 -> 79 but 1001 x 1003 x 1005 74 -> 91.
  const int copies = int(fix_a) + int(fix_b) + int(fix_c);
  const double work = static_cast<double>(a.m) * a.n * a.k;
  const double least = a.dtype == GINN_HIP_F32 ? 536870912. : (copies >= 2 ? 2147483648. : 268435456.);
  if (a.m < 256 || a.n < 256 || a.k < 256 || work < least) return kUnsupported;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  GH_HIP(hipStreamIsCapturing(ctx->stream, &capturing));
  if (capturing != hipStreamCaptureStatusNone) return kUnsupported;

  const ginn_hip_dtype dt = static_cast<ginn_hip_dtype>(a.dtype);
  // When all three matrices of a 16-bit product are copied anyway, the copies are zero-padded to whole tiles
  // as well (rows and columns to multiples of 128, K to the K tile): the tuned kernels then take the product
  // whole, where the ragged rows and columns of 4095 x 4097 x 4099 cost the any-shape kernel more than the
  // core costs (435 -> 212 us; 2047 x 2049 x 2051 106 -> 76 us).  fp32 keeps its extents (the same padding
  // there: 1311 -> 1366 us and 228 -> 298 us).
  const bool whole_tiles = fix_a && fix_b && fix_c && a.dtype != GINN_HIP_F32;
  const int bk = static_cast<int>(128 / es);
  auto up = [](int v, int unit) { return (v + unit - 1) / unit * unit; };
  const int mp = whole_tiles ? up(a.m, 128) : a.m, np = whole_tiles ? up(a.n, 128) : a.n;
  const int kp = whole_tiles ? up(a.k, bk) : a.k;
  // A copy: a stored rows_p x cols_p matrix with a padded leading dimension, zeroed when larger than the
  // rows x cols matrix at src, which is copied in when `fill`.
  struct Copy {
    const void* src = nullptr;
    int rows = 0, cols = 0, ld_src = 0, rows_p = 0, cols_p = 0, ld = 0;
    bool fill = false;
    void* block = nullptr;
    size_t bytes = 0;
  };
  Copy copies_[5];
  int used = 0;
  auto plan = [&](const void* src, int rows, int cols, int ld_src, int rows_p, int cols_p, bool fill) {
    Copy& c = copies_[used];
    c.src = src;
    c.rows = rows;
    c.cols = cols;
    c.ld_src = ld_src;
    c.rows_p = rows_p;
    c.cols_p = cols_p;
    c.ld = up(rows_p, 64);
    c.fill = fill;
    c.bytes = static_cast<size_t>(c.ld) * cols_p * es;
    return used++;
  };
  const bool an = a.op_a == GINN_HIP_OP_N, bn = a.op_b == GINN_HIP_OP_N;
  int ia = -1, ib = -1, ic = -1, ip = -1, ibias = -1;
  if (fix_a) ia = plan(a.A, an ? a.m : a.k, an ? a.k : a.m, a.lda, an ? mp : kp, an ? kp : mp, true);
  if (fix_b) ib = plan(a.B, bn ? a.k : a.n, bn ? a.n : a.k, a.ldb, bn ? kp : np, bn ? np : kp, true);
  if (fix_c) {
    // The epilogue reads the old values from the kept pre-activation when there is one, from C otherwise.
    ic = plan(a.C, a.m, a.n, a.ldc, mp, np, a.beta != 0.f && !a.pre);
    if (a.pre) ip = plan(a.pre, a.m, a.n, a.ldc, mp, np, a.beta != 0.f);
  }
  if (a.bias && (fix_bias || mp != a.m)) ibias = plan(a.bias, a.m, 1, a.m, mp, 1, true);
  // All blocks first, before anything is written: when the device (or the budget for temporaries) has no
  // room for them the product still runs where it is, on the any-shape kernels, as it did before this
  // path existed.  Nothing of C or the kept pre-activation has been touched at that point.
  size_t total = 0;
  for (int i = 0; i < used; ++i) total += copies_[i].bytes;
  if (total > ctx->gemm_temp_budget) return kUnsupported;
  for (int i = 0; i < used; ++i) {
    if (ginn_hip_malloc(ctx, copies_[i].bytes, &copies_[i].block) != kOk) {
      for (int j = 0; j < i; ++j) (void)ginn_hip_free(ctx, copies_[j].block);
      clear_error();
      return kUnsupported;
    }
  }
  int rc = kOk;
  for (int i = 0; i < used && rc == kOk; ++i) {
    const Copy& c = copies_[i];
    if (c.rows_p != c.rows || c.cols_p != c.cols) rc = ginn_hip_memset(ctx, c.block, 0, c.bytes);
    if (rc == kOk && c.fill) rc = ginn_hip_copy_2d(ctx, dt, c.rows, c.cols, c.src, c.ld_src, c.block, c.ld, 0);
  }
  GemmArgs b = a;
  b.m = mp;
  b.n = np;
  b.k = kp;
  if (ia >= 0) {
    b.A = copies_[ia].block;
    b.lda = copies_[ia].ld;
  }
  if (ib >= 0) {
    b.B = copies_[ib].block;
    b.ldb = copies_[ib].ld;
  }
  if (ic >= 0) {
    b.C = copies_[ic].block;
    b.ldc = copies_[ic].ld;
  }
  if (ip >= 0) b.pre = copies_[ip].block;
  if (ibias >= 0) b.bias = copies_[ibias].block;
  if (rc == kOk) rc = launch_gemm(ctx, b);
  if (rc == kOk && ic >= 0) rc = ginn_hip_copy_2d(ctx, dt, a.m, a.n, b.C, b.ldc, a.C, a.ldc, 0);
  if (rc == kOk && ip >= 0) rc = ginn_hip_copy_2d(ctx, dt, a.m, a.n, b.pre, b.ldc, a.pre, a.ldc, 0);
  for (int i = 0; i < used; ++i) {
    const int rc_free = ginn_hip_free(ctx, copies_[i].block);
    if (rc == kOk) rc = rc_free;
  }
  return rc;
}

// Extents that are no multiples of the tuned kernels' tiles (4000^3; m = 1000) left a product on
// the any-shape kernel, several times slower than its aligned neighbours (fp16 4000^3: 596 us
// against 112 us for 4096^3).  With leading dimensions and pointers that allow 16-byte accesses the
// product is cut instead: the last K % (K tile) values over the whole output first (any-shape
// kernel, the caller's beta), then the aligned core (tuned kernels) and the ragged rows and columns
// around it (any-shape kernel) over the whole K tiles, adding to that, with the caller's epilogue.
// A 16-bit sum is then rounded to the storage type once in between, as between the (W, X) pairs of
// an Affine.
//
// The same cut with 256 as the unit, tried before the 128 x 128 kernel takes a 16-bit product whole: extents
// that are multiples of 128 but not of 256 keep the 256 x 256 kernel for the core when that has the tiles
// the kernel wants, and leave strips of 128 .. 255 rows / columns to the 128 x 128 kernel.
int launch_gemm_ragged(ginn_hip_ctx* ctx, const GemmArgs& a, int unit) {
  if (a.batch != 1 || a.acols || a.bcols || a.ccols) return kUnsupported;
  if (unit == 256 && (a.dtype == GINN_HIP_F32 || a.k < 256)) return kUnsupported;
  const long long es = static_cast<long long>(dtype_size(a.dtype));
  const int per16 = static_cast<int>(16 / es), bk = static_cast<int>(128 / es);
  if (a.lda % per16 || a.ldb % per16 || a.ldc % per16) return kUnsupported;
  auto aligned16 = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  if (!aligned16(a.A) || !aligned16(a.B) || !aligned16(a.C) || (a.pre && !aligned16(a.pre)) ||
      (a.bias && !aligned16(a.bias)))
    return kUnsupported;
  const int m0 = a.m / unit * unit, k0 = a.k / bk * bk;
  // With a K-contiguous B the 128 x 128 kernel masks a partly filled last tile column itself.
  const int n0 = unit == 128 && a.op_b == GINN_HIP_OP_N ? a.n : a.n / unit * unit;
  if (m0 == a.m && n0 == a.n && k0 == a.k) return kUnsupported;
  if (unit == 256) {
    // Only what the 128 x 128 kernel would otherwise take whole, and only for a core the 256 x 256 kernel takes.
    if (a.m % 128 || a.n % 128 || k0 != a.k) return kUnsupported;
    if (static_cast<long long>(m0 / 256) * (n0 / 256) * 16 < 9ll * ctx->num_cus) return kUnsupported;
  }
  if (m0 < 256 || n0 < 256 || k0 < 4 * bk) return kUnsupported;
  // Worth the extra launches: a core of at least 512^3 multiply-adds that is most of the product.  Ragged
  // rows cost more than a ragged K (their few rows times all of K are a slow shape for the any-shape
  // kernel): only from 4 (fp32) or 8 x as much on, and not for the 16-bit types with a K-contiguous A whose K
  // allows 16-byte loads, where the any-shape kernel alone is as fast (measured, us before -> after: fp16 NN 4000^3 596 -> 217,
  // 2000^3 106 -> 59, 1024 x 1024 x 1000 20.6 -> 11.7; fp32 NN 4000^3 1220 -> 996, 2000^3 242 -> 185,
  // 1000 x 1024 x 1024 42.7 -> 29.8; but fp16 TN 4000^3 239 -> 357, 1000^3 14.6 -> 21.2).
  const double core = static_cast<double>(m0) * n0 * k0, all = static_cast<double>(a.m) * a.n * a.k;
  if (core < 134217728. || core < (unit == 256 ? 0.85 : 0.75) * all) return kUnsupported;
  const bool f32 = a.dtype == GINN_HIP_F32;
  if (unit == 128 && m0 < a.m &&
      (core < (f32 ? 536870912. : 1073741824.) || (!f32 && a.op_a == GINN_HIP_OP_T && a.k % per16 == 0)))
    return kUnsupported;

  const char* A = static_cast<const char*>(a.A);
  const char* B = static_cast<const char*>(a.B);
  const bool at = a.op_a == GINN_HIP_OP_T, bt = a.op_b == GINN_HIP_OP_T;
  // Byte offsets of row r / K index kk of op(A), column c / K index kk of op(B), element (r, c) of C.
  auto a_at = [&](long long r, long long kk) { return A + (at ? r * a.lda + kk : kk * a.lda + r) * es; };
  auto b_at = [&](long long kk, long long c) { return B + (bt ? kk * a.ldb + c : c * a.ldb + kk) * es; };
  auto c_at = [&](void* base, long long r, long long c) {
    return base ? static_cast<void*>(static_cast<char*>(base) + (c * a.ldc + r) * es) : nullptr;
  };
  float beta = a.beta;
  if (k0 < a.k) {
    GemmArgs t = a;
    t.k = a.k - k0;
    t.A = a_at(0, k0);
    t.B = b_at(k0, 0);
    t.bias = nullptr;
    t.act = GINN_HIP_ACT_IDENTITY;
    if (int rc = launch_gemm_generic(ctx, t)) return rc;
    beta = 1.f;
  }
  GemmArgs c = a;
  c.m = m0;
  c.n = n0;
  c.k = k0;
  c.beta = beta;
  if (int rc = launch_gemm(ctx, c)) return rc;
  if (n0 < a.n) {  // the columns right of the core, all rows
    GemmArgs f = a;
    f.n = a.n - n0;
    f.k = k0;
    f.beta = beta;
    f.B = b_at(0, n0);
    f.C = c_at(a.C, 0, n0);
    f.pre = c_at(a.pre, 0, n0);
    if (int rc = launch_gemm(ctx, f)) return rc;
  }
  if (m0 < a.m) {  // the rows below the core, its columns
    GemmArgs f = a;
    f.m = a.m - m0;
    f.n = n0;
    f.k = k0;
    f.beta = beta;
    f.A = a_at(m0, 0);
    f.C = c_at(a.C, m0, 0);
    f.pre = c_at(a.pre, m0, 0);
    if (a.bias) f.bias = static_cast<const char*>(a.bias) + static_cast<long long>(m0) * es;
    if (int rc = launch_gemm(ctx, f)) return rc;
  }
  return kOk;
}

}  // namespace

int launch_gemm(ginn_hip_ctx* ctx, const GemmArgs& a) {
  if (int rc = check_gemm_args("gemm", a)) return rc;
  if (a.m == 0 || a.n == 0 || a.batch == 0) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  const bool plain = a.bias == nullptr && a.pre == nullptr &&
                     a.act == GINN_HIP_ACT_IDENTITY && a.bcols == nullptr && a.ccols == nullptr && a.acols == nullptr;
  // Degenerate batched dot: m = n = 1 with contiguous operands.
  if (plain && a.m == 1 && a.n == 1 && a.batch > 1 && a.stride_a == a.k &&
      a.stride_b == a.k && a.stride_c == 1 &&
      (a.op_a == GINN_HIP_OP_T || a.lda == 1) &&
      (a.op_b == GINN_HIP_OP_N || a.ldb == 1)) {
    return ginn_hip_col_dot_batched(ctx, static_cast<ginn_hip_dtype>(a.dtype), a.k,
                                    a.batch, a.A, a.B, a.beta, a.C);
  }
  // 16-bit products with a few columns: the 128 x 64 matrix-core kernel with split K reads A as fast as
  // the vector-ALU kernel and has the arithmetic for free (fp16 4096 x n x 4096: 7.9-8.5 us for n = 1 .. 8
  // against 8.5-15.2 us); the vector-ALU kernel keeps fp32 (whose matrix pipe is 16 x slower) and the 16-bit
  // shapes the matrix-core kernel does not take (unaligned operands, odd extents).
  int rc = launch_gemm_strip(ctx, a);
  if (rc != kUnsupported) return rc;
  if (a.dtype != GINN_HIP_F32 && a.batch == 1 && a.n <= 8) rc = launch_gemm_mid(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_ksplit(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_skinny(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_fast16(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_ragged(ctx, a, 256);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_bsmall(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_mid(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_realigned(ctx, a);
  if (rc != kUnsupported) return rc;
  rc = launch_gemm_ragged(ctx, a, 128);
  if (rc != kUnsupported) return rc;
  return launch_gemm_generic(ctx, a);
}

}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" {

int ginn_hip_gemm(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, ginn_hip_op op_a,
                  ginn_hip_op op_b, int m, int n, int k, const void* A, int lda,
                  const void* B, int ldb, float beta, void* C, int ldc) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm: ctx is NULL");
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
  return launch_gemm(ctx, a);
}

int ginn_hip_gemm_strided_batched(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                  ginn_hip_op op_a, ginn_hip_op op_b, int m,
                                  int n, int k, const void* A, int lda,
                                  long long stride_a, const void* B, int ldb,
                                  long long stride_b, float beta, void* C,
                                  int ldc, long long stride_c, int batch) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm_strided_batched: ctx is NULL");
  GemmArgs a{};
  a.dtype = dtype;
  a.op_a = op_a;
  a.op_b = op_b;
  a.m = m;
  a.n = n;
  a.k = k;
  a.A = A;
  a.lda = lda;
  a.stride_a = stride_a;
  a.B = B;
  a.ldb = ldb;
  a.stride_b = stride_b;
  a.beta = beta;
  a.C = C;
  a.ldc = ldc;
  a.stride_c = stride_c;
  a.batch = batch;
  return launch_gemm(ctx, a);
}

int ginn_hip_gemm_strided_batched2(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, ginn_hip_op op_a, ginn_hip_op op_b,
                                   int m, int n, int k, const void* A, int lda, long long stride_a,
                                   long long stride_a2, const void* B, int ldb, long long stride_b,
                                   long long stride_b2, float beta, void* C, int ldc, long long stride_c,
                                   long long stride_c2, int batch_inner, int batch_outer) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm_strided_batched2: ctx is NULL");
  GH_CHECK_ARG(batch_inner >= 0 && batch_outer >= 0, "ginn_hip_gemm_strided_batched2: negative batch (%d x %d)",
               batch_inner, batch_outer);
  GH_CHECK_ARG(static_cast<long long>(batch_inner) * batch_outer < (1ll << 31),
               "ginn_hip_gemm_strided_batched2: %d x %d slices are too many", batch_inner, batch_outer);
  GH_CHECK_ARG(stride_a2 >= 0 && stride_b2 >= 0 && stride_c2 >= 0, "ginn_hip_gemm_strided_batched2: negative stride");
  GemmArgs a{};
  a.dtype = dtype;
  a.op_a = op_a;
  a.op_b = op_b;
  a.m = m;
  a.n = n;
  a.k = k;
  a.A = A;
  a.lda = lda;
  a.stride_a = stride_a;
  a.B = B;
  a.ldb = ldb;
  a.stride_b = stride_b;
  a.beta = beta;
  a.C = C;
  a.ldc = ldc;
  a.stride_c = stride_c;
  a.batch = batch_inner * batch_outer;
  if (int rc = check_gemm_args("gemm_strided_batched2", a)) return rc;
  if (m == 0 || n == 0 || a.batch == 0) return kOk;
  if (batch_outer == 1) return launch_gemm(ctx, a);
  // All slices in one launch where the small-slice kernel takes the shape; level by level otherwise.
  if (k > 0) {
    GemmArgs two = a;
    two.batch_inner = batch_inner;
    two.stride_a2 = stride_a2;
    two.stride_b2 = stride_b2;
    two.stride_c2 = stride_c2;
    GH_HIP(hipSetDevice(ctx->device));
    const int rc = launch_gemm_bsmall(ctx, two);
    if (rc != kUnsupported) return rc;
  }
  const long long es = static_cast<long long>(dtype_size(dtype));
  a.batch = batch_inner;
  for (int o = 0; o < batch_outer; ++o) {
    a.A = A ? static_cast<const char*>(A) + o * stride_a2 * es : nullptr;
    a.B = B ? static_cast<const char*>(B) + o * stride_b2 * es : nullptr;
    a.C = static_cast<char*>(C) + o * stride_c2 * es;
    if (int rc = launch_gemm(ctx, a)) return rc;
  }
  return kOk;
}

int ginn_hip_gemm_grouped(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                          ginn_hip_op op_a, int m, int k, const void* A,
                          int lda, int groups, const void* const* host_B,
                          const int* host_n, const int* host_ldb, float beta,
                          void* const* host_C, const int* host_ldc) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm_grouped: ctx is NULL");
  GH_CHECK_ARG(dtype_valid(dtype), "ginn_hip_gemm_grouped: unknown dtype %d", dtype);
  GH_CHECK_ARG(groups >= 0, "ginn_hip_gemm_grouped: negative group count");
  if (groups == 0 || m == 0) return kOk;
  GH_CHECK_ARG(host_B && host_n && host_ldb && host_C && host_ldc,
               "ginn_hip_gemm_grouped: NULL table");
  const size_t es = dtype_size(dtype);
  const int vec = static_cast<int>(16 / es);
  // One entry per column of the gathered right-hand side / scattered output.
  std::vector<const void*> bcols;
  std::vector<void*> ccols;
  bool vec_ld = true, vec_c = true;
  for (int g = 0; g < groups; ++g) {
    GH_CHECK_ARG(host_n[g] >= 0, "ginn_hip_gemm_grouped: group %d has n=%d", g, host_n[g]);
    if (host_n[g] == 0) continue;
    GH_CHECK_ARG(host_C[g] != nullptr && (k == 0 || host_B[g] != nullptr),
                 "ginn_hip_gemm_grouped: group %d has a NULL operand", g);
    GH_CHECK_ARG(host_ldb[g] >= (k > 1 ? k : 1), "ginn_hip_gemm_grouped: group %d ldb=%d < k=%d", g, host_ldb[g], k);
    GH_CHECK_ARG(host_ldc[g] >= (m > 1 ? m : 1), "ginn_hip_gemm_grouped: group %d ldc=%d < m=%d", g, host_ldc[g], m);
    const bool one = host_n[g] == 1;
    vec_ld = vec_ld && reinterpret_cast<uintptr_t>(host_B[g]) % 16 == 0 && (one || host_ldb[g] % vec == 0);
    vec_c = vec_c && reinterpret_cast<uintptr_t>(host_C[g]) % (4 * es) == 0 && (one || host_ldc[g] % 4 == 0);
    for (int j = 0; j < host_n[g]; ++j) {
      bcols.push_back(static_cast<const char*>(host_B[g]) + es * (size_t)j * host_ldb[g]);
      ccols.push_back(static_cast<char*>(host_C[g]) + es * (size_t)j * host_ldc[g]);
    }
  }
  const size_t total = bcols.size();
  if (total == 0) return kOk;
  GH_CHECK_ARG(total <= 0x7fffffffu, "ginn_hip_gemm_grouped: too many columns");
  std::lock_guard<std::mutex> lock(ctx->mutex);
  const size_t table = total * sizeof(void*);
  // The staging ring holds 1 MiB: split larger tables into slices.
  const size_t slice = 32768;
  for (size_t i = 0; i < total; i += slice) {
    const size_t cnt = total - i < slice ? total - i : slice;
    if (int rc = stage_to_workspace(ctx, i * sizeof(void*), bcols.data() + i, cnt * sizeof(void*))) return rc;
    if (int rc = stage_to_workspace(ctx, table + i * sizeof(void*), ccols.data() + i, cnt * sizeof(void*))) return rc;
  }
  GemmArgs a{};
  a.dtype = dtype;
  a.op_a = op_a;
  a.op_b = GINN_HIP_OP_N;
  a.m = m;
  a.n = static_cast<int>(total);
  a.k = k;
  a.A = A;
  a.lda = lda;
  a.beta = beta;
  a.batch = 1;
  a.bcols = static_cast<const void* const*>(ctx->workspace);
  a.ccols = reinterpret_cast<void* const*>(static_cast<char*>(ctx->workspace) + table);
  a.cols_vec_ld = vec_ld;
  a.cols_vec_c = vec_c;
  a.cols_in_workspace = true;
  if (int rc = check_gemm_args("ginn_hip_gemm_grouped", a)) return rc;
  GH_HIP(hipSetDevice(ctx->device));
  return launch_gemm_generic(ctx, a);
}

int ginn_hip_gemm_gathered(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                           ginn_hip_op op_a, ginn_hip_op op_b, int m, int n,
                           int k, const void* A, int lda, const void* B,
                           int ldb, const void* const* dev_b_cols, float beta,
                           void* C, int ldc, void* const* dev_c_cols,
                           int cols_aligned) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm_gathered: ctx is NULL");
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
  a.bcols = dev_b_cols;
  a.ccols = dev_c_cols;
  a.cols_vec_ld = cols_aligned != 0;
  a.cols_vec_c = cols_aligned != 0;
  if (int rc = check_gemm_args("ginn_hip_gemm_gathered", a)) return rc;
  if (m == 0 || n == 0) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  // Without a table this is an ordinary product and takes the ordinary route.
  if (!a.bcols && !a.ccols) return launch_gemm(ctx, a);
  if (int rc = launch_gemm_ksplit(ctx, a); rc != kUnsupported) return rc;
  return launch_gemm_generic(ctx, a);
}

int ginn_hip_gemm_outer_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int m, int n, int k,
                            const void* const* dev_a_cols, const void* const* dev_b_cols, float beta, void* C,
                            int ldc, int cols_aligned) {
  GH_CHECK_ARG(ctx, "ginn_hip_gemm_outer_sum: ctx is NULL");
  GH_CHECK_ARG(k == 0 || (dev_a_cols && dev_b_cols), "ginn_hip_gemm_outer_sum: NULL table");
  GemmArgs a{};
  a.dtype = dtype;
  a.op_a = GINN_HIP_OP_N;
  a.op_b = GINN_HIP_OP_T;
  a.m = m;
  a.n = n;
  a.k = k;
  a.beta = beta;
  a.C = C;
  a.ldc = ldc;
  a.batch = 1;
  if (k > 0) {
    a.acols = dev_a_cols;
    a.bcols = dev_b_cols;
  } else {  // an empty sum: C <- beta * C through the ordinary route
    a.lda = m > 1 ? m : 1;
    a.ldb = n > 1 ? n : 1;
  }
  a.cols_vec_ld = cols_aligned != 0;
  if (int rc = check_gemm_args("ginn_hip_gemm_outer_sum", a)) return rc;
  if (m == 0 || n == 0) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  if (k == 0) return launch_gemm(ctx, a);
  if (int rc = launch_gemm_ksplit(ctx, a); rc != kUnsupported) return rc;
  return launch_gemm_generic(ctx, a);
}

int ginn_hip_affine_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                        ginn_hip_act act, int m, int n, int pairs,
                        const void* const* host_W, const void* const* host_X,
                        const int* host_k, const void* bias, void* pre,
                        void* Y) {
  GH_CHECK_ARG(ctx, "ginn_hip_affine_fwd: ctx is NULL");
  GH_CHECK_ARG(dtype_valid(dtype), "ginn_hip_affine_fwd: unknown dtype %d", dtype);
  GH_CHECK_ARG(pairs >= 1, "ginn_hip_affine_fwd: needs at least one (W, X) pair");
  GH_CHECK_ARG(host_W && host_X && host_k, "ginn_hip_affine_fwd: NULL table");
  GH_CHECK_ARG(m >= 0 && n >= 0, "ginn_hip_affine_fwd: negative dimension");
  GH_CHECK_ARG(act >= GINN_HIP_ACT_IDENTITY && act <= GINN_HIP_ACT_SOFTMAX,
               "ginn_hip_affine_fwd: activation %d cannot be carried by an Affine", act);
  if (m == 0 || n == 0) return kOk;
  GH_CHECK_ARG(Y != nullptr, "ginn_hip_affine_fwd: Y is NULL");
  GH_CHECK_ARG(act != GINN_HIP_ACT_SOFTMAX || pre != nullptr,
               "ginn_hip_affine_fwd: SOFTMAX needs the pre-activation buffer");
  // The buffer the products accumulate into: the stored pre-activation when
  // there is one, the output otherwise (ginn/node/affine.h:44-46).
  void* acc_buf = pre ? pre : Y;
  const bool softmax = act == GINN_HIP_ACT_SOFTMAX;
  for (int p = 0; p < pairs; ++p) {
    const bool first = p == 0, last = p == pairs - 1;
    GemmArgs a{};
    a.dtype = dtype;
    a.op_a = GINN_HIP_OP_N;
    a.op_b = GINN_HIP_OP_N;
    a.m = m;
    a.n = n;
    a.k = host_k[p];
    a.A = host_W[p];
    a.lda = m;
    a.B = host_X[p];
    a.ldb = host_k[p] > 1 ? host_k[p] : 1;
    a.beta = first ? 0.f : 1.f;
    a.ldc = m;
    a.batch = 1;
    a.bias = first ? bias : nullptr;
    if (last && !softmax) {
      // Final product carries the activation; writes Y and, if kept, pre.
      a.C = Y;
      a.pre = pre;
      a.act = act;
    } else {
      a.C = acc_buf;
    }
    if (int rc = launch_gemm(ctx, a)) return rc;
  }
  if (softmax) return launch_softmax_fwd(ctx, dtype, m, n, pre, Y);
  return kOk;
}

}  // extern "C"
