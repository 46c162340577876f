// fp32 products with a small output: one launch, the sum over K split inside
// the workgroup.  The merged products of an autobatched recurrent cell
// (ginn/autobatch.h:149-183: W [1024 x 384] times the states of the sequences
// still alive, and its gradients) have a few hundred 32 x 32 output tiles at
// most.  Tiles of 64 x 64 with K split over workgroups fill the machine but
// need a second launch that folds the partial sums, which costs as much as
// the product itself (4 us against 7).  Here a workgroup of 16 waves owns one
// 32 x 32 tile and every wave walks one sixteenth of K on its own, without a
// barrier in the loop: an operand whose rows are contiguous in memory arrives
// in the matrix instruction's layout as it is loaded, a K-contiguous one is
// turned through a slice of LDS that belongs to the wave.  The 16 partial
// tiles meet in LDS and are added in wave order.
#include "common.h"

namespace ginn_hip {
namespace {
namespace ksplit {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// Loads through pointers of the global address space: the compiler then issues
// global loads, which do not count against the LDS counter as flat loads do.
typedef const float __attribute__((address_space(1)))* gfloat;
typedef const f32x4 __attribute__((address_space(1)))* gfloat4;
typedef const float* const __attribute__((address_space(1)))* gtable;
__device__ __forceinline__ float gload(const float* p) { return *(gfloat)p; }
__device__ __forceinline__ f32x4 gload4(const float* p) { return *(gfloat4)p; }
__device__ __forceinline__ const float* gload_ptr(const float* const* p) { return *(gtable)p; }

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kStep = 16;   // values of K per step of a wave
constexpr int kDepth = 4;   // steps whose operands are on their way
// Two tile sizes.  32 x 32 (`v_mfma_f32_32x32x2f32`: a lane holds row lane % 32 and supplies one of
// the instruction's 2 values of K, 8 instructions per step) and 16 x 16 (`v_mfma_f32_16x16x4f32`:
// row lane % 16, one of 4 values of K, 4 instructions per step).  A tile is worked on by ONE CU,
// whose fp32 matrix pipes do 256 flops per cycle: a 32 x 32 tile over K = 1024 keeps it busy for
// 8192 cycles (3.9 us) however the waves share the work, so a product with few 32 x 32 tiles (the
// W^T dY of the recurrent cell: 60-96) is cut into 16 x 16 tiles instead, four times as many.
template <int TS>
struct Shape {
  static constexpr int kGroups = 64 / TS;        // lane groups = values of K per matrix instruction
  static constexpr int kValues = kStep / kGroups;  // values of K a lane supplies per step = instructions per step
  static constexpr int kAcc = TS * TS / 64;      // accumulator registers
};
// A K-contiguous operand of a 32-row tile is read as 64-byte runs (4 lanes per row, 16 rows per
// load) and turned into the matrix instruction's layout (one row per lane, 8 consecutive values)
// through a slice of LDS that belongs to the wave: [32 rows][4 vectors of 4], vector q of row r at
// position q ^ ((r >> 2) & 3) (no bank conflicts either way).  With 16 rows a lane's 4 consecutive
// values ARE one 16-byte load, 4 lanes per row: no staging.
constexpr int kStageFloats = 32 * kStep;
static_assert(2 * kStageFloats == 32 * 32, "the staging slices and the partial tiles share the LDS");

struct Params {
  const float* A;
  const float* B;
  float* C;
  int m, n, k;
  int lda, ldb, ldc;
  float beta;
  const float* bias;
  float* pre;
  int act;
  const float* const* acols;  // A by stored columns (op_a N only)
  const float* const* bcols;  // B by stored columns
  float* const* ccols;        // C by columns
  int k_per_wave;             // a multiple of kStep
};

// One operand of a wave: TS rows of op(X) (rows of A, columns of B).  KC: K is
// the contiguous dimension in memory.  TABLE: the stored columns are given by
// their addresses.  Every load is unconditional from a clamped, valid address;
// what lies outside the operand is zeroed when the values are used, so that
// nothing waits for a load where it is issued.
template <int TS, bool KC, bool TABLE>
struct Operand {
  static constexpr int kGroups = Shape<TS>::kGroups, kValues = Shape<TS>::kValues;
  const float* row_lo = nullptr;  // KC, 32 rows: rows lane / 4 and lane / 4 + 16 (clamped); 16 rows: row lane % 16
  const float* row_hi = nullptr;
  const float* base = nullptr;    // otherwise: the lane's row (clamped) in the first stored column
  const float* const* cols = nullptr;
  long long ld = 0;
  int row = 0;
  bool ok = false;  // row lane % TS lies inside the operand

  __device__ __forceinline__ void init(const float* X, int ld_, const float* const* table, int first, int extent,
                                       int lane) {
    ld = ld_;
    cols = table;
    ok = first + (lane % TS) < extent;
    if (KC && TS == 32) {
      const int lo = min(first + (lane >> 2), extent - 1), hi = min(first + (lane >> 2) + 16, extent - 1);
      row_lo = TABLE ? gload_ptr(table + lo) : X + lo * ld;
      row_hi = TABLE ? gload_ptr(table + hi) : X + hi * ld;
    } else if (KC) {
      const int r = min(first + (lane % TS), extent - 1);
      row_lo = TABLE ? gload_ptr(table + r) : X + r * ld;
    } else {
      row = min(first + (lane % TS), extent - 1);
      base = TABLE ? nullptr : X + row;
    }
  }

  // The lane's share of K = j .. j + 15, j < k_end.  KC, 32 rows: values
  // j + 4 (lane % 4) + 0 .. 3 of its two rows; otherwise the kValues values
  // j + kValues (lane / TS) + t of its row.  Positions beyond k_end repeat earlier ones.
  __device__ __forceinline__ void fetch(int j, int k_end, int lane, float (&v)[kValues]) const {
    if (KC && TS == 32) {
      // k_end is a multiple of 4 (the launcher sees to it): a vector that would
      // begin beyond it repeats the last one.
      const int kk = min(j + 4 * (lane & 3), k_end - 4);
      const f32x4 lo = gload4(row_lo + kk);
      const f32x4 hi = gload4(row_hi + kk);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        v[t] = lo[t];
        v[4 + t] = hi[t];
      }
    } else if (KC) {
      const int kk = min(j + 4 * (lane / TS), k_end - 4);
      const f32x4 q = gload4(row_lo + kk);
#pragma unroll
      for (int t = 0; t < 4; ++t) v[t] = q[t];
    } else {
      const int kk = j + kValues * (lane / TS);
      const float* from[kValues];
#pragma unroll
      for (int t = 0; t < kValues; ++t) {
        const int at = min(kk + t, k_end - 1);
        from[t] = TABLE ? gload_ptr(cols + at) + row : base + at * ld;
      }
#pragma unroll
      for (int t = 0; t < kValues; ++t) v[t] = gload(from[t]);
    }
  }

  // v as the matrix instruction wants it: the values K = j + kValues (lane / TS) + t
  // of row lane % TS, zero outside the operand.  KC with 32 rows: through the wave's own LDS
  // slice (a wave's LDS accesses execute in order, so no barrier is needed
  // between this step's reads and the next step's writes).
  __device__ __forceinline__ void arrange(float* stage, int j, int k_end, int lane, float (&v)[kValues]) const {
    if constexpr (KC && TS == 32) {
      const int srow = lane >> 2, q = lane & 3;
      const int swz = (srow >> 2) & 3;  // the same for srow and srow + 16
      *reinterpret_cast<f32x4*>(stage + srow * kStep + ((q ^ swz) << 2)) = f32x4{v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4*>(stage + (srow + 16) * kStep + ((q ^ swz) << 2)) = f32x4{v[4], v[5], v[6], v[7]};
      const int r = lane & 31, h = lane >> 5, rs = (r >> 2) & 3;
      const f32x4 q0 = *reinterpret_cast<const f32x4*>(stage + r * kStep + (((2 * h) ^ rs) << 2));
      const f32x4 q1 = *reinterpret_cast<const f32x4*>(stage + r * kStep + (((2 * h + 1) ^ rs) << 2));
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        v[t] = q0[t];
        v[4 + t] = q1[t];
      }
    }
    const int kk = j + kValues * (lane / TS);
#pragma unroll
    for (int t = 0; t < kValues; ++t) v[t] = ok && kk + t < k_end ? v[t] : 0.f;
  }
};

template <int TS, bool AKC, bool BKC, bool ATAB, bool BTAB>
__global__ __launch_bounds__(kThreads) void gemm_ksplit_kernel(Params p) {
  constexpr int kValues = Shape<TS>::kValues, kAcc = Shape<TS>::kAcc;
  typedef float acc_t __attribute__((ext_vector_type(kAcc)));
  __shared__ __align__(16) float lds[kWaves * TS * TS];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register: K ranges and branches are per wave
  const int m0 = blockIdx.x * TS, n0 = blockIdx.y * TS;
  Operand<TS, AKC, ATAB> opa;
  Operand<TS, BKC, BTAB> opb;
  opa.init(p.A, p.lda, p.acols, m0, p.m, lane);
  opb.init(p.B, p.ldb, p.bcols, n0, p.n, lane);
  float* stage_a = lds + wave * 2 * kStageFloats;  // used with 32 rows only
  float* stage_b = stage_a + kStageFloats;
  const int k_begin = wave * p.k_per_wave;
  const int k_end = min(p.k, k_begin + p.k_per_wave);

  acc_t acc;
#pragma unroll
  for (int e = 0; e < kAcc; ++e) acc[e] = 0.f;
  if (k_begin < k_end) {
    // Lane group g of the wave supplies K = j + kValues g + t in the t-th instruction of a step.
    float a[kDepth][kValues], b[kDepth][kValues];
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      if (k_begin + kStep * d < k_end) {
        opa.fetch(k_begin + kStep * d, k_end, lane, a[d]);
        opb.fetch(k_begin + kStep * d, k_end, lane, b[d]);
      }
    }
    for (int j = k_begin; j < k_end; j += kStep * kDepth) {
#pragma unroll
      for (int d = 0; d < kDepth; ++d) {
        if (j + kStep * d < k_end) {
          opa.arrange(stage_a, j + kStep * d, k_end, lane, a[d]);
          opb.arrange(stage_b, j + kStep * d, k_end, lane, b[d]);
#pragma unroll
          for (int t = 0; t < kValues; ++t) {
            if constexpr (TS == 32) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[d][t], b[d][t], acc, 0, 0, 0);
            else acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][t], b[d][t], acc, 0, 0, 0);
          }
          const int next = j + kStep * (d + kDepth);
          if (next < k_end) {
            opa.fetch(next, k_end, lane, a[d]);
            opb.fetch(next, k_end, lane, b[d]);
          }
        }
      }
    }
  }
  __syncthreads();  // the partial tiles take the place of the staging slices
  float* mine = lds + wave * TS * TS;
  if constexpr (TS == 32) {
    // Accumulator element 4 q + i of a lane is row 8 q + 4 h + i of column r.
    // A column's 32 rows lie in 8 chunks of 4; chunk c of column r sits at
    // position c ^ (r & 7), which spreads the 16-byte stores of a wave over all banks.
    const int r = lane & 31, h = lane >> 5;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int chunk = 2 * q + h;
      f32x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = acc[4 * q + i];
      *reinterpret_cast<f32x4*>(mine + r * TS + ((chunk ^ (r & 7)) << 2)) = v;
    }
  } else {
    // Accumulator element i of a lane is row 4 (lane / 16) + i of column lane % 16: the wave's
    // 16-byte stores fill the 16 x 16 tile, column after column, without gaps.
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = acc[i];
    *reinterpret_cast<f32x4*>(mine + (lane & 15) * TS + ((lane >> 4) << 2)) = v;
  }
  __syncthreads();
  if (threadIdx.x >= TS * TS) return;
  const int row = threadIdx.x % TS, col = threadIdx.x / TS;
  const int at = TS == 32 ? col * TS + ((((row >> 2) ^ (col & 7)) << 2) | (row & 3)) : col * TS + row;
  float sum = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) sum += lds[w * TS * TS + at];
  const int grow = m0 + row, gcol = n0 + col;
  if (grow >= p.m || gcol >= p.n) return;
  const long long off = static_cast<long long>(gcol) * p.ldc + grow;
  float* out = p.ccols ? p.ccols[gcol] + grow : p.C + off;
  float* keep = p.pre ? p.pre + off : nullptr;
  if (p.beta != 0.f) sum += p.beta * (keep ? *keep : *out);
  if (p.bias) sum += p.bias[grow];
  if (keep) *keep = sum;
  if (p.act != GINN_HIP_ACT_IDENTITY) sum = act_forward<kFastMath<F32>>(p.act, sum);
  *out = sum;
}

template <int TS, bool AKC, bool BKC>
int launch_layout(ginn_hip_ctx* ctx, const Params& p) {
  const dim3 grid((p.m + TS - 1) / TS, (p.n + TS - 1) / TS);
  // Column tables: A only when its columns are what is stored (op_a N).
  if (!AKC && p.acols) {
    if (p.bcols) gemm_ksplit_kernel<TS, AKC, BKC, true, true><<<grid, kThreads, 0, ctx->stream>>>(p);
    else gemm_ksplit_kernel<TS, AKC, BKC, true, false><<<grid, kThreads, 0, ctx->stream>>>(p);
  } else {
    if (p.bcols) gemm_ksplit_kernel<TS, AKC, BKC, false, true><<<grid, kThreads, 0, ctx->stream>>>(p);
    else gemm_ksplit_kernel<TS, AKC, BKC, false, false><<<grid, kThreads, 0, ctx->stream>>>(p);
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

template <int TS>
int launch_tile(ginn_hip_ctx* ctx, const Params& p, bool akc, bool bkc) {
  if (akc) return bkc ? launch_layout<TS, true, true>(ctx, p) : launch_layout<TS, true, false>(ctx, p);
  return bkc ? launch_layout<TS, false, true>(ctx, p) : launch_layout<TS, false, false>(ctx, p);
}

}  // namespace ksplit
}  // namespace

int launch_gemm_ksplit(ginn_hip_ctx* ctx, const GemmArgs& a) {
  using namespace ksplit;
  if (a.dtype != GINN_HIP_F32 || a.batch != 1) return kUnsupported;
  if (a.pre && a.ccols) return kUnsupported;
  // Every wave reads its share of both operand panels itself: that pays while a
  // wave's share of K is at most twice what it asks for at once (kDepth steps)
  // and there is one workgroup per CU at most (measured against the kernels
  // that share operands through LDS and fold a split K in a second launch:
  // 1024 x 64 x 2048 7.8-9.5 against 12.9 us, 2048 x 128 x 2048 16.2-17.5
  // against 18.5-19.5 us; 4096 x 64 x 4096 30.9-33.7 against 26.5-27.4 us).
  if (a.k < 32 || a.k > 2 * kWaves * kStep * kDepth) return kUnsupported;
  const long long tiles = static_cast<long long>((a.m + 31) / 32) * ((a.n + 31) / 32);
  if (tiles > ctx->num_cus) return kUnsupported;
  // A narrow right-hand side under a left operand of several MiB is one pass over that operand at
  // memory speed: the skinny kernels' case.
  if (a.n <= 16 && static_cast<long long>(a.m) * a.k > (1ll << 20)) return kUnsupported;
  const bool akc = a.op_a == GINN_HIP_OP_T, bkc = a.op_b == GINN_HIP_OP_N;
  if (a.acols && akc) return kUnsupported;
  // The longer sums of a handful of tiles with both operands K-contiguous: the split-K kernels are ahead
  // (64 x 64 x 2048: 7.4 against 9.5 us; from 256 x 256 on this kernel is, 9.7 against 12.4 us).
  if (a.k > kWaves * kStep * kDepth && akc && bkc && tiles <= 16 && !a.bcols && !a.ccols) return kUnsupported;
  Params p;
  p.A = static_cast<const float*>(a.A);
  p.B = static_cast<const float*>(a.B);
  p.C = static_cast<float*>(a.C);
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.lda = a.lda;
  p.ldb = a.ldb;
  p.ldc = a.ldc;
  p.beta = a.beta;
  p.bias = static_cast<const float*>(a.bias);
  p.pre = static_cast<float*>(a.pre);
  p.act = a.act;
  p.acols = reinterpret_cast<const float* const*>(a.acols);
  p.bcols = reinterpret_cast<const float* const*>(a.bcols);
  p.ccols = reinterpret_cast<float* const*>(a.ccols);
  p.k_per_wave = ((a.k + kWaves - 1) / kWaves + kStep - 1) / kStep * kStep;
  // K-contiguous operands are read as 16-byte vectors, also at the end of K.
  if ((akc || bkc) && a.k % 4 != 0) return kUnsupported;
  auto aligned = [](const void* ptr, int ld) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && ld % 4 == 0; };
  if (akc && !aligned(a.A, a.lda)) return kUnsupported;
  if (bkc && !(a.bcols ? a.cols_vec_ld : aligned(a.B, a.ldb))) return kUnsupported;
  // Few 32 x 32 tiles with a long sum: 16 x 16 tiles put four times as many CUs to work (see Shape),
  // and read the operands twice as often.  Measured where that stops to pay: with a row-contiguous A
  // two small tiles per CU are still ahead (512 x 256 x 1024: 7.9 us on 512 small tiles, 9.5 us on
  // 128 large ones), with both operands K-contiguous one per CU is the limit (384 x 256 x 1024:
  // 9.7 us on 384 small tiles, 8.8 us on 96 large ones).
  const long long small_tiles = static_cast<long long>((a.m + 15) / 16) * ((a.n + 15) / 16);
  if (tiles * 2 <= ctx->num_cus && a.k >= 256 && small_tiles <= (akc ? 1 : 2) * static_cast<long long>(ctx->num_cus))
    return launch_tile<16>(ctx, p, akc, bkc);
  return launch_tile<32>(ctx, p, akc, bkc);
}

}  // namespace ginn_hip
