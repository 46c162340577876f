// Generic LDS-tiled MFMA product for any shape, leading dimension and
// alignment: column-major C = op(A) op(B) + beta C with an optional
// bias + nonlinearity epilogue, one launch for a whole strided batch.
//
// Both operands are seen as a logical [R x K] matrix (R = m for A, R = n for
// B) whose element (r, k) lives at p[r * ld + k] when K is the contiguous
// dimension (op(A) = A^T, op(B) = B) or at p[k * ld + r] when R is
// (op(A) = A, op(B) = B^T).  Tiles go global -> registers -> LDS; the next
// K-slab is fetched into registers while the current one feeds the matrix
// cores.
//
// This header holds the kernel template; each gemm_generic_<dtype>_<v|s>.hip
// instantiates one scalar type with vector (v) or element-wise (s) global
// loads so that the variants compile in parallel.
#ifndef GINN_HIP_GEMM_GENERIC_H
#define GINN_HIP_GEMM_GENERIC_H

#include <type_traits>

#include "common.h"

namespace ginn_hip {
namespace generic {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;  // 4 waves arranged 2 x 2 over the block tile

struct KParams {
  const void* A;
  const void* B;
  void* C;
  int m, n, k;
  int lda, ldb, ldc;
  long long sa, sb, sc;
  float beta;
  const void* bias;
  void* pre;
  int act;
  int vec_c;  // C (and pre) may be accessed as 4-element vectors
  // Grouped launch: B and C are given per (virtual) column, n = their count.
  const void* const* bcols;
  void* const* ccols;
  // A given by the bases of its stored columns (only for A stored [m x k]:
  // entry j is column j, position j along the sum).
  const void* const* acols;
  // Split-K (batch == 1 only): blockIdx.z selects a K range of k_chunk
  // (a multiple of the K slab); the fp32 partial tile goes to
  // partial[z][col * m + row] and a second kernel folds the splits and
  // applies the epilogue.
  int splits;
  int k_chunk;
  float* partial;
};

// Per-dtype tile constants.  VEC elements = 16 bytes.
template <typename T>
struct Cfg;
template <>
struct Cfg<F32> {
  static constexpr int BK = 16, VEC = 4, KSTEP = 2;
  using vec_t = f32x4;
};
template <>
struct Cfg<F16> {
  static constexpr int BK = 32, VEC = 8, KSTEP = 16;
  using vec_t = u16x8;
};
template <>
struct Cfg<BF16> {
  static constexpr int BK = 32, VEC = 8, KSTEP = 16;
  using vec_t = u16x8;
};

// LDS tile of one operand.  16-bit types: [row][k] (K innermost, so that one
// lane reads its 8 consecutive k of one row as 16 bytes).  fp32: [k][row]
// (row innermost: the 32 lanes of an MFMA operand read 32 consecutive rows).
template <typename T, int ROWS>
struct LdsTile;
template <int ROWS>
struct LdsTile<F32, ROWS> {
  static constexpr int LD = ROWS + 4;
  alignas(16) float d[Cfg<F32>::BK * LD];
  __device__ __forceinline__ float& at(int row, int k) { return d[k * LD + row]; }
};
template <int ROWS>
struct LdsTile<F16, ROWS> {
  static constexpr int LD = Cfg<F16>::BK + 8;
  alignas(16) uint16_t d[ROWS * LD];
  __device__ __forceinline__ uint16_t& at(int row, int k) { return d[row * LD + k]; }
};
template <int ROWS>
struct LdsTile<BF16, ROWS> {
  static constexpr int LD = Cfg<BF16>::BK + 8;
  alignas(16) uint16_t d[ROWS * LD];
  __device__ __forceinline__ uint16_t& at(int row, int k) { return d[row * LD + k]; }
};

// Global -> register fetch of one [ROWS x BK] slab.  KC: K contiguous in
// memory.  VECLD: 16-byte loads are legal (aligned base, ld and extents along
// the contiguous dimension are multiples of VEC); otherwise element loads.
template <typename T, int ROWS, bool KC, bool VECLD>
struct Fetch {
  using S = typename T::storage;
  using V = typename Cfg<T>::vec_t;
  static constexpr int BK = Cfg<T>::BK;
  static constexpr int VEC = Cfg<T>::VEC;
  static constexpr int NV = ROWS * BK / VEC / kThreads;
  static_assert(ROWS * BK % (VEC * kThreads) == 0, "slab must split evenly");
  V r[NV];

  __device__ __forceinline__ static void coords(int i, int tid, int& row, int& kk) {
    const int v = tid + i * kThreads;
    if (KC) {
      row = v / (BK / VEC);
      kk = (v % (BK / VEC)) * VEC;
    } else {
      kk = v / (ROWS / VEC);
      row = (v % (ROWS / VEC)) * VEC;
    }
  }

  // `cols`, when not NULL, gives the base of every STORED column of the
  // operand instead of p + column * ld: row r of the logical [R x K] operand
  // when K is contiguous (a gathered right-hand side), position k along K
  // otherwise (the same columns as the transposed operand of a product that
  // sums over them).
  __device__ __forceinline__ void load(const S* __restrict__ p, int ld, int row0,
                                       int k0, int R, int K, int tid,
                                       const S* const* __restrict__ cols = nullptr) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int row, kk;
      coords(i, tid, row, kk);
      const int gr = row0 + row, gk = k0 + kk;
      V val;
#pragma unroll
      for (int j = 0; j < VEC; ++j) val[j] = S(0);
      if (VECLD) {
        if (gr < R && gk < K) {
          if (cols) {
            val = *reinterpret_cast<const V*>(KC ? cols[gr] + gk : cols[gk] + gr);
          } else {
            const long long off = KC ? (long long)gr * ld + gk : (long long)gk * ld + gr;
            val = *reinterpret_cast<const V*>(p + off);
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const int r_j = KC ? gr : gr + j;
          const int k_j = KC ? gk + j : gk;
          if (r_j < R && k_j < K) {
            if (cols) {
              val[j] = KC ? cols[r_j][k_j] : cols[k_j][r_j];
            } else {
              const long long off = KC ? (long long)r_j * ld + k_j : (long long)k_j * ld + r_j;
              val[j] = p[off];
            }
          }
        }
      }
      r[i] = val;
    }
  }

  __device__ __forceinline__ void store(LdsTile<T, ROWS>& t, int tid) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int row, kk;
      coords(i, tid, row, kk);
      // The register vector runs along K (KC) or along rows (!KC); the LDS
      // tile is K-innermost for 16-bit types and row-innermost for fp32.
      constexpr bool kLdsKInner = !std::is_same<T, F32>::value;
      if (KC == kLdsKInner) {
        *reinterpret_cast<V*>(&t.at(row, kk)) = r[i];
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if (KC)
            t.at(row, kk + j) = r[i][j];
          else
            t.at(row + j, kk) = r[i][j];
        }
      }
    }
  }
};

// One K-slab of matrix-core work for a wave: TM x TN tiles of 32 x 32.
template <typename T, int BM, int BN, int TM, int TN>
__device__ __forceinline__ void mma_slab(LdsTile<T, BM>& as, LdsTile<T, BN>& bs,
                                         f32x16 (&acc)[TM][TN], int wm, int wn,
                                         int lane) {
  constexpr int BK = Cfg<T>::BK;
  constexpr int KSTEP = Cfg<T>::KSTEP;
  const int l32 = lane & 31, lhi = lane >> 5;
#pragma unroll
  for (int ks = 0; ks < BK / KSTEP; ++ks) {
    if constexpr (std::is_same<T, F32>::value) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = as.at(wm + i * 32 + l32, ks * 2 + lhi);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = bs.at(wn + j * 32 + l32, ks * 2 + lhi);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    } else {
      u16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = *reinterpret_cast<const u16x8*>(&as.at(wm + i * 32 + l32, ks * 16 + lhi * 8));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = *reinterpret_cast<const u16x8*>(&bs.at(wn + j * 32 + l32, ks * 16 + lhi * 8));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if constexpr (std::is_same<T, F16>::value)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(f16x8, a[i]), __builtin_bit_cast(f16x8, b[j]), acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, a[i]), __builtin_bit_cast(bf16x8, b[j]), acc[i][j], 0, 0, 0);
        }
    }
  }
}

template <typename T, int BM, int BN, bool AKC, bool BKC, bool VECLD>
__global__ __launch_bounds__(kThreads) void gemm_generic_kernel(KParams p) {
  using S = typename T::storage;
  constexpr int BK = Cfg<T>::BK;
  constexpr int WM = BM / 2, WN = BN / 2;   // wave tile
  constexpr int TM = WM / 32, TN = WN / 32; // 32 x 32 MFMA tiles per wave
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold one MFMA tile");

  __shared__ LdsTile<T, BM> as[2];
  __shared__ LdsTile<T, BN> bs[2];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = (wave & 1) * WM;
  const int wn = (wave >> 1) * WN;
  const int m0 = blockIdx.x * BM;
  const int n0 = blockIdx.y * BN;
  const bool split = p.splits > 1;
  const long long bz = split ? 0 : blockIdx.z;
  const int k_begin = split ? blockIdx.z * p.k_chunk : 0;
  const int k_end = split ? min(p.k, k_begin + p.k_chunk) : p.k;

  const S* A = static_cast<const S*>(p.A) + bz * p.sa;
  const S* B = static_cast<const S*>(p.B) + bz * p.sb;
  S* C = static_cast<S*>(p.C) + bz * p.sc;
  S* P = p.pre ? static_cast<S*>(p.pre) + bz * p.sc : nullptr;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Slab kt is multiplied from LDS buffer kt % 2 while slabs kt + 1 .. kt +
  // kDepth - 1 are on their way in registers: a slab arrives kDepth - 1
  // iterations after it was asked for, which covers the memory latency (one
  // iteration of a 64 x 64 tile is a fraction of it), and there is one barrier
  // per iteration: it separates the products on a buffer from the next
  // store into it.  Register set j holds slab kt with kt % kDepth == j.
  constexpr int kDepth = 4;
  Fetch<T, BM, AKC, VECLD> fa[kDepth];
  Fetch<T, BN, BKC, VECLD> fb[kDepth];
  const S* const* bcols = reinterpret_cast<const S* const*>(p.bcols);
  const S* const* acols = reinterpret_cast<const S* const*>(p.acols);

  const int ktiles = (k_end - k_begin + BK - 1) / BK;
  if (ktiles > 0) {
#pragma unroll
    for (int j = 0; j < kDepth; ++j)
      if (j < ktiles) {
        fa[j].load(A, p.lda, m0, k_begin + j * BK, p.m, k_end, tid, acols);
        fb[j].load(B, p.ldb, n0, k_begin + j * BK, p.n, k_end, tid, bcols);
      }
    fa[0].store(as[0], tid);
    fb[0].store(bs[0], tid);
    __syncthreads();
    for (int kt0 = 0; kt0 < ktiles; kt0 += kDepth) {
#pragma unroll
      for (int j = 0; j < kDepth; ++j) {
        const int kt = kt0 + j;
        if (kt < ktiles) {
          if (kt + kDepth < ktiles) {  // set j (slab kt) went to LDS an iteration ago
            fa[j].load(A, p.lda, m0, k_begin + (kt + kDepth) * BK, p.m, k_end, tid, acols);
            fb[j].load(B, p.ldb, n0, k_begin + (kt + kDepth) * BK, p.n, k_end, tid, bcols);
          }
          mma_slab<T, BM, BN, TM, TN>(as[j & 1], bs[j & 1], acc, wm, wn, lane);
          if (kt + 1 < ktiles) {
            fa[(j + 1) % kDepth].store(as[(j + 1) & 1], tid);
            fb[(j + 1) % kDepth].store(bs[(j + 1) & 1], tid);
          }
          __syncthreads();
        }
      }
    }
  }

  // Epilogue.  Accumulator element e of tile (i, j) is row
  // 8 * (e / 4) + 4 * (lane / 32) + e % 4, column lane % 32.
  const int l32 = lane & 31, lhi = lane >> 5;
  if (split) {
    float* part = p.partial + (size_t)blockIdx.z * p.m * p.n;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn + j * 32 + l32;
        if (col >= p.n) continue;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          // The four values of a lane are consecutive rows of one column:
          // one 16-byte store when the partial columns keep that alignment.
          const int row0 = m0 + wm + i * 32 + 8 * b + 4 * lhi;
          if (p.m % 4 == 0 && row0 + 3 < p.m) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * b + e];
            *reinterpret_cast<f32x4*>(part + (size_t)col * p.m + row0) = v;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (row0 + e < p.m) part[(size_t)col * p.m + row0 + e] = acc[i][j][4 * b + e];
          }
        }
      }
    return;
  }
  const S* bias = static_cast<const S*>(p.bias);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn + j * 32 + l32;
      if (col >= p.n) continue;
      // Column bases of the output, of the stored pre-activation and of the
      // matrix that beta scales (the pre-activation buffer when there is one).
      S* ccol = p.ccols ? static_cast<S*>(p.ccols[col]) : C + (long long)col * p.ldc;
      S* pcol = P ? P + (long long)col * p.ldc : nullptr;
      const S* cin = pcol ? pcol : ccol;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int row = m0 + wm + i * 32 + 8 * b + 4 * lhi;
        if (row >= p.m) continue;
        const int off = row;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * b + e];
        const bool full = p.vec_c && row + 3 < p.m;
        if (full) {
          if (p.beta != 0.f) {
            if constexpr (std::is_same<T, F32>::value) {
              const f32x4 old = *reinterpret_cast<const f32x4*>(cin + off);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] += p.beta * old[e];
            } else {
              const u16x4 old = *reinterpret_cast<const u16x4*>(cin + off);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] += p.beta * to_float<T>(old[e]);
            }
          }
          if (bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += to_float<T>(bias[row + e]);
          }
          if constexpr (std::is_same<T, F32>::value) {
            if (pcol) *reinterpret_cast<f32x4*>(pcol + off) = f32x4{v[0], v[1], v[2], v[3]};
            if (p.act != GINN_HIP_ACT_IDENTITY) act_forward_n<kFastMath<T>, 4>(p.act, v);
            *reinterpret_cast<f32x4*>(ccol + off) = f32x4{v[0], v[1], v[2], v[3]};
          } else {
            if (pcol) {
              u16x4 o;
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = from_float<T>(v[e]);
              *reinterpret_cast<u16x4*>(pcol + off) = o;
            }
            if (p.act != GINN_HIP_ACT_IDENTITY) act_forward_n<kFastMath<T>, 4>(p.act, v);
            u16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = from_float<T>(v[e]);
            *reinterpret_cast<u16x4*>(ccol + off) = o;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (row + e >= p.m) continue;
            float x = v[e];
            if (p.beta != 0.f) x += p.beta * to_float<T>(cin[off + e]);
            if (bias) x += to_float<T>(bias[row + e]);
            if (pcol) pcol[off + e] = from_float<T>(x);
            if (p.act != GINN_HIP_ACT_IDENTITY) x = act_forward<kFastMath<T>>(p.act, x);
            ccol[off + e] = from_float<T>(x);
          }
        }
      }
    }
  }
}

template <typename T, int BM, int BN, bool AKC, bool BKC, bool VECLD>
inline int launch_one(ginn_hip_ctx* ctx, const KParams& p, int batch) {
  dim3 grid((p.m + BM - 1) / BM, (p.n + BN - 1) / BN, p.splits > 1 ? p.splits : batch);
  gemm_generic_kernel<T, BM, BN, AKC, BKC, VECLD>
      <<<grid, dim3(kThreads), 0, ctx->stream>>>(p);
  GH_HIP(hipGetLastError());
  return kOk;
}

template <typename T, int BM, int BN, bool VECLD>
inline int launch_layout(ginn_hip_ctx* ctx, const KParams& p, int batch, bool akc, bool bkc) {
  if (akc) {
    if (bkc) return launch_one<T, BM, BN, true, true, VECLD>(ctx, p, batch);
    return launch_one<T, BM, BN, true, false, VECLD>(ctx, p, batch);
  }
  if (bkc) return launch_one<T, BM, BN, false, true, VECLD>(ctx, p, batch);
  return launch_one<T, BM, BN, false, false, VECLD>(ctx, p, batch);
}


// Folds the split-K partials and applies the epilogue:
// C = act(sum_z partial[z] + beta * C + bias), pre keeps the value before act.
// A block owns 64 consecutive outputs; its 4 waves take every 4th split and
// combine through LDS (always in the same order), so that also a small output
// with many splits is folded by many threads.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(KParams p) {
  using S = typename T::storage;
  __shared__ float red[4][64];
  const size_t total = (size_t)p.m * p.n;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  S* C = static_cast<S*>(p.C);
  S* P = static_cast<S*>(p.pre);
  const S* bias = static_cast<const S*>(p.bias);
  for (size_t base = (size_t)blockIdx.x * 64; base < total; base += (size_t)gridDim.x * 64) {
    const size_t i = base + tx;
    float v = 0.f;
    if (i < total) {
#pragma unroll 4
      for (int z = ty; z < p.splits; z += 4) v += p.partial[(size_t)z * total + i];
    }
    red[ty][tx] = v;
    __syncthreads();
    if (ty == 0 && i < total) {
      v = (red[0][tx] + red[1][tx]) + (red[2][tx] + red[3][tx]);
      const int row = (int)(i % p.m);
      const size_t col = i / p.m;
      const size_t off = col * p.ldc + row;
      // Scattered output columns come from the table (never with `pre`).
      S* out = p.ccols ? static_cast<S*>(p.ccols[col]) + row : C + off;
      if (p.beta != 0.f) v += p.beta * to_float<T>(P ? P[off] : *out);
      if (bias) v += to_float<T>(bias[row]);
      if (P) P[off] = from_float<T>(v);
      if (p.act != GINN_HIP_ACT_IDENTITY) v = act_forward<kFastMath<T>>(p.act, v);
      *out = from_float<T>(v);
    }
    __syncthreads();
  }
}

// The same fold for a large output with few splits: a thread owns 4
// consecutive rows of one column (m % 4 == 0) and reads its partials as
// 16-byte vectors; the splits are added in index order as above.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_wide_kernel(KParams p) {
  using S = typename T::storage;
  const size_t quads = (size_t)p.m * p.n / 4;
  const size_t total = (size_t)p.m * p.n;
  S* C = static_cast<S*>(p.C);
  S* P = static_cast<S*>(p.pre);
  const S* bias = static_cast<const S*>(p.bias);
  for (size_t q = (size_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += (size_t)gridDim.x * 256) {
    const size_t i = q * 4;
    float4 v = *reinterpret_cast<const float4*>(p.partial + i);
#pragma unroll 4
    for (int z = 1; z < p.splits; ++z) {
      const float4 w = *reinterpret_cast<const float4*>(p.partial + (size_t)z * total + i);
      v.x += w.x;
      v.y += w.y;
      v.z += w.z;
      v.w += w.w;
    }
    const int row = (int)(i % p.m);
    const size_t off = (i / p.m) * p.ldc + row;
    float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x = r[e];
      if (p.beta != 0.f) x += p.beta * to_float<T>((P ? P : C)[off + e]);
      if (bias) x += to_float<T>(bias[row + e]);
      if (P) P[off + e] = from_float<T>(x);
      if (p.act != GINN_HIP_ACT_IDENTITY) x = act_forward<kFastMath<T>>(p.act, x);
      r[e] = x;
    }
    if (p.ldc % 4 == 0 && reinterpret_cast<uintptr_t>(C) % (4 * sizeof(S)) == 0) {
      if constexpr (sizeof(S) == 4) {
        *reinterpret_cast<float4*>(C + off) = make_float4(r[0], r[1], r[2], r[3]);
      } else {
        uint2 pk;
        pk.x = (uint32_t)from_float<T>(r[0]) | ((uint32_t)from_float<T>(r[1]) << 16);
        pk.y = (uint32_t)from_float<T>(r[2]) | ((uint32_t)from_float<T>(r[3]) << 16);
        *reinterpret_cast<uint2*>(C + off) = pk;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) C[off + e] = from_float<T>(r[e]);
    }
  }
}

// Picks the fold: wide for a large output with few splits, otherwise the one
// that spreads the splits of an output over 4 waves.
template <typename T>
int launch_reduce(ginn_hip_ctx* ctx, const KParams& p) {
  const size_t total = (size_t)p.m * p.n;
  if (!p.ccols && p.m % 4 == 0 && p.splits <= 16 && total >= (size_t)ctx->num_cus * 1024 &&
      reinterpret_cast<uintptr_t>(p.partial) % 16 == 0) {
    size_t blocks = (total / 4 + 255) / 256;
    const size_t cap = (size_t)ctx->num_cus * 16;
    if (blocks > cap) blocks = cap;
    splitk_reduce_wide_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(p);
  } else {
    size_t blocks = (total + 63) / 64;
    const size_t cap = (size_t)ctx->num_cus * 32;
    if (blocks > cap) blocks = cap;
    splitk_reduce_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(p);
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

// Entry of one (scalar type, load mode) variant.  `big` selects 128 x 128
// block tiles (vector loads only), otherwise 64 x 64.
template <typename T, bool VECLD>
int launch_variant(ginn_hip_ctx* ctx, const KParams& p, int batch, bool akc,
                   bool bkc, bool big) {
  int rc;
  if (VECLD && big) rc = launch_layout<T, 128, 128, VECLD>(ctx, p, batch, akc, bkc);
  else rc = launch_layout<T, 64, 64, VECLD>(ctx, p, batch, akc, bkc);
  if (rc != kOk || p.splits <= 1) return rc;
  return launch_reduce<T>(ctx, p);
}

// Each variant is instantiated in exactly one translation unit.
#define GINN_HIP_GENERIC_VARIANT(PREFIX, T, VECLD)                             \
  PREFIX template int launch_variant<T, VECLD>(ginn_hip_ctx*, const KParams&,  \
                                               int, bool, bool, bool);

#ifndef GINN_HIP_GENERIC_INSTANTIATE
GINN_HIP_GENERIC_VARIANT(extern, F32, true)
GINN_HIP_GENERIC_VARIANT(extern, F32, false)
GINN_HIP_GENERIC_VARIANT(extern, F16, true)
GINN_HIP_GENERIC_VARIANT(extern, F16, false)
GINN_HIP_GENERIC_VARIANT(extern, BF16, true)
GINN_HIP_GENERIC_VARIANT(extern, BF16, false)
#endif

}  // namespace generic
}  // namespace ginn_hip

#endif  // GINN_HIP_GEMM_GENERIC_H
