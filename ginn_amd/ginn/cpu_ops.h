// The host layer's own arithmetic for tensors on cpu(): plain loops with fp32
// accumulation behind the nodes of the product path (Prod, BatchedProd,
// Affine, the nonlinearities, Add / Subtract / CwiseProd / the scalar forms,
// Sum / Mean, PickNegLogSoftmax), so that the same graph code runs on either
// device as in the reference (ginn/node/prod.h:31-46, ginn/node/affine.h:49-53,
// ginn/nonlin.h:67-300, where the CPU side is Eigen expressions).  A reference
// point for the device path, single-threaded like the reference's Eigen build;
// nothing here is called for a tensor on the HIP device.
#ifndef GINN_CPU_OPS_H
#define GINN_CPU_OPS_H

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <type_traits>
#include <vector>

#include <ginn/def.h>

namespace ginn {
namespace host {

template <typename S>
inline float get(const S* p, size_t i) {
  return static_cast<float>(p[i]);
}
template <typename S>
inline void put(S* p, size_t i, float v) {
  p[i] = S(v);
}

// An operand as fp32, column-major with leading dimension ld: the tensor's own
// memory for Real, a converted copy (kept in `keep`) for the 16-bit types.
template <typename S>
inline const float* as_f32(const S* src, size_t ld, size_t cols, std::vector<float>& keep) {
  if constexpr (std::is_same_v<S, float>) {
    return src;
  } else {
    keep.resize(ld * cols);
    for (size_t i = 0; i < ld * cols; ++i) keep[i] = static_cast<float>(src[i]);
    return keep.data();
  }
}

// ---------------------------------------------------------------------------------------------------------
// C[m x n] = op(A)[m x k] * op(B)[k x n] + beta * C, column-major, fp32 accumulation, one rounding to S.
//
// The inner loops are written on vectors of W floats (GCC / clang vector types) and exist twice: eight-wide with
// fused multiply-adds, compiled for AVX2 + FMA and taken when the processor has both (asked once at run time:
// the library itself is built for any x86-64), and four-wide for everything else.
// ---------------------------------------------------------------------------------------------------------
template <int W>
struct Vec {
  typedef float type __attribute__((vector_size(W * sizeof(float)), aligned(4)));
};
// Unaligned vector access through the pointer (V is the vector type in scope).
#define GINN_VLD(p) (*reinterpret_cast<const V*>(p))
#define GINN_VST(p, v) (*reinterpret_cast<V*>(p) = (v))
// (A float operand beside a vector is spread over the lanes by the compiler.)

// Narrow or small products.  Without a transposed A: up to four columns of C per sweep over a column of A
// (c_j += a_l * b(l, j)).  With one: dot products of contiguous columns, W partial sums each.
template <int W>
__attribute__((always_inline)) inline void sweep_impl(bool ta, bool tb, int m, int n, int k, const float* a, int lda,
                                                      const float* b, int ldb, float beta, float* c, int ldc) {
  using V = typename Vec<W>::type;
  auto b_at = [&](int l, int j) { return tb ? b[j + static_cast<size_t>(l) * ldb] : b[l + static_cast<size_t>(j) * ldb]; };
  if (!ta) {
    for (int j0 = 0; j0 < n; j0 += 4) {
      const int nj = std::min(4, n - j0);
      float* cols[4];
      for (int jj = 0; jj < 4; ++jj) cols[jj] = c + static_cast<size_t>(j0 + std::min(jj, nj - 1)) * ldc;
      for (int jj = 0; jj < nj; ++jj) {
        if (beta == 0.f) std::fill(cols[jj], cols[jj] + m, 0.f);
        else if (beta != 1.f)
          for (int i = 0; i < m; ++i) cols[jj][i] *= beta;
      }
      for (int l = 0; l < k; ++l) {
        const float* al = a + static_cast<size_t>(l) * lda;
        if (nj == 4) {
          const float b0 = b_at(l, j0), b1 = b_at(l, j0 + 1), b2 = b_at(l, j0 + 2), b3 = b_at(l, j0 + 3);
          float *c0 = cols[0], *c1 = cols[1], *c2 = cols[2], *c3 = cols[3];
          int i = 0;
          for (; i + W <= m; i += W) {
            const V av = GINN_VLD(al + i);
            GINN_VST(c0 + i, GINN_VLD(c0 + i) + av * b0);
            GINN_VST(c1 + i, GINN_VLD(c1 + i) + av * b1);
            GINN_VST(c2 + i, GINN_VLD(c2 + i) + av * b2);
            GINN_VST(c3 + i, GINN_VLD(c3 + i) + av * b3);
          }
          for (; i < m; ++i) {
            const float v = al[i];
            c0[i] += v * b0;
            c1[i] += v * b1;
            c2[i] += v * b2;
            c3[i] += v * b3;
          }
        } else {
          for (int jj = 0; jj < nj; ++jj) {
            const float bs = b_at(l, j0 + jj);
            float* cj = cols[jj];
            int i = 0;
            for (; i + W <= m; i += W) GINN_VST(cj + i, GINN_VLD(cj + i) + GINN_VLD(al + i) * bs);
            for (; i < m; ++i) cj[i] += al[i] * bs;
          }
        }
      }
    }
  } else {
    // op(A)(i, l) = A(l, i): column i of the stored A against column j of op(B)
    std::vector<float> bcol(tb ? static_cast<size_t>(k) : 0);
    for (int j = 0; j < n; ++j) {
      const float* bj = b + static_cast<size_t>(j) * ldb;
      if (tb) {
        for (int l = 0; l < k; ++l) bcol[static_cast<size_t>(l)] = b_at(l, j);
        bj = bcol.data();
      }
      float* cj = c + static_cast<size_t>(j) * ldc;
      for (int i = 0; i < m; ++i) {
        const float* ai = a + static_cast<size_t>(i) * lda;
        V acc = {};
        int l = 0;
        for (; l + W <= k; l += W) acc += GINN_VLD(ai + l) * GINN_VLD(bj + l);
        float sum = 0.f;
        for (int e = 0; e < W; ++e) sum += acc[e];
        for (; l < k; ++l) sum += ai[l] * bj[l];
        cj[i] = beta == 0.f ? sum : sum + beta * cj[i];
      }
    }
  }
}

// Everything else: the classic packed scheme.  op(A) is cut into blocks of kMc rows x kKc sums, stored as panels
// of kMr rows (one sum after the other), op(B) into panels of kNr columns; a register tile of kMr x kNr sums runs
// over one pair of panels.  Panels are padded with zeros, so the tile loop has no edges; edge tiles are stored
// through a small buffer.
constexpr int kMr = 16, kNr = 6, kKc = 256, kMc = 128, kNc = 1536;

// tile[j * kMr + i] = sum_l ap[l * kMr + i] * bp[l * kNr + j]; two vectors of rows per sweep, so that the
// 2 x kNr sums stay in registers (four-wide: two sweeps of eight rows).
template <int W>
__attribute__((always_inline)) inline void tile_impl(int kc, const float* ap, const float* bp, float* tile) {
  using V = typename Vec<W>::type;
  for (int r0 = 0; r0 < kMr; r0 += 2 * W) {
    V acc[kNr][2] = {};
    const float* a = ap + r0;
    const float* b = bp;
    for (int l = 0; l < kc; ++l, a += kMr, b += kNr) {
      const V a0 = GINN_VLD(a), a1 = GINN_VLD(a + W);
#pragma GCC unroll 6
      for (int j = 0; j < kNr; ++j) {
        const float bj = b[j];
        acc[j][0] += a0 * bj;
        acc[j][1] += a1 * bj;
      }
    }
    for (int j = 0; j < kNr; ++j) {
      GINN_VST(tile + j * kMr + r0, acc[j][0]);
      GINN_VST(tile + j * kMr + r0 + W, acc[j][1]);
    }
  }
}

inline void sweep_narrow(bool ta, bool tb, int m, int n, int k, const float* a, int lda, const float* b, int ldb,
                         float beta, float* c, int ldc) {
  sweep_impl<4>(ta, tb, m, n, k, a, lda, b, ldb, beta, c, ldc);
}
inline void tile_narrow(int kc, const float* ap, const float* bp, float* tile) { tile_impl<4>(kc, ap, bp, tile); }
#if defined(__x86_64__) && (defined(__GNUC__) || defined(__clang__)) && !defined(GINN_HOST_GEMM_PLAIN)
__attribute__((target("avx2,fma"))) inline void sweep_wide(bool ta, bool tb, int m, int n, int k, const float* a,
                                                           int lda, const float* b, int ldb, float beta, float* c,
                                                           int ldc) {
  sweep_impl<8>(ta, tb, m, n, k, a, lda, b, ldb, beta, c, ldc);
}
__attribute__((target("avx2,fma"))) inline void tile_wide(int kc, const float* ap, const float* bp, float* tile) {
  tile_impl<8>(kc, ap, bp, tile);
}
inline bool has_wide_vectors() {
  static const bool yes = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
  return yes;
}
#else
inline void sweep_wide(bool ta, bool tb, int m, int n, int k, const float* a, int lda, const float* b, int ldb,
                       float beta, float* c, int ldc) {
  sweep_narrow(ta, tb, m, n, k, a, lda, b, ldb, beta, c, ldc);
}
inline void tile_wide(int kc, const float* ap, const float* bp, float* tile) { tile_narrow(kc, ap, bp, tile); }
inline bool has_wide_vectors() { return false; }
#endif

#undef GINN_VLD
#undef GINN_VST

// c (fp32, leading dimension ldc) = op(a) op(b) + beta * c
inline void gemm_packed(bool ta, bool tb, int m, int n, int k, const float* a, int lda, const float* b, int ldb,
                        float beta, float* c, int ldc) {
  const bool wide = has_wide_vectors();
  // packed blocks, kept per thread between calls (a fresh 1.5 MB block per call costs more than a small product)
  static thread_local std::vector<float> apack, bpack;
  const size_t kc_max = static_cast<size_t>(std::min(k, kKc));
  const size_t a_need = kc_max * static_cast<size_t>((std::min(m, kMc) + kMr - 1) / kMr * kMr);
  const size_t b_need = kc_max * static_cast<size_t>((std::min(n, kNc) + kNr - 1) / kNr * kNr);
  if (apack.size() < a_need) apack.resize(a_need);
  if (bpack.size() < b_need) bpack.resize(b_need);
  float tile[kMr * kNr];
  for (int jc = 0; jc < n; jc += kNc) {
    const int nc = std::min(kNc, n - jc);
    for (int pc = 0; pc < k; pc += kKc) {
      const int kc = std::min(kKc, k - pc);
      // op(B)[pc .. pc + kc, jc .. jc + nc] as panels of kNr columns
      for (int j0 = 0; j0 < nc; j0 += kNr) {
        float* dst = bpack.data() + static_cast<size_t>(j0) * kc;
        for (int jj = 0; jj < kNr; ++jj) {
          const int j = jc + j0 + jj;
          if (j0 + jj >= nc) {
            for (int l = 0; l < kc; ++l) dst[l * kNr + jj] = 0.f;
          } else if (tb) {  // op(B)(l, j) = B(j, l)
            const float* src = b + j + static_cast<size_t>(pc) * ldb;
            for (int l = 0; l < kc; ++l) dst[l * kNr + jj] = src[static_cast<size_t>(l) * ldb];
          } else {
            const float* src = b + pc + static_cast<size_t>(j) * ldb;
            for (int l = 0; l < kc; ++l) dst[l * kNr + jj] = src[l];
          }
        }
      }
      for (int ic = 0; ic < m; ic += kMc) {
        const int mc = std::min(kMc, m - ic);
        // op(A)[ic .. ic + mc, pc .. pc + kc] as panels of kMr rows
        for (int i0 = 0; i0 < mc; i0 += kMr) {
          float* dst = apack.data() + static_cast<size_t>(i0) * kc;
          const int mr = std::min(kMr, mc - i0);
          if (ta) {  // op(A)(i, l) = A(l, i): a row of the panel is a contiguous piece of a stored column
            for (int ii = 0; ii < kMr; ++ii) {
              if (ii >= mr) {
                for (int l = 0; l < kc; ++l) dst[l * kMr + ii] = 0.f;
              } else {
                const float* src = a + pc + static_cast<size_t>(ic + i0 + ii) * lda;
                for (int l = 0; l < kc; ++l) dst[l * kMr + ii] = src[l];
              }
            }
          } else {
            for (int l = 0; l < kc; ++l) {
              const float* src = a + (ic + i0) + static_cast<size_t>(pc + l) * lda;
              for (int ii = 0; ii < mr; ++ii) dst[l * kMr + ii] = src[ii];
              for (int ii = mr; ii < kMr; ++ii) dst[l * kMr + ii] = 0.f;
            }
          }
        }
        for (int j0 = 0; j0 < nc; j0 += kNr) {
          const int nr = std::min(kNr, nc - j0);
          const float* bp = bpack.data() + static_cast<size_t>(j0) * kc;
          for (int i0 = 0; i0 < mc; i0 += kMr) {
            const int mr = std::min(kMr, mc - i0);
            const float* ap = apack.data() + static_cast<size_t>(i0) * kc;
            if (wide) tile_wide(kc, ap, bp, tile);
            else tile_narrow(kc, ap, bp, tile);
            float* out = c + (ic + i0) + static_cast<size_t>(jc + j0) * ldc;
            if (pc == 0 && beta == 0.f) {
              for (int j = 0; j < nr; ++j)
                for (int i = 0; i < mr; ++i) out[i + static_cast<size_t>(j) * ldc] = tile[j * kMr + i];
            } else {
              const float scale = pc == 0 ? beta : 1.f;
              for (int j = 0; j < nr; ++j)
                for (int i = 0; i < mr; ++i) {
                  float& o = out[i + static_cast<size_t>(j) * ldc];
                  o = scale * o + tile[j * kMr + i];
                }
            }
          }
        }
      }
    }
  }
}

template <typename S>
void gemm(bool ta, bool tb, int m, int n, int k, const S* A, int lda, const S* B, int ldb, float beta, S* C,
          int ldc) {
  if (m <= 0 || n <= 0) return;
  std::vector<float> keep_a, keep_b;
  const float* a = as_f32(A, static_cast<size_t>(lda), static_cast<size_t>(ta ? m : k), keep_a);
  const float* b = as_f32(B, static_cast<size_t>(ldb), static_cast<size_t>(tb ? k : n), keep_b);
  // fp32 results form in C itself; the 16-bit types get the product alone in fp32 first and one rounding after
  constexpr bool in_place = std::is_same_v<S, float>;
  std::vector<float> sums(in_place ? 0 : static_cast<size_t>(m) * n);
  float* c = in_place ? reinterpret_cast<float*>(C) : sums.data();
  const int ldsum = in_place ? ldc : m;
  const float inner_beta = in_place ? beta : 0.f;
  if (n < kNr || m < kMr || k < 8 || static_cast<double>(m) * n * k < 32768.) {
    if (has_wide_vectors()) sweep_wide(ta, tb, m, n, k, a, lda, b, ldb, inner_beta, c, ldsum);
    else sweep_narrow(ta, tb, m, n, k, a, lda, b, ldb, inner_beta, c, ldsum);
  } else {
    gemm_packed(ta, tb, m, n, k, a, lda, b, ldb, inner_beta, c, ldsum);
  }
  if (in_place) return;
  for (int j = 0; j < n; ++j) {
    S* out = C + static_cast<size_t>(j) * ldc;
    const float* cj = sums.data() + static_cast<size_t>(j) * m;
    if (beta != 0.f)
      for (int i = 0; i < m; ++i) put(out, static_cast<size_t>(i), cj[i] + beta * get(out, static_cast<size_t>(i)));
    else
      for (int i = 0; i < m; ++i) put(out, static_cast<size_t>(i), cj[i]);
  }
}

// The nonlinearities (ginn/nonlin.h:67-300) on one value; `code` as in the device library.
inline float act_forward(int code, float x) {
  switch (code) {
    case GINN_HIP_ACT_TANH: return std::tanh(x);
    case GINN_HIP_ACT_RELU: return x > 0.f ? x : 0.f;
    case GINN_HIP_ACT_SIGMOID: return 0.5f * std::tanh(0.5f * x) + 0.5f;  // ginn/nonlin.h:141-144
    case GINN_HIP_ACT_GELU: return 0.5f * x * (1.f + std::erf(x * 0.70710678118654752440f));  // :281-283
    case GINN_HIP_ACT_GELU2: {  // :250-254
      const float a = 0.79788456080286535588f, b = 0.044715f;
      return 0.5f * x * (1.f + std::tanh(a * (x + b * x * x * x)));
    }
    case GINN_HIP_ACT_LOG: return std::log(x);
    case GINN_HIP_ACT_SQRT: return std::sqrt(x);
    default: return x;
  }
}
// d f(x) / dx from the input x and the output y (each nonlinearity's `backward` there).
inline float act_derivative(int code, float x, float y) {
  switch (code) {
    case GINN_HIP_ACT_TANH: return 1.f - y * y;
    case GINN_HIP_ACT_RELU: return y > 0.f ? 1.f : 0.f;
    case GINN_HIP_ACT_SIGMOID: return y * (1.f - y);
    case GINN_HIP_ACT_GELU:  // :290-296
      return 0.5f * (1.f + std::erf(x * 0.70710678118654752440f)) +
             x * std::exp(-0.5f * x * x) * 0.39894228040143267794f;
    case GINN_HIP_ACT_GELU2: {  // :262-266, written without the division by x
      const float a = 0.79788456080286535588f, b = 0.044715f;
      const float t = std::tanh(a * (x + b * x * x * x));
      return 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * a * (1.f + 3.f * b * x * x);
    }
    case GINN_HIP_ACT_LOG: return 1.f / x;
    case GINN_HIP_ACT_SQRT: return 0.5f / y;
    default: return 1.f;
  }
}

// y = f(x) over [rows x cols]; SOFTMAX is taken per column (ginn/nonlin.h:150-175).
template <typename S>
void nonlin_forward(int code, int rows, int cols, const S* x, S* y) {
  if (code == GINN_HIP_ACT_SOFTMAX) {
    std::vector<float> e(static_cast<size_t>(rows));
    for (int c = 0; c < cols; ++c) {
      const S* xc = x + static_cast<size_t>(c) * rows;
      S* yc = y + static_cast<size_t>(c) * rows;
      float mx = -INFINITY, sum = 0.f;
      for (int r = 0; r < rows; ++r) mx = std::max(mx, get(xc, r));
      for (int r = 0; r < rows; ++r) sum += (e[r] = std::exp(get(xc, r) - mx));
      for (int r = 0; r < rows; ++r) put(yc, r, e[r] / sum);
    }
    return;
  }
  const size_t n = static_cast<size_t>(rows) * cols;
  for (size_t i = 0; i < n; ++i) put(y, i, act_forward(code, get(x, i)));
}
// dx (+)= f'(x, y) (*) dy; SOFTMAX: dx = y (*) (dy - <dy, y>) per column (ginn/nonlin.h:177-184).
template <typename S>
void nonlin_backward(int code, int rows, int cols, const S* dy, const S* x, const S* y, S* dx, bool accumulate) {
  if (code == GINN_HIP_ACT_SOFTMAX) {
    for (int c = 0; c < cols; ++c) {
      const size_t o = static_cast<size_t>(c) * rows;
      float dot = 0.f;
      for (int r = 0; r < rows; ++r) dot += get(dy, o + r) * get(y, o + r);
      for (int r = 0; r < rows; ++r) {
        const float v = get(y, o + r) * (get(dy, o + r) - dot);
        put(dx, o + r, accumulate ? get(dx, o + r) + v : v);
      }
    }
    return;
  }
  const size_t n = static_cast<size_t>(rows) * cols;
  for (size_t i = 0; i < n; ++i) {
    const float v = get(dy, i) * act_derivative(code, x ? get(x, i) : 0.f, y ? get(y, i) : 0.f);
    put(dx, i, accumulate ? get(dx, i) + v : v);
  }
}

// dst (+)= alpha * x + shift; dst (+)= a (*) b; dst (+)= a + sign * b.
template <typename S>
void scale_shift(size_t n, float alpha, float shift, const S* x, S* dst, bool accumulate) {
  for (size_t i = 0; i < n; ++i) {
    const float v = alpha * get(x, i) + shift;
    put(dst, i, accumulate ? get(dst, i) + v : v);
  }
}
template <typename S>
void cwise_prod(size_t n, const S* a, const S* b, S* dst, bool accumulate) {
  for (size_t i = 0; i < n; ++i) {
    const float v = get(a, i) * get(b, i);
    put(dst, i, accumulate ? get(dst, i) + v : v);
  }
}
template <typename S>
void add_n(size_t n, const std::vector<const S*>& srcs, S* dst, bool accumulate) {
  for (size_t i = 0; i < n; ++i) {
    float v = accumulate ? get(dst, i) : 0.f;
    for (const S* s : srcs) v += get(s, i);
    put(dst, i, v);
  }
}

// sum of all elements (scale = 1) or their mean (scale = 1 / n), fp32 accumulation.
template <typename S>
float sum_all(size_t n, const S* x) {
  double s = 0.;
  for (size_t i = 0; i < n; ++i) s += get(x, i);
  return static_cast<float>(s);
}

// PickNegLogSoftmax per column (ginn/node/pick.h: -log softmax(x)[index]) and its gradient
// dx (+)= (softmax(x) - onehot(index)) * dy[c].
template <typename S>
void pick_nls_forward(int rows, int cols, const S* x, const int* index, S* out) {
  for (int c = 0; c < cols; ++c) {
    const S* xc = x + static_cast<size_t>(c) * rows;
    float mx = -INFINITY, sum = 0.f;
    for (int r = 0; r < rows; ++r) mx = std::max(mx, get(xc, r));
    for (int r = 0; r < rows; ++r) sum += std::exp(get(xc, r) - mx);
    put(out, c, -(get(xc, index[c]) - mx - std::log(sum)));
  }
}
template <typename S>
void pick_nls_backward(int rows, int cols, const S* x, const int* index, const S* dy, S* dx, bool accumulate) {
  for (int c = 0; c < cols; ++c) {
    const size_t o = static_cast<size_t>(c) * rows;
    float mx = -INFINITY, sum = 0.f;
    for (int r = 0; r < rows; ++r) mx = std::max(mx, get(x, o + r));
    for (int r = 0; r < rows; ++r) sum += std::exp(get(x, o + r) - mx);
    const float g = get(dy, c);
    for (int r = 0; r < rows; ++r) {
      const float v = (std::exp(get(x, o + r) - mx) / sum - (r == index[c] ? 1.f : 0.f)) * g;
      put(dx, o + r, accumulate ? get(dx, o + r) + v : v);
    }
  }
}

// dst (+)= src over a [rows x cols] window with leading dimensions lds / ldd (Slice, Cat, RowwiseCat, Chip).
template <typename S>
void copy_2d(Size rows, Size cols, const S* src, Size lds, S* dst, Size ldd, bool accumulate) {
  for (Size c = 0; c < cols; ++c)
    for (Size r = 0; r < rows; ++r) {
      if constexpr (std::is_arithmetic_v<S> && !std::is_floating_point_v<S>) {
        dst[c * ldd + r] = src[c * lds + r];  // integer tensors are only moved
      } else {
        const float v = get(src, c * lds + r);
        put(dst, c * ldd + r, accumulate ? get(dst, c * ldd + r) + v : v);
      }
    }
}

// dst[permuted index] (+)= src[index]: dst has extents dims[perm[0]], dims[perm[1]], ... (PermuteNode).
template <typename S>
void permute(const std::vector<Size>& dims, const std::vector<Size>& perm, const S* src, S* dst, bool accumulate) {
  const size_t rank = dims.size();
  std::vector<Size> src_stride(rank), dst_stride_of_src_axis(rank), idx(rank, 0);
  Size run = 1, total = 1;
  for (size_t i = 0; i < rank; ++i) {
    src_stride[i] = run;
    run *= dims[i];
  }
  total = run;
  run = 1;
  for (size_t j = 0; j < rank; ++j) {  // axis j of dst runs along axis perm[j] of src
    dst_stride_of_src_axis[static_cast<size_t>(perm[j])] = run;
    run *= dims[static_cast<size_t>(perm[j])];
  }
  for (Size lin = 0; lin < total; ++lin) {
    Size d = 0;
    for (size_t i = 0; i < rank; ++i) d += idx[i] * dst_stride_of_src_axis[i];
    const float v = get(src, lin);
    put(dst, d, accumulate ? get(dst, d) + v : v);
    for (size_t i = 0; i < rank; ++i) {  // next index of src, first axis fastest
      if (++idx[i] < dims[i]) break;
      idx[i] = 0;
    }
  }
}

// LayerNorm per column (ginn/node/layernorm.h:31-74): y = (x - mean) / std, std = sqrt(mean((x - mean)^2) + eps);
// dx (+)= (dy - mean(dy) - y <dy, y> / rows) / std.
template <typename S>
void layernorm_forward(int rows, int cols, const S* x, float eps, S* y, float* std_out) {
  for (int c = 0; c < cols; ++c) {
    const size_t o = static_cast<size_t>(c) * rows;
    double mean = 0., var = 0.;
    for (int r = 0; r < rows; ++r) mean += get(x, o + r);
    mean /= rows;
    for (int r = 0; r < rows; ++r) {
      const double d = get(x, o + r) - mean;
      var += d * d;
    }
    const float sd = std::sqrt(static_cast<float>(var / rows) + eps);
    std_out[c] = sd;
    for (int r = 0; r < rows; ++r) put(y, o + r, (get(x, o + r) - static_cast<float>(mean)) / sd);
  }
}
template <typename S>
void layernorm_backward(int rows, int cols, const S* dy, const S* y, const float* std_in, S* dx, bool accumulate) {
  for (int c = 0; c < cols; ++c) {
    const size_t o = static_cast<size_t>(c) * rows;
    double sum = 0., dot = 0.;
    for (int r = 0; r < rows; ++r) {
      sum += get(dy, o + r);
      dot += static_cast<double>(get(dy, o + r)) * get(y, o + r);
    }
    const float m = static_cast<float>(sum / rows), d = static_cast<float>(dot / rows);
    for (int r = 0; r < rows; ++r) {
      const float v = (get(dy, o + r) - m - get(y, o + r) * d) / std_in[c];
      put(dx, o + r, accumulate ? get(dx, o + r) + v : v);
    }
  }
}

// CwiseProdAdd (ginn/node/common.h:251-316): y = a (*) (b + bias) + c, b and c per row when `broadcast`.
template <typename S>
void cwise_prod_add_forward(int rows, int cols, const S* a, const S* b, const S* c, float bias, bool broadcast, S* y) {
  const size_t n = static_cast<size_t>(rows) * cols;
  for (size_t i = 0; i < n; ++i) {
    const size_t j = broadcast ? i % rows : i;
    put(y, i, get(a, i) * (get(b, j) + bias) + get(c, j));
  }
}
// da (+)= dy (*) (b + bias); db += dy (*) a; dc += dy (row sums when `broadcast`).
template <typename S>
void cwise_prod_add_backward(int rows, int cols, const S* dy, const S* a, const S* b, float bias, bool broadcast, S* da,
                             bool da_accumulate, S* db, S* dc) {
  const size_t n = static_cast<size_t>(rows) * cols, nb = broadcast ? static_cast<size_t>(rows) : n;
  std::vector<float> sb, sc;
  if (db) sb.assign(nb, 0.f);
  if (dc) sc.assign(nb, 0.f);
  for (size_t i = 0; i < n; ++i) {
    const size_t j = broadcast ? i % rows : i;
    const float g = get(dy, i);
    if (da) {
      const float v = g * (get(b, j) + bias);
      put(da, i, da_accumulate ? get(da, i) + v : v);
    }
    if (db) sb[j] += g * get(a, i);
    if (dc) sc[j] += g;
  }
  for (size_t j = 0; j < nb; ++j) {
    if (db) put(db, j, get(db, j) + sb[j]);
    if (dc) put(dc, j, get(dc, j) + sc[j]);
  }
}

// x viewed as [mask_size x batch]: entries whose mask value is 0 become `value` (InPlaceMask).
template <typename S>
void mask_fill(size_t mask_size, size_t batch, const S* mask, float value, S* x) {
  for (size_t z = 0; z < batch; ++z)
    for (size_t i = 0; i < mask_size; ++i)
      if (get(mask, i) == 0.f) put(x, z * mask_size + i, value);
}

}  // namespace host
}  // namespace ginn

#endif  // GINN_CPU_OPS_H
