// Companions of the product path inside a transformer block: column layer
// normalisation, the gamma / beta affine that follows it, axis permutation,
// masked fill and the causal (upper triangular) mask.  All are bandwidth
// bound; statistics and reductions are carried in fp32 whatever the storage.
#include "common.h"
#include "reduce_rows.h"
#include "kernel_util.h"
#include "vec_access.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;

// One wave per column: mean, then the mean of squared deviations (two passes,
// as the reference evaluates them), then the normalised values.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void layernorm_fwd_kernel(int rows, int cols,
                                                               const typename T::storage* x, float eps,
                                                               typename T::storage* y,  // may be x (in place)
                                                               float* __restrict__ std_out,
                                                               // optional second result z = y * (gamma + mb) + beta,
                                                               // gamma / beta one value per row (from y as stored)
                                                               const typename T::storage* __restrict__ gamma,
                                                               const typename T::storage* __restrict__ beta, float mb,
                                                               typename T::storage* __restrict__ z) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * kWaves + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * kWaves;
  const float inv_rows = 1.f / static_cast<float>(rows);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    float s = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) s += v[e];
    }
    const float mean = wave_sum(s) * inv_rows;
    float q = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) q += (v[e] - mean) * (v[e] - mean);
    }
    const float sd = sqrtf(wave_sum(q) * inv_rows + eps);
    const float inv = 1.f / sd;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = (v[e] - mean) * inv;
      st<T, V>(y + base + r, v);
      if (z) {
        float gv[V], bv[V];
        ld<T, V>(gamma + r, gv);
        ld<T, V>(beta + r, bv);
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = to_float<T>(from_float<T>(v[e])) * (gv[e] + mb) + bv[e];
        st<T, V>(z + base + r, v);
      }
    }
    if (lane == 0) std_out[c] = sd;
  }
}

// dx (+)= (dy - mean(dy) - y * (dy . y) / rows) / std, one wave per column.
// Without `accumulate`, dx may be dy itself (the in-place node): a lane reads
// its elements of dy right before it writes the same elements of dx, after
// the column's sums are complete.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void layernorm_bwd_kernel(int rows, int cols,
                                                               const typename T::storage* dy,
                                                               const typename T::storage* __restrict__ y,
                                                               const float* __restrict__ std_in,
                                                               typename T::storage* dx, int accumulate) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * kWaves + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * kWaves;
  const float inv_rows = 1.f / static_cast<float>(rows);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    float s = 0.f, d = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float g[V], yv[V];
      ld<T, V>(dy + base + r, g);
      ld<T, V>(y + base + r, yv);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        s += g[e];
        d += g[e] * yv[e];
      }
    }
    const float gmean = wave_sum(s) * inv_rows;
    const float dot = wave_sum(d) * inv_rows;
    const float inv = 1.f / std_in[c];
    for (int r = lane * V; r < rows; r += 64 * V) {
      float g[V], yv[V], old[V];
      ld<T, V>(dy + base + r, g);
      ld<T, V>(y + base + r, yv);
#pragma unroll
      for (int e = 0; e < V; ++e) old[e] = 0.f;
      if (accumulate) ld<T, V>(dx + base + r, old);
#pragma unroll
      for (int e = 0; e < V; ++e) old[e] += (g[e] - gmean - yv[e] * dot) * inv;
      st<T, V>(dx + base + r, old);
    }
  }
}

// Backward of z = LayerNorm(x) * (gamma + mb) + beta in one pass over dz: the
// gradient of the normalised values da = dz * (gamma + mb) (rounded to the
// storage type, as the separate CwiseProdAdd backward stores it) is formed on
// the fly and pushed through the LayerNorm formula above into dx; the row sums
// dgamma += sum_c dz (*) y and dbeta += sum_c dz stay in registers over the
// columns of a wave and leave as one fp32 partial row per workgroup.  One wave
// per column, rows <= 64 * V * ITERS (ITERS vectors per lane; at most kLnRowIters).
// A column is one load -> two wave sums -> store chain, and the waves on a CU
// are all the chains it overlaps: workgroups of 8 waves (up to 256 registers
// each: the longest columns keep 5 x 32 values per lane), at most two per CU,
// a partial row each (768 x 4096 bf16: 17.3 us with one workgroup of 4 waves
// per CU, four columns one after the other in each wave).
constexpr int kLnRowIters = 4;
constexpr int kLnBwdWaves = 8;
template <typename T, int V, int ITERS>
__global__ __launch_bounds__(kLnBwdWaves * 64) void layernorm_affine_bwd_kernel(
    int rows, int cols, const typename T::storage* __restrict__ dz, const typename T::storage* __restrict__ y,
    const float* __restrict__ std_in, const typename T::storage* __restrict__ gamma, float mb,
    typename T::storage* dx, int accumulate, float* __restrict__ part_g, float* __restrict__ part_b) {
  __shared__ float red[kLnBwdWaves][64 * V];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int wave = blockIdx.x * kLnBwdWaves + w;
  const int nwaves = gridDim.x * kLnBwdWaves;
  const float inv_rows = 1.f / static_cast<float>(rows);
  float scale[ITERS][V], sg[ITERS][V], sb[ITERS][V];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int r = (it * 64 + lane) * V;
#pragma unroll
    for (int e = 0; e < V; ++e) scale[it][e] = sg[it][e] = sb[it][e] = 0.f;
    if (r < rows) {
      ld<T, V>(gamma + r, scale[it]);
#pragma unroll
      for (int e = 0; e < V; ++e) scale[it][e] += mb;
    }
  }
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    float g[ITERS][V], yv[ITERS][V];
    float s = 0.f, d = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int r = (it * 64 + lane) * V;
#pragma unroll
      for (int e = 0; e < V; ++e) g[it][e] = yv[it][e] = 0.f;
      if (r < rows) {
        ld<T, V>(dz + base + r, g[it]);
        ld<T, V>(y + base + r, yv[it]);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          sg[it][e] += g[it][e] * yv[it][e];
          sb[it][e] += g[it][e];
          g[it][e] = to_float<T>(from_float<T>(g[it][e] * scale[it][e]));  // da as the separate kernel stores it
          s += g[it][e];
          d += g[it][e] * yv[it][e];
        }
      }
    }
    if (dx) {
      const float gmean = wave_sum(s) * inv_rows;
      const float dot = wave_sum(d) * inv_rows;
      const float inv = 1.f / std_in[c];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int r = (it * 64 + lane) * V;
        if (r < rows) {
          float old[V];
#pragma unroll
          for (int e = 0; e < V; ++e) old[e] = 0.f;
          if (accumulate) ld<T, V>(dx + base + r, old);
#pragma unroll
          for (int e = 0; e < V; ++e) old[e] += (g[it][e] - gmean - yv[it][e] * dot) * inv;
          st<T, V>(dx + base + r, old);
        }
      }
    }
  }
  if (!part_g) return;
  // The waves' row sums -> one partial row per workgroup (the others hand theirs to wave 0).
#pragma unroll
  for (int which = 0; which < 2; ++which) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int r = (it * 64 + lane) * V;
      float (&mine)[V] = which ? sb[it] : sg[it];
      __syncthreads();
#pragma unroll
      for (int e = 0; e < V; ++e) red[w][lane * V + e] = mine[e];
      __syncthreads();
      if (w == 0 && r < rows) {
        float* out = (which ? part_b : part_g) + static_cast<size_t>(blockIdx.x) * rows + r;
#pragma unroll
        for (int e = 0; e < V; ++e) {
          float t = 0.f;
#pragma unroll
          for (int k = 0; k < kLnBwdWaves; ++k) t += red[k][lane * V + e];
          out[e] = t;
        }
      }
    }
  }
}

// y = a * (b + mb) + c; with `broadcast`, b and c are [rows] vectors applied
// to every column (rows is a multiple of V then).
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void cwise_prod_add_fwd_kernel(int rows, size_t n,
                                                                    const typename T::storage* __restrict__ a,
                                                                    const typename T::storage* __restrict__ b,
                                                                    const typename T::storage* __restrict__ c,
                                                                    float mb, int broadcast,
                                                                    typename T::storage* __restrict__ y) {
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * V; i < n;
       i += static_cast<size_t>(gridDim.x) * kBlock * V) {
    const size_t j = broadcast ? i % rows : i;
    float av[V], bv[V], cv[V];
    ld<T, V>(a + i, av);
    ld<T, V>(b + j, bv);
    ld<T, V>(c + j, cv);
#pragma unroll
    for (int e = 0; e < V; ++e) av[e] = av[e] * (bv[e] + mb) + cv[e];
    st<T, V>(y + i, av);
  }
}

// Not broadcast: everything is elementwise.
template <typename T>
__global__ __launch_bounds__(kBlock) void cwise_prod_add_bwd_flat_kernel(size_t n,
                                                                         const typename T::storage* __restrict__ dy,
                                                                         const typename T::storage* __restrict__ a,
                                                                         const typename T::storage* __restrict__ b,
                                                                         float mb, typename T::storage* da,
                                                                         typename T::storage* db,
                                                                         typename T::storage* dc, int add_da) {
  for (size_t i = blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * kBlock) {
    const float g = to_float<T>(dy[i]);
    if (da) da[i] = from_float<T>((add_da ? to_float<T>(da[i]) : 0.f) + g * (to_float<T>(b[i]) + mb));
    if (db) db[i] = from_float<T>(to_float<T>(db[i]) + g * to_float<T>(a[i]));
    if (dc) dc[i] = from_float<T>(to_float<T>(dc[i]) + g);
  }
}

// Broadcast: da is finished here, the row sums for db and dc leave fp32
// partials per column chunk.
template <typename T, int V>
__global__ __launch_bounds__(rowred::kBlock) void cwise_prod_add_bwd_bcast_kernel(
    int nrows, int cols, int cols_per_chunk, const typename T::storage* __restrict__ dy,
    const typename T::storage* __restrict__ a, const typename T::storage* __restrict__ b, float mb,
    typename T::storage* da, float* __restrict__ part_b, float* __restrict__ part_c, int add_da) {
  __shared__ float red[rowred::kSlices * V * 64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int r = (blockIdx.x * rowred::kRowsPerBlock + tx) * V;
  const int c0 = blockIdx.y * cols_per_chunk;
  const int c1 = min(cols, c0 + cols_per_chunk);
  float sb[V], sc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) sb[e] = sc[e] = 0.f;
  if (r < nrows) {
    float scale[V];
    ld<T, V>(b + r, scale);
#pragma unroll
    for (int e = 0; e < V; ++e) scale[e] += mb;
    // Four columns per step, all their loads issued before the first use (a
    // block has only a few columns per wave; one at a time would pay a memory
    // latency for each, and the store into da keeps the compiler from moving
    // the next column's loads up by itself).
    constexpr int U = 4;
    for (int c = c0 + ty; c < c1; c += U * rowred::kSlices) {
      float g[U][V], av[U][V], d[U][V];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int cu = c + u * rowred::kSlices;
#pragma unroll
        for (int e = 0; e < V; ++e) g[u][e] = av[u][e] = d[u][e] = 0.f;
        if (cu < c1) {
          const size_t i = static_cast<size_t>(cu) * nrows + r;
          ld<T, V>(dy + i, g[u]);
          ld<T, V>(a + i, av[u]);
          if (da && add_da) ld<T, V>(da + i, d[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int cu = c + u * rowred::kSlices;
        if (cu < c1) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            sb[e] += g[u][e] * av[u][e];
            sc[e] += g[u][e];
          }
          if (da) {
#pragma unroll
            for (int e = 0; e < V; ++e) d[u][e] += g[u][e] * scale[e];
            st<T, V>(da + static_cast<size_t>(cu) * nrows + r, d[u]);
          }
        }
      }
    }
  }
  rowred::combine_v<V>(sb, red);
  rowred::combine_v<V>(sc, red);
  if (ty == 0 && r < nrows) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      part_b[static_cast<size_t>(blockIdx.y) * nrows + r + e] = sb[e];
      part_c[static_cast<size_t>(blockIdx.y) * nrows + r + e] = sc[e];
    }
  }
}

constexpr int kMaxRank = 8;
struct PermuteDesc {
  int rank;
  long long out_dim[kMaxRank];     // extents of the result
  long long src_stride[kMaxRank];  // stride in the source of each result axis
};

// Gather by result index: consecutive threads write consecutive addresses.
// V > 1: axis 0 stays in place and its extent is a multiple of V, so V
// consecutive result elements are V consecutive source elements.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void permute_gather_kernel(PermuteDesc d, size_t n,
                                                                const typename T::storage* __restrict__ src,
                                                                typename T::storage* dst, int accumulate) {
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * V; i < n;
       i += static_cast<size_t>(gridDim.x) * kBlock * V) {
    size_t rest = i, off = 0;
    for (int k = 0; k < d.rank; ++k) {
      const size_t e = static_cast<size_t>(d.out_dim[k]);
      off += (rest % e) * static_cast<size_t>(d.src_stride[k]);
      rest /= e;
    }
    float v[V];
    ld<T, V>(src + off, v);
    if (accumulate) {
      float old[V];
      ld<T, V>(dst + i, old);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] += old[e];
    }
    st<T, V>(dst + i, v);
  }
}

// The result's fastest axis is not the source's: 32 x 32 tiles over (result
// axis 0, the result axis `p` that is the source's axis 0) go through LDS so
// that both the reads and the writes run along contiguous addresses.
struct TiledDesc {
  PermuteDesc d;
  int p;                    // result axis that is source axis 0
  long long out_stride_p;   // stride of axis p in the result
  long long tiles0, tilesp; // tile counts along the two tiled axes
};

template <typename T>
__global__ __launch_bounds__(kBlock) void permute_tiled_kernel(TiledDesc t, size_t n_tiles,
                                                               const typename T::storage* __restrict__ src,
                                                               typename T::storage* dst, int accumulate) {
  __shared__ float tile[32][33];
  const PermuteDesc& d = t.d;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  for (size_t tile_id = blockIdx.x; tile_id < n_tiles; tile_id += gridDim.x) {
    size_t rest = tile_id;
    const long long t0 = static_cast<long long>(rest % t.tiles0);
    rest /= t.tiles0;
    const long long tp = static_cast<long long>(rest % t.tilesp);
    rest /= t.tilesp;
    // the remaining result axes (all but 0 and p), in order
    size_t src_off = 0, dst_off = 0, out_stride = 1;
    for (int k = 0; k < d.rank; ++k) {
      if (k != 0 && k != t.p) {
        const size_t e = static_cast<size_t>(d.out_dim[k]);
        const size_t idx = rest % e;
        rest /= e;
        src_off += idx * static_cast<size_t>(d.src_stride[k]);
        dst_off += idx * out_stride;
      }
      out_stride *= static_cast<size_t>(d.out_dim[k]);
    }
    const long long i0 = t0 * 32, ip = tp * 32;
    // read: source axis 0 (= result axis p) is contiguous -> tx walks it
#pragma unroll
    for (int j = 0; j < 32; j += 8) {
      const long long a0 = i0 + ty + j, ap = ip + tx;
      if (a0 < d.out_dim[0] && ap < d.out_dim[t.p])
        tile[ty + j][tx] = to_float<T>(src[src_off + a0 * d.src_stride[0] + ap]);
    }
    __syncthreads();
    // write: result axis 0 is contiguous -> tx walks it
#pragma unroll
    for (int j = 0; j < 32; j += 8) {
      const long long a0 = i0 + tx, ap = ip + ty + j;
      if (a0 < d.out_dim[0] && ap < d.out_dim[t.p]) {
        const size_t o = dst_off + static_cast<size_t>(a0) + static_cast<size_t>(ap * t.out_stride_p);
        float v = tile[tx][ty + j];
        if (accumulate) v += to_float<T>(dst[o]);
        dst[o] = from_float<T>(v);
      }
    }
    __syncthreads();
  }
}

// The same for the 16-bit types when both tiled extents are multiples of 4 and
// the operands 8-byte aligned: 64 x 64 tiles, every global access 8 bytes (four
// elements along the contiguous axis), so a thread moves 32 bytes each way
// instead of 8 and a wave's run is 128 contiguous bytes instead of 64.
template <typename T>
__global__ __launch_bounds__(kBlock) void permute_tiled64_kernel(TiledDesc t, size_t n_tiles,
                                                                 const uint16_t* __restrict__ src, uint16_t* dst,
                                                                 int accumulate) {
  typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
  constexpr int kStride = 68;  // halfs per LDS row: 8-byte aligned rows, spread over the banks
  __shared__ __attribute__((aligned(8))) uint16_t tile[64 * kStride];  // [axis p][axis 0]
  const PermuteDesc& d = t.d;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 groups of 4 elements x 16 rows
  for (size_t tile_id = blockIdx.x; tile_id < n_tiles; tile_id += gridDim.x) {
    size_t rest = tile_id;
    const long long t0 = static_cast<long long>(rest % t.tiles0);
    rest /= t.tiles0;
    const long long tp = static_cast<long long>(rest % t.tilesp);
    rest /= t.tilesp;
    size_t src_off = 0, dst_off = 0, out_stride = 1;
    for (int k = 0; k < d.rank; ++k) {
      if (k != 0 && k != t.p) {
        const size_t e = static_cast<size_t>(d.out_dim[k]);
        const size_t idx = rest % e;
        rest /= e;
        src_off += idx * static_cast<size_t>(d.src_stride[k]);
        dst_off += idx * out_stride;
      }
      out_stride *= static_cast<size_t>(d.out_dim[k]);
    }
    const long long i0 = t0 * 64, ip = tp * 64;
    // read along the source's contiguous axis (result axis p), store transposed
#pragma unroll
    for (int j = 0; j < 64; j += 16) {
      const long long a0 = i0 + ty + j, ap = ip + 4 * tx;
      if (a0 < d.out_dim[0] && ap < d.out_dim[t.p]) {
        const u16x4 v = *reinterpret_cast<const u16x4*>(src + src_off + a0 * d.src_stride[0] + ap);
#pragma unroll
        for (int e = 0; e < 4; ++e) tile[(4 * tx + e) * kStride + ty + j] = v[e];
      }
    }
    __syncthreads();
    // write along the result's contiguous axis
#pragma unroll
    for (int j = 0; j < 64; j += 16) {
      const long long a0 = i0 + 4 * tx, ap = ip + ty + j;
      if (a0 < d.out_dim[0] && ap < d.out_dim[t.p]) {
        u16x4 v = *reinterpret_cast<const u16x4*>(&tile[(ty + j) * kStride + 4 * tx]);
        uint16_t* o = dst + dst_off + static_cast<size_t>(a0) + static_cast<size_t>(ap * t.out_stride_p);
        if (accumulate) {
          const u16x4 old = *reinterpret_cast<const u16x4*>(o);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = from_float<T>(to_float<T>(old[e]) + to_float<T>(v[e]));
        }
        *reinterpret_cast<u16x4*>(o) = v;
      }
    }
    __syncthreads();
  }
}

// mask_size is a multiple of V when V > 1.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void mask_fill_kernel(size_t mask_size, size_t n,
                                                           const typename T::storage* __restrict__ mask, float value,
                                                           typename T::storage* x) {
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * V; i < n;
       i += static_cast<size_t>(gridDim.x) * kBlock * V) {
    float m[V], v[V];
    ld<T, V>(mask + i % mask_size, m);
    bool any = false;
#pragma unroll
    for (int e = 0; e < V; ++e) any = any || m[e] == 0.f;
    if (!any) continue;
    ld<T, V>(x + i, v);
#pragma unroll
    for (int e = 0; e < V; ++e)
      if (m[e] == 0.f) v[e] = value;
    st<T, V>(x + i, v);
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void upper_tri_kernel(int n, typename T::storage* dst) {
  const size_t total = static_cast<size_t>(n) * n;
  const typename T::storage one = from_float<T>(1.f), zero = from_float<T>(0.f);
  for (size_t i = blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * kBlock) {
    const size_t r = i % n, c = i / n;
    dst[i] = r <= c ? one : zero;
  }
}

}  // namespace
}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" {

int ginn_hip_layernorm_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, float eps,
                           void* y, float* std_out) {
  GH_CHECK_ARG(ctx, "ginn_hip_layernorm_fwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_layernorm_fwd: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && y && std_out, "ginn_hip_layernorm_fwd: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(cols), kWaves, ctx->num_cus);
  const bool vec = vec8_ok({x, y}, {static_cast<size_t>(rows)});
  GH_DISPATCH_DTYPE_V(dtype, vec, (layernorm_fwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), eps, static_cast<T::storage*>(y), std_out, nullptr, nullptr, 0.f,
      nullptr)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_layernorm_affine_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, float eps,
                                  const void* gamma, const void* beta, float multiplier_bias, void* y, float* std_out,
                                  void* z) {
  GH_CHECK_ARG(ctx, "ginn_hip_layernorm_affine_fwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_layernorm_affine_fwd: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && gamma && beta && y && std_out && z, "ginn_hip_layernorm_affine_fwd: NULL pointer");
  GH_CHECK_ARG(z != x && z != y, "ginn_hip_layernorm_affine_fwd: z must be an array of its own");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(cols), kWaves, ctx->num_cus);
  const bool vec = vec8_ok({x, y, z, gamma, beta}, {static_cast<size_t>(rows)});
  GH_DISPATCH_DTYPE_V(dtype, vec, (layernorm_fwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), eps, static_cast<T::storage*>(y), std_out,
      static_cast<const T::storage*>(gamma), static_cast<const T::storage*>(beta), multiplier_bias,
      static_cast<T::storage*>(z))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_layernorm_affine_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dz,
                                  const void* y, const float* std_in, const void* gamma, float multiplier_bias,
                                  void* dx, int accumulate, void* dgamma, void* dbeta) {
  GH_CHECK_ARG(ctx, "ginn_hip_layernorm_affine_bwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_layernorm_affine_bwd: negative dimension");
  if (rows == 0 || cols == 0 || (!dx && !dgamma && !dbeta)) return kOk;
  GH_CHECK_ARG(dz && y && std_in && gamma, "ginn_hip_layernorm_affine_bwd: NULL pointer");
  GH_CHECK_ARG((dgamma == nullptr) == (dbeta == nullptr),
               "ginn_hip_layernorm_affine_bwd: dgamma and dbeta come together");
  GH_CHECK_ARG(dx != dz && dx != y, "ginn_hip_layernorm_affine_bwd: dx must not be an input");
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({dz, y, dx, gamma}, {static_cast<size_t>(rows)});
  const int per_iter = 64 * (vec ? 8 : 1);
  if (rows > per_iter * kLnRowIters) {
    // A column longer than a wave holds in registers: the two steps one after the other, through a
    // temporary for the gradient of the normalised values.
    void* da = nullptr;
    const size_t bytes = static_cast<size_t>(rows) * cols * dtype_size(dtype);
    if (int rc = ginn_hip_malloc(ctx, bytes, &da)) return rc;
    int rc = ginn_hip_memset(ctx, da, 0, bytes);
    if (rc == kOk)
      rc = ginn_hip_cwise_prod_add_bwd(ctx, dtype, rows, cols, dz, y, gamma, multiplier_bias, 1, da, dgamma, dbeta);
    if (rc == kOk && dx)
      rc = (accumulate ? ginn_hip_layernorm_bwd : ginn_hip_layernorm_bwd_assign)(ctx, dtype, rows, cols, da, y,
                                                                                  std_in, dx);
    const int rc_free = ginn_hip_free(ctx, da);
    return rc != kOk ? rc : rc_free;
  }
  std::lock_guard<std::mutex> lock(ctx->mutex);
  // At most two workgroups per CU: every workgroup leaves a partial row for the fold.
  unsigned grid = grid_for(static_cast<size_t>(cols), kLnBwdWaves, ctx->num_cus);
  const unsigned cap = 2 * static_cast<unsigned>(ctx->num_cus);
  if (grid > cap) grid = cap;
  const size_t part_bytes = static_cast<size_t>(grid) * rows * sizeof(float);
  rowred::Partials room{nullptr, false};
  if (dgamma) {
    GH_CHECK_ARG(2 * part_bytes <= ctx->workspace_bytes, "ginn_hip_layernorm_affine_bwd: workspace too small for %d rows",
                 rows);
    room = rowred::take_partials(ctx, 2 * part_bytes);
  }
  float* part_g = room.base;
  float* part_b = part_g ? part_g + static_cast<size_t>(grid) * rows : nullptr;
  const int iters = (rows + per_iter - 1) / per_iter;
#define GH_LN_BWD(ITERS)                                                                                       \
  GH_DISPATCH_DTYPE_V(dtype, vec, (layernorm_affine_bwd_kernel<T, V, ITERS><<<grid, kLnBwdWaves * 64, 0, ctx->stream>>>( \
      rows, cols, static_cast<const T::storage*>(dz), static_cast<const T::storage*>(y), std_in,              \
      static_cast<const T::storage*>(gamma), multiplier_bias, static_cast<T::storage*>(dx), accumulate,       \
      part_g, part_b)))
  if (iters <= 1) {
    GH_LN_BWD(1);
  } else if (iters == 2) {
    GH_LN_BWD(2);
  } else {
    GH_LN_BWD(kLnRowIters);
  }
#undef GH_LN_BWD
  GH_HIP(hipGetLastError());
  if (dgamma)
    return rowred::finish(ctx, {dtype, rows, static_cast<int>(grid), 1, part_g, part_b, dgamma, dbeta}, room.deferred);
  return kOk;
}

static int layernorm_bwd(const char* who, ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dy,
                         const void* y, const float* std_in, void* dx, int accumulate) {
  GH_CHECK_ARG(ctx, "%s: ctx is NULL", who);
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "%s: negative dimension", who);
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(dy && y && std_in && dx, "%s: NULL pointer", who);
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(cols), kWaves, ctx->num_cus);
  const bool vec = vec8_ok({dy, y, dx}, {static_cast<size_t>(rows)});
  GH_DISPATCH_DTYPE_V(dtype, vec, (layernorm_bwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(dy), static_cast<const T::storage*>(y), std_in,
      static_cast<T::storage*>(dx), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_layernorm_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dy, const void* y,
                           const float* std_in, void* dx) {
  return layernorm_bwd("ginn_hip_layernorm_bwd", ctx, dtype, rows, cols, dy, y, std_in, dx, 1);
}

int ginn_hip_layernorm_bwd_assign(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dy,
                                  const void* y, const float* std_in, void* dx) {
  return layernorm_bwd("ginn_hip_layernorm_bwd_assign", ctx, dtype, rows, cols, dy, y, std_in, dx, 0);
}

int ginn_hip_cwise_prod_add_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* a,
                                const void* b, const void* c, float multiplier_bias, int broadcast, void* y) {
  GH_CHECK_ARG(ctx, "ginn_hip_cwise_prod_add_fwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_cwise_prod_add_fwd: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(a && b && c && y, "ginn_hip_cwise_prod_add_fwd: NULL pointer");
  if (dtype == GINN_HIP_I32)
    return launch_int_arith(ctx, kIntMulAdd, static_cast<size_t>(rows) * cols, broadcast ? static_cast<size_t>(rows) : 0,
                            a, b, c, static_cast<int>(multiplier_bias), 0, y, 0);
  GH_HIP(hipSetDevice(ctx->device));
  const size_t n = static_cast<size_t>(rows) * cols;
  const bool vec = vec8_ok({a, b, c, y}, {static_cast<size_t>(rows)});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (cwise_prod_add_fwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, n, static_cast<const T::storage*>(a), static_cast<const T::storage*>(b),
      static_cast<const T::storage*>(c), multiplier_bias, broadcast, static_cast<T::storage*>(y))));
  GH_HIP(hipGetLastError());
  return kOk;
}

static int cwise_prod_add_bwd(const char* who, ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols,
                              const void* dy, const void* a, const void* b, float multiplier_bias, int broadcast,
                              void* da, void* db, void* dc, int add_da) {
  GH_CHECK_ARG(ctx, "%s: ctx is NULL", who);
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "%s: negative dimension", who);
  if (rows == 0 || cols == 0 || (!da && !db && !dc)) return kOk;
  GH_CHECK_ARG(dy && a && b, "%s: NULL pointer", who);
  GH_HIP(hipSetDevice(ctx->device));
  if (!broadcast) {
    const size_t n = static_cast<size_t>(rows) * cols;
    const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
    GH_DISPATCH_DTYPE(dtype, (cwise_prod_add_bwd_flat_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
        n, static_cast<const T::storage*>(dy), static_cast<const T::storage*>(a), static_cast<const T::storage*>(b),
        multiplier_bias, static_cast<T::storage*>(da), static_cast<T::storage*>(db), static_cast<T::storage*>(dc),
        add_da)));
    GH_HIP(hipGetLastError());
    return kOk;
  }
  std::lock_guard<std::mutex> lock(ctx->mutex);  // the workspace holds the partials
  const bool vec = vec8_ok({dy, a, b, da}, {static_cast<size_t>(rows)});
  const rowred::Plan plan = rowred::plan(rows, cols, ctx->num_cus, ctx->workspace_bytes, 2, vec ? 8 : 1);
  GH_CHECK_ARG(plan.chunks >= 1, "%s: workspace too small for %d rows", who, rows);
  const rowred::Partials room = rowred::take_partials(ctx, 2 * static_cast<size_t>(plan.chunks) * rows * sizeof(float));
  float* part_b = room.base;
  float* part_c = part_b + static_cast<size_t>(plan.chunks) * rows;
  GH_DISPATCH_DTYPE_V(dtype, vec, (cwise_prod_add_bwd_bcast_kernel<T, V><<<dim3(plan.row_blocks, plan.chunks),
                                                                           rowred::kBlock, 0, ctx->stream>>>(
      rows, cols, plan.cols_per_chunk, static_cast<const T::storage*>(dy), static_cast<const T::storage*>(a),
      static_cast<const T::storage*>(b), multiplier_bias, static_cast<T::storage*>(da), part_b, part_c, add_da)));
  GH_HIP(hipGetLastError());
  if (db || dc) return rowred::finish(ctx, {dtype, rows, plan.chunks, 1, part_b, part_c, db, dc}, room.deferred);
  return kOk;
}

int ginn_hip_cwise_prod_add_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dy,
                                const void* a, const void* b, float multiplier_bias, int broadcast, void* da,
                                void* db, void* dc) {
  return cwise_prod_add_bwd("ginn_hip_cwise_prod_add_bwd", ctx, dtype, rows, cols, dy, a, b, multiplier_bias, broadcast,
                            da, db, dc, 1);
}

int ginn_hip_cwise_prod_add_bwd_assign(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dy,
                                       const void* a, const void* b, float multiplier_bias, int broadcast, void* da,
                                       void* db, void* dc) {
  return cwise_prod_add_bwd("ginn_hip_cwise_prod_add_bwd_assign", ctx, dtype, rows, cols, dy, a, b, multiplier_bias,
                            broadcast, da, db, dc, 0);
}

int ginn_hip_permute(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rank, const long long* host_dims,
                     const int* host_perm, const void* src, void* dst, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_permute: ctx is NULL");
  GH_CHECK_ARG(rank >= 1 && rank <= kMaxRank, "ginn_hip_permute: rank %d not in 1..%d", rank, kMaxRank);
  GH_CHECK_ARG(host_dims && host_perm, "ginn_hip_permute: NULL dims or perm");
  long long src_stride[kMaxRank];
  bool seen[kMaxRank] = {};
  size_t n = 1;
  for (int k = 0; k < rank; ++k) {
    GH_CHECK_ARG(host_dims[k] >= 0, "ginn_hip_permute: negative dimension");
    GH_CHECK_ARG(host_perm[k] >= 0 && host_perm[k] < rank && !seen[host_perm[k]],
                 "ginn_hip_permute: perm is not a permutation of 0..%d", rank - 1);
    seen[host_perm[k]] = true;
    src_stride[k] = static_cast<long long>(n);
    n *= static_cast<size_t>(host_dims[k]);
  }
  if (n == 0) return kOk;
  GH_CHECK_ARG(src && dst, "ginn_hip_permute: NULL pointer");
  GH_CHECK_ARG(src != dst, "ginn_hip_permute: in-place permutation is not supported");
  PermuteDesc d{};
  d.rank = rank;
  for (int k = 0; k < rank; ++k) {
    d.out_dim[k] = host_dims[host_perm[k]];
    d.src_stride[k] = src_stride[host_perm[k]];
  }
  GH_HIP(hipSetDevice(ctx->device));
  if (host_perm[0] != 0 && d.out_dim[0] >= 8) {
    TiledDesc t{};
    t.d = d;
    for (int k = 0; k < rank; ++k)
      if (host_perm[k] == 0) t.p = k;
    if (d.out_dim[t.p] >= 8) {
      long long stride = 1;
      for (int k = 0; k < t.p; ++k) stride *= d.out_dim[k];
      t.out_stride_p = stride;
      if (dtype != GINN_HIP_F32 && d.out_dim[0] % 4 == 0 && d.out_dim[t.p] % 4 == 0 &&
          reinterpret_cast<uintptr_t>(src) % 8 == 0 && reinterpret_cast<uintptr_t>(dst) % 8 == 0) {
        t.tiles0 = (d.out_dim[0] + 63) / 64;
        t.tilesp = (d.out_dim[t.p] + 63) / 64;
        size_t n_tiles = static_cast<size_t>(t.tiles0) * t.tilesp;
        for (int k = 1; k < rank; ++k)
          if (k != t.p) n_tiles *= static_cast<size_t>(d.out_dim[k]);
        const unsigned grid = grid_for(n_tiles, 1, ctx->num_cus * 4);
        if (dtype == GINN_HIP_F16)
          permute_tiled64_kernel<F16><<<grid, kBlock, 0, ctx->stream>>>(
              t, n_tiles, static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), accumulate);
        else
          permute_tiled64_kernel<BF16><<<grid, kBlock, 0, ctx->stream>>>(
              t, n_tiles, static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), accumulate);
        GH_HIP(hipGetLastError());
        return kOk;
      }
      t.tiles0 = (d.out_dim[0] + 31) / 32;
      t.tilesp = (d.out_dim[t.p] + 31) / 32;
      size_t n_tiles = static_cast<size_t>(t.tiles0) * t.tilesp;
      for (int k = 1; k < rank; ++k)
        if (k != t.p) n_tiles *= static_cast<size_t>(d.out_dim[k]);
      const unsigned grid = grid_for(n_tiles, 1, ctx->num_cus * 4);
      GH_DISPATCH_DTYPE(dtype, (permute_tiled_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
          t, n_tiles, static_cast<const T::storage*>(src), static_cast<T::storage*>(dst), accumulate)));
      GH_HIP(hipGetLastError());
      return kOk;
    }
  }
  const bool vec = host_perm[0] == 0 && vec8_ok({src, dst}, {static_cast<size_t>(host_dims[0])});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (permute_gather_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      d, n, static_cast<const T::storage*>(src), static_cast<T::storage*>(dst), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_mask_fill(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t mask_size, size_t batch, const void* mask,
                       float value, void* x) {
  GH_CHECK_ARG(ctx, "ginn_hip_mask_fill: ctx is NULL");
  if (mask_size == 0 || batch == 0) return kOk;
  GH_CHECK_ARG(mask && x, "ginn_hip_mask_fill: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  const size_t n = mask_size * batch;
  const bool vec = vec8_ok({mask, x}, {mask_size});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (mask_fill_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      mask_size, n, static_cast<const T::storage*>(mask), value, static_cast<T::storage*>(x))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_upper_tri(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int n, void* dst) {
  GH_CHECK_ARG(ctx, "ginn_hip_upper_tri: ctx is NULL");
  GH_CHECK_ARG(n >= 0, "ginn_hip_upper_tri: negative size");
  if (n == 0) return kOk;
  GH_CHECK_ARG(dst, "ginn_hip_upper_tri: NULL pointer");
  if (dtype == GINN_HIP_I32) return launch_int_upper_tri(ctx, static_cast<size_t>(n), dst);
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(n) * n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (upper_tri_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(n, static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

}  // extern "C"
