// Product kernel with 128 x 128 block tiles (and 128 x 64 / 64 x 128 variants)
// for fp16 / bf16 (fp32 accumulate) and fp32: the mid-size aligned 16-bit
// shapes, where a 256 x 256 tiling leaves most of the chip idle, and every
// aligned fp32 shape with enough tiles.
//
// Block tile (64 FM) x (64 FN) x 128 bytes of K (64 16-bit or 32 fp32 values)
// with FM, FN in {1, 2}: the output is split over a 2 x 2 grid of wave
// quadrants, (32 FM) x (32 FN) = FM x FN MFMA 32 x 32 tiles each (32x32x16 for
// the 16-bit types, 32x32x2 for fp32), and every quadrant is worked on by two
// waves that split K (512 threads = 8 waves).  128 x 128 is the work horse;
// 128 x 64 and 64 x 128 take the shapes with a 64-wide side (attention
// products with head size 64, right-hand sides of 64 columns).  Four LDS
// stages filled by direct global -> LDS loads keep up to three K tiles in
// flight per CU.  A K tile is four sub-steps of 32 bytes of K, two per wave; a
// wave's fragment reads run two of its sub-steps (= one K tile) ahead of the
// MFMAs, with waits by count, and the one barrier per K tile is passed a whole
// tile before the data it guards is multiplied, so that neither LDS latency
// nor the barrier is exposed at a tile boundary.  Optional split-K over
// blockIdx.z (fp32 partial tiles, folded by the common reduce kernel) for
// products whose output has few tiles but a long K (weight gradients).
//
// LDS layouts of an operand tile of R = 64 F rows (XOR swizzles applied on the
// global side of the direct loads):
//   K-contiguous operand: [R rows][8 chunks of 16 B], chunk ^ ((row >> 1) & 7);
//   row-contiguous operand, 16 bit: [64 k][R / 8 chunks of 16 B], chunk ^ (4 * (k & 3))
//     for R = 128 and chunk ^ (4 * ((k >> 1) & 1)) for R = 64, which puts the four
//     k-rows a 16-lane transposing read touches into different banks;
//   row-contiguous operand, fp32: [32 k][R / 4 chunks of 16 B], unswizzled (read
//     4 bytes per lane along the rows).
#ifndef GINN_HIP_GEMM_MID_H
#define GINN_HIP_GEMM_MID_H

#include <type_traits>

#include "common.h"

namespace ginn_hip {
namespace mid {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Sixteen zero bytes in device memory: where a direct load must deliver zeros (K values beyond the end of
// a ragged K) its lane reads them from here instead of the operand.
static __device__ __attribute__((aligned(16))) const unsigned int kZeroChunk[4] = {0u, 0u, 0u, 0u};

constexpr int kRowBytes = 128;  // bytes of one K tile along K: 64 16-bit or 32 fp32 values
constexpr int kThreads = 512;   // 8 waves
// LDS stages per tile shape.  The loads of a workgroup's next stages are all it has in flight.  Measured (bf16,
// one MI355X, stages 4 / deeper): 64 x 64 tiles (16 KiB stages) 768 x 768 x 4096 17.2 / 15.9-16.0 us with 6 or 8
// stages, 1024^3 and 1000^3 level; 128 x 128 tiles (32 KiB) get SLOWER with a fifth stage (768 x 4096 x 3072 TN
// 24.5 -> 27.7 us, K = 8192 57.7 -> 63.3 us, fp32 2048^3 130 -> 136 us: their K loop is not waiting for latency) and
// 128 x 64 tiles do not care (6 against 4 stages within 1 %).  GPT layer: 380 -> 384 TFLOP/s with 8 / 4 / 4.
#ifndef GH_MID_STAGES_11
#define GH_MID_STAGES_11 8
#endif
#ifndef GH_MID_STAGES_21
#define GH_MID_STAGES_21 4
#endif
#ifndef GH_MID_STAGES_22
#define GH_MID_STAGES_22 4
#endif
constexpr int stages_for(int fm, int fn) {
  return fm + fn == 2 ? GH_MID_STAGES_11 : (fm + fn == 3 ? GH_MID_STAGES_21 : GH_MID_STAGES_22);
}

enum Epilogue { kPlain = 0, kGeneral = 1, kPartial = 2 };

template <int FM, int FN>
struct Geo {
  static constexpr int BM = 64 * FM, BN = 64 * FN;
  static constexpr int kTileA = BM * kRowBytes;       // bytes of one A tile
  static constexpr int kTileB = BN * kRowBytes;
  static constexpr int kStageBytes = kTileA + kTileB;
  static constexpr int kStages = stages_for(FM, FN);
  static_assert(kStages >= 3 && kStages <= 8, "pipeline depth");
  static constexpr int kLdsBytes = kStages * kStageBytes;
  static_assert(kLdsBytes <= 160 * 1024, "the stages must fit the LDS of a CU");
  // Epilogue staging inside the first two stages, per wave:
  //   plain: 32 FN columns x 32 FM halfs, column stride 64 FM + 16 bytes;
  //   general: 32 columns x 32 FM floats per pass, column stride 128 FM + 16 bytes.
  static constexpr int kEpiColStride = 64 * FM + 16;
  static constexpr int kF32ColStride = 128 * FM + 16;
  static constexpr int kEpiWaveBytes =
      (32 * FN * kEpiColStride > 32 * kF32ColStride) ? 32 * FN * kEpiColStride : 32 * kF32ColStride;
  static_assert(4 * kEpiWaveBytes <= 2 * kStageBytes, "staging must fit two stages");
};

struct MidParams {
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
  int tiles_m, tiles_n;
  int group;      // tile rows walked together (0: plain column-major tile order)
  int k_tiles;    // K tiles per split
  float* partial; // split-K: [split][n][m] fp32
};

__device__ __forceinline__ int swz_kc(int row) { return (row >> 1) & 7; }
// Row-contiguous 16-bit tiles: XOR of the chunk position that puts the four
// k-rows a 16-lane transposing read touches into different banks.  fp32 tiles
// are read 4 bytes per lane along the rows and need none.
template <int F, int ES>
__device__ __forceinline__ int swz_rc(int kr) {
  if (ES == 4) return 0;
  return F == 2 ? 4 * (kr & 3) : 4 * ((kr >> 1) & 1);
}

// Element offset, relative to the tile origin at K offset 0, of the 16-byte
// chunk that lands at linear LDS chunk position v of an operand tile of 64 F
// rows; ES = element size in bytes.
// Tile rows from `valid` on (a tile that reaches beyond the matrix) re-read a
// row inside it: in bounds, and what they produce is never stored.
template <bool KC, int F, int ES>
__device__ __forceinline__ long long chunk_src(int v, int ld, int valid) {
  constexpr int kPer = 16 / ES;  // elements per chunk
  if (KC) {
    const int row = v >> 3, pc = v & 7;
    return (long long)min(row, valid - 1) * ld + ((pc ^ swz_kc(row)) * kPer);
  }
  constexpr int kChunks = 64 * F * ES / 16;  // per k-row
  const int kr = v / kChunks, pj = v % kChunks;
  const int row0 = (pj ^ swz_rc<F, ES>(kr)) * kPer;  // first of the chunk's rows
  return (long long)kr * ld + (row0 < valid ? row0 : 0);
}

// Byte offset inside a K-contiguous tile of lane's 16 bytes of the fragment
// rows r0 .. r0+31, sub-step ks (16 k values).
__device__ __forceinline__ int kc_offset(int r0, int ks, int lane) {
  const int row = r0 + (lane & 31);
  const int c = 2 * ks + (lane >> 5);
  return row * 128 + ((c ^ swz_kc(row)) * 16);
}

// Byte offset inside a row-contiguous tile of half t (k + 4t .. k + 4t + 3)
// of the transposed fragment: a 16-lane group reads 4 k-rows x 32 bytes and
// every lane receives 4 k values of its own row.
template <int F>
__device__ __forceinline__ int tr_offset(int r0, int ks, int t, int lane) {
  const int g = lane >> 4, s = lane & 15, h = g & 1, q = g >> 1;
  const int mcol = r0 + 16 * h + 4 * (s & 3);
  const int j = mcol >> 3, within = (mcol & 7) * 2;
  const int kr = 16 * ks + 8 * q + 4 * t + (s >> 2);
  return kr * (128 * F) + ((j ^ swz_rc<F, 2>(kr)) * 16) + within;
}

// fp32 row-contiguous tile [32 k][64 F rows]: byte offset of lane's element of
// the fragment rows r0 .. r0+31 for the MFMA that multiplies k = 8 s + jj
// (lanes 0..31) and 8 s + 4 + jj (lanes 32..63), at (s, jj) = (0, 0); the
// others lie (8 s + jj) * 256 F bytes further.
template <int F>
__device__ __forceinline__ int rc32_offset(int r0, int lane) {
  return (4 * (lane >> 5)) * (256 * F) + (r0 + (lane & 31)) * 4;
}

// LDS fragment reads go through inline assembly, and so do their waits: the
// kernel keeps the reads of two sub-steps in flight and waits with a count
// (LDS reads complete in order), which the compiler would not do across the
// direct loads in flight (it places a full vmcnt(0) wait in front of the
// transposing-read builtin).  A value is usable after lgkm_wait<N>() with N =
// the number of LDS reads issued after it, followed by claim() on its registers.
template <int OFF>
__device__ __forceinline__ u32x2 tr_issue(uint32_t lds_byte_addr) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(lds_byte_addr), "n"(OFF) : "memory");
  return v;
}
template <int OFF>
__device__ __forceinline__ u32x4 b128_issue(uint32_t lds_byte_addr) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_byte_addr), "n"(OFF) : "memory");
  return v;
}
template <int OFF>
__device__ __forceinline__ uint32_t b32_issue(uint32_t lds_byte_addr) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  uint32_t v;
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(lds_byte_addr), "n"(OFF) : "memory");
  return v;
}
template <int N>
__device__ __forceinline__ void lgkm_wait() {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(N) : "memory");
}
// Ties registers to the wait in front of it: their first use cannot be moved
// above this point.
__device__ __forceinline__ void claim(u32x2& v) { asm volatile("" : "+v"(v) : : "memory"); }
__device__ __forceinline__ void claim(u32x4& v) { asm volatile("" : "+v"(v) : : "memory"); }
__device__ __forceinline__ void claim(uint32_t& v) { asm volatile("" : "+v"(v) : : "memory"); }
// One fragment pair (16 bytes per lane and operand) into the 32 x 32 tile c:
// a single 32x32x16 MFMA for the 16-bit types, four 32x32x2 MFMAs for fp32
// (component j of both operands per MFMA).
template <typename T>
__device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (std::is_same<T, F32>::value) {
    // (components through named scalars: a bit cast applied to a vector
    // element expression directly reads element 0 every time)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t ua = a[j], ub = b[j];
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(ua), __uint_as_float(ub), c, 0, 0, 0);
    }
    return c;
  } else if constexpr (std::is_same<T, BF16>::value) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
  }
}

// f(R) for R = N, N - 1, ..., 1 as compile-time constants.
template <int N, typename F>
__device__ __forceinline__ void tail_tiles(F&& f) {
  if constexpr (N >= 1) {
    f(std::integral_constant<int, N>{});
    tail_tiles<N - 1>(f);
  }
}

// 8 waves: waves 4 .. 7 own the same output quadrants as waves 0 .. 3 but take
// sub-steps 2, 3 of every K tile (waves 0 .. 3: sub-steps 0, 1) and hand their
// sums over through LDS at the end.  A SIMD so holds two waves, and one issues
// while the other waits: beside its 4 MFMAs a sub-step needs LDS reads, waits
// and address arithmetic, and one wave per SIMD is bound by instruction issue,
// not by the matrix pipe, LDS or the loads.  For the same reason the loop is
// kept lean: LDS addresses are per-lane bases plus immediate offsets, the
// loads take a scalar base plus a 32-bit lane offset, and the steady state of
// the K loop carries no conditions.
template <typename T, bool AKC, bool BKC, int EPI, int FM, int FN>
__global__ __launch_bounds__(kThreads) void gemm_mid_kernel(MidParams p) {
  using G = Geo<FM, FN>;
  constexpr int kStages = G::kStages;
  constexpr int ES = sizeof(typename T::storage);  // 2 or 4
  constexpr int BK = kRowBytes / ES;               // 64 or 32 k values per K tile
  constexpr bool F32IN = ES == 4;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int quad = wave & 3, kgroup = wave >> 2;
  const int wm = (quad & 1) * 32 * FM, wn = (quad >> 1) * 32 * FN;

  // Workgroup ids are dealt round-robin to the 8 XCDs: give each XCD a
  // contiguous range of the tile sequence, walked in column panels of `group`
  // tile rows, so that concurrently running tiles share operands in its L2.
  int pid = blockIdx.x;
  if (p.group > 0) {
    const int per = (p.tiles_m * p.tiles_n) >> 3;
    pid = (pid & 7) * per + (pid >> 3);
    const int width = p.group * p.tiles_n;
    const int first_m = (pid / width) * p.group;
    const int gsz = min(p.tiles_m - first_m, p.group);
    const int in_group = pid % width;
    pid = (in_group / gsz) * p.tiles_m + first_m + in_group % gsz;
  }
  const int m0 = (pid % p.tiles_m) * G::BM, n0 = (pid / p.tiles_m) * G::BN;
  const long long bz = blockIdx.y;
  const int split = blockIdx.z;

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int kt_total = (p.k + BK - 1) / BK;
  const int kt0 = split * p.k_tiles;
  const int KT = min(p.k_tiles, kt_total - kt0);
  // K values in the last K tile of the product when K is no multiple of the tile (0: it is): the lanes
  // whose 16 bytes lie beyond them load zeros instead.  Only the split that holds that tile sees it.
  const int k_rem = (kt0 + KT == kt_total) ? p.k % BK : 0;

  // ---- direct loads.  Thread `tid` moves chunk v = i * 512 + tid (i < F) of an
  // operand tile; the swizzle only involves row bits below 32 (KC) / k bits
  // below 16 (RC), so the lane-dependent part of the source offset is the same
  // for every i and the i-dependent part is uniform.
  constexpr int kRowsPerPass = kThreads / 8;  // tile rows (KC) one pass of 512 chunks covers
  // rows (KC) or k-rows (RC: 64 F ES / 16 chunks per k-row) covered by one pass
  constexpr int kRcRowsPerPassA = kThreads / (64 * FM * ES / 16);
  constexpr int kRcRowsPerPassB = kThreads / (64 * FN * ES / 16);
  const long long a_istep = (AKC ? (long long)kRowsPerPass : (long long)kRcRowsPerPassA) * p.lda * ES;
  const long long b_istep = (BKC ? (long long)kRowsPerPass : (long long)kRcRowsPerPassB) * p.ldb * ES;
  const long long a_kstep = (AKC ? (long long)BK : (long long)BK * p.lda) * ES;
  const long long b_kstep = (BKC ? (long long)BK : (long long)BK * p.ldb) * ES;
  // m and n need not fill the last tile row / column: tile rows beyond them
  // re-read a valid one (K-contiguous operand: the last valid row; row-contiguous
  // operand: the chunk of 16 bytes at the tile's first row, extents along the
  // rows being multiples of 16 bytes) -- in bounds, and what they produce is
  // never stored.
  const int m_valid = min(G::BM, p.m - m0), n_valid = min(G::BN, p.n - n0);
  uint32_t a_off[FM], b_off[FN];  // byte offsets of this thread's chunks from the tile origin
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    if (AKC) {
      const int row = i * kRowsPerPass + (tid >> 3);
      a_off[i] = (uint32_t)((long long)min(row, m_valid - 1) * p.lda * ES + (((tid & 7) ^ swz_kc(row)) * 16));
    } else {
      a_off[i] = (uint32_t)(chunk_src<AKC, FM, ES>(tid, p.lda, m_valid) * ES + i * a_istep);
    }
  }
#pragma unroll
  for (int i = 0; i < FN; ++i) {
    if (BKC) {
      const int row = i * kRowsPerPass + (tid >> 3);
      b_off[i] = (uint32_t)((long long)min(row, n_valid - 1) * p.ldb * ES + (((tid & 7) ^ swz_kc(row)) * 16));
    } else {
      b_off[i] = (uint32_t)(chunk_src<BKC, FN, ES>(tid, p.ldb, n_valid) * ES + i * b_istep);
    }
  }
  // Whether this thread's chunk of the LAST, partly filled K tile holds K values
  // of the product (K-contiguous operand: its chunk along K, the same in every
  // pass; row-contiguous operand: the k-row, by pass).
  constexpr int kPerChunk = 16 / ES;
  const bool a_kc_ok = (((tid & 7) ^ swz_kc(tid >> 3)) * kPerChunk) < k_rem;
  const bool b_kc_ok = a_kc_ok;
  const int a_rc_kr = tid / (64 * FM * ES / 16), b_rc_kr = tid / (64 * FN * ES / 16);
  // Origins of the next tile to load (uniform).
  const char* a_next = static_cast<const char*>(p.A) +
                       (bz * p.sa + (AKC ? (long long)m0 * p.lda : (long long)m0)) * ES + kt0 * a_kstep;
  const char* b_next = static_cast<const char*>(p.B) +
                       (bz * p.sb + (BKC ? (long long)n0 * p.ldb : (long long)n0)) * ES + kt0 * b_kstep;
  // The direct loads of the next tile into stage buf; the LDS address is
  // wave-uniform, lane l lands 16 * l bytes behind it.
  auto issue_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      uint32_t off = a_off[i];
      asm volatile("" : "+v"(off));  // keeps (scalar base) + (32-bit lane offset) apart for the addressing mode
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(a_next + off),
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + (i * kThreads + wave * 64) * 16), 16, 0,
          0);
    }
#pragma unroll
    for (int i = 0; i < FN; ++i) {
      uint32_t off = b_off[i];
      asm volatile("" : "+v"(off));
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(b_next + off),
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + G::kTileA +
                                                    (i * kThreads + wave * 64) * 16),
          16, 0, 0);
    }
    a_next += a_kstep;
    b_next += b_kstep;
  };
  // The same for the partly filled last K tile: a lane whose 16 bytes lie beyond
  // K reads zeros (a per-lane address instead of scalar base + lane offset).
  auto issue_last_tile = [&](int buf) {
    const char* zeros = reinterpret_cast<const char*>(kZeroChunk);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const bool ok = AKC ? a_kc_ok : (i * kRcRowsPerPassA + a_rc_kr) < k_rem;
      const char* g = ok ? a_next + a_off[i] : zeros;
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)g,
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + (i * kThreads + wave * 64) * 16), 16, 0,
          0);
    }
#pragma unroll
    for (int i = 0; i < FN; ++i) {
      const bool ok = BKC ? b_kc_ok : (i * kRcRowsPerPassB + b_rc_kr) < k_rem;
      const char* g = ok ? b_next + b_off[i] : zeros;
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)g,
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + G::kTileA +
                                                    (i * kThreads + wave * 64) * 16),
          16, 0, 0);
    }
  };
  constexpr int kLoads = FM + FN;  // direct loads per thread and K tile
  // Waits until at most `newer` whole tiles of this thread's direct loads are pending.
  static_assert((kStages - 2) * kLoads < 64, "vmcnt is a 6-bit counter");
  auto wait_tiles = [&](int newer) {
    switch (newer) {
      case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kLoads) : "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * kLoads) : "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(3 * kLoads) : "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(4 * kLoads) : "memory"); break;
      case 5: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(5 * kLoads) : "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(6 * kLoads) : "memory"); break;
    }
  };

  // ---- fragment reads.  This wave takes sub-steps ks0, ks0 + 1 of every K
  // tile, one fragment set each; while a set is multiplied the reads of the
  // other are in flight, and a set is refilled (from the next tile) right
  // after its MFMAs.  A K-contiguous fragment is one 16-byte read whose
  // swizzled address depends on the sub-step (a base per sub-step); a
  // row-contiguous one is two transposing 8-byte reads (halves) at a per-lane
  // base plus sub-step * 2048 F + half * 512 F.
  const int ks0 = kgroup * 2;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  uint32_t abase[AKC ? 2 * FM : FM], bbase[BKC ? 2 * FN : FN];  // offsets inside a stage
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    if (AKC) {
      abase[2 * i] = kc_offset(wm + i * 32, ks0, lane);
      abase[2 * i + 1] = kc_offset(wm + i * 32, ks0 + 1, lane);
    } else if (F32IN) {
      abase[i] = rc32_offset<FM>(wm + i * 32, lane) + ks0 * 8 * 256 * FM;
    } else {
      abase[i] = tr_offset<FM>(wm + i * 32, ks0, 0, lane);
    }
  }
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    if (BKC) {
      bbase[2 * j] = G::kTileA + kc_offset(wn + j * 32, ks0, lane);
      bbase[2 * j + 1] = G::kTileA + kc_offset(wn + j * 32, ks0 + 1, lane);
    } else if (F32IN) {
      bbase[j] = G::kTileA + rc32_offset<FN>(wn + j * 32, lane) + ks0 * 8 * 256 * FN;
    } else {
      bbase[j] = G::kTileA + tr_offset<FN>(wn + j * 32, ks0, 0, lane);
    }
  }
  uint32_t acur[AKC ? 2 * FM : FM], bcur[BKC ? 2 * FN : FN];  // the same inside the stage being read
  auto set_stage = [&](int buf) {
    const uint32_t sb = lds_base + buf * G::kStageBytes;
#pragma unroll
    for (int i = 0; i < (AKC ? 2 * FM : FM); ++i) acur[i] = abase[i] + sb;
#pragma unroll
    for (int j = 0; j < (BKC ? 2 * FN : FN); ++j) bcur[j] = bbase[j] + sb;
  };
  // A fragment is 16 bytes per lane: one read (K-contiguous), two transposing
  // halves (row-contiguous, 16 bit) or four single values (row-contiguous fp32).
  u32x4 qa[2][FM], qb[2][FN];
  u32x2 ha[2][2 * FM], hb[2][2 * FN];
  constexpr int kReadsA = AKC ? FM : (F32IN ? 4 * FM : 2 * FM);
  constexpr int kReadsB = BKC ? FN : (F32IN ? 4 * FN : 2 * FN);
  // LDS reads per set; the wait immediate is a 4-bit field, and with 16 reads
  // per set "at most 15 pending" still implies that the older set is complete.
  constexpr int kReads = kReadsA + kReadsB > 15 ? 15 : kReadsA + kReadsB;
  // Reads of the wave's sub-step J (0 or 1) of the stage set_stage() chose.
  auto issue_frags = [&](auto J) {
    constexpr int j = decltype(J)::value;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if constexpr (AKC) {
        qa[j][i] = b128_issue<0>(acur[2 * i + j]);
      } else if constexpr (F32IN) {
        qa[j][i][0] = b32_issue<(8 * j + 0) * 256 * FM>(acur[i]);
        qa[j][i][1] = b32_issue<(8 * j + 1) * 256 * FM>(acur[i]);
        qa[j][i][2] = b32_issue<(8 * j + 2) * 256 * FM>(acur[i]);
        qa[j][i][3] = b32_issue<(8 * j + 3) * 256 * FM>(acur[i]);
      } else {
        ha[j][2 * i] = tr_issue<j * 2048 * FM>(acur[i]);
        ha[j][2 * i + 1] = tr_issue<j * 2048 * FM + 512 * FM>(acur[i]);
      }
    }
#pragma unroll
    for (int jn = 0; jn < FN; ++jn) {
      if constexpr (BKC) {
        qb[j][jn] = b128_issue<0>(bcur[2 * jn + j]);
      } else if constexpr (F32IN) {
        qb[j][jn][0] = b32_issue<(8 * j + 0) * 256 * FN>(bcur[jn]);
        qb[j][jn][1] = b32_issue<(8 * j + 1) * 256 * FN>(bcur[jn]);
        qb[j][jn][2] = b32_issue<(8 * j + 2) * 256 * FN>(bcur[jn]);
        qb[j][jn][3] = b32_issue<(8 * j + 3) * 256 * FN>(bcur[jn]);
      } else {
        hb[j][2 * jn] = tr_issue<j * 2048 * FN>(bcur[jn]);
        hb[j][2 * jn + 1] = tr_issue<j * 2048 * FN + 512 * FN>(bcur[jn]);
      }
    }
  };
  // After the wait for set f: its registers may be used.
  auto claim_frags = [&](int f) {
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if constexpr (AKC || F32IN) {
        claim(qa[f][i]);
      } else {
        claim(ha[f][2 * i]);
        claim(ha[f][2 * i + 1]);
        qa[f][i] = __builtin_shufflevector(ha[f][2 * i], ha[f][2 * i + 1], 0, 1, 2, 3);
      }
    }
#pragma unroll
    for (int jn = 0; jn < FN; ++jn) {
      if constexpr (BKC || F32IN) {
        claim(qb[f][jn]);
      } else {
        claim(hb[f][2 * jn]);
        claim(hb[f][2 * jn + 1]);
        qb[f][jn] = __builtin_shufflevector(hb[f][2 * jn], hb[f][2 * jn + 1], 0, 1, 2, 3);
      }
    }
  };
  auto multiply = [&](int f) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int jn = 0; jn < FN; ++jn)
        acc[i][jn] = mma<T>(qa[f][i], qb[f][jn], acc[i][jn]);
  };
  const std::integral_constant<int, 0> J0;
  const std::integral_constant<int, 1> J1;

  // One K tile.  MORE: another tile follows; PEND: how many of the tiles kt + 2 .. kt + kStages - 2 exist
  // (their loads may stay pending); ISSUE: tile kt + kStages - 1 exists and is asked for now;
  // LAST: it is the last one and may be partly filled.
  auto k_tile = [&](int kt, auto MORE, auto PEND, auto ISSUE, auto LAST) {
    constexpr bool more = decltype(MORE)::value, t3 = decltype(ISSUE)::value;
    constexpr int pend = decltype(PEND)::value;
    constexpr bool last = decltype(LAST)::value;
    __builtin_amdgcn_sched_barrier(0);
    if (more) {
      // Tile kt + 1 is needed from here on (the refills below read it): its
      // loads have landed once only those of the tiles behind it are pending.  After
      // the barrier every wave's share is in LDS and every wave has finished
      // reading tile kt - 1, whose stage the loads of tile kt + kStages - 1 overwrite.
      wait_tiles(pend);
      __builtin_amdgcn_s_barrier();
      if (t3) {
        if (last && k_rem != 0) issue_last_tile((kt + kStages - 1) % kStages);
        else issue_tile((kt + kStages - 1) % kStages);
      }
      set_stage((kt + 1) % kStages);
    }
    // A set is complete once only the reads of the other one are pending.
    lgkm_wait<kReads>();
    claim_frags(0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(0);
    // fp32: an MFMA keeps the pipe for 64 cycles, so the refills of a set may go out between its MFMAs as their
    // registers fall free (the compiler places them; the order of the reads among themselves, which the
    // waits by count rely on, stays).  16 bit: the refills follow the set's MFMAs as a block.
    if constexpr (!F32IN) __builtin_amdgcn_sched_barrier(0);
    if (more) {
      issue_frags(J0);
      lgkm_wait<kReads>();
    } else {
      lgkm_wait<0>();
    }
    claim_frags(1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(1);
    if constexpr (!F32IN) __builtin_amdgcn_sched_barrier(0);
    if (more) issue_frags(J1);
  };

  // Tiles 0 .. kStages - 2 go out at once; tile kt + kStages - 1 follows at the barrier of K tile kt.
#pragma unroll
  for (int s = 0; s < kStages - 1; ++s)
    if (s < KT) {
      if (s == KT - 1 && k_rem != 0) issue_last_tile(s);
      else issue_tile(s);
    }
  wait_tiles(min(kStages - 2, KT - 1));
  __builtin_amdgcn_s_barrier();  // every wave's share of tile 0 is in LDS
  set_stage(0);
  issue_frags(J0);
  issue_frags(J1);
  {
    const std::true_type yes;
    const std::false_type no;
    int kt = 0;
    // Steady state: every tile up to kt + kStages exists.  Then the tile that asks for the last one, the
    // tiles that ask for nothing (one pending tile fewer each), and the last tile.
    for (; kt + kStages < KT; ++kt) k_tile(kt, yes, std::integral_constant<int, kStages - 3>{}, yes, no);
    if (kt + kStages - 1 < KT) k_tile(kt++, yes, std::integral_constant<int, kStages - 3>{}, yes, yes);
    tail_tiles<kStages - 2>([&](auto R) {  // R tiles follow this one
      constexpr int r = decltype(R)::value;
      if (kt + r < KT) k_tile(kt++, yes, std::integral_constant<int, r - 1>{}, no, no);
    });
    k_tile(kt, no, std::integral_constant<int, 0>{}, no, no);
  }

  {
    // Waves 4 .. 7 hand their sums to the wave of the same quadrant: value
    // (tile, element) of lane l at float (tile * 16 + element) * 64 + l of the
    // quadrant's region (conflict-free), inside the stages, which nobody reads
    // any more after the barrier.
    float* xch = reinterpret_cast<float*>(lds) + quad * (FM * FN * 16 * 64);
    static_assert(4 * FM * FN * 16 * 64 * 4 <= 2 * G::kStageBytes, "exchange must fit two stages");
    __builtin_amdgcn_s_barrier();
    if (kgroup == 1) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int jn = 0; jn < FN; ++jn)
#pragma unroll
          for (int e = 0; e < 16; ++e) xch[((i * FN + jn) * 16 + e) * 64 + lane] = acc[i][jn][e];
    }
    __syncthreads();
    if (kgroup == 1) return;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int jn = 0; jn < FN; ++jn)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][jn][e] += xch[((i * FN + jn) * 16 + e) * 64 + lane];
  }

  // ------------------------------------------------------------------ epilogue
  // Accumulator element e of tile (i, j): row 8 (e / 4) + 4 (lane / 32) + e % 4,
  // column lane % 32.
  const int l32 = lane & 31, lhi = lane >> 5;
  if (EPI == kPartial) {
    float* out = p.partial + (size_t)split * p.m * p.n;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const f32x4 v = {acc[i][j][4 * b], acc[i][j][4 * b + 1], acc[i][j][4 * b + 2], acc[i][j][4 * b + 3]};
          const size_t col = n0 + wn + j * 32 + l32;
          const size_t row = m0 + wm + i * 32 + 8 * b + 4 * lhi;
          if (col < (size_t)p.n && row < (size_t)p.m) *reinterpret_cast<f32x4*>(out + col * p.m + row) = v;
        }
    return;
  }

  if constexpr (F32IN) {
    // fp32 output: a lane holds 4 consecutive rows of a column, stored as one
    // 16-byte vector straight from the accumulators.
    float* C = static_cast<float*>(p.C) + bz * p.sc;
    float* P = p.pre ? static_cast<float*>(p.pre) + bz * p.sc : nullptr;
    const float* bias = static_cast<const float*>(p.bias);
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          f32x4 v = {acc[i][j][4 * b], acc[i][j][4 * b + 1], acc[i][j][4 * b + 2], acc[i][j][4 * b + 3]};
          const size_t col = n0 + wn + j * 32 + l32;
          const size_t row = m0 + wm + i * 32 + 8 * b + 4 * lhi;
          if (col >= (size_t)p.n || row >= (size_t)p.m) continue;
          const size_t off = col * p.ldc + row;
          if (EPI == kGeneral) {
            if (p.beta != 0.f) v += p.beta * *reinterpret_cast<const f32x4*>((P ? P : C) + off);
            if (bias) v += *reinterpret_cast<const f32x4*>(bias + row);
            if (P) *reinterpret_cast<f32x4*>(P + off) = v;
            if (p.act != GINN_HIP_ACT_IDENTITY) {
              float w[4] = {v[0], v[1], v[2], v[3]};
              act_forward_n<kFastMath<T>, 4>(p.act, w);
              v = f32x4{w[0], w[1], w[2], w[3]};
            }
          }
          *reinterpret_cast<f32x4*>(C + off) = v;
        }
  } else {
  // The stages are reused for staging: wait until every wave is past its last
  // fragment read.
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  uint16_t* C = static_cast<uint16_t*>(p.C) + bz * p.sc;
  char* stage = lds + wave * G::kEpiWaveBytes;
  // a column of the wave's tile is 32 FM rows = 4 FM chunks of 8 rows
  constexpr int kRowChunks = 4 * FM;
  constexpr int kColsPerIter = 64 / kRowChunks;
  const int sub = lane / kRowChunks, chunk = lane % kRowChunks;
  // A bias alone (no old C, no activation, no kept pre-activation) is added to the accumulators where they
  // are -- a lane holds four consecutive rows per group -- and the tile leaves through the plain path: the
  // same single rounding of acc + bias without the fp32 staging of the general path.
  const bool bias_only = EPI == kGeneral && p.beta == 0.f && p.act == GINN_HIP_ACT_IDENTITY && p.pre == nullptr;
  if (bias_only && p.bias) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int r = m0 + wm + i * 32 + 8 * b + 4 * lhi;
        u16x4 bv = {0, 0, 0, 0};
        if (r < p.m) bv = *reinterpret_cast<const u16x4*>(static_cast<const uint16_t*>(p.bias) + r);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float add = to_float<T>(bv[e]);
#pragma unroll
          for (int j = 0; j < FN; ++j) acc[i][j][4 * b + e] += add;
        }
      }
  }
  if (EPI == kPlain || bias_only) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          u16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = from_float<T>(acc[i][j][4 * b + e]);
          *reinterpret_cast<u16x4*>(stage + (j * 32 + l32) * G::kEpiColStride + (i * 32 + 8 * b + 4 * lhi) * 2) = o;
        }
    // each wave reads back only what it wrote itself
#pragma unroll
    for (int it = 0; it < 32 * FN / kColsPerIter; ++it) {
      const int col = it * kColsPerIter + sub;
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + col * G::kEpiColStride + chunk * 16);
      if (n0 + wn + col < p.n && m0 + wm + chunk * 8 < p.m)
        *reinterpret_cast<u32x4*>(C + (long long)(n0 + wn + col) * p.ldc + m0 + wm + chunk * 8) = v;
    }
  } else {
    // General epilogue: C = act(acc + beta * C + bias), optionally keeping the
    // pre-activation; fp32 staging in passes of 32 columns, every value
    // rounded once.
    uint16_t* P = p.pre ? static_cast<uint16_t*>(p.pre) + bz * p.sc : nullptr;
    const int row = m0 + wm + chunk * 8;
    const bool row_ok = row < p.m;  // m is a multiple of 8: a chunk of rows is inside or outside
    float bias8[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) bias8[e] = 0.f;
    if (p.bias && row_ok) {
      const u16x8 bv = *reinterpret_cast<const u16x8*>(static_cast<const uint16_t*>(p.bias) + row);
#pragma unroll
      for (int e = 0; e < 8; ++e) bias8[e] = to_float<T>(bv[e]);
    }
#pragma unroll
    for (int pass = 0; pass < FN; ++pass) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const f32x4 v = {acc[i][pass][4 * b], acc[i][pass][4 * b + 1], acc[i][pass][4 * b + 2],
                           acc[i][pass][4 * b + 3]};
          *reinterpret_cast<f32x4*>(stage + l32 * G::kF32ColStride + (i * 32 + 8 * b + 4 * lhi) * 4) = v;
        }
      // All reads of the old C of the pass are issued before the first is
      // used, and the activation is a compile-time constant inside the loop.
      constexpr int kIters = 32 / kColsPerIter;
      const uint16_t* Cin = P ? P : C;
      u16x8 old[kIters];
      if (p.beta != 0.f) {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
          const int col = n0 + wn + pass * 32 + it * kColsPerIter + sub;
          old[it] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
          if (col < p.n && row_ok) old[it] = *reinterpret_cast<const u16x8*>(Cin + (long long)col * p.ldc + row);
        }
      }
      GH_SWITCH_ACT(p.act, {
        _Pragma("unroll") for (int it = 0; it < kIters; ++it) {
          const int lcol = it * kColsPerIter + sub;
          const char* src = stage + lcol * G::kF32ColStride + chunk * 32;
          const f32x4 lo = *reinterpret_cast<const f32x4*>(src);
          const f32x4 hi = *reinterpret_cast<const f32x4*>(src + 16);
          float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          if (n0 + wn + pass * 32 + lcol < p.n && row_ok) {
            const long long off = (long long)(n0 + wn + pass * 32 + lcol) * p.ldc + row;
            if (p.beta != 0.f) {
              _Pragma("unroll") for (int e = 0; e < 8; ++e) v[e] += p.beta * to_float<T>(old[it][e]);
            }
            _Pragma("unroll") for (int e = 0; e < 8; ++e) v[e] += bias8[e];
            u16x8 o;
            if (P) {
              _Pragma("unroll") for (int e = 0; e < 8; ++e) o[e] = from_float<T>(v[e]);
              *reinterpret_cast<u16x8*>(P + off) = o;
            }
            _Pragma("unroll") for (int e = 0; e < 8; ++e) o[e] = from_float<T>(act_forward_c<kFastMath<T>, ACT>(v[e]));
            *reinterpret_cast<u16x8*>(C + off) = o;
          }
        }
      })
      // the next pass overwrites what this one's readers are using: a wave
      // only touches its own slice, so waiting for its own reads is enough
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
  }

  }
}

template <typename T, bool AKC, bool BKC, int FM, int FN>
int launch_epi(ginn_hip_ctx* ctx, const MidParams& p, int batch, int splits, int epi) {
  using G = Geo<FM, FN>;
  const dim3 grid(p.tiles_m * p.tiles_n, batch, splits);
  // Only the stages a short K loop touches are allocated (at least two: the
  // epilogue staging lives there), so that more workgroups fit on a CU then.
  const int stages = p.k_tiles < 2 ? 2 : (p.k_tiles < G::kStages ? p.k_tiles : G::kStages);
  const int lds_bytes = stages * G::kStageBytes;
#define GH_MID_LAUNCH(E)                                                                          \
  {                                                                                               \
    auto fn = gemm_mid_kernel<T, AKC, BKC, E, FM, FN>;                                          \
    static std::atomic<unsigned long long> lds_allowed{0};                                        \
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn),         \
                             G::kLdsBytes));                                                      \
    fn<<<grid, dim3(kThreads), lds_bytes, ctx->stream>>>(p);                                      \
  }
  if (epi == kPartial) GH_MID_LAUNCH(kPartial)
  else if (epi == kGeneral) GH_MID_LAUNCH(kGeneral)
  else GH_MID_LAUNCH(kPlain)
#undef GH_MID_LAUNCH
  GH_HIP(hipGetLastError());
  return kOk;
}

// One (FM, FN) shape: three scalar types, four layouts, three epilogues.
template <int FM, int FN>
int launch_shape(ginn_hip_ctx* ctx, const MidParams& p, int dtype, int batch, int splits, int epi, bool akc,
                 bool bkc) {
#define GH_MID_LAYOUT(T)                                                                          \
  if (akc) {                                                                                      \
    if (bkc) return launch_epi<T, true, true, FM, FN>(ctx, p, batch, splits, epi);                \
    return launch_epi<T, true, false, FM, FN>(ctx, p, batch, splits, epi);                        \
  }                                                                                               \
  if (bkc) return launch_epi<T, false, true, FM, FN>(ctx, p, batch, splits, epi);                 \
  return launch_epi<T, false, false, FM, FN>(ctx, p, batch, splits, epi);
  if (dtype == GINN_HIP_F16) {
    GH_MID_LAYOUT(F16)
  }
  if (dtype == GINN_HIP_F32) {
    GH_MID_LAYOUT(F32)
  }
  GH_MID_LAYOUT(BF16)
#undef GH_MID_LAYOUT
}

// Each shape is instantiated in its own translation unit.
extern template int launch_shape<2, 2>(ginn_hip_ctx*, const MidParams&, int, int, int, int, bool, bool);
extern template int launch_shape<2, 1>(ginn_hip_ctx*, const MidParams&, int, int, int, int, bool, bool);
extern template int launch_shape<1, 2>(ginn_hip_ctx*, const MidParams&, int, int, int, int, bool, bool);
extern template int launch_shape<1, 1>(ginn_hip_ctx*, const MidParams&, int, int, int, int, bool, bool);

}  // namespace mid
}  // namespace ginn_hip

#endif  // GINN_HIP_GEMM_MID_H
