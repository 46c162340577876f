// Tuned fp16 / bf16 (fp32-accumulate) product for large aligned shapes.
//
// Block tile 256 x 256 x 64, 256 threads = 4 waves (one per SIMD), each wave
// owns a 128 x 128 output tile = 4 x 4 MFMA 32x32x16 tiles (256 accumulator
// registers).  Two 64 KiB LDS stages; operands go global -> LDS directly
// (global_load_lds, 16 bytes per lane) so that no registers are spent on
// staging.  Each wave software-pipelines its own work in a pinned order:
// under the 16 MFMAs of a K sub-step it issues the LDS fragment reads of the
// next sub-step, and -- after the single barrier of the K-step -- the global
// loads of the tile two steps ahead, one every other MFMA, so that the
// texture addresser sees an even stream instead of bursts.
//
// LDS layouts (both unpadded; conflicts are avoided by XOR-ing the 16-byte
// chunk position, applied on the global side of the direct loads):
//   K-contiguous operand ("KC": A^T, or B):  [256 rows][8 chunks]; chunk
//     position = chunk ^ ((row >> 1) & 7); a lane's MFMA operand (8 k of one
//     row) is one ds_read_b128.
//   row-contiguous operand ("RC": A, or B^T): [64 k][32 chunks]; chunk
//     position = chunk ^ (4 * (k & 3)); a lane's operand is two
//     ds_read_b64_tr_b16 (the 16-lane transposing read of gfx950).  A
//     transposing read serves 32 lanes per cycle = two 16-lane groups x 4
//     k-rows x 32 bytes; the k-rows lie 512 bytes apart (the same banks), and
//     the XOR moves row i by 64 i bytes, so the four rows' 64 bytes fall into
//     four different quarters of the 64 banks.
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "common.h"

namespace ginn_hip {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Sixteen zero bytes in device memory: where a direct load must deliver zeros (K values beyond the end of
// a ragged K) its lane reads them from here instead of the operand.
__device__ __attribute__((aligned(16))) const unsigned int kZeroChunk[4] = {0u, 0u, 0u, 0u};

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = 256 * BK * 2;       // one operand, one stage: 32 KiB
constexpr int kStageBytes = 2 * kTileBytes;    // A + B
// Epilogue staging: per wave 128 columns of 128 halfs, column stride 272 B
// (16-byte aligned, spreads the 32 column-lanes over the banks).
constexpr int kEpiColStride = 272;
constexpr int kEpiWaveBytes = 128 * kEpiColStride;
constexpr int kLdsBytes = 4 * kEpiWaveBytes;   // 139264 >= 2 * kStageBytes
static_assert(kLdsBytes >= 2 * kStageBytes, "epilogue staging must cover the pipeline stages");

struct FastParams {
  const uint16_t* A;
  const uint16_t* B;
  uint16_t* C;
  int m, n, k;
  int lda, ldb, ldc;
  long long sa, sb, sc;
  float beta;
  const uint16_t* bias;
  uint16_t* pre;
  int act;
  int tiles_m, tiles_n;
  int group;  // tile rows walked together (0: plain column-major tile order)
};

__device__ __forceinline__ int swz_kc(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz_rc(int kr) { return 4 * (kr & 3); }

// Element offset, relative to the tile origin at K offset 0, of the 16-byte
// chunk that lands at linear LDS chunk position v of the tile.
// Tile rows from `valid` on (a tile that reaches beyond the matrix) re-read a
// row inside it -- K-contiguous operand: the last valid row; row-contiguous
// operand: the 16 bytes at the tile's first row (extents along the rows are
// multiples of 8) -- in bounds, and what they produce is never stored.
template <bool KC>
__device__ __forceinline__ long long chunk_src(int v, int ld, int valid) {
  if (KC) {
    const int row = v >> 3, pc = v & 7;
    return (long long)min(row, valid - 1) * ld + ((pc ^ swz_kc(row)) * 8);
  }
  const int kr = v >> 5, pj = v & 31;
  const int row0 = (pj ^ swz_rc(kr)) * 8;
  return (long long)kr * ld + (row0 < valid ? row0 : 0);
}

// Byte offset inside a K-contiguous tile of lane's 16 bytes of the fragment
// rows r0 .. r0+31, sub-step ks (16 k values).  Fragment r0 + 32 r lies
// 4096 r bytes further (the swizzle involves row bits 1 .. 3 only).
__device__ __forceinline__ int kc_offset(int r0, int ks, int lane) {
  const int row = r0 + (lane & 31);
  const int c = 2 * ks + (lane >> 5);
  return row * 128 + ((c ^ swz_kc(row)) * 16);
}

// Byte offset inside a row-contiguous tile of half t (k + 4t .. k + 4t + 3)
// of the transposed fragment.  A 16-lane group reads 4 k-rows x 32 bytes and
// every lane receives 4 k values of its own row.  Sub-step ks, half t lie
// 8192 ks + 2048 t bytes behind (ks, t) = (0, 0): the swizzle involves k bits
// 0, 1 only, which come from the lane.
__device__ __forceinline__ int tr_offset(int r0, int ks, int t, int lane) {
  const int g = lane >> 4, s = lane & 15, h = g & 1, q = g >> 1;
  const int mcol = r0 + 16 * h + 4 * (s & 3);
  const int j = mcol >> 3, within = (mcol & 7) * 2;
  const int kr = 16 * ks + 8 * q + 4 * t + (s >> 2);
  return kr * 512 + ((j ^ swz_rc(kr)) * 16) + within;
}

// LDS fragment reads through inline assembly, address = per-lane base +
// immediate offset.  The compiler neither sees an LDS access here (it would
// otherwise place a full vmcnt(0) wait in front of it because of the in-flight
// global -> LDS loads) nor tracks its completion: settle() must run before
// the values are used.
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
// Waits for all outstanding LDS operations; the registers are in/out operands
// so that none of their uses can be scheduled above the wait.
__device__ __forceinline__ void settle(u32x2 (&h)[8]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(h[0]), "+v"(h[1]), "+v"(h[2]), "+v"(h[3]), "+v"(h[4]), "+v"(h[5]),
                 "+v"(h[6]), "+v"(h[7])
               :
               : "memory");
}
__device__ __forceinline__ void settle(u32x4 (&q)[4]) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]) : : "memory");
}

template <bool BF>
__device__ __forceinline__ f32x16 mma(u16x8 a, u16x8 b, f32x16 c) {
  if (BF)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order.
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// EPI: 0 = plain store (beta == 0, no bias / activation / pre-activation), staged through LDS for
// full-line stores; 1 = general epilogue; 2 = a bias alone: added to the accumulators where they are (a lane
// holds four consecutive rows per group), then the plain store -- the same single rounding of acc + bias
// as the general path, without its fp32 staging.  An instantiation of its own: as a run-time branch
// inside the general one it made that kernel spill.
template <typename T, bool AKC, bool BKC, int EPI>
__global__ __launch_bounds__(kThreads) void gemm_fast16_kernel(FastParams p) {
  constexpr bool BF = std::is_same<T, BF16>::value;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave & 1) * 128, wn = (wave >> 1) * 128;

  // Workgroup ids are dealt round-robin to the 8 XCDs, each with a private L2:
  // give every XCD a contiguous range of the tile sequence, and order that
  // sequence in column panels of `group` tile rows so that the tiles running
  // together on one XCD share A rows and B columns.
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
  const int m0 = (pid % p.tiles_m) * BM, n0 = (pid / p.tiles_m) * BN;
  const long long bz = blockIdx.y;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int KT = (p.k + BK - 1) / BK;
  // K values in the last K tile (64 unless K is no multiple of the tile): lanes
  // whose 16 bytes of that tile lie beyond them load zeros instead.
  const int k_lim = p.k - (KT - 1) * BK;
  const int m_valid = min(BM, p.m - m0), n_valid = min(BN, p.n - n0);

  // Thread `tid` moves chunk v = i * 256 + tid (i = 0..7) of each operand; the
  // lane-dependent part of the source offset does not depend on i because the
  // swizzle only involves row bits below 32 (KC) / k bits below 8 (RC).  A
  // load takes a scalar tile origin plus a 32-bit per-thread offset.
  const long long a_kstep = (AKC ? (long long)BK : (long long)BK * p.lda) * 2;
  const long long b_kstep = (BKC ? (long long)BK : (long long)BK * p.ldb) * 2;
  uint32_t a_off[8], b_off[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a_off[i] = (uint32_t)(chunk_src<AKC>(i * kThreads + tid, p.lda, m_valid) * 2);
    b_off[i] = (uint32_t)(chunk_src<BKC>(i * kThreads + tid, p.ldb, n_valid) * 2);
  }
  // The chunk along K that this thread moves of a K-contiguous tile (the same in
  // every pass) holds K values of the last tile; k-row of pass 0 of a
  // row-contiguous tile (pass i: 8 i further).
  const bool kc_ok = (((tid & 7) ^ swz_kc(tid >> 3)) * 8) < k_lim;
  const int rc_kr = tid >> 5;
  const char* a_tile = reinterpret_cast<const char*>(p.A + bz * p.sa) +
                       (AKC ? (long long)m0 * p.lda : (long long)m0) * 2;
  const char* b_tile = reinterpret_cast<const char*>(p.B + bz * p.sb) +
                       (BKC ? (long long)n0 * p.ldb : (long long)n0) * 2;

  // Direct load number q (0..15) into stage buf of the tile whose origins are
  // ga / gb: even q = A chunk q / 2, odd q = B chunk q / 2.  The LDS address is
  // wave-uniform; lane l lands 16 * l bytes behind it.
  auto issue_q = [&](const char* ga, const char* gb, int buf, int q) {
    const int i = q >> 1;
    char* l = lds + buf * kStageBytes + ((q & 1) ? kTileBytes : 0);
    uint32_t& off = (q & 1) ? b_off[i] : a_off[i];
    asm volatile("" : "+v"(off));  // keeps (scalar origin) + (32-bit offset) apart for the addressing mode
    const char* g = ((q & 1) ? gb : ga) + off;
    const int vbase = i * kThreads + wave * 64;
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)g,
                                     (void __attribute__((address_space(3)))*)(l + vbase * 16), 16,
                                     0, 0);
  };

  // The same for the last K tile, which K may fill only in part: a per-lane
  // address, the lanes beyond K read zeros.
  auto issue_q_last = [&](const char* ga, const char* gb, int buf, int q) {
    const int i = q >> 1;
    char* l = lds + buf * kStageBytes + ((q & 1) ? kTileBytes : 0);
    const bool kc = (q & 1) ? BKC : AKC;
    const bool ok = kc ? kc_ok : (8 * i + rc_kr) < k_lim;
    const char* g = ((q & 1) ? gb : ga) + ((q & 1) ? b_off[i] : a_off[i]);
    if (!ok) g = reinterpret_cast<const char*>(kZeroChunk);
    const int vbase = i * kThreads + wave * 64;
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)g,
                                     (void __attribute__((address_space(3)))*)(l + vbase * 16), 16,
                                     0, 0);
  };

  // Fragment sets: one in use, one being filled.  A K-contiguous fragment is
  // one 16-byte read (a base per sub-step, 4096 bytes per fragment), a
  // row-contiguous one two transposing 8-byte reads (a base per fragment,
  // 8192 bytes per sub-step, 2048 per half).
  u32x4 qa[2][4], qb[2][4];
  u32x2 ha[2][8], hb[2][8];
  uint32_t acur[4], bcur[4];  // bases inside the stage being read
  {
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      acur[x] = lds_base + (AKC ? kc_offset(wm, x, lane) : tr_offset(wm + x * 32, 0, 0, lane));
      bcur[x] = lds_base + kTileBytes + (BKC ? kc_offset(wn, x, lane) : tr_offset(wn + x * 32, 0, 0, lane));
    }
  }
  // Moves the bases to the other stage (delta = +- kStageBytes).
  auto switch_stage = [&](int delta) {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      acur[x] += delta;
      bcur[x] += delta;
    }
  };

  // Fragment read R (0..3: A fragment R, 4..7: B fragment R - 4) of sub-step
  // KS of the current stage into set f.
  auto read_one = [&](auto KS, int f, auto R) {
    constexpr int ks = decltype(KS)::value, r = decltype(R)::value;
    if constexpr (r < 4) {
      if constexpr (AKC) {
        qa[f][r] = b128_issue<r * 4096>(acur[ks]);
      } else {
        ha[f][2 * r] = tr_issue<ks * 8192>(acur[r]);
        ha[f][2 * r + 1] = tr_issue<ks * 8192 + 2048>(acur[r]);
      }
    } else {
      constexpr int rb = r - 4;
      if constexpr (BKC) {
        qb[f][rb] = b128_issue<rb * 4096>(bcur[ks]);
      } else {
        hb[f][2 * rb] = tr_issue<ks * 8192>(bcur[rb]);
        hb[f][2 * rb + 1] = tr_issue<ks * 8192 + 2048>(bcur[rb]);
      }
    }
  };
  // Completes the reads of set f and assembles the 128-bit operands.
  auto finish = [&](int f) {
    if (AKC) {
      settle(qa[f]);
    } else {
      settle(ha[f]);
#pragma unroll
      for (int i = 0; i < 4; ++i) qa[f][i] = __builtin_shufflevector(ha[f][2 * i], ha[f][2 * i + 1], 0, 1, 2, 3);
    }
    if (BKC) {
      settle(qb[f]);
    } else {
      settle(hb[f]);
#pragma unroll
      for (int j = 0; j < 4; ++j) qb[f][j] = __builtin_shufflevector(hb[f][2 * j], hb[f][2 * j + 1], 0, 1, 2, 3);
    }
  };

  // One sub-step in pinned order: 16 MFMAs on fragment set f; between them the
  // 8 fragment reads of sub-step KS of the current stage (RD) and 8 direct
  // loads of the tile at ga / gb (LD), the latter after every other MFMA.
  // LAST: the tile loaded is the last one (loads by per-lane address).
  auto substep = [&](int f, auto rd_c, auto KS, auto ld_c, auto last_c, const char* ga, const char* gb, int lbuf,
                     int lq0) {
    constexpr bool RD = decltype(rd_c)::value;
    constexpr bool LD = decltype(ld_c)::value;
    constexpr bool LAST = decltype(last_c)::value;
    static_for<16>([&](auto IDX) {
      constexpr int idx = decltype(IDX)::value;
      constexpr int i = idx >> 2, j = idx & 3;
      acc[i][j] = mma<BF>(__builtin_bit_cast(u16x8, qa[f][i]), __builtin_bit_cast(u16x8, qb[f][j]), acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (LD && (idx & 1) == 0) {
        if constexpr (LAST) issue_q_last(ga, gb, lbuf, (idx >> 1) + lq0);
        else issue_q(ga, gb, lbuf, (idx >> 1) + lq0);
      }
      // B fragments first: the next sub-step's first four MFMAs need all of them.
      if constexpr (RD && idx < 8) read_one(KS, f ^ 1, std::integral_constant<int, (idx < 4 ? idx + 4 : idx - 4)>{});
      __builtin_amdgcn_sched_barrier(0);
    });
    if (RD) finish(f ^ 1);
    __builtin_amdgcn_sched_barrier(0);
  };

  // Origins of tile kt + 1 while K-step kt runs.
  const char* a_nx = a_tile + a_kstep;
  const char* b_nx = b_tile + b_kstep;
  const std::integral_constant<int, 0> K0;
  const std::integral_constant<int, 1> K1;
  const std::integral_constant<int, 2> K2;
  const std::integral_constant<int, 3> K3;

  // One K-step.  HEAD: the second half of tile kt+1's loads is still to be
  // issued (first sub-step); NEXT: tile kt+1 exists; TAIL: tile kt+2 exists
  // (first half of its loads goes into the stage released by the barrier).
  // Compile-time flags keep every sub-step one basic block.
  // HLAST / TLAST: the tile that HEAD / TAIL loads is the product's last one.
  auto kstep = [&](int kt, auto head_c, auto next_c, auto tail_c, auto hlast_c, auto tlast_c) {
    constexpr bool HEAD = decltype(head_c)::value;
    constexpr bool NEXT = decltype(next_c)::value;
    constexpr bool TAIL = decltype(tail_c)::value;
    const int buf = kt & 1;
    // The tile origins stay whole scalar values (not re-derived from kt and
    // folded into the per-lane address arithmetic).
    const char* a_n2 = a_nx + a_kstep;
    const char* b_n2 = b_nx + b_kstep;
    asm volatile("" : "+s"(a_nx), "+s"(b_nx), "+s"(a_n2), "+s"(b_n2));
    substep(0, std::true_type{}, K1, std::integral_constant<bool, HEAD>{}, hlast_c, a_nx, b_nx, buf ^ 1, 8);
    substep(1, std::true_type{}, K2, std::false_type{}, std::false_type{}, nullptr, nullptr, 0, 0);
    substep(0, std::true_type{}, K3, std::false_type{}, std::false_type{}, nullptr, nullptr, 0, 0);
    // Every fragment read of tile kt has completed (finish); tile kt+1 must
    // have landed before anyone reads it, and the stage of tile kt is free
    // once all waves are here.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (NEXT) switch_stage(buf ? -kStageBytes : kStageBytes);
    substep(1, std::integral_constant<bool, NEXT>{}, K0, std::integral_constant<bool, TAIL>{}, tlast_c, a_n2, b_n2, buf,
            0);
    a_nx = a_n2;
    b_nx = b_n2;
  };

  // Prologue: tiles 0 and 1 in full, first fragments of tile 0.
  if (KT == 1) {
#pragma unroll
    for (int q = 0; q < 16; ++q) issue_q_last(a_tile, b_tile, 0, q);
  } else {
#pragma unroll
    for (int q = 0; q < 16; ++q) issue_q(a_tile, b_tile, 0, q);
    if (KT == 2) {
#pragma unroll
      for (int q = 0; q < 16; ++q) issue_q_last(a_nx, b_nx, 1, q);
    } else {
#pragma unroll
      for (int q = 0; q < 16; ++q) issue_q(a_nx, b_nx, 1, q);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  static_for<8>([&](auto R) { read_one(K0, 0, R); });
  finish(0);
  __builtin_amdgcn_sched_barrier(0);

  using Y = std::true_type;
  using N = std::false_type;
  // Tile t is loaded by the TAIL of K-step t - 2 and the HEAD of K-step t - 1:
  // the last tile by K-steps KT - 3 and KT - 2, which are peeled for it.
  if (KT == 1) {
    kstep(0, N{}, N{}, N{}, N{}, N{});
  } else if (KT == 2) {
    kstep(0, N{}, Y{}, N{}, N{}, N{});
    kstep(1, N{}, N{}, N{}, N{}, N{});
  } else {
    int kt = 1;
    if (KT == 3) {
      kstep(0, N{}, Y{}, Y{}, N{}, Y{});
    } else {
      kstep(0, N{}, Y{}, Y{}, N{}, N{});
      for (; kt + 3 < KT; ++kt) kstep(kt, Y{}, Y{}, Y{}, N{}, N{});
      kstep(kt++, Y{}, Y{}, Y{}, N{}, Y{});
    }
    kstep(kt, Y{}, Y{}, N{}, Y{}, N{});
    kstep(kt + 1, N{}, N{}, N{}, N{}, N{});
  }

  // ------------------------------------------------------------------ epilogue
  // Accumulator element e of tile (i, j): row 8 (e / 4) + 4 (lane / 32) + e % 4,
  // column lane % 32.
  const int l32 = lane & 31, lhi = lane >> 5;
  uint16_t* C = p.C + bz * p.sc;
  if constexpr (EPI == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int r = wm + i * 32 + 8 * b + 4 * lhi;
        u16x4 bv = {0, 0, 0, 0};
        if (r < m_valid) bv = *reinterpret_cast<const u16x4*>(p.bias + m0 + r);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float add = to_float<T>(bv[e]);
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j][4 * b + e] += add;
        }
      }
  }
  if constexpr (EPI != 1) {
    // All LDS reads and direct loads of every wave ended before the last
    // barrier, so each wave may overwrite its own slice right away: write the
    // rounded tile column-major, read it back 16 bytes per lane, store full
    // 256-byte column segments.
    char* stage = lds + wave * kEpiWaveBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          u16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = from_float<T>(acc[i][j][4 * b + e]);
          *reinterpret_cast<u16x4*>(stage + (j * 32 + l32) * kEpiColStride +
                                    (i * 32 + 8 * b + 4 * lhi) * 2) = o;
        }
    const int sub = lane >> 4, chunk = lane & 15;
#pragma unroll 4
    for (int it = 0; it < 32; ++it) {
      const int col = it * 4 + sub;
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + col * kEpiColStride + chunk * 16);
      if (wn + col < n_valid && wm + chunk * 8 < m_valid)
        *reinterpret_cast<u32x4*>(C + (long long)(n0 + wn + col) * p.ldc + m0 + wm + chunk * 8) = v;
    }
  } else {
    // General epilogue: C = act(acc + beta * C + bias), optionally keeping the
    // pre-activation.  The fp32 tile is staged through the wave's LDS slice in
    // two passes of 64 columns so that C, bias and pre move as 16-byte vectors
    // of 8 consecutive rows and every value is rounded exactly once.
    uint16_t* P = p.pre ? p.pre + bz * p.sc : nullptr;
    char* stage = lds + wave * kEpiWaveBytes;
    constexpr int kF32ColStride = 128 * 4 + 16;
    static_assert(64 * kF32ColStride <= kEpiWaveBytes, "fp32 staging must fit the wave slice");
    const int sub = lane >> 4, chunk = lane & 15;
    auto write_pass = [&](auto pass_c) {
      constexpr int PASS = decltype(pass_c)::value;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const f32x4 v = {acc[i][2 * PASS + jj][4 * b], acc[i][2 * PASS + jj][4 * b + 1],
                             acc[i][2 * PASS + jj][4 * b + 2], acc[i][2 * PASS + jj][4 * b + 3]};
            *reinterpret_cast<f32x4*>(stage + (jj * 32 + l32) * kF32ColStride +
                                      (i * 32 + 8 * b + 4 * lhi) * 4) = v;
          }
    };
    auto read_pass = [&](int pass) {
      const int row = m0 + wm + chunk * 8;
      const bool row_ok = wm + chunk * 8 < m_valid;  // m is a multiple of 8: a chunk of rows is inside or outside
      float bias8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) bias8[e] = 0.f;
      if (p.bias && row_ok) {
        const u16x8 bv = *reinterpret_cast<const u16x8*>(p.bias + row);
#pragma unroll
        for (int e = 0; e < 8; ++e) bias8[e] = to_float<T>(bv[e]);
      }
      typedef float f32x4 __attribute__((ext_vector_type(4)));
      const uint16_t* Cin = P ? P : C;
      // One column of the pass: 8 rows per lane from the staged fp32 tile.
      auto finish = [&](int lcol, bool with_old, const u16x8& old) {
        if (!row_ok || wn + pass * 64 + lcol >= n_valid) return;
        const char* src = stage + lcol * kF32ColStride + chunk * 32;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(src);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(src + 16);
        float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const long long off = (long long)(n0 + wn + pass * 64 + lcol) * p.ldc + row;
        if (with_old) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += p.beta * to_float<T>(old[e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += bias8[e];
        u16x8 o;
        if (P) {
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = from_float<T>(v[e]);
          *reinterpret_cast<u16x8*>(P + off) = o;
        }
        if (p.act != GINN_HIP_ACT_IDENTITY) act_forward_n<kFastMath<T>, 8>(p.act, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = from_float<T>(v[e]);
        *reinterpret_cast<u16x8*>(C + off) = o;
      };
      if (p.beta != 0.f) {
        // Accumulating: the reads of the old C of eight columns are issued
        // before the first is used.  One at a time, each of the 32 steps of a
        // tile waited for memory with nothing else to run on the CU, and an
        // accumulating product cost 64 % more than a plain one on a short K.
        constexpr int kBatch = 8;
#pragma unroll 1
        for (int it0 = 0; it0 < 16; it0 += kBatch) {
          u16x8 old[kBatch];
#pragma unroll
          for (int u = 0; u < kBatch; ++u) {
            const int lcol = (it0 + u) * 4 + sub;  // column inside the pass
            old[u] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (row_ok && wn + pass * 64 + lcol < n_valid)
              old[u] = *reinterpret_cast<const u16x8*>(Cin + (long long)(n0 + wn + pass * 64 + lcol) * p.ldc + row);
          }
#pragma unroll
          for (int u = 0; u < kBatch; ++u) finish((it0 + u) * 4 + sub, true, old[u]);
        }
      } else {
        const u16x8 none = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
        for (int it = 0; it < 16; ++it) finish(it * 4 + sub, false, none);
      }
    };
    write_pass(std::integral_constant<int, 0>{});
    read_pass(0);
    write_pass(std::integral_constant<int, 1>{});
    read_pass(1);
  }
}

template <typename T, bool AKC, bool BKC>
int launch_epi(ginn_hip_ctx* ctx, const FastParams& p, int batch, int general) {
  const dim3 grid(p.tiles_m * p.tiles_n, batch);
  if (general == 2) {
    auto fn = gemm_fast16_kernel<T, AKC, BKC, 2>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), kLdsBytes));
    fn<<<grid, dim3(kThreads), kLdsBytes, ctx->stream>>>(p);
  } else if (general == 1) {
    auto fn = gemm_fast16_kernel<T, AKC, BKC, 1>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), kLdsBytes));
    fn<<<grid, dim3(kThreads), kLdsBytes, ctx->stream>>>(p);
  } else {
    auto fn = gemm_fast16_kernel<T, AKC, BKC, 0>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), kLdsBytes));
    fn<<<grid, dim3(kThreads), kLdsBytes, ctx->stream>>>(p);
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

template <typename T>
int launch_layout(ginn_hip_ctx* ctx, const FastParams& p, int batch, bool akc, bool bkc, int general) {
  if (akc) {
    if (bkc) return launch_epi<T, true, true>(ctx, p, batch, general);
    return launch_epi<T, true, false>(ctx, p, batch, general);
  }
  if (bkc) return launch_epi<T, false, true>(ctx, p, batch, general);
  return launch_epi<T, false, false>(ctx, p, batch, general);
}

}  // namespace

int launch_gemm_fast16(ginn_hip_ctx* ctx, const GemmArgs& a) {
  if (a.dtype != GINN_HIP_F16 && a.dtype != GINN_HIP_BF16) return kUnsupported;
  if (a.bcols || a.ccols) return kUnsupported;
  if (a.k < 4 * BK) return kUnsupported;
  // Extents need not be multiples of the tile: the last tile row / column and the last K tile are masked
  // inside the kernel.  Every run of elements that is contiguous in memory (the rows of C and of a
  // row-contiguous operand, K along a K-contiguous one) must be a whole number of 16-byte chunks.
  if (a.m % 8 || (a.op_b == GINN_HIP_OP_T && a.n % 8)) return kUnsupported;
  if ((a.op_a == GINN_HIP_OP_T || a.op_b == GINN_HIP_OP_N) && a.k % 8) return kUnsupported;
  if (a.lda % 8 || a.ldb % 8 || a.ldc % 8) return kUnsupported;
  auto aligned16 = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  if (!aligned16(a.A) || !aligned16(a.B) || !aligned16(a.C)) return kUnsupported;
  if (a.pre && !aligned16(a.pre)) return kUnsupported;
  if (a.bias && reinterpret_cast<uintptr_t>(a.bias) % 8) return kUnsupported;
  if (a.batch > 1 && (a.stride_a % 8 || a.stride_b % 8 || a.stride_c % 8)) return kUnsupported;
  const int tiles_m = (a.m + BM - 1) / BM, tiles_n = (a.n + BN - 1) / BN;
  const long long tiles = (long long)tiles_m * tiles_n;
  // Tiles that reach beyond the matrix multiply for nothing: with more than an eighth of the work wasted
  // the 128 x 128 kernel, whose edge tiles waste less, takes the product.
  if ((double)tiles * BM * BN > 1.125 * (double)a.m * a.n) return kUnsupported;
  // With tiles for fewer than 9/16 of the CUs too much of the chip idles and
  // the 128 x 128 kernel is the better fit (measured, bf16: 3072^3 = 144 tiles
  // 61 us here against 78-79 us there; 2048 x 4096 x 2048 = 128 tiles level at
  // 42-43 us; 2560^3 = 100 tiles 51-55 against 46 us).
  if (tiles * a.batch * 16 < ctx->num_cus * 9) return kUnsupported;
  // Per-lane byte offsets inside one operand tile are kept in 32 bits.
  if ((long long)a.lda * 256 * 2 >= (1ll << 31) || (long long)a.ldb * 256 * 2 >= (1ll << 31))
    return kUnsupported;

  FastParams p;
  p.A = static_cast<const uint16_t*>(a.A);
  p.B = static_cast<const uint16_t*>(a.B);
  p.C = static_cast<uint16_t*>(a.C);
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.lda = a.lda;
  p.ldb = a.ldb;
  p.ldc = a.ldc;
  p.sa = a.stride_a;
  p.sb = a.stride_b;
  p.sc = a.stride_c;
  p.beta = a.beta;
  p.bias = static_cast<const uint16_t*>(a.bias);
  p.pre = static_cast<uint16_t*>(a.pre);
  p.act = a.act;
  p.tiles_m = tiles_m;
  p.tiles_n = tiles_n;
  const bool akc = a.op_a == GINN_HIP_OP_T;
  const bool bkc = a.op_b == GINN_HIP_OP_N;
  // XCD-aware ordering needs the tile count to split evenly over the 8 XCDs.
  p.group = (tiles % 8 == 0) ? ((akc && bkc) ? 4 : 8) : 0;
  if (p.group > p.tiles_m) p.group = p.tiles_m;
  // 0 = plain, 1 = general, 2 = a bias alone (see the kernel)
  const bool bias_only = a.bias && a.beta == 0.f && !a.pre && a.act == GINN_HIP_ACT_IDENTITY;
  const int general = bias_only ? 2 : (a.beta != 0.f || a.bias || a.pre || a.act != GINN_HIP_ACT_IDENTITY) ? 1 : 0;
  if (a.dtype == GINN_HIP_F16) return launch_layout<F16>(ctx, p, a.batch, akc, bkc, general);
  return launch_layout<BF16>(ctx, p, a.batch, akc, bkc, general);
}

}  // namespace ginn_hip
