// Batched 16-bit products whose slices are small and memory bound: the products
// of an attention block (ginn/node/prod.h:93-169 through gpu_batched_gemm,
// ginn/prod.h:69-135), Q K^T [T x 64][64 x T] and P V [T x T][T x 64] and their
// four gradient products, for some hundred (batch, head) slices.  Each slice
// is a few tiles and a few K tiles of work; what a launch costs is the latency
// of a workgroup's load -> multiply -> store chain times the number of rounds
// of workgroups.  The 128 x 128 family (gemm_mid.h) runs 8 waves per workgroup
// with at least 64 KiB of LDS, so two workgroups share a CU.  This kernel is the
// same tile arithmetic with 4 waves and one or two LDS stages (24-36 KiB for a
// single K tile), so four or five workgroups share a CU and overlap each
// other's latencies; nothing is pipelined inside a workgroup beyond a second
// stage for K loops of more than one tile.  beta = 0, no bias / activation
// (everything else stays on the 128 x 128 family).
//
// LDS layouts, direct global -> LDS loads, swizzles and fragment reads are
// those of gemm_mid.h (helpers reused from there).
#include "gemm_mid.h"
#include "kernel_util.h"

namespace ginn_hip {
namespace bsmall {

using namespace mid;  // u32x4, f32x16, chunk_src, kc_offset, tr_offset, tr_issue, b128_issue, mma, ...

constexpr int kThreadsB = 256;  // 4 waves: a 2 x 2 grid of (32 FM) x (32 FN) quadrants

struct Params {
  const void* A;
  const void* B;
  void* C;
  int m, n, k;
  int lda, ldb, ldc;
  long long sa, sb, sc;
  // slice z at (z % inner) * s + (z / inner) * s2 (inner = batch for a plain strided batch)
  long long sa2, sb2, sc2;
  int inner;
  int tiles_m, tiles_n;  // per slice
  int batch;
  int whole_lines;  // columns of C start on 128-byte lines
  int xcd_spread;  // workgroup ids are dealt to 8 XCDs round robin: give every XCD a contiguous run of slices
};

template <int FM, int FN>
struct GeoB {
  static constexpr int BM = 64 * FM, BN = 64 * FN;
  static constexpr int kTileA = BM * kRowBytes, kTileB = BN * kRowBytes;
  static constexpr int kStageBytes = kTileA + kTileB;
  static constexpr int kEpiColStride = 64 * FM + 16;  // bytes: 32 FM halfs of a column + padding
  static constexpr int kEpiWaveBytes = 32 * FN * kEpiColStride;
  static constexpr int lds_bytes(int stages) {
    return stages * kStageBytes > 4 * kEpiWaveBytes ? stages * kStageBytes : 4 * kEpiWaveBytes;
  }
};

// EDGE: extents that are no multiples of the tile (or result columns that do not start on 128-byte
// lines): masked stores through the cache; without it every store is a whole line and non-temporal.
template <typename T, bool AKC, bool BKC, int FM, int FN, bool EDGE>
__global__ __launch_bounds__(kThreadsB) void gemm_bsmall_kernel(Params p) {
  using G = GeoB<FM, FN>;
  constexpr int ES = 2;
  constexpr int BK = kRowBytes / ES;  // 64
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave & 1) * 32 * FM, wn = (wave >> 1) * 32 * FN;

  const int tiles = p.tiles_m * p.tiles_n;
  int pid = blockIdx.x;
  if (p.xcd_spread) {
    const int per = (tiles * p.batch) >> 3;
    pid = (pid & 7) * per + (pid >> 3);
  }
  const int bz = pid / tiles;
  const int tile = pid % tiles;
  const long long z_in = bz % p.inner, z_out = bz / p.inner;
  const int m0 = (tile % p.tiles_m) * G::BM, n0 = (tile / p.tiles_m) * G::BN;
  const int KT = (p.k + BK - 1) / BK;
  // K values in the last K tile (64 unless K is no multiple of the tile): the lanes whose 16 bytes of that
  // tile lie beyond them load zeros.  Tile rows beyond m / n re-read rows inside the matrix (chunk_src) and
  // what they produce is not stored.
  const int k_lim = p.k - (KT - 1) * BK;
  const int m_valid = EDGE ? min(G::BM, p.m - m0) : G::BM, n_valid = EDGE ? min(G::BN, p.n - n0) : G::BN;

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // ---- direct loads: thread tid moves chunks v = i * 256 + tid of each operand tile.
  constexpr int kPassA = 2 * FM, kPassB = 2 * FN;  // (64 F rows x 8 chunks) / 256 threads
  uint32_t a_off[kPassA], b_off[kPassB];
#pragma unroll
  for (int i = 0; i < kPassA; ++i)
    a_off[i] = (uint32_t)(chunk_src<AKC, FM, ES>(i * kThreadsB + tid, p.lda, m_valid) * ES);
#pragma unroll
  for (int i = 0; i < kPassB; ++i)
    b_off[i] = (uint32_t)(chunk_src<BKC, FN, ES>(i * kThreadsB + tid, p.ldb, n_valid) * ES);
  // This thread's chunk along K of a K-contiguous tile (the same in every pass); its k-row of pass 0 of a
  // row-contiguous tile (8 FM or 8 FN chunks per k-row).
  const bool kc_ok = (((tid & 7) ^ swz_kc(tid >> 3)) * 8) < k_lim;
  constexpr int kRowsPerPassA = kThreadsB / (8 * FM), kRowsPerPassB = kThreadsB / (8 * FN);
  const int a_rc_kr = tid / (8 * FM), b_rc_kr = tid / (8 * FN);
  const long long a_kstep = (AKC ? (long long)BK : (long long)BK * p.lda) * ES;
  const long long b_kstep = (BKC ? (long long)BK : (long long)BK * p.ldb) * ES;
  const char* a_next =
      static_cast<const char*>(p.A) +
      (z_in * p.sa + z_out * p.sa2 + (AKC ? (long long)m0 * p.lda : (long long)m0)) * ES;
  const char* b_next =
      static_cast<const char*>(p.B) +
      (z_in * p.sb + z_out * p.sb2 + (BKC ? (long long)n0 * p.ldb : (long long)n0)) * ES;
  auto issue_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kPassA; ++i) {
      uint32_t off = a_off[i];
      asm volatile("" : "+v"(off));  // keeps (scalar base) + (32-bit lane offset) apart for the addressing mode
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(a_next + off),
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + (i * kThreadsB + wave * 64) * 16), 16,
          0, 0);
    }
#pragma unroll
    for (int i = 0; i < kPassB; ++i) {
      uint32_t off = b_off[i];
      asm volatile("" : "+v"(off));
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(b_next + off),
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + G::kTileA +
                                                    (i * kThreadsB + wave * 64) * 16),
          16, 0, 0);
    }
    a_next += a_kstep;
    b_next += b_kstep;
  };
  // The last K tile: per-lane addresses, zeros beyond K.
  auto issue_last_tile = [&](int buf) {
    const char* zeros = reinterpret_cast<const char*>(kZeroChunk);
#pragma unroll
    for (int i = 0; i < kPassA; ++i) {
      const bool ok = AKC ? kc_ok : (i * kRowsPerPassA + a_rc_kr) < k_lim;
      const char* g = ok ? a_next + a_off[i] : zeros;
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)g,
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + (i * kThreadsB + wave * 64) * 16), 16,
          0, 0);
    }
#pragma unroll
    for (int i = 0; i < kPassB; ++i) {
      const bool ok = BKC ? kc_ok : (i * kRowsPerPassB + b_rc_kr) < k_lim;
      const char* g = ok ? b_next + b_off[i] : zeros;
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)g,
          (void __attribute__((address_space(3)))*)(lds + buf * G::kStageBytes + G::kTileA +
                                                    (i * kThreadsB + wave * 64) * 16),
          16, 0, 0);
    }
  };
  constexpr int kLoads = kPassA + kPassB;

  // ---- fragment addresses inside a stage: one per 32-row block and, for a
  // K-contiguous operand, per sub-step (the swizzle depends on it).
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  uint32_t abase[AKC ? 4 * FM : FM], bbase[BKC ? 4 * FN : FN];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    if (AKC) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) abase[4 * i + ks] = kc_offset(wm + i * 32, ks, lane);
    } else {
      abase[i] = tr_offset<FM>(wm + i * 32, 0, 0, lane);
    }
  }
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    if (BKC) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) bbase[4 * j + ks] = G::kTileA + kc_offset(wn + j * 32, ks, lane);
    } else {
      bbase[j] = G::kTileA + tr_offset<FN>(wn + j * 32, 0, 0, lane);
    }
  }

  // All four sub-steps of the K tile in stage `buf`: the reads of a sub-step
  // are issued together, then multiplied.
  auto multiply_tile = [&](int buf) {
    const uint32_t sb = lds_base + buf * G::kStageBytes;
    auto sub_step = [&](auto KS) {
      constexpr int ks = decltype(KS)::value;
      u32x4 qa[FM], qb[FN];
      u32x2 ha[2 * FM], hb[2 * FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        if constexpr (AKC) {
          qa[i] = b128_issue<0>(sb + abase[4 * i + ks]);
        } else {
          ha[2 * i] = tr_issue<ks * 2048 * FM>(sb + abase[i]);
          ha[2 * i + 1] = tr_issue<ks * 2048 * FM + 512 * FM>(sb + abase[i]);
        }
      }
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if constexpr (BKC) {
          qb[j] = b128_issue<0>(sb + bbase[4 * j + ks]);
        } else {
          hb[2 * j] = tr_issue<ks * 2048 * FN>(sb + bbase[j]);
          hb[2 * j + 1] = tr_issue<ks * 2048 * FN + 512 * FN>(sb + bbase[j]);
        }
      }
      lgkm_wait<0>();
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        if constexpr (AKC) {
          claim(qa[i]);
        } else {
          claim(ha[2 * i]);
          claim(ha[2 * i + 1]);
          qa[i] = __builtin_shufflevector(ha[2 * i], ha[2 * i + 1], 0, 1, 2, 3);
        }
      }
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if constexpr (BKC) {
          claim(qb[j]);
        } else {
          claim(hb[2 * j]);
          claim(hb[2 * j + 1]);
          qb[j] = __builtin_shufflevector(hb[2 * j], hb[2 * j + 1], 0, 1, 2, 3);
        }
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = mma<T>(qa[i], qb[j], acc[i][j]);
    };
    sub_step(std::integral_constant<int, 0>{});
    sub_step(std::integral_constant<int, 1>{});
    sub_step(std::integral_constant<int, 2>{});
    sub_step(std::integral_constant<int, 3>{});
  };

  // ---- K loop: tile kt + 1 is on its way while tile kt is multiplied.
  const bool ragged_k = EDGE && k_lim != BK;
  if (KT == 1 && ragged_k) issue_last_tile(0);
  else issue_tile(0);
  for (int kt = 0; kt < KT; ++kt) {
    if (kt + 1 < KT) {
      // its stage was read last for tile kt - 1: every wave is past the barrier below
      if (kt + 2 == KT && ragged_k) issue_last_tile((kt + 1) & 1);
      else issue_tile((kt + 1) & 1);
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kLoads) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();  // every wave's share of tile kt is in LDS
    multiply_tile(kt & 1);
    __builtin_amdgcn_s_barrier();  // every wave has read tile kt: its stage may be overwritten
  }

  // ---- epilogue: round, stage through the wave's own LDS slice (the last
  // barrier above freed the stages), store 16-byte column segments.
  uint16_t* C = static_cast<uint16_t*>(p.C) + z_in * p.sc + z_out * p.sc2;
  char* stage = lds + wave * G::kEpiWaveBytes;
  const int l32 = lane & 31, lhi = lane >> 5;
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
  constexpr int kRowChunks = 4 * FM;  // 16-byte chunks per column of the wave's tile
  constexpr int kColsPerIter = 64 / kRowChunks;
  const int sub = lane / kRowChunks, chunk = lane % kRowChunks;
#pragma unroll
  for (int it = 0; it < 32 * FN / kColsPerIter; ++it) {
    const int col = it * kColsPerIter + sub;
    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + col * G::kEpiColStride + chunk * 16);
    u32x4* dst = reinterpret_cast<u32x4*>(C + (long long)(n0 + wn + col) * p.ldc + m0 + wm + chunk * 8);
    if constexpr (EDGE) {
      // Neighbouring workgroups complete each other's 128-byte lines, which only the cache can merge
      // (T = 504: 20.8 us with non-temporal stores, 13.1 us with these).
      if (wn + col < n_valid && wm + chunk * 8 < m_valid) *dst = v;
    } else {
      __builtin_nontemporal_store(v, dst);
    }
  }
}

template <typename T, bool AKC, bool BKC, int FM, int FN>
int launch_one(ginn_hip_ctx* ctx, const Params& p) {
  using G = GeoB<FM, FN>;
  const int stages = p.k > 64 ? 2 : 1;
  const int lds_bytes = G::lds_bytes(stages);
  const long long blocks = (long long)p.tiles_m * p.tiles_n * p.batch;
  const bool edge = p.m % G::BM != 0 || p.n % G::BN != 0 || p.k % 64 != 0 || !p.whole_lines;
  if (edge) {
    auto fn = gemm_bsmall_kernel<T, AKC, BKC, FM, FN, true>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), G::lds_bytes(2)));
    fn<<<dim3(static_cast<unsigned>(blocks)), dim3(kThreadsB), lds_bytes, ctx->stream>>>(p);
  } else {
    auto fn = gemm_bsmall_kernel<T, AKC, BKC, FM, FN, false>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), G::lds_bytes(2)));
    fn<<<dim3(static_cast<unsigned>(blocks)), dim3(kThreadsB), lds_bytes, ctx->stream>>>(p);
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

template <typename T, int FM, int FN>
int launch_layout(ginn_hip_ctx* ctx, const Params& p, bool akc, bool bkc) {
  if (akc) {
    if (bkc) return launch_one<T, true, true, FM, FN>(ctx, p);
    return launch_one<T, true, false, FM, FN>(ctx, p);
  }
  if (bkc) return launch_one<T, false, true, FM, FN>(ctx, p);
  return launch_one<T, false, false, FM, FN>(ctx, p);
}

template <typename T>
int launch_shape(ginn_hip_ctx* ctx, const Params& p, int fm, int fn, bool akc, bool bkc) {
  if (fm == 2 && fn == 2) return launch_layout<T, 2, 2>(ctx, p, akc, bkc);
  if (fm == 2) return launch_layout<T, 2, 1>(ctx, p, akc, bkc);
  if (fn == 2) return launch_layout<T, 1, 2>(ctx, p, akc, bkc);
  return launch_layout<T, 1, 1>(ctx, p, akc, bkc);
}

}  // namespace bsmall

int launch_gemm_bsmall(ginn_hip_ctx* ctx, const GemmArgs& a) {
  if (a.dtype != GINN_HIP_F16 && a.dtype != GINN_HIP_BF16) return kUnsupported;
  if (a.batch < 2 || a.beta != 0.f || a.bias || a.pre || a.act != GINN_HIP_ACT_IDENTITY || a.bcols || a.ccols)
    return kUnsupported;
  if (a.k < 64) return kUnsupported;
  // Extents need not be multiples of the tile (a sequence length of 504): the last tile row / column and
  // the last K tile are masked inside the kernel; every run of elements that is contiguous in memory must
  // be a whole number of 16-byte chunks.
  if (a.m % 8 || (a.op_b == GINN_HIP_OP_T && a.n % 8)) return kUnsupported;
  if ((a.op_a == GINN_HIP_OP_T || a.op_b == GINN_HIP_OP_N) && a.k % 8) return kUnsupported;
  // Slices of little arithmetic per byte: one side of 64 (the head size) or a single K tile, and small enough
  // that a slice is a handful of tiles; the other batched shapes gain from the deeper pipeline of gemm_mid.h.
  const bool slim = a.k == 64 || a.m == 64 || a.n == 64;
  if (!slim || a.m > 1024 || a.n > 1024 || a.k > 1024) return kUnsupported;
  if (a.lda % 8 || a.ldb % 8 || a.ldc % 8 || a.stride_a % 8 || a.stride_b % 8 || a.stride_c % 8) return kUnsupported;
  const bool two_level = a.batch_inner > 0;
  if (two_level && (a.stride_a2 % 8 || a.stride_b2 % 8 || a.stride_c2 % 8 || a.batch % a.batch_inner)) return kUnsupported;
  auto aligned16 = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  if (!aligned16(a.A) || !aligned16(a.B) || !aligned16(a.C)) return kUnsupported;
  if ((long long)a.lda * 128 * 2 >= (1ll << 31) || (long long)a.ldb * 128 * 2 >= (1ll << 31)) return kUnsupported;
  // 128-wide tiles unless the extent is a multiple of 64 only, or a ragged one whose last 128 would be
  // less than half full.
  auto wide = [](int extent) { return extent % 128 == 0 || (extent % 64 != 0 && (extent - 1) % 128 >= 64) ? 2 : 1; };
  const int fm = wide(a.m), fn = wide(a.n);
  bsmall::Params p;
  p.A = a.A;
  p.B = a.B;
  p.C = a.C;
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.lda = a.lda;
  p.ldb = a.ldb;
  p.ldc = a.ldc;
  p.sa = a.stride_a;
  p.sb = a.stride_b;
  p.sc = a.stride_c;
  p.inner = two_level ? a.batch_inner : a.batch;
  p.sa2 = two_level ? a.stride_a2 : 0;
  p.sb2 = two_level ? a.stride_b2 : 0;
  p.sc2 = two_level ? a.stride_c2 : 0;
  p.tiles_m = (a.m + 64 * fm - 1) / (64 * fm);
  p.tiles_n = (a.n + 64 * fn - 1) / (64 * fn);
  p.batch = a.batch;
  p.whole_lines = a.ldc % 64 == 0 && a.stride_c % 64 == 0 && p.sc2 % 64 == 0 && reinterpret_cast<uintptr_t>(a.C) % 128 == 0;
  const long long blocks = (long long)p.tiles_m * p.tiles_n * a.batch;
  if (blocks < ctx->num_cus || blocks > (1ll << 30)) return kUnsupported;
  p.xcd_spread = blocks % 8 == 0 ? 1 : 0;
  GH_HIP(hipSetDevice(ctx->device));
  const bool akc = a.op_a == GINN_HIP_OP_T, bkc = a.op_b == GINN_HIP_OP_N;
  if (a.dtype == GINN_HIP_F16) return bsmall::launch_shape<F16>(ctx, p, fm, fn, akc, bkc);
  return bsmall::launch_shape<BF16>(ctx, p, fm, fn, akc, bkc);
}

}  // namespace ginn_hip
