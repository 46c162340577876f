// Shape selection and split-K policy of the 128 x 128 family of product kernels
// (fp16 / bf16: mid-size shapes; fp32: every aligned shape with enough tiles).
#include <algorithm>

#include "gemm_mid.h"

namespace ginn_hip {

int launch_gemm_mid(ginn_hip_ctx* ctx, const GemmArgs& a) {
  using namespace mid;
  if (a.dtype != GINN_HIP_F16 && a.dtype != GINN_HIP_BF16 && a.dtype != GINN_HIP_F32) return kUnsupported;
  const int es = static_cast<int>(dtype_size(a.dtype));
  const int bk = kRowBytes / es;   // k values per K tile
  const int per16 = 16 / es;       // elements per 16 bytes
  if (a.bcols || a.ccols) return kUnsupported;
  if (a.k < bk) return kUnsupported;
  // Extents need not be multiples of the tile: the last tile row / column and the last K tile are masked
  // inside the kernel.  What must hold is that every run of elements that is contiguous in memory -- the
  // rows of C and of a row-contiguous operand, K along a K-contiguous one -- is a whole number of 16-byte
  // chunks, so that a chunk lies inside or outside the matrix.
  const bool any_n = a.op_b == GINN_HIP_OP_N;
  if (a.m % per16) return kUnsupported;
  if (!any_n && a.n % per16) return kUnsupported;
  if ((a.op_a == GINN_HIP_OP_T || any_n) && a.k % per16) return kUnsupported;
  // 128 x 128 when both extents allow, else the variant with one 64-wide side.  A last tile row / column
  // that is less than half full: the 64-wide side for a narrow output, for which the wasted half tile
  // counts; a wide one keeps 128 (4096 x 4000 x 4096 fp16: 194-221 us on 128 x 64).
  auto wide = [](int extent) {
    if (extent % 128 == 0) return 2;
    if (extent % 64 == 0) return 1;
    return (extent <= 64 || ((extent - 1) % 128 < 64 && extent < 512)) ? 1 : 2;
  };
  int fm = wide(a.m), fn = wide(a.n);
  // (Both sides 64 wide only by the tile counts below.)
  if (fm == 1 && fn == 1) {
    if (a.n > 64) fn = 2;
    else if (a.m > 64) fm = 2;
  }
  if (a.lda % per16 || a.ldb % per16 || a.ldc % per16) return kUnsupported;
  auto aligned16 = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  if (!aligned16(a.A) || !aligned16(a.B) || !aligned16(a.C)) return kUnsupported;
  if (a.pre && !aligned16(a.pre)) return kUnsupported;
  if (a.bias && !aligned16(a.bias)) return kUnsupported;
  if (a.batch > 1 && (a.stride_a % per16 || a.stride_b % per16 || a.stride_c % per16)) return kUnsupported;
  // Per-lane byte offsets inside one operand tile are kept in 32 bits.
  if ((long long)a.lda * 128 * es >= (1ll << 31) || (long long)a.ldb * 128 * es >= (1ll << 31)) return kUnsupported;
  // fp32: the matrix pipe is 16 x slower per flop than for the 16-bit types, so
  // what counts is how many CUs have work.  With fewer than half a 128 x 128
  // tile per CU the 128 x 64 shape doubles the tiles, and K is split (below)
  // until about every CU has a workgroup; if that still leaves most of the
  // chip idle the generic kernel's 64 x 64 tiles do better.
  const bool f32 = a.dtype == GINN_HIP_F32;
  bool f32_small = false, f32_tiny_tiles = false;
  if (f32) {
    const long long tiles128 = (long long)((a.m + 127) / 128) * ((a.n + 127) / 128) * a.batch;
    if (tiles128 * 2 < ctx->num_cus) {
      f32_small = true;
      // 64 x 64 tiles when they give most CUs a workgroup without a K split:
      // the same matrix-pipe time per CU as 128 x 64 tiles over half of K each,
      // and no partial tiles to fold in a second launch (which costs what
      // some 20 K tiles of such a workgroup cost: the fewer the tiles, the
      // shorter the K up to which that holds).
      const long long tiles64 = (long long)((a.m + 63) / 64) * ((a.n + 63) / 64) * a.batch;
      const int kt = (a.k + bk - 1) / bk;
      const bool enough = tiles64 >= ctx->num_cus || (tiles64 * 4 >= 3 * ctx->num_cus && kt <= 64) ||
                          (tiles64 * 8 >= 3 * ctx->num_cus && kt <= 32);
      if (enough && tiles64 <= 2 * ctx->num_cus)
        fm = 1, fn = 1, f32_tiny_tiles = true;
      else if (fm == 2 && fn == 2) fn = 1;
      const long long tiles = (long long)((a.m + 64 * fm - 1) / (64 * fm)) * ((a.n + 64 * fn - 1) / (64 * fn)) * a.batch;
      const long long by_k = a.batch == 1 ? std::max(1, kt / 2) : 1;
      if (tiles * by_k * 4 < ctx->num_cus) return kUnsupported;
    }
  }

  // 16-bit types: a workgroup's time is the latency chain of its K loop, not
  // the matrix pipe, so with 128-wide tiles for at most half of the CUs the
  // 64 x 64 shape (four times the workgroups, a quarter of the bytes per K
  // tile each) is faster (1024^3: 9.8 -> 5.4 us; 512^3: 6.7 -> 3.8 us); with
  // more tiles than that the larger shapes win (1536^3: 13.4 against 16.2 us).
  // With a K-contiguous B the last tile column may be partly filled; the
  // narrowest right-hand sides (n <= 8, 4096 x n x 4096) stay 5 % faster on
  // 128 x 64 tiles.
  if (!f32 && (a.n % 64 == 0 || a.n > 8)) {
    const long long tiles_now = (long long)((a.m + 64 * fm - 1) / (64 * fm)) * ((a.n + 64 * fn - 1) / (64 * fn)) * a.batch;
    const long long tiles64 = (long long)((a.m + 63) / 64) * ((a.n + 63) / 64) * a.batch;
    // (Two 64 x 64 workgroups per CU over a very long K run level with one 128-wide one:
    // 2048 x 1024 x 8192 49-57 against 51-52 us; those keep the larger shape.)
    if (tiles_now * 2 <= ctx->num_cus && !(tiles64 > ctx->num_cus && a.k / bk > 64)) fm = 1, fn = 1;
  }
  MidParams p;
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
  p.beta = a.beta;
  p.bias = a.bias;
  p.pre = a.pre;
  p.act = a.act;
  p.tiles_m = (a.m + 64 * fm - 1) / (64 * fm);
  p.tiles_n = (a.n + 64 * fn - 1) / (64 * fn);
  p.partial = nullptr;
  const long long tiles = (long long)p.tiles_m * p.tiles_n;
  p.group = (tiles % 8 == 0) ? 8 : 0;
  if (p.group > p.tiles_m) p.group = p.tiles_m;
  // Few tiles per XCD: make an XCD's share an exact block of g tile rows x (share / g) tile columns with the
  // smallest g + share / g, the operand panels its L2 has to fetch (12 x 12 tiles of 64 x 64 over K = 4096:
  // blocks of 6 x 3 instead of 8 rows x 2.25 columns, 16.2 -> 14.0 us; nothing changes for the other shapes
  // measured).  Larger outputs keep panels of 8 rows.
  if (p.group > 0 && tiles / 8 <= 32) {
    const int per = (int)(tiles / 8);
    int best = 0, cost = 1 << 30;
    for (int g = 1; g <= p.tiles_m && g <= per; ++g) {
      if (per % g || p.tiles_m % g || p.tiles_n % (per / g)) continue;
      if (g + per / g <= cost) {
        best = g;
        cost = g + per / g;
      }
    }
    if (best) p.group = best;
  }
  const bool akc = a.op_a == GINN_HIP_OP_T;
  const bool bkc = a.op_b == GINN_HIP_OP_N;
  const int kt_total = (a.k + bk - 1) / bk;

  // Split K when the output has tiles for less than half of the CUs and K is
  // long: a split costs a second launch and moves its fp32 partial tiles
  // through memory twice, so every split keeps at least 8 K tiles (a K tile
  // takes about 0.4 us on a lightly loaded chip, the fold about 5 us) and all
  // partials together stay below 8 MiB.
  int splits = 1;
  if (f32_small) {
    // fp32 with few tiles: a K tile costs 0.85 us of matrix-pipe time per
    // 128 x 64 tile, so splits down to 2 K tiles still pay for the fold.
    if (a.batch == 1 && kt_total >= 4 && !f32_tiny_tiles) {
      const size_t per = (size_t)a.m * a.n * sizeof(float);
      long long s = ctx->num_cus / tiles;
      if (s > kt_total / 2) s = kt_total / 2;
      if (s > 32) s = 32;
      if ((size_t)s * per > (8u << 20)) s = (long long)((8u << 20) / per);
      if ((size_t)s * per > ctx->workspace_bytes) s = (long long)(ctx->workspace_bytes / per);
      splits = s < 2 ? 1 : (int)s;
    }
  } else if (a.batch == 1 && tiles * 2 <= ctx->num_cus && kt_total >= 24) {
    const size_t per = (size_t)a.m * a.n * sizeof(float);
    long long s = ctx->num_cus / tiles;
    if (s > kt_total / 8) s = kt_total / 8;
    if (s > 32) s = 32;
    if ((size_t)s * per > (8u << 20)) s = (long long)((8u << 20) / per);
    if ((size_t)s * per > ctx->workspace_bytes) s = (long long)(ctx->workspace_bytes / per);
    splits = s < 2 ? 1 : (int)s;
  }
  p.k_tiles = (kt_total + splits - 1) / splits;
  splits = (kt_total + p.k_tiles - 1) / p.k_tiles;
  const bool general = a.beta != 0.f || a.bias || a.pre || a.act != GINN_HIP_ACT_IDENTITY;
  auto launch = [&](int batch, int nsplit, int epi) {
    if (fm == 2 && fn == 2) return launch_shape<2, 2>(ctx, p, a.dtype, batch, nsplit, epi, akc, bkc);
    if (fm == 2) return launch_shape<2, 1>(ctx, p, a.dtype, batch, nsplit, epi, akc, bkc);
    if (fn == 1) return launch_shape<1, 1>(ctx, p, a.dtype, batch, nsplit, epi, akc, bkc);
    return launch_shape<1, 2>(ctx, p, a.dtype, batch, nsplit, epi, akc, bkc);
  };
  if (splits == 1) return launch(a.batch, 1, general ? kGeneral : kPlain);
  std::lock_guard<std::mutex> lock(ctx->mutex);  // the workspace holds the partial tiles
  p.partial = static_cast<float*>(ctx->workspace);
  const int rc = launch(1, splits, kPartial);
  if (rc != kOk) return rc;
  return launch_splitk_reduce(ctx, a, splits, p.partial);
}

}  // namespace ginn_hip
