// Product with a narrow right-hand side (n <= 16), C[m x n] = A[m x k] * B[k x n], both stored as given (NN),
// as ONE launch without a split of K over workgroups, for an A of a few MiB: there the second launch that
// folds the partial sums of the kernels which split K costs as much as the product itself.
//
// A workgroup owns a strip of 16 rows of A over all of K.  A column of the strip is 32 bytes (64 for
// fp32): too short a piece of memory on its own, but the strips that share a 128-byte line are given to
// workgroups that run side by side on ONE XCD (workgroup ids are dealt to the 8 XCDs round robin, so XCD x
// gets the strips x S / 8 .. (x + 1) S / 8 - 1): the line is fetched from memory once and served to the
// neighbours by that XCD's L2.  Measured with loads alone on 4096 x 4096: 5.5-6.0 TB/s this way, 1.6-2.7 TB/s
// with neighbouring strips on different XCDs (every XCD fetches every line).
//
// The four waves of a workgroup split K and work on their own: a wave moves its part of the strip from
// memory into LDS with direct loads (16 bytes per lane; a load instruction is 32 (16) consecutive columns
// of the strip, which land as [column][16 rows], the layout the operand reads want), four buffers of 4
// loads each, and the B values of the same K range next to them ([n][k], 16-byte chunks XOR-placed by n
// so that the 16 columns a read touches lie in different banks; lanes of columns beyond n load nothing).
// Per 16 columns of a 16-bit strip that is one transposing LDS read (the A operand of v_mfma_f32_16x16x16:
// 16 rows x 16 k), one 8-byte read (the B operand) and one MFMA; fp32 takes four v_mfma_f32_16x16x4 with
// 4-byte reads.  No barrier inside the loop: a wave reads only what it loaded.  The waves' sums meet in LDS
// at the end; beta, bias, activation and the kept pre-activation are applied there.  Columns n .. 15 of the
// MFMA compute on whatever the B buffer holds and are never stored.
//
// What it reaches (fp16 4096 x 1 x 4096, kernel alone): 5.9 us with the loads of A only, 6.3 with the
// epilogue, 7.6 with the loads of B (one more load instruction in five), 8.5 us with operand reads and
// MFMAs -- level with the two launches of the split kernels at that size, ahead below it.  The loads alone are
// bound by what a CU's first-level cache takes in: it fetches whole 128-byte lines of which the strip uses a
// quarter, 512 KiB per CU for this A, the same as with full lines on a quarter of the CUs.  (A vector-ALU form
// for n <= 4 with B in LDS as fp32 was measured too: 13.6 us, unpacking and multiplying 16-bit rows one by one.)
#include <type_traits>

#include "common.h"

namespace ginn_hip {
namespace {

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kRows = 16;            // rows of a strip
constexpr int kLoadsA = 4;           // direct loads of A per buffer and wave: 4 KiB = 256 bytes of K per row chunk
constexpr int kBuffers = 4;          // per wave: three on their way while one is multiplied
constexpr int kBufA = kLoadsA * 1024;
// Bytes of one buffer with NB loads of B (each 1 KiB: 256 bytes of K for four columns of B).
constexpr int buffer_bytes(int nb) { return kBufA + nb * 1024; }
constexpr int lds_bytes(int nb) { return kWaves * kBuffers * buffer_bytes(nb); }

// Four consecutive elements as floats: 16 bytes of fp32, 8 bytes of a 16-bit type.
template <typename T>
__device__ __forceinline__ void load4(const typename T::storage* ptr, float (&v)[4]) {
  if constexpr (sizeof(typename T::storage) == 4) {
    const f32x4 q = *reinterpret_cast<const f32x4*>(ptr);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = q[e];
  } else {
    const u32x2 raw = *reinterpret_cast<const u32x2*>(ptr);
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      v[2 * e] = to_float<T>(static_cast<uint16_t>(raw[e] & 0xffffu));
      v[2 * e + 1] = to_float<T>(static_cast<uint16_t>(raw[e] >> 16));
    }
  }
}
template <typename T>
__device__ __forceinline__ void store4(typename T::storage* ptr, const float (&v)[4]) {
  if constexpr (sizeof(typename T::storage) == 4) {
    *reinterpret_cast<f32x4*>(ptr) = f32x4{v[0], v[1], v[2], v[3]};
  } else {
    u32x2 raw;
#pragma unroll
    for (int e = 0; e < 2; ++e)
      raw[e] = static_cast<uint32_t>(from_float<T>(v[2 * e])) | (static_cast<uint32_t>(from_float<T>(v[2 * e + 1])) << 16);
    *reinterpret_cast<u32x2*>(ptr) = raw;
  }
}

struct StripParams {
  const void* A;
  const void* B;
  void* C;
  int m, n, k;
  int lda, ldb, ldc;
  float beta;
  const void* bias;
  void* pre;
  int act;
  int strips;
};

// NB: direct loads of B per buffer (each brings 256 bytes of K for four columns): ceil(n / 4), so that every
// load instruction has at least one active lane -- one whose lanes are all beyond n would be branched around,
// and the waits below count load instructions.
template <typename T, int NB, bool GENERAL>
__global__ __launch_bounds__(kThreads) void gemm_strip_kernel(StripParams p) {
  using S = typename T::storage;
  constexpr int ES = sizeof(S);
  constexpr int LPC = kRows * ES / 16;       // lanes per column of the strip: 2 or 4
  constexpr int CPL = 64 / LPC;              // columns per load instruction: 32 or 16
  constexpr int BUFK = kLoadsA * CPL;        // K values per buffer: 128 or 64 (256 bytes of K either way)
  static_assert(BUFK * ES == 256, "a B buffer row holds 256 bytes of K");
  constexpr int SC = ES == 2 ? 64 : 16;      // columns per step of four MFMAs: 4 x 16 or 4 x 4
  constexpr int kBuf = buffer_bytes(NB);
  constexpr int kLoads = kLoadsA + NB;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // Strips that share memory lines run side by side on one XCD.
  int s = blockIdx.x;
  const int even = p.strips & ~7;
  if (s < even) s = (s & 7) * (even >> 3) + (s >> 3);
  const int r0 = s * kRows;
  const int rows_valid = min(kRows, p.m - r0);  // a multiple of 16 / ES

  // This wave's K range, in units of 16.
  const int units = p.k >> 4;
  const int kw0 = (units * wave / kWaves) << 4, kw1 = (units * (wave + 1) / kWaves) << 4;
  const int span = kw1 - kw0;
  const int n_buffers = (span + BUFK - 1) / BUFK;

  char* const wlds = lds + wave * (kBuffers * kBuf);
  // A: lane l of a load moves the 16 bytes `part` of column l / LPC; a part beyond the rows of the matrix
  // re-reads part 0 (in bounds; its rows are never stored).
  const int part = lane % LPC, lcol = lane / LPC;
  const int a_row_off = (part * (16 / ES) < rows_valid ? part * 16 : 0);
  const char* const a_base = static_cast<const char*>(p.A) + static_cast<size_t>(r0) * ES + a_row_off;
  // B: lane l of load i moves, for column n = 4 i + l / 16, the chunk that lands at position l % 16 of the
  // column's 256 bytes, which is chunk (l % 16) ^ n of the buffer's K range; columns beyond n are not loaded.
  const int b_pos = lane & 15;

  // Buffer number b of this wave (K range kw0 + b BUFK ...) into its slot b % kBuffers.
  auto issue_buffer = [&](int b) {
    const int kb = kw0 + b * BUFK;
    char* la = wlds + (b % kBuffers) * kBuf;
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i) {
      const int col = min(kb + i * CPL + lcol, p.k - 1);
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(a_base + static_cast<size_t>(col) * p.lda * ES),
          (void __attribute__((address_space(3)))*)(la + i * 1024), 16, 0, 0);
    }
    char* lb = la + kBufA;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int ncol = 4 * i + (lane >> 4);
      int kk = kb + ((b_pos ^ ncol) * (16 / ES));
      kk = min(kk, p.k - 16 / ES);  // k is a multiple of 16: the last chunk is whole
      // Lanes of columns beyond n load nothing (their part of the buffer is never multiplied into a stored
      // column): every workgroup reads all of B, and the same few lines asked for by a thousand waves at
      // once are what an XCD's L2 serves slowest.
      if (ncol < p.n)
        __builtin_amdgcn_global_load_lds(
            (const void __attribute__((address_space(1)))*)(static_cast<const char*>(p.B) +
                                                            (static_cast<size_t>(ncol) * p.ldb + kk) * ES),
            (void __attribute__((address_space(3)))*)(lb + i * 1024), 16, 0, 0);
    }
  };
  // Waits until all but the `newer` most recently issued buffers have landed.
  auto wait_buffers = [&](int newer) {
    switch (newer) {
      case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kLoads) : "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * kLoads) : "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(3 * kLoads) : "memory"); break;
    }
  };

  // Operand addresses inside a buffer for the 16 columns starting at its column 0.
  const int n16 = lane & 15, g = lane >> 4;
  uint32_t a_addr;
  if constexpr (ES == 2) {
    // transposing read: lane (s = n16, group g) names 8 bytes (4 rows) of column 4 g + s / 4 and receives
    // the four K values 4 g .. 4 g + 3 of row s
    a_addr = (4 * g + (n16 >> 2)) * 32 + (n16 & 3) * 8;
  } else {
    a_addr = g * 64 + n16 * 4;  // A[row n16][column g], columns 64 bytes apart
  }
  const uint32_t lds_w = (uint32_t)(uintptr_t)wlds;
  const int nb16 = min(n16, 4 * NB - 1);  // the column of B this lane reads: only 4 NB columns are loaded

  // The operands of step t (columns t SC .. of the wave's range): eight LDS reads, four MFMAs.  A 16-bit
  // step whose range ends early re-reads its last 16 columns (those MFMAs are left out).
  typedef typename std::conditional<ES == 2, u32x2, uint32_t>::type Operand;
  // Two accumulators, so that consecutive MFMAs do not wait for each other.
  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  auto issue_reads = [&](int t, Operand (&fa)[4], Operand (&fb)[4]) {
    const int col = t * SC;                       // relative to kw0
    const uint32_t base = lds_w + ((col / BUFK) % kBuffers) * kBuf;
    const int c = col % BUFK;                     // inside the buffer
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if constexpr (ES == 2) {
        const int cu = c + 16 * min(u, (span - col - 16) >> 4);
        const int kq = cu + 4 * g;                // B[k = cu + 4 g .. + 3][n16]: 8 bytes inside chunk kq / 8
        const uint32_t aa = base + a_addr + cu * 32;
        const uint32_t ba = base + kBufA + nb16 * 256 + (((kq >> 3) ^ nb16) * 16) + (kq & 7) * 2;
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(fa[u]) : "v"(aa) : "memory");
        asm volatile("ds_read_b64 %0, %1" : "=v"(fb[u]) : "v"(ba) : "memory");
      } else {
        const int kq = c + 4 * u + g;             // column of this lane in MFMA u
        const uint32_t aa = base + a_addr + (c + 4 * u) * 64;
        const uint32_t ba = base + kBufA + nb16 * 256 + (((kq >> 2) ^ nb16) * 16) + (kq & 3) * 4;
        asm volatile("ds_read_b32 %0, %1" : "=v"(fa[u]) : "v"(aa) : "memory");
        asm volatile("ds_read_b32 %0, %1" : "=v"(fb[u]) : "v"(ba) : "memory");
      }
    }
  };
  auto multiply = [&](int t, Operand (&fa)[4], Operand (&fb)[4]) {
    // (ties the operands to the wait in front of this call)
    asm volatile("" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]),
                      "+v"(fb[3])
                 :
                 : "memory");
    const int left = span - t * SC;  // columns from this step on
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      f32x4& acc = (u & 1) ? acc1 : acc0;
      if constexpr (ES == 2) {
        if (16 * u < left) {
          if constexpr (std::is_same<T, BF16>::value) {
            acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, fa[u]),
                                                            __builtin_bit_cast(s16x4, fb[u]), acc, 0, 0, 0);
          } else {
            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, fa[u]),
                                                        __builtin_bit_cast(f16x4, fb[u]), acc, 0, 0, 0);
          }
        }
      } else {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(fa[u]), __uint_as_float(fb[u]), acc, 0, 0, 0);
      }
    }
  };

  // Pipeline: kBuffers buffers on their way.  Two steps per turn, both sets of operand reads issued before
  // the first MFMA, every wait inside the turn (no register that an LDS read is still to fill is carried
  // around the loop, where the compiler might copy it); a buffer's slot is refilled once the reads of its
  // last step have completed.
  constexpr int kStepsPerBuffer = BUFK / SC;  // 2 or 4
  static_assert(kStepsPerBuffer % 2 == 0, "a turn of two steps stays inside one buffer");
  const int n_steps = (span + SC - 1) / SC;
  int issued = 0;
  for (; issued < kBuffers && issued < n_buffers; ++issued) issue_buffer(issued);
  Operand fa0[4], fb0[4], fa1[4], fb1[4];
  for (int t = 0; t < n_steps; t += 2) {
    if (t % kStepsPerBuffer == 0) wait_buffers(issued - t / kStepsPerBuffer - 1);
    const bool two = t + 1 < n_steps;
    issue_reads(t, fa0, fb0);
    if (two) {
      issue_reads(t + 1, fa1, fb1);
      asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");  // in order: step t has arrived
    } else {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    multiply(t, fa0, fb0);
    if (two) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      multiply(t + 1, fa1, fb1);
    }
    // every read of this turn has completed: after the buffer's last step its slot takes the next buffer
    if ((t + 2) % kStepsPerBuffer == 0 && issued < n_buffers) issue_buffer(issued++);
  }

  // The four waves' sums: acc[j] = row 4 g + j, column n16.
  const f32x4 acc = acc0 + acc1;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  float* xch = reinterpret_cast<float*>(lds);  // [wave][column n16][16 rows]
  *reinterpret_cast<f32x4*>(xch + (wave * 16 + n16) * 16 + 4 * g) = acc;
  __syncthreads();
  if (wave != 0 || n16 >= p.n) return;
  f32x4 v = acc;
#pragma unroll
  for (int w = 1; w < kWaves; ++w) v += *reinterpret_cast<const f32x4*>(xch + (w * 16 + n16) * 16 + 4 * g);
  const int row = r0 + 4 * g;
  if (4 * g >= rows_valid) return;  // rows_valid is a multiple of 4
  const size_t off = static_cast<size_t>(n16) * p.ldc + row;
  S* C = static_cast<S*>(p.C);
  float out[4] = {v[0], v[1], v[2], v[3]};
  if constexpr (GENERAL) {
    S* P = static_cast<S*>(p.pre);
    if (p.beta != 0.f) {
      float old[4];
      load4<T>((P ? P : C) + off, old);
#pragma unroll
      for (int e = 0; e < 4; ++e) out[e] += p.beta * old[e];
    }
    if (p.bias) {
      float b4[4];
      load4<T>(static_cast<const S*>(p.bias) + row, b4);
#pragma unroll
      for (int e = 0; e < 4; ++e) out[e] += b4[e];
    }
    if (P) store4<T>(P + off, out);
    if (p.act != GINN_HIP_ACT_IDENTITY) act_forward_n<kFastMath<T>, 4>(p.act, out);
  }
  store4<T>(C + off, out);
}

template <typename T, int NB>
int launch_general(ginn_hip_ctx* ctx, const StripParams& p, bool general) {
  if (general) {
    auto fn = gemm_strip_kernel<T, NB, true>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), lds_bytes(NB)));
    fn<<<dim3(p.strips), dim3(kThreads), lds_bytes(NB), ctx->stream>>>(p);
  } else {
    auto fn = gemm_strip_kernel<T, NB, false>;
    static std::atomic<unsigned long long> lds_allowed{0};
    GH_HIP(allow_dynamic_lds(lds_allowed, ctx->device, reinterpret_cast<const void*>(fn), lds_bytes(NB)));
    fn<<<dim3(p.strips), dim3(kThreads), lds_bytes(NB), ctx->stream>>>(p);
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

template <typename T>
int launch_width(ginn_hip_ctx* ctx, const StripParams& p, bool general) {
  if (p.n <= 4) return launch_general<T, 1>(ctx, p, general);
  if (p.n <= 8) return launch_general<T, 2>(ctx, p, general);
  if (p.n <= 12) return launch_general<T, 3>(ctx, p, general);
  return launch_general<T, 4>(ctx, p, general);
}

}  // namespace

int launch_gemm_strip(ginn_hip_ctx* ctx, const GemmArgs& a) {
  if (a.dtype != GINN_HIP_F16 && a.dtype != GINN_HIP_BF16 && a.dtype != GINN_HIP_F32) return kUnsupported;
  if (a.op_a != GINN_HIP_OP_N || a.op_b != GINN_HIP_OP_N || a.batch != 1 || a.acols || a.bcols || a.ccols)
    return kUnsupported;
  if (a.n < 1 || a.n > 16) return kUnsupported;
  const int es = static_cast<int>(dtype_size(a.dtype));
  const int per16 = 16 / es;
  // Whole 16-byte chunks along the rows of A and C and along K of B; K in whole MFMA steps.
  if (a.m % per16 || a.k % 16 || a.lda % per16 || a.ldb % per16) return kUnsupported;
  if (a.ldc % 4 || (a.ldc * es) % 8) return kUnsupported;
  auto aligned = [](const void* ptr, int to) { return reinterpret_cast<uintptr_t>(ptr) % to == 0; };
  if (!aligned(a.A, 16) || !aligned(a.B, 16) || !aligned(a.C, 4 * es)) return kUnsupported;
  if (a.pre && !aligned(a.pre, 4 * es)) return kUnsupported;
  if (a.bias && !aligned(a.bias, 4 * es)) return kUnsupported;
  // Worth it when reading A is the work and the strips fill the chip (at least a strip for every other CU,
  // 16 MFMA steps per wave) -- and up to the size of A from which the second launch of the kernels that split
  // K over workgroups no longer counts.  Measured against those, one launch each / product with its fold, us:
  // fp16 2048 x 4 x 2048 5.0 / 9.0, 4096 x 1 x 1024 3.5 / 6.6, 4096 x 16 x 2048 6.8 / 8.2, 2048 x 1 x 4096
  // 7.5 / 8.7, 4096 x n x 4096 level (8.5-10.6 / 8.4-10.2), 8192 x 1 x 8192 31 / 24; fp32 4096 x 16 x 1024
  // 6.5 / 8.5, 4096 x 16 x 2048 10.7 / 12.1, but 4096 x 1 x 2048 9.5 / 8.2, 4096 x 1 x 4096 18.5 / 15.0.
  const int strips = (a.m + kRows - 1) / kRows;
  if (strips * 2 < ctx->num_cus || a.k < 1024) return kUnsupported;
  const long long a_bytes = static_cast<long long>(a.m) * a.k * es;
  if (es == 2 ? a_bytes > (24ll << 20) : (a.n < 8 || strips < ctx->num_cus || a_bytes > (32ll << 20)))
    return kUnsupported;
  if (static_cast<long long>(a.lda) * es * a.k >= (1ll << 40)) return kUnsupported;
  StripParams p;
  p.A = a.A;
  p.B = a.B;
  p.C = a.C;
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.lda = a.lda;
  p.ldb = a.ldb;
  p.ldc = a.ldc;
  p.beta = a.beta;
  p.bias = a.bias;
  p.pre = a.pre;
  p.act = a.act;
  p.strips = strips;
  const bool general = a.beta != 0.f || a.bias || a.pre || a.act != GINN_HIP_ACT_IDENTITY;
  GH_HIP(hipSetDevice(ctx->device));
  switch (a.dtype) {
    case GINN_HIP_F16: return launch_width<F16>(ctx, p, general);
    case GINN_HIP_BF16: return launch_width<BF16>(ctx, p, general);
    default: return launch_width<F32>(ctx, p, general);
  }
}

}  // namespace ginn_hip

