// GEMM family (mm / addmm / bmm / linear) for gfx950.
//
// MFMA path (bf16 / fp16 storage, fp32 accumulation): each 256-thread workgroup (4 waves as
// 2x2) owns a BM x BN tile of C and walks K in steps of 64. Tiles of A and B are staged through
// double-buffered LDS in a K-major layout (one 128-byte line of 64 K-values per matrix row),
// with the 16-byte chunks of every line XOR-swizzled by the row number so that both the
// workgroup's stores and the waves' ds_read_b128 operand fetches are bank-conflict free.
// Every wave computes a (BM/2) x (BN/2) sub-tile with v_mfma_f32_32x32x16 instructions.
// B may be stored K-major ([N,K] rows: the `weight.t()` view of a Linear layer) or N-major
// ([K,N] rows); the N-major case is transposed in registers on its way into LDS.
// The epilogue adds the bias in fp32, applies the optional GELU, casts once and stores.
// Workgroups are numbered so that the 32 tiles resident on one XCD form a compact patch of
// C and share A/B panels through that XCD's L2.
//
// Fallback path: a 64x64 SIMT tile kernel that takes any dtype, strides and alignment.
//
// Arithmetic contract: fp32 accumulate, bias added in fp32 before the single down-cast
// (torch_mojo_backend/eager_kernels/matmul_ops.mojo:2651-2720).
#include <type_traits>

#include "gemm_mfma.h"
#include "gemm_ring.h"
#include "gemm_stream64.h"
#include "gemm_f32.h"

namespace tmb {

// ---------------------------------------------------------------------------
// Epilogue math
// ---------------------------------------------------------------------------
// ---------------------------------------------------------------------------
// SIMT fallback: any dtype / stride / alignment. 64x64 tile, BK = 16, 4x4 per thread.
// ---------------------------------------------------------------------------
template <typename T, int EPI>
__global__ __launch_bounds__(256) void gemm_simt_kernel(
    T* __restrict__ c, const T* __restrict__ a, const T* __restrict__ b,
    const T* __restrict__ bias, int64_t m, int64_t n, int64_t k, int64_t sa_m, int64_t sa_k,
    int64_t sb_k, int64_t sb_n, int64_t ldc, int64_t stride_a, int64_t stride_b,
    int64_t stride_c, int64_t tiles_n, bool twice) {
  constexpr int TM = 64, TN = 64, TK = 16;
  __shared__ float As[TK][TM + 4];
  __shared__ float Bs[TK][TN + 4];
  const int64_t batch = blockIdx.y;
  const int64_t tile = blockIdx.x;
  const int64_t tm = tile / tiles_n, tn = tile - tm * tiles_n;
  const int64_t m0 = tm * TM, n0 = tn * TN;
  a += batch * stride_a;
  b += batch * stride_b;
  c += batch * stride_c;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int64_t k0 = 0; k0 < k; k0 += TK) {
    // A tile: 64 rows x 16 k = 1024 elements, 4 per thread.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + i * 256;
      int r, kk;
      if (sa_k == 1) { r = e >> 4; kk = e & 15; } else { r = e & 63; kk = e >> 6; }
      const int64_t gm = m0 + r, gk = k0 + kk;
      As[kk][r] = (gm < m && gk < k) ? to_f32(a[gm * sa_m + gk * sa_k]) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + i * 256;
      int cidx, kk;
      if (sb_k == 1) { cidx = e >> 4; kk = e & 15; } else { cidx = e & 63; kk = e >> 6; }
      const int64_t gn = n0 + cidx, gk = k0 + kk;
      Bs[kk][cidx] = (gn < n && gk < k) ? to_f32(b[gk * sb_k + gn * sb_n]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t gm = m0 + ty * 4 + i;
    if (gm >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gn = n0 + tx * 4 + j;
      if (gn >= n) continue;
      float v = acc[i][j];
      if (bias != nullptr) v += to_f32(bias[gn]);
      c[gm * ldc + gn] = finish<T, EPI>(v, twice);
    }
  }
}

// Tile choice. 256x256 has the best reuse per byte staged through LDS, but it runs one workgroup
// per CU; narrow outputs and short-K products (attention's q.k^T and att.v) are load/store bound
// and want more, smaller workgroups in flight.
template <typename T, bool B_KMAJOR, int EPI>
static int mfma_pick_tile(const GemmArgs& g, int64_t batch, hipStream_t stream) {
  auto tiles = [&](int64_t bm, int64_t bn) { return ((g.m + bm - 1) / bm) * ((g.n + bn - 1) / bn) * batch; };
  // Direct-to-LDS ring kernel for long enough K. 256x256 (8 waves, 64-deep stages: every row
  // of a K-major operand is fetched as one whole 128-byte line) has the best steady state; it
  // is used when its tiles fill the 256 CUs in nearly whole rounds, otherwise smaller tiles cut
  // the idle tail. N-major B is staged in whole 16-byte column chunks, so N must be a multiple
  // of 8 there (nothing past column N-1 is ever read).
  if (g.k >= 256 && g.n > 64 && (B_KMAJOR || g.n % 8 == 0)) {
    const int64_t t256 = tiles(256, 256);
    // One partial round of 256 x 256 tiles (at least 144 of the 256 CUs busy) still beats smaller
    // tiles in several rounds: 16384 x 768 x 3072 runs in 66-72 us so, against 76-88 us with the
    // best smaller tile. (The 16x16x32 MFMA helps there from K = 2048 on with K-major B and from
    // K = 8192 on with N-major B: 16384 x 768 x 50304 runs in 1.05 against 1.14 ms.)
    if (g.k % 64 == 0 && t256 >= 144 && t256 <= 256 && t256 * 10 < 256 * 9) {
      if (g.k >= (B_KMAJOR ? 2048 : 8192))
        return launch_ring<T, 256, 256, 64, 2, 4, 2, B_KMAJOR, EPI, false, false, true>(g, batch, stream);
      return launch_ring<T, 256, 256, 64, 2, 4, 2, B_KMAJOR, EPI, false, false, false>(g, batch, stream);
    }
    // Short K: the prologue and epilogue of a tile weigh as much as its main loop, so rings that
    // leave room for two workgroups per CU (72 KB of LDS each) win by overlapping them.
    if (g.k % 32 == 0) {
      // (with the 16x16x32 MFMA and one fragment slot: four waves per SIMD, +2-4 %)
      if (!B_KMAJOR && g.k < 4096 && tiles(128, 256) >= 256)
        return launch_ring<T, 128, 256, 32, 2, 4, 3, B_KMAJOR, EPI, false, false, true>(g, batch, stream);
      // (K not a multiple of 64 only: the 64-deep form of this tile below is 5-10 % faster)
      if (B_KMAJOR && g.k % 64 != 0 && g.k <= 1024 && g.n <= 2304 && tiles(256, 128) >= 512)
        return launch_ring<T, 256, 128, 32, 4, 2, 3, B_KMAJOR, EPI>(g, batch, stream);
    }
    if (g.k % 64 == 0) {
      const int64_t rounds = (t256 + 255) / 256;
      if (t256 >= 768 || t256 * 10 >= rounds * 256 * 9) {
        // (the 16x16x32 MFMA: +3-6 % at long K, +2-4 % at K = 768 .. 3072; a short-K product
        // whose output streams to memory, as the 50257-wide vocabulary projection, loses 4 %)
        const bool streamed = g.m * g.n * batch * 2 >= (int64_t{256} << 20);
        if (g.k >= 4096 || !streamed)
          return launch_ring<T, 256, 256, 64, 2, 4, 2, B_KMAJOR, EPI, false, false, true>(g, batch, stream);
        return launch_ring<T, 256, 256, 64, 2, 4, 2, B_KMAJOR, EPI, false, false, false>(g, batch, stream);
      }
      // (from three quarters of a round on: 8192 x 768 x 3072 runs in 39-42 us here against
      // 50-55 us with 128 x 128 tiles)
      if (tiles(256, 128) >= 192)
        return launch_ring<T, 256, 128, 64, 4, 2, 3, B_KMAJOR, EPI>(g, batch, stream);
    }
    if (g.k % 32 == 0 && tiles(128, 128) >= 32) {
      // (16x16x32 MFMA, one k-step per 32-deep stage: +5-7 % for K-major B once the launch has
      // a few rounds of tiles; level or behind for small launches and for N-major B, whose
      // fragments need twice the LDS instructions; the 32-deep configurations that run four
      // waves per SIMD have no registers for its fragments at all)
      if constexpr (B_KMAJOR) {
        if (tiles(128, 128) >= 512)
          return launch_ring<T, 128, 128, 32, 2, 2, 4, B_KMAJOR, EPI, false, false, true>(g, batch, stream);
      }
      return launch_ring<T, 128, 128, 32, 2, 2, 4, B_KMAJOR, EPI>(g, batch, stream);
    }
  }
  // Register-staged kernel for the rest (short K, K not a multiple of 32, ragged N-major N).
  if (g.n <= 64) return launch_mfma<T, 256, 64, 4, 1, B_KMAJOR, EPI>(g, batch, stream);
  if (g.k <= 128 || tiles(128, 128) >= 128)
    return launch_mfma<T, 128, 128, 2, 2, B_KMAJOR, EPI>(g, batch, stream);
  return launch_mfma<T, 64, 64, 2, 2, B_KMAJOR, EPI>(g, batch, stream);
}

template <typename T, int EPI>
static int launch_simt(const GemmArgs& g, int64_t batch, int trans_a, int trans_b,
                       hipStream_t stream) {
  const int64_t tiles_m = (g.m + 63) / 64, tiles_n = (g.n + 63) / 64;
  const int64_t tiles = tiles_m * tiles_n;
  if (tiles >= (int64_t{1} << 31) || batch > 65535) return TMB_ERR_UNSUPPORTED;
  const int64_t sa_m = trans_a ? 1 : g.lda, sa_k = trans_a ? g.lda : 1;
  const int64_t sb_k = trans_b ? 1 : g.ldb, sb_n = trans_b ? g.ldb : 1;
  gemm_simt_kernel<T, EPI><<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(batch)), dim3(256), 0, stream>>>(
      static_cast<T*>(g.c), static_cast<const T*>(g.a), static_cast<const T*>(g.b),
      static_cast<const T*>(g.bias), g.m, g.n, g.k, sa_m, sa_k, sb_k, sb_n, g.ldc, g.stride_a,
      g.stride_b, g.stride_c, tiles_n, g.round_like_unfused != 0);
  return check_launch();
}

// A stored [K, M] with B stored [K, N] (both "k-outer": the weight-gradient product dy^T x):
// the ring kernel stages A the way it stages N-major B. Needs whole 16-byte chunks along m and n
// and enough K for the ring.
template <typename T>
static int mfma_transposed_a(const GemmArgs& g, int64_t batch, hipStream_t stream) {
  const int64_t t256 = ((g.m + 255) / 256) * ((g.n + 255) / 256) * batch;
  // When the last round of 256 x 256 tiles would leave more than a fifth of the launch's slots
  // empty, 128 x 256 tiles on two workgroups per CU end with a shorter tail: the weight gradient
  // of a vocabulary projection, 50304 x 768 x 16384, runs in 1.11 against 1.23 ms.
  const int64_t rounds = (t256 + 255) / 256;
  const int64_t t128x256 = ((g.m + 127) / 128) * ((g.n + 255) / 256) * batch;
  if (t256 * 5 < rounds * 256 * 4 && t128x256 >= 512)
    return launch_ring<T, 128, 256, 32, 2, 4, 3, false, TMB_EPI_NONE, true, false, true>(g, batch, stream);
  if (g.k % 64 == 0 && t256 >= 192)
    return launch_ring<T, 256, 256, 64, 2, 4, 2, false, TMB_EPI_NONE, true>(g, batch, stream);
  return launch_ring<T, 128, 128, 32, 2, 2, 4, false, TMB_EPI_NONE, true>(g, batch, stream);
}

static bool mfma_transposed_a_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b,
                                       int epilogue) {
  if (!trans_a || trans_b || epilogue != TMB_EPI_NONE) return false;
  if (g.k % 32 != 0 || g.k < 256 || g.m % 8 != 0 || g.n % 8 != 0 || g.n <= 64) return false;
  if (g.lda % 8 != 0 || g.ldb % 8 != 0 || !aligned16(g.a) || !aligned16(g.b)) return false;
  if (batch > 1 && (g.stride_a % 8 != 0 || g.stride_b % 8 != 0)) return false;
  const int64_t a_span = g.k * g.lda * 2, b_span = g.k * g.ldb * 2;
  return a_span < (int64_t{1} << 32) && b_span < (int64_t{1} << 32);
}

static bool mfma_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b) {
  if (trans_a) return false;
  if (g.k % 8 != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0) return false;
  if (!aligned16(g.a) || !aligned16(g.b)) return false;
  if (batch > 1 && (g.stride_a % 8 != 0 || g.stride_b % 8 != 0)) return false;
  if (g.m < 1 || g.n < 1 || g.k < 8) return false;
  // the kernel addresses operands with 32-bit byte offsets from their base
  const int64_t a_span = g.m * g.lda * 2, b_span = (trans_b ? g.n : g.k) * g.ldb * 2;
  if (a_span >= (int64_t{1} << 32) || b_span >= (int64_t{1} << 32)) return false;
  (void)trans_b;
  return true;
}

// Split-K: products with few output tiles and a long K (weight gradients, narrow projections)
// leave most CUs idle. K is cut into `splits` runs of whole stages (equal to within one stage)
// that run as the y dimension of one launch of a ring kernel and store fp32 partials
// [splits][M][N] into a workspace; a second kernel adds them in split order and applies bias,
// epilogue and the one cast, so the result is still "fp32 accumulation, one rounding" and depends
// on the shape only.
//
// Tile and split count come from a small cost model (all in microseconds): the 256 x 256 x 64
// kernel sustains about 1240 TFLOP/s over 256 one-per-CU workgroups, the 128 x 128 x 32 kernel
// about 900 TFLOP/s over 512 two-per-CU workgroups; the launch takes ceil(units / slots) rounds of
// one unit's time, the reduction reads splits * M * N * 4 bytes at about 4 TB/s.
struct SplitKPlan {
  int splits;  // 0: not used
  int tile;    // 128 or 256
  int64_t k_chunk;  // fp32 kernel only: equal chunks
};
static SplitKPlan splitk_plan(int64_t batch, int64_t m, int64_t n, int64_t k) {
  SplitKPlan p{0, 0, 0};
  if (batch != 1 || k < 2048 || k % 32 != 0 || n <= 64 || m < 1) return p;
  const int64_t t128 = ((m + 127) / 128) * ((n + 127) / 128);
  if (t128 >= 256) return p;  // at least one tile per CU: no split
  const int64_t t256 = ((m + 255) / 256) * ((n + 255) / 256);
  double best = 0.0;
  for (int tile = 128; tile <= 256; tile += 128) {
    const int bk = tile == 128 ? 32 : 64;
    if (k % bk != 0) continue;
    if (tile == 256 && (m <= 128 || n <= 128)) continue;
    const int64_t tiles = tile == 128 ? t128 : t256;
    const int64_t slots = tile == 128 ? 512 : 256;
    const double unit_rate = tile == 128 ? 900e6 / 512 : 1240e6 / 256;  // FLOP per us per workgroup
    for (int64_t splits = 2; splits <= 16; ++splits) {
      if (k / bk / splits < 8) break;  // at least 8 stages per split
      const double chunk = static_cast<double>(k) / splits;
      // (a 128-tile workgroup that has its CU to itself runs about 1.7 times faster than one of
      // two: 768 x 768 x 16384 in 5 splits of 36 tiles takes 32 us)
      const double alone = (tile == 128 && tiles * splits <= 256) ? 1.7 : 1.0;
      const double unit = 2.0 * tile * tile * chunk / (unit_rate * alone);
      const double rounds = static_cast<double>((tiles * splits + slots - 1) / slots);
      const double reduce = 3.0 + static_cast<double>(splits) * m * n * 4.0 / 4e6;
      const double cost = rounds * unit + reduce;
      if (p.splits == 0 || cost < best) {
        best = cost;
        p.splits = static_cast<int>(splits);
        p.tile = tile;
      }
    }
  }
  return p;
}

template <typename T, int EPI>
static int launch_splitk(const GemmArgs& g, const SplitKPlan& plan, int trans_a, int trans_b,
                         float* workspace, hipStream_t stream) {
  GemmArgs part = g;
  part.c = workspace;
  part.bias = nullptr;
  part.residual = nullptr;
  part.ldc = g.n;
  part.stride_c = g.m * g.n;
  part.stride_a = 0;
  part.stride_b = 0;
  part.splits = plan.splits;
  int rc;
  if (plan.tile == 256) {
    // (a split's run of K is short: the 32x32x16 MFMA, as for short unsplit products)
    if (trans_a)
      rc = launch_ring<T, 256, 256, 64, 2, 4, 2, false, TMB_EPI_NONE, true, true, false>(part, plan.splits, stream);
    else if (trans_b)
      rc = launch_ring<T, 256, 256, 64, 2, 4, 2, true, TMB_EPI_NONE, false, true, false>(part, plan.splits, stream);
    else
      rc = launch_ring<T, 256, 256, 64, 2, 4, 2, false, TMB_EPI_NONE, false, true, false>(part, plan.splits, stream);
  } else if (trans_a) {
    rc = launch_ring<T, 128, 128, 32, 2, 2, 4, false, TMB_EPI_NONE, true, true>(part, plan.splits, stream);
  } else if (trans_b) {
    rc = launch_ring<T, 128, 128, 32, 2, 2, 4, true, TMB_EPI_NONE, false, true>(part, plan.splits, stream);
  } else {
    rc = launch_ring<T, 128, 128, 32, 2, 2, 4, false, TMB_EPI_NONE, false, true>(part, plan.splits, stream);
  }
  if (rc != 0) return rc;
  launch_splitk_reduce<T, EPI>(static_cast<T*>(g.c), workspace, static_cast<const T*>(g.bias), g.m,
                               g.n, g.ldc, plan.splits, g.round_like_unfused != 0, stream);
  return check_launch();
}

// fp32 products run 16 times slower on the matrix cores than 16-bit ones, so a 128 x 128 tile
// with a few hundred K already takes tens of microseconds and the split pays from much shorter K.
// Chunks are whole 16-byte groups of K so that every chunk keeps the operands' alignment.
static SplitKPlan splitk_plan_f32(int64_t batch, int64_t m, int64_t n, int64_t k) {
  SplitKPlan p{0, 0, 0};
  if (batch != 1 || k < 128 || m < 1 || n < 1) return p;
  const int64_t tiles = ((m + kF32BM - 1) / kF32BM) * ((n + kF32BN - 1) / kF32BN);
  if (tiles >= 256) return p;
  int64_t splits = 512 / tiles;
  if (splits > 16) splits = 16;
  if (splits > k / 64) splits = k / 64;
  while (splits >= 2 && k % (splits * 4) != 0) --splits;
  if (splits < 2) return p;
  p.splits = static_cast<int>(splits);
  p.tile = 128;
  p.k_chunk = k / splits;
  return p;
}

template <int EPI>
static int launch_splitk_f32(const GemmArgs& g, const SplitKPlan& plan, int trans_a, int trans_b,
                             float* workspace, hipStream_t stream) {
  GemmArgs part = g;
  part.c = workspace;
  part.bias = nullptr;
  part.k = plan.k_chunk;
  part.ldc = g.n;
  part.stride_c = g.m * g.n;
  part.stride_a = trans_a ? plan.k_chunk * g.lda : plan.k_chunk;
  part.stride_b = trans_b ? plan.k_chunk : plan.k_chunk * g.ldb;
  const int rc = launch_f32_mfma<TMB_EPI_NONE>(part, plan.splits, trans_a, trans_b, stream);
  if (rc != 0) return rc;
  launch_splitk_reduce<float, EPI>(static_cast<float*>(g.c), workspace,
                                   static_cast<const float*>(g.bias), g.m, g.n, g.ldc, plan.splits,
                                   false, stream);
  return check_launch();
}

template <typename T, int EPI>
static int gemm_typed(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, bool half,
                      hipStream_t stream, void* workspace = nullptr, size_t workspace_bytes = 0) {
  if constexpr (!__is_same(T, float)) {
    if (half && workspace != nullptr && g.residual == nullptr) {
      const SplitKPlan plan = splitk_plan(batch, g.m, g.n, g.k);
      const bool operands_ok =
          trans_a ? mfma_transposed_a_eligible(g, batch, trans_a, trans_b, TMB_EPI_NONE)
                  : (mfma_eligible(g, batch, trans_a, trans_b) && (trans_b || g.n % 8 == 0));
      if (plan.splits > 0 && operands_ok && g.m * g.n < (int64_t{1} << 31) &&
          workspace_bytes >= static_cast<size_t>(plan.splits) * g.m * g.n * 4)
        return launch_splitk<T, EPI>(g, plan, trans_a, trans_b, static_cast<float*>(workspace),
                                     stream);
    }
    if (half && mfma_transposed_a_eligible(g, batch, trans_a, trans_b, EPI))
      return mfma_transposed_a<T>(g, batch, stream);
    if (half && !trans_a && stream64_eligible(g, batch, trans_b, EPI)) {
      return trans_b ? launch_stream64<T, true>(g, batch, stream)
                     : launch_stream64<T, false>(g, batch, stream);
    }
    if (half && mfma_eligible(g, batch, trans_a, trans_b)) {
      return trans_b ? mfma_pick_tile<T, true, EPI>(g, batch, stream)
                     : mfma_pick_tile<T, false, EPI>(g, batch, stream);
    }
  }
  if constexpr (__is_same(T, float)) {
    if (g.residual == nullptr && f32_mfma_eligible(g, batch, trans_a, trans_b)) {
      const SplitKPlan plan = splitk_plan_f32(batch, g.m, g.n, g.k);
      if (plan.splits > 0 && workspace != nullptr && g.m * g.n < (int64_t{1} << 31) &&
          workspace_bytes >= static_cast<size_t>(plan.splits) * g.m * g.n * 4)
        return launch_splitk_f32<EPI>(g, plan, trans_a, trans_b, static_cast<float*>(workspace),
                                      stream);
      return launch_f32_mfma<EPI>(g, batch, trans_a, trans_b, stream);
    }
  }
  return launch_simt<T, EPI>(g, batch, trans_a, trans_b, stream);
}

template <typename T>
static int gemm_epi(const GemmArgs& g, int64_t batch, int ta, int tb, int epilogue,
                    hipStream_t stream, void* ws, size_t ws_bytes) {
  switch (epilogue) {
    case TMB_EPI_NONE: return gemm_typed<T, TMB_EPI_NONE>(g, batch, ta, tb, true, stream, ws, ws_bytes);
    case TMB_EPI_GELU_TANH: return gemm_typed<T, TMB_EPI_GELU_TANH>(g, batch, ta, tb, true, stream, ws, ws_bytes);
    case TMB_EPI_GELU_ERF: return gemm_typed<T, TMB_EPI_GELU_ERF>(g, batch, ta, tb, true, stream, ws, ws_bytes);
    default: return TMB_ERR_INVALID_ARGUMENT;
  }
}

// Fills C with epilogue(bias) (or zeros) when k == 0.
template <typename T, int EPI>
__global__ void gemm_k0_kernel(T* c, const T* bias, int64_t m, int64_t n, int64_t ldc,
                               int64_t stride_c, bool twice) {
  T* cb = c + static_cast<int64_t>(blockIdx.y) * stride_c;
  const int64_t total = m * n;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / n, col = i - r * n;
    const float v = bias != nullptr ? to_f32(bias[col]) : 0.0f;
    cb[r * ldc + col] = finish<T, EPI>(v, twice);
  }
}

}  // namespace tmb

static int gemm_entry(void* c, const void* a, const void* b, const void* bias,
                      const void* residual, int64_t batch, int64_t m, int64_t n, int64_t k,
                      int64_t lda, int64_t ldb, int64_t ldc, int64_t ldr, int64_t stride_a,
                      int64_t stride_b, int64_t stride_c, int64_t stride_r, int trans_a,
                      int trans_b, int dtype, int epilogue_flags, void* stream,
                      void* workspace = nullptr, size_t workspace_bytes = 0,
                      int residual_dtype = -1, int out_dtype = -1) {
  using namespace tmb;
  if (batch < 0 || m < 0 || n < 0 || k < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (epilogue_flags < 0 || (epilogue_flags & ~(0xff | TMB_EPI_ROUND_LIKE_UNFUSED)) != 0)
    return TMB_ERR_INVALID_ARGUMENT;
  const int epilogue = epilogue_flags & 0xff;
  const bool twice = (epilogue_flags & TMB_EPI_ROUND_LIKE_UNFUSED) != 0;
  if (epilogue < TMB_EPI_NONE || epilogue > TMB_EPI_GELU_ERF) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F32 && dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (residual_dtype < 0) residual_dtype = dtype;
  if (out_dtype < 0) out_dtype = dtype;
  if ((residual_dtype != dtype && residual_dtype != TMB_F32) ||
      (out_dtype != dtype && out_dtype != TMB_F32))
    return TMB_ERR_UNSUPPORTED;
  const bool resid_f32 = residual != nullptr && residual_dtype == TMB_F32 && dtype != TMB_F32;
  const bool out_f32 = out_dtype == TMB_F32 && dtype != TMB_F32;
  if (batch == 0 || m == 0 || n == 0) return TMB_OK;
  if (c == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  if (k > 0 && (a == nullptr || b == nullptr)) return TMB_ERR_INVALID_ARGUMENT;
  // Leading dimensions must cover the stored row of each operand.
  if (ldc < n) return TMB_ERR_INVALID_ARGUMENT;
  if (k > 0) {
    if (lda < (trans_a ? m : k)) return TMB_ERR_INVALID_ARGUMENT;
    if (ldb < (trans_b ? k : n)) return TMB_ERR_INVALID_ARGUMENT;
  }
  if (batch > 65535) return TMB_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GemmArgs g{c, a, b, bias, m, n, k, lda, ldb, ldc, stride_a, stride_b, stride_c, 0, 0, 0, residual, ldr, stride_r};
  g.round_like_unfused = twice ? 1 : 0;
  g.resid_f32 = resid_f32 ? 1 : 0;
  g.out_f32 = out_f32 ? 1 : 0;
  if (out_f32 && residual == nullptr) return TMB_ERR_UNSUPPORTED;  // fp32 C exists for the residual form only
  if (residual != nullptr) {
    // only the MFMA kernels carry the second epilogue step; the caller adds separately otherwise
    if (dtype == TMB_F32 || k == 0 || ldr < n || !mfma_eligible(g, batch, trans_a, trans_b))
      return TMB_ERR_UNSUPPORTED;
    // fp32 operands of the epilogue and an epilogue that stays in fp32 exist without GELU only
    if ((resid_f32 || out_f32 || !twice) && epilogue != TMB_EPI_NONE) return TMB_ERR_UNSUPPORTED;
    if ((resid_f32 || out_f32) && twice) return TMB_ERR_INVALID_ARGUMENT;
  }
  if (k == 0) {
    const unsigned blocks = static_cast<unsigned>((m * n + 255) / 256 > 4096 ? 4096 : (m * n + 255) / 256);
    dim3 grid(blocks, static_cast<unsigned>(batch));
#define TMB_K0(T)                                                                                   \
  switch (epilogue) {                                                                               \
    case TMB_EPI_NONE: gemm_k0_kernel<T, TMB_EPI_NONE><<<grid, 256, 0, s>>>((T*)c, (const T*)bias, m, n, ldc, stride_c, twice); break; \
    case TMB_EPI_GELU_TANH: gemm_k0_kernel<T, TMB_EPI_GELU_TANH><<<grid, 256, 0, s>>>((T*)c, (const T*)bias, m, n, ldc, stride_c, twice); break; \
    default: gemm_k0_kernel<T, TMB_EPI_GELU_ERF><<<grid, 256, 0, s>>>((T*)c, (const T*)bias, m, n, ldc, stride_c, twice); break; \
  }
    if (dtype == TMB_F32) { TMB_K0(float) } else if (dtype == TMB_F16) { TMB_K0(f16_t) } else { TMB_K0(bf16_t) }
#undef TMB_K0
    return check_launch();
  }
  switch (dtype) {
    case TMB_F32: return gemm_epi<float>(g, batch, trans_a, trans_b, epilogue, s, workspace, workspace_bytes);
    case TMB_F16: return gemm_epi<f16_t>(g, batch, trans_a, trans_b, epilogue, s, workspace, workspace_bytes);
    default: return gemm_epi<bf16_t>(g, batch, trans_a, trans_b, epilogue, s, workspace, workspace_bytes);
  }
}

extern "C" int tmb_gemm(void* c, const void* a, const void* b, const void* bias, int64_t batch,
                        int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc,
                        int64_t stride_a, int64_t stride_b, int64_t stride_c, int trans_a,
                        int trans_b, int dtype, int epilogue, void* stream) {
  return gemm_entry(c, a, b, bias, nullptr, batch, m, n, k, lda, ldb, ldc, 0, stride_a, stride_b,
                    stride_c, 0, trans_a, trans_b, dtype, epilogue, stream);
}

extern "C" size_t tmb_gemm_workspace_bytes(int64_t batch, int64_t m, int64_t n, int64_t k,
                                           int dtype) {
  if (dtype != TMB_F32 && dtype != TMB_F16 && dtype != TMB_BF16) return 0;
  const tmb::SplitKPlan plan = dtype == TMB_F32 ? tmb::splitk_plan_f32(batch, m, n, k)
                                                : tmb::splitk_plan(batch, m, n, k);
  if (plan.splits == 0 || m * n >= (int64_t{1} << 31)) return 0;
  return static_cast<size_t>(plan.splits) * static_cast<size_t>(m) * static_cast<size_t>(n) * 4;
}

extern "C" int tmb_gemm_ws(void* c, const void* a, const void* b, const void* bias, int64_t batch,
                           int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t stride_a, int64_t stride_b, int64_t stride_c, int trans_a,
                           int trans_b, int dtype, int epilogue, void* workspace,
                           size_t workspace_bytes, void* stream) {
  return gemm_entry(c, a, b, bias, nullptr, batch, m, n, k, lda, ldb, ldc, 0, stride_a, stride_b,
                    stride_c, 0, trans_a, trans_b, dtype, epilogue, stream, workspace,
                    workspace_bytes);
}

extern "C" int tmb_gemm_residual(void* c, const void* a, const void* b, const void* bias,
                                 const void* residual, int64_t batch, int64_t m, int64_t n,
                                 int64_t k, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldr,
                                 int64_t stride_a, int64_t stride_b, int64_t stride_c,
                                 int64_t stride_r, int trans_a, int trans_b, int dtype,
                                 int residual_dtype, int out_dtype, int epilogue, void* stream) {
  if (residual == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  if (residual_dtype < 0 || out_dtype < 0) return TMB_ERR_INVALID_ARGUMENT;
  return gemm_entry(c, a, b, bias, residual, batch, m, n, k, lda, ldb, ldc, ldr, stride_a,
                    stride_b, stride_c, stride_r, trans_a, trans_b, dtype, epilogue, stream, nullptr,
                    0, residual_dtype, out_dtype);
}
