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
#include "tmb_common.h"

namespace tmb {

// ---------------------------------------------------------------------------
// Epilogue math
// ---------------------------------------------------------------------------
// Bias has already been added in fp32. With a GELU epilogue the sum is first rounded to the
// storage type, so that the fused kernel returns exactly what addmm followed by a separate
// gelu returns; then one final cast.
template <typename T, int EPI>
__device__ __forceinline__ T finish(float v) {
  v = pin_f32(v);  // acc + bias is an fp32 sum; it is rounded to T as a separate step
  if constexpr (EPI == TMB_EPI_NONE) {
    return from_f32<T>(v);
  } else {
    const float r = to_f32(from_f32<T>(v));
    return from_f32<T>(EPI == TMB_EPI_GELU_TANH ? gelu_tanh_f32(r) : gelu_erf_f32(r));
  }
}

// ---------------------------------------------------------------------------
// SIMT fallback: any dtype / stride / alignment. 64x64 tile, BK = 16, 4x4 per thread.
// ---------------------------------------------------------------------------
template <typename T, int EPI>
__global__ __launch_bounds__(256) void gemm_simt_kernel(
    T* __restrict__ c, const T* __restrict__ a, const T* __restrict__ b,
    const T* __restrict__ bias, int64_t m, int64_t n, int64_t k, int64_t sa_m, int64_t sa_k,
    int64_t sb_k, int64_t sb_n, int64_t ldc, int64_t stride_a, int64_t stride_b,
    int64_t stride_c, int64_t tiles_n) {
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
      c[gm * ldc + gn] = finish<T, EPI>(v);
    }
  }
}

// ---------------------------------------------------------------------------
// MFMA path
// ---------------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
  static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<f16_t> {
  static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

constexpr int kBK = 64;          // K extent of one LDS stage (64 x 2 bytes = one 128-byte line)
constexpr int kLineBytes = 128;

// Byte offset of 16-byte chunk `chunk` (0..7) of line `row` inside a swizzled tile.
__device__ __forceinline__ int lds_offset(int row, int chunk) {
  return row * kLineBytes + (((chunk ^ row ^ (row >> 3)) & 7) << 4);
}

struct GemmArgs {
  void* c;
  const void* a;
  const void* b;
  const void* bias;
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  int64_t stride_a, stride_b, stride_c;
  int tiles_m, tiles_n;
};

// Maps the launch-order workgroup id to a tile so that each XCD (workgroups are dealt to the
// 8 XCDs round-robin) works on a contiguous run of tiles, walked in column-major groups of
// `kGroupM` tile rows.
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int kXcds = 8;
  constexpr int kGroupM = 8;
  const int total = tiles_m * tiles_n;
  const int q = total / kXcds, r = total % kXcds;
  const int xcd = pid % kXcds, idx = pid / kXcds;
  const int tile = xcd * q + (xcd < r ? xcd : r) + idx;
  const int per_group = kGroupM * tiles_n;
  const int group = tile / per_group;
  const int first_m = group * kGroupM;
  const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  const int in_group = tile - group * per_group;
  tm = first_m + in_group % gsz;
  tn = in_group / gsz;
}

// B_KMAJOR: B is stored [N, K] (ldb = row pitch of an N-row); otherwise [K, N].
template <typename T, int BM, int BN, bool B_KMAJOR, int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmArgs g) {
  constexpr int WM = BM / 2, WN = BN / 2;   // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;  // 32x32 MFMA tiles per wave
  constexpr int A_BYTES = BM * kLineBytes, B_BYTES = BN * kLineBytes;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_LOADS = BM / 32;  // 16-byte chunks per thread per stage
  constexpr int B_LOADS = BN / 32;
  constexpr int B_BLOCKS = (BN + 255) / 256;  // 8x8 transpose blocks per thread (N-major B)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  int tile_m, tile_n;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
  const int64_t m0 = static_cast<int64_t>(tile_m) * BM;
  const int64_t n0 = static_cast<int64_t>(tile_n) * BN;
  const int64_t batch = blockIdx.y;
  const T* __restrict__ A = static_cast<const T*>(g.a) + batch * g.stride_a;
  const T* __restrict__ B = static_cast<const T*>(g.b) + batch * g.stride_b;
  T* __restrict__ C = static_cast<T*>(g.c) + batch * g.stride_c;
  const int64_t M = g.m, N = g.n, K = g.k;

  // ---- global -> register staging -------------------------------------------------------
  u32x4_t a_stage[A_LOADS];
  u32x4_t b_stage[B_KMAJOR ? B_LOADS : B_BLOCKS * 8];
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};

  const int ld_row = tid >> 3;   // 0..31
  const int ld_chunk = tid & 7;  // 16-byte chunk inside the 128-byte line

  auto load_a = [&](int64_t k0) {
    const int64_t kk = k0 + ld_chunk * 8;
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
      int64_t row = m0 + ld_row + j * 32;
      row = row < M ? row : M - 1;
      a_stage[j] = (kk < K) ? *reinterpret_cast<const u32x4_t*>(A + row * g.lda + kk) : zero4;
    }
  };
  auto load_b = [&](int64_t k0) {
    if constexpr (B_KMAJOR) {
      const int64_t kk = k0 + ld_chunk * 8;
#pragma unroll
      for (int j = 0; j < B_LOADS; ++j) {
        int64_t row = n0 + ld_row + j * 32;
        row = row < N ? row : N - 1;
        b_stage[j] = (kk < K) ? *reinterpret_cast<const u32x4_t*>(B + row * g.ldb + kk) : zero4;
      }
    } else {
      // Thread owns an 8(k) x 8(n) block: k-chunk kc = blk / (BN/8), n-group ng = blk % (BN/8).
#pragma unroll
      for (int q = 0; q < B_BLOCKS; ++q) {
        const int blk = tid + q * 256;
        const int kc = blk / (BN / 8), ng = blk % (BN / 8);
        const int64_t nn = n0 + ng * 8;
        const bool active = blk < BN;  // BN blocks in total (8 k-chunks x BN/8 n-groups)
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const int64_t kk = k0 + kc * 8 + r;
          u32x4_t v = zero4;
          if (active && kk < K) {
            const T* src = B + kk * g.ldb + nn;
            if (nn + 8 <= N) {
              v = *reinterpret_cast<const u32x4_t*>(src);
            } else {
              // ragged right edge: element-wise, never past column N-1
              unsigned short e[8];
#pragma unroll
              for (int t = 0; t < 8; ++t)
                e[t] = (nn + t < N) ? reinterpret_cast<const unsigned short*>(src)[t]
                                    : static_cast<unsigned short>(0);
              v[0] = e[0] | (static_cast<uint32_t>(e[1]) << 16);
              v[1] = e[2] | (static_cast<uint32_t>(e[3]) << 16);
              v[2] = e[4] | (static_cast<uint32_t>(e[5]) << 16);
              v[3] = e[6] | (static_cast<uint32_t>(e[7]) << 16);
            }
          }
          b_stage[q * 8 + r] = v;
        }
      }
    }
  };
  auto store_stage = [&](int buf) {
    unsigned char* sa = smem + buf * STAGE_BYTES;
    unsigned char* sb = sa + A_BYTES;
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
      const int row = ld_row + j * 32;
      *reinterpret_cast<u32x4_t*>(sa + lds_offset(row, ld_chunk)) = a_stage[j];
    }
    if constexpr (B_KMAJOR) {
#pragma unroll
      for (int j = 0; j < B_LOADS; ++j) {
        const int row = ld_row + j * 32;
        *reinterpret_cast<u32x4_t*>(sb + lds_offset(row, ld_chunk)) = b_stage[j];
      }
    } else {
#pragma unroll
      for (int q = 0; q < B_BLOCKS; ++q) {
        const int blk = tid + q * 256;
        if (blk < BN) {
          const int kc = blk / (BN / 8), ng = blk % (BN / 8);
          // 8x8 transpose of 16-bit elements: out[i] holds k = 0..7 for column i.
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            u32x4_t o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const uint32_t lo = b_stage[q * 8 + 2 * j][i >> 1];
              const uint32_t hi = b_stage[q * 8 + 2 * j + 1][i >> 1];
              o[j] = (i & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
            }
            const int row = ng * 8 + i;
            *reinterpret_cast<u32x4_t*>(sb + lds_offset(row, kc)) = o;
          }
        }
      }
    }
  };

  // ---- accumulators ---------------------------------------------------------------------
  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;  // which 8-wide K half of the 16-wide MFMA step

  auto compute_stage = [&](int buf) {
    const unsigned char* sa = smem + buf * STAGE_BYTES;
    const unsigned char* sb = sa + A_BYTES;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      u32x4_t af[TM], bf[TN];
      const int chunk = ks * 2 + frag_half;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm * WM + i * 32 + frag_row;
        af[i] = *reinterpret_cast<const u32x4_t*>(sa + lds_offset(row, chunk));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn * WN + j * 32 + frag_row;
        bf[j] = *reinterpret_cast<const u32x4_t*>(sb + lds_offset(row, chunk));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::run(af[i], bf[j], acc[i][j]);
    }
  };

  // ---- main loop ------------------------------------------------------------------------
  const int64_t k_tiles = (K + kBK - 1) / kBK;
  load_a(0);
  load_b(0);
  store_stage(0);
  __syncthreads();
  for (int64_t kt = 0; kt < k_tiles; ++kt) {
    const int buf = static_cast<int>(kt & 1);
    const bool more = kt + 1 < k_tiles;
    if (more) {
      load_a((kt + 1) * kBK);
      load_b((kt + 1) * kBK);
    }
    compute_stage(buf);
    if (more) store_stage(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue -------------------------------------------------------------------------
  // MFMA 32x32 result layout: lane holds column (lane & 31); register e holds row
  // 8*(e/4) + 4*(lane>>5) + (e&3).
  const T* __restrict__ bias = static_cast<const T*>(g.bias);
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int64_t col = n0 + wn * WN + j * 32 + (lane & 31);
    const bool col_ok = col < N;
    const float bv = (bias != nullptr && col_ok) ? to_f32(bias[col]) : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int64_t row_base = m0 + wm * WM + i * 32 + 4 * (lane >> 5);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t row = row_base + 8 * (e >> 2) + (e & 3);
        if (col_ok && row < M) {
          C[row * g.ldc + col] = finish<T, EPI>(acc[i][j][e] + bv);
        }
      }
    }
  }
}

template <typename T, int BM, int BN, bool B_KMAJOR, int EPI>
static int launch_mfma(const GemmArgs& base, int64_t batch, hipStream_t stream) {
  constexpr int SMEM = 2 * (BM + BN) * kLineBytes;
  static bool configured = false;
  auto kernel = gemm_mfma_kernel<T, BM, BN, B_KMAJOR, EPI>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    if (e != hipSuccess) return static_cast<int>(e);
    configured = true;
  }
  GemmArgs g = base;
  g.tiles_m = static_cast<int>((g.m + BM - 1) / BM);
  g.tiles_n = static_cast<int>((g.n + BN - 1) / BN);
  const int64_t tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (tiles >= (int64_t{1} << 31) || batch > 65535) return TMB_ERR_UNSUPPORTED;
  kernel<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(batch)), dim3(256), SMEM, stream>>>(g);
  return check_launch();
}

template <typename T, bool B_KMAJOR, int EPI>
static int mfma_pick_tile(const GemmArgs& g, int64_t batch, hipStream_t stream) {
  // Big tiles when they still fill the 256 CUs, otherwise the 128x128 tile.
  const int64_t big_tiles = ((g.m + 255) / 256) * ((g.n + 255) / 256) * batch;
  if (big_tiles >= 192) return launch_mfma<T, 256, 256, B_KMAJOR, EPI>(g, batch, stream);
  return launch_mfma<T, 128, 128, B_KMAJOR, EPI>(g, batch, stream);
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
      g.stride_b, g.stride_c, tiles_n);
  return check_launch();
}

static bool mfma_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b) {
  if (trans_a) return false;
  if (g.k % 8 != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0) return false;
  if (!aligned16(g.a) || !aligned16(g.b)) return false;
  if (batch > 1 && (g.stride_a % 8 != 0 || g.stride_b % 8 != 0)) return false;
  if (g.m < 1 || g.n < 1 || g.k < 8) return false;
  (void)trans_b;
  return true;
}

template <typename T, int EPI>
static int gemm_typed(const GemmArgs& g, int64_t batch, int trans_a, int trans_b, bool half,
                      hipStream_t stream) {
  if constexpr (!__is_same(T, float)) {
    if (half && mfma_eligible(g, batch, trans_a, trans_b)) {
      return trans_b ? mfma_pick_tile<T, true, EPI>(g, batch, stream)
                     : mfma_pick_tile<T, false, EPI>(g, batch, stream);
    }
  }
  return launch_simt<T, EPI>(g, batch, trans_a, trans_b, stream);
}

template <typename T>
static int gemm_epi(const GemmArgs& g, int64_t batch, int ta, int tb, int epilogue,
                    hipStream_t stream) {
  switch (epilogue) {
    case TMB_EPI_NONE: return gemm_typed<T, TMB_EPI_NONE>(g, batch, ta, tb, true, stream);
    case TMB_EPI_GELU_TANH: return gemm_typed<T, TMB_EPI_GELU_TANH>(g, batch, ta, tb, true, stream);
    case TMB_EPI_GELU_ERF: return gemm_typed<T, TMB_EPI_GELU_ERF>(g, batch, ta, tb, true, stream);
    default: return TMB_ERR_INVALID_ARGUMENT;
  }
}

// Fills C with epilogue(bias) (or zeros) when k == 0.
template <typename T, int EPI>
__global__ void gemm_k0_kernel(T* c, const T* bias, int64_t m, int64_t n, int64_t ldc,
                               int64_t stride_c) {
  T* cb = c + static_cast<int64_t>(blockIdx.y) * stride_c;
  const int64_t total = m * n;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / n, col = i - r * n;
    const float v = bias != nullptr ? to_f32(bias[col]) : 0.0f;
    cb[r * ldc + col] = finish<T, EPI>(v);
  }
}

}  // namespace tmb

extern "C" int tmb_gemm(void* c, const void* a, const void* b, const void* bias, int64_t batch,
                        int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc,
                        int64_t stride_a, int64_t stride_b, int64_t stride_c, int trans_a,
                        int trans_b, int dtype, int epilogue, void* stream) {
  using namespace tmb;
  if (batch < 0 || m < 0 || n < 0 || k < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (epilogue < TMB_EPI_NONE || epilogue > TMB_EPI_GELU_ERF) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F32 && dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
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
  GemmArgs g{c, a, b, bias, m, n, k, lda, ldb, ldc, stride_a, stride_b, stride_c, 0, 0};
  if (k == 0) {
    const unsigned blocks = static_cast<unsigned>((m * n + 255) / 256 > 4096 ? 4096 : (m * n + 255) / 256);
    dim3 grid(blocks, static_cast<unsigned>(batch));
#define TMB_K0(T)                                                                                   \
  switch (epilogue) {                                                                               \
    case TMB_EPI_NONE: gemm_k0_kernel<T, TMB_EPI_NONE><<<grid, 256, 0, s>>>((T*)c, (const T*)bias, m, n, ldc, stride_c); break; \
    case TMB_EPI_GELU_TANH: gemm_k0_kernel<T, TMB_EPI_GELU_TANH><<<grid, 256, 0, s>>>((T*)c, (const T*)bias, m, n, ldc, stride_c); break; \
    default: gemm_k0_kernel<T, TMB_EPI_GELU_ERF><<<grid, 256, 0, s>>>((T*)c, (const T*)bias, m, n, ldc, stride_c); break; \
  }
    if (dtype == TMB_F32) { TMB_K0(float) } else if (dtype == TMB_F16) { TMB_K0(f16_t) } else { TMB_K0(bf16_t) }
#undef TMB_K0
    return check_launch();
  }
  switch (dtype) {
    case TMB_F32: return gemm_epi<float>(g, batch, trans_a, trans_b, epilogue, s);
    case TMB_F16: return gemm_epi<f16_t>(g, batch, trans_a, trans_b, epilogue, s);
    default: return gemm_epi<bf16_t>(g, batch, trans_a, trans_b, epilogue, s);
  }
}
