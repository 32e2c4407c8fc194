// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32: true fp32 products, fp32 accumulation).
//
// One workgroup of 2 x 2 waves owns a 128 x 128 tile of C, each wave a 64 x 64 quarter (2 x 2
// MFMA tiles, 64 accumulator registers). K is walked in stages of 16: stage s+1 travels from
// global memory into registers (two 16-byte loads per operand and thread) while stage s is
// multiplied out of LDS, then the registers go to the other LDS buffer and one barrier closes the
// stage. An fp32 MFMA takes 64 cycles for two 4-byte operands per lane, so LDS bandwidth is far
// from mattering; the layouts below only keep the 16-byte stores aligned.
//
// LDS layouts: an operand stored with K contiguous (A [M, K], B [N, K]) is kept [row][16 + 4];
// an operand stored with its M or N extent contiguous (A [K, M], B [K, N]) is kept [16][128 + 4].
//
// As in the 16-bit kernels the MFMA gets the B fragment first, so a lane ends up with one row m
// of C and four consecutive columns per register quad: 16-byte stores after bias and epilogue.
#pragma once

#include "gemm_mfma.h"

namespace tmb {

constexpr int kF32BM = 128, kF32BN = 128, kF32BK = 16;
constexpr int kF32PitchK = kF32BK + 4;    // floats per tile row, K contiguous
constexpr int kF32PitchMN = 128 + 4;      // floats per k line, M / N contiguous

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// One operand's share of a stage: two 16-byte chunks per thread.
template <bool K_CONTIGUOUS>
struct F32Stage {
  f32x4_t v[2];

  // base: first element of the operand for this batch. `row0`: first tile row (m or n) of the
  // tile, `rows`: the operand's extent in that direction, `ld`: leading dimension in floats.
  __device__ __forceinline__ void load(const float* __restrict__ base, int64_t ld, int64_t row0,
                                       int64_t rows, int64_t k0, int64_t K, int tid) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = tid + 256 * i;
      const f32x4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (K_CONTIGUOUS) {
        const int r = idx >> 2, kc = idx & 3;
        int64_t row = row0 + r;
        row = row < rows ? row : rows - 1;  // rows past the edge are computed and never stored
        const int64_t gk = k0 + 4 * kc;
        v[i] = gk < K ? *reinterpret_cast<const f32x4_t*>(base + row * ld + gk) : zero;
      } else {
        const int kr = idx >> 5, c4 = idx & 31;
        const int64_t gk = k0 + kr, col = row0 + 4 * c4;
        v[i] = (gk < K && col < rows) ? *reinterpret_cast<const f32x4_t*>(base + gk * ld + col)
                                      : zero;
      }
    }
  }

  __device__ __forceinline__ void store(float* __restrict__ tile, int tid) const {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = tid + 256 * i;
      if constexpr (K_CONTIGUOUS) {
        *reinterpret_cast<f32x4_t*>(tile + (idx >> 2) * kF32PitchK + 4 * (idx & 3)) = v[i];
      } else {
        *reinterpret_cast<f32x4_t*>(tile + (idx >> 5) * kF32PitchMN + 4 * (idx & 31)) = v[i];
      }
    }
  }

  // Element (row r of the tile, k) of the staged tile.
  static __device__ __forceinline__ float at(const float* __restrict__ tile, int r, int k) {
    if constexpr (K_CONTIGUOUS) return tile[r * kF32PitchK + k];
    else return tile[k * kF32PitchMN + r];
  }

  static constexpr int kFloats = K_CONTIGUOUS ? 128 * kF32PitchK : kF32BK * kF32PitchMN;
};

template <int EPI, bool A_MMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const GemmArgs g) {
  using StageA = F32Stage<!A_MMAJOR>;
  using StageB = F32Stage<B_KMAJOR>;
  constexpr int kBuf = StageA::kFloats + StageB::kFloats;
  __shared__ __align__(16) float lds[2 * kBuf];

  int tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t batch = blockIdx.y;
  const float* __restrict__ A = static_cast<const float*>(g.a) + batch * g.stride_a;
  const float* __restrict__ B = static_cast<const float*>(g.b) + batch * g.stride_b;
  float* __restrict__ C = static_cast<float*>(g.c) + batch * g.stride_c;
  const int64_t m0 = static_cast<int64_t>(tm) * kF32BM, n0 = static_cast<int64_t>(tn) * kF32BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 31, lk = lane >> 5;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  StageA sa;
  StageB sb;
  const int64_t stages = (g.k + kF32BK - 1) / kF32BK;
  sa.load(A, g.lda, m0, g.m, 0, g.k, tid);
  sb.load(B, g.ldb, n0, g.n, 0, g.k, tid);
  sa.store(lds, tid);
  sb.store(lds + StageA::kFloats, tid);
  __syncthreads();

  for (int64_t s = 0; s < stages; ++s) {
    const float* __restrict__ ta = lds + (s & 1) * kBuf;
    const float* __restrict__ tb = ta + StageA::kFloats;
    const bool more = s + 1 < stages;
    if (more) {
      sa.load(A, g.lda, m0, g.m, (s + 1) * kF32BK, g.k, tid);
      sb.load(B, g.ldb, n0, g.n, (s + 1) * kF32BK, g.k, tid);
    }
#pragma unroll
    for (int ks = 0; ks < kF32BK / 2; ++ks) {
      float af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = StageA::at(ta, wm * 64 + i * 32 + lr, 2 * ks + lk);
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = StageB::at(tb, wn * 64 + j * 32 + lr, 2 * ks + lk);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (more) {
      float* __restrict__ next = lds + ((s + 1) & 1) * kBuf;
      sa.store(next, tid);
      sb.store(next + StageA::kFloats, tid);
    }
    __syncthreads();
  }

  // Lane holds row lr of each 32 x 32 result and columns 8q + 4 * lk + {0..3}.
  const float* __restrict__ bias = static_cast<const float*>(g.bias);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int64_t row = m0 + wm * 64 + i * 32 + lr;
    if (row >= g.m) continue;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = n0 + wn * 64 + j * 32 + 8 * q + 4 * lk;
        if (col >= g.n) continue;
        float* dst = C + row * g.ldc + col;
        float out[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = acc[i][j][4 * q + e];
          if (bias != nullptr && col + e < g.n) v += bias[col + e];
          out[e] = finish<float, EPI>(v, false);
        }
        if (col + 4 <= g.n) {
          const f32x4_unaligned_t v = {out[0], out[1], out[2], out[3]};
          if (g.stream_c) __builtin_nontemporal_store(v, reinterpret_cast<f32x4_unaligned_t*>(dst));
          else *reinterpret_cast<f32x4_unaligned_t*>(dst) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (col + e < g.n) dst[e] = out[e];
        }
      }
  }
}

// 16-byte loads need whole, aligned chunks along each operand's contiguous direction.
static inline bool f32_mfma_eligible(const GemmArgs& g, int64_t batch, int trans_a, int trans_b) {
  if (g.m < 1 || g.n < 1 || g.k < 1) return false;
  if (g.lda % 4 != 0 || g.ldb % 4 != 0) return false;
  if ((reinterpret_cast<uintptr_t>(g.a) & 15) != 0 || (reinterpret_cast<uintptr_t>(g.b) & 15) != 0)
    return false;
  if (batch > 1 && (g.stride_a % 4 != 0 || g.stride_b % 4 != 0)) return false;
  if (trans_a ? g.m % 4 != 0 : g.k % 4 != 0) return false;
  if (trans_b ? g.k % 4 != 0 : g.n % 4 != 0) return false;
  const int64_t tiles_m = (g.m + kF32BM - 1) / kF32BM, tiles_n = (g.n + kF32BN - 1) / kF32BN;
  return tiles_m * tiles_n < (int64_t{1} << 30) && tiles_m < (1 << 24) && tiles_n < (1 << 24);
}

template <int EPI>
static int launch_f32_mfma(GemmArgs g, int64_t batch, int trans_a, int trans_b,
                           hipStream_t stream) {
  g.tiles_m = static_cast<int>((g.m + kF32BM - 1) / kF32BM);
  g.tiles_n = static_cast<int>((g.n + kF32BN - 1) / kF32BN);
  g.stream_c = batch * g.m * g.n * 4 > (int64_t{256} << 20);
  const dim3 grid(static_cast<unsigned>(g.tiles_m * g.tiles_n), static_cast<unsigned>(batch));
  if (trans_a) {
    if (trans_b) gemm_f32_mfma_kernel<EPI, true, true><<<grid, 256, 0, stream>>>(g);
    else gemm_f32_mfma_kernel<EPI, true, false><<<grid, 256, 0, stream>>>(g);
  } else {
    if (trans_b) gemm_f32_mfma_kernel<EPI, false, true><<<grid, 256, 0, stream>>>(g);
    else gemm_f32_mfma_kernel<EPI, false, false><<<grid, 256, 0, stream>>>(g);
  }
  return check_launch();
}

}  // namespace tmb
