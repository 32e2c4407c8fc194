// Row softmax / log-softmax for gfx950.
//
// Fast path: the whole row lives in registers (one HBM read + one HBM write per element).
// A row is covered by WPR cooperating waves; every lane owns VPL 16-byte vectors that are
// interleaved so that each wave-wide load instruction touches 1 KiB of consecutive memory.
// Reductions are DPP within a wave and a fixed-order LDS combine across the row's waves.
//
// Generic path: any alignment / any width, one 256-thread block per row, three passes
// (the second and third read come from L2 for rows that fit there).
//
// Arithmetic follows the reference CPU kernels (fp32 max, fp32 sum of exp(x-m), one cast):
// torch_mojo_backend/eager_kernels/nn_ops.mojo:428-455 and reduction_ops.mojo:874-895.
#include "tmb_common.h"

namespace tmb {

template <typename TIn, typename TOut, int WPR, int VPL, bool LOG, int BLOCK>
__global__ __launch_bounds__(BLOCK) void softmax_regs_kernel(TOut* __restrict__ out,
                                                             const TIn* __restrict__ in,
                                                             int64_t rows, int cols) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int ROWS_PER_BLOCK = WAVES / WPR;
  __shared__ float slot[WAVES];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int group = wave / WPR;
  const int wave_in_row = wave - group * WPR;
  int64_t row = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + group;
  const bool valid = row < rows;
  if (!valid) row = rows - 1;  // stay in lock-step with the block's barriers; stores are masked

  const int nvec = cols / EPV;
  const TIn* src = in + row * static_cast<int64_t>(cols);
  TOut* dst = out + row * static_cast<int64_t>(cols);

  float x[VPL][EPV];
  const float neg_inf = -__builtin_inff();
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    if (vi < nvec) {
      Vec16<TIn> t = load_vec16(src + static_cast<int64_t>(vi) * EPV);
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[v][e] = to_f32(t.v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[v][e] = neg_inf;
    }
  }

  float m = neg_inf;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) m = fmaxf(m, x[v][e]);
  m = wave_max(m);
  m = group_reduce(m, slot, wave, group * WPR, WPR, MaxOp{});

  float s = 0.0f;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float ex = exp_f32(x[v][e] - m);
      if (LOG) {
        x[v][e] = x[v][e] - m;
      } else {
        x[v][e] = ex;
      }
      s += ex;
    }
  s = wave_sum(s);
  s = group_reduce(s, slot, wave, group * WPR, WPR, SumOp{});

  if (LOG) {
    const float lg = logf(s);
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[v][e] -= lg;
  } else {
    const float inv = 1.0f / s;
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[v][e] *= inv;
  }

  if (valid) {
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const int vi = (v * WPR + wave_in_row) * kWave + lane;
      if (vi < nvec) store_converted<TOut, EPV>(dst + static_cast<int64_t>(vi) * EPV, x[v]);
    }
  }
}

// Any width / alignment. One block per row.
template <typename TIn, typename TOut, bool LOG>
__global__ __launch_bounds__(256) void softmax_generic_kernel(TOut* __restrict__ out,
                                                              const TIn* __restrict__ in,
                                                              int64_t rows, int64_t cols) {
  __shared__ float slot[4];
  const int wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const TIn* src = in + row * cols;
    TOut* dst = out + row * cols;
    float m = -__builtin_inff();
    for (int64_t j = threadIdx.x; j < cols; j += 256) m = fmaxf(m, to_f32(src[j]));
    m = wave_max(m);
    m = group_reduce(m, slot, wave, 0, 4, MaxOp{});
    float s = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += 256) s += exp_f32(to_f32(src[j]) - m);
    s = wave_sum(s);
    s = group_reduce(s, slot, wave, 0, 4, SumOp{});
    if (LOG) {
      const float lg = logf(s);
      for (int64_t j = threadIdx.x; j < cols; j += 256)
        dst[j] = from_f32<TOut>(to_f32(src[j]) - m - lg);
    } else {
      const float inv = 1.0f / s;
      for (int64_t j = threadIdx.x; j < cols; j += 256)
        dst[j] = from_f32<TOut>(exp_f32(to_f32(src[j]) - m) * inv);
    }
  }
}

template <typename TIn, typename TOut, bool LOG, int WPR, int VPL, int BLOCK>
static int launch_regs(TOut* out, const TIn* in, int64_t rows, int64_t cols, hipStream_t stream) {
  constexpr int ROWS_PER_BLOCK = (BLOCK / kWave) / WPR;
  const int64_t blocks = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  softmax_regs_kernel<TIn, TOut, WPR, VPL, LOG, BLOCK>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(BLOCK), 0, stream>>>(out, in, rows,
                                                                         static_cast<int>(cols));
  return check_launch();
}

template <typename TIn, typename TOut, bool LOG>
static int softmax_dispatch(TOut* out, const TIn* in, int64_t rows, int64_t cols,
                            hipStream_t stream) {
  constexpr int EPV = Vec16<TIn>::N;
  const bool vec_ok = (cols % EPV == 0) && aligned16(in) && aligned16(out) &&
                      rows < (int64_t{1} << 31);
  const int64_t nvec = cols / EPV;
  if (vec_ok && nvec <= 8192) {
    if (nvec <= 64) return launch_regs<TIn, TOut, LOG, 1, 1, 256>(out, in, rows, cols, stream);
    if (nvec <= 128) return launch_regs<TIn, TOut, LOG, 1, 2, 256>(out, in, rows, cols, stream);
    if (nvec <= 256) return launch_regs<TIn, TOut, LOG, 1, 4, 256>(out, in, rows, cols, stream);
    if (nvec <= 512) return launch_regs<TIn, TOut, LOG, 1, 8, 256>(out, in, rows, cols, stream);
    if (nvec <= 1024) return launch_regs<TIn, TOut, LOG, 4, 4, 256>(out, in, rows, cols, stream);
    if (nvec <= 2048) return launch_regs<TIn, TOut, LOG, 4, 8, 256>(out, in, rows, cols, stream);
    if (nvec <= 4096)
      return launch_regs<TIn, TOut, LOG, 16, 4, 1024>(out, in, rows, cols, stream);
    return launch_regs<TIn, TOut, LOG, 16, 8, 1024>(out, in, rows, cols, stream);
  }
  const int64_t blocks = rows < 65536 * 16 ? rows : 65536 * 16;
  softmax_generic_kernel<TIn, TOut, LOG>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(out, in, rows, cols);
  return check_launch();
}

template <bool LOG>
static int softmax_by_dtype(void* out, const void* in, int64_t rows, int64_t cols, int in_dtype,
                            int out_dtype, hipStream_t s) {
  if (in_dtype == TMB_F32 && out_dtype == TMB_F32)
    return softmax_dispatch<float, float, LOG>((float*)out, (const float*)in, rows, cols, s);
  if (in_dtype == TMB_F16 && out_dtype == TMB_F16)
    return softmax_dispatch<f16_t, f16_t, LOG>((f16_t*)out, (const f16_t*)in, rows, cols, s);
  if (in_dtype == TMB_BF16 && out_dtype == TMB_BF16)
    return softmax_dispatch<bf16_t, bf16_t, LOG>((bf16_t*)out, (const bf16_t*)in, rows, cols, s);
  if (in_dtype == TMB_F16 && out_dtype == TMB_F32)
    return softmax_dispatch<f16_t, float, LOG>((float*)out, (const f16_t*)in, rows, cols, s);
  if (in_dtype == TMB_BF16 && out_dtype == TMB_F32)
    return softmax_dispatch<bf16_t, float, LOG>((float*)out, (const bf16_t*)in, rows, cols, s);
  return TMB_ERR_UNSUPPORTED;
}

}  // namespace tmb

extern "C" int tmb_softmax_rows(void* out, const void* in, int64_t rows, int64_t cols,
                                int in_dtype, int out_dtype, int log_mode, void* stream) {
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return log_mode ? tmb::softmax_by_dtype<true>(out, in, rows, cols, in_dtype, out_dtype, s)
                  : tmb::softmax_by_dtype<false>(out, in, rows, cols, in_dtype, out_dtype, s);
}
