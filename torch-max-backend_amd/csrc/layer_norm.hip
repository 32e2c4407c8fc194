// Layer norm forward over the last dimension for gfx950.
//
// Fast path: the row is loaded once into registers (16-byte vectors), both statistics passes
// run on registers, the normalised row is written once. Statistics are the reference's two-pass
// form, in fp32: mean = sum(x)/cols; var = sum((x-mean)^2)/cols; rstd = 1/sqrt(var+eps)
// (torch_mojo_backend/eager_kernels/nn_ops.mojo:299-326). A row whose variance is NaN
// (it contains NaN or an infinity) reports NaN for the mean as well
// (normalization_forward_kernels.mojo:60-70).
#include "tmb_common.h"

namespace tmb {

template <typename T, int WPR, int VPL, int BLOCK>
__global__ __launch_bounds__(BLOCK) void layer_norm_regs_kernel(
    T* __restrict__ out, float* __restrict__ mean_out, float* __restrict__ rstd_out,
    const T* __restrict__ in, const T* __restrict__ gamma, const T* __restrict__ beta,
    int64_t rows, int cols, float eps) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int ROWS_PER_BLOCK = WAVES / WPR;
  __shared__ float slot[WAVES];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int group = wave / WPR;
  const int wave_in_row = wave - group * WPR;
  int64_t row = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + group;
  const bool valid = row < rows;
  if (!valid) row = rows - 1;

  const int nvec = cols / EPV;
  const T* src = in + row * static_cast<int64_t>(cols);
  T* dst = out + row * static_cast<int64_t>(cols);

  float x[VPL][EPV];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    if (vi < nvec) {
      Vec16<T> t = load_vec16(src + static_cast<int64_t>(vi) * EPV);
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[v][e] = to_f32(t.v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[v][e] = 0.0f;
    }
  }

  float s = 0.0f;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) s += x[v][e];
  s = wave_sum(s);
  s = group_reduce(s, slot, wave, group * WPR, WPR, SumOp{});
  float mean = s / static_cast<float>(cols);

  float q = 0.0f;
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    if (vi < nvec) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float d = x[v][e] - mean;
        x[v][e] = d;
        q += d * d;
      }
    }
  }
  q = wave_sum(q);
  q = group_reduce(q, slot, wave, group * WPR, WPR, SumOp{});
  const float var = q / static_cast<float>(cols);
  const float rstd = 1.0f / sqrtf(var + eps);
  if (var != var) mean = var;

  if (valid) {
    if (wave_in_row == 0 && lane == 0) {
      if (mean_out) mean_out[row] = mean;
      if (rstd_out) rstd_out[row] = rstd;
    }
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const int vi = (v * WPR + wave_in_row) * kWave + lane;
      if (vi < nvec) {
        float y[EPV];
        if (gamma != nullptr) {
          Vec16<T> g = load_vec16(gamma + static_cast<int64_t>(vi) * EPV);
#pragma unroll
          for (int e = 0; e < EPV; ++e) y[e] = x[v][e] * rstd * to_f32(g.v[e]);
        } else {
#pragma unroll
          for (int e = 0; e < EPV; ++e) y[e] = x[v][e] * rstd;
        }
        if (beta != nullptr) {
          Vec16<T> b = load_vec16(beta + static_cast<int64_t>(vi) * EPV);
#pragma unroll
          for (int e = 0; e < EPV; ++e) y[e] += to_f32(b.v[e]);
        }
        store_converted<T, EPV>(dst + static_cast<int64_t>(vi) * EPV, y);
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void layer_norm_generic_kernel(
    T* __restrict__ out, float* __restrict__ mean_out, float* __restrict__ rstd_out,
    const T* __restrict__ in, const T* __restrict__ gamma, const T* __restrict__ beta,
    int64_t rows, int64_t cols, float eps) {
  __shared__ float slot[4];
  const int wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* src = in + row * cols;
    T* dst = out + row * cols;
    float s = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += 256) s += to_f32(src[j]);
    s = wave_sum(s);
    s = group_reduce(s, slot, wave, 0, 4, SumOp{});
    float mean = s / static_cast<float>(cols);
    float q = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += 256) {
      const float d = to_f32(src[j]) - mean;
      q += d * d;
    }
    q = wave_sum(q);
    q = group_reduce(q, slot, wave, 0, 4, SumOp{});
    const float var = q / static_cast<float>(cols);
    const float rstd = 1.0f / sqrtf(var + eps);
    const float center = mean;
    if (var != var) mean = var;
    if (threadIdx.x == 0) {
      if (mean_out) mean_out[row] = mean;
      if (rstd_out) rstd_out[row] = rstd;
    }
    for (int64_t j = threadIdx.x; j < cols; j += 256) {
      float y = (to_f32(src[j]) - center) * rstd;
      if (gamma != nullptr) y *= to_f32(gamma[j]);
      if (beta != nullptr) y += to_f32(beta[j]);
      dst[j] = from_f32<T>(y);
    }
  }
}

template <typename T, int WPR, int VPL, int BLOCK>
static int launch_ln(T* out, float* mean, float* rstd, const T* x, const T* g, const T* b,
                     int64_t rows, int64_t cols, float eps, hipStream_t stream) {
  constexpr int ROWS_PER_BLOCK = (BLOCK / kWave) / WPR;
  const int64_t blocks = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  layer_norm_regs_kernel<T, WPR, VPL, BLOCK>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(BLOCK), 0, stream>>>(
          out, mean, rstd, x, g, b, rows, static_cast<int>(cols), eps);
  return check_launch();
}

template <typename T>
static int layer_norm_dispatch(void* out_, float* mean, float* rstd, const void* x_,
                               const void* g_, const void* b_, int64_t rows, int64_t cols,
                               float eps, hipStream_t stream) {
  T* out = static_cast<T*>(out_);
  const T* x = static_cast<const T*>(x_);
  const T* g = static_cast<const T*>(g_);
  const T* b = static_cast<const T*>(b_);
  constexpr int EPV = Vec16<T>::N;
  const bool vec_ok = (cols % EPV == 0) && aligned16(x) && aligned16(out) &&
                      (g == nullptr || aligned16(g)) && (b == nullptr || aligned16(b)) &&
                      rows < (int64_t{1} << 31);
  const int64_t nvec = cols / EPV;
  if (vec_ok && nvec <= 8192) {
    if (nvec <= 64) return launch_ln<T, 1, 1, 256>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    if (nvec <= 128) return launch_ln<T, 1, 2, 256>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    if (nvec <= 256) return launch_ln<T, 1, 4, 256>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    if (nvec <= 512) return launch_ln<T, 1, 8, 256>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    if (nvec <= 1024) return launch_ln<T, 4, 4, 256>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    if (nvec <= 2048) return launch_ln<T, 4, 8, 256>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    if (nvec <= 4096) return launch_ln<T, 16, 4, 1024>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
    return launch_ln<T, 16, 8, 1024>(out, mean, rstd, x, g, b, rows, cols, eps, stream);
  }
  const int64_t blocks = rows < 65536 * 16 ? rows : 65536 * 16;
  layer_norm_generic_kernel<T><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(
      out, mean, rstd, x, g, b, rows, cols, eps);
  return check_launch();
}

}  // namespace tmb

extern "C" int tmb_layer_norm_rows(void* out, float* mean, float* rstd, const void* x,
                                   const void* gamma, const void* beta, int64_t rows,
                                   int64_t cols, double eps, int dtype, void* stream) {
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (out == nullptr || x == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float e = static_cast<float>(eps);
  switch (dtype) {
    case TMB_F32:
      return tmb::layer_norm_dispatch<float>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
    case TMB_F16:
      return tmb::layer_norm_dispatch<tmb::f16_t>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
    case TMB_BF16:
      return tmb::layer_norm_dispatch<tmb::bf16_t>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
    default:
      return TMB_ERR_UNSUPPORTED;
  }
}
