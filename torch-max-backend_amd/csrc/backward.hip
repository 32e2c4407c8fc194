// Backward twins of the hot ops for gfx950: GELU, softmax / log-softmax and layer norm.
//
// All of them are bound by HBM traffic and use the forward kernels' layout: a row lives in the
// registers of WPR cooperating waves (VPL 16-byte vectors per lane and input stream), loads are
// non-temporal (every element is read once), reductions are DPP inside a wave and a fixed-order
// LDS combine across the waves of a row, arithmetic is fp32 with one cast on store.
//
// Formulas follow the reference:
//   gelu_backward          eager_kernels/activation_backward_ops.mojo:50-73
//   log_softmax backward   aten_functions.py:788-833  (grad - exp(out) * sum(grad))
//   softmax backward       out * (grad - sum(grad * out))
//   layer norm backward    eager_kernels/aten_fast.py:2797-2913 (LayerNormBackwardF32):
//                          dx = rstd * (g dy - mean(g dy) - xhat mean(g dy xhat)),
//                          dgamma = sum_rows dy xhat, dbeta = sum_rows dy
#include <type_traits>

#include "tmb_common.h"

namespace tmb {

// ---------------------------------------------------------------------------
// GELU backward
// ---------------------------------------------------------------------------
__device__ __forceinline__ float gelu_grad_erf(float x, float g) {
#pragma clang fp contract(off)
  const float cdf = 0.5f * (1.0f + erff(x * 0.7071067811865476f));
  const float pdf = 0.3989422804014327f * exp_f32(-0.5f * (x * x));
  return g * (cdf + x * pdf);
}
__device__ __forceinline__ float gelu_grad_tanh(float x, float g) {
#pragma clang fp contract(off)
  constexpr float kBeta = 0.7978845608028654f, kKappa = 0.044715f;
  const float x2 = x * x;
  const float inner = kBeta * (x + kKappa * (x2 * x));
  // tanh(u) = 1 - 2 / (1 + e^(2u)); e^(2u) overflows to +inf (t = 1) and underflows to 0 (t = -1)
  const float e = __builtin_amdgcn_exp2f(inner * 2.8853900817779268f);
  const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
  const float d = 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * kBeta * (1.0f + 3.0f * kKappa * x2);
  return g * d;
}

template <typename T, bool TANH>
__global__ __launch_bounds__(256) void gelu_backward_kernel(T* __restrict__ out,
                                                            const T* __restrict__ grad,
                                                            const T* __restrict__ in,
                                                            int64_t numel, int64_t nvec) {
  constexpr int EPV = Vec16<T>::N;
  const bool stream = numel * static_cast<int64_t>(3 * sizeof(T)) >= kStreamStoreBytes;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid < nvec) {
    const Vec16<T> xv = load_vec16_stream(in + tid * EPV);
    const Vec16<T> gv = load_vec16_stream(grad + tid * EPV);
    float y[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float x = to_f32(xv.v[e]), g = to_f32(gv.v[e]);
      y[e] = TANH ? gelu_grad_tanh(x, g) : gelu_grad_erf(x, g);
    }
    store_converted_hinted<T, EPV>(out + tid * EPV, y, stream);
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = nvec * EPV + tid; i < numel; i += stride) {
    const float x = to_f32(in[i]), g = to_f32(grad[i]);
    out[i] = from_f32<T>(TANH ? gelu_grad_tanh(x, g) : gelu_grad_erf(x, g));
  }
}

template <typename T>
static int launch_gelu_backward(void* out_, const void* grad_, const void* in_, int64_t numel,
                                int tanh_mode, hipStream_t s) {
  T* out = static_cast<T*>(out_);
  const T* grad = static_cast<const T*>(grad_);
  const T* in = static_cast<const T*>(in_);
  constexpr int EPV = Vec16<T>::N;
  const int64_t nvec = (aligned16(in) && aligned16(out) && aligned16(grad)) ? numel / EPV : 0;
  const int64_t work = nvec > 0 ? nvec : numel;
  int64_t blocks = (work + 255) / 256;
  if (blocks > (int64_t{1} << 30)) blocks = int64_t{1} << 30;
  if (blocks < 1) blocks = 1;
  if (tanh_mode)
    gelu_backward_kernel<T, true><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(out, grad, in, numel, nvec);
  else
    gelu_backward_kernel<T, false><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(out, grad, in, numel, nvec);
  return check_launch();
}

// ---------------------------------------------------------------------------
// softmax / log-softmax backward (from the saved output)
// ---------------------------------------------------------------------------
template <typename T, int WPR, int VPL, bool LOG, int BLOCK>
__global__ __launch_bounds__(BLOCK) void softmax_backward_regs_kernel(T* __restrict__ gin,
                                                                      const T* __restrict__ gout,
                                                                      const T* __restrict__ y,
                                                                      int64_t rows, int cols) {
  constexpr int EPV = Vec16<T>::N;
  const bool stream = rows * cols * static_cast<int64_t>(3 * sizeof(T)) >= kStreamStoreBytes;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int GROUPS = WAVES / WPR;
  __shared__ float slot[WAVES];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int group = wave / WPR, wave_in_row = wave - group * WPR;
  const int nvec = cols / EPV;
  int64_t row = static_cast<int64_t>(blockIdx.x) * GROUPS + group;
  const bool live = row < rows;
  if (!live) row = rows - 1;  // keep lock-step for the barriers; nothing is stored
  const T* gsrc = gout + row * static_cast<int64_t>(cols);
  const T* ysrc = y + row * static_cast<int64_t>(cols);

  float g[VPL][EPV], o[VPL][EPV];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    const bool ok = vi < nvec;
    const int64_t at = static_cast<int64_t>(ok ? vi : 0) * EPV;
    const Vec16<T> gv = load_vec16_stream(gsrc + at);
    const Vec16<T> yv = load_vec16_stream(ysrc + at);
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      g[v][e] = ok ? to_f32(gv.v[e]) : 0.0f;
      o[v][e] = ok ? to_f32(yv.v[e]) : (LOG ? -__builtin_inff() : 0.0f);
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) s += LOG ? g[v][e] : g[v][e] * o[v][e];
  s = wave_sum(s);
  s = group_reduce(s, slot, wave, group * WPR, WPR, SumOp{});
  if (!live) return;
  T* dst = gin + row * static_cast<int64_t>(cols);
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    float r[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e)
      r[e] = LOG ? g[v][e] - exp_for<T>(o[v][e]) * s : o[v][e] * (g[v][e] - s);
    if (vi < nvec) store_converted_hinted<T, EPV>(dst + static_cast<int64_t>(vi) * EPV, r, stream);
  }
}

// Long rows of any width at any element alignment (the gradient of a [rows, 50257] log-softmax):
// one 1024-thread workgroup per row, both operands held in registers in their storage type (a
// lane's share of a 16-bit row of 65536 columns is 2 x 32 registers); every element is read once
// and written once. PEEL: the three rows sit at the same offset from a 16-byte boundary, the
// vectors start at the first boundary inside the row and every vector access is aligned; the
// elements in front of the first vector and after the last one are held one each by the first
// lanes of wave 0. Without PEEL the vectors start with the row and the accesses are unaligned.
template <typename T, int VPL, bool LOG, bool PEEL>
__global__ __launch_bounds__(1024) void softmax_backward_long_rows_kernel(
    T* __restrict__ gin, const T* __restrict__ gout, const T* __restrict__ y, int cols) {
  constexpr int EPV = Vec16<T>::N;
  const bool stream = static_cast<int64_t>(gridDim.x) * cols * static_cast<int64_t>(3 * sizeof(T)) >= kStreamStoreBytes;
  constexpr int WAVES = 16;
  __shared__ float slot[WAVES];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * cols;
  const T* gsrc = gout + base;
  const T* ysrc = y + base;
  T* dst = gin + base;
  int head = 0;
  if constexpr (PEEL) {
    const int off = static_cast<int>((reinterpret_cast<uintptr_t>(gsrc) & 15u) / sizeof(T));
    head = off ? EPV - off : 0;
  }
  const int nvec = (cols - head) / EPV;
  const int tail_from = head + nvec * EPV;
  int edge = -1;
  if (wave == 0 && lane < 8 && lane < head) edge = lane;
  if (wave == 0 && lane >= 8 && lane < 16 && tail_from + lane - 8 < cols) edge = tail_from + lane - 8;

  // LATE_Y (sixteen vectors per lane: fp32 rows beyond 32768 columns): the row sum of the log form
  // needs the gradient only, so the saved output is fetched after the reduction, vector by vector
  constexpr bool LATE_Y = VPL > 8;
  static_assert(!LATE_Y || LOG, "the plain form needs both operands for its row sum");
  Vec16<T> gv[VPL], yv[LATE_Y ? 1 : VPL];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WAVES + wave) * kWave + lane;
    const unsigned at = static_cast<unsigned>(head + (vi < nvec ? vi : 0) * EPV);
    if constexpr (PEEL) {
      gv[v] = load_vec16_stream(gsrc + at);
      if constexpr (!LATE_Y) yv[v] = load_vec16_stream(ysrc + at);
    } else {
      gv[v] = load_vec16_unaligned(gsrc + at);
      if constexpr (!LATE_Y) yv[v] = load_vec16_unaligned(ysrc + at);
    }
  }
  float gt = 0.0f, yt = 0.0f;
  if (edge >= 0) {
    gt = to_f32(gsrc[edge]);
    yt = to_f32(ysrc[edge]);
  }
  float s = LOG ? gt : gt * yt;
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WAVES + wave) * kWave + lane;
    float part = 0.0f;
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      if constexpr (LOG) {
        part += to_f32(gv[v].v[e]);
      } else {
        part += to_f32(gv[v].v[e]) * to_f32(yv[v].v[e]);
      }
    }
    s += vi < nvec ? part : 0.0f;  // an empty slot holds a copy of vector 0
  }
  s = wave_sum(s);
  s = group_reduce(s, slot, wave, 0, WAVES, SumOp{});
  constexpr int CHUNK = LATE_Y ? 2 : VPL;  // vectors of the saved output in flight at a time
#pragma unroll
  for (int v0 = 0; v0 < VPL; v0 += CHUNK) {
    Vec16<T> late[CHUNK];
    if constexpr (LATE_Y) {
#pragma unroll
      for (int c = 0; c < CHUNK; ++c) {
        const int vi = ((v0 + c) * WAVES + wave) * kWave + lane;
        const unsigned at = static_cast<unsigned>(head + (vi < nvec ? vi : 0) * EPV);
        if constexpr (PEEL) {
          late[c] = load_vec16_stream(ysrc + at);
        } else {
          late[c] = load_vec16_unaligned(ysrc + at);
        }
      }
    }
#pragma unroll
    for (int c = 0; c < CHUNK; ++c) {
      const int v = v0 + c;
      const int vi = (v * WAVES + wave) * kWave + lane;
      float r[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float g = to_f32(gv[v].v[e]);
        const float o = to_f32(LATE_Y ? late[c].v[e] : yv[LATE_Y ? 0 : v].v[e]);
        r[e] = LOG ? g - exp_for<T>(o) * s : o * (g - s);
      }
      if (vi < nvec) {
        T* at = dst + static_cast<unsigned>(head + vi * EPV);
        if constexpr (PEEL) {
          store_converted_hinted<T, EPV>(at, r, stream);
        } else {
          store_converted_unaligned<T, EPV>(at, r);
        }
      }
    }
  }
  if (edge >= 0) dst[edge] = from_f32<T>(LOG ? gt - exp_for<T>(yt) * s : yt * (gt - s));
}

template <typename T, int VPL, bool LOG>
static int launch_softmax_backward_long_rows(T* gin, const T* gout, const T* y, int64_t rows,
                                             int64_t cols, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(rows)), block(1024);
  const int c = static_cast<int>(cols);
  const uintptr_t a = reinterpret_cast<uintptr_t>(gin) & 15u;
  if (a == (reinterpret_cast<uintptr_t>(gout) & 15u) && a == (reinterpret_cast<uintptr_t>(y) & 15u)) {
    softmax_backward_long_rows_kernel<T, VPL, LOG, true><<<grid, block, 0, stream>>>(gin, gout, y, c);
  } else {
    softmax_backward_long_rows_kernel<T, VPL, LOG, false><<<grid, block, 0, stream>>>(gin, gout, y, c);
  }
  return check_launch();
}

// Any width / alignment: one workgroup per row, the row is read twice (the second time from L2).
template <typename T, bool LOG>
__global__ __launch_bounds__(256) void softmax_backward_generic_kernel(T* __restrict__ gin,
                                                                       const T* __restrict__ gout,
                                                                       const T* __restrict__ y,
                                                                       int64_t rows, int64_t cols) {
  __shared__ float slot[4];
  const int wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* gsrc = gout + row * cols;
    const T* ysrc = y + row * cols;
    float s = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += 256)
      s += LOG ? to_f32(gsrc[j]) : to_f32(gsrc[j]) * to_f32(ysrc[j]);
    s = wave_sum(s);
    s = group_reduce(s, slot, wave, 0, 4, SumOp{});
    for (int64_t j = threadIdx.x; j < cols; j += 256) {
      const float g = to_f32(gsrc[j]), o = to_f32(ysrc[j]);
      gin[row * cols + j] = from_f32<T>(LOG ? g - exp_for<T>(o) * s : o * (g - s));
    }
  }
}

template <typename T, bool LOG>
static int softmax_backward_dispatch(void* gin_, const void* gout_, const void* y_, int64_t rows,
                                     int64_t cols, hipStream_t stream) {
  T* gin = static_cast<T*>(gin_);
  const T* gout = static_cast<const T*>(gout_);
  const T* y = static_cast<const T*>(y_);
  constexpr int EPV = Vec16<T>::N;
  const bool vec_ok = cols % EPV == 0 && aligned16(gin) && aligned16(gout) && aligned16(y) &&
                      rows < (int64_t{1} << 31);
  const int64_t nvec = cols / EPV;
#define TMB_SB(WPR, VPL, BLOCK)                                                                   \
  {                                                                                               \
    constexpr int RPB = (BLOCK / kWave) / WPR;                                                    \
    const int64_t blocks = (rows + RPB - 1) / RPB;                                                \
    softmax_backward_regs_kernel<T, WPR, VPL, LOG, BLOCK>                                         \
        <<<dim3(static_cast<unsigned>(blocks)), dim3(BLOCK), 0, stream>>>(gin, gout, y, rows,     \
                                                                         static_cast<int>(cols)); \
    return check_launch();                                                                        \
  }
  if (vec_ok && nvec <= 16 * 64 * 4) {
    // same geometry rule as the forward kernel: light waves, up to 16 per row
    if (nvec <= 64) TMB_SB(1, 1, 256)
    if (nvec <= 128) TMB_SB(2, 1, 256)
    if (nvec <= 256) TMB_SB(2, 2, 256)
    if (nvec <= 512) TMB_SB(4, 2, 256)
    if (nvec <= 1024) TMB_SB(8, 2, 512)
    if (nvec <= 2048) TMB_SB(16, 2, 1024)
    TMB_SB(16, 4, 1024)
  }
#undef TMB_SB
  // ragged or unaligned rows long enough to occupy a 1024-thread workgroup (eight 16-bit vector
  // pairs per lane plus the products of the plain softmax form do not fit the 128 registers of
  // such a workgroup: that form stops at four)
  const int64_t max_vec = 1024 * ((!LOG && sizeof(T) == 2) ? 4 : 8);
  if (cols >= 4096 && cols / EPV <= max_vec && rows < (int64_t{1} << 31)) {
    if (cols / EPV <= 1024 * 2)
      return launch_softmax_backward_long_rows<T, 2, LOG>(gin, gout, y, rows, cols, stream);
    if (cols / EPV <= 1024 * 4)
      return launch_softmax_backward_long_rows<T, 4, LOG>(gin, gout, y, rows, cols, stream);
    if constexpr (LOG || sizeof(T) != 2)
      return launch_softmax_backward_long_rows<T, 8, LOG>(gin, gout, y, rows, cols, stream);
  }
  if constexpr (LOG && sizeof(T) == 4) {  // fp32 rows of up to 65536 columns (a vocabulary)
    if (cols >= 4096 && cols / EPV <= 1024 * 16 && rows < (int64_t{1} << 31))
      return launch_softmax_backward_long_rows<T, 16, LOG>(gin, gout, y, rows, cols, stream);
  }
  const int64_t blocks = rows < 65536 * 16 ? rows : 65536 * 16;
  softmax_backward_generic_kernel<T, LOG>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(gin, gout, y, rows, cols);
  return check_launch();
}

// ---------------------------------------------------------------------------
// layer norm backward: grad_input
// ---------------------------------------------------------------------------
// rstd * (g dy - mean(g dy) - xhat * mean(g dy xhat)) with b1 = -rstd * mean(g dy) and
// b2 = -rstd * mean(g dy xhat): two multiply-adds per element.
__device__ __forceinline__ float grad_input_of(float gd, float xh, float rs, float b1, float b2) {
  return __builtin_fmaf(gd, rs, __builtin_fmaf(xh, b2, b1));
}

// The vector, or zeros: four selects for the 16 bytes instead of one per element.
template <typename T>
__device__ __forceinline__ Vec16<T> keep_if(const Vec16<T>& v, bool keep) {
  const raw16_t zero = {0u, 0u, 0u, 0u};
  const raw16_t r = keep ? __builtin_bit_cast(raw16_t, v) : zero;
  return __builtin_bit_cast(Vec16<T>, r);
}

template <typename T, int WPR, int VPL, int BLOCK>
__global__ __launch_bounds__(BLOCK) void layer_norm_backward_dx_kernel(
    T* __restrict__ dx, const T* __restrict__ dy, const T* __restrict__ x,
    const float* __restrict__ mean, const float* __restrict__ rstd, const T* __restrict__ gamma,
    int64_t rows, int cols) {
  constexpr int EPV = Vec16<T>::N;
  const bool stream = rows * cols * static_cast<int64_t>(3 * sizeof(T)) >= kStreamStoreBytes;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int GROUPS = WAVES / WPR;
  __shared__ float slot[WAVES];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int group = wave / WPR, wave_in_row = wave - group * WPR;
  const int nvec = cols / EPV;
  const float inv_n = 1.0f / static_cast<float>(cols);
  int64_t row = static_cast<int64_t>(blockIdx.x) * GROUPS + group;
  const bool live = row < rows;
  if (!live) row = rows - 1;
  const T* dsrc = dy + row * static_cast<int64_t>(cols);
  const T* xsrc = x + row * static_cast<int64_t>(cols);
  const float mu = mean[row], rs = rstd[row];

  float gd[VPL][EPV], xh[VPL][EPV];  // gamma*dy and xhat
  float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    const bool ok = vi < nvec;
    const int64_t at = static_cast<int64_t>(ok ? vi : 0) * EPV;
    const Vec16<T> dv = load_vec16_stream(dsrc + at);
    const Vec16<T> xv = load_vec16_stream(xsrc + at);
    Vec16<T> gv;
    if (gamma != nullptr) gv = load_vec16(gamma + at);
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float d = to_f32(dv.v[e]) * (gamma != nullptr ? to_f32(gv.v[e]) : 1.0f);
      gd[v][e] = ok ? d : 0.0f;
      xh[v][e] = ok ? (to_f32(xv.v[e]) - mu) * rs : 0.0f;
      s1 += gd[v][e];
      s2 += gd[v][e] * xh[v][e];
    }
  }
  s1 = wave_sum(s1);
  s1 = group_reduce(s1, slot, wave, group * WPR, WPR, SumOp{});
  s2 = wave_sum(s2);
  s2 = group_reduce(s2, slot, wave, group * WPR, WPR, SumOp{});
  if (!live) return;
  const float b1 = -rs * (s1 * inv_n), b2 = -rs * (s2 * inv_n);
  T* dst = dx + row * static_cast<int64_t>(cols);
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    float r[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) r[e] = grad_input_of(gd[v][e], xh[v][e], rs, b1, b2);
    if (vi < nvec) store_converted_hinted<T, EPV>(dst + static_cast<int64_t>(vi) * EPV, r, stream);
  }
}

// grad_input and the parameter-gradient partials in one pass: a group of WPR waves walks `walk`
// rows, one from each sweep of all the launch's groups over the matrix (group g takes rows g,
// g + groups, g + 2 groups, ...: at any moment the launch reads one contiguous span; a run of
// consecutive rows per group, whose starts lie a power of two apart, measured 3-12 % slower);
// every lane keeps the column sums of dy*xhat and dy for the columns it owns in registers and
// writes them once, as one fp32 partial row per group, at the end. dy and x are read exactly once.
// EXTRA: as in the narrow kernel below (round(dx) + addend is stored, its column sums are a third
// partial row per group).
template <typename T, int WPR, int VPL, int BLOCK, bool EXTRA = false>
__global__ __launch_bounds__(BLOCK) void layer_norm_backward_fused_kernel(
    T* __restrict__ dx, float* __restrict__ partial, const T* __restrict__ dy,
    const T* __restrict__ x, const float* __restrict__ mean, const float* __restrict__ rstd,
    const T* __restrict__ gamma, int64_t rows, int cols, int64_t walk,
    const T* __restrict__ addend = nullptr) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int NR = EXTRA ? 3 : 2;
  constexpr int XV = EXTRA ? VPL : 1;
  const bool stream = rows * cols * static_cast<int64_t>(3 * sizeof(T)) >= kStreamStoreBytes;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int GROUPS = WAVES / WPR;
  __shared__ float slot[WAVES];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int group = wave / WPR, wave_in_row = wave - group * WPR;
  const int nvec = cols / EPV;
  const float inv_n = 1.0f / static_cast<float>(cols);
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * GROUPS + group;
  const int64_t step = static_cast<int64_t>(gridDim.x) * GROUPS;  // groups of the launch

  float gf[VPL][EPV];  // gamma, unpacked once
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    Vec16<T> gv;
    if (gamma != nullptr) gv = load_vec16(gamma + static_cast<int64_t>(vi < nvec ? vi : 0) * EPV);
#pragma unroll
    for (int e = 0; e < EPV; ++e) gf[v][e] = gamma != nullptr ? to_f32(gv.v[e]) : 1.0f;
  }
  float dg[VPL][EPV], db[VPL][EPV], ds[XV][EPV];
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) dg[v][e] = db[v][e] = 0.0f;
#pragma unroll
  for (int v = 0; v < XV; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) ds[v][e] = 0.0f;

  // every group of the workgroup runs `walk` iterations (the reductions contain barriers); rows
  // past the end re-read the last row and contribute nothing
  for (int64_t i = 0; i < walk; ++i) {
    int64_t row = gid + i * step;
    const bool live = row < rows;
    if (!live) row = rows - 1;
    const T* dsrc = dy + row * static_cast<int64_t>(cols);
    const T* xsrc = x + row * static_cast<int64_t>(cols);
    const float mu = mean[row], rs = rstd[row];
    float gd[VPL][EPV], xh[VPL][EPV];
    Vec16<T> av[XV];
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const int vi = (v * WPR + wave_in_row) * kWave + lane;
      const bool ok = vi < nvec && live;
      const int64_t at = static_cast<int64_t>(vi < nvec ? vi : 0) * EPV;
      // (lanes past the row and rows past the end take part with dy = 0: see the narrow kernel)
      const Vec16<T> dv = keep_if(load_vec16_stream(dsrc + at), ok);
      const Vec16<T> xv = load_vec16_stream(xsrc + at);
      if constexpr (EXTRA)
        av[v] = load_vec16_stream((addend != nullptr ? addend : dy) + row * static_cast<int64_t>(cols) + at);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float d = to_f32(dv.v[e]);
        const float h = (to_f32(xv.v[e]) - mu) * rs;
        gd[v][e] = d * gf[v][e];
        xh[v][e] = h;
        s1 += gd[v][e];
        s2 += gd[v][e] * h;
        dg[v][e] += d * h;
        db[v][e] += d;
      }
    }
    s1 = wave_sum(s1);
    s1 = group_reduce(s1, slot, wave, group * WPR, WPR, SumOp{});
    s2 = wave_sum(s2);
    s2 = group_reduce(s2, slot, wave, group * WPR, WPR, SumOp{});
    if (live) {
      const float b1 = -rs * (s1 * inv_n), b2 = -rs * (s2 * inv_n);
      T* dst = dx + row * static_cast<int64_t>(cols);
#pragma unroll
      for (int v = 0; v < VPL; ++v) {
        const int vi = (v * WPR + wave_in_row) * kWave + lane;
        float r[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) r[e] = grad_input_of(gd[v][e], xh[v][e], rs, b1, b2);
        if constexpr (EXTRA) {
          // the two roundings of separate kernels: dx to T, then the sum to T
          const Vec16<T> az = keep_if(av[v], addend != nullptr);
#pragma unroll
          for (int e = 0; e < EPV; ++e) {
            r[e] = to_f32(from_f32<T>(pin_f32(r[e]))) + to_f32(az.v[e]);
            r[e] = to_f32(from_f32<T>(pin_f32(r[e])));
            ds[v][e] += vi < nvec ? r[e] : 0.0f;
          }
        }
        if (vi < nvec) store_converted_hinted<T, EPV>(dst + static_cast<int64_t>(vi) * EPV, r, stream);
      }
    }
  }
  float* pg = partial + (gid * NR + 0) * static_cast<int64_t>(cols);
  float* pb = partial + (gid * NR + 1) * static_cast<int64_t>(cols);
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WPR + wave_in_row) * kWave + lane;
    if (vi < nvec) {
      store_converted<float, EPV>(pg + static_cast<int64_t>(vi) * EPV, dg[v]);
      store_converted<float, EPV>(pb + static_cast<int64_t>(vi) * EPV, db[v]);
      if constexpr (EXTRA)
        store_converted<float, EPV>(partial + (gid * NR + 2) * static_cast<int64_t>(cols) +
                                        static_cast<int64_t>(vi) * EPV, ds[v]);
    }
  }
}

// Rows of up to 1024 columns: one wave per row and no barrier inside the walk. A wave takes
// `walk` rows, one from each sweep of all the launch's waves over the matrix (wave w takes rows
// w, w + waves, w + 2 waves, ...), two rows per iteration so that four row reads are in flight
// per wave; every lane keeps the column sums of dy * xhat and dy for its own columns in
// registers. At the end the four waves of a workgroup add their sums through LDS in wave order
// and the workgroup writes one fp32 partial row.
// EXTRA: the residual stream's form. grad_input is stored as round(dx) + addend (addend may be
// null) and the column sums of what was stored leave as a third partial row per workgroup.
template <typename T, int VPL, bool EXTRA = false>
__global__ __launch_bounds__(256) void layer_norm_backward_narrow_kernel(
    T* __restrict__ dx, float* __restrict__ partial, const T* __restrict__ dy,
    const T* __restrict__ x, const float* __restrict__ mean, const float* __restrict__ rstd,
    const T* __restrict__ gamma, int64_t rows, int cols, int64_t walk,
    const T* __restrict__ addend = nullptr) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int NR = EXTRA ? 3 : 2;    // partial rows per workgroup
  constexpr int XV = EXTRA ? VPL : 1;  // (arrays of the extra outputs shrink to one vector without them)
  const bool stream = rows * cols * static_cast<int64_t>(3 * sizeof(T)) >= kStreamStoreBytes;
  constexpr int WIDTH = VPL * kWave * EPV;  // columns a wave covers
  __shared__ float sums[4][NR][WIDTH];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nvec = cols / EPV;
  const float inv_n = 1.0f / static_cast<float>(cols);
  const int64_t wid = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  const int64_t step = static_cast<int64_t>(gridDim.x) * 4;  // waves of the launch

  float gf[VPL][EPV];  // gamma, unpacked once
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = v * kWave + lane;
    Vec16<T> gv;
    if (gamma != nullptr) gv = load_vec16(gamma + static_cast<int64_t>(vi < nvec ? vi : 0) * EPV);
#pragma unroll
    for (int e = 0; e < EPV; ++e) gf[v][e] = gamma != nullptr ? to_f32(gv.v[e]) : 1.0f;
  }
  float dg[VPL][EPV], db[VPL][EPV], ds[XV][EPV];
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) dg[v][e] = db[v][e] = 0.0f;
#pragma unroll
  for (int v = 0; v < XV; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) ds[v][e] = 0.0f;

  for (int64_t i = 0; i < walk; i += 2) {
    Vec16<T> dv[2][VPL], xv[2][VPL], av[2][XV];
    int64_t row[2];
    bool live[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      row[r] = wid + (i + r) * step;
      live[r] = row[r] < rows && i + r < walk;
      if (!live[r]) row[r] = rows - 1;  // any valid row: its values are masked out below
#pragma unroll
      for (int v = 0; v < VPL; ++v) {
        const int vi = v * kWave + lane;
        const int64_t at = row[r] * static_cast<int64_t>(cols) + static_cast<int64_t>(vi < nvec ? vi : 0) * EPV;
        dv[r][v] = load_vec16_stream(dy + at);
        xv[r][v] = load_vec16_stream(x + at);
        // (without an addend the load re-reads dy and is cleared below: a load under a
        // condition would make every later wait a wait for all loads)
        if constexpr (EXTRA) av[r][v] = load_vec16_stream((addend != nullptr ? addend : dy) + at);
      }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const float mu = mean[row[r]], rs = rstd[row[r]];
      float gd[VPL][EPV], xh[VPL][EPV];
      float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int v = 0; v < VPL; ++v) {
        // lanes past the row and rows past the end take part with dy = 0 (whole vectors are
        // cleared, not elements): every sum they feed then gets 0, whatever x they re-read
        const Vec16<T> dz = keep_if(dv[r][v], v * kWave + lane < nvec && live[r]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float d = to_f32(dz.v[e]);
          const float h = (to_f32(xv[r][v].v[e]) - mu) * rs;
          gd[v][e] = d * gf[v][e];
          xh[v][e] = h;
          s1 += gd[v][e];
          s2 += gd[v][e] * h;
          dg[v][e] += d * h;
          db[v][e] += d;
        }
      }
      s1 = wave_sum(s1);
      s2 = wave_sum(s2);
      if (live[r]) {
        const float b1 = -rs * (s1 * inv_n), b2 = -rs * (s2 * inv_n);
        T* dst = dx + row[r] * static_cast<int64_t>(cols);
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
          const int vi = v * kWave + lane;
          float out[EPV];
#pragma unroll
          for (int e = 0; e < EPV; ++e) out[e] = grad_input_of(gd[v][e], xh[v][e], rs, b1, b2);
          if constexpr (EXTRA) {
            // the two roundings of separate kernels: dx to T, then the sum to T
            const Vec16<T> az = keep_if(av[r][v], addend != nullptr);
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
              out[e] = to_f32(from_f32<T>(pin_f32(out[e]))) + to_f32(az.v[e]);
              out[e] = to_f32(from_f32<T>(pin_f32(out[e])));
              ds[v][e] += vi < nvec ? out[e] : 0.0f;
            }
          }
          if (vi < nvec) store_converted_hinted<T, EPV>(dst + static_cast<int64_t>(vi) * EPV, out, stream);
        }
      }
    }
  }
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const int c = (v * kWave + lane) * EPV + e;
      sums[wave][0][c] = dg[v][e];
      sums[wave][1][c] = db[v][e];
      if constexpr (EXTRA) sums[wave][2][c] = ds[v][e];
    }
  __syncthreads();
  float* out = partial + static_cast<int64_t>(blockIdx.x) * NR * cols;
  for (int c = threadIdx.x; c < NR * cols; c += 256) {
    const int which = c / cols, col = c - which * cols;
    out[c] = ((sums[0][which][col] + sums[1][which][col]) + sums[2][which][col]) + sums[3][which][col];
  }
}

// Rows per wave of the narrow kernel: about 512 workgroups (2048 waves), 4 to 64 rows each, even.
static int64_t narrow_walk(int64_t rows) {
  int64_t walk = (rows + 2047) / 2048;
  if (walk < 4) walk = 4;
  if (walk > 64) walk = 64;
  return (walk + 1) / 2 * 2;
}
static int64_t narrow_groups(int64_t rows) {
  const int64_t per_block = 4 * narrow_walk(rows);
  return (rows + per_block - 1) / per_block;
}

// Geometry of the fused kernel (a pure function of the shape: the workspace size and the order
// of the final summation follow from it): waves per row as in the forward kernels, about 2048
// waves in flight for rows of up to four waves and 4096 for wider ones (measured best of
// 1024 .. 16384 in both classes: more groups cost more partial rows, fewer leave the memory
// system short of requests), 8 to 64 rows per group, partial rows for whole workgroups.
struct FusedPlan {
  int wpr, groups_per_block;
  int64_t walk, groups, padded_groups;
};
static FusedPlan fused_plan(int64_t rows, int64_t nvec) {
  FusedPlan p;
  p.wpr = nvec <= 64 ? 1 : nvec <= 256 ? 2 : nvec <= 512 ? 4 : nvec <= 1024 ? 8 : 16;
  const int block = nvec <= 512 ? 256 : nvec <= 1024 ? 512 : 1024;
  p.groups_per_block = block / kWave / p.wpr;
  const int64_t target = (p.wpr >= 8 ? 4096 : 2048) / p.wpr;
  p.walk = (rows + target - 1) / target;
  if (p.walk < 8) p.walk = 8;
  if (p.walk > 64) p.walk = 64;
  p.groups = (rows + p.walk - 1) / p.walk;
  p.padded_groups = (p.groups + p.groups_per_block - 1) / p.groups_per_block * p.groups_per_block;
  return p;
}

template <typename T>
__global__ __launch_bounds__(256) void layer_norm_backward_dx_generic_kernel(
    T* __restrict__ dx, const T* __restrict__ dy, const T* __restrict__ x,
    const float* __restrict__ mean, const float* __restrict__ rstd, const T* __restrict__ gamma,
    int64_t rows, int64_t cols) {
  __shared__ float slot[4];
  const int wave = threadIdx.x >> 6;
  const float inv_n = 1.0f / static_cast<float>(cols);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* dsrc = dy + row * cols;
    const T* xsrc = x + row * cols;
    const float mu = mean[row], rs = rstd[row];
    float s1 = 0.0f, s2 = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += 256) {
      const float d = to_f32(dsrc[j]) * (gamma != nullptr ? to_f32(gamma[j]) : 1.0f);
      s1 += d;
      s2 += d * ((to_f32(xsrc[j]) - mu) * rs);
    }
    s1 = wave_sum(s1);
    s1 = group_reduce(s1, slot, wave, 0, 4, SumOp{});
    s2 = wave_sum(s2);
    s2 = group_reduce(s2, slot, wave, 0, 4, SumOp{});
    const float b1 = -rs * (s1 * inv_n), b2 = -rs * (s2 * inv_n);
    for (int64_t j = threadIdx.x; j < cols; j += 256) {
      const float d = to_f32(dsrc[j]) * (gamma != nullptr ? to_f32(gamma[j]) : 1.0f);
      const float xh = (to_f32(xsrc[j]) - mu) * rs;
      dx[row * cols + j] = from_f32<T>(grad_input_of(d, xh, rs, b1, b2));
    }
  }
}

// ---------------------------------------------------------------------------
// layer norm backward: grad_weight / grad_bias (sums over the rows, per column)
// A workgroup owns 64 column vectors (VEC: 16 bytes each, otherwise single elements) and a slab
// of rows; its four waves take every fourth row of the slab, so each wave-wide load covers 1 KiB
// of one row. Partials go to an fp32 workspace [slabs][2][cols]; a second kernel adds the slabs
// in order. No atomics: the result depends on the shape only.
// ---------------------------------------------------------------------------
constexpr int kParamWaves = 4;

template <typename T, bool VEC>
__global__ __launch_bounds__(kParamWaves* kWave) void layer_norm_param_partial_kernel(
    float* __restrict__ partial, const T* __restrict__ dy, const T* __restrict__ x,
    const float* __restrict__ mean, const float* __restrict__ rstd, int64_t rows, int64_t cols,
    int64_t rows_per_slab) {
  constexpr int EPV = VEC ? Vec16<T>::N : 1;
  __shared__ float lds[kParamWaves][2][kWave * EPV];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * kWave + lane;  // vector / element index
  const int64_t col0 = unit * EPV;
  const bool ok = col0 < cols;
  const int64_t slab = blockIdx.y;
  const int64_t r_begin = slab * rows_per_slab;
  const int64_t r_end = r_begin + rows_per_slab < rows ? r_begin + rows_per_slab : rows;
  float dg[EPV], db[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) dg[e] = db[e] = 0.0f;
  // four rows of the wave's share in flight at a time (eight independent 16-byte loads per lane)
  constexpr int kUnroll = 4;
  for (int64_t row0 = r_begin + wave; row0 < r_end; row0 += kParamWaves * kUnroll) {
    if constexpr (VEC) {
      Vec16<T> dv[kUnroll], xv[kUnroll];
      float mu[kUnroll], rs[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int64_t row = row0 + u * kParamWaves;
        const bool in = row < r_end && ok;
        if (row >= r_end) row = r_end - 1;  // a valid address; the values are not used
        mu[u] = mean[row];
        rs[u] = in ? rstd[row] : 0.0f;
        dv[u] = load_vec16_stream(dy + row * cols + (ok ? col0 : 0));
        xv[u] = load_vec16_stream(x + row * cols + (ok ? col0 : 0));
        if (!in) {
#pragma unroll
          for (int e = 0; e < EPV; ++e) dv[u].v[e] = from_f32<T>(0.0f);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float d = to_f32(dv[u].v[e]);
          dg[e] += d * ((to_f32(xv[u].v[e]) - mu[u]) * rs[u]);
          db[e] += d;
        }
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int64_t row = row0 + u * kParamWaves;
        if (row < r_end && ok) {
          const float d = to_f32(dy[row * cols + col0]);
          dg[0] += d * ((to_f32(x[row * cols + col0]) - mean[row]) * rstd[row]);
          db[0] += d;
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < EPV; ++e) {
    lds[wave][0][lane * EPV + e] = dg[e];
    lds[wave][1][lane * EPV + e] = db[e];
  }
  __syncthreads();
  // fixed order over the waves; thread t finishes element t (and t + 256, ...) of the tile
  for (int i = threadIdx.x; i < kWave * EPV; i += kParamWaves * kWave) {
    const int64_t col = static_cast<int64_t>(blockIdx.x) * kWave * EPV + i;
    if (col < cols) {
      float sg = lds[0][0][i], sb = lds[0][1][i];
#pragma unroll
      for (int w = 1; w < kParamWaves; ++w) {
        sg += lds[w][0][i];
        sb += lds[w][1][i];
      }
      partial[(slab * 2 + 0) * cols + col] = sg;
      partial[(slab * 2 + 1) * cols + col] = sb;
    }
  }
}

// 32 columns per workgroup; the 32 threads that share a column take every 32nd slab and their
// sums are added in thread order (fixed), so the result depends on the shape only. A slab holds NR
// partial rows (grad_gamma, grad_beta and, with NR = 3, the column sums of grad_input).
template <typename T, int NR = 2>
__global__ __launch_bounds__(1024) void layer_norm_param_final_kernel(
    T* __restrict__ dgamma, T* __restrict__ dbeta, const float* __restrict__ partial, int64_t cols,
    int64_t slabs, T* __restrict__ dsum = nullptr) {
  __shared__ float lds[NR][32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t col = static_cast<int64_t>(blockIdx.x) * 32 + tx;
  float acc[NR];
#pragma unroll
  for (int k = 0; k < NR; ++k) acc[k] = 0.0f;
  if (col < cols) {
    int64_t s = ty;
    for (; s + 96 < slabs; s += 128) {  // 4 * NR loads in flight, added in slab order
      float v[NR][4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < NR; ++k) v[k][u] = partial[((s + 32 * u) * NR + k) * cols + col];
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < NR; ++k) acc[k] += v[k][u];
    }
    for (; s < slabs; s += 32)
#pragma unroll
      for (int k = 0; k < NR; ++k) acc[k] += partial[(s * NR + k) * cols + col];
  }
#pragma unroll
  for (int k = 0; k < NR; ++k) lds[k][ty][tx] = acc[k];
  __syncthreads();
  if (ty == 0 && col < cols) {
    float t[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) t[k] = lds[k][0][tx];
    for (int i = 1; i < 32; ++i)
#pragma unroll
      for (int k = 0; k < NR; ++k) t[k] += lds[k][i][tx];
    if (dgamma != nullptr) dgamma[col] = from_f32<T>(t[0]);
    if (dbeta != nullptr) dbeta[col] = from_f32<T>(t[1]);
    if constexpr (NR == 3)
      if (dsum != nullptr) dsum[col] = from_f32<T>(t[2]);
  }
}

// Slabs of rows for the parameter gradients: enough workgroups to fill the GPU, each with at
// least 64 rows (pure function of the shape: the workspace size and the summation order follow).
static int64_t param_slabs(int64_t rows, int64_t cols, int epv) {
  const int64_t col_tiles = (cols + 64 * epv - 1) / (64 * epv);
  int64_t slabs = (1024 + col_tiles - 1) / col_tiles;
  const int64_t by_rows = (rows + 63) / 64;
  if (slabs > by_rows) slabs = by_rows;
  if (slabs < 1) slabs = 1;
  if (slabs > 65535) slabs = 65535;
  return slabs;
}

template <typename T>
static bool param_vec_ok(const void* dy, const void* x, int64_t cols) {
  return cols % Vec16<T>::N == 0 && aligned16(dy) && aligned16(x);
}

template <typename T>
static int layer_norm_backward_dispatch(void* dx_, void* dgamma_, void* dbeta_, const void* dy_,
                                        const void* x_, const float* mean, const float* rstd,
                                        const void* gamma_, int64_t rows, int64_t cols,
                                        void* workspace, size_t workspace_bytes,
                                        hipStream_t stream, const void* addend_ = nullptr,
                                        void* dsum_ = nullptr) {
  T* dx = static_cast<T*>(dx_);
  const T* dy = static_cast<const T*>(dy_);
  const T* x = static_cast<const T*>(x_);
  const T* gamma = static_cast<const T*>(gamma_);
  const T* addend = static_cast<const T*>(addend_);
  // the residual stream's form (an addend, column sums of grad_input, or both) exists in the two
  // one-pass kernels only
  const bool extra = addend_ != nullptr || dsum_ != nullptr;
  constexpr int EPV = Vec16<T>::N;
  // (rows of up to 1024 columns are at most two 16-bit or four fp32 vectors per lane)
  constexpr int kNarrowVpl = 1024 / (kWave * EPV);
  int rc = 0;
  if (dx != nullptr && (dgamma_ != nullptr || dbeta_ != nullptr) && cols % EPV == 0 && cols <= 1024 &&
      aligned16(dx) && aligned16(dy) && aligned16(x) && (gamma == nullptr || aligned16(gamma)) &&
      (addend == nullptr || aligned16(addend)) && rows < (int64_t{1} << 31)) {
    const int64_t nvec = cols / EPV;
    const int64_t walk = narrow_walk(rows), groups = narrow_groups(rows);
    const int nr = extra ? 3 : 2;
    if (workspace == nullptr || workspace_bytes < static_cast<size_t>(groups) * nr * cols * 4)
      return TMB_ERR_WORKSPACE;
    float* partial = static_cast<float*>(workspace);
    const dim3 grid(static_cast<unsigned>(groups));
#define TMB_LN(VPL)                                                                              \
  if constexpr (VPL <= kNarrowVpl) {                                                             \
    if (extra)                                                                                   \
      layer_norm_backward_narrow_kernel<T, VPL, true><<<grid, dim3(256), 0, stream>>>(           \
          dx, partial, dy, x, mean, rstd, gamma, rows, static_cast<int>(cols), walk, addend);    \
    else                                                                                         \
      layer_norm_backward_narrow_kernel<T, VPL, false><<<grid, dim3(256), 0, stream>>>(          \
          dx, partial, dy, x, mean, rstd, gamma, rows, static_cast<int>(cols), walk);            \
  }
    if (nvec <= 64) { TMB_LN(1) }
    else if (nvec <= 128) { TMB_LN(2) }
    else if (nvec <= 192) { TMB_LN(3) }
    else { TMB_LN(4) }
#undef TMB_LN
    rc = check_launch();
    if (rc != 0) return rc;
    const dim3 fgrid(static_cast<unsigned>((cols + 31) / 32));
    if (extra)
      layer_norm_param_final_kernel<T, 3><<<fgrid, dim3(1024), 0, stream>>>(
          static_cast<T*>(dgamma_), static_cast<T*>(dbeta_), partial, cols, groups, static_cast<T*>(dsum_));
    else
      layer_norm_param_final_kernel<T, 2><<<fgrid, dim3(1024), 0, stream>>>(
          static_cast<T*>(dgamma_), static_cast<T*>(dbeta_), partial, cols, groups);
    return check_launch();
  }
  if (dx != nullptr && (dgamma_ != nullptr || dbeta_ != nullptr) && cols % EPV == 0 &&
      cols / EPV > 128 && cols / EPV <= 16 * 64 * 2 && aligned16(dx) && aligned16(dy) && aligned16(x) &&
      (gamma == nullptr || aligned16(gamma)) && (addend == nullptr || aligned16(addend)) &&
      rows < (int64_t{1} << 31)) {
    const int64_t nvec = cols / EPV;
    const FusedPlan plan = fused_plan(rows, nvec);
    const int nr = extra ? 3 : 2;
    if (workspace == nullptr ||
        workspace_bytes < static_cast<size_t>(plan.padded_groups) * nr * cols * 4)
      return TMB_ERR_WORKSPACE;
    float* partial = static_cast<float*>(workspace);
    const dim3 grid(static_cast<unsigned>(plan.padded_groups / plan.groups_per_block));
#define TMB_LF(WPR, VPL, BLOCK)                                                                      \
  if (extra)                                                                                         \
    layer_norm_backward_fused_kernel<T, WPR, VPL, BLOCK, true><<<grid, dim3(BLOCK), 0, stream>>>(    \
        dx, partial, dy, x, mean, rstd, gamma, rows, static_cast<int>(cols), plan.walk, addend);     \
  else                                                                                               \
    layer_norm_backward_fused_kernel<T, WPR, VPL, BLOCK, false><<<grid, dim3(BLOCK), 0, stream>>>(   \
        dx, partial, dy, x, mean, rstd, gamma, rows, static_cast<int>(cols), plan.walk);
    // (groups past the last row write partial rows of zeros, which the final stage adds)
    if (nvec <= 64) { TMB_LF(1, 1, 256) }
    else if (nvec <= 128) { TMB_LF(2, 1, 256) }
    else if (nvec <= 256) { TMB_LF(2, 2, 256) }
    else if (nvec <= 512) { TMB_LF(4, 2, 256) }
    else if (nvec <= 1024) { TMB_LF(8, 2, 512) }
    else { TMB_LF(16, 2, 1024) }
#undef TMB_LF
    rc = check_launch();
    if (rc != 0) return rc;
    const dim3 fgrid(static_cast<unsigned>((cols + 31) / 32));
    if (extra)
      layer_norm_param_final_kernel<T, 3><<<fgrid, dim3(1024), 0, stream>>>(
          static_cast<T*>(dgamma_), static_cast<T*>(dbeta_), partial, cols, plan.padded_groups,
          static_cast<T*>(dsum_));
    else
      layer_norm_param_final_kernel<T, 2><<<fgrid, dim3(1024), 0, stream>>>(
          static_cast<T*>(dgamma_), static_cast<T*>(dbeta_), partial, cols, plan.padded_groups);
    return check_launch();
  }
  if (extra) return TMB_ERR_UNSUPPORTED;
  if (dx != nullptr) {
    const bool vec_ok = cols % EPV == 0 && aligned16(dx) && aligned16(dy) && aligned16(x) &&
                        (gamma == nullptr || aligned16(gamma)) && rows < (int64_t{1} << 31);
    const int64_t nvec = cols / EPV;
    bool done = false;
#define TMB_LB(WPR, VPL, BLOCK)                                                                  \
  {                                                                                              \
    constexpr int RPB = (BLOCK / kWave) / WPR;                                                   \
    const int64_t blocks = (rows + RPB - 1) / RPB;                                               \
    layer_norm_backward_dx_kernel<T, WPR, VPL, BLOCK>                                            \
        <<<dim3(static_cast<unsigned>(blocks)), dim3(BLOCK), 0, stream>>>(                       \
            dx, dy, x, mean, rstd, gamma, rows, static_cast<int>(cols));                         \
    done = true;                                                                                 \
  }
    if (vec_ok && nvec <= 16 * 64 * 4) {
      if (nvec <= 64) TMB_LB(1, 1, 256)
      else if (nvec <= 128) TMB_LB(2, 1, 256)
      else if (nvec <= 256) TMB_LB(2, 2, 256)
      else if (nvec <= 512) TMB_LB(4, 2, 256)
      else if (nvec <= 1024) TMB_LB(8, 2, 512)
      else if (nvec <= 2048) TMB_LB(16, 2, 1024)
      else TMB_LB(16, 4, 1024)
    }
#undef TMB_LB
    if (!done) {
      const int64_t blocks = rows < 65536 * 16 ? rows : 65536 * 16;
      layer_norm_backward_dx_generic_kernel<T>
          <<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(dx, dy, x, mean, rstd,
                                                                         gamma, rows, cols);
    }
    rc = check_launch();
    if (rc != 0) return rc;
  }
  if (dgamma_ == nullptr && dbeta_ == nullptr) return rc;
  const bool vec = param_vec_ok<T>(dy, x, cols);
  const int epv = vec ? EPV : 1;
  const int64_t slabs = param_slabs(rows, cols, epv);
  if (workspace == nullptr || workspace_bytes < static_cast<size_t>(slabs) * 2 * cols * 4)
    return TMB_ERR_WORKSPACE;
  const int64_t rows_per_slab = (rows + slabs - 1) / slabs;
  const int64_t col_tiles = (cols + 64 * epv - 1) / (64 * epv);
  if (col_tiles >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  float* partial = static_cast<float*>(workspace);
  const dim3 grid(static_cast<unsigned>(col_tiles), static_cast<unsigned>(slabs));
  if (vec)
    layer_norm_param_partial_kernel<T, true><<<grid, dim3(kParamWaves * kWave), 0, stream>>>(
        partial, dy, x, mean, rstd, rows, cols, rows_per_slab);
  else
    layer_norm_param_partial_kernel<T, false><<<grid, dim3(kParamWaves * kWave), 0, stream>>>(
        partial, dy, x, mean, rstd, rows, cols, rows_per_slab);
  rc = check_launch();
  if (rc != 0) return rc;
  layer_norm_param_final_kernel<T><<<dim3(static_cast<unsigned>((cols + 31) / 32)), dim3(1024), 0, stream>>>(
      static_cast<T*>(dgamma_), static_cast<T*>(dbeta_), partial, cols, slabs);
  return check_launch();
}

}  // namespace tmb

extern "C" int tmb_gelu_backward(void* grad_in, const void* grad_out, const void* in, int64_t numel,
                                 int dtype, int approximate_tanh, void* stream) {
  if (numel < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (numel == 0) return TMB_OK;
  if (grad_in == nullptr || grad_out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case TMB_F32: return tmb::launch_gelu_backward<float>(grad_in, grad_out, in, numel, approximate_tanh, s);
    case TMB_F16: return tmb::launch_gelu_backward<tmb::f16_t>(grad_in, grad_out, in, numel, approximate_tanh, s);
    case TMB_BF16: return tmb::launch_gelu_backward<tmb::bf16_t>(grad_in, grad_out, in, numel, approximate_tanh, s);
    default: return TMB_ERR_UNSUPPORTED;
  }
}

namespace tmb {

// What a cross-entropy loss sends back to the logits, from the saved log-probabilities in one
// pass: dx[r, c] = g[c] - exp(logp[r, c]) * s with g the dense NLL gradient of row r (-w at the
// row's target, 0 elsewhere) and s its row sum (-w), i.e. the arithmetic of
// softmax_backward_long_rows_kernel on that gradient without the gradient ever being stored. w is
// grad_out / total_weight (mean), grad_out (sum) or grad_out[r] (no reduction), rounded to the
// tensor type as the separate kernel would have stored it; rows whose target is ignore_index or
// no class get zeros. The rows of dx have a pitch of their own (ldo >= cols, whole 16-byte
// vectors, zero beyond cols), so the products that consume the result need no padded copy of it.
// A workgroup takes 256 * U vectors of one row: aligned stores, loads wherever the input row lies.
template <typename T, int U>
__global__ __launch_bounds__(256) void nll_log_softmax_backward_kernel(
    T* __restrict__ dx, const T* __restrict__ logp, const int64_t* __restrict__ target,
    const T* __restrict__ grad_out, const T* __restrict__ total_weight, int64_t cols, int64_t ldi,
    int64_t ldo, int chunks, int reduction, int64_t ignore_index) {
  constexpr int EPV = Vec16<T>::N;
  const int64_t row = blockIdx.x / chunks;
  const int chunk = static_cast<int>(blockIdx.x - row * chunks);
  const int64_t t = target[row];
  const bool valid = t != ignore_index && t >= 0 && t < cols;
  float w = 0.0f;
  if (valid) {
    if (reduction == 1) w = to_f32(grad_out[0]) / to_f32(total_weight[0]);
    else if (reduction == 2) w = to_f32(grad_out[0]);
    else w = to_f32(grad_out[row]);
  }
  const float g_t = to_f32(from_f32<T>(-w));  // the gradient at the target, as it would be stored
  const float s = g_t;                         // the row sum of that gradient
  const T* src = logp + row * ldi;
  T* dst = dx + row * ldo;
  const bool stream = static_cast<int64_t>(gridDim.x) * 256 * U * 32 >= kStreamStoreBytes;
  const int64_t nvec_out = ldo / EPV;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t vi = (static_cast<int64_t>(chunk) * U + u) * 256 + threadIdx.x;
    if (vi >= nvec_out) continue;
    const int64_t c0 = vi * EPV;
    float r[EPV];
    if (c0 + EPV <= cols) {
      const Vec16<T> y = load_vec16_unaligned(src + c0);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float g = (c0 + e == t) ? g_t : 0.0f;
        r[e] = valid ? g - exp_for<T>(to_f32(y.v[e])) * s : 0.0f;
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const int64_t c = c0 + e;
        const float g = (c == t) ? g_t : 0.0f;
        r[e] = (valid && c < cols) ? g - exp_for<T>(to_f32(src[c < cols ? c : 0])) * s : 0.0f;
      }
    }
    store_converted_hinted<T, EPV>(dst + c0, r, stream);
  }
}

template <typename T>
static int nll_log_softmax_backward_dispatch(void* dx, const void* logp, const int64_t* target,
                                             const void* grad_out, const void* total_weight,
                                             int64_t rows, int64_t cols, int64_t ldi, int64_t ldo,
                                             int reduction, int64_t ignore_index, hipStream_t stream) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int U = 4;
  if (ldo % EPV != 0 || ldo < cols || ldi < cols || !aligned16(dx)) return TMB_ERR_INVALID_ARGUMENT;
  const int64_t nvec_out = ldo / EPV;
  const int64_t chunks = (nvec_out + 256 * U - 1) / (256 * U);
  if (rows * chunks >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  nll_log_softmax_backward_kernel<T, U><<<dim3(static_cast<unsigned>(rows * chunks)), dim3(256), 0, stream>>>(
      static_cast<T*>(dx), static_cast<const T*>(logp), target, static_cast<const T*>(grad_out),
      static_cast<const T*>(total_weight), cols, ldi, ldo, static_cast<int>(chunks), reduction,
      ignore_index);
  return check_launch();
}

}  // namespace tmb

extern "C" int tmb_nll_log_softmax_backward_rows(void* dx, const void* logp, const int64_t* target,
                                                 const void* grad_out, const void* total_weight,
                                                 int64_t rows, int64_t cols, int64_t ldi, int64_t ldo,
                                                 int reduction, int64_t ignore_index, int dtype,
                                                 void* stream) {
  if (rows < 0 || cols < 0 || reduction < 0 || reduction > 2) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (dx == nullptr || logp == nullptr || target == nullptr || grad_out == nullptr ||
      (reduction == 1 && total_weight == nullptr))
    return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  using namespace tmb;
  switch (dtype) {
    case TMB_F32:
      return nll_log_softmax_backward_dispatch<float>(dx, logp, target, grad_out, total_weight, rows, cols,
                                                      ldi, ldo, reduction, ignore_index, s);
    case TMB_F16:
      return nll_log_softmax_backward_dispatch<f16_t>(dx, logp, target, grad_out, total_weight, rows, cols,
                                                      ldi, ldo, reduction, ignore_index, s);
    case TMB_BF16:
      return nll_log_softmax_backward_dispatch<bf16_t>(dx, logp, target, grad_out, total_weight, rows, cols,
                                                       ldi, ldo, reduction, ignore_index, s);
    default: return TMB_ERR_UNSUPPORTED;
  }
}

extern "C" int tmb_softmax_backward_rows(void* grad_in, const void* grad_out, const void* out,
                                         int64_t rows, int64_t cols, int dtype, int log_mode,
                                         void* stream) {
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (grad_in == nullptr || grad_out == nullptr || out == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  using namespace tmb;
  switch (dtype) {
    case TMB_F32:
      return log_mode ? softmax_backward_dispatch<float, true>(grad_in, grad_out, out, rows, cols, s)
                      : softmax_backward_dispatch<float, false>(grad_in, grad_out, out, rows, cols, s);
    case TMB_F16:
      return log_mode ? softmax_backward_dispatch<f16_t, true>(grad_in, grad_out, out, rows, cols, s)
                      : softmax_backward_dispatch<f16_t, false>(grad_in, grad_out, out, rows, cols, s);
    case TMB_BF16:
      return log_mode ? softmax_backward_dispatch<bf16_t, true>(grad_in, grad_out, out, rows, cols, s)
                      : softmax_backward_dispatch<bf16_t, false>(grad_in, grad_out, out, rows, cols, s);
    default: return TMB_ERR_UNSUPPORTED;
  }
}

extern "C" size_t tmb_layer_norm_backward_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
  if (rows <= 0 || cols <= 0) return 0;
  // sized for the scalar geometry when the vector one does not apply: take the larger of both
  const int epv = dtype == TMB_F32 ? 4 : 8;
  int64_t most = tmb::param_slabs(rows, cols, epv);
  const int64_t scalar = tmb::param_slabs(rows, cols, 1);
  if (scalar > most) most = scalar;
  if (cols % epv == 0) {
    const int64_t fused = tmb::fused_plan(rows, cols / epv).padded_groups;
    if (fused > most) most = fused;
    const int64_t narrow = tmb::narrow_groups(rows);
    if (cols <= 1024 && narrow > most) most = narrow;
  }
  return static_cast<size_t>(most) * 2 * static_cast<size_t>(cols) * 4;
}

extern "C" size_t tmb_layer_norm_backward_add_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
  if (rows <= 0 || cols <= 0) return 0;
  const int epv = dtype == TMB_F32 ? 4 : 8;
  // (16-bit rows of more than 8192 columns run 1024-thread workgroups, whose 128 registers per
  // lane the third set of column sums does not fit)
  if (cols % epv != 0 || cols / epv > (dtype == TMB_F32 ? 16 * 64 * 2 : 16 * 64)) return 0;
  const int64_t groups = cols <= 1024 ? tmb::narrow_groups(rows) : tmb::fused_plan(rows, cols / epv).padded_groups;
  return static_cast<size_t>(groups) * 3 * static_cast<size_t>(cols) * 4;
}

extern "C" int tmb_layer_norm_backward_add_rows(void* grad_in, void* grad_gamma, void* grad_beta,
                                                void* grad_sum, const void* grad_out, const void* in,
                                                const float* mean, const float* rstd,
                                                const void* gamma, const void* addend, int64_t rows,
                                                int64_t cols, int dtype, void* workspace,
                                                size_t workspace_bytes, void* stream) {
  if (rows <= 0 || cols <= 0) return TMB_ERR_INVALID_ARGUMENT;
  if (grad_in == nullptr || grad_gamma == nullptr || grad_beta == nullptr || grad_out == nullptr ||
      in == nullptr || mean == nullptr || rstd == nullptr || (addend == nullptr && grad_sum == nullptr))
    return TMB_ERR_INVALID_ARGUMENT;
  if (tmb_layer_norm_backward_add_workspace_bytes(rows, cols, dtype) == 0) return TMB_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  using namespace tmb;
  switch (dtype) {
    case TMB_F32:
      return layer_norm_backward_dispatch<float>(grad_in, grad_gamma, grad_beta, grad_out, in, mean, rstd, gamma, rows, cols, workspace, workspace_bytes, s, addend, grad_sum);
    case TMB_F16:
      return layer_norm_backward_dispatch<f16_t>(grad_in, grad_gamma, grad_beta, grad_out, in, mean, rstd, gamma, rows, cols, workspace, workspace_bytes, s, addend, grad_sum);
    case TMB_BF16:
      return layer_norm_backward_dispatch<bf16_t>(grad_in, grad_gamma, grad_beta, grad_out, in, mean, rstd, gamma, rows, cols, workspace, workspace_bytes, s, addend, grad_sum);
    default: return TMB_ERR_UNSUPPORTED;
  }
}

extern "C" int tmb_layer_norm_backward_rows(void* grad_in, void* grad_gamma, void* grad_beta,
                                            const void* grad_out, const void* in,
                                            const float* mean, const float* rstd,
                                            const void* gamma, int64_t rows, int64_t cols,
                                            int dtype, void* workspace, size_t workspace_bytes,
                                            void* stream) {
  if (rows < 0 || cols <= 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0) return TMB_OK;  // the caller zero-fills the parameter gradients of an empty batch
  if (grad_out == nullptr || in == nullptr || mean == nullptr || rstd == nullptr)
    return TMB_ERR_INVALID_ARGUMENT;
  if (grad_in == nullptr && grad_gamma == nullptr && grad_beta == nullptr) return TMB_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  using namespace tmb;
  switch (dtype) {
    case TMB_F32:
      return layer_norm_backward_dispatch<float>(grad_in, grad_gamma, grad_beta, grad_out, in, mean, rstd, gamma, rows, cols, workspace, workspace_bytes, s);
    case TMB_F16:
      return layer_norm_backward_dispatch<f16_t>(grad_in, grad_gamma, grad_beta, grad_out, in, mean, rstd, gamma, rows, cols, workspace, workspace_bytes, s);
    case TMB_BF16:
      return layer_norm_backward_dispatch<bf16_t>(grad_in, grad_gamma, grad_beta, grad_out, in, mean, rstd, gamma, rows, cols, workspace, workspace_bytes, s);
    default: return TMB_ERR_UNSUPPORTED;
  }
}
