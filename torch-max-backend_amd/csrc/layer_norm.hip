// Layer norm forward over the last dimension for gfx950.
//
// Fast path: the row is loaded once into registers (16-byte vectors), both statistics passes
// run on registers, the normalised row is written once. Statistics are the reference's two-pass
// form, in fp32: mean = sum(x)/cols; var = sum((x-mean)^2)/cols; rstd = 1/sqrt(var+eps)
// (torch_mojo_backend/eager_kernels/nn_ops.mojo:299-326). A row whose variance is NaN
// (it contains NaN or an infinity) reports NaN for the mean as well
// (normalization_forward_kernels.mojo:60-70).
#include <type_traits>

#include "tmb_common.h"

namespace tmb {

// Same work decomposition as the softmax kernel: WPR waves per row, or (WPR == 1) RPW rows per
// wave with all loads issued up front. gamma/beta are fetched before the statistics so their
// latency hides behind the reductions.
//
// AFFINE_LDS (long rows): gamma and beta are copied into LDS once per workgroup, the workgroup
// then walks many rows (grid-stride), so the affine parameters cost LDS reads instead of a
// second and third pass through L2 for every row.
template <typename T, int WPR, int VPL, int RPW, bool STREAM, bool AFFINE_LDS, int BLOCK>
__global__ __launch_bounds__(BLOCK) void layer_norm_regs_kernel(
    T* __restrict__ out, float* __restrict__ mean_out, float* __restrict__ rstd_out,
    const T* __restrict__ in, const T* __restrict__ gamma, const T* __restrict__ beta,
    int64_t rows, int cols, float eps, int64_t row_span) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int GROUPS = WAVES / WPR;
  static_assert(WPR == 1 || RPW == 1, "several rows per wave only without cross-wave reductions");
  __shared__ float slot[WAVES];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int group = wave / WPR;
  const int wave_in_row = wave - group * WPR;
  const int nvec = cols / EPV;
  const float n = static_cast<float>(cols);

  extern __shared__ __attribute__((aligned(16))) unsigned char affine_lds[];
  T* lds_gamma = reinterpret_cast<T*>(affine_lds);
  T* lds_beta = lds_gamma + cols;
  if constexpr (AFFINE_LDS) {
    for (int vi = threadIdx.x; vi < nvec; vi += BLOCK) {
      if (gamma != nullptr) store_vec16(lds_gamma + vi * EPV, load_vec16(gamma + vi * EPV));
      if (beta != nullptr) store_vec16(lds_beta + vi * EPV, load_vec16(beta + vi * EPV));
    }
    __syncthreads();
  }

  // Short rows: gamma/beta are fetched once, before the first row's statistics (their latency
  // hides behind the reductions), and stay in registers for every row the workgroup walks.
  // Long rows would pay for that with occupancy; they fetch them (from LDS or L2) in groups of
  // four vectors right before use.
  constexpr bool PREFETCH_AFFINE = !AFFINE_LDS && VPL <= 4;
  constexpr int AFF = PREFETCH_AFFINE ? VPL : (VPL < 4 ? VPL : 4);  // vectors held at a time
  Vec16<T> gv[AFF], bv[AFF];
  auto load_affine = [&](int v_first) {
#pragma unroll
    for (int u = 0; u < AFF; ++u) {
      const int vi = ((v_first + u) * WPR + wave_in_row) * kWave + lane;
      const int64_t at = static_cast<int64_t>(vi < nvec ? vi : 0) * EPV;
      if constexpr (AFFINE_LDS) {
        if (gamma != nullptr) gv[u] = load_vec16(lds_gamma + at);
        if (beta != nullptr) bv[u] = load_vec16(lds_beta + at);
      } else {
        if (gamma != nullptr) gv[u] = load_vec16(gamma + at);
        if (beta != nullptr) bv[u] = load_vec16(beta + at);
      }
    }
  };
  if constexpr (PREFETCH_AFFINE) load_affine(0);

  // A workgroup walks `row_span` consecutive rows (a whole number of its row groups).
  const int64_t rows_per_block = static_cast<int64_t>(GROUPS) * RPW;
  const int64_t span_begin = static_cast<int64_t>(blockIdx.x) * row_span;
  const int64_t span_end = span_begin + row_span < rows ? span_begin + row_span : rows;
  for (int64_t block_row = span_begin; block_row < span_end; block_row += rows_per_block) {
  const int64_t row0 = block_row + static_cast<int64_t>(group) * RPW;

  float x[RPW][VPL][EPV];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    int64_t row = row0 + r;
    if (row >= rows) row = rows - 1;
    const T* src = in + row * static_cast<int64_t>(cols);
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      // Lanes past the end of the row re-read vector 0 (always valid) and discard it: no
      // branch, so all of a wave's loads are issued back to back.
      const int vi = (v * WPR + wave_in_row) * kWave + lane;
      const bool ok = vi < nvec;
      const int64_t at = static_cast<int64_t>(ok ? vi : 0) * EPV;
      // the row is read exactly once: non-temporal whatever the size (measured: 36 -> 26 us on
      // 32768 x 768 bf16); STREAM only decides how the output is stored
      const Vec16<T> t = load_vec16_stream(src + at);
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[r][v][e] = ok ? to_f32(t.v[e]) : 0.0f;
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    float s = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) s += x[r][v][e];
    s = wave_sum(s);
    s = group_reduce(s, slot, wave, group * WPR, WPR, SumOp{});
    float mean = s / n;

    float q = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const int vi = (v * WPR + wave_in_row) * kWave + lane;
      const bool ok = vi < nvec;
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float d = ok ? x[r][v][e] - mean : 0.0f;
        x[r][v][e] = d;
        q += d * d;
      }
    }
    q = wave_sum(q);
    q = group_reduce(q, slot, wave, group * WPR, WPR, SumOp{});
    const float var = q / n;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (var != var) mean = var;

    const int64_t row = row0 + r;
    if (row < rows) {
      if (wave_in_row == 0 && lane == 0) {
        if (mean_out) mean_out[row] = mean;
        if (rstd_out) rstd_out[row] = rstd;
      }
      T* dst = out + row * static_cast<int64_t>(cols);
#pragma unroll
      for (int v0 = 0; v0 < VPL; v0 += AFF) {
        if constexpr (!PREFETCH_AFFINE) load_affine(v0);
#pragma unroll
        for (int u = 0; u < AFF; ++u) {
          const int v = v0 + u;
          const int vi = (v * WPR + wave_in_row) * kWave + lane;
          float y[EPV];
          if (gamma != nullptr) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) y[e] = x[r][v][e] * rstd * to_f32(gv[u].v[e]);
          } else {
#pragma unroll
            for (int e = 0; e < EPV; ++e) y[e] = x[r][v][e] * rstd;
          }
          if (beta != nullptr) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) y[e] += to_f32(bv[u].v[e]);
          }
          if (vi < nvec) store_converted<T, EPV, STREAM>(dst + static_cast<int64_t>(vi) * EPV, y);
        }
      }
    }
  }
  }  // rows of this workgroup's span
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
  constexpr int EPV = Vec16<T>::N;
  constexpr int RPW = 1;
  constexpr int ROWS_PER_BLOCK = (BLOCK / kWave) / WPR * RPW;
  const int64_t groups = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;  // row groups of a workgroup
  const bool stream_hint = rows * cols * static_cast<int64_t>(2 * sizeof(T)) >= (int64_t{256} << 20);
  const dim3 block(BLOCK);
  const int c = static_cast<int>(cols);
  // `walk` row groups per workgroup, consecutive in memory
  auto launch = [&](auto lds_tag, int64_t walk, size_t lds_bytes) {
    constexpr bool LDS = decltype(lds_tag)::value;
    const int64_t blocks = (groups + walk - 1) / walk;
    const dim3 grid(static_cast<unsigned>(blocks));
    const int64_t span = walk * ROWS_PER_BLOCK;
    if (stream_hint)
      layer_norm_regs_kernel<T, WPR, VPL, RPW, true, LDS, BLOCK><<<grid, block, lds_bytes, stream>>>(out, mean, rstd, x, g, b, rows, c, eps, span);
    else
      layer_norm_regs_kernel<T, WPR, VPL, RPW, false, LDS, BLOCK><<<grid, block, lds_bytes, stream>>>(out, mean, rstd, x, g, b, rows, c, eps, span);
    return check_launch();
  };
  // Long 16-bit rows with affine parameters: gamma/beta staged in LDS by a few workgroups that
  // each walk many rows (for fp32 the LDS reads would cost as much as the L2 re-reads they
  // replace).
  const size_t lds_bytes = static_cast<size_t>(cols) * sizeof(T) * 2;
  if constexpr (VPL >= 8 && sizeof(T) == 2) {
    if ((g != nullptr || b != nullptr) && lds_bytes <= 65536) {
      const int64_t persistent = 256 * (BLOCK >= 1024 ? 2 : 8);
      return launch(std::true_type{}, (groups + persistent - 1) / persistent, lds_bytes);
    }
  }
  // Short rows keep gamma/beta in registers: a workgroup that walks a few consecutive row
  // groups re-uses them (more than four measured slower: too few workgroups in flight).
  const int64_t walk = VPL <= 4 ? (groups >= 16384 ? 4 : (groups >= 4096 ? 2 : 1)) : 1;
  return launch(std::false_type{}, walk, 0);
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
  constexpr int MAXV = 64 / EPV;  // at most 64 fp32 values of a row per lane
  const bool vec_ok = (cols % EPV == 0) && aligned16(x) && aligned16(out) &&
                      (g == nullptr || aligned16(g)) && (b == nullptr || aligned16(b)) &&
                      rows < (int64_t{1} << 31);
  const int64_t nvec = cols / EPV;
#define TMB_LN(WPR, VPL, BLOCK) \
  return launch_ln<T, WPR, VPL, BLOCK>(out, mean, rstd, x, g, b, rows, cols, eps, stream)
  if (vec_ok && nvec <= 16 * 64 * MAXV) {
    if (nvec <= 64) TMB_LN(1, 1, 256);
    if (nvec <= 128) TMB_LN(1, 2, 256);
    if (nvec <= 256) TMB_LN(1, 4, 256);
    if constexpr (MAXV >= 16) {
      // fp32: rows shared by four waves, two or four vectors per lane (measured 5-10 % faster
      // than one wave per row)
      if (nvec <= 512) TMB_LN(4, 2, 256);
      if (nvec <= 1024) TMB_LN(4, 4, 256);
    } else {
      if (nvec <= 512) TMB_LN(1, 8, 256);  // 16-bit: gamma/beta through LDS
    }
    if (nvec <= 4 * 64 * MAXV / 2) TMB_LN(4, MAXV / 2, 256);
    if (nvec <= 4 * 64 * MAXV) TMB_LN(4, MAXV, 256);
    if (nvec <= 16 * 64 * MAXV / 2) TMB_LN(16, MAXV / 2, 1024);
    TMB_LN(16, MAXV, 1024);
  }
#undef TMB_LN
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
