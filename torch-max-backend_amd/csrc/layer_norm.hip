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

// Sum over the G lanes (16, 32 or 64, aligned) that share a row; every one of them gets the
// result. DPP butterflies inside 16 lanes, cross-lane permutes above that: a fixed order.
template <int G>
__device__ __forceinline__ float lanes_sum(float v) {
  v += dpp_f32<kDppQuadXor1>(v);
  v += dpp_f32<kDppQuadXor2>(v);
  v += dpp_f32<kDppRowHalfMirror>(v);
  v += dpp_f32<kDppRowMirror>(v);
  if constexpr (G >= 32) v += __shfl_xor(v, 16, kWave);
  if constexpr (G >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}

// A row is owned by G consecutive lanes: part of a wave (16 or 32 lanes: short rows keep every
// lane busy, a wave then works on 4 or 2 rows at once), one wave, or G/64 waves that meet in LDS.
// Each lane holds VPL 16-byte vectors of the row (G * VPL >= cols / EPV; the vectors of a row
// are interleaved so that one load instruction of the group covers G * 16 consecutive bytes), so
// the row is read once and both statistics passes run on registers.
//
// The grid is persistent: about 16 waves per CU, each group walking rows with the grid's
// stride, gamma and beta fetched once per lane (kept packed in their storage type) instead of
// once per row. A group's next row is requested right after the current row's stores; asking
// for it earlier (as soon as the current row is unpacked into fp32 registers) was measured on
// every geometry and changes nothing where the stores are non-temporal, except 4096-column fp32
// rows, which lose 4 % (88 -> 92 us): the other waves of the CU already cover the latency.
// The input may be wider than the output (fp32 rows normalised into a 16-bit
// tensor: the residual stream of a 16-bit model kept in fp32); gamma and beta have the output's
// type.
template <typename TIn, typename TOut, int G, int VPL, bool STREAM, int BLOCK>
__global__ __launch_bounds__(BLOCK) void layer_norm_rows_kernel(
    TOut* __restrict__ out, float* __restrict__ mean_out, float* __restrict__ rstd_out,
    const TIn* __restrict__ in, const TOut* __restrict__ gamma, const TOut* __restrict__ beta,
    int64_t rows, int cols, float eps) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int GPB = BLOCK / G;            // rows a workgroup works on at once
  constexpr int WPR = G > 64 ? G / 64 : 1;  // waves per row
  constexpr int SUB = G > 64 ? 64 : G;
  static_assert(BLOCK % G == 0 && GPB >= 1, "workgroup holds whole row groups");
  static_assert(sizeof(TOut) <= sizeof(TIn), "the output is never wider than the input");
  __shared__ float slot[2][2][BLOCK / kWave];  // [row parity][statistic][wave]

  const int tid = threadIdx.x;
  const int g = tid / G, l = tid % G;
  const int wave = tid >> 6;
  const int nvec = cols / EPV;
  const float n = static_cast<float>(cols);
  const int64_t total = static_cast<int64_t>(gridDim.x) * GPB;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * GPB + g;
  const int64_t iters = (rows + total - 1) / total;  // the same for every group: barriers stay matched

  typedef TOut param_t __attribute__((ext_vector_type(EPV)));
  typedef param_t __attribute__((aligned(sizeof(TOut)))) param_unaligned_t;
  param_t gv[VPL], bv[VPL];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = v * G + l;
    const int at = (vi < nvec ? vi : 0) * EPV;
    if (gamma != nullptr) gv[v] = *reinterpret_cast<const param_unaligned_t*>(gamma + at);
    if (beta != nullptr) bv[v] = *reinterpret_cast<const param_unaligned_t*>(beta + at);
  }

  auto load_row = [&](int64_t row, Vec16<TIn> (&raw)[VPL]) {
    if (row >= rows) row = rows - 1;  // keeps the groups in lock step; stores are masked
    const TIn* src = in + row * static_cast<int64_t>(cols);
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      // lanes past the end of the row re-read vector 0 (always valid) and discard it: no branch,
      // all loads of the group are issued back to back; the row is read exactly once, so the
      // loads are non-temporal whatever the size (STREAM only decides how the output is stored)
      const int vi = v * G + l;
      raw[v] = load_vec16_stream(src + static_cast<int64_t>(vi < nvec ? vi : 0) * EPV);
    }
  };
  Vec16<TIn> raw[VPL];
  load_row(gid, raw);
  for (int64_t it = 0; it < iters; ++it) {
    const int64_t row = it * total + gid;
    // Rows alternate between two sets of LDS slots: a wave that writes a slot for row it + 2 has
    // passed both barriers of row it + 1, which every wave reaches only after its last read of
    // row it's slots. Two barriers per row instead of three.
    float(&meet)[2][BLOCK / kWave] = slot[it & 1];
    float x[VPL][EPV];
    float s = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const bool ok = v * G + l < nvec;
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        x[v][e] = ok ? to_f32(raw[v].v[e]) : 0.0f;
        s += x[v][e];
      }
    }
    s = lanes_sum<SUB>(s);
    if constexpr (WPR > 1) {
      if ((tid & 63) == 0) meet[0][wave] = s;
      __syncthreads();
      s = meet[0][g * WPR];
#pragma unroll
      for (int w = 1; w < WPR; ++w) s += meet[0][g * WPR + w];
    }
    float mean = s / n;
    float q = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const bool ok = v * G + l < nvec;
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float d = ok ? x[v][e] - mean : 0.0f;
        x[v][e] = d;
        q += d * d;
      }
    }
    q = lanes_sum<SUB>(q);
    if constexpr (WPR > 1) {
      if ((tid & 63) == 0) meet[1][wave] = q;
      __syncthreads();
      q = meet[1][g * WPR];
#pragma unroll
      for (int w = 1; w < WPR; ++w) q += meet[1][g * WPR + w];
    }
    const float var = q / n;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (var != var) mean = var;
    if (row < rows) {
      if (l == 0) {
        if (mean_out) mean_out[row] = mean;
        if (rstd_out) rstd_out[row] = rstd;
      }
      TOut* dst = out + row * static_cast<int64_t>(cols);
#pragma unroll
      for (int v = 0; v < VPL; ++v) {
        const int vi = v * G + l;
        float y[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          y[e] = x[v][e] * rstd;
          if (gamma != nullptr) y[e] *= to_f32(gv[v][e]);
          if (beta != nullptr) y[e] += to_f32(bv[v][e]);
        }
        if (vi < nvec) {
          TOut* at = dst + static_cast<int64_t>(vi) * EPV;
          if constexpr (sizeof(TOut) == sizeof(TIn)) {
            store_converted<TOut, EPV, STREAM>(at, y);
          } else {
            // four fp32 values in, four 16-bit values out: one 8-byte store per vector
            param_t o;
#pragma unroll
            for (int e = 0; e < EPV; ++e) o[e] = from_f32<TOut>(y[e]);
            if constexpr (STREAM) {
              __builtin_nontemporal_store(o, reinterpret_cast<param_t*>(at));
            } else {
              *reinterpret_cast<param_t*>(at) = o;
            }
          }
        }
      }
    }
    if (it + 1 < iters) load_row(row + total, raw);
  }
}

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void layer_norm_generic_kernel(
    TOut* __restrict__ out, float* __restrict__ mean_out, float* __restrict__ rstd_out,
    const TIn* __restrict__ in, const TOut* __restrict__ gamma, const TOut* __restrict__ beta,
    int64_t rows, int64_t cols, float eps) {
  __shared__ float slot[4];
  const int wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const TIn* src = in + row * cols;
    TOut* dst = out + row * cols;
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
      dst[j] = from_f32<TOut>(y);
    }
  }
}

template <typename TIn, typename TOut, int G, int VPL, int BLOCK, int WAVES_PER_CU = 16>
static int launch_ln(TOut* out, float* mean, float* rstd, const TIn* x, const TOut* g, const TOut* b,
                     int64_t rows, int64_t cols, float eps, hipStream_t stream) {
  constexpr int GPB = BLOCK / G;
  const int64_t max_grid = (rows + GPB - 1) / GPB;
  // about 16 waves per CU, every workgroup walking the same number of rows (measured on
  // 32768 x 768 and 16384 x 4096: fewer waves leave the memory system short of requests, more
  // only add ramp and tail); 8 where a lane holds four vectors of a two-wave row
  int64_t grid = static_cast<int64_t>(compute_units()) * WAVES_PER_CU / (BLOCK / kWave);
  if (grid >= max_grid) {
    grid = max_grid;
  } else {
    const int64_t walk = (max_grid + grid - 1) / grid;
    grid = (max_grid + walk - 1) / walk;
  }
  // Non-temporal stores once input and output together are larger than the L2s (8 x 4 MB):
  // measured 4-5 % faster on 100 ... 200 MB passes ([32768, 768] bf16: 20.3 -> 19.4 us,
  // fp32: 37.0 -> 35.4 us), 10 % where the output alone is 134 MB.
  const bool stream_hint =
      rows * cols * static_cast<int64_t>(sizeof(TIn) + sizeof(TOut)) >= (int64_t{64} << 20);
  const dim3 grid3(static_cast<unsigned>(grid)), block(BLOCK);
  const int c = static_cast<int>(cols);
  if (stream_hint)
    layer_norm_rows_kernel<TIn, TOut, G, VPL, true, BLOCK><<<grid3, block, 0, stream>>>(out, mean, rstd, x, g, b, rows, c, eps);
  else
    layer_norm_rows_kernel<TIn, TOut, G, VPL, false, BLOCK><<<grid3, block, 0, stream>>>(out, mean, rstd, x, g, b, rows, c, eps);
  return check_launch();
}

template <typename TIn, typename TOut>
static int layer_norm_dispatch(void* out_, float* mean, float* rstd, const void* x_,
                               const void* g_, const void* b_, int64_t rows, int64_t cols,
                               float eps, hipStream_t stream) {
  TOut* out = static_cast<TOut*>(out_);
  const TIn* x = static_cast<const TIn*>(x_);
  const TOut* g = static_cast<const TOut*>(g_);
  const TOut* b = static_cast<const TOut*>(b_);
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int MAXV = 64 / EPV;  // at most 64 fp32 values of a row per lane
  constexpr uintptr_t kOutAlign = EPV * sizeof(TOut) - 1;  // one output vector per input vector
  const bool vec_ok = (cols % EPV == 0) && aligned16(x) &&
                      (reinterpret_cast<uintptr_t>(out) & kOutAlign) == 0 && rows < (int64_t{1} << 31);
  const int64_t nvec = cols / EPV;
#define TMB_LN(G, VPL, BLOCK) \
  return launch_ln<TIn, TOut, G, VPL, BLOCK>(out, mean, rstd, x, g, b, rows, cols, eps, stream)
#define TMB_LN8(G, VPL, BLOCK) \
  return launch_ln<TIn, TOut, G, VPL, BLOCK, 8>(out, mean, rstd, x, g, b, rows, cols, eps, stream)
  if (vec_ok && nvec <= 1024 * MAXV) {
    // the narrowest group that holds the row in at most four vectors per lane; measured on
    // 768- and 4096-column rows, where 32 x 3 / 64 x 3 and 256 x 2 / 256 x 4 run at the speed
    // of a plain copy of the same bytes
    if (nvec <= 16) TMB_LN(16, 1, 256);
    if (nvec <= 32) TMB_LN(16, 2, 256);
    if (nvec <= 48) TMB_LN(16, 3, 256);
    if (nvec <= 64) TMB_LN(32, 2, 256);
    if (nvec <= 96) TMB_LN(32, 3, 256);
    if (nvec <= 128) TMB_LN(64, 2, 256);
    if (nvec <= 192) TMB_LN(64, 3, 256);
    if (nvec <= 256) TMB_LN(64, 4, 256);
    if (nvec <= 384) TMB_LN(128, 3, 256);
    if (nvec <= 512) {
      // 16-bit rows of 4096 columns: two waves with four vectors per lane, eight waves per CU,
      // run at the speed of a copy (45.7 us on [16384, 4096] bf16 against 47.0 us for four waves
      // with two vectors, and 5 us less when the chip comes out of idle)
      if constexpr (sizeof(TIn) == 2) TMB_LN8(128, 4, 256);
      TMB_LN(256, 2, 512);
    }
    if (nvec <= 768) TMB_LN(256, 3, 512);
    if (nvec <= 1024) TMB_LN(256, 4, 512);
    if (nvec <= 2048) TMB_LN(512, 4, 512);
    if (nvec <= 4096) TMB_LN(1024, 4, 1024);
    if (nvec <= 8192) TMB_LN(1024, 8, 1024);
    if constexpr (MAXV >= 16) TMB_LN(1024, 16, 1024);
  }
#undef TMB_LN
#undef TMB_LN8
  const int64_t blocks = rows < 65536 * 16 ? rows : 65536 * 16;
  layer_norm_generic_kernel<TIn, TOut><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(
      out, mean, rstd, x, g, b, rows, cols, eps);
  return check_launch();
}

}  // namespace tmb

extern "C" int tmb_layer_norm_rows(void* out, float* mean, float* rstd, const void* x,
                                   const void* gamma, const void* beta, int64_t rows,
                                   int64_t cols, double eps, int in_dtype, int dtype, void* stream) {
  using namespace tmb;
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F32 && dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (in_dtype != dtype && in_dtype != TMB_F32) return TMB_ERR_UNSUPPORTED;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (out == nullptr || x == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float e = static_cast<float>(eps);
  if (in_dtype == TMB_F32) {
    switch (dtype) {
      case TMB_F32: return layer_norm_dispatch<float, float>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
      case TMB_F16: return layer_norm_dispatch<float, f16_t>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
      default: return layer_norm_dispatch<float, bf16_t>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
    }
  }
  if (dtype == TMB_F16)
    return layer_norm_dispatch<f16_t, f16_t>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
  return layer_norm_dispatch<bf16_t, bf16_t>(out, mean, rstd, x, gamma, beta, rows, cols, e, s);
}
