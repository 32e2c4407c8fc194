// Reductions over the LEADING dimension of a row-major [rows, cols] matrix: out[c] = op over r of
// in[r, c] (sum, mean, amax). This is the bias gradient of a linear layer (sum of dy over all
// tokens) and every `sum(x, dim=0)` of a graph; the row kernels would need the matrix transposed
// first. Bound by HBM: the input is read once, with every load a coalesced piece of a row.
//
// Two launches, a fixed order of additions that depends on the shape only (no atomics):
//   1. reduce_cols_partial_kernel: workgroup (g, s) owns 64 lanes x one 16-byte vector of columns
//      and slab s of the rows; its four waves take every fourth row of the slab, four rows in
//      flight each, and meet in LDS in wave order; one float32 partial row per slab.
//   2. reduce_cols_final_kernel: eight threads per column add every eighth slab each, in order,
//      and meet in LDS in lane order; one scale (mean) and one cast.
// Replaces the reference's route for these shapes: permute + contiguous copy into [kept, reduced]
// order (op_utils/__init__.mojo:651-720) followed by `SumSpec` / `MeanSpec` / `AmaxSpec`
// (eager_kernels/reduction_ops.mojo:1094-1184).
#include "tmb_common.h"

namespace tmb {

struct ColsPlan {
  int64_t groups;         // column groups of 64 vectors
  int64_t slabs;          // row slabs
  int64_t rows_per_slab;
};

// Must stay a pure function of (rows, cols, vector width): the workspace size and the order of
// the final additions follow from it.
static ColsPlan cols_plan(int64_t rows, int64_t cols, int epv) {
  ColsPlan p;
  p.groups = (cols + 64 * epv - 1) / (64 * epv);
  int64_t slabs = (2048 + p.groups - 1) / p.groups;  // about 8 workgroups per CU
  const int64_t most = (rows + 15) / 16;             // at least 16 rows per slab
  if (slabs > most) slabs = most;
  if (slabs > 256) slabs = 256;                      // the final stage walks them eight at a time
  if (slabs < 1) slabs = 1;
  p.rows_per_slab = ((rows + slabs - 1) / slabs + 15) / 16 * 16;
  p.slabs = (rows + p.rows_per_slab - 1) / p.rows_per_slab;
  return p;
}

// max that propagates NaN, as torch.amax does
__device__ __forceinline__ float max_nan(float a, float b) {
  return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b);
}

template <typename T, bool MAX, bool VEC>
__global__ __launch_bounds__(256) void reduce_cols_partial_kernel(float* __restrict__ partial,
                                                                  const T* __restrict__ in,
                                                                  int64_t rows, int64_t cols,
                                                                  int64_t rows_per_slab) {
  constexpr int EPV = VEC ? Vec16<T>::N : 1;
  constexpr int WIDTH = 64 * EPV;  // columns of a workgroup
  __shared__ float comb[4][WIDTH];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t col0 = (static_cast<int64_t>(blockIdx.x) * 64 + lane) * EPV;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * rows_per_slab;
  const int64_t r1 = r0 + rows_per_slab < rows ? r0 + rows_per_slab : rows;
  const bool live = col0 < cols;
  const float init = MAX ? -__builtin_inff() : 0.0f;
  float acc[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) acc[e] = init;
  auto take = [&](const T* p) {
    if constexpr (VEC) {
      const Vec16<T> v = load_vec16_stream(p);
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc[e] = MAX ? max_nan(acc[e], to_f32(v.v[e])) : acc[e] + to_f32(v.v[e]);
    } else {
      acc[0] = MAX ? max_nan(acc[0], to_f32(*p)) : acc[0] + to_f32(*p);
    }
  };
  if (live) {
    const T* base = in + col0;
    int64_t r = r0 + wave;
    for (; r + 12 < r1; r += 16) {  // four rows of this wave in flight
      if constexpr (VEC) {
        const Vec16<T> a = load_vec16_stream(base + r * cols), b = load_vec16_stream(base + (r + 4) * cols);
        const Vec16<T> c = load_vec16_stream(base + (r + 8) * cols), d = load_vec16_stream(base + (r + 12) * cols);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float fa = to_f32(a.v[e]), fb = to_f32(b.v[e]), fc = to_f32(c.v[e]), fd = to_f32(d.v[e]);
          acc[e] = MAX ? max_nan(max_nan(acc[e], fa), max_nan(max_nan(fb, fc), fd))
                       : ((acc[e] + fa) + fb) + (fc + fd);
        }
      } else {
        const float fa = to_f32(base[r * cols]), fb = to_f32(base[(r + 4) * cols]);
        const float fc = to_f32(base[(r + 8) * cols]), fd = to_f32(base[(r + 12) * cols]);
        acc[0] = MAX ? max_nan(max_nan(acc[0], fa), max_nan(max_nan(fb, fc), fd))
                     : ((acc[0] + fa) + fb) + (fc + fd);
      }
    }
    for (; r < r1; r += 4) take(base + r * cols);
  }
#pragma unroll
  for (int e = 0; e < EPV; ++e) comb[wave][lane * EPV + e] = acc[e];
  __syncthreads();
  float* dst = partial + static_cast<int64_t>(blockIdx.y) * cols;
  for (int c = threadIdx.x; c < WIDTH; c += 256) {
    const int64_t col = static_cast<int64_t>(blockIdx.x) * WIDTH + c;
    if (col < cols) {
      const float a = comb[0][c], b = comb[1][c], x = comb[2][c], y = comb[3][c];
      dst[col] = MAX ? max_nan(max_nan(a, b), max_nan(x, y)) : (a + b) + (x + y);
    }
  }
}

// 32 columns x 8 slab lanes per workgroup: thread (column c, lane q) adds slabs q, q + 8, q + 16, ...
// in that order, eight loads in flight; the eight results meet in LDS and are added in lane order.
// (One thread per column walking all slabs ran 14 us on 256 slabs x 768 columns: three
// workgroups on the whole chip, 32 dependent round trips to memory each.)
template <typename T, bool MAX>
__global__ __launch_bounds__(256) void reduce_cols_final_kernel(T* __restrict__ out,
                                                                const float* __restrict__ partial,
                                                                int64_t cols, int64_t slabs,
                                                                float scale) {
  __shared__ float part[8][32];
  const int c = threadIdx.x & 31, q = threadIdx.x >> 5;
  const int64_t col = static_cast<int64_t>(blockIdx.x) * 32 + c;
  float acc = 0.0f;
  if (col < cols && q < slabs) {
    acc = partial[q * cols + col];
    int64_t s = q + 8;
    for (; s + 56 < slabs; s += 64) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = partial[(s + 8 * u) * cols + col];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc = MAX ? max_nan(acc, v[u]) : acc + v[u];
    }
    for (; s < slabs; s += 8) {
      const float v = partial[s * cols + col];
      acc = MAX ? max_nan(acc, v) : acc + v;
    }
  }
  part[q][c] = acc;
  __syncthreads();
  if (q != 0 || col >= cols) return;
  const int lanes = slabs < 8 ? static_cast<int>(slabs) : 8;
  float r = part[0][c];
  for (int i = 1; i < lanes; ++i) r = MAX ? max_nan(r, part[i][c]) : r + part[i][c];
  out[col] = from_f32<T>(MAX ? r : r * scale);
}

template <typename T>
static int launch_reduce_cols(void* out, const void* in, int64_t rows, int64_t cols, int op,
                              void* workspace, size_t workspace_bytes, hipStream_t stream) {
  constexpr int EPV = Vec16<T>::N;
  const bool vec = cols % EPV == 0 && aligned16(in);
  const ColsPlan p = cols_plan(rows, cols, vec ? EPV : 1);
  if (workspace == nullptr || workspace_bytes < static_cast<size_t>(p.slabs * cols) * sizeof(float))
    return TMB_ERR_WORKSPACE;
  if ((cols + 31) / 32 >= (int64_t{1} << 31) || p.slabs > 65535) return TMB_ERR_UNSUPPORTED;
  float* partial = static_cast<float*>(workspace);
  const T* src = static_cast<const T*>(in);
  const dim3 grid(static_cast<unsigned>(p.groups), static_cast<unsigned>(p.slabs));
  const bool is_max = op == TMB_AMAX;
#define TMB_RC(MAX, VEC) \
  reduce_cols_partial_kernel<T, MAX, VEC><<<grid, dim3(256), 0, stream>>>(partial, src, rows, cols, p.rows_per_slab)
  if (is_max) { if (vec) TMB_RC(true, true); else TMB_RC(true, false); }
  else { if (vec) TMB_RC(false, true); else TMB_RC(false, false); }
#undef TMB_RC
  int rc = check_launch();
  if (rc != 0) return rc;
  const dim3 fgrid(static_cast<unsigned>((cols + 31) / 32));
  const float scale = op == TMB_MEAN ? 1.0f / static_cast<float>(rows) : 1.0f;
  if (is_max)
    reduce_cols_final_kernel<T, true><<<fgrid, dim3(256), 0, stream>>>(static_cast<T*>(out), partial, cols, p.slabs, scale);
  else
    reduce_cols_final_kernel<T, false><<<fgrid, dim3(256), 0, stream>>>(static_cast<T*>(out), partial, cols, p.slabs, scale);
  return check_launch();
}

}  // namespace tmb

extern "C" size_t tmb_reduce_cols_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
  if (rows <= 0 || cols <= 0) return 0;
  const int epv = dtype == TMB_F32 ? 4 : 8;
  // the scalar plan (unaligned input) never needs more slabs than the vector plan: size for both
  const tmb::ColsPlan a = tmb::cols_plan(rows, cols, epv), b = tmb::cols_plan(rows, cols, 1);
  const int64_t slabs = a.slabs > b.slabs ? a.slabs : b.slabs;
  return static_cast<size_t>(slabs * cols) * sizeof(float);
}

extern "C" int tmb_reduce_cols(void* out, const void* in, int64_t rows, int64_t cols, int op,
                               int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace tmb;
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (op != TMB_SUM && op != TMB_MEAN && op != TMB_AMAX)
    return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F32 && dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (cols == 0) return TMB_OK;
  if (rows == 0) return TMB_ERR_UNSUPPORTED;  // identities of an empty reduction: the caller's rule
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case TMB_F32: return launch_reduce_cols<float>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    case TMB_F16: return launch_reduce_cols<f16_t>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    default: return launch_reduce_cols<bf16_t>(out, in, rows, cols, op, workspace, workspace_bytes, s);
  }
}
