// Row softmax / log-softmax for gfx950.
//
// Fast path: the whole row lives in registers (one HBM read + one HBM write per element).
// A row is covered by WPR cooperating waves; every lane owns VPL 16-byte vectors that are
// interleaved so that each wave-wide load instruction touches 1 KiB of consecutive memory.
// Reductions are DPP within a wave and a fixed-order LDS combine across the row's waves.
//
// Long rows that are ragged (cols not a whole number of vectors) or not 16-byte aligned: the
// same, one 1024-thread workgroup per row, with the vectors starting at the first 16-byte
// boundary inside the row (or unaligned vector accesses where input and output differ there).
//
// Generic path: any alignment / any width, one 256-thread block per row, three passes
// (the second and third read come from L2 for rows that fit there).
//
// Arithmetic follows the reference CPU kernels (fp32 max, fp32 sum of exp(x-m), one cast):
// torch_mojo_backend/eager_kernels/nn_ops.mojo:428-455 and reduction_ops.mojo:874-895.
#include "tmb_common.h"

namespace tmb {

// WPR waves cooperate on a row (WPR > 1: one row per group of waves); with WPR == 1 every wave
// owns RPW independent rows whose loads are all issued before any arithmetic, which keeps more
// bytes in flight for short rows. STREAM selects non-temporal loads/stores (tensors larger than
// the Infinity Cache).
//
// SCALED: the attention form of the reference kernel (nn_ops.mojo:413-493, `_softmax_rows(scale,
// causal, q_len)`): x*scale before the max, and with q_len > 0 column j of row r takes part only
// if j <= r % q_len (the rest comes out as exact zeros). round_scaled rounds x*scale to the
// storage type first, which is what a separate `mul` kernel in front of the softmax would have
// stored: a graph that fuses mul + masked_fill + softmax into this kernel then gets the bits
// of the unfused pipeline. Vectors that are masked out entirely are not fetched (their lanes
// re-read vector 0 of the row), so a causal softmax reads about half of its input.
struct SoftmaxScale {
  float scale;
  int round_scaled;
  int q_len;
};

template <typename TIn, typename TOut, int WPR, int VPL, int RPW, bool LOG, bool STREAM, bool SCALED,
          int BLOCK>
__global__ __launch_bounds__(BLOCK) void softmax_regs_kernel(TOut* __restrict__ out,
                                                             const TIn* __restrict__ in,
                                                             int64_t rows, int cols,
                                                             SoftmaxScale sc) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int GROUPS = WAVES / WPR;
  static_assert(WPR == 1 || RPW == 1, "several rows per wave only without cross-wave reductions");
  __shared__ float slot[WAVES];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int group = wave / WPR;
  const int wave_in_row = wave - group * WPR;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * GROUPS + group) * RPW;
  const int nvec = cols / EPV;
  const float neg_inf = -__builtin_inff();

  float x[RPW][VPL][EPV];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    int64_t row = row0 + r;
    if (row >= rows) row = rows - 1;  // keep lock-step; stores are masked below
    const TIn* src = in + row * static_cast<int64_t>(cols);
    // last column that takes part (causal), or the whole row
    const int last_col = (SCALED && sc.q_len > 0) ? static_cast<int>(row % sc.q_len) : cols - 1;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      // Lanes past the end of the row re-read vector 0 (always valid) and discard it: no
      // branch, so all of a wave's loads are issued back to back.
      const int vi = (v * WPR + wave_in_row) * kWave + lane;
      const bool ok = SCALED ? (vi < nvec && vi * EPV <= last_col) : vi < nvec;
      const int64_t at = static_cast<int64_t>(ok ? vi : 0) * EPV;
      // read once: non-temporal whatever the size; STREAM only decides how the output is stored
      const Vec16<TIn> t = load_vec16_stream(src + at);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        if constexpr (SCALED) {
          float xs = to_f32(t.v[e]) * sc.scale;
          if (sc.round_scaled) xs = to_f32(from_f32<TIn>(xs));
          x[r][v][e] = (ok && vi * EPV + e <= last_col) ? xs : neg_inf;
        } else {
          x[r][v][e] = ok ? to_f32(t.v[e]) : neg_inf;
        }
      }
    }
  }

#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    float m = neg_inf;
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) m = fmaxf(m, x[r][v][e]);
    m = wave_max(m);
    m = group_reduce(m, slot, wave, group * WPR, WPR, MaxOp{});

    float s = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float ex = exp_for<TOut>(x[r][v][e] - m);
        if (LOG) {
          x[r][v][e] = x[r][v][e] - m;
        } else {
          x[r][v][e] = ex;
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
        for (int e = 0; e < EPV; ++e) x[r][v][e] -= lg;
    } else {
      const float inv = 1.0f / s;
#pragma unroll
      for (int v = 0; v < VPL; ++v)
#pragma unroll
        for (int e = 0; e < EPV; ++e) x[r][v][e] *= inv;
    }

    const int64_t row = row0 + r;
    if (row < rows) {
      TOut* dst = out + row * static_cast<int64_t>(cols);
#pragma unroll
      for (int v = 0; v < VPL; ++v) {
        const int vi = (v * WPR + wave_in_row) * kWave + lane;
        if (vi < nvec)
          store_converted<TOut, EPV, STREAM>(dst + static_cast<int64_t>(vi) * EPV, x[r][v]);
      }
    }
  }
}

// Long rows of any width at any element alignment (a [rows, 50257] logits tensor: the pitch is
// odd, so no row but the first starts on a 16-byte boundary): one 1024-thread workgroup per row,
// the row in registers as in the kernel above, one read and one write per element, where the
// generic kernel reads three times with element accesses.
// PEEL: input and output rows sit at the same offset from a 16-byte boundary (same pitch, both
// tensors aligned). The vectors then start at the first boundary inside the row and every vector
// access is aligned, which measures 25-30 % faster than unaligned ones (16384 x 50257 bf16: 0.67
// against 0.94 ms); the up to EPV - 1 elements in front of the first vector and after the last one
// are held one each by the first lanes of wave 0. Without PEEL the vectors start with the row
// and are fetched and stored with unaligned 16-byte accesses.
template <typename TIn, typename TOut, int VPL, bool LOG, bool PEEL, bool STREAM>
__global__ __launch_bounds__(1024) void softmax_long_rows_kernel(TOut* __restrict__ out,
                                                                 const TIn* __restrict__ in,
                                                                 int cols) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int WAVES = 16;
  static_assert(!PEEL || sizeof(TIn) == sizeof(TOut), "one offset for both rows");
  __shared__ float slot[WAVES];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const float neg_inf = -__builtin_inff();
  const TIn* src = in + static_cast<int64_t>(blockIdx.x) * cols;
  TOut* dst = out + static_cast<int64_t>(blockIdx.x) * cols;
  // columns [0, head) precede the first vector, [head + nvec * EPV, cols) follow the last one
  int head = 0;
  if constexpr (PEEL) {
    const int off = static_cast<int>((reinterpret_cast<uintptr_t>(src) & 15u) / sizeof(TIn));
    head = off ? EPV - off : 0;
  }
  const int nvec = (cols - head) / EPV;
  const int tail_from = head + nvec * EPV;
  // lanes 0 .. 7 of wave 0: a head element each; lanes 8 .. 15: a tail element each
  int edge = -1;
  if (wave == 0 && lane < 8 && lane < head) edge = lane;
  if (wave == 0 && lane >= 8 && lane < 16 && tail_from + lane - 8 < cols) edge = tail_from + lane - 8;

  float x[VPL][EPV];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WAVES + wave) * kWave + lane;
    const bool ok = vi < nvec;
    const TIn* at = src + head + static_cast<int64_t>(ok ? vi : 0) * EPV;
    Vec16<TIn> t;
    if constexpr (PEEL) {
      // (non-temporal: with plain loads the 16384 x 50257 bf16 case takes 0.94 instead of 0.70 ms)
      t = load_vec16_stream(at);
    } else {
      t = load_vec16_unaligned(at);
    }
#pragma unroll
    for (int e = 0; e < EPV; ++e) x[v][e] = ok ? to_f32(t.v[e]) : neg_inf;
  }
  float xt = neg_inf;
  if (edge >= 0) xt = to_f32(src[edge]);

  float m = xt;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) m = fmaxf(m, x[v][e]);
  m = wave_max(m);
  m = group_reduce(m, slot, wave, 0, WAVES, MaxOp{});

  const float ext = exp_for<TOut>(xt - m);
  xt = LOG ? xt - m : ext;
  float s = ext;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float ex = exp_for<TOut>(x[v][e] - m);
      x[v][e] = LOG ? x[v][e] - m : ex;
      s += ex;
    }
  s = wave_sum(s);
  s = group_reduce(s, slot, wave, 0, WAVES, SumOp{});
  const float lg = logf(s), inv = 1.0f / s;

#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int vi = (v * WAVES + wave) * kWave + lane;
#pragma unroll
    for (int e = 0; e < EPV; ++e) x[v][e] = LOG ? x[v][e] - lg : x[v][e] * inv;
    if (vi < nvec) {
      TOut* at = dst + head + static_cast<int64_t>(vi) * EPV;
      if constexpr (PEEL) {
        store_converted<TOut, EPV, STREAM>(at, x[v]);
      } else {
        store_converted_unaligned<TOut, EPV>(at, x[v]);
      }
    }
  }
  if (edge >= 0) dst[edge] = from_f32<TOut>(LOG ? xt - lg : xt * inv);
}

// The same row kernel for rows that fit 64 registers per lane, so that two 1024-thread
// workgroups share a CU and one row's stores run under the other's loads (the kernel above, with
// 64 .. 128 registers, leaves a CU to one row at a time: 0.61-0.63 of the memory peak on
// 16384 x 50257). 16-bit rows stay in their storage type (four registers per vector) and are
// converted again in each of the three passes, with the exponential taken twice (one multiply and
// one v_exp_f32 each for a 16-bit result). fp32 rows (transformed in place) would need 8 or 13
// vectors per lane there, which spills: they run in 512-thread workgroups (below).
// BLOCK = 512: fp32 rows, transformed in place in up to 100 registers per lane: two workgroups
// of eight waves share a CU at 128 registers each, where the kernel above runs one of sixteen.
// HELD < VPL: only the first HELD vectors of a lane stay in registers; the others (a fifth of a
// 50257-wide fp32 row) are read again in each pass, from the L2 they were fetched into (two rows
// per CU leave 64 x 40 KB of such vectors per XCD). The arithmetic per element is the same either
// way.
template <typename TIn, typename TOut, int VPL, bool LOG, bool PEEL, bool STREAM, int BLOCK = 1024,
          int HELD = VPL>
__global__ __launch_bounds__(BLOCK, BLOCK == 1024 ? 8 : 4) void softmax_long_rows_lean_kernel(
    TOut* __restrict__ out, const TIn* __restrict__ in, int cols) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int WAVES = BLOCK / kWave;
  constexpr bool IN_PLACE = sizeof(TIn) == 4;
  static_assert(!PEEL || sizeof(TIn) == sizeof(TOut), "one offset for both rows");
  static_assert(BLOCK == 1024 || BLOCK == 512, "two workgroups per CU either way");
  static_assert(HELD * 4 <= (BLOCK == 1024 ? 32 : 84),
                "the row must leave room for the rest in 64 (128) registers");
  static_assert(HELD == VPL || sizeof(TIn) == 4, "rows are read again in the in-place form only");
  __shared__ float slot[WAVES];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const float neg_inf = -__builtin_inff();
  const TIn* src = in + static_cast<int64_t>(blockIdx.x) * cols;
  TOut* dst = out + static_cast<int64_t>(blockIdx.x) * cols;
  int head = 0;
  if constexpr (PEEL) {
    const int off = static_cast<int>((reinterpret_cast<uintptr_t>(src) & 15u) / sizeof(TIn));
    head = off ? EPV - off : 0;
  }
  const int nvec = (cols - head) / EPV;
  const int tail_from = head + nvec * EPV;
  int edge = -1;
  if (wave == 0 && lane < 8 && lane < head) edge = lane;
  if (wave == 0 && lane >= 8 && lane < 16 && tail_from + lane - 8 < cols) edge = tail_from + lane - 8;

  // vector slots past the end of the row hold -inf in every element: exp gives 0, nothing is
  // stored from them. Addresses are a uniform row base plus a 32-bit byte offset per lane.
  const char* src_b = reinterpret_cast<const char*>(src + head);
  char* dst_b = reinterpret_cast<char*>(dst + head);
  const uint32_t lane_vec = static_cast<uint32_t>(wave * kWave + lane);
  Vec16<TIn> raw[HELD];
  // vector v of the lane, -inf in every element past the end of the row; `again`: a vector that
  // is not held (plain loads: it is wanted from the L2 twice more)
  auto fetch = [&](int v, bool again) {
    const uint32_t vi = lane_vec + v * (WAVES * kWave);
    const bool ok = vi < static_cast<uint32_t>(nvec);
    const TIn* at = reinterpret_cast<const TIn*>(src_b + (ok ? vi : 0u) * 16u);
    Vec16<TIn> t;
    if constexpr (PEEL) {
      t = again ? load_vec16(at) : load_vec16_stream(at);
    } else {
      t = load_vec16_unaligned(at);
    }
    const raw16_t all_neg_inf = sizeof(TIn) == 4 ? raw16_t{0xff800000u, 0xff800000u, 0xff800000u, 0xff800000u}
                                : (__is_same(TIn, bf16_t) ? raw16_t{0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u}
                                                          : raw16_t{0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u});
    return ok ? t : __builtin_bit_cast(Vec16<TIn>, all_neg_inf);
  };
#pragma unroll
  for (int v = 0; v < HELD; ++v) raw[v] = fetch(v, false);
  float xt = neg_inf;
  if (edge >= 0) xt = to_f32(src[edge]);
  // 16-bit rows: the compiler must not carry the converted values from one pass to the next
  // (that is the register budget this kernel exists to avoid), so the raw vectors are made
  // opaque between the passes
  auto forget = [&]() {
    if constexpr (!IN_PLACE) {
#pragma unroll
      for (int v = 0; v < HELD; ++v) {
        raw16_t r = __builtin_bit_cast(raw16_t, raw[v]);
        asm volatile("" : "+v"(r));
        raw[v] = __builtin_bit_cast(Vec16<TIn>, r);
      }
    }
  };

  float m = xt;
#pragma unroll
  for (int v = HELD; v < VPL; v += 2) {  // (two at a time, behind the loads of the held ones)
    __builtin_amdgcn_sched_barrier(0);
    const Vec16<TIn> t0 = fetch(v, true);
    const Vec16<TIn> t1 = fetch(v + 1 < VPL ? v + 1 : v, true);
#pragma unroll
    for (int e = 0; e < EPV; ++e) m = fmaxf(m, fmaxf(to_f32(t0.v[e]), to_f32(t1.v[e])));
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int v = 0; v < HELD; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) m = fmaxf(m, to_f32(raw[v].v[e]));
  m = wave_max(m);
  m = group_reduce(m, slot, wave, 0, WAVES, MaxOp{});
  forget();

  const float ext = exp_for<TOut>(xt - m);
  xt = LOG ? xt - m : ext;
  float s = ext;
#pragma unroll
  for (int v = 0; v < HELD; ++v) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float d = to_f32(raw[v].v[e]) - m;
      const float ex = exp_for<TOut>(d);
      if constexpr (IN_PLACE) raw[v].v[e] = LOG ? d : ex;
      s += ex;
    }
    if constexpr (BLOCK == 512) __builtin_amdgcn_sched_barrier(0);  // (one vector's temporaries at a time)
  }
  // (in the order of the held form: the sum is the same; two vectors in flight at a time)
#pragma unroll
  for (int v = HELD; v < VPL; v += 2) {
    const Vec16<TIn> t0 = fetch(v, true);
    const Vec16<TIn> t1 = fetch(v + 1 < VPL ? v + 1 : v, true);
#pragma unroll
    for (int e = 0; e < EPV; ++e) s += exp_for<TOut>(to_f32(t0.v[e]) - m);
    if (v + 1 < VPL) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) s += exp_for<TOut>(to_f32(t1.v[e]) - m);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  s = wave_sum(s);
  s = group_reduce(s, slot, wave, 0, WAVES, SumOp{});
  const float lg = logf(s), inv = 1.0f / s;
  forget();

#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const uint32_t vi = lane_vec + v * (WAVES * kWave);
    float y[EPV];
    Vec16<TIn> t;
    if (v >= HELD) t = fetch(v, true);  // (compile-time: the loop is unrolled)
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      if (v >= HELD) {
        const float d = to_f32(t.v[e]) - m;
        y[e] = LOG ? d - lg : exp_for<TOut>(d) * inv;
      } else if constexpr (IN_PLACE) {
        y[e] = LOG ? to_f32(raw[v].v[e]) - lg : to_f32(raw[v].v[e]) * inv;
      } else {
        const float d = to_f32(raw[v].v[e]) - m;
        y[e] = LOG ? d - lg : exp_for<TOut>(d) * inv;
      }
    }
    if (vi < static_cast<uint32_t>(nvec)) {
      // (a uniform base per vector plus one lane offset for all of them: an offset per vector
      // would be kept in a register each from the loads on)
      TOut* at = reinterpret_cast<TOut*>(dst_b + static_cast<size_t>(v) * (WAVES * kWave * EPV * sizeof(TOut)) +
                                         lane_vec * static_cast<uint32_t>(EPV * sizeof(TOut)));
      if constexpr (PEEL) {
        store_converted<TOut, EPV, STREAM>(at, y);
      } else {
        store_converted_unaligned<TOut, EPV>(at, y);
      }
    }
    if constexpr (BLOCK == 512) __builtin_amdgcn_sched_barrier(0);
  }
  if (edge >= 0) dst[edge] = from_f32<TOut>(LOG ? xt - lg : xt * inv);
}

template <typename TIn, typename TOut, int VPL, bool LOG, int BLOCK = 1024, int HELD = VPL>
static int launch_long_rows(TOut* out, const TIn* in, int64_t rows, int64_t cols,
                            hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(rows)), block(BLOCK);
  const int c = static_cast<int>(cols);
  // rows that fit 52 registers per lane take the kernel that shares a CU between two rows
  // (16-bit rows in 1024-thread workgroups; fp32 rows, which would spill there, in 512-thread
  // workgroups with twice the registers)
  constexpr bool LEAN = (sizeof(TIn) == 2 && VPL > 4) || BLOCK == 512;
#define TMB_LONG(PEEL, STREAM)                                                                        \
  do {                                                                                                \
    if constexpr (LEAN)                                                                               \
      softmax_long_rows_lean_kernel<TIn, TOut, VPL, LOG, PEEL, STREAM, BLOCK, HELD><<<grid, block, 0, stream>>>(out, in, c); \
    else                                                                                              \
      softmax_long_rows_kernel<TIn, TOut, VPL, LOG, PEEL, STREAM><<<grid, block, 0, stream>>>(out, in, c);      \
  } while (0)
  if constexpr (sizeof(TIn) == sizeof(TOut)) {
    if ((reinterpret_cast<uintptr_t>(in) & 15u) == (reinterpret_cast<uintptr_t>(out) & 15u)) {
      if (rows * cols * static_cast<int64_t>(sizeof(TIn) + sizeof(TOut)) >= (int64_t{256} << 20)) {
        TMB_LONG(true, true);
      } else {
        TMB_LONG(true, false);
      }
      return check_launch();
    }
  }
  TMB_LONG(false, false);
#undef TMB_LONG
  return check_launch();
}

// Any width / alignment. One block per row.
template <typename TIn, typename TOut, bool LOG, bool SCALED>
__global__ __launch_bounds__(256) void softmax_generic_kernel(TOut* __restrict__ out,
                                                              const TIn* __restrict__ in,
                                                              int64_t rows, int64_t cols,
                                                              SoftmaxScale sc) {
  __shared__ float slot[4];
  const int wave = threadIdx.x >> 6;
  const float neg_inf = -__builtin_inff();
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const TIn* src = in + row * cols;
    TOut* dst = out + row * cols;
    const int64_t last_col = (SCALED && sc.q_len > 0) ? row % sc.q_len : cols - 1;
    auto value = [&](int64_t j) {
      if constexpr (SCALED) {
        if (j > last_col) return neg_inf;
        float xs = to_f32(src[j]) * sc.scale;
        if (sc.round_scaled) xs = to_f32(from_f32<TIn>(xs));
        return xs;
      } else {
        return to_f32(src[j]);
      }
    };
    float m = neg_inf;
    for (int64_t j = threadIdx.x; j < cols; j += 256) m = fmaxf(m, value(j));
    m = wave_max(m);
    m = group_reduce(m, slot, wave, 0, 4, MaxOp{});
    float s = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += 256) s += exp_for<TOut>(value(j) - m);
    s = wave_sum(s);
    s = group_reduce(s, slot, wave, 0, 4, SumOp{});
    if (LOG) {
      const float lg = logf(s);
      for (int64_t j = threadIdx.x; j < cols; j += 256)
        dst[j] = from_f32<TOut>(value(j) - m - lg);
    } else {
      const float inv = 1.0f / s;
      for (int64_t j = threadIdx.x; j < cols; j += 256)
        dst[j] = from_f32<TOut>(exp_for<TOut>(value(j) - m) * inv);
    }
  }
}

template <typename TIn, typename TOut, bool LOG, bool SCALED, int WPR, int VPL, int BLOCK>
static int launch_regs(TOut* out, const TIn* in, int64_t rows, int64_t cols, SoftmaxScale sc,
                       hipStream_t stream) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int RPW = 1;  // several rows per wave measured slower at every width
  constexpr int ROWS_PER_BLOCK = (BLOCK / kWave) / WPR * RPW;
  const int64_t blocks = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  // Streams when the tensor cannot live in the 256 MB Infinity Cache anyway.
  const bool stream_hint = rows * cols * static_cast<int64_t>(sizeof(TIn) + sizeof(TOut)) >= (int64_t{256} << 20);
  if (stream_hint) {
    softmax_regs_kernel<TIn, TOut, WPR, VPL, RPW, LOG, true, SCALED, BLOCK>
        <<<dim3(static_cast<unsigned>(blocks)), dim3(BLOCK), 0, stream>>>(out, in, rows, static_cast<int>(cols), sc);
  } else {
    softmax_regs_kernel<TIn, TOut, WPR, VPL, RPW, LOG, false, SCALED, BLOCK>
        <<<dim3(static_cast<unsigned>(blocks)), dim3(BLOCK), 0, stream>>>(out, in, rows, static_cast<int>(cols), sc);
  }
  return check_launch();
}

template <typename TIn, typename TOut, bool LOG, bool SCALED>
static int softmax_dispatch(TOut* out, const TIn* in, int64_t rows, int64_t cols, SoftmaxScale sc,
                            hipStream_t stream) {
  constexpr int EPV = Vec16<TIn>::N;
  constexpr int MAXV = 64 / EPV;  // at most 64 fp32 values of a row per lane
  const bool vec_ok = (cols % EPV == 0) && aligned16(in) && aligned16(out) &&
                      rows < (int64_t{1} << 31);
  const int64_t nvec = cols / EPV;
  if (vec_ok && nvec <= 16 * 64 * MAXV) {
// Measured on this GPU (fp32 rows of 256 .. 4096 columns): the fewer bytes a wave holds, the
    // better the loads and stores of different waves interleave; one or two vectors per lane and
    // more waves per row beat one wave per row by 8-12 %.
    if (nvec <= 64) return launch_regs<TIn, TOut, LOG, SCALED, 1, 1, 256>(out, in, rows, cols, sc, stream);
    if (nvec <= 128) {
      // 16-bit rows of 1024 columns: one wave per row with two vectors per lane (no LDS, no
      // barrier) measured 63 us against 66-69 us for two waves per row on [98304, 1024] bf16
      if constexpr (sizeof(TIn) == 2)
        return launch_regs<TIn, TOut, LOG, SCALED, 1, 2, 256>(out, in, rows, cols, sc, stream);
      return launch_regs<TIn, TOut, LOG, SCALED, 2, 1, 256>(out, in, rows, cols, sc, stream);
    }
    if (nvec <= 256) return launch_regs<TIn, TOut, LOG, SCALED, 2, 2, 256>(out, in, rows, cols, sc, stream);
    if (nvec <= 512) return launch_regs<TIn, TOut, LOG, SCALED, 4, 2, 256>(out, in, rows, cols, sc, stream);
    if (nvec <= 1024) return launch_regs<TIn, TOut, LOG, SCALED, 8, 2, 512>(out, in, rows, cols, sc, stream);
    if (nvec <= 2048) return launch_regs<TIn, TOut, LOG, SCALED, 16, 2, 1024>(out, in, rows, cols, sc, stream);
    if (nvec <= 4096) return launch_regs<TIn, TOut, LOG, SCALED, 16, 4, 1024>(out, in, rows, cols, sc, stream);
    if constexpr (MAXV >= 16) {
      if (nvec <= 8192) return launch_regs<TIn, TOut, LOG, SCALED, 16, 8, 1024>(out, in, rows, cols, sc, stream);
    }
    return launch_regs<TIn, TOut, LOG, SCALED, 16, MAXV, 1024>(out, in, rows, cols, sc, stream);
  }
  if constexpr (!SCALED) {
    // ragged or unaligned rows long enough to occupy a 1024-thread workgroup (a row needs at most
    // cols / EPV vector slots, whatever its offset)
    if (cols >= 4096 && cols / EPV <= 1024 * MAXV && rows < (int64_t{1} << 31)) {
      if (cols / EPV <= 1024 * 2) return launch_long_rows<TIn, TOut, 2, LOG>(out, in, rows, cols, stream);
      if (cols / EPV <= 1024 * 4) return launch_long_rows<TIn, TOut, 4, LOG>(out, in, rows, cols, stream);
      if constexpr (MAXV == 8) {  // 16-bit rows: up to 65536 columns in 32 registers
        if (cols / EPV <= 1024 * 7) return launch_long_rows<TIn, TOut, 7, LOG>(out, in, rows, cols, stream);
        return launch_long_rows<TIn, TOut, 8, LOG>(out, in, rows, cols, stream);
      } else {
        if constexpr (sizeof(TIn) == 4) {
          // (16384 x 50257 log-softmax: 1.30 -> 1.26 ms)
          if (cols / EPV <= 512 * 13) return launch_long_rows<TIn, TOut, 13, LOG, 512>(out, in, rows, cols, stream);
          if (cols / EPV <= 512 * 25) return launch_long_rows<TIn, TOut, 25, LOG, 512, (LOG ? 17 : 15)>(out, in, rows, cols, stream);
        }
        return launch_long_rows<TIn, TOut, MAXV, LOG>(out, in, rows, cols, stream);
      }
    }
  }
  const int64_t blocks = rows < 65536 * 16 ? rows : 65536 * 16;
  softmax_generic_kernel<TIn, TOut, LOG, SCALED>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(out, in, rows, cols, sc);
  return check_launch();
}

template <bool LOG, bool SCALED>
static int softmax_by_dtype(void* out, const void* in, int64_t rows, int64_t cols, int in_dtype,
                            int out_dtype, SoftmaxScale sc, hipStream_t s) {
  if (in_dtype == TMB_F32 && out_dtype == TMB_F32)
    return softmax_dispatch<float, float, LOG, SCALED>((float*)out, (const float*)in, rows, cols, sc, s);
  if (in_dtype == TMB_F16 && out_dtype == TMB_F16)
    return softmax_dispatch<f16_t, f16_t, LOG, SCALED>((f16_t*)out, (const f16_t*)in, rows, cols, sc, s);
  if (in_dtype == TMB_BF16 && out_dtype == TMB_BF16)
    return softmax_dispatch<bf16_t, bf16_t, LOG, SCALED>((bf16_t*)out, (const bf16_t*)in, rows, cols, sc, s);
  if constexpr (!SCALED) {  // widening outputs exist for the plain form only
    if (in_dtype == TMB_F16 && out_dtype == TMB_F32)
      return softmax_dispatch<f16_t, float, LOG, false>((float*)out, (const f16_t*)in, rows, cols, sc, s);
    if (in_dtype == TMB_BF16 && out_dtype == TMB_F32)
      return softmax_dispatch<bf16_t, float, LOG, false>((float*)out, (const bf16_t*)in, rows, cols, sc, s);
  }
  return TMB_ERR_UNSUPPORTED;
}

}  // namespace tmb

extern "C" int tmb_softmax_rows(void* out, const void* in, int64_t rows, int64_t cols,
                                int in_dtype, int out_dtype, int log_mode, void* stream) {
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const tmb::SoftmaxScale none{1.0f, 0, 0};
  return log_mode
             ? tmb::softmax_by_dtype<true, false>(out, in, rows, cols, in_dtype, out_dtype, none, s)
             : tmb::softmax_by_dtype<false, false>(out, in, rows, cols, in_dtype, out_dtype, none, s);
}

extern "C" int tmb_softmax_rows_scaled(void* out, const void* in, int64_t rows, int64_t cols,
                                       int dtype, float scale, int round_scaled, int64_t q_len,
                                       void* stream) {
  if (rows < 0 || cols < 0 || q_len < 0 || q_len > 0x7fffffff) return TMB_ERR_INVALID_ARGUMENT;
  if (!(scale == scale)) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return TMB_OK;
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const tmb::SoftmaxScale sc{scale, round_scaled ? 1 : 0, static_cast<int>(q_len)};
  return tmb::softmax_by_dtype<false, true>(out, in, rows, cols, dtype, dtype, sc, s);
}
