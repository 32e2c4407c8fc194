// Row reductions (sum / mean / amax) and first-occurrence argmax for gfx950.
//
// Work decomposition depends only on (rows, cols): every row is cut into `splits` contiguous
// chunks; one workgroup streams one chunk with 16-byte loads (scalar head/tail for unaligned
// rows, e.g. 50257-wide vocab rows), reduces it in a fixed order (per-lane strided accumulate
// -> DPP wave tree -> LDS combine in wave order) and either writes the final value
// (splits == 1) or a partial into the caller's workspace, which a second launch combines in
// chunk order. No atomics anywhere, so floating-point results are bit-reproducible.
//
// Arithmetic contract (torch_mojo_backend/eager_kernels/reduction_ops.mojo:161-194,
// nn_ops.mojo:981-1027, nn_ops.mojo:1424-1478): floats accumulate in fp32 and are cast once;
// integers reduce in their own type; argmax keeps the lower index among equal values at
// every combine step.
#include "tmb_common.h"

#include <mutex>

namespace tmb {

// Scratch of the entry point that allocates nothing (tmb_reduce_rows_static): the partials of a
// split reduction live in this array instead of a caller's workspace. Every GPU the library runs
// on holds its own copy until the process ends. In host code the name `scratch` is only a handle
// for hipGetSymbolAddress; kernels get the per-device address that call returns.
constexpr size_t kStaticScratchBytes = TMB_REDUCE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kRedBlock = 256;
constexpr int kRedWaves = kRedBlock / kWave;

struct SplitPlan {
  int splits;
  int64_t chunk;  // elements per chunk (multiple of 64 unless splits == 1)
};

// Must stay a pure function of (rows, cols): the Python side sizes the workspace from it and
// reproducibility relies on it.
static SplitPlan plan_splits(int64_t rows, int64_t cols) {
  constexpr int64_t kTargetBlocks = 8192;   // 32 chunks per CU on 256 CUs: dynamic balance
  constexpr int64_t kMinChunk = 16384;      // elements; below this a split is not worth a launch
  constexpr int64_t kMaxChunk = int64_t{1} << 30;
  int64_t splits = 1;
  if (rows < kTargetBlocks / 2) {
    splits = (kTargetBlocks + rows - 1) / rows;
    const int64_t by_size = cols / kMinChunk;
    if (splits > by_size) splits = by_size;
    if (splits < 1) splits = 1;
  }
  const int64_t need = (cols + kMaxChunk - 1) / kMaxChunk;
  if (splits < need) splits = need;
  if (splits > 8192) splits = 8192;
  int64_t chunk = (cols + splits - 1) / splits;
  if (splits > 1) {
    chunk = (chunk + 63) / 64 * 64;
    splits = (cols + chunk - 1) / chunk;
  }
  return SplitPlan{static_cast<int>(splits), chunk};
}

// ---------------------------------------------------------------------------
// Value reductions
// ---------------------------------------------------------------------------
template <typename Acc>
struct AccSum {
  using acc_t = Acc;
  static __device__ __forceinline__ Acc identity() { return Acc(0); }
  static __device__ __forceinline__ Acc combine(Acc a, Acc b) { return a + b; }
};
// Float max carried as (value, saw_nan) so the streaming loop is one v_max + one compare.
struct FMax {
  float v;
  bool nan;
};
struct AccFMax {
  using acc_t = FMax;
  static __device__ __forceinline__ FMax identity() { return FMax{-__builtin_inff(), false}; }
  static __device__ __forceinline__ FMax combine(FMax a, FMax b) {
    return FMax{fmaxf(a.v, b.v), a.nan || b.nan};
  }
};
template <typename I>
struct AccIMax {
  using acc_t = I;
  static __device__ __forceinline__ I identity() {
    if constexpr (sizeof(I) == 8) {
      return static_cast<I>(INT64_MIN);
    } else {
      return static_cast<I>(INT32_MIN);
    }
  }
  static __device__ __forceinline__ I combine(I a, I b) { return a > b ? a : b; }
};

template <typename T>
__device__ __forceinline__ void accumulate(float& acc, T x) { acc += to_f32(x); }
__device__ __forceinline__ void accumulate(int64_t& acc, int64_t x) { acc += x; }
template <typename T>
__device__ __forceinline__ void accumulate(FMax& acc, T x) {
  const float f = to_f32(x);
  acc.v = fmaxf(acc.v, f);
  acc.nan = acc.nan || (f != f);
}
__device__ __forceinline__ void accumulate_imax(int64_t& acc, int64_t x) { acc = x > acc ? x : acc; }
__device__ __forceinline__ void accumulate_imax(int32_t& acc, int32_t x) { acc = x > acc ? x : acc; }

template <typename Policy, typename T, bool IMAX>
__device__ __forceinline__ void acc_one(typename Policy::acc_t& acc, T x) {
  if constexpr (IMAX) {
    accumulate_imax(acc, x);
  } else {
    accumulate(acc, x);
  }
}

// Generic (non-fp32-sum) wave butterfly; used for exact/associative combines.
template <typename V>
__device__ __forceinline__ V shfl_xor_any(V v, int mask) {
  static_assert(sizeof(V) % 4 == 0, "4-byte multiples only");
  union {
    V v;
    int w[sizeof(V) / 4];
  } a, b;
  a.v = v;
#pragma unroll
  for (int i = 0; i < static_cast<int>(sizeof(V) / 4); ++i) b.w[i] = __shfl_xor(a.w[i], mask, kWave);
  return b.v;
}

struct FMaxPacked {
  float v;
  int nan;
};

template <typename Policy>
__device__ __forceinline__ typename Policy::acc_t wave_combine(typename Policy::acc_t a) {
  using A = typename Policy::acc_t;
  if constexpr (__is_same(A, float)) {
    return wave_sum(a);
  } else if constexpr (__is_same(A, FMax)) {
    const float v = wave_max(a.v);
    const bool any_nan = __builtin_amdgcn_ballot_w64(a.nan) != 0;
    return FMax{v, any_nan};
  } else {
#pragma unroll
    for (int mask = 1; mask < kWave; mask <<= 1) a = Policy::combine(a, shfl_xor_any(a, mask));
    return a;
  }
}

// Streams [p, p+n) with `NT` cooperating threads (this thread is `tid`) in a fixed order.
template <typename Policy, typename T, bool IMAX, int NT>
__device__ __forceinline__ typename Policy::acc_t stream_range(const T* __restrict__ p, int64_t n,
                                                               int tid) {
  using A = typename Policy::acc_t;
  constexpr int EPV = Vec16<T>::N;
  A acc0 = Policy::identity(), acc1 = Policy::identity();
  A acc2 = Policy::identity(), acc3 = Policy::identity();
  const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
  int64_t head = static_cast<int64_t>(((16u - (addr & 15u)) & 15u) / sizeof(T));
  if (head > n) head = n;
  if (tid < head) acc_one<Policy, T, IMAX>(acc0, p[tid]);
  const T* body = p + head;
  const int64_t nvec = (n - head) / EPV;
  int64_t i = tid;
  for (; i + 3 * NT < nvec; i += 4 * NT) {
    const Vec16<T> v0 = load_vec16_stream(body + i * EPV);
    const Vec16<T> v1 = load_vec16_stream(body + (i + NT) * EPV);
    const Vec16<T> v2 = load_vec16_stream(body + (i + 2 * NT) * EPV);
    const Vec16<T> v3 = load_vec16_stream(body + (i + 3 * NT) * EPV);
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      acc_one<Policy, T, IMAX>(acc0, v0.v[e]);
      acc_one<Policy, T, IMAX>(acc1, v1.v[e]);
      acc_one<Policy, T, IMAX>(acc2, v2.v[e]);
      acc_one<Policy, T, IMAX>(acc3, v3.v[e]);
    }
  }
  for (; i < nvec; i += NT) {
    const Vec16<T> v0 = load_vec16_stream(body + i * EPV);
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc_one<Policy, T, IMAX>(acc0, v0.v[e]);
  }
  const int64_t tail = head + nvec * EPV;
  if (tail + tid < n) acc_one<Policy, T, IMAX>(acc1, p[tail + tid]);
  return Policy::combine(Policy::combine(acc0, acc1), Policy::combine(acc2, acc3));
}

template <typename A>
struct AccStore {  // what a partial looks like in the workspace (8 bytes per partial)
  static __device__ __forceinline__ void put(void* ws, int64_t i, A a) {
    static_cast<A*>(ws)[i] = a;
  }
  static __device__ __forceinline__ A get(const void* ws, int64_t i) {
    return static_cast<const A*>(ws)[i];
  }
};
template <>
struct AccStore<FMax> {
  static __device__ __forceinline__ void put(void* ws, int64_t i, FMax a) {
    static_cast<FMaxPacked*>(ws)[i] = FMaxPacked{a.v, a.nan ? 1 : 0};
  }
  static __device__ __forceinline__ FMax get(const void* ws, int64_t i) {
    const FMaxPacked p = static_cast<const FMaxPacked*>(ws)[i];
    return FMax{p.v, p.nan != 0};
  }
};

template <typename TOut, typename A>
__device__ __forceinline__ TOut finalize(A a, int op, int64_t cols) {
  if constexpr (__is_same(A, FMax)) {
    return from_f32<TOut>(a.nan ? __builtin_nanf("") : a.v);
  } else if constexpr (__is_same(A, float)) {
    return from_f32<TOut>(op == TMB_MEAN ? a / static_cast<float>(cols) : a);
  } else {
    return static_cast<TOut>(a);
  }
}

// One workgroup per (row, split) chunk.
template <typename Policy, typename T, bool IMAX>
__global__ __launch_bounds__(kRedBlock) void reduce_chunk_kernel(T* __restrict__ out,
                                                                 void* __restrict__ ws,
                                                                 const T* __restrict__ in,
                                                                 int64_t rows, int64_t cols,
                                                                 int splits, int64_t chunk, int op) {
  using A = typename Policy::acc_t;
  __shared__ A slot[kRedWaves];
  const int64_t item = blockIdx.x;
  const int64_t row = item / splits;
  const int split = static_cast<int>(item - row * splits);
  const int64_t c0 = static_cast<int64_t>(split) * chunk;
  int64_t n = cols - c0;
  if (n > chunk) n = chunk;
  A acc = stream_range<Policy, T, IMAX, kRedBlock>(in + row * cols + c0, n, threadIdx.x);
  acc = wave_combine<Policy>(acc);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) slot[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    A r = slot[0];
#pragma unroll
    for (int w = 1; w < kRedWaves; ++w) r = Policy::combine(r, slot[w]);
    if (splits == 1) {
      out[row] = finalize<T>(r, op, cols);
    } else {
      AccStore<A>::put(ws, item, r);
    }
  }
}

// One wave per row: rows that are short enough that a workgroup per row would idle lanes.
template <typename Policy, typename T, bool IMAX>
__global__ __launch_bounds__(kRedBlock) void reduce_wave_kernel(T* __restrict__ out,
                                                                const T* __restrict__ in,
                                                                int64_t rows, int64_t cols, int op) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRedWaves + (threadIdx.x >> 6);
  if (row >= rows) return;  // wave-uniform
  auto acc = stream_range<Policy, T, IMAX, kWave>(in + row * cols, cols, threadIdx.x & 63);
  acc = wave_combine<Policy>(acc);
  if ((threadIdx.x & 63) == 0) out[row] = finalize<T>(acc, op, cols);
}

// Second stage: combines the `splits` partials of each row. Thread t takes partials t, t+NT, ...
// (independent loads, all in flight at once), then the usual wave tree and a fixed-order
// combine across waves.
template <typename Policy, typename T, int kFinalBlock>
__global__ __launch_bounds__(kFinalBlock) void reduce_final_kernel(T* __restrict__ out,
                                                                  const void* __restrict__ ws,
                                                                  int64_t rows, int64_t cols,
                                                                  int splits, int op) {
  using A = typename Policy::acc_t;
  constexpr int WAVES = kFinalBlock / kWave;
  __shared__ A slot[WAVES];
  const int64_t row = blockIdx.x;
  A acc = Policy::identity();
  for (int i = threadIdx.x; i < splits; i += kFinalBlock)
    acc = Policy::combine(acc, AccStore<A>::get(ws, row * splits + i));
  acc = wave_combine<Policy>(acc);
  if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    A r = slot[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) r = Policy::combine(r, slot[w]);
    out[row] = finalize<T>(r, op, cols);
  }
}

template <typename Policy, typename T, bool IMAX>
static int launch_reduce(void* out_, const void* in_, int64_t rows, int64_t cols, int op,
                         void* ws, size_t ws_bytes, hipStream_t stream) {
  T* out = static_cast<T*>(out_);
  const T* in = static_cast<const T*>(in_);
  const SplitPlan plan = plan_splits(rows, cols);
  if (plan.splits == 1 && cols * static_cast<int64_t>(sizeof(T)) <= 8192) {
    const int64_t blocks = (rows + kRedWaves - 1) / kRedWaves;
    if (blocks >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
    reduce_wave_kernel<Policy, T, IMAX>
        <<<dim3(static_cast<unsigned>(blocks)), dim3(kRedBlock), 0, stream>>>(out, in, rows, cols, op);
    return check_launch();
  }
  const int64_t items = rows * plan.splits;
  if (items >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  if (plan.splits > 1) {
    if (ws == nullptr || ws_bytes < static_cast<size_t>(items) * 16) return TMB_ERR_WORKSPACE;
  }
  reduce_chunk_kernel<Policy, T, IMAX><<<dim3(static_cast<unsigned>(items)), dim3(kRedBlock), 0, stream>>>(
      out, ws, in, rows, cols, plan.splits, plan.chunk, op);
  int rc = check_launch();
  if (rc != 0 || plan.splits == 1) return rc;
  if (plan.splits > 256) {
    reduce_final_kernel<Policy, T, 1024><<<dim3(static_cast<unsigned>(rows)), dim3(1024), 0, stream>>>(
        out, ws, rows, cols, plan.splits, op);
  } else {
    reduce_final_kernel<Policy, T, 64><<<dim3(static_cast<unsigned>(rows)), dim3(64), 0, stream>>>(
        out, ws, rows, cols, plan.splits, op);
  }
  return check_launch();
}

// ---------------------------------------------------------------------------
// Argmax
// ---------------------------------------------------------------------------
template <typename V>
struct Best {
  V val;
  int64_t idx;
};

template <typename V>
__device__ __forceinline__ bool is_nan(V v) {
  if constexpr (__is_same(V, float)) {
    return v != v;
  } else {
    return false;
  }
}

// true when b must replace a: NaN beats numbers, greater beats smaller, ties keep the lower index.
template <typename V>
__device__ __forceinline__ bool replaces(const Best<V>& a, const Best<V>& b) {
  if (a.idx < 0) return b.idx >= 0;
  if (b.idx < 0) return false;
  const bool an = is_nan(a.val), bn = is_nan(b.val);
  if (an || bn) {
    if (an && bn) return b.idx < a.idx;
    return bn;
  }
  if (b.val > a.val) return true;
  if (b.val == a.val) return b.idx < a.idx;
  return false;
}

template <typename V>
__device__ __forceinline__ Best<V> best_combine(Best<V> a, Best<V> b) {
  return replaces(a, b) ? b : a;
}

template <typename T>
struct ArgTraits {
  using val_t = float;
  static __device__ __forceinline__ float conv(T x) { return to_f32(x); }
};
template <>
struct ArgTraits<int64_t> {
  using val_t = int64_t;
  static __device__ __forceinline__ int64_t conv(int64_t x) { return x; }
};
template <>
struct ArgTraits<int32_t> {
  using val_t = int32_t;
  static __device__ __forceinline__ int32_t conv(int32_t x) { return x; }
};

// Per-thread scan in ascending index order: strict "greater" keeps the first occurrence;
// the first NaN sticks.
template <typename V>
__device__ __forceinline__ void scan_one(V& best, int& best_off, V x, int off) {
  bool take;
  if constexpr (__is_same(V, float)) {
    take = (best_off < 0) || (x > best) || ((x != x) && (best == best));
  } else {
    take = (best_off < 0) || (x > best);
  }
  best = take ? x : best;
  best_off = take ? off : best_off;
}

// U 16-byte loads per lane are requested before the first of them is compared; a batch that
// reaches past the end of the range is cut short lane by lane, so there is no one-load-at-a-time
// remainder loop (a row of 50257 floats over 1024 lanes is 12.3 vectors per lane: two batches of
// seven instead of three of four plus one).
template <typename T, int NT, int U = 4>
__device__ __forceinline__ Best<typename ArgTraits<T>::val_t> argmax_range(const T* __restrict__ p,
                                                                           int64_t n, int tid,
                                                                           int64_t base) {
  using V = typename ArgTraits<T>::val_t;
  constexpr int EPV = Vec16<T>::N;
  V best = V(0);
  int off = -1;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
  int head = static_cast<int>(((16u - (addr & 15u)) & 15u) / sizeof(T));
  if (head > n) head = static_cast<int>(n);
  if (tid < head) scan_one(best, off, ArgTraits<T>::conv(p[tid]), tid);
  const T* body = p + head;
  const int nvec = static_cast<int>((n - head) / EPV);
  for (int i = tid; i < nvec; i += U * NT) {
    Vec16<T> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i + u * NT < nvec) v[u] = load_vec16_stream(body + static_cast<int64_t>(i + u * NT) * EPV);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i + u * NT < nvec) {
#pragma unroll
        for (int e = 0; e < EPV; ++e)
          scan_one(best, off, ArgTraits<T>::conv(v[u].v[e]), head + (i + u * NT) * EPV + e);
      }
  }
  const int tail = head + nvec * EPV;
  if (tail + tid < n) scan_one(best, off, ArgTraits<T>::conv(p[tail + tid]), tail + tid);
  return Best<V>{best, off < 0 ? int64_t{-1} : base + off};
}

template <typename V>
__device__ __forceinline__ Best<V> wave_best(Best<V> b) {
#pragma unroll
  for (int mask = 1; mask < kWave; mask <<= 1) {
    Best<V> o;
    o.val = shfl_xor_any(b.val, mask);
    o.idx = shfl_xor_any(b.idx, mask);
    b = best_combine(b, o);
  }
  return b;
}

template <typename V>
struct alignas(16) BestSlot {
  int64_t idx;
  V val;
};

template <typename T, int BLK, int U = 4>
__global__ __launch_bounds__(BLK) void argmax_chunk_kernel(int64_t* __restrict__ out,
                                                           void* __restrict__ ws,
                                                           const T* __restrict__ in, int64_t rows,
                                                           int64_t cols, int splits,
                                                           int64_t chunk) {
  using V = typename ArgTraits<T>::val_t;
  constexpr int WAVES = BLK / kWave;
  __shared__ BestSlot<V> slot[WAVES];
  const int64_t item = blockIdx.x;
  const int64_t row = item / splits;
  const int split = static_cast<int>(item - row * splits);
  const int64_t c0 = static_cast<int64_t>(split) * chunk;
  int64_t n = cols - c0;
  if (n > chunk) n = chunk;
  Best<V> b = argmax_range<T, BLK, U>(in + row * cols + c0, n, threadIdx.x, c0);
  b = wave_best(b);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) slot[wave] = BestSlot<V>{b.idx, b.val};
  __syncthreads();
  if (threadIdx.x == 0) {
    Best<V> r{slot[0].val, slot[0].idx};
#pragma unroll
    for (int w = 1; w < WAVES; ++w) r = best_combine(r, Best<V>{slot[w].val, slot[w].idx});
    if (splits == 1) {
      out[row] = r.idx;
    } else {
      static_cast<BestSlot<V>*>(ws)[item] = BestSlot<V>{r.idx, r.val};
    }
  }
}

template <typename T, int kFinalBlock>
__global__ __launch_bounds__(kFinalBlock) void argmax_final_kernel(int64_t* __restrict__ out,
                                                                  const void* __restrict__ ws,
                                                                  int64_t rows, int splits) {
  using V = typename ArgTraits<T>::val_t;
  constexpr int WAVES = kFinalBlock / kWave;
  __shared__ BestSlot<V> slot[WAVES];
  const int64_t row = blockIdx.x;
  Best<V> b{V(0), int64_t{-1}};
  for (int i = threadIdx.x; i < splits; i += kFinalBlock) {
    const BestSlot<V> s = static_cast<const BestSlot<V>*>(ws)[row * splits + i];
    b = best_combine(b, Best<V>{s.val, s.idx});
  }
  b = wave_best(b);
  if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = BestSlot<V>{b.idx, b.val};
  __syncthreads();
  if (threadIdx.x == 0) {
    Best<V> r{slot[0].val, slot[0].idx};
#pragma unroll
    for (int w = 1; w < WAVES; ++w) r = best_combine(r, Best<V>{slot[w].val, slot[w].idx});
    out[row] = r.idx;
  }
}

// ---------------------------------------------------------------------------
// Argmax of floating-point rows, a vector at a time.
//
// The scan above spends six to seven instructions on every element (three compares, two
// selects and their mask arithmetic), and a wave64 instruction occupies its SIMD for four
// cycles: 25 M elements are 4-5 us of vector ALU time on the whole chip, next to 15 us of memory
// time. Here a lane looks at one 16-byte vector at a time: the vector's maximum (v_max3),
// one strict compare with the lane's maximum so far, and on "greater" the lane keeps that vector
// (raw) and its number. Strict "greater" keeps the first vector that reached the lane's maximum,
// and the first element equal to the maximum inside the kept vector is the lane's first
// occurrence. v_max ignores NaN, so a float sum of everything the lane saw runs beside it: it is
// NaN exactly when the lane saw a NaN or infinities of both signs, and then the whole workgroup
// redoes its range with the exact scan (first NaN wins), reading it again. Half the instructions
// per element, nothing kept in registers but one vector.
//
// Work units are small (256 lanes, at most seven vectors each, about 28 KB): measured on
// [512, 50257] fp32, eight units per row plus the combining launch take 20 us where one
// 1024-lane workgroup per row took 23 (the units alone 17; a plain read of the same bytes 15.7).
// ---------------------------------------------------------------------------
constexpr int kArgBlock = 256;
constexpr int kArgMaxVectors = 7;  // per lane

template <typename T>
struct LaneBest {
  float m;
  Vec16<T> kept;
  int u;
  float sum;
};

template <typename T>
__device__ __forceinline__ void lane_step(LaneBest<T>& t, const Vec16<T>& x, int u) {
  constexpr int EPV = Vec16<T>::N;
  float f[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) f[e] = to_f32(x.v[e]);
  float m = __builtin_fmaxf(f[0], f[1]);
  float s = f[0] + f[1];
#pragma unroll
  for (int e = 2; e < EPV; e += 2) {
    m = __builtin_fmaxf(__builtin_fmaxf(m, f[e]), f[e + 1]);
    s += f[e] + f[e + 1];
  }
  const bool take = m > t.m;
  t.m = take ? m : t.m;
  const raw16_t xr = __builtin_bit_cast(raw16_t, x), kr = __builtin_bit_cast(raw16_t, t.kept);
  raw16_t nr;
#pragma unroll
  for (int w = 0; w < 4; ++w) nr[w] = take ? xr[w] : kr[w];
  t.kept = __builtin_bit_cast(Vec16<T>, nr);
  t.u = take ? u : t.u;
  t.sum += s;
}

__device__ __forceinline__ int wave_min_i32(int v) {
  v = min(v, dpp_i32<kDppQuadXor1>(v));
  v = min(v, dpp_i32<kDppQuadXor2>(v));
  v = min(v, dpp_i32<kDppRowHalfMirror>(v));
  v = min(v, dpp_i32<kDppRowMirror>(v));
  v = min(v, __shfl_xor(v, 16, kWave));
  return min(v, __shfl_xor(v, 32, kWave));
}

// One workgroup per (row, split): columns [split * chunk, min(cols, (split + 1) * chunk)) of the
// row, chunk <= kArgBlock * U vectors. splits == 1 writes the row's index, otherwise a
// (value, index) partial for argmax_final_kernel.
// BLOCK = 1024, P = 2: a whole row of up to 1024 * 2 * U vectors per workgroup, in two batches
// of U vectors per lane (two such workgroups share a CU at 64 registers): when there is at least
// a row per CU, the launch that combines the partials costs more than the finer units save.
template <typename T, int U, int BLOCK = kArgBlock, int P = 1>
__global__ __launch_bounds__(BLOCK, BLOCK == 1024 ? 8 : 1) void argmax_vec_kernel(int64_t* __restrict__ out,
                                                                               void* __restrict__ ws,
                                                                               const T* __restrict__ in,
                                                                               int64_t cols, int splits, int chunk) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int WAVES = BLOCK / kWave;
  constexpr int kNone = 0x7fffffff;
  __shared__ float smax[WAVES];
  __shared__ int sflag[WAVES];
  __shared__ int soff[WAVES];
  __shared__ BestSlot<float> sbest[WAVES];
  const int tid = threadIdx.x, wave = tid >> 6;
  const int64_t item = blockIdx.x;
  const int64_t row = item / splits;
  const int split = static_cast<int>(item - row * splits);
  const int64_t c0 = static_cast<int64_t>(split) * chunk;
  const T* p = in + row * cols + c0;
  int n = static_cast<int>(cols - c0 < chunk ? cols - c0 : chunk);
  const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
  int head = static_cast<int>(((16u - (addr & 15u)) & 15u) / sizeof(T));
  if (head > n) head = n;
  const T* body = p + head;
  const int nvec = (n - head) / EPV;
  const int tail = head + nvec * EPV;
  // up to EPV - 1 elements in front of the first and behind the last whole vector: one each for
  // the first lanes. Lanes without one (and vector slots past the end, below) read element 0 /
  // vector 0 again instead of branching: a copy can equal the maximum but never raise it, and a
  // lane that kept a copy is recognised by its vector number.
  const bool has_head = tid < head, has_tail = tail + tid < n;
  const float hv = to_f32(__builtin_nontemporal_load(p + (has_head ? tid : 0)));
  const float tv = to_f32(__builtin_nontemporal_load(p + (has_tail ? tail + tid : 0)));
  const float ninf = -__builtin_inff();
  LaneBest<T> t;
  t.m = ninf;
  t.u = -1;
  t.sum = 0.0f;
#pragma unroll 1
  for (int pass = 0; pass < P; ++pass) {  // (not unrolled: the batches must not share registers)
    Vec16<T> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t at = static_cast<uint32_t>(tid + (pass * U + u) * BLOCK);
      v[u] = load_vec16_stream(body + static_cast<size_t>(at < static_cast<uint32_t>(nvec) ? at : 0u) * EPV);
    }
    if (pass == 0) t.kept = v[0];
#pragma unroll
    for (int u = 0; u < U; ++u) lane_step(t, v[u], pass * U + u);
  }

  // the lane's candidate, in ascending index order: head element, kept vector, tail element
  float m = ninf;
  int off = kNone;
  if (tid < nvec) {
    // u < 0: nothing exceeded -inf, so every element seen is -inf (or NaN: caught below) and the
    // first of them is element 0 of the lane's first vector
    const int u = t.u < 0 ? 0 : t.u;
    const int vi = tid + u * BLOCK;
    if (vi < nvec) {
      int e = EPV - 1;
#pragma unroll
      for (int k = EPV - 2; k >= 0; --k) e = to_f32(t.kept.v[k]) == t.m ? k : e;
      if (t.u < 0) e = 0;
      m = t.m;
      off = head + vi * EPV + e;
    }
    // vi >= nvec: a copy of vector 0 exceeded everything this lane owns, so lane 0 holds a
    // greater value and this lane cannot win
  }
  if (has_head && (off == kNone || !(m > hv))) { m = hv; off = tid; }
  if (has_tail && (off == kNone || tv > m)) { m = tv; off = tail + tid; }
  const float sum = t.sum + hv + tv;
  const float wm = wave_reduce(m, MaxOp{});
  const int wf = __any(sum != sum) ? 1 : 0;
  if ((tid & 63) == 0) { smax[wave] = wm; sflag[wave] = wf; }
  __syncthreads();
  float M = smax[0];
  int flag = sflag[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) { M = __builtin_fmaxf(M, smax[w]); flag |= sflag[w]; }
  if (flag == 0) {
    off = (off != kNone && m == M) ? off : kNone;
    off = wave_min_i32(off);
    if ((tid & 63) == 0) soff[wave] = off;
    __syncthreads();
    if (tid == 0) {
      int first = soff[0];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) first = min(first, soff[w]);
      if (splits == 1) {
        out[row] = first;
      } else {
        static_cast<BestSlot<float>*>(ws)[item] = BestSlot<float>{c0 + first, M};
      }
    }
  } else {
    Best<float> b = argmax_range<T, BLOCK, 4>(p, n, tid, c0);
    b = wave_best(b);
    if ((tid & 63) == 0) sbest[wave] = BestSlot<float>{b.idx, b.val};
    __syncthreads();
    if (tid == 0) {
      Best<float> r{sbest[0].val, sbest[0].idx};
#pragma unroll
      for (int w = 1; w < WAVES; ++w) r = best_combine(r, Best<float>{sbest[w].val, sbest[w].idx});
      if (splits == 1) {
        out[row] = r.idx;
      } else {
        static_cast<BestSlot<float>*>(ws)[item] = BestSlot<float>{r.idx, r.val};
      }
    }
  }
}

// How a floating-point argmax is cut into work units: a pure function of the shape. Rows
// shorter than kArgVecMinCols elements stay with the kernels above.
constexpr int64_t kArgVecMinCols = 2048;
struct ArgPlan {
  int splits;
  int chunk;    // elements
  int vectors;  // per lane, upper bound
};
static bool argmax_vec_plan(int64_t rows, int64_t cols, int elem_size, ArgPlan* plan) {
  if (rows <= 0 || cols < kArgVecMinCols || cols >= (int64_t{1} << 31) - 4096) return false;
  const int64_t epv = 16 / elem_size;
  const int64_t nvec = cols / epv;
  const int64_t unit_max = static_cast<int64_t>(kArgBlock) * kArgMaxVectors;  // vectors
  int64_t splits = (nvec + unit_max - 1) / unit_max;
  // few rows: more, smaller units (down to one vector per lane) until about eight per CU exist
  int64_t wanted = (2048 + rows - 1) / rows;
  const int64_t finest = nvec / kArgBlock;
  if (wanted > finest) wanted = finest;
  if (splits < wanted) splits = wanted;
  if (splits < 1) splits = 1;
  int64_t chunk;
  for (;; ++splits) {
    chunk = ((cols + splits - 1) / splits + 63) / 64 * 64;
    // a unit may start up to epv - 1 elements before its first whole vector
    if (chunk / epv <= unit_max) break;
  }
  splits = (cols + chunk - 1) / chunk;
  if (rows * splits >= (int64_t{1} << 31)) return false;
  plan->splits = static_cast<int>(splits);
  plan->chunk = static_cast<int>(chunk);
  plan->vectors = static_cast<int>((chunk / epv + kArgBlock - 1) / kArgBlock);
  return true;
}

// fp32 rows that one 1024-thread workgroup holds in two batches, at least one row per CU: one
// launch, no workspace.
static bool argmax_whole_rows(int64_t rows, int64_t cols, int elem_size) {
  return elem_size == 4 && rows >= 256 && rows < (int64_t{1} << 31) && cols >= kArgVecMinCols &&
         cols / 4 <= 1024 * 2 * kArgMaxVectors;
}

template <typename T>
static int launch_argmax_vec(int64_t* out, const T* in, int64_t rows, int64_t cols, const ArgPlan& plan,
                             void* ws, size_t ws_bytes, hipStream_t stream) {
  const int64_t items = rows * plan.splits;
  if (plan.splits > 1 && (ws == nullptr || ws_bytes < static_cast<size_t>(items) * 16)) return TMB_ERR_WORKSPACE;
  const dim3 grid(static_cast<unsigned>(items)), block(kArgBlock);
#define TMB_ARG(U) argmax_vec_kernel<T, U><<<grid, block, 0, stream>>>(out, ws, in, cols, plan.splits, plan.chunk)
  if (plan.vectors <= 1) TMB_ARG(1);
  else if (plan.vectors <= 2) TMB_ARG(2);
  else if (plan.vectors <= 4) TMB_ARG(4);
  else TMB_ARG(kArgMaxVectors);
#undef TMB_ARG
  int rc = check_launch();
  if (rc != 0 || plan.splits == 1) return rc;
  argmax_final_kernel<T, 64><<<dim3(static_cast<unsigned>(rows)), dim3(64), 0, stream>>>(out, ws, rows, plan.splits);
  return check_launch();
}

template <typename T>
static int launch_argmax(int64_t* out, const void* in_, int64_t rows, int64_t cols, void* ws,
                         size_t ws_bytes, hipStream_t stream) {
  const T* in = static_cast<const T*>(in_);
  if constexpr (__is_same(typename ArgTraits<T>::val_t, float)) {
    // (512 x 50257 fp32: 17.1 + 2.7 us in units and a combining launch, 19.3 us as whole rows)
    if (argmax_whole_rows(rows, cols, static_cast<int>(sizeof(T)))) {
      argmax_vec_kernel<T, kArgMaxVectors, 1024, 2><<<dim3(static_cast<unsigned>(rows)), dim3(1024), 0, stream>>>(
          out, ws, in, cols, 1, static_cast<int>((cols + 63) / 64 * 64));
      return check_launch();
    }
    ArgPlan vec;
    if (argmax_vec_plan(rows, cols, static_cast<int>(sizeof(T)), &vec))
      return launch_argmax_vec<T>(out, in, rows, cols, vec, ws, ws_bytes, stream);
  }
  const SplitPlan plan = plan_splits(rows, cols);
  // At least one row per CU and only a few chunks per row: one 1024-thread workgroup per row does
  // the same work per thread in a single launch (the second stage alone costs 4-5 us).
  if (plan.splits > 1 && plan.splits <= 4 && rows >= 256 && rows < (int64_t{1} << 31) &&
      cols < (int64_t{1} << 30)) {
    argmax_chunk_kernel<T, 1024, 7><<<dim3(static_cast<unsigned>(rows)), dim3(1024), 0, stream>>>(
        out, ws, in, rows, cols, 1, cols);
    return check_launch();
  }
  const int64_t items = rows * plan.splits;
  if (items >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  if (plan.splits > 1) {
    if (ws == nullptr || ws_bytes < static_cast<size_t>(items) * 16) return TMB_ERR_WORKSPACE;
  }
  argmax_chunk_kernel<T, kRedBlock><<<dim3(static_cast<unsigned>(items)), dim3(kRedBlock), 0, stream>>>(
      out, ws, in, rows, cols, plan.splits, plan.chunk);
  int rc = check_launch();
  if (rc != 0 || plan.splits == 1) return rc;
  if (plan.splits > 256) {
    argmax_final_kernel<T, 1024><<<dim3(static_cast<unsigned>(rows)), dim3(1024), 0, stream>>>(
        out, ws, rows, plan.splits);
  } else {
    argmax_final_kernel<T, 64><<<dim3(static_cast<unsigned>(rows)), dim3(64), 0, stream>>>(
        out, ws, rows, plan.splits);
  }
  return check_launch();
}

}  // namespace tmb

extern "C" size_t tmb_reduce_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
  (void)dtype;
  if (rows <= 0 || cols <= 0) return 0;
  const tmb::SplitPlan plan = tmb::plan_splits(rows, cols);
  if (plan.splits == 1) return 0;
  return static_cast<size_t>(rows) * static_cast<size_t>(plan.splits) * 16;
}

extern "C" size_t tmb_argmax_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
  if (rows <= 0 || cols <= 0) return 0;
  const int elem = dtype == TMB_F32 ? 4 : (dtype == TMB_F16 || dtype == TMB_BF16 ? 2 : 0);
  if (elem != 0 && tmb::argmax_whole_rows(rows, cols, elem)) return 0;
  tmb::ArgPlan plan;
  if (elem != 0 && tmb::argmax_vec_plan(rows, cols, elem, &plan))
    return plan.splits == 1 ? 0 : static_cast<size_t>(rows) * static_cast<size_t>(plan.splits) * 16;
  return tmb_reduce_workspace_bytes(rows, cols, dtype);
}

extern "C" int tmb_reduce_rows(void* out, const void* in, int64_t rows, int64_t cols, int op,
                               int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace tmb;
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (op != TMB_SUM && op != TMB_MEAN && op != TMB_AMAX) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0) return TMB_OK;
  if (cols == 0) return TMB_ERR_INVALID_ARGUMENT;  // empty rows have no max/mean; caller decides
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool is_max = op == TMB_AMAX;
  switch (dtype) {
    case TMB_F32:
      return is_max ? launch_reduce<AccFMax, float, false>(out, in, rows, cols, op, workspace, workspace_bytes, s)
                    : launch_reduce<AccSum<float>, float, false>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    case TMB_F16:
      return is_max ? launch_reduce<AccFMax, f16_t, false>(out, in, rows, cols, op, workspace, workspace_bytes, s)
                    : launch_reduce<AccSum<float>, f16_t, false>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    case TMB_BF16:
      return is_max ? launch_reduce<AccFMax, bf16_t, false>(out, in, rows, cols, op, workspace, workspace_bytes, s)
                    : launch_reduce<AccSum<float>, bf16_t, false>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    case TMB_I64:
      if (op == TMB_MEAN) return TMB_ERR_UNSUPPORTED;
      return is_max ? launch_reduce<AccIMax<int64_t>, int64_t, true>(out, in, rows, cols, op, workspace, workspace_bytes, s)
                    : launch_reduce<AccSum<int64_t>, int64_t, false>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    case TMB_I32:
      if (!is_max) return TMB_ERR_UNSUPPORTED;
      return launch_reduce<AccIMax<int32_t>, int32_t, true>(out, in, rows, cols, op, workspace, workspace_bytes, s);
    default:
      return TMB_ERR_UNSUPPORTED;
  }
}

namespace tmb {

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};
static int g_scratch_rc[kMaxDevices] = {};   // a failed lookup is remembered, not retried

// Device address of `scratch` on the device `stream` belongs to (the current device for the
// null stream), looked up once per device with that device current.
static int static_scratch(hipStream_t stream, void** ptr) {
  int current = -1;
  hipError_t e = hipGetDevice(&current);
  if (e != hipSuccess) return static_cast<int>(e);
  int dev = current;
  if (stream != nullptr) {
    hipDevice_t of_stream = 0;
    e = hipStreamGetDevice(stream, &of_stream);
    if (e != hipSuccess) return static_cast<int>(e);
    dev = static_cast<int>(of_stream);
  }
  if (dev < 0 || dev >= kMaxDevices) return TMB_ERR_UNSUPPORTED;
  // Kernels are launched on the current device: a stream of another one cannot take them.
  if (dev != current) return TMB_ERR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr && g_scratch_rc[dev] == 0) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) g_scratch_rc[dev] = static_cast<int>(e);
    else if (p == nullptr) g_scratch_rc[dev] = static_cast<int>(hipErrorInvalidSymbol);
    else g_scratch_ptr[dev] = p;
  }
  if (g_scratch_rc[dev] != 0) return g_scratch_rc[dev];
  *ptr = g_scratch_ptr[dev];
  return TMB_OK;
}

}  // namespace tmb

extern "C" int tmb_reduce_rows_static(void* out, const void* in, int64_t rows, int64_t cols, int op,
                                      int dtype, void* stream) {
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  const size_t need = tmb_reduce_workspace_bytes(rows, cols, dtype);
  if (need > tmb::kStaticScratchBytes) return TMB_ERR_SCRATCH_LIMIT;
  if (need == 0) return tmb_reduce_rows(out, in, rows, cols, op, dtype, nullptr, 0, stream);
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  void* ws = nullptr;
  const int rc = tmb::static_scratch(static_cast<hipStream_t>(stream), &ws);
  if (rc != TMB_OK) return rc;
  // Every partial the second stage reads is written by the first stage of the same call, so
  // nothing in the array has to start at zero.
  return tmb_reduce_rows(out, in, rows, cols, op, dtype, ws, tmb::kStaticScratchBytes, stream);
}

extern "C" int tmb_argmax_rows(int64_t* out, const void* in, int64_t rows, int64_t cols,
                               int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace tmb;
  if (rows < 0 || cols < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0) return TMB_OK;
  if (cols == 0) return TMB_ERR_INVALID_ARGUMENT;
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case TMB_F32: return launch_argmax<float>(out, in, rows, cols, workspace, workspace_bytes, s);
    case TMB_F16: return launch_argmax<f16_t>(out, in, rows, cols, workspace, workspace_bytes, s);
    case TMB_BF16: return launch_argmax<bf16_t>(out, in, rows, cols, workspace, workspace_bytes, s);
    case TMB_I64: return launch_argmax<int64_t>(out, in, rows, cols, workspace, workspace_bytes, s);
    case TMB_I32: return launch_argmax<int32_t>(out, in, rows, cols, workspace, workspace_bytes, s);
    default: return TMB_ERR_UNSUPPORTED;
  }
}
