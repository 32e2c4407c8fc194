// Shared device helpers for the gfx950 (MI355X, wave64) kernels of libtmb_hip.
//
// Everything here is written for CDNA4 only: 64-lane wavefronts, DPP row
// operations for intra-wave reductions, 16-byte vector memory accesses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tmb_hip.h"

namespace tmb {

using bf16_t = __bf16;
using f16_t = _Float16;

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Scalar conversions. All arithmetic is done in fp32; storage types are cast
// exactly once on the way out (round-to-nearest-even, the hardware default).
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return static_cast<T>(v);
}

// 16-byte vector of storage elements.
template <typename T>
struct alignas(16) Vec16 {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

template <typename T>
__device__ __forceinline__ Vec16<T> load_vec16(const T* p) {
  return *reinterpret_cast<const Vec16<T>*>(p);
}
template <typename T>
__device__ __forceinline__ void store_vec16(T* p, const Vec16<T>& v) {
  *reinterpret_cast<Vec16<T>*>(p) = v;
}

// Streaming variants: data that is touched exactly once is moved with the non-temporal hint so
// it does not displace reusable lines (gamma/beta, partials) from L2 / Infinity Cache.
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t raw16_t;
template <typename T>
__device__ __forceinline__ Vec16<T> load_vec16_stream(const T* p) {
  const raw16_t r = __builtin_nontemporal_load(reinterpret_cast<const raw16_t*>(p));
  return __builtin_bit_cast(Vec16<T>, r);
}
template <typename T>
__device__ __forceinline__ void store_vec16_stream(T* p, const Vec16<T>& v) {
  __builtin_nontemporal_store(__builtin_bit_cast(raw16_t, v), reinterpret_cast<raw16_t*>(p));
}

// The same 16 bytes at an address that is only element-aligned (rows of an odd pitch, as in a
// [rows, 50257] tensor): global memory takes unaligned vector accesses on this target, and one
// 16-byte access per lane beats 16 / sizeof(T) element accesses by far.
typedef raw16_t __attribute__((aligned(2))) raw16_a2_t;
typedef raw16_t __attribute__((aligned(4))) raw16_a4_t;
template <typename T>
__device__ __forceinline__ Vec16<T> load_vec16_unaligned(const T* p) {
  if constexpr (sizeof(T) == 2) {
    const raw16_t r = *reinterpret_cast<const raw16_a2_t*>(p);
    return __builtin_bit_cast(Vec16<T>, r);
  } else {
    const raw16_t r = *reinterpret_cast<const raw16_a4_t*>(p);
    return __builtin_bit_cast(Vec16<T>, r);
  }
}
template <typename T>
__device__ __forceinline__ void store_vec16_unaligned(T* p, const Vec16<T>& v) {
  if constexpr (sizeof(T) == 2) {
    *reinterpret_cast<raw16_a2_t*>(p) = __builtin_bit_cast(raw16_t, v);
  } else {
    *reinterpret_cast<raw16_a4_t*>(p) = __builtin_bit_cast(raw16_t, v);
  }
}
// N fp32 values as TOut elements at an element-aligned address (several 16-byte stores when TOut
// is wider than the type N was counted in).
template <typename TOut, int N>
__device__ __forceinline__ void store_converted_unaligned(TOut* p, const float (&x)[N]) {
  constexpr int OUT_PER_VEC = 16 / sizeof(TOut);
  static_assert(N % OUT_PER_VEC == 0, "vector width mismatch");
#pragma unroll
  for (int c = 0; c < N / OUT_PER_VEC; ++c) {
    Vec16<TOut> o;
#pragma unroll
    for (int e = 0; e < OUT_PER_VEC; ++e) o.v[e] = from_f32<TOut>(x[c * OUT_PER_VEC + e]);
    store_vec16_unaligned(p + c * OUT_PER_VEC, o);
  }
}

// Stores N = 16/sizeof(TIn) fp32 values as TOut elements. When TOut is wider
// than TIn (half_to_float softmax) this issues several 16-byte stores.
template <typename TOut, int N, bool STREAM = false>
__device__ __forceinline__ void store_converted(TOut* p, const float (&x)[N]) {
  constexpr int OUT_PER_VEC = 16 / sizeof(TOut);
  static_assert(N % OUT_PER_VEC == 0, "vector width mismatch");
#pragma unroll
  for (int c = 0; c < N / OUT_PER_VEC; ++c) {
    Vec16<TOut> o;
#pragma unroll
    for (int e = 0; e < OUT_PER_VEC; ++e) o.v[e] = from_f32<TOut>(x[c * OUT_PER_VEC + e]);
    if (STREAM) {
      store_vec16_stream(p + c * OUT_PER_VEC, o);
    } else {
      store_vec16(p + c * OUT_PER_VEC, o);
    }
  }
}

// The same with the hint chosen at run time (a wave-uniform flag, usually "the tensors of this
// launch are larger than the L2s"). The empty asm keeps the two stores from being merged into
// one, which would drop the hint.
template <typename TOut, int N>
__device__ __forceinline__ void store_converted_hinted(TOut* p, const float (&x)[N], bool stream) {
  if (stream) {
    store_converted<TOut, N, true>(p, x);
    asm volatile("" ::: "memory");
  } else {
    store_converted<TOut, N, false>(p, x);
  }
}
// Outputs of a pass whose tensors together exceed this are written once and not read again
// before they have left every cache: non-temporal stores measured 2-9 % faster there (the eight
// L2s hold 32 MB).
constexpr int64_t kStreamStoreBytes = int64_t{64} << 20;

// ---------------------------------------------------------------------------
// exp with fp32-accurate argument reduction on top of v_exp_f32 (2^x).
// x*log2(e) is formed as hi+lo so the result keeps ~1-2 ulp even for |x|~80.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float exp_f32(float x) {
#pragma clang fp contract(off)
  constexpr float kLog2eHi = 1.44269502162933349609375f;   // float(log2 e)
  constexpr float kLog2eLo = 1.92596299112661746e-08f;     // log2 e - hi
  constexpr float kLn2 = 0.693147180559945309417f;
  float hi = x * kLog2eHi;
  float lo = __builtin_fmaf(x, kLog2eHi, -hi) + x * kLog2eLo;
  float e = __builtin_amdgcn_exp2f(hi);
  // 2^(hi+lo) = 2^hi * (1 + lo*ln2 + ...), |lo| < 1e-5 so first order is exact to fp32.
  float r = __builtin_fmaf(e, lo * kLn2, e);
  // Overflow: e is +inf and inf*lo + inf would be NaN for negative lo; keep the +inf.
  r = (e == __builtin_inff()) ? e : r;
  // exp(-inf) must be exactly 0 (lo is NaN when x is -inf).
  return (x == -__builtin_inff()) ? 0.0f : r;
}

// exp for results that are stored in 16 bits: one multiply and v_exp_f32. The rounding of
// x*log2(e) costs at most 6e-8 |x log2 e| in the exponent, i.e. below 6e-6 relative wherever the
// result is a normal number: 1 % of half an fp16 ulp.
__device__ __forceinline__ float exp_f32_for16(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269502162933349609375f);
}
template <typename TOut>
__device__ __forceinline__ float exp_for(float x) {
  if constexpr (sizeof(TOut) == 2) {
    return exp_f32_for16(x);
  } else {
    return exp_f32(x);
  }
}

// Pins a value in a VGPR as an fp32 number. The compiler otherwise folds an fp32 multiply or
// add into the following fp32->fp16 conversion (v_fma_mixlo_f16: one rounding instead of two),
// and whether it does so depends on the surrounding code — which would make the same formula
// round differently in two kernels.
__device__ __forceinline__ float pin_f32(float v) {
  asm volatile("" : "+v"(v));
  return v;
}

// ---------------------------------------------------------------------------
// GELU, shared by the GEMM epilogue and the standalone kernel. Floating-point contraction is
// switched off inside so that both users execute the same instruction sequence and a fused
// GEMM+GELU is bit-identical to the GEMM followed by the elementwise kernel.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh_f32(float x) {
#pragma clang fp contract(off)
  // 0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)), u = sqrt(2/pi) (x + 0.044715 x^3): no
  // cancellation for negative x, one v_exp_f32 and one v_rcp_f32. With the constants folded,
  // -2u log2(e) = x (c1 + c2 x^2); its three roundings cost at most 2e-7 |arg| in the exponent,
  // i.e. < 3e-6 relative wherever the result is above 1e-7 |x|.
  constexpr float c1 = -2.302208198144325f;   // -2 log2(e) sqrt(2/pi)
  constexpr float c2 = -0.1029432395800235f;  // c1 * 0.044715
  const float arg = x * __builtin_fmaf(x * x, c2, c1);
  const float e = __builtin_amdgcn_exp2f(arg);  // +inf for very negative x: the quotient is -0
  return pin_f32(x * __builtin_amdgcn_rcpf(1.0f + e));
}
__device__ __forceinline__ float gelu_erf_f32(float x) {
#pragma clang fp contract(off)
  return pin_f32(0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)));
}

// ---------------------------------------------------------------------------
// Wave64 reductions built on DPP row operations. After the four DPP steps all
// 16 lanes of a DPP row hold that row's reduction; the four rows are combined
// through v_readlane in a fixed order, so the result is wave-uniform and
// bit-reproducible from launch to launch.
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

constexpr int kDppQuadXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i <- lane 7-i within 8
constexpr int kDppRowMirror = 0x140;      // lane i <- lane 15-i within 16

__device__ __forceinline__ float readlane_f32(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

struct SumOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
// max that propagates NaN like torch.amax / torch.max do.
struct MaxNanOp {
  __device__ __forceinline__ float operator()(float a, float b) const {
    return (a != a) ? a : ((b != b) ? b : (a > b ? a : b));
  }
};
// plain max for softmax (rows containing NaN produce NaN through the exp/sum anyway).
struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

template <typename Op>
__device__ __forceinline__ float wave_reduce(float v, Op op) {
  v = op(v, dpp_f32<kDppQuadXor1>(v));
  v = op(v, dpp_f32<kDppQuadXor2>(v));
  v = op(v, dpp_f32<kDppRowHalfMirror>(v));
  v = op(v, dpp_f32<kDppRowMirror>(v));
  float r0 = readlane_f32(v, 0), r1 = readlane_f32(v, 16);
  float r2 = readlane_f32(v, 32), r3 = readlane_f32(v, 48);
  return op(op(r0, r1), op(r2, r3));
}

__device__ __forceinline__ float wave_sum(float v) { return wave_reduce(v, SumOp{}); }
__device__ __forceinline__ float wave_max(float v) { return wave_reduce(v, MaxOp{}); }

// Reduction across the waves that cooperate on one row. `slot` is an LDS array
// of at least (waves in block) floats; `group` is the index of the first wave
// of the row's group, `n` the number of waves per row. Fixed combine order.
template <typename Op>
__device__ __forceinline__ float group_reduce(float wave_val, float* slot, int wave, int group0,
                                              int n, Op op) {
  if (n == 1) return wave_val;
  __syncthreads();  // protect slot reuse between successive reductions
  if ((threadIdx.x & (kWave - 1)) == 0) slot[wave] = wave_val;
  __syncthreads();
  float r = slot[group0];
  for (int i = 1; i < n; ++i) r = op(r, slot[group0 + i]);
  return r;
}

inline int check_launch() {
  hipError_t e = hipGetLastError();
  return static_cast<int>(e);
}

// CUs of the current device (queried once per process).
inline int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace tmb
