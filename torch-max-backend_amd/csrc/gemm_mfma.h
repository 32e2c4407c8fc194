// MFMA GEMM kernel for gfx950 (bf16 / fp16 storage, fp32 accumulation).
//
// One workgroup of WAVES_M x WAVES_N waves owns a BM x BN tile of C and walks K in stages of 64.
// Stage k+1 is fetched from global memory into registers while stage k is multiplied out of LDS;
// after the multiply the registers are written to the other LDS buffer, one barrier closes the
// stage, and the first operand fragments of the next stage are fetched from LDS *before* the
// last quarter of the current stage's MFMAs is issued, so that the LDS latency after the
// barrier is covered by matrix work. Operand fragments are double-buffered in registers.
//
// LDS layout: K-major, one 128-byte line (64 K-values) per matrix row; the eight 16-byte chunks
// of a line are XOR-swizzled with (row ^ row>>3) so that ds_read_b128 fragment fetches, the
// workgroup's row-wise stores and the transposed stores of an N-major B are all bank-conflict
// free.
//
// The MFMA is issued with the operands swapped (B fragment first): the 32x32 result then holds,
// per lane, one row m of C and four consecutive columns n per register quad, which the epilogue
// turns into 8-byte stores after adding the bias in fp32 (and the optional GELU).
#pragma once

#include "tmb_common.h"

namespace tmb {

// Bias has already been added in fp32. A GELU epilogue works on that fp32 sum and the result is
// cast once (the reference's rule for everything it fuses into a GEMM: form the value in fp32,
// cast exactly once, matmul_ops.mojo:2651-2657). With `twice` the sum is first rounded to the
// storage type, so that the fused kernel returns exactly the bits of addmm followed by a
// separate gelu kernel.
template <typename T, int EPI>
__device__ __forceinline__ T finish(float v, bool twice) {
  v = pin_f32(v);  // acc + bias is an fp32 sum; it is rounded to T as a separate step
  if constexpr (EPI == TMB_EPI_NONE) {
    return from_f32<T>(v);
  } else {
    const float r = twice ? to_f32(from_f32<T>(v)) : v;
    return from_f32<T>(EPI == TMB_EPI_GELU_TANH ? gelu_tanh_f32(r) : gelu_erf_f32(r));
  }
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
  static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<f16_t> {
  static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

// v_mfma_f32_16x16x32: a lane holds row (lane % 16) and eight consecutive k starting at
// 8 * (lane / 16) of each operand; of the 16 x 16 result it holds column (lane % 16) and rows
// 4 * (lane / 16) + {0..3}. Per multiply-add it reads and writes half as many accumulator
// registers as the 32x32x16 form and draws measurably less power: a loop of nothing but MFMAs on
// random bf16 operands sustains 2.02 PFLOP/s against 1.79 PFLOP/s, the clock being set by the
// power the matrix pipes draw.
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4v_t;
template <typename T>
struct Mfma16;
template <>
struct Mfma16<bf16_t> {
  static __device__ __forceinline__ f32x4v_t run(u32x4_t a, u32x4_t b, f32x4v_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma16<f16_t> {
  static __device__ __forceinline__ f32x4v_t run(u32x4_t a, u32x4_t b, f32x4v_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

constexpr int kBK = 64;  // K extent of one LDS stage (64 x 2 bytes = one 128-byte line)
constexpr int kLineBytes = 128;

// Byte offset of 16-byte chunk `chunk` (0..7) of line `row` inside a swizzled tile.
__device__ __forceinline__ int lds_offset(int row, int chunk) {
  return row * kLineBytes + (((chunk ^ row ^ (row >> 3)) & 7) << 4);
}

struct GemmArgs {
  void* c;
  const void* a;
  const void* b;
  const void* bias;
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  int64_t stride_a, stride_b, stride_c;
  int tiles_m, tiles_n;
  int stream_c;  // C is larger than the 256 MB Infinity Cache: store it non-temporally
  // optional second epilogue step: C = T(float(T(epilogue(acc + bias))) + float(residual)),
  // i.e. what a separate elementwise add after the GEMM would store (MFMA kernels only)
  const void* residual;
  int64_t ldr, stride_r;
  // round_like_unfused: every fused step rounds to the storage type where a separate kernel
  // would have stored (bit-identical to the unfused graph); otherwise the epilogue stays in fp32
  // up to the one cast. resid_f32 / out_f32: the residual operand / C are fp32 although A and B
  // are 16-bit (a residual stream kept in fp32); both need round_like_unfused == 0.
  int round_like_unfused = 0;
  int resid_f32 = 0;
  int out_f32 = 0;
  // persistent kernels with a streamed output: workgroups start in four phases this many 10 ns
  // ticks apart, so that their store bursts do not all hit memory at the same moment
  int stagger_ticks = 0;
  // fp32-partial launches (split-K): blockIdx.y is the split; split z of `splits` multiplies the
  // K stages [stages * z / splits, stages * (z + 1) / splits) and stores partial z (0: not split)
  int splits = 0;
  // a split launch whose workgroups all run at once: the (split, tile) pairs, split-major, are
  // dealt to the 8 XCDs in runs of this many, so that an XCD works on tiles of one or two splits
  // and their operand slices are fetched into its L2 once (0: blockIdx.y is the split)
  int xcd_chunk = 0;
};

// Maps the launch-order workgroup id to a tile so that each XCD (workgroups are dealt to the
// 8 XCDs round-robin) works on a contiguous run of tiles, walked in column-major groups of
// `kGroupM` tile rows.
// (tile_of_index: the walk itself, from a position in it)
__device__ __forceinline__ void tile_of_index(int tile, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int kGroupM = 8;
  const int per_group = kGroupM * tiles_n;
  const int group = tile / per_group;
  const int first_m = group * kGroupM;
  const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  const int in_group = tile - group * per_group;
  tm = first_m + in_group % gsz;
  tn = in_group / gsz;
}
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int kXcds = 8;
  const int total = tiles_m * tiles_n;
  const int q = total / kXcds, r = total % kXcds;
  const int xcd = pid % kXcds, idx = pid / kXcds;
  tile_of_index(xcd * q + (xcd < r ? xcd : r) + idx, tiles_m, tiles_n, tm, tn);
}

// Epilogue. A lane of the (operand-swapped) MFMA result holds, for row lane%32 of a 32x32 tile,
// columns 8q + 4*(lane/32) + {0..3}, q = 0..3: stored straight from there, every store
// instruction would scatter 8-byte pieces over 32 rows and memory would see partial lines
// (measured: 1.9x the output bytes written). So a wave stages one 32-row band of its tile in
// LDS (the operand buffers are free by then) and writes it out row by row: 16 bytes per lane,
// consecutive lanes along a row, whole 128-byte lines per row where the tile is 64 wide.
//
// stage_tile: +bias (fp32) -> optional GELU -> one cast, 4 x 8 bytes into the band. The
// epilogue is bound by its vector-ALU instruction count (both waves of a SIMD run it at the same
// time, with the matrix pipe idle), so values are converted and packed two at a time and the
// bias is unpacked to fp32 once per wave tile.
typedef __attribute__((address_space(3))) unsigned char lds_byte_t;
typedef __attribute__((address_space(3))) u32x2_t lds_u32x2_t;
typedef __attribute__((address_space(3))) u32x4_t lds_u32x4v_t;

template <int WN>
struct BandLayout {
  static constexpr int PITCH = WN * 2 + 16;  // bytes; the pad spreads the rows over the banks
  static constexpr int BYTES = 32 * PITCH;
};

typedef u32x2_t __attribute__((aligned(2))) u32x2_unaligned_t;

// The four bias values a lane needs for columns col .. col+3 (zeros past N or without bias),
// packed as stored. One 8-byte load where the row allows it.
template <typename T>
__device__ __forceinline__ u32x2_t load_bias4(const T* __restrict__ bias, int64_t col, int64_t N) {
  u32x2_t out = {0u, 0u};
  if (bias == nullptr || col >= N) return out;
  if (col + 4 <= N) return *reinterpret_cast<const u32x2_unaligned_t*>(bias + col);
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (col + e < N)
      out[e >> 1] |= static_cast<uint32_t>(__builtin_bit_cast(unsigned short, bias[col + e]))
                     << (16 * (e & 1));
  return out;
}

template <typename T>
__device__ __forceinline__ float unpack_elem(u32x2_t v, int e) {
  return to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(v[e >> 1] >> (16 * (e & 1)))));
}

// Two fp32 values rounded to T (nearest even) and packed, low half first. On this target the
// bf16 form is a single v_cvt_pk_bf16_f32.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef T tx2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, tx2_t));
}

template <typename T, int EPI>
__device__ __forceinline__ uint32_t finish2(float a, float b, bool twice) {
  a = pin_f32(a);  // acc + bias is an fp32 sum; it is rounded to T as a separate step
  b = pin_f32(b);
  if constexpr (EPI == TMB_EPI_NONE) {
    return pack2<T>(a, b);
  } else {
    if (twice) {  // wave-uniform
      const uint32_t p = pack2<T>(a, b);
      a = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(p)));
      b = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(p >> 16)));
    }
    return EPI == TMB_EPI_GELU_TANH ? pack2<T>(gelu_tanh_f32(a), gelu_tanh_f32(b))
                                    : pack2<T>(gelu_erf_f32(a), gelu_erf_f32(b));
  }
}

// One 32x32 accumulator tile into the band: +bias (fp32) -> optional GELU -> one cast, 4 x 8
// bytes per lane. `bias` holds the lane's 16 bias values as fp32 (zeros without a bias).
template <typename T, int EPI>
__device__ __forceinline__ void stage_tile(const f32x16_t& acc, lds_byte_t* dst,
                                           const float (&bias)[16], bool twice) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    u32x2_t packed;
    packed[0] = finish2<T, EPI>(acc[4 * q + 0] + bias[4 * q + 0], acc[4 * q + 1] + bias[4 * q + 1], twice);
    packed[1] = finish2<T, EPI>(acc[4 * q + 2] + bias[4 * q + 2], acc[4 * q + 3] + bias[4 * q + 3], twice);
    *(lds_u32x2_t*)(dst + 16 * q) = packed;
  }
}

// The fp32 form of the band, for epilogues that go on in fp32 after the bias (a residual added
// before the one cast, or an fp32 output): 16 bytes per lane and 8-column group, row pitch
// WN * 4 + 16 bytes, which keeps both the 16-byte writes (16 lanes = 16 rows, 4 banks apart)
// and the row-wise 16-byte reads free of bank conflicts.
template <int WN>
struct BandLayoutF32 {
  static constexpr int PITCH = WN * 4 + 16;
  static constexpr int BYTES = 32 * PITCH;
};
typedef float f32x4_lds_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) f32x4_lds_t lds_f32x4_t;

__device__ __forceinline__ void stage_tile_f32(const f32x16_t& acc, lds_byte_t* dst,
                                               const float (&bias)[16]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const f32x4_lds_t v = {acc[4 * q + 0] + bias[4 * q + 0], acc[4 * q + 1] + bias[4 * q + 1],
                           acc[4 * q + 2] + bias[4 * q + 2], acc[4 * q + 3] + bias[4 * q + 3]};
    *(lds_f32x4_t*)(dst + 32 * q) = v;
  }
}

// Writes the staged 32 x WN band to C: a lane stores 8 columns (16 bytes) at once, consecutive
// lanes along the row. Rows of C need not start on 16-byte boundaries (an odd pitch, as with a
// 50257-wide vocabulary, leaves them 2-byte aligned): global memory takes unaligned vector
// accesses on this target, and one 16-byte store per lane beats eight 2-byte ones by far.
typedef u32x4_t __attribute__((aligned(2))) u32x4_unaligned_t;

template <typename T>
__device__ __forceinline__ uint32_t add_pair(uint32_t x, uint32_t r) {
  const float x0 = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(x)));
  const float x1 = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(x >> 16)));
  const float r0 = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(r)));
  const float r1 = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(r >> 16)));
  return static_cast<uint32_t>(__builtin_bit_cast(unsigned short, from_f32<T>(x0 + r0))) |
         (static_cast<uint32_t>(__builtin_bit_cast(unsigned short, from_f32<T>(x1 + r1))) << 16);
}

template <typename T, int WN, bool STREAM>
__device__ __forceinline__ void flush_band(const lds_byte_t* band, T* __restrict__ C, int64_t ldc,
                                           int64_t row0, int64_t col0, int64_t M, int64_t N,
                                           const T* __restrict__ R, int64_t ldr, int lane) {
  constexpr int PITCH = BandLayout<WN>::PITCH;
  constexpr int LPR = WN / 8;    // lanes per row
  constexpr int RPP = 64 / LPR;  // rows per pass
#pragma unroll
  for (int p = 0; p < 32 / RPP; ++p) {
    const int r = p * RPP + lane / LPR;
    const int c = (lane % LPR) * 8;
    u32x4_t v = *(const lds_u32x4v_t*)(band + r * PITCH + c * 2);
    const int64_t row = row0 + r, col = col0 + c;
    if (row < M && col < N) {
      T* dst = C + row * ldc + col;
      if (R != nullptr) {  // wave-uniform
        const T* rsrc = R + row * ldr + col;
        u32x4_t rv = {0u, 0u, 0u, 0u};
        if (col + 8 <= N) {
          rv = *reinterpret_cast<const u32x4_unaligned_t*>(rsrc);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < N)
              rv[e >> 1] |= static_cast<uint32_t>(__builtin_bit_cast(unsigned short, rsrc[e]))
                            << (16 * (e & 1));
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = add_pair<T>(v[e], rv[e]);
      }
      if (col + 8 <= N) {
        // STREAM is a template parameter on purpose: as a run-time branch the two stores are
        // merged and the non-temporal hint is lost
        if constexpr (STREAM) {
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4_unaligned_t*>(dst));
        } else {
          *reinterpret_cast<u32x4_unaligned_t*>(dst) = v;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N)
            dst[e] = __builtin_bit_cast(T, static_cast<unsigned short>(v[e >> 1] >> (16 * (e & 1))));
      }
    }
  }
}

// What the epilogue does after bias (and GELU): nothing, or "+ residual", in the storage type
// (twice) or in fp32 before the one cast.
struct EpilogueArgs {
  const void* residual;  // [M, N] with pitch ldr (already offset to the batch entry) or nullptr
  int64_t ldr;
  bool twice;            // round to the storage type after every fused step
  bool resid_f32;        // residual elements are fp32 (else T)
  bool out_f32;          // C elements are fp32 (else T)
  // the fp32 band is needed unless everything is rounded step by step in T
  __device__ __forceinline__ bool wide() const {
    return residual != nullptr && (!twice || resid_f32 || out_f32);
  }
};

typedef float f32x4_g_t __attribute__((ext_vector_type(4)));
typedef f32x4_g_t __attribute__((aligned(4))) f32x4_g_unaligned_t;

// Writes the staged fp32 band (32 x WN) to C: a lane takes 8 columns of a row, adds the residual
// (8 x T or 8 x fp32) in fp32 and stores 8 x T (one 16-byte store) or 8 x fp32.
// The fp32 residual of a whole wave tile of 16x16 accumulators (AM x AN tiles), held in
// registers: 8 values per lane, pass and band of flush_band_wide. Only for wave tiles where that
// is at most 64 registers per lane, and only when N is a multiple of 8 (a lane's eight columns
// are then inside C or outside as a whole). The loads carry no conditions: lanes outside C read
// a valid address whose value is never used, so nothing but the loads' latency stands between
// the request and the next instruction.
template <int AM, int AN>
struct ResidualTile {
  static constexpr int WN = AN * 16;
  static constexpr int LPR = WN / 8, RPP = 64 / LPR, PASSES = 32 / RPP, BANDS = AM / 2;
  static constexpr bool FITS = BANDS * PASSES * 8 <= 64;
  f32x4_g_t v[FITS ? BANDS : 1][FITS ? PASSES : 1][2];
  bool loaded = false;  // wave-uniform
  __device__ __forceinline__ void request(const EpilogueArgs& ep, int64_t row0, int64_t col0, int64_t M,
                                          int64_t N, int lane) {
    if constexpr (FITS) {
      loaded = ep.wide() && ep.resid_f32 && N % 8 == 0;
      if (!loaded) return;
      int64_t col = col0 + (lane % LPR) * 8;
      col = col < N ? col : 0;
      const float* base = static_cast<const float*>(ep.residual) + col;
#pragma unroll
      for (int b = 0; b < BANDS; ++b)
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
          int64_t row = row0 + b * 32 + p * RPP + lane / LPR;
          row = row < M ? row : M - 1;
          const float* src = base + row * ep.ldr;
          v[b][p][0] = *reinterpret_cast<const f32x4_g_unaligned_t*>(src);
          v[b][p][1] = *reinterpret_cast<const f32x4_g_unaligned_t*>(src + 4);
        }
    }
  }
};

// PRE and pre != nullptr: the fp32 residual was requested by the caller before (`pre`: this
// band of a ResidualTile), so no pass waits for memory.
template <typename T, int WN, bool STREAM, bool PRE = false>
__device__ __forceinline__ void flush_band_wide(const lds_byte_t* band, void* __restrict__ Cv,
                                                int64_t ldc, int64_t row0, int64_t col0, int64_t M,
                                                int64_t N, const EpilogueArgs& ep, int lane,
                                                const f32x4_g_t (*pre)[2] = nullptr) {
  constexpr int PITCH = BandLayoutF32<WN>::PITCH;
  constexpr int LPR = WN / 8;    // lanes per row
  constexpr int RPP = 64 / LPR;  // rows per pass
#pragma unroll
  for (int p = 0; p < 32 / RPP; ++p) {
    const int r = p * RPP + lane / LPR;
    const int c = (lane % LPR) * 8;
    const f32x4_lds_t lo = *(const lds_f32x4_t*)(band + r * PITCH + c * 4);
    const f32x4_lds_t hi = *(const lds_f32x4_t*)(band + r * PITCH + c * 4 + 16);
    float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    const int64_t row = row0 + r, col = col0 + c;
    if (row >= M || col >= N) continue;
    const bool whole = col + 8 <= N;
    if (PRE && pre != nullptr) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] += pre[p][0][e];
        v[4 + e] += pre[p][1][e];
      }
    } else if (ep.resid_f32) {
      const float* rsrc = static_cast<const float*>(ep.residual) + row * ep.ldr + col;
      if (whole) {
        const f32x4_g_t r0 = *reinterpret_cast<const f32x4_g_unaligned_t*>(rsrc);
        const f32x4_g_t r1 = *reinterpret_cast<const f32x4_g_unaligned_t*>(rsrc + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] += r0[e];
          v[4 + e] += r1[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N) v[e] += rsrc[e];
      }
    } else {
      const T* rsrc = static_cast<const T*>(ep.residual) + row * ep.ldr + col;
      if (whole) {
        const u32x4_t rv = *reinterpret_cast<const u32x4_unaligned_t*>(rsrc);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[e] += to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(rv[e >> 1] >> (16 * (e & 1)))));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N) v[e] += to_f32(rsrc[e]);
      }
    }
    if (ep.out_f32) {
      float* dst = static_cast<float*>(Cv) + row * ldc + col;
      if (whole) {
        const f32x4_g_t o0 = {v[0], v[1], v[2], v[3]}, o1 = {v[4], v[5], v[6], v[7]};
        if constexpr (STREAM) {
          __builtin_nontemporal_store(o0, reinterpret_cast<f32x4_g_unaligned_t*>(dst));
          __builtin_nontemporal_store(o1, reinterpret_cast<f32x4_g_unaligned_t*>(dst + 4));
        } else {
          *reinterpret_cast<f32x4_g_unaligned_t*>(dst) = o0;
          *reinterpret_cast<f32x4_g_unaligned_t*>(dst + 4) = o1;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N) dst[e] = v[e];
      }
    } else {
      T* dst = static_cast<T*>(Cv) + row * ldc + col;
      if (whole) {
        const u32x4_t o = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]), pack2<T>(v[4], v[5]),
                           pack2<T>(v[6], v[7])};
        if constexpr (STREAM) {
          __builtin_nontemporal_store(o, reinterpret_cast<u32x4_unaligned_t*>(dst));
        } else {
          *reinterpret_cast<u32x4_unaligned_t*>(dst) = o;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N) dst[e] = from_f32<T>(v[e]);
      }
    }
  }
}

// The whole wave tile (TM x TN tiles of 32x32), one 32-row band at a time through `band`
// (wave-private, BandLayout<WN>::BYTES, or BandLayoutF32<WN>::BYTES when ep.wide()). The caller
// has synchronised the workgroup so that nobody still reads operands from the LDS that `band`
// overlays.
template <typename T, int EPI, int TM, int TN, bool STREAM>
__device__ __forceinline__ void store_wave_tile_impl(f32x16_t (&acc)[TM][TN], lds_byte_t* band,
                                                void* __restrict__ Cv, int64_t ldc, int64_t row0,
                                                int64_t col0, int64_t M, int64_t N,
                                                const T* __restrict__ bias,
                                                const EpilogueArgs& ep, int lane) {
  constexpr int WN = TN * 32;
  // The bias a lane adds depends on its columns only: fetched once for the whole wave tile
  // (the operand fragments' registers are free by now).
  float bias_f[TN][16];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const u32x2_t b4 = load_bias4<T>(bias, col0 + j * 32 + 4 * (lane >> 5) + 8 * q, N);
#pragma unroll
      for (int e = 0; e < 4; ++e) bias_f[j][4 * q + e] = unpack_elem<T>(b4, e);
    }
  if constexpr (EPI == TMB_EPI_NONE) {
    if (ep.wide()) {  // wave-uniform
      constexpr int PITCH = BandLayoutF32<WN>::PITCH;
      lds_byte_t* mine = band + (lane & 31) * PITCH + 16 * (lane >> 5);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        if (row0 + i * 32 >= M) break;  // wave-uniform
#pragma unroll
        for (int j = 0; j < TN; ++j) stage_tile_f32(acc[i][j], mine + j * 128, bias_f[j]);
        flush_band_wide<T, WN, STREAM>(band, Cv, ldc, row0 + i * 32, col0, M, N, ep, lane);
      }
      return;
    }
  }
  constexpr int PITCH = BandLayout<WN>::PITCH;
  lds_byte_t* mine = band + (lane & 31) * PITCH + 8 * (lane >> 5);
  T* __restrict__ C = static_cast<T*>(Cv);
  const T* __restrict__ R = static_cast<const T*>(ep.residual);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (row0 + i * 32 >= M) break;  // wave-uniform
#pragma unroll
    for (int j = 0; j < TN; ++j)
      stage_tile<T, EPI>(acc[i][j], mine + j * 64, bias_f[j], ep.twice);
    flush_band<T, WN, STREAM>(band, C, ldc, row0 + i * 32, col0, M, N, R, ep.ldr, lane);
  }
}

template <typename T, int EPI, int TM, int TN>
__device__ __forceinline__ void store_wave_tile(f32x16_t (&acc)[TM][TN], lds_byte_t* band,
                                                void* __restrict__ C, int64_t ldc, int64_t row0,
                                                int64_t col0, int64_t M, int64_t N,
                                                const T* __restrict__ bias, bool stream,
                                                const EpilogueArgs& ep, int lane) {
  if (stream) {
    store_wave_tile_impl<T, EPI, TM, TN, true>(acc, band, C, ldc, row0, col0, M, N, bias, ep, lane);
  } else {
    store_wave_tile_impl<T, EPI, TM, TN, false>(acc, band, C, ldc, row0, col0, M, N, bias, ep, lane);
  }
}

// The same for accumulators of 16x16 tiles (operand-swapped v_mfma_f32_16x16x32: a lane holds
// row lane % 16 and columns 4 * (lane / 16) + {0..3} of a tile): AM x AN tiles, two tile rows per
// 32-row band. The band layouts and the flush are shared with the 32x32 form.
template <typename T, int EPI, int AM, int AN, bool STREAM>
__device__ __forceinline__ void store_wave_tile16_impl(f32x4v_t (&acc)[AM][AN], lds_byte_t* band,
                                                  void* __restrict__ Cv, int64_t ldc, int64_t row0,
                                                  int64_t col0, int64_t M, int64_t N,
                                                  const T* __restrict__ bias,
                                                  const EpilogueArgs& ep, int lane,
                                                  const ResidualTile<AM, AN>* pre) {
  constexpr int WN = AN * 16;
  static_assert(AM % 2 == 0, "whole 32-row bands");
  float bias_f[AN][4];
#pragma unroll
  for (int j = 0; j < AN; ++j) {
    const u32x2_t b4 = load_bias4<T>(bias, col0 + j * 16 + 4 * (lane >> 4), N);
#pragma unroll
    for (int e = 0; e < 4; ++e) bias_f[j][e] = unpack_elem<T>(b4, e);
  }
  if constexpr (EPI == TMB_EPI_NONE) {
    if (ep.wide()) {  // wave-uniform
      constexpr int PITCH = BandLayoutF32<WN>::PITCH;
      lds_byte_t* mine = band + (lane & 15) * PITCH + 16 * (lane >> 4);
      constexpr bool PRE = ResidualTile<AM, AN>::FITS;  // then `pre` may hold an fp32 residual
#pragma unroll
      for (int b = 0; b < AM / 2; ++b) {
        if (row0 + b * 32 >= M) break;  // wave-uniform
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int j = 0; j < AN; ++j) {
            const f32x4v_t& a = acc[2 * b + h][j];
            const f32x4_lds_t v = {a[0] + bias_f[j][0], a[1] + bias_f[j][1], a[2] + bias_f[j][2],
                                   a[3] + bias_f[j][3]};
            *(lds_f32x4_t*)(mine + h * 16 * PITCH + j * 64) = v;
          }
        flush_band_wide<T, WN, STREAM, PRE>(band, Cv, ldc, row0 + b * 32, col0, M, N, ep, lane,
                                            pre->loaded ? pre->v[PRE ? b : 0] : nullptr);
      }
      return;
    }
  }
  constexpr int PITCH = BandLayout<WN>::PITCH;
  lds_byte_t* mine = band + (lane & 15) * PITCH + 8 * (lane >> 4);
  T* __restrict__ C = static_cast<T*>(Cv);
  const T* __restrict__ R = static_cast<const T*>(ep.residual);
#pragma unroll
  for (int b = 0; b < AM / 2; ++b) {
    if (row0 + b * 32 >= M) break;  // wave-uniform
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < AN; ++j) {
        const f32x4v_t& a = acc[2 * b + h][j];
        u32x2_t packed;
        packed[0] = finish2<T, EPI>(a[0] + bias_f[j][0], a[1] + bias_f[j][1], ep.twice);
        packed[1] = finish2<T, EPI>(a[2] + bias_f[j][2], a[3] + bias_f[j][3], ep.twice);
        *(lds_u32x2_t*)(mine + h * 16 * PITCH + j * 32) = packed;
      }
    flush_band<T, WN, STREAM>(band, C, ldc, row0 + b * 32, col0, M, N, R, ep.ldr, lane);
  }
}

template <typename T, int EPI, int AM, int AN>
__device__ __forceinline__ void store_wave_tile16(f32x4v_t (&acc)[AM][AN], lds_byte_t* band,
                                                  void* __restrict__ C, int64_t ldc, int64_t row0,
                                                  int64_t col0, int64_t M, int64_t N,
                                                  const T* __restrict__ bias, bool stream,
                                                  const EpilogueArgs& ep, int lane,
                                                  const ResidualTile<AM, AN>* pre) {
  if (stream) {
    store_wave_tile16_impl<T, EPI, AM, AN, true>(acc, band, C, ldc, row0, col0, M, N, bias, ep, lane, pre);
  } else {
    store_wave_tile16_impl<T, EPI, AM, AN, false>(acc, band, C, ldc, row0, col0, M, N, bias, ep, lane, pre);
  }
}

// The batch entry's epilogue description out of the launch arguments.
template <typename T>
__device__ __forceinline__ EpilogueArgs epilogue_args(const GemmArgs& g, int64_t batch) {
  const void* r = nullptr;
  if (g.residual != nullptr) {
    r = g.resid_f32 ? static_cast<const void*>(static_cast<const float*>(g.residual) + batch * g.stride_r)
                    : static_cast<const void*>(static_cast<const T*>(g.residual) + batch * g.stride_r);
  }
  return EpilogueArgs{r, g.ldr, g.round_like_unfused != 0, g.resid_f32 != 0, g.out_f32 != 0};
}

// Split-K partials: the wave tile's fp32 accumulators go to P [M, N] (pitch ldp, in floats) as
// they are; a lane holds four consecutive columns of one row per 8-column group, so lanes l and
// l+32 together write 32 contiguous bytes of a row. The partials are summed by
// splitk_reduce_kernel, which also applies bias, epilogue and the one cast.
typedef float f32x4_unaligned_t __attribute__((ext_vector_type(4), aligned(4)));

template <int TM, int TN>
__device__ __forceinline__ void store_wave_tile_f32(f32x16_t (&acc)[TM][TN], float* __restrict__ P,
                                                    int64_t ldp, int64_t row0, int64_t col0,
                                                    int64_t M, int64_t N, int lane) {
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int64_t row = row0 + i * 32 + (lane & 31);
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = col0 + j * 32 + 8 * q + 4 * (lane >> 5);
        float* dst = P + row * ldp + col;
        if (col + 4 <= N) {
          f32x4_unaligned_t v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                 acc[i][j][4 * q + 3]};
          *reinterpret_cast<f32x4_unaligned_t*>(dst) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (col + e < N) dst[e] = acc[i][j][4 * q + e];
        }
      }
  }
}

// The same for 16x16 accumulator tiles: lanes l, l+16, l+32, l+48 write 64 contiguous bytes.
template <int AM, int AN>
__device__ __forceinline__ void store_wave_tile16_f32(f32x4v_t (&acc)[AM][AN], float* __restrict__ P,
                                                      int64_t ldp, int64_t row0, int64_t col0,
                                                      int64_t M, int64_t N, int lane) {
#pragma unroll
  for (int i = 0; i < AM; ++i) {
    const int64_t row = row0 + i * 16 + (lane & 15);
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < AN; ++j) {
      const int64_t col = col0 + j * 16 + 4 * (lane >> 4);
      float* dst = P + row * ldp + col;
      if (col + 4 <= N) {
        f32x4_unaligned_t v = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        *reinterpret_cast<f32x4_unaligned_t*>(dst) = v;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < N) dst[e] = acc[i][j][e];
      }
    }
  }
}

// c[m, n] = epilogue(sum over the splits (in order) of partial[s][m][n] + bias[n]), one cast.
// VEC = 4: four consecutive columns per thread (n % 4 == 0 keeps them in one row).
template <typename T, int EPI, int VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(T* __restrict__ c,
                                                            const float* __restrict__ partial,
                                                            const T* __restrict__ bias, int64_t m,
                                                            int64_t n, int64_t ldc, int splits,
                                                            bool twice) {
  const int64_t total = m * n;
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * VEC;
  if (i >= total) return;
  float sum[VEC];
  if constexpr (VEC == 4) {
    typedef float f32x4_aligned_t __attribute__((ext_vector_type(4)));
    f32x4_aligned_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_aligned_t*>(partial + i));
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[e] = v[e];
    for (int s = 1; s < splits; ++s) {
      v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_aligned_t*>(partial + s * total + i));
#pragma unroll
      for (int e = 0; e < 4; ++e) sum[e] += v[e];
    }
  } else {
    sum[0] = partial[i];
    for (int s = 1; s < splits; ++s) sum[0] += partial[s * total + i];
  }
  const int64_t row = i / n, col = i - row * n;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    if (bias != nullptr) sum[e] += to_f32(bias[col + e]);
    c[row * ldc + col + e] = finish<T, EPI>(sum[e], twice);
  }
}

// Launches the reduction over `splits` partials (workspace is 16-byte aligned or the scalar form runs).
template <typename T, int EPI>
static inline void launch_splitk_reduce(T* c, const float* partial, const T* bias, int64_t m,
                                        int64_t n, int64_t ldc, int splits, bool twice,
                                        hipStream_t stream) {
  const int64_t total = m * n;
  if (n % 4 == 0 && (reinterpret_cast<uintptr_t>(partial) & 15) == 0) {
    const int64_t threads = total / 4;
    splitk_reduce_kernel<T, EPI, 4><<<dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream>>>(
        c, partial, bias, m, n, ldc, splits, twice);
  } else {
    splitk_reduce_kernel<T, EPI, 1><<<dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream>>>(
        c, partial, bias, m, n, ldc, splits, twice);
  }
}

// B_KMAJOR: B is stored [N, K] (ldb = pitch of an N-row); otherwise [K, N].
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KMAJOR, int EPI>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_mfma_kernel(GemmArgs g) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 MFMA tiles per wave
  constexpr int A_BYTES = BM * kLineBytes, B_BYTES = BN * kLineBytes;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int ROWS_PER_PASS = NT / 8;           // rows covered by one 16-byte load per thread
  constexpr int A_LOADS = BM / ROWS_PER_PASS;
  constexpr int B_LOADS = BN / ROWS_PER_PASS;
  constexpr int B_BLOCKS = (BN + NT - 1) / NT;    // 8x8 transpose blocks per thread (N-major B)
  constexpr int KSTEPS = kBK / 16;
  static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile/threads mismatch");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  int tile_m, tile_n;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
  const int64_t m0 = static_cast<int64_t>(tile_m) * BM;
  const int64_t n0 = static_cast<int64_t>(tile_n) * BN;
  const int64_t batch = blockIdx.y;
  const T* __restrict__ A = static_cast<const T*>(g.a) + batch * g.stride_a;
  const T* __restrict__ B = static_cast<const T*>(g.b) + batch * g.stride_b;
  T* __restrict__ C = static_cast<T*>(g.c) + batch * g.stride_c;
  const int64_t M = g.m, N = g.n, K = g.k;

  // ---- global -> register staging -------------------------------------------------------
  const int ld_row = tid >> 3;   // row inside one pass
  const int ld_chunk = tid & 7;  // 16-byte chunk inside the 128-byte line
  u32x4_t a_stage[A_LOADS];
  u32x4_t b_stage[B_KMAJOR ? B_LOADS : B_BLOCKS * 8];
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};

  // Per-lane byte offsets from the (wave-uniform) operand base are computed once, with rows
  // clamped to the last valid one (results of such rows are never stored), so the main loop
  // needs no predication and addresses are "uniform base + 32-bit lane offset".
  const unsigned char* a_base = reinterpret_cast<const unsigned char*>(A);
  const unsigned char* b_base = reinterpret_cast<const unsigned char*>(B);
  uint32_t a_off[A_LOADS];
#pragma unroll
  for (int j = 0; j < A_LOADS; ++j) {
    int64_t row = m0 + ld_row + j * ROWS_PER_PASS;
    row = row < M ? row : M - 1;
    a_off[j] = static_cast<uint32_t>((row * g.lda + ld_chunk * 8) * 2);
  }
  uint32_t b_off[B_KMAJOR ? B_LOADS : 1];
  if constexpr (B_KMAJOR) {
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) {
      int64_t row = n0 + ld_row + j * ROWS_PER_PASS;
      row = row < N ? row : N - 1;
      b_off[j] = static_cast<uint32_t>((row * g.ldb + ld_chunk * 8) * 2);
    }
  }

  // FULL: every 16-byte chunk of the stage lies below K (no predication).
  auto load_stage = [&](int64_t k0, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    const bool k_ok = FULL || (k0 + ld_chunk * 8 < K);
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j)
      a_stage[j] = k_ok ? *reinterpret_cast<const u32x4_t*>(a_base + k0 * 2 + a_off[j]) : zero4;
    if constexpr (B_KMAJOR) {
#pragma unroll
      for (int j = 0; j < B_LOADS; ++j)
        b_stage[j] = k_ok ? *reinterpret_cast<const u32x4_t*>(b_base + k0 * 2 + b_off[j]) : zero4;
    } else {
      // Thread owns 8(k) x 8(n) blocks: k-chunk kc = blk / (BN/8), n-group ng = blk % (BN/8).
#pragma unroll
      for (int q = 0; q < B_BLOCKS; ++q) {
        const int blk = tid + q * NT;
        const int kc = blk / (BN / 8), ng = blk % (BN / 8);
        const int64_t nn = n0 + ng * 8;
        const bool active = (BN % NT == 0) || (blk < BN);
        const bool whole = nn + 8 <= N;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const int64_t kk = k0 + kc * 8 + r;
          u32x4_t v = zero4;
          if (active && (FULL || kk < K)) {
            const T* src = B + kk * g.ldb + nn;
            if (whole) {
              v = *reinterpret_cast<const u32x4_t*>(src);
            } else {
              // ragged right edge: element-wise, never past column N-1
              unsigned short e[8];
#pragma unroll
              for (int t = 0; t < 8; ++t)
                e[t] = (nn + t < N) ? reinterpret_cast<const unsigned short*>(src)[t]
                                    : static_cast<unsigned short>(0);
              v[0] = e[0] | (static_cast<uint32_t>(e[1]) << 16);
              v[1] = e[2] | (static_cast<uint32_t>(e[3]) << 16);
              v[2] = e[4] | (static_cast<uint32_t>(e[5]) << 16);
              v[3] = e[6] | (static_cast<uint32_t>(e[7]) << 16);
            }
          }
          b_stage[q * 8 + r] = v;
        }
      }
    }
  };
  auto store_stage = [&](int buf) {
    unsigned char* sa = smem + buf * STAGE_BYTES;
    unsigned char* sb = sa + A_BYTES;
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
      const int row = ld_row + j * ROWS_PER_PASS;
      *reinterpret_cast<u32x4_t*>(sa + lds_offset(row, ld_chunk)) = a_stage[j];
    }
    if constexpr (B_KMAJOR) {
#pragma unroll
      for (int j = 0; j < B_LOADS; ++j) {
        const int row = ld_row + j * ROWS_PER_PASS;
        *reinterpret_cast<u32x4_t*>(sb + lds_offset(row, ld_chunk)) = b_stage[j];
      }
    } else {
#pragma unroll
      for (int q = 0; q < B_BLOCKS; ++q) {
        const int blk = tid + q * NT;
        if ((BN % NT == 0) || (blk < BN)) {
          const int kc = blk / (BN / 8), ng = blk % (BN / 8);
          // 8x8 transpose of 16-bit elements: out[i] holds k = 0..7 for column i.
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            u32x4_t o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const uint32_t lo = b_stage[q * 8 + 2 * j][i >> 1];
              const uint32_t hi = b_stage[q * 8 + 2 * j + 1][i >> 1];
              o[j] = (i & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
            }
            const int row = ng * 8 + i;
            *reinterpret_cast<u32x4_t*>(sb + lds_offset(row, kc)) = o;
          }
        }
      }
    }
  };

  // ---- accumulators and fragments -------------------------------------------------------
  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;  // which 8-wide K half of the 16-wide MFMA step
  u32x4_t af[2][TM], bf[2][TN];

  auto load_frags = [&](int buf, int ks, int slot) {
    const unsigned char* sa = smem + buf * STAGE_BYTES;
    const unsigned char* sb = sa + A_BYTES;
    const int chunk = ks * 2 + frag_half;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm * WM + i * 32 + frag_row;
      af[slot][i] = *reinterpret_cast<const u32x4_t*>(sa + lds_offset(row, chunk));
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = wn * WN + j * 32 + frag_row;
      bf[slot][j] = *reinterpret_cast<const u32x4_t*>(sb + lds_offset(row, chunk));
    }
  };
  auto mfma_step = [&](int slot) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::run(bf[slot][j], af[slot][i], acc[i][j]);
  };

  // ---- main loop ------------------------------------------------------------------------
  const int64_t k_tiles = (K + kBK - 1) / kBK;
  const int64_t full_tiles = K / kBK;  // stages that need no K predication
  if (full_tiles > 0) {
    load_stage(0, std::true_type{});
  } else {
    load_stage(0, std::false_type{});
  }
  store_stage(0);
  __syncthreads();
  load_frags(0, 0, 0);
  for (int64_t kt = 0; kt < k_tiles; ++kt) {
    const int buf = static_cast<int>(kt & 1);
    const bool more = kt + 1 < k_tiles;
    if (more) {
      if (kt + 1 < full_tiles) {
        load_stage((kt + 1) * kBK, std::true_type{});
      } else {
        load_stage((kt + 1) * kBK, std::false_type{});
      }
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS - 1; ++ks) {
      load_frags(buf, ks + 1, (ks + 1) & 1);
      mfma_step(ks & 1);
    }
    if (more) store_stage(buf ^ 1);
    __syncthreads();
    if (more) load_frags(buf ^ 1, 0, 0);  // KSTEPS is even: slot 0 is free again
    mfma_step((KSTEPS - 1) & 1);
  }

  // ---- epilogue -------------------------------------------------------------------------
  const T* __restrict__ bias = static_cast<const T*>(g.bias);
  __syncthreads();  // every wave is done with the operand buffers: reuse them for the output
  static_assert(WAVES_M * WAVES_N * BandLayout<WN>::BYTES <= 2 * STAGE_BYTES, "band staging");
  static_assert(WAVES_M * WAVES_N * BandLayoutF32<WN>::BYTES <= 2 * STAGE_BYTES, "fp32 band staging");
  const EpilogueArgs ep = epilogue_args<T>(g, blockIdx.y);
  lds_byte_t* band = (lds_byte_t*)smem +
                     wave * (ep.wide() ? BandLayoutF32<WN>::BYTES : BandLayout<WN>::BYTES);
  void* Cout = g.out_f32 ? static_cast<void*>(static_cast<float*>(g.c) + batch * g.stride_c)
                         : static_cast<void*>(C);
  store_wave_tile<T, EPI, TM, TN>(acc, band, Cout, g.ldc, m0 + wm * WM, n0 + wn * WN, M, N, bias,
                                  g.stream_c != 0, ep, lane);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KMAJOR, int EPI>
static int launch_mfma(const GemmArgs& base, int64_t batch, hipStream_t stream) {
  constexpr int SMEM = 2 * (BM + BN) * kLineBytes;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  static bool configured = false;
  auto kernel = gemm_mfma_kernel<T, BM, BN, WAVES_M, WAVES_N, B_KMAJOR, EPI>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    if (e != hipSuccess) return static_cast<int>(e);
    configured = true;
  }
  GemmArgs g = base;
  g.tiles_m = static_cast<int>((g.m + BM - 1) / BM);
  g.tiles_n = static_cast<int>((g.n + BN - 1) / BN);
  g.stream_c = g.m * g.n * batch * (g.out_f32 ? 4 : 2) >= (int64_t{256} << 20);
  const int64_t tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (tiles >= (int64_t{1} << 31) || batch > 65535) return TMB_ERR_UNSUPPORTED;
  // A product whose whole K fits one stage (attention's q.k^T with head size 64) never touches
  // the second buffer: with half the LDS twice as many workgroups share a CU, and the load,
  // multiply and store phases of different tiles overlap (such products are bound by their
  // output stores, not by the matrix cores). The output bands overlay the stage.
  constexpr int WN = BN / WAVES_N;
  constexpr int kBands = WAVES_M * WAVES_N * BandLayoutF32<WN>::BYTES;
  constexpr int kOneStage = (BM + BN) * kLineBytes > kBands ? (BM + BN) * kLineBytes : kBands;
  const int smem = g.k <= kBK ? kOneStage : SMEM;
  kernel<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(batch)), dim3(NT), smem, stream>>>(g);
  return check_launch();
}

}  // namespace tmb
