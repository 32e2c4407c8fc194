// MFMA GEMM with direct-to-LDS loads for gfx950: A [M,K] K-major; B either [N,K] (K-major, the
// transposed view of a weight) or [K,N] (N-major).
//
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight into LDS (lane l
// of a wave lands at base + 16*l), so no staging registers and no ds_write instructions are
// spent on the operands. K is walked in stages of BK (32 or 64); R stages form a ring in LDS
// and up to R-1 of them are in flight while one is multiplied. Each wave waits only for its own
// loads of the stage needed next (s_waitcnt vmcnt(N) with N = the loads of the younger
// stages), then one s_barrier makes every wave's part of that stage visible. The 256 x 256 x 64
// tile, whose two whole stages would fill 128 KB, keeps two buffers for A and three for B instead
// (160 KB): B is requested two stages ahead, so only half of a stage has to land within one step.
//
// LDS stage layout of a K-major operand: one line of BK*2 bytes per matrix row, its 16-byte
// chunks XOR-swizzled (ring_swizzle): a ds_read_b128 is served sixteen lanes at a time from 64
// banks (256 bytes), and the fragment fetch of 16 consecutive rows then touches 16 distinct
// 16-byte bank groups. The swizzle is applied on the global side: each lane of a load picks the
// source chunk that belongs at its LDS slot.
//
// N-major B is staged as it lies in memory, [BK k][BN n], and its fragments are fetched with
// ds_read_b64_tr_b16: sixteen lanes read a 4(k) x 16(n) block as 8-byte row pieces and get it
// back transposed (lane = n, four consecutive k), which is the MFMA operand layout, so no
// shuffle or repacking is spent on the transpose. Its 16-byte chunks are XOR-swizzled with
// 4*(k%4), which spreads the four k-rows of such a block over distinct banks, and with
// 2*((k/8)%2), which does the same for two groups of 16 lanes that read blocks eight k apart
// (the 16-row fragments of v_mfma_f32_16x16x32).
//
// The ring is unrolled by hand (stage indices are compile-time), so every fragment read is a
// per-lane base register plus an immediate offset.
#pragma once

#include <type_traits>
#include <utility>

#include "gemm_mfma.h"

// Diagnostic builds of the ring kernels (`sh build.sh -DTMB_GEMM_DIAG=n`, results are wrong by
// construction): what a launch takes without one of its parts. 1: no epilogue (one dword per
// lane keeps the products alive); 2: no operand fetch (the DMA is skipped: whatever LDS holds is
// multiplied); 3: every tile fetches the operands of tile (0, 0) (all L2 hits); 4: 1 and 2.
#ifndef TMB_GEMM_DIAG
#define TMB_GEMM_DIAG 0
#endif

namespace tmb {

typedef __attribute__((address_space(3))) void lds_void_t;

// XOR swizzle of the 16-byte chunks of a K-major LDS line of LINE bytes (64 or 128). A
// ds_read_b128 is served sixteen lanes at a time from 64 banks (a 256-byte window); 256/LINE
// consecutive rows share a window, so the swizzle must differ between rows that are a multiple
// of 256/LINE apart: (row / (256/LINE)) mod (LINE/16). Adding 32 rows leaves it unchanged.
template <int LINE>
__device__ __forceinline__ int ring_swizzle(int row) {
  return (row / (256 / LINE)) & (LINE / 16 - 1);
}

template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), unrolled at compile time.
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// s_waitcnt with vmcnt = VM, lgkmcnt = 0 (expcnt left at its maximum).
template <int VM>
__device__ __forceinline__ void wait_vm_lgkm0() {
  static_assert(VM >= 0 && VM < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt((VM & 0xF) | (7 << 4) | (0 << 8) | ((VM >> 4) << 14));
}

typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;

// Waves per SIMD the kernel is compiled for: as many workgroups as the ring leaves room for in
// the 160 KB LDS (at most two: a second workgroup overlaps its prologue and epilogue with the
// first one's main loop), provided the accumulators fit the register share that leaves.
constexpr int ring_waves_per_simd(int bm, int bn, int bk, int waves, int stages) {
  const int lds = stages * (bm + bn) * bk * 2;
  const int wgs = 160 * 1024 / lds >= 2 ? 2 : 1;
  const int acc = (bm * bn) / (waves * 64);  // fp32 accumulator registers per lane
  const int want = wgs * waves / 4;
  return (want >= 1 && acc + 64 <= 512 / want) ? want : (waves / 4 >= 1 ? waves / 4 : 1);
}

template <int BM, int BN, int BK, int WAVES, int R>
constexpr bool kRingPersistent = ring_waves_per_simd(BM, BN, BK, WAVES, R) <= 2;

// A_MMAJOR: A is stored [K, M] (the transposed view of a [K, M] matrix: the weight-gradient
// product dy^T x); it is then staged and read exactly like N-major B.
// OUT_F32: a split-K launch: the batch index is the split, the accumulators are stored as fp32
// partials (no bias, no epilogue, no cast).
// MI16_: multiply with v_mfma_f32_16x16x32 instead of v_mfma_f32_32x32x16.
template <typename T, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int R, bool B_KMAJOR, int EPI,
          bool A_MMAJOR = false, bool OUT_F32 = false, bool MI16_ = (BK == 64)>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64,
                             ring_waves_per_simd(BM, BN, BK, WAVES_M* WAVES_N, R))
void gemm_ring_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  // v_mfma_f32_16x16x32 takes k-steps of 32: two per 64-deep stage, one per 32-deep stage (the
  // fragment slots then alternate from stage to stage, or there is only one, see below). Large
  // products are limited by the power the chip may draw, and this form draws less per
  // multiply-add: +3-8 % at K >= 4096, +2-4 % at K = 768 .. 3072; the launcher keeps the
  // 32x32x16 form where it measured faster (short K with a streamed output, split-K partials,
  // small launches, N-major B on the 128 x 128 x 32 tile).
  static_assert(!MI16_ || BK == 64 || !(R == 2 && BM == 256 && BN == 256),
                "the split ring is 64 deep");
  constexpr bool MI16 = MI16_;
  constexpr int FRAG = MI16 ? 16 : 32;                // rows of an operand fragment
  constexpr int TM = WM / FRAG, TN = WN / FRAG;       // result tiles per wave
  constexpr int LINE = BK * 2;         // bytes of one row of a K-major operand per stage
  constexpr int KSTEPS = BK / (MI16 ? 32 : 16);       // MFMA k-steps per stage
  constexpr int KCHUNKS = MI16 ? 4 : 2;               // 16-byte chunks of a row per k-step
  constexpr int LPR = LINE / 16;       // lanes (16-byte chunks) per row of a load
  constexpr int RPG = 1024 / LINE;     // rows per 1 KiB load
  constexpr int A_BYTES = BM * LINE, B_BYTES = BN * LINE;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = A_BYTES / 1024 / NW, B_GROUPS = B_BYTES / 1024 / NW;  // loads per wave
  constexpr int PER_STAGE = A_GROUPS + B_GROUPS;
  static_assert(BK == 32 || BK == 64, "a stage is 32 or 64 deep");
  // The 256 x 256 x 64 tile fills 128 KB with two whole stages, which leaves a stage's loads less
  // than one step to arrive. Its ring is therefore split: two buffers for A (requested one stage
  // ahead) and three for B (two stages ahead), 160 KB in all. Halving the burst that has to land
  // within one step is worth 3-9 % at K = 8192 and nothing at short K.
  constexpr bool SPLIT_RING = (R == 2 && BM == 256 && BN == 256 && BK == 64);
  constexpr int RING_BYTES = SPLIT_RING ? 2 * A_BYTES + 3 * B_BYTES : R * STAGE_BYTES;
  static_assert(R >= 2 && RING_BYTES <= 160 * 1024, "ring does not fit the 160 KB LDS");
  static_assert(A_GROUPS >= 1 && B_GROUPS >= 1 && A_BYTES % (1024 * NW) == 0 &&
                    B_BYTES % (1024 * NW) == 0,
                "tile does not split into whole 1 KiB loads per wave");
  __shared__ __attribute__((aligned(1024))) unsigned char ring[RING_BYTES];

  // All workgroups of a persistent launch finish their tiles at the same time; with an output
  // that streams to memory their store bursts then collide while the matrix pipes idle. A start
  // offset of a few microseconds per phase keeps them apart for the whole launch (measured on a
  // 32768 x 50257 x 768 product: 2.62 -> 2.44 ms with four phases 5 us apart; 8 or 12 us less).
  if (g.stagger_ticks > 0) {
    const uint64_t t0 = wall_clock64();
    const uint64_t wait = static_cast<uint64_t>((blockIdx.x / 8) % 4) * g.stagger_ticks;
    while (wall_clock64() - t0 < wait) __builtin_amdgcn_s_sleep(8);
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  int64_t m0 = 0, n0 = 0;  // origin of the tile being worked on (set per tile below)
  int64_t batch = blockIdx.y;
  int64_t only_tile = -1;  // >= 0: this workgroup's one tile, as a position in the walk of tiles
  if constexpr (OUT_F32) {
    if (g.xcd_chunk > 0) {
      const uint32_t pair = (blockIdx.x % 8) * static_cast<uint32_t>(g.xcd_chunk) + blockIdx.x / 8;
      const uint32_t tiles = static_cast<uint32_t>(g.tiles_m) * static_cast<uint32_t>(g.tiles_n);
      if (pair >= tiles * static_cast<uint32_t>(g.splits)) return;  // (the whole workgroup, before any barrier)
      batch = __builtin_amdgcn_readfirstlane(static_cast<int>(pair / tiles));
      only_tile = __builtin_amdgcn_readfirstlane(static_cast<int>(pair % tiles));
    }
  }
  const int64_t M = g.m, N = g.n;
  T* __restrict__ C = static_cast<T*>(g.c) + batch * g.stride_c;
  const unsigned char* a_base =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(g.a) + batch * g.stride_a);
  const unsigned char* b_base =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(g.b) + batch * g.stride_b);

  // Lane -> (row inside a 1 KiB load, LDS slot); the source chunk is slot ^ swizzle(row).
  // Rows past the edge re-read the last valid row; their results are never stored.
  const int r_in = lane / LPR, slot = lane % LPR;
  uint32_t a_off[A_GROUPS], b_off[B_GROUPS];
  auto plan_tile_loads = [&]() {
#pragma unroll
  for (int j = 0; j < A_GROUPS; ++j) {
    if constexpr (!A_MMAJOR) {
      const int row = (wave * A_GROUPS + j) * RPG + r_in;
      const int chunk = slot ^ ring_swizzle<LINE>(row);
      int64_t grow = m0 + row;
      grow = grow < M ? grow : M - 1;
      a_off[j] = static_cast<uint32_t>((grow * g.lda + chunk * 8) * 2);
    } else {
      // stage bytes [group*1024 + 16*lane] = k-row (BM*2 bytes each), swizzled 16-byte slot
      const int at = (wave * A_GROUPS + j) * 1024 + lane * 16;
      const int krow = at / (BM * 2);
      const int chunk = ((at % (BM * 2)) >> 4) ^ ((krow & 3) << 2) ^ (((krow >> 3) & 1) << 1);
      int64_t col = m0 + chunk * 8;
      col = col < M ? col : m0;  // rows past the edge: any valid address, never stored
      a_off[j] = static_cast<uint32_t>((krow * g.lda + col) * 2);
    }
  }
#pragma unroll
  for (int j = 0; j < B_GROUPS; ++j) {
    if constexpr (B_KMAJOR) {
      const int row = (wave * B_GROUPS + j) * RPG + r_in;
      const int chunk = slot ^ ring_swizzle<LINE>(row);
      int64_t grow = n0 + row;
      grow = grow < N ? grow : N - 1;
      b_off[j] = static_cast<uint32_t>((grow * g.ldb + chunk * 8) * 2);
    } else {
      // stage bytes [group*1024 + 16*lane] = k-row (BN*2 bytes each), swizzled 16-byte slot
      const int at = (wave * B_GROUPS + j) * 1024 + lane * 16;
      const int krow = at / (BN * 2);
      const int chunk = ((at % (BN * 2)) >> 4) ^ ((krow & 3) << 2) ^ (((krow >> 3) & 1) << 1);
      int64_t col = n0 + chunk * 8;
      col = col < N ? col : n0;  // columns past the edge: any valid address, never stored
      b_off[j] = static_cast<uint32_t>((krow * g.ldb + col) * 2);
    }
  }
  };
  const int64_t b_kstep = B_KMAJOR ? 2 : g.ldb * 2;  // bytes per unit of k in B
  const int64_t a_kstep = A_MMAJOR ? g.lda * 2 : 2;

  // The loads are written as inline assembly: M0 carries the LDS destination of the wave's
  // 1 KiB, the SGPR pair the tile's base at this k, the VGPR the lane's byte offset. Issued
  // through the compiler's own builtin, every later LDS wait in the loop degrades to
  // lgkmcnt(0) (it orders the DMA against all LDS traffic), which stalls each MFMA group on
  // loads issued for the next one. The compiler does not see these loads at all, so the
  // vmcnt waits below are placed by hand. In the 256 x 256 x 64
  // kernel sc1 (agent scope) makes the load skip the per-CU cache, which these once-read lines
  // only pass through: 2-8 % at K = 8192; the smaller tiles measured 2-8 % slower with it.
  typedef __attribute__((address_space(3))) unsigned char lds_u8;
  const uint32_t ring_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_u8*)ring));
  const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t a_m0 = ring_lds + wave_s * (A_GROUPS * 1024);
  const uint32_t b_m0 = ring_lds + A_BYTES + wave_s * (B_GROUPS * 1024);
  auto dma16 = [](uint32_t m0, uint32_t voff, const unsigned char* sbase) {
    if constexpr (TMB_GEMM_DIAG == 2 || TMB_GEMM_DIAG == 4) return;
    if constexpr (SPLIT_RING) {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 sc1"
                   :
                   : "s"(m0), "v"(voff), "s"(sbase)
                   : "memory", "m0");
    } else {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :
                   : "s"(m0), "v"(voff), "s"(sbase)
                   : "memory", "m0");
    }
  };
  auto fetch_a = [&](uint32_t off, int64_t k0) {
    const unsigned char* ak = a_base + k0 * a_kstep;
#pragma unroll
    for (int j = 0; j < A_GROUPS; ++j) dma16(a_m0 + off + j * 1024, a_off[j], ak);
  };
  auto fetch_b = [&](uint32_t off, int64_t k0) {
    const unsigned char* bk = b_base + k0 * b_kstep;
#pragma unroll
    for (int j = 0; j < B_GROUPS; ++j) dma16(b_m0 + off + j * 1024, b_off[j], bk);
  };
  auto fetch_stage = [&](uint32_t stage_off, int64_t k0) {
    fetch_a(stage_off, k0);
    fetch_b(stage_off, k0);
  };

  using acc_t = std::conditional_t<MI16, f32x4v_t, f32x16_t>;
  acc_t acc[TM][TN];

  // Fragment addresses as LDS byte offsets inside a stage: one per-lane register per k-step
  // (the XOR swizzle is not additive in the k chunk) and, for N-major B, per 32-column tile;
  // the 32-row tile index (and the k-step of N-major B) is an immediate offset of the ds_read.
  // a fragment is FRAG rows; lane -> (row, which eight k of the k-step)
  const int frag_row = lane & (FRAG - 1), frag_half = lane / FRAG;
  const int frag_swz = ring_swizzle<LINE>(frag_row);
  int a_lane[KSTEPS], b_lane[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    const int slot16 = ((ks * KCHUNKS + frag_half) ^ frag_swz) << 4;
    a_lane[ks] = (wm * WM + frag_row) * LINE + slot16;
    b_lane[ks] = A_BYTES + (wn * WN + frag_row) * LINE + slot16;
  }
  // N-major B: this lane's source piece of the transposed read. Within 16 lanes, lane j16 reads
  // k-row j16/4 and the 4 columns starting at 4*(j16%4); lanes 16..31 take the next 16 columns
  // and lanes 32..63 the upper eight k of the MFMA step.
  int bt_lane[TN];
  if constexpr (!B_KMAJOR) {
    // (16-row fragments: all four groups of 16 lanes read the same 16 columns, eight k apart)
    const int j16 = lane & 15, q = j16 >> 2, nsub = MI16 ? 0 : (lane >> 4) & 1;
    const int krow = frag_half * 8 + q;  // + k-step and + 4, which leave krow % 4 == q
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int ncol = wn * WN + j * FRAG + nsub * 16 + (j16 & 3) * 4;
      bt_lane[j] = A_BYTES + krow * (BN * 2) + (((ncol >> 3) ^ (q << 2) ^ ((frag_half & 1) << 1)) << 4) +
                   (ncol & 7) * 2;
    }
  }
  int at_lane[TM];
  if constexpr (A_MMAJOR) {
    const int j16 = lane & 15, q = j16 >> 2, msub = MI16 ? 0 : (lane >> 4) & 1;
    const int krow = frag_half * 8 + q;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mcol = wm * WM + i * FRAG + msub * 16 + (j16 & 3) * 4;
      at_lane[i] = krow * (BM * 2) + (((mcol >> 3) ^ (q << 2) ^ ((frag_half & 1) << 1)) << 4) +
                   (mcol & 7) * 2;
    }
  }
  typedef __attribute__((address_space(3))) u32x4_t lds_u32x4_t;
  u32x4_t af[2][TM], bf[2][TN];
  // ks is a compile-time constant at every call site (the k-step loop is unrolled).
  // (a_stage_off, b_stage_off): where the stage's A and B parts start; b_lane / bt_lane and b_m0
  // already carry the A_BYTES that separate the two inside a whole stage
  auto load_frags2 = [&](uint32_t a_stage_off, uint32_t b_stage_off, int ks, int s) {
    lds_u8* stage = (lds_u8*)ring + a_stage_off;
    lds_u8* stage_b = (lds_u8*)ring + b_stage_off;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if constexpr (!A_MMAJOR) {
        af[s][i] = *(const lds_u32x4_t*)(stage + a_lane[ks] + i * (FRAG * LINE));
      } else {
        lds_u8* src = stage + at_lane[i] + ks * (MI16 ? 32 : 16) * (BM * 2);
        const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(src));
        const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(src + 4 * (BM * 2)));
        typedef short i16x8_t __attribute__((ext_vector_type(8)));
        const i16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        af[s][i] = __builtin_bit_cast(u32x4_t, both);
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if constexpr (B_KMAJOR) {
        bf[s][j] = *(const lds_u32x4_t*)(stage_b + b_lane[ks] + j * (FRAG * LINE));
      } else {
        lds_u8* src = stage_b + bt_lane[j] + ks * (MI16 ? 32 : 16) * (BN * 2);
        const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(src));
        const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(src + 4 * (BN * 2)));
        typedef short i16x8_t __attribute__((ext_vector_type(8)));
        const i16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        bf[s][j] = __builtin_bit_cast(u32x4_t, both);
      }
    }
  };
  auto load_frags = [&](uint32_t stage_off, int ks, int s) {
    load_frags2(stage_off, stage_off, ks, s);
  };
  // tile rows [i0, i1) of the k-step whose fragments sit in slot s
  auto mfma_rows = [&](int s, int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (MI16) acc[i][j] = Mfma16<T>::run(bf[s][j], af[s][i], acc[i][j]);
        else acc[i][j] = Mfma<T>::run(bf[s][j], af[s][i], acc[i][j]);
      }
  };
  auto mfma_step = [&](int s) { mfma_rows(s, 0, TM); };
  // The barrier that ends a stage sits before the last k-step's MFMAs, which cover the LDS
  // latency of the next stage's first fragments. With two k-steps per stage that would be the
  // middle of the stage, and the stage requested at its start would have to land in half of
  // it: half of the last k-step is therefore issued before the barrier.
  constexpr int EARLY = MI16 ? TM / 2 : 0;
  // Four waves per SIMD leave a wave 128 registers, which the accumulators and two slots of
  // 16-row fragments exceed: such a configuration keeps one slot (the other waves of the SIMD
  // cover the LDS latency after the barrier).
  constexpr bool SINGLE_SLOT =
      MI16 && KSTEPS == 1 && ring_waves_per_simd(BM, BN, BK, WAVES_M * WAVES_N, R) >= 4;

  // Ring position as a byte offset that lives in an SGPR (every wave computes the same value).
  auto next_stage = [](uint32_t off) {
    return off + STAGE_BYTES == R * STAGE_BYTES ? 0u : off + STAGE_BYTES;
  };

  // One ring step: tile t sits in stage `cur` with its first fragments already in slot 0; the
  // stage before `cur` was multiplied in the previous step and is refilled with tile t+R-1.
  // INFLIGHT = tiles younger than t+1 whose loads may still be outstanding when t+1 is waited
  // for. sched_barrier(0): nothing is scheduled across. Left alone, the scheduler sinks each
  // fragment load to just before its MFMA and reuses one register for all of them, which puts
  // the LDS latency back on the critical path.
  // P: the fragment slot the stage's first k-step sits in. With an even number of k-steps per
  // stage it is always 0; a 32-deep stage multiplied with 16x16x32 is a single k-step, so the
  // slot alternates from stage to stage and the loops below run the steps in pairs.
  auto step = [&](uint32_t cur, uint32_t nxt, uint32_t pre, int64_t k_pre, auto issue_tag,
                  auto inflight_tag, auto parity_tag) {
    constexpr bool ISSUE = decltype(issue_tag)::value;
    constexpr int INFLIGHT = decltype(inflight_tag)::value;
    constexpr int P = decltype(parity_tag)::value;
    if constexpr (ISSUE) fetch_stage(pre, k_pre);
    if constexpr (SINGLE_SLOT) {
      mfma_step(0);
      __builtin_amdgcn_sched_barrier(0);
      wait_vm_lgkm0<INFLIGHT * PER_STAGE>();
      __builtin_amdgcn_s_barrier();
      load_frags(nxt, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    static_for<KSTEPS - 1>([&](auto ks_tag) {
      constexpr int ks = decltype(ks_tag)::value;
      load_frags(cur, ks + 1, (P + ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_step((P + ks) & 1);
      __builtin_amdgcn_sched_barrier(0);
    });
    constexpr int LAST = (P + KSTEPS - 1) & 1;
    if constexpr (EARLY > 0) {
      mfma_rows(LAST, 0, EARLY);
      __builtin_amdgcn_sched_barrier(0);
    }
    wait_vm_lgkm0<INFLIGHT * PER_STAGE>();
    __builtin_amdgcn_s_barrier();
    load_frags(nxt, 0, (P + KSTEPS) & 1);
    __builtin_amdgcn_sched_barrier(0);
    mfma_rows(LAST, EARLY, TM);
    __builtin_amdgcn_sched_barrier(0);
  };

  // The launcher guarantees k % BK == 0 and at least R-1 stages of k.
  int64_t k_tiles = g.k / BK;
  if constexpr (OUT_F32) {
    if (g.splits > 0) {
      const int64_t first = k_tiles * batch / g.splits, last = k_tiles * (batch + 1) / g.splits;
      a_base += first * BK * a_kstep;
      b_base += first * BK * b_kstep;
      k_tiles = last - first;
    }
  }
  // Persistent workgroups: the grid covers the CUs once and each workgroup walks the tile list
  // with the grid's stride, which hands every XCD the same sequence of tiles as one launch per
  // tile would. The stores of a tile drain while the next tile's operands are already being
  // fetched and multiplied.
  const int64_t total_tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  const EpilogueArgs ep = epilogue_args<T>(g, batch);
  // An fp32 residual is requested as a whole in front of the epilogue's first band where the
  // wave's share fits 64 registers: one wait for memory per wave tile instead of one per pass
  // (32768 x 768 x 768 with an fp32 residual stream: 81 -> 72 us). Such a launch stays a
  // sequence of phases in which either the matrix pipes or memory work, on all CUs at once
  // (43 us of the one, 19 us of residual reads, 15 us of stores). Two ways of mixing them were
  // measured and dropped: start offsets between workgroups add their own length, and a finished
  // tile held in registers, leaving two stores per step under the next tile's loads while the
  // next residual is requested early, is no faster (74 us): loads and stores retire in order, so
  // the waits for the operands then wait for the stores as well. Requesting the residual in front
  // of the tile's operand loads instead of here changes nothing either (72.9 us).
  ResidualTile<MI16 ? TM : 2, MI16 ? TN : 1> resid;
  // (only where 64 more registers are to be had: one workgroup of eight waves per CU)
  constexpr bool RESID_EARLY = MI16 && !OUT_F32 && EPI == TMB_EPI_NONE && decltype(resid)::FITS &&
                               BM == 256 && BN == 128 && BK == 64 && NW == 8;
  auto run_tile = [&](int64_t pid) {
  {
    int tile_m, tile_n;
    if (only_tile >= 0) tile_of_index(static_cast<int>(pid), g.tiles_m, g.tiles_n, tile_m, tile_n);
    else tile_of_block(static_cast<int>(pid), g.tiles_m, g.tiles_n, tile_m, tile_n);
    m0 = TMB_GEMM_DIAG == 3 ? 0 : static_cast<int64_t>(tile_m) * BM;
    n0 = TMB_GEMM_DIAG == 3 ? 0 : static_cast<int64_t>(tile_n) * BN;
    plan_tile_loads();
    m0 = static_cast<int64_t>(tile_m) * BM;
    n0 = static_cast<int64_t>(tile_n) * BN;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < (MI16 ? 4 : 16); ++e) acc[i][j][e] = 0.0f;
  }
  if constexpr (SPLIT_RING) {
    // A buffer i at i * A_BYTES, B buffer j at 2 * A_BYTES + j * B_BYTES (offsets below leave out
    // the A_BYTES that b_m0 / b_lane carry). Step t requests A of stage t+1 into the buffer of
    // stage t-1 and B of stage t+2 into the buffer of stage t-1; both were released by the
    // barrier of step t-1. The launcher guarantees at least two stages of k.
    constexpr uint32_t B0 = A_BYTES;
    auto a_next = [](uint32_t o) { return o == 0 ? static_cast<uint32_t>(A_BYTES) : 0u; };
    auto b_next = [](uint32_t o) {
      return o + B_BYTES == B0 + 3 * B_BYTES ? B0 : o + static_cast<uint32_t>(B_BYTES);
    };
    fetch_a(0, 0);
    fetch_b(B0, 0);
    fetch_b(B0 + B_BYTES, BK);
    wait_vm_lgkm0<B_GROUPS>();
    __builtin_amdgcn_s_barrier();
    load_frags2(0, B0, 0, 0);
    uint32_t a_cur = 0, b_cur = B0;
    auto split_step = [&](int64_t t, auto issue_b_tag) {
      constexpr bool ISSUE_B = decltype(issue_b_tag)::value;
      const uint32_t a_n = a_next(a_cur), b_n = b_next(b_cur);
      // A (needed at the end of this step) is requested at once, B (needed a step later) one
      // load per k-step, which keeps the request queue shorter (1-2 %)
      fetch_a(a_n, (t + 1) * BK);
      const uint32_t b_t = b_next(b_n);
      const unsigned char* bk2 = b_base + (t + 2) * BK * b_kstep;
      if constexpr (MI16) {
        // two k-steps of TM tile rows: B's loads go out between pairs of tile rows of the first
        // (+2-3 % over issuing them with A's; spreading A's loads as well costs 2-3 %: they are
        // needed at this step's barrier and want every cycle of it)
        static_assert(B_GROUPS <= TM / 2, "one B load per pair of tile rows");
        load_frags2(a_cur, b_cur, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        static_for<TM / 2>([&](auto r_tag) {
          constexpr int r = decltype(r_tag)::value;
          mfma_rows(0, 2 * r, 2 * r + 2);
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (ISSUE_B && r < B_GROUPS) dma16(b_m0 + b_t + r * 1024, b_off[r], bk2);
          __builtin_amdgcn_sched_barrier(0);
        });
      } else {
      if constexpr (ISSUE_B) {
        dma16(b_m0 + b_t, b_off[0], bk2);
#pragma unroll
        for (int j = KSTEPS; j < B_GROUPS; ++j) dma16(b_m0 + b_t + j * 1024, b_off[j], bk2);
      }
      static_for<KSTEPS - 1>([&](auto ks_tag) {
        constexpr int ks = decltype(ks_tag)::value;
        load_frags2(a_cur, b_cur, ks + 1, (ks + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (ISSUE_B && ks + 1 < B_GROUPS && ks + 1 < KSTEPS)
          dma16(b_m0 + b_t + (ks + 1) * 1024, b_off[ks + 1], bk2);
        __builtin_amdgcn_sched_barrier(0);
        mfma_step(ks & 1);
        __builtin_amdgcn_sched_barrier(0);
      });
      }
      // A of the next stage is older than B of the one after it: only the latter may be pending
      if constexpr (EARLY > 0) {
        mfma_rows((KSTEPS - 1) & 1, 0, EARLY);
        __builtin_amdgcn_sched_barrier(0);
      }
      wait_vm_lgkm0<ISSUE_B ? B_GROUPS : 0>();
      __builtin_amdgcn_s_barrier();
      load_frags2(a_n, b_n, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      mfma_rows((KSTEPS - 1) & 1, EARLY, TM);
      __builtin_amdgcn_sched_barrier(0);
      a_cur = a_n;
      b_cur = b_n;
    };
#pragma unroll 1
    for (int64_t t = 0; t + 2 < k_tiles; ++t) split_step(t, std::true_type{});
    split_step(k_tiles - 2, std::false_type{});
    static_for<KSTEPS - 1>([&](auto ks_tag) {
      constexpr int ks = decltype(ks_tag)::value;
      load_frags2(a_cur, b_cur, ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_step(ks & 1);
      __builtin_amdgcn_sched_barrier(0);
    });
    mfma_step((KSTEPS - 1) & 1);
  } else {
  {
    uint32_t off = 0;
#pragma unroll
    for (int t = 0; t < R - 1; ++t) {
      fetch_stage(off, t * BK);
      off += STAGE_BYTES;
    }
  }
  wait_vm_lgkm0<(R - 2) * PER_STAGE>();
  __builtin_amdgcn_s_barrier();
  load_frags(0, 0, 0);
  uint32_t cur = 0, pre = (R - 1) * STAGE_BYTES;
  // main part: every step also requests tile t+R-1
  auto main_step = [&](int64_t t, auto parity_tag) {
    const uint32_t nxt = next_stage(cur);
    step(cur, nxt, pre, (t + (R - 1)) * BK, std::true_type{},
         std::integral_constant<int, R - 2>{}, parity_tag);
    pre = cur;
    cur = nxt;
  };
  // the last R-1 tiles are already in flight or resident; the in-flight count runs down
  auto finish = [&](auto parity_tag) {
    constexpr int P0 = decltype(parity_tag)::value;
    static_for<R - 2>([&](auto s) {
      constexpr int P = (P0 + decltype(s)::value * KSTEPS) & 1;
      const uint32_t nxt = next_stage(cur);
      step(cur, nxt, pre, 0, std::false_type{},
           std::integral_constant<int, R - 3 - decltype(s)::value>{}, std::integral_constant<int, P>{});
      pre = cur;
      cur = nxt;
    });
    constexpr int P = SINGLE_SLOT ? 0 : (P0 + (R - 2) * KSTEPS) & 1;
    static_for<KSTEPS - 1>([&](auto ks_tag) {
      constexpr int ks = decltype(ks_tag)::value;
      load_frags(cur, ks + 1, (P + ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_step((P + ks) & 1);
      __builtin_amdgcn_sched_barrier(0);
    });
    mfma_step((P + KSTEPS - 1) & 1);
  };
  if constexpr (KSTEPS % 2 == 0 || SINGLE_SLOT) {
#pragma unroll 1
    for (int64_t t = 0; t + (R - 1) < k_tiles; ++t) main_step(t, std::integral_constant<int, 0>{});
    finish(std::integral_constant<int, 0>{});
  } else {
    int64_t t = 0;
#pragma unroll 1
    for (; t + R < k_tiles; t += 2) {
      main_step(t, std::integral_constant<int, 0>{});
      main_step(t + 1, std::integral_constant<int, 1>{});
    }
    if (t + (R - 1) < k_tiles) {  // wave-uniform
      main_step(t, std::integral_constant<int, 0>{});
      finish(std::integral_constant<int, 1>{});
    } else {
      finish(std::integral_constant<int, 0>{});
    }
  }
  }  // whole-stage ring

  if constexpr (OUT_F32) {
    float* P = static_cast<float*>(g.c) + batch * g.stride_c;
    if constexpr (MI16) store_wave_tile16_f32<TM, TN>(acc, P, g.ldc, m0 + wm * WM, n0 + wn * WN, M, N, lane);
    else store_wave_tile_f32<TM, TN>(acc, P, g.ldc, m0 + wm * WM, n0 + wn * WN, M, N, lane);
    return;
  }
  const T* __restrict__ bias = static_cast<const T*>(g.bias);
  __syncthreads();  // every wave is done with the ring: reuse it for the output
  static_assert(NW * BandLayout<WN>::BYTES <= RING_BYTES, "band staging");
  static_assert(NW * BandLayoutF32<WN>::BYTES <= RING_BYTES, "fp32 band staging");
  if constexpr (RESID_EARLY) resid.request(ep, m0 + wm * WM, n0 + wn * WN, M, N, lane);
  lds_byte_t* band = (lds_byte_t*)ring +
                     wave * (ep.wide() ? BandLayoutF32<WN>::BYTES : BandLayout<WN>::BYTES);
  void* Cout = g.out_f32 ? static_cast<void*>(static_cast<float*>(g.c) + batch * g.stride_c)
                         : static_cast<void*>(C);
  if constexpr (TMB_GEMM_DIAG == 1 || TMB_GEMM_DIAG == 4) {
    float keep = 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) keep += acc[i][j][0] + acc[i][j][3];
    static_cast<float*>(Cout)[wave * 64 + lane] = keep;
  } else if constexpr (MI16) {
    store_wave_tile16<T, EPI, TM, TN>(acc, band, Cout, g.ldc, m0 + wm * WM, n0 + wn * WN, M, N, bias,
                                      g.stream_c != 0, ep, lane, &resid);
  } else {
    store_wave_tile<T, EPI, TM, TN>(acc, band, Cout, g.ldc, m0 + wm * WM, n0 + wn * WN, M, N, bias,
                                    g.stream_c != 0, ep, lane);
  }
  };
  // Configurations compiled for four waves per SIMD have no registers to spare for the loop
  // state; their second resident workgroup already overlaps the tile boundaries.
  // (one call site for run_tile: called from two, it is no longer inlined)
  if constexpr (kRingPersistent<BM, BN, BK, WAVES_M * WAVES_N, R>) {
    const int64_t stride = only_tile >= 0 ? total_tiles : static_cast<int64_t>(gridDim.x);
#pragma unroll 1
    for (int64_t pid = only_tile >= 0 ? only_tile : static_cast<int64_t>(blockIdx.x); pid < total_tiles;
         pid += stride) {
      run_tile(pid);
      __syncthreads();  // the staging bands overlay the ring: all read back before the next fetch
    }
  } else {
    run_tile(only_tile >= 0 ? only_tile : static_cast<int64_t>(blockIdx.x));
  }
#endif
}

// Reads one dword of every 128-byte line of [p, p + bytes) with plain loads, which leaves the
// lines in the Infinity Cache (non-temporal loads do not). Run in front of a product whose output
// streams to memory: all XCDs walk the columns of B in step, so every tile of B is asked for by
// all of them at the same moment and by nobody again; when B is not cached each of these
// requests is a first miss that waits behind the output's stores in the memory controllers,
// longer than the ring's two stages of lookahead cover. 16384 x 50257 x 768 behind other work:
// 1.69-1.87 ms as it is, 1.14-1.19 ms behind a 22 us pass over the 77 MB of B (which is also what
// the same launch takes when it runs twice in a row).
__global__ __launch_bounds__(256) void warm_lines_kernel(const uint32_t* __restrict__ p, int64_t lines,
                                                         int64_t last_dword) {
  uint32_t seen = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < lines;
       i += static_cast<int64_t>(gridDim.x) * 256)
    seen ^= p[i * 32];
  if (blockIdx.x == 0 && threadIdx.x == 0) seen ^= p[last_dword];
  asm volatile("" : : "v"(seen));  // the loads have no other use
}

// Whether B is worth that pass: one matrix of 4 .. 128 MB (it has to fit beside the rest of the
// working set in the 256 MB cache).
inline void warm_b_for_streamed_output(const GemmArgs& g, int64_t batch, bool b_kmajor,
                                       hipStream_t stream) {
  if (!g.stream_c || batch != 1) return;
  const int64_t bytes = b_kmajor ? ((g.n - 1) * g.ldb + g.k) * 2 : ((g.k - 1) * g.ldb + g.n) * 2;
  if (bytes < (int64_t{4} << 20) || bytes > (int64_t{128} << 20)) return;
  const int64_t lines = bytes / 128;
  const int64_t blocks = (lines + 255) / 256;
  warm_lines_kernel<<<dim3(static_cast<unsigned>(blocks < 2048 ? blocks : 2048)), dim3(256), 0, stream>>>(
      static_cast<const uint32_t*>(g.b), lines, bytes / 4 - 1);
}

template <typename T, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int R, bool B_KMAJOR, int EPI,
          bool A_MMAJOR = false, bool OUT_F32 = false, bool MI16_ = (BK == 64)>
static int launch_ring(const GemmArgs& base, int64_t batch, hipStream_t stream) {
  GemmArgs g = base;
  g.tiles_m = static_cast<int>((g.m + BM - 1) / BM);
  g.tiles_n = static_cast<int>((g.n + BN - 1) / BN);
  g.stream_c = g.m * g.n * batch * (g.out_f32 ? 4 : 2) >= (int64_t{256} << 20);
  const int64_t tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (tiles >= (int64_t{1} << 31) || batch > 65535) return TMB_ERR_UNSUPPORTED;
  // as many workgroups as the device holds at once (a multiple of the 8 XCDs), shared between
  // the batch entries; each walks the tile list
  constexpr int kWgPerCu = ring_waves_per_simd(BM, BN, BK, WAVES_M * WAVES_N, R) * 4 /
                                       (WAVES_M * WAVES_N) >= 2 ? 2 : 1;
  int64_t resident = static_cast<int64_t>(compute_units()) * kWgPerCu / batch;
  resident = resident / 8 * 8;
  if (resident < 8) resident = 8;
  // (a launch whose workgroups all fit the device at once gets one workgroup per tile)
  const bool fits = tiles * batch <= static_cast<int64_t>(compute_units()) * kWgPerCu;
  const int64_t grid_x =
      (!kRingPersistent<BM, BN, BK, WAVES_M * WAVES_N, R> || tiles < resident || fits) ? tiles
                                                                                       : resident;
  // four start phases 5 us apart when every workgroup walks several tiles of a streamed output
  g.stagger_ticks = (g.stream_c && !OUT_F32 && grid_x == resident && tiles >= 4 * resident) ? 500 : 0;
  if (grid_x == resident && tiles >= 4 * resident) warm_b_for_streamed_output(g, batch, B_KMAJOR, stream);
  unsigned grid_y = static_cast<unsigned>(batch);
  int64_t grid_x_launch = grid_x;
  if constexpr (OUT_F32) {
    // (3072 x 768 x 32768 in 7 splits of 36 tiles: 559 -> 258 MB fetched past the L2s, 170 -> 162 us
    // with the reduction; 768 x 768 x 32768: 71 -> 59 us)
    if (g.splits > 0 && batch == g.splits && fits) {
      g.xcd_chunk = static_cast<int>((tiles * batch + 7) / 8);
      grid_x_launch = int64_t{8} * g.xcd_chunk;
      grid_y = 1;
    }
  }
  gemm_ring_kernel<T, BM, BN, BK, WAVES_M, WAVES_N, R, B_KMAJOR, EPI, A_MMAJOR, OUT_F32, MI16_>
      <<<dim3(static_cast<unsigned>(grid_x_launch), grid_y),
         dim3(WAVES_M * WAVES_N * 64), 0, stream>>>(g);
  return check_launch();
}

}  // namespace tmb
