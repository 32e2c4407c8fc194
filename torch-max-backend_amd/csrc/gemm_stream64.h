// Batched products with K = 64 (attention's q.k^T with head size 64, [b, m, 64] x [b, 64, n]):
// 2 * 64 FLOP per output element, so the kernel is bound by its output stores, and what has to be
// kept small is everything else a tile costs. One 128 x 128 tile is one LDS stage (a 128-byte
// line per row of a K-major operand), so the tiles of a launch are run as one stream of stages:
// persistent workgroups, operands by direct-to-LDS loads (no address arithmetic per tile beyond
// one scalar base: the launcher only takes shapes without edge tiles), tile i+1 in flight while
// tile i is multiplied and stored, the output bands overlaying the stage that was just consumed.
//
// Per tile and workgroup: barrier, request tile i+1, 16 MFMAs per wave on tile i, barrier, bands,
// wait for tile i+1 (requested a whole multiply-and-convert phase earlier), stores of tile i.
// The stores of a tile are only waited for one full iteration later.
#pragma once

#include "gemm_ring.h"

namespace tmb {

template <typename T, bool B_KMAJOR, int BUFS = 2, int BM = 128, int BN = 128, int WAVES_M = 2>
__global__ __launch_bounds__(256, BUFS == 2 ? 2 : 4) void gemm_k64_stream_kernel(GemmArgs g, int64_t total_tiles) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BK = 64, LINE = 128, NW = 4, WAVES_N = NW / WAVES_M;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32, KSTEPS = 4;
  static_assert(BK == 64 && WM % 32 == 0 && WN % 32 == 0, "wave tiles are whole 32 x 32 MFMA tiles");
  constexpr int LPR = LINE / 16, RPG = 1024 / LINE;
  constexpr int A_BYTES = BM * LINE, B_BYTES = BN * LINE, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = A_BYTES / 1024 / NW, B_GROUPS = B_BYTES / 1024 / NW;
  static_assert(NW * BandLayout<WN>::BYTES <= STAGE_BYTES, "bands overlay one stage");
  __shared__ __attribute__((aligned(1024))) unsigned char ring[BUFS * STAGE_BYTES];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r_in = lane / LPR, slot = lane % LPR;
  // lane offsets inside a tile (no edge tiles: nothing to clamp)
  uint32_t a_off[A_GROUPS], b_off[B_GROUPS];
#pragma unroll
  for (int j = 0; j < A_GROUPS; ++j) {
    const int row = (wave * A_GROUPS + j) * RPG + r_in;
    const int chunk = slot ^ ring_swizzle<LINE>(row);
    a_off[j] = static_cast<uint32_t>((static_cast<int64_t>(row) * g.lda + chunk * 8) * 2);
  }
#pragma unroll
  for (int j = 0; j < B_GROUPS; ++j) {
    if constexpr (B_KMAJOR) {
      const int row = (wave * B_GROUPS + j) * RPG + r_in;
      const int chunk = slot ^ ring_swizzle<LINE>(row);
      b_off[j] = static_cast<uint32_t>((static_cast<int64_t>(row) * g.ldb + chunk * 8) * 2);
    } else {
      const int at = (wave * B_GROUPS + j) * 1024 + lane * 16;
      const int krow = at / (BN * 2);
      const int chunk = ((at % (BN * 2)) >> 4) ^ ((krow & 3) << 2);
      b_off[j] = static_cast<uint32_t>((static_cast<int64_t>(krow) * g.ldb + chunk * 8) * 2);
    }
  }
  typedef __attribute__((address_space(3))) unsigned char lds_u8;
  const uint32_t ring_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_u8*)ring));
  const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t a_m0 = ring_lds + wave_s * (A_GROUPS * 1024);
  const uint32_t b_m0 = ring_lds + A_BYTES + wave_s * (B_GROUPS * 1024);
  auto dma16 = [](uint32_t m0, uint32_t voff, const unsigned char* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0), "v"(voff), "s"(sbase)
                 : "memory", "m0");
  };
  const int tiles_per_batch = g.tiles_m * g.tiles_n;
  struct TileAt {
    int64_t batch, m0, n0;
  };
  auto locate = [&](int64_t tile) {
    const int64_t b = tile / tiles_per_batch;
    const int t = static_cast<int>(tile - b * tiles_per_batch);
    const int tm = t / g.tiles_n, tn = t - tm * g.tiles_n;
    return TileAt{b, static_cast<int64_t>(tm) * BM, static_cast<int64_t>(tn) * BN};
  };
  auto fetch = [&](const TileAt& at, uint32_t stage_off) {
    const unsigned char* ab = reinterpret_cast<const unsigned char*>(
        static_cast<const T*>(g.a) + at.batch * g.stride_a + at.m0 * g.lda);
    const unsigned char* bb = reinterpret_cast<const unsigned char*>(
        static_cast<const T*>(g.b) + at.batch * g.stride_b + (B_KMAJOR ? at.n0 * g.ldb : at.n0));
#pragma unroll
    for (int j = 0; j < A_GROUPS; ++j) dma16(a_m0 + stage_off + j * 1024, a_off[j], ab);
#pragma unroll
    for (int j = 0; j < B_GROUPS; ++j) dma16(b_m0 + stage_off + j * 1024, b_off[j], bb);
  };

  // fragment addresses inside a stage (as in the ring kernel)
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int frag_swz = ring_swizzle<LINE>(frag_row);
  int a_lane[KSTEPS], b_lane[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    const int slot16 = ((ks * 2 + frag_half) ^ frag_swz) << 4;
    a_lane[ks] = (wm * WM + frag_row) * LINE + slot16;
    b_lane[ks] = A_BYTES + (wn * WN + frag_row) * LINE + slot16;
  }
  int bt_lane[TN];
  if constexpr (!B_KMAJOR) {
    const int j16 = lane & 15, q = j16 >> 2, nsub = (lane >> 4) & 1;
    const int krow = frag_half * 8 + q;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int ncol = wn * WN + j * 32 + nsub * 16 + (j16 & 3) * 4;
      bt_lane[j] = A_BYTES + krow * (BN * 2) + (((ncol >> 3) ^ (q << 2)) << 4) + (ncol & 7) * 2;
    }
  }
  typedef __attribute__((address_space(3))) u32x4_t lds_u32x4_t;

  const EpilogueArgs ep{nullptr, 0, false, false, false};
  const T* __restrict__ bias = static_cast<const T*>(g.bias);
  int64_t tile = blockIdx.x;
  if (tile >= total_tiles) return;  // whole workgroup
  if constexpr (BUFS == 2) {
    fetch(locate(tile), 0);
    wait_vm_lgkm0<0>();
  }
  uint32_t cur = 0;
#pragma unroll 1
  for (; tile < total_tiles; tile += gridDim.x) {
    const TileAt at = locate(tile);
    // everyone has read its bands out of the other stage (previous tile) and has seen this
    // tile's operands land (each wave waited for its own loads before its stores)
    __builtin_amdgcn_s_barrier();
    const int64_t next = tile + gridDim.x;
    const uint32_t other = BUFS == 2 ? cur ^ static_cast<uint32_t>(STAGE_BYTES) : 0u;
    if constexpr (BUFS == 2) {
      if (next < total_tiles) fetch(locate(next), other);
    } else {
      fetch(at, 0);
      wait_vm_lgkm0<0>();
      __builtin_amdgcn_s_barrier();
    }

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    lds_u8* stage = (lds_u8*)ring + cur;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      u32x4_t af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = *(const lds_u32x4_t*)(stage + a_lane[ks] + i * (32 * LINE));
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (B_KMAJOR) {
          bf[j] = *(const lds_u32x4_t*)(stage + b_lane[ks] + j * (32 * LINE));
        } else {
          lds_u8* src = stage + bt_lane[j] + ks * 16 * (BN * 2);
          const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(src));
          const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(src + 4 * (BN * 2)));
          typedef short i16x8_t __attribute__((ext_vector_type(8)));
          const i16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          bf[j] = __builtin_bit_cast(u32x4_t, both);
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::run(bf[j], af[i], acc[i][j]);
    }
    __syncthreads();  // every wave is done with this stage's operands: the bands overlay it
    // The loads of the next tile (requested above) are older than anything this wave still has
    // in flight except the previous tile's stores: waiting for all of them here, before this
    // tile's stores are issued, never waits for a store younger than one whole iteration.
    wait_vm_lgkm0<0>();
    lds_byte_t* band = (lds_byte_t*)ring + cur + wave * BandLayout<WN>::BYTES;
    T* C = static_cast<T*>(g.c) + at.batch * g.stride_c;
    store_wave_tile<T, TMB_EPI_NONE, TM, TN>(acc, band, C, g.ldc, at.m0 + wm * WM, at.n0 + wn * WN,
                                            g.m, g.n, bias, g.stream_c != 0, ep, lane);
    cur = other;
  }
#endif
}

// Shapes the stream kernel takes: K = 64, whole 128 x 128 tiles, 16-byte aligned operands whose
// rows are whole 16-byte chunks, no epilogue beyond the bias, no residual.
inline bool stream64_eligible(const GemmArgs& g, int64_t batch, int trans_b, int epilogue) {
  if (g.k != 64 || g.m % 128 != 0 || g.n % 128 != 0 || epilogue != TMB_EPI_NONE) return false;
  if (g.residual != nullptr || g.out_f32) return false;
  if (g.lda % 8 != 0 || g.ldb % 8 != 0 || !aligned16(g.a) || !aligned16(g.b)) return false;
  if (batch > 1 && (g.stride_a % 8 != 0 || g.stride_b % 8 != 0)) return false;
  // lane offsets are 32-bit byte offsets inside one tile's rows
  const int64_t a_span = 128 * g.lda * 2, b_span = (trans_b ? 128 : 64) * g.ldb * 2;
  if (a_span >= (int64_t{1} << 32) || b_span >= (int64_t{1} << 32)) return false;
  const int64_t tiles = (g.m / 128) * (g.n / 128) * batch;
  return tiles >= 512 && tiles < (int64_t{1} << 40);
}

template <typename T, bool B_KMAJOR, int BUFS = 2, int BM = 128, int BN = 128, int WAVES_M = 2>
static int launch_stream64(const GemmArgs& base, int64_t batch, hipStream_t stream,
                           int64_t grid_override = 0, int stream_override = -1) {
  GemmArgs g = base;
  g.tiles_m = static_cast<int>(g.m / BM);
  g.tiles_n = static_cast<int>(g.n / BN);
  // written once, 64 FLOP per byte pair: non-temporal stores whatever the size (measured 34 ->
  // 25 us on [48, 1024, 64] x [48, 64, 1024], where plain stores also leave through L2)
  g.stream_c = 1;
  const int64_t total = static_cast<int64_t>(g.tiles_m) * g.tiles_n * batch;
  int64_t grid = static_cast<int64_t>(compute_units()) * 2;
  if (grid_override > 0) grid = grid_override;
  if (stream_override >= 0) g.stream_c = stream_override;
  if (grid > total) grid = total;
  gemm_k64_stream_kernel<T, B_KMAJOR, BUFS, BM, BN, WAVES_M><<<dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream>>>(g, total);
  return check_launch();
}

}  // namespace tmb
