// Fused attention backward for gfx950: dq, dk, dv of out = softmax(scale * q k^T [+ causal mask]) v
// from q, k, v, out, the gradient of out and the forward's per-row log-sum-exp, without the
// [batch, heads, q_len, kv_len] probabilities ever reaching memory. Two launches, neither with
// atomics, so results do not depend on scheduling:
//
//   1. attention_bwd_dq_kernel: one workgroup = 128 queries of one (batch, head), 32 per wave, a
//      lane owning one query (as in the forward kernel). It first forms
//      delta = rowsum(dout * out) and lse * log2(e) for its queries and stores both for the second
//      launch, then walks the keys in blocks of 64 through an LDS ring:
//        S^T  = K Q^T, dP^T = V dout^T              (keys as MFMA rows, the query as the column)
//        P^T  = exp2(S^T * scale * log2 e - lse2),  dS^T = P^T (dP^T - delta) * scale
//        dQ^T += K^T dS^T                           (K^T by transposed LDS reads)
//   2. attention_bwd_dkv_kernel: one workgroup = 128 keys, 32 per wave, a lane owning one key
//      (K and V rows stay in registers); queries stream through the LDS ring in blocks of 64
//      together with their lse2 and delta:
//        S = Q K^T, dP = dout V^T                   (queries as MFMA rows, the key as the column)
//        P, dS as above
//        dV^T += dout^T P,  dK^T += Q^T dS          (dout^T, Q^T by transposed LDS reads)
//
// Scores and probabilities are recomputed in both launches (7 products instead of the minimal 5);
// in exchange there is no float32 dq accumulator to zero, add into and convert. P and dS are
// rounded to the storage type before they enter a product, as the forward kernel rounds P.
//
// Replaces the backward of the reference's fused attention
// (eager_kernels/aten_fast.py:4089-4170 `fast_fa4_bf16_d64_causal_backward`, which needs the same
// inputs and two float32 statistics buffers; registered as
// aten::_scaled_dot_product_flash_attention_backward, mojo_device/mojo_device_aten_ops.py:881).
#include "attention_tiles.h"

namespace tmb {

struct AttnBwdArgs {
  void* dq;
  void* dk;
  void* dv;
  const void* dout;
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const float* lse;  // [batch, heads, q_len]
  float* delta;      // [batch, heads, q_len] rowsum(dout * out), written by the dq launch
  float* lse2;       // [batch, heads, q_len] lse * log2(e), written by the dq launch
  int64_t q_sb, q_sh, q_st;  // element strides: batch, head, token (head_dim is contiguous)
  int64_t k_sb, k_sh, k_st;
  int64_t v_sb, v_sh, v_st;
  int64_t o_sb, o_sh, o_st;
  int64_t do_sb, do_sh, do_st;
  int64_t dq_sb, dq_sh, dq_st;
  int64_t dk_sb, dk_sh, dk_st;
  int64_t dv_sb, dv_sh, dv_st;
  int heads, q_len, kv_len;
  float scale;
  int causal;
};

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kBwdKvBuf = 2 * kAttnTile;            // dq launch: K + V
constexpr int kBwdQBuf = 2 * kAttnTile + 2 * 256;   // dk/dv launch: Q + dout + lse2 + delta

// The 4 x 16 bytes a lane holds of row `row` as the B operand of a head-dim contraction.
template <typename T>
__device__ __forceinline__ void load_operand_row(u32x4_t (&f)[4], const T* base, int64_t row,
                                                 int64_t stride, int half) {
  const T* src = base + row * stride + 8 * half;
#pragma unroll
  for (int s = 0; s < 4; ++s) f[s] = *reinterpret_cast<const u32x4_t*>(src + 16 * s);
}

// acc^T tile store: register r of tile dt is head-dim 32 dt + 8 (r / 4) + 4 half + r % 4
template <typename T>
__device__ __forceinline__ void store_row(T* dst, const f32x16_t (&acc)[2], int half) {
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2_t packed;
      packed[0] = pack2<T>(acc[dt][4 * g], acc[dt][4 * g + 1]);
      packed[1] = pack2<T>(acc[dt][4 * g + 2], acc[dt][4 * g + 3]);
      *reinterpret_cast<u32x2_t*>(dst + dt * 32 + g * 8 + half * 4) = packed;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void attention_bwd_dq_kernel(AttnBwdArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(1024))) unsigned char lds[kAttnStages * kBwdKvBuf];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  // query blocks are paired (n-1-u, then u) under a causal mask and rotated over the XCDs, as in
  // the forward kernel
  const int n_qb = (a.q_len + kAttnBQ - 1) / kAttnBQ;
  const bool paired = a.causal && n_qb > 1;
  const int units = paired ? (n_qb + 1) / 2 : n_qb;
  const int wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int bh = wg / units;
  const int unit = wg % units;
  const int b = bh / a.heads, h = bh % a.heads;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((attn_lds_u8*)lds));
  const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int ld_row = lane >> 3, ld_slot = lane & 7;
  const unsigned char* kp =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh);
  const unsigned char* vp =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh);
  auto fetch_block = [&](int blk, uint32_t buf_off) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = (wave * 2 + j) * 8 + ld_row;  // key inside the block
      int key = blk * kAttnBKV + row;
      key = key < a.kv_len ? key : a.kv_len - 1;    // masked later; any valid row will do
      const int chunk = ld_slot ^ attn_swz(row);
      const uint32_t k_off = static_cast<uint32_t>((static_cast<int64_t>(key) * a.k_st + chunk * 8) * 2);
      const uint32_t v_off = static_cast<uint32_t>((static_cast<int64_t>(key) * a.v_st + chunk * 8) * 2);
      const uint32_t dst = lds_base + buf_off + (wave_s * 2 + j) * 1024;
      attn_dma16(dst, k_off, kp);
      attn_dma16(dst + kAttnTile, v_off, vp);
    }
  };
  int row_off[4], tr_off[2][2];
#pragma unroll
  for (int s = 0; s < 4; ++s) row_off[s] = attn_row_read(lane, s);
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 2; ++r) tr_off[dt][r] = attn_tr_read(lane, dt, r);

  auto run_qblock = [&](const int qb) {
    const int q0 = qb * kAttnBQ, qw0 = q0 + wave * 32;
    const int qi = qw0 + (lane & 31);
    const int qrow = qi < a.q_len ? qi : a.q_len - 1;  // rows past the end are never stored
    const int64_t stat = (static_cast<int64_t>(b) * a.heads + h) * a.q_len + qrow;

    u32x4_t qf[4], dof[4];
    load_operand_row<T>(qf, static_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh, qrow, a.q_st, half);
    load_operand_row<T>(dof, static_cast<const T*>(a.dout) + b * a.do_sb + h * a.do_sh, qrow, a.do_st, half);
    float delta = 0.0f;
    {
      u32x4_t of[4];
      load_operand_row<T>(of, static_cast<const T*>(a.out) + b * a.o_sb + h * a.o_sh, qrow, a.o_st, half);
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float g0, g1, o0, o1;
          unpack2<T>(dof[s][e], g0, g1);
          unpack2<T>(of[s][e], o0, o1);
          delta = __builtin_fmaf(g0, o0, delta);
          delta = __builtin_fmaf(g1, o1, delta);
        }
      delta += other_half(delta, lane);
    }
    const float lse2 = a.lse[stat] * kLog2e;
    if (half == 0 && qi < a.q_len) {
      a.delta[stat] = delta;
      a.lse2[stat] = lse2;
    }

    int n_blocks = (a.kv_len + kAttnBKV - 1) / kAttnBKV;
    if (a.causal) {
      const int last_q = (q0 + kAttnBQ < a.q_len ? q0 + kAttnBQ : a.q_len) - 1;
      const int need = last_q / kAttnBKV + 1;  // keys 0..last_q
      n_blocks = n_blocks < need ? n_blocks : need;
    }
    f32x16_t acc_dq[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_dq[dt][e] = 0.0f;
    const float c = a.scale * kLog2e;

    fetch_block(0, 0);
    if (n_blocks > 1) fetch_block(1, kBwdKvBuf);
    uint32_t buf_off = 0;                  // ring position of block `blk`
    uint32_t free_off = 2 * kBwdKvBuf;     // the buffer read two iterations ago
    for (int blk = 0; blk < n_blocks; ++blk) {
      // each wave has 4 loads per block in flight; block blk+1 (if any) may stay outstanding
      if (blk + 1 < n_blocks) {
        __builtin_amdgcn_s_waitcnt(4 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(4) lgkmcnt(0)
      } else {
        __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(0) lgkmcnt(0)
      }
      __builtin_amdgcn_s_barrier();
      if (blk + 2 < n_blocks) fetch_block(blk + 2, free_off);
      const uint32_t cur_off = buf_off;
      free_off = buf_off;
      buf_off = buf_off + kBwdKvBuf == kAttnStages * kBwdKvBuf ? 0 : buf_off + kBwdKvBuf;

      const int kb = blk * kAttnBKV;
      if (a.causal && kb > qw0 + 31) continue;  // wave-uniform: every key lies above the diagonal
      attn_lds_u8* k_tile = (attn_lds_u8*)lds + cur_off;
      attn_lds_u8* v_tile = k_tile + kAttnTile;

      uint32_t dsf[2][8];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        f32x16_t acc_s, acc_dp;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc_s[e] = acc_dp[e] = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const u32x4_t kf = *(const attn_lds_u32x4_t*)(k_tile + row_off[s] + kt * 32 * kAttnRow);
          acc_s = Mfma<T>::run(kf, qf[s], acc_s);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const u32x4_t vf = *(const attn_lds_u32x4_t*)(v_tile + row_off[s] + kt * 32 * kAttnRow);
          acc_dp = Mfma<T>::run(vf, dof[s], acc_dp);
        }
        // register r is key kb + 32 kt + 8 (r / 4) + 4 half + r % 4 of query qi
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          float ds[2];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int key = kb + kt * 32 + ((r + i) >> 2) * 8 + half * 4 + ((r + i) & 3);
            const bool hidden = (a.causal && key > qi) || key >= a.kv_len;
            const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[r + i], c, -lse2));
            ds[i] = hidden ? 0.0f : p * (acc_dp[r + i] - delta) * a.scale;
          }
          dsf[kt][r >> 1] = pack2<T>(ds[0], ds[1]);
        }
      }
      // dQ^T += K^T dS^T over the 64 keys, k-step s = keys 16 s .. 16 s + 15 in register order
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        u32x4_t dsb;
#pragma unroll
        for (int e = 0; e < 4; ++e) dsb[e] = dsf[s >> 1][4 * (s & 1) + e];
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          const u32x4_t kt_op = attn_tr_operand(k_tile + s * 16 * kAttnRow, tr_off[dt][0], tr_off[dt][1]);
          acc_dq[dt] = Mfma<T>::run(kt_op, dsb, acc_dq[dt]);
        }
      }
    }
    if (qi < a.q_len)
      store_row<T>(static_cast<T*>(a.dq) + b * a.dq_sb + h * a.dq_sh + static_cast<int64_t>(qi) * a.dq_st,
                   acc_dq, half);
  };
  run_qblock(n_qb - 1 - unit);
  if (paired && unit != n_qb - 1 - unit) {
    __syncthreads();  // every wave is done with the K/V ring of the first block
    run_qblock(unit);
  }
#endif
}

template <typename T>
__global__ __launch_bounds__(256) void attention_bwd_dkv_kernel(AttnBwdArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(1024))) unsigned char lds[kAttnStages * kBwdQBuf];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  // Under a causal mask key block u meets the queries from 128 u on: its cost falls with u, so a
  // workgroup takes blocks u and n-1-u, and the pairs are rotated over the XCDs.
  const int n_kb = (a.kv_len + kAttnBQ - 1) / kAttnBQ;
  const bool paired = a.causal && n_kb > 1;
  const int units = paired ? (n_kb + 1) / 2 : n_kb;
  const int wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int bh = wg / units;
  const int unit = wg % units;
  const int b = bh / a.heads, h = bh % a.heads;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((attn_lds_u8*)lds));
  const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int ld_row = lane >> 3, ld_slot = lane & 7;
  const unsigned char* qp =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh);
  const unsigned char* dop =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.dout) + b * a.do_sb + h * a.do_sh);
  const int64_t stat0 = (static_cast<int64_t>(b) * a.heads + h) * a.q_len;
  // waves 0, 2 bring the block's lse2 and waves 1, 3 its delta (the same 256 bytes twice over:
  // every wave then has five loads per block in flight and one wait count serves all)
  const unsigned char* statp =
      reinterpret_cast<const unsigned char*>(((wave_s & 1) ? a.delta : a.lse2) + stat0);
  const uint32_t stat_dst = 2 * kAttnTile + (wave_s & 1) * 256;
  auto fetch_block = [&](int blk, uint32_t buf_off) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = (wave * 2 + j) * 8 + ld_row;  // query inside the block
      int query = blk * kAttnBKV + row;
      query = query < a.q_len ? query : a.q_len - 1;  // masked later; any valid row will do
      const int chunk = ld_slot ^ attn_swz(row);
      const uint32_t q_off = static_cast<uint32_t>((static_cast<int64_t>(query) * a.q_st + chunk * 8) * 2);
      const uint32_t do_off = static_cast<uint32_t>((static_cast<int64_t>(query) * a.do_st + chunk * 8) * 2);
      const uint32_t dst = lds_base + buf_off + (wave_s * 2 + j) * 1024;
      attn_dma16(dst, q_off, qp);
      attn_dma16(dst + kAttnTile, do_off, dop);
    }
    int query = blk * kAttnBKV + lane;
    query = query < a.q_len ? query : a.q_len - 1;
    attn_dma4(lds_base + buf_off + stat_dst, static_cast<uint32_t>(query) * 4u, statp);
  };
  int row_off[4], tr_off[2][2];
#pragma unroll
  for (int s = 0; s < 4; ++s) row_off[s] = attn_row_read(lane, s);
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 2; ++r) tr_off[dt][r] = attn_tr_read(lane, dt, r);
  const int n_qblocks = (a.q_len + kAttnBKV - 1) / kAttnBKV;

  auto run_kblock = [&](const int kblock) {
    const int k0 = kblock * kAttnBQ, kw0 = k0 + wave * 32;
    const int ki = kw0 + (lane & 31);
    const int krow = ki < a.kv_len ? ki : a.kv_len - 1;  // columns past the end are never stored
    u32x4_t kf[4], vf[4];
    load_operand_row<T>(kf, static_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh, krow, a.k_st, half);
    load_operand_row<T>(vf, static_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh, krow, a.v_st, half);

    // queries below the block's first key see none of its keys
    int first = a.causal ? k0 / kAttnBKV : 0;
    first = first < n_qblocks ? first : n_qblocks;
    const int n_blocks = n_qblocks - first;
    f32x16_t acc_dk[2], acc_dv[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_dk[dt][e] = acc_dv[dt][e] = 0.0f;
    const float c = a.scale * kLog2e;

    if (n_blocks > 0) fetch_block(first, 0);
    if (n_blocks > 1) fetch_block(first + 1, kBwdQBuf);
    uint32_t buf_off = 0;
    uint32_t free_off = 2 * kBwdQBuf;
    for (int it = 0; it < n_blocks; ++it) {
      const int blk = first + it;
      if (it + 1 < n_blocks) {
        __builtin_amdgcn_s_waitcnt(5 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(5) lgkmcnt(0)
      } else {
        __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(0) lgkmcnt(0)
      }
      __builtin_amdgcn_s_barrier();
      if (it + 2 < n_blocks) fetch_block(blk + 2, free_off);
      const uint32_t cur_off = buf_off;
      free_off = buf_off;
      buf_off = buf_off + kBwdQBuf == kAttnStages * kBwdQBuf ? 0 : buf_off + kBwdQBuf;

      const int q0 = blk * kAttnBKV;
      if (a.causal && q0 + kAttnBKV - 1 < kw0) continue;  // wave-uniform: every query is above
      attn_lds_u8* q_tile = (attn_lds_u8*)lds + cur_off;
      attn_lds_u8* do_tile = q_tile + kAttnTile;
      attn_lds_u8* stats = q_tile + 2 * kAttnTile;

      uint32_t pf[2][8], dsf[2][8];
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        f32x16_t acc_s, acc_dp;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc_s[e] = acc_dp[e] = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const u32x4_t qf = *(const attn_lds_u32x4_t*)(q_tile + row_off[s] + qt * 32 * kAttnRow);
          acc_s = Mfma<T>::run(qf, kf[s], acc_s);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const u32x4_t dof = *(const attn_lds_u32x4_t*)(do_tile + row_off[s] + qt * 32 * kAttnRow);
          acc_dp = Mfma<T>::run(dof, vf[s], acc_dp);
        }
        // register r is query q0 + 32 qt + 8 (r / 4) + 4 half + r % 4 against key ki
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int qoff = qt * 32 + g * 8 + half * 4;
          const attn_f32x4_t l4 = *(const attn_lds_f32x4_t*)(stats + qoff * 4);
          const attn_f32x4_t d4 = *(const attn_lds_f32x4_t*)(stats + 256 + qoff * 4);
          float p[4], ds[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int query = q0 + qoff + i;
            const bool hidden = (a.causal && ki > query) || query >= a.q_len;
            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[4 * g + i], c, -l4[i]));
            p[i] = hidden ? 0.0f : e;
            ds[i] = hidden ? 0.0f : e * (acc_dp[4 * g + i] - d4[i]) * a.scale;
          }
          pf[qt][2 * g] = pack2<T>(p[0], p[1]);
          pf[qt][2 * g + 1] = pack2<T>(p[2], p[3]);
          dsf[qt][2 * g] = pack2<T>(ds[0], ds[1]);
          dsf[qt][2 * g + 1] = pack2<T>(ds[2], ds[3]);
        }
      }
      // dV^T += dout^T P and dK^T += Q^T dS over the 64 queries, k-step s = queries 16 s .. 16 s + 15
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        u32x4_t pb, dsb;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pb[e] = pf[s >> 1][4 * (s & 1) + e];
          dsb[e] = dsf[s >> 1][4 * (s & 1) + e];
        }
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          const u32x4_t dot_op = attn_tr_operand(do_tile + s * 16 * kAttnRow, tr_off[dt][0], tr_off[dt][1]);
          acc_dv[dt] = Mfma<T>::run(dot_op, pb, acc_dv[dt]);
          const u32x4_t qt_op = attn_tr_operand(q_tile + s * 16 * kAttnRow, tr_off[dt][0], tr_off[dt][1]);
          acc_dk[dt] = Mfma<T>::run(qt_op, dsb, acc_dk[dt]);
        }
      }
    }
    if (ki < a.kv_len) {
      store_row<T>(static_cast<T*>(a.dk) + b * a.dk_sb + h * a.dk_sh + static_cast<int64_t>(ki) * a.dk_st,
                   acc_dk, half);
      store_row<T>(static_cast<T*>(a.dv) + b * a.dv_sb + h * a.dv_sh + static_cast<int64_t>(ki) * a.dv_st,
                   acc_dv, half);
    }
  };
  run_kblock(unit);
  if (paired && unit != n_kb - 1 - unit) {
    __syncthreads();  // every wave is done with the ring of the first block
    run_kblock(n_kb - 1 - unit);
  }
#endif
}

}  // namespace tmb

extern "C" int64_t tmb_attention_bwd_workspace_bytes(int64_t batch, int64_t heads, int64_t q_len) {
  if (batch < 0 || heads < 0 || q_len < 0) return 0;
  return 2 * batch * heads * q_len * static_cast<int64_t>(sizeof(float));
}

extern "C" int tmb_attention_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q,
                                 const void* k, const void* v, const void* out, const void* lse,
                                 void* workspace, int64_t batch, int64_t heads, int64_t q_len,
                                 int64_t kv_len, int64_t head_dim, const int64_t* q_strides,
                                 const int64_t* k_strides, const int64_t* v_strides,
                                 const int64_t* out_strides, const int64_t* dout_strides,
                                 const int64_t* dq_strides, const int64_t* dk_strides,
                                 const int64_t* dv_strides, float scale, int causal, int dtype,
                                 void* stream) {
  using namespace tmb;
  if (batch < 0 || heads < 0 || q_len < 0 || kv_len < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (head_dim != 64) return TMB_ERR_UNSUPPORTED;
  if (!(scale == scale)) return TMB_ERR_INVALID_ARGUMENT;
  if (!(scale > 0.0f) || scale > 3.0e38f) return TMB_ERR_UNSUPPORTED;
  if (batch == 0 || heads == 0 || (q_len == 0 && kv_len == 0)) return TMB_OK;
  if (q_len == 0 || kv_len == 0) return TMB_ERR_UNSUPPORTED;  // zero gradients: left to the caller
  const int64_t* all[] = {q_strides, k_strides, v_strides, out_strides, dout_strides,
                          dq_strides, dk_strides, dv_strides};
  for (const int64_t* s : all)
    if (!s) return TMB_ERR_INVALID_ARGUMENT;
  if (!dq || !dk || !dv || !dout || !q || !k || !v || !out || !lse || !workspace)
    return TMB_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(lse) & 3) || (reinterpret_cast<uintptr_t>(workspace) & 15))
    return TMB_ERR_INVALID_ARGUMENT;
  if (batch * heads * ((q_len + kAttnBQ - 1) / kAttnBQ) >= (int64_t{1} << 31) ||
      batch * heads * ((kv_len + kAttnBQ - 1) / kAttnBQ) >= (int64_t{1} << 31) ||
      q_len >= (int64_t{1} << 30) || kv_len >= (int64_t{1} << 30))
    return TMB_ERR_UNSUPPORTED;
  // 16-byte loads of q/k/v/out/dout rows and 8-byte stores of gradient rows
  auto aligned = [](const void* p, const int64_t* s, int64_t mult, uintptr_t mask) {
    return (reinterpret_cast<uintptr_t>(p) & mask) == 0 && s[0] % mult == 0 && s[1] % mult == 0 &&
           s[2] % mult == 0 && s[0] >= 0 && s[1] >= 0 && s[2] >= 0;
  };
  if (!aligned(q, q_strides, 8, 15) || !aligned(k, k_strides, 8, 15) ||
      !aligned(v, v_strides, 8, 15) || !aligned(out, out_strides, 8, 15) ||
      !aligned(dout, dout_strides, 8, 15) || !aligned(dq, dq_strides, 4, 7) ||
      !aligned(dk, dk_strides, 4, 7) || !aligned(dv, dv_strides, 4, 7))
    return TMB_ERR_UNSUPPORTED;
  // streamed rows are addressed with 32-bit byte offsets from the (batch, head) base
  auto fits = [](int64_t len, int64_t stride) { return (len * stride + 64) * 2 < (int64_t{1} << 32); };
  if (!fits(kv_len, k_strides[2]) || !fits(kv_len, v_strides[2]) || !fits(q_len, q_strides[2]) ||
      !fits(q_len, dout_strides[2]) || q_len * 4 >= (int64_t{1} << 32))
    return TMB_ERR_UNSUPPORTED;
  float* delta = static_cast<float*>(workspace);
  AttnBwdArgs a{dq, dk, dv, dout, q, k, v, out, static_cast<const float*>(lse), delta,
                delta + batch * heads * q_len,
                q_strides[0], q_strides[1], q_strides[2],
                k_strides[0], k_strides[1], k_strides[2],
                v_strides[0], v_strides[1], v_strides[2],
                out_strides[0], out_strides[1], out_strides[2],
                dout_strides[0], dout_strides[1], dout_strides[2],
                dq_strides[0], dq_strides[1], dq_strides[2],
                dk_strides[0], dk_strides[1], dk_strides[2],
                dv_strides[0], dv_strides[1], dv_strides[2],
                static_cast<int>(heads), static_cast<int>(q_len), static_cast<int>(kv_len),
                scale, causal ? 1 : 0};
  auto units_of = [&](int64_t len) {
    const int64_t n = (len + kAttnBQ - 1) / kAttnBQ;
    return (causal && n > 1) ? (n + 1) / 2 : n;
  };
  const dim3 grid_q(static_cast<unsigned>(units_of(q_len) * batch * heads));
  const dim3 grid_k(static_cast<unsigned>(units_of(kv_len) * batch * heads));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == TMB_BF16) {
    attention_bwd_dq_kernel<bf16_t><<<grid_q, dim3(256), 0, s>>>(a);
    attention_bwd_dkv_kernel<bf16_t><<<grid_k, dim3(256), 0, s>>>(a);
  } else {
    attention_bwd_dq_kernel<f16_t><<<grid_q, dim3(256), 0, s>>>(a);
    attention_bwd_dkv_kernel<f16_t><<<grid_k, dim3(256), 0, s>>>(a);
  }
  return check_launch();
}
