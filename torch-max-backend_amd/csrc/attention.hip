// Fused attention forward for gfx950: out = softmax(scale * q k^T [+ causal mask]) v without the
// [batch, heads, q_len, kv_len] score tensor ever reaching memory.
//
// One workgroup = 128 queries of one (batch, head): 4 waves x 32 queries. Keys and values are
// walked in blocks of 64; a block's K and V rows (128 bytes each: head_dim 64 x 2 bytes) go
// global -> LDS with global_load_lds_dwordx4 into a ring of three buffers, the next two blocks
// in flight while the current one is multiplied (one block of lookahead leaves every iteration
// waiting for an L2 round trip). Per block and wave:
//   S^T = K_blk Q^T    v_mfma_f32_32x32x16 with the keys as rows: a lane then holds 32 scores of
//                      ONE query (column lane%32), so the row max / row sum of the softmax are
//                      in-lane reductions plus one exchange between lanes l and l^32;
//   online softmax     running max m and sum l per query, accumulator rescaled by exp(m - m');
//   O^T += V_blk^T P^T the exponentials, rounded to the storage type, are already laid out as
//                      the MFMA's B operand (k = keys, in the order the score registers hold
//                      them); V^T comes from ds_read_b64_tr_b16 in that same key order.
// Q stays in registers for the whole kernel (loaded once, straight from global memory).
//
// Arithmetic follows the reference's unfused chain (aten_functions.py:443-677 builds
// softmax(q k^T * scale + mask) v from the same pieces; eager twin aten_fast.py:5177-5285):
// fp32 scores, fp32 softmax statistics, probabilities rounded to the storage type before they
// multiply V. With round_like_unfused the scores and their scaled value are rounded to the
// storage type too, as a separate bmm and mul kernel would have stored them. The one
// difference that remains is that probabilities are rounded before, not after, the division by
// the row sum.
#include "attention_tiles.h"

namespace tmb {

struct AttnArgs {
  void* out;
  float* lse;  // may be null: [batch, heads, q_len] log-sum-exp of the scaled, masked scores
  const void* q;
  const void* k;
  const void* v;
  int64_t q_sb, q_sh, q_st;  // element strides: batch, head, token (head_dim is contiguous)
  int64_t k_sb, k_sh, k_st;
  int64_t v_sb, v_sh, v_st;
  int64_t o_sb, o_sh, o_st;
  int heads, q_len, kv_len;
  float scale;
  int causal;
  int round_like_unfused;
};

constexpr int kAttnBuf = 2 * kAttnTile;         // K + V

template <typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void attention_fwd_kernel(
    AttnArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(1024))) unsigned char lds[kAttnStages * kAttnBuf];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  // Under a causal mask a query block's cost grows with its index, so a workgroup takes two
  // query blocks of one (batch, head): block n-1-u and then block u, which together always walk
  // the same number of key blocks. Every workgroup then carries the same load, and the
  // workgroups of one (batch, head), which read the same K and V, are numbered onto one XCD.
  const int n_qb = (a.q_len + kAttnBQ - 1) / kAttnBQ;
  const bool paired = a.causal && n_qb > 1;
  const int units = paired ? (n_qb + 1) / 2 : n_qb;
  const int wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int bh = wg / units;
  const int unit = wg % units;
  const int b = bh / a.heads, h = bh % a.heads;
  auto run_qblock = [&](const int qb) {
  const int q0 = qb * kAttnBQ, qw0 = q0 + wave * 32;
  const int qi = qw0 + (lane & 31);
  const float neg_inf = -__builtin_inff();

  const T* qp = static_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh;
  const unsigned char* kp =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh);
  const unsigned char* vp =
      reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh);

  // Q as the B operand of S^T = K Q^T: column = query lane%32, k = head-dim 16s + 8*half + 0..7
  u32x4_t qf[4];
  {
    const int qrow = qi < a.q_len ? qi : a.q_len - 1;  // rows past the end are never stored
    const T* src = qp + static_cast<int64_t>(qrow) * a.q_st + 8 * half;
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = *reinterpret_cast<const u32x4_t*>(src + 16 * s);
  }

  int n_blocks = (a.kv_len + kAttnBKV - 1) / kAttnBKV;
  if (a.causal) {
    const int last_q = (q0 + kAttnBQ < a.q_len ? q0 + kAttnBQ : a.q_len) - 1;
    const int need = last_q / kAttnBKV + 1;  // keys 0..last_q
    n_blocks = n_blocks < need ? n_blocks : need;
  }

  // DMA plan: a 1 KiB load covers 8 rows; the wave issues loads 2w and 2w+1 of K and of V.
  // Lane -> (row inside the load, 16-byte slot); the source chunk is the slot un-swizzled.
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((attn_lds_u8*)lds));
  const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int ld_row = lane >> 3, ld_slot = lane & 7;
  auto dma16 = [](uint32_t m0, uint32_t voff, const unsigned char* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0), "v"(voff), "s"(sbase)
                 : "memory", "m0");
  };
  auto fetch_block = [&](int blk, uint32_t buf_off) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = (wave * 2 + j) * 8 + ld_row;  // key inside the block
      int key = blk * kAttnBKV + row;
      key = key < a.kv_len ? key : a.kv_len - 1;    // masked later; any valid row will do
      const int k_chunk = ld_slot ^ ((row >> 1) & 7);
      const int v_chunk = ld_slot ^ (((row >> 1) & 1) << 2);
      const uint32_t k_off = static_cast<uint32_t>((static_cast<int64_t>(key) * a.k_st + k_chunk * 8) * 2);
      const uint32_t v_off = static_cast<uint32_t>((static_cast<int64_t>(key) * a.v_st + v_chunk * 8) * 2);
      const uint32_t dst = lds_base + buf_off + (wave_s * 2 + j) * 1024;
      dma16(dst, k_off, kp);
      dma16(dst + kAttnTile, v_off, vp);
    }
  };

  // fragment addresses (bytes inside a buffer)
  int k_lane[4];  // K rows as the A operand: row = key lane%32, chunk 2s + half, swizzled
#pragma unroll
  for (int s = 0; s < 4; ++s)
    k_lane[s] = (lane & 31) * kAttnRow + (((2 * s + half) ^ (((lane & 31) >> 1) & 7)) << 4);
  int v_lane[2];  // V^T through the transposed read, per 32-wide head-dim tile
  {
    const int j16 = lane & 15, qq = j16 >> 2, nsub = (lane >> 4) & 1;
    const int key = 4 * half + qq;  // + 16s + 8r
#pragma unroll
    for (int dt = 0; dt < 2; ++dt) {
      const int d0 = dt * 32 + nsub * 16 + (j16 & 3) * 4;
      v_lane[dt] = kAttnTile + key * kAttnRow + ((((d0 >> 3) ^ (((qq >> 1) & 1) << 2))) << 4) +
                   (d0 & 7) * 2;
    }
  }

  f32x16_t acc_o[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc_o[dt][e] = 0.0f;
  float m_run = neg_inf, l_run = 0.0f;

  fetch_block(0, 0);
  if (n_blocks > 1) fetch_block(1, kAttnBuf);
  uint32_t buf_off = 0;                 // ring position of block `blk`
  uint32_t free_off = 2 * kAttnBuf;     // the buffer read two iterations ago
  for (int blk = 0; blk < n_blocks; ++blk) {
    // Each wave has 4 loads per block in flight; block blk+1 (if any) may stay outstanding.
    // Once every wave has block `blk`, the buffer of block blk-1 is free for block blk+2.
    if (blk + 1 < n_blocks) {
      __builtin_amdgcn_s_waitcnt(4 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(4) lgkmcnt(0)
    } else {
      __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(0) lgkmcnt(0)
    }
    __builtin_amdgcn_s_barrier();
    if (blk + 2 < n_blocks) fetch_block(blk + 2, free_off);
    const uint32_t cur_off = buf_off;
    free_off = buf_off;
    buf_off = buf_off + kAttnBuf == kAttnStages * kAttnBuf ? 0 : buf_off + kAttnBuf;

    const int kb = blk * kAttnBKV;
    if (a.causal && kb > qw0 + 31) continue;  // wave-uniform: every key lies above the diagonal
    attn_lds_u8* buf = (attn_lds_u8*)lds + cur_off;

    f32x16_t acc_s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_s[kt][e] = 0.0f;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4_t kf = *(const attn_lds_u32x4_t*)(buf + k_lane[s] + kt * 32 * kAttnRow);
        acc_s[kt] = Mfma<T>::run(kf, qf[s], acc_s[kt]);
      }
    }

    // scores of query qi: register r of tile kt is key kb + 32kt + 8(r/4) + 4*half + r%4.
    // The running maximum is kept on the unscaled scores (scale > 0 keeps the order) and the
    // scale rides in the exponent: exp(scale*(x - m)) = exp2(x*c - m*c), c = scale*log2(e),
    // one FMA and one v_exp_f32 per score. The exponential's error (a few 1e-6 relative from
    // the fp32 argument) disappears in the rounding of the probability to the storage type.
    const bool need_mask = (a.causal && kb + kAttnBKV - 1 > qw0) || kb + kAttnBKV > a.kv_len;
    // (the two optional passes are whole loops under one wave-uniform branch each: tested per
    // element they cost an exec-mask save/restore per score)
    if (a.round_like_unfused) {
      // what a bmm kernel and then a mul kernel would have stored; the scale is applied here,
      // so the exponent below uses log2(e) alone
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float x = to_f32(from_f32<T>(acc_s[kt][r]));
          acc_s[kt][r] = to_f32(from_f32<T>(x * a.scale));
        }
    }
    if (need_mask) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kb + kt * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
          const bool hidden = (a.causal && key > qi) || key >= a.kv_len;
          acc_s[kt][r] = hidden ? neg_inf : acc_s[kt][r];
        }
    }
    float m_blk = neg_inf;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) m_blk = fmaxf(m_blk, acc_s[kt][r]);
    m_blk = fmaxf(m_blk, other_half(m_blk, lane));
    const float m_new = fmaxf(m_run, m_blk);
    const float m_use = m_new == neg_inf ? 0.0f : m_new;  // nothing visible yet: keep exp finite
    const float c = a.round_like_unfused ? 1.4426950408889634f : a.scale * 1.4426950408889634f;
    const float mc = m_use * c;
    const float alpha = __builtin_amdgcn_exp2f(m_run * c - mc);  // m_run = -inf gives 0
    float l_blk = 0.0f;
    uint32_t pf[2][8];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[kt][r], c, -mc));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[kt][r + 1], c, -mc));
        l_blk += p0 + p1;
        pf[kt][r >> 1] = pack2<T>(p0, p1);
      }
    l_blk += other_half(l_blk, lane);
    l_run = l_run * alpha + l_blk;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_o[dt][e] *= alpha;

    // O^T += V^T P^T over the 64 keys: k-step s covers keys 16s..16s+15 in the order
    // (half, i) -> 16s + 8(i/4) + 4*half + i%4, which is how the score registers are ordered
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      u32x4_t pb;
#pragma unroll
      for (int e = 0; e < 4; ++e) pb[e] = pf[s >> 1][4 * (s & 1) + e];
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) {
        attn_lds_u8* src = buf + v_lane[dt] + s * 16 * kAttnRow;
        const attn_i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_i16x4_t*)src);
        const attn_i16x4_t hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_i16x4_t*)(src + 8 * kAttnRow));
        typedef short i16x8_t __attribute__((ext_vector_type(8)));
        const i16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        acc_o[dt] = Mfma<T>::run(__builtin_bit_cast(u32x4_t, both), pb, acc_o[dt]);
      }
    }
  }

  // out[b, qi, h, d]: register r of tile dt is d = 32dt + 8(r/4) + 4*half + r%4
  if (a.lse != nullptr && half == 0 && qi < a.q_len)
    a.lse[(static_cast<int64_t>(b) * a.heads + h) * a.q_len + qi] =
        m_run * (a.round_like_unfused ? 1.0f : a.scale) + logf(l_run);
  if (qi < a.q_len) {
    const float inv = 1.0f / l_run;
    T* dst = static_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + static_cast<int64_t>(qi) * a.o_st;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_t packed;
        packed[0] = pack2<T>(acc_o[dt][4 * g] * inv, acc_o[dt][4 * g + 1] * inv);
        packed[1] = pack2<T>(acc_o[dt][4 * g + 2] * inv, acc_o[dt][4 * g + 3] * inv);
        *reinterpret_cast<u32x2_t*>(dst + dt * 32 + g * 8 + half * 4) = packed;
      }
  }
  };
  run_qblock(n_qb - 1 - unit);
  if (paired && unit != n_qb - 1 - unit) {
    __syncthreads();  // every wave is done with the K/V ring of the first block
    run_qblock(unit);
  }
#endif
}

// ---------------------------------------------------------------------------
// Few queries per (batch, head): the decode step of a generation loop. One wave per query row;
// the work is reading K and V once, so there is no MFMA: D/8 lanes share a key (16 bytes of the
// row each), a wave covers 64/(D/8) keys per step with whole-row loads, every key group keeps its
// own running maximum, sum and output chunk (online softmax), and the groups are merged at the
// end. An optional boolean mask (broadcastable, True = takes part) and the top-left aligned
// causal rule are applied to the scores; a row without any key comes out as NaN, as in ATen.
// ---------------------------------------------------------------------------
struct AttnDecodeArgs {
  void* out;
  const void* q;
  const void* k;
  const void* v;
  const unsigned char* mask;      // may be null
  int64_t q_sb, q_sh, q_st;
  int64_t k_sb, k_sh, k_st;
  int64_t v_sb, v_sh, v_st;
  int64_t o_sb, o_sh, o_st;
  int64_t m_sb, m_sh, m_st, m_ss;  // mask element strides (0 where it broadcasts)
  int64_t rows;                    // batch * heads * q_len
  int heads, q_len, kv_len;
  float scale;
  int causal;
};

template <typename T, int D>
__global__ __launch_bounds__(256) void attention_decode_kernel(AttnDecodeArgs a) {
  constexpr int LPK = D / 8;        // lanes per key
  constexpr int KPI = kWave / LPK;  // keys per step of a wave
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;  // whole waves leave; no barriers below
  const int t = static_cast<int>(row % a.q_len);
  const int64_t bh = row / a.q_len;
  const int h = static_cast<int>(bh % a.heads);
  const int64_t b = bh / a.heads;
  const int sub = lane % LPK, kg = lane / LPK;

  const T* qrow = static_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh + t * a.q_st + sub * 8;
  const T* kbase = static_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh + sub * 8;
  const T* vbase = static_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh + sub * 8;
  const unsigned char* mrow =
      a.mask == nullptr ? nullptr : a.mask + b * a.m_sb + h * a.m_sh + t * a.m_st;

  const float c = a.scale * 1.44269504088896340736f;  // scores in the log2 domain
  float qf[8];
  {
    const Vec16<T> qv = load_vec16(qrow);
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] = to_f32(qv.v[e]) * c;
  }
  const float neg_inf = -__builtin_inff();
  float m = neg_inf, l = 0.0f, acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0f;

  const int last = a.causal ? (t < a.kv_len - 1 ? t : a.kv_len - 1) : a.kv_len - 1;
  for (int s0 = 0; s0 <= last; s0 += KPI) {
    const int s = s0 + kg;
    bool valid = s <= last;
    if (valid && mrow != nullptr) valid = mrow[s * a.m_ss] != 0;
    const int sr = s <= last ? s : last;  // a readable row for lanes without a key
    const Vec16<T> kv = load_vec16_stream(kbase + static_cast<int64_t>(sr) * a.k_st);
    const Vec16<T> vv = load_vec16_stream(vbase + static_cast<int64_t>(sr) * a.v_st);
    float x = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) x = __builtin_fmaf(qf[e], to_f32(kv.v[e]), x);
#pragma unroll
    for (int w = 1; w < LPK; w <<= 1) x += __shfl_xor(x, w, kWave);
    if (valid) {
      const float m_new = fmaxf(m, x);
      const float corr = __builtin_amdgcn_exp2f(m - m_new);  // 0 on the first key (m = -inf)
      const float p = __builtin_amdgcn_exp2f(x - m_new);
      l = l * corr + p;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = acc[e] * corr + p * to_f32(vv.v[e]);
      m = m_new;
    }
  }
  // merge the key groups (lanes with equal `sub`)
  float big = m;
#pragma unroll
  for (int w = LPK; w < kWave; w <<= 1) big = fmaxf(big, __shfl_xor(big, w, kWave));
  const float wgt = m == neg_inf ? 0.0f : __builtin_amdgcn_exp2f(m - big);
  l *= wgt;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] *= wgt;
#pragma unroll
  for (int w = LPK; w < kWave; w <<= 1) {
    l += __shfl_xor(l, w, kWave);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], w, kWave);
  }
  if (kg == 0) {
    float r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = acc[e] / l;  // 0/0 = NaN for a row without keys
    T* dst = static_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + t * a.o_st + sub * 8;
    store_converted<T, 8>(dst, r);
  }
}

}  // namespace tmb

extern "C" int tmb_attention_fwd(void* out, void* lse, const void* q, const void* k, const void* v,
                                 int64_t batch, int64_t heads, int64_t q_len, int64_t kv_len,
                                 int64_t head_dim, const int64_t* q_strides,
                                 const int64_t* k_strides, const int64_t* v_strides,
                                 const int64_t* out_strides, float scale, int causal,
                                 int round_like_unfused, int dtype, void* stream) {
  using namespace tmb;
  if (batch < 0 || heads < 0 || q_len < 0 || kv_len < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (head_dim != 64) return TMB_ERR_UNSUPPORTED;
  if (!(scale == scale)) return TMB_ERR_INVALID_ARGUMENT;
  if (!(scale > 0.0f) || scale > 3.0e38f) return TMB_ERR_UNSUPPORTED;  // the running maximum assumes it
  if (batch == 0 || heads == 0 || q_len == 0) return TMB_OK;
  if (kv_len == 0) return TMB_ERR_UNSUPPORTED;  // every row empty: left to the caller
  if (!out || !q || !k || !v || !q_strides || !k_strides || !v_strides || !out_strides)
    return TMB_ERR_INVALID_ARGUMENT;
  if (batch * heads * ((q_len + kAttnBQ - 1) / kAttnBQ) >= (int64_t{1} << 31) ||
      q_len >= (int64_t{1} << 30) || kv_len >= (int64_t{1} << 30))
    return TMB_ERR_UNSUPPORTED;
  // 16-byte loads of q/k/v rows and 8-byte stores of out rows
  auto aligned = [](const void* p, const int64_t* s, int64_t mult, uintptr_t mask) {
    return (reinterpret_cast<uintptr_t>(p) & mask) == 0 && s[0] % mult == 0 && s[1] % mult == 0 &&
           s[2] % mult == 0 && s[0] >= 0 && s[1] >= 0 && s[2] >= 0;
  };
  if (!aligned(q, q_strides, 8, 15) || !aligned(k, k_strides, 8, 15) ||
      !aligned(v, v_strides, 8, 15) || !aligned(out, out_strides, 4, 7))
    return TMB_ERR_UNSUPPORTED;
  // K and V rows are addressed with 32-bit byte offsets from the (batch, head) base
  if ((kv_len * k_strides[2] + 64) * 2 >= (int64_t{1} << 32) ||
      (kv_len * v_strides[2] + 64) * 2 >= (int64_t{1} << 32))
    return TMB_ERR_UNSUPPORTED;
  if (lse != nullptr && (reinterpret_cast<uintptr_t>(lse) & 3)) return TMB_ERR_INVALID_ARGUMENT;
  AttnArgs a{out, static_cast<float*>(lse), q, k, v,
             q_strides[0], q_strides[1], q_strides[2],
             k_strides[0], k_strides[1], k_strides[2],
             v_strides[0], v_strides[1], v_strides[2],
             out_strides[0], out_strides[1], out_strides[2],
             static_cast<int>(heads), static_cast<int>(q_len), static_cast<int>(kv_len),
             scale, causal ? 1 : 0, round_like_unfused ? 1 : 0};
  const int64_t n_qb = (q_len + kAttnBQ - 1) / kAttnBQ;
  const int64_t units = (causal && n_qb > 1) ? (n_qb + 1) / 2 : n_qb;  // query-block pairs when causal
  const dim3 grid(static_cast<unsigned>(units * batch * heads));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == TMB_BF16) {
    attention_fwd_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(a);
  } else {
    attention_fwd_kernel<f16_t><<<grid, dim3(256), 0, s>>>(a);
  }
  return check_launch();
}

extern "C" int tmb_attention_decode(void* out, const void* q, const void* k, const void* v,
                                    const void* mask, int64_t batch, int64_t heads, int64_t q_len,
                                    int64_t kv_len, int64_t head_dim, const int64_t* q_strides,
                                    const int64_t* k_strides, const int64_t* v_strides,
                                    const int64_t* out_strides, const int64_t* mask_strides,
                                    float scale, int causal, int dtype, void* stream) {
  using namespace tmb;
  if (batch < 0 || heads < 0 || q_len < 0 || kv_len < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (head_dim != 64 && head_dim != 128) return TMB_ERR_UNSUPPORTED;
  if (!(scale == scale)) return TMB_ERR_INVALID_ARGUMENT;
  if (batch == 0 || heads == 0 || q_len == 0) return TMB_OK;
  if (kv_len == 0) return TMB_ERR_UNSUPPORTED;
  if (!out || !q || !k || !v || !q_strides || !k_strides || !v_strides || !out_strides ||
      (mask != nullptr && !mask_strides))
    return TMB_ERR_INVALID_ARGUMENT;
  if (heads >= (int64_t{1} << 31) || q_len >= (int64_t{1} << 31) || kv_len >= (int64_t{1} << 31) ||
      batch * heads * q_len >= (int64_t{1} << 33))
    return TMB_ERR_UNSUPPORTED;
  auto aligned = [](const void* p, const int64_t* s) {
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && s[0] % 8 == 0 && s[1] % 8 == 0 &&
           s[2] % 8 == 0 && s[0] >= 0 && s[1] >= 0 && s[2] >= 0;
  };
  if (!aligned(q, q_strides) || !aligned(k, k_strides) || !aligned(v, v_strides) ||
      !aligned(out, out_strides))
    return TMB_ERR_UNSUPPORTED;
  if (mask != nullptr)
    for (int i = 0; i < 4; ++i)
      if (mask_strides[i] < 0) return TMB_ERR_UNSUPPORTED;
  AttnDecodeArgs a{out, q, k, v, static_cast<const unsigned char*>(mask),
                   q_strides[0], q_strides[1], q_strides[2],
                   k_strides[0], k_strides[1], k_strides[2],
                   v_strides[0], v_strides[1], v_strides[2],
                   out_strides[0], out_strides[1], out_strides[2],
                   mask ? mask_strides[0] : 0, mask ? mask_strides[1] : 0,
                   mask ? mask_strides[2] : 0, mask ? mask_strides[3] : 0,
                   batch * heads * q_len, static_cast<int>(heads), static_cast<int>(q_len),
                   static_cast<int>(kv_len), scale, causal ? 1 : 0};
  const dim3 grid(static_cast<unsigned>((a.rows + 3) / 4));
  hipStream_t s = static_cast<hipStream_t>(stream);
#define TMB_AD(T, D) attention_decode_kernel<T, D><<<grid, dim3(256), 0, s>>>(a)
  if (dtype == TMB_BF16) {
    if (head_dim == 64) TMB_AD(bf16_t, 64); else TMB_AD(bf16_t, 128);
  } else {
    if (head_dim == 64) TMB_AD(f16_t, 64); else TMB_AD(f16_t, 128);
  }
#undef TMB_AD
  return check_launch();
}
