// Pieces shared by the fused attention kernels (forward and backward): 64-row x 128-byte tiles of
// head_dim-64 rows in LDS, filled by global_load_lds_dwordx4 and read either as MFMA operand rows
// (16-byte reads) or transposed (ds_read_b64_tr_b16).
#pragma once
#include "gemm_mfma.h"

namespace tmb {

typedef __attribute__((address_space(3))) unsigned char attn_lds_u8;
typedef __attribute__((address_space(3))) u32x4_t attn_lds_u32x4_t;
typedef short attn_i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) attn_i16x4_t attn_lds_i16x4_t;
typedef float attn_f32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) attn_f32x4_t attn_lds_f32x4_t;

constexpr int kAttnBQ = 128;     // queries (forward, dQ) or keys (dK/dV) per workgroup
constexpr int kAttnBKV = 64;     // rows of one streamed tile
constexpr int kAttnRow = 128;    // bytes of one tile row (head_dim 64)
constexpr int kAttnTile = kAttnBKV * kAttnRow;  // 8 KiB
constexpr int kAttnStages = 3;                  // LDS ring: one block in use, two in flight

// the value lane l^32 holds
__device__ __forceinline__ float other_half(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2,
                                                                __builtin_bit_cast(int, x)));
}

// One wave-wide direct-to-LDS load: lane i's 16 bytes at sbase + voff land at m0 + 16 i.
__device__ __forceinline__ void attn_dma16(uint32_t m0, uint32_t voff, const unsigned char* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(m0), "v"(voff), "s"(sbase)
               : "memory", "m0");
}
// The same with 4 bytes per lane: lane i's dword lands at m0 + 4 i.
__device__ __forceinline__ void attn_dma4(uint32_t m0, uint32_t voff, const unsigned char* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(m0), "v"(voff), "s"(sbase)
               : "memory", "m0");
}

// Swizzle of a tile that is read both ways: 16-byte chunk c of row r sits at chunk c ^ swz(r).
// Operand-row reads touch 16 consecutive rows at one chunk: rows of one parity (the parity picks
// the half of the 64 banks) must land on 8 different chunks, so swz is a bijection of (r >> 1) & 7.
// Transposed reads touch rows r and r + 2 at the same four chunks in one pass: bit 1 of the row
// goes to bit 2 of the chunk so that they part.
__device__ __forceinline__ int attn_swz(int row) {
  return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}

// Byte offset, inside a tile, of the 16 bytes lane `lane` reads as its share of operand-row
// `lane % 32` at k-step s (head-dim 16 s + 8 (lane / 32) ...); add 32 * kAttnRow for rows 32..63.
__device__ __forceinline__ int attn_row_read(int lane, int s) {
  const int row = lane & 31, half = lane >> 5;
  return row * kAttnRow + (((2 * s + half) ^ attn_swz(row)) << 4);
}

// Byte offset, inside a tile, of lane `lane`'s 8 bytes of the transposed read that yields the A
// operand [head-dim 32 dt .. 32 dt + 31] x [tile rows 8 r + 4 (lane / 32) + 0..3]; add
// 16 s * kAttnRow for the rows of k-step s. The four rows come out in the order the MFMA result
// registers hold them, so a result tile can be the B operand of this product unchanged.
__device__ __forceinline__ int attn_tr_read(int lane, int dt, int r) {
  const int half = lane >> 5, j16 = lane & 15, qq = j16 >> 2, nsub = (lane >> 4) & 1;
  const int row = 8 * r + 4 * half + qq;
  const int d0 = dt * 32 + nsub * 16 + (j16 & 3) * 4;
  return row * kAttnRow + (((d0 >> 3) ^ attn_swz(row)) << 4) + (d0 & 7) * 2;
}

// A operand of one k-step from two transposed reads (rows +0..3 and +8..11 of the step)
__device__ __forceinline__ u32x4_t attn_tr_operand(attn_lds_u8* tile, int off_lo, int off_hi) {
  const attn_i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_i16x4_t*)(tile + off_lo));
  const attn_i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_i16x4_t*)(tile + off_hi));
  typedef short i16x8_t __attribute__((ext_vector_type(8)));
  const i16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(u32x4_t, both);
}

// Workgroups are dealt to the 8 XCDs round-robin by their linear id, and each XCD has its own L2.
// This renumbering gives every XCD one contiguous run of logical ids, so that the workgroups
// that share operands (the query blocks of one (batch, head) all walk the same K and V; the key
// blocks of one head all walk the same Q and dout) sit on one XCD at about the same time and the
// operands come from memory once instead of once per XCD.
__device__ __forceinline__ int xcd_contiguous_id(int id, int n) {
  const int q = n >> 3, r = n & 7;
  const int xcd = id & 7, slot = id >> 3;
  return (xcd < r ? xcd * (q + 1) : r * (q + 1) + (xcd - r) * q) + slot;
}

template <typename T>
__device__ __forceinline__ void unpack2(uint32_t v, float& a, float& b) {
  a = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(v)));
  b = to_f32(__builtin_bit_cast(T, static_cast<unsigned short>(v >> 16)));
}

}  // namespace tmb
