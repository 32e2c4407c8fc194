// Library identity, status strings, the standalone GELU and the bandwidth-yardstick copy kernel.
#include "tmb_common.h"

namespace tmb {

// Grid-stride over 16-byte vectors; scalar tail. `in`/`out` must be 16-byte aligned for the
// vector body (the launcher checks and otherwise runs everything through the scalar loop).
template <typename T, bool TANH>
__global__ __launch_bounds__(256) void gelu_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                   int64_t numel, int64_t nvec) {
  constexpr int EPV = Vec16<T>::N;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool stream = numel * static_cast<int64_t>(2 * sizeof(T)) >= kStreamStoreBytes;
  for (int64_t i = tid; i < nvec; i += stride) {
    const Vec16<T> v = load_vec16_stream(in + i * EPV);  // read once
    float y[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float x = to_f32(v.v[e]);
      y[e] = TANH ? gelu_tanh_f32(x) : gelu_erf_f32(x);
    }
    store_converted_hinted<T, EPV>(out + i * EPV, y, stream);
  }
  for (int64_t i = nvec * EPV + tid; i < numel; i += stride) {
    const float x = to_f32(in[i]);
    out[i] = from_f32<T>(TANH ? gelu_tanh_f32(x) : gelu_erf_f32(x));
  }
}

template <typename T>
static int launch_gelu(void* out_, const void* in_, int64_t numel, int tanh_mode, hipStream_t s) {
  T* out = static_cast<T*>(out_);
  const T* in = static_cast<const T*>(in_);
  constexpr int EPV = Vec16<T>::N;
  const int64_t nvec = (aligned16(in) && aligned16(out)) ? numel / EPV : 0;
  int64_t work = nvec > 0 ? nvec : numel;
  // one 16-byte vector per thread, consecutive blocks on consecutive memory: measured faster on
  // this GPU than a capped grid whose threads stride through the tensor
  int64_t blocks = (work + 255) / 256;
  if (blocks > (int64_t{1} << 30)) blocks = int64_t{1} << 30;
  if (blocks < 1) blocks = 1;
  if (tanh_mode)
    gelu_kernel<T, true><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(out, in, numel, nvec);
  else
    gelu_kernel<T, false><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(out, in, numel, nvec);
  return check_launch();
}

// Each block moves one contiguous 16 KiB piece (4 x 16 bytes per thread, non-temporal both
// ways): on this GPU that is the fastest plain copy (6.1-6.2 TB/s; a persistent grid-stride
// loop over the same data reaches 4.5-5.7).
__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ out,
                                                   const uint4* __restrict__ in, size_t nvec,
                                                   unsigned char* __restrict__ out_tail,
                                                   const unsigned char* __restrict__ in_tail,
                                                   size_t tail) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4* src = reinterpret_cast<const u32x4*>(in);
  u32x4* dst = reinterpret_cast<u32x4*>(out);
  const size_t base = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
  u32x4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (base + u * 256 < nvec) v[u] = __builtin_nontemporal_load(src + base + u * 256);
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (base + u * 256 < nvec) __builtin_nontemporal_store(v[u], dst + base + u * 256);
  if (blockIdx.x == 0 && threadIdx.x < tail) out_tail[threadIdx.x] = in_tail[threadIdx.x];
}

// out[r, :] = a[r, :] followed by b[r, :] for contiguous a [rows, a_units] and b [rows, b_units]
// of UNIT-sized pieces: the append of a key/value cache (a long row and a short one) in one
// launch. One thread moves four pieces of the output, 256 apart.
template <typename UNIT, typename IDX>
__global__ __launch_bounds__(256) void cat2_rows_kernel(UNIT* __restrict__ out,
                                                        const UNIT* __restrict__ a,
                                                        const UNIT* __restrict__ b, IDX total,
                                                        IDX a_units, IDX b_units) {
  const IDX out_units = a_units + b_units;
  const IDX base = static_cast<IDX>(blockIdx.x) * 1024 + threadIdx.x;
  UNIT v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const IDX i = base + u * 256;
    if (i < total) {
      const IDX row = i / out_units, c = i - row * out_units;
      v[u] = c < a_units ? a[row * a_units + c] : b[row * b_units + (c - a_units)];
    }
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const IDX i = base + u * 256;
    if (i < total) out[i] = v[u];
  }
}

template <typename UNIT>
int launch_cat2(void* out, const void* a, const void* b, int64_t rows, int64_t a_bytes,
                int64_t b_bytes, hipStream_t s) {
  const int64_t au = a_bytes / static_cast<int64_t>(sizeof(UNIT));
  const int64_t bu = b_bytes / static_cast<int64_t>(sizeof(UNIT));
  const int64_t total = rows * (au + bu);
  const int64_t blocks = (total + 1023) / 1024;
  if (blocks >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(blocks));
  if (total + 1024 < (int64_t{1} << 32)) {
    cat2_rows_kernel<UNIT, uint32_t><<<grid, dim3(256), 0, s>>>(
        static_cast<UNIT*>(out), static_cast<const UNIT*>(a), static_cast<const UNIT*>(b),
        static_cast<uint32_t>(total), static_cast<uint32_t>(au), static_cast<uint32_t>(bu));
  } else {
    cat2_rows_kernel<UNIT, uint64_t><<<grid, dim3(256), 0, s>>>(
        static_cast<UNIT*>(out), static_cast<const UNIT*>(a), static_cast<const UNIT*>(b),
        static_cast<uint64_t>(total), static_cast<uint64_t>(au), static_cast<uint64_t>(bu));
  }
  return check_launch();
}

// out[r, :] = in[r, :row_units] followed by zeros up to the output pitch, for rows whose source
// pitch or start is only element-aligned (UNIT = the element: 2 or 4 bytes): what the matrix-core
// kernels need when an operand's rows are not whole 16-byte vectors (a 50257-wide vocabulary as
// the contraction or the transposed dimension). One thread writes one aligned 16-byte vector of
// the output from one (possibly unaligned) 16-byte load; global memory takes unaligned vector
// accesses on this target.
template <typename UNIT, typename IDX>
__global__ __launch_bounds__(256) void pad_rows_kernel(uint4* __restrict__ out,
                                                       const UNIT* __restrict__ in, IDX total,
                                                       IDX out_vecs, IDX row_units,
                                                       int64_t in_pitch_units) {
  constexpr int PER = 16 / static_cast<int>(sizeof(UNIT));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef u32x4 __attribute__((aligned(2))) u32x4_unaligned;  // element alignment is all the source has
  const IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const IDX row = i / out_vecs, v = i - row * out_vecs;
  const IDX first = v * PER;
  const UNIT* src = in + static_cast<int64_t>(row) * in_pitch_units + first;
  u32x4 val = {0u, 0u, 0u, 0u};
  if (first + PER <= row_units) {
    val = *reinterpret_cast<const u32x4_unaligned*>(src);
  } else if (first < row_units) {
    UNIT piece[PER];
#pragma unroll
    for (int e = 0; e < PER; ++e) piece[e] = first + e < row_units ? src[e] : UNIT{0};
    __builtin_memcpy(&val, piece, 16);
  }
  __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(out) + i);
}

template <typename UNIT>
int launch_pad_rows(void* out, const void* in, int64_t rows, int64_t row_units,
                    int64_t in_pitch_units, int64_t out_pitch_units, hipStream_t s) {
  constexpr int PER = 16 / static_cast<int>(sizeof(UNIT));
  const int64_t out_vecs = out_pitch_units / PER;
  const int64_t total = rows * out_vecs;
  const int64_t blocks = (total + 255) / 256;
  if (blocks >= (int64_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(blocks));
  if (total < (int64_t{1} << 32) && row_units < (int64_t{1} << 32)) {
    pad_rows_kernel<UNIT, uint32_t><<<grid, dim3(256), 0, s>>>(
        static_cast<uint4*>(out), static_cast<const UNIT*>(in), static_cast<uint32_t>(total),
        static_cast<uint32_t>(out_vecs), static_cast<uint32_t>(row_units), in_pitch_units);
  } else {
    pad_rows_kernel<UNIT, uint64_t><<<grid, dim3(256), 0, s>>>(
        static_cast<uint4*>(out), static_cast<const UNIT*>(in), static_cast<uint64_t>(total),
        static_cast<uint64_t>(out_vecs), static_cast<uint64_t>(row_units), in_pitch_units);
  }
  return check_launch();
}

}  // namespace tmb

extern "C" int tmb_pad_rows(void* out, const void* in, int64_t rows, int64_t row_len,
                            int64_t in_pitch, int64_t out_pitch, int itemsize, void* stream) {
  if (rows < 0 || row_len < 0 || in_pitch < 0 || out_pitch < row_len) return TMB_ERR_INVALID_ARGUMENT;
  if (itemsize != 2 && itemsize != 4) return TMB_ERR_UNSUPPORTED;
  if (rows == 0 || out_pitch == 0) return TMB_OK;
  if (!out || (row_len && !in)) return TMB_ERR_INVALID_ARGUMENT;
  if ((out_pitch * itemsize) % 16 != 0 || !tmb::aligned16(out) ||
      (reinterpret_cast<uintptr_t>(in) % static_cast<uintptr_t>(itemsize)) != 0)
    return TMB_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return itemsize == 2
             ? tmb::launch_pad_rows<uint16_t>(out, in, rows, row_len, in_pitch, out_pitch, s)
             : tmb::launch_pad_rows<uint32_t>(out, in, rows, row_len, in_pitch, out_pitch, s);
}

extern "C" int tmb_cat2_rows(void* out, const void* a, const void* b, int64_t rows,
                             int64_t a_row_bytes, int64_t b_row_bytes, void* stream) {
  if (rows < 0 || a_row_bytes < 0 || b_row_bytes < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (rows == 0 || a_row_bytes + b_row_bytes == 0) return TMB_OK;
  if (!out || (a_row_bytes && !a) || (b_row_bytes && !b)) return TMB_ERR_INVALID_ARGUMENT;
  if (rows >= (int64_t{1} << 40) || a_row_bytes >= (int64_t{1} << 40) ||
      b_row_bytes >= (int64_t{1} << 40))
    return TMB_ERR_UNSUPPORTED;
  // the widest piece that divides both row lengths and every base address
  const uintptr_t bits = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(a) |
                         reinterpret_cast<uintptr_t>(b) | static_cast<uintptr_t>(a_row_bytes) |
                         static_cast<uintptr_t>(b_row_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if ((bits & 15) == 0) return tmb::launch_cat2<uint4>(out, a, b, rows, a_row_bytes, b_row_bytes, s);
  if ((bits & 3) == 0) return tmb::launch_cat2<uint32_t>(out, a, b, rows, a_row_bytes, b_row_bytes, s);
  if ((bits & 1) == 0) return tmb::launch_cat2<uint16_t>(out, a, b, rows, a_row_bytes, b_row_bytes, s);
  return tmb::launch_cat2<uint8_t>(out, a, b, rows, a_row_bytes, b_row_bytes, s);
}

extern "C" int tmb_version(void) { return 1000; }

extern "C" const char* tmb_status_string(int code) {
  switch (code) {
    case TMB_OK: return "ok";
    case TMB_ERR_INVALID_ARGUMENT: return "invalid argument";
    case TMB_ERR_UNSUPPORTED: return "unsupported dtype/shape for this build";
    case TMB_ERR_WORKSPACE: return "workspace missing or too small";
    case TMB_ERR_SCRATCH_LIMIT: return "shape needs more scratch than the library's static array holds";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown status";
}

extern "C" int tmb_gelu(void* out, const void* in, int64_t numel, int dtype, int approximate_tanh,
                        void* stream) {
  if (numel < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (numel == 0) return TMB_OK;
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case TMB_F32: return tmb::launch_gelu<float>(out, in, numel, approximate_tanh, s);
    case TMB_F16: return tmb::launch_gelu<tmb::f16_t>(out, in, numel, approximate_tanh, s);
    case TMB_BF16: return tmb::launch_gelu<tmb::bf16_t>(out, in, numel, approximate_tanh, s);
    default: return TMB_ERR_UNSUPPORTED;
  }
}

namespace tmb {
// The read half of copy_kernel: every block reads one contiguous 16 KiB piece and keeps nothing.
// The loads stay alive through a store that only happens when the piece folds to one particular
// 32-bit pattern.
__global__ __launch_bounds__(256) void read_kernel(const uint4* __restrict__ in, size_t nvec,
                                                   uint32_t* __restrict__ sink) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4* src = reinterpret_cast<const u32x4*>(in);
  const size_t base = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
  u32x4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
    v[u] = __builtin_nontemporal_load(src + (base + u * 256 < nvec ? base + u * 256 : 0));
  const u32x4 x = v[0] ^ v[1] ^ v[2] ^ v[3];
  if ((x[0] ^ x[1] ^ x[2] ^ x[3]) == 0x9e3779b9u && x[0] == 0x7f4a7c15u) sink[0] = x[1];
}
}  // namespace tmb

extern "C" int tmb_read_bytes(const void* in, size_t bytes, void* sink, void* stream) {
  if (bytes < 16) return TMB_OK;
  if (in == nullptr || sink == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  if (!tmb::aligned16(in)) return TMB_ERR_UNSUPPORTED;
  const size_t nvec = bytes / 16;
  const size_t blocks = (nvec + 1023) / 1024;
  if (blocks >= (size_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  tmb::read_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream)>>>(static_cast<const uint4*>(in), nvec,
                                                         static_cast<uint32_t*>(sink));
  return tmb::check_launch();
}

extern "C" int tmb_copy_bytes(void* out, const void* in, size_t bytes, void* stream) {
  if (bytes == 0) return TMB_OK;
  if (out == nullptr || in == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  if (!tmb::aligned16(out) || !tmb::aligned16(in)) return TMB_ERR_UNSUPPORTED;
  const size_t nvec = bytes / 16, tail = bytes % 16;
  size_t blocks = (nvec + 1023) / 1024;
  if (blocks < 1) blocks = 1;
  if (blocks >= (size_t{1} << 31)) return TMB_ERR_UNSUPPORTED;
  tmb::copy_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream)>>>(
      static_cast<uint4*>(out), static_cast<const uint4*>(in), nvec,
      static_cast<unsigned char*>(out) + nvec * 16,
      static_cast<const unsigned char*>(in) + nvec * 16, tail);
  return tmb::check_launch();
}

namespace tmb {

// out[i, :] = table[indices[i], :]: 16-byte chunks when a row is whole chunks and everything is
// aligned, single elements otherwise. An index outside [0, num_rows) reads row 0 or the last row
// instead (the reference's kernel and PyTorch's leave that case undefined / trap; a stray read
// must not fault the device).
template <typename IDX, typename CHUNK>
__global__ __launch_bounds__(256) void gather_rows_kernel(CHUNK* __restrict__ out,
                                                          const CHUNK* __restrict__ table,
                                                          const IDX* __restrict__ indices,
                                                          int64_t num_indices, int64_t chunks_per_row,
                                                          int64_t num_rows) {
  const int64_t total = num_indices * chunks_per_row;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t r = i / chunks_per_row, c = i - r * chunks_per_row;
    int64_t row = static_cast<int64_t>(indices[r]);
    row = row < 0 ? 0 : (row >= num_rows ? num_rows - 1 : row);
    out[i] = table[row * chunks_per_row + c];
  }
}

template <typename IDX>
static int launch_gather_rows(void* out, const void* table, const void* indices,
                              int64_t num_indices, int64_t row_bytes, int64_t num_rows,
                              hipStream_t stream) {
  const IDX* idx = static_cast<const IDX*>(indices);
  auto blocks_for = [](int64_t total) {
    int64_t b = (total + 255) / 256;
    return static_cast<unsigned>(b > 65536 * 4 ? 65536 * 4 : (b < 1 ? 1 : b));
  };
  if (row_bytes % 16 == 0 && aligned16(out) && aligned16(table)) {
    const int64_t cpr = row_bytes / 16;
    gather_rows_kernel<IDX, uint4><<<dim3(blocks_for(num_indices * cpr)), dim3(256), 0, stream>>>(
        static_cast<uint4*>(out), static_cast<const uint4*>(table), idx, num_indices, cpr, num_rows);
  } else if (row_bytes % 4 == 0) {
    const int64_t cpr = row_bytes / 4;
    gather_rows_kernel<IDX, uint32_t><<<dim3(blocks_for(num_indices * cpr)), dim3(256), 0, stream>>>(
        static_cast<uint32_t*>(out), static_cast<const uint32_t*>(table), idx, num_indices, cpr,
        num_rows);
  } else {
    const int64_t cpr = row_bytes / 2;  // 16-bit elements, odd row length
    gather_rows_kernel<IDX, uint16_t><<<dim3(blocks_for(num_indices * cpr)), dim3(256), 0, stream>>>(
        static_cast<uint16_t*>(out), static_cast<const uint16_t*>(table), idx, num_indices, cpr,
        num_rows);
  }
  return check_launch();
}

}  // namespace tmb

extern "C" int tmb_gather_rows(void* out, const void* table, const void* indices,
                               int64_t num_indices, int64_t row_len, int64_t num_rows, int dtype,
                               int index_dtype, void* stream) {
  if (num_indices < 0 || row_len < 0 || num_rows < 0) return TMB_ERR_INVALID_ARGUMENT;
  if (dtype != TMB_F32 && dtype != TMB_F16 && dtype != TMB_BF16) return TMB_ERR_UNSUPPORTED;
  if (index_dtype != TMB_I64 && index_dtype != TMB_I32) return TMB_ERR_UNSUPPORTED;
  if (num_indices == 0 || row_len == 0) return TMB_OK;
  if (num_rows == 0) return TMB_ERR_INVALID_ARGUMENT;  // nothing to read from
  if (out == nullptr || table == nullptr || indices == nullptr) return TMB_ERR_INVALID_ARGUMENT;
  const int64_t row_bytes = row_len * (dtype == TMB_F32 ? 4 : 2);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return index_dtype == TMB_I64
             ? tmb::launch_gather_rows<int64_t>(out, table, indices, num_indices, row_bytes, num_rows, s)
             : tmb::launch_gather_rows<int32_t>(out, table, indices, num_indices, row_bytes, num_rows, s);
}
