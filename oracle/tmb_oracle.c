/* CPU oracle for the hot ATen ops — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library;
 * it is the checker the HIP kernels are compared with, never a fallback for them.
 *
 * Each function restates, in plain C, the arithmetic of one CPU kernel body of the reference
 * (paths relative to torch_mojo_backend/eager_kernels/):
 *   orc_gemm        matmul_ops.mojo:2671-2720  (_cpu_gemm_naive: sequential-k fp32 accumulate,
 *                                               bias added in fp32, one cast) and :2651-2657
 *   orc_softmax     nn_ops.mojo:428-455        (max, sum of exp(x-m), exp(x-m)/denom; fp32)
 *                   reduction_ops.mojo:874-895 (log-softmax: x - m - log(denom))
 *   orc_softmax_scaled nn_ops.mojo:413-493     (`_softmax_rows(scale, causal, q_len)`: x*scale, causal
 *                                               rows keep j <= r % q_len, the rest is zero)
 *   orc_attention   aten_functions.py:443-677  (scaled dot product attention as the reference builds
 *                                               it: matmul, *scale, causal mask, softmax, matmul;
 *                                               every stage stored in the tensor dtype)
 *   orc_attention_lse / orc_attention_backward
 *                   aten_fast.py:4050-4170 (the fused attention's float32 log-sum-exp output and
 *                   its backward: the kernel source is a vendored third-party Mojo port of
 *                   FlashAttention, so the oracle restates the published algorithm, Dao 2023
 *                   "FlashAttention-2" algorithm 2: P = exp(S - L), dV = P^T dO, dP = dO V^T,
 *                   dS = P o (dP - rowsum(dO o O)), dQ = dS K, dK = dS^T Q, S scaled; P and dS
 *                   are rounded to the tensor dtype before their products, sums are fp32)
 *   orc_layer_norm  nn_ops.mojo:299-326        (two-pass mean / centered variance, fp32) with the
 *                                               NaN-mean rule of normalization_forward_kernels.mojo:60-70
 *   orc_reduce      reduction_ops.mojo:161-194 (fp32 accumulator for floats, own type for ints,
 *                                               one cast) and nn_ops.mojo:981-1027 (mean)
 *   orc_argmax      nn_ops.mojo:1488-1505      (sequential strict-greater scan from index 0).
 *                   Deviation, on purpose: a NaN counts as the maximum (first NaN wins), which
 *                   is what ATen does and what the reference's tests compare with; the
 *                   reference's scan only keeps a NaN that sits at index 0.
 *   orc_gelu        activation_forward_kernels.mojo:22-56 (fp32 inside, one cast)
 *   orc_gelu_backward       activation_backward_ops.mojo:50-73 (`_exact_grad`, `_tanh_grad`)
 *   orc_gather_rows         nn_ops.mojo:1153-1176 (`_gather0`: out[i] = table[idx[i / row_len] *
 *                           row_len + i % row_len]); out-of-range indices read the nearest row
 *   orc_softmax_backward    ../aten_functions.py:788-833 (grad - exp(out) * sum(grad)) and its
 *                           softmax twin out * (grad - sum(grad * out))
 *   orc_nll_log_softmax_backward  loss_ops.mojo:234-311 (dense NLL gradient) followed by
 *                           orc_softmax_backward's log form
 *   orc_layer_norm_backward aten_fast.py:2797-2913 (LayerNormBackwardF32: grad_input from the
 *                           saved mean / rstd, grad_weight = sum dy*xhat, grad_bias = sum dy)
 *
 * Pinning: tests/test_oracle_pins.py checks every function against float64 closed forms,
 * brute-force Python loops on tiny inputs, mathematical invariants and PyTorch CPU eager (the
 * comparison the reference's own tests make, torch_mojo_backend/testing.py:186-229), and against
 * the fixtures under tests/golden/. The low-order bits of Modular MAX's CPU kernels (a
 * third-party dependency that is not part of the reference tree) are not observable here, so
 * bit-level parity with MAX is "parity unpinned"; parity is pinned at assert_close tolerances.
 *
 * dtype codes match include/tmb_hip.h: 0 f32, 1 f16, 2 bf16, 3 i64, 4 i32.
 * Rows are processed in parallel with OpenMP when compiled with -fopenmp.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2, ORC_I64 = 3, ORC_I32 = 4 };
enum { ORC_SUM = 0, ORC_MEAN = 1, ORC_AMAX = 2 };
enum { ORC_EPI_NONE = 0, ORC_EPI_GELU_TANH = 1, ORC_EPI_GELU_ERF = 2 };

static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }
static uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest even */
  return (uint16_t)(u >> 16);
}
static float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    float v = (float)man * 5.9604644775390625e-08f; /* 2^-24 */
    return sign ? -v : v;
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}
static uint16_t f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);            /* NaN */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);           /* >= 65536 -> inf (65520 rounds below) */
  if (a < 0x33000000u) return sign;                                   /* < 2^-25 -> 0 */
  int e = (int)(a >> 23) - 127;
  uint32_t man = (a & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (e < -14) { shift = 13 + (-14 - e); base = 0; }                  /* subnormal half */
  else { shift = 13; base = (uint32_t)(e + 15) << 10; man &= 0x7fffffu; }
  uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  uint32_t r = base + q; /* carry into the exponent is the right answer, incl. -> inf */
  return (uint16_t)(sign | r);
}

static float load_f(const void* p, int64_t i, int dtype) {
  switch (dtype) {
    case ORC_F32: return ((const float*)p)[i];
    case ORC_F16: return f16_to_f32(((const uint16_t*)p)[i]);
    default: return bf16_to_f32(((const uint16_t*)p)[i]);
  }
}
static void store_f(void* p, int64_t i, int dtype, float v) {
  switch (dtype) {
    case ORC_F32: ((float*)p)[i] = v; break;
    case ORC_F16: ((uint16_t*)p)[i] = f32_to_f16(v); break;
    default: ((uint16_t*)p)[i] = f32_to_bf16(v); break;
  }
}
static float round_to(float v, int dtype) {
  if (dtype == ORC_F16) return f16_to_f32(f32_to_f16(v));
  if (dtype == ORC_BF16) return bf16_to_f32(f32_to_bf16(v));
  return v;
}

static float gelu_tanh(float x) {
  const float k = 0.7978845608028654f;
  return 0.5f * x * (1.0f + tanhf(k * (x + 0.044715f * x * x * x)));
}
static float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }

/* C[b] = epi(op(A[b]) op(B[b]) + bias). The GELU epilogue acts on the value already rounded to
 * the storage dtype, i.e. exactly what an unfused addmm followed by gelu produces. */
/* epilogue = ORC_EPI_* | ORC_EPI_ROUND_LIKE_UNFUSED. The value is formed in fp32 from the
 * accumulator to the one cast (matmul_ops.mojo:2651-2657: "forming A@B + bias in fp32 and casting
 * to the output dtype exactly once"), also through a GELU and a residual add that a caller fuses
 * into the product; with the flag it is rounded to `dtype` wherever a separate kernel would have
 * stored it (after the bias, after the GELU). `residual` ([batch][m][n], pitch ldr, type
 * residual_dtype) may be NULL; `out_dtype` is the type of c. */
enum { ORC_EPI_ROUND_LIKE_UNFUSED = 0x100 };

int orc_gemm_residual(void* c, const void* a, const void* b, const void* bias, const void* residual,
                      int64_t batch, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                      int64_t ldc, int64_t ldr, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                      int64_t stride_r, int trans_a, int trans_b, int dtype, int residual_dtype,
                      int out_dtype, int epilogue_flags) {
  if (dtype != ORC_F32 && dtype != ORC_F16 && dtype != ORC_BF16) return -2;
  const int epilogue = epilogue_flags & 0xff;
  const int twice = (epilogue_flags & ORC_EPI_ROUND_LIKE_UNFUSED) != 0;
  const int64_t sa_m = trans_a ? 1 : lda, sa_k = trans_a ? lda : 1;
  const int64_t sb_k = trans_b ? 1 : ldb, sb_n = trans_b ? ldb : 1;
  const int64_t total_rows = batch * m;
#pragma omp parallel for schedule(static)
  for (int64_t row = 0; row < total_rows; ++row) {
    const int64_t bz = row / m, i = row % m;
    for (int64_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (int64_t kk = 0; kk < k; ++kk) {
        acc += load_f(a, bz * stride_a + i * sa_m + kk * sa_k, dtype) *
               load_f(b, bz * stride_b + kk * sb_k + j * sb_n, dtype);
      }
      if (bias) acc += load_f(bias, j, dtype);
      if (epilogue != ORC_EPI_NONE) {
        if (twice) acc = round_to(acc, dtype);
        acc = epilogue == ORC_EPI_GELU_TANH ? gelu_tanh(acc) : gelu_erf(acc);
      }
      if (residual) {
        if (twice) acc = round_to(acc, dtype);
        acc += load_f(residual, bz * stride_r + i * ldr + j, residual_dtype);
      }
      store_f(c, bz * stride_c + i * ldc + j, out_dtype, acc);
    }
  }
  return 0;
}

int orc_gemm(void* c, const void* a, const void* b, const void* bias, int64_t batch, int64_t m,
             int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
             int64_t stride_b, int64_t stride_c, int trans_a, int trans_b, int dtype,
             int epilogue) {
  return orc_gemm_residual(c, a, b, bias, 0, batch, m, n, k, lda, ldb, ldc, 0, stride_a, stride_b,
                           stride_c, 0, trans_a, trans_b, dtype, dtype, dtype, epilogue);
}

int orc_softmax(void* out, const void* in, int64_t rows, int64_t cols, int in_dtype,
                int out_dtype, int log_mode) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * cols;
    float m = -INFINITY;
    for (int64_t j = 0; j < cols; ++j) {
      float x = load_f(in, base + j, in_dtype);
      if (x > m) m = x;
      if (x != x) m = x; /* a NaN anywhere poisons the row, as it does through exp/sum */
    }
    float denom = 0.0f;
    for (int64_t j = 0; j < cols; ++j) denom += expf(load_f(in, base + j, in_dtype) - m);
    if (log_mode) {
      const float lg = logf(denom);
      for (int64_t j = 0; j < cols; ++j)
        store_f(out, base + j, out_dtype, load_f(in, base + j, in_dtype) - m - lg);
    } else {
      for (int64_t j = 0; j < cols; ++j)
        store_f(out, base + j, out_dtype, expf(load_f(in, base + j, in_dtype) - m) / denom);
    }
  }
  return 0;
}

/* Attention softmax: y = softmax_j(x*scale) over the columns j <= r % q_len (all columns when
 * q_len == 0); masked columns give 0. round_scaled rounds x*scale to the storage type first
 * (the value a separate mul would have stored). */
int orc_softmax_scaled(void* out, const void* in, int64_t rows, int64_t cols, int dtype,
                       float scale, int round_scaled, int64_t q_len) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * cols;
    const int64_t last = q_len > 0 ? r % q_len : cols - 1;
    float m = -INFINITY;
    for (int64_t j = 0; j <= last && j < cols; ++j) {
      float x = load_f(in, base + j, dtype) * scale;
      if (round_scaled) { store_f(out, base + j, dtype, x); x = load_f(out, base + j, dtype); }
      if (x > m) m = x;
      if (x != x) m = x;
    }
    float denom = 0.0f;
    for (int64_t j = 0; j <= last && j < cols; ++j) {
      float x = load_f(in, base + j, dtype) * scale;
      if (round_scaled) { store_f(out, base + j, dtype, x); x = load_f(out, base + j, dtype); }
      denom += expf(x - m);
    }
    for (int64_t j = 0; j < cols; ++j) {
      float y = 0.0f;
      if (j <= last) {
        float x = load_f(in, base + j, dtype) * scale;
        if (round_scaled) { store_f(out, base + j, dtype, x); x = load_f(out, base + j, dtype); }
        y = expf(x - m) / denom;
      }
      store_f(out, base + j, dtype, y);
    }
  }
  return 0;
}

/* out[b,t,h,:] = softmax_j(scale * q[b,h,t,:].k[b,h,j,:]) v[b,h,j,:]; q,k,v are [B,H,T|S,D]
 * contiguous, out is [B,T,H,D] contiguous. Stage by stage like the unfused graph: scores
 * (fp32 accumulate) rounded to dtype, times scale rounded to dtype, masked, softmax in fp32
 * rounded to dtype, second product accumulated in fp32 and rounded once. */
int orc_attention(void* out, const void* q, const void* k, const void* v, int64_t B, int64_t H,
                  int64_t T, int64_t S, int64_t D, float scale, int causal, int dtype) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t bh = 0; bh < B * H; ++bh) {
    for (int64_t t = 0; t < T; ++t) {
      const int64_t b = bh / H, h = bh % H;
      float sc[S > 0 ? S : 1];
      const int64_t last = causal ? (t < S - 1 ? t : S - 1) : S - 1;
      float m = -INFINITY;
      for (int64_t j = 0; j <= last; ++j) {
        float acc = 0.0f;
        for (int64_t d = 0; d < D; ++d)
          acc += load_f(q, (bh * T + t) * D + d, dtype) * load_f(k, (bh * S + j) * D + d, dtype);
        acc = round_to(acc, dtype);
        acc = round_to(acc * scale, dtype);
        sc[j] = acc;
        if (acc > m) m = acc;
        if (acc != acc) m = acc;
      }
      float denom = 0.0f;
      for (int64_t j = 0; j <= last; ++j) denom += expf(sc[j] - m);
      for (int64_t j = 0; j <= last; ++j) sc[j] = round_to(expf(sc[j] - m) / denom, dtype);
      for (int64_t d = 0; d < D; ++d) {
        float acc = 0.0f;
        for (int64_t j = 0; j <= last; ++j) acc += sc[j] * load_f(v, (bh * S + j) * D + d, dtype);
        store_f(out, ((b * T + t) * H + h) * D + d, dtype, acc);
      }
    }
  }
  return 0;
}

/* lse[b,h,t] = log sum_j exp(scale * q[b,h,t,:].k[b,h,j,:]) over the keys the causal rule keeps
 * (j <= t), in double from the stored operands, rounded to float once. */
int orc_attention_lse(float* lse, const void* q, const void* k, int64_t B, int64_t H, int64_t T,
                      int64_t S, int64_t D, float scale, int causal, int dtype) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t bh = 0; bh < B * H; ++bh) {
    for (int64_t t = 0; t < T; ++t) {
      const int64_t last = causal ? (t < S - 1 ? t : S - 1) : S - 1;
      double sc[S > 0 ? S : 1];
      double m = -INFINITY;
      for (int64_t j = 0; j <= last; ++j) {
        double acc = 0.0;
        for (int64_t d = 0; d < D; ++d)
          acc += (double)load_f(q, (bh * T + t) * D + d, dtype) * (double)load_f(k, (bh * S + j) * D + d, dtype);
        sc[j] = acc * (double)scale;
        if (sc[j] > m) m = sc[j];
      }
      double denom = 0.0;
      for (int64_t j = 0; j <= last; ++j) denom += exp(sc[j] - m);
      lse[bh * T + t] = (float)(m + log(denom));
    }
  }
  return 0;
}

/* Gradients of orc_attention's output with respect to q, k, v. q, k, v, dq, dk, dv are
 * [B,H,T|S,D] contiguous; out and dout are [B,T,H,D] contiguous as orc_attention writes them; lse
 * is [B,H,T] float32. fp32 scores, P = exp(scale * s - lse) and dS = P * (dP - delta) * scale are
 * rounded to dtype before the products that consume them, every sum is fp32 and each result is
 * rounded once. */
int orc_attention_backward(void* dq, void* dk, void* dv, const void* dout, const void* q,
                           const void* k, const void* v, const void* out, const float* lse,
                           int64_t B, int64_t H, int64_t T, int64_t S, int64_t D, float scale,
                           int causal, int dtype) {
#pragma omp parallel for schedule(static)
  for (int64_t bh = 0; bh < B * H; ++bh) {
    const int64_t b = bh / H, h = bh % H;
    float* p = (float*)malloc(sizeof(float) * (size_t)(T * S > 0 ? T * S : 1));
    float* ds = (float*)malloc(sizeof(float) * (size_t)(T * S > 0 ? T * S : 1));
    for (int64_t t = 0; t < T; ++t) {
      const int64_t orow = ((b * T + t) * H + h) * D;
      float delta = 0.0f;
      for (int64_t d = 0; d < D; ++d) delta += load_f(dout, orow + d, dtype) * load_f(out, orow + d, dtype);
      for (int64_t j = 0; j < S; ++j) {
        const int hidden = causal && j > t;
        float s = 0.0f, dp = 0.0f;
        for (int64_t d = 0; d < D; ++d) {
          s += load_f(q, (bh * T + t) * D + d, dtype) * load_f(k, (bh * S + j) * D + d, dtype);
          dp += load_f(dout, orow + d, dtype) * load_f(v, (bh * S + j) * D + d, dtype);
        }
        const float pr = hidden ? 0.0f : expf(s * scale - lse[bh * T + t]);
        p[t * S + j] = round_to(pr, dtype);
        ds[t * S + j] = round_to(pr * (dp - delta) * scale, dtype);
      }
    }
    for (int64_t t = 0; t < T; ++t)
      for (int64_t d = 0; d < D; ++d) {
        float acc = 0.0f;
        for (int64_t j = 0; j < S; ++j) acc += ds[t * S + j] * load_f(k, (bh * S + j) * D + d, dtype);
        store_f(dq, (bh * T + t) * D + d, dtype, acc);
      }
    for (int64_t j = 0; j < S; ++j)
      for (int64_t d = 0; d < D; ++d) {
        float acc_k = 0.0f, acc_v = 0.0f;
        for (int64_t t = 0; t < T; ++t) {
          acc_k += ds[t * S + j] * load_f(q, (bh * T + t) * D + d, dtype);
          acc_v += p[t * S + j] * load_f(dout, ((b * T + t) * H + h) * D + d, dtype);
        }
        store_f(dk, (bh * S + j) * D + d, dtype, acc_k);
        store_f(dv, (bh * S + j) * D + d, dtype, acc_v);
      }
    free(p);
    free(ds);
  }
  return 0;
}

/* `in_dtype` is the type of x, `dtype` the type of out, gamma and beta (the same, or a 16-bit
 * output normalised from an fp32 row: the statistics and the normalisation then use the fp32
 * values and the result is cast once). */
int orc_layer_norm_mixed(void* out, float* mean_out, float* rstd_out, const void* x,
                         const void* gamma, const void* beta, int64_t rows, int64_t cols,
                         double eps, int in_dtype, int dtype) {
  const float e = (float)eps;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * cols;
    float total = 0.0f;
    for (int64_t j = 0; j < cols; ++j) total += load_f(x, base + j, in_dtype);
    float mean = total / (float)cols;
    float var_sum = 0.0f;
    for (int64_t j = 0; j < cols; ++j) {
      const float d = load_f(x, base + j, in_dtype) - mean;
      var_sum += d * d;
    }
    const float var = var_sum / (float)cols;
    const float rstd = 1.0f / sqrtf(var + e);
    for (int64_t j = 0; j < cols; ++j) {
      float y = (load_f(x, base + j, in_dtype) - mean) * rstd;
      if (gamma) y *= load_f(gamma, j, dtype);
      if (beta) y += load_f(beta, j, dtype);
      store_f(out, base + j, dtype, y);
    }
    if (var != var) mean = var;
    if (mean_out) mean_out[r] = mean;
    if (rstd_out) rstd_out[r] = rstd;
  }
  return 0;
}

int orc_layer_norm(void* out, float* mean_out, float* rstd_out, const void* x, const void* gamma,
                   const void* beta, int64_t rows, int64_t cols, double eps, int dtype) {
  return orc_layer_norm_mixed(out, mean_out, rstd_out, x, gamma, beta, rows, cols, eps, dtype, dtype);
}

int orc_reduce(void* out, const void* in, int64_t rows, int64_t cols, int op, int dtype) {
  if (dtype == ORC_I64 || dtype == ORC_I32) {
    if (op == ORC_MEAN) return -2;
    if (dtype == ORC_I32 && op == ORC_SUM) return -2;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
      if (dtype == ORC_I64) {
        const int64_t* p = (const int64_t*)in + r * cols;
        int64_t acc = op == ORC_SUM ? 0 : INT64_MIN;
        for (int64_t j = 0; j < cols; ++j) acc = op == ORC_SUM ? acc + p[j] : (p[j] > acc ? p[j] : acc);
        ((int64_t*)out)[r] = acc;
      } else {
        const int32_t* p = (const int32_t*)in + r * cols;
        int32_t acc = INT32_MIN;
        for (int64_t j = 0; j < cols; ++j) acc = p[j] > acc ? p[j] : acc;
        ((int32_t*)out)[r] = acc;
      }
    }
    return 0;
  }
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * cols;
    float acc = op == ORC_AMAX ? -INFINITY : 0.0f;
    int saw_nan = 0;
    for (int64_t j = 0; j < cols; ++j) {
      const float x = load_f(in, base + j, dtype);
      if (op == ORC_AMAX) { if (x > acc) acc = x; if (x != x) saw_nan = 1; }
      else acc += x;
    }
    if (op == ORC_AMAX && saw_nan) acc = NAN;
    if (op == ORC_MEAN) acc = acc / (float)cols;
    store_f(out, r, dtype, acc);
  }
  return 0;
}

int orc_argmax(int64_t* out, const void* in, int64_t rows, int64_t cols, int dtype) {
  if (cols <= 0) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    int64_t best_idx = 0;
    if (dtype == ORC_I64) {
      const int64_t* p = (const int64_t*)in + r * cols;
      int64_t best = p[0];
      for (int64_t j = 1; j < cols; ++j) if (p[j] > best) { best = p[j]; best_idx = j; }
    } else if (dtype == ORC_I32) {
      const int32_t* p = (const int32_t*)in + r * cols;
      int32_t best = p[0];
      for (int64_t j = 1; j < cols; ++j) if (p[j] > best) { best = p[j]; best_idx = j; }
    } else {
      const int64_t base = r * cols;
      float best = load_f(in, base, dtype);
      for (int64_t j = 1; j < cols; ++j) {
        const float v = load_f(in, base + j, dtype);
        if (v > best || (v != v && best == best)) { best = v; best_idx = j; }
      }
    }
    out[r] = best_idx;
  }
  return 0;
}

int orc_gelu(void* out, const void* in, int64_t numel, int dtype, int approximate_tanh) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < numel; ++i) {
    const float x = load_f(in, i, dtype);
    store_f(out, i, dtype, approximate_tanh ? gelu_tanh(x) : gelu_erf(x));
  }
  return 0;
}

int orc_gelu_backward(void* out, const void* grad, const void* in, int64_t numel, int dtype,
                      int approximate_tanh) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < numel; ++i) {
    const float x = load_f(in, i, dtype), g = load_f(grad, i, dtype);
    float d;
    if (approximate_tanh) {
      const float beta = 0.7978845608028654f, kappa = 0.044715f;
      const float x2 = x * x;
      const float t = tanhf(beta * (x + kappa * (x2 * x)));
      d = 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * beta * (1.0f + 3.0f * kappa * x2);
    } else {
      const float cdf = 0.5f * (1.0f + erff(x * 0.7071067811865476f));
      const float pdf = 0.3989422804014327f * expf(-0.5f * (x * x));
      d = cdf + x * pdf;
    }
    store_f(out, i, dtype, g * d);
  }
  return 0;
}

int orc_softmax_backward(void* gin, const void* gout, const void* y, int64_t rows, int64_t cols,
                         int dtype, int log_mode) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * cols;
    float s = 0.0f;
    for (int64_t j = 0; j < cols; ++j) {
      const float g = load_f(gout, base + j, dtype);
      s += log_mode ? g : g * load_f(y, base + j, dtype);
    }
    for (int64_t j = 0; j < cols; ++j) {
      const float g = load_f(gout, base + j, dtype), o = load_f(y, base + j, dtype);
      store_f(gin, base + j, dtype, log_mode ? g - expf(o) * s : o * (g - s));
    }
  }
  return 0;
}

/* The dense gradient of the negative log-likelihood loss with respect to the log-probabilities
 * (loss_ops.mojo:234-311: scale = grad_output / total_weight for the mean, grad_output for the
 * sum, grad_output[row] without reduction; -scale at a row's target when that is a class and not
 * ignore_index, 0 elsewhere), stored in the tensor type, and the log-softmax backward of it
 * (orc_softmax_backward): what a cross-entropy loss sends back to the logits. reduction: 0 none,
 * 1 mean, 2 sum (ATen's codes). scratch: rows * cols elements of the tensor type. */
int orc_nll_log_softmax_backward(void* dx, const void* logp, const int64_t* target,
                                 const void* grad_out, const void* total_weight, int64_t rows,
                                 int64_t cols, int reduction, int64_t ignore_index, int dtype,
                                 void* scratch) {
  float scale = 0.0f;
  if (reduction == 1) scale = load_f(grad_out, 0, dtype) / load_f(total_weight, 0, dtype);
  else if (reduction == 2) scale = load_f(grad_out, 0, dtype);
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t t = target[r];
    const int valid = t != ignore_index && t >= 0 && t < cols;
    const float g = valid ? -(reduction == 0 ? load_f(grad_out, r, dtype) : scale) : 0.0f;
    for (int64_t j = 0; j < cols; ++j) store_f(scratch, r * cols + j, dtype, (valid && j == t) ? g : 0.0f);
  }
  return orc_softmax_backward(dx, scratch, logp, rows, cols, dtype, 1);
}

/* dgamma / dbeta are accumulated row after row in fp32 (any of the outputs may be NULL). */
int orc_layer_norm_backward(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x,
                            const float* mean, const float* rstd, const void* gamma,
                            int64_t rows, int64_t cols, int dtype, float* scratch) {
  float* sg = scratch;          /* [cols] */
  float* sb = scratch + cols;   /* [cols] */
  for (int64_t j = 0; j < 2 * cols; ++j) scratch[j] = 0.0f;
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * cols;
    const float mu = mean[r], rs = rstd[r];
    float s1 = 0.0f, s2 = 0.0f;
    for (int64_t j = 0; j < cols; ++j) {
      const float d = load_f(dy, base + j, dtype);
      const float gd = d * (gamma ? load_f(gamma, j, dtype) : 1.0f);
      const float xh = (load_f(x, base + j, dtype) - mu) * rs;
      s1 += gd;
      s2 += gd * xh;
      sg[j] += d * xh;
      sb[j] += d;
    }
    if (dx) {
      const float m1 = s1 / (float)cols, m2 = s2 / (float)cols;
      for (int64_t j = 0; j < cols; ++j) {
        const float gd = load_f(dy, base + j, dtype) * (gamma ? load_f(gamma, j, dtype) : 1.0f);
        const float xh = (load_f(x, base + j, dtype) - mu) * rs;
        store_f(dx, base + j, dtype, rs * (gd - m1 - xh * m2));
      }
    }
  }
  for (int64_t j = 0; j < cols; ++j) {
    if (dgamma) store_f(dgamma, j, dtype, sg[j]);
    if (dbeta) store_f(dbeta, j, dtype, sb[j]);
  }
  return 0;
}

/* Round-trip helpers so the tests can pin the 16-bit conversions themselves. */
void orc_convert_to_f32(float* out, const void* in, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; ++i) out[i] = load_f(in, i, dtype);
}
void orc_convert_from_f32(void* out, const float* in, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; ++i) store_f(out, i, dtype, in[i]);
}

/* Element-by-element restatement of the reference's flat gather loop. index_dtype: 3 = int64,
 * 4 = int32. */
int orc_gather_rows(void* out, const void* table, const void* indices, int64_t num_indices,
                    int64_t row_len, int64_t num_rows, int dtype, int index_dtype) {
  const int64_t esize = dtype == 0 ? 4 : 2;
  if (num_rows <= 0 && num_indices * row_len > 0) return 1;
  for (int64_t i = 0; i < num_indices * row_len; ++i) {
    int64_t row = index_dtype == 3 ? ((const int64_t*)indices)[i / row_len]
                                   : (int64_t)((const int32_t*)indices)[i / row_len];
    if (row < 0) row = 0;
    if (row >= num_rows) row = num_rows - 1;
    const char* src = (const char*)table + (row * row_len + i % row_len) * esize;
    char* dst = (char*)out + i * esize;
    for (int64_t b = 0; b < esize; ++b) dst[b] = src[b];
  }
  return 0;
}
