/*
 * oa_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the optimizer hot path of tascj/offload_adam,
 * written from the reference's formulas.  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may call it; nothing the library ships routes
 * through it.  Build: see oracle/Makefile (gcc, -ffp-contract=off, no
 * fast-math: every float operation below is one IEEE binary32 rounding).
 *
 * Each function cites the reference lines it follows (paths relative to the
 * reference repository root).
 *
 * What pins each function (tests/test_oracle_*.py):
 *   philox4x32_10          Random123 known-answer vectors
 *   triton_randint         the words of Triton 3.6.0's own tl.randint (run by its CPU
 *                          interpreter; tests/golden/triton_randint.npz)
 *   sr_round               exhaustive over the 65536 low halves x edge draws
 *   fp31 / custom split    brute force over all low halves, round-trip identities
 *   adam_*                 closed forms (t=1), fp64 evaluation (<= 1 ulp),
 *                          torch.optim.AdamW in fp32, an independent torch-eager
 *                          restatement (bit-exact)
 *   norm / clip            fp64 evaluation, closed forms
 *   codecs                 the reference tests' anchors (tests/test_int8.py:43-63,
 *                          tests/test_int4.py:52-69, tests/test_nf4.py:42-56,
 *                          tests/test_nvfp4.py:51-63,233-359,470-498), torch's own
 *                          float8_e4m3fn cast, an independent torch restatement, and
 *                          the outputs of the reference's own pure-torch quantisers
 *                          on its seed-0 test shapes, an outlier tensor and tie /
 *                          threshold-edge inputs (tests/golden/codec_fixtures.npz)
 * No function is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---------------------------------------------------------------- bits */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float oaref_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN -> quiet NaN keeping the sign */
uint16_t oaref_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* fp32 -> IEEE binary16 bits, round to nearest even */
uint16_t oaref_f32_to_f16(float f) {
  uint32_t u = f2u(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536 -> inf (65520 handled below) */
  if (a < 0x33000000u) return (uint16_t)sign;              /* < 2^-25 -> 0 */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t mant = (a & 0x7FFFFFu) | 0x800000u;
  uint32_t shift, half;
  if (e < -14) {
    shift = (uint32_t)(13 + (-14 - e)); /* subnormal target */
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)(e + 15) << 10) | ((mant >> 13) & 0x3FFu);
  uint32_t rem = mant & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
  return (uint16_t)(sign | q); /* a carry into the exponent (up to inf) is correct */
}

float oaref_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
  if (e == 0) return u2f(sign) + (sign ? -1.0f : 1.0f) * (float)m * 0x1p-24f;
  if (e == 31) return u2f(sign | 0x7F800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* --------------------------------------------------------------- Philox
 * Philox4x32-10 as evaluated by triton.language.random.philox_impl
 * (Triton 3.6.0, language/random.py:13-41), the generator behind
 * tl.randint at kernels/stochastic_rounding.py:77. */
void oaref_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t pb = (uint64_t)0xCD9E8D57u * c2;
    uint64_t pa = (uint64_t)0xD2511F53u * c0;
    uint32_t n0 = (uint32_t)(pb >> 32) ^ c1 ^ k0;
    uint32_t n2 = (uint32_t)(pa >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)pb;
    c3 = (uint32_t)pa;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* tl.randint(seed, offset) for int32 offsets (language/random.py:44-105):
 * counter (offset, 0, 0, 0), key (seed_lo, seed_hi), word 0. */
uint32_t oaref_triton_randint(uint64_t seed, int64_t offset) {
  uint32_t ctr[4] = {(uint32_t)offset, (uint32_t)((uint64_t)offset >> 32), 0, 0};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  oaref_philox4x32_10(ctr, key, out);
  return out[0];
}

/* 16 random bits of element i for each layout of the library
 * (0 = Triton-compatible, 1 = one Philox block per 8 elements). */
uint32_t oaref_rand16(uint64_t seed, int64_t i, int layout) {
  if (layout == 0) return oaref_triton_randint(seed, i) & 0xFFFFu;
  uint64_t j = (uint64_t)i >> 3;
  uint32_t ctr[4] = {(uint32_t)j, (uint32_t)(j >> 32), 1u, 0u};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  oaref_philox4x32_10(ctr, key, out);
  uint32_t e = (uint32_t)i & 7u;
  return (out[e >> 1] >> ((e & 1u) * 16u)) & 0xFFFFu;
}

/* _fp32_to_bf16_sr, kernels/stochastic_rounding.py:25-34 */
uint16_t oaref_sr_round(float x, uint32_t r16) {
  int32_t bits = (int32_t)f2u(x);
  int32_t frac = bits & 0xFFFF;
  uint32_t trunc = (uint32_t)bits & 0xFFFF0000u;
  uint32_t out = ((int32_t)r16 < frac) ? trunc + 0x10000u : trunc;
  return (uint16_t)(out >> 16);
}

/* ---------------------------------------------------- fp31 / custom split */

/* round_to_fp31, kernels/fp31_master.py:26-34 (arithmetic shifts on int32) */
uint32_t oaref_round_to_fp31(uint32_t x) {
  int32_t xi = (int32_t)x;
  int32_t last = xi & 1, second = (xi >> 1) & 1;
  int32_t t = (xi >> 1) + (last & second);
  return (uint32_t)t << 1;
}

/* decompose, kernels/fp31_master.py:37-45 */
void oaref_fp31_decompose(float x, uint16_t* p_bf16, int16_t* err) {
  uint32_t x31 = oaref_round_to_fp31(f2u(x));
  uint16_t b = oaref_f32_to_bf16(u2f(x31));
  int32_t e32 = (int32_t)(x31 - ((uint32_t)b << 16));
  *p_bf16 = b;
  *err = (int16_t)(e32 >> 1);
}

/* reconstruct, kernels/fp31_master.py:48-54 */
float oaref_fp31_reconstruct(uint16_t p_bf16, int16_t err) {
  return u2f(((uint32_t)p_bf16 << 16) + ((uint32_t)(int32_t)err << 1));
}

/* decompose, kernels/fp32_master_custom_rounding.py:33-43 */
void oaref_custom_decompose(float x, uint16_t* p_bf16, int16_t* err) {
  int32_t xi = (int32_t)f2u(x);
  uint16_t b = (uint16_t)((uint32_t)((int32_t)((uint32_t)xi + 0x8000u) >> 16) & 0xFFFFu);
  *p_bf16 = b;
  *err = (int16_t)(uint16_t)((f2u(x) - ((uint32_t)b << 16)) & 0xFFFFu);
}

/* reconstruct, kernels/fp32_master_custom_rounding.py:46-54; the stored error
 * is always applied (the int16 != 0x8000 guard on line 48 is always true). */
float oaref_custom_reconstruct(uint16_t p_bf16, int16_t err) {
  return u2f(((uint32_t)p_bf16 << 16) + (uint32_t)(int32_t)err);
}

/* ------------------------------------------------------------------ Adam
 * One element of the shared update, kernels/fp32_master.py:46-53 (identical in
 * the other three kernels).  All fp32; lr*wd and 1-beta_hat are fp32 scalar
 * operations inside the Triton kernel. */
static inline void adam_core(float* M, float g, float* m, float* v, float lr, float wd,
                             float b1h, float b2h, float eps, int decoupled) {
  float Mv = *M;
  if (decoupled) {
    float lr_wd = lr * wd;
    Mv = Mv - lr_wd * Mv;
  } else {
    g = g + wd * Mv;
  }
  float omb1 = 1.0f - b1h, omb2 = 1.0f - b2h;
  float mv = *m + omb1 * (g - *m);
  float gg = g * g;
  float vv = *v + omb2 * (gg - *v);
  float denom = sqrtf(vv) + eps;
  float num = lr * mv;
  Mv = Mv - num / denom;
  *M = Mv; *m = mv; *v = vv;
}

/* grad after the reference's separate grad.mul_(clip_coef) pass
 * (offload_adam.py:450-451): bf16 * bf16 scalar in fp32, rounded to bf16. */
static inline float clipped_grad(uint16_t g, const uint16_t* clip) {
  float gf = oaref_bf16_to_f32(g);
  if (!clip) return gf;
  return oaref_bf16_to_f32(oaref_f32_to_bf16(gf * oaref_bf16_to_f32(*clip)));
}

/* adam_step_fp32_master_kernel, kernels/fp32_master.py:19-59 */
void oaref_adam_fp32_master(uint16_t* p_out, const uint16_t* g, uint16_t* m, uint16_t* v,
                            float* master, int64_t n, float lr, float wd, float b1h,
                            float b2h, float eps, int decoupled, const uint16_t* clip) {
  for (int64_t i = 0; i < n; ++i) {
    float M = master[i], mf = oaref_bf16_to_f32(m[i]), vf = oaref_bf16_to_f32(v[i]);
    float gf = clipped_grad(g[i], clip);
    adam_core(&M, gf, &mf, &vf, lr, wd, b1h, b2h, eps, decoupled);
    p_out[i] = oaref_f32_to_bf16(M);
    m[i] = oaref_f32_to_bf16(mf);
    v[i] = oaref_f32_to_bf16(vf);
    master[i] = M;
  }
}

/* adam_step_stochastic_rounding_kernel, kernels/stochastic_rounding.py:37-79.
 * layout 0/1: bits from oaref_rand16(seed, i, layout); layout 2: rand16[i]. */
void oaref_adam_stochastic_rounding(uint16_t* p, const uint16_t* g, uint16_t* m,
                                    uint16_t* v, int64_t n, float lr, float wd, float b1h,
                                    float b2h, float eps, int decoupled, uint64_t seed,
                                    int layout, const uint16_t* rand16,
                                    const uint16_t* clip) {
  for (int64_t i = 0; i < n; ++i) {
    float M = oaref_bf16_to_f32(p[i]);
    float mf = oaref_bf16_to_f32(m[i]), vf = oaref_bf16_to_f32(v[i]);
    float gf = clipped_grad(g[i], clip);
    adam_core(&M, gf, &mf, &vf, lr, wd, b1h, b2h, eps, decoupled);
    m[i] = oaref_f32_to_bf16(mf);
    v[i] = oaref_f32_to_bf16(vf);
    uint32_t r = (layout == 2) ? rand16[i] : oaref_rand16(seed, i, layout);
    p[i] = oaref_sr_round(M, r);
  }
}

/* adam_step_fp31_master_kernel, kernels/fp31_master.py:57-100 */
void oaref_adam_fp31_master(uint16_t* p, const uint16_t* g, uint16_t* m, uint16_t* v,
                            int16_t* err, int64_t n, float lr, float wd, float b1h,
                            float b2h, float eps, int decoupled, const uint16_t* clip) {
  for (int64_t i = 0; i < n; ++i) {
    float M = oaref_fp31_reconstruct(p[i], err[i]);
    float mf = oaref_bf16_to_f32(m[i]), vf = oaref_bf16_to_f32(v[i]);
    float gf = clipped_grad(g[i], clip);
    adam_core(&M, gf, &mf, &vf, lr, wd, b1h, b2h, eps, decoupled);
    m[i] = oaref_f32_to_bf16(mf);
    v[i] = oaref_f32_to_bf16(vf);
    oaref_fp31_decompose(M, &p[i], &err[i]);
  }
}

/* adam_step_fp32_master_custom_rounding_kernel,
 * kernels/fp32_master_custom_rounding.py:57-100 */
void oaref_adam_custom_rounding(uint16_t* p, const uint16_t* g, uint16_t* m, uint16_t* v,
                                int16_t* err, int64_t n, float lr, float wd, float b1h,
                                float b2h, float eps, int decoupled,
                                const uint16_t* clip) {
  for (int64_t i = 0; i < n; ++i) {
    float M = oaref_custom_reconstruct(p[i], err[i]);
    float mf = oaref_bf16_to_f32(m[i]), vf = oaref_bf16_to_f32(v[i]);
    float gf = clipped_grad(g[i], clip);
    adam_core(&M, gf, &mf, &vf, lr, wd, b1h, b2h, eps, decoupled);
    m[i] = oaref_f32_to_bf16(mf);
    v[i] = oaref_f32_to_bf16(vf);
    oaref_custom_decompose(M, &p[i], &err[i]);
  }
}

/* ----------------------------------------------------------- norm / clip */

/* torch.norm(grad, 2.0) on a bf16 tensor (offload_adam.py:504-505, 531-532):
 * sqrt of the sum of squares, result in the input dtype.  Evaluated here in
 * double and rounded once to fp32 and then bf16; torch's fp32 accumulation
 * order is not specified, so callers compare within one bf16 ulp. */
uint16_t oaref_grad_norm_bf16(const uint16_t* g, int64_t n) {
  double s = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    double x = (double)oaref_bf16_to_f32(g[i]);
    s += x * x;
  }
  return oaref_f32_to_bf16((float)sqrt(s));
}

/* Sum of squares in double (for callers that need the unrounded value). */
double oaref_sumsq_f64(const uint16_t* g, int64_t n) {
  double s = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    double x = (double)oaref_bf16_to_f32(g[i]);
    s += x * x;
  }
  return s;
}

/* total = vector_norm(stack(norms), 2) in bf16 (offload_adam.py:560). */
uint16_t oaref_total_norm_bf16(const uint16_t* norms, int64_t n) {
  return oaref_grad_norm_bf16(norms, n);
}

/* clip_coef = clamp(max_norm / (total + 1e-6), max=1.0), offload_adam.py:561,
 * all on 0-dim bf16 tensors, each op computed in fp32 and rounded to bf16.
 * Python-scalar / Tensor is Tensor.__rtruediv__ = reciprocal() * scalar. */
uint16_t oaref_clip_coef_bf16(uint16_t total, float max_norm) {
  uint16_t t1 = oaref_f32_to_bf16(oaref_bf16_to_f32(total) + 1e-6f);
  uint16_t r = oaref_f32_to_bf16(1.0f / oaref_bf16_to_f32(t1));
  uint16_t c = oaref_f32_to_bf16(oaref_bf16_to_f32(r) * max_norm);
  float cf = oaref_bf16_to_f32(c);
  if (cf != cf) return c;
  return (cf > 1.0f) ? (uint16_t)0x3F80u : c;
}

/* ---------------------------------------------------------------- codecs
 * Inputs are fp32 (bf16/fp16 sources widen exactly).  `out_dtype`:
 * 0 = fp32, 1 = bf16, 2 = fp16; 16-bit results are returned as bit patterns
 * in a uint16_t buffer, fp32 results in a float buffer. */

static inline void store_out(void* out, int64_t idx, float val, int out_dtype) {
  if (out_dtype == 0) ((float*)out)[idx] = val;
  else if (out_dtype == 1) ((uint16_t*)out)[idx] = oaref_f32_to_bf16(val);
  else ((uint16_t*)out)[idx] = oaref_f32_to_f16(val);
}

/* quantize_int8_per_channel, qweight/int8.py:30-49.  scale_f32 receives the
 * unrounded fp32 scale (the reference casts it to the scale dtype afterwards). */
void oaref_quant_int8(const float* x, int64_t rows, int64_t cols, int8_t* q,
                      float* scale_f32) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float absmax = 0.0f;
    for (int64_t c = 0; c < cols; ++c) absmax = fmaxf(absmax, fabsf(xr[c]));
    float scale = absmax / 127.0f;
    float inv = 1.0f / fmaxf(scale, 1e-12f);
    for (int64_t c = 0; c < cols; ++c) {
      float t = rintf(xr[c] * inv);
      t = fminf(fmaxf(t, -128.0f), 127.0f);
      q[r * cols + c] = (int8_t)t;
    }
    scale_f32[r] = scale;
  }
}

/* dequantize_int8_per_channel, qweight/int8.py:52-57: weight.to(dtype) * scale
 * computed in the scale dtype (fp32 product, one rounding).  `scale` holds the
 * stored scales widened to fp32. */
void oaref_dequant_int8(const int8_t* q, const float* scale, int64_t rows, int64_t cols,
                        void* out, int out_dtype) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c)
      store_out(out, r * cols + c, (float)q[r * cols + c] * scale[r], out_dtype);
}

/* quantize_int4_groupwise + pack_int4_gptq, qweight/int4.py:30-48, 61-92.
 * qweight: (cols/8, rows) int32, scale_f32: (cols/group, rows) fp32. */
void oaref_quant_int4(const float* x, int64_t rows, int64_t cols, int64_t group,
                      int32_t* qweight, float* scale_f32) {
  int64_t n_groups = cols / group;
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t gi = 0; gi < n_groups; ++gi) {
      const float* xg = x + r * cols + gi * group;
      float absmax = 0.0f;
      for (int64_t c = 0; c < group; ++c) absmax = fmaxf(absmax, fabsf(xg[c]));
      float scale = absmax / 8.0f;
      float inv = 1.0f / fmaxf(scale, 1e-12f);
      scale_f32[gi * rows + r] = scale;
      for (int64_t k = 0; k < group / 8; ++k) {
        uint32_t word = 0;
        for (int i = 0; i < 8; ++i) {
          float t = rintf(xg[k * 8 + i] * inv);
          t = fminf(fmaxf(t, -8.0f), 7.0f);
          uint32_t u = (uint32_t)((int32_t)t + 8);
          word |= u << (4 * i);
        }
        qweight[(gi * (group / 8) + k) * rows + r] = (int32_t)word;
      }
    }
  }
}

/* unpack_int4_gptq + scale multiply (qweight/int4.py:51-58 and the dequant used
 * by tests/test_int4.py:28-38): (u - 8) in the scale dtype times the scale. */
void oaref_dequant_int4(const int32_t* qweight, const float* scale, int64_t rows,
                        int64_t cols, int64_t group, void* out, int out_dtype) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      uint32_t word = (uint32_t)qweight[(c / 8) * rows + r];
      int32_t sv = (int32_t)((word >> (4 * (c % 8))) & 0xFu) - 8;
      store_out(out, r * cols + c, (float)sv * scale[(c / group) * rows + r], out_dtype);
    }
}

/* NF4_LUT, qweight/nf4.py:35-52 */
static const float NF4_LUT[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};

float oaref_nf4_lut(int i) { return NF4_LUT[i & 15]; }

/* quantize_nf4_blockwise + pack_nf4, qweight/nf4.py:74-83, 102-135.
 * packed: (rows, cols/2) bytes, even column in the high nibble;
 * absmax: rows * (cols/block) fp32. */
void oaref_quant_nf4(const float* x, int64_t rows, int64_t cols, int64_t block,
                     uint8_t* packed, float* absmax_out) {
  int64_t n_groups = cols / block;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t gi = 0; gi < n_groups; ++gi) {
      const float* xg = x + r * cols + gi * block;
      float absmax = 0.0f;
      for (int64_t c = 0; c < block; ++c) absmax = fmaxf(absmax, fabsf(xg[c]));
      float inv = 1.0f / fmaxf(absmax, 1e-12f);
      absmax_out[r * n_groups + gi] = absmax;
      for (int64_t c = 0; c < block; c += 2) {
        uint8_t code[2];
        for (int h = 0; h < 2; ++h) {
          float nv = xg[c + h] * inv;
          int best = 0;
          float bd = INFINITY;
          for (int i = 0; i < 16; ++i) {
            float d = fabsf(nv - NF4_LUT[i]);
            if (d < bd) { bd = d; best = i; }
          }
          code[h] = (uint8_t)best;
        }
        packed[r * (cols / 2) + (gi * block + c) / 2] = (uint8_t)((code[0] << 4) | code[1]);
      }
    }
}

/* fp32 LUT gather times fp32 absmax, cast at the end: the computation of
 * _dequant_nf4_kernel (qweight/nf4.py:160-220) and of the reference check in
 * tests/test_nf4.py:104-112. */
void oaref_dequant_nf4(const uint8_t* packed, const float* absmax, int64_t rows,
                       int64_t cols, int64_t block, void* out, int out_dtype) {
  int64_t n_groups = cols / block;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      uint8_t b = packed[r * (cols / 2) + c / 2];
      int code = (c & 1) ? (b & 0xF) : (b >> 4);
      store_out(out, r * cols + c, NF4_LUT[code] * absmax[r * n_groups + c / block],
                out_dtype);
    }
}

/* FP4_E2M1_LUT, qweight/nvfp4.py:34-51 */
static const float FP4_LUT[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                  -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

float oaref_fp4_lut(int i) { return FP4_LUT[i & 15]; }

/* fp32 -> float8_e4m3fn bits as torch's cast does (round to nearest even,
 * subnormals down to 2^-9, no infinity, anything that rounds beyond 448 -> NaN
 * 0x7F).  The NVFP4 path only feeds it values in [0, 448]. */
uint8_t oaref_f32_to_e4m3fn(float f) {
  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7FFFFFFFu;
  if (a >= 0x43F00000u) return (uint8_t)(sign | 0x7Fu); /* >= 480, inf, NaN */
  if (a < 0x3C800000u) {
    /* below 2^-6: subnormal grid of 2^-9; RNE via the magic-number add */
    float mag = u2f(a);
    float t = mag * 512.0f; /* exact */
    float q = rintf(t);
    return (uint8_t)(sign | (uint8_t)q); /* q == 8 encodes 2^-6, the first normal */
  }
  uint32_t mant_odd = (a >> 20) & 1u;
  a += ((uint32_t)(7 - 127) << 23) + 0x7FFFFu; /* rebias exponent, round */
  a += mant_odd;
  return (uint8_t)(sign | (uint8_t)(a >> 20));
}

/* float8_e4m3fn bits -> fp32 (_fp8_e4m3_bits_to_fp32, qweight/nvfp4.py:216-238) */
float oaref_e4m3fn_to_f32(uint8_t b) {
  uint32_t sign = ((uint32_t)b & 0x80u) << 24;
  uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
  if (e == 0xFu && m == 7u) return u2f(sign | 0x7FC00000u);
  if (e == 0) return u2f(sign | f2u((float)m * (1.0f / 512.0f)));
  return u2f(sign | ((e + 120u) << 23) | (m << 20));
}

/* _quantize_fp4_e2m1_rne, qweight/nvfp4.py:100-130 */
uint8_t oaref_fp4_e2m1_code(float x) {
  float ax = fabsf(x);
  uint8_t code = 0;
  if (ax > 0.25f) code = 1;
  if (ax >= 0.75f) code = 2;
  if (ax > 1.25f) code = 3;
  if (ax >= 1.75f) code = 4;
  if (ax > 2.5f) code = 5;
  if (ax >= 3.5f) code = 6;
  if (ax > 5.0f) code = 7;
  return (uint8_t)(code | ((f2u(x) >> 31) << 3));
}

/* tensor amax -> global scale, qweight/nvfp4.py:150-151 */
float oaref_nvfp4_global_scale(const float* x, int64_t n) {
  float amax = 0.0f;
  for (int64_t i = 0; i < n; ++i) amax = fmaxf(amax, fabsf(x[i]));
  amax = fmaxf(amax, 1e-12f);
  return amax / (448.0f * 6.0f);
}

/* quantize_nvfp4_blockwise + pack_fp4, qweight/nvfp4.py:72-81, 133-173.
 * packed: (rows, cols/2), even column in the LOW nibble; scale8: (rows, cols/16)
 * e4m3fn bits; returns the fp32 global scale. */
float oaref_quant_nvfp4(const float* x, int64_t rows, int64_t cols, uint8_t* packed,
                        uint8_t* scale8) {
  const int64_t B = 16;
  int64_t n_groups = cols / B;
  float gs = oaref_nvfp4_global_scale(x, rows * cols);
  float inv_global = 1.0f / gs;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t gi = 0; gi < n_groups; ++gi) {
      const float* xg = x + r * cols + gi * B;
      float amax = 0.0f;
      for (int64_t c = 0; c < B; ++c) amax = fmaxf(amax, fabsf(xg[c]));
      amax = fmaxf(amax, 1e-12f);
      float bs32 = amax / 6.0f;
      uint8_t s8 = oaref_f32_to_e4m3fn(bs32 * inv_global);
      scale8[r * n_groups + gi] = s8;
      float eff = oaref_e4m3fn_to_f32(s8) * gs;
      float inv_eff = 1.0f / fmaxf(eff, 1e-12f);
      for (int64_t c = 0; c < B; c += 2) {
        uint8_t lo = oaref_fp4_e2m1_code(xg[c] * inv_eff);
        uint8_t hi = oaref_fp4_e2m1_code(xg[c + 1] * inv_eff);
        packed[r * (cols / 2) + (gi * B + c) / 2] = (uint8_t)((hi << 4) | lo);
      }
    }
  return gs;
}

/* dequantize_nvfp4_blockwise, qweight/nvfp4.py:176-191 */
void oaref_dequant_nvfp4(const uint8_t* packed, const uint8_t* scale8, float gs,
                         int64_t rows, int64_t cols, void* out, int out_dtype) {
  const int64_t B = 16;
  int64_t n_groups = cols / B;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      uint8_t b = packed[r * (cols / 2) + c / 2];
      int code = (c & 1) ? (b >> 4) : (b & 0xF);
      float eff = oaref_e4m3fn_to_f32(scale8[r * n_groups + c / B]) * gs;
      store_out(out, r * cols + c, FP4_LUT[code] * eff, out_dtype);
    }
}

/* ------------------------------------------------ array forms for the tests */

void oaref_sr_round_array(const float* x, const uint16_t* r, int64_t n, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = oaref_sr_round(x[i], r[i]);
}

/* which: 0 = fp31 split, 1 = custom-rounding split */
void oaref_split_array(const uint32_t* xbits, int64_t n, int which, uint16_t* p_out,
                       int16_t* err_out, uint32_t* recon_bits) {
  for (int64_t i = 0; i < n; ++i) {
    float x = u2f(xbits[i]);
    if (which == 0) {
      oaref_fp31_decompose(x, &p_out[i], &err_out[i]);
      recon_bits[i] = f2u(oaref_fp31_reconstruct(p_out[i], err_out[i]));
    } else {
      oaref_custom_decompose(x, &p_out[i], &err_out[i]);
      recon_bits[i] = f2u(oaref_custom_reconstruct(p_out[i], err_out[i]));
    }
  }
}

/* kind: 0 = bf16, 1 = fp16 (uint16 out), 2 = e4m3fn (uint8 out) */
void oaref_narrow_array(const float* x, int64_t n, int kind, void* out) {
  for (int64_t i = 0; i < n; ++i) {
    if (kind == 0) ((uint16_t*)out)[i] = oaref_f32_to_bf16(x[i]);
    else if (kind == 1) ((uint16_t*)out)[i] = oaref_f32_to_f16(x[i]);
    else ((uint8_t*)out)[i] = oaref_f32_to_e4m3fn(x[i]);
  }
}

void oaref_fp4_code_array(const float* x, int64_t n, uint8_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = oaref_fp4_e2m1_code(x[i]);
}

void oaref_rand16_array(uint64_t seed, int64_t start, int64_t n, int layout, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = (uint16_t)oaref_rand16(seed, start + i, layout);
}
