/*
 * Scalar C restatement of the quantised-linear arithmetic — TEST INFRASTRUCTURE ONLY.
 *
 * A second, independent statement of the same algorithms as oracle/nf4_oracle.py and
 * oracle/fake_quant_oracle.py, written with explicit integer emulation of bfloat16 rounding instead of
 * PyTorch's bf16 tensors, so that a mistake in either (a missing rounding step, a wrong nibble, a wrong
 * tie rule) shows up as a disagreement between the two.  Nothing shipped links against this file.
 *
 *   ref_nf4_quantize     to_nf4 / NF4Tensor.from_tensor        (torchao; called at
 *                        torchtune/modules/peft/lora.py:86, torchtune/modules/low_precision/nf4_linear.py:49)
 *   ref_nf4_dequantize   NF4Tensor.get_original_weight         (torchao; reached from
 *                        torchtune/modules/common_utils.py:57 and every linear_nf4 call)
 *   ref_fq_per_token     FakeQuantizer, int8 per-token asymmetric  (torchao; torchtune/modules/peft/lora.py:232,258)
 *   ref_fq_per_group     FakeQuantizer, int4 per-group symmetric   (torchao; torchtune/modules/peft/lora.py:245,259)
 *   ref_quantize_per_group  convert() to real int4 values       (torchao; recipes/quantize.py:92)
 *   ref_fq_per_group_uint4_asym  FakeQuantizer / convert of the weight-only "4w-qat" scheme
 *                        (torchao Int4WeightOnlyQATQuantizer; torchtune/training/quantization.py:27,125-127)
 *
 * Parity status: bit-level agreement with torchao is PARITY UNPINNED (torchao is not available and the
 * reference's tests hold no vectors for these functions); the restatement is pinned by the checks listed in
 * oracle/nf4_oracle.py.
 *
 * Build: make -C oracle   ->  oracle/_build/libttamd_oracle.so
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static const float NF4[16] = {-1.0f,
                              -0.6961928009986877f,
                              -0.5250730514526367f,
                              -0.39491748809814453f,
                              -0.28444138169288635f,
                              -0.18477343022823334f,
                              -0.09105003625154495f,
                              0.0f,
                              0.07958029955625534f,
                              0.16093020141124725f,
                              0.24611230194568634f,
                              0.33791524171829224f,
                              0.44070982933044434f,
                              0.5626170039176941f,
                              0.7229568362236023f,
                              1.0f};

static uint32_t bits_of(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  return u;
}
static float float_of(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

/* round an fp32 value to the nearest bfloat16 (ties to even); result returned as fp32 */
static float to_bf16(float f) {
  uint32_t u = bits_of(f);
  if (isnan(f)) return float_of((u | 0x00400000u) & 0xffff0000u);
  uint32_t keep = u & 0xffff0000u;
  uint32_t rest = u & 0x0000ffffu;
  if (rest > 0x8000u || (rest == 0x8000u && (keep & 0x00010000u))) keep += 0x00010000u;
  return float_of(keep);
}

/* "round in the tensor dtype" */
static float rd(float f, int is_bf16) { return is_bf16 ? to_bf16(f) : f; }

static float load_elem(const void* p, int64_t i, int is_bf16) {
  if (is_bf16) return float_of(((uint32_t)((const uint16_t*)p)[i]) << 16);
  return ((const float*)p)[i];
}
static void store_elem(void* p, int64_t i, float v, int is_bf16) {
  if (is_bf16)
    ((uint16_t*)p)[i] = (uint16_t)(bits_of(to_bf16(v)) >> 16);
  else
    ((float*)p)[i] = v;
}

/* max as torch.max defines it: NaN wins */
static float tmax(float a, float b) {
  if (isnan(a)) return a;
  if (isnan(b)) return b;
  return a > b ? a : b;
}

static int nearest_code(float scaled, int is_bf16) {
  /* first minimum of the dtype-rounded distances; an all-NaN row reports index 0 */
  int arg = 0;
  float best = fabsf(rd(scaled - rd(NF4[0], is_bf16), is_bf16));
  for (int j = 1; j < 16; ++j) {
    float d = fabsf(rd(scaled - rd(NF4[j], is_bf16), is_bf16));
    if (d < best) {
      best = d;
      arg = j;
    }
  }
  return arg;
}

/* absmax_out: caller-provided float[numel / block_size] scratch */
void ref_nf4_quantize(const void* w, int is_bf16, int64_t numel, int block_size, int scaler_block_size,
                      uint8_t* qdata, int8_t* qscalers, void* qfactor, void* scaler_mean, float* absmax_out) {
  const int64_t n_blocks = numel / block_size;
  const int64_t n_sb = n_blocks / scaler_block_size;
  double total = 0.0;
  for (int64_t b = 0; b < n_blocks; ++b) {
    float m = fabsf(load_elem(w, b * block_size, is_bf16));
    for (int i = 1; i < block_size; ++i) m = tmax(m, fabsf(load_elem(w, b * block_size + i, is_bf16)));
    absmax_out[b] = m;
    total += (double)m;
    for (int i = 0; i < block_size; i += 2) {
      int64_t e = b * block_size + i;
      int c0 = nearest_code(rd(load_elem(w, e, is_bf16) / m, is_bf16), is_bf16);
      int c1 = nearest_code(rd(load_elem(w, e + 1, is_bf16) / m, is_bf16), is_bf16);
      qdata[e / 2] = (uint8_t)((c0 << 4) | c1);
    }
  }
  const float mean = rd((float)(total / (double)n_blocks), is_bf16);
  store_elem(scaler_mean, 0, mean, is_bf16);
  for (int64_t s = 0; s < n_sb; ++s) {
    const float* a = absmax_out + s * scaler_block_size;
    float m2 = 0.0f;
    for (int i = 0; i < scaler_block_size; ++i) m2 = tmax(m2, fabsf(rd(a[i] - mean, is_bf16)));
    /* 256 / (2 * m2): Tensor.__rtruediv__ evaluates reciprocal() * 256, each rounded in dtype */
    const float twice = rd(2.0f * m2, is_bf16);
    const float factor = rd(rd(1.0f / twice, is_bf16) * 256.0f, is_bf16);
    store_elem(qfactor, s, factor, is_bf16);
    for (int i = 0; i < scaler_block_size; ++i) {
      float q = rintf(rd(rd(a[i] - mean, is_bf16) * factor, is_bf16));
      int qi;
      if (isnan(q))
        qi = 0;
      else if (q < -128.0f)
        qi = -128;
      else if (q > 127.0f)
        qi = 127;
      else
        qi = (int)q;
      qscalers[s * scaler_block_size + i] = (int8_t)qi;
    }
  }
}

void ref_nf4_dequantize(const uint8_t* qdata, const int8_t* qscalers, const void* qfactor, const void* scaler_mean,
                        int is_bf16, int64_t numel, int block_size, int scaler_block_size, void* out) {
  const float mean = load_elem(scaler_mean, 0, is_bf16);
  for (int64_t e = 0; e < numel; ++e) {
    const int64_t b = e / block_size;
    const float factor = load_elem(qfactor, b / scaler_block_size, is_bf16);
    const float scaler = rd(rd((float)qscalers[b] / factor, is_bf16) + mean, is_bf16);
    const uint8_t byte = qdata[e >> 1];
    const int code = (e & 1) ? (byte & 0x0f) : (byte >> 4);
    store_elem(out, e, rd(rd(NF4[code], is_bf16) * scaler, is_bf16), is_bf16);
  }
}

/* ---- QAT fake quantisation ------------------------------------------------------------------------- */

static const float F32_EPS = 1.1920928955078125e-07f;

/* per-token (per-row) asymmetric int8; qparams in fp32.  scale_out / zp_out may be NULL */
void ref_fq_per_token_qp(const void* x, int is_bf16, int qp_bf16, int64_t rows, int64_t K, void* out, float* scale_out,
                         int32_t* zp_out) {
  for (int64_t r = 0; r < rows; ++r) {
    float mn = load_elem(x, r * K, is_bf16), mx = mn;
    for (int64_t k = 1; k < K; ++k) {
      float v = load_elem(x, r * K + k, is_bf16);
      mn = v < mn ? v : mn;
      mx = v > mx ? v : mx;
    }
    mn = mn < 0.0f ? mn : 0.0f;
    mx = mx > 0.0f ? mx : 0.0f;
    float scale = (mx - mn) / 255.0f;
    if (!(scale > F32_EPS)) scale = F32_EPS;
    const float dmin = mn / scale, dmax = mx / scale;
    float zp = ((-128.0f + dmin) + (127.0f + dmax) > 0.0f) ? (-128.0f - dmin) : (127.0f - dmax);
    zp = zp < -128.0f ? -128.0f : (zp > 127.0f ? 127.0f : zp);
    zp = rintf(zp);
    if (qp_bf16) scale = to_bf16(scale); /* scale_precision = bf16: the rounded scale quantises and dequantises */
    const float inv = 1.0f / scale;
    for (int64_t k = 0; k < K; ++k) {
      float q = rintf(load_elem(x, r * K + k, is_bf16) * inv) + zp;
      q = q < -128.0f ? -128.0f : (q > 127.0f ? 127.0f : q);
      /* (q - zp) is an integer of magnitude <= 255: exact in either dtype */
      store_elem(out, r * K + k, (q - zp) * scale, is_bf16);
    }
    if (scale_out) scale_out[r] = scale;
    if (zp_out) zp_out[r] = (int32_t)zp;
  }
}

void ref_fq_per_token(const void* x, int is_bf16, int64_t rows, int64_t K, void* out, float* scale_out,
                      int32_t* zp_out) {
  ref_fq_per_token_qp(x, is_bf16, 0, rows, K, out, scale_out, zp_out);
}

static float group_scale(const void* w, int64_t base, int g, int is_bf16) {
  float mn = load_elem(w, base, is_bf16), mx = mn;
  for (int i = 1; i < g; ++i) {
    float v = load_elem(w, base + i, is_bf16);
    mn = v < mn ? v : mn;
    mx = v > mx ? v : mx;
  }
  mn = mn < 0.0f ? mn : 0.0f;
  mx = mx > 0.0f ? mx : 0.0f;
  float amax = -mn > mx ? -mn : mx;
  float scale = amax / 7.5f; /* (qmax - qmin) / 2 with qmin,qmax = -8,7 */
  if (!(scale > F32_EPS)) scale = F32_EPS;
  return scale;
}

/* per-group symmetric int4 along K; fq_out and/or q_out may be NULL */
void ref_fq_per_group_qp(const void* w, int is_bf16, int qp_bf16, int64_t rows, int64_t K, int g, void* fq_out,
                         int8_t* q_out, float* scale_out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t k0 = 0; k0 < K; k0 += g) {
      float scale = group_scale(w, r * K + k0, g, is_bf16);
      if (qp_bf16) scale = to_bf16(scale);
      const float inv = 1.0f / scale;
      for (int i = 0; i < g; ++i) {
        float q = rintf(load_elem(w, r * K + k0 + i, is_bf16) * inv);
        q = q < -8.0f ? -8.0f : (q > 7.0f ? 7.0f : q);
        /* the reference goes through an integer tensor here, so -0.0 becomes +0.0 */
        if (fq_out) store_elem(fq_out, r * K + k0 + i, (float)(int)q * scale, is_bf16);
        if (q_out) q_out[r * K + k0 + i] = (int8_t)q;
      }
      if (scale_out) scale_out[r * (K / g) + k0 / g] = scale;
    }
}

void ref_fq_per_group(const void* w, int is_bf16, int64_t rows, int64_t K, int g, void* fq_out, int8_t* q_out,
                      float* scale_out) {
  ref_fq_per_group_qp(w, is_bf16, 0, rows, K, g, fq_out, q_out, scale_out);
}

/* per-group asymmetric uint4 with a floating-point zero point (the weight-only "4w-qat" scheme), every operation
 * rounded to the tensor dtype, qparams additionally to bf16 when qp_bf16; fq_out, q_out (one code per byte),
 * scale_out, zero_out may each be NULL */
void ref_fq_per_group_uint4_asym(const void* w, int is_bf16, int qp_bf16, int64_t rows, int64_t K, int g, void* fq_out,
                                 uint8_t* q_out, float* scale_out, float* zero_out) {
#define RND(v) (is_bf16 ? to_bf16(v) : (v))
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t k0 = 0; k0 < K; k0 += g) {
      float mn = load_elem(w, r * K + k0, is_bf16), mx = mn;
      for (int i = 1; i < g; ++i) {
        const float v = load_elem(w, r * K + k0 + i, is_bf16);
        if (v < mn) mn = v;
        if (v > mx) mx = v;
      }
      float range = RND(mx - mn);
      float scale = RND(range / 15.0f);
      if (scale < 1e-6f) scale = RND(1e-6f);
      float eight = RND(scale * 8.0f);
      float zero = RND(mn + eight);
      if (qp_bf16) {
        scale = to_bf16(scale);
        zero = to_bf16(zero);
      }
      eight = RND(scale * 8.0f);
      const float lowest = RND(zero - eight);
      for (int i = 0; i < g; ++i) {
        const float d = RND(load_elem(w, r * K + k0 + i, is_bf16) - lowest);
        float q = rintf(RND(d / scale));
        q = q < 0.0f ? 0.0f : (q > 15.0f ? 15.0f : q);
        if (q_out) q_out[r * K + k0 + i] = (uint8_t)q;
        if (fq_out) {
          const float t = RND((q - 8.0f) * scale);
          store_elem(fq_out, r * K + k0 + i, t + zero, is_bf16);
        }
      }
      if (scale_out) scale_out[r * (K / g) + k0 / g] = scale;
      if (zero_out) zero_out[r * (K / g) + k0 / g] = zero;
    }
#undef RND
}

/* ---------------------------------------------------------------------------------------------------
 * Checkers for two shortcuts of the bf16 quantise kernel (they restate nothing of the reference; they
 * prove, by enumeration, that the shortcuts cannot change a result).
 * ------------------------------------------------------------------------------------------------- */

/* Shortcut 1: with y = 1/a divided once per block, q = fma(fma(-x*y, a, x), y, x*y) must round to the same
 * bf16 as the correctly rounded x / a.  Enumerates every bf16 divisor a with bit pattern in [a_lo, a_hi) and
 * every bf16 numerator 0 <= x <= a (signs are symmetric); returns the number of pairs that differ.  The `_upto`
 * form takes numerators up to max_quotient * a (the weight-only uint4 kernel divides a group's offsets, up to 15 steps
 * and a rounding's worth more, by its scale). */
#if defined(__x86_64__)
__attribute__((target("fma")))
#endif
int64_t ref_check_shared_reciprocal_division_upto(int a_lo, int a_hi, float max_quotient) {
  int64_t bad = 0;
  for (int ai = a_lo; ai < a_hi; ++ai) {
    const float a = float_of((uint32_t)ai << 16);
    const float y = 1.0f / a;
    const float top = a * max_quotient;
    for (int xi = 0; xi < 0x7F80; ++xi) {
      const float x = float_of((uint32_t)xi << 16);
      if (x > top) break;
      const float q0 = x * y;
      const float r = fmaf(-q0, a, x);
      const float q1 = fmaf(r, y, q0);
      if (bits_of(to_bf16(x / a)) != bits_of(to_bf16(q1))) ++bad;
    }
  }
  return bad;
}

#if defined(__x86_64__)
__attribute__((target("fma")))
#endif
int64_t ref_check_shared_reciprocal_division(int a_lo, int a_hi) {
  return ref_check_shared_reciprocal_division_upto(a_lo, a_hi, 1.0f);
}

/* Shortcut 2: the code of a scaled bf16 value is looked up in a table that only spans magnitudes 2^-5 .. 1.
 * Returns the number of bf16 patterns below 2^-5 (either sign) whose code is not 7, plus 1 if NaN is not code 0;
 * table_out, if not NULL, receives the codes of magnitudes 0x3D00..0x3F80 for sign 0 then sign 1 (2 x 641 bytes). */
int ref_check_code_table(uint8_t* table_out) {
  int bad = 0;
  for (int sign = 0; sign < 2; ++sign)
    for (int mag = 0; mag <= 0x3F80; ++mag) {
      const int c = nearest_code(float_of(((uint32_t)sign << 31) | ((uint32_t)mag << 16)), 1);
      if (mag < 0x3D00) {
        if (c != 7) ++bad;
      } else if (table_out) {
        table_out[sign * 641 + (mag - 0x3D00)] = (uint8_t)c;
      }
    }
  if (nearest_code(float_of(0x7fc00000u), 1) != 0) ++bad;
  return bad;
}
