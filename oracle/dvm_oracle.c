/* CPU oracle for the DVM vector / matmul path. TEST INFRASTRUCTURE ONLY: it is
 * used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
 * bench.py as the checker; the product (dvm_amd) never links or calls it.
 *
 * Each function restates, in plain scalar C, what the reference's device VM
 * computes for one operator family (file:line under the reference tree):
 *   - element functors: src/vm_gpu.cu:198-329 ("compute in fp32, round once"
 *     for fp16 / bf16 through the F16Tag / BF16Tag accessors :162-181);
 *   - f32 -> bf16 round-to-nearest-even bit trick: src/vm_gpu.cu:155-160;
 *   - host scalar codecs (fp16, bf16 with NaN -> 0x7fc0): src/dvm.cc:78-186;
 *   - compare -> 1/0 in the operand type: src/vm_gpu.cu:331-349,377-399;
 *   - select: src/vm_gpu.cu:401-410;
 *   - sum with fp64 accumulation: src/vm_gpu.cu:111-135,779-866; max / min
 *     follow the identities of src/ops.cc:103-108 (no GPU reference exists);
 *   - matmul: fp32 accumulation, one rounding to the output type on write-out,
 *     src/vm_aic.cce:20-31,364-430 (Ascend semantics; no GPU reference exists).
 * Pinned by tests/test_oracle.py against the constants and NumPy closed forms
 * the reference's own tests use (see that file's header for the list).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

typedef union {
  uint32_t u;
  float f;
} u32f;

/* ---- fp16 / bf16 ---------------------------------------------------------- */

float ora_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  u32f r;
  if (exp == 0) {
    if (man == 0) {
      r.u = sign;
      return r.f;
    }
    /* subnormal: man * 2^-24 */
    float v = ldexpf((float)man, -24);
    r.f = v;
    r.u |= sign;
    return r.f;
  }
  if (exp == 31) {
    r.u = sign | 0x7f800000u | (man << 13);
    return r.f;
  }
  r.u = sign | ((exp + 112u) << 23) | (man << 13);
  return r.f;
}

/* IEEE round-to-nearest-even, the rounding of __float2half_rn (src/vm_gpu.cu:153). */
uint16_t ora_f32_to_f16(float f) {
  u32f x;
  x.f = f;
  uint16_t sign = (uint16_t)((x.u >> 16) & 0x8000u);
  uint32_t a = x.u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (a == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  if (e > 15) return (uint16_t)(sign | 0x7c00u);
  int shift; /* bits dropped from the 24-bit significand */
  int32_t he;
  if (e >= -14) {
    shift = 13;
    he = e + 15;
  } else {
    shift = 13 + (-14 - e);
    he = 0;
    if (shift > 25) return sign;
  }
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept += 1;
  uint32_t out;
  if (he == 0) {
    out = kept; /* subnormal; a carry into bit 10 makes it the smallest normal */
  } else {
    out = ((uint32_t)he << 10) + (kept - 0x400u); /* a carry out of the mantissa bumps the exponent */
  }
  if (out >= 0x7c00u) out = 0x7c00u;
  return (uint16_t)(sign | out);
}

float ora_bf16_to_f32(uint16_t h) {
  u32f r;
  r.u = (uint32_t)h << 16;
  return r.f;
}

/* Device conversion: no NaN special case (src/vm_gpu.cu:155-160). */
uint16_t ora_f32_to_bf16_dev(float f) {
  u32f x;
  x.f = f;
  uint32_t lsb = (x.u >> 16) & 1u;
  x.u += 0x7fffu + lsb;
  return (uint16_t)(x.u >> 16);
}

/* Host scalar codec: NaN -> 0x7fc0 (src/dvm.cc:173-186). */
uint16_t ora_f32_to_bf16_host(float f) {
  if (isnan(f)) return 0x7fc0u;
  return ora_f32_to_bf16_dev(f);
}

/* Rounds a float to the value set of element type t (1 fp16, 2 bf16, others unchanged).
 * bf16 and NaN: the bit trick the reference's device code uses (src/vm_gpu.cu:155-160, ora_f32_to_bf16_dev
 * above) has no NaN case; it keeps every NaN whose low mantissa half does not carry out (the default quiet NaN
 * 0x7fc00000 among them, which is what arithmetic produces) but turns the payloads 0x7fff8000..0x7fffffff into
 * -0.0 and the like. The gfx950 hardware conversion keeps every NaN a NaN. The oracle follows the hardware
 * here: a NaN stays a NaN. For every input that is not a NaN the two agree bit for bit. */
static float round_to(int t, float v) {
  if (t == 1) return ora_f16_to_f32(ora_f32_to_f16(v));
  if (t == 2) return isnan(v) ? v : ora_bf16_to_f32(ora_f32_to_bf16_dev(v));
  return v;
}

/* ---- element functors (float class: values carried as fp32) ------------------ */
/* op ids follow dvm::UnaryType / dvm::BinaryType of include/dvm.h. */

void ora_unary_f(int op, int t, const float *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float a = x[i], r;
    switch (op) {
      case 0: r = sqrtf(a); break;
      case 1: r = fabsf(a); break;
      case 2: r = logf(a); break;
      case 3: r = expf(a); break;
      case 5: r = isfinite(a) ? 1.0f : 0.0f; break;
      case 7: r = nearbyintf(a); break;
      case 8: r = floorf(a); break;
      case 9: r = ceilf(a); break;
      case 10: r = truncf(a); break;
      default: r = a; break;
    }
    y[i] = round_to(t, r);
  }
}

void ora_abs_i32(const int32_t *x, int32_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = x[i] < 0 ? (int32_t)(0u - (uint32_t)x[i]) : x[i];
}

void ora_binary_f(int op, int t, const float *a, const float *b, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float p = a[i], q = b[i], r;
    switch (op) {
      case 6: r = p + q; break;
      case 7: r = p - q; break;
      case 8: r = p * q; break;
      case 9: r = p / q; break;
      case 10: r = powf(p, q); break;
      case 11: r = p > q ? p : q; break;
      case 12: r = p < q ? p : q; break;
      case 13: r = (p != 0.0f && q != 0.0f) ? 1.0f : 0.0f; break;
      case 14: r = (p != 0.0f || q != 0.0f) ? 1.0f : 0.0f; break;
      default: r = 0.0f; break;
    }
    y[i] = round_to(t, r);
  }
}

void ora_binary_i32(int op, const int32_t *a, const int32_t *b, int32_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    uint32_t p = (uint32_t)a[i], q = (uint32_t)b[i];
    switch (op) {
      case 6: y[i] = (int32_t)(p + q); break;
      case 7: y[i] = (int32_t)(p - q); break;
      case 8: y[i] = (int32_t)(p * q); break;
      case 11: y[i] = a[i] > b[i] ? a[i] : b[i]; break;
      case 12: y[i] = a[i] < b[i] ? a[i] : b[i]; break;
      default: y[i] = 0; break;
    }
  }
}

static int cmp_f(int op, float p, float q) {
  switch (op) {
    case 0: return p == q;
    case 1: return p != q;
    case 2: return p > q;
    case 3: return p >= q;
    case 4: return p < q;
    default: return p <= q;
  }
}

void ora_compare_f(int op, const float *a, const float *b, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = cmp_f(op, a[i], b[i]) ? 1.0f : 0.0f;
}

void ora_compare_i32(int op, const int32_t *a, const int32_t *b, int32_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    int r;
    switch (op) {
      case 0: r = a[i] == b[i]; break;
      case 1: r = a[i] != b[i]; break;
      case 2: r = a[i] > b[i]; break;
      case 3: r = a[i] >= b[i]; break;
      case 4: r = a[i] < b[i]; break;
      default: r = a[i] <= b[i]; break;
    }
    y[i] = r;
  }
}

/* cond holds 1/0 in the operand type; 4-byte lanes cover both classes. */
void ora_select_32(const uint32_t *cond, const uint32_t *a, const uint32_t *b, uint32_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = (cond[i] << 1) != 0 ? a[i] : b[i];
}

/* ---- casts ------------------------------------------------------------------- */

void ora_round_f(int t, const float *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = round_to(t, x[i]);
}
/* The reference's functor is a C cast (src/vm_gpu.cu:299-301). Its device compiler turns that into the saturating
 * conversion of the PTX ISA (cvt.rzi.s32.f32: truncation toward zero, a value beyond the range gives the nearest end
 * of the range, NaN gives 0); the same cast on the host is undefined for those inputs, so they are spelled out. */
static int32_t f_to_i32(float x) {
  if (x != x) return 0;
  if (x >= 2147483648.0f) return INT32_MAX;
  if (x <= -2147483648.0f) return INT32_MIN;
  return (int32_t)x;
}
void ora_f_to_i32(const float *x, int32_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = f_to_i32(x[i]);
}
void ora_i32_to_f(int t, const int32_t *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = round_to(t, (float)x[i]);
}
void ora_f_to_bool(const float *x, uint8_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = x[i] != 0.0f ? 1 : 0;
}
void ora_f16_bits_to_f32(const uint16_t *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = ora_f16_to_f32(x[i]);
}
void ora_f32_to_f16_bits(const float *x, uint16_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = ora_f32_to_f16(x[i]);
}
void ora_bf16_bits_to_f32(const uint16_t *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = ora_bf16_to_f32(x[i]);
}
void ora_f32_to_bf16_bits(const float *x, uint16_t *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = ora_f32_to_bf16_host(x[i]);
}

/* ---- reduce over the middle axis of [outer, red, inner] -------------------------- */
/* kind: 0 sum (fp64 accumulation, rounded once), 1 max, 2 min (NaN propagates, as NumPy). */
void ora_reduce_f32(int kind, const float *x, size_t outer, size_t red, size_t inner, float *y) {
  for (size_t o = 0; o < outer; ++o) {
    for (size_t i = 0; i < inner; ++i) {
      const float *p = x + o * red * inner + i;
      if (kind == 0) {
        double acc = 0.0;
        for (size_t r = 0; r < red; ++r) acc += (double)p[r * inner];
        y[o * inner + i] = (float)acc;
      } else {
        float acc = kind == 1 ? -INFINITY : INFINITY;
        for (size_t r = 0; r < red; ++r) {
          float v = p[r * inner];
          if (v != v) acc = v;
          else if (acc == acc && (kind == 1 ? v > acc : v < acc)) acc = v;
        }
        y[o * inner + i] = acc;
      }
    }
  }
}

/* ---- matmul: C[m,n] = sum_k A[m,k] * B[k,n] (+ bias[n]) in fp32, rounded once to type t ---- */
/* a, b are fp32 copies of the fp16 / bf16 operands; trans flags give the storage layout. */
void ora_matmul(const float *a, const float *b, const float *bias, float *c, size_t m, size_t n, size_t k, int trans_a,
                int trans_b, int t) {
  for (size_t i = 0; i < m; ++i) {
    for (size_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (size_t p = 0; p < k; ++p) {
        float x = trans_a ? a[p * m + i] : a[i * k + p];
        float y = trans_b ? b[j * k + p] : b[p * n + j];
        acc += x * y;
      }
      if (bias) acc += bias[j];
      c[i * n + j] = round_to(t, acc);
    }
  }
}

/* ---- whole-config restatements used as the CPU baseline ------------------------------ */
/* Batch-norm forward, training statistics, NCHW fp32: per channel mean and biased variance in
 * fp64, then (x - mean) / sqrt(var + eps) * gamma + beta in fp32 op by op, as the fused graph does. */
void ora_batchnorm_nchw(const float *x, const float *gamma, const float *beta, float *y, size_t n, size_t c, size_t hw,
                        float eps) {
  const double cnt = (double)n * (double)hw;
  for (size_t ch = 0; ch < c; ++ch) {
    double s = 0.0;
    for (size_t i = 0; i < n; ++i) {
      const float *p = x + (i * c + ch) * hw;
      for (size_t j = 0; j < hw; ++j) s += p[j];
    }
    const float mean = (float)s * (float)(1.0 / cnt);
    double q = 0.0;
    for (size_t i = 0; i < n; ++i) {
      const float *p = x + (i * c + ch) * hw;
      for (size_t j = 0; j < hw; ++j) {
        float d = p[j] - mean;
        q += (double)(d * d);
      }
    }
    const float var = (float)q * (float)(1.0 / cnt);
    const float sd = sqrtf(var + eps);
    for (size_t i = 0; i < n; ++i) {
      const float *p = x + (i * c + ch) * hw;
      float *o = y + (i * c + ch) * hw;
      for (size_t j = 0; j < hw; ++j) o[j] = (p[j] - mean) / sd * gamma[ch] + beta[ch];
    }
  }
}
