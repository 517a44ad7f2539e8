/*
 * CPU oracle (plain scalar C) for the NVFP4 path of ac4k_kernel.
 *
 * TEST INFRASTRUCTURE ONLY: linked or loaded only by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, as the
 * checker.  The shipped library never calls into it.
 *
 * This restatement follows the reference *kernels'* strided indexing and
 * operation order, evaluated in IEEE-754 round-to-nearest fp32 (build with
 * -ffp-contract=off, no fast-math):
 *   lib/cuda/sm120/quantize_nvfp4.cu:49-157   nvfp4 quantize
 *   lib/cuda/common/math.cuh:39-80            cvt.rn.satfinite e4m3 / e2m1, nibble order
 *   python/ac4k_kernel/ops/quant.py:33-59     global scale
 *   lib/cuda/sm120/quantize_fp8.cu:57-185     per-row fp8
 *   lib/cuda/sm120/quantize_int8.cu:55-168    per-row int8
 *   lib/cuda/sm120/linear_nvfp4.cu:586-633    linear epilogue order
 *   lib/cuda/sm120/mma.cuh:13-56              block-scaled dot product
 * The conversions are written at bit level (integer rounding), on purpose
 * differently from oracle/nvfp4_oracle.py (torch casts and threshold
 * compares); tests/test_oracle_*.py checks the two against each other.
 *
 * Pinning status: as stated in oracle/nvfp4_oracle.py (int8 quantize and the
 * NaN/Inf/all-zero edges are "parity unpinned" against reference-held vectors).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t align_up64(int64_t a, int64_t b) { return ceil_div64(a, b) * b; }

/* cvt.rn.satfinite.e4m3.f32 : RNE; |x| >= 448 and inf -> +-448; NaN -> 0x7F. */
uint8_t oracle_f32_to_e4m3(float f) {
  uint32_t u = f32_bits(f);
  uint32_t a = u & 0x7fffffffu;
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  if (a > 0x7f800000u) return 0x7f;
  if (a >= 0x43e00000u) return sign | 0x7e; /* 448.0f = 0x43e00000 */
  int e = (int)(a >> 23) - 127;
  if (e < -6) {
    /* subnormal grid: multiples of 2^-9; the scaling by 2^9 is exact */
    float q = nearbyintf(bits_f32(a) * 512.0f); /* 0..8, ties to even */
    return sign | (uint8_t)q;                   /* 8 -> 0x08 = 2^-6, the first normal */
  }
  uint32_t m = a & 0x7fffffu;
  uint32_t keep = m >> 20, rest = m & 0xfffffu;
  if (rest > 0x80000u || (rest == 0x80000u && (keep & 1u))) keep++;
  uint32_t code = ((uint32_t)(e + 7) << 3) + keep; /* mantissa carry bumps the exponent */
  if (code > 0x7e) code = 0x7e;
  return sign | (uint8_t)code;
}

float oracle_e4m3_to_f32(uint8_t b) {
  int e = (b >> 3) & 0xf, m = b & 7;
  float v;
  if (e == 0xf && m == 7)
    v = NAN;
  else if (e == 0)
    v = ldexpf((float)m, -9);
  else
    v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return (b & 0x80) ? -v : v;
}

/* cvt.rn.satfinite.e2m1.f32 : grid {0,.5,1,1.5,2,3,4,6}, ties to the even code,
 * saturate to 6, sign kept for zero, NaN -> 0x7. */
uint8_t oracle_f32_to_e2m1(float f) {
  uint32_t u = f32_bits(f);
  uint8_t sign = (uint8_t)((u >> 28) & 0x8u);
  float a = fabsf(f);
  if (a != a) return 0x7;
  int code;
  if (a < 2.0f)
    code = (int)nearbyintf(a * 2.0f); /* step 0.5: 0,.5,1,1.5,2 -> codes 0..4 */
  else if (a < 4.0f)
    code = 2 + (int)nearbyintf(a); /* step 1: 2,3,4 -> codes 4,5,6 */
  else if (a <= 6.0f)
    code = 4 + (int)nearbyintf(a * 0.5f); /* step 2: 4,6 -> codes 6,7 */
  else
    code = 7;
  return sign | (uint8_t)code;
}

static const float kE2M1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
float oracle_e2m1_to_f32(uint8_t c) {
  float v = kE2M1[c & 7];
  return (c & 8) ? -v : v;
}

/* cvt.rni.sat.s8.f32 */
int8_t oracle_f32_to_s8(float f) {
  if (f != f) return 0;
  float r = nearbyintf(f);
  if (r > 127.0f) r = 127.0f;
  if (r < -128.0f) r = -128.0f;
  return (int8_t)r;
}

/* quant.py:33-59: gs = fp32(max|x|) / max_scale, out starts at 0 and takes a max. */
float oracle_global_scale_bf16(const uint16_t *x, int64_t n, float max_scale) {
  uint16_t amax = 0;
  for (int64_t i = 0; i < n; ++i) {
    uint16_t a = x[i] & 0x7fffu;
    if (a > 0x7f80u) continue; /* NaN is skipped by max */
    if (a > amax) amax = a;
  }
  float gs = bf16_to_f32(amax) / max_scale;
  return gs > 0.0f ? gs : 0.0f;
}

/* Position in the reduce dim that output element `k` (0..Kp) is read from
 * (quantize_nvfp4.cu:86-100): inside every 32-group, out[t*8+q*2+r] = in[q*8+t*2+r]. */
static inline int64_t nvfp4_src_pos(int64_t k, int swizzle) {
  if (!swizzle) return k;
  int64_t g = k / 32, p = k % 32;
  int64_t t = p / 8, q = (p % 8) / 2, r = p % 2;
  return g * 32 + q * 8 + t * 2 + r;
}

/* in: 4-D [d0,d1,R,K] addressed with element strides; out [d0,d1,R,Kp/2];
 * sf [d0,d1,Kp/64,Rp,4] (e4m3 bits). */
void oracle_quantize_nvfp4(uint8_t *out, uint8_t *sf, const uint16_t *in, float gs, int64_t d0,
                           int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                           int64_t sK, int swizzle) {
  const int64_t Kp = align_up64(K, 64), Rp = align_up64(R, 16);
  const float alpha = 1.0f / gs;
  for (int64_t i0 = 0; i0 < d0; ++i0)
    for (int64_t i1 = 0; i1 < d1; ++i1) {
      const int64_t lead = i0 * d1 + i1;
      for (int64_t r = 0; r < Rp; ++r)
        for (int64_t kb = 0; kb < Kp; kb += 16) {
          uint8_t *sfp = sf + 4 * ((lead * (Kp / 64) + kb / 64) * Rp + r) + (kb % 64) / 16;
          if (r >= R) {
            *sfp = 0;
            continue;
          }
          float x[16], m = 0.0f;
          for (int i = 0; i < 16; ++i) {
            int64_t k = nvfp4_src_pos(kb + i, swizzle);
            x[i] = k < K ? bf16_to_f32(in[i0 * s0 + i1 * s1 + r * sR + k * sK]) : 0.0f;
            float a = fabsf(x[i]);
            if (a > m) m = a; /* NaN compares false: skipped like __hmax2 */
          }
          float sixth = m * 0.16666666666666666f;
          float s32 = alpha * sixth;
          uint8_t code = oracle_f32_to_e4m3(s32);
          float s = oracle_e4m3_to_f32(code);
          float o = (s != 0.0f) ? alpha * (1.0f / s) : 0.0f;
          *sfp = code;
          uint8_t *op = out + (lead * R + r) * (Kp / 2) + kb / 2;
          for (int i = 0; i < 16; i += 2) {
            uint8_t lo = oracle_f32_to_e2m1(x[i] * o);
            uint8_t hi = oracle_f32_to_e2m1(x[i + 1] * o);
            op[i / 2] = (uint8_t)(lo | (hi << 4));
          }
        }
    }
}

/* quantize_fp8.cu:141-151: inside every 16-group, out[t*4+q*2+r] = in[q*8+t*2+r]. */
static inline int64_t fp8_src_pos(int64_t k, int swizzle) {
  if (!swizzle) return k;
  int64_t g = k / 16, p = k % 16;
  int64_t t = p / 4, q = (p % 4) / 2, r = p % 2;
  return g * 16 + q * 8 + t * 2 + r;
}

static float row_amax(const uint16_t *row, int64_t K, int64_t sK) {
  float m = 0.0f;
  for (int64_t k = 0; k < K; ++k) {
    float a = fabsf(bf16_to_f32(row[k * sK]));
    if (a > m) m = a;
  }
  return m;
}

/* out [d0,d1,R,Kp16] e4m3 bits; sf [d0,d1,Rp] fp32. */
void oracle_quantize_fp8(uint8_t *out, float *sf, const uint16_t *in, float smax, int64_t d0,
                         int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                         int64_t sK, int swizzle) {
  const int64_t Kp = align_up64(K, 16), Rp = align_up64(R, 16);
  for (int64_t i0 = 0; i0 < d0; ++i0)
    for (int64_t i1 = 0; i1 < d1; ++i1) {
      const int64_t lead = i0 * d1 + i1;
      for (int64_t r = 0; r < Rp; ++r) {
        if (r >= R) {
          sf[lead * Rp + r] = 0.0f / smax;
          continue;
        }
        const uint16_t *row = in + i0 * s0 + i1 * s1 + r * sR;
        float amax = row_amax(row, K, sK);
        sf[lead * Rp + r] = amax / smax;
        float recp = smax / amax;
        uint8_t *op = out + (lead * R + r) * Kp;
        for (int64_t k = 0; k < Kp; ++k) {
          int64_t src = fp8_src_pos(k, swizzle);
          float x = src < K ? bf16_to_f32(row[src * sK]) : 0.0f;
          op[k] = oracle_f32_to_e4m3(x * recp);
        }
      }
    }
}

void oracle_quantize_int8(int8_t *out, float *sf, const uint16_t *in, int32_t smax_i, int64_t d0,
                          int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                          int64_t sK) {
  const int64_t Kp = align_up64(K, 16), Rp = align_up64(R, 16);
  const float smax = (float)smax_i;
  for (int64_t i0 = 0; i0 < d0; ++i0)
    for (int64_t i1 = 0; i1 < d1; ++i1) {
      const int64_t lead = i0 * d1 + i1;
      for (int64_t r = 0; r < Rp; ++r) {
        if (r >= R) {
          sf[lead * Rp + r] = 0.0f / smax;
          continue;
        }
        const uint16_t *row = in + i0 * s0 + i1 * s1 + r * sR;
        float amax = row_amax(row, K, sK);
        sf[lead * Rp + r] = amax / smax;
        float recp = smax / amax;
        int8_t *op = out + (lead * R + r) * Kp;
        for (int64_t k = 0; k < Kp; ++k) {
          float x = k < K ? bf16_to_f32(row[k * sK]) : 0.0f;
          op[k] = oracle_f32_to_s8(x * recp);
        }
      }
    }
}

/* D[m,n] = (sum_j sfA[m,j] sfB[n,j] sum_{i<16} a b) * (gsA*gsB) + bias[n], fp32 out.
 * A [M,K/2], B [N,K/2] packed; sf dword of (row, 64-chunk c) at sf[(c*Rp + row)*4 ..].
 * The block sums are exact in double; the running sum is kept in double and rounded to
 * fp32 once, which is what "fp32 accumulation, order hardware-defined" is compared to. */
void oracle_linear_nvfp4(float *D, const uint8_t *A, const uint8_t *A_sf, float A_gs,
                         const uint8_t *B, const uint8_t *B_sf, float B_gs, const float *bias,
                         int64_t M, int64_t N, int64_t K) {
  const int64_t Mp = align_up64(M, 16), Np = align_up64(N, 16), kb = K / 2;
  const float scale = A_gs * B_gs;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t j = 0; j < K / 16; ++j) {
        float sa = oracle_e4m3_to_f32(A_sf[((j / 4) * Mp + m) * 4 + j % 4]);
        float sb = oracle_e4m3_to_f32(B_sf[((j / 4) * Np + n) * 4 + j % 4]);
        double blk = 0.0;
        for (int i = 0; i < 8; ++i) {
          uint8_t ab = A[m * kb + j * 8 + i], bb = B[n * kb + j * 8 + i];
          blk += (double)oracle_e2m1_to_f32(ab & 0xf) * (double)oracle_e2m1_to_f32(bb & 0xf);
          blk += (double)oracle_e2m1_to_f32(ab >> 4) * (double)oracle_e2m1_to_f32(bb >> 4);
        }
        acc += (double)sa * (double)sb * blk;
      }
      float d = (float)acc * scale;
      if (bias) d += bias[n];
      D[m * N + n] = d;
    }
}
