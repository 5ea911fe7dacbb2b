/*
 * oracle.c — CPU restatement of bunker's Qwen3.5 decode hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library or its host layer
 * may link, load or call this file; it exists so that tests, the smoke check
 * and the benchmark's CPU-baseline leg have an independent answer to compare
 * the HIP kernels with.
 *
 * Each function follows the reference source lines cited above it (paths are
 * relative to the skyne98/bunker tree).
 *
 * Arithmetic rules (shared with the HIP kernels, so that results agree to the
 * bit wherever the mathematics allows and do not depend on launch shapes):
 *   - reductions whose order the reference leaves open (tt.sum / tt.dot) are
 *     accumulated in double and rounded once to f32;
 *   - exp, log and 1/sqrt are evaluated in double and rounded once to f32;
 *   - elementwise f32 arithmetic is done exactly as written, one IEEE
 *     operation per written operation (build with -ffp-contract=off); a fused
 *     multiply-add appears only where fmaf() is written;
 *   - the two k-reductions of the gated-DeltaNet step use f32 fmaf chains over
 *     16 consecutive rows followed by a sequential sum of the 8 chain results
 *     (the "canonical order"; pass rows_per_chain = 0 for double accumulation).
 *
 * Pinning status (which independent check fixes each function):
 *   orc_encode_half / orc_f32to16   exhaustive fp16 round trip + hand vectors
 *   orc_pack_q8_1                   tie vectors, |x-d*q|<=d/2, amax->+-127
 *   orc_legacy_dequant_i8           tests/test_dequant.ts:15-21 known answer
 *   orc_legacy_qmm                  brute-force float dot of dequantised values
 *   orc_i8_gemm                     tests/test_q4k_pipeline.ts:111-116 triple loop
 *   orc_q4k_* (144-byte block)      PARITY UNPINNED by the reference (the
 *                                   reference never uses this layout); pinned by
 *                                   the published ggml layout, a hand-built
 *                                   block, pack/unpack round trips and the
 *                                   integer-dot special case
 *   orc_quantize_q4k                PARITY UNPINNED against ggml (absent); invariants:
 *                                   constant blocks, representable grids, fitted error
 *                                   <= min/max grid error, reconstruction error bound
 *   orc_f32_to_half_rne             exhaustive round trip of all 65536 halves, midpoints,
 *                                   numpy float16 on random values
 *   orc_gdn_step                    closed-form invariants (beta=0, S=0) and a
 *                                   numpy float64 restatement of refGDN
 *   orc_attn_decode_paged           numpy float64 softmax, len=1, page permutation
 *   orc_rmsnorm/swiglu/conv1d/rope  numpy float64 closed forms, pos=0 identity
 *   orc_argmax                      prototypes/test_argmax.ts:33-44 vector + ties
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* Threads the row / head loops below run on (the benchmark's CPU-baseline leg times one thread and all cores). */
ORC_API void orc_set_threads(int n) { if (n >= 1) omp_set_num_threads(n); }
ORC_API int orc_max_threads(void) { return omp_get_max_threads(); }

/* ------------------------------------------------------------------ */
/* scalar conversions                                                   */
/* ------------------------------------------------------------------ */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* bench/bench.ts:41-51 encodeHalf: the JS number is first rounded to f32
 * (DataView.setFloat32), then the mantissa is TRUNCATED to 10 bits;
 * results below the fp16 normal range flush to signed zero, above it to Inf. */
ORC_API uint16_t orc_encode_half(double v) {
  if (v == 0) return 0;
  uint32_t bits = f2u((float)v);
  uint32_t s = (bits >> 16) & 0x8000u, e = (bits >> 23) & 0xffu, m = bits & 0x7fffffu;
  int ne = (int)e - 127 + 15;
  if (ne >= 31) return (uint16_t)(s | 0x7c00u);
  if (ne <= 0) return (uint16_t)s;
  return (uint16_t)(s | ((uint32_t)ne << 10) | (m >> 13));
}

/* src/kernel.ts:16-32 f32to16: same truncation, but NaN keeps a quiet bit. */
ORC_API void orc_f32to16(const float* x, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    uint32_t v = f2u(x[i]);
    uint32_t sign = (v >> 16) & 0x8000u, ex = (v >> 23) & 0xffu, mant = v & 0x7fffffu;
    if (ex == 0) { out[i] = (uint16_t)sign; continue; }
    if (ex == 0xff) { out[i] = (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0)); continue; }
    int e16 = (int)ex - 127 + 15;
    if (e16 >= 0x1f) { out[i] = (uint16_t)(sign | 0x7c00u); continue; }
    if (e16 <= 0) { out[i] = (uint16_t)sign; continue; }
    out[i] = (uint16_t)(sign | ((uint32_t)e16 << 10) | (mant >> 13));
  }
}

/* Exact IEEE binary16 -> binary32 (denormals honoured). */
ORC_API float orc_half_to_float(uint16_t h) {
  uint32_t s = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  if (e == 0) {
    if (m == 0) return u2f(s);
    float f = (float)m * 5.9604644775390625e-08f; /* m * 2^-24 */
    return s ? -f : f;
  }
  if (e == 31) return u2f(s | 0x7f800000u | (m << 13));
  return u2f(s | ((e - 15 + 127) << 23) | (m << 13));
}

/* src/dsl.ts:955-975 half_to_float: exponent field 0 returns +0.0 (denormals
 * flushed); exponent 31 is treated as an ordinary exponent. */
ORC_API float orc_half_to_float_ftz(uint16_t h) {
  uint32_t sgn = h & 0x8000u, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  if (e == 0) return 0.0f;
  return u2f((sgn << 16) | ((e - 15 + 127) << 23) | (m << 13));
}

/* f32 -> bf16, round to nearest even (what arith.truncf lowers to). */
ORC_API uint16_t orc_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x7fffffu)) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
ORC_API float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
#define BF(h) orc_bf16_to_f32(h)
#define TOBF(f) orc_f32_to_bf16(f)

/* transcendental helpers: evaluated in double, rounded once */
static inline float sigmoidf_(float v) { return (float)(1.0 / (1.0 + exp(-(double)v))); }
static inline float rsqrt_(double v) { return (float)(1.0 / sqrt(v)); }

/* ------------------------------------------------------------------ */
/* Q8_1 activation quantizer                                            */
/* ------------------------------------------------------------------ */

/* ECMAScript Math.round: nearest integer, ties toward +infinity. */
static inline double js_round(double v) {
  double r = floor(v);
  if (v - r >= 0.5) r += 1.0;
  return r;
}

/* bench/bench.ts:53-72 packQ8_1.  Block layout (bench/bench.ts:6):
 * int8 q[32] @0, fp16 d @32, fp16 s @34; n need not be a multiple of 32
 * (missing elements quantize to 0). */
ORC_API void orc_pack_q8_1(const float* x, int64_t n, uint8_t* out) {
  int64_t nb = (n + 31) / 32;
  for (int64_t b = 0; b < nb; b++) {
    int64_t off = b * 32;
    int len = (int)((n - off) < 32 ? (n - off) : 32);
    double amax = 0;
    for (int i = 0; i < len; i++) { double a = fabs((double)x[off + i]); if (a > amax) amax = a; }
    double d = amax / 127.0;
    double div = d != 0 ? d : 1.0;
    double sum = 0;
    for (int i = 0; i < 32; i++) {
      double q = i < len ? js_round((double)x[off + i] / div) : 0.0;
      double c = q < -128 ? -128 : (q > 127 ? 127 : q);
      out[b * 36 + i] = (uint8_t)(int8_t)c;
      sum += q;
    }
    uint16_t hd = orc_encode_half(d), hs = orc_encode_half(sum * d);
    memcpy(out + b * 36 + 32, &hd, 2);
    memcpy(out + b * 36 + 34, &hs, 2);
  }
}

/* ------------------------------------------------------------------ */
/* legacy 20-byte / 32-element block (the reference's own "Q4_K")       */
/* ------------------------------------------------------------------ */

/* tests/test_dequant.ts:13-24, src/kernel.ts:455-456: byte j of a block gives
 * elements 2j (low nibble) and 2j+1 (high nibble), each minus 8. */
ORC_API void orc_legacy_dequant_i8(const uint8_t* blocks, int64_t nblocks, int8_t* out) {
  for (int64_t b = 0; b < nblocks; b++)
    for (int j = 0; j < 16; j++) {
      uint8_t q = blocks[b * 20 + j];
      out[b * 32 + 2 * j] = (int8_t)((q & 15) - 8);
      out[b * 32 + 2 * j + 1] = (int8_t)((q >> 4) - 8);
    }
}

/* bench/bench.ts:74-96 packQ4_K_col: column c of a K x N f32 matrix becomes
 * nb blocks; d=(max-min)/15, dmin=min, q=clamp(round((v-dmin)/(d||1)),0,15). */
ORC_API void orc_legacy_pack_q4k_col(const float* data, int K, int N, uint8_t* out) {
  int nb = (K + 31) / 32;
  for (int c = 0; c < N; c++)
    for (int b = 0; b < nb; b++) {
      uint8_t* blk = out + ((int64_t)c * nb + b) * 20;
      double v[32]; int len = 0;
      for (int k = b * 32; k < (b + 1) * 32 && k < K; k++) v[len++] = data[(int64_t)k * N + c];
      double mn = INFINITY, mx = -INFINITY;
      for (int i = 0; i < len; i++) { if (v[i] < mn) mn = v[i]; if (v[i] > mx) mx = v[i]; }
      double d = (mx - mn) / 15.0, dmin = mn, div = d != 0 ? d : 1.0;
      for (int i = 0; i < 16; i++) {
        double lo = 2 * i < len ? js_round((v[2 * i] - dmin) / div) : 0;
        double hi = 2 * i + 1 < len ? js_round((v[2 * i + 1] - dmin) / div) : 0;
        int l = (int)(lo < 0 ? 0 : lo > 15 ? 15 : lo), h = (int)(hi < 0 ? 0 : hi > 15 ? 15 : hi);
        blk[i] = (uint8_t)(l | (h << 4));
      }
      uint16_t hd = orc_encode_half(d), hm = orc_encode_half(dmin);
      memcpy(blk + 16, &hd, 2); memcpy(blk + 18, &hm, 2);
    }
}

/* bench/bench.ts:10-38 qmm: C[row,col] = sum_b d4*d8*s1 + dm*d8*s2 with the
 * flush-to-zero fp16 decode the kernel DSL supplies; f32 accumulation in block
 * order exactly as written. */
ORC_API void orc_legacy_qmm(const uint8_t* A, const uint8_t* B, float* C, int M, int N, int K) {
  int nb = K / 32;
  for (int row = 0; row < M; row++)
    for (int col = 0; col < N; col++) {
      float sum = 0;
      for (int b = 0; b < nb; b++) {
        const uint8_t* a = A + ((int64_t)row * nb + b) * 36;
        const uint8_t* w = B + ((int64_t)col * nb + b) * 20;
        uint16_t h8, h4, hm;
        memcpy(&h8, a + 32, 2); memcpy(&h4, w + 16, 2); memcpy(&hm, w + 18, 2);
        float d8 = orc_half_to_float_ftz(h8), d4 = orc_half_to_float_ftz(h4), dm = orc_half_to_float_ftz(hm);
        int s1 = 0, s2 = 0;
        for (int i = 0; i < 16; i++) {
          int q4 = w[i], lo = q4 & 15, hi = (q4 >> 4) & 15;
          int q8lo = (int8_t)a[2 * i], q8hi = (int8_t)a[2 * i + 1];
          s1 += lo * q8lo + hi * q8hi;
          s2 += q8lo + q8hi;
        }
        sum += d4 * d8 * (float)s1 + dm * d8 * (float)s2;
      }
      C[(int64_t)row * N + col] = sum;
    }
}

/* tests/test_q4k_pipeline.ts:111-116: C[i,j] = sum_k A[i,k]*B[k,j], int32. */
ORC_API void orc_i8_gemm(const int8_t* A, const int8_t* B, int32_t* C, int M, int N, int K) {
  for (int i = 0; i < M; i++)
    for (int j = 0; j < N; j++) {
      int32_t s = 0;
      for (int k = 0; k < K; k++) s += (int32_t)A[(int64_t)i * K + k] * (int32_t)B[(int64_t)k * N + j];
      C[(int64_t)i * N + j] = s;
    }
}

/* ------------------------------------------------------------------ */
/* 144-byte Q4_K super-block (ggml block_q4_K; not in the reference)    */
/* ------------------------------------------------------------------ */
/* layout: fp16 d @0, fp16 dmin @2, uint8 scales[12] @4, uint8 qs[128] @16.
 * ggml get_scale_min_k4: j<4: sc=scales[j]&63, m=scales[j+4]&63;
 * j>=4: sc=(scales[j+4]&15)|((scales[j-4]>>6)<<4), m=(scales[j+4]>>4)|((scales[j]>>6)<<4).
 * element e=64g+32h+l uses nibble h of qs[32g+l] and sub-block j=2g+h;
 * w_e = d*sc_j*nib - dmin*m_j. */

ORC_API void orc_q4k_unpack_scales(const uint8_t* scales, uint8_t* sc, uint8_t* m) {
  for (int j = 0; j < 8; j++) {
    if (j < 4) { sc[j] = scales[j] & 63; m[j] = scales[j + 4] & 63; }
    else {
      sc[j] = (uint8_t)((scales[j + 4] & 15) | ((scales[j - 4] >> 6) << 4));
      m[j] = (uint8_t)((scales[j + 4] >> 4) | ((scales[j] >> 6) << 4));
    }
  }
}

ORC_API void orc_q4k_pack_scales(const uint8_t* sc, const uint8_t* m, uint8_t* scales) {
  for (int j = 0; j < 4; j++) {
    scales[j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
    scales[j + 4] = (uint8_t)((m[j] & 63) | ((m[j + 4] >> 4) << 6));
    scales[j + 8] = (uint8_t)((sc[j + 4] & 15) | ((m[j + 4] & 15) << 4));
  }
}

/* nibbles in element order: out[256*b + e] in 0..15 */
ORC_API void orc_q4k_nibbles(const uint8_t* blocks, int64_t nblocks, uint8_t* out) {
  for (int64_t b = 0; b < nblocks; b++) {
    const uint8_t* qs = blocks + b * 144 + 16;
    for (int g = 0; g < 4; g++)
      for (int l = 0; l < 32; l++) {
        out[b * 256 + 64 * g + l] = qs[32 * g + l] & 15;
        out[b * 256 + 64 * g + 32 + l] = qs[32 * g + l] >> 4;
      }
  }
}

ORC_API void orc_q4k_dequant(const uint8_t* blocks, int64_t nblocks, float* out) {
  for (int64_t b = 0; b < nblocks; b++) {
    const uint8_t* blk = blocks + b * 144;
    uint16_t hd, hm; memcpy(&hd, blk, 2); memcpy(&hm, blk + 2, 2);
    float d = orc_half_to_float(hd), dmin = orc_half_to_float(hm);
    uint8_t sc[8], m[8]; orc_q4k_unpack_scales(blk + 4, sc, m);
    const uint8_t* qs = blk + 16;
    for (int g = 0; g < 4; g++)
      for (int l = 0; l < 32; l++) {
        float d0 = d * (float)sc[2 * g], m0 = dmin * (float)m[2 * g];
        float d1 = d * (float)sc[2 * g + 1], m1 = dmin * (float)m[2 * g + 1];
        out[b * 256 + 64 * g + l] = d0 * (float)(qs[32 * g + l] & 15) - m0;
        out[b * 256 + 64 * g + 32 + l] = d1 * (float)(qs[32 * g + l] >> 4) - m1;
      }
  }
}

/* ---- f32 weights -> Q4_K super-blocks ------------------------------- */
/* The reference quantizes weights only into its legacy 20-byte block
 * (packQ4_K_col, bench/bench.ts:74-96: per-32 min/max affine).  For the
 * 144-byte super-block the published algorithm is ggml's
 * quantize_row_q4_K_ref with make_qkx2_quants (ggml-quants.c; ggml is not a
 * dependency of the reference, so no version is pinned): per 32-element
 * sub-block a weighted least-squares fit of (scale, min) over 21 candidate
 * grids, weights av_x + |x|; then the 8 scales and 8 mins of a super-block are
 * quantized to 6 bits against their maxima, d and dmin stored as
 * round-to-nearest-even fp16, and the nibbles re-derived from the stored
 * (fp16, 6-bit) values.  All arithmetic is f32, one IEEE operation per written
 * operation, sums in ascending element order.
 * PARITY UNPINNED against ggml itself (absent here); pinned by invariants:
 * constant sub-blocks, exactly representable grids, fitted error <= min/max
 * grid error, and the reconstruction error bound. */

/* round to nearest, ties to even, of |v| <= 2^22 (ggml nearest_int) */
static inline int nearest_int_(float v) {
  float t = v + 12582912.f;
  int32_t i; memcpy(&i, &t, 4);
  return (i & 0x007fffff) - 0x00400000;
}

/* IEEE f32 -> fp16, round to nearest even, subnormals kept */
ORC_API uint16_t orc_f32_to_half_rne(float f) {
  uint32_t u = f2u(f), sign = (u >> 16) & 0x8000u;
  u &= 0x7fffffffu;
  if (u > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (u == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
  int e = (int)(u >> 23) - 127 + 15;
  if (e >= 31) return (uint16_t)(sign | 0x7c00u);
  if (e <= 0) {                                   /* |f| < 2^-14: multiples of 2^-24 */
    float scaled = u2f(u) * 16777216.0f;          /* exact scaling (or a flush of f32 denormals toward 0) */
    return (uint16_t)(sign | (uint32_t)lrintf(scaled));   /* default rounding mode = nearest even; 1024 = smallest normal */
  }
  uint32_t mant = u & 0x7fffffu, h = ((uint32_t)e << 10) | (mant >> 13), rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;    /* a carry runs into the exponent, up to Inf */
  return (uint16_t)(sign | h);
}

/* make_qkx2_quants(n=32, nmax=15, rmin=-1, rdelta=0.1, nstep=20, use_mad=false) */
static float qkx2_fit32_(const float* x, const float* weights, uint8_t* L, float* the_min) {
  const int n = 32, nmax = 15, nstep = 20;
  const float rmin = -1.f, rdelta = 0.1f;
  uint8_t Laux[32];
  float min = x[0], max = x[0];
  float sum_w = weights[0];
  float sum_x = sum_w * x[0];
  for (int i = 1; i < n; i++) {
    if (x[i] < min) min = x[i];
    if (x[i] > max) max = x[i];
    float w = weights[i];
    sum_w += w;
    sum_x += w * x[i];
  }
  if (min > 0) min = 0;
  if (max == min) {
    for (int i = 0; i < n; i++) L[i] = 0;
    *the_min = -min;
    return 0.f;
  }
  float iscale = (float)nmax / (max - min);
  float scale = 1 / iscale;
  float best = 0;
  for (int i = 0; i < n; i++) {
    int l = nearest_int_(iscale * (x[i] - min));
    l = l < 0 ? 0 : (l > nmax ? nmax : l);
    L[i] = (uint8_t)l;
    float diff = scale * (float)L[i] + min - x[i];
    diff = diff * diff;
    best += weights[i] * diff;
  }
  for (int is = 0; is <= nstep; is++) {
    iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
    float sum_l = 0, sum_l2 = 0, sum_xl = 0;
    for (int i = 0; i < n; i++) {
      int l = nearest_int_(iscale * (x[i] - min));
      l = l < 0 ? 0 : (l > nmax ? nmax : l);
      Laux[i] = (uint8_t)l;
      float w = weights[i];
      sum_l += w * (float)l;
      sum_l2 += w * (float)l * (float)l;
      sum_xl += w * (float)l * x[i];
    }
    float D = sum_w * sum_l2 - sum_l * sum_l;
    if (D > 0) {
      float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
      float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
      if (this_min > 0) {
        this_min = 0;
        this_scale = sum_xl / sum_l2;
      }
      float err = 0;
      for (int i = 0; i < n; i++) {
        float diff = this_scale * (float)Laux[i] + this_min - x[i];
        diff = diff * diff;
        err += weights[i] * diff;
      }
      if (err < best) {
        for (int i = 0; i < n; i++) L[i] = Laux[i];
        best = err;
        scale = this_scale;
        min = this_min;
      }
    }
  }
  *the_min = -min;
  return scale;
}

/* the fit alone, for the invariants that hold before the 6-bit step */
ORC_API float orc_qkx2_fit32(const float* x, const float* weights, uint8_t* L, float* the_min) {
  return qkx2_fit32_(x, weights, L, the_min);
}

/* x: n f32 values, n a multiple of 256; out: n/256 blocks of 144 bytes */
ORC_API void orc_quantize_q4k(const float* x, int64_t n, uint8_t* out) {
  int64_t nb = n / 256;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < nb; b++) {
    const float* xb = x + b * 256;
    uint8_t* blk = out + b * 144;
    uint8_t L[256];
    float weights[32], mins[8], scales[8];
    float max_scale = 0, max_min = 0;
    for (int j = 0; j < 8; j++) {
      float sum_x2 = 0;
      for (int l = 0; l < 32; l++) sum_x2 += xb[32 * j + l] * xb[32 * j + l];
      float av_x = sqrtf(sum_x2 / 32);
      for (int l = 0; l < 32; l++) weights[l] = av_x + fabsf(xb[32 * j + l]);
      scales[j] = qkx2_fit32_(xb + 32 * j, weights, L + 32 * j, &mins[j]);
      if (scales[j] > max_scale) max_scale = scales[j];
      if (mins[j] > max_min) max_min = mins[j];
    }
    float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    uint8_t sc[8], m[8];
    for (int j = 0; j < 8; j++) {
      uint8_t ls = (uint8_t)nearest_int_(inv_scale * scales[j]);
      uint8_t lm = (uint8_t)nearest_int_(inv_min * mins[j]);
      sc[j] = ls > 63 ? 63 : ls;
      m[j] = lm > 63 ? 63 : lm;
    }
    orc_q4k_pack_scales(sc, m, blk + 4);
    uint16_t hd = orc_f32_to_half_rne(max_scale / 63.f), hm = orc_f32_to_half_rne(max_min / 63.f);
    memcpy(blk, &hd, 2); memcpy(blk + 2, &hm, 2);
    for (int j = 0; j < 8; j++) {
      const float d = orc_half_to_float(hd) * (float)sc[j];
      if (!d) continue;
      const float dm = orc_half_to_float(hm) * (float)m[j];
      for (int i = 0; i < 32; i++) {
        int l = nearest_int_((xb[32 * j + i] + dm) / d);
        L[32 * j + i] = (uint8_t)(l < 0 ? 0 : (l > 15 ? 15 : l));
      }
    }
    for (int g = 0; g < 4; g++)
      for (int l = 0; l < 32; l++) blk[16 + 32 * g + l] = (uint8_t)(L[64 * g + l] | (L[64 * g + 32 + l] << 4));
  }
}

/* Dequantise-then-GEMV: y[n] = sum_k w[n,k]*x[k].  acc64=0: f32 accumulation
 * in ascending k (the straightforward host loop); acc64=1: double accumulation
 * of the same f32 products' exact values, rounded once. */
ORC_API void orc_gemv_q4k_f32(const uint8_t* W, const float* x, float* y, int N, int K, int acc64) {
  int nb = K / 256;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++) {
    float wrow[256];
    float accf = 0; double accd = 0;
    for (int b = 0; b < nb; b++) {
      orc_q4k_dequant(W + ((int64_t)n * nb + b) * 144, 1, wrow);
      const float* xb = x + b * 256;
      if (acc64) for (int e = 0; e < 256; e++) accd += (double)wrow[e] * (double)xb[e];
      else for (int e = 0; e < 256; e++) accf += wrow[e] * xb[e];
    }
    y[n] = acc64 ? (float)accd : accf;
  }
}

/* Integer sub-block dots I[n, K/32]: I_j = sum_l nib*q8 (int32). */
ORC_API void orc_q4k_q8_1_subdots(const uint8_t* W, const uint8_t* xq, int32_t* I, int N, int K) {
  int nb = K / 256;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++)
    for (int b = 0; b < nb; b++) {
      const uint8_t* qs = W + ((int64_t)n * nb + b) * 144 + 16;
      for (int j = 0; j < 8; j++) {
        const int8_t* q8 = (const int8_t*)(xq + (int64_t)(b * 8 + j) * 36);
        int g = j >> 1, h = j & 1;
        int32_t s = 0;
        for (int l = 0; l < 32; l++) {
          int nib = h ? (qs[32 * g + l] >> 4) : (qs[32 * g + l] & 15);
          s += nib * (int)q8[l];
        }
        I[(int64_t)n * (K / 32) + b * 8 + j] = s;
      }
    }
}

/* Q4_K x Q8_1 GEMV: y_n = sum_blk [ d*sum_j sc_j*(d8_j*I_j) - dmin*sum_j m_j*s8_j ].
 * The min term uses the STORED fp16 s of each Q8_1 block.  acc64 as above. */
ORC_API void orc_gemv_q4k_q8_1(const uint8_t* W, const uint8_t* xq, float* y, int N, int K, int acc64) {
  int nb = K / 256;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; n++) {
    float accf = 0; double accd = 0;
    for (int b = 0; b < nb; b++) {
      const uint8_t* blk = W + ((int64_t)n * nb + b) * 144;
      uint16_t hd, hm; memcpy(&hd, blk, 2); memcpy(&hm, blk + 2, 2);
      float d = orc_half_to_float(hd), dmin = orc_half_to_float(hm);
      uint8_t sc[8], m[8]; orc_q4k_unpack_scales(blk + 4, sc, m);
      const uint8_t* qs = blk + 16;
      float sf = 0, mf = 0; double sd = 0, md = 0;
      for (int j = 0; j < 8; j++) {
        const uint8_t* xb = xq + (int64_t)(b * 8 + j) * 36;
        const int8_t* q8 = (const int8_t*)xb;
        uint16_t h8, hs; memcpy(&h8, xb + 32, 2); memcpy(&hs, xb + 34, 2);
        float d8 = orc_half_to_float(h8), s8 = orc_half_to_float(hs);
        int g = j >> 1, h = j & 1;
        int32_t I = 0;
        for (int l = 0; l < 32; l++) {
          int nib = h ? (qs[32 * g + l] >> 4) : (qs[32 * g + l] & 15);
          I += nib * (int)q8[l];
        }
        if (acc64) { sd += (double)sc[j] * ((double)d8 * (double)I); md += (double)m[j] * (double)s8; }
        else { sf += (float)sc[j] * (d8 * (float)I); mf += (float)m[j] * s8; }
      }
      if (acc64) accd += (double)d * sd - (double)dmin * md;
      else accf += d * sf - dmin * mf;
    }
    y[n] = acc64 ? (float)accd : accf;
  }
}

/* ------------------------------------------------------------------ */
/* glue ops (bf16 I/O, f32 elementwise, double reductions)              */
/* ------------------------------------------------------------------ */

/* src/emitters.ts:31-45 embed: X[0:H] = E[token, :] (bf16 row copy). */
ORC_API void orc_embed(const uint16_t* E, int32_t token, uint16_t* out, int H) {
  memcpy(out, E + (int64_t)token * H, (size_t)H * 2);
}

/* src/fusion.ts:310-322 emitRmsNorm: y = bf16((x*rsqrt(mean(x^2)+1e-6))*(1+w)). */
ORC_API void orc_rmsnorm(const uint16_t* x, const uint16_t* w, uint16_t* out, int N) {
  double ss = 0;
  for (int i = 0; i < N; i++) { float v = BF(x[i]); ss += (double)v * (double)v; }
  float rstd = rsqrt_(ss / (double)N + 1e-6);
  for (int i = 0; i < N; i++) {
    float y = BF(x[i]) * rstd;
    out[i] = TOBF(y * (1.0f + BF(w[i])));
  }
}

/* src/fusion.ts:295-299 emitCast (to bf16). */
ORC_API void orc_cast_bf16(const float* x, uint16_t* out, int N) {
  for (int i = 0; i < N; i++) out[i] = TOBF(x[i]);
}

/* src/fusion.ts:301-308 emitAdd: bf16(f32(a)+f32(b)). */
ORC_API void orc_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out, int N) {
  for (int i = 0; i < N; i++) out[i] = TOBF(BF(a[i]) + BF(b[i]));
}


/* src/fusion.ts:324-330 emitSwiGLU: bf16((g*(1/(1+exp(-g))))*u), g,u f32. */
ORC_API void orc_swiglu(const float* g, const float* u, uint16_t* out, int N) {
  for (int i = 0; i < N; i++) out[i] = TOBF((g[i] * sigmoidf_(g[i])) * u[i]);
}

/* src/emitters.ts:48-72 emitConv1d: r=(w0*s0+w1*s1)+(w2*s2+w3*x);
 * out=bf16(r*sigmoid(r)); new state rows = (s1, s2, x). weight [C,4] bf16. */
ORC_API void orc_conv1d_decode(const uint16_t* x, const uint16_t* st, const uint16_t* w,
                               uint16_t* out, uint16_t* st_new, int C) {
  for (int c = 0; c < C; c++) {
    float xv = BF(x[c]), s0 = BF(st[c]), s1 = BF(st[C + c]), s2 = BF(st[2 * C + c]);
    float w0 = BF(w[4 * c]), w1 = BF(w[4 * c + 1]), w2 = BF(w[4 * c + 2]), w3 = BF(w[4 * c + 3]);
    float r = (w0 * s0 + w1 * s1) + (w2 * s2 + w3 * xv);
    out[c] = TOBF(r * sigmoidf_(r));
    st_new[c] = st[C + c]; st_new[C + c] = st[2 * C + c]; st_new[2 * C + c] = x[c];
  }
}

/* src/emitters.ts:123-147 emitQNorm / emitKNorm: per-head
 * bf16((x*rsqrt(mean(x^2)+1e-6))*(1+w)); the input row stride per head is
 * in_stride elements (2*HD for the interleaved [q,gate] buffer, HD for k). */
ORC_API void orc_headnorm(const uint16_t* x, const uint16_t* w, uint16_t* out,
                          int nheads, int HD, int in_stride) {
  for (int h = 0; h < nheads; h++) {
    const uint16_t* xh = x + (int64_t)h * in_stride;
    double ss = 0;
    for (int i = 0; i < HD; i++) { float v = BF(xh[i]); ss += (double)v * (double)v; }
    float rstd = rsqrt_(ss / (double)HD + 1e-6);
    for (int i = 0; i < HD; i++)
      out[(int64_t)h * HD + i] = TOBF((BF(xh[i]) * rstd) * (1.0f + BF(w[i])));
  }
}

/* prototypes/decode.ts:865-871 rope tables: f_i = 1/pow(theta, 2i/rot_dim),
 * cos/sin evaluated in double, stored f32, layout [max_len, rot_dim/2]. */
ORC_API void orc_rope_tables(float* cos_t, float* sin_t, int max_len, int rot_dim, double theta) {
  int half = rot_dim / 2;
  for (int p = 0; p < max_len; p++)
    for (int i = 0; i < half; i++) {
      double f = 1.0 / pow(theta, 2.0 * i / rot_dim);
      cos_t[(int64_t)p * half + i] = (float)cos(p * f);
      sin_t[(int64_t)p * half + i] = (float)sin(p * f);
    }
}

/* src/emitters.ts:150-183 emitRoPE/emitRoPEK: in place, pairs (i, i+half) of
 * the first 2*half dims of every head: x1'=x1*c-x2*s, x2'=x2*c+x1*s. */
ORC_API void orc_rope(uint16_t* x, const float* cos_t, const float* sin_t, int pos,
                      int nheads, int HD, int half) {
  for (int h = 0; h < nheads; h++)
    for (int i = 0; i < half; i++) {
      uint16_t* p1 = x + (int64_t)h * HD + i; uint16_t* p2 = p1 + half;
      float x1 = BF(*p1), x2 = BF(*p2);
      float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
      *p1 = TOBF(x1 * c - x2 * s);
      *p2 = TOBF(x2 * c + x1 * s);
    }
}

/* prototypes/decode.ts:746-791 two-stage argmax, equivalent to one strict ">"
 * scan in ascending index from -FLT_MAX: lowest index wins ties, NaN never wins. */
ORC_API void orc_argmax(const float* logits, int64_t n, float* val, int32_t* idx) {
  float best = -3.40282347e38f; int32_t bi = 0;
  for (int64_t i = 0; i < n; i++) if (logits[i] > best) { best = logits[i]; bi = (int32_t)i; }
  *val = best; *idx = bi;
}

/* ------------------------------------------------------------------ */
/* gated DeltaNet single-token step                                     */
/* ------------------------------------------------------------------ */
/* src/emitters.ts:75-120 emitGDN (== prototypes/decode.ts:314-388), one head
 * at a time.  conv_out holds [q(Hg*dk) | k(Hg*dk) | v(Hg*dv)] bf16.
 *   q^ = q*rsqrt(sum q^2 + 1e-6)*dk^-1/2 ;  k^ = k*rsqrt(sum k^2 + 1e-6)
 *   g = exp(-exp(A_log)*softplus(a+dt_bias)), softplus = ln(1+e^x)
 *   beta = 1/(1+exp(-b))
 *   Sd = g*S ; kS[v] = sum_k k^[k]*Sd[k,v] ; delta = (v-kS)*beta
 *   S' = Sd + k^ (x) delta ; o[v] = sum_k q^[k]*S'[k,v]
 *   out = bf16( o*rsqrt(mean(o^2)+1e-6) * norm_w * (z*sigmoid(z)) )
 * S is [Hg, dk, dv] f32 row-major.  dk must equal dv (the reference reads v
 * with the key tile shape).  rows_per_chain: 16 = canonical f32 order of the
 * two k-reductions, 0 = double accumulation. */
ORC_API void orc_gdn_step(const uint16_t* conv_out, const uint16_t* z, const float* A_log,
                          const uint16_t* dt_bias, const float* a_p, const float* b_p,
                          const float* norm_w, const float* S_in, uint16_t* out, float* S_out,
                          int Hg, int dk, int dv, int rows_per_chain) {
  int KEYDIM = Hg * dk;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < Hg; h++) {
    float* qn = (float*)malloc(sizeof(float) * (size_t)(2 * dk + 3 * dv));
    float *kn = qn + dk, *vv = kn + dk, *delta = vv + dv, *o = delta + dv;
    double sq = 0, sk = 0;
    for (int i = 0; i < dk; i++) {
      float q = BF(conv_out[h * dk + i]), k = BF(conv_out[KEYDIM + h * dk + i]);
      sq += (double)q * q; sk += (double)k * k;
    }
    float qr = rsqrt_(sq + 1e-6), kr = rsqrt_(sk + 1e-6);
    float qscale = qr * (float)(1.0 / sqrt((double)dk));
    for (int i = 0; i < dk; i++) {
      qn[i] = BF(conv_out[h * dk + i]) * qscale;
      kn[i] = BF(conv_out[KEYDIM + h * dk + i]) * kr;
    }
    for (int i = 0; i < dv; i++) vv[i] = BF(conv_out[2 * KEYDIM + h * dv + i]);
    float sp_in = a_p[h] + BF(dt_bias[h]);
    float softplus = (float)log1p(exp((double)sp_in));
    float decay = (float)exp(-(double)((float)exp((double)A_log[h]) * softplus));
    float beta = sigmoidf_(b_p[h]);
    const float* S = S_in + (int64_t)h * dk * dv;
    float* Sn = S_out + (int64_t)h * dk * dv;
    for (int v = 0; v < dv; v++) {
      float kS;
      if (rows_per_chain > 0) {
        kS = 0.0f;
        for (int k0 = 0; k0 < dk; k0 += rows_per_chain) {
          float acc = 0.0f;
          for (int k = k0; k < k0 + rows_per_chain; k++) acc = fmaf(kn[k], S[k * dv + v] * decay, acc);
          kS += acc;
        }
      } else {
        double acc = 0;
        for (int k = 0; k < dk; k++) acc += (double)kn[k] * (double)(S[k * dv + v] * decay);
        kS = (float)acc;
      }
      delta[v] = (vv[v] - kS) * beta;
    }
    for (int k = 0; k < dk; k++)
      for (int v = 0; v < dv; v++) Sn[k * dv + v] = fmaf(kn[k], delta[v], S[k * dv + v] * decay);
    double oss = 0;
    for (int v = 0; v < dv; v++) {
      if (rows_per_chain > 0) {
        float ov = 0.0f;
        for (int k0 = 0; k0 < dk; k0 += rows_per_chain) {
          float acc = 0.0f;
          for (int k = k0; k < k0 + rows_per_chain; k++) acc = fmaf(qn[k], Sn[k * dv + v], acc);
          ov += acc;
        }
        o[v] = ov;
      } else {
        double acc = 0;
        for (int k = 0; k < dk; k++) acc += (double)qn[k] * (double)Sn[k * dv + v];
        o[v] = (float)acc;
      }
      oss += (double)o[v] * o[v];
    }
    float orstd = rsqrt_(oss / (double)dv + 1e-6);
    for (int v = 0; v < dv; v++) {
      float zv = BF(z[h * dv + v]);
      float zs = zv * sigmoidf_(zv);
      out[h * dv + v] = TOBF(((o[v] * orstd) * norm_w[v]) * zs);
    }
    free(qn);
  }
}

/* Core recurrence only (prototypes/gdn_gated.ts:67-88 refGDN at T=1, with the
 * delta-rule beta of src/emitters.ts:105): q,k already L2-normalised bf16,
 * no 1/sqrt(dk), g is the log-decay (S scaled by exp(g)), beta given, o -> bf16.
 *   S' = exp(g)*S + k (x) ((v - (exp(g)*S)^T k)*beta) ; o = S'^T q */
ORC_API void orc_gdn_core(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                          const float* g, const float* beta, const float* S_in,
                          uint16_t* out, float* S_out, int Hg, int dk, int dv) {
#pragma omp parallel for schedule(static)
  for (int h = 0; h < Hg; h++) {
    float decay = (float)exp((double)g[h]);
    const float* S = S_in + (int64_t)h * dk * dv;
    float* Sn = S_out + (int64_t)h * dk * dv;
    float* delta = (float*)malloc(sizeof(float) * (size_t)dv);
    for (int j = 0; j < dv; j++) {
      double acc = 0;
      for (int i = 0; i < dk; i++) acc += (double)BF(k[h * dk + i]) * (double)(S[i * dv + j] * decay);
      delta[j] = (BF(v[h * dv + j]) - (float)acc) * beta[h];
    }
    for (int i = 0; i < dk; i++)
      for (int j = 0; j < dv; j++) Sn[i * dv + j] = fmaf(BF(k[h * dk + i]), delta[j], S[i * dv + j] * decay);
    for (int j = 0; j < dv; j++) {
      double acc = 0;
      for (int i = 0; i < dk; i++) acc += (double)BF(q[h * dk + i]) * (double)Sn[i * dv + j];
      out[h * dv + j] = TOBF((float)acc);
    }
    free(delta);
  }
}

/* ------------------------------------------------------------------ */
/* decode attention over a paged bf16 GQA KV cache                      */
/* ------------------------------------------------------------------ */
/* Math of src/emitters.ts:188-226 emitFA2Attn (scores*1/sqrt(HD) over the
 * valid prefix, softmax, sum p*V, optional *sigmoid(gate)) and
 * prototypes/fa2_vllm.ts:114-139 refAttn, over this build's cache layout:
 * page p holds [kv_head][page_size][HD] bf16, one array for K and one for V;
 * block_table[b, i] names the page of tokens [i*page_size, (i+1)*page_size).
 * Also returns lse = m + ln(sum exp(s-m)) per (batch, q head).
 * gate (may be NULL): bf16, gate for q head h of batch b at
 * gate[b*gate_bstride + h*gate_hstride + i]. */
ORC_API void orc_attn_decode_paged(const uint16_t* q, const uint16_t* kc, const uint16_t* vc,
                                   const int32_t* block_table, int bt_stride, const int32_t* ctx_len,
                                   const uint16_t* gate, int gate_bstride, int gate_hstride,
                                   uint16_t* out, float* lse, int B, int NH, int NKV, int HD,
                                   int page_size) {
  int G = NH / NKV;
  double scale = 1.0 / sqrt((double)HD);
#pragma omp parallel for schedule(dynamic) collapse(2)
  for (int b = 0; b < B; b++)
    for (int h = 0; h < NH; h++) {
      int len = ctx_len[b], kv = h / G;
      const uint16_t* qh = q + ((int64_t)b * NH + h) * HD;
      double* s = (double*)malloc(sizeof(double) * (size_t)(len + HD));
      double* acc = s + len;
      double m = -INFINITY;
      for (int t = 0; t < len; t++) {
        int page = block_table[(int64_t)b * bt_stride + t / page_size];
        const uint16_t* kr = kc + (((int64_t)page * NKV + kv) * page_size + t % page_size) * HD;
        double d = 0;
        for (int i = 0; i < HD; i++) d += (double)BF(qh[i]) * (double)BF(kr[i]);
        s[t] = d * scale; if (s[t] > m) m = s[t];
      }
      double l = 0;
      for (int i = 0; i < HD; i++) acc[i] = 0;
      for (int t = 0; t < len; t++) {
        int page = block_table[(int64_t)b * bt_stride + t / page_size];
        const uint16_t* vr = vc + (((int64_t)page * NKV + kv) * page_size + t % page_size) * HD;
        double p = exp(s[t] - m); l += p;
        for (int i = 0; i < HD; i++) acc[i] += p * (double)BF(vr[i]);
      }
      for (int i = 0; i < HD; i++) {
        float o = (float)(acc[i] / l);
        if (gate) {
          float gv = BF(gate[(int64_t)b * gate_bstride + (int64_t)h * gate_hstride + i]);
          o = o * sigmoidf_(gv);
        }
        out[((int64_t)b * NH + h) * HD + i] = TOBF(o);
      }
      if (lse) lse[(int64_t)b * NH + h] = (float)(m + log(l));
      free(s);
    }
}

/* Write one token's k and v (bf16 [NKV, HD]) into the paged cache at position pos
 * (the cache write that emitFA2Attn does before scoring, src/emitters.ts:202-205). */
ORC_API void orc_kv_append(const uint16_t* k, const uint16_t* v, uint16_t* kc, uint16_t* vc,
                           const int32_t* block_table, int pos, int NKV, int HD, int page_size) {
  int page = block_table[pos / page_size];
  for (int kv = 0; kv < NKV; kv++) {
    int64_t off = (((int64_t)page * NKV + kv) * page_size + pos % page_size) * HD;
    memcpy(kc + off, k + (int64_t)kv * HD, (size_t)HD * 2);
    memcpy(vc + off, v + (int64_t)kv * HD, (size_t)HD * 2);
  }
}
