// Weight quantizer: f32 / bf16 rows -> 144-byte Q4_K super-blocks, on the device, at model load.
//
// The reference packs weights only into its legacy 20-byte block (packQ4_K_col, bench/bench.ts:74-96).  The
// super-block's published quantizer is ggml's quantize_row_q4_K_ref (make_qkx2_quants with nmax 15, rmin -1,
// rdelta 0.1, 20 steps, squared error, weights av_x + |x|): a weighted least-squares fit of (scale, min) per
// 32-element sub-block over 21 candidate grids, 6-bit quantization of the 8 scales and 8 mins against their
// maxima, fp16 (nearest-even) d and dmin, nibbles re-derived from the stored values.
//
// One lane per sub-block: the fit is a chain of f32 sums in ascending element order, so a lane runs it exactly
// as the host loop does (one IEEE operation per written operation) and the bytes equal the host's.  The eight
// lanes of a super-block meet only for the two maxima (order-free), the 12 scale bytes (an OR) and the nibble
// pairing of sub-blocks 2g and 2g+1.  The work is ALU-bound (about 13 thousand operations per sub-block), not
// memory-bound: a load-time kernel, not part of the decode step.
#include "ops.h"

namespace bk {

// ggml nearest_int: round to nearest even for |v| <= 2^22
__device__ __forceinline__ int nearest_int(float v) {
  const float t = __fadd_rn(v, 12582912.f);
  return (int)(__float_as_uint(t) & 0x007fffffu) - 0x00400000;
}
__device__ __forceinline__ int clamp_i(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }
__device__ __forceinline__ uint16_t f32_to_half_rne(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

// 4 nibbles (16 bits) -> 4 bytes
__device__ __forceinline__ uint32_t spread4(uint32_t h) {
  h &= 0xffffu;
  h = (h | (h << 8)) & 0x00ff00ffu;
  return (h | (h << 4)) & 0x0f0f0f0fu;
}

template <bool BF16>
__global__ __launch_bounds__(256) void quantize_q4k_kernel(const void* __restrict__ src, uint8_t* __restrict__ out,
                                                           int64_t nsub) {
  constexpr int NMAX = 15, NSTEP = 20;
  const int64_t sub_raw = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool live = sub_raw < nsub;                 // nsub is a multiple of 8: a super-block's lanes are all live or all not
  const int64_t sub = live ? sub_raw : nsub - 1;
  const int j = threadIdx.x & 7;

  float x[32];
  if (BF16) {
    const uint4* p = (const uint4*)src + sub * 4;
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const uint4 v = p[t];
      const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; k++) {
        x[8 * t + 2 * k] = __uint_as_float(u[k] << 16);
        x[8 * t + 2 * k + 1] = __uint_as_float(u[k] & 0xffff0000u);
      }
    }
  } else {
    const float4* p = (const float4*)src + sub * 8;
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const float4 v = p[t];
      x[4 * t] = v.x; x[4 * t + 1] = v.y; x[4 * t + 2] = v.z; x[4 * t + 3] = v.w;
    }
  }

  // ---- weights and the sums that do not depend on the grid
  float sum_x2 = 0.f;
#pragma unroll
  for (int i = 0; i < 32; i++) sum_x2 = __fadd_rn(sum_x2, __fmul_rn(x[i], x[i]));
  // sqrtf is the correctly rounded square root (the _rn intrinsic of this toolchain is the approximate one)
  const float av_x = sqrtf(__fdiv_rn(sum_x2, 32.f));
  float w[32];
#pragma unroll
  for (int i = 0; i < 32; i++) w[i] = __fadd_rn(av_x, fabsf(x[i]));

  float mn = x[0], mx = x[0];
  float sum_w = w[0];
  float sum_x = __fmul_rn(sum_w, x[0]);
#pragma unroll
  for (int i = 1; i < 32; i++) {
    if (x[i] < mn) mn = x[i];
    if (x[i] > mx) mx = x[i];
    sum_w = __fadd_rn(sum_w, w[i]);
    sum_x = __fadd_rn(sum_x, __fmul_rn(w[i], x[i]));
  }
  if (mn > 0.f) mn = 0.f;

  uint32_t Lp[4] = {0u, 0u, 0u, 0u};            // nibble i & 7 of Lp[i >> 3] = L[i]
  float scale = 0.f;
  if (!(mx == mn)) {
    float iscale = __fdiv_rn((float)NMAX, __fsub_rn(mx, mn));
    scale = __fdiv_rn(1.f, iscale);
    float best = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const int l = clamp_i(nearest_int(__fmul_rn(iscale, __fsub_rn(x[i], mn))), 0, NMAX);
      Lp[i >> 3] |= (uint32_t)l << (4 * (i & 7));
      float diff = __fsub_rn(__fadd_rn(__fmul_rn(scale, (float)l), mn), x[i]);
      diff = __fmul_rn(diff, diff);
      best = __fadd_rn(best, __fmul_rn(w[i], diff));
    }
    // as published, a candidate grid starts at the current best min (the fitted one once a candidate has won)
#pragma unroll 1
    for (int is = 0; is <= NSTEP; is++) {
      iscale = __fdiv_rn(__fadd_rn(__fadd_rn(-1.f, __fmul_rn(0.1f, (float)is)), (float)NMAX), __fsub_rn(mx, mn));
      float sum_l = 0.f, sum_l2 = 0.f, sum_xl = 0.f;
      float lf[32];
      uint32_t Ap[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int i = 0; i < 32; i++) {
        const int l = clamp_i(nearest_int(__fmul_rn(iscale, __fsub_rn(x[i], mn))), 0, NMAX);
        Ap[i >> 3] |= (uint32_t)l << (4 * (i & 7));
        lf[i] = (float)l;
        const float wl = __fmul_rn(w[i], lf[i]);
        sum_l = __fadd_rn(sum_l, wl);
        sum_l2 = __fadd_rn(sum_l2, __fmul_rn(wl, lf[i]));
        sum_xl = __fadd_rn(sum_xl, __fmul_rn(wl, x[i]));
      }
      const float D = __fsub_rn(__fmul_rn(sum_w, sum_l2), __fmul_rn(sum_l, sum_l));
      if (D > 0.f) {
        float this_scale = __fdiv_rn(__fsub_rn(__fmul_rn(sum_w, sum_xl), __fmul_rn(sum_x, sum_l)), D);
        float this_min = __fdiv_rn(__fsub_rn(__fmul_rn(sum_l2, sum_x), __fmul_rn(sum_l, sum_xl)), D);
        if (this_min > 0.f) {
          this_min = 0.f;
          this_scale = __fdiv_rn(sum_xl, sum_l2);
        }
        float err = 0.f;
#pragma unroll
        for (int i = 0; i < 32; i++) {
          float diff = __fsub_rn(__fadd_rn(__fmul_rn(this_scale, lf[i]), this_min), x[i]);
          diff = __fmul_rn(diff, diff);
          err = __fadd_rn(err, __fmul_rn(w[i], diff));
        }
        if (err < best) {
#pragma unroll
          for (int t = 0; t < 4; t++) Lp[t] = Ap[t];
          best = err;
          scale = this_scale;
          mn = this_min;
        }
      }
    }
  }
  const float the_min = -mn;

  // ---- the super-block: 8 lanes
  float max_scale = scale > 0.f ? scale : 0.f, max_min = the_min > 0.f ? the_min : 0.f;
  max_scale = fmaxf(max_scale, dpp_f32<DPP_QUAD_XOR1>(max_scale));
  max_scale = fmaxf(max_scale, dpp_f32<DPP_QUAD_XOR2>(max_scale));
  max_scale = fmaxf(max_scale, dpp_f32<DPP_ROW_HALF_MIRROR>(max_scale));
  max_min = fmaxf(max_min, dpp_f32<DPP_QUAD_XOR1>(max_min));
  max_min = fmaxf(max_min, dpp_f32<DPP_QUAD_XOR2>(max_min));
  max_min = fmaxf(max_min, dpp_f32<DPP_ROW_HALF_MIRROR>(max_min));
  const float inv_scale = max_scale > 0.f ? __fdiv_rn(63.f, max_scale) : 0.f;
  const float inv_min = max_min > 0.f ? __fdiv_rn(63.f, max_min) : 0.f;
  uint32_t ls = (uint32_t)nearest_int(__fmul_rn(inv_scale, scale)) & 0xffu;       // the uint8_t of the host loop
  uint32_t lm = (uint32_t)nearest_int(__fmul_rn(inv_min, the_min)) & 0xffu;
  ls = ls > 63u ? 63u : ls;
  lm = lm > 63u ? 63u : lm;
  const uint16_t hd = f32_to_half_rne(__fdiv_rn(max_scale, 63.f)), hm = f32_to_half_rne(__fdiv_rn(max_min, 63.f));

  const float d = __fmul_rn(half_to_f32(hd), (float)ls);
  if (d != 0.f) {
    const float dm = __fmul_rn(half_to_f32(hm), (float)lm);
#pragma unroll
    for (int t = 0; t < 4; t++) Lp[t] = 0u;
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const int l = clamp_i(nearest_int(__fdiv_rn(__fadd_rn(x[i], dm), d)), 0, 15);
      Lp[i >> 3] |= (uint32_t)l << (4 * (i & 7));
    }
  }

  // 12 scale bytes: every lane ORs in its own bits
  const int sh = 8 * (j & 3);
  uint32_t w0, w1, w2;
  if (j < 4) { w0 = ls << sh; w1 = lm << sh; w2 = 0u; }
  else { w0 = ((ls >> 4) << 6) << sh; w1 = ((lm >> 4) << 6) << sh; w2 = ((ls & 15u) | ((lm & 15u) << 4)) << sh; }
  w0 |= (uint32_t)dpp_i32<DPP_QUAD_XOR1>((int)w0); w0 |= (uint32_t)dpp_i32<DPP_QUAD_XOR2>((int)w0);
  w0 |= (uint32_t)dpp_i32<DPP_ROW_HALF_MIRROR>((int)w0);
  w1 |= (uint32_t)dpp_i32<DPP_QUAD_XOR1>((int)w1); w1 |= (uint32_t)dpp_i32<DPP_QUAD_XOR2>((int)w1);
  w1 |= (uint32_t)dpp_i32<DPP_ROW_HALF_MIRROR>((int)w1);
  w2 |= (uint32_t)dpp_i32<DPP_QUAD_XOR1>((int)w2); w2 |= (uint32_t)dpp_i32<DPP_QUAD_XOR2>((int)w2);
  w2 |= (uint32_t)dpp_i32<DPP_ROW_HALF_MIRROR>((int)w2);

  // byte l of group g = L[2g][l] | L[2g+1][l] << 4: the pair exchanges its nibbles, each lane stores 16 bytes
  uint32_t other[4];
#pragma unroll
  for (int t = 0; t < 4; t++) other[t] = (uint32_t)dpp_i32<DPP_QUAD_XOR1>((int)Lp[t]);
  const bool odd = j & 1;
  uint32_t q[4];
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const int e = (odd ? 16 : 0) + 4 * t;                          // first of the four elements of this dword
    const uint32_t lo = (odd ? other[e >> 3] : Lp[e >> 3]) >> (4 * (e & 7));
    const uint32_t hi = (odd ? Lp[e >> 3] : other[e >> 3]) >> (4 * (e & 7));
    q[t] = spread4(lo) | (spread4(hi) << 4);
  }
  if (live) {
    uint8_t* blk = out + (sub >> 3) * 144;
    *(uint4*)(blk + 16 + 32 * (j >> 1) + (odd ? 16 : 0)) = make_uint4(q[0], q[1], q[2], q[3]);
    if (j == 0) *(uint4*)blk = make_uint4((uint32_t)hd | ((uint32_t)hm << 16), w0, w1, w2);
  }
}

int launch_quantize_q4k(const void* w, int w_dtype, void* out, int64_t rows, int K) {
  BK_REQUIRE(w && out, "quantize_q4k: null pointer");
  BK_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "quantize_q4k: w_dtype must be 0 (f32) or 1 (bf16)");
  BK_REQUIRE(rows > 0 && K > 0 && K % 256 == 0, "quantize_q4k: rows=%lld K=%d: K must be a positive multiple of 256",
             (long long)rows, K);
  BK_REQUIRE(((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0, "quantize_q4k: pointers must be 16-byte aligned");
  const int64_t nsub = rows * (K / 32);
  const int64_t wgs = (nsub + 255) / 256;
  BK_REQUIRE(wgs <= 0x7fffffff, "quantize_q4k: too many elements for one launch");
  if (w_dtype == DT_BF16) hipLaunchKernelGGL(quantize_q4k_kernel<true>, dim3((unsigned)wgs), dim3(256), 0, stream(), w, (uint8_t*)out, nsub);
  else hipLaunchKernelGGL(quantize_q4k_kernel<false>, dim3((unsigned)wgs), dim3(256), 0, stream(), w, (uint8_t*)out, nsub);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
