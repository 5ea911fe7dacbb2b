// Q8_1 activation quantizer and the nibble dequant kernels.
#include "ops.h"

namespace bk {

// ---------------------------------------------------------------- Q8_1
// One 32-lane half-wave per Q8_1 block, one element per lane.  Follows
// packQ8_1 (bench/bench.ts:53-72): d = amax/127 and the quotient x/d are
// evaluated in double, rounding is "nearest, ties toward +infinity"
// (ECMAScript Math.round), s = trunc16(float(sum(q) * d)) with the unrounded d.
template <int XDT>
__global__ __launch_bounds__(256) void quantize_q8_1_kernel(const void* __restrict__ xin,
                                                            uint8_t* __restrict__ out, int K, int nblk) {
  const int l = threadIdx.x & 31;
  const int blk = blockIdx.x * 8 + (threadIdx.x >> 5);
  const int row = blockIdx.y;
  const int e = blk * 32 + l;
  float v = 0.0f;
  if (blk < nblk && e < K) {
    if (XDT == DT_F32) v = ((const float*)xin)[(int64_t)row * K + e];
    else v = bf16_to_f32(((const uint16_t*)xin)[(int64_t)row * K + e]);
  }
  float amax = row16_max(fabsf(v));
  amax = fmaxf(amax, __shfl_xor(amax, 16));
  const double d = div127_f64((double)amax);
  int q = q8_1_round(v, q8_1_inv(amax), d != 0.0 ? d : 1.0);
  int sum = row16_sum_i32(q);
  sum += __shfl_xor(sum, 16);
  q = q < -128 ? -128 : (q > 127 ? 127 : q);
  if (blk < nblk) {
    uint8_t* o = out + ((int64_t)row * nblk + blk) * 36;
    o[l] = (uint8_t)(int8_t)q;
    if (l == 0) {
      uint16_t hd = f32_to_half_trunc((float)d);
      uint16_t hs = f32_to_half_trunc((float)((double)sum * d));
      *(uint32_t*)(o + 32) = (uint32_t)hd | ((uint32_t)hs << 16);
    }
  }
}

int launch_quantize_q8_1(const void* x, int x_dtype, void* out, int K, int batch) {
  BK_REQUIRE(x && out, "quantize_q8_1: null pointer");
  BK_REQUIRE(K > 0 && batch > 0 && batch <= 65535, "quantize_q8_1: bad K=%d batch=%d", K, batch);
  BK_REQUIRE(x_dtype == DT_F32 || x_dtype == DT_BF16, "quantize_q8_1: x_dtype must be 0 (f32) or 1 (bf16)");
  const int nblk = (K + 31) / 32;
  dim3 grid((nblk + 7) / 8, batch);
  if (x_dtype == DT_F32)
    hipLaunchKernelGGL(quantize_q8_1_kernel<DT_F32>, grid, dim3(256), 0, stream(), x, (uint8_t*)out, K, nblk);
  else
    hipLaunchKernelGGL(quantize_q8_1_kernel<DT_BF16>, grid, dim3(256), 0, stream(), x, (uint8_t*)out, K, nblk);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- legacy 20-byte block
// tests/test_dequant.ts:13-24: byte j -> elements 2j (low nibble - 8), 2j+1 (high - 8).
// One thread per input dword (4 bytes -> 8 int8 outputs).
__global__ __launch_bounds__(256) void dequant_legacy_i8_kernel(const uint32_t* __restrict__ in,
                                                                uint2* __restrict__ out, int64_t ndw) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= ndw) return;
  const int64_t blk = t >> 2;
  const int j = (int)(t & 3);
  const uint32_t q = in[blk * 5 + j];
  uint32_t lo = q & 0x0f0f0f0fu, hi = (q >> 4) & 0x0f0f0f0fu;
  // interleave bytes: out = [lo0,hi0,lo1,hi1 | lo2,hi2,lo3,hi3], then subtract 8 per byte
  uint32_t a = (lo & 0xffu) | ((hi & 0xffu) << 8) | ((lo & 0xff00u) << 8) | ((hi & 0xff00u) << 16);
  uint32_t b = ((lo >> 16) & 0xffu) | (((hi >> 16) & 0xffu) << 8) | (((lo >> 16) & 0xff00u) << 8) |
               (((hi >> 16) & 0xff00u) << 16);
  // per-byte (v - 8) without borrow between bytes: v in 0..15, so (v + 0xf8) & 0xff
  a = ((a + 0x78787878u) ^ 0x80808080u);
  b = ((b + 0x78787878u) ^ 0x80808080u);
  out[blk * 4 + j] = make_uint2(a, b);
}

int launch_dequant_legacy_i8(const void* blocks, void* out, int64_t nblocks) {
  BK_REQUIRE(blocks && out, "dequant_legacy_i8: null pointer");
  BK_REQUIRE(nblocks > 0 && nblocks < ((int64_t)1 << 36), "dequant_legacy_i8: bad nblocks");
  const int64_t ndw = nblocks * 4;
  hipLaunchKernelGGL(dequant_legacy_i8_kernel, dim3((unsigned)((ndw + 255) / 256)), dim3(256), 0, stream(),
                     (const uint32_t*)blocks, (uint2*)out, ndw);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- 144-byte super-block
struct Q4KScales { uint32_t sc[8], m[8]; };

// 6-bit scale/min j of a block whose scales bytes 0..11 are s0|s1|s2 (little-endian dwords).
__device__ __forceinline__ void q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j, uint32_t& sc, uint32_t& m) {
  const int sh = 8 * (j & 3);
  if (j < 4) {
    sc = (s0 >> sh) & 63u;
    m = (s1 >> sh) & 63u;
  } else {
    const uint32_t t = (s2 >> sh) & 0xffu;
    sc = (t & 15u) | (((s0 >> (sh + 6)) & 3u) << 4);
    m = (t >> 4) | (((s1 >> (sh + 6)) & 3u) << 4);
  }
}

// One thread per qs dword: 4 low nibbles -> sub-block 2g, 4 high nibbles -> sub-block 2g+1.
template <bool F32OUT>
__global__ __launch_bounds__(256) void q4k_unpack_kernel(const uint32_t* __restrict__ in, void* __restrict__ out,
                                                         int64_t ndw) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= ndw) return;
  const int64_t blk = t >> 5;
  const int i = (int)(t & 31), g = i >> 3, l0 = (i & 7) * 4;
  const uint32_t* b = in + blk * 36;
  const uint32_t q = b[4 + i];
  const uint32_t lo = q & 0x0f0f0f0fu, hi = (q >> 4) & 0x0f0f0f0fu;
  if (!F32OUT) {
    uint32_t* o = (uint32_t*)out + blk * 64;
    o[16 * g + (l0 >> 2)] = lo;
    o[16 * g + 8 + (l0 >> 2)] = hi;
  } else {
    const uint32_t hdr = b[0];
    const float d = half_to_f32((uint16_t)(hdr & 0xffffu)), dmin = half_to_f32((uint16_t)(hdr >> 16));
    uint32_t sc0, m0, sc1, m1;
    q4k_scale_min(b[1], b[2], b[3], 2 * g, sc0, m0);
    q4k_scale_min(b[1], b[2], b[3], 2 * g + 1, sc1, m1);
    const float d0 = __fmul_rn(d, (float)sc0), mm0 = __fmul_rn(dmin, (float)m0);
    const float d1 = __fmul_rn(d, (float)sc1), mm1 = __fmul_rn(dmin, (float)m1);
    float4 a, c;
    // separate multiply and subtract (no fused multiply-add): bit-identical to a plain host loop
    a.x = __fsub_rn(__fmul_rn(d0, (float)(lo & 0xffu)), mm0);
    a.y = __fsub_rn(__fmul_rn(d0, (float)((lo >> 8) & 0xffu)), mm0);
    a.z = __fsub_rn(__fmul_rn(d0, (float)((lo >> 16) & 0xffu)), mm0);
    a.w = __fsub_rn(__fmul_rn(d0, (float)(lo >> 24)), mm0);
    c.x = __fsub_rn(__fmul_rn(d1, (float)(hi & 0xffu)), mm1);
    c.y = __fsub_rn(__fmul_rn(d1, (float)((hi >> 8) & 0xffu)), mm1);
    c.z = __fsub_rn(__fmul_rn(d1, (float)((hi >> 16) & 0xffu)), mm1);
    c.w = __fsub_rn(__fmul_rn(d1, (float)(hi >> 24)), mm1);
    float4* o = (float4*)out + blk * 64;
    o[16 * g + (l0 >> 2)] = a;
    o[16 * g + 8 + (l0 >> 2)] = c;
  }
}

static int launch_q4k_unpack(const void* blocks, void* out, int64_t nblocks, bool f32out) {
  BK_REQUIRE(blocks && out, "q4k unpack: null pointer");
  BK_REQUIRE(nblocks > 0 && nblocks < ((int64_t)1 << 33), "q4k unpack: bad nblocks");
  const int64_t ndw = nblocks * 32;
  dim3 grid((unsigned)((ndw + 255) / 256));
  if (f32out)
    hipLaunchKernelGGL(q4k_unpack_kernel<true>, grid, dim3(256), 0, stream(), (const uint32_t*)blocks, out, ndw);
  else
    hipLaunchKernelGGL(q4k_unpack_kernel<false>, grid, dim3(256), 0, stream(), (const uint32_t*)blocks, out, ndw);
  BK_LAUNCH_CHECK();
  return BK_OK;
}
int launch_q4k_nibbles(const void* blocks, void* out, int64_t nblocks) { return launch_q4k_unpack(blocks, out, nblocks, false); }
int launch_q4k_dequant_f32(const void* blocks, void* out, int64_t nblocks) { return launch_q4k_unpack(blocks, out, nblocks, true); }

// ---------------------------------------------------------------- calibration kernels
// Plain streaming read / copy of a buffer with the access pattern of the GEMV (16 bytes per
// lane, several loads in flight): what the memory system gives a kernel that does nothing else.
// Used to calibrate counters and to put the GEMV's GB/s next to an achievable ceiling.
template <int U, bool NT>
__global__ __launch_bounds__(256) void memread_kernel(const uint4* __restrict__ p, int64_t n16, uint32_t* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  uint32_t acc = 0;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + (U - 1) * stride < n16; i += U * stride) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (NT) {
        typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
        const u32x4_t t = __builtin_nontemporal_load((const u32x4_t*)(p + i + u * stride));
        v[u] = make_uint4(t.x, t.y, t.z, t.w);
      } else {
        v[u] = p[i + u * stride];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) { const uint4 a = p[i]; acc ^= a.x ^ a.y ^ a.z ^ a.w; }
  if (acc == 0x9e3779b9u) sink[0] = acc;       // practically never true: keeps the loads alive
}
__global__ __launch_bounds__(256) void memcopy_kernel(const uint4* __restrict__ p, uint4* __restrict__ q, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) q[i] = p[i];
}

int g_tune_mr_unroll = 4, g_tune_mr_cap = 8, g_tune_mr_nt = 0;

int launch_memread(const void* src, int64_t bytes, void* sink) {
  BK_REQUIRE(src && sink && bytes >= 16 && bytes % 16 == 0, "memread: bad arguments");
  const int64_t n16 = bytes / 16;
  const int U = g_tune_mr_unroll;
  int64_t wgs = (n16 + 256 * U - 1) / (256 * U);
  if (wgs > (int64_t)num_cus() * g_tune_mr_cap) wgs = (int64_t)num_cus() * g_tune_mr_cap;
  dim3 grid((unsigned)wgs), block(256);
  const uint4* p = (const uint4*)src; uint32_t* sk = (uint32_t*)sink;
  const bool nt = g_tune_mr_nt != 0;
#define MR(UU) do { if (nt) hipLaunchKernelGGL((memread_kernel<UU, true>), grid, block, 0, stream(), p, n16, sk); \
                    else hipLaunchKernelGGL((memread_kernel<UU, false>), grid, block, 0, stream(), p, n16, sk); } while (0)
  if (U == 1) MR(1); else if (U == 2) MR(2); else if (U == 8) MR(8); else if (U == 16) MR(16); else MR(4);
#undef MR
  BK_LAUNCH_CHECK();
  return BK_OK;
}
int launch_memcopy(const void* src, void* dst, int64_t bytes) {
  BK_REQUIRE(src && dst && bytes >= 16 && bytes % 16 == 0, "memcopy: bad arguments");
  const int64_t n16 = bytes / 16;
  int64_t wgs = (n16 + 255) / 256;
  if (wgs > num_cus() * 16) wgs = num_cus() * 16;
  hipLaunchKernelGGL(memcopy_kernel, dim3((unsigned)wgs), dim3(256), 0, stream(), (const uint4*)src, (uint4*)dst, n16);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
