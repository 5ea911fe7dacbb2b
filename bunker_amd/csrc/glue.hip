// Small bf16/f32 ops around the matmuls of one decode step: embed, RMSNorm, cast,
// add, SwiGLU, conv1d, per-head q/k norm, RoPE, argmax.  Every activation carries a
// leading batch dimension; all math is f32 with bf16 (round-to-nearest-even) I/O,
// as in src/fusion.ts:295-330 and src/emitters.ts:31-255.
#include <type_traits>
#include "ops.h"
#include "gemv_tile.h"

namespace bk {

// ---------------------------------------------------------------- embed
// src/emitters.ts:31-45: X[b, 0:H] = E[id[b], :] (bf16 row copy).  The id is a scalar
// argument (batch 1, as the reference passes it) or comes from an int32 device array.
__global__ __launch_bounds__(256) void embed_kernel(const uint16_t* __restrict__ E, const int32_t* __restrict__ ids,
                                                    int32_t id_scalar, uint16_t* __restrict__ out, int H, int vocab) {
  const int b = blockIdx.y;
  int id = ids ? ids[b] : id_scalar;
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);     // out-of-range ids are clamped, never read out of bounds
  const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (i < H) *(uint4*)(out + (int64_t)b * H + i) = *(const uint4*)(E + (int64_t)id * H + i);
}

int launch_embed(const void* E, const int32_t* ids_dev, int32_t id_scalar, void* out, int H, int vocab, int batch) {
  BK_REQUIRE(E && out, "embed: null pointer");
  BK_REQUIRE(H > 0 && H % 8 == 0 && vocab > 0 && batch > 0 && batch <= 65535, "embed: bad H=%d vocab=%d batch=%d", H, vocab, batch);
  BK_REQUIRE(ids_dev || batch == 1, "embed: a scalar token id serves batch 1 only");
  hipLaunchKernelGGL(embed_kernel, dim3((H / 8 + 255) / 256, batch), dim3(256), 0, stream(), (const uint16_t*)E, ids_dev,
                     id_scalar, (uint16_t*)out, H, vocab);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- RMSNorm
// src/fusion.ts:310-322: y = bf16((x * rsqrt(mean(x^2) + 1e-6)) * (1 + w)).  One
// workgroup per row, 8 elements per thread per pass.  With `xq` set the bf16 result
// is also quantized to Q8_1 in the same pass (four lanes share one 32-element block),
// which is what the following matmuls consume.
// ONE: the row has at most 2048 elements: a thread's 8 values and weights stay in registers between the two passes
// (one memory round trip instead of two).
// ROWS (with QUANT and ONE): the launch also multiplies a few short matrices (the 16-row a and b projections of a
// Gated-DeltaNet layer) with the row it has just quantized, so that the batched matmul behind it is left with the
// tiles of the large matrices only.  Workgroup (row, 0) does the norm's own job; workgroups (row, 1 + j) repeat the norm
// and the quantization on their own CU, keep the Q8_1 row in LDS and take eight of those rows each, two per wave, with
// the GEMV's row arithmetic (same int32 dots, same f64 fold, one rounding to f32).
struct SmallRows {
  const uint8_t* W[2];    // Q4_K matrices [n[i], N]
  float* out[2];          // f32 [rows, n[i]]
  int n[2];
};
// (the forms without small rows take an empty struct in their place: 40 bytes of arguments instead of 80, one 64-byte
// line less for a launch of four microseconds to fetch)
struct NoSmallRows {};
template <bool QUANT, bool ONE, bool ROWS = false>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                      uint16_t* __restrict__ out, uint8_t* __restrict__ xq, int N,
                                                      std::conditional_t<ROWS, SmallRows, NoSmallRows> sr = {}) {
  static_assert(!ROWS || (QUANT && ONE), "the small rows need the quantized row of a single pass");
  __shared__ double lds[4];
  __shared__ __align__(16) uint8_t xq_l[ROWS ? 2048 / 32 * 36 : 16];
  const bool own = !ROWS || blockIdx.y == 0;      // this workgroup writes the norm's results
  const int row = blockIdx.x;
  const uint16_t* xr = x + (int64_t)row * N;
  double ss = 0.0;     // squares of bf16 values are exact in f32; their sum is carried in double
  uint4 keep = make_uint4(0, 0, 0, 0), keepw = keep;
  if (ONE && threadIdx.x * 8 < N) keepw = *(const uint4*)(w + threadIdx.x * 8);
  for (int i = threadIdx.x * 8; i < N; i += 256 * 8) {
    const uint4 v = *(const uint4*)(xr + i);
    if (ONE) keep = v;
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float a = __uint_as_float(u[j] << 16), b = __uint_as_float(u[j] & 0xffff0000u);
      ss += (double)(a * a) + (double)(b * b);
    }
  }
  // the weight rows of the small matrices do not depend on the norm: requested behind the row itself (loads return in
  // issue order), they arrive while the sum is reduced and the row scaled and quantized
  uint4 sr_hdr[2] = {}, sr_q[2] = {};
  if constexpr (ROWS) if (!own) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nb = N / 256, blk = min(lane >> 3, nb - 1), c = lane & 7;
#pragma unroll
    for (int k = 0; k < 2; k++) {
      const int r = min(((int)blockIdx.y - 1) * 8 + wave * 2 + k, sr.n[0] + sr.n[1] - 1);      // past the end: the last row again
      const bool second = r >= sr.n[0];
      const uint8_t* rp = (second ? sr.W[1] : sr.W[0]) + (int64_t)(second ? r - sr.n[0] : r) * nb * 144 + blk * 144;
      sr_hdr[k] = load_w16(rp); sr_q[k] = load_w16(rp + 16 + 16 * c);
    }
  }
  ss = block_sum_f64<4>(ss, lds);
  const float rstd = rsqrt_f64(ss / (double)N + 1e-6);
  for (int i = threadIdx.x * 8; i < N; i += 256 * 8) {
    const uint4 v = ONE ? keep : *(const uint4*)(xr + i);
    const uint4 wv = ONE ? keepw : *(const uint4*)(w + i);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w}, uw[4] = {wv.x, wv.y, wv.z, wv.w};
    uint32_t o[4];
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float a = __uint_as_float(u[j] << 16), b = __uint_as_float(u[j] & 0xffff0000u);
      const float wa = __uint_as_float(uw[j] << 16), wb = __uint_as_float(uw[j] & 0xffff0000u);
      const uint16_t ha = f32_to_bf16(__fmul_rn(__fmul_rn(a, rstd), __fadd_rn(1.0f, wa)));
      const uint16_t hb = f32_to_bf16(__fmul_rn(__fmul_rn(b, rstd), __fadd_rn(1.0f, wb)));
      o[j] = (uint32_t)ha | ((uint32_t)hb << 16);
      f[2 * j] = bf16_to_f32(ha); f[2 * j + 1] = bf16_to_f32(hb);
    }
    if (out && own) *(uint4*)(out + (int64_t)row * N + i) = make_uint4(o[0], o[1], o[2], o[3]);
    if (QUANT) {
      // Q8_1 of the bf16-rounded values: block = 4 consecutive lanes x 8 elements
      uint32_t pk[2];
      const uint32_t ds = quad_q8_1(f, pk);
      if (own) {
        uint8_t* ob = xq + ((int64_t)row * (N / 32) + i / 32) * 36;
        uint32_t* oq = (uint32_t*)(ob + (i & 31));
        oq[0] = pk[0]; oq[1] = pk[1];
        if ((i & 31) == 0) *(uint32_t*)(ob + 32) = ds;
      } else if constexpr (ROWS) {
        uint8_t* ob = xq_l + (i / 32) * 36;
        uint32_t* oq = (uint32_t*)(ob + (i & 31));
        oq[0] = pk[0]; oq[1] = pk[1];
        if ((i & 31) == 0) *(uint32_t*)(ob + 32) = ds;
      }
    }
  }
  if constexpr (ROWS) {
    if (own) return;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nb = N / 256, blk = lane >> 3, c = lane & 7;
    const bool active = blk < nb;                       // lanes past the row add exact zeros
    const ScaleSel sel = make_scale_sel(c);
    XQ xs;
    load_xq(xs, xq_l, min(blk, nb - 1), c, active);
#pragma unroll
    for (int k = 0; k < 2; k++) {
      const int r = ((int)blockIdx.y - 1) * 8 + wave * 2 + k;
      if (r >= sr.n[0] + sr.n[1]) break;                // wave-uniform
      const bool second = r >= sr.n[0];
      const int rr = second ? r - sr.n[0] : r;
      int I0, I1;
      const double tot = wave_sum_f64(slot_dot(sr_hdr[k], sr_q[k], xs, sel, I0, I1, (c & 1) != 0));
      if (lane == 0) (second ? sr.out[1] : sr.out[0])[(int64_t)row * (second ? sr.n[1] : sr.n[0]) + rr] = (float)tot;
    }
  }
}

int g_tune_small_rows = 1;     // 0: the short matrices of a projection group stay in the batched matmul

// rmsnorm -> Q8_1 (into xq) together with the products of two short matrices with the quantized rows (see SmallRows)
int launch_rmsnorm_small_rows(const void* x, const void* w, void* xq, int N, int rows, const void* Wa, const void* Wb, float* out_a,
                              float* out_b, int na, int nb_rows) {
  BK_REQUIRE(x && w && xq && Wa && Wb && out_a && out_b, "rmsnorm_small_rows: null pointer");
  BK_REQUIRE(N > 0 && N % 256 == 0 && N <= 2048 && rows > 0 && rows <= 65535, "rmsnorm_small_rows: N=%d must be a multiple of 256 up to 2048 (rows=%d)", N, rows);
  BK_REQUIRE(na > 0 && nb_rows > 0 && na + nb_rows <= 64, "rmsnorm_small_rows: %d + %d rows (at most 64 together)", na, nb_rows);
  BK_REQUIRE(((uintptr_t)Wa & 15) == 0 && ((uintptr_t)Wb & 15) == 0, "rmsnorm_small_rows: misaligned matrix");
  SmallRows sr;
  sr.W[0] = (const uint8_t*)Wa; sr.W[1] = (const uint8_t*)Wb; sr.out[0] = out_a; sr.out[1] = out_b; sr.n[0] = na; sr.n[1] = nb_rows;
  hipLaunchKernelGGL((rmsnorm_kernel<true, true, true>), dim3(rows, 1 + (na + nb_rows + 7) / 8), dim3(256), 0, stream(),
                     (const uint16_t*)x, (const uint16_t*)w, (uint16_t*)nullptr, (uint8_t*)xq, N, sr);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

int launch_rmsnorm(const void* x, const void* w, void* out, void* xq, int N, int rows) {
  BK_REQUIRE(x && w && (out || xq), "rmsnorm: null pointer");
  BK_REQUIRE(N > 0 && N % 32 == 0 && rows > 0, "rmsnorm: N=%d must be a positive multiple of 32 (rows=%d)", N, rows);
  const uint16_t *xp = (const uint16_t*)x, *wp = (const uint16_t*)w;
  const bool one = N <= 2048;
  if (xq && one) hipLaunchKernelGGL((rmsnorm_kernel<true, true>), dim3(rows), dim3(256), 0, stream(), xp, wp, (uint16_t*)out, (uint8_t*)xq, N);
  else if (xq) hipLaunchKernelGGL((rmsnorm_kernel<true, false>), dim3(rows), dim3(256), 0, stream(), xp, wp, (uint16_t*)out, (uint8_t*)xq, N);
  else if (one) hipLaunchKernelGGL((rmsnorm_kernel<false, true>), dim3(rows), dim3(256), 0, stream(), xp, wp, (uint16_t*)out, (uint8_t*)nullptr, N);
  else hipLaunchKernelGGL((rmsnorm_kernel<false, false>), dim3(rows), dim3(256), 0, stream(), xp, wp, (uint16_t*)out, (uint8_t*)nullptr, N);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- elementwise
constexpr int EW_CAST = EW_CAST_OP, EW_ADD = EW_ADD_OP, EW_SWIGLU = EW_SWIGLU_OP;

// cast:   out = bf16(x)                      x f32            src/fusion.ts:295-299
// add:    out = bf16(f32(a) + f32(b))        a, b bf16        src/fusion.ts:301-308
// swiglu: out = bf16((g * sigmoid(g)) * u)   g, u f32         src/fusion.ts:324-330
template <int OP>
__global__ __launch_bounds__(256) void elementwise_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                          uint16_t* __restrict__ out, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= n) return;
  float r[4];
  if (OP == EW_CAST) {
    const float4 v = *(const float4*)((const float*)a + i);
    r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
  } else if (OP == EW_ADD) {
    const uint2 va = *(const uint2*)((const uint16_t*)a + i), vb = *(const uint2*)((const uint16_t*)b + i);
    r[0] = __uint_as_float(va.x << 16) + __uint_as_float(vb.x << 16);
    r[1] = __uint_as_float(va.x & 0xffff0000u) + __uint_as_float(vb.x & 0xffff0000u);
    r[2] = __uint_as_float(va.y << 16) + __uint_as_float(vb.y << 16);
    r[3] = __uint_as_float(va.y & 0xffff0000u) + __uint_as_float(vb.y & 0xffff0000u);
  } else {
    const float4 g = *(const float4*)((const float*)a + i), u = *(const float4*)((const float*)b + i);
    r[0] = __fmul_rn(__fmul_rn(g.x, sigmoid_f64(g.x)), u.x);
    r[1] = __fmul_rn(__fmul_rn(g.y, sigmoid_f64(g.y)), u.y);
    r[2] = __fmul_rn(__fmul_rn(g.z, sigmoid_f64(g.z)), u.z);
    r[3] = __fmul_rn(__fmul_rn(g.w, sigmoid_f64(g.w)), u.w);
  }
  uint2 o;
  o.x = (uint32_t)f32_to_bf16(r[0]) | ((uint32_t)f32_to_bf16(r[1]) << 16);
  o.y = (uint32_t)f32_to_bf16(r[2]) | ((uint32_t)f32_to_bf16(r[3]) << 16);
  *(uint2*)(out + i) = o;
}

int launch_elementwise(int op, const void* a, const void* b, void* out, int64_t n) {
  BK_REQUIRE(a && out && (op == EW_CAST || b), "elementwise: null pointer");
  BK_REQUIRE(n > 0 && n % 4 == 0, "elementwise: n=%lld must be a positive multiple of 4", (long long)n);
  dim3 grid((unsigned)((n / 4 + 255) / 256)), block(256);
  if (op == EW_CAST) hipLaunchKernelGGL(elementwise_kernel<EW_CAST>, grid, block, 0, stream(), a, b, (uint16_t*)out, n);
  else if (op == EW_ADD) hipLaunchKernelGGL(elementwise_kernel<EW_ADD>, grid, block, 0, stream(), a, b, (uint16_t*)out, n);
  else if (op == EW_SWIGLU) hipLaunchKernelGGL(elementwise_kernel<EW_SWIGLU>, grid, block, 0, stream(), a, b, (uint16_t*)out, n);
  else return set_error(BK_ERR_ARG, "elementwise: unknown op %d", op);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// swiglu with both forms of the result: bf16 (optional) and the Q8_1 blocks the down projection consumes, so that no
// separate quantizer pass reads the activation again.  A thread owns 8 consecutive elements, four lanes one Q8_1 block.
__global__ __launch_bounds__(256) void swiglu_q8_1_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                          uint16_t* __restrict__ out, uint8_t* __restrict__ out_q8, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= n) return;                     // n is a multiple of 32: the four lanes of a block leave together
  const float4 g0 = *(const float4*)(g + i), g1 = *(const float4*)(g + i + 4);
  const float4 u0 = *(const float4*)(u + i), u1 = *(const float4*)(u + i + 4);
  const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
  const float uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
  uint16_t ob[8];
  float f[8];
#pragma unroll
  for (int k = 0; k < 8; k++) {
    ob[k] = f32_to_bf16(__fmul_rn(__fmul_rn(gv[k], sigmoid_f64(gv[k])), uv[k]));
    f[k] = bf16_to_f32(ob[k]);
  }
  if (out) {
    uint4 o;
    o.x = (uint32_t)ob[0] | ((uint32_t)ob[1] << 16); o.y = (uint32_t)ob[2] | ((uint32_t)ob[3] << 16);
    o.z = (uint32_t)ob[4] | ((uint32_t)ob[5] << 16); o.w = (uint32_t)ob[6] | ((uint32_t)ob[7] << 16);
    *(uint4*)(out + i) = o;
  }
  uint32_t pk[2];
  const uint32_t ds = quad_q8_1(f, pk);
  uint8_t* blk = out_q8 + (i / 32) * 36;
  *(uint2*)(blk + (i & 31)) = make_uint2(pk[0], pk[1]);
  if ((i & 31) == 0) *(uint32_t*)(blk + 32) = ds;
}

int launch_swiglu_q8_1(const float* g, const float* u, void* out, void* out_q8, int64_t n) {
  BK_REQUIRE(g && u && out_q8, "swiglu_q8_1: null pointer");
  BK_REQUIRE(n > 0 && n % 32 == 0, "swiglu_q8_1: n=%lld must be a positive multiple of 32", (long long)n);
  hipLaunchKernelGGL(swiglu_q8_1_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, stream(), g, u, (uint16_t*)out,
                     (uint8_t*)out_q8, n);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- conv1d decode
// src/emitters.ts:48-72: r = (w0*s0 + w1*s1) + (w2*s2 + w3*x); out = bf16(r * sigmoid(r));
// new state rows = (s1, s2, x).  state [B, 3, C] bf16, weight [C, 4] bf16.  The new state may be
// written over the old one: a thread reads its two channels' rows before it writes them.
__global__ __launch_bounds__(256) void conv1d_decode_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ st,
                                                            const uint16_t* __restrict__ w, uint16_t* __restrict__ out,
                                                            uint16_t* __restrict__ stn, int C) {
  const int b = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 2;
  if (c >= C) return;
  const uint32_t xv = *(const uint32_t*)(x + (int64_t)b * C + c);
  const uint16_t* sb = st + (int64_t)b * 3 * C;
  const uint32_t s0 = *(const uint32_t*)(sb + c), s1 = *(const uint32_t*)(sb + C + c), s2 = *(const uint32_t*)(sb + 2 * C + c);
  const uint4 wv = *(const uint4*)(w + 4 * c);          // 8 bf16: channel c taps 0..3, channel c+1 taps 0..3
  uint32_t o = 0;
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const uint32_t wl = k ? wv.z : wv.x, wh = k ? wv.w : wv.y;
    const float w0 = __uint_as_float(wl << 16), w1 = __uint_as_float(wl & 0xffff0000u);
    const float w2 = __uint_as_float(wh << 16), w3 = __uint_as_float(wh & 0xffff0000u);
    const float f0 = k ? __uint_as_float(s0 & 0xffff0000u) : __uint_as_float(s0 << 16);
    const float f1 = k ? __uint_as_float(s1 & 0xffff0000u) : __uint_as_float(s1 << 16);
    const float f2 = k ? __uint_as_float(s2 & 0xffff0000u) : __uint_as_float(s2 << 16);
    const float fx = k ? __uint_as_float(xv & 0xffff0000u) : __uint_as_float(xv << 16);
    // products of two bf16 values are exact in f32, so fusing them into the additions changes nothing
    const float r = __fadd_rn(__fadd_rn(w0 * f0, w1 * f1), __fadd_rn(w2 * f2, w3 * fx));
    o |= (uint32_t)f32_to_bf16(__fmul_rn(r, sigmoid_f64(r))) << (16 * k);
  }
  *(uint32_t*)(out + (int64_t)b * C + c) = o;
  uint16_t* nb = stn + (int64_t)b * 3 * C;
  *(uint32_t*)(nb + c) = s1;
  *(uint32_t*)(nb + C + c) = s2;
  *(uint32_t*)(nb + 2 * C + c) = xv;
}

int launch_conv1d_decode(const void* x, const void* st, const void* w, void* out, void* st_new, int C, int batch) {
  BK_REQUIRE(x && st && w && out && st_new, "conv1d_decode: null pointer");
  BK_REQUIRE(C > 0 && C % 2 == 0 && batch > 0 && batch <= 65535, "conv1d_decode: bad C=%d batch=%d", C, batch);
  hipLaunchKernelGGL(conv1d_decode_kernel, dim3((C / 2 + 255) / 256, batch), dim3(256), 0, stream(), (const uint16_t*)x,
                     (const uint16_t*)st, (const uint16_t*)w, (uint16_t*)out, (uint16_t*)st_new, C);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- conv1d over a run of T tokens
// The same 4-tap causal convolution + SiLU for T consecutive tokens of ONE sequence (prefill form,
// prototypes/conv1d.ts:53-61, with the three rows of carried state in place of zero padding): token t reads
// rows t-3 .. t of the virtual sequence [state row 0, 1, 2, x_0 .. x_{T-1}].  Same expression per channel as
// conv1d_decode, so T single-token steps give the same bits.  The new state (the last three rows of the
// virtual sequence) is written by a second kernel after every token has read the old one, so it may be
// updated in place.
__global__ __launch_bounds__(256) void conv1d_prefill_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ st,
                                                             const uint16_t* __restrict__ w, uint16_t* __restrict__ out, int C) {
  const int t = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 2;
  if (c >= C) return;
  uint32_t rows[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int r = t - 3 + j;
    rows[j] = *(const uint32_t*)((r >= 0 ? x + (int64_t)r * C : st + (int64_t)(3 + r) * C) + c);
  }
  const uint4 wv = *(const uint4*)(w + 4 * c);
  uint32_t o = 0;
#pragma unroll
  for (int k = 0; k < 2; k++) {
    const uint32_t wl = k ? wv.z : wv.x, wh = k ? wv.w : wv.y;
    const float w0 = __uint_as_float(wl << 16), w1 = __uint_as_float(wl & 0xffff0000u);
    const float w2 = __uint_as_float(wh << 16), w3 = __uint_as_float(wh & 0xffff0000u);
    float f[4];
#pragma unroll
    for (int j = 0; j < 4; j++) f[j] = k ? __uint_as_float(rows[j] & 0xffff0000u) : __uint_as_float(rows[j] << 16);
    const float r = __fadd_rn(__fadd_rn(w0 * f[0], w1 * f[1]), __fadd_rn(w2 * f[2], w3 * f[3]));
    o |= (uint32_t)f32_to_bf16(__fmul_rn(r, sigmoid_f64(r))) << (16 * k);
  }
  *(uint32_t*)(out + (int64_t)t * C + c) = o;
}
__global__ __launch_bounds__(256) void conv1d_prefill_state_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ st,
                                                                   uint16_t* __restrict__ stn, int C, int T) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * 2;
  if (c >= C) return;
  uint32_t rows[3];
#pragma unroll
  for (int j = 0; j < 3; j++) {
    const int r = T - 3 + j;
    rows[j] = *(const uint32_t*)((r >= 0 ? x + (int64_t)r * C : st + (int64_t)(3 + r) * C) + c);
  }
#pragma unroll
  for (int j = 0; j < 3; j++) *(uint32_t*)(stn + (int64_t)j * C + c) = rows[j];
}

int launch_conv1d_prefill(const void* x, const void* st, const void* w, void* out, void* st_new, int C, int T) {
  BK_REQUIRE(x && st && w && out && st_new, "conv1d_prefill: null pointer");
  BK_REQUIRE(C > 0 && C % 2 == 0 && T > 0 && T <= 65535, "conv1d_prefill: bad C=%d T=%d", C, T);
  BK_REQUIRE(out != x, "conv1d_prefill: the output must not overwrite the input rows");
  const int wgs = (C / 2 + 255) / 256;
  hipLaunchKernelGGL(conv1d_prefill_kernel, dim3(wgs, T), dim3(256), 0, stream(), (const uint16_t*)x, (const uint16_t*)st,
                     (const uint16_t*)w, (uint16_t*)out, C);
  hipLaunchKernelGGL(conv1d_prefill_state_kernel, dim3(wgs), dim3(256), 0, stream(), (const uint16_t*)x, (const uint16_t*)st,
                     (uint16_t*)st_new, C, T);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- per-head norm (+ RoPE)
// src/emitters.ts:123-147 emitQNorm / emitKNorm: bf16((x * rsqrt(mean(x^2) + 1e-6)) * (1 + w))
// per head of HD values; the input rows are `in_stride` apart (2*HD for the interleaved
// [q | gate] buffer of q_proj, HD for k).  One wavefront per (batch, head).
// With cos/sin tables the rotation of src/emitters.ts:150-183 is applied to the
// bf16-rounded result in the same kernel: pairs (i, i + half), i < half:
//   x1' = bf16(x1*c - x2*s), x2' = bf16(x2*c + x1*s).
__global__ __launch_bounds__(64) void headnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                      uint16_t* __restrict__ out, int nheads, int HD, int in_stride,
                                                      int64_t in_bstride, const float* __restrict__ cos_t,
                                                      const float* __restrict__ sin_t, const int32_t* __restrict__ pos_dev,
                                                      int pos_scalar, int half, int max_len) {
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const uint16_t* xh = x + (int64_t)b * in_bstride + (int64_t)h * in_stride;
  uint16_t* oh = out + ((int64_t)b * nheads + h) * HD;
  double ss = 0.0;
  for (int i = lane; i < HD; i += 64) { const float v = bf16_to_f32(xh[i]); ss += (double)(v * v); }
  ss = wave_sum_f64(ss);
  const float rstd = rsqrt_f64(ss / (double)HD + 1e-6);
  auto normed = [&](int i) { return f32_to_bf16(__fmul_rn(__fmul_rn(bf16_to_f32(xh[i]), rstd), __fadd_rn(1.0f, bf16_to_f32(w[i])))); };
  if (!cos_t) {
    for (int i = lane; i < HD; i += 64) oh[i] = normed(i);
    return;
  }
  // a position from device memory is held inside the table (the host checks only scalar positions)
  const int pos = min(max(pos_dev ? pos_dev[b] : pos_scalar, 0), max_len - 1);
  for (int i = lane; i < HD; i += 64) {
    if (i >= 2 * half) {
      oh[i] = normed(i);
    } else if (i < half) {
      const float x1 = bf16_to_f32(normed(i)), x2 = bf16_to_f32(normed(i + half));
      const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
      oh[i] = f32_to_bf16(__fsub_rn(__fmul_rn(x1, c), __fmul_rn(x2, s)));
      oh[i + half] = f32_to_bf16(__fadd_rn(__fmul_rn(x2, c), __fmul_rn(x1, s)));
    }
  }
}

int launch_headnorm(const void* x, const void* w, void* out, int nheads, int HD, int in_stride, int64_t in_bstride,
                    int batch, const float* cos_t, const float* sin_t, const int32_t* pos_dev, int pos_scalar, int half,
                    int max_len) {
  BK_REQUIRE(x && w && out, "headnorm: null pointer");
  BK_REQUIRE(nheads > 0 && HD > 0 && in_stride >= HD && batch > 0 && batch <= 65535, "headnorm: bad shape");
  if (cos_t) {
    BK_REQUIRE(sin_t && half > 0 && 2 * half <= HD, "headnorm+rope: bad tables / half=%d", half);
    BK_REQUIRE(max_len >= 1 && (pos_dev || (pos_scalar >= 0 && pos_scalar < max_len)), "rope: pos=%d outside the table (max_len=%d)", pos_scalar, max_len);
  }
  hipLaunchKernelGGL(headnorm_kernel, dim3(nheads, batch), dim3(64), 0, stream(), (const uint16_t*)x, (const uint16_t*)w,
                     (uint16_t*)out, nheads, HD, in_stride, in_bstride, cos_t, sin_t, pos_dev, pos_scalar, half, max_len);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// src/emitters.ts:150-183 emitRoPE / emitRoPEK: in place on bf16 [B, nheads, HD].
__global__ __launch_bounds__(256) void rope_kernel(uint16_t* __restrict__ x, const float* __restrict__ cos_t,
                                                   const float* __restrict__ sin_t, const int32_t* __restrict__ pos_dev,
                                                   int pos_scalar, int nheads, int HD, int half, int max_len) {
  const int b = blockIdx.y;
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= nheads * half) return;
  const int h = t / half, i = t % half;
  const int pos = min(max(pos_dev ? pos_dev[b] : pos_scalar, 0), max_len - 1);     // device positions are held inside the table
  uint16_t* p1 = x + ((int64_t)b * nheads + h) * HD + i;
  uint16_t* p2 = p1 + half;
  const float x1 = bf16_to_f32(*p1), x2 = bf16_to_f32(*p2);
  const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
  *p1 = f32_to_bf16(__fsub_rn(__fmul_rn(x1, c), __fmul_rn(x2, s)));
  *p2 = f32_to_bf16(__fadd_rn(__fmul_rn(x2, c), __fmul_rn(x1, s)));
}

int launch_rope(void* x, const float* cos_t, const float* sin_t, const int32_t* pos_dev, int pos_scalar, int nheads,
                int HD, int half, int max_len, int batch) {
  BK_REQUIRE(x && cos_t && sin_t, "rope: null pointer");
  BK_REQUIRE(nheads > 0 && half > 0 && 2 * half <= HD && batch > 0 && batch <= 65535, "rope: bad shape");
  BK_REQUIRE(max_len >= 1 && (pos_dev || (pos_scalar >= 0 && pos_scalar < max_len)), "rope: pos=%d outside the table (max_len=%d)", pos_scalar, max_len);
  hipLaunchKernelGGL(rope_kernel, dim3((nheads * half + 255) / 256, batch), dim3(256), 0, stream(), (uint16_t*)x, cos_t, sin_t,
                     pos_dev, pos_scalar, nheads, HD, half, max_len);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- argmax
// prototypes/decode.ts:746-791: stage 1 takes the maximum of a tile and its index,
// stage 2 walks the partials in index order with a strict ">", so the lowest index
// wins ties; the running maximum starts at -FLT_MAX and NaN never wins.
constexpr float ARGMAX_INIT = -3.40282347e38f;
constexpr int ARGMAX_TILE = 1024;     // one 16-byte load per thread: a short instruction stream on many CUs (the op is latency-bound)

__device__ __forceinline__ void argmax_merge(float& v, int& i, float ov, int oi) {
  // (ov, oi) beats (v, i) when larger, or equal with a lower index
  if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}
__device__ __forceinline__ void argmax_wave(float& v, int& i) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(v, off);
    const int oi = __shfl_xor(i, off);
    argmax_merge(v, i, ov, oi);
  }
}

__global__ __launch_bounds__(256) void argmax_stage1_kernel(const float* __restrict__ logits, float* __restrict__ pv,
                                                            int32_t* __restrict__ pi, int n, int ntiles, bool vec4) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int b = blockIdx.y, tile = blockIdx.x;
  const float* L = logits + (int64_t)b * n;
  float v = ARGMAX_INIT; int idx = 0x7fffffff;
  const int base = tile * ARGMAX_TILE;
  const int e0 = base + threadIdx.x * 4;
  if (vec4 && e0 + 3 < n) {
    const float4 x = *(const float4*)(L + e0);          // elements in index order, strict >: the lowest index wins a tie
    if (x.x > v) { v = x.x; idx = e0; }
    if (x.y > v) { v = x.y; idx = e0 + 1; }
    if (x.z > v) { v = x.z; idx = e0 + 2; }
    if (x.w > v) { v = x.w; idx = e0 + 3; }
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int e = e0 + j;
      if (e < n) { const float x = L[e]; if (x > v) { v = x; idx = e; } }
    }
  }
  argmax_wave(v, idx);
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = v; si[threadIdx.x >> 6] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; k++) argmax_merge(v, idx, sv[k], si[k]);
    pv[(int64_t)b * ntiles + tile] = v;
    pi[(int64_t)b * ntiles + tile] = idx;
  }
}

__global__ __launch_bounds__(64) void argmax_stage2_kernel(const float* __restrict__ pv, const int32_t* __restrict__ pi,
                                                           float* __restrict__ val, int32_t* __restrict__ idx, int ntiles) {
  const int b = blockIdx.x;
  float v = ARGMAX_INIT; int i = 0x7fffffff;
  for (int t = threadIdx.x; t < ntiles; t += 64) argmax_merge(v, i, pv[(int64_t)b * ntiles + t], pi[(int64_t)b * ntiles + t]);
  argmax_wave(v, i);
  if (threadIdx.x == 0) {
    val[b] = v;
    idx[b] = (i == 0x7fffffff) ? 0 : i;     // nothing above -FLT_MAX: index 0, like the sequential scan
  }
}

size_t argmax_workspace_bytes(int n, int batch) { return (size_t)batch * ((n + ARGMAX_TILE - 1) / ARGMAX_TILE) * 8; }

int launch_argmax(const float* logits, float* val, int32_t* idx, void* workspace, int n, int batch) {
  BK_REQUIRE(logits && val && idx && workspace, "argmax: null pointer");
  BK_REQUIRE(n > 0 && batch > 0 && batch <= 65535, "argmax: bad n=%d batch=%d", n, batch);
  const int ntiles = (n + ARGMAX_TILE - 1) / ARGMAX_TILE;
  float* pv = (float*)workspace;
  int32_t* pi = (int32_t*)(pv + (size_t)batch * ntiles);
  const bool vec4 = n % 4 == 0 && ((uintptr_t)logits & 15) == 0;      // every row then starts on a 16-byte boundary
  hipLaunchKernelGGL(argmax_stage1_kernel, dim3(ntiles, batch), dim3(256), 0, stream(), logits, pv, pi, n, ntiles, vec4);
  hipLaunchKernelGGL(argmax_stage2_kernel, dim3(batch), dim3(64), 0, stream(), pv, pi, val, idx, ntiles);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- token feedback
// What the host loop of src/runner.ts:150-160 does between tokens, on the device: the
// argmax index of every sequence becomes its next token id, positions advance by one and
// (token, logit) is appended to a history the host reads at the end.
__global__ __launch_bounds__(256) void advance_kernel(const int32_t* __restrict__ idx, const float* __restrict__ val,
                                                      int32_t* __restrict__ ids, int32_t* __restrict__ pos,
                                                      int32_t* __restrict__ hist, int32_t* __restrict__ counter, int batch,
                                                      int max_steps, int max_pos) {
  const int c = counter[0];
  __syncthreads();
  for (int b = threadIdx.x; b < batch; b += 256) {
    if (c < max_steps) {
      hist[((int64_t)c * batch + b) * 2] = idx[b];
      hist[((int64_t)c * batch + b) * 2 + 1] = __float_as_int(val[b]);
    }
    ids[b] = idx[b];
    // positions stop at max_pos (the cache capacity): a replay past it finds pos == max_pos, which the cache writers skip
    const int p = pos[b];
    if (p < max_pos) pos[b] = p + 1;
  }
  if (threadIdx.x == 0) counter[0] = c + 1;
}

// argmax's second stage, the token feedback above and the embedding of the next step's token in one launch (one
// workgroup per sequence): what would be three launches of a few microseconds each between two tokens.  `counter` holds
// one step count per sequence here (every workgroup advances its own).
__global__ __launch_bounds__(256) void argmax_feed_kernel(const float* __restrict__ pv, const int32_t* __restrict__ pi,
                                                          float* __restrict__ val, int32_t* __restrict__ idx, int ntiles,
                                                          int32_t* __restrict__ ids, int32_t* __restrict__ pos,
                                                          int32_t* __restrict__ hist, int32_t* __restrict__ counter, int batch,
                                                          int max_steps, int max_pos, const uint16_t* __restrict__ E,
                                                          uint16_t* __restrict__ x, int H, int vocab) {
  __shared__ float sv[4];
  __shared__ int si[4];
  __shared__ int s_id;
  const int b = blockIdx.x;
  float v = ARGMAX_INIT; int i = 0x7fffffff;
  for (int t = threadIdx.x; t < ntiles; t += 256) argmax_merge(v, i, pv[(int64_t)b * ntiles + t], pi[(int64_t)b * ntiles + t]);
  argmax_wave(v, i);
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = v; si[threadIdx.x >> 6] = i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; k++) argmax_merge(v, i, sv[k], si[k]);
    i = (i == 0x7fffffff) ? 0 : i;          // nothing above -FLT_MAX: index 0, like the sequential scan
    val[b] = v; idx[b] = i;
    const int c = counter[b];
    if (c < max_steps) {
      hist[((int64_t)c * batch + b) * 2] = i;
      hist[((int64_t)c * batch + b) * 2 + 1] = __float_as_int(v);
    }
    counter[b] = c + 1;
    ids[b] = i;
    const int p = pos[b];
    if (p < max_pos) pos[b] = p + 1;      // positions stop at the cache capacity, as in advance_kernel
    s_id = i < 0 ? 0 : (i >= vocab ? vocab - 1 : i);
  }
  __syncthreads();
  const int id = s_id;
  for (int e = threadIdx.x * 8; e < H; e += 256 * 8) *(uint4*)(x + (int64_t)b * H + e) = *(const uint4*)(E + (int64_t)id * H + e);
}

int launch_argmax_feed(const float* logits, float* val, int32_t* idx, void* workspace, int n, int batch, int32_t* ids, int32_t* pos,
                       int32_t* hist, int32_t* counter, int max_steps, int max_pos, const void* E, void* x, int H) {
  BK_REQUIRE(logits && val && idx && workspace && ids && pos && hist && counter && E && x, "argmax_feed: null pointer");
  BK_REQUIRE(n > 0 && batch > 0 && batch <= 65535 && max_steps > 0 && max_pos > 0, "argmax_feed: bad n=%d batch=%d max_steps=%d max_pos=%d", n,
             batch, max_steps, max_pos);
  BK_REQUIRE(H > 0 && H % 8 == 0 && ((uintptr_t)E & 15) == 0 && ((uintptr_t)x & 15) == 0, "argmax_feed: H=%d must be a multiple of 8, rows 16-byte aligned", H);
  const int ntiles = (n + ARGMAX_TILE - 1) / ARGMAX_TILE;
  float* pv = (float*)workspace;
  int32_t* pi = (int32_t*)(pv + (size_t)batch * ntiles);
  const bool vec4 = n % 4 == 0 && ((uintptr_t)logits & 15) == 0;
  hipLaunchKernelGGL(argmax_stage1_kernel, dim3(ntiles, batch), dim3(256), 0, stream(), logits, pv, pi, n, ntiles, vec4);
  hipLaunchKernelGGL(argmax_feed_kernel, dim3(batch), dim3(256), 0, stream(), pv, pi, val, idx, ntiles, ids, pos, hist, counter, batch,
                     max_steps, max_pos, (const uint16_t*)E, (uint16_t*)x, H, n);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

int launch_advance(const int32_t* idx, const float* val, int32_t* ids, int32_t* pos, int32_t* hist, int32_t* counter, int batch,
                   int max_steps, int max_pos) {
  BK_REQUIRE(idx && val && ids && pos && hist && counter, "advance: null pointer");
  BK_REQUIRE(batch > 0 && max_steps > 0 && max_pos > 0, "advance: bad batch=%d max_steps=%d max_pos=%d", batch, max_steps, max_pos);
  hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(256), 0, stream(), idx, val, ids, pos, hist, counter, batch, max_steps, max_pos);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
