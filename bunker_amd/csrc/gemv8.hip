// Q4_K x Q8_1 GEMV, second layout: eight weight rows per wavefront.
//
// Lane (grp = lane >> 3, c = lane & 7) works on row `8*task + grp` and, inside every
// super-block of that row, on the 16-byte nibble chunk c (low nibbles: second half or first
// half of sub-block 2*(c>>1), high nibbles: sub-block 2*(c>>1)+1).  A wave-wide 16-byte load
// therefore fetches one whole super-block of eight consecutive rows (8 x 128 contiguous bytes
// plus the 8-way broadcast headers); the wave walks K block by block with several blocks in
// flight, every lane keeps a private double accumulator, and only at the end of the row are
// the eight lanes of a group added up (3 DPP steps) — one cross-lane reduction per row
// instead of one per block round.  Lane pairs first add their two 16-element half dots
// (exact int32), so that lane c owns the whole sub-block c and folds it with its own scale.
//
// The activation (Q8_1) is staged once per workgroup in LDS, int8 data at a 32-byte stride
// and (d, s) as float pairs; all eight row groups of a wave read the same addresses
// (broadcast).  Up to four matrices that share the activation run in one launch ("groups"),
// each with its own epilogue; a second kernel computes gate and up rows together and ends
// in SwiGLU and the Q8_1 quantization of the result (32 rows per workgroup = one block).
//
// Arithmetic as in gemv.hip: exact integer dots, every later term exact in double, one
// rounding to f32 per output, so results do not depend on this layout.
#include "ops.h"

namespace bk {

constexpr int G8_WAVES = 4;
constexpr int G8_UNROLL = 4;      // super-blocks in flight per lane

__device__ __forceinline__ int sdot4_(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

// scale and min of sub-block c from the 12 packed bytes (dwords s0, s1, s2); c is lane-constant
__device__ __forceinline__ void scale_min_c(int c, uint32_t s0, uint32_t s1, uint32_t s2, int& sc, int& m) {
  const uint32_t sh = 8u * (c & 3);
  const bool hi = c >= 4;
  const uint32_t t = s2 >> sh;
  const uint32_t a = hi ? t : (s0 >> sh);
  const uint32_t b = hi ? (t >> 4) : (s1 >> sh);
  const uint32_t wlo = hi ? 4u : 6u, whi = hi ? 2u : 0u;
  sc = (int)(__builtin_amdgcn_ubfe(a, 0, wlo) | (__builtin_amdgcn_ubfe(s0, sh + 6, whi) << 4));
  m = (int)(__builtin_amdgcn_ubfe(b, 0, wlo) | (__builtin_amdgcn_ubfe(s1, sh + 6, whi) << 4));
}

// Sum over the 8 lanes of a group (aligned octet); every lane of the octet gets the total.
__device__ __forceinline__ double octet_sum_f64(double v) {
  v += dpp_f64<DPP_QUAD_XOR1>(v);
  v += dpp_f64<DPP_QUAD_XOR2>(v);
  v += dpp_f64<DPP_ROW_HALF_MIRROR>(v);
  return v;
}

// ---- activation staging: Q8_1 rows (36-byte blocks) -> LDS [b][blocks*32 bytes] + float2 [b][blocks].
// The rows of a batch are contiguous and a row is a multiple of 16 bytes, so the whole activation is
// copied as 16-byte pieces, four per thread requested before any is scattered (one memory round trip
// for K <= 14336 at batch 1).
__device__ __forceinline__ void stage_xq(const uint8_t* __restrict__ xq, int nblk, int B, uint8_t* lds_q, float2* lds_s) {
  const int chunks = B * nblk * 9 / 4;                  // nblk is a multiple of 8
  const uint4* src = (const uint4*)xq;
  for (int base = threadIdx.x; base < chunks; base += 4 * blockDim.x) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int ch = base + u * blockDim.x;
      v[u] = ch < chunks ? src[ch] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int ch = base + u * blockDim.x;
      if (ch >= chunks) continue;
      const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const int i = ch * 4 + k, blk = i / 9, kk = i - blk * 9;   // blk counts over all batch rows
        if (kk < 8) ((uint32_t*)lds_q)[blk * 8 + kk] = w[k];
        else lds_s[blk] = make_float2(half_to_f32((uint16_t)(w[k] & 0xffffu)), half_to_f32((uint16_t)(w[k] >> 16)));
      }
    }
  }
}

// One super-block of one row for one lane: adds its share to acc[b] for every batch row.
template <int B>
__device__ __forceinline__ void block_dot(const uint4& hdr, const uint4& q, int blk, int c, int nblk_x, const uint8_t* lds_q,
                                          const float2* lds_s, double* acc) {
  const float d = half_to_f32((uint16_t)(hdr.x & 0xffffu)), dmin = half_to_f32((uint16_t)(hdr.x >> 16));
  int sc, m;
  scale_min_c(c, hdr.y, hdr.z, hdr.w, sc, m);
  const uint32_t l0 = q.x & 0x0f0f0f0fu, l1 = q.y & 0x0f0f0f0fu, l2 = q.z & 0x0f0f0f0fu, l3 = q.w & 0x0f0f0f0fu;
  const uint32_t h0 = (q.x >> 4) & 0x0f0f0f0fu, h1 = (q.y >> 4) & 0x0f0f0f0fu, h2 = (q.z >> 4) & 0x0f0f0f0fu,
                 h3 = (q.w >> 4) & 0x0f0f0f0fu;
  const int g = c >> 1, half = c & 1;
  const double dm = (double)m;
#pragma unroll
  for (int b = 0; b < B; b++) {
    const int xb = b * nblk_x + blk * 8;
    const uint4 xl = *(const uint4*)(lds_q + (xb + 2 * g) * 32 + 16 * half);
    const uint4 xh = *(const uint4*)(lds_q + (xb + 2 * g + 1) * 32 + 16 * half);
    const float2 ds = lds_s[xb + c];
    int i0 = sdot4_(l0, xl.x, 0); i0 = sdot4_(l1, xl.y, i0); i0 = sdot4_(l2, xl.z, i0); i0 = sdot4_(l3, xl.w, i0);
    int i1 = sdot4_(h0, xh.x, 0); i1 = sdot4_(h1, xh.y, i1); i1 = sdot4_(h2, xh.z, i1); i1 = sdot4_(h3, xh.w, i1);
    i0 += dpp_i32<DPP_QUAD_XOR1>(i0);      // whole sub-block 2g
    i1 += dpp_i32<DPP_QUAD_XOR1>(i1);      // whole sub-block 2g+1
    const int p = __mul24(sc, half ? i1 : i0);                        // lane c owns sub-block c: 6 x 17 bits, exact
    acc[b] = fma((double)(d * ds.x), (double)p, acc[b]);               // d*d8: 11 x 11 significand bits, exact in f32
    acc[b] = fma(-(double)(dmin * ds.y), dm, acc[b]);
  }
}

enum : int { G8_F32 = 0, G8_BF16 = 1, G8_BF16_ADD = 2 };

struct G8Group {
  const uint8_t* W;
  void* out;
  const uint16_t* res;   // residual (G8_BF16_ADD), bf16 [B, N]
  int N, epi;
};
struct G8Args {
  G8Group g[4];
  int wg_first[5];       // first workgroup of each group; wg_first[ngroups] = grid size
  int ngroups;
  const uint8_t* xq;     // Q8_1 [B, nb*8 blocks]
  int nb;                // super-blocks per row
};

__device__ __forceinline__ void g8_store(const G8Group& G, int b, int row, float v) {
  const int64_t o = (int64_t)b * G.N + row;
  if (G.epi == G8_F32) ((float*)G.out)[o] = v;
  else if (G.epi == G8_BF16) ((uint16_t*)G.out)[o] = f32_to_bf16(v);
  else ((uint16_t*)G.out)[o] = f32_to_bf16(bf16_to_f32(f32_to_bf16(v)) + bf16_to_f32(G.res[o]));   // cast, then add
}

// KS = 1: a workgroup owns 32 rows (8 per wave).  KS = 4: a workgroup owns 8 rows and its four
// waves split K (blocks w, w+4, ...); the partial sums meet in LDS.  For matrices with few rows.
template <int KS, int B>
__global__ __launch_bounds__(G8_WAVES * 64) void gemv8_kernel(G8Args A) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int nblk_x = A.nb * 8;
  uint8_t* lds_q = smem;
  float2* lds_s = (float2*)(smem + (size_t)B * nblk_x * 32);
  __shared__ double part[G8_WAVES][8][B];

  // Select the group with scalar selects over fields that are all fetched up front: indexing the
  // argument block with a computed index would put a second, dependent kernel-argument fetch on
  // the critical path of every workgroup.
  const int wgx = (int)blockIdx.x;
  const bool s1 = A.ngroups > 1 && wgx >= A.wg_first[1], s2 = A.ngroups > 2 && wgx >= A.wg_first[2],
             s3 = A.ngroups > 3 && wgx >= A.wg_first[3];
  G8Group G;
  G.W = s3 ? A.g[3].W : s2 ? A.g[2].W : s1 ? A.g[1].W : A.g[0].W;
  G.out = s3 ? A.g[3].out : s2 ? A.g[2].out : s1 ? A.g[1].out : A.g[0].out;
  G.res = s3 ? A.g[3].res : s2 ? A.g[2].res : s1 ? A.g[1].res : A.g[0].res;
  G.N = s3 ? A.g[3].N : s2 ? A.g[2].N : s1 ? A.g[1].N : A.g[0].N;
  G.epi = s3 ? A.g[3].epi : s2 ? A.g[2].epi : s1 ? A.g[1].epi : A.g[0].epi;
  const int lw = wgx - (s3 ? A.wg_first[3] : s2 ? A.wg_first[2] : s1 ? A.wg_first[1] : 0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = lane >> 3, c = lane & 7;
  const int row = (KS == 1 ? lw * 32 + wave * 8 : lw * 8) + grp;
  const uint8_t* rp = G.W + (int64_t)min(row, G.N - 1) * A.nb * 144;

  // the first weight loads go out before the activation is staged
  const int blk0 = KS == 1 ? 0 : wave, bstep = KS == 1 ? 1 : G8_WAVES;
  uint4 hdr[G8_UNROLL], q[G8_UNROLL];
#pragma unroll
  for (int u = 0; u < G8_UNROLL; u++) {
    const int blk = min(blk0 + u * bstep, A.nb - 1);
    hdr[u] = *(const uint4*)(rp + blk * 144);
    q[u] = *(const uint4*)(rp + blk * 144 + 16 + 16 * c);
  }
  stage_xq(A.xq, nblk_x, B, lds_q, lds_s);
  __syncthreads();

  double acc[B];
#pragma unroll
  for (int b = 0; b < B; b++) acc[b] = 0.0;
  // rolling prefetch: as soon as a block's registers are consumed, the block G8_UNROLL steps ahead is requested
  for (int base = blk0; base < A.nb; base += G8_UNROLL * bstep) {
#pragma unroll
    for (int u = 0; u < G8_UNROLL; u++) {
      const int blk = base + u * bstep;
      if (blk < A.nb) {
        const uint4 h = hdr[u], qq = q[u];
        const int nxt = blk + G8_UNROLL * bstep;
        if (nxt < A.nb) {
          hdr[u] = *(const uint4*)(rp + nxt * 144);
          q[u] = *(const uint4*)(rp + nxt * 144 + 16 + 16 * c);
        }
        block_dot<B>(h, qq, blk, c, nblk_x, lds_q, lds_s, acc);
      }
    }
  }
#pragma unroll
  for (int b = 0; b < B; b++) acc[b] = octet_sum_f64(acc[b]);

  if (KS == 1) {
    if (c == 0 && row < G.N) {
#pragma unroll
      for (int b = 0; b < B; b++) g8_store(G, b, row, (float)acc[b]);
    }
  } else {
    if (c == 0) {
#pragma unroll
      for (int b = 0; b < B; b++) part[wave][grp][b] = acc[b];
    }
    __syncthreads();
    if (wave == 0 && c == 0 && row < G.N) {
#pragma unroll
      for (int b = 0; b < B; b++)
        g8_store(G, b, row, (float)((part[0][grp][b] + part[1][grp][b]) + (part[2][grp][b] + part[3][grp][b])));
    }
  }
}

// gate and up rows together, SwiGLU, Q8_1 of the result: a workgroup owns rows n0..n0+31 of both
// matrices, i.e. one Q8_1 block of the output.  act bf16 [B, N] is optional (0 = not stored).
struct G8SwigluArgs {
  const uint8_t *Wg, *Wu, *xq;
  uint16_t* act;
  uint8_t* act_q8;       // Q8_1 [B, N/32 blocks]
  int N, nb;
};

template <int B>
__global__ __launch_bounds__(G8_WAVES * 64) void gemv8_swiglu_q8_kernel(G8SwigluArgs A) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int nblk_x = A.nb * 8;
  uint8_t* lds_q = smem;
  float2* lds_s = (float2*)(smem + (size_t)B * nblk_x * 32);
  __shared__ float lds_act[B][32];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = lane >> 3, c = lane & 7;
  const int row = blockIdx.x * 32 + wave * 8 + grp;              // N is a multiple of 32
  const uint8_t* rg = A.Wg + (int64_t)row * A.nb * 144;
  const uint8_t* ru = A.Wu + (int64_t)row * A.nb * 144;
  constexpr int U = 2;
  uint4 hg[U], qg[U], hu[U], qu[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const int blk = min(u, A.nb - 1);
    hg[u] = *(const uint4*)(rg + blk * 144); qg[u] = *(const uint4*)(rg + blk * 144 + 16 + 16 * c);
    hu[u] = *(const uint4*)(ru + blk * 144); qu[u] = *(const uint4*)(ru + blk * 144 + 16 + 16 * c);
  }
  stage_xq(A.xq, nblk_x, B, lds_q, lds_s);
  __syncthreads();

  double ag[B], au[B];
#pragma unroll
  for (int b = 0; b < B; b++) { ag[b] = 0.0; au[b] = 0.0; }
  for (int base = 0; base < A.nb; base += U) {
    uint4 hgn[U], qgn[U], hun[U], qun[U];
    if (base + U < A.nb) {
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int blk = min(base + U + u, A.nb - 1);
        hgn[u] = *(const uint4*)(rg + blk * 144); qgn[u] = *(const uint4*)(rg + blk * 144 + 16 + 16 * c);
        hun[u] = *(const uint4*)(ru + blk * 144); qun[u] = *(const uint4*)(ru + blk * 144 + 16 + 16 * c);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (base + u < A.nb) {
        block_dot<B>(hg[u], qg[u], base + u, c, nblk_x, lds_q, lds_s, ag);
        block_dot<B>(hu[u], qu[u], base + u, c, nblk_x, lds_q, lds_s, au);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) { hg[u] = hgn[u]; qg[u] = qgn[u]; hu[u] = hun[u]; qu[u] = qun[u]; }
  }
#pragma unroll
  for (int b = 0; b < B; b++) {
    const float gv = (float)octet_sum_f64(ag[b]), uv = (float)octet_sum_f64(au[b]);
    if (c == 0) {
      // src/fusion.ts:324-330: bf16((g * sigmoid(g)) * u)
      const uint16_t h = f32_to_bf16(__fmul_rn(__fmul_rn(gv, sigmoid_f64(gv)), uv));
      if (A.act) A.act[(int64_t)b * A.N + row] = h;
      lds_act[b][wave * 8 + grp] = bf16_to_f32(h);
    }
  }
  __syncthreads();
  // Q8_1 of the 32 bf16 results (bench/bench.ts:53-72): batch row b on the 32-lane half (b & 1) of wave (b >> 1)
  const int bq = wave * 2 + (lane >> 5), l = lane & 31;
  if (bq < B) {
    const float v = lds_act[bq][l];
    float amax = row16_max(fabsf(v));
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    const double d = (double)amax / 127.0;
    const double qd = (double)v / (d != 0.0 ? d : 1.0);
    double r = floor(qd);
    if (qd - r >= 0.5) r += 1.0;
    int qi = (int)r;
    int sum = row16_sum_i32(qi);
    sum += __shfl_xor(sum, 16);
    qi = qi < -128 ? -128 : (qi > 127 ? 127 : qi);
    uint8_t* o = A.act_q8 + ((int64_t)bq * (A.N / 32) + blockIdx.x) * 36;
    o[l] = (uint8_t)(int8_t)qi;
    if (l == 0)
      *(uint32_t*)(o + 32) = (uint32_t)f32_to_half_trunc((float)d) | ((uint32_t)f32_to_half_trunc((float)((double)sum * d)) << 16);
  }
}

// ---------------------------------------------------------------- launchers
int g_tune_ks_rows = 16384;      // matrices with at most this many rows split K over the four waves of a workgroup

static size_t g8_lds_bytes(int nb, int B) { return (size_t)B * nb * 8 * (32 + 8); }

int launch_gemv_group(const void* xq, int K, int batch, int ngroups, const void* const* W, void* const* out,
                      const void* const* res, const int* N, const int* epi) {
  BK_REQUIRE(xq && ngroups >= 1 && ngroups <= 4, "gemv_group: bad arguments");
  BK_REQUIRE(K > 0 && K % 256 == 0, "gemv: K=%d must be a positive multiple of 256", K);
  BK_REQUIRE(batch >= 1 && batch <= 65535, "gemv: bad batch=%d", batch);
  BK_REQUIRE(((uintptr_t)xq & 15) == 0, "gemv: xq must be 16-byte aligned");
  const int nb = K / 256;
  BK_REQUIRE(g8_lds_bytes(nb, 1) <= 64 * 1024, "gemv: K=%d is too large for the LDS staging of the activation", K);
  int total_rows = 0;
  for (int i = 0; i < ngroups; i++) {
    BK_REQUIRE(W[i] && out[i] && N[i] > 0, "gemv: null pointer or N <= 0 in group %d", i);
    BK_REQUIRE(((uintptr_t)W[i] & 15) == 0, "gemv: W must be 16-byte aligned");
    BK_REQUIRE(epi[i] == G8_F32 || epi[i] == G8_BF16 || epi[i] == G8_BF16_ADD, "gemv: bad epilogue %d", epi[i]);
    BK_REQUIRE(epi[i] != G8_BF16_ADD || res[i], "gemv: the add epilogue needs a residual");
    total_rows += N[i];
  }
  // few rows: four waves split K over the same 8 rows, so that enough waves are in flight
  const bool ksplit = total_rows <= g_tune_ks_rows && nb >= 4;
  const int rows_per_wg = ksplit ? 8 : 32;
  for (int b0 = 0; b0 < batch;) {
    const int left = batch - b0;
    int B = left >= 4 ? 4 : (left >= 2 ? 2 : 1);
    while (g8_lds_bytes(nb, B) > 64 * 1024) B >>= 1;
    G8Args A{};
    A.ngroups = ngroups; A.nb = nb;
    A.xq = (const uint8_t*)xq + (size_t)b0 * nb * 8 * 36;
    int wg = 0;
    for (int i = 0; i < ngroups; i++) {
      const size_t osz = epi[i] == G8_F32 ? 4 : 2;
      A.g[i].W = (const uint8_t*)W[i];
      A.g[i].out = (uint8_t*)out[i] + (size_t)b0 * N[i] * osz;
      A.g[i].res = res[i] ? (const uint16_t*)res[i] + (size_t)b0 * N[i] : nullptr;
      A.g[i].N = N[i]; A.g[i].epi = epi[i];
      A.wg_first[i] = wg;
      wg += (N[i] + rows_per_wg - 1) / rows_per_wg;
    }
    for (int i = ngroups; i < 5; i++) A.wg_first[i] = wg;
    const dim3 grid(wg), block(G8_WAVES * 64);
    const size_t lds = g8_lds_bytes(nb, B);
#define G8_LAUNCH(KS_, B_) hipLaunchKernelGGL((gemv8_kernel<KS_, B_>), grid, block, lds, stream(), A)
    if (ksplit) { if (B == 4) G8_LAUNCH(4, 4); else if (B == 2) G8_LAUNCH(4, 2); else G8_LAUNCH(4, 1); }
    else { if (B == 4) G8_LAUNCH(1, 4); else if (B == 2) G8_LAUNCH(1, 2); else G8_LAUNCH(1, 1); }
#undef G8_LAUNCH
    BK_LAUNCH_CHECK();
    b0 += B;
  }
  return BK_OK;
}

int launch_gemv_swiglu_q8(const void* Wg, const void* Wu, const void* xq, void* act, void* act_q8, int N, int K, int batch) {
  BK_REQUIRE(Wg && Wu && xq && act_q8, "gemv_swiglu: null pointer");
  BK_REQUIRE(K > 0 && K % 256 == 0 && N > 0 && N % 32 == 0, "gemv_swiglu: K=%d must be a multiple of 256 and N=%d of 32", K, N);
  BK_REQUIRE(batch >= 1 && batch <= 65535, "gemv_swiglu: bad batch=%d", batch);
  BK_REQUIRE((((uintptr_t)Wg | (uintptr_t)Wu | (uintptr_t)xq) & 15) == 0, "gemv_swiglu: misaligned pointer");
  const int nb = K / 256;
  BK_REQUIRE(g8_lds_bytes(nb, 1) <= 64 * 1024, "gemv_swiglu: K=%d is too large for the LDS staging", K);
  for (int b0 = 0; b0 < batch;) {
    const int left = batch - b0;
    int B = left >= 4 ? 4 : (left >= 2 ? 2 : 1);
    while (g8_lds_bytes(nb, B) > 64 * 1024) B >>= 1;
    G8SwigluArgs A{};
    A.Wg = (const uint8_t*)Wg; A.Wu = (const uint8_t*)Wu;
    A.xq = (const uint8_t*)xq + (size_t)b0 * nb * 8 * 36;
    A.act = act ? (uint16_t*)act + (size_t)b0 * N : nullptr;
    A.act_q8 = (uint8_t*)act_q8 + (size_t)b0 * (N / 32) * 36;
    A.N = N; A.nb = nb;
    const dim3 grid(N / 32), block(G8_WAVES * 64);
    const size_t lds = g8_lds_bytes(nb, B);
    if (B == 4) hipLaunchKernelGGL((gemv8_swiglu_q8_kernel<4>), grid, block, lds, stream(), A);
    else if (B == 2) hipLaunchKernelGGL((gemv8_swiglu_q8_kernel<2>), grid, block, lds, stream(), A);
    else hipLaunchKernelGGL((gemv8_swiglu_q8_kernel<1>), grid, block, lds, stream(), A);
    BK_LAUNCH_CHECK();
    b0 += B;
  }
  return BK_OK;
}

}  // namespace bk
