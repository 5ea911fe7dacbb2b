// Batched decode matmul: C[B, N] = Xq[B, K] . W[N, K]^T for B <= 32 activation rows in
// Q8_1 and W in Q4_K, on the int8 matrix cores.  Precedent in the reference:
// int8MatmulTTIR (src/kernel.ts:397-417), i8 x i8 -> i32 exact, and its documented
// post-scale (experiments/q4k_q81_final.ts:214-217).
//
// One v_mfma_i32_32x32x32_i8 consumes exactly one 32-element sub-block of K for a tile
// of 32 activation rows (M) x 32 weight rows (N), so the matrix core produces the exact
// int32 sub-block dots I_j[b, n].  A lane owns weight row n = lane % 32 and 16 of the 32
// batch rows; it folds the dots with the scales in double, in the same way the GEMV does
// (every term exact, ~1e-16 accumulation error, one rounding to f32), so the batched
// path returns the same bits as the batch-1 path:
//   y[b, n] = sum_blk ( d * sum_j d8_j[b] * (sc_j * I_j) - dmin * sum_j m_j * s8_j[b] )
// Batches of more than 32 rows are cut into 32-row tiles along blockIdx.y (one launch, every tile its own workgroup).
// A workgroup owns one 32 x 32 output tile; its NW wavefronts split K by super-block (wave w takes
// blocks w, w + NW, ...) and add their double partials in wave order through LDS at the end.  The
// int8 activation operand is read straight from the Q8_1 rows (16-byte pieces, L2-resident); only
// the activation scales of the wave's current super-block are staged in LDS, as doubles.
#include "ops.h"

namespace bk {

typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(16))) int i32x16_t;

enum : int { GEPI_F32 = 0, GEPI_BF16 = 1, GEPI_BF16_ADD = 2 };

// rows of the 32x32 accumulator held by a lane: r = 0..15 -> 8*(r/4) + 4*(lane/32) + r%4
__device__ __forceinline__ int mfma32_row(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

// Up to four matrices that share the activation rows run as one launch: their 32-row tiles are laid end to end.
struct MfmaGroup {
  const uint8_t* W;
  void* out;
  const uint16_t* res;
  int N, epi;
};
struct MfmaArgs {
  MfmaGroup g[4];
  int tile_first[5];      // first tile of each matrix; tile_first[i >= ngroups] = number of tiles
  const uint8_t* xq;
  int nb, B;
};

template <int NW, bool PF>
__global__ __launch_bounds__(64 * NW) void gemm_q4k_q8_1_mfma_kernel(MfmaArgs A) {
  // one buffer, two uses: during the K loop (d8, s8) of activation block (j, b) of each wave's current super-block, as
  // doubles [NW][8][32]; afterwards the waves' partial sums [NW][16][64]
  constexpr int LDS_DS_BYTES = NW * 8 * 32 * 16, LDS_PART_BYTES = NW > 1 ? NW * 16 * 64 * 8 : 0;
  __shared__ __align__(16) unsigned char lds_raw[LDS_DS_BYTES > LDS_PART_BYTES ? LDS_DS_BYTES : LDS_PART_BYTES];
  double2 (*lds_ds)[8][32] = (double2 (*)[8][32])lds_raw;

  const int tile = blockIdx.x;
  const bool s1 = tile >= A.tile_first[1], s2 = tile >= A.tile_first[2], s3 = tile >= A.tile_first[3];
  const uint8_t* __restrict__ W = s3 ? A.g[3].W : s2 ? A.g[2].W : s1 ? A.g[1].W : A.g[0].W;
  void* __restrict__ out = s3 ? A.g[3].out : s2 ? A.g[2].out : s1 ? A.g[1].out : A.g[0].out;
  const uint16_t* __restrict__ res = s3 ? A.g[3].res : s2 ? A.g[2].res : s1 ? A.g[1].res : A.g[0].res;
  const int N = s3 ? A.g[3].N : s2 ? A.g[2].N : s1 ? A.g[1].N : A.g[0].N;
  const int EPI = s3 ? A.g[3].epi : s2 ? A.g[2].epi : s1 ? A.g[1].epi : A.g[0].epi;
  const int nb = A.nb;
  const int b0 = blockIdx.y * 32;                     // first batch row of this tile
  const int B = min(32, A.B - b0);
  const uint8_t* __restrict__ xq = A.xq + (int64_t)b0 * nb * 8 * 36;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int n0 = (tile - (s3 ? A.tile_first[3] : s2 ? A.tile_first[2] : s1 ? A.tile_first[1] : 0)) * 32;
  const int n = min(n0 + col, N - 1);                 // rows past N recompute row N-1 and are not stored
  const uint8_t* wrow = W + (int64_t)n * nb * 144;
  const int64_t xrow_bytes = (int64_t)nb * 8 * 36;
  // A operand: batch row `col` (rows past B re-read row B-1; their results are not stored)
  const uint8_t* xrow = xq + (int64_t)min(col, B - 1) * xrow_bytes + 16 * half;

  double acc[16];
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0;

  // weights of this lane's row: header + its half of every 32-byte nibble group.  A wave with several super-blocks
  // requests the next one's weights (the HBM round trip) behind the current one's activation loads, so that only the
  // first super-block waits for memory; the requests are unconditional (clamped) to keep the waits countable.
  uint4 hdr_n, qs_n[4];
  {
    const uint8_t* wp = wrow + min(wave, nb - 1) * 144;
    hdr_n = *(const uint4*)wp;
#pragma unroll
    for (int g = 0; g < 4; g++) qs_n[g] = *(const uint4*)(wp + 16 + 32 * g + 16 * half);
  }
  for (int blk = wave; blk < nb; blk += NW) {
    // activations: the lane's 16 int8 of each of the 8 sub-blocks (4-byte aligned 16-byte loads)
    uint4 xa4[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const uint32_t* p = (const uint32_t*)(xrow + (int64_t)(blk * 8 + j) * 36);
      xa4[j] = make_uint4(p[0], p[1], p[2], p[3]);
    }
    uint32_t dsraw[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int t = lane + 64 * i;
      dsraw[i] = *(const uint32_t*)(xq + (int64_t)min(t >> 3, B - 1) * xrow_bytes + (int64_t)(blk * 8 + (t & 7)) * 36 + 32);
    }
    const uint4 hdr = hdr_n;
    uint4 qs[4];
#pragma unroll
    for (int g = 0; g < 4; g++) qs[g] = qs_n[g];
    if (PF) {
      const uint8_t* wp = wrow + min(blk + NW, nb - 1) * 144;
      hdr_n = *(const uint4*)wp;
#pragma unroll
      for (int g = 0; g < 4; g++) qs_n[g] = *(const uint4*)(wp + 16 + 32 * g + 16 * half);
    }
    // scales of the 32 x 8 activation blocks of this super-block -> LDS of this wave, 4 per lane
    __builtin_amdgcn_wave_barrier();     // the previous super-block's scales have been consumed by every lane
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int t = lane + 64 * i;
      const uint32_t ds = dsraw[i];
      lds_ds[wave][t & 7][t >> 3] = make_double2((double)half_to_f32((uint16_t)(ds & 0xffffu)), (double)half_to_f32((uint16_t)(ds >> 16)));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    const float d = half_to_f32((uint16_t)(hdr.x & 0xffffu)), dmin = half_to_f32((uint16_t)(hdr.x >> 16));
    // all eight 6-bit scales and mins of the block, four per dword
    const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu, m_lo = hdr.z & 0x3f3f3f3fu;
    const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
    const uint32_t m_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);

    const float dmin_neg = -dmin;
    // A = activations (M = batch row), B = weights (N = weight row): result[r] = I_j[b = mfma32_row(r), n = col]
    auto dots = [&](int j) {
      const uint4 q = qs[j >> 1];
      i32x4_t wb;
      if (j & 1) {
        wb = (i32x4_t){(int)((q.x >> 4) & 0x0f0f0f0fu), (int)((q.y >> 4) & 0x0f0f0f0fu), (int)((q.z >> 4) & 0x0f0f0f0fu),
                       (int)((q.w >> 4) & 0x0f0f0f0fu)};
      } else {
        wb = (i32x4_t){(int)(q.x & 0x0f0f0f0fu), (int)(q.y & 0x0f0f0f0fu), (int)(q.z & 0x0f0f0f0fu), (int)(q.w & 0x0f0f0f0fu)};
      }
      const i32x4_t xa = (i32x4_t){(int)xa4[j].x, (int)xa4[j].y, (int)xa4[j].z, (int)xa4[j].w};
      i32x16_t c;
#pragma unroll
      for (int r = 0; r < 16; r++) c[r] = 0;
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(xa, wb, c, 0, 0, 0);
    };
    // The fold runs as a pipeline over the 16 groups (sub-block j, eight of the lane's sixteen outputs): the activation
    // scales of group g+1 are requested from LDS and the matrix instruction of sub-block j+1 is issued before group g
    // is folded, so neither latency is exposed.  Per sub-block the lane's row contributes two factors, both exact in f32
    // (11-bit x 6-bit): d * sc_j and -dmin * m_j; every term (d*sc_j) * (d8 * I) and (-dmin*m_j) * s8 is exact in double.
    double2 dsa[8], dsb[8];
#pragma unroll
    for (int r = 0; r < 8; r++) dsa[r] = lds_ds[wave][0][mfma32_row(r, half)];
    i32x16_t c = dots(0), cn = c;
#pragma unroll
    for (int g = 0; g < 16; g++) {
      const int j = g >> 1, r0 = 8 * (g & 1);
      double2 (&cur)[8] = (g & 1) ? dsb : dsa;
      double2 (&nxt)[8] = (g & 1) ? dsa : dsb;
      if (g + 1 < 16) {
#pragma unroll
        for (int r = 0; r < 8; r++) nxt[r] = lds_ds[wave][(g + 1) >> 1][mfma32_row(8 * ((g + 1) & 1) + r, half)];
      }
      if (!(g & 1) && j + 1 < 8) cn = dots(j + 1);
      __builtin_amdgcn_sched_barrier(0);
      const double dsc = (double)(d * (float)(((j < 4 ? sc_lo : sc_hi) >> (8 * (j & 3))) & 0xffu));
      const double dmm = (double)(dmin_neg * (float)(((j < 4 ? m_lo : m_hi) >> (8 * (j & 3))) & 0xffu));
#pragma unroll
      for (int r = 0; r < 8; r++) {
        const double t = cur[r].x * (double)c[r0 + r];            // d8 * I: 11-bit x 17-bit, exact
        acc[r0 + r] = fma(dsc, t, acc[r0 + r]);
        acc[r0 + r] = fma(dmm, cur[r].y, acc[r0 + r]);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (g & 1) c = cn;
    }
    if (!PF) {
      const uint8_t* wp = wrow + min(blk + NW, nb - 1) * 144;
      hdr_n = *(const uint4*)wp;
#pragma unroll
      for (int g = 0; g < 4; g++) qs_n[g] = *(const uint4*)(wp + 16 + 32 * g + 16 * half);
    }
  }

  auto store = [&](int r, double total) {
    const int b = mfma32_row(r, half);
    if (n0 + col >= N || b >= B) return;
    const int64_t o = (int64_t)(b0 + b) * N + n0 + col;
    const float v = (float)total;
    if (EPI == GEPI_F32) ((float*)out)[o] = v;
    else if (EPI == GEPI_BF16) ((uint16_t*)out)[o] = f32_to_bf16(v);
    else ((uint16_t*)out)[o] = f32_to_bf16(bf16_to_f32(f32_to_bf16(v)) + bf16_to_f32(res[o]));
  };
  if (NW > 1) {
    // every wave leaves its 16 partial sums per lane in LDS; then wave w finishes outputs r = w*16/NW .. of every lane:
    // the partials are added in wave order, and the conversions and stores are spread over all waves
    double* part = (double*)lds_raw;
    __syncthreads();                       // all waves are done with the activation scales that share the buffer
#pragma unroll
    for (int r = 0; r < 16; r++) part[(wave * 16 + r) * 64 + lane] = acc[r];
    __syncthreads();
    constexpr int R = 16 / NW;
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      const int r = wave * R + rr;
      double t = part[r * 64 + lane];
#pragma unroll
      for (int w = 1; w < NW; w++) t += part[(w * 16 + r) * 64 + lane];
      store(r, t);
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) store(r, acc[r]);
  }
}

int g_tune_gemm_nw = 0;      // waves per tile (1, 2, 4, 8); 0 = chosen from the shape
int g_tune_gemm_pf = -1;     // next-block weight prefetch: 0 off, 1 on, -1 = chosen from the shape

int launch_gemm_group_mfma(const void* xq, int K, int batch, int ngroups, const void* const* W, void* const* out,
                           const void* const* res, const int* N, const int* epi) {
  BK_REQUIRE(xq && ngroups >= 1 && ngroups <= 4, "gemm_q4k_q8_1_mfma: bad arguments");
  BK_REQUIRE(K > 0 && K % 256 == 0, "gemm_q4k_q8_1_mfma: K=%d must be a positive multiple of 256", K);
  BK_REQUIRE(batch >= 1 && batch <= 32 * 65535, "gemm_q4k_q8_1_mfma: bad batch=%d", batch);
  BK_REQUIRE(((uintptr_t)xq & 3) == 0, "gemm_q4k_q8_1_mfma: xq must be 4-byte aligned");
  MfmaArgs A{};
  A.xq = (const uint8_t*)xq; A.nb = K / 256; A.B = batch;
  int tiles = 0;
  for (int i = 0; i < ngroups; i++) {
    BK_REQUIRE(W[i] && out[i] && N[i] > 0 && ((uintptr_t)W[i] & 15) == 0, "gemm_q4k_q8_1_mfma: matrix %d: null, misaligned or N <= 0", i);
    BK_REQUIRE(epi[i] == GEPI_F32 || epi[i] == GEPI_BF16 || epi[i] == GEPI_BF16_ADD, "gemm_q4k_q8_1_mfma: bad epilogue %d", epi[i]);
    BK_REQUIRE(epi[i] != GEPI_BF16_ADD || res[i], "gemm_q4k_q8_1_mfma: the add epilogue needs a residual");
    A.g[i].W = (const uint8_t*)W[i]; A.g[i].out = out[i]; A.g[i].res = (const uint16_t*)res[i]; A.g[i].N = N[i]; A.g[i].epi = epi[i];
    A.tile_first[i] = tiles;
    tiles += (N[i] + 31) / 32;
  }
  for (int i = ngroups; i < 5; i++) A.tile_first[i] = tiles;
  // waves per tile (measured on the decode shapes at batch 32): long rows split eight ways, K = 2048 four ways,
  // and two ways when the tiles alone fill the chip many times over (lm_head)
  const int btiles = (batch + 31) / 32;
  const int64_t wgs = (int64_t)tiles * btiles;
  int nw = g_tune_gemm_nw;
  if (nw <= 0) {
    nw = A.nb >= 16 ? 8 : (A.nb >= 4 ? 4 : (A.nb >= 2 ? 2 : 1));
    if (wgs <= num_cus() + num_cus() / 4 && A.nb >= 8) nw = 8;          // about a tile per CU: one super-block per wave
    if (wgs >= 8 * num_cus() && nw > 2) nw = 2;
  }
  nw = nw >= 8 ? 8 : (nw >= 4 ? 4 : (nw >= 2 ? 2 : 1));
  // next-block weight prefetch for waves with several super-blocks; not when the chip is full of tiles anyway
  // (it costs 20 registers: two waves per SIMD instead of three)
  const bool pf = g_tune_gemm_pf >= 0 ? g_tune_gemm_pf != 0 : ((A.nb + nw - 1) / nw >= 2 && wgs * nw <= 8 * num_cus());
  const dim3 grid(tiles, btiles);
#define BK_GEMM_LAUNCH(NWV)                                                                                             \
  {                                                                                                                     \
    if (pf) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<NWV, true>), grid, dim3(64 * NWV), 0, stream(), A);           \
    else hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<NWV, false>), grid, dim3(64 * NWV), 0, stream(), A);             \
  }
  if (nw == 8) BK_GEMM_LAUNCH(8)
  else if (nw == 4) BK_GEMM_LAUNCH(4)
  else if (nw == 2) BK_GEMM_LAUNCH(2)
  else BK_GEMM_LAUNCH(1)
#undef BK_GEMM_LAUNCH
  BK_LAUNCH_CHECK();
  return BK_OK;
}

int launch_gemm_q4k_q8_1_mfma(const void* W, const void* xq, void* y, int N, int K, int batch, int out_dtype,
                              const void* residual) {
  BK_REQUIRE(W && xq && y, "gemm_q4k_q8_1_mfma: null pointer");
  BK_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "gemm_q4k_q8_1_mfma: out_dtype must be 0 (f32) or 1 (bf16)");
  BK_REQUIRE(!(residual && out_dtype != DT_BF16), "gemm_q4k_q8_1_mfma: a residual needs bf16 output");
  const int epi = out_dtype == DT_F32 ? GEPI_F32 : (residual ? GEPI_BF16_ADD : GEPI_BF16);
  return launch_gemm_group_mfma(xq, K, batch, 1, &W, &y, &residual, &N, &epi);
}

}  // namespace bk
