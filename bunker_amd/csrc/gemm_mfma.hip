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

template <int EPI, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_q4k_q8_1_mfma_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq,
                                                                     void* __restrict__ out, const uint16_t* __restrict__ res,
                                                                     int N, int nb, int B) {
  __shared__ double lds_d8[NW][8][32], lds_s8[NW][8][32];
  __shared__ double lds_acc[NW > 1 ? 16 * 64 : 1];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int n0 = blockIdx.x * 32;
  const int n = min(n0 + col, N - 1);                 // rows past N recompute row N-1 and are not stored
  const uint8_t* wrow = W + (int64_t)n * nb * 144;
  const int64_t xrow_bytes = (int64_t)nb * 8 * 36;
  // A operand: batch row `col` (rows past B re-read row B-1; their results are not stored)
  const uint8_t* xrow = xq + (int64_t)min(col, B - 1) * xrow_bytes + 16 * half;

  double acc[16];
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0;

  for (int blk = wave; blk < nb; blk += NW) {
    // weights of this lane's row: header + its half of every 32-byte nibble group
    const uint4 hdr = *(const uint4*)(wrow + blk * 144);
    uint4 qs[4];
#pragma unroll
    for (int g = 0; g < 4; g++) qs[g] = *(const uint4*)(wrow + blk * 144 + 16 + 32 * g + 16 * half);
    // activations: the lane's 16 int8 of each of the 8 sub-blocks (4-byte aligned 16-byte loads)
    uint4 xa4[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const uint32_t* p = (const uint32_t*)(xrow + (int64_t)(blk * 8 + j) * 36);
      xa4[j] = make_uint4(p[0], p[1], p[2], p[3]);
    }
    // scales of the 32 x 8 activation blocks of this super-block -> LDS of this wave, 4 per lane
    __builtin_amdgcn_wave_barrier();     // the previous super-block's scales have been consumed by every lane
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int t = lane + 64 * i;
      const int b = t >> 3, j = t & 7;
      const uint32_t ds = *(const uint32_t*)(xq + (int64_t)min(b, B - 1) * xrow_bytes + (int64_t)(blk * 8 + j) * 36 + 32);
      lds_d8[wave][j][b] = (double)half_to_f32((uint16_t)(ds & 0xffffu));
      lds_s8[wave][j][b] = (double)half_to_f32((uint16_t)(ds >> 16));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    const float d = half_to_f32((uint16_t)(hdr.x & 0xffffu)), dmin = half_to_f32((uint16_t)(hdr.x >> 16));
    // all eight 6-bit scales and mins of the block, four per dword
    const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu, m_lo = hdr.z & 0x3f3f3f3fu;
    const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
    const uint32_t m_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);

    double sblk[16], mblk[16];
#pragma unroll
    for (int r = 0; r < 16; r++) { sblk[r] = 0.0; mblk[r] = 0.0; }

#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int g = j >> 1;
      const uint4 q = qs[g];
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
      // A = activations (M = batch row), B = weights (N = weight row): c[r] = I_j[b = mfma32_row(r), n = col]
      c = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa, wb, c, 0, 0, 0);
      const int sc = (int)(((j < 4 ? sc_lo : sc_hi) >> (8 * (j & 3))) & 0xffu);
      const double mj = (double)(((j < 4 ? m_lo : m_hi) >> (8 * (j & 3))) & 0xffu);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int b = mfma32_row(r, half);
        const int p = __mul24(sc, c[r]);                            // 6-bit x 17-bit: exact
        sblk[r] = fma(lds_d8[wave][j][b], (double)p, sblk[r]);
        mblk[r] = fma(mj, lds_s8[wave][j][b], mblk[r]);
      }
    }
    const double dd = (double)d, dm = (double)dmin;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] += dd * sblk[r] - dm * mblk[r];
  }

  if (NW > 1) {
    // partial sums meet in wave order; the last wave ends up with the totals
    for (int w = 0; w < NW; w++) {
      if (wave == w) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          if (w > 0) acc[r] += lds_acc[r * 64 + lane];
          if (w < NW - 1) lds_acc[r * 64 + lane] = acc[r];
        }
      }
      if (w < NW - 1) __syncthreads();
    }
    if (wave != NW - 1) return;
  }

  if (n0 + col < N) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int b = mfma32_row(r, half);
      if (b >= B) continue;
      const int64_t o = (int64_t)b * N + n0 + col;
      const float v = (float)acc[r];
      if (EPI == GEPI_F32) ((float*)out)[o] = v;
      else if (EPI == GEPI_BF16) ((uint16_t*)out)[o] = f32_to_bf16(v);
      else ((uint16_t*)out)[o] = f32_to_bf16(bf16_to_f32(f32_to_bf16(v)) + bf16_to_f32(res[o]));
    }
  }
}

int g_tune_gemm_nw = 0;      // waves per tile (1, 2, 4, 8); 0 = chosen from the shape

template <int NW>
static void launch_gemm_nw(int epi, dim3 grid, const uint8_t* w, const uint8_t* x, void* y, const uint16_t* r, int N, int nb, int batch) {
  const dim3 block(64 * NW);
  if (epi == GEPI_F32) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<GEPI_F32, NW>), grid, block, 0, stream(), w, x, y, r, N, nb, batch);
  else if (epi == GEPI_BF16) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<GEPI_BF16, NW>), grid, block, 0, stream(), w, x, y, r, N, nb, batch);
  else hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<GEPI_BF16_ADD, NW>), grid, block, 0, stream(), w, x, y, r, N, nb, batch);
}

int launch_gemm_q4k_q8_1_mfma(const void* W, const void* xq, void* y, int N, int K, int batch, int out_dtype,
                              const void* residual) {
  BK_REQUIRE(W && xq && y, "gemm_q4k_q8_1_mfma: null pointer");
  BK_REQUIRE(N > 0 && K > 0 && K % 256 == 0, "gemm_q4k_q8_1_mfma: K=%d must be a positive multiple of 256 (N=%d)", K, N);
  BK_REQUIRE(batch >= 1 && batch <= 32, "gemm_q4k_q8_1_mfma: batch=%d must be 1..32", batch);
  BK_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "gemm_q4k_q8_1_mfma: out_dtype must be 0 (f32) or 1 (bf16)");
  BK_REQUIRE(!(residual && out_dtype != DT_BF16), "gemm_q4k_q8_1_mfma: a residual needs bf16 output");
  BK_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)xq & 3) == 0, "gemm_q4k_q8_1_mfma: W must be 16-byte and xq 4-byte aligned");
  const dim3 grid((N + 31) / 32);
  const uint8_t* w = (const uint8_t*)W; const uint8_t* x = (const uint8_t*)xq; const uint16_t* r = (const uint16_t*)residual;
  const int nb = K / 256;
  const int epi = out_dtype == DT_F32 ? GEPI_F32 : (residual ? GEPI_BF16_ADD : GEPI_BF16);
  // waves per tile (measured on the decode shapes at batch 32): long rows split eight ways, K = 2048 four ways,
  // and two ways when the tiles alone fill the chip many times over (lm_head)
  int nw = g_tune_gemm_nw;
  if (nw <= 0) {
    const int tiles = (N + 31) / 32;
    nw = nb >= 16 ? 8 : (nb >= 4 ? 4 : (nb >= 2 ? 2 : 1));
    if (tiles >= 8 * num_cus() && nw > 2) nw = 2;
  }
  if (nw >= 8) launch_gemm_nw<8>(epi, grid, w, x, y, r, N, nb, batch);
  else if (nw >= 4) launch_gemm_nw<4>(epi, grid, w, x, y, r, N, nb, batch);
  else if (nw >= 2) launch_gemm_nw<2>(epi, grid, w, x, y, r, N, nb, batch);
  else launch_gemm_nw<1>(epi, grid, w, x, y, r, N, nb, batch);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
