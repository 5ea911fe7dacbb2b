// Q4_K dequant-GEMV kernels for gfx950: y[N] = W[N,K] . x[K], W in 144-byte
// super-blocks, streamed once from HBM with 128-bit loads.
//
// Lane mapping (all kernels here).  A wavefront walks whole weight rows.  The
// 128 nibble bytes of a super-block are 8 chunks of 16 bytes; "slot"
// s = 64*round + lane covers chunk c = s & 7 of block s >> 3, so one wave-wide
// 16-byte load fetches the nibbles of 8 consecutive blocks (1 KiB contiguous
// but for the 16-byte headers, which a second, 8-way broadcast load fetches).
// Chunk c holds, for l in [16*(c&1), 16*(c&1)+16), the low nibbles of
// sub-block 2*(c>>1) and the high nibbles of sub-block 2*(c>>1)+1.  The slice
// of the activation a lane needs therefore depends on the lane only, not on
// the row: it is loaded once into registers and reused for every row.
//
// Arithmetic.  The sub-block dots are exact int32.  Everything after them is carried
// in double: d*d8 (two fp16 values) is exact in f32, times the 6-bit scale and the
// integer dot it is exact in double, so a row's value is a sum of exactly known terms
// with ~1e-16 relative accumulation error, rounded once to f32.  The result therefore
// does not depend on the lane mapping, the launch shape or the batch size, and equals
// a plain host loop in double to the bit (up to ~1e-8 probability per output).
#include "gemv_tile.h"

namespace bk {

// NR = number of 64-slot rounds per row (K = 2048*NR when the row fills every round);
// RPI = rows a wave handles per step (all their loads are issued before any is consumed).
template <int NR, int EPI, int RPI>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_q4k_q8_1_kernel(
    const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq_all, void* __restrict__ y,
    const uint16_t* __restrict__ res, int N, int nb) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * GEMV_WAVES;
  const int bidx = blockIdx.y;
  const uint8_t* xq = xq_all + (int64_t)bidx * nb * 8 * 36;
  const int c = lane & 7;
  const ScaleSel sel = make_scale_sel(c);
  const int64_t row_bytes = (int64_t)nb * 144;
  const int64_t ybase = (int64_t)bidx * N;
  const bool odd = c & 1;
  const int step = nwaves * RPI;
  int row0 = wave * RPI;

  int boff[NR];   // byte offset of the slot's block inside a row
#pragma unroll
  for (int r = 0; r < NR; r++) {
    const int blk = r * 8 + (lane >> 3);
    boff[r] = (blk < nb ? blk : 0) * 144;
  }
  RowTile<NR, RPI> t0;
  XQ x[NR];
#pragma unroll
  for (int r = 0; r < NR; r++) {
    const int blk = r * 8 + (lane >> 3);
    load_xq(x[r], xq, blk, c, blk < nb);
  }

  for (; row0 < N; row0 += step) {
    load_rows<NR, RPI>(t0, W, row_bytes, row0, N, boff, c);
    fold_rows<NR, EPI, RPI>(t0, x, sel, odd, lane, y, res, ybase, row0, N);
  }
}

// ---------------------------------------------------------------- rows through LDS
// Same lane mapping and arithmetic as above, but the weight bytes travel HBM -> registers ->
// LDS -> registers: a step's RPI rows are contiguous in memory (RPI * NR * 72 pieces of 16 bytes),
// so the wave fetches them with fully coalesced loads (lane l takes piece l, l + 64, ...: every
// 128-byte line is requested exactly once and no header is fetched eight times), parks them in
// its private LDS tile and reads headers and nibble chunks back in the (block, chunk) mapping.
// The loads of the next step are in flight while the current step is folded.
template <int NR, int EPI, int RPI>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_q4k_q8_1_lds_kernel(
    const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq_all, void* __restrict__ y,
    const uint16_t* __restrict__ res, int N) {
  constexpr int PIECES = RPI * NR * 72;
  __shared__ uint4 tiles[GEMV_WAVES][PIECES];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int wave = blockIdx.x * GEMV_WAVES + wv;
  const int nwaves = gridDim.x * GEMV_WAVES;
  const int bidx = blockIdx.y;
  constexpr int nb = NR * 8;
  const uint8_t* xq = xq_all + (int64_t)bidx * nb * 8 * 36;
  const int c = lane & 7, b = lane >> 3;
  const ScaleSel sel = make_scale_sel(c);
  constexpr int64_t row_bytes = (int64_t)nb * 144;
  const int64_t last_piece_off = (int64_t)N * row_bytes - 16;
  const int64_t ybase = (int64_t)bidx * N;
  const bool odd = c & 1;
  const int step = nwaves * RPI;
  int row0 = wave * RPI;
  uint4* tile = tiles[wv];

  // the activation slice first, the weight rows right behind it: loads return in issue order, and the slice
  // (cache-resident) must not queue up behind rows that come from HBM
  XQ x[NR];
#pragma unroll
  for (int r = 0; r < NR; r++) load_xq(x[r], xq, r * 8 + b, c, true);

  StageRegs<NR, RPI> g;
  stage_load<NR, RPI>(g, W, (int64_t)min(row0, N - 1) * row_bytes, last_piece_off, lane);

  while (row0 < N) {
    stage_park<NR, RPI>(g, tile, lane);
    if (row0 + step < N) stage_load<NR, RPI>(g, W, (int64_t)(row0 + step) * row_bytes, last_piece_off, lane);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    RowTile<NR, RPI> t;
#pragma unroll
    for (int i = 0; i < RPI; i++) {
#pragma unroll
      for (int r = 0; r < NR; r++) {
        const int blk = (i * NR + r) * 72 + b * 9;       // piece index of the block header
        t.hdr[i][r] = tile[blk];
        t.q[i][r] = tile[blk + 1 + c];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                     // every lane has read its pieces before the tile is overwritten
    fold_rows<NR, EPI, RPI>(t, x, sel, odd, lane, y, res, ybase, row0, N);
    row0 += step;
  }
}

// Any K that is a multiple of 256: rounds are a run-time loop and the activation
// slice is re-read (from L2) in every round.
template <int EPI>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_q4k_q8_1_generic_kernel(
    const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq_all, void* __restrict__ y,
    const uint16_t* __restrict__ res, int N, int nb) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * GEMV_WAVES;
  const int bidx = blockIdx.y;
  const uint8_t* xq = xq_all + (int64_t)bidx * nb * 8 * 36;
  const int c = lane & 7;
  const ScaleSel sel = make_scale_sel(c);
  const int64_t row_bytes = (int64_t)nb * 144;
  const int rounds = (nb + 7) / 8;
  for (int row = wave; row < N; row += nwaves) {
    const uint8_t* rp = W + (int64_t)row * row_bytes;
    double acc = 0.0;
    for (int r = 0; r < rounds; r++) {
      const int blk = r * 8 + (lane >> 3);
      const bool active = blk < nb;
      XQ x;
      load_xq(x, xq, blk, c, active);
      const int bo = (active ? blk : 0) * 144;
      const uint4 hdr = *(const uint4*)(rp + bo);
      const uint4 q = *(const uint4*)(rp + bo + 16 + 16 * c);
      int I0, I1;
      acc += slot_dot(hdr, q, x, sel, I0, I1, c & 1);
    }
    const float tot = (float)wave_sum_f64(acc);
    if (lane == 0) store_out<EPI>(y, res, (int64_t)bidx * N + row, tot);
  }
}

// Exact int32 sub-block dots I[N, 8*nb]: lane pairs (c even, c odd) hold the two
// 16-element halves of sub-blocks 2g and 2g+1.
__global__ __launch_bounds__(GEMV_WAVES * 64) void q4k_q8_1_subdots_kernel(
    const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq, int32_t* __restrict__ I, int N, int nb) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * GEMV_WAVES;
  const int c = lane & 7;
  const ScaleSel sel = make_scale_sel(c);
  const int64_t row_bytes = (int64_t)nb * 144;
  const int rounds = (nb + 7) / 8;
  for (int row = wave; row < N; row += nwaves) {
    const uint8_t* rp = W + (int64_t)row * row_bytes;
    for (int r = 0; r < rounds; r++) {
      const int blk = r * 8 + (lane >> 3);
      const bool active = blk < nb;
      XQ x;
      load_xq(x, xq, blk, c, active);
      const int bo = (active ? blk : 0) * 144;
      const uint4 hdr = *(const uint4*)(rp + bo);
      const uint4 q = *(const uint4*)(rp + bo + 16 + 16 * c);
      int I0, I1;
      (void)slot_dot(hdr, q, x, sel, I0, I1, c & 1);
      const int s0 = I0 + dpp_i32<DPP_QUAD_XOR1>(I0);
      const int s1 = I1 + dpp_i32<DPP_QUAD_XOR1>(I1);
      if (active) I[(int64_t)row * nb * 8 + blk * 8 + c] = (c & 1) ? s1 : s0;
    }
  }
}

int g_tune_gemv_impl = 2;               // 2: rows staged through LDS when K is a multiple of 2048 (else as 0),
                                        // 0: direct loads in the (block, chunk) mapping
int g_tune_rpi = 0, g_tune_cap = 16;     // tuning hooks (bk_tune_set): rows per wave step (0: from the shape), workgroups per CU
int g_tune_steps = 0;                    // > 0: the grid that gives every wave this many row steps (the last one may be short)

// Workgroups for a launch that needs `wgs` of them at one row step per wave.  Up to the cap (16 per CU) that many; a
// longer matrix gets the grid in which every wave takes exactly two steps (the second one's rows are in flight while
// the first is folded).  Measured on the 151936 x 2048 matrix, four rows per step: one step per wave 28.9 us, two 27.4,
// three 28.7, four 29.4, eight 30.6, and 28.0-29.3 with the grid cut at the cap, where some waves take three steps and
// the rest two.
int gemv_grid_for(int wgs) {
  if (g_tune_steps > 0) return (wgs + g_tune_steps - 1) / g_tune_steps;
  const int cap = num_cus() * g_tune_cap;
  return wgs <= cap ? wgs : (wgs + 1) / 2;
}

static int gemv_grid(int N, int rows_per_wg) { return gemv_grid_for((N + rows_per_wg - 1) / rows_per_wg); }

template <int NR, int EPI>
static void launch_q8_1_rpi(dim3 block, const uint8_t* w, const uint8_t* x, void* y, const uint16_t* r, int N, int nb, int batch) {
  const int rpi = (g_tune_rpi == 1 || g_tune_rpi == 2) ? g_tune_rpi : 4;
  dim3 grid(gemv_grid(N, GEMV_WAVES * rpi), batch);
  if (rpi == 1) hipLaunchKernelGGL((gemv_q4k_q8_1_kernel<NR, EPI, 1>), grid, block, 0, stream(), w, x, y, r, N, nb);
  else if (rpi == 2) hipLaunchKernelGGL((gemv_q4k_q8_1_kernel<NR, EPI, 2>), grid, block, 0, stream(), w, x, y, r, N, nb);
  else { grid.x = gemv_grid(N, GEMV_WAVES * 4); hipLaunchKernelGGL((gemv_q4k_q8_1_kernel<NR, EPI, 4>), grid, block, 0, stream(), w, x, y, r, N, nb); }
}

template <int NR, int EPI>
static void launch_q8_1_lds(dim3 block, const uint8_t* w, const uint8_t* x, void* y, const uint16_t* r, int N, int batch) {
  // rows of 2048: two rows per wave step while the matrix is small (twice the workgroups in flight: qkv 3.95 -> 3.65 us,
  // gate+up 4.8 -> 4.7), four for a long one (lm_head: 29.8 us against 33 with two)
  const int rpi = NR == 1 ? ((g_tune_rpi == 2 || (g_tune_rpi == 0 && N <= 16384)) ? 2 : 4) : 2;
  dim3 grid(gemv_grid(N, GEMV_WAVES * rpi), batch);
  if (NR == 1 && rpi == 4) hipLaunchKernelGGL((gemv_q4k_q8_1_lds_kernel<NR, EPI, (NR == 1 ? 4 : 2)>), grid, block, 0, stream(), w, x, y, r, N);
  else hipLaunchKernelGGL((gemv_q4k_q8_1_lds_kernel<NR, EPI, 2>), grid, block, 0, stream(), w, x, y, r, N);
}

template <int EPI>
static void launch_q8_1_variant(const void* W, const void* xq, void* y, const void* res, int N, int nb, int batch) {
  const int rounds = (nb + 7) / 8;
  dim3 block(GEMV_WAVES * 64);
  dim3 grid(1, batch);
  const uint8_t* w = (const uint8_t*)W; const uint8_t* x = (const uint8_t*)xq; const uint16_t* r = (const uint16_t*)res;
  switch (rounds) {
    case 1: if (g_tune_gemv_impl == 2 && nb == 8) launch_q8_1_lds<1, EPI>(block, w, x, y, r, N, batch); else launch_q8_1_rpi<1, EPI>(block, w, x, y, r, N, nb, batch);
      break;
    case 2: if (g_tune_gemv_impl == 2 && nb == 16) launch_q8_1_lds<2, EPI>(block, w, x, y, r, N, batch); else launch_q8_1_rpi<2, EPI>(block, w, x, y, r, N, nb, batch);
      break;
    case 3: if (g_tune_gemv_impl == 2 && nb == 24) launch_q8_1_lds<3, EPI>(block, w, x, y, r, N, batch); else launch_q8_1_rpi<3, EPI>(block, w, x, y, r, N, nb, batch);
      break;
    default:
      grid.x = gemv_grid(N, GEMV_WAVES);
      hipLaunchKernelGGL((gemv_q4k_q8_1_generic_kernel<EPI>), grid, block, 0, stream(), w, x, y, r, N, nb);
  }
}

int launch_gemv_q4k_q8_1(const void* W, const void* xq, void* y, int N, int K, int batch, int out_dtype,
                         const void* residual) {
  BK_REQUIRE(W && xq && y, "gemv_q4k_q8_1: null pointer");
  BK_REQUIRE(N > 0 && K > 0 && K % 256 == 0, "gemv_q4k_q8_1: K=%d must be a positive multiple of 256 (N=%d)", K, N);
  BK_REQUIRE(batch > 0 && batch <= 65535, "gemv_q4k_q8_1: bad batch=%d", batch);
  BK_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "gemv_q4k_q8_1: out_dtype must be 0 (f32) or 1 (bf16)");
  BK_REQUIRE(!(residual && out_dtype != DT_BF16), "gemv_q4k_q8_1: a residual needs bf16 output");
  BK_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)xq & 3) == 0, "gemv_q4k_q8_1: W must be 16-byte and xq 4-byte aligned");
  const int nb = K / 256;
  if (out_dtype == DT_F32) launch_q8_1_variant<EPI_F32>(W, xq, y, nullptr, N, nb, batch);
  else if (!residual) launch_q8_1_variant<EPI_BF16>(W, xq, y, nullptr, N, nb, batch);
  else launch_q8_1_variant<EPI_BF16_ADD>(W, xq, y, residual, N, nb, batch);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

int launch_q4k_q8_1_subdots(const void* W, const void* xq, int32_t* I, int N, int K) {
  BK_REQUIRE(W && xq && I, "q4k_q8_1_subdots: null pointer");
  BK_REQUIRE(N > 0 && K > 0 && K % 256 == 0, "q4k_q8_1_subdots: K=%d must be a positive multiple of 256", K);
  BK_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)xq & 3) == 0, "q4k_q8_1_subdots: misaligned pointer");
  hipLaunchKernelGGL(q4k_q8_1_subdots_kernel, dim3(gemv_grid(N, GEMV_WAVES)), dim3(GEMV_WAVES * 64), 0, stream(),
                     (const uint8_t*)W, (const uint8_t*)xq, I, N, K / 256);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- f32 activations
// Dequantise-and-dot with x in f32: per slot, 16 low-nibble and 16 high-nibble
// weights against 32 activation values held in registers.
//   y += d*sc0*sum(nib_lo*x_lo) - dmin*m0*sum(x_lo) + d*sc1*sum(nib_hi*x_hi) - dmin*m1*sum(x_hi)
struct XF {
  float lo[16], hi[16];
  float sum_c;   // sum of the 32 activations of sub-block c (for the lane's share of the mins)
};

__device__ __forceinline__ float nibdot4(uint32_t n4, const float* x, float acc) {
  acc = fmaf((float)(n4 & 0xffu), x[0], acc);
  acc = fmaf((float)((n4 >> 8) & 0xffu), x[1], acc);
  acc = fmaf((float)((n4 >> 16) & 0xffu), x[2], acc);
  acc = fmaf((float)(n4 >> 24), x[3], acc);
  return acc;
}

template <int NR>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_q4k_f32_kernel(
    const uint8_t* __restrict__ W, const float* __restrict__ xf, float* __restrict__ y, int N, int nb) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * GEMV_WAVES;
  const int c = lane & 7, g = c >> 1, half = c & 1;
  const ScaleSel sel = make_scale_sel(c);
  const int64_t row_bytes = (int64_t)nb * 144;
  const int rounds = NR > 0 ? NR : (nb + 7) / 8;

  XF x[NR > 0 ? NR : 1];
  int boff[NR > 0 ? NR : 1];
  auto load_x = [&](XF& xx, int blk, bool active) {
    if (!active) {
#pragma unroll
      for (int i = 0; i < 16; i++) { xx.lo[i] = 0.0f; xx.hi[i] = 0.0f; }
      xx.sum_c = 0.0f;
      return;
    }
    const float4* p0 = (const float4*)(xf + blk * 256 + 64 * g + 16 * half);
    const float4* p1 = (const float4*)(xf + blk * 256 + 64 * g + 32 + 16 * half);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float4 a = p0[i], b = p1[i];
      xx.lo[4 * i] = a.x; xx.lo[4 * i + 1] = a.y; xx.lo[4 * i + 2] = a.z; xx.lo[4 * i + 3] = a.w;
      xx.hi[4 * i] = b.x; xx.hi[4 * i + 1] = b.y; xx.hi[4 * i + 2] = b.z; xx.hi[4 * i + 3] = b.w;
    }
    // sum of sub-block c = elements [32c', ...): sub-block j covers 64*(j>>1) + 32*(j&1) + [0,32)
    const float4* ps = (const float4*)(xf + blk * 256 + 64 * (c >> 1) + 32 * (c & 1));
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) { const float4 v = ps[i]; s += (v.x + v.y) + (v.z + v.w); }
    xx.sum_c = s;
  };
  if (NR > 0) {
#pragma unroll
    for (int r = 0; r < (NR > 0 ? NR : 1); r++) {
      const int blk = r * 8 + (lane >> 3);
      load_x(x[r], blk, blk < nb);
      boff[r] = (blk < nb ? blk : 0) * 144;
    }
  }

  for (int row = wave; row < N; row += nwaves) {
    const uint8_t* rp = W + (int64_t)row * row_bytes;
    float acc = 0.0f;
#pragma unroll
    for (int r = 0; r < rounds; r++) {
      const int ri = NR > 0 ? r : 0;
      if (NR == 0) {
        const int blk = r * 8 + (lane >> 3);
        load_x(x[0], blk, blk < nb);
        boff[0] = (blk < nb ? blk : 0) * 144;
      }
      const uint4 hdr = *(const uint4*)(rp + boff[ri]);
      const uint4 q = *(const uint4*)(rp + boff[ri] + 16 + 16 * c);
      const float d = half_to_f32((uint16_t)(hdr.x & 0xffffu));
      const float dmin = half_to_f32((uint16_t)(hdr.x >> 16));
      uint32_t sc, m;
      lane_scale_min(sel, hdr.y, hdr.z, hdr.w, sc, m);
      const float fsc = d * (float)sc;
      const float fm = (dmin * (float)m) * x[ri].sum_c;
      float a = 0.0f, b = 0.0f;
      a = nibdot4(q.x & 0x0f0f0f0fu, &x[ri].lo[0], a);
      b = nibdot4((q.x >> 4) & 0x0f0f0f0fu, &x[ri].hi[0], b);
      a = nibdot4(q.y & 0x0f0f0f0fu, &x[ri].lo[4], a);
      b = nibdot4((q.y >> 4) & 0x0f0f0f0fu, &x[ri].hi[4], b);
      a = nibdot4(q.z & 0x0f0f0f0fu, &x[ri].lo[8], a);
      b = nibdot4((q.z >> 4) & 0x0f0f0f0fu, &x[ri].hi[8], b);
      a = nibdot4(q.w & 0x0f0f0f0fu, &x[ri].lo[12], a);
      b = nibdot4((q.w >> 4) & 0x0f0f0f0fu, &x[ri].hi[12], b);
      const float f0 = dpp_f32<DPP_PAIR_EVEN>(fsc);
      const float f1 = dpp_f32<DPP_PAIR_ODD>(fsc);
      acc += (f0 * a + f1 * b) - fm;
    }
    const float tot = wave_sum(acc);
    if (lane == 0) y[row] = tot;
  }
}

int launch_gemv_q4k_f32(const void* W, const float* x, float* y, int N, int K) {
  BK_REQUIRE(W && x && y, "gemv_q4k_f32: null pointer");
  BK_REQUIRE(N > 0 && K > 0 && K % 256 == 0, "gemv_q4k_f32: K=%d must be a positive multiple of 256 (N=%d)", K, N);
  BK_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)x & 15) == 0, "gemv_q4k_f32: W and x must be 16-byte aligned");
  const int nb = K / 256, rounds = (nb + 7) / 8;
  dim3 block(GEMV_WAVES * 64), grid(gemv_grid(N, GEMV_WAVES));
  const uint8_t* w = (const uint8_t*)W;
  switch (rounds) {
    case 1: hipLaunchKernelGGL((gemv_q4k_f32_kernel<1>), grid, block, 0, stream(), w, x, y, N, nb); break;
    case 2: hipLaunchKernelGGL((gemv_q4k_f32_kernel<2>), grid, block, 0, stream(), w, x, y, N, nb); break;
    default: hipLaunchKernelGGL((gemv_q4k_f32_kernel<0>), grid, block, 0, stream(), w, x, y, N, nb);
  }
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
