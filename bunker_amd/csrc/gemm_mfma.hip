// Batched decode matmul: C[B, N] = Xq[B, K] . W[N, K]^T for tiles of up to 32 activation rows in
// Q8_1 and W in Q4_K, on the int8 matrix cores.  Precedent in the reference:
// int8MatmulTTIR (src/kernel.ts:397-417), i8 x i8 -> i32 exact, and its documented
// post-scale (experiments/q4k_q81_final.ts:214-217).
//
// One v_mfma_i32_32x32x32_i8 consumes exactly one 32-element sub-block of K for a tile
// of 32 weight rows (M) x 32 activation rows (N), so the matrix core produces the exact
// int32 sub-block dots I_j[n, b].  A lane owns activation row b = lane % 32 and 16 of the 32
// weight rows; it folds the dots with the scales in double, in the same way the GEMV does
// (every term exact, ~1e-16 accumulation error, one rounding to f32), so the batched
// path returns the same bits as the batch-1 path:
//   y[b, n] = sum_blk ( d * sum_j d8_j[b] * (sc_j * I_j) - dmin * sum_j m_j * s8_j[b] )
// The first sum is folded on the vector unit: per dot one 24-bit integer multiply by the 6-bit scale (a byte the
// lane's 16 rows share with its half of the wave, fetched from LDS 16 at a time), one conversion and one FMA with
// the lane's own activation scale; d comes in once per super-block.  The second sum is a small dense product over
// the sub-blocks of K and runs on the double-precision matrix instruction (v_mfma_f64_16x16x4_f64), in its own
// accumulators that join the others once, at the end.
//
// Batches of more than 32 rows are cut into 32-row tiles (one launch, every (weight tile, batch tile) its own workgroup).
// A workgroup owns one 32 x 32 output tile; its NW wavefronts split K by super-block (wave w takes
// blocks w, w + NW, ...) and add their double partials in wave order through LDS at the end.
// Each wave copies the 32 x 144 weight bytes and the 32 x 288 activation bytes of its super-block into its own
// part of LDS with loads in which four neighbouring lanes cover 64 contiguous bytes (a lane-per-row load touches 64
// cache lines per instruction and leaves the kernel bound by the rate of the L1's address path), one super-block
// ahead of the arithmetic, and every operand is then read from LDS.
#include "ops.h"

namespace bk {

typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(16))) int i32x16_t;
typedef __attribute__((ext_vector_type(4))) double f64x4_t;

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
  int nb, B, tiles, btiles;
  uint8_t* out_q8;        // SwiGLU form: g[0] = gate (out = bf16 activation or null), g[1] = up; Q8_1 blocks of the activation
};

// Compact argument blocks (a launch pays for every 64-byte line of kernel arguments, about a quarter of a microsecond;
// MfmaArgs has three lines): one matrix in 56 bytes, the SwiGLU pair in 60.  The kernel rebuilds MfmaArgs in registers.
struct MfmaArgs1 {
  const uint8_t* W; void* out; const uint16_t* res; const uint8_t* xq;
  int N, epi, nb, B, tiles, btiles;
};
struct MfmaArgsSw {
  const uint8_t *Wg, *Wu; void* act; uint8_t* act_q8; const uint8_t* xq;
  int N, nb, B, tiles, btiles;
};
__device__ __forceinline__ const MfmaArgs& mfma_args_full(const MfmaArgs& A) { return A; }
__device__ __forceinline__ MfmaArgs mfma_args_full(const MfmaArgs1& P) {
  MfmaArgs A;
  const MfmaGroup g{P.W, P.out, P.res, P.N, P.epi};
  A.g[0] = g; A.g[1] = g; A.g[2] = g; A.g[3] = g;
  A.tile_first[0] = 0; A.tile_first[1] = A.tile_first[2] = A.tile_first[3] = A.tile_first[4] = P.tiles;
  A.xq = P.xq; A.nb = P.nb; A.B = P.B; A.tiles = P.tiles; A.btiles = P.btiles; A.out_q8 = nullptr;
  return A;
}
__device__ __forceinline__ MfmaArgs mfma_args_full(const MfmaArgsSw& P) {
  MfmaArgs A;
  const MfmaGroup g0{P.Wg, P.act, nullptr, P.N, 0}, g1{P.Wu, nullptr, nullptr, P.N, 0};
  A.g[0] = g0; A.g[1] = g1; A.g[2] = g1; A.g[3] = g1;
  A.tile_first[0] = 0; A.tile_first[1] = A.tile_first[2] = A.tile_first[3] = A.tile_first[4] = P.tiles;
  A.xq = P.xq; A.nb = P.nb; A.B = P.B; A.tiles = P.tiles; A.btiles = P.btiles; A.out_q8 = P.act_q8;
  return A;
}

enum : int { GX_ROW = 292, GW_ROW = 144, GX_BYTES = 32 * GX_ROW, GW_BYTES = 32 * GW_ROW, G_WAVE_LDS = GX_BYTES + GW_BYTES + 512 };

// SWIGLU: the workgroup holds 2 NW waves; waves 0..NW-1 form the tile of 32 gate rows, waves NW..2NW-1 the tile of the
// same 32 up rows, and the last step writes act = bf16(silu(g) * u) and its Q8_1 block instead of g and u.
// TR: weight rows of the tile.  16 or 8 (the other rows of the matrix instruction repeat them and are ignored) for launches
// with so few tiles that the time is the length of one wave's instruction stream: a half or a quarter of the fold per
// super-block, two or four times the tiles.
template <int NW, bool SWIGLU, int TR = 32, typename ARGS = MfmaArgs>
__global__ __launch_bounds__(64 * NW * (SWIGLU ? 2 : 1)) void gemm_q4k_q8_1_mfma_kernel(ARGS A_in) {
  const auto& A = mfma_args_full(A_in);
  static_assert(TR == 32 || TR == 16 || TR == 8, "tiles of 32, 16 or 8 weight rows");
  static_assert(!(SWIGLU && TR != 32), "the SwiGLU form quantizes 32 outputs at a time");
  constexpr int WAVES = NW * (SWIGLU ? 2 : 1);
  constexpr int RF = TR / 2;               // weight rows per lane
  constexpr int TN = TR >= 16 ? TR / 16 : 1;   // 16-row groups (min term; a tile of 8 fills half of one, the rest repeats it)
  // Per wave: the activation rows of the current super-block as they lie in memory (288 bytes, rows 292 apart so that
  // the lanes of a read fall into different banks), the weight rows (144 bytes each), and 512 bytes of weight scales
  // in the order the fold reads them (the 6-bit scales as bytes [8 sub-blocks][2 halves][16 rows], then d as doubles
  // [2 halves][16 rows]).  After the K loop the same memory holds the waves' partial sums [WAVES][16][64].
  __shared__ __align__(16) unsigned char lds_raw[WAVES * G_WAVE_LDS];
  static_assert(G_WAVE_LDS >= 16 * 64 * 8 && G_WAVE_LDS % 16 == 0, "the partial sums share the staging memory");

  // Workgroup -> (weight tile, batch tile).  With several batch tiles the workgroups that share a weight tile run next
  // to each other on one XCD (consecutive workgroup ids go round the 8 XCDs), batch tile fastest: the weight tile comes
  // from memory once and its other readers find it in that XCD's L2, where the activation rows stay resident.
  int tile = blockIdx.x, btile = 0;
  if (A.btiles > 1) {
    const int per_xcd = (A.tiles * A.btiles + 7) >> 3;
    const int v = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (v >= A.tiles * A.btiles) return;
    tile = v / A.btiles;
    btile = v - tile * A.btiles;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kw = SWIGLU ? wave % NW : wave;           // this wave's place in the split of K
  const bool s1 = !SWIGLU && tile >= A.tile_first[1], s2 = !SWIGLU && tile >= A.tile_first[2], s3 = !SWIGLU && tile >= A.tile_first[3];
  const uint8_t* __restrict__ W = SWIGLU ? (wave >= NW ? A.g[1].W : A.g[0].W) : s3 ? A.g[3].W : s2 ? A.g[2].W : s1 ? A.g[1].W : A.g[0].W;
  void* __restrict__ out = s3 ? A.g[3].out : s2 ? A.g[2].out : s1 ? A.g[1].out : A.g[0].out;
  const uint16_t* __restrict__ res = s3 ? A.g[3].res : s2 ? A.g[2].res : s1 ? A.g[1].res : A.g[0].res;
  const int N = s3 ? A.g[3].N : s2 ? A.g[2].N : s1 ? A.g[1].N : A.g[0].N;
  const int EPI = s3 ? A.g[3].epi : s2 ? A.g[2].epi : s1 ? A.g[1].epi : A.g[0].epi;
  const int nb = A.nb;
  const int b0 = btile * 32;                          // first batch row of this tile
  const int B = min(32, A.B - b0);
  const int64_t wrow_bytes = (int64_t)nb * 144, xrow_bytes = (int64_t)nb * 8 * 36;
  const uint8_t* __restrict__ xq = A.xq + (int64_t)b0 * xrow_bytes;

  const int half = lane >> 5, col = lane & 31, q4 = lane >> 4, l16 = lane & 15;
  const int n0 = (tile - (s3 ? A.tile_first[3] : s2 ? A.tile_first[2] : s1 ? A.tile_first[1] : 0)) * TR;
  unsigned char* const ldsX = lds_raw + wave * G_WAVE_LDS;
  unsigned char* const ldsW = ldsX + GX_BYTES;
  unsigned char* const stage = ldsW + GW_BYTES;

  // Copy maps.  Activations: instruction i = 2c + h covers bytes 64c.. of rows 16h + lane/4, 16 bytes per lane (the
  // last chunk has 32 bytes per row: lanes 2, 3 of a quad repeat lane 1's piece and do not store).  Rows past B re-read
  // row B-1 (their results are not stored).  Weights: piece p = lane + 64 i of the 288 16-byte pieces, row p / 9; rows
  // past N re-read row N-1.
  const int rq = lane >> 2, k4 = lane & 3;
  const uint8_t* xsrc[2] = {xq + (int64_t)min(rq, B - 1) * xrow_bytes + 16 * k4, xq + (int64_t)min(16 + rq, B - 1) * xrow_bytes + 16 * k4};
  const int xtail = 16 * min(k4, 1) - 16 * k4;                 // moves lanes 2, 3 back onto piece 17 in the last chunk
  unsigned char* const xdst[2] = {ldsX + rq * GX_ROW + 16 * k4, ldsX + (16 + rq) * GX_ROW + 16 * k4};
  const uint8_t* const wbase = W + (int64_t)n0 * wrow_bytes;
  uint32_t woff[5];
#pragma unroll
  for (int i = 0; i < 5; i++) {
    const int p = min(lane + 64 * i, TR * 9 - 1), row = p / 9;
    woff[i] = (uint32_t)((min(n0 + row, N - 1) - n0) * (int)wrow_bytes + (p - 9 * row) * 16);
  }
  uint4 xr[10], wr0, wr1, wr2, wr3, wr4;
#define GM_FETCH(BLK)                                                                                                  \
  {                                                                                                                    \
    const int fb_ = (BLK);                                                                                             \
    _Pragma("unroll") for (int i = 0; i < 10; i++) {                                                                   \
      const uint32_t* p_ = (const uint32_t*)(xsrc[i & 1] + (int64_t)fb_ * 288 + 64 * (i >> 1) + (i >= 8 ? xtail : 0)); \
      xr[i] = make_uint4(p_[0], p_[1], p_[2], p_[3]); /* 4-byte aligned 16-byte load */                                \
    }                                                                                                                  \
    wr0 = *(const uint4*)(wbase + (int64_t)fb_ * 144 + woff[0]);                                                       \
    wr1 = *(const uint4*)(wbase + (int64_t)fb_ * 144 + woff[1]);                                                       \
    if (TR >= 16) wr2 = *(const uint4*)(wbase + (int64_t)fb_ * 144 + woff[2]);                                         \
    if (TR == 32) {                                                                                                    \
      wr3 = *(const uint4*)(wbase + (int64_t)fb_ * 144 + woff[3]);                                                     \
      wr4 = *(const uint4*)(wbase + (int64_t)fb_ * 144 + woff[4]);                                                     \
    }                                                                                                                  \
  }

  // where the lane's own weight row sits among the rows of its half: row = 8g + 4h + v  ->  [h][4g + v]
  const int wcol = col & (TR - 1);
  const int stage_slot = ((wcol >> 2) & 1) * 16 + 4 * (wcol >> 3) + (wcol & 3);
  const unsigned char* const myW = ldsW + wcol * GW_ROW;        // int8 operands: weight row col, batch row col,
  const unsigned char* const myX = ldsX + col * GX_ROW;         // bytes 16*half.. of every sub-block

  double acc[RF];
#pragma unroll
  for (int r = 0; r < RF; r++) acc[r] = 0.0;
  f64x4_t accm[TN][2];
#pragma unroll
  for (int t = 0; t < 2 * TN; t++) accm[t >> 1][t & 1] = (f64x4_t){0.0, 0.0, 0.0, 0.0};

  GM_FETCH(min(kw, nb - 1));            // requests are unconditional (clamped): the waits stay countable
  for (int blk = kw; blk < nb; blk += NW) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();     // the previous super-block has been consumed by every lane
#pragma unroll
    for (int i = 0; i < 10; i++) {
      uint32_t* p = (uint32_t*)(xdst[i & 1] + 64 * (i >> 1));
      if (i < 8 || k4 < 2) { p[0] = xr[i].x; p[1] = xr[i].y; p[2] = xr[i].z; p[3] = xr[i].w; }
    }
    *(uint4*)(ldsW + lane * 16) = wr0;
    if (TR == 8) {
      if (lane < 8) *(uint4*)(ldsW + (lane + 64) * 16) = wr1;
    } else if (TR == 16) {
      *(uint4*)(ldsW + (lane + 64) * 16) = wr1;
      if (lane < 16) *(uint4*)(ldsW + (lane + 128) * 16) = wr2;
    } else {
      *(uint4*)(ldsW + (lane + 64) * 16) = wr1;
      *(uint4*)(ldsW + (lane + 128) * 16) = wr2;
      *(uint4*)(ldsW + (lane + 192) * 16) = wr3;
      if (lane < 32) *(uint4*)(ldsW + (lane + 256) * 16) = wr4;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // the next super-block's bytes travel while this one is folded.  Waves that split K have one to three blocks each: their
    // last pass requests nothing (a clamped request would double the loads of a one-block wave; out_proj at batch 32
    // 6.7 -> 6.2 us); a lone wave walks all of K and keeps the branch-free clamped request (1 % faster at 1024 rows)
    if (NW == 1 || blk + NW < nb) GM_FETCH(min(blk + NW, nb - 1));

    // the 6-bit scales of the lane's weight row (half 0 stages sub-blocks 0..3, half 1 sub-blocks 4..7) and its d
    {
      const uint4 hdr = *(const uint4*)myW;
      const uint32_t scw = half ? ((hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4)) : (hdr.y & 0x3f3f3f3fu);
#pragma unroll
      for (int i = 0; i < 4; i++) stage[(4 * half + i) * 32 + stage_slot] = (unsigned char)(scw >> (8 * i));
      if (!half) ((double*)(stage + 256))[stage_slot] = (double)half_to_f32((uint16_t)(hdr.x & 0xffffu));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // A = weights (M = weight row), B = activations (N = batch row): result[r] = I_j[n = mfma32_row(r), b = col]
    auto unpack = [](const uint4 q, int odd) {
      if (odd) return (i32x4_t){(int)((q.x >> 4) & 0x0f0f0f0fu), (int)((q.y >> 4) & 0x0f0f0f0fu), (int)((q.z >> 4) & 0x0f0f0f0fu),
                                (int)((q.w >> 4) & 0x0f0f0f0fu)};
      return (i32x4_t){(int)(q.x & 0x0f0f0f0fu), (int)(q.y & 0x0f0f0f0fu), (int)(q.z & 0x0f0f0f0fu), (int)(q.w & 0x0f0f0f0fu)};
    };
    auto load_x = [&](int j) {
      const uint32_t* xp = (const uint32_t*)(myX + j * 36 + 16 * half);
      return (i32x4_t){(int)xp[0], (int)xp[1], (int)xp[2], (int)xp[3]};
    };
    auto mfma = [](i32x4_t wb, i32x4_t xa) {
      i32x16_t z;
#pragma unroll
      for (int r = 0; r < 16; r++) z[r] = 0;
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(wb, xa, z, 0, 0, 0);
    };
    // The fold runs as a pipeline over the sub-blocks: the operands and scale bytes of sub-block j+1 are requested from
    // LDS before sub-block j is folded and its matrix instruction is issued halfway through that fold, when they have
    // arrived; the second half of the fold covers the matrix instruction's latency.  sc_j * I_j is an integer below 2^23;
    // its product with d8_j (11 bits) is exact inside the FMA, and so is d (11 bits) times the sum over the eight
    // sub-blocks as long as that sum has not been rounded (the terms of one activation row lie within a few binades of
    // each other).
    double S1[RF];
    uint4 q = *(const uint4*)(myW + 16 + 16 * half), qn = q;
    uint4 scb = *(const uint4*)(stage + 16 * half), scn = scb;
    uint32_t dsw = *(const uint32_t*)(myX + 32), dsn = dsw;
    i32x4_t xn = load_x(0);
    i32x16_t c = mfma(unpack(q, 0), xn), cn = c;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      if (j + 1 < 8) {
        scn = *(const uint4*)(stage + (j + 1) * 32 + 16 * half);
        dsn = *(const uint32_t*)(myX + (j + 1) * 36 + 32);
        xn = load_x(j + 1);
        if (j & 1) qn = *(const uint4*)(myW + 16 + 32 * ((j + 1) >> 1) + 16 * half);
      }
      __builtin_amdgcn_sched_barrier(0);
      const double d8 = (double)half_to_f32((uint16_t)(dsw & 0xffffu));
      const uint32_t scv[4] = {scb.x, scb.y, scb.z, scb.w};
#pragma unroll
      for (int r = 0; r < RF / 2; r++) {
        const double t = (double)__mul24(c[r], (int)((scv[r >> 2] >> (8 * (r & 3))) & 0xffu));
        S1[r] = j == 0 ? d8 * t : fma(d8, t, S1[r]);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (j + 1 < 8) {
        if (j & 1) q = qn;
        cn = mfma(unpack(q, (j + 1) & 1), xn);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = RF / 2; r < RF; r++) {
        const double t = (double)__mul24(c[r], (int)((scv[r >> 2] >> (8 * (r & 3))) & 0xffu));
        S1[r] = j == 0 ? d8 * t : fma(d8, t, S1[r]);
      }
      __builtin_amdgcn_sched_barrier(0);
      c = cn; scb = scn; dsw = dsn;
    }
    {
      const double2* dd = (const double2*)(stage + 256 + 128 * half);
#pragma unroll
      for (int r = 0; r < RF; r += 2) {
        const double2 v = dd[r >> 1];
        acc[r] = fma(v.x, S1[r], acc[r]);
        acc[r + 1] = fma(v.y, S1[r + 1], acc[r + 1]);
      }
    }
    // min term: accm[tn][tb] += (-dmin * m_j)[16 rows x 4 sub-blocks] . s8_j[4 sub-blocks x 16 batch rows], for the
    // sub-blocks 0..3 and then 4..7; a lane supplies row 16 t + l16 of either side at sub-blocks q4 and 4 + q4
    double am[TN][2], bm[2][2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
      if (t < TN) {
        const uint4 hm = *(const uint4*)(ldsW + ((16 * t + l16) & (TR - 1)) * GW_ROW);
        const float dmin_neg = -half_to_f32((uint16_t)(hm.x >> 16));
        const uint32_t zb = (hm.z >> (8 * q4)) & 0xffu, wb = (hm.w >> (8 * q4)) & 0xffu;
        am[t][0] = (double)(dmin_neg * (float)(zb & 63u));
        am[t][1] = (double)(dmin_neg * (float)((wb >> 4) | ((zb >> 6) << 4)));
      }
      const unsigned char* xs = ldsX + (16 * t + l16) * GX_ROW + q4 * 36 + 34;
      bm[t][0] = (double)half_to_f32(*(const uint16_t*)xs);
      bm[t][1] = (double)half_to_f32(*(const uint16_t*)(xs + 144));
    }
#pragma unroll
    for (int k = 0; k < 2; k++)
#pragma unroll
      for (int t = 0; t < 2 * TN; t++)
        accm[t >> 1][t & 1] = __builtin_amdgcn_mfma_f64_16x16x4f64(am[t >> 1][k], bm[t & 1][k], accm[t >> 1][t & 1], 0, 0, 0);
  }

  // The min-term accumulators hold element (n = 16 tn + 4 v + q4, b = 16 tb + l16); they reach the lanes that own those
  // outputs through this wave's part of the buffer.  Slot (r, lane) of a wave's part sits at r*64 + (lane ^ (r + 16*half)):
  // the swizzle keeps the transposed reads of the last step free of bank conflicts.
  double* part = (double*)lds_raw + wave * 16 * 64;
  __syncthreads();                         // all waves are done with the scales that share the buffer
#pragma unroll
  for (int t = 0; t < 2 * TN; t++)
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int n = 16 * (t >> 1) + 4 * v + q4, b = 16 * (t & 1) + l16;
      const int rr = 4 * (n >> 3) + (n & 3), hh = (n >> 2) & 1;
      part[rr * 64 + ((b + 32 * hh) ^ (rr + 16 * hh))] = accm[t >> 1][t & 1][v];
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int r = 0; r < RF; r++) acc[r] += part[r * 64 + (lane ^ (r + 16 * half))];

  // Last step: every wave leaves its 16 partial sums per lane in LDS; the threads then finish the outputs with the
  // weight row along the lanes (contiguous stores): thread (wave w, lane) takes row lane % 32 and batch rows
  // 2 (w R + i) + lane / 32, and adds the waves' partials in wave order.
  __builtin_amdgcn_wave_barrier();         // slot (r, lane) was read above by this lane only
#pragma unroll
  for (int r = 0; r < RF; r++) part[r * 64 + (lane ^ (r + 16 * half))] = acc[r];
  __syncthreads();
  const double* all = (const double*)lds_raw;
  // the thread's output row fn of the tile and its batch rows fb0 + FB * (wave R + i): 32 rows -> (lane % 32, lane / 32),
  // 16 rows -> (lane % 16, lane / 16), 8 rows -> (lane % 8, lane / 8)
  constexpr int R = TR / 2 / WAVES > 0 ? TR / 2 / WAVES : 1, FB = 64 / TR;
  if (wave * R * FB >= 32) return;         // (a 16-row tile gives each of eight waves one batch-row pair; an 8-row tile is finished by four waves)
  const int fn = lane & (TR - 1), fb0 = lane / TR;
  const int rr = 4 * (fn >> 3) + (fn & 3), hh = (fn >> 2) & 1;
  float y[SWIGLU ? 1 : R], u_[SWIGLU ? R : 1], g_[SWIGLU ? R : 1];
#pragma unroll
  for (int i = 0; i < R; i++) {
    const int b = FB * (wave * R + i) + fb0;
    const int slot = rr * 64 + ((b + 32 * hh) ^ (rr + 16 * hh));
    if (SWIGLU) {
      double gd = all[slot], ud = all[NW * 16 * 64 + slot];
#pragma unroll
      for (int w = 1; w < NW; w++) { gd += all[w * 16 * 64 + slot]; ud += all[(NW + w) * 16 * 64 + slot]; }
      g_[i] = (float)gd; u_[i] = (float)ud;
    } else {
      double t = all[slot];
#pragma unroll
      for (int w = 1; w < NW; w++) t += all[w * 16 * 64 + slot];
      y[i] = (float)t;
    }
  }
  if (SWIGLU) {
    // g and u were rounded to f32 like the matmul's own outputs; the 32 lanes of a half hold one Q8_1 block of the activation
    uint16_t* act = (uint16_t*)A.g[0].out;
#pragma unroll
    for (int i = 0; i < R; i++) {
      const int b = FB * (wave * R + i) + fb0;
      const uint16_t a16 = f32_to_bf16(__fmul_rn(__fmul_rn(g_[i], sigmoid_f64(g_[i])), u_[i]));
      const bool valid = b < B;
      if (valid && act) act[(int64_t)(b0 + b) * N + n0 + col] = a16;
      lane32_q8_1_store(bf16_to_f32(a16), A.out_q8 + ((int64_t)(b0 + b) * (N / 32) + (n0 >> 5)) * 36, col, valid);
    }
    return;
  }
  const bool n_ok = n0 + fn < N;
  const int64_t o0 = (int64_t)b0 * N + n0 + fn;
  if (EPI == GEPI_F32) {
#pragma unroll
    for (int i = 0; i < R; i++) {
      const int b = FB * (wave * R + i) + fb0;
      if (n_ok && b < B) ((float*)out)[o0 + (int64_t)b * N] = y[i];
    }
  } else if (EPI == GEPI_BF16) {
#pragma unroll
    for (int i = 0; i < R; i++) {
      const int b = FB * (wave * R + i) + fb0;
      if (n_ok && b < B) ((uint16_t*)out)[o0 + (int64_t)b * N] = f32_to_bf16(y[i]);
    }
  } else {
    uint16_t rv[R];
#pragma unroll
    for (int i = 0; i < R; i++) {
      const int b = FB * (wave * R + i) + fb0;
      rv[i] = (n_ok && b < B) ? res[o0 + (int64_t)b * N] : (uint16_t)0;
    }
#pragma unroll
    for (int i = 0; i < R; i++) {
      const int b = FB * (wave * R + i) + fb0;
      if (n_ok && b < B) ((uint16_t*)out)[o0 + (int64_t)b * N] = f32_to_bf16(bf16_to_f32(f32_to_bf16(y[i])) + bf16_to_f32(rv[i]));
    }
  }
}

#undef GM_FETCH

int g_tune_gemm_nw = 0;      // waves per tile (1, 2, 4, 8); 0 = chosen from the shape
int g_tune_gemm_r16 = -1;    // narrow tiles (single batch tile only): 0 off, 1 = 16 weight rows, 2 = 8, -1 = from the shape

template <typename ARGS>
static void launch_mfma_plain(int tr, int nw, dim3 grid, const ARGS& A) {
  if (tr == 16) {
    if (nw >= 8) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<8, false, 16, ARGS>), grid, dim3(512), 0, stream(), A);
    else hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<4, false, 16, ARGS>), grid, dim3(256), 0, stream(), A);
  } else if (tr == 8) {
    if (nw >= 8) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<8, false, 8, ARGS>), grid, dim3(512), 0, stream(), A);
    else hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<4, false, 8, ARGS>), grid, dim3(256), 0, stream(), A);
  } else if (nw == 8) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<8, false, 32, ARGS>), grid, dim3(512), 0, stream(), A);
  else if (nw == 4) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<4, false, 32, ARGS>), grid, dim3(256), 0, stream(), A);
  else if (nw == 2) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<2, false, 32, ARGS>), grid, dim3(128), 0, stream(), A);
  else hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<1, false, 32, ARGS>), grid, dim3(64), 0, stream(), A);
}

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
  // One batch tile and so few weight tiles that CUs would stay empty: tiles of 16 weight rows (twice as many
  // workgroups, half the fold per wave) when that still leaves half of them empty... of 8 when a quarter.  Measured on the
  // 64-tile shapes at batch 32.
  int tr = 32;
  if (batch <= 32) {
    if (g_tune_gemm_r16 >= 0) tr = g_tune_gemm_r16 == 0 ? 32 : (g_tune_gemm_r16 == 1 ? 16 : 8);
    else if (A.nb >= 4) tr = 4 * tiles <= num_cus() ? 8 : (2 * tiles <= num_cus() ? 16 : 32);
  }
  if (tr != 32) {
    tiles = 0;
    for (int i = 0; i < ngroups; i++) { A.tile_first[i] = tiles; tiles += (N[i] + tr - 1) / tr; }
  }
  for (int i = ngroups; i < 5; i++) A.tile_first[i] = tiles;
  // waves per tile (measured on the decode shapes at batch 32): long rows split eight ways, K = 2048 four ways,
  // and not at all when the tiles alone fill the chip many times over (lm_head, prompt batches)
  const int btiles = (batch + 31) / 32;
  const int64_t wgs = (int64_t)tiles * btiles;
  int nw = g_tune_gemm_nw;
  if (nw <= 0) {
    nw = A.nb >= 16 ? 8 : (A.nb >= 4 ? 4 : (A.nb >= 2 ? 2 : 1));
    if (wgs <= num_cus() && A.nb >= 8) nw = 8;                            // at most a tile per CU: one super-block per wave
    if (wgs > num_cus() && nw == 8) nw = 4;     // eight waves' LDS leaves room for one workgroup per CU: no second round for a few tiles
    if (wgs >= 8 * num_cus()) nw = 1;                                     // the tiles alone fill the chip many times over
  }
  nw = nw >= 8 ? 8 : (nw >= 4 ? 4 : (nw >= 2 ? 2 : 1));
  A.tiles = tiles; A.btiles = btiles;
  const dim3 grid(btiles > 1 ? (unsigned)(8 * ((wgs + 7) / 8)) : (unsigned)tiles);
  if (ngroups == 1) {
    const MfmaArgs1 P{A.g[0].W, A.g[0].out, A.g[0].res, A.xq, A.g[0].N, A.g[0].epi, A.nb, A.B, tiles, btiles};
    launch_mfma_plain(tr, nw, grid, P);
  } else {
    launch_mfma_plain(tr, nw, grid, A);
  }
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

namespace bk {

// gate and up projections with the SwiGLU and the Q8_1 quantization of its result in the last step of the matmul:
// act[b, n] = bf16(silu(g) * u) (src/fusion.ts:324-330 on the two matmuls' f32 outputs), written as bf16 (if `act` is
// given) and as the Q8_1 blocks the down projection reads.
int launch_gemm_swiglu_mfma(const void* xq, int K, int batch, const void* Wg, const void* Wu, int N, void* act, void* act_q8) {
  BK_REQUIRE(xq && Wg && Wu && act_q8, "gemm_swiglu_mfma: null pointer");
  BK_REQUIRE(K > 0 && K % 256 == 0, "gemm_swiglu_mfma: K=%d must be a positive multiple of 256", K);
  BK_REQUIRE(N > 0 && N % 32 == 0, "gemm_swiglu_mfma: N=%d must be a positive multiple of 32", N);
  BK_REQUIRE(batch >= 1 && batch <= 32 * 65535, "gemm_swiglu_mfma: bad batch=%d", batch);
  BK_REQUIRE(((uintptr_t)xq & 3) == 0 && ((uintptr_t)Wg & 15) == 0 && ((uintptr_t)Wu & 15) == 0 && ((uintptr_t)act_q8 & 3) == 0,
             "gemm_swiglu_mfma: misaligned pointer");
  MfmaArgs A{};
  A.xq = (const uint8_t*)xq; A.nb = K / 256; A.B = batch;
  A.g[0].W = (const uint8_t*)Wg; A.g[0].out = act; A.g[0].N = N;
  A.g[1].W = (const uint8_t*)Wu; A.g[1].N = N;
  A.out_q8 = (uint8_t*)act_q8;
  const int tiles = N / 32, btiles = (batch + 31) / 32;
  for (int i = 0; i < 5; i++) A.tile_first[i] = i ? tiles : 0;
  A.tiles = tiles; A.btiles = btiles;
  const int64_t wgs = (int64_t)tiles * btiles;
  // waves per tile as in the plain form (each workgroup holds two tiles, so at most four per tile)
  int nw = g_tune_gemm_nw;
  if (nw <= 0) {
    nw = A.nb >= 4 ? 4 : (A.nb >= 2 ? 2 : 1);
    if (2 * wgs >= 8 * num_cus()) nw = 1;
  }
  nw = nw >= 4 ? 4 : (nw >= 2 ? 2 : 1);
  const dim3 grid(btiles > 1 ? (unsigned)(8 * ((wgs + 7) / 8)) : (unsigned)tiles);
  const MfmaArgsSw P{A.g[0].W, A.g[1].W, act, (uint8_t*)act_q8, A.xq, N, A.nb, A.B, tiles, btiles};
  if (nw == 4) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<4, true, 32, MfmaArgsSw>), grid, dim3(512), 0, stream(), P);
  else if (nw == 2) hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<2, true, 32, MfmaArgsSw>), grid, dim3(256), 0, stream(), P);
  else hipLaunchKernelGGL((gemm_q4k_q8_1_mfma_kernel<1, true, 32, MfmaArgsSw>), grid, dim3(128), 0, stream(), P);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
