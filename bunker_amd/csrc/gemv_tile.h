// Device building blocks shared by the Q4_K x Q8_1 GEMV kernels: the (block, chunk) lane mapping,
// the per-slot fold, the shared row reductions and the staging of weight rows through LDS.
#pragma once
#include "ops.h"

namespace bk {

constexpr int GEMV_WAVES = 4;           // waves per workgroup

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
  return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// Lane c of an 8-lane group extracts scale and min of sub-block j = c from the
// 12 packed bytes (dwords s0, s1, s2).  cA/cW/cB are lane constants:
//   c < 4 : sc = (s0 >> 8c) & 63 ; m = (s1 >> 8c) & 63
//   c >= 4: sc = ((s2 >> 8(c-4)) & 15) | ((s0 >> (8(c-4)+6)) & 3) << 4 ; m likewise from s1
struct ScaleSel {
  uint32_t sh;     // 8 * (c & 3)
  uint32_t wlo;    // 6 or 4 : width of the low field
  uint32_t whi;    // 0 or 2 : width of the high field
  bool hi;         // c >= 4
};
__device__ __forceinline__ ScaleSel make_scale_sel(int c) {
  ScaleSel s;
  s.sh = 8u * (c & 3);
  s.hi = c >= 4;
  s.wlo = s.hi ? 4u : 6u;
  s.whi = s.hi ? 2u : 0u;
  return s;
}
__device__ __forceinline__ uint32_t bfe(uint32_t v, uint32_t off, uint32_t width) {
  return __builtin_amdgcn_ubfe(v, off, width);
}
__device__ __forceinline__ void lane_scale_min(const ScaleSel& s, uint32_t s0, uint32_t s1, uint32_t s2,
                                               uint32_t& sc, uint32_t& m) {
  const uint32_t t = s2 >> s.sh;
  const uint32_t a = s.hi ? t : (s0 >> s.sh);
  const uint32_t b = s.hi ? (t >> 4) : (s1 >> s.sh);
  sc = bfe(a, 0, s.wlo) | (bfe(s0, s.sh + 6, s.whi) << 4);
  m = bfe(b, 0, s.wlo) | (bfe(s1, s.sh + 6, s.whi) << 4);
}

// quad_perm:[0,0,2,2] and [1,1,3,3]: the even / odd lane of each lane pair
constexpr int DPP_PAIR_EVEN = 0xA0;
constexpr int DPP_PAIR_ODD = 0xF5;

// Activation slice of one slot, Q8_1 layout (int8 q[32] @0, fp16 d @32, fp16 s @34).
struct XQ {
  uint32_t lo[4], hi[4];   // 16 int8 of sub-block 2g and of sub-block 2g+1
  float d8c, s8c;          // d and s of sub-block c (the sub-block this lane folds)
};

__device__ __forceinline__ void load_xq(XQ& x, const uint8_t* __restrict__ xq, int blk, int c, bool active) {
  if (!active) {
#pragma unroll
    for (int i = 0; i < 4; i++) { x.lo[i] = 0; x.hi[i] = 0; }
    x.d8c = 0.0f; x.s8c = 0.0f;
    return;
  }
  const int g = c >> 1, half = c & 1;
  const uint32_t* p0 = (const uint32_t*)(xq + (int64_t)(blk * 8 + 2 * g) * 36 + 16 * half);
  const uint32_t* p1 = (const uint32_t*)(xq + (int64_t)(blk * 8 + 2 * g + 1) * 36 + 16 * half);
#pragma unroll
  for (int i = 0; i < 4; i++) { x.lo[i] = p0[i]; x.hi[i] = p1[i]; }
  const uint32_t ds = *(const uint32_t*)(xq + (int64_t)(blk * 8 + c) * 36 + 32);
  x.d8c = half_to_f32((uint16_t)(ds & 0xffffu));
  x.s8c = half_to_f32((uint16_t)(ds >> 16));
}

// One slot's contribution to a row (double).  I0/I1 are the exact int32 half-sub-block dots
// (low / high nibbles).  The two lanes of a pair (c even, c odd) hold the two 16-element halves of
// sub-blocks 2g and 2g+1: they add them up, and lane c then owns the whole sub-block c and folds
// it with its own scale, so no scale has to travel between lanes:
//   term = (d * d8_c) * (sc_c * I_c) - (dmin * s8_c) * m_c        every product exact in double
__device__ __forceinline__ double slot_dot(const uint4& hdr, const uint4& q, const XQ& x, const ScaleSel& sel,
                                          int& I0, int& I1, bool odd) {
  const float d = half_to_f32((uint16_t)(hdr.x & 0xffffu));
  const float dmin = half_to_f32((uint16_t)(hdr.x >> 16));
  uint32_t sc, m;
  lane_scale_min(sel, hdr.y, hdr.z, hdr.w, sc, m);
  int a = 0, b = 0;
  a = sdot4(q.x & 0x0f0f0f0fu, x.lo[0], a);
  b = sdot4((q.x >> 4) & 0x0f0f0f0fu, x.hi[0], b);
  a = sdot4(q.y & 0x0f0f0f0fu, x.lo[1], a);
  b = sdot4((q.y >> 4) & 0x0f0f0f0fu, x.hi[1], b);
  a = sdot4(q.z & 0x0f0f0f0fu, x.lo[2], a);
  b = sdot4((q.z >> 4) & 0x0f0f0f0fu, x.hi[2], b);
  a = sdot4(q.w & 0x0f0f0f0fu, x.lo[3], a);
  b = sdot4((q.w >> 4) & 0x0f0f0f0fu, x.hi[3], b);
  I0 = a; I1 = b;
  const int s0 = a + dpp_i32<DPP_QUAD_XOR1>(a);          // whole sub-block 2g
  const int s1 = b + dpp_i32<DPP_QUAD_XOR1>(b);          // whole sub-block 2g+1
  const int p = __mul24((int)sc, odd ? s1 : s0);         // 6 x 17 bits: exact
  const double t = (double)(dmin * x.s8c) * (double)m;   // 11 x 11 bits exact in f32, then exact in double
  return fma((double)(d * x.d8c), (double)p, -t);
}

// Sum of four per-lane doubles (four rows) over the 64 lanes with shared steps: after two
// exchange-and-halve steps a lane carries one row, row(lane) = 2*(lane & 1) + ((lane >> 1) & 1),
// and the remaining steps keep lane mod 4.  Every lane ends with the total of its row.
__device__ __forceinline__ double wave_sum4_f64(double a0, double a1, double a2, double a3, int lane) {
  const bool o1 = lane & 1, o2 = lane & 2;
  // step 1 (partner lane ^ 1): even lanes keep rows 0,1 and give away rows 2,3
  const double k0 = o1 ? a2 : a0, k1 = o1 ? a3 : a1, g0 = o1 ? a0 : a2, g1 = o1 ? a1 : a3;
  const double b0 = k0 + dpp_f64<DPP_QUAD_XOR1>(g0), b1 = k1 + dpp_f64<DPP_QUAD_XOR1>(g1);
  // step 2 (partner lane ^ 2): lanes with bit 1 clear keep the first of their two rows
  const double k = o2 ? b1 : b0, g = o2 ? b0 : b1;
  double v = k + dpp_f64<DPP_QUAD_XOR2>(g);
  v += dpp_f64<0x124>(v);      // row_ror:4  (lane i gets lane (i+4) mod 16 of its row of 16)
  v += dpp_f64<0x128>(v);      // row_ror:8
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

// Two rows: one exchange-and-halve step, then lane parity is kept; lane L ends with row L & 1.
__device__ __forceinline__ double wave_sum2_f64(double a0, double a1, int lane) {
  const bool o1 = lane & 1;
  const double k = o1 ? a1 : a0, g = o1 ? a0 : a1;
  double v = k + dpp_f64<DPP_QUAD_XOR1>(g);
  v += dpp_f64<DPP_QUAD_XOR2>(v);
  v += dpp_f64<0x124>(v);      // row_ror:4
  v += dpp_f64<0x128>(v);      // row_ror:8
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

// Weights are read once: nontemporal loads keep them from displacing the activation in the caches.
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_nt;
__device__ __forceinline__ uint4 load_w16(const uint8_t* p) {
  const u32x4_nt t = __builtin_nontemporal_load((const u32x4_nt*)p);
  return make_uint4(t.x, t.y, t.z, t.w);
}

enum : int { EPI_F32 = 0, EPI_BF16 = 1, EPI_BF16_ADD = 2 };

template <int EPI>
__device__ __forceinline__ void store_out(void* __restrict__ y, const uint16_t* __restrict__ res, int64_t i, float v) {
  if (EPI == EPI_F32) {
    ((float*)y)[i] = v;
  } else if (EPI == EPI_BF16) {
    ((uint16_t*)y)[i] = f32_to_bf16(v);
  } else {
    // gemm(f32) -> cast(bf16) -> add(bf16, bf16): two roundings, as the model graph orders them
    const float c = bf16_to_f32(f32_to_bf16(v));
    ((uint16_t*)y)[i] = f32_to_bf16(c + bf16_to_f32(res[i]));
  }
}

template <int NR, int RPI>
struct RowTile {
  uint4 hdr[RPI][NR], q[RPI][NR];
};

template <int NR, int RPI>
__device__ __forceinline__ void load_rows(RowTile<NR, RPI>& t, const uint8_t* __restrict__ W, int64_t row_bytes, int row0, int N,
                                          const int (&boff)[NR], int c) {
#pragma unroll
  for (int i = 0; i < RPI; i++) {
    const int row = min(row0 + i, N - 1);     // rows past the end re-read the last row; their results are dropped
    const uint8_t* rp = W + (int64_t)row * row_bytes;
#pragma unroll
    for (int r = 0; r < NR; r++) {
      t.hdr[i][r] = load_w16(rp + boff[r]);
      t.q[i][r] = load_w16(rp + boff[r] + 16 + 16 * c);
    }
  }
}

template <int NR, int EPI, int RPI>
__device__ __forceinline__ void fold_rows(const RowTile<NR, RPI>& t, const XQ (&x)[NR], const ScaleSel& sel, bool odd, int lane,
                                          void* __restrict__ y, const uint16_t* __restrict__ res, int64_t ybase, int row0, int N) {
  double acc[RPI];
#pragma unroll
  for (int i = 0; i < RPI; i++) {
    acc[i] = 0.0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
      int I0, I1;
      acc[i] += slot_dot(t.hdr[i][r], t.q[i][r], x[r], sel, I0, I1, odd);
    }
  }
  if (RPI == 4) {
    const double tot = wave_sum4_f64(acc[0], acc[1], acc[2], acc[3], lane);
    const int row = row0 + 2 * (lane & 1) + ((lane >> 1) & 1);
    if (lane < 4 && row < N) store_out<EPI>(y, res, ybase + row, (float)tot);
  } else {
#pragma unroll
    for (int i = 0; i < RPI; i++) {
      const float tot = (float)wave_sum_f64(acc[i]);
      if (lane == 0 && row0 + i < N) store_out<EPI>(y, res, ybase + row0 + i, tot);
    }
  }
}

// Folds a tile and returns, in every lane, the total of the tile row that lane ends up with:
// row 2*(lane & 1) + ((lane >> 1) & 1) for RPI = 4, row lane & 1 for RPI = 2.
template <int NR, int RPI>
__device__ __forceinline__ double fold_rows_total(const RowTile<NR, RPI>& t, const XQ (&x)[NR], const ScaleSel& sel, bool odd,
                                                  int lane) {
  static_assert(RPI == 2 || RPI == 4, "two or four rows per step");
  double acc[RPI];
#pragma unroll
  for (int i = 0; i < RPI; i++) {
    acc[i] = 0.0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
      int I0, I1;
      acc[i] += slot_dot(t.hdr[i][r], t.q[i][r], x[r], sel, I0, I1, odd);
    }
  }
  if (RPI == 4) return wave_sum4_f64(acc[0], acc[1], acc[2], acc[RPI - 1], lane);
  return wave_sum2_f64(acc[0], acc[1], lane);
}

template <int NR, int RPI>
struct StageRegs {
  static constexpr int PIECES = RPI * NR * 72;
  static constexpr int LOADS = (PIECES + 63) / 64;
  uint4 v[LOADS];
};

template <int NR, int RPI>
__device__ __forceinline__ void stage_load(StageRegs<NR, RPI>& g, const uint8_t* __restrict__ W, int64_t tile_off,
                                           int64_t last_piece_off, int lane) {
#pragma unroll
  for (int u = 0; u < StageRegs<NR, RPI>::LOADS; u++) {
    // every lane loads in every round (lanes past the tile re-request its last piece), so that the number of
    // loads in flight is known at compile time
    const int piece = min(lane + 64 * u, StageRegs<NR, RPI>::PIECES - 1);
    const int64_t off = tile_off + (int64_t)piece * 16;
    g.v[u] = load_w16(W + (off < last_piece_off ? off : last_piece_off));   // past the matrix: re-read its last piece
  }
}

template <int NR, int RPI>
__device__ __forceinline__ void stage_park(const StageRegs<NR, RPI>& g, uint4* __restrict__ tile, int lane) {
#pragma unroll
  for (int u = 0; u < StageRegs<NR, RPI>::LOADS; u++) {
    const int piece = lane + 64 * u;
    if (piece < StageRegs<NR, RPI>::PIECES) tile[piece] = g.v[u];
  }
}

}  // namespace bk
