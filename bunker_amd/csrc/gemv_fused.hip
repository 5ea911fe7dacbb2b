// Q4_K x Q8_1 GEMV with the surrounding glue folded in: one launch serves
//   [RMSNorm | bf16 -> Q8_1 | Q8_1 as given]  ->  up to four matrices over the same activation
//   ->  per matrix: f32 | bf16 | bf16(bf16(y) + residual)      or, for a (gate, up) pair, SwiGLU.
//
// Prologue.  Every workgroup prepares the activation row itself: 256 threads x 8 elements per
// pass, the sum of squares in double through the same block reduction as the stand-alone
// RMSNorm kernel, the Q8_1 blocks by groups of four lanes.  The quantized row lives in LDS in
// the Q8_1 byte layout; each lane then takes its slice into registers as the plain GEMV does.
// The activation loads go out first and the first weight rows right behind them, so the prologue
// runs while the weight rows are on their way.
//
// Rows.  As in the LDS-staged GEMV: a wave step fetches RPI contiguous rows with coalesced
// 16-byte loads, parks them in the wave's LDS tile and reads them back in the (block, chunk)
// mapping.  The matrices of a launch are laid end to end in "step" space; a step belongs to
// exactly one matrix.  For SwiGLU a step holds RPI/2 rows of the gate matrix and the same rows
// of the up matrix, so that the lanes that end up with g and u of one output row are neighbours.
//
// Arithmetic is that of gemv.hip and glue.hip, operation for operation, so a fused launch gives
// the bits of the node-by-node sequence rmsnorm -> gemm [-> cast -> add | -> swiglu].
#include "gemv_tile.h"

namespace bk {

// PRO_GNORM: the activation is the raw output of the column-slab GDN step (gdn.hip gdn_slab_kernel) and goes through
// that op's gated RMS norm first (src/emitters.ts:110-118): per head of 128, o * rsqrt(mean(o^2) + 1e-6) * norm_w * (z *
// sigmoid(z)) -> bf16, with the sum of squares taken from the four slab sums the step left (added as (s0 + s1) + (s2 +
// s3): the association of the one-workgroup form's block reduction, so the bits agree).
enum : int { PRO_Q8 = 0, PRO_BF16 = 1, PRO_RMSNORM = 2, PRO_GNORM = 3 };
// EPI_CONV (matrix 0 only): the row's bf16 output is channel `row` of conv1d_decode's input and goes through the 4-tap
// causal convolution + SiLU at once (src/emitters.ts:48-72): out = bf16(r * sigmoid(r)), r = (w0 s0 + w1 s1) + (w2 s2 +
// w3 x), and the channel's state rows become (s1, s2, x).  The lane that read a channel's rows rewrites them, so the
// state may be updated in place.
enum : int { EPI_CONV = 3 };

struct FusedGroup {
  const uint8_t* W;
  void* out;
  const uint16_t* res;
  int N, epi;
};
struct FusedArgs {
  FusedGroup g[4];
  int step_first[5];     // first step of each matrix; step_first[i >= ngroups] = total steps
  int ngroups;
  int nwg;               // workgroups along x (read from here: gridDim would pull 256 bytes of implicit arguments into the block)
  const void* x;         // PRO_Q8: Q8_1 [batch, K/32 blocks]; PRO_GNORM: the GDN step's raw block per sequence; else bf16 [batch, K]
  const uint16_t* norm_w; // PRO_RMSNORM: bf16 [K]; PRO_GNORM: f32 [128]
};
// What only the conv-epilogue and gated-norm forms read.  Kept out of FusedArgs: with these 32 bytes in every kernel's
// argument block the other forms measured 0.2-0.4 us slower per launch (19 us over a decode step).
struct FusedArgsX : FusedArgs {
  // EPI_CONV: conv state bf16 [batch, 3, C] (in, new; may alias), taps bf16 [C, 4]; C = rows of matrix 0
  const uint16_t* conv_st;
  uint16_t* conv_st_new;
  const uint16_t* conv_w;
  int64_t x_bstride;     // PRO_GNORM: bytes between two sequences' raw blocks
};

// Compact argument blocks.  A kernel's first instructions wait for its argument block, and the block arrives cache line
// by cache line: every 64 bytes less measured 0.2-0.3 us per launch (one-matrix launches 168 -> 64 bytes: 11 us over the
// decode step).  The launcher picks the smallest form that holds the launch; the kernel rebuilds the full form in
// registers (step_first from the row counts) and runs unchanged.
//   FusedArgs1: one matrix (out_proj, o_proj, down, lm_head: half of the step's launches), 64 bytes
//   FusedArgs2: the SwiGLU pair, 52 bytes
//   FusedArgsC: up to four matrices without residuals, 104 bytes; with the conv epilogue's operands (FusedArgsCX) 128
//               (unused slots repeat the last matrix)
struct FusedArgs1 {
  FusedGroup g0;
  const void* x;
  const uint16_t* norm_w;
  int64_t x_bstride;
  int steps, nwg;
};
struct FusedArgs2 {
  const uint8_t *Wg, *Wu;
  void* out;
  const void* x;
  const uint16_t* norm_w;
  int N, steps, nwg;
};
struct FusedArgsC {
  const uint8_t* W[4];
  void* out[4];
  const void* x;
  const uint16_t* norm_w;
  int N[4];
  int epi4;              // epilogue of matrix i in bits 8 i .. 8 i + 7
  int ngroups;           // | workgroups along x << 8
};
struct FusedArgsCX : FusedArgsC {
  const uint16_t* conv_st;
  uint16_t* conv_st_new;
  const uint16_t* conv_w;
};
__device__ __forceinline__ const FusedArgs& fused_args_full(const FusedArgs& A, int) { return A; }
__device__ __forceinline__ const FusedArgsX& fused_args_full(const FusedArgsX& A, int) { return A; }
__device__ __forceinline__ FusedArgsX fused_args_full(const FusedArgs1& P, int) {
  FusedArgsX A;
  A.g[0] = P.g0; A.g[1] = P.g0; A.g[2] = P.g0; A.g[3] = P.g0;
  const int steps = P.steps;
  A.step_first[0] = 0; A.step_first[1] = steps; A.step_first[2] = steps; A.step_first[3] = steps; A.step_first[4] = steps;
  A.ngroups = 1; A.nwg = P.nwg; A.x = P.x; A.norm_w = P.norm_w;
  A.conv_st = nullptr; A.conv_st_new = nullptr; A.conv_w = nullptr; A.x_bstride = P.x_bstride;
  return A;
}
__device__ __forceinline__ FusedArgsX fused_args_full(const FusedArgs2& P, int) {
  FusedArgsX A;
  A.g[0].W = P.Wg; A.g[0].out = P.out; A.g[0].res = nullptr; A.g[0].N = P.N; A.g[0].epi = EPI_BF16;
  A.g[1].W = P.Wu; A.g[1].out = P.out; A.g[1].res = nullptr; A.g[1].N = P.N; A.g[1].epi = EPI_BF16;
  A.g[2] = A.g[1]; A.g[3] = A.g[1];
  A.step_first[0] = 0; A.step_first[1] = P.steps; A.step_first[2] = P.steps; A.step_first[3] = P.steps; A.step_first[4] = P.steps;
  A.ngroups = 2; A.nwg = P.nwg; A.x = P.x; A.norm_w = P.norm_w;
  A.conv_st = nullptr; A.conv_st_new = nullptr; A.conv_w = nullptr; A.x_bstride = 0;
  return A;
}
// The several-matrix forms are read where they lie (their arrays are indexed by the step's matrix: rebuilt in registers
// they would end up in private memory); step_first comes from the row counts.
__device__ __forceinline__ const FusedArgsC& fused_args_full(const FusedArgsC& A, int) { return A; }
__device__ __forceinline__ const FusedArgsCX& fused_args_full(const FusedArgsCX& A, int) { return A; }

// The operands of one channel of the convolution, requested ahead of the step's arithmetic
struct ConvRegs {
  uint16_t s0, s1, s2;
  uint2 w;
};
template <typename AX>
__device__ __forceinline__ void conv_regs_load(ConvRegs& c, const AX& A, int bidx, int C, int ch) {
  ch = min(ch, C - 1);
  const uint16_t* sb = A.conv_st + (int64_t)bidx * 3 * C;
  c.s0 = sb[ch]; c.s1 = sb[C + ch]; c.s2 = sb[2 * C + ch];
  c.w = *(const uint2*)(A.conv_w + 4 * (int64_t)ch);
}
template <typename AX>
__device__ __forceinline__ uint16_t conv_regs_apply(const ConvRegs& c, const AX& A, int bidx, int C, int ch, uint16_t x) {
  const float w0 = __uint_as_float(c.w.x << 16), w1 = __uint_as_float(c.w.x & 0xffff0000u);
  const float w2 = __uint_as_float(c.w.y << 16), w3 = __uint_as_float(c.w.y & 0xffff0000u);
  // products of two bf16 values are exact in f32
  const float r = __fadd_rn(__fadd_rn(w0 * bf16_to_f32(c.s0), w1 * bf16_to_f32(c.s1)),
                            __fadd_rn(w2 * bf16_to_f32(c.s2), w3 * bf16_to_f32(x)));
  uint16_t* nb = A.conv_st_new + (int64_t)bidx * 3 * C;
  nb[ch] = c.s1; nb[C + ch] = c.s2; nb[2 * C + ch] = x;
  return f32_to_bf16(__fmul_rn(r, sigmoid_f64(r)));
}

// PRO_GNORM: what a thread holds of the raw block: 8 outputs, their gates, the norm weights, the head's four slab sums
struct GnormRegs {
  float4 o[2], zs[2], nw[2];
  double2 ss[2];
};
__device__ __forceinline__ void gnorm_load(GnormRegs& r, const uint8_t* __restrict__ raw, const float* __restrict__ norm_w, int K) {
  const int i = threadIdx.x * 8;                       // K = 2048: one pass of 256 threads x 8 elements
  const float* o = (const float*)raw;
  const float* zs = o + K;
  const double* ss = (const double*)(zs + K);
  r.o[0] = *(const float4*)(o + i); r.o[1] = *(const float4*)(o + i + 4);
  r.zs[0] = *(const float4*)(zs + i); r.zs[1] = *(const float4*)(zs + i + 4);
  r.nw[0] = *(const float4*)(norm_w + (i & 127)); r.nw[1] = *(const float4*)(norm_w + (i & 127) + 4);
  r.ss[0] = *(const double2*)(ss + (i >> 7) * 4); r.ss[1] = *(const double2*)(ss + (i >> 7) * 4 + 2);
}
__device__ __forceinline__ void stage_gnorm(const GnormRegs& g, uint8_t* lds_xq) {
  const double tot = (g.ss[0].x + g.ss[0].y) + (g.ss[1].x + g.ss[1].y);
  const float orstd = rsqrt_f64(tot / 128.0 + 1e-6);
  const float o[8] = {g.o[0].x, g.o[0].y, g.o[0].z, g.o[0].w, g.o[1].x, g.o[1].y, g.o[1].z, g.o[1].w};
  const float z[8] = {g.zs[0].x, g.zs[0].y, g.zs[0].z, g.zs[0].w, g.zs[1].x, g.zs[1].y, g.zs[1].z, g.zs[1].w};
  const float w[8] = {g.nw[0].x, g.nw[0].y, g.nw[0].z, g.nw[0].w, g.nw[1].x, g.nw[1].y, g.nw[1].z, g.nw[1].w};
  float f[8];
#pragma unroll
  for (int j = 0; j < 8; j++) f[j] = bf16_to_f32(f32_to_bf16(__fmul_rn(__fmul_rn(__fmul_rn(o[j], orstd), w[j]), z[j])));
  uint32_t pk[2];
  const uint32_t ds = quad_q8_1(f, pk);
  const int i = threadIdx.x * 8;
  uint8_t* ob = lds_xq + (i / 32) * 36;
  uint32_t* oq = (uint32_t*)(ob + (i & 31));
  oq[0] = pk[0]; oq[1] = pk[1];
  if ((i & 31) == 0) *(uint32_t*)(ob + 32) = ds;
  __syncthreads();
}

// What a step needs to know about its matrix (all wave-uniform).
struct StepSel {
  const uint8_t* W;
  void* out;
  const uint16_t* res;
  int N, epi, row0;
};

struct StepFirst { int f1, f2, f3, total; };
__device__ __forceinline__ StepFirst step_first_of(const FusedArgs& A, int) {
  return StepFirst{A.step_first[1], A.step_first[2], A.step_first[3], A.step_first[4]};
}
__device__ __forceinline__ StepFirst step_first_of(const FusedArgsC& P, int rps) {
  const int s0 = (P.N[0] + rps - 1) / rps;
  const int ng = P.ngroups & 0xff;
  const int s1 = s0 + (ng > 1 ? (P.N[1] + rps - 1) / rps : 0);
  const int s2 = s1 + (ng > 2 ? (P.N[2] + rps - 1) / rps : 0);
  const int s3 = s2 + (ng > 3 ? (P.N[3] + rps - 1) / rps : 0);
  return StepFirst{s0, s1, s2, s3};
}
__device__ __forceinline__ int workgroups_x(const FusedArgs& A) { return A.nwg; }
__device__ __forceinline__ int workgroups_x(const FusedArgsC& A) { return (int)((unsigned)A.ngroups >> 8); }
__device__ __forceinline__ int rows_of_first(const FusedArgs& A) { return A.g[0].N; }
__device__ __forceinline__ int rows_of_first(const FusedArgsC& A) { return A.N[0]; }
__device__ __forceinline__ const uint8_t* second_matrix(const FusedArgs& A) { return A.g[1].W; }
__device__ __forceinline__ const uint8_t* second_matrix(const FusedArgsC& A) { return A.W[1]; }

template <int ROWS_PER_STEP>
__device__ __forceinline__ StepSel select_step(const FusedArgs& A, const StepFirst& F, int s) {
  const bool s1 = s >= F.f1, s2 = s >= F.f2, s3 = s >= F.f3;
  StepSel r;
  r.W = s3 ? A.g[3].W : s2 ? A.g[2].W : s1 ? A.g[1].W : A.g[0].W;
  r.out = s3 ? A.g[3].out : s2 ? A.g[2].out : s1 ? A.g[1].out : A.g[0].out;
  r.res = s3 ? A.g[3].res : s2 ? A.g[2].res : s1 ? A.g[1].res : A.g[0].res;
  r.N = s3 ? A.g[3].N : s2 ? A.g[2].N : s1 ? A.g[1].N : A.g[0].N;
  r.epi = s3 ? A.g[3].epi : s2 ? A.g[2].epi : s1 ? A.g[1].epi : A.g[0].epi;
  r.row0 = (s - (s3 ? F.f3 : s2 ? F.f2 : s1 ? F.f1 : 0)) * ROWS_PER_STEP;
  return r;
}
template <int ROWS_PER_STEP>
__device__ __forceinline__ StepSel select_step(const FusedArgsC& A, const StepFirst& F, int s) {
  const bool s1 = s >= F.f1, s2 = s >= F.f2, s3 = s >= F.f3;
  StepSel r;
  r.W = s3 ? A.W[3] : s2 ? A.W[2] : s1 ? A.W[1] : A.W[0];
  r.out = s3 ? A.out[3] : s2 ? A.out[2] : s1 ? A.out[1] : A.out[0];
  r.res = nullptr;
  r.N = s3 ? A.N[3] : s2 ? A.N[2] : s1 ? A.N[1] : A.N[0];
  r.epi = (A.epi4 >> (s3 ? 24 : s2 ? 16 : s1 ? 8 : 0)) & 0xff;
  r.row0 = (s - (s3 ? F.f3 : s2 ? F.f2 : s1 ? F.f1 : 0)) * ROWS_PER_STEP;
  return r;
}

// ---- prologue: activation row -> Q8_1 in LDS (36-byte blocks).  K = 256 * KB elements in NR = ceil(KB / 8) passes of
// 256 threads x 8 elements; in the last pass of a K that is not a multiple of 2048 the threads past the row take no part
// (their loads are clamped, their values zero).
// Everything the prologue reads from memory (the row and, for RMSNorm, the norm weight) is requested up front.
// Loads return to a wave in the order they were issued, so these go out BEFORE the weight rows: the prologue then
// waits for a few small, cache-resident loads only and runs while the weight rows are still on their way.
template <int KB>
struct ActRegs {
  static constexpr int NR = (KB + 7) / 8, K = KB * 256;
  uint4 xv[NR], wv[NR];
};
template <int PRO, int KB>
__device__ __forceinline__ void act_load(ActRegs<KB>& r, const uint16_t* __restrict__ xr, const uint16_t* __restrict__ w) {
  constexpr int K = ActRegs<KB>::K;
#pragma unroll
  for (int p = 0; p < ActRegs<KB>::NR; p++) {
    const int i = min((int)threadIdx.x * 8 + p * 2048, K - 8);
    r.xv[p] = *(const uint4*)(xr + i);
    if (PRO == PRO_RMSNORM) r.wv[p] = *(const uint4*)(w + i);
  }
}
template <int PRO, int KB>
__device__ __forceinline__ void stage_activation(const ActRegs<KB>& regs, uint8_t* lds_xq, double* lds_red) {
  constexpr int NR = ActRegs<KB>::NR, K = ActRegs<KB>::K;
  const uint4 (&xv)[NR] = regs.xv;
  const uint4 (&wv)[NR] = regs.wv;
  float rstd = 0.0f;
  if (PRO == PRO_RMSNORM) {
    double ss = 0.0;
#pragma unroll
    for (int p = 0; p < NR; p++) {
      const bool valid = (p + 1) * 2048 <= K || (int)threadIdx.x * 8 + p * 2048 < K;
      const uint32_t u[4] = {xv[p].x, xv[p].y, xv[p].z, xv[p].w};
      double sp = 0.0;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float a = __uint_as_float(u[j] << 16), b = __uint_as_float(u[j] & 0xffff0000u);
        sp += (double)(a * a) + (double)(b * b);
      }
      ss += valid ? sp : 0.0;
    }
    ss = block_sum_f64<4>(ss, lds_red);
    rstd = rsqrt_f64(ss / (double)K + 1e-6);
  }
#pragma unroll
  for (int p = 0; p < NR; p++) {
    const int i = threadIdx.x * 8 + p * 2048;
    const bool valid = (p + 1) * 2048 <= K || i < K;        // whole quads (K is a multiple of 32)
    const uint32_t u[4] = {xv[p].x, xv[p].y, xv[p].z, xv[p].w};
    float f[8];
    if (PRO == PRO_RMSNORM) {
      const uint32_t uw[4] = {wv[p].x, wv[p].y, wv[p].z, wv[p].w};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float a = __uint_as_float(u[j] << 16), b = __uint_as_float(u[j] & 0xffff0000u);
        const float wa = __uint_as_float(uw[j] << 16), wb = __uint_as_float(uw[j] & 0xffff0000u);
        f[2 * j] = bf16_to_f32(f32_to_bf16(__fmul_rn(__fmul_rn(a, rstd), __fadd_rn(1.0f, wa))));
        f[2 * j + 1] = bf16_to_f32(f32_to_bf16(__fmul_rn(__fmul_rn(b, rstd), __fadd_rn(1.0f, wb))));
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        f[2 * j] = __uint_as_float(u[j] << 16);
        f[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
      }
    }
    uint32_t pk[2];
    const uint32_t ds = quad_q8_1(f, pk);
    if (valid) {
      uint8_t* ob = lds_xq + (i / 32) * 36;
      uint32_t* oq = (uint32_t*)(ob + (i & 31));
      oq[0] = pk[0]; oq[1] = pk[1];
      if ((i & 31) == 0) *(uint32_t*)(ob + 32) = ds;
    }
  }
  __syncthreads();
}

// Rows of KB super-blocks: 9 * KB pieces of 16 bytes each, RPI rows per wave step.
template <int KB, int RPI>
struct FusedStage {
  static constexpr int PIECES = RPI * KB * 9;
  static constexpr int LOADS = (PIECES + 63) / 64;
  uint4 v[LOADS];
};

// ---- weight rows of one step: coalesced 16-byte pieces; with SWIGLU the second half of the tile
// comes from the up matrix (same rows)
template <int KB, int RPI, bool SWIGLU>
__device__ __forceinline__ void fused_stage_load(FusedStage<KB, RPI>& g, const uint8_t* __restrict__ W0,
                                                 const uint8_t* __restrict__ W1, int row0, int N, int lane) {
  constexpr int PIECES = FusedStage<KB, RPI>::PIECES;
  constexpr int64_t row_bytes = (int64_t)KB * 144;
  const int64_t last = (int64_t)N * row_bytes - 16;
  const int64_t base = (int64_t)row0 * row_bytes;
#pragma unroll
  for (int u = 0; u < FusedStage<KB, RPI>::LOADS; u++) {
    // every lane loads in every round (lanes past the tile re-request its last piece): the number of loads in
    // flight is then known at compile time and waits can be counted instead of draining the queue
    const int piece = min(lane + 64 * u, PIECES - 1);
    const bool second = SWIGLU && piece >= PIECES / 2;
    const int64_t off = base + (int64_t)(second ? piece - PIECES / 2 : piece) * 16;
    const uint8_t* W = second ? W1 : W0;
    g.v[u] = load_w16(W + (off < last ? off : last));       // past the matrix: re-read its last piece
  }
}
template <int KB, int RPI>
__device__ __forceinline__ void fused_stage_park(const FusedStage<KB, RPI>& g, uint4* __restrict__ tile, int lane) {
#pragma unroll
  for (int u = 0; u < FusedStage<KB, RPI>::LOADS; u++) {
    const int piece = lane + 64 * u;
    if (piece < FusedStage<KB, RPI>::PIECES) tile[piece] = g.v[u];
  }
}

// KB = super-blocks per row (K = 256 * KB).  Lane (b, c) folds super-block 8r + b in pass r; when KB is not a multiple of 8
// the lanes past the row in the last pass read a clamped block and an all-zero activation slice, which adds exact zeros.
template <int KB, int RPI, int PRO, bool SWIGLU, bool CONV = false, typename ARGS = FusedArgs>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_fused_kernel(ARGS A_in) {
  const auto& A = fused_args_full(A_in, SWIGLU ? RPI / 2 : RPI);
  static_assert(!CONV || (!SWIGLU && RPI == 4 && PRO == PRO_RMSNORM), "the conv epilogue exists for the form the decode step asks for");
  constexpr int NR = (KB + 7) / 8;
  constexpr int RP = KB * 9;                 // 16-byte pieces per row
  constexpr int PIECES = RPI * RP;
  constexpr int K = KB * 256;
  constexpr int ROWS_PER_STEP = SWIGLU ? RPI / 2 : RPI;
  __shared__ uint4 tiles[GEMV_WAVES][PIECES];
  static_assert(PRO != PRO_GNORM || KB == 8, "the gated-norm prologue is written for rows of 2048 (16 heads of 128)");
  __shared__ __align__(16) uint8_t lds_xq[PRO == PRO_Q8 ? 16 : (K / 32) * 36];
  __shared__ double lds_red[4];

  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = workgroups_x(A) * GEMV_WAVES;
  const int bidx = blockIdx.y;
  const int c = lane & 7, b = lane >> 3;
  const ScaleSel sel = make_scale_sel(c);
  const bool odd = c & 1;
  const StepFirst F = step_first_of(A, ROWS_PER_STEP);
  const int total = F.total;
  uint4* tile = tiles[wv];

  [[maybe_unused]] ActRegs<KB> act;
  [[maybe_unused]] GnormRegs gn;
  if constexpr (PRO == PRO_GNORM) gnorm_load(gn, (const uint8_t*)A.x + (int64_t)bidx * A.x_bstride, (const float*)A.norm_w, K);
  else if constexpr (PRO != PRO_Q8) act_load<PRO, KB>(act, (const uint16_t*)A.x + (int64_t)bidx * K, A.norm_w);

  int s = blockIdx.x * GEMV_WAVES + wv;
  StepSel cur = select_step<ROWS_PER_STEP>(A, F, s < total ? s : 0);
  FusedStage<KB, RPI> g;
  // unconditional (a wave without a step of its own requests step 0): with a branch around these loads the
  // prologue's first wait could not be counted and would drain the weight rows as well
  // EPI_CONV: the channel's state rows and taps, requested ahead of the weight rows (they come from L2 and are back
  // long before the step's dots are folded); lanes 0..RPI-1 hold the step's rows
  const int rl_conv = 2 * (lane & 1) + ((lane >> 1) & 1);
  [[maybe_unused]] ConvRegs cr, crn;       // touched only by the CONV form (unused, they would end up as LDS-backed arrays)
  if constexpr (CONV) conv_regs_load(cr, A, bidx, rows_of_first(A), cur.row0 + rl_conv);      // unconditional: rows of the other matrices read a clamped channel
  fused_stage_load<KB, RPI, SWIGLU>(g, cur.W, second_matrix(A), cur.row0, cur.N, lane);

  XQ x[NR];
  if (PRO == PRO_Q8) {
    const uint8_t* xq = (const uint8_t*)A.x + (int64_t)bidx * (K / 32) * 36;
#pragma unroll
    for (int r = 0; r < NR; r++) load_xq(x[r], xq, r * 8 + b, c, (r + 1) * 8 <= KB || r * 8 + b < KB);
  } else {
    if constexpr (PRO == PRO_GNORM) stage_gnorm(gn, lds_xq);
    else stage_activation<PRO, KB>(act, lds_xq, lds_red);
#pragma unroll
    for (int r = 0; r < NR; r++) load_xq(x[r], lds_xq, r * 8 + b, c, (r + 1) * 8 <= KB || r * 8 + b < KB);
  }

  while (s < total) {
    fused_stage_park<KB, RPI>(g, tile, lane);
    const int sn = s + nwaves;
    StepSel nxt = cur;
    if constexpr (CONV) crn = cr;
    if (sn < total) {
      nxt = select_step<ROWS_PER_STEP>(A, F, sn);
      if constexpr (CONV) conv_regs_load(crn, A, bidx, rows_of_first(A), nxt.row0 + rl_conv);
      fused_stage_load<KB, RPI, SWIGLU>(g, nxt.W, second_matrix(A), nxt.row0, nxt.N, lane);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    RowTile<NR, RPI> t;
#pragma unroll
    for (int i = 0; i < RPI; i++) {
#pragma unroll
      for (int r = 0; r < NR; r++) {
        const int blk = i * RP + min(r * 8 + b, KB - 1) * 9;
        t.hdr[i][r] = tile[blk];
        t.q[i][r] = tile[blk + 1 + c];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();       // every lane has read its pieces before the tile is overwritten

    const double tot = fold_rows_total<NR, RPI>(t, x, sel, odd, lane);
    const int rl = RPI == 4 ? 2 * (lane & 1) + ((lane >> 1) & 1) : (lane & 1);     // tile row this lane holds
    const float v = (float)tot;
    if (SWIGLU) {
      // tile rows: gate row0, gate row0+1, up row0, up row0+1 -> lanes 0..3 hold g0, u0, g1, u1
      const float other = dpp_f32<DPP_QUAD_XOR1>(v);
      const int row = cur.row0 + (lane >> 1);
      if (lane < 4 && !(lane & 1) && row < cur.N) {
        // src/fusion.ts:324-330: bf16((g * sigmoid(g)) * u)
        ((uint16_t*)cur.out)[(int64_t)bidx * cur.N + row] = f32_to_bf16(__fmul_rn(__fmul_rn(v, sigmoid_f64(v)), other));
      }
    } else {
      const int row = cur.row0 + rl;
      if (lane < RPI && row < cur.N) {
        const int64_t o = (int64_t)bidx * cur.N + row;
        if (cur.epi == EPI_F32) store_out<EPI_F32>(cur.out, cur.res, o, v);
        else if (cur.epi == EPI_BF16) store_out<EPI_BF16>(cur.out, cur.res, o, v);
        else if (CONV && cur.epi == EPI_CONV) {
          if constexpr (CONV) ((uint16_t*)cur.out)[o] = conv_regs_apply(cr, A, bidx, cur.N, row, f32_to_bf16(v));
        } else store_out<EPI_BF16_ADD>(cur.out, cur.res, o, v);
      }
    }
    s = sn;
    cur = nxt;
    if constexpr (CONV) cr = crn;
  }
}

// Row lengths with a compiled kernel: 1024, 2048, 3584, 4096, 6144 (4, 8, 14, 16, 24 super-blocks); SwiGLU pairs for 1024 and 2048.
bool gemv_fused_fast_path(int K, int batch, bool swiglu) {
  const bool k_ok = swiglu ? (K == 1024 || K == 2048) : (K == 1024 || K == 2048 || K == 3584 || K == 4096 || K == 6144);
  return k_ok && batch >= 1 && batch < 8;
}

template <int KB, int RPI, bool SWIGLU>
static void launch_fused_pro(int pro, dim3 grid, const FusedArgsX& AX) {
  const dim3 block(GEMV_WAVES * 64);
  bool any_res = false;
  for (int i = 0; i < AX.ngroups; i++) any_res = any_res || AX.g[i].res != nullptr;
  if constexpr (SWIGLU) {
    FusedArgs2 P{};
    P.Wg = AX.g[0].W; P.Wu = AX.g[1].W; P.out = AX.g[0].out; P.x = AX.x; P.norm_w = AX.norm_w; P.N = AX.g[0].N; P.steps = AX.step_first[4]; P.nwg = (int)grid.x;
    if (pro == PRO_Q8) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_Q8, true, false, FusedArgs2>), grid, block, 0, stream(), P);
    else if (pro == PRO_BF16) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_BF16, true, false, FusedArgs2>), grid, block, 0, stream(), P);
    else hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_RMSNORM, true, false, FusedArgs2>), grid, block, 0, stream(), P);
    return;
  } else {
    if (AX.ngroups == 1) {         // one matrix
      FusedArgs1 P{};
      P.g0 = AX.g[0]; P.x = AX.x; P.norm_w = AX.norm_w; P.x_bstride = AX.x_bstride; P.steps = AX.step_first[4]; P.nwg = (int)grid.x;
      if (pro == PRO_Q8) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_Q8, false, false, FusedArgs1>), grid, block, 0, stream(), P);
      else if (pro == PRO_BF16) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_BF16, false, false, FusedArgs1>), grid, block, 0, stream(), P);
      else if (pro == PRO_RMSNORM) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_RMSNORM, false, false, FusedArgs1>), grid, block, 0, stream(), P);
      else if constexpr (KB == 8) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_GNORM, false, false, FusedArgs1>), grid, block, 0, stream(), P);
      return;
    }
    if (!any_res && pro != PRO_GNORM) {      // several matrices, no residual: the 104 / 128-byte forms
      FusedArgsCX P{};
      for (int i = 0; i < 4; i++) {
        const int j = i < AX.ngroups ? i : AX.ngroups - 1;
        P.W[i] = AX.g[j].W; P.out[i] = AX.g[j].out; P.N[i] = AX.g[j].N; P.epi4 |= (AX.g[j].epi & 0xff) << (8 * i);
      }
      P.x = AX.x; P.norm_w = AX.norm_w; P.ngroups = AX.ngroups | (int)(grid.x << 8);
      P.conv_st = AX.conv_st; P.conv_st_new = AX.conv_st_new; P.conv_w = AX.conv_w;
      if constexpr (KB == 8 || KB == 4) {
        if (pro == PRO_RMSNORM && AX.conv_st) { hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_RMSNORM, false, true, FusedArgsCX>), grid, block, 0, stream(), P); return; }
      }
      const FusedArgsC& C = P;
      if (pro == PRO_Q8) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_Q8, false, false, FusedArgsC>), grid, block, 0, stream(), C);
      else if (pro == PRO_BF16) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_BF16, false, false, FusedArgsC>), grid, block, 0, stream(), C);
      else hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_RMSNORM, false, false, FusedArgsC>), grid, block, 0, stream(), C);
      return;
    }
    if constexpr (KB == 8) {
      if (pro == PRO_GNORM) { hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_GNORM, false, false, FusedArgsX>), grid, block, 0, stream(), AX); return; }
    }
    if constexpr (KB == 8 || KB == 4) {
      if (pro == PRO_RMSNORM && AX.conv_st) { hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_RMSNORM, false, true, FusedArgsX>), grid, block, 0, stream(), AX); return; }
    }
    const FusedArgs& A = AX;
    if (pro == PRO_Q8) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_Q8, false>), grid, block, 0, stream(), A);
    else if (pro == PRO_BF16) hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_BF16, false>), grid, block, 0, stream(), A);
    else hipLaunchKernelGGL((gemv_fused_kernel<KB, RPI, PRO_RMSNORM, false>), grid, block, 0, stream(), A);
  }
}

int g_tune_fused_cap = 0;     // workgroups per CU of the fused GEMV (0: chosen by the launcher)

// Fast path only (gemv_fused_fast_path says whether it applies); the caller composes the same
// result from separate kernels otherwise.
int launch_gemv_fused(int pro, const void* x, const void* norm_w, int K, int batch, int ngroups, const void* const* W,
                      void* const* out, const void* const* res, const int* N, const int* epi, bool swiglu, const FusedConv* conv) {
  BK_REQUIRE(pro == PRO_Q8 || pro == PRO_BF16 || pro == PRO_RMSNORM || pro == PRO_GNORM, "gemv_fused: bad prologue %d", pro);
  BK_REQUIRE(x && ((pro != PRO_RMSNORM && pro != PRO_GNORM) || norm_w), "gemv_fused: null activation or norm weight");
  BK_REQUIRE(pro != PRO_GNORM || (K == 2048 && !swiglu), "gemv_fused: the gated-norm prologue serves K = 2048 (16 heads of 128), got K=%d", K);
  BK_REQUIRE(gemv_fused_fast_path(K, batch, swiglu), "gemv_fused: K=%d batch=%d is outside the fused kernel's shapes", K, batch);
  BK_REQUIRE(ngroups >= 1 && ngroups <= 4 && (!swiglu || ngroups == 2), "gemv_fused: bad number of matrices %d", ngroups);
  BK_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)norm_w & 15) == 0, "gemv_fused: activation and norm weight must be 16-byte aligned");
  const int KB = K / 256, RPI = KB <= 8 ? 4 : 2;
  const int rows_per_step = swiglu ? RPI / 2 : RPI;
  FusedArgsX A{};
  A.ngroups = ngroups; A.x = x; A.norm_w = (const uint16_t*)norm_w;
  A.x_bstride = pro == PRO_GNORM ? (int64_t)gdn_raw_bytes(K / 128, 1) : 0;
  if (conv) {
    BK_REQUIRE(!swiglu && pro == PRO_RMSNORM && (KB == 8 || KB == 4) && epi[0] == EPI_CONV && conv->st && conv->st_new && conv->w && ((uintptr_t)conv->w & 7) == 0,
               "gemv_fused: the conv epilogue serves matrix 0 of an rmsnorm group with K = 1024 or 2048 (state, new state and 8-byte aligned taps given)");
    A.conv_st = (const uint16_t*)conv->st; A.conv_st_new = (uint16_t*)conv->st_new; A.conv_w = (const uint16_t*)conv->w;
  }
  int steps = 0;
  for (int i = 0; i < ngroups; i++) {
    BK_REQUIRE(W[i] && N[i] > 0 && ((uintptr_t)W[i] & 15) == 0, "gemv_fused: matrix %d: null, misaligned or N <= 0", i);
    A.g[i].W = (const uint8_t*)W[i];
    A.g[i].N = N[i];
    if (swiglu) {
      BK_REQUIRE(N[i] == N[0], "gemv_fused: gate and up must have the same number of rows");
      A.g[i].out = out[0]; A.g[i].res = nullptr; A.g[i].epi = EPI_BF16;
      A.step_first[i] = 0;
      if (i == 0) { BK_REQUIRE(out[0], "gemv_fused: null output"); steps = (N[0] + rows_per_step - 1) / rows_per_step; }
    } else {
      BK_REQUIRE(out[i], "gemv_fused: matrix %d: null output", i);
      BK_REQUIRE(epi[i] == EPI_F32 || epi[i] == EPI_BF16 || epi[i] == EPI_BF16_ADD || (epi[i] == EPI_CONV && i == 0 && conv),
                 "gemv_fused: bad epilogue %d", epi[i]);
      BK_REQUIRE(epi[i] != EPI_BF16_ADD || res[i], "gemv_fused: the add epilogue needs a residual");
      A.g[i].out = out[i]; A.g[i].res = (const uint16_t*)res[i]; A.g[i].epi = epi[i];
      A.step_first[i] = steps;
      steps += (N[i] + rows_per_step - 1) / rows_per_step;
    }
  }
  for (int i = swiglu ? 1 : ngroups; i < 5; i++) A.step_first[i] = steps;
  if (swiglu) A.step_first[0] = 0;
  int wgs = (steps + GEMV_WAVES - 1) / GEMV_WAVES;
  // With a prologue every workgroup repeats the RMSNorm / Q8_1 work of the row, so fewer, longer-lived workgroups win:
  // two per CU measured best (three per CU, one step per wave: 4 % slower over the decode step; one per CU: the rows
  // in flight no longer cover the memory latency).  Without a prologue the plain GEMV's rule applies.
  if (g_tune_fused_cap > 0 || pro != PRO_Q8) {
    const int cap = num_cus() * (g_tune_fused_cap > 0 ? g_tune_fused_cap : 2);
    if (wgs > cap) wgs = cap;
  } else {
    wgs = gemv_grid_for(wgs);
  }
  BK_REQUIRE(wgs < (1 << 23), "gemv_fused: %d workgroups exceed what the argument block encodes", wgs);
  A.nwg = wgs;
  const dim3 grid(wgs, batch);
  if (swiglu && KB == 4) launch_fused_pro<4, 4, true>(pro, grid, A);
  else if (swiglu) launch_fused_pro<8, 4, true>(pro, grid, A);
  else if (KB == 4) launch_fused_pro<4, 4, false>(pro, grid, A);
  else if (KB == 8) launch_fused_pro<8, 4, false>(pro, grid, A);
  else if (KB == 14) launch_fused_pro<14, 2, false>(pro, grid, A);
  else if (KB == 16) launch_fused_pro<16, 2, false>(pro, grid, A);
  else launch_fused_pro<24, 2, false>(pro, grid, A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
