// Causal attention for the tokens of a prompt, tiled: a query tile against K/V tiles through LDS on the bf16 matrix
// cores (the form of prototypes/fa2_vllm.ts:114-139 for many query rows at once; its host loop is the checker's).
// The decode kernel run per token reads every K/V page once per token (or per pair of tokens); here the 128 query rows
// of a workgroup — 128 / G consecutive tokens x the G query heads that share a KV head — read each K/V tile of 64
// tokens once, from LDS.
//
// Both products are computed transposed, as in the decode kernel (attn.hip), so that a query row stays in one lane
// (two lanes: the halves of the wave) from the scores to the output and nothing moves between lanes but one maximum:
//   S^T[tok, row] = sum_d K[tok, d] * Q[row, d]       v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q in registers
//   O^T[d, row]   = sum_tok V^T[d, tok] * P^T[tok, row]    same instruction, A = V (dim-major pages) from LDS, B = P
// A lane of the S^T result holds, for its row, rows 8g + 4h + v (g, v = 0..3, h = its half of the wave) of the first
// product's 32; those rows are given K tokens in an order (bits 2 and 3 of the row number exchanged) that makes
// registers 8j .. 8j+7 the 8 consecutive tokens 16j + 8h .. + 8: they are the B operand of the second product as they
// stand, and its A operand, the same 8 tokens of one dim, is one 16-byte read of a V row.  Softmax is the running-maximum form in f32 (base-2 exponent); the weights enter the
// second product as bf16.  Results agree with the f64 checker to the 2e-2 of the matrix-instruction decode kernel,
// not to the bit: the double-precision kernel (attn_exact.hip) stays the default of the prompt path.
#include "attn_args.h"

namespace bk {

typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

// two f32 -> two bf16 (round to nearest even) in one instruction, a in the low half
__device__ __forceinline__ uint32_t pk_bf16(float a, float b) { return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){a, b}, bf16x2_t)); }

constexpr int PF_THREADS = 256;
constexpr int PF_ROWS = 128;                 // query rows (token, head) of a workgroup; 32 per wave
constexpr int PF_TILE = 64;                  // K/V tokens per tile = 4 pages
constexpr int PF_KBYTES = PF_TILE * ATT_HD * 2;      // a K tile in LDS: 64 rows of 512 bytes
constexpr int PF_VBYTES = ATT_HD * PF_TILE * 2;      // a V tile in LDS: 256 dim rows of 128 bytes (4 pages x 16 tokens)
constexpr int PF_BUF = PF_KBYTES + PF_VBYTES;
constexpr int PF_MAX_PAGES = 4096;           // block-table entries a workgroup keeps in LDS (contexts up to 65536 tokens)

struct PrefillAttnArgs {
  const uint16_t* q;               // bf16 [T, NH, 256], normalised and rotated
  const uint16_t *kc, *vc;         // the caches (pages of one sequence through block_table)
  const int32_t* block_table;      // int32 [max_pages]
  const int32_t* pos;              // int32 [T]: token t attends to cache positions 0 .. pos[t]
  const uint16_t* gate;            // optional output gate, bf16, element (t, head, d) at t * gate_bstride + head * gate_hstride + d
  int64_t gate_bstride, gate_hstride;
  uint16_t* out;                   // bf16 [T, NH, 256]
  int T, NH, NKV, G, gshift, QT, max_ctx;
  float scale_log2;                // softmax scale times log2(e)
};

// K/V tiles travel from memory straight into LDS (lds_dma16: lane l of a wave fills the l-th 16-byte
// slot of a 1 KiB piece of LDS from an address of its own choosing), two tiles deep: no registers hold them and no
// wave spends instructions on the copy.  A slot's position is fixed by the lane, so rows cannot be padded against bank
// conflicts; instead the 16-byte units of a row are stored exclusive-or'ed with a few bits of the row number
// (K: unit ^ (row % 16); V: unit ^ ((dim / 2) % 8)), which spreads the 32 rows of an operand read over all banks.
__global__ __launch_bounds__(PF_THREADS) void attn_prefill_kernel(PrefillAttnArgs A) {
  __shared__ __align__(1024) unsigned char lds_tiles[2 * PF_BUF];
  __shared__ int lds_len[PF_ROWS];
  __shared__ int lds_bt[PF_MAX_PAGES];
  __shared__ int lds_maxlen;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5, col = lane & 31;
  const int kvh = blockIdx.y;
  const int t0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * A.QT;      // the longest rows (last tokens) start first

  if (tid == 0) lds_maxlen = 0;
  __syncthreads();
  if (tid < PF_ROWS) {
    const int t = t0 + tid;
    const int len = (tid < A.QT && t < A.T) ? min(max(A.pos[t] + 1, 0), A.max_ctx) : 0;
    lds_len[tid] = len;
    if (len > 0) atomicMax(&lds_maxlen, len);
  }
  __syncthreads();
  const int maxlen = lds_maxlen;
  if (maxlen == 0) return;
  const int npages = (maxlen + ATT_PAGE - 1) / ATT_PAGE;
  const int ntiles = (maxlen + PF_TILE - 1) / PF_TILE;
  for (int i = tid; i < npages; i += PF_THREADS) lds_bt[i] = A.block_table[i];
  __syncthreads();

  // this lane's query row: token t0 + m / G, head kvh * G + m % G
  const int m = 32 * wave + col;
  const int tq = t0 + (m >> A.gshift);
  const int head = kvh * A.G + (m & (A.G - 1));
  const int mylen = lds_len[m >> A.gshift];
  uint4 qreg[16];
  {
    const uint16_t* qp = A.q + ((int64_t)min(tq, A.T - 1) * A.NH + head) * ATT_HD + 8 * half;
#pragma unroll
    for (int s = 0; s < 16; s++) qreg[s] = *(const uint4*)(qp + 16 * s);
  }

  // A page past the longest row (the last tile may be short) reads the last page again; its tokens are masked below.
  auto page_base = [&](int pg) -> int64_t { return ((int64_t)lds_bt[min(pg, npages - 1)] * A.NKV + kvh) * (ATT_PAGE * ATT_HD); };
  // Copy of tile `tile` into buffer tile % 2.  Round i of wave w fills the 1 KiB piece 4 i + w: K rows 2 (4 i + w) and
  // + 1 (lane / 32 picks the row, lane % 32 the slot), V dim rows 8 (4 i + w) .. + 8 (lane / 8 the row, lane % 8 the slot).
  auto copy_tile = [&](int tile) {
    unsigned char* kb = lds_tiles + (tile & 1) * PF_BUF;
    unsigned char* vb = kb + PF_KBYTES;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int piece = 4 * i + wave;
      const int row = 2 * piece + (lane >> 5), unit = (lane & 31) ^ (row & 15);
      const uint16_t* src = A.kc + page_base(tile * 4 + (row >> 4)) + (row & 15) * ATT_HD + unit * 8;
      lds_dma16(src, kb + piece * 1024);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int piece = 4 * i + wave;
      const int dim = 8 * piece + (lane >> 3), unit = (lane & 7) ^ ((dim >> 1) & 7);     // unit = 2 * page + half of the page's tokens
      const uint16_t* src = A.vc + page_base(tile * 4 + (unit >> 1)) + dim * ATT_PAGE + (unit & 1) * 8;
      lds_dma16(src, vb + piece * 1024);
    }
  };
  // What the cache holds behind the longest row need not be a number, and 0 * NaN would reach the output: the values
  // of those tokens become zeros in LDS (the tile that holds the end of the rows only; thread = dim).
  auto land_tile = [&](int tile) {
    __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): this wave's pieces are in LDS
    __syncthreads();
    const int first_bad = maxlen - tile * PF_TILE;
    if (tile < ntiles && first_bad < PF_TILE) {
      unsigned char* vrow = lds_tiles + (tile & 1) * PF_BUF + PF_KBYTES + tid * (PF_TILE * 2);
      for (int tk = max(first_bad, 0); tk < PF_TILE; tk++) *(uint16_t*)(vrow + (((tk >> 3) ^ ((tid >> 1) & 7)) * 16) + (tk & 7) * 2) = 0;
      __syncthreads();
    }
  };

  f32x16_t o[8];
#pragma unroll
  for (int dt = 0; dt < 8; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
  float mrow = -INFINITY, lrow = 0.0f;

  // the shortest row of the wave decides from which tile on the causal mask has to be applied
  int wave_minlen = mylen;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) wave_minlen = min(wave_minlen, __shfl_xor(wave_minlen, off));

  // Row `col` of the first product's A operand is K token tau(col) of the 32 (bits 2 and 3 of col exchanged): the
  // result registers 8 jj .. 8 jj + 7 of a lane then belong to the 8 consecutive tokens 16 jj + 8 half .. + 8, which is
  // one 16-byte unit of a V row — the B operand of the second product needs no shuffle and its A operand is one read.
  const int tau = (col & 0x13) | ((col & 4) << 1) | ((col & 8) >> 1);
  const int khs = half ^ (tau & 15);           // unit 2 sl + half of K row 32 u + tau sits at ((2 sl) ^ khs) * 16
  const int vhs = half ^ ((col >> 1) & 7);     // unit 2 jj + half of V row 32 dt + col sits at ((2 jj) ^ vhs) * 16
  int koff[8], voff[4];
#pragma unroll
  for (int sl = 0; sl < 8; sl++) koff[sl] = tau * (ATT_HD * 2) + (((2 * sl) ^ khs) * 16);      // sl + 8: 256 bytes further
#pragma unroll
  for (int jj = 0; jj < 4; jj++) voff[jj] = col * (PF_TILE * 2) + (((2 * jj) ^ vhs) * 16);

  copy_tile(0);
  land_tile(0);
  for (int tile = 0; tile < ntiles; tile++) {
    const int tok_base = tile * PF_TILE;
    const unsigned char* lds_k = lds_tiles + (tile & 1) * PF_BUF;
    const unsigned char* lds_v = lds_k + PF_KBYTES;
    // the next tile goes to the other buffer, which every wave left at the last barrier
    if (tile + 1 < ntiles) copy_tile(tile + 1);
    {

    // ---- scores, transposed: s[u][r] = S^T[token 32 u + 16 (r / 8) + 8 half + r % 8, this lane's row].  The A operands
    // come from LDS in batches of eight 16-byte reads (four dim slices x the two token halves), requested a batch ahead
    // of the eight matrix instructions that use them: a read directly in front of its instruction costs the whole LDS
    // latency per instruction, with one wave per SIMD and nothing else to run.
    f32x16_t s[2];
    {
      f32x16_t zero16;
#pragma unroll
      for (int r = 0; r < 16; r++) zero16[r] = 0.0f;
      uint4 ka[2][4];
      auto kread = [&](int bt, uint4 (&dst)[4]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int sl = 2 * bt + (i >> 1);
          dst[i] = *(const uint4*)(lds_k + koff[sl & 7] + (sl >> 3) * 256 + (i & 1) * 32 * (ATT_HD * 2));
        }
      };
      kread(0, ka[0]);
#pragma unroll
      for (int bt = 0; bt < 8; bt++) {
        if (bt + 1 < 8) kread(bt + 1, ka[(bt + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; i++)
          s[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka[bt & 1][i]),
                                                             __builtin_bit_cast(bf16x8_t, qreg[2 * bt + (i >> 1)]),
                                                             (bt == 0 && i < 2) ? zero16 : s[i & 1], 0, 0, 0);   // (an inline 0 operand)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- running-maximum softmax of the row (base 2).  The maximum is taken over the raw scores (the scale is positive);
    // scale and subtraction are one fused multiply-add in front of the hardware exponential (v_exp_f32: 1 ulp, results
    // below 2^-126 become 0 — far inside the 2e-2 of this kernel).
    if (tok_base + PF_TILE > wave_minlen) {                         // (wave-uniform) the tile crosses the end of a row
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (tok_base + 32 * u + 16 * (r >> 3) + 8 * half + (r & 7) >= mylen) s[u][r] = -INFINITY;
    }
    float mloc = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
      for (int r = 0; r < 16; r++) mloc = fmaxf(mloc, s[u][r]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32)) * A.scale_log2;
    // The reference exponent of a row follows its maximum only when that has grown by more than 2^24 (or is the first):
    // weights up to 2^24 are as exact in bf16 and f32 as weights up to 1, and the 128 accumulators of a lane need their
    // rescaling pass in a few early tiles only instead of in every tile where some row of the wave sees a new maximum.
    const float mnew = (mloc > mrow + 24.0f) ? mloc : mrow;
    const float msub = mnew == -INFINITY ? 0.0f : mnew;             // a row without any token so far: every weight is 0
    const float alpha = mnew == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(mrow - mnew);   // (first tile with a token: exp2(-inf) = 0 times the zeros)
    mrow = mnew;
    float psum = 0.0f;
    uint4 pb[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float p[8];
#pragma unroll
      for (int e = 0; e < 8; e++) { p[e] = __builtin_amdgcn_exp2f(__fmaf_rn(s[j >> 1][8 * (j & 1) + e], A.scale_log2, -msub)); psum += p[e]; }
      pb[j] = make_uint4(pk_bf16(p[0], p[1]), pk_bf16(p[2], p[3]), pk_bf16(p[4], p[5]), pk_bf16(p[6], p[7]));
    }
    lrow = lrow * alpha + psum;
    if (__builtin_expect(__ballot(alpha != 1.0f) != 0ull, 0)) {        // (rare after the first tiles, see above)
#pragma unroll
      for (int dt = 0; dt < 8; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          // (the accumulators live in the matrix unit's registers; the empty statement pins each one there at this
          // point, so that the copy to a vector register the multiply needs is made here, in the rare branch, and
          // not for all 128 at the top of every tile)
          float x = o[dt][r];
          asm volatile("" : "+a"(x));
          o[dt][r] = x * alpha;
        }
    }
    // ---- values: O^T[dim 32 dt + .., row] += V^T . P^T over the four 16-token slices, the A operands again a batch
    // (one slice, eight dim tiles) ahead
    {
      uint4 va[2][4];
      auto vread = [&](int b, uint4 (&dst)[4]) {       // batch b: slice b / 2, dim tiles 4 (b % 2) .. + 4
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i] = *(const uint4*)(lds_v + voff[b >> 1] + (4 * (b & 1) + i) * 32 * (PF_TILE * 2));
      };
      vread(0, va[0]);
#pragma unroll
      for (int b = 0; b < 8; b++) {
        if (b + 1 < 8) vread(b + 1, va[(b + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int dt = 4 * (b & 1) + i;
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, va[b & 1][i]), __builtin_bit_cast(bf16x8_t, pb[b >> 1]), o[dt], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    }
    land_tile(tile + 1);           // (also the barrier behind which this tile's buffer may be overwritten)
  }

  // ---- output: the row's two lanes hold dims 32 dt + 8 (r / 4) + 4 half + r % 4
  const float ltot = lrow + __shfl_xor(lrow, 32);
  if (mylen <= 0 || tq >= A.T) return;
  const float inv = ltot > 0.0f ? 1.0f / ltot : 0.0f;
  uint16_t* op = A.out + ((int64_t)tq * A.NH + head) * ATT_HD;
  const uint16_t* gp = A.gate ? A.gate + (int64_t)tq * A.gate_bstride + (int64_t)head * A.gate_hstride : nullptr;
#pragma unroll
  for (int dt = 0; dt < 8; dt++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const int d = 32 * dt + 8 * g + 4 * half;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = o[dt][4 * g + e] * inv;
      if (gp) {
        const uint2 gw = *(const uint2*)(gp + d);
        v[0] = __fmul_rn(v[0], sigmoid_f64(__uint_as_float(gw.x << 16)));
        v[1] = __fmul_rn(v[1], sigmoid_f64(__uint_as_float(gw.x & 0xffff0000u)));
        v[2] = __fmul_rn(v[2], sigmoid_f64(__uint_as_float(gw.y << 16)));
        v[3] = __fmul_rn(v[3], sigmoid_f64(__uint_as_float(gw.y & 0xffff0000u)));
      }
      *(uint2*)(op + d) = make_uint2(pk_bf16(v[0], v[1]), pk_bf16(v[2], v[3]));
    }
}

bool attn_prefill_tiled_serves(int NH, int NKV, int max_ctx) {
  if (NKV <= 0 || NH % NKV) return false;
  const int G = NH / NKV;
  return (G == 1 || G == 2 || G == 4 || G == 8 || G == 16) && (max_ctx + ATT_PAGE - 1) / ATT_PAGE <= PF_MAX_PAGES;
}

int launch_attn_prefill_tiled(const void* q, const void* kc, const void* vc, const int32_t* block_table, const int32_t* pos, int max_ctx,
                              const void* gate, int64_t gate_bstride, int64_t gate_hstride, void* out, int T, int NH, int NKV, int HD,
                              int page_size) {
  BK_REQUIRE(q && kc && vc && block_table && pos && out, "attn_prefill: null pointer");
  BK_REQUIRE(HD == ATT_HD && page_size == ATT_PAGE, "attn_prefill: this build serves head_dim 256 and 16-token pages (got %d, %d)", HD, page_size);
  BK_REQUIRE(T >= 1 && T <= 65535 * 8 && NKV >= 1 && NKV <= 65535 && max_ctx >= 1, "attn_prefill: bad T=%d / NKV=%d / max_ctx=%d", T, NKV, max_ctx);
  BK_REQUIRE(attn_prefill_tiled_serves(NH, NKV, max_ctx),
             "attn_prefill: the tiled kernel serves 1, 2, 4, 8 or 16 query heads per KV head and contexts up to %d tokens (NH=%d NKV=%d max_ctx=%d)",
             PF_MAX_PAGES * ATT_PAGE, NH, NKV, max_ctx);
  BK_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)kc & 15) == 0 && ((uintptr_t)vc & 15) == 0 && ((uintptr_t)out & 7) == 0 &&
             ((uintptr_t)gate & 7) == 0 && gate_bstride % 4 == 0 && gate_hstride % 4 == 0, "attn_prefill: misaligned pointer or gate stride");
  PrefillAttnArgs A{};
  A.q = (const uint16_t*)q; A.kc = (const uint16_t*)kc; A.vc = (const uint16_t*)vc; A.block_table = block_table; A.pos = pos;
  A.gate = (const uint16_t*)gate; A.gate_bstride = gate_bstride; A.gate_hstride = gate_hstride; A.out = (uint16_t*)out;
  A.T = T; A.NH = NH; A.NKV = NKV; A.G = NH / NKV; A.max_ctx = max_ctx;
  A.gshift = 0;
  while ((1 << A.gshift) < A.G) A.gshift++;
  A.QT = PF_ROWS / A.G;
  A.scale_log2 = (float)(1.4426950408889634 / sqrt((double)ATT_HD));
  const dim3 grid((T + A.QT - 1) / A.QT, NKV);
  hipLaunchKernelGGL(attn_prefill_kernel, grid, dim3(PF_THREADS), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
