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
#include <algorithm>
#include <type_traits>
#include "attn_args.h"

namespace bk {

int g_tune_prefill_ksplit = 0;    // runs along K/V of the tiled prompt attention (0: from the shape)
int g_tune_prefill_xmap = 1;      // 0: plain three-dimensional grid instead of the XCD-aware mapping

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
  // ksplit > 1: blockIdx.z cuts the K/V tiles of a workgroup into ksplit runs (a launch with fewer workgroups than CUs);
  // every run leaves its rows unnormalised, a second kernel joins them
  int ksplit, nx, xmap;             // nx: query tiles; xmap: 0 = three-dimensional grid, 1 / 2 = XCD-aware one-dimensional grid (see the kernel)
  float* part_o;                   // f32 [ksplit, T, NH, 256]
  float* part_ml;                  // f32 [ksplit, T, NH, 2]: reference exponent (base 2), sum of weights
};

// K/V tiles travel from memory straight into LDS (lds_dma16_s: lane l of a wave fills the l-th 16-byte slot of a 1 KiB
// piece of LDS from an address of its own choosing), two tiles deep: no registers hold them and no wave spends
// instructions on the copy.  A slot's position is fixed by the lane, so rows cannot be padded against bank conflicts;
// instead a piece holds exactly what one operand read of the matrix instructions takes, in lane order or a permutation of
// it inside each group of 16 lanes, and every transfer reads from one page (a scalar base per page, a constant offset
// per lane: no address arithmetic in the tile loop):
//   K piece (page p, dim group sp): slot 16 c + t = dims 32 sp + 8 c .. + 8 of token t of the page (c = 0..3);
//     the read of dim slice sl = 2 sp + e for token rows 32 u + tau(col) finds token tau at piece (2 u + tau / 16, sp),
//     slot 16 (2 e + half) + tau % 16
//   V piece (page jj, dim tile dt): slot 32 h + c = tokens 8 h .. + 8 of the page for dim 32 dt + c: lane l reads slot l
__global__ __launch_bounds__(PF_THREADS) void attn_prefill_kernel(PrefillAttnArgs A) {
  __shared__ __align__(1024) unsigned char lds_tiles[2 * PF_BUF];
  __shared__ int lds_len[PF_ROWS];
  __shared__ __align__(16) int lds_bt[PF_MAX_PAGES + 4];        // (+ 4: the last tile's four entries always exist)
  __shared__ int lds_maxlen;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5, col = lane & 31;
  // Workgroup -> (query tile x, KV head, run).  The workgroups of one (KV head, run) read the same K/V tiles at about the
  // same time: where the number of such groups divides 8 or is a multiple of it (xmap > 0) the launch is one-dimensional
  // and a group's workgroups run on the same XCD(s) - consecutive workgroup ids go round the 8 XCDs - so that a tile comes
  // from memory once per group and its other readers find it in that XCD's L2; the query tiles of a group are dealt out
  // to its XCDs in turn, longest rows first on each.
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  if (A.xmap > 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, groups = A.NKV * max(A.ksplit, 1);
    int g;
    if (A.xmap == 1) { const int P = 8 / groups; g = xcd / P; bx = slot * P + xcd % P; }     // P XCDs per group
    else { g = xcd * (groups >> 3) + slot / A.nx; bx = slot % A.nx; }                          // groups / 8 groups per XCD
    if (bx >= A.nx) return;
    by = g % A.NKV; bz = g / A.NKV;
  }
  const int kvh = by;
  const int t0 = (A.nx - 1 - bx) * A.QT;      // the longest rows (last tokens) start first

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
  if (maxlen == 0) return;                  // no row has a context: nothing is written (the join skips such rows too)
  const int npages = (maxlen + ATT_PAGE - 1) / ATT_PAGE;
  const int ntiles_all = (maxlen + PF_TILE - 1) / PF_TILE;
  // this workgroup's run of tiles (the whole context unless the launch is cut along K/V)
  const int zsplit = bz;
  const int tile_lo = A.ksplit > 1 ? (int)((int64_t)zsplit * ntiles_all / A.ksplit) : 0;
  const int ntiles = A.ksplit > 1 ? (int)((int64_t)(zsplit + 1) * ntiles_all / A.ksplit) : ntiles_all;
  // a page past the longest row (the last tile may be short) reads the last page again; its tokens are masked below
  for (int i = tid; i < 4 * ntiles_all; i += PF_THREADS) lds_bt[i] = A.block_table[min(i, npages - 1)];
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

  // Transfers of the K and of the V part of a tile into buffer tile % 2.  Round i of wave w fills piece 4 i + w: page
  // i / 2 of the tile, K dim group / V dim tile 4 (i % 2) + w.  `off` holds the byte offsets of the tile's four pages in
  // the caches (scalar registers).
  const uint32_t kvoff0 = (uint32_t)((lane & 15) * (ATT_HD * 2) + (lane >> 4) * 16 + wave * 64);      // bytes inside the page's K block; + 256 for odd i
  const uint32_t vvoff0 = (uint32_t)((32 * wave + col) * (ATT_PAGE * 2) + half * 16);                 // bytes inside the page's V block; + 4096 for odd i
  const uint32_t kvoff1 = kvoff0 + 256, vvoff1 = vvoff0 + 4096;
  const int64_t page_bytes = (int64_t)A.NKV * (ATT_PAGE * ATT_HD * 2);
  const unsigned char* kc_head = (const unsigned char*)A.kc + (int64_t)kvh * (ATT_PAGE * ATT_HD * 2);
  const unsigned char* vc_head = (const unsigned char*)A.vc + (int64_t)kvh * (ATT_PAGE * ATT_HD * 2);
  struct PageOff { int64_t b[4]; };
  auto page_offsets = [&](const int4& pg4) {        // pg4: the four block-table entries, the same in every lane
    PageOff r;
    r.b[0] = __builtin_amdgcn_readfirstlane(pg4.x) * page_bytes; r.b[1] = __builtin_amdgcn_readfirstlane(pg4.y) * page_bytes;
    r.b[2] = __builtin_amdgcn_readfirstlane(pg4.z) * page_bytes; r.b[3] = __builtin_amdgcn_readfirstlane(pg4.w) * page_bytes;
    return r;
  };
  auto tile_entries = [&](int tile) { return *(const int4*)&lds_bt[4 * tile]; };
  auto copy_k1 = [&](int tile, const PageOff& off, int i) {
    lds_dma16_s(kc_head + off.b[i >> 1], (i & 1) ? kvoff1 : kvoff0, lds_tiles + (tile & 1) * PF_BUF + (4 * i + wave) * 1024);
  };
  auto copy_v1 = [&](int tile, const PageOff& off, int i) {
    lds_dma16_s(vc_head + off.b[i >> 1], (i & 1) ? vvoff1 : vvoff0, lds_tiles + (tile & 1) * PF_BUF + PF_KBYTES + (4 * i + wave) * 1024);
  };
  // What the cache holds behind the longest row need not be a number, and 0 * NaN would reach the output: the values
  // of those tokens become zeros in LDS (the tile that holds the end of the rows only; thread = dim).
  auto land_tile = [&](int tile) {
    __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): this wave's pieces are in LDS
    __syncthreads();
    const int first_bad = maxlen - tile * PF_TILE;
    if (tile < ntiles && first_bad < PF_TILE) {
      unsigned char* vt = lds_tiles + (tile & 1) * PF_BUF + PF_KBYTES + ((tid >> 5) * 64 + (tid & 31)) * 16;      // dim tid: piece (jj, tid / 32), slot 32 h + tid % 32
      for (int tk = max(first_bad, 0); tk < PF_TILE; tk++) *(uint16_t*)(vt + (tk >> 4) * 8192 + ((tk >> 3) & 1) * 512 + (tk & 7) * 2) = 0;
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
  wave_minlen = __builtin_amdgcn_readfirstlane(wave_minlen);       // (the same in every lane: a scalar branch below, not a masked region)

  // Row `col` of the first product's A operand is K token tau(col) of the 32 (bits 2 and 3 of col exchanged): the
  // result registers 8 jj .. 8 jj + 7 of a lane then belong to the 8 consecutive tokens 16 jj + 8 half .. + 8, which is
  // one 16-byte unit of a V row — the B operand of the second product needs no shuffle and its A operand is one read.
  const int tau = (col & 0x13) | ((col & 4) << 1) | ((col & 8) >> 1);
  const int kread_off = (tau >> 4) * 8192 + ((tau & 15) + 16 * half) * 16;      // + u * 16384 + (sl / 2) * 1024 + (sl % 2) * 512
  const int vread_off = lane * 16;                                            // + (jj * 8 + dt) * 1024

  // ---- The tile loop, software-pipelined by hand: a wave is alone on its SIMD, so the matrix unit only stays busy while
  // the same wave issues other work between two matrix instructions.  Iteration t runs
  //   A: the first product of tile t + 1 (32 matrix instructions), between them the softmax of tile t and the eight
  //      transfers of K of tile t + 2,
  //   B: the second product of tile t (32 matrix instructions), between them the eight transfers of V of tile t + 1 (in
  //      its first half) and the read-out of the scores of tile t + 1 (in its second half).
  // The transfers go into the buffers that iteration t - 1 finished with.  They stand between the matrix instructions
  // because a wave waits at the issue of a transfer until the CU's path from the caches to LDS has taken it (about 30
  // cycles; all sixteen in one burst at the top of the iteration: 1600 of 5200 cycles per tile), and without a branch
  // around them because behind a branch the compiler gathers the softmax in front of the whole product; past the last
  // tile the last tile simply travels again, into a buffer nobody reads any more.  One wait + barrier per iteration: both
  // parts are read right behind it (K of tile t + 2 by A of iteration t + 1, V of tile t + 1 by its B).
  f32x16_t s[2];                        // scores of the current tile, in vector registers
  uint4 pb[4];
  float alpha = 1.0f;

  // phase A.  MM: compute sn = S^T of the K tile at lds_k.  SM: softmax of s -> pb, alpha, mrow, lrow.
  auto phase_a = [&](auto MMc, auto SMc, const unsigned char* lds_k, f32x16_t (&sn)[2], int ktile, const PageOff& koffs) {
    constexpr bool MM = decltype(MMc)::value, SM = decltype(SMc)::value;
    f32x16_t zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.0f;
    uint4 ka[2][4];
    auto kread = [&](int bt, uint4 (&dst)[4]) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int sl = 2 * bt + (i >> 1);
        dst[i] = *(const uint4*)(lds_k + kread_off + (i & 1) * 16384 + (sl >> 1) * 1024 + (sl & 1) * 512);
      }
    };
    float mloc = -INFINITY, mnew = 0.0f, msub = 0.0f, psum = 0.0f, mloc2 = 0.0f;
    if constexpr (MM) kread(0, ka[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int bt = 0; bt < 8; bt++) {
      if constexpr (MM) {
        if (bt + 1 < 8) kread(bt + 1, ka[(bt + 1) & 1]);
        // (the operand requested last is used first: the one wait in front of it covers the other three, and the
        // requests of the next batch, issued in front of this batch's products, have four products' time to arrive)
#pragma unroll
        for (int i = 3; i >= 0; i--)
          sn[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka[bt & 1][i]),
                                                              __builtin_bit_cast(bf16x8_t, qreg[2 * bt + (i >> 1)]),
                                                              (bt == 0 && i >= 2) ? zero16 : sn[i & 1], 0, 0, 0);
      }
      if constexpr (SM) {
        // running-maximum softmax of the row (base 2), cut into eight pieces.  The maximum is taken over the raw scores
        // (the scale is positive); scale and subtraction are one fused multiply-add in front of the hardware exponential
        // (v_exp_f32: 1 ulp, results below 2^-126 become 0 - far inside the 2e-2 of this kernel).
        if (bt == 0 || bt == 1) {
#pragma unroll
          for (int r = 0; r < 16; r++) mloc = fmaxf(mloc, s[bt][r]);
          if (bt == 1) mloc2 = __shfl_xor(mloc, 32);
        }
        if (bt == 2) {
          mloc = fmaxf(mloc, mloc2) * A.scale_log2;
          // The reference exponent of a row follows its maximum only when that has grown by more than 2^24 (or is the
          // first): weights up to 2^24 are as exact in bf16 and f32 as weights up to 1, and the 128 accumulators of a
          // lane need their rescaling pass in a few early tiles only.
          mnew = (mloc > mrow + 24.0f) ? mloc : mrow;
          msub = mnew == -INFINITY ? 0.0f : mnew;             // a row without any token so far: every weight is 0
          alpha = mnew == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(mrow - mnew);   // (first tile with a token: exp2(-inf) = 0 times the zeros)
          mrow = mnew;
        }
        if (bt >= 3 && bt <= 6) {
          const int j = bt - 3;
          float p[8];
#pragma unroll
          for (int e = 0; e < 8; e++) { p[e] = __builtin_amdgcn_exp2f(__fmaf_rn(s[j >> 1][8 * (j & 1) + e], A.scale_log2, -msub)); psum += p[e]; }
          pb[j] = make_uint4(pk_bf16(p[0], p[1]), pk_bf16(p[2], p[3]), pk_bf16(p[4], p[5]), pk_bf16(p[6], p[7]));
        }
        if (bt == 7) lrow = lrow * alpha + psum;
      }
      if constexpr (MM && SM) {
        // the next batch's four operand reads, then one matrix instruction and this piece's share of the vector work, four times
        constexpr int NV = 7;
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x402, NV, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (MM && SM) {
        copy_k1(ktile, koffs, bt);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // the rows that end inside the tile are cut off
  auto mask_scores = [&](int tile) {
    const int tok_base = tile * PF_TILE;
    if (tok_base + PF_TILE > wave_minlen) {                         // (wave-uniform) the tile crosses the end of a row
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          if (tok_base + 32 * u + 16 * (r >> 3) + 8 * half + (r & 7) >= mylen) s[u][r] = -INFINITY;
          if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);       // (a few comparison masks at a time: all 32 at once spill scalar registers)
        }
    }
  };
  // scores 8 q .. 8 q + 7 of sn leave the matrix unit's registers (once: pinned, or the masked branch makes the compiler
  // read them out in front of the branch and again behind it)
  auto take_scores = [&](f32x16_t (&sn)[2], int q) {
#pragma unroll
    for (int e = 0; e < 8; e++) { float x = sn[q >> 1][8 * (q & 1) + e]; asm volatile("" : "+v"(x)); s[q >> 1][8 * (q & 1) + e] = x; }
  };
  using std::true_type;
  using std::false_type;

  PageOff offs_next{};                  // pages of tile t + 1 (V transfers of iteration t; they were the K transfers of t - 1)
  if (tile_lo < ntiles) {
    const PageOff o0 = page_offsets(tile_entries(tile_lo));
    offs_next = page_offsets(tile_entries(min(tile_lo + 1, ntiles - 1)));
#pragma unroll
    for (int i = 0; i < 8; i++) copy_k1(tile_lo, o0, i);
#pragma unroll
    for (int i = 0; i < 8; i++) copy_v1(tile_lo, o0, i);
#pragma unroll
    for (int i = 0; i < 8; i++) copy_k1(tile_lo + 1, offs_next, i);
  }
  land_tile(tile_lo);
  if (tile_lo < ntiles) {
    f32x16_t sn[2];
    phase_a(true_type{}, false_type{}, lds_tiles + (tile_lo & 1) * PF_BUF, sn, 0, offs_next);
#pragma unroll
    for (int q = 0; q < 4; q++) take_scores(sn, q);
    mask_scores(tile_lo);
  }
#ifdef PF_PROF
  long long pc[8] = {0, 0, 0, 0, 0, 0, 0, 0}, pt = clock64(), pn;
#define PF_MARK(k) { __builtin_amdgcn_sched_barrier(0); pn = clock64(); pc[k] += pn - pt; pt = pn; __builtin_amdgcn_sched_barrier(0); }
#else
#define PF_MARK(k)
#endif
  int4 entries2 = tile_lo < ntiles ? tile_entries(min(tile_lo + 2, ntiles - 1)) : make_int4(0, 0, 0, 0);   // block-table entries of tile t + 2
  for (int tile = tile_lo; tile < ntiles; tile++) {
    PF_MARK(0)
    const unsigned char* lds_v = lds_tiles + (tile & 1) * PF_BUF + PF_KBYTES;
    const unsigned char* lds_kn = lds_tiles + ((tile + 1) & 1) * PF_BUF;
    const PageOff voffs = offs_next;                       // tile t + 1
    const PageOff koffs = page_offsets(entries2);         // tile t + 2 (read from LDS an iteration ago)
    offs_next = koffs;
    entries2 = tile_entries(min(tile + 3, ntiles - 1));
    PF_MARK(1)
    f32x16_t sn[2];
    if (tile + 1 < ntiles) phase_a(true_type{}, true_type{}, lds_kn, sn, tile + 2, koffs);
    else phase_a(false_type{}, true_type{}, lds_kn, sn, 0, koffs);
    PF_MARK(2)
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
    PF_MARK(3)
    // ---- values: O^T[dim 32 dt + .., row] += V^T . P^T over the four 16-token slices, the A operands a batch
    // (one slice, four dim tiles) ahead
    {
      uint4 va[2][4];
      auto vread = [&](int b, uint4 (&dst)[4]) {       // batch b: slice b / 2, dim tiles 4 (b % 2) .. + 4
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i] = *(const uint4*)(lds_v + vread_off + ((b >> 1) * 8 + 4 * (b & 1) + i) * 1024);
      };
      vread(0, va[0]);
#pragma unroll
      for (int b = 0; b < 8; b++) {
        if (b + 1 < 8) vread(b + 1, va[(b + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 3; i >= 0; i--) {                  // (last request first, as above)
          const int dt = 4 * (b & 1) + i;
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, va[b & 1][i]), __builtin_bit_cast(bf16x8_t, pb[b >> 1]), o[dt], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (b < 4) { copy_v1(tile + 1, voffs, 2 * b); copy_v1(tile + 1, voffs, 2 * b + 1); }      // (early: they must have arrived at the end of the iteration)
        if (b >= 4) take_scores(sn, b - 4);           // (sn is complete long before; past the last tile it holds nothing and is not used)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    PF_MARK(4)
    if (tile + 1 < ntiles) mask_scores(tile + 1);
    PF_MARK(5)
    land_tile(tile + 1);           // (also the barrier behind which this tile's buffers may be overwritten)
    PF_MARK(6)
  }
#ifdef PF_PROF
  if (bx == 3 && by == 0 && bz == 0 && lane == 0)
    printf("wave %d tiles %d: top %lld copy %lld A %lld rescale %lld B %lld take %lld land %lld\n", wave, ntiles - tile_lo, pc[0], pc[1], pc[2], pc[3], pc[4], pc[5], pc[6]);
#endif

  // ---- output: the row's two lanes hold dims 32 dt + 8 (r / 4) + 4 half + r % 4
  const float ltot = lrow + __shfl_xor(lrow, 32);
  if (mylen <= 0 || tq >= A.T) return;
  if (A.ksplit > 1) {
    // the run's share of the row as it stands: a row that saw no token in this run leaves (-inf, 0) and is skipped by the join
    const int64_t prow = ((int64_t)zsplit * A.T + tq) * A.NH + head;
    if (half == 0) *(float2*)(A.part_ml + prow * 2) = make_float2(mrow, ltot);
    float* po = A.part_o + prow * ATT_HD;
#pragma unroll
    for (int dt = 0; dt < 8; dt++)
#pragma unroll
      for (int g = 0; g < 4; g++)
        *(float4*)(po + 32 * dt + 8 * g + 4 * half) = make_float4(o[dt][4 * g], o[dt][4 * g + 1], o[dt][4 * g + 2], o[dt][4 * g + 3]);
    return;
  }
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

// Join of the runs of a launch cut along K/V: a wave per (token, head), lane = four dims, four rows per workgroup.
__global__ __launch_bounds__(256) void attn_prefill_join_kernel(PrefillAttnArgs A) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);        // row = t * NH + head
  if (r >= (int64_t)A.T * A.NH) return;
  const int t = (int)(r / A.NH), head = (int)(r - (int64_t)t * A.NH), d = 4 * lane;
  if (min(max(A.pos[t] + 1, 0), A.max_ctx) <= 0) return;         // a row without context is left alone, as in the uncut launch
  float m[4], l[4], M = -INFINITY;
  float4 o[4];
#pragma unroll
  for (int z = 0; z < 4; z++) {                                   // all requests first (a run that does not exist reads run 0 again)
    const int64_t pr = (int64_t)(z < A.ksplit ? z : 0) * A.T * A.NH + r;
    const float2 ml = *(const float2*)(A.part_ml + pr * 2);
    o[z] = *(const float4*)(A.part_o + pr * ATT_HD + d);
    m[z] = z < A.ksplit ? ml.x : -INFINITY; l[z] = ml.y;
    M = fmaxf(M, m[z]);
  }
  uint2 gw = make_uint2(0, 0);
  if (A.gate) gw = *(const uint2*)(A.gate + (int64_t)t * A.gate_bstride + (int64_t)head * A.gate_hstride + d);
  float L = 0.0f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int z = 0; z < 4; z++) {
    if (m[z] != -INFINITY) {                                      // (wave-uniform; a run in which the row saw no token holds nothing usable)
      const float w = __builtin_amdgcn_exp2f(m[z] - M);
      L += l[z] * w;
      acc.x += o[z].x * w; acc.y += o[z].y * w; acc.z += o[z].z * w; acc.w += o[z].w * w;
    }
  }
  const float inv = L > 0.0f ? 1.0f / L : 0.0f;
  float v[4] = {acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv};
  if (A.gate) {
    v[0] = __fmul_rn(v[0], sigmoid_f64(__uint_as_float(gw.x << 16)));
    v[1] = __fmul_rn(v[1], sigmoid_f64(__uint_as_float(gw.x & 0xffff0000u)));
    v[2] = __fmul_rn(v[2], sigmoid_f64(__uint_as_float(gw.y << 16)));
    v[3] = __fmul_rn(v[3], sigmoid_f64(__uint_as_float(gw.y & 0xffff0000u)));
  }
  *(uint2*)(A.out + r * ATT_HD + d) = make_uint2(pk_bf16(v[0], v[1]), pk_bf16(v[2], v[3]));
}

bool attn_prefill_tiled_serves(int NH, int NKV, int max_ctx) {
  if (NKV <= 0 || NH % NKV) return false;
  const int G = NH / NKV;
  return (G == 1 || G == 2 || G == 4 || G == 8 || G == 16) && (max_ctx + ATT_PAGE - 1) / ATT_PAGE <= PF_MAX_PAGES;
}

// How many runs along K/V a launch is cut into: as many as it takes to give every CU a workgroup (at most 4), while a run
// keeps at least 8 tiles of the longest context.
int attn_prefill_ksplit(int T, int NH, int NKV, int max_ctx) {
  if (g_tune_prefill_ksplit > 0) return g_tune_prefill_ksplit > 4 ? 4 : g_tune_prefill_ksplit;
  const int QT = PF_ROWS / (NH / NKV);
  const int wgs = ((T + QT - 1) / QT) * NKV;
  int ks = num_cus() / (wgs > 0 ? wgs : 1);
  const int by_len = ((max_ctx + PF_TILE - 1) / PF_TILE) / 8;
  if (ks > by_len) ks = by_len;
  return ks < 1 ? 1 : (ks > 4 ? 4 : ks);
}
size_t attn_prefill_workspace_bytes(int T, int NH, int NKV, int max_ctx) {
  const int ks = attn_prefill_ksplit(T, NH, NKV, max_ctx);
  return ks > 1 ? (size_t)ks * T * NH * (ATT_HD + 2) * sizeof(float) : 0;
}

int launch_attn_prefill_tiled(const void* q, const void* kc, const void* vc, const int32_t* block_table, const int32_t* pos, int max_ctx,
                              const void* gate, int64_t gate_bstride, int64_t gate_hstride, void* out, int T, int NH, int NKV, int HD,
                              int page_size, void* workspace, size_t workspace_bytes) {
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
  A.ksplit = attn_prefill_ksplit(T, NH, NKV, max_ctx);
  {   // a workspace smaller than the cut asks for (none at all: the plain launch) holds fewer runs
    const size_t per_run = (size_t)T * NH * (ATT_HD + 2) * sizeof(float);
    const int fits = workspace ? (int)std::min<size_t>(workspace_bytes / per_run, 4) : 0;
    if (A.ksplit > fits) A.ksplit = fits > 1 ? fits : 1;
  }
  if (A.ksplit > 1) {
    A.part_o = (float*)workspace;
    A.part_ml = A.part_o + (size_t)A.ksplit * T * NH * ATT_HD;
  }
  A.nx = (T + A.QT - 1) / A.QT;
  const int groups = NKV * A.ksplit;
  A.xmap = g_tune_prefill_xmap == 0 ? 0 : (8 % groups == 0 ? 1 : (groups % 8 == 0 ? 2 : 0));
  dim3 grid(A.nx, NKV, A.ksplit);
  if (A.xmap == 1) grid = dim3(8 * ((A.nx + 8 / groups - 1) / (8 / groups)));
  else if (A.xmap == 2) grid = dim3(A.nx * groups);
  hipLaunchKernelGGL(attn_prefill_kernel, grid, dim3(PF_THREADS), 0, stream(), A);
  if (A.ksplit > 1) hipLaunchKernelGGL(attn_prefill_join_kernel, dim3((unsigned)(((int64_t)T * NH + 3) / 4)), dim3(256), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
