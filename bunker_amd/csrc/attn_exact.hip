// Decode attention in double precision: the same split-K, paged, grouped-query attention as attn.hip, with every
// product and sum carried in f64, so that the result is the correctly rounded value of the mathematical expression
// (up to ~1e-15 relative before the single rounding to f32) and therefore the same bf16 bits as the host loop of
// prototypes/fa2_vllm.ts:114-139 evaluated in JavaScript numbers (doubles) — whatever the split count, the tile
// order or the batch.  bf16 x bf16 products are exact in f64; the order of the additions only moves the ~1e-16 tail.
//
// A workgroup walks its page range in tiles of 64 tokens (4 pages) with 16 waves in two roles, 8 score waves and 8
// value waves, one tile apart:
//   1. (score waves) the K rows of the tile go to LDS (coalesced 16-byte loads, one page per round of the 512 threads);
//   2. scores: lane = token, wave = 32 of the 256 dims.  The lane converts its 32 K values to f64 once and multiplies
//      each into the 8 query heads of the group.  A query value is the same for all lanes: it is the DPP operand of
//      v_fmac_f64 (row_newbcast:n = lane n of every row of 16 lanes, for all lanes of the row), read from registers
//      that hold 16 query values each, the same 16 in all four rows, loaded once per workgroup — no cross-lane
//      reduction, no operand traffic, the conversions are shared by the 8 heads.  The 8 partial sums per (head, token)
//      meet through LDS in wave order;
//   3. weights: wave = head.  p = exp(s - ref) in f64; `ref` is a reference exponent per head, set from the first
//      tile's maximum and moved only when a score exceeds it by more than 600 (f64 has the range: no running-max
//      rescale per tile), the sum of p is kept per lane;
//   4. (value waves, one step later) values: wave = 8 tokens of the tile, lane = 4 of the 256 dims (V pages are
//      dim-major, so a lane's 8 tokens of a dim are one 16-byte load and the wave's loads are contiguous); the weights
//      of the wave's 8 tokens x 8 heads sit in four register pairs (16 per pair, again the same in every row) and
//      enter the FMAs through the same DPP broadcast.
// Three barriers per step separate 1 | 2 | 3; the value waves do a quarter, a half and a quarter of their tile in the
// three intervals, so the vector unit always has work of both roles to choose from (4 waves per SIMD) and the waits
// of one role (barriers, LDS, memory) are covered by the other.  Every load is issued a step ahead of its use and
// unconditionally, so the waits count loads instead of draining the queue.
// The value waves' accumulators are added in a fixed tree through LDS; partials of the splits are f64 and a second
// kernel merges them.  Roughly 90 vector instructions per (token, KV head), three quarters of them f64 FMAs.
#include <type_traits>

#include "attn_args.h"

namespace bk {

constexpr int EX_SW = 8;                          // score waves of a workgroup; as many value waves
constexpr int EX_THREADS = 2 * EX_SW * 64;
constexpr int EX_TILE = 64;                       // tokens per tile = 4 pages
constexpr int EX_TILE_PAGES = EX_TILE / ATT_PAGE;
constexpr int EX_COLS = 8;                        // query heads per KV head served by one workgroup
constexpr int EX_KROW = ATT_HD * 2 + 16;          // bytes of a K row in LDS: 16 bytes of padding spread the rows over the banks
constexpr double EX_REF_SLACK = 600.0;            // exp() of up to this much above the reference exponent stays far from overflow

constexpr int EX_PROW = EX_COLS + 1;              // doubles per token row of the weights in LDS (padded against bank conflicts)

// A bf16 value widened to f64 has an all-zero low word, so the query copy holds the high words only.
__device__ __forceinline__ double f64_from_high(uint32_t hi) { return __builtin_bit_cast(double, (uint64_t)hi << 32); }
__device__ __forceinline__ uint32_t bf16_to_f64_high(uint16_t b) {
  return (uint32_t)(__builtin_bit_cast(uint64_t, (double)bf16_to_f32(b)) >> 32);
}

__device__ __forceinline__ double bf16lo_to_f64(uint32_t w) { return (double)__uint_as_float(w << 16); }
__device__ __forceinline__ double bf16hi_to_f64(uint32_t w) { return (double)__uint_as_float(w & 0xffff0000u); }

// acc[c] += bsrc(lane 8 * E + c of the lane's row of 16) * v for the 8 columns c: eight v_fmac_f64 whose first factor is
// read through the DPP row broadcast (the only DPP form of the f64 unit).  The compiler does not see a DPP instruction
// inside the asm block and inserts none of the idle cycles one needs: the two in front keep the distance from a vector
// instruction that may have written `bsrc` just before; the five a DPP read needs behind a vector instruction that
// writes the execution mask (v_cmpx) are not paid for, because the compiled kernel contains no such instruction —
// tests/test_isa_checks.py compiles this file and fails if one appears.
template <int E>
__device__ __forceinline__ void fmac8_bcast(double (&a)[EX_COLS], double bsrc, double v) {
  static_assert(E == 0 || E == 1, "half of the row");
  if (E == 0)
    asm("s_nop 1\n\t"
        "v_fmac_f64_dpp %0, %8, %9 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %1, %8, %9 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %2, %8, %9 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %3, %8, %9 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %4, %8, %9 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %5, %8, %9 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %6, %8, %9 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %7, %8, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf"
        : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
        : "v"(bsrc), "v"(v));
  else
    asm("s_nop 1\n\t"
        "v_fmac_f64_dpp %0, %8, %9 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %1, %8, %9 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %2, %8, %9 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %3, %8, %9 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %4, %8, %9 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %5, %8, %9 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %6, %8, %9 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %7, %8, %9 row_newbcast:15 row_mask:0xf bank_mask:0xf"
        : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
        : "v"(bsrc), "v"(v));
}

// One head's RMS norm and rotation, the arithmetic of attn_prep_kernel (attn.hip) to the bit: lane holds elements
// lane + 64 j.  `sh` is 256 bf16 of LDS that belong to the calling wave alone.
__device__ __forceinline__ void head_norm_rope(const uint16_t* xh, const uint16_t* w, const float* cos_t, const float* sin_t, int pos, int half,
                                               uint16_t* sh, uint16_t (&o)[ATT_HD / 64], int lane) {
  float xv[ATT_HD / 64];
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < ATT_HD / 64; j++) { xv[j] = bf16_to_f32(xh[lane + 64 * j]); ss += (double)(xv[j] * xv[j]); }
  ss = wave_sum_f64(ss);
  const float rstd = rsqrt_f64(ss / (double)ATT_HD + 1e-6);
#pragma unroll
  for (int j = 0; j < ATT_HD / 64; j++) {
    const int i = lane + 64 * j;
    sh[i] = f32_to_bf16(__fmul_rn(__fmul_rn(xv[j], rstd), __fadd_rn(1.0f, bf16_to_f32(w[i]))));
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int j = 0; j < ATT_HD / 64; j++) {
    const int i = lane + 64 * j;
    o[j] = sh[i];
    if (i < 2 * half) {
      const int i1 = i < half ? i : i - half;
      const float x1 = bf16_to_f32(sh[i1]), x2 = bf16_to_f32(sh[i1 + half]);
      const float c = cos_t[(int64_t)pos * half + i1], sn = sin_t[(int64_t)pos * half + i1];
      o[j] = i < half ? f32_to_bf16(__fsub_rn(__fmul_rn(x1, c), __fmul_rn(x2, sn)))
                      : f32_to_bf16(__fadd_rn(__fmul_rn(x2, c), __fmul_rn(x1, sn)));
    }
  }
}

// PREP: the step's preparation happens here instead of in a launch of its own (one new token per sequence, at
// position len - 1).  Every workgroup normalises and rotates its 8 query heads itself (score wave = head).  The
// workgroup whose pages hold the new position does the same for the key, stores key and value in the cache for the
// steps to come, and takes both from LDS / registers where its tiles reach that token, so nothing waits for memory
// that this launch itself writes.  A position outside the cache appends nothing, like attn_prep_kernel.
template <bool NT, bool PREP>
__global__ __launch_bounds__(EX_THREADS) void attn_exact_kernel(AttnArgs A) {
  // K tile (33792 bytes) and the exchange buffer of the partial scores (8 waves x 8 heads x 64 tokens x 8 = 32768 bytes);
  // the same memory carries the accumulator tree at the end (4 waves x 8 x 256 doubles = 65536 bytes)
  __shared__ __align__(16) unsigned char lds_raw[EX_TILE * EX_KROW + EX_SW * EX_COLS * EX_TILE * 8];
  __shared__ __align__(16) double lds_p[2][EX_TILE][EX_PROW];   // weights of a tile, [token][head]; even / odd tiles
  __shared__ double lds_alpha[2][EX_COLS], lds_m[EX_COLS], lds_l[EX_COLS];
  __shared__ int lds_rescale[2];                // set by a head that moved its reference exponent in an even / odd tile
  __shared__ int lds_bt[ATT_MAX_PPS];
  __shared__ __align__(16) uint16_t lds_knew[PREP ? ATT_HD : 8];   // the new token's key, normalised and rotated
  __shared__ uint16_t lds_vnew[PREP ? ATT_HD : 8];                 // and its value
  unsigned char* ktile = lds_raw;
  double (*xch)[EX_COLS][EX_TILE] = (double (*)[EX_COLS][EX_TILE])(lds_raw + EX_TILE * EX_KROW);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool value_role = wave >= EX_SW;                       // waves 0..7 score, waves 8..15 accumulate values
  const int w8 = wave & (EX_SW - 1);
  const int tid8 = threadIdx.x & (EX_SW * 64 - 1);             // thread index within the role
  int split, b, p_begin, p_end;
  if (!attn_wg_range(A, lane, b, split, p_begin, p_end)) return;
  const int row = __builtin_amdgcn_readfirstlane(b);          // one query row per workgroup (tpw = 1)
  const int kvh = blockIdx.y;
  const int len_raw = (A.ctx_len ? A.ctx_len[row] : A.ctx_scalar) + A.ctx_add;
  const int len = min(len_raw, A.max_ctx);                     // a length above the bound is read as the bound
  const int lim = min(len, p_end * ATT_PAGE);                  // tokens of this split end here
  const int npg = max(p_end - p_begin, 0);
  const int ntiles = (npg + EX_TILE_PAGES - 1) / EX_TILE_PAGES;

  for (int i = threadIdx.x; i < npg; i += EX_THREADS)
    lds_bt[i] = A.block_table ? A.block_table[(int64_t)row * A.bt_stride + p_begin + i] : row * A.bt_stride + p_begin + i;
  if (threadIdx.x < 2) lds_rescale[threadIdx.x] = 0;
  __syncthreads();

  // a page past the range (the last tile may be short) reads the last page again; its tokens are masked below
  auto page_base = [&](int i) -> int64_t { return ((int64_t)lds_bt[min(i, npg - 1)] * A.NKV + kvh) * (ATT_PAGE * ATT_HD); };
  auto ld16 = [&](const uint16_t* p) -> uint4 {
    const u32x4_nt* p4 = (const u32x4_nt*)p;
    const u32x4_nt t4 = NT ? __builtin_nontemporal_load(p4) : *p4;
    return make_uint4(t4[0], t4[1], t4[2], t4[3]);
  };

  // ---- preparation: q of this group into LDS (high words, [dim][head], in the exchange buffer, which the first tile
  // overwrites only behind the next barrier), the new key into lds_knew, key and value into the cache
  int new_tile = -1, new_row = 0;                 // tile and row within the tile of the new token, if this workgroup holds it
  if (PREP) {
    uint32_t* lds_q = (uint32_t*)xch;
    uint16_t* sh = (uint16_t*)(lds_q + ATT_HD * EX_COLS) + wave * ATT_HD;
    const int pos_raw = len_raw - 1;
    const int pos = min(max(pos_raw, 0), A.pmax_len - 1);
    const int ppage = pos / ATT_PAGE - p_begin, slot = pos % ATT_PAGE;
    const bool holds = pos == pos_raw && ppage >= 0 && ppage < npg;
    if (holds) {
      new_tile = __builtin_amdgcn_readfirstlane(ppage / EX_TILE_PAGES);
      new_row = __builtin_amdgcn_readfirstlane((ppage % EX_TILE_PAGES) * ATT_PAGE + slot);
    }
    if (!value_role) {
      uint16_t o[ATT_HD / 64];
      if (w8 < A.G)
        head_norm_rope(A.pq + ((int64_t)row * A.NH + kvh * A.G + w8) * 2 * ATT_HD, A.pqw, A.pcos, A.psin, pos, A.phalf, sh, o, lane);
#pragma unroll
      for (int j = 0; j < ATT_HD / 64; j++) lds_q[(lane + 64 * j) * EX_COLS + w8] = w8 < A.G ? bf16_to_f64_high(o[j]) : 0u;
    } else if (holds) {
      const int64_t base = ((int64_t)lds_bt[ppage] * A.NKV + kvh) * (ATT_PAGE * ATT_HD);
      if (w8 == 0) {
        uint16_t o[ATT_HD / 64];
        head_norm_rope(A.pk + ((int64_t)row * A.NKV + kvh) * ATT_HD, A.pkw, A.pcos, A.psin, pos, A.phalf, sh, o, lane);
#pragma unroll
        for (int j = 0; j < ATT_HD / 64; j++) {
          lds_knew[lane + 64 * j] = o[j];
          A.kcw[base + slot * ATT_HD + lane + 64 * j] = o[j];
        }
      } else if (w8 == 1) {
        const uint16_t* vp = A.pv + ((int64_t)row * A.NKV + kvh) * ATT_HD;
#pragma unroll
        for (int j = 0; j < ATT_HD / 64; j++) {
          const uint16_t x = vp[lane + 64 * j];
          lds_vnew[lane + 64 * j] = x;
          A.vcw[base + (lane + 64 * j) * ATT_PAGE + slot] = x;
        }
      }
    }
    __syncthreads();
  }

  // The two roles meet at three barriers per step.  In step s the score waves take tile s through [K rows -> LDS |
  // scores | weights]; the value waves add tile s - 1 (whose weights the third barrier of step s - 1 published) in three
  // pieces, one per interval, so that neither role waits long for the other and the vector unit always has work of
  // both kinds to choose from (4 waves per SIMD, 2 of each).
  if (!value_role) {
    // the wave's 32 dims x 8 heads of q: register pair g holds dims 2g, 2g + 1 (lane n of a row: dim 2g + n / 8, head n % 8)
    double qreg[16];
    if (PREP) {
      const uint32_t* qw = (const uint32_t*)xch + w8 * 32 * EX_COLS + (lane & 15);
#pragma unroll
      for (int g = 0; g < 16; g++) qreg[g] = f64_from_high(qw[g * 16]);
    } else {
      const uint32_t* qw = A.qf + (((int64_t)row * A.NKV + kvh) * ATT_HD + w8 * 32) * EX_COLS + (lane & 15);
#pragma unroll
      for (int g = 0; g < 16; g++) qreg[g] = f64_from_high(qw[g * 16]);
    }
    auto load_k = [&](int tile, uint4 (&kr)[EX_TILE_PAGES]) {      // round r of the 512 threads covers page r of the tile (8 KiB)
#pragma unroll
      for (int r = 0; r < EX_TILE_PAGES; r++) kr[r] = ld16(A.kc + page_base(tile * EX_TILE_PAGES + r) + tid8 * 8);
    };
    double l_lane = 0.0;            // wave = head: this lane's share of the sum of weights
    double mref = -INFINITY;        // wave = head: the reference exponent
    uint4 kpre[EX_TILE_PAGES];      // K of the next tile, requested a whole step ahead
    if (ntiles > 0) load_k(0, kpre);
    for (int tile = 0; tile <= ntiles && ntiles > 0; tile++) {      // (an empty page range: neither role enters its loop)
      const bool live = tile < ntiles;                             // the last step only drains the value waves
      if (live) {
#pragma unroll
        for (int r = 0; r < EX_TILE_PAGES; r++) {
          const int krow_i = r * ATT_PAGE + (tid8 >> 5);
          uint4 kv = kpre[r];
          // the new token's row comes from LDS: what memory returned for it may be older than this launch's store
          if (PREP && tile == new_tile && krow_i == new_row) kv = *(const uint4*)(lds_knew + (tid8 & 31) * 8);
          *(uint4*)(ktile + krow_i * EX_KROW + (tid8 & 31) * 16) = kv;
        }
      }
      __syncthreads();
      if (live) {
        load_k(min(tile + 1, ntiles - 1), kpre);         // unconditional (the last tile again), so that the waits stay countable
        // ---- scores: lane = token, this wave's 32 dims
        double sacc[EX_COLS];
#pragma unroll
        for (int c = 0; c < EX_COLS; c++) sacc[c] = 0.0;
        const uint4* krow = (const uint4*)(ktile + lane * EX_KROW + w8 * 64);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const uint4 kk = krow[i];
          const uint32_t w[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
          for (int wi = 0; wi < 4; wi++) {
            fmac8_bcast<0>(sacc, qreg[i * 4 + wi], bf16lo_to_f64(w[wi]));
            fmac8_bcast<1>(sacc, qreg[i * 4 + wi], bf16hi_to_f64(w[wi]));
          }
        }
#pragma unroll
        for (int c = 0; c < EX_COLS; c++) xch[w8][c][lane] = sacc[c];
      }
      __syncthreads();
      if (live) {
        // ---- weights: wave = head
        double s = 0.0;
#pragma unroll
        for (int w2 = 0; w2 < EX_SW; w2++) s += xch[w2][w8][lane];
        s *= (double)A.scale;
        const int tok = (p_begin + tile * EX_TILE_PAGES) * ATT_PAGE + lane;
        const bool valid = tok < lim;
        const float smax = wave_max(valid ? (float)s : -INFINITY);
        double alpha = 1.0;
        if (smax > -INFINITY && (mref == -INFINITY || (double)smax > mref + EX_REF_SLACK)) {      // wave-uniform, rare after the first tile
          if (mref != -INFINITY) { alpha = exp(mref - (double)smax); l_lane *= alpha; }
          mref = (double)smax;
        }
        const double p = valid ? exp(s - mref) : 0.0;
        l_lane += p;
        lds_p[tile & 1][lane][w8] = p;
        if (lane == 0) {
          lds_alpha[tile & 1][w8] = alpha;
          if (alpha != 1.0) lds_rescale[tile & 1] = 1;
        }
      }
      __syncthreads();
    }
    const double lt = wave_sum_f64(l_lane);
    if (lane == 0) { lds_l[w8] = lt; lds_m[w8] = mref; }
  }

  double acc[EX_COLS][4];
#pragma unroll
  for (int c = 0; c < EX_COLS; c++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[c][j] = 0.0;
  if (value_role) {
    // wave: tokens 8 * w8 .. + 8 of a tile; lane: dims lane + 64 j.  vreg[j] holds the 8 tokens of dim lane + 64 j and is
    // requested again, for the next tile, as soon as the piece that uses it is done: every load has a step to arrive
    uint4 vreg[4];
    auto load_v = [&](int tile, int j) {
      const int64_t base = page_base(tile * EX_TILE_PAGES + (w8 >> 1)) + (w8 & 1) * 8;
      vreg[j] = ld16(A.vc + base + (lane + 64 * j) * ATT_PAGE);
    };
    if (ntiles > 0) {
#pragma unroll
      for (int j = 0; j < 4; j++) load_v(0, j);
    }
    double preg[4];
    for (int step = 0; step <= ntiles && ntiles > 0; step++) {
      const int t = step - 1;                                      // the tile whose values are added in this step
      const bool live = t >= 0;
      const int tok0 = (p_begin + t * EX_TILE_PAGES) * ATT_PAGE + w8 * 8;
      const bool tail = tok0 + 8 > lim;
      // one dim-group j of the tile: 8 tokens x 8 heads; a token past the context has weight 0, but what its cache slot
      // holds need not be a number: it enters as 0 (only the tile that holds the end of the context pays for the test)
      auto piece = [&](int j, auto tail_c) {
        constexpr bool TAIL = decltype(tail_c)::value;
        const uint32_t vw[4] = {vreg[j].x, vreg[j].y, vreg[j].z, vreg[j].w};
        double a[EX_COLS];
#pragma unroll
        for (int c = 0; c < EX_COLS; c++) a[c] = acc[c][j];
#pragma unroll
        for (int h = 0; h < 4; h++) {
          const bool in0 = !TAIL || tok0 + 2 * h < lim, in1 = !TAIL || tok0 + 2 * h + 1 < lim;
          fmac8_bcast<0>(a, preg[h], in0 ? bf16lo_to_f64(vw[h]) : 0.0);
          fmac8_bcast<1>(a, preg[h], in1 ? bf16hi_to_f64(vw[h]) : 0.0);
        }
#pragma unroll
        for (int c = 0; c < EX_COLS; c++) acc[c][j] = a[c];
      };
      // the piece's arithmetic, then the request for the same dims of the next tile (issued in every step, for the last
      // tile again behind the end: a load behind a branch would leave the number of loads in flight unknown at the waits)
      auto pieces = [&](int j) {
        if (live) {
          if (tail) piece(j, std::true_type{});
          else piece(j, std::false_type{});
        }
        load_v(min(t + 1, ntiles - 1), j);
      };
      if (PREP && live && t == new_tile && w8 == (new_row >> 3)) {
        // the new token's value, from LDS (see the key above): element new_row % 8 of each of the four loads
        const int e = new_row & 7;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const uint32_t vn = lds_vnew[lane + 64 * j];
          uint32_t vw[4] = {vreg[j].x, vreg[j].y, vreg[j].z, vreg[j].w};
#pragma unroll
          for (int h = 0; h < 4; h++)
            if ((e >> 1) == h) vw[h] = (e & 1) ? (vw[h] & 0x0000ffffu) | (vn << 16) : (vw[h] & 0xffff0000u) | vn;
          vreg[j] = make_uint4(vw[0], vw[1], vw[2], vw[3]);
        }
      }
      if (live) {
        // a head whose reference exponent moved in this tile (first tile aside: rare) rescales what was summed under the old one
        if (__builtin_amdgcn_readfirstlane(lds_rescale[t & 1])) {
#pragma unroll
          for (int c = 0; c < EX_COLS; c++) {
            const double al = lds_alpha[t & 1][c];
#pragma unroll
            for (int j = 0; j < 4; j++) acc[c][j] *= al;
          }
        }
        // the weights of this wave's 8 tokens: pair h holds tokens 2h, 2h + 1 (lane n of a row: token 2h + n / 8, head n % 8)
#pragma unroll
        for (int h = 0; h < 4; h++) preg[h] = lds_p[t & 1][w8 * 8 + 2 * h + ((lane & 15) >> 3)][lane & 7];
      }
      pieces(0);
      __syncthreads();
      // the flag of tile t has been read by every value wave; tile t + 2 sets it again two steps from now
      if (live && w8 == 0 && lane == 0) lds_rescale[t & 1] = 0;
      pieces(1);
      pieces(2);
      __syncthreads();
      pieces(3);
      __syncthreads();
    }
  }

  // ---- the accumulators of the 8 value waves as ((0+4)+(2+6)) + ((1+5)+(3+7)); every wave of the workgroup walks the barriers
  __syncthreads();
  double* red = (double*)lds_raw;
  auto put = [&](int slot) {
#pragma unroll
    for (int c = 0; c < EX_COLS; c++)
#pragma unroll
      for (int j = 0; j < 4; j++) red[((slot * EX_COLS + c) * 4 + j) * 64 + lane] = acc[c][j];
  };
  auto get = [&](int slot) {
#pragma unroll
    for (int c = 0; c < EX_COLS; c++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[c][j] += red[((slot * EX_COLS + c) * 4 + j) * 64 + lane];
  };
  // a wave puts into the slot it alone read in the round before, so one barrier per round is enough
  if (value_role && w8 >= 4) put(w8 - 4);
  __syncthreads();
  if (value_role && w8 < 4) get(w8);
  if (value_role && (w8 == 2 || w8 == 3)) put(w8);
  __syncthreads();
  if (value_role && w8 < 2) get(w8 + 2);
  if (value_role && w8 == 1) put(1);
  __syncthreads();
  if (!value_role || w8 != 0) return;
  get(1);

  if (A.splits == 1) {
#pragma unroll
    for (int c = 0; c < EX_COLS; c++) {
      if (c >= A.G) break;
      const int head = kvh * A.G + c;
      const double L = lds_l[c], M = lds_m[c];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int d = lane + 64 * j;
        // a sequence without context (length <= 0 found in device memory) has no weights: zeros and lse = -inf
        float o = L > 0.0 ? (float)(acc[c][j] / L) : 0.0f;
        if (A.gate) {
          const float gv = bf16_to_f32(A.gate[(int64_t)row * A.gate_bstride + (int64_t)head * A.gate_hstride + d]);
          o = __fmul_rn(o, sigmoid_f64(gv));
        }
        A.out[((int64_t)row * A.NH + head) * ATT_HD + d] = f32_to_bf16(o);
      }
      if (lane == 0 && A.lse) A.lse[(int64_t)row * A.NH + head] = L > 0.0 ? (float)(M + log(L)) : -INFINITY;
    }
  } else {
    const int64_t pidx = A.slots > 0 ? (int64_t)kvh * A.slots + blockIdx.x : ((int64_t)row * A.NKV + kvh) * A.splits + split;
    double* po = A.part_o64 + pidx * EX_COLS * ATT_HD;
#pragma unroll
    for (int c = 0; c < EX_COLS; c++)
#pragma unroll
      for (int j = 0; j < 4; j++) po[c * ATT_HD + lane + 64 * j] = acc[c][j];
    if (lane < EX_COLS) {
      A.part_ml64[(pidx * EX_COLS + lane) * 2] = lds_m[lane];
      A.part_ml64[(pidx * EX_COLS + lane) * 2 + 1] = lds_l[lane];
    }
  }
}

// Merge of the f64 split partials: one workgroup per (head, query row), thread = dim.  The weights exp(ref_s - max ref)
// of all splits are computed side by side first (thread = split), the partial outputs are then added in split order.
// Its argument block holds only what the merge reads (92 bytes: two 64-byte lines of kernel arguments, AttnArgs has five).
struct AttnMergeArgs {
  const double* part_o64;
  const double* part_ml64;
  const int2* plan;
  const uint16_t* gate;
  uint16_t* out;
  uint8_t* out_q8;
  float* lse;
  int64_t gate_bstride, gate_hstride;
  int NH, NKV, G, splits, slots;
};
template <int PRE>
__global__ __launch_bounds__(256) void attn_exact_merge_kernel(AttnMergeArgs A) {
  __shared__ double wsh[ATT_MAX_SPLITS];
  __shared__ float redm[4];
  __shared__ double redl[4];
  const int head = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const int kvh = head / A.G, c = head % A.G;
  int64_t p0 = ((int64_t)b * A.NKV + kvh) * A.splits;
  int nsplit = A.splits;
  if (A.slots > 0) {
    const int2 pl = A.plan[b];
    nsplit = pl.y;
    p0 = (int64_t)kvh * A.slots + pl.x;
  }
  const bool has = d < nsplit;
  const double ms = has ? A.part_ml64[((p0 + d) * EX_COLS + c) * 2] : -INFINITY;
  const double ls = has ? A.part_ml64[((p0 + d) * EX_COLS + c) * 2 + 1] : 0.0;
  const uint16_t gbits = A.gate ? A.gate[(int64_t)b * A.gate_bstride + (int64_t)head * A.gate_hstride + d] : (uint16_t)0;
  // The partial outputs of the first PRE splits (4, 16 or 64, by the split count of the launch) are requested right behind the exponents, all at once and
  // unconditionally (a split past the last one reads the last one again and gets weight 0): they travel while the
  // weights are worked out, and the kernel waits for memory once instead of once per pair of splits.
  const double* po = A.part_o64 + (p0 * EX_COLS + c) * ATT_HD + d;
  double pv[PRE];
#pragma unroll
  for (int s = 0; s < PRE; s++) pv[s] = po[(int64_t)min(s, nsplit - 1) * EX_COLS * ATT_HD];
  // the reference exponents are f32 values (or -inf), so their maximum is found in f32 without loss
  float Mf = wave_max((float)ms);
  if ((d & 63) == 0) redm[d >> 6] = Mf;
  __syncthreads();
  const double M = (double)fmaxf(fmaxf(redm[0], redm[1]), fmaxf(redm[2], redm[3]));
  const double w = (ms == -INFINITY) ? 0.0 : exp(ms - M);
  wsh[d] = w;
  double L = wave_sum_f64(ls * w);
  if ((d & 63) == 0) redl[d >> 6] = L;
  __syncthreads();
  L = (redl[0] + redl[1]) + (redl[2] + redl[3]);
  const float gsig = A.gate ? sigmoid_f64(bf16_to_f32(gbits)) : 1.0f;
  double o0 = 0.0, o1 = 0.0;
#pragma unroll
  for (int s = 0; s < PRE; s += 2) {
    o0 = fma(pv[s], wsh[s], o0);              // wsh[s] = 0 for s >= nsplit
    o1 = fma(pv[s + 1], wsh[s + 1], o1);
  }
  int s = PRE;
  for (; s + 2 <= nsplit; s += 2) {
    o0 = fma(po[(int64_t)(s + 0) * EX_COLS * ATT_HD], wsh[s + 0], o0);
    o1 = fma(po[(int64_t)(s + 1) * EX_COLS * ATT_HD], wsh[s + 1], o1);
  }
  if (s < nsplit) o0 = fma(po[(int64_t)s * EX_COLS * ATT_HD], wsh[s], o0);
  float o = L > 0.0 ? (float)((o0 + o1) / L) : 0.0f;          // no context at all: zeros, lse = -inf
  if (A.gate) o = __fmul_rn(o, gsig);
  const uint16_t ob = f32_to_bf16(o);
  A.out[((int64_t)b * A.NH + head) * ATT_HD + d] = ob;
  if (A.out_q8) lane32_q8_1_store(bf16_to_f32(ob), A.out_q8 + (((int64_t)b * A.NH + head) * (ATT_HD / 32) + (d >> 5)) * 36, d & 31);
  if (d == 0 && A.lse) A.lse[(int64_t)b * A.NH + head] = L > 0.0 ? (float)(M + log(L)) : -INFINITY;
}

// q bf16 [rows, NH, 256] -> high words of the f64 values [rows, NKV, 256, 8]: column c < G of (row, kv head) is head
// kvh * G + c, the rest zeros
__global__ __launch_bounds__(256) void attn_q_to_f64_kernel(const uint16_t* __restrict__ q, uint32_t* __restrict__ qf, int NH, int NKV, int G) {
  const int kvh = blockIdx.x, row = blockIdx.y, d = threadIdx.x;
  uint32_t* o = qf + (((int64_t)row * NKV + kvh) * ATT_HD + d) * EX_COLS;
#pragma unroll
  for (int c = 0; c < EX_COLS; c++)
    o[c] = c < G ? bf16_to_f64_high(q[((int64_t)row * NH + kvh * G + c) * ATT_HD + d]) : 0u;
}

size_t attn_exact_qf_bytes(int rows, int NKV) { return (size_t)rows * NKV * ATT_HD * EX_COLS * sizeof(uint32_t); }
size_t attn_exact_workspace_bytes(int rows, int NKV, int max_splits) {
  return (size_t)rows * NKV * max_splits * EX_COLS * (ATT_HD + 2) * sizeof(double) + 64 * sizeof(int2) + attn_exact_qf_bytes(rows, NKV);
}

// Called by launch_attn_decode with the split plan already in A (same planning as the matrix-instruction form).
// workspace: partial outputs, partial (ref, sum), plan, then the f64 copy of q unless the caller has one (qf_ready).
int launch_attn_exact(AttnArgs A, const void* q, const uint32_t* qf_ready, void* workspace, size_t workspace_bytes, bool nt, dim3 grid,
                      int batch) {
  BK_REQUIRE(A.tpw == 1, "attn_decode (exact): one query row per workgroup");
  BK_REQUIRE(A.G <= EX_COLS, "attn_decode (exact): at most %d query heads per KV head (got %d)", EX_COLS, A.G);
  const size_t npart = A.splits > 1 ? (size_t)batch * A.NKV * A.splits : 0;
  const size_t need = npart * EX_COLS * (ATT_HD + 2) * sizeof(double) + 64 * sizeof(int2) + (qf_ready || A.pq ? 0 : attn_exact_qf_bytes(batch, A.NKV));
  BK_REQUIRE(workspace && workspace_bytes >= need, "attn_decode (exact): workspace of %zu bytes needed for %d splits (got %zu)", need, A.splits,
             workspace_bytes);
  A.part_o64 = (double*)workspace;
  A.part_ml64 = A.part_o64 + npart * EX_COLS * ATT_HD;
  A.plan = (int2*)(A.part_ml64 + npart * EX_COLS * 2);
  if (A.pq) {
    A.qf = nullptr;                            // the kernel makes its own query copy, in LDS
  } else if (qf_ready) {
    A.qf = qf_ready;
  } else {
    uint32_t* qf = (uint32_t*)(A.plan + 64);
    hipLaunchKernelGGL(attn_q_to_f64_kernel, dim3(A.NKV, batch), dim3(256), 0, stream(), (const uint16_t*)q, qf, A.NH, A.NKV, A.G);
    A.qf = qf;
  }
  BK_REQUIRE(((uintptr_t)A.qf & 63) == 0, "attn_decode (exact): the f64 query copy must be 64-byte aligned");
  const dim3 block(EX_THREADS);
  if (A.pq) {
    if (nt) hipLaunchKernelGGL((attn_exact_kernel<true, true>), grid, block, 0, stream(), A);
    else hipLaunchKernelGGL((attn_exact_kernel<false, true>), grid, block, 0, stream(), A);
  } else {
    if (nt) hipLaunchKernelGGL((attn_exact_kernel<true, false>), grid, block, 0, stream(), A);
    else hipLaunchKernelGGL((attn_exact_kernel<false, false>), grid, block, 0, stream(), A);
  }
  if (A.splits > 1) {
    const dim3 mgrid(A.NH, batch);
    const AttnMergeArgs M{A.part_o64, A.part_ml64, A.plan, A.gate, A.out, A.out_q8, A.lse, A.gate_bstride, A.gate_hstride,
                          A.NH, A.NKV, A.G, A.splits, A.slots};
    if (A.splits <= 4) hipLaunchKernelGGL(attn_exact_merge_kernel<4>, mgrid, dim3(256), 0, stream(), M);
    else if (A.splits <= 16) hipLaunchKernelGGL(attn_exact_merge_kernel<16>, mgrid, dim3(256), 0, stream(), M);
    else hipLaunchKernelGGL(attn_exact_merge_kernel<64>, mgrid, dim3(256), 0, stream(), M);
  }
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
