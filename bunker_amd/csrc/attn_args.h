// Shared by the two decode-attention kernels (attn.hip: bf16 matrix instructions; attn_exact.hip: double precision):
// cache geometry, the argument block, and the cut of a sequence's pages into per-workgroup ranges.
#pragma once
#include "ops.h"

namespace bk {

constexpr int ATT_HD = 256;
constexpr int ATT_PAGE = 16;
constexpr int ATT_WAVES = 4;
constexpr int ATT_MAX_PPS = 1024;     // pages per split (the split's page table is staged in LDS)
constexpr int ATT_MAX_SPLITS = 256;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_nt;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_nt;

struct AttnArgs {
  const uint16_t* q;          // bf16 [B, NH, 256]
  const uint16_t* kc;         // K pages
  const uint16_t* vc;         // V pages (dim-major inside a page)
  const int32_t* block_table; // int32 [B, bt_stride]; null = identity (page i of sequence b is b*bt_stride + i)
  const int32_t* ctx_len;     // int32 [B]; null = ctx_scalar for every sequence; ctx_add is added to either
  const uint16_t* gate;       // bf16 or null: gate of (b, head, i) at gate[b*gate_bstride + head*gate_hstride + i]
  uint16_t* out;              // bf16 [B, NH, 256]
  uint8_t* out_q8;            // optional: the same outputs as Q8_1 blocks [B, NH*256/32] (written by the merge kernel)
  float* lse;                 // f32 [B, NH] or null
  float* part_o;              // f32 [B, NKV, splits, 16, 256] unnormalised partial outputs
  float* part_ml;             // f32 [B, NKV, splits, 16, 2] (max, sum)
  int2* plan;                 // balanced form: (first slot, number of splits) of every sequence, behind the partials
  // double-precision form (attn_exact.hip): q widened to f64 [rows, NKV, 256, 8 columns], partials in f64
  const uint32_t* qf;          // column c of (row, kv head) is query head kvh * G + c (c < G <= 8; the other columns hold zeros)
  double* part_o64;           // f64 [partials, 8, 256] unnormalised partial outputs
  double* part_ml64;          // f64 [partials, 8, 2] (reference exponent, sum)
  int64_t gate_bstride, gate_hstride;
  int bt_stride, ctx_scalar, ctx_add, NH, NKV, G, splits, pages_per_split;
  int tpw, rows;              // query rows per workgroup (1, or 2 consecutive rows of one sequence: prompt tokens), rows in all
  int max_pages;              // pages of the longest context the caller allows
  int max_ctx;                // that context in tokens: a length above it is read as max_ctx (also inside the last page)
  int rel;                    // 1: lengths in device memory, every sequence cuts its own pages into `splits` equal ranges
  int slots;                  // > 0: balanced form, this many workgroup slots per KV head shared by the rows (rows <= 64)
  float scale;
  // Double-precision form with the step's preparation folded in (decode only: one new token per sequence): the query
  // heads are normalised and rotated by every workgroup for itself, and the workgroup whose pages hold the new position
  // normalises and rotates the key, appends key and value to the cache and uses them from registers / LDS.
  const uint16_t *pq, *pk, *pv;      // q|gate bf16 [B, NH, 2*256]; k, v bf16 [B, NKV, 256]; pq == null: no preparation
  const uint16_t *pqw, *pkw;         // norm weights bf16 [256]
  const float *pcos, *psin;          // f32 [max_len, half]
  uint16_t *kcw, *vcw;               // the caches, writable
  int phalf, pmax_len;
};


__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
}

// ceil(a / b) for 0 <= a < 2^24, b >= 1, inv_b ~ 1 / b: the float quotient is off by less than one, the remainder settles it
__device__ __forceinline__ int ceil_div_rcp(int a, int b, float inv_b) {
  int q = (int)((float)a * inv_b);
  int r = a - q * b;
  if (r < 0) { q -= 1; r += b; }
  if (r >= b) { q += 1; r -= b; }
  return q + (r > 0 ? 1 : 0);
}

// Balanced plan, computed by every wave for itself: lane i < rows holds sequence i's pages `np`, its number of splits
// `ns` and the first slot `first` of its splits.  The page budget of a slot is ceil(total / slots); when the round-up
// of the sequences' split counts does not fit the slots, it is taken for rows - 1 slots fewer, which always fits
// (sum ceil(np_i / t) <= total / t + rows - rows / t).  Sums and the prefix sum stay in the lanes (DPP), no LDS.
__device__ __forceinline__ void attn_balanced_plan(const AttnArgs& A, int lane, int& np, int& ns, int& first) {
  // a length outside 1 .. max_ctx (the caller's mistake) still plans inside the block table and the slots
  np = lane < A.rows ? min(max((A.ctx_len[lane] + A.ctx_add + ATT_PAGE - 1) / ATT_PAGE, 1), A.max_pages) : 0;
  const int t16 = row16_sum_i32(np);
  const int total = (__builtin_amdgcn_readlane(t16, 0) + __builtin_amdgcn_readlane(t16, 16)) +
                    (__builtin_amdgcn_readlane(t16, 32) + __builtin_amdgcn_readlane(t16, 48));
  int incl = 0;
  for (int attempt = 0; attempt < 2; attempt++) {
    const int over = attempt ? A.slots - (A.rows - 1) : A.slots;
    const int budget = ceil_div_rcp(total, over, __builtin_amdgcn_rcpf((float)over));
    ns = ceil_div_rcp(np, budget, __builtin_amdgcn_rcpf((float)budget));
    // inclusive prefix sum: inside each row of 16 lanes by row shifts (lanes without a source read 0), then the rows before
    int v = ns;
    v += dpp_i32<0x111>(v);      // row_shr:1
    v += dpp_i32<0x112>(v);      // row_shr:2
    v += dpp_i32<0x114>(v);      // row_shr:4
    v += dpp_i32<0x118>(v);      // row_shr:8
    const int r0 = __builtin_amdgcn_readlane(v, 15), r1 = __builtin_amdgcn_readlane(v, 31), r2 = __builtin_amdgcn_readlane(v, 47);
    const int row = lane >> 4;
    incl = v + (row == 0 ? 0 : row == 1 ? r0 : row == 2 ? r0 + r1 : r0 + r1 + r2);
    const int used = r0 + r1 + r2 + __builtin_amdgcn_readlane(v, 63);
    if (used <= A.slots) break;
  }
  first = incl - ns;
}

// The page range [p_begin, p_end) of this workgroup's split and the sequence (query row group) it belongs to, for the
// three forms of the cut (plain: equal ranges of the host's bound; relative: of the length found in device memory;
// balanced: slots shared out by length).  Returns false for a slot of the balanced form that no sequence uses (the
// whole workgroup leaves).  `len_max` is the longest context among the workgroup's query rows.
__device__ __forceinline__ bool attn_wg_range(const AttnArgs& A, int lane, int& b, int& split, int& p_begin, int& p_end) {
  split = blockIdx.x; b = blockIdx.z;
  int pps = A.pages_per_split;
  if (A.slots > 0) {                            // balanced form: slot blockIdx.x belongs to the sequence whose range holds it
    int np, ns, first;
    attn_balanced_plan(A, lane, np, ns, first);
    const unsigned long long own = __ballot((int)blockIdx.x >= first && (int)blockIdx.x < first + ns);
    if (own == 0) return false;                 // a slot past the last one in use
    b = __ffsll(own) - 1;
    split = blockIdx.x - __builtin_amdgcn_readlane(first, b);
    const int nsb = __builtin_amdgcn_readlane(ns, b);
    pps = ceil_div_rcp(__builtin_amdgcn_readlane(np, b), nsb, __builtin_amdgcn_rcpf((float)nsb));
    // the merge kernel finds the sequence's partials through this pair
    if (split == 0 && blockIdx.y == 0 && threadIdx.x == 0) A.plan[b] = make_int2(blockIdx.x, nsb);
  }
  const int row0 = b * A.tpw;
  const int ntk = min(A.tpw, A.rows - row0);
  int len_max = (A.ctx_len ? A.ctx_len[row0] : A.ctx_scalar) + A.ctx_add;
  if (ntk > 1) len_max = max(len_max, A.ctx_len[row0 + 1] + A.ctx_add);
  const int npages = min((len_max + ATT_PAGE - 1) / ATT_PAGE, A.max_pages);
  if (A.rel) pps = ceil_div_rcp(npages, A.splits, __builtin_amdgcn_rcpf((float)A.splits));   // equal parts of its own context
  p_begin = split * pps;
  p_end = min(npages, p_begin + pps);
  return true;
}

// attn_exact.hip, called by launch_attn_decode with the cut of the pages already in A
int launch_attn_exact(AttnArgs A, const void* q, const uint32_t* qf_ready, void* workspace, size_t workspace_bytes, bool nt, dim3 grid, int batch);

}  // namespace bk
