// Split-K decode attention over a paged bf16 GQA KV cache (one query token per
// sequence).  Math of src/emitters.ts:188-226 (scores * 1/sqrt(HD) over the valid
// prefix, softmax, sum p*V, optional * sigmoid(gate)) with the log-sum-exp returned,
// on a cache that is shared by the query heads of a KV group and cut into 16-token
// pages.
//
// Cache layout (per layer; one array for K, one for V; HD = 256, page = 16 tokens):
//   K page p, kv head h:  bf16 [16 tok][256 dim]   at ((p*NKV + h) * 4096) elements
//   V page p, kv head h:  bf16 [256 dim][16 tok]   at ((p*NKV + h) * 4096) elements
// V is stored dim-major inside the page so that both matrix products read their
// MFMA operands straight from global memory with contiguous 16/8-byte pieces:
//   S^T[tok, head] = sum_d K[tok, d] * Q[head, d]        v_mfma_f32_16x16x32_bf16, A = K page
//   O^T[d, head]   = sum_tok V^T[d, tok] * P^T[tok, head] v_mfma_f32_16x16x16_bf16, A = V page,
// and P^T comes out of the first product in exactly the register layout the second
// wants as its B operand (fed as two bf16 terms, hi + lo, so that P carries 16 bits).
// The query heads of a KV group (<= 16) are the N dimension; when a prompt is processed and the group has at most 8 heads,
// two consecutive tokens of the sequence share a workgroup (columns 0..G-1 and G..2G-1, each masked to its own length),
// so a K/V page is read once for both.
//
// grid = (splits, NKV, B), 4 waves per workgroup.  Each wave walks pages of its
// split with its own running (max, sum, O^T); the four are merged through LDS in a
// fixed order; with more than one split the workgroup partials go to a workspace
// and a second kernel merges them, again in a fixed order.
//
// Lengths that live in device memory (a captured decode step, a ragged batch): the host cannot size the splits, and
// cutting every sequence into equal page ranges of the LONGEST context the cache allows leaves the workgroups behind a
// short context without work.  Two forms, chosen on the host from the bound alone:
//  - relative: every workgroup divides its own sequence's pages by the number of splits (one division after the length
//    has arrived); all workgroups of a sequence work, long sequences take longer than short ones;
//  - balanced (large shares, where the page loop and not the start-up decides the time): the batch's workgroup slots
//    (B * splits, grid = (slots, NKV)) are handed out in proportion to the lengths.  Every workgroup derives the plan
//    from the B lengths itself (sums and a prefix sum in the lanes, no extra launch) and takes at most
//    ceil(total pages / slots) pages, up to a rounding allowance; the first workgroup of a sequence leaves (first slot,
//    splits) for the merge kernel.
// With every length at the bound both give the page ranges of the plain form and the same bits.
#include "attn_args.h"

namespace bk {

// PF = pages a wave requests ahead of the one it computes on (0 or 2).  Loads are issued
// unconditionally (past its last page a wave requests a few fixed, cached lines instead), so the number of loads in
// flight at every wait is known when the kernel is compiled and a wait covers only the page needed.
template <int PF, bool NT>
__global__ __launch_bounds__(ATT_WAVES * 64) void attn_decode_kernel(AttnArgs A) {
  __shared__ float lds_o2[2][ATT_HD][16];       // exchange buffers for the merge of the four waves, 2 x 16 KiB
  __shared__ float lds_m[ATT_WAVES][16], lds_l[ATT_WAVES][16];
  __shared__ int lds_bt[ATT_MAX_PPS];           // physical page of every page of this split

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int split, b, p_begin, p_end;                 // b: workgroup's first query row is b * tpw
  if (!attn_wg_range(A, lane, b, split, p_begin, p_end)) return;
  const int kvh = blockIdx.y;
  const int n = lane & 15, kg = lane >> 4;      // n: token (A operand) / head (B operand, C column); kg: lane group
  // column n of the products: head n % G of query row b * tpw + n / G; a row past the last one repeats the first (not stored)
  const int row0 = b * A.tpw;
  const int ntk = min(A.tpw, A.rows - row0);    // query rows of this workgroup
  const int tk_n = n / A.G;
  const bool col_valid = tk_n < ntk;
  const int row_n = row0 + (col_valid ? tk_n : 0);
  const int len = min((A.ctx_len ? A.ctx_len[row_n] : A.ctx_scalar) + A.ctx_add, A.max_ctx);       // of this lane's column
  int len_wg = len;                             // the longest column: what the cache holds behind it need not be a number
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) len_wg = max(len_wg, __shfl_xor(len_wg, off));

  // Q as the B operand of the first product: lane (column n, group kg) holds dims 32*s + 8*kg .. +8
  uint4 qreg[8];
  {
    const bool valid = col_valid;
    const uint16_t* qp = A.q + ((int64_t)row_n * A.NH + kvh * A.G + (valid ? n % A.G : 0)) * ATT_HD + 8 * kg;
#pragma unroll
    for (int s = 0; s < 8; s++) qreg[s] = valid ? *(const uint4*)(qp + 32 * s) : make_uint4(0, 0, 0, 0);
  }

  f32x4_t oacc[16];
#pragma unroll
  for (int t = 0; t < 16; t++) oacc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;     // running max of head n (same in the 4 lanes that share n)
  float l_run = 0.0f;          // this lane's share of the running sum (tokens 4*kg .. 4*kg+3 of every page)

  // The page table of the split is read once, into LDS: a table lookup in front of every page would
  // put a dependent global load (and a wait for everything in flight) between the page requests.
  for (int i = threadIdx.x; i < p_end - p_begin; i += ATT_WAVES * 64)
    lds_bt[i] = A.block_table ? A.block_table[(int64_t)row0 * A.bt_stride + p_begin + i] : row0 * A.bt_stride + p_begin + i;
  __syncthreads();
  // A request past the wave's last page (issued only to keep the number of loads in flight fixed; its registers are
  // never computed on) goes to the first bytes of the cache with every lane on the same address: a handful of cache
  // lines instead of a second and third trip of the last page through memory, which nontemporal loads would make.
  auto load_page = [&](int pg, int last_pg, uint4 (&kr)[8], uint2 (&vr)[16]) {
    const bool real = pg <= last_pg;
    const int phys = lds_bt[min(pg, last_pg) - p_begin];
    const int64_t base = real ? ((int64_t)phys * A.NKV + kvh) * (ATT_PAGE * ATT_HD) : 0;
    // K page as the A operand: lane (token n, group kg) holds dims 32*s + 8*kg .. +8
    const uint16_t* kp = A.kc + base + (real ? n * ATT_HD + 8 * kg : 0);
#pragma unroll
    for (int s = 0; s < 8; s++) {
      const u32x4_nt* p4 = (const u32x4_nt*)(kp + 32 * s);
      const u32x4_nt t4 = NT ? __builtin_nontemporal_load(p4) : *p4;
      kr[s] = make_uint4(t4[0], t4[1], t4[2], t4[3]);
    }
    // V page as the A operand: lane (dim 16*t + n, group kg) holds tokens 4*kg .. +4
    const uint16_t* vp = A.vc + base + (real ? n * ATT_PAGE + 4 * kg : 0);
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const u32x2_nt* p2 = (const u32x2_nt*)(vp + t * 16 * ATT_PAGE);
      const u32x2_nt t2 = NT ? __builtin_nontemporal_load(p2) : *p2;
      vr[t] = make_uint2(t2[0], t2[1]);
    }
  };
  auto compute_page = [&](const uint4 (&kreg)[8], const uint2 (&vreg)[16], int pg) {
    f32x4_t s4 = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; s++)
      s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kreg[s]), __builtin_bit_cast(bf16x8_t, qreg[s]),
                                                   s4, 0, 0, 0);
    // lane holds S^T[token 4*kg + r][head n], r = 0..3
    float sc[4];
    const int tok0 = pg * ATT_PAGE + 4 * kg;
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      sc[r] = (tok0 + r < len) ? s4[r] * A.scale : -INFINITY;
      tmax = fmaxf(tmax, sc[r]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);
    // a column whose own length ends before this page (the shorter of two rows) has seen nothing yet: keep exp() off inf - inf
    const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;
    const float alpha = __expf(m_run - m_ref);     // exp(-inf) = 0 on the first page
    float p[4], psum = 0.0f;
#pragma unroll
    for (int r = 0; r < 4; r++) { p[r] = __expf(sc[r] - m_ref); psum += p[r]; }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (alpha != 1.0f) {
#pragma unroll
      for (int t = 0; t < 16; t++) { oacc[t][0] *= alpha; oacc[t][1] *= alpha; oacc[t][2] *= alpha; oacc[t][3] *= alpha; }
    }
    // P goes in as hi + lo (two bf16 values, 16 significand bits together): the matrix pipe has
    // time to spare, and a single bf16 rounding of P would show up as a one-ulp change in a large
    // share of the bf16 outputs at short contexts
    float plo[4];
#pragma unroll
    for (int r = 0; r < 4; r++) plo[r] = p[r] - bf16_to_f32(f32_to_bf16(p[r]));
    const uint2 pb = make_uint2(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]));
    const uint2 pl = make_uint2(pack_bf16x2(plo[0], plo[1]), pack_bf16x2(plo[2], plo[3]));
    // the values of tokens behind every column's end enter as zeros (their weights are 0, but 0 * NaN is not)
    const uint32_t vm0 = (tok0 < len_wg ? 0x0000ffffu : 0u) | (tok0 + 1 < len_wg ? 0xffff0000u : 0u);
    const uint32_t vm1 = (tok0 + 2 < len_wg ? 0x0000ffffu : 0u) | (tok0 + 3 < len_wg ? 0xffff0000u : 0u);
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const uint2 vv = make_uint2(vreg[t].x & vm0, vreg[t].y & vm1);
      oacc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, vv), __builtin_bit_cast(short4_t, pb),
                                                          oacc[t], 0, 0, 0);
      oacc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, vv), __builtin_bit_cast(short4_t, pl),
                                                          oacc[t], 0, 0, 0);
    }
  };

  {
    int pg = p_begin + wave;
    if (PF == 0) {
      for (; pg < p_end; pg += ATT_WAVES) {
        uint4 kr[8]; uint2 vr[16];
        load_page(pg, pg, kr, vr);
        compute_page(kr, vr, pg);
      }
    } else if (pg < p_end) {
      const int last = pg + ((p_end - 1 - pg) / ATT_WAVES) * ATT_WAVES;      // this wave's last page
      uint4 k0[8], k1[8], k2[8];
      uint2 v0[16], v1[16], v2[16];
      load_page(pg, last, k0, v0);
      load_page(pg + ATT_WAVES, last, k1, v1);
      while (true) {
        load_page(pg + 2 * ATT_WAVES, last, k2, v2); compute_page(k0, v0, pg); pg += ATT_WAVES; if (pg > last) break;
        load_page(pg + 2 * ATT_WAVES, last, k0, v0); compute_page(k1, v1, pg); pg += ATT_WAVES; if (pg > last) break;
        load_page(pg + 2 * ATT_WAVES, last, k1, v1); compute_page(k2, v2, pg); pg += ATT_WAVES; if (pg > last) break;
      }
    }
  }

  // ---- merge the four waves as (0 + 1) + (2 + 3): two exchange rounds through LDS, a third for the transposed write
  float l_tot = l_run + __shfl_xor(l_run, 16);
  l_tot += __shfl_xor(l_tot, 32);
  if (kg == 0) { lds_m[wave][n] = m_run; lds_l[wave][n] = l_tot; }
  __syncthreads();
  float M = lds_m[0][n];
#pragma unroll
  for (int w = 1; w < ATT_WAVES; w++) M = fmaxf(M, lds_m[w][n]);
  const float wscale = (m_run == -INFINITY) ? 0.0f : __expf(m_run - M);
  float L = 0.0f;
#pragma unroll
  for (int w = 0; w < ATT_WAVES; w++) {
    const float mw = lds_m[w][n];
    L += (mw == -INFINITY) ? 0.0f : lds_l[w][n] * __expf(mw - M);
  }
#pragma unroll
  for (int t = 0; t < 16; t++) { oacc[t][0] *= wscale; oacc[t][1] *= wscale; oacc[t][2] *= wscale; oacc[t][3] *= wscale; }
  auto put = [&](int buf) {
#pragma unroll
    for (int t = 0; t < 16; t++)
#pragma unroll
      for (int r = 0; r < 4; r++) lds_o2[buf][16 * t + 4 * kg + r][n] = oacc[t][r];
  };
  // between waves a lane hands its accumulators to the same lane of the other wave: 16-byte pieces in lane order
  // (the [dim][head] layout above is only needed for the write below)
  f32x4_t (*xch)[16][64] = (f32x4_t (*)[16][64])lds_o2;
  auto hand = [&](int buf) {
#pragma unroll
    for (int t = 0; t < 16; t++) xch[buf][t][lane] = oacc[t];
  };
  auto add = [&](int buf) {
#pragma unroll
    for (int t = 0; t < 16; t++) oacc[t] += xch[buf][t][lane];
  };
  if (wave & 1) hand(wave >> 1);          // waves 1 and 3 hand over
  __syncthreads();
  if (!(wave & 1)) add(wave >> 1);        // 0 += 1 (buffer 0), 2 += 3 (buffer 1)
  if (wave == 2) hand(1);                 // buffer 1 was read by wave 2 alone, so it can take the sum straight away
  __syncthreads();
  if (wave == 0) { add(1); put(0); }      // (0 + 1) + (2 + 3), then out for the transposed write (buffer 0: wave 0 was its only reader)
  __syncthreads();
  const float (*lds_o)[16] = lds_o2[0];

  // ---- write: thread = dim, loop over the G heads of the group
  const int d = threadIdx.x;   // 0..255
  const int ncols = A.G * ntk;
  if (A.splits == 1) {
    for (int c = 0; c < ncols; c++) {
      const int head = kvh * A.G + c % A.G;
      const int64_t row = row0 + c / A.G;
      // M and L live in the lanes with n == c; fetch them through LDS
      float Mh = lds_m[0][c];
      for (int w = 1; w < ATT_WAVES; w++) Mh = fmaxf(Mh, lds_m[w][c]);
      float Lh = 0.0f;
      for (int w = 0; w < ATT_WAVES; w++) {
        const float mw = lds_m[w][c];
        Lh += (mw == -INFINITY) ? 0.0f : lds_l[w][c] * __expf(mw - Mh);
      }
      // a sequence without context (length <= 0 found in device memory) has no weights: zeros and lse = -inf
      float o = Lh > 0.0f ? lds_o[d][c] / Lh : 0.0f;
      if (A.gate) {
        const float gv = bf16_to_f32(A.gate[row * A.gate_bstride + (int64_t)head * A.gate_hstride + d]);
        o = __fmul_rn(o, sigmoid_f64(gv));
      }
      A.out[(row * A.NH + head) * ATT_HD + d] = f32_to_bf16(o);
      if (d == 0 && A.lse) A.lse[row * A.NH + head] = Lh > 0.0f ? Mh + logf(Lh) : -INFINITY;
    }
  } else {
    const int64_t pidx = A.slots > 0 ? (int64_t)kvh * A.slots + blockIdx.x : ((int64_t)b * A.NKV + kvh) * A.splits + split;
    float* po = A.part_o + pidx * 16 * ATT_HD;
    for (int c = 0; c < ncols; c++) po[c * ATT_HD + d] = lds_o[d][c];
    if (kg == 0 && wave == 0 && n < ncols) {
      A.part_ml[(pidx * 16 + n) * 2] = M;
      A.part_ml[(pidx * 16 + n) * 2 + 1] = L;
    }
  }
}

// Merge of the split partials: one workgroup per (head, batch), thread = dim.  The weights
// exp(m_s - M) of all splits are computed side by side first (thread = split) and kept in LDS, so the
// loop over the partial outputs has nothing but independent loads in it.
__global__ __launch_bounds__(256) void attn_merge_kernel(AttnArgs A) {
  __shared__ float wsh[ATT_MAX_SPLITS];
  __shared__ float redm[4], redl[4];
  const int head = blockIdx.x, b = blockIdx.y, d = threadIdx.x;      // b: query row
  const int kvh = head / A.G, h = (b % A.tpw) * A.G + head % A.G;     // h: the row's column in its workgroup's partials
  int64_t p0 = ((int64_t)(b / A.tpw) * A.NKV + kvh) * A.splits;
  int nsplit = A.splits;
  if (A.slots > 0) {
    const int2 pl = A.plan[b];
    nsplit = pl.y;
    p0 = (int64_t)kvh * A.slots + pl.x;
  }
  const bool has = d < nsplit;
  const float ms = has ? A.part_ml[((p0 + d) * 16 + h) * 2] : -INFINITY;
  const float ls = has ? A.part_ml[((p0 + d) * 16 + h) * 2 + 1] : 0.0f;
  float M = wave_max(ms);
  if ((d & 63) == 0) redm[d >> 6] = M;
  __syncthreads();
  M = fmaxf(fmaxf(redm[0], redm[1]), fmaxf(redm[2], redm[3]));
  const float w = (ms == -INFINITY) ? 0.0f : __expf(ms - M);
  wsh[d] = w;
  float L = wave_sum(ls * w);
  if ((d & 63) == 0) redl[d >> 6] = L;
  __syncthreads();
  L = (redl[0] + redl[1]) + (redl[2] + redl[3]);
  // the output gate does not depend on the partials: requested and evaluated ahead of them
  const float gsig = A.gate ? sigmoid_f64(bf16_to_f32(A.gate[(int64_t)b * A.gate_bstride + (int64_t)head * A.gate_hstride + d])) : 1.0f;
  const float* po = A.part_o + (p0 * 16 + h) * ATT_HD + d;
  float o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
  int s = 0;
  for (; s + 4 <= nsplit; s += 4) {
    o0 = fmaf(po[(int64_t)(s + 0) * 16 * ATT_HD], wsh[s + 0], o0);
    o1 = fmaf(po[(int64_t)(s + 1) * 16 * ATT_HD], wsh[s + 1], o1);
    o2 = fmaf(po[(int64_t)(s + 2) * 16 * ATT_HD], wsh[s + 2], o2);
    o3 = fmaf(po[(int64_t)(s + 3) * 16 * ATT_HD], wsh[s + 3], o3);
  }
  // the last one to three splits keep their own accumulators, so that splits without pages behind them change nothing
  if (s < nsplit) o0 = fmaf(po[(int64_t)s * 16 * ATT_HD], wsh[s], o0);
  if (s + 1 < nsplit) o1 = fmaf(po[(int64_t)(s + 1) * 16 * ATT_HD], wsh[s + 1], o1);
  if (s + 2 < nsplit) o2 = fmaf(po[(int64_t)(s + 2) * 16 * ATT_HD], wsh[s + 2], o2);
  float o = L > 0.0f ? ((o0 + o1) + (o2 + o3)) / L : 0.0f;      // no context at all: zeros, lse = -inf
  if (A.gate) o = __fmul_rn(o, gsig);
  const uint16_t ob = f32_to_bf16(o);
  A.out[((int64_t)b * A.NH + head) * ATT_HD + d] = ob;
  if (A.out_q8) lane32_q8_1_store(bf16_to_f32(ob), A.out_q8 + (((int64_t)b * A.NH + head) * (ATT_HD / 32) + (d >> 5)) * 36, d & 31);
  if (d == 0 && A.lse) A.lse[(int64_t)b * A.NH + head] = L > 0.0f ? M + logf(L) : -INFINITY;
}

int g_tune_attn_nt = -1;   // K/V pages through nontemporal loads: 0 off, 1 on, -1 = from the size of the read
int g_tune_attn_bal = -1;  // lengths in device memory: 0 = plain splits of the bound, 1 = balanced plan wherever it can run, 2 = relative, -1 = by share

size_t attn_workspace_bytes(int batch, int NKV, int max_splits) {
  return (size_t)batch * NKV * max_splits * 16 * (ATT_HD + 2) * sizeof(float) + 64 * sizeof(int2);
}

int attn_choose_splits(int batch, int NKV, int max_ctx) {
  const int pages = (max_ctx + ATT_PAGE - 1) / ATT_PAGE;
  // aim at one workgroup per CU (measured best at every size: a CU cannot keep more page requests in flight than one
  // workgroup issues, and longer splits amortise start-up and merge), but keep at least one page per wave in a split
  int want = (num_cus() + batch * NKV - 1) / (batch * NKV);
  int cap = (pages + ATT_WAVES - 1) / ATT_WAVES;
  int s = want < cap ? want : cap;
  const int need = (pages + ATT_MAX_PPS - 1) / ATT_MAX_PPS;     // a split's page table must fit its LDS copy
  if (s < need) s = need;
  return s < 1 ? 1 : (s > ATT_MAX_SPLITS ? ATT_MAX_SPLITS : s);
}

int launch_attn_decode(const void* q, const void* kc, const void* vc, const int32_t* block_table, int bt_stride,
                       const int32_t* ctx_len, int ctx_scalar, int ctx_add, int max_ctx, const void* gate, int64_t gate_bstride,
                       int64_t gate_hstride, void* out, float* lse, void* workspace, size_t workspace_bytes, int batch,
                       int NH, int NKV, int HD, int page_size, int splits, void* out_q8, int tpw, int exact, const uint32_t* qf_ready,
                       const AttnPrepFuse* prep) {
  BK_REQUIRE((q || prep) && kc && vc && out, "attn_decode: null pointer");
  BK_REQUIRE(HD == ATT_HD && page_size == ATT_PAGE, "attn_decode: this build serves head_dim 256 and 16-token pages (got %d, %d)", HD, page_size);
  BK_REQUIRE(NKV > 0 && NH > 0 && NH % NKV == 0 && NH / NKV <= 16, "attn_decode: NH=%d NKV=%d (group must be <= 16)", NH, NKV);
  BK_REQUIRE(batch > 0 && batch <= 65535 && NKV <= 65535, "attn_decode: bad batch=%d", batch);
  BK_REQUIRE(ctx_len || ctx_scalar + ctx_add >= 1, "attn_decode: context length must be >= 1");
  BK_REQUIRE(max_ctx >= 1 && (ctx_len || ctx_scalar + ctx_add <= max_ctx), "attn_decode: context %d exceeds max_ctx=%d", ctx_scalar + ctx_add, max_ctx);
  // bt_stride 0 with a table: every row of the batch reads the same sequence's pages (the tokens of one prompt)
  BK_REQUIRE(bt_stride >= (max_ctx + ATT_PAGE - 1) / ATT_PAGE || (block_table && bt_stride == 0),
             "attn_decode: block table rows hold %d pages, context needs %d", bt_stride, (max_ctx + ATT_PAGE - 1) / ATT_PAGE);
  BK_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)kc & 15) == 0 && ((uintptr_t)vc & 15) == 0, "attn_decode: q, K and V must be 16-byte aligned");
  // tpw = 2: rows 2i and 2i+1 are consecutive tokens of one sequence (a prompt) and share a workgroup
  BK_REQUIRE(tpw == 1 || (tpw == 2 && 2 * (NH / NKV) <= 16 && block_table && bt_stride == 0 && ctx_len),
             "attn_decode: two rows per workgroup need a group of at most 8 heads, one shared block table and per-row lengths");
  const int groups = (batch + tpw - 1) / tpw;
  if (splits <= 0) splits = attn_choose_splits(groups, NKV, max_ctx);
  // a context the host knows sizes the splits itself; lengths in device memory leave only their bound
  const int pages = ((ctx_len ? max_ctx : ctx_scalar + ctx_add) + ATT_PAGE - 1) / ATT_PAGE;
  if (splits > pages) splits = pages;
  BK_REQUIRE(splits <= ATT_MAX_SPLITS, "attn_decode: at most %d splits", ATT_MAX_SPLITS);
  BK_REQUIRE((pages + splits - 1) / splits <= ATT_MAX_PPS, "attn_decode: %d pages in %d splits exceed %d pages per split", pages, splits, ATT_MAX_PPS);
  AttnArgs A{};
  A.q = (const uint16_t*)q; A.kc = (const uint16_t*)kc; A.vc = (const uint16_t*)vc;
  A.block_table = block_table; A.ctx_len = ctx_len; A.gate = (const uint16_t*)gate;
  A.out = (uint16_t*)out; A.lse = lse; A.out_q8 = splits > 1 ? (uint8_t*)out_q8 : nullptr;
  A.gate_bstride = gate_bstride; A.gate_hstride = gate_hstride;
  A.bt_stride = bt_stride; A.ctx_scalar = ctx_scalar; A.ctx_add = ctx_add; A.NH = NH; A.NKV = NKV; A.G = NH / NKV;
  A.splits = splits; A.pages_per_split = (pages + splits - 1) / splits;
  A.tpw = tpw; A.rows = batch;
  // lengths in device memory: balanced plan where a workgroup's share of the bound is long (64 pages and up: below that
  // start-up and merge decide the time and the plan's own cost of about a microsecond is not won back), else relative
  // splits; the rows of a prompt keep the plain form (paired and single rows must cut alike).
  // balanced: the batch shares batch * splits slots; a slot's page budget is largest when rows - 1 slots are held back
  A.slots = 0; A.rel = 0; A.max_pages = pages; A.max_ctx = ctx_len ? max_ctx : ctx_scalar + ctx_add;
  const bool prompt_rows = block_table && bt_stride == 0;
  if (ctx_len && tpw == 1 && !prompt_rows && splits > 1 && g_tune_attn_bal != 0) {
    const bool can_balance = batch <= 64 && batch * splits <= ATT_MAX_SPLITS && (int64_t)batch * pages < (1 << 24) &&
        ((int64_t)batch * pages + (batch * splits - batch)) / (batch * splits - batch + 1) <= ATT_MAX_PPS;
    const bool want_balance = g_tune_attn_bal == 1 || (g_tune_attn_bal < 0 && A.pages_per_split >= 64);
    if (can_balance && want_balance) A.slots = batch * splits;
    else if (pages < (1 << 24)) A.rel = 1;
  }
  A.scale = (float)(1.0 / sqrt((double)HD));
  // A cache read that is larger than what the memory-side cache can still hold when the next token comes round (decode
  // at large batch x context) bypasses the caches; prompt rows re-read the same pages and keep the plain loads.
  const bool nt = g_tune_attn_nt >= 0 ? g_tune_attn_nt != 0
                                      : (tpw == 1 && (int64_t)batch * NKV * max_ctx * ATT_HD * 4 >= ((int64_t)128 << 20));
  const dim3 grid(A.slots > 0 ? A.slots : splits, NKV, A.slots > 0 ? 1 : groups), block(ATT_WAVES * 64);
  if (exact) {
    // double-precision form: same cut of the pages, its own kernels and workspace layout
    if (prep) {
      BK_REQUIRE(tpw == 1 && !(block_table && bt_stride == 0), "attn_decode: the folded preparation serves one new token per sequence");
      BK_REQUIRE(prep->qg && prep->k && prep->v && prep->qw && prep->kw && prep->cos_t && prep->sin_t, "attn_decode: null preparation input");
      BK_REQUIRE(prep->half > 0 && 2 * prep->half <= HD && prep->max_len >= 1 && (prep->max_len + ATT_PAGE - 1) / ATT_PAGE <= bt_stride,
                 "attn_decode: bad rotary width %d or capacity %d", prep->half, prep->max_len);
      A.pq = (const uint16_t*)prep->qg; A.pk = (const uint16_t*)prep->k; A.pv = (const uint16_t*)prep->v;
      A.pqw = (const uint16_t*)prep->qw; A.pkw = (const uint16_t*)prep->kw; A.pcos = prep->cos_t; A.psin = prep->sin_t;
      A.phalf = prep->half; A.pmax_len = prep->max_len; A.kcw = (uint16_t*)kc; A.vcw = (uint16_t*)vc;
    }
    int rc = launch_attn_exact(A, q, qf_ready, workspace, workspace_bytes, nt, grid, batch);
    if (rc) return rc;
    if (splits == 1 && out_q8) return launch_quantize_q8_1(out, DT_BF16, out_q8, NH * HD, batch);
    return BK_OK;
  }
  if (splits > 1) {
    BK_REQUIRE(workspace && workspace_bytes >= attn_workspace_bytes(batch, NKV, splits),
               "attn_decode: workspace of %zu bytes needed for %d splits", attn_workspace_bytes(batch, NKV, splits), splits);
    A.part_o = (float*)workspace;
    A.part_ml = A.part_o + (size_t)batch * NKV * splits * 16 * ATT_HD;
    A.plan = (int2*)(A.part_ml + (size_t)batch * NKV * splits * 16 * 2);
  }
  // waves with three pages or more keep two pages in flight ahead of the one they work on
  if (A.pages_per_split >= 3 * ATT_WAVES) {
    if (nt) hipLaunchKernelGGL((attn_decode_kernel<2, true>), grid, block, 0, stream(), A);
    else hipLaunchKernelGGL((attn_decode_kernel<2, false>), grid, block, 0, stream(), A);
  } else {
    if (nt) hipLaunchKernelGGL((attn_decode_kernel<0, true>), grid, block, 0, stream(), A);
    else hipLaunchKernelGGL((attn_decode_kernel<0, false>), grid, block, 0, stream(), A);
  }
  if (splits > 1) hipLaunchKernelGGL(attn_merge_kernel, dim3(NH, batch), dim3(256), 0, stream(), A);
  BK_LAUNCH_CHECK();
  // a single split writes its output from the attention kernel itself; its Q8_1 copy then takes the stand-alone quantizer
  if (splits == 1 && out_q8) return launch_quantize_q8_1(out, DT_BF16, out_q8, NH * HD, batch);
  return BK_OK;
}

// ---------------------------------------------------------------- split-K attention that allocates nothing
// For callers that cannot allocate (code under graph capture, tight serving loops): the partial results of the splits go
// to a fixed array in device memory instead of a caller's workspace.  Every GPU the library runs on holds its own copy
// of the array at its own address, which the host learns once per device from hipGetSymbolAddress; in host code the
// array's name is not a device address and is never passed to a kernel or a copy.
constexpr int NOALLOC_MAX_PARTIALS = 1024;        // batch * NKV * splits workgroup partials of 16 x (256 + 2) floats
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)NOALLOC_MAX_PARTIALS * 16 * (ATT_HD + 2) * sizeof(float) + 64 * sizeof(int2);
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];      // 16.1 MiB per GPU, for the life of the process
constexpr int NOALLOC_MAX_DEVICES = 64;
static void* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};

// called by bk_init with `device` current: the address of this device's copy of `scratch`
int attn_noalloc_setup(int device) {
  BK_REQUIRE(device >= 0 && device < NOALLOC_MAX_DEVICES, "attn_noalloc_setup: device %d beyond the %d this build keeps an address for", device,
             NOALLOC_MAX_DEVICES);
  void* p = nullptr;
  BK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  BK_REQUIRE(p != nullptr, "attn_noalloc_setup: no device address for the scratch array");
  g_scratch_ptr[device] = p;
  return BK_OK;
}
void attn_noalloc_teardown(int device) {
  if (device >= 0 && device < NOALLOC_MAX_DEVICES) g_scratch_ptr[device] = nullptr;
}

// The arguments of launch_attn_decode without the workspace.  Nothing in the array has to start at zero: every
// partial a merge reads was written by the attention kernel of the same call (also for splits without pages).
int launch_attn_decode_noalloc(int device, const void* q, const void* kc, const void* vc, const int32_t* block_table, int bt_stride,
                               const int32_t* ctx_len, int max_ctx, const void* gate, int64_t gate_bstride, int64_t gate_hstride,
                               void* out, float* lse, int batch, int NH, int NKV, int HD, int page_size, int splits) {
  BK_REQUIRE(device >= 0 && device < NOALLOC_MAX_DEVICES && g_scratch_ptr[device], "attn_decode_noalloc: bk_init has not set up device %d", device);
  BK_REQUIRE(batch > 0 && NKV > 0 && max_ctx >= 1, "attn_decode_noalloc: bad batch=%d NKV=%d max_ctx=%d", batch, NKV, max_ctx);
  const int64_t groups = (int64_t)batch * NKV;
  if (splits <= 0) {
    // the library's own choice, held to what the array takes (one split needs no partials at all)
    splits = attn_choose_splits(batch, NKV, max_ctx);
    if (groups * splits > NOALLOC_MAX_PARTIALS) splits = (int)(NOALLOC_MAX_PARTIALS / groups);
    if (splits < 1) splits = 1;
  }
  const int pages = (max_ctx + ATT_PAGE - 1) / ATT_PAGE;
  if (splits > pages) splits = pages;
  BK_REQUIRE(splits == 1 || groups * splits <= NOALLOC_MAX_PARTIALS,
             "attn_decode_noalloc: batch %d x %d KV heads x %d splits = %lld partial results exceed the %d of the built-in scratch "
             "(use fewer splits, or bk_attn_decode with a workspace)", batch, NKV, splits, (long long)(groups * splits), NOALLOC_MAX_PARTIALS);
  return launch_attn_decode(q, kc, vc, block_table, bt_stride, ctx_len, 0, 0, max_ctx, gate, gate_bstride, gate_hstride, out, lse,
                            g_scratch_ptr[device], NOALLOC_SCRATCH_BYTES, batch, NH, NKV, HD, page_size, splits, nullptr, 1, 0, nullptr, nullptr);
}

// ---------------------------------------------------------------- per-head norm + RoPE + cache append in one launch
// qnorm -> rope, knorm -> ropek and the cache write (src/emitters.ts:123-183, 202-205) as one kernel:
// one wavefront per (role, head, sequence).  Query heads go to `qout` (bf16 [B, NH, 256]); the
// normalised, rotated key goes straight into its K page and the value into its V page (dim-major),
// so neither passes through memory a second time.  Arithmetic as in the stand-alone kernels:
//   n[i] = bf16((x[i] * rstd) * (1 + w[i])), rstd from the sum of squares in double;
//   pairs (i, i + half), i < half: x1' = bf16(x1*c - x2*s), x2' = bf16(x2*c + x1*s).
struct PrepArgs {
  const uint16_t *qg, *k, *v;      // q|gate bf16 [B, NH, 2*256]; k, v bf16 [B, NKV, 256]
  const uint16_t *qw, *kw;         // norm weights bf16 [256]
  const float *cos_t, *sin_t;      // f32 [max_len, half]
  const int32_t* pos_dev; int pos_scalar;
  uint16_t *qout, *kc, *vc;
  uint32_t* qf;                    // optional: the query heads also widened to f64, high words [B, NKV, 256, 8], for the double-precision attention
  const int32_t* block_table; int bt_stride;
  int NH, NKV, half, max_len;
};

__global__ __launch_bounds__(64) void attn_prep_kernel(PrepArgs A) {
  __shared__ uint16_t sh[ATT_HD];
  const int role = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  // A position read from device memory cannot be checked by the host: one outside the cache (a loop replayed past its
  // capacity) writes nothing, like the masked store of src/emitters.ts:203-205, and reads the tables at the nearest row.
  const int pos_raw = A.pos_dev ? A.pos_dev[b] : A.pos_scalar;
  const int pos = min(max(pos_raw, 0), A.max_len - 1);
  const bool in_cache = pos == pos_raw;
  const int pg = pos / ATT_PAGE, slot = pos % ATT_PAGE;
  const bool is_q = role < A.NH, is_k = !is_q && role < A.NH + A.NKV;
  if (!is_q && !in_cache) return;
  const int kvh = is_q ? 0 : (is_k ? role - A.NH : role - A.NH - A.NKV);
  const int phys = A.block_table ? A.block_table[(int64_t)b * A.bt_stride + pg] : b * A.bt_stride + pg;
  const int64_t base = ((int64_t)phys * A.NKV + kvh) * (ATT_PAGE * ATT_HD);
  if (!is_q && !is_k) {
    const uint16_t* vp = A.v + ((int64_t)b * A.NKV + kvh) * ATT_HD;
    for (int i = lane; i < ATT_HD; i += 64) A.vc[base + i * ATT_PAGE + slot] = vp[i];
    return;
  }
  const uint16_t* xh = is_q ? A.qg + ((int64_t)b * A.NH + role) * 2 * ATT_HD : A.k + ((int64_t)b * A.NKV + kvh) * ATT_HD;
  const uint16_t* w = is_q ? A.qw : A.kw;
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
  __syncthreads();
  uint16_t* dst = is_q ? A.qout + ((int64_t)b * A.NH + role) * ATT_HD : A.kc + base + slot * ATT_HD;
  const int half = A.half;
#pragma unroll
  for (int j = 0; j < ATT_HD / 64; j++) {
    const int i = lane + 64 * j;
    uint16_t o = sh[i];
    if (i < 2 * half) {
      const int i1 = i < half ? i : i - half;
      const float x1 = bf16_to_f32(sh[i1]), x2 = bf16_to_f32(sh[i1 + half]);
      const float c = A.cos_t[(int64_t)pos * half + i1], sn = A.sin_t[(int64_t)pos * half + i1];
      o = i < half ? f32_to_bf16(__fsub_rn(__fmul_rn(x1, c), __fmul_rn(x2, sn)))
                   : f32_to_bf16(__fadd_rn(__fmul_rn(x2, c), __fmul_rn(x1, sn)));
    }
    dst[i] = o;
    if (is_q && A.qf) {
      const int G = A.NH / A.NKV;
      A.qf[(((int64_t)b * A.NKV + role / G) * ATT_HD + i) * 8 + role % G] = (uint32_t)(__builtin_bit_cast(uint64_t, (double)bf16_to_f32(o)) >> 32);
    }
  }
}

int launch_attn_prep(const void* qg, const void* k, const void* v, const void* qw, const void* kw, const float* cos_t,
                     const float* sin_t, const int32_t* pos_dev, int pos_scalar, int half, int max_len, void* qout, void* kc,
                     void* vc, const int32_t* block_table, int bt_stride, int batch, int NH, int NKV, int HD, int page_size, uint32_t* qf) {
  BK_REQUIRE(qg && k && v && qw && kw && cos_t && sin_t && qout && kc && vc, "attn_prep: null pointer");
  BK_REQUIRE(HD == ATT_HD && page_size == ATT_PAGE, "attn_prep: head_dim 256 and 16-token pages only");
  BK_REQUIRE(batch > 0 && batch <= 65535 && NH > 0 && NKV > 0 && half > 0 && 2 * half <= HD, "attn_prep: bad shape");
  BK_REQUIRE(max_len >= 1 && (bt_stride == 0 || (max_len + ATT_PAGE - 1) / ATT_PAGE <= bt_stride),
             "attn_prep: max_len=%d exceeds the %d pages of a block table row", max_len, bt_stride);
  BK_REQUIRE(pos_dev || (pos_scalar >= 0 && pos_scalar < max_len && pos_scalar / ATT_PAGE < bt_stride),
             "attn_prep: pos=%d outside the cache (max_len=%d)", pos_scalar, max_len);
  PrepArgs A{};
  A.qg = (const uint16_t*)qg; A.k = (const uint16_t*)k; A.v = (const uint16_t*)v; A.qw = (const uint16_t*)qw; A.kw = (const uint16_t*)kw;
  A.cos_t = cos_t; A.sin_t = sin_t; A.pos_dev = pos_dev; A.pos_scalar = pos_scalar;
  A.qout = (uint16_t*)qout; A.kc = (uint16_t*)kc; A.vc = (uint16_t*)vc; A.block_table = block_table; A.bt_stride = bt_stride;
  A.NH = NH; A.NKV = NKV; A.half = half; A.max_len = max_len;
  BK_REQUIRE(!qf || (NH % NKV == 0 && NH / NKV <= 8), "attn_prep: the f64 query copy serves groups of at most 8 heads");
  A.qf = qf;
  hipLaunchKernelGGL(attn_prep_kernel, dim3(NH + 2 * NKV, batch), dim3(64), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

// ---------------------------------------------------------------- cache append
// The cache write of src/emitters.ts:202-205: token `pos` of every sequence gets this
// step's k and v (bf16 [B, NKV, 256]); V goes in dim-major.
__global__ __launch_bounds__(256) void kv_append_kernel(const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                        uint16_t* __restrict__ kc, uint16_t* __restrict__ vc,
                                                        const int32_t* __restrict__ block_table, int bt_stride,
                                                        const int32_t* __restrict__ pos_dev, int pos_scalar, int NKV,
                                                        int max_len) {
  const int kvh = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const int pos = pos_dev ? pos_dev[b] : pos_scalar;
  if (pos < 0 || pos >= max_len) return;      // outside the cache: nothing is written (src/emitters.ts:203-205 masks the same store)
  const int pg = pos / ATT_PAGE, slot = pos % ATT_PAGE;
  const int phys = block_table ? block_table[(int64_t)b * bt_stride + pg] : b * bt_stride + pg;
  const int64_t base = ((int64_t)phys * NKV + kvh) * (ATT_PAGE * ATT_HD);
  const int64_t src = ((int64_t)b * NKV + kvh) * ATT_HD + d;
  kc[base + slot * ATT_HD + d] = k[src];
  vc[base + d * ATT_PAGE + slot] = v[src];
}

int launch_kv_append(const void* k, const void* v, void* kc, void* vc, const int32_t* block_table, int bt_stride,
                     const int32_t* pos_dev, int pos_scalar, int max_len, int batch, int NKV, int HD, int page_size) {
  BK_REQUIRE(k && v && kc && vc, "kv_append: null pointer");
  BK_REQUIRE(max_len >= 1 && (max_len + ATT_PAGE - 1) / ATT_PAGE <= bt_stride, "kv_append: max_len=%d exceeds the %d pages of a block table row",
             max_len, bt_stride);
  BK_REQUIRE(HD == ATT_HD && page_size == ATT_PAGE, "kv_append: head_dim 256 and 16-token pages only");
  BK_REQUIRE(batch > 0 && batch <= 65535 && NKV > 0 && NKV <= 65535, "kv_append: bad shape");
  BK_REQUIRE(pos_dev || (pos_scalar >= 0 && pos_scalar < max_len), "kv_append: pos=%d outside the cache (max_len=%d)", pos_scalar, max_len);
  hipLaunchKernelGGL(kv_append_kernel, dim3(NKV, batch), dim3(256), 0, stream(), (const uint16_t*)k, (const uint16_t*)v,
                     (uint16_t*)kc, (uint16_t*)vc, block_table, bt_stride, pos_dev, pos_scalar, NKV, max_len);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
