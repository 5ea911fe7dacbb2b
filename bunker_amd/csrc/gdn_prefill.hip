// Gated DeltaNet over a run of T prompt tokens: the recurrence of gdn.hip applied token after token with the
// state held in registers, so S is read once and written once per run instead of once per token.
// (The reference's prefill prototypes use the chunked form, prototypes/gdn_fast.ts and gdn_solve_tril.ts; this
// is the sequential form, which gives the bits of T single-token steps: src/emitters.ts:75-120.)
//
// Three kernels:
//   prep     per (token, head): q^ = q * rsqrt(sum q^2 + 1e-6) / sqrt(128), k^ = k * rsqrt(sum k^2 + 1e-6),
//            decay = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b); all tokens in parallel
//   scan     per (head, slab of 32 v columns): lane (row group kg, column c) owns rows 16*kg .. 16*kg+15 of
//            one column; per token: decay, kS by an fmaf chain over the 16 rows and the sum of the 8 group
//            results in order, delta, update, o the same way.  The order of every sum is the one the
//            single-token kernel uses, so the results are equal to the bit.
//   outnorm  per (token, head): gated RMSNorm of the 128 outputs with z, bf16 result; all tokens in parallel
#include "ops.h"

namespace bk {

constexpr int GP_D = 128;
constexpr int GP_COLS = 32;                 // v columns per scan workgroup
constexpr int GP_SLABS = GP_D / GP_COLS;    // 4
constexpr int GP_KG = 8;                    // row groups
constexpr int GP_ROWS = GP_D / GP_KG;       // 16 rows per thread

struct GdnPrefillArgs {
  const uint16_t* conv_out;   // bf16 [T, 3*Hg*128]: q | k | v
  const uint16_t* z;          // bf16 [T, Hg*128]
  const float* A_log;         // f32 [Hg]
  const uint16_t* dt_bias;    // bf16 [Hg]
  const float* a_p;           // f32 [T, Hg]
  const float* b_p;           // f32 [T, Hg]
  const float* norm_w;        // f32 [128]
  const float* S_in;          // f32 [Hg, 128, 128]
  float* S_out;
  uint16_t* out;              // bf16 [T, Hg*128]
  float* qk;                  // scratch f32 [T, Hg, 2, 128]: q^, k^
  float* gates;               // scratch f32 [T, Hg, 2]: decay, beta
  float* o_raw;               // scratch f32 [T, Hg, 128]
  int Hg, T;
};

// One wave per (token, head, q | k) row of 128 values, two per lane; a workgroup's four waves take 64 consecutive rows,
// i.e. 32 (token, head) pairs, whose gates — a chain of double-precision exponentials and logarithms, several hundred
// instructions long whether one lane runs it or 64 — are worked out side by side by 32 lanes of the first wave.
// (The squares of bf16 values are exact in f32 and their sum over a row is exact in f64, so the order of that sum —
// here lane pairs first, in the single-token kernel 64-lane halves first — does not show in the result.)
constexpr int GP_PREP_ROWS = 64;
__global__ __launch_bounds__(256) void gdn_prefill_prep_kernel(GdnPrefillArgs A) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int KEYDIM = A.Hg * GP_D;
  const int64_t nrows = (int64_t)A.T * A.Hg * 2;
  const int64_t row0 = (int64_t)blockIdx.x * GP_PREP_ROWS;
  if (wave == 0 && lane < GP_PREP_ROWS / 2) {
    const int64_t th = (row0 >> 1) + lane;
    if (th < (int64_t)A.T * A.Hg) {
      const int h = (int)(th % A.Hg);
      const float sp_in = A.a_p[th] + bf16_to_f32(A.dt_bias[h]);
      const float softplus = (float)log1p(exp((double)sp_in));
      A.gates[th * 2] = (float)exp(-(double)((float)exp((double)A.A_log[h]) * softplus));
      A.gates[th * 2 + 1] = sigmoid_f64(A.b_p[th]);
    }
  }
  for (int it = 0; it < GP_PREP_ROWS / 4; it++) {
    const int64_t rowi = row0 + 4 * it + wave;       // (t, h, q | k) in the order of A.qk
    if (rowi >= nrows) break;
    const int isk = (int)(rowi & 1);
    const int64_t th = rowi >> 1;
    const int t = (int)(th / A.Hg), h = (int)(th - (int64_t)t * A.Hg);
    const uint32_t pair = *(const uint32_t*)(A.conv_out + (int64_t)t * 3 * KEYDIM + (isk ? KEYDIM : 0) + h * GP_D + 2 * lane);
    const float x0 = __uint_as_float(pair << 16), x1 = __uint_as_float(pair & 0xffff0000u);
    const double tot = wave_sum_f64((double)(x0 * x0) + (double)(x1 * x1));
    const float rs = rsqrt_f64(tot + 1e-6);
    const float f = isk ? rs : rs * 0.08838834764831845f;     // 1/sqrt(128) on q
    *(float2*)(A.qk + rowi * GP_D + 2 * lane) = make_float2(x0 * f, x1 * f);
  }
}

// The scan.  A workgroup owns 32 v columns of one head; its four wavefronts are independent: wavefront w owns columns
// 8w .. 8w+7, lane (column c = lane / 8, row group kg = lane % 8) holds rows 16*kg .. 16*kg+15 of its column for the
// whole run.  The eight row-group results of a column sit in eight neighbouring lanes, so they meet through lane
// permutes (no LDS round trip, no barrier) and every lane adds them in group order.  The per-token operands (q^, k^,
// v, decay, beta) are staged in LDS a block of GP_TB tokens at a time, the next block's global loads in flight while
// the current block is computed; the workgroup synchronises once per block, for that hand-over only.
constexpr int GP_TB = 16;

struct TokenIn {
  float4 k[4], q[4];
  float v, decay, beta;
};

// Sum over the eight row groups of a column in group order, ((p0 + p1) + ... + p7): the lanes of the lower quad
// hold p0..p3 themselves (quad broadcasts) and fetch p4..p7 from the upper quad (mirror within the eight lanes).
// Lanes of the upper quad end up with another order of additions; they take the lower quad's result when `all`.
template <bool ALL>
__device__ __forceinline__ float group_sum8(float x, bool upper) {
  const float a0 = dpp_f32<0x00>(x), a1 = dpp_f32<0x55>(x), a2 = dpp_f32<0xAA>(x), a3 = dpp_f32<0xFF>(x);   // own quad's four
  const float b0 = dpp_f32<DPP_ROW_HALF_MIRROR>(a0), b1 = dpp_f32<DPP_ROW_HALF_MIRROR>(a1);                  // the other quad's
  const float b2 = dpp_f32<DPP_ROW_HALF_MIRROR>(a2), b3 = dpp_f32<DPP_ROW_HALF_MIRROR>(a3);
  const float s = ((((((a0 + a1) + a2) + a3) + b0) + b1) + b2) + b3;
  if (!ALL) return s;                                         // valid in the lower quad only
  const float lower = dpp_f32<DPP_ROW_HALF_MIRROR>(s);
  return upper ? lower : s;
}

struct ScanState {
  float S[GP_ROWS];
};
// one token of the recurrence for this lane's 16 rows of one column; returns the column's output (lower quad)
__device__ __forceinline__ float scan_token(ScanState& st, const TokenIn& in, bool upper) {
  const float kr[GP_ROWS] = {in.k[0].x, in.k[0].y, in.k[0].z, in.k[0].w, in.k[1].x, in.k[1].y, in.k[1].z, in.k[1].w,
                             in.k[2].x, in.k[2].y, in.k[2].z, in.k[2].w, in.k[3].x, in.k[3].y, in.k[3].z, in.k[3].w};
  const float qr[GP_ROWS] = {in.q[0].x, in.q[0].y, in.q[0].z, in.q[0].w, in.q[1].x, in.q[1].y, in.q[1].z, in.q[1].w,
                             in.q[2].x, in.q[2].y, in.q[2].z, in.q[2].w, in.q[3].x, in.q[3].y, in.q[3].z, in.q[3].w};
  float acc = 0.f;
#pragma unroll
  for (int r = 0; r < GP_ROWS; r++) {
    st.S[r] *= in.decay;
    acc = fmaf(kr[r], st.S[r], acc);
  }
  const float kS = group_sum8<true>(acc, upper);
  const float d = (in.v - kS) * in.beta;
  acc = 0.f;
#pragma unroll
  for (int r = 0; r < GP_ROWS; r++) {
    st.S[r] = fmaf(kr[r], d, st.S[r]);
    acc = fmaf(qr[r], st.S[r], acc);
  }
  return group_sum8<false>(acc, upper);
}

__global__ __launch_bounds__(256) void gdn_prefill_scan_kernel(GdnPrefillArgs A) {
  __shared__ __align__(16) float s_qk[2][GP_TB][2 * GP_D];     // q^ | k^ of each staged token
  __shared__ float s_v[2][GP_TB][GP_COLS];
  __shared__ float s_g[2][GP_TB][2];
  const int h = blockIdx.x, slab = blockIdx.y, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int kg = lane & 7, c = wave * 8 + (lane >> 3);        // column within the slab
  const bool upper = (lane & 4) != 0;
  const int col = slab * GP_COLS + c;
  const int64_t KEYDIM = (int64_t)A.Hg * GP_D;
  const float* Sp = A.S_in + (int64_t)h * GP_D * GP_D + (int64_t)(kg * GP_ROWS) * GP_D + col;
  ScanState st;
#pragma unroll
  for (int r = 0; r < GP_ROWS; r++) st.S[r] = Sp[(int64_t)r * GP_D];

  // staging: thread tid moves float4 pieces tid, tid+256, tid+512, tid+768 of the block's 16 x 256 floats of q^/k^,
  // two v values and one gate value; token indices past the end repeat the last token (never consumed)
  float4 gq0, gq1, gq2, gq3;
  uint32_t gv;
  float gg;
#define GP_STAGE_LOAD(T0)                                                                                              \
  {                                                                                                                    \
    const float* qk_h = A.qk + (int64_t)h * 2 * GP_D + (tid % 64) * 4;                                                 \
    const int64_t tstride = (int64_t)A.Hg * 2 * GP_D;                                                                  \
    gq0 = *(const float4*)(qk_h + min((T0) + tid / 64, A.T - 1) * tstride);                                            \
    gq1 = *(const float4*)(qk_h + min((T0) + 4 + tid / 64, A.T - 1) * tstride);                                        \
    gq2 = *(const float4*)(qk_h + min((T0) + 8 + tid / 64, A.T - 1) * tstride);                                        \
    gq3 = *(const float4*)(qk_h + min((T0) + 12 + tid / 64, A.T - 1) * tstride);                                       \
    gv = *(const uint32_t*)(A.conv_out + (int64_t)min((T0) + tid / 16, A.T - 1) * 3 * KEYDIM + 2 * KEYDIM + h * GP_D + \
                            slab * GP_COLS + (tid % 16) * 2);                                                          \
    gg = A.gates[((int64_t)min((T0) + (tid & 31) / 2, A.T - 1) * A.Hg + h) * 2 + (tid & 1)];                           \
  }
#define GP_STAGE_STORE(BUF)                                                              \
  {                                                                                      \
    *(float4*)&s_qk[BUF][tid / 64][(tid % 64) * 4] = gq0;                                \
    *(float4*)&s_qk[BUF][4 + tid / 64][(tid % 64) * 4] = gq1;                            \
    *(float4*)&s_qk[BUF][8 + tid / 64][(tid % 64) * 4] = gq2;                            \
    *(float4*)&s_qk[BUF][12 + tid / 64][(tid % 64) * 4] = gq3;                           \
    s_v[BUF][tid / 16][(tid % 16) * 2] = __uint_as_float(gv << 16);                      \
    s_v[BUF][tid / 16][(tid % 16) * 2 + 1] = __uint_as_float(gv & 0xffff0000u);          \
    if (tid < 32) s_g[BUF][tid / 2][tid & 1] = gg;                                       \
  }
  auto token_read = [&](TokenIn& in, int buf, int t) {
    const float4* qp = (const float4*)&s_qk[buf][t][kg * GP_ROWS];
    const float4* kp = (const float4*)&s_qk[buf][t][GP_D + kg * GP_ROWS];
#pragma unroll
    for (int r = 0; r < 4; r++) { in.q[r] = qp[r]; in.k[r] = kp[r]; }
    in.v = s_v[buf][t][c];
    in.decay = s_g[buf][t][0];
    in.beta = s_g[buf][t][1];
  };

  GP_STAGE_LOAD(0)
  GP_STAGE_STORE(0)
  __syncthreads();
  int buf = 0;
  for (int t0 = 0; t0 < A.T; t0 += GP_TB) {
    const int nt = min(GP_TB, A.T - t0);
    GP_STAGE_LOAD(t0 + GP_TB)                                  // next block (clamped), in flight during this block
    float* orow = A.o_raw + ((int64_t)t0 * A.Hg + h) * GP_D + col;
    const int64_t ostride = (int64_t)A.Hg * GP_D;
    if (nt == GP_TB) {
      // a full block, unrolled: two operand sets alternate, the next token's LDS reads are issued ahead of the
      // arithmetic of the current one, and the output chain of one token overlaps the kS chain of the next
      TokenIn in0, in1;
      token_read(in0, buf, 0);
#pragma unroll
      for (int tt = 0; tt < GP_TB; tt += 2) {
        token_read(in1, buf, tt + 1);
        const float o0 = scan_token(st, in0, upper);
        if (kg == 0) orow[(int64_t)tt * ostride] = o0;
        if (tt + 2 < GP_TB) token_read(in0, buf, tt + 2);
        const float o1 = scan_token(st, in1, upper);
        if (kg == 0) orow[(int64_t)(tt + 1) * ostride] = o1;
      }
    } else {
      for (int tt = 0; tt < nt; tt++) {
        TokenIn in;
        token_read(in, buf, tt);
        const float o = scan_token(st, in, upper);
        if (kg == 0) orow[(int64_t)tt * ostride] = o;
      }
    }
    GP_STAGE_STORE(buf ^ 1)    // nobody reads buf ^ 1 in this block; the barrier below publishes it and retires buf
    __syncthreads();
    buf ^= 1;
  }
#undef GP_STAGE_LOAD
#undef GP_STAGE_STORE
  float* So = A.S_out + (int64_t)h * GP_D * GP_D + (int64_t)(kg * GP_ROWS) * GP_D + col;
#pragma unroll
  for (int r = 0; r < GP_ROWS; r++) So[(int64_t)r * GP_D] = st.S[r];
}

// One wave per (token, head): the 128 outputs two per lane, 16 rows per workgroup.  (The sum of squares is taken in
// double; its last bit may depend on the order of the additions, which the rounding of its inverse root to f32 absorbs.)
__global__ __launch_bounds__(256) void gdn_prefill_outnorm_kernel(GdnPrefillArgs A) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t nrows = (int64_t)A.T * A.Hg;
  for (int it = 0; it < GP_PREP_ROWS / 4; it++) {
    const int64_t th = (int64_t)blockIdx.x * GP_PREP_ROWS + 4 * it + wave;
    if (th >= nrows) break;
    const float2 o = *(const float2*)(A.o_raw + th * GP_D + 2 * lane);
    const uint32_t zp = *(const uint32_t*)(A.z + th * GP_D + 2 * lane);
    const float2 nw = *(const float2*)(A.norm_w + 2 * lane);
    const float z0 = __uint_as_float(zp << 16), z1 = __uint_as_float(zp & 0xffff0000u);
    const double oss = wave_sum_f64((double)o.x * (double)o.x + (double)o.y * (double)o.y);
    const float orstd = rsqrt_f64(oss / (double)GP_D + 1e-6);
    const float zs0 = z0 * sigmoid_f64(z0), zs1 = z1 * sigmoid_f64(z1);
    const uint32_t r0 = f32_to_bf16(((o.x * orstd) * nw.x) * zs0), r1 = f32_to_bf16(((o.y * orstd) * nw.y) * zs1);
    *(uint32_t*)(A.out + th * GP_D + 2 * lane) = r0 | (r1 << 16);
  }
}

static size_t gdn_prefill_base_bytes(int Hg, int T) { return (((size_t)T * Hg * (2 * GP_D + GP_D + 2) * sizeof(float)) + 255) & ~(size_t)255; }

size_t gdn_prefill_workspace_bytes(int Hg, int T, bool chunked) {
  return gdn_prefill_base_bytes(Hg, T) + (chunked ? gdn_chunk_workspace_bytes(Hg, T) : 0);
}

int launch_gdn_prefill(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                       const float* b_p, const float* norm_w, const float* S_in, void* out, float* S_out, void* workspace,
                       size_t workspace_bytes, int Hg, int T, bool chunked) {
  BK_REQUIRE(conv_out && z && A_log && dt_bias && a_p && b_p && norm_w && S_in && out && S_out && workspace, "gdn_prefill: null pointer");
  BK_REQUIRE(Hg > 0 && Hg <= 65535 && T > 0 && T <= 65535, "gdn_prefill: bad Hg=%d T=%d", Hg, T);
  BK_REQUIRE(workspace_bytes >= gdn_prefill_workspace_bytes(Hg, T, chunked), "gdn_prefill: workspace of %zu bytes, need %zu", workspace_bytes,
             gdn_prefill_workspace_bytes(Hg, T, chunked));
  BK_REQUIRE(((uintptr_t)workspace & 15) == 0, "gdn_prefill: workspace must be 16-byte aligned");
  GdnPrefillArgs A{};
  A.conv_out = (const uint16_t*)conv_out; A.z = (const uint16_t*)z; A.A_log = A_log; A.dt_bias = (const uint16_t*)dt_bias;
  A.a_p = a_p; A.b_p = b_p; A.norm_w = norm_w; A.S_in = S_in; A.S_out = S_out; A.out = (uint16_t*)out;
  A.qk = (float*)workspace;
  A.o_raw = A.qk + (size_t)T * Hg * 2 * GP_D;
  A.gates = A.o_raw + (size_t)T * Hg * GP_D;
  A.Hg = Hg; A.T = T;
  hipLaunchKernelGGL(gdn_prefill_prep_kernel, dim3((unsigned)(((int64_t)T * Hg * 2 + GP_PREP_ROWS - 1) / GP_PREP_ROWS)), dim3(256), 0, stream(), A);
  if (chunked) {
    // the chunked form of the recurrence (gdn_chunk.hip) between the same preparation and output norm
    const size_t base = gdn_prefill_base_bytes(Hg, T);
    const int rc = launch_gdn_chunked_core(conv_out, A_log, dt_bias, a_p, A.qk, A.gates, S_in, S_out, A.o_raw, (uint8_t*)workspace + base,
                                           workspace_bytes - base, Hg, T);
    if (rc) return rc;
  } else {
    hipLaunchKernelGGL(gdn_prefill_scan_kernel, dim3(Hg, GP_SLABS), dim3(256), 0, stream(), A);
  }
  hipLaunchKernelGGL(gdn_prefill_outnorm_kernel, dim3((unsigned)(((int64_t)T * Hg + GP_PREP_ROWS - 1) / GP_PREP_ROWS)), dim3(256), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
