// Gated DeltaNet over a run of T prompt tokens: the recurrence of gdn.hip applied token after token with the
// state held in registers, so S is read once and written once per run instead of once per token.
// (The reference's prefill prototypes use the chunked form, prototypes/gdn_fast.ts and gdn_solve_tril.ts; this
// is the sequential form, which gives the bits of T single-token steps: src/emitters.ts:75-120.)
//
// Three kernels:
//   prep     per (token, head): q^ = q * rsqrt(sum q^2 + 1e-6) / sqrt(128), k^ = k * rsqrt(sum k^2 + 1e-6),
//            decay = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b); all tokens in parallel
//   scan     per (head, slab of 32 v columns): thread (row group kg, column c) owns rows 16*kg .. 16*kg+15 of
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

__global__ __launch_bounds__(256) void gdn_prefill_prep_kernel(GdnPrefillArgs A) {
  __shared__ double red[4];
  const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x;
  const int KEYDIM = A.Hg * GP_D;
  const bool isk = tid >= 128;
  const int i = tid & 127;
  const uint16_t* row = A.conv_out + (int64_t)t * 3 * KEYDIM;
  const float x = bf16_to_f32(row[(isk ? KEYDIM : 0) + h * GP_D + i]);
  const double ss = wave_sum_f64((double)(x * x));       // square of a bf16 value: exact in f32
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  const double tot = isk ? (red[2] + red[3]) : (red[0] + red[1]);
  const float rs = rsqrt_f64(tot + 1e-6);
  const int64_t th = (int64_t)t * A.Hg + h;
  A.qk[(th * 2 + (isk ? 1 : 0)) * GP_D + i] = isk ? x * rs : x * (rs * 0.08838834764831845f);     // 1/sqrt(128)
  if (tid == 0) {
    const float sp_in = A.a_p[th] + bf16_to_f32(A.dt_bias[h]);
    const float softplus = (float)log1p(exp((double)sp_in));
    A.gates[th * 2] = (float)exp(-(double)((float)exp((double)A.A_log[h]) * softplus));
    A.gates[th * 2 + 1] = sigmoid_f64(A.b_p[th]);
  }
}

struct ScanIn {
  float4 k[4], q[4];
  float v, decay, beta;
};
__device__ __forceinline__ void scan_load(ScanIn& in, const GdnPrefillArgs& A, int t, int h, int kg, int col) {
  const int64_t th = (int64_t)t * A.Hg + h;
  const float4* qp = (const float4*)(A.qk + th * 2 * GP_D + kg * GP_ROWS);
  const float4* kp = (const float4*)(A.qk + (th * 2 + 1) * GP_D + kg * GP_ROWS);
#pragma unroll
  for (int r = 0; r < 4; r++) { in.q[r] = qp[r]; in.k[r] = kp[r]; }
  in.v = bf16_to_f32(A.conv_out[(int64_t)t * 3 * A.Hg * GP_D + 2 * A.Hg * GP_D + h * GP_D + col]);
  in.decay = A.gates[th * 2];
  in.beta = A.gates[th * 2 + 1];
}

__global__ __launch_bounds__(256) void gdn_prefill_scan_kernel(GdnPrefillArgs A) {
  __shared__ float part_k[GP_KG][GP_COLS], part_o[GP_KG][GP_COLS];
  const int h = blockIdx.x, slab = blockIdx.y, tid = threadIdx.x;
  const int kg = tid / GP_COLS, c = tid % GP_COLS;
  const int col = slab * GP_COLS + c;
  const float* Sp = A.S_in + (int64_t)h * GP_D * GP_D + (int64_t)(kg * GP_ROWS) * GP_D + col;
  float S[GP_ROWS];
#pragma unroll
  for (int r = 0; r < GP_ROWS; r++) S[r] = Sp[(int64_t)r * GP_D];

  ScanIn cur, nxt;
  scan_load(cur, A, 0, h, kg, col);
  for (int t = 0; t < A.T; t++) {
    // the next token's operands are requested before this token's arithmetic (clamped: the last request is a repeat)
    scan_load(nxt, A, t + 1 < A.T ? t + 1 : t, h, kg, col);
    const float kr[GP_ROWS] = {cur.k[0].x, cur.k[0].y, cur.k[0].z, cur.k[0].w, cur.k[1].x, cur.k[1].y, cur.k[1].z, cur.k[1].w,
                               cur.k[2].x, cur.k[2].y, cur.k[2].z, cur.k[2].w, cur.k[3].x, cur.k[3].y, cur.k[3].z, cur.k[3].w};
    const float qr[GP_ROWS] = {cur.q[0].x, cur.q[0].y, cur.q[0].z, cur.q[0].w, cur.q[1].x, cur.q[1].y, cur.q[1].z, cur.q[1].w,
                               cur.q[2].x, cur.q[2].y, cur.q[2].z, cur.q[2].w, cur.q[3].x, cur.q[3].y, cur.q[3].z, cur.q[3].w};
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < GP_ROWS; r++) {
      S[r] *= cur.decay;
      acc = fmaf(kr[r], S[r], acc);
    }
    part_k[kg][c] = acc;
    __syncthreads();
    float kS = 0.f;
#pragma unroll
    for (int j = 0; j < GP_KG; j++) kS += part_k[j][c];
    const float d = (cur.v - kS) * cur.beta;
    acc = 0.f;
#pragma unroll
    for (int r = 0; r < GP_ROWS; r++) {
      S[r] = fmaf(kr[r], d, S[r]);
      acc = fmaf(qr[r], S[r], acc);
    }
    part_o[kg][c] = acc;
    __syncthreads();
    // part_k is rewritten only after the next token's first barrier has been passed by every thread, part_o only
    // after its second: two buffers, two barriers per token
    if (tid < GP_COLS) {
      float o = 0.f;
#pragma unroll
      for (int j = 0; j < GP_KG; j++) o += part_o[j][tid];
      A.o_raw[((int64_t)t * A.Hg + h) * GP_D + slab * GP_COLS + tid] = o;
    }
    cur = nxt;
  }
  float* So = A.S_out + (int64_t)h * GP_D * GP_D + (int64_t)(kg * GP_ROWS) * GP_D + col;
#pragma unroll
  for (int r = 0; r < GP_ROWS; r++) So[(int64_t)r * GP_D] = S[r];
}

__global__ __launch_bounds__(128) void gdn_prefill_outnorm_kernel(GdnPrefillArgs A) {
  __shared__ double red[2];
  const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x;
  const int64_t th = (int64_t)t * A.Hg + h;
  const float o = A.o_raw[th * GP_D + tid];
  const float zin = bf16_to_f32(A.z[th * GP_D + tid]);
  const double oss = wave_sum_f64((double)o * (double)o);
  if ((tid & 63) == 0) red[tid >> 6] = oss;
  __syncthreads();
  const float orstd = rsqrt_f64((red[0] + red[1]) / (double)GP_D + 1e-6);
  const float zs = zin * sigmoid_f64(zin);
  A.out[th * GP_D + tid] = f32_to_bf16(((o * orstd) * A.norm_w[tid]) * zs);
}

size_t gdn_prefill_workspace_bytes(int Hg, int T) {
  return (size_t)T * Hg * (2 * GP_D + GP_D + 2) * sizeof(float);
}

int launch_gdn_prefill(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                       const float* b_p, const float* norm_w, const float* S_in, void* out, float* S_out, void* workspace,
                       size_t workspace_bytes, int Hg, int T) {
  BK_REQUIRE(conv_out && z && A_log && dt_bias && a_p && b_p && norm_w && S_in && out && S_out && workspace, "gdn_prefill: null pointer");
  BK_REQUIRE(Hg > 0 && Hg <= 65535 && T > 0 && T <= 65535, "gdn_prefill: bad Hg=%d T=%d", Hg, T);
  BK_REQUIRE(workspace_bytes >= gdn_prefill_workspace_bytes(Hg, T), "gdn_prefill: workspace of %zu bytes, need %zu", workspace_bytes,
             gdn_prefill_workspace_bytes(Hg, T));
  BK_REQUIRE(((uintptr_t)workspace & 15) == 0, "gdn_prefill: workspace must be 16-byte aligned");
  GdnPrefillArgs A{};
  A.conv_out = (const uint16_t*)conv_out; A.z = (const uint16_t*)z; A.A_log = A_log; A.dt_bias = (const uint16_t*)dt_bias;
  A.a_p = a_p; A.b_p = b_p; A.norm_w = norm_w; A.S_in = S_in; A.S_out = S_out; A.out = (uint16_t*)out;
  A.qk = (float*)workspace;
  A.o_raw = A.qk + (size_t)T * Hg * 2 * GP_D;
  A.gates = A.o_raw + (size_t)T * Hg * GP_D;
  A.Hg = Hg; A.T = T;
  hipLaunchKernelGGL(gdn_prefill_prep_kernel, dim3(Hg, T), dim3(256), 0, stream(), A);
  hipLaunchKernelGGL(gdn_prefill_scan_kernel, dim3(Hg, GP_SLABS), dim3(256), 0, stream(), A);
  hipLaunchKernelGGL(gdn_prefill_outnorm_kernel, dim3(Hg, T), dim3(128), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
