// Gated DeltaNet over a run of T prompt tokens in the chunked form (the form of the reference's prefill prototypes:
// prototypes/gdn_fast.ts kernels kkt_fwd / solve_tril / recompute_w_u / fwd_h / fwd_o, prototypes/gdn_solve_tril.ts),
// as an alternative to the token-by-token scan of gdn_prefill.hip.  The recurrence
//     S_t = d_t S_{t-1} + k_t u_t^T,   u_t = beta_t (v_t - d_t S_{t-1}^T k_t),   o_t = S_t^T q_t
// is cut into chunks of 64 tokens.  With g_t the sum of log d over the chunk up to t and S_0 the state at its start:
//     (I + N) U = diag(beta) V - diag(beta e^g) K S_0,     N[t][j] = beta_t e^(g_t - g_j) (k_t . k_j)  for j < t
//     => U = Uv - W S_0,   T = (I + N)^-1,   Uv = T diag(beta) V,   W = T diag(beta e^g) K        (chunks in parallel)
//     S_C = e^(g_C) S_0 + K^T diag(e^(g_C - g)) U                                                 (chunk after chunk)
//     O = diag(e^g) Q S_0 + M U,   M[t][j] = e^(g_t - g_j) (q_t . k_j)  for j <= t               (chunks in parallel)
// Every product runs on the f32 matrix instruction (v_mfma_f32_32x32x2_f32: f32 operands, f32 sums), so the results
// differ from the scan's by the order of the additions only — about 1e-6 relative on the state — but not to the bit:
// the scan stays the default of the prompt path, this form is chosen with chunked=1.
// The reference multiplies in f16 (dot16, gdn_fast.ts:15); f32 operands are the tighter choice the hardware offers at
// the same instruction count.
#include "ops.h"

namespace bk {

typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int GC_C = 64;       // tokens per chunk
constexpr int GC_D = 128;      // key and value width of a head
constexpr int GC_LD = GC_D + 1;   // row stride of the [64][128] operands in LDS: the 32 rows of an operand read fall into different banks

struct GdnChunkArgs {
  const uint16_t* conv_out;   // bf16 [T, 3*Hg*128]: q | k | v
  const float* A_log;         // f32 [Hg]
  const uint16_t* dt_bias;    // bf16 [Hg]
  const float* a_p;           // f32 [T, Hg]
  const float* qk;            // f32 [T, Hg, 2, 128]: q^ (scaled), k^   (gdn_prefill_prep_kernel)
  const float* gates;         // f32 [T, Hg, 2]: decay, beta
  const float* S_in;          // f32 [Hg, 128, 128]
  float* S_out;
  float* G;                   // f32 [Hg, nC, 64]: sum of log decay from the chunk's first token
  float* W;                   // f32 [Hg, nC, 64, 128]
  float* U;                   // f32 [Hg, nC, 64, 128]: Uv, replaced by U as the states pass
  float* Hs;                  // f32 [Hg, nC, 128, 128]: the state at the start of every chunk
  float* o_raw;               // f32 [T, Hg, 128]
  int Hg, T, nC;
};

// row of the 32x32 result held in register r of a lane in half `half` of the wave (its column is lane % 32)
__device__ __forceinline__ int mrow(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

__device__ __forceinline__ f32x16_t zero16() {
  f32x16_t z;
#pragma unroll
  for (int r = 0; r < 16; r++) z[r] = 0.0f;
  return z;
}

// acc += sum over STEPS steps of A-operand fa(step) x B-operand fb(step): the operands of 16 steps are fetched (from LDS,
// memory or registers, as fa / fb say) before the 16 matrix instructions of the 16 steps before them are issued, so a
// wave that has nothing else to run does not sit out an operand's latency in front of every instruction.
template <int STEPS, class FA, class FB>
__device__ __forceinline__ f32x16_t mfma_run(f32x16_t acc, FA fa, FB fb) {
  static_assert(STEPS % 16 == 0, "whole batches");
  float a[2][16], b[2][16];
#pragma unroll
  for (int i = 0; i < 16; i++) { a[0][i] = fa(i); b[0][i] = fb(i); }
#pragma unroll
  for (int bt = 0; bt < STEPS / 16; bt++) {
    if (bt + 1 < STEPS / 16) {
#pragma unroll
      for (int i = 0; i < 16; i++) { a[(bt + 1) & 1][i] = fa(16 * (bt + 1) + i); b[(bt + 1) & 1][i] = fb(16 * (bt + 1) + i); }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 16; i++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[bt & 1][i], b[bt & 1][i], acc, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  return acc;
}

// Rows of 128 f32 from memory (`stride` floats apart) straight into the padded rows of an LDS operand: lane l of a wave
// fills float l of a half row (lds_dma4), the waves of the workgroup take the half rows in turn.  Nothing
// waits here; the caller waits for its own requests (vmcnt) and then for the other waves' (barrier).
__device__ __forceinline__ void rows_to_lds(const float* src, int64_t stride, int row_last, float (*dst)[GC_LD], int wave, int lane) {
  const unsigned char* base = lds_opaque(dst);
  const float* lane_src = src + lane;
#pragma unroll
  for (int i = 0; i < GC_C * 2 / 4; i++) {
    const int piece = 4 * i + wave, hh = piece & 1;
    // (the row number passes through an empty statement: its address arithmetic — scalar, 64-bit — is then done
    // here, between two transfers, instead of for all 32 pieces ahead of the first, which runs out of scalar registers)
    int r = piece >> 1;
    asm volatile("" : "+s"(r));
    lds_dma4(lane_src + (int64_t)min(r, row_last) * stride + 64 * hh, base + ((piece >> 1) * GC_LD + 64 * hh) * 4);
  }
}
__device__ __forceinline__ void wait_own_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }      // vmcnt(0)
// ---- kernel 1, per (head, chunk): g, T = (I + N)^-1, W, Uv
__global__ __launch_bounds__(256) void gdn_chunk_wu_kernel(GdnChunkArgs A) {
  __shared__ float Ks[GC_C][GC_LD], Vs[GC_C][GC_LD];
  __shared__ float Ns[GC_C][GC_C + 1], Ts[GC_C][GC_C + 1];
  __shared__ float g_s[GC_C], beta_s[GC_C], cw_s[GC_C];
  const int h = blockIdx.x, c = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5,
            col = lane & 31;
  const int t0 = c * GC_C, KEYDIM = A.Hg * GC_D;
  // k^ of the chunk's tokens (rows past the run repeat the last token: beta = 0 keeps them out of every sum); v as f32
  const int last = min(GC_C, A.T - t0) - 1;
  rows_to_lds(A.qk + (((int64_t)t0 * A.Hg + h) * 2 + 1) * GC_D, (int64_t)A.Hg * 2 * GC_D, last, Ks, wave, lane);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int e = tid + 256 * i, tt = e >> 4, i8 = (e & 15) * 8;
    const uint4 raw = *(const uint4*)(A.conv_out + (int64_t)(t0 + min(tt, last)) * 3 * KEYDIM + 2 * KEYDIM + h * GC_D + i8);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int q = 0; q < 4; q++) {
      Vs[tt][i8 + 2 * q] = __uint_as_float(w[q] << 16);
      Vs[tt][i8 + 2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u);
    }
  }
  if (tid < GC_C) {
    const int t = t0 + tid;
    const bool valid = t < A.T;
    const int64_t th = (int64_t)min(t, A.T - 1) * A.Hg + h;
    // log of the decay, as gdn_prefill_prep_kernel forms the decay itself; a token past the run leaves the state alone
    const float sp_in = A.a_p[th] + bf16_to_f32(A.dt_bias[h]);
    const float softplus = (float)log1p(exp((double)sp_in));
    float g = valid ? -((float)exp((double)A.A_log[h]) * softplus) : 0.0f;
    const float beta = valid ? A.gates[th * 2 + 1] : 0.0f;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float up = __shfl_up(g, off);
      if (lane >= off) g += up;
    }
    g_s[tid] = g; beta_s[tid] = beta; cw_s[tid] = beta * expf(g);
    A.G[((int64_t)h * A.nC + c) * GC_C + tid] = g;
  }
  wait_own_loads();
  __syncthreads();
  // K K^T: wave w owns tile (w / 2, w % 2); tile (0, 1) lies above the diagonal
  {
    const int ti = wave >> 1, tj = wave & 1;
    f32x16_t acc = zero16();
    if (wave != 1)
      acc = mfma_run<GC_D / 2>(acc, [&](int s) { return Ks[32 * ti + col][2 * s + half]; }, [&](int s) { return Ks[32 * tj + col][2 * s + half]; });
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int t = 32 * ti + mrow(r, half), j = 32 * tj + col;
      Ns[t][j] = j < t ? beta_s[t] * expf(g_s[t] - g_s[j]) * acc[r] : 0.0f;
    }
  }
  __syncthreads();
  // T = (I + N)^-1 in two levels.  Waves 0 and 1 invert the diagonal 32x32 blocks by forward substitution (lane =
  // column, row i needs rows 0 .. i-1); the block under the diagonal is then T21 = -T22 (N21 T11), two matrix products.
  if (wave < 2) {
    const int o32 = 32 * wave;
    float Tr[32];
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const float nrow = Ns[o32 + i][o32 + col];
      float a = col == i ? 1.0f : 0.0f;
#pragma unroll
      for (int j = 0; j < i; j++) a -= __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(nrow), j)) * Tr[j];
      Tr[i] = a;
      if (half == 0) { Ts[o32 + i][o32 + col] = a; if (wave == 0) Ts[i][32 + col] = 0.0f; }
    }
  }
  __syncthreads();
  if (wave == 0) {
    f32x16_t X = mfma_run<16>(zero16(), [&](int s) { return Ns[32 + col][2 * s + half]; }, [&](int s) { return Ts[2 * s + half][col]; });
    // X = N21 T11 takes N21's place (this wave is its only reader), then T21 = -(T22 X)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < 16; r++) Ns[32 + mrow(r, half)][col] = X[r];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x16_t Y = mfma_run<16>(zero16(), [&](int s) { return Ts[32 + col][32 + 2 * s + half]; }, [&](int s) { return Ns[32 + 2 * s + half][col]; });
#pragma unroll
    for (int r = 0; r < 16; r++) Ts[32 + mrow(r, half)][col] = -Y[r];
  }
  __syncthreads();
  // W = T diag(beta e^g) K and Uv = T diag(beta) V: wave w owns the 32 columns 32 w .. of both, T's zeros above the diagonal skipped
  const int64_t hc = (int64_t)h * A.nC + c;
#pragma unroll
  for (int which = 0; which < 2; which++)
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
      const float (*B)[GC_LD] = which ? Vs : Ks;
      const float* coef = which ? beta_s : cw_s;
      auto fa = [&](int s) { const int j = 2 * s + half; return Ts[32 * tt + col][j] * coef[j]; };
      auto fb = [&](int s) { return B[2 * s + half][32 * wave + col]; };
      const f32x16_t acc = tt ? mfma_run<32>(zero16(), fa, fb) : mfma_run<16>(zero16(), fa, fb);
      float* dst = (which ? A.U : A.W) + (hc * GC_C + 32 * tt) * GC_D + 32 * wave + col;
#pragma unroll
      for (int r = 0; r < 16; r++) dst[(int64_t)mrow(r, half) * GC_D] = acc[r];
    }
}

// ---- kernel 2, per (head, slab of 32 value columns): the states, chunk after chunk.  Wave w keeps rows 32 w .. + 32
// of the slab in the accumulators of one 32x32 tile.  W and k^ of a chunk arrive in LDS while the chunk before is worked
// on: k^ in one of two buffers, requested a whole chunk ahead; W in its single buffer as soon as the last reader of the
// previous W is done.
__global__ __launch_bounds__(256) void gdn_chunk_state_kernel(GdnChunkArgs A) {
  __shared__ float Wc[GC_C][GC_LD], Kc[2][GC_C][GC_LD];
  __shared__ float red[4][GC_C][33];
  __shared__ float Ut[GC_C][33];
  __shared__ float g_s[2][GC_C];
  const int h = blockIdx.x, sl = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5,
            col = lane & 31;
  const int64_t kstride = (int64_t)A.Hg * 2 * GC_D;
  auto k_rows = [&](int c) { return A.qk + (((int64_t)c * GC_C * A.Hg + h) * 2 + 1) * GC_D; };
  auto last_row = [&](int c) { return min(GC_C, A.T - c * GC_C) - 1; };
  f32x16_t S;
  {
    const float* Si = A.S_in + (int64_t)h * GC_D * GC_D + 32 * sl + col;
#pragma unroll
    for (int r = 0; r < 16; r++) S[r] = Si[(int64_t)(32 * wave + mrow(r, half)) * GC_D];
  }
  rows_to_lds(A.W + (int64_t)h * A.nC * GC_C * GC_D, GC_D, GC_C - 1, Wc, wave, lane);
  rows_to_lds(k_rows(0), kstride, last_row(0), Kc[0], wave, lane);
  if (tid < GC_C) g_s[0][tid] = A.G[(int64_t)h * A.nC * GC_C + tid];
  wait_own_loads();
  for (int c = 0; c < A.nC; c++) {
    const int64_t hc = (int64_t)h * A.nC + c;
    __syncthreads();                                   // W, k^ and g of this chunk are in LDS; the previous chunk's readers are done
    // requests of this step, oldest first: k^ of the next chunk, its g, this chunk's Uv (used after the first product)
    const bool more = c + 1 < A.nC;
    if (more) rows_to_lds(k_rows(c + 1), kstride, last_row(c + 1), Kc[(c + 1) & 1], wave, lane);
    const float gnext = A.G[(hc + (more ? 1 : 0)) * GC_C + (tid & 63)];
    float uv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int e = tid + 256 * i;
      uv[i] = A.U[(hc * GC_C + (e >> 5)) * GC_D + 32 * sl + (e & 31)];
    }
    {
      float* Ho = A.Hs + hc * GC_D * GC_D + 32 * sl + col;
#pragma unroll
      for (int r = 0; r < 16; r++) Ho[(int64_t)(32 * wave + mrow(r, half)) * GC_D] = S[r];
    }
    // this wave's share of W S: the sum over its 32 rows of S, taken in the order the accumulator holds them
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
      const f32x16_t P = mfma_run<16>(zero16(), [&](int r) { return Wc[32 * tt + col][32 * wave + mrow(r, half)]; }, [&](int r) { return S[r]; });
#pragma unroll
      for (int r = 0; r < 16; r++) red[wave][32 * tt + mrow(r, half)][col] = P[r];
    }
    __syncthreads();
    if (more) rows_to_lds(A.W + (hc + 1) * GC_C * GC_D, GC_D, GC_C - 1, Wc, wave, lane);
    const float* gc = g_s[c & 1];
    const float gC = gc[GC_C - 1];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int e = tid + 256 * i, t = e >> 5, n = e & 31;
      const float u = uv[i] - (((red[0][t][n] + red[1][t][n]) + red[2][t][n]) + red[3][t][n]);
      Ut[t][n] = u * expf(gC - gc[t]);
      A.U[(hc * GC_C + t) * GC_D + 32 * sl + n] = u;
    }
    if (tid < GC_C) g_s[(c + 1) & 1][tid] = gnext;
    __syncthreads();
    const float dC = expf(gC);
#pragma unroll
    for (int r = 0; r < 16; r++) S[r] *= dC;
    const float (*Kcur)[GC_LD] = Kc[c & 1];
    S = mfma_run<GC_C / 2>(S, [&](int s) { return Kcur[2 * s + half][32 * wave + col]; }, [&](int s) { return Ut[2 * s + half][col]; });
    // the 8 stores of U are the youngest requests of this wave; everything older — the next chunk's W and k^ among
    // it — has to be in LDS before the barrier at the top, the stores may stay in flight
    __builtin_amdgcn_s_waitcnt(0x0F70 | 8);            // vmcnt(8)
  }
  float* So = A.S_out + (int64_t)h * GC_D * GC_D + 32 * sl + col;
#pragma unroll
  for (int r = 0; r < 16; r++) So[(int64_t)(32 * wave + mrow(r, half)) * GC_D] = S[r];
}

// ---- kernel 3, per (head, chunk): the outputs
__global__ __launch_bounds__(256) void gdn_chunk_out_kernel(GdnChunkArgs A) {
  __shared__ float Qs[GC_C][GC_LD], Ks[GC_C][GC_LD], Us[GC_C][GC_LD];
  __shared__ float Ms[GC_C][GC_C + 1];
  __shared__ float g_s[GC_C];
  const int h = blockIdx.x, c = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5,
            col = lane & 31;
  const int t0 = c * GC_C;
  const int64_t hc = (int64_t)h * A.nC + c;
  {
    // (rows past the run repeat the last token; their U rows are zero and their outputs are not stored)
    const int last = min(GC_C, A.T - t0) - 1;
    const float* qk = A.qk + ((int64_t)t0 * A.Hg + h) * 2 * GC_D;
    rows_to_lds(qk, (int64_t)A.Hg * 2 * GC_D, last, Qs, wave, lane);
    rows_to_lds(qk + GC_D, (int64_t)A.Hg * 2 * GC_D, last, Ks, wave, lane);
    rows_to_lds(A.U + hc * GC_C * GC_D, GC_D, GC_C - 1, Us, wave, lane);
  }
  if (tid < GC_C) g_s[tid] = A.G[hc * GC_C + tid];
  wait_own_loads();
  __syncthreads();
  {
    const int ti = wave >> 1, tj = wave & 1;
    f32x16_t acc = zero16();
    if (wave != 1)
      acc = mfma_run<GC_D / 2>(acc, [&](int s) { return Qs[32 * ti + col][2 * s + half]; }, [&](int s) { return Ks[32 * tj + col][2 * s + half]; });
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int t = 32 * ti + mrow(r, half), j = 32 * tj + col;
      Ms[t][j] = j <= t ? expf(g_s[t] - g_s[j]) * acc[r] : 0.0f;
    }
  }
  __syncthreads();
  // wave w owns value columns 32 w .. + 32: diag(e^g) Q S_0, the state read straight from memory as the B operand
  // (mfma_run keeps a lane's loads 16 ahead of the instructions that use them), then M U
  const float* Hc = A.Hs + hc * GC_D * GC_D + 32 * wave + col;
#pragma unroll
  for (int tt = 0; tt < 2; tt++) {
    f32x16_t acc = mfma_run<GC_D / 2>(zero16(), [&](int s) { return Qs[32 * tt + col][2 * s + half]; },
                                      [&](int s) { return Hc[(int64_t)(2 * s + half) * GC_D]; });
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] *= expf(g_s[32 * tt + mrow(r, half)]);
    {
      auto fa = [&](int s) { return Ms[32 * tt + col][2 * s + half]; };
      auto fb = [&](int s) { return Us[2 * s + half][32 * wave + col]; };
      acc = tt ? mfma_run<32>(acc, fa, fb) : mfma_run<16>(acc, fa, fb);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int t = t0 + 32 * tt + mrow(r, half);
      if (t < A.T) A.o_raw[((int64_t)t * A.Hg + h) * GC_D + 32 * wave + col] = acc[r];
    }
  }
}

size_t gdn_chunk_workspace_bytes(int Hg, int T) {
  const size_t nC = (size_t)(T + GC_C - 1) / GC_C;
  return (size_t)Hg * nC * (GC_C + 2 * GC_C * GC_D + GC_D * GC_D) * sizeof(float);
}

// Called by launch_gdn_prefill after its preparation kernel and before its output norm; `workspace` is this form's own.
int launch_gdn_chunked_core(const void* conv_out, const float* A_log, const void* dt_bias, const float* a_p, const float* qk, const float* gates,
                            const float* S_in, float* S_out, float* o_raw, void* workspace, size_t workspace_bytes, int Hg, int T) {
  BK_REQUIRE(workspace && workspace_bytes >= gdn_chunk_workspace_bytes(Hg, T), "gdn_prefill (chunked): workspace of %zu bytes, need %zu",
             workspace_bytes, gdn_chunk_workspace_bytes(Hg, T));
  GdnChunkArgs A{};
  A.conv_out = (const uint16_t*)conv_out; A.A_log = A_log; A.dt_bias = (const uint16_t*)dt_bias; A.a_p = a_p; A.qk = qk; A.gates = gates;
  A.S_in = S_in; A.S_out = S_out; A.o_raw = o_raw; A.Hg = Hg; A.T = T; A.nC = (T + GC_C - 1) / GC_C;
  BK_REQUIRE(A.nC <= 65535, "gdn_prefill (chunked): T=%d is too long for one launch", T);
  const size_t per = (size_t)Hg * A.nC;
  A.G = (float*)workspace;
  A.W = A.G + per * GC_C;
  A.U = A.W + per * GC_C * GC_D;
  A.Hs = A.U + per * GC_C * GC_D;
  hipLaunchKernelGGL(gdn_chunk_wu_kernel, dim3(Hg, A.nC), dim3(256), 0, stream(), A);
  hipLaunchKernelGGL(gdn_chunk_state_kernel, dim3(Hg, GC_D / 32), dim3(256), 0, stream(), A);
  hipLaunchKernelGGL(gdn_chunk_out_kernel, dim3(Hg, A.nC), dim3(256), 0, stream(), A);
  return BK_OK;
}

}  // namespace bk
