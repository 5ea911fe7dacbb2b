// Gated DeltaNet single-token recurrent update (src/emitters.ts:75-120,
// prototypes/decode.ts:314-388; recurrence of prototypes/gdn_gated.ts:67-88).
//
//   Sd = g*S ; kS[v] = sum_k k^[k]*Sd[k,v] ; delta = (v - kS)*beta
//   S' = Sd + k^ (x) delta ; o[v] = sum_k q^[k]*S'[k,v]
//
// S is f32 [B, Hg, 128(k), 128(v)], row-major.  Every v column is independent, so a
// head is cut into CS column slabs, one 256-thread workgroup each.  A thread owns
// ROWS k-rows x 4 v-columns of the slab in registers for the whole step: S is read
// from HBM once (float4, rows of the slab contiguous) and S' written once; the two
// k-reductions are in-thread fmaf chains over the owned rows plus one LDS exchange
// across the row groups, summed in group order.  With the whole head in one workgroup
// (CS = 1) that is "chains of 16 consecutive rows, then the 8 chain results in order",
// the order the CPU checker follows; norms and gates are evaluated in double.
#include "ops.h"

namespace bk {

constexpr int GDN_D = 128;          // dk = dv = 128
constexpr int GDN_THREADS = 256;
typedef __attribute__((ext_vector_type(4))) float f32x4_nt;

struct GdnArgs {
  // q, k, v: bf16, element (b, h, i) at ptr[b*bstride + h*128 + i]
  const uint16_t *q, *k, *v;
  int64_t qkv_bstride;
  // fused mode (src/emitters.ts:86-99): decay and beta from A_log, dt_bias, a_p, b_p; gated RMSNorm with z, norm_w
  const uint16_t* z;        // bf16 [B, Hg*128]
  const float* A_log;       // f32 [Hg]
  const uint16_t* dt_bias;  // bf16 [Hg]
  const float* a_p;         // f32 [B, Hg]
  const float* b_p;         // f32 [B, Hg]
  const float* norm_w;      // f32 [128]
  // core mode: decay = exp(g), beta given; q, k used as they are
  const float* g;           // f32 [B, Hg]
  const float* beta;        // f32 [B, Hg]
  const float* S_in;
  float* S_out;
  uint16_t* out;            // bf16 [B, Hg*128]
  uint8_t* out_q8;          // optional: the same outputs as Q8_1 blocks [B, Hg*128/32] for the matmul that follows
  int Hg;
  // conv mode (src/emitters.ts:48-72 folded in): q, k, v above point into the raw qkv projection and every
  // channel first goes through the 4-tap causal convolution + SiLU; its state rows are shifted in the same pass
  const uint16_t* conv_st;  // bf16 [B, 3, C]
  const uint16_t* conv_w;   // bf16 [C, 4]
  uint16_t* conv_st_new;    // bf16 [B, 3, C], may alias conv_st
  int C;
};

// One channel of conv1d_decode: r = (w0*s0 + w1*s1) + (w2*s2 + w3*x); out = bf16(r * sigmoid(r)), new state rows
// (s1, s2, x).  Loading and computing are separate so that a kernel can request everything it needs first.
struct ConvIn {
  uint16_t x, s0, s1, s2;
  uint2 w;
};
__device__ __forceinline__ ConvIn conv_load(const GdnArgs& A, int b, int ch, const uint16_t* xrow) {
  const uint16_t* sb = A.conv_st + (int64_t)b * 3 * A.C;
  ConvIn c;
  c.x = xrow[ch]; c.s0 = sb[ch]; c.s1 = sb[A.C + ch]; c.s2 = sb[2 * A.C + ch];
  c.w = *(const uint2*)(A.conv_w + 4 * (int64_t)ch);
  return c;
}
// The thread that read a channel's rows is the one that rewrites them, so the state may be updated in place.
__device__ __forceinline__ uint16_t conv_apply(const GdnArgs& A, int b, int ch, const ConvIn& c) {
  const float w0 = __uint_as_float(c.w.x << 16), w1 = __uint_as_float(c.w.x & 0xffff0000u);
  const float w2 = __uint_as_float(c.w.y << 16), w3 = __uint_as_float(c.w.y & 0xffff0000u);
  // products of two bf16 values are exact in f32
  const float r = __fadd_rn(__fadd_rn(w0 * bf16_to_f32(c.s0), w1 * bf16_to_f32(c.s1)),
                            __fadd_rn(w2 * bf16_to_f32(c.s2), w3 * bf16_to_f32(c.x)));
  uint16_t* nb = A.conv_st_new + (int64_t)b * 3 * A.C;
  nb[ch] = c.s1; nb[A.C + ch] = c.s2; nb[2 * A.C + ch] = c.x;
  return f32_to_bf16(__fmul_rn(r, sigmoid_f64(r)));
}

template <int CS, bool FUSED, bool CONV = false, bool NT = false>
__global__ __launch_bounds__(GDN_THREADS) void gdn_step_kernel(GdnArgs A) {
  static_assert(!CONV || FUSED, "the convolution is part of the fused op only");
  constexpr int COLS = GDN_D / CS;          // v columns of this workgroup
  constexpr int VQ = COLS / 4;              // float4 column groups
  constexpr int KG = GDN_THREADS / VQ;      // k-row groups
  constexpr int ROWS = GDN_D / KG;          // rows per thread
  static_assert(!FUSED || CS == 1, "the gated norm needs the whole head in one workgroup");
  __shared__ float kn[GDN_D], qn[GDN_D];
  __shared__ float part[KG][COLS];
  __shared__ double red[4];
  __shared__ __align__(8) uint16_t vsh[CONV ? GDN_D : 4];

  const int h = blockIdx.x, slab = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x;
  const int vq = tid % VQ, kg = tid / VQ;
  const int col0 = slab * COLS + vq * 4;    // first of the thread's 4 columns (within the head)
  const int64_t bh = (int64_t)b * A.Hg + h;

  const uint16_t* qp = A.q + (int64_t)b * A.qkv_bstride + h * GDN_D;
  const uint16_t* kp = A.k + (int64_t)b * A.qkv_bstride + h * GDN_D;
  const uint16_t* vp = A.v + (int64_t)b * A.qkv_bstride + h * GDN_D;
  const uint16_t* xrow = A.q + (int64_t)b * A.qkv_bstride;
  const bool isk = tid >= 128;              // fused mode: threads 0..127 hold q, 128..255 hold k
  const int i = tid & 127;

  // Loads come back in the order they were issued.  The small operands (q, k, v, the conv taps and state, the gate
  // inputs) are requested first and the 64 KiB of S right behind them: the norms and gates are then computed while
  // S is still on its way from HBM.
  ConvIn cqk{}, cv{};
  uint16_t xbits = 0;
  uint2 vv_g = make_uint2(0, 0);
  float zin = 0.0f, nw = 0.0f, ap = 0.0f, bp = 0.0f, alog = 0.0f, dtb = 0.0f;
  const int ch_qk = (int)((isk ? kp : qp) - xrow) + i, ch_v = (int)(vp - xrow) + i;
  if (FUSED) {
    if (CONV) {
      cqk = conv_load(A, b, ch_qk, xrow);
      cv = conv_load(A, b, ch_v, xrow);      // every thread loads (no branch around loads: waits stay countable); q threads use it
    } else {
      xbits = (isk ? kp : qp)[i];
    }
    ap = A.a_p[bh]; bp = A.b_p[bh]; alog = A.A_log[h]; dtb = bf16_to_f32(A.dt_bias[h]);
    zin = bf16_to_f32(A.z[bh * GDN_D + i]); nw = A.norm_w[i];
  } else {
    xbits = tid < 128 ? qp[tid] : kp[tid - 128];
  }
  if (!CONV) vv_g = *(const uint2*)(vp + col0);

  const float* Sp = A.S_in + bh * GDN_D * GDN_D;
  float4 S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    const f32x4_nt* sp = (const f32x4_nt*)(Sp + (int64_t)(kg * ROWS + r) * GDN_D + col0);
    const f32x4_nt t = NT ? __builtin_nontemporal_load(sp) : *sp;
    S[r] = make_float4(t[0], t[1], t[2], t[3]);
  }

  float decay, beta, zs = 0.0f;     // zs: the output gate z * sigmoid(z), evaluated while S is still on its way
  if (FUSED) {
    float x;
    if (CONV) {
      x = bf16_to_f32(conv_apply(A, b, ch_qk, cqk));
      if (!isk) vsh[i] = conv_apply(A, b, ch_v, cv);
    } else {
      x = bf16_to_f32(xbits);
    }
    const double ss = wave_sum_f64((double)(x * x));       // square of a bf16 value: exact in f32
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const double tot = isk ? (red[2] + red[3]) : (red[0] + red[1]);
    const float rs = rsqrt_f64(tot + 1e-6);
    if (isk) kn[i] = x * rs;
    else qn[i] = x * (rs * 0.08838834764831845f);     // 1/sqrt(128)
    const float sp_in = ap + dtb;
    const float softplus = (float)log1p(exp((double)sp_in));
    decay = (float)exp(-(double)((float)exp((double)alog) * softplus));
    beta = sigmoid_f64(bp);
    zs = zin * sigmoid_f64(zin);
  } else {
    if (tid < 128) qn[tid] = bf16_to_f32(xbits);
    else kn[tid - 128] = bf16_to_f32(xbits);
    decay = (float)exp((double)A.g[bh]);
    beta = A.beta[bh];
  }
  __syncthreads();

  float kr[ROWS], qr[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; r++) { kr[r] = kn[kg * ROWS + r]; qr[r] = qn[kg * ROWS + r]; }

  // decay, then the thread's share of kS
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    S[r].x *= decay; S[r].y *= decay; S[r].z *= decay; S[r].w *= decay;
    acc.x = fmaf(kr[r], S[r].x, acc.x); acc.y = fmaf(kr[r], S[r].y, acc.y);
    acc.z = fmaf(kr[r], S[r].z, acc.z); acc.w = fmaf(kr[r], S[r].w, acc.w);
  }
  *(float4*)&part[kg][vq * 4] = acc;
  __syncthreads();
  // all partials are requested before the first is added (the fence keeps the compiler from pairing every LDS read
  // with its use, which would expose the LDS latency KG times); the sum keeps its order
  float4 pk[KG];
#pragma unroll
  for (int j = 0; j < KG; j++) pk[j] = *(const float4*)&part[j][vq * 4];
  __builtin_amdgcn_sched_barrier(0);
  float4 kS = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int j = 0; j < KG; j++) { kS.x += pk[j].x; kS.y += pk[j].y; kS.z += pk[j].z; kS.w += pk[j].w; }
  __syncthreads();   // part is reused for o below
  const uint2 vv = CONV ? *(const uint2*)(vsh + col0) : vv_g;
  float4 d;
  d.x = (__uint_as_float(vv.x << 16) - kS.x) * beta;
  d.y = (__uint_as_float(vv.x & 0xffff0000u) - kS.y) * beta;
  d.z = (__uint_as_float(vv.y << 16) - kS.z) * beta;
  d.w = (__uint_as_float(vv.y & 0xffff0000u) - kS.w) * beta;

  float* So = A.S_out + bh * GDN_D * GDN_D;
  acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    S[r].x = fmaf(kr[r], d.x, S[r].x); S[r].y = fmaf(kr[r], d.y, S[r].y);
    S[r].z = fmaf(kr[r], d.z, S[r].z); S[r].w = fmaf(kr[r], d.w, S[r].w);
    {
      f32x4_nt* sp = (f32x4_nt*)(So + (int64_t)(kg * ROWS + r) * GDN_D + col0);
      const f32x4_nt t = {S[r].x, S[r].y, S[r].z, S[r].w};
      if (NT) __builtin_nontemporal_store(t, sp); else *sp = t;
    }
    acc.x = fmaf(qr[r], S[r].x, acc.x); acc.y = fmaf(qr[r], S[r].y, acc.y);
    acc.z = fmaf(qr[r], S[r].z, acc.z); acc.w = fmaf(qr[r], S[r].w, acc.w);
  }
  *(float4*)&part[kg][vq * 4] = acc;
  __syncthreads();

  // o[v] for the slab: thread t < COLS sums column t over the row groups
  float o = 0.0f;
  if (tid < COLS) {
#pragma unroll
    for (int j = 0; j < KG; j++) o += part[j][tid];
  }
  uint16_t* outp = A.out + bh * GDN_D + slab * COLS;
  if (!FUSED) {
    if (tid < COLS) outp[tid] = f32_to_bf16(o);
    return;
  }
  // gated RMSNorm over the 128 outputs of the head (threads 0..127 = waves 0, 1)
  const double oss = wave_sum_f64((double)o * (double)o);
  if ((tid & 63) == 0) red[tid >> 6] = oss;
  __syncthreads();
  if (tid < GDN_D) {
    const float orstd = rsqrt_f64((red[0] + red[1]) / (double)GDN_D + 1e-6);
    const uint16_t ob = f32_to_bf16(((o * orstd) * nw) * zs);
    outp[tid] = ob;
    if (A.out_q8) lane32_q8_1_store(bf16_to_f32(ob), A.out_q8 + (bh * (GDN_D / 32) + (tid >> 5)) * 36, tid & 31);
  }
}

// Column-slab form of the fused step for few (sequence, head) pairs, where one 256-thread workgroup per head leaves most
// of the chip idle and its one CU fetches all 64 KiB of the head's state: a head is cut into four slabs of 32 columns,
// one wavefront each.  Lane (kg = lane / 8, vq = lane % 8) owns rows 16 kg .. 16 kg + 15 and four columns of the slab,
// so both k-reductions keep the canonical order (fmaf chains over 16 consecutive rows, then the 8 chain results in
// order) and S' and o have the bits of the one-workgroup form.  Every slab works out the head's norms and gates itself
// (the inputs are convolved already: the projection in front of this launch applies conv1d in its last step).  What needs
// the whole head - the gated RMS norm - moves into the matmul behind it: a slab leaves its 32 raw outputs o (f32), the
// output gate z * sigmoid(z) (f32) and the sum of o^2 over its columns (f64) in `raw`:
//   raw, per sequence: f32 o[Hg * 128] | f32 zs[Hg * 128] | f64 ssq[Hg][4]
struct GdnRawLayout {
  int Hg;
  __host__ __device__ size_t floats() const { return (size_t)Hg * GDN_D * 2; }
  __host__ __device__ size_t bytes() const { return floats() * 4 + (size_t)Hg * 4 * 8; }
};
// The slab kernel's own argument block: 76 bytes, two 64-byte lines of kernel arguments instead of the three of GdnArgs
// (a launch of a few microseconds pays about a quarter of a microsecond per line).
struct GdnSlabArgs {
  const uint16_t* conv_out;   // bf16 [B, 3 * Hg * 128]: q | k | v after conv1d
  const uint16_t* z;
  const float* A_log;
  const uint16_t* dt_bias;
  const float* a_p;
  const float* b_p;
  const float* S_in;
  float* S_out;
  uint8_t* raw;
  int Hg;
};
template <bool NT>
__global__ __launch_bounds__(64) void gdn_slab_kernel(GdnSlabArgs A) {
  uint8_t* __restrict__ raw_base = A.raw;
  constexpr int CS = 4, COLS = GDN_D / CS, KG = 8, ROWS = 16;
  __shared__ float kn[GDN_D], qn[GDN_D];
  __shared__ float part[KG][COLS];
  const int h = blockIdx.x, slab = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
  const int vq = lane & 7, kg = lane >> 3;
  const int col0 = slab * COLS + vq * 4;
  const int64_t bh = (int64_t)b * A.Hg + h;
  const int keydim = A.Hg * GDN_D;
  const uint16_t* qp = A.conv_out + (int64_t)b * 3 * keydim + h * GDN_D;
  const uint16_t* kp = qp + keydim;
  const uint16_t* vp = kp + keydim;

  // small operands first, the 16 KiB of S right behind them (loads return in order)
  const uint32_t q2 = *(const uint32_t*)(qp + 2 * lane), k2 = *(const uint32_t*)(kp + 2 * lane);
  const uint2 vv = *(const uint2*)(vp + col0);
  const float ap = A.a_p[bh], bp = A.b_p[bh], alog = A.A_log[h], dtb = bf16_to_f32(A.dt_bias[h]);
  const float zin = bf16_to_f32(A.z[bh * GDN_D + slab * COLS + (lane & 31)]);
  const float* Sp = A.S_in + bh * GDN_D * GDN_D;
  float4 S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    const f32x4_nt* sp = (const f32x4_nt*)(Sp + (int64_t)(kg * ROWS + r) * GDN_D + col0);
    const f32x4_nt t = NT ? __builtin_nontemporal_load(sp) : *sp;
    S[r] = make_float4(t[0], t[1], t[2], t[3]);
  }

  const float q0 = __uint_as_float(q2 << 16), q1 = __uint_as_float(q2 & 0xffff0000u);
  const float k0 = __uint_as_float(k2 << 16), k1 = __uint_as_float(k2 & 0xffff0000u);
  const double ssq = wave_sum_f64((double)(q0 * q0) + (double)(q1 * q1));      // squares of bf16 values: exact in f32
  const double ssk = wave_sum_f64((double)(k0 * k0) + (double)(k1 * k1));
  const float rq = rsqrt_f64(ssq + 1e-6) * 0.08838834764831845f, rk = rsqrt_f64(ssk + 1e-6);
  qn[2 * lane] = q0 * rq; qn[2 * lane + 1] = q1 * rq;
  kn[2 * lane] = k0 * rk; kn[2 * lane + 1] = k1 * rk;
  const float sp_in = ap + dtb;
  const float softplus = (float)log1p(exp((double)sp_in));
  const float decay = (float)exp(-(double)((float)exp((double)alog) * softplus));
  const float beta = sigmoid_f64(bp);
  const float zs = zin * sigmoid_f64(zin);
  __syncthreads();

  float kr[ROWS], qr[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; r++) { kr[r] = kn[kg * ROWS + r]; qr[r] = qn[kg * ROWS + r]; }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    S[r].x *= decay; S[r].y *= decay; S[r].z *= decay; S[r].w *= decay;
    acc.x = fmaf(kr[r], S[r].x, acc.x); acc.y = fmaf(kr[r], S[r].y, acc.y);
    acc.z = fmaf(kr[r], S[r].z, acc.z); acc.w = fmaf(kr[r], S[r].w, acc.w);
  }
  *(float4*)&part[kg][vq * 4] = acc;
  __syncthreads();
  float4 pk[KG];
#pragma unroll
  for (int j = 0; j < KG; j++) pk[j] = *(const float4*)&part[j][vq * 4];
  __builtin_amdgcn_sched_barrier(0);
  float4 kS = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int j = 0; j < KG; j++) { kS.x += pk[j].x; kS.y += pk[j].y; kS.z += pk[j].z; kS.w += pk[j].w; }
  __syncthreads();   // part is reused for o below
  float4 d;
  d.x = (__uint_as_float(vv.x << 16) - kS.x) * beta;
  d.y = (__uint_as_float(vv.x & 0xffff0000u) - kS.y) * beta;
  d.z = (__uint_as_float(vv.y << 16) - kS.z) * beta;
  d.w = (__uint_as_float(vv.y & 0xffff0000u) - kS.w) * beta;

  float* So = A.S_out + bh * GDN_D * GDN_D;
  acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    S[r].x = fmaf(kr[r], d.x, S[r].x); S[r].y = fmaf(kr[r], d.y, S[r].y);
    S[r].z = fmaf(kr[r], d.z, S[r].z); S[r].w = fmaf(kr[r], d.w, S[r].w);
    {
      f32x4_nt* sp = (f32x4_nt*)(So + (int64_t)(kg * ROWS + r) * GDN_D + col0);
      const f32x4_nt t = {S[r].x, S[r].y, S[r].z, S[r].w};
      if (NT) __builtin_nontemporal_store(t, sp); else *sp = t;
    }
    acc.x = fmaf(qr[r], S[r].x, acc.x); acc.y = fmaf(qr[r], S[r].y, acc.y);
    acc.z = fmaf(qr[r], S[r].z, acc.z); acc.w = fmaf(qr[r], S[r].w, acc.w);
  }
  *(float4*)&part[kg][vq * 4] = acc;
  __syncthreads();
  // lanes 0..31 and 32..63 both sum column lane % 32 (the same bits); the sum of squares then covers each column twice
  float o = 0.0f;
#pragma unroll
  for (int j = 0; j < KG; j++) o += part[j][lane & 31];
  const double oss = wave_sum_f64(lane < 32 ? (double)o * (double)o : 0.0);
  const GdnRawLayout L{A.Hg};
  float* rawf = (float*)(raw_base + (size_t)b * L.bytes());
  if (lane < 32) {
    rawf[h * GDN_D + slab * COLS + lane] = o;
    rawf[A.Hg * GDN_D + h * GDN_D + slab * COLS + lane] = zs;
  }
  if (lane == 0) ((double*)(rawf + L.floats()))[h * 4 + slab] = oss;
}

int g_tune_gdn_cs = 0;    // column slabs per head for the core entry point (0 = from the shape)
int g_tune_gdn_nt = -1;   // state through nontemporal loads and stores: 0 off, 1 on, -1 = from the shape

static int check_common(const GdnArgs& A, int batch) {
  BK_REQUIRE(A.q && A.k && A.v && A.S_in && A.S_out && A.out, "gdn_step: null pointer");
  BK_REQUIRE(A.Hg > 0 && A.Hg <= 65535 && batch > 0 && batch <= 65535, "gdn_step: bad Hg=%d batch=%d", A.Hg, batch);
  BK_REQUIRE(((uintptr_t)A.S_in & 15) == 0 && ((uintptr_t)A.S_out & 15) == 0, "gdn_step: S must be 16-byte aligned");
  BK_REQUIRE(((uintptr_t)A.v & 7) == 0 && (A.qkv_bstride % 4) == 0, "gdn_step: v must be 8-byte aligned");
  return BK_OK;
}

int launch_gdn_fused(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                     const float* b_p, const float* norm_w, const float* S_in, void* out, float* S_out, int Hg, int batch) {
  GdnArgs A{};
  const int KEYDIM = Hg * GDN_D;
  A.q = (const uint16_t*)conv_out; A.k = A.q + KEYDIM; A.v = A.q + 2 * KEYDIM;
  A.qkv_bstride = 3 * (int64_t)KEYDIM;
  A.z = (const uint16_t*)z; A.A_log = A_log; A.dt_bias = (const uint16_t*)dt_bias; A.a_p = a_p; A.b_p = b_p; A.norm_w = norm_w;
  A.S_in = S_in; A.S_out = S_out; A.out = (uint16_t*)out; A.Hg = Hg;
  BK_REQUIRE(conv_out && z && A_log && dt_bias && a_p && b_p && norm_w, "gdn_delta_rule: null pointer");
  int rc = check_common(A, batch);
  if (rc) return rc;
  hipLaunchKernelGGL((gdn_step_kernel<1, true>), dim3(Hg, 1, batch), dim3(GDN_THREADS), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

int launch_gdn_conv_fused(const void* qkv, const void* conv_st, const void* conv_w, const void* z, const float* A_log,
                          const void* dt_bias, const float* a_p, const float* b_p, const float* norm_w, const float* S_in,
                          void* out, void* conv_st_new, float* S_out, void* out_q8, int Hg, int batch) {
  GdnArgs A{};
  A.out_q8 = (uint8_t*)out_q8;
  const int KEYDIM = Hg * GDN_D;
  A.q = (const uint16_t*)qkv; A.k = A.q + KEYDIM; A.v = A.q + 2 * KEYDIM;
  A.qkv_bstride = 3 * (int64_t)KEYDIM;
  A.z = (const uint16_t*)z; A.A_log = A_log; A.dt_bias = (const uint16_t*)dt_bias; A.a_p = a_p; A.b_p = b_p; A.norm_w = norm_w;
  A.S_in = S_in; A.S_out = S_out; A.out = (uint16_t*)out; A.Hg = Hg;
  A.conv_st = (const uint16_t*)conv_st; A.conv_w = (const uint16_t*)conv_w; A.conv_st_new = (uint16_t*)conv_st_new; A.C = 3 * KEYDIM;
  BK_REQUIRE(qkv && z && A_log && dt_bias && a_p && b_p && norm_w && conv_st && conv_w && conv_st_new, "gdn_conv: null pointer");
  BK_REQUIRE(((uintptr_t)conv_w & 7) == 0, "gdn_conv: the conv weight must be 8-byte aligned");
  int rc = check_common(A, batch);
  if (rc) return rc;
  // 128 (sequence, head) pairs move 16 MB of state per layer: over the layers of a model that is more than the 256 MB
  // memory-side cache holds until the next token, so the state bypasses the caches (+6 % tok/s at batch 32); smaller
  // batches find their state still cached one token later and keep the plain accesses
  const bool nt = g_tune_gdn_nt >= 0 ? g_tune_gdn_nt != 0 : (int64_t)Hg * batch >= 128;
  if (nt) hipLaunchKernelGGL((gdn_step_kernel<1, true, true, true>), dim3(Hg, 1, batch), dim3(GDN_THREADS), 0, stream(), A);
  else hipLaunchKernelGGL((gdn_step_kernel<1, true, true, false>), dim3(Hg, 1, batch), dim3(GDN_THREADS), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

size_t gdn_raw_bytes(int Hg, int batch) { return GdnRawLayout{Hg}.bytes() * (size_t)batch; }

// gdn_delta_rule without its gated norm, in column slabs (see gdn_slab_kernel): conv_out is [q | k | v] bf16 after conv1d
int launch_gdn_slabs(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                     const float* b_p, const float* S_in, void* raw, float* S_out, int Hg, int batch) {
  GdnArgs A{};
  const int KEYDIM = Hg * GDN_D;
  A.q = (const uint16_t*)conv_out; A.k = A.q + KEYDIM; A.v = A.q + 2 * KEYDIM;
  A.qkv_bstride = 3 * (int64_t)KEYDIM;
  A.z = (const uint16_t*)z; A.A_log = A_log; A.dt_bias = (const uint16_t*)dt_bias; A.a_p = a_p; A.b_p = b_p;
  A.S_in = S_in; A.S_out = S_out; A.out = (uint16_t*)raw; A.Hg = Hg;
  BK_REQUIRE(conv_out && z && A_log && dt_bias && a_p && b_p && raw, "gdn_slabs: null pointer");
  BK_REQUIRE(((uintptr_t)raw & 15) == 0 && ((uintptr_t)conv_out & 3) == 0, "gdn_slabs: raw must be 16-byte aligned, conv_out 4-byte aligned");
  int rc = check_common(A, batch);
  if (rc) return rc;
  const bool nt = g_tune_gdn_nt >= 0 ? g_tune_gdn_nt != 0 : (int64_t)Hg * batch >= 128;
  GdnSlabArgs P{A.q, A.z, A.A_log, A.dt_bias, A.a_p, A.b_p, A.S_in, A.S_out, (uint8_t*)raw, Hg};
  if (nt) hipLaunchKernelGGL((gdn_slab_kernel<true>), dim3(Hg, 4, batch), dim3(64), 0, stream(), P);
  else hipLaunchKernelGGL((gdn_slab_kernel<false>), dim3(Hg, 4, batch), dim3(64), 0, stream(), P);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

int launch_gdn_core(const void* q, const void* k, const void* v, const float* g, const float* beta, const float* S_in,
                    void* out, float* S_out, int Hg, int batch) {
  GdnArgs A{};
  A.q = (const uint16_t*)q; A.k = (const uint16_t*)k; A.v = (const uint16_t*)v;
  A.qkv_bstride = (int64_t)Hg * GDN_D;
  A.g = g; A.beta = beta; A.S_in = S_in; A.S_out = S_out; A.out = (uint16_t*)out; A.Hg = Hg;
  BK_REQUIRE(g && beta, "gdn_core: null pointer");
  int rc = check_common(A, batch);
  if (rc) return rc;
  // up to a few (batch, head) pairs per CU: cut every head into two column slabs (measured best at 32 .. 512 pairs)
  const int64_t pairs = (int64_t)Hg * batch;
  const int cs = g_tune_gdn_cs > 0 ? g_tune_gdn_cs : (pairs <= 4 * num_cus() ? 2 : 1);
  if (cs == 4)
    hipLaunchKernelGGL((gdn_step_kernel<4, false>), dim3(Hg, 4, batch), dim3(GDN_THREADS), 0, stream(), A);
  else if (cs == 2)
    hipLaunchKernelGGL((gdn_step_kernel<2, false>), dim3(Hg, 2, batch), dim3(GDN_THREADS), 0, stream(), A);
  else
    hipLaunchKernelGGL((gdn_step_kernel<1, false>), dim3(Hg, 1, batch), dim3(GDN_THREADS), 0, stream(), A);
  BK_LAUNCH_CHECK();
  return BK_OK;
}

}  // namespace bk
