// Shared host/device helpers for the gfx950 decode kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bk {

// ---------------------------------------------------------------- host side
// Every launcher returns 0 on success or a negative code after recording a
// message that bk_last_error() hands to the caller.
enum : int {
  BK_OK = 0,
  BK_ERR_ARG = -1,      // bad argument (null pointer, unsupported shape)
  BK_ERR_HIP = -2,      // a HIP runtime call failed
  BK_ERR_STATE = -3,    // library not initialised / unknown handle
  BK_ERR_UNSUPPORTED = -4,
};

int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
hipStream_t stream();   // the stream every kernel of this library is launched on
int num_cus();

#define BK_HIP(call)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess)                                                              \
      return ::bk::set_error(::bk::BK_ERR_HIP, "%s failed: %s (%s:%d)", #call,         \
                             hipGetErrorString(e_), __FILE__, __LINE__);               \
  } while (0)

#define BK_REQUIRE(cond, ...)                                          \
  do {                                                                 \
    if (!(cond)) return ::bk::set_error(::bk::BK_ERR_ARG, __VA_ARGS__); \
  } while (0)

#define BK_LAUNCH_CHECK()                                                              \
  do {                                                                                 \
    hipError_t e_ = hipGetLastError();                                                 \
    if (e_ != hipSuccess)                                                              \
      return ::bk::set_error(::bk::BK_ERR_HIP, "kernel launch failed: %s (%s:%d)",     \
                             hipGetErrorString(e_), __FILE__, __LINE__);               \
  } while (0)

// ---------------------------------------------------------------- device side
#if defined(__HIPCC__)

constexpr int WAVE = 64;

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// f32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950: one instruction, denormals kept, NaN quieted).
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

// Exact IEEE binary16 -> binary32 (v_cvt_f32_f16 honours denormals).
__device__ __forceinline__ float half_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}

// Truncating binary32 -> binary16 used for the Q8_1 scales: drop the low 13
// mantissa bits, flush below the normal range to signed zero, overflow to Inf.
__device__ __forceinline__ uint16_t f32_to_half_trunc(float v) {
  uint32_t bits = __float_as_uint(v);
  if ((bits & 0x7fffffffu) == 0) return 0;
  uint32_t s = (bits >> 16) & 0x8000u, e = (bits >> 23) & 0xffu, m = bits & 0x7fffffu;
  int ne = (int)e - 127 + 15;
  if (ne >= 31) return (uint16_t)(s | 0x7c00u);
  if (ne <= 0) return (uint16_t)s;
  return (uint16_t)(s | ((uint32_t)ne << 10) | (m >> 13));
}

// DPP controls (GFX9 encoding)
constexpr int DPP_QUAD_XOR1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ float readlane_f32(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Sum over each aligned group of 16 lanes; every lane of the group gets the total.
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<DPP_QUAD_XOR1>(v);
  v += dpp_f32<DPP_QUAD_XOR2>(v);
  v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
  v += dpp_f32<DPP_ROW_MIRROR>(v);
  return v;
}
// Sum over the whole 64-lane wavefront; the result is wave-uniform.  The order
// of additions is fixed, so the result does not depend on the launch shape.
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return (readlane_f32(v, 0) + readlane_f32(v, 16)) + (readlane_f32(v, 32) + readlane_f32(v, 48));
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_f32<DPP_QUAD_XOR1>(v));
  v = fmaxf(v, dpp_f32<DPP_QUAD_XOR2>(v));
  v = fmaxf(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v));
  v = fmaxf(v, dpp_f32<DPP_ROW_MIRROR>(v));
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  return fmaxf(fmaxf(readlane_f32(v, 0), readlane_f32(v, 16)), fmaxf(readlane_f32(v, 32), readlane_f32(v, 48)));
}
__device__ __forceinline__ int row16_sum_i32(int v) {
  v += dpp_i32<DPP_QUAD_XOR1>(v);
  v += dpp_i32<DPP_QUAD_XOR2>(v);
  v += dpp_i32<DPP_ROW_HALF_MIRROR>(v);
  v += dpp_i32<DPP_ROW_MIRROR>(v);
  return v;
}

// Transcendentals are evaluated in double and rounded once to f32, and written f32
// arithmetic uses one IEEE operation per written operation (__fmul_rn & co. keep the
// compiler from fusing), so that these values equal a plain host computation to the bit.
__device__ __forceinline__ float sigmoid_f64(float v) { return (float)(1.0 / (1.0 + exp(-(double)v))); }
// (float)(1 / sqrt(v)) for a normal positive v: the hardware's reciprocal square root estimate (about 2^-26 relative)
// and one third-order correction y += y * e * (1/2 + 3/8 e), e = 1 - v y^2, leave y within an ulp or so of the double
// value of 1/sqrt(v) (2^-78 from the iteration, the rest is rounding), which is then rounded once to f32: the same float as
// the host's correctly rounded sqrt and division give unless the double lies within ~1e-16 of an f32 rounding boundary.
__device__ __forceinline__ float rsqrt_f64(double v) {
  const double y = __builtin_amdgcn_rsq(v);
  const double e = fma(-v * y, y, 1.0);
  return (float)fma(y, e * fma(0.375, e, 0.5), y);
}

// a / 127 in double, correctly rounded, for any finite f32 value a: q1 = a * c with c = fl(1/127), the exact residual
// r = a - 127 q1 by FMA, q = q1 + r c (checked against the division for all 2^23 significands).
__device__ __forceinline__ double div127_f64(double a) {
  const double c = 1.0 / 127.0;
  const double q1 = a * c;
  return fma(fma(-127.0, q1, a), c, q1);
}

__device__ __forceinline__ double readlane_f64(double v, int lane) {
  const long long b = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffll), lane);
  const int hi = __builtin_amdgcn_readlane((int)(b >> 32), lane);
  return __builtin_bit_cast(double, ((long long)hi << 32) | (unsigned int)lo);
}
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
  const long long b = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_update_dpp(0, (int)(b & 0xffffffffll), CTRL, 0xF, 0xF, true);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xF, 0xF, true);
  return __builtin_bit_cast(double, ((long long)hi << 32) | (unsigned int)lo);
}
// Wave-wide sum in double, wave-uniform result.
__device__ __forceinline__ double wave_sum_f64(double v) {
  v += dpp_f64<DPP_QUAD_XOR1>(v);
  v += dpp_f64<DPP_QUAD_XOR2>(v);
  v += dpp_f64<DPP_ROW_HALF_MIRROR>(v);
  v += dpp_f64<DPP_ROW_MIRROR>(v);
  return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}

// Q8_1 rounding of one value: q = floor(fl64(f / d) + 0.5) with d = fl64(amax / 127) (bench/bench.ts:53-72,
// ECMAScript Math.round).  The quotient is first formed in f32 (t = f * (127 / amax), off by less than 5e-5 from
// the double quotient); only when t + 0.5 lies within 2e-4 of an integer — where the two could round
// differently — is the double division carried out.  Both paths return the reference's integer.
__device__ __forceinline__ int q8_1_round_exact(float f, double div) {
  const double qd = (double)f / div;
  double r = floor(qd);
  if (qd - r >= 0.5) r += 1.0;
  return (int)r;
}
__device__ __forceinline__ int q8_1_round(float f, float inv, double div) {
  const float u = f * inv + 0.5f;
  if (fabsf(u - rintf(u)) < 2e-4f) return q8_1_round_exact(f, div);      // rare
  return (int)floorf(u);
}
// 127 / amax to within two ulps (the f32 quotient above tolerates it), 0 for an all-zero block
__device__ __forceinline__ float q8_1_inv(float amax) { return amax != 0.0f ? 127.0f * __builtin_amdgcn_rcpf(amax) : 0.0f; }

// Q8_1 of one 32-element block held by four consecutive lanes (8 values each, already rounded to
// the activation's storage type).  d = amax/127 in double, s = trunc16(float(sum(q) * d)) with the
// unrounded d.  Returns the lane's 8 int8 in pk[0..1] and the packed (d, s) halves, the same in all four lanes.
__device__ __forceinline__ uint32_t quad_q8_1(const float (&f)[8], uint32_t (&pk)[2]) {
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 8; j++) amax = fmaxf(amax, fabsf(f[j]));
  amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR1>(amax));
  amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR2>(amax));
  const double d = div127_f64((double)amax), div = d != 0.0 ? d : 1.0;
  const float inv = q8_1_inv(amax);
  // all eight quotients in f32 first; one test tells whether any of them sits near a rounding boundary
  float u[8];
  bool near = false;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    u[j] = f[j] * inv + 0.5f;
    near = near || fabsf(u[j] - rintf(u[j])) < 2e-4f;
  }
  int q[8];
#pragma unroll
  for (int j = 0; j < 8; j++) q[j] = (int)floorf(u[j]);
  if (near) {                                     // rare: those values are decided by the double quotient
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (fabsf(u[j] - rintf(u[j])) < 2e-4f) q[j] = q8_1_round_exact(f[j], div);
  }
  int sum = 0;
  pk[0] = 0; pk[1] = 0;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    sum += q[j];
    const int c = q[j] < -128 ? -128 : (q[j] > 127 ? 127 : q[j]);
    pk[j >> 2] |= (uint32_t)(c & 0xff) << (8 * (j & 3));
  }
  sum += dpp_i32<DPP_QUAD_XOR1>(sum);
  sum += dpp_i32<DPP_QUAD_XOR2>(sum);
  return (uint32_t)f32_to_half_trunc((float)d) | ((uint32_t)f32_to_half_trunc((float)((double)sum * d)) << 16);
}

// Q8_1 of one 32-element block whose values sit one per lane in an aligned group of 32 lanes (all 32 active): every lane
// stores its int8, the first lane of the group the (d, s) pair (`store` = false for a whole group: nothing is written).
// `blk` points at the 36-byte block, l = lane % 32.
__device__ __forceinline__ void lane32_q8_1_store(float v, uint8_t* __restrict__ blk, int l, bool store = true) {
  float amax = row16_max(fabsf(v));
  amax = fmaxf(amax, __shfl_xor(amax, 16));
  const double d = div127_f64((double)amax);
  int q = q8_1_round(v, q8_1_inv(amax), d != 0.0 ? d : 1.0);
  int sum = row16_sum_i32(q);
  sum += __shfl_xor(sum, 16);
  q = q < -128 ? -128 : (q > 127 ? 127 : q);
  if (!store) return;                      // the group took part in the exchanges above; nothing of it is kept
  blk[l] = (uint8_t)(int8_t)q;
  if (l == 0)
    *(uint32_t*)(blk + 32) = (uint32_t)f32_to_half_trunc((float)d) | ((uint32_t)f32_to_half_trunc((float)((double)sum * d)) << 16);
}

// Block-wide sum in double for blockDim.x = 64 * NW; every thread gets the total.
template <int NW>
__device__ __forceinline__ double block_sum_f64(double v, double* lds) {
  v = wave_sum_f64(v);
  if (NW == 1) return v;
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) lds[w] = v;
  __syncthreads();
  double t = 0.0;
#pragma unroll
  for (int i = 0; i < NW; i++) t += lds[i];
  __syncthreads();
  return t;
}

#endif  // __HIPCC__
// Memory -> LDS without a register in between: lane l of the wave fills the l-th 16-byte (4-byte) slot of the LDS piece
// that starts at `lds_piece` (the same address in every lane) from an address of its own choosing.  Written as
// instructions, not through the compiler's builtin: the compiler would put a wait for the whole transfer in front of the
// next LDS access of any kind (it cannot tell which LDS bytes a transfer in flight will write), and a tile requested
// a step ahead would be waited for at once.  The caller waits itself (s_waitcnt vmcnt) before the barrier that hands
// the piece to its readers.  m0 carries the LDS address; nothing else in these kernels uses that register.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_dma16(const void* src, const void* lds_piece) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"((uint32_t)(uintptr_t)lds_piece) : "memory", "m0");
}
// the same with the address as a wave-uniform base (scalar registers) plus a 32-bit byte offset per lane: a run of
// transfers from one page costs no vector arithmetic
__device__ __forceinline__ void lds_dma16_s(const void* sbase, uint32_t voff, const void* lds_piece) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"((uint32_t)(uintptr_t)lds_piece) : "memory", "m0");
}
__device__ __forceinline__ void lds_dma4(const void* src, const void* lds_piece) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(src), "s"((uint32_t)(uintptr_t)lds_piece) : "memory", "m0");
}
// An LDS address the compiler has to take as it comes: computed from this value, the addresses of a run of transfers
// are one scalar addition each at the point of use; computed from the array's name they are loop invariants, all of them
// kept in scalar registers across the loop (and spilled: a run has dozens).
__device__ __forceinline__ const unsigned char* lds_opaque(const void* p) {
  uint32_t a = (uint32_t)(uintptr_t)p;
  asm volatile("" : "+s"(a));
  return (const unsigned char*)(uintptr_t)a;
}
#pragma clang diagnostic pop

}  // namespace bk
