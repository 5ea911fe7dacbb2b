// Typed entry points and the per-op launch surface (bk_kernel_create / bk_launch)
// that stands in for compileAndLoad + cuLaunch (src/ttir.ts:488-491, 321-348).
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/bunker_hip.h"
#include "ops.h"

namespace bk {

#define BK_NEED_INIT() \
  do { if (!inited()) return set_error(BK_ERR_STATE, "bk_init has not been called"); } while (0)

template <typename T>
static inline T* P(uint64_t v) { return (T*)(uintptr_t)v; }

// ---------------------------------------------------------------- kernel handles
struct Kernel;
typedef int (*RunFn)(Kernel&, const uint64_t* slots);

struct Kernel {
  std::string op, spec;
  std::map<std::string, int64_t> p;
  RunFn run = nullptr;
  int nslots = 0;
  void* scratch = nullptr;     // per-handle device workspace, allocated at create time
  size_t scratch_bytes = 0;
  int generation = 0;          // how often the slot has been reused
  int64_t get(const char* k, int64_t def) const {
    auto it = p.find(k);
    return it == p.end() ? def : it->second;
  }
  bool has(const char* k) const { return p.count(k) != 0; }
};

static std::vector<Kernel> g_kernels;
static std::vector<int> g_free_slots;          // destroyed handles' slots, taken again by bk_kernel_create
// handle = slot | generation << 20: a handle kept past its bk_kernel_destroy does not name the slot's next kernel
enum : int { HANDLE_SLOTS = 1 << 20, HANDLE_GENS = 1 << 10 };
static int handle_of(int slot) { return slot | ((g_kernels[slot].generation & (HANDLE_GENS - 1)) << 20); }
static Kernel* kernel_of(int handle) {
  const int slot = handle & (HANDLE_SLOTS - 1);
  if (handle < 0 || slot >= (int)g_kernels.size()) return nullptr;
  Kernel& k = g_kernels[slot];
  return (k.run && handle_of(slot) == handle) ? &k : nullptr;
}

// bk_shutdown: every handle's workspace goes back to the device and the handles become invalid
void kernels_release_all() {
  for (Kernel& k : g_kernels)
    if (k.scratch) (void)hipFree(k.scratch);
  g_kernels.clear();
  g_free_slots.clear();
}

std::string kernel_label(int kernel) {
  const Kernel* k = kernel_of(kernel);
  return k ? k->spec : "?";
}

static int need(Kernel& k, const char* key) {
  if (!k.has(key)) return set_error(BK_ERR_ARG, "kernel '%s': missing parameter %s=", k.op.c_str(), key);
  return BK_OK;
}
static int alloc_scratch(Kernel& k, size_t bytes) {
  BK_HIP(hipMalloc(&k.scratch, bytes));
  k.scratch_bytes = bytes;
  return BK_OK;
}

// ---- op: quantize_q8_1   slots: x, out      params: K, batch=1, bf16=0
static int run_quantize(Kernel& k, const uint64_t* s) {
  return launch_quantize_q8_1(P<void>(s[0]), (int)k.get("bf16", 0), P<void>(s[1]), (int)k.get("K", 0), (int)k.get("batch", 1));
}
// ---- op: gemv_q4k_q8_1   slots: W, xq, y    params: N, K, batch=1, cast=0
static int run_gemv(Kernel& k, const uint64_t* s) {
  return launch_gemv_q4k_q8_1(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), (int)k.get("N", 0), (int)k.get("K", 0),
                              (int)k.get("batch", 1), (int)k.get("cast", 0), nullptr);
}
// ---- op: gemm (the model graph's M=1 matmul, src/model.ts:71-73)
// slots: A (bf16 [batch,K]), B (Q4_K [N,K]), out (f32, or bf16 with cast=1)
// params: N, K, cast=0, batch=1.  A is quantized to Q8_1 into the handle's workspace first.
// Batches of GEMM_MFMA_MIN_BATCH rows and more go to the int8 MFMA kernel (32 rows per tile), smaller
// ones stream the weights once per row through the GEMV; mfma=0/1 in the spec forces either.
constexpr int GEMM_MFMA_MIN_BATCH = 8;
static int matmul_q8_1(const void* W, const void* xq, void* y, int N, int K, int batch, int out_dtype, const void* res, int force) {
  const bool mfma = force >= 0 ? force != 0 : batch >= GEMM_MFMA_MIN_BATCH;
  if (!mfma) return launch_gemv_q4k_q8_1(W, xq, y, N, K, batch, out_dtype, res);
  return launch_gemm_q4k_q8_1_mfma(W, xq, y, N, K, batch, out_dtype, res);
}
// several matrices over the same activation rows (the kernel cuts the batch into 32-row tiles)
static int matmul_group_mfma(const void* xq, int K, int batch, int G, const void* const* W, void* const* out, const void* const* res,
                             const int* N, const int* epi) {
  return launch_gemm_group_mfma(xq, K, batch, G, W, out, res, N, epi);
}
static int run_gemm(Kernel& k, const uint64_t* s) {
  const int N = (int)k.get("N", 0), K = (int)k.get("K", 0), batch = (int)k.get("batch", 1);
  int rc = launch_quantize_q8_1(P<void>(s[0]), DT_BF16, k.scratch, K, batch);
  if (rc) return rc;
  return matmul_q8_1(P<void>(s[1]), k.scratch, P<void>(s[2]), N, K, batch, (int)k.get("cast", 0), nullptr, (int)k.get("mfma", -1));
}

// ---- op: gemv_fused — rmsnorm / quantize + up to four matmuls over one activation + their cast / add / swiglu
// consumers (src/model.ts:65-73, 161-191 as one launch; the node-by-node result to the bit).
// params: K, pro (0: x is Q8_1, 1: x is bf16, 2: x is bf16 and goes through rmsnorm with norm_w first, 3: x is the raw
//         block of a gdn_slabs op and goes through that op's gated RMS norm with norm_w (f32 [128]) first: K = 2048, batch < 8),
//         G matrices with N<i>, epi<i> (0: f32, 1: bf16, 2: bf16(bf16(y) + residual), 3 (matrix 0, pro=2, K = 1024 or
//         2048, batch < 8): bf16, then conv1d_decode over the N0 channels), swiglu=0|1 (G=2: gate, up), batch=1
// slots:  x, [norm_w if pro=2|3], then per matrix: W, [residual if epi=2 | conv_state_in, conv_w if epi=3], out,
//         [conv_state_new if epi=3]      (swiglu: x, [norm_w], Wg, Wu, out [, out as Q8_1 blocks when q8out=1: batch >= 8 only])
// Shapes outside the fused kernel (K other than 1024, 2048, 3584, 4096, 6144, or batch >= 8) run as rmsnorm/quantize,
// matmuls, swiglu.
static int run_gemv_fused(Kernel& k, const uint64_t* s) {
  const int K = (int)k.get("K", 0), pro = (int)k.get("pro", 0), G = (int)k.get("G", 1), batch = (int)k.get("batch", 1);
  const bool swiglu = k.get("swiglu", 0) != 0;
  int si = 0;
  const void* x = P<void>(s[si++]);
  const void* nw = (pro == 2 || pro == 3) ? P<void>(s[si++]) : nullptr;
  const void* W[4] = {}; void* out[4] = {}; const void* res[4] = {}; int N[4] = {}, epi[4] = {};
  FusedConv conv{};
  char key[16];
  for (int i = 0; i < G; i++) {
    snprintf(key, sizeof key, "N%d", i); N[i] = (int)k.get(key, 0);
    snprintf(key, sizeof key, "epi%d", i); epi[i] = (int)k.get(key, 0);
    W[i] = P<void>(s[si++]);
    if (swiglu) continue;
    if (epi[i] == 2) res[i] = P<void>(s[si++]);
    if (epi[i] == 3) { conv.st = P<void>(s[si]); conv.w = P<void>(s[si + 1]); si += 2; }
    out[i] = P<void>(s[si++]);
    if (epi[i] == 3) conv.st_new = P<void>(s[si++]);
  }
  if (swiglu) out[0] = P<void>(s[si++]);
  void* q8out = swiglu && k.get("q8out", 0) ? P<void>(s[si++]) : nullptr;      // composed path only (build_gemv_fused checks)
  if (gemv_fused_fast_path(K, batch, swiglu)) return launch_gemv_fused(pro, x, nw, K, batch, G, W, out, res, N, epi, swiglu, conv.st ? &conv : nullptr);
  int rc;
  const void* xq = x;
  // The GDN layers' projections at hidden size 2048: qkv and z are 256 tiles of the batched matmul, one per CU with eight
  // waves each, and the 16-row a and b would add two (a second, four-wave form: 11.9 us instead of 8.7 at batch 32).
  // Those two run inside the norm's launch instead, on CUs it leaves idle.
  int Gm = G;
  if (pro == 2 && !swiglu && G == 4 && batch >= GEMM_MFMA_MIN_BATCH && batch <= 32 && K == 2048 && epi[2] == 0 && epi[3] == 0 &&
      N[2] + N[3] <= 64 && g_tune_small_rows != 0) {
    const int big = (N[0] + 31) / 32 + (N[1] + 31) / 32, all = big + (N[2] + 31) / 32 + (N[3] + 31) / 32;
    if (big <= num_cus() && all > num_cus()) Gm = 2;
  }
  if (pro == 2 && Gm == 2 && G == 4) {
    if ((rc = launch_rmsnorm_small_rows(x, nw, k.scratch, K, batch, W[2], W[3], (float*)out[2], (float*)out[3], N[2], N[3]))) return rc;
    xq = k.scratch;
  } else if (pro == 2) { if ((rc = launch_rmsnorm(x, nw, nullptr, k.scratch, K, batch))) return rc; xq = k.scratch; }
  else if (pro == 1) { if ((rc = launch_quantize_q8_1(x, DT_BF16, k.scratch, K, batch))) return rc; xq = k.scratch; }
  if (swiglu) {
    // batched and with a Q8_1 result: SwiGLU and the quantization are the matmul kernel's last step
    if (q8out && batch >= GEMM_MFMA_MIN_BATCH) return launch_gemm_swiglu_mfma(xq, K, batch, W[0], W[1], N[0], out[0], q8out);
    float* g = (float*)((uint8_t*)k.scratch + (size_t)batch * (K / 32) * 36);
    float* u = g + (size_t)batch * N[0];
    if (batch >= GEMM_MFMA_MIN_BATCH) {
      void* gu[2] = {g, u}; const void* nores[2] = {nullptr, nullptr}; const int n2[2] = {N[0], N[0]}, e2[2] = {0, 0};
      if ((rc = matmul_group_mfma(xq, K, batch, 2, W, gu, nores, n2, e2))) return rc;
    } else {
      if ((rc = matmul_q8_1(W[0], xq, g, N[0], K, batch, DT_F32, nullptr, -1))) return rc;
      if ((rc = matmul_q8_1(W[1], xq, u, N[0], K, batch, DT_F32, nullptr, -1))) return rc;
    }
    if (q8out) return launch_swiglu_q8_1(g, u, out[0], q8out, (int64_t)batch * N[0]);
    return launch_elementwise(EW_SWIGLU_OP, g, u, out[0], (int64_t)batch * N[0]);
  }
  if (batch >= GEMM_MFMA_MIN_BATCH) return matmul_group_mfma(xq, K, batch, Gm, W, out, res, N, epi);
  for (int i = 0; i < G; i++)
    if ((rc = matmul_q8_1(W[i], xq, out[i], N[i], K, batch, epi[i] == 0 ? DT_F32 : DT_BF16, res[i], -1))) return rc;
  return BK_OK;
}
static int build_gemv_fused(Kernel& k) {
  int rc;
  if ((rc = need(k, "K")) || (rc = need(k, "N0"))) return rc;
  const int64_t K = k.get("K", 0), pro = k.get("pro", 0), G = k.get("G", 1), batch = k.get("batch", 1);
  const bool swiglu = k.get("swiglu", 0) != 0;
  BK_REQUIRE(K > 0 && K % 256 == 0, "gemv_fused: K=%lld must be a positive multiple of 256", (long long)K);
  BK_REQUIRE(pro >= 0 && pro <= 3 && G >= 1 && G <= 4 && batch >= 1 && batch <= 4096, "gemv_fused: bad pro/G/batch");
  BK_REQUIRE(pro != 3 || (K == 2048 && !swiglu && gemv_fused_fast_path((int)K, (int)batch, false)),
             "gemv_fused: pro=3 (gated norm of a gdn_slabs block) serves K = 2048 at batch < 8");
  BK_REQUIRE(!swiglu || G == 2, "gemv_fused: swiglu needs G=2 (gate, up)");
  int nslots = 1 + (pro >= 2 ? 1 : 0);
  char key[16];
  for (int i = 0; i < G; i++) {
    snprintf(key, sizeof key, "N%d", i);
    BK_REQUIRE(k.get(key, 0) > 0, "gemv_fused: missing or bad %s", key);
    BK_REQUIRE(!swiglu || k.get(key, 0) == k.get("N0", 0), "gemv_fused: gate and up must have the same N");
    BK_REQUIRE(!swiglu || k.get(key, 0) % 4 == 0, "gemv_fused: swiglu needs N to be a multiple of 4");
    snprintf(key, sizeof key, "epi%d", i);
    const int64_t e = k.get(key, 0);
    BK_REQUIRE((e >= 0 && e <= 2) || (e == 3 && i == 0 && pro == 2 && !swiglu && (K == 2048 || K == 1024) && gemv_fused_fast_path((int)K, (int)batch, false)),
               "gemv_fused: bad %s (3 = conv1d behind matrix 0 of an rmsnorm group with K = 1024 or 2048 at batch < 8)", key);
    nslots += swiglu ? 1 : (e == 2 ? 3 : (e == 3 ? 5 : 2));
  }
  if (swiglu) nslots += 1;
  if (k.get("q8out", 0)) {
    BK_REQUIRE(swiglu && !gemv_fused_fast_path((int)K, (int)batch, true) && k.get("N0", 0) % 32 == 0,
               "gemv_fused: q8out=1 (SwiGLU result also as Q8_1) is served by the batched path only (batch >= 8), N a multiple of 32");
    nslots += 1;
  }
  if ((rc = alloc_scratch(k, (size_t)(batch * (K / 32) * 36) + (swiglu ? (size_t)(2 * batch * k.get("N0", 0) * 4) : 0)))) return rc;
  k.run = run_gemv_fused; k.nslots = nslots;
  return BK_OK;
}

// ---- op: embed (src/model.ts:53-56)   slots: embed.weight, token_id, out
// params: H, VOCAB, batch=1, ids_dev=0 (1: slot 1 is a device pointer to int32 [batch])
static int run_embed(Kernel& k, const uint64_t* s) {
  const bool dev = k.get("ids_dev", 0) != 0;
  return launch_embed(P<void>(s[0]), dev ? P<int32_t>(s[1]) : nullptr, dev ? 0 : (int32_t)(uint32_t)s[1], P<void>(s[2]),
                      (int)k.get("H", 0), (int)k.get("VOCAB", 0), (int)k.get("batch", 1));
}
// ---- op: rmsnorm (src/model.ts:65-67)   slots: x, w, out     params: N, batch=1
static int run_rmsnorm(Kernel& k, const uint64_t* s) {
  return launch_rmsnorm(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), nullptr, (int)k.get("N", 0), (int)k.get("batch", 1));
}
// ---- op: rmsnorm_q8_1   slots: x, w, out (bf16, may be 0), xq (Q8_1)   params: N, batch=1
static int run_rmsnorm_q8(Kernel& k, const uint64_t* s) {
  return launch_rmsnorm(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), (int)k.get("N", 0), (int)k.get("batch", 1));
}
// ---- ops: cast (x, out), add (a, b, out), swiglu (g, u, out)   params: N, batch=1
static int run_cast(Kernel& k, const uint64_t* s) {
  return launch_elementwise(EW_CAST_OP, P<void>(s[0]), nullptr, P<void>(s[1]), k.get("N", 0) * k.get("batch", 1));
}
static int run_add(Kernel& k, const uint64_t* s) {
  return launch_elementwise(EW_ADD_OP, P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), k.get("N", 0) * k.get("batch", 1));
}
static int run_swiglu(Kernel& k, const uint64_t* s) {
  return launch_elementwise(EW_SWIGLU_OP, P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), k.get("N", 0) * k.get("batch", 1));
}
// ---- op: conv1d_decode (src/model.ts:77-87)   slots: qkv, conv_state_in, weight, out, conv_state_new
static int run_conv1d(Kernel& k, const uint64_t* s) {
  return launch_conv1d_decode(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), P<void>(s[4]), (int)k.get("QKVD", 0),
                              (int)k.get("batch", 1));
}
// ---- op: gdn_delta_rule (src/model.ts:94-109)
// slots: conv_out, z, A_log, dt_bias, a_p, b_p, norm_w, s_state_in, out, s_state_new     params: LVH, batch=1
static int run_gdn(Kernel& k, const uint64_t* s) {
  return launch_gdn_fused(P<void>(s[0]), P<void>(s[1]), P<float>(s[2]), P<void>(s[3]), P<float>(s[4]), P<float>(s[5]),
                          P<float>(s[6]), P<float>(s[7]), P<void>(s[8]), P<float>(s[9]), (int)k.get("LVH", 0), (int)k.get("batch", 1));
}
// ---- op: gdn_conv = conv1d_decode + gdn_delta_rule in one launch (the conv output never reaches memory)
// slots: qkv, conv_state_in, conv_w, z, A_log, dt_bias, a_p, b_p, norm_w, s_state_in, out, conv_state_new, s_state_new
// params: LVH (= number of key heads), batch=1, q8out=0 (1: one more slot, the output again as Q8_1 blocks [batch, ZD/32]
//         for the out_proj matmul, written by the same threads that write the bf16 output)
static int run_gdn_conv(Kernel& k, const uint64_t* s) {
  return launch_gdn_conv_fused(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), P<float>(s[4]), P<void>(s[5]),
                               P<float>(s[6]), P<float>(s[7]), P<float>(s[8]), P<float>(s[9]), P<void>(s[10]), P<void>(s[11]),
                               P<float>(s[12]), k.get("q8out", 0) ? P<void>(s[13]) : nullptr, (int)k.get("LVH", 0),
                               (int)k.get("batch", 1));
}
// ---- op: gdn_slabs = gdn_delta_rule without its gated norm, four column slabs per head (few sequences: every slab on
// a CU of its own).  The raw outputs go to `raw` (per sequence: f32 o[LVH*128] | f32 z*sigmoid(z)[LVH*128] | f64 sum of
// o^2 per (head, slab)), which the out_proj matmul's prologue turns into the op's output (gemv_fused pro=3).
// slots: conv_out, z, A_log, dt_bias, a_p, b_p, s_state_in, raw, s_state_new      params: LVH, batch=1
static int run_gdn_slabs(Kernel& k, const uint64_t* s) {
  return launch_gdn_slabs(P<void>(s[0]), P<void>(s[1]), P<float>(s[2]), P<void>(s[3]), P<float>(s[4]), P<float>(s[5]), P<float>(s[6]),
                          P<void>(s[7]), P<float>(s[8]), (int)k.get("LVH", 0), (int)k.get("batch", 1));
}
// ---- ops: qnorm (q-gate buffer, w, out; NH heads, input rows 2*HD apart), knorm (k, w, out; NKV heads)
static int run_qnorm(Kernel& k, const uint64_t* s) {
  const int HD = (int)k.get("HD", 0), NH = (int)k.get("NH", 0);
  return launch_headnorm(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), NH, HD, 2 * HD, (int64_t)NH * 2 * HD, (int)k.get("batch", 1),
                         nullptr, nullptr, nullptr, 0, 0, 0);
}
static int run_knorm(Kernel& k, const uint64_t* s) {
  const int HD = (int)k.get("HD", 0), NKV = (int)k.get("NKV", 0);
  return launch_headnorm(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), NKV, HD, HD, (int64_t)NKV * HD, (int)k.get("batch", 1),
                         nullptr, nullptr, nullptr, 0, 0, 0);
}
// ---- ops: rope / ropek (src/model.ts:133-143)   slots: Q (in place), rope_cos, rope_sin, pos
// params: HD, NH | NKV, ROT_HALF, MAX_LEN, batch=1, pos_dev=0 (1: slot 3 is a device pointer to int32 [batch])
static int run_rope(Kernel& k, const uint64_t* s) {
  const bool dev = k.get("pos_dev", 0) != 0;
  const int nh = (int)(k.has("NH") ? k.get("NH", 0) : k.get("NKV", 0));
  return launch_rope(P<void>(s[0]), P<float>(s[1]), P<float>(s[2]), dev ? P<int32_t>(s[3]) : nullptr, dev ? 0 : (int)(int32_t)s[3],
                     nh, (int)k.get("HD", 0), (int)k.get("ROT_HALF", 0), (int)k.get("MAX_LEN", 0), (int)k.get("batch", 1));
}
// Attention ops: exact=1 (the default) runs the double-precision kernels, whose outputs are the bits of the host loop
// (prototypes/fa2_vllm.ts:114-139 in doubles); exact=0 the bf16 matrix-instruction kernels (within 2e-2).
static size_t fa2_qn_bytes(int rows, int NH, int HD) { return ((size_t)rows * NH * HD * 2 + 255) / 256 * 256; }
static size_t fa2_ws_bytes(int rows, int NKV, int splits, int exact) {
  if (exact) return attn_exact_workspace_bytes(rows, NKV, splits > 1 ? splits : 0);
  return splits > 1 ? attn_workspace_bytes(rows, NKV, splits) : 0;
}
// ---- op: fa2_attn (src/model.ts:144-157)
// slots: q, k, v, qgate, kv_k_in, kv_v_in, pos, out, kv_k_new, kv_v_new; like the reference's emitter only
// kv_*_in are touched (the caller maps in and new to one buffer).  This step's k, v go into the cache at
// pos, then the query attends to tokens 0..pos.  Each sequence owns MAX_LEN/16 consecutive pages.
// params: HD, NH, NKV, MAX_LEN, batch=1, pos_dev=0
static int run_fa2(Kernel& k, const uint64_t* s) {
  const bool dev = k.get("pos_dev", 0) != 0;
  const int HD = (int)k.get("HD", 0), NH = (int)k.get("NH", 0), NKV = (int)k.get("NKV", 0), batch = (int)k.get("batch", 1);
  const int max_len = (int)k.get("MAX_LEN", 0), bt_stride = (max_len + 15) / 16;
  const int32_t* pos_dev = dev ? P<int32_t>(s[6]) : nullptr;
  const int pos = dev ? 0 : (int)(int32_t)s[6];
  if (!dev) BK_REQUIRE(pos >= 0 && pos < max_len, "fa2_attn: pos=%d outside the cache (MAX_LEN=%d)", pos, max_len);
  int rc = launch_kv_append(P<void>(s[1]), P<void>(s[2]), P<void>(s[4]), P<void>(s[5]), nullptr, bt_stride, pos_dev, pos, max_len, batch, NKV, HD, 16);
  if (rc) return rc;
  // the context of each sequence is its pos + 1
  return launch_attn_decode(P<void>(s[0]), P<void>(s[4]), P<void>(s[5]), nullptr, bt_stride, pos_dev, pos, 1, max_len,
                            P<uint16_t>(s[3]) + HD, (int64_t)NH * 2 * HD, 2 * HD, P<void>(s[7]), nullptr, k.scratch, k.scratch_bytes,
                            batch, NH, NKV, HD, 16, (int)k.get("splits", 0), nullptr, 1, (int)k.get("exact", 1));
}
// ---- op: fa2_fused = qnorm, rope, knorm, ropek, fa2_attn of src/model.ts:126-157 as two launches (split attention
// with the norms, the rotation and the cache append inside; merge with the output gate), or as three with the
// preparation as a launch of its own (prep_fused=0, and always with exact=0).
// slots: qgate (q_proj output, [q | gate] per head), k, v, q_norm.weight, k_norm.weight, rope_cos, rope_sin, pos,
//        kv_k, kv_v, out [, out as Q8_1 blocks when q8out=1]        params: HD, NH, NKV, MAX_LEN, ROT_HALF, batch=1, pos_dev=0, q8out=0,
//        exact=1, prep_fused=1
static int run_fa2_fused(Kernel& k, const uint64_t* s) {
  const bool dev = k.get("pos_dev", 0) != 0;
  const int HD = (int)k.get("HD", 0), NH = (int)k.get("NH", 0), NKV = (int)k.get("NKV", 0), batch = (int)k.get("batch", 1);
  const int max_len = (int)k.get("MAX_LEN", 0), bt_stride = (max_len + 15) / 16, half = (int)k.get("ROT_HALF", 0);
  const int32_t* pos_dev = dev ? P<int32_t>(s[7]) : nullptr;
  const int pos = dev ? 0 : (int)(int32_t)s[7];
  // workspace: normalised, rotated q as bf16 [batch, NH, HD]; exact=1: the same as f64 [batch, NKV, HD, 8] (written by the
  // prep kernel, unused columns stay zero from creation); then the partials of the splits
  const int exact = (int)k.get("exact", 1);
  const size_t qn_bytes = fa2_qn_bytes(batch, NH, HD), qf_bytes = exact ? attn_exact_qf_bytes(batch, NKV) : 0;
  void* qn = k.scratch;
  uint32_t* qf = exact ? (uint32_t*)((uint8_t*)k.scratch + qn_bytes) : nullptr;
  void* ws = (uint8_t*)k.scratch + qn_bytes + qf_bytes;
  if (exact && k.get("prep_fused", 1) != 0) {
    // one launch less: the attention kernel prepares q itself and the workgroup that holds the new position appends k, v
    BK_REQUIRE(dev || (pos >= 0 && pos < max_len), "attn_prep: pos=%d outside the cache (max_len=%d)", pos, max_len);
    const AttnPrepFuse pf{P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), P<void>(s[4]), P<float>(s[5]), P<float>(s[6]), half, max_len};
    return launch_attn_decode(nullptr, P<void>(s[8]), P<void>(s[9]), nullptr, bt_stride, pos_dev, pos, 1, max_len, P<uint16_t>(s[0]) + HD,
                              (int64_t)NH * 2 * HD, 2 * HD, P<void>(s[10]), nullptr, ws, k.scratch_bytes - qn_bytes - qf_bytes,
                              batch, NH, NKV, HD, 16, (int)k.get("splits", 0), k.get("q8out", 0) ? P<void>(s[11]) : nullptr, 1, 1, nullptr, &pf);
  }
  int rc = launch_attn_prep(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), P<void>(s[4]), P<float>(s[5]), P<float>(s[6]),
                            pos_dev, pos, half, max_len, qn, P<void>(s[8]), P<void>(s[9]), nullptr, bt_stride, batch, NH, NKV, HD, 16, qf);
  if (rc) return rc;
  return launch_attn_decode(qn, P<void>(s[8]), P<void>(s[9]), nullptr, bt_stride, pos_dev, pos, 1, max_len, P<uint16_t>(s[0]) + HD,
                            (int64_t)NH * 2 * HD, 2 * HD, P<void>(s[10]), nullptr, ws, k.scratch_bytes - qn_bytes - qf_bytes,
                            batch, NH, NKV, HD, 16, (int)k.get("splits", 0), k.get("q8out", 0) ? P<void>(s[11]) : nullptr, 1, exact, qf);
}
// ---- prefill ops: T consecutive tokens of ONE sequence per launch (rows of the activation buffers = tokens)
// conv1d_prefill   slots: qkv [T, QKVD], conv_state_in [3, QKVD], weight, out [T, QKVD], conv_state_new    params: QKVD, T
static int run_conv1d_prefill(Kernel& k, const uint64_t* s) {
  return launch_conv1d_prefill(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), P<void>(s[4]), (int)k.get("QKVD", 0),
                               (int)k.get("T", 0));
}
// gdn_prefill      slots as gdn_delta_rule with T rows in conv_out, z, a_p, b_p, out and one state     params: LVH, T,
//                  chunked=0 (1: the recurrence in chunks of 64 tokens on the f32 matrix instruction — the scan's results up to the order of the additions)
static int run_gdn_prefill(Kernel& k, const uint64_t* s) {
  return launch_gdn_prefill(P<void>(s[0]), P<void>(s[1]), P<float>(s[2]), P<void>(s[3]), P<float>(s[4]), P<float>(s[5]),
                            P<float>(s[6]), P<float>(s[7]), P<void>(s[8]), P<float>(s[9]), k.scratch, k.scratch_bytes,
                            (int)k.get("LVH", 0), (int)k.get("T", 0), k.get("chunked", 0) != 0);
}
// fa2_prefill      the norm + rotation + cache append of fa2_fused for T tokens at positions pos[t], then causal attention:
//                  token t attends to cache positions 0 .. pos[t] of the sequence whose pages block_table lists.
// slots: qgate [T, NH, 2*HD], k [T, NKV, HD], v, q_norm.weight, k_norm.weight, rope_cos, rope_sin, pos (int32 [T], device),
//        block_table (int32 [MAX_LEN/16], device), kv_k, kv_v, out [T, NH*HD]          params: HD, NH, NKV, MAX_LEN, ROT_HALF, T
static int run_fa2_prefill(Kernel& k, const uint64_t* s) {
  const int HD = (int)k.get("HD", 0), NH = (int)k.get("NH", 0), NKV = (int)k.get("NKV", 0), T = (int)k.get("T", 0);
  const int max_len = (int)k.get("MAX_LEN", 0), half = (int)k.get("ROT_HALF", 0);
  const int32_t* pos = P<int32_t>(s[7]);
  const int32_t* table = P<int32_t>(s[8]);
  BK_REQUIRE(pos && table, "fa2_prefill: null position or block table pointer");
  const int exact = (int)k.get("exact", 1);
  const size_t qn_bytes = fa2_qn_bytes(T, NH, HD), qf_bytes = exact ? attn_exact_qf_bytes(T, NKV) : 0;
  void* qn = k.scratch;
  uint32_t* qf = exact ? (uint32_t*)((uint8_t*)k.scratch + qn_bytes) : nullptr;
  void* ws = (uint8_t*)k.scratch + qn_bytes + qf_bytes;
  int rc = launch_attn_prep(P<void>(s[0]), P<void>(s[1]), P<void>(s[2]), P<void>(s[3]), P<void>(s[4]), P<float>(s[5]), P<float>(s[6]),
                            pos, 0, half, max_len, qn, P<void>(s[9]), P<void>(s[10]), table, 0, T, NH, NKV, HD, 16, qf);
  if (rc) return rc;
  if (k.get("tiled", 0))
    return launch_attn_prefill_tiled(qn, P<void>(s[9]), P<void>(s[10]), table, pos, max_len, P<uint16_t>(s[0]) + HD, (int64_t)NH * 2 * HD, 2 * HD,
                                     P<void>(s[11]), T, NH, NKV, HD, 16, ws, k.scratch_bytes - qn_bytes - qf_bytes);
  return launch_attn_decode(qn, P<void>(s[9]), P<void>(s[10]), table, 0, pos, 0, 1, max_len, P<uint16_t>(s[0]) + HD,
                            (int64_t)NH * 2 * HD, 2 * HD, P<void>(s[11]), nullptr, ws, k.scratch_bytes - qn_bytes - qf_bytes,
                            T, NH, NKV, HD, 16, (int)k.get("splits", 0), nullptr, k.get("pair", 0) ? 2 : 1, exact, qf);
}

// ---- op: argmax (src/model.ts:198-201)   slots: logits, val, idx     params: VOCAB, batch=1
static int run_argmax(Kernel& k, const uint64_t* s) {
  return launch_argmax(P<float>(s[0]), P<float>(s[1]), P<int32_t>(s[2]), k.scratch, (int)k.get("VOCAB", 0), (int)k.get("batch", 1));
}

// ---- op: argmax_feed = argmax + advance + the next step's embed (device-resident loop: two launches instead of four)
// slots: logits, val, idx, token ids, positions, history, counters (int32 [batch], one per sequence), embed.weight, x (next step's input)
// params: VOCAB, H, batch, max_steps, max_pos
static int run_argmax_feed(Kernel& k, const uint64_t* s) {
  return launch_argmax_feed(P<float>(s[0]), P<float>(s[1]), P<int32_t>(s[2]), k.scratch, (int)k.get("VOCAB", 0), (int)k.get("batch", 1),
                            P<int32_t>(s[3]), P<int32_t>(s[4]), P<int32_t>(s[5]), P<int32_t>(s[6]), (int)k.get("max_steps", 0),
                            (int)k.get("max_pos", 0), P<void>(s[7]), P<void>(s[8]), (int)k.get("H", 0));
}

// ---- op: advance   slots: argmax idx, argmax val, token ids, positions, history, counter    params: batch, max_steps, max_pos
// (max_pos = the cache capacity MAX_LEN: positions are not advanced past it, and the cache writers skip a position that reached it)
static int run_advance(Kernel& k, const uint64_t* s) {
  return launch_advance(P<int32_t>(s[0]), P<float>(s[1]), P<int32_t>(s[2]), P<int32_t>(s[3]), P<int32_t>(s[4]), P<int32_t>(s[5]),
                        (int)k.get("batch", 1), (int)k.get("max_steps", 0), (int)k.get("max_pos", 0));
}

static int build_kernel(Kernel& k) {
  int rc;
  struct Simple { const char* op; RunFn run; int nslots; const char* need1; const char* need2; };
  static const Simple simple[] = {
      {"embed", run_embed, 3, "H", "VOCAB"},       {"rmsnorm", run_rmsnorm, 3, "N", nullptr},
      {"rmsnorm_q8_1", run_rmsnorm_q8, 4, "N", nullptr}, {"cast", run_cast, 2, "N", nullptr},
      {"add", run_add, 3, "N", nullptr},            {"swiglu", run_swiglu, 3, "N", nullptr},
      {"conv1d_decode", run_conv1d, 5, "QKVD", nullptr}, {"gdn_delta_rule", run_gdn, 10, "LVH", nullptr},
      {"gdn_conv", run_gdn_conv, 13, "LVH", nullptr},   {"gdn_slabs", run_gdn_slabs, 9, "LVH", nullptr},
      {"qnorm", run_qnorm, 3, "HD", "NH"},          {"knorm", run_knorm, 3, "HD", "NKV"},
      {"rope", run_rope, 4, "HD", "NH"},            {"ropek", run_rope, 4, "HD", "NKV"},
      {"advance", run_advance, 6, "batch", "max_steps"},
  };
  for (const Simple& sp : simple) {
    if (k.op != sp.op) continue;
    if ((rc = need(k, sp.need1))) return rc;
    if (sp.need2 && (rc = need(k, sp.need2))) return rc;
    if (k.op == "rope" || k.op == "ropek") {
      if ((rc = need(k, "ROT_HALF")) || (rc = need(k, "MAX_LEN"))) return rc;
    }
    if (k.op == "advance" && (rc = need(k, "max_pos"))) return rc;
    if (k.op == "gdn_delta_rule" || k.op == "gdn_conv" || k.op == "gdn_slabs")
      BK_REQUIRE(k.get("LKD", 128) == 128 && k.get("LVD", 128) == 128, "gdn_delta_rule: dk = dv = 128 only");
    k.run = sp.run; k.nslots = sp.nslots + (k.op == "gdn_conv" && k.get("q8out", 0) ? 1 : 0);
    return BK_OK;
  }
  if (k.op == "fa2_attn") {
    if ((rc = need(k, "HD")) || (rc = need(k, "NH")) || (rc = need(k, "NKV")) || (rc = need(k, "MAX_LEN"))) return rc;
    const int batch = (int)k.get("batch", 1), NKV = (int)k.get("NKV", 0), max_len = (int)k.get("MAX_LEN", 0);
    BK_REQUIRE(batch >= 1 && NKV >= 1 && max_len >= 1, "fa2_attn: bad batch/NKV/MAX_LEN");
    BK_REQUIRE(max_len % 16 == 0, "fa2_attn: MAX_LEN=%d must be a multiple of the 16-token page (a sequence owns MAX_LEN/16 pages)", max_len);
    int splits = (int)k.get("splits", 0);
    if (splits <= 0) { splits = attn_choose_splits(batch, NKV, max_len); k.p["splits"] = splits; }
    const int exact = (int)k.get("exact", 1);
    BK_REQUIRE(!exact || k.get("NH", 0) / NKV <= 8, "fa2_attn: exact=1 serves at most 8 query heads per KV head (exact=0 takes 16)");
    if ((splits > 1 || exact) && (rc = alloc_scratch(k, fa2_ws_bytes(batch, NKV, splits, exact)))) return rc;
    k.run = run_fa2; k.nslots = 10;
    return BK_OK;
  }
  if (k.op == "fa2_fused") {
    if ((rc = need(k, "HD")) || (rc = need(k, "NH")) || (rc = need(k, "NKV")) || (rc = need(k, "MAX_LEN")) || (rc = need(k, "ROT_HALF"))) return rc;
    const int batch = (int)k.get("batch", 1), NKV = (int)k.get("NKV", 0), max_len = (int)k.get("MAX_LEN", 0);
    BK_REQUIRE(batch >= 1 && NKV >= 1 && max_len >= 1 && k.get("NH", 0) >= 1 && k.get("HD", 0) >= 1, "fa2_fused: bad batch/NH/NKV/HD/MAX_LEN");
    BK_REQUIRE(max_len % 16 == 0, "fa2_fused: MAX_LEN=%d must be a multiple of the 16-token page (a sequence owns MAX_LEN/16 pages)", max_len);
    int splits = (int)k.get("splits", 0);
    if (splits <= 0) { splits = attn_choose_splits(batch, NKV, max_len); k.p["splits"] = splits; }
    const int exact = (int)k.get("exact", 1);
    BK_REQUIRE(!exact || k.get("NH", 0) / NKV <= 8, "fa2_fused: exact=1 serves at most 8 query heads per KV head (exact=0 takes 16)");
    const size_t qbytes = fa2_qn_bytes(batch, (int)k.get("NH", 0), (int)k.get("HD", 0));
    if ((rc = alloc_scratch(k, qbytes + fa2_ws_bytes(batch, NKV, splits, exact)))) return rc;
    if (exact) BK_HIP(hipMemset(k.scratch, 0, k.scratch_bytes));        // columns of the f64 query copy past the group stay zero
    k.run = run_fa2_fused; k.nslots = 11 + (k.get("q8out", 0) ? 1 : 0);
    return BK_OK;
  }
  if (k.op == "conv1d_prefill") {
    if ((rc = need(k, "QKVD")) || (rc = need(k, "T"))) return rc;
    k.run = run_conv1d_prefill; k.nslots = 5;
    return BK_OK;
  }
  if (k.op == "gdn_prefill") {
    if ((rc = need(k, "LVH")) || (rc = need(k, "T"))) return rc;
    BK_REQUIRE(k.get("LVH", 0) >= 1 && k.get("T", 0) >= 1 && k.get("T", 0) <= 65535, "gdn_prefill: bad LVH/T");
    if ((rc = alloc_scratch(k, gdn_prefill_workspace_bytes((int)k.get("LVH", 0), (int)k.get("T", 0), k.get("chunked", 0) != 0)))) return rc;
    k.run = run_gdn_prefill; k.nslots = 10;
    return BK_OK;
  }
  if (k.op == "fa2_prefill") {
    for (const char* p : {"HD", "NH", "NKV", "MAX_LEN", "ROT_HALF", "T"})
      if ((rc = need(k, p))) return rc;
    const int T = (int)k.get("T", 0), NKV = (int)k.get("NKV", 0), max_len = (int)k.get("MAX_LEN", 0);
    BK_REQUIRE(T >= 1 && T <= 65535 && NKV >= 1 && max_len >= 1 && max_len % 16 == 0, "fa2_prefill: bad T/NKV/MAX_LEN (MAX_LEN a multiple of 16)");
    // two consecutive tokens per workgroup where their heads fit the 16 columns of the products (pair=0 switches it off)
    const int NHq = (int)k.get("NH", 0);
    const int exact = (int)k.get("exact", 1);
    BK_REQUIRE(!exact || NHq / NKV <= 8, "fa2_prefill: exact=1 serves at most 8 query heads per KV head (exact=0 takes 16)");
    // (the double-precision kernel takes one token per workgroup)
    // exact=0: query tiles against K/V tiles (attn_prefill.hip) where that kernel serves the shape, unless tiled=0 asks for
    // the decode kernel per token (pair) instead
    const bool tiled = !exact && k.get("tiled", 1) != 0 && attn_prefill_tiled_serves(NHq, NKV, max_len);
    BK_REQUIRE(tiled || k.get("tiled", 0) == 0, "fa2_prefill: tiled=1 needs exact=0 and 1, 2, 4, 8 or 16 query heads per KV head (NH=%d NKV=%d MAX_LEN=%d)",
               NHq, NKV, max_len);
    k.p["tiled"] = tiled;
    const int tpw = (!exact && !tiled && NKV <= NHq && 2 * (NHq / NKV) <= 16 && T >= 2 && k.get("pair", 1) != 0) ? 2 : 1;
    k.p["pair"] = tpw == 2;
    int splits = (int)k.get("splits", 0);
    if (splits <= 0) { splits = attn_choose_splits((T + tpw - 1) / tpw, NKV, max_len); k.p["splits"] = splits; }
    const size_t qbytes = fa2_qn_bytes(T, (int)k.get("NH", 0), (int)k.get("HD", 0));
    const size_t ws_bytes = tiled ? attn_prefill_workspace_bytes(T, NHq, NKV, max_len) : fa2_ws_bytes(T, NKV, splits, exact);
    if ((rc = alloc_scratch(k, qbytes + ws_bytes))) return rc;
    if (exact) BK_HIP(hipMemset(k.scratch, 0, k.scratch_bytes));
    k.run = run_fa2_prefill; k.nslots = 12;
    return BK_OK;
  }
  if (k.op == "argmax") {
    if ((rc = need(k, "VOCAB"))) return rc;
    const int batch = (int)k.get("batch", 1), V = (int)k.get("VOCAB", 0);
    BK_REQUIRE(batch >= 1 && V >= 1, "argmax: bad VOCAB/batch");
    if ((rc = alloc_scratch(k, argmax_workspace_bytes(V, batch)))) return rc;
    k.run = run_argmax; k.nslots = 3;
    return BK_OK;
  }
  if (k.op == "argmax_feed") {
    for (const char* p : {"VOCAB", "H", "max_steps", "max_pos"})
      if ((rc = need(k, p))) return rc;
    const int batch = (int)k.get("batch", 1), V = (int)k.get("VOCAB", 0);
    BK_REQUIRE(batch >= 1 && V >= 1, "argmax_feed: bad VOCAB/batch");
    if ((rc = alloc_scratch(k, argmax_workspace_bytes(V, batch)))) return rc;
    k.run = run_argmax_feed; k.nslots = 9;
    return BK_OK;
  }
  if (k.op == "gemv_fused") return build_gemv_fused(k);
  if (k.op == "quantize_q8_1") {
    if ((rc = need(k, "K"))) return rc;
    k.run = run_quantize; k.nslots = 2;
  } else if (k.op == "gemv_q4k_q8_1") {
    if ((rc = need(k, "N")) || (rc = need(k, "K"))) return rc;
    k.run = run_gemv; k.nslots = 3;
  } else if (k.op == "gemm") {
    if ((rc = need(k, "N")) || (rc = need(k, "K"))) return rc;
    const int64_t K = k.get("K", 0), batch = k.get("batch", 1);
    BK_REQUIRE(K > 0 && K % 256 == 0, "gemm: K=%lld must be a positive multiple of 256", (long long)K);
    BK_REQUIRE(batch >= 1 && batch <= 4096, "gemm: bad batch=%lld", (long long)batch);
    if ((rc = alloc_scratch(k, (size_t)(batch * (K / 32) * 36)))) return rc;
    k.run = run_gemm; k.nslots = 3;
  } else {
    return set_error(BK_ERR_UNSUPPORTED, "no kernel for op '%s'", k.op.c_str());
  }
  return BK_OK;
}

}  // namespace bk

using namespace bk;

extern "C" {

// Tuning hooks for measurements: "gemv_impl" (0 direct loads, 2 rows through LDS), "gemv_rpi" (rows per wave step),
// "gemv_cap" (workgroups per CU), "gemm_nw" (waves per MFMA tile), "memread_*" (calibration read kernel).
int bk_tune_set(const char* key, int value) {
  BK_REQUIRE(key, "bk_tune_set: null key");
  // values that size a grid are checked here: the launchers divide by them
  if (!strcmp(key, "gemv_cap") || !strcmp(key, "memread_cap"))
    BK_REQUIRE(value >= 1 && value <= 1024, "bk_tune_set: %s=%d outside 1..1024", key, value);
  if (!strcmp(key, "gemv_rpi")) BK_REQUIRE(value == 0 || value == 1 || value == 2 || value == 4, "bk_tune_set: gemv_rpi=%d (0, 1, 2 or 4)", value);
  if (!strcmp(key, "gemv_rpi")) bk::g_tune_rpi = value;
  else if (!strcmp(key, "gemv_cap")) bk::g_tune_cap = value;
  else if (!strcmp(key, "gemv_steps")) { BK_REQUIRE(value >= 0 && value <= 1024, "bk_tune_set: gemv_steps=%d outside 0..1024", value); bk::g_tune_steps = value; }
  else if (!strcmp(key, "gemv_impl")) bk::g_tune_gemv_impl = value;
  else if (!strcmp(key, "gdn_cs")) bk::g_tune_gdn_cs = value;
  else if (!strcmp(key, "fused_cap")) bk::g_tune_fused_cap = value;
  else if (!strcmp(key, "attn_nt")) bk::g_tune_attn_nt = value;
  else if (!strcmp(key, "attn_bal")) bk::g_tune_attn_bal = value;
  else if (!strcmp(key, "prefill_xmap")) bk::g_tune_prefill_xmap = value != 0;
  else if (!strcmp(key, "prefill_ksplit")) { BK_REQUIRE(value >= 0 && value <= 4, "bk_tune_set: prefill_ksplit=%d outside 0..4", value); bk::g_tune_prefill_ksplit = value; }
  else if (!strcmp(key, "gemm_r16")) bk::g_tune_gemm_r16 = value;
  else if (!strcmp(key, "small_rows")) bk::g_tune_small_rows = value;
  else if (!strcmp(key, "gdn_nt")) bk::g_tune_gdn_nt = value;
  else if (!strcmp(key, "gemm_nw")) bk::g_tune_gemm_nw = value;
  else if (!strcmp(key, "memread_unroll")) bk::g_tune_mr_unroll = value;
  else if (!strcmp(key, "memread_cap")) bk::g_tune_mr_cap = value;
  else if (!strcmp(key, "memread_nt")) bk::g_tune_mr_nt = value;
  else return set_error(BK_ERR_ARG, "bk_tune_set: unknown key '%s'", key);
  return BK_OK;
}

int bk_kernel_create(const char* spec) {
  BK_NEED_INIT();
  if (capturing()) return set_error(BK_ERR_STATE, "bk_kernel_create: not legal between bk_capture_begin and bk_capture_end");
  BK_REQUIRE(spec && *spec, "bk_kernel_create: empty spec");
  Kernel k;
  k.spec = spec;
  std::istringstream in(spec);
  std::string tok;
  if (!(in >> k.op)) return set_error(BK_ERR_ARG, "bk_kernel_create: empty spec");
  while (in >> tok) {
    size_t eq = tok.find('=');
    if (eq == std::string::npos || eq == 0 || eq + 1 >= tok.size())
      return set_error(BK_ERR_ARG, "bk_kernel_create: expected key=value, got '%s'", tok.c_str());
    char* end = nullptr;
    long long v = strtoll(tok.c_str() + eq + 1, &end, 10);
    if (*end) return set_error(BK_ERR_ARG, "bk_kernel_create: '%s' is not an integer", tok.c_str());
    k.p[tok.substr(0, eq)] = v;
  }
  int rc = build_kernel(k);
  if (rc) {
    if (k.scratch) (void)hipFree(k.scratch);
    return rc;
  }
  // a destroyed handle's slot is taken again (a server that builds a loop per request would otherwise grow the table
  // without bound); the generation in the upper bits makes a stale handle number an error instead of another kernel
  if (!g_free_slots.empty()) {
    const int slot = g_free_slots.back();
    g_free_slots.pop_back();
    k.generation = g_kernels[slot].generation + 1;
    g_kernels[slot] = k;
    return handle_of(slot);
  }
  BK_REQUIRE(g_kernels.size() < (size_t)HANDLE_SLOTS, "bk_kernel_create: more than %d live handles", HANDLE_SLOTS);
  g_kernels.push_back(k);
  return handle_of((int)g_kernels.size() - 1);
}

int bk_launch(int kernel, const uint64_t* slots, int nslots) {
  BK_NEED_INIT();
  Kernel* kp = kernel_of(kernel);
  if (!kp) return set_error(BK_ERR_STATE, "bk_launch: unknown or destroyed kernel handle %d", kernel);
  Kernel& k = *kp;
  BK_REQUIRE(slots, "bk_launch: null slots");
  BK_REQUIRE(nslots >= k.nslots, "bk_launch: '%s' takes %d argument slots, got %d", k.op.c_str(), k.nslots, nslots);
  if (prof_on()) {
    int rc = prof_begin(kernel);
    if (rc) return rc;
    rc = k.run(k, slots);
    int rc2 = prof_end();
    return rc ? rc : rc2;
  }
  return k.run(k, slots);
}

int bk_kernel_destroy(int kernel) {
  BK_NEED_INIT();
  if (capturing()) return set_error(BK_ERR_STATE, "bk_kernel_destroy: not legal between bk_capture_begin and bk_capture_end");
  const int slot = kernel & (HANDLE_SLOTS - 1);
  if (kernel < 0 || slot >= (int)g_kernels.size()) return set_error(BK_ERR_STATE, "bk_kernel_destroy: unknown kernel handle %d", kernel);
  Kernel& k = g_kernels[slot];
  if (!k.run || handle_of(slot) != kernel) return BK_OK;      // destroyed before
  if (k.scratch) {
    BK_HIP(hipDeviceSynchronize());               // launches that still use the workspace finish first
    BK_HIP(hipFree(k.scratch));
  }
  k.scratch = nullptr; k.scratch_bytes = 0; k.run = nullptr;
  k.p.clear();
  k.spec = k.op + " [destroyed]";
  g_free_slots.push_back(slot);
  return BK_OK;
}

int bk_kernel_describe(int kernel, char* buf, int cap) {
  BK_REQUIRE(buf && cap > 0, "bk_kernel_describe: bad buffer");
  const int slot = kernel & (HANDLE_SLOTS - 1);
  if (kernel < 0 || slot >= (int)g_kernels.size() || handle_of(slot) != kernel)
    return set_error(BK_ERR_STATE, "unknown kernel handle %d", kernel);
  snprintf(buf, cap, "%s [%d slots]", g_kernels[slot].spec.c_str(), g_kernels[slot].nslots);
  return BK_OK;
}

int bk_memread(uint64_t src, int64_t bytes, uint64_t sink) {
  BK_NEED_INIT();
  return launch_memread(P<void>(src), bytes, P<void>(sink));
}
int bk_memcopy(uint64_t src, uint64_t dst, int64_t bytes) {
  BK_NEED_INIT();
  return launch_memcopy(P<void>(src), P<void>(dst), bytes);
}
int bk_quantize_q8_1(uint64_t x, int x_dtype, uint64_t out, int K, int batch) {
  BK_NEED_INIT();
  return launch_quantize_q8_1(P<void>(x), x_dtype, P<void>(out), K, batch);
}
int bk_quantize_q4k(uint64_t w, int w_dtype, uint64_t out, int64_t rows, int K) {
  BK_NEED_INIT();
  return launch_quantize_q4k(P<void>(w), w_dtype, P<void>(out), rows, K);
}
int bk_gemv_q4k_f32(uint64_t W, uint64_t x, uint64_t y, int N, int K) {
  BK_NEED_INIT();
  return launch_gemv_q4k_f32(P<void>(W), P<float>(x), P<float>(y), N, K);
}
int bk_gemv_q4k_q8_1(uint64_t W, uint64_t xq, uint64_t y, int N, int K, int batch, int out_dtype, uint64_t residual) {
  BK_NEED_INIT();
  return launch_gemv_q4k_q8_1(P<void>(W), P<void>(xq), P<void>(y), N, K, batch, out_dtype, P<void>(residual));
}
int bk_gemm_q4k_q8_1(uint64_t W, uint64_t xq, uint64_t y, int N, int K, int batch, int out_dtype, uint64_t residual) {
  BK_NEED_INIT();
  return matmul_q8_1(P<void>(W), P<void>(xq), P<void>(y), N, K, batch, out_dtype, P<void>(residual), 1);
}
int bk_q4k_q8_1_subdots(uint64_t W, uint64_t xq, uint64_t I, int N, int K) {
  BK_NEED_INIT();
  return launch_q4k_q8_1_subdots(P<void>(W), P<void>(xq), P<int32_t>(I), N, K);
}
int bk_dequant_legacy_i8(uint64_t blocks, uint64_t out, int64_t nblocks) {
  BK_NEED_INIT();
  return launch_dequant_legacy_i8(P<void>(blocks), P<void>(out), nblocks);
}
int bk_q4k_nibbles(uint64_t blocks, uint64_t out, int64_t nblocks) {
  BK_NEED_INIT();
  return launch_q4k_nibbles(P<void>(blocks), P<void>(out), nblocks);
}
int bk_q4k_dequant_f32(uint64_t blocks, uint64_t out, int64_t nblocks) {
  BK_NEED_INIT();
  return launch_q4k_dequant_f32(P<void>(blocks), P<void>(out), nblocks);
}

int bk_gdn_core(uint64_t q, uint64_t k, uint64_t v, uint64_t g, uint64_t beta, uint64_t S_in, uint64_t out, uint64_t S_out,
                int Hg, int batch) {
  BK_NEED_INIT();
  return launch_gdn_core(P<void>(q), P<void>(k), P<void>(v), P<float>(g), P<float>(beta), P<float>(S_in), P<void>(out),
                         P<float>(S_out), Hg, batch);
}
int bk_attn_plan(int batch, int NKV, int max_ctx, int* splits, uint64_t* workspace_bytes) {
  BK_NEED_INIT();
  BK_REQUIRE(splits && workspace_bytes, "bk_attn_plan: null out");
  BK_REQUIRE(batch > 0 && NKV > 0 && max_ctx > 0, "bk_attn_plan: bad shape");
  int s = *splits > 0 ? *splits : attn_choose_splits(batch, NKV, max_ctx);
  const int pages = (max_ctx + 15) / 16;
  if (s > pages) s = pages;
  *splits = s;
  *workspace_bytes = s > 1 ? attn_workspace_bytes(batch, NKV, s) : 0;
  return BK_OK;
}
int bk_attn_decode(uint64_t q, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride, uint64_t ctx_len, int max_ctx,
                   uint64_t gate, int64_t gate_bstride, int64_t gate_hstride, uint64_t out, uint64_t lse, uint64_t workspace,
                   uint64_t workspace_bytes, int batch, int NH, int NKV, int HD, int page_size, int splits) {
  BK_NEED_INIT();
  BK_REQUIRE(ctx_len, "bk_attn_decode: ctx_len is required");
  return launch_attn_decode(P<void>(q), P<void>(kc), P<void>(vc), P<int32_t>(block_table), bt_stride, P<int32_t>(ctx_len), 0, 0,
                            max_ctx, P<void>(gate), gate_bstride, gate_hstride, P<void>(out), P<float>(lse), P<void>(workspace),
                            (size_t)workspace_bytes, batch, NH, NKV, HD, page_size, splits);
}
int bk_attn_plan_exact(int batch, int NKV, int max_ctx, int* splits, uint64_t* workspace_bytes) {
  BK_NEED_INIT();
  BK_REQUIRE(splits && workspace_bytes, "bk_attn_plan_exact: null out");
  BK_REQUIRE(batch > 0 && NKV > 0 && max_ctx > 0, "bk_attn_plan_exact: bad shape");
  int s = *splits > 0 ? *splits : attn_choose_splits(batch, NKV, max_ctx);
  const int pages = (max_ctx + 15) / 16;
  if (s > pages) s = pages;
  *splits = s;
  *workspace_bytes = attn_exact_workspace_bytes(batch, NKV, s > 1 ? s : 0);
  return BK_OK;
}
int bk_attn_decode_exact(uint64_t q, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride, uint64_t ctx_len, int max_ctx,
                         uint64_t gate, int64_t gate_bstride, int64_t gate_hstride, uint64_t out, uint64_t lse, uint64_t workspace,
                         uint64_t workspace_bytes, int batch, int NH, int NKV, int HD, int page_size, int splits) {
  BK_NEED_INIT();
  BK_REQUIRE(ctx_len, "bk_attn_decode_exact: ctx_len is required");
  return launch_attn_decode(P<void>(q), P<void>(kc), P<void>(vc), P<int32_t>(block_table), bt_stride, P<int32_t>(ctx_len), 0, 0,
                            max_ctx, P<void>(gate), gate_bstride, gate_hstride, P<void>(out), P<float>(lse), P<void>(workspace),
                            (size_t)workspace_bytes, batch, NH, NKV, HD, page_size, splits, nullptr, 1, 1, nullptr);
}
int bk_attn_decode_noalloc(uint64_t q, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride, uint64_t ctx_len, int max_ctx,
                           uint64_t gate, int64_t gate_bstride, int64_t gate_hstride, uint64_t out, uint64_t lse, int batch, int NH,
                           int NKV, int HD, int page_size, int splits) {
  BK_NEED_INIT();
  BK_REQUIRE(ctx_len, "bk_attn_decode_noalloc: ctx_len is required");
  return launch_attn_decode_noalloc(current_device(), P<void>(q), P<void>(kc), P<void>(vc), P<int32_t>(block_table), bt_stride,
                                    P<int32_t>(ctx_len), max_ctx, P<void>(gate), gate_bstride, gate_hstride, P<void>(out), P<float>(lse),
                                    batch, NH, NKV, HD, page_size, splits);
}
int bk_kv_append(uint64_t k, uint64_t v, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride, uint64_t pos, int max_len,
                 int batch, int NKV, int HD, int page_size) {
  BK_NEED_INIT();
  BK_REQUIRE(pos, "bk_kv_append: pos is required");
  return launch_kv_append(P<void>(k), P<void>(v), P<void>(kc), P<void>(vc), P<int32_t>(block_table), bt_stride, P<int32_t>(pos), 0,
                          max_len, batch, NKV, HD, page_size);
}

}  // extern "C"
