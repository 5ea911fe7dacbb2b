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
  int64_t get(const char* k, int64_t def) const {
    auto it = p.find(k);
    return it == p.end() ? def : it->second;
  }
  bool has(const char* k) const { return p.count(k) != 0; }
};

static std::vector<Kernel> g_kernels;

std::string kernel_label(int kernel) {
  if (kernel < 0 || kernel >= (int)g_kernels.size()) return "?";
  return g_kernels[kernel].spec;
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
static int run_gemm(Kernel& k, const uint64_t* s) {
  const int N = (int)k.get("N", 0), K = (int)k.get("K", 0), batch = (int)k.get("batch", 1);
  int rc = launch_quantize_q8_1(P<void>(s[0]), DT_BF16, k.scratch, K, batch);
  if (rc) return rc;
  return launch_gemv_q4k_q8_1(P<void>(s[1]), k.scratch, P<void>(s[2]), N, K, batch, (int)k.get("cast", 0), nullptr);
}

static int build_kernel(Kernel& k) {
  int rc;
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

int bk_kernel_create(const char* spec) {
  BK_NEED_INIT();
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
  g_kernels.push_back(k);
  return (int)g_kernels.size() - 1;
}

int bk_launch(int kernel, const uint64_t* slots, int nslots) {
  BK_NEED_INIT();
  if (kernel < 0 || kernel >= (int)g_kernels.size()) return set_error(BK_ERR_STATE, "bk_launch: unknown kernel handle %d", kernel);
  Kernel& k = g_kernels[kernel];
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

int bk_kernel_describe(int kernel, char* buf, int cap) {
  if (kernel < 0 || kernel >= (int)g_kernels.size()) return set_error(BK_ERR_STATE, "unknown kernel handle %d", kernel);
  BK_REQUIRE(buf && cap > 0, "bk_kernel_describe: bad buffer");
  snprintf(buf, cap, "%s [%d slots]", g_kernels[kernel].spec.c_str(), g_kernels[kernel].nslots);
  return BK_OK;
}

int bk_quantize_q8_1(uint64_t x, int x_dtype, uint64_t out, int K, int batch) {
  BK_NEED_INIT();
  return launch_quantize_q8_1(P<void>(x), x_dtype, P<void>(out), K, batch);
}
int bk_gemv_q4k_f32(uint64_t W, uint64_t x, uint64_t y, int N, int K) {
  BK_NEED_INIT();
  return launch_gemv_q4k_f32(P<void>(W), P<float>(x), P<float>(y), N, K);
}
int bk_gemv_q4k_q8_1(uint64_t W, uint64_t xq, uint64_t y, int N, int K, int batch, int out_dtype, uint64_t residual) {
  BK_NEED_INIT();
  return launch_gemv_q4k_q8_1(P<void>(W), P<void>(xq), P<void>(y), N, K, batch, out_dtype, P<void>(residual));
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

}  // extern "C"
