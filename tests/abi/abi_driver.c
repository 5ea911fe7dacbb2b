/* A plain C99 caller of libbunker_hip.so: includes the public header, links the library, and drives the Q8_1
 * quantizer and the Q4_K x Q8_1 GEMV through both launch surfaces (typed entry points and bk_kernel_create /
 * bk_launch with cuLaunch-style 8-byte slots, src/ttir.ts:321-348).  The compiler checks every call against the
 * declarations of include/bunker_hip.h, which a ctypes binding cannot do.
 *
 * usage: abi_driver <input.bin>
 *   input.bin: int32 N, int32 K, then N*K/256*144 bytes of Q4_K super-blocks, then K f32 activations.
 * prints:  "xq <hex of K/32 Q8_1 blocks>", "y <N f32 bit patterns as hex>", "y_launch <the same via bk_launch>",
 *          "subdot0 <K/32 int32 of row 0>"; exit code 0.  Exit code 2 with "ERROR: ..." when a call fails. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "bunker_hip.h"

#define CHECK(call)                                                             \
  do {                                                                          \
    int rc_ = (call);                                                           \
    if (rc_ != 0) {                                                             \
      printf("ERROR: %s -> %d: %s\n", #call, rc_, bk_last_error());             \
      return 2;                                                                 \
    }                                                                           \
  } while (0)

static void print_hex(const char* tag, const unsigned char* p, size_t n) {
  size_t i;
  printf("%s ", tag);
  for (i = 0; i < n; i++) printf("%02x", p[i]);
  printf("\n");
}

static void print_words(const char* tag, const uint32_t* p, size_t n) {
  size_t i;
  printf("%s", tag);
  for (i = 0; i < n; i++) printf(" %08x", p[i]);
  printf("\n");
}

int main(int argc, char** argv) {
  int32_t dims[2];
  int N, K, kernel;
  size_t wbytes, qbytes;
  unsigned char *W, *xq;
  float* x;
  uint32_t *y, *sub;
  uint64_t dW = 0, dx = 0, dxq = 0, dy = 0, dy2 = 0, dsub = 0, slots[3];
  char spec[96], info[256];
  FILE* f;

  if (argc != 2) { printf("ERROR: usage: abi_driver <input.bin>\n"); return 2; }
  f = fopen(argv[1], "rb");
  if (!f) { printf("ERROR: cannot open %s\n", argv[1]); return 2; }
  if (fread(dims, sizeof(int32_t), 2, f) != 2) { printf("ERROR: short header\n"); return 2; }
  N = dims[0]; K = dims[1];
  if (N <= 0 || K <= 0 || K % 256 != 0) { printf("ERROR: bad shape %d x %d\n", N, K); return 2; }
  wbytes = (size_t)N * (size_t)(K / 256) * 144u;
  qbytes = (size_t)(K / 32) * 36u;
  W = (unsigned char*)malloc(wbytes); x = (float*)malloc((size_t)K * 4u);
  xq = (unsigned char*)malloc(qbytes); y = (uint32_t*)malloc((size_t)N * 4u); sub = (uint32_t*)malloc((size_t)(K / 32) * 4u);
  if (!W || !x || !xq || !y || !sub) { printf("ERROR: out of memory\n"); return 2; }
  if (fread(W, 1, wbytes, f) != wbytes || fread(x, 4, (size_t)K, f) != (size_t)K) { printf("ERROR: short input\n"); return 2; }
  fclose(f);

  CHECK(bk_init(0));
  CHECK(bk_device_info(info, (int)sizeof info));
  printf("device %s\n", info);
  CHECK(bk_alloc(wbytes, &dW)); CHECK(bk_alloc((uint64_t)K * 4u, &dx)); CHECK(bk_alloc(qbytes, &dxq));
  CHECK(bk_alloc((uint64_t)N * 4u, &dy)); CHECK(bk_alloc((uint64_t)N * 4u, &dy2));
  CHECK(bk_alloc((uint64_t)N * (uint64_t)(K / 32) * 4u, &dsub));
  CHECK(bk_htod(dW, W, wbytes)); CHECK(bk_htod(dx, x, (uint64_t)K * 4u));

  /* typed entry points */
  CHECK(bk_quantize_q8_1(dx, 0, dxq, K, 1));
  CHECK(bk_gemv_q4k_q8_1(dW, dxq, dy, N, K, 1, 0, 0));
  CHECK(bk_q4k_q8_1_subdots(dW, dxq, dsub, N, K));
  CHECK(bk_sync());
  CHECK(bk_dtoh(xq, dxq, qbytes)); print_hex("xq", xq, qbytes);
  CHECK(bk_dtoh(y, dy, (uint64_t)N * 4u)); print_words("y", y, (size_t)N);
  CHECK(bk_dtoh(sub, dsub, (uint64_t)(K / 32) * 4u)); print_words("subdot0", sub, (size_t)(K / 32));

  /* the reference's surface: compileAndLoad -> handle, cuLaunch -> 8-byte slots (W, xq, y) */
  snprintf(spec, sizeof spec, "gemv_q4k_q8_1 N=%d K=%d", N, K);
  kernel = bk_kernel_create(spec);
  if (kernel < 0) { printf("ERROR: bk_kernel_create(\"%s\") -> %d: %s\n", spec, kernel, bk_last_error()); return 2; }
  slots[0] = dW; slots[1] = dxq; slots[2] = dy2;
  CHECK(bk_launch(kernel, slots, 3));
  CHECK(bk_sync());
  CHECK(bk_dtoh(y, dy2, (uint64_t)N * 4u)); print_words("y_launch", y, (size_t)N);
  CHECK(bk_kernel_destroy(kernel));

  /* an error must come back as a code and a message, not as a crash */
  if (bk_gemv_q4k_q8_1(dW, dxq, dy, N, K + 1, 1, 0, 0) == 0) { printf("ERROR: K not a multiple of 256 was accepted\n"); return 2; }
  printf("refused %s\n", bk_last_error());

  CHECK(bk_free(dW)); CHECK(bk_free(dx)); CHECK(bk_free(dxq)); CHECK(bk_free(dy)); CHECK(bk_free(dy2)); CHECK(bk_free(dsub));
  CHECK(bk_shutdown());
  free(W); free(x); free(xq); free(y); free(sub);
  printf("ok\n");
  return 0;
}
