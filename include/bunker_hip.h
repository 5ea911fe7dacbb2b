/*
 * bunker_hip.h — C ABI of libbunker_hip.so: bunker's Qwen3.5 single-token decode
 * hot path as pre-compiled gfx950 (MI355X) HIP kernels.
 *
 * The library replaces, for this path only, the two native boundaries of the
 * reference: the Triton shim (shim/triton_shim.c:139-141, bound at
 * src/ttir.ts:137-141) and the CUDA driver binding (src/ttir.ts:225-248), and it
 * carries the kernels that src/emitters.ts and src/fusion.ts:264-355 used to
 * generate.  Conventions, chosen so that bun:ffi, ctypes and plain C can all
 * bind it:
 *   - only scalars and raw pointers cross the boundary, never structs;
 *   - device pointers are uint64_t (bun passes bigint, src/ttir.ts:266-271);
 *   - every function returns int32: 0 = ok, < 0 = error; bk_last_error() then
 *     returns a message owned by the library (thread-local, never freed by the
 *     caller);
 *   - launches are asynchronous on the selected stream of the library (its first
 *     stream unless bk_stream_use chose another); bk_sync() waits for all of them;
 *   - single-threaded use, like the reference (one JS thread, one context): the
 *     selected stream, an open capture, the kernel handles and the profiler table
 *     are state of the process, not of a thread.  A host with several threads
 *     must call the library from one of them (or under one lock); only
 *     bk_last_error()'s message is kept per thread.
 */
#ifndef BUNKER_HIP_H
#define BUNKER_HIP_H

#include <stdint.h>

#if defined(__GNUC__)
#define BK_API __attribute__((visibility("default")))
#else
#define BK_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* ---- runtime: replaces cu()/cuAlloc/cuHtoD/cuDtoH/cuFree/cuSync (src/ttir.ts:225-285) */
BK_API int bk_init(int device);                      /* cuInit + cuCtxCreate, src/ttir.ts:249-258 */
BK_API int bk_shutdown(void);
BK_API const char* bk_last_error(void);              /* the "ERROR:" string of triton_shim.c:146-149 */
BK_API int bk_device_info(char* buf, int cap);       /* "name|gcnArch|CUs|bytes" for logs */
BK_API int bk_alloc(uint64_t bytes, uint64_t* out);  /* cuAlloc, src/ttir.ts:266-271 */
BK_API int bk_free(uint64_t ptr);                    /* cuFree, src/ttir.ts:283 */
BK_API int bk_htod(uint64_t dst, const void* src, uint64_t bytes);   /* cuHtoD, src/ttir.ts:273-276 */
BK_API int bk_dtoh(void* dst, uint64_t src, uint64_t bytes);         /* cuDtoH, src/ttir.ts:278-281 */
BK_API int bk_dtod(uint64_t dst, uint64_t src, uint64_t bytes);
BK_API int bk_memset(uint64_t dst, int value, uint64_t bytes);
BK_API int bk_sync(void);                            /* cuSync, src/ttir.ts:285 */
/* Pinned host staging and copies that do not wait (cuHtoDAsync / cuDtoHAsync, src/ttir.ts:305-317):
 * enqueued on the library's stream; the host buffer must stay untouched until bk_sync or an event
 * recorded after the copy has been waited for (bk_event_sync). */
BK_API int bk_host_alloc(uint64_t bytes, uint64_t* out);
BK_API int bk_host_free(uint64_t ptr);
BK_API int bk_htod_async(uint64_t dst, const void* src, uint64_t bytes);
BK_API int bk_dtoh_async(void* dst, uint64_t src, uint64_t bytes);

/* ---- timing: replaces the cuEvent* calls of src/ttir.ts:352-417 */
BK_API int bk_event_create(uint64_t* out);
BK_API int bk_event_record(uint64_t ev);             /* on the selected stream */
BK_API int bk_event_elapsed_ms(uint64_t start, uint64_t stop, float* ms);  /* waits for stop */
BK_API int bk_event_sync(uint64_t ev);                /* host waits until the event has happened */
BK_API int bk_event_destroy(uint64_t ev);
/* Further streams for work that may overlap (the reference runs everything on stream 0, src/ttir.ts:321-348, and its
 * prompt prototypes have no counterpart): after bk_stream_use(s) launches, copies and bk_event_record go to stream s
 * (0 = the library's first stream); bk_stream_wait_event makes the selected stream wait for an event recorded on
 * another one.  bk_sync and bk_free wait for all streams.  Single host thread, like every other call here. */
BK_API int bk_stream_create(uint64_t* out);
BK_API int bk_stream_use(uint64_t stream);
BK_API int bk_stream_wait_event(uint64_t ev);
BK_API int bk_stream_destroy(uint64_t stream);
BK_API int bk_prof_enable(int on);                   /* BUNKER_GPU_PROF=1: an event pair around every bk_launch */
BK_API int bk_prof_reset(void);                      /* profGpuReset, src/ttir.ts:385-388 */
BK_API int bk_prof_report(char* buf, int cap);       /* profGpuReport, src/ttir.ts:391-417; text table */

/* ---- launch-overhead removal: record everything enqueued between begin and end
 * into a HIP graph (stream capture) and replay it with one call.  The reference
 * tried the same with CUDA graphs through bun:ffi and gave up on struct-pointer
 * crashes (LOG.md:710-738); here the graph lives behind scalar handles.
 * Between begin and end only launches are legal: alloc, free, memset, copies,
 * sync, event waits, a stream switch, a graph launch, bk_kernel_create and
 * bk_kernel_destroy (they allocate, clear and free a handle's workspace) return
 * an error (state -3, "not legal between bk_capture_begin and bk_capture_end")
 * and leave the capture open. */
BK_API int bk_capture_begin(void);
BK_API int bk_capture_end(uint64_t* graph);
BK_API int bk_graph_launch(uint64_t graph);
BK_API int bk_graph_destroy(uint64_t graph);
/* Number of kernel launches the graph replays (one op may be several: a batched matmul is a quantizer launch and a
 * matrix launch).  For reports; the reference counts launches per step by hand (LOG.md:580). */
BK_API int bk_graph_node_count(uint64_t graph, int* count);

/* Launch-shape knobs for experiments and tests; the defaults (0, or -1 = chosen from the shape) are the tuned values:
 * "gemv_rpi", "gemv_cap", "gemv_steps", "gemv_impl", "fused_cap" (GEMV rows per wave step, workgroups per CU up to
 * which a wave takes one step, row steps per wave, kernel variant),
 * "gemm_nw" (waves per matmul tile: 1, 2, 4, 8), "gemm_r16" (narrow matmul tiles: 1 = 16 weight rows, 2 = 8), "small_rows" (0: the two 16-row
 * matrices of a batched projection group stay in the matmul instead of the norm's launch), "gdn_cs" (column slabs of the
 * GDN core op), "gdn_nt" / "attn_nt" (state / cache pages through nontemporal accesses), "attn_bal" (attention splits
 * under lengths in device memory: 0 = equal ranges of max_ctx, 2 = of each sequence's own length, 1 = the batch's
 * workgroups shared out by length, -1 = 1 for long ranges, else 2), "prefill_ksplit" (runs along K/V of the tiled prompt
 * attention, 1..4; 0 = from the shape; read when an fa2_prefill handle is created), "prefill_xmap" (0: that kernel's workgroups in grid
 * order instead of grouped by XCD).  No counterpart in the reference. */
BK_API int bk_tune_set(const char* key, int value);

/* ---- per-op launch surface: replaces compileAndLoad + cuLaunch
 * (src/ttir.ts:488-491, 321-348).  bk_kernel_create takes the op name of the
 * model graph (src/model.ts) and the constants that the reference baked into
 * the TTIR text, e.g. "gemm N=6144 K=2048 cast=1", and returns a handle >= 0
 * (the LoadedKernel.fn of the reference).  bk_launch takes the same 8-byte
 * argument slots cuLaunch packs, in the same order (pointers as u64, i32
 * scalars in the low 4 bytes); grid and block are the kernel's own business. */
BK_API int bk_kernel_create(const char* spec);
BK_API int bk_launch(int kernel, const uint64_t* slots, int nslots);
/* Handles of ops with intermediate results (gemm, gemv_fused, fa2_*, argmax, gdn_prefill) own a device workspace,
 * allocated by bk_kernel_create.  bk_kernel_destroy waits for the device, returns the workspace and makes the handle
 * invalid: its slot is taken again by a later bk_kernel_create under a new handle number (slot | generation << 20), so
 * a process that builds and destroys handles per request does not grow the table, and a handle kept past its destroy
 * is refused instead of naming another kernel; bk_shutdown releases every handle and every graph of bk_capture_end
 * that was not destroyed.  cuModuleUnload is the reference's nearest counterpart (its kernels own no device memory,
 * src/ttir.ts:488-491). */
BK_API int bk_kernel_destroy(int kernel);
BK_API int bk_kernel_describe(int kernel, char* buf, int cap);

/* Calibration kernels: a plain streaming read (16 bytes per lane, result discarded into the
 * 4-byte sink) and a plain copy, both of `bytes` (multiple of 16).  They give the achievable
 * HBM rate next to the GEMV's and the scale of the FETCH_SIZE / WRITE_SIZE counters. */
BK_API int bk_memread(uint64_t src, int64_t bytes, uint64_t sink);
BK_API int bk_memcopy(uint64_t src, uint64_t dst, int64_t bytes);

/* ---- typed entry points (C / ctypes drivers, parity tests, benchmark) ---- */

/* Q8_1 activation quantizer: packQ8_1, bench/bench.ts:53-72 (host-only in the
 * reference).  x is [batch, K] f32 (x_dtype 0) or bf16 (1); out is
 * [batch, K/32] blocks of 36 bytes: int8 q[32] @0, fp16 d @32, fp16 s @34. */
BK_API int bk_quantize_q8_1(uint64_t x, int x_dtype, uint64_t out, int K, int batch);

/* Weight quantizer, run once at model load: w is [rows, K] f32 (w_dtype 0) or bf16 (1),
 * K a multiple of 256; out is rows * K/256 super-blocks of 144 bytes, row-major.  The
 * reference quantizes weights only into its legacy 20-byte block (packQ4_K_col,
 * bench/bench.ts:74-96) from the bf16 checkpoint tensors its loaders place on the device
 * (prototypes/safetensors_loader.ts:13-78, prototypes/decode.ts:64-75); for the super-block this
 * is the published ggml fit (quantize_row_q4_K_ref / make_qkx2_quants), evaluated per sub-block
 * in the host loop's own operation order so the bytes equal a host run's. */
BK_API int bk_quantize_q4k(uint64_t w, int w_dtype, uint64_t out, int64_t rows, int K);

/* Q4_K dequantize + f32 GEMV on 144-byte super-blocks: y[N] = W[N,K] . x[K],
 * x f32.  The dequant-then-dot the reference's CPU path computes (packers and
 * dot of bench/bench.ts:10-96) with no activation quantization. */
BK_API int bk_gemv_q4k_f32(uint64_t W, uint64_t x, uint64_t y, int N, int K);

/* Q4_K x Q8_1 GEMV: qmm, bench/bench.ts:10-38, on super-blocks; the decode
 * path's M=1 "gemm" (src/fusion.ts:276-293, prototypes/decode.ts:123-186).
 * y is f32 [batch, N] (out_dtype 0) or bf16 (1, the graph's cast=true);
 * residual (0 or bf16 [batch, N]) is added after the bf16 rounding, giving
 * bf16(f32(bf16(acc)) + f32(res)): model.ts:110-117's gemm -> cast -> add. */
BK_API int bk_gemv_q4k_q8_1(uint64_t W, uint64_t xq, uint64_t y, int N, int K, int batch,
                     int out_dtype, uint64_t residual);

/* The same product for a batch of activation rows on the int8 matrix cores
 * (v_mfma_i32_32x32x32_i8: one 32-element sub-block of K per instruction, 32 batch
 * rows x 32 weight rows per tile); precedent: int8MatmulTTIR, src/kernel.ts:397-417,
 * with the post-scale of experiments/q4k_q81_final.ts:214-217.  Arguments as
 * bk_gemv_q4k_q8_1; returns the same bits as that function for every batch row. */
BK_API int bk_gemm_q4k_q8_1(uint64_t W, uint64_t xq, uint64_t y, int N, int K, int batch,
                            int out_dtype, uint64_t residual);

/* Exact int32 sub-block dots I[N, K/32] of the same product (parity hook). */
BK_API int bk_q4k_q8_1_subdots(uint64_t W, uint64_t xq, uint64_t I, int N, int K);

/* Nibble dequant kernels: DequantKernel, src/kernel.ts:584-713.
 * legacy: 20-byte blocks -> int8 (nib-8), interleaved lo/hi (tests/test_dequant.ts:13-24).
 * q4k:    144-byte super-blocks -> uint8 nibbles in element order, or f32 weights. */
BK_API int bk_dequant_legacy_i8(uint64_t blocks, uint64_t out, int64_t nblocks);
BK_API int bk_q4k_nibbles(uint64_t blocks, uint64_t out, int64_t nblocks);
BK_API int bk_q4k_dequant_f32(uint64_t blocks, uint64_t out, int64_t nblocks);

/* Gated DeltaNet single-token update, core recurrence (prototypes/gdn_gated.ts:67-88
 * refGDN at T=1 with the delta-rule beta of src/emitters.ts:105):
 *   S' = exp(g)*S + k (x) ((v - (exp(g)*S)^T k) * beta),  o = S'^T q  -> bf16.
 * q, k, v bf16 [batch, Hg, 128] (q, k already normalised); g, beta f32 [batch, Hg];
 * S f32 [batch, Hg, 128, 128]; S_out may alias S_in.  The fused form of the decode
 * step (norms, gates, gated RMSNorm; src/emitters.ts:75-120) is the "gdn_delta_rule"
 * op of bk_kernel_create. */
BK_API int bk_gdn_core(uint64_t q, uint64_t k, uint64_t v, uint64_t g, uint64_t beta, uint64_t S_in,
                       uint64_t out, uint64_t S_out, int Hg, int batch);

/* Split-K decode attention over a paged bf16 GQA cache: the math of emitFA2Attn
 * (src/emitters.ts:188-226) and refAttn (prototypes/fa2_vllm.ts:114-139) for one
 * query token per sequence, plus lse = max + ln(sum exp).
 * q bf16 [batch, NH, 256]; out bf16 [batch, NH, 256]; lse f32 [batch, NH] or 0.
 * Cache: 16-token pages; K page (p, kv head h) is bf16 [16][256] and V page is
 * bf16 [256][16] (dim-major), both at element offset (p*NKV + h)*4096.
 * block_table int32 [batch, bt_stride] (0 = sequence b owns pages b*bt_stride..),
 * ctx_len int32 [batch].  gate: 0, or bf16 with the gate of (b, head, i) at
 * gate[b*gate_bstride + head*gate_hstride + i] (output *= sigmoid(gate)).
 * splits: 0 = let the library choose; with more than one split the caller passes
 * a workspace of the size bk_attn_plan() returns.  max_ctx bounds the lengths (and the
 * block table); the page ranges of the splits follow the lengths found in ctx_len
 * at run time, so a bound far above the contexts costs nothing.
 * Lengths live in device memory, so the host cannot check them: a length above max_ctx is
 * read as max_ctx (no page beyond the block table row is touched); a length <= 0 gives
 * an all-zero output row and lse = -inf. */
BK_API int bk_attn_plan(int batch, int NKV, int max_ctx, int* splits, uint64_t* workspace_bytes);
BK_API int bk_attn_decode(uint64_t q, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride,
                          uint64_t ctx_len, int max_ctx, uint64_t gate, int64_t gate_bstride,
                          int64_t gate_hstride, uint64_t out, uint64_t lse, uint64_t workspace,
                          uint64_t workspace_bytes, int batch, int NH, int NKV, int HD, int page_size,
                          int splits);
/* The same attention in double precision.  No GPU kernel exists in the reference for it; the arithmetic is that of its host
 * loop refAttn (prototypes/fa2_vllm.ts:114-139), which runs in JavaScript numbers, i.e. doubles: every bf16 x bf16 product
 * and every sum is carried in f64, exp() is evaluated in f64, and the quotient is rounded once to f32 (then gate, then
 * bf16).  The result does not depend on the number of splits or the batch beyond ~1e-15 relative before that rounding,
 * so the bf16 outputs equal a host evaluation in doubles bit for bit, and the decode step stays reproducible token for
 * token.  Arguments as bk_attn_decode; NH / NKV <= 8; the workspace (size from bk_attn_plan_exact, needed also for one
 * split) holds an f64 copy of q and the f64 partials.  About as fast as bk_attn_decode where the cache read dominates. */
BK_API int bk_attn_plan_exact(int batch, int NKV, int max_ctx, int* splits, uint64_t* workspace_bytes);
BK_API int bk_attn_decode_exact(uint64_t q, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride,
                                uint64_t ctx_len, int max_ctx, uint64_t gate, int64_t gate_bstride,
                                int64_t gate_hstride, uint64_t out, uint64_t lse, uint64_t workspace,
                                uint64_t workspace_bytes, int batch, int NH, int NKV, int HD, int page_size,
                                int splits);
/* bk_attn_decode for callers that cannot allocate device memory or bring a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments and same
 * results (bit for bit, for the same number of splits) as bk_attn_decode, without workspace / workspace_bytes: the
 * partial results of the splits go to a fixed 16.1 MiB array that each GPU holds from library load to process end.
 * Limit: batch * NKV * splits <= 1024 partial results; splits = 0 lets the library choose within that limit, an
 * explicit split count beyond it is refused with an error.  The call allocates and frees nothing.  All calls on a GPU
 * share the one array: two calls that overlap on that GPU (different streams) race, calls on one stream do not. */
BK_API int bk_attn_decode_noalloc(uint64_t q, uint64_t kc, uint64_t vc, uint64_t block_table, int bt_stride,
                                  uint64_t ctx_len, int max_ctx, uint64_t gate, int64_t gate_bstride,
                                  int64_t gate_hstride, uint64_t out, uint64_t lse, int batch, int NH, int NKV,
                                  int HD, int page_size, int splits);
/* The cache write of emitFA2Attn (src/emitters.ts:202-205): k, v bf16 [batch, NKV, 256]
 * of this step go to token pos[b] of every sequence (pos int32 [batch] on the device).
 * max_len is the capacity of a sequence in tokens (at most 16 * bt_stride): a position
 * outside 0 .. max_len-1 writes nothing, as the reference's store is masked
 * (boundaryCheck, src/emitters.ts:203-205). */
BK_API int bk_kv_append(uint64_t k, uint64_t v, uint64_t kc, uint64_t vc, uint64_t block_table,
                        int bt_stride, uint64_t pos, int max_len, int batch, int NKV, int HD,
                        int page_size);

#ifdef __cplusplus
}
#endif
#endif /* BUNKER_HIP_H */
