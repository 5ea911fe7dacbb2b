// hip.ts — the runtime half of src/ttir.ts bound to libbunker_hip.so (gfx950 / MI355X) with bun:ffi.
//
// Drop this file next to src/ttir.ts and change the import of src/runner.ts, src/model.ts' callers and the decode
// scripts (prototypes/decode_graph.ts) from "./ttir" to "./hip": the names, argument meaning and error behaviour of
// cu, cuAlloc, cuHtoD, cuDtoH, cuFree, cuSync, cuHtoDAsync, cuDtoHAsync, cuCopySync, compileAndLoad, cuLaunch,
// LoadedKernel, profGpuReset and profGpuReport are those of src/ttir.ts:223-491.  What changes underneath:
//   - compileAndLoad takes an op spec ("gemm N=6144 K=2048 cast=1": the op name of src/model.ts plus the constants
//     the emitters baked into TTIR text) instead of TTIR; no Triton, no PTX, nothing is compiled at run time;
//   - cuLaunch packs the same 8-byte slots (src/ttir.ts:321-348) and ignores grid and block: the kernels of the
//     library own their launch shape;
//   - one step can be recorded into a HIP graph and replayed (captureBegin / captureEnd / graphLaunch), which the
//     reference could not do through bun:ffi (LOG.md:710-738).
// Only scalars and raw pointers cross the boundary (no structs by pointer, LOG.md:730-733).  Single-threaded use,
// as in the reference.  The symbol table below lists every function of include/bunker_hip.h with its C types
// (int -> i32, int64_t -> i64, uint64_t -> u64, any pointer -> ptr); tests/test_abi.py checks it against the header.
import { dlopen, ptr as ffiPtr, CString } from "bun:ffi";

const LIB_PATH = process.env.BUNKER_HIP_LIB ?? `${import.meta.dir}/../bunker_amd/libbunker_hip.so`;

const SYMBOLS = {
  bk_init:                  { args: ["i32"], returns: "i32" },
  bk_shutdown:              { args: [], returns: "i32" },
  bk_last_error:            { args: [], returns: "ptr" },
  bk_device_info:           { args: ["ptr", "i32"], returns: "i32" },
  bk_alloc:                 { args: ["u64", "ptr"], returns: "i32" },
  bk_free:                  { args: ["u64"], returns: "i32" },
  bk_htod:                  { args: ["u64", "ptr", "u64"], returns: "i32" },
  bk_dtoh:                  { args: ["ptr", "u64", "u64"], returns: "i32" },
  bk_dtod:                  { args: ["u64", "u64", "u64"], returns: "i32" },
  bk_memset:                { args: ["u64", "i32", "u64"], returns: "i32" },
  bk_sync:                  { args: [], returns: "i32" },
  bk_host_alloc:            { args: ["u64", "ptr"], returns: "i32" },
  bk_host_free:             { args: ["u64"], returns: "i32" },
  bk_htod_async:            { args: ["u64", "ptr", "u64"], returns: "i32" },
  bk_dtoh_async:            { args: ["ptr", "u64", "u64"], returns: "i32" },
  bk_event_create:          { args: ["ptr"], returns: "i32" },
  bk_event_record:          { args: ["u64"], returns: "i32" },
  bk_event_elapsed_ms:      { args: ["u64", "u64", "ptr"], returns: "i32" },
  bk_event_sync:            { args: ["u64"], returns: "i32" },
  bk_event_destroy:         { args: ["u64"], returns: "i32" },
  bk_stream_create:         { args: ["ptr"], returns: "i32" },
  bk_stream_use:            { args: ["u64"], returns: "i32" },
  bk_stream_wait_event:     { args: ["u64"], returns: "i32" },
  bk_stream_destroy:        { args: ["u64"], returns: "i32" },
  bk_prof_enable:           { args: ["i32"], returns: "i32" },
  bk_prof_reset:            { args: [], returns: "i32" },
  bk_prof_report:           { args: ["ptr", "i32"], returns: "i32" },
  bk_capture_begin:         { args: [], returns: "i32" },
  bk_capture_end:           { args: ["ptr"], returns: "i32" },
  bk_graph_launch:          { args: ["u64"], returns: "i32" },
  bk_graph_destroy:         { args: ["u64"], returns: "i32" },
  bk_graph_node_count:      { args: ["u64", "ptr"], returns: "i32" },
  bk_tune_set:              { args: ["ptr", "i32"], returns: "i32" },
  bk_kernel_create:         { args: ["ptr"], returns: "i32" },
  bk_launch:                { args: ["i32", "ptr", "i32"], returns: "i32" },
  bk_kernel_destroy:        { args: ["i32"], returns: "i32" },
  bk_kernel_describe:       { args: ["i32", "ptr", "i32"], returns: "i32" },
  bk_memread:               { args: ["u64", "i64", "u64"], returns: "i32" },
  bk_memcopy:               { args: ["u64", "u64", "i64"], returns: "i32" },
  bk_quantize_q8_1:         { args: ["u64", "i32", "u64", "i32", "i32"], returns: "i32" },
  bk_quantize_q4k:          { args: ["u64", "i32", "u64", "i64", "i32"], returns: "i32" },
  bk_gemv_q4k_f32:          { args: ["u64", "u64", "u64", "i32", "i32"], returns: "i32" },
  bk_gemv_q4k_q8_1:         { args: ["u64", "u64", "u64", "i32", "i32", "i32", "i32", "u64"], returns: "i32" },
  bk_gemm_q4k_q8_1:         { args: ["u64", "u64", "u64", "i32", "i32", "i32", "i32", "u64"], returns: "i32" },
  bk_q4k_q8_1_subdots:      { args: ["u64", "u64", "u64", "i32", "i32"], returns: "i32" },
  bk_dequant_legacy_i8:     { args: ["u64", "u64", "i64"], returns: "i32" },
  bk_q4k_nibbles:           { args: ["u64", "u64", "i64"], returns: "i32" },
  bk_q4k_dequant_f32:       { args: ["u64", "u64", "i64"], returns: "i32" },
  bk_gdn_core:              { args: ["u64", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "i32", "i32"], returns: "i32" },
  bk_attn_plan:             { args: ["i32", "i32", "i32", "ptr", "ptr"], returns: "i32" },
  bk_attn_decode:           { args: ["u64", "u64", "u64", "u64", "i32", "u64", "i32", "u64", "i64", "i64", "u64", "u64", "u64", "u64", "i32", "i32", "i32", "i32", "i32", "i32"], returns: "i32" },
  bk_attn_plan_exact:       { args: ["i32", "i32", "i32", "ptr", "ptr"], returns: "i32" },
  bk_attn_decode_exact:     { args: ["u64", "u64", "u64", "u64", "i32", "u64", "i32", "u64", "i64", "i64", "u64", "u64", "u64", "u64", "i32", "i32", "i32", "i32", "i32", "i32"], returns: "i32" },
  bk_attn_decode_noalloc:   { args: ["u64", "u64", "u64", "u64", "i32", "u64", "i32", "u64", "i64", "i64", "u64", "u64", "i32", "i32", "i32", "i32", "i32", "i32"], returns: "i32" },
  bk_kv_append:             { args: ["u64", "u64", "u64", "u64", "u64", "i32", "u64", "i32", "i32", "i32", "i32", "i32"], returns: "i32" },
} as const;

let _lib: any = null;
let _inited = false;

function lastError(): string {
  const p = _lib.bk_last_error();
  return p ? new CString(p).toString() : "";
}

/** src/ttir.ts:223-258: load the library and create the context once; returns the symbol table. */
export function cu() {
  if (!_lib) _lib = dlopen(LIB_PATH, SYMBOLS).symbols;
  if (!_inited) {
    const dev = Number(process.env.BUNKER_HIP_DEVICE ?? "0");
    if (_lib.bk_init(dev) !== 0) throw new Error(`bk_init(${dev}) failed: ${lastError()}`);
    if (process.env.BUNKER_GPU_PROF === "1") _lib.bk_prof_enable(1);
    _inited = true;
  }
  return _lib;
}

function check(rc: number, what: string): void {
  if (rc !== 0) throw new Error(`${what} failed (rc=${rc}): ${lastError()}`);
}

function asBuffer(host: Buffer | ArrayBuffer): Buffer {
  return host instanceof ArrayBuffer ? Buffer.from(host) : host;
}

/** src/ttir.ts:266-271 */
export function cuAlloc(bytes: number | bigint): bigint {
  const out = Buffer.alloc(8);
  const rc = cu().bk_alloc(BigInt(bytes), out);
  if (rc !== 0) throw new Error(`cuMemAlloc failed (rc=${rc}, ${bytes} bytes): ${lastError()}`);
  return out.readBigUInt64LE(0);
}
/** src/ttir.ts:273-276 */
export function cuHtoD(devPtr: bigint, hostBuf: Buffer | ArrayBuffer, bytes?: number | bigint): void {
  const buf = asBuffer(hostBuf);
  check(cu().bk_htod(devPtr, buf, BigInt(bytes ?? buf.byteLength)), "cuMemcpyHtoD");
}
/** src/ttir.ts:278-281 */
export function cuDtoH(hostBuf: Buffer | ArrayBuffer, devPtr: bigint, bytes?: number | bigint): void {
  const buf = asBuffer(hostBuf);
  check(cu().bk_dtoh(buf, devPtr, BigInt(bytes ?? buf.byteLength)), "cuMemcpyDtoH");
}
/** src/ttir.ts:283 */
export function cuFree(devPtr: bigint): void { cu().bk_free(devPtr); }
/** src/ttir.ts:285 */
export function cuSync(): number { return cu().bk_sync(); }

// src/ttir.ts:286-317: copies that do not wait.  The reference keeps a side stream for them; here they are queued on
// the library's selected stream, in order with the launches.  The host buffer must be pinned for the copy to be
// asynchronous (hostAlloc below) and must stay untouched until cuCopySync.
export function cuHtoDAsync(devPtr: bigint, hostBuf: Buffer | ArrayBuffer, bytes?: number | bigint): void {
  const buf = asBuffer(hostBuf);
  check(cu().bk_htod_async(devPtr, buf, BigInt(bytes ?? buf.byteLength)), "cuMemcpyHtoDAsync");
}
export function cuDtoHAsync(hostBuf: Buffer | ArrayBuffer, devPtr: bigint, bytes?: number | bigint): void {
  const buf = asBuffer(hostBuf);
  check(cu().bk_dtoh_async(buf, devPtr, BigInt(bytes ?? buf.byteLength)), "cuMemcpyDtoHAsync");
}
export function cuCopySync(): number { return cu().bk_sync(); }

/** Pinned host memory for the asynchronous copies: returns the address; wrap it with bun:ffi's toArrayBuffer. */
export function hostAlloc(bytes: number | bigint): bigint {
  const out = Buffer.alloc(8);
  check(cu().bk_host_alloc(BigInt(bytes), out), "bk_host_alloc");
  return out.readBigUInt64LE(0);
}
export function hostFree(p: bigint): void { cu().bk_host_free(p); }

/** src/ttir.ts:350 */
export interface LoadedKernel { module: number; fn: number; shmem: number; }

const _labels = new Map<number, string>();

/** src/ttir.ts:488-491 with an op spec in the place of the TTIR text; throws the library's message on failure
 *  (the shim's "ERROR:" convention, src/ttir.ts:166-174).  funcName and numWarps are accepted and ignored. */
export function compileAndLoad(spec: string, funcName = "kernel", numWarps = 4, label?: string): LoadedKernel {
  const h = cu().bk_kernel_create(Buffer.from(spec + "\0", "utf-8"));
  if (h < 0) throw new Error(`ERROR: ${lastError()} (spec "${spec}")`);
  _labels.set(h, label ?? funcName ?? spec);
  return { module: 0, fn: h, shmem: 0 };
}
/** Give back the workspace a kernel handle owns (cuModuleUnload's place). */
export function unload(k: LoadedKernel): void { cu().bk_kernel_destroy(k.fn); _labels.delete(k.fn); }

/** src/ttir.ts:321-348: each argument goes into one 8-byte slot (bigint -> u64, number -> i64, so an i32 scalar is the
 *  low four bytes); returns the library's code without throwing.  grid and block are ignored. */
export function cuLaunch(k: LoadedKernel, grid: [number, number, number], block: [number, number, number],
                         args: (bigint | number)[]): number {
  const slots = Buffer.alloc(args.length * 8);      // referenced until the call returns (LOG.md:728-729)
  for (let i = 0; i < args.length; i++) {
    const a = args[i];
    if (typeof a === "bigint") slots.writeBigUInt64LE(a, i * 8);
    else slots.writeBigInt64LE(BigInt(a), i * 8);
  }
  return cu().bk_launch(k.fn, slots, args.length);
}

/** src/ttir.ts:385-388 */
export function profGpuReset(): void { cu().bk_prof_reset(); }
/** src/ttir.ts:391-417: the table comes from the library (one event pair around every bk_launch, BUNKER_GPU_PROF=1). */
export function profGpuReport(): void {
  if (process.env.BUNKER_GPU_PROF !== "1") return;
  const buf = Buffer.alloc(1 << 16);
  cu().bk_prof_report(buf, buf.length);
  console.log(new CString(ffiPtr(buf)).toString());
}

// ── one decode step as a HIP graph (no counterpart that works in the reference, LOG.md:710-738) ──
/** Everything launched between captureBegin and captureEnd is recorded instead of run. */
export function captureBegin(): void { check(cu().bk_capture_begin(), "bk_capture_begin"); }
export function captureEnd(): bigint {
  const out = Buffer.alloc(8);
  check(cu().bk_capture_end(out), "bk_capture_end");
  return out.readBigUInt64LE(0);
}
export function graphLaunch(graph: bigint): number { return cu().bk_graph_launch(graph); }
export function graphDestroy(graph: bigint): void { cu().bk_graph_destroy(graph); }
/** Kernel launches one replay of the graph stands for. */
export function graphNodeCount(graph: bigint): number {
  const out = Buffer.alloc(4);
  check(cu().bk_graph_node_count(graph, out), "bk_graph_node_count");
  return out.readInt32LE(0);
}

/** Quantize a bf16 / f32 weight [rows, K] that is already on the device to Q4_K super-blocks (model load). */
export function quantizeQ4K(w: bigint, isBf16: boolean, rows: number, K: number): bigint {
  const out = cuAlloc(BigInt(rows) * BigInt(K / 256) * 144n);
  check(cu().bk_quantize_q4k(w, isBf16 ? 1 : 0, out, BigInt(rows), K), "bk_quantize_q4k");
  return out;
}

export function deviceInfo(): string {
  const buf = Buffer.alloc(256);
  cu().bk_device_info(buf, buf.length);
  return new CString(ffiPtr(buf)).toString();
}

export default { cu, cuAlloc, cuHtoD, cuDtoH, cuFree, cuSync, cuLaunch, compileAndLoad };
