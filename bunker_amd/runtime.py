"""Launch surface of the decode path over ``libbunker_hip.so``.

Host-side counterpart of the reference's runtime boundary (src/ttir.ts:225-491):
the same function names and argument meaning — ``cuAlloc``, ``cuHtoD``, ``cuDtoH``,
``cuFree``, ``cuSync``, ``compileAndLoad``, ``cuLaunch``, ``profGpuReset``,
``profGpuReport`` — bound with ctypes to the C ABI of ``include/bunker_hip.h``
instead of to libcuda and the Triton shim.  Device pointers are plain ints, as
they are bigints in the reference.

There is no CPU fallback: importing works anywhere, but every call needs the
compiled library and an MI355X and raises ``BunkerError`` otherwise.
"""
from __future__ import annotations

import ctypes as C
import os
import re
from dataclasses import dataclass
from typing import Sequence

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libbunker_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_PKG), "include", "bunker_hip.h")


class BunkerError(RuntimeError):
    pass


_lib = None
_inited = False

u64, i32, i64, vp = C.c_uint64, C.c_int, C.c_int64, C.c_void_p
_SIGS = {
    "bk_init": [i32], "bk_shutdown": [], "bk_device_info": [C.c_char_p, i32],
    "bk_alloc": [u64, C.POINTER(u64)], "bk_free": [u64],
    "bk_htod": [u64, vp, u64], "bk_dtoh": [vp, u64, u64], "bk_dtod": [u64, u64, u64],
    "bk_memset": [u64, i32, u64], "bk_sync": [],
    "bk_host_alloc": [u64, C.POINTER(u64)], "bk_host_free": [u64],
    "bk_htod_async": [u64, vp, u64], "bk_dtoh_async": [vp, u64, u64], "bk_event_sync": [u64],
    "bk_stream_create": [C.POINTER(u64)], "bk_stream_use": [u64], "bk_stream_wait_event": [u64], "bk_stream_destroy": [u64],
    "bk_event_create": [C.POINTER(u64)], "bk_event_record": [u64],
    "bk_event_elapsed_ms": [u64, u64, C.POINTER(C.c_float)], "bk_event_destroy": [u64],
    "bk_prof_enable": [i32], "bk_prof_reset": [], "bk_prof_report": [C.c_char_p, i32],
    "bk_capture_begin": [], "bk_capture_end": [C.POINTER(u64)], "bk_graph_launch": [u64],
    "bk_graph_destroy": [u64], "bk_graph_node_count": [u64, C.POINTER(C.c_int)],
    "bk_tune_set": [C.c_char_p, i32],
    "bk_kernel_create": [C.c_char_p], "bk_launch": [i32, C.POINTER(u64), i32], "bk_kernel_destroy": [i32],
    "bk_kernel_describe": [i32, C.c_char_p, i32],
    "bk_memread": [u64, i64, u64], "bk_memcopy": [u64, u64, i64],
    "bk_quantize_q8_1": [u64, i32, u64, i32, i32],
    "bk_quantize_q4k": [u64, i32, u64, i64, i32],
    "bk_gemv_q4k_f32": [u64, u64, u64, i32, i32],
    "bk_gemv_q4k_q8_1": [u64, u64, u64, i32, i32, i32, i32, u64],
    "bk_gemm_q4k_q8_1": [u64, u64, u64, i32, i32, i32, i32, u64],
    "bk_q4k_q8_1_subdots": [u64, u64, u64, i32, i32],
    "bk_dequant_legacy_i8": [u64, u64, i64], "bk_q4k_nibbles": [u64, u64, i64],
    "bk_q4k_dequant_f32": [u64, u64, i64],
    "bk_gdn_core": [u64, u64, u64, u64, u64, u64, u64, u64, i32, i32],
    "bk_attn_plan": [i32, i32, i32, C.POINTER(i32), C.POINTER(u64)],
    "bk_attn_decode": [u64, u64, u64, u64, i32, u64, i32, u64, i64, i64, u64, u64, u64, u64, i32, i32, i32, i32, i32, i32],
    "bk_attn_plan_exact": [i32, i32, i32, C.POINTER(i32), C.POINTER(u64)],
    "bk_attn_decode_exact": [u64, u64, u64, u64, i32, u64, i32, u64, i64, i64, u64, u64, u64, u64, i32, i32, i32, i32, i32, i32],
    "bk_attn_decode_noalloc": [u64, u64, u64, u64, i32, u64, i32, u64, i64, i64, u64, u64, i32, i32, i32, i32, i32, i32],
    "bk_kv_append": [u64, u64, u64, u64, u64, i32, u64, i32, i32, i32, i32, i32],
}


def declared_symbols() -> list[str]:
    """Every function name that include/bunker_hip.h declares."""
    with open(HEADER_PATH) as f:
        return re.findall(r"^BK_API\s+[\w\s\*]+?\b(bk_\w+)\(", f.read(), flags=re.M)


def load_library(path: str | None = None):
    """dlopen the C-ABI library (no GPU needed) and attach argument types."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise BunkerError(
            f"{p} is missing: build it with `make -C bunker_amd/csrc` (hipcc --offload-arch=gfx950); "
            "there is no CPU fallback for the decode kernels")
    lib = C.CDLL(p)
    lib.bk_last_error.restype = C.c_char_p
    lib.bk_last_error.argtypes = []
    for name, args in _SIGS.items():
        fn = getattr(lib, name)
        fn.restype = i32
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def _check(rc: int, what: str = "") -> int:
    if rc < 0:
        msg = _lib.bk_last_error().decode("utf-8", "replace") if _lib is not None else ""
        raise BunkerError(f"{what}: {msg} (rc={rc})" if what else f"{msg} (rc={rc})")
    return rc


def cu(device: int = 0):
    """Initialise the device once and return the bound library (src/ttir.ts:225-262)."""
    global _inited
    lib = load_library()
    if not _inited:
        _check(lib.bk_init(device), "bk_init")
        _inited = True
    return lib


def device_info() -> dict:
    buf = C.create_string_buffer(256)
    _check(cu().bk_device_info(buf, 256), "bk_device_info")
    name, arch, cus, mem = buf.value.decode().split("|")
    return {"name": name, "arch": arch, "cus": int(cus), "mem_bytes": int(mem)}


# ---------------------------------------------------------------- memory (src/ttir.ts:266-285)
def cuAlloc(nbytes: int) -> int:
    out = u64(0)
    _check(cu().bk_alloc(int(nbytes), C.byref(out)), f"cuAlloc({nbytes})")
    return int(out.value)


def _host_view(buf):
    if isinstance(buf, np.ndarray):
        if not buf.flags.c_contiguous:
            raise BunkerError("host array must be C-contiguous")
        return buf.ctypes.data, buf.nbytes
    mv = memoryview(buf)
    arr = np.frombuffer(mv, dtype=np.uint8)
    return arr.ctypes.data, arr.nbytes


def cuHtoD(dev: int, host, nbytes: int | None = None) -> None:
    addr, n = _host_view(host)
    _check(cu().bk_htod(dev, addr, int(nbytes if nbytes is not None else n)), "cuHtoD")


def cuDtoH(host, dev: int, nbytes: int | None = None) -> None:
    addr, n = _host_view(host)
    _check(cu().bk_dtoh(addr, dev, int(nbytes if nbytes is not None else n)), "cuDtoH")


def cuFree(dev: int) -> None:
    _check(cu().bk_free(dev), "cuFree")


def cuSync() -> int:
    return _check(cu().bk_sync(), "cuSync")


def cuMemset(dev: int, value: int, nbytes: int) -> None:
    _check(cu().bk_memset(dev, value, nbytes), "cuMemset")


def cuDtoD(dst: int, src: int, nbytes: int) -> None:
    _check(cu().bk_dtod(dst, src, nbytes), "cuDtoD")


def cuHtoDAsync(dev: int, host, nbytes: int | None = None) -> None:
    """Enqueue the copy and return (src/ttir.ts:305-308); ``host`` must be pinned (``cuAllocHost``) and left
    untouched until ``cuSync`` or an event recorded after the copy has been waited for."""
    addr, n = _host_view(host)
    _check(cu().bk_htod_async(dev, addr, int(nbytes if nbytes is not None else n)), "cuHtoDAsync")


def cuDtoHAsync(host, dev: int, nbytes: int | None = None) -> None:
    addr, n = _host_view(host)
    _check(cu().bk_dtoh_async(addr, dev, int(nbytes if nbytes is not None else n)), "cuDtoHAsync")


class PinnedBuffer:
    """Page-locked host staging memory, viewed as a numpy uint8 array (``.array``)."""

    def __init__(self, nbytes: int):
        out = u64(0)
        _check(cu().bk_host_alloc(int(nbytes), C.byref(out)), f"cuAllocHost({nbytes})")
        self.ptr = int(out.value)
        self.nbytes = int(nbytes)
        self.array = np.ctypeslib.as_array((C.c_uint8 * self.nbytes).from_address(self.ptr))

    def free(self) -> None:
        if self.ptr:
            self.array = None
            _check(cu().bk_host_free(self.ptr), "cuFreeHost")
            self.ptr = 0


def cuAllocHost(nbytes: int) -> PinnedBuffer:
    return PinnedBuffer(nbytes)


def to_device(arr: np.ndarray) -> int:
    """Allocate and upload a numpy array; returns the device pointer."""
    arr = np.ascontiguousarray(arr)
    p = cuAlloc(max(arr.nbytes, 1))
    if arr.nbytes:
        cuHtoD(p, arr)
    return p


def from_device(dev: int, shape, dtype) -> np.ndarray:
    out = np.empty(shape, dtype)
    if out.nbytes:
        cuDtoH(out, dev)
    return out


# ---------------------------------------------------------------- kernels (src/ttir.ts:321-350, 488-491)
@dataclass(frozen=True)
class LoadedKernel:
    module: int
    fn: int
    shmem: int
    label: str = ""


def compileAndLoad(spec: str, funcName: str | None = None, numWarps: int = 4, label: str | None = None) -> LoadedKernel:
    """Look up the pre-compiled kernel for an op spec such as ``"gemm N=6144 K=2048 cast=1"``.

    Takes the place of compileAndLoad(ttir, funcName, numWarps, label): the op name and
    the constants the reference baked into TTIR text arrive in ``spec``; ``funcName`` and
    ``numWarps`` are accepted for call-site compatibility and ignored.
    """
    h = _check(cu().bk_kernel_create(spec.encode()), f"compileAndLoad({spec!r})")
    return LoadedKernel(module=0, fn=h, shmem=0, label=label or spec)


def unloadKernel(k: LoadedKernel) -> None:
    """Give the handle's device workspace back (cuModuleUnload is the reference's nearest call); the handle is invalid afterwards."""
    _check(cu().bk_kernel_destroy(k.fn), "bk_kernel_destroy")


def cuLaunch(k: LoadedKernel, grid: Sequence[int], block: Sequence[int], args: Sequence[int]) -> int:
    """Launch with the reference's slot packing: one 8-byte slot per argument.

    ``grid`` and ``block`` are accepted and ignored (each kernel owns its launch shape).
    Returns the library's return code without raising, as cuLaunch returns the driver's.
    """
    n = len(args)
    slots = (u64 * n)(*[int(a) & 0xFFFFFFFFFFFFFFFF for a in args])
    return cu().bk_launch(k.fn, slots, n)


def tune_set(key: str, value: int) -> None:
    _check(cu().bk_tune_set(key.encode(), int(value)), "bk_tune_set")


def last_error() -> str:
    return load_library().bk_last_error().decode("utf-8", "replace")


def profGpuEnable(on: bool = True) -> None:
    _check(cu().bk_prof_enable(1 if on else 0))


def profGpuReset() -> None:
    _check(cu().bk_prof_reset(), "profGpuReset")


def profGpuReport(print_fn=print) -> str:
    buf = C.create_string_buffer(1 << 16)
    _check(cu().bk_prof_report(buf, len(buf)), "profGpuReport")
    text = buf.value.decode()
    if print_fn:
        print_fn(text)
    return text


class Event:
    """HIP event on the library's stream (the cuEvent* calls of src/ttir.ts:352-417)."""

    def __init__(self):
        h = u64(0)
        _check(cu().bk_event_create(C.byref(h)), "bk_event_create")
        self.h = int(h.value)

    def record(self):
        _check(cu().bk_event_record(self.h), "bk_event_record")
        return self

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float(0)
        _check(cu().bk_event_elapsed_ms(self.h, stop.h, C.byref(ms)), "bk_event_elapsed_ms")
        return float(ms.value)

    def sync(self):
        _check(cu().bk_event_sync(self.h), "bk_event_sync")

    def destroy(self):
        if self.h:
            cu().bk_event_destroy(self.h)
            self.h = 0


def eventSync(ev: "Event") -> None:
    ev.sync()


_cur_stream = 0      # handle of the selected stream (0 = the library's first)


def _use_stream(h: int) -> None:
    global _cur_stream
    _check(cu().bk_stream_use(h), "bk_stream_use")
    _cur_stream = h


class Stream:
    """A further stream of the library: ``with stream: ...`` sends launches, copies and event records there;
    ``stream.wait(event)`` orders it behind an event recorded on another stream."""

    def __init__(self):
        h = u64(0)
        _check(cu().bk_stream_create(C.byref(h)), "bk_stream_create")
        self.h = int(h.value)
        self._prev: list[int] = []

    def __enter__(self):
        self._prev.append(_cur_stream)
        _use_stream(self.h)
        return self

    def __exit__(self, *exc):
        _use_stream(self._prev.pop())
        return False

    def wait(self, ev: "Event") -> None:
        """Work queued on this stream from now on starts after ``ev`` has happened."""
        prev = _cur_stream
        _use_stream(self.h)
        try:
            _check(cu().bk_stream_wait_event(ev.h), "bk_stream_wait_event")
        finally:
            _use_stream(prev)

    def destroy(self):
        if self.h:
            if _cur_stream == self.h:
                _use_stream(0)
            cu().bk_stream_destroy(self.h)
            self.h = 0


def streamWaitEvent(ev: "Event") -> None:
    """The stream selected now (the first one outside a ``with Stream``) waits for ``ev``."""
    _check(cu().bk_stream_wait_event(ev.h), "bk_stream_wait_event")


class Graph:
    """A recorded launch sequence: ``with Graph() as g: ...launches...`` then ``g.launch()``.

    Everything enqueued inside the ``with`` block is captured into a HIP graph instead of
    running; only kernel launches are legal there (no alloc, copy, sync or event call).
    """

    def __init__(self):
        self.h = 0

    def __enter__(self):
        _check(cu().bk_capture_begin(), "bk_capture_begin")
        return self

    def __exit__(self, et, ev, tb):
        h = u64(0)
        rc = cu().bk_capture_end(C.byref(h))
        if et is None:
            _check(rc, "bk_capture_end")
        self.h = int(h.value)
        return False

    def launch(self):
        _check(cu().bk_graph_launch(self.h), "bk_graph_launch")

    def node_count(self) -> int:
        n = C.c_int(0)
        _check(cu().bk_graph_node_count(self.h, C.byref(n)), "bk_graph_node_count")
        return n.value

    def destroy(self):
        if self.h:
            cu().bk_graph_destroy(self.h)
            self.h = 0


# ---------------------------------------------------------------- typed entry points
F32, BF16 = 0, 1


def memread(src: int, nbytes: int, sink: int) -> None:
    _check(cu().bk_memread(src, nbytes, sink), "bk_memread")


def memcopy(src: int, dst: int, nbytes: int) -> None:
    _check(cu().bk_memcopy(src, dst, nbytes), "bk_memcopy")


def quantize_q8_1(x: int, out: int, K: int, batch: int = 1, x_dtype: int = F32) -> None:
    _check(cu().bk_quantize_q8_1(x, x_dtype, out, K, batch), "bk_quantize_q8_1")


def quantize_q4k(w: int, out: int, rows: int, K: int, w_dtype: int = BF16) -> None:
    """[rows, K] f32 / bf16 weights on the device -> rows * K/256 Q4_K super-blocks (144 bytes each)."""
    _check(cu().bk_quantize_q4k(w, w_dtype, out, rows, K), "bk_quantize_q4k")


def gemv_q4k_f32(W: int, x: int, y: int, N: int, K: int) -> None:
    _check(cu().bk_gemv_q4k_f32(W, x, y, N, K), "bk_gemv_q4k_f32")


def gemv_q4k_q8_1(W: int, xq: int, y: int, N: int, K: int, batch: int = 1, out_dtype: int = F32,
                  residual: int = 0) -> None:
    _check(cu().bk_gemv_q4k_q8_1(W, xq, y, N, K, batch, out_dtype, residual), "bk_gemv_q4k_q8_1")


def gemm_q4k_q8_1(W: int, xq: int, y: int, N: int, K: int, batch: int, out_dtype: int = F32, residual: int = 0) -> None:
    _check(cu().bk_gemm_q4k_q8_1(W, xq, y, N, K, batch, out_dtype, residual), "bk_gemm_q4k_q8_1")


def q4k_q8_1_subdots(W: int, xq: int, I: int, N: int, K: int) -> None:
    _check(cu().bk_q4k_q8_1_subdots(W, xq, I, N, K), "bk_q4k_q8_1_subdots")


def dequant_legacy_i8(blocks: int, out: int, nblocks: int) -> None:
    _check(cu().bk_dequant_legacy_i8(blocks, out, nblocks), "bk_dequant_legacy_i8")


def q4k_nibbles(blocks: int, out: int, nblocks: int) -> None:
    _check(cu().bk_q4k_nibbles(blocks, out, nblocks), "bk_q4k_nibbles")


def q4k_dequant_f32(blocks: int, out: int, nblocks: int) -> None:
    _check(cu().bk_q4k_dequant_f32(blocks, out, nblocks), "bk_q4k_dequant_f32")


def gdn_core(q: int, k: int, v: int, g: int, beta: int, S_in: int, out: int, S_out: int, Hg: int, batch: int = 1) -> None:
    _check(cu().bk_gdn_core(q, k, v, g, beta, S_in, out, S_out, Hg, batch), "bk_gdn_core")


def attn_plan(batch: int, NKV: int, max_ctx: int, splits: int = 0) -> tuple[int, int]:
    """Returns (splits, workspace_bytes) the attention kernel will use for this shape."""
    s = i32(splits); nbytes = u64(0)
    _check(cu().bk_attn_plan(batch, NKV, max_ctx, C.byref(s), C.byref(nbytes)), "bk_attn_plan")
    return int(s.value), int(nbytes.value)


def attn_decode(q: int, kc: int, vc: int, block_table: int, bt_stride: int, ctx_len: int, max_ctx: int, out: int,
                lse: int, batch: int, NH: int = 16, NKV: int = 2, HD: int = 256, page_size: int = 16, splits: int = 0,
                workspace: int = 0, workspace_bytes: int = 0, gate: int = 0, gate_bstride: int = 0,
                gate_hstride: int = 0) -> None:
    _check(cu().bk_attn_decode(q, kc, vc, block_table, bt_stride, ctx_len, max_ctx, gate, gate_bstride, gate_hstride,
                               out, lse, workspace, workspace_bytes, batch, NH, NKV, HD, page_size, splits),
           "bk_attn_decode")


def attn_plan_exact(batch: int, NKV: int, max_ctx: int, splits: int = 0):
    """(splits, workspace bytes) of the double-precision form; the workspace is needed for a single split too."""
    s, nbytes = i32(splits), u64(0)
    _check(cu().bk_attn_plan_exact(batch, NKV, max_ctx, C.byref(s), C.byref(nbytes)), "bk_attn_plan_exact")
    return s.value, nbytes.value


def attn_decode_exact(q: int, kc: int, vc: int, block_table: int, bt_stride: int, ctx_len: int, max_ctx: int, out: int,
                      lse: int, batch: int, NH: int = 16, NKV: int = 2, HD: int = 256, page_size: int = 16, splits: int = 0,
                      workspace: int = 0, workspace_bytes: int = 0, gate: int = 0, gate_bstride: int = 0,
                      gate_hstride: int = 0) -> None:
    """``attn_decode`` with every product and sum in f64: the bits of a host evaluation in doubles."""
    _check(cu().bk_attn_decode_exact(q, kc, vc, block_table, bt_stride, ctx_len, max_ctx, gate, gate_bstride, gate_hstride,
                                     out, lse, workspace, workspace_bytes, batch, NH, NKV, HD, page_size, splits),
           "bk_attn_decode_exact")


def attn_decode_noalloc(q: int, kc: int, vc: int, block_table: int, bt_stride: int, ctx_len: int, max_ctx: int, out: int,
                        lse: int, batch: int, NH: int = 16, NKV: int = 2, HD: int = 256, page_size: int = 16, splits: int = 0,
                        gate: int = 0, gate_bstride: int = 0, gate_hstride: int = 0) -> None:
    """``attn_decode`` without a workspace: split partials go to the library's fixed per-GPU array (batch * NKV * splits <= 1024)."""
    _check(cu().bk_attn_decode_noalloc(q, kc, vc, block_table, bt_stride, ctx_len, max_ctx, gate, gate_bstride, gate_hstride,
                                       out, lse, batch, NH, NKV, HD, page_size, splits), "bk_attn_decode_noalloc")


def kv_append(k: int, v: int, kc: int, vc: int, block_table: int, bt_stride: int, pos: int, max_len: int, batch: int,
              NKV: int = 2, HD: int = 256, page_size: int = 16) -> None:
    """``max_len``: capacity of a sequence in tokens; a position outside 0..max_len-1 writes nothing."""
    _check(cu().bk_kv_append(k, v, kc, vc, block_table, bt_stride, pos, max_len, batch, NKV, HD, page_size), "bk_kv_append")


def v_pages_to_device_layout(vc) -> "np.ndarray":
    """[pages, NKV, 16 tok, 256 dim] -> the library's dim-major V pages [pages, NKV, 256 dim, 16 tok]."""
    return np.ascontiguousarray(np.asarray(vc).transpose(0, 1, 3, 2))
