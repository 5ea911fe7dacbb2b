"""Checkpoint path of the decode step: safetensors / GGUF files -> device-resident weights by graph name.

Counterpart of the reference's loaders: ``loadSafeTensors`` (prototypes/safetensors_loader.ts:13-78: one
device buffer for the whole data section, chunked uploads, tensors are views ``devPtr = base + offset``),
``loadWeights`` (prototypes/decode.ts:64-75) and the graph-name -> checkpoint-name mapping ``safeKey``
(prototypes/decode_graph.ts:97-108).  What is added for this path: every ``gemm`` weight is quantized on the
device to Q4_K super-blocks (``bk_quantize_q4k``) as it arrives, and the quantized model can be written to and
read from a GGUF file (tensor type 12 = Q4_K, same 144-byte block), so a second start skips the quantizer.

Uploads go through two pinned staging buffers and asynchronous copies, so reading the file overlaps the
transfer of the previous chunk.  Nothing here computes on the host: conversions between f32 and bf16 of the few
small tensors whose checkpoint type differs from the graph's are the only arithmetic.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass, field

import numpy as np

from . import runtime as rt
from .graph import Graph
from .model import Dims, buildModelGraph

DType = str        # "BF16" | "F16" | "F32" | "I64" | "I32" | "I8" | "U8" | "BOOL" | "F64"  (safetensors_loader.ts:7)
_ST_ITEMSIZE = {"BF16": 2, "F16": 2, "F32": 4, "I64": 8, "I32": 4, "I16": 2, "I8": 1, "U8": 1, "BOOL": 1, "F64": 8}
_ST_NUMPY = {"BF16": np.uint16, "F16": np.uint16, "F32": np.float32, "I64": np.int64, "I32": np.int32, "I16": np.int16,
             "I8": np.int8, "U8": np.uint8, "BOOL": np.uint8, "F64": np.float64}

CHUNK_BYTES = 64 << 20
_DT_BYTES = {"bf16": 2, "f32": 4, "i32": 4, "f16": 2}


def tensor_bytes(t) -> int:
    n = 1
    for d in t.type.shape:
        n *= d
    return n // 256 * 144 if t.type.dtype == "q4_k" else n * _DT_BYTES[t.type.dtype]


@dataclass
class Tensor:
    """safetensors_loader.ts:8 — a view into the file's device buffer."""
    name: str
    devPtr: int
    shape: list
    dtype: DType
    nbytes: int


@dataclass
class SafeTensorsFile:
    tensors: dict
    base: int = 0
    metadata: dict = field(default_factory=dict)

    def free(self) -> None:
        if self.base:
            rt.cuFree(self.base)
            self.base = 0
            self.tensors = {}


# ------------------------------------------------------------------------------------------ safetensors
def readSafeTensorsHeader(path: str):
    """(header dict without ``__metadata__``, metadata dict, offset of the data section, file size).

    Layout: u64 little-endian header length, that many bytes of JSON ``{name: {dtype, shape, data_offsets:
    [begin, end]}}`` with offsets relative to the data section (decode.ts:66-74)."""
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: not a safetensors file (shorter than 8 bytes)")
        (hl,) = struct.unpack("<Q", head)
        f.seek(0, 2)
        size = f.tell()
        if hl <= 0 or 8 + hl > size:
            raise ValueError(f"{path}: header length {hl} does not fit the file ({size} bytes)")
        f.seek(8)
        header = json.loads(f.read(hl).decode("utf-8"))
    meta = header.pop("__metadata__", {}) or {}
    data_start = 8 + hl
    for name, info in header.items():
        b, e = info["data_offsets"]
        n = int(np.prod(info["shape"], dtype=np.int64)) if info["shape"] else 1
        if info["dtype"] not in _ST_ITEMSIZE:
            raise ValueError(f"{path}: tensor '{name}' has unknown dtype {info['dtype']}")
        if e - b != n * _ST_ITEMSIZE[info["dtype"]] or b < 0 or data_start + e > size:
            raise ValueError(f"{path}: tensor '{name}' has inconsistent offsets {b}..{e} for shape {info['shape']}")
    return header, meta, data_start, size


READ_THREADS = 4      # a chunk's file read is split over this many threads (os.preadv releases the interpreter lock)


def _read_chunk(fd: int, view: memoryview, file_off: int, pool) -> None:
    """File bytes [file_off, file_off + len(view)) into ``view``: one copy out of the page cache is a single core's
    memcpy (4-5 GB/s here), so the chunk is cut into pieces that several threads read side by side."""
    n = len(view)
    piece = -(-n // READ_THREADS)
    piece += -piece % 4096

    def rd(lo):
        hi = min(lo + piece, n)
        got = 0
        while lo + got < hi:
            k = os.preadv(fd, [view[lo + got:hi]], file_off + lo + got)
            if k <= 0:
                raise IOError(f"short read: wanted {hi - lo} bytes at offset {file_off + lo}, got {got}")
            got += k

    for fut in [pool.submit(rd, lo) for lo in range(0, n, piece)]:
        fut.result()


def _upload_range(f, file_off: int, nbytes: int, dev: int, chunk_bytes: int = CHUNK_BYTES) -> None:
    """File bytes [file_off, file_off + nbytes) -> device memory at ``dev``, double-buffered through pinned memory."""
    if nbytes <= 0:
        return
    from concurrent.futures import ThreadPoolExecutor
    chunk = int(min(chunk_bytes, nbytes))
    bufs = [rt.cuAllocHost(chunk), rt.cuAllocHost(chunk)]
    done = [rt.Event(), rt.Event()]
    used = [False, False]
    pool = ThreadPoolExecutor(READ_THREADS)
    try:
        off, i = 0, 0
        while off < nbytes:
            n = min(chunk, nbytes - off)
            if used[i]:
                rt.eventSync(done[i])                 # the copy that last read this staging buffer has finished
            _read_chunk(f.fileno(), memoryview(bufs[i].array).cast("B")[:n], file_off + off, pool)
            rt.cuHtoDAsync(dev + off, bufs[i].array, n)
            done[i].record()
            used[i] = True
            off += n
            i ^= 1
        rt.cuSync()
    finally:
        pool.shutdown(wait=True)
        rt.cuSync()
        for b in bufs:
            b.free()
        for e in done:
            e.destroy()


def loadSafeTensors(path: str, chunk_bytes: int = CHUNK_BYTES) -> SafeTensorsFile:
    """The whole data section in ONE device buffer; tensors are offsets into it (safetensors_loader.ts:13-78)."""
    header, meta, data_start, size = readSafeTensorsHeader(path)
    nbytes = size - data_start
    base = rt.cuAlloc(max(nbytes, 16))
    try:
        with open(path, "rb", buffering=0) as f:
            _upload_range(f, data_start, nbytes, base, chunk_bytes)
    except Exception:
        rt.cuFree(base)
        raise
    tensors = {}
    for name, info in header.items():
        b, e = info["data_offsets"]
        tensors[name] = Tensor(name, base + b, list(info["shape"]), info["dtype"], e - b)
    return SafeTensorsFile(tensors, base, meta)


def writeSafeTensors(path: str, tensors: dict, metadata: dict | None = None, align: int = 16) -> None:
    """``tensors``: name -> (dtype string, numpy array holding the raw values; bf16/f16 as uint16 bit patterns).

    The format allows no gap between tensors (the published reader rejects a data section with holes), so alignment
    can only come from the order: with ``align`` > 1 the tensors whose byte size is a multiple of ``align`` are
    written first (each then starts on an ``align``-byte boundary: device views of them can be read with 16-byte
    loads), the others behind them by falling power-of-two divisor of their size; ``align=1`` keeps the given order
    (files from other writers: any element-aligned offset occurs)."""
    def grain(nbytes: int) -> int:
        g = 1
        while g < align and nbytes % (2 * g) == 0:
            g *= 2
        return g

    items = [(name, dtype, np.asarray(arr, order="C")) for name, (dtype, arr) in tensors.items()]      # keeps shape ()
    if align > 1:
        items.sort(key=lambda it: -grain(it[2].nbytes))           # stable: the given order inside a class
    header, off, blobs = {}, 0, []
    for name, dtype, arr in items:
        if arr.dtype.itemsize != _ST_ITEMSIZE[dtype]:
            raise ValueError(f"'{name}': array item size {arr.dtype.itemsize} does not match dtype {dtype}")
        header[name] = {"dtype": dtype, "shape": list(arr.shape), "data_offsets": [off, off + arr.nbytes]}
        blobs.append(arr.tobytes())
        off += arr.nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((-(8 + len(hj))) % 16)          # the data section starts 16-byte aligned in the file
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


# ------------------------------------------------------------------------------------------ GGUF (v3)
GGUF_MAGIC = 0x46554747            # "GGUF"
GGML_F32, GGML_F16, GGML_Q4_K, GGML_I32, GGML_BF16 = 0, 1, 12, 26, 30
# type -> (name, bytes per block, elements per block)
_GGML = {GGML_F32: ("F32", 4, 1), GGML_F16: ("F16", 2, 1), GGML_Q4_K: ("Q4_K", 144, 256), GGML_I32: ("I32", 4, 1),
         GGML_BF16: ("BF16", 2, 1)}
_GV_FMT = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_GV_STRING, _GV_ARRAY = 8, 9


@dataclass
class GGUFTensorInfo:
    name: str
    shape: list          # row-major (outermost first); the file stores the reverse (ne[0] = innermost)
    ggml_type: int
    offset: int          # from the start of the data section
    nbytes: int


def _gguf_nbytes(shape, t) -> int:
    _, bpb, epb = _GGML[t]
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    if shape and shape[-1] % epb:
        raise ValueError(f"innermost dimension {shape[-1]} is not a multiple of the block size {epb}")
    return n // epb * bpb


def _r(f, fmt):
    n = struct.calcsize(fmt)
    b = f.read(n)
    if len(b) != n:
        raise ValueError("GGUF: unexpected end of file")
    return struct.unpack(fmt, b)[0]


def _r_str(f) -> str:
    n = _r(f, "<Q")
    if n > (1 << 24):
        raise ValueError(f"GGUF: string of {n} bytes")
    return f.read(n).decode("utf-8")


def _r_val(f, t):
    if t in _GV_FMT:
        return _r(f, _GV_FMT[t])
    if t == _GV_STRING:
        return _r_str(f)
    if t == _GV_ARRAY:
        et, n = _r(f, "<I"), _r(f, "<Q")
        return [_r_val(f, et) for _ in range(n)]
    raise ValueError(f"GGUF: unknown metadata value type {t}")


def readGGUF(path: str):
    """(metadata dict, [GGUFTensorInfo], offset of the data section in the file)."""
    with open(path, "rb") as f:
        if _r(f, "<I") != GGUF_MAGIC:
            raise ValueError(f"{path}: not a GGUF file")
        version = _r(f, "<I")
        if version not in (2, 3):
            raise ValueError(f"{path}: GGUF version {version} is not supported")
        nt, nkv = _r(f, "<Q"), _r(f, "<Q")
        meta = {}
        for _ in range(nkv):
            k = _r_str(f)
            meta[k] = _r_val(f, _r(f, "<I"))
        infos = []
        for _ in range(nt):
            name = _r_str(f)
            nd = _r(f, "<I")
            ne = [_r(f, "<Q") for _ in range(nd)]
            t, off = _r(f, "<I"), _r(f, "<Q")
            if t not in _GGML:
                raise ValueError(f"{path}: tensor '{name}' has ggml type {t}; this loader reads F32, F16, BF16, I32 and Q4_K")
            shape = list(reversed(ne))
            infos.append(GGUFTensorInfo(name, shape, t, off, _gguf_nbytes(shape, t)))
        align = int(meta.get("general.alignment", 32))
        pos = f.tell()
        data_start = (pos + align - 1) // align * align
        f.seek(0, 2)
        size = f.tell()
    for i in infos:
        if i.offset % align or data_start + i.offset + i.nbytes > size:
            raise ValueError(f"{path}: tensor '{i.name}' lies outside the file or off the {align}-byte grid")
    return meta, infos, data_start


def _w_str(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _w_val(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<I", 7) + struct.pack("<?", v)
    if isinstance(v, int):
        return (struct.pack("<I", 4) + struct.pack("<I", v)) if 0 <= v < (1 << 32) else (struct.pack("<I", 11) + struct.pack("<q", v))
    if isinstance(v, float):
        return struct.pack("<I", 6) + struct.pack("<f", v)
    if isinstance(v, str):
        return struct.pack("<I", _GV_STRING) + _w_str(v)
    raise TypeError(f"GGUF metadata value {v!r}")


def writeGGUF(path: str, tensors: dict, metadata: dict | None = None, alignment: int = 32) -> None:
    """``tensors``: name -> (ggml type, row-major shape, numpy array of raw bytes/values)."""
    meta = {"general.architecture": "qwen35", "general.alignment": alignment, **(metadata or {})}
    head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(meta))
    for k, v in meta.items():
        head += _w_str(k) + _w_val(v)
    off, blobs = 0, []
    for name, (t, shape, arr) in tensors.items():
        arr = np.ascontiguousarray(arr)
        if arr.nbytes != _gguf_nbytes(shape, t):
            raise ValueError(f"'{name}': {arr.nbytes} bytes for shape {shape} of {_GGML[t][0]}")
        head += _w_str(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in reversed(shape))
        head += struct.pack("<IQ", t, off)
        blobs.append((off, arr))
        off += (arr.nbytes + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * ((-len(head)) % alignment))
        start = f.tell()
        for o, arr in blobs:
            f.seek(start + o)
            f.write(arr.tobytes())
        f.truncate(start + off)


def loadGGUF(path: str, chunk_bytes: int = CHUNK_BYTES):
    """The data section in one device buffer; returns (SafeTensorsFile-like holder with dtype = ggml type name, metadata)."""
    meta, infos, data_start = readGGUF(path)
    nbytes = max((i.offset + i.nbytes for i in infos), default=0)
    base = rt.cuAlloc(max(nbytes, 16))
    try:
        with open(path, "rb", buffering=0) as f:
            _upload_range(f, data_start, nbytes, base, chunk_bytes)
    except Exception:
        rt.cuFree(base)
        raise
    tensors = {i.name: Tensor(i.name, base + i.offset, i.shape, _GGML[i.ggml_type][0], i.nbytes) for i in infos}
    return SafeTensorsFile(tensors, base, meta)


# ------------------------------------------------------------------------------------------ model weights
def safeKey(name: str, W) -> str | None:
    """Graph tensor name -> checkpoint tensor name (prototypes/decode_graph.ts:97-108).  The reference ties
    lm_head to the embedding; here a checkpoint's own ``lm_head.weight`` wins when it has one."""
    if name == "lm_head.weight":
        for k in ("lm_head.weight", "model.language_model.embed_tokens.weight", "model.embed_tokens.weight"):
            if k in W:
                return k
        return None
    if name == "embed.weight":
        for k in ("embed.weight", "model.language_model.embed_tokens.weight", "model.embed_tokens.weight"):
            if k in W:
                return k
        return None
    if name == "final.norm.weight":
        for k in ("final.norm.weight", "model.language_model.norm.weight", "model.norm.weight"):
            if k in W:
                return k
        return None
    if name.startswith("model."):
        prefixed = "model.language_model." + name[len("model."):]
        if prefixed in W:
            return prefixed
    return name if name in W else None


def _bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x7FFFFF) != 0)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return np.where(nan, (u >> 16) | 0x40, r).astype(np.uint16)


def _to_f32(bits: np.ndarray, dtype: DType) -> np.ndarray:
    if dtype == "F32":
        return bits.view(np.float32)
    if dtype == "BF16":
        return (bits.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    if dtype == "F16":
        return bits.view(np.float16).astype(np.float32)
    raise ValueError(f"cannot convert {dtype} to f32")


@dataclass
class LoadedModel:
    """Device pointers by graph weight name (``DecodeEnv(..., device_weights=model.weights)``)."""
    dims: Dims
    weights: dict
    quantized_bytes: int = 0
    source_bytes: int = 0
    _owned: list = field(default_factory=list)
    _files: list = field(default_factory=list)

    def free(self) -> None:
        for p in self._owned:
            rt.cuFree(p)
        for f in self._files:
            f.free()
        self._owned, self._files, self.weights = [], [], {}

    def host_weight(self, graph: Graph, name: str) -> np.ndarray:
        """Raw bytes of one resident weight (tests, export)."""
        return rt.from_device(self.weights[name], (tensor_bytes(graph.tensors[name]),), np.uint8)


def rope_tables(D: Dims):
    """cos/sin f32 [MAX_LEN, ROT_HALF], f_i = theta^(-2i/ROT_DIM) in double (prototypes/decode_graph.ts:120-131)."""
    i = np.arange(D.ROT_HALF, dtype=np.float64)
    f = 1.0 / np.power(D.ROPE_THETA, 2.0 * i / D.ROT_DIM)
    ang = np.arange(D.MAX_LEN, dtype=np.float64)[:, None] * f[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def loadQwen35(path: str, D: Dims, graph: Graph | None = None, keep_source: bool = False) -> LoadedModel:
    """A bf16 / f16 / f32 safetensors checkpoint, or a GGUF file written by ``saveGGUF`` -> resident weights.

    Every weight the graph declares is looked up through ``safeKey``, checked against the declared shape, and
      * ``q4_k`` tensors: quantized on the device from the uploaded bf16 / f32 rows (or taken as they are when the
        file already holds Q4_K blocks);
      * other tensors: used in place when the checkpoint type is the declared one, else converted (small tensors:
        A_log, norm weights).
    The uploaded source buffer is released at the end unless a non-quantized tensor still points into it."""
    graph = graph or buildModelGraph(D, 1)
    is_gguf = path.endswith(".gguf")
    src = loadGGUF(path) if is_gguf else loadSafeTensors(path)
    W = src.tensors
    model = LoadedModel(D, {})
    model.source_bytes = sum(t.nbytes for t in W.values())
    views_into_source = False
    try:
        for name, t in graph.tensors.items():
            if t.role != "weight":
                continue
            if name in ("rope_cos", "rope_sin"):
                cos_t, sin_t = rope_tables(D)
                p = rt.to_device(cos_t if name == "rope_cos" else sin_t)
                model._owned.append(p)
                model.weights[name] = p
                continue
            key = safeKey(name, W)
            if key is None:
                raise KeyError(f"loadQwen35: '{name}' has no tensor in {path}")
            st = W[key]
            shape = list(t.type.shape)
            if list(st.shape) != shape:
                raise ValueError(f"loadQwen35: '{key}' has shape {st.shape}, the graph declares {shape} for '{name}'")
            want = t.type.dtype
            if want == "q4_k":
                N, K = shape
                if st.dtype == "Q4_K":
                    model.weights[name] = st.devPtr
                    views_into_source = True
                    continue
                if st.dtype not in ("BF16", "F32"):
                    raise ValueError(f"loadQwen35: '{key}' is {st.dtype}; the quantizer reads BF16 or F32")
                if K % 256:
                    raise ValueError(f"loadQwen35: '{key}' has K={K}, not a multiple of the 256-element super-block")
                out = rt.cuAlloc(N * (K // 256) * 144)
                model._owned.append(out)
                srcp, tmp = st.devPtr, 0
                if srcp % 16:                      # checkpoint offsets are only element-aligned; the kernel reads 16 bytes at a time
                    tmp = srcp = rt.cuAlloc(st.nbytes)
                    rt.cuDtoD(tmp, st.devPtr, st.nbytes)
                rt.quantize_q4k(srcp, out, N, K, rt.BF16 if st.dtype == "BF16" else rt.F32)
                if tmp:
                    rt.cuSync()
                    rt.cuFree(tmp)
                model.weights[name] = out
                model.quantized_bytes += N * (K // 256) * 144
                continue
            have = {"BF16": "bf16", "F32": "f32", "F16": "f16", "I32": "i32"}.get(st.dtype)
            if have == want:
                model.weights[name] = st.devPtr
                views_into_source = True
                continue
            host = rt.from_device(st.devPtr, (st.nbytes,), np.uint8)
            vals = _to_f32(host, st.dtype).reshape(shape)
            conv = vals.astype(np.float32) if want == "f32" else _bf16_bits(vals) if want == "bf16" else None
            if conv is None:
                raise ValueError(f"loadQwen35: cannot convert '{key}' from {st.dtype} to {want}")
            p = rt.to_device(conv)
            model._owned.append(p)
            model.weights[name] = p
        rt.cuSync()
    except Exception:
        model.free()
        src.free()
        raise
    if views_into_source or keep_source:
        if not keep_source and not is_gguf:
            _compact(model, src, graph)
        else:
            model._files.append(src)
    else:
        src.free()
    return model


def _compact(model: LoadedModel, src: SafeTensorsFile, graph: Graph) -> None:
    """Copy the non-quantized tensors that still point into the checkpoint buffer into one small buffer and
    release the checkpoint buffer (the bf16 source of the linear weights is most of it)."""
    lo, hi = src.base, src.base + max((t.devPtr - src.base + t.nbytes for t in src.tensors.values()), default=0)
    inside = [n for n, p in model.weights.items() if lo <= p < hi]
    sizes = {n: (tensor_bytes(graph.tensors[n]) + 255) // 256 * 256 for n in inside}
    buf = rt.cuAlloc(max(sum(sizes.values()), 16))
    off = 0
    for n in inside:
        rt.cuDtoD(buf + off, model.weights[n], tensor_bytes(graph.tensors[n]))
        model.weights[n] = buf + off
        off += sizes[n]
    rt.cuSync()
    model._owned.append(buf)
    src.free()


def saveGGUF(model: LoadedModel, path: str, graph: Graph | None = None) -> None:
    """The resident weights (Q4_K linear weights, bf16 / f32 others) under their graph names."""
    graph = graph or buildModelGraph(model.dims, 1)
    types = {"q4_k": GGML_Q4_K, "bf16": GGML_BF16, "f32": GGML_F32, "i32": GGML_I32}
    tensors = {}
    for name, p in model.weights.items():
        if name in ("rope_cos", "rope_sin"):
            continue
        t = graph.tensors[name]
        raw = rt.from_device(p, (tensor_bytes(t),), np.uint8)
        tensors[name] = (types[t.type.dtype], list(t.type.shape), raw)
    d = model.dims
    writeGGUF(path, tensors, {"qwen35.hidden": d.H, "qwen35.vocab": d.VOCAB, "qwen35.layers": d.NL, "qwen35.ffn": d.INTER})
