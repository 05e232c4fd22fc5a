"""`GPTRSCHK` v2 checkpoints: indexed, random-access model files (docs/formats.md:15-64;
crates/gpt-rs/src/checkpoint/loader.rs, saver.rs; scripts/gptrs_eval/checkpoint.py).

    magic "GPTRSCHK" | version u32 = 2 | config_len u32 | config_json | index_len u32 | index | tensor payloads

config_json is {"kind": "gpt" | "ministral" | ..., "config": {...}} (an untagged object is a legacy GPT config,
loader.rs).  The index lists, per tensor: name_len u32, name (UTF-8), stored_base_id u128 (0 = derive from the
name), rank u32, dims u64 x rank, dtype_tag u32, one legacy byte, absolute offset u64, byte_len u64; everything
little-endian, payloads row-major.  dtype tags are the PTIR ones (F32 = 0, F16 = 1, BF16 = 2, SI32 = 3); the
reference reads f32 and i32 only, this reader also takes bf16 / f16 payloads (as raw 16-bit words).

The reader maps the file and hands out views, so a model is uploaded tensor by tensor without ever holding the
whole file in host memory.
"""
from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from typing import Any, Dict, Iterator, List, Mapping, Optional, Tuple

import numpy as np

MAGIC = b"GPTRSCHK"
VERSION = 2
_NP_OF_TAG = {0: np.dtype("<f4"), 1: np.dtype("<u2"), 2: np.dtype("<u2"), 3: np.dtype("<i4")}
DTYPE_OF_TAG = {0: "F32", 1: "F16", 2: "Bf16", 3: "Si32"}
TAG_OF_DTYPE = {v: k for k, v in DTYPE_OF_TAG.items()}


class CheckpointError(ValueError):
    pass


@dataclass(frozen=True)
class Entry:
    name: str
    base_id: int
    dims: Tuple[int, ...]
    dtype_tag: int
    flag: int          # the legacy byte (the Python exporter stores requires_grad there); ignored by readers
    offset: int        # absolute file offset of the payload
    byte_len: int

    @property
    def dtype(self) -> str:
        return DTYPE_OF_TAG[self.dtype_tag]


class _Cursor:
    def __init__(self, buf, pos: int, end: int, what: str):
        self.buf, self.pos, self.end, self.what = buf, pos, end, what

    def take(self, n: int) -> bytes:
        if n < 0 or self.pos + n > self.end:
            raise CheckpointError(f"checkpoint {self.what} is truncated")
        out = bytes(self.buf[self.pos:self.pos + n])
        self.pos += n
        return out

    def u32(self) -> int:
        return struct.unpack("<I", self.take(4))[0]

    def u64(self) -> int:
        return struct.unpack("<Q", self.take(8))[0]


class Checkpoint:
    """Read side.  `with Checkpoint(path) as ck: ck.kind, ck.config, ck.names(), ck.array(name)`."""

    def __init__(self, path: str):
        self._file = open(path, "rb")
        try:
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError as e:   # empty file
            self._file.close()
            raise CheckpointError("invalid checkpoint magic header") from e
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    # -- parsing -------------------------------------------------------------------------
    def _parse(self):
        size = len(self._map)
        head = _Cursor(self._map, 0, size, "header")
        if head.take(8) != MAGIC:
            raise CheckpointError("invalid checkpoint magic header")
        version = head.u32()
        if version != VERSION:
            raise CheckpointError(f"unsupported checkpoint version {version}")
        try:
            cfg = json.loads(head.take(head.u32()).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise CheckpointError(f"checkpoint config is not valid JSON: {e}") from e
        if not isinstance(cfg, dict):
            raise CheckpointError("checkpoint config must be a JSON object")
        if "kind" in cfg and "config" in cfg:
            self.kind, self.config = str(cfg["kind"]), cfg["config"]
            self.runtime = cfg.get("runtime")
        else:                       # legacy untagged GPT config (loader.rs wraps it the same way)
            self.kind, self.config, self.runtime = "gpt", cfg, None
        index_len = head.u32()
        idx = _Cursor(self._map, head.pos, head.pos + index_len, "index")
        if idx.end > size:
            raise CheckpointError("checkpoint index is truncated")
        self.entries: List[Entry] = []
        self._by_name: Dict[str, Entry] = {}
        for _ in range(idx.u32()):
            name = idx.take(idx.u32()).decode("utf-8")
            base_id = int.from_bytes(idx.take(16), "little")
            dims = tuple(idx.u64() for _ in range(idx.u32()))
            tag = idx.u32()
            if tag not in _NP_OF_TAG:
                raise CheckpointError(f"unknown dtype tag {tag} in checkpoint")
            flag = idx.take(1)[0]
            offset, byte_len = idx.u64(), idx.u64()
            count = int(np.prod(dims, dtype=np.int64)) if dims else 1
            if byte_len != count * _NP_OF_TAG[tag].itemsize:
                raise CheckpointError(f"tensor `{name}`: byte length {byte_len} does not match shape {list(dims)}")
            if offset + byte_len > size:
                raise CheckpointError(f"tensor `{name}`: payload runs past the end of the file")
            if name in self._by_name:
                raise CheckpointError(f"tensor `{name}` appears twice in the checkpoint index")
            e = Entry(name, base_id, dims, tag, flag, offset, byte_len)
            self.entries.append(e)
            self._by_name[name] = e

    # -- access --------------------------------------------------------------------------
    def names(self) -> List[str]:
        return [e.name for e in self.entries]

    def entry(self, name: str) -> Entry:
        try:
            return self._by_name[name]
        except KeyError:
            raise CheckpointError(f"tensor `{name}` not found in checkpoint") from None

    def __contains__(self, name: str) -> bool:
        return name in self._by_name

    def array(self, name: str) -> np.ndarray:
        """Read-only view of the payload in the file mapping (f32 / i32; bf16 and f16 as their 16-bit words)."""
        e = self.entry(name)
        return np.frombuffer(self._map, dtype=_NP_OF_TAG[e.dtype_tag], count=e.byte_len // _NP_OF_TAG[e.dtype_tag].itemsize,
                             offset=e.offset).reshape(e.dims)

    def __iter__(self) -> Iterator[Entry]:
        return iter(self.entries)

    def close(self):
        m, f = getattr(self, "_map", None), getattr(self, "_file", None)
        self._map = self._file = None
        if m is not None:
            try:
                m.close()
            except BufferError:   # views handed out by array() are still alive: the mapping goes with them
                pass
        if f is not None:
            f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _index_bytes(items, data_start: int) -> bytes:
    out = bytearray(struct.pack("<I", len(items)))
    rel = 0
    for name, dims, tag, flag, nbytes in items:
        nb = name.encode("utf-8")
        out += struct.pack("<I", len(nb)) + nb + (0).to_bytes(16, "little")
        out += struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", int(d)) for d in dims)
        out += struct.pack("<I", tag) + bytes([flag]) + struct.pack("<QQ", data_start + rel, nbytes)
        rel += nbytes
    return bytes(out)


def write_checkpoint(path: str, kind: str, config: Mapping[str, Any], tensors: Mapping[str, np.ndarray],
                     dtypes: Optional[Mapping[str, str]] = None, flags: Optional[Mapping[str, bool]] = None,
                     runtime: Optional[Mapping[str, Any]] = None) -> None:
    """Write side, as the exporters do (scripts/gptrs_eval/checkpoint.py): tensors sorted by name, stored ids 0,
    compact JSON config.  float32 / int32 arrays store as they are; `dtypes[name] = "Bf16"` stores a float32
    array rounded to bf16 (tag 2), uint16 arrays given as "Bf16" / "F16" store their words."""
    from .ptir import f32_to_bf16_bits
    items, payloads = [], []
    for name in sorted(tensors):
        arr = np.asarray(tensors[name], order="C")   # (ascontiguousarray would turn a rank-0 tensor into rank 1)
        want = (dtypes or {}).get(name)
        if want in ("Bf16", "F16") and arr.dtype == np.uint16:
            tag, data = TAG_OF_DTYPE[want], arr.astype("<u2").tobytes()
        elif want == "Bf16" and arr.dtype == np.float32:
            tag, data = 2, f32_to_bf16_bits(arr).astype("<u2").tobytes()
        elif want in (None, "F32") and arr.dtype == np.float32:
            tag, data = 0, arr.astype("<f4").tobytes()
        elif want in (None, "Si32") and arr.dtype == np.int32:
            tag, data = 3, arr.astype("<i4").tobytes()
        else:
            raise CheckpointError(f"unsupported dtype for {name}: {arr.dtype} as {want}")
        items.append((name, tuple(int(d) for d in arr.shape), tag, 1 if (flags or {}).get(name) else 0, len(data)))
        payloads.append(data)
    doc = {"kind": str(kind), "config": dict(config)}
    if runtime:   # runtime-only knobs, e.g. {"weight_streaming": {...}} (docs/formats.md:32, model/config.rs:31-40)
        doc["runtime"] = dict(runtime)
    cfg = json.dumps(doc, separators=(",", ":")).encode("utf-8")
    index_len = len(_index_bytes(items, 0))
    data_start = len(MAGIC) + 4 + 4 + len(cfg) + 4 + index_len
    with open(path, "wb") as f:
        f.write(MAGIC + struct.pack("<II", VERSION, len(cfg)) + cfg + struct.pack("<I", index_len))
        f.write(_index_bytes(items, data_start))
        for data in payloads:
            f.write(data)
