"""ctypes binding of libgptrs_hip.so: the `PortableBackend` surface
(crates/gpt-rs/src/backend/spec.rs:1287-1349) as a Python class.

There is no CPU fallback: constructing HipBackend without the built library or without
a visible GPU raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Sequence

import numpy as np

from .ptir import Program, TensorSpec, bf16_bits_to_f32

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgptrs_hip.so")

DTYPE_TAG = {"F32": 0, "F16": 1, "Bf16": 2, "Si32": 3, "I1": 4, "Si8": 5, "Ui8": 6}
TAG_DTYPE = {v: k for k, v in DTYPE_TAG.items()}
NP_OF = {"F32": np.float32, "Si32": np.int32, "I1": np.uint8, "Bf16": np.uint16, "Si8": np.int8, "Ui8": np.uint8}

EXPORTS = [
    "gptrs_hip_create", "gptrs_hip_destroy", "gptrs_hip_backend_name", "gptrs_hip_materialize",
    "gptrs_hip_to_literal", "gptrs_hip_tensor_retain", "gptrs_hip_tensor_release", "gptrs_hip_tensor_spec",
    "gptrs_hip_run_program", "gptrs_hip_run_program_donate", "gptrs_hip_execute_instruction",
    "gptrs_hip_param_get", "gptrs_hip_param_set", "gptrs_hip_supports_decode_sampling",
    "gptrs_hip_sample_decode_token", "gptrs_hip_sample_decode_token_begin", "gptrs_hip_sample_decode_token_wait",
    "gptrs_hip_decode_token_tensor", "gptrs_hip_sample_decode_rows_begin", "gptrs_hip_sample_decode_rows_wait",
    "gptrs_hip_decode_rows_tensor", "gptrs_hip_sample_decode_rows_into", "gptrs_hip_fusion_report", "gptrs_hip_last_error", "gptrs_hip_synchronize", "gptrs_hip_set_option",
    "gptrs_hip_counter",
]


class BackendError(RuntimeError):
    """BackendError (spec.rs:1224-1228); `kind` in {"spec", "unimplemented", "execution"}."""

    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code
        self.kind = {1: "spec", 2: "unimplemented", 3: "execution"}.get(code, "execution")


class _Desc(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_uint32), ("rank", ctypes.c_uint32), ("dims", ctypes.POINTER(ctypes.c_int64))]


_lib = None


def load_library(path: str = LIB_PATH):
    """Loads the shared library and declares every entry point of include/gptrs_hip.h."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise FileNotFoundError(f"{path} is missing: run `python __graft_entry__.py build` (hipcc, gfx950) first")
    lib = ctypes.CDLL(path)
    vp, cp, sz = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t
    pvp = ctypes.POINTER(ctypes.c_void_p)
    lib.gptrs_hip_create.argtypes = [ctypes.c_int, pvp]
    lib.gptrs_hip_destroy.argtypes = [vp]
    lib.gptrs_hip_destroy.restype = None
    lib.gptrs_hip_backend_name.argtypes = [vp]
    lib.gptrs_hip_backend_name.restype = cp
    lib.gptrs_hip_materialize.argtypes = [vp, ctypes.POINTER(_Desc), vp, sz, pvp]
    lib.gptrs_hip_to_literal.argtypes = [vp, vp, vp, sz]
    lib.gptrs_hip_tensor_retain.argtypes = [vp]
    lib.gptrs_hip_tensor_retain.restype = None
    lib.gptrs_hip_tensor_release.argtypes = [vp]
    lib.gptrs_hip_tensor_release.restype = None
    lib.gptrs_hip_tensor_spec.argtypes = [vp, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_int64), sz]
    lib.gptrs_hip_run_program.argtypes = [vp, cp, sz, ctypes.c_uint64, pvp, sz, pvp, sz]
    lib.gptrs_hip_run_program_donate.argtypes = [vp, cp, sz, ctypes.c_uint64, pvp, ctypes.POINTER(ctypes.c_uint8), sz, pvp, sz]
    lib.gptrs_hip_execute_instruction.argtypes = [vp, cp, sz, pvp, sz, pvp]
    lib.gptrs_hip_param_get.argtypes = [vp, cp, pvp]
    lib.gptrs_hip_param_set.argtypes = [vp, cp, vp]
    lib.gptrs_hip_supports_decode_sampling.argtypes = [vp, ctypes.c_float, ctypes.c_int, ctypes.c_int]
    lib.gptrs_hip_sample_decode_token.argtypes = [vp, vp, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                                  ctypes.POINTER(ctypes.c_int64)]
    lib.gptrs_hip_sample_decode_token_begin.argtypes = [vp, vp, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                                        ctypes.POINTER(ctypes.c_int64)]
    lib.gptrs_hip_sample_decode_token_wait.argtypes = [vp, ctypes.c_int64, ctypes.POINTER(ctypes.c_int64)]
    lib.gptrs_hip_decode_token_tensor.argtypes = [vp, pvp]
    lib.gptrs_hip_sample_decode_rows_begin.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_int64)]
    lib.gptrs_hip_sample_decode_rows_wait.argtypes = [vp, ctypes.c_int64, ctypes.POINTER(ctypes.c_int32), sz]
    lib.gptrs_hip_decode_rows_tensor.argtypes = [vp, ctypes.c_int64, pvp]
    lib.gptrs_hip_sample_decode_rows_into.argtypes = [vp, vp, vp]
    lib.gptrs_hip_fusion_report.argtypes = [cp, sz, ctypes.POINTER(ctypes.c_int64), sz, ctypes.c_char_p, sz, ctypes.POINTER(sz)]
    lib.gptrs_hip_last_error.argtypes = []
    lib.gptrs_hip_last_error.restype = cp
    lib.gptrs_hip_synchronize.argtypes = [vp]
    lib.gptrs_hip_set_option.argtypes = [vp, cp, ctypes.c_int64]
    lib.gptrs_hip_counter.argtypes = [vp, cp]
    lib.gptrs_hip_counter.restype = ctypes.c_int64
    _lib = lib
    return lib


def fusion_report(program: Program, bcast_len: Optional[Sequence[int]] = None) -> List[str]:
    """gptrs_hip_fusion_report: the instructions that remain of `program` after the backend's fusion pass, one string
    each (no device needed).  `bcast_len[i]` > 0 marks input i as a handle the backend made by broadcasting a vector of
    that many values (a derived parameter of the reference's parameter-only fold)."""
    lib = load_library()
    js = program.json_bytes
    n_in = len(program.param_specs)
    lens = (ctypes.c_int64 * max(n_in, 1))(*([int(v) for v in bcast_len] if bcast_len is not None else [0] * n_in))
    needed = ctypes.c_size_t(0)
    code = lib.gptrs_hip_fusion_report(js, len(js), lens, n_in, None, 0, ctypes.byref(needed))
    if code == 0:
        buf = ctypes.create_string_buffer(needed.value)
        code = lib.gptrs_hip_fusion_report(js, len(js), lens, n_in, buf, needed.value, ctypes.byref(needed))
    if code != 0:
        raise BackendError(code, lib.gptrs_hip_last_error().decode("utf-8", "replace"))
    return buf.value.decode().splitlines()


class TensorHandle:
    """Reference-counted device tensor (`PortableBackend::TensorHandle`)."""

    __slots__ = ("backend", "ptr", "spec")

    def __init__(self, backend: "HipBackend", ptr: int, spec: TensorSpec):
        self.backend, self.ptr, self.spec = backend, ptr, spec

    def __del__(self):
        ptr, self.ptr = self.ptr, None
        if ptr and self.backend is not None and self.backend._handle:
            self.backend._lib.gptrs_hip_tensor_release(ptr)


class _ParamResolver:
    """ParamResolver (crates/gpt-rs/src/backend/param_resolver.rs:11-19) over the C ABI."""

    def __init__(self, backend: "HipBackend"):
        self.b = backend

    def get(self, stable_id: bytes) -> Optional[TensorHandle]:
        out = ctypes.c_void_p()
        self.b._check(self.b._lib.gptrs_hip_param_get(self.b._handle, bytes(stable_id), ctypes.byref(out)))
        if not out.value:
            return None
        return TensorHandle(self.b, out.value, self.b._spec_of(out.value))

    def set(self, stable_id: bytes, handle: TensorHandle):
        self.b._check(self.b._lib.gptrs_hip_param_set(self.b._handle, bytes(stable_id), handle.ptr))


class HipBackend:
    def __init__(self, device: int = 0):
        self._lib = load_library()
        self._handle = None
        out = ctypes.c_void_p()
        self._check(self._lib.gptrs_hip_create(device, ctypes.byref(out)))
        self._handle = out.value
        self._params = _ParamResolver(self)

    # -- plumbing ----------------------------------------------------------------------
    def _check(self, code: int):
        if code != 0:
            raise BackendError(code, self._lib.gptrs_hip_last_error().decode("utf-8", "replace"))

    def _spec_of(self, ptr: int) -> TensorSpec:
        dt = ctypes.c_uint32()
        dims = (ctypes.c_int64 * 8)()
        rank = self._lib.gptrs_hip_tensor_spec(ptr, ctypes.byref(dt), dims, 8)
        return TensorSpec(TAG_DTYPE[dt.value], tuple(dims[i] for i in range(rank)))

    def close(self):
        if self._handle:
            h, self._handle = self._handle, None
            self._lib.gptrs_hip_destroy(h)

    def __del__(self):
        # handles may outlive us in arbitrary order at interpreter exit; leak rather than double free
        pass

    # -- PortableBackend -----------------------------------------------------------------
    def backend_name(self) -> str:
        return self._lib.gptrs_hip_backend_name(self._handle).decode()

    def param_resolver(self) -> _ParamResolver:
        return self._params

    def materialize(self, spec: TensorSpec, data) -> TensorHandle:
        """TensorInit::Literal (bytes / numpy array) or TensorInit::Zeroed (data is None)."""
        dims = (ctypes.c_int64 * max(len(spec.dims), 1))(*spec.dims)
        desc = _Desc(DTYPE_TAG[spec.dtype], len(spec.dims), dims)
        out = ctypes.c_void_p()
        if data is None:
            self._check(self._lib.gptrs_hip_materialize(self._handle, ctypes.byref(desc), None, 0, ctypes.byref(out)))
        else:
            if isinstance(data, np.ndarray):
                arr = np.ascontiguousarray(data)
                ptr, n = arr.ctypes.data, arr.nbytes
                self._check(self._lib.gptrs_hip_materialize(self._handle, ctypes.byref(desc), ptr, n, ctypes.byref(out)))
            else:
                buf = bytes(data)
                self._check(self._lib.gptrs_hip_materialize(self._handle, ctypes.byref(desc), buf, len(buf), ctypes.byref(out)))
        return TensorHandle(self, out.value, spec)

    def to_literal(self, handle: TensorHandle) -> bytes:
        n = handle.spec.byte_len()
        buf = ctypes.create_string_buffer(max(n, 1))
        self._check(self._lib.gptrs_hip_to_literal(self._handle, handle.ptr, buf, n))
        return buf.raw[:n]

    def to_numpy(self, handle: TensorHandle) -> np.ndarray:
        """to_literal decoded to numpy (bf16 widened to float32)."""
        spec = handle.spec
        arr = np.empty(spec.dims, dtype=NP_OF[spec.dtype])
        self._check(self._lib.gptrs_hip_to_literal(self._handle, handle.ptr, arr.ctypes.data, arr.nbytes))
        if spec.dtype == "Bf16":
            return bf16_bits_to_f32(arr).reshape(spec.dims)
        return arr

    def run_program(self, program: Program, inputs: Sequence[TensorHandle],
                    donate: Optional[Sequence[bool]] = None) -> List[TensorHandle]:
        n_in, n_out = len(inputs), len(program.result_specs)
        in_arr = (ctypes.c_void_p * max(n_in, 1))(*[h.ptr for h in inputs])
        out_arr = (ctypes.c_void_p * max(n_out, 1))()
        js = program.json_bytes
        if donate is not None and any(donate):
            don = (ctypes.c_uint8 * max(n_in, 1))(*[1 if d else 0 for d in donate])
            code = self._lib.gptrs_hip_run_program_donate(self._handle, js, len(js), program.key, in_arr, don, n_in, out_arr, n_out)
        else:
            code = self._lib.gptrs_hip_run_program(self._handle, js, len(js), program.key, in_arr, n_in, out_arr, n_out)
        self._check(code)
        return [TensorHandle(self, out_arr[i], program.result_specs[i]) for i in range(n_out)]

    def run_program_json(self, js: bytes, key: int, inputs: Sequence[TensorHandle], n_out: int) -> List[TensorHandle]:
        n_in = len(inputs)
        in_arr = (ctypes.c_void_p * max(n_in, 1))(*[h.ptr for h in inputs])
        out_arr = (ctypes.c_void_p * max(n_out, 1))()
        self._check(self._lib.gptrs_hip_run_program(self._handle, js, len(js), key, in_arr, n_in, out_arr, n_out))
        return [TensorHandle(self, out_arr[i], self._spec_of(out_arr[i])) for i in range(n_out)]

    def execute_instruction(self, instruction_json: bytes, inputs: Sequence[TensorHandle]) -> TensorHandle:
        n_in = len(inputs)
        in_arr = (ctypes.c_void_p * max(n_in, 1))(*[h.ptr for h in inputs])
        out = ctypes.c_void_p()
        self._check(self._lib.gptrs_hip_execute_instruction(self._handle, instruction_json, len(instruction_json), in_arr, n_in, ctypes.byref(out)))
        return TensorHandle(self, out.value, self._spec_of(out.value))

    def supports_decode_sampling(self, temperature: float = 0.0, top_k: Optional[int] = None,
                                 random_u: Optional[float] = None) -> bool:
        return bool(self._lib.gptrs_hip_supports_decode_sampling(self._handle, temperature, top_k is not None, random_u is not None))

    def sample_decode_token(self, logits: TensorHandle, temperature: float = 0.0, top_k: Optional[int] = None,
                            random_u: Optional[float] = None) -> Optional[int]:
        tok = ctypes.c_int64(-1)
        self._check(self._lib.gptrs_hip_sample_decode_token(self._handle, logits.ptr, temperature, top_k is not None,
                                                            random_u is not None, random_u or 0.0, ctypes.byref(tok)))
        return None if tok.value < 0 else int(tok.value)

    def sample_decode_token_begin(self, logits: TensorHandle, temperature: float = 0.0, top_k: Optional[int] = None,
                                  random_u: Optional[float] = None) -> Optional[int]:
        """Queues the sampling and returns a ticket at once (None: not served here); see sample_decode_token_wait."""
        ticket = ctypes.c_int64(-1)
        self._check(self._lib.gptrs_hip_sample_decode_token_begin(self._handle, logits.ptr, temperature, top_k is not None,
                                                                  random_u is not None, random_u or 0.0, ctypes.byref(ticket)))
        return None if ticket.value < 0 else int(ticket.value)

    def sample_decode_token_wait(self, ticket: int) -> int:
        tok = ctypes.c_int64(-1)
        self._check(self._lib.gptrs_hip_sample_decode_token_wait(self._handle, ticket, ctypes.byref(tok)))
        return int(tok.value)

    def decode_token_tensor(self) -> TensorHandle:
        """si32[1] handle over the device copy of the last sampled token."""
        out = ctypes.c_void_p()
        self._check(self._lib.gptrs_hip_decode_token_tensor(self._handle, ctypes.byref(out)))
        return TensorHandle(self, out.value, self._spec_of(out.value))

    def sample_decode_rows_begin(self, logits: TensorHandle) -> int:
        """Queues the greedy token of every row of logits [rows, vocab]; returns a ticket for sample_decode_rows_wait."""
        ticket = ctypes.c_int64(-1)
        self._check(self._lib.gptrs_hip_sample_decode_rows_begin(self._handle, logits.ptr, ctypes.byref(ticket)))
        return int(ticket.value)

    def sample_decode_rows_wait(self, ticket: int, rows: int) -> list:
        buf = (ctypes.c_int32 * rows)()
        self._check(self._lib.gptrs_hip_sample_decode_rows_wait(self._handle, ticket, buf, rows))
        return [int(v) for v in buf]

    def sample_decode_rows_into(self, logits: TensorHandle, tokens_out: TensorHandle):
        """Queues the greedy token of every row of logits [rows <= 64, vocab] into tokens_out (si32[rows]); the call
        allocates nothing on the device."""
        self._check(self._lib.gptrs_hip_sample_decode_rows_into(self._handle, logits.ptr, tokens_out.ptr))

    def decode_rows_tensor(self, rows: int) -> TensorHandle:
        """si32[rows] handle over the device copy of the tokens of the last sample_decode_rows_begin."""
        out = ctypes.c_void_p()
        self._check(self._lib.gptrs_hip_decode_rows_tensor(self._handle, rows, ctypes.byref(out)))
        return TensorHandle(self, out.value, self._spec_of(out.value))

    # -- extras ----------------------------------------------------------------------------
    def synchronize(self):
        self._check(self._lib.gptrs_hip_synchronize(self._handle))

    def set_option(self, name: str, value: int):
        self._check(self._lib.gptrs_hip_set_option(self._handle, name.encode(), int(value)))

    def counter(self, name: str) -> int:
        return int(self._lib.gptrs_hip_counter(self._handle, name.encode()))
