"""PortableBackend-shaped wrapper around the CPU oracle, so the model drivers in
gpt.rs_amd/models.py run unchanged against it (test infrastructure only)."""
from __future__ import annotations

import json
from typing import List, Optional, Sequence

import numpy as np

import __graft_entry__ as entry

po = entry.load_oracle()


class _Resolver:
    def __init__(self):
        self.map = {}

    def get(self, sid: bytes):
        return self.map.get(bytes(sid))

    def set(self, sid: bytes, handle):
        self.map[bytes(sid)] = handle


class OracleHandle:
    def __init__(self, t, spec):
        self.t, self.spec = t, spec


class OracleBackend:
    def __init__(self):
        self._params = _Resolver()
        self._parsed = {}

    def backend_name(self):
        return "oracle"

    def param_resolver(self):
        return self._params

    def materialize(self, spec, data):
        if data is None:
            arr = np.zeros(spec.dims, dtype=po.NP_DTYPES[spec.dtype])
            return OracleHandle(po.OTensor(spec.dtype, arr), spec)
        if isinstance(data, np.ndarray):
            data = data.tobytes()
        return OracleHandle(po.OTensor.from_bytes(spec.dtype, spec.dims, bytes(data)), spec)

    def to_literal(self, h) -> bytes:
        return h.t.to_bytes()

    def to_numpy(self, h) -> np.ndarray:
        return h.t.a

    def run_program(self, program, inputs: Sequence[OracleHandle], donate=None) -> List[OracleHandle]:
        key = program.key
        if key not in self._parsed:
            self._parsed[key] = json.loads(program.json_bytes)
        outs = po.run_program(self._parsed[key], [h.t for h in inputs])
        return [OracleHandle(t, s) for t, s in zip(outs, program.result_specs)]

    def sample_decode_token(self, logits, temperature=0.0, top_k=None, random_u=None) -> Optional[int]:
        a = logits.t.a
        row = a[-1] if a.ndim == 2 else a
        if top_k is not None:
            return None
        if temperature > 0.0:
            return None if random_u is None else po.sample_temperature(row, temperature, random_u)
        return po.argmax_first(row)

    def synchronize(self):
        pass
