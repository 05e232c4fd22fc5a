"""MI355X (gfx950) PTIR backend for gpt.rs: host-side mirror of the reference interface.

The directory name carries a dot, so Python cannot import it by name; load it with
`__graft_entry__.load_package()` (registers it as module `gptrs_amd`).

    ptir        PTIR program model + builder DSL + serde-JSON wire form
    functional  emitters for the LM functionals, op for op as the reference emits them
    models      GPT-2 / Ministral drivers and the greedy Generator, generic over a backend
    quant       weight-only int8 / int4-g128 packing
    backend     ctypes binding of libgptrs_hip.so (the PortableBackend surface)
    build       hipcc build of libgptrs_hip.so
"""
from . import ptir, functional, models  # noqa: F401
from .ptir import FunctionBuilder, Program, Tensor, TensorSpec  # noqa: F401


def hip_backend(device: int = 0):
    """Constructs the HIP backend (raises when the library or a GPU is missing)."""
    from .backend import HipBackend
    return HipBackend(device)
