"""ctypes binding of libmoe_a2a.so (the C ABI declared in include/moe_a2a.h).

There is no fallback: if the library is missing or a call fails, this raises.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import os

PKG_DIR = Path(__file__).resolve().parent
# MOE_A2A_LIBRARY points at another build of the same ABI (used to compare tuning variants)
LIBRARY = Path(os.environ.get("MOE_A2A_LIBRARY") or PKG_DIR / "libmoe_a2a.so")

F16, BF16 = 0, 1


class Shape(C.Structure):
    """struct moe_a2a_shape"""

    _fields_ = [
        ("world_size", C.c_int32),
        ("rank", C.c_int32),
        ("num_experts", C.c_int32),
        ("experts_per_token", C.c_int32),
        ("hidden_dim", C.c_int32),
        ("max_num_tokens", C.c_int32),
    ]


class MoeA2AError(RuntimeError):
    pass


_P, _I = C.c_void_p, C.c_int32
_SP = C.POINTER(Shape)

# name -> argument types; every function returns int (status) unless noted
SIGNATURES = {
    "moe_a2a_dispatch_send": [_SP, _P, _P, _I, _P, _P, _P, _P, _P],
    "moe_a2a_plan_send": [_SP, _P, _I, _P, _P, _P, _P, _P, _P],
    "moe_a2a_dispatch_recv": [_SP, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P],
    "moe_a2a_dispatch_recv_long": [_SP, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P],
    "moe_a2a_dispatch_recv_static": [_SP, _P, _P, _P, _I, _I, _P, _P, _P, C.POINTER(C.c_void_p), _P],
    "moe_a2a_combine_send": [_SP, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P],
    "moe_a2a_combine_recv": [_SP, _P, _P, _P, _I, _I, _P, _I, _P, _I, _I, _P],
    "moe_a2a_combine_recv_long": [_SP, _P, _P, _P, _I, _I, _P, _I, _P, _I, _I, _P, _P],
    "moe_a2a_expert_scale": [_SP, _P, _P, _I, _I, _I, _P, _P],
    "moe_a2a_expert_gemm": [_SP, _P, _P, _I, _P, _P, _I, _I, _I, _P, _P],
    "moe_a2a_linear": [_P, _P, _P, _I, _I, _I, _I, _P, _P],
    "moe_a2a_exchange_local": [_I, _I, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _P],
    "moe_a2a_exchange_gather_local": [_I, _I, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _P],
    "moe_a2a_dispatch_recv_compact": [_SP, _P, _P, _P, _I, _I, _P, _P, _P, _P, _I, _P, _P],
    "moe_a2a_expert_scale_compact": [_SP, _P, _P, _I, _I, _I, _I, _P, _P],
    "moe_a2a_expert_gemm_compact": [_SP, _P, _P, _I, _I, _P, _P, _I, _I, _I, _P, _P],
    "moe_a2a_combine_send_compact": [_SP, _P, _P, _P, _I, _I, _I, _P, _P, _P, _P, _P],
}
STRING_FUNCTIONS = {"moe_a2a_version": [], "moe_a2a_build_id": [], "moe_a2a_strerror": [_I]}

_lib = None


def load() -> C.CDLL:
    """Load the library once. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIBRARY.exists():
        raise MoeA2AError(
            f"{LIBRARY} is missing: build it with `python -m amd_distributed_2025_amd.build` "
            "(there is no CPU fallback for this path)"
        )
    lib = C.CDLL(str(LIBRARY))
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = args, C.c_int
    for name, args in STRING_FUNCTIONS.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = args, C.c_char_p
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().moe_a2a_strerror(status).decode()
        raise MoeA2AError(f"{what}: status {status} ({msg})")


def call(name: str, *args) -> None:
    check(getattr(load(), name)(*args), name)
