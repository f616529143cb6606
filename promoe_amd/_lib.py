"""ctypes binding of libmoe_engine.so (the C ABI declared in include/*.h).

The library is the product; there is no fallback: a missing or unloadable library
raises at import of this module.
"""
from __future__ import annotations

import ctypes as C
import os

import torch  # noqa: F401  (loads the process-wide HIP runtime the library binds to)

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmoe_engine.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "promoe_amd: %s is missing; build it with `python -m promoe_amd.build` "
        "(hipcc --offload-arch=gfx950)" % LIB_PATH)

lib = C.CDLL(LIB_PATH)

MOE_OK, MOE_EINVAL, MOE_EHIP, MOE_ESTATE, MOE_ENOMEM, MOE_ENOTRESIDENT = 0, -1, -2, -3, -4, -5
ROUTE_SOFTMAX_TOPK, ROUTE_SOFTMAX_TOPK_RENORM, ROUTE_TOPK_SOFTMAX = 0, 1, 2

vp, i32, i64, u64 = C.c_void_p, C.c_int, C.c_int64, C.c_uint64


class Int4Layout(C.Structure):
    _fields_ = [(n, i64) for n in ("off13_q", "off13_s", "off13_z", "off2_q", "off2_s", "off2_z",
                                   "total_bytes")]


class MoeError(RuntimeError):
    pass


def _sig(name, argtypes, restype=i32):
    f = getattr(lib, name)
    f.argtypes = argtypes
    f.restype = restype
    return f


_sig("moe_last_error", [], C.c_char_p)
_sig("moe_int4_layout_make", [i32, i32, C.POINTER(Int4Layout)])
_sig("moe_gate_logits", [vp, vp, vp, vp, i32, i32, i32, i32, vp])
_sig("moe_topk", [vp, i32, i32, i32, i32, i32, vp, vp, vp])
_sig("moe_dispatch", [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp])
_sig("moe_experts_decode_int4", [vp, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp])
_sig("moe_combine", [vp, vp, vp, vp, vp, vp, i32, i32, i32, vp])


def check(rc: int, what: str = ""):
    if rc != 0:
        raise MoeError("%s failed (%d): %s" % (what, rc, lib.moe_last_error().decode()))


def ptr(t) -> int:
    """Device/host address of a torch tensor (None -> NULL)."""
    return 0 if t is None else t.data_ptr()


def cur_stream() -> int:
    return torch.cuda.current_stream().cuda_stream
