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
FMT_INT4_G128, FMT_BF16, FMT_Q4K = 0, 1, 2

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
_sig("moe_gate_logits_pair", [vp, vp, vp, vp, i32, i32, i32, i32, vp, vp, vp, i32, i32, vp])
_sig("moe_topk", [vp, i32, i32, i32, i32, i32, vp, vp, vp])
_sig("moe_dispatch", [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp])
_sig("moe_dispatch_workspace_bytes", [i32, i32, i32], C.c_int64)
_sig("moe_dispatch_ws", [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp, i64, vp, vp])
_sig("moe_route_decode", [vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp, vp])
_sig("moe_experts_decode_int4", [vp, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp])
_sig("moe_experts_decode_int4_publish", [vp, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32,
                                          vp, vp, vp, vp, i32, vp])
_sig("moe_topk_dispatch", [vp, i32, i32, i32, i32, i32] + [vp] * 10 + [i32, vp, vp, vp, i32, vp])
_sig("moe_gate_route_ws_bytes", [i32, i32], i64)
_sig("moe_gate_topk_dispatch", [vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, i32, i32] + [vp] * 10 +
     [i32, vp, vp, vp, i32, vp, i32, i32, vp, vp])
_sig("moe_decode_batch_int4_gate_fits", [i32] * 7, i32)
_sig("moe_decode_batch_int4_gate", [vp, i32, vp, vp, i32, vp, i32, vp, i32, i32, i32, i32, i32, i32, i32] + [vp] * 13 +
     [i32] + [vp] * 8 + [i32, i32, vp])
_sig("moe_noalloc_scratch_bytes", [], i64)
_sig("moe_decode_token_int4_noalloc", [vp, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp, vp])
_sig("moe_decode_token_int4", [vp, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp] + [vp] * 15 + [vp, vp, vp, i32, i32, vp, vp, vp])
_sig("moe_gate_ws_bytes", [], i64)
_sig("moe_decode_token_late_expert_int4", [vp, i32, i32, u64, i32, vp, vp, vp, vp])
_sig("moe_decode_token_int4_gate", [vp, vp, vp, i32, vp, i32, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp] + [vp] * 15 +
     [vp, vp, vp, i32, i32, vp, vp, vp])
_sig("moe_predictor_windows", [vp, vp, vp])
_sig("moe_predictor_set_model", [vp, i32, i32, vp, vp, i32])
_sig("moe_predictor_start", [vp])
_sig("moe_predictor_stats", [vp, vp, vp])
_sig("moe_predictor_set_min_precision", [vp, C.c_float])
_sig("moe_predictor_precision", [vp, vp, vp])
_sig("moe_predictor_wait_idle", [vp, C.c_int])
_sig("moe_q4k_layout_make", [i32, i32, C.POINTER(Int4Layout)])
_sig("moe_experts_decode_q4k", [vp, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp])
_sig("moe_prefill_workspace_bytes", [i32, i32, i32], C.c_int64)
_sig("moe_prefill_tile_rows", [])
_sig("moe_experts_prefill", [vp, i32, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp])
_sig("moe_experts_prefill_pieces", [vp, i32, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp, vp, vp, vp, vp, i32, vp, vp, i32, vp])
_sig("moe_prefill_shared_splits", [i32, i32, i32, i32])
_sig("moe_kernel_timing", [i32])
_sig("moe_kernel_timing_read", [i32, C.POINTER(C.c_double), C.POINTER(i32)])
_sig("moe_combine", [vp, vp, vp, vp, vp, i32, vp, i32, i32, i32, vp])
_sig("moe_combine_splits", [vp, vp, vp, vp, vp, i32, vp, i32, i32, i32, i32, vp])
_sig("moe_decode_shared_splits", [i32, i32, i32, i32])


def check(rc: int, what: str = ""):
    if rc != 0:
        raise MoeError("%s failed (%d): %s" % (what, rc, lib.moe_last_error().decode()))


def ptr(t) -> int:
    """Device/host address of a torch tensor (None -> NULL)."""
    return 0 if t is None else t.data_ptr()


def cur_stream() -> int:
    return torch.cuda.current_stream().cuda_stream

# ---- engine (include/moe_engine.h) ----
BACKEND_HIP, BACKEND_HOST = 0, 1
sz = C.c_size_t
pp = C.POINTER(vp)


class Counters(C.Structure):
    _fields_ = [(n, u64) for n in ("hit", "miss", "ready", "unready", "prefetch_hit", "prefetch_miss",
                                   "activated", "wait_us", "h2d_bytes", "h2d_copies", "evictions",
                                   "forwards")]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


class LayerDesc(C.Structure):
    _fields_ = [("H", i32), ("I", i32), ("I_sh", i32), ("top_k", i32), ("route_mode", i32), ("fmt", i32),
                ("shared_gated", i32), ("gate_w", vp), ("gate_bias", vp), ("shared", vp)]


_sig("moe_cfg_create", [i32, i32], vp)
_sig("moe_cfg_destroy", [vp], None)
_sig("moe_cfg_set", [vp, C.c_char_p, C.c_char_p])
_sig("moe_cfg_set_params", [vp, C.POINTER(C.c_char_p), i32])
_sig("moe_cfg_finalize", [vp])
_sig("moe_cfg_get", [vp, C.c_char_p, C.c_char_p, i32])
_sig("moe_engine_create", [vp, i32, vp, pp])
_sig("moe_engine_destroy", [vp], None)
_sig("moe_host_alloc", [sz], vp)
_sig("moe_host_free", [vp], None)
_sig("moe_register_param", [vp, i32, i32, i32, vp, sz, sz])
_sig("moe_pin_host", [vp, C.POINTER(i32)])
_sig("moe_init_slots", [vp])
_sig("moe_slot_distribution", [i64, i32, C.POINTER(i64)])
_sig("moe_slot_info", [vp, i32, C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)])
_sig("moe_launch", [vp])
_sig("moe_expert_param_ptr", [vp, i32, i32, i32, pp])
_sig("moe_expert_ptr_table", [vp, i32, pp])
_sig("moe_flush_table", [vp, i32, vp])
_sig("moe_expert_status", [vp, i32, i32])
_sig("moe_is_in_cache", [vp, i32, i32])
_sig("moe_expert_num_ready", [vp, i32, i32])
_sig("moe_report_layer_logits", [vp, i32, vp, i32, i32, i32])
_sig("moe_report_one_layer", [vp, i32, vp, i64])
_sig("moe_wait_expert", [vp, i32, i32])
_sig("moe_expert_launched", [vp, i32, i32])
_sig("moe_layer_done", [vp, i32])
_sig("moe_acquire_layer", [vp, i32, vp, i64])
_sig("moe_release_layer", [vp, i32])
_sig("moe_release_experts", [vp, i32, vp, i64])
_sig("moe_prefetch_layer", [vp, i32, vp, i64, i32])
_sig("moe_attach_predictor", [vp, i32])
_sig("moe_update_priority", [vp, vp, i32, i32])
_sig("moe_oracle_load", [vp, vp, i64, vp, i64, vp, i64, vp, i64])
_sig("moe_set_seq", [vp, u64])
_sig("moe_streams", [vp, pp, pp])
_sig("moe_drain", [vp])
_sig("moe_get_counters", [vp, C.POINTER(Counters)])
_sig("moe_report", [vp, i32, C.c_char_p, i32])
_sig("moe_set_layer", [vp, i32, C.POINTER(LayerDesc)])
_sig("moe_forward_prepare", [vp, i32])
_sig("moe_forward", [vp, i32, vp, i32, vp])
_sig("moe_last_routing", [vp, pp, pp, pp])
_sig("moe_last_routing_host", [vp, i32, i32, vp, vp])
