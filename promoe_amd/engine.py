"""Python face of the expert-cache engine, named after the reference's pybind
classes (src/cpp_worker/adapter.cpp:13-158) so that host code written against
`sparse_llm_cache.cpp_worker` reads the same: ModuleMeta, ModelLoader, PrefetchMngr.
Everything delegates to libmoe_engine.so; nothing is computed here.
"""
from __future__ import annotations

import ctypes as C
from typing import Sequence

import numpy as np
import torch

from . import _lib as L
from ._lib import lib, check

EXPERT_STATUS = ("idle", "fetching", "ready", "launching", "using")  # utils.hpp:38-49


class ModuleMeta:
    """ModuleMeta(num_layer, num_expert) (adapter.cpp:14-40)."""

    def __init__(self, num_layer: int, num_expert: int):
        self._h = lib.moe_cfg_create(num_layer, num_expert)
        if not self._h:
            raise L.MoeError(lib.moe_last_error().decode())
        self.num_layer, self.num_expert = num_layer, num_expert
        self.param_name_list: list[str] = []
        self._finalized = False

    def __del__(self):
        if getattr(self, "_h", None) and lib is not None:
            lib.moe_cfg_destroy(self._h)
            self._h = None

    def init_param_list(self, names: Sequence[str]):
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        check(lib.moe_cfg_set_params(self._h, arr, len(names)), "init_param_list")
        self.param_name_list = list(names)

    def init_from_map(self, config_map: dict):
        """All values as strings; "None" selects the default (utils/__init__.py:263-288)."""
        for k, v in config_map.items():
            check(lib.moe_cfg_set(self._h, str(k).encode(), str(v).encode()), "init_from_map")

    def handle_uninited_configs(self):
        check(lib.moe_cfg_finalize(self._h), "handle_uninited_configs")
        self._finalized = True

    def get(self, key: str) -> str:
        buf = C.create_string_buffer(512)
        n = lib.moe_cfg_get(self._h, key.encode(), buf, 512)
        if n < 0:
            raise L.MoeError(lib.moe_last_error().decode())
        return buf.value.decode()

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        try:
            v = self.get(name)
        except L.MoeError:
            raise AttributeError(name)
        if v in ("true", "false"):
            return v == "true"
        for cast in (int, float):
            try:
                return cast(v)
            except ValueError:
                pass
        return v

    def param_id(self, name: str) -> int:
        return self.param_name_list.index(name)


class PinnedBuffer:
    """Pinned host memory from the library (hipHostMalloc), viewed as a numpy array."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = lib.moe_host_alloc(self.nbytes)
        if not self.ptr:
            raise MemoryError(lib.moe_last_error().decode())
        self.array = np.ctypeslib.as_array((C.c_uint8 * max(self.nbytes, 1)).from_address(self.ptr))[: self.nbytes]

    def free(self):
        if self.ptr:
            self.array = None
            lib.moe_host_free(self.ptr)
            self.ptr = None

    def __del__(self):
        self.free()


class PrefetchMngr:
    """ModelLoader + CacheMngr + PrefetchMngr of the reference behind one handle
    (adapter.cpp:53-106).  Method names follow the reference."""

    def __init__(self, meta: ModuleMeta, backend: int = L.BACKEND_HIP, compute_stream: int = 0):
        if not meta._finalized:
            meta.handle_uninited_configs()
        self.metas = meta
        h = C.c_void_p()
        check(lib.moe_engine_create(meta._h, backend, compute_stream, C.byref(h)), "PrefetchMngr")
        self._h = h
        self._keep = []   # host buffers registered with the engine
        self.backend = backend
        self._compute_stream_handle = None
        self._ext_stream = None

    def close(self):
        if getattr(self, "_h", None) and lib is not None:
            lib.moe_engine_destroy(self._h)
            self._h = None
            self._keep = []

    def __del__(self):
        self.close()

    # -- ModelLoader --
    def add_one_expert_param(self, host, layer_id: int, expert_id: int, name_or_id, alloc_nbytes: int = 0):
        """host: PinnedBuffer slice (numpy uint8 view), numpy array or CPU tensor; kept alive here."""
        pid = name_or_id if isinstance(name_or_id, int) else self.metas.param_id(name_or_id)
        if isinstance(host, torch.Tensor):
            assert not host.is_cuda and host.is_contiguous()
            addr, nbytes = host.data_ptr(), host.numel() * host.element_size()
        else:
            host = np.ascontiguousarray(host) if not host.flags["C_CONTIGUOUS"] else host
            addr, nbytes = host.ctypes.data, host.nbytes
        self._keep.append(host)
        check(lib.moe_register_param(self._h, layer_id, expert_id, pid, addr, nbytes, alloc_nbytes),
              "add_one_expert_param")

    def pin_memory(self) -> int:
        n = C.c_int(0)
        check(lib.moe_pin_host(self._h, C.byref(n)), "pin_memory")
        return n.value

    def ref_one_expert_param(self, layer_id: int, expert_id: int, name_or_id) -> int:
        """Device address of the parameter of a resident expert, 0 if it holds no slot."""
        pid = name_or_id if isinstance(name_or_id, int) else self.metas.param_id(name_or_id)
        out = C.c_void_p()
        check(lib.moe_expert_param_ptr(self._h, layer_id, expert_id, pid, C.byref(out)), "ref_one_expert_param")
        return out.value or 0

    # -- PrefetchMngr --
    def init_gpu_mem_buffer(self):
        check(lib.moe_init_slots(self._h), "init_gpu_mem_buffer")

    def launch_thread(self):
        check(lib.moe_launch(self._h), "launch_thread")

    def report_moe_layer_logits(self, layer_id: int, hidden=None, seq_len: int | None = None):
        if hidden is not None:
            B, S, H = (hidden.shape if len(hidden.shape) == 3 else (1,) + tuple(hidden.shape))
            p = hidden.ctypes.data if isinstance(hidden, np.ndarray) else hidden.data_ptr()
        else:
            B, S, H, p = 1, int(seq_len or 1), 0, 0
        check(lib.moe_report_layer_logits(self._h, layer_id, p, B, S, H), "report_moe_layer_logits")

    def report_one_layer(self, layer_id: int, experts):
        """experts: CPU int64 tensor or numpy array, reordered IN PLACE."""
        if isinstance(experts, torch.Tensor):
            assert experts.dtype == torch.int64 and not experts.is_cuda and experts.is_contiguous()
            addr, n = experts.data_ptr(), experts.numel()
        else:
            assert experts.dtype == np.int64 and experts.flags["C_CONTIGUOUS"]
            addr, n = experts.ctypes.data, experts.size
        check(lib.moe_report_one_layer(self._h, layer_id, addr, n), "report_one_layer")
        return experts

    def report_one_expert(self, layer_id: int, expert_id: int):
        check(lib.moe_wait_expert(self._h, layer_id, int(expert_id)), "report_one_expert")

    def one_expert_done(self, layer_id: int, expert_id: int):
        check(lib.moe_expert_launched(self._h, layer_id, int(expert_id)), "one_expert_done")

    def one_moe_layer_done(self, layer_id: int):
        check(lib.moe_layer_done(self._h, layer_id), "one_moe_layer_done")

    def acquire_layer(self, layer_id: int, experts: np.ndarray):
        check(lib.moe_acquire_layer(self._h, layer_id, experts.ctypes.data, experts.size), "acquire_layer")
        return experts

    def release_layer(self, layer_id: int):
        check(lib.moe_release_layer(self._h, layer_id), "release_layer")

    def release_experts(self, layer_id: int, experts):
        ids = np.ascontiguousarray(np.asarray(experts, dtype=np.int64))
        check(lib.moe_release_experts(self._h, layer_id, ids.ctypes.data, ids.size), "release_experts")

    def prefetch_layer(self, layer_id: int, experts, blocking: bool = True) -> bool:
        ids = np.ascontiguousarray(np.asarray(experts, dtype=np.int64))
        rc = lib.moe_prefetch_layer(self._h, layer_id, ids.ctypes.data, ids.size, 1 if blocking else 0)
        if rc == 1:
            return False
        check(rc, "prefetch_layer")
        return True

    def drain(self):
        check(lib.moe_drain(self._h), "drain")

    def attach_predictor(self, attached: bool = True):
        check(lib.moe_attach_predictor(self._h, int(attached)), "attach_predictor")

    # -- built-in predictor (linear model per source -> destination layer pair) --
    def predictor_windows(self):
        """[(first, last)] for source layers 0..L: the destination layers each one predicts."""
        n = int(self.metas.num_layer) + 1
        a, b = (C.c_int * n)(), (C.c_int * n)()
        check(lib.moe_predictor_windows(self._h, a, b), "predictor_windows")
        return list(zip(a, b))

    def set_predictor_model(self, src: int, dst: int, w, bias=None):
        """w bf16 [E, H] (device tensor; numpy uint16 bit patterns on the host backend), bias fp32 [E] or None."""
        self._keep.append((w, bias))
        H = int(w.shape[1])
        wp = w.ctypes.data if isinstance(w, np.ndarray) else L.ptr(w)
        bp = None if bias is None else (bias.ctypes.data if isinstance(bias, np.ndarray) else L.ptr(bias))
        check(lib.moe_predictor_set_model(self._h, src, dst, wp, bp, H), "set_predictor_model")

    def start_predictor(self):
        check(lib.moe_predictor_start(self._h), "start_predictor")

    def predictor_stats(self, settle_ms: int = 2000) -> dict:
        """Counters of the predictor thread, read once it has worked off the reports so far (or after settle_ms)."""
        lib.moe_predictor_wait_idle(self._h, settle_ms)
        a, b = C.c_uint64(), C.c_uint64()
        check(lib.moe_predictor_stats(self._h, C.byref(a), C.byref(b)), "predictor_stats")
        return {"jobs": a.value, "requests": b.value}

    def set_predictor_min_precision(self, t: float):
        """Requests for a layer whose predictions have lately been right for less than the share t go out empty
        (0 = never: the reference's behaviour)."""
        check(lib.moe_predictor_set_min_precision(self._h, float(t)), "set_predictor_min_precision")

    def predictor_precision(self):
        """(moving average of the predictions' precision per destination layer, requests sent empty so far)"""
        p = np.zeros(int(self.metas.num_layer), np.float32)
        n = C.c_uint64()
        check(lib.moe_predictor_precision(self._h, p.ctypes.data, C.byref(n)), "predictor_precision")
        return p, n.value

    def update_priority(self, p: np.ndarray, starting_layer: int = 0):
        p = np.ascontiguousarray(p, dtype=np.float32)
        check(lib.moe_update_priority(self._h, p.ctypes.data, p.shape[0], starting_layer), "update_priority")

    # -- CacheMngr / CacheOracle --
    def set_cur_seq(self, seq_id: int):
        check(lib.moe_set_seq(self._h, seq_id), "set_cur_seq")

    def load_oracle(self, entry_metas, prefill_expert_len, prefill_expert_selection, decode_expert_selection):
        em = np.ascontiguousarray(entry_metas, dtype=np.int64).reshape(-1, 2)
        pl = np.ascontiguousarray(prefill_expert_len, dtype=np.int32)
        ps = np.ascontiguousarray(prefill_expert_selection, dtype=np.int32)
        ds = np.ascontiguousarray(decode_expert_selection, dtype=np.int32)
        check(lib.moe_oracle_load(self._h, em.ctypes.data, em.shape[0], pl.ctypes.data, pl.shape[0],
                                  ps.ctypes.data, ps.shape[2] if ps.ndim == 3 else 0, ds.ctypes.data,
                                  ds.shape[2] if ds.ndim == 3 else 0), "load_oracle")

    def is_in_cache(self, layer_id: int, expert_id: int) -> bool:
        return lib.moe_is_in_cache(self._h, layer_id, expert_id) == 1

    def expert_status(self, layer_id: int, expert_id: int) -> str:
        return EXPERT_STATUS[lib.moe_expert_status(self._h, layer_id, expert_id)]

    def num_ready(self, layer_id: int, expert_id: int) -> int:
        return lib.moe_expert_num_ready(self._h, layer_id, expert_id)

    def slot_info(self, group: int = -1):
        n, b, s = C.c_int64(), C.c_int64(), C.c_int64()
        check(lib.moe_slot_info(self._h, group, C.byref(n), C.byref(b), C.byref(s)), "slot_info")
        return n.value, b.value, s.value

    def expert_ptr_table(self, layer_id: int) -> int:
        out = C.c_void_p()
        check(lib.moe_expert_ptr_table(self._h, layer_id, C.byref(out)), "expert_ptr_table")
        return out.value

    def flush_table(self, layer_id: int, stream: int = 0):
        check(lib.moe_flush_table(self._h, layer_id, stream), "flush_table")

    @property
    def compute_stream(self) -> int:
        a, b = C.c_void_p(), C.c_void_p()
        check(lib.moe_streams(self._h, C.byref(a), C.byref(b)), "streams")
        return a.value or 0

    @property
    def copy_stream(self) -> int:
        a, b = C.c_void_p(), C.c_void_p()
        check(lib.moe_streams(self._h, C.byref(a), C.byref(b)), "streams")
        return b.value or 0

    def counters(self) -> dict:
        c = L.Counters()
        check(lib.moe_get_counters(self._h, C.byref(c)), "counters")
        return c.as_dict()

    def report(self, skip_first_prompts: int = 0) -> dict:
        buf = C.create_string_buffer(8192)
        check(min(lib.moe_report(self._h, skip_first_prompts, buf, 8192), 0), "report")
        out = {}
        for line in buf.value.decode().splitlines():
            k, _, v = line.partition(":")
            out[k] = float(v)
        return out

    # -- fused forward --
    def set_layer(self, layer_id: int, H, I, I_sh, top_k, route_mode, gate_w, gate_bias=None, shared=None,
                  shared_gated=False, fmt: int = L.FMT_INT4_G128):
        d = L.LayerDesc(H, I, I_sh, top_k, route_mode, fmt, int(shared_gated), L.ptr(gate_w), L.ptr(gate_bias),
                        L.ptr(shared))
        self._keep.append((gate_w, gate_bias, shared))
        check(lib.moe_set_layer(self._h, layer_id, C.byref(d)), "set_layer")

    def forward_prepare(self, max_tokens: int):
        check(lib.moe_forward_prepare(self._h, max_tokens), "forward_prepare")

    def forward(self, layer_id: int, x: torch.Tensor, out: torch.Tensor | None = None,
                stream_guard: bool = True) -> torch.Tensor:
        """One MoE layer on the engine's compute stream.  Created from torch's legacy default stream (handle 0)
        the engine has a private non-blocking stream, as the reference has (prefetcher.cpp:407-413); callers are
        meant to make it torch's current stream (utils/__init__.py:293; `hf.inject_model` does).  When torch's
        current stream is another one, stream_guard orders the two around the call (x is complete before the
        kernels read it, the output before torch uses it); a caller that has synchronised itself passes False."""
        assert x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous()
        if out is None:
            out = torch.empty_like(x)
        guard = None
        if stream_guard and self.backend == L.BACKEND_HIP:
            cur = torch.cuda.current_stream(x.device)
            cs = self._compute_stream_handle
            if cs is None:
                cs = self._compute_stream_handle = self.compute_stream
            if cur.cuda_stream != cs:
                if self._ext_stream is None:
                    self._ext_stream = torch.cuda.ExternalStream(cs, device=x.device)
                guard = (cur, self._ext_stream)
                guard[1].wait_stream(cur)
        check(lib.moe_forward(self._h, layer_id, x.data_ptr(), x.shape[0], out.data_ptr()), "moe_forward")
        if guard is not None:
            guard[0].wait_stream(guard[1])
        return out

    def last_routing(self):
        a, b, c = C.c_void_p(), C.c_void_p(), C.c_void_p()
        check(lib.moe_last_routing(self._h, C.byref(a), C.byref(b), C.byref(c)), "last_routing")
        return a.value, b.value, c.value


    def last_routing_idx(self, T: int, k: int) -> np.ndarray:
        """Expert indices [T, k] of the last forward, copied back after the stream has drained (a checking aid)."""
        out = np.empty((T, k), np.int32)
        check(lib.moe_last_routing_host(self._h, T, k, out.ctypes.data, None), "last_routing_idx")
        return out


def slot_distribution(num_buffers: int, n_groups: int) -> list[int]:
    out = (C.c_int64 * n_groups)()
    check(lib.moe_slot_distribution(num_buffers, n_groups, out), "slot_distribution")
    return list(out)
