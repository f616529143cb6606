"""Host-side mirror of the reference's patched MoE module and its hooks.

The reference patches a HuggingFace MoE block so that its forward calls
`self.report_experts(unique_ids)` after routing and then runs the experts in the returned
order (utils/__init__.py:82-96; stand-in module eval/demo-simulate/transformers-deepseek-moe.py:36-49),
with `ExpertHook` around every expert (utils/hooks.py:187-198) and `MoeLayerHook` around the
block (utils/hooks.py:200-223).  `SparseMoeBlock` is that block on top of the HIP kernels:

  fused=True   one `moe_forward` call of the C ABI (the hook sequence runs inside the library)
  fused=False  the reference's own structure: routing kernels, `report_experts`, then one
               kernel launch per expert between `ExpertHook.pre_forward` / `post_forward`,
               reading the expert's parameters through the engine's slot table.

torch is device memory and streams here; all arithmetic is in libmoe_engine.so.
"""
from __future__ import annotations

import numpy as np
import torch

from . import _lib as L
from . import ops
from .engine import PrefetchMngr


class ExpertHook:
    """utils/hooks.py:187-198: wait for the expert before its forward, release it after."""

    def __init__(self, prefetch_mngr: PrefetchMngr):
        self.prefetch_mngr = prefetch_mngr

    def pre_forward(self, module, *args, **kwargs):
        self.prefetch_mngr.report_one_expert(module._layer_id, module._expert_id)
        return args, kwargs

    def post_forward(self, module, output):
        self.prefetch_mngr.one_expert_done(module._layer_id, module._expert_id)
        return output


class MoeLayerHook:
    """utils/hooks.py:200-223: layer 0 reports its input, every layer reports its output as
    the next layer's input, then closes the layer."""

    def __init__(self, prefetch_mngr: PrefetchMngr):
        self.prefetch_mngr = prefetch_mngr

    def pre_forward(self, module, *args, **kwargs):
        if module._layer_id == 0:
            self.prefetch_mngr.report_moe_layer_logits(module._layer_id, args[0])
        return args, kwargs

    def post_forward(self, module, output):
        self.prefetch_mngr.report_moe_layer_logits(module._layer_id + 1, output)
        self.prefetch_mngr.one_moe_layer_done(module._layer_id)
        return output


class Expert:
    """One routed expert: identity only, its parameters live in the engine's slots."""

    def __init__(self, layer_id: int, expert_id: int):
        self._layer_id, self._expert_id = layer_id, expert_id


class _TableRow:
    def __init__(self, addr: int):
        self._addr = addr

    def data_ptr(self) -> int:
        return self._addr


class SparseMoeBlock:
    def __init__(self, prefetch_mngr: PrefetchMngr, layer_id: int, num_expert: int, H: int, I: int, I_sh: int,
                 top_k: int, route_mode: int, gate_w: torch.Tensor, gate_bias: torch.Tensor | None = None,
                 shared: torch.Tensor | None = None, shared_gated: bool = False, fmt: int = L.FMT_INT4_G128,
                 fused: bool = True):
        self._prefetch_mngr, self._layer_id = prefetch_mngr, layer_id
        self.E, self.H, self.I, self.I_sh, self.k, self.mode = num_expert, H, I, I_sh, top_k, route_mode
        self.gate_w, self.gate_bias, self.shared, self.shared_gated, self.fmt = gate_w, gate_bias, shared, shared_gated, fmt
        self.fused = fused
        self.experts = [Expert(layer_id, e) for e in range(num_expert)]
        self._expert_hook = ExpertHook(prefetch_mngr)
        self._layer_hook = MoeLayerHook(prefetch_mngr)
        prefetch_mngr.set_layer(layer_id, H, I, I_sh, top_k, route_mode, gate_w, gate_bias, shared,
                                shared_gated=shared_gated, fmt=fmt)

    # the method the reference installs on the module (utils/__init__.py:82-89)
    def report_experts(self, experts: torch.Tensor) -> torch.Tensor:
        self._prefetch_mngr.report_one_layer(self._layer_id, experts)
        return experts

    def _expert_forward(self, expert: Expert, x, d: ops.Dispatch, unit_row: torch.Tensor, ws, with_shared: bool):
        pm = self._prefetch_mngr
        table = _TableRow(pm.expert_ptr_table(self._layer_id))
        pm.flush_table(self._layer_id, torch.cuda.current_stream().cuda_stream)
        one = ops.Dispatch.__new__(ops.Dispatch)
        one.__dict__.update(d.__dict__)
        one.units, one.max_units = unit_row, unit_row.shape[0]
        sh = self.shared if with_shared else None
        if self.fmt == L.FMT_BF16 or x.shape[0] > ops.gemv_max_tokens(self.fmt):
            return ops.experts_prefill(x, one, table, sh, self.H, self.I, self.I_sh, self.fmt, ws=ws)
        return ops.experts_decode_int4(x, one, table, sh, self.H, self.I, self.I_sh,
                                       ws=None if ws is None else ws[:5]) + (None,)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.fused:
            return self._prefetch_mngr.forward(self._layer_id, x)
        self._layer_hook.pre_forward(self, x)
        T, E, k = x.shape[0], self.E, self.k
        if self.gate_bias is None:
            logits = ops.gate_logits(x, self.gate_w, None)
        else:   # the bias covers the routed experts; the shared-gate row (row E) has none
            logits = torch.empty(T, self.gate_w.shape[0], dtype=torch.float32, device=x.device)
            ops.gate_logits(x, self.gate_w[:E], self.gate_bias, out=logits[:, :E])
            if self.gate_w.shape[0] > E:
                ops.gate_logits(x, self.gate_w[E:], None, out=logits[:, E:])
        idx, w = ops.topk(logits, k, self.mode, E=E)
        d = ops.dispatch(idx, E)
        n_act = int(d.n_active.cpu()[0])
        units = d.units[:n_act].cpu()
        experts = units[:, 0].to(torch.int64).contiguous()      # the unique ids, ascending
        experts = self.report_experts(experts)                   # reordered in place by the engine
        row_of = {int(units[i, 0]): i for i in range(n_act)}
        ws = None
        first = True
        for e in experts.tolist():
            expert = self.experts[e]
            self._expert_hook.pre_forward(expert)
            unit_row = d.units[row_of[e]: row_of[e] + 1]
            ws = self._expert_forward(expert, x, d, unit_row, ws, with_shared=first and self.I_sh > 0)
            first = False
            self._expert_hook.post_forward(expert, None)
        assert ws is not None and int(ws[2].cpu()[0]) == 0, "an expert was not resident at launch"
        sg = logits[:, E] if self.shared_gated else None
        y = ops.combine(ws[0], ws[1], w, d.pos_of_pair, sg, T, self.H, k)
        return self._layer_hook.post_forward(self, y)

    __call__ = forward
