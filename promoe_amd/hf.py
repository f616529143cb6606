"""Model surgery: put the expert cache and the fused MoE layer under a Hugging Face model.

The reference's `inject_model` (reference: src/sparse_llm_cache/utils/__init__.py:147-338) walks a
loaded model, registers every expert's parameters with the loader, moves everything that is not an
expert to the GPU, replaces the experts' storage by slot-backed tensors, and hooks the MoE blocks so
that `report_experts`, the per-expert hooks and the layer hooks run around the model's own expert
loop.  Here the same walk ends in ONE call per MoE block: the block's forward becomes
`moe_forward` (gate, routing, cache hooks, experts, combine and shared expert inside the engine),
and the experts' weights live in pinned host memory as slot images instead of module parameters.

Works on the stock `transformers` sparse blocks that keep their experts in fused tensors
(`experts.gate_up_proj [E, 2I, H]`, `experts.down_proj [E, H, I]`, `gate.weight [E, H]`):
Qwen2-MoE (softmax -> top-k, optional renormalisation, sigmoid-gated shared expert), Mixtral
(softmax -> top-k -> renormalise, which is the softmax over the selected logits) and the DeepSeek
family (DeepSeek-MoE / DeepSeek-V2-Lite: softmax -> greedy top-k without renormalisation, a plain
shared expert `shared_experts` of n_shared_experts * I columns; the reference's metas for it are
utils/common_metas.py:17-41 and 69-94).  In the DeepSeek models the first decoder layers are dense:
MoE layers are numbered from 0 in model order, so decoder layer i is engine layer
i - first_k_dense_replace (the reference subtracts the same 1, common_metas.py:19-23).
"""
from __future__ import annotations

import types

import numpy as np
import torch

from . import _lib as L
from . import layout as LY
from . import quant
from .engine import ModuleMeta, PrefetchMngr, PinnedBuffer


def find_moe_blocks(model):
    """[(qualified name, module)] of the sparse MoE blocks, in model order."""
    out = []
    for name, mod in model.named_modules():
        ex = getattr(mod, "experts", None)
        gate = getattr(mod, "gate", None)
        if ex is not None and gate is not None and hasattr(ex, "gate_up_proj") and hasattr(ex, "down_proj") \
                and hasattr(gate, "weight"):
            out.append((name, mod))
    return out


def _route_mode(block) -> int:
    gate = block.gate
    if hasattr(gate, "topk_method"):                         # DeepSeek router
        if gate.topk_method != "greedy":
            raise NotImplementedError("DeepSeek routing method %r (only 'greedy' top-k is supported)" % gate.topk_method)
        return L.ROUTE_SOFTMAX_TOPK
    if hasattr(gate, "norm_topk_prob"):                      # Qwen2-MoE router
        return L.ROUTE_SOFTMAX_TOPK_RENORM if gate.norm_topk_prob else L.ROUTE_SOFTMAX_TOPK
    return L.ROUTE_TOPK_SOFTMAX                              # Mixtral: renormalised top-k of the softmax


def _shared_expert(block):
    """The block's always-on expert: Qwen2-MoE calls it shared_expert, the DeepSeek family shared_experts."""
    sh = getattr(block, "shared_expert", None)
    return sh if sh is not None else getattr(block, "shared_experts", None)


def _bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().to(torch.bfloat16).contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _expert_image(gate_w, up_w, down_w, H, I, fmt):
    """One SwiGLU expert (torch weights [I,H], [I,H], [H,I]) -> slot image."""
    if fmt == "bf16":
        return LY.pack_expert_bf16(_bf16_bits(gate_w), _bf16_bits(up_w), _bf16_bits(down_w))
    ex = [quant.quantize_int4(w.detach().float().cpu()) for w in (gate_w, up_w, down_w)]
    return LY.pack_expert_int4(ex[0], ex[1], ex[2], H, I)


def inject_model(model, device="cuda:0", fmt: str = "bf16", max_tokens: int = 4096, drop_expert_params: bool = True,
                 **cfg) -> PrefetchMngr:
    """Move the model's dense parts to `device` in bf16, keep its experts in pinned host memory behind the
    slot cache, and route every sparse block through the engine.  Returns the engine (also kept as
    `model._prefetch_mngr`, the attribute the reference attaches, utils/__init__.py:66-70).
    On return torch's current stream is the engine's compute stream: run the model on it.

    fmt "bf16" keeps the experts' weights as they are (rounded to bf16); "int4" quantises them to
    int4-g128 on the way in.  cfg: engine configuration keys (cache_rate, cache_policy, ...).
    The shapes must fit the kernels: H and I multiples of 128 (bf16) / 128 and 16 (int4)."""
    if fmt not in ("bf16", "int4"):
        raise ValueError("fmt must be 'bf16' or 'int4'")
    blocks = find_moe_blocks(model)
    if not blocks:
        raise ValueError("the model has no sparse MoE block with fused expert tensors")
    b0 = blocks[0][1]
    E, two_i, H = b0.experts.gate_up_proj.shape
    I = two_i // 2
    top_k = int(getattr(b0.gate, "top_k", getattr(b0, "top_k", 0)))
    sh0 = _shared_expert(b0)
    I_sh = sh0.gate_proj.weight.shape[0] if sh0 is not None else 0
    total = LY.bf16_expert_bytes(H, I) if fmt == "bf16" else LY.int4_layout(H, I)["total_bytes"]
    chunks = [("w", 0, total)] if fmt == "bf16" else LY.split_chunks_int4(H, I)

    m = ModuleMeta(len(blocks), E)
    m.init_param_list([c[0] for c in chunks])
    d = {"num_expert_per_token": str(top_k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    # images first (from the weights as loaded), then the dense parts go to the device
    stage = PinnedBuffer(total * len(blocks) * E)
    shared_imgs = []
    for l, (name, blk) in enumerate(blocks):
        gu, dn = blk.experts.gate_up_proj, blk.experts.down_proj
        if tuple(gu.shape) != (E, 2 * I, H) or tuple(dn.shape) != (E, H, I):
            raise ValueError("block %s differs in shape from the first block" % name)
        # DeepSeek scales the routed experts' sum by a constant; it goes into their down projections (multiplied in
        # fp32, before the one rounding to bf16 / the quantisation of the image)
        scale = float(getattr(blk.gate, "routed_scaling_factor", 1.0) or 1.0)
        for e in range(E):
            img = _expert_image(gu[e, :I], gu[e, I:], dn[e] if scale == 1.0 else dn[e].detach().float() * scale, H, I, fmt)
            base = (l * E + e) * total
            stage.array[base: base + total] = img
        sh = _shared_expert(blk)
        shared_imgs.append(None if sh is None else
                           _expert_image(sh.gate_proj.weight, sh.up_proj.weight, sh.down_proj.weight, H, I_sh, fmt))
        if drop_expert_params:      # the experts no longer live in the module (nor, later, on the device)
            blk.experts.gate_up_proj = torch.nn.Parameter(torch.empty(0), requires_grad=False)
            blk.experts.down_proj = torch.nn.Parameter(torch.empty(0), requires_grad=False)
            if sh is not None:
                for lin in (sh.gate_proj, sh.up_proj, sh.down_proj):
                    lin.weight = torch.nn.Parameter(torch.empty(0), requires_grad=False)
    model.to(device=device, dtype=torch.bfloat16)
    torch.cuda.set_device(device)
    # a stream of torch's own is handed over as it is; from the legacy default stream (handle 0) the
    # engine makes a private compute stream, and torch is switched onto it, as the reference does
    # (utils/__init__.py:293: torch's current stream := the engine's compute stream)
    pm = PrefetchMngr(m, backend=L.BACKEND_HIP, compute_stream=torch.cuda.current_stream().cuda_stream)
    pm._keep.append(stage)
    if pm.compute_stream != torch.cuda.current_stream().cuda_stream:
        prev = torch.cuda.current_stream()
        torch.cuda.synchronize()
        torch.cuda.set_stream(torch.cuda.ExternalStream(pm.compute_stream, device=device))
        engine_close = pm.close

        def close():  # the stream dies with the engine: give torch its own stream back first
            torch.cuda.synchronize()
            torch.cuda.set_stream(prev)
            engine_close()
        pm.close = close
    for l in range(len(blocks)):
        for e in range(E):
            base = (l * E + e) * total
            for cname, off, n in chunks:
                pm.add_one_expert_param(stage.array[base + off: base + off + n], l, e, cname)
    pm.init_gpu_mem_buffer()
    for l, (name, blk) in enumerate(blocks):
        gw = blk.gate.weight.detach().to(torch.bfloat16)
        sg = getattr(blk, "shared_expert_gate", None)
        if sg is not None:
            gw = torch.cat([gw, sg.weight.detach().to(torch.bfloat16).reshape(1, H)])
        sh = None if shared_imgs[l] is None else torch.from_numpy(np.ascontiguousarray(shared_imgs[l])).to(device)
        pm.set_layer(l, H, I, I_sh, top_k, _route_mode(blk), gw.contiguous(), None, sh, shared_gated=sg is not None,
                     fmt=L.FMT_BF16 if fmt == "bf16" else L.FMT_INT4_G128)
    pm.forward_prepare(max_tokens)
    pm.launch_thread()

    def make_forward(layer_id):
        def forward(self, hidden_states):
            shape = hidden_states.shape
            x = hidden_states.reshape(-1, shape[-1]).to(torch.bfloat16).contiguous()
            if x.shape[0] > max_tokens:
                raise ValueError("%d tokens in one forward, the engine was prepared for %d" % (x.shape[0], max_tokens))
            y = pm.forward(layer_id, x)
            return y.reshape(shape).to(hidden_states.dtype)
        return forward

    for l, (name, blk) in enumerate(blocks):
        blk._layer_id = l                                   # the reference's metadata attribute (utils/__init__.py:25-31)
        blk.forward = types.MethodType(make_forward(l), blk)
    model._prefetch_mngr = pm
    return pm
