"""On-disk expert weights -> slot images of the engine.

Two readers, both host side (numpy):

* GPTQ checkpoints in safetensors files.  The reference registers the `qweight`, `*zero*` and
  `*scale*` buffers of every module matching `layers.<l>.mlp.experts.<e>`
  (reference: src/sparse_llm_cache/utils/__init__.py:39-60) and leaves the arithmetic to the
  AutoGPTQ/exllama kernels; here the same tensors are repacked once into the int4-g128 slot layout.
  AutoGPTQ stores, per linear layer with K inputs and N outputs,
      qweight int32 [K/8, N]   nibble j of row r = q[8r + j, n]
      qzeros  int32 [K/g, N/8] nibble j of column c = zero[g, 8c + j]  (format "gptq": zero - 1 is stored)
      scales  fp16  [K/g, N]
      g_idx   int32 [K]        group of input k (must be k // g: no activation reordering)
  and w[k, n] = (q[k, n] - zero[g, n]) * scales[g, n].

* GGUF files with q4_K expert tensors (llama.cpp naming: `blk.<l>.ffn_{gate,up,down}_exps.weight`
  holding all experts of a layer, `ffn_gate_inp.weight` the router, `*_shexp` the shared expert;
  reference: README.md:29-34 names q4_k_m files as its llama.cpp input).  The 144-byte blocks are
  taken as they are and re-tiled by layout.pack_expert_q4k.
"""
from __future__ import annotations

import re
import struct

import numpy as np

from . import layout as LY

GROUP = LY.GROUP

# ---------------------------------------------------------------------------------------------
# GPTQ
# ---------------------------------------------------------------------------------------------

_SHIFTS = (np.arange(8, dtype=np.uint32) * 4)


def _unpack_rows(packed: np.ndarray) -> np.ndarray:
    """int32 [R, C] -> uint8 [8R, C]: nibble j of row r becomes row 8r + j."""
    p = np.ascontiguousarray(packed).view(np.uint32)
    out = (p[:, None, :] >> _SHIFTS[None, :, None]) & 0xF
    return out.reshape(p.shape[0] * 8, p.shape[1]).astype(np.uint8)


def _unpack_cols(packed: np.ndarray) -> np.ndarray:
    """int32 [R, C] -> uint8 [R, 8C]: nibble j of column c becomes column 8c + j."""
    p = np.ascontiguousarray(packed).view(np.uint32)
    out = (p[:, :, None] >> _SHIFTS[None, None, :]) & 0xF
    return out.reshape(p.shape[0], p.shape[1] * 8).astype(np.uint8)


def gptq_to_exchange(qweight, qzeros, scales, g_idx=None, zero_plus_one: bool = True):
    """One GPTQ linear layer -> the exchange triple layout.pack_expert_int4 takes:
    (qweight int32 [N, K/8] nibbles along K, scales fp16 [N, G], qzeros int32 flat over [N, G]).

    zero_plus_one: checkpoint format "gptq" (AutoGPTQ v1) stores zero - 1 in 4 bits and its kernels
    add the one back modulo 16; format "gptq_v2" stores the zero itself (pass False)."""
    qweight = np.asarray(qweight)
    qzeros = np.asarray(qzeros)
    scales = np.asarray(scales)
    if qweight.dtype != np.int32 or qzeros.dtype != np.int32 or qweight.ndim != 2 or qzeros.ndim != 2:
        raise ValueError("GPTQ qweight/qzeros must be 2-D int32 tensors")
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    G = qzeros.shape[0]
    if K % GROUP or K // GROUP != G:
        raise ValueError("only group size %d is supported (K=%d, %d groups)" % (GROUP, K, G))
    if qzeros.shape[1] * 8 != N or scales.shape != (G, N):
        raise ValueError("GPTQ tensor shapes disagree: qweight %s qzeros %s scales %s"
                         % (qweight.shape, qzeros.shape, scales.shape))
    if g_idx is not None:
        gi = np.asarray(g_idx).reshape(-1)
        if gi.size != K or not np.array_equal(gi, np.arange(K) // GROUP):
            raise ValueError("activation-ordered checkpoints (desc_act: g_idx is not k // %d) are not supported" % GROUP)
    q = _unpack_rows(qweight)                      # [K, N]
    z = _unpack_cols(qzeros)                       # [G, N]
    if zero_plus_one:
        z = (z + 1) & 0xF
    qt = np.ascontiguousarray(q.T).astype(np.uint32).reshape(N, K // 8, 8)
    qx = np.zeros((N, K // 8), np.uint32)
    for j in range(8):
        qx |= qt[:, :, j] << np.uint32(4 * j)
    zt = np.ascontiguousarray(z.T).astype(np.uint32).reshape(-1)          # [N, G] flat
    pad = (-zt.size) % 8
    zt = np.concatenate([zt, np.zeros(pad, np.uint32)]).reshape(-1, 8)
    zx = np.zeros(zt.shape[0], np.uint32)
    for j in range(8):
        zx |= zt[:, j] << np.uint32(4 * j)
    sx = np.ascontiguousarray(scales.astype(np.float16).T)                 # [N, G]
    return qx.view(np.int32), sx, zx.view(np.int32)


class SafetensorsIndex:
    """Tensor name -> file over one or more safetensors shards (read lazily, numpy framework)."""

    def __init__(self, paths):
        from safetensors import safe_open
        if isinstance(paths, (str, bytes)):
            paths = [paths]
        self._open = safe_open
        self.file_of = {}
        for p in paths:
            with safe_open(p, framework="np") as f:
                for k in f.keys():
                    self.file_of[k] = p

    def __contains__(self, name):
        return name in self.file_of

    def get(self, name) -> np.ndarray:
        if name not in self.file_of:
            raise KeyError("tensor %r is in none of the files" % name)
        with self._open(self.file_of[name], framework="np") as f:
            return f.get_tensor(name)

    def names(self):
        return list(self.file_of)


# projection names per model family, in (gate, up, down) order
# (reference: utils/common_metas.py:17-186 parses the same module paths for layer and expert ids)
PROJ_NAMES = {"deepseek": ("gate_proj", "up_proj", "down_proj"),
              "qwen": ("gate_proj", "up_proj", "down_proj"),
              "mixtral": ("w1", "w3", "w2")}
EXPERT_PREFIX = {"deepseek": "model.layers.{l}.mlp.experts.{e}",
                 "qwen": "model.layers.{l}.mlp.experts.{e}",
                 "mixtral": "model.layers.{l}.block_sparse_moe.experts.{e}"}
SHARED_PREFIX = {"deepseek": "model.layers.{l}.mlp.shared_experts",
                 "qwen": "model.layers.{l}.mlp.shared_expert"}
# checkpoint layer index of MoE layer 0 (DeepSeek-MoE's first decoder layer is dense: the reference
# numbers its MoE layers from checkpoint layer 1, utils/common_metas.py:19-23)
FIRST_MOE_LAYER = {"deepseek": 1, "qwen": 0, "mixtral": 0}


def gptq_module_image(index: SafetensorsIndex, prefix: str, H: int, proj=("gate_proj", "up_proj", "down_proj"),
                      zero_plus_one: bool = True) -> np.ndarray:
    """Slot image (uint8) of one SwiGLU module stored as three GPTQ linears under `prefix`."""
    ex = []
    I = None
    for i, name in enumerate(proj):
        base = "%s.%s." % (prefix, name)
        gi = index.get(base + "g_idx") if (base + "g_idx") in index else None
        t = gptq_to_exchange(index.get(base + "qweight"), index.get(base + "qzeros"), index.get(base + "scales"),
                             gi, zero_plus_one)
        N, K = t[0].shape[0], t[0].shape[1] * 8
        if i < 2:
            if K != H:
                raise ValueError("%sqweight has %d inputs, the layer has H=%d" % (base, K, H))
            I = N if I is None else I
            if N != I:
                raise ValueError("gate and up projections of %s differ in size" % prefix)
        elif (N, K) != (H, I):
            raise ValueError("%sqweight is %dx%d, expected %dx%d" % (base, N, K, H, I))
        ex.append(t)
    return LY.pack_expert_int4(ex[0], ex[1], ex[2], H, I)


def gptq_layer_images(index: SafetensorsIndex, layer: int, num_expert: int, H: int, family: str = "deepseek",
                      zero_plus_one: bool = True):
    """(list of routed expert images, shared expert image or None) of MoE layer `layer` (counted as
    the engine counts them, from 0)."""
    proj = PROJ_NAMES[family]
    layer = layer + FIRST_MOE_LAYER[family]
    routed = [gptq_module_image(index, EXPERT_PREFIX[family].format(l=layer, e=e), H, proj, zero_plus_one)
              for e in range(num_expert)]
    shared = None
    sp = SHARED_PREFIX.get(family)
    if sp and (sp.format(l=layer) + "." + proj[0] + ".qweight") in index:
        shared = gptq_module_image(index, sp.format(l=layer), H, proj, zero_plus_one)
    return routed, shared


# ---------------------------------------------------------------------------------------------
# GGUF
# ---------------------------------------------------------------------------------------------

GGML_F32, GGML_F16, GGML_Q4_K, GGML_Q6_K, GGML_BF16 = 0, 1, 12, 14, 30
# (elements per block, bytes per block) of the types this reader can size
_GGML_BLOCK = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34),
               10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
               30: (1, 2)}
_GGML_NAME = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 10: "Q2_K", 11: "Q3_K",
              12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 30: "BF16"}
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}


class GGUFFile:
    """Minimal GGUF (version 2 and 3, little endian) reader: metadata and tensor directory are
    parsed, tensor data is memory-mapped."""

    def __init__(self, path: str):
        self.path = path
        self._mm = np.memmap(path, dtype=np.uint8, mode="r")
        self._pos = 0
        if self._mm.size < 24 or bytes(self._mm[0:4]) != b"GGUF":
            raise ValueError("%s is not a GGUF file" % path)
        self._pos = 4
        self.version = self._rd("<I")
        if self.version not in (2, 3):
            raise ValueError("GGUF version %d is not supported" % self.version)
        n_tensors, n_kv = self._rd("<Q"), self._rd("<Q")
        self.metadata = {}
        for _ in range(n_kv):
            key = self._rd_str()
            self.metadata[key] = self._rd_value(self._rd("<I"))
        self.tensors = {}
        for _ in range(n_tensors):
            name = self._rd_str()
            nd = self._rd("<I")
            ne = [self._rd("<Q") for _ in range(nd)]       # ne[0] is the contiguous dimension
            typ, off = self._rd("<I"), self._rd("<Q")
            self.tensors[name] = (tuple(ne), typ, off)
        align = int(self.metadata.get("general.alignment", 32))
        self.data_start = (self._pos + align - 1) // align * align

    def _rd(self, fmt):
        n = struct.calcsize(fmt)
        if self._pos + n > self._mm.size:
            raise ValueError("truncated GGUF file")
        v = struct.unpack(fmt, bytes(self._mm[self._pos:self._pos + n]))[0]
        self._pos += n
        return v

    def _rd_str(self):
        n = self._rd("<Q")
        if self._pos + n > self._mm.size:
            raise ValueError("truncated GGUF file")
        s = bytes(self._mm[self._pos:self._pos + n]).decode("utf-8", "replace")
        self._pos += n
        return s

    def _rd_value(self, t):
        if t in _SCALAR:
            return self._rd(_SCALAR[t])
        if t == 8:
            return self._rd_str()
        if t == 9:
            et, n = self._rd("<I"), self._rd("<Q")
            return [self._rd_value(et) for _ in range(n)]
        raise ValueError("unknown GGUF metadata type %d" % t)

    def nbytes(self, name) -> int:
        ne, typ, _ = self.tensors[name]
        if typ not in _GGML_BLOCK:
            raise NotImplementedError("ggml type %d of %s" % (typ, name))
        per, size = _GGML_BLOCK[typ]
        n = int(np.prod(ne))
        if ne[0] % per:
            raise ValueError("%s: row length %d is not a multiple of the block size %d" % (name, ne[0], per))
        return n // per * size

    def raw(self, name) -> np.ndarray:
        if name not in self.tensors:
            raise KeyError("no tensor %r in %s" % (name, self.path))
        _, _, off = self.tensors[name]
        a = self.data_start + off
        b = a + self.nbytes(name)
        if b > self._mm.size:
            raise ValueError("%s reaches past the end of the file" % name)
        return self._mm[a:b]

    def q4k_blocks(self, name) -> np.ndarray:
        """uint8 view [..., ne1, ne0/256, 144] (outermost dimension first) of a Q4_K tensor."""
        ne, typ, _ = self.tensors[name]
        if typ != GGML_Q4_K:
            raise NotImplementedError("%s is stored as %s; only Q4_K expert tensors are supported"
                                      % (name, _GGML_NAME.get(typ, str(typ))))
        if ne[0] % 256:
            raise ValueError("%s: row length %d is not a multiple of 256" % (name, ne[0]))
        shape = tuple(reversed(ne[1:])) + (ne[0] // 256, 144)
        return self.raw(name).reshape(shape)

    def q6k_blocks(self, name) -> np.ndarray:
        """uint8 view [..., ne1, ne0/256, 210] (outermost dimension first) of a Q6_K tensor."""
        ne, typ, _ = self.tensors[name]
        if typ != GGML_Q6_K:
            raise NotImplementedError("%s is stored as %s, not Q6_K" % (name, _GGML_NAME.get(typ, str(typ))))
        if ne[0] % 256:
            raise ValueError("%s: row length %d is not a multiple of 256" % (name, ne[0]))
        shape = tuple(reversed(ne[1:])) + (ne[0] // 256, 210)
        return self.raw(name).reshape(shape)

    def expert_q4k_blocks(self, name) -> np.ndarray:
        """An expert tensor as q4_K blocks [..., rows, cols/256, 144].  Q4_K tensors are handed out as they
        are.  Q6_K tensors (the ffn_down tensors of a q4_k_m file) are dequantised and quantised again to
        q4_K, the one block format the expert kernels read: a lossy step (a weight moves by at most half a
        q4_K step of its 32-wide sub-block), so the result is not what llama.cpp computes from the file."""
        typ = self.tensors[name][1]
        if typ == GGML_Q4_K:
            return self.q4k_blocks(name)
        if typ == GGML_Q6_K:
            from .quant import dequant_q6k, quantize_q4k
            b6 = self.q6k_blocks(name)
            w = dequant_q6k(b6)                               # [..., rows, cols]
            lead = w.shape[:-2]
            q = quantize_q4k(w.reshape(-1, w.shape[-1]))
            return q.reshape(lead + (w.shape[-2], w.shape[-1] // 256, 144))
        raise NotImplementedError("%s is stored as %s; expert tensors must be Q4_K or Q6_K"
                                  % (name, _GGML_NAME.get(typ, str(typ))))

    def dense(self, name) -> np.ndarray:
        """fp32 array (outermost dimension first) of an F32 / F16 / BF16 tensor."""
        ne, typ, _ = self.tensors[name]
        shape = tuple(reversed(ne))
        r = self.raw(name)
        if typ == GGML_F32:
            return np.array(r.view(np.float32).reshape(shape))
        if typ == GGML_F16:
            return r.view(np.float16).reshape(shape).astype(np.float32)
        if typ == GGML_BF16:
            return (r.view(np.uint16).astype(np.uint32) << 16).view(np.float32).reshape(shape)
        raise NotImplementedError("%s is stored as %s" % (name, _GGML_NAME.get(typ, str(typ))))

    def moe_layers(self):
        """Indices of the blocks that hold merged expert tensors."""
        pat = re.compile(r"blk\.(\d+)\.ffn_gate_exps\.weight$")
        return sorted(int(m.group(1)) for m in (pat.match(n) for n in self.tensors) if m)


def gguf_layer_images(g: GGUFFile, layer: int):
    """One MoE layer of a GGUF file -> dict with
    routed: list of q4_K slot images, shared: image or None, gate_w: fp32 [E, H],
    shared_gate: fp32 [H] or None, H, I, I_sh, E."""
    p = "blk.%d." % layer
    gate = g.q4k_blocks(p + "ffn_gate_exps.weight")      # [E, I, H/256, 144]
    up = g.q4k_blocks(p + "ffn_up_exps.weight")
    down = g.expert_q4k_blocks(p + "ffn_down_exps.weight")   # [E, H, I/256, 144]; Q6_K in a q4_k_m file
    E, I, H = gate.shape[0], gate.shape[1], gate.shape[2] * 256
    if up.shape != gate.shape or down.shape != (E, H, I // 256, 144):
        raise ValueError("expert tensors of block %d disagree in shape" % layer)
    routed = [LY.pack_expert_q4k(gate[e], up[e], down[e], H, I) for e in range(E)]
    out = {"routed": routed, "shared": None, "shared_gate": None, "H": H, "I": I, "I_sh": 0, "E": E,
           "gate_w": g.dense(p + "ffn_gate_inp.weight")}
    if (p + "ffn_gate_shexp.weight") in g.tensors:
        sg = g.q4k_blocks(p + "ffn_gate_shexp.weight")   # [I_sh, H/256, 144]
        su = g.q4k_blocks(p + "ffn_up_shexp.weight")
        sd = g.expert_q4k_blocks(p + "ffn_down_shexp.weight")
        out["I_sh"] = sg.shape[0]
        out["shared"] = LY.pack_expert_q4k(sg, su, sd, H, sg.shape[0])
        if (p + "ffn_gate_inp_shexp.weight") in g.tensors:
            out["shared_gate"] = g.dense(p + "ffn_gate_inp_shexp.weight").reshape(-1)
    return out


# ---------------------------------------------------------------------------------------------
# images -> a running engine
# ---------------------------------------------------------------------------------------------

def engine_from_images(layers, fmt: str, top_k: int, route_mode: int, device, max_tokens: int = 64, **cfg):
    """Register the expert images of a stack of MoE layers (pinned host memory), describe the
    layers and start the engine: what `inject_model` does with a loaded checkpoint in the reference
    (utils/__init__.py:147-338: register expert params, pin, init the slot buffers, attach, launch).

    layers: one dict per MoE layer with `routed` (list of uint8 images), `shared` (image or None),
    `gate_w` fp32 [E, H], optional `gate_bias` fp32 [E], optional `shared_gate` fp32 [H], and H, I, I_sh.
    fmt: "int4" or "q4k".  cfg: engine configuration keys (cache_rate, cache_policy, ...)."""
    import torch
    from . import _lib as L
    from .engine import ModuleMeta, PrefetchMngr, PinnedBuffer
    if fmt not in ("int4", "q4k"):
        raise ValueError("fmt must be 'int4' or 'q4k'")
    n_layer, E = len(layers), len(layers[0]["routed"])
    H, I, I_sh = layers[0]["H"], layers[0]["I"], layers[0]["I_sh"]
    total = (LY.q4k_layout(H, I) if fmt == "q4k" else LY.int4_layout(H, I))["total_bytes"]
    chunks = [("w", 0, total)] if fmt == "q4k" else LY.split_chunks_int4(H, I)
    m = ModuleMeta(n_layer, E)
    m.init_param_list([c[0] for c in chunks])
    d = {"num_expert_per_token": str(top_k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    pm = PrefetchMngr(m, backend=L.BACKEND_HIP, compute_stream=torch.cuda.current_stream().cuda_stream)
    stage = PinnedBuffer(total * n_layer * E)
    pm._keep.append(stage)
    for l, lay in enumerate(layers):
        if (lay["H"], lay["I"], lay["I_sh"], len(lay["routed"])) != (H, I, I_sh, E):
            raise ValueError("layer %d differs in shape from layer 0" % l)
        for e, img in enumerate(lay["routed"]):
            if img.size != total:
                raise ValueError("image of expert %d of layer %d has %d bytes, expected %d" % (e, l, img.size, total))
            base = (l * E + e) * total
            stage.array[base: base + total] = img
            for name, off, n in chunks:
                pm.add_one_expert_param(stage.array[base + off: base + off + n], l, e, name)
    pm.init_gpu_mem_buffer()
    for l, lay in enumerate(layers):
        gw = torch.from_numpy(np.ascontiguousarray(lay["gate_w"], np.float32)).to(torch.bfloat16).to(device)
        gated = lay.get("shared_gate") is not None
        if gated:
            sg = torch.from_numpy(np.ascontiguousarray(lay["shared_gate"], np.float32).reshape(1, H))
            gw = torch.cat([gw, sg.to(torch.bfloat16).to(device)])
        bias = lay.get("gate_bias")
        bias = None if bias is None else torch.from_numpy(np.ascontiguousarray(bias, np.float32)).to(device)
        sh = None if lay["shared"] is None else torch.from_numpy(np.ascontiguousarray(lay["shared"])).to(device)
        pm.set_layer(l, H, I, I_sh, top_k, route_mode, gw, bias, sh, shared_gated=gated,
                     fmt=L.FMT_Q4K if fmt == "q4k" else L.FMT_INT4_G128)
    pm.forward_prepare(max_tokens)
    pm.launch_thread()
    return pm
