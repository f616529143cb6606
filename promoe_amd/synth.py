"""Synthetic int4 MoE layer stacks of the benchmark shapes (random-init, seeded).

Weights are drawn directly in the slot layout: uniform nibbles, fp16 scales around
0.007 (what min/max quantisation of N(0,0.02) weights in groups of 128 gives) and
uniform zero points.  Activations ~N(0,1) bf16; gate weights ~N(0,0.02) bf16 with an
optional per-expert logit bias b_e = -s*ln(rank_e) (seeded rank permutation) that
makes expert popularity follow roughly Zipf(s).
"""
from __future__ import annotations

import numpy as np
import torch

from . import layout as LY
from . import _lib as L
from .engine import ModuleMeta, PrefetchMngr, PinnedBuffer


def random_int4_images(n: int, H: int, I: int, device, gen: torch.Generator) -> torch.Tensor:
    """n expert images [n, total_bytes] uint8 on `device`."""
    lay = LY.int4_layout(H, I)
    buf = torch.randint(0, 256, (n, lay["total_bytes"]), dtype=torch.uint8, device=device, generator=gen)
    for off_s, rows, G in ((lay["off13_s"], 2 * I, H // 128), (lay["off2_s"], H, I // 128)):
        ns = rows * G
        sc = (torch.rand(n, ns, device=device, generator=gen) * 0.004 + 0.005).to(torch.float16)
        buf[:, off_s: off_s + ns * 2] = sc.view(torch.uint8)
    return buf


def random_q4k_images(n: int, H: int, I: int, device, gen: torch.Generator) -> torch.Tensor:
    """n q4_K expert images [n, total_bytes] uint8: uniform nibbles, 6-bit scales and mins, fp16 d and
    dmin around 1e-4 (weights of a few 1e-2 in magnitude)."""
    lay = LY.q4k_layout(H, I)
    buf = torch.randint(0, 256, (n, lay["total_bytes"]), dtype=torch.uint8, device=device, generator=gen)
    for s0, z0, end in ((lay["off13_s"], lay["off13_z"], lay["off2_q"]), (lay["off2_s"], lay["off2_z"], lay["total_bytes"])):
        buf[:, s0:z0] &= 63
        nd = (end - z0) // 2
        d = (torch.rand(n, nd, device=device, generator=gen) * 1e-4 + 5e-5).to(torch.float16)
        buf[:, z0:end] = d.view(torch.uint8)
    return buf


def zipf_bias(E: int, s: float, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    rank = rng.permutation(E) + 1
    return (-s * np.log(rank.astype(np.float64))).astype(np.float32)


class Int4Stack:
    """L MoE layers of E int4 experts: images in pinned host memory, dense parts on the GPU."""

    def __init__(self, L_: int, E: int, H: int, I: int, I_sh: int, top_k: int, device, zipf: float | None = 1.2,
                 seed: int = 0, route_mode: int = L.ROUTE_SOFTMAX_TOPK):
        self.L, self.E, self.H, self.I, self.I_sh, self.k, self.mode = L_, E, H, I, I_sh, top_k, route_mode
        self.device = device
        gen = torch.Generator(device=device).manual_seed(seed)
        self.expert_bytes = LY.int4_layout(H, I)["total_bytes"]
        self.chunks = LY.split_chunks_int4(H, I)
        self.stage = PinnedBuffer(self.expert_bytes * L_ * E)
        host = torch.from_numpy(self.stage.array).view(L_, E, self.expert_bytes)
        self.gate_w, self.gate_bias, self.shared = [], [], []
        for l in range(L_):
            imgs = random_int4_images(E, H, I, device, gen)
            host[l].copy_(imgs)
            del imgs
            self.gate_w.append((torch.randn(E, H, device=device, generator=gen) * 0.02).to(torch.bfloat16))
            self.gate_bias.append(None if zipf is None else torch.from_numpy(zipf_bias(E, zipf, seed * 1000 + 2 + l)).to(device))
            self.shared.append(random_int4_images(1, H, I_sh, device, gen)[0] if I_sh else None)
        torch.cuda.synchronize()

    def engine(self, max_tokens: int, **cfg) -> PrefetchMngr:
        m = ModuleMeta(self.L, self.E)
        m.init_param_list([c[0] for c in self.chunks])
        d = {"num_expert_per_token": str(self.k)}
        d.update({a: str(b) for a, b in cfg.items()})
        m.init_from_map(d)
        m.handle_uninited_configs()
        pm = PrefetchMngr(m, backend=L.BACKEND_HIP, compute_stream=torch.cuda.current_stream().cuda_stream)
        pm._keep.append(self)
        for l in range(self.L):
            for e in range(self.E):
                base = (l * self.E + e) * self.expert_bytes
                for name, off, n in self.chunks:
                    pm.add_one_expert_param(self.stage.array[base + off: base + off + n], l, e, name)
        pm.init_gpu_mem_buffer()
        for l in range(self.L):
            pm.set_layer(l, self.H, self.I, self.I_sh, self.k, self.mode, self.gate_w[l], self.gate_bias[l],
                         self.shared[l])
        pm.forward_prepare(max_tokens)
        pm.launch_thread()
        return pm

    def acts(self, T: int, n: int, seed: int = 1):
        gen = torch.Generator(device=self.device).manual_seed(seed)
        return [torch.randn(T, self.H, device=self.device, generator=gen).to(torch.bfloat16) for _ in range(n)]
