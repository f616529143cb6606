"""Seeded synthetic MoE layers for the tests (weights ~N(0,0.02), activations ~N(0,1))."""
from __future__ import annotations

import numpy as np
import torch

from oracle import moe_oracle as O
from promoe_amd import layout as LY


class Int4Layer:
    """One int4-g128 MoE layer: exchange-format weights, fp32 dequantised weights (oracle
    side) and packed slot images (product side)."""

    def __init__(self, H, I, E, I_sh=0, seed=0, shared_gate=False, zipf=None):
        self.H, self.I, self.E, self.I_sh = H, I, E, I_sh
        g = torch.Generator().manual_seed(seed)

        def mat(n, k):
            return (torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02).numpy()

        self.wg = O.round_bf16(mat(E, H))
        self.bias = O.zipf_gate_bias(E, zipf, seed=2) if zipf else None
        self.experts_fp32, self.slots = [], []
        for _ in range(E):
            deq, img = self._make_expert(mat(I, H), mat(I, H), mat(H, I), H, I)
            self.experts_fp32.append(deq)
            self.slots.append(img)
        self.shared_fp32 = self.shared_img = None
        if I_sh:
            self.shared_fp32, self.shared_img = self._make_expert(mat(I_sh, H), mat(I_sh, H), mat(H, I_sh), H, I_sh)
        self.shared_gate = O.round_bf16(mat(1, H))[0] if shared_gate else None

    @staticmethod
    def _make_expert(wgate, wup, wdown, H, I):
        ex, deq = [], []
        for w, (n, k) in ((wgate, (I, H)), (wup, (I, H)), (wdown, (H, I))):
            q, s, z = O.quantize_int4(w)
            qw, qz = O.pack_int4(q, z)
            ex.append((qw, s, qz))
            deq.append(O.dequant_int4(qw, s, qz, n, k))
        return tuple(deq), LY.pack_expert_int4(ex[0], ex[1], ex[2], H, I)


class Bf16Layer:
    """One bf16 MoE layer: bf16-representable fp32 weights (oracle side) and expert images
    in the blocked bf16 slot layout (w13 = gate rows then up rows, then w2)."""

    def __init__(self, H, I, E, I_sh=0, seed=0, shared_gate=False, zipf=None):
        self.H, self.I, self.E, self.I_sh = H, I, E, I_sh
        g = torch.Generator().manual_seed(seed)

        def mat(n, k):
            return O.round_bf16((torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02).numpy())

        self.wg = mat(E, H)
        self.bias = O.zipf_gate_bias(E, zipf, seed=2) if zipf else None
        self.experts_fp32, self.slots = [], []
        for _ in range(E):
            ws = (mat(I, H), mat(I, H), mat(H, I))
            self.experts_fp32.append(ws)
            self.slots.append(self.image(ws))
        self.shared_fp32 = self.shared_img = None
        if I_sh:
            self.shared_fp32 = (mat(I_sh, H), mat(I_sh, H), mat(H, I_sh))
            self.shared_img = self.image(self.shared_fp32)
        self.shared_gate = mat(1, H)[0] if shared_gate else None

    @staticmethod
    def image(ws):
        return LY.pack_expert_bf16(*[O.f32_to_bf16_bits(w) for w in ws])



class Q4KLayer:
    """One q4_K MoE layer: ggml-format blocks quantised from N(0,0.02) weights, their fp32
    dequantisation (oracle side) and the repacked slot images (product side)."""

    def __init__(self, H, I, E, I_sh=0, seed=0, shared_gate=False, zipf=None):
        self.H, self.I, self.E, self.I_sh = H, I, E, I_sh
        g = torch.Generator().manual_seed(seed)

        def mat(n, k):
            return (torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02).numpy()

        self.wg = O.round_bf16(mat(E, H))
        self.bias = O.zipf_gate_bias(E, zipf, seed=2) if zipf else None
        self.experts_fp32, self.slots = [], []
        for _ in range(E):
            deq, img = self._make_expert(mat(I, H), mat(I, H), mat(H, I), H, I)
            self.experts_fp32.append(deq)
            self.slots.append(img)
        self.shared_fp32 = self.shared_img = None
        if I_sh:
            self.shared_fp32, self.shared_img = self._make_expert(mat(I_sh, H), mat(I_sh, H), mat(H, I_sh), H, I_sh)
        self.shared_gate = O.round_bf16(mat(1, H))[0] if shared_gate else None

    @staticmethod
    def _make_expert(wgate, wup, wdown, H, I):
        blocks = [O.quantize_q4k(w) for w in (wgate, wup, wdown)]
        deq = tuple(O.dequant_q4k(b, n, k) for b, (n, k) in zip(blocks, ((I, H), (I, H), (H, I))))
        return deq, LY.pack_expert_q4k(blocks[0], blocks[1], blocks[2], H, I)
