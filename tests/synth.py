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


# ---- fast synthesis for layers at the configured sizes ---------------------------------------
# The classes above go through the oracle's numpy quantiser and the product's numpy packer (tens of
# seconds per Mixtral-sized matrix).  The ones below do the same arithmetic with multi-threaded torch
# ops and dequantise an expert only when a check asks for it; tests/test_synth_fast.py pins them against
# the numpy path (quantiser, packer and dequantiser, bit for bit) on small shapes.

_NIB_SHIFT_T = (0, 16, 4, 20, 8, 24, 12, 28)   # bit position of element i of a dword in the slot layout


def fast_quantize_int4(w: torch.Tensor):
    """torch restatement of oracle.quantize_int4: w[N,K] fp32 -> (q u8 [N,K], s fp16 [N,G], z u8 [N,G])."""
    N, K = w.shape
    G = K // 128
    wg_ = w.reshape(N, G, 128)
    mn = torch.clamp(wg_.amin(dim=2), max=0.0)
    mx = torch.clamp(wg_.amax(dim=2), min=0.0)
    scale = (mx - mn) / 15.0
    scale = torch.where(scale <= 0, torch.ones_like(scale), scale).to(torch.float16)
    s32 = scale.float()
    zero = torch.clamp(torch.round(-mn / s32), 0, 15)
    q = torch.clamp(torch.round(wg_ / s32[:, :, None]) + zero[:, :, None], 0, 15).to(torch.uint8)
    return q.reshape(N, K), scale, zero.to(torch.uint8)


def fast_dequant_int4(q, s, z):
    N, K = q.shape
    G = K // 128
    return ((q.reshape(N, G, 128).float() - z[:, :, None].float()) * s.float()[:, :, None]).reshape(N, K)


def fast_tile_int4(q, s, z):
    """torch restatement of layout.tile_int4 -> (q tiles, scale tiles, zero tiles) as uint8 tensors."""
    N, K = q.shape
    G = K // 128
    q6 = q.to(torch.int32).reshape(N // 16, 16, G, 4, 4, 8)
    dw = torch.zeros(q6.shape[:-1], dtype=torch.int32)
    for i in range(8):
        dw |= q6[..., i] << _NIB_SHIFT_T[i]
    qt = dw.permute(0, 2, 3, 1, 4).contiguous().view(torch.uint8).reshape(-1)
    st = s.reshape(N // 16, 16, G).permute(0, 2, 1).contiguous().view(torch.uint8).reshape(-1)
    z3 = z.reshape(N // 16, 16, G).permute(0, 2, 1).reshape(N // 16, G, 8, 2)
    zt = (z3[..., 0] | (z3[..., 1] << 4)).contiguous().reshape(-1)
    return qt, st, zt


def fast_pack_expert_int4(gate, up, down, H, I):
    """(q, s, z) triples of W_gate[I,H], W_up[I,H], W_down[H,I] -> slot image (uint8 numpy array)."""
    lay = LY.int4_layout(H, I)

    def interleave(a, b):
        nb = a.shape[0] // 16
        return torch.stack([a.reshape(nb, 16, -1), b.reshape(nb, 16, -1)], dim=1).reshape(2 * a.shape[0], -1)

    t13 = fast_tile_int4(*[interleave(a, b) for a, b in zip(gate, up)])
    t2 = fast_tile_int4(*down)
    buf = torch.zeros(lay["total_bytes"], dtype=torch.uint8)
    for off, arr in zip(("off13_q", "off13_s", "off13_z", "off2_q", "off2_s", "off2_z"), t13 + t2):
        buf[lay[off]: lay[off] + arr.numel()] = arr
    return buf.numpy()


class LazyInt4Layer:
    """An int4-g128 MoE layer at a configured size: slot images for every expert, quantised tensors kept
    as (q, s, z), fp32 weights of an expert made on demand (`expert_fp32(e)`, cached) so that a check
    only pays for the experts a batch activates."""

    def __init__(self, H, I, E, I_sh=0, seed=0, shared_gate=False, zipf=None, alias_of=None, perm=None):
        self.H, self.I, self.E, self.I_sh = H, I, E, I_sh
        g = torch.Generator().manual_seed(seed)

        def mat(n, k):
            return torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02

        self.wg = O.round_bf16(mat(E, H).numpy())
        self.bias = O.zipf_gate_bias(E, zipf, seed=2) if zipf else None
        if alias_of is not None:
            # the experts of another layer in another order (perm[e] = its expert id): distinct routing
            # and distinct (layer, expert) -> weights mapping without quantising a second set
            self._qsz = [alias_of._qsz[p] for p in perm]
            self.slots = [alias_of.slots[p] for p in perm]
            self._shared_qsz, self.shared_img = alias_of._shared_qsz, alias_of.shared_img
        else:
            self._qsz, self.slots = [], []
            for _ in range(E):
                qsz = [fast_quantize_int4(mat(n, k)) for n, k in ((I, H), (I, H), (H, I))]
                self._qsz.append(qsz)
                self.slots.append(fast_pack_expert_int4(*qsz, H, I))
            self._shared_qsz = self.shared_img = None
            if I_sh:
                self._shared_qsz = [fast_quantize_int4(mat(n, k)) for n, k in ((I_sh, H), (I_sh, H), (H, I_sh))]
                self.shared_img = fast_pack_expert_int4(*self._shared_qsz, H, I_sh)
        self.shared_gate = O.round_bf16(mat(1, H).numpy())[0] if shared_gate else None
        self._cache = {}

    def expert_fp32(self, e):
        if e not in self._cache:
            self._cache[e] = tuple(fast_dequant_int4(*t).numpy() for t in self._qsz[e])
        return self._cache[e]

    def drop_cache(self):
        self._cache.clear()

    @property
    def shared_fp32(self):
        if self._shared_qsz is None:
            return None
        if "sh" not in self._cache:
            self._cache["sh"] = tuple(fast_dequant_int4(*t).numpy() for t in self._shared_qsz)
        return self._cache["sh"]

    def experts_for(self, idx):
        """The `experts` argument of the oracle's forward: real weights for the experts in idx, None elsewhere."""
        need = set(int(e) for e in np.unique(idx))
        return [self.expert_fp32(e) if e in need else None for e in range(self.E)]
