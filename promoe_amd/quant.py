"""Weight quantisers producing the int4 exchange format (host side, torch CPU).

Per-group (128 along K) min/max asymmetric: s = (max-min)/15 stored as fp16,
z = round(-min/s) in 0..15, q = clip(round(w/s)+z, 0, 15); w ~ (q - z)*s.
"""
from __future__ import annotations

import numpy as np
import torch

GROUP = 128


def quantize_int4(w: torch.Tensor):
    """w [N,K] fp32 -> (qweight int32 [N,K/8], scales fp16 [N,G], qzeros int32 flat) as numpy."""
    w = w.to(torch.float32)
    N, K = w.shape
    assert K % GROUP == 0
    G = K // GROUP
    wg = w.reshape(N, G, GROUP)
    mn = wg.amin(dim=2).clamp(max=0.0)
    mx = wg.amax(dim=2).clamp(min=0.0)
    scale = (mx - mn) / 15.0
    scale = torch.where(scale <= 0, torch.ones_like(scale), scale).to(torch.float16)
    s32 = scale.to(torch.float32)
    zero = torch.clamp(torch.round(-mn / s32), 0, 15)
    q = torch.clamp(torch.round(wg / s32[:, :, None]) + zero[:, :, None], 0, 15).to(torch.int32)
    q = q.reshape(N, K // 8, 8)
    shifts = torch.arange(8, dtype=torch.int32) * 4
    qweight = (q << shifts).sum(dim=2, dtype=torch.int64)
    qweight = qweight.to(torch.int64).numpy().astype(np.uint32).view(np.int32)
    z = zero.to(torch.int64).reshape(-1).numpy().astype(np.uint32)
    pad = (-z.size) % 8
    z = np.concatenate([z, np.zeros(pad, np.uint32)]).reshape(-1, 8)
    qz = np.zeros(z.shape[0], np.uint32)
    for j in range(8):
        qz |= z[:, j] << np.uint32(4 * j)
    return qweight, scale.numpy(), qz.view(np.int32)


QK_K = 256


def dequant_q6k(blocks: np.ndarray) -> np.ndarray:
    """ggml block_q6_K bytes [..., nb, 210] -> fp32 [..., nb * 256] (w = d * scale * (q - 32); vectorised)."""
    b = np.asarray(blocks, np.uint8)
    lead = b.shape[:-1]
    ql = b[..., 0:128].reshape(lead + (2, 2, 32)).astype(np.int32)      # [half][which 32 bytes][l]
    qh = b[..., 128:192].reshape(lead + (2, 32)).astype(np.int32)       # [half][l]
    sc = np.ascontiguousarray(b[..., 192:208]).view(np.int8).reshape(lead + (2, 8)).astype(np.float32)
    d = np.ascontiguousarray(b[..., 208:210]).view(np.float16).reshape(lead).astype(np.float32)
    # the four 32-weight runs of a half: (ql[0] low, ql[1] low, ql[0] high, ql[1] high) with qh bits 0-1, 2-3, 4-5, 6-7
    q = np.stack([(ql[..., 0, :] & 0xF) | (((qh >> 0) & 3) << 4),
                  (ql[..., 1, :] & 0xF) | (((qh >> 2) & 3) << 4),
                  (ql[..., 0, :] >> 4) | (((qh >> 4) & 3) << 4),
                  (ql[..., 1, :] >> 4) | (((qh >> 6) & 3) << 4)], axis=-2) - 32     # [..., half, 4, 32]
    # scale index of element l of run j: l // 16 + 2 j
    scj = sc.reshape(lead + (2, 4, 2))                                                # [..., half, j, l // 16]
    w = d[..., None, None, None] * np.repeat(scj, 16, axis=-1) * q.astype(np.float32)
    return w.reshape(lead[:-1] + (lead[-1] * QK_K,)).astype(np.float32)


def quantize_q4k(w: np.ndarray) -> np.ndarray:
    """fp32 [N, K] -> ggml block_q4_K bytes [N, K/256, 144]: min/max per 32-wide sub-block, 6-bit scale and
    min against the super-block maxima (not ggml's iterative search; the blocks are valid q4_K and the
    weights they stand for are defined by their bytes alone)."""
    w = np.asarray(w, np.float32)
    N, K = w.shape
    assert K % QK_K == 0
    nb = K // QK_K
    wb = w.reshape(N, nb, 8, 32)
    mn = np.maximum(-wb.min(axis=3), 0.0)
    mx = wb.max(axis=3)
    sub_scale = np.maximum((mx + mn) / 15.0, 0.0)
    d = (sub_scale.max(axis=2) / 63.0).astype(np.float16)
    dmin = (mn.max(axis=2) / 63.0).astype(np.float16)
    d32, dm32 = d.astype(np.float32), dmin.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d32[:, :, None] > 0, np.rint(sub_scale / d32[:, :, None]), 0)
        mq = np.where(dm32[:, :, None] > 0, np.rint(mn / dm32[:, :, None]), 0)
    sc = np.clip(sc, 0, 63).astype(np.int32)
    mq = np.clip(mq, 0, 63).astype(np.int32)
    eff_s, eff_m = d32[:, :, None] * sc, dm32[:, :, None] * mq
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(eff_s[..., None] > 0, np.rint((wb + eff_m[..., None]) / eff_s[..., None]), 0)
    q = np.clip(q, 0, 15).astype(np.uint8)
    out = np.zeros((N, nb, 144), np.uint8)
    out[:, :, 0:2] = d.reshape(N, nb, 1).view(np.uint8).reshape(N, nb, 2)
    out[:, :, 2:4] = dmin.reshape(N, nb, 1).view(np.uint8).reshape(N, nb, 2)
    for j in range(4):
        out[:, :, 4 + j] = (sc[:, :, j] & 63) | ((sc[:, :, j + 4] >> 4) << 6)
        out[:, :, 8 + j] = (mq[:, :, j] & 63) | ((mq[:, :, j + 4] >> 4) << 6)
        out[:, :, 12 + j] = (sc[:, :, j + 4] & 0xF) | ((mq[:, :, j + 4] & 0xF) << 4)
    q4 = q.reshape(N, nb, 4, 2, 32)
    out[:, :, 16:144] = (q4[:, :, :, 0, :] | (q4[:, :, :, 1, :] << 4)).reshape(N, nb, 128)
    return out
