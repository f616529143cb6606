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
