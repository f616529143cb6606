"""Host-side repacking of expert weights into the engine's cache-slot layout.

The exchange format a caller hands over for an int4 matrix W[N,K] is the plain one
(`qweight` int32 [N,K/8] low-nibble-first along K, `scales` fp16 [N,K/128], `qzeros`
uint4 packed 8 per int32 over the flat index n*G+g).  The slot layout (see
include/moe_kernels.h) tiles it 16 rows x 128 k so that one 64-lane dwordx4 load is
one tile and interleaves the nibbles so that a shift+mask yields bf16 pairs.

Reference counterpart: the reference copies whatever tensors the quantisation
backend registered, chunk by chunk (worker.cpp:84-105); the repack replaces
AutoGPTQ's exllama `post_init` shuffle that the reference has to drive through
temp_move_expert_to_gpu (prefetcher.cpp:663-697, utils/hooks.py:402-440).
"""
from __future__ import annotations

import numpy as np

GROUP = 128

# bit position of element i (0..7) of a dword in the slot layout
_NIB_SHIFT = np.array([0, 16, 4, 20, 8, 24, 12, 28], dtype=np.uint32)


def int4_layout(H: int, I: int) -> dict:
    """Section offsets of one int4 expert (mirror of moe_int4_layout_make)."""
    assert H % 128 == 0 and I % 128 == 0
    n13, g13, n2, g2 = 2 * I, H // 128, H, I // 128
    o = 0
    out = {}
    for name, sz in (("off13_q", n13 * H // 2), ("off13_s", n13 * g13 * 2), ("off13_z", n13 * g13 // 2),
                     ("off2_q", n2 * I // 2), ("off2_s", n2 * g2 * 2), ("off2_z", n2 * g2 // 2)):
        out[name] = o
        o += sz
    out["total_bytes"] = o
    return out


def _unpack_exchange(qweight, scales, qzeros, N, K):
    G = K // GROUP
    qw = np.ascontiguousarray(qweight).view(np.uint32).reshape(N, K // 8)
    q = np.stack([(qw >> np.uint32(4 * j)) & np.uint32(0xF) for j in range(8)], axis=2).reshape(N, K)
    qz = np.ascontiguousarray(qzeros).view(np.uint32).reshape(-1)
    z = np.stack([(qz >> np.uint32(4 * j)) & np.uint32(0xF) for j in range(8)], axis=1).reshape(-1)[: N * G]
    s = np.ascontiguousarray(scales).view(np.float16).reshape(N, G)
    return q.astype(np.uint32), s, z.reshape(N, G).astype(np.uint8)


def tile_int4(q: np.ndarray, s: np.ndarray, z: np.ndarray):
    """q[N,K] (0..15), s[N,G] fp16, z[N,G] (0..15) -> (qtiles u8, stiles u8, ztiles u8)."""
    N, K = q.shape
    assert N % 16 == 0 and K % GROUP == 0
    G = K // GROUP
    # [rb, r, g, qd, j, i] -> tile order [rb, g, qd, r, j] with i packed into a dword
    q6 = q.astype(np.uint32).reshape(N // 16, 16, G, 4, 4, 8)
    dw = np.zeros(q6.shape[:-1], np.uint32)
    for i in range(8):
        dw |= q6[..., i] << _NIB_SHIFT[i]
    dw = dw.transpose(0, 2, 3, 1, 4)          # [rb, g, qd, r, j]; lane = qd*16 + r
    qt = np.ascontiguousarray(dw).view(np.uint8).reshape(-1)
    st = np.ascontiguousarray(s.astype(np.float16).reshape(N // 16, 16, G).transpose(0, 2, 1)).view(np.uint8).reshape(-1)
    z3 = z.astype(np.uint8).reshape(N // 16, 16, G).transpose(0, 2, 1).reshape(N // 16, G, 8, 2)
    zt = np.ascontiguousarray(z3[..., 0] | (z3[..., 1] << 4)).reshape(-1)
    return qt, st, zt


def pack_expert_int4(gate, up, down, H: int, I: int) -> np.ndarray:
    """gate/up/down: (qweight, scales, qzeros) in the exchange format for W_gate[I,H],
    W_up[I,H], W_down[H,I].  Returns the slot image (uint8, total_bytes)."""
    lay = int4_layout(H, I)
    qg, sg, zg = _unpack_exchange(*gate, I, H)
    qu, su, zu = _unpack_exchange(*up, I, H)
    qd, sd, zd = _unpack_exchange(*down, H, I)

    def interleave(a, b):  # 16-row blocks: gate block, up block, gate block, ...
        nb = a.shape[0] // 16
        return np.stack([a.reshape(nb, 16, -1), b.reshape(nb, 16, -1)], axis=1).reshape(2 * a.shape[0], -1)

    q13, s13, z13 = interleave(qg, qu), interleave(sg, su), interleave(zg, zu)
    buf = np.zeros(lay["total_bytes"], np.uint8)
    for off, arr in zip(("off13_q", "off13_s", "off13_z"), tile_int4(q13, s13, z13)):
        buf[lay[off]: lay[off] + arr.size] = arr
    for off, arr in zip(("off2_q", "off2_s", "off2_z"), tile_int4(qd, sd, zd)):
        buf[lay[off]: lay[off] + arr.size] = arr
    return buf


def split_chunks_int4(H: int, I: int):
    """(name, offset, nbytes) of the six copy chunks of an int4 expert, in slot order."""
    lay = int4_layout(H, I)
    names = ["off13_q", "off13_s", "off13_z", "off2_q", "off2_s", "off2_z"]
    ends = [lay[n] for n in names[1:]] + [lay["total_bytes"]]
    return [(n.replace("off", "w"), lay[n], e - lay[n]) for n, e in zip(names, ends)]


# ---- bf16 experts -------------------------------------------------------------------
# A matrix W[N,K] is stored as blocks of 32 rows x 64 k (2048 elements, 4 KiB).  Block
# (nb, kb) lies at element offset (((nb//4)*(K/64) + kb)*4 + nb%4)*2048: the four blocks of a
# 128-row group are adjacent for each k slab.  The slabs of group g are stored rotated: slab
# kb sits at position (kb + g*s) % (K/64), s = slab_step(K/64), which keeps groups that are
# read in step on different DRAM channels.  Inside a block the order is [j][q][n][e] with
# k = 64kb + 32q + 8j + e: the 64 lanes (lane = 32q + n) of a wave read 16 bytes each of one
# contiguous KiB per j, already in the operand order of v_mfma_f32_32x32x16_bf16.

def slab_step(nk: int) -> int:
    """Smallest odd s >= 3 coprime with nk."""
    import math
    s = 3
    while math.gcd(s, nk) != 1:
        s += 2
    return s


def tile_bf16(w_bits: np.ndarray) -> np.ndarray:
    """w_bits uint16 [N,K] (bf16 bit patterns) -> flat uint16 array in the block layout."""
    N, K = w_bits.shape
    assert N % 128 == 0 and K % 64 == 0
    nk = K // 64
    t = w_bits.reshape(N // 128, 4, 32, nk, 2, 4, 8)      # g w n kb q j e
    t = np.ascontiguousarray(t.transpose(0, 3, 1, 5, 4, 2, 6))  # g kb w j q n e
    s = slab_step(nk)
    for g in range(N // 128):
        t[g] = np.roll(t[g], (g * s) % nk, axis=0)
    return t.reshape(-1)


def untile_bf16(flat: np.ndarray, N: int, K: int) -> np.ndarray:
    nk = K // 64
    t = flat.reshape(N // 128, nk, 4, 4, 2, 32, 8).copy()       # g kb w j q n e
    s = slab_step(nk)
    for g in range(N // 128):
        t[g] = np.roll(t[g], -((g * s) % nk), axis=0)
    return np.ascontiguousarray(t.transpose(0, 2, 5, 1, 4, 3, 6)).reshape(N, K)


def pack_expert_bf16(gate_bits, up_bits, down_bits) -> np.ndarray:
    """Slot image of one bf16 expert: tiled w13 (gate rows, then up rows) followed by tiled w2."""
    w13 = np.concatenate([gate_bits, up_bits], axis=0)
    return np.concatenate([tile_bf16(w13), tile_bf16(down_bits)]).view(np.uint8)


def bf16_expert_bytes(H: int, I: int) -> int:
    return 3 * I * H * 2


# ---- q4_K experts -------------------------------------------------------------------
# The information of ggml's block_q4_K (fp16 d and dmin per 256 weights, a 6-bit scale and
# min per 32-wide sub-block, 4-bit quants) in the tile order of the int4 kernels: nibble
# tiles as in tile_int4; section s = [N/16][G][64] byte pairs (sc, m), lane l = 16*qd + r of
# tile (rb, g) holding row 16rb + r, sub-block 4*(g&1) + qd of super-block g//2; section z =
# [N/16][G/2][16] pairs (fp16 d, fp16 dmin).

def q4k_layout(H: int, I: int) -> dict:
    from ._lib import lib, Int4Layout, check
    import ctypes as C
    out = Int4Layout()
    check(lib.moe_q4k_layout_make(H, I, C.byref(out)), "moe_q4k_layout_make")
    return {n: int(getattr(out, n)) for n, _ in Int4Layout._fields_}


def _q4k_fields(blocks: np.ndarray, N: int, K: int):
    """ggml blocks uint8 [N, K/256, 144] -> q [N,K] (0..15), sc, mn [N, K/32] (0..63), d, dmin fp16 [N, K/256]."""
    b = np.asarray(blocks, np.uint8).reshape(N, K // 256, 144)
    d = b[:, :, 0:2].copy().view(np.float16)[:, :, 0]
    dmin = b[:, :, 2:4].copy().view(np.float16)[:, :, 0]
    s = b[:, :, 4:16].astype(np.int32)
    sc = np.zeros(s.shape[:2] + (8,), np.int32)
    mn = np.zeros_like(sc)
    for j in range(8):
        if j < 4:
            sc[:, :, j] = s[:, :, j] & 63
            mn[:, :, j] = s[:, :, j + 4] & 63
        else:
            sc[:, :, j] = (s[:, :, j + 4] & 0xF) | ((s[:, :, j - 4] >> 6) << 4)
            mn[:, :, j] = (s[:, :, j + 4] >> 4) | ((s[:, :, j] >> 6) << 4)
    qs = b[:, :, 16:144].reshape(N, K // 256, 4, 32)
    q = np.stack([qs & 0xF, qs >> 4], axis=3).reshape(N, K)   # chunk c: low nibbles then high nibbles
    return q.astype(np.uint32), sc.reshape(N, K // 32), mn.reshape(N, K // 32), d, dmin


def tile_q4k(blocks: np.ndarray, N: int, K: int):
    """One matrix of ggml q4_K blocks -> (q tiles, s section, z section) as uint8 arrays."""
    assert N % 16 == 0 and K % 256 == 0
    G = K // GROUP
    q, sc, mn, d, dmin = _q4k_fields(blocks, N, K)
    q6 = q.reshape(N // 16, 16, G, 4, 4, 8)
    dw = np.zeros(q6.shape[:-1], np.uint32)
    for i in range(8):
        dw |= q6[..., i] << _NIB_SHIFT[i]
    qt = np.ascontiguousarray(dw.transpose(0, 2, 3, 1, 4)).view(np.uint8).reshape(-1)   # [rb, g, qd, r, j]
    pair = (sc.astype(np.uint16) | (mn.astype(np.uint16) << 8)).reshape(N // 16, 16, G, 4)  # [rb, r, g, qd]
    st = np.ascontiguousarray(pair.transpose(0, 2, 3, 1)).view(np.uint8).reshape(-1)         # [rb, g, qd, r]
    dd = (d.view(np.uint16).astype(np.uint32) | (dmin.view(np.uint16).astype(np.uint32) << 16))
    zt = np.ascontiguousarray(dd.reshape(N // 16, 16, G // 2).transpose(0, 2, 1)).view(np.uint8).reshape(-1)
    return qt, st, zt


def pack_expert_q4k(gate_blocks, up_blocks, down_blocks, H: int, I: int) -> np.ndarray:
    """Slot image of one q4_K expert from its three matrices in ggml block form
    ([I, H/256, 144], [I, H/256, 144], [H, I/256, 144])."""
    lay = q4k_layout(H, I)
    g = np.asarray(gate_blocks, np.uint8).reshape(I, H // 256, 144)
    u = np.asarray(up_blocks, np.uint8).reshape(I, H // 256, 144)
    # gate / up rows interleaved in 16-row blocks, as in the int4 layout
    w13 = np.stack([g.reshape(I // 16, 16, H // 256, 144), u.reshape(I // 16, 16, H // 256, 144)], axis=1)
    w13 = w13.reshape(2 * I, H // 256, 144)
    buf = np.zeros(lay["total_bytes"], np.uint8)
    q13, s13, z13 = tile_q4k(w13, 2 * I, H)
    q2, s2, z2 = tile_q4k(down_blocks, H, I)
    for off, arr in ((lay["off13_q"], q13), (lay["off13_s"], s13), (lay["off13_z"], z13),
                     (lay["off2_q"], q2), (lay["off2_s"], s2), (lay["off2_z"], z2)):
        buf[off: off + arr.size] = arr
    assert lay["off2_z"] + z2.size == lay["total_bytes"]
    return buf
