"""CPU oracle for the MoE-layer arithmetic (TEST INFRASTRUCTURE ONLY).

This file is the checker, never the product: only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it.  The product path (promoe_amd/)
runs hand-written HIP kernels and fails loudly without them.

What it restates
----------------
The reference (huwf5/promoe) contains no MoE arithmetic of its own; its hot path
is the *patched HuggingFace MoE module* whose contract is visible through the
stand-in `SimulateMoeLayer.forward` (eval/demo-simulate/transformers-deepseek-moe.py:36-49:
`expert_ids = self.report_experts(expert_ids)` then one expert call per id in the
returned order) and the hook sites (src/sparse_llm_cache/utils/__init__.py:82-96).
The arithmetic restated here is the published HuggingFace semantics those modules
implement: fp32 softmax over all experts, top-k, per-expert SwiGLU MLP
(gate_proj/up_proj/silu/down_proj) on the expert's tokens, weighted `index_add_`
combine, shared expert added afterwards (optionally scaled by sigmoid(x.w_s)).

Pinning status (what fixes each function, beyond re-typing a formula)
---------------------------------------------------------------------
* gate_logits_ordered / topk_route: closed forms; cross-checked in tests against
  float64 matmul, brute-force argsort on tiny inputs, constructed ties and the
  identity softmax(top-k logits) == renorm(top-k of softmax).
* dispatch: == numpy stable argsort; bijection/count invariants; brute force.
* int4 g128: pack->unpack round trip, closed form w=(q-z)*s, hand-built blocks.
* q4_K: hand-built known-answer super-blocks (all-zero, single nibble, max scale).
* swiglu_expert / moe_forward: reduce to torch F.linear/F.silu in fp32; the whole
  layer is checked against stock transformers' Qwen2-MoE, Mixtral and DeepSeek-V2
  sparse blocks run in fp32 (tests/test_oracle_vs_transformers.py).
* The exact bf16<->fp32 cast order of the external patched module is NOT pinned
  by anything in the reference ("parity unpinned" for that detail); it is covered
  by the 2e-2 output tolerance against this fp32 path.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

GROUP = 128  # int4 quantisation group size along K

# --------------------------------------------------------------------------
# bf16 helpers (bit-exact, round-to-nearest-even)
# --------------------------------------------------------------------------

def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rnd = ((u >> 16) & 1) + 0x7FFF
    return ((u + rnd) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_bf16(a: np.ndarray) -> np.ndarray:
    """fp32 -> nearest bf16 -> fp32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a))


# --------------------------------------------------------------------------
# k1 gating
# --------------------------------------------------------------------------

def gate_logits(x: np.ndarray, wg: np.ndarray) -> np.ndarray:
    """logits[T,E] = x[T,H] . wg[E,H]^T in fp32 (HF: F.linear(x.float(), w.float())).

    Summation order is whatever the BLAS picks; use gate_logits_ordered when
    bit-exact agreement with the HIP kernel is needed."""
    return F.linear(torch.from_numpy(np.asarray(x, np.float32)),
                    torch.from_numpy(np.asarray(wg, np.float32))).numpy()


def gate_logits_ordered(x: np.ndarray, wg: np.ndarray) -> np.ndarray:
    """Same product with the summation order fixed, so that fp32 results are
    bit-reproducible: 64 partial sums; partial l adds the products of
    k = c*512 + 8*l + i for c ascending then i = 0..7 ascending (one fp32
    rounding per add; every bf16*bf16 product is exact in fp32), then a butterfly
    p[l] += p[l ^ m] for m = 32,16,8,4,2,1.  x and wg must hold bf16-representable
    values."""
    x = np.asarray(x, np.float32)
    wg = np.asarray(wg, np.float32)
    T, H = x.shape
    E = wg.shape[0]
    Hp = (H + 511) // 512 * 512
    xp = np.zeros((T, Hp), np.float32); xp[:, :H] = x
    wp = np.zeros((E, Hp), np.float32); wp[:, :H] = wg
    xp = xp.reshape(T, 1, Hp // 512, 64, 8)
    wp = wp.reshape(1, E, Hp // 512, 64, 8)
    acc = np.zeros((T, E, 64), np.float32)
    for c in range(Hp // 512):
        for i in range(8):
            prod = (xp[:, :, c, :, i] * wp[:, :, c, :, i]).astype(np.float32)  # exact
            acc = (acc + prod).astype(np.float32)
    for m in (32, 16, 8, 4, 2, 1):
        idx = np.arange(64) ^ m
        acc = (acc + acc[:, :, idx]).astype(np.float32)
    return acc[:, :, 0].copy()


MODE_SOFTMAX_TOPK = 0          # DeepSeek-MoE, Qwen-MoE (norm_topk_prob=False)
MODE_SOFTMAX_TOPK_RENORM = 1   # Qwen-MoE with norm_topk_prob=True
MODE_TOPK_SOFTMAX = 2          # Mixtral: top-k of logits, softmax over the selected


def topk_route(logits: np.ndarray, k: int, mode: int = MODE_SOFTMAX_TOPK):
    """Returns (idx[T,k] int32, w[T,k] float32).

    Selection is on the logits, descending, ties broken toward the LOWER expert
    index.  softmax is monotone, so this equals top-k of the softmax except where
    two distinct logits round to the same probability (there the rule still
    prefers the larger logit).  Weights: fp32 softmax over all E (modes 0/1) or
    over the k selected logits (mode 2); mode 1 divides by the sum of the k."""
    logits = np.asarray(logits, np.float32)
    T, E = logits.shape
    # stable argsort of -logits: equal values keep ascending index order
    order = np.argsort(-logits.astype(np.float64), axis=1, kind="stable")
    idx = order[:, :k].astype(np.int32)
    sel = np.take_along_axis(logits, idx.astype(np.int64), axis=1)
    mx = logits.max(axis=1, keepdims=True)
    if mode == MODE_TOPK_SOFTMAX:
        ex = np.exp((sel - mx).astype(np.float32)).astype(np.float32)
        w = ex / ex.sum(axis=1, keepdims=True, dtype=np.float32)
    else:
        ex_all = np.exp((logits - mx).astype(np.float32)).astype(np.float32)
        den = ex_all.sum(axis=1, keepdims=True, dtype=np.float32)
        w = np.exp((sel - mx).astype(np.float32)).astype(np.float32) / den
        if mode == MODE_SOFTMAX_TOPK_RENORM:
            w = w / w.sum(axis=1, keepdims=True, dtype=np.float32)
    return idx, w.astype(np.float32)


# --------------------------------------------------------------------------
# k2 dispatch
# --------------------------------------------------------------------------

def dispatch(topk_idx: np.ndarray, num_expert: int):
    """Stable token->expert permutation of the T*k (token, slot) pairs.

    pair p = t*k + j.  Returns counts[E], offsets[E+1] (exclusive scan),
    sorted_pair[T*k] (pairs ordered by expert, ascending p within an expert) and
    pos_of_pair[T*k] (its inverse)."""
    flat = np.asarray(topk_idx, np.int64).reshape(-1)
    counts = np.bincount(flat, minlength=num_expert).astype(np.int32)
    offsets = np.zeros(num_expert + 1, np.int32)
    offsets[1:] = np.cumsum(counts)
    sorted_pair = np.argsort(flat, kind="stable").astype(np.int32)
    pos_of_pair = np.empty_like(sorted_pair)
    pos_of_pair[sorted_pair] = np.arange(flat.size, dtype=np.int32)
    return counts, offsets, sorted_pair, pos_of_pair


# --------------------------------------------------------------------------
# int4 asymmetric, group 128 along K.  Exchange format:
#   qweight int32 [N, K/8]    nibble j of word i holds q[n, 8i+j] (low nibble first)
#   scales  fp16  [N, K/128]
#   qzeros  int32 [ceil(N*G/8)] nibble (n*G+g) of the flat array, low nibble first
#   w = (q - z) * s
# --------------------------------------------------------------------------

def quantize_int4(w: np.ndarray):
    """Per-group min/max asymmetric quantisation of w[N,K] (fp32)."""
    w = np.asarray(w, np.float32)
    N, K = w.shape
    assert K % GROUP == 0
    G = K // GROUP
    wg = w.reshape(N, G, GROUP)
    mn = np.minimum(wg.min(axis=2), 0.0)
    mx = np.maximum(wg.max(axis=2), 0.0)
    scale = ((mx - mn) / 15.0).astype(np.float32)
    scale = np.where(scale <= 0, 1.0, scale).astype(np.float16)
    s32 = scale.astype(np.float32)
    zero = np.clip(np.rint(-mn / s32), 0, 15).astype(np.uint8)
    q = np.clip(np.rint(wg / s32[:, :, None]) + zero[:, :, None], 0, 15).astype(np.uint8)
    return q.reshape(N, K), scale, zero


def pack_int4(q: np.ndarray, zero: np.ndarray):
    """q[N,K] uint8 (0..15), zero[N,G] uint8 -> (qweight int32 [N,K/8], qzeros int32 flat)."""
    N, K = q.shape
    q32 = q.astype(np.uint32).reshape(N, K // 8, 8)
    qweight = np.zeros((N, K // 8), np.uint32)
    for j in range(8):
        qweight |= q32[:, :, j] << (4 * j)
    z = zero.astype(np.uint32).reshape(-1)
    pad = (-z.size) % 8
    z = np.concatenate([z, np.zeros(pad, np.uint32)]).reshape(-1, 8)
    qzeros = np.zeros(z.shape[0], np.uint32)
    for j in range(8):
        qzeros |= z[:, j] << (4 * j)
    return qweight.view(np.int32), qzeros.view(np.int32)


def unpack_int4(qweight: np.ndarray, qzeros: np.ndarray, N: int, K: int):
    G = K // GROUP
    qw = np.asarray(qweight).view(np.uint32).reshape(N, K // 8)
    q = np.stack([(qw >> (4 * j)) & 0xF for j in range(8)], axis=2).reshape(N, K).astype(np.uint8)
    qz = np.asarray(qzeros).view(np.uint32).reshape(-1)
    z = np.stack([(qz >> (4 * j)) & 0xF for j in range(8)], axis=1).reshape(-1)[: N * G]
    return q, z.reshape(N, G).astype(np.uint8)


def dequant_int4(qweight, scales, qzeros, N: int, K: int) -> np.ndarray:
    q, z = unpack_int4(qweight, qzeros, N, K)
    G = K // GROUP
    s = np.asarray(scales, np.float16).astype(np.float32).reshape(N, G)
    w = (q.reshape(N, G, GROUP).astype(np.float32) - z[:, :, None].astype(np.float32)) * s[:, :, None]
    return w.reshape(N, K).astype(np.float32)


# --------------------------------------------------------------------------
# q4_K (ggml block_q4_K): 256 weights per super-block, 144 bytes:
#   fp16 d, fp16 dmin, 12 bytes of packed 6-bit (scale, min) for 8 sub-blocks of 32,
#   128 bytes of nibbles.   w = d*sc_j*q - dmin*m_j
# Nibble order (ggml): for each 64-weight chunk c (0..3), bytes qs[32c .. 32c+31]:
#   low nibbles are weights 64c+0..31 (sub-block 2c), high nibbles 64c+32..63 (2c+1).
def dequant_gptq(qweight, qzeros, scales, g_idx=None, zero_plus_one: bool = True) -> np.ndarray:
    """AutoGPTQ checkpoint tensors of one linear layer -> fp32 weight [N, K] (out x in).

    Restates the published AutoGPTQ 4-bit convention (the library itself is not part of the
    reference tree: the reference only moves these buffers, utils/__init__.py:39-60):
    qweight int32 [K/8, N] packs 8 inputs per word, low nibble first; qzeros int32 [G, N/8] packs 8
    outputs per word; format "gptq" stores zero - 1 and adds the one back modulo 16; scales [G, N];
    w[k, n] = (q[k, n] - zero[g_idx[k], n]) * scales[g_idx[k], n].  Plain loops over the nibbles on
    purpose (the product code uses a vectorised transpose)."""
    qw = np.asarray(qweight).view(np.uint32)
    qz = np.asarray(qzeros).view(np.uint32)
    sc = np.asarray(scales, np.float16).astype(np.float32)
    K, N = qw.shape[0] * 8, qw.shape[1]
    G = qz.shape[0]
    gi = np.arange(K) // (K // G) if g_idx is None else np.asarray(g_idx).reshape(-1)
    w = np.zeros((N, K), np.float32)
    for k in range(K):
        q = (qw[k // 8, :] >> np.uint32(4 * (k % 8))) & 0xF                    # [N]
        g = int(gi[k])
        z = np.array([(qz[g, n // 8] >> np.uint32(4 * (n % 8))) & 0xF for n in range(N)], np.int64)
        if zero_plus_one:
            z = (z + 1) & 0xF
        w[:, k] = (q.astype(np.float32) - z.astype(np.float32)) * sc[g, :]
    return w


# --------------------------------------------------------------------------
QK_K = 256
Q4K_BYTES = 144


def q4k_unpack_scales(sc12: np.ndarray):
    """12 bytes -> (sc[8], m[8]) 6-bit values (ggml get_scale_min_k4)."""
    s = np.asarray(sc12, np.uint8).astype(np.int32)
    sc = np.zeros(8, np.int32); mn = np.zeros(8, np.int32)
    for j in range(8):
        if j < 4:
            sc[j] = s[j] & 63
            mn[j] = s[j + 4] & 63
        else:
            sc[j] = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
            mn[j] = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
    return sc, mn


def q4k_pack_scales(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Inverse of q4k_unpack_scales."""
    sc = np.asarray(sc, np.int32); mn = np.asarray(mn, np.int32)
    out = np.zeros(12, np.int32)
    for j in range(4):
        out[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        out[j + 4] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        out[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    return out.astype(np.uint8)


def dequant_q4k_block(blk: np.ndarray) -> np.ndarray:
    """One 144-byte block -> 256 fp32 weights."""
    blk = np.asarray(blk, np.uint8)
    d = blk[0:2].view(np.float16)[0].astype(np.float32)
    dmin = blk[2:4].view(np.float16)[0].astype(np.float32)
    sc, mn = q4k_unpack_scales(blk[4:16])
    qs = blk[16:144]
    out = np.zeros(QK_K, np.float32)
    for c in range(4):
        b = qs[32 * c: 32 * c + 32].astype(np.int32)
        d1 = d * np.float32(sc[2 * c]); m1 = dmin * np.float32(mn[2 * c])
        d2 = d * np.float32(sc[2 * c + 1]); m2 = dmin * np.float32(mn[2 * c + 1])
        out[64 * c: 64 * c + 32] = d1 * (b & 0xF).astype(np.float32) - m1
        out[64 * c + 32: 64 * c + 64] = d2 * (b >> 4).astype(np.float32) - m2
    return out


def dequant_q4k(blocks: np.ndarray, N: int, K: int) -> np.ndarray:
    """blocks uint8 [N, K/256, 144] -> fp32 [N, K] (vectorised form of the above)."""
    b = np.asarray(blocks, np.uint8).reshape(N, K // QK_K, Q4K_BYTES)
    d = b[:, :, 0:2].copy().view(np.float16)[:, :, 0].astype(np.float32)
    dmin = b[:, :, 2:4].copy().view(np.float16)[:, :, 0].astype(np.float32)
    s = b[:, :, 4:16].astype(np.int32)
    sc = np.zeros(s.shape[:2] + (8,), np.int32); mn = np.zeros_like(sc)
    for j in range(8):
        if j < 4:
            sc[:, :, j] = s[:, :, j] & 63
            mn[:, :, j] = s[:, :, j + 4] & 63
        else:
            sc[:, :, j] = (s[:, :, j + 4] & 0xF) | ((s[:, :, j - 4] >> 6) << 4)
            mn[:, :, j] = (s[:, :, j + 4] >> 4) | ((s[:, :, j] >> 6) << 4)
    qs = b[:, :, 16:144].reshape(N, K // QK_K, 4, 32).astype(np.int32)
    lo = (qs & 0xF).astype(np.float32); hi = (qs >> 4).astype(np.float32)
    q = np.stack([lo, hi], axis=3).reshape(N, K // QK_K, 8, 32)
    w = (d[:, :, None] * sc.astype(np.float32))[:, :, :, None] * q \
        - (dmin[:, :, None] * mn.astype(np.float32))[:, :, :, None]
    return w.reshape(N, K).astype(np.float32)


def quantize_q4k(w: np.ndarray) -> np.ndarray:
    """Simple q4_K quantiser (min/max per sub-block, 6-bit scale/min against the
    super-block maxima).  It produces VALID q4_K blocks; it does not reproduce
    ggml's iterative make_qkx2 search, which is irrelevant for parity because the
    dequantised weights are defined by the block bytes alone."""
    w = np.asarray(w, np.float32)
    N, K = w.shape
    assert K % QK_K == 0
    nb = K // QK_K
    wb = w.reshape(N, nb, 8, 32)
    mn = np.maximum(-wb.min(axis=3), 0.0)                # min offset (>=0)
    mx = wb.max(axis=3)
    sub_scale = np.maximum((mx + mn) / 15.0, 0.0)
    d = (sub_scale.max(axis=2) / 63.0).astype(np.float16)
    dmin = (mn.max(axis=2) / 63.0).astype(np.float16)
    d32 = d.astype(np.float32); dm32 = dmin.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d32[:, :, None] > 0, np.rint(sub_scale / d32[:, :, None]), 0)
        mq = np.where(dm32[:, :, None] > 0, np.rint(mn / dm32[:, :, None]), 0)
    sc = np.clip(sc, 0, 63).astype(np.int32); mq = np.clip(mq, 0, 63).astype(np.int32)
    eff_s = d32[:, :, None] * sc; eff_m = dm32[:, :, None] * mq
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(eff_s[..., None] > 0, np.rint((wb + eff_m[..., None]) / eff_s[..., None]), 0)
    q = np.clip(q, 0, 15).astype(np.uint8)
    out = np.zeros((N, nb, Q4K_BYTES), np.uint8)
    out[:, :, 0:2] = d.reshape(N, nb, 1).view(np.uint8).reshape(N, nb, 2)
    out[:, :, 2:4] = dmin.reshape(N, nb, 1).view(np.uint8).reshape(N, nb, 2)
    for j in range(4):
        out[:, :, 4 + j] = (sc[:, :, j] & 63) | ((sc[:, :, j + 4] >> 4) << 6)
        out[:, :, 8 + j] = (mq[:, :, j] & 63) | ((mq[:, :, j + 4] >> 4) << 6)
        out[:, :, 12 + j] = (sc[:, :, j + 4] & 0xF) | ((mq[:, :, j + 4] & 0xF) << 4)
    q4 = q.reshape(N, nb, 4, 2, 32)
    out[:, :, 16:144] = (q4[:, :, :, 0, :] | (q4[:, :, :, 1, :] << 4)).reshape(N, nb, 128)
    return out


# --------------------------------------------------------------------------
# q6_K (ggml block_q6_K): 256 weights per block, 210 bytes: ql[128] (low 4 bits), qh[64] (high 2 bits),
# int8 scales[16] (one per 16 weights), fp16 d.   w = d * scale * (q - 32), q in 0..63.
# Not in the reference tree (it names the q4_k_m file type, README.md:29-34, whose ffn_down tensors
# llama.cpp stores as Q6_K); restated from ggml's published dequantize_row_q6_K, loop for loop.
Q6K_BYTES = 210


def dequant_q6k_block(blk: np.ndarray) -> np.ndarray:
    """One 210-byte block -> 256 fp32 weights (plain loops on purpose)."""
    blk = np.asarray(blk, np.uint8)
    ql, qh = blk[0:128].astype(np.int32), blk[128:192].astype(np.int32)
    sc = blk[192:208].view(np.int8).astype(np.int32)
    d = np.float32(blk[208:210].view(np.float16)[0])
    y = np.zeros(256, np.float32)
    for half in range(2):                       # 128 weights per half
        qlh, qhh, sch, yo = ql[64 * half:], qh[32 * half:], sc[8 * half:], 128 * half
        for l in range(32):
            i_s = l // 16
            q1 = ((qlh[l] & 0xF) | (((qhh[l] >> 0) & 3) << 4)) - 32
            q2 = ((qlh[l + 32] & 0xF) | (((qhh[l] >> 2) & 3) << 4)) - 32
            q3 = ((qlh[l] >> 4) | (((qhh[l] >> 4) & 3) << 4)) - 32
            q4 = ((qlh[l + 32] >> 4) | (((qhh[l] >> 6) & 3) << 4)) - 32
            y[yo + l] = d * np.float32(sch[i_s + 0]) * np.float32(q1)
            y[yo + l + 32] = d * np.float32(sch[i_s + 2]) * np.float32(q2)
            y[yo + l + 64] = d * np.float32(sch[i_s + 4]) * np.float32(q3)
            y[yo + l + 96] = d * np.float32(sch[i_s + 6]) * np.float32(q4)
    return y


def dequant_q6k(blocks: np.ndarray, N: int, K: int) -> np.ndarray:
    blocks = np.asarray(blocks, np.uint8).reshape(N, K // QK_K, Q6K_BYTES)
    out = np.zeros((N, K), np.float32)
    for n in range(N):
        for b in range(K // QK_K):
            out[n, b * QK_K:(b + 1) * QK_K] = dequant_q6k_block(blocks[n, b])
    return out


# --------------------------------------------------------------------------
# k3/k4 expert product, k5 combine, whole-layer forward (HF structure)
# --------------------------------------------------------------------------

def swiglu_expert(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
                  w_down: torch.Tensor) -> torch.Tensor:
    """down_proj(silu(gate_proj(x)) * up_proj(x)); all fp32; weights [out,in]."""
    return F.linear(F.silu(F.linear(x, w_gate)) * F.linear(x, w_up), w_down)


def moe_forward(x, wg, experts, k, mode=MODE_SOFTMAX_TOPK, shared=None, shared_gate=None,
                logits=None, expert_order=None):
    """One MoE layer forward in fp32, structured like the patched HF module the
    reference hooks (per-expert loop in `expert_order`, default ascending id —
    the order `report_experts` returns, utils/__init__.py:84-88).

    x [T,H] fp32 (bf16-representable), wg [E,H], experts: list of (w_gate[I,H],
    w_up[I,H], w_down[H,I]) fp32 (already dequantised), shared: optional
    (w_gate, w_up, w_down), shared_gate: optional w_s[H] (sigmoid-gated shared).
    Returns dict(out[T,H], idx, w, logits)."""
    x_t = torch.from_numpy(np.asarray(x, np.float32))
    if logits is None:
        logits = gate_logits_ordered(np.asarray(x, np.float32), np.asarray(wg, np.float32))
    idx, w = topk_route(logits, k, mode)
    T, H = x_t.shape
    out = torch.zeros(T, H, dtype=torch.float32)
    idx_t = torch.from_numpy(idx.astype(np.int64)); w_t = torch.from_numpy(w)
    act = np.unique(idx) if expert_order is None else np.asarray(expert_order)
    for e in act:
        tok, slot = torch.where(idx_t == int(e))
        if tok.numel() == 0:
            continue
        wge, wue, wde = (torch.from_numpy(np.asarray(a, np.float32)) for a in experts[int(e)])
        y = swiglu_expert(x_t[tok], wge, wue, wde) * w_t[tok, slot].unsqueeze(1)
        out.index_add_(0, tok, y)
    if shared is not None:
        ws = [torch.from_numpy(np.asarray(a, np.float32)) for a in shared]
        ys = swiglu_expert(x_t, *ws)
        if shared_gate is not None:
            g = torch.sigmoid(F.linear(x_t, torch.from_numpy(np.asarray(shared_gate, np.float32)).reshape(1, -1)))
            ys = ys * g
        out = out + ys
    return dict(out=out.numpy(), idx=idx, w=w, logits=logits)


# --------------------------------------------------------------------------
# seeded synthetic data of the benchmark configurations
# --------------------------------------------------------------------------

def zipf_gate_bias(num_expert: int, s: float, seed: int = 2) -> np.ndarray:
    """b_e = -s*log(rank_e) with a seeded rank permutation: added to the gate logits
    it makes expert popularity follow roughly Zipf(s)."""
    rng = np.random.default_rng(seed)
    rank = rng.permutation(num_expert) + 1
    return (-s * np.log(rank.astype(np.float64))).astype(np.float32)


def synth_weights(shape, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).numpy()


def synth_acts(T, H, seed=1):
    g = torch.Generator().manual_seed(seed)
    return round_bf16(torch.randn(T, H, generator=g, dtype=torch.float32).numpy())
