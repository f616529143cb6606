"""What pins the arithmetic oracle: closed forms, brute force, identities, known-answer
blocks.  A plausible mistake (dropped term, wrong sign/index, transposed operand) fails one."""
import numpy as np
import torch

from oracle import moe_oracle as O


def test_bf16_rounding_is_nearest_even():
    a = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.1415927, 65504.0, 1e-8], np.float32)
    got = O.round_bf16(a)
    ref = torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    assert np.array_equal(got, ref)
    # ties: 1 + 2^-8 is exactly half way between 1 and 1+2^-7 -> even (1.0); 1 + 3*2^-8 -> 1+2^-6
    assert O.round_bf16(np.array([1 + 2.0 ** -8], np.float32))[0] == 1.0
    assert O.round_bf16(np.array([1 + 3 * 2.0 ** -8], np.float32))[0] == 1 + 2.0 ** -6


def test_gate_logits_ordered_matches_float64_and_shape_transposes():
    rng = np.random.default_rng(0)
    x = O.round_bf16(rng.normal(0, 1, (5, 640)).astype(np.float32))
    w = O.round_bf16(rng.normal(0, 0.02, (7, 640)).astype(np.float32))
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    got = O.gate_logits_ordered(x, w)
    assert got.shape == (5, 7)
    assert np.allclose(got, ref, rtol=0, atol=2e-6)
    assert np.allclose(O.gate_logits(x, w), ref, rtol=0, atol=2e-6)
    # one-hot rows pick single weights exactly (catches a wrong index / transposed operand)
    x1 = np.zeros((2, 640), np.float32); x1[0, 3] = 1.0; x1[1, 639] = 2.0
    g = O.gate_logits_ordered(x1, w)
    assert np.array_equal(g[0], w[:, 3]) and np.array_equal(g[1], 2 * w[:, 639])


def test_topk_route_bruteforce_ties_and_identity():
    rng = np.random.default_rng(1)
    for T, E, k in ((6, 8, 2), (4, 64, 6), (3, 60, 4)):
        lg = rng.normal(0, 2, (T, E)).astype(np.float32)
        lg[0, 5] = lg[0, 2]                       # a tie inside the row
        idx, w = O.topk_route(lg, k, O.MODE_SOFTMAX_TOPK)
        for t in range(T):                         # brute force: sort by (-value, index)
            order = sorted(range(E), key=lambda e: (-float(lg[t, e]), e))[:k]
            assert list(idx[t]) == order
        p = torch.softmax(torch.from_numpy(lg), dim=1).numpy()
        assert np.allclose(w, np.take_along_axis(p, idx.astype(np.int64), 1), rtol=1e-6)
        # Mixtral: softmax over the selected logits == renormalised top-k of the full softmax
        _, w2 = O.topk_route(lg, k, O.MODE_TOPK_SOFTMAX)
        _, w1 = O.topk_route(lg, k, O.MODE_SOFTMAX_TOPK_RENORM)
        assert np.allclose(w2, w1, rtol=2e-6) and np.allclose(w2.sum(1), 1, atol=1e-6)
    lg = np.full((1, 6), 0.25, np.float32)        # all equal -> the k lowest indices
    assert list(O.topk_route(lg, 3)[0][0]) == [0, 1, 2]
    # selection on logits agrees with torch.topk on the fp32 softmax where values are distinct
    lg = rng.normal(0, 1, (16, 64)).astype(np.float32)
    ti = torch.topk(torch.softmax(torch.from_numpy(lg), 1), 6, dim=1).indices.numpy()
    assert np.array_equal(O.topk_route(lg, 6)[0], ti)


def test_dispatch_invariants_and_bruteforce():
    rng = np.random.default_rng(2)
    for T, k, E in ((1, 6, 64), (7, 2, 4), (0, 3, 8), (50, 4, 60)):
        idx = np.stack([rng.choice(E, k, replace=False) for _ in range(T)]).astype(np.int32) if T else np.zeros((0, k), np.int32)
        c, off, sp, pp = O.dispatch(idx, E)
        P = T * k
        assert c.sum() == P and off[0] == 0 and off[-1] == P and np.array_equal(np.diff(off), c)
        assert sorted(sp) == list(range(P)) and np.array_equal(sp[pp], np.arange(P))
        flat = idx.reshape(-1)
        brute = sorted(range(P), key=lambda p: (int(flat[p]), p))   # stable by construction
        assert list(sp) == brute
        assert np.all(np.diff(flat[sp]) >= 0)


def test_int4_roundtrip_closed_form_and_hand_block():
    rng = np.random.default_rng(3)
    w = rng.normal(0, 0.02, (16, 256)).astype(np.float32)
    q, s, z = O.quantize_int4(w)
    qw, qz = O.pack_int4(q, z)
    q2, z2 = O.unpack_int4(qw, qz, 16, 256)
    assert np.array_equal(q, q2) and np.array_equal(z, z2)
    deq = O.dequant_int4(qw, s, qz, 16, 256)
    assert np.abs(deq - w).max() <= 0.51 * s.astype(np.float32).max()      # within half a step
    # hand-built: row 0 group 1 has q = 0..15 repeating, z = 3, s = 0.5 -> w = (q-3)/2
    q = np.zeros((1, 256), np.uint8); q[0, 128:] = np.arange(128) % 16
    z = np.array([[0, 3]], np.uint8); s = np.array([[1.0, 0.5]], np.float16)
    qw, qz = O.pack_int4(q, z)
    assert qw.view(np.uint32)[0, 16] == 0x76543210 and qw.view(np.uint32)[0, 17] == 0xFEDCBA98   # low nibble first
    assert qz.view(np.uint32)[0] == 0x30
    d = O.dequant_int4(qw, s, qz, 1, 256)
    assert np.array_equal(d[0, :128], np.zeros(128)) and np.array_equal(d[0, 128:144], (np.arange(16) - 3) / 2)


def test_q4k_known_answer_blocks():
    blk = np.zeros(144, np.uint8)
    assert np.array_equal(O.dequant_q4k_block(blk), np.zeros(256, np.float32))        # all-zero block
    # d = 2, dmin = 1, every sub-block scale 3 / min 5, every nibble 7 -> 2*3*7 - 1*5 = 37
    blk[0:2] = np.array([2.0], np.float16).view(np.uint8)
    blk[2:4] = np.array([1.0], np.float16).view(np.uint8)
    blk[4:16] = O.q4k_pack_scales(np.full(8, 3), np.full(8, 5))
    blk[16:] = 0x77
    assert np.array_equal(O.dequant_q4k_block(blk), np.full(256, 37, np.float32))
    # 6-bit fields above 15 use the split encoding; a single nibble lands where ggml puts it
    sc = np.array([1, 2, 3, 4, 63, 33, 17, 48]); mn = np.array([0, 9, 8, 7, 40, 63, 16, 1])
    packed = O.q4k_pack_scales(sc, mn)
    s2, m2 = O.q4k_unpack_scales(packed)
    assert np.array_equal(s2, sc) and np.array_equal(m2, mn)
    blk[4:16] = packed
    blk[16:] = 0
    blk[16 + 32 * 2 + 5] = 0xA0          # chunk 2, byte 5, HIGH nibble -> weight 64*2 + 32 + 5, sub-block 5
    w = O.dequant_q4k_block(blk)
    assert w[165] == 2.0 * 33 * 10 - 1.0 * 63
    assert w[164] == -63.0 and w[133] == -40.0 and w[0] == 0.0
    # vectorised form == block form, and the quantiser produces valid blocks close to the input
    rng = np.random.default_rng(4)
    wts = rng.normal(0, 0.02, (4, 512)).astype(np.float32)
    blocks = O.quantize_q4k(wts)
    deq = O.dequant_q4k(blocks, 4, 512)
    assert np.array_equal(deq[1, 256:], O.dequant_q4k_block(blocks[1, 1]))
    assert np.abs(deq - wts).max() < 0.01


def test_swiglu_and_forward_reduce_to_library_routines():
    rng = np.random.default_rng(5)
    H, I, E, T, k = 32, 48, 6, 5, 2
    x = O.round_bf16(rng.normal(0, 1, (T, H)).astype(np.float32))
    wg = O.round_bf16(rng.normal(0, 0.3, (E, H)).astype(np.float32))
    ex = [tuple(rng.normal(0, 0.1, s).astype(np.float32) for s in ((I, H), (I, H), (H, I))) for _ in range(E)]
    sh = tuple(rng.normal(0, 0.1, s).astype(np.float32) for s in ((2 * I, H), (2 * I, H), (H, 2 * I)))
    sg = rng.normal(0, 0.3, H).astype(np.float32)
    r = O.moe_forward(x, wg, ex, k, O.MODE_SOFTMAX_TOPK, shared=sh, shared_gate=sg)
    # dense restatement in float64: every token through its k experts
    out = np.zeros((T, H))
    silu = lambda a: a / (1 + np.exp(-a))
    for t in range(T):
        for j in range(k):
            g, u, d = (m.astype(np.float64) for m in ex[r["idx"][t, j]])
            out[t] += r["w"][t, j] * (d @ (silu(g @ x[t]) * (u @ x[t])))
        g, u, d = (m.astype(np.float64) for m in sh)
        out[t] += (d @ (silu(g @ x[t]) * (u @ x[t]))) / (1 + np.exp(-(sg.astype(np.float64) @ x[t])))
    assert np.allclose(r["out"], out, rtol=1e-4, atol=1e-5)
    # linearity of the combine: scaling the routed weights scales the routed part
    r0 = O.moe_forward(x, wg, ex, k, O.MODE_SOFTMAX_TOPK)
    assert np.allclose(O.moe_forward(x, wg, ex, k, O.MODE_SOFTMAX_TOPK, expert_order=list(range(E))[::-1])["out"],
                       r0["out"], rtol=1e-5, atol=1e-6)      # expert order only changes rounding
    # k = E with renormalisation: weights sum to one
    assert np.allclose(O.topk_route(r["logits"], E, O.MODE_SOFTMAX_TOPK_RENORM)[1].sum(1), 1, atol=1e-6)
