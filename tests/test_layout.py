"""The slot layout written by promoe_amd.layout, read back exactly as the header
documents it, must reproduce the oracle's dequantised weights bit for bit."""
import numpy as np

from oracle import moe_oracle as O
from promoe_amd import layout as LY


def read_tiles(buf, off_q, off_s, off_z, N, K):
    """Decode a tiled matrix following include/moe_kernels.h (independent of the packer)."""
    G = K // 128
    q = np.frombuffer(buf, np.uint32, count=N * K // 8, offset=off_q).reshape(N // 16, G, 64, 4)
    s = np.frombuffer(buf, np.float16, count=N * G, offset=off_s).reshape(N // 16, G, 16)
    z = np.frombuffer(buf, np.uint8, count=N * G // 2, offset=off_z).reshape(N // 16, G, 8)
    W = np.zeros((N, K), np.float32)
    for lane in range(64):
        r, qd = lane & 15, lane >> 4
        zz = ((z[:, :, r // 2] >> (4 * (r & 1))) & 15).astype(np.float32)
        ss = s[:, :, r].astype(np.float32)
        for j in range(4):
            dw = q[:, :, lane, j]
            for i in range(8):
                sh = 2 * i if i % 2 == 0 else 16 + 2 * (i - 1)
                qq = ((dw >> np.uint32(sh)) & np.uint32(15)).astype(np.float32)
                k = np.arange(G) * 128 + 32 * qd + 8 * j + i
                n = np.arange(N // 16) * 16 + r
                W[n[:, None], k[None, :]] = (qq - zz) * ss
    return W


def test_pack_expert_matches_oracle_dequant():
    H, I = 256, 384
    rng = np.random.default_rng(0)
    mats = {}
    ex = {}
    for name, (n, k) in (("gate", (I, H)), ("up", (I, H)), ("down", (H, I))):
        w = rng.normal(0, 0.02, (n, k)).astype(np.float32)
        q, s, z = O.quantize_int4(w)
        qw, qz = O.pack_int4(q, z)
        ex[name] = (qw, s, qz)
        mats[name] = O.dequant_int4(qw, s, qz, n, k)
    img = LY.pack_expert_int4(ex["gate"], ex["up"], ex["down"], H, I)
    lay = LY.int4_layout(H, I)
    assert img.size == lay["total_bytes"] == 3 * I * H // 2 + 3 * I * H // 128 * 2 + 3 * I * H // 128 // 2
    w13 = read_tiles(img.tobytes(), lay["off13_q"], lay["off13_s"], lay["off13_z"], 2 * I, H)
    w13 = w13.reshape(I // 16, 2, 16, H)
    assert np.array_equal(w13[:, 0].reshape(I, H), mats["gate"])
    assert np.array_equal(w13[:, 1].reshape(I, H), mats["up"])
    w2 = read_tiles(img.tobytes(), lay["off2_q"], lay["off2_s"], lay["off2_z"], H, I)
    assert np.array_equal(w2, mats["down"])


def test_layout_sizes_match_published_shapes():
    # DeepSeek-MoE-16B expert: 4,494,336 bytes; Mixtral: 91,521,024
    assert LY.int4_layout(2048, 1408)["total_bytes"] == 4494336
    assert LY.int4_layout(4096, 14336)["total_bytes"] == 91521024
    chunks = LY.split_chunks_int4(2048, 1408)
    assert sum(c[2] for c in chunks) == 4494336 and chunks[0][1] == 0


def test_product_quantizer_matches_oracle_quantizer():
    import torch
    from promoe_amd.quant import quantize_int4
    rng = np.random.default_rng(1)
    w = rng.normal(0, 0.02, (48, 384)).astype(np.float32)
    q, s, z = O.quantize_int4(w)
    qw, qz = O.pack_int4(q, z)
    pw, ps, pz = quantize_int4(torch.from_numpy(w))
    assert np.array_equal(ps.view(np.uint16), s.view(np.uint16))
    assert np.array_equal(pw, qw) and np.array_equal(pz, qz)


def test_q4k_repack_keeps_every_field():
    """The q4_K slot image holds the same numbers as the ggml blocks: dequantising from the
    repacked sections reproduces the oracle's dequantisation bit for bit."""
    import numpy as np
    from oracle import moe_oracle as O
    from promoe_amd import layout as LY
    rng = np.random.default_rng(0)
    N, K = 32, 512
    blocks = O.quantize_q4k(rng.normal(0, 0.02, (N, K)).astype(np.float32))
    ref = O.dequant_q4k(blocks, N, K)
    qt, st, zt = LY.tile_q4k(blocks, N, K)
    G = K // 128
    dw = qt.view(np.uint32).reshape(N // 16, G, 4, 16, 4)          # [rb, g, qd, r, j]
    sm = st.view(np.uint16).reshape(N // 16, G, 4, 16)             # [rb, g, qd, r]
    dd = zt.view(np.uint32).reshape(N // 16, G // 2, 16)           # [rb, sb, r]
    out = np.zeros((N, K), np.float32)
    shift = [0, 16, 4, 20, 8, 24, 12, 28]
    for rb in range(N // 16):
        for g in range(G):
            for qd in range(4):
                for r in range(16):
                    d = np.array([dd[rb, g // 2, r] & 0xffff], np.uint16).view(np.float16)[0].astype(np.float32)
                    dmin = np.array([dd[rb, g // 2, r] >> 16], np.uint16).view(np.float16)[0].astype(np.float32)
                    sc, mn = np.float32(sm[rb, g, qd, r] & 0xff), np.float32(sm[rb, g, qd, r] >> 8)
                    for j in range(4):
                        for i in range(8):
                            q = np.float32((dw[rb, g, qd, r, j] >> np.uint32(shift[i])) & np.uint32(15))
                            out[16 * rb + r, 128 * g + 32 * qd + 8 * j + i] = d * sc * q - dmin * mn
    assert np.array_equal(out, ref)
