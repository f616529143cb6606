"""On-disk formats -> slot images: GPTQ safetensors and GGUF q4_K (CPU only).

The files are written here from seeded synthetic tensors (no checkpoint can be fetched); what is
checked is that a weight read through the reader dequantises to exactly the value the format's
published formula gives for the bytes in the file."""
import struct

import numpy as np
import pytest

from oracle import moe_oracle as O
from promoe_amd import formats as F
from promoe_amd import layout as LY


def _gptq_linear(rng, K, N, zero_plus_one=True, with_wrap=True):
    """Random GPTQ tensors of one linear layer + the (q, zero, scale) they encode."""
    G = K // 128
    q = rng.integers(0, 16, (K, N), dtype=np.uint32)
    zero = rng.integers(1 if zero_plus_one else 0, 16, (G, N), dtype=np.uint32)
    if with_wrap and zero_plus_one:
        zero[0, :4] = 0              # stored as 15: the v1 kernels wrap 15 + 1 to 0
    scales = (rng.random((G, N)).astype(np.float32) * 0.01 + 0.001).astype(np.float16)
    qweight = np.zeros((K // 8, N), np.uint32)
    for j in range(8):
        qweight |= q[j::8, :] << np.uint32(4 * j)
    stored = (zero - 1) & 0xF if zero_plus_one else zero
    qzeros = np.zeros((G, N // 8), np.uint32)
    for j in range(8):
        qzeros |= stored[:, j::8] << np.uint32(4 * j)
    g_idx = (np.arange(K) // 128).astype(np.int32)
    w = (q.astype(np.float32) - zero[np.arange(K) // 128, :].astype(np.float32)) * \
        scales.astype(np.float32)[np.arange(K) // 128, :]
    return dict(qweight=qweight.view(np.int32), qzeros=qzeros.view(np.int32), scales=scales, g_idx=g_idx), w.T.copy()


@pytest.mark.parametrize("v1", [True, False])
def test_gptq_linear_to_exchange_matches_published_formula(v1):
    rng = np.random.default_rng(3)
    K, N = 256, 48
    t, w = _gptq_linear(rng, K, N, zero_plus_one=v1)
    # the loop restatement of the format agrees with the construction ...
    assert np.array_equal(O.dequant_gptq(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], v1), w)
    # ... and the repacked triple dequantises to the same weights, bit for bit
    qx, sx, zx = F.gptq_to_exchange(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], v1)
    assert np.array_equal(O.dequant_int4(qx, sx, zx, N, K), w)


def test_gptq_rejects_what_the_layout_cannot_hold():
    rng = np.random.default_rng(4)
    t, _ = _gptq_linear(rng, 256, 16)
    perm = t["g_idx"].copy(); perm[[0, 200]] = perm[[200, 0]]
    with pytest.raises(ValueError, match="activation-ordered"):
        F.gptq_to_exchange(t["qweight"], t["qzeros"], t["scales"], perm)
    with pytest.raises(ValueError, match="group size"):
        F.gptq_to_exchange(t["qweight"], t["qzeros"][:1], t["scales"][:1])
    with pytest.raises(ValueError):
        F.gptq_to_exchange(t["qweight"].astype(np.int64), t["qzeros"], t["scales"])


def _write_gptq_layer(path_a, path_b, rng, H, I, I_sh, E, hf_layer, family="deepseek"):
    from safetensors.numpy import save_file
    proj = F.PROJ_NAMES[family]
    tensors, deq = {}, {}
    mods = [(F.EXPERT_PREFIX[family].format(l=hf_layer, e=e), I) for e in range(E)]
    if I_sh:
        mods.append((F.SHARED_PREFIX[family].format(l=hf_layer), I_sh))
    for prefix, inter in mods:
        ws = []
        for name, (K, N) in zip(proj, ((H, inter), (H, inter), (inter, H))):
            t, w = _gptq_linear(rng, K, N)
            for k, v in t.items():
                tensors["%s.%s.%s" % (prefix, name, k)] = v
            ws.append(w)
        deq[prefix] = ws
    names = sorted(tensors)
    save_file({n: tensors[n] for n in names[::2]}, path_a)     # two shards, interleaved
    save_file({n: tensors[n] for n in names[1::2]}, path_b)
    return deq


def test_gptq_safetensors_layer_to_slot_images(tmp_path):
    rng = np.random.default_rng(5)
    H, I, I_sh, E = 256, 128, 256, 3
    a, b = str(tmp_path / "model-00001.safetensors"), str(tmp_path / "model-00002.safetensors")
    deq = _write_gptq_layer(a, b, rng, H, I, I_sh, E, hf_layer=1)     # DeepSeek: MoE layer 0 = checkpoint layer 1
    idx = F.SafetensorsIndex([a, b])
    routed, shared = F.gptq_layer_images(idx, 0, E, H, family="deepseek")
    assert len(routed) == E and shared is not None
    lay = LY.int4_layout(H, I)
    assert all(img.dtype == np.uint8 and img.size == lay["total_bytes"] for img in routed)
    assert shared.size == LY.int4_layout(H, I_sh)["total_bytes"]
    # an image is the packing of the repacked triples: same bytes as packing the format's weights directly
    for e in range(E):
        prefix = F.EXPERT_PREFIX["deepseek"].format(l=1, e=e)
        ex = []
        for name in F.PROJ_NAMES["deepseek"]:
            base = "%s.%s." % (prefix, name)
            ex.append(F.gptq_to_exchange(idx.get(base + "qweight"), idx.get(base + "qzeros"), idx.get(base + "scales"),
                                         idx.get(base + "g_idx")))
        assert np.array_equal(routed[e], LY.pack_expert_int4(ex[0], ex[1], ex[2], H, I))
        for t, w in zip(ex, deq[prefix]):
            N, K = w.shape
            assert np.array_equal(O.dequant_int4(t[0], t[1], t[2], N, K), w)
    with pytest.raises(KeyError):
        F.gptq_layer_images(idx, 0, E + 1, H, family="deepseek")


# ---- GGUF -----------------------------------------------------------------------------------

def _gguf_str(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _write_gguf(path, kvs, tensors, align=32, version=3):
    """tensors: list of (name, ne tuple (innermost first), ggml type, bytes)."""
    out = bytearray(b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(kvs)))
    for key, (t, v) in kvs.items():
        out += _gguf_str(key) + struct.pack("<I", t)
        if t == 8:
            out += _gguf_str(v)
        elif t == 9:
            et, items = v
            out += struct.pack("<IQ", et, len(items))
            for it in items:
                out += _gguf_str(it) if et == 8 else struct.pack(F._SCALAR[et], it)
        else:
            out += struct.pack(F._SCALAR[t], v)
    off = 0
    offs = []
    for name, ne, typ, data in tensors:
        offs.append(off)
        off = (off + len(data) + align - 1) // align * align
    for (name, ne, typ, data), o in zip(tensors, offs):
        out += _gguf_str(name) + struct.pack("<I", len(ne)) + b"".join(struct.pack("<Q", d) for d in ne)
        out += struct.pack("<IQ", typ, o)
    out += b"\0" * ((-len(out)) % align)
    base = len(out)
    for (name, ne, typ, data), o in zip(tensors, offs):
        out += b"\0" * (base + o - len(out))
        out += data
    open(path, "wb").write(bytes(out))


@pytest.mark.parametrize("align", [32, 64])
def test_gguf_q4k_layer_to_slot_images(tmp_path, align):
    rng = np.random.default_rng(6)
    H, I, I_sh, E = 256, 512, 256, 3

    def blocks(n, k):
        return O.quantize_q4k(rng.normal(0, 0.02, (n, k)).astype(np.float32))

    gate = np.stack([blocks(I, H) for _ in range(E)])       # [E, I, H/256, 144]
    up = np.stack([blocks(I, H) for _ in range(E)])
    down = np.stack([blocks(H, I) for _ in range(E)])
    sg, su, sd = blocks(I_sh, H), blocks(I_sh, H), blocks(H, I_sh)
    wg = rng.normal(0, 0.02, (E, H)).astype(np.float32)
    wsg = rng.normal(0, 0.02, (H,)).astype(np.float16)
    kvs = {"general.architecture": (8, "qwen2moe"), "general.alignment": (4, align), "qwen2moe.expert_count": (4, E),
           "tokenizer.ggml.tokens": (9, (8, ["a", "bc", "def"])), "some.floats": (9, (6, [1.0, 2.5])),
           "general.file_type": (4, 15), "x.flag": (7, True), "x.big": (10, 2 ** 40)}
    tensors = [("token_embd.weight", (H, 7), F.GGML_F16, rng.normal(0, 1, (7, H)).astype(np.float16).tobytes()),
               ("blk.0.ffn_gate_inp.weight", (H, E), F.GGML_F32, wg.tobytes()),
               ("blk.0.ffn_gate_exps.weight", (H, I, E), F.GGML_Q4_K, gate.tobytes()),
               ("blk.0.ffn_up_exps.weight", (H, I, E), F.GGML_Q4_K, up.tobytes()),
               ("blk.0.ffn_down_exps.weight", (I, H, E), F.GGML_Q4_K, down.tobytes()),
               ("blk.0.ffn_gate_shexp.weight", (H, I_sh), F.GGML_Q4_K, sg.tobytes()),
               ("blk.0.ffn_up_shexp.weight", (H, I_sh), F.GGML_Q4_K, su.tobytes()),
               ("blk.0.ffn_down_shexp.weight", (I_sh, H), F.GGML_Q4_K, sd.tobytes()),
               ("blk.0.ffn_gate_inp_shexp.weight", (H,), F.GGML_F16, wsg.tobytes()),
               ("blk.1.ffn_down_exps.weight", (256, 16, 1), F.GGML_Q6_K, bytes(210 * 16))]
    path = str(tmp_path / "m.gguf")
    _write_gguf(path, kvs, tensors, align=align)
    g = F.GGUFFile(path)
    assert g.version == 3 and g.metadata["general.architecture"] == "qwen2moe"
    assert g.metadata["tokenizer.ggml.tokens"] == ["a", "bc", "def"] and g.metadata["x.big"] == 2 ** 40
    assert g.moe_layers() == [0]
    lay = F.gguf_layer_images(g, 0)
    assert (lay["H"], lay["I"], lay["I_sh"], lay["E"]) == (H, I, I_sh, E)
    assert np.array_equal(lay["gate_w"], wg)
    assert np.array_equal(lay["shared_gate"], wsg.astype(np.float32))
    for e in range(E):
        assert np.array_equal(lay["routed"][e], LY.pack_expert_q4k(gate[e], up[e], down[e], H, I))
    assert np.array_equal(lay["shared"], LY.pack_expert_q4k(sg, su, sd, H, I_sh))
    # what the reader hands out dequantises to what the block bytes in the file say
    assert np.array_equal(O.dequant_q4k(g.q4k_blocks("blk.0.ffn_down_exps.weight")[1], H, I), O.dequant_q4k(down[1], H, I))
    with pytest.raises(NotImplementedError, match="Q6_K"):
        g.q4k_blocks("blk.1.ffn_down_exps.weight")
    with pytest.raises(KeyError):
        g.raw("blk.9.none")


def test_gguf_rejects_bad_files(tmp_path):
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGML" + bytes(40))
    with pytest.raises(ValueError, match="not a GGUF"):
        F.GGUFFile(str(p))
    p.write_bytes(b"GGUF" + struct.pack("<IQQ", 1, 0, 0))
    with pytest.raises(ValueError, match="version"):
        F.GGUFFile(str(p))
    p.write_bytes(b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + struct.pack("<Q", 1000))
    with pytest.raises(ValueError, match="truncated"):
        F.GGUFFile(str(p))


# ---- Q6_K (the ffn_down tensors of a q4_k_m file) ---------------------------------------------

def _random_q6k_blocks(rng, shape):
    b = rng.integers(0, 256, shape + (210,), dtype=np.uint8)
    b[..., 192:208] = rng.integers(-60, 61, shape + (16,), dtype=np.int8).view(np.uint8)
    d = (rng.random(shape) * 2e-5 + 1e-5).astype(np.float16)
    b[..., 208:210] = d[..., None].view(np.uint8).reshape(shape + (2,))
    return b


def test_oracle_q6k_known_answers():
    """The loop restatement against the closed form of the layout: weight i of a block has scale i // 16,
    low nibble in ql[64 h + 32 (j & 1) + l] (high nibble for j >= 2) and its two high bits at bit 2 j of
    qh[32 h + l], with h = i // 128, j = (i % 128) // 32, l = i % 32; w = d * scale * (q - 32)."""
    blk = np.zeros(210, np.uint8)
    blk[192:208] = np.ones(16, np.int8).view(np.uint8)
    blk[208:210] = np.array([1.0], np.float16).view(np.uint8)
    assert np.array_equal(O.dequant_q6k_block(blk), np.full(256, -32.0, np.float32))     # q = 0 everywhere
    one = blk.copy(); one[0] = 0x0F; one[128] = 0x03                                       # weight 0: q = 63
    y = O.dequant_q6k_block(one)
    assert y[0] == 31.0 and np.all(np.delete(y, 0) == -32.0)
    hi = blk.copy(); hi[64 + 32 + 5] = 0x70; hi[128 + 32 + 5] = 0x80                       # h=1, j=3, l=5: q = 7 | 2<<4
    y = O.dequant_q6k_block(hi)
    assert y[128 + 96 + 5] == float((7 | (2 << 4)) - 32) and np.sum(y != -32.0) == 1
    rng = np.random.default_rng(11)
    for _ in range(4):
        b = _random_q6k_blocks(rng, ())
        ql, qh = b[0:128].astype(int), b[128:192].astype(int)
        sc = b[192:208].view(np.int8).astype(np.float32)
        d = np.float32(b[208:210].view(np.float16)[0])
        want = np.zeros(256, np.float32)
        for i in range(256):
            h, j, l = i // 128, (i % 128) // 32, i % 32
            byte = ql[64 * h + 32 * (j & 1) + l]
            q = ((byte >> 4) if j >= 2 else (byte & 0xF)) | (((qh[32 * h + l] >> (2 * j)) & 3) << 4)
            want[i] = d * sc[i // 16] * np.float32(q - 32)
        assert np.array_equal(O.dequant_q6k_block(b), want)


def test_product_q6k_and_q4k_quantiser_match_the_oracle():
    from promoe_amd import quant as Q
    rng = np.random.default_rng(12)
    b = _random_q6k_blocks(rng, (3, 5, 2))                      # [E, rows, blocks per row]
    got = Q.dequant_q6k(b)
    assert got.shape == (3, 5, 512)
    for e in range(3):
        assert np.array_equal(got[e], O.dequant_q6k(b[e], 5, 512))
    w = rng.normal(0, 0.02, (16, 512)).astype(np.float32)
    w[3, 32:64] = 0.0
    assert np.array_equal(Q.quantize_q4k(w), O.quantize_q4k(w))


def test_gguf_q6k_down_tensors_are_requantised(tmp_path):
    """A q4_k_m-style layer: gate / up in Q4_K, down in Q6_K.  The down tensors reach the slot image as q4_K
    blocks made from their exact Q6_K values; the step is lossy and its size is checked."""
    rng = np.random.default_rng(13)
    H, I, E = 256, 512, 2
    gate = np.stack([O.quantize_q4k(rng.normal(0, 0.02, (I, H)).astype(np.float32)) for _ in range(E)])
    up = np.stack([O.quantize_q4k(rng.normal(0, 0.02, (I, H)).astype(np.float32)) for _ in range(E)])
    down6 = _random_q6k_blocks(rng, (E, H, I // 256))
    wg = rng.normal(0, 0.02, (E, H)).astype(np.float32)
    tensors = [("blk.0.ffn_gate_inp.weight", (H, E), F.GGML_F32, wg.tobytes()),
               ("blk.0.ffn_gate_exps.weight", (H, I, E), F.GGML_Q4_K, gate.tobytes()),
               ("blk.0.ffn_up_exps.weight", (H, I, E), F.GGML_Q4_K, up.tobytes()),
               ("blk.0.ffn_down_exps.weight", (I, H, E), F.GGML_Q6_K, down6.tobytes())]
    path = str(tmp_path / "q4km.gguf")
    _write_gguf(path, {"general.architecture": (8, "qwen2moe")}, tensors)
    g = F.GGUFFile(path)
    lay = F.gguf_layer_images(g, 0)
    for e in range(E):
        exact = O.dequant_q6k(down6[e], H, I)                    # what the file says
        q4 = O.quantize_q4k(exact)
        assert np.array_equal(lay["routed"][e], LY.pack_expert_q4k(gate[e], up[e], q4, H, I))
        back = O.dequant_q4k(q4, H, I)
        rms = float(np.sqrt(np.mean((back - exact) ** 2)) / np.sqrt(np.mean(exact ** 2)))
        assert rms < 0.12, rms
    with pytest.raises(NotImplementedError, match="Q4_K or Q6_K"):
        bad = str(tmp_path / "bad.gguf")
        _write_gguf(bad, {}, [("blk.0.ffn_down_exps.weight", (256, 4, 1), 8, bytes(34 * 32))])
        F.GGUFFile(bad).expert_q4k_blocks("blk.0.ffn_down_exps.weight")
