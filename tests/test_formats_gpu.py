"""Expert weights read from GPTQ safetensors / GGUF q4_K files, run through the HIP kernels and
compared with the fp32 restatement on the weights the files' formats define."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from promoe_amd import formats as F
from tests.test_formats import _write_gptq_layer, _write_gguf

pytestmark = pytest.mark.gpu
TOL = 2e-2


@pytest.fixture(scope="module")
def cuda():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


def _bf16(a, dev):
    return torch.from_numpy(O.f32_to_bf16_bits(a).view(np.int16)).view(torch.bfloat16).to(dev)


def _run(dev, x, wg, routed, shared, H, I, I_sh, k, fmt, shared_gate=None):
    from promoe_amd import ops
    E = len(routed)
    xd = _bf16(x, dev)
    wg_all = wg if shared_gate is None else np.concatenate([wg, shared_gate[None, :]], axis=0)
    logits = ops.gate_logits(xd, _bf16(wg_all, dev), None)
    idx, w = ops.topk(logits, k, 0, E=E)
    d = ops.dispatch(idx, E)
    slots = [torch.from_numpy(np.ascontiguousarray(s)).to(dev) for s in routed]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=dev)
    sh = torch.from_numpy(np.ascontiguousarray(shared)).to(dev) if shared is not None else None
    if fmt == "q4k":
        pr, ps, err, _, _ = ops.experts_decode_q4k(xd, d, table, sh, H, I, I_sh)
    else:
        pr, ps, err, _, _ = ops.experts_decode_int4(xd, d, table, sh, H, I, I_sh)
    sg = logits[:, E] if shared_gate is not None else None
    y = ops.combine(pr, ps, w, d.pos_of_pair, sg, x.shape[0], H, k)
    torch.cuda.synchronize()
    assert int(err.cpu()[0]) == 0
    return y.float().cpu().numpy(), idx.cpu().numpy()


def test_gptq_file_through_decode_kernels(cuda, tmp_path):
    print("case formats_gptq", flush=True)
    rng = np.random.default_rng(8)
    H, I, I_sh, E, k, T = 256, 128, 256, 4, 2, 3
    a, b = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    deq = _write_gptq_layer(a, b, rng, H, I, I_sh, E, hf_layer=1)
    idx = F.SafetensorsIndex([a, b])
    routed, shared = F.gptq_layer_images(idx, 0, E, H, family="deepseek")
    wg = O.round_bf16(rng.normal(0, 0.02, (E, H)).astype(np.float32))
    x = O.synth_acts(T, H, seed=3)
    y, ridx = _run(cuda, x, wg, routed, shared, H, I, I_sh, k, "int4")
    experts = [tuple(deq[F.EXPERT_PREFIX["deepseek"].format(l=1, e=e)]) for e in range(E)]
    ref = O.moe_forward(x, wg, experts, k, 0, shared=tuple(deq[F.SHARED_PREFIX["deepseek"].format(l=1)]),
                        logits=O.gate_logits_ordered(x, wg))
    assert np.array_equal(ridx, ref["idx"])
    assert np.abs(y - ref["out"]).max() <= TOL * np.abs(ref["out"]).max()


def test_gguf_file_through_decode_kernels(cuda, tmp_path):
    print("case formats_gguf", flush=True)
    rng = np.random.default_rng(9)
    H, I, I_sh, E, k, T = 256, 512, 256, 4, 2, 2

    def blocks(n, kk):
        return O.quantize_q4k(rng.normal(0, 0.02, (n, kk)).astype(np.float32))

    gate = np.stack([blocks(I, H) for _ in range(E)]); up = np.stack([blocks(I, H) for _ in range(E)])
    down = np.stack([blocks(H, I) for _ in range(E)])
    sg, su, sd = blocks(I_sh, H), blocks(I_sh, H), blocks(H, I_sh)
    wg = O.round_bf16(rng.normal(0, 0.02, (E, H)).astype(np.float32))
    wsg = O.round_bf16(rng.normal(0, 0.02, (H,)).astype(np.float32))
    tensors = [("blk.0.ffn_gate_inp.weight", (H, E), F.GGML_F32, wg.tobytes()),
               ("blk.0.ffn_gate_exps.weight", (H, I, E), F.GGML_Q4_K, gate.tobytes()),
               ("blk.0.ffn_up_exps.weight", (H, I, E), F.GGML_Q4_K, up.tobytes()),
               ("blk.0.ffn_down_exps.weight", (I, H, E), F.GGML_Q4_K, down.tobytes()),
               ("blk.0.ffn_gate_shexp.weight", (H, I_sh), F.GGML_Q4_K, sg.tobytes()),
               ("blk.0.ffn_up_shexp.weight", (H, I_sh), F.GGML_Q4_K, su.tobytes()),
               ("blk.0.ffn_down_shexp.weight", (I_sh, H), F.GGML_Q4_K, sd.tobytes()),
               ("blk.0.ffn_gate_inp_shexp.weight", (H,), F.GGML_F32, wsg.tobytes())]
    path = str(tmp_path / "m.gguf")
    _write_gguf(path, {"general.architecture": (8, "qwen2moe")}, tensors)
    lay = F.gguf_layer_images(F.GGUFFile(path), 0)
    x = O.synth_acts(T, H, seed=4)
    y, ridx = _run(cuda, x, lay["gate_w"], lay["routed"], lay["shared"], H, I, I_sh, k, "q4k", shared_gate=lay["shared_gate"])
    experts = [(O.dequant_q4k(gate[e], I, H), O.dequant_q4k(up[e], I, H), O.dequant_q4k(down[e], H, I)) for e in range(E)]
    shared = (O.dequant_q4k(sg, I_sh, H), O.dequant_q4k(su, I_sh, H), O.dequant_q4k(sd, H, I_sh))
    ref = O.moe_forward(x, wg, experts, k, 0, shared=shared, shared_gate=wsg, logits=O.gate_logits_ordered(x, wg))
    assert np.array_equal(ridx, ref["idx"])
    assert np.abs(y - ref["out"]).max() <= TOL * np.abs(ref["out"]).max()


def test_gguf_file_through_the_cache_engine(cuda, tmp_path):
    """Two q4_K layers from a GGUF file, half of the experts resident: file -> images -> slot cache ->
    moe_forward, against the fp32 restatement on the weights the block bytes define."""
    print("case formats_gguf_engine", flush=True)
    rng = np.random.default_rng(10)
    H, I, E, k = 256, 256, 8, 2

    def blocks(n, kk):
        return O.quantize_q4k(rng.normal(0, 0.02, (n, kk)).astype(np.float32))

    tensors, ref_layers = [], []
    for l in range(2):
        gate = np.stack([blocks(I, H) for _ in range(E)]); up = np.stack([blocks(I, H) for _ in range(E)])
        down = np.stack([blocks(H, I) for _ in range(E)])
        wg = O.round_bf16(rng.normal(0, 0.05, (E, H)).astype(np.float32))
        p = "blk.%d." % l
        tensors += [(p + "ffn_gate_inp.weight", (H, E), F.GGML_F32, wg.tobytes()),
                    (p + "ffn_gate_exps.weight", (H, I, E), F.GGML_Q4_K, gate.tobytes()),
                    (p + "ffn_up_exps.weight", (H, I, E), F.GGML_Q4_K, up.tobytes()),
                    (p + "ffn_down_exps.weight", (I, H, E), F.GGML_Q4_K, down.tobytes())]
        ref_layers.append((wg, [(O.dequant_q4k(gate[e], I, H), O.dequant_q4k(up[e], I, H), O.dequant_q4k(down[e], H, I))
                                for e in range(E)]))
    path = str(tmp_path / "two.gguf")
    _write_gguf(path, {"general.architecture": (8, "mixtral")}, tensors)
    g = F.GGUFFile(path)
    assert g.moe_layers() == [0, 1]
    pm = F.engine_from_images([F.gguf_layer_images(g, l) for l in g.moe_layers()], "q4k", k, 2, cuda,
                              cache_rate=0.5, cache_policy="lru")
    try:
        for step, T in enumerate([1, 3, 1, 20]):
            for l in range(2):
                x = O.synth_acts(T, H, seed=50 + 2 * step + l)
                y = pm.forward(l, _bf16(x, cuda))
                torch.cuda.synchronize()
                wg, experts = ref_layers[l]
                ref = O.moe_forward(x, wg, experts, k, 2, logits=O.gate_logits_ordered(x, wg))
                err = np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()
                assert err <= TOL, (step, l, err)
        c = pm.counters()
        assert c["miss"] > 0 and c["hit"] > 0
    finally:
        pm.close()
