"""Size-independent properties of the HIP path at the full benchmark shapes (no oracle needed)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _images(kind, n, H, I, dev, gen):
    from promoe_amd import synth
    if kind == "bf16":
        return (torch.randn(n, 3 * I * H, device=dev, generator=gen) * 0.02).to(torch.bfloat16).view(torch.uint8)
    if kind == "q4k":
        return synth.random_q4k_images(n, H, I, dev, gen)
    return synth.random_int4_images(n, H, I, dev, gen)


def _experts(kind, x, d, table, shared, H, I, I_sh):
    from promoe_amd import ops, _lib as L
    fmt = {"int4": L.FMT_INT4_G128, "q4k": L.FMT_Q4K, "bf16": L.FMT_BF16}[kind]
    if kind == "bf16" or x.shape[0] > ops.gemv_max_tokens(fmt):
        return ops.experts_prefill(x, d, table, shared, H, I, I_sh, fmt)[:3]
    if kind == "q4k":
        return ops.experts_decode_q4k(x, d, table, shared, H, I, I_sh)[:3]
    return ops.experts_decode_int4(x, d, table, shared, H, I, I_sh)[:3]


@pytest.mark.parametrize("name,kind,T,H,E,I,k,I_sh", [
    ("deepseek decode", "int4", 16, 2048, 64, 1408, 6, 2816),
    ("deepseek prefill", "int4", 2048, 2048, 64, 1408, 6, 2816),
    ("qwen1.5 prefill", "bf16", 2048, 2048, 60, 1408, 4, 5632),
    ("mixtral decode", "int4", 1, 4096, 8, 14336, 2, 0),
    ("mixtral decode 64 tokens", "int4", 64, 4096, 8, 14336, 2, 0),
    ("deepseek decode 64 tokens", "int4", 64, 2048, 64, 1408, 6, 2816),
    ("mixtral prefill", "int4", 4096, 4096, 8, 14336, 2, 0),
    ("qwen2 decode", "q4k", 3, 3584, 64, 2560, 8, 0),
    ("qwen2 prefill", "q4k", 512, 3584, 64, 2560, 8, 0),
])
def test_identical_experts_collapse_to_one_expert(cuda, name, kind, T, H, E, I, k, I_sh):
    """If every routed expert holds the same weights and the routing weights are renormalised to sum
    to one, the layer output is the output of that one expert (plus the shared expert), whatever the
    routing: y_moe == y_dense with E = 1, k = 1.  Exercises gate, top-k, dispatch, the expert kernels
    through a slot table whose E entries alias one slot, and combine, at the full layer shape."""
    from promoe_amd import ops, _lib as L
    print(f"case identical_experts {name}", flush=True)
    gen = torch.Generator(device=cuda).manual_seed(3)
    x = torch.randn(T, H, device=cuda, generator=gen).to(torch.bfloat16)
    wg = (torch.randn(E, H, device=cuda, generator=gen) * 0.02).to(torch.bfloat16)
    img = _images(kind, 1, H, I, cuda, gen)[0]
    shared = _images(kind, 1, H, I_sh, cuda, gen)[0] if I_sh else None
    table = torch.full((E,), img.data_ptr(), dtype=torch.int64, device=cuda)
    logits = ops.gate_logits(x, wg)
    idx, w = ops.topk(logits, k, L.ROUTE_SOFTMAX_TOPK_RENORM)
    assert torch.allclose(w.sum(1), torch.ones(T, device=cuda), atol=1e-5)
    d = ops.dispatch(idx, E)
    # the dispatch is a bijection of the T*k pairs with counts that add up
    sp = d.sorted_pair.cpu().numpy()[:T * k]
    assert np.array_equal(np.sort(sp), np.arange(T * k)) and int(d.counts.sum()) == T * k
    part_r, part_s, err = _experts(kind, x, d, table, shared, H, I, I_sh)
    y = ops.combine(part_r, part_s, w, d.pos_of_pair, None, T, H, k)
    # dense run: one expert, every token routed to it with weight one
    idx1 = torch.zeros(T, 1, dtype=torch.int32, device=cuda)
    w1 = torch.ones(T, 1, dtype=torch.float32, device=cuda)
    d1 = ops.dispatch(idx1, 1)
    pr1, ps1, err1 = _experts(kind, x, d1, table[:1].contiguous(), shared, H, I, I_sh)
    y1 = ops.combine(pr1, ps1, w1, d1.pos_of_pair, None, T, H, 1)
    torch.cuda.synchronize()
    assert int(err.cpu()[0]) == 0 and int(err1.cpu()[0]) == 0
    a, b = y.float(), y1.float()
    rel = float((a - b).abs().max() / b.abs().max())
    print(f"  max |y_moe - y_dense| / max |y_dense| = {rel:.3e}", flush=True)
    assert torch.isfinite(a).all() and rel <= 1e-2
