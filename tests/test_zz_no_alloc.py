"""The entry point that allocates nothing (moe_decode_token_int4_noalloc: its workspaces live in a device
array inside the library) against moe_decode_token_int4 with caller workspaces, through the C ABI: the same
kernels on the same inputs, so y must be equal bit for bit.  Two calls in a row, the second on a smaller
layer (the array keeps the first call's contents); a selected expert without a slot raises the caller's
error word; shapes beyond the array are refused."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from promoe_amd import _lib as L
from tests.synth import Int4Layer

pytestmark = pytest.mark.gpu
TOL = 2e-2


def bf16_dev(a, dev):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16).to(dev)


def one_case(layer, k, mode, gated, dev, seed):
    from promoe_amd import ops
    H, I, E, I_sh = layer.H, layer.I, layer.E, layer.I_sh
    slots = [torch.from_numpy(s).to(dev) for s in layer.slots]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=dev)
    shared = torch.from_numpy(layer.shared_img).to(dev) if I_sh else None
    wg_np = layer.wg if not gated else np.concatenate([layer.wg, layer.shared_gate[None, :]], axis=0)
    wg = bf16_dev(wg_np, dev)
    bias = None if layer.bias is None else torch.from_numpy(
        np.concatenate([layer.bias, np.zeros(wg_np.shape[0] - E, np.float32)])).to(dev)
    x = O.synth_acts(1, H, seed=seed)
    xd = bf16_dev(x, dev)
    logits = ops.gate_logits(xd, wg, bias)
    sg = logits[:, E] if gated else None
    # the existing entry point, every workspace a caller tensor
    unit_ws = torch.zeros(32 * k, dtype=torch.uint8, device=dev)
    y_ref = torch.full((1, H), float("nan"), dtype=torch.bfloat16, device=dev)
    ws = ops.decode_token_int4(xd, logits, E, k, mode, table, shared, H, I, I_sh, phases=5, unit_ws=unit_ws,
                               sg_logit=sg, y=y_ref)
    # the entry point without workspaces
    y = torch.full((1, H), float("nan"), dtype=torch.bfloat16, device=dev)
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    ops.decode_token_int4_noalloc(xd, logits, E, k, mode, table, shared, H, I, I_sh, y, err, sg_logit=sg)
    torch.cuda.synchronize()
    assert int(ws[5].cpu()[0]) == 0 and int(err.cpu()[0]) == 0
    assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16))          # bit for bit
    lg = O.gate_logits_ordered(x, layer.wg)
    if layer.bias is not None:
        lg = (lg + layer.bias[None, :]).astype(np.float32)
    ref = O.moe_forward(x, layer.wg, layer.experts_fp32, k, mode, shared=layer.shared_fp32,
                        shared_gate=layer.shared_gate, logits=lg)
    a = y.float().cpu().numpy()
    assert np.abs(a - ref["out"]).max() <= TOL * np.abs(ref["out"]).max()
    return table, shared, xd, logits, sg


def test_no_alloc_entry_point_equals_the_workspace_one(cuda):
    from promoe_amd import ops
    print("case no-alloc entry point, DeepSeek-shaped layer then a smaller one", flush=True)
    assert 0 < L.lib.moe_noalloc_scratch_bytes() <= 160 * 1024
    big = Int4Layer(H=2048, I=1408, E=16, I_sh=2816, seed=21, zipf=1.2)
    small = Int4Layer(H=256, I=384, E=8, I_sh=256, seed=22, shared_gate=True)
    one_case(big, 6, 0, False, cuda, seed=1)
    # second call in a row, smaller in every dimension, other routing convention, gated shared expert
    table, shared, xd, logits, sg = one_case(small, 2, 2, True, cuda, seed=2)
    # and the big one again: whatever the small call left in the array does not leak into this result
    one_case(big, 6, 0, False, cuda, seed=3)
    # a selected expert without a slot: the caller's error word is raised
    y = torch.zeros(1, 256, dtype=torch.bfloat16, device=cuda)
    err = torch.zeros(1, dtype=torch.int32, device=cuda)
    ops.decode_token_int4_noalloc(xd, logits, 8, 2, 2, torch.zeros_like(table), shared, 256, 384, 256, y, err, sg_logit=sg)
    torch.cuda.synchronize()
    assert int(err.cpu()[0]) == 1
    # beyond the array: refused with a clear error, nothing launched
    with pytest.raises(L.MoeError, match="beyond the static scratch"):
        ops.decode_token_int4_noalloc(xd, logits, 8, 2, 2, table, shared, 256, 36864, 256, y, err, sg_logit=sg)
    with pytest.raises(L.MoeError, match="beyond the static scratch"):
        ops.decode_token_int4_noalloc(xd, logits, 300, 2, 2, table, shared, 256, 384, 256, y, err, sg_logit=sg)


def test_no_alloc_entry_point_in_a_replayed_graph(cuda):
    """What the entry point is for: a caller under HIP graph capture.  The gate logits and the entry point are
    recorded once and replayed for three different inputs, with eager work and synchronisations between the
    replays; every replay must equal the eager workspace entry point bit for bit."""
    from promoe_amd import ops
    print("case no-alloc entry point recorded into a HIP graph and replayed", flush=True)
    layer = Int4Layer(H=2048, I=1408, E=16, I_sh=2816, seed=23, zipf=1.2)
    H, I, E, I_sh, k, mode = layer.H, layer.I, layer.E, layer.I_sh, 6, 0
    slots = [torch.from_numpy(s).to(cuda) for s in layer.slots]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=cuda)
    shared = torch.from_numpy(layer.shared_img).to(cuda)
    wg = bf16_dev(layer.wg, cuda)
    bias = None if layer.bias is None else torch.from_numpy(layer.bias).to(cuda)
    xd = bf16_dev(O.synth_acts(1, H, seed=30), cuda)
    logits = ops.gate_logits(xd, wg, bias)
    y = torch.zeros(1, H, dtype=torch.bfloat16, device=cuda)
    err = torch.zeros(1, dtype=torch.int32, device=cuda)
    # once eagerly: the library looks up its array's address on the first call on a device
    ops.decode_token_int4_noalloc(xd, logits, E, k, mode, table, shared, H, I, I_sh, y, err)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side, capture_error_mode="thread_local"):
            ops.gate_logits(xd, wg, bias, out=logits)
            ops.decode_token_int4_noalloc(xd, logits, E, k, mode, table, shared, H, I, I_sh, y, err)
    torch.cuda.synchronize()
    unit_ws = torch.zeros(32 * k, dtype=torch.uint8, device=cuda)
    for seed in (31, 32, 33):
        x_new = bf16_dev(O.synth_acts(1, H, seed=seed), cuda)
        xd.copy_(x_new)                                    # eager work between the replays
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        lg_ref = ops.gate_logits(x_new, wg, bias)
        y_ref = torch.full((1, H), float("nan"), dtype=torch.bfloat16, device=cuda)
        ws = ops.decode_token_int4(x_new, lg_ref, E, k, mode, table, shared, H, I, I_sh, phases=5, unit_ws=unit_ws,
                                   y=y_ref)
        torch.cuda.synchronize()
        assert int(ws[5].cpu()[0]) == 0 and int(err.cpu()[0]) == 0
        assert torch.equal(logits, lg_ref)
        assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16)), seed
