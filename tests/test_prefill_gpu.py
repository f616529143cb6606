"""Parity of the MFMA prefill expert kernels (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.synth import Bf16Layer, Int4Layer, Q4KLayer

pytestmark = pytest.mark.gpu

TOL = 2e-2  # max |y - ref| / max |ref|


def bf16_dev(a, dev):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16).to(dev)


def run_prefill_gpu(layer, x, k, mode, dev, resident=None):
    from promoe_amd import ops, _lib as L
    H, I, E, I_sh = layer.H, layer.I, layer.E, layer.I_sh
    T = x.shape[0]
    xd = bf16_dev(x, dev)
    wg = layer.wg
    if layer.shared_gate is not None:
        wg = np.concatenate([wg, layer.shared_gate[None, :]], axis=0)
    bias = None
    if layer.bias is not None:
        bias = torch.from_numpy(np.concatenate([layer.bias, np.zeros(wg.shape[0] - E, np.float32)])).to(dev)
    logits = ops.gate_logits(xd, bf16_dev(wg, dev), bias)
    idx, w = ops.topk(logits, k, mode, E=E)
    d = ops.dispatch(idx, E)
    slots = [torch.from_numpy(s).to(dev) for s in layer.slots]
    table = torch.tensor([0 if (resident is not None and e not in resident) else slots[e].data_ptr()
                          for e in range(E)], dtype=torch.int64, device=dev)
    shared = torch.from_numpy(layer.shared_img).to(dev) if I_sh else None
    fmt = L.FMT_BF16 if isinstance(layer, Bf16Layer) else (L.FMT_Q4K if isinstance(layer, Q4KLayer) else L.FMT_INT4_G128)
    part_r, part_s, err, h_r, h_s, _ = ops.experts_prefill(xd, d, table, shared, H, I, I_sh, fmt)
    sg = logits[:, E] if layer.shared_gate is not None else None
    y = ops.combine(part_r, part_s, w, d.pos_of_pair, sg, T, H, k)
    torch.cuda.synchronize()
    return dict(y=y.float().cpu().numpy(), idx=idx.cpu().numpy(), w=w.cpu().numpy(),
                logits=logits.cpu().numpy(), err=int(err.cpu()[0]), d=d)


def check_prefill(layer, T, k, mode, dev, seed=1):
    x = O.synth_acts(T, layer.H, seed=seed)
    got = run_prefill_gpu(layer, x, k, mode, dev)
    lg = O.gate_logits_ordered(x, layer.wg)
    if layer.bias is not None:
        lg = (lg + layer.bias[None, :]).astype(np.float32)
    ref = O.moe_forward(x, layer.wg, layer.experts_fp32, k, mode, shared=layer.shared_fp32,
                        shared_gate=layer.shared_gate, logits=lg)
    assert got["err"] == 0
    assert np.array_equal(got["idx"], ref["idx"])
    _, _, sp, _ = O.dispatch(ref["idx"], layer.E)
    assert np.array_equal(got["d"].sorted_pair.cpu().numpy()[:T * k], sp)
    err = np.abs(got["y"] - ref["out"]).max() / np.abs(ref["out"]).max()
    print(f"  T={T} k={k} mode={mode} max-rel-err={err:.3e}", flush=True)
    assert err <= TOL
    return err


@pytest.mark.parametrize("T", [1, 17, 128, 129, 300, 700])
def test_prefill_layer_small(cuda, T):
    print(f"case prefill_small T={T}", flush=True)
    check_prefill(Bf16Layer(H=256, I=384, E=8, I_sh=256, seed=3), T, 2, 0, cuda)


def test_prefill_layer_small_variants(cuda):
    print("case prefill_small_variants", flush=True)
    # no shared expert, Mixtral routing
    check_prefill(Bf16Layer(H=512, I=128, E=8, I_sh=0, seed=4), 200, 2, 2, cuda)
    # sigmoid-gated shared expert, renormalised routing, Zipf bias: some experts get no token
    check_prefill(Bf16Layer(H=256, I=256, E=60, I_sh=512, seed=5, shared_gate=True, zipf=1.4), 150, 4, 1, cuda)
    # more units than one scan pass is not needed (E <= 1024), K not a multiple of 128
    check_prefill(Bf16Layer(H=768, I=640, E=4, I_sh=128, seed=6), 260, 2, 0, cuda)


def test_prefill_non_resident_expert_is_reported(cuda):
    print("case prefill_non_resident", flush=True)
    layer = Bf16Layer(H=256, I=128, E=4, I_sh=0, seed=7)
    got = run_prefill_gpu(layer, O.synth_acts(64, 256), 2, 0, cuda, resident={0, 1})
    assert got["err"] == 1


def test_prefill_layer_qwen_shape(cuda):
    print("case prefill_qwen T=2048", flush=True)
    # Qwen1.5-MoE-A2.7B layer: H 2048, 60 experts x I 1408, top-4, sigmoid-gated shared expert I 5632
    layer = Bf16Layer(H=2048, I=1408, E=60, I_sh=5632, seed=0, shared_gate=True)
    check_prefill(layer, 2048, 4, 0, cuda)


# ---- int4-g128 experts through the same entry point ----

@pytest.mark.parametrize("T", [1, 17, 96, 97, 193, 400, 700])
def test_prefill_int4_layer_small(cuda, T):
    print(f"case prefill_int4_small T={T}", flush=True)
    check_prefill(Int4Layer(H=256, I=384, E=8, I_sh=256, seed=3), T, 2, 0, cuda)


def test_prefill_int4_layer_small_variants(cuda):
    print("case prefill_int4_small_variants", flush=True)
    check_prefill(Int4Layer(H=512, I=128, E=8, I_sh=0, seed=4), 200, 2, 2, cuda)
    check_prefill(Int4Layer(H=256, I=256, E=60, I_sh=512, seed=5, shared_gate=True, zipf=1.4), 150, 4, 1, cuda)
    check_prefill(Int4Layer(H=768, I=640, E=4, I_sh=128, seed=6), 260, 2, 0, cuda)


def test_prefill_int4_non_resident_expert_is_reported(cuda):
    print("case prefill_int4_non_resident", flush=True)
    layer = Int4Layer(H=256, I=128, E=4, I_sh=0, seed=7)
    got = run_prefill_gpu(layer, O.synth_acts(64, 256), 2, 0, cuda, resident={0, 1})
    assert got["err"] == 1


def test_prefill_int4_deepseek_shape(cuda):
    print("case prefill_int4_deepseek T=512", flush=True)
    # DeepSeek-MoE-16B layer shape; 16 experts instead of 64 keeps host-side quantisation short
    layer = Int4Layer(H=2048, I=1408, E=16, I_sh=2816, seed=0, zipf=1.2)
    check_prefill(layer, 512, 6, 0, cuda)


# ---- q4_K experts ----

@pytest.mark.parametrize("T", [1, 17, 97, 193, 400])
def test_prefill_q4k_layer_small(cuda, T):
    print(f"case prefill_q4k_small T={T}", flush=True)
    check_prefill(Q4KLayer(H=256, I=512, E=8, I_sh=256, seed=3), T, 2, 0, cuda)


def test_prefill_q4k_variants(cuda):
    print("case prefill_q4k_variants", flush=True)
    check_prefill(Q4KLayer(H=512, I=256, E=8, I_sh=0, seed=4), 200, 2, 2, cuda)
    check_prefill(Q4KLayer(H=256, I=256, E=60, I_sh=512, seed=5, shared_gate=True, zipf=1.1), 515, 8, 0, cuda)


def test_prefill_wide_shared_expert_in_pieces(cuda):
    """A shared expert much wider than the routed ones over few tokens: the w2 pass cuts its reduction into
    windows (moe_prefill_shared_splits) and leaves one piece of partial rows per window for the combine."""
    from promoe_amd import _lib as L
    print("case prefill shared expert in pieces", flush=True)
    assert L.lib.moe_prefill_shared_splits(L.FMT_Q4K, 130, 256, 16384) == 4
    assert L.lib.moe_prefill_shared_splits(L.FMT_INT4_G128, 200, 256, 8192) == 2
    assert L.lib.moe_prefill_shared_splits(L.FMT_BF16, 130, 256, 16384) == 1       # nibble formats only
    assert L.lib.moe_prefill_shared_splits(L.FMT_INT4_G128, 2048, 2048, 2816) == 1  # DeepSeek shape: 22 groups
    assert L.lib.moe_prefill_shared_splits(L.FMT_Q4K, 512, 3584, 20480) == 4        # Qwen2-57B shape
    check_prefill(Q4KLayer(H=256, I=256, E=4, I_sh=16384, seed=6, shared_gate=True), 130, 2, 0, cuda)
    check_prefill(Int4Layer(H=256, I=128, E=4, I_sh=8192, seed=7), 200, 2, 1, cuda)
    check_prefill(Int4Layer(H=512, I=128, E=4, I_sh=8192, seed=8), 70, 2, 0, cuda)   # 1 x 2 tiles: 2 pieces, short last tile
