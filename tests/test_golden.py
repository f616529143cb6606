"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from the oracle):
the oracle must keep reproducing them bit for bit, and the HIP path must match them."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = 2e-2


def load(name):
    return np.load(os.path.join(G, name), allow_pickle=False)


def test_oracle_reproduces_routing_fixture():
    f = load("routing_T5_H256_E60_k4.npz")
    logits = O.gate_logits_ordered(f["x"], f["wg"])
    assert np.array_equal(logits.view(np.uint32), f["logits"].view(np.uint32))
    for mode in (0, 1, 2):
        idx, w = O.topk_route(logits, 4, mode)
        assert np.array_equal(idx, f["idx_m%d" % mode])
        assert np.array_equal(w.view(np.uint32), f["w_m%d" % mode].view(np.uint32))
    # the tie between experts 1 and 3 resolves to the lower index wherever both are candidates
    for t in range(5):
        row = list(f["idx_m0"][t])
        if 3 in row:
            assert 1 in row and row.index(1) < row.index(3)
    counts, offsets, sp, pp = O.dispatch(f["idx_m0"], 60)
    for a, b in ((counts, "counts"), (offsets, "offsets"), (sp, "sorted_pair"), (pp, "pos_of_pair")):
        assert np.array_equal(a, f[b]), b


@pytest.mark.gpu
def test_hip_routing_matches_fixture(cuda):
    from promoe_amd import ops
    f = load("routing_T5_H256_E60_k4.npz")
    x = torch.from_numpy(f["x"]).to(torch.bfloat16).to(cuda)
    wg = torch.from_numpy(f["wg"]).to(torch.bfloat16).to(cuda)
    logits = ops.gate_logits(x, wg)
    assert np.array_equal(logits.cpu().numpy().view(np.uint32), f["logits"].view(np.uint32))
    for mode in (0, 1, 2):
        idx, w = ops.topk(logits, 4, mode)
        assert np.array_equal(idx.cpu().numpy(), f["idx_m%d" % mode])
        assert np.allclose(w.cpu().numpy(), f["w_m%d" % mode], rtol=2e-6, atol=1e-9)
    idx, _ = ops.topk(logits, 4, 0)
    d = ops.dispatch(idx, 60)
    assert np.array_equal(d.counts.cpu().numpy(), f["counts"])
    assert np.array_equal(d.offsets.cpu().numpy(), f["offsets"])
    assert np.array_equal(d.sorted_pair.cpu().numpy()[:20], f["sorted_pair"])
    assert np.array_equal(d.pos_of_pair.cpu().numpy()[:20], f["pos_of_pair"])
    idx2, w2, d2 = ops.topk_dispatch(logits, 4, 60, 0)
    assert np.array_equal(idx2.cpu().numpy(), f["idx_m0"]) and np.array_equal(d2.sorted_pair.cpu().numpy()[:20], f["sorted_pair"])


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["int4", "q4k", "bf16"])
def test_hip_layer_forward_matches_fixture(cuda, kind):
    """The expert images and expected outputs come from the fixture file alone."""
    from promoe_amd import ops, _lib as L
    f = load("layer_%s_H256_E4_k2.npz" % kind)
    H, E, k = 256, 4, 2
    I = I_sh = 256 if kind == "q4k" else 128
    fmt = {"int4": L.FMT_INT4_G128, "q4k": L.FMT_Q4K, "bf16": L.FMT_BF16}[kind]
    slots = [torch.from_numpy(s.copy()).to(cuda) for s in f["slots"]]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=cuda)
    shared = torch.from_numpy(f["shared_img"].copy()).to(cuda)
    wg = torch.from_numpy(np.concatenate([f["wg"], f["shared_gate"][None, :]])).to(torch.bfloat16).to(cuda)
    bias = torch.from_numpy(np.concatenate([f["bias"], np.zeros(1, np.float32)])).to(cuda)
    for T in (1, 3, 40):
        x = torch.from_numpy(f["x_T%d" % T]).to(torch.bfloat16).to(cuda)
        logits = ops.gate_logits(x, wg, bias)
        idx, w = ops.topk(logits, k, 0, E=E)
        assert np.array_equal(idx.cpu().numpy(), f["idx_T%d" % T])
        d = ops.dispatch(idx, E)
        if kind == "bf16" or T > ops.gemv_max_tokens(fmt):
            part_r, part_s, err = ops.experts_prefill(x, d, table, shared, H, I, I_sh, fmt)[:3]
        elif kind == "q4k":
            part_r, part_s, err = ops.experts_decode_q4k(x, d, table, shared, H, I, I_sh)[:3]
        else:
            part_r, part_s, err = ops.experts_decode_int4(x, d, table, shared, H, I, I_sh)[:3]
        y = ops.combine(part_r, part_s, w, d.pos_of_pair, logits[:, E], T, H, k)
        torch.cuda.synchronize()
        assert int(err.cpu()[0]) == 0
        ref = f["y_T%d" % T]
        e = np.abs(y.float().cpu().numpy() - ref).max() / np.abs(ref).max()
        print(f"  golden {kind} T={T}: max-rel-err {e:.3e}", flush=True)
        assert e <= TOL
