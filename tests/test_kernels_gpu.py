"""Parity of the HIP kernels (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.synth import Int4Layer, Q4KLayer

pytestmark = pytest.mark.gpu

TOL = 2e-2  # max |y - ref| / max |ref|  (stated output tolerance of the path)


def bf16_dev(a, dev):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16).to(dev)


@pytest.mark.parametrize("T,H,E", [(1, 2048, 64), (4, 2048, 64), (16, 2048, 64), (5, 4096, 8),
                                   (3, 3584, 65), (7, 256, 60), (2, 2048, 61),
                                   (17, 2048, 64), (515, 3584, 65), (300, 4096, 8), (2048, 2048, 61), (33, 256, 3)])
def test_gate_logits_bit_exact(cuda, T, H, E):
    from promoe_amd import ops
    print(f"case gate_logits T={T} H={H} E={E}", flush=True)
    x = O.synth_acts(T, H, seed=1)
    wg = O.round_bf16(O.synth_weights((E, H), seed=0))
    bias = O.zipf_gate_bias(E, 1.2)
    got = ops.gate_logits(bf16_dev(x, cuda), bf16_dev(wg, cuda)).cpu().numpy()
    ref = O.gate_logits_ordered(x, wg)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    got_b = ops.gate_logits(bf16_dev(x, cuda), bf16_dev(wg, cuda), torch.from_numpy(bias).to(cuda)).cpu().numpy()
    assert np.array_equal(got_b.view(np.uint32), (ref + bias[None, :]).astype(np.float32).view(np.uint32))
    # and the order-free product agrees to fp32 rounding
    assert np.allclose(got, (x.astype(np.float64) @ wg.astype(np.float64).T), rtol=0, atol=1e-4)


@pytest.mark.parametrize("T,H,E,E2", [(1, 2048, 65, 640), (1, 2048, 64, 192), (3, 256, 8, 5), (16, 4096, 8, 70)])
def test_gate_logits_pair_bit_exact(cuda, T, H, E, E2):
    """Two matrices in one launch (the predictor's score rows behind the gate's): the bits of two launches."""
    from promoe_amd import ops
    print(f"case gate_logits_pair T={T} H={H} E={E} E2={E2}", flush=True)
    x = bf16_dev(O.synth_acts(T, H, seed=4), cuda)
    wg = bf16_dev(O.round_bf16(O.synth_weights((E, H), seed=5)), cuda)
    wg2 = bf16_dev(O.round_bf16(O.synth_weights((E2, H), seed=6)), cuda)
    b2 = torch.from_numpy(np.linspace(-1, 1, E2).astype(np.float32)).to(cuda)
    a, b = ops.gate_logits_pair(x, wg, None, wg2, b2)
    assert torch.equal(a, ops.gate_logits(x, wg)) and torch.equal(b, ops.gate_logits(x, wg2, b2))


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("T,E,k", [(1, 64, 6), (16, 64, 6), (33, 60, 4), (5, 8, 2), (9, 64, 8), (4, 200, 8)])
def test_topk_routing(cuda, T, E, k, mode):
    from promoe_amd import ops
    print(f"case topk T={T} E={E} k={k} mode={mode}", flush=True)
    rng = np.random.default_rng(T * 1000 + E + k)
    logits = rng.normal(0, 2, (T, E)).astype(np.float32)
    # constructed ties: duplicate values inside rows, including at the k-th boundary
    logits[:, E // 2] = logits[:, 1]
    if T > 2:
        logits[2, :] = 0.5
    idx, w = ops.topk(torch.from_numpy(logits).to(cuda), k, mode)
    ridx, rw = O.topk_route(logits, k, mode)
    assert np.array_equal(idx.cpu().numpy(), ridx)
    assert np.allclose(w.cpu().numpy(), rw, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("T,k,E,single", [(1, 6, 64, False), (4, 6, 64, False), (16, 6, 64, False),
                                          (2048, 4, 60, False), (4096, 2, 8, False), (515, 8, 64, False),
                                          (300, 3, 200, False), (0, 6, 64, False),
                                          # P >= 2048 pairs, E <= 256: one workgroup per 1024 pairs (ragged last one)
                                          (342, 6, 64, False), (700, 6, 256, False), (2048, 6, 64, False),
                                          (10000, 6, 64, False), (8192, 8, 128, False),
                                          # and the one-workgroup kernel on the same sizes
                                          (2048, 4, 60, True), (515, 8, 64, True), (700, 6, 300, False)])
def test_dispatch_bit_exact(cuda, T, k, E, single):
    from promoe_amd import ops
    print(f"case dispatch T={T} k={k} E={E} single={single}", flush=True)
    rng = np.random.default_rng(T + k + E)
    # distinct experts per token, skewed popularity
    p = 1.0 / np.arange(1, E + 1) ** 1.2
    p /= p.sum()
    idx = np.stack([rng.choice(E, size=k, replace=False, p=p) for _ in range(T)]).astype(np.int32) \
        if T else np.zeros((0, k), np.int32)
    d = ops.dispatch(torch.from_numpy(idx).to(cuda).reshape(T, k), E, single_workgroup=single)
    d.check()
    counts, offsets, sp, pp = O.dispatch(idx, E)
    P = T * k
    assert np.array_equal(d.counts.cpu().numpy(), counts)
    assert np.array_equal(d.offsets.cpu().numpy(), offsets)
    assert np.array_equal(d.sorted_pair.cpu().numpy()[:P], sp)
    assert np.array_equal(d.pos_of_pair.cpu().numpy()[:P], pp)
    assert np.array_equal(d.sorted_tok.cpu().numpy()[:P], sp // k)
    act = np.nonzero(counts)[0]
    n_act = int(d.n_active.cpu()[0])
    assert n_act == min(len(act), d.max_units)
    units = d.units.cpu().numpy()[:n_act]
    assert np.array_equal(units[:, 0], act[:n_act])
    assert np.array_equal(units[:, 1], counts[act[:n_act]])
    assert np.array_equal(units[:, 2], offsets[act[:n_act]])
    assert np.array_equal(d.active_ids.cpu().numpy()[:n_act], act[:n_act])
    assert np.all(d.units.cpu().numpy()[n_act:d.max_units, 1] == 0)


def test_dispatch_workspace_reused(cuda):
    """Calls that share one workspace: the barrier words are zero again after each call, whatever the grid."""
    from promoe_amd import ops
    from promoe_amd._lib import lib, ptr, cur_stream, check
    E, k = 64, 6
    ws_bytes = int(lib.moe_dispatch_workspace_bytes(4096, k, E))
    assert ws_bytes > 0 and int(lib.moe_dispatch_workspace_bytes(300, k, E)) == 0
    ws = torch.zeros(ws_bytes // 4 + 1, dtype=torch.int32, device=cuda)
    err = torch.zeros(1, dtype=torch.int32, device=cuda)
    rng = np.random.default_rng(5)
    for T in (4096, 400, 2048, 3, 4096):
        print(f"case dispatch_ws T={T}", flush=True)
        idx = np.stack([rng.choice(E, size=k, replace=False) for _ in range(T)]).astype(np.int32)
        d = ops.Dispatch(T, k, E, min(E, T * k), cuda)
        check(lib.moe_dispatch_ws(ptr(torch.from_numpy(idx).to(cuda)), T, k, E, ptr(d.counts), ptr(d.offsets),
                                  ptr(d.sorted_pair), ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units),
                                  ptr(d.n_active), ptr(d.active_ids), d.max_units, ptr(ws), ws_bytes, ptr(err),
                                  cur_stream()), "moe_dispatch_ws")
        counts, offsets, sp, pp = O.dispatch(idx, E)
        assert int(err.item()) == 0
        assert np.array_equal(d.counts.cpu().numpy(), counts)
        assert np.array_equal(d.offsets.cpu().numpy(), offsets)
        assert np.array_equal(d.sorted_pair.cpu().numpy()[:T * k], sp)
        assert np.array_equal(d.pos_of_pair.cpu().numpy()[:T * k], pp)
        assert not ws[:16].any().item()


def run_layer_gpu(layer, x, k, mode, dev, resident=None, host_units=False):
    """gate -> topk -> dispatch -> int4 decode experts -> combine, all on the GPU."""
    from promoe_amd import ops
    H, I, E, I_sh = layer.H, layer.I, layer.E, layer.I_sh
    T = x.shape[0]
    xd = bf16_dev(x, dev)
    wg = layer.wg
    if layer.shared_gate is not None:
        wg = np.concatenate([wg, layer.shared_gate[None, :]], axis=0)
    logits = ops.gate_logits(xd, bf16_dev(wg, dev),
                             None if layer.bias is None else torch.from_numpy(
                                 np.concatenate([layer.bias, np.zeros(wg.shape[0] - E, np.float32)])).to(dev))
    idx, w = ops.topk(logits, k, mode, E=E)
    d = ops.dispatch(idx, E)
    slots = [torch.from_numpy(s).to(dev) for s in layer.slots]
    table = torch.tensor([0 if (resident is not None and e not in resident) else slots[e].data_ptr()
                          for e in range(E)], dtype=torch.int64, device=dev)
    shared = torch.from_numpy(layer.shared_img).to(dev) if I_sh else None
    if isinstance(layer, Q4KLayer):
        part_r, part_s, err, h_r, h_s = ops.experts_decode_q4k(xd, d, table, shared, H, I, I_sh)
    else:
        part_r, part_s, err, h_r, h_s = ops.experts_decode_int4(xd, d, table, shared, H, I, I_sh, host_units=host_units)
    sg = logits[:, E] if layer.shared_gate is not None else None
    y = ops.combine(part_r, part_s, w, d.pos_of_pair, sg, T, H, k)
    torch.cuda.synchronize()
    return dict(y=y.float().cpu().numpy(), idx=idx.cpu().numpy(), w=w.cpu().numpy(),
                logits=logits.cpu().numpy(), err=int(err.cpu()[0]), d=d)


def check_layer(layer, T, k, mode, dev, seed=1):
    x = O.synth_acts(T, layer.H, seed=seed)
    got = run_layer_gpu(layer, x, k, mode, dev)
    lg = O.gate_logits_ordered(x, layer.wg)
    if layer.bias is not None:
        lg = (lg + layer.bias[None, :]).astype(np.float32)
    ref = O.moe_forward(x, layer.wg, layer.experts_fp32, k, mode, shared=layer.shared_fp32,
                        shared_gate=layer.shared_gate, logits=lg)
    assert got["err"] == 0
    assert np.array_equal(got["logits"][:, :layer.E].view(np.uint32), lg.view(np.uint32))
    assert np.array_equal(got["idx"], ref["idx"])          # routing bit-exact
    counts, offsets, sp, pp = O.dispatch(ref["idx"], layer.E)
    assert np.array_equal(got["d"].sorted_pair.cpu().numpy()[:T * k], sp)  # permutation bit-exact
    err = np.abs(got["y"] - ref["out"]).max() / np.abs(ref["out"]).max()
    print(f"  T={T} k={k} mode={mode} max-rel-err={err:.3e}", flush=True)
    assert err <= TOL
    # units resolved on the host and passed in the kernel arguments: same kernels, same bits
    got2 = run_layer_gpu(layer, x, k, mode, dev, host_units=True)
    assert got2["err"] == 0 and np.array_equal(got2["y"], got["y"])
    return err


@pytest.mark.parametrize("T", [1, 2, 3, 4, 7, 16, 21])
def test_decode_layer_small(cuda, T):
    print(f"case decode_small T={T}", flush=True)
    layer = Int4Layer(H=256, I=384, E=8, I_sh=256, seed=3)
    check_layer(layer, T, 2, 0, cuda)


def test_decode_layer_small_variants(cuda):
    print("case decode_small_variants", flush=True)
    # no shared expert, Mixtral routing
    check_layer(Int4Layer(H=512, I=128, E=8, I_sh=0, seed=4), 5, 2, 2, cuda)
    # sigmoid-gated shared expert, renormalised routing, Zipf bias
    check_layer(Int4Layer(H=256, I=256, E=60, I_sh=512, seed=5, shared_gate=True, zipf=1.1), 6, 4, 1, cuda)
    # odd group counts per wave (G = 3 and 5)
    check_layer(Int4Layer(H=384, I=640, E=4, I_sh=128, seed=6), 3, 2, 0, cuda)


@pytest.mark.parametrize("T", [3, 16, 20, 33, 40, 50, 64, 70])
def test_decode_layer_long_reduction(cuda, T):
    """Reductions longer than 2048 and batches of more than 16 tokens take the chunked-K GEMV: group counts
    that leave a partial last chunk and an odd number of weight steps (G = 18, 17, 20) in chunks of 8, 4 and
    2 groups; passes of 16, 32 and 64 rows picked per unit by the rows it has left (E = 4, k = 2: about T / 2
    rows per routed unit, T rows for the shared expert: 33 = one partial 64-row pass, 70 = a 64-row pass and
    a 16-row pass, 20 and 40 = partial 32-row passes)."""
    print(f"case decode_long_reduction T={T}", flush=True)
    layer = Int4Layer(H=2304, I=2176, E=4, I_sh=2560, seed=8)
    check_layer(layer, T, 2, 0, cuda)


@pytest.mark.parametrize("T", [1, 4, 16, 32, 64])
def test_decode_layer_deepseek_shape(cuda, T):
    print(f"case decode_deepseek T={T}", flush=True)
    # DeepSeek-MoE-16B layer shape; 16 experts instead of 64 keeps host-side quantisation short
    layer = Int4Layer(H=2048, I=1408, E=16, I_sh=2816, seed=0, zipf=1.2)
    check_layer(layer, T, 6, 0, cuda)


def test_non_resident_expert_is_reported(cuda):
    print("case non_resident", flush=True)
    layer = Int4Layer(H=256, I=128, E=4, I_sh=0, seed=7)
    x = O.synth_acts(2, 256)
    got = run_layer_gpu(layer, x, 2, 0, cuda, resident=set())
    assert got["err"] == 1


@pytest.mark.parametrize("T,H,E,k,mode,extra", [(1, 2048, 64, 6, 0, 0), (4, 2048, 64, 6, 0, 1), (16, 2048, 64, 6, 1, 0),
                                               (3, 4096, 8, 2, 2, 0), (16, 3584, 64, 8, 0, 1), (7, 256, 60, 4, 0, 0)])
def test_fused_route_equals_separate_kernels(cuda, T, H, E, k, mode, extra):
    from promoe_amd import ops
    print(f"case route_decode T={T} H={H} E={E} k={k} mode={mode} extra={extra}", flush=True)
    x = bf16_dev(O.synth_acts(T, H, seed=5), cuda)
    wg = bf16_dev(O.round_bf16(O.synth_weights((E + extra, H), seed=6)), cuda)
    bias = torch.from_numpy(O.zipf_gate_bias(E, 1.2)).to(cuda)
    lg, idx, w, d = ops.route_decode(x, wg, bias, E, k, mode)
    lg_ref = ops.gate_logits(x, wg[:E].contiguous(), bias)
    idx_ref, w_ref = ops.topk(lg_ref, k, mode)
    d_ref = ops.dispatch(idx_ref, E)
    assert torch.equal(lg[:, :E], lg_ref) and torch.equal(idx, idx_ref) and torch.equal(w, w_ref)
    if extra:
        assert torch.equal(lg[:, E:], ops.gate_logits(x, wg[E:].contiguous()))
    P = T * k
    for name in ("counts", "offsets", "n_active"):
        assert torch.equal(getattr(d, name), getattr(d_ref, name)), name
    for name in ("sorted_pair", "pos_of_pair", "sorted_tok"):
        assert torch.equal(getattr(d, name)[:P], getattr(d_ref, name)[:P]), name
    assert torch.equal(d.units, d_ref.units) and torch.equal(d.active_ids, d_ref.active_ids)


@pytest.mark.parametrize("T", [1, 2, 3, 4, 16, 21, 33, 40, 64])
def test_decode_q4k_layer_small(cuda, T):
    """One token: the dot-product GEMV; more: the chunked-K matrix-core form with passes of 16, 32 and 64 rows
    (E = 8, k = 2: the shared expert has T rows, a routed unit about T / 4)."""
    print(f"case decode_q4k_small T={T}", flush=True)
    check_layer(Q4KLayer(H=256, I=512, E=8, I_sh=256, seed=3), T, 2, 0, cuda)


@pytest.mark.parametrize("T", [3, 20, 48])
def test_decode_q4k_long_reduction_split_shared_expert(cuda, T):
    """A shared expert wide enough that its w2 reduction is split over workgroups (I_sh = 8192: 64 groups in 2 or
    4 windows, each window a whole number of super-blocks), group counts that leave partial chunks (I = 768: 6
    groups against chunks of 8 and 4), few experts with many rows each."""
    from promoe_amd import ops, _lib as L
    print(f"case decode_q4k_split T={T}", flush=True)
    assert ops.shared_splits(L.FMT_Q4K, T, 512, 8192) > 1
    check_layer(Q4KLayer(H=512, I=768, E=4, I_sh=8192, seed=11), T, 2, 0, cuda)


def test_decode_q4k_qwen2_shape(cuda):
    print("case decode_q4k_qwen2", flush=True)
    # Qwen2-57B-A14B layer shape (H 3584, I 2560, sigmoid-gated shared expert), fewer experts and a
    # smaller shared expert than the model to keep host-side quantisation short
    layer = Q4KLayer(H=3584, I=2560, E=8, I_sh=5120, seed=1, shared_gate=True, zipf=1.1)
    for T in (1, 3):
        check_layer(layer, T, 4, 0, cuda)


@pytest.mark.parametrize("H,I,E,k,mode,I_sh,zipf", [(2048, 1408, 16, 6, 0, 2816, 1.2), (256, 384, 8, 2, 2, 256, None),
                                                    (256, 256, 60, 4, 1, 512, 1.1), (512, 128, 200, 8, 0, 0, None),
                                                    # 8, 12, 28 and 1 quantisation groups per row: two and three tiles
                                                    # in flight per wave and block, a partial second chunk, waves
                                                    # without a group
                                                    (1024, 256, 8, 2, 0, 128, None), (1536, 384, 8, 3, 1, 0, None),
                                                    (3584, 256, 8, 2, 2, 256, None), (128, 128, 8, 2, 0, 128, None)])
def test_token_decode_routes_in_kernel_like_separate_kernels(cuda, H, I, E, k, mode, I_sh, zipf):
    """One token: the w13 kernel derives the routing itself.  Indices, weights, dispatch arrays and
    the layer output must equal those of gate -> top-k -> dispatch -> experts -> combine, bit for bit."""
    from promoe_amd import ops
    print(f"case token_route H={H} I={I} E={E} k={k} mode={mode}", flush=True)
    layer = Int4Layer(H=H, I=I, E=E, I_sh=I_sh, seed=11, zipf=zipf)
    slots = [torch.from_numpy(s).to(cuda) for s in layer.slots]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=cuda)
    shared = torch.from_numpy(layer.shared_img).to(cuda) if I_sh else None
    wg = bf16_dev(layer.wg, cuda)
    bias = None if layer.bias is None else torch.from_numpy(layer.bias).to(cuda)
    for seed in range(3):
        x = O.synth_acts(1, H, seed=seed)
        if seed == 2:   # constructed ties in the logits: equal gate rows give equal logits
            wg = wg.clone(); wg[3] = wg[1]; wg[E - 1] = wg[1]
            if bias is not None:
                bias = bias.clone(); bias[3] = bias[1]; bias[E - 1] = bias[1]
        xd = bf16_dev(x, cuda)
        logits = ops.gate_logits(xd, wg, bias)
        idx, w = ops.topk(logits, k, mode)
        d = ops.dispatch(idx, E)
        part_r, part_s, err, _, _ = ops.experts_decode_int4(xd, d, table, shared, H, I, I_sh)
        y_ref = ops.combine(part_r, part_s, w, d.pos_of_pair, None, 1, H, k)
        idx2, w2, d2, pr2, ps2, err2, _, _ = ops.decode_token_int4(xd, logits, E, k, mode, table, shared, H, I, I_sh)
        y = ops.combine(pr2, ps2, w2, d2.pos_of_pair, None, 1, H, k)
        torch.cuda.synchronize()
        assert int(err.cpu()[0]) == 0 and int(err2.cpu()[0]) == 0
        assert torch.equal(idx, idx2) and torch.equal(w.view(torch.int32), w2.view(torch.int32))
        for name in ("counts", "offsets", "sorted_pair", "pos_of_pair", "sorted_tok", "n_active"):
            assert torch.equal(getattr(d, name), getattr(d2, name)), name
        na = int(d.n_active.cpu()[0])
        assert torch.equal(d.units[:na], d2.units[:na]) and torch.equal(d.active_ids[:na], d2.active_ids[:na])
        assert torch.equal(y_ref, y)


@pytest.mark.parametrize("H,I,E,k,mode,I_sh,zipf,gated", [
    (2048, 1408, 16, 6, 0, 2816, 1.2, False), (256, 384, 8, 2, 2, 256, None, True), (256, 256, 60, 4, 1, 512, 1.1, False),
    (512, 128, 200, 8, 0, 0, None, False), (4096, 14336, 4, 2, 2, 0, None, False), (3584, 2560, 8, 8, 0, 20480, 1.1, True),
    (256, 128, 4, 1, 0, 0, None, False)])
def test_token_decode_w2_and_combine_in_one_launch(cuda, H, I, E, k, mode, I_sh, zipf, gated):
    """One token: phase bit 2 runs w2 over all units and the weighted combine in one launch.  Same
    routing outputs as the two-launch form; y within bf16 rounding of it (other summation order),
    and within 2e-2 of the fp32 restatement."""
    from promoe_amd import ops
    print(f"case token_w2c H={H} I={I} E={E} k={k} mode={mode} I_sh={I_sh}", flush=True)
    layer = Int4Layer(H=H, I=I, E=E, I_sh=I_sh, seed=5, zipf=zipf, shared_gate=gated)
    slots = [torch.from_numpy(s).to(cuda) for s in layer.slots]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=cuda)
    shared = torch.from_numpy(layer.shared_img).to(cuda) if I_sh else None
    wg_np = layer.wg if not gated else np.concatenate([layer.wg, layer.shared_gate[None, :]], axis=0)
    wg = bf16_dev(wg_np, cuda)
    bias = None if layer.bias is None else torch.from_numpy(
        np.concatenate([layer.bias, np.zeros(wg_np.shape[0] - E, np.float32)])).to(cuda)
    unit_ws = torch.zeros(32 * k, dtype=torch.uint8, device=cuda)
    for seed in range(2):
        x = O.synth_acts(1, H, seed=seed + 20)
        xd = bf16_dev(x, cuda)
        logits = ops.gate_logits(xd, wg, bias)
        sg = logits[:, E] if gated else None
        idx, w, d, pr, ps, err, _, _ = ops.decode_token_int4(xd, logits, E, k, mode, table, shared, H, I, I_sh)
        y_ref = ops.combine(pr, ps, w, d.pos_of_pair, sg, 1, H, k)
        y = torch.full((1, H), float("nan"), dtype=torch.bfloat16, device=cuda)
        idx2, w2, d2, _, _, err2, _, _ = ops.decode_token_int4(xd, logits, E, k, mode, table, shared, H, I, I_sh,
                                                               phases=5, unit_ws=unit_ws, sg_logit=sg, y=y)
        torch.cuda.synchronize()
        assert int(err.cpu()[0]) == 0 and int(err2.cpu()[0]) == 0
        assert torch.equal(idx, idx2) and torch.equal(w.view(torch.int32), w2.view(torch.int32))
        assert torch.equal(d.units[:k], d2.units[:k])
        a, b = y.float().cpu().numpy(), y_ref.float().cpu().numpy()
        assert np.isfinite(a).all()
        assert np.abs(a - b).max() <= 1e-2 * np.abs(b).max(), (np.abs(a - b).max(), np.abs(b).max())
        lg = O.gate_logits_ordered(x, layer.wg)
        if layer.bias is not None:
            lg = (lg + layer.bias[None, :]).astype(np.float32)
        ref = O.moe_forward(x, layer.wg, layer.experts_fp32, k, mode, shared=layer.shared_fp32,
                            shared_gate=layer.shared_gate, logits=lg)
        assert np.array_equal(idx2.cpu().numpy(), ref["idx"])
        assert np.abs(a - ref["out"]).max() <= TOL * np.abs(ref["out"]).max()


@pytest.mark.parametrize("H,I,E,k,mode,I_sh,zipf,gated", [
    (2048, 1408, 64, 6, 0, 2816, 1.2, False), (256, 384, 8, 2, 2, 256, None, True), (256, 256, 60, 4, 1, 512, 1.1, True),
    (512, 128, 200, 8, 0, 0, None, False), (4096, 14336, 4, 2, 2, 0, None, False), (4608, 128, 130, 3, 0, 128, 1.1, True)])
def test_token_decode_gate_rows_in_the_w13_launch(cuda, H, I, E, k, mode, I_sh, zipf, gated):
    """One token, two launches: the w13 launch sums the gate rows in its first workgroups and hands the logits to
    its routing waves.  Logits, routing and y must equal those of gate launch + the same kernels, bit for bit, on
    successive calls over one hand-over workspace (a word of an earlier call must never pass for a new one)."""
    from promoe_amd import ops
    print(f"case token_gate H={H} I={I} E={E} k={k} mode={mode} I_sh={I_sh}", flush=True)
    layer = Int4Layer(H=H, I=I, E=E, I_sh=I_sh, seed=7, zipf=zipf, shared_gate=gated)
    slots = [torch.from_numpy(s).to(cuda) for s in layer.slots]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=cuda)
    shared = torch.from_numpy(layer.shared_img).to(cuda) if I_sh else None
    wg_np = layer.wg if not gated else np.concatenate([layer.wg, layer.shared_gate[None, :]], axis=0)
    wg = bf16_dev(wg_np, cuda)
    bias_e = None if layer.bias is None else torch.from_numpy(layer.bias).to(cuda)     # the routed rows only
    bias_all = None if layer.bias is None else torch.from_numpy(
        np.concatenate([layer.bias, np.zeros(wg_np.shape[0] - E, np.float32)])).to(cuda)
    unit_ws = torch.zeros(32 * k, dtype=torch.uint8, device=cuda)
    unit_ws2 = torch.zeros(32 * k, dtype=torch.uint8, device=cuda)
    gws = ops.GateWorkspace(cuda)
    ws2 = None
    for seed in range(4):
        x = O.synth_acts(1, H, seed=seed + 40)
        if seed == 3:   # constructed ties
            wg = wg.clone(); wg[3] = wg[1]; wg[E - 1] = wg[1]
            if bias_e is not None:
                bias_e = bias_e.clone(); bias_e[3] = bias_e[1]; bias_e[E - 1] = bias_e[1]
                bias_all = bias_all.clone(); bias_all[3] = bias_all[1]; bias_all[E - 1] = bias_all[1]
        xd = bf16_dev(x, cuda)
        logits = ops.gate_logits(xd, wg, bias_all)
        sg = logits[:, E] if gated else None
        y_ref = torch.full((1, H), float("nan"), dtype=torch.bfloat16, device=cuda)
        idx, w, d, _, _, err, h_r, h_s = ops.decode_token_int4(xd, logits, E, k, mode, table, shared, H, I, I_sh,
                                                                phases=5, unit_ws=unit_ws, sg_logit=sg, y=y_ref)
        logits2 = torch.full_like(logits, float("nan"))
        sg2 = logits2[:, E] if gated else None
        y = torch.full((1, H), float("nan"), dtype=torch.bfloat16, device=cuda)
        # every other call with up to 64 experts: the slot table travels in the launch arguments, and the device
        # table it must then not read holds zeros
        by_value = E <= 64 and seed % 2 == 1
        ws2 = ops.decode_token_int4(xd, logits2, E, k, mode, torch.zeros_like(table) if by_value else table, shared,
                                    H, I, I_sh, ws=ws2, phases=5, unit_ws=unit_ws2, sg_logit=sg2, y=y,
                                    gate=(wg, bias_e, gws), expert_ptr_host=table.cpu() if by_value else None)
        idx2, w2, d2, _, _, err2, h_r2, h_s2 = ws2
        torch.cuda.synchronize()
        assert int(err.cpu()[0]) == 0 and int(err2.cpu()[0]) == 0
        assert torch.equal(logits.view(torch.int32), logits2.view(torch.int32))
        assert torch.equal(idx, idx2) and torch.equal(w.view(torch.int32), w2.view(torch.int32))
        for name in ("counts", "offsets", "sorted_pair", "pos_of_pair", "sorted_tok", "n_active"):
            assert torch.equal(getattr(d, name), getattr(d2, name)), name
        assert torch.equal(d.units[:k], d2.units[:k])
        assert torch.equal(h_r.view(torch.int16), h_r2.view(torch.int16))
        assert torch.equal(y_ref.view(torch.int16), y.view(torch.int16))
    assert gws.seq == 4


@pytest.mark.parametrize("T,E,k,mode", [(1, 64, 6, 0), (4, 64, 6, 0), (16, 64, 6, 1), (16, 60, 4, 2), (7, 200, 8, 0),
                                        (16, 8, 2, 2), (3, 256, 32, 0), (32, 64, 6, 0), (64, 64, 8, 1), (33, 60, 4, 2)])
def test_topk_dispatch_in_one_launch_equals_separate_kernels(cuda, T, E, k, mode):
    from promoe_amd import ops
    print(f"case topk_dispatch T={T} E={E} k={k} mode={mode}", flush=True)
    rng = np.random.default_rng(T * 131 + E + k)
    logits = rng.normal(0, 2, (T, E + 1)).astype(np.float32)
    logits[:, E // 2] = logits[:, 1]          # ties
    lg = torch.from_numpy(logits).to(cuda)
    idx, w = ops.topk(lg, k, mode, E=E)
    d = ops.dispatch(idx, E)
    idx2, w2, d2 = ops.topk_dispatch(lg[:, :E] if False else lg, k, E, mode) if False else ops.topk_dispatch(lg, k, E, mode)
    torch.cuda.synchronize()
    assert torch.equal(idx, idx2) and torch.equal(w.view(torch.int32), w2.view(torch.int32))
    for name in ("counts", "offsets", "sorted_pair", "pos_of_pair", "sorted_tok", "n_active", "units", "active_ids"):
        assert torch.equal(getattr(d, name), getattr(d2, name)), name


@pytest.mark.parametrize("parts", [1, 8])
@pytest.mark.parametrize("T,E,k,mode,H,rows_extra,with_bias",
                         [(2, 64, 6, 0, 2048, 0, False), (4, 64, 6, 0, 2048, 0, False), (16, 64, 6, 1, 2048, 1, True),
                          (16, 60, 4, 2, 2048, 1, False), (7, 200, 8, 0, 1024, 0, True), (5, 8, 2, 2, 4096, 0, False),
                          (3, 256, 32, 0, 520, 1, True), (32, 64, 6, 0, 2048, 0, False), (32, 16, 8, 1, 3584, 1, False)])
def test_gate_topk_dispatch_in_one_launch_equals_separate_kernels(cuda, T, E, k, mode, H, rows_extra, with_bias, parts):
    """The launch that sums the gate rows and routes (workgroup 0 polls the logits the others hand over) against
    the gate launch followed by the routing launch: same bits everywhere, on three calls that share a workspace."""
    from promoe_amd import ops
    print(f"case gate_topk_dispatch T={T} E={E} k={k} mode={mode} H={H} rows={E + rows_extra} bias={with_bias} parts={parts}",
          flush=True)
    rng = np.random.default_rng(T * 977 + E * 31 + k + H)
    rows = E + rows_extra
    wg = torch.from_numpy(rng.normal(0, 0.05, (rows, H)).astype(np.float32)).to(cuda).to(torch.bfloat16)
    wg[E // 2] = wg[1]          # ties
    bias = torch.from_numpy(rng.normal(0, 0.3, E).astype(np.float32)).to(cuda) if with_bias else None
    if bias is not None:
        bias[E // 2] = bias[1]
    gws = ops.GateWorkspace(cuda, 32, 257)
    for rep in range(3):
        x = torch.from_numpy(rng.normal(0, 1, (T, H)).astype(np.float32)).to(cuda).to(torch.bfloat16)
        lg = torch.empty(T, rows, dtype=torch.float32, device=cuda)
        lg_e = ops.gate_logits(x, wg[:E].contiguous(), bias)
        lg[:, :E] = lg_e
        if rows_extra:
            lg[:, E:] = ops.gate_logits(x, wg[E:].contiguous(), None)
        idx, w, d = ops.topk_dispatch(lg, k, E, mode)
        lg2, idx2, w2, d2, err = ops.gate_topk_dispatch(x, wg, bias, E, k, mode, gws, parts=parts)
        torch.cuda.synchronize()
        assert int(err.item()) == 0
        assert torch.equal(lg.view(torch.int32), lg2.view(torch.int32))
        assert torch.equal(idx, idx2) and torch.equal(w.view(torch.int32), w2.view(torch.int32))
        for name in ("counts", "offsets", "sorted_pair", "pos_of_pair", "sorted_tok", "n_active", "units", "active_ids"):
            assert torch.equal(getattr(d, name), getattr(d2, name)), name
    assert gws.seq == 3


@pytest.mark.parametrize("T,H,I,E,k,mode,I_sh,zipf,gated", [
    (4, 2048, 1408, 64, 6, 0, 2816, 1.2, False), (2, 2048, 1408, 64, 6, 0, 2816, 1.2, False),
    (8, 2048, 1408, 64, 6, 1, 2816, 1.2, True), (3, 256, 384, 8, 2, 2, 256, None, True),
    (7, 256, 256, 60, 4, 1, 512, 1.1, True), (5, 512, 128, 200, 8, 0, 0, None, False),
    (4, 4096, 14336, 4, 2, 2, 0, None, False), (8, 1024, 128, 130, 3, 0, 128, 1.1, True),
    (6, 384, 256, 256, 32, 0, 0, None, False),
    # from 9 tokens on (and where whole rows of 5 to 8 tokens do not fit beside a second workgroup): the chunked-K form
    (16, 2048, 1408, 64, 6, 0, 2816, 1.2, False), (12, 2048, 1408, 64, 6, 1, 2816, 1.2, True),
    (8, 4096, 14336, 4, 2, 2, 0, None, False), (16, 256, 384, 8, 2, 2, 256, None, True),
    (9, 512, 128, 200, 8, 0, 0, None, False), (13, 256, 256, 60, 4, 1, 512, 1.1, True),
    (16, 384, 256, 256, 32, 0, 0, None, False)])
def test_batch_decode_gate_rows_and_routing_in_the_w13_launch(cuda, T, H, I, E, k, mode, I_sh, zipf, gated):
    """2 to 16 tokens: the w13 launch sums the gate rows, every unit's workgroups route by themselves and one
    workgroup publishes the routing.  Logits, routing arrays, h rows and partial rows must equal those of the
    gate + routing launch followed by the expert launches, bit for bit, on successive calls over one hand-over
    workspace."""
    from promoe_amd import ops
    print(f"case batch_gate T={T} H={H} I={I} E={E} k={k} mode={mode} I_sh={I_sh}", flush=True)
    layer = Int4Layer(H=H, I=I, E=E, I_sh=I_sh, seed=11, zipf=zipf, shared_gate=gated)
    rows = E + (1 if gated else 0)
    assert ops.decode_batch_int4_gate_fits(T, E, k, H, I, I_sh, rows)
    slots = [torch.from_numpy(s).to(cuda) for s in layer.slots]
    table = torch.tensor([s.data_ptr() for s in slots], dtype=torch.int64, device=cuda)
    shared = torch.from_numpy(layer.shared_img).to(cuda) if I_sh else None
    wg_np = layer.wg if not gated else np.concatenate([layer.wg, layer.shared_gate[None, :]], axis=0)
    wg = bf16_dev(wg_np, cuda)
    bias_e = None if layer.bias is None else torch.from_numpy(layer.bias).to(cuda)
    gws = ops.GateWorkspace(cuda, 16, 257)
    gws_ref = ops.GateWorkspace(cuda, 16, 257)
    # 9 to 15 tokens: the separate launches take the whole-row GEMV where it fits and the fused launch the chunked-K
    # one (another summation order): the routing is compared bit for bit, the products within rounding
    same_form = not (9 <= T <= 15)
    P = T * k
    for seed in range(4):
        x = O.synth_acts(T, H, seed=seed + 70)
        if seed == 3:   # constructed ties
            wg = wg.clone(); wg[E // 2] = wg[1]; wg[E - 1] = wg[1]
            if bias_e is not None:
                bias_e = bias_e.clone(); bias_e[E // 2] = bias_e[1]; bias_e[E - 1] = bias_e[1]
        xd = bf16_dev(x, cuda)
        lg, idx, w, d, err0 = ops.gate_topk_dispatch(xd, wg, bias_e, E, k, mode, gws_ref)
        part_r, part_s, err, h_r, h_s = ops.experts_decode_int4(xd, d, table, shared, H, I, I_sh)
        # every other call with up to 64 experts: the slot table travels in the launch arguments, and the device
        # table it must then not read holds zeros (a read would skip every unit and raise the error word)
        by_value = E <= 64 and seed % 2 == 1
        lg2, idx2, w2, d2, part_r2, part_s2, err2, h_r2, h_s2 = ops.decode_batch_int4_gate(
            xd, wg, bias_e, E, k, mode, torch.zeros_like(table) if by_value else table, shared, H, I, I_sh, gws,
            expert_ptr_host=table.cpu() if by_value else None)
        torch.cuda.synchronize()
        assert int(err0.item()) == 0 and int(err.item()) == 0 and int(err2.item()) == 0
        assert torch.equal(lg.view(torch.int32), lg2.view(torch.int32))
        assert torch.equal(idx, idx2) and torch.equal(w.view(torch.int32), w2.view(torch.int32))
        for name in ("counts", "offsets", "sorted_pair", "pos_of_pair", "sorted_tok", "n_active", "units", "active_ids"):
            assert torch.equal(getattr(d, name), getattr(d2, name)), name
        if same_form:
            assert torch.equal(h_r[:P].view(torch.int16), h_r2[:P].view(torch.int16))
            assert torch.equal(part_r[:P].view(torch.int32), part_r2[:P].view(torch.int32))
            if I_sh:
                assert torch.equal(h_s.view(torch.int16), h_s2.view(torch.int16))
                assert torch.equal(part_s.view(torch.int32), part_s2.view(torch.int32))
        else:
            pairs = [(h_r[:P], h_r2[:P], 2.0 ** -6), (part_r[:P], part_r2[:P], 2.0 ** -5)]
            if I_sh:
                pairs += [(h_s, h_s2, 2.0 ** -6), (part_s, part_s2, 2.0 ** -5)]
            for p, q, tol in pairs:
                p, q = p.float(), q.float()
                assert float((p - q).abs().max()) <= tol * float(p.abs().max())
    assert gws.seq == 4
