"""The fused MoE-layer forward through the expert cache on a real GPU: outputs against
the CPU oracle while experts are fetched, evicted and re-fetched underneath."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from oracle import cache_oracle as CO
from promoe_amd import _lib as L
from promoe_amd import engine as EG
from promoe_amd import layout as LY
from tests.synth import Int4Layer, Bf16Layer, Q4KLayer

pytestmark = pytest.mark.gpu
TOL = 2e-2


def build_engine(layers, k, dev, mode=0, max_tokens=64, **cfg):
    """Register every expert image (pinned host memory, six chunks each for int4, one for
    bf16) and start the engine."""
    Lyr, E = len(layers), layers[0].E
    H, I, I_sh = layers[0].H, layers[0].I, layers[0].I_sh
    bf16, q4k = isinstance(layers[0], Bf16Layer), isinstance(layers[0], Q4KLayer)
    total = (LY.bf16_expert_bytes(H, I) if bf16 else LY.q4k_layout(H, I)["total_bytes"] if q4k
             else LY.int4_layout(H, I)["total_bytes"])
    chunks = [("w", 0, total)] if (bf16 or q4k) else LY.split_chunks_int4(H, I)
    m = EG.ModuleMeta(Lyr, E)
    m.init_param_list([c[0] for c in chunks])
    d = {"num_expert_per_token": str(k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    pm = EG.PrefetchMngr(m, backend=L.BACKEND_HIP, compute_stream=torch.cuda.current_stream().cuda_stream)
    stage = EG.PinnedBuffer(total * Lyr * E)
    pm._keep.append(stage)
    for l, layer in enumerate(layers):
        for e in range(E):
            base = (l * E + e) * total
            stage.array[base: base + total] = layer.slots[e]
            for name, off, n in chunks:
                pm.add_one_expert_param(stage.array[base + off: base + off + n], l, e, name)
    assert pm.pin_memory() == 0
    pm.init_gpu_mem_buffer()
    for l, layer in enumerate(layers):
        gw = torch.from_numpy(layer.wg).to(torch.bfloat16).to(dev)
        bias = None if layer.bias is None else torch.from_numpy(layer.bias).to(dev)
        sh = torch.from_numpy(layer.shared_img).to(dev) if I_sh else None
        gated = getattr(layer, "shared_gate", None) is not None
        if gated:
            gw = torch.cat([gw, torch.from_numpy(layer.shared_gate[None, :]).to(torch.bfloat16).to(dev)])
        pm.set_layer(l, H, I, I_sh, k, mode, gw, bias, sh, shared_gated=gated,
                     fmt=L.FMT_BF16 if bf16 else (L.FMT_Q4K if q4k else L.FMT_INT4_G128))
    pm.forward_prepare(max_tokens)
    pm.launch_thread()
    return pm


def ref_forward(layer, x, k, mode):
    lg = O.gate_logits_ordered(x, layer.wg)
    if layer.bias is not None:
        lg = (lg + layer.bias[None, :]).astype(np.float32)
    return O.moe_forward(x, layer.wg, layer.experts_fp32, k, mode, shared=layer.shared_fp32,
                         shared_gate=getattr(layer, "shared_gate", None), logits=lg)


@pytest.mark.parametrize("impl", ["vmm", "slab"])
def test_forward_through_cache_matches_oracle(cuda, impl, monkeypatch):
    print(f"case engine_forward impl={impl}", flush=True)
    monkeypatch.setenv("SPARSE_CACHE_PHYSICAL_MEM_IMPL", impl)
    Lyr, E, k = 2, 16, 4
    layers = [Int4Layer(H=256, I=384, E=E, I_sh=256, seed=10 + l, zipf=1.2) for l in range(Lyr)]
    pm = build_engine(layers, k, cuda, cache_rate=0.375, cache_policy="lru")
    assert pm.slot_info()[0] == CO.cache_len(0.375, Lyr, E) == 12
    sim = CO.CacheSim(Lyr, E, 6, k, cache_rate=0.375, policy="lru")
    worst = 0.0
    for step, T in enumerate([1, 1, 4, 1, 16, 2, 1, 33, 1, 1]):
        for l in range(Lyr):
            x = O.synth_acts(T, 256, seed=100 + step * Lyr + l)
            y = pm.forward(l, torch.from_numpy(x).to(torch.bfloat16).to(cuda))
            torch.cuda.synchronize()
            ref = ref_forward(layers[l], x, k, 0)
            err = np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()
            worst = max(worst, err)
            assert err <= TOL, (step, l, err)
            # the cache bookkeeping follows the restated reference logic
            ids = sim.report_one_layer(l, np.unique(ref["idx"]))
            for e in ids:
                sim.wait_expert(l, e); sim.expert_launched(l, e)
            sim.drain()
            pm.drain()
            assert [e for e in range(E) if pm.is_in_cache(l, e)] == sim.resident(l), (step, l)
    c = pm.counters()
    print(f"  worst max-rel-err {worst:.3e}; counters {c}", flush=True)
    for key in ("hit", "miss", "evictions", "activated"):
        assert c[key] == sim.ctr[key], key
    assert c["miss"] > 0 and c["evictions"] > 0 and c["hit"] > 0
    assert c["h2d_bytes"] == c["miss"] * LY.int4_layout(256, 384)["total_bytes"]
    assert c["forwards"] == 10
    pm.close()


def test_forward_all_resident_has_no_misses_after_warmup(cuda):
    print("case engine_forward all-resident", flush=True)
    layer = Int4Layer(H=256, I=256, E=8, I_sh=0, seed=20)
    pm = build_engine([layer], 2, cuda, mode=2, cache_rate=1.0, cache_policy="fifo")
    for rep in range(3):
        for T in (1, 5):
            x = O.synth_acts(T, 256, seed=rep * 7 + T)
            y = pm.forward(0, torch.from_numpy(x).to(torch.bfloat16).to(cuda))
            torch.cuda.synchronize()
            ref = ref_forward(layer, x, 2, 2)
            assert np.abs(y.float().cpu().numpy() - ref["out"]).max() <= TOL * np.abs(ref["out"]).max()
    c = pm.counters()
    assert c["miss"] <= 8 and c["evictions"] == 0
    # with every expert in its slot the forward runs without a host round trip; results and
    # the (lazily accounted) hit counters must not change character
    pm.acquire_layer(0, np.arange(8, dtype=np.int64))
    pm.release_layer(0)
    c0 = pm.counters()
    n_act = 0
    # 24, 32: routing tail in one launch above 16 tokens; 40, 64: separate routing kernels, still the GEMV kernels
    for T in (1, 5, 16, 2, 24, 32, 40, 64):
        x = O.synth_acts(T, 256, seed=50 + T)
        y = pm.forward(0, torch.from_numpy(x).to(torch.bfloat16).to(cuda))
        torch.cuda.synchronize()
        ref = ref_forward(layer, x, 2, 2)
        assert np.abs(y.float().cpu().numpy() - ref["out"]).max() <= TOL * np.abs(ref["out"]).max()
        n_act += len(np.unique(ref["idx"]))
    c1 = pm.counters()
    assert c1["miss"] == c0["miss"] and c1["hit"] - c0["hit"] == n_act and c1["activated"] - c0["activated"] == n_act
    pm.close()


def test_stepwise_hooks_on_gpu_expose_resident_parameters(cuda):
    """The reference's per-expert hook order with the slot pointers it would hand to a kernel."""
    print("case engine stepwise", flush=True)
    H, I, E = 256, 128, 6
    layer = Int4Layer(H=H, I=I, E=E, I_sh=0, seed=30)
    pm = build_engine([layer], 2, cuda, cache_rate=0.5, cache_policy="lru", num_predict_expert_per_layer=0)
    lay = LY.int4_layout(H, I)
    for ids in ([0, 3], [3, 4], [5, 0], [1, 2]):
        ids = np.array(ids, np.int64)
        pm.report_one_layer(0, ids)
        for e in ids:
            pm.report_one_expert(0, int(e))
            addr = pm.ref_one_expert_param(0, int(e), "w13_q")
            assert addr != 0
            # read the slot back from HBM: it must hold the registered image
            import ctypes, os
            hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
            back = np.empty(lay["total_bytes"], np.uint8)
            assert hip.hipMemcpy(ctypes.c_void_p(back.ctypes.data), ctypes.c_void_p(addr),
                                 ctypes.c_size_t(lay["total_bytes"]), 2) == 0
            assert np.array_equal(back, layer.slots[int(e)])
            pm.one_expert_done(0, int(e))
        pm.one_moe_layer_done(0)
    assert sum(pm.is_in_cache(0, e) for e in range(E)) == 3
    pm.close()


@pytest.mark.parametrize("kind", ["int4", "bf16", "q4k"])
def test_forward_prefill_sizes_through_cache(cuda, kind):
    """Token groups of prefill size take the matrix-core kernels (bf16 layers always do);
    experts are still fetched and evicted underneath, one launch per missed expert."""
    print(f"case engine_forward_prefill kind={kind}", flush=True)
    Lyr, E, k = 2, 16, 4
    mk = {"int4": Int4Layer, "bf16": Bf16Layer, "q4k": Q4KLayer}[kind]
    layers = [mk(H=256, I=512 if kind == "q4k" else 384, E=E, I_sh=256, seed=30 + l, zipf=1.2, shared_gate=True)
              for l in range(Lyr)]
    pm = build_engine(layers, k, cuda, max_tokens=512, cache_rate=0.5, cache_policy="lru")
    sim = CO.CacheSim(Lyr, E, 6 if kind == "int4" else 1, k, cache_rate=0.5, policy="lru")
    worst = 0.0
    for step, T in enumerate([300, 1, 17, 512, 3, 129]):
        for l in range(Lyr):
            x = O.synth_acts(T, 256, seed=200 + step * Lyr + l)
            y = pm.forward(l, torch.from_numpy(x).to(torch.bfloat16).to(cuda))
            torch.cuda.synchronize()
            ref = ref_forward(layers[l], x, k, 0)
            err = np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()
            worst = max(worst, err)
            assert err <= TOL, (step, l, T, err)
            ids = sim.report_one_layer(l, np.unique(ref["idx"]))
            for e in ids:
                sim.wait_expert(l, e); sim.expert_launched(l, e)
            sim.drain()
            pm.drain()
            assert [e for e in range(E) if pm.is_in_cache(l, e)] == sim.resident(l), (step, l)
    c = pm.counters()
    print(f"  worst max-rel-err {worst:.3e}; counters {c}", flush=True)
    for key in ("hit", "miss", "evictions"):
        assert c[key] == sim.ctr[key], key
    assert c["miss"] > 0
    pm.close()


@pytest.mark.parametrize("fused", [True, False])
def test_patched_module_mirror_matches_oracle(cuda, fused):
    """The module-level mirror of the reference's patched MoE block: `report_experts` after
    routing, ExpertHook around every expert launch (unfused) or one fused call."""
    from promoe_amd.module import SparseMoeBlock
    print(f"case module_mirror fused={fused}", flush=True)
    Lyr, E, k = 2, 16, 4
    layers = [Int4Layer(H=256, I=384, E=E, I_sh=256, seed=40 + l, zipf=1.2) for l in range(Lyr)]
    pm = build_engine(layers, k, cuda, max_tokens=64, cache_rate=0.5, cache_policy="lru")
    blocks = []
    for l, layer in enumerate(layers):
        gw = torch.from_numpy(layer.wg).to(torch.bfloat16).to(cuda)
        bias = torch.from_numpy(layer.bias).to(cuda)
        sh = torch.from_numpy(layer.shared_img).to(cuda)
        blocks.append(SparseMoeBlock(pm, l, E, 256, 384, 256, k, 0, gw, bias, sh, fused=fused))
    sim = CO.CacheSim(Lyr, E, 6, k, cache_rate=0.5, policy="lru")
    for step, T in enumerate([1, 4, 40, 1, 16]):
        for l in range(Lyr):
            x = O.synth_acts(T, 256, seed=300 + step * Lyr + l)
            y = blocks[l](torch.from_numpy(x).to(torch.bfloat16).to(cuda))
            torch.cuda.synchronize()
            ref = ref_forward(layers[l], x, k, 0)
            err = np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()
            assert err <= TOL, (step, l, T, err)
            ids = sim.report_one_layer(l, np.unique(ref["idx"]))
            for e in ids:
                sim.wait_expert(l, e); sim.expert_launched(l, e)
            sim.drain()
            pm.drain()
            assert [e for e in range(E) if pm.is_in_cache(l, e)] == sim.resident(l), (step, l)
    c = pm.counters()
    for key in ("hit", "miss", "evictions"):
        assert c[key] == sim.ctr[key], key
    pm.close()


@pytest.mark.parametrize("E,batch,steps,rate", [(16, 3, 12, 0.375), (80, 3, 12, 0.05), (16, 12, 12, 0.375),
                                                (24, 16, 10, 0.2)])
def test_forward_single_token_starts_before_the_host_knows_the_routing(cuda, E, batch, steps, rate):
    """Demand fetching only (no prefetch producer): a forward of one token (or of a decode batch of up to 16) launches
    the self-routing expert kernel on whatever is resident, learns the routing from pinned memory and serves the
    misses afterwards.  Outputs, residency and counters must still follow the reference logic.  Up to 64 experts
    the launches carry the slot table in their arguments; with 80 they read the device table, refreshed in the
    stream after every miss."""
    print(f"case engine_forward optimistic E={E} batch={batch}", flush=True)
    Lyr, k = 3, 4
    layers = [Int4Layer(H=256, I=384, E=E, I_sh=256, seed=50 + l, zipf=1.2) for l in range(Lyr)]
    cfg = dict(cache_rate=rate, cache_policy="lru", num_predict_expert_per_layer=0, reorder_experts=True,
               early_preempt=True)
    pm = build_engine(layers, k, cuda, **cfg)
    sim = CO.CacheSim(Lyr, E, 6, k, cache_rate=rate, policy="lru", num_predict=0, reorder=True, early_preempt=True)
    worst = 0.0
    for step in range(steps):
        T = 1 if step % 5 and batch < 8 else batch    # mostly single tokens with a few small batches in between, or batches only
        for l in range(Lyr):
            x = O.synth_acts(T, 256, seed=400 + step * Lyr + l)
            y = pm.forward(l, torch.from_numpy(x).to(torch.bfloat16).to(cuda))
            torch.cuda.synchronize()
            ref = ref_forward(layers[l], x, k, 0)
            err = np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()
            worst = max(worst, err)
            assert err <= TOL, (step, l, T, err)
            ids = sim.report_one_layer(l, np.unique(ref["idx"]))
            for e in ids:
                sim.wait_expert(l, e); sim.expert_launched(l, e)
            sim.drain()
            pm.drain()
            assert [e for e in range(E) if pm.is_in_cache(l, e)] == sim.resident(l), (step, l)
    c = pm.counters()
    print(f"  worst max-rel-err {worst:.3e}; counters {c}", flush=True)
    for key in ("hit", "miss", "evictions", "activated"):
        assert c[key] == sim.ctr[key], key
    assert c["miss"] > 0 and c["hit"] > 0 and c["evictions"] > 0
    pm.close()


def test_builtin_predictor_prefetches_what_the_next_layers_route_to(cuda):
    """Models of the pairs (src -> dst) = the gate of dst, and every layer of a token sees the same
    hidden state: the predictions are the true routings, so layers 1.. find their experts prefetched.
    Outputs stay those of the oracle; demand misses drop against the same run without a predictor."""
    print("case engine_predictor", flush=True)
    Lyr, E, k, H = 4, 16, 2, 256
    layers = [Int4Layer(H=H, I=128, E=E, I_sh=0, seed=30 + l) for l in range(Lyr)]
    xs = [O.synth_acts(1, H, seed=700 + t) for t in range(12)]

    def run(with_predictor):
        pm = build_engine(layers, k, cuda, cache_rate=0.25, cache_policy="lru", num_predict_expert_per_layer=k,
                          layer_predict_interval=1, layer_predict_max_window=2, limit_layer_0_window=2)
        if with_predictor:
            for src, (a, b) in enumerate(pm.predictor_windows()):
                for dst in range(a, b):
                    pm.set_predictor_model(src, dst, torch.from_numpy(layers[dst].wg).to(torch.bfloat16).to(cuda), None)
            pm.start_predictor()
        worst = 0.0
        for x in xs:
            xd = torch.from_numpy(x).to(torch.bfloat16).to(cuda)
            for l in range(Lyr):
                y = pm.forward(l, xd)
                torch.cuda.synchronize()
                ref = ref_forward(layers[l], x, k, 0)
                worst = max(worst, float(np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()))
        pm.drain()
        c = pm.counters()
        st = pm.predictor_stats() if with_predictor else None
        pm.close()
        return worst, c, st

    w0, c0, _ = run(False)
    w1, c1, st = run(True)
    assert w0 <= TOL and w1 <= TOL
    assert st["jobs"] == len(xs) * 3 and st["requests"] == len(xs) * Lyr
    assert c1["prefetch_hit"] > 0
    assert c1["miss"] * 2 < c0["miss"]
    print(f"  demand misses {c0['miss']} -> {c1['miss']}, ready {c0['ready']} -> {c1['ready']}, "
          f"prefetch hits {c1['prefetch_hit']}", flush=True)


def test_trained_predictor_models_beat_demand_fetching_on_held_out_steps(cuda, tmp_path):
    """The training script end to end: a trace of decode steps whose hidden state drifts from layer to layer (the
    destination layer's routing is only partly determined by what a source layer sees), one ridge-regression
    model per (source -> destination) pair fitted on 300 tokens, written to and read back from a model directory
    in the reference's "{src}-{dst}" naming, attached to the engine; on 40 held-out tokens the run with these
    models takes fewer demand misses than the same run without a predictor, and the outputs stay the oracle's."""
    from promoe_amd import predictor_train as PT
    print("case engine_trained_predictor", flush=True)
    Lyr, E, k, H = 4, 16, 2, 256
    layers = [Int4Layer(H=H, I=128, E=E, I_sh=0, seed=130 + l) for l in range(Lyr)]
    rng = np.random.default_rng(17)

    def token():
        """Hidden states at the inputs of layers 0..L of one token, rounded to bf16 as the engine sees them."""
        x = rng.normal(size=H).astype(np.float32)
        hs = []
        for l in range(Lyr + 1):
            hs.append(O.round_bf16(x[None, :])[0])
            x = ((x + 0.5 * rng.normal(size=H)) / np.sqrt(1.25)).astype(np.float32)
        return hs

    cfg = dict(cache_rate=0.25, cache_policy="lru", num_predict_expert_per_layer=k, layer_predict_interval=1,
               layer_predict_max_window=2, limit_layer_0_window=2)
    pm = build_engine(layers, k, cuda, **cfg)
    windows = pm.predictor_windows()
    pm.close()
    trace = PT.Trace(Lyr, H, E)
    for _ in range(300):
        hs = token()
        trace.begin_token()
        for l in range(Lyr + 1):
            trace.add_layer(l, hs[l], O.gate_logits(hs[l][None, :], layers[l].wg)[0] if l < Lyr else None)
        trace.end_token()
    models = PT.fit_all(trace, windows, ridge=1e-2)
    PT.save_dir(str(tmp_path / "models"), models)
    held_out = [token() for _ in range(40)]

    def run(with_predictor):
        pm = build_engine(layers, k, cuda, **cfg)
        if with_predictor:
            assert PT.attach(pm, str(tmp_path / "models"), device=cuda) == len(models)
        worst = 0.0
        for hs in held_out:
            for l in range(Lyr):
                y = pm.forward(l, torch.from_numpy(hs[l][None, :]).to(torch.bfloat16).to(cuda))
                torch.cuda.synchronize()
                ref = ref_forward(layers[l], hs[l][None, :], k, 0)
                worst = max(worst, float(np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()))
        pm.drain()
        c = pm.counters()
        pm.close()
        return worst, c

    w0, c0 = run(False)
    w1, c1 = run(True)
    print(f"  demand misses {c0['miss']} -> {c1['miss']}, prefetch hits {c1['prefetch_hit']}, prefetch copies "
          f"{c1['prefetch_miss']}", flush=True)
    assert w0 <= TOL and w1 <= TOL
    assert c1["prefetch_hit"] > 0
    assert c1["miss"] < c0["miss"]


@pytest.mark.parametrize("T", [1, 3, 12])
def test_one_token_path_under_wrong_prefetches(cuda, T):
    """A predictor with random models keeps evicting experts the tokens are about to use, while the one-token
    path (and that of a decode batch of up to 16 tokens) launches its kernels on table snapshots: the outputs must
    stay the oracle's (the slot-group guard and the late classification of evicted experts are what this exercises)."""
    print(f"case engine_wrong_prefetch T={T}", flush=True)
    Lyr, E, k, H = 3, 16, 4, 256
    layers = [Int4Layer(H=H, I=128, E=E, I_sh=128, seed=60 + l, zipf=1.1) for l in range(Lyr)]
    pm = build_engine(layers, k, cuda, cache_rate=0.3, cache_policy="lru", num_predict_expert_per_layer=k,
                      layer_predict_interval=1, layer_predict_max_window=2, limit_layer_0_window=2)
    g = torch.Generator().manual_seed(5)
    for src, (a, b) in enumerate(pm.predictor_windows()):
        for dst in range(a, b):
            pm.set_predictor_model(src, dst, torch.randn(E, H, generator=g).to(torch.bfloat16).to(cuda), None)
    pm.start_predictor()
    worst = 0.0
    for t in range(30):
        for l in range(Lyr):
            # (the predictor acts on one-token steps only, as the reference's does: batches alternate with them and
            # meet what their prefetches left behind)
            x = O.synth_acts(T if t % 2 else 1, H, seed=900 + t * Lyr + l)
            y = pm.forward(l, torch.from_numpy(x).to(torch.bfloat16).to(cuda))
            torch.cuda.synchronize()
            ref = ref_forward(layers[l], x, k, 0)
            worst = max(worst, float(np.abs(y.float().cpu().numpy() - ref["out"]).max() / np.abs(ref["out"]).max()))
    pm.drain()
    c = pm.counters()
    pm.close()
    print(f"  worst rel err {worst:.3e}, misses {c['miss']}, prefetch copies {c['prefetch_miss']}, evictions {c['evictions']}",
          flush=True)
    assert worst <= TOL
    assert c["prefetch_miss"] > 0 and c["evictions"] > 0 and c["miss"] > 0


@pytest.mark.parametrize("cached", [False, True])
def test_engines_without_a_synchronisation_per_call(cuda, cached):
    """Forwards issued back to back, nothing synchronised in between, inputs made by torch right before the
    call on torch's own stream: a second engine over the same layers must give the first one's outputs.
    cached = False: both hold every expert (bit-identical outputs; this is what the stream guard of
    PrefetchMngr.forward is for: from the default stream each engine has a private compute stream).
    cached = True: the second one runs at cache rate 0.3 with a predictor whose models are right for half of
    the layer pairs and random for the other half, so demand fetches, prefetches and evictions go on under the
    kernels of both.  MOE_SOAK_STEPS lengthens the run (30000 steps = 120000 forwards were run this way)."""
    import os
    print(f"case engine_async cached={cached}", flush=True)
    steps = int(os.environ.get("MOE_SOAK_STEPS", "400"))
    Lyr, E, k, H, I, I_sh = 4, 32, 4, 1024, 512, 512
    layers = [Int4Layer(H=H, I=I, E=E, I_sh=I_sh, seed=70 + l, zipf=1.1) for l in range(Lyr)]
    A = build_engine(layers, k, cuda, cache_rate=1.0, cache_policy="lru")
    if cached:
        B = build_engine(layers, k, cuda, cache_rate=0.3, cache_policy="lru", num_predict_expert_per_layer=k,
                         layer_predict_interval=1, layer_predict_max_window=2, limit_layer_0_window=2)
        g = torch.Generator().manual_seed(5)
        for src, (a, b) in enumerate(B.predictor_windows()):
            for dst in range(a, b):
                m = (torch.from_numpy(layers[dst].wg) if (src + dst) % 2 else torch.randn(E, H, generator=g))
                B.set_predictor_model(src, dst, m.to(torch.bfloat16).to(cuda), None)
        B.start_predictor()
    else:
        B = build_engine(layers, k, cuda, cache_rate=1.0, cache_policy="lru")
    rng = np.random.default_rng(0)
    gx = torch.Generator(device=cuda).manual_seed(100)
    pend, worst = [], 0.0
    for s in range(steps):
        T = int(rng.choice([1, 1, 1, 1, 1, 1, 2, 4, 16, 40]))
        for l in range(Lyr):
            x = torch.randn(T, H, device=cuda, generator=gx).to(torch.bfloat16)
            pend.append((s, l, T, A.forward(l, x), B.forward(l, x)))
        if s % 100 == 99 or s == steps - 1:
            torch.cuda.synchronize()
            for (s_, l_, T_, ya, yb) in pend:
                a, b = ya.float(), yb.float()
                err = float((a - b).abs().max() / a.abs().max().clamp_min(1e-6))
                assert err <= (1e-2 if cached else 0.0), f"step {s_} layer {l_} T {T_}: {err:.3e}"
                worst = max(worst, err)
            pend = []
    A.drain(); B.drain()
    c = B.counters()
    A.close(); B.close()
    print(f"  {steps} steps, worst {worst:.2e}, misses {c['miss']}, prefetch hits {c['prefetch_hit']}, "
          f"evictions {c['evictions']}", flush=True)
    if cached:
        assert c["miss"] > 0 and c["evictions"] > 0 and c["prefetch_hit"] > 0
