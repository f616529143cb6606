"""Built-in predictor on the host backend: layer windows against the restated mapping, and the
request / budget / progress protocol with models whose predictions are known."""
import os

import numpy as np
import torch
import pytest

from oracle import cache_oracle as CO
from oracle import moe_oracle as O
from promoe_amd import _lib as L
from promoe_amd import engine as EG


def make(Lyr, E, k, **cfg):
    m = EG.ModuleMeta(Lyr, E)
    m.init_param_list(["w"])
    d = {"num_expert_per_token": str(k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    pm = EG.PrefetchMngr(m, backend=L.BACKEND_HOST)
    for l in range(Lyr):
        for e in range(E):
            pm.add_one_expert_param(np.full(64, l * E + e, np.uint8), l, e, "w")
    pm.init_gpu_mem_buffer()
    pm.launch_thread()
    return pm


@pytest.mark.parametrize("Lyr,interval,window,limit0,cross", [(4, 1, 2, 2, False), (6, 1, 3, 1, False), (6, 2, 3, -1, False),
                                                              (5, 1, 1, 1, False), (4, 1, 2, 2, True), (27, 1, 3, 3, False)])
def test_windows_follow_the_reference_mapping(Lyr, interval, window, limit0, cross):
    pm = make(Lyr, 4, 2, layer_predict_interval=interval, layer_predict_max_window=window, limit_layer_0_window=limit0,
              layer_predict_replace_first_input_with_last_output=cross, predict_input_mode="moe_layer_logits")
    got = pm.predictor_windows()
    want = CO.predict_layer_mapping(Lyr, interval, window, int(pm.metas.limit_layer_0_window), cross)
    assert got == want
    pm.close()


def test_known_windows():
    # hand-derived from predictor.cpp:8-46: L=4, interval 1, window 2, layer 0 window 2
    assert CO.predict_layer_mapping(4, 1, 2, 2, False) == [(0, 2), (2, 3), (3, 4), (4, 4), (0, 0)]
    # cross-token: the last output predicts what layer 0's input did, layer 0 predicts nothing
    assert CO.predict_layer_mapping(4, 1, 2, 2, True) == [(0, 0), (2, 3), (3, 4), (4, 4), (0, 2)]
    # window 1: every layer predicts itself only
    assert CO.predict_layer_mapping(3, 1, 1, 1, False) == [(0, 1), (1, 2), (2, 3), (0, 0)]


def _bf16(a):
    return O.f32_to_bf16_bits(np.ascontiguousarray(a, np.float32))


def test_requests_follow_the_models_and_the_protocol_keeps_in_step():
    Lyr, E, k, H = 4, 8, 2, 64
    rng = np.random.default_rng(0)
    pm = make(Lyr, E, k, cache_rate=0.5, cache_policy="lru", num_predict_expert_per_layer=2,
              layer_predict_interval=1, layer_predict_max_window=2, limit_layer_0_window=2,
              predict_input_mode="moe_layer_logits")
    wins = pm.predictor_windows()
    assert wins == [(0, 2), (2, 3), (3, 4), (4, 4), (0, 0)]
    with pytest.raises(L.MoeError):
        pm.set_predictor_model(1, 1, _bf16(np.zeros((E, H))))          # layer 1 predicts layer 2 only
    # model of (src, dst): one-hot rows, so that the score of expert e is x[dst * E + e]
    for src, (a, b) in enumerate(wins):
        for dst in range(a, b):
            w = np.zeros((E, H), np.float32)
            w[np.arange(E), dst * E + np.arange(E)] = 1.0
            pm.set_predictor_model(src, dst, _bf16(w), None)
    pm.start_predictor()
    want = {}
    for tok in range(6):
        x = np.zeros(H, np.float32)
        chosen = {}
        for l in range(Lyr):
            top = rng.choice(E, size=2, replace=False)
            x[l * E + top[0]] = 3.0; x[l * E + top[1]] = 2.0           # ranked: top[0] then top[1]
            chosen[l] = [int(top[0]), int(top[1])]
        xb = _bf16(x.reshape(1, 1, H))
        for l in range(Lyr):
            pm.report_moe_layer_logits(l, xb)
            ids = np.array(sorted(chosen[l]), np.int64)
            order = pm.report_one_layer(l, ids)                        # waits for the layer's request
            for e in order:
                pm.report_one_expert(l, int(e)); pm.one_expert_done(l, int(e))
            pm.one_moe_layer_done(l)
        pm.drain()
        want[tok] = chosen
    st = pm.predictor_stats()
    assert st["jobs"] == 6 * 3 and st["requests"] == 6 * Lyr           # sources 0, 1, 2 have windows; 4 layers per token
    c = pm.counters()
    # layers 1..3 are requested before they run: their experts are prefetched, only layer 0 (predicted
    # from its own input, a moment before use) and evictions can miss
    assert c["prefetch_hit"] + c["prefetch_miss"] > 0
    assert c["ready"] >= 6 * 3 * k * 0.9
    # a prefill step: empty requests, nothing to wait for
    pm.report_moe_layer_logits(0, None, seq_len=5)
    for l in range(Lyr):
        if l:
            pm.report_moe_layer_logits(l, None, seq_len=5)
        ids = np.arange(4, dtype=np.int64)
        for e in pm.report_one_layer(l, ids):
            pm.report_one_expert(l, int(e)); pm.one_expert_done(l, int(e))
        pm.one_moe_layer_done(l)
    assert pm.predictor_stats()["requests"] == 7 * Lyr
    pm.close()


@pytest.mark.parametrize("right", [True, False])
def test_requests_of_a_layer_with_poor_predictions_go_out_empty(right):
    """Precision feedback (moe_predictor_set_min_precision): with models that rank the experts the layers then
    route to, the averages stay at 1 and every request goes out; with models that rank OTHER experts the averages
    fall and, from then on, the requests go out empty (no prefetch copies), while the protocol keeps in step."""
    Lyr, E, k, H = 4, 8, 2, 64
    rng = np.random.default_rng(3)
    pm = make(Lyr, E, k, cache_rate=0.5, cache_policy="lru", num_predict_expert_per_layer=2,
              layer_predict_interval=1, layer_predict_max_window=2, limit_layer_0_window=2,
              predict_input_mode="moe_layer_logits")
    for src, (a, b) in enumerate(pm.predictor_windows()):
        for dst in range(a, b):
            w = np.zeros((E, H), np.float32)
            # right: the score of expert e is x[dst * E + e]; wrong: that of expert (e + 4) mod 8
            w[np.arange(E), dst * E + (np.arange(E) + (0 if right else 4)) % E] = 1.0
            pm.set_predictor_model(src, dst, _bf16(w), None)
    pm.set_predictor_min_precision(0.5)
    pm.start_predictor()
    n_tok = 16
    copies_at = {}
    for tok in range(n_tok):
        x = np.zeros(H, np.float32)
        chosen = {}
        for l in range(Lyr):
            top = rng.choice(4, size=2, replace=False)            # experts 0..3: the wrong models rank 4..7
            x[l * E + top[0]] = 3.0; x[l * E + top[1]] = 2.0
            chosen[l] = sorted(int(t) for t in top)
        xb = _bf16(x.reshape(1, 1, H))
        for l in range(Lyr):
            pm.report_moe_layer_logits(l, xb)
            for e in pm.report_one_layer(l, np.array(chosen[l], np.int64)):
                pm.report_one_expert(l, int(e)); pm.one_expert_done(l, int(e))
            pm.one_moe_layer_done(l)
        pm.drain()
        copies_at[tok] = pm.counters()["prefetch_miss"]
    prec, withheld = pm.predictor_precision()
    assert pm.predictor_stats()["requests"] == n_tok * Lyr            # empty or not, every layer got its request
    if right:
        assert withheld == 0 and (prec > 0.99).all()
    else:
        assert (prec < 0.2).all() and withheld >= (n_tok - 6) * Lyr
        assert copies_at[n_tok - 1] == copies_at[7]                   # nothing was prefetched once the averages fell
        assert copies_at[2] > 0
    pm.close()


def test_start_needs_every_model():
    pm = make(3, 4, 2, layer_predict_interval=1, layer_predict_max_window=1, limit_layer_0_window=1,
              predict_input_mode="moe_layer_logits")
    pm.set_predictor_model(0, 0, _bf16(np.zeros((4, 16))))
    with pytest.raises(L.MoeError, match="no model"):
        pm.start_predictor()
    pm.close()


def test_request_over_a_leftover_copy_of_the_same_layer(monkeypatch):
    """Layer 0 is predicted from its own input, so a wrong prediction's copy can still be running when the
    next token asks for layer 0 again.  The hook refuses such a request (as the reference does); the
    built-in predictor queues it behind the copy instead of failing the forward."""
    monkeypatch.setenv("MOE_HOST_COPY_DELAY_US", "100000")             # every copy takes 100 ms
    Lyr, E, k, H = 2, 8, 2, 64
    pm = make(Lyr, E, k, cache_rate=0.5, cache_policy="lru", num_predict_expert_per_layer=2,
              layer_predict_interval=1, layer_predict_max_window=2, limit_layer_0_window=2,
              predict_input_mode="moe_layer_logits")
    assert pm.predictor_windows() == [(0, 2), (2, 2), (0, 0)]
    for l in range(Lyr):                                               # warm the cache: experts 0..3 of each layer
        for e in pm.report_one_layer(l, np.arange(4, dtype=np.int64)):
            pm.report_one_expert(l, int(e)); pm.one_expert_done(l, int(e))
        pm.one_moe_layer_done(l)
    pm.drain()
    absent = [[e for e in range(E) if pm.expert_status(l, e) == "idle"] for l in range(Lyr)]
    assert all(len(a) == 4 for a in absent)
    for dst in range(Lyr):                                             # always predict two experts that are not cached
        w = np.zeros((E, H), np.float32)
        w[absent[dst][0], 0] = 2.0; w[absent[dst][1], 0] = 1.0
        pm.set_predictor_model(0, dst, _bf16(w), None)
    pm.start_predictor()
    xb = _bf16(np.ones((1, 1, H), np.float32))
    for tok in range(3):                                               # the tokens only use cached experts: no demand copy to wait for
        for l in range(Lyr):
            pm.report_moe_layer_logits(l, xb)
            cached = [e for e in range(E) if pm.expert_status(l, e) in ("ready", "using")][:k]
            assert len(cached) == k
            for e in pm.report_one_layer(l, np.array(cached, np.int64)):
                pm.report_one_expert(l, int(e)); pm.one_expert_done(l, int(e))
            pm.one_moe_layer_done(l)
    pm.drain()
    assert pm.predictor_stats()["requests"] == 3 * Lyr
    pm.close()


# ---- training script and model directory (the reference's "{src}-{dst}" directory, predictor.cpp:610-636) ----

def test_fit_pair_recovers_a_known_linear_map():
    """Closed form: when the destination logits ARE a linear function of the source hidden state, the ridge fit
    with a vanishing penalty returns that function (a wrong normal equation, a transposed operand or a missing
    intercept would not)."""
    from promoe_amd import predictor_train as PT
    rng = np.random.default_rng(0)
    A = rng.normal(size=(12, 48)).astype(np.float32)
    b = rng.normal(size=12).astype(np.float32)
    X = rng.normal(size=(400, 48)).astype(np.float32) + 3.0      # a mean away from zero: the intercept matters
    W, bb = PT.fit_pair(X, X @ A.T + b, ridge=1e-10)
    assert np.abs(W - A).max() < 1e-4 and np.abs(bb - b).max() < 1e-3
    # the penalty shrinks the weights and leaves the fit of the mean to the intercept
    W2, bb2 = PT.fit_pair(X, X @ A.T + b, ridge=10.0)
    assert np.linalg.norm(W2) < 0.5 * np.linalg.norm(A)
    assert np.abs((X @ W2.T + bb2).mean(0) - (X @ A.T + b).mean(0)).max() < 1e-3


def test_model_directory_round_trip_and_missing_pair(tmp_path):
    from promoe_amd import predictor_train as PT
    rng = np.random.default_rng(1)
    windows = [(0, 2), (2, 3), (3, 3), (3, 3)]          # source 0 -> layers 0, 1; source 1 -> layer 2
    models = {(s, d): (rng.normal(size=(8, 32)).astype(np.float32), rng.normal(size=8).astype(np.float32))
              for s, (a, b) in enumerate(windows) for d in range(a, b)}
    PT.save_dir(str(tmp_path / "m"), models)
    assert sorted(f for f in os.listdir(tmp_path / "m")) == ["0-0.safetensors", "0-1.safetensors", "1-2.safetensors"]
    back = PT.load_dir(str(tmp_path / "m"), windows)
    for key, (W, b) in models.items():
        w2, b2 = back[key]
        assert w2.dtype == torch.bfloat16
        assert torch.equal(w2, torch.from_numpy(W).to(torch.bfloat16)) and np.array_equal(b2.numpy(), b)
    os.remove(tmp_path / "m" / "1-2.safetensors")
    with pytest.raises(FileNotFoundError):
        PT.load_dir(str(tmp_path / "m"), windows)
    # a trace survives its file
    tr = PT.Trace(3, 32, 8)
    for _ in range(5):
        tr.begin_token()
        for l in range(4):
            tr.add_layer(l, rng.normal(size=32), rng.normal(size=8) if l < 3 else None)
        tr.end_token()
    tr.save(str(tmp_path / "t.npz"))
    tr2 = PT.Trace.load(str(tmp_path / "t.npz"))
    assert np.array_equal(tr2.hidden, tr.hidden) and np.array_equal(tr2.logits, tr.logits) and tr2.L == 3
