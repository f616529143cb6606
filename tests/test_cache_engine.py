"""Host logic of the expert-cache engine (C ABI, host backend) against the CPU
restatement of the reference's cache manager / scheduler, plus what pins that
restatement (closed forms, textbook models, brute force)."""
import ctypes as C
import itertools
from collections import OrderedDict

import numpy as np
import pytest

from oracle import cache_oracle as CO
from promoe_amd import _lib as L
from promoe_amd import engine as EG


def make_engine(Lyr, E, k, P=2, nbytes=64, **cfg):
    m = EG.ModuleMeta(Lyr, E)
    names = ["p%d" % i for i in range(P)]
    m.init_param_list(names)
    d = {"num_expert_per_token": str(k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    pm = EG.PrefetchMngr(m, backend=L.BACKEND_HOST)
    bufs = {}
    for l in range(Lyr):
        for e in range(E):
            for p in range(P):
                b = np.full(nbytes, (l * E + e) * 4 + p, np.uint8)
                b[1] = p
                bufs[(l, e, p)] = b
                pm.add_one_expert_param(b, l, e, names[p])
    pm.init_gpu_mem_buffer()
    pm.launch_thread()
    return pm, bufs


def slot_bytes(pm, l, e, p, n):
    addr = pm.ref_one_expert_param(l, e, p)
    assert addr
    return np.ctypeslib.as_array((C.c_uint8 * n).from_address(addr)).copy()


# ------------------------------------------------------------------ configuration
def test_config_defaults_dialects_and_errors():
    m = EG.ModuleMeta(27, 64)
    m.init_param_list(["a", "b", "c"])
    m.init_from_map({"num_expert_per_token": "6", "moe-cache-rate": "0.375", "moe_cache_policy": "fifo",
                     "num-predict": "None", "cross_token_pred": "True", "model_arch_string": "DeepSeek-X",
                     "cache_only": ""})
    m.handle_uninited_configs()
    assert abs(m.cache_rate - 0.375) < 1e-7 and m.cache_policy == "fifo"
    assert m.num_predict_expert_per_layer == 6          # -1 -> num_expert_per_token
    assert m.reorder_experts and m.early_preempt and m.chunk_prefetch  # inferred from num_predict > 0
    assert m.layer_predict_replace_first_input_with_last_output is True
    assert m.max_prefetch_layer_distance == 26          # -1 -> L-1
    assert m.model_arch_string == "deepseek-x" and m.limit_layer_0_window == 3
    assert m.cache_only is False and m.per_layer_cache is True

    m2 = EG.ModuleMeta(2, 4)
    m2.init_param_list(["w"])
    m2.init_from_map({"num_expert_per_token": "2", "num_predict_expert_per_layer": "0"})
    m2.handle_uninited_configs()
    assert not m2.reorder_experts and not m2.early_preempt and m2.limit_layer_0_window == 1

    for bad in ({"num_expert_per_token": "2", "no_such_key": "1"},      # unknown key
                {"cache_rate": "0.5"},                                   # required key missing
                {"num_expert_per_token": "None"},
                {"num_expert_per_token": "2", "cache_rate": "abc"},
                {"num_expert_per_token": "2", "cache_policy": "mru"}):
        mb = EG.ModuleMeta(2, 4)
        mb.init_param_list(["w"])
        mb.init_from_map(bad)
        with pytest.raises(L.MoeError):
            mb.handle_uninited_configs()
    md = EG.ModuleMeta(2, 4)
    with pytest.raises(L.MoeError):                                       # duplicate after dialect translation
        md.init_from_map({"cache_rate": "0.5", "moe-cache-rate": "0.25"})


# ------------------------------------------------------------------ slot arithmetic
def test_slot_distribution_known_answers():
    assert CO.remainder_order(5) == [0, 1, 3, 4, 2]                      # hand-derived from cache.cpp:9-53
    assert CO.remainder_order(8) == [0, 1, 5, 3, 7, 4, 6, 2]        # mid 5; (2,5)->3, (6,8)->7; rest [2,4,6] -> 4, 6, 2
    assert CO.cache_len(0.375, 27, 64) == 648 and CO.slot_distribution(648, 27) == [24] * 27
    assert CO.cache_len(0.5, 32, 8) == 128 and CO.slot_distribution(128, 32) == [4] * 32
    assert CO.cache_len(0.375, 28, 64) == 672 and CO.slot_distribution(672, 28) == [24] * 28
    assert CO.slot_distribution(7, 5) == [2, 2, 1, 1, 1]
    for n, g in itertools.product(range(0, 70, 3), range(1, 12)):
        d = EG.slot_distribution(n, g)
        assert d == CO.slot_distribution(n, g)
        assert sum(d) == n and max(d) - min(d) <= 1
        assert sorted(CO.remainder_order(g)) == list(range(g))


def test_engine_slot_counts_follow_cache_rate():
    pm, _ = make_engine(5, 8, 2, cache_rate=0.3)
    n = CO.cache_len(0.3, 5, 8)
    assert pm.slot_info()[0] == n == 12
    assert [pm.slot_info(g)[0] for g in range(5)] == CO.slot_distribution(n, 5)
    pm.close()
    pm, _ = make_engine(5, 8, 2, cache_rate=0.3, per_layer_cache=False)
    assert pm.slot_info(0)[0] == 12
    pm.close()


# ------------------------------------------------------------------ what pins the oracle's policies
def test_oracle_lru_fifo_match_textbook():
    rng = np.random.default_rng(0)
    for policy in ("lru", "fifo"):
        sim = CO.CacheSim(1, 16, 1, 1, cache_rate=0.25, policy=policy, num_predict=0)
        model = OrderedDict()
        misses = 0
        for e in rng.integers(0, 16, 400):
            ids = sim.report_one_layer(0, [e])
            sim.wait_expert(0, ids[0]); sim.expert_launched(0, ids[0]); sim.layer_done(0)
            if e in model:
                if policy == "lru":
                    model.move_to_end(e)
            else:
                misses += 1
                if len(model) == 4:
                    model.popitem(last=False)
                model[e] = 1
            assert sim.resident(0) == sorted(model)
        assert sim.ctr["miss"] == misses and sim.ctr["hit"] == 400 - misses


def belady_min_misses(trace, cap):
    """Brute force: fewest misses over ALL eviction choices."""
    best = [len(trace) + 1]

    def rec(i, cache, m):
        if m >= best[0]:
            return
        if i == len(trace):
            best[0] = m
            return
        e = trace[i]
        if e in cache:
            rec(i + 1, cache, m)
        elif len(cache) < cap:
            rec(i + 1, cache | {e}, m + 1)
        else:
            for v in cache:
                rec(i + 1, (cache - {v}) | {e}, m + 1)
    rec(0, frozenset(), 0)
    return best[0]


def test_oracle_min_is_belady_optimal():
    rng = np.random.default_rng(1)
    for trial in range(6):
        trace = [int(x) for x in rng.integers(0, 5, 11)]
        E, cap = 5, 2
        sim = CO.CacheSim(1, E, 1, 1, cache_rate=cap / E, policy="min", num_predict=0)
        dec = np.array(trace, np.int32).reshape(-1, 1, 1)
        em = np.stack([np.zeros(len(trace), np.int64), np.arange(len(trace))], 1)
        sim.oracles = CO.load_oracle(1, E, em, np.zeros((1, 1), np.int32), np.zeros((1, 1, 1), np.int32), dec)
        sim.set_cur_seq(0)
        # one empty prefill tick precedes the decode tokens in the oracle's clock
        for e in trace:
            ids = sim.report_one_layer(0, [e]); sim.wait_expert(0, ids[0]); sim.expert_launched(0, ids[0])
        assert sim.ctr["miss"] == belady_min_misses(trace, cap)


def test_oracle_nn_evicts_lowest_priority():
    sim = CO.CacheSim(1, 8, 1, 2, cache_rate=0.5, policy="nn", num_predict=0)
    pr = np.array([[0.9, 0.1, 0.5, 0.3, 0.7, 0.2, 0.8, 0.4]], np.float32)
    for e in (0, 1, 2, 3):
        ids = sim.report_one_layer(0, [e]); sim.wait_expert(0, e); sim.expert_launched(0, e)
    sim.update_priority(pr)          # predicted probabilities replace the recency counters
    ids = sim.report_one_layer(0, [4]); sim.wait_expert(0, 4); sim.expert_launched(0, 4)
    assert sim.evicted_log == [(0, 1)]                      # 0.1 is the lowest
    ids = sim.report_one_layer(0, [5]); sim.wait_expert(0, 5); sim.expert_launched(0, 5)
    assert sim.evicted_log[-1] == (0, 3)                    # then 0.3; expert 4 carries max_priority+1


def test_oracle_static_keeps_first_arrivals():
    sim = CO.CacheSim(1, 8, 1, 1, cache_rate=0.5, policy="static-1", num_predict=0)
    for e in (0, 1, 2, 3, 4, 5, 0, 6):
        ids = sim.report_one_layer(0, [e]); sim.wait_expert(0, e); sim.expert_launched(0, e)
    # 0,1,2 became permanent when 1,2,3 arrived; the last slot rotates: 3 -> 4 -> 5 -> 6
    assert sim.resident(0) == [0, 1, 2, 6]
    assert sim.evicted_log == [(0, 3), (0, 4), (0, 5)]


# ------------------------------------------------------------------ engine == oracle on traces
def zipf_trace(rng, steps, Lyr, E, k, s=1.2):
    p = 1.0 / np.arange(1, E + 1) ** s
    p /= p.sum()
    perm = [rng.permutation(E) for _ in range(Lyr)]
    return [[np.sort(perm[l][rng.choice(E, size=k, replace=False, p=p)]) for l in range(Lyr)] for _ in range(steps)]


def drive(pm, sim, trace, Lyr, prefetch=None, check_each=True):
    for step, layers in enumerate(trace):
        for l in range(Lyr):
            if prefetch is not None:
                nxt = (l + 1) % Lyr
                ids_pf = prefetch(step, nxt)
                a = pm.prefetch_layer(nxt, ids_pf, blocking=False)
                b = sim.prefetch_layer(nxt, ids_pf)
                assert a == b
                pm.drain(); sim.drain()
            ids = np.array(layers[l], np.int64)
            got = pm.report_one_layer(l, ids.copy())
            ref = sim.report_one_layer(l, ids)
            assert list(got) == ref, (step, l)
            for e in ref:
                pm.report_one_expert(l, e); sim.wait_expert(l, e)
                pm.one_expert_done(l, e); sim.expert_launched(l, e)
            pm.one_moe_layer_done(l); sim.layer_done(l)
            if check_each:
                pm.drain(); sim.drain()
                assert [e for e in range(sim.E) if pm.is_in_cache(l, e)] == sim.resident(l), (step, l)
    pm.drain(); sim.drain()
    c = pm.counters()
    for key in ("hit", "miss", "prefetch_hit", "prefetch_miss", "activated", "evictions", "h2d_copies"):
        assert c[key] == sim.ctr[key], key
    return c


@pytest.mark.parametrize("policy", ["lru", "fifo", "static-1", "static-2", "nn"])
@pytest.mark.parametrize("num_predict", [0, -1])
def test_engine_matches_oracle_demand_only(policy, num_predict):
    Lyr, E, k, P = 3, 16, 3, 3
    rng = np.random.default_rng(hash((policy, num_predict)) % 1000)
    pm, _ = make_engine(Lyr, E, k, P=P, cache_rate=0.4, cache_policy=policy,
                        num_predict_expert_per_layer=num_predict)
    sim = CO.CacheSim(Lyr, E, P, k, cache_rate=0.4, policy=policy, num_predict=num_predict)
    c = drive(pm, sim, zipf_trace(rng, 40, Lyr, E, k), Lyr)
    assert c["hit"] + c["miss"] >= c["activated"]
    pm.close()


def test_engine_matches_oracle_nn_with_priority_updates():
    Lyr, E, k, P = 2, 12, 2, 1
    rng = np.random.default_rng(5)
    pm, _ = make_engine(Lyr, E, k, P=P, cache_rate=0.5, cache_policy="nn", num_predict_expert_per_layer=0)
    sim = CO.CacheSim(Lyr, E, P, k, cache_rate=0.5, policy="nn", num_predict=0)
    for rnd in range(6):
        drive(pm, sim, zipf_trace(rng, 5, Lyr, E, k), Lyr)
        pr = rng.random((Lyr, E)).astype(np.float32) if rnd % 2 == 0 else rng.random((1, E)).astype(np.float32)
        start = 0 if pr.shape[0] == Lyr else 1
        pm.update_priority(pr, start); sim.update_priority(pr, start)
    pm.close()


def test_engine_matches_oracle_min_policy():
    Lyr, E, k, P = 2, 8, 2, 1
    rng = np.random.default_rng(9)
    steps = 30
    trace = zipf_trace(rng, steps, Lyr, E, k)
    dec = np.array([[t[l] for l in range(Lyr)] for t in trace], np.int32)
    em = np.stack([np.zeros(steps, np.int64), np.arange(steps)], 1)
    plen = np.zeros((1, Lyr), np.int32); psel = np.zeros((1, Lyr, 1), np.int32)
    pm, _ = make_engine(Lyr, E, k, P=P, cache_rate=0.5, cache_policy="min", num_predict_expert_per_layer=0)
    sim = CO.CacheSim(Lyr, E, P, k, cache_rate=0.5, policy="min", num_predict=0)
    pm.load_oracle(em, plen, psel, dec)
    sim.oracles = CO.load_oracle(Lyr, E, em, plen, psel, dec)
    pm.set_cur_seq(0); sim.set_cur_seq(0)
    c = drive(pm, sim, trace, Lyr)
    # Belady never does worse than LRU on the same trace
    sim_lru = CO.CacheSim(Lyr, E, P, k, cache_rate=0.5, policy="lru", num_predict=0)
    for t in trace:
        for l in range(Lyr):
            for e in sim_lru.report_one_layer(l, t[l]):
                sim_lru.wait_expert(l, e); sim_lru.expert_launched(l, e)
    assert c["miss"] <= sim_lru.ctr["miss"]
    # an access the oracle did not record is an error, not an abort
    with pytest.raises(L.MoeError):
        ids = np.array([0, 1], np.int64)
        pm.report_one_layer(0, ids)
        for e in ids:
            pm.report_one_expert(0, int(e))
    pm.close()


@pytest.mark.parametrize("chunk", [True, False])
def test_engine_matches_oracle_with_prefetch_requests(chunk):
    Lyr, E, k, P = 3, 16, 3, 3
    rng = np.random.default_rng(11)
    trace = zipf_trace(rng, 30, Lyr, E, k)
    pm, _ = make_engine(Lyr, E, k, P=P, cache_rate=0.4, cache_policy="lru", chunk_prefetch=chunk)
    sim = CO.CacheSim(Lyr, E, P, k, cache_rate=0.4, policy="lru", chunk_prefetch=chunk)

    def predictor(step, layer):   # half right, half wrong guesses of the next layer's experts
        nstep = step + (1 if layer == 0 else 0)
        truth = trace[min(nstep, len(trace) - 1)][layer]
        return [int(truth[0]), int((truth[1] + 1) % E), int(truth[2])]
    c = drive(pm, sim, trace, Lyr, prefetch=predictor)
    assert c["prefetch_hit"] + c["prefetch_miss"] > 0 and c["ready"] > 0
    pm.close()


# ------------------------------------------------------------------ state machine, data, errors
def test_status_machine_and_slot_contents():
    pm, bufs = make_engine(2, 6, 2, P=2, cache_rate=0.5, cache_policy="lru", num_predict_expert_per_layer=0)
    assert pm.expert_status(0, 1) == "idle" and pm.ref_one_expert_param(0, 1, 0) == 0
    ids = np.array([1, 4], np.int64)
    pm.report_one_layer(0, ids)
    pm.report_one_expert(0, 1)
    assert pm.expert_status(0, 1) == "launching" and pm.num_ready(0, 1) == 2
    for p in range(2):
        assert np.array_equal(slot_bytes(pm, 0, 1, p, 64), bufs[(0, 1, p)])
    pm.one_expert_done(0, 1)
    assert pm.expert_status(0, 1) == "ready"          # using -> ready once the event fired
    pm.report_one_expert(0, 4); pm.one_expert_done(0, 4)
    # fill the 3 slots of layer 0 and evict the least recently used (expert 1)
    for e in (2, 0):
        ids = np.array([e], np.int64); pm.report_one_layer(0, ids); pm.report_one_expert(0, e); pm.one_expert_done(0, e)
    assert not pm.is_in_cache(0, 1) and pm.expert_status(0, 1) == "idle" and pm.num_ready(0, 1) == 0
    assert pm.ref_one_expert_param(0, 1, 0) == 0
    assert np.array_equal(slot_bytes(pm, 0, 0, 1, 64), bufs[(0, 0, 1)])
    pm.close()


def test_wait_on_unreported_expert_is_an_error_not_a_hang():
    pm, _ = make_engine(1, 4, 2, cache_rate=0.5, cache_policy="lru")   # early_preempt on
    with pytest.raises(L.MoeError):
        pm.report_one_expert(0, 3)
    pm.close()
    pm, _ = make_engine(1, 4, 2, cache_rate=0.5, cache_policy="lru")
    with pytest.raises(L.MoeError):
        pm.one_expert_done(0, 2)                                        # launching -> using from idle
    with pytest.raises(L.MoeError):                                       # the engine stays failed, like the abort it replaces
        pm.report_one_layer(0, np.array([1], np.int64))
    pm.close()


def test_reorder_puts_resident_experts_first():
    pm, _ = make_engine(1, 8, 3, P=1, cache_rate=0.5, cache_policy="lru")
    for e in (5, 2):
        ids = np.array([e], np.int64); pm.report_one_layer(0, ids); pm.report_one_expert(0, e); pm.one_expert_done(0, e)
    ids = np.array([1, 2, 3, 5], np.int64)
    pm.report_one_layer(0, ids)
    assert list(ids) == [2, 5, 1, 3]                  # stable within each class
    for e in ids:
        pm.report_one_expert(0, int(e)); pm.one_expert_done(0, int(e))
    c = pm.counters()
    # 2 and 5 were usable at once; whether 3 had landed when its hook fired depends on timing
    assert c["ready"] + c["unready"] == 6 and c["ready"] >= 2
    assert c["hit"] == 2 and c["miss"] == 4
    pm.close()


def test_prefetch_budget_and_report():
    pm, _ = make_engine(3, 8, 2, P=1, cache_rate=0.5, cache_policy="lru", max_prefetch_layer_distance=1)
    assert pm.prefetch_layer(1, [0, 1], blocking=False) is True
    assert pm.prefetch_layer(2, [0, 1], blocking=False) is False      # budget exhausted
    pm.drain()
    assert pm.is_in_cache(1, 0) and pm.expert_status(1, 0) == "ready"
    pm.report_moe_layer_logits(0, None, seq_len=1)
    for l in range(3):
        ids = np.array([0, 1], np.int64); pm.report_one_layer(l, ids)
        for e in ids:
            pm.report_one_expert(l, int(e)); pm.one_expert_done(l, int(e))
        pm.one_moe_layer_done(l)
    assert pm.prefetch_layer(2, [3], blocking=False) is True          # report_one_layer returned budget
    rep = pm.report()
    assert rep["num_decode_iter"] == 1 and rep["decode_stage_hit_cnt"] == 2 and rep["decode_stage_miss_cnt"] == 4
    assert abs(rep["decode_stage_hit_rate"] - 2 / 6) < 1e-6
    pm.close()


def test_concurrent_fetch_keeps_data_and_bounds(monkeypatch):
    """Slow copies force the partial / in-flight branches; invariants must hold."""
    monkeypatch.setenv("MOE_HOST_COPY_DELAY_US", "200")
    Lyr, E, k, P = 2, 12, 3, 3
    rng = np.random.default_rng(3)
    pm, bufs = make_engine(Lyr, E, k, P=P, cache_rate=0.34, cache_policy="lru")
    trace = zipf_trace(rng, 25, Lyr, E, k, s=0.8)
    for step, layers in enumerate(trace):
        for l in range(Lyr):
            nxt = (l + 1) % Lyr
            guess = trace[min(step + (nxt == 0), len(trace) - 1)][nxt]
            try:
                pm.prefetch_layer(nxt, [int(guess[0]), int((guess[1] + 1) % E)], blocking=False)
            except L.MoeError:
                pass   # a copy of that layer is still in flight: the reference would refuse as well
            ids = np.array(layers[l], np.int64)
            pm.report_one_layer(l, ids)
            assert sorted(ids) == sorted(layers[l])
            for e in ids:
                pm.report_one_expert(l, int(e))
                for p in range(P):
                    assert np.array_equal(slot_bytes(pm, l, int(e), p, 64), bufs[(l, int(e), p)])
                pm.one_expert_done(l, int(e))
            pm.one_moe_layer_done(l)
            assert sum(pm.is_in_cache(l, e) for e in range(E)) <= pm.slot_info(l)[0]
    pm.drain()
    pm.close()


@pytest.mark.timeout(60)
def test_forward_protocol_with_more_active_experts_than_slots():
    """The order the fused forward drives the hooks in: resident experts launched and
    released as one group, then each missed expert waited for, launched and marked.
    More active experts than slots must stream through without blocking."""
    Lyr, E, k, P = 1, 16, 4, 2
    rng = np.random.default_rng(21)
    pm, bufs = make_engine(Lyr, E, k, P=P, cache_rate=0.25, cache_policy="lru")   # 4 slots
    sim = CO.CacheSim(Lyr, E, P, k, cache_rate=0.25, policy="lru")
    for step in range(20):
        n = int(rng.integers(1, 13))
        ids = np.sort(rng.choice(E, size=n, replace=False)).astype(np.int64)
        ref = sim.report_one_layer(0, ids)
        pm.report_one_layer(0, ids)
        assert list(ids) == ref
        now = [int(e) for e in ids if pm.expert_status(0, int(e)) == "launching"]
        later = [int(e) for e in ids if int(e) not in now]
        pm.release_experts(0, now)
        for e in ref:
            if e in now:
                sim.wait_expert(0, e); sim.expert_launched(0, e)
        for e in later:
            pm.report_one_expert(0, e)
            for p in range(P):
                assert np.array_equal(slot_bytes(pm, 0, e, p, 64), bufs[(0, e, p)])
            pm.one_expert_done(0, e)
        for e in ref:
            if e not in now:
                sim.wait_expert(0, e); sim.expert_launched(0, e)
        pm.one_moe_layer_done(0); sim.layer_done(0)
        pm.drain(); sim.drain()
        assert [e for e in range(E) if pm.is_in_cache(0, e)] == sim.resident(0)
    c = pm.counters()
    assert c["miss"] == sim.ctr["miss"] and c["hit"] == sim.ctr["hit"] and c["evictions"] == sim.ctr["evictions"]
    pm.close()
