"""Trace replay tool: the engine (host backend) driven by a routing trace, against the CPU
restatement of the reference's cache manager and against what the policies' theory fixes."""
import csv
import json

import numpy as np
import pytest

from oracle import cache_oracle as CO
from promoe_amd import simulate as S

LYR, E, K = 3, 16, 2


@pytest.fixture(scope="module")
def trace():
    return S.synthetic_trace(3, LYR, E, K, prompt_len=6, reply_len=12, zipf=1.1, seed=4)


def _oracle_replay(trace, policy, rate, reorder):
    sim = CO.CacheSim(LYR, E, 1, K, cache_rate=rate, policy=policy, num_predict=0, reorder=reorder, early_preempt=False)
    if policy == "min":
        sim.oracles = CO.load_oracle(LYR, E, *S.oracle_tensors(trace, LYR, K))
    for si, s in enumerate(sorted(trace, key=int)):
        if policy == "min":
            sim.set_cur_seq(si)
        for _, layers in S.sequence_forwards(trace[s], LYR):
            for l, ids in enumerate(layers):
                for e in sim.report_one_layer(l, np.asarray(ids, np.int64)):
                    sim.wait_expert(l, e); sim.expert_launched(l, e)
                sim.layer_done(l)
    sim.drain()
    return sim.ctr


def test_trace_shape_and_forwards(trace):
    seq = trace["0"]
    fw = S.sequence_forwards(seq, LYR)
    assert len(fw) == 1 + 12 and fw[0][0] == 6 and all(n == 1 for n, _ in fw[1:])
    union = sorted(set(e for t in range(6) for e in seq["1"][str(t)]))
    assert fw[0][1][1] == union                       # prefill: sorted union of the prompt tokens' experts
    assert fw[3][1][2] == seq["2"][str(6 + 2)]        # decode forward r: token prompt_len + r
    assert len(S.sequence_forwards(seq, LYR, max_new_tokens=5)) == 6
    em, plen, psel, dsel = S.oracle_tensors(trace, LYR, K)
    assert em.shape == (36, 2) and plen.shape == (3, LYR) and dsel.shape == (36, LYR, K)
    assert list(psel[0, 1, :plen[0, 1]]) == union


@pytest.mark.parametrize("policy,reorder", [("lru", False), ("lru", True), ("fifo", False), ("min", False)])
def test_replay_counts_equal_the_restated_cache_manager(trace, policy, reorder):
    rep = S.replay(trace, LYR, E, K, cache_policy=policy, per_layer_cache=True, reorder_experts=reorder,
                   early_preempt=False, num_predict_expert_per_layer=0, cache_rate=0.25)
    ctr = _oracle_replay(trace, policy, 0.25, reorder)
    for key in ("hit", "miss", "activated", "evictions"):
        assert rep["counter_" + key] == ctr[key], key
    dec = rep["decode_stage_hit_cnt"] + rep["decode_stage_miss_cnt"]
    # the report averages over the forwards of a stage (the reference dumps averages, profiler.hpp:253-319)
    assert abs(dec - LYR * K) < 1e-6 and rep["num_prefill_iter"] == 3 and rep["num_decode_iter"] == 36


def test_full_cache_misses_only_cold_and_rates_are_monotone(trace):
    touched = set()
    for s in trace.values():
        for _, layers in S.sequence_forwards(s, LYR):
            for l, ids in enumerate(layers):
                touched.update((l, e) for e in ids)
    full = S.replay(trace, LYR, E, K, cache_policy="lru", reorder_experts=False, early_preempt=False,
                    num_predict_expert_per_layer=0, cache_rate=1.0)
    assert full["counter_miss"] == len(touched) and full["counter_evictions"] == 0
    rows = S.sweep(trace, LYR, E, K, policies=("lru", "min"), per_layer=(True,), reorder=(False,),
                   cache_rates=[2 / 16, 4 / 16, 8 / 16, 1.0])
    lru = [r["decode_stage_hit_rate"] for r in rows if r["cache_policy"] == "lru"]
    mn = [r["decode_stage_hit_rate"] for r in rows if r["cache_policy"] == "min"]
    assert lru == sorted(lru) and mn == sorted(mn)      # LRU and MIN are stack algorithms: more slots never hurt
    assert all(b >= a for a, b in zip(lru, mn))          # Belady is optimal


def test_cli_and_json_round_trip(trace, tmp_path):
    p = tmp_path / "trace.json"
    p.write_text(json.dumps(trace))
    out = tmp_path / "sweep.csv"
    S.main(["--trace", str(p), "--layers", str(LYR), "--experts", str(E), "--top-k", str(K), "--policies", "lru",
            "--cache-rates", "0.25,0.5", "--out", str(out)])
    rows = list(csv.DictReader(open(out)))
    assert list(rows[0].keys()) == S.CSV_COLUMNS and len(rows) == 2 * 2 * 2
    direct = S.replay(S.load_trace(str(p)), LYR, E, K, cache_policy="lru", per_layer_cache=True, reorder_experts=False,
                      early_preempt=False, num_predict_expert_per_layer=0, cache_rate=0.25)
    r0 = [r for r in rows if r["per_layer_cache"] == "True" and r["reorder_experts"] == "False" and r["cache_rate"] == "0.25"][0]
    assert abs(float(r0["decode_stage_hit_rate"]) - direct["decode_stage_hit_rate"]) < 1e-9
    with pytest.raises(SystemExit):
        S.main(["--layers", "2"])
