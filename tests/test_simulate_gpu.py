"""The trace replay on the HIP backend: the reference's stand-in model with experts that are NOT empty
(eval/demo-simulate/transformers-deepseek-moe.py:27-88 replays with experts that do nothing).  Every copy is
a real one from pinned host memory into an HBM slot; at every hook the slot is read back and must hold the
expert's bytes; hit / miss / eviction counts must equal those of the restated reference cache manager and
of the same replay on the host backend."""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import cache_oracle as CO
from promoe_amd import _lib as L
from promoe_amd import simulate as S

pytestmark = pytest.mark.gpu
LYR, E, K, NBYTES = 4, 32, 4, 8192


def _sim_counts(trace, policy, rate, reorder):
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


@pytest.mark.parametrize("policy,reorder", [("lru", False), ("lru", True), ("min", False)])
def test_trace_replay_with_real_copies(cuda, policy, reorder):
    print(f"case simulate on the HIP backend policy={policy} reorder={reorder}", flush=True)
    trace = S.synthetic_trace(3, LYR, E, K, prompt_len=8, reply_len=16, zipf=1.2, seed=7)
    hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
    seen = {"n": 0}

    def check_slot(pm, l, e):      # between report_one_expert and one_expert_done: the slot holds the expert
        addr = pm.ref_one_expert_param(l, e, "w")
        assert addr != 0, (l, e)
        back = np.empty(NBYTES, np.uint8)
        assert hip.hipMemcpy(ctypes.c_void_p(back.ctypes.data), ctypes.c_void_p(addr), ctypes.c_size_t(NBYTES), 2) == 0
        assert np.array_equal(back, S.expert_pattern(l, e, E, NBYTES)), (l, e)
        seen["n"] += 1

    cfg = dict(cache_policy=policy, per_layer_cache=True, reorder_experts=reorder, early_preempt=False,
               num_predict_expert_per_layer=0, cache_rate=0.25)
    rep = S.replay(trace, LYR, E, K, backend=L.BACKEND_HIP, expert_bytes=NBYTES, on_expert=check_slot, **cfg)
    host = S.replay(trace, LYR, E, K, **cfg)
    ctr = _sim_counts(trace, policy, 0.25, reorder)
    for key in ("hit", "miss", "activated", "evictions"):
        assert rep["counter_" + key] == ctr[key] == host["counter_" + key], key
    assert rep["counter_miss"] > 0 and rep["counter_evictions"] > 0 and seen["n"] == rep["counter_activated"]
    assert rep["counter_h2d_bytes"] == rep["counter_miss"] * NBYTES
    for col in S.CSV_COLUMNS[4:6]:
        assert abs(rep[col] - host[col]) < 1e-12, col
