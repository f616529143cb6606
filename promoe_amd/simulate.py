"""Trace replay through the cache engine without a model or a GPU.

The reference evaluates cache policies by replaying a recorded routing trace through its cache manager
with a stand-in model whose experts do nothing (reference:
eval/demo-simulate/transformers-deepseek-moe.py:27-88; sweep eval/demo-simulate/runner.py:36-45; result
table eval/demo-simulate/output.csv).  This module does the same with this engine on its host backend:
every hook of a layer forward is called in the reference's order, copies are memcpy's, and the
per-stage counters come from the engine's own report.

Trace format (the reference's JSON, transformers-deepseek-moe.py:66-88):
    trace[str(seq)]["prompt_len"]                 -> int
    trace[str(seq)][str(layer)][str(token_idx)]   -> list of expert ids of that token in that layer
Token indices below prompt_len belong to the prompt; a prefill forward sees, per layer, the sorted
union of the prompt tokens' experts, a decode forward the experts of one token.

Usage:  python -m promoe_amd.simulate --synthetic --out sweep.csv
        python -m promoe_amd.simulate --trace trace.json --layers 27 --experts 64 --top-k 6
"""
from __future__ import annotations

import argparse
import csv
import json
import sys

import numpy as np

from . import _lib as L
from .engine import ModuleMeta, PrefetchMngr

CSV_COLUMNS = ["cache_policy", "per_layer_cache", "reorder_experts", "cache_rate", "decode_stage_hit_rate",
               "prefill_stage_hit_rate", "decode_stage_ready_rate", "prefill_stage_ready_rate"]


def load_trace(path: str) -> dict:
    with open(path) as f:
        return json.load(f)


def synthetic_trace(n_seq: int, n_layer: int, n_expert: int, top_k: int, prompt_len: int = 32, reply_len: int = 32,
                    zipf: float = 1.2, seed: int = 0) -> dict:
    """Seeded stand-in for a recorded trace: per layer a Zipf(zipf) popularity over a random expert
    permutation, top_k distinct experts per token."""
    rng = np.random.default_rng(seed)
    p = 1.0 / np.arange(1, n_expert + 1) ** zipf
    p /= p.sum()
    perm = [rng.permutation(n_expert) for _ in range(n_layer)]
    trace = {}
    for s in range(n_seq):
        seq = {"prompt_len": prompt_len}
        for l in range(n_layer):
            seq[str(l)] = {str(t): sorted(int(e) for e in perm[l][rng.choice(n_expert, size=top_k, replace=False, p=p)])
                           for t in range(prompt_len + reply_len)}
        trace[str(s)] = seq
    return trace


def sequence_forwards(seq: dict, n_layer: int, max_new_tokens: int | None = None):
    """[(seq_len, [ids of layer 0, ids of layer 1, ...]), ...]: the prefill forward, then one forward
    per reply token (transformers-deepseek-moe.py:66-88)."""
    prompt_len = int(seq["prompt_len"])
    reply_len = len(seq["0"]) - prompt_len
    if max_new_tokens is not None:
        reply_len = min(reply_len, max_new_tokens)
    prefill = []
    for l in range(n_layer):
        ids = set()
        for t in range(prompt_len):
            ids.update(seq[str(l)][str(t)])
        prefill.append(sorted(ids))
    out = [(prompt_len, prefill)]
    for t in range(prompt_len, prompt_len + reply_len):
        out.append((1, [list(seq[str(l)][str(t)]) for l in range(n_layer)]))
    return out


def oracle_tensors(trace: dict, n_layer: int, top_k: int, max_new_tokens: int | None = None):
    """The four arrays the MIN policy is loaded from (reference: cache.cpp:592-644 reads them as
    entry_to_metas [n_decode_forward, 2] = (sequence, reply index), prefill_expert_len [n_seq, L],
    prefill_expert_selection [n_seq, L, max_len], decode_expert_selection [n_decode_forward, L, k])."""
    seqs = sorted(trace, key=int)
    fw = [sequence_forwards(trace[s], n_layer, max_new_tokens) for s in seqs]
    max_len = max(max(len(ids) for ids in f[0][1]) for f in fw)
    plen = np.zeros((len(seqs), n_layer), np.int32)
    psel = np.zeros((len(seqs), n_layer, max(max_len, 1)), np.int32)
    metas, dsel = [], []
    for si, f in enumerate(fw):
        for l, ids in enumerate(f[0][1]):
            plen[si, l] = len(ids)
            psel[si, l, :len(ids)] = ids
        for r, (_, layers) in enumerate(f[1:]):
            metas.append((si, r))
            row = np.zeros((n_layer, top_k), np.int32)
            for l, ids in enumerate(layers):
                if len(ids) != top_k:
                    raise ValueError("a decode token of sequence %s has %d experts in layer %d, expected %d"
                                     % (seqs[si], len(ids), l, top_k))
                row[l] = ids
            dsel.append(row)
    em = np.asarray(metas, np.int64).reshape(-1, 2)
    ds = np.stack(dsel) if dsel else np.zeros((0, n_layer, top_k), np.int32)
    return em, plen, psel, ds


def expert_pattern(layer: int, expert: int, n_expert: int, nbytes: int) -> np.ndarray:
    """The bytes the replay gives expert (layer, expert) on the HIP backend: distinct per expert, never zero."""
    rng = np.random.default_rng(1000003 * layer + expert)
    return rng.integers(1, 256, nbytes, dtype=np.uint8)


def replay(trace: dict, n_layer: int, n_expert: int, top_k: int, max_new_tokens: int | None = None,
           skip_first_prompts: int = 0, backend: int = L.BACKEND_HOST, expert_bytes: int = 64, on_expert=None,
           **cfg) -> dict:
    """One configuration: every sequence of the trace through a fresh engine; returns the engine's
    report (per-stage hit / ready / prefetch-hit counts and rates) plus its raw counters.

    backend L.BACKEND_HOST (default): no GPU, copies are memcpy's, the experts carry no weights (the
    reference's stand-in model, whose experts do nothing).  L.BACKEND_HIP: the same hook sequence with
    real slots in HBM and real copies from pinned host memory on the copy stream; every expert holds
    expert_pattern(...) of expert_bytes bytes.  on_expert(pm, layer, expert) is called between
    report_one_expert and one_expert_done, when the expert's slot must hold its bytes."""
    if backend == L.BACKEND_HIP:
        return _replay_hip(trace, n_layer, n_expert, top_k, max_new_tokens, skip_first_prompts, expert_bytes,
                           on_expert, cfg)
    m = ModuleMeta(n_layer, n_expert)
    m.init_param_list(["w"])
    d = {"num_expert_per_token": str(top_k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    pm = PrefetchMngr(m, backend=L.BACKEND_HOST)
    bufs = []
    for l in range(n_layer):
        for e in range(n_expert):
            b = np.zeros(64, np.uint8)            # the experts carry no weights: only residency is simulated
            bufs.append(b)
            pm.add_one_expert_param(b, l, e, "w")
    pm._keep.append(bufs)
    pm.init_gpu_mem_buffer()
    pm.launch_thread()
    try:
        return _drive(pm, trace, n_layer, top_k, max_new_tokens, skip_first_prompts, on_expert, cfg)
    finally:
        pm.close()


def _drive(pm, trace, n_layer, top_k, max_new_tokens, skip_first_prompts, on_expert, cfg) -> dict:
    """The hook sequence of the reference's stand-in model, forward by forward
    (transformers-deepseek-moe.py:36-49 inside :66-88)."""
    if str(cfg.get("cache_policy", "")).lower() == "min":
        pm.load_oracle(*oracle_tensors(trace, n_layer, top_k, max_new_tokens))
    for si, s in enumerate(sorted(trace, key=int)):
        pm.set_cur_seq(si)
        for seq_len, layers in sequence_forwards(trace[s], n_layer, max_new_tokens):
            pm.report_moe_layer_logits(0, None, seq_len=seq_len)
            for l, ids in enumerate(layers):
                order = pm.report_one_layer(l, np.asarray(ids, np.int64))
                for e in order:
                    pm.report_one_expert(l, int(e))
                    if on_expert is not None:
                        on_expert(pm, l, int(e))
                    pm.one_expert_done(l, int(e))
                pm.one_moe_layer_done(l)
    pm.drain()
    out = pm.report(skip_first_prompts)
    out.update({"counter_" + k: v for k, v in pm.counters().items()})
    return out


def _replay_hip(trace, n_layer, n_expert, top_k, max_new_tokens, skip_first_prompts, expert_bytes, on_expert, cfg):
    from .engine import PinnedBuffer
    m = ModuleMeta(n_layer, n_expert)
    m.init_param_list(["w"])
    d = {"num_expert_per_token": str(top_k)}
    d.update({a: str(b) for a, b in cfg.items()})
    m.init_from_map(d)
    m.handle_uninited_configs()
    pm = PrefetchMngr(m, backend=L.BACKEND_HIP, compute_stream=0)   # the engine makes its own compute stream
    stage = PinnedBuffer(expert_bytes * n_layer * n_expert)
    pm._keep.append(stage)
    for l in range(n_layer):
        for e in range(n_expert):
            base = (l * n_expert + e) * expert_bytes
            stage.array[base: base + expert_bytes] = expert_pattern(l, e, n_expert, expert_bytes)
            pm.add_one_expert_param(stage.array[base: base + expert_bytes], l, e, "w")
    pm.init_gpu_mem_buffer()
    pm.launch_thread()
    try:
        return _drive(pm, trace, n_layer, top_k, max_new_tokens, skip_first_prompts, on_expert, cfg)
    finally:
        pm.close()


def sweep(trace: dict, n_layer: int, n_expert: int, top_k: int, policies=("min", "lru"), per_layer=(True, False),
          reorder=(False, True), cache_rates=None, max_new_tokens: int | None = None):
    """The reference's policy sweep (runner.py:36-45): demand fetching only, no early pre-emption."""
    if cache_rates is None:
        cache_rates = [c / 64 for c in (1, 2, 4, 8, 12, 16, 24, 32, 48, 64)]
    rows = []
    for policy in policies:
        for pl in per_layer:
            for ro in reorder:
                for rate in cache_rates:
                    rep = replay(trace, n_layer, n_expert, top_k, max_new_tokens, cache_policy=policy,
                                 per_layer_cache=pl, reorder_experts=ro, early_preempt=False,
                                 num_predict_expert_per_layer=0, cache_rate=rate)
                    rows.append({"cache_policy": policy, "per_layer_cache": pl, "reorder_experts": ro,
                                 "cache_rate": rate, **{c: rep[c] for c in CSV_COLUMNS[4:]}})
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--trace", help="routing trace (JSON, the reference's format)")
    ap.add_argument("--synthetic", action="store_true", help="use a seeded Zipf trace instead of a file")
    ap.add_argument("--layers", type=int, default=27)
    ap.add_argument("--experts", type=int, default=64)
    ap.add_argument("--top-k", type=int, default=6)
    ap.add_argument("--sequences", type=int, default=4)
    ap.add_argument("--prompt-len", type=int, default=32)
    ap.add_argument("--reply-len", type=int, default=32)
    ap.add_argument("--zipf", type=float, default=1.2)
    ap.add_argument("--max-new-tokens", type=int, default=None)
    ap.add_argument("--policies", default="min,lru")
    ap.add_argument("--cache-rates", default=None, help="comma separated; default: the reference's ten rates")
    ap.add_argument("--out", default="-")
    a = ap.parse_args(argv)
    if bool(a.trace) == bool(a.synthetic):
        ap.error("give exactly one of --trace and --synthetic")
    trace = load_trace(a.trace) if a.trace else synthetic_trace(a.sequences, a.layers, a.experts, a.top_k,
                                                                a.prompt_len, a.reply_len, a.zipf)
    rates = [float(x) for x in a.cache_rates.split(",")] if a.cache_rates else None
    rows = sweep(trace, a.layers, a.experts, a.top_k, policies=a.policies.split(","), cache_rates=rates,
                 max_new_tokens=a.max_new_tokens)
    f = sys.stdout if a.out == "-" else open(a.out, "w", newline="")
    w = csv.DictWriter(f, fieldnames=CSV_COLUMNS)
    w.writeheader()
    w.writerows(rows)
    if f is not sys.stdout:
        f.close()


if __name__ == "__main__":
    main()
