#!/usr/bin/env python3
"""MoE-layer decode benchmark on one MI355X.

Workload (BASELINE.json configs[1]): one DeepSeek-MoE-16B-shaped MoE layer in decode,
int4-g128 experts (hidden 2048, 64 routed experts of intermediate 1408, top-6 softmax
without renormalisation, shared expert of intermediate 2816), bf16 activations, gate
logits biased to Zipf(1.2) popularity.  A step is one layer forward (gate -> top-k ->
dispatch -> cache hooks -> grouped int4 SwiGLU experts -> combine) over T tokens; steps
walk a stack of 27 such layers (7.8 GB of expert images) so that no step finds its
weights in a cache left warm by the previous one.

value      tokens/s with every routed expert resident in its HBM slot (steady-state hits)
roofline   HBM roofline of the dominant kernel (int4 w13 + SwiGLU GEMV)
cache_run  the same stack at cache rate 0.375 (24 of 64 experts per layer resident, LRU);
           PCIe-inclusive, reported beside `value`, never as it
cpu_baseline  the fp32 CPU restatement (per-expert F.linear loop) timed on this host
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2700)
    ap.add_argument("--warmup", type=int, default=270)
    ap.add_argument("--tokens", type=int, default=1, help="tokens per step (decode batch): 1 to 64 stay on the GEMV kernels")
    ap.add_argument("--layers", type=int, default=27)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-cache-run", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill (matrix-core) legs")
    ap.add_argument("--only", default="", help="profiling aid: run only these prefill legs (comma list of "
                    "qwen, deepseek, mixtral, qwen2q4k; other = the decode legs of the other configurations; tN = the "
                    "DeepSeek-shaped decode layer at N tokens per step) and print their "
                    "results, without the decode benchmark")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="profiling aid: also run a plain 256 MiB read + 256 MiB write elementwise kernel three "
                         "times, the known-size reference for FETCH_SIZE / WRITE_SIZE counters")
    return ap.parse_args()


def timed_steps(pm, xs, L_, steps, torch):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        pm.forward(i % L_, xs[i % len(xs)], out=xs_out, stream_guard=False)  # inputs are complete (synchronised above)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def launches_timed(torch, launch_n, n, replay_once=False):
    """Average duration (us) of n launches issued by launch_n(n) on the current stream, between ONE HIP event pair.
    The launches go into a HIP graph first and the graph is replayed between the events: issued one by one from
    Python (a ctypes call costs the host about 10 us) a kernel shorter than that is timed at the host's pace, not at
    its own.  launch_n must only launch kernels (no allocation, no synchronisation, nothing that clears memory).
    replay_once: the launches carry a sequence number in their arguments that must not come twice (the launches
    that hand their gate logits over inside the launch): one graph is recorded and replayed untimed, a second one
    with the following numbers is recorded and its FIRST replay is the timed one.
    Falls back to the plain loop when the capture is refused."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    try:
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side, capture_error_mode="thread_local"):
                launch_n(n)
            g.replay()                      # once untimed
            torch.cuda.synchronize()
            if replay_once:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side, capture_error_mode="thread_local"):
                    launch_n(n)
                torch.cuda.synchronize()
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n, "a HIP graph of %d launches replayed between one HIP event pair" % n
    except Exception as ex:  # noqa: BLE001 - any refusal of the capture: time the plain loop
        print("[bench] graph capture refused (%s): timing the plain launch loop" % str(ex).split("\n")[0][:120],
              file=sys.stderr, flush=True)
        torch.cuda.synchronize()
        e0.record()
        launch_n(n)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n, "%d back-to-back launches between one HIP event pair" % n


PROFILE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")
DECODE_SOURCES = ["promoe_amd/csrc/moe_kernels.hip", "promoe_amd/csrc/moe_device.h"]
PREFILL_SOURCES = ["promoe_amd/csrc/moe_prefill.hip", "promoe_amd/csrc/moe_device.h"]


def source_hash(sources):
    import hashlib
    h = hashlib.sha256()
    root = os.path.dirname(os.path.abspath(__file__))
    for rel in sources:
        with open(os.path.join(root, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def recorded(fname, key, hash_key, sources):
    """A figure that cannot be measured in-process (HBM bytes per launch from FETCH_SIZE / WRITE_SIZE counter runs,
    a kernel's duration inside the timed steps from rocprofv3's kernel trace), read from the committed summary
    `profiles/<fname>` (a line `<key>: <number>`); None when the summary is missing or was taken on other kernel
    sources than the ones in the tree (the summary records their hash in the line `<hash_key>: <16 hex digits>`)."""
    import re
    try:
        text = open(os.path.join(PROFILE_DIR, fname)).read()
    except OSError:
        return None
    m = re.search(r"^\s*%s:\s*([0-9.]+)\s*$" % re.escape(key), text, re.M)
    hsh = re.search(r"^\s*%s:\s*([0-9a-f]{16})\s*$" % re.escape(hash_key), text, re.M)
    if not m or not hsh or hsh.group(1) != source_hash(sources):
        return None
    v = float(m.group(1))
    return int(v) if v == int(v) else v


def recorded_decode(key, fname="hbm_traffic_decode_and_prefill.md"):
    return recorded(fname, key, "decode_kernel_source_sha256_16", DECODE_SOURCES)


def recorded_prefill(key, fname="hbm_traffic_decode_and_prefill.md"):
    return recorded(fname, key, "prefill_kernel_source_sha256_16", PREFILL_SOURCES)


def cpu_baseline(T, H, I, E, I_sh, k, threads, budget_s=12.0):
    """The oracle's fp32 forward in the reference's structure (per-expert loop), on host cores."""
    import numpy as np
    import torch
    from oracle import moe_oracle as O
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    mk = lambda n, kk: (torch.randn(n, kk, generator=g) * 0.02).numpy()
    experts = [(mk(I, H), mk(I, H), mk(H, I)) for _ in range(E)]
    shared = (mk(I_sh, H), mk(I_sh, H), mk(H, I_sh))
    wg = O.round_bf16(mk(E, H))
    bias = O.zipf_gate_bias(E, 1.2)
    # a bounded sample: layer steps of the same shape until about 12 s of CPU work are spent
    times = []
    t_begin = time.perf_counter()
    rep = 0
    while rep < 5 or (time.perf_counter() - t_begin < budget_s and rep < 5000):
        x = O.synth_acts(T, H, seed=rep + 1)
        t0 = time.perf_counter()
        lg = (O.gate_logits(x, wg) + bias[None, :]).astype(np.float32)
        O.moe_forward(x, wg, experts, k, 0, shared=shared, logits=lg)
        times.append(time.perf_counter() - t0)
        rep += 1
    steady = times[2:] if len(times) > 4 else times[1:]
    return T * len(steady) / sum(steady), statistics.median(steady), len(steady)


MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 / fp16


def prefill_leg(torch, name, T, H, E, I, k, I_sh, fmt, gated, mode, steps=20):
    """One MoE layer forward at prefill size on the matrix-core kernels (all experts resident,
    uniform gate): whole-layer time and the two expert GEMM launches on their own."""
    from promoe_amd import ops, synth, layout as LY, _lib as L
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16)
    wg = (torch.randn(E + (1 if gated else 0), H, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    if fmt == L.FMT_BF16:
        img = (torch.randn(E, 3 * I * H, device=dev, generator=g) * 0.02).to(torch.bfloat16)
        sh = (torch.randn(3 * I_sh * H, device=dev, generator=g) * 0.02).to(torch.bfloat16) if I_sh else None
        wbytes = E * 3 * I * H * 2 + 3 * I_sh * H * 2
    elif fmt == L.FMT_Q4K:
        img = synth.random_q4k_images(E, H, I, dev, g)
        sh = synth.random_q4k_images(1, H, I_sh, dev, g)[0] if I_sh else None
        wbytes = E * LY.q4k_layout(H, I)["total_bytes"] + (LY.q4k_layout(H, I_sh)["total_bytes"] if I_sh else 0)
    else:
        img = synth.random_int4_images(E, H, I, dev, g)
        sh = synth.random_int4_images(1, H, I_sh, dev, g)[0] if I_sh else None
        wbytes = E * LY.int4_layout(H, I)["total_bytes"] + (LY.int4_layout(H, I_sh)["total_bytes"] if I_sh else 0)
    table = torch.tensor([img[e].data_ptr() for e in range(E)], dtype=torch.int64, device=dev)
    y = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    logits = torch.empty(T, wg.shape[0], dtype=torch.float32, device=dev)
    d = ops.Dispatch(T, k, E, min(E, T * k), dev)
    ws = None

    def layer():
        nonlocal ws
        ops.gate_logits(x, wg, None, out=logits)
        idx, w = ops.topk(logits, k, mode, E=E)
        ops.dispatch(idx, E, out=d)
        ws = ops.experts_prefill(x, d, table, sh, H, I, I_sh, fmt, ws=ws)
        ops.combine(ws[0], ws[1], w, d.pos_of_pair, logits[:, E] if gated else None, T, H, k, out=y)

    def timed(fn, n):
        fn(); fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n

    t_layer = timed(layer, steps)
    assert int(ws[2].cpu()[0]) == 0
    t_w13 = timed(lambda: ops.experts_prefill(x, d, table, sh, H, I, I_sh, fmt, phases=1, ws=ws), steps)
    t_w2 = timed(lambda: ops.experts_prefill(x, d, table, sh, H, I, I_sh, fmt, phases=2, ws=ws), steps)
    flops = 2.0 * T * k * 3 * I * H + 2.0 * T * 3 * I_sh * H
    ach = flops * 2 / 3 / t_w13 / 1e12
    tag = name.split("-")[0].split(".")[0].lower() + ("_q4k" if fmt == L.FMT_Q4K else ("_bf16" if fmt == L.FMT_BF16 else "_int4"))
    return {"workload": name, "tokens": T, "tokens_per_s": T / t_layer, "ms_per_layer": t_layer * 1e3,
            "expert_flops": flops, "weight_bytes": wbytes,
            "layer_TFLOPs": (flops + 2.0 * T * wg.shape[0] * H) / t_layer / 1e12,
            "roofline": {"bound": "mfma", "kernel": "k_prefill_%s<true> (w13 + SwiGLU, routed + shared in one launch)" %
                         ("gemm" if fmt == L.FMT_BF16 else ("int4<q4_K>" if fmt == L.FMT_Q4K else "int4")),
                         "achieved": ach, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": ach / MFMA_PEAK_TFLOPS,
                         # HBM bytes per launch from the committed FETCH_SIZE / WRITE_SIZE counter summary (null for a
                         # leg without counters, or when the kernel sources changed since they were taken)
                         "traffic": recorded_prefill("prefill_%s_w13_traffic_bytes_per_launch" % tag), "avg_launch_us": t_w13 * 1e6,
                         "algorithmic_flops_per_launch": flops * 2 / 3,
                         "method": "%d back-to-back launches (tile-list kernel included) between one HIP event pair" % steps},
            "w2_launch_us": t_w2 * 1e6, "w2_TFLOPs": flops / 3 / t_w2 / 1e12}


def decode_leg(torch, name, fmt, T, H, E, I, k, I_sh, gated, mode, layers, zipf, steps=200):
    """Decode-size MoE layer forward at kernel level, every expert resident in HBM (images of `layers`
    layers in rotation, far more than the caches hold): route -> experts -> combine on one stream."""
    import numpy as np
    from promoe_amd import ops, synth, layout as LY, _lib as L
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(9)
    q4k = fmt == L.FMT_Q4K
    mk = synth.random_q4k_images if q4k else synth.random_int4_images
    lay = LY.q4k_layout if q4k else LY.int4_layout
    tiles = T > ops.gemv_max_tokens(fmt)   # the rule of moe_forward: larger token groups take the matrix-core tile kernels
    if tiles:
        def run_experts(x, d_, table, sh, H_, I_, I_sh_, phases=3, ws=None):
            return ops.experts_prefill(x, d_, table, sh, H_, I_, I_sh_, fmt, phases=phases, ws=ws)
    else:
        run_experts = ops.experts_decode_q4k if q4k else ops.experts_decode_int4
    imgs, shs, gws, biases, tables = [], [], [], [], []
    for l in range(layers):
        imgs.append(mk(E, H, I, dev, g))
        shs.append(mk(1, H, I_sh, dev, g)[0] if I_sh else None)
        gws.append((torch.randn(E + (1 if gated else 0), H, device=dev, generator=g) * 0.02).to(torch.bfloat16))
        b = None
        if zipf:
            b = torch.from_numpy(np.concatenate([synth.zipf_bias(E, zipf, 100 + l), np.zeros(1 if gated else 0, np.float32)])).to(dev)
        biases.append(b)
        tables.append(torch.tensor([imgs[l][e].data_ptr() for e in range(E)], dtype=torch.int64, device=dev))
    xs = [torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16) for _ in range(8)]
    y = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    rows = E + (1 if gated else 0)
    logits = torch.empty(T, rows, dtype=torch.float32, device=dev)
    d = ops.Dispatch(T, k, E, min(E, T * k), dev)
    ws = None
    nact = []

    # one token, int4: the path moe_forward takes (routing inside the w13 kernel, w2 + combine in one launch)
    token_path = T == 1 and not q4k
    unit_ws = torch.zeros(32 * k, dtype=torch.uint8, device=dev)
    ws_tok = None
    # 2 to 16 tokens, int4: likewise (gate rows and routing inside the w13 launch, then w2, then the combine)
    batch_path = (not q4k) and T >= 2 and ops.decode_batch_int4_gate_fits(T, E, k, H, I, I_sh, rows)
    gate_ws = ops.GateWorkspace(dev, max(T, 1), rows) if batch_path else None
    ws_b = None

    def step(i, phases=3, route=True):
        nonlocal ws, ws_tok, ws_b
        l, x = i % layers, xs[i % len(xs)]
        if batch_path:
            ws_b = ops.decode_batch_int4_gate(x, gws[l], biases[l], E, k, mode, tables[l], shs[l], H, I, I_sh, gate_ws,
                                              phases=phases, ws=ws_b)
            if phases == 3:
                ops.combine(ws_b[4], ws_b[5], ws_b[2], ws_b[3].pos_of_pair, ws_b[0][:, E] if gated else None, T, H, k, out=y)
            return
        if token_path and phases == 3:
            ops.gate_logits(x, gws[l], biases[l], out=logits)
            ws_tok = ops.decode_token_int4(x, logits, E, k, mode, tables[l], shs[l], H, I, I_sh, ws=ws_tok, phases=5,
                                           unit_ws=unit_ws, sg_logit=logits[:, E] if gated else None, y=y)
            return
        if route:
            ops.gate_logits(x, gws[l], biases[l], out=logits)
            idx, w = ops.topk(logits, k, mode, E=E)
            ops.dispatch(idx, E, out=d)
            step.w = w
        ws = run_experts(x, d, tables[l], shs[l], H, I, I_sh, phases=phases, ws=ws)
        if phases == 3:
            ops.combine(ws[0], ws[1], step.w, d.pos_of_pair, logits[:, E] if gated else None, T, H, k, out=y)

    def timed(fn, n):
        for i in range(min(n, 2 * layers)):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n

    for i in range(4 * layers):
        step(i)
        nact.append(int((ws_tok[2] if token_path else (ws_b[3] if batch_path else d)).n_active.cpu()[0]))
    if token_path:   # the one-token path against the separate kernels on the same input
        y_tok = y.float().clone()
        token_path = False
        step(4 * layers - 1)
        token_path = True
        assert int(ws_tok[5].cpu()[0]) == 0
        assert float((y_tok - y.float()).abs().max()) <= 1e-2 * float(y.float().abs().max())
    assert int((ws_b[6] if batch_path else ws[2]).cpu()[0]) == 0
    t_layer = timed(step, steps)
    # the w13 + SwiGLU GEMV alone, back to back, with the routing of the last full step kept
    for i in range(2 * layers):
        step(i, phases=1, route=False)
    torch.cuda.synchronize()
    w13_us_leg, w13_method = launches_timed(torch, lambda n: [step(i, phases=1, route=False) for i in range(n)] and None, steps,
                                            replay_once=batch_path)
    t_w13 = w13_us_leg * 1e-6
    D = float(np.mean(nact))
    D_last = nact[-1]
    lr = lay(H, I)
    ls = lay(H, I_sh) if I_sh else {"total_bytes": 0, "off2_q": 0}
    step_bytes = D * lr["total_bytes"] + ls["total_bytes"] + rows * H * 2 + 2 * T * H * 2
    w13_bytes = D_last * lr["off2_q"] + ls["off2_q"] + 2 * T * H
    if batch_path:   # the launch also reads the gate matrix and its bias
        w13_bytes += rows * H * 2 + E * 4
    ach = w13_bytes / t_w13 / 1e9
    return {"workload": name, "tokens": T, "layers_in_rotation": layers, "tokens_per_s": T / t_layer,
            "us_per_layer": t_layer * 1e6, "distinct_routed_experts_per_step": D,
            "algorithmic_bytes_per_step": step_bytes, "layer_GBps": step_bytes / t_layer / 1e9,
            "roofline": {"bound": "hbm", "kernel": ("k_gemv_int4_mfma%s<route> (gate rows + routing + w13 + SwiGLU in one launch)"
                                                    % ("" if T <= 8 and H <= 2048 else "_kc")) if batch_path else
                                                   ("k_prefill_int4 (w13 + SwiGLU)" if tiles else
                                                    "k_gemv_int4%s (w13 + SwiGLU)" % (("_mfma_kc<q4_K>" if T > 1 else "<q4_K>") if q4k else ("_mfma_kc" if (T > 16 or H > 2048) and T > 1 else ("_mfma" if T > 1 else "")))),
                         "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None,
                         "algorithmic_bytes_per_launch": w13_bytes, "avg_launch_us": t_w13 * 1e6,
                         "method": w13_method}}


def other_configs(torch):
    """Decode legs of the Mixtral-shaped int4 and Qwen2-57B-shaped q4_K configurations."""
    from promoe_amd import _lib as L
    out = []
    for T in (1, 64):
        out.append(decode_leg(torch, "Mixtral-8x7B-shaped layer, int4-g128 experts, decode T=%d, all resident, "
                              "uniform routing" % T, L.FMT_INT4_G128, T, 4096, 8, 14336, 2, 0, False, 2, 4, None,
                              steps=60 if T == 1 else 20))
    out.append(decode_leg(torch, "Qwen2-57B-A14B-shaped layer, q4_K experts, decode T=3 (three sequences), all "
                          "resident, Zipf(1.1)", L.FMT_Q4K, 3, 3584, 64, 2560, 8, 20480, True, 0, 3, 1.1, steps=60))
    out.append(decode_leg(torch, "Qwen2-57B-A14B-shaped layer, q4_K experts, decode T=32, all resident, Zipf(1.1)",
                          L.FMT_Q4K, 32, 3584, 64, 2560, 8, 20480, True, 0, 3, 1.1, steps=30))
    return out


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)" % a.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    from promoe_amd import synth, layout as LY
    from promoe_amd._lib import lib
    if a.copy_calibration:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    if a.only:
        from promoe_amd import _lib as L
        legs = {"qwen": ("Qwen1.5-MoE-A2.7B-shaped layer, bf16 experts, prefill T=2048, all resident",
                         2048, 2048, 60, 1408, 4, 5632, L.FMT_BF16, True, 0, 20),
                "deepseek": ("DeepSeek-MoE-16B-shaped layer, int4-g128 experts, prefill T=2048, all resident",
                             2048, 2048, 64, 1408, 6, 2816, L.FMT_INT4_G128, False, 0, 20),
                "mixtral": ("Mixtral-8x7B-shaped layer, int4-g128 experts, prefill T=4096, all resident",
                            4096, 4096, 8, 14336, 2, 0, L.FMT_INT4_G128, False, 2, 5)}
        legs["qwen2q4k"] = ("Qwen2-57B-A14B-shaped layer, q4_K experts, prefill T=512, all resident",
                            512, 3584, 64, 2560, 8, 20480, L.FMT_Q4K, True, 0, 10)
        names = a.only.split(",")
        res = {"prefill": [prefill_leg(torch, *legs[n][:-1], steps=legs[n][-1]) for n in names if n in legs]}
        if "other" in names:
            res["other_decode_configs"] = other_configs(torch)
        # t4, t16, t64, ...: the decode kernels of the DeepSeek-shaped layer at that many tokens per step
        tn = [int(n[1:]) for n in names if n[:1] == "t" and n[1:].isdigit()]
        if tn:
            res["decode_by_T"] = [decode_leg(torch, "DeepSeek-MoE-16B-shaped layer, int4-g128 experts, decode T=%d, all "
                                             "resident, Zipf(1.2)" % t, L.FMT_INT4_G128, t, 2048, 64, 1408, 6, 2816, False, 0,
                                             8, 1.2, steps=108) for t in tn]
        print(json.dumps(res))
        return

    global xs_out
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    H, I, E, I_sh, k, L_ = 2048, 1408, 64, 2816, 6, a.layers
    T = a.tokens
    t_setup = time.perf_counter()
    stack = synth.Int4Stack(L_, E, H, I, I_sh, k, dev, zipf=1.2, seed=0)
    print("[bench] stack of %d layers x %d experts (%.2f GB of images) built in %.1f s" %
          (L_, E, stack.expert_bytes * L_ * E / 1e9, time.perf_counter() - t_setup), file=sys.stderr, flush=True)

    # ---- steady-state hits: every expert resident -------------------------------------
    pm = stack.engine(max(64, T), cache_rate=1.0, cache_policy="lru")
    import numpy as np
    for l in range(L_):                      # bring every expert into its slot
        pm.acquire_layer(l, np.arange(E, dtype=np.int64))
        pm.release_layer(l)
    pm.drain()
    base_ctr = pm.counters()

    def run(Tn, steps, warmup):
        global xs_out
        xs = stack.acts(Tn, 8, seed=1)
        xs_out = torch.empty_like(xs[0])
        timed_steps(pm, xs, L_, warmup, torch)
        return timed_steps(pm, xs, L_, steps, torch)

    # `value`: median over repeats of a timed region of at least --steps steps and at least 0.2 s (a 20-step
    # region is 0.4 ms of wall clock: one scheduler hiccup on the host moves it by 10 %)
    dt_probe = run(T, a.steps, a.warmup)
    n_timed = max(a.steps, int(0.2 / max(dt_probe / a.steps, 1e-7)) + 1)
    n_timed = (n_timed + L_ - 1) // L_ * L_                 # whole passes over the layer stack
    xs_v = stack.acts(T, 8, seed=1)
    xs_out = torch.empty_like(xs_v[0])
    reps = sorted(timed_steps(pm, xs_v, L_, n_timed, torch) for _ in range(5))
    dt = reps[len(reps) // 2] * a.steps / n_timed           # per --steps steps, from the median repeat
    c1 = pm.counters()
    assert c1["miss"] == base_ctr["miss"], "steady-state run took cache misses"
    value = T * a.steps / dt
    timing = {"timed_steps_per_repeat": n_timed, "repeats": len(reps), "statistic": "median",
              "ms_per_step_min": reps[0] / n_timed * 1e3, "ms_per_step_max": reps[-1] / n_timed * 1e3,
              "first_region_of_exactly_steps_ms_per_step": dt_probe / a.steps * 1e3}

    xs = stack.acts(T, 8, seed=1)
    d_steps = min(a.steps, 20 * L_)
    act0 = pm.counters()["activated"]
    timed_steps(pm, xs, L_, d_steps, torch)
    # distinct routed experts per step (D) for the algorithmic byte count
    D = (pm.counters()["activated"] - act0) / d_steps
    lay_r, lay_s = LY.int4_layout(H, I), LY.int4_layout(H, I_sh)
    w13_bytes = D * lay_r["off2_q"] + lay_s["off2_q"] + 2 * T * H       # w13 sections + x
    layer_bytes = D * lay_r["total_bytes"] + lay_s["total_bytes"] + E * H * 2 + 2 * T * H * 2

    # dominant kernel (w13 + SwiGLU GEMV): average duration over back-to-back launches on the
    # launch stream, bracketed by ONE pair of HIP events (agrees with rocprofv3's kernel trace)
    from promoe_amd import ops
    routed = []
    tables = []
    for l in range(L_):
        lg = ops.gate_logits(xs[0], stack.gate_w[l], stack.gate_bias[l])
        idx_l, _ = ops.topk(lg, k, 0)
        routed.append(ops.dispatch(idx_l, E))
        tables.append(pm.expert_ptr_table(l))
        pm.flush_table(l, torch.cuda.current_stream().cuda_stream)
    P = T * k
    ws = (torch.empty(P, H, dtype=torch.float32, device=dev), torch.empty(T, H, dtype=torch.float32, device=dev),
          torch.zeros(1, dtype=torch.int32, device=dev), torch.empty(P, I, dtype=torch.bfloat16, device=dev),
          torch.empty(T, I_sh, dtype=torch.bfloat16, device=dev))

    class _Tab:  # the engine's device table row, addressed like a tensor
        def __init__(self, p): self.p = p
        def data_ptr(self): return self.p

    # one token: the timed path runs the w13 GEMV that sums the gate rows in its first workgroups and derives the
    # routing itself; measure that kernel (launched as moe_forward launches it: the gate logits are an output)
    logits_out = torch.empty(1, E + 1, dtype=torch.float32, device=dev)
    gate_ws = ops.GateWorkspace(dev)
    ws_tok = None

    # 2 to 16 tokens: likewise (the w13 launch of a batch sums the gate rows and routes by itself)
    batch_fused = T >= 2 and ops.decode_batch_int4_gate_fits(T, E, k, H, I, I_sh, E)
    gate_ws_b = ops.GateWorkspace(dev, T, E + 1) if batch_fused else None
    ws_b = None

    def w13_only(n):
        nonlocal ws_tok, ws_b
        for i in range(n):
            l = i % L_
            if batch_fused:
                ws_b = ops.decode_batch_int4_gate(xs[i % len(xs)], stack.gate_w[l], stack.gate_bias[l], E, k, 0, _Tab(tables[l]),
                                                  stack.shared[l], H, I, I_sh, gate_ws_b, phases=1, ws=ws_b)
            elif T == 1:
                ws_tok = ops.decode_token_int4(xs[i % len(xs)], logits_out, E, k, 0, _Tab(tables[l]), stack.shared[l], H, I,
                                               I_sh, ws=ws_tok, phases=1, gate=(stack.gate_w[l], stack.gate_bias[l], gate_ws))
            else:
                ops.experts_decode_int4(xs[0], routed[l], _Tab(tables[l]), stack.shared[l], H, I, I_sh, phases=1, ws=ws)
    w13_only(2 * L_)
    torch.cuda.synchronize()
    n_k = 20 * L_
    w13_us, w13_method = launches_timed(torch, w13_only, n_k, replay_once=(T == 1 or batch_fused))
    assert int((ws_tok[5] if T == 1 else (ws_b[6] if batch_fused else ws[2])).cpu()[0]) == 0
    D_k = float(np.mean([int(r.n_active.cpu()[0]) for r in routed]))
    if batch_fused:   # (the launches above route xs[i % 8] themselves: take the last one's count)
        D_k = float(int(ws_b[3].n_active.cpu()[0]))
    gate_bytes = (E * H * 2 + E * 4) if (T == 1 or batch_fused) else 0   # gate rows + bias, read by the same launch
    w13_bytes_k = D_k * lay_r["off2_q"] + lay_s["off2_q"] + 2 * T * H + gate_bytes
    achieved = w13_bytes_k / (w13_us * 1e-6) / 1e9
    # the same kernel inside the timed steps (between the w2 + combine launches of the neighbouring steps), from
    # the committed rocprofv3 kernel trace of this command; null when the kernel sources changed since
    in_path_us = recorded_decode("decode_w13_in_path_avg_us", "decode_deepseek_int4_T1_kernel_trace.md") if (T == 1 and L_ == 27) else None
    roofline = {"bound": "hbm", "kernel": ("k_w13_token (gate rows + routing + w13 + SwiGLU in one launch)" if T == 1 else
                                           ("k_gemv_int4_mfma%s<route> (gate rows + routing + w13 + SwiGLU in one launch)" % ("" if T <= 8 else "_kc")
                                            if batch_fused else "k_gemv_int4_mfma (w13 + SwiGLU)")),
                "achieved": achieved,
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                # HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs of this kernel at this
                # workload (T=1, 27 layers), scaled by a copy kernel of known size; not measurable in-process:
                # read from the committed counter summary, null when the kernel sources changed since
                "traffic": recorded_decode("decode_w13_traffic_bytes_per_launch") if (T == 1 and L_ == 27) else None,
                "algorithmic_bytes_per_launch": w13_bytes_k, "avg_launch_us": w13_us,
                "avg_launch_us_in_timed_steps": in_path_us,
                "frac_in_timed_steps": (w13_bytes_k / (in_path_us * 1e-6) / 1e9 / HBM_PEAK_GBS) if in_path_us else None,
                "distinct_routed_experts_per_launch": D_k,
                "method": w13_method + "; avg_launch_us_in_timed_steps: rocprofv3 --kernel-trace of this command "
                                       "(profiles/decode_deepseek_int4_T1_kernel_trace.md)"}
    step_us = dt / a.steps * 1e6
    layer = {"algorithmic_bytes_per_step": layer_bytes, "us_per_step": step_us,
             "wall_GBps": layer_bytes / (dt / a.steps) / 1e9,
             "frac_of_hbm_peak": layer_bytes / (dt / a.steps) / 1e9 / HBM_PEAK_GBS,
             "launches_per_step": 2 if T == 1 else (3 if batch_fused else 4),
             "w2_combine_avg_us_in_timed_steps": recorded_decode("decode_w2c_in_path_avg_us", "decode_deepseek_int4_T1_kernel_trace.md") if (T == 1 and L_ == 27) else None}

    sweep = {}
    if not a.no_sweep:
        for Tn in (1, 4, 16, 64):
            if Tn == T:
                sweep[str(Tn)] = value
                continue
            d2 = run(Tn, 20 * L_, 2 * L_)
            sweep[str(Tn)] = Tn * 20 * L_ / d2
    pm.close()

    # ---- the configured cache rate: 24 of 64 experts per layer resident, LRU ------------
    cache_run = None
    as_configured = None
    if not a.no_cache_run:
        def cache_leg(Tn, predict=None, min_precision=0.0):
            """predict: None (demand fetching only), "exact" (every layer of a token sees one hidden state, so the
            gate-as-predictor is always right: what prefetching can hide at best) or "drifting" (the hidden state
            of a token drifts from layer to layer, x_l+1 = x_l + 0.5 noise: predictions made from an earlier
            layer's input are sometimes wrong, as with a real model).  min_precision: requests for a layer whose
            predictions were lately right for less than this share go out empty (0: all go out, as in the
            reference)."""
            cfg = dict(cache_rate=0.375, cache_policy="lru", reorder_experts=True, early_preempt=True,
                       num_predict_expert_per_layer=k if predict else 0)
            if predict:
                cfg.update(layer_predict_interval=1, layer_predict_max_window=10, limit_layer_0_window=10)
            pm2 = stack.engine(16, **cfg)
            if predict:
                # the built-in predictor with the destination layer's gate as the model of every pair
                for src, (f0, f1) in enumerate(pm2.predictor_windows()):
                    for dst in range(f0, f1):
                        pm2.set_predictor_model(src, dst, stack.gate_w[dst], stack.gate_bias[dst])
                if min_precision > 0:
                    pm2.set_predictor_min_precision(min_precision)
                pm2.start_predictor()
            n_tok = 64
            base = stack.acts(Tn, n_tok, seed=3)
            if predict == "drifting":
                gen = torch.Generator(device=dev).manual_seed(11)
                xs2 = []
                for t in range(n_tok):
                    x = base[t].float()
                    row = []
                    for l in range(L_):
                        row.append(x.to(torch.bfloat16))
                        x = (x + 0.5 * torch.randn(x.shape, device=dev, generator=gen)) / (1.25 ** 0.5)
                    xs2.append(row)
                act = lambda step, l: xs2[step % n_tok][l]
            else:
                act = lambda step, l: base[step % n_tok]
            out2 = torch.empty_like(base[0])
            n2 = 40 * L_
            for i in range(10 * L_):              # fill the slots along the Zipf popularity
                pm2.forward(i % L_, act(i // L_, i % L_), out=out2, stream_guard=False)
            torch.cuda.synchronize()
            c0 = pm2.counters()
            t0 = time.perf_counter()
            for i in range(n2):
                pm2.forward(i % L_, act(10 + i // L_, i % L_), out=out2, stream_guard=False)
            torch.cuda.synchronize()
            d3 = time.perf_counter() - t0
            c2 = pm2.counters()
            withheld = pm2.predictor_precision()[1] if predict else None
            pm2.close()
            dl = {kk: c2[kk] - c0[kk] for kk in ("hit", "miss", "prefetch_hit", "prefetch_miss", "ready", "unready",
                                                 "wait_us", "h2d_bytes")}
            return {"cache_rate": 0.375, "policy": "lru", "tokens_per_step": Tn, "tokens_per_s": Tn * n2 / d3,
                    "ms_per_step": d3 / n2 * 1e3,
                    "hit_rate": dl["hit"] / max(dl["hit"] + dl["miss"], 1), "h2d_GB": dl["h2d_bytes"] / 1e9,
                    "h2d_GBps": dl["h2d_bytes"] / d3 / 1e9, "steps": n2, "misses": dl["miss"],
                    "wait_us_per_miss": dl["wait_us"] / max(dl["miss"], 1) if not predict else None,
                    "prefetch_hits": dl["prefetch_hit"], "prefetch_copies": dl["prefetch_miss"],
                    "ready_rate": dl["ready"] / max(dl["ready"] + dl["unready"], 1), "wait_us_total": dl["wait_us"],
                    "predictor_min_precision": min_precision if predict else None, "requests_sent_empty": withheld}
        cache_run = cache_leg(T)
        if T == 1:
            cache_run["with_predictor"] = cache_leg(T, "exact")
            # mispredictions cost copies that evict useful experts: with the predictor's precision feedback on
            # (requests for layers it lately got wrong go out empty) and with every request sent as ranked
            cache_run["with_predictor_drifting_hidden_state"] = cache_leg(T, "drifting", min_precision=0.5)
            cache_run["with_predictor_drifting_hidden_state_every_request_sent"] = cache_leg(T, "drifting")
        # the decode configuration as configured (cache rate 0.375, LRU, demand fetching): T = 1, 4, 16
        as_configured = {}
        for Tn in (1, 4, 16):
            r = cache_run if Tn == T else cache_leg(Tn)
            as_configured[str(Tn)] = {kk: r[kk] for kk in ("tokens_per_s", "ms_per_step", "hit_rate", "h2d_GBps", "misses", "steps")}

    prefill = None
    if not a.no_prefill:
        from promoe_amd import _lib as L
        prefill = [
            prefill_leg(torch, "Qwen1.5-MoE-A2.7B-shaped layer, bf16 experts, prefill T=2048, all resident",
                        2048, 2048, 60, 1408, 4, 5632, L.FMT_BF16, True, 0),
            prefill_leg(torch, "DeepSeek-MoE-16B-shaped layer, int4-g128 experts, prefill T=2048, all resident",
                        2048, 2048, 64, 1408, 6, 2816, L.FMT_INT4_G128, False, 0),
            prefill_leg(torch, "Mixtral-8x7B-shaped layer, int4-g128 experts, prefill T=4096, all resident",
                        4096, 4096, 8, 14336, 2, 0, L.FMT_INT4_G128, False, 2, steps=5),
        ]

    others = None
    if not a.no_prefill:
        others = other_configs(torch)
        from promoe_amd import _lib as L
        prefill.append(prefill_leg(torch, "Qwen2-57B-A14B-shaped layer, q4_K experts, prefill T=512, all resident",
                                   512, 3584, 64, 2560, 8, 20480, L.FMT_Q4K, True, 0, steps=10))

    cpu = None
    cpu_more = None
    if not a.no_cpu:
        threads = 8   # the reference's own torch.set_num_threads(8) (utils/__init__.py:343)
        ncpu = os.cpu_count() or threads
        try:
            ncpu = min(ncpu, len(os.sched_getaffinity(0)))
        except AttributeError:
            pass
        v, med, n_cpu = cpu_baseline(T, H, I, E, I_sh, k, threads)
        cpu = {"value": v, "unit": "tokens/s", "cores": threads, "kind": "port",
               "sample": "the oracle's fp32 per-expert forward (F.linear) of one layer of the same shape, T=%d: %d "
                         "layer steps in about 12 s after 2 warm-ups (median %.1f ms/step); host has %d logical "
                         "cores" % (T, n_cpu, med * 1e3, ncpu)}
        cpu_more = []
        for Tn, thr in ((T, ncpu), (128, threads), (128, ncpu)):   # all cores, and the reference's CPU-runnable T = 128
            if (Tn, thr) == (T, threads):
                continue
            v2, med2, n2c = cpu_baseline(Tn, H, I, E, I_sh, k, thr, budget_s=5.0)
            cpu_more.append({"value": v2, "unit": "tokens/s", "cores": thr, "kind": "port", "tokens_per_step": Tn,
                             "sample": "same forward, T=%d, %d threads: %d layer steps in about 5 s (median %.1f ms/step)"
                                       % (Tn, thr, n2c, med2 * 1e3)})

    roofline_by_T = None
    if not a.no_sweep and T == 1:
        from promoe_amd import _lib as L
        roofline_by_T = {}
        for Tn in (4, 16):
            leg = decode_leg(torch, "DeepSeek-MoE-16B-shaped layer, int4-g128 experts, decode T=%d, all resident, "
                             "Zipf(1.2)" % Tn, L.FMT_INT4_G128, Tn, H, E, I, k, I_sh, False, 0, 8, 1.2, steps=216)
            # a layer step as moe_forward runs it (the timed loop of tokens_per_s_by_T); the leg's own step
            # is launched kernel by kernel from Python and runs at the host's pace
            us_layer = Tn / sweep[str(Tn)] * 1e6 if str(Tn) in sweep else leg["us_per_layer"]
            gbps = leg["algorithmic_bytes_per_step"] / us_layer / 1e3
            leg["roofline"]["traffic"] = recorded_decode("decode_T%d_w13_traffic_bytes_per_launch" % Tn)
            roofline_by_T[str(Tn)] = {"roofline": leg["roofline"], "us_per_layer": us_layer,
                                      "us_per_layer_launched_from_python": leg["us_per_layer"],
                                      "layer_GBps": gbps, "layer_frac_of_hbm_peak": gbps / HBM_PEAK_GBS,
                                      "distinct_routed_experts_per_step": leg["distinct_routed_experts_per_step"],
                                      "algorithmic_bytes_per_step": leg["algorithmic_bytes_per_step"]}

    out = {"metric": "moe_layer_decode_tokens_per_s", "value": value, "unit": "tokens/s", "n_gpus": 1,
           "steps": a.steps, "warmup": a.warmup, "ms_per_step": dt / a.steps * 1e3, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "DeepSeek-MoE-16B-shaped MoE layer, int4-g128 experts, decode T=%d, "
                                  "steady-state hits (all routed experts resident), %d-layer stack" % (T, L_),
                      "hidden": H, "experts": E, "intermediate": I, "shared_intermediate": I_sh, "top_k": k,
                      "tokens_per_step": T, "layers": L_, "zipf": 1.2,
                      "weights": "random int4-g128 images (uniform nibbles and zero points, fp16 scales 0.005 to 0.009): "
                                 "the kernels' time does not depend on the values"},
           "timing": timing, "c2_as_configured_tokens_per_s": as_configured,
           "roofline": roofline, "roofline_by_T": roofline_by_T, "cpu_baseline": cpu, "cpu_baseline_more": cpu_more,
           "layer": layer, "tokens_per_s_by_T": sweep, "cache_run": cache_run, "prefill": prefill, "other_decode_configs": others}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
