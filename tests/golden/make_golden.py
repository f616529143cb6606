"""Writes the golden vectors of tests/golden/ from the CPU oracle (seeded, small).

The reference holds no fixtures for this path (its MoE arithmetic is external), so these
vectors pin the ORACLE: tests/test_golden.py checks that the oracle still reproduces them
and the GPU tests compare the HIP path against the same files.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import moe_oracle as O  # noqa: E402
from tests.synth import Int4Layer, Q4KLayer, Bf16Layer  # noqa: E402


def routing_case():
    T, H, E, k = 5, 256, 60, 4
    x = O.synth_acts(T, H, seed=7)
    wg = O.round_bf16(O.synth_weights((E, H), seed=8))
    wg[3] = wg[1]                      # a tie between experts 1 and 3 in every row
    logits = O.gate_logits_ordered(x, wg)
    out = dict(x=x, wg=wg, logits=logits)
    for mode in (0, 1, 2):
        idx, w = O.topk_route(logits, k, mode)
        out["idx_m%d" % mode] = idx
        out["w_m%d" % mode] = w
    counts, offsets, sp, pp = O.dispatch(out["idx_m0"], E)
    out.update(counts=counts, offsets=offsets, sorted_pair=sp, pos_of_pair=pp)
    np.savez_compressed(os.path.join(HERE, "routing_T5_H256_E60_k4.npz"), **out)


def layer_case(kind):
    mk = {"int4": Int4Layer, "q4k": Q4KLayer, "bf16": Bf16Layer}[kind]
    H, E, k = 256, 4, 2
    I = I_sh = 256 if kind == "q4k" else 128
    layer = mk(H=H, I=I, E=E, I_sh=I_sh, seed=21, shared_gate=True, zipf=1.2)
    out = dict(wg=layer.wg, bias=layer.bias, shared_gate=layer.shared_gate,
               slots=np.stack(layer.slots), shared_img=layer.shared_img)
    for T in (1, 3, 40):
        x = O.synth_acts(T, H, seed=30 + T)
        lg = (O.gate_logits_ordered(x, layer.wg) + layer.bias[None, :]).astype(np.float32)
        ref = O.moe_forward(x, layer.wg, layer.experts_fp32, k, 0, shared=layer.shared_fp32,
                            shared_gate=layer.shared_gate, logits=lg)
        out["x_T%d" % T] = x
        out["y_T%d" % T] = ref["out"]
        out["idx_T%d" % T] = ref["idx"]
    np.savez_compressed(os.path.join(HERE, "layer_%s_H256_E4_k2.npz" % kind), **out)


if __name__ == "__main__":
    routing_case()
    for kind in ("int4", "q4k", "bf16"):
        layer_case(kind)
    print("written:", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
