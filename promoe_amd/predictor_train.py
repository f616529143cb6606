"""Training and storage of the built-in predictor's models.

The reference's `SepPredictor` keeps one model per (source layer -> destination layer) pair and loads them from a
directory of files named "{src}-{dst}.pt" (src/cpp_worker/predictor.cpp:610-636: TorchScript modules that map the
hidden state seen at `src` to scores over the experts of `dst`; the pairs are those of
`build_predict_layer_mapping`, predictor.cpp:8-46).  The models themselves and the script that trained them are
not part of the reference tree.

Here a pair's model is linear, `scores = W x + b` with W [E, H] (what the engine's predictor evaluates on the GPU),
and this module

* records a trace of decode steps: the hidden state at the input of every MoE layer (and behind the last one)
  and the gate logits of every layer (`Trace`);
* fits each pair by ridge regression of the destination layer's gate logits on the source layer's hidden state
  (`fit_pair`, `fit_all`): the closed form (X^T X + lambda I)^-1 X^T Y in float64;
* writes / reads a model directory in the reference's naming with weights-only files, "{src}-{dst}.safetensors"
  holding `weight` [E, H] bf16 and `bias` [E] fp32 (`save_dir`, `load_dir`); nothing executable is stored or
  loaded (no TorchScript, no pickle);
* hands a directory to an engine (`attach`): every pair of `PrefetchMngr.predictor_windows()` must be present,
  as in the reference, where a missing file is a failed check.

Command line: python -m promoe_amd.predictor_train --trace trace.npz --out models/ [--ridge 1e-2]
(trace.npz: `hidden` [N, L + 1, H] float32, `logits` [N, L, E] float32, as `Trace.save` writes it).
"""
from __future__ import annotations

import argparse
import os

import numpy as np
import torch


class Trace:
    """Decode steps of one model: hidden[n, l] = input of MoE layer l (l = L: the output of the last layer),
    logits[n, l] = gate logits of layer l at that step."""

    def __init__(self, num_layer: int, hidden_size: int, num_expert: int):
        self.L, self.H, self.E = num_layer, hidden_size, num_expert
        self._hidden, self._logits = [], []
        self._cur_h = self._cur_l = None

    def begin_token(self):
        self._cur_h = np.zeros((self.L + 1, self.H), np.float32)
        self._cur_l = np.zeros((self.L, self.E), np.float32)

    def add_layer(self, layer: int, hidden, logits=None):
        """hidden [H] (or [1, H]) at the input of `layer` (layer = L: behind the last layer); logits [E] of `layer`."""
        self._cur_h[layer] = np.asarray(hidden, np.float32).reshape(-1)
        if logits is not None:
            self._cur_l[layer] = np.asarray(logits, np.float32).reshape(-1)[: self.E]

    def end_token(self):
        self._hidden.append(self._cur_h)
        self._logits.append(self._cur_l)
        self._cur_h = self._cur_l = None

    @property
    def hidden(self) -> np.ndarray:
        return np.stack(self._hidden) if self._hidden else np.zeros((0, self.L + 1, self.H), np.float32)

    @property
    def logits(self) -> np.ndarray:
        return np.stack(self._logits) if self._logits else np.zeros((0, self.L, self.E), np.float32)

    def save(self, path: str):
        np.savez(path, hidden=self.hidden, logits=self.logits)

    @staticmethod
    def load(path: str) -> "Trace":
        z = np.load(path, allow_pickle=False)
        h, lg = z["hidden"], z["logits"]
        t = Trace(lg.shape[1], h.shape[2], lg.shape[2])
        t._hidden, t._logits = list(h), list(lg)
        return t


def fit_pair(x_src: np.ndarray, logits_dst: np.ndarray, ridge: float = 1e-2):
    """Ridge regression of logits_dst [N, E] on x_src [N, H] with an intercept: returns (W [E, H], b [E]) float32
    minimising |X W^T + b - Y|^2 + ridge * N * |W|^2 (the intercept is not penalised)."""
    X = torch.from_numpy(np.asarray(x_src, np.float64))
    Y = torch.from_numpy(np.asarray(logits_dst, np.float64))
    n = X.shape[0]
    if n == 0:
        raise ValueError("fit_pair: empty trace")
    mx, my = X.mean(0, keepdim=True), Y.mean(0, keepdim=True)
    Xc, Yc = X - mx, Y - my
    A = Xc.T @ Xc + ridge * n * torch.eye(X.shape[1], dtype=torch.float64)
    W = torch.linalg.solve(A, Xc.T @ Yc).T          # [E, H]
    b = (my - mx @ W.T).reshape(-1)
    return W.float().numpy(), b.float().numpy()


def fit_all(trace: Trace, windows, ridge: float = 1e-2) -> dict:
    """windows[src] = (first, last): the destination layers source layer `src` predicts (`predictor_windows()`).
    Returns {(src, dst): (W, b)}."""
    H_, L_ = trace.hidden, trace.logits
    models = {}
    for src, (a, b) in enumerate(windows):
        for dst in range(a, b):
            models[(src, dst)] = fit_pair(H_[:, src], L_[:, dst], ridge)
    return models


def _bf16_bits(w: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(w, np.float32)).to(torch.bfloat16)


def save_dir(path: str, models: dict):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    for (src, dst), (W, b) in models.items():
        save_file({"weight": _bf16_bits(W).contiguous(), "bias": torch.from_numpy(np.ascontiguousarray(b, np.float32))},
                  os.path.join(path, "%d-%d.safetensors" % (src, dst)))


def load_dir(path: str, windows) -> dict:
    """{(src, dst): (weight bf16 [E, H], bias fp32 [E])} for every pair of `windows`; a missing pair is an error
    (predictor.cpp:624 loads every pair of the mapping)."""
    from safetensors.torch import load_file
    if not os.path.isdir(path):
        raise FileNotFoundError("predictor model path is not a directory: %s" % path)
    out = {}
    for src, (a, b) in enumerate(windows):
        for dst in range(a, b):
            f = os.path.join(path, "%d-%d.safetensors" % (src, dst))
            if not os.path.exists(f):
                raise FileNotFoundError("predictor model of the pair %d -> %d is missing: %s" % (src, dst, f))
            t = load_file(f)
            w, bias = t["weight"], t.get("bias")
            if w.dtype != torch.bfloat16 or w.dim() != 2:
                raise ValueError("%s: weight must be bf16 [E, H]" % f)
            out[(src, dst)] = (w, None if bias is None else bias.float())
    return out


def attach(pm, path: str, device=None):
    """Load the directory into the engine's predictor (the models of all its pairs) and start it."""
    models = load_dir(path, pm.predictor_windows())
    for (src, dst), (w, bias) in models.items():
        if device is not None:
            w = w.to(device)
            bias = None if bias is None else bias.to(device)
            pm.set_predictor_model(src, dst, w, bias)
        else:   # host backend: bit patterns in numpy
            pm.set_predictor_model(src, dst, w.view(torch.int16).numpy().view(np.uint16),
                                   None if bias is None else bias.numpy())
    pm.start_predictor()
    return len(models)


def main():
    ap = argparse.ArgumentParser(description="Fit the (src -> dst) expert predictors from a recorded trace")
    ap.add_argument("--trace", required=True, help="npz written by Trace.save")
    ap.add_argument("--out", required=True, help="model directory to write ({src}-{dst}.safetensors)")
    ap.add_argument("--ridge", type=float, default=1e-2)
    ap.add_argument("--windows", required=True,
                    help="pairs as 'first:last' per source layer 0..L, comma separated (PrefetchMngr.predictor_windows())")
    a = ap.parse_args()
    tr = Trace.load(a.trace)
    windows = [tuple(int(v) for v in w.split(":")) for w in a.windows.split(",")]
    if len(windows) != tr.L + 1:
        raise SystemExit("need %d windows (source layers 0..L), got %d" % (tr.L + 1, len(windows)))
    models = fit_all(tr, windows, a.ridge)
    save_dir(a.out, models)
    print("wrote %d models to %s" % (len(models), a.out))


if __name__ == "__main__":
    main()
