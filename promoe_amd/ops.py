"""Thin torch-tensor wrappers over the kernel entry points of the C ABI.

torch is used for device memory and streams only; every op below runs a
hand-written HIP kernel from libmoe_engine.so on torch's current stream.
"""
from __future__ import annotations

import torch

from . import _lib as L
from ._lib import lib, ptr, cur_stream, check


def gemv_max_tokens(fmt: int) -> int:
    """Largest token group moe_forward sends to the GEMV kernels; larger ones (and every bf16 layer) take
    the matrix-core tile kernels."""
    return 0 if fmt == L.FMT_BF16 else 64


def _dev(t):
    assert t.is_cuda and t.is_contiguous(), "expected a contiguous device tensor"
    return t


def gate_logits(x: torch.Tensor, wg: torch.Tensor, bias: torch.Tensor | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor:
    """x [T,H] bf16, wg [E,H] bf16 -> logits [T,E] fp32 (fixed summation order)."""
    T, H = x.shape
    E = wg.shape[0]
    assert x.dtype == torch.bfloat16 and wg.dtype == torch.bfloat16 and wg.shape[1] == H
    if out is None:
        out = torch.empty(T, E, dtype=torch.float32, device=x.device)
    check(lib.moe_gate_logits(ptr(_dev(x)), ptr(_dev(wg)), ptr(bias), ptr(out), T, H, E,
                              out.stride(0), cur_stream()), "moe_gate_logits")
    return out


def gate_logits_pair(x: torch.Tensor, wg: torch.Tensor, bias, wg2: torch.Tensor, bias2):
    """Two matrices over the same activations in one launch (T <= 128): (logits [T,E], logits2 [T,E2])."""
    T, H = x.shape
    E, E2 = wg.shape[0], wg2.shape[0]
    out = torch.empty(T, E, dtype=torch.float32, device=x.device)
    out2 = torch.empty(T, E2, dtype=torch.float32, device=x.device)
    check(lib.moe_gate_logits_pair(ptr(_dev(x)), ptr(_dev(wg)), ptr(bias), ptr(out), T, H, E, E, ptr(_dev(wg2)),
                                   ptr(bias2), ptr(out2), E2, E2, cur_stream()), "moe_gate_logits_pair")
    return out, out2


def topk(logits: torch.Tensor, k: int, mode: int = L.ROUTE_SOFTMAX_TOPK, E: int | None = None):
    T = logits.shape[0]
    E = logits.shape[1] if E is None else E
    idx = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    check(lib.moe_topk(ptr(_dev(logits)), T, E, logits.stride(0), k, mode, ptr(idx), ptr(w),
                       cur_stream()), "moe_topk")
    return idx, w


class Dispatch:
    """Device buffers produced by moe_dispatch."""

    def __init__(self, T: int, k: int, E: int, max_units: int, device):
        P = T * k
        i32 = dict(dtype=torch.int32, device=device)
        self.T, self.k, self.E, self.max_units = T, k, E, max_units
        self.counts = torch.empty(E, **i32)
        self.offsets = torch.empty(E + 1, **i32)
        self.sorted_pair = torch.empty(max(P, 1), **i32)
        self.pos_of_pair = torch.empty(max(P, 1), **i32)
        self.sorted_tok = torch.empty(max(P, 1), **i32)
        self.units = torch.empty(max(max_units, 1), 4, **i32)
        self.n_active = torch.empty(1, **i32)
        self.active_ids = torch.empty(max(max_units, 1), dtype=torch.int64, device=device)
        self.err = torch.zeros(1, **i32)

    def check(self):
        """Raises if the multi-workgroup dispatch kernel reported a time-out (synchronises)."""
        if int(self.err.item()):
            raise L.MoeError("moe_dispatch_ws: a workgroup did not get the others' counts in time")


_dispatch_ws: dict = {}


def dispatch(idx: torch.Tensor, E: int, max_units: int | None = None, out: Dispatch | None = None,
             single_workgroup: bool = False) -> Dispatch:
    T, k = idx.shape
    if max_units is None:
        max_units = min(E, T * k)
    d = out if out is not None else Dispatch(T, k, E, max_units, idx.device)
    ws_bytes = 0 if single_workgroup else int(lib.moe_dispatch_workspace_bytes(T, k, E))
    if ws_bytes:
        # prefill batches: one workgroup per 1024 pairs.  One workspace per device, zeroed when it is made (the
        # kernel leaves its barrier words zero); calls on a device must not overlap.  d.err is raised by a
        # workgroup that did not get the others' counts within a second (Dispatch.check reads it).
        ws = _dispatch_ws.get(idx.device)
        if ws is None or ws.numel() * 4 < ws_bytes:
            ws = _dispatch_ws[idx.device] = torch.zeros(ws_bytes // 4 + 1, dtype=torch.int32, device=idx.device)
        check(lib.moe_dispatch_ws(ptr(_dev(idx)), T, k, E, ptr(d.counts), ptr(d.offsets), ptr(d.sorted_pair),
                                  ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units), ptr(d.n_active),
                                  ptr(d.active_ids), max_units, ptr(ws), ws_bytes, ptr(d.err), cur_stream()),
              "moe_dispatch_ws")
        return d
    check(lib.moe_dispatch(ptr(_dev(idx)), T, k, E, ptr(d.counts), ptr(d.offsets), ptr(d.sorted_pair),
                           ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units), ptr(d.n_active),
                           ptr(d.active_ids), max_units, cur_stream()), "moe_dispatch")
    return d


def topk_dispatch(logits: torch.Tensor, k: int, E: int, mode: int = L.ROUTE_SOFTMAX_TOPK):
    """Top-k and dispatch in one launch for T <= 64.  Returns (idx, w, Dispatch)."""
    T = logits.shape[0]
    idx = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    d = Dispatch(T, k, E, min(E, T * k), logits.device)
    check(lib.moe_topk_dispatch(ptr(_dev(logits)), T, E, logits.stride(0), k, mode, ptr(idx), ptr(w), ptr(d.counts),
                                ptr(d.offsets), ptr(d.sorted_pair), ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units),
                                ptr(d.n_active), ptr(d.active_ids), d.max_units, 0, 0, 0, 0, cur_stream()),
          "moe_topk_dispatch")
    return idx, w, d


def gate_topk_dispatch(x, wg, bias, E: int, k: int, mode: int, gws: "GateWorkspace", parts: int = 1):
    """Gate logits, top-k and dispatch in one launch for 2 <= T <= 32.  wg may carry one extra row (shared gate,
    no bias).  Returns (logits [T, rows], idx, w, Dispatch, err int32[1])."""
    T, H = x.shape
    rows = wg.shape[0]
    dev = x.device
    need = int(lib.moe_gate_route_ws_bytes(T, rows))
    if gws.buf.numel() < need:
        raise L.MoeError("gate workspace of %d bytes, %d needed" % (gws.buf.numel(), need))
    logits = torch.empty(T, rows, dtype=torch.float32, device=dev)
    idx = torch.empty(T, k, dtype=torch.int32, device=dev)
    w = torch.empty(T, k, dtype=torch.float32, device=dev)
    d = Dispatch(T, k, E, min(E, T * k), dev)
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    check(lib.moe_gate_topk_dispatch(ptr(_dev(x)), ptr(_dev(wg)), ptr(bias), E if bias is not None else 0, ptr(logits),
                                     T, H, E, rows, rows, k, mode, ptr(idx), ptr(w), ptr(d.counts), ptr(d.offsets),
                                     ptr(d.sorted_pair), ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units),
                                     ptr(d.n_active), ptr(d.active_ids), d.max_units, 0, 0, 0, 0, ptr(gws.buf),
                                     gws.next_seq(), parts, ptr(err), cur_stream()),
          "moe_gate_topk_dispatch")
    return logits, idx, w, d, err


_route_counter = {}


def route_decode(x, wg, bias, E: int, k: int, mode: int = L.ROUTE_SOFTMAX_TOPK):
    """Fused gate logits + top-k + dispatch for T <= 64.  wg may carry one extra row (shared gate)."""
    if x.device not in _route_counter:   # the launch counter of the fused kernel: zero between calls
        _route_counter[x.device] = torch.zeros(1, dtype=torch.int32, device=x.device)
    T, H = x.shape
    rows = wg.shape[0]
    logits = torch.empty(T, rows, dtype=torch.float32, device=x.device)
    idx = torch.empty(T, k, dtype=torch.int32, device=x.device)
    w = torch.empty(T, k, dtype=torch.float32, device=x.device)
    d = Dispatch(T, k, E, min(E, T * k), x.device)
    check(lib.moe_route_decode(ptr(_dev(x)), ptr(_dev(wg)), ptr(bias), ptr(logits), T, H, E, rows, rows, k, mode,
                               ptr(idx), ptr(w), ptr(d.counts), ptr(d.offsets), ptr(d.sorted_pair),
                               ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units), ptr(d.n_active),
                               ptr(d.active_ids), d.max_units, ptr(_route_counter[x.device]), cur_stream()),
          "moe_route_decode")
    return logits, idx, w, d


def experts_decode_int4(x, d: Dispatch, expert_ptr: torch.Tensor, shared: torch.Tensor | None,
                        H: int, I: int, I_sh: int, host_units: bool = False, phases: int = 3, ws=None):
    """Returns (part_r [P,H] fp32, part_s [T,H] fp32 or None, err int32[1])."""
    T, k = d.T, d.k
    P = T * k
    dev = x.device
    if ws is not None:          # caller-provided workspace (part_r, part_s, err, h_r, h_s)
        part_r, part_s, err, h_r, h_s = ws
    else:
        h_r = torch.empty(max(P, 1), max(I, 1), dtype=torch.bfloat16, device=dev)
        part_r = torch.empty(max(P, 1), H, dtype=torch.float32, device=dev)
        h_s = part_s = None
        if shared is not None:
            h_s = torch.empty(T, I_sh, dtype=torch.bfloat16, device=dev)
            part_s = torch.empty(T, H, dtype=torch.float32, device=dev)
        err = torch.zeros(1, dtype=torch.int32, device=dev)
    uh = th = None
    if host_units:   # unit list and slot table resolved on the host, sent in the kernel arguments
        uh = d.units.cpu().contiguous()
        th = expert_ptr.cpu().contiguous()
    check(lib.moe_experts_decode_int4(ptr(_dev(x)), T, H, I, I_sh if shared is not None else 0, k,
                                      ptr(d.units), d.max_units, ptr(d.sorted_tok), ptr(expert_ptr),
                                      ptr(shared), ptr(h_r), ptr(h_s), ptr(part_r), ptr(part_s),
                                      ptr(err), ptr(uh), ptr(th), phases, cur_stream()), "moe_experts_decode_int4")
    return part_r, part_s, err, h_r, h_s


class GateWorkspace:
    """Hand-over area of the launches that compute the gate logits themselves (moe_decode_token_int4_gate):
    zeroed once; every call takes the next sequence number."""

    def __init__(self, dev, T: int = 1, rows: int = 1):
        nbytes = max(int(lib.moe_gate_ws_bytes()), int(lib.moe_gate_route_ws_bytes(T, rows)))
        self.buf = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.seq = 0

    def next_seq(self) -> int:
        self.seq = self.seq + 1 if self.seq < 0x7fffffff else 1
        return self.seq


def decode_batch_int4_gate_fits(T: int, E: int, k: int, H: int, I: int, I_sh: int, rows: int) -> bool:
    return bool(lib.moe_decode_batch_int4_gate_fits(T, E, k, H, I, I_sh, rows))


def decode_batch_int4_gate(x, wg, bias, E: int, k: int, mode: int, expert_ptr, shared, H: int, I: int, I_sh: int,
                           gws: "GateWorkspace", phases: int = 3, ws=None, expert_ptr_host=None):
    """2 to 16 tokens: gate rows, routing and w13 in one launch (phase bit 0), w2 over the published unit list (bit 1).
    expert_ptr_host: a CPU int64 tensor holding the slot table (E <= 64): both launches take the table from their
    arguments instead of reading expert_ptr.
    wg may carry one extra row (shared gate, no bias); ws: the tuple an earlier call returned (nothing is allocated).
    Returns (logits [T, rows], idx, w, Dispatch, part_r, part_s, err, h_r, h_s)."""
    T = x.shape[0]
    rows = wg.shape[0]
    dev = x.device
    P = T * k
    if ws is not None:
        logits, idx, w, d, part_r, part_s, err, h_r, h_s = ws
    else:
        logits = torch.empty(T, rows, dtype=torch.float32, device=dev)
        idx = torch.empty(T, k, dtype=torch.int32, device=dev)
        w = torch.empty(T, k, dtype=torch.float32, device=dev)
        d = Dispatch(T, k, E, min(E, P), dev)
        h_r = torch.empty(P, I, dtype=torch.bfloat16, device=dev)
        part_r = torch.empty(P, H, dtype=torch.float32, device=dev)
        h_s = part_s = None
        if shared is not None:
            h_s = torch.empty(T, I_sh, dtype=torch.bfloat16, device=dev)
            part_s = torch.empty(T, H, dtype=torch.float32, device=dev)
        err = torch.zeros(1, dtype=torch.int32, device=dev)
    if gws.buf.numel() < int(lib.moe_gate_route_ws_bytes(T, rows)):
        raise L.MoeError("gate workspace too small")
    check(lib.moe_decode_batch_int4_gate(ptr(_dev(x)), T, ptr(_dev(wg)), ptr(bias), rows, ptr(gws.buf), gws.next_seq(),
                                         ptr(logits), rows, E, k, mode, H, I, I_sh if shared is not None else 0,
                                         ptr(expert_ptr), ptr(expert_ptr_host), ptr(shared), ptr(idx), ptr(w), ptr(d.counts),
                                         ptr(d.offsets), ptr(d.sorted_pair), ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units),
                                         ptr(d.n_active), ptr(d.active_ids), d.max_units, ptr(h_r), ptr(h_s),
                                         ptr(part_r), ptr(part_s), ptr(err), 0, 0, 0, 0, phases, cur_stream()),
          "moe_decode_batch_int4_gate")
    return logits, idx, w, d, part_r, part_s, err, h_r, h_s


def decode_token_int4(x, logits, E: int, k: int, mode: int, expert_ptr, shared, H: int, I: int, I_sh: int, ws=None,
                      phases: int = 3, unit_ws=None, sg_logit=None, y=None, gate=None, expert_ptr_host=None):
    """One token: routing inside the w13 kernel.  Returns (idx, w, Dispatch, part_r, part_s, err, h_r, h_s).
    expert_ptr_host: a CPU int64 tensor holding the slot table (E <= 64): the routing launch takes the table from its
    arguments instead of reading expert_ptr.
    gate = (gate_w [rows, H] bf16, bias [E] or None, GateWorkspace): the launch computes the gate logits too and
    `logits` (rows fp32) is an output."""
    dev = x.device
    if ws is None:
        idx = torch.empty(1, k, dtype=torch.int32, device=dev)
        w = torch.empty(1, k, dtype=torch.float32, device=dev)
        d = Dispatch(1, k, E, min(E, k), dev)
        h_r = torch.empty(k, I, dtype=torch.bfloat16, device=dev)
        part_r = torch.empty(k, H, dtype=torch.float32, device=dev)
        h_s = part_s = None
        if shared is not None:
            h_s = torch.empty(1, I_sh, dtype=torch.bfloat16, device=dev)
            part_s = torch.empty(1, H, dtype=torch.float32, device=dev)
        err = torch.zeros(1, dtype=torch.int32, device=dev)
    else:
        idx, w, d, part_r, part_s, err, h_r, h_s = ws
    if gate is not None:
        gw, gb, gws = gate
        check(lib.moe_decode_token_int4_gate(ptr(_dev(x)), ptr(gw), ptr(gb), gw.shape[0], ptr(gws.buf), gws.next_seq(),
                                             ptr(logits), E, k, mode, H, I, I_sh if shared is not None else 0,
                                             ptr(expert_ptr), ptr(expert_ptr_host), ptr(shared), ptr(idx), ptr(w), ptr(d.counts),
                                             ptr(d.offsets), ptr(d.sorted_pair), ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units),
                                             ptr(d.n_active), ptr(d.active_ids), ptr(h_r), ptr(h_s), ptr(part_r),
                                             ptr(part_s), ptr(err), ptr(unit_ws), 0, 0, 0, phases, ptr(sg_logit), ptr(y),
                                             cur_stream()),
              "moe_decode_token_int4_gate")
        return idx, w, d, part_r, part_s, err, h_r, h_s
    check(lib.moe_decode_token_int4(ptr(_dev(x)), ptr(logits), E, k, mode, H, I, I_sh if shared is not None else 0,
                                    ptr(expert_ptr), ptr(expert_ptr_host), ptr(shared), ptr(idx), ptr(w), ptr(d.counts),
                                    ptr(d.offsets), ptr(d.sorted_pair), ptr(d.pos_of_pair), ptr(d.sorted_tok), ptr(d.units),
                                    ptr(d.n_active), ptr(d.active_ids), ptr(h_r), ptr(h_s), ptr(part_r), ptr(part_s),
                                    ptr(err), ptr(unit_ws), 0, 0, 0, phases, ptr(sg_logit), ptr(y), cur_stream()),
          "moe_decode_token_int4")
    return idx, w, d, part_r, part_s, err, h_r, h_s


def decode_token_int4_noalloc(x, logits, E: int, k: int, mode: int, expert_ptr, shared, H: int, I: int, I_sh: int,
                              y, err, sg_logit=None):
    """One token, routing to y in two launches, with every workspace in the library's static device array:
    nothing is allocated here or in the library (x, logits, y and err are the caller's)."""
    check(lib.moe_decode_token_int4_noalloc(ptr(_dev(x)), ptr(logits), E, k, mode, H, I,
                                            I_sh if shared is not None else 0, ptr(expert_ptr), ptr(shared),
                                            ptr(sg_logit), ptr(y), ptr(err), cur_stream()),
          "moe_decode_token_int4_noalloc")
    return y


def experts_decode_q4k(x, d: Dispatch, expert_ptr: torch.Tensor, shared: torch.Tensor | None,
                       H: int, I: int, I_sh: int, phases: int = 3, ws=None):
    """q4_K flavour of experts_decode_int4 (device-side unit list)."""
    T, k = d.T, d.k
    P = T * k
    dev = x.device
    if ws is not None:
        part_r, part_s, err, h_r, h_s = ws
    else:
        h_r = torch.empty(max(P, 1), max(I, 1), dtype=torch.bfloat16, device=dev)
        part_r = torch.empty(max(P, 1), H, dtype=torch.float32, device=dev)
        h_s = part_s = None
        if shared is not None:
            h_s = torch.empty(T, I_sh, dtype=torch.bfloat16, device=dev)
            # the w2 pass may split the shared expert's reduction: one set of partial rows per split
            part_s = torch.empty(shared_splits(L.FMT_Q4K, T, H, I_sh) * T, H, dtype=torch.float32, device=dev)
        err = torch.zeros(1, dtype=torch.int32, device=dev)
    if part_s is not None:
        pieces = shared_splits(L.FMT_Q4K, T, H, I_sh)
        if part_s.shape[0] != pieces * T:   # a workspace made for another batch size
            part_s = torch.empty(pieces * T, H, dtype=torch.float32, device=dev)
    check(lib.moe_experts_decode_q4k(ptr(_dev(x)), T, H, I, I_sh if shared is not None else 0, k,
                                     ptr(d.units), d.max_units, ptr(d.sorted_tok), ptr(expert_ptr),
                                     ptr(shared), ptr(h_r), ptr(h_s), ptr(part_r), ptr(part_s),
                                     ptr(err), phases, cur_stream()), "moe_experts_decode_q4k")
    return part_r, part_s, err, h_r, h_s


def experts_prefill(x, d: Dispatch, expert_ptr: torch.Tensor, shared: torch.Tensor | None,
                    H: int, I: int, I_sh: int, fmt: int = L.FMT_BF16, phases: int = 3, ws=None):
    """MFMA grouped expert product.  Returns (part_r, part_s, err, h_r, h_s, tiles).  part_s has S*T rows, S =
    moe_prefill_shared_splits pieces of the shared expert's w2 product (combine adds them; S = 1 mostly)."""
    T, k = d.T, d.k
    P = T * k
    dev = x.device
    if ws is not None:
        part_r, part_s, err, h_r, h_s, tiles = ws
    else:
        h_r = torch.empty(max(P, 1), max(I, 1), dtype=torch.bfloat16, device=dev)
        part_r = torch.empty(max(P, 1), H, dtype=torch.float32, device=dev)
        h_s = part_s = None
        if shared is not None:
            h_s = torch.empty(T, I_sh, dtype=torch.bfloat16, device=dev)
            part_s = torch.empty(int(lib.moe_prefill_shared_splits(fmt, T, H, I_sh)) * T, H, dtype=torch.float32, device=dev)
        err = torch.zeros(1, dtype=torch.int32, device=dev)
        tiles = torch.empty(max(int(lib.moe_prefill_workspace_bytes(T, k, d.max_units)), 16), dtype=torch.uint8, device=dev)
    pieces = 1
    if part_s is not None:
        pieces = int(lib.moe_prefill_shared_splits(fmt, T, H, I_sh))
        if part_s.shape[0] != pieces * T:   # a workspace made for another batch size or format
            part_s = torch.empty(pieces * T, H, dtype=torch.float32, device=dev)
    check(lib.moe_experts_prefill_pieces(ptr(_dev(x)), T, H, I, I_sh if shared is not None else 0, k, fmt,
                                         ptr(d.units), d.max_units, ptr(d.sorted_tok), ptr(expert_ptr),
                                         ptr(shared), ptr(h_r), ptr(h_s), ptr(part_r), ptr(part_s), pieces, ptr(tiles),
                                         ptr(err), phases, cur_stream()), "moe_experts_prefill")
    return part_r, part_s, err, h_r, h_s, tiles


def shared_splits(fmt: int, T: int, H: int, I_sh: int) -> int:
    """Pieces the decode w2 pass leaves the shared expert's partial rows in (1 unless q4_K with a long reduction)."""
    return int(lib.moe_decode_shared_splits(fmt, T, H, I_sh)) if I_sh else 1


def combine(part_r, part_s, topk_w, pos_of_pair, shared_gate_logit, T: int, H: int, k: int,
            out: torch.Tensor | None = None, pieces: int | None = None):
    """part_s [S*T, H]: S > 1 when the shared expert's reduction was split (piece s = rows s*T .. s*T+T-1).
    pieces: S as the expert launch left it (shared_splits / moe_prefill_shared_splits); inferred from the rows of
    part_s when not given, which is only right for a part_s made for exactly this T."""
    dev = (part_r if part_r is not None else part_s).device
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    sg_stride = shared_gate_logit.stride(0) if shared_gate_logit is not None else 0
    if part_s is None:
        n_splits = 1
    elif pieces is not None:
        n_splits = int(pieces)
        assert part_s.shape[0] >= n_splits * T, "part_s holds fewer rows than pieces x tokens"
    else:
        assert part_s.shape[0] % max(T, 1) == 0, "part_s was made for another batch size: pass pieces"
        n_splits = max(1, part_s.shape[0] // max(T, 1))
    check(lib.moe_combine_splits(ptr(part_r), ptr(part_s), ptr(topk_w), ptr(pos_of_pair),
                                 ptr(shared_gate_logit), sg_stride, ptr(out), T, H, k, n_splits, cur_stream()),
          "moe_combine")
    return out
