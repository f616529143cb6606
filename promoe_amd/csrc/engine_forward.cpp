// Fused MoE-layer forward on top of the cache engine: the patched MoE module's
// forward (contract: eval/demo-simulate/transformers-deepseek-moe.py:36-49 of the
// reference) as one call.  gate -> top-k -> dispatch run on the device; the active
// expert list comes back to the host once (the reference's `unique().cpu()` sync
// point), the cache hooks run in the reference's order, experts that are already
// resident go out as ONE grouped launch, missed experts follow one by one as their
// copies land (the returned order of report_one_layer), then combine.
#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>

#include "engine_internal.h"

struct LayerState {
  int max_tokens = 0, max_k = 0, max_units = 0;
  int E = 0, H = 0, I = 0, I_sh = 0;
  float *logits = nullptr, *topk_w = nullptr, *part_r = nullptr, *part_s = nullptr;
  size_t part_s_elems = 0;  // floats behind part_s
  int *idx = nullptr, *counts = nullptr, *offsets = nullptr, *sorted_pair = nullptr, *pos_of_pair = nullptr,
      *sorted_tok = nullptr, *n_active = nullptr;
  unsigned char *unit_ws = nullptr;  // resolved units of the one-token path (16 bytes each)
  // one-token launches that compute their gate logits themselves: hand-over words (zeroed once) and the number
  // of the last such launch (every launch takes the next one, so no word of an earlier launch passes for a new one)
  unsigned char *gate_ws = nullptr;
  size_t gate_ws_bytes = 0;
  int gate_seq = 0;
  moe_unit *units = nullptr, *units_sub = nullptr;
  int64_t *active_ids = nullptr;
  void *h_r = nullptr, *h_s = nullptr, *tiles_ws = nullptr;
  unsigned char *disp_ws = nullptr;  // workspace of the prefill batches' dispatch (starts with its zeroed barrier words)
  int64_t disp_ws_bytes = 0;
  // pinned host mirrors
  moe_unit *units_host = nullptr, *units_sub_host = nullptr;
  int *n_active_host = nullptr, *opt_seq = nullptr;
  // error words the kernels raise when a selected expert has no slot, in pinned host memory so that the host
  // sees them without a copy: one per layer for launches in which that must not happen (checked at the next
  // call and when the engine drains), one for launches that are allowed to meet non-resident experts
  int *err_host = nullptr, *err_loose = nullptr;
  int *err_loose_dev = nullptr;  // device word for launches whose every workgroup of a skipped unit raises it
  // error words of the w2 + combine launches that go out before the host knows the routing, and what the host
  // expects of each once it does: 1 = must stay zero (every selected expert was resident at launch), 2 = may be
  // set (an expert was missing; that launch's output is recomputed), 0 = none outstanding.  Two words per layer,
  // used in turn: the word a turn re-arms was last written by the launch of two turns ago, and between that
  // launch and now the host has seen the sequence word of a LATER w13 kernel of the same stream (the one of the
  // turn in between), so that launch is over and its word final.  With one word per layer and a single layer, the
  // host could re-arm the word before the previous turn's launch had raised it.
  int *err_spec = nullptr;
  std::vector<char> spec_state;
  std::vector<unsigned> spec_turn;
  std::vector<unsigned char> late_last;   // per layer: experts the last turn had to wait for
  int num_layer = 0;
  std::vector<void *> dev_allocs, host_allocs;
  hipEvent_t ev = nullptr;
  int sub_cursor = 0;
  // routing results of calls that ran without a host round trip, accounted later
  struct Pending {
    int layer = -1, max_units = 0;
    hipEvent_t ev = nullptr;
    moe_unit *units = nullptr;
    int *n_active = nullptr;
    bool busy = false;
    // routing stored by the kernel itself into `units`: ready when *seq == seq_expected (no event)
    int *seq = nullptr;
    int seq_expected = 0;
    bool by_seq = false;
  };
  int seq_counter = 0;
  static const int kPending = 8;
  Pending pend[kPending];
  int pend_head = 0;
};

void moe_forward_free(LayerState *s) {
  if (!s) return;
  for (auto p : s->dev_allocs) (void)hipFree(p);
  for (auto p : s->host_allocs) (void)hipHostFree(p);
  if (s->ev) (void)hipEventDestroy(s->ev);
  for (auto &p : s->pend) if (p.ev) (void)hipEventDestroy(p.ev);
  delete s;
}

#define HIPC(call)                                          \
  do {                                                      \
    if (int rc_ = moe_check_hip((call), #call)) return rc_; \
  } while (0)

extern "C" int moe_set_layer(moe_engine *eng, int layer, const moe_layer_desc *d) {
  if (!eng || !d) { moe_set_error("moe_set_layer: null"); return MOE_EINVAL; }
  if (layer < 0 || layer >= eng->cfg.num_layer) { moe_set_error("moe_set_layer: bad layer %d", layer); return MOE_EINVAL; }
  if (d->H <= 0 || d->H % 128 || d->I <= 0 || d->I % 128 || d->I_sh < 0 || d->I_sh % 128 || d->top_k <= 0 ||
      d->top_k > eng->cfg.num_expert || d->route_mode < 0 || d->route_mode > 2 || !d->gate_w ||
      (d->I_sh > 0 && !d->shared) || (d->shared_gated && d->I_sh == 0)) {
    moe_set_error("moe_set_layer: bad descriptor (H=%d I=%d I_sh=%d k=%d)", d->H, d->I, d->I_sh, d->top_k);
    return MOE_EINVAL;
  }
  if (d->fmt != MOE_FMT_INT4_G128 && d->fmt != MOE_FMT_BF16 && d->fmt != MOE_FMT_Q4K) { moe_set_error("moe_set_layer: weight format %d not supported by this entry point", d->fmt); return MOE_EINVAL; }
  if (d->fmt == MOE_FMT_BF16 && (d->H % 256 || d->I % 128 || d->I_sh % 128)) {
    moe_set_error("moe_set_layer: bf16 experts need H %% 256 == 0 and I %% 128 == 0 (H=%d I=%d I_sh=%d)", d->H, d->I, d->I_sh);
    return MOE_EINVAL;
  }
  if (d->fmt == MOE_FMT_Q4K && (d->H % 256 || d->I % 256 || d->I_sh % 256)) {
    moe_set_error("moe_set_layer: q4_K experts need H and I multiples of 256 (H=%d I=%d I_sh=%d)", d->H, d->I, d->I_sh);
    return MOE_EINVAL;
  }
  eng->layer_desc[layer] = *d;
  return MOE_OK;
}

template <typename T>
static int dalloc(LayerState *s, T **p, size_t n) {
  void *q = nullptr;
  HIPC(hipMalloc(&q, (n ? n : 1) * sizeof(T)));
  s->dev_allocs.push_back(q);
  *p = (T *)q;
  return MOE_OK;
}
template <typename T>
static int halloc(LayerState *s, T **p, size_t n) {
  void *q = nullptr;
  HIPC(hipHostMalloc(&q, (n ? n : 1) * sizeof(T), hipHostMallocDefault));
  s->host_allocs.push_back(q);
  *p = (T *)q;
  return MOE_OK;
}

extern "C" int moe_forward_prepare(moe_engine *eng, int max_tokens) {
  if (!eng || max_tokens <= 0) { moe_set_error("moe_forward_prepare: bad argument"); return MOE_EINVAL; }
  if (eng->be->compute_stream() == nullptr && eng->be->copy_stream() == nullptr) {
    moe_set_error("moe_forward_prepare: the host backend has no compute path");
    return MOE_ESTATE;
  }
  int H = 0, I = 0, I_sh = 0, k = 0;
  for (auto &d : eng->layer_desc) {
    if (!d.gate_w) continue;
    H = std::max(H, d.H); I = std::max(I, d.I); I_sh = std::max(I_sh, d.I_sh); k = std::max(k, d.top_k);
  }
  if (H == 0) { moe_set_error("moe_forward_prepare: no layer described (moe_set_layer)"); return MOE_ESTATE; }
  if (eng->fw) {
    // a second prepare: account the routings still pending, let the stream drain, and take every expert off
    // the sequence words of the old workspace (their launches are over) before that memory goes away
    if (int rc = moe_forward_harvest(eng, true)) return rc;
    HIPC(hipStreamSynchronize((hipStream_t)eng->be->compute_stream()));
    if (int rc = moe_forward_check_kernels(eng)) return rc;
    engine_drop_seq_releases(eng);
    // the fetch thread polls a sequence word without the lock.  No expert points at the old words any more (taken
    // off under the lock just now, and a poll takes its pointer under the lock), so once the poll that may be in
    // flight is over (it is bounded: 100 us, then an event of the drained stream) nothing reads the old workspace
    while (eng->seq_pollers.load(std::memory_order_acquire) != 0) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
    }
    moe_forward_free(eng->fw);
    eng->fw = nullptr;
  }
  LayerState *s = new LayerState();
  eng->fw = s;
  const int E = eng->cfg.num_expert, T = max_tokens;
  const size_t P = (size_t)T * k;
  s->max_tokens = T; s->max_k = k; s->E = E; s->H = H; s->I = I; s->I_sh = I_sh;
  s->max_units = (int)std::min<size_t>(E, P);
  int rc = 0;
  rc |= dalloc(s, &s->logits, (size_t)T * (E + 1));
  rc |= dalloc(s, &s->topk_w, P);
  rc |= dalloc(s, &s->idx, P);
  rc |= dalloc(s, &s->counts, E);
  rc |= dalloc(s, &s->offsets, E + 1);
  rc |= dalloc(s, &s->sorted_pair, P);
  rc |= dalloc(s, &s->pos_of_pair, P);
  rc |= dalloc(s, &s->sorted_tok, P);
  rc |= dalloc(s, &s->n_active, 1);
  rc |= dalloc(s, &s->err_loose_dev, 1);
  rc |= dalloc(s, &s->unit_ws, (size_t)32 * std::max(k, 1));
  s->gate_ws_bytes = (size_t)std::max<int64_t>(moe_gate_ws_bytes(), moe_gate_route_ws_bytes(std::min(T, 32), E + 1));
  rc |= dalloc(s, &s->gate_ws, s->gate_ws_bytes);
  rc |= dalloc(s, &s->units, s->max_units);
  rc |= dalloc(s, &s->units_sub, (size_t)s->max_units * 2);
  rc |= dalloc(s, &s->active_ids, s->max_units);
  rc |= dalloc(s, (uint16_t **)&s->h_r, P * I);
  rc |= dalloc(s, (uint16_t **)&s->h_s, (size_t)T * I_sh);
  rc |= dalloc(s, &s->part_r, P * H);
  // q4_K decode batches (at most 64 tokens) may leave the shared expert's partial rows in up to 8 pieces, and so
  // may a prefill batch of a nibble format whose shared expert is wide (pieces x tokens rows, largest over the
  // batch sizes the workspace admits)
  size_t rows_s = T > 128 ? T : 128;
  for (int t = 1; t <= T; ++t) {
    rows_s = std::max(rows_s, (size_t)t * (size_t)moe_prefill_shared_splits(MOE_FMT_Q4K, t, H, I_sh));
    if (t <= 64) rows_s = std::max(rows_s, (size_t)t * (size_t)moe_decode_shared_splits(MOE_FMT_Q4K, t, H, I_sh));
  }
  rc |= dalloc(s, &s->part_s, rows_s * H);
  s->part_s_elems = rows_s * H;
  rc |= dalloc(s, (unsigned char **)&s->tiles_ws, (size_t)moe_prefill_workspace_bytes(T, k, s->max_units));
  s->disp_ws_bytes = moe_dispatch_workspace_bytes(T, k, E);
  if (s->disp_ws_bytes) rc |= dalloc(s, &s->disp_ws, (size_t)s->disp_ws_bytes);
  rc |= halloc(s, &s->units_host, s->max_units);
  rc |= halloc(s, &s->units_sub_host, (size_t)s->max_units * 2);
  rc |= halloc(s, &s->n_active_host, 1);
  s->num_layer = eng->cfg.num_layer;
  rc |= halloc(s, &s->err_host, eng->cfg.num_layer);
  rc |= halloc(s, &s->err_loose, 1);
  rc |= halloc(s, &s->err_spec, (size_t)2 * eng->cfg.num_layer);
  rc |= halloc(s, &s->opt_seq, 1);
  for (auto &p : s->pend) {
    rc |= halloc(s, &p.units, s->max_units);
    rc |= halloc(s, &p.n_active, 1);
    rc |= halloc(s, &p.seq, 1);
    if (p.seq) *p.seq = 0;
    if (hipEventCreateWithFlags(&p.ev, hipEventDisableTiming) != hipSuccess) rc = 1;
  }
  if (rc) return MOE_EHIP;
  memset(s->err_host, 0, sizeof(int) * eng->cfg.num_layer);
  *s->err_loose = 0;
  memset(s->err_spec, 0, sizeof(int) * 2 * eng->cfg.num_layer);
  s->spec_state.assign((size_t)2 * eng->cfg.num_layer, 0);
  s->spec_turn.assign(eng->cfg.num_layer, 0);
  s->late_last.assign(eng->cfg.num_layer, 0);
  HIPC(hipMemset(s->gate_ws, 0, s->gate_ws_bytes));
  if (s->disp_ws) HIPC(hipMemset(s->disp_ws, 0, 64));
  *s->opt_seq = 0;
  HIPC(hipEventCreateWithFlags(&s->ev, hipEventDisableTiming));
  return MOE_OK;
}

// A strict error word is up: some launch of that layer skipped a selected expert, so what it combined is
// wrong.  The engine fails (every later call reports it), as the reference would abort on a broken invariant.
int moe_forward_check_kernels(moe_engine *eng) {
  LayerState *s = eng->fw;
  if (!s) return MOE_OK;
  for (int l = 0; l < s->num_layer; ++l)
    if (((volatile int *)s->err_host)[l] || (s->spec_state[2 * l] == 1 && ((volatile int *)s->err_spec)[2 * l]) ||
        (s->spec_state[2 * l + 1] == 1 && ((volatile int *)s->err_spec)[2 * l + 1]))
      return engine_fail(eng, "a kernel of layer %d met a selected expert without a slot: its output is wrong", l);
  return MOE_OK;
}

int moe_forward_harvest(moe_engine *eng, bool wait) {
  LayerState *s = eng->fw;
  if (!s) return MOE_OK;
  for (int i = 0; i < LayerState::kPending; ++i) {
    LayerState::Pending &p = s->pend[(s->pend_head + i) % LayerState::kPending];  // oldest first
    if (!p.busy) continue;
    if (p.by_seq) {
      volatile int *sq = p.seq;
      if (*sq != p.seq_expected) {
        if (!wait) break;
        // the launch that writes it is already in the compute stream
        if (hipStreamSynchronize((hipStream_t)eng->be->compute_stream()) != hipSuccess) return MOE_EHIP;
        if (*sq != p.seq_expected) { moe_set_error("routing of layer %d never reached the host", p.layer); return MOE_EHIP; }
      }
      __atomic_thread_fence(__ATOMIC_ACQUIRE);
    } else if (wait) { if (hipEventSynchronize(p.ev) != hipSuccess) return MOE_EHIP; }
    else if (hipEventQuery(p.ev) != hipSuccess) { (void)hipGetLastError(); break; }
    const int n = std::min(*p.n_active, p.max_units);
    if (int rc = engine_account_hits(eng, p.layer, p.units, n)) return rc;
    p.busy = false;
  }
  return MOE_OK;
}

// Expert product of one launch group.  Token groups of prefill size (and every bf16 layer)
// go to the matrix-core tile kernels, decode batches to the bandwidth-bound GEMV kernels.
static bool use_prefill(const moe_layer_desc &d, int T) {
  if (d.fmt == MOE_FMT_BF16) return true;
  // nibble formats: up to 64 tokens the grouped launch is bound by the weight stream, and the decode kernels
  // (a workgroup streams four block pairs of a unit over the whole reduction, 16 to 64 token rows per pass)
  // stream it faster than the tile kernels, whose tiles are short at these batch sizes (measured on the
  // 2048 x 1408 and 4096 x 14336 int4 shapes and the 3584 x 2560 q4_K shape)
  return T > 64 && d.H % 256 == 0 && d.I % 128 == 0 && d.I_sh % 128 == 0;
}

static int shared_pieces(const moe_layer_desc &d, int T, const LayerState *s);
// pub / pub_seq: the pending slot whose pinned unit list the w13 launch fills (decode_publishes), or null
static int run_units(moe_engine *eng, const moe_layer_desc &d, LayerState *s, const void *x, int T,
                     const moe_unit *units_dev, const moe_unit *units_host, int n_units, bool with_shared,
                     int layer, const uint64_t *table, hipStream_t st, LayerState::Pending *pub = nullptr,
                     int pub_seq = 0) {
  if (use_prefill(d, T))
    return moe_experts_prefill_pieces(x, T, d.H, d.I, with_shared ? d.I_sh : 0, d.top_k, d.fmt, units_dev, n_units,
                                      s->sorted_tok, table, with_shared ? d.shared : nullptr, s->h_r, s->h_s, s->part_r,
                                      s->part_s, with_shared ? shared_pieces(d, T, s) : 1, s->tiles_ws,
                                      s->err_host + layer, 3, st);
  if (d.fmt == MOE_FMT_Q4K)
    return moe_experts_decode_q4k(x, T, d.H, d.I, with_shared ? d.I_sh : 0, d.top_k, units_dev, n_units,
                                  s->sorted_tok, table, with_shared ? d.shared : nullptr, s->h_r, s->h_s,
                                  s->part_r, s->part_s, s->err_host + layer, 3, st);
  // the host knows the units and the slot addresses: they travel in the kernel arguments
  const uint64_t *table_host = units_host ? eng->h_table + (size_t)layer * eng->cfg.num_expert : nullptr;
  return moe_experts_decode_int4_publish(x, T, d.H, d.I, with_shared ? d.I_sh : 0, d.top_k, units_dev, n_units,
                                         s->sorted_tok, table, with_shared ? d.shared : nullptr, s->h_r, s->h_s,
                                         s->part_r, s->part_s, s->err_host + layer, units_host, table_host, 3,
                                         s->n_active, pub ? pub->units : nullptr, pub ? pub->n_active : nullptr,
                                         pub ? pub->seq : nullptr, pub_seq, st);
}

// a decode batch whose w13 launch can send the unit list to the host itself (int4 GEMV kernels, 2 tokens and more)
static bool decode_publishes(const moe_layer_desc &d, int T, int max_units) {
  return d.fmt == MOE_FMT_INT4_G128 && T >= 2 && !use_prefill(d, T) && max_units > 0 && d.I > 0;
}

// pieces the expert launch of run_units leaves the shared expert's partial rows in
static int shared_pieces(const moe_layer_desc &d, int T, const LayerState *s) {
  if (d.I_sh <= 0) return 1;
  if (use_prefill(d, T)) {
    // (what the workspace was sized for; a layer narrower than the widest one could ask for more pieces than fit)
    const int sp = moe_prefill_shared_splits(d.fmt, T, d.H, d.I_sh);
    return (size_t)sp * T * d.H <= s->part_s_elems ? sp : 1;
  }
  return d.fmt == MOE_FMT_Q4K ? moe_decode_shared_splits(MOE_FMT_Q4K, T, d.H, d.I_sh) : 1;
}

// what the one-token w2 + combine kernel asks of a layer (its waves stage what they need themselves, so the
// widths of the experts do not matter; a lane per unit holds the unit's address)
// launches that take a host copy of the slot table carry at most this many entries in their arguments
static constexpr int kTableByValueMax = 64;
static bool table_by_value(int E) {   // MOE_TABLE_BY_VALUE=0: always refresh and read the device table
  static const bool on = [] { const char *e = getenv("MOE_TABLE_BY_VALUE"); return !e || atoi(e) != 0; }();
  return on && E <= kTableByValueMax;
}

static bool w2c_fits(const moe_layer_desc &d, int k) { return d.H % 16 == 0 && k < 64; }


// Gate logits, top-k and dispatch of a decode batch of 2 to 32 tokens: one launch (the gate rows' workgroups hand
// the logits to the routing workgroup inside it), or the gate launch(es) and the routing launch
static int gate_parts_env() {
  static const int v = [] { const char *e = getenv("MOE_GATE_ROUTE"); return e ? atoi(e) : 1; }();
  return v;
}
static int route_batch(const moe_layer_desc &d, LayerState *s, const void *x, int T, int E, int k, int n_gate_rows, int ldl,
                       int max_units, int layer, moe_unit *host_units, int *host_n, int *host_seq, int seq_val,
                       hipStream_t st) {
  int rc;
  const int parts = gate_parts_env();
  if (T >= 2 && d.H % 8 == 0 && (parts == 1 || parts == 8) &&
      moe_gate_route_ws_bytes(T, n_gate_rows) <= (int64_t)s->gate_ws_bytes) {
    s->gate_seq = s->gate_seq < 0x7fffffff ? s->gate_seq + 1 : 1;
    return moe_gate_topk_dispatch(x, d.gate_w, d.gate_bias, d.gate_bias ? E : 0, s->logits, T, d.H, E, n_gate_rows, ldl, k,
                                  d.route_mode, s->idx, s->topk_w, s->counts, s->offsets, s->sorted_pair, s->pos_of_pair,
                                  s->sorted_tok, s->units, s->n_active, s->active_ids, max_units, host_units, host_n,
                                  host_seq, seq_val, s->gate_ws, s->gate_seq, parts, s->err_host + layer, st);
  }
  if (!d.gate_bias) {
    if ((rc = moe_gate_logits(x, d.gate_w, nullptr, s->logits, T, d.H, n_gate_rows, ldl, st))) return rc;
  } else {
    // the bias covers the routed experts only; the shared-gate row (row E) has none
    if ((rc = moe_gate_logits(x, d.gate_w, d.gate_bias, s->logits, T, d.H, E, ldl, st))) return rc;
    if (d.shared_gated &&
        (rc = moe_gate_logits(x, (const uint16_t *)d.gate_w + (size_t)E * d.H, nullptr, s->logits + E, T, d.H, 1, ldl, st)))
      return rc;
  }
  return moe_topk_dispatch(s->logits, T, E, ldl, k, d.route_mode, s->idx, s->topk_w, s->counts, s->offsets,
                           s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                           max_units, host_units, host_n, host_seq, seq_val, st);
}

// a decode batch whose w13 launch computes the gate logits and routes by itself (int4, 2 to 8 tokens)
static bool batch_routes_in_w13(const moe_layer_desc &d, const LayerState *s, int T, int E, int k, int n_gate_rows) {
  static const bool on = [] { const char *e = getenv("MOE_BATCH_ROUTE"); return !e || atoi(e) != 0; }();
  return on && d.fmt == MOE_FMT_INT4_G128 && !use_prefill(d, T) &&
         moe_decode_batch_int4_gate_fits(T, E, k, d.H, d.I, d.I_sh, n_gate_rows) &&
         moe_gate_route_ws_bytes(T, n_gate_rows) <= (int64_t)s->gate_ws_bytes;
}

extern "C" int moe_forward(moe_engine *eng, int layer, const void *x, int T, void *y) {
  if (!eng) { moe_set_error("null engine"); return MOE_EINVAL; }
  if (!eng->fatal.empty()) { moe_set_error("engine is in a failed state: %s", eng->fatal.c_str()); return MOE_ESTATE; }
  if (layer < 0 || layer >= eng->cfg.num_layer || !x || !y || T <= 0) { moe_set_error("moe_forward: bad argument"); return MOE_EINVAL; }
  LayerState *s = eng->fw;
  const moe_layer_desc &d = eng->layer_desc[layer];
  if (!s || !d.gate_w) { moe_set_error("moe_forward: layer %d not described or workspace not prepared", layer); return MOE_ESTATE; }
  if (T > s->max_tokens) { moe_set_error("moe_forward: T=%d exceeds the prepared workspace (%d)", T, s->max_tokens); return MOE_EINVAL; }
  if (!eng->launched) { moe_set_error("engine not launched"); return MOE_ESTATE; }
  const int E = eng->cfg.num_expert, k = d.top_k;
  hipStream_t st = (hipStream_t)eng->be->compute_stream();
  const int n_gate_rows = E + (d.shared_gated ? 1 : 0);
  const int ldl = E + 1;
  int rc;
  // hook order of the reference (utils/hooks.py:216-223)
  // the layer hook's pre_forward: this block's input (decode: what the built-in predictor reads)
  if ((rc = moe_forward_check_kernels(eng))) return rc;  // of earlier calls: the words arrive without a copy
  // (a one-token step that will launch its gate kernel below takes the predictor's score rows into that launch)
  const bool token_kernels = T == 1 && d.fmt == MOE_FMT_INT4_G128 && E <= 256 && k <= 32 &&
                             eng->cfg.early_preempt && eng->cfg.reorder_experts && (size_t)d.H * 2 + 8192 <= 60 * 1024;
  const void *pred_w = nullptr; const float *pred_b = nullptr; float *pred_out = nullptr; int pred_rows = 0;
  bool pred_fused = token_kernels && moe_predictor_fused_rows(eng, layer, d.H, &pred_w, &pred_b, &pred_out, &pred_rows);
  if (pred_fused) {
    if ((rc = moe_report_layer_logits_bookkeeping(eng, layer, T))) return rc;
  } else if ((rc = moe_report_layer_logits(eng, layer, x, 1, T, d.H))) return rc;
  const int max_units = (int)std::min<size_t>(E, (size_t)T * k);
  if ((rc = moe_forward_harvest(eng, false))) return rc;
  // Every expert of the layer resident, and the layer's slot group can hold them all: there
  // is nothing for the host to decide, so no round trip.  The kernels take the device-built
  // unit list; the routing comes back asynchronously and the hits are accounted when it lands.
  bool all_resident = false;
  {
    SpinGuard lk(eng->mu);
    // (with a predictor attached the hooks' budget / progress bookkeeping has to run: no short cut)
    all_resident = eng->cfg.per_layer_cache && eng->cfg.early_preempt && (int)eng->group_of(layer).full_len == E &&
                   eng->layer_complete[layer] == E && !eng->predictor_attached;
  }
  if (all_resident && T == 1 && d.fmt == MOE_FMT_INT4_G128 && E <= 256 && k <= 32 && (size_t)d.H * 2 + 8192 <= 60 * 1024) {
    // one token: the w13 launch computes the gate logits in its first workgroups and routes by itself (no gate,
    // top-k or dispatch launches): two launches per step
    const uint64_t *table = nullptr;
    if ((rc = moe_expert_ptr_table(eng, layer, &table))) return rc;
    if ((rc = moe_flush_table(eng, layer, st))) return rc;
    LayerState::Pending &p = s->pend[s->pend_head];
    if (p.busy && (rc = moe_forward_harvest(eng, true))) return rc;
    s->pend_head = (s->pend_head + 1) % LayerState::kPending;
    // the kernel stores the unit list into the pending slot's pinned memory and then the sequence word
    const int seq = ++s->seq_counter;
    const float *sg0 = d.shared_gated ? s->logits + E : nullptr;
    const bool w2c = w2c_fits(d, k);  // w2 and the combine in one launch
    s->gate_seq = s->gate_seq < 0x7fffffff ? s->gate_seq + 1 : 1;
    if ((rc = moe_decode_token_int4_gate(x, d.gate_w, d.gate_bias, n_gate_rows, s->gate_ws, s->gate_seq, s->logits, E, k,
                                         d.route_mode, d.H, d.I, d.I_sh, table, nullptr,
                                         d.I_sh > 0 ? d.shared : nullptr, s->idx, s->topk_w, s->counts, s->offsets,
                                         s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                                         s->h_r, s->h_s, s->part_r, s->part_s, s->err_host + layer, s->unit_ws, p.units, p.seq, seq,
                                         w2c ? 5 : 3, sg0, y, st)))
      return rc;
    *p.n_active = k;
    p.layer = layer; p.max_units = max_units; p.busy = true; p.by_seq = true; p.seq_expected = seq;
    if (!w2c &&
        (rc = moe_combine(s->part_r, d.I_sh > 0 ? s->part_s : nullptr, s->topk_w, s->pos_of_pair, sg0, ldl, y, T, d.H, k, st)))
      return rc;
    if (layer + 1 == eng->cfg.num_layer && (rc = moe_report_layer_logits(eng, layer + 1, y, 1, T, d.H))) return rc;
    return moe_layer_done(eng, layer);
  }
  // One token that may meet non-resident experts: start the expert kernels on whatever is resident BEFORE
  // the host knows the routing.  The w13 kernel routes by itself, skips experts whose table entry is 0 and
  // hands the unit list to the host through pinned memory; the host then runs the cache hooks in the
  // reference's order (hits were computed already, misses are fetched and computed one by one) while the GPU
  // works.  From the table snapshot until the hooks have marked the hits, the layer's slot group is guarded:
  // prefetch and demand traffic may evict, but no copy into one of its slots starts.
  const bool optimistic = !all_resident && token_kernels;
  if (pred_fused && !optimistic) {  // (cannot happen while a predictor rules out the all-resident short cut)
    pred_fused = false;
    if ((rc = moe_predictor_on_logits(eng, layer, x, 1, T, d.H))) return rc;
  }
  if (optimistic) {
    const int rows1 = d.gate_bias ? E : n_gate_rows;
    if (pred_fused) {
      if ((rc = moe_gate_logits_pair(x, d.gate_w, d.gate_bias, s->logits, T, d.H, rows1, ldl, pred_w, pred_b, pred_out,
                                     pred_rows, pred_rows, st)))
        return rc;
      if (d.gate_bias && d.shared_gated &&
          (rc = moe_gate_logits(x, (const uint16_t *)d.gate_w + (size_t)E * d.H, nullptr, s->logits + E, T, d.H, 1, ldl, st)))
        return rc;
    }  // (without the predictor's rows the w13 launch below computes the gate logits itself)
    const uint64_t *table = nullptr;
    if ((rc = moe_expert_ptr_table(eng, layer, &table))) return rc;
    // what the kernel will find resident: exactly these experts get computed by it
    std::vector<char> resident_at_launch(E);
    // Up to 64 experts the launches below carry the slot table in their arguments (the routing launch) or take
    // resolved units (the others): the device table is not read, and its refresh after a miss, a copy in the stream
    // in front of the routing launch, is not made (it held the routing back from the host, and with it the demand
    // copy of the next miss, by 5 to 7 us).
    uint64_t tab_now[kTableByValueMax];
    const uint64_t *tab_host = table_by_value(E) ? tab_now : nullptr;
    if ((rc = tab_host ? moe_snapshot_table_guarded(eng, layer, tab_now, resident_at_launch.data())
                       : moe_flush_table_guarded(eng, layer, st, resident_at_launch.data())))
      return rc;
    struct GuardRelease {  // on every way out, errors included
      moe_engine *eng; int layer; bool armed;
      void release() { if (armed) { armed = false; moe_guard_release(eng, layer); } }
      ~GuardRelease() { release(); }
    } guard{eng, layer, true};
    const int seq = ++s->seq_counter;
    if (pred_fused) {
      rc = moe_decode_token_int4(x, s->logits, E, k, d.route_mode, d.H, d.I, d.I_sh, table, tab_host,
                                 d.I_sh > 0 ? d.shared : nullptr, s->idx, s->topk_w, s->counts, s->offsets,
                                 s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                                 s->h_r, s->h_s, s->part_r, s->part_s, s->err_loose, s->unit_ws, s->units_host, s->opt_seq, seq, 1,
                                 nullptr, nullptr, st);
    } else {
      s->gate_seq = s->gate_seq < 0x7fffffff ? s->gate_seq + 1 : 1;
      rc = moe_decode_token_int4_gate(x, d.gate_w, d.gate_bias, n_gate_rows, s->gate_ws, s->gate_seq, s->logits, E, k,
                                      d.route_mode, d.H, d.I, d.I_sh, table, tab_host,
                                      d.I_sh > 0 ? d.shared : nullptr, s->idx, s->topk_w, s->counts, s->offsets,
                                      s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                                      s->h_r, s->h_s, s->part_r, s->part_s, s->err_loose, s->unit_ws, s->units_host, s->opt_seq, seq, 1,
                                      nullptr, nullptr, st);
    }
    if (rc) return rc;
    // the predictor's scores came out of the gate launch above: complete once this kernel's sequence word arrives
    if (pred_fused && (rc = moe_predictor_scores_pending(eng, layer, s->opt_seq, seq))) return rc;
    // The w2 pass with the combine goes out at once as well, as if nothing were missing: in most steps nothing
    // is, and then the GPU has this layer's kernels queued while the host runs the hooks and is never waited
    // for.  When an expert turns out to be missing, its output is recomputed below (the kernel skips the
    // missing expert and raises its own error word, which the host then knows to expect).
    const float *sgo = d.shared_gated ? s->logits + E : nullptr;
    const bool spec_w2c = w2c_fits(d, k);
    const int sw = 2 * layer + (int)(s->spec_turn[layer] & 1u);   // this turn's word
    if (spec_w2c) {
      s->spec_turn[layer]++;
      if (s->spec_state[sw] == 1 && ((volatile int *)s->err_spec)[sw])   // the launch of two turns ago: final
        return engine_fail(eng, "a kernel of layer %d met a selected expert without a slot: its output is wrong", layer);
      s->spec_state[sw] = 0;
      s->err_spec[sw] = 0;
      if ((rc = moe_decode_token_int4(x, s->logits, E, k, d.route_mode, d.H, d.I, d.I_sh, table, nullptr,
                                      d.I_sh > 0 ? d.shared : nullptr, s->idx, s->topk_w, s->counts, s->offsets,
                                      s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                                      s->h_r, s->h_s, s->part_r, s->part_s, s->err_spec + sw, s->unit_ws,
                                      nullptr, nullptr, 0, 4, sgo, y, st)))
        return rc;
    }
    {  // the routing arrives a few microseconds after the kernel starts
      volatile int *sq = s->opt_seq;
      const auto t0 = std::chrono::steady_clock::now();
      unsigned spins = 0;
      while (*sq != seq) {
        if ((++spins & 1023u) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::seconds(5)) {
          HIPC(hipStreamSynchronize(st));
          if (*sq != seq) { moe_set_error("routing of layer %d never reached the host", layer); return MOE_EHIP; }
        }
      }
      __atomic_thread_fence(__ATOMIC_ACQUIRE);
    }
    const int n_act = k;
    std::vector<int64_t> ids(n_act);
    std::unordered_map<int, moe_unit> unit_of;
    for (int u = 0; u < n_act; ++u) { ids[u] = s->units_host[u].expert; unit_of[s->units_host[u].expert] = s->units_host[u]; }
    if ((rc = moe_report_one_layer(eng, layer, ids.data(), n_act))) return rc;
    std::vector<int64_t> later, now_ids;
    {
      SpinGuard lk(eng->mu);
      for (int i = 0; i < n_act; ++i) {
        // resident at launch and still there (now `launching`: nobody overwrites it): computed already.
        // A missed expert whose copy has landed meanwhile is `launching` too, but still has to be computed;
        // so has one that a prefetch evicted between the snapshot and now (its slot was intact while the
        // guard stood, but is free to be overwritten from here on).
        Expert *ex = eng->ex(layer, (int)ids[i]);
        if (resident_at_launch[(int)ids[i]] && ex->status.load() == kLaunching && ex->num_ready == eng->cfg.num_per_expert_param &&
            eng->h_table[(size_t)layer * E + ids[i]] != 0)
          now_ids.push_back(ids[i]);
        else
          later.push_back(ids[i]);
      }
      eng->ctr.ready += (uint64_t)now_ids.size();
    }
    guard.release();
    // With every selected expert resident the launch above was the whole layer.  Otherwise the late experts
    // follow as their copies land: each one's w13 launch alone (it also writes the expert's slot address into the
    // step's published unit list), then w2 over ALL units with the combine in one launch, which overwrites what the
    // speculative launch left in y.  That needs every late expert in a slot of its own until the last launch
    // (they stay `launching` till then): only when the layer's slot group has room for that; else the w2 pass
    // goes out again without the combine, every late expert runs w13 and w2 and is released at once, and the
    // combine closes the layer (three more launches per step instead of one per late expert plus one).
    const bool w2c = later.empty() && spec_w2c;
    if (spec_w2c) s->spec_state[sw] = later.empty() ? 1 : 2;
    bool late_w13_only = false;
    if (!w2c && spec_w2c) {
      SpinGuard lk(eng->mu);
      late_w13_only = later.size() + now_ids.size() <= eng->group_of(layer).full_len;
    }
    if (!w2c && !late_w13_only &&
        (rc = moe_decode_token_int4(x, s->logits, E, k, d.route_mode, d.H, d.I, d.I_sh, table, nullptr,
                                    d.I_sh > 0 ? d.shared : nullptr, s->idx, s->topk_w, s->counts, s->offsets,
                                    s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                                    s->h_r, s->h_s, s->part_r, s->part_s, s->err_loose, s->unit_ws,
                                    nullptr, nullptr, 0, 2, sgo, y, st)))
      return rc;
    // no event in the stream (one costs the step about 4 us of GPU time): the experts count as in use until
    // the routing word of a LATER one-token step arrives, whose kernel starts behind everything queued here
    if (!now_ids.empty() &&
        (rc = moe_release_experts_seq(eng, layer, now_ids.data(), (int64_t)now_ids.size(), s->opt_seq, seq + 1)))
      return rc;
    s->sub_cursor = 0;
    for (int64_t id : later) {
      if ((rc = moe_wait_expert(eng, layer, (int)id))) return rc;
      if (late_w13_only) {
        uint64_t addr = 0;
        {
          SpinGuard lk(eng->mu);
          addr = eng->h_table[(size_t)layer * E + id];
        }
        if ((rc = moe_decode_token_late_expert_int4(x, d.H, d.I, addr, unit_of[(int)id].row0, s->h_r, s->unit_ws,
                                                    s->err_host + layer, st)))
          return rc;
        continue;   // still `launching`: the w2 + combine launch below reads its slot too
      }
      moe_unit *slot_h = s->units_sub_host + s->sub_cursor;
      *slot_h = unit_of[(int)id];
      // (an int4 decode launch of one unit takes the unit and its slot address in the kernel arguments: no device
      // copy of the unit, and the device table is not read, so its flush, a copy in the stream in front of the
      // launch, waits for the layer's next turn)
      if ((rc = run_units(eng, d, s, x, T, s->units_sub + s->sub_cursor, slot_h, 1, false, layer, table, st))) return rc;
      s->sub_cursor++;
      if ((rc = moe_expert_launched(eng, layer, (int)id))) return rc;
    }
    if (late_w13_only) {
      if ((rc = moe_decode_token_int4(x, s->logits, E, k, d.route_mode, d.H, d.I, d.I_sh, table, nullptr,
                                      d.I_sh > 0 ? d.shared : nullptr, s->idx, s->topk_w, s->counts, s->offsets,
                                      s->sorted_pair, s->pos_of_pair, s->sorted_tok, s->units, s->n_active, s->active_ids,
                                      s->h_r, s->h_s, s->part_r, s->part_s, s->err_host + layer, s->unit_ws,
                                      nullptr, nullptr, 0, 4, sgo, y, st)))
        return rc;
      for (int64_t id : later)
        if ((rc = moe_expert_launched(eng, layer, (int)id))) return rc;
    } else if (!w2c &&
               (rc = moe_combine(s->part_r, d.I_sh > 0 ? s->part_s : nullptr, s->topk_w, s->pos_of_pair, sgo, ldl, y, T, d.H, k, st)))
      return rc;
    if (layer + 1 == eng->cfg.num_layer && (rc = moe_report_layer_logits(eng, layer + 1, y, 1, T, d.H))) return rc;
    return moe_layer_done(eng, layer);
  }
  bool routed_by_tail = false, w13_publishes = false;
  int tail_seq = 0, host_seq = 0;  // host_seq != 0: the unit list comes to units_host with this value in *opt_seq
  if (all_resident && batch_routes_in_w13(d, s, T, E, k, n_gate_rows)) {
    // 2 to 8 tokens, nothing for the host to decide: the w13 launch sums the gate rows, routes by itself and hands
    // the unit list to the host through the pending slot's pinned memory; then w2 and the combine (three launches)
    LayerState::Pending &p = s->pend[s->pend_head];
    if (p.busy && (rc = moe_forward_harvest(eng, true))) return rc;
    s->pend_head = (s->pend_head + 1) % LayerState::kPending;
    const int seq = ++s->seq_counter;
    const uint64_t *table = nullptr;
    if ((rc = moe_expert_ptr_table(eng, layer, &table))) return rc;
    if ((rc = moe_flush_table(eng, layer, st))) return rc;
    s->gate_seq = s->gate_seq < 0x7fffffff ? s->gate_seq + 1 : 1;
    if ((rc = moe_decode_batch_int4_gate(x, T, d.gate_w, d.gate_bias, n_gate_rows, s->gate_ws, s->gate_seq, s->logits, ldl, E,
                                         k, d.route_mode, d.H, d.I, d.I_sh, table, nullptr, d.I_sh > 0 ? d.shared : nullptr, s->idx,
                                         s->topk_w, s->counts, s->offsets, s->sorted_pair, s->pos_of_pair, s->sorted_tok,
                                         s->units, s->n_active, s->active_ids, max_units, s->h_r, s->h_s, s->part_r,
                                         s->part_s, s->err_host + layer, p.units, p.n_active, p.seq, seq, 3, st)))
      return rc;
    p.layer = layer; p.max_units = max_units; p.busy = true; p.by_seq = true; p.seq_expected = seq;
    const float *sg0 = d.shared_gated ? s->logits + E : nullptr;
    if ((rc = moe_combine_splits(s->part_r, d.I_sh > 0 ? s->part_s : nullptr, s->topk_w, s->pos_of_pair, sg0, ldl, y, T, d.H, k,
                                 1, st)))
      return rc;
    if (layer + 1 == eng->cfg.num_layer && (rc = moe_report_layer_logits(eng, layer + 1, y, 1, T, d.H))) return rc;
    return moe_layer_done(eng, layer);
  }
  static const bool batch_spec_on = [] { const char *e = getenv("MOE_BATCH_SPEC"); return !e || atoi(e) != 0; }();
  // (more than 8 tokens: only while the layer's last turn missed at most one expert; with several misses a step the
  // time is in the copies, which start no earlier this way, and the recomputed units cost more than the wait saved:
  // 16 tokens at cache rate 0.375 370 -> 379 us per step, at 0.97 85 -> 77)
  if (!all_resident && batch_spec_on && eng->cfg.early_preempt && eng->cfg.reorder_experts &&
      (T <= 8 || s->late_last[layer] <= 1) && batch_routes_in_w13(d, s, T, E, k, n_gate_rows)) {
    // 2 to 16 tokens that may meet non-resident experts: as for one token, the expert launches go out BEFORE the host
    // knows the routing.  The self-routing w13 launch and the w2 launch behind it compute what is resident (a unit
    // whose table entry is 0 is skipped and raises the loose error word) and hand the unit list to the host, which
    // runs the cache hooks in the reference's order while the GPU works; the units that were not resident follow as
    // their copies land, then the combine.  The GPU used to idle from the end of the routing launch until the host had
    // seen the routing, run the hooks and launched (about 8 us per step).  The slot group is guarded from the table
    // snapshot until the hooks have marked the hits, as in the one-token path.
    const uint64_t *table = nullptr;
    if ((rc = moe_expert_ptr_table(eng, layer, &table))) return rc;
    std::vector<char> resident_at_launch(E);
    uint64_t tab_now[kTableByValueMax];   // (the launches carry the table in their arguments: no refresh of the device table)
    const uint64_t *tab_host = table_by_value(E) ? tab_now : nullptr;
    if ((rc = tab_host ? moe_snapshot_table_guarded(eng, layer, tab_now, resident_at_launch.data())
                       : moe_flush_table_guarded(eng, layer, st, resident_at_launch.data())))
      return rc;
    struct GuardRelease {  // on every way out, errors included
      moe_engine *eng; int layer; bool armed;
      void release() { if (armed) { armed = false; moe_guard_release(eng, layer); } }
      ~GuardRelease() { release(); }
    } guard{eng, layer, true};
    const int seq = ++s->seq_counter;
    s->gate_seq = s->gate_seq < 0x7fffffff ? s->gate_seq + 1 : 1;
    if ((rc = moe_decode_batch_int4_gate(x, T, d.gate_w, d.gate_bias, n_gate_rows, s->gate_ws, s->gate_seq, s->logits, ldl, E,
                                         k, d.route_mode, d.H, d.I, d.I_sh, table, tab_host, d.I_sh > 0 ? d.shared : nullptr, s->idx,
                                         s->topk_w, s->counts, s->offsets, s->sorted_pair, s->pos_of_pair, s->sorted_tok,
                                         s->units, s->n_active, s->active_ids, max_units, s->h_r, s->h_s, s->part_r,
                                         s->part_s, s->err_loose_dev, s->units_host, s->n_active_host, s->opt_seq, seq, 3, st)))
      return rc;
    {  // the routing arrives a few microseconds after the launch starts
      volatile int *sq = s->opt_seq;
      const auto t0 = std::chrono::steady_clock::now();
      unsigned spins = 0;
      while (*sq != seq) {
        if ((++spins & 1023u) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::seconds(5)) {
          HIPC(hipStreamSynchronize(st));
          if (*sq != seq) { moe_set_error("routing of layer %d never reached the host", layer); return MOE_EHIP; }
        }
      }
      __atomic_thread_fence(__ATOMIC_ACQUIRE);
    }
    const int n_act = std::min(*s->n_active_host, max_units);
    std::vector<int64_t> ids(n_act);
    std::unordered_map<int, moe_unit> unit_of;
    for (int u = 0; u < n_act; ++u) { ids[u] = s->units_host[u].expert; unit_of[s->units_host[u].expert] = s->units_host[u]; }
    if ((rc = moe_report_one_layer(eng, layer, ids.data(), n_act))) return rc;
    std::vector<int64_t> later, now_ids;
    {
      SpinGuard lk(eng->mu);
      for (int i = 0; i < n_act; ++i) {
        // resident at launch and still there (now `launching`): computed already; anything else (missed, or evicted
        // by a prefetch between the snapshot and the hooks) is computed when it is usable
        Expert *ex = eng->ex(layer, (int)ids[i]);
        if (resident_at_launch[(int)ids[i]] && ex->status.load() == kLaunching && ex->num_ready == eng->cfg.num_per_expert_param &&
            eng->h_table[(size_t)layer * E + ids[i]] != 0)
          now_ids.push_back(ids[i]);
        else
          later.push_back(ids[i]);
      }
      eng->ctr.ready += (uint64_t)now_ids.size();
    }
    s->late_last[layer] = (unsigned char)std::min<size_t>(later.size(), 255);
    guard.release();
    // launching -> using.  No event in the stream where that is safe: the experts count as in use until the sequence
    // word of a LATER launch arrives.  A batch can route to more experts than the layer has slots, and then a demand
    // copy of this very step picks one of these experts as its victim: it would stand for the 100 us the fetch thread
    // gives the word before it falls back to an event (16 tokens at cache rate 0.375: 373 -> 381-389 us per step), so
    // such a step releases against an event recorded now.  (With the routed experts no more than the slots, the
    // victims of this step's copies are experts it did not touch: they are the least recently used.)
    if (!now_ids.empty()) {
      size_t slots_of_layer;
      {
        SpinGuard lk(eng->mu);
        slots_of_layer = eng->group_of(layer).full_len;
      }
      rc = (size_t)n_act <= slots_of_layer && eng->cfg.per_layer_cache
               ? moe_release_experts_seq(eng, layer, now_ids.data(), (int64_t)now_ids.size(), s->opt_seq, seq + 1)
               : moe_release_experts(eng, layer, now_ids.data(), (int64_t)now_ids.size());
      if (rc) return rc;
    }
    s->sub_cursor = 0;
    for (int64_t id : later) {
      if ((rc = moe_wait_expert(eng, layer, (int)id))) return rc;
      moe_unit *slot_h = s->units_sub_host + s->sub_cursor;
      *slot_h = unit_of[(int)id];
      // (one unit by value: its slot address travels in the kernel arguments, the device table is not read)
      if ((rc = run_units(eng, d, s, x, T, s->units_sub + s->sub_cursor, slot_h, 1, false, layer, table, st))) return rc;
      s->sub_cursor++;
      if ((rc = moe_expert_launched(eng, layer, (int)id))) return rc;
    }
    const float *sgo = d.shared_gated ? s->logits + E : nullptr;
    if ((rc = moe_combine_splits(s->part_r, d.I_sh > 0 ? s->part_s : nullptr, s->topk_w, s->pos_of_pair, sgo, ldl, y, T, d.H, k, 1,
                                 st)))
      return rc;
    if (layer + 1 == eng->cfg.num_layer && (rc = moe_report_layer_logits(eng, layer + 1, y, 1, T, d.H))) return rc;
    return moe_layer_done(eng, layer);
  }
  if (all_resident && T <= 32 && E <= 256 && k <= 32 && T * k <= 512) {
    // decode batch, nothing for the host to decide: logits, then top-k + dispatch in one launch that
    // also hands the unit list to the host through the next pending slot's pinned memory
    LayerState::Pending &pn = s->pend[s->pend_head];
    if (pn.busy && (rc = moe_forward_harvest(eng, true))) return rc;
    tail_seq = ++s->seq_counter;
    // the unit list reaches the host from the w13 launch where that one can carry it (its stores to pinned memory
    // hold the routing launch for about 2 us, and nothing in the w13 launch waits for them), else from here
    w13_publishes = decode_publishes(d, T, max_units);
    if ((rc = route_batch(d, s, x, T, E, k, n_gate_rows, ldl, max_units, layer, w13_publishes ? nullptr : pn.units,
                          w13_publishes ? nullptr : pn.n_active, w13_publishes ? nullptr : pn.seq, tail_seq, st)))
      return rc;
    routed_by_tail = true;
  } else if (T <= 32 && E <= 256 && k <= 32 && T * k <= 512) {
    // decode batch whose routing the host has to see before it can go on (experts may be missing): logits, then
    // top-k + dispatch in one launch that stores the unit list into pinned host memory and, behind it, a sequence
    // word; the host polls the word below.  Two copies, an event and a blocking wait for it took 15-20 us per step.
    host_seq = ++s->seq_counter;
    if ((rc = route_batch(d, s, x, T, E, k, n_gate_rows, ldl, max_units, layer, s->units_host, s->n_active_host, s->opt_seq,
                          host_seq, st)))
      return rc;
  } else {
    if (!d.gate_bias) {
      if ((rc = moe_gate_logits(x, d.gate_w, nullptr, s->logits, T, d.H, n_gate_rows, ldl, st))) return rc;
    } else {
      // the bias covers the routed experts only; the shared-gate row (row E) has none
      if ((rc = moe_gate_logits(x, d.gate_w, d.gate_bias, s->logits, T, d.H, E, ldl, st))) return rc;
      if (d.shared_gated &&
          (rc = moe_gate_logits(x, (const uint16_t *)d.gate_w + (size_t)E * d.H, nullptr, s->logits + E, T, d.H, 1, ldl, st)))
        return rc;
    }
    if ((rc = moe_topk(s->logits, T, E, ldl, k, d.route_mode, s->idx, s->topk_w, st))) return rc;
    // (the workspace is sized for max_tokens: a smaller batch needs no more of it)
    if ((rc = moe_dispatch_ws(s->idx, T, k, E, s->counts, s->offsets, s->sorted_pair, s->pos_of_pair, s->sorted_tok,
                              s->units, s->n_active, s->active_ids, max_units, s->disp_ws, s->disp_ws_bytes,
                              s->err_host + layer, st)))
      return rc;
  }
  if (all_resident) {
    LayerState::Pending &p = s->pend[s->pend_head];
    if (p.busy && (rc = moe_forward_harvest(eng, true))) return rc;
    s->pend_head = (s->pend_head + 1) % LayerState::kPending;
    p.layer = layer; p.max_units = max_units; p.busy = true;
    if (routed_by_tail) {  // the routing kernel stores the unit list in the slot's pinned memory itself
      p.by_seq = true; p.seq_expected = tail_seq;
    } else {
      HIPC(hipMemcpyAsync(p.units, s->units, sizeof(moe_unit) * max_units, hipMemcpyDeviceToHost, st));
      HIPC(hipMemcpyAsync(p.n_active, s->n_active, sizeof(int), hipMemcpyDeviceToHost, st));
      HIPC(hipEventRecord(p.ev, st));
      p.by_seq = false;
    }
    const uint64_t *table = nullptr;
    if ((rc = moe_expert_ptr_table(eng, layer, &table))) return rc;
    if ((rc = moe_flush_table(eng, layer, st))) return rc;
    if ((rc = run_units(eng, d, s, x, T, s->units, nullptr, max_units, d.I_sh > 0, layer, table, st,
                        w13_publishes ? &p : nullptr, tail_seq)))
      return rc;
    const float *sg0 = d.shared_gated ? s->logits + E : nullptr;
    if ((rc = moe_combine_splits(s->part_r, d.I_sh > 0 ? s->part_s : nullptr, s->topk_w, s->pos_of_pair, sg0, ldl, y, T, d.H, k,
                                 shared_pieces(d, T, s), st)))
      return rc;
    if (layer + 1 == eng->cfg.num_layer && (rc = moe_report_layer_logits(eng, layer + 1, y, 1, T, d.H))) return rc;
    return moe_layer_done(eng, layer);
  }
  // the active expert list comes back to the host
  if (host_seq) {
    volatile int *sq = s->opt_seq;
    const auto t0 = std::chrono::steady_clock::now();
    unsigned spins = 0;
    while (*sq != host_seq) {
      if ((++spins & 1023u) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::seconds(5)) {
        HIPC(hipStreamSynchronize(st));
        if (*sq != host_seq) { moe_set_error("routing of layer %d never reached the host", layer); return MOE_EHIP; }
      }
    }
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
  } else {
    HIPC(hipMemcpyAsync(s->units_host, s->units, sizeof(moe_unit) * max_units, hipMemcpyDeviceToHost, st));
    HIPC(hipMemcpyAsync(s->n_active_host, s->n_active, sizeof(int), hipMemcpyDeviceToHost, st));
    HIPC(hipEventRecord(s->ev, st));
    HIPC(hipEventSynchronize(s->ev));
  }
  const int n_act = *s->n_active_host;
  std::vector<int64_t> ids(n_act);
  std::unordered_map<int, moe_unit> unit_of;
  for (int u = 0; u < n_act; ++u) { ids[u] = s->units_host[u].expert; unit_of[s->units_host[u].expert] = s->units_host[u]; }
  // report_experts (utils/__init__.py:84-88): in-place reorder, hits -> launching, misses queued
  if ((rc = moe_report_one_layer(eng, layer, ids.data(), n_act))) return rc;
  const uint64_t *table = nullptr;
  if ((rc = moe_expert_ptr_table(eng, layer, &table))) return rc;
  // resident experts: one grouped launch, together with the shared expert
  std::vector<int64_t> later, now_ids;
  int n_now = 0;
  s->sub_cursor = 0;
  moe_unit *sub_h = s->units_sub_host;
  {
    SpinGuard lk(eng->mu);
    for (int i = 0; i < n_act; ++i) {
      Expert *e = eng->ex(layer, (int)ids[i]);
      if (eng->cfg.early_preempt && e->status.load() == kLaunching) { sub_h[n_now++] = unit_of[(int)ids[i]]; now_ids.push_back(ids[i]); }
      else later.push_back(ids[i]);
    }
    eng->ctr.ready += (uint64_t)n_now;
  }
  s->late_last[layer] = (unsigned char)std::min<size_t>(later.size(), 255);
  // int4 decode launches of up to 64 units take the units and their slot addresses in the kernel arguments
  // (run_units hands over the host copies): the device copy of a sub-list is then never read, and its
  // host-to-device copy would only put 4 us into the stream in front of the launch.  The same holds for the
  // refresh of the device table after a miss, which such a launch does not read either.
  const bool by_value = d.fmt == MOE_FMT_INT4_G128 && !use_prefill(d, T);
  if (!(by_value && n_now <= 64) && (rc = moe_flush_table(eng, layer, st))) return rc;
  const moe_unit *units_now = s->units;
  if (!later.empty() || n_now != n_act) {
    if (n_now && !(by_value && n_now <= 64))
      HIPC(hipMemcpyAsync(s->units_sub, sub_h, sizeof(moe_unit) * n_now, hipMemcpyHostToDevice, st));
    units_now = s->units_sub;
    s->sub_cursor = n_now;
  }
  if (n_now > 0 || d.I_sh > 0)
    if ((rc = run_units(eng, d, s, x, T, units_now, units_now == s->units ? s->units_host : sub_h, n_now, d.I_sh > 0,
                        layer, table, st)))
      return rc;
  // launching -> using right away: the demand copies queued for the missed experts may
  // pick these slots as victims and must only wait for this launch, not for the whole layer
  if (n_now > 0 && (rc = moe_release_experts(eng, layer, now_ids.data(), n_now))) return rc;
  // missed experts in the returned order, one at a time as their copies land
  for (int64_t id : later) {
    if ((rc = moe_wait_expert(eng, layer, (int)id))) return rc;
    if (!by_value && (rc = moe_flush_table(eng, layer, st))) return rc;  // (by value: the device table is not read)
    moe_unit *slot_h = s->units_sub_host + s->sub_cursor;
    *slot_h = unit_of[(int)id];
    if (!by_value) HIPC(hipMemcpyAsync(s->units_sub + s->sub_cursor, slot_h, sizeof(moe_unit), hipMemcpyHostToDevice, st));
    if ((rc = run_units(eng, d, s, x, T, s->units_sub + s->sub_cursor, slot_h, 1, false, layer, table, st))) return rc;
    s->sub_cursor++;
    if ((rc = moe_expert_launched(eng, layer, (int)id))) return rc;
  }
  const float *sg = d.shared_gated ? s->logits + E : nullptr;
  if ((rc = moe_combine_splits(s->part_r, d.I_sh > 0 ? s->part_s : nullptr, s->topk_w, s->pos_of_pair, sg, ldl, y, T, d.H, k,
                               shared_pieces(d, T, s), st)))
    return rc;
  // MoeLayerHook.post_forward (utils/hooks.py:220-223)
  if (layer + 1 == eng->cfg.num_layer && (rc = moe_report_layer_logits(eng, layer + 1, y, 1, T, d.H))) return rc;
  return moe_layer_done(eng, layer);
}

extern "C" int moe_last_routing(moe_engine *eng, const int **idx, const float **w, const int **sorted_pair) {
  if (!eng || !eng->fw) { moe_set_error("moe_last_routing: no forward workspace"); return MOE_ESTATE; }
  if (idx) *idx = eng->fw->idx;
  if (w) *w = eng->fw->topk_w;
  if (sorted_pair) *sorted_pair = eng->fw->sorted_pair;
  return MOE_OK;
}

extern "C" int moe_last_routing_host(moe_engine *eng, int T, int k, int *idx_host, float *w_host) {
  if (!eng || !eng->fw) { moe_set_error("moe_last_routing_host: no forward workspace"); return MOE_ESTATE; }
  LayerState *s = eng->fw;
  if (T <= 0 || k <= 0 || T > s->max_tokens || k > s->max_k) { moe_set_error("moe_last_routing_host: T=%d k=%d outside the workspace", T, k); return MOE_EINVAL; }
  HIPC(hipStreamSynchronize((hipStream_t)eng->be->compute_stream()));
  const size_t n = (size_t)T * k;
  if (idx_host) HIPC(hipMemcpy(idx_host, s->idx, n * sizeof(int), hipMemcpyDeviceToHost));
  if (w_host) HIPC(hipMemcpy(w_host, s->topk_w, n * sizeof(float), hipMemcpyDeviceToHost));
  return MOE_OK;
}
