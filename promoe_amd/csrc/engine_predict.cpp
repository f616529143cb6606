// Built-in prefetch predictor: one linear model per (source layer -> destination layer) pair,
// evaluated on the GPU on the hidden state a layer hook reports, ranked on a host thread, turned
// into prefetch requests for the destination layers.
//
// The reference runs per-pair TorchScript models on the CPU (SepPredictor, predictor.cpp:496-607,
// model files "<src>-<dst>.pt", predictor.cpp:610-636) from a PredictWorker thread that updates the
// NN policy's priorities, ranks the top n experts per destination layer, takes one unit of the
// run-ahead budget per layer, queues a PrefetchLayerTask and posts the layer's progress
// (worker.cpp:6-77).  The layer windows are those of build_predict_layer_mapping
// (predictor.cpp:8-46).  Here the model of a pair is a matrix [E, H] (+ optional bias [E]): the
// scores are x . W^T + b, computed by the gate-logits kernel on the compute stream right behind the
// layer input; the host thread sees them through pinned memory and an event.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <deque>
#include <map>
#include <numeric>
#include <thread>

#include "engine_internal.h"
#include "moe_kernels.h"

struct PredictModel { const void *w = nullptr; const float *bias = nullptr; };
struct PredictJob {
  int src = 0; int seq_len = 0;
  // scores written by a launch the caller queued itself: they are complete once *seq_word has reached seq_value
  // (a later kernel of the stream stores it when it starts); no event
  const volatile int *seq_word = nullptr; int seq_value = 0;
};

struct PredictorState {
  std::vector<std::pair<int, int>> window;          // [L + 1]: destination layers [first, second) of source l
  std::map<std::pair<int, int>, PredictModel> models;
  int max_win = 0, H = 0;
  // [L + 1][max_win][E].  Device backend: pinned host memory; the score kernel stores into it through
  // scores_dev, its device-side address (no copy in the stream), the thread reads it after the event
  float *scores_dev = nullptr, *scores_host = nullptr;
  // device backend: the models of one source layer stacked into one [n_dst * E, H] matrix (and bias
  // vector, if any of them has one), so that a report costs one launch whatever the window
  std::vector<void *> stack_w;
  std::vector<float *> stack_b;
  std::vector<void *> events;                            // one per source layer
  std::thread th;
  std::mutex mu;
  std::condition_variable cv, cv_idle;
  bool busy = false;                                     // a job is being processed
  std::deque<PredictJob> q;
  bool exit = false, started = false, host_math = false;
  uint64_t n_jobs = 0, n_requests = 0;
  std::string error;                                     // first failure on the thread
  // How good the requests for each destination layer have been (optional; off = every request goes out as
  // ranked, which is what the reference does): of the experts a request would have to copy (ranked, not resident),
  // the share that the layer then routed to, as a moving average per destination layer.  A request for a layer whose average is below min_precision goes
  // out empty (the layer's progress count stays in step, nothing is copied): a wrong prefetch costs a copy on the
  // host link and evicts an expert that may be needed, so below about one half it loses more than it hides.
  float min_precision = 0.f;
  std::vector<float> precision;                          // [L], starts at 1
  std::vector<std::vector<int64_t>> last_pred;           // [L]: the ranking made for the layer's next turn
  uint64_t n_withheld = 0;
};

// predictor.cpp:8-46
static std::vector<std::pair<int, int>> layer_windows(const moe_cfg &c) {
  const int L = c.num_layer;
  std::vector<int> pl(L + 1, 0);
  int stop = 0;
  for (int l = 0; l < L; l += std::max(1, c.layer_predict_interval)) {
    int window = c.layer_predict_max_window;
    if (l == 0 && c.limit_layer_0_window != -1) window = c.limit_layer_0_window;
    pl[l] = stop;
    pl[l + 1] = std::min(l % L + window, L);
    stop = pl[l + 1];
  }
  for (int l = 1; l <= L; ++l) pl[l] = std::max(pl[l], pl[l - 1]);
  std::vector<std::pair<int, int>> ret(L + 1, {0, 0});
  for (int l = 0; l < L; ++l) ret[l] = {pl[l], pl[l + 1]};
  if (c.cross_token_pred) { ret[L] = ret[0]; ret[0] = {0, 0}; }
  return ret;
}

static PredictorState *state_of(moe_engine *eng) {
  if (!eng->pred) {
    auto *p = new PredictorState();
    p->window = layer_windows(eng->cfg);
    for (auto &w : p->window) p->max_win = std::max(p->max_win, w.second - w.first);
    p->precision.assign(eng->cfg.num_layer, 1.f);
    p->last_pred.assign(eng->cfg.num_layer, {});
    eng->pred = p;
  }
  return eng->pred;
}

extern "C" int moe_predictor_windows(moe_engine *eng, int *first, int *last) {
  if (!eng || !first || !last) { moe_set_error("moe_predictor_windows: null argument"); return MOE_EINVAL; }
  PredictorState *p = state_of(eng);
  for (size_t l = 0; l < p->window.size(); ++l) { first[l] = p->window[l].first; last[l] = p->window[l].second; }
  return MOE_OK;
}

extern "C" int moe_predictor_set_model(moe_engine *eng, int src, int dst, const void *w, const float *bias, int H) {
  if (!eng || !w || H <= 0 || H % 8) { moe_set_error("moe_predictor_set_model: bad argument"); return MOE_EINVAL; }
  PredictorState *p = state_of(eng);
  if (p->started) { moe_set_error("moe_predictor_set_model: the predictor is running"); return MOE_ESTATE; }
  if (src < 0 || src > eng->cfg.num_layer || dst < p->window[src].first || dst >= p->window[src].second) {
    moe_set_error("moe_predictor_set_model: layer %d does not predict layer %d (its window is [%d, %d))", src, dst,
                  src >= 0 && src <= eng->cfg.num_layer ? p->window[src].first : 0,
                  src >= 0 && src <= eng->cfg.num_layer ? p->window[src].second : 0);
    return MOE_EINVAL;
  }
  if (p->H && p->H != H) { moe_set_error("moe_predictor_set_model: models disagree in H (%d, %d)", p->H, H); return MOE_EINVAL; }
  p->H = H;
  p->models[{src, dst}] = PredictModel{w, bias};
  return MOE_OK;
}

// scores of the host backend (cache tests without a device): the kernel's sum in plain loops
static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static void host_scores(const uint16_t *x, const uint16_t *w, const float *bias, float *out, int H, int E) {
  for (int e = 0; e < E; ++e) {
    float acc = 0.f;
    for (int k = 0; k < H; ++k) acc += bf16_to_f32(x[k]) * bf16_to_f32(w[(size_t)e * H + k]);
    out[e] = bias ? acc + bias[e] : acc;
  }
}

static void predictor_fail(moe_engine *eng, PredictorState *p, const char *what) {
  std::lock_guard<std::mutex> lk(p->mu);
  if (p->error.empty()) p->error = std::string(what) + ": " + moe_last_error();
  (void)eng;
}

static void predictor_loop(moe_engine *eng, PredictorState *p) {
  const int E = eng->cfg.num_expert;
  std::vector<int64_t> ids;
  std::vector<int> order(E);
  std::vector<float> prob(E);
  for (;;) {
    PredictJob job;
    {
      std::unique_lock<std::mutex> lk(p->mu);
      p->cv.wait(lk, [&] { return p->exit || !p->q.empty(); });
      if (p->exit) return;
      job = p->q.front();
      p->q.pop_front();
      p->busy = true;
    }
    const auto win = p->window[job.src];
    bool decode = job.seq_len == 1;
    if (decode && job.seq_word) {
      const auto t0 = std::chrono::steady_clock::now();
      unsigned spins = 0;
      while (*job.seq_word - job.seq_value < 0) {
        if ((++spins & 255u) == 0) {
          if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) {  // not within 2 ms: the stream itself
            if (hipStreamSynchronize((hipStream_t)eng->be->compute_stream()) != hipSuccess) { predictor_fail(eng, p, "stream"); decode = false; }
            break;
          }
          std::lock_guard<std::mutex> lk(p->mu);
          if (p->exit) return;
        }
      }
      __atomic_thread_fence(__ATOMIC_ACQUIRE);
    } else if (decode && !p->host_math && eng->be->event_sync(p->events[job.src]) != 0) { predictor_fail(eng, p, "event"); decode = false; }
    for (int dst = win.first; dst < win.second; ++dst) {
      int64_t n = 0;
      if (decode) {  // prefill: an empty request per layer keeps the progress count in step (predictor.cpp:513-517)
        const float *s = p->scores_host + ((size_t)job.src * p->max_win + (dst - win.first)) * E;
        if (eng->cfg.cache_policy == "nn") {  // worker.cpp:19-21: the policy ranks by predicted probability
          float mx = s[0];
          for (int e = 1; e < E; ++e) mx = std::max(mx, s[e]);
          float den = 0.f;
          for (int e = 0; e < E; ++e) { prob[e] = std::exp(s[e] - mx); den += prob[e]; }
          for (int e = 0; e < E; ++e) prob[e] /= den;
          if (moe_update_priority(eng, prob.data(), 1, dst) != MOE_OK) predictor_fail(eng, p, "update_priority");
        }
        std::iota(order.begin(), order.end(), 0);
        n = std::min<int64_t>(std::max(eng->cfg.num_predict_expert_per_layer, 0), E);
        std::partial_sort(order.begin(), order.begin() + n, order.end(),
                          [&](int a, int b) { return s[a] > s[b] || (s[a] == s[b] && a < b); });
        ids.assign(order.begin(), order.begin() + n);
        // what this request would copy: the ranked experts that are not resident now.  They are what a wrong
        // prediction costs (the resident ones cost nothing either way), so they are what the layer's routing is
        // scored against - the ranking as a whole looks good whenever the popular experts are resident.
        std::vector<int64_t> would_copy;
        {
          SpinGuard lk(eng->mu);
          for (int64_t e : ids)
            if (!eng->resident.count(eng->ex(dst, (int)e))) would_copy.push_back(e);
        }
        std::lock_guard<std::mutex> lk(p->mu);
        p->last_pred[dst] = would_copy;              // scored when the layer reports its routing
        if (p->min_precision > 0.f && p->precision[dst] < p->min_precision && !would_copy.empty()) { n = 0; p->n_withheld++; }
      }
      {  // a copy of this layer still in flight is a leftover of the layer's previous turn and normally over
         // in a moment: give it that moment, so that the new tasks do not queue behind it for nothing
        std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
        const auto t0 = std::chrono::steady_clock::now();
        while (!eng->exiting && eng->current.e && eng->current.e->layer == dst &&
               std::chrono::steady_clock::now() - t0 < std::chrono::microseconds(500))
          eng->cv_state.wait_for(lk, std::chrono::microseconds(50));
      }
      // ... but not for ever: the copy may be waiting for the slot-group guard of the very forward that waits
      // for this request
      const int rc = moe_prefetch_layer_over(eng, dst, ids.data(), n, 1, true);
      if (rc == MOE_ESTATE && eng->exiting) return;
      if (rc != MOE_OK) {  // keep the layer's progress in step so that report_one_layer does not wait for ever
        predictor_fail(eng, p, "prefetch_layer");
        SpinGuard lk(eng->mu);
        eng->progress++;
        eng->cv_sem.notify_all();
      }
      std::lock_guard<std::mutex> lk(p->mu);
      p->n_requests++;
    }
    std::lock_guard<std::mutex> lk(p->mu);
    p->n_jobs++;
    p->busy = false;
    p->cv_idle.notify_all();
  }
}

extern "C" int moe_predictor_start(moe_engine *eng) {
  if (!eng) { moe_set_error("moe_predictor_start: null"); return MOE_EINVAL; }
  PredictorState *p = state_of(eng);
  if (p->started) return MOE_OK;
  if (!eng->launched) { moe_set_error("moe_predictor_start: engine not launched"); return MOE_ESTATE; }
  const int L = eng->cfg.num_layer, E = eng->cfg.num_expert;
  for (int src = 0; src <= L; ++src)
    for (int dst = p->window[src].first; dst < p->window[src].second; ++dst)
      if (!p->models.count({src, dst})) { moe_set_error("moe_predictor_start: no model for %d -> %d", src, dst); return MOE_ESTATE; }
  // every layer must be predicted by exactly one source, or report_one_layer would wait for a request that never comes
  std::vector<int> cover(L, 0);
  for (int src = 0; src <= L; ++src)
    for (int dst = p->window[src].first; dst < p->window[src].second; ++dst) cover[dst]++;
  for (int l = 0; l < L; ++l)
    if (cover[l] != 1) { moe_set_error("moe_predictor_start: layer %d is predicted %d times", l, cover[l]); return MOE_ESTATE; }
  p->host_math = eng->be->compute_stream() == nullptr && eng->be->copy_stream() == nullptr;
  const size_t n = (size_t)(L + 1) * std::max(p->max_win, 1) * E;
  if (p->host_math) {
    p->scores_host = new float[n]();
  } else {
    if (moe_check_hip(hipHostMalloc((void **)&p->scores_host, n * sizeof(float), hipHostMallocDefault), "hipHostMalloc(predictor scores)"))
      return MOE_EHIP;
    if (moe_check_hip(hipHostGetDevicePointer((void **)&p->scores_dev, p->scores_host, 0), "hipHostGetDevicePointer(predictor scores)"))
      return MOE_EHIP;
    for (int l = 0; l <= L; ++l) p->events.push_back(eng->be->event_create());
    p->stack_w.assign(L + 1, nullptr);
    p->stack_b.assign(L + 1, nullptr);
    const size_t wb = (size_t)E * p->H * 2;
    for (int src = 0; src <= L; ++src) {
      const auto win = p->window[src];
      const int nd = win.second - win.first;
      if (nd <= 0) continue;
      bool any_bias = false;
      for (int dst = win.first; dst < win.second; ++dst) any_bias |= p->models[{src, dst}].bias != nullptr;
      if (moe_check_hip(hipMalloc(&p->stack_w[src], wb * nd), "hipMalloc(predictor models)")) return MOE_EHIP;
      if (any_bias) {
        if (moe_check_hip(hipMalloc((void **)&p->stack_b[src], (size_t)nd * E * sizeof(float)), "hipMalloc(predictor bias)")) return MOE_EHIP;
        if (moe_check_hip(hipMemset(p->stack_b[src], 0, (size_t)nd * E * sizeof(float)), "hipMemset(predictor bias)")) return MOE_EHIP;
      }
      for (int dst = win.first; dst < win.second; ++dst) {
        const PredictModel &m = p->models[{src, dst}];
        const size_t i = (size_t)(dst - win.first);
        if (moe_check_hip(hipMemcpy((char *)p->stack_w[src] + i * wb, m.w, wb, hipMemcpyDeviceToDevice), "hipMemcpy(predictor model)"))
          return MOE_EHIP;
        if (m.bias && moe_check_hip(hipMemcpy(p->stack_b[src] + i * E, m.bias, (size_t)E * sizeof(float), hipMemcpyDeviceToDevice),
                                    "hipMemcpy(predictor bias)"))
          return MOE_EHIP;
      }
    }
  }
  p->started = true;
  p->th = std::thread(predictor_loop, eng, p);
  SpinGuard lk(eng->mu);
  eng->predictor_attached = true;
  return MOE_OK;
}

// called by moe_report_layer_logits: hidden [B*S, H] bf16 of layer `layer` (device memory; host memory on the host backend)
int moe_predictor_on_logits(moe_engine *eng, int layer, const void *hidden, int B, int S, int H) {
  PredictorState *p = eng->pred;
  if (!p || !p->started) return MOE_OK;
  const auto win = p->window[layer];
  if (win.first >= win.second) return MOE_OK;  // this layer predicts nothing
  const bool decode = S == 1 && B == 1;
  if (decode) {
    if (!hidden || H != p->H) { moe_set_error("predictor: layer %d reported a hidden state of width %d, the models take %d", layer, H, p->H); return MOE_EINVAL; }
    const int E = eng->cfg.num_expert;
    if (p->host_math) {
      for (int dst = win.first; dst < win.second; ++dst) {
        const PredictModel &m = p->models[{layer, dst}];
        const size_t off = ((size_t)layer * p->max_win + (dst - win.first)) * E;
        host_scores((const uint16_t *)hidden, (const uint16_t *)m.w, m.bias, p->scores_host + off, H, E);
      }
    } else {
      // one launch for the whole window: the stacked models' rows are the window's (dst, expert) pairs in order
      const size_t off = (size_t)layer * p->max_win * E;
      const int rows = (win.second - win.first) * E;
      if (int rc = moe_gate_logits(hidden, p->stack_w[layer], p->stack_b[layer], p->scores_dev + off, 1, H, rows, rows,
                                   eng->be->compute_stream()))
        return rc;
      if (eng->be->event_record(p->events[layer], eng->be->compute_stream()) != 0) return MOE_EHIP;
    }
  }
  {
    std::lock_guard<std::mutex> lk(p->mu);
    if (!p->error.empty()) { moe_set_error("predictor thread: %s", p->error.c_str()); return MOE_ESTATE; }
    p->q.push_back(PredictJob{layer, decode ? 1 : std::max(S, 2)});
  }
  p->cv.notify_all();
  return MOE_OK;
}

// A one-token forward that launches the gate-logits kernel itself can take the window's score rows into that
// launch (moe_gate_logits_pair): this hands out the stacked models of `layer` and where their scores go.  False:
// nothing to fuse (no predictor, the host backend, an empty window, another hidden width).
bool moe_predictor_fused_rows(moe_engine *eng, int layer, int H, const void **w, const float **bias, float **out, int *rows) {
  PredictorState *p = eng->pred;
  if (!p || !p->started || p->host_math || layer < 0 || layer >= (int)p->window.size()) return false;
  const auto win = p->window[layer];
  if (win.first >= win.second || H != p->H || !p->stack_w[layer]) return false;
  const int E = eng->cfg.num_expert;
  *w = p->stack_w[layer];
  *bias = p->stack_b[layer];
  *out = p->scores_dev + (size_t)layer * p->max_win * E;
  *rows = (win.second - win.first) * E;
  return true;
}

// ... and this queues the job: the scores are complete once *seq_word has reached seq_value, which a later kernel
// of the same stream stores into pinned memory when it starts.  The thread polls that word instead of waiting for
// an event, which would cost the stream a few microseconds per step.
int moe_predictor_scores_pending(moe_engine *eng, int layer, const int *seq_word, int seq_value) {
  PredictorState *p = eng->pred;
  if (!p || !p->started) return MOE_OK;
  {
    std::lock_guard<std::mutex> lk(p->mu);
    if (!p->error.empty()) { moe_set_error("predictor thread: %s", p->error.c_str()); return MOE_ESTATE; }
    PredictJob j; j.src = layer; j.seq_len = 1; j.seq_word = seq_word; j.seq_value = seq_value;
    p->q.push_back(j);
  }
  p->cv.notify_all();
  return MOE_OK;
}

void moe_predictor_observe(moe_engine *eng, int layer, const int64_t *ids, int64_t n) {
  PredictorState *p = eng->pred;
  if (!p || !p->started || layer < 0 || layer >= (int)p->last_pred.size()) return;
  std::lock_guard<std::mutex> lk(p->mu);
  std::vector<int64_t> &pred = p->last_pred[layer];
  if (pred.empty()) return;
  int hit = 0;
  for (int64_t e : pred)
    for (int64_t i = 0; i < n; ++i)
      if (ids[i] == e) { ++hit; break; }
  p->precision[layer] = 0.8f * p->precision[layer] + 0.2f * (float)hit / (float)pred.size();
  pred.clear();
}

extern "C" int moe_predictor_set_min_precision(moe_engine *eng, float min_precision) {
  if (!eng || !(min_precision >= 0.f && min_precision <= 1.f)) { moe_set_error("moe_predictor_set_min_precision: bad argument"); return MOE_EINVAL; }
  PredictorState *p = state_of(eng);
  std::lock_guard<std::mutex> lk(p->mu);
  p->min_precision = min_precision;
  return MOE_OK;
}

extern "C" int moe_predictor_precision(moe_engine *eng, float *precision, uint64_t *n_withheld) {
  if (!eng || !eng->pred) { moe_set_error("moe_predictor_precision: no predictor"); return MOE_ESTATE; }
  PredictorState *p = eng->pred;
  std::lock_guard<std::mutex> lk(p->mu);
  if (precision) for (size_t l = 0; l < p->precision.size(); ++l) precision[l] = p->precision[l];
  if (n_withheld) *n_withheld = p->n_withheld;
  return MOE_OK;
}

extern "C" int moe_predictor_wait_idle(moe_engine *eng, int timeout_ms) {
  if (!eng || !eng->pred) { moe_set_error("moe_predictor_wait_idle: no predictor"); return MOE_ESTATE; }
  PredictorState *p = eng->pred;
  std::unique_lock<std::mutex> lk(p->mu);
  const bool idle = p->cv_idle.wait_for(lk, std::chrono::milliseconds(timeout_ms < 0 ? 0 : timeout_ms),
                                        [&] { return p->exit || (p->q.empty() && !p->busy); });
  return idle ? MOE_OK : 1;
}

extern "C" int moe_predictor_stats(moe_engine *eng, uint64_t *n_jobs, uint64_t *n_requests) {
  if (!eng || !eng->pred) { moe_set_error("moe_predictor_stats: no predictor"); return MOE_ESTATE; }
  std::lock_guard<std::mutex> lk(eng->pred->mu);
  if (n_jobs) *n_jobs = eng->pred->n_jobs;
  if (n_requests) *n_requests = eng->pred->n_requests;
  return MOE_OK;
}

void moe_predictor_free(moe_engine *eng) {
  PredictorState *p = eng->pred;
  if (!p) return;
  {
    std::lock_guard<std::mutex> lk(p->mu);
    p->exit = true;
  }
  p->cv.notify_all();
  if (p->th.joinable()) p->th.join();
  if (p->host_math) delete[] p->scores_host;
  else {
    for (void *w : p->stack_w) if (w) (void)hipFree(w);
    for (float *b : p->stack_b) if (b) (void)hipFree(b);
    if (p->scores_host) (void)hipHostFree(p->scores_host);
  }
  delete p;
  eng->pred = nullptr;
}
