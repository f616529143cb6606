// Internal types of the expert-cache engine.
#pragma once
#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <functional>
#include <list>
#include <map>
#include <memory>
#include <cstdlib>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "moe_common.h"
#include "moe_engine.h"

std::string moe_translate_key(const std::string &key);

struct moe_cfg {
  int num_layer = 0, num_expert = 0, num_expert_per_token = 0;
  std::string model_arch_string;
  float cache_rate = 0.5f;
  int num_predict_expert_per_layer = -1;
  bool reorder_experts = false, early_preempt = false, chunk_prefetch = false;
  std::string predict_input_mode_str = "moe_layer_logits";
  int predict_input_mode = 7;
  std::string predictor_type_str = "sep";
  std::string predictor_model_path;
  int layer_predict_interval = 1, layer_predict_max_window = 3;
  bool cross_token_pred = false;
  int limit_layer_0_window = -1, limit_layer_0_num_predict = -1;
  int max_prefetch_layer_distance = -1;
  bool cache_only = false, per_layer_cache = true, promote_hit_in_prefetch = true;
  std::string cache_policy = "lru";
  int predict_input_reuse_distance_max = 10, predict_input_decay = 2;
  // non-config
  int num_per_expert_param = 0;
  std::vector<std::string> param_names;
  // env
  unsigned sleep_on_report_logits_us = 0;
  float expert_mem_scale = 1.0f;
  int num_dummy_params = 0;
  std::string physical_mem_impl = "vmm";  // the reference's default is tensor_global_unified (a slab)
  std::string logical_mem_impl = "table";
  bool pool_vmm = true;

  std::map<std::string, std::string> staged;
  bool finalized = false;
};

enum ExpertStatus { kIdle = 0, kFetching = 1, kReady = 2, kLaunching = 3, kUsing = 4 };

struct HostChunk {
  const void *ptr = nullptr;
  size_t nbytes = 0, alloc = 0;
};

struct Expert {
  int layer = 0, idx = 0;
  std::vector<HostChunk> chunks;
  int slot = -1;      // index into moe_engine::slots, -1 = none
  int num_ready = 0;  // chunks already copied
  std::atomic<int> status{kIdle};
  void *event = nullptr;      // (not owned) event recorded after the last launch that reads the slot
  void *own_event = nullptr;  // per-expert event of the stepwise API (prefetcher.cpp:263)
  // alternative to `event`: the launches that read the slot are over once *seq_ptr has reached seq_need
  // (a word a LATER kernel of the same stream stores into host memory when it starts)
  const volatile int *seq_ptr = nullptr;
  int seq_need = 0;
  bool seq_reached() const { return !seq_ptr || (int)((unsigned)*seq_ptr - (unsigned)seq_need) >= 0; }
  size_t total_alloc() const { size_t t = 0; for (auto &c : chunks) t += c.alloc; return t; }
};

// ---- eviction policies (cache.hpp:6-224, cache.cpp:313-583) ----
struct Policy {
  virtual ~Policy() {}
  virtual Expert *select_for_evict() = 0;
  virtual int evict(Expert *) = 0;
  virtual int on_hit(Expert *, bool precise) = 0;
  virtual int on_miss(Expert *, bool precise) = 0;
  virtual void update_all_priority() {}
  virtual void update_priority(Expert *, float) {}
  virtual int set_cur_seq(uint64_t) { return 0; }
  virtual std::string to_string() { return ""; }
};

// binary min-heap with the reference's exact sift rules (utils.hpp:273-361)
struct MinHeap {
  struct Node { float priority; int idx; Expert *e; };
  std::vector<Node *> buf;
  void swap_(int i, int j) { std::swap(buf[i], buf[j]); buf[i]->idx = i; buf[j]->idx = j; }
  void down(int i) {
    for (;;) {
      int l = 2 * i + 1, r = 2 * i + 2, s = i;
      if (l < (int)buf.size() && buf[l]->priority < buf[s]->priority) s = l;
      if (r < (int)buf.size() && buf[r]->priority < buf[s]->priority) s = r;
      if (s == i) return;
      swap_(i, s);
      i = s;
    }
  }
  void up(int i) {
    while (i > 0) {
      int p = (i - 1) / 2;
      if (buf[p]->priority > buf[i]->priority) { swap_(p, i); i = p; } else break;
    }
  }
  void push(Node *n) { n->idx = (int)buf.size(); buf.push_back(n); up(n->idx); }
  void update(Node *n, float p) {
    float o = n->priority;
    n->priority = p;
    if (p < o) up(n->idx); else down(n->idx);
  }
  void remove(Node *n) {
    int i = n->idx;
    swap_(i, (int)buf.size() - 1);
    buf.pop_back();
    if (i < (int)buf.size()) down(i);
  }
  void rebuild() { for (int i = (int)buf.size() / 2; i >= 0; --i) if (i < (int)buf.size()) down(i); }
  Node *front() { return buf.empty() ? nullptr : buf[0]; }
};

struct SeqOracle { std::unordered_map<Expert *, std::vector<int64_t>> use_times; };

struct Group {
  std::unique_ptr<Policy> policy;
  std::vector<int> unused;  // free slot indices; taken from the back
  size_t full_len = 0;
  // > 0 while a kernel runs on a snapshot of the slot table whose selection the host does not know yet:
  // evictions go on, but no copy into a slot of this group starts (fetch thread waits)
  int guard = 0;
};

// The engine's mutex is held for a microsecond or so at a time, by three threads (the caller's, the fetch thread, the
// predictor's).  A thread that finds it taken and sleeps on it pays the kernel's wake-up, 5 us and more, and leaves
// the mutex in its contended state, where every unlock is a system call.  So everybody tries for a while before
// sleeping.  MOE_LOCK_SPINS=0: sleep at once.
static inline int moe_lock_spins() {
  static const int n = [] { const char *e = getenv("MOE_LOCK_SPINS"); return e ? atoi(e) : 2000; }();
  return n;
}
static inline void moe_spin_lock(std::mutex &m) {
  for (int i = 0, n = moe_lock_spins(); i < n; ++i) {
    if (m.try_lock()) return;
#if defined(__x86_64__)
    __builtin_ia32_pause();
#endif
  }
  m.lock();
}
static inline void moe_spin_lock(std::unique_lock<std::mutex> &lk) {
  for (int i = 0, n = moe_lock_spins(); i < n; ++i) {
    if (lk.try_lock()) return;
#if defined(__x86_64__)
    __builtin_ia32_pause();
#endif
  }
  lk.lock();
}
struct SpinGuard {
  std::mutex &m;
  explicit SpinGuard(std::mutex &mu) : m(mu) { moe_spin_lock(m); }
  ~SpinGuard() { m.unlock(); }
  SpinGuard(const SpinGuard &) = delete;
  SpinGuard &operator=(const SpinGuard &) = delete;
};

struct CopyTask {
  int start = 0, stop = 0;
  bool precise = false;
  Expert *e = nullptr;
  Expert *wait_victim = nullptr;  // slot's previous owner still in flight on the compute stream
};

// ---- device backend ----
struct Backend {
  virtual ~Backend() {}
  virtual int alloc_pool(size_t slot_bytes, size_t n_slots, size_t reserve_slots, bool vmm,
                         void **base, size_t *stride) = 0;
  virtual int alloc_table(size_t n_entries, uint64_t **dev, uint64_t **host_mirror) = 0;
  virtual int copy_h2d(void *dst, const void *src, size_t n) = 0;  // queued on the copy stream
  virtual int copy_sync() = 0;
  virtual int flush_table(uint64_t *dev, const uint64_t *host, size_t n, void *stream) = 0;
  virtual void *event_create() = 0;
  virtual int event_record(void *ev, void *stream) = 0;
  virtual int event_sync(void *ev) = 0;
  virtual bool event_done(void *ev) = 0;
  virtual void *compute_stream() = 0;
  virtual void *copy_stream() = 0;
  virtual bool is_pinned(const void *p) = 0;
};
Backend *moe_make_hip_backend(void *compute_stream, bool cache_only);
Backend *moe_make_host_backend();

struct Series { std::vector<uint64_t> v; };

struct LayerState;  // forward workspace, engine_forward.cpp
struct PredictorState;  // built-in predictor, engine_predict.cpp

struct moe_engine {
  moe_cfg cfg;
  std::unique_ptr<Backend> be;
  std::vector<std::unique_ptr<Expert>> experts;  // [L*E]
  Expert *ex(int l, int e) { return experts[(size_t)l * cfg.num_expert + e].get(); }

  // slot pool
  void *pool_base = nullptr;
  size_t slot_bytes = 0, slot_stride = 0, n_slots = 0;
  std::vector<size_t> chunk_off;  // offset of each parameter chunk inside a slot
  std::vector<Group> groups;
  Group &group_of(int layer) { return groups[cfg.per_layer_cache ? layer : 0]; }
  std::unordered_map<Expert *, int> resident;  // expert -> slot (includes the copy in flight)
  uint64_t *d_table = nullptr, *h_table = nullptr;
  std::vector<char> table_dirty;  // per layer
  std::vector<void *> dummy_bufs;
  std::vector<void *> layer_event;  // one per layer, used by moe_release_layer
  void *proof_event = nullptr;      // recorded by the fetch thread when a sequence word does not come
  std::vector<int> layer_complete;  // fully fetched resident experts per layer

  // NN / MIN policy state (cache.hpp:262-266)
  std::vector<float> priority;  // [L*E]
  float max_priority = 1.17549435e-38f;
  std::unordered_map<uint64_t, SeqOracle> oracles;

  // scheduler
  std::mutex mu;
  std::condition_variable cv_work, cv_state;
  std::deque<CopyTask> precise_q;
  std::vector<std::deque<CopyTask>> layer_q;
  CopyTask current;  // the one copy in flight (current.e == nullptr: none)
  std::atomic<unsigned> task_epoch{0};  // bumped with every queued task
  std::atomic<int> seq_pollers{0};      // fetch thread inside its unlocked poll of a sequence word
  std::thread fetch_thread;
  bool launched = false, exiting = false, slots_ready = false;
  std::string fatal;  // first broken invariant (the reference would have aborted)

  // prefetch run-ahead budget / progress (worker.hpp:294,308-314)
  long budget = 0, progress = 0;
  bool predictor_attached = false;
  std::condition_variable cv_sem;

  // counters
  moe_counters ctr{};
  moe_counters fwd_base{};  // value at the start of the current forward
  std::vector<uint64_t> s_hit, s_miss, s_ready, s_unready, s_phit, s_pmiss, s_act, s_wait, s_seqlen;

  // fused forward
  std::vector<moe_layer_desc> layer_desc;
  LayerState *fw = nullptr;
  PredictorState *pred = nullptr;

  ~moe_engine();
};

int engine_fail(moe_engine *eng, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void moe_forward_free(LayerState *);
void moe_predictor_free(moe_engine *eng);
int moe_predictor_on_logits(moe_engine *eng, int layer, const void *hidden, int B, int S, int H);
bool moe_predictor_fused_rows(moe_engine *eng, int layer, int H, const void **w, const float **bias, float **out, int *rows);
int moe_predictor_scores_pending(moe_engine *eng, int layer, const int *seq_word, int seq_value);
// the routing of a decode step at `layer` (before the hooks reorder it): what the layer's last prediction is scored against
void moe_predictor_observe(moe_engine *eng, int layer, const int64_t *ids, int64_t n);
// moe_report_layer_logits without the predictor's part (the caller runs that part itself)
int moe_report_layer_logits_bookkeeping(moe_engine *eng, int layer, int S);
// launching -> using without an event: the experts count as in use until *seq_ptr reaches seq_need
// slot table of `layer` to the device (if changed) and the same residency as a byte vector, taken in one
// critical section together with raising the group's guard; moe_guard_release lowers it again
int moe_flush_table_guarded(moe_engine *eng, int layer, void *stream, char *resident_out);
int moe_snapshot_table_guarded(moe_engine *eng, int layer, uint64_t *table_out, char *resident_out);
void moe_guard_release(moe_engine *eng, int layer);
int moe_prefetch_layer_over(moe_engine *eng, int layer, const int64_t *ids, int64_t n, int blocking, bool over_copy);
// every expert that waits for a sequence word becomes ready (the caller has drained the compute stream)
void engine_drop_seq_releases(moe_engine *eng);
// fails the engine when a kernel raised a strict error word of the forward workspace
int moe_forward_check_kernels(moe_engine *eng);
int moe_release_experts_seq(moe_engine *eng, int layer, const int64_t *ids, int64_t n, const volatile int *seq_ptr, int seq_need);
// account demand hits of experts that were launched without a host round trip
int engine_account_hits(moe_engine *eng, int layer, const moe_unit *units, int n);
// collect the routing results of earlier moe_forward calls (wait: block until all are in)
int moe_forward_harvest(moe_engine *eng, bool wait);
