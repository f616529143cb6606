// Expert-cache engine: registry, slot pool, eviction policies, fetch scheduling.
//
// Structure (differs from the reference on purpose): the reference confines cache
// state to a spinning scheduler thread and hands it tasks from the caller
// (prefetcher.hpp:64-97, worker.hpp:113-142).  Here the same task handlers run
// inline in the calling thread under one mutex, and a single blocking fetch thread
// owns the copy engine: it pops the next copy task (demand queue first, then the
// speculative queues by ascending layer, prefetcher.cpp:143-161), assigns/evicts a
// slot, copies one task's chunks on the side stream, and posts completion.
// There is no unlocker thread: `using -> ready` is resolved lazily from the
// expert's event whenever a victim or a hit needs it.
#include <stdarg.h>
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <queue>
#include <set>

#include "engine_internal.h"

int engine_fail(moe_engine *eng, const char *fmt, ...) {
  char buf[400];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  if (eng && eng->fatal.empty()) eng->fatal = buf;
  moe_set_error("%s", buf);
  return MOE_ESTATE;
}

#define ENG_CHECK(eng, cond, ...) \
  do { if (!(cond)) return engine_fail((eng), __VA_ARGS__); } while (0)

// ---------------------------------------------------------------------------
// policies
// ---------------------------------------------------------------------------
namespace {

struct PolicyFIFO : Policy {  // cache.cpp:313-321
  moe_engine *eng;
  std::deque<Expert *> q;
  explicit PolicyFIFO(moe_engine *e) : eng(e) {}
  Expert *select_for_evict() override { return q.empty() ? nullptr : q.front(); }
  int evict(Expert *e) override {
    ENG_CHECK(eng, !q.empty() && q.front() == e, "fifo: evict of a non-front expert");
    q.pop_front();
    return 0;
  }
  int on_hit(Expert *, bool) override { return 0; }
  int on_miss(Expert *e, bool) override { q.push_back(e); return 0; }
};

struct PolicyLRU : Policy {  // cache.hpp:32-57, cache.cpp:322-339
  moe_engine *eng;
  std::list<Expert *> ll;
  std::unordered_map<Expert *, std::list<Expert *>::iterator> map;
  explicit PolicyLRU(moe_engine *e) : eng(e) {}
  Expert *select_for_evict() override { return ll.empty() ? nullptr : ll.front(); }
  int evict(Expert *e) override {
    auto it = map.find(e);
    ENG_CHECK(eng, it != map.end(), "lru: evict of an unknown expert");
    ll.erase(it->second);
    map.erase(it);
    return 0;
  }
  int on_hit(Expert *e, bool) override {
    auto it = map.find(e);
    ENG_CHECK(eng, it != map.end(), "lru: hit on an expert that is not tracked");
    ll.splice(ll.end(), ll, it->second);
    return 0;
  }
  int on_miss(Expert *e, bool) override {
    ENG_CHECK(eng, !map.count(e), "lru: miss on an expert that is already tracked");
    ll.push_back(e);
    map[e] = std::prev(ll.end());
    return 0;
  }
  std::string to_string() override {
    std::string s;
    for (auto *e : ll) s += std::to_string(e->idx) + ",";
    return s;
  }
};

struct PolicyStatic : Policy {  // cache.hpp:58-80, cache.cpp:340-381
  moe_engine *eng;
  size_t max_alt;
  std::list<Expert *> ll;
  std::unordered_map<Expert *, std::list<Expert *>::iterator> map;
  std::unordered_set<Expert *> persisted;
  PolicyStatic(moe_engine *e, int n) : eng(e), max_alt(n) {}
  Expert *select_for_evict() override { return ll.empty() ? nullptr : ll.front(); }
  int on_hit(Expert *e, bool) override {
    ENG_CHECK(eng, map.count(e) || persisted.count(e), "static: hit on an untracked expert");
    return 0;
  }
  int on_miss(Expert *e, bool) override {
    ENG_CHECK(eng, !map.count(e) && !persisted.count(e), "static: miss on a tracked expert");
    if (ll.size() == max_alt) {  // the oldest rotating entry becomes permanent
      Expert *p = ll.front();
      ll.pop_front();
      map.erase(p);
      persisted.insert(p);
    }
    ENG_CHECK(eng, ll.size() < max_alt, "static: rotating buffer overflow");
    ll.push_back(e);
    map[e] = std::prev(ll.end());
    return 0;
  }
  int evict(Expert *e) override {
    auto it = map.find(e);
    ENG_CHECK(eng, it != map.end() && !persisted.count(e), "static: evict of a persisted/unknown expert");
    ll.erase(it->second);
    map.erase(it);
    return 0;
  }
};

struct PolicyHeapBase : Policy {
  moe_engine *eng;
  MinHeap heap;
  std::unordered_map<Expert *, MinHeap::Node *> map;
  std::vector<MinHeap::Node *> free_nodes;
  explicit PolicyHeapBase(moe_engine *e) : eng(e) {}
  ~PolicyHeapBase() override {
    for (auto &kv : map) delete kv.second;
    for (auto *n : free_nodes) delete n;
  }
  MinHeap::Node *new_node() {
    if (free_nodes.empty()) return new MinHeap::Node();
    auto *n = free_nodes.back();
    free_nodes.pop_back();
    return n;
  }
  Expert *select_for_evict() override { return heap.front() ? heap.front()->e : nullptr; }
  int evict(Expert *e) override {
    auto it = map.find(e);
    ENG_CHECK(eng, it != map.end(), "heap policy: evict of an unknown expert");
    heap.remove(it->second);
    free_nodes.push_back(it->second);
    map.erase(it);
    return 0;
  }
  int insert(Expert *e, float p) {
    ENG_CHECK(eng, !map.count(e), "heap policy: miss on a tracked expert");
    auto *n = new_node();
    n->e = e;
    n->priority = p;
    map[e] = n;
    heap.push(n);
    return 0;
  }
  std::string to_string() override {
    auto v = heap.buf;
    std::sort(v.begin(), v.end(), [](MinHeap::Node *a, MinHeap::Node *b) { return a->priority > b->priority; });
    std::string s;
    for (auto *n : v) s += "(" + std::to_string(n->priority) + "," + std::to_string(n->e->idx) + "),";
    return s;
  }
};

struct PolicyNN : PolicyHeapBase {  // cache.hpp:81-126, cache.cpp:383-399
  using PolicyHeapBase::PolicyHeapBase;
  float prio(Expert *e) { return eng->priority[(size_t)e->layer * eng->cfg.num_expert + e->idx]; }
  int on_hit(Expert *e, bool) override {
    ENG_CHECK(eng, map.count(e), "nn: hit on an untracked expert");
    return 0;
  }
  int on_miss(Expert *e, bool) override { return insert(e, prio(e)); }
  void update_all_priority() override {
    for (auto &kv : map) kv.second->priority = prio(kv.first);
    heap.rebuild();
  }
  void update_priority(Expert *e, float p) override {
    auto it = map.find(e);
    if (it != map.end()) heap.update(it->second, p);
  }
};

struct PolicyMIN : PolicyHeapBase {  // cache.hpp:146-224, cache.cpp:490-583
  using PolicyHeapBase::PolicyHeapBase;
  SeqOracle *cur = nullptr;
  int64_t now = -1;
  std::unordered_map<Expert *, size_t> next_idx;
  int set_cur_seq(uint64_t seq) override {
    auto it = eng->oracles.find(seq);
    ENG_CHECK(eng, it != eng->oracles.end(), "min: no oracle loaded for sequence %llu", (unsigned long long)seq);
    cur = &it->second;
    now = -1;
    for (auto &kv : next_idx) kv.second = 0;
    for (auto &kv : map) {
      ENG_CHECK(eng, next_idx.count(kv.first), "min: cached expert without a use index");
      kv.second->priority = -(float)cur->use_times[kv.first][0];
    }
    heap.rebuild();
    return 0;
  }
  int advance(Expert *e, bool precise, float *prio) {
    ENG_CHECK(eng, cur != nullptr, "min: set_cur_seq was not called");
    auto &ut = cur->use_times[e];
    ENG_CHECK(eng, !ut.empty(), "min: expert missing from the oracle");
    size_t &i = next_idx[e];  // inserts 0
    if (precise) {
      ENG_CHECK(eng, i < ut.size(), "min: access beyond the recorded trace");
      ENG_CHECK(eng, now <= ut[i], "min: out-of-order access (%lld > %lld)", (long long)now, (long long)ut[i]);
      now = ut[i];
      ++i;
      ENG_CHECK(eng, i < ut.size(), "min: access beyond the recorded trace");
    }
    *prio = -(float)ut[i];
    return 0;
  }
  int on_hit(Expert *e, bool precise) override {
    float p;
    if (int rc = advance(e, precise, &p)) return rc;
    auto it = map.find(e);
    ENG_CHECK(eng, it != map.end(), "min: hit on an untracked expert");
    heap.update(it->second, p);
    return 0;
  }
  int on_miss(Expert *e, bool precise) override {
    float p;
    if (int rc = advance(e, precise, &p)) return rc;
    return insert(e, p);
  }
};

Policy *make_policy(moe_engine *eng, const std::string &name) {
  if (name == "fifo") return new PolicyFIFO(eng);
  if (name == "lru") return new PolicyLRU(eng);
  if (name == "static-1") return new PolicyStatic(eng, 1);
  if (name == "static-2") return new PolicyStatic(eng, 2);
  if (name == "nn") return new PolicyNN(eng);
  if (name == "min") return new PolicyMIN(eng);
  return nullptr;
}

// order in which slot groups receive the remainder (cache.cpp:9-53): breadth-first
// midpoints of [begin,end); once a width-1 interval is met with others pending, the
// rest is flattened and traversed again.
void bi_traverse(const std::vector<int> &arr, int begin, int end, std::vector<int> &ret) {
  if (begin == end) return;
  std::deque<std::pair<int, int>> q;
  q.push_back({begin, end});
  while (!q.empty()) {
    auto [l, r] = q.front();
    q.pop_front();
    if (l == r) continue;
    if (r - l == 1) {
      if (q.empty()) { ret.push_back(arr[l]); return; }
      std::vector<int> rest;
      for (int i = l; i < r; ++i) rest.push_back(arr[i]);
      while (!q.empty()) {
        auto [l2, r2] = q.front();
        q.pop_front();
        for (int i = l2; i < r2; ++i) rest.push_back(arr[i]);
      }
      bi_traverse(rest, 0, (int)rest.size(), ret);
      return;
    }
    const int mid = (l + r) / 2;
    ret.push_back(arr[mid]);
    if (l < mid) q.push_back({l, mid});
    if (mid + 1 < r) q.push_back({mid + 1, r});
  }
}

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

extern "C" int moe_slot_distribution(int64_t num_buffers, int n_groups, int64_t *out) {
  if (num_buffers < 0 || n_groups <= 0 || !out) { moe_set_error("moe_slot_distribution: bad argument"); return MOE_EINVAL; }
  const int64_t base = num_buffers / n_groups, rem = num_buffers % n_groups;
  std::vector<int> cand(n_groups), order;
  for (int i = 0; i < n_groups; ++i) cand[i] = i;
  if (n_groups > 2) {
    order.push_back(0);
    order.push_back(1);
    bi_traverse(cand, 2, n_groups, order);
  } else {
    order = cand;
  }
  for (int i = 0; i < n_groups; ++i) out[order[i]] = base + (i < rem ? 1 : 0);
  return MOE_OK;
}

// ---------------------------------------------------------------------------
// cache manager (cache.cpp:229-312)
// ---------------------------------------------------------------------------
static inline size_t flat(moe_engine *eng, Expert *e) { return (size_t)e->layer * eng->cfg.num_expert + e->idx; }

static void set_table(moe_engine *eng, Expert *e, bool resident_complete) {
  uint64_t v = resident_complete && e->slot >= 0 ? (uint64_t)((char *)eng->pool_base + (size_t)e->slot * eng->slot_stride) : 0;
  if (eng->h_table && eng->h_table[flat(eng, e)] != v) {
    eng->h_table[flat(eng, e)] = v;
    eng->table_dirty[e->layer] = 1;
  }
}

static int cache_hit(moe_engine *eng, Expert *e, bool precise) {
  (precise ? eng->ctr.hit : eng->ctr.prefetch_hit)++;
  Group &g = eng->group_of(e->layer);
  if (int rc = g.policy->on_hit(e, precise)) return rc;
  if (precise) {
    eng->max_priority += 1;
    g.policy->update_priority(e, eng->max_priority);
    if (eng->cfg.cache_policy == "nn") eng->priority[flat(eng, e)] = eng->max_priority;
  }
  return 0;
}

// returns in *victim_wait the previous owner of the slot when it is still
// launching/in use on the compute stream (the copy must wait for it)
static int cache_miss(moe_engine *eng, Expert *in, bool precise, Expert **victim_wait) {
  (precise ? eng->ctr.miss : eng->ctr.prefetch_miss)++;
  *victim_wait = nullptr;
  Group &g = eng->group_of(in->layer);
  if (precise) {
    eng->max_priority += 1;
    if (eng->cfg.cache_policy == "nn") eng->priority[flat(eng, in)] = eng->max_priority;
  }
  if (!g.unused.empty()) {
    in->slot = g.unused.back();
    g.unused.pop_back();
    if (int rc = g.policy->on_miss(in, precise)) return rc;
    eng->resident[in] = in->slot;
    return 0;
  }
  Expert *v = g.policy->select_for_evict();
  ENG_CHECK(eng, v != nullptr, "cache miss in a slot group without slots (layer %d)", in->layer);
  ENG_CHECK(eng, v != in, "policy selected the incoming expert as victim");
  if (int rc = g.policy->evict(v)) return rc;
  if (int rc = g.policy->on_miss(in, precise)) return rc;
  auto it = eng->resident.find(v);
  ENG_CHECK(eng, it != eng->resident.end(), "victim is not resident");
  const int slot = it->second;
  eng->resident.erase(it);
  eng->resident[in] = slot;
  eng->ctr.evictions++;
  const int st = v->status.load();
  if (st == kReady) {
    v->status = kIdle;
  } else if (st == kUsing || st == kLaunching) {
    *victim_wait = v;  // deferred: the fetch thread waits before overwriting the slot
  } else {
    ENG_CHECK(eng, st == kFetching, "evicting an expert in state %d", st);
    v->status = kIdle;  // a partially fetched expert
  }
  ENG_CHECK(eng, v->slot == slot, "slot bookkeeping mismatch");
  if (v->num_ready == eng->cfg.num_per_expert_param) eng->layer_complete[v->layer]--;
  v->num_ready = 0;
  if (*victim_wait == nullptr) {
    set_table(eng, v, false);
    v->slot = -1;
  }  // else: the victim keeps its slot address until the fetch thread has waited for it,
     // as the reference's logical tensor keeps its mapping until the copy starts (worker.cpp:98-101)
  in->slot = slot;
  return 0;
}

// ---------------------------------------------------------------------------
// scheduler handlers (all called with eng->mu held)
// ---------------------------------------------------------------------------
static inline bool in_cache(moe_engine *eng, Expert *e) { return eng->resident.count(e) != 0; }

// every queued task bumps the engine's task counter (under the engine lock): what that engine's idle fetch thread
// polls before it sleeps
static void add_task(moe_engine *eng, std::deque<CopyTask> &q, Expert *e, int start, int stop, bool precise) {
  CopyTask t;
  t.e = e; t.start = start; t.stop = stop; t.precise = precise;
  q.push_back(t);
  eng->task_epoch.fetch_add(1, std::memory_order_release);
}

// `ready -> launching` of a demand hit (prefetcher.cpp:51,105).  `using` is resolved
// here instead of by an unlocker thread: new launches on the same stream may read the
// slot while older ones still do.
static int make_launching(moe_engine *eng, Expert *e) {
  const int st = e->status.load();
  if (st == kReady || st == kUsing || st == kLaunching) { e->status = kLaunching; return 0; }
  return engine_fail(eng, "transfer ready->launching, but expert %d.%d is in state %d", e->layer, e->idx, st);
}

// prefetcher.cpp:6-42
static void reorder_experts(moe_engine *eng, int layer, int64_t *ids, int64_t n) {
  std::vector<Expert *> done, going, partial, miss;
  const int P = eng->cfg.num_per_expert_param;
  for (int64_t i = 0; i < n; ++i) {
    Expert *e = eng->ex(layer, (int)ids[i]);
    if (e == eng->current.e) going.push_back(e);
    else if (in_cache(eng, e)) (e->num_ready == P ? done : partial).push_back(e);
    else miss.push_back(e);
  }
  int64_t k = 0;
  for (auto *e : done) ids[k++] = e->idx;
  for (auto *e : going) ids[k++] = e->idx;
  for (auto *e : partial) ids[k++] = e->idx;
  for (auto *e : miss) ids[k++] = e->idx;
}

// shared tail of preempt_one_expert / preempt_one_layer_without_reorder_
// (prefetcher.cpp:44-70, 102-124)
static int preempt_resident(moe_engine *eng, Expert *e) {
  const int P = eng->cfg.num_per_expert_param;
  if (e->num_ready == P) {
    if (int rc = make_launching(eng, e)) return rc;
    return cache_hit(eng, e, true);
  }
  if (e == eng->current.e) {
    eng->current.precise = true;
    if (eng->current.stop == P) return cache_hit(eng, e, true);
    add_task(eng, eng->precise_q, e, eng->current.stop, P, true);
    return 0;
  }
  add_task(eng, eng->precise_q, e, e->num_ready, P, true);
  return 0;
}

static int preempt_one_expert(moe_engine *eng, int layer, int64_t id) {
  Expert *e = eng->ex(layer, (int)id);
  if (!in_cache(eng, e)) { add_task(eng, eng->precise_q, e, 0, eng->cfg.num_per_expert_param, true); return 0; }
  return preempt_resident(eng, e);
}

// prefetcher.cpp:72-125
static int preempt_one_layer(moe_engine *eng, int layer, const int64_t *ids, int64_t n) {
  const int P = eng->cfg.num_per_expert_param;
  bool preceding_in_cache = true;
  for (int64_t i = 0; i < n; ++i) {
    Expert *e = eng->ex(layer, (int)ids[i]);
    if (!in_cache(eng, e)) {
      preceding_in_cache = false;
      add_task(eng, eng->precise_q, e, 0, P, true);
      continue;
    }
    if (!preceding_in_cache) {  // may be evicted by a preceding miss: redundant demand task
      add_task(eng, eng->precise_q, e, 0, P, true);
      continue;
    }
    if (int rc = preempt_resident(eng, e)) return rc;
  }
  return 0;
}

// prefetcher.cpp:143-161
static bool pop_next_task(moe_engine *eng, CopyTask &t) {
  if (!eng->precise_q.empty()) { t = eng->precise_q.front(); eng->precise_q.pop_front(); return true; }
  for (auto &q : eng->layer_q)
    if (!q.empty()) { t = q.front(); q.pop_front(); return true; }
  return false;
}

// prefetcher.cpp:613-659.  *sent = false: nothing to copy (duplicate)
static int send_one_job(moe_engine *eng, CopyTask &t, bool *sent) {
  const int P = eng->cfg.num_per_expert_param;
  *sent = false;
  t.wait_victim = nullptr;
  Expert *e = t.e;
  if (e->slot < 0) {
    ENG_CHECK(eng, t.start == 0, "copy task for a non-resident expert does not start at chunk 0");
    ENG_CHECK(eng, e->num_ready == 0, "non-resident expert with ready chunks");
    if (int rc = cache_miss(eng, e, t.precise, &t.wait_victim)) return rc;
    ENG_CHECK(eng, e->status.load() == kIdle, "transfer idle->fetching, but expert %d.%d is in state %d",
              e->layer, e->idx, e->status.load());
    e->status = kFetching;
  } else {
    if (t.precise || t.start == 0)
      if (int rc = cache_hit(eng, e, t.precise)) return rc;
    if (e->num_ready >= t.stop) {  // fully duplicated task
      if (t.precise) {
        ENG_CHECK(eng, e->num_ready == P, "duplicate demand task on a partial expert");
        const int st = e->status.load();
        if (st == kReady || st == kUsing) e->status = kLaunching;
      }
      return 0;
    } else if (e->num_ready > t.start) {
      t.start = e->num_ready;
    } else {
      ENG_CHECK(eng, e->num_ready == t.start, "copy task skips chunks");
    }
  }
  eng->current = t;
  *sent = true;
  return 0;
}

// prefetcher.cpp:556-570
static int fetch_done(moe_engine *eng) {
  const int P = eng->cfg.num_per_expert_param;
  Expert *e = eng->current.e;
  e->num_ready = eng->current.stop;
  if (eng->current.stop == P) {
    ENG_CHECK(eng, e->status.load() == kFetching, "fetch done for an expert in state %d", e->status.load());
    e->status = eng->current.precise ? kLaunching : kReady;
    set_table(eng, e, true);
    eng->layer_complete[e->layer]++;
  }
  eng->current.e = nullptr;
  return 0;
}

static void resolve_using(moe_engine *eng, Expert *v, std::unique_lock<std::mutex> &lk) {
  // wait until the compute stream is past the victim, then release it (cache.cpp:291-297,
  // worker.cpp:78-83)
  for (;;) {
    const int st = v->status.load();
    if (st == kReady) { v->status = kIdle; return; }
    if (st == kIdle) return;
    if (st == kUsing) {
      if (v->seq_ptr) {
        // released against a sequence word: it normally arrives with the caller's next launch; if it
        // does not (the caller stopped, or took another path), an event recorded now proves the same
        const volatile int *sp = v->seq_ptr;
        const int need = v->seq_need;
        eng->seq_pollers.fetch_add(1, std::memory_order_acq_rel);  // (under the lock: see moe_forward_prepare)
        lk.unlock();
        const auto t0 = std::chrono::steady_clock::now();
        bool reached = false;
        while (!(reached = (int)((unsigned)*sp - (unsigned)need) >= 0) &&
               std::chrono::steady_clock::now() - t0 < std::chrono::microseconds(100)) {}
        eng->seq_pollers.fetch_sub(1, std::memory_order_acq_rel);  // sp is not read again
        if (!reached) {
          moe_spin_lock(lk);
          if (!eng->proof_event) eng->proof_event = eng->be->event_create();
          void *pe = eng->proof_event;
          if (pe) eng->be->event_record(pe, eng->be->compute_stream());
          lk.unlock();
          if (pe) eng->be->event_sync(pe);
        }
        moe_spin_lock(lk);
        if (v->status.load() == kUsing && v->seq_ptr == sp && v->seq_need == need) { v->seq_ptr = nullptr; v->status = kReady; }
        continue;
      }
      void *ev = v->event;
      if (ev) { lk.unlock(); eng->be->event_sync(ev); moe_spin_lock(lk); }
      if (v->status.load() == kUsing) v->status = kReady;
      continue;
    }
    if (eng->exiting) return;
    eng->cv_state.wait_for(lk, std::chrono::milliseconds(1));  // launching: caller has not launched yet
  }
}

static void fetch_thread_main(moe_engine *eng) {
  std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
  while (!eng->exiting) {
    CopyTask t;
    if (!eng->fatal.empty() || !pop_next_task(eng, t)) {
      // A decode loop brings the next task within tens of microseconds, and waking this thread up from the
      // condition variable would cost that task 10-50 us before its copy starts: poll the task counter for a
      // while without the lock first (tasks are queued under the lock, so none can slip in between the last
      // look at the counter below and the wait).
      const unsigned ep = eng->task_epoch.load(std::memory_order_acquire);
      if (eng->fatal.empty()) {
        lk.unlock();
        const auto t0 = std::chrono::steady_clock::now();
        for (unsigned spins = 0; eng->task_epoch.load(std::memory_order_acquire) == ep; ++spins) {
#if defined(__x86_64__)
          __builtin_ia32_pause();
#endif
          if ((spins & 63u) == 63u && std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(500)) break;
        }
        moe_spin_lock(lk);
      }
      if (eng->task_epoch.load(std::memory_order_acquire) == ep && !eng->exiting) eng->cv_work.wait(lk);
      continue;
    }
    bool sent = false;
    if (send_one_job(eng, t, &sent) != 0 || !sent) {
      eng->current.e = nullptr;
      eng->cv_state.notify_all();
      continue;
    }
    Expert *e = eng->current.e;
    const int start = eng->current.start, stop = eng->current.stop;
    // a kernel may be reading any slot of this group through a table snapshot: the slot stays as it is
    // until the caller has seen that kernel's selection and protected what it uses
    // (a guard stands for the few microseconds between a one-token launch and the hooks of its layer: look again
    // every microsecond or so, without the lock in between, before falling back to timed waits; the release
    // notifies, but waking up from it would cost the demand copy of that very layer 10-50 us)
    {
      const auto g0 = std::chrono::steady_clock::now();
      while (eng->group_of(e->layer).guard > 0 && !eng->exiting) {
        if (std::chrono::steady_clock::now() - g0 < std::chrono::microseconds(300)) {
          lk.unlock();
#if defined(__x86_64__)
          for (int i = 0; i < 32; ++i) __builtin_ia32_pause();
#endif
          moe_spin_lock(lk);
        } else {
          eng->cv_state.wait_for(lk, std::chrono::microseconds(50));
        }
      }
    }
    if (Expert *v = eng->current.wait_victim) {
      resolve_using(eng, v, lk);
      if (v->slot == e->slot && !in_cache(eng, v)) { set_table(eng, v, false); v->slot = -1; }
    }
    char *dst = (char *)eng->pool_base + (size_t)e->slot * eng->slot_stride;
    lk.unlock();
    int rc = 0;
    size_t bytes = 0;
    // chunks that are neighbours both in host memory and in the slot go out as one copy
    for (int c = start; c < stop && rc == 0;) {
      const HostChunk &hc = e->chunks[c];
      size_t n = hc.nbytes;
      int c2 = c + 1;
      while (c2 < stop && e->chunks[c2].nbytes && n &&
             (const char *)e->chunks[c2].ptr == (const char *)hc.ptr + n &&
             eng->chunk_off[c2] == eng->chunk_off[c] + n) {
        n += e->chunks[c2].nbytes;
        ++c2;
      }
      if (n) rc = eng->be->copy_h2d(dst + eng->chunk_off[c], hc.ptr, n);
      bytes += n;
      c = c2;
    }
    if (rc == 0) rc = eng->be->copy_sync();
    moe_spin_lock(lk);
    if (rc != 0) engine_fail(eng, "host->slot copy failed: %s", moe_last_error());
    eng->ctr.h2d_bytes += bytes;
    eng->ctr.h2d_copies += (uint64_t)(stop - start);
    fetch_done(eng);
    eng->cv_state.notify_all();
  }
}

// ---------------------------------------------------------------------------
// engine lifetime
// ---------------------------------------------------------------------------
moe_engine::~moe_engine() {
  {
    std::lock_guard<std::mutex> lk(mu);
    exiting = true;
  }
  cv_work.notify_all();
  cv_state.notify_all();
  cv_sem.notify_all();
  moe_predictor_free(this);
  if (fetch_thread.joinable()) fetch_thread.join();
  if (fw) { moe_forward_free(fw); fw = nullptr; }
}

extern "C" int moe_engine_create(const moe_cfg *cfg, int backend, void *compute_stream, moe_engine **out) {
  if (!cfg || !out) { moe_set_error("moe_engine_create: null argument"); return MOE_EINVAL; }
  if (!cfg->finalized) { moe_set_error("moe_engine_create: configuration not finalized"); return MOE_ESTATE; }
  Backend *be = nullptr;
  if (backend == MOE_BACKEND_HIP) be = moe_make_hip_backend(compute_stream, cfg->cache_only);
  else if (backend == MOE_BACKEND_HOST) be = moe_make_host_backend();
  else { moe_set_error("moe_engine_create: unknown backend %d", backend); return MOE_EINVAL; }
  if (!be) return MOE_EHIP;
  moe_engine *eng = new moe_engine();
  eng->cfg = *cfg;
  eng->be.reset(be);
  const int L = cfg->num_layer, E = cfg->num_expert;
  eng->experts.resize((size_t)L * E);
  for (int l = 0; l < L; ++l)
    for (int e = 0; e < E; ++e) {
      auto x = std::make_unique<Expert>();
      x->layer = l; x->idx = e;
      x->chunks.resize(cfg->num_per_expert_param);
      eng->experts[(size_t)l * E + e] = std::move(x);
    }
  eng->groups.resize(cfg->per_layer_cache ? L : 1);
  for (auto &g : eng->groups) g.policy.reset(make_policy(eng, cfg->cache_policy));
  eng->priority.assign((size_t)L * E, 0.f);
  eng->layer_q.resize(L);
  eng->table_dirty.assign(L, 0);
  eng->layer_event.assign(L, nullptr);
  eng->layer_complete.assign(L, 0);
  eng->budget = cfg->max_prefetch_layer_distance;
  eng->layer_desc.resize(L);
  for (auto &d : eng->layer_desc) memset(&d, 0, sizeof d);
  *out = eng;
  return MOE_OK;
}

extern "C" void moe_engine_destroy(moe_engine *eng) { delete eng; }

#define ENG_GUARD(eng)                                                        \
  if (!(eng)) { moe_set_error("null engine"); return MOE_EINVAL; }            \
  if (!(eng)->fatal.empty()) { moe_set_error("engine is in a failed state: %s", (eng)->fatal.c_str()); return MOE_ESTATE; }

static int check_le(moe_engine *eng, int layer, int expert) {
  if (layer < 0 || layer >= eng->cfg.num_layer || expert < 0 || expert >= eng->cfg.num_expert) {
    moe_set_error("layer/expert out of range (%d, %d)", layer, expert);
    return MOE_EINVAL;
  }
  return 0;
}

extern "C" int moe_register_param(moe_engine *eng, int layer, int expert, int param_id,
                                  const void *host_ptr, size_t nbytes, size_t alloc_nbytes) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, expert)) return rc;
  if (param_id < 0 || param_id >= eng->cfg.num_per_expert_param || (!host_ptr && nbytes)) {
    moe_set_error("moe_register_param: bad param_id %d or null pointer", param_id);
    return MOE_EINVAL;
  }
  if (eng->slots_ready) { moe_set_error("moe_register_param: slots already initialised"); return MOE_ESTATE; }
  HostChunk &c = eng->ex(layer, expert)->chunks[param_id];
  c.ptr = host_ptr; c.nbytes = nbytes; c.alloc = alloc_nbytes ? alloc_nbytes : nbytes;
  return MOE_OK;
}

extern "C" int moe_pin_host(moe_engine *eng, int *n_unpinned) {
  ENG_GUARD(eng);
  int n = 0;
  for (auto &e : eng->experts)
    for (auto &c : e->chunks)
      if (c.ptr && c.nbytes && !eng->be->is_pinned(c.ptr)) ++n;
  if (n_unpinned) *n_unpinned = n;
  return MOE_OK;
}

extern "C" int moe_init_slots(moe_engine *eng) {
  ENG_GUARD(eng);
  if (eng->slots_ready) { moe_set_error("moe_init_slots: already done"); return MOE_ESTATE; }
  const moe_cfg &c = eng->cfg;
  const int L = c.num_layer, E = c.num_expert, P = c.num_per_expert_param;
  // dummy chunks emulate larger experts (model_loader.cpp:33-60)
  if (c.num_dummy_params > 0) {
    size_t cur = 0;
    Expert *e0 = eng->ex(0, 0);
    for (int i = 0; i < P - c.num_dummy_params; ++i) cur += e0->chunks[i].nbytes;
    long dummy = (long)(cur * (c.expert_mem_scale - 1));
    long per = round_up((size_t)(dummy / c.num_dummy_params), 16);
    void *buf = moe_host_alloc(per);
    if (!buf) return MOE_ENOMEM;
    memset(buf, 0, per);
    eng->dummy_bufs.push_back(buf);
    for (auto &e : eng->experts)
      for (int i = P - c.num_dummy_params; i < P; ++i) { e->chunks[i].ptr = buf; e->chunks[i].nbytes = per; e->chunks[i].alloc = per; }
  }
  size_t max_bytes = 0;
  Expert *example = eng->ex(0, 0);
  for (auto &e : eng->experts) {
    const size_t t = e->total_alloc();
    if (t > max_bytes) { max_bytes = t; example = e.get(); }
  }
  if (max_bytes == 0) { moe_set_error("moe_init_slots: no expert parameters registered"); return MOE_ESTATE; }
  eng->chunk_off.assign(P, 0);
  size_t off = 0;
  for (int i = 0; i < P; ++i) { eng->chunk_off[i] = off; off += example->chunks[i].alloc; }
  for (auto &e : eng->experts)  // every expert must fit the example's chunk grid
    for (int i = 0; i < P; ++i)
      if (e->chunks[i].nbytes > example->chunks[i].alloc) {
        moe_set_error("expert %d.%d chunk %d (%zu B) exceeds the slot's chunk size (%zu B)", e->layer, e->idx, i,
                      e->chunks[i].nbytes, example->chunks[i].alloc);
        return MOE_EINVAL;
      }
  // cache_len (prefetcher.cpp:169-174): float arithmetic, then round
  const float want = c.cache_rate * L * E;
  int64_t cache_len = (int64_t)std::round(want);
  if (cache_len > (int64_t)L * E) cache_len = (int64_t)L * E;
  const int G = (int)eng->groups.size();
  std::vector<int64_t> per(G);
  moe_slot_distribution(cache_len, G, per.data());
  eng->slot_bytes = max_bytes;
  eng->n_slots = (size_t)cache_len;
  if (cache_len > 0) {
    int rc = eng->be->alloc_pool(max_bytes, (size_t)cache_len, (size_t)L * E, c.pool_vmm, &eng->pool_base, &eng->slot_stride);
    if (rc) return rc;
  }
  int next = 0;
  for (int g = 0; g < G; ++g) {
    eng->groups[g].full_len = (size_t)per[g];
    for (int64_t i = 0; i < per[g]; ++i) eng->groups[g].unused.push_back(next++);
  }
  if (int rc = eng->be->alloc_table((size_t)L * E, &eng->d_table, &eng->h_table)) return rc;
  memset(eng->h_table, 0, sizeof(uint64_t) * L * E);
  std::fill(eng->table_dirty.begin(), eng->table_dirty.end(), 1);
  // cache.cpp:130-131
  eng->cfg.num_predict_expert_per_layer = std::min<int>(c.num_predict_expert_per_layer, (int)eng->groups[0].full_len);
  eng->slots_ready = true;
  return MOE_OK;
}

extern "C" int moe_slot_info(moe_engine *eng, int group, int64_t *n_slots, int64_t *slot_bytes, int64_t *stride) {
  ENG_GUARD(eng);
  if (!eng->slots_ready) { moe_set_error("slots not initialised"); return MOE_ESTATE; }
  if (group < -1 || group >= (int)eng->groups.size()) { moe_set_error("bad group %d", group); return MOE_EINVAL; }
  if (n_slots) *n_slots = group < 0 ? (int64_t)eng->n_slots : (int64_t)eng->groups[group].full_len;
  if (slot_bytes) *slot_bytes = (int64_t)eng->slot_bytes;
  if (stride) *stride = (int64_t)eng->slot_stride;
  return MOE_OK;
}

extern "C" int moe_launch(moe_engine *eng) {
  ENG_GUARD(eng);
  if (!eng->slots_ready) { moe_set_error("moe_launch: call moe_init_slots first"); return MOE_ESTATE; }
  if (eng->launched) return MOE_OK;
  eng->launched = true;
  eng->fetch_thread = std::thread(fetch_thread_main, eng);
  return MOE_OK;
}

// ---------------------------------------------------------------------------
// lookup
// ---------------------------------------------------------------------------
extern "C" int moe_expert_param_ptr(moe_engine *eng, int layer, int expert, int param_id, void **out) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, expert)) return rc;
  if (!out || param_id < 0 || param_id >= eng->cfg.num_per_expert_param) { moe_set_error("bad param_id"); return MOE_EINVAL; }
  SpinGuard lk(eng->mu);
  Expert *e = eng->ex(layer, expert);
  *out = e->slot < 0 ? nullptr : (char *)eng->pool_base + (size_t)e->slot * eng->slot_stride + eng->chunk_off[param_id];
  return MOE_OK;
}

extern "C" int moe_expert_ptr_table(moe_engine *eng, int layer, const uint64_t **out) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if (!eng->slots_ready || !out) { moe_set_error("slots not initialised"); return MOE_ESTATE; }
  *out = eng->d_table + (size_t)layer * eng->cfg.num_expert;
  return MOE_OK;
}

extern "C" int moe_flush_table(moe_engine *eng, int layer, void *stream) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if (!eng->slots_ready) { moe_set_error("slots not initialised"); return MOE_ESTATE; }
  SpinGuard lk(eng->mu);
  if (!eng->table_dirty[layer]) return MOE_OK;
  eng->table_dirty[layer] = 0;
  const size_t o = (size_t)layer * eng->cfg.num_expert;
  return eng->be->flush_table(eng->d_table + o, eng->h_table + o, eng->cfg.num_expert, stream);
}

int moe_flush_table_guarded(moe_engine *eng, int layer, void *stream, char *resident_out) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if (!eng->slots_ready) { moe_set_error("slots not initialised"); return MOE_ESTATE; }
  SpinGuard lk(eng->mu);
  const size_t o = (size_t)layer * eng->cfg.num_expert;
  if (eng->table_dirty[layer]) {
    eng->table_dirty[layer] = 0;
    if (int rc = eng->be->flush_table(eng->d_table + o, eng->h_table + o, eng->cfg.num_expert, stream)) return rc;
  }
  for (int e = 0; e < eng->cfg.num_expert; ++e) resident_out[e] = eng->h_table[o + e] != 0;
  eng->group_of(layer).guard++;
  return MOE_OK;
}

// The guarded snapshot without the copy to the device: for launches that carry the table in their arguments.  The
// device table stays marked as it was, so a later launch that reads it still gets its flush.
int moe_snapshot_table_guarded(moe_engine *eng, int layer, uint64_t *table_out, char *resident_out) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if (!eng->slots_ready) { moe_set_error("slots not initialised"); return MOE_ESTATE; }
  SpinGuard lk(eng->mu);
  const size_t o = (size_t)layer * eng->cfg.num_expert;
  for (int e = 0; e < eng->cfg.num_expert; ++e) {
    table_out[e] = eng->h_table[o + e];
    resident_out[e] = table_out[e] != 0;
  }
  eng->group_of(layer).guard++;
  return MOE_OK;
}

void moe_guard_release(moe_engine *eng, int layer) {
  {
    SpinGuard lk(eng->mu);
    Group &g = eng->group_of(layer);
    if (g.guard > 0) g.guard--;
  }
  eng->cv_state.notify_all();
}

extern "C" int moe_expert_status(moe_engine *eng, int layer, int expert) {
  if (!eng || check_le(eng, layer, expert)) return MOE_EINVAL;
  SpinGuard lk(eng->mu);
  Expert *e = eng->ex(layer, expert);
  if (e->status.load() == kUsing && (e->seq_ptr ? e->seq_reached() : (!e->event || eng->be->event_done(e->event)))) {
    e->seq_ptr = nullptr;
    e->status = kReady;
  }
  return e->status.load();
}
extern "C" int moe_is_in_cache(moe_engine *eng, int layer, int expert) {
  if (!eng || check_le(eng, layer, expert)) return MOE_EINVAL;
  SpinGuard lk(eng->mu);
  return in_cache(eng, eng->ex(layer, expert)) ? 1 : 0;
}
extern "C" int moe_expert_num_ready(moe_engine *eng, int layer, int expert) {
  if (!eng || check_le(eng, layer, expert)) return MOE_EINVAL;
  SpinGuard lk(eng->mu);
  return eng->ex(layer, expert)->num_ready;
}

// ---------------------------------------------------------------------------
// hook sequence
// ---------------------------------------------------------------------------
int moe_report_layer_logits_bookkeeping(moe_engine *eng, int layer, int S) {
  ENG_GUARD(eng);
  if (layer < 0 || layer > eng->cfg.num_layer) { moe_set_error("bad layer %d", layer); return MOE_EINVAL; }
  SpinGuard lk(eng->mu);
  if (layer == 0) eng->s_seqlen.push_back((uint64_t)S);  // prefetcher.cpp:452-455
  return MOE_OK;
}

extern "C" int moe_report_layer_logits(moe_engine *eng, int layer, const void *hidden, int B, int S, int H) {
  if (int rc = moe_report_layer_logits_bookkeeping(eng, layer, S)) return rc;
  return moe_predictor_on_logits(eng, layer, hidden, B, S, H);  // prefetcher.cpp:451-452
}

static int report_one_layer_locked(moe_engine *eng, int layer, int64_t *ids, int64_t n,
                                   std::unique_lock<std::mutex> &lk) {
  for (int64_t i = 0; i < n; ++i)
    if (ids[i] < 0 || ids[i] >= eng->cfg.num_expert) { moe_set_error("expert id %lld out of range", (long long)ids[i]); return MOE_EINVAL; }
  if (eng->predictor_attached) {  // consume_prefetch_layer_progress (worker.hpp:312-314)
    eng->cv_sem.wait(lk, [&] { return eng->progress > 0 || eng->exiting; });
    if (eng->progress > 0) eng->progress--;
    // the layer's request for this turn has been issued: a decode step (prefetcher.cpp:467: at most top-k ids)
    // tells the built-in predictor what the layer routed to, before the hooks reorder the ids
    if (n > 0 && n <= std::max(eng->cfg.num_expert_per_token, 1)) moe_predictor_observe(eng, layer, ids, n);
  }
  // PreemptTask (prefetcher.cpp:521-537)
  if (eng->cfg.reorder_experts) reorder_experts(eng, layer, ids, n);
  if (eng->cfg.early_preempt) {
    if (int rc = preempt_one_layer(eng, layer, ids, n)) return rc;
    eng->budget++;
    eng->cv_sem.notify_all();
  }
  eng->layer_q[layer].clear();
  eng->ctr.activated += (uint64_t)n;
  eng->cv_work.notify_all();
  return MOE_OK;
}

extern "C" int moe_report_one_layer(moe_engine *eng, int layer, int64_t *ids, int64_t n) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if ((n > 0 && !ids) || n < 0) { moe_set_error("moe_report_one_layer: bad ids"); return MOE_EINVAL; }
  if (!eng->launched) { moe_set_error("engine not launched"); return MOE_ESTATE; }
  std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
  return report_one_layer_locked(eng, layer, ids, n, lk);
}

static bool is_queued(moe_engine *eng, Expert *e) {
  if (eng->current.e == e) return true;
  for (auto &t : eng->precise_q) if (t.e == e) return true;
  return false;
}

static int wait_expert_locked(moe_engine *eng, Expert *e, std::unique_lock<std::mutex> &lk) {
  if (e->status.load() == kLaunching) { eng->ctr.ready++; return MOE_OK; }
  eng->ctr.unready++;
  if (!is_queued(eng, e)) {
    moe_set_error("wait on expert %d.%d which has no demand fetch pending (state %d): it was not reported",
                  e->layer, e->idx, e->status.load());
    return MOE_ESTATE;
  }
  const auto t0 = std::chrono::steady_clock::now();
  eng->cv_work.notify_all();
  // a demand copy is over in about 100 us: poll the expert's state (an atomic) without the lock for that long before
  // sleeping on the condition variable, whose wake-up alone costs 10-50 us per miss
  lk.unlock();
  while (e->status.load(std::memory_order_acquire) != kLaunching &&
         std::chrono::steady_clock::now() - t0 < std::chrono::microseconds(400)) {
#if defined(__x86_64__)
    for (int i = 0; i < 64; ++i) __builtin_ia32_pause();
#else
    std::this_thread::yield();
#endif
  }
  moe_spin_lock(lk);
  eng->cv_state.wait(lk, [&] { return e->status.load() == kLaunching || eng->exiting || !eng->fatal.empty(); });
  eng->ctr.wait_us += (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count();
  if (!eng->fatal.empty()) { moe_set_error("engine failed while waiting: %s", eng->fatal.c_str()); return MOE_ESTATE; }
  return MOE_OK;
}

extern "C" int moe_wait_expert(moe_engine *eng, int layer, int expert) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, expert)) return rc;
  if (!eng->launched) { moe_set_error("engine not launched"); return MOE_ESTATE; }
  std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
  if (!eng->cfg.early_preempt) {  // PreemptOneExpertTask (prefetcher.cpp:225-233)
    if (int rc = preempt_one_expert(eng, layer, expert)) return rc;
    eng->cv_work.notify_all();
  }
  return wait_expert_locked(eng, eng->ex(layer, expert), lk);
}

extern "C" int moe_expert_launched(moe_engine *eng, int layer, int expert) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, expert)) return rc;
  std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
  Expert *e = eng->ex(layer, expert);
  ENG_CHECK(eng, e->status.load() == kLaunching, "transfer launching->using, but expert %d.%d is in state %d", layer,
            expert, e->status.load());
  if (!e->own_event) e->own_event = eng->be->event_create();
  e->event = e->own_event;
  e->seq_ptr = nullptr;
  if (e->event) eng->be->event_record(e->event, eng->be->compute_stream());
  e->status = kUsing;
  eng->cv_state.notify_all();
  return MOE_OK;
}

static void push_forward_series(moe_engine *eng) {
  auto &c = eng->ctr;
  auto &b = eng->fwd_base;
  eng->s_act.push_back(c.activated - b.activated);
  eng->s_hit.push_back(c.hit - b.hit);
  eng->s_miss.push_back(c.miss - b.miss);
  eng->s_ready.push_back(c.ready - b.ready);
  eng->s_unready.push_back(c.unready - b.unready);
  eng->s_phit.push_back(c.prefetch_hit - b.prefetch_hit);
  eng->s_pmiss.push_back(c.prefetch_miss - b.prefetch_miss);
  eng->s_wait.push_back(c.wait_us - b.wait_us);
  c.forwards++;
  b = c;
}

extern "C" int moe_layer_done(moe_engine *eng, int layer) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  SpinGuard lk(eng->mu);
  if (!eng->cfg.early_preempt) { eng->budget++; eng->cv_sem.notify_all(); }
  if (layer == eng->cfg.num_layer - 1) push_forward_series(eng);
  return MOE_OK;
}

extern "C" int moe_acquire_layer(moe_engine *eng, int layer, int64_t *ids, int64_t n) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if ((n > 0 && !ids) || n < 0) { moe_set_error("moe_acquire_layer: bad ids"); return MOE_EINVAL; }
  if (!eng->launched) { moe_set_error("engine not launched"); return MOE_ESTATE; }
  {
    std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
    if (int rc = report_one_layer_locked(eng, layer, ids, n, lk)) return rc;
    for (int64_t i = 0; i < n; ++i) {
      if (!eng->cfg.early_preempt) {
        if (int rc = preempt_one_expert(eng, layer, ids[i])) return rc;
        eng->cv_work.notify_all();
      }
      if (int rc = wait_expert_locked(eng, eng->ex(layer, (int)ids[i]), lk)) return rc;
    }
  }
  return moe_flush_table(eng, layer, eng->be->compute_stream());
}

extern "C" int moe_release_experts(moe_engine *eng, int layer, const int64_t *ids, int64_t n) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if ((n > 0 && !ids) || n < 0) { moe_set_error("moe_release_experts: bad ids"); return MOE_EINVAL; }
  SpinGuard lk(eng->mu);
  void *ev = nullptr;
  for (int64_t i = 0; i < n; ++i) {
    if (ids[i] < 0 || ids[i] >= eng->cfg.num_expert) { moe_set_error("expert id out of range"); return MOE_EINVAL; }
    Expert *x = eng->ex(layer, (int)ids[i]);
    ENG_CHECK(eng, x->status.load() == kLaunching, "transfer launching->using, but expert %d.%d is in state %d", layer,
              (int)ids[i], x->status.load());
    if (!ev) {
      if (!eng->layer_event[layer]) eng->layer_event[layer] = eng->be->event_create();
      ev = eng->layer_event[layer];
      if (ev) eng->be->event_record(ev, eng->be->compute_stream());
    }
    x->event = ev;
    x->seq_ptr = nullptr;
    x->status = kUsing;
  }
  eng->cv_state.notify_all();
  return MOE_OK;
}

int moe_release_experts_seq(moe_engine *eng, int layer, const int64_t *ids, int64_t n, const volatile int *seq_ptr, int seq_need) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  SpinGuard lk(eng->mu);
  for (int64_t i = 0; i < n; ++i) {
    if (ids[i] < 0 || ids[i] >= eng->cfg.num_expert) { moe_set_error("expert id out of range"); return MOE_EINVAL; }
    Expert *x = eng->ex(layer, (int)ids[i]);
    ENG_CHECK(eng, x->status.load() == kLaunching, "transfer launching->using, but expert %d.%d is in state %d", layer,
              (int)ids[i], x->status.load());
    x->event = nullptr;
    x->seq_ptr = seq_ptr;
    x->seq_need = seq_need;
    x->status = kUsing;
  }
  eng->cv_state.notify_all();
  return MOE_OK;
}

extern "C" int moe_release_layer(moe_engine *eng, int layer) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  SpinGuard lk(eng->mu);
  void *ev = nullptr;
  for (int e = 0; e < eng->cfg.num_expert; ++e) {
    Expert *x = eng->ex(layer, e);
    if (x->status.load() != kLaunching) continue;
    if (!ev) {
      // one event per layer call, shared by the experts it used
      if (!eng->layer_event[layer]) eng->layer_event[layer] = eng->be->event_create();
      ev = eng->layer_event[layer];
      if (ev) eng->be->event_record(ev, eng->be->compute_stream());
    }
    x->event = ev;
    x->seq_ptr = nullptr;
    x->status = kUsing;
  }
  eng->cv_state.notify_all();
  return MOE_OK;
}

// ---------------------------------------------------------------------------
// prefetch request hook
// ---------------------------------------------------------------------------
extern "C" int moe_prefetch_layer(moe_engine *eng, int layer, const int64_t *ids, int64_t n, int blocking) {
  return moe_prefetch_layer_over(eng, layer, ids, n, blocking, false);
}

// over_copy: accept the request although a copy of the same layer is still in flight.  The copy is a leftover
// of the layer's previous turn; the new tasks queue up behind it, and one that names the same expert is dropped
// as a duplicate when its turn comes.  The hook above refuses, as the reference does; the built-in predictor
// cannot: the copy may be held back by the slot-group guard of a forward that itself waits for this request.
int moe_prefetch_layer_over(moe_engine *eng, int layer, const int64_t *ids, int64_t n, int blocking, bool over_copy) {
  ENG_GUARD(eng);
  if (int rc = check_le(eng, layer, 0)) return rc;
  if ((n > 0 && !ids) || n < 0) { moe_set_error("moe_prefetch_layer: bad ids"); return MOE_EINVAL; }
  if (!eng->launched) { moe_set_error("engine not launched"); return MOE_ESTATE; }
  std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
  for (int64_t i = 0; i < n; ++i)
    if (ids[i] < 0 || ids[i] >= eng->cfg.num_expert) { moe_set_error("expert id out of range"); return MOE_EINVAL; }
  // run-ahead budget (worker.cpp:41-53)
  if (eng->exiting) return MOE_ESTATE;  // a producer that arrives after shutdown began must not sleep on the budget
  if (eng->budget <= 0) {
    if (!blocking) return 1;
    eng->cv_sem.wait(lk, [&] { return eng->budget > 0 || eng->exiting; });
    if (eng->exiting) return MOE_ESTATE;
  }
  eng->budget--;
  // PrefetchLayerTask (prefetcher.cpp:585-611)
  if (!eng->layer_q[layer].empty()) { moe_set_error("prefetch request for layer %d while its queue is not empty", layer); return MOE_ESTATE; }
  if (!over_copy && eng->current.e && eng->current.e->layer == layer) {
    moe_set_error("prefetch request for layer %d while a copy of that layer is in flight (expert %d, chunks %d..%d, %s, guard %d, progress %ld, budget %ld)",
                  layer, eng->current.e->idx, eng->current.start, eng->current.stop, eng->current.precise ? "demand" : "speculative",
                  eng->group_of(layer).guard, eng->progress, eng->budget);
    return MOE_ESTATE;
  }
  if (layer == 0 && eng->cfg.limit_layer_0_num_predict != -1) n = std::min<int64_t>(n, eng->cfg.limit_layer_0_num_predict);
  const int P = eng->cfg.num_per_expert_param;
  for (int64_t i = 0; i < n; ++i) {
    Expert *e = eng->ex(layer, (int)ids[i]);
    if (eng->cfg.promote_hit_in_prefetch && in_cache(eng, e))
      if (int rc = cache_hit(eng, e, false)) return rc;
    if (eng->cfg.chunk_prefetch) {
      // one task per parameter, as in the reference, except that a parameter of at most an eighth of its
      // predecessor's bytes (the scale and zero sections behind a nibble section) rides in that one's task: every
      // task costs the fetch thread a stream synchronisation and two turns of the lock (about 13 us), which
      // is more than such a section takes on the link.  A demand fetch still preempts between the tasks.
      for (int j = 0; j < P;) {
        int j2 = j + 1;
        while (j2 < P && e->chunks[j2].nbytes * 8 <= e->chunks[j].nbytes) ++j2;
        add_task(eng, eng->layer_q[layer], e, j, j2, false);
        j = j2;
      }
    }
    else add_task(eng, eng->layer_q[layer], e, 0, P, false);
  }
  eng->progress++;
  eng->cv_sem.notify_all();
  eng->cv_work.notify_all();
  return MOE_OK;
}

extern "C" int moe_attach_predictor(moe_engine *eng, int attached) {
  ENG_GUARD(eng);
  SpinGuard lk(eng->mu);
  eng->predictor_attached = attached != 0;
  return MOE_OK;
}

extern "C" int moe_update_priority(moe_engine *eng, const float *p, int n_layers, int starting_layer) {
  ENG_GUARD(eng);
  const int L = eng->cfg.num_layer, E = eng->cfg.num_expert;
  if (!p || n_layers <= 0 || starting_layer < 0 || starting_layer + n_layers > L) { moe_set_error("moe_update_priority: bad range"); return MOE_EINVAL; }
  if (eng->cfg.cache_policy != "nn") { moe_set_error("moe_update_priority: policy is %s, not nn", eng->cfg.cache_policy.c_str()); return MOE_ESTATE; }
  SpinGuard lk(eng->mu);
  std::copy(p, p + (size_t)n_layers * E, eng->priority.begin() + (size_t)starting_layer * E);
  eng->max_priority = *std::max_element(eng->priority.begin(), eng->priority.end());
  std::set<Group *> gs;
  for (int l = starting_layer; l < starting_layer + n_layers; ++l) gs.insert(&eng->group_of(l));
  if (n_layers == L) for (auto &g : eng->groups) gs.insert(&g);
  for (auto *g : gs) g->policy->update_all_priority();
  return MOE_OK;
}

// cache.cpp:592-644
extern "C" int moe_oracle_load(moe_engine *eng, const int64_t *entry_metas, int64_t n_entries,
                               const int32_t *prefill_len, int64_t n_seq, const int32_t *prefill_sel,
                               int64_t max_prefill_len, const int32_t *decode_sel, int64_t k) {
  ENG_GUARD(eng);
  if (n_seq < 0 || n_entries < 0 || (n_seq && (!prefill_len || !prefill_sel)) || (n_entries && (!entry_metas || !decode_sel))) {
    moe_set_error("moe_oracle_load: bad argument");
    return MOE_EINVAL;
  }
  const int L = eng->cfg.num_layer, E = eng->cfg.num_expert;
  SpinGuard lk(eng->mu);
  std::vector<int64_t> reply_len(n_seq, 0);
  for (int64_t i = 0; i < n_entries; ++i) {
    const int64_t s = entry_metas[2 * i];
    if (s < 0 || s >= n_seq) { moe_set_error("moe_oracle_load: entry %lld names sequence %lld", (long long)i, (long long)s); return MOE_EINVAL; }
    reply_len[s]++;
  }
  int64_t begin = 0;
  for (int64_t s = 0; s < n_seq; ++s) {
    SeqOracle &so = eng->oracles[(uint64_t)s];
    so.use_times.clear();
    for (auto &e : eng->experts) so.use_times[e.get()];
    int64_t time = 0;
    for (int l = 0; l < L; ++l) {
      const int32_t len = prefill_len[s * L + l];
      for (int32_t o = 0; o < len && o < max_prefill_len; ++o) {
        const int32_t id = prefill_sel[(s * L + l) * max_prefill_len + o];
        if (id < 0 || id >= E) { moe_set_error("moe_oracle_load: bad expert id"); return MOE_EINVAL; }
        so.use_times[eng->ex(l, id)].push_back(time);
      }
      time++;
    }
    for (int64_t r = 0; r < reply_len[s]; ++r) {
      const int64_t row = begin + r;
      if (entry_metas[2 * row] != s || entry_metas[2 * row + 1] != r) {
        moe_set_error("moe_oracle_load: entries must be grouped by sequence in token order (row %lld)", (long long)row);
        return MOE_EINVAL;
      }
      for (int l = 0; l < L; ++l) {
        for (int64_t o = 0; o < k; ++o) {
          const int32_t id = decode_sel[(row * L + l) * k + o];
          if (id < 0 || id >= E) { moe_set_error("moe_oracle_load: bad expert id"); return MOE_EINVAL; }
          so.use_times[eng->ex(l, id)].push_back(time);
        }
        time++;
      }
    }
    begin += reply_len[s];
    for (auto &kv : so.use_times) kv.second.push_back(std::numeric_limits<int64_t>::max());
  }
  return MOE_OK;
}

extern "C" int moe_set_seq(moe_engine *eng, uint64_t seq_id) {
  ENG_GUARD(eng);
  SpinGuard lk(eng->mu);
  for (auto &g : eng->groups)
    if (int rc = g.policy->set_cur_seq(seq_id)) return rc;
  return MOE_OK;
}

extern "C" int moe_drain(moe_engine *eng) {
  ENG_GUARD(eng);
  if (!eng->launched) return MOE_OK;
  std::unique_lock<std::mutex> lk(eng->mu, std::defer_lock);
  moe_spin_lock(lk);
  eng->cv_work.notify_all();
  eng->cv_state.wait(lk, [&] {
    if (eng->exiting || !eng->fatal.empty()) return true;
    if (eng->current.e || !eng->precise_q.empty()) return false;
    for (auto &q : eng->layer_q) if (!q.empty()) return false;
    return true;
  });
  if (!eng->fatal.empty()) { moe_set_error("engine failed: %s", eng->fatal.c_str()); return MOE_ESTATE; }
  lk.unlock();
  return moe_forward_check_kernels(eng);
}

void engine_drop_seq_releases(moe_engine *eng) {
  SpinGuard lk(eng->mu);
  for (auto &x : eng->experts)
    if (x->seq_ptr) {
      x->seq_ptr = nullptr;
      if (x->status.load() == kUsing) x->status = kReady;
    }
  eng->cv_state.notify_all();
}

extern "C" int moe_streams(moe_engine *eng, void **compute, void **copy) {
  ENG_GUARD(eng);
  if (compute) *compute = eng->be->compute_stream();
  if (copy) *copy = eng->be->copy_stream();
  return MOE_OK;
}

int engine_account_hits(moe_engine *eng, int layer, const moe_unit *units, int n) {
  SpinGuard lk(eng->mu);
  for (int i = 0; i < n; ++i) {
    if (units[i].expert < 0 || units[i].expert >= eng->cfg.num_expert) continue;
    Expert *e = eng->ex(layer, units[i].expert);
    if (!in_cache(eng, e)) continue;
    if (int rc = cache_hit(eng, e, true)) return rc;
    eng->ctr.ready++;
    eng->ctr.activated++;
  }
  return MOE_OK;
}

extern "C" int moe_get_counters(moe_engine *eng, moe_counters *out) {
  if (!eng || !out) { moe_set_error("moe_get_counters: null"); return MOE_EINVAL; }
  if (eng->fw) moe_forward_harvest(eng, true);
  SpinGuard lk(eng->mu);
  *out = eng->ctr;
  return MOE_OK;
}

// prefetcher.cpp:327-402: means over decode (seq_len <= 1) and prefill forwards,
// after skipping the first `skip` prompts.
extern "C" int moe_report(moe_engine *eng, int skip, char *buf, int buflen) {
  if (!eng || !buf || buflen <= 0) { moe_set_error("moe_report: bad argument"); return MOE_EINVAL; }
  SpinGuard lk(eng->mu);
  const size_t n = std::min(eng->s_hit.size(), eng->s_seqlen.size());
  size_t start = n;
  int seen = 0;
  for (size_t i = 0; i < n; ++i)
    if (eng->s_seqlen[i] > 1 && seen++ == skip) { start = i; break; }
  if (skip == 0) start = 0;
  std::string s;
  auto pair = [&](const std::vector<uint64_t> &on, const std::vector<uint64_t> &off, bool decode, const char *stage, const char *what) {
    double a = 0, b = 0; size_t c = 0;
    for (size_t i = start; i < n; ++i)
      if ((eng->s_seqlen[i] <= 1) == decode) { a += on[i]; b += off[i]; ++c; }
    if (c) { a /= c; b /= c; }
    char line[256];
    const char *offname = !strcmp(what, "ready") ? "unready" : (!strcmp(what, "hit") ? "miss" : "prefetch_miss");
    snprintf(line, sizeof line, "%s_stage_%s_cnt:%g\n%s_stage_%s_cnt:%g\n%s_stage_%s_rate:%g\n", stage, what, a, stage, offname, b,
             stage, what, (a + b) > 0 ? a / (a + b) : 0.0);
    s += line;
  };
  for (int d = 1; d >= 0; --d) {
    const char *st = d ? "decode" : "prefill";
    pair(eng->s_ready, eng->s_unready, d, st, "ready");
    pair(eng->s_hit, eng->s_miss, d, st, "hit");
    pair(eng->s_phit, eng->s_pmiss, d, st, "prefetch_hit");
  }
  size_t np = 0, nd = 0;
  double wd = 0, wp = 0;
  for (size_t i = start; i < n; ++i) {
    if (eng->s_seqlen[i] <= 1) { nd++; wd += eng->s_wait[i]; } else { np++; wp += eng->s_wait[i]; }
  }
  char line[256];
  snprintf(line, sizeof line, "decode_stage_wait_time:%g\nprefill_stage_wait_time:%g\nnum_prefill_iter:%zu\nnum_decode_iter:%zu\n",
           nd ? wd / nd / 1000.0 : 0.0, np ? wp / np / 1000.0 : 0.0, np, nd);
  s += line;
  snprintf(buf, buflen, "%s", s.c_str());
  return (int)s.size();
}
