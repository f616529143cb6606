"""CPU restatement of the reference's expert-cache logic (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.

Single-threaded, synchronous model of huwf5/promoe's cache manager, eviction
policies and fetch scheduler: every queued copy completes, in queue order, when
`drain()` runs.  That is the behaviour of the reference whenever its fetch thread
has caught up with the caller, which is the only regime whose results do not
depend on thread timing; the tests drive the engine into the same regime.

Reference sources restated (paths under src/cpp_worker/):
  slot distribution ............ cache.cpp:9-94 (bi_traverse, init_gpu_mem_buffer)
  cache_len ..................... prefetcher.cpp:162-177
  CacheMngr::hit / miss ......... cache.cpp:229-312
  FIFO / LRU / Static / NN / MIN  cache.hpp:24-224, cache.cpp:313-399,490-583
  MinHeap ....................... utils.hpp:273-361
  CacheOracle::load_from_tensor . cache.cpp:592-644
  reorder_experts ............... prefetcher.cpp:6-42
  preempt_one_layer/_expert ..... prefetcher.cpp:44-125
  pop_next_task / send_one_job .. prefetcher.cpp:143-161, 613-659
  FetchDone ..................... prefetcher.cpp:556-570
  PrefetchLayerTask ............. prefetcher.cpp:585-611
  wait_expert counters .......... prefetcher.cpp:241-260
  ExpertStatus .................. utils.hpp:38-49

Pinning: bi_traverse / distribution against hand-derived answers from the source
(G=5 -> [0,1,3,4,2]; 648 over 27 -> 24 each; 128 over 32 -> 4 each) and the
max-min<=1 invariant; LRU/FIFO against textbook deque models; MIN against
brute-force Belady on small traces; NN against a sorted-by-priority model; the
reference holds no golden vectors for this path (its only committed results,
eval/demo-simulate/output.csv, need an external trace).
"""
from __future__ import annotations

import math
from collections import deque

import numpy as np

IDLE, FETCHING, READY, LAUNCHING, USING = range(5)
INT64_MAX = (1 << 63) - 1
FLT_MIN = float(np.finfo(np.float32).tiny)


# ---------------------------------------------------------------- slot arithmetic
def bi_traverse(arr, begin, end, ret):
    if begin == end:
        return
    q = deque([(begin, end)])
    while q:
        l, r = q.popleft()
        if l == r:
            continue
        if r - l == 1:
            if not q:
                ret.append(arr[l])
                return
            rest = list(arr[l:r])
            while q:
                l2, r2 = q.popleft()
                rest.extend(arr[l2:r2])
            bi_traverse(rest, 0, len(rest), ret)
            return
        mid = (l + r) // 2
        ret.append(arr[mid])
        if l < mid:
            q.append((l, mid))
        if mid + 1 < r:
            q.append((mid + 1, r))


def remainder_order(n_groups: int):
    cand = list(range(n_groups))
    if n_groups > 2:
        order = [0, 1]
        bi_traverse(cand, 2, n_groups, order)
        return order
    return cand


def slot_distribution(num_buffers: int, n_groups: int):
    base, rem = divmod(num_buffers, n_groups)
    out = [0] * n_groups
    for i, g in enumerate(remainder_order(n_groups)):
        out[g] = base + (1 if i < rem else 0)
    assert max(out) - min(out) <= 1
    return out


def cache_len(cache_rate: float, num_layer: int, num_expert: int) -> int:
    """round(cache_rate * L * E) evaluated in float32 like the reference's expression."""
    v = np.float32(np.float32(np.float32(cache_rate) * np.float32(num_layer)) * np.float32(num_expert))
    return int(math.floor(float(v) + 0.5))


# ---------------------------------------------------------------- min-heap (utils.hpp:273-361)
class MinHeap:
    def __init__(self):
        self.buf = []  # nodes: [priority, idx, key]

    def _swap(self, i, j):
        b = self.buf
        b[i], b[j] = b[j], b[i]
        b[i][1], b[j][1] = i, j

    def down(self, i):
        b = self.buf
        while True:
            l, r, s = 2 * i + 1, 2 * i + 2, i
            if l < len(b) and b[l][0] < b[s][0]:
                s = l
            if r < len(b) and b[r][0] < b[s][0]:
                s = r
            if s == i:
                return
            self._swap(i, s)
            i = s

    def up(self, i):
        b = self.buf
        while i > 0:
            p = (i - 1) // 2
            if b[p][0] > b[i][0]:
                self._swap(p, i)
                i = p
            else:
                break

    def push(self, node):
        node[1] = len(self.buf)
        self.buf.append(node)
        self.up(node[1])

    def update(self, node, p):
        o = node[0]
        node[0] = p
        if p < o:
            self.up(node[1])
        else:
            self.down(node[1])

    def remove(self, node):
        i = node[1]
        self._swap(i, len(self.buf) - 1)
        self.buf.pop()
        if i < len(self.buf):
            self.down(i)

    def rebuild(self):
        for i in range(len(self.buf) // 2, -1, -1):
            if i < len(self.buf):
                self.down(i)

    def front(self):
        return self.buf[0][2]


f32 = lambda x: float(np.float32(x))


# ---------------------------------------------------------------- policies
class PolicyFIFO:
    def __init__(self, sim):
        self.q = deque()

    def select(self):
        return self.q[0]

    def evict(self, e):
        assert self.q[0] == e
        self.q.popleft()

    def on_hit(self, e, precise):
        pass

    def on_miss(self, e, precise):
        self.q.append(e)

    def update_priority(self, e, p):
        pass


class PolicyLRU(PolicyFIFO):
    def evict(self, e):
        self.q.remove(e)

    def on_hit(self, e, precise):
        self.q.remove(e)
        self.q.append(e)

    def on_miss(self, e, precise):
        assert e not in self.q
        self.q.append(e)


class PolicyStatic:
    def __init__(self, sim, n):
        self.n, self.q, self.persisted = n, deque(), set()

    def select(self):
        return self.q[0]

    def evict(self, e):
        assert e in self.q and e not in self.persisted
        self.q.remove(e)

    def on_hit(self, e, precise):
        assert e in self.q or e in self.persisted

    def on_miss(self, e, precise):
        assert e not in self.q and e not in self.persisted
        if len(self.q) == self.n:
            self.persisted.add(self.q.popleft())
        self.q.append(e)

    def update_priority(self, e, p):
        pass


class PolicyNN:
    def __init__(self, sim):
        self.sim, self.heap, self.map = sim, MinHeap(), {}

    def select(self):
        return self.heap.front()

    def evict(self, e):
        self.heap.remove(self.map.pop(e))

    def on_hit(self, e, precise):
        assert e in self.map

    def on_miss(self, e, precise):
        assert e not in self.map
        node = [f32(self.sim.priority[e]), 0, e]
        self.map[e] = node
        self.heap.push(node)

    def update_all(self):
        for e, node in self.map.items():
            node[0] = f32(self.sim.priority[e])
        self.heap.rebuild()

    def update_priority(self, e, p):
        if e in self.map:
            self.heap.update(self.map[e], f32(p))


class PolicyMIN:
    def __init__(self, sim):
        self.sim, self.heap, self.map = sim, MinHeap(), {}
        self.cur, self.now, self.next_idx = None, -1, {}

    def select(self):
        return self.heap.front()

    def evict(self, e):
        self.heap.remove(self.map.pop(e))

    def set_cur_seq(self, seq):
        self.cur = self.sim.oracles[seq]
        self.now = -1
        for e in self.next_idx:
            self.next_idx[e] = 0
        for e, node in self.map.items():
            node[0] = f32(-self.cur[e][0])
        self.heap.rebuild()

    def _advance(self, e, precise):
        ut = self.cur[e]
        i = self.next_idx.setdefault(e, 0)
        if precise:
            assert i < len(ut) and self.now <= ut[i], "out-of-order access"
            self.now = ut[i]
            i += 1
            self.next_idx[e] = i
        return f32(-ut[i])

    def on_hit(self, e, precise):
        self.heap.update(self.map[e], self._advance(e, precise))

    def on_miss(self, e, precise):
        p = self._advance(e, precise)
        assert e not in self.map
        node = [p, 0, e]
        self.map[e] = node
        self.heap.push(node)

    def update_priority(self, e, p):
        pass


def load_oracle(L, E, entry_metas, prefill_len, prefill_sel, decode_sel):
    """use_times[(l,e)] per sequence (cache.cpp:592-644)."""
    entry_metas = np.asarray(entry_metas).reshape(-1, 2)
    n_seq = len(prefill_len)
    reply_len = np.bincount(entry_metas[:, 0], minlength=n_seq) if len(entry_metas) else np.zeros(n_seq, int)
    out, begin = {}, 0
    for s in range(n_seq):
        ut = {(l, e): [] for l in range(L) for e in range(E)}
        time = 0
        for l in range(L):
            for o in range(int(prefill_len[s][l])):
                ut[(l, int(prefill_sel[s][l][o]))].append(time)
            time += 1
        for r in range(int(reply_len[s])):
            for l in range(L):
                for o in range(np.asarray(decode_sel).shape[2]):
                    ut[(l, int(decode_sel[begin + r][l][o]))].append(time)
                time += 1
        begin += int(reply_len[s])
        for v in ut.values():
            v.append(INT64_MAX)
        out[s] = ut
    return out


def predict_layer_mapping(L, interval, window, limit_layer_0_window, cross_token):
    """Destination layers [first, last) each source layer 0..L predicts (predictor.cpp:8-46)."""
    pl = [0] * (L + 1)
    stop = 0
    for l in range(0, L, max(interval, 1)):
        w = window
        if l == 0 and limit_layer_0_window != -1:
            w = limit_layer_0_window
        pl[l] = stop
        pl[l + 1] = min(l % L + w, L)
        stop = pl[l + 1]
    for l in range(1, L + 1):
        if pl[l] < pl[l - 1]:
            pl[l] = pl[l - 1]
    ret = [(pl[l], pl[l + 1]) for l in range(L)] + [(0, 0)]
    if cross_token:
        ret[L] = ret[0]
        ret[0] = (0, 0)
    return ret


# ---------------------------------------------------------------- cache + scheduler
class CacheSim:
    """Experts are keyed (layer, expert)."""

    def __init__(self, L, E, P, k, cache_rate=0.5, policy="lru", per_layer_cache=True,
                 num_predict=-1, reorder=None, early_preempt=None, chunk_prefetch=None,
                 promote_hit_in_prefetch=True, max_prefetch_layer_distance=-1,
                 limit_layer_0_num_predict=-1):
        self.L, self.E, self.P, self.k = L, E, P, k
        if num_predict == -1:
            num_predict = k
        pf = num_predict > 0
        self.reorder = pf if reorder is None else reorder
        self.early_preempt = pf if early_preempt is None else early_preempt
        self.chunk_prefetch = pf if chunk_prefetch is None else chunk_prefetch
        self.promote = promote_hit_in_prefetch
        self.policy_name = policy
        self.per_layer = per_layer_cache
        self.limit0 = limit_layer_0_num_predict
        G = L if per_layer_cache else 1
        self.cache_len = min(cache_len(cache_rate, L, E), L * E)
        self.group_len = slot_distribution(self.cache_len, G)
        self.num_predict = min(num_predict, self.group_len[0])
        self.unused, nxt = [], 0
        for g in range(G):
            self.unused.append(list(range(nxt, nxt + self.group_len[g])))
            nxt += self.group_len[g]
        mk = {"fifo": PolicyFIFO, "lru": PolicyLRU, "nn": PolicyNN, "min": PolicyMIN,
              "static-1": lambda s: PolicyStatic(s, 1), "static-2": lambda s: PolicyStatic(s, 2)}[policy]
        self.policies = [mk(self) for _ in range(G)]
        self.priority = {(l, e): 0.0 for l in range(L) for e in range(E)}
        self.max_priority = FLT_MIN
        self.oracles = {}
        self.slot = {}                       # resident expert -> slot (prefetched_experts)
        self.status = {k_: IDLE for k_ in self.priority}
        self.num_ready = {k_: 0 for k_ in self.priority}
        self.precise_q, self.layer_q = deque(), [deque() for _ in range(L)]
        self.current = None
        self.ctr = dict(hit=0, miss=0, ready=0, unready=0, prefetch_hit=0, prefetch_miss=0,
                        activated=0, evictions=0, h2d_copies=0)
        self.budget = (L - 1) if max_prefetch_layer_distance == -1 else max_prefetch_layer_distance
        self.evicted_log = []
        self.blocked_on = None

    def g(self, layer):
        return layer if self.per_layer else 0

    def in_cache(self, e):
        return e in self.slot

    # CacheMngr::hit / miss
    def cache_hit(self, e, precise):
        self.ctr["hit" if precise else "prefetch_hit"] += 1
        pol = self.policies[self.g(e[0])]
        pol.on_hit(e, precise)
        if precise:
            self.max_priority = f32(self.max_priority + 1)
            pol.update_priority(e, self.max_priority)
            if self.policy_name == "nn":
                self.priority[e] = self.max_priority

    def cache_miss(self, e, precise):
        self.ctr["miss" if precise else "prefetch_miss"] += 1
        gi = self.g(e[0])
        pol = self.policies[gi]
        if precise:
            self.max_priority = f32(self.max_priority + 1)
            if self.policy_name == "nn":
                self.priority[e] = self.max_priority
        if self.unused[gi]:
            self.slot[e] = self.unused[gi].pop()
            pol.on_miss(e, precise)
            return None
        v = pol.select()
        assert v != e
        pol.evict(v)
        pol.on_miss(e, precise)
        self.slot[e] = self.slot.pop(v)
        self.ctr["evictions"] += 1
        self.evicted_log.append(v)
        self.num_ready[v] = 0
        if self.status[v] == LAUNCHING:
            # acquired by the caller but not launched yet: the copy into its slot has to wait
            # until the caller is past it (cache.cpp:291-297); `using` resolves at once here
            # because every event of this model has already fired
            return v
        self.status[v] = IDLE
        return None

    # scheduler
    def _add(self, q, e, start, stop, precise):
        q.append(dict(e=e, start=start, stop=stop, precise=precise))

    def _make_launching(self, e):
        assert self.status[e] in (READY, USING, LAUNCHING), (e, self.status[e])
        self.status[e] = LAUNCHING

    def reorder_experts(self, layer, ids):
        done, going, partial, miss = [], [], [], []
        for i in ids:
            e = (layer, int(i))
            if self.current is not None and self.current["e"] == e:
                going.append(i)
            elif self.in_cache(e):
                (done if self.num_ready[e] == self.P else partial).append(i)
            else:
                miss.append(i)
        return done + going + partial + miss

    def _preempt_resident(self, e):
        if self.num_ready[e] == self.P:
            self._make_launching(e)
            self.cache_hit(e, True)
        elif self.current is not None and self.current["e"] == e:
            self.current["precise"] = True
            if self.current["stop"] == self.P:
                self.cache_hit(e, True)
            else:
                self._add(self.precise_q, e, self.current["stop"], self.P, True)
        else:
            self._add(self.precise_q, e, self.num_ready[e], self.P, True)

    def preempt_one_expert(self, layer, i):
        e = (layer, int(i))
        if not self.in_cache(e):
            self._add(self.precise_q, e, 0, self.P, True)
        else:
            self._preempt_resident(e)

    def preempt_one_layer(self, layer, ids):
        preceding = True
        for i in ids:
            e = (layer, int(i))
            if not self.in_cache(e):
                preceding = False
                self._add(self.precise_q, e, 0, self.P, True)
            elif not preceding:
                self._add(self.precise_q, e, 0, self.P, True)
            else:
                self._preempt_resident(e)

    def report_one_layer(self, layer, ids):
        ids = [int(i) for i in ids]
        if self.reorder:
            ids = self.reorder_experts(layer, ids)
        if self.early_preempt:
            self.preempt_one_layer(layer, ids)
            self.budget += 1
        self.layer_q[layer].clear()
        self.ctr["activated"] += len(ids)
        return ids

    def send_one_job(self, t):
        e = t["e"]
        if e not in self.slot:
            assert t["start"] == 0 and self.num_ready[e] == 0
            self.blocked_on = self.cache_miss(e, t["precise"])
            assert self.status[e] == IDLE
            self.status[e] = FETCHING
        else:
            if t["precise"] or t["start"] == 0:
                self.cache_hit(e, t["precise"])
            if self.num_ready[e] >= t["stop"]:
                if t["precise"]:
                    assert self.num_ready[e] == self.P
                    if self.status[e] in (READY, USING):
                        self.status[e] = LAUNCHING
                return False
            elif self.num_ready[e] > t["start"]:
                t["start"] = self.num_ready[e]
            else:
                assert self.num_ready[e] == t["start"]
        self.current = t
        return True

    def fetch_done(self):
        t = self.current
        e = t["e"]
        self.ctr["h2d_copies"] += t["stop"] - t["start"]
        self.num_ready[e] = t["stop"]
        if t["stop"] == self.P:
            assert self.status[e] == FETCHING
            self.status[e] = LAUNCHING if t["precise"] else READY
        self.current = None

    def drain(self, until=None):
        """Run the fetch thread's loop until it has nothing to do, is blocked on a victim
        the caller still has to launch, or (until=e) expert e became usable."""
        while True:
            if until is not None and self.status[until] == LAUNCHING:
                return
            if self.current is not None:          # a copy waiting for its victim
                v = self.blocked_on
                if self.status[v] == LAUNCHING:
                    return
                self.status[v] = IDLE
                self.blocked_on = None
                self.fetch_done()
                continue
            if self.precise_q:
                t = self.precise_q.popleft()
            else:
                t = None
                for q in self.layer_q:
                    if q:
                        t = q.popleft()
                        break
                if t is None:
                    return
            if self.send_one_job(t):
                if self.blocked_on is not None:
                    continue
                self.fetch_done()

    def wait_expert(self, layer, i):
        e = (layer, int(i))
        if not self.early_preempt:
            self.preempt_one_expert(layer, i)
        if self.status[e] == LAUNCHING:
            self.ctr["ready"] += 1
        else:
            self.ctr["unready"] += 1
            self.drain(until=e)
            assert self.status[e] == LAUNCHING, (e, self.status[e])

    def expert_launched(self, layer, i):
        e = (layer, int(i))
        assert self.status[e] == LAUNCHING
        self.status[e] = USING

    def layer_done(self, layer):
        if not self.early_preempt:
            self.budget += 1

    def prefetch_layer(self, layer, ids):
        if self.budget <= 0:
            return False
        self.budget -= 1
        assert not self.layer_q[layer]
        ids = [int(i) for i in ids]
        if layer == 0 and self.limit0 != -1:
            ids = ids[: self.limit0]
        for i in ids:
            e = (layer, i)
            if self.promote and self.in_cache(e):
                self.cache_hit(e, False)
            if self.chunk_prefetch:
                for j in range(self.P):
                    self._add(self.layer_q[layer], e, j, j + 1, False)
            else:
                self._add(self.layer_q[layer], e, 0, self.P, False)
        return True

    def update_priority(self, p, starting_layer=0):
        p = np.asarray(p, np.float32)
        for dl in range(p.shape[0]):
            for e in range(self.E):
                self.priority[(starting_layer + dl, e)] = float(p[dl, e])
        self.max_priority = f32(max(self.priority.values()))
        groups = {self.g(starting_layer + dl) for dl in range(p.shape[0])}
        if p.shape[0] == self.L:
            groups = set(range(len(self.policies)))
        for gi in groups:
            self.policies[gi].update_all()

    def set_cur_seq(self, seq):
        for pol in self.policies:
            pol.set_cur_seq(seq)

    def resident(self, layer):
        return sorted(e[1] for e in self.slot if e[0] == layer)
