// Host-side stress of the cache engine for the sanitizers (ThreadSanitizer / AddressSanitizer builds,
// see tests/cpp/Makefile): host backend, three threads at work (caller, fetch thread, predictor thread),
// the hook sequence of many decode tokens with random routing, random predictor models, some prefill
// steps in between, policy nn so that priorities are updated from the predictor thread.
// No GPU code is linked: the kernel entry points the engine refers to are stubs that fail (kernel_stubs.cpp).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include <algorithm>

#include "moe_engine.h"

#define CK(call)                                                                         \
  do {                                                                                   \
    const int rc_ = (call);                                                              \
    if (rc_ != 0) { fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, moe_last_error()); return 1; } \
  } while (0)

static uint16_t bf16(float f) { uint32_t u; memcpy(&u, &f, 4); return (uint16_t)(u >> 16); }

int main(int argc, char **argv) {
  const int L = 6, E = 16, K = 3, H = 64, P = 2;
  const int tokens = argc > 1 ? atoi(argv[1]) : 300;
  const std::string policy = argc > 2 ? argv[2] : "nn";
  moe_cfg *cfg = moe_cfg_create(L, E);
  const char *names[P] = {"a", "b"};
  CK(moe_cfg_set_params(cfg, names, P));
  CK(moe_cfg_set(cfg, "num_expert_per_token", "3"));
  CK(moe_cfg_set(cfg, "cache_rate", "0.4"));
  CK(moe_cfg_set(cfg, "cache_policy", policy.c_str()));
  CK(moe_cfg_set(cfg, "num_predict_expert_per_layer", "3"));
  CK(moe_cfg_set(cfg, "layer_predict_interval", "1"));
  CK(moe_cfg_set(cfg, "layer_predict_max_window", "3"));
  CK(moe_cfg_set(cfg, "limit_layer_0_window", "3"));
  CK(moe_cfg_finalize(cfg));
  moe_engine *eng = nullptr;
  CK(moe_engine_create(cfg, MOE_BACKEND_HOST, nullptr, &eng));
  std::vector<std::vector<uint8_t>> bufs;
  for (int l = 0; l < L; ++l)
    for (int e = 0; e < E; ++e)
      for (int p = 0; p < P; ++p) {
        bufs.emplace_back(256, (uint8_t)(l * E + e));
        CK(moe_register_param(eng, l, e, p, bufs.back().data(), bufs.back().size(), 0));
      }
  CK(moe_init_slots(eng));
  CK(moe_launch(eng));
  std::mt19937 rng(7);
  std::normal_distribution<float> nd(0.f, 1.f);
  std::vector<int> first(L + 1), last(L + 1);
  CK(moe_predictor_windows(eng, first.data(), last.data()));
  std::vector<std::vector<uint16_t>> models;
  for (int src = 0; src <= L; ++src)
    for (int dst = first[src]; dst < last[src]; ++dst) {
      models.emplace_back((size_t)E * H);
      for (auto &v : models.back()) v = bf16(nd(rng));
      CK(moe_predictor_set_model(eng, src, dst, models.back().data(), nullptr, H));
    }
  CK(moe_predictor_start(eng));
  std::vector<uint16_t> x(H);
  std::vector<int64_t> ids;
  for (int t = 0; t < tokens; ++t) {
    const bool prefill = t % 17 == 5;
    const int S = prefill ? 9 : 1;
    for (int l = 0; l < L; ++l) {
      for (auto &v : x) v = bf16(nd(rng));
      CK(moe_report_layer_logits(eng, l, prefill ? nullptr : x.data(), 1, S, H));
      ids.clear();
      const int n = prefill ? 8 : K;
      std::vector<int> perm(E);
      for (int e = 0; e < E; ++e) perm[e] = e;
      std::shuffle(perm.begin(), perm.end(), rng);
      for (int i = 0; i < n; ++i) ids.push_back(perm[i]);
      std::sort(ids.begin(), ids.end());
      CK(moe_report_one_layer(eng, l, ids.data(), (int64_t)ids.size()));
      for (int64_t e : ids) {
        CK(moe_wait_expert(eng, l, (int)e));
        void *p0 = nullptr;
        CK(moe_expert_param_ptr(eng, l, (int)e, 0, &p0));
        if (!p0 || *(uint8_t *)p0 != (uint8_t)(l * E + e)) { fprintf(stderr, "slot of %d.%d holds the wrong bytes\n", l, (int)e); return 1; }
        CK(moe_expert_launched(eng, l, (int)e));
      }
      CK(moe_layer_done(eng, l));
    }
    if (t % 50 == 49) CK(moe_drain(eng));
  }
  CK(moe_drain(eng));
  moe_counters c;
  CK(moe_get_counters(eng, &c));
  uint64_t jobs = 0, reqs = 0;
  CK(moe_predictor_stats(eng, &jobs, &reqs));
  printf("tokens %d policy %s: hit %llu miss %llu prefetch_hit %llu prefetch_miss %llu evictions %llu, predictor jobs %llu requests %llu\n",
         tokens, policy.c_str(), (unsigned long long)c.hit, (unsigned long long)c.miss, (unsigned long long)c.prefetch_hit,
         (unsigned long long)c.prefetch_miss, (unsigned long long)c.evictions, (unsigned long long)jobs, (unsigned long long)reqs);
  if (reqs != (uint64_t)tokens * L) { fprintf(stderr, "expected %d requests\n", tokens * L); return 1; }
  moe_engine_destroy(eng);
  moe_cfg_destroy(cfg);
  return 0;
}
