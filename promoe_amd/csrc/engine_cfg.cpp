// Configuration object of the engine: the key/value surface of the reference's
// ModuleMeta (utils.hpp:127-192; parsing rules utils.cpp:54-273).
#include "engine_internal.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>

namespace {

std::string lower(std::string s) {
  std::transform(s.begin(), s.end(), s.begin(), ::tolower);
  return s;
}
bool is_on(const std::string &s) {
  const std::string l = lower(s);
  return l == "on" || l == "true" || l == "1";
}

// llama.cpp dialect (utils.cpp:147-172)
const std::map<std::string, std::string> &dialects() {
  static const std::map<std::string, std::string> d = {
      {"cross_token_pred", "layer_predict_replace_first_input_with_last_output"},
      {"predict_using_last_token_output", "layer_predict_replace_first_input_with_last_output"},
      {"num_predict", "num_predict_expert_per_layer"},
      {"predict_interval", "layer_predict_interval"},
      {"predict_window", "layer_predict_max_window"},
      {"moe_cache_policy", "cache_policy"},
      {"moe_cache_rate", "cache_rate"},
      {"pred_model_path", "predictor_model_path"},
  };
  return d;
}

const char *kKnownKeys[] = {"model_arch_string", "num_expert_per_token", "cache_rate",
                            "num_predict_expert_per_layer", "reorder_experts", "early_preempt",
                            "chunk_prefetch", "predict_input_mode", "predictor_type",
                            "predictor_model_path", "layer_predict_interval",
                            "layer_predict_max_window",
                            "layer_predict_replace_first_input_with_last_output",
                            "limit_layer_0_window", "limit_layer_0_num_predict",
                            "max_prefetch_layer_distance", "cache_only", "per_layer_cache",
                            "promote_hit_in_prefetch", "cache_policy",
                            "predict_input_reuse_distance_max", "predict_input_decay"};

const char *kPredictModes[] = {"no_predict", "one_token", "decode_cumsum", "last_use_distance",
                               "weighted_decode_cumsum", "first_moe_attn_input_logits",
                               "moe_attn_input_logits", "moe_layer_logits"};
const char *kPolicies[] = {"lru", "fifo", "nn", "min", "static-1", "static-2"};

}  // namespace

std::string moe_translate_key(const std::string &key_in) {
  std::string key = key_in;
  std::replace(key.begin(), key.end(), '-', '_');
  auto it = dialects().find(key);
  return it == dialects().end() ? key : it->second;
}

extern "C" moe_cfg *moe_cfg_create(int num_layer, int num_expert) {
  if (num_layer <= 0 || num_expert <= 0) {
    moe_set_error("moe_cfg_create: num_layer and num_expert must be positive");
    return nullptr;
  }
  moe_cfg *c = new moe_cfg();
  c->num_layer = num_layer;
  c->num_expert = num_expert;
  return c;
}

extern "C" void moe_cfg_destroy(moe_cfg *cfg) { delete cfg; }

extern "C" int moe_cfg_set(moe_cfg *cfg, const char *key, const char *value) {
  if (!cfg || !key || !value) { moe_set_error("moe_cfg_set: null argument"); return MOE_EINVAL; }
  if (cfg->finalized) { moe_set_error("moe_cfg_set: configuration already finalized"); return MOE_ESTATE; }
  const std::string k = moe_translate_key(key);
  if (cfg->staged.count(k)) {
    moe_set_error("duplicate config key %s", k.c_str());  // utils.cpp:165-168
    return MOE_EINVAL;
  }
  cfg->staged[k] = value;
  return MOE_OK;
}

extern "C" int moe_cfg_set_params(moe_cfg *cfg, const char *const *names, int n) {
  if (!cfg || (n > 0 && !names) || n < 0) { moe_set_error("moe_cfg_set_params: bad argument"); return MOE_EINVAL; }
  cfg->param_names.clear();
  for (int i = 0; i < n; ++i) cfg->param_names.push_back(names[i] ? names[i] : "");
  cfg->num_per_expert_param = n;
  return MOE_OK;
}

extern "C" int moe_cfg_finalize(moe_cfg *cfg) {
  if (!cfg) { moe_set_error("moe_cfg_finalize: null"); return MOE_EINVAL; }
  if (cfg->finalized) return MOE_OK;
  auto m = cfg->staged;
  bool bad = false;
  auto is_default = [](const std::string &v) { return v == "None" || v.empty(); };
  auto opt_str = [&](const char *key, const std::string &def) -> std::string {
    auto it = m.find(key);
    if (it == m.end()) return def;
    std::string v = it->second;
    m.erase(it);
    return is_default(v) ? def : v;
  };
  auto opt_int = [&](const char *key, int def) -> int {
    const std::string v = opt_str(key, std::to_string(def));
    char *end = nullptr;
    long r = strtol(v.c_str(), &end, 10);
    if (end == v.c_str()) { moe_set_error("invalid key %s with value %s", key, v.c_str()); bad = true; return def; }
    return (int)r;
  };
  auto opt_float = [&](const char *key, float def) -> float {
    const std::string v = opt_str(key, std::to_string(def));
    char *end = nullptr;
    float r = strtof(v.c_str(), &end);
    if (end == v.c_str()) { moe_set_error("invalid key %s with value %s", key, v.c_str()); bad = true; return def; }
    return r;
  };
  auto opt_bool = [&](const char *key, bool def) -> bool { return is_on(opt_str(key, def ? "true" : "false")); };

  cfg->model_arch_string = opt_str("model_arch_string", cfg->model_arch_string);
  {
    auto it = m.find("num_expert_per_token");
    if (it == m.end()) { moe_set_error("required key num_expert_per_token not found"); return MOE_EINVAL; }
    if (is_default(it->second)) {
      moe_set_error("required key num_expert_per_token is %s, should be a non-empty string", it->second.c_str());
      return MOE_EINVAL;
    }
    cfg->num_expert_per_token = opt_int("num_expert_per_token", 0);
    if (bad) return MOE_EINVAL;
    if (cfg->num_expert_per_token <= 0 || cfg->num_expert_per_token > cfg->num_expert) {
      moe_set_error("num_expert_per_token=%d out of range", cfg->num_expert_per_token);
      return MOE_EINVAL;
    }
  }
  cfg->cache_rate = opt_float("cache_rate", cfg->cache_rate);
  cfg->num_predict_expert_per_layer = opt_int("num_predict_expert_per_layer", cfg->num_predict_expert_per_layer);
  if (cfg->num_predict_expert_per_layer == -1) cfg->num_predict_expert_per_layer = cfg->num_expert_per_token;
  const bool pf = cfg->num_predict_expert_per_layer > 0;
  cfg->reorder_experts = opt_bool("reorder_experts", pf);
  cfg->early_preempt = opt_bool("early_preempt", pf);
  cfg->chunk_prefetch = opt_bool("chunk_prefetch", pf);

  cfg->predict_input_mode_str = opt_str("predict_input_mode", cfg->predict_input_mode_str);
  cfg->predict_input_mode = -1;
  for (int i = 0; i < 8; ++i)
    if (cfg->predict_input_mode_str == kPredictModes[i]) cfg->predict_input_mode = i;
  if (cfg->predict_input_mode < 0) {
    moe_set_error("unknown predict_input_mode %s", cfg->predict_input_mode_str.c_str());
    return MOE_EINVAL;
  }
  cfg->predictor_type_str = opt_str("predictor_type", cfg->predictor_type_str);
  if (cfg->predictor_type_str != "legacy" && cfg->predictor_type_str != "sep") {
    moe_set_error("unknown predictor_type %s", cfg->predictor_type_str.c_str());
    return MOE_EINVAL;
  }
  cfg->predictor_model_path = opt_str("predictor_model_path", cfg->predictor_model_path);
  cfg->layer_predict_interval = opt_int("layer_predict_interval", cfg->layer_predict_interval);
  cfg->layer_predict_max_window = opt_int("layer_predict_max_window", cfg->layer_predict_max_window);
  cfg->cross_token_pred = opt_bool("layer_predict_replace_first_input_with_last_output", cfg->cross_token_pred);
  cfg->limit_layer_0_window = opt_int("limit_layer_0_window", cfg->limit_layer_0_window);
  cfg->limit_layer_0_num_predict = opt_int("limit_layer_0_num_predict", cfg->limit_layer_0_num_predict);
  cfg->max_prefetch_layer_distance = opt_int("max_prefetch_layer_distance", cfg->max_prefetch_layer_distance);
  cfg->cache_only = opt_bool("cache_only", cfg->cache_only);
  cfg->per_layer_cache = opt_bool("per_layer_cache", cfg->per_layer_cache);
  cfg->promote_hit_in_prefetch = opt_bool("promote_hit_in_prefetch", cfg->promote_hit_in_prefetch);
  cfg->cache_policy = opt_str("cache_policy", cfg->cache_policy);
  cfg->predict_input_reuse_distance_max = opt_int("predict_input_reuse_distance_max", cfg->predict_input_reuse_distance_max);
  cfg->predict_input_decay = opt_int("predict_input_decay", cfg->predict_input_decay);
  if (bad) return MOE_EINVAL;

  if (!m.empty()) {  // utils.cpp:137-144
    std::string all;
    for (auto &kv : m) all += kv.first + " = " + kv.second + "; ";
    moe_set_error("unrecognized configs: %s", all.c_str());
    return MOE_EINVAL;
  }
  bool okp = false;
  for (const char *p : kPolicies) okp |= cfg->cache_policy == p;
  if (!okp) { moe_set_error("unknown cache_policy %s", cfg->cache_policy.c_str()); return MOE_EINVAL; }
  if (!(cfg->cache_rate >= 0.f)) { moe_set_error("cache_rate must be >= 0"); return MOE_EINVAL; }

  // handle_uninited_configs (utils.cpp:222-273)
  if (cfg->max_prefetch_layer_distance == -1) cfg->max_prefetch_layer_distance = cfg->num_layer - 1;
  if (const char *e = getenv("SPARSE_CACHE_PHYSICAL_MEM_IMPL")) cfg->physical_mem_impl = e;
  if (const char *e = getenv("SPARSE_CACHE_LOGICAL_MEM_IMPL")) cfg->logical_mem_impl = e;
  if (const char *e = getenv("SPARSE_CACHE_SLEEP_ON_REPORT_LOGITS_US")) cfg->sleep_on_report_logits_us = (unsigned)strtoul(e, nullptr, 10);
  if (const char *e = getenv("SPARSE_CACHE_EXPERT_MEM_SCALE")) cfg->expert_mem_scale = strtof(e, nullptr);
  cfg->model_arch_string = lower(cfg->model_arch_string);
  if (cfg->limit_layer_0_window == -1)
    cfg->limit_layer_0_window = cfg->model_arch_string.find("deepseek") != std::string::npos
                                    ? cfg->layer_predict_max_window : 1;
  {
    // physical slot pool implementation: the reference's names map onto the two pools here
    const std::string &p = cfg->physical_mem_impl;
    if (p == "tensor" || p == "tensor_unified" || p == "tensor_global_unified" || p == "slab") cfg->pool_vmm = false;
    else if (p == "cudriver" || p == "cudriver_unified" || p == "vmm") cfg->pool_vmm = true;
    else { moe_set_error("unknown physical_mem_impl %s", p.c_str()); return MOE_EINVAL; }
  }
  if (cfg->expert_mem_scale != 1.0f) {
    if (!(cfg->expert_mem_scale > 1.0f)) { moe_set_error("expert_mem_scale must be > 1"); return MOE_EINVAL; }
    cfg->num_dummy_params = (int)std::ceil(cfg->num_per_expert_param * (cfg->expert_mem_scale - 1));
    for (int i = 0; i < cfg->num_dummy_params; ++i) cfg->param_names.push_back("dummy-" + std::to_string(i));
    cfg->num_per_expert_param += cfg->num_dummy_params;
  }
  if (cfg->num_per_expert_param <= 0) { moe_set_error("no per-expert parameter list (moe_cfg_set_params)"); return MOE_EINVAL; }
  cfg->finalized = true;
  return MOE_OK;
}

extern "C" int moe_cfg_get(const moe_cfg *cfg, const char *key_in, char *buf, int buflen) {
  if (!cfg || !key_in || !buf || buflen <= 0) { moe_set_error("moe_cfg_get: bad argument"); return MOE_EINVAL; }
  const std::string key = moe_translate_key(key_in);
  std::string v;
  auto b = [](bool x) { return std::string(x ? "true" : "false"); };
  if (key == "num_layer") v = std::to_string(cfg->num_layer);
  else if (key == "num_expert") v = std::to_string(cfg->num_expert);
  else if (key == "model_arch_string") v = cfg->model_arch_string;
  else if (key == "num_expert_per_token") v = std::to_string(cfg->num_expert_per_token);
  else if (key == "cache_rate") v = std::to_string(cfg->cache_rate);
  else if (key == "num_predict_expert_per_layer") v = std::to_string(cfg->num_predict_expert_per_layer);
  else if (key == "reorder_experts") v = b(cfg->reorder_experts);
  else if (key == "early_preempt") v = b(cfg->early_preempt);
  else if (key == "chunk_prefetch") v = b(cfg->chunk_prefetch);
  else if (key == "predict_input_mode") v = cfg->predict_input_mode_str;
  else if (key == "predictor_type") v = cfg->predictor_type_str;
  else if (key == "predictor_model_path") v = cfg->predictor_model_path;
  else if (key == "layer_predict_interval") v = std::to_string(cfg->layer_predict_interval);
  else if (key == "layer_predict_max_window") v = std::to_string(cfg->layer_predict_max_window);
  else if (key == "layer_predict_replace_first_input_with_last_output") v = b(cfg->cross_token_pred);
  else if (key == "limit_layer_0_window") v = std::to_string(cfg->limit_layer_0_window);
  else if (key == "limit_layer_0_num_predict") v = std::to_string(cfg->limit_layer_0_num_predict);
  else if (key == "max_prefetch_layer_distance") v = std::to_string(cfg->max_prefetch_layer_distance);
  else if (key == "cache_only") v = b(cfg->cache_only);
  else if (key == "per_layer_cache") v = b(cfg->per_layer_cache);
  else if (key == "promote_hit_in_prefetch") v = b(cfg->promote_hit_in_prefetch);
  else if (key == "cache_policy") v = cfg->cache_policy;
  else if (key == "predict_input_reuse_distance_max") v = std::to_string(cfg->predict_input_reuse_distance_max);
  else if (key == "predict_input_decay") v = std::to_string(cfg->predict_input_decay);
  else if (key == "num_per_expert_param") v = std::to_string(cfg->num_per_expert_param);
  else if (key == "num_dummy_params") v = std::to_string(cfg->num_dummy_params);
  else if (key == "physical_mem_impl") v = cfg->physical_mem_impl;
  else if (key == "logical_mem_impl") v = cfg->logical_mem_impl;
  else if (key == "expert_mem_scale") v = std::to_string(cfg->expert_mem_scale);
  else if (key == "sleep_on_report_logits_us") v = std::to_string(cfg->sleep_on_report_logits_us);
  else { moe_set_error("moe_cfg_get: unknown key %s", key.c_str()); return MOE_EINVAL; }
  (void)kKnownKeys;
  snprintf(buf, buflen, "%s", v.c_str());
  return (int)v.size();
}
