/*
 * moe_engine.h — C ABI of the expert-cache engine: configuration, expert registry,
 * HBM slot pool, eviction policies, demand/speculative fetch scheduling, counters,
 * and the fused MoE-layer forward that runs on top of them.
 *
 * Each entry point names the reference interface it replaces
 * (paths relative to the reference tree, src/cpp_worker/... unless noted).
 * Unlike the reference, which aborts the process on any failed check
 * (logging.cc:77-81), every function returns 0 or a negative MOE_E* code and
 * leaves a message in moe_last_error().
 *
 * Threading: like the reference's pybind surface (adapter.cpp has no
 * gil_scoped_release) the API is meant to be driven from one thread; cache state
 * is guarded by one mutex and a single background fetch thread issues the
 * host->HBM copies one chunk at a time, demand fetches first.
 */
#ifndef MOE_ENGINE_H
#define MOE_ENGINE_H

#include <stddef.h>
#include <stdint.h>

#include "moe_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct moe_cfg moe_cfg;
typedef struct moe_engine moe_engine;

/* ---- configuration: ModuleMeta (utils.hpp:127-192, utils.cpp:54-273, adapter.cpp:14-40) ---- */

/* ModuleMeta(num_layer, num_expert) */
moe_cfg *moe_cfg_create(int num_layer, int num_expert);
void moe_cfg_destroy(moe_cfg *cfg);
/* One entry of the map given to ModuleMeta::init_from_map.  Keys are the reference's
 * (and its llama.cpp dialect: '-' == '_', cross_token_pred, num_predict, predict_interval,
 * predict_window, moe_cache_policy, moe_cache_rate, pred_model_path, utils.cpp:147-172).
 * The value "None" or "" selects the default.  A key given twice (after dialect
 * translation) is an error. */
int moe_cfg_set(moe_cfg *cfg, const char *key, const char *value);
/* ModuleMeta::init_param_list: names of the per-expert parameter chunks, in copy order */
int moe_cfg_set_params(moe_cfg *cfg, const char *const *names, int n);
/* init_from_map + handle_uninited_configs: validates (unknown key, missing
 * num_expert_per_token, bad number -> MOE_EINVAL), fills defaults, applies the
 * SPARSE_CACHE_* environment overrides (utils.cpp:222-273). */
int moe_cfg_finalize(moe_cfg *cfg);
/* value of a (canonical) key as text; returns length or <0 */
int moe_cfg_get(const moe_cfg *cfg, const char *key, char *buf, int buflen);

/* ---- engine lifetime: ModelLoader + CacheMngr + PrefetchMngr (adapter.cpp:53-106) ---- */

#define MOE_BACKEND_HIP 0  /* slots in HBM, copies by hipMemcpyAsync on a side stream */
#define MOE_BACKEND_HOST 1 /* slots in host memory, copies by memcpy: CPU tests of the cache logic */

/* ModelLoader(meta) + PrefetchMngr(meta, loader, predictor) (model_loader.cpp:8-21,
 * prefetcher.cpp:286-432).  compute_stream: hipStream_t the caller launches on
 * (0 = the engine creates one, like create_compute_stream=true). */
int moe_engine_create(const moe_cfg *cfg, int backend, void *compute_stream, moe_engine **out);
/* ~PrefetchMngr (prefetcher.cpp:480-493): stops the fetch thread */
void moe_engine_destroy(moe_engine *eng);

/* pinned host memory for expert images (Tensor::pin_memory, model_loader.hpp:52-54).
 * Memory that already exists cannot be pinned afterwards on this platform, so the
 * caller allocates its staging here and fills it. */
void *moe_host_alloc(size_t nbytes);
void moe_host_free(void *p);

/* ModelLoader::add_one_expert_param (model_loader.hpp:282-288, model_loader.cpp:23-31).
 * The engine does not own host memory; it must stay valid for the engine's life.
 * alloc_nbytes = 0 means nbytes. */
int moe_register_param(moe_engine *eng, int layer, int expert, int param_id, const void *host_ptr,
                       size_t nbytes, size_t alloc_nbytes);
/* ModelLoader::pin_memory (model_loader.cpp:62-72): reports how many registered
 * chunks are NOT in pinned memory (copies from those are staged by the runtime). */
int moe_pin_host(moe_engine *eng, int *n_unpinned);

/* PrefetchMngr::init_gpu_mem_buffer + CacheMngr::init_gpu_mem_buffer
 * (prefetcher.cpp:162-177, cache.cpp:57-132): cache_len = round(cache_rate*L*E)
 * spread over the slot groups, every slot sized for the largest expert. */
int moe_init_slots(moe_engine *eng);
/* the slot count arithmetic alone (cache.cpp:57-94): out[n_groups] */
int moe_slot_distribution(int64_t num_buffers, int n_groups, int64_t *out);
int moe_slot_info(moe_engine *eng, int group, int64_t *n_slots, int64_t *slot_bytes,
                  int64_t *stride_bytes);
/* PrefetchMngr::launch_thread (prefetcher.cpp:269-285) */
int moe_launch(moe_engine *eng);

/* ---- slot lookup ---- */
/* ModelLoader::ref_one_expert_param (model_loader.hpp:308-313): device address of a
 * parameter chunk of a RESIDENT expert; *out = NULL when the expert holds no slot
 * (the reference aliases slot 0 instead, prefetcher.cpp:176). */
int moe_expert_param_ptr(moe_engine *eng, int layer, int expert, int param_id, void **out);
/* device array uint64[num_expert] of slot base addresses of `layer` (0 = not resident);
 * what the kernels indirect through.  Valid after moe_init_slots. */
int moe_expert_ptr_table(moe_engine *eng, int layer, const uint64_t **out);
/* make the device copy of the table of `layer` current on `stream` */
int moe_flush_table(moe_engine *eng, int layer, void *stream);
/* ExpertStatus (utils.hpp:38-49): 0 idle, 1 fetching, 2 ready, 3 launching, 4 using */
int moe_expert_status(moe_engine *eng, int layer, int expert);
int moe_is_in_cache(moe_engine *eng, int layer, int expert);
int moe_expert_num_ready(moe_engine *eng, int layer, int expert);

/* ---- the hook sequence of one MoE layer ---- */
/* PrefetchMngr::report_moe_layer_logits (prefetcher.cpp:447-460): dims [B,S,H]; records
 * kSeqLen at layer 0.  hidden may be NULL (no predictor attached). */
int moe_report_layer_logits(moe_engine *eng, int layer, const void *hidden, int B, int S, int H);
/* PrefetchMngr::report_one_layer (prefetcher.cpp:188-202): ids is a HOST int64 buffer,
 * reordered IN PLACE [ready, current copy, partial, miss]; hits become `launching`,
 * misses get demand copies queued; the layer's speculative queue is cleared. */
int moe_report_one_layer(moe_engine *eng, int layer, int64_t *ids, int64_t n);
/* PrefetchMngr::report_one_expert (prefetcher.cpp:225-260): blocks until usable */
int moe_wait_expert(moe_engine *eng, int layer, int expert);
/* PrefetchMngr::one_expert_done (prefetcher.cpp:236-239,261-267): records the
 * expert's event on the compute stream; launching -> using (-> ready once the event fired) */
int moe_expert_launched(moe_engine *eng, int layer, int expert);
/* PrefetchMngr::one_moe_layer_done (prefetcher.cpp:203-223) */
int moe_layer_done(moe_engine *eng, int layer);
/* fused form of the three calls above for a whole layer: report_one_layer, wait for
 * every id, flush the slot table on the compute stream. */
int moe_acquire_layer(moe_engine *eng, int layer, int64_t *ids, int64_t n);
/* one event for the layer on the compute stream; every launching expert -> using.
 * Only valid when every expert acquired for the layer has been launched
 * (after moe_acquire_layer). */
int moe_release_layer(moe_engine *eng, int layer);
/* same for an explicit list of launched experts (one shared event) */
int moe_release_experts(moe_engine *eng, int layer, const int64_t *ids, int64_t n);

/* ---- prefetch request hook: PrefetchLayerTask (prefetcher.hpp:52-58, worker.cpp:41-68) ---- */
/* Queue speculative copies of `ids` (ranked) for a future layer.  Takes one unit of
 * the run-ahead budget (initially max_prefetch_layer_distance, returned by
 * report_one_layer / layer_done); blocking=0 returns 1 when no budget is left.
 * With chunk_prefetch an expert is queued as one task per registered parameter (a demand
 * fetch can overtake between tasks), except that a parameter of at most an eighth of its
 * predecessor's bytes shares the predecessor's task. */
int moe_prefetch_layer(moe_engine *eng, int layer, const int64_t *ids, int64_t n, int blocking);
/* When 1, report_one_layer first waits until a prefetch request (possibly empty) for
 * that layer was issued (PredictWorker::consume_prefetch_layer_progress, worker.hpp:312-314). */
int moe_attach_predictor(moe_engine *eng, int attached);
/* CacheMngr::update_priority (cache.cpp:400-430,584-591): predicted probabilities
 * p[n_layers, num_expert] for layers starting_layer.. (policy "nn") */
int moe_update_priority(moe_engine *eng, const float *p, int n_layers, int starting_layer);

/* ---- built-in predictor: what the reference's SepPredictor + PredictWorker do (predictor.cpp:496-607,
 * worker.cpp:6-77) with one linear model per (source layer -> destination layer) pair, scored on
 * the GPU.  Source layer l (0..L; L = the last layer's output) predicts the layers of its window
 * (build_predict_layer_mapping, predictor.cpp:8-46, from layer_predict_interval,
 * layer_predict_max_window, limit_layer_0_window and
 * layer_predict_replace_first_input_with_last_output).  When a decode step (B = S = 1) reports the
 * hidden state of layer l (moe_report_layer_logits; moe_forward does it with every block's input), the
 * scores x . W^T + b of every destination layer are computed on the compute stream; a host thread
 * ranks the top num_predict_expert_per_layer experts (ties: lower id), feeds the softmax of the scores
 * to the NN policy (moe_update_priority) and issues the prefetch requests.  Prefill steps issue empty
 * requests.  Starting the predictor attaches it (see moe_attach_predictor). ---- */
/* first[l], last[l] for l = 0..L: destination layers [first, last) of source layer l */
int moe_predictor_windows(moe_engine *eng, int *first, int *last);
/* model of one pair: w bf16 [num_expert, H] and bias fp32 [num_expert] or NULL, device memory (host memory on
 * the host backend) that stays valid until moe_predictor_start, which copies the models of a source layer
 * into one matrix (the host backend keeps reading the caller's memory); dst must lie in the window of src */
int moe_predictor_set_model(moe_engine *eng, int src, int dst, const void *w, const float *bias, int H);
/* after moe_launch: needs a model for every pair of every window, and every layer covered once */
int moe_predictor_start(moe_engine *eng);
int moe_predictor_stats(moe_engine *eng, uint64_t *n_jobs, uint64_t *n_requests);
/* waits until the predictor thread has worked off every report so far (its counters lag the hooks by a
 * moment); 0 = idle, 1 = still busy after timeout_ms (it may be waiting for the run-ahead budget, which only
 * further layers release).  No counterpart in the reference, whose worker is joined at exit only. */
int moe_predictor_wait_idle(moe_engine *eng, int timeout_ms);
/* Requests scored against what the layers then route to.  Every decode step's routing of a layer
 * (moe_report_one_layer) is compared with the ranking the predictor made for that turn: of the ranked experts
 * that were not resident when the request was made (the ones it has to copy; a turn whose ranked experts were
 * all resident is not scored), the share that was routed to, kept as a moving average per destination layer
 * (0.8 old + 0.2 new, starting at 1).  moe_predictor_set_min_precision(t), t in (0, 1]: a request for a layer whose average is below t
 * goes out EMPTY (as a prefill step's does: the layer's progress count stays in step and nothing is copied)
 * until the average has recovered; the ranking is still made and scored.  t = 0 (the default): every request
 * goes out as ranked, as in the reference (worker.cpp:41-68), whose PredictWorker has no such feedback.
 * moe_predictor_precision: the averages (num_layer floats) and the number of requests sent empty so far. */
int moe_predictor_set_min_precision(moe_engine *eng, float min_precision);
int moe_predictor_precision(moe_engine *eng, float *precision, uint64_t *n_withheld);

/* ---- Belady policy hooks: CacheOracle / set_cur_seq (adapter.cpp:62-70, cache.cpp:592-644) ---- */
int moe_oracle_load(moe_engine *eng, const int64_t *entry_metas, int64_t n_entries,
                    const int32_t *prefill_len, int64_t n_seq, const int32_t *prefill_sel,
                    int64_t max_prefill_len, const int32_t *decode_sel, int64_t k);
int moe_set_seq(moe_engine *eng, uint64_t seq_id);

/* Block until no copy task is queued or in flight (no reference counterpart: the
 * reference's spinning threads offer no quiescence point; tests and orderly shutdown
 * need one). */
int moe_drain(moe_engine *eng);

/* ---- streams (adapter.cpp:92-93) ---- */
int moe_streams(moe_engine *eng, void **compute, void **copy);

/* ---- counters: TimeProfiler (profiler.hpp:253-319, prefetcher.cpp:71-78,246-258) ---- */
typedef struct moe_counters {
  uint64_t hit, miss;                   /* slot resident / not when demanded */
  uint64_t ready, unready;              /* usable / not when the expert hook fired */
  uint64_t prefetch_hit, prefetch_miss; /* same for speculative requests */
  uint64_t activated;                   /* experts reported by report_one_layer */
  uint64_t wait_us;                     /* time spent blocked in wait_expert */
  uint64_t h2d_bytes, h2d_copies;       /* host->slot traffic */
  uint64_t evictions;
  uint64_t forwards;                    /* completed passes over all layers */
} moe_counters;
int moe_get_counters(moe_engine *eng, moe_counters *out);
/* the reference's end-of-run report (prefetcher.cpp:327-402) as key:value lines */
int moe_report(moe_engine *eng, int skip_first_prompts, char *buf, int buflen);

/* ---- fused MoE-layer forward (the patched module's forward as one call) ---- */
typedef struct moe_layer_desc {
  int H, I, I_sh;       /* hidden, routed intermediate, shared intermediate (0 = none) */
  int top_k, route_mode, fmt;
  int shared_gated;      /* 1: shared output scaled by sigmoid(x . gate_w[E]) (row E of gate_w) */
  const void *gate_w;    /* device bf16 [E (+1 if shared_gated), H] */
  const float *gate_bias; /* device fp32 [E] or NULL */
  const void *shared;    /* device: resident shared expert in slot layout, or NULL */
} moe_layer_desc;
int moe_set_layer(moe_engine *eng, int layer, const moe_layer_desc *desc);
/* allocate the forward workspace for up to max_tokens tokens per call */
int moe_forward_prepare(moe_engine *eng, int max_tokens);
/* y[T,H] = MoE layer `layer` applied to x[T,H] (device bf16) on the compute stream:
 * gate -> top-k -> dispatch -> (host: slot lookup / demand fetch) -> experts -> combine.
 * Drives the same hook sequence a patched module would. */
int moe_forward(moe_engine *eng, int layer, const void *x, int T, void *y);
/* routing of the last moe_forward call of this layer (device pointers; valid until the next call) */
int moe_last_routing(moe_engine *eng, const int **idx, const float **w, const int **sorted_pair);
/* the same routing copied to the host once the compute stream has drained: idx_host [T*k] int32 and/or
 * w_host [T*k] fp32 (either may be NULL).  A checking aid with no reference counterpart (the reference's
 * module keeps its routing in torch tensors of its own). */
int moe_last_routing_host(moe_engine *eng, int T, int k, int *idx_host, float *w_host);

#ifdef __cplusplus
}
#endif
#endif
