/*
 * moe_kernels.h — C ABI of the MoE-layer compute kernels (gfx950 / MI355X).
 *
 * These entry points are what a host (the patched MoE module of the reference,
 * or llama.cpp through the reference's libmoe_cache.so) binds instead of the
 * per-expert kernels the reference outsources to cuBLAS / exllama / HQQ / ggml.
 * The reference itself has no source for them: its MoE module contract is only
 * visible through its stand-in
 *   eval/demo-simulate/transformers-deepseek-moe.py:36-49  (SimulateMoeLayer.forward)
 * and the hook sites src/sparse_llm_cache/utils/__init__.py:82-96.
 *
 * Conventions: every function returns 0 on success or a negative MOE_E* code and
 * never aborts (the reference aborts on any failed check, logging.cc:77-81).
 * All pointers are DEVICE pointers unless the name ends in _host.  `stream` is a
 * hipStream_t passed as void* (NULL = the null stream).  Nothing here allocates.
 */
#ifndef MOE_KERNELS_H
#define MOE_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_OK 0
#define MOE_EINVAL (-1)   /* bad argument / unsupported shape */
#define MOE_EHIP (-2)     /* a HIP runtime call failed: see moe_last_error() */
#define MOE_ESTATE (-3)   /* call not valid in the current engine state */
#define MOE_ENOMEM (-4)
#define MOE_ENOTRESIDENT (-5)

/* gating conventions (k1) */
#define MOE_ROUTE_SOFTMAX_TOPK 0        /* DeepSeek-MoE / Qwen-MoE: softmax over E, top-k, no renorm */
#define MOE_ROUTE_SOFTMAX_TOPK_RENORM 1 /* same, weights divided by their sum */
#define MOE_ROUTE_TOPK_SOFTMAX 2        /* Mixtral: top-k of logits, softmax over the k */

/* weight formats of an expert (all weights [out,in]) */
#define MOE_FMT_INT4_G128 0 /* tiled int4, group 128 along K, fp16 scales, uint4 zeros */
#define MOE_FMT_BF16 1      /* bf16: w13 [2I,H] (gate rows then up rows) then w2 [H,I], each matrix in
                             * blocks of 32 rows x 64 k (4 KiB; block (nb,kb) at element (((nb/4)*K/64+kb)*4+nb%4)*2048,
                             * inside a block element [j][q][n][e] is W[32nb+n][64kb+32q+8j+e]) */

#define MOE_FMT_Q4K 2       /* ggml q4_K information (fp16 d, dmin per 256 weights; 6-bit scale and min per
                             * 32) repacked: nibbles in the int4 tile order, one (scale, min) byte pair per
                             * tile lane, one (d, dmin) fp16 pair per row and super-block; see
                             * moe_q4k_layout_make.  w = d*sc*q - dmin*m. */

const char *moe_last_error(void);

/*
 * Byte layout of ONE int4 expert inside a cache slot (or inside the resident
 * shared-expert buffer).  Section offsets are from the expert's base address.
 *
 *  w13 = gate_proj and up_proj [I,H] interleaved in 16-row blocks: row-block 2b
 *        holds gate rows 16b..16b+15, row-block 2b+1 the up rows 16b..16b+15.
 *  w2  = down_proj [H,I].
 *  A matrix W[N,K] is stored as tiles (rb = n/16, g = k/128), tile (rb,g) at
 *  q + (rb*G + g)*1024 bytes: 64 lanes x 4 dwords; lane l holds row 16rb + (l&15),
 *  k = 128g + 32(l>>4) + 8j + 0..7 in dword j, with element k+i at bit
 *  (i even ? 2i : 16 + 2(i-1)) (so (dword >> 4m) & 0x000f000f is the pair
 *  (k+2m, k+2m+1)).  scales: fp16 [N/16][G][16]; zeros: 4 bit [N/16][G][16]
 *  (8 bytes per tile, row r in byte r/2, low nibble first).  w = (q - z) * s.
 */
typedef struct moe_int4_layout {
  int64_t off13_q, off13_s, off13_z;
  int64_t off2_q, off2_s, off2_z;
  int64_t total_bytes; /* = 3*I*H/2 + 3*I*H/128*2 + 3*I*H/128/2 */
} moe_int4_layout;

/* H, I multiples of 128 and 16.  Reference counterpart: the per-param chunk list
 * registered through ModelLoader::add_one_expert_param (model_loader.hpp:282-288),
 * laid end to end as ExpertMemHanlderTensorUnified does (model_loader.cpp:208-234). */
int moe_int4_layout_make(int H, int I, moe_int4_layout *out);

/* q4_K experts.  Same section order as the int4 layout (q, s, z per matrix; the struct is
 * reused): q = nibble tiles exactly as above; s = [N/16][G][64] byte pairs (sc, m): lane l of
 * tile (rb, g) owns row 16rb + (l&15), sub-block 4*(g&1) + (l>>4) of super-block g/2;
 * z = [N/16][G/2][16] pairs (fp16 d, fp16 dmin).  148 bytes per 256 weights (ggml: 144).
 * H, I multiples of 256.  Source of the format: ggml block_q4_K, which the reference reaches
 * through its llama.cpp fork (README.md:29-34, 45-54); it holds no q4_K code of its own. */
int moe_q4k_layout_make(int H, int I, moe_int4_layout *out);

/* k1a: logits[t*ldl + e] = sum_k x[t,k]*wg[e,k] (+ bias[e]); bf16 inputs, fp32 result.
 * Summation order is fixed (64 lane partials over k = c*512 + 8*lane + i, then an
 * xor butterfly 32..1) so the result is bit-reproducible.  H % 8 == 0. */
int moe_gate_logits(const void *x_bf16, const void *wg_bf16, const float *bias, float *logits,
                    int T, int H, int E, int ldl, void *stream);

/* moe_gate_logits for two matrices over the same activations in ONE launch (T <= 128): wg [E, H] (+ bias) into
 * logits (row stride ldl), wg2 [E2, H] (+ bias2) into logits2 (row stride ldl2); the same bits as two calls.
 * The engine uses it to let the built-in predictor's score rows (engine_predict.cpp; the reference evaluates its
 * per-pair models in PredictWorker, worker.cpp:6-77) ride in the layer's own gate launch. */
int moe_gate_logits_pair(const void *x_bf16, const void *wg_bf16, const float *bias, float *logits, int T, int H,
                         int E, int ldl, const void *wg2_bf16, const float *bias2, float *logits2, int E2,
                         int ldl2, void *stream);

/* k1b: top-k routing.  Selection on the logits, ties toward the lower expert index.
 * idx [T,k] int32, w [T,k] fp32.  E <= 256, k <= 32. */
int moe_topk(const float *logits, int T, int E, int ldl, int k, int mode, int *idx, float *w,
             void *stream);

/* one active routed expert of a layer call */
typedef struct moe_unit {
  int32_t expert; /* expert id, -1 = unused entry */
  int32_t m;      /* tokens routed to it */
  int32_t row0;   /* first row in the sorted pair order */
  int32_t pad;
} moe_unit;

/* k2: stable dispatch of the P = T*k (token,slot) pairs (pair p = t*k + j).
 * counts[E], offsets[E+1], sorted_pair[P], pos_of_pair[P], sorted_tok[P] (= p / k),
 * units[max_units] (active experts ascending id, rest m = 0), n_active[1],
 * active_ids[max_units] int64 (the `unique expert ids` list the reference's module
 * hands to report_experts, utils/__init__.py:84-88). */
int moe_dispatch(const int *idx, int T, int k, int E, int *counts, int *offsets, int *sorted_pair,
                 int *pos_of_pair, int *sorted_tok, moe_unit *units, int *n_active,
                 int64_t *active_ids, int max_units, void *stream);

/* k2 with a workspace, for prefill batches: the same arrays, bit for bit, from one workgroup per 1024 pairs when
 * P = T*k >= 2048 and E <= 256 (otherwise, or with ws NULL or smaller than moe_dispatch_workspace_bytes, this is
 * moe_dispatch).  ws: device memory whose first 64 bytes are zero before the first call (the kernel leaves them
 * zero); calls that share a workspace must not overlap.  err: word that a workgroup raises when the others'
 * counts do not arrive within a second (device memory or pinned host memory).
 * moe_dispatch_workspace_bytes returns 0 where the workspace would not be used. */
int64_t moe_dispatch_workspace_bytes(int T, int k, int E);
int moe_dispatch_ws(const int *idx, int T, int k, int E, int *counts, int *offsets, int *sorted_pair,
                    int *pos_of_pair, int *sorted_tok, moe_unit *units, int *n_active,
                    int64_t *active_ids, int max_units, void *ws, int64_t ws_bytes, int *err, void *stream);

/* k1a+k1b+k2 in one launch for decode batches (T <= 16, E <= 256, T*k <= 512): same results,
 * bit for bit, as moe_gate_logits + moe_topk + moe_dispatch.  E_rows = E, or E+1 when row E of
 * wg is the shared expert's gate vector (its logit lands in logits[t*ldl + E], no bias).
 * counter: one device word, zero before the first call; the workgroup that finishes its
 * logits last runs the routing and leaves the word zero again. */
int moe_route_decode(const void *x_bf16, const void *wg_bf16, const float *bias, float *logits,
                     int T, int H, int E, int E_rows, int ldl, int k, int mode, int *idx, float *w,
                     int *counts, int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok,
                     moe_unit *units, int *n_active, int64_t *active_ids, int max_units,
                     unsigned *counter, void *stream);

/* k1b + k2 in one launch (one workgroup) for decode batches: T <= 64, E <= 256, T*k <= 512; same
 * results, bit for bit, as moe_topk + moe_dispatch.  units_host_out / n_active_host_out /
 * seq_host_out (optional, pinned HOST memory): the kernel also stores the unit list and its length
 * there and then, once those stores have completed, seq_value into *seq_host_out. */
int moe_topk_dispatch(const float *logits, int T, int E, int ldl, int k, int mode, int *idx, float *w,
                      int *counts, int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok,
                      moe_unit *units, int *n_active, int64_t *active_ids, int max_units,
                      moe_unit *units_host_out, int *n_active_host_out, int *seq_host_out, int seq_value,
                      void *stream);

/* k1a + k1b + k2 in one launch for decode batches (2 <= T <= 32, E <= 256, T*k <= 512): same results, bit for
 * bit, as moe_gate_logits + moe_topk_dispatch (reference: the gate's linear layer, the top-k and the expert
 * grouping of the patched sparse block, utils/__init__.py:84-141).  Workgroup 0 routes; the other workgroups sum
 * the gate rows (a wave per (token, row)) and hand every logit to it through gate_ws as a (value, gate_seq) word,
 * which it polls (bounded: on a time-out *err |= 1); the logits also land in logits[t*ldl + e].
 *   E_rows = E, or E+1 when row E of wg is the shared expert's gate vector; bias covers rows 0 .. n_bias-1.
 *   gate_ws: moe_gate_route_ws_bytes(T, E_rows) of device memory, zeroed once (the area of
 *   moe_decode_token_int4_gate may be shared when it is that large); gate_seq: nonzero, never used before on gate_ws.
 *   parts: 8 = every gate row is summed once per part of the chip and travels through that part's second-level
 *   cache (plus one device-scope copy as the fallback), 1 = summed once and handed over at device scope.
 *   units_host_out .. seq_value: as in moe_topk_dispatch. */
int64_t moe_gate_route_ws_bytes(int T, int E_rows);
int moe_gate_topk_dispatch(const void *x_bf16, const void *wg_bf16, const float *bias, int n_bias, float *logits,
                           int T, int H, int E, int E_rows, int ldl, int k, int mode, int *idx, float *w,
                           int *counts, int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok,
                           moe_unit *units, int *n_active, int64_t *active_ids, int max_units,
                           moe_unit *units_host_out, int *n_active_host_out, int *seq_host_out, int seq_value,
                           void *gate_ws, int gate_seq, int parts, int *err, void *stream);

/* k1a + k1b + k2 + the w13 half of k3 in ONE launch for decode batches of 2 to 8 tokens (reference: the gate's
 * linear layer, top-k, expert grouping and the experts' first two projections of the patched sparse block,
 * utils/__init__.py:84-141): the launch sums the gate rows in its first workgroups, every workgroup of a unit slot
 * derives the routing itself from the handed-over logits, and one workgroup publishes the routing (all arrays of
 * moe_topk_dispatch, bit for bit, and the optional host copy).  Results equal moe_gate_topk_dispatch followed by
 * moe_experts_decode_int4, bit for bit.  phases: bit 0 = that launch, bit 1 = the w2 launch over the published
 * unit list.  max_units must be min(E, T k); gate_ws / gate_seq as in moe_gate_topk_dispatch
 * (moe_gate_route_ws_bytes(T, n_gate_rows) bytes).  moe_decode_batch_int4_gate_fits says whether a shape is taken.
 *   expert_ptr_host (optional, E <= 64): a HOST copy of the slot table.  Both launches then carry the table in
 *   their arguments and do not read expert_ptr, so a caller whose table changed since the last launch needs no
 *   copy in the stream in front of this one (a cache that has just loaded an expert).  NULL: expert_ptr is read. */
int moe_decode_batch_int4_gate_fits(int T, int E, int k, int H, int I, int I_sh, int n_gate_rows);
int moe_decode_batch_int4_gate(const void *x_bf16, int T, const void *gate_w_bf16, const float *gate_bias,
                               int n_gate_rows, void *gate_ws, int gate_seq, float *logits, int ldl, int E, int k,
                               int mode, int H, int I, int I_sh, const uint64_t *expert_ptr,
                               const uint64_t *expert_ptr_host, const void *shared_ptr,
                               int *idx, float *w, int *counts, int *offsets, int *sorted_pair, int *pos_of_pair,
                               int *sorted_tok, moe_unit *units, int *n_active, int64_t *active_ids, int max_units,
                               void *h_r, void *h_s, float *part_r, float *part_s, int *err,
                               moe_unit *units_host_out, int *n_active_host_out, int *seq_host_out, int seq_value,
                               int phases, void *stream);

/* k3 (decode): int4 grouped SwiGLU expert product through the slot table.
 *   expert_ptr[e] : device address of expert e's slot (0 = not resident -> *err |= 1)
 *   shared_ptr    : resident shared expert (intermediate I_sh) or NULL
 *   h_r [P, I] bf16, h_s [T, I_sh] bf16, part_r [P, H] fp32, part_s [T, H] fp32: workspaces
 * Rows of the routed buffers follow the sorted pair order of moe_dispatch.
 * Covers tokens-per-expert of any size by passes of 16 rows (32 in the w2 pass above 48 tokens);
 * meant for T <= 64.
 * units_host / expert_ptr_host (HOST copies of the unit list and of the slot table row,
 * both optional): when given and max_units <= 64 the units travel in the kernel arguments
 * and the kernels read neither `units` nor `expert_ptr`.
 * phases: bit 0 = w13 + SwiGLU (x -> h), bit 1 = w2 (h -> partial rows); 3 = both. */
int moe_experts_decode_int4(const void *x_bf16, int T, int H, int I, int I_sh, int k,
                            const moe_unit *units, int max_units, const int *sorted_tok,
                            const uint64_t *expert_ptr, const void *shared_ptr, void *h_r,
                            void *h_s, float *part_r, float *part_s, int *err,
                            const moe_unit *units_host, const uint64_t *expert_ptr_host,
                            int phases, void *stream);

/* The same, with the step's unit list sent to the host by the w13 launch (T >= 2, device unit list, phase bit 0):
 * one more workgroup copies units[0 .. *n_active) and the count into units_host_out / n_active_host_out (pinned
 * HOST memory) and then, once those stores have completed, stores seq_value into *seq_host_out, while the other
 * workgroups stream weights.  A routing launch that publishes itself (moe_topk_dispatch with its host arguments)
 * is held by those stores for about 2 us; here nothing waits for them.  units_host_out NULL: moe_experts_decode_int4. */
int moe_experts_decode_int4_publish(const void *x_bf16, int T, int H, int I, int I_sh, int k,
                                    const moe_unit *units, int max_units, const int *sorted_tok,
                                    const uint64_t *expert_ptr, const void *shared_ptr, void *h_r,
                                    void *h_s, float *part_r, float *part_s, int *err,
                                    const moe_unit *units_host, const uint64_t *expert_ptr_host,
                                    int phases, const int *n_active, moe_unit *units_host_out,
                                    int *n_active_host_out, int *seq_host_out, int seq_value, void *stream);

/* k1b + k2 + k3 for ONE token: the w13 kernel derives the routing itself from the gate logits
 * (same selection, tie rule and weights as moe_topk, same arrays as moe_dispatch, bit for bit)
 * and publishes it for the w2 pass, moe_combine and the host, so a decode step is
 * moe_gate_logits -> moe_decode_token_int4 -> moe_combine.  E <= 256.  logits: E fp32 values.
 * Every selected expert must be resident (expert_ptr[e] != 0), else *err |= 1.
 * unit_ws (optional): 32*k bytes of device memory; the first pass leaves the resolved units (slot
 * address, row) there and the w2 pass starts from one load instead of unit -> table -> address.
 * units_host_out / seq_host_out (optional, pinned HOST memory): the kernel also stores the k
 * units there and then, once those stores have completed, seq_value into *seq_host_out, so a host
 * that polls the word gets the routing without a copy or an event.
 * phases: bit 0 = routing + w13 + SwiGLU, bit 1 = w2 into partial rows (needs the units of an
 * earlier bit-0 call), bit 2 = w2 and the weighted combine in ONE launch, straight into y_bf16 [H]
 * (needs unit_ws of 32*k bytes; shared_gate_logit = the shared expert's gate logit or NULL; every
 * selected expert resident).  Bits 1 and 2 exclude each other.
 * expert_ptr_host (optional, E <= 64): a HOST copy of the slot table; the launch of phase bit 0 then carries the
 * table in its arguments and does not read expert_ptr (no copy of a changed table in front of the launch). */
int moe_decode_token_int4(const void *x_bf16, const float *logits, int E, int k, int mode, int H, int I,
                          int I_sh, const uint64_t *expert_ptr, const uint64_t *expert_ptr_host,
                          const void *shared_ptr, int *idx, float *w,
                          int *counts, int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok,
                          moe_unit *units, int *n_active, int64_t *active_ids, void *h_r, void *h_s,
                          float *part_r, float *part_s, int *err, void *unit_ws, moe_unit *units_host_out,
                          int *seq_host_out, int seq_value, int phases, const float *shared_gate_logit,
                          void *y_bf16, void *stream);


/* One token, an expert whose copy landed after the step's routing launch (moe_decode_token_int4 with phase bit
 * 0 skipped it and published its unit with slot address 0): w13 + SwiGLU of that one unit, h_r row `pos` (the
 * unit's position in the step's unit list), and the unit's slot address written into unit_ws[pos], so that a
 * following moe_decode_token_int4 with phase bit 2 (w2 + combine over all units) finds it.  The cache's
 * counterpart in the reference: the per-expert forward between report_one_expert and one_expert_done
 * (utils/__init__.py:89-95). */
int moe_decode_token_late_expert_int4(const void *x_bf16, int H, int I, uint64_t slot_addr, int pos, void *h_r,
                                      void *unit_ws, int *err, void *stream);

/* k1a + k1b + k2 + k3 for ONE token: moe_decode_token_int4 whose launch of phase bit 0 also computes the gate
 * logits, so a decode step is two launches (this one, then w2 + combine) instead of three.  The first
 * ceil(n_gate_rows / 4) workgroups sum the gate rows (a wave per row, the summation order of moe_gate_logits:
 * the same bits) and hand every logit to the routing waves of the same launch through gate_ws as a (value,
 * gate_seq) word; the routing waves poll until every word carries gate_seq (bounded: on a time-out *err |= 1).
 *   gate_w [n_gate_rows, H] bf16, n_gate_rows = E, or E + 1 with the shared expert's gate vector as row E;
 *   gate_bias [E] or NULL (the routed rows only); logits [n_gate_rows] fp32 is an OUTPUT here.
 *   gate_ws: moe_gate_ws_bytes() of device memory, zeroed once by the caller; gate_seq: a nonzero number that no
 *   earlier call with the same gate_ws used (count upwards), so nothing has to be cleared between calls.
 * Because gate_seq is a launch argument, a HIP graph that records this call replays one number: inside a graph
 * use moe_gate_logits + moe_decode_token_int4.  No counterpart in the reference (its gate is torch's). */
int64_t moe_gate_ws_bytes(void);
int moe_decode_token_int4_gate(const void *x_bf16, const void *gate_w, const float *gate_bias, int n_gate_rows,
                               void *gate_ws, int gate_seq, float *logits, int E, int k, int mode, int H, int I,
                               int I_sh, const uint64_t *expert_ptr, const uint64_t *expert_ptr_host,
                               const void *shared_ptr, int *idx, float *w,
                               int *counts, int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok,
                               moe_unit *units, int *n_active, int64_t *active_ids, void *h_r, void *h_s,
                               float *part_r, float *part_s, int *err, void *unit_ws, moe_unit *units_host_out,
                               int *seq_host_out, int seq_value, int phases, const float *shared_gate_logit,
                               void *y_bf16, void *stream);

/* moe_decode_token_int4 with phases = 5 (routing + w13 + SwiGLU, then w2 + combine into y_bf16 [H]) that
 * allocates nothing and takes no workspace: the routing arrays, the h vectors and the resolved units live in
 * a device array of moe_noalloc_scratch_bytes() (under 160 KiB) that is part of the library image; each GPU
 * the library runs on holds its copy until the process ends.  No counterpart in the reference: it is for
 * callers that cannot allocate or hand over workspaces (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  Inputs and outputs are the caller's: x, logits (E fp32), the slot table,
 * the shared expert, y, and the error word err (device or pinned host memory, cleared by the caller; set to 1
 * when a selected expert is not resident).  Limits: E <= 256, k <= 32, k*I + I_sh <= 71680 (the room
 * the array has for the h vectors), H <= 16384; beyond them MOE_EINVAL.  All calls on one GPU share the array:
 * calls that overlap on one GPU (two streams, two threads) race; calls on one stream are ordered. */
int64_t moe_noalloc_scratch_bytes(void);
int moe_decode_token_int4_noalloc(const void *x_bf16, const float *logits, int E, int k, int mode, int H, int I,
                                  int I_sh, const uint64_t *expert_ptr, const void *shared_ptr,
                                  const float *shared_gate_logit, void *y_bf16, int *err, void *stream);

/* k3 for q4_K experts: same buffers as moe_experts_decode_int4, device-side unit list only.
 * One token: dot products on the vector ALU in bf16 x (128 + q), scales applied per sub-block in fp32.  Two tokens
 * and more (any T; moe_forward sends up to 64): the chunked-K matrix-core kernel, every weight dequantised to fp16
 * (d sc q - dmin m, the arithmetic of moe_experts_prefill for this format) against fp16 activations, fp32
 * accumulation; activations must stay below 65504 in magnitude there.
 * Exception to "same buffers": part_s.  With few output rows and a long reduction (H / 32 block pairs, I_sh columns: Qwen2-57B's
 * shared expert is 112 block pairs over 20480 columns) the w2 pass splits the shared expert's reduction over
 * moe_decode_shared_splits(MOE_FMT_Q4K, T, H, I_sh) = S workgroups per block pair; split s writes its partial
 * rows to part_s + s*T*H, so part_s must hold S*T*H floats and the combine must be told
 * (moe_combine_splits).  S = 1 for every other format.  No reference counterpart (the reference leaves the
 * arithmetic to llama.cpp's kernels, adapter-llama.cpp:12-46). */
int moe_decode_shared_splits(int fmt, int T, int H, int I_sh);
int moe_experts_decode_q4k(const void *x_bf16, int T, int H, int I, int I_sh, int k,
                           const moe_unit *units, int max_units, const int *sorted_tok,
                           const uint64_t *expert_ptr, const void *shared_ptr, void *h_r, void *h_s,
                           float *part_r, float *part_s, int *err, int phases, void *stream);

/* k4 (prefill): grouped SwiGLU expert product on the matrix cores for large token groups.
 * Same arguments and buffer meanings as moe_experts_decode_int4 (rows of h_r / part_r in the
 * sorted pair order; expert_ptr[e] == 0 for an active expert sets *err |= 1 and skips it).
 *   fmt       : MOE_FMT_BF16 (expert image = blocked w13 [2I,H] then blocked w2 [H,I]; bf16 MFMA),
 *               MOE_FMT_INT4_G128 or MOE_FMT_Q4K (nibble tiles dequantised in registers to fp16
 *               operands, activations converted bf16 -> fp16 on the way into LDS; tiles of 192 rows)
 *   tiles_ws  : device workspace of moe_prefill_workspace_bytes(T, k, max_units) bytes; the
 *               list of row tiles per expert is built there by a kernel, so the host
 *               needs no copy of the dispatch counts.
 * Between the two passes h_r / h_s hold bf16 for MOE_FMT_BF16 and fp16 for the nibble formats (whose matrix-core
 * operands are fp16: the w2 pass then stages them without a conversion); both passes of a batch go through this entry.
 * H % 256 == 0, I % 128 == 0, I_sh % 128 == 0.  The reference leaves this product to the
 * framework's own expert modules (SimulateMoeLayer.forward, transformers-deepseek-moe.py:36-49). */
int64_t moe_prefill_workspace_bytes(int T, int k, int max_units);
int moe_prefill_tile_rows(void);
int moe_experts_prefill(const void *x_bf16, int T, int H, int I, int I_sh, int k, int fmt,
                        const moe_unit *units, int max_units, const int *sorted_tok,
                        const uint64_t *expert_ptr, const void *shared_ptr, void *h_r, void *h_s,
                        float *part_r, float *part_s, void *tiles_ws, int *err, int phases,
                        void *stream);

/* The same with the shared expert's partial rows of the w2 pass in shared_pieces pieces (1, 2, 4 or 8; nibble
 * formats only): part_s holds shared_pieces * T rows, piece s at part_s + s*T*H, each the product over one window
 * of the I_sh columns; moe_combine_splits adds them.  moe_prefill_shared_splits(fmt, T, H, I_sh) = the number of
 * pieces worth taking: more than 1 where the shared expert's workgroups of that pass (ceil(T/128) * H/256, each over
 * the whole reduction) are few and the reduction is long, so that they would outlast the rest of the launch
 * (Qwen2-57B shape at 512 tokens: 4).  No reference counterpart (see moe_decode_shared_splits). */
int moe_prefill_shared_splits(int fmt, int T, int H, int I_sh);
int moe_experts_prefill_pieces(const void *x_bf16, int T, int H, int I, int I_sh, int k, int fmt,
                               const moe_unit *units, int max_units, const int *sorted_tok,
                               const uint64_t *expert_ptr, const void *shared_ptr, void *h_r, void *h_s,
                               float *part_r, float *part_s, int shared_pieces, void *tiles_ws, int *err,
                               int phases, void *stream);

/* k5: y[t,:] = sum_j w[t,j] * part_r[pos_of_pair[t*k+j],:] + g_t * part_s[t,:], bf16 out.
 * g_t = sigmoid(shared_gate_logit[t*sg_stride]) when shared_gate_logit != NULL, else 1;
 * part_s may be NULL (no shared expert). */
int moe_combine(const float *part_r, const float *part_s, const float *topk_w,
                const int *pos_of_pair, const float *shared_gate_logit, int sg_stride, void *y_bf16,
                int T, int H, int k, void *stream);
/* the same with a shared expert whose partial rows come in n_shared_splits pieces (piece s at part_s + s*T*H),
 * added in piece order before the gate is applied; n_shared_splits = 1 is moe_combine */
int moe_combine_splits(const float *part_r, const float *part_s, const float *topk_w,
                       const int *pos_of_pair, const float *shared_gate_logit, int sg_stride, void *y_bf16,
                       int T, int H, int k, int n_shared_splits, void *stream);

/* Per-kernel timing with HIP events recorded on the launch stream around every kernel
 * the launchers below start (no reference counterpart; used by the benchmark to report
 * kernel durations).  kernel_id: 0 gate logits, 1 top-k, 2 dispatch, 3 decode w13+SwiGLU,
 * 4 decode w2, 5 combine, 6 prefill w13, 7 prefill w2.  enable=1 clears earlier records. */
int moe_kernel_timing(int enable);
int moe_kernel_timing_read(int kernel_id, double *total_ms, int *calls);

#ifdef __cplusplus
}
#endif
#endif
