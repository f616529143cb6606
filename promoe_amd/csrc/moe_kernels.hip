// MoE-layer kernels for gfx950 (MI355X): gating, top-k, stable dispatch,
// int4-group-dequant SwiGLU GEMV through the expert slot table, combine.
// wave64 throughout; no other target is supported.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "moe_kernels.h"
#include "moe_common.h"
#include "moe_device.h"

// The sum of one (token, gate row) pair by one wave, in a fixed order (bit-reproducible): lane partials over
// k = 512 c + 8 lane + j with one fma chain, then the xor butterfly 32..1.  Every lane returns the sum.
// All loads of the row go out back to back, without a condition around any of them (a lane past the end of the row
// reads column 0 and drops the result): with a condition per 512-column chunk the compiler put a full wait for
// memory between the chunks, and a 2048-wide row took four round trips to memory instead of one.
template <int NCH>
static __device__ __forceinline__ float gate_row_partial(const uint16_t *__restrict__ xr, const uint16_t *__restrict__ wr,
                                                         const int H, const int lane) {
  uint4 xq[NCH], wq[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int k = c * 512 + 8 * lane;
    const int kk = k < H ? k : 0;
    xq[c] = *(const uint4 *)(xr + kk);
    wq[c] = *(const uint4 *)(wr + kk);
  }
  float acc = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    float t = acc;
    t = fmaf(bf16lo(xq[c].x), bf16lo(wq[c].x), t);
    t = fmaf(bf16hi(xq[c].x), bf16hi(wq[c].x), t);
    t = fmaf(bf16lo(xq[c].y), bf16lo(wq[c].y), t);
    t = fmaf(bf16hi(xq[c].y), bf16hi(wq[c].y), t);
    t = fmaf(bf16lo(xq[c].z), bf16lo(wq[c].z), t);
    t = fmaf(bf16hi(xq[c].z), bf16hi(wq[c].z), t);
    t = fmaf(bf16lo(xq[c].w), bf16lo(wq[c].w), t);
    t = fmaf(bf16hi(xq[c].w), bf16hi(wq[c].w), t);
    acc = (c * 512 + 8 * lane < H) ? t : acc;
  }
  return acc;
}

static __device__ __forceinline__ float gate_row_sum(const uint16_t *__restrict__ xr, const uint16_t *__restrict__ wr,
                                                     const int H, const int lane) {
  float acc = 0.f;
  const int nch = (H + 511) >> 9;  // wave-uniform
  switch (nch) {
    case 1: acc = gate_row_partial<1>(xr, wr, H, lane); break;
    case 2: acc = gate_row_partial<2>(xr, wr, H, lane); break;
    case 3: acc = gate_row_partial<3>(xr, wr, H, lane); break;
    case 4: acc = gate_row_partial<4>(xr, wr, H, lane); break;
    case 5: acc = gate_row_partial<5>(xr, wr, H, lane); break;
    case 6: acc = gate_row_partial<6>(xr, wr, H, lane); break;
    case 7: acc = gate_row_partial<7>(xr, wr, H, lane); break;
    case 8: acc = gate_row_partial<8>(xr, wr, H, lane); break;
    default:
      for (int c = 0; c < H; c += 512) {
        const int k = c + 8 * lane;
        if (k < H) {
          const uint4 xv = *(const uint4 *)(xr + k);
          const uint4 wv = *(const uint4 *)(wr + k);
          acc = fmaf(bf16lo(xv.x), bf16lo(wv.x), acc);
          acc = fmaf(bf16hi(xv.x), bf16hi(wv.x), acc);
          acc = fmaf(bf16lo(xv.y), bf16lo(wv.y), acc);
          acc = fmaf(bf16hi(xv.y), bf16hi(wv.y), acc);
          acc = fmaf(bf16lo(xv.z), bf16lo(wv.z), acc);
          acc = fmaf(bf16hi(xv.z), bf16hi(wv.z), acc);
          acc = fmaf(bf16lo(xv.w), bf16lo(wv.w), acc);
          acc = fmaf(bf16hi(xv.w), bf16hi(wv.w), acc);
        }
      }
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc = acc + __shfl_xor(acc, m, 64);
  return acc;
}

// ---------------------------------------------------------------------------
// k1a gate logits: one wave per (token, expert row)
// ---------------------------------------------------------------------------
// (wg2, bias2, logits2, E2, ldl2: a second matrix over the same activations whose rows follow the first one's in
// the grid, or E2 = 0: the built-in predictor's score rows ride in the layer's own gate launch)
__global__ __launch_bounds__(256) void k_gate_logits(const uint16_t *__restrict__ x,
                                                      const uint16_t *__restrict__ wg,
                                                      const float *__restrict__ bias,
                                                      float *__restrict__ logits, int H, int E,
                                                      int ldl, const uint16_t *__restrict__ wg2,
                                                      const float *__restrict__ bias2,
                                                      float *__restrict__ logits2, int E2, int ldl2) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int e = blockIdx.x * 4 + w;
  const int t = blockIdx.y;
  const int nb1 = (E + 3) >> 2;
  if ((int)blockIdx.x >= nb1) {  // uniform per workgroup
    e = ((int)blockIdx.x - nb1) * 4 + w;
    wg = wg2; bias = bias2; logits = logits2; E = E2; ldl = ldl2;
  }
  if (e >= E) return;
  // (requested in front of the row: behind the sum it is one more trip to memory)
  const float bias_e = bias ? bias[e] : 0.f;
  asm volatile("" :: "v"(bias_e));
  const float acc = gate_row_sum(x + (size_t)t * H, wg + (size_t)e * H, H, lane);
  if (lane == 0) logits[(size_t)t * ldl + e] = bias ? acc + bias_e : acc;
}

// Large T: a workgroup takes 16 tokens (8 waves x 2) and a group of gate rows.  The rows are staged in LDS once
// per workgroup; a wave keeps the activations of its two tokens in registers as fp32 (the lane's columns
// 512 c + 8 lane + j) and walks the rows, so a gate row is fetched once per 16 tokens, converted once per two,
// and the inner loop is one LDS read per eight fma's of each token.  Each (token, row) sum is formed in exactly
// the order of k_gate_logits (lane partials over k = 512 c + 8 lane + j with one fma chain, then the xor
// butterfly 32..1): same bits.
#define GATE_WAVES 8
#define GATE_TW 2                        // tokens per wave
#define GATE_TT (GATE_WAVES * GATE_TW)  // tokens per workgroup
template <int NCH>  // 512-column chunks of a row (H <= 512 NCH)
__global__ __launch_bounds__(64 * GATE_WAVES) void k_gate_logits_rows(const uint16_t *__restrict__ x,
                                                                      const uint16_t *__restrict__ wg,
                                                                      const float *__restrict__ bias,
                                                                      float *__restrict__ logits, int T, int H,
                                                                      int E, int ldl, int rows_per_block) {
  extern __shared__ uint4 gws[];  // [rows of this workgroup][H/8]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int vpr = H >> 3;
  const int e0 = blockIdx.y * rows_per_block;
  const int nrow = (E - e0) < rows_per_block ? (E - e0) : rows_per_block;
  const uint4 *wsrc = (const uint4 *)(wg + (size_t)e0 * H);
  for (int i = tid; i < nrow * vpr; i += 64 * GATE_WAVES) gws[i] = wsrc[i];
  const int t0 = blockIdx.x * GATE_TT + w * GATE_TW;
  float xf[GATE_TW][NCH][8];
#pragma unroll
  for (int t = 0; t < GATE_TW; ++t) {
    const int tt = (t0 + t) < T ? (t0 + t) : T - 1;  // a token past the end repeats the last one (not stored)
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int k = c * 512 + 8 * lane;
      const uint4 v = k < H ? *(const uint4 *)(x + (size_t)tt * H + k) : make_uint4(0, 0, 0, 0);
      xf[t][c][0] = bf16lo(v.x); xf[t][c][1] = bf16hi(v.x); xf[t][c][2] = bf16lo(v.y); xf[t][c][3] = bf16hi(v.y);
      xf[t][c][4] = bf16lo(v.z); xf[t][c][5] = bf16hi(v.z); xf[t][c][6] = bf16lo(v.w); xf[t][c][7] = bf16hi(v.w);
    }
  }
  __syncthreads();
  // four rows per trip (rows past the end are clamped and not stored): eight independent chains.  Their eight
  // butterflies run as one: at the steps 32, 16 and 8 a lane keeps one half of its values and sends the other, so
  // every sum has the operands the plain butterfly gives it (own + partner's, and a + b = b + a), with 10
  // exchanges instead of 48.  Lane L then holds the sum of chain 4 (L>>3 & 1) + 2 (L>>4 & 1) + (L>>5 & 1).
  constexpr int GR = 4;
  const bool h32 = lane & 32, h16 = lane & 16, h8 = lane & 8;
  const int mine = 4 * ((lane >> 3) & 1) + 2 * ((lane >> 4) & 1) + ((lane >> 5) & 1);  // chain = 2 * row + token
  for (int r = 0; r < nrow; r += GR) {
    float acc[GR * GATE_TW];
#pragma unroll
    for (int i = 0; i < GR * GATE_TW; ++i) acc[i] = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int k = c * 512 + 8 * lane;
      if (k < H) {
#pragma unroll
        for (int q = 0; q < GR; ++q) {
          const int rq = r + q < nrow ? r + q : nrow - 1;
          const uint4 wv = gws[rq * vpr + (k >> 3)];
          const float wf[8] = {bf16lo(wv.x), bf16hi(wv.x), bf16lo(wv.y), bf16hi(wv.y),
                               bf16lo(wv.z), bf16hi(wv.z), bf16lo(wv.w), bf16hi(wv.w)};
#pragma unroll
          for (int t = 0; t < GATE_TW; ++t) {
            float a = acc[q * GATE_TW + t];
#pragma unroll
            for (int j = 0; j < 8; ++j) a = fmaf(xf[t][c][j], wf[j], a);
            acc[q * GATE_TW + t] = a;
          }
        }
      }
    }
    static_assert(GR * GATE_TW == 8, "the reduction below folds eight chains");
    float u[4], v2[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float keep = h32 ? acc[2 * i + 1] : acc[2 * i], send = h32 ? acc[2 * i] : acc[2 * i + 1];
      u[i] = keep + __shfl_xor(send, 32, 64);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const float keep = h16 ? u[2 * i + 1] : u[2 * i], send = h16 ? u[2 * i] : u[2 * i + 1];
      v2[i] = keep + __shfl_xor(send, 16, 64);
    }
    float z;
    {
      const float keep = h8 ? v2[1] : v2[0], send = h8 ? v2[0] : v2[1];
      z = keep + __shfl_xor(send, 8, 64);
    }
    z = z + __shfl_xor(z, 4, 64);
    z = z + __shfl_xor(z, 2, 64);
    z = z + __shfl_xor(z, 1, 64);
    const int rq = r + (mine >> 1), tq = t0 + (mine & 1);
    if ((lane & 7) == 0 && rq < nrow && tq < T)
      logits[(size_t)tq * ldl + e0 + rq] = bias ? z + bias[e0 + rq] : z;
  }
}

// ---------------------------------------------------------------------------
// k1b top-k: one wave per token, E <= 256
// ---------------------------------------------------------------------------
// The top-k of one token by one wave: lane l holds logits l, l + 64, ... (NR columns in use, E <= 64 NR).  k rounds of
// a wave-wide maximum (DPP row shifts and broadcasts: no LDS round trips); the winner of a round is the lowest expert
// id that holds the maximum (lowest column first, then lowest lane).  Lane j keeps the j-th choice, so the softmax
// terms of the choices are one expf per lane, added in choice order.  COH: the logits were written by other
// workgroups of this very launch and are read at device scope, past the L1.  s_idx / s_mask (LDS, optional): the
// indices again and the token's experts as a bit mask [4 x 64], for a dispatch in the same kernel.
template <int NR, bool COH>
static __device__ __forceinline__ void topk_token(const float *__restrict__ row, const int E, const int k, const int mode,
                                                  const int lane, int *__restrict__ idx, float *__restrict__ wout,
                                                  int *s_idx, unsigned long long *s_mask) {
  const float NEG = -__builtin_inff();
  float v[NR], v0[NR];
  unsigned long long msel[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int e = lane + 64 * r;
    v[r] = (e < E) ? (COH ? __hip_atomic_load(row + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : row[e]) : NEG;
    v0[r] = v[r];
    msel[r] = 0ull;
  }
  float my_v = 0.f;  // lane j keeps the j-th selected logit
  for (int j = 0; j < k; ++j) {
    float bvl = v[0];
#pragma unroll
    for (int r = 1; r < NR; ++r) bvl = fmaxf(bvl, v[r]);
    const float bv = wave_max_f32(bvl);
    int wr = -1, wl = 0;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const unsigned long long mr = __ballot(v[r] == bv);
      if (wr < 0 && mr) { wr = r; wl = (int)__builtin_ctzll(mr); }
    }
    if (wr < 0) { wr = 0; wl = j; }  // NaN logits match nothing: stay inside the expert range
#pragma unroll
    for (int r = 0; r < NR; ++r)
      if (r == wr) {
        if (lane == wl) v[r] = NEG;
        msel[r] |= 1ull << wl;
      }
    if (lane == j) {
      my_v = bv;
      const int bi = wl + 64 * wr;
      idx[j] = bi;
      if (s_idx) s_idx[j] = bi;
    }
  }
  if (s_mask && lane == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) s_mask[r] = r < NR ? msel[r < NR ? r : 0] : 0ull;
  }
  // weights: the row maximum is the first choice; the softmax denominator over all E per lane in column order, then
  // the xor butterfly; the sum over the choices in choice order
  const float mx = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_v), 0));
  float den = 0.f;
#pragma unroll
  for (int r = 0; r < NR; ++r)
    if (lane + 64 * r < E) den += expf(v0[r] - mx);
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) den = den + __shfl_xor(den, m, 64);
  const float ex = expf(my_v - mx);
  float sum_sel = 0.f;
  for (int j = 0; j < k; ++j)
    sum_sel += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ex), j));
  float wgt;
  if (mode == MOE_ROUTE_TOPK_SOFTMAX) {
    wgt = ex / sum_sel;
  } else {
    wgt = ex / den;
    if (mode == MOE_ROUTE_SOFTMAX_TOPK_RENORM) wgt = wgt / (sum_sel / den);
  }
  if (lane < k) wout[lane] = wgt;
}

__global__ __launch_bounds__(256) void k_topk(const float *__restrict__ logits, int T, int E,
                                               int ldl, int k, int mode, int *__restrict__ idx,
                                               float *__restrict__ wout) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + w;
  if (t >= T) return;
  const float *row = logits + (size_t)t * ldl;
  int *ir = idx + (size_t)t * k;
  float *wr = wout + (size_t)t * k;
  // one instantiation per number of 64-wide logit columns: a 64-expert layer pays for one
  if (E <= 64) topk_token<1, false>(row, E, k, mode, lane, ir, wr, nullptr, nullptr);
  else if (E <= 128) topk_token<2, false>(row, E, k, mode, lane, ir, wr, nullptr, nullptr);
  else topk_token<4, false>(row, E, k, mode, lane, ir, wr, nullptr, nullptr);
}

// ---------------------------------------------------------------------------
// k2 dispatch: single workgroup, LDS histogram -> scan -> stable permutation
// ---------------------------------------------------------------------------
#define DISP_MAXE 1024
#define DISP_THREADS 1024
__global__ __launch_bounds__(DISP_THREADS) void k_dispatch(
    const int *__restrict__ idx, int P, int k, int E, int nbits, int *__restrict__ counts,
    int *__restrict__ offsets, int *__restrict__ sorted_pair, int *__restrict__ pos_of_pair,
    int *__restrict__ sorted_tok, moe_unit *__restrict__ units, int *__restrict__ n_active,
    long long *__restrict__ active_ids, int max_units) {
  __shared__ int s_cnt[DISP_MAXE];
  __shared__ int s_off[DISP_MAXE + 1];
  __shared__ int s_run[DISP_MAXE];
  __shared__ int s_uidx[DISP_MAXE];
  __shared__ int s_wsum[16], s_wact[16], s_tot;
  extern __shared__ int s_w[];  // [16][E]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;

  for (int e = tid; e < E; e += DISP_THREADS) { s_cnt[e] = 0; s_run[e] = 0; }
  __syncthreads();
  for (int p = tid; p < P; p += DISP_THREADS) {
    const int e = idx[p];
    if ((unsigned)e < (unsigned)E) atomicAdd(&s_cnt[e], 1);
  }
  __syncthreads();
  // exclusive scan over experts (thread e owns expert e; E <= 1024)
  {
    const int c = (tid < E) ? s_cnt[tid] : 0;
    const int a = c > 0 ? 1 : 0;
    int sc = c, sa = a;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int oc = __shfl_up(sc, d, 64), oa = __shfl_up(sa, d, 64);
      if (lane >= d) { sc += oc; sa += oa; }
    }
    if (lane == 63) { s_wsum[w] = sc; s_wact[w] = sa; }
    __syncthreads();
    int bc = 0, ba = 0;
    for (int i = 0; i < w; ++i) { bc += s_wsum[i]; ba += s_wact[i]; }
    const int excl = bc + sc - c, uidx = ba + sa - a;
    if (tid < E) {
      s_off[tid] = excl;
      s_uidx[tid] = uidx;
      counts[tid] = c;
      offsets[tid] = excl;
      if (a && uidx < max_units) {
        moe_unit u; u.expert = tid; u.m = c; u.row0 = excl; u.pad = 0;
        units[uidx] = u;
        active_ids[uidx] = tid;
      }
    }
    if (tid == DISP_THREADS - 1) {
      const int tot_act = ba + sa;
      offsets[E] = bc + sc;
      s_off[E] = bc + sc;
      *n_active = tot_act < max_units ? tot_act : max_units;
      s_tot = tot_act;
    }
    __syncthreads();
    const int tot_act = s_tot;
    for (int u = tot_act + tid; u < max_units; u += DISP_THREADS) {
      moe_unit z; z.expert = -1; z.m = 0; z.row0 = 0; z.pad = 0;
      units[u] = z;
      active_ids[u] = -1;
    }
  }
  __syncthreads();
  // stable ranking, 1024 pairs at a time
  for (int base = 0; base < P; base += DISP_THREADS) {
    for (int i = tid; i < 16 * E; i += DISP_THREADS) s_w[i] = 0;
    __syncthreads();
    const int p = base + tid;
    int e = (p < P) ? idx[p] : -1;
    const bool valid = (unsigned)e < (unsigned)E;
    unsigned long long peers = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (e >> b) & 1;
      const unsigned long long bal = __ballot(valid && bit);
      peers &= bit ? bal : ~bal;
    }
    const int rank = __popcll(peers & ((1ull << lane) - 1ull));
    if (valid && rank == 0) s_w[w * E + e] = __popcll(peers);
    __syncthreads();
    for (int ee = tid; ee < E; ee += DISP_THREADS) {
      int run = s_run[ee];
      for (int ww = 0; ww < 16; ++ww) {
        const int c = s_w[ww * E + ee];
        s_w[ww * E + ee] = run;
        run += c;
      }
      s_run[ee] = run;
    }
    __syncthreads();
    if (valid) {
      const int pos = s_off[e] + s_w[w * E + e] + rank;
      sorted_pair[pos] = p;
      pos_of_pair[p] = pos;
      sorted_tok[pos] = p / k;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// k2 for prefill batches: the same arrays from P / 1024 workgroups in one launch.  A workgroup ranks its own
// (at most 1024) consecutive pairs as k_dispatch does and stores its per-expert counts; once every workgroup
// has done so (a counter in the workspace tells; all of them are resident, the grid is at most 64) each one adds
// up the counts of all (the totals, hence the offsets) and of the workgroups before it (where its own pairs of an
// expert start), and scatters.  The barrier words are zero at launch and are left zero.  A workgroup that waits
// longer than a second raises the error word and goes on with what it has (positions stay inside the arrays).
// ---------------------------------------------------------------------------
#define DISPM_MAXB 64
__global__ __launch_bounds__(DISP_THREADS) void k_dispatch_multi(
    const int *__restrict__ idx, int P, int chunk, int k, int E, int nbits, int *__restrict__ counts,
    int *__restrict__ offsets, int *__restrict__ sorted_pair, int *__restrict__ pos_of_pair,
    int *__restrict__ sorted_tok, moe_unit *__restrict__ units, int *__restrict__ n_active,
    long long *__restrict__ active_ids, int max_units, int *hist, unsigned *sync, int *err) {
  __shared__ int s_base[256], s_all[256], s_pre[256];  // E <= 256 (checked by the launcher)
  __shared__ int s_wsum[16], s_wact[16], s_tot;
  extern __shared__ int s_w[];  // [16][E]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int b = blockIdx.x, NB = gridDim.x;
  // ---- stable rank of the workgroup's pairs among themselves ---------------------------------------
  const int p0 = b * chunk;
  const int np = (P - p0) < chunk ? (P - p0) : chunk;
  const int p = p0 + tid;
  const int e = tid < np ? idx[p] : -1;
  for (int i = tid; i < 16 * E; i += DISP_THREADS) s_w[i] = 0;
  if (tid < 256) { s_all[tid] = 0; s_pre[tid] = 0; }
  __syncthreads();
  const bool valid = (unsigned)e < (unsigned)E;
  unsigned long long peers = __ballot(valid);
  for (int bit_i = 0; bit_i < nbits; ++bit_i) {
    const bool bit = (e >> bit_i) & 1;
    const unsigned long long bal = __ballot(valid && bit);
    peers &= bit ? bal : ~bal;
  }
  const int rank = __popcll(peers & ((1ull << lane) - 1ull));
  if (valid && rank == 0) s_w[w * E + e] = __popcll(peers);
  __syncthreads();
  for (int ee = tid; ee < E; ee += DISP_THREADS) {
    int run = 0;
    for (int ww = 0; ww < 16; ++ww) {
      const int c = s_w[ww * E + ee];
      s_w[ww * E + ee] = run;
      run += c;
    }
    __hip_atomic_store(hist + (size_t)b * E + ee, run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // ---- every workgroup's counts are out ------------------------------------------------------------
  // (the counts are stored and read at device scope, past the caches that are not coherent between workgroups;
  // one thread orders them: its release follows the workgroup's barrier, its acquire precedes the next one)
  __syncthreads();
  if (tid == 0) {
    __hip_atomic_fetch_add(sync, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    const long long t_start = wall_clock64();
    int polls = 0;
    while (__hip_atomic_load(sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)NB) {
      if ((++polls & 63) == 0 && wall_clock64() - t_start > 100000000ll) {  // one second of the 100 MHz counter
        moe_raise_err(err);
        break;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  __syncthreads();
  // ---- totals, the counts of the workgroups in front, exclusive scan over experts (thread e owns expert e) ----
  {
    // all NB * E counts are requested at once (a thread per count, then LDS adds): one trip to memory
    for (int i = tid; i < NB * E; i += DISP_THREADS) {
      const int cb = __hip_atomic_load(hist + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int bb = i / E, ee = i - bb * E;
      if (cb) {
        atomicAdd(&s_all[ee], cb);
        if (bb < b) atomicAdd(&s_pre[ee], cb);
      }
    }
    __syncthreads();
    const int c = tid < E ? s_all[tid] : 0, pre = tid < E ? s_pre[tid] : 0;
    const int a = c > 0 ? 1 : 0;
    int sc = c, sa = a;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int oc = __shfl_up(sc, d, 64), oa = __shfl_up(sa, d, 64);
      if (lane >= d) { sc += oc; sa += oa; }
    }
    if (lane == 63) { s_wsum[w] = sc; s_wact[w] = sa; }
    __syncthreads();
    int bc = 0, ba = 0;
    for (int i = 0; i < w; ++i) { bc += s_wsum[i]; ba += s_wact[i]; }
    const int excl = bc + sc - c, uidx = ba + sa - a;
    if (tid < E) {
      s_base[tid] = excl + pre;
      if (b == 0) {
        counts[tid] = c;
        offsets[tid] = excl;
        if (a && uidx < max_units) {
          moe_unit u; u.expert = tid; u.m = c; u.row0 = excl; u.pad = 0;
          units[uidx] = u;
          active_ids[uidx] = tid;
        }
      }
    }
    if (tid == DISP_THREADS - 1) {
      const int tot_act = ba + sa;
      if (b == 0) {
        offsets[E] = bc + sc;
        *n_active = tot_act < max_units ? tot_act : max_units;
      }
      s_tot = tot_act;
    }
    __syncthreads();
    if (b == 0)
      for (int u = s_tot + tid; u < max_units; u += DISP_THREADS) {
        moe_unit z; z.expert = -1; z.m = 0; z.row0 = 0; z.pad = 0;
        units[u] = z;
        active_ids[u] = -1;
      }
  }
  if (valid) {
    const int pos = s_base[e] + s_w[w * E + e] + rank;
    sorted_pair[pos] = p;
    pos_of_pair[p] = pos;
    sorted_tok[pos] = p / k;
  }
  // the last workgroup through the barrier clears it for the next launch
  if (tid == 0) {
    if (__hip_atomic_fetch_add(sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)NB - 1u) {
      __hip_atomic_store(sync, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(sync + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ---------------------------------------------------------------------------
// k1+k2 fused for decode batches (T <= 16, E <= 256, T*k <= 512): the grid of k_gate_logits
// computes the logits (same arithmetic, same bits); the workgroup that finishes last (a
// device-scope counter tells it) then runs the top-k routing (one wave per token) and the
// stable dispatch on its own.  Three launches become one, and the logits are still spread
// over as many workgroups as before.  The counter must be zero at launch and is left zero.
// ---------------------------------------------------------------------------
#define ROUTE_MAXT 64
#define ROUTE_MAXP 512
struct RouteArgs {
  const uint16_t *x, *wg;
  const float *bias;
  float *logits;
  int T, H, E, Erows, ldl, k, mode, nbits, max_units;
  int *idx; float *w;
  int *counts, *offsets, *sorted_pair, *pos_of_pair, *sorted_tok;
  moe_unit *units; int *n_active; long long *active_ids;
  unsigned *counter;
  moe_unit *host_units; int *host_n_active; int *host_seq; int host_seq_val, pad_;
  // k_gate_route: bias rows, the hand-over area of the gate rows (copies of g_copy_words words: one per part of the
  // chip and a device-scope one), the launch's sequence number, and the word raised when the hand-over times out
  int n_bias, g_seq, g_copy_words, g_parts;  // g_parts: 8 = every item once per part of the chip, 1 = once
  unsigned long long *g_stamp;
  int *err;
};

// top-k (one wave per token) and stable dispatch by ONE workgroup of NW waves; the bodies of
// k_topk and k_dispatch.  With host_units set the unit list also goes straight into pinned host
// memory, followed (once those stores have completed) by the sequence word the host polls.
// NR: 64-wide logit columns in use (E <= 64 NR); COH: the logits were written by other workgroups of this very launch
// and are read at device scope, past the L1 (k_route_decode); a launch of its own reads them plainly
template <int NW, int NR, bool COH>
static __device__ __forceinline__ void route_tail_n(const RouteArgs &a, int *s_idx, unsigned long long *s_mask, int *s_off,
                                                    int *s_wsum, int *s_wact, int &s_tot) {
  constexpr int NT = NW * 64;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int E = a.E, T = a.T, k = a.k, P = T * k;
  // ---- phase 2: top-k, wave w takes tokens w, w+NW, ... (the selection, tie rule and weights of k_topk) -------
  // besides the indices, every token leaves the set of its experts as a bit mask: the dispatch below counts bits
  for (int t = w; t < T; t += NW)
    topk_token<NR, COH>(a.logits + (size_t)t * a.ldl, E, k, a.mode, lane, a.idx + (size_t)t * k, a.w + (size_t)t * k,
                        s_idx + t * k, s_mask + t * 4);
  __syncthreads();
  // ---- phase 3: dispatch (the arrays of k_dispatch).  A token holds an expert at most once, so the pairs of an
  // expert in pair order are its tokens in token order: count of expert e = tokens whose mask has bit e, position of
  // pair (t, e) = offset of e + tokens before t whose mask has bit e.  Thread e owns expert e; three barriers. ----
  {
    int c = 0;
    if (tid < E) {
      const int r = tid >> 6, bit = tid & 63;
      for (int t = 0; t < T; ++t) c += (int)((s_mask[t * 4 + r] >> bit) & 1ull);
    }
    const int act = c > 0 ? 1 : 0;
    int sc = c, sa = act;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int oc = __shfl_up(sc, d, 64), oa = __shfl_up(sa, d, 64);
      if (lane >= d) { sc += oc; sa += oa; }
    }
    if (lane == 63) { s_wsum[w] = sc; s_wact[w] = sa; }
    __syncthreads();
    int bc = 0, ba = 0;
    for (int i = 0; i < w; ++i) { bc += s_wsum[i]; ba += s_wact[i]; }
    const int excl = bc + sc - c, uidx = ba + sa - act;
    if (tid < E) {
      s_off[tid] = excl;
      a.counts[tid] = c;
      a.offsets[tid] = excl;
      if (act && uidx < a.max_units) {
        moe_unit u; u.expert = tid; u.m = c; u.row0 = excl; u.pad = 0;
        a.units[uidx] = u;
        a.active_ids[uidx] = tid;
        if (a.host_units) host_store_unit(a.host_units, uidx, tid, c, excl);
      }
    }
    if (tid == NT - 1) {
      const int tot_act = ba + sa;
      a.offsets[E] = bc + sc;
      *a.n_active = tot_act < a.max_units ? tot_act : a.max_units;
      if (a.host_units) host_store_i32(a.host_n_active, tot_act < a.max_units ? tot_act : a.max_units);
      s_tot = tot_act;
    }
    __syncthreads();
    for (int u = s_tot + tid; u < a.max_units; u += NT) {
      moe_unit z; z.expert = -1; z.m = 0; z.row0 = 0; z.pad = 0;
      a.units[u] = z;
      a.active_ids[u] = -1;
    }
  }
  for (int p = tid; p < P; p += NT) {
    const int e = s_idx[p], t = p / k;
    const int r = e >> 6, bit = e & 63;
    int rank = 0;
    for (int tt = 0; tt < t; ++tt) rank += (int)((s_mask[tt * 4 + r] >> bit) & 1ull);
    const int pos = s_off[e] + rank;
    a.sorted_pair[pos] = p;
    a.pos_of_pair[p] = pos;
    a.sorted_tok[pos] = t;
  }
  if (a.host_units) {
    host_stores_done();
    __syncthreads();
    if (tid == 0) __hip_atomic_store(a.host_seq, a.host_seq_val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

template <int NW, bool COH>
static __device__ __forceinline__ void route_tail(const RouteArgs &a, int *s_idx, unsigned long long *s_mask, int *s_off,
                                                  int *s_wsum, int *s_wact, int &s_tot) {
  // one instantiation per number of logit columns: a 64-expert layer pays for one
  if (a.E <= 64) route_tail_n<NW, 1, COH>(a, s_idx, s_mask, s_off, s_wsum, s_wact, s_tot);
  else if (a.E <= 128) route_tail_n<NW, 2, COH>(a, s_idx, s_mask, s_off, s_wsum, s_wact, s_tot);
  else route_tail_n<NW, 4, COH>(a, s_idx, s_mask, s_off, s_wsum, s_wact, s_tot);
}

__global__ __launch_bounds__(256) void k_route_decode(const RouteArgs a) {
  __shared__ int s_last;
  __shared__ int s_idx[ROUTE_MAXP];
  __shared__ unsigned long long s_mask[ROUTE_MAXT * 4];
  __shared__ int s_off[257];
  __shared__ int s_wsum[4], s_wact[4], s_tot;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int H = a.H, E = a.E, T = a.T, k = a.k, P = T * k;
  // ---- phase 1: one wave per (token, gate row) ------------------------------------------
  {
    const int e = blockIdx.x * 4 + w, t = blockIdx.y;
    if (e < a.Erows) {
      const uint16_t *xr = a.x + (size_t)t * H;
      const uint16_t *wr = a.wg + (size_t)e * H;
      float acc = 0.f;
      for (int c = 0; c < H; c += 512) {
        const int kk = c + 8 * lane;
        if (kk < H) {
          const uint4 xv = *(const uint4 *)(xr + kk);
          const uint4 wv = *(const uint4 *)(wr + kk);
          acc = fmaf(bf16lo(xv.x), bf16lo(wv.x), acc);
          acc = fmaf(bf16hi(xv.x), bf16hi(wv.x), acc);
          acc = fmaf(bf16lo(xv.y), bf16lo(wv.y), acc);
          acc = fmaf(bf16hi(xv.y), bf16hi(wv.y), acc);
          acc = fmaf(bf16lo(xv.z), bf16lo(wv.z), acc);
          acc = fmaf(bf16hi(xv.z), bf16hi(wv.z), acc);
          acc = fmaf(bf16lo(xv.w), bf16lo(wv.w), acc);
          acc = fmaf(bf16hi(xv.w), bf16hi(wv.w), acc);
        }
      }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) acc = acc + __shfl_xor(acc, m, 64);
      if (lane == 0) a.logits[(size_t)t * a.ldl + e] = (a.bias && e < E) ? acc + a.bias[e] : acc;
    }
  }
  // ---- who is last? ------------------------------------------------------------------------
  // (one thread orders the workgroup's logits: its release follows the barrier, and the last workgroup's acquire
  // precedes the next one; a fence by every wave costs several microseconds of cache write-backs)
  __syncthreads();
  if (tid == 0) {
    const unsigned prev = __hip_atomic_fetch_add(a.counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    s_last = prev == gridDim.x * gridDim.y - 1u;
    if (s_last) __hip_atomic_store(a.counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last) return;
  route_tail<4, true>(a, s_idx, s_mask, s_off, s_wsum, s_wact, s_tot);
}

// k1b + k2 in one launch for decode batches whose logits exist already: one workgroup of NW waves
// (a wave per token in the top-k phase: 4 waves are enough for T <= 4 and their barriers are cheaper)
template <int NW>
__global__ __launch_bounds__(64 * NW) void k_topk_dispatch(const RouteArgs a) {
  __shared__ int s_idx[ROUTE_MAXP];
  __shared__ unsigned long long s_mask[ROUTE_MAXT * 4];
  __shared__ int s_off[257];
  __shared__ int s_wsum[NW], s_wact[NW], s_tot;
  route_tail<NW, false>(a, s_idx, s_mask, s_off, s_wsum, s_wact, s_tot);
}

// ---------------------------------------------------------------------------
// k3 int4 grouped GEMV (decode).  One workgroup (4 waves) owns two adjacent
// 16-row blocks of one unit's matrix; wave w takes the K groups w, w+4, w+8, ...
//   SWIGLU: blocks are (gate rows, up rows) -> out = silu(g)*u, bf16, 16 values
//   else  : plain product, fp32, 32 values
// The load section is straight-line code (clamped addresses instead of branches):
// activations and scale/zero sections first, then the weight tiles, so that the small
// loads can be staged in LDS while the tiles are still in flight.
// ---------------------------------------------------------------------------
struct GemvClass {
  const uint16_t *act;  // bf16 activations [rows, act_stride] (act_stride 0: one shared row)
  const int *gather;    // row -> activation row (NULL = identity)
  void *out;            // bf16 (SWIGLU) or fp32
  long long off_q, off_s, off_z;
  int K, G, act_stride, out_stride, nblk;
  int ksplit;           // q4_K, shared expert's w2 pass: workgroups per block pair, each over 1/ksplit of the
                        // reduction, partial rows to out + split * T * out_stride (0 or 1: the whole reduction)
};
#define GEMV_MAX_KUNITS 64
struct KUnit { unsigned long long base; int m, row0; };
struct GemvArgs {
  GemvClass cls[2];  // 0 = shared expert, 1 = routed experts
  const moe_unit *units;                 // device-built unit list (NULL: use ku[])
  const unsigned long long *expert_ptr;  // device slot table, indexed by expert id
  const unsigned char *shared_base;
  int n_sh_blocks, T;
  int *err;
  union {
    KUnit ku[GEMV_MAX_KUNITS];           // units resolved on the host, passed by value: the
                                         // weight loads then depend on no global load
    // tab_n > 0 (launches that take their units from device memory and so leave ku unused): the slot table of
    // experts 0 .. tab_n - 1 by value.  The device table is then not read, and no copy that refreshes it has to
    // stand in the stream in front of the launch.
    unsigned long long tab[GEMV_MAX_KUNITS];
  };
  int tab_n, tab_pad;
  // one-token launches that route inside the kernel (ROUTE): inputs and the routing outputs
  const float *r_logits;
  int r_E, r_k, r_mode, r_pad;
  int *r_idx; float *r_w;
  int *r_counts, *r_offsets, *r_sorted_pair, *r_pos_of_pair, *r_sorted_tok;
  moe_unit *r_units; int *r_n_active; long long *r_active_ids;
  // optional copy of the unit list straight into pinned host memory, then a sequence word
  moe_unit *r_host_units; int *r_host_seq; int r_host_seq_val, r_pad2;
  // w13 launches of a decode batch can carry the step's unit list (made by an earlier launch) to the host:
  // one more workgroup at the end of the grid copies it into pinned host memory and then stores the sequence word
  moe_unit *p_host_units; int *p_host_n_active; int *p_host_seq; const int *p_n_active;
  int p_seq_val, p_max_units;
  KUnit *r_kunits;              // routing publisher: resolved units (slot address, rows) for the w2 pass
  float *r_unit_w;              // and the routing weight per unit position
  const KUnit *kunits_dev;      // device-side resolved units: one load instead of unit -> table -> address
  // one-token launches that also compute the gate logits: the first g_nblk workgroups sum the g_rows gate rows
  // (a wave per row, once per part of the chip) and hand each logit to the routing waves of the same launch as a
  // (value, g_seq) pair; g_nblk = 0: the logits come from an earlier launch (r_logits)
  const uint16_t *g_w; const float *g_bias; unsigned long long *g_stamp; float *g_logits_out;
  int g_rows, g_nbias, g_nblk, g_seq;
  int unit_slots;               // chunked-K launches of more than 16 tokens: slots of `units` when at most 64, else 0
  int pairs;                    // T k of the step (0: unknown)
  int row_split;                // w2 launches of more than 32 tokens: a unit of more than 32 rows has two workgroups
                                // per group of block pairs, rows 0..31 and 32.., and so has the shared expert
  // w13 launches of a decode batch that sum the gate rows and route by themselves (k_gemv_int4_mfma<.., ROUTE>):
  // 8-byte words per copy of the hand-over area, row stride of the logits in memory
  int g_copy_words, g_ldl;
  // workgroups from this grid index on first look for the routing that an earlier workgroup on their part of the
  // chip has left behind (they start when the first round of workgroups ends)
  int g_cache_from;
  int g_parts;   // 8: the gate rows are summed once per part of the chip (hand-over through that part's second-level
                 // cache), 1: once, handed over at device scope
};

// Gate logits handed over inside a launch.  A logit travels as one 8-byte word (value, sequence number of the
// launch), so a reader needs no flag and no fence: it polls the words until all of them carry its launch's number.
// The numbers of successive launches on one workspace differ, so a word left by an earlier launch is never taken
// for a new one and nothing has to be cleared.
// The chip has eight parts (XCDs), each with its own second-level cache, which is the point of coherence for the
// compute units of that part only.  A word written at device scope (past those caches) took 1.5 to 2.5 us to
// become visible while the launch's weight streams were running, against 0.3 us through the second-level cache
// of one part.  So the gate rows are summed once PER PART (the gate workgroups come in groups of eight, workgroup i
// lands on part i mod 8; each reads its real part number from the hardware register and writes the copy of that
// part), and a routing wave polls the copy of the part it runs on with loads that bypass the first-level cache.
// Nothing depends on where the hardware places a workgroup: the gate workgroups of the first group also write
// every word at device scope into a ninth copy, and a routing wave whose own part's copy stays incomplete for
// GATE_LOCAL_SPINS polls goes on with that one.
#define GATE_PARTS 8
#define GATE_COPIES (GATE_PARTS + 1)  // one per part + the device-scope copy
#define GATE_COPY_WORDS 512           // 8-byte words per copy (E + 1 <= 257 in use)
#define GATE_LOCAL_SPINS 64u
#define GATE_POLL_LIMIT (1u << 20)
static __device__ __forceinline__ int xcc_id() {  // HW_REG_XCC_ID, bits 3:0
  return (int)(__builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11)) & (GATE_PARTS - 1));
}
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

#ifdef MOE_STAMPS
static __device__ unsigned long long g_stamps[1024 * 8];
#define STAMP(i) do { if (lane == 0 && blockIdx.x < 1024) g_stamps[blockIdx.x * 8 + (i)] = wall_clock64(); } while (0)
#define STAMPV(i, v) do { if (lane == 0 && blockIdx.x < 1024) g_stamps[blockIdx.x * 8 + (i)] = (v); } while (0)
extern "C" int moe_debug_stamps_read(void *dst) { return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_stamps), sizeof(g_stamps)); }
#else
#define STAMP(i)
#define STAMPV(i, v)
#endif
static __device__ __forceinline__ void gate_rows_stamped(const GemvArgs &a, const int lane, const int w) {
  const int e = ((int)blockIdx.x >> 3) * 4 + w;   // eight workgroups (one per part of the chip) per block of four rows
  if (e >= a.g_rows) return;
  if (w == 0) { STAMP(0); STAMPV(7, (unsigned long long)xcc_id()); }
  const int H = a.cls[1].K;
  // (requested in front of the row: behind the sum it was one more trip to memory, 0.1 to 2 us)
  const float bias_e = (a.g_bias && e < a.g_nbias) ? a.g_bias[e] : 0.f;
  asm volatile("" :: "v"(bias_e));
  const float acc = gate_row_sum(a.cls[1].act, a.g_w + (size_t)e * H, H, lane);
  const float val = (a.g_bias && e < a.g_nbias) ? acc + bias_e : acc;
  const u32x2_t word = {__float_as_uint(val), (u32)a.g_seq};
  if (w == 0) STAMP(5);
  if (lane == 0)  // into the second-level cache of this part
    __builtin_amdgcn_raw_buffer_store_b64(word, make_rsrc(a.g_stamp + (size_t)xcc_id() * GATE_COPY_WORDS, GATE_COPY_WORDS * 8),
                                          e * 8, 0, 1 /* sc0 */);
  if (((int)blockIdx.x & 7) == 0) {
    const unsigned long long word64 = ((unsigned long long)word.y << 32) | word.x;
    if (lane == 1)
      __hip_atomic_store(a.g_stamp + (size_t)GATE_PARTS * GATE_COPY_WORDS + e, word64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (lane == 0) a.g_logits_out[e] = val;  // for the kernels behind this launch (and the host)
  }
#ifdef MOE_STAMPS
  if (w == 0) { asm volatile("" ::: "memory"); STAMP(1); asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); STAMP(2); }
#endif
}

// k1a + k1b + k2 in one launch for decode batches (2 to 32 tokens): workgroup 0 is the routing workgroup of
// k_topk_dispatch, the others sum the gate rows and hand every logit to it as a (value, sequence number) word, the
// way the one-token launch does (see gate_rows_stamped): each work item (a token and NW gate rows, a wave per row,
// the summation order of k_gate_logits) is done by eight workgroups in a row, one per part of the chip in the
// usual placement; each writes the copy of the part it finds itself on through that part's second-level cache,
// the first of the eight also a device-scope copy and the plain logits for the kernels behind this launch.  The
// routing workgroup polls the copy of its own part (a thread per word, loads past the first-level cache) and
// after GATE_LOCAL_SPINS rounds the device-scope copy, keeps the logits in LDS and goes on as k_topk_dispatch.
// A word that never arrives raises *err after GATE_POLL_LIMIT rounds instead of holding the launch.
#define GROUTE_MAX_ROWS 264  // LDS row stride of the logits: E <= 256 and a shared-gate row, padded
template <int NW>
__global__ __launch_bounds__(64 * NW) void k_gate_route(const RouteArgs a) {
  __shared__ int s_idx[ROUTE_MAXP];
  __shared__ unsigned long long s_mask[ROUTE_MAXT * 4];
  __shared__ int s_off[257];
  __shared__ int s_wsum[NW], s_wact[NW], s_tot;
  __shared__ float s_logits[(NW == 4 ? 4 : 32) * GROUTE_MAX_ROWS];
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int T = a.T, Erows = a.Erows, H = a.H;
  if (blockIdx.x > 0) {
    const int q = (int)blockIdx.x - 1;
    const bool per_part = a.g_parts == GATE_PARTS;
    const int item = per_part ? q >> 3 : q;
    const int nrb = (Erows + NW - 1) / NW;
    const int t = item / nrb, e = (item - t * nrb) * NW + w;
    if (e >= Erows) return;
    const bool biased = a.bias && e < a.n_bias;
    const float bias_e = biased ? a.bias[e] : 0.f;
    asm volatile("" :: "v"(bias_e));  // requested in front of the row
    const float acc = gate_row_sum(a.x + (size_t)t * H, a.wg + (size_t)e * H, H, lane);
    const float val = biased ? acc + bias_e : acc;
    const u32x2_t word = {__float_as_uint(val), (u32)a.g_seq};
    const int wi = t * Erows + e;
    if (per_part && lane == 0)
      __builtin_amdgcn_raw_buffer_store_b64(word, make_rsrc(a.g_stamp + (size_t)xcc_id() * a.g_copy_words,
                                                            (u32)a.g_copy_words * 8u), wi * 8, 0, 1 /* sc0 */);
    if (!per_part || (q & 7) == 0) {
      const unsigned long long word64 = ((unsigned long long)word.y << 32) | word.x;
      if (lane == 1)
        __hip_atomic_store(a.g_stamp + (size_t)GATE_PARTS * a.g_copy_words + wi, word64, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0) a.logits[(size_t)t * a.ldl + e] = val;
    }
    return;
  }
  // the routing workgroup: collect the logits
  {
    const rsrc_t rl = make_rsrc(a.g_stamp + (size_t)xcc_id() * a.g_copy_words, (u32)a.g_copy_words * 8u);
    const unsigned long long *cg = a.g_stamp + (size_t)GATE_PARTS * a.g_copy_words;
    const int nw = T * Erows;
    const unsigned local_spins = a.g_parts == GATE_PARTS ? GATE_LOCAL_SPINS : 0u;
    bool timeout = false;
    for (int wi = tid; wi < nw; wi += 64 * NW) {
      unsigned spins = 0;
      u32x2_t word;
      for (;;) {
        if (spins < local_spins) {
          word = __builtin_amdgcn_raw_buffer_load_b64(rl, wi * 8, 0, 16 /* sc1: past the first-level cache */);
        } else {
          const unsigned long long w64 = __hip_atomic_load(cg + wi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          word.x = (u32)w64; word.y = (u32)(w64 >> 32);
        }
        if ((int)word.y == a.g_seq) break;
        if (++spins >= GATE_POLL_LIMIT) { timeout = true; break; }
        __builtin_amdgcn_s_sleep(2);
      }
      const int t = wi / Erows;
      s_logits[t * GROUTE_MAX_ROWS + (wi - t * Erows)] = __uint_as_float(word.x);
    }
    if (timeout && a.err) moe_raise_err(a.err);
  }
  __syncthreads();
  RouteArgs b = a;
  b.logits = s_logits;  // (generic loads from LDS)
  b.ldl = GROUTE_MAX_ROWS;
  route_tail<NW, false>(b, s_idx, s_mask, s_off, s_wsum, s_wact, s_tot);
}

// Work item of a GEMV workgroup, resolved from the kernel arguments without dependent
// loads when the units travel by value: both classes and the first 8 units are fetched
// in one batch of scalar loads and selected with scalar ops (a dependent second fetch
// costs ~0.5 us of kernel time at these sizes).
struct GemvWork {
  GemvClass c;
  const unsigned char *base;
  int m, row0, b;
  int half;  // row_split: which half of the unit's rows
};
// The publishing workgroup of a w13 launch (the last one of its grid): the unit list of the step goes from device
// memory to the host's pinned copy while the other workgroups stream weights, then the sequence word the host
// polls.  In the routing kernel itself these stores held the launch for 1.8 us; here nothing waits for them.
static __device__ __forceinline__ void gemv_publish_units(const GemvArgs &a) {
  const int tid = threadIdx.x;
  int n = *a.p_n_active;
  n = n < a.p_max_units ? n : a.p_max_units;
  for (int u = tid; u < n; u += 256) {
    const moe_unit un = a.units[u];
    host_store_unit(a.p_host_units, u, un.expert, un.m, un.row0);
  }
  if (tid == 0) host_store_i32(a.p_host_n_active, n);
  host_stores_done();
  __syncthreads();
  if (tid == 0) __hip_atomic_store(a.p_host_seq, a.p_seq_val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Slot address of expert e: from the kernel arguments when the launch carries the table, else from the device table.
static __device__ __forceinline__ unsigned long long slot_of(const GemvArgs &a, const int e) {
  return a.tab_n > 0 ? (e < a.tab_n ? a.tab[e] : 0ull) : a.expert_ptr[e];
}
// The same for an expert id that is the same in every lane: the address comes back in scalar registers, so that the
// buffer descriptors made from it need no loop over the lanes' values (an indexed read of the argument block is a
// vector load to the compiler, and everything derived from it counts as different per lane).
static __device__ __forceinline__ unsigned long long slot_of_uniform(const GemvArgs &a, const int e) {
  const unsigned long long v = slot_of(a, e);
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(v >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// Host side: the table by value when the caller has a host copy and it fits, else the device table.
static void gemv_set_table(GemvArgs &a, const uint64_t *expert_ptr, const uint64_t *expert_ptr_host, int E) {
  a.expert_ptr = (const unsigned long long *)expert_ptr;
  a.tab_n = 0;
  if (expert_ptr_host && E > 0 && E <= GEMV_MAX_KUNITS) {
    for (int e = 0; e < E; ++e) a.tab[e] = expert_ptr_host[e];
    a.tab_n = E;
  }
}

// bx: the workgroup's index among the working ones (launches with a publishing workgroup put that one first)
// BY_ROWS (device-built unit list of at most 64 slots, a.unit_slots > 0): position u of the grid takes the unit of
// rank u when the units are ordered by the passes they need (more than 32 rows, 17 to 32, 1 to 16, none; list
// order inside a class).  The workgroups of the units with the most rows then start first and those of the unused
// slots last, instead of a popular expert starting when the first round of workgroups has finished.
template <bool DEVUNITS, bool BY_ROWS = false>
static __device__ __forceinline__ GemvWork gemv_resolve(const GemvArgs &a, const int bx, const int lane = 0) {
  GemvWork wk;
  const GemvClass c0 = a.cls[0], c1 = a.cls[1];
  const int n_sh = a.n_sh_blocks;
  const bool sh = bx < n_sh;
  GemvClass &c = wk.c;
  c.act = sh ? c0.act : c1.act; c.gather = sh ? c0.gather : c1.gather; c.out = sh ? c0.out : c1.out;
  c.off_q = sh ? c0.off_q : c1.off_q; c.off_s = sh ? c0.off_s : c1.off_s; c.off_z = sh ? c0.off_z : c1.off_z;
  c.K = sh ? c0.K : c1.K; c.G = sh ? c0.G : c1.G; c.act_stride = sh ? c0.act_stride : c1.act_stride;
  c.out_stride = sh ? c0.out_stride : c1.out_stride; c.nblk = sh ? c0.nblk : c1.nblk; c.ksplit = sh ? c0.ksplit : c1.ksplit;
  const int rr = sh ? bx : bx - n_sh;
  const int u = sh ? 0 : rr / c.nblk;
  wk.b = rr - u * c.nblk;
  wk.half = 0;
  if (BY_ROWS && sh && a.row_split) {  // the shared expert's workgroups come twice, one set per half of the rows
    wk.half = bx >= (n_sh >> 1) ? 1 : 0;
    wk.b = bx - (wk.half ? (n_sh >> 1) : 0);
  }
  if (DEVUNITS) {
    if (sh) {
      wk.m = a.T; wk.row0 = 0; wk.base = a.shared_base;
    } else {
      if (a.kunits_dev) {
        const KUnit kd = a.kunits_dev[u];
        wk.m = kd.m; wk.row0 = kd.row0;
        wk.base = (const unsigned char *)kd.base;
      } else if (BY_ROWS && a.unit_slots > 0) {
        const rsrc_t ru = make_rsrc(a.units, (u32)a.unit_slots * 16u);
        const u32x4_t ul = __builtin_amdgcn_raw_buffer_load_b128(ru, lane * 16, 0, 0);  // past the list: zeros
        const int ml = (int)ul.y;
        const unsigned long long c3 = __ballot(ml > 32), c2 = __ballot(ml > 16 && ml <= 32),
                                 c1 = __ballot(ml > 0 && ml <= 16), c0 = ~(c3 | c2 | c1);
        const unsigned long long below = (1ull << lane) - 1ull;
        const int n3 = __popcll(c3), n2 = __popcll(c2), n1 = __popcll(c1);
        const int rank = ml > 32 ? __popcll(c3 & below)
                         : ml > 16 ? n3 + __popcll(c2 & below)
                         : ml > 0 ? n3 + n2 + __popcll(c1 & below) : n3 + n2 + n1 + __popcll(c0 & below);
        // row_split: the n3 units of more than 32 rows take two positions each (rows 0..31, rows 32..)
        int ur = u;
        if (a.row_split) {
          if (u < 2 * n3) { wk.half = u & 1; ur = u >> 1; }
          else ur = u - n3;
        }
        const unsigned long long hit = __ballot(rank == ur);
        if (hit == 0ull) {  // a position past the list
          wk.m = 0; wk.row0 = 0; wk.base = nullptr;
        } else {
          const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)hit) - 1);  // exactly one lane
          const int ue = __builtin_amdgcn_readlane((int)ul.x, src);
          wk.m = __builtin_amdgcn_readlane(ml, src);
          wk.row0 = __builtin_amdgcn_readlane((int)ul.z, src);
          wk.base = wk.m > 0 ? (const unsigned char *)slot_of_uniform(a, ue) : nullptr;
        }
      } else {
        const moe_unit ud = a.units[u];
        wk.m = ud.m; wk.row0 = ud.row0;
        wk.base = ud.m > 0 ? (const unsigned char *)slot_of_uniform(a, ud.expert) : nullptr;
      }
    }
  } else {
    // the first 8 units sit at fixed argument offsets: fetched with the rest, picked by scalar selects
    unsigned long long ub = a.ku[0].base;
    int um = a.ku[0].m, ur = a.ku[0].row0;
#pragma unroll
    for (int i = 1; i < 8; ++i) {
      const bool hit = u == i;
      ub = hit ? a.ku[i].base : ub; um = hit ? a.ku[i].m : um; ur = hit ? a.ku[i].row0 : ur;
    }
    if (u >= 8) { ub = a.ku[u].base; um = a.ku[u].m; ur = a.ku[u].row0; }
    wk.m = sh ? a.T : um; wk.row0 = sh ? 0 : ur;
    ub = sh ? (unsigned long long)a.shared_base : ub;
    // uniform by construction; say so, or the buffer resources end up in vector registers
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)ub);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(ub >> 32));
    wk.base = (const unsigned char *)(((unsigned long long)hi << 32) | lo);
  }
  return wk;
}

// Q4K: same nibble tiles, but the scale data is per 32-wide sub-block (= one lane's k quarter):
// section s holds (6-bit scale, 6-bit min) byte pairs [N/16][G][64 lanes], section z holds
// (fp16 d, fp16 dmin) pairs [N/16][G/2][16 rows]; w = d*sc*q - dmin*m.
// One token: every workgroup derives the routing itself from the gate logits instead of
// reading a unit list made by two earlier launches.  With one token the dispatch is trivial
// (unit u = the u-th smallest selected expert id, one row each), and the top-k of <= 256
// logits is k rounds of a wave-wide maximum built from DPP row shifts and broadcasts (no LDS,
// no scalar round trips): lane l holds logits l, l+64, ...; the winner of a round is the
// lowest expert id that holds the maximum - the order and the tie rule of k_topk.  One spare
// workgroup publishes the routing (indices, weights, dispatch arrays, unit list) for the
// later kernels and the host.
// Block order: the routed experts' workgroups, then one workgroup that only publishes the routing (its first
// wave), then the shared expert's.  With the shared expert's workgroups in front, their tile requests (issued 0.3 us
// after the launch, nothing to wait for) stood in the compute units' memory pipelines ahead of the logit loads of
// the routed workgroups that share those compute units, and a tenth of the routed workgroups knew their expert
// 2 us later than the others.
template <int NR>
static __device__ __forceinline__ GemvWork gemv_resolve_route_n(const GemvArgs &a, int lane, int w, const int bx) {
  GemvWork wk;
  const int E = a.r_E, k = a.r_k;
  const int n_rt = k * a.cls[1].nblk + 1;
  const bool sh = bx >= n_rt;
  wk.c = sh ? a.cls[0] : a.cls[1];
  const int rr = sh ? bx - n_rt : bx;
  const bool publisher = !sh && rr == k * wk.c.nblk;
  const int u = (sh || publisher) ? 0 : rr / wk.c.nblk;
  wk.b = rr - u * wk.c.nblk;
  if (sh) {
    wk.m = 1; wk.row0 = 0; wk.base = a.shared_base;
    return wk;
  }
  // One wave of the workgroup derives the routing and hands the unit's slot address to the others through
  // LDS: four waves doing the same rounds would each take their turn on the SIMDs.  Workgroups b, b + 256, ...
  // share a compute unit when the grid is resident as a whole; they route on different SIMDs.
  __shared__ unsigned s_route_base[2];
  const int rw = publisher ? 0 : ((bx >> 8) & 3);
  wk.m = publisher ? 0 : 1; wk.row0 = u;
  if (w == rw) {
  const float NEG = -__builtin_inff();
  float v[NR], v0[NR];
  unsigned long long ptrs[NR];  // slot addresses of the lane's candidates, fetched alongside the logits
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int e = lane + 64 * r;
    v[r] = (e < E && a.g_nblk == 0) ? a.r_logits[e] : NEG;
    ptrs[r] = (e < E) ? slot_of(a, e) : 0ull;
  }
  bool gate_timeout = false;
  if (a.g_nblk) {
    // the logits come from the gate workgroups of this launch (the first of the grid, so they are running or
    // done when this one starts): poll the copy of this part of the chip until every word carries this launch's
    // number; should that copy stay incomplete, go on with the device-scope copy
    const rsrc_t rl = make_rsrc(a.g_stamp + (size_t)xcc_id() * GATE_COPY_WORDS, GATE_COPY_WORDS * 8);
    const unsigned long long *cg = a.g_stamp + (size_t)GATE_PARTS * GATE_COPY_WORDS;
    unsigned spins = 0;
    STAMP(0); STAMPV(7, (unsigned long long)xcc_id());
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const int e = lane + 64 * r;
        if (e < E) {
          u32x2_t word;
          if (spins < GATE_LOCAL_SPINS) {
            word = __builtin_amdgcn_raw_buffer_load_b64(rl, e * 8, 0, 16 /* sc1: past the first-level cache */);
          } else {
            const unsigned long long w64 = __hip_atomic_load(cg + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            word.x = (u32)w64; word.y = (u32)(w64 >> 32);
          }
          v[r] = __uint_as_float(word.x);
          ok = ok && (int)word.y == a.g_seq;
        }
      }
      if (spins == 0) STAMP(1);
      if (__ballot(!ok) == 0ull) break;
      if (++spins >= GATE_POLL_LIMIT) { gate_timeout = true; break; }  // (never seen; the launch then reports an error)
      __builtin_amdgcn_s_sleep(2);
    }
    STAMP(2); STAMPV(3, spins);
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) v0[r] = v[r];
  unsigned long long msel[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) msel[r] = 0ull;
  float mx = 0.f, sum_sel = 0.f, my_v = 0.f;  // the last three only matter to the publisher
  int my_e = 0;
  for (int j = 0; j < k; ++j) {
    float bv = v[0];
#pragma unroll
    for (int r = 1; r < NR; ++r) bv = fmaxf(bv, v[r]);
    const float best = wave_max_f32(bv);
    // the lowest expert id holding the maximum: lowest column r first, then lowest lane
    int wr = -1, wl = 0;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const unsigned long long mr = __ballot(v[r] == best);
      if (wr < 0 && mr) { wr = r; wl = (int)__builtin_ctzll(mr); }
    }
    if (wr < 0) { wr = 0; wl = j; }  // NaN logits match nothing: stay inside the expert range
#pragma unroll
    for (int r = 0; r < NR; ++r)
      if (r == wr) {
        if (lane == wl) v[r] = NEG;
        msel[r] |= 1ull << wl;
      }
    if (lane == j) { my_v = best; my_e = wl + 64 * wr; }
  }
  // unit u = the u-th smallest selected id
  int cum = 0;
  bool found = false;
  unsigned lo = 0, hi = 0;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int cnt = __popcll(msel[r]);
    if (!found && u < cum + cnt) {
      unsigned long long mm = msel[r];
      for (int i = 0; i < u - cum; ++i) mm &= mm - 1;
      const int src = (int)__builtin_ctzll(mm);  // expert 64 r + src
      lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)ptrs[r], src);
      hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(ptrs[r] >> 32), src);
      found = true;
    }
    cum += cnt;
  }
  if (gate_timeout) { lo = 0; hi = 0; }  // reported as a unit without a slot
  STAMP(4);
  if (lane == 0) { s_route_base[0] = lo; s_route_base[1] = hi; }

  if (publisher) {  // publish the routing: weights as in k_topk, arrays as in k_dispatch (T = 1)
    // position of a pair = rank of its expert id among the selected
    int below[NR], cb = 0;
#pragma unroll
    for (int r = 0; r < NR; ++r) { below[r] = cb; cb += __popcll(msel[r]); }
    int pos = 0;
    {
      const int r_ = my_e >> 6, l_ = my_e & 63;
#pragma unroll
      for (int r = 0; r < NR; ++r)
        if (r == r_) pos = below[r] + __popcll(msel[r] & ((1ull << l_) - 1ull));
    }
    // a host that waits for the routing gets it first: the unit list, then (once those stores have
    // completed) the sequence word it polls; weights and dispatch arrays follow
    if (a.r_host_units) {
      if (lane < k) host_store_unit(a.r_host_units, pos, my_e, 1, pos);
      if (a.r_host_seq) {
        host_stores_done();
        if (lane == 0) __hip_atomic_store(a.r_host_seq, a.r_host_seq_val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
    // sum over the selected logits in choice order (the order of k_topk), maximum = choice 0
    mx = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_v), 0));
#pragma unroll 1
    for (int j = 0; j < k; ++j)
      sum_sel += expf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_v), j)) - mx);
    float den = 0.f;
#pragma unroll
    for (int r = 0; r < NR; ++r)
      if (lane + 64 * r < E) den += expf(v0[r] - mx);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) den = den + __shfl_xor(den, m, 64);
    const float ex = expf(my_v - mx);
    float wgt;
    if (a.r_mode == MOE_ROUTE_TOPK_SOFTMAX) {
      wgt = ex / sum_sel;
    } else {
      wgt = ex / den;
      if (a.r_mode == MOE_ROUTE_SOFTMAX_TOPK_RENORM) wgt = wgt / (sum_sel / den);
    }
    // dispatch of the k pairs of the one token
    if (lane < k) {
      a.r_idx[lane] = my_e;
      a.r_w[lane] = wgt;
      a.r_sorted_pair[pos] = lane;
      a.r_pos_of_pair[lane] = pos;
      a.r_sorted_tok[pos] = 0;
      moe_unit un; un.expert = my_e; un.m = 1; un.row0 = pos; un.pad = 0;
      a.r_units[pos] = un;
      a.r_active_ids[pos] = my_e;
      if (a.r_kunits) { KUnit kd; kd.base = slot_of(a, my_e); kd.m = 1; kd.row0 = pos; a.r_kunits[pos] = kd; a.r_unit_w[pos] = wgt; }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const int e = lane + 64 * r;
      if (e < E) {
        const bool selb = (msel[r] >> lane) & 1ull;
        a.r_counts[e] = selb ? 1 : 0;
        a.r_offsets[e] = below[r] + __popcll(msel[r] & ((1ull << lane) - 1ull));
      }
    }
    if (lane == 0) { a.r_offsets[E] = k; *a.r_n_active = k; }
  }
  }
  __syncthreads();
  wk.base = (const unsigned char *)(((unsigned long long)s_route_base[1] << 32) | s_route_base[0]);
  return wk;
}

static __device__ __forceinline__ GemvWork gemv_resolve_route(const GemvArgs &a, int lane, int w, int bx) {
  // one instantiation per number of 64-wide logit columns: a 64-expert layer pays for one column only
  if (a.r_E <= 64) return gemv_resolve_route_n<1>(a, lane, w, bx);
  if (a.r_E <= 128) return gemv_resolve_route_n<2>(a, lane, w, bx);
  return gemv_resolve_route_n<4>(a, lane, w, bx);
}

// ---------------------------------------------------------------------------
// Decode batches of 2 to 8 tokens whose w13 launch sums the gate rows and routes by itself (the step is then
// three launches: this one, w2, combine).  Grid: the gate workgroups (a token and four gate rows each, a wave per
// row, once per part of the chip: see gate_rows_stamped), ONE workgroup that publishes the routing for the later
// launches and the host (the routing workgroup of k_gate_route), the shared expert's workgroups, then one set of
// workgroups per unit slot (min(E, T k) slots).  A workgroup of slot u derives the routing itself: wave w takes
// the tokens w, w + 4 (polls their logit words in the copy of its part of the chip, k rounds of wave-wide
// maxima: the selection and tie rule of topk_token) and leaves every token's experts as a bit mask in LDS; after
// one barrier every wave counts, per expert (a lane per expert and 64-wide column), the tokens that chose it,
// finds the u-th expert in use (units are in expert order), its rows' first position (the counts of all experts
// below it, from ballots of the count's bits) and the tokens of the unit as a bit mask (a token holds an expert
// at most once, so a unit's rows are its tokens in token order).  Every workgroup works from the same words with
// the same rounds, so all of them and the publisher agree.
// ---------------------------------------------------------------------------
#define RB_MAXT 16
#define RB_MAX_UNITS 256   // unit slots of such a launch: min(E, T k) <= 256
// gate rows of a batch: a workgroup takes four gate rows (a wave per row) and TG = ceil(T / 4) tokens; the row is
// read once and every token's sum is the fma chain of gate_row_partial over the same chunks, then the same
// butterfly (so the bits are those of gate_row_sum); all loads of a wave go out before the first fma
template <int NCH, int TG>
static __device__ __forceinline__ void gate_rows_multi(const uint16_t *__restrict__ x, const uint16_t *__restrict__ wr,
                                                       const int H, const int lane, const int t0, const int T,
                                                       float (&out)[TG]) {
  uint4 wq[NCH], xq[TG][NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int k = c * 512 + 8 * lane;
    wq[c] = *(const uint4 *)(wr + (k < H ? k : 0));
  }
#pragma unroll
  for (int i = 0; i < TG; ++i) {
    const int t = t0 + i < T ? t0 + i : T - 1;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int k = c * 512 + 8 * lane;
      xq[i][c] = *(const uint4 *)(x + (size_t)t * H + (k < H ? k : 0));
    }
  }
#pragma unroll
  for (int i = 0; i < TG; ++i) {
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      float t = acc;
      t = fmaf(bf16lo(xq[i][c].x), bf16lo(wq[c].x), t);
      t = fmaf(bf16hi(xq[i][c].x), bf16hi(wq[c].x), t);
      t = fmaf(bf16lo(xq[i][c].y), bf16lo(wq[c].y), t);
      t = fmaf(bf16hi(xq[i][c].y), bf16hi(wq[c].y), t);
      t = fmaf(bf16lo(xq[i][c].z), bf16lo(wq[c].z), t);
      t = fmaf(bf16hi(xq[i][c].z), bf16hi(wq[c].z), t);
      t = fmaf(bf16lo(xq[i][c].w), bf16lo(wq[c].w), t);
      t = fmaf(bf16hi(xq[i][c].w), bf16hi(wq[c].w), t);
      acc = (c * 512 + 8 * lane < H) ? t : acc;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc = acc + __shfl_xor(acc, m, 64);
    out[i] = acc;
  }
}

template <int TG>
static __device__ __forceinline__ void gate_rows_batch_tg(const GemvArgs &a, const int lane, const int w, const int q) {
  const int Erows = a.g_rows, H = a.cls[1].K, T = a.T;
  const bool per_part = a.g_parts == GATE_PARTS;
  const int item = per_part ? q >> 3 : q;
  const int nrb = (Erows + 3) >> 2;
  const int tgi = item / nrb, e = (item - tgi * nrb) * 4 + w;
  const int t0 = tgi * TG;
  if (e >= Erows) return;
  const bool biased = a.g_bias && e < a.g_nbias;
  const float bias_e = biased ? a.g_bias[e] : 0.f;
  asm volatile("" :: "v"(bias_e));  // requested in front of the row
  float acc[TG];
  const uint16_t *wr = a.g_w + (size_t)e * H;
  const int nch = (H + 511) >> 9;  // wave-uniform
  switch (nch) {
    case 1: gate_rows_multi<1, TG>(a.cls[1].act, wr, H, lane, t0, T, acc); break;
    case 2: gate_rows_multi<2, TG>(a.cls[1].act, wr, H, lane, t0, T, acc); break;
    case 4: gate_rows_multi<4, TG>(a.cls[1].act, wr, H, lane, t0, T, acc); break;
    case 8:  // (TG = 2 runs in the whole-row kernel, whose waves keep under 128 registers; 8 x 8 vectors do not fit)
      if constexpr (TG != 2 && TG != 8) { gate_rows_multi<8, TG>(a.cls[1].act, wr, H, lane, t0, T, acc); break; }
    default:
#pragma unroll
      for (int i = 0; i < TG; ++i)
        acc[i] = gate_row_sum(a.cls[1].act + (size_t)(t0 + i < T ? t0 + i : T - 1) * H, wr, H, lane);
  }
  const rsrc_t rl = make_rsrc(a.g_stamp + (size_t)xcc_id() * a.g_copy_words, (u32)a.g_copy_words * 8u);
#pragma unroll
  for (int i = 0; i < TG; ++i) {
    const int t = t0 + i;
    if (t < T) {
      const float val = biased ? acc[i] + bias_e : acc[i];
      const u32x2_t word = {__float_as_uint(val), (u32)a.g_seq};
      const int wi = t * Erows + e;
      if (per_part && lane == 0) __builtin_amdgcn_raw_buffer_store_b64(word, rl, wi * 8, 0, 1 /* sc0 */);
      if (!per_part || (q & 7) == 0) {
        const unsigned long long word64 = ((unsigned long long)word.y << 32) | word.x;
        if (lane == 1)
          __hip_atomic_store(a.g_stamp + (size_t)GATE_PARTS * a.g_copy_words + wi, word64, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) a.g_logits_out[(size_t)t * a.g_ldl + e] = val;
      }
    }
  }
}

// LDS the publishing workgroup of such a launch takes from the launch's dynamic area
#define RB_PUBLISH_LDS (2048 + 2048 + 1040 + 48 + RB_MAXT * GROUTE_MAX_ROWS * 4)
static __device__ __forceinline__ void route_publish_batch(const GemvArgs &a, unsigned char *smem) {
  int *s_idx = (int *)smem;                                            // [ROUTE_MAXP]
  unsigned long long *s_mask = (unsigned long long *)(smem + 2048);    // [RB_MAXT .. ROUTE_MAXT][4]
  int *s_off = (int *)(smem + 4096);                                   // [257]
  int *s_wsum = (int *)(smem + 4096 + 1040), *s_wact = s_wsum + 4, *s_tot = s_wsum + 8;
  float *s_logits = (float *)(smem + 4096 + 1040 + 48);                // [T][GROUTE_MAX_ROWS]
  const int tid = threadIdx.x;
  const int T = a.T, Erows = a.g_rows;
  {
    const rsrc_t rl = make_rsrc(a.g_stamp + (size_t)xcc_id() * a.g_copy_words, (u32)a.g_copy_words * 8u);
    const unsigned long long *cg = a.g_stamp + (size_t)GATE_PARTS * a.g_copy_words;
    const int nw = T * Erows;
    const unsigned local_spins = a.g_parts == GATE_PARTS ? GATE_LOCAL_SPINS : 0u;
    bool timeout = false;
    for (int wi = tid; wi < nw; wi += 256) {
      unsigned spins = 0;
      u32x2_t word;
      for (;;) {
        if (spins < local_spins) {
          word = __builtin_amdgcn_raw_buffer_load_b64(rl, wi * 8, 0, 16 /* sc1: past the first-level cache */);
        } else {
          const unsigned long long w64 = __hip_atomic_load(cg + wi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          word.x = (u32)w64; word.y = (u32)(w64 >> 32);
        }
        if ((int)word.y == a.g_seq) break;
        if (++spins >= GATE_POLL_LIMIT) { timeout = true; break; }
        __builtin_amdgcn_s_sleep(2);
      }
      const int t = wi / Erows;
      s_logits[t * GROUTE_MAX_ROWS + (wi - t * Erows)] = __uint_as_float(word.x);
    }
    if (timeout) moe_raise_err(a.err);
  }
  __syncthreads();
  RouteArgs b;
  b.x = nullptr; b.wg = nullptr; b.bias = nullptr;
  b.logits = s_logits; b.T = T; b.H = a.cls[1].K; b.E = a.r_E; b.Erows = Erows; b.ldl = GROUTE_MAX_ROWS; b.k = a.r_k;
  b.mode = a.r_mode; b.nbits = 0; b.max_units = a.p_max_units;
  b.idx = a.r_idx; b.w = a.r_w; b.counts = a.r_counts; b.offsets = a.r_offsets; b.sorted_pair = a.r_sorted_pair;
  b.pos_of_pair = a.r_pos_of_pair; b.sorted_tok = a.r_sorted_tok; b.units = a.r_units; b.n_active = a.r_n_active;
  b.active_ids = a.r_active_ids; b.counter = nullptr;
  b.host_units = a.r_host_units; b.host_n_active = a.p_host_n_active; b.host_seq = a.r_host_seq;
  b.host_seq_val = a.r_host_seq_val; b.pad_ = 0;
  b.n_bias = 0; b.g_seq = 0; b.g_copy_words = 0; b.g_parts = 0; b.g_stamp = nullptr; b.err = a.err;
  route_tail<4, false>(b, s_idx, s_mask, s_off, s_wsum, s_wact, *s_tot);
}

// rr: the workgroup's index among those of the unit slots.  tokmask: the unit's tokens.
// TPW: tokens per wave (wave w takes the tokens w, w + 4, ...; their selection rounds are interleaved)
template <int NR, int TPW>
static __device__ __forceinline__ GemvWork gemv_resolve_route_batch_n(const GemvArgs &a, const int lane, const int w,
                                                                      const int rr, unsigned &tokmask) {
  __shared__ unsigned long long s_sel[RB_MAXT][4];
  GemvWork wk;
  wk.c = a.cls[1];
  const int E = a.r_E, k = a.r_k, T = a.T, Erows = a.g_rows;
  const int u = rr / wk.c.nblk;
  wk.b = rr - u * wk.c.nblk;
  wk.half = 0;
  const float NEG = -__builtin_inff();
  // Unit records of this part of the chip: four (value, launch number) words per unit slot (slot address low and
  // high, rows << 16 | first row position, token mask), written through this part's second-level cache by every
  // workgroup that has derived the routing.  A workgroup that starts late (grid index from g_cache_from on: the
  // first round of workgroups is over by then) reads its slot's record instead of polling logits and selecting;
  // if the record is not there it derives the routing like the others.  All writers write the same values.
  const rsrc_t rrec = make_rsrc(a.g_stamp + (size_t)GATE_COPIES * a.g_copy_words + (size_t)xcc_id() * (RB_MAX_UNITS * 4),
                                RB_MAX_UNITS * 32u);
  if ((int)blockIdx.x >= a.g_cache_from) {
    __shared__ unsigned s_rec[5];
    if (w == 0) {
      const u32x2_t word = __builtin_amdgcn_raw_buffer_load_b64(rrec, (u * 4 + (lane & 3)) * 8, 0, 16 /* sc1 */);
      const bool ok = (int)word.y == a.g_seq;
      const bool all = (__ballot(ok) & 0xfull) == 0xfull;
      if (lane < 4) s_rec[lane] = word.x;
      if (lane == 0) s_rec[4] = all ? 1u : 0u;
    }
    __syncthreads();
    if (s_rec[4]) {
      wk.m = (int)(s_rec[2] >> 16);
      wk.row0 = (int)(s_rec[2] & 0xffffu);
      tokmask = s_rec[3];
      wk.base = (const unsigned char *)(((unsigned long long)s_rec[1] << 32) | s_rec[0]);
      return wk;
    }
  }
  unsigned long long ptrs[NR];  // slot addresses of the lane's experts, requested in front of the logits
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int e = lane + 64 * r;
    ptrs[r] = (e < E) ? slot_of(a, e) : 0ull;
  }
  const rsrc_t rl = make_rsrc(a.g_stamp + (size_t)xcc_id() * a.g_copy_words, (u32)a.g_copy_words * 8u);
  const unsigned long long *cg = a.g_stamp + (size_t)GATE_PARTS * a.g_copy_words;
  float v[TPW][NR];
  bool gate_timeout = false;
  {
    const unsigned local_spins = a.g_parts == GATE_PARTS ? GATE_LOCAL_SPINS : 0u;
    unsigned spins = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int i = 0; i < TPW; ++i) {
        const int t = w + 4 * i;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
          const int e = lane + 64 * r;
          v[i][r] = NEG;
          if (e < E && t < T) {
            u32x2_t word;
            if (spins < local_spins) {
              word = __builtin_amdgcn_raw_buffer_load_b64(rl, (t * Erows + e) * 8, 0, 16 /* sc1: past the first-level cache */);
            } else {
              const unsigned long long w64 = __hip_atomic_load(cg + t * Erows + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              word.x = (u32)w64; word.y = (u32)(w64 >> 32);
            }
            v[i][r] = __uint_as_float(word.x);
            ok = ok && (int)word.y == a.g_seq;
          }
        }
      }
      if (__ballot(!ok) == 0ull) break;
      if (++spins >= GATE_POLL_LIMIT) { gate_timeout = true; break; }  // (the launch then reports an error)
      __builtin_amdgcn_s_sleep(2);
    }
  }
  unsigned long long msel[TPW][NR];
#pragma unroll
  for (int i = 0; i < TPW; ++i)
#pragma unroll
    for (int r = 0; r < NR; ++r) msel[i][r] = 0ull;
  for (int j = 0; j < k; ++j) {
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
      float bv = v[i][0];
#pragma unroll
      for (int r = 1; r < NR; ++r) bv = fmaxf(bv, v[i][r]);
      const float best = wave_max_f32(bv);
      int wr = -1, wl = 0;
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const unsigned long long mr = __ballot(v[i][r] == best);
        if (wr < 0 && mr) { wr = r; wl = (int)__builtin_ctzll(mr); }
      }
      if (wr < 0) { wr = 0; wl = j; }  // NaN logits match nothing: stay inside the expert range
#pragma unroll
      for (int r = 0; r < NR; ++r)
        if (r == wr) {
          if (lane == wl) v[i][r] = NEG;
          msel[i][r] |= 1ull << wl;
        }
    }
  }
  __shared__ int s_timeout[4];
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
      const int t = w + 4 * i;
      if (t < T) {
#pragma unroll
        for (int r = 0; r < NR; ++r) s_sel[t][r] = gate_timeout ? 0ull : msel[i][r];
      }
    }
    s_timeout[w] = gate_timeout ? 1 : 0;
    if (gate_timeout) moe_raise_err(a.err);
  }
  __syncthreads();
  const bool gate_timeout_any = (s_timeout[0] | s_timeout[1] | s_timeout[2] | s_timeout[3]) != 0;  // (no records then)
  // per expert (this lane's, per column): its tokens
  int cnt[NR];
  unsigned mk[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) { cnt[r] = 0; mk[r] = 0u; }
#pragma unroll
  for (int t = 0; t < 4 * TPW; ++t) {
    if (t < T) {
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const unsigned bit = (unsigned)((s_sel[t][r] >> lane) & 1ull);
        cnt[r] += (int)bit;
        mk[r] |= bit << t;
      }
    }
  }
  int cum_act = 0, cum_rows = 0, m = 0, row0 = 0;
  unsigned tm = 0u, lo = 0u, hi = 0u;
  bool found = false;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const unsigned long long actm = __ballot(cnt[r] > 0);
    const unsigned long long b0 = __ballot((cnt[r] & 1) != 0), b1 = __ballot((cnt[r] & 2) != 0),
                             b2 = __ballot((cnt[r] & 4) != 0), b3 = __ballot((cnt[r] & 8) != 0),
                             b4 = __ballot((cnt[r] & 16) != 0);
    const int na = __popcll(actm);
    if (!found && u < cum_act + na) {
      unsigned long long mm = actm;
      for (int i = 0; i < u - cum_act; ++i) mm &= mm - 1;
      const int src = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(mm));  // expert 64 r + src
      const unsigned long long sb = (1ull << src) - 1ull;
      row0 = cum_rows + __popcll(b0 & sb) + 2 * __popcll(b1 & sb) + 4 * __popcll(b2 & sb) + 8 * __popcll(b3 & sb) +
             16 * __popcll(b4 & sb);
      m = __builtin_amdgcn_readlane(cnt[r], src);
      tm = (unsigned)__builtin_amdgcn_readlane((int)mk[r], src);
      lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)ptrs[r], src);
      hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(ptrs[r] >> 32), src);
      found = true;
    }
    if (w == 0 && !gate_timeout_any && cnt[r] > 0) {  // this lane's expert is a unit: leave its record
      const unsigned long long lb = (1ull << lane) - 1ull;
      const int ui = cum_act + __popcll(actm & lb);
      const int rw = cum_rows + __popcll(b0 & lb) + 2 * __popcll(b1 & lb) + 4 * __popcll(b2 & lb) + 8 * __popcll(b3 & lb) +
                     16 * __popcll(b4 & lb);
      if (ui < RB_MAX_UNITS) {
        const u32 seq = (u32)a.g_seq;
        __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{(u32)ptrs[r], seq}, rrec, (ui * 4 + 0) * 8, 0, 1 /* sc0 */);
        __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{(u32)(ptrs[r] >> 32), seq}, rrec, (ui * 4 + 1) * 8, 0, 1);
        __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{((u32)cnt[r] << 16) | (u32)rw, seq}, rrec, (ui * 4 + 2) * 8, 0, 1);
        __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{mk[r], seq}, rrec, (ui * 4 + 3) * 8, 0, 1);
      }
    }
    cum_act += na;
    cum_rows += __popcll(b0) + 2 * __popcll(b1) + 4 * __popcll(b2) + 8 * __popcll(b3) + 16 * __popcll(b4);
  }
  if (w == 0 && !gate_timeout_any) {  // the slots past the last unit: records of no rows
    const int nslots = a.p_max_units < RB_MAX_UNITS ? a.p_max_units : RB_MAX_UNITS;
    for (int ui = cum_act + (lane >> 2); ui < nslots; ui += 16)
      __builtin_amdgcn_raw_buffer_store_b64(u32x2_t{0u, (u32)a.g_seq}, rrec, (ui * 4 + (lane & 3)) * 8, 0, 1 /* sc0 */);
  }
  wk.m = found ? m : 0;
  wk.row0 = row0;
  tokmask = tm;
  wk.base = (const unsigned char *)(((unsigned long long)hi << 32) | lo);
  return wk;
}

// TPW: the launch's tokens per wave (1: up to 4 tokens, 2: up to 8, 4: up to 16); E up to 64 pays for one column
template <int TPW>
static __device__ __forceinline__ GemvWork gemv_resolve_route_batch(const GemvArgs &a, int lane, int w, int rr, unsigned &tokmask) {
  if (a.r_E <= 64) return gemv_resolve_route_batch_n<1, TPW>(a, lane, w, rr, tokmask);
  return gemv_resolve_route_batch_n<4, TPW>(a, lane, w, rr, tokmask);
}

// the i-th token (i-th set bit) of a unit's token mask
static __device__ __forceinline__ int nth_token(unsigned mask, const int i) {
#pragma unroll
  for (int q = 0; q < RB_MAXT - 1; ++q)
    if (q < i) mask &= mask - 1u;
  return mask ? __builtin_ctz(mask) : 0;
}

template <int TMAX, bool SWIGLU, int CH, bool DEVUNITS, bool Q4K = false>
__global__ __launch_bounds__(256, (TMAX == 1 ? 3 : 2)) void k_gemv_int4(const GemvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, qd = lane >> 4;

  const GemvWork wk = gemv_resolve<DEVUNITS>(a, (int)blockIdx.x);
  const GemvClass &c = wk.c;
  const int m = wk.m, row0 = wk.row0;
  const unsigned char *base = wk.base;
  if (m <= 0) return;
  if (base == nullptr) {
    if (tid == 0 && wk.b == 0) moe_raise_err(a.err);  // one store per missing unit (the word may be host memory)
    return;
  }
  // a unit that travels by value and arrived late (its copy landed after the step's routing launch had published
  // the unit list with slot address 0): its address goes into the published list, for the w2 + combine launch
  if (!DEVUNITS && SWIGLU && a.r_kunits && blockIdx.x == (unsigned)a.n_sh_blocks && tid == 0)
    a.r_kunits[row0].base = (unsigned long long)base;
  // Gt groups per row block in memory; this workgroup reduces over the window [g0, g0 + G) of them (the whole
  // row unless the class is split: then `split` of c.ksplit workgroups share a block pair)
  const int Gt = c.G;
  const int nsp = (Q4K && c.ksplit > 1) ? c.ksplit : 1;
  const int split = nsp > 1 ? wk.b % nsp : 0;
  const int b = nsp > 1 ? wk.b / nsp : wk.b;
  const int G = Gt / nsp, g0 = split * G;
  const int K = G * 128, KS = K >> 5;
  // LDS: activations, their 32-wide sums, the scale/zero sections of the two row blocks,
  // and the cross-wave reduction buffer
  uint16_t *xs = (uint16_t *)smem;                                    // [TMAX][K]
  float *xsum = (float *)(smem + (size_t)TMAX * K * 2);              // [TMAX][K/32]
  uint16_t *s_sc = (uint16_t *)(xsum + (size_t)TMAX * KS);            // [2][G][16] fp16 | Q4K: [2][G][64] (sc, m)
  const int SCB = Q4K ? 128 : 32, ZZB = Q4K ? 32 : 8;                // bytes of section s / z per tile
  unsigned char *s_zz = (unsigned char *)s_sc + 2 * G * SCB;          // [2][G][8] | Q4K: [2][G/2][16] (d, dmin)
  float *red = (float *)(s_zz + 2 * G * ZZB);                         // [4][TMAX][2][16]

  const int GPW = (G - w + 3) >> 2;  // groups of this wave: g = w + 4j, j < GPW
  const int rbA = 2 * b;
  // tiles of block A then block B are contiguous: 2*G KiB
  const rsrc_t rq = make_rsrc(base + c.off_q + ((size_t)rbA * Gt + g0) * 1024, (u32)(Gt + G) * 1024u);
  const rsrc_t rs = make_rsrc(base + c.off_s + ((size_t)rbA * Gt + g0) * SCB, (u32)(Gt + G) * SCB);
  const rsrc_t rz = make_rsrc(base + c.off_z + ((size_t)rbA * Gt + g0) * ZZB, (u32)(Gt + G) * ZZB);
  const rsrc_t rx = make_rsrc((const unsigned char *)c.act + (size_t)g0 * 256, 0x7fffffffu);
  const int zsh = (r & 1) * 4;
  const int vec_per_row = K >> 3;
  const int n_sc = 2 * G * SCB / 4;   // dwords of section s
  const int n_zz = 2 * G * ZZB / 4;   // dwords of section z
  constexpr int XT = TMAX < 2 ? TMAX : 2;  // rows whose first 256 vectors are staged through registers
  const Q4Consts q4c = q4_consts();

  for (int t0 = 0; t0 < m; t0 += TMAX) {
    const int mc = (m - t0) < TMAX ? (m - t0) : TMAX;
    // ---- straight-line load section: small loads first, then the weight tiles --------------
    uint4 xv[XT];
#pragma unroll
    for (int t = 0; t < XT; ++t) {
      const int row = row0 + t0 + (t < mc ? t : 0);
      const int arow = c.gather ? c.gather[row] : row;  // uniform: a scalar load
      // threads past the row's end re-read vector 0 (staged nowhere): never past the tensor
      xv[t] = bload16(rx, (tid < vec_per_row ? tid : 0) * 16, arow * c.act_stride * 2);
    }
    // dword i of the LDS copy [2][G] of a section lies at i * 4 in memory, plus the gap between the two blocks'
    // windows for the second block (no gap when the window is the whole row)
    const int sc_half = G * SCB / 4, zz_half = G * ZZB / 4, sc_gap = (Gt - G) * SCB, zz_gap = (Gt - G) * ZZB;
    const u32 msc0 = bload4(rs, tid * 4 + (tid >= sc_half ? sc_gap : 0), 0);
    const u32 msc1 = bload4(rs, (tid + 256) * 4 + (tid + 256 >= sc_half ? sc_gap : 0), 0);
    const u32 mzz = bload4(rz, tid * 4 + (tid >= zz_half ? zz_gap : 0), 0);
    uint4 wa[CH], wb[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int g = j < GPW ? w + 4 * j : 0;  // clamped: tile 0 always exists
      wa[j] = bload16_nt(rq, lane * 16, g * 1024);
      wb[j] = bload16_nt(rq, lane * 16, (Gt + g) * 1024);
    }
    // ---- stage: x -> LDS (+ 32-wide sums via a quad reduction), scale/zero -> LDS ----------
#pragma unroll
    for (int t = 0; t < XT; ++t) {
      float ps = sum8_bf16(xv[t]);
      ps += __shfl_xor(ps, 1, 64);
      ps += __shfl_xor(ps, 2, 64);
      if (tid < vec_per_row && t < mc) {
        ((uint4 *)xs)[t * vec_per_row + tid] = xv[t];
        if ((tid & 3) == 0) xsum[(t * vec_per_row + tid) >> 2] = ps;
      }
    }
    if (tid < n_sc) ((u32 *)s_sc)[tid] = msc0;
    if (tid + 256 < n_sc) ((u32 *)s_sc)[tid + 256] = msc1;
    if (tid < n_zz) ((u32 *)s_zz)[tid] = mzz;
    // leftovers (more rows, K > 2048): plain loops
    for (int t = 0; t < mc; ++t) {
      const int row = row0 + t0 + t;
      const int arow = c.gather ? c.gather[row] : row;
      for (int v = tid + (t < XT ? 256 : 0); v < vec_per_row; v += 256) {
        const uint4 x4 = bload16(rx, v * 16, arow * c.act_stride * 2);
        float ps = sum8_bf16(x4);
        ps += __shfl_xor(ps, 1, 64);
        ps += __shfl_xor(ps, 2, 64);
        ((uint4 *)xs)[t * vec_per_row + v] = x4;
        if ((tid & 3) == 0) xsum[(t * vec_per_row + v) >> 2] = ps;
      }
    }
    for (int i = tid + 512; i < n_sc; i += 256) ((u32 *)s_sc)[i] = bload4(rs, i * 4 + (i >= sc_half ? sc_gap : 0), 0);
    for (int i = tid + 256; i < n_zz; i += 256) ((u32 *)s_zz)[i] = bload4(rz, i * 4 + (i >= zz_half ? zz_gap : 0), 0);
    __syncthreads();

    float accA[TMAX], accB[TMAX];
#pragma unroll
    for (int t = 0; t < TMAX; ++t) { accA[t] = 0.f; accB[t] = 0.f; }

    for (int jc = 0; jc < GPW; jc += CH) {
      if (jc > 0) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
          const int g = jc + j < GPW ? w + 4 * (jc + j) : 0;
          wa[j] = bload16_nt(rq, lane * 16, g * 1024);
          wb[j] = bload16_nt(rq, lane * 16, (Gt + g) * 1024);
        }
      }
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        const bool valid = jc + j < GPW;
        const int g = valid ? w + 4 * (jc + j) : 0;
        // a clamped (duplicate) tile contributes through a zero scale
        float fsa, fsb, fza, fzb;  // contribution of a lane: fs * D - fz' * xq with fz' = fs * fz
        if (Q4K) {
          const u32 smA = s_sc[g * 64 + lane], smB = s_sc[(G + g) * 64 + lane];
          const u32 ddA = ((const u32 *)s_zz)[(g >> 1) * 16 + r], ddB = ((const u32 *)s_zz)[((G + g) >> 1) * 16 + r];
          fsa = valid ? half_bits_to_f32((uint16_t)ddA) * (float)(smA & 0xff) : 0.f;
          fsb = valid ? half_bits_to_f32((uint16_t)ddB) * (float)(smB & 0xff) : 0.f;
          // w = fs*q - dmin*m = fs*(128+q) - (128*fs + dmin*m)
          fza = valid ? fmaf(128.f, fsa, half_bits_to_f32((uint16_t)(ddA >> 16)) * (float)(smA >> 8)) : 0.f;
          fzb = valid ? fmaf(128.f, fsb, half_bits_to_f32((uint16_t)(ddB >> 16)) * (float)(smB >> 8)) : 0.f;
        } else {
          // (unconditional reads, then a select: a read under the condition becomes a branch that splits
          // the unrolled loop into blocks, and the register allocation gets worse for it)
          const float fsa_ = half_bits_to_f32(s_sc[g * 16 + r]), fsb_ = half_bits_to_f32(s_sc[(G + g) * 16 + r]);
          fsa = valid ? fsa_ : 0.f;
          fsb = valid ? fsb_ : 0.f;
          fza = 128.f + (float)((s_zz[g * 8 + (r >> 1)] >> zsh) & 15);
          fzb = 128.f + (float)((s_zz[(G + g) * 8 + (r >> 1)] >> zsh) & 15);
        }
#pragma unroll
        for (int t = 0; t < TMAX; ++t) {
          if (t < mc) {
            const uint4 *xp = (const uint4 *)(xs + (size_t)t * K + g * 128 + qd * 32);
            const uint4 x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
            const float xq = xsum[t * KS + g * 4 + qd];
            float dA = dot8_q4(wa[j].x, x0, 0.f, q4c);
            float dB = dot8_q4(wb[j].x, x0, 0.f, q4c);
            dA = dot8_q4(wa[j].y, x1, dA, q4c); dB = dot8_q4(wb[j].y, x1, dB, q4c);
            dA = dot8_q4(wa[j].z, x2, dA, q4c); dB = dot8_q4(wb[j].z, x2, dB, q4c);
            dA = dot8_q4(wa[j].w, x3, dA, q4c); dB = dot8_q4(wb[j].w, x3, dB, q4c);
            if (Q4K) {
              accA[t] = fmaf(fsa, dA, fmaf(-fza, xq, accA[t]));
              accB[t] = fmaf(fsb, dB, fmaf(-fzb, xq, accB[t]));
            } else {
              accA[t] = fmaf(fsa, dA - fza * xq, accA[t]);
              accB[t] = fmaf(fsb, dB - fzb * xq, accB[t]);
            }
          }
        }
        // keep the scheduler from hoisting the next tile's LDS reads (register pressure)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // reduce the four k-quarters of the wave, then the four waves
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
      accA[t] += __shfl_xor(accA[t], 16, 64); accA[t] += __shfl_xor(accA[t], 32, 64);
      accB[t] += __shfl_xor(accB[t], 16, 64); accB[t] += __shfl_xor(accB[t], 32, 64);
      if (lane < 16 && t < mc) {
        red[((w * TMAX + t) * 2 + 0) * 16 + lane] = accA[t];
        red[((w * TMAX + t) * 2 + 1) * 16 + lane] = accB[t];
      }
    }
    __syncthreads();
    if (SWIGLU) {
      for (int i = tid; i < mc * 16; i += 256) {
        const int t = i >> 4, rr2 = i & 15;
        float ga = 0.f, up = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) {
          ga += red[((ww * TMAX + t) * 2 + 0) * 16 + rr2];
          up += red[((ww * TMAX + t) * 2 + 1) * 16 + rr2];
        }
        const float hv = ga / (1.f + expf(-ga)) * up;
        ((uint16_t *)c.out)[(size_t)(row0 + t0 + t) * c.out_stride + b * 16 + rr2] = f32_to_bf16(hv);
      }
    } else {
      for (int i = tid; i < mc * 32; i += 256) {
        const int t = i >> 5, ab = (i >> 4) & 1, rr2 = i & 15;
        float v = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) v += red[((ww * TMAX + t) * 2 + ab) * 16 + rr2];
        ((float *)c.out)[((size_t)split * a.T + (row0 + t0 + t)) * c.out_stride + (2 * b + ab) * 16 + rr2] = v;
      }
    }
    if (t0 + TMAX < m) __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// w13 + SwiGLU for ONE token with the routing derived in the kernel (int4-g128): the kernel of a one-token step.
// Same work split and the same order of every sum as k_gemv_int4<1, true, CH> (bit-identical h), but after the
// barrier that hands the routing over, a wave depends on no other wave until the final reduction: it reads
// the 256 bytes of the activation row that each of its own groups needs (16 bytes per lane), the 32 + 8 bytes of
// scales and zeros of each of its own tiles (one dword per lane each) and its tiles, in that order, and keeps the
// small ones in a wave-private LDS area (a wave's LDS operations complete in order: no barrier).  With the whole
// row and both scale sections staged by all four waves, a barrier stood between the requests and the first
// product, and the last wave's small loads gated all four.
// Measured with a time stamp per wave in the barrier form: routing known 1.5-1.8 us after entry (3.7-4.2 us for
// the workgroups that shared a compute unit with the shared expert's, hence the block order of
// gemv_resolve_route_n), activations and scales staged 1.6 us later, products 4 x 0.28 us.
// LDS per wave: [CH][128] bf16 activations, [CH][4] sums, [2 CH][8] scale dwords, [2 CH][2] zero dwords; then
// [4][2][16] partial sums.
// ---------------------------------------------------------------------------
#define W13T_WAVE_DW(ch) ((ch) * 64 + (ch) * 4 + (ch) * 16 + (ch) * 4)
static size_t w13_token_lds(int ch) { return (size_t)4 * W13T_WAVE_DW(ch) * 4 + 4 * 2 * 16 * 4; }

template <int CH>
__global__ __launch_bounds__(256, 3) void k_w13_token(const GemvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, qd = lane >> 4;
  if ((int)blockIdx.x < a.g_nblk) {  // a gate workgroup (uniform per workgroup)
    gate_rows_stamped(a, lane, w);
    return;
  }
  const GemvWork wk = gemv_resolve_route(a, lane, w, (int)blockIdx.x - a.g_nblk);  // ends with a barrier (routed workgroups)
  const GemvClass &c = wk.c;
  const unsigned char *base = wk.base;
  if (wk.m <= 0) return;
  if (base == nullptr) {
    if (tid == 0 && wk.b == 0) moe_raise_err(a.err);  // one store per missing unit (the word may be host memory)
    return;
  }
  const int G = c.G, b = wk.b;
  u32 *wl = (u32 *)smem + w * W13T_WAVE_DW(CH);
  uint16_t *xs = (uint16_t *)wl;                        // [CH][128]
  float *xsum = (float *)(wl + CH * 64);                // [CH][4]
  u32 *wsc = wl + CH * 68;                              // [2 CH][8]: block A's groups, then block B's
  u32 *wzz = wsc + CH * 16;                             // [2 CH][2]
  float *red = (float *)((u32 *)smem + 4 * W13T_WAVE_DW(CH));  // [4][2][16]
  const int GPW = (G - w + 3) >> 2;  // groups of this wave: g = w + 4j, j < GPW
  const int rbA = 2 * b;             // tiles of block A then block B are contiguous: 2 G KiB
  const rsrc_t rx = make_rsrc((const unsigned char *)c.act, (u32)c.K * 2u);
  const rsrc_t rq = make_rsrc(base + c.off_q + (size_t)rbA * G * 1024, (u32)(2 * G) * 1024u);
  const rsrc_t rs = make_rsrc(base + c.off_s + (size_t)rbA * G * 32, (u32)(2 * G) * 32u);
  const rsrc_t rz = make_rsrc(base + c.off_z + (size_t)rbA * G * 8, (u32)(2 * G) * 8u);
  const int zsh = (r & 1) * 4;
  const Q4Consts q4c = q4_consts();
  // the lane's share of the wave's small loads: 16 bytes of group xj's activations, dword scd of scale chunk scj
  // (chunks: block A's groups 0..CH-1, then block B's), dword zzd of zero chunk zzj
  const int xj = lane >> 4, xpart = lane & 15, scj = lane >> 3, scd = lane & 7, zzj = lane >> 1, zzd = lane & 1;
  const uint16_t *wsc_h = (const uint16_t *)wsc;
  const unsigned char *wzz_b = (const unsigned char *)wzz;
  float accA = 0.f, accB = 0.f;
  for (int jc = 0; jc < GPW; jc += CH) {
    uint4 xv = make_uint4(0u, 0u, 0u, 0u);
    u32 sd = 0, zd = 0;
    if (xj < CH) {
      const int g = jc + xj < GPW ? w + 4 * (jc + xj) : 0;  // clamped: group 0 always exists
      xv = bload16(rx, g * 256 + xpart * 16, 0);
    }
    if (scj < 2 * CH) {
      const int j = scj < CH ? scj : scj - CH;
      const int g = jc + j < GPW ? w + 4 * (jc + j) : 0;
      sd = bload4(rs, (((scj < CH ? 0 : G) + g) * 8 + scd) * 4, 0);
    }
    if (zzj < 2 * CH) {
      const int j = zzj < CH ? zzj : zzj - CH;
      const int g = jc + j < GPW ? w + 4 * (jc + j) : 0;
      zd = bload4(rz, (((zzj < CH ? 0 : G) + g) * 2 + zzd) * 4, 0);
    }
    uint4 wa[CH], wb[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int g = jc + j < GPW ? w + 4 * (jc + j) : 0;
      wa[j] = bload16_nt(rq, lane * 16, g * 1024);
      wb[j] = bload16_nt(rq, lane * 16, (G + g) * 1024);
    }
    {
      float ps = sum8_bf16(xv);
      ps += __shfl_xor(ps, 1, 64);
      ps += __shfl_xor(ps, 2, 64);
      if (xj < CH) {
        ((uint4 *)xs)[lane] = xv;
        if ((lane & 3) == 0) xsum[lane >> 2] = ps;
      }
    }
    if (scj < 2 * CH) wsc[lane] = sd;
    if (zzj < 2 * CH) wzz[lane] = zd;
    // (lanes read below what other lanes of the wave stored above: a wave's LDS operations complete in order; the
    // wave barrier is no instruction, it keeps the compiler from moving the reads in front of the stores)
    __builtin_amdgcn_wave_barrier();
    // everything the products need besides the tiles is read and converted before the first tile is waited
    // for: what a wave does after its last byte has arrived (all tiles of a wave arrive together) is the tail
    // of the launch, and only the unpacking and the dot products have to be in it
    float fsa[CH], fsb[CH], fza[CH], fzb[CH], xq[CH];
    uint4 xr[CH][4];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const bool valid = jc + j < GPW;
      // a clamped (duplicate) tile contributes through a zero scale
      const float fsa_ = half_bits_to_f32(wsc_h[j * 16 + r]), fsb_ = half_bits_to_f32(wsc_h[(CH + j) * 16 + r]);
      fsa[j] = valid ? fsa_ : 0.f;
      fsb[j] = valid ? fsb_ : 0.f;
      xq[j] = xsum[j * 4 + qd];
      fza[j] = 128.f + (float)((wzz_b[j * 8 + (r >> 1)] >> zsh) & 15);
      fzb[j] = 128.f + (float)((wzz_b[(CH + j) * 8 + (r >> 1)] >> zsh) & 15);
      const uint4 *xp = (const uint4 *)(xs + j * 128 + qd * 32);
      xr[j][0] = xp[0]; xr[j][1] = xp[1]; xr[j][2] = xp[2]; xr[j][3] = xp[3];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      float dA = dot8_q4(wa[j].x, xr[j][0], 0.f, q4c);
      float dB = dot8_q4(wb[j].x, xr[j][0], 0.f, q4c);
      dA = dot8_q4(wa[j].y, xr[j][1], dA, q4c); dB = dot8_q4(wb[j].y, xr[j][1], dB, q4c);
      dA = dot8_q4(wa[j].z, xr[j][2], dA, q4c); dB = dot8_q4(wb[j].z, xr[j][2], dB, q4c);
      dA = dot8_q4(wa[j].w, xr[j][3], dA, q4c); dB = dot8_q4(wb[j].w, xr[j][3], dB, q4c);
      accA = fmaf(fsa[j], dA - fza[j] * xq[j], accA);  // (the expression of k_gemv_int4: the same bits)
      accB = fmaf(fsb[j], dB - fzb[j] * xq[j], accB);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_wave_barrier();  // the next chunk's stores stay behind this chunk's reads
  }
  // reduce the four k-quarters of the wave, then the four waves
  accA += __shfl_xor(accA, 16, 64); accA += __shfl_xor(accA, 32, 64);
  accB += __shfl_xor(accB, 16, 64); accB += __shfl_xor(accB, 32, 64);
  if (lane < 16) {
    red[(w * 2 + 0) * 16 + lane] = accA;
    red[(w * 2 + 1) * 16 + lane] = accB;
  }
  if (w == 0) STAMP(5);
  __syncthreads();
  if (tid < 16) {
    float ga = 0.f, up = 0.f;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) {
      ga += red[(ww * 2 + 0) * 16 + tid];
      up += red[(ww * 2 + 1) * 16 + tid];
    }
    const float hv = ga / (1.f + expf(-ga)) * up;
    ((uint16_t *)c.out)[(size_t)wk.row0 * c.out_stride + b * 16 + tid] = f32_to_bf16(hv);
  }
  if (w == 0) STAMP(6);
}

// ---------------------------------------------------------------------------
// k3 (w2) + k5 for ONE token in one launch: a workgroup of 16 waves owns 8 output rows and walks
// the w2 tiles of those rows over ALL units (the k routed experts and the shared expert), weighting
// each unit as it accumulates, so the combine needs no launch of its own and no partial rows in memory.
//   An item is one quantisation group (128 columns) of one unit.  A tile holds 16 rows; the workgroup wants 8
//   of them, so a wave reads the halves of TWO items with one load: lanes whose tile row is 0..7 take the first,
//   the others the second, each its row & 7 of the workgroup's half.  The two items of a load are groups 2j and
//   2j + 1 of ONE unit (a unit with an odd number of groups ends with a load whose second item does not exist and
//   reads zeros).  Wave w takes the loads w, w + 16, ... of the list (unit 0's loads, unit 1's, ..., the shared
//   expert's) and requests up to W2C_CHUNK of them, each with the 256 bytes of the unit's h vector that its
//   items need, before the first product; it shares nothing with the other waves until the final sum.
//   H/8 workgroups: twice the compute units of a 16-row split, which is what the load latency wants.
// ---------------------------------------------------------------------------
#define W2C_WAVES 16
struct W2cArgs {
  const KUnit *kunits;   // resolved routed units (slot address; row = position of the unit's h vector)
  const float *unit_w;   // routing weight per unit position
  const uint16_t *h_r, *h_s;
  const unsigned char *shared_base;
  const float *sg_logit;  // shared expert's gate logit or NULL
  long long off_q, off_s, off_z, sh_off_q, sh_off_s, sh_off_z;
  int k, I, I_sh, H, G, G_sh;
  uint16_t *y;
  int *err;
};

// NI = items a wave reads with one load = 16 / (rows per workgroup); W2C_CHUNK = loads a wave keeps in flight
// (3 covers the whole share of a wave at 2048 x 1408 with six units; long reductions such as 4096 x 14336
// take 6, so that a wave's share is two round trips to memory instead of three or more)
template <int NI, int W2C_CHUNK>
__global__ __launch_bounds__(64 * W2C_WAVES, 1) void k_w2_combine_token(const W2cArgs a) {
  extern __shared__ __align__(16) unsigned char wsm[];
  constexpr int RW = 16 / NI;  // rows of this workgroup
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, qd = lane >> 4;
  // rows 16*b16 + RW*part .. + RW-1.  The two workgroups that share a 16-row tile (NI = 2) read the same lines of
  // its scale and zero sections; workgroup i runs on the part of the chip i mod 8 that has its own second-level
  // cache, so the pair is given indices that are equal mod 8 and the second one finds those lines there (with
  // adjacent indices both fetched them from memory: 1.09 x the launch's bytes)
  int b16 = blockIdx.x / NI, part = blockIdx.x % NI;
  if (NI == 2 && (gridDim.x & 15) == 0) {
    const int q = (int)blockIdx.x >> 3;
    part = q & 1;
    b16 = (q >> 1) * 8 + ((int)blockIdx.x & 7);
  }
  const int mine = r / RW;                                  // which item of the group this lane works on
  const int rr = RW * part + (r % RW);                      // its row inside the 16-row tile
  const int k = a.k, I = a.I, I_sh = a.I_sh, G = a.G, G_sh = a.G_sh;
  // wave-private LDS: the 128 activations of each item of the wave's current chunk, and their 32-wide sums.
  // A wave stages what its own items need and nothing else: no barrier between the requests and the products.
  constexpr int WAVE_DW = W2C_CHUNK * NI * 64 + W2C_CHUNK * NI * 4;
  uint16_t *hs = (uint16_t *)((u32 *)wsm + w * WAVE_DW);   // [W2C_CHUNK][NI][128] bf16
  float *xsum = (float *)((u32 *)wsm + w * WAVE_DW + W2C_CHUNK * NI * 64);  // [W2C_CHUNK][NI][4]
  float *red = (float *)((u32 *)wsm + W2C_WAVES * WAVE_DW);  // [W2C_WAVES][RW]
  const int zsh = (rr & 1) * 4;
  const int lj = lane >> 4, lpart = lane & 15;  // staging: 16 bytes of item lj of a group (lanes < 16 NI)
  // lane u holds unit u's slot address and weight (lane k: the shared expert); read back with readlane
  u32 ub_lo = 0, ub_hi = 0;
  float uw = 0.f;
  if (lane < k) {
    const unsigned long long ub = a.kunits[lane].base;
    ub_lo = (u32)ub; ub_hi = (u32)(ub >> 32);
    uw = a.unit_w[lane];
  } else if (lane == k) {
    const unsigned long long ub = (unsigned long long)a.shared_base;
    ub_lo = (u32)ub; ub_hi = (u32)(ub >> 32);
    uw = a.sg_logit ? 1.f / (1.f + expf(-a.sg_logit[0])) : 1.f;
  }

  // a selected expert that is not resident (slot address 0) is skipped below and reported here, by one wave of
  // the launch: the word may live in pinned host memory, where a store per wave would be thousands of
  // transactions over the host link
  if (blockIdx.x == 0 && w == 0) {
    const bool miss = (lane < k || (lane == k && I_sh > 0)) && ub_lo == 0 && ub_hi == 0;
    if (__ballot(miss) != 0ull && lane == 0) moe_raise_err(a.err);
  }
  const Q4Consts q4c = q4_consts();
  float acc = 0.f;
  // A unit's groups are padded to a multiple of NI, so the NI items a wave reads with one load belong to ONE unit
  // and everything about them but the lane's own byte offsets is wave-uniform: per load the scalar unit builds
  // four buffer descriptors (tiles, scales, zeros, the unit's h vector) whose lengths end at the unit's real
  // groups, and a padded, absent or not resident item reads zeros through them (zero weights, scale and
  // activations: no branch and no per-lane bookkeeping).  With the items enumerated without padding, a load's items
  // could straddle two units and every lane walked them with selects and 64-bit address arithmetic: 370 vector
  // operations per wave in front of the first request, 2 us on a SIMD that runs four such waves.
  const int GP = (G + NI - 1) / NI, GP_sh = (G_sh + NI - 1) / NI;  // loads per routed unit, for the shared expert
  // cursor of the wave's current load: unit u (k = the shared expert), load gp of that unit
  int u = 0, gp = w;
  while (u < k && gp >= GP) { gp -= GP; ++u; }
  // the lane's byte offsets inside a load's tiles, scale and zero sections and activations
  const int vq = mine * 1024 + (qd * 16 + rr) * 16, vs = mine * 32 + 2 * rr, vz = mine * 8 + (rr >> 1);
  const int vh = lj * 256 + lpart * 16;
  while (u < k || gp < GP_sh) {
    u32x4_t wt[W2C_CHUNK];
    u32 sc[W2C_CHUNK], zz[W2C_CHUNK];
    float wgt[W2C_CHUNK];
    uint4 hv[W2C_CHUNK];  // the lane's 16 bytes of the load's activations on their way into LDS
    // ---- request this chunk --------------------------------------------------------------------
#pragma unroll
    for (int c = 0; c < W2C_CHUNK; ++c) {
      const bool valid = u < k || gp < GP_sh;
      const bool shd = u >= k;
      const u32 lo = __builtin_amdgcn_readlane(ub_lo, u), hi = __builtin_amdgcn_readlane(ub_hi, u);
      wgt[c] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(u32, uw), u));
      const unsigned char *bp = (const unsigned char *)(((unsigned long long)hi << 32) | lo);
      const bool live = valid && bp != nullptr;
      const int Gu = shd ? G_sh : G;
      const u32 n = live ? (u32)Gu : 0u;  // groups the descriptors cover: none for a load that does not exist
      const size_t blk = (size_t)b16 * Gu;
      const rsrc_t rq = make_rsrc(bp + (shd ? a.sh_off_q : a.off_q) + blk * 1024, n * 1024u);
      const rsrc_t rs = make_rsrc(bp + (shd ? a.sh_off_s : a.off_s) + blk * 32, n * 32u);
      const rsrc_t rz = make_rsrc(bp + (shd ? a.sh_off_z : a.off_z) + blk * 8, n * 8u);
      const rsrc_t rh = make_rsrc(shd ? a.h_s : a.h_r + (size_t)u * I, n * 256u);
      const int g0 = NI * gp;
      // the activations first: memory answers a wave in order, and the products need them with the first tile
      hv[c] = make_uint4(0u, 0u, 0u, 0u);
      if (lj < NI) hv[c] = bload16(rh, vh + g0 * 256, 0);
      const uint4 t4 = bload16_nt(rq, vq + g0 * 1024, 0);
      wt[c] = u32x4_t{t4.x, t4.y, t4.z, t4.w};
      sc[c] = bload2(rs, vs + g0 * 32, 0);
      zz[c] = bload1(rz, vz + g0 * 8, 0);
      if (valid) {  // next load of this wave
        gp += W2C_WAVES;
        while (u < k && gp >= GP) { gp -= GP; ++u; }
      }
    }
    // ---- the chunk's activations (+ 32-wide sums) into the wave's own LDS area ----------------------
#pragma unroll
    for (int c = 0; c < W2C_CHUNK; ++c) {
      float ps = sum8_bf16(hv[c]);
      ps += __shfl_xor(ps, 1, 64);
      ps += __shfl_xor(ps, 2, 64);
      if (lj < NI) {
        ((uint4 *)hs)[(c * NI + lj) * 16 + lpart] = hv[c];
        if ((lane & 3) == 0) xsum[(c * NI + lj) * 4 + (lpart >> 2)] = ps;
      }
    }
    __builtin_amdgcn_wave_barrier();  // (no instruction: the reads below stay behind the stores of other lanes)
    // ---- products: no branch, an absent item has zero weights, a zero scale and zero activations
#pragma unroll
    for (int c = 0; c < W2C_CHUNK; ++c) {
      const uint4 *xp = (const uint4 *)(hs + (c * NI + mine) * 128 + qd * 32);  // the lane's 32 activations
      const uint4 x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
      const float xq = xsum[(c * NI + mine) * 4 + qd];
      const float d0 = dot8_q4(wt[c].x, x0, 0.f, q4c), d1 = dot8_q4(wt[c].y, x1, 0.f, q4c);
      const float d2 = dot8_q4(wt[c].z, x2, 0.f, q4c), d3 = dot8_q4(wt[c].w, x3, 0.f, q4c);
      const float d = (d0 + d1) + (d2 + d3);
      const float fs = half_bits_to_f32((uint16_t)sc[c]);
      const float fz = 128.f + (float)((zz[c] >> zsh) & 15);
      acc = fmaf(wgt[c] * fs, d - fz * xq, acc);
    }
    __builtin_amdgcn_wave_barrier();  // the next chunk's stores stay behind this chunk's reads
  }
  // the items of the groups, the four k quarters of the wave, then the waves
#pragma unroll
  for (int m = RW; m < 16; m <<= 1) acc += __shfl_xor(acc, m, 64);
  acc += __shfl_xor(acc, 16, 64);
  acc += __shfl_xor(acc, 32, 64);
  if (lane < RW) red[w * RW + lane] = acc;
  __syncthreads();
  if (tid < RW) {
    float v = 0.f;
#pragma unroll
    for (int ww = 0; ww < W2C_WAVES; ++ww) v += red[ww * RW + tid];
    a.y[b16 * 16 + RW * part + tid] = f32_to_bf16(v);
  }
}

// ---------------------------------------------------------------------------
// k3, matrix-core form: same work split and load section as k_gemv_int4, but the
// products run on v_mfma_f32_16x16x32_bf16 with the (up to 16) tokens of the unit as
// the N dimension, so the weight tiles are dequantised once for all tokens.
//   A (16 rows x 32 k): lane l = row l&15, k-chunk l>>4 -> exactly one dequantised dword
//   B (32 k x 16 tok) : lane l = token l&15, k-chunk l>>4 -> 16 bytes of that token's row
//   D (16 x 16)       : lane l holds rows 4(l>>4)+i, token l&15
// Per tile (one quantisation group): D_g = sum (128+q) x ; acc += s_row (D_g - (128+z_row) X_tok,g).
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
// two fp16 scales and their two zero nibbles (bits 0..7 of z) -> (s0, -s0 (128 + z0), s1, -s1 (128 + z1))
static __device__ __forceinline__ float4 scale_zero_pair(u32 sc, u32 z) {
  const float s0 = half_bits_to_f32((uint16_t)sc), s1 = half_bits_to_f32((uint16_t)(sc >> 16));
  return make_float4(s0, -s0 * (128.f + (float)(z & 15)), s1, -s1 * (128.f + (float)((z >> 4) & 15)));
}
typedef float f32x4_t __attribute__((ext_vector_type(4)));

static __device__ __forceinline__ bf16x8_t deq8_bf16(u32 w, const Q4Consts &q) {
  const u32 M = q.M, C = q.C;  // in vector registers: one v_and_or_b32 per pair
  u32x4_t v;
  v.x = (w & M) | C; v.y = ((w >> 4) & M) | C; v.z = ((w >> 8) & M) | C; v.w = ((w >> 12) & M) | C;
  return __builtin_bit_cast(bf16x8_t, v);
}
static __device__ __forceinline__ bf16x8_t as_bf16x8(const uint4 &x) {
  u32x4_t v; v.x = x.x; v.y = x.y; v.z = x.z; v.w = x.w;
  return __builtin_bit_cast(bf16x8_t, v);
}

// ROUTE (w13 pass, device-side slot table): the launch sums the gate rows and routes by itself, see
// gemv_resolve_route_batch_n; a unit's token rows then come from its token mask, not from a list in memory
template <bool SWIGLU, int CH, bool DEVUNITS, bool ROUTE = false>
__global__ __launch_bounds__(256, (ROUTE ? 4 : 2)) void k_gemv_int4_mfma(const GemvArgs a, const int TB, const int RPW_R, const int RPW_S) {
  constexpr int NP = 1, NB = 2 * NP;  // block pairs / 16-row blocks per iteration
  constexpr int PF = 4;               // activation pieces in flight while staging
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, qd = lane >> 4;
  const Q4Consts q4c = q4_consts();

  // a publishing workgroup comes first in the grid: it is over long before the ones that stream weights
  const bool publishes = !ROUTE && SWIGLU && DEVUNITS && a.p_host_units != nullptr;
  if (publishes && blockIdx.x == 0) {
    gemv_publish_units(a);
    return;
  }
  int bx = (int)blockIdx.x - (publishes ? 1 : 0);
  unsigned tokmask = 0u;   // ROUTE: the tokens of a routed unit
  bool masked = false;
  GemvWork wk;
  if constexpr (ROUTE) {
    if (bx < a.g_nblk) {
      if (a.T <= 4) gate_rows_batch_tg<1>(a, lane, w, bx);
      else gate_rows_batch_tg<2>(a, lane, w, bx);
      return;
    }
    bx -= a.g_nblk;
    if (bx == 0) { route_publish_batch(a, smem); return; }
    bx -= 1;
    if (bx < a.n_sh_blocks) {
      wk.c = a.cls[0]; wk.b = bx; wk.half = 0; wk.m = a.T; wk.row0 = 0; wk.base = a.shared_base;
    } else {
      if (a.T <= 4) wk = gemv_resolve_route_batch<1>(a, lane, w, bx - a.n_sh_blocks, tokmask);
      else wk = gemv_resolve_route_batch<2>(a, lane, w, bx - a.n_sh_blocks, tokmask);
      masked = true;
    }
  } else {
    wk = gemv_resolve<DEVUNITS>(a, bx);
  }
  const GemvClass &c = wk.c;
  const int m = wk.m, row0 = wk.row0;
  const unsigned char *base = wk.base;
  if (m <= 0) return;
  if (base == nullptr) {
    if (tid == 0) moe_raise_err(a.err);
    return;
  }
  const int K = c.K, G = c.G;
  // block pairs of this workgroup: the shared expert sees every token, so its workgroups take fewer
  const int RPW = bx < a.n_sh_blocks ? RPW_S : RPW_R;
  const int XS = K * 2 + 16;  // padded row stride (bytes): 16 token rows hit 16 distinct bank quads
  unsigned char *xs = smem;                                           // [TB][XS]
  float *xsum = (float *)(smem + (size_t)TB * XS);                    // [TB][G]
  // per (block, group, row): scale s and -s (128 + zero), so that a row's update is two fma's
  float *s_f = xsum + (((size_t)TB * G + 3) & ~(size_t)3);            // [NB][G][16][2], 16-B aligned
  float *red = s_f + NB * G * 32;                                     // [4][NB][16 rows][16 tok]

  const int GPW = (G - w + 3) >> 2;
  const rsrc_t rx = make_rsrc(c.act, 0x7fffffffu);
  const int vec_per_row = K >> 3;
  const int n_sc = NB * G * 8;  // scale dwords (two rows each) of one iteration

  for (int t0 = 0; t0 < m; t0 += TB) {
    const int mc = (m - t0) < TB ? (m - t0) : TB;
   // RPW consecutive (gate,up) / (row,row) block pairs per workgroup: the activations are staged
   // once and the fixed per-workgroup cost is spread over more weight tiles
   for (int pp = 0; pp < RPW; pp += NP) {
    const int b = wk.b * RPW + pp;
    const int rbA = 2 * b;
    const rsrc_t rq = make_rsrc(base + c.off_q + (size_t)rbA * G * 1024, (u32)NB * G * 1024u);
    const rsrc_t rs = make_rsrc(base + c.off_s + (size_t)rbA * G * 32, (u32)NB * G * 32u);
    const rsrc_t rz = make_rsrc(base + c.off_z + (size_t)rbA * G * 8, (u32)NB * G * 8u);
    // ---- straight-line load section ------------------------------------------------------
    const int row_first = row0 + t0;
    const int arow0 = (ROUTE && masked) ? __builtin_amdgcn_readfirstlane(nth_token(tokmask, t0))
                                        : (c.gather ? c.gather[row_first] : row_first);
    const uint4 xv0 = bload16(rx, (tid < vec_per_row ? tid : 0) * 16, arow0 * c.act_stride * 2);
    // scale dword e = (block, group, row pair j) and the zero dword that holds its two nibbles
    const int zoff = ((tid >> 3) * 2 + ((tid & 7) >> 2)) * 4;
    const u32 msc0 = bload4(rs, tid * 4, 0), msc1 = bload4(rs, tid * 4, 1024);
    const u32 mz0 = bload4(rz, zoff, 0), mz1 = bload4(rz, zoff, 256);
    uint4 wt[CH][NB];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int g = j < GPW ? w + 4 * j : 0;
#pragma unroll
      for (int n = 0; n < NB; ++n) wt[j][n] = bload16_nt(rq, lane * 16, (n * G + g) * 1024);
    }
    // ---- stage x rows (+ per-group sums over 128 values = 16 consecutive vectors) ----------
    if (pp == 0) {
      float ps = sum8_bf16(xv0);
      ps += __shfl_xor(ps, 1, 64); ps += __shfl_xor(ps, 2, 64);
      ps += __shfl_xor(ps, 4, 64); ps += __shfl_xor(ps, 8, 64);
      if (tid < vec_per_row) {
        *(uint4 *)(xs + (size_t)tid * 16) = xv0;
        if ((tid & 15) == 0) xsum[tid >> 4] = ps;
      }
    }
    const int zsh = 8 * (tid & 3);  // the pair's nibbles inside its zero dword
    if (tid < n_sc) ((float4 *)s_f)[tid] = scale_zero_pair(msc0, mz0 >> zsh);
    if (tid + 256 < n_sc) ((float4 *)s_f)[tid + 256] = scale_zero_pair(msc1, mz1 >> zsh);
    // remaining (row, 256-vector chunk) pieces, PF loads in flight at a time; piece 0 is
    // the early load above
    if (pp == 0) {
      const int cpr = (vec_per_row + 255) >> 8;  // chunks per row
      const int total = mc * cpr;
      // row index of every token of this pass, one per lane (lanes >= mc repeat the last)
      const int grow = row_first + (lane < mc ? lane : mc - 1);
      const int arow_l = (ROUTE && masked) ? nth_token(tokmask, t0 + (lane < mc ? lane : mc - 1))
                                           : (c.gather ? c.gather[grow] : grow);
      for (int pb = 1; pb < total; pb += PF) {
        uint4 xb[PF];
#pragma unroll
        for (int q = 0; q < PF; ++q) {
          // groups of four past the end are skipped (uniform branch); inside a group the index is clamped
          if ((q & 3) == 0 || pb + (q & ~3) < total) {
            const int pi = pb + q < total ? pb + q : 0;
            const int t = pi / cpr, ch = pi - t * cpr;
            const int v = tid + 256 * ch;
            const int arow = __builtin_amdgcn_readlane(arow_l, t);
            xb[q] = bload16(rx, (v < vec_per_row ? v : 0) * 16, arow * c.act_stride * 2);
          } else {
            xb[q] = make_uint4(0u, 0u, 0u, 0u);
          }
        }
#pragma unroll
        for (int q = 0; q < PF; ++q) {
          const int pi = pb + q;
          if (pi >= total) break;
          const int t = pi / cpr, ch = pi - t * cpr;
          const int v = tid + 256 * ch;
          float ps = sum8_bf16(xb[q]);
          ps += __shfl_xor(ps, 1, 64); ps += __shfl_xor(ps, 2, 64);
          ps += __shfl_xor(ps, 4, 64); ps += __shfl_xor(ps, 8, 64);
          if (v < vec_per_row) {
            *(uint4 *)(xs + (size_t)t * XS + (size_t)v * 16) = xb[q];
            if ((tid & 15) == 0) xsum[t * G + (v >> 4)] = ps;
          }
        }
      }
    }
    for (int i = tid + 512; i < n_sc; i += 256)
      ((float4 *)s_f)[i] = scale_zero_pair(bload4(rs, i * 4, 0), bload4(rz, zoff + (i >> 8) * 256, 0) >> zsh);
    __syncthreads();

    f32x4_t acc[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) acc[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int tok = r < mc ? r : mc - 1;  // lanes past the last token repeat it (ignored later)
    const unsigned char *xrow = xs + (size_t)tok * XS + qd * 64;

    for (int jc = 0; jc < GPW; jc += CH) {
      if (jc > 0) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
          const int g = jc + j < GPW ? w + 4 * (jc + j) : 0;
#pragma unroll
          for (int n = 0; n < NB; ++n) wt[j][n] = bload16_nt(rq, lane * 16, (n * G + g) * 1024);
        }
      }
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        if (jc + j < GPW) {  // (uniform: a partial last chunk holds a clamped, duplicate tile)
          const int g = w + 4 * (jc + j);
          const uint4 *xp = (const uint4 *)(xrow + g * 256);
          const bf16x8_t x0 = as_bf16x8(xp[0]), x1 = as_bf16x8(xp[1]), x2 = as_bf16x8(xp[2]), x3 = as_bf16x8(xp[3]);
          const float xg = xsum[tok * G + g];
          f32x4_t d[NB];
#pragma unroll
          for (int n = 0; n < NB; ++n) d[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int n = 0; n < NB; ++n) d[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(deq8_bf16(wt[j][n].x, q4c), x0, d[n], 0, 0, 0);
#pragma unroll
          for (int n = 0; n < NB; ++n) d[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(deq8_bf16(wt[j][n].y, q4c), x1, d[n], 0, 0, 0);
#pragma unroll
          for (int n = 0; n < NB; ++n) d[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(deq8_bf16(wt[j][n].z, q4c), x2, d[n], 0, 0, 0);
#pragma unroll
          for (int n = 0; n < NB; ++n) d[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(deq8_bf16(wt[j][n].w, q4c), x3, d[n], 0, 0, 0);
#pragma unroll
          for (int n = 0; n < NB; ++n) {
            // (s, -s (128 + z)) of the 4 rows this lane owns in D: rows 4qd..4qd+3
            const float4 *sf = (const float4 *)(s_f + ((n * G + g) * 16 + 4 * qd) * 2);
            const float4 f0 = sf[0], f1 = sf[1];
            acc[n][0] = fmaf(f0.x, d[n][0], fmaf(f0.y, xg, acc[n][0]));
            acc[n][1] = fmaf(f0.z, d[n][1], fmaf(f0.w, xg, acc[n][1]));
            acc[n][2] = fmaf(f1.x, d[n][2], fmaf(f1.y, xg, acc[n][2]));
            acc[n][3] = fmaf(f1.z, d[n][3], fmaf(f1.w, xg, acc[n][3]));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // cross-wave reduction: red[w][block][row][tok]
#pragma unroll
    for (int n = 0; n < NB; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[((w * NB + n) * 16 + 4 * qd + i) * 16 + r] = acc[n][i];
    __syncthreads();
    {
      const int row = tid >> 4, t = tid & 15;  // 256 threads = 16 rows x 16 tokens
      float v[NB];
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        v[n] = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) v[n] += red[((ww * NB + n) * 16 + row) * 16 + t];
      }
      if (t < mc) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
          const float va = v[2 * q], vb = v[2 * q + 1];
          if (SWIGLU) {
            const float hv = va / (1.f + expf(-va)) * vb;
            ((uint16_t *)c.out)[(size_t)(row_first + t) * c.out_stride + (b + q) * 16 + row] = f32_to_bf16(hv);
          } else {
            float *o = (float *)c.out + (size_t)(row_first + t) * c.out_stride + 2 * (b + q) * 16 + row;
            o[0] = va;
            o[16] = vb;
          }
        }
      }
    }
    if (pp + NP < RPW) __syncthreads();
   }
    if (t0 + TB < m) __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// k3, matrix-core form for long reductions and for up to 32 rows per pass.  Same tiles, same
// products and the same scale/zero correction as k_gemv_int4_mfma, different work split:
//   * KS waves own one block pair (gate/up blocks, or two row blocks) over the whole reduction; a
//     workgroup = 4 / KS adjacent pairs of one unit.  KS = 1: no cross-wave reduction at all; KS = 2, 4
//     (launches with few block pairs): the waves of a pair take 1 / KS of every chunk's groups and their
//     sums meet in LDS once, at the end, in a fixed order;
//   * the activations are staged CG groups (CG x 128 columns) at a time, double-buffered, one
//     barrier per chunk, so the LDS footprint does not grow with K (two workgroups per CU at any K);
//   * the weight tiles of the wave's next step and the activations and scales of the next chunk
//     are in flight while the current ones are worked on;
//   * NT = 2: two 16-token column blocks per pass share every dequantised weight tile.
// ---------------------------------------------------------------------------
// Length of the activations' buffer resource in the chunked-K kernels, and the offset that stands for "no row": the
// first byte past it, so that such a load is out of range by any reading of the range rule (first byte or last
// byte of the access, no 32-bit wrap) and returns zeros without a memory request.
#define KC_NO_ROW 0x7fffff00u
#ifdef MOE_STAMPS
#ifndef KC_STAMP_SW
#define KC_STAMP_SW true
#endif
#define KC_STAMP(i) do { if (SWIGLU == KC_STAMP_SW) STAMP(i); } while (0)
#define KC_STAMPV(i, v) do { if (SWIGLU == KC_STAMP_SW) STAMPV(i, v); } while (0)
#else
#define KC_STAMP(i)
#define KC_STAMPV(i, v)
#endif

// One pass of the chunked-K form: rows row_first .. row_first + mc - 1 (mc <= 16 NT) of one unit against the block
// pair b of its matrix.  Every thread of the workgroup takes part (barriers inside).
// MASKED with tokmask != 0: the pass's rows are the tokens of that bit mask (a unit of a launch that routes by
// itself, all of its rows in this one pass) instead of c.gather's
template <bool SWIGLU, int NT, int CG, int KS, bool MASKED = false>
static __device__ __forceinline__ void kc_pass(const GemvClass &c, unsigned char *smem, const rsrc_t rq, const rsrc_t rs,
                                               const rsrc_t rz, const rsrc_t rx, const int b, const int row_first,
                                               const int mc, const Q4Consts &q4c, const unsigned tokmask = 0u) {
  constexpr int NB = 2;                // 16-row blocks per wave
  constexpr int GW = CG / KS;          // groups per wave and chunk
  constexpr int WS = GW < 4 ? GW : 4;  // groups per weight step
  constexpr int SPC = GW / WS;         // weight steps per wave and chunk
  constexpr int TBK = 16 * NT;         // token rows per pass
  constexpr int XSC = CG * 256 + 16;   // padded row stride of a staged chunk (bytes)
  constexpr int XV = CG * 16;          // 16-byte vectors per row and chunk
  constexpr int NPC = TBK * XV / 256;  // vectors per thread and chunk
  constexpr int NSE = NB * GW * 8;     // scale dwords (two rows each) per wave and chunk
  constexpr int NSD = (NSE + 63) / 64;
  static_assert(CG % KS == 0 && GW >= 1 && GW == SPC * WS && (SPC == 1 || SPC == 2) && NPC >= 1, "chunk shape");
  static_assert(4 * NB * NT * 4 * 64 * 4 <= 2 * TBK * XSC, "the partial sums reuse the activation buffers");
  // the thread index is made opaque per pass: what a pass shape derives from it (staging addresses, scale
  // indices) would otherwise be hoisted out of the caller's loop over passes, for all shapes at once, and
  // the registers that holds spill
  int tid_ = threadIdx.x;
  asm volatile("" : "+v"(tid_));
  const int tid = tid_, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, qd = lane >> 4;
  const int kh = w % KS;  // which part of every chunk this wave takes
  const int K = c.K, G = c.G;
  unsigned char *xs = smem;                                   // [2][TBK][XSC]
  float *xsum = (float *)(smem + (size_t)2 * TBK * XSC);      // [2][TBK][CG]
  float *sfw = xsum + 2 * TBK * CG + w * (NB * CG * 32);      // this wave's [NB][GW][16 rows][2]
  const int NCH = (G + CG - 1) / CG;  // activation chunks
  // first group of this wave's weight step i (steps past the end of the reduction are empty;
  // the non-empty ones are a prefix)
  auto step_group = [&](const int i) { return (i / SPC) * CG + kh * GW + (i % SPC) * WS; };

  // byte offset of the activation row behind each of this thread's vectors (rows past the last token: -1, their
  // loads go past the end of the buffer resource, which returns zeros and asks the memory for nothing; they are
  // staged but never read)
  int xoff[NPC];
#pragma unroll
  for (int i = 0; i < NPC; ++i) {
    const int row = (tid + 256 * i) / XV;
    const int gr = row_first + (row < mc ? row : mc - 1);
    if (MASKED && tokmask != 0u) xoff[i] = row < mc ? nth_token(tokmask, row) * c.act_stride * 2 : -1;
    else xoff[i] = row < mc ? (c.gather ? c.gather[gr] : gr) * c.act_stride * 2 : -1;
  }
  uint4 xr[NPC];
  u32 scr[NSD], zr[NSD];
  // loads of one chunk: activations, this wave's scale dwords and the zero dwords that hold their
  // nibbles (groups past the end of the reduction: zero activations, zero scales)
  auto load_chunk = [&](const int ch) {
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int kv = ch * XV + ((tid + 256 * i) & (XV - 1));
      // columns past K: any valid address; chunk_begin zeroes them (a select here would wait for the load)
      xr[i] = bload16(rx, xoff[i] < 0 ? (int)KC_NO_ROW : xoff[i] + (kv * 8 < K ? kv * 16 : 0), 0);
    }
#pragma unroll
    for (int i = 0; i < NSD; ++i) {
      const int e = lane + 64 * i;
      const int n = e / (GW * 8), g = ch * CG + kh * GW + ((e % (GW * 8)) >> 3), j = e & 7;
      const bool ok = e < NSE && g < G;
      scr[i] = bload4(rs, ok ? ((n * G + g) * 8 + j) * 4 : 0x7ffffff0, 0);
      zr[i] = bload4(rz, ok ? (n * G + g) * 8 + (j >> 2) * 4 : 0x7ffffff0, 0);
    }
  };
  auto load_w = [&](const int i, uint4 (&wt_)[WS][NB]) {
    const int g0 = step_group(i);
#pragma unroll
    for (int j = 0; j < WS; ++j) {
      const int g = g0 + j < G ? g0 + j : G - 1;
#pragma unroll
      // (plain loads here: popular experts take several passes at 32 and 64 tokens and find their tiles in the caches;
      // marked non-temporal, a 64-token step took 128.8 instead of 126.9 us)
      for (int n = 0; n < NB; ++n) wt_[j][n] = bload16(rq, lane * 16, (n * G + g) * 1024);
    }
  };
  f32x4_t acc[NB][NT];
#pragma unroll
  for (int n = 0; n < NB; ++n)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[n][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  int tokl[NT];  // lanes past the last token repeat it (their columns are not stored)
#pragma unroll
  for (int t = 0; t < NT; ++t) tokl[t] = 16 * t + r < mc ? 16 * t + r : mc - 1;

  // registers -> LDS for chunk ch, barrier, then the next chunk's loads
  auto chunk_begin = [&](const int ch) {
    const int cb = ch & 1;
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int p = tid + 256 * i;
      const int row = p / XV, v = p & (XV - 1);
      const uint4 xq = (ch * XV + v) * 8 < K ? xr[i] : make_uint4(0u, 0u, 0u, 0u);
      float ps = sum8_bf16(xq);
      ps += __shfl_xor(ps, 1, 64); ps += __shfl_xor(ps, 2, 64);
      ps += __shfl_xor(ps, 4, 64); ps += __shfl_xor(ps, 8, 64);
      *(uint4 *)(xs + ((size_t)cb * TBK + row) * XSC + (size_t)v * 16) = xq;
      if ((tid & 15) == 0) xsum[(cb * TBK + row) * CG + (v >> 4)] = ps;
    }
#pragma unroll
    for (int i = 0; i < NSD; ++i) {
      const int e = lane + 64 * i;
      if (e < NSE) ((float4 *)sfw)[e] = scale_zero_pair(scr[i], zr[i] >> (8 * (e & 3)));
    }
    __syncthreads();
    if (ch == 0) KC_STAMP(2);
    // unconditional (past the end: clamped addresses, zero scales), so that every iteration issues the
    // same number of loads and the waits for the prefetched registers can be exact
    load_chunk(ch + 1);
  };
  // this wave's weight step i on the tiles in cur; the next step's tiles go to nxt first
  auto step = [&](const int i, uint4 (&cur)[WS][NB], uint4 (&nxt)[WS][NB]) {
    const int g0 = step_group(i);
    load_w(i + 1, nxt);  // unconditional, clamped: see chunk_begin
    if (g0 >= G) return;
    const int cb = (i / SPC) & 1;
#pragma unroll
    for (int j = 0; j < WS; ++j) {
      if (g0 + j < G) {  // uniform
        const int gl = (i % SPC) * WS + j;  // group within this wave's part of the chunk
        const int gq = kh * GW + gl;        // and within the chunk
        if constexpr (NT >= 4) {
          // wide passes: the dequantised tiles of both blocks stay in registers and the token blocks pass by
          // (32 + 16 registers live, where activations-first holds 16 NT + 16)
          bf16x8_t wd[NB][4];
          float4 f0[NB], f1[NB];
#pragma unroll
          for (int n = 0; n < NB; ++n) {
            wd[n][0] = deq8_bf16(cur[j][n].x, q4c); wd[n][1] = deq8_bf16(cur[j][n].y, q4c);
            wd[n][2] = deq8_bf16(cur[j][n].z, q4c); wd[n][3] = deq8_bf16(cur[j][n].w, q4c);
            const float4 *sf = (const float4 *)(sfw + ((n * GW + gl) * 16 + 4 * qd) * 2);
            f0[n] = sf[0]; f1[n] = sf[1];
          }
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const uint4 *xp = (const uint4 *)(xs + ((size_t)cb * TBK + tokl[t]) * XSC + gq * 256 + qd * 64);
            const bf16x8_t x0 = as_bf16x8(xp[0]), x1 = as_bf16x8(xp[1]), x2 = as_bf16x8(xp[2]), x3 = as_bf16x8(xp[3]);
            const float xg = xsum[(cb * TBK + tokl[t]) * CG + gq];
#pragma unroll
            for (int n = 0; n < NB; ++n) {
              f32x4_t d = f32x4_t{0.f, 0.f, 0.f, 0.f};
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[n][0], x0, d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[n][1], x1, d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[n][2], x2, d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[n][3], x3, d, 0, 0, 0);
              acc[n][t][0] = fmaf(f0[n].x, d[0], fmaf(f0[n].y, xg, acc[n][t][0]));
              acc[n][t][1] = fmaf(f0[n].z, d[1], fmaf(f0[n].w, xg, acc[n][t][1]));
              acc[n][t][2] = fmaf(f1[n].x, d[2], fmaf(f1[n].y, xg, acc[n][t][2]));
              acc[n][t][3] = fmaf(f1[n].z, d[3], fmaf(f1[n].w, xg, acc[n][t][3]));
            }
          }
          __builtin_amdgcn_sched_barrier(0);  // keeps the next group's dequantisation out of this one's registers
        } else {
          bf16x8_t xv[NT][4];
          float xg[NT];
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const uint4 *xp = (const uint4 *)(xs + ((size_t)cb * TBK + tokl[t]) * XSC + gq * 256 + qd * 64);
            xv[t][0] = as_bf16x8(xp[0]); xv[t][1] = as_bf16x8(xp[1]);
            xv[t][2] = as_bf16x8(xp[2]); xv[t][3] = as_bf16x8(xp[3]);
            xg[t] = xsum[(cb * TBK + tokl[t]) * CG + gq];
          }
#pragma unroll
          for (int n = 0; n < NB; ++n) {
            const bf16x8_t w0 = deq8_bf16(cur[j][n].x, q4c), w1 = deq8_bf16(cur[j][n].y, q4c);
            const bf16x8_t w2 = deq8_bf16(cur[j][n].z, q4c), w3 = deq8_bf16(cur[j][n].w, q4c);
            // (s, -s (128 + z)) of the 4 rows this lane owns in D: rows 4qd..4qd+3
            const float4 *sf = (const float4 *)(sfw + ((n * GW + gl) * 16 + 4 * qd) * 2);
            const float4 f0 = sf[0], f1 = sf[1];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              f32x4_t d = f32x4_t{0.f, 0.f, 0.f, 0.f};
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, xv[t][0], d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, xv[t][1], d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2, xv[t][2], d, 0, 0, 0);
              d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w3, xv[t][3], d, 0, 0, 0);
              acc[n][t][0] = fmaf(f0.x, d[0], fmaf(f0.y, xg[t], acc[n][t][0]));
              acc[n][t][1] = fmaf(f0.z, d[1], fmaf(f0.w, xg[t], acc[n][t][1]));
              acc[n][t][2] = fmaf(f1.x, d[2], fmaf(f1.y, xg[t], acc[n][t][2]));
              acc[n][t][3] = fmaf(f1.z, d[3], fmaf(f1.w, xg[t], acc[n][t][3]));
            }
          }
        }
      }
    }
  };

  uint4 wA[WS][NB], wB[WS][NB];
  load_chunk(0);
  load_w(0, wA);
  if constexpr (SPC == 2) {
    for (int ch = 0; ch < NCH; ++ch) {
      chunk_begin(ch);
      step(2 * ch, wA, wB);
      step(2 * ch + 1, wB, wA);
    }
  } else {
    for (int ch = 0; ch < NCH; ch += 2) {
      chunk_begin(ch);
      step(ch, wA, wB);
      if (ch + 1 < NCH) {
        chunk_begin(ch + 1);
        step(ch + 1, wB, wA);
      }
    }
  }
  KC_STAMP(3);
  if constexpr (KS > 1) {
    // the sums of a pair's waves meet in the activation buffers (free once every wave is done with them)
    __syncthreads();
    float *red = (float *)smem;  // [4 waves][NB][NT][4][64 lanes]
    if (kh != 0) {
#pragma unroll
      for (int n = 0; n < NB; ++n)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) red[((w * NB + n) * NT + t) * 256 + i * 64 + lane] = acc[n][t][i];
    }
    __syncthreads();
    if (kh == 0) {
#pragma unroll
      for (int q = 1; q < KS; ++q)
#pragma unroll
        for (int n = 0; n < NB; ++n)
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[n][t][i] += red[(((w + q) * NB + n) * NT + t) * 256 + i * 64 + lane];
    }
  }
  // every lane holds 4 consecutive rows of both blocks for one token per column block
  if (kh == 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (16 * t + r < mc) {
        const size_t orow = (size_t)(row_first + 16 * t + r) * c.out_stride;
        if (SWIGLU) {
          u32 h[2];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const float g0 = acc[0][t][2 * i], g1 = acc[0][t][2 * i + 1];
            const float h0 = g0 / (1.f + expf(-g0)) * acc[1][t][2 * i];
            const float h1 = g1 / (1.f + expf(-g1)) * acc[1][t][2 * i + 1];
            h[i] = (u32)f32_to_bf16(h0) | ((u32)f32_to_bf16(h1) << 16);
          }
          *(uint2 *)((uint16_t *)c.out + orow + b * 16 + 4 * qd) = make_uint2(h[0], h[1]);
        } else {
#pragma unroll
          for (int n = 0; n < NB; ++n)
            *(float4 *)((float *)c.out + orow + (2 * b + n) * 16 + 4 * qd) =
                make_float4(acc[n][t][0], acc[n][t][1], acc[n][t][2], acc[n][t][3]);
        }
      }
    }
  }
}

// The same pass over q4_K tiles.  A lane's 32 weights of a tile are one 32-wide sub-block of its row, with its own
// 6-bit (scale, min) pair under the (d, dmin) of the row's 256-wide super-block, so nothing can be factored out
// of a group's products: every weight is dequantised completely (d sc q - dmin m, one packed fp16 fma per pair, the
// arithmetic of the tile kernels for longer batches) and the products accumulate on the matrix cores in fp32.  The
// activations are staged as fp16 (exact from bf16); no sums of activations are needed.  The (scale, min) pair and
// the (d, dmin) pair of a tile travel with it, one 2-byte and one 4-byte load per lane.
// Gt: groups per row block in memory; the pass reduces over the window of G groups that the resources start at.
template <bool SWIGLU, int NT, int CG, int KS>
static __device__ __forceinline__ void kc_pass_q4k(const GemvClass &c, unsigned char *smem, const rsrc_t rq,
                                                   const rsrc_t rs, const rsrc_t rz, const rsrc_t rx, const int Gt,
                                                   const int G, const int b, const size_t out_row0, const int row_first,
                                                   const int mc, const DeqF16Consts &dqc) {
  constexpr int NB = 2, GW = CG / KS, WS = GW < 4 ? GW : 4, SPC = GW / WS, TBK = 16 * NT;
  constexpr int XSC = CG * 256 + 16, XV = CG * 16, NPC = TBK * XV / 256;
  static_assert(CG % KS == 0 && GW >= 1 && GW == SPC * WS && (SPC == 1 || SPC == 2) && NPC >= 1, "chunk shape");
  static_assert(4 * NB * NT * 4 * 64 * 4 <= 2 * TBK * XSC, "the partial sums reuse the activation buffers");
  int tid_ = threadIdx.x;
  asm volatile("" : "+v"(tid_));  // see kc_pass
  const int tid = tid_, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, qd = lane >> 4;
  const int kh = w % KS;
  const int K = G * 128;
  unsigned char *xs = smem;  // [2][TBK][XSC] fp16
  const int NCH = (G + CG - 1) / CG;
  auto step_group = [&](const int i) { return (i / SPC) * CG + kh * GW + (i % SPC) * WS; };

  int xoff[NPC];
#pragma unroll
  for (int i = 0; i < NPC; ++i) {
    const int row = (tid + 256 * i) / XV;
    const int gr = row_first + (row < mc ? row : mc - 1);
    xoff[i] = row < mc ? (c.gather ? c.gather[gr] : gr) * c.act_stride * 2 : -1;
  }
  uint4 xr[NPC];
  auto load_chunk = [&](const int ch) {
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int kv = ch * XV + ((tid + 256 * i) & (XV - 1));
      xr[i] = bload16(rx, xoff[i] < 0 ? (int)KC_NO_ROW : xoff[i] + (kv * 8 < K ? kv * 16 : 0), 0);
    }
  };
  struct Tiles { uint4 q[WS][NB]; u32 sm[WS][NB], dd[WS][NB]; };
  auto load_w = [&](const int i, Tiles &t_) {
    const int g0 = step_group(i);
#pragma unroll
    for (int j = 0; j < WS; ++j) {
      const int g = g0 + j < G ? g0 + j : G - 1;
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        const int tile = n * Gt + g;
        t_.q[j][n] = bload16_nt(rq, lane * 16, tile * 1024);
        t_.sm[j][n] = bload2(rs, lane * 2, tile * 128);
        t_.dd[j][n] = bload4(rz, r * 4, (tile >> 1) * 64);
      }
    }
  };
  f32x4_t acc[NB][NT];
#pragma unroll
  for (int n = 0; n < NB; ++n)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[n][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  int tokl[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) tokl[t] = 16 * t + r < mc ? 16 * t + r : mc - 1;

  auto chunk_begin = [&](const int ch) {
    const int cb = ch & 1;
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int p = tid + 256 * i;
      const int row = p / XV, v = p & (XV - 1);
      const bool in = (ch * XV + v) * 8 < K;
      uint4 xq;
      xq.x = in ? bf16x2_to_f16x2(xr[i].x) : 0u; xq.y = in ? bf16x2_to_f16x2(xr[i].y) : 0u;
      xq.z = in ? bf16x2_to_f16x2(xr[i].z) : 0u; xq.w = in ? bf16x2_to_f16x2(xr[i].w) : 0u;
      *(uint4 *)(xs + ((size_t)cb * TBK + row) * XSC + (size_t)v * 16) = xq;
    }
    __syncthreads();
    load_chunk(ch + 1);  // unconditional: see kc_pass
  };
  // the 8 fp16 weights behind each dword of a lane's tile row
  auto deq_tile = [&](const uint4 &q, const u32 sm, const u32 dd, f16x8_t (&wd)[4]) {
    const float s16 = 16.f * half_bits_to_f32((uint16_t)dd) * (float)(sm & 0xffu);
    const float cz = -s16 - half_bits_to_f32((uint16_t)(dd >> 16)) * (float)(sm >> 8);
    const u32 sb = f2h_bits(s16), cb = f2h_bits(cz);
    const u32 s2 = sb | (sb << 16), c2 = cb | (cb << 16);
    wd[0] = deq8_f16(q.x, s2, c2, dqc); wd[1] = deq8_f16(q.y, s2, c2, dqc);
    wd[2] = deq8_f16(q.z, s2, c2, dqc); wd[3] = deq8_f16(q.w, s2, c2, dqc);
  };
  auto step = [&](const int i, const Tiles &cur, Tiles &nxt) {
    const int g0 = step_group(i);
    load_w(i + 1, nxt);
    if (g0 >= G) return;
    const int cb = (i / SPC) & 1;
#pragma unroll
    for (int j = 0; j < WS; ++j) {
      if (g0 + j < G) {  // uniform
        const int gq = kh * GW + (i % SPC) * WS + j;  // group within the chunk
        if constexpr (NT >= 4) {
          f16x8_t wd[NB][4];
#pragma unroll
          for (int n = 0; n < NB; ++n) deq_tile(cur.q[j][n], cur.sm[j][n], cur.dd[j][n], wd[n]);
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const f16x8_t *xp = (const f16x8_t *)(xs + ((size_t)cb * TBK + tokl[t]) * XSC + gq * 256 + qd * 64);
            const f16x8_t x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
#pragma unroll
            for (int n = 0; n < NB; ++n) {
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[n][0], x0, acc[n][t], 0, 0, 0);
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[n][1], x1, acc[n][t], 0, 0, 0);
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[n][2], x2, acc[n][t], 0, 0, 0);
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[n][3], x3, acc[n][t], 0, 0, 0);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        } else {
          f16x8_t xv[NT][4];
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const f16x8_t *xp = (const f16x8_t *)(xs + ((size_t)cb * TBK + tokl[t]) * XSC + gq * 256 + qd * 64);
            xv[t][0] = xp[0]; xv[t][1] = xp[1]; xv[t][2] = xp[2]; xv[t][3] = xp[3];
          }
#pragma unroll
          for (int n = 0; n < NB; ++n) {
            f16x8_t wd[4];
            deq_tile(cur.q[j][n], cur.sm[j][n], cur.dd[j][n], wd);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[0], xv[t][0], acc[n][t], 0, 0, 0);
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[1], xv[t][1], acc[n][t], 0, 0, 0);
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[2], xv[t][2], acc[n][t], 0, 0, 0);
              acc[n][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wd[3], xv[t][3], acc[n][t], 0, 0, 0);
            }
          }
        }
      }
    }
  };

  Tiles wA, wB;
  load_chunk(0);
  load_w(0, wA);
  if constexpr (SPC == 2) {
    for (int ch = 0; ch < NCH; ++ch) {
      chunk_begin(ch);
      step(2 * ch, wA, wB);
      step(2 * ch + 1, wB, wA);
    }
  } else {
    for (int ch = 0; ch < NCH; ch += 2) {
      chunk_begin(ch);
      step(ch, wA, wB);
      if (ch + 1 < NCH) {
        chunk_begin(ch + 1);
        step(ch + 1, wB, wA);
      }
    }
  }
  if constexpr (KS > 1) {
    __syncthreads();
    float *red = (float *)smem;  // [4 waves][NB][NT][4][64 lanes]
    if (kh != 0) {
#pragma unroll
      for (int n = 0; n < NB; ++n)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) red[((w * NB + n) * NT + t) * 256 + i * 64 + lane] = acc[n][t][i];
    }
    __syncthreads();
    if (kh == 0) {
#pragma unroll
      for (int q = 1; q < KS; ++q)
#pragma unroll
        for (int n = 0; n < NB; ++n)
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[n][t][i] += red[(((w + q) * NB + n) * NT + t) * 256 + i * 64 + lane];
    }
  }
  if (kh == 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (16 * t + r < mc) {
        if (SWIGLU) {
          const size_t orow = (size_t)(row_first + 16 * t + r) * c.out_stride;
          u32 h[2];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const float g0 = acc[0][t][2 * i], g1 = acc[0][t][2 * i + 1];
            const float h0 = g0 / (1.f + expf(-g0)) * acc[1][t][2 * i];
            const float h1 = g1 / (1.f + expf(-g1)) * acc[1][t][2 * i + 1];
            h[i] = (u32)f32_to_bf16(h0) | ((u32)f32_to_bf16(h1) << 16);
          }
          *(uint2 *)((uint16_t *)c.out + orow + b * 16 + 4 * qd) = make_uint2(h[0], h[1]);
        } else {
          const size_t orow = (out_row0 + (size_t)(row_first + 16 * t + r)) * c.out_stride;
#pragma unroll
          for (int n = 0; n < NB; ++n)
            *(float4 *)((float *)c.out + orow + (2 * b + n) * 16 + 4 * qd) =
                make_float4(acc[n][t][0], acc[n][t][1], acc[n][t][2], acc[n][t][3]);
        }
      }
    }
  }
}

// The kernel: a workgroup walks the rows of its unit in passes and picks every pass's width by the rows that are
// left: 64 rows (NT = 4, chunks of 2 groups) when more than 32 remain, 32 rows (NT = 2, chunks of 4) when more
// than 16 remain, else 16 rows (chunks of 8), as far as NTMAX allows.  The three shapes stage the same number of
// activation bytes per chunk, so the LDS footprint is that of the 16-row shape.  A unit's weights are streamed and
// dequantised once per pass, so a popular expert (and the shared expert, which sees every token) costs one stream
// where 16-row passes cost up to four.
// q4_K: the shared expert's w2 class may be split (c.ksplit workgroups per group of block pairs, each over 1 / ksplit
// of the reduction, partial rows to their own copy of the output: see k_gemv_int4).
// ROUTE (int4 w13 pass of at most 16 tokens): the launch sums the gate rows and routes by itself, as
// k_gemv_int4_mfma<.., ROUTE> does (see gemv_resolve_route_batch_n)
template <bool SWIGLU, bool DEVUNITS, int NTMAX, int KS, bool Q4K = false, bool ROUTE = false>
__global__ __launch_bounds__(256, 2) void k_gemv_int4_mfma_kc(const GemvArgs a) {
  constexpr int NB = 2;
  static_assert(!ROUTE || (SWIGLU && DEVUNITS && NTMAX == 1 && !Q4K), "routing launches: int4 w13, 16-row passes");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  KC_STAMP(0);

  // a publishing workgroup comes first in the grid: it is over long before the ones that stream weights
  const bool publishes = !ROUTE && SWIGLU && DEVUNITS && a.p_host_units != nullptr;
  if (publishes && blockIdx.x == 0) {
    gemv_publish_units(a);
    return;
  }
  int bx = (int)blockIdx.x - (publishes ? 1 : 0);
  unsigned tokmask = 0u;   // ROUTE: the tokens of a routed unit
  GemvWork wk;
  if constexpr (ROUTE) {
    if (bx < a.g_nblk) {
      if (a.T <= 8) gate_rows_batch_tg<4>(a, lane, w, bx);
      else gate_rows_batch_tg<8>(a, lane, w, bx);
      return;
    }
    bx -= a.g_nblk;
    if (bx == 0) { route_publish_batch(a, smem); return; }
    bx -= 1;
    if (bx < a.n_sh_blocks) {
      wk.c = a.cls[0]; wk.b = bx; wk.half = 0; wk.m = a.T; wk.row0 = 0; wk.base = a.shared_base;
    } else {
      wk = gemv_resolve_route_batch<4>(a, lane, w, bx - a.n_sh_blocks, tokmask);
    }
  } else {
    wk = gemv_resolve<DEVUNITS, (NTMAX > 1)>(a, bx, lane);
  }
  const GemvClass &c = wk.c;
  const int m = wk.m, row0 = wk.row0;
  const unsigned char *base = wk.base;
  KC_STAMPV(5, (unsigned long long)(m + 1));
  if (m <= 0) return;
  if (base == nullptr) {
    if (tid == 0) moe_raise_err(a.err);
    return;
  }
  KC_STAMP(1);
  const int Gt = c.G;
  const int nsp = (Q4K && c.ksplit > 1) ? c.ksplit : 1;
  const int split = nsp > 1 ? wk.b % nsp : 0;
  const int G = Gt / nsp, g0 = split * G;   // this workgroup's window of the reduction
  const int b = (nsp > 1 ? wk.b / nsp : wk.b) * (4 / KS) + w / KS;  // the wave's block pair
  const int rbA = 2 * b;
  constexpr int SCB = Q4K ? 128 : 32, ZZB = Q4K ? 32 : 8;  // bytes of section s / z per tile
  const rsrc_t rq = make_rsrc(base + c.off_q + ((size_t)rbA * Gt + g0) * 1024, (u32)(Gt + G) * 1024u);
  const rsrc_t rs = make_rsrc(base + c.off_s + ((size_t)rbA * Gt + g0) * SCB, (u32)(Gt + G) * SCB);
  const rsrc_t rz = make_rsrc(base + c.off_z + ((size_t)rbA * Gt + g0) * ZZB, (u32)(Gt + G) * ZZB);
  const rsrc_t rx = make_rsrc((const unsigned char *)c.act + (size_t)g0 * 256, KC_NO_ROW);
  const Q4Consts q4c = q4_consts();
  const DeqF16Consts dqc = deq_f16_consts();
  const size_t orow0 = (size_t)split * a.T;

  // rows of this workgroup: all of the unit's, or one half of a unit of more than 32 rows (row_split)
  int r_lo = 0, r_hi = m;
  if (NTMAX > 1 && a.row_split) {
    if (m > 32) { r_lo = wk.half ? 32 : 0; r_hi = wk.half ? m : 32; }
    else if (wk.half) return;
  }
  for (int t0 = r_lo; t0 < r_hi;) {
    const int left = r_hi - t0;
    if (NTMAX >= 4 && left > 32) {
      const int mc = left < 64 ? left : 64;
      if constexpr (Q4K) kc_pass_q4k<SWIGLU, 4, 2, KS>(c, smem, rq, rs, rz, rx, Gt, G, b, orow0, row0 + t0, mc, dqc);
      else kc_pass<SWIGLU, 4, 2, KS>(c, smem, rq, rs, rz, rx, b, row0 + t0, mc, q4c);
      t0 += 64;
    } else if (NTMAX >= 2 && left > 16) {
      const int mc = left < 32 ? left : 32;
      if constexpr (Q4K) kc_pass_q4k<SWIGLU, 2, 4, KS>(c, smem, rq, rs, rz, rx, Gt, G, b, orow0, row0 + t0, mc, dqc);
      else kc_pass<SWIGLU, 2, 4, KS>(c, smem, rq, rs, rz, rx, b, row0 + t0, mc, q4c);
      t0 += 32;
    } else {
      const int mc = left < 16 ? left : 16;
      if constexpr (Q4K) kc_pass_q4k<SWIGLU, 1, 8, KS>(c, smem, rq, rs, rz, rx, Gt, G, b, orow0, row0 + t0, mc, dqc);
      else kc_pass<SWIGLU, 1, 8, KS, ROUTE>(c, smem, rq, rs, rz, rx, b, row0 + t0, mc, q4c, tokmask);
      t0 += 16;
    }
    if (t0 < r_hi) __syncthreads();  // the next pass restages chunk buffer 0
  }
  KC_STAMP(4);
}

// ---------------------------------------------------------------------------
// k5 combine
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_combine(const float *__restrict__ part_r,
                                                  const float *__restrict__ part_s,
                                                  const float *__restrict__ topk_w,
                                                  const int *__restrict__ pos_of_pair,
                                                  const float *__restrict__ sg_logit,
                                                  int sg_stride, uint16_t *__restrict__ y, int H,
                                                  int k, int n_sh_splits) {
  const int t = blockIdx.y;
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (n >= H) return;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  // eight partial rows at a time: positions and weights first, then the rows, then the
  // fma chain in pair order (two round trips per eight rows instead of two per row)
  for (int j0 = 0; j0 < k; j0 += 8) {
    float wj[8];
    int pos[8];
    float4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int jj = j0 + j < k ? j0 + j : k - 1;
      wj[j] = topk_w[(size_t)t * k + jj];
      pos[j] = pos_of_pair[(size_t)t * k + jj];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *(const float4 *)(part_r + (size_t)pos[j] * H + n);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j0 + j < k) {
        acc.x = fmaf(wj[j], v[j].x, acc.x); acc.y = fmaf(wj[j], v[j].y, acc.y);
        acc.z = fmaf(wj[j], v[j].z, acc.z); acc.w = fmaf(wj[j], v[j].w, acc.w);
      }
  }
  if (part_s) {
    const float g = sg_logit ? 1.f / (1.f + expf(-sg_logit[(size_t)t * sg_stride])) : 1.f;
    float4 v = *(const float4 *)(part_s + (size_t)t * H + n);
    // a shared expert whose reduction was split over workgroups: its partial rows, added in split order
    for (int sp = 1; sp < n_sh_splits; ++sp) {
      const float4 u = *(const float4 *)(part_s + ((size_t)sp * gridDim.y + t) * H + n);
      v.x += u.x; v.y += u.y; v.z += u.z; v.w += u.w;
    }
    acc.x = fmaf(g, v.x, acc.x); acc.y = fmaf(g, v.y, acc.y);
    acc.z = fmaf(g, v.z, acc.z); acc.w = fmaf(g, v.w, acc.w);
  }
  uint2 o;
  o.x = (u32)f32_to_bf16(acc.x) | ((u32)f32_to_bf16(acc.y) << 16);
  o.y = (u32)f32_to_bf16(acc.z) | ((u32)f32_to_bf16(acc.w) << 16);
  *(uint2 *)(y + (size_t)t * H + n) = o;
}

// ---------------------------------------------------------------------------
// host launchers (C ABI)
// ---------------------------------------------------------------------------
extern "C" int moe_int4_layout_make(int H, int I, moe_int4_layout *out) {
  if (!out || H <= 0 || I <= 0 || H % 128 || I % 128) {
    moe_set_error("moe_int4_layout_make: H and I must be positive multiples of 128 (H=%d I=%d)", H, I);
    return MOE_EINVAL;
  }
  const int64_t n13 = 2LL * I, g13 = H / 128, n2 = H, g2 = I / 128;
  int64_t o = 0;
  out->off13_q = o; o += n13 * H / 2;
  out->off13_s = o; o += n13 * g13 * 2;
  out->off13_z = o; o += n13 * g13 / 2;
  out->off2_q = o; o += n2 * (int64_t)I / 2;
  out->off2_s = o; o += n2 * g2 * 2;
  out->off2_z = o; o += n2 * g2 / 2;
  out->total_bytes = o;
  return MOE_OK;
}

extern "C" int moe_gate_logits(const void *x, const void *wg, const float *bias, float *logits,
                               int T, int H, int E, int ldl, void *stream) {
  if (!x || !wg || !logits || T < 0 || H <= 0 || H % 8 || E <= 0 || ldl < E || T > 65535) {
    moe_set_error("moe_gate_logits: bad argument (T=%d H=%d E=%d ldl=%d)", T, H, E, ldl);
    return MOE_EINVAL;
  }
  if (T == 0) return MOE_OK;
  // up to 128 tokens a wave per (token, gate row) is faster than the token-tile kernel (8 us against 18 us
  // at 128 tokens, 2048 columns, 64 rows)
  if (T > 128 && H <= 4096) {
    // about two workgroups per compute unit, and at most 72 KB of gate rows per workgroup so that two fit the LDS
    static bool attr_set = false;
    if (!attr_set) {
      for (const void *f : {(const void *)k_gate_logits_rows<2>, (const void *)k_gate_logits_rows<4>,
                            (const void *)k_gate_logits_rows<8>})
        if (int rc = moe_check_hip(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 72 * 1024),
                                   "hipFuncSetAttribute(k_gate_logits_rows)"))
          return rc;
      attr_set = true;
    }
    const int tiles = (T + GATE_TT - 1) / GATE_TT;
    int rows_per_block = E;
    while (rows_per_block > 1 && ((size_t)rows_per_block * H * 2 > 72 * 1024 ||
                                  (size_t)tiles * ((E + rows_per_block - 1) / rows_per_block) < 512))
      rows_per_block = (rows_per_block + 1) / 2;
    const size_t lds = (size_t)rows_per_block * H * 2;
    dim3 grid(tiles, (E + rows_per_block - 1) / rows_per_block);
    moe_ktimer_begin(MOE_K_GATE, (hipStream_t)stream);
    if (H <= 1024)
      hipLaunchKernelGGL(k_gate_logits_rows<2>, grid, dim3(64 * GATE_WAVES), lds, (hipStream_t)stream, (const uint16_t *)x,
                         (const uint16_t *)wg, bias, logits, T, H, E, ldl, rows_per_block);
    else if (H <= 2048)
      hipLaunchKernelGGL(k_gate_logits_rows<4>, grid, dim3(64 * GATE_WAVES), lds, (hipStream_t)stream, (const uint16_t *)x,
                         (const uint16_t *)wg, bias, logits, T, H, E, ldl, rows_per_block);
    else
      hipLaunchKernelGGL(k_gate_logits_rows<8>, grid, dim3(64 * GATE_WAVES), lds, (hipStream_t)stream, (const uint16_t *)x,
                         (const uint16_t *)wg, bias, logits, T, H, E, ldl, rows_per_block);
    moe_ktimer_end(MOE_K_GATE, (hipStream_t)stream);
    return moe_check_launch("k_gate_logits_rows");
  }
  dim3 grid((E + 3) / 4, T);
  moe_ktimer_begin(MOE_K_GATE, (hipStream_t)stream);
  hipLaunchKernelGGL(k_gate_logits, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x,
                     (const uint16_t *)wg, bias, logits, H, E, ldl, (const uint16_t *)nullptr, (const float *)nullptr,
                     (float *)nullptr, 0, 0);
  moe_ktimer_end(MOE_K_GATE, (hipStream_t)stream);
  return moe_check_launch("k_gate_logits");
}

// Two matrices over the same activations in one launch (decode batches, T <= 128): rows of wg into logits, rows
// of wg2 into logits2, each (token, row) sum with the bits of moe_gate_logits.
extern "C" int moe_gate_logits_pair(const void *x, const void *wg, const float *bias, float *logits, int T, int H,
                                    int E, int ldl, const void *wg2, const float *bias2, float *logits2, int E2,
                                    int ldl2, void *stream) {
  if (!x || !wg || !logits || !wg2 || !logits2 || T <= 0 || T > 128 || H <= 0 || H % 8 || E <= 0 || ldl < E ||
      E2 <= 0 || ldl2 < E2) {
    moe_set_error("moe_gate_logits_pair: bad argument (T=%d H=%d E=%d E2=%d)", T, H, E, E2);
    return MOE_EINVAL;
  }
  dim3 grid((E + 3) / 4 + (E2 + 3) / 4, T);
  moe_ktimer_begin(MOE_K_GATE, (hipStream_t)stream);
  hipLaunchKernelGGL(k_gate_logits, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x,
                     (const uint16_t *)wg, bias, logits, H, E, ldl, (const uint16_t *)wg2, bias2, logits2, E2, ldl2);
  moe_ktimer_end(MOE_K_GATE, (hipStream_t)stream);
  return moe_check_launch("k_gate_logits");
}

extern "C" int moe_topk(const float *logits, int T, int E, int ldl, int k, int mode, int *idx,
                        float *w, void *stream) {
  if (!logits || !idx || !w || T < 0 || E <= 0 || E > 256 || k <= 0 || k > 32 || k > E ||
      ldl < E || mode < 0 || mode > 2) {
    moe_set_error("moe_topk: bad argument (T=%d E=%d k=%d mode=%d)", T, E, k, mode);
    return MOE_EINVAL;
  }
  if (T == 0) return MOE_OK;
  moe_ktimer_begin(MOE_K_TOPK, (hipStream_t)stream);
  hipLaunchKernelGGL(k_topk, dim3((T + 3) / 4), dim3(256), 0, (hipStream_t)stream, logits, T, E,
                     ldl, k, mode, idx, w);
  moe_ktimer_end(MOE_K_TOPK, (hipStream_t)stream);
  return moe_check_launch("k_topk");
}

extern "C" int moe_dispatch(const int *idx, int T, int k, int E, int *counts, int *offsets,
                            int *sorted_pair, int *pos_of_pair, int *sorted_tok, moe_unit *units,
                            int *n_active, int64_t *active_ids, int max_units, void *stream) {
  if ((!idx && T > 0) || !counts || !offsets || !sorted_pair || !pos_of_pair || !sorted_tok ||
      !units || !n_active || !active_ids || T < 0 || k <= 0 || E <= 0 || E > DISP_MAXE ||
      max_units < 0) {
    moe_set_error("moe_dispatch: bad argument (T=%d k=%d E=%d)", T, k, E);
    return MOE_EINVAL;
  }
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const size_t lds = (size_t)16 * E * sizeof(int);
  moe_ktimer_begin(MOE_K_DISPATCH, (hipStream_t)stream);
  hipLaunchKernelGGL(k_dispatch, dim3(1), dim3(DISP_THREADS), lds, (hipStream_t)stream, idx,
                     T * k, k, E, nbits, counts, offsets, sorted_pair, pos_of_pair, sorted_tok,
                     units, n_active, (long long *)active_ids, max_units);
  moe_ktimer_end(MOE_K_DISPATCH, (hipStream_t)stream);
  return moe_check_launch("k_dispatch");
}

// Dispatch with a workspace: P = T*k >= 2048 pairs of E <= 256 experts go to k_dispatch_multi (one workgroup per
// 1024 pairs, at most 64), anything else to moe_dispatch.  The workspace starts with the two barrier words, which
// must be zero before the first call and are zero again after every call.
extern "C" int64_t moe_dispatch_workspace_bytes(int T, int k, int E) {
  const long long P = (long long)T * k;
  if (T <= 0 || k <= 0 || E <= 0 || E > 256 || P < 2048 || P > (long long)DISPM_MAXB * DISP_THREADS) return 0;
  const long long nb = (P + DISP_THREADS - 1) / DISP_THREADS;
  return 64 + nb * E * (long long)sizeof(int);
}

extern "C" int moe_dispatch_ws(const int *idx, int T, int k, int E, int *counts, int *offsets,
                               int *sorted_pair, int *pos_of_pair, int *sorted_tok, moe_unit *units,
                               int *n_active, int64_t *active_ids, int max_units, void *ws, int64_t ws_bytes,
                               int *err, void *stream) {
  const int64_t need = moe_dispatch_workspace_bytes(T, k, E);
  if (need == 0 || !ws || ws_bytes < need || !err)
    return moe_dispatch(idx, T, k, E, counts, offsets, sorted_pair, pos_of_pair, sorted_tok, units, n_active,
                        active_ids, max_units, stream);
  if (!idx || !counts || !offsets || !sorted_pair || !pos_of_pair || !sorted_tok || !units || !n_active ||
      !active_ids || max_units < 0 || ((uintptr_t)ws & 3)) {
    moe_set_error("moe_dispatch_ws: bad argument (T=%d k=%d E=%d)", T, k, E);
    return MOE_EINVAL;
  }
  const int P = T * k;
  const int nb = (P + DISP_THREADS - 1) / DISP_THREADS;
  const int chunk = (P + nb - 1) / nb;
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const size_t lds = (size_t)16 * E * sizeof(int);
  moe_ktimer_begin(MOE_K_DISPATCH, (hipStream_t)stream);
  hipLaunchKernelGGL(k_dispatch_multi, dim3(nb), dim3(DISP_THREADS), lds, (hipStream_t)stream, idx, P, chunk, k, E,
                     nbits, counts, offsets, sorted_pair, pos_of_pair, sorted_tok, units, n_active,
                     (long long *)active_ids, max_units, (int *)((char *)ws + 64), (unsigned *)ws, err);
  moe_ktimer_end(MOE_K_DISPATCH, (hipStream_t)stream);
  return moe_check_launch("k_dispatch_multi");
}

template <int TMAX, bool SW, int CH>
static int launch_gemv(const GemvArgs &a, int grid, size_t lds, hipStream_t s) {
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    hipError_t e = hipFuncSetAttribute((const void *)k_gemv_int4<TMAX, SW, CH, true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void *)k_gemv_int4<TMAX, SW, CH, false>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      moe_set_error("hipFuncSetAttribute(max dynamic LDS): %s", hipGetErrorString(e));
      return MOE_EHIP;
    }
    attr_set = true;
  }
  moe_ktimer_begin(SW ? MOE_K_W13 : MOE_K_W2, s);
  if (a.units) hipLaunchKernelGGL((k_gemv_int4<TMAX, SW, CH, true>), dim3(grid), dim3(256), lds, s, a);
  else hipLaunchKernelGGL((k_gemv_int4<TMAX, SW, CH, false>), dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(SW ? MOE_K_W13 : MOE_K_W2, s);
  return moe_check_launch("k_gemv_int4");
}

static size_t gemv_lds(int tmax, int K) {
  const size_t G = K / 128;
  return (size_t)tmax * K * 2 + (size_t)tmax * (K / 32) * 4 + 2 * G * 32 + 2 * G * 8 +
         (size_t)4 * tmax * 2 * 16 * 4;
}

template <bool SW, int CH>
static int launch_gemv_c(const GemvArgs &a, int grid, int tmax, size_t lds, hipStream_t s) {
  switch (tmax) {
    case 1: return launch_gemv<1, SW, CH>(a, grid, lds, s);
    case 2: return launch_gemv<2, SW, CH>(a, grid, lds, s);
    case 4: return launch_gemv<4, SW, CH>(a, grid, lds, s);
    case 8: return launch_gemv<8, SW, CH>(a, grid, lds, s);
    default: return launch_gemv<16, SW, CH>(a, grid, lds, s);
  }
}

static size_t gemv_q4k_lds(int tmax, int K) {
  const size_t G = K / 128;
  return (size_t)tmax * K * 2 + (size_t)tmax * (K / 32) * 4 + 2 * G * 128 + 2 * G * 32 +
         (size_t)4 * tmax * 2 * 16 * 4;
}

template <bool SW, int TMAX>
static int launch_gemv_q4k_t(const GemvArgs &a, int grid, size_t lds, hipStream_t s) {
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    if (int rc = moe_check_hip(hipFuncSetAttribute((const void *)k_gemv_int4<TMAX, SW, 2, true, true>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024),
                               "hipFuncSetAttribute(k_gemv_int4 q4k)"))
      return rc;
    attr_set = true;
  }
  moe_ktimer_begin(SW ? MOE_K_W13 : MOE_K_W2, s);
  hipLaunchKernelGGL((k_gemv_int4<TMAX, SW, 2, true, true>), dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(SW ? MOE_K_W13 : MOE_K_W2, s);
  return moe_check_launch("k_gemv_int4<q4k>");
}

template <bool SW>
static int launch_gemv_q4k(const GemvArgs &a, int grid, int T, int Kmax, hipStream_t s) {
  if (T > 1) {  // matrix-core form, passes of 16, 32 or 64 rows per unit
    if (T > 32) return launch_gemv_mfma_kc<SW, 4, true>(a, grid, s);
    if (T > 16) return launch_gemv_mfma_kc<SW, 2, true>(a, grid, s);
    return launch_gemv_mfma_kc<SW, 1, true>(a, grid, s);
  }
  // rows per pass: the smallest power of two >= T (at most 16) whose activations fit LDS; a unit with more
  // rows than that streams its weights once per pass (three tokens against a 20480-column reduction: two
  // rows per pass, two passes)
  int tmax = 1;
  while (tmax < T && tmax < 16) tmax <<= 1;
  while (tmax > 1 && gemv_q4k_lds(tmax, Kmax) > 150 * 1024) tmax >>= 1;
  const size_t lds = gemv_q4k_lds(tmax, Kmax);
  if (lds > 150 * 1024) { moe_set_error("k_gemv_int4<q4k>: K=%d does not fit LDS", Kmax); return MOE_EINVAL; }
  switch (tmax) {
    case 1: return launch_gemv_q4k_t<SW, 1>(a, grid, lds, s);
    case 2: return launch_gemv_q4k_t<SW, 2>(a, grid, lds, s);
    case 4: return launch_gemv_q4k_t<SW, 4>(a, grid, lds, s);
    case 8: return launch_gemv_q4k_t<SW, 8>(a, grid, lds, s);
    default: return launch_gemv_q4k_t<SW, 16>(a, grid, lds, s);
  }
}

// nb: 16-row blocks per iteration (2, or 4 in the 16-token form)
static size_t gemv_mfma_lds(int tb, int K, int nb) {
  const size_t G = K / 128;
  return (size_t)tb * (K * 2 + 16) + (((size_t)tb * G + 3) & ~(size_t)3) * 4 + nb * G * 128 +
         (size_t)4 * nb * 256 * 4;
}

// Routed block pairs per workgroup of the whole-row matrix-core GEMV and what the shared expert's workgroups take
// (see launch_gemv_mfma)
static void gemv_mfma_rpw(const GemvArgs &a, int units, int *rpw_out, int *rpw_s_out) {
  int rpw = 1;
  while (rpw < 4 && units * a.cls[1].nblk / (rpw * 2) >= 1024 && a.cls[1].nblk % (rpw * 2) == 0) rpw *= 2;
  int rpw_s = 1;
  if (a.n_sh_blocks > 0 && a.cls[0].K <= a.cls[1].K)
    while (rpw_s < rpw && a.cls[0].nblk % (rpw_s * 2) == 0) rpw_s *= 2;
  *rpw_out = rpw; *rpw_s_out = rpw_s;
}

template <bool SW, int CH>
static int launch_gemv_mfma(const GemvArgs &a_in, int grid_in, int tb, size_t lds, hipStream_t s) {
  GemvArgs a = a_in;
  const int units = a.cls[1].nblk > 0 ? (grid_in - a.n_sh_blocks) / a.cls[1].nblk : 0;
  // routed block pairs per workgroup: enough workgroups to fill the chip twice, then fewer, larger ones.
  // The shared expert's workgroups stage every token row.  With a reduction longer than the routed
  // experts' (w2 of a wide shared expert) they are the long ones of the launch and keep one pair each:
  // four pairs each cost the 16-token step of a 2048 x 2816 shared expert about 8 us.  Otherwise they
  // take what the routed ones take (more, smaller workgroups only add staging traffic).
  int rpw, rpw_s;
  gemv_mfma_rpw(a, units, &rpw, &rpw_s);
  if (a.n_sh_blocks > 0) { a.cls[0].nblk /= rpw_s; a.n_sh_blocks /= rpw_s; }
  a.cls[1].nblk /= rpw;
  const int grid = a.n_sh_blocks + units * a.cls[1].nblk + (SW && a.units && a.p_host_units ? 1 : 0);
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    hipError_t e = hipFuncSetAttribute((const void *)k_gemv_int4_mfma<SW, CH, true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void *)k_gemv_int4_mfma<SW, CH, false>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      moe_set_error("hipFuncSetAttribute(max dynamic LDS): %s", hipGetErrorString(e));
      return MOE_EHIP;
    }
    attr_set = true;
  }
  moe_ktimer_begin(SW ? MOE_K_W13 : MOE_K_W2, s);
  if (a.units) hipLaunchKernelGGL((k_gemv_int4_mfma<SW, CH, true>), dim3(grid), dim3(256), lds, s, a, tb, rpw, rpw_s);
  else hipLaunchKernelGGL((k_gemv_int4_mfma<SW, CH, false>), dim3(grid), dim3(256), lds, s, a, tb, rpw, rpw_s);
  moe_ktimer_end(SW ? MOE_K_W13 : MOE_K_W2, s);
  return moe_check_launch("k_gemv_int4_mfma");
}

static size_t gemv_mfma_kc_lds(int nt, int cg) {
  return (size_t)2 * 16 * nt * (cg * 256 + 16) + (size_t)2 * 16 * nt * cg * 4 + (size_t)4 * 2 * cg * 32 * 4;
}

// chunked-K form: a workgroup takes 4 / KS block pairs of a unit (both classes' pair counts are
// multiples of four: I and H are multiples of 128)
template <bool SW, int NTMAX, int KS, bool Q4K = false>
static int launch_gemv_mfma_kc_ks(const GemvArgs &a_in, int grid_in, hipStream_t s) {
  constexpr int PW = 4 / KS;
  GemvArgs a = a_in;
  const int units = a.cls[1].nblk > 0 ? (grid_in - a.n_sh_blocks) / a.cls[1].nblk : 0;
  // q4_K, shared expert's w2 class: nblk counts ksplit workgroups per block pair
  const int nsp = (Q4K && a.n_sh_blocks > 0 && a.cls[0].ksplit > 1) ? a.cls[0].ksplit : 1;
  if ((a.n_sh_blocks > 0 && (a.cls[0].nblk % nsp || (a.cls[0].nblk / nsp) % 4)) || (units > 0 && a.cls[1].nblk % 4)) {
    moe_set_error("k_gemv_int4_mfma_kc: block pairs per unit not a multiple of 4");
    return MOE_EINVAL;
  }
  if (Q4K && ((a.n_sh_blocks > 0 && (a.cls[0].G % (2 * nsp))) || (units > 0 && a.cls[1].G % 2))) {
    moe_set_error("k_gemv_int4_mfma_kc<q4_K>: a reduction window must hold whole 256-wide super-blocks");
    return MOE_EINVAL;
  }
  if (a.n_sh_blocks > 0) { a.cls[0].nblk /= PW; a.n_sh_blocks /= PW; }
  a.cls[1].nblk /= PW;
  a.unit_slots = (NTMAX > 1 && a.units && units <= 64) ? units : 0;
  // w2 pass above 32 tokens: its launch ends with the workgroups of the units that have the most rows (the shared
  // expert's above all: every token's row against the longest reduction), and the chip has room beside them, so
  // those units get a second workgroup per group of block pairs for the rows from 32 on.  At most pairs / 33 units
  // can have more than 32 rows.  The weights of such a unit are streamed twice (few units, from the caches the
  // second time).
  int units_grid = units;
  if (!SW && NTMAX >= 4 && a.unit_slots > 0 && a.pairs > 0 && !a.kunits_dev) {
    a.row_split = 1;
    const int extra = a.pairs / 33 < units ? a.pairs / 33 : units;
    units_grid = units + extra;
    a.n_sh_blocks *= 2;
  } else if (!SW && NTMAX >= 4 && !a.units && !a.kunits_dev && units > 0 && units <= GEMV_MAX_KUNITS) {
    // the same split for units that travel by value: the halves become entries of their own, most rows first
    int heavy = 0;
    for (int u = 0; u < units; ++u) heavy += a.ku[u].m > 32;
    if (units + heavy <= GEMV_MAX_KUNITS) {
      KUnit out[GEMV_MAX_KUNITS];
      int n = 0;
      for (int u = 0; u < units; ++u)
        if (a.ku[u].m > 32) {
          out[n++] = KUnit{a.ku[u].base, 32, a.ku[u].row0};
          out[n++] = KUnit{a.ku[u].base, a.ku[u].m - 32, a.ku[u].row0 + 32};
        }
      for (int u = 0; u < units; ++u)
        if (a.ku[u].m <= 32) out[n++] = a.ku[u];
      for (int u = 0; u < n; ++u) a.ku[u] = out[u];
      a.row_split = 1;
      units_grid = n;
      a.n_sh_blocks *= 2;
    }
  }
  const int grid = a.n_sh_blocks + units_grid * a.cls[1].nblk + (SW && a.units && a.p_host_units ? 1 : 0);
  size_t lds = gemv_mfma_kc_lds(1, 8);  // the widest of the pass shapes the kernel may pick
  if (NTMAX >= 2 && gemv_mfma_kc_lds(2, 4) > lds) lds = gemv_mfma_kc_lds(2, 4);
  if (NTMAX >= 4 && gemv_mfma_kc_lds(4, 2) > lds) lds = gemv_mfma_kc_lds(4, 2);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void *)k_gemv_int4_mfma_kc<SW, true, NTMAX, KS, Q4K>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void *)k_gemv_int4_mfma_kc<SW, false, NTMAX, KS, Q4K>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      moe_set_error("hipFuncSetAttribute(max dynamic LDS): %s", hipGetErrorString(e));
      return MOE_EHIP;
    }
    attr_set = true;
  }
  moe_ktimer_begin(SW ? MOE_K_W13 : MOE_K_W2, s);
  if (a.units) hipLaunchKernelGGL((k_gemv_int4_mfma_kc<SW, true, NTMAX, KS, Q4K>), dim3(grid), dim3(256), lds, s, a);
  else hipLaunchKernelGGL((k_gemv_int4_mfma_kc<SW, false, NTMAX, KS, Q4K>), dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(SW ? MOE_K_W13 : MOE_K_W2, s);
  return moe_check_launch("k_gemv_int4_mfma_kc");
}

// Waves per block pair: two for launches of few block pairs (under 384 workgroups of four pairs with every
// unit slot in use; the unit list is made on the device, the host only knows its capacity), else one.
// Measured: 256 workgroups (4096 x 14336 w2, 8 units) 101 us with one wave per pair, 77 us with two; 484
// workgroups (2048 x 1408 w13, 20 units) 19.5 us against 25.7 us.  Four never paid.
template <bool SW, int NTMAX, bool Q4K = false>
static int launch_gemv_mfma_kc(const GemvArgs &a, int grid, hipStream_t s) {
  if (grid / 4 >= 384) return launch_gemv_mfma_kc_ks<SW, NTMAX, 1, Q4K>(a, grid, s);
  return launch_gemv_mfma_kc_ks<SW, NTMAX, 2, Q4K>(a, grid, s);
}

template <bool SW>
static int launch_gemv_t(const GemvArgs &a, int grid, int T, int Kmax, int G_routed, hipStream_t s) {
  // tiles in flight per wave and block: the routed class's groups per wave, at most 4
  // (a partial last chunk re-reads a tile, so pick the chunk that divides best)
  const int gpw = (G_routed + 3) / 4;
  int ch = gpw >= 4 ? ((gpw % 4 == 0) ? 4 : (gpw % 3 == 0 ? 3 : 4)) : gpw;
  if (ch < 1) ch = 1;
  if (T > 1) {  // matrix-core forms; one token takes the dot2 GEMV below
    // token rows the whole-row form would stage, and whether two of its workgroups then share a CU
    int tb_full = 1;
    while (tb_full < T && tb_full < 16) tb_full <<= 1;
    const bool whole_rows_fit = gemv_mfma_lds(tb_full, Kmax, 2) <= 80 * 1024;
    // chunked-K form: 16 tokens and more, and reductions too long for the whole-row form (measured on
    // the 2048 x 1408 (+ 2816 shared) and 4096 x 14336 shapes; the w2 pass gains from 32-token passes
    // above 48 tokens - at 40 and 48 they tie on the first shape and lose 128 to 85 us on the second -,
    // the w13 pass only under skewed routing)
    if (T >= 16 || !whole_rows_fit) {
      if (T > 32) return launch_gemv_mfma_kc<SW, 4>(a, grid, s);
      if (T > 16) return launch_gemv_mfma_kc<SW, 2>(a, grid, s);
      return launch_gemv_mfma_kc<SW, 1>(a, grid, s);
    }
    int tb = 1;
    while (tb < T && tb < 16) tb <<= 1;
    while (tb > 1 && gemv_mfma_lds(tb, Kmax, 2) > 150 * 1024) tb >>= 1;
    // sixteen token rows that leave room for one workgroup per CU only: eight rows and two workgroups
    // are faster when that fits (units with more than eight tokens take a second pass)
    if (tb == 16 && gemv_mfma_lds(16, Kmax, 2) > 80 * 1024 && gemv_mfma_lds(8, Kmax, 2) <= 80 * 1024) tb = 8;
    const size_t lds = gemv_mfma_lds(tb, Kmax, 2);
    if (lds > 150 * 1024) { moe_set_error("k_gemv_int4_mfma: K=%d does not fit LDS", Kmax); return MOE_EINVAL; }
    switch (ch) {
      case 1: return launch_gemv_mfma<SW, 1>(a, grid, tb, lds, s);
      case 2: return launch_gemv_mfma<SW, 2>(a, grid, tb, lds, s);
      case 3: return launch_gemv_mfma<SW, 3>(a, grid, tb, lds, s);
      default: return launch_gemv_mfma<SW, 4>(a, grid, tb, lds, s);
    }
  }
  // rows per pass: the smallest bucket >= T that fits the LDS budget
  int tmax = 1;
  while (tmax < T && tmax < 16) tmax <<= 1;
  while (tmax > 1 && gemv_lds(tmax, Kmax) > 150 * 1024) tmax >>= 1;
  const size_t lds = gemv_lds(tmax, Kmax);
  if (lds > 150 * 1024) {
    moe_set_error("k_gemv_int4: K=%d does not fit LDS", Kmax);
    return MOE_EINVAL;
  }
  switch (ch) {
    case 1: return launch_gemv_c<SW, 1>(a, grid, tmax, lds, s);
    case 2: return launch_gemv_c<SW, 2>(a, grid, tmax, lds, s);
    case 3: return launch_gemv_c<SW, 3>(a, grid, tmax, lds, s);
    default: return launch_gemv_c<SW, 4>(a, grid, tmax, lds, s);
  }
}

extern "C" int moe_experts_decode_int4(const void *x, int T, int H, int I, int I_sh, int k,
                                       const moe_unit *units, int max_units, const int *sorted_tok,
                                       const uint64_t *expert_ptr, const void *shared_ptr,
                                       void *h_r, void *h_s, float *part_r, float *part_s,
                                       int *err, const moe_unit *units_host,
                                       const uint64_t *expert_ptr_host, int phases, void *stream) {
  return moe_experts_decode_int4_publish(x, T, H, I, I_sh, k, units, max_units, sorted_tok, expert_ptr, shared_ptr, h_r,
                                         h_s, part_r, part_s, err, units_host, expert_ptr_host, phases, nullptr,
                                         nullptr, nullptr, nullptr, 0, stream);
}

// tab_host/tab_E: a host copy of the slot table to put into the arguments of launches that take the device unit list
static int experts_decode_int4_impl(const void *x, int T, int H, int I, int I_sh, int k,
                                    const moe_unit *units, int max_units, const int *sorted_tok,
                                    const uint64_t *expert_ptr, const void *shared_ptr,
                                    void *h_r, void *h_s, float *part_r, float *part_s,
                                    int *err, const moe_unit *units_host,
                                    const uint64_t *expert_ptr_host, int phases,
                                    const int *n_active, moe_unit *units_host_out, int *n_active_host_out,
                                    int *seq_host_out, int seq_value, const uint64_t *tab_host, int tab_E, void *stream);

extern "C" int moe_experts_decode_int4_publish(const void *x, int T, int H, int I, int I_sh, int k,
                                               const moe_unit *units, int max_units, const int *sorted_tok,
                                               const uint64_t *expert_ptr, const void *shared_ptr,
                                               void *h_r, void *h_s, float *part_r, float *part_s,
                                               int *err, const moe_unit *units_host,
                                               const uint64_t *expert_ptr_host, int phases,
                                               const int *n_active, moe_unit *units_host_out, int *n_active_host_out,
                                               int *seq_host_out, int seq_value, void *stream) {
  return experts_decode_int4_impl(x, T, H, I, I_sh, k, units, max_units, sorted_tok, expert_ptr, shared_ptr, h_r, h_s, part_r,
                                  part_s, err, units_host, expert_ptr_host, phases, n_active, units_host_out,
                                  n_active_host_out, seq_host_out, seq_value, nullptr, 0, stream);
}

static int experts_decode_int4_impl(const void *x, int T, int H, int I, int I_sh, int k,
                                    const moe_unit *units, int max_units, const int *sorted_tok,
                                    const uint64_t *expert_ptr, const void *shared_ptr,
                                    void *h_r, void *h_s, float *part_r, float *part_s,
                                    int *err, const moe_unit *units_host,
                                    const uint64_t *expert_ptr_host, int phases,
                                    const int *n_active, moe_unit *units_host_out, int *n_active_host_out,
                                    int *seq_host_out, int seq_value, const uint64_t *tab_host, int tab_E, void *stream) {
  if (units_host_out && (T < 2 || !units || units_host || !n_active || !n_active_host_out || !seq_host_out ||
                         !(phases & 1) || max_units <= 0)) {
    moe_set_error("moe_experts_decode_int4_publish: publishing needs T >= 2, the device unit list, its length and "
                  "the w13 phase (T=%d phases=%d)", T, phases);
    return MOE_EINVAL;
  }
  if (!x || T <= 0 || H <= 0 || H % 128 || I < 0 || I % 128 || I_sh < 0 || I_sh % 128 || !err ||
      (max_units > 0 && ((!units && !units_host) || !sorted_tok || (!expert_ptr && !expert_ptr_host) || !h_r || !part_r || I == 0)) ||
      (shared_ptr && (!h_s || !part_s || I_sh == 0))) {
    moe_set_error("moe_experts_decode_int4: bad argument (T=%d H=%d I=%d I_sh=%d)", T, H, I, I_sh);
    return MOE_EINVAL;
  }
  moe_int4_layout lr, ls;
  memset(&lr, 0, sizeof lr); memset(&ls, 0, sizeof ls);
  if (max_units > 0 && moe_int4_layout_make(H, I, &lr)) return MOE_EINVAL;
  if (shared_ptr && moe_int4_layout_make(H, I_sh, &ls)) return MOE_EINVAL;
  const bool sh = shared_ptr != nullptr;
  hipStream_t s = (hipStream_t)stream;

  GemvArgs a;
  memset(&a, 0, sizeof a);
  a.units = units; a.expert_ptr = (const unsigned long long *)expert_ptr;
  a.shared_base = (const unsigned char *)shared_ptr; a.T = T; a.err = err;
  a.pairs = k > 0 ? T * k : 0;
  if (units && !units_host && tab_host) gemv_set_table(a, expert_ptr, tab_host, tab_E);
  if (units_host && expert_ptr_host && max_units <= GEMV_MAX_KUNITS) {
    a.units = nullptr;
    for (int u = 0; u < max_units; ++u) {
      const moe_unit &h = units_host[u];
      a.ku[u].m = h.m; a.ku[u].row0 = h.row0;
      a.ku[u].base = (h.m > 0 && h.expert >= 0) ? expert_ptr_host[h.expert] : 0;
    }
  }
  if (units_host_out) {
    a.p_host_units = units_host_out; a.p_host_n_active = n_active_host_out; a.p_host_seq = seq_host_out;
    a.p_n_active = n_active; a.p_seq_val = seq_value; a.p_max_units = max_units;
  }
  // pass 1: w13 + SwiGLU
  // one token: every row reads activation row 0 (stride 0), no gather load on the critical path
  a.cls[0] = GemvClass{(const uint16_t *)x, nullptr, h_s, ls.off13_q, ls.off13_s, ls.off13_z,
                       H, H / 128, T == 1 ? 0 : H, I_sh, I_sh / 16, 0};
  a.cls[1] = GemvClass{(const uint16_t *)x, T == 1 ? nullptr : sorted_tok, h_r, lr.off13_q, lr.off13_s,
                       lr.off13_z, H, H / 128, T == 1 ? 0 : H, I, I / 16, 0};
  a.n_sh_blocks = sh ? I_sh / 16 : 0;
  int grid = a.n_sh_blocks + max_units * (I / 16);
  if (grid > 0 && (phases & 1)) {
    int rc = launch_gemv_t<true>(a, grid, T, H, H / 128, s);
    if (rc) return rc;
  }
  // pass 2: w2
  a.cls[0] = GemvClass{(const uint16_t *)h_s, nullptr, part_s, ls.off2_q, ls.off2_s, ls.off2_z,
                       I_sh, I_sh / 128, I_sh, H, H / 32, 0};
  a.cls[1] = GemvClass{(const uint16_t *)h_r, nullptr, part_r, lr.off2_q, lr.off2_s, lr.off2_z,
                       I, I / 128, I, H, H / 32, 0};
  a.n_sh_blocks = sh ? H / 32 : 0;
  grid = a.n_sh_blocks + max_units * (H / 32);
  if (grid > 0 && (phases & 2)) {
    int rc = launch_gemv_t<false>(a, grid, T, I_sh > I ? I_sh : I, (max_units > 0 ? I : I_sh) / 128, s);
    if (rc) return rc;
  }
  return MOE_OK;
}

template <int CH>
static int launch_gemv_mfma_route(const GemvArgs &a_in, int units, int tb, size_t lds, hipStream_t s) {
  GemvArgs a = a_in;
  int rpw, rpw_s;
  gemv_mfma_rpw(a, units, &rpw, &rpw_s);
  if (a.n_sh_blocks > 0) { a.cls[0].nblk /= rpw_s; a.n_sh_blocks /= rpw_s; }
  a.cls[1].nblk /= rpw;
  const int grid = a.g_nblk + 1 + a.n_sh_blocks + units * a.cls[1].nblk;
  {  // workgroups the chip holds at once (four per compute unit by registers), and the gate workgroups' places again
    int per_cu = (int)((160 * 1024) / (lds + 4096));
    per_cu = per_cu > 4 ? 4 : (per_cu < 1 ? 1 : per_cu);
    a.g_cache_from = 256 * per_cu + a.g_nblk;
  }
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    if (int rc = moe_check_hip(hipFuncSetAttribute((const void *)k_gemv_int4_mfma<true, CH, true, true>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024),
                               "hipFuncSetAttribute(k_gemv_int4_mfma, routing)"))
      return rc;
    attr_set = true;
  }
  moe_ktimer_begin(MOE_K_W13, s);
  hipLaunchKernelGGL((k_gemv_int4_mfma<true, CH, true, true>), dim3(grid), dim3(256), lds, s, a, tb, rpw, rpw_s);
  moe_ktimer_end(MOE_K_W13, s);
  return moe_check_launch("k_gemv_int4_mfma<route>");
}

template <int KS>
static int launch_gemv_mfma_kc_route(const GemvArgs &a_in, int units, hipStream_t s) {
  constexpr int PW = 4 / KS;
  GemvArgs a = a_in;
  if ((a.n_sh_blocks > 0 && a.cls[0].nblk % 4) || a.cls[1].nblk % 4) {
    moe_set_error("k_gemv_int4_mfma_kc: block pairs per unit not a multiple of 4");
    return MOE_EINVAL;
  }
  if (a.n_sh_blocks > 0) { a.cls[0].nblk /= PW; a.n_sh_blocks /= PW; }
  a.cls[1].nblk /= PW;
  a.unit_slots = 0;
  const int grid = a.g_nblk + 1 + a.n_sh_blocks + units * a.cls[1].nblk;
  a.g_cache_from = 256 * 2 + a.g_nblk;  // two workgroups per compute unit at a time
  const size_t lds = gemv_mfma_kc_lds(1, 8);
  static_assert(RB_PUBLISH_LDS <= 64 * 1024, "the publishing workgroup's LDS");
  static bool attr_set = false;
  if (!attr_set) {
    // (the kernel also has a few hundred bytes of static LDS: dynamic + static must stay within 160 KB)
    if (int rc = moe_check_hip(hipFuncSetAttribute((const void *)k_gemv_int4_mfma_kc<true, true, 1, KS, false, true>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024),
                               "hipFuncSetAttribute(k_gemv_int4_mfma_kc, routing)"))
      return rc;
    attr_set = true;
  }
  moe_ktimer_begin(MOE_K_W13, s);
  hipLaunchKernelGGL((k_gemv_int4_mfma_kc<true, true, 1, KS, false, true>), dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(MOE_K_W13, s);
  return moe_check_launch("k_gemv_int4_mfma_kc<route>");
}

// whole-row form (up to 8 tokens whose rows leave room for two workgroups per compute unit) or chunked-K form
static bool batch_route_whole_rows(int T, int H) {
  if (T > 8) return false;
  int tb = 1;
  while (tb < T) tb <<= 1;
  return gemv_mfma_lds(tb, H, 2) <= 80 * 1024;
}

// whether moe_decode_batch_int4_gate takes a batch of T tokens of this shape
extern "C" int moe_decode_batch_int4_gate_fits(int T, int E, int k, int H, int I, int I_sh, int n_gate_rows) {
  if (T < 2 || T > RB_MAXT || E <= 0 || E > 256 || k <= 0 || k > 32 || k > E || T * k > ROUTE_MAXP || H <= 0 || H % 128 ||
      I <= 0 || I % 128 || I_sh < 0 || I_sh % 128 || n_gate_rows < E || n_gate_rows > E + 1)
    return 0;
  return 1;
}

extern "C" int moe_decode_batch_int4_gate(const void *x, int T, const void *gate_w, const float *gate_bias,
                                          int n_gate_rows, void *gate_ws, int gate_seq, float *logits, int ldl, int E,
                                          int k, int mode, int H, int I, int I_sh, const uint64_t *expert_ptr,
                                          const uint64_t *expert_ptr_host,
                                          const void *shared_ptr, int *idx, float *w, int *counts, int *offsets,
                                          int *sorted_pair, int *pos_of_pair, int *sorted_tok, moe_unit *units,
                                          int *n_active, int64_t *active_ids, int max_units, void *h_r, void *h_s,
                                          float *part_r, float *part_s, int *err, moe_unit *units_host_out,
                                          int *n_active_host_out, int *seq_host_out, int seq_value, int phases,
                                          void *stream) {
  if (!moe_decode_batch_int4_gate_fits(T, E, k, H, I, I_sh, n_gate_rows)) {
    moe_set_error("moe_decode_batch_int4_gate: shape not taken (T=%d E=%d k=%d H=%d I=%d I_sh=%d rows=%d)", T, E, k, H, I,
                  I_sh, n_gate_rows);
    return MOE_EINVAL;
  }
  const int mu = E < T * k ? E : T * k;
  if (!x || !gate_w || !gate_ws || gate_seq == 0 || !logits || ldl < n_gate_rows || !expert_ptr || !idx || !w || !counts ||
      !offsets || !sorted_pair || !pos_of_pair || !sorted_tok || !units || !n_active || !active_ids || max_units != mu ||
      !h_r || !part_r || !err || mode < 0 || mode > 2 || (shared_ptr && (!h_s || !part_s || I_sh == 0)) ||
      (units_host_out && (!n_active_host_out || !seq_host_out))) {
    moe_set_error("moe_decode_batch_int4_gate: bad argument (T=%d max_units=%d, %d expected)", T, max_units, mu);
    return MOE_EINVAL;
  }
  hipStream_t s = (hipStream_t)stream;
  if (phases & 1) {
    moe_int4_layout lr, ls;
    memset(&lr, 0, sizeof lr); memset(&ls, 0, sizeof ls);
    if (moe_int4_layout_make(H, I, &lr)) return MOE_EINVAL;
    if (shared_ptr && moe_int4_layout_make(H, I_sh, &ls)) return MOE_EINVAL;
    const bool sh = shared_ptr != nullptr;
    GemvArgs a;
    memset(&a, 0, sizeof a);
    gemv_set_table(a, expert_ptr, expert_ptr_host, E);
    a.shared_base = (const unsigned char *)shared_ptr; a.T = T; a.err = err; a.pairs = T * k;
    a.r_E = E; a.r_k = k; a.r_mode = mode; a.r_idx = idx; a.r_w = w; a.r_counts = counts; a.r_offsets = offsets;
    a.r_sorted_pair = sorted_pair; a.r_pos_of_pair = pos_of_pair; a.r_sorted_tok = sorted_tok; a.r_units = units;
    a.r_n_active = n_active; a.r_active_ids = (long long *)active_ids;
    a.r_host_units = units_host_out; a.p_host_n_active = units_host_out ? n_active_host_out : nullptr;
    a.r_host_seq = units_host_out ? seq_host_out : nullptr; a.r_host_seq_val = seq_value; a.p_max_units = max_units;
    a.g_w = (const uint16_t *)gate_w; a.g_bias = gate_bias; a.g_stamp = (unsigned long long *)gate_ws;
    a.g_logits_out = logits; a.g_ldl = ldl; a.g_rows = n_gate_rows; a.g_nbias = gate_bias ? E : 0; a.g_seq = gate_seq;
    a.g_copy_words = T * n_gate_rows > GATE_COPY_WORDS ? T * n_gate_rows : GATE_COPY_WORDS;
    a.cls[0] = GemvClass{(const uint16_t *)x, nullptr, h_s, ls.off13_q, ls.off13_s, ls.off13_z, H, H / 128, H, I_sh, I_sh / 16, 0};
    a.cls[1] = GemvClass{(const uint16_t *)x, nullptr, h_r, lr.off13_q, lr.off13_s, lr.off13_z, H, H / 128, H, I, I / 16, 0};
    a.n_sh_blocks = sh ? I_sh / 16 : 0;
    const bool whole = batch_route_whole_rows(T, H);
    const int tg = !whole ? (T <= 8 ? 4 : 8) : (T <= 4 ? 1 : 2);   // tokens per gate workgroup: what the kernel instantiates
    a.g_parts = GATE_PARTS;
    a.g_nblk = a.g_parts * ((T + tg - 1) / tg) * ((n_gate_rows + 3) / 4);
    int rc;
    if (!whole) {
      rc = (a.n_sh_blocks + max_units * (I / 16)) / 4 >= 384 ? launch_gemv_mfma_kc_route<1>(a, max_units, s)
                                                             : launch_gemv_mfma_kc_route<2>(a, max_units, s);
    } else {
      int tb = 1;
      while (tb < T) tb <<= 1;
      size_t lds = gemv_mfma_lds(tb, H, 2);
      if (lds < RB_PUBLISH_LDS) lds = RB_PUBLISH_LDS;
      const int gpw = (H / 128 + 3) / 4;
      int ch = gpw >= 4 ? ((gpw % 4 == 0) ? 4 : (gpw % 3 == 0 ? 3 : 4)) : gpw;
      if (ch < 1) ch = 1;
      switch (ch) {
        case 1: rc = launch_gemv_mfma_route<1>(a, max_units, tb, lds, s); break;
        case 2: rc = launch_gemv_mfma_route<2>(a, max_units, tb, lds, s); break;
        case 3: rc = launch_gemv_mfma_route<3>(a, max_units, tb, lds, s); break;
        default: rc = launch_gemv_mfma_route<4>(a, max_units, tb, lds, s); break;
      }
    }
    if (rc) return rc;
  }
  if (phases & 2)  // w2 over the unit list the first launch published
    return experts_decode_int4_impl(x, T, H, I, shared_ptr ? I_sh : 0, k, units, max_units, sorted_tok, expert_ptr, shared_ptr,
                                    h_r, h_s, part_r, part_s, err, nullptr, nullptr, 2, nullptr, nullptr, nullptr, nullptr, 0,
                                    expert_ptr_host, E, stream);
  return MOE_OK;
}

extern "C" int moe_decode_token_late_expert_int4(const void *x, int H, int I, uint64_t slot_addr, int pos, void *h_r,
                                                 void *unit_ws, int *err, void *stream) {
  if (!x || !h_r || !unit_ws || !err || !slot_addr || pos < 0 || H <= 0 || H % 128 || I <= 0 || I % 128) {
    moe_set_error("moe_decode_token_late_expert_int4: bad argument (H=%d I=%d pos=%d)", H, I, pos);
    return MOE_EINVAL;
  }
  moe_int4_layout lr;
  if (moe_int4_layout_make(H, I, &lr)) return MOE_EINVAL;
  GemvArgs a;
  memset(&a, 0, sizeof a);
  a.T = 1; a.err = err;
  a.ku[0].base = slot_addr; a.ku[0].m = 1; a.ku[0].row0 = pos;
  a.r_kunits = (KUnit *)unit_ws;
  a.cls[0] = GemvClass{(const uint16_t *)x, nullptr, nullptr, 0, 0, 0, H, H / 128, 0, 0, 0, 0};
  a.cls[1] = GemvClass{(const uint16_t *)x, nullptr, h_r, lr.off13_q, lr.off13_s, lr.off13_z, H, H / 128, 0, I, I / 16, 0};
  a.n_sh_blocks = 0;
  return launch_gemv_t<true>(a, I / 16, 1, H, H / 128, (hipStream_t)stream);
}

template <int CH>
static int launch_gemv_route(const GemvArgs &a, int grid, size_t lds, hipStream_t s) {
  moe_ktimer_begin(MOE_K_W13, s);
  hipLaunchKernelGGL((k_w13_token<CH>), dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(MOE_K_W13, s);
  return moe_check_launch("k_w13_token");
}

// gate_w != NULL: the launch of phase bit 0 computes the gate logits itself (moe_decode_token_int4_gate)
static int decode_token_int4_impl(const void *gate_w, const float *gate_bias, int n_gate_rows, void *gate_ws,
                                  int gate_seq, const void *x, const float *logits, int E, int k, int mode, int H, int I,
                                     int I_sh, const uint64_t *expert_ptr, const uint64_t *expert_ptr_host,
                                     const void *shared_ptr, int *idx,
                                     float *w, int *counts, int *offsets, int *sorted_pair, int *pos_of_pair,
                                     int *sorted_tok, moe_unit *units, int *n_active, int64_t *active_ids,
                                     void *h_r, void *h_s, float *part_r, float *part_s, int *err,
                                     void *unit_ws, moe_unit *units_host_out, int *seq_host_out, int seq_value,
                                     int phases, const float *shared_gate_logit, void *y_bf16, void *stream) {
  if (gate_w && (!gate_ws || n_gate_rows < E || n_gate_rows > E + 1 || n_gate_rows > GATE_COPY_WORDS || !(phases & 1))) {
    moe_set_error("moe_decode_token_int4_gate: needs the gate workspace, E or E + 1 gate rows (%d for E=%d) and "
                  "phase bit 0", n_gate_rows, E);
    return MOE_EINVAL;
  }
  if (!x || !logits || !expert_ptr || !idx || !w || !counts || !offsets || !sorted_pair || !pos_of_pair || !sorted_tok ||
      !units || !n_active || !active_ids || !h_r || !part_r || !err || E <= 0 || E > 256 || k <= 0 || k > 32 || k > E ||
      mode < 0 || mode > 2 || H <= 0 || H % 128 || I <= 0 || I % 128 || I_sh < 0 || I_sh % 128 ||
      (shared_ptr && (!h_s || !part_s || I_sh == 0))) {
    moe_set_error("moe_decode_token_int4: bad argument (E=%d k=%d H=%d I=%d I_sh=%d)", E, k, H, I, I_sh);
    return MOE_EINVAL;
  }
  moe_int4_layout lr, ls;
  memset(&lr, 0, sizeof lr); memset(&ls, 0, sizeof ls);
  if (moe_int4_layout_make(H, I, &lr)) return MOE_EINVAL;
  if (shared_ptr && moe_int4_layout_make(H, I_sh, &ls)) return MOE_EINVAL;
  const bool sh = shared_ptr != nullptr;
  hipStream_t s = (hipStream_t)stream;
  GemvArgs a;
  memset(&a, 0, sizeof a);
  a.units = units; gemv_set_table(a, expert_ptr, expert_ptr_host, E);
  a.shared_base = (const unsigned char *)shared_ptr; a.T = 1; a.err = err;
  a.r_logits = logits; a.r_E = E; a.r_k = k; a.r_mode = mode; a.r_idx = idx; a.r_w = w; a.r_counts = counts;
  a.r_offsets = offsets; a.r_sorted_pair = sorted_pair; a.r_pos_of_pair = pos_of_pair; a.r_sorted_tok = sorted_tok;
  a.r_units = units; a.r_n_active = n_active; a.r_active_ids = (long long *)active_ids;
  a.r_host_units = units_host_out; a.r_host_seq = units_host_out ? seq_host_out : nullptr; a.r_host_seq_val = seq_value;
  a.r_kunits = (KUnit *)unit_ws;
  a.r_unit_w = unit_ws ? (float *)((KUnit *)unit_ws + k) : nullptr;
  // pass 1: w13 + SwiGLU, routing derived in the kernel
  a.cls[0] = GemvClass{(const uint16_t *)x, nullptr, h_s, ls.off13_q, ls.off13_s, ls.off13_z, H, H / 128, 0, I_sh, I_sh / 16, 0};
  a.cls[1] = GemvClass{(const uint16_t *)x, nullptr, h_r, lr.off13_q, lr.off13_s, lr.off13_z, H, H / 128, 0, I, I / 16, 0};
  a.n_sh_blocks = sh ? I_sh / 16 : 0;
  int grid = a.n_sh_blocks + k * (I / 16) + 1;  // + the publishing workgroup
  if (gate_w) {  // + the gate workgroups (a wave per row), in front of all others
    a.g_w = (const uint16_t *)gate_w; a.g_bias = gate_bias; a.g_stamp = (unsigned long long *)gate_ws;
    a.g_logits_out = (float *)logits; a.g_rows = n_gate_rows; a.g_nbias = E; a.g_nblk = GATE_PARTS * ((n_gate_rows + 3) / 4);
    a.g_seq = gate_seq;
    grid += a.g_nblk;
  }
  {
    const int gpw = (H / 128 + 3) / 4;
    int ch = gpw >= 4 ? ((gpw % 4 == 0) ? 4 : (gpw % 3 == 0 ? 3 : 4)) : gpw;
    if (ch < 1) ch = 1;
    const size_t lds = w13_token_lds(ch);
    int rc = MOE_OK;
    if (phases & 1) switch (ch) {
      case 1: rc = launch_gemv_route<1>(a, grid, lds, s); break;
      case 2: rc = launch_gemv_route<2>(a, grid, lds, s); break;
      case 3: rc = launch_gemv_route<3>(a, grid, lds, s); break;
      default: rc = launch_gemv_route<4>(a, grid, lds, s); break;
    }
    if (rc) return rc;
  }
  if (phases & 4) {  // w2 and the combine in one launch, straight into y
    if (!unit_ws || !y_bf16 || (H % 16) || k >= 64) {
      moe_set_error("moe_decode_token_int4: the fused w2 + combine pass needs unit_ws, y and k < 64");
      return MOE_EINVAL;
    }
    W2cArgs c;
    memset(&c, 0, sizeof c);
    c.kunits = (const KUnit *)unit_ws; c.unit_w = (const float *)((const KUnit *)unit_ws + k);
    c.h_r = (const uint16_t *)h_r; c.h_s = (const uint16_t *)h_s; c.shared_base = (const unsigned char *)shared_ptr;
    c.sg_logit = shared_gate_logit;
    c.off_q = lr.off2_q; c.off_s = lr.off2_s; c.off_z = lr.off2_z;
    c.sh_off_q = ls.off2_q; c.sh_off_s = ls.off2_s; c.sh_off_z = ls.off2_z;
    c.k = k; c.I = I; c.I_sh = sh ? I_sh : 0; c.H = H; c.G = I / 128; c.G_sh = sh ? I_sh / 128 : 0;
    c.y = (uint16_t *)y_bf16; c.err = err;
    // two workgroups per 16-row tile (8 rows each): 256 workgroups at H = 2048, one per compute unit; one
    // workgroup per tile took 10.0 us where two take 6.8 us, four no less
    moe_ktimer_begin(MOE_K_W2, s);
    // loads per wave: the (unit, group) items, two per load, over the 16 waves
    const int loads_per_wave = (k * ((c.G + 1) / 2) + (c.G_sh + 1) / 2 + W2C_WAVES - 1) / W2C_WAVES;
    // LDS: per wave the activations and sums of one chunk's items, then the partial sums of the waves
    auto lds = [](int ni, int chunk) { return (size_t)W2C_WAVES * (chunk * ni * 68) * 4 + W2C_WAVES * 16 * 4; };
    if (loads_per_wave <= 3) hipLaunchKernelGGL((k_w2_combine_token<2, 3>), dim3(H / 8), dim3(64 * W2C_WAVES), lds(2, 3), s, c);
    else if (H / 16 >= 256)  // one workgroup per 16-row tile already gives every compute unit one: whole tiles
      hipLaunchKernelGGL((k_w2_combine_token<1, 7>), dim3(H / 16), dim3(64 * W2C_WAVES), lds(1, 7), s, c);
    else hipLaunchKernelGGL((k_w2_combine_token<2, 6>), dim3(H / 8), dim3(64 * W2C_WAVES), lds(2, 6), s, c);
    moe_ktimer_end(MOE_K_W2, s);
    return moe_check_launch("k_w2_combine_token");
  }
  if (!(phases & 2)) return MOE_OK;
  // pass 2: w2 over the unit list the first pass published
  a.cls[0] = GemvClass{(const uint16_t *)h_s, nullptr, part_s, ls.off2_q, ls.off2_s, ls.off2_z, I_sh, I_sh / 128, I_sh, H, H / 32, 0};
  a.cls[1] = GemvClass{(const uint16_t *)h_r, nullptr, part_r, lr.off2_q, lr.off2_s, lr.off2_z, I, I / 128, I, H, H / 32, 0};
  a.n_sh_blocks = sh ? H / 32 : 0;
  a.kunits_dev = (const KUnit *)unit_ws;
  grid = a.n_sh_blocks + k * (H / 32);
  return launch_gemv_t<false>(a, grid, 1, I_sh > I ? I_sh : I, I / 128, s);
}

extern "C" int moe_decode_token_int4(const void *x, const float *logits, int E, int k, int mode, int H, int I,
                                     int I_sh, const uint64_t *expert_ptr, const uint64_t *expert_ptr_host,
                                     const void *shared_ptr, int *idx,
                                     float *w, int *counts, int *offsets, int *sorted_pair, int *pos_of_pair,
                                     int *sorted_tok, moe_unit *units, int *n_active, int64_t *active_ids,
                                     void *h_r, void *h_s, float *part_r, float *part_s, int *err,
                                     void *unit_ws, moe_unit *units_host_out, int *seq_host_out, int seq_value,
                                     int phases, const float *shared_gate_logit, void *y_bf16, void *stream) {
  return decode_token_int4_impl(nullptr, nullptr, 0, nullptr, 0, x, logits, E, k, mode, H, I, I_sh, expert_ptr,
                                expert_ptr_host, shared_ptr,
                                idx, w, counts, offsets, sorted_pair, pos_of_pair, sorted_tok, units, n_active, active_ids,
                                h_r, h_s, part_r, part_s, err, unit_ws, units_host_out, seq_host_out, seq_value, phases,
                                shared_gate_logit, y_bf16, stream);
}

extern "C" int64_t moe_gate_ws_bytes(void) { return (int64_t)GATE_COPIES * GATE_COPY_WORDS * 8; }

extern "C" int moe_decode_token_int4_gate(const void *x, const void *gate_w, const float *gate_bias, int n_gate_rows,
                                          void *gate_ws, int gate_seq, float *logits, int E, int k, int mode, int H,
                                          int I, int I_sh, const uint64_t *expert_ptr, const uint64_t *expert_ptr_host,
                                          const void *shared_ptr, int *idx,
                                          float *w, int *counts, int *offsets, int *sorted_pair, int *pos_of_pair,
                                          int *sorted_tok, moe_unit *units, int *n_active, int64_t *active_ids,
                                          void *h_r, void *h_s, float *part_r, float *part_s, int *err,
                                          void *unit_ws, moe_unit *units_host_out, int *seq_host_out, int seq_value,
                                          int phases, const float *shared_gate_logit, void *y_bf16, void *stream) {
  if (!gate_w) { moe_set_error("moe_decode_token_int4_gate: no gate matrix"); return MOE_EINVAL; }
  return decode_token_int4_impl(gate_w, gate_bias, n_gate_rows, gate_ws, gate_seq, x, logits, E, k, mode, H, I, I_sh,
                                expert_ptr, expert_ptr_host, shared_ptr, idx, w, counts, offsets, sorted_pair, pos_of_pair,
                                sorted_tok, units, n_active, active_ids, h_r, h_s, part_r, part_s, err, unit_ws, units_host_out,
                                seq_host_out, seq_value, phases, shared_gate_logit, y_bf16, stream);
}

// ---------------------------------------------------------------------------
// One token without any allocation: moe_decode_token_int4 with phases = 5 whose workspaces (routing
// arrays, h vectors, resolved units) live in a file-scope device array instead of caller buffers.
// Every GPU holds its own copy of the array at its own address until the process ends.
// ---------------------------------------------------------------------------
#define NOALLOC_MAX_E 256
#define NOALLOC_MAX_K 32
#define NOALLOC_MAX_H_ELEMS 71680   /* k*I + I_sh bf16 values: the room the scratch array has for the h vectors */
struct NoAllocScratch {
  int idx[NOALLOC_MAX_K];
  float w[NOALLOC_MAX_K];
  int counts[NOALLOC_MAX_E];
  int offsets[NOALLOC_MAX_E + 1];
  int sorted_pair[NOALLOC_MAX_K], pos_of_pair[NOALLOC_MAX_K], sorted_tok[NOALLOC_MAX_K];
  int n_active, pad_[2];
  moe_unit units[NOALLOC_MAX_K];
  long long active_ids[NOALLOC_MAX_K];
  unsigned char unit_ws[32 * NOALLOC_MAX_K];
  uint16_t h[NOALLOC_MAX_H_ELEMS];   // h_r [k][I], then h_s [I_sh] at the next 16-byte boundary
};
static __device__ __align__(256) unsigned char scratch[sizeof(NoAllocScratch)];
static_assert(sizeof(NoAllocScratch) <= 160 * 1024, "scratch array grew past its stated maximum");

#define NOALLOC_MAX_DEVICES 64
static NoAllocScratch *g_scratch_dev[NOALLOC_MAX_DEVICES];  // device address of `scratch` per GPU, set once

extern "C" int64_t moe_noalloc_scratch_bytes(void) { return (int64_t)sizeof(NoAllocScratch); }

extern "C" int moe_decode_token_int4_noalloc(const void *x, const float *logits, int E, int k, int mode, int H,
                                             int I, int I_sh, const uint64_t *expert_ptr, const void *shared_ptr,
                                             const float *shared_gate_logit, void *y_bf16, int *err, void *stream) {
  if (!err || !y_bf16) { moe_set_error("moe_decode_token_int4_noalloc: y and err are required"); return MOE_EINVAL; }
  if (E <= 0 || E > NOALLOC_MAX_E || k <= 0 || k > NOALLOC_MAX_K || I <= 0 || I_sh < 0 || I % 128 || I_sh % 128 ||
      (size_t)k * I + (shared_ptr ? I_sh : 0) > NOALLOC_MAX_H_ELEMS) {
    moe_set_error("moe_decode_token_int4_noalloc: shape beyond the static scratch (E=%d <= %d, k=%d <= %d, "
                  "k*I + I_sh = %zu <= %d)", E, NOALLOC_MAX_E, k, NOALLOC_MAX_K,
                  (size_t)k * I + (shared_ptr ? I_sh : 0), NOALLOC_MAX_H_ELEMS);
    return MOE_EINVAL;
  }
  int dev = -1;
  if (int rc = moe_check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) { moe_set_error("moe_decode_token_int4_noalloc: device %d not supported", dev); return MOE_EINVAL; }
  NoAllocScratch *ws = __atomic_load_n(&g_scratch_dev[dev], __ATOMIC_ACQUIRE);
  if (!ws) {
    // the array's name is a host-side stand-in: ask the runtime where this device keeps it
    void *p = nullptr;
    if (int rc = moe_check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
    if (!p) { moe_set_error("moe_decode_token_int4_noalloc: no device address for the scratch array"); return MOE_EHIP; }
    ws = (NoAllocScratch *)p;
    __atomic_store_n(&g_scratch_dev[dev], ws, __ATOMIC_RELEASE);
  }
  uint16_t *h_r = ws->h;
  uint16_t *h_s = ws->h + (((size_t)k * I + 7) & ~(size_t)7);
  // phases 5 never touches the partial-row buffers; the entry point it shares wants them non-null
  float *unused_part = (float *)ws->h;
  return moe_decode_token_int4(x, logits, E, k, mode, H, I, I_sh, expert_ptr, nullptr, shared_ptr, ws->idx, ws->w, ws->counts,
                               ws->offsets, ws->sorted_pair, ws->pos_of_pair, ws->sorted_tok, ws->units, &ws->n_active,
                               (int64_t *)ws->active_ids, h_r, shared_ptr ? h_s : nullptr, unused_part,
                               shared_ptr ? unused_part : nullptr, err, ws->unit_ws, nullptr, nullptr, 0, 5,
                               shared_gate_logit, y_bf16, stream);
}

extern "C" int moe_q4k_layout_make(int H, int I, moe_int4_layout *out) {
  if (!out || H <= 0 || I <= 0 || H % 256 || I % 256) {
    moe_set_error("moe_q4k_layout_make: H and I must be positive multiples of 256 (H=%d I=%d)", H, I);
    return MOE_EINVAL;
  }
  const int64_t n13 = 2ll * I * H, n2 = (int64_t)H * I;
  out->off13_q = 0;
  out->off13_s = out->off13_q + n13 / 2;        // (sc, m) byte pairs: 2 bytes per 32 weights
  out->off13_z = out->off13_s + n13 / 16;       // (d, dmin) fp16 pairs: 4 bytes per 256 weights
  out->off2_q = out->off13_z + n13 / 64;
  out->off2_s = out->off2_q + n2 / 2;
  out->off2_z = out->off2_s + n2 / 16;
  out->total_bytes = out->off2_z + n2 / 64;
  return MOE_OK;
}

// Workgroups per block pair of the shared expert's w2 pass (q4_K decode): with few output rows (H / 32 block
// pairs) and a long reduction every block pair is one long workgroup, and a reduction that does not fit the LDS
// with all token rows costs a pass over the weights per row group.  Splitting the reduction over 2, 4 or 8
// workgroups gives the launch enough of them and keeps every token row of a decode batch in one pass; each
// split writes its own partial rows and the combine adds them in split order.
extern "C" int moe_decode_shared_splits(int fmt, int T, int H, int I_sh) {
  if (fmt != MOE_FMT_Q4K || T <= 0 || H <= 0 || I_sh <= 0 || I_sh % 256) return 1;
  const int pairs = H / 32, G = I_sh / 128;
  int sp = 1;
  // as long as the launch has under 448 shared workgroups and a split keeps at least 16 groups (a whole number
  // of 256-wide super-blocks)
  while (sp < 8 && pairs * sp < 448 && G % (sp * 4) == 0 && G / (sp * 2) >= 16) sp *= 2;
  return sp;
}

extern "C" int moe_experts_decode_q4k(const void *x, int T, int H, int I, int I_sh, int k,
                                      const moe_unit *units, int max_units, const int *sorted_tok,
                                      const uint64_t *expert_ptr, const void *shared_ptr,
                                      void *h_r, void *h_s, float *part_r, float *part_s,
                                      int *err, int phases, void *stream) {
  if (!x || T <= 0 || H <= 0 || H % 256 || I < 0 || I % 256 || I_sh < 0 || I_sh % 256 || !err ||
      (max_units > 0 && (!units || !sorted_tok || !expert_ptr || !h_r || !part_r || I == 0)) ||
      (shared_ptr && (!h_s || !part_s || I_sh == 0))) {
    moe_set_error("moe_experts_decode_q4k: bad argument (T=%d H=%d I=%d I_sh=%d)", T, H, I, I_sh);
    return MOE_EINVAL;
  }
  moe_int4_layout lr, ls;
  memset(&lr, 0, sizeof lr); memset(&ls, 0, sizeof ls);
  if (max_units > 0 && moe_q4k_layout_make(H, I, &lr)) return MOE_EINVAL;
  if (shared_ptr && moe_q4k_layout_make(H, I_sh, &ls)) return MOE_EINVAL;
  const bool sh = shared_ptr != nullptr;
  hipStream_t s = (hipStream_t)stream;
  GemvArgs a;
  memset(&a, 0, sizeof a);
  a.units = units; a.expert_ptr = (const unsigned long long *)expert_ptr;
  a.shared_base = (const unsigned char *)shared_ptr; a.T = T; a.err = err;
  a.pairs = k > 0 ? T * k : 0;
  a.cls[0] = GemvClass{(const uint16_t *)x, nullptr, h_s, ls.off13_q, ls.off13_s, ls.off13_z,
                       H, H / 128, T == 1 ? 0 : H, I_sh, I_sh / 16, 0};
  a.cls[1] = GemvClass{(const uint16_t *)x, T == 1 ? nullptr : sorted_tok, h_r, lr.off13_q, lr.off13_s,
                       lr.off13_z, H, H / 128, T == 1 ? 0 : H, I, I / 16, 0};
  a.n_sh_blocks = sh ? I_sh / 16 : 0;
  int grid = a.n_sh_blocks + max_units * (I / 16);
  if (grid > 0 && (phases & 1))
    if (int rc = launch_gemv_q4k<true>(a, grid, T, H, s)) return rc;
  const int sp = sh ? moe_decode_shared_splits(MOE_FMT_Q4K, T, H, I_sh) : 1;
  a.cls[0] = GemvClass{(const uint16_t *)h_s, nullptr, part_s, ls.off2_q, ls.off2_s, ls.off2_z,
                       I_sh, I_sh / 128, I_sh, H, (H / 32) * sp, sp};
  a.cls[1] = GemvClass{(const uint16_t *)h_r, nullptr, part_r, lr.off2_q, lr.off2_s, lr.off2_z,
                       I, I / 128, I, H, H / 32, 0};
  a.n_sh_blocks = sh ? (H / 32) * sp : 0;
  grid = a.n_sh_blocks + max_units * (H / 32);
  if (grid > 0 && (phases & 2))
    if (int rc = launch_gemv_q4k<false>(a, grid, T, I_sh / sp > I ? I_sh / sp : I, s)) return rc;
  return MOE_OK;
}

extern "C" int moe_route_decode(const void *x, const void *wg, const float *bias, float *logits,
                                int T, int H, int E, int E_rows, int ldl, int k, int mode, int *idx,
                                float *w, int *counts, int *offsets, int *sorted_pair,
                                int *pos_of_pair, int *sorted_tok, moe_unit *units, int *n_active,
                                int64_t *active_ids, int max_units, unsigned *counter, void *stream) {
  if (!x || !wg || !logits || !idx || !w || !counts || !offsets || !sorted_pair || !pos_of_pair ||
      !sorted_tok || !units || !n_active || !active_ids || !counter || T <= 0 || T > 16 || H <= 0 || H % 8 ||
      E <= 0 || E > 256 || E_rows < E || E_rows > E + 1 || ldl < E_rows || k <= 0 || k > 32 || k > E ||
      T * k > ROUTE_MAXP || mode < 0 || mode > 2 || max_units < 0) {
    moe_set_error("moe_route_decode: bad argument (T=%d H=%d E=%d k=%d)", T, H, E, k);
    return MOE_EINVAL;
  }
  RouteArgs a;
  a.x = (const uint16_t *)x; a.wg = (const uint16_t *)wg; a.bias = bias; a.logits = logits;
  a.T = T; a.H = H; a.E = E; a.Erows = E_rows; a.ldl = ldl; a.k = k; a.mode = mode;
  a.nbits = 0;
  while ((1 << a.nbits) < E) ++a.nbits;
  a.max_units = max_units; a.idx = idx; a.w = w; a.counts = counts; a.offsets = offsets;
  a.sorted_pair = sorted_pair; a.pos_of_pair = pos_of_pair; a.sorted_tok = sorted_tok;
  a.units = units; a.n_active = n_active; a.active_ids = (long long *)active_ids;
  a.counter = counter;
  a.host_units = nullptr; a.host_n_active = nullptr; a.host_seq = nullptr; a.host_seq_val = 0; a.pad_ = 0;
  moe_ktimer_begin(MOE_K_GATE, (hipStream_t)stream);
  hipLaunchKernelGGL(k_route_decode, dim3((E_rows + 3) / 4, T), dim3(256), 0, (hipStream_t)stream, a);
  moe_ktimer_end(MOE_K_GATE, (hipStream_t)stream);
  return moe_check_launch("k_route_decode");
}

extern "C" int moe_topk_dispatch(const float *logits, int T, int E, int ldl, int k, int mode, int *idx, float *w,
                                 int *counts, int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok,
                                 moe_unit *units, int *n_active, int64_t *active_ids, int max_units,
                                 moe_unit *units_host_out, int *n_active_host_out, int *seq_host_out, int seq_value,
                                 void *stream) {
  if (!logits || !idx || !w || !counts || !offsets || !sorted_pair || !pos_of_pair || !sorted_tok || !units ||
      !n_active || !active_ids || T <= 0 || T > ROUTE_MAXT || E <= 0 || E > 256 || ldl < E || k <= 0 || k > 32 ||
      k > E || T * k > ROUTE_MAXP || mode < 0 || mode > 2 || max_units < 0 ||
      (units_host_out && (!n_active_host_out || !seq_host_out))) {
    moe_set_error("moe_topk_dispatch: bad argument (T=%d E=%d k=%d)", T, E, k);
    return MOE_EINVAL;
  }
  RouteArgs a;
  memset(&a, 0, sizeof a);
  a.logits = (float *)logits; a.T = T; a.E = E; a.Erows = E; a.ldl = ldl; a.k = k; a.mode = mode;
  while ((1 << a.nbits) < E) ++a.nbits;
  a.max_units = max_units; a.idx = idx; a.w = w; a.counts = counts; a.offsets = offsets;
  a.sorted_pair = sorted_pair; a.pos_of_pair = pos_of_pair; a.sorted_tok = sorted_tok;
  a.units = units; a.n_active = n_active; a.active_ids = (long long *)active_ids;
  a.host_units = units_host_out; a.host_n_active = n_active_host_out; a.host_seq = seq_host_out; a.host_seq_val = seq_value;
  moe_ktimer_begin(MOE_K_TOPK, (hipStream_t)stream);
  if (T <= 4) hipLaunchKernelGGL(k_topk_dispatch<4>, dim3(1), dim3(256), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(k_topk_dispatch<16>, dim3(1), dim3(1024), 0, (hipStream_t)stream, a);
  moe_ktimer_end(MOE_K_TOPK, (hipStream_t)stream);
  return moe_check_launch("k_topk_dispatch");
}

// Bytes of the hand-over area of moe_gate_topk_dispatch for batches of up to T tokens over Erows gate rows
// (zeroed once by the caller; also large enough for moe_decode_token_int4_gate on the same area)
extern "C" int64_t moe_gate_route_ws_bytes(int T, int Erows) {
  if (T < 1 || Erows < 1) return 0;
  const int64_t words = (int64_t)T * Erows > GATE_COPY_WORDS ? (int64_t)T * Erows : GATE_COPY_WORDS;
  // the logit words of every copy, then the unit records of every part (moe_decode_batch_int4_gate)
  return (int64_t)GATE_COPIES * words * 8 + (int64_t)GATE_PARTS * RB_MAX_UNITS * 32;
}

extern "C" int moe_gate_topk_dispatch(const void *x, const void *wg, const float *bias, int n_bias, float *logits, int T,
                                      int H, int E, int Erows, int ldl, int k, int mode, int *idx, float *w, int *counts,
                                      int *offsets, int *sorted_pair, int *pos_of_pair, int *sorted_tok, moe_unit *units,
                                      int *n_active, int64_t *active_ids, int max_units, moe_unit *units_host_out,
                                      int *n_active_host_out, int *seq_host_out, int seq_value, void *gate_ws,
                                      int gate_seq, int parts, int *err, void *stream) {
  if (!x || !wg || !logits || !idx || !w || !counts || !offsets || !sorted_pair || !pos_of_pair || !sorted_tok || !units ||
      !n_active || !active_ids || !gate_ws || !err || T < 2 || T > 32 || H <= 0 || H % 8 || E <= 0 || E > 256 ||
      Erows < E || Erows > E + 1 || ldl < Erows || k <= 0 || k > 32 || k > E || T * k > ROUTE_MAXP || mode < 0 || mode > 2 ||
      max_units < 0 || n_bias < 0 || n_bias > Erows || gate_seq == 0 || (parts != 1 && parts != GATE_PARTS) ||
      (units_host_out && (!n_active_host_out || !seq_host_out))) {
    moe_set_error("moe_gate_topk_dispatch: bad argument (T=%d H=%d E=%d rows=%d k=%d)", T, H, E, Erows, k);
    return MOE_EINVAL;
  }
  RouteArgs a;
  memset(&a, 0, sizeof a);
  a.x = (const uint16_t *)x; a.wg = (const uint16_t *)wg; a.bias = bias; a.n_bias = bias ? n_bias : 0;
  a.logits = logits; a.T = T; a.H = H; a.E = E; a.Erows = Erows; a.ldl = ldl; a.k = k; a.mode = mode;
  while ((1 << a.nbits) < E) ++a.nbits;
  a.max_units = max_units; a.idx = idx; a.w = w; a.counts = counts; a.offsets = offsets;
  a.sorted_pair = sorted_pair; a.pos_of_pair = pos_of_pair; a.sorted_tok = sorted_tok;
  a.units = units; a.n_active = n_active; a.active_ids = (long long *)active_ids;
  a.host_units = units_host_out; a.host_n_active = n_active_host_out; a.host_seq = seq_host_out; a.host_seq_val = seq_value;
  a.g_stamp = (unsigned long long *)gate_ws; a.g_seq = gate_seq; a.err = err;
  a.g_copy_words = T * Erows > GATE_COPY_WORDS ? T * Erows : GATE_COPY_WORDS;
  a.g_parts = parts;
  hipStream_t s = (hipStream_t)stream;
  moe_ktimer_begin(MOE_K_TOPK, s);
  if (T <= 4) {
    const int items = T * ((Erows + 3) / 4);
    hipLaunchKernelGGL(k_gate_route<4>, dim3(1 + parts * items), dim3(256), 0, s, a);
  } else {
    const int items = T * ((Erows + 15) / 16);
    hipLaunchKernelGGL(k_gate_route<16>, dim3(1 + parts * items), dim3(1024), 0, s, a);
  }
  moe_ktimer_end(MOE_K_TOPK, s);
  return moe_check_launch("k_gate_route");
}

extern "C" int moe_combine_splits(const float *part_r, const float *part_s, const float *topk_w,
                                  const int *pos_of_pair, const float *sg_logit, int sg_stride, void *y,
                                  int T, int H, int k, int n_shared_splits, void *stream) {
  if (!y || T < 0 || H <= 0 || H % 4 || k < 0 || (k > 0 && (!part_r || !topk_w || !pos_of_pair)) ||
      T > 65535 || n_shared_splits < 1 || n_shared_splits > 8) {
    moe_set_error("moe_combine: bad argument (T=%d H=%d k=%d splits=%d)", T, H, k, n_shared_splits);
    return MOE_EINVAL;
  }
  if (T == 0) return MOE_OK;
  dim3 grid((H / 4 + 255) / 256, T);
  moe_ktimer_begin(MOE_K_COMBINE, (hipStream_t)stream);
  hipLaunchKernelGGL(k_combine, grid, dim3(256), 0, (hipStream_t)stream, part_r, part_s, topk_w,
                     pos_of_pair, sg_logit, sg_stride, (uint16_t *)y, H, k, n_shared_splits);
  moe_ktimer_end(MOE_K_COMBINE, (hipStream_t)stream);
  return moe_check_launch("k_combine");
}

extern "C" int moe_combine(const float *part_r, const float *part_s, const float *topk_w,
                           const int *pos_of_pair, const float *sg_logit, int sg_stride, void *y,
                           int T, int H, int k, void *stream) {
  return moe_combine_splits(part_r, part_s, topk_w, pos_of_pair, sg_logit, sg_stride, y, T, H, k, 1, stream);
}
