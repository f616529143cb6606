// MoE-layer kernels for gfx950 (MI355X): gating, top-k, stable dispatch,
// int4-group-dequant SwiGLU GEMV through the expert slot table, combine.
// wave64 throughout; no other target is supported.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "moe_kernels.h"
#include "moe_common.h"

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32;

// ---------------------------------------------------------------------------
// small device helpers
// ---------------------------------------------------------------------------
static __device__ __forceinline__ float bf16lo(u32 v) { return __uint_as_float(v << 16); }
static __device__ __forceinline__ float bf16hi(u32 v) { return __uint_as_float(v & 0xffff0000u); }
static __device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even
  u32 u = __float_as_uint(f);
  u32 r = ((u >> 16) & 1u) + 0x7fffu;
  return (uint16_t)((u + r) >> 16);
}
static __device__ __forceinline__ float dot2bf(u32 a, u32 b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                         __builtin_bit_cast(bf16x2_t, b), c, false);
}
static __device__ __forceinline__ float half_bits_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
// 8 int4 weights (interleaved nibble order) x 8 bf16 activations; the weights
// enter as the exact bf16 values 128+q (0x4300 | q), the caller removes 128*sum(x).
static __device__ __forceinline__ float dot8_q4(u32 w, const uint4 &x, float acc) {
  const u32 M = 0x000f000fu, C = 0x43004300u;
  acc = dot2bf((w & M) | C, x.x, acc);
  acc = dot2bf(((w >> 4) & M) | C, x.y, acc);
  acc = dot2bf(((w >> 8) & M) | C, x.z, acc);
  acc = dot2bf(((w >> 12) & M) | C, x.w, acc);
  return acc;
}

// ---------------------------------------------------------------------------
// k1a gate logits: one wave per (token, expert row)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_gate_logits(const uint16_t *__restrict__ x,
                                                      const uint16_t *__restrict__ wg,
                                                      const float *__restrict__ bias,
                                                      float *__restrict__ logits, int H, int E,
                                                      int ldl) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int e = blockIdx.x * 4 + w, t = blockIdx.y;
  if (e >= E) return;
  const uint16_t *xr = x + (size_t)t * H;
  const uint16_t *wr = wg + (size_t)e * H;
  float acc = 0.f;
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
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc = acc + __shfl_xor(acc, m, 64);
  if (lane == 0) logits[(size_t)t * ldl + e] = bias ? acc + bias[e] : acc;
}

// ---------------------------------------------------------------------------
// k1b top-k: one wave per token, E <= 256
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_topk(const float *__restrict__ logits, int T, int E,
                                               int ldl, int k, int mode, int *__restrict__ idx,
                                               float *__restrict__ wout) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + w;
  if (t >= T) return;
  const float NEG = -__builtin_inff();
  float v[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int e = lane + 64 * r;
    v[r] = (e < E) ? logits[(size_t)t * ldl + e] : NEG;
  }
  // row max (== first selected value) and softmax denominator over all E
  float mx = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  float den = 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (lane + 64 * r < E) den += expf(v[r] - mx);
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) den = den + __shfl_xor(den, m, 64);

  float sel_v = 0.f;  // lane j keeps the j-th selected logit
  float sum_sel = 0.f;
  for (int j = 0; j < k; ++j) {
    // local best, ties to the lower index
    float bv = v[0];
    int bi = lane;
#pragma unroll
    for (int r = 1; r < 4; ++r) {
      if (v[r] > bv) { bv = v[r]; bi = lane + 64 * r; }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const float ov = __shfl_xor(bv, m, 64);
      const int oi = __shfl_xor(bi, m, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (bi == lane + 64 * r) v[r] = NEG;
    if (lane == j) sel_v = bv;
    if (lane == 0) idx[(size_t)t * k + j] = bi;
    sum_sel += expf(bv - mx);
  }
  // weights
  const float ex = expf(sel_v - mx);
  float wgt;
  if (mode == MOE_ROUTE_TOPK_SOFTMAX) {
    wgt = ex / sum_sel;
  } else {
    wgt = ex / den;
    if (mode == MOE_ROUTE_SOFTMAX_TOPK_RENORM) wgt = wgt / (sum_sel / den);
  }
  if (lane < k) wout[(size_t)t * k + lane] = wgt;
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
// k3 int4 grouped GEMV (decode).  One workgroup (4 waves) owns two adjacent
// 16-row blocks of one unit's matrix; the waves split the K groups.
//   SWIGLU: blocks are (gate rows, up rows) -> out = silu(g)*u, bf16, 16 values
//   else  : plain product, fp32, 32 values
// ---------------------------------------------------------------------------
struct GemvClass {
  const uint16_t *act;  // bf16 activations [rows, act_stride]
  const int *gather;    // row -> activation row (NULL = identity)
  void *out;            // bf16 (SWIGLU) or fp32
  long long off_q, off_s, off_z;
  int K, G, act_stride, out_stride, nblk;
};
struct GemvArgs {
  GemvClass cls[2];  // 0 = shared expert, 1 = routed experts
  const moe_unit *units;
  const unsigned long long *expert_ptr;
  const unsigned char *shared_base;
  int n_sh_blocks, T;
  int *err;
};

template <int TMAX, bool SWIGLU>
__global__ __launch_bounds__(256) void k_gemv_int4(const GemvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r = lane & 15, qd = lane >> 4;

  int ci, b, m, row0;
  const unsigned char *base;
  if ((int)blockIdx.x < a.n_sh_blocks) {
    ci = 0; b = blockIdx.x; m = a.T; row0 = 0; base = a.shared_base;
  } else {
    ci = 1;
    const int rr = blockIdx.x - a.n_sh_blocks;
    const int u = rr / a.cls[1].nblk;
    b = rr - u * a.cls[1].nblk;
    const moe_unit ud = a.units[u];
    m = ud.m; row0 = ud.row0;
    if (m <= 0) return;
    base = (const unsigned char *)a.expert_ptr[ud.expert];
    if (base == nullptr) {
      if (tid == 0) atomicOr(a.err, 1);
      return;
    }
  }
  const GemvClass &c = a.cls[ci];
  const int K = c.K, G = c.G, KS = K >> 5;
  uint16_t *xs = (uint16_t *)smem;                                // [TMAX][K]
  float *xsum = (float *)(smem + (size_t)TMAX * K * 2);          // [TMAX][K/32]
  float *red = xsum + (size_t)TMAX * KS;                          // [4][TMAX][2][16]

  const int g0 = (w * G) >> 2, g1 = ((w + 1) * G) >> 2;
  const int rbA = 2 * b, rbB = 2 * b + 1;
  const uint4 *qA = (const uint4 *)(base + c.off_q) + (size_t)rbA * G * 64 + lane;
  const uint4 *qB = (const uint4 *)(base + c.off_q) + (size_t)rbB * G * 64 + lane;
  const uint16_t *sA = (const uint16_t *)(base + c.off_s) + (size_t)rbA * G * 16 + r;
  const uint16_t *sB = (const uint16_t *)(base + c.off_s) + (size_t)rbB * G * 16 + r;
  const unsigned char *zA = base + c.off_z + (size_t)rbA * G * 8 + (r >> 1);
  const unsigned char *zB = base + c.off_z + (size_t)rbB * G * 8 + (r >> 1);
  const int zsh = (r & 1) * 4;

  constexpr int CH = 4;
  uint4 wa[CH], wb[CH];
  uint16_t sa[CH], sb[CH];
  unsigned char za[CH], zb[CH];
  auto load_chunk = [&](int gc) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int g = gc + i;
      if (g < g1) {
        wa[i] = qA[(size_t)g * 64];
        wb[i] = qB[(size_t)g * 64];
        sa[i] = sA[g * 16];
        sb[i] = sB[g * 16];
        za[i] = zA[g * 8];
        zb[i] = zB[g * 8];
      }
    }
  };

  for (int t0 = 0; t0 < m; t0 += TMAX) {
    const int mc = (m - t0) < TMAX ? (m - t0) : TMAX;
    load_chunk(g0);  // weights in flight while the activations are staged
    // stage activations
    const int vec_per_row = K >> 3;
    for (int i = tid; i < mc * vec_per_row; i += 256) {
      const int t = i / vec_per_row, v = i - t * vec_per_row;
      const int row = row0 + t0 + t;
      const int arow = c.gather ? c.gather[row] : row;
      ((uint4 *)xs)[(size_t)t * vec_per_row + v] =
          ((const uint4 *)(c.act + (size_t)arow * c.act_stride))[v];
    }
    __syncthreads();
    for (int i = tid; i < mc * KS; i += 256) {
      const int t = i / KS, s = i - t * KS;
      const uint4 *p = (const uint4 *)(xs + (size_t)t * K + s * 32);
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4 v = p[j];
        acc += bf16lo(v.x); acc += bf16hi(v.x); acc += bf16lo(v.y); acc += bf16hi(v.y);
        acc += bf16lo(v.z); acc += bf16hi(v.z); acc += bf16lo(v.w); acc += bf16hi(v.w);
      }
      xsum[i] = acc;
    }
    __syncthreads();

    float accA[TMAX], accB[TMAX];
#pragma unroll
    for (int t = 0; t < TMAX; ++t) { accA[t] = 0.f; accB[t] = 0.f; }

    for (int gc = g0; gc < g1; gc += CH) {
      uint4 ca[CH], cb[CH];
      float fsa[CH], fsb[CH], fza[CH], fzb[CH];
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        ca[i] = wa[i]; cb[i] = wb[i];
        fsa[i] = half_bits_to_f32(sa[i]); fsb[i] = half_bits_to_f32(sb[i]);
        fza[i] = 128.f + (float)((za[i] >> zsh) & 15);
        fzb[i] = 128.f + (float)((zb[i] >> zsh) & 15);
      }
      if (gc + CH < g1) load_chunk(gc + CH);
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int g = gc + i;
        if (g < g1) {
#pragma unroll
          for (int t = 0; t < TMAX; ++t) {
            if (t < mc) {
              const uint4 *xp = (const uint4 *)(xs + (size_t)t * K + g * 128 + qd * 32);
              const uint4 x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
              const float xq = xsum[t * KS + g * 4 + qd];
              float dA = dot8_q4(ca[i].x, x0, 0.f);
              float dB = dot8_q4(cb[i].x, x0, 0.f);
              dA = dot8_q4(ca[i].y, x1, dA); dB = dot8_q4(cb[i].y, x1, dB);
              dA = dot8_q4(ca[i].z, x2, dA); dB = dot8_q4(cb[i].z, x2, dB);
              dA = dot8_q4(ca[i].w, x3, dA); dB = dot8_q4(cb[i].w, x3, dB);
              accA[t] = fmaf(fsa[i], dA - fza[i] * xq, accA[t]);
              accB[t] = fmaf(fsb[i], dB - fzb[i] * xq, accB[t]);
            }
          }
        }
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
        const int t = i >> 4, rr = i & 15;
        float ga = 0.f, up = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) {
          ga += red[((ww * TMAX + t) * 2 + 0) * 16 + rr];
          up += red[((ww * TMAX + t) * 2 + 1) * 16 + rr];
        }
        const float hv = ga / (1.f + expf(-ga)) * up;
        ((uint16_t *)c.out)[(size_t)(row0 + t0 + t) * c.out_stride + b * 16 + rr] = f32_to_bf16(hv);
      }
    } else {
      for (int i = tid; i < mc * 32; i += 256) {
        const int t = i >> 5, ab = (i >> 4) & 1, rr = i & 15;
        float v = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) v += red[((ww * TMAX + t) * 2 + ab) * 16 + rr];
        ((float *)c.out)[(size_t)(row0 + t0 + t) * c.out_stride + (2 * b + ab) * 16 + rr] = v;
      }
    }
    __syncthreads();
  }
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
                                                  int k) {
  const int t = blockIdx.y;
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (n >= H) return;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int j = 0; j < k; ++j) {
    const float wj = topk_w[(size_t)t * k + j];
    const int pos = pos_of_pair[(size_t)t * k + j];
    const float4 v = *(const float4 *)(part_r + (size_t)pos * H + n);
    acc.x = fmaf(wj, v.x, acc.x); acc.y = fmaf(wj, v.y, acc.y);
    acc.z = fmaf(wj, v.z, acc.z); acc.w = fmaf(wj, v.w, acc.w);
  }
  if (part_s) {
    const float g = sg_logit ? 1.f / (1.f + expf(-sg_logit[(size_t)t * sg_stride])) : 1.f;
    const float4 v = *(const float4 *)(part_s + (size_t)t * H + n);
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
  dim3 grid((E + 3) / 4, T);
  moe_ktimer_begin(MOE_K_GATE, (hipStream_t)stream);
  hipLaunchKernelGGL(k_gate_logits, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x,
                     (const uint16_t *)wg, bias, logits, H, E, ldl);
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

template <int TMAX, bool SW>
static int launch_gemv(const GemvArgs &a, int grid, size_t lds, hipStream_t s) {
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    hipError_t e = hipFuncSetAttribute((const void *)k_gemv_int4<TMAX, SW>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      moe_set_error("hipFuncSetAttribute(max dynamic LDS): %s", hipGetErrorString(e));
      return MOE_EHIP;
    }
    attr_set = true;
  }
  moe_ktimer_begin(SW ? MOE_K_W13 : MOE_K_W2, s);
  hipLaunchKernelGGL((k_gemv_int4<TMAX, SW>), dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(SW ? MOE_K_W13 : MOE_K_W2, s);
  return moe_check_launch("k_gemv_int4");
}

static size_t gemv_lds(int tmax, int K) {
  return (size_t)tmax * K * 2 + (size_t)tmax * (K / 32) * 4 + (size_t)4 * tmax * 2 * 16 * 4;
}

template <bool SW>
static int launch_gemv_t(const GemvArgs &a, int grid, int T, int Kmax, hipStream_t s) {
  // rows per pass: the smallest bucket >= T that fits the LDS budget
  int tmax = 1;
  while (tmax < T && tmax < 16) tmax <<= 1;
  while (tmax > 1 && gemv_lds(tmax, Kmax) > 150 * 1024) tmax >>= 1;
  const size_t lds = gemv_lds(tmax, Kmax);
  if (lds > 150 * 1024) {
    moe_set_error("k_gemv_int4: K=%d does not fit LDS", Kmax);
    return MOE_EINVAL;
  }
  switch (tmax) {
    case 1: return launch_gemv<1, SW>(a, grid, lds, s);
    case 2: return launch_gemv<2, SW>(a, grid, lds, s);
    case 4: return launch_gemv<4, SW>(a, grid, lds, s);
    case 8: return launch_gemv<8, SW>(a, grid, lds, s);
    default: return launch_gemv<16, SW>(a, grid, lds, s);
  }
}

extern "C" int moe_experts_decode_int4(const void *x, int T, int H, int I, int I_sh, int k,
                                       const moe_unit *units, int max_units, const int *sorted_tok,
                                       const uint64_t *expert_ptr, const void *shared_ptr,
                                       void *h_r, void *h_s, float *part_r, float *part_s,
                                       int *err, void *stream) {
  if (!x || T <= 0 || H <= 0 || H % 128 || I < 0 || I % 128 || I_sh < 0 || I_sh % 128 || !err ||
      (max_units > 0 && (!units || !sorted_tok || !expert_ptr || !h_r || !part_r || I == 0)) ||
      (shared_ptr && (!h_s || !part_s || I_sh == 0))) {
    moe_set_error("moe_experts_decode_int4: bad argument (T=%d H=%d I=%d I_sh=%d)", T, H, I, I_sh);
    return MOE_EINVAL;
  }
  (void)k;
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
  // pass 1: w13 + SwiGLU
  a.cls[0] = GemvClass{(const uint16_t *)x, nullptr, h_s, ls.off13_q, ls.off13_s, ls.off13_z,
                       H, H / 128, H, I_sh, I_sh / 16};
  a.cls[1] = GemvClass{(const uint16_t *)x, sorted_tok, h_r, lr.off13_q, lr.off13_s, lr.off13_z,
                       H, H / 128, H, I, I / 16};
  a.n_sh_blocks = sh ? I_sh / 16 : 0;
  int grid = a.n_sh_blocks + max_units * (I / 16);
  if (grid > 0) {
    int rc = launch_gemv_t<true>(a, grid, T, H, s);
    if (rc) return rc;
  }
  // pass 2: w2
  a.cls[0] = GemvClass{(const uint16_t *)h_s, nullptr, part_s, ls.off2_q, ls.off2_s, ls.off2_z,
                       I_sh, I_sh / 128, I_sh, H, H / 32};
  a.cls[1] = GemvClass{(const uint16_t *)h_r, nullptr, part_r, lr.off2_q, lr.off2_s, lr.off2_z,
                       I, I / 128, I, H, H / 32};
  a.n_sh_blocks = sh ? H / 32 : 0;
  grid = a.n_sh_blocks + max_units * (H / 32);
  if (grid > 0) {
    int rc = launch_gemv_t<false>(a, grid, T, I_sh > I ? I_sh : I, s);
    if (rc) return rc;
  }
  return MOE_OK;
}

extern "C" int moe_combine(const float *part_r, const float *part_s, const float *topk_w,
                           const int *pos_of_pair, const float *sg_logit, int sg_stride, void *y,
                           int T, int H, int k, void *stream) {
  if (!y || T < 0 || H <= 0 || H % 4 || k < 0 || (k > 0 && (!part_r || !topk_w || !pos_of_pair)) ||
      T > 65535) {
    moe_set_error("moe_combine: bad argument (T=%d H=%d k=%d)", T, H, k);
    return MOE_EINVAL;
  }
  if (T == 0) return MOE_OK;
  dim3 grid((H / 4 + 255) / 256, T);
  moe_ktimer_begin(MOE_K_COMBINE, (hipStream_t)stream);
  hipLaunchKernelGGL(k_combine, grid, dim3(256), 0, (hipStream_t)stream, part_r, part_s, topk_w,
                     pos_of_pair, sg_logit, sg_stride, (uint16_t *)y, H, k);
  moe_ktimer_end(MOE_K_COMBINE, (hipStream_t)stream);
  return moe_check_launch("k_combine");
}
