// Prefill-sized expert groups on the matrix cores (gfx950): grouped GEMM over the
// tokens dispatched to each expert, bf16 operands, fp32 accumulation.
//
//   w13 pass: h[rows, I]   = silu(A Wg^T) * (A Wu^T)     A = gathered activations
//   w2  pass: part[rows,H] = h W2^T
//
// Workgroup = 512 threads (8 waves) -> a tile of up to 256 rows x (128+128) columns: for
// w13 the two column halves are the SAME columns of gate and up (SwiGLU fused in the
// epilogue), for w2 they are adjacent column blocks.  K advances 64 at a time; the
// activation slab goes global -> registers -> double-buffered LDS, the weight fragments go
// global -> registers in operand order and feed v_mfma_f32_32x32x16_bf16 directly.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

#include "moe_common.h"
#include "moe_kernels.h"

typedef unsigned int u32;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const u32x4_t g_uint4;

#define PF_BM 256     // most rows of one tile (8 blocks of 32)
#define PF_BM_SHARED 256     // rows per tile of the dense shared expert in the w13 pass
#define PF_BM_SHARED_W2 128  // and in its w2 pass, which has few column tiles (H/256) and a long K
#define PF_BNH 128   // columns per half
#define PF_BK 64
#define PF_LDK 72    // LDS row stride in bf16 (64 + 8 pad = 144 bytes: conflict-free b128 reads)

struct PfTile {
  unsigned long long w_base;  // expert image base (device address)
  int row0;                   // first row (sorted pair order / token order for the shared expert)
  int rows;                   // valid rows in this tile (<= PF_BM)
};
// one GEMM problem class of a launch (routed experts / shared expert)
struct PfClass {
  const uint16_t *act;  // bf16 activations
  const int *gather;    // row -> activation row, or NULL
  void *out;            // bf16 h (SWIGLU) or fp32 partial rows
  const PfTile *tiles;
  const int *n_tiles_real;  // device: tiles actually in use (<= n_mtiles, the launch's upper bound)
  long long w_off;      // byte offset of the matrix inside the expert image
  long long half_delta; // weight-row offset of the second column half relative to the first
  int act_stride, out_stride, K, n_ntiles, n_mtiles, n_cols_per_tile;
  int m_fastest;        // block order inside the class
  int slab_step;        // storage rotation per 128-row group: smallest odd s >= 3 coprime with K/64
  int n_blocks;         // n_mtiles * n_ntiles
};
struct PfArgs {
  PfClass c[2];
  int n_blocks_total;  // blocks of c[0] come first
};

static __device__ __forceinline__ uint16_t pf_f32_to_bf16(float f) {
  u32 u = __float_as_uint(f);
  u32 r = ((u >> 16) & 1u) + 0x7fffu;
  return (uint16_t)((u + r) >> 16);
}

// Main loop of one wave.  The workgroup has 8 waves: wave w = 0..3 of group g = 0..1 owns
// columns 32w..32w+31 of both column halves and the 32-row blocks g, g+2, g+4, g+6 of the
// tile (NBW of them are live), 128 accumulator registers; the two waves that share a SIMD
// (same w) fill each other's stalls.  The weight operand never touches LDS: a wave loads its
// fragments straight from global memory, where they lie in operand order (blocks of 32 rows
// x 64 k, one contiguous KiB per MFMA step); the second group's loads of the same fragments
// hit in the CU's vector L1.  Within a 64-wide K slab lane half q = lane/32 takes
// k = 32q + 8j + 0..7 for MFMA j: both operands use the same permutation of k, which a dot
// product allows.
template <int NBW>
static __device__ __forceinline__ void pf_mainloop(f32x16_t (&acc)[4][2], uint16_t *As, const uint16_t *const (&a_ptr)[4],
                                                   const uint16_t *b0p, const uint16_t *b1p, int nk, int rot0, int rot1, int nb, int tid) {
  const int lane = tid & 63, g = tid >> 8;
  const int kc = tid & 7, r0 = tid >> 3;  // staging: row r0 + 64 i (block 2i + g), 16-byte chunk kc
  const int fr = lane & 31, q = lane >> 5;
  u32x4_t ra[4], bufA[2][4], bufB[2][4];
  auto gloadA = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (2 * i + g < nb) ra[i] = *(g_uint4 *)(a_ptr[i] + kt * PF_BK);
  };
  auto gloadB = [&](u32x4_t(&b)[2][4], int kt) {
    int k0 = kt + rot0, k1 = kt + rot1;  // slab position inside the 128-row group's storage
    k0 = k0 >= nk ? k0 - nk : k0;
    k1 = k1 >= nk ? k1 - nk : k1;
#pragma unroll
    for (int j = 0; j < 4; ++j) b[0][j] = *(g_uint4 *)(b0p + (size_t)k0 * 8192 + 512 * j);
#pragma unroll
    for (int j = 0; j < 4; ++j) b[1][j] = *(g_uint4 *)(b1p + (size_t)k1 * 8192 + 512 * j);
  };
  auto sstore = [&](int st) {
    uint16_t *A_ = As + st * PF_BM * PF_LDK;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (2 * i + g < nb) *(u32x4_t *)(A_ + (r0 + 64 * i) * PF_LDK + kc * 8) = ra[i];
  };
  auto compute = [&](int st, const u32x4_t(&b)[2][4]) {
    const uint16_t *A_ = As + st * PF_BM * PF_LDK + (32 * g + fr) * PF_LDK + 32 * q;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      bf16x8_t fa[NBW > 0 ? NBW : 1];
#pragma unroll
      for (int i = 0; i < NBW; ++i) fa[i] = *(const bf16x8_t *)(A_ + 64 * i * PF_LDK + 8 * j);
#pragma unroll
      for (int i = 0; i < NBW; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          acc[i][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], __builtin_bit_cast(bf16x8_t, b[h][j]), acc[i][h], 0, 0, 0);
    }
  };
  // one K slab: the weight fragments of slab kt are in `cur`; slab kt+1's are requested into
  // `nxt`, and its activations go through registers into the other LDS stage
  auto step = [&](int kt, const u32x4_t(&cur)[2][4], u32x4_t(&nxt)[2][4]) {
    if (kt + 1 < nk) {
      gloadA(kt + 1);
      if (NBW > 0) gloadB(nxt, kt + 1);
    }
    compute(kt & 1, cur);
    if (kt + 1 < nk) {
      sstore((kt + 1) & 1);
      __syncthreads();
    }
  };
  gloadA(0);
  if (NBW > 0) gloadB(bufA, 0);
  sstore(0);
  __syncthreads();
  for (int kt = 0; kt < nk; kt += 2) {  // nk is even (K % 128 == 0)
    step(kt, bufA, bufB);
    step(kt + 1, bufB, bufA);
  }
}

template <bool SWIGLU>
__global__ __launch_bounds__(512, 1) void k_prefill_gemm(const PfArgs a) {
  extern __shared__ __align__(16) uint16_t As[];  // [2][PF_BM][PF_LDK]
  const int tid = threadIdx.x, lane = tid & 63, w = (tid >> 6) & 3, g = tid >> 8;

  // XCD-aware order: workgroup i runs on XCD i % 8; give every XCD one contiguous range of
  // the block list, so that blocks that share an operand (n tiles of one m tile for the
  // routed experts, m tiles of one n tile for the shared expert) meet in one L2.
  // Each class occupies a multiple of 8 physical blocks, so physical id % 8 is the XCD inside
  // either class and the heavy and the light class are both spread over all XCDs.
  const int pad0 = (a.c[0].n_blocks + 7) & ~7;
  const int ci = (int)blockIdx.x >= pad0;
  const int pb = ci ? blockIdx.x - pad0 : blockIdx.x;
  // only the tiles in use are spread over the XCDs; the launch covers an upper bound
  const int n_mt = *a.c[ci].n_tiles_real;
  const int n_real = n_mt * a.c[ci].n_ntiles;
  const int per_xcd = (n_real + 7) >> 3;
  if ((pb >> 3) >= per_xcd) return;
  int bid = (pb & 7) * per_xcd + (pb >> 3);
  if (bid >= n_real) return;
  const PfClass &c = a.c[ci];
  int mt, nt;
  if (c.m_fastest) { nt = bid / n_mt; mt = bid - nt * n_mt; }
  else { mt = bid / c.n_ntiles; nt = bid - mt * c.n_ntiles; }
  const PfTile tile = c.tiles[mt];
  if (tile.rows <= 0) return;
  const int K = c.K;
  const int n0 = nt * c.n_cols_per_tile;
  const uint16_t *W = (const uint16_t *)(tile.w_base + c.w_off);

  const int kc = tid & 7, r0 = tid >> 3;
  const uint16_t *a_ptr[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = r0 + 64 * i;
    row = row < tile.rows ? row : 0;  // rows past the group's end re-read row 0 (never stored)
    const int grow = tile.row0 + row;
    const int arow = c.gather ? c.gather[grow] : grow;
    a_ptr[i] = c.act + (size_t)arow * c.act_stride + kc * 8;
  }
  // weight blocks of 32 rows x 64 k (2048 elements); the 4 blocks of a 128-row group are
  // adjacent for each k slab, so one slab of a column half is 16 KiB of contiguous memory
  const uint16_t *b0 = W + ((size_t)(n0 / 128) * (K / PF_BK) * 4 + w) * 2048 + lane * 8;
  const uint16_t *b1 = b0 + (size_t)(c.half_delta / 128) * (K / PF_BK) * 8192;

  f32x16_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][h][e] = 0.f;

  const int nk = K / PF_BK;
  // the slabs of 128-row group G are stored rotated by (G * c.slab_step) % nk, so that groups
  // read in step (same slab at the same time) stream from different DRAM channels
  const int G0 = n0 / 128, G1 = G0 + (int)(c.half_delta / 128);
  const int rot0 = (int)((unsigned)(G0 * c.slab_step) % (unsigned)nk), rot1 = (int)((unsigned)(G1 * c.slab_step) % (unsigned)nk);
  const int nb = (tile.rows + 31) >> 5;
  const int nbw = (nb - g + 1) >> 1;  // live blocks of this wave group (uniform per wave)
  switch (nbw) {
    case 0: pf_mainloop<0>(acc, As, a_ptr, b0, b1, nk, rot0, rot1, nb, tid); break;
    case 1: pf_mainloop<1>(acc, As, a_ptr, b0, b1, nk, rot0, rot1, nb, tid); break;
    case 2: pf_mainloop<2>(acc, As, a_ptr, b0, b1, nk, rot0, rot1, nb, tid); break;
    case 3: pf_mainloop<3>(acc, As, a_ptr, b0, b1, nk, rot0, rot1, nb, tid); break;
    default: pf_mainloop<4>(acc, As, a_ptr, b0, b1, nk, rot0, rot1, nb, tid); break;
  }
  // epilogue.  acc element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l%32
  const int col = 32 * w + (lane & 31);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = 32 * (2 * i + g) + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
      if (row < tile.rows) {
        const size_t orow = (size_t)(tile.row0 + row) * c.out_stride;
        if (SWIGLU) {
          const float gt = acc[i][0][e], up = acc[i][1][e];
          ((uint16_t *)c.out)[orow + n0 + col] = pf_f32_to_bf16(gt / (1.f + expf(-gt)) * up);
        } else {
          ((float *)c.out)[orow + n0 + col] = acc[i][0][e];
          ((float *)c.out)[orow + n0 + PF_BNH + col] = acc[i][1][e];
        }
      }
    }
}

static int pf_gcd(int a, int b) { return b ? pf_gcd(b, a % b) : a; }
static int pf_slab_step(int nk) {
  int s = 3;
  while (pf_gcd(s, nk) != 1) s += 2;
  return s;
}

static int pf_launch(bool swiglu, const PfArgs &a, hipStream_t s) {
  if (a.n_blocks_total <= 0) return MOE_OK;
  const int grid = ((a.c[0].n_blocks + 7) & ~7) + ((a.c[1].n_blocks + 7) & ~7);
  const size_t lds = (size_t)2 * PF_BM * PF_LDK * 2;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e1 = hipFuncSetAttribute((const void *)k_prefill_gemm<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipError_t e2 = hipFuncSetAttribute((const void *)k_prefill_gemm<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (int rc = moe_check_hip(e1 != hipSuccess ? e1 : e2, "hipFuncSetAttribute(k_prefill_gemm)")) return rc;
    attr_set = true;
  }
  moe_ktimer_begin(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  if (swiglu) hipLaunchKernelGGL(k_prefill_gemm<true>, dim3(grid), dim3(512), lds, s, a);
  else hipLaunchKernelGGL(k_prefill_gemm<false>, dim3(grid), dim3(512), lds, s, a);
  moe_ktimer_end(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  return moe_check_launch("k_prefill_gemm");
}

// ---- tile list ------------------------------------------------------------------------
// One entry per tile of every active expert's token group (routed list: groups of more than
// 256 rows are split evenly), and one per 256 / 128 tokens for the shared expert's two passes.  Built on the device from the dispatch result, so
// the host never needs the counts: the launch covers the upper bound on the number of
// blocks and entries past the real count have rows = 0.
__global__ __launch_bounds__(1024) void k_prefill_tiles(const moe_unit *__restrict__ units, int max_units,
                                                        const unsigned long long *__restrict__ expert_ptr,
                                                        PfTile *__restrict__ tiles, int n_tiles_max,
                                                        PfTile *__restrict__ sh_tiles, int n_sh_tiles,
                                                        PfTile *__restrict__ sh_tiles2, int n_sh_tiles2,
                                                        unsigned long long shared_base, int T, int *__restrict__ n_real,
                                                        int *__restrict__ err) {
  __shared__ int scan[1024];
  const int tid = threadIdx.x;
  int total_prev = 0;
  for (int base = 0; base < max_units; base += 1024) {
    const int u = base + tid;
    int m = 0, row0 = 0;
    unsigned long long wb = 0;
    if (u < max_units) {
      const moe_unit un = units[u];
      if (un.m > 0 && un.expert >= 0) {
        wb = expert_ptr[un.expert];
        if (wb) { m = un.m; row0 = un.row0; }
        else atomicOr(err, 1);
      }
    }
    const int nt = (m + PF_BM - 1) / PF_BM;
    // rows of a group are split evenly over its tiles, in multiples of 32
    const int per = nt ? ((((m + nt - 1) / nt) + 31) & ~31) : 0;
    scan[tid] = nt;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
      const int v = tid >= d ? scan[tid - d] : 0;
      __syncthreads();
      scan[tid] += v;
      __syncthreads();
    }
    const int first = total_prev + scan[tid] - nt;
    for (int i = 0; i < nt; ++i)
      if (first + i < n_tiles_max) {
        PfTile t;
        t.w_base = wb; t.row0 = row0 + i * per; t.rows = max(0, min(per, m - i * per));
        tiles[first + i] = t;
      }
    total_prev += scan[1023];
    __syncthreads();
  }
  if (tid == 0) { n_real[0] = min(total_prev, n_tiles_max); n_real[1] = n_sh_tiles; n_real[2] = n_sh_tiles2; }
  for (int i = total_prev + tid; i < n_tiles_max; i += 1024) {
    PfTile t; t.w_base = 0; t.row0 = 0; t.rows = 0;
    tiles[i] = t;
  }
  for (int i = tid; i < n_sh_tiles; i += 1024) {
    PfTile t; t.w_base = shared_base; t.row0 = i * PF_BM_SHARED; t.rows = min(PF_BM_SHARED, T - i * PF_BM_SHARED);
    sh_tiles[i] = t;
  }
  for (int i = tid; i < n_sh_tiles2; i += 1024) {
    PfTile t; t.w_base = shared_base; t.row0 = i * PF_BM_SHARED_W2; t.rows = min(PF_BM_SHARED_W2, T - i * PF_BM_SHARED_W2);
    sh_tiles2[i] = t;
  }
}

extern "C" int moe_prefill_tile_rows(void) { return PF_BM; }

extern "C" int64_t moe_prefill_workspace_bytes(int T, int k, int max_units) {
  const int64_t P = (int64_t)T * k;
  return (P / PF_BM + max_units + (T + PF_BM_SHARED - 1) / PF_BM_SHARED + (T + PF_BM_SHARED_W2 - 1) / PF_BM_SHARED_W2 + 3) * (int64_t)sizeof(PfTile);
}

extern "C" int moe_experts_prefill(const void *x_bf16, int T, int H, int I, int I_sh, int k, int fmt,
                                   const moe_unit *units, int max_units, const int *sorted_tok,
                                   const uint64_t *expert_ptr, const void *shared_ptr, void *h_r, void *h_s,
                                   float *part_r, float *part_s, void *tiles_ws, int *err, int phases,
                                   void *stream) {
  hipStream_t s = (hipStream_t)stream;
  if (T == 0) return MOE_OK;
  if (!x_bf16 || T < 0 || k <= 0 || max_units < 0 || !units || !sorted_tok || !expert_ptr || !tiles_ws || !err ||
      !h_r || !part_r || (shared_ptr && (!h_s || !part_s || I_sh <= 0))) {
    moe_set_error("moe_experts_prefill: NULL or negative argument");
    return MOE_EINVAL;
  }
  if (fmt != MOE_FMT_BF16) {
    moe_set_error("moe_experts_prefill: weight format %d not supported by the prefill kernels", fmt);
    return MOE_EINVAL;
  }
  if (H % 256 || I % 128 || (shared_ptr && I_sh % 128)) {
    moe_set_error("moe_experts_prefill: H %% 256 == 0 and I %% 128 == 0 required (H=%d I=%d I_sh=%d)", H, I, I_sh);
    return MOE_EINVAL;
  }
  const long long P = (long long)T * k;
  const int n_r = (int)(P / PF_BM) + max_units;
  const int n_s = shared_ptr ? (T + PF_BM_SHARED - 1) / PF_BM_SHARED : 0;
  const int n_s2 = shared_ptr ? (T + PF_BM_SHARED_W2 - 1) / PF_BM_SHARED_W2 : 0;
  int *n_real = (int *)tiles_ws;  // [0] routed tiles in use, [1] shared tiles (w13 pass), [2] shared tiles (w2 pass)
  PfTile *tiles = (PfTile *)tiles_ws + 1, *sh_tiles = tiles + n_r, *sh_tiles2 = sh_tiles + n_s;
  hipLaunchKernelGGL(k_prefill_tiles, dim3(1), dim3(1024), 0, s, units, max_units,
                     (const unsigned long long *)expert_ptr, tiles, n_r, sh_tiles, n_s, sh_tiles2, n_s2,
                     (unsigned long long)(uintptr_t)shared_ptr, T, n_real, err);
  if (int rc = moe_check_launch("k_prefill_tiles")) return rc;
  for (int w2 = 0; w2 < 2; ++w2) {
    if (!(phases & (w2 ? 2 : 1))) continue;
    PfArgs a;
    memset(&a, 0, sizeof a);
    // the shared expert (long K in the w2 pass, dense rows) goes first, the routed groups fill in behind it
    int n = 0;
    for (int shared = 1; shared >= 0; --shared) {
      if (shared && !shared_ptr) continue;
      PfClass &c = a.c[n++];
      const int Ii = shared ? I_sh : I;
      c.tiles = shared ? (w2 ? sh_tiles2 : sh_tiles) : tiles;
      c.n_mtiles = shared ? (w2 ? n_s2 : n_s) : n_r;
      c.n_tiles_real = n_real + (shared ? (w2 ? 2 : 1) : 0);
      c.m_fastest = shared;
      if (!w2) {  // w13 [2I, H]: gate rows 0..I-1, up rows I..2I-1
        c.act = (const uint16_t *)x_bf16; c.gather = shared ? nullptr : sorted_tok; c.act_stride = H;
        c.out = shared ? h_s : h_r; c.out_stride = Ii;
        c.K = H; c.w_off = 0; c.half_delta = Ii; c.n_cols_per_tile = PF_BNH; c.n_ntiles = Ii / PF_BNH;
      } else {    // w2 [H, I] after w13 in the expert image
        c.act = (const uint16_t *)(shared ? h_s : h_r); c.gather = nullptr; c.act_stride = Ii;
        c.out = shared ? (void *)part_s : (void *)part_r; c.out_stride = H;
        c.K = Ii; c.w_off = (long long)2 * Ii * H * 2; c.half_delta = PF_BNH; c.n_cols_per_tile = 2 * PF_BNH;
        c.n_ntiles = H / (2 * PF_BNH);
      }
      c.n_blocks = c.n_mtiles * c.n_ntiles;
      c.slab_step = pf_slab_step(c.K / PF_BK);
      a.n_blocks_total += c.n_blocks;
    }
    if (int rc = pf_launch(!w2, a, s)) return rc;
  }
  return MOE_OK;
}
