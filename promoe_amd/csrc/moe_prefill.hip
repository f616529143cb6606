// Prefill-sized expert groups on the matrix cores (gfx950): grouped GEMM over the
// tokens dispatched to each expert, bf16 operands, fp32 accumulation.
//
//   w13 pass: h[rows, I]  = silu(A Wg^T) * (A Wu^T)     A = gathered activations
//   w2  pass: part[rows,H] = h W2^T
//
// Workgroup = 256 threads (4 waves, 2x2) -> a 128-row x (128+128)-column tile: for w13
// the two column halves are the SAME columns of gate and up (SwiGLU fused in the
// epilogue), for w2 they are adjacent column blocks.  K advances 64 at a time through a
// double-buffered LDS stage (global -> registers -> LDS), fragments are read with
// ds_read_b128 and fed to v_mfma_f32_32x32x16_bf16; each wave owns 64 x (64+64) outputs
// (128 accumulator registers).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "moe_common.h"
#include "moe_kernels.h"

typedef unsigned int u32;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const u32x4_t g_uint4;

#define PF_BM 128
#define PF_BNH 128   // columns per half
#define PF_BK 64
#define PF_LDK 72    // LDS row stride in bf16 (64 + 8 pad = 144 bytes: conflict-free b128 reads)

struct PfTile {
  unsigned long long w_base;  // expert image base (device address)
  int row0;                   // first row (sorted pair order / token order for the shared expert)
  int rows;                   // valid rows in this tile (<= PF_BM)
};
struct PfArgs {
  const uint16_t *act;  // bf16 activations
  const int *gather;    // row -> activation row, or NULL
  void *out;            // bf16 h (SWIGLU) or fp32 partial
  const PfTile *tiles;
  long long w_off;      // byte offset of the matrix inside the expert image
  long long half_delta; // element offset from the first column half's weight rows to the second's
  int act_stride, out_stride, K, n_ntiles, n_mtiles, n_cols_per_tile;
};

static __device__ __forceinline__ float pf_bf16_to_f32(uint16_t b) { return __uint_as_float((u32)b << 16); }
static __device__ __forceinline__ uint16_t pf_f32_to_bf16(float f) {
  u32 u = __float_as_uint(f);
  u32 r = ((u >> 16) & 1u) + 0x7fffu;
  return (uint16_t)((u + r) >> 16);
}

template <bool SWIGLU>
__global__ __launch_bounds__(256, 1) void k_prefill_gemm(const PfArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t *As = (uint16_t *)smem;                                  // [2][128][72]
  uint16_t *Bs = As + 2 * PF_BM * PF_LDK;                           // [2][256][72]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int wm = w >> 1, wn = w & 1;

  // XCD-aware order: the 8 XCDs take contiguous ranges of tiles, so that tiles sharing an
  // activation block (same m tile, consecutive n tiles) meet in one L2
  const int grid = gridDim.x;
  int bid = blockIdx.x;
  if ((grid & 7) == 0) bid = (bid & 7) * (grid >> 3) + (bid >> 3);
  const int mt = bid / a.n_ntiles, nt = bid - mt * a.n_ntiles;
  const PfTile tile = a.tiles[mt];
  if (tile.rows <= 0) return;
  const int K = a.K;
  const int n0 = nt * a.n_cols_per_tile;
  const uint16_t *W = (const uint16_t *)(tile.w_base + a.w_off);

  // global -> register staging: A 128 rows x 8 chunks (4 per thread), B 256 rows x 8 chunks (8 per thread)
  const int kc = tid & 7;       // 16-byte chunk inside the 64-wide K slab
  const int r0 = tid >> 3;      // 0..31
  const uint16_t *a_ptr[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = r0 + 32 * i;
    row = row < tile.rows ? row : 0;  // rows past the group's end re-read row 0 (never stored)
    const int grow = tile.row0 + row;
    const int arow = a.gather ? a.gather[grow] : grow;
    a_ptr[i] = a.act + (size_t)arow * a.act_stride + kc * 8;
  }
  const uint16_t *b_ptr[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int brow = r0 + 32 * i;  // 0..255: first half then second half
    const long long wrow = brow < PF_BNH ? (long long)(n0 + brow) : a.half_delta + (n0 + brow - PF_BNH);
    b_ptr[i] = W + wrow * K + kc * 8;
  }
  u32x4_t ra[4], rb[8];
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) ra[i] = *(g_uint4 *)(a_ptr[i] + k0);
#pragma unroll
    for (int i = 0; i < 8; ++i) rb[i] = *(g_uint4 *)(b_ptr[i] + k0);
  };
  auto sstore = [&](int st) {
    uint16_t *A_ = As + st * PF_BM * PF_LDK, *B_ = Bs + st * 2 * PF_BNH * PF_LDK;
#pragma unroll
    for (int i = 0; i < 4; ++i) *(u32x4_t *)(A_ + (r0 + 32 * i) * PF_LDK + kc * 8) = ra[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) *(u32x4_t *)(B_ + (r0 + 32 * i) * PF_LDK + kc * 8) = rb[i];
  };

  f32x16_t acc[2][2][2];  // [a: 32-row block][b: 32-col block][half]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][h][e] = 0.f;

  const int nk = K / PF_BK;
  gload(0);
  sstore(0);
  __syncthreads();
  const int fr = lane & 31, fk = (lane >> 5) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int st = kt & 1;
    if (kt + 1 < nk) gload((kt + 1) * PF_BK);
    const uint16_t *A_ = As + st * PF_BM * PF_LDK + (64 * wm + fr) * PF_LDK + fk;
    const uint16_t *B_ = Bs + st * 2 * PF_BNH * PF_LDK + (64 * wn + fr) * PF_LDK + fk;
#pragma unroll
    for (int j = 0; j < PF_BK / 16; ++j) {
      bf16x8_t fa[2], fb[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = *(const bf16x8_t *)(A_ + 32 * i * PF_LDK + 16 * j);
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int h = 0; h < 2; ++h) fb[b][h] = *(const bf16x8_t *)(B_ + (h * PF_BNH + 32 * b) * PF_LDK + 16 * j);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            acc[i][b][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[b][h], acc[i][b][h], 0, 0, 0);
    }
    if (kt + 1 < nk) {
      sstore(st ^ 1);
      __syncthreads();
    }
  }
  // epilogue.  acc element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l%32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = 64 * wm + 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        const int col = 64 * wn + 32 * b + (lane & 31);
        if (row < tile.rows) {
          const size_t orow = (size_t)(tile.row0 + row) * a.out_stride;
          if (SWIGLU) {
            const float g = acc[i][b][0][e], u = acc[i][b][1][e];
            ((uint16_t *)a.out)[orow + n0 + col] = pf_f32_to_bf16(g / (1.f + expf(-g)) * u);
          } else {
            ((float *)a.out)[orow + n0 + col] = acc[i][b][0][e];
            ((float *)a.out)[orow + n0 + PF_BNH + col] = acc[i][b][1][e];
          }
        }
      }
}

static int pf_launch(bool swiglu, const PfArgs &a, hipStream_t s) {
  const size_t lds = (size_t)2 * (PF_BM + 2 * PF_BNH) * PF_LDK * 2;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e1 = hipFuncSetAttribute((const void *)k_prefill_gemm<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipError_t e2 = hipFuncSetAttribute((const void *)k_prefill_gemm<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (int rc = moe_check_hip(e1 != hipSuccess ? e1 : e2, "hipFuncSetAttribute(k_prefill_gemm)")) return rc;
    attr_set = true;
  }
  const int grid = a.n_mtiles * a.n_ntiles;
  if (grid <= 0) return MOE_OK;
  moe_ktimer_begin(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  if (swiglu) hipLaunchKernelGGL(k_prefill_gemm<true>, dim3(grid), dim3(256), lds, s, a);
  else hipLaunchKernelGGL(k_prefill_gemm<false>, dim3(grid), dim3(256), lds, s, a);
  moe_ktimer_end(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  return moe_check_launch("k_prefill_gemm");
}


// ---- tile list ------------------------------------------------------------------------
// One entry per 128-row block of every active expert's token group (routed list), and one
// per 128 tokens for the shared expert.  Built on the device from the dispatch result, so
// the host never needs the counts: the launch covers the upper bound on the number of
// blocks and entries past the real count have rows = 0.
__global__ __launch_bounds__(1024) void k_prefill_tiles(const moe_unit *__restrict__ units, int max_units,
                                                        const unsigned long long *__restrict__ expert_ptr,
                                                        PfTile *__restrict__ tiles, int n_tiles_max,
                                                        PfTile *__restrict__ sh_tiles, int n_sh_tiles,
                                                        unsigned long long shared_base, int T, int *__restrict__ err) {
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
        t.w_base = wb; t.row0 = row0 + i * PF_BM; t.rows = min(PF_BM, m - i * PF_BM);
        tiles[first + i] = t;
      }
    total_prev += scan[1023];
    __syncthreads();
  }
  for (int i = total_prev + tid; i < n_tiles_max; i += 1024) {
    PfTile t; t.w_base = 0; t.row0 = 0; t.rows = 0;
    tiles[i] = t;
  }
  for (int i = tid; i < n_sh_tiles; i += 1024) {
    PfTile t; t.w_base = shared_base; t.row0 = i * PF_BM; t.rows = min(PF_BM, T - i * PF_BM);
    sh_tiles[i] = t;
  }
}

extern "C" int moe_prefill_tile_rows(void) { return PF_BM; }

extern "C" int64_t moe_prefill_workspace_bytes(int T, int k, int max_units) {
  const int64_t P = (int64_t)T * k;
  return (P / PF_BM + max_units + (T + PF_BM - 1) / PF_BM + 2) * (int64_t)sizeof(PfTile);
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
  const int n_s = shared_ptr ? (T + PF_BM - 1) / PF_BM : 0;
  PfTile *tiles = (PfTile *)tiles_ws, *sh_tiles = tiles + n_r;
  hipLaunchKernelGGL(k_prefill_tiles, dim3(1), dim3(1024), 0, s, units, max_units,
                     (const unsigned long long *)expert_ptr, tiles, n_r, sh_tiles, n_s,
                     (unsigned long long)(uintptr_t)shared_ptr, T, err);
  if (int rc = moe_check_launch("k_prefill_tiles")) return rc;
  PfArgs a;
  for (int pass = 0; pass < 4; ++pass) {
    const bool shared = pass & 1, w2 = pass >> 1;
    if (shared && !shared_ptr) continue;
    if (!(phases & (w2 ? 2 : 1))) continue;
    const int Ii = shared ? I_sh : I;
    memset(&a, 0, sizeof a);
    a.tiles = shared ? sh_tiles : tiles;
    a.n_mtiles = shared ? n_s : n_r;
    if (!w2) {  // w13 [2I, H]: gate rows 0..I-1, up rows I..2I-1
      a.act = (const uint16_t *)x_bf16; a.gather = shared ? nullptr : sorted_tok; a.act_stride = H;
      a.out = shared ? h_s : h_r; a.out_stride = Ii;
      a.K = H; a.w_off = 0; a.half_delta = Ii; a.n_cols_per_tile = PF_BNH; a.n_ntiles = Ii / PF_BNH;
    } else {    // w2 [H, I] after w13 in the expert image
      a.act = (const uint16_t *)(shared ? h_s : h_r); a.gather = nullptr; a.act_stride = Ii;
      a.out = shared ? part_s : part_r; a.out_stride = H;
      a.K = Ii; a.w_off = (long long)2 * Ii * H * 2; a.half_delta = PF_BNH; a.n_cols_per_tile = 2 * PF_BNH;
      a.n_ntiles = H / (2 * PF_BNH);
    }
    if (int rc = pf_launch(!w2, a, s)) return rc;
  }
  return MOE_OK;
}
