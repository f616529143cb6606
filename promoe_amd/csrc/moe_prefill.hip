// Prefill-sized expert groups on the matrix cores (gfx950): grouped GEMM over the
// tokens dispatched to each expert, bf16 operands, fp32 accumulation.
//
//   w13 pass: h[rows, I]   = silu(A Wg^T) * (A Wu^T)     A = gathered activations
//   w2  pass: part[rows,H] = h W2^T
//
// bf16 experts: workgroup = 256 threads (4 waves, one per SIMD) -> a tile of up to 256 rows x (128+128)
// columns: for w13 the two column halves are the SAME columns of gate and up (SwiGLU fused in the epilogue),
// for w2 they are adjacent column blocks.  K advances 64 at a time; the activation slab goes global -> LDS
// directly (a ring of four slabs), the weight fragments go global -> registers in operand order and feed
// v_mfma_f32_32x32x16_bf16.  int4 / q4_K experts: 8 waves, fragments dequantised in registers (below).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>
#include <type_traits>

#include "moe_common.h"
#include "moe_kernels.h"
#include "moe_device.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

#define PF_BM 256     // most rows of one tile (8 blocks of 32)
#define PF_BM_SHARED 256     // rows per tile of the dense shared expert in the w13 pass
#define PF_BM_SHARED_W2 128  // and in its w2 pass, which has few column tiles (H/256) and a long K
#define PF_BNH 128   // columns per half
#define PF_BK 64

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
  long long off_s, off_z; // int4: byte offsets of the scale / zero sections (w_off = the nibble section)
  int act_stride, out_stride, K, n_ntiles, n_mtiles, n_cols_per_tile;
  int m_fastest;        // block order inside the class
  int slab_step;        // storage rotation per 128-row group: smallest odd s >= 3 coprime with K/64
  int n_blocks;         // n_mtiles * n_ntiles * ksplit
  int ksplit;           // int4 / q4_K w2 pass of the shared expert: workgroups per tile, each over 1/ksplit of the
                        // reduction, partial rows to out + split * split_stride (0 or 1: the whole reduction)
  long long split_stride;  // elements between the pieces of out
};
struct PfArgs {
  PfClass c[2];
  int n_blocks_total;  // blocks of c[0] come first
};

// silu(g) * u with the hardware's 2^x and reciprocal (1 ulp each; the result is rounded to bf16 by the caller,
// round to nearest even in hardware): a tile's epilogue computes 128 of these per lane
static __device__ __forceinline__ float pf_silu_mul(float g, float u) {
  return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * -1.44269504088896f)) * u;
}

// Which class and which block of it a physical workgroup takes: the blocks of class 0 come first, each class
// padded to a multiple of 8 blocks, so that physical id % 8 is the XCD inside either class.  (Alternating the
// classes in groups of 8 was measured: no gain in the w13 launch, 19 % slower in the w2 launch.)
static __device__ __forceinline__ void pf_block_of(const PfArgs &a, int &ci, int &pb) {
  const int pad0 = (a.c[0].n_blocks + 7) & ~7;
  ci = (int)blockIdx.x >= pad0;
  pb = ci ? (int)blockIdx.x - pad0 : (int)blockIdx.x;
}

// ---- bf16 experts: main loop of one wave ------------------------------------------------------------
// One wave per SIMD, 512 registers each: wave w owns columns 32w..32w+31 of both column halves and ALL row
// blocks of the tile (up to 8 x 32 rows: 256 accumulator registers, which the compiler keeps in the
// accumulation half of the register file), so every weight fragment is fetched by exactly one wave of the
// workgroup.  The weights lie in HBM in operand order (blocks of 32 rows x 64 k, one contiguous KiB per MFMA
// step; within a 64-wide K slab lane half q = lane / 32 takes k = 32 q + 8 j + 0..7 for MFMA j: both operands
// use the same permutation of k, which a dot product allows) and never touch LDS.
// What a single wave per SIMD needs, since nothing else fills its stalls (each measured on the Qwen1.5 shape
// and in a stand-alone loop of the same structure):
//   * weight fragments and activations are requested three slabs ahead (four register sets of fragments,
//     four activation slabs in LDS);
//   * the requests are spread between the products, at most one behind each, instead of standing in a block
//     at the head of a slab where the matrix core runs dry behind them (stand-alone loop, streaming from HBM:
//     1.29 -> 1.53 PFLOP/s);
//   * the activation fragment of a product is read from LDS four product groups ahead, and nothing may move
//     across the pinned order (left to itself the scheduler puts every read right in front of its own
//     products and waits for it there: an LDS round trip per pair of products);
//   * no vector instruction computes an address inside the loop (buffer addressing: lane offsets that never
//     change, slab offsets in scalars; LDS addresses with compile-time ring slots).
#define PF_ST 4                      // register sets of weight fragments: requested three slabs ahead
#define PF4_SLAB (PF_BM * PF_BK)     // bf16 elements of one activation slab in LDS (rows of 128 bytes, no padding)
#define PF4_RING 4                   // slabs in LDS: one being read, three on their way
#define PF_FD 4                      // LDS reads in flight in front of the products
typedef __attribute__((address_space(3))) void pf_lds_void;
typedef __attribute__((address_space(1))) const void pf_g_void;
// s_waitcnt that waits for all but the N most recent vector-memory operations and for nothing else
#define PF_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 15) | (7 << 4) | (15 << 8) | (((N) >> 4) << 14))

typedef int pf_i32x4_t __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t pf_rsrc_t;

// Activations go global -> LDS directly (no registers, no LDS store instructions): transfer n of wave w
// brings rows 32 n + 8 w .. + 7 of the slab, 8 lanes per row.  An LDS row is 128 bytes = 8 chunks of 16; the
// chunk that holds k = 8 c .. 8 c + 7 of row r sits in slot c ^ ((r >> 1) & 7), so the 16 lanes that a
// ds_read_b128 serves together (16 rows, one chunk index) fall on 16 different bank groups.  The lanes choose
// their global address accordingly; the LDS side of the transfer is fixed (lane l writes 16 bytes at 16 l).
// All addresses are buffer addresses (lane offset in a register that never changes, slab offset in a scalar):
// with one wave per SIMD every vector instruction that is not a product is issue time taken from the products.
// NTW: the weight fragments are read with the non-temporal hint (a routed expert's tile is the only reader of
// its fragments: they only pass through the caches); the shared expert's row tiles all read the same fragments
// and those are requested with plain loads, so that the second-level cache keeps them for the next row tile
template <int NB, bool NTW>
static __device__ __forceinline__ void pf_mainloop(f32x16_t (&acc)[8][2], unsigned lds_base, const pf_i32x4_t ra_rsrc,
                                                    const int (&a_voff)[8], const pf_rsrc_t rb, int b_delta1, int nk, int rot0,
                                                    int rot1, int tid) {
  const int lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fr = lane & 31, q = lane >> 5;
  constexpr int NL = NB + 8;   // requests of a step: NB activation transfers, 8 weight fragments
  constexpr int NS = 4 * NB;   // groups of two products
  u32x4_t bw[PF_ST][2][4];
  const int b_voff = lane * 16;
  // transfer n of slab kt_ into ring slot `slot` (past the end: the last slab again, into a slot nobody reads)
  auto dma = [&](int n, int kt_, int slot) {
    const int kt = kt_ < nk ? kt_ : nk - 1;
    // Written as assembly on purpose: the compiler, told that a load writes LDS, waits for ALL such loads in
    // front of every barrier and LDS read, which would end the run-ahead; here the waits are placed by hand
    // (PF_VMCNT below).  Its own counts for the fragment loads then include fewer operations than are in
    // flight, which only makes its waits for those loads earlier, never later.
    const unsigned lds_addr = lds_base + (unsigned)(slot * PF4_SLAB + (32 * n + 8 * w) * PF_BK) * 2u;
    __asm__ volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :: "s"(lds_addr), "v"(a_voff[n]), "s"(ra_rsrc), "s"(kt * (PF_BK * 2)) : "memory", "m0");
  };
  auto bslab = [&](int kt_, int rot) {
    const int kt = kt_ < nk ? kt_ : nk - 1;  // past the end: the last slab once more (never used)
    const int k = kt + rot;                  // slab position inside the 128-row group's storage
    return (k >= nk ? k - nk : k) * 16384;   // bytes
  };
  // LDS byte address of the lane's fragment of MFMA step j in row block 0 of slot 0 (chunk 4 q + j of its row)
  unsigned faddr[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) faddr[j] = lds_base + (unsigned)(fr * PF_BK + (((4 * q + j) ^ ((fr >> 1) & 7)) * 8)) * 2u;
  auto lds_frag = [&](int slot, int g) {
    typedef __attribute__((address_space(3))) const bf16x8_t lds_frag_t;
    return *(lds_frag_t *)(uintptr_t)(faddr[g / NB] + (unsigned)(slot * PF4_SLAB + 32 * (g % NB) * PF_BK) * 2u);
  };
  // slab kt (ring slot S = kt % 4, a compile-time number in the unrolled loop): its weight fragments are in
  // `cur`.  Requested meanwhile, at most one request behind every product: the activations (into slot
  // (S + 3) % 4) and the fragments (into `far`) of slab kt + 3.
  auto step = [&](auto S_, int kt, const u32x4_t(&cur)[2][4], u32x4_t(&far)[2][4]) {
    constexpr int S = decltype(S_)::value;
    const int sb0 = bslab(kt + 3, rot0), sb1 = bslab(kt + 3, rot1) + b_delta1;
    // product group g = MFMA step j = g / NB of row block i = g % NB; its activation fragment is read from LDS
    // PF_FD groups ahead of its products
    bf16x8_t fa[PF_FD + 1];
#pragma unroll
    for (int g = 0; g < PF_FD && g < NS; ++g) fa[g] = lds_frag(S, g);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < NS; ++g) {
      acc[g % NB][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[g % (PF_FD + 1)], __builtin_bit_cast(bf16x8_t, cur[0][g / NB]),
                                                               acc[g % NB][0], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (g + PF_FD < NS) fa[(g + PF_FD) % (PF_FD + 1)] = lds_frag(S, g + PF_FD);
      __builtin_amdgcn_sched_barrier(0);
      acc[g % NB][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[g % (PF_FD + 1)], __builtin_bit_cast(bf16x8_t, cur[1][g / NB]),
                                                               acc[g % NB][1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < NL; ++n)
        if (n * NS / NL == g) {  // request n of this step goes out behind product group g
          if (n < NB) dma(n, kt + 3, (S + 3) % PF4_RING);
          else if (n - NB < 4) far[0][n - NB] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_voff + 1024 * (n - NB), sb0, NTW ? 2 : 0);
          else far[1][n - NB - 4] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_voff + 1024 * (n - NB - 4), sb1, NTW ? 2 : 0);
        }
      __builtin_amdgcn_sched_barrier(0);
    }
    // slab kt + 1 must have landed before anybody reads it: its transfers are two steps old, issued before
    // the 8 fragment loads of their own step and the NB + 8 requests of each of the two steps since
    PF_VMCNT(2 * NB + 24);
    __syncthreads();
  };
  auto gloadB = [&](u32x4_t(&b)[2][4], int kt) {
    const int sb0 = bslab(kt, rot0), sb1 = bslab(kt, rot1) + b_delta1;
#pragma unroll
    for (int j = 0; j < 4; ++j) b[0][j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_voff + 1024 * j, sb0, NTW ? 2 : 0);
#pragma unroll
    for (int j = 0; j < 4; ++j) b[1][j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_voff + 1024 * j, sb1, NTW ? 2 : 0);
  };
#pragma unroll
  for (int t = 0; t < 3; ++t) {
#pragma unroll
    for (int n = 0; n < NB; ++n) dma(n, t, t);
    gloadB(bw[t], t);
  }
  PF_VMCNT(0);
  __syncthreads();
  typedef std::integral_constant<int, 0> S0; typedef std::integral_constant<int, 1> S1;
  typedef std::integral_constant<int, 2> S2; typedef std::integral_constant<int, 3> S3;
  for (int kt = 0; kt < nk; kt += 4) {  // nk is even; no separate tail: its register assignment would differ
    step(S0(), kt, bw[0], bw[3]);      // from the loop's and the compiler would spill around the loop's back edge
    step(S1(), kt + 1, bw[1], bw[0]);
    if (kt + 2 < nk) {
      step(S2(), kt + 2, bw[2], bw[1]);
      step(S3(), kt + 3, bw[3], bw[2]);
    }
  }
}

template <bool SWIGLU>
__global__ __launch_bounds__(256, 1) void k_prefill_gemm(const PfArgs a) {
  extern __shared__ __align__(16) uint16_t As[];  // [PF4_RING][PF_BM][PF_BK]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  // XCD-aware order: workgroup i runs on XCD i % 8; give every XCD one contiguous range of the block list,
  // so that blocks that share an operand (n tiles of one m tile for the routed experts, m tiles of one n
  // tile for the shared expert) meet in one L2.  Only the tiles in use are spread over the XCDs; the launch
  // covers an upper bound.
  int ci, pb;
  pf_block_of(a, ci, pb);
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

  // transfer n of this wave brings rows 32 n + 8 w .. + 7, 8 lanes per row; the lane in slot s of row r
  // fetches chunk s ^ ((r >> 1) & 7).  Byte offsets from the activation tensor's base (< 2 GiB, checked by the launcher)
  int a_voff[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int rt = 32 * i + 8 * w + (lane >> 3);
    const int row = rt < tile.rows ? rt : 0;  // rows past the group's end re-read row 0 (never stored)
    const int grow = tile.row0 + row;
    const int arow = c.gather ? c.gather[grow] : grow;
    a_voff[i] = (arow * c.act_stride + (((lane & 7) ^ ((rt >> 1) & 7)) * 8)) * 2;
  }
  pf_i32x4_t ra_rsrc;
  {
    const unsigned long long ab = (unsigned long long)c.act;
    ra_rsrc.x = __builtin_amdgcn_readfirstlane((int)(unsigned)ab);
    ra_rsrc.y = __builtin_amdgcn_readfirstlane((int)(unsigned)(ab >> 32));
    ra_rsrc.z = 0x7fffffff; ra_rsrc.w = 0x00020000;
  }
  // weight blocks of 32 rows x 64 k (4 KiB); the 4 blocks of a 128-row group are adjacent for each k slab, so
  // one slab of a column half is 16 KiB of contiguous memory; wave w reads block w
  const int nk = K / PF_BK;
  const unsigned char *wb = (const unsigned char *)W + ((size_t)(n0 / 128) * nk * 4 + w) * 4096;
  const unsigned long long wbu = (unsigned long long)wb;
  const pf_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      (void *)(((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(wbu >> 32)) << 32) |
               (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)wbu)), 0, 0x7fffffff, 0x00020000);
  const int b_delta1 = (int)(c.half_delta / 128) * nk * 16384;

  f32x16_t acc[8][2];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][h][e] = 0.f;

  const int G0 = n0 / 128, G1 = G0 + (int)(c.half_delta / 128);
  const int rot0 = (int)((unsigned)(G0 * c.slab_step) % (unsigned)nk), rot1 = (int)((unsigned)(G1 * c.slab_step) % (unsigned)nk);
  const int nb = (tile.rows + 31) >> 5;  // live row blocks (uniform for the workgroup)
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)As;
#define PF_LOOPS(NTW_)                                                                                          \
  switch (nb) {                                                                                             \
    case 1: pf_mainloop<1, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    case 2: pf_mainloop<2, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    case 3: pf_mainloop<3, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    case 4: pf_mainloop<4, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    case 5: pf_mainloop<5, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    case 6: pf_mainloop<6, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    case 7: pf_mainloop<7, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
    default: pf_mainloop<8, NTW_>(acc, lds_base, ra_rsrc, a_voff, rb, b_delta1, nk, rot0, rot1, tid); break; \
  }
  if (c.m_fastest) { PF_LOOPS(false) } else { PF_LOOPS(true) }   // (m_fastest: the shared expert's class)
#undef PF_LOOPS
  // epilogue.  acc element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l%32
  const int col = 32 * w + (lane & 31);
  if constexpr (SWIGLU) {
    // The h tile (rows x 128 bf16) goes through LDS, so that it leaves in 16-byte stores that cover whole 256-byte
    // rows: straight from the accumulators a lane stores 2 bytes at a time (128 store instructions per lane, each
    // covering two 64-byte pieces of two rows).  The activation ring is free once every wave has left the main loop
    // and the transfers still on their way into it (the slabs requested past the end) have landed.
    constexpr int HS = 2 * PF_BNH + 16;  // padded row stride in bytes
    static_assert((size_t)PF_BM * HS <= (size_t)PF4_RING * PF4_SLAB * 2, "the h tile fits the activation ring");
    unsigned char *hs = (unsigned char *)As;
    PF_VMCNT(0);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < nb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
          *(__bf16 *)(hs + row * HS + col * 2) = (__bf16)pf_silu_mul(acc[i][0][e], acc[i][1][e]);
        }
      }
    __syncthreads();
    const int chunk = tid & 15;
    for (int row = tid >> 4; row < tile.rows; row += 16) {
      const uint4 v = *(const uint4 *)(hs + row * HS + chunk * 16);
      *(uint4 *)((__bf16 *)c.out + (size_t)(tile.row0 + row) * c.out_stride + n0 + 8 * chunk) = v;
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
      if (row < tile.rows) {
        const size_t orow = (size_t)(tile.row0 + row) * c.out_stride;
        if (SWIGLU) {
          ((__bf16 *)c.out)[orow + n0 + col] = (__bf16)pf_silu_mul(acc[i][0][e], acc[i][1][e]);
        } else {
          ((float *)c.out)[orow + n0 + col] = acc[i][0][e];
          ((float *)c.out)[orow + n0 + PF_BNH + col] = acc[i][1][e];
        }
      }
    }
}

// ---- int4-g128 experts ----------------------------------------------------------------
// Same tiling as the bf16 kernel (8 waves, tile of up to 256 rows, wave w of group g owns 64
// weight rows and the 32-row blocks g, g+2, ...), K advances one quantisation group (128) at
// a time.  The int4 tiles of the slot layout are already in the operand order of
// v_mfma_f32_16x16x32_f16 (lane = row l&15, k quarter l>>4, dword j = 8 consecutive k), so a
// wave loads them straight into registers and dequantises there: a nibble pair is shifted and masked
// into the mantissas of two fp16 values 1 + q/16 and one packed fma per pair applies scale and zero
// (deq8_f16 below).  gfx950 has packed fp16 arithmetic
// but no packed bf16 arithmetic, hence fp16 operands: activations are converted bf16 -> fp16
// while they are staged into LDS (exact for |x| < 65504 outside the fp16 subnormal range); the h rows
// between the two passes are written as fp16 by the w13 epilogue, so the w2 pass stages them as they are.
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const uint16_t g_u16;
typedef __attribute__((address_space(1))) const unsigned char g_u8;

#define PI_LDK 136  // LDS row stride in fp16 (128 + 8 pad = 272 bytes)
#define PI_BM 192   // most rows of one tile: 6 blocks of 32 (96 accumulator registers per wave)

// buffer resource over [p, p+bytes): loads past the end return 0 instead of faulting
static __device__ __forceinline__ rsrc_t pf_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, (int)bytes, 0x00020000);
}
static __device__ __forceinline__ const unsigned char *pf_uniform(const unsigned char *p) {
  const unsigned long long v = (unsigned long long)p;
  const u32 lo = __builtin_amdgcn_readfirstlane((u32)v), hi = __builtin_amdgcn_readfirstlane((u32)(v >> 32));
  return (const unsigned char *)(((unsigned long long)hi << 32) | lo);
}

struct PiMeta { u32 sc[4]; u32 zz[4]; };  // raw fp16 scale bits / zero nibble of the lane's row in the 4 tiles

// ACT16: the activations are fp16 already (the h rows this kernel's w13 pass wrote, or a converted copy of x):
// staged as they are, without the three vector operations per pair of the bf16 -> fp16 conversion
// Gt: quantisation groups per weight row in memory; this workgroup reduces over the window [g0, g0 + G) of them
template <int NBW, bool Q4K, bool ACT16>
static __device__ __forceinline__ void pi_mainloop(f32x4_t (&acc)[4][6], uint16_t *As, const rsrc_t rx, const u32 (&a_off)[6],
                                                   const rsrc_t rq, const rsrc_t rs, const rsrc_t rz, int Gt, int g0, int G,
                                                   int nb, int tid) {
  const int lane = tid & 63, g = tid >> 8;
  const int r = lane & 15, qd = lane >> 4;
  const int ch = tid & 15, r0 = tid >> 4;  // staging: row r0 + 32 i (block i), 16-byte chunk ch of the 128-k group
  const DeqF16Consts dqc = deq_f16_consts();
  u32x4_t ra[3], wA[4], wB[4];
  PiMeta mA, mB;
  // activations of the next group travel in two halves (row blocks 0..2, then 3..5) through
  // the same three staging registers
  auto gloadA = [&](int gi, int half) {
#pragma unroll
    for (int i = 0; i < 3; ++i)  // unconditional (blocks past the tile's end re-read its first rows): the same
      ra[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, a_off[3 * half + i], (g0 + gi) * 256, 0);  // number of loads in every iteration
  };
  auto sstore = [&](int st, int half) {
    uint16_t *A_ = As + st * PI_BM * PI_LDK;
#pragma unroll
    for (int i = 0; i < 3; ++i)
      if (3 * half + i < nb) {
        u32x4_t v = ra[i];
        if (!ACT16) {
          v.x = bf16x2_to_f16x2(ra[i].x); v.y = bf16x2_to_f16x2(ra[i].y);
          v.z = bf16x2_to_f16x2(ra[i].z); v.w = bf16x2_to_f16x2(ra[i].w);
        }
        *(u32x4_t *)(A_ + (r0 + 32 * (3 * half + i)) * PI_LDK + ch * 8) = v;
      }
  };
  auto gloadW = [&](u32x4_t(&wq)[4], PiMeta &m, int gi) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int gm = g0 + gi;  // the group in memory
      wq[t] = __builtin_amdgcn_raw_buffer_load_b128(rq, lane * 16, (t * Gt + gm) * 1024, 0);
      if (Q4K) {  // (sc, m) byte pair of the lane's sub-block; (d, dmin) of the row's super-block
        m.sc[t] = __builtin_amdgcn_raw_buffer_load_b16(rs, 2 * lane, (t * Gt + gm) * 128, 0);
        m.zz[t] = __builtin_amdgcn_raw_buffer_load_b32(rz, 4 * r, (t * (Gt >> 1) + (gm >> 1)) * 64, 0);
      } else {
        m.sc[t] = __builtin_amdgcn_raw_buffer_load_b16(rs, 2 * r, (t * Gt + gm) * 32, 0);
        m.zz[t] = __builtin_amdgcn_raw_buffer_load_b8(rz, r >> 1, (t * Gt + gm) * 8, 0);
      }
    }
  };
  // S = 16 s and C of deq8_f16 for the lane's row in the 4 tiles of a group, once per group
  auto prep = [&](const PiMeta &m, u32 (&s2)[4], u32 (&c2)[4]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float s16, cz;
      if (Q4K) {
        s16 = 16.f * __builtin_bit_cast(float, h2f_bits(m.zz[t] & 0xffffu)) * (float)(m.sc[t] & 0xffu);
        const float dmn = __builtin_bit_cast(float, h2f_bits(m.zz[t] >> 16)) * (float)((m.sc[t] >> 8) & 0xffu);
        cz = -s16 - dmn;
      } else {
        const float sf = __builtin_bit_cast(float, h2f_bits(m.sc[t] & 0xffffu));
        s16 = 16.f * sf;
        cz = -(16.f + (float)((m.zz[t] >> (4 * (r & 1))) & 15u)) * sf;
      }
      const u32 sb = f2h_bits(s16), cb = f2h_bits(cz);
      s2[t] = sb | (sb << 16);
      c2[t] = cb | (cb << 16);
    }
  };
  auto compute2 = [&](int st, const u32x4_t(&wq)[4], const u32 (&s2)[4], const u32 (&z2)[4], int j0) {
    const uint16_t *A_ = As + st * PI_BM * PI_LDK + (32 * g + r) * PI_LDK + 32 * qd;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int j = j0 + jj;
      f16x8_t wd[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) wd[t] = deq8_f16(wq[t][j], s2[t], z2[t], dqc);
#pragma unroll
      for (int tb = 0; tb < 2 * NBW; ++tb) {
        const f16x8_t xa = *(const f16x8_t *)(A_ + (64 * (tb >> 1) + 16 * (tb & 1)) * PI_LDK + 8 * j);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t][tb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, wd[t], acc[t][tb], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto step = [&](int gi, const u32x4_t(&cur)[4], const PiMeta &mc, u32x4_t(&nxt)[4], PiMeta &mn) {
    const bool more = gi + 1 < G;
    // unconditional requests (the last group asks for itself once more), pinned in front of the products: with
    // loads under conditions the compiler's waits for the current tiles also wait for the ones just requested
    const int gn = more ? gi + 1 : gi;
    gloadA(gn, 0);
    if (NBW > 0) gloadW(nxt, mn, gn);
    __builtin_amdgcn_sched_barrier(0);
    u32 s2[4], c2[4];
    if (NBW > 0) prep(mc, s2, c2);
    if (NBW > 0) compute2(gi & 1, cur, s2, c2, 0);
    if (more) sstore((gi + 1) & 1, 0);
    gloadA(gn, 1);
    __builtin_amdgcn_sched_barrier(0);
    if (NBW > 0) compute2(gi & 1, cur, s2, c2, 2);
    if (more) {
      if (nb > 3) sstore((gi + 1) & 1, 1);
      __syncthreads();
    }
  };
  gloadA(0, 0);
  if (NBW > 0) gloadW(wA, mA, 0);
  sstore(0, 0);
  if (nb > 3) {
    gloadA(0, 1);
    sstore(0, 1);
  }
  __syncthreads();
  for (int gi = 0; gi < G; gi += 2) {
    step(gi, wA, mA, wB, mB);
    if (gi + 1 < G) step(gi + 1, wB, mB, wA, mA);
  }
}

template <bool SWIGLU, bool Q4K, bool ACT16>
__global__ __launch_bounds__(512, 1) void k_prefill_int4(const PfArgs a) {
  extern __shared__ __align__(16) uint16_t As[];  // [2][PI_BM][PI_LDK] fp16
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane((tid >> 6) & 3), g = tid >> 8;
  const int r = lane & 15, qd = lane >> 4;

  // block order: as in k_prefill_gemm
  int ci, pb;
  pf_block_of(a, ci, pb);
  const PfClass &c = a.c[ci];
  const int n_mt = *c.n_tiles_real;
  // a class whose reduction is split has ksplit workgroups per tile: the pieces of one tile are `n_tiles`
  // blocks apart, so that the first piece of every tile starts before the second of any
  const int ks = c.ksplit > 1 ? c.ksplit : 1;
  const int n_tiles = n_mt * c.n_ntiles;
  const int n_real = n_tiles * ks;
  const int per_xcd = (n_real + 7) >> 3;
  if ((pb >> 3) >= per_xcd) return;
  int bid = (pb & 7) * per_xcd + (pb >> 3);
  if (bid >= n_real) return;
  const int split = bid / n_tiles;
  bid -= split * n_tiles;
  int mt, nt;
  if (c.m_fastest) { nt = bid / n_mt; mt = bid - nt * n_mt; }
  else { mt = bid / c.n_ntiles; nt = bid - mt * c.n_ntiles; }
  const PfTile tile = c.tiles[mt];
  if (tile.rows <= 0) return;
  const int K = c.K, G = K >> 7;
  // this workgroup's window of quantisation groups (only the w2 pass is ever split: a constant 0 in the w13 pass)
  const int Gw = SWIGLU ? G : G / ks, g0 = SWIGLU ? 0 : split * Gw;

  const int ch = tid & 15, r0 = tid >> 4;
  u32 a_off[6];  // byte offsets into the activation matrix (< 2^31: checked by the launcher)
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    int row = r0 + 32 * i;
    row = row < tile.rows ? row : 0;  // rows past the group's end re-read row 0 (never stored)
    const int grow = tile.row0 + row;
    const int arow = c.gather ? c.gather[grow] : grow;
    a_off[i] = ((u32)arow * (u32)c.act_stride + ch * 8) * 2;
  }
  // the wave's 4 consecutive 16-row blocks: (gate, up, gate, up) of two 16-column blocks of
  // h in the w13 pass, 64 consecutive output columns in the w2 pass
  const int rb0 = 16 * nt + 4 * w;
  const unsigned char *base = pf_uniform((const unsigned char *)tile.w_base);
  const rsrc_t rq = pf_rsrc(base + c.w_off + (size_t)rb0 * G * 1024, 4u * G * 1024u);
  const rsrc_t rs = pf_rsrc(base + c.off_s + (size_t)rb0 * G * (Q4K ? 128 : 32), 4u * G * (Q4K ? 128u : 32u));
  const rsrc_t rz = pf_rsrc(base + c.off_z + (size_t)rb0 * G * (Q4K ? 32 : 8), 4u * G * (Q4K ? 32u : 8u));
  const rsrc_t rx = pf_rsrc(c.act, 0x7fffffffu);

  f32x4_t acc[4][6];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int tb = 0; tb < 6; ++tb) acc[t][tb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int nb = (tile.rows + 31) >> 5;
  const int nbw = (nb - g + 1) >> 1;
  switch (nbw) {
    case 0: pi_mainloop<0, Q4K, ACT16>(acc, As, rx, a_off, rq, rs, rz, G, g0, Gw, nb, tid); break;
    case 1: pi_mainloop<1, Q4K, ACT16>(acc, As, rx, a_off, rq, rs, rz, G, g0, Gw, nb, tid); break;
    case 2: pi_mainloop<2, Q4K, ACT16>(acc, As, rx, a_off, rq, rs, rz, G, g0, Gw, nb, tid); break;
    default: pi_mainloop<3, Q4K, ACT16>(acc, As, rx, a_off, rq, rs, rz, G, g0, Gw, nb, tid); break;
  }
  // epilogue.  acc[t][tb] element i of lane l: weight row r of tile t, token row
  // 32*(2*(tb/2)+g) + 16*(tb%2) + 4*qd + i of the tile
#pragma unroll
  for (int tb = 0; tb < 6; ++tb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 32 * (2 * (tb >> 1) + g) + 16 * (tb & 1) + 4 * qd + i;
      if (row < tile.rows) {
        const size_t orow = (size_t)(tile.row0 + row) * c.out_stride;
        if (SWIGLU) {
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            const float gt = acc[2 * b][tb][i], up = acc[2 * b + 1][tb][i];
            ((_Float16 *)c.out)[orow + 16 * (rb0 / 2 + b) + r] = (_Float16)pf_silu_mul(gt, up);  // h in fp16: what the w2 pass stages
          }
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) ((float *)c.out)[(size_t)split * c.split_stride + orow + 16 * (rb0 + t) + r] = acc[t][tb][i];
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

template <bool Q4K>
static int pi_launch(bool swiglu, bool x16, const PfArgs &a, hipStream_t s) {
  if (a.n_blocks_total <= 0) return MOE_OK;
  const int grid = ((a.c[0].n_blocks + 7) & ~7) + ((a.c[1].n_blocks + 7) & ~7);
  const size_t lds = (size_t)2 * PI_BM * PI_LDK * 2;
  static bool attr_set = false;
  if (!attr_set) {
    for (const void *f : {(const void *)k_prefill_int4<true, Q4K, false>, (const void *)k_prefill_int4<true, Q4K, true>,
                          (const void *)k_prefill_int4<false, Q4K, true>})
      if (int rc = moe_check_hip(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                                 "hipFuncSetAttribute(k_prefill_int4)"))
        return rc;
    attr_set = true;
  }
  moe_ktimer_begin(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  // the w2 pass reads the fp16 h rows of the w13 pass; the w13 pass reads bf16 x, or its fp16 copy when there is one
  if (swiglu && x16) hipLaunchKernelGGL((k_prefill_int4<true, Q4K, true>), dim3(grid), dim3(512), lds, s, a);
  else if (swiglu) hipLaunchKernelGGL((k_prefill_int4<true, Q4K, false>), dim3(grid), dim3(512), lds, s, a);
  else hipLaunchKernelGGL((k_prefill_int4<false, Q4K, true>), dim3(grid), dim3(512), lds, s, a);
  moe_ktimer_end(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  return moe_check_launch("k_prefill_int4");
}

static int pf_launch(bool swiglu, const PfArgs &a, hipStream_t s) {
  if (a.n_blocks_total <= 0) return MOE_OK;
  const int grid = ((a.c[0].n_blocks + 7) & ~7) + ((a.c[1].n_blocks + 7) & ~7);
  const size_t lds = (size_t)PF4_RING * PF4_SLAB * 2;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e1 = hipFuncSetAttribute((const void *)k_prefill_gemm<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipError_t e2 = hipFuncSetAttribute((const void *)k_prefill_gemm<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (int rc = moe_check_hip(e1 != hipSuccess ? e1 : e2, "hipFuncSetAttribute(k_prefill_gemm)")) return rc;
    attr_set = true;
  }
  moe_ktimer_begin(swiglu ? MOE_K_PREFILL_W13 : MOE_K_PREFILL_W2, s);
  if (swiglu) hipLaunchKernelGGL(k_prefill_gemm<true>, dim3(grid), dim3(256), lds, s, a);
  else hipLaunchKernelGGL(k_prefill_gemm<false>, dim3(grid), dim3(256), lds, s, a);
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
                                                        unsigned long long shared_base, int T, int cap, int cap_s, int cap_s2,
                                                        int *__restrict__ n_real, int *__restrict__ err) {
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
        else moe_raise_err(err);
      }
    }
    const int nt = (m + cap - 1) / cap;
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
    PfTile t; t.w_base = shared_base; t.row0 = i * cap_s; t.rows = min(cap_s, T - i * cap_s);
    sh_tiles[i] = t;
  }
  for (int i = tid; i < n_sh_tiles2; i += 1024) {
    PfTile t; t.w_base = shared_base; t.row0 = i * cap_s2; t.rows = min(cap_s2, T - i * cap_s2);
    sh_tiles2[i] = t;
  }
}

extern "C" int moe_prefill_tile_rows(void) { return PF_BM; }

extern "C" int64_t moe_prefill_workspace_bytes(int T, int k, int max_units) {
  const int64_t P = (int64_t)T * k;
  return (P / 128 + max_units + 2 * ((T + 127) / 128) + 3) * (int64_t)sizeof(PfTile);  // covers every tile height in use (>= 128)
}

// Pieces the w2 pass leaves the shared expert's partial rows in (moe_experts_prefill_pieces).  The shared expert's
// workgroups of that pass each reduce over all of I_sh; where there are few of them (ceil(T/128) row tiles x H/256
// column tiles) and the reduction is long, they outlast everything else in the launch: Qwen2-57B shape (H 3584,
// I_sh 20480) at 512 tokens, 56 workgroups over 160 groups each: 371 us for the launch, 285 us with the reduction in 4
// windows (8 windows: no shorter, and the combine reads twice the partial rows).  Then the reduction is cut into 2, 4
// or 8 windows of at least 32 groups, a workgroup per tile and window, until there are 192 of them.
extern "C" int moe_prefill_shared_splits(int fmt, int T, int H, int I_sh) {
  if ((fmt != MOE_FMT_INT4_G128 && fmt != MOE_FMT_Q4K) || T <= 0 || H <= 0 || I_sh <= 0) return 1;
  const int tiles = ((T + PF_BM_SHARED_W2 - 1) / PF_BM_SHARED_W2) * (H / (2 * PF_BNH));
  const int G = I_sh / 128;
  int s = 1;
  while (s < 8 && tiles * s < 192 && G % (s * 4) == 0 && G / (s * 2) >= 32) s *= 2;
  return s;
}

extern "C" int moe_experts_prefill(const void *x_bf16, int T, int H, int I, int I_sh, int k, int fmt,
                                   const moe_unit *units, int max_units, const int *sorted_tok,
                                   const uint64_t *expert_ptr, const void *shared_ptr, void *h_r, void *h_s,
                                   float *part_r, float *part_s, void *tiles_ws, int *err, int phases,
                                   void *stream) {
  return moe_experts_prefill_pieces(x_bf16, T, H, I, I_sh, k, fmt, units, max_units, sorted_tok, expert_ptr, shared_ptr,
                                    h_r, h_s, part_r, part_s, 1, tiles_ws, err, phases, stream);
}

extern "C" int moe_experts_prefill_pieces(const void *x_bf16, int T, int H, int I, int I_sh, int k, int fmt,
                                          const moe_unit *units, int max_units, const int *sorted_tok,
                                          const uint64_t *expert_ptr, const void *shared_ptr, void *h_r, void *h_s,
                                          float *part_r, float *part_s, int shared_pieces, void *tiles_ws, int *err,
                                          int phases, void *stream) {
  hipStream_t s = (hipStream_t)stream;
  if (T == 0) return MOE_OK;
  if (shared_pieces != 1 && shared_pieces != 2 && shared_pieces != 4 && shared_pieces != 8) {
    moe_set_error("moe_experts_prefill: shared_pieces = %d (1, 2, 4 or 8)", shared_pieces);
    return MOE_EINVAL;
  }
  if (shared_pieces > 1 && (!shared_ptr || (fmt != MOE_FMT_INT4_G128 && fmt != MOE_FMT_Q4K) ||
                            (I_sh / 128) % (shared_pieces * 2) != 0)) {
    moe_set_error("moe_experts_prefill: %d pieces need an int4 / q4_K shared expert whose I_sh / 128 is a multiple of %d "
                  "(I_sh=%d)", shared_pieces, shared_pieces * 2, I_sh);
    return MOE_EINVAL;
  }
  if (!x_bf16 || T < 0 || k <= 0 || max_units < 0 || !units || !sorted_tok || !expert_ptr || !tiles_ws || !err ||
      !h_r || !part_r || (shared_ptr && (!h_s || !part_s || I_sh <= 0))) {
    moe_set_error("moe_experts_prefill: NULL or negative argument");
    return MOE_EINVAL;
  }
  if (fmt != MOE_FMT_BF16 && fmt != MOE_FMT_INT4_G128 && fmt != MOE_FMT_Q4K) {
    moe_set_error("moe_experts_prefill: weight format %d not supported by the prefill kernels", fmt);
    return MOE_EINVAL;
  }
  const bool q4k = fmt == MOE_FMT_Q4K;
  const bool int4 = fmt == MOE_FMT_INT4_G128 || q4k;  // nibble tiles + fp16 operands
  if (q4k && (H % 256 || I % 256 || (shared_ptr && I_sh % 256))) {
    moe_set_error("moe_experts_prefill: q4_K experts need H, I multiples of 256 (H=%d I=%d I_sh=%d)", H, I, I_sh);
    return MOE_EINVAL;
  }
  {
    const long long widest = I > H ? I : H, rows = (long long)T * (k > 1 ? k : 1);
    if (rows * widest * 2 >= (1ll << 31) || (shared_ptr && (long long)T * (I_sh > H ? I_sh : H) * 2 >= (1ll << 31))) {
      moe_set_error("moe_experts_prefill: activation buffers of 2 GiB or more are not supported (T=%d k=%d)", T, k);
      return MOE_EINVAL;
    }
  }
  if (H % 256 || I % 128 || (shared_ptr && I_sh % 128)) {
    moe_set_error("moe_experts_prefill: H %% 256 == 0 and I %% 128 == 0 required (H=%d I=%d I_sh=%d)", H, I, I_sh);
    return MOE_EINVAL;
  }
  const long long P = (long long)T * k;
  const int cap = int4 ? PI_BM : PF_BM, cap_s = int4 ? PI_BM : PF_BM_SHARED, cap_s2 = PF_BM_SHARED_W2;
  const int n_r = (int)(P / cap) + max_units;
  const int n_s = shared_ptr ? (T + cap_s - 1) / cap_s : 0;
  const int n_s2 = shared_ptr ? (T + cap_s2 - 1) / cap_s2 : 0;
  int *n_real = (int *)tiles_ws;  // [0] routed tiles in use, [1] shared tiles (w13 pass), [2] shared tiles (w2 pass)
  PfTile *tiles = (PfTile *)tiles_ws + 1, *sh_tiles = tiles + n_r, *sh_tiles2 = sh_tiles + n_s;
  hipLaunchKernelGGL(k_prefill_tiles, dim3(1), dim3(1024), 0, s, units, max_units,
                     (const unsigned long long *)expert_ptr, tiles, n_r, sh_tiles, n_s, sh_tiles2, n_s2,
                     (unsigned long long)(uintptr_t)shared_ptr, T, cap, cap_s, cap_s2, n_real, err);
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
      if (int4) {
        moe_int4_layout lay;
        if (int rc = q4k ? moe_q4k_layout_make(H, Ii, &lay) : moe_int4_layout_make(H, Ii, &lay)) return rc;
        c.w_off = w2 ? lay.off2_q : lay.off13_q;
        c.off_s = w2 ? lay.off2_s : lay.off13_s;
        c.off_z = w2 ? lay.off2_z : lay.off13_z;
      }
      c.ksplit = (w2 && shared && int4) ? shared_pieces : 1;
      c.split_stride = (long long)T * H;
      c.n_blocks = c.n_mtiles * c.n_ntiles * c.ksplit;
      c.slab_step = pf_slab_step(c.K / PF_BK);
      a.n_blocks_total += c.n_blocks;
    }
    if (int rc = q4k ? pi_launch<true>(!w2, false, a, s) : (int4 ? pi_launch<false>(!w2, false, a, s) : pf_launch(!w2, a, s))) return rc;
  }
  return MOE_OK;
}
