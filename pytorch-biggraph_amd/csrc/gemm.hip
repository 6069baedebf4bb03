// Batched fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_16x16x4_f32).
//
// C[b] = alpha * A[b] * B[b] + beta * C[b] for small and medium matrices, many
// per launch: the chunked score matrices S = A * N^T, their backward products
// dA = dS * N and dN = dS^T * A, and the `linear` operator.  One workgroup of
// four 64-lane waves (2 x 2) owns a BM x BN tile of C; A and B tiles of depth 16
// are staged through LDS, double buffered with register prefetch of the next
// tile.  An MFMA step contracts 4 values of k, one per group of 16 lanes; group
// g takes k = 4 g + step, so that the 4 values a lane needs over the 4 steps of
// a tile are adjacent in k.  An operand whose k axis is contiguous in memory is
// kept as tile[r][k] and a lane fetches its 4 values with one 128-bit LDS read;
// an operand whose other axis is contiguous is kept as tile[k][r].  All operand
// values of a depth-16 tile are read into registers before the 64 MFMAs of the
// tile, which then issue back to back.
//
// HALF variants (config.half_precision: both operands hold float16 numbers): the same
// tiles and the same lanes' values, converted to fp16 in registers (exactly) after the LDS
// read and contracted by ONE v_mfma_f32_16x16x16_f16 per depth-16 tile instead of four
// fp32 steps: lane group g holds k = 4 g .. 4 g + 3 in both layouts.  Sums stay fp32; the
// result is rounded to a float16 number when it is stored.
#include "pbg_internal.h"

namespace pbg {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

// acc[i][j] += A-tile i (rows) x B-tile j (columns) over the 16 values of k the lanes hold in fa / fb
template <bool HALF, int TM, int TN>
__device__ __forceinline__ void tile_products(const float4v (&fa)[TM], const float4v (&fb)[TN], float4v (&acc)[TM][TN]) {
  if constexpr (HALF) {
    half4v ha[TM], hb[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) ha[i] = (half4v){(_Float16)fa[i][0], (_Float16)fa[i][1], (_Float16)fa[i][2], (_Float16)fa[i][3]};
#pragma unroll
    for (int j = 0; j < TN; ++j) hb[j] = (half4v){(_Float16)fb[j][0], (_Float16)fb[j][1], (_Float16)fb[j][2], (_Float16)fb[j][3]};
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x16f16(ha[i], hb[j], acc[i][j], 0, 0, 0);
  } else {
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
  }
}

constexpr int kGemmThreads = 256;
constexpr int BK = 16;
constexpr int kFoldTiles = 8;  // depth-16 tiles per partial sum (128 values of k)

struct Quad {
  float v[4];
};

// Four consecutive floats starting at p; only the first `count` are in bounds.
__device__ __forceinline__ Quad load_quad(const float* __restrict__ p, int count, bool vec_ok) {
  Quad q;
  if (count >= 4 && vec_ok) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    q.v[0] = x.x; q.v[1] = x.y; q.v[2] = x.z; q.v[3] = x.w;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) q.v[i] = (i < count) ? p[i] : 0.f;
  }
  return q;
}

// Stages one operand tile.  ROWS = BM (for A) or BN (for B); the tile covers
// rows [r0, r0 + ROWS) of the operand's non-contracted axis and k in [k0, k0+BK).
//   KMAJOR = false: element (r, k) at base[r * ld + k]   (k contiguous)
//   KMAJOR = true : element (r, k) at base[k * ld + r]   (r contiguous)
template <int ROWS, bool KMAJOR>
struct TileLoader {
  static constexpr int kQuads = ROWS / 64;
  // Row strides of 4 (mod 16) floats: the 16 lanes of a group read 16 rows of
  // tile[r][k] 128 bits each without sharing a bank, and the 4 k-rows of
  // tile[k][r] that the 4 groups read start 16 banks apart.
  static constexpr int kStride = KMAJOR ? ROWS + 4 : BK + 4;
  static constexpr int kTileFloats = KMAJOR ? BK * (ROWS + 4) : ROWS * (BK + 4);
  Quad regs[kQuads];

  // (r, k) of the first element of this thread's quad number `it`
  static __device__ __forceinline__ int quad_r(int it) {
    return KMAJOR ? ((threadIdx.x & 15) + 16 * it) * 4 : (threadIdx.x >> 2) + 64 * it;
  }
  static __device__ __forceinline__ int quad_k() { return KMAJOR ? (threadIdx.x >> 4) : (threadIdx.x & 3) << 2; }

  // A whole depth-16 tile inside [0, kmax), every quad 16-byte aligned.  Rows
  // past rmax are read from clamped addresses: they only feed C entries that
  // are never stored.  (KMAJOR needs rmax % 4 == 0 and rmax >= 4.)
  __device__ __forceinline__ void fetch_full(const float* __restrict__ base, int ld, int r0, int k0, int rmax) {
#pragma unroll
    for (int it = 0; it < kQuads; ++it) {
      const float* p;
      if (!KMAJOR) {
        const int gr = min(r0 + quad_r(it), rmax - 1);
        p = base + (int64_t)gr * ld + k0 + quad_k();
      } else {
        const int gr = min(r0 + quad_r(it), rmax - 4);
        p = base + (int64_t)(k0 + quad_k()) * ld + gr;
      }
      const float4 x = *reinterpret_cast<const float4*>(p);
      regs[it].v[0] = x.x; regs[it].v[1] = x.y; regs[it].v[2] = x.z; regs[it].v[3] = x.w;
    }
  }

  // Any tile: elements out of bounds read as zero.
  __device__ __forceinline__ void fetch_edge(const float* __restrict__ base, int ld, int r0, int k0, int rmax, int kmax,
                                             bool vec_ok) {
#pragma unroll
    for (int it = 0; it < kQuads; ++it) {
      const int gr = r0 + quad_r(it), gk = k0 + quad_k();
      if (!KMAJOR) {
        int count = (gr < rmax) ? (kmax - gk) : 0;
        count = count < 0 ? 0 : count;
        regs[it] = load_quad(base + (int64_t)(gr < rmax ? gr : 0) * ld + gk, count, vec_ok);
      } else {
        int count = (gk < kmax) ? (rmax - gr) : 0;
        count = count < 0 ? 0 : count;
        regs[it] = load_quad(base + (int64_t)(gk < kmax ? gk : 0) * ld + gr, count, vec_ok);
      }
    }
  }

  __device__ __forceinline__ void stash(float* __restrict__ tile) const {
#pragma unroll
    for (int it = 0; it < kQuads; ++it) {
      float* dst = KMAJOR ? &tile[quad_k() * kStride + quad_r(it)] : &tile[quad_r(it) * kStride + quad_k()];
      *reinterpret_cast<float4*>(dst) = make_float4(regs[it].v[0], regs[it].v[1], regs[it].v[2], regs[it].v[3]);
    }
  }

  // The lane's operand values for the 4 MFMA steps of the tile: row `r` of the
  // tile, k = 4 * group + step.
  static __device__ __forceinline__ float4v operand(const float* __restrict__ tile, int r, int group) {
    if (!KMAJOR) return *reinterpret_cast<const float4v*>(&tile[r * kStride + group * 4]);
    float4v f;
#pragma unroll
    for (int s = 0; s < 4; ++s) f[s] = tile[(group * 4 + s) * kStride + r];
    return f;
  }
};

template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, bool HALF>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_kernel(GemmArgs g, int a_vec, int b_vec) {
  constexpr int TM = BM / 2 / 16;  // MFMA tiles per wave along m
  constexpr int TN = BN / 2 / 16;
  using LoadA = TileLoader<BM, A_KMAJOR>;
  using LoadB = TileLoader<BN, B_KMAJOR>;
  __shared__ __attribute__((aligned(16))) float lds_a[2][LoadA::kTileFloats];
  __shared__ __attribute__((aligned(16))) float lds_b[2][LoadB::kTileFloats];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm0 = (wave >> 1) * (BM / 2);
  const int wn0 = (wave & 1) * (BN / 2);
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  const int nk = (g.k + BK - 1) / BK;
  const int nk_full = g.k / BK;
  const bool a_full = a_vec && (!A_KMAJOR || (g.m % 4 == 0 && g.m >= 4));
  const bool b_full = b_vec && (!B_KMAJOR || (g.n % 4 == 0 && g.n >= 4));

  for (int batch = blockIdx.z; batch < g.batch; batch += gridDim.z) {
    const float* __restrict__ a = g.a + (int64_t)batch * g.stride_a;
    const float* __restrict__ b =
        g.b + (int64_t)batch * g.stride_b + (g.b_index ? g.b_index[batch] * g.b_index_stride : 0);
    float* __restrict__ c = g.c + (int64_t)batch * g.stride_c;

    // Blocked summation: `acc` collects kFoldTiles depth-16 tiles, then is folded
    // into `tot`.  A single accumulator over k = 1000 is a sequential fp32 sum of
    // 250 partial products, whose rounding errors add up coherently when the terms
    // are alike (a power-law batch repeats the same rows); two levels keep the
    // error at that of a blocked CPU BLAS.
    float4v acc[TM][TN], tot[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
        tot[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
      }

    LoadA la;
    LoadB lb;
    auto fetch = [&](int kt) {
      if (a_full && kt < nk_full) la.fetch_full(a, g.lda, m0, kt * BK, g.m);
      else la.fetch_edge(a, g.lda, m0, kt * BK, g.m, g.k, a_vec);
      if (b_full && kt < nk_full) lb.fetch_full(b, g.ldb, n0, kt * BK, g.n);
      else lb.fetch_edge(b, g.ldb, n0, kt * BK, g.n, g.k, b_vec);
    };
    fetch(0);
    __syncthreads();  // previous batch iteration may still be reading LDS
    la.stash(lds_a[0]);
    lb.stash(lds_b[0]);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < nk) fetch(kt + 1);
      float4v fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = LoadA::operand(lds_a[cur], wm0 + i * 16 + (lane & 15), lane >> 4);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = LoadB::operand(lds_b[cur], wn0 + j * 16 + (lane & 15), lane >> 4);
      tile_products<HALF, TM, TN>(fa, fb, acc);
      if ((kt & (kFoldTiles - 1)) == kFoldTiles - 1) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            tot[i][j] += acc[i][j];
            acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
          }
      }
      if (kt + 1 < nk) {
        la.stash(lds_a[cur ^ 1]);
        lb.stash(lds_b[cur ^ 1]);
      }
      __syncthreads();
    }

    // D[i = 4 * (lane / 16) + r][j = lane % 16] lives in register r of the lane.
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn0 + j * 16 + (lane & 15);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = m0 + wm0 + i * 16 + 4 * (lane >> 4) + r;
          if (row < g.m && col < g.n) {
            float* dst = c + (int64_t)row * g.ldc + col;
            float v = g.alpha * (tot[i][j][r] + acc[i][j][r]);
            // HALF: the product is a Half tensor of its own before autograd adds it to what is there
            // (two roundings: of the product, then of the sum)
            if (g.beta != 0.f) v = (HALF ? (float)(_Float16)v : v) + g.beta * *dst;
            *dst = HALF ? (float)(_Float16)v : v;
          }
        }
      }
    }
  }
}

// ---- 128 x 128 tiles fed by direct global -> LDS loads -------------------------
//
// When every quad of both operands is 16-byte aligned, the tiles skip the
// registers: each lane of global_load_lds_dwordx4 names 16 bytes of global
// memory, and the wave's 64 quads land in 1 KiB of LDS in lane order.  Three
// LDS stages hold tiles kt, kt+1 and kt+2, so a tile has two tiles' worth of
// MFMA time to arrive, and no registers or LDS store instructions are spent on
// staging.  Bank conflicts are avoided by which quad a lane fetches rather than
// by padding: in tile[r][k] the 4 k-quads of row r are rotated by (r / 4) % 4,
// and in tile[k][r] the 32 r-quads of k-row k by 4 * ((k / 4) % 4).
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(1))) const void* global_void_ptr;

constexpr int kDmaTile = 128;
constexpr int kDmaStages = 3;
constexpr int kDmaTileFloats = kDmaTile * BK;

template <bool KMAJOR>
struct DmaTile {
  // This wave fetches 2 of the 8 KiB-sized pieces of a tile.  next[it] is the
  // lane's quad of piece 2 * wave + it in the next tile to fetch; rows past rmax
  // are fetched from clamped addresses (they only feed C entries that are never
  // stored).
  const float* next[2];
  int ld;

  __device__ __forceinline__ void start(const float* __restrict__ base, int ld_, int r0, int rmax, int wave,
                                        int lane) {
    ld = ld_;
#pragma unroll
    for (int it = 0; it < 2; ++it) next[it] = quad(base, ld_, r0, 0, rmax, 1 << 30, wave * 2 + it, lane);
  }

  static __device__ __forceinline__ const float* quad(const float* __restrict__ base, int ld, int r0, int k0,
                                                       int rmax, int kmax, int piece, int lane) {
    if (!KMAJOR) {
      const int r = piece * 16 + (lane >> 2);
      const int q = (lane & 3) ^ ((r >> 2) & 3);
      return base + (int64_t)min(r0 + r, rmax - 1) * ld + min(k0 + q * 4, kmax - 4);
    }
    const int k = piece * 2 + (lane >> 5);
    const int rq = (lane & 31) ^ (((k >> 2) & 3) << 2);
    return base + (int64_t)min(k0 + k, kmax - 1) * ld + min(r0 + rq * 4, rmax - 4);
  }

  // Issued as assembly: the compiler would make every later LDS read wait for
  // all outstanding loads of this kind, and the stages exist to avoid that.
  // The kernel orders them itself (PBG_WAIT_VMCNT, then a barrier).
  static __device__ __forceinline__ void load_to_lds(const float* p, float* lds_piece) {
    const unsigned lds_at = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lds_void_ptr)lds_piece);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_at), "v"(p) : "memory", "m0");
  }

  // Fetches the next tile, all 16 values of k inside the operand.
  __device__ __forceinline__ void issue(float* stage, int wave) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      load_to_lds(next[it], stage + (wave * 2 + it) * 256);
      next[it] += KMAJOR ? (int64_t)BK * ld : BK;
    }
  }

  // Fetches the last tile when k stops inside it: k past kmax is fetched from
  // clamped addresses too, and the caller zeroes those values in registers.
  static __device__ __forceinline__ void issue_tail(const float* __restrict__ base, int ld, int r0, int k0, int rmax,
                                                    int kmax, float* stage, int wave, int lane) {
#pragma unroll
    for (int it = 0; it < 2; ++it)
      load_to_lds(quad(base, ld, r0, k0, rmax, kmax, wave * 2 + it, lane), stage + (wave * 2 + it) * 256);
  }

  // The lane's operand values for the 4 MFMA steps of the tile: row r, k = 4 * group + step.
  static __device__ __forceinline__ float4v operand(const float* __restrict__ stage, int r, int group) {
    if (!KMAJOR) return *reinterpret_cast<const float4v*>(&stage[r * BK + ((group ^ ((r >> 2) & 3)) << 2)]);
    float4v f;
    const int col = ((((r >> 2) ^ (group << 2))) << 2) + (r & 3);
#pragma unroll
    for (int s = 0; s < 4; ++s) f[s] = stage[(group * 4 + s) * kDmaTile + col];
    return f;
  }
};

// s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt in
// bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at their maxima).
#define PBG_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

template <bool A_KMAJOR, bool B_KMAJOR, bool HALF>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_dma_kernel(GemmArgs g) {
  constexpr int TM = 4, TN = 4;
  __shared__ __attribute__((aligned(16))) float lds_a[kDmaStages][kDmaTileFloats];
  __shared__ __attribute__((aligned(16))) float lds_b[kDmaStages][kDmaTileFloats];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm0 = (wave >> 1) * 64;
  const int wn0 = (wave & 1) * 64;
  const int m0 = blockIdx.y * kDmaTile;
  const int n0 = blockIdx.x * kDmaTile;
  const int nk = (g.k + BK - 1) / BK;

  for (int batch = blockIdx.z; batch < g.batch; batch += gridDim.z) {
    const float* __restrict__ a = g.a + (int64_t)batch * g.stride_a;
    const float* __restrict__ b =
        g.b + (int64_t)batch * g.stride_b + (g.b_index ? g.b_index[batch] * g.b_index_stride : 0);
    float* __restrict__ c = g.c + (int64_t)batch * g.stride_c;

    float4v acc[TM][TN], tot[TM][TN];  // two-level sum, as in gemm_kernel
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
        tot[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
      }

    DmaTile<A_KMAJOR> da;
    DmaTile<B_KMAJOR> db;
    da.start(a, g.lda, m0, g.m, wave, lane);
    db.start(b, g.ldb, n0, g.n, wave, lane);
    auto issue = [&](int kt) {  // called for kt = 0, 1, 2, ... in order
      const int st = kt % kDmaStages;
      if (kt * BK + BK <= g.k) {
        da.issue(lds_a[st], wave);
        db.issue(lds_b[st], wave);
      } else {
        DmaTile<A_KMAJOR>::issue_tail(a, g.lda, m0, kt * BK, g.m, g.k, lds_a[st], wave, lane);
        DmaTile<B_KMAJOR>::issue_tail(b, g.ldb, n0, kt * BK, g.n, g.k, lds_b[st], wave, lane);
      }
    };
    // the previous product's stores have left, and all its LDS reads are done
    PBG_WAIT_VMCNT(0);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < kDmaStages - 1; ++t)
      if (t < nk) issue(t);

    for (int kt = 0; kt < nk; ++kt) {
      // tile kt has landed once only the loads of later tiles (4 each) are in flight
      const int later = min(kDmaStages - 2, nk - 1 - kt);
      if (later >= 2) PBG_WAIT_VMCNT(8);
      else if (later == 1) PBG_WAIT_VMCNT(4);
      else PBG_WAIT_VMCNT(0);
      __syncthreads();  // every wave's pieces of tile kt; stage of tile kt-1 is free
      const float* __restrict__ ta = lds_a[kt % kDmaStages];
      const float* __restrict__ tb = lds_b[kt % kDmaStages];
      float4v fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = DmaTile<A_KMAJOR>::operand(ta, wm0 + i * 16 + (lane & 15), lane >> 4);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = DmaTile<B_KMAJOR>::operand(tb, wn0 + j * 16 + (lane & 15), lane >> 4);
      if (kt + kDmaStages - 1 < nk) issue(kt + kDmaStages - 1);
      if (kt * BK + BK > g.k) {  // k tail: the clamped loads brought in values that are not part of the sum
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const bool live = kt * BK + 4 * (lane >> 4) + s < g.k;
#pragma unroll
          for (int i = 0; i < TM; ++i) fa[i][s] = live ? fa[i][s] : 0.f;
#pragma unroll
          for (int j = 0; j < TN; ++j) fb[j][s] = live ? fb[j][s] : 0.f;
        }
      }
      tile_products<HALF, TM, TN>(fa, fb, acc);
      if ((kt & (kFoldTiles - 1)) == kFoldTiles - 1) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            tot[i][j] += acc[i][j];
            acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
          }
      }
    }

    // The store addresses do not change from one product to the next; computed
    // from a value the compiler cannot see through, they are not kept in
    // registers across the k loop.
    int elane = lane;
    asm volatile("" : "+v"(elane));
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn0 + j * 16 + (elane & 15);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = m0 + wm0 + i * 16 + 4 * (elane >> 4) + r;
          if (row < g.m && col < g.n) {
            float* dst = c + (int64_t)row * g.ldc + col;
            float v = g.alpha * (tot[i][j][r] + acc[i][j][r]);
            // HALF: the product is a Half tensor of its own before autograd adds it to what is there
            // (two roundings: of the product, then of the sum)
            if (g.beta != 0.f) v = (HALF ? (float)(_Float16)v : v) + g.beta * *dst;
            *dst = HALF ? (float)(_Float16)v : v;
          }
        }
      }
    }
  }
}

template <bool HALF>
void launch_dma(const GemmArgs& g, hipStream_t stream) {
  dim3 grid((unsigned)ceil_div(g.n, kDmaTile), (unsigned)ceil_div(g.m, kDmaTile),
            (unsigned)(g.batch < 65535 ? g.batch : 65535));
  dim3 block(kGemmThreads);
  if (!g.a_kmajor && !g.b_kmajor)
    hipLaunchKernelGGL((gemm_dma_kernel<false, false, HALF>), grid, block, 0, stream, g);
  else if (!g.a_kmajor && g.b_kmajor)
    hipLaunchKernelGGL((gemm_dma_kernel<false, true, HALF>), grid, block, 0, stream, g);
  else if (g.a_kmajor && !g.b_kmajor)
    hipLaunchKernelGGL((gemm_dma_kernel<true, false, HALF>), grid, block, 0, stream, g);
  else
    hipLaunchKernelGGL((gemm_dma_kernel<true, true, HALF>), grid, block, 0, stream, g);
}

template <int BM, int BN, bool HALF>
void launch(const GemmArgs& g, int a_vec, int b_vec, hipStream_t stream) {
  dim3 grid((unsigned)ceil_div(g.n, BN), (unsigned)ceil_div(g.m, BM), (unsigned)(g.batch < 65535 ? g.batch : 65535));
  dim3 block(kGemmThreads);
  if (!g.a_kmajor && !g.b_kmajor)
    hipLaunchKernelGGL((gemm_kernel<BM, BN, false, false, HALF>), grid, block, 0, stream, g, a_vec, b_vec);
  else if (!g.a_kmajor && g.b_kmajor)
    hipLaunchKernelGGL((gemm_kernel<BM, BN, false, true, HALF>), grid, block, 0, stream, g, a_vec, b_vec);
  else if (g.a_kmajor && !g.b_kmajor)
    hipLaunchKernelGGL((gemm_kernel<BM, BN, true, false, HALF>), grid, block, 0, stream, g, a_vec, b_vec);
  else
    hipLaunchKernelGGL((gemm_kernel<BM, BN, true, true, HALF>), grid, block, 0, stream, g, a_vec, b_vec);
}

bool quad_aligned(const float* p, int ld, int64_t stride) {
  return ((uintptr_t)p % 16 == 0) && (ld % 4 == 0) && (stride % 4 == 0);
}

}  // namespace

int gemm_f32(const GemmArgs& g, hipStream_t stream) {
  if (g.batch <= 0 || g.m <= 0 || g.n <= 0) return PBG_OK;
  if (g.k < 0) return fail(PBG_ERR_INVALID, "gemm_f32: negative k");
  const int a_vec = quad_aligned(g.a, g.lda, g.stride_a);
  const int b_vec = quad_aligned(g.b, g.ldb, g.stride_b) && (g.b_index_stride % 4 == 0);
  // clamped quads of the direct-to-LDS kernel stay inside the operand when
  // k, and the contiguous axis of a k-major operand, are multiples of 4
  const bool dma_ok = a_vec && b_vec && g.k % 4 == 0 && g.k >= BK && (!g.a_kmajor || (g.m % 4 == 0 && g.m >= 4)) &&
                      (!g.b_kmajor || (g.n % 4 == 0 && g.n >= 4));
  // (a product of at most 64 values of k is bound by writing its output: the smaller tile pads less)
  const bool small = g.m <= 96 || g.n <= 96 || (!dma_ok && g.k <= 64);
  if (g.half) {
    if (small) launch<64, 64, true>(g, a_vec, b_vec, stream);
    else if (dma_ok) launch_dma<true>(g, stream);
    else launch<128, 128, true>(g, a_vec, b_vec, stream);
  } else {
    if (small) launch<64, 64, false>(g, a_vec, b_vec, stream);
    else if (dma_ok) launch_dma<false>(g, stream);
    else launch<128, 128, false>(g, a_vec, b_vec, stream);
  }
  return check_launch("gemm_f32");
}

}  // namespace pbg

extern "C" int pbg_gemm_f32(const float* a, const float* b, float* c, int32_t batch, int32_t m, int32_t n, int32_t k,
                            int32_t lda, int32_t ldb, int32_t ldc, int64_t stride_a, int64_t stride_b,
                            int64_t stride_c, int32_t a_kmajor, int32_t b_kmajor, float alpha, float beta,
                            pbg_stream_t stream) {
  if (batch < 0 || m < 0 || n < 0 || k < 0) return pbg::fail(PBG_ERR_INVALID, "pbg_gemm_f32: negative size");
  if (batch == 0 || m == 0 || n == 0) return PBG_OK;
  if (!a || !b || !c) return pbg::fail(PBG_ERR_INVALID, "pbg_gemm_f32: null pointer");
  pbg::GemmArgs g{};
  g.a = a; g.b = b; g.c = c;
  g.stride_a = stride_a; g.stride_b = stride_b; g.stride_c = stride_c;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.m = m; g.n = n; g.k = k; g.batch = batch;
  g.a_kmajor = a_kmajor; g.b_kmajor = b_kmajor;
  g.alpha = alpha; g.beta = beta;
  return pbg::gemm_f32(g, (hipStream_t)stream);
}

extern "C" int pbg_gemm_f16(const float* a, const float* b, float* c, int32_t batch, int32_t m, int32_t n, int32_t k,
                            int32_t lda, int32_t ldb, int32_t ldc, int64_t stride_a, int64_t stride_b,
                            int64_t stride_c, int32_t a_kmajor, int32_t b_kmajor, float alpha, float beta,
                            pbg_stream_t stream) {
  if (batch < 0 || m < 0 || n < 0 || k < 0) return pbg::fail(PBG_ERR_INVALID, "pbg_gemm_f16: negative size");
  if (batch == 0 || m == 0 || n == 0) return PBG_OK;
  if (!a || !b || !c) return pbg::fail(PBG_ERR_INVALID, "pbg_gemm_f16: null pointer");
  pbg::GemmArgs g{};
  g.a = a; g.b = b; g.c = c;
  g.stride_a = stride_a; g.stride_b = stride_b; g.stride_c = stride_c;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.m = m; g.n = n; g.k = k; g.batch = batch;
  g.a_kmajor = a_kmajor; g.b_kmajor = b_kmajor;
  g.alpha = alpha; g.beta = beta;
  g.half = 1;
  return pbg::gemm_f32(g, (hipStream_t)stream);
}
