// Batched fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_16x16x4_f32).
//
// C[b] = alpha * A[b] * B[b] + beta * C[b] for small and medium matrices, many
// per launch: the chunked score matrices S = A * N^T, their backward products
// dA = dS * N and dN = dS^T * A, and the `linear` operator.  One workgroup of
// four 64-lane waves (2 x 2) owns a BM x BN tile of C; A and B tiles of depth 16
// are staged through LDS in k-major layout (row stride = tile + 16 floats, which
// spreads the 4 k-rows a wave reads per MFMA over disjoint bank halves), double
// buffered with register prefetch of the next tile.
#include "pbg_internal.h"

namespace pbg {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kGemmThreads = 256;
constexpr int BK = 16;
constexpr int PAD = 16;
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
  static constexpr int kQuads = ROWS * BK / 4 / kGemmThreads;
  Quad regs[kQuads];

  __device__ __forceinline__ void fetch(const float* __restrict__ base, int ld, int r0, int k0, int rmax, int kmax,
                                        bool vec_ok) {
#pragma unroll
    for (int it = 0; it < kQuads; ++it) {
      const int idx = threadIdx.x + it * kGemmThreads;
      if (!KMAJOR) {
        const int r = idx >> 2, kq = (idx & 3) << 2;
        const int gr = r0 + r, gk = k0 + kq;
        int count = (gr < rmax) ? (kmax - gk) : 0;
        count = count < 0 ? 0 : count;
        regs[it] = load_quad(base + (int64_t)(gr < rmax ? gr : 0) * ld + gk, count, vec_ok);
      } else {
        constexpr int QPR = ROWS / 4;  // quads per k-row
        const int k = idx / QPR, rq = (idx % QPR) << 2;
        const int gk = k0 + k, gr = r0 + rq;
        int count = (gk < kmax) ? (rmax - gr) : 0;
        count = count < 0 ? 0 : count;
        regs[it] = load_quad(base + (int64_t)(gk < kmax ? gk : 0) * ld + gr, count, vec_ok);
      }
    }
  }

  // LDS tile layout: tile[k][r], row stride ROWS + PAD.
  __device__ __forceinline__ void stash(float* __restrict__ tile) const {
#pragma unroll
    for (int it = 0; it < kQuads; ++it) {
      const int idx = threadIdx.x + it * kGemmThreads;
      if (!KMAJOR) {
        const int r = idx >> 2, kq = (idx & 3) << 2;
#pragma unroll
        for (int i = 0; i < 4; ++i) tile[(kq + i) * (ROWS + PAD) + r] = regs[it].v[i];
      } else {
        constexpr int QPR = ROWS / 4;
        const int k = idx / QPR, rq = (idx % QPR) << 2;
        *reinterpret_cast<float4*>(&tile[k * (ROWS + PAD) + rq]) =
            make_float4(regs[it].v[0], regs[it].v[1], regs[it].v[2], regs[it].v[3]);
      }
    }
  }
};

template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_kernel(GemmArgs g, int a_vec, int b_vec) {
  constexpr int TM = BM / 2 / 16;  // MFMA tiles per wave along m
  constexpr int TN = BN / 2 / 16;
  __shared__ __attribute__((aligned(16))) float lds_a[2][BK * (BM + PAD)];
  __shared__ __attribute__((aligned(16))) float lds_b[2][BK * (BN + PAD)];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm0 = (wave >> 1) * (BM / 2);
  const int wn0 = (wave & 1) * (BN / 2);
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  const int nk = (g.k + BK - 1) / BK;

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

    TileLoader<BM, A_KMAJOR> la;
    TileLoader<BN, B_KMAJOR> lb;
    la.fetch(a, g.lda, m0, 0, g.m, g.k, a_vec);
    lb.fetch(b, g.ldb, n0, 0, g.n, g.k, b_vec);
    __syncthreads();  // previous batch iteration may still be reading LDS
    la.stash(lds_a[0]);
    lb.stash(lds_b[0]);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < nk) {
        la.fetch(a, g.lda, m0, (kt + 1) * BK, g.m, g.k, a_vec);
        lb.fetch(b, g.ldb, n0, (kt + 1) * BK, g.n, g.k, b_vec);
      }
      const float* __restrict__ ta = lds_a[cur];
      const float* __restrict__ tb = lds_b[cur];
#pragma unroll
      for (int kk = 0; kk < BK / 4; ++kk) {
        const int krow = kk * 4 + (lane >> 4);
        float fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = ta[krow * (BM + PAD) + wm0 + i * 16 + (lane & 15)];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = tb[krow * (BN + PAD) + wn0 + j * 16 + (lane & 15)];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
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
            if (g.beta != 0.f) v += g.beta * *dst;
            *dst = v;
          }
        }
      }
    }
  }
}

template <int BM, int BN>
void launch(const GemmArgs& g, int a_vec, int b_vec, hipStream_t stream) {
  dim3 grid((unsigned)ceil_div(g.n, BN), (unsigned)ceil_div(g.m, BM), (unsigned)(g.batch < 65535 ? g.batch : 65535));
  dim3 block(kGemmThreads);
  if (!g.a_kmajor && !g.b_kmajor)
    hipLaunchKernelGGL((gemm_kernel<BM, BN, false, false>), grid, block, 0, stream, g, a_vec, b_vec);
  else if (!g.a_kmajor && g.b_kmajor)
    hipLaunchKernelGGL((gemm_kernel<BM, BN, false, true>), grid, block, 0, stream, g, a_vec, b_vec);
  else if (g.a_kmajor && !g.b_kmajor)
    hipLaunchKernelGGL((gemm_kernel<BM, BN, true, false>), grid, block, 0, stream, g, a_vec, b_vec);
  else
    hipLaunchKernelGGL((gemm_kernel<BM, BN, true, true>), grid, block, 0, stream, g, a_vec, b_vec);
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
  if (g.m <= 96 || g.n <= 96) {
    launch<64, 64>(g, a_vec, b_vec, stream);
  } else {
    launch<128, 128>(g, a_vec, b_vec, stream);
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
