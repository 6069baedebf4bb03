// The `linear` operator with one relation per edge (LinearDynamicOperator,
// operators.py:252-269) on the matrix cores.
//
// The reference gathers W[rel] into a [B, D, D] tensor and multiplies row by
// row.  Here the edges of a call are sorted by (relation, batch) once; all
// edges of one relation then share one D x D operand and the products become
// GEMMs over segments of the sorted order:
//
//   seg_linear_apply   out[e] (+)= W[rel_e] x_e  or  W[rel_e]^T x_e.  A workgroup
//                      owns 64 consecutive sorted positions x 64 output columns.
//                      Positions of several relations may share a tile: the tile
//                      is swept once per relation present in it, with the rows of
//                      the other relations zeroed in the A operand, into the
//                      same accumulators.
//   seg_linear_update  dW[r] = sum over a (relation, batch) run of dz_e (x) x_e,
//                      followed by AsyncAdagrad (async_adagrad.py:75-85), run
//                      after run in batch order.  A workgroup owns one 64 x 64
//                      tile of one relation's matrix and keeps it (and its
//                      Adagrad sum) in registers over all the relation's runs.
//                      A relation with many edges in the call would make that
//                      one long chain of dependent steps: the gradients of its
//                      runs do not depend on one another, so other workgroups
//                      compute them first (one per run, or per part of a run)
//                      and the relation's workgroup only adds them up and takes
//                      the Adagrad steps.
//
// Both use v_mfma_f32_16x16x4_f32 with depth-16 tiles staged through LDS
// (k-major, row stride 80 floats), double buffered.
#include "pbg_internal.h"

#include <algorithm>

namespace pbg {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int BM = 64, BN = 64, BK = 16, LD = 80;
constexpr int kFoldTiles = 8;  // depth-16 tiles per partial sum, see gemm.hip

struct Quad {
  float v[4];
};

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

__device__ __forceinline__ int clamp_count(int c) { return c < 0 ? 0 : (c > 4 ? 4 : c); }

// first index in [lo, hi) whose key is >= want (hi if none)
__device__ __forceinline__ int64_t lower_bound(const uint64_t* __restrict__ keys, int64_t lo, int64_t hi, uint64_t want) {
  while (lo < hi) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if (keys[mid] < want) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// one depth-16 step of a 64 x 64 tile: wave (wm0, wn0) owns 32 x 32
__device__ __forceinline__ void mfma_tile(const float* __restrict__ ta, const float* __restrict__ tb, int wm0, int wn0,
                                          int lane, float4v (&acc)[2][2]) {
#pragma unroll
  for (int kk = 0; kk < BK / 4; ++kk) {
    const int krow = kk * 4 + (lane >> 4);
    float fa[2], fb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[i] = ta[krow * LD + wm0 + i * 16 + (lane & 15)];
#pragma unroll
    for (int j = 0; j < 2; ++j) fb[j] = tb[krow * LD + wn0 + j * 16 + (lane & 15)];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
  }
}

// Row of the [batches, rows_per_batch, dim] array `base` that belongs to edge e = k * B + q.
__device__ __forceinline__ int64_t edge_row(uint32_t e, int edges_per_batch, int64_t batch_stride) {
  return (int64_t)(e / (uint32_t)edges_per_batch) * batch_stride + (e % (uint32_t)edges_per_batch);
}

// VEC: dim is a multiple of 4 and both operands are 16-byte aligned, so a quad is whole or absent: it is loaded
// without a branch from an address clamped into the operand and dropped afterwards (a load inside a branch makes
// everything behind the branch wait for ALL loads in flight, which would undo the prefetch below).
template <bool TRANS, bool VEC>
__global__ __launch_bounds__(kThreads) void seg_linear_apply_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, int64_t n, int kbits, int edges_per_batch,
    const float* __restrict__ in, int64_t in_batch_stride, const float* __restrict__ w, int dim,
    float* __restrict__ out, int64_t out_batch_stride, int accumulate) {
  constexpr int vec_ok = VEC;
  __shared__ __attribute__((aligned(16))) float lds_a[2][BK * LD];
  __shared__ __attribute__((aligned(16))) float lds_b[2][BK * LD];
  __shared__ int64_t rel_s[BM];
  __shared__ uint32_t edge_s[BM];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  const int64_t pos0 = (int64_t)blockIdx.x * BM;
  const int n0 = blockIdx.y * BN;
  const int cnt = (int)((n - pos0) < BM ? (n - pos0) : BM);
  if (tid < BM) {
    const bool ok = tid < cnt;
    rel_s[tid] = ok ? (int64_t)(keys[pos0 + tid] >> kbits) : -1;
    edge_s[tid] = ok ? vals[pos0 + tid] : 0u;
  }
  __syncthreads();

  // A operand: thread -> (row ar of the tile, 4 consecutive k)
  const int ar = tid >> 2, akq = (tid & 3) << 2;
  const float* arow = in + edge_row(edge_s[ar], edges_per_batch, in_batch_stride) * dim;
  // B operand of relation r: B(k, j) = W_r[j][k] (W x) or W_r[k][j] (W^T x)
  const int bj = TRANS ? ((tid & 15) << 2) : (tid >> 2);  // column (or first of 4 columns) of the tile
  const int bk = TRANS ? (tid >> 4) : ((tid & 3) << 2);   // k (or first of 4 k)

  float4v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};

  const int nk = (dim + BK - 1) / BK;
  int a = 0;
  while (a < cnt) {
    const int64_t rel = rel_s[a];
    int b = a + 1;
    while (b < cnt && rel_s[b] == rel) ++b;
    const float* wr = w + rel * (int64_t)dim * dim;
    const bool row_on = ar >= a && ar < b;
    const bool wave_on = a < wm0 + 32 && b > wm0;  // the wave's 32 rows meet [a, b)

    auto quad_or_zero = [&](const float* p, bool keep) {
      const float4 x = *reinterpret_cast<const float4*>(p);
      Quad q;
      q.v[0] = keep ? x.x : 0.f; q.v[1] = keep ? x.y : 0.f; q.v[2] = keep ? x.z : 0.f; q.v[3] = keep ? x.w : 0.f;
      return q;
    };
    auto fetch_a = [&](int k0) {
      if constexpr (VEC) return quad_or_zero(arow + min(k0 + akq, dim - 4), row_on && k0 + akq < dim);
      const int count = row_on ? clamp_count(dim - (k0 + akq)) : 0;
      return load_quad(arow + k0 + akq, count, vec_ok);
    };
    auto fetch_b = [&](int k0) {
      if constexpr (VEC) {
        const bool keep = k0 + bk < dim && n0 + bj < dim;
        if (TRANS) return quad_or_zero(wr + (int64_t)min(k0 + bk, dim - 1) * dim + min(n0 + bj, dim - 4), keep);
        return quad_or_zero(wr + (int64_t)min(n0 + bj, dim - 1) * dim + min(k0 + bk, dim - 4), keep);
      }
      if (TRANS) {
        const int count = (k0 + bk < dim) ? clamp_count(dim - (n0 + bj)) : 0;
        return load_quad(wr + (int64_t)(k0 + bk) * dim + n0 + bj, count, vec_ok);
      }
      const int count = (n0 + bj < dim) ? clamp_count(dim - (k0 + bk)) : 0;
      return load_quad(wr + (int64_t)(n0 + bj) * dim + k0 + bk, count, vec_ok);
    };
    auto stash = [&](int buf, const Quad& qa, const Quad& qb) {
#pragma unroll
      for (int i = 0; i < 4; ++i) lds_a[buf][(akq + i) * LD + ar] = qa.v[i];
      if (TRANS) {
        *reinterpret_cast<float4*>(&lds_b[buf][bk * LD + bj]) = make_float4(qb.v[0], qb.v[1], qb.v[2], qb.v[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_b[buf][(bk + i) * LD + bj] = qb.v[i];
      }
    };

    // operands travel two tiles ahead of the products (registers), one tile ahead sits in LDS
    Quad qa = fetch_a(0), qb = fetch_b(0);
    Quad ra = fetch_a(BK), rb = fetch_b(BK);  // (past the last tile: counts of zero, clamped addresses)
    __syncthreads();  // the previous sweep may still be reading LDS
    stash(0, qa, qb);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      qa = ra;
      qb = rb;
      if (VEC || kt + 2 < nk) {
        ra = fetch_a((kt + 2) * BK);
        rb = fetch_b((kt + 2) * BK);
      }
      if (wave_on) mfma_tile(lds_a[cur], lds_b[cur], wm0, wn0, lane, acc);
      if (kt + 1 < nk) stash(cur ^ 1, qa, qb);
      __syncthreads();
    }
    a = b;
  }

  // D[i = 4 * (lane / 16) + r][j = lane % 16] lives in register r of the lane
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = wm0 + i * 16 + 4 * (lane >> 4) + r;
      if (row >= cnt) continue;
      float* orow = out + edge_row(edge_s[row], edges_per_batch, out_batch_stride) * dim;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn0 + j * 16 + (lane & 15);
        if (col < dim) orow[col] = accumulate ? orow[col] + acc[i][j][r] : acc[i][j][r];
      }
    }
  }
}

// rel_start[r] = first sorted position whose relation is >= r, for r in [0, num_relations]
__global__ void rel_start_kernel(const uint64_t* __restrict__ keys, int64_t n, int kbits, int num_relations,
                                 uint32_t* __restrict__ rel_start) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r > num_relations) return;
  rel_start[r] = (uint32_t)lower_bound(keys, 0, n, (uint64_t)r << kbits);
}

constexpr uint32_t kNone = 0xffffffffu;

// rel_order: the relations by decreasing power of two of their edge count, so that
// the workgroups with the longest chains of steps are dispatched first (any order
// gives the same result; which of two relations of one size class comes first is
// left to the atomics).  A relation with at least hot_min edges is "hot": it gets
// a slot (hot_slot[r], hot_list[slot] = r, *hot_count slots in all; which slot is
// left to the atomics too, the set of hot relations is not).  One workgroup.
__global__ __launch_bounds__(1024) void rel_plan_kernel(const uint32_t* __restrict__ rel_start, int num_relations,
                                                        uint32_t hot_min, uint32_t* __restrict__ rel_order,
                                                        uint32_t* __restrict__ hot_slot,
                                                        uint32_t* __restrict__ hot_count,
                                                        uint32_t* __restrict__ hot_list) {
  __shared__ unsigned count[34], base[34], nhot;
  const int t = threadIdx.x;
  if (t < 34) count[t] = 0u;
  if (t == 0) nhot = 0u;
  __syncthreads();
  auto size_class = [&](uint32_t c) { return c == 0u ? 33 : __clz((int)c); };  // 0 for the largest counts
  for (int r = t; r < num_relations; r += 1024) {
    const uint32_t c = rel_start[r + 1] - rel_start[r];
    atomicAdd(&count[size_class(c)], 1u);
    uint32_t slot = kNone;
    if (c >= hot_min) {
      slot = atomicAdd(&nhot, 1u);
      hot_list[slot] = (uint32_t)r;
    }
    hot_slot[r] = slot;
  }
  __syncthreads();
  if (t == 0) {
    unsigned run = 0u;
    for (int b = 0; b < 34; ++b) {
      base[b] = run;
      run += count[b];
    }
    *hot_count = nhot;
  }
  __syncthreads();
  for (int r = t; r < num_relations; r += 1024)
    rel_order[atomicAdd(&base[size_class(rel_start[r + 1] - rel_start[r])], 1u)] = (uint32_t)r;
}

// run_start[slot * (num_batches + 1) + b]: first sorted position of the run (hot_list[slot], batch b);
// entry num_batches is the end of the relation.
__global__ void run_start_kernel(const uint64_t* __restrict__ keys, const uint32_t* __restrict__ rel_start, int kbits,
                                 int num_batches, const uint32_t* __restrict__ hot_count,
                                 const uint32_t* __restrict__ hot_list, uint32_t* __restrict__ run_start) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t slot = i / (num_batches + 1);
  const int b = (int)(i % (num_batches + 1));
  if (slot >= (int64_t)*hot_count) return;
  const uint64_t rel = hot_list[slot];
  const int64_t lo = rel_start[rel], hi = rel_start[rel + 1];
  run_start[i] = (uint32_t)(b == num_batches ? hi : lower_bound(keys, lo, hi, (rel << kbits) | (uint64_t)b));
}

// Where the gradient tiles of the hot relations' runs are, and how the relations are walked.
struct HotRuns {
  const uint32_t* rel_order;  // [num_relations]
  const uint32_t* hot_slot;   // [num_relations], kNone: not hot
  const uint32_t* hot_count;  // [1]
  const uint32_t* hot_list;   // [*hot_count]
  const uint32_t* run_start;  // [*hot_count][num_batches + 1]
  float* part;                // null: no relation is hot
  int num_batches, splits;
};

// A workgroup streams ALL edges of its relation, kStage sorted positions per
// step, whatever batch they belong to; the rows of step s + 1 are requested
// before the products of step s and written to LDS after them.  A step that
// holds edges of several batches is swept once per batch with the other
// batches' rows masked in the A operand; whenever the batch changes, the
// finished batch's gradient tile gets its Adagrad step and the accumulators
// start over.  The kernel is kept small on purpose (dynamic loops, one copy of
// every phase): most workgroups live for a few steps only, and code that does
// not stay in the instruction cache is paid for by each of them.
//
// RUNS = false, grid (relation in rel_order, tile): as above; for a hot relation
// the gradient tiles of its runs are read from `part` instead of being computed.
// RUNS = true, grid ((slot * num_batches + batch) * splits + split, tile): the
// gradient tile of one part of one run of a hot relation, streamed the same way
// and written to part[(blockIdx.x * tiles^2 + tile) * 256 + thread][16] in the
// MFMA result layout.
constexpr int kStage = 32;  // edges per step

template <bool VEC, bool RUNS>
__global__ __launch_bounds__(kThreads, 4) void seg_linear_update_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, const uint32_t* __restrict__ rel_start,
    int kbits, const float* __restrict__ dz, const float* __restrict__ x, int dim, float* __restrict__ w,
    float* __restrict__ wsum, float lr, HotRuns hot) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][kStage * LD];
  __shared__ __attribute__((aligned(16))) float lds_b[2][kStage * LD];
  // (the batch of a staged edge sits in the padding of its row of lds_a, column BM: with an array of its own
  // the kernel's LDS would be 256 bytes above a quarter of the compute unit's)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  const int tiles = (dim + BN - 1) / BN;
  const int o0 = (blockIdx.y / tiles) * BM, i0 = (blockIdx.y % tiles) * BN;
  uint64_t rel;
  int64_t lo, hi;
  float4v* part_out = nullptr;
  if (RUNS) {
    const int per_slot = hot.num_batches * hot.splits;
    const uint32_t slot = blockIdx.x / per_slot;
    if (slot >= *hot.hot_count) return;
    const int batch = (blockIdx.x % per_slot) / hot.splits, split = blockIdx.x % hot.splits;
    rel = hot.hot_list[slot];
    const uint32_t* rs = hot.run_start + (int64_t)slot * (hot.num_batches + 1) + batch;
    const int64_t run_lo = rs[0], len = (int64_t)rs[1] - run_lo;
    lo = run_lo + len * split / hot.splits;
    hi = run_lo + len * (split + 1) / hot.splits;
    part_out = reinterpret_cast<float4v*>(hot.part + (((int64_t)blockIdx.x * tiles * tiles + blockIdx.y) * kThreads + tid) * 16);
    if (lo == hi) {
#pragma unroll
      for (int i = 0; i < 4; ++i) part_out[i] = (float4v){0.f, 0.f, 0.f, 0.f};
      return;
    }
  } else {
    rel = hot.rel_order[blockIdx.x];  // busiest relations first
    lo = rel_start[rel], hi = rel_start[rel + 1];
    if (lo == hi) return;  // the relation does not occur in this call: zero gradient, no change
  }
  float* wr = w + (int64_t)rel * dim * dim;
  float* sr = wsum + (int64_t)rel * dim * dim;
  const uint32_t batch_mask = (1u << kbits) - 1u;

  // this lane's 16 cells of the tile, in the MFMA result layout
  float wt[2][2][4], ht[2][2][4];
  if (!RUNS) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int o = o0 + wm0 + i * 16 + 4 * (lane >> 4) + r, c = i0 + wn0 + j * 16 + (lane & 15);
          const bool ok = o < dim && c < dim;
          wt[i][j][r] = ok ? wr[(int64_t)o * dim + c] : 0.f;
          ht[i][j][r] = ok ? sr[(int64_t)o * dim + c] : 0.f;
        }
  }
  auto write_back = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int o = o0 + wm0 + i * 16 + 4 * (lane >> 4) + r, c = i0 + wn0 + j * 16 + (lane & 15);
          if (o < dim && c < dim) {
            wr[(int64_t)o * dim + c] = wt[i][j][r];
            sr[(int64_t)o * dim + c] = ht[i][j][r];
          }
        }
  };

  // staging: thread -> edges kk and kk + 16 of the step, 4 consecutive columns.
  // Loads are issued unconditionally from addresses clamped into bounds and
  // masked afterwards (no branches around memory instructions).
  const int kk = tid >> 4, q4 = (tid & 15) << 2;
  const int count_a = clamp_count(dim - (o0 + q4)), count_b = clamp_count(dim - (i0 + q4));
  const int col_a = o0 + q4, col_b = i0 + q4;
  auto load_id = [&](int64_t pos, uint32_t* edge, uint32_t* batch) {
    const bool on = pos < hi;
    const int64_t at = on ? pos : hi - 1;
    const uint32_t e = vals[at];
    const uint32_t k = (uint32_t)keys[at] & batch_mask;
    *edge = on ? e : kNone;
    *batch = on ? k : kNone;
  };
  auto fetch_one = [&](const float* __restrict__ base, int64_t row, int col, int count, bool on, Quad* q) {
    if (VEC) {  // dim % 4 == 0: a quad is whole or absent
      const int cc = col <= dim - 4 ? col : dim - 4;
      const float4 v = *reinterpret_cast<const float4*>(base + row + cc);
      const bool keep = on && count == 4;
      q->v[0] = keep ? v.x : 0.f; q->v[1] = keep ? v.y : 0.f; q->v[2] = keep ? v.z : 0.f; q->v[3] = keep ? v.w : 0.f;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int cc = col + i < dim ? col + i : dim - 1;
        const float v = base[row + cc];
        q->v[i] = (on && i < count) ? v : 0.f;
      }
    }
  };

  float4v acc[2][2], tot[2][2];
  auto reset = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
        tot[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
      }
  };
  auto adagrad = [&]() {  // AsyncAdagrad of one batch on the tile (async_adagrad.py:75-85)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // One such step per run and matrix cell is most of this kernel's arithmetic when the
          // runs are short: the hardware's square root and reciprocal (1 ulp each) in place
          // of the correctly rounded sequences.
          const float g = tot[i][j][r] + acc[i][j][r];
          const float sum = ht[i][j][r] + g * g;
          ht[i][j][r] = sum;
          wt[i][j][r] += -lr * g * __builtin_amdgcn_rcpf(__builtin_amdgcn_sqrtf(sum) + 1e-10f);
        }
  };
  reset();

  if (!RUNS && hot.part != nullptr) {
    const uint32_t slot = hot.hot_slot[rel];
    if (slot != kNone) {
      // the runs' gradient tiles are there already: add up the parts of each, one Adagrad step per batch
      const int64_t stride = (int64_t)tiles * tiles * kThreads * 4;  // float4v per part
      const float4v* src = reinterpret_cast<const float4v*>(hot.part) +
                           ((int64_t)slot * hot.num_batches * hot.splits * tiles * tiles + blockIdx.y) * kThreads * 4 + tid * 4;
#pragma unroll 2
      for (int b = 0; b < hot.num_batches; ++b) {
        for (int sp = 0; sp < hot.splits; ++sp, src += stride) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) tot[i][j] += src[i * 2 + j];
        }
        adagrad();
        reset();
      }
      write_back();
      return;
    }
  }

  const int nk = (int)((hi - lo + kStage - 1) / kStage);
  // edge numbers run two steps ahead of the products, rows one step ahead
  uint32_t eid[2], ebt[2], sbt[2];
  Quad ra[2], rb[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) load_id(lo + kk + 16 * h, &eid[h], &ebt[h]);
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const bool on = eid[h] != kNone;
    const int64_t row = on ? (int64_t)eid[h] * dim : 0;
    fetch_one(dz, row, col_a, count_a, on, &ra[h]);
    fetch_one(x, row, col_b, count_b, on, &rb[h]);
    sbt[h] = ebt[h];
    load_id(lo + kStage + kk + 16 * h, &eid[h], &ebt[h]);
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    *reinterpret_cast<float4*>(&lds_a[0][(kk + 16 * h) * LD + q4]) = make_float4(ra[h].v[0], ra[h].v[1], ra[h].v[2], ra[h].v[3]);
    *reinterpret_cast<float4*>(&lds_b[0][(kk + 16 * h) * LD + q4]) = make_float4(rb[h].v[0], rb[h].v[1], rb[h].v[2], rb[h].v[3]);
    if ((tid & 15) == 0) lds_a[0][(kk + 16 * h) * LD + BM] = __uint_as_float(sbt[h]);
  }
  __syncthreads();

  uint32_t cur = kNone;  // batch whose gradient the accumulators hold
  int steps = 0;         // depth-4 products accumulated since the last fold
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bool on = eid[h] != kNone;
        const int64_t row = on ? (int64_t)eid[h] * dim : 0;
        fetch_one(dz, row, col_a, count_a, on, &ra[h]);  // rows of step kt + 1
        fetch_one(x, row, col_b, count_b, on, &rb[h]);
        sbt[h] = ebt[h];
        load_id(lo + (int64_t)(kt + 2) * kStage + kk + 16 * h, &eid[h], &ebt[h]);  // addresses of step kt + 2
      }
    }
    // batch of each staged edge in lanes 0..31; run heads as a bit mask
    const uint32_t mine = __float_as_uint(lds_a[buf][(lane & (kStage - 1)) * LD + BM]);
    const uint32_t prev = (uint32_t)__shfl_up((int)mine, 1, 64);
    const uint32_t valid = (uint32_t)__ballot(lane < kStage && mine != kNone);
    uint32_t heads = (uint32_t)__ballot(lane < kStage && mine != kNone && (lane == 0 || prev != mine));
    const int count = __popc(valid);  // valid edges are a prefix of the step
    const float* __restrict__ ta = lds_a[buf];
    const float* __restrict__ tb = lds_b[buf];
    while (heads != 0u) {
      const int a = __ffs((int)heads) - 1;
      heads &= heads - 1;
      const int b = heads != 0u ? __ffs((int)heads) - 1 : count;
      const uint32_t bt = (uint32_t)__builtin_amdgcn_readlane((int)mine, a);
      if (!RUNS && bt != cur) {  // (a part of a run is of one batch)
        if (cur != kNone) adagrad();
        reset();
        steps = 0;
        cur = bt;
      }
      for (int k4 = a >> 2; k4 < (b + 3) >> 2; ++k4) {
        const int krow = k4 * 4 + (lane >> 4);
        const bool on = krow >= a && krow < b;
        float fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[i] = on ? ta[krow * LD + wm0 + i * 16 + (lane & 15)] : 0.f;
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[j] = tb[krow * LD + wn0 + j * 16 + (lane & 15)];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        if ((++steps & (4 * kFoldTiles - 1)) == 0) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              tot[i][j] += acc[i][j];
              acc[i][j] = (float4v){0.f, 0.f, 0.f, 0.f};
            }
        }
      }
    }
    if (kt + 1 < nk) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        *reinterpret_cast<float4*>(&lds_a[buf ^ 1][(kk + 16 * h) * LD + q4]) = make_float4(ra[h].v[0], ra[h].v[1], ra[h].v[2], ra[h].v[3]);
        *reinterpret_cast<float4*>(&lds_b[buf ^ 1][(kk + 16 * h) * LD + q4]) = make_float4(rb[h].v[0], rb[h].v[1], rb[h].v[2], rb[h].v[3]);
        if ((tid & 15) == 0) lds_a[buf ^ 1][(kk + 16 * h) * LD + BM] = __uint_as_float(sbt[h]);
      }
    }
    __syncthreads();
  }
  if (RUNS) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) part_out[i * 2 + j] = tot[i][j] + acc[i][j];
    return;
  }
  if (cur != kNone) adagrad();
  write_back();
}

bool aligned16(const void* p) { return (uintptr_t)p % 16 == 0; }

}  // namespace

int seg_linear_apply(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, int edges_per_batch,
                     const float* in, int64_t in_batch_stride, const float* w, int dim, bool transpose_w, float* out,
                     int64_t out_batch_stride, bool accumulate, hipStream_t stream) {
  if (n <= 0) return PBG_OK;
  const bool vec_ok = dim % 4 == 0 && aligned16(in) && aligned16(w);
  const dim3 grid((unsigned)ceil_div(n, BM), (unsigned)ceil_div(dim, BN)), block(kThreads);
#define PBG_SEG_APPLY(TRANS, VEC)                                                                                        \
  hipLaunchKernelGGL((seg_linear_apply_kernel<TRANS, VEC>), grid, block, 0, stream, keys, vals, n, kbits, edges_per_batch, \
                     in, in_batch_stride, w, dim, out, out_batch_stride, (int)accumulate)
  if (transpose_w) {
    if (vec_ok) PBG_SEG_APPLY(true, true);
    else PBG_SEG_APPLY(true, false);
  } else {
    if (vec_ok) PBG_SEG_APPLY(false, true);
    else PBG_SEG_APPLY(false, false);
  }
#undef PBG_SEG_APPLY
  return check_launch("seg_linear_apply");
}

namespace {

constexpr size_t kPartBudget = (size_t)1 << 30;  // bytes of run gradients at most

// How the gradients of hot relations' runs are laid out for a call of n edges.
struct HotPlan {
  int splits;        // parts per run
  int64_t slots;     // hot relations at most (0: none)
  uint32_t hot_min;  // edges from which a relation is hot
  size_t part_bytes_per_slot;
};

HotPlan hot_plan(int64_t n, int dim, int num_batches) {
  const int tiles = (int)ceil_div(dim, BN);
  HotPlan p;
  // a chain of about 64 additions per hot relation: runs of few batches are cut into parts
  p.splits = num_batches >= 64 ? 1 : (64 + num_batches - 1) / num_batches;
  p.part_bytes_per_slot = (size_t)num_batches * p.splits * tiles * tiles * kThreads * 16 * sizeof(float);
  // Below about 16 steps of kStage edges the chain is as short as the additions would be.
  const int64_t least = 16 * kStage;
  int64_t slots = n / least;
  if ((size_t)slots * p.part_bytes_per_slot > kPartBudget) slots = (int64_t)(kPartBudget / p.part_bytes_per_slot);
  // the grid of the run kernel is slots * num_batches * splits workgroups in x
  const int64_t grid_cap = ((int64_t)1 << 31) - 1;
  if (slots * num_batches * p.splits > grid_cap) slots = grid_cap / ((int64_t)num_batches * p.splits);
  p.slots = slots;
  // at most n / hot_min relations have hot_min edges: never more than `slots`
  p.hot_min = slots > 0 ? (uint32_t)std::max<int64_t>(least, n / slots + 1) : 0xffffffffu;
  return p;
}

struct HotLayout {
  size_t rel_order, hot_slot, hot_count, hot_list, run_start, part, total;
};

HotLayout hot_layout(int num_relations, const HotPlan& p, int num_batches) {
  HotLayout l;
  size_t at = align_up(((size_t)num_relations + 1) * sizeof(uint32_t), 256);  // rel_start comes first
  auto take = [&](size_t count, size_t size) {
    const size_t here = at;
    at = align_up(at + count * size, 256);
    return here;
  };
  l.rel_order = take(num_relations, 4);
  l.hot_slot = take(num_relations, 4);
  l.hot_count = take(1, 4);
  l.hot_list = take(std::max<int64_t>(p.slots, 1), 4);
  l.run_start = take((size_t)p.slots * (num_batches + 1), 4);
  l.part = take((size_t)p.slots, p.part_bytes_per_slot);
  l.total = at;
  return l;
}

}  // namespace

size_t seg_linear_update_temp_bytes(int num_relations, int64_t n, int dim, int num_batches) {
  return hot_layout(num_relations, hot_plan(n, dim, num_batches), num_batches).total;
}

int seg_linear_update(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, int num_batches,
                      const float* dz, const float* x, int dim, int num_relations, float* w, float* wsum, float lr,
                      void* temp, hipStream_t stream) {
  if (n <= 0 || num_relations <= 0) return PBG_OK;
  if (n >= ((int64_t)1 << 32) - 1) return fail(PBG_ERR_UNSUPPORTED, "seg_linear_update: too many edges");
  if (num_batches < 1 || ((int64_t)num_batches - 1) >> kbits != 0)
    return fail(PBG_ERR_INVALID, "seg_linear_update: num_batches does not fit the key's batch bits");
  const HotPlan hp = hot_plan(n, dim, num_batches);
  const HotLayout hl = hot_layout(num_relations, hp, num_batches);
  char* base = (char*)temp;
  uint32_t* rel_start = (uint32_t*)base;
  uint32_t* hot_count = (uint32_t*)(base + hl.hot_count);
  uint32_t* hot_list = (uint32_t*)(base + hl.hot_list);
  uint32_t* run_start = (uint32_t*)(base + hl.run_start);
  hipLaunchKernelGGL(rel_start_kernel, dim3((unsigned)ceil_div(num_relations + 1, 256)), dim3(256), 0, stream, keys, n,
                     kbits, num_relations, rel_start);
  hipLaunchKernelGGL(rel_plan_kernel, dim3(1), dim3(1024), 0, stream, rel_start, num_relations, hp.hot_min,
                     (uint32_t*)(base + hl.rel_order), (uint32_t*)(base + hl.hot_slot), hot_count, hot_list);
  HotRuns hot;
  hot.rel_order = (const uint32_t*)(base + hl.rel_order);
  hot.hot_slot = (const uint32_t*)(base + hl.hot_slot);
  hot.hot_count = hot_count;
  hot.hot_list = hot_list;
  hot.run_start = run_start;
  hot.part = hp.slots > 0 ? (float*)(base + hl.part) : nullptr;
  hot.num_batches = num_batches;
  hot.splits = hp.splits;
  const int vec_ok = dim % 4 == 0 && aligned16(dz) && aligned16(x);
  const int tiles = (int)ceil_div(dim, BN);
  const dim3 block(kThreads);
  if (hp.slots > 0) {
    hipLaunchKernelGGL(run_start_kernel, dim3((unsigned)ceil_div(hp.slots * (num_batches + 1), 256)), dim3(256), 0, stream,
                       keys, rel_start, kbits, num_batches, hot_count, hot_list, run_start);
    const dim3 grid((unsigned)(hp.slots * num_batches * hp.splits), (unsigned)(tiles * tiles));
    if (vec_ok) {
      hipLaunchKernelGGL((seg_linear_update_kernel<true, true>), grid, block, 0, stream, keys, vals, rel_start, kbits, dz,
                         x, dim, w, wsum, lr, hot);
    } else {
      hipLaunchKernelGGL((seg_linear_update_kernel<false, true>), grid, block, 0, stream, keys, vals, rel_start, kbits,
                         dz, x, dim, w, wsum, lr, hot);
    }
  }
  const dim3 grid((unsigned)num_relations, (unsigned)(tiles * tiles));
  if (vec_ok) {
    hipLaunchKernelGGL((seg_linear_update_kernel<true, false>), grid, block, 0, stream, keys, vals, rel_start, kbits, dz,
                       x, dim, w, wsum, lr, hot);
  } else {
    hipLaunchKernelGGL((seg_linear_update_kernel<false, false>), grid, block, 0, stream, keys, vals, rel_start, kbits, dz,
                       x, dim, w, wsum, lr, hot);
  }
  return check_launch("seg_linear_update");
}

}  // namespace pbg
