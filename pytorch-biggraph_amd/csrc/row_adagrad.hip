// Row gather and RowAdagrad updates: bandwidth kernels.
//
// A row of `dim` floats is moved by one wavefront with 128-bit accesses when
// dim % 4 == 0 (lane l owns float4 number l, l + 64, ...), so a 400-byte row
// (dim 100) is one coalesced request of 25 lanes and a 4 KiB row (dim 1024) is
// four full-wave requests.
#include <mutex>
#include <cstdlib>

#include "pbg_internal.h"
#include "row_ops.h"

namespace pbg {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
constexpr int kRowThreads = 256;  // 4 waves per block, one row per wave


// ---- gather ----------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(kRowThreads) void gather_rows_kernel(const float* __restrict__ table, int64_t num_rows,
                                                                  int dim, const int64_t* __restrict__ idx,
                                                                  int64_t n, float* __restrict__ out,
                                                                  int32_t* __restrict__ oob_flag) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  if (i >= n) return;
  const int64_t r = idx[i];
  const bool ok = r >= 0 && r < num_rows;
  if (!ok && lane == 0 && oob_flag) *oob_flag = 1;
  if (VEC) {
    const int nv = dim >> 2;
    const float4* src = reinterpret_cast<const float4*>(table + (ok ? r : 0) * (int64_t)dim);
    float4* dst = reinterpret_cast<float4*>(out + i * (int64_t)dim);
    // the output is written once and read by somebody else later: streaming stores
    for (int v = lane; v < nv; v += kWave) {
      const float4 x = ok ? src[v] : make_float4(0.f, 0.f, 0.f, 0.f);
      __builtin_nontemporal_store((float4v){x.x, x.y, x.z, x.w}, reinterpret_cast<float4v*>(dst) + v);
    }
  } else {
    const float* src = table + (ok ? r : 0) * (int64_t)dim;
    float* dst = out + i * (int64_t)dim;
    for (int d = lane; d < dim; d += kWave) dst[d] = ok ? src[d] : 0.f;
  }
}

// Rows of at most 4 * LPR floats (dim % 4 == 0): LPR lanes per row, one 128-bit
// word per lane, and U rows per lane group, so that a wave has 64 / LPR * U row
// reads in flight at once.  A short row is a single memory request; the kernel
// is as fast as the number of requests the chip keeps outstanding.
template <int LPR, int U>
__global__ __launch_bounds__(kRowThreads) void gather_rows_multi_kernel(const float* __restrict__ table,
                                                                        int64_t num_rows, int dim,
                                                                        const int64_t* __restrict__ idx, int64_t n,
                                                                        float* __restrict__ out,
                                                                        int32_t* __restrict__ oob_flag) {
  constexpr int kGroups = kWave / LPR;      // rows a wave moves per step
  constexpr int kRowsPerWave = kGroups * U;
  const int lane = threadIdx.x & 63;
  const int q = lane / LPR, v = lane % LPR;
  const int64_t wave = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  const int64_t base = wave * kRowsPerWave + q;
  const bool col_ok = v < (dim >> 2);
  int64_t r[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kGroups;
    r[u] = i < n ? idx[i] : 0;
  }
  float4 x[U];
  bool bad = false;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const bool in = base + u * kGroups < n;
    const bool ok = r[u] >= 0 && r[u] < num_rows;
    bad |= in && !ok;
    x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (ok && col_ok && in)
      x[u] = reinterpret_cast<const float4*>(table + r[u] * (int64_t)dim)[v];
  }
  if (bad && v == 0 && oob_flag) *oob_flag = 1;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kGroups;
    if (col_ok && i < n) {
      float4v* dst = reinterpret_cast<float4v*>(out + i * (int64_t)dim) + v;
      __builtin_nontemporal_store((float4v){x[u].x, x[u].y, x[u].z, x[u].w}, dst);
    }
  }
}

// ---- segmented RowAdagrad over sorted keys -----------------------------------
// Keys are (row << kbits | worker), sorted.  Equal keys form a "run" (the
// duplicates of one row inside one worker's batch, to be summed); the runs of
// one row are applied one Adagrad update after another in worker order, exactly
// as if the workers' sparse steps had been applied in sequence.  Power-law
// graphs make single runs hundreds of rows long, so the summation is spread
// over three kernels, all deterministic and in place in grad_rows:
//   tile_reduce   one wave per tile of kTile sorted positions sums every piece
//                 (maximal stretch of equal keys inside the tile) longer than 1
//                 into the gradient row of the piece's first position;
//   run_combine   one wave per tile border; the first border a run crosses adds
//                 the pieces of the later tiles into the row of the run's first
//                 position;
//   row_update    a wave per few sorted positions; at each position that starts
//                 a row it walks the row's runs (one gradient row each), the
//                 keys of the next 64 positions held in registers.
// In a single-worker call (kbits == 0: a row has ONE run, all its duplicates) nearly all
// runs are two or three positions long.  Sending those through tile_reduce costs a read of
// every row of the run, a write of the sum and another read of it; instead a run of at most
// kFoldMax positions -- wherever it lies -- is left alone by tile_reduce and run_combine and
// summed, in position order, by the update kernel as it reads it.  Longer runs (a hot row of
// a power-law graph) keep the three-kernel scheme.  Whether a run is short is decided from
// its length alone, so the three kernels agree, and the sort says whether any long run
// exists at all (`long_runs`): where none does, tile_reduce and run_combine return at once.
// (With several workers a row has a run per worker and the update kernels' loop over them is
// latency bound: the extra loads cost more there than they save.  row_walk_kernel, which
// streams a table row's whole stretch anyway, takes every whole run that lies inside one
// tile, whatever its length.)
constexpr int kTile = 32;

template <int NV, bool VEC>
struct RowRegs {
  static constexpr int W = VEC ? 4 : 1;
  float v[NV * W];

  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int q = 0; q < NV * W; ++q) v[q] = 0.f;
  }
  __device__ __forceinline__ void load(const float* __restrict__ p, int nv, int lane) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = i * kWave + lane;
      if (VEC) {
        const float4 x = (e < nv) ? reinterpret_cast<const float4*>(p)[e] : make_float4(0.f, 0.f, 0.f, 0.f);
        v[i * W + 0] = x.x; v[i * W + 1] = x.y; v[i * W + 2] = x.z; v[i * W + 3] = x.w;
      } else {
        v[i] = (e < nv) ? p[e] : 0.f;
      }
    }
  }
  __device__ __forceinline__ void add(const float* __restrict__ p, int nv, int lane) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = i * kWave + lane;
      if (e < nv) {
        if (VEC) {
          const float4 x = reinterpret_cast<const float4*>(p)[e];
          v[i * W + 0] += x.x; v[i * W + 1] += x.y; v[i * W + 2] += x.z; v[i * W + 3] += x.w;
        } else {
          v[i] += p[e];
        }
      }
    }
  }
  // the same with the whole row switched off by `on` (the load is still an ordinary, hoistable one)
  __device__ __forceinline__ void add_if(const float* __restrict__ p, int nv, int lane, bool on) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = i * kWave + lane;
      if (VEC) {
        const float4 x = (on && e < nv) ? reinterpret_cast<const float4*>(p)[e] : make_float4(0.f, 0.f, 0.f, 0.f);
        v[i * W + 0] += x.x; v[i * W + 1] += x.y; v[i * W + 2] += x.z; v[i * W + 3] += x.w;
      } else {
        v[i] += (on && e < nv) ? p[e] : 0.f;
      }
    }
  }
  __device__ __forceinline__ void add(const RowRegs& o) {
#pragma unroll
    for (int q = 0; q < NV * W; ++q) v[q] += o.v[q];
  }
  __device__ __forceinline__ void store(float* __restrict__ p, int nv, int lane) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = i * kWave + lane;
      if (e < nv) {
        if (VEC) {
          reinterpret_cast<float4*>(p)[e] = make_float4(v[i * W + 0], v[i * W + 1], v[i * W + 2], v[i * W + 3]);
        } else {
          p[e] = v[i];
        }
      }
    }
  }
};

// First position in (start, n) whose key, shifted right by `shift`, differs from
// `want`; all 64 lanes scan together.
__device__ __forceinline__ int64_t scan_end(const uint64_t* __restrict__ keys, int64_t start, int64_t n,
                                            uint64_t want, int shift, int lane) {
  int64_t base = start + 1;
  while (true) {
    const int64_t j = base + lane;
    const bool same = (j < n) && ((keys[j] >> shift) == want);
    const uint64_t m = __ballot(same);
    if (m != ~0ull) return base + (__ffsll((unsigned long long)~m) - 1);
    base += kWave;
  }
}

// value of lane `l` (uniform) of a per-lane 32-bit / 64-bit quantity
__device__ __forceinline__ uint32_t lane_u32(uint32_t v, int l) {
  return (uint32_t)__builtin_amdgcn_readlane((int)v, l);
}
__device__ __forceinline__ uint64_t lane_u64(uint64_t v, int l) {
  const uint32_t lo = lane_u32((uint32_t)v, l), hi = lane_u32((uint32_t)(v >> 32), l);
  return ((uint64_t)hi << 32) | lo;
}

// The sort's word on runs of more than kFoldMax equal keys (kLongWords words, any of them raised); wave-uniform.
__device__ __forceinline__ bool any_long_run(const uint32_t* __restrict__ long_runs) {
  uint32_t any = 0u;
#pragma unroll
  for (int w = 0; w < kLongWords / kWave; ++w) any |= long_runs[w * kWave + (threadIdx.x & 63)];
  return __ballot(any != 0u) != 0ull;
}

// One workgroup (kRowThreads = 256 threads): the totals of batch b, summed in a fixed order.
__device__ __forceinline__ void batch_sums_block(const BatchSums& bs, int b) {
  __shared__ float sh[kRowThreads];
  __shared__ long long shv[2][kRowThreads];
  const float* rows = bs.lossrow + (int64_t)b * bs.per_batch;
  const int* viol = bs.violrow + (int64_t)b * bs.per_batch * 2;
  float acc = 0.f;
  long long v0 = 0, v1 = 0;
  for (int q = threadIdx.x; q < bs.per_batch; q += kRowThreads) {
    acc += rows[q];
    v0 += viol[q * 2];
    v1 += viol[q * 2 + 1];
  }
  sh[threadIdx.x] = acc;
  shv[0][threadIdx.x] = v0;
  shv[1][threadIdx.x] = v1;
  __syncthreads();
  for (int off = kRowThreads / 2; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) {
      sh[threadIdx.x] += sh[threadIdx.x + off];
      shv[0][threadIdx.x] += shv[0][threadIdx.x + off];
      shv[1][threadIdx.x] += shv[1][threadIdx.x + off];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    bs.loss_out[b] = sh[0];
    bs.violators[b * 2] = (unsigned long long)shv[0][0];
    bs.violators[b * 2 + 1] = (unsigned long long)shv[1][0];
  }
}

// leave_mode 0: every piece of two or more positions is summed; 1 (single-worker calls): pieces of runs
// of at most kFoldMax positions are left to the update kernel; 2 (row_walk_kernel follows): whole runs
// inside the tile are left alone.
template <int NV, bool VEC>
__global__ __launch_bounds__(kRowThreads) void tile_reduce_kernel(const uint64_t* __restrict__ keys,
                                                                  const uint32_t* __restrict__ vals, int64_t n,
                                                                  float* __restrict__ grad_rows, int dim,
                                                                  int leave_mode, const uint32_t* __restrict__ long_runs,
                                                                  BatchSums sums, unsigned tile_blocks) {
  if (blockIdx.x >= tile_blocks) {  // the workgroups behind the tiles': one per batch of `sums`
    batch_sums_block(sums, (int)(blockIdx.x - tile_blocks));
    return;
  }
  if (leave_mode == 1 && long_runs && !any_long_run(long_runs)) return;  // the sort saw no run of more than kFoldMax positions
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  const int64_t begin = tile * kTile;
  if (begin >= n) return;
  const int64_t end = (begin + kTile < n) ? begin + kTile : n;
  const int nv = VEC ? (dim >> 2) : dim;
  // one key and one value per lane for the whole tile, then pieces are found with ballots
  const int64_t mine = begin + lane;
  const uint64_t key = (mine < end) ? keys[mine] : 0ull;
  const uint32_t val = (mine < end) ? vals[mine] : 0u;
  const uint64_t prev = __shfl_up(key, 1, 64);
  const bool starts = (mine < end) && (lane == 0 || prev != key);
  uint64_t heads = __ballot(starts);  // bit l set: a piece starts at begin + l
  // How far the runs at the tile's two edges go on outside it, up to kFoldMax positions each way:
  // lanes 0 .. kFoldMax - 1 look at the positions before the tile (nearest first), the next kFoldMax at those after it.
  int before = 0, after = 0;
  if (leave_mode != 0) {
    const uint64_t first_key = lane_u64(key, 0), last_key = lane_u64(key, (int)(end - begin) - 1);
    const int64_t q = lane < kFoldMax ? begin - 1 - lane : end + (lane - kFoldMax);
    const bool there = lane < 2 * kFoldMax && q >= 0 && q < n;
    const uint64_t other = there ? keys[q] : 0ull;
    constexpr uint32_t kAll = (1u << kFoldMax) - 1u;
    const uint32_t same_before = (uint32_t)__ballot(there && lane < kFoldMax && other == first_key) & kAll;
    const uint32_t same_after = (uint32_t)(__ballot(there && lane >= kFoldMax && other == last_key) >> kFoldMax) & kAll;
    before = same_before == kAll ? kFoldMax : __ffs((int)~same_before) - 1;  // leading ones
    after = same_after == kAll ? kFoldMax : __ffs((int)~same_after) - 1;
  }
  // Only a piece of two or more positions has anything to sum: a start whose next position exists and is no start.
  // (Without duplicates -- most tiles of most calls -- the loop below does not run at all.)
  const int len = (int)(end - begin);
  uint64_t multi = heads & ~(heads >> 1) & (((1ull << len) - 1ull) >> 1);
  while (multi != 0ull) {
    const int a = __ffsll((unsigned long long)multi) - 1;
    multi &= multi - 1;
    const uint64_t later = heads & ~((2ull << a) - 1ull);
    const int b = later != 0ull ? (__ffsll((unsigned long long)later) - 1) : len;
    if (leave_mode != 0) {
      const bool whole = (a > 0 || before == 0) && (b < (int)(end - begin) || after == 0);
      if (leave_mode == 2 && whole) continue;  // (a single position needs no sum either way)
      const int run_len = (b - a) + (a == 0 ? before : 0) + (b == (int)(end - begin) ? after : 0);
      if (leave_mode == 1 && run_len <= kFoldMax) continue;
    }
    if (b - a < 2) continue;
    RowRegs<NV, VEC> acc;
    float* head = grad_rows + (int64_t)lane_u32(val, a) * dim;
    acc.load(head, nv, lane);
    int j = a + 1;
    for (; j + 1 < b; j += 2) {  // two rows in flight
      RowRegs<NV, VEC> x, y;
      x.load(grad_rows + (int64_t)lane_u32(val, j) * dim, nv, lane);
      y.load(grad_rows + (int64_t)lane_u32(val, j + 1) * dim, nv, lane);
      acc.add(x);
      acc.add(y);
    }
    if (j < b) acc.add(grad_rows + (int64_t)lane_u32(val, j) * dim, nv, lane);
    acc.store(head, nv, lane);
  }
}

// One wave per tile border: if a run crosses the border and this is the first
// border it crosses, add the pieces of all later tiles into the run's head row.
template <int NV, bool VEC>
__global__ __launch_bounds__(kRowThreads) void run_combine_kernel(const uint64_t* __restrict__ keys,
                                                                  const uint32_t* __restrict__ vals, int64_t n,
                                                                  float* __restrict__ grad_rows, int dim,
                                                                  int leave_mode, const uint32_t* __restrict__ long_runs) {
  if (leave_mode == 1 && long_runs && !any_long_run(long_runs)) return;  // as in tile_reduce_kernel
  const int lane = threadIdx.x & 63;
  const int64_t b = ((int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6) + 1) * kTile;
  if (b >= n) return;
  // window of the tile before the border (lanes 0..31) and the tile after it (lanes 32..63)
  const int64_t p = b - kTile + lane;
  const uint64_t kk = keys[p < n ? p : n - 1];
  const uint64_t key = lane_u64(kk, kTile);
  if (lane_u64(kk, kTile - 1) != key) return;  // no run crosses this border
  const uint64_t same = __ballot(p < n && kk == key);
  const uint32_t not_before = ~(uint32_t)same;  // zero bits: positions of the run in the tile before the border
  const int head_lane = not_before ? 32 - __clz(not_before) : 0;
  if (head_lane == 0 && b - kTile > 0 && keys[b - kTile - 1] == key) return;  // an earlier border owns this run
  const uint32_t not_after = ~(uint32_t)(same >> 32);
  // a run that begins and ends inside the window shows its whole length: a short one is the update kernel's
  if (leave_mode == 1 && head_lane > 0 && not_after != 0u && (kTile - head_lane) + (__ffs((int)not_after) - 1) <= kFoldMax)
    return;
  const int64_t end = not_after ? b + (__ffs(not_after) - 1) : scan_end(keys, b + kTile - 1, n, key, 0, lane);
  const int nv = VEC ? (dim >> 2) : dim;
  RowRegs<NV, VEC> acc;
  float* head = grad_rows + (int64_t)vals[b - kTile + head_lane] * dim;
  acc.load(head, nv, lane);
  for (int64_t base = b; base < end; base += (int64_t)kTile * kWave) {  // 64 pieces' first positions per round
    const int64_t q = base + (int64_t)lane * kTile;
    const uint32_t v = q < end ? vals[q] : 0u;
    const int64_t left = (end - base + kTile - 1) / kTile;
    const int count = left < kWave ? (int)left : kWave;
    int j = 0;
    for (; j + 1 < count; j += 2) {
      RowRegs<NV, VEC> x, y;
      x.load(grad_rows + (int64_t)lane_u32(v, j) * dim, nv, lane);
      y.load(grad_rows + (int64_t)lane_u32(v, j + 1) * dim, nv, lane);
      acc.add(x);
      acc.add(y);
    }
    if (j < count) acc.add(grad_rows + (int64_t)lane_u32(v, j) * dim, nv, lane);
  }
  acc.store(head, nv, lane);
}

// With COSB the gradient rows are gradients at the NORMALISED row y = x / |x| (the step scored on a normalised
// copy of the table, see CosBack): a run's summed gradient first goes back through the normalisation,
// g <- (g - y <y, g>) / |x|, which is linear in g and so may follow the sum over the run's duplicates.
template <int NV, bool VEC, bool COSB = false>
__device__ __forceinline__ float adagrad_apply(RowRegs<NV, VEC>& w, const RowRegs<NV, VEC>& g_in, float gsum, float fdim,
                                               float lr, const RowRegs<NV, VEC>* y = nullptr, float inv = 0.f) {
  RowRegs<NV, VEC> g = g_in;
  if (COSB) {
    float dot = 0.f;
#pragma unroll
    for (int q = 0; q < NV * RowRegs<NV, VEC>::W; ++q) dot += y->v[q] * g.v[q];
    dot = wave_sum(dot);
#pragma unroll
    for (int q = 0; q < NV * RowRegs<NV, VEC>::W; ++q) g.v[q] = (g.v[q] - dot * y->v[q]) * inv;
  }
  float sq = 0.f;
#pragma unroll
  for (int q = 0; q < NV * RowRegs<NV, VEC>::W; ++q) sq += g.v[q] * g.v[q];
  gsum += wave_sum(sq) / fdim;
  const float stdv = sqrtf(gsum) + 1e-10f;
#pragma unroll
  for (int q = 0; q < NV * RowRegs<NV, VEC>::W; ++q) w.v[q] += (-lr * g.v[q]) / stdv;
  return gsum;
}

// first position in [lo, hi) whose key is >= want (hi if none)
__device__ __forceinline__ int64_t lower_bound_key(const uint64_t* __restrict__ keys, int64_t lo, int64_t hi,
                                                   uint64_t want) {
  while (lo < hi) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if (keys[mid] < want) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// One wave looks at R consecutive sorted positions; a position that starts a row
// gets the row's update.  All loads that do not depend on each other (the R key
// windows, then the weight rows and first gradient rows of the positions that
// turned out to be row heads) are issued together: the kernel lives on memory
// latency, and the rows in flight per wave are what hides it.
template <int NV, bool VEC, int R, bool COSB = false>
__global__ __launch_bounds__(kRowThreads) void row_update_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, int64_t n, int kbits,
    const float* __restrict__ grad_rows, int dim, float* __restrict__ w0, float* __restrict__ g0, int64_t rows0,
    float* __restrict__ w1, float* __restrict__ g1, int64_t rows1, float lr, CosBack cb) {
  const int lane = threadIdx.x & 63;
  const int64_t first = ((int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6)) * R;
  if (first >= n) return;
  const int nv = VEC ? (dim >> 2) : dim;
  const float fdim = (float)dim;
  // one coalesced look at each position and the 63 sorted positions after it
  uint64_t kk[R], before[R];
  uint32_t vv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t i = first + r < n ? first + r : n - 1;
    const int64_t p = i + lane < n ? i + lane : n - 1;
    kk[r] = keys[p];
    vv[r] = vals[p];
    before[r] = keys[i > 0 ? i - 1 : 0];
  }
  bool head[R];
  float* wrow[R];
  float* gptr[R];
  float gsum[R];
  RowRegs<NV, VEC> w[R], g[R];
  RowRegs<NV, VEC> y[COSB ? R : 1];
  float inv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t i = first + r;
    const uint64_t row = lane_u64(kk[r], 0) >> kbits;
    // out-of-range indices are parked past both tables
    head[r] = i < n && !(i > 0 && (before[r] >> kbits) == row) && (int64_t)row < rows0 + rows1;
    inv[r] = 0.f;
    if (!head[r]) continue;
    if ((int64_t)row < rows0) {
      wrow[r] = w0 + (int64_t)row * dim;
      gptr[r] = g0 + row;
    } else {
      wrow[r] = w1 + ((int64_t)row - rows0) * dim;
      gptr[r] = g1 + ((int64_t)row - rows0);
    }
    if (COSB) {
      const bool t0 = (int64_t)row < rows0;
      y[COSB ? r : 0].load(t0 ? cb.y0 + (int64_t)row * dim : cb.y1 + ((int64_t)row - rows0) * dim, nv, lane);
      inv[r] = t0 ? cb.inv0[row] : cb.inv1[(int64_t)row - rows0];
    }
    w[r].load(wrow[r], nv, lane);
    gsum[r] = *gptr[r];
    g[r].load(grad_rows + (int64_t)lane_u32(vv[r], 0) * dim, nv, lane);  // each run's sum sits in its first row ...
    if (kbits == 0) {  // ... unless it is a short run, left to this kernel: summed here in position order
      const uint64_t same = __ballot(i + lane < n && kk[r] == lane_u64(kk[r], 0));
      const int run_len = ~same != 0ull ? __ffsll((unsigned long long)~same) - 1 : kWave;
      const bool fold = run_len <= kFoldMax;
#pragma unroll
      for (int t = 1; t < 4; ++t)  // the common lengths with their loads in flight together
        g[r].add_if(grad_rows + (int64_t)lane_u32(vv[r], t) * dim, nv, lane, fold && t < run_len);
      for (int t = 4; fold && t < run_len; t += 2) {  // two rows in flight
        RowRegs<NV, VEC> x, y;
        x.load(grad_rows + (int64_t)lane_u32(vv[r], t) * dim, nv, lane);
        y.zero();
        if (t + 1 < run_len) y.load(grad_rows + (int64_t)lane_u32(vv[r], t + 1) * dim, nv, lane);
        g[r].add(x);
        g[r].add(y);
      }
    }
  }
  int long_r = -1;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!head[r]) continue;
    const int64_t i = first + r;
    const uint64_t row = lane_u64(kk[r], 0) >> kbits;
    const uint64_t in_row = __ballot(i + lane < n && (kk[r] >> kbits) == row);
    if (~in_row != 0ull) {
      // the row ends inside the window: its runs are known from the keys in registers
      const int len = __ffsll((unsigned long long)~in_row) - 1;
      const uint64_t up = __shfl_up(kk[r], 1, 64);
      uint64_t heads = __ballot(lane < len && (lane == 0 || up != kk[r]));  // first position of every run
      heads &= heads - 1;
      while (heads != 0ull) {  // the next run's row is in flight while this one is applied
        const int a = __ffsll((unsigned long long)heads) - 1;
        heads &= heads - 1;
        RowRegs<NV, VEC> next;
        next.load(grad_rows + (int64_t)lane_u32(vv[r], a) * dim, nv, lane);
        gsum[r] = adagrad_apply<NV, VEC, COSB>(w[r], g[r], gsum[r], fdim, lr, &y[COSB ? r : 0], inv[r]);
        g[r] = next;
      }
      gsum[r] = adagrad_apply<NV, VEC, COSB>(w[r], g[r], gsum[r], fdim, lr, &y[COSB ? r : 0], inv[r]);
    } else if (kbits == 0) {  // a single-worker call has one run per row
      gsum[r] = adagrad_apply<NV, VEC, COSB>(w[r], g[r], gsum[r], fdim, lr, &y[COSB ? r : 0], inv[r]);
    } else {
      // A long row: handled after this loop.  There is at most one per wave (the positions after its head belong
      // to it), so the code below exists once instead of once per position, in the registers that this loop's rows
      // no longer need.
      long_r = r;
      continue;
    }
    w[r].store(wrow[r], nv, lane);
    if (lane == 0) *gptr[r] = gsum[r];
  }
  if (long_r < 0) return;
  // (only the position is carried out of the loop above: the row's weights, sum and first gradient are fetched again)
  const int64_t i = first + long_r;
  const uint64_t row = keys[i] >> kbits;
  float* long_wrow = (int64_t)row < rows0 ? w0 + (int64_t)row * dim : w1 + ((int64_t)row - rows0) * dim;
  float* long_gptr = (int64_t)row < rows0 ? g0 + row : g1 + ((int64_t)row - rows0);
  RowRegs<NV, VEC> lw, lg, ly;
  float linv = 0.f;
  if (COSB) {
    const bool t0 = (int64_t)row < rows0;
    ly.load(t0 ? cb.y0 + (int64_t)row * dim : cb.y1 + ((int64_t)row - rows0) * dim, nv, lane);
    linv = t0 ? cb.inv0[row] : cb.inv1[(int64_t)row - rows0];
  }
  lw.load(long_wrow, nv, lane);
  float lsum = *long_gptr;
  lg.load(grad_rows + (int64_t)vals[i] * dim, nv, lane);
  // A long row (a hot entity of a power-law graph): one run per batch that names it, hundreds of positions
  // each.  Lane l finds the first position of batch b0 + l by binary search in the sorted keys, 64 batches at
  // once, and fetches the number of the gradient row there; the runs are then applied in batch order with the
  // next kAhead runs' gradients in flight.  (Walking from run to run costs a chain of dependent loads per run:
  // the keys of every 64 positions of the run, the row's number, the row.)
  // The starts do not decrease with the batch, and an absent batch has the start of the next one present: the
  // runs still to apply are the starts that differ from the one before them -- from 0, the run in hand, at first.
  constexpr int kRowRegs = NV * RowRegs<NV, VEC>::W;
  constexpr int kAhead = kRowRegs > 16 ? 1 : (kRowRegs * R > 16 ? 4 : (kRowRegs > 4 ? 2 : 8));  // (within the registers of the loop above)
  const int nb = 1 << kbits;
  const int64_t row_end = lower_bound_key(keys, i, n, (row + 1) << kbits);
  uint32_t last_st = 0;
#pragma unroll 1
  for (int b0 = 0; b0 < nb; b0 += kWave) {
    const int b = b0 + lane;
    const int64_t at = b < nb ? lower_bound_key(keys, i, row_end, (row << kbits) | (uint64_t)b) : row_end;
    const uint32_t st = (uint32_t)(at - i);
    const uint32_t sv = vals[at < n ? at : n - 1];
    uint32_t st_prev = (uint32_t)__shfl_up((int)st, 1, 64);
    if (lane == 0) st_prev = last_st;
    uint64_t todo = __ballot(b < nb && st != st_prev && (int64_t)st < row_end - i);
    last_st = lane_u32(st, kWave - 1);
#pragma unroll 1
    while (todo != 0ull) {
      int js[kAhead];
      RowRegs<NV, VEC> nx[kAhead];
      const int j0 = __ffsll((unsigned long long)todo) - 1;
#pragma unroll
      for (int t = 0; t < kAhead; ++t) {
        js[t] = todo != 0ull ? __ffsll((unsigned long long)todo) - 1 : -1;
        todo &= todo - 1;  // (0 stays 0)
      }
      // all loads are issued before the first is used; slots past the last run read the first row again and are dropped
#pragma unroll
      for (int t = 0; t < kAhead; ++t)
        nx[t].load(grad_rows + (int64_t)lane_u32(sv, js[t] >= 0 ? js[t] : j0) * dim, nv, lane);
#pragma unroll
      for (int t = 0; t < kAhead; ++t) {
        if (js[t] < 0) break;
        lsum = adagrad_apply<NV, VEC, COSB>(lw, lg, lsum, fdim, lr, &ly, linv);
        lg = nx[t];
      }
    }
  }
  lsum = adagrad_apply<NV, VEC, COSB>(lw, lg, lsum, fdim, lr, &ly, linv);
  lw.store(long_wrow, nv, lane);
  if (lane == 0) *long_gptr = lsum;
}

// One wave per TABLE row, for calls whose gradient rows outnumber the tables' rows many
// times over (a small entity table under a thousand uniform negatives per chunk and 64
// workers: every row has a run in nearly every worker's batch).  Walking the sorted
// positions from their side (row_update_kernel) then spends its time in the chain
// of dependent loads along a row's runs.  Here the wave finds its row's first position
// by a 64-ary search, then walks the row's stretch of sorted positions window by
// window: the rows to read -- the head row of every run, or all rows of a short run that
// tile_reduce left alone -- are known from the keys of the window alone, so
// R of them are in flight at a time whatever run they belong to, and the runs' Adagrad
// steps follow in worker order on registers.
template <int NV, bool VEC, int R, bool COSB = false>
__global__ __launch_bounds__(kRowThreads) void row_walk_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, int64_t n, int kbits,
    const float* __restrict__ grad_rows, int dim, float* __restrict__ w0, float* __restrict__ g0, int64_t rows0,
    float* __restrict__ w1, float* __restrict__ g1, int64_t rows1, float lr, CosBack cb) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  if (row >= rows0 + rows1) return;
  const uint64_t target = (uint64_t)row << kbits;
  // first position whose key is >= target; every round the 64 lanes probe the range at equal distances
  int64_t lo = 0, hi = n;
  while (hi > lo) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t p = lo + (int64_t)(lane + 1) * step - 1;
    const bool below = p < hi && keys[p] < target;
    const int cnt = __popcll(__ballot(below));  // the keys are sorted: the probes below the target are the first cnt
    const int64_t nhi = lo + (int64_t)(cnt + 1) * step - 1;
    lo += (int64_t)cnt * step;
    hi = nhi < hi ? nhi : hi;
  }
  const int64_t s = lo;
  if (s >= n || (keys[s] >> kbits) != (uint64_t)row) return;
  const int nv = VEC ? (dim >> 2) : dim;
  const float fdim = (float)dim;
  float* wrow = row < rows0 ? w0 + row * dim : w1 + (row - rows0) * dim;
  float* gptr = row < rows0 ? g0 + row : g1 + (row - rows0);
  RowRegs<NV, VEC> w, acc, y;
  float inv = 0.f;
  if (COSB) {
    y.load(row < rows0 ? cb.y0 + row * dim : cb.y1 + (row - rows0) * dim, nv, lane);
    inv = row < rows0 ? cb.inv0[row] : cb.inv1[row - rows0];
  }
  w.load(wrow, nv, lane);
  float gsum = *gptr;
  acc.zero();
  for (int64_t wb = s & ~(int64_t)(kWave - 1);; wb += kWave) {
    const int64_t p = wb + lane;
    const bool inb = p < n;
    const uint64_t key = inb ? keys[p] : ~0ull;
    const uint32_t val = inb ? vals[p] : 0u;
    const bool in_row = inb && p >= s && (key >> kbits) == (uint64_t)row;
    const uint64_t m_in = __ballot(in_row);
    if (m_in == 0ull) break;
    // the keys just outside the window (only looked at where a neighbour inside is in the row)
    const uint64_t key_before = wb > 0 ? keys[wb - 1] : ~key;
    const uint64_t key_after = wb + kWave < n ? keys[wb + kWave] : ~0ull;
    uint64_t prev = __shfl_up(key, 1, 64), next = __shfl_down(key, 1, 64);
    if (lane == 0) prev = key_before;
    if (lane == kWave - 1) next = key_after;
    const uint64_t starts = __ballot(in_row && (p == 0 || prev != key));   // first position of a run
    const uint64_t lasts = __ballot(in_row && (p == n - 1 || next != key));  // last position of a run
    // the rows to read, and the positions after which a run is complete
    uint64_t todo = 0ull, done = 0ull;
    for (uint64_t st = starts; st != 0ull; st &= st - 1) {
      const int a = __ffsll((unsigned long long)st) - 1;
      const uint64_t from = lasts & (~0ull << a);
      const int e = from != 0ull ? __ffsll((unsigned long long)from) - 1 : -1;  // -1: the run goes on past the window
      const int len = e - a + 1;
      if (e >= 0 && len >= 2 && (a / kTile) == (e / kTile)) {  // a whole run inside one tile (the window starts at a multiple of kTile): summed here
        todo |= ((2ull << e) - 1) & (~0ull << a);
        done |= 1ull << e;
      } else {  // the run's sum is in its first row (tile_reduce, run_combine)
        todo |= 1ull << a;
        done |= 1ull << a;
      }
    }
    while (todo != 0ull) {
      int pos[R];
      const int first = __ffsll((unsigned long long)todo) - 1;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        pos[r] = todo != 0ull ? __ffsll((unsigned long long)todo) - 1 : -1;
        todo &= todo - 1;  // (0 stays 0)
      }
      // all R loads are issued before the first is used; slots past the end read the first row again and are dropped
      RowRegs<NV, VEC> x[R];
#pragma unroll
      for (int r = 0; r < R; ++r)
        x[r].load(grad_rows + (int64_t)lane_u32(val, pos[r] >= 0 ? pos[r] : first) * dim, nv, lane);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (pos[r] < 0) break;
        acc.add(x[r]);
        if ((done >> pos[r]) & 1ull) {
          gsum = adagrad_apply<NV, VEC, COSB>(w, acc, gsum, fdim, lr, &y, inv);
          acc.zero();
        }
      }
    }
    if (!(m_in >> (kWave - 1))) break;  // the row's stretch ended inside the window
  }
  w.store(wrow, nv, lane);
  if (lane == 0) *gptr = gsum;
}

// The same for rows of at most 128 floats (dim % 4 == 0): half a wave per sorted
// position, one 128-bit word per lane, so a wave keeps twice as many rows in
// flight for the same registers.  The two halves of a wave run the same code on
// different positions; everything that is uniform per position is uniform per
// half only, so values cross lanes through shuffles inside the half, never
// through scalar registers.
__device__ __forceinline__ uint64_t half_bcast_u64(uint64_t v, int src) {
  const uint32_t lo = (uint32_t)__shfl((int)(uint32_t)v, src, 64);
  const uint32_t hi = (uint32_t)__shfl((int)(uint32_t)(v >> 32), src, 64);
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ float half_sum(float v) {  // sum over the 32 lanes of a half, in every lane
  v = row16_sum(v);
  return v + __shfl_xor(v, 16, 64);
}
constexpr int kMaxBatchSlots = 8;  // batches per lane of a half wave: 256 batches per call at most
__device__ __forceinline__ float4 load_or_zero(const float* __restrict__ p, bool has) {
  return has ? *reinterpret_cast<const float4*>(p) : make_float4(0.f, 0.f, 0.f, 0.f);
}
__device__ __forceinline__ void add4(float4& a, const float4& b) {
  a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
}
template <bool COSB = false>
__device__ __forceinline__ float adagrad_apply_half(float4& w, const float4& g_in, float gsum, float fdim, float lr,
                                                    const float4& y = float4(), float inv = 0.f) {
  float4 g = g_in;
  if (COSB) {  // (see adagrad_apply)
    const float dot = half_sum((y.x * g.x + y.y * g.y) + (y.z * g.z + y.w * g.w));
    g.x = (g.x - dot * y.x) * inv;
    g.y = (g.y - dot * y.y) * inv;
    g.z = (g.z - dot * y.z) * inv;
    g.w = (g.w - dot * y.w) * inv;
  }
  gsum += half_sum(g.x * g.x + g.y * g.y + g.z * g.z + g.w * g.w) / fdim;
  const float stdv = sqrtf(gsum) + 1e-10f;
  w.x += (-lr * g.x) / stdv;
  w.y += (-lr * g.y) / stdv;
  w.z += (-lr * g.z) / stdv;
  w.w += (-lr * g.w) / stdv;
  return gsum;
}

template <int R, bool COSB = false>
__global__ __launch_bounds__(kRowThreads) void row_update_half_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, int64_t n, int kbits,
    const float* __restrict__ grad_rows, int dim, float* __restrict__ w0, float* __restrict__ g0, int64_t rows0,
    float* __restrict__ w1, float* __restrict__ g1, int64_t rows1, float lr, CosBack cb) {
  const int lane = threadIdx.x & 63, gl = lane & 31, gbase = lane & 32;
  const int64_t first = ((((int64_t)blockIdx.x * kRowThreads) + threadIdx.x) >> 5) * R;
  const bool has = gl < (dim >> 2);
  const int col = gl << 2;
  const float fdim = (float)dim;
  // one coalesced look at each position and the 31 sorted positions after it
  uint64_t kk[R], before[R];
  uint32_t vv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t i = first + r < n ? first + r : n - 1;
    const int64_t p = i + gl < n ? i + gl : n - 1;
    kk[r] = keys[p];
    vv[r] = vals[p];
    before[r] = keys[i > 0 ? i - 1 : 0];
  }
  bool head[R];
  float* wrow[R];
  float* gptr[R];
  float gsum[R];
  float4 w[R], g[R], y[R];
  float inv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t i = first + r;
    const uint64_t row = half_bcast_u64(kk[r], gbase) >> kbits;
    // out-of-range indices are parked past both tables
    head[r] = i < n && !(i > 0 && (before[r] >> kbits) == row) && (int64_t)row < rows0 + rows1;
    y[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    inv[r] = 0.f;
    if (!head[r]) continue;
    if ((int64_t)row < rows0) {
      wrow[r] = w0 + (int64_t)row * dim + col;
      gptr[r] = g0 + row;
    } else {
      wrow[r] = w1 + ((int64_t)row - rows0) * dim + col;
      gptr[r] = g1 + ((int64_t)row - rows0);
    }
    if (COSB) {
      const bool t0 = (int64_t)row < rows0;
      y[r] = load_or_zero((t0 ? cb.y0 + (int64_t)row * dim : cb.y1 + ((int64_t)row - rows0) * dim) + col, has);
      inv[r] = t0 ? cb.inv0[row] : cb.inv1[(int64_t)row - rows0];
    }
    w[r] = load_or_zero(wrow[r], has);
    gsum[r] = *gptr[r];
    g[r] = load_or_zero(grad_rows + (int64_t)__shfl((int)vv[r], gbase, 64) * dim + col, has);
    if (kbits == 0) {  // the row's one run, if it is a short one left to this kernel: summed here in position order
      const uint32_t same = (uint32_t)(__ballot(i + gl < n && kk[r] == half_bcast_u64(kk[r], gbase)) >> gbase);
      const int run_len = same != 0xffffffffu ? __ffs((int)~same) - 1 : 32;
      const bool fold = run_len <= kFoldMax;
#pragma unroll
      for (int t = 1; t < 4; ++t)  // the common lengths with their loads in flight together
        add4(g[r], load_or_zero(grad_rows + (int64_t)__shfl((int)vv[r], gbase + t, 64) * dim + col, has && fold && t < run_len));
      for (int t0 = 4; fold && t0 < run_len; t0 += 4) {  // (the halves of a wave may differ in their counts; a half reads its own lanes)
        float4 x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          x[u] = load_or_zero(grad_rows + (int64_t)__shfl((int)vv[r], gbase + min(t0 + u, 31), 64) * dim + col,
                              has && t0 + u < run_len);
#pragma unroll
        for (int u = 0; u < 4; ++u) add4(g[r], x[u]);
      }
    }
  }
  int long_r = -1;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!head[r]) continue;
    const int64_t i = first + r;
    const uint64_t row = half_bcast_u64(kk[r], gbase) >> kbits;
    const uint32_t in_row = (uint32_t)(__ballot(i + gl < n && (kk[r] >> kbits) == row) >> gbase);
    if (in_row != 0xffffffffu) {
      // the row ends inside the window: its runs are known from the keys in registers
      const int len = __ffs((int)~in_row) - 1;
      const uint64_t up = __shfl_up((unsigned long long)kk[r], 1, 64);
      uint32_t heads = (uint32_t)(__ballot(gl < len && (gl == 0 || up != kk[r])) >> gbase);  // first position of every run
      heads &= heads - 1;
      while (heads != 0u) {  // the next run's row is in flight while this one is applied
        const int a = __ffs((int)heads) - 1;
        heads &= heads - 1;
        const float4 next = load_or_zero(grad_rows + (int64_t)__shfl((int)vv[r], gbase + a, 64) * dim + col, has);
        gsum[r] = adagrad_apply_half<COSB>(w[r], g[r], gsum[r], fdim, lr, y[r], inv[r]);
        g[r] = next;
      }
      gsum[r] = adagrad_apply_half<COSB>(w[r], g[r], gsum[r], fdim, lr, y[r], inv[r]);
    } else if (kbits == 0) {  // a single-worker call has one run per row
      gsum[r] = adagrad_apply_half<COSB>(w[r], g[r], gsum[r], fdim, lr, y[r], inv[r]);
    } else {
      // A long row: handled after this loop.  There is at most one per half wave (the
      // positions after its head belong to it), so the code below exists once
      // instead of once per position.
      long_r = r;
      continue;
    }
    if (has) *reinterpret_cast<float4*>(wrow[r]) = w[r];
    if (gl == 0) *gptr[r] = gsum[r];
  }
  if (long_r < 0) return;
  // (only the position is carried out of the loop above: the row's weights, sum
  // and first gradient are fetched again rather than held in registers by every
  // half wave that has no long row)
  const int64_t long_i = first + long_r;
  const uint64_t long_row = keys[long_i] >> kbits;
  float* long_wrow;
  float* long_gptr;
  if ((int64_t)long_row < rows0) {
    long_wrow = w0 + (int64_t)long_row * dim + col;
    long_gptr = g0 + long_row;
  } else {
    long_wrow = w1 + ((int64_t)long_row - rows0) * dim + col;
    long_gptr = g1 + ((int64_t)long_row - rows0);
  }
  float4 long_y = make_float4(0.f, 0.f, 0.f, 0.f);
  float long_inv = 0.f;
  if (COSB) {
    const bool t0 = (int64_t)long_row < rows0;
    long_y = load_or_zero((t0 ? cb.y0 + (int64_t)long_row * dim : cb.y1 + ((int64_t)long_row - rows0) * dim) + col, has);
    long_inv = t0 ? cb.inv0[long_row] : cb.inv1[(int64_t)long_row - rows0];
  }
  float4 long_w = load_or_zero(long_wrow, has);
  float long_gsum = *long_gptr;
  float4 long_g = load_or_zero(grad_rows + (int64_t)vals[long_i] * dim + col, has);
  // A long row (a hot entity of a power-law graph): one run per batch that names
  // it.  Lane l finds the first position of batch b0 + l by binary search in the
  // sorted keys, 32 batches at once, and fetches the number of the gradient row
  // there; the runs are then applied in batch order with the next run's gradient
  // in flight.  (Walking the runs one after the other costs two dependent memory
  // round trips per 32 positions.)
  const int nb = 1 << kbits;
  const int64_t row_end = lower_bound_key(keys, long_i, n, (long_row + 1) << kbits);
  // (The starts do not decrease with the batch, and an absent batch has the start of the next one present: the runs
  // still to apply are the starts that differ from the one before them -- from 0, the run in hand, for the first.)
  uint32_t last_st = 0;  // the start of the last batch of the 32 before
  constexpr int kAhead = 8;  // gradient rows in flight: a hot row's runs are otherwise one memory round trip each
#pragma unroll 1
  for (int b0 = 0; b0 < nb; b0 += 32) {
    const int b = b0 + gl;
    const int64_t at = b < nb ? lower_bound_key(keys, long_i, row_end, (long_row << kbits) | (uint64_t)b) : row_end;
    const uint32_t st = (uint32_t)(at - long_i);    // first position of batch b (of the next batch present, if absent)
    const uint32_t sv = vals[at < n ? at : n - 1];  // and the gradient row there
    uint32_t st_prev = (uint32_t)__shfl_up((int)st, 1, 32);
    if (gl == 0) st_prev = last_st;
    uint32_t todo = (uint32_t)(__ballot(b < nb && st != st_prev && (int64_t)st < row_end - long_i) >> gbase);
    last_st = (uint32_t)__shfl((int)st, gbase + 31, 64);
#pragma unroll 1
    while (todo != 0u) {
      int js[kAhead];
      float4 nx[kAhead];
#pragma unroll
      for (int t = 0; t < kAhead; ++t) {
        js[t] = todo != 0u ? __ffs((int)todo) - 1 : -1;
        todo &= todo - 1;  // (0 stays 0)
      }
#pragma unroll
      for (int t = 0; t < kAhead; ++t) {
        const uint32_t v_b = (uint32_t)__shfl((int)sv, gbase + (js[t] >= 0 ? js[t] : 0), 64);
        nx[t] = load_or_zero(grad_rows + (int64_t)v_b * dim + col, has && js[t] >= 0);
      }
#pragma unroll
      for (int t = 0; t < kAhead; ++t) {
        if (js[t] < 0) break;
        long_gsum = adagrad_apply_half<COSB>(long_w, long_g, long_gsum, fdim, lr, long_y, long_inv);
        long_g = nx[t];
      }
    }
  }
  long_gsum = adagrad_apply_half<COSB>(long_w, long_g, long_gsum, fdim, lr, long_y, long_inv);
  if (has) *reinterpret_cast<float4*>(long_wrow) = long_w;
  if (gl == 0) *long_gptr = long_gsum;
}

// ---- dense branches ------------------------------------------------------------
__global__ __launch_bounds__(kRowThreads) void row_adagrad_dense_kernel(float* __restrict__ w, float* __restrict__ gs,
                                                                        int64_t num_rows, int dim,
                                                                        const float* __restrict__ grad, float lr) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  if (r >= num_rows) return;
  const float* g = grad + r * (int64_t)dim;
  float sq = 0.f;
  for (int d = lane; d < dim; d += kWave) sq += g[d] * g[d];
  const float delta = wave_sum(sq) / (float)dim;
  const float gsum = gs[r] + delta;
  const float stdv = sqrtf(gsum) + 1e-10f;
  float* wr = w + r * (int64_t)dim;
  for (int d = lane; d < dim; d += kWave) wr[d] += -lr * (g[d] / stdv);
  if (lane == 0) gs[r] = gsum;
}

__global__ void async_adagrad_dense_kernel(float* __restrict__ p, float* __restrict__ s, const float* __restrict__ g,
                                           int64_t numel, float lr, float eps) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= numel) return;
  const float gi = g[i];
  const float sum = s[i] + gi * gi;
  s[i] = sum;
  p[i] += -lr * (gi / (sqrtf(sum) + eps));
}

template <bool VEC, bool COSB>
int launch_sorted(int nvec, const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, float* grad_rows,
                  int dim, float* w0, float* g0, int64_t rows0, float* w1, float* g1, int64_t rows1, float lr,
                  const uint32_t* long_runs, CosBack cb, BatchSums sums, hipStream_t stream) {
  const int wpb = kRowThreads / kWave;
  const dim3 block(kRowThreads);
  const unsigned tile_blocks = (unsigned)ceil_div(ceil_div(n, kTile), wpb);
  const dim3 tile_grid(tile_blocks + (unsigned)sums.batches);
  const int64_t borders = ceil_div(n, kTile) - 1;
  const dim3 border_grid((unsigned)ceil_div(borders > 0 ? borders : 1, wpb));
  // gradient rows outnumbering the tables' rows 32 times over: a wave per table row (row_walk_kernel)
  const int64_t table_rows = rows0 + rows1;
  const bool walk = kbits > 0 && table_rows > 0 && n >= 32 * table_rows && getenv("PBG_DISABLE_ROW_WALK") == nullptr;
  const dim3 walk_grid((unsigned)ceil_div(table_rows > 0 ? table_rows : 1, wpb));
  const int leave_mode = walk ? 2 : (kbits == 0 ? 1 : 0);
#define PBG_LAUNCH(NV)                                                                                             \
  do {                                                                                                             \
    hipLaunchKernelGGL((tile_reduce_kernel<NV, VEC>), tile_grid, block, 0, stream, keys, vals, n, grad_rows, dim,       \
                       leave_mode, long_runs, sums, tile_blocks);                                                  \
    if (borders > 0)                                                                                              \
      hipLaunchKernelGGL((run_combine_kernel<NV, VEC>), border_grid, block, 0, stream, keys, vals, n, grad_rows, dim,  \
                         leave_mode, long_runs);                                                                   \
    if (walk) {                                                                                                    \
      constexpr int R = NV <= 2 ? 8 : (NV <= 4 ? 4 : 2);                                                           \
      hipLaunchKernelGGL((row_walk_kernel<NV, VEC, R, COSB>), walk_grid, block, 0, stream, keys, vals, n, kbits,      \
                         grad_rows, dim, w0, g0, rows0, w1, g1, rows1, lr, cb);                                    \
    } else if (VEC && dim <= 128) {                                                                                \
      constexpr int R = 4;                                                                                         \
      const dim3 hgrid((unsigned)ceil_div(ceil_div(n, R) * 32, kRowThreads));                                      \
      hipLaunchKernelGGL((row_update_half_kernel<R, COSB>), hgrid, block, 0, stream, keys, vals, n, kbits,        \
                         grad_rows, dim, w0, g0, rows0, w1, g1, rows1, lr, cb);                                    \
    } else {                                                                                                       \
      constexpr int R = NV <= 2 ? 4 : (NV <= 4 ? 2 : 1);                                                           \
      const dim3 ugrid((unsigned)ceil_div(ceil_div(n, R), wpb));                                                   \
      hipLaunchKernelGGL((row_update_kernel<NV, VEC, R, COSB>), ugrid, block, 0, stream, keys, vals, n, kbits,    \
                         grad_rows, dim, w0, g0, rows0, w1, g1, rows1, lr, cb);                                    \
    }                                                                                                              \
  } while (0)
  if (nvec <= 1) PBG_LAUNCH(1);
  else if (nvec <= 2) PBG_LAUNCH(2);
  else if (nvec <= 4) PBG_LAUNCH(4);
  else if (nvec <= 8) PBG_LAUNCH(8);
  else if (nvec <= 16) PBG_LAUNCH(16);
  else if constexpr (!VEC) {  // (a dim that is no multiple of 4: one float per lane and register)
    if (nvec <= 32) PBG_LAUNCH(32);
    else if (nvec <= 64) PBG_LAUNCH(64);
    else return fail(PBG_ERR_UNSUPPORTED, "row_adagrad: dim %d too large", dim);
  } else return fail(PBG_ERR_UNSUPPORTED, "row_adagrad: dim %d too large", dim);
#undef PBG_LAUNCH
  return PBG_OK;
}

}  // namespace

int row_adagrad_sorted(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, float* grad_rows,
                       int dim, float* w0, float* g0, int64_t rows0, float* w1, float* g1, int64_t rows1, float lr,
                       hipStream_t stream, const uint32_t* long_runs, const CosBack* cos_back, const BatchSums* sums_in) {
  const BatchSums sums = sums_in ? *sums_in : BatchSums{nullptr, nullptr, 0, 0, nullptr, nullptr};
  if (n <= 0) {  // no gradient rows: a launch that only carries the sums, if any
    if (sums.batches > 0) {
      hipLaunchKernelGGL((tile_reduce_kernel<1, true>), dim3((unsigned)sums.batches), dim3(kRowThreads), 0, stream, keys, vals,
                         (int64_t)0, grad_rows, dim, 0, (const uint32_t*)nullptr, sums, 0u);
      return check_launch("row_adagrad_sorted");
    }
    return PBG_OK;
  }
  int rc;
  const CosBack none{nullptr, nullptr, nullptr, nullptr};
  if (cos_back) {
    if (dim % 4 != 0) return fail(PBG_ERR_UNSUPPORTED, "row_adagrad: the normalisation backward needs dim %% 4 == 0");
    rc = launch_sorted<true, true>((int)ceil_div(dim / 4, kWave), keys, vals, n, kbits, grad_rows, dim, w0, g0, rows0, w1,
                                   g1, rows1, lr, long_runs, *cos_back, sums, stream);
  } else if (dim % 4 == 0) {
    rc = launch_sorted<true, false>((int)ceil_div(dim / 4, kWave), keys, vals, n, kbits, grad_rows, dim, w0, g0, rows0, w1,
                                    g1, rows1, lr, long_runs, none, sums, stream);
  } else {
    rc = launch_sorted<false, false>((int)ceil_div(dim, kWave), keys, vals, n, kbits, grad_rows, dim, w0, g0, rows0, w1, g1,
                                     rows1, lr, long_runs, none, sums, stream);
  }
  if (rc != PBG_OK) return rc;
  return check_launch("row_adagrad_sorted");
}

}  // namespace pbg

using namespace pbg;

extern "C" int pbg_gather_rows(const float* table, int64_t num_rows, int32_t dim, const int64_t* idx, int64_t n,
                               float* out, int32_t* oob_flag, pbg_stream_t stream) {
  if (n < 0 || dim <= 0 || num_rows < 0) return fail(PBG_ERR_INVALID, "pbg_gather_rows: bad sizes");
  if (n == 0) return PBG_OK;
  if (!table || !idx || !out) return fail(PBG_ERR_INVALID, "pbg_gather_rows: null pointer");
  const dim3 grid((unsigned)ceil_div(n, kRowThreads / kWave)), block(kRowThreads);
  hipStream_t s = (hipStream_t)stream;
  const bool vec = dim % 4 == 0 && ((uintptr_t)table % 16 == 0) && ((uintptr_t)out % 16 == 0);
  if (vec && dim <= 256) {
    constexpr int kU = 8;
    const int waves_per_block = kRowThreads / kWave;
    if (dim <= 64) {
      const dim3 g((unsigned)ceil_div(n, (int64_t)waves_per_block * 4 * kU));
      hipLaunchKernelGGL((gather_rows_multi_kernel<16, kU>), g, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
    } else if (dim <= 128) {
      const dim3 g((unsigned)ceil_div(n, (int64_t)waves_per_block * 2 * kU));
      hipLaunchKernelGGL((gather_rows_multi_kernel<32, kU>), g, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
    } else {
      const dim3 g((unsigned)ceil_div(n, (int64_t)waves_per_block * kU));
      hipLaunchKernelGGL((gather_rows_multi_kernel<64, kU>), g, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
    }
  } else if (vec) {
    hipLaunchKernelGGL(gather_rows_kernel<true>, grid, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
  } else {
    hipLaunchKernelGGL(gather_rows_kernel<false>, grid, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
  }
  return check_launch("pbg_gather_rows");
}

namespace {
// torch.embedding_renorm_ (what F.embedding(max_norm=...) runs first, model.py:61,90-96) in two
// passes, so that no wave reads a row that another is rewriting: the first only reads the
// table and keeps a too-long row and its scale per index, the second writes row * scale.
// Equal indices keep the same row and scale and write the same bytes.  One wave per index.
__global__ __launch_bounds__(kRowThreads) void renorm_scan_kernel(const float* __restrict__ table, int64_t num_rows,
                                                                  int dim, const int64_t* __restrict__ idx, int64_t n,
                                                                  float max_norm, float* __restrict__ kept,
                                                                  float* __restrict__ scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t i = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  if (i >= n) return;
  const int64_t id = idx[i];
  float sc = 0.f;
  if (id >= 0 && id < num_rows) {
    const float* row = table + id * dim;
    float sq = 0.f;
    for (int d = lane; d < dim; d += kWave) sq += row[d] * row[d];
    const float norm = sqrtf(wave_sum(sq));
    if (norm > max_norm) {
      sc = max_norm / (norm + 1e-7f);
      for (int d = lane; d < dim; d += kWave) kept[i * dim + d] = row[d];
    }
  }
  if (lane == 0) scale[i] = sc;
}

__global__ __launch_bounds__(kRowThreads) void renorm_apply_kernel(float* __restrict__ table, int dim,
                                                                   const int64_t* __restrict__ idx, int64_t n,
                                                                   const float* __restrict__ kept,
                                                                   const float* __restrict__ scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t i = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  if (i >= n) return;
  const float sc = scale[i];
  if (sc == 0.f) return;
  float* row = table + idx[i] * dim;
  for (int d = lane; d < dim; d += kWave) row[d] = kept[i * dim + d] * sc;
}
}  // namespace

extern "C" size_t pbg_embedding_renorm_workspace_bytes(int64_t n, int32_t dim) {
  const size_t nn = (size_t)(n > 0 ? n : 1);
  return align_up(nn * (size_t)(dim > 0 ? dim : 1) * sizeof(float), 256) + align_up(nn * sizeof(float), 256);
}

extern "C" int pbg_embedding_renorm(float* table, int64_t num_rows, int32_t dim, const int64_t* idx, int64_t n,
                                    float max_norm, void* workspace, size_t workspace_bytes, pbg_stream_t stream) {
  if (n < 0 || dim <= 0 || num_rows < 0) return fail(PBG_ERR_INVALID, "pbg_embedding_renorm: bad sizes");
  if (!(max_norm > 0.f)) return fail(PBG_ERR_INVALID, "pbg_embedding_renorm: max_norm must be positive");
  if (n == 0) return PBG_OK;
  if (!table || !idx) return fail(PBG_ERR_INVALID, "pbg_embedding_renorm: null pointer");
  if (!workspace || workspace_bytes < pbg_embedding_renorm_workspace_bytes(n, dim))
    return fail(PBG_ERR_WORKSPACE, "pbg_embedding_renorm: workspace needs %zu bytes, got %zu",
                pbg_embedding_renorm_workspace_bytes(n, dim), workspace_bytes);
  float* kept = (float*)workspace;
  float* scale = (float*)((char*)workspace + align_up((size_t)n * dim * sizeof(float), 256));
  const dim3 grid((unsigned)ceil_div(n, kRowThreads / kWave)), block(kRowThreads);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(renorm_scan_kernel, grid, block, 0, s, table, num_rows, dim, idx, n, max_norm, kept, scale);
  hipLaunchKernelGGL(renorm_apply_kernel, grid, block, 0, s, table, dim, idx, n, kept, scale);
  return check_launch("pbg_embedding_renorm");
}

namespace {
struct SparseWs {
  uint64_t* keys_a; uint64_t* keys_b; uint32_t* vals_a; uint32_t* vals_b; void* temp;
  size_t total;
};
SparseWs carve_sparse(void* base, int64_t n) {
  SparseWs w;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return (char*)base + o; };
  const size_t nn = (size_t)(n > 0 ? n : 1);
  w.keys_a = (uint64_t*)take(nn * 8);
  w.keys_b = (uint64_t*)take(nn * 8);
  w.vals_a = (uint32_t*)take(nn * 4);
  w.vals_b = (uint32_t*)take(nn * 4);
  w.temp = take(sort_temp_bytes(n));
  w.total = off;
  return w;
}
}  // namespace

extern "C" size_t pbg_row_adagrad_sparse_workspace_bytes(int64_t n) { return carve_sparse(nullptr, n).total; }

extern "C" int pbg_row_adagrad_sparse(float* weight, float* state_sum, int64_t num_rows, int32_t dim,
                                      const int64_t* idx, float* grad_rows, int64_t n, float lr,
                                      void* workspace, size_t workspace_bytes, pbg_stream_t stream) {
  if (n < 0 || dim <= 0 || num_rows < 0) return fail(PBG_ERR_INVALID, "pbg_row_adagrad_sparse: bad sizes");
  if (n == 0) return PBG_OK;  // row_adagrad.py:81-82
  if (!weight || !state_sum || !idx || !grad_rows) return fail(PBG_ERR_INVALID, "pbg_row_adagrad_sparse: null pointer");
  if ((uintptr_t)weight % 16 != 0 || (uintptr_t)grad_rows % 16 != 0)
    return fail(PBG_ERR_INVALID, "pbg_row_adagrad_sparse: weight and grad_rows must be 16-byte aligned");
  SparseWs ws = carve_sparse(workspace, n);
  if (!workspace || workspace_bytes < ws.total)
    return fail(PBG_ERR_WORKSPACE, "pbg_row_adagrad_sparse: workspace needs %zu bytes", ws.total);
  hipStream_t s = (hipStream_t)stream;
  uint64_t* skeys;
  uint32_t* svals;
  const uint32_t* long_runs;
  int rc = sort_pairs(ws.keys_a, ws.vals_a, ws.keys_b, ws.vals_b, n, 0, bits_for((uint64_t)num_rows), ws.temp, s,
                      &skeys, &svals, &long_runs, idx, num_rows);
  if (rc != PBG_OK) return rc;
  // out-of-range indices are parked at key == num_rows and are skipped by the update
  return row_adagrad_sorted(skeys, svals, n, 0, grad_rows, dim, weight, state_sum, num_rows, nullptr,
                            nullptr, 0, lr, s, long_runs);
}

// ---------------------------------------------------------------------------
// The same step for callers that cannot allocate (HIP graph capture, serving loops):
// the sort's keys, values and counters live in a file-scope device array instead of
// a caller-provided workspace.  Every GPU holds its own copy of the array at its own
// address, looked up once per device; all calls on a GPU share it.
// ---------------------------------------------------------------------------
namespace {
constexpr int64_t kStaticMaxIndices = (int64_t)1 << 20;
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;  // 24 bytes per index + the sort's counters
}  // namespace

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (the symbol's name is a host-side
// stand-in, not an address a kernel can use).
int static_scratch(void** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail(PBG_ERR_LAUNCH, "pbg_row_adagrad_sparse_static: hipGetDevice: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= kMaxDevices) return fail(PBG_ERR_UNSUPPORTED, "pbg_row_adagrad_sparse_static: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr)
      return fail(PBG_ERR_LAUNCH, "pbg_row_adagrad_sparse_static: hipGetSymbolAddress: %s", hipGetErrorString(err));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return PBG_OK;
}
}  // namespace

extern "C" int64_t pbg_row_adagrad_sparse_static_max_indices(void) { return kStaticMaxIndices; }

extern "C" int pbg_row_adagrad_sparse_static(float* weight, float* state_sum, int64_t num_rows, int32_t dim,
                                             const int64_t* idx, float* grad_rows, int64_t n, float lr,
                                             pbg_stream_t stream) {
  if (n > kStaticMaxIndices)
    return fail(PBG_ERR_WORKSPACE, "pbg_row_adagrad_sparse_static: n = %lld exceeds the built-in scratch (at most %lld indices); "
                "use pbg_row_adagrad_sparse with a workspace", (long long)n, (long long)kStaticMaxIndices);
  if (n > 0 && carve_sparse(nullptr, n).total > kStaticScratchBytes)
    return fail(PBG_ERR_WORKSPACE, "pbg_row_adagrad_sparse_static: n = %lld needs more than the built-in scratch", (long long)n);
  void* ptr = nullptr;
  int rc = static_scratch(&ptr);
  if (rc != PBG_OK) return rc;
  // The sort clears its own counters and overwrites keys and values before it reads
  // them, so what the previous call left in the array does not matter.
  return pbg_row_adagrad_sparse(weight, state_sum, num_rows, dim, idx, grad_rows, n, lr, ptr, kStaticScratchBytes, stream);
}

extern "C" int pbg_row_adagrad_dense(float* weight, float* state_sum, int64_t num_rows, int32_t dim,
                                     const float* grad, float lr, pbg_stream_t stream) {
  if (dim <= 0 || num_rows < 0) return fail(PBG_ERR_INVALID, "pbg_row_adagrad_dense: bad sizes");
  if (num_rows == 0) return PBG_OK;
  if (!weight || !state_sum || !grad) return fail(PBG_ERR_INVALID, "pbg_row_adagrad_dense: null pointer");
  hipLaunchKernelGGL(row_adagrad_dense_kernel, dim3((unsigned)ceil_div(num_rows, kRowThreads / kWave)),
                     dim3(kRowThreads), 0, (hipStream_t)stream, weight, state_sum, num_rows, dim, grad, lr);
  return check_launch("pbg_row_adagrad_dense");
}

extern "C" int pbg_async_adagrad_dense(float* param, float* state_sum, const float* grad, int64_t numel, float lr,
                                       float eps, pbg_stream_t stream) {
  if (numel < 0) return fail(PBG_ERR_INVALID, "pbg_async_adagrad_dense: bad size");
  if (numel == 0) return PBG_OK;
  if (!param || !state_sum || !grad) return fail(PBG_ERR_INVALID, "pbg_async_adagrad_dense: null pointer");
  hipLaunchKernelGGL(async_adagrad_dense_kernel, dim3((unsigned)ceil_div(numel, 256)), dim3(256), 0,
                     (hipStream_t)stream, param, state_sum, grad, numel, lr, eps);
  return check_launch("pbg_async_adagrad_dense");
}
