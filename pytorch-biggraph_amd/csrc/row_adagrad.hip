// Row gather and RowAdagrad updates: bandwidth kernels.
//
// A row of `dim` floats is moved by one wavefront with 128-bit accesses when
// dim % 4 == 0 (lane l owns float4 number l, l + 64, ...), so a 400-byte row
// (dim 100) is one coalesced request of 25 lanes and a 4 KiB row (dim 1024) is
// four full-wave requests.
#include "pbg_internal.h"

namespace pbg {
namespace {

constexpr int kRowThreads = 256;  // 4 waves per block, one row per wave
constexpr int kMaxV4 = 4;         // float4 per lane: covers dim <= 1024

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

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
    for (int v = lane; v < nv; v += kWave) dst[v] = ok ? src[v] : make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    const float* src = table + (ok ? r : 0) * (int64_t)dim;
    float* dst = out + i * (int64_t)dim;
    for (int d = lane; d < dim; d += kWave) dst[d] = ok ? src[d] : 0.f;
  }
}

// ---- segmented RowAdagrad over sorted keys -----------------------------------
// One wave per sorted position; only the wave sitting on the first key of a row
// works.  It walks the row's keys: equal keys (same worker) are summed, then one
// Adagrad update is applied per worker in ascending worker order, exactly as if
// the workers' sparse steps had been applied one after another.
template <int NV, bool VEC>
__global__ __launch_bounds__(kRowThreads) void row_adagrad_sorted_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, int64_t n, int kbits,
    const float* __restrict__ grad_rows, int dim, float* __restrict__ w0, float* __restrict__ g0, int64_t rows0,
    float* __restrict__ w1, float* __restrict__ g1, int64_t rows1, float lr) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
  if (i >= n) return;
  const uint64_t row = keys[i] >> kbits;
  if (i > 0 && (keys[i - 1] >> kbits) == row) return;
  if ((int64_t)row >= rows0 + rows1) return;  // out-of-range indices are parked past both tables

  float* wrow;
  float* gptr;
  if ((int64_t)row < rows0) {
    wrow = w0 + (int64_t)row * dim;
    gptr = g0 + row;
  } else {
    wrow = w1 + ((int64_t)row - rows0) * dim;
    gptr = g1 + ((int64_t)row - rows0);
  }
  constexpr int W = VEC ? 4 : 1;
  float w[NV * W];
  const int nv = VEC ? (dim >> 2) : dim;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int e = v * kWave + lane;
    if (VEC) {
      float4 x = (e < nv) ? reinterpret_cast<const float4*>(wrow)[e] : make_float4(0.f, 0.f, 0.f, 0.f);
      w[v * 4 + 0] = x.x; w[v * 4 + 1] = x.y; w[v * 4 + 2] = x.z; w[v * 4 + 3] = x.w;
    } else {
      w[v] = (e < nv) ? wrow[e] : 0.f;
    }
  }
  float gsum = *gptr;
  const float fdim = (float)dim;
  int64_t j = i;
  while (j < n && (keys[j] >> kbits) == row) {
    const uint64_t key = keys[j];
    float g[NV * W];
#pragma unroll
    for (int q = 0; q < NV * W; ++q) g[q] = 0.f;
    while (j < n && keys[j] == key) {
      const float* grow = grad_rows + (int64_t)vals[j] * dim;
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const int e = v * kWave + lane;
        if (e < nv) {
          if (VEC) {
            float4 x = reinterpret_cast<const float4*>(grow)[e];
            g[v * 4 + 0] += x.x; g[v * 4 + 1] += x.y; g[v * 4 + 2] += x.z; g[v * 4 + 3] += x.w;
          } else {
            g[v] += grow[e];
          }
        }
      }
      ++j;
    }
    float sq = 0.f;
#pragma unroll
    for (int q = 0; q < NV * W; ++q) sq += g[q] * g[q];
    const float delta = wave_sum(sq) / fdim;
    gsum += delta;
    const float stdv = sqrtf(gsum) + 1e-10f;
#pragma unroll
    for (int q = 0; q < NV * W; ++q) w[q] += (-lr * g[q]) / stdv;
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int e = v * kWave + lane;
    if (e < nv) {
      if (VEC) {
        reinterpret_cast<float4*>(wrow)[e] = make_float4(w[v * 4 + 0], w[v * 4 + 1], w[v * 4 + 2], w[v * 4 + 3]);
      } else {
        wrow[e] = w[v];
      }
    }
  }
  if (lane == 0) *gptr = gsum;
}

// keys for the stand-alone sparse step: key = row index, value = position
__global__ void make_keys_kernel(const int64_t* __restrict__ idx, int64_t n, int64_t num_rows,
                                 uint64_t* __restrict__ keys, uint32_t* __restrict__ vals) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t r = idx[i];
  if (r < 0 || r >= num_rows) r = num_rows;  // parked past the table, skipped by the update
  keys[i] = (uint64_t)r;
  vals[i] = (uint32_t)i;
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

template <bool VEC>
int launch_sorted(int nvec, const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, const float* grad_rows,
                  int dim, float* w0, float* g0, int64_t rows0, float* w1, float* g1, int64_t rows1, float lr,
                  hipStream_t stream) {
  const dim3 grid((unsigned)ceil_div(n, kRowThreads / kWave)), block(kRowThreads);
#define PBG_LAUNCH(NV)                                                                                          \
  hipLaunchKernelGGL((row_adagrad_sorted_kernel<NV, VEC>), grid, block, 0, stream, keys, vals, n, kbits, grad_rows, \
                     dim, w0, g0, rows0, w1, g1, rows1, lr)
  if (nvec <= 1) PBG_LAUNCH(1);
  else if (nvec <= 2) PBG_LAUNCH(2);
  else if (nvec <= 4) PBG_LAUNCH(4);
  else if (nvec <= 8) PBG_LAUNCH(8);
  else if (nvec <= 16) PBG_LAUNCH(16);
  else return fail(PBG_ERR_UNSUPPORTED, "row_adagrad: dim %d too large", dim);
#undef PBG_LAUNCH
  return PBG_OK;
}

}  // namespace

int row_adagrad_sorted(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, const float* grad_rows,
                       int dim, float* w0, float* g0, int64_t rows0, float* w1, float* g1, int64_t rows1, float lr,
                       hipStream_t stream) {
  if (n <= 0) return PBG_OK;
  int rc;
  if (dim % 4 == 0) {
    rc = launch_sorted<true>((int)ceil_div(dim / 4, kWave), keys, vals, n, kbits, grad_rows, dim, w0, g0, rows0, w1,
                             g1, rows1, lr, stream);
  } else {
    rc = launch_sorted<false>((int)ceil_div(dim, kWave), keys, vals, n, kbits, grad_rows, dim, w0, g0, rows0, w1, g1,
                              rows1, lr, stream);
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
  if (vec) {
    hipLaunchKernelGGL(gather_rows_kernel<true>, grid, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
  } else {
    hipLaunchKernelGGL(gather_rows_kernel<false>, grid, block, 0, s, table, num_rows, dim, idx, n, out, oob_flag);
  }
  return check_launch("pbg_gather_rows");
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
                                      const int64_t* idx, const float* grad_rows, int64_t n, float lr,
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
  hipLaunchKernelGGL(make_keys_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s, idx, n, num_rows, ws.keys_a,
                     ws.vals_a);
  int rc = sort_pairs(ws.keys_a, ws.vals_a, ws.keys_b, ws.vals_b, n, bits_for((uint64_t)num_rows), ws.temp, s);
  if (rc != PBG_OK) return rc;
  // out-of-range indices were parked at key == num_rows and are skipped by the update
  return row_adagrad_sorted(ws.keys_b, ws.vals_b, n, 0, grad_rows, dim, weight, state_sum, num_rows, nullptr,
                            nullptr, 0, lr, s);
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
