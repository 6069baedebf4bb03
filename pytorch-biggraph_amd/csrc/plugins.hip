// Stand-alone forward / backward kernels behind the plugin classes: relation
// operators, comparators and loss functions called one at a time (as the
// reference's own unit tests do).  The training step does not use these: it
// runs the fused pipeline of step.hip.
#include "pbg_internal.h"
#include "row_ops.h"

namespace pbg {
namespace {

constexpr int kRowThreads = 256;
constexpr int kWavesPerBlock = kRowThreads / kWave;

dim3 wave_grid(int64_t jobs) { return dim3((unsigned)ceil_div(jobs > 0 ? jobs : 1, kWavesPerBlock)); }

#define PBG_DISPATCH_NVH(nvh, KERNEL, grid, stream, ...)                                                    \
  do {                                                                                                     \
    if ((nvh) <= 1) hipLaunchKernelGGL((KERNEL<1>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);        \
    else if ((nvh) <= 2) hipLaunchKernelGGL((KERNEL<2>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);   \
    else if ((nvh) <= 4) hipLaunchKernelGGL((KERNEL<4>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);   \
    else if ((nvh) <= 8) hipLaunchKernelGGL((KERNEL<8>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);   \
    else if ((nvh) <= 16) hipLaunchKernelGGL((KERNEL<16>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__); \
    else hipLaunchKernelGGL((KERNEL<32>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);                  \
  } while (0)

int nvh_for(int dim) { return (int)ceil_div((dim + 1) / 2, kWave); }

// ---------------------------------------------------------------------------
// operators
// ---------------------------------------------------------------------------
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void operator_forward_kernel(int op, int D, int64_t n,
                                                                       const float* __restrict__ x,
                                                                       const float* __restrict__ p0,
                                                                       const float* __restrict__ p1,
                                                                       const int64_t* __restrict__ rel, int64_t num_ops,
                                                                       float* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  const int H = (D + 1) / 2;
  const int64_t r = rel ? clamp_index(rel[i], num_ops) : 0;
  const RowV<NVH> xr = row_load<NVH>(x + i * D, D, H, lane);
  row_store<NVH>(y + i * D, op_forward<NVH>(op, xr, p0, p1, r, D, H, lane), D, H, lane);
}

// dx for every row; parameter gradients accumulated with float atomics (the
// caller zero-fills dp0 / dp1).  A static operator first sums over the rows a
// wave visits, so it issues one atomic per element and wave.
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void operator_backward_kernel(
    int op, int D, int64_t n, const float* __restrict__ x, const float* __restrict__ dy, const float* __restrict__ p0,
    const float* __restrict__ p1, const int64_t* __restrict__ rel, int64_t num_ops, float* __restrict__ dx,
    float* __restrict__ dp0, float* __restrict__ dp1) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
  const int H = (D + 1) / 2;
  RowV<NVH> acc0 = row_zero<NVH>();  // static operator: running parameter gradient (p0 | real)
  RowV<NVH> acc1 = row_zero<NVH>();  // complex: imag, stored in a[0]
  auto flush = [&](int64_t r, const RowV<NVH>& g0, const RowV<NVH>& g1) {
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      const int h = v * kWave + lane;
      if (h >= H) continue;
      if (op == PBG_OP_COMPLEX_DIAGONAL) {
        atomicAdd(&dp0[r * H + h], g0.a[0][v]);
        atomicAdd(&dp1[r * H + h], g1.a[0][v]);
      } else {
        atomicAdd(&dp0[r * D + h], g0.a[0][v]);
        if (H + h < D) atomicAdd(&dp0[r * D + H + h], g0.a[1][v]);
      }
    }
  };
  for (int64_t i = wave; i < n; i += nwaves) {
    const int64_t r = rel ? clamp_index(rel[i], num_ops) : 0;
    const RowV<NVH> g = row_load<NVH>(dy + i * D, D, H, lane);
    row_store<NVH>(dx + i * D, op_backward<NVH>(op, g, p0, p1, r, D, H, lane), D, H, lane);
    if (op == PBG_OP_NONE) continue;
    RowV<NVH> g0 = row_zero<NVH>(), g1 = row_zero<NVH>();
    if (op == PBG_OP_TRANSLATION) {
      g0 = g;
    } else {
      const RowV<NVH> xr = row_load<NVH>(x + i * D, D, H, lane);
#pragma unroll
      for (int v = 0; v < NVH; ++v) {
        if (op == PBG_OP_DIAGONAL) {
          g0.a[0][v] = xr.a[0][v] * g.a[0][v];
          g0.a[1][v] = xr.a[1][v] * g.a[1][v];
        } else {  // complex: d/d real, d/d imag
          g0.a[0][v] = xr.a[0][v] * g.a[0][v] + xr.a[1][v] * g.a[1][v];
          g1.a[0][v] = xr.a[0][v] * g.a[1][v] - xr.a[1][v] * g.a[0][v];
        }
      }
    }
    if (rel) {
      flush(r, g0, g1);
    } else {
      row_axpy<NVH>(acc0, 1.0f, g0);
      row_axpy<NVH>(acc1, 1.0f, g1);
    }
  }
  if (!rel && op != PBG_OP_NONE) flush(0, acc0, acc1);
}

// dynamic `linear`: y_i = W[rel_i] x_i, one wave per row (operators.py:259-269)
__global__ __launch_bounds__(kRowThreads) void linear_rows_forward_kernel(int D, int64_t n, const float* __restrict__ x,
                                                                          const float* __restrict__ w,
                                                                          const int64_t* __restrict__ rel,
                                                                          int64_t num_ops, float* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  const float* m = w + clamp_index(rel[i], num_ops) * D * D;
  const float* xr = x + i * D;
  for (int o = 0; o < D; ++o) {
    float acc = 0.f;
    for (int d = lane; d < D; d += kWave) acc += m[(int64_t)o * D + d] * xr[d];
    acc = wave_sum(acc);
    if (lane == 0) y[i * D + o] = acc;
  }
}

// dx_i = W[rel_i]^T dy_i ; dW[rel_i] += dy_i x_i^T (atomics)
__global__ __launch_bounds__(kRowThreads) void linear_rows_backward_kernel(int D, int64_t n, const float* __restrict__ x,
                                                                           const float* __restrict__ dy,
                                                                           const float* __restrict__ w,
                                                                           const int64_t* __restrict__ rel,
                                                                           int64_t num_ops, float* __restrict__ dx,
                                                                           float* __restrict__ dw) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  const int64_t r = clamp_index(rel[i], num_ops);
  const float* m = w + r * D * D;
  float* gm = dw + r * D * D;
  const float* xr = x + i * D;
  const float* g = dy + i * D;
  for (int d = lane; d < D; d += kWave) {
    float acc = 0.f;
    const float xd = xr[d];
    for (int o = 0; o < D; ++o) {
      const float go = g[o];
      acc += m[(int64_t)o * D + d] * go;
      atomicAdd(&gm[(int64_t)o * D + d], go * xd);
    }
    dx[i * D + d] = acc;
  }
}

// ---------------------------------------------------------------------------
// comparators
// ---------------------------------------------------------------------------
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void prepare_kernel(int cmp, int D, int64_t n, const float* __restrict__ x,
                                                              float* __restrict__ y, float* __restrict__ aux) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  const int H = (D + 1) / 2;
  RowV<NVH> r = row_load<NVH>(x + i * D, D, H, lane);
  const float a = prepare_row<NVH>(cmp, r);
  if (y) row_store<NVH>(y + i * D, r, D, H, lane);
  if (aux && lane == 0) aux[i] = a;
}

template <int NVH>
__global__ __launch_bounds__(kRowThreads) void prepare_backward_kernel(int cmp, int D, int64_t n,
                                                                       const float* __restrict__ dy,
                                                                       const float* __restrict__ y,
                                                                       const float* __restrict__ aux,
                                                                       float* __restrict__ dx) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  const int H = (D + 1) / 2;
  const RowV<NVH> g = row_load<NVH>(dy + i * D, D, H, lane);
  const RowV<NVH> yr = row_load<NVH>(y + i * D, D, H, lane);
  row_store<NVH>(dx + i * D, prepare_backward<NVH>(cmp, g, yr, aux ? aux[i] : 0.f), D, H, lane);
}

// pos[i] = kappa(lp_i, rp_i) (model.py:177,207,267-274)
__global__ __launch_bounds__(kRowThreads) void pos_scores_kernel(int cmp, int D, int64_t n, const float* __restrict__ lp,
                                                                 const float* __restrict__ rp, float* __restrict__ pos) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  float acc = 0.f;
  const float* a = lp + i * D;
  const float* b = rp + i * D;
  if (cmp == PBG_CMP_L2 || cmp == PBG_CMP_SQUARED_L2) {
    for (int d = lane; d < D; d += kWave) {
      const float t = a[d] - b[d];
      acc += t * t;
    }
    acc = wave_sum(acc);
    acc = cmp == PBG_CMP_L2 ? -sqrtf(fmaxf(acc, 1e-30f)) : -acc;  // model.py:267-274 | :300
  } else {
    for (int d = lane; d < D; d += kWave) acc += a[d] * b[d];
    acc = wave_sum(acc);
  }
  if (lane == 0) pos[i] = acc;
}

// l2 epilogue (model.py:228-246): s[c,i,j] <- -sqrt(max(a2[c,i] - 2 s + b2[c,j], 1e-30));
// squared_l2 (model.py:228-236,301-302): s[c,i,j] <- -(a2[c,i] - 2 s + b2[c,j])
__global__ void l2_epilogue_kernel(int cmp, float* __restrict__ s, const float* __restrict__ a2,
                                   const float* __restrict__ b2, int64_t chunks, int P, int N) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= chunks * P * N) return;
  const int64_t row = e / N;  // c * P + i
  const int j = (int)(e % N);
  const int64_t c = row / P;
  const float q = fmaf(-2.0f, s[e], b2[c * N + j]) + a2[row];
  s[e] = cmp == PBG_CMP_L2 ? -sqrtf(fmaxf(q, 1e-30f)) : -q;
}

// l2 backward, step 1: g[c,i,j] (dLoss/dscore) -> -2 dLoss/dq in `out`; rowsum of dLoss/dq
__global__ __launch_bounds__(kRowThreads) void l2_grad_kernel(int cmp, const float* __restrict__ g,
                                                              const float* __restrict__ score, int64_t rows, int N,
                                                              float* __restrict__ out, float* __restrict__ rowsum) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  float acc = 0.f;
  for (int j = lane; j < N; j += kWave) {
    const float t = score[row * N + j];
    // score = -sqrt(q): dq = g / (2 score), none where the clamp is active; score = -q: dq = -g
    const float dq = cmp == PBG_CMP_SQUARED_L2 ? -g[row * N + j] : ((t * t > 1e-30f) ? g[row * N + j] * 0.5f / t : 0.f);
    acc += dq;
    out[row * N + j] = -2.0f * dq;
  }
  acc = wave_sum(acc);
  if (lane == 0) rowsum[row] = acc;
}

// positive-pair and diagonal terms added on top of the GEMM results.
//   role 0 (positives, n = C*P rows): dst[i] += dpos[i] * dkappa/dself + 2 rowsum[i] * self[i]   (l2)
//                                     dst[i] += dpos[i] * other[i]                                (dot / cos)
//   role 1 (negatives of one side, l2 only): dst[c,j] -= colsum_j(dq2[c]) * self[c,j]
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void comparator_terms_kernel(int cmp, int role, int D, int64_t n, int P, int N,
                                                                       const float* __restrict__ self,
                                                                       const float* __restrict__ other,
                                                                       const float* __restrict__ dpos,
                                                                       const float* __restrict__ pos,
                                                                       const float* __restrict__ rowsum,
                                                                       const float* __restrict__ dq2,
                                                                       float* __restrict__ dst) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= n) return;
  const int H = (D + 1) / 2;
  RowV<NVH> d = row_load<NVH>(dst + i * D, D, H, lane);
  const RowV<NVH> s = row_load<NVH>(self + i * D, D, H, lane);
  if (role == 0) {
    const RowV<NVH> o = row_load<NVH>(other + i * D, D, H, lane);
    if (cmp == PBG_CMP_L2 || cmp == PBG_CMP_SQUARED_L2) {
      const float p = pos[i];
      if (cmp == PBG_CMP_SQUARED_L2 || p * p > 1e-30f) {
        const float coef = cmp == PBG_CMP_L2 ? dpos[i] / p : -2.0f * dpos[i];
#pragma unroll
        for (int v = 0; v < NVH; ++v) {
          d.a[0][v] += coef * (s.a[0][v] - o.a[0][v]);
          d.a[1][v] += coef * (s.a[1][v] - o.a[1][v]);
        }
      }
      if (rowsum) row_axpy<NVH>(d, 2.0f * rowsum[i], s);
    } else {
      row_axpy<NVH>(d, dpos[i], o);
    }
  } else {
    const int64_t c = i / N;
    const int j = (int)(i % N);
    const float* base = dq2 + c * P * N + j;
    float acc = 0.f;
    for (int r = lane; r < P; r += kWave) acc += base[(int64_t)r * N];
    row_axpy<NVH>(d, -wave_sum(acc), s);
  }
  row_store<NVH>(dst + i * D, d, D, H, lane);
}

__global__ void fill_kernel(float* p, int64_t n, float v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ---------------------------------------------------------------------------
// losses (losses.py:53-161)
// ---------------------------------------------------------------------------
// One wave per positive.  mode 0: rowloss[i] = weighted loss of row i.
// mode 1: dpos[i], dneg[i, :] scaled by *upstream.
__global__ __launch_bounds__(kRowThreads) void loss_rows_kernel(int loss, float margin, int64_t P, int N,
                                                                const float* __restrict__ pos,
                                                                const float* __restrict__ neg,
                                                                const float* __restrict__ weight, int mode,
                                                                const float* __restrict__ upstream,
                                                                float* __restrict__ rowloss, float* __restrict__ dpos,
                                                                float* __restrict__ dneg) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (i >= P) return;
  const float s = pos[i];
  const float w = weight ? weight[i] : 1.0f;
  const float up = mode == 1 ? *upstream * w : 0.f;
  const float* row = neg + i * N;
  float* drow = mode == 1 ? dneg + i * N : nullptr;
  float acc = 0.f, dp = 0.f;
  if (N == 0 && loss != PBG_LOSS_LOGISTIC) {  // losses.py:101-102,140-141
    if (lane == 0) {
      if (mode == 0) rowloss[i] = 0.f;
      else dpos[i] = 0.f;
    }
    return;
  }
  if (loss == PBG_LOSS_RANKING) {
    for (int j = lane; j < N; j += kWave) {
      const float x = (row[j] - s) + margin;
      if (x > 0.f) acc += x;
      const float g = (x >= 0.f) ? up : 0.f;
      dp -= g;
      if (drow) drow[j] = g;
    }
  } else if (loss == PBG_LOSS_LOGISTIC) {
    const float inv_n = N > 0 ? 1.0f / (float)N : 0.f;
    if (lane == 0) {
      acc += softplusf(-s);
      dp += (sigmoidf(s) - 1.0f) * up;
    }
    for (int j = lane; j < N; j += kWave) {
      float sg;
      acc += softplus_sigmoid(row[j], &sg) * inv_n;
      if (drow) drow[j] = sg * inv_n * up;
    }
  } else {
    float mx = s;
    for (int j = lane; j < N; j += kWave) mx = fmaxf(mx, row[j]);
    mx = wave_max(mx);
    float z = 0.f;
    for (int j = lane; j < N; j += kWave) z += expf(row[j] - mx);
    z = wave_sum(z) + expf(s - mx);
    const float inv_z = 1.0f / z;
    if (lane == 0) {
      acc += (mx + logf(z)) - s;
      dp += (expf(s - mx) * inv_z - 1.0f) * up;
    }
    if (drow)
      for (int j = lane; j < N; j += kWave) drow[j] = expf(row[j] - mx) * inv_z * up;
  }
  if (mode == 0) {
    acc = wave_sum(acc) * w;
    if (lane == 0) rowloss[i] = acc;
  } else {
    dp = wave_sum(dp);
    if (lane == 0) dpos[i] = dp;
  }
}

__global__ __launch_bounds__(256) void sum_rows_kernel(const float* __restrict__ rows, int64_t n, float* __restrict__ out) {
  __shared__ float sh[256];
  float acc = 0.f;
  for (int64_t q = threadIdx.x; q < n; q += 256) acc += rows[q];
  sh[threadIdx.x] = acc;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) *out = sh[0];
}

bool valid_op(int op) { return op >= PBG_OP_NONE && op <= PBG_OP_AFFINE; }
bool valid_cmp(int cmp) { return cmp >= PBG_CMP_DOT && cmp <= PBG_CMP_SQUARED_L2; }

struct CmpWs {
  float *a2_l, *a2_r, *b2_l, *b2_r;  // squared norms: lhs_pos, rhs_pos rows [C*P]; lhs_neg [C*Ln]; rhs_neg [C*Rn]
  float *dq_l, *dq_r;                // [C,P,Ln], [C,P,Rn]
  float *rs_l, *rs_r;                // [C*P]
  size_t total;
};
CmpWs carve_cmp(void* base, int64_t C, int P, int Ln, int Rn) {
  CmpWs w;
  size_t off = 0;
  auto take = [&](size_t count) {
    size_t o = off;
    off += align_up((count > 0 ? count : 1) * sizeof(float), 256);
    return base ? (float*)((char*)base + o) : nullptr;
  };
  w.a2_l = take(C * P); w.a2_r = take(C * P); w.b2_l = take(C * Ln); w.b2_r = take(C * Rn);
  w.dq_l = take(C * P * Ln); w.dq_r = take(C * P * Rn);
  w.rs_l = take(C * P); w.rs_r = take(C * P);
  w.total = off;
  return w;
}

}  // namespace
}  // namespace pbg

using namespace pbg;

extern "C" int pbg_operator_forward(int32_t op, int32_t dim, int64_t n_rows, const float* x, const float* p0,
                                    const float* p1, const int64_t* rel, int64_t num_ops, float* y,
                                    pbg_stream_t stream) {
  if (!valid_op(op)) return fail(PBG_ERR_INVALID, "pbg_operator_forward: unknown operator %d", op);
  if (dim <= 0 || dim > kMaxDim || n_rows < 0) return fail(PBG_ERR_INVALID, "pbg_operator_forward: bad sizes");
  if (op == PBG_OP_COMPLEX_DIAGONAL && dim % 2 != 0)
    return fail(PBG_ERR_INVALID, "Need even dimension as 1st half is real and 2nd half is imaginary coordinates");
  if (n_rows == 0) return PBG_OK;
  if (!x || !y || (op != PBG_OP_NONE && !p0) || ((op == PBG_OP_COMPLEX_DIAGONAL || op == PBG_OP_AFFINE) && !p1))
    return fail(PBG_ERR_INVALID, "pbg_operator_forward: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (op == PBG_OP_AFFINE) {  // the matrix product, then the translation in place (operators.py:109-115, 283-293)
    const int rc = pbg_operator_forward(PBG_OP_LINEAR, dim, n_rows, x, p0, nullptr, rel, num_ops, y, stream);
    if (rc != PBG_OK) return rc;
    return pbg_operator_forward(PBG_OP_TRANSLATION, dim, n_rows, y, p1, nullptr, rel, num_ops, y, stream);
  }
  if (op == PBG_OP_LINEAR) {
    if (!rel) {
      GemmArgs g{};
      g.a = x; g.lda = dim; g.a_kmajor = 0; g.b = p0; g.ldb = dim; g.b_kmajor = 0; g.c = y; g.ldc = dim;
      g.m = (int)n_rows; g.n = dim; g.k = dim; g.batch = 1; g.alpha = 1.f; g.beta = 0.f;
      if (n_rows > INT32_MAX) return fail(PBG_ERR_UNSUPPORTED, "pbg_operator_forward: too many rows");
      return gemm_f32(g, s);
    }
    hipLaunchKernelGGL(linear_rows_forward_kernel, wave_grid(n_rows), dim3(kRowThreads), 0, s, dim, n_rows, x, p0, rel,
                       num_ops, y);
    return check_launch("pbg_operator_forward");
  }
  PBG_DISPATCH_NVH(nvh_for(dim), operator_forward_kernel, wave_grid(n_rows), s, op, dim, n_rows, x, p0, p1, rel,
                   num_ops, y);
  return check_launch("pbg_operator_forward");
}

extern "C" int pbg_operator_backward(int32_t op, int32_t dim, int64_t n_rows, const float* x, const float* dy,
                                     const float* p0, const float* p1, const int64_t* rel, int64_t num_ops, float* dx,
                                     float* dp0, float* dp1, pbg_stream_t stream) {
  if (!valid_op(op)) return fail(PBG_ERR_INVALID, "pbg_operator_backward: unknown operator %d", op);
  if (dim <= 0 || dim > kMaxDim || n_rows < 0) return fail(PBG_ERR_INVALID, "pbg_operator_backward: bad sizes");
  if (n_rows == 0) return PBG_OK;
  if (!x || !dy || !dx || (op != PBG_OP_NONE && (!p0 || !dp0)) ||
      ((op == PBG_OP_COMPLEX_DIAGONAL || op == PBG_OP_AFFINE) && (!p1 || !dp1)))
    return fail(PBG_ERR_INVALID, "pbg_operator_backward: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (op == PBG_OP_AFFINE) {
    // the translation's gradient first (it leaves a copy of dy in dx), then the matrix's, which writes dx
    const int rc = pbg_operator_backward(PBG_OP_TRANSLATION, dim, n_rows, x, dy, p1, nullptr, rel, num_ops, dx, dp1,
                                         nullptr, stream);
    if (rc != PBG_OK) return rc;
    return pbg_operator_backward(PBG_OP_LINEAR, dim, n_rows, x, dy, p0, nullptr, rel, num_ops, dx, dp0, nullptr, stream);
  }
  if (op == PBG_OP_LINEAR) {
    if (!rel) {
      if (n_rows > INT32_MAX) return fail(PBG_ERR_UNSUPPORTED, "pbg_operator_backward: too many rows");
      GemmArgs g{};  // dx = dy * W
      g.a = dy; g.lda = dim; g.a_kmajor = 0; g.b = p0; g.ldb = dim; g.b_kmajor = 1; g.c = dx; g.ldc = dim;
      g.m = (int)n_rows; g.n = dim; g.k = dim; g.batch = 1; g.alpha = 1.f; g.beta = 0.f;
      int rc = gemm_f32(g, s);
      if (rc != PBG_OK) return rc;
      GemmArgs h{};  // dW += dy^T * x
      h.a = dy; h.lda = dim; h.a_kmajor = 1; h.b = x; h.ldb = dim; h.b_kmajor = 1; h.c = dp0; h.ldc = dim;
      h.m = dim; h.n = dim; h.k = (int)n_rows; h.batch = 1; h.alpha = 1.f; h.beta = 1.f;
      return gemm_f32(h, s);
    }
    hipLaunchKernelGGL(linear_rows_backward_kernel, wave_grid(n_rows), dim3(kRowThreads), 0, s, dim, n_rows, x, dy, p0,
                       rel, num_ops, dx, dp0);
    return check_launch("pbg_operator_backward");
  }
  int64_t waves = n_rows < 2048 ? n_rows : 2048;
  if (rel) waves = n_rows;
  PBG_DISPATCH_NVH(nvh_for(dim), operator_backward_kernel, wave_grid(waves), s, op, dim, n_rows, x, dy, p0, p1, rel,
                   num_ops, dx, dp0, dp1);
  return check_launch("pbg_operator_backward");
}

extern "C" int pbg_comparator_prepare(int32_t cmp, int32_t dim, int64_t n, const float* x, float* y, float* aux,
                                      pbg_stream_t stream) {
  if (!valid_cmp(cmp)) return fail(PBG_ERR_INVALID, "pbg_comparator_prepare: unknown comparator %d", cmp);
  if (dim <= 0 || dim > kMaxDim || n < 0) return fail(PBG_ERR_INVALID, "pbg_comparator_prepare: bad sizes");
  if (n == 0) return PBG_OK;
  if (!x || !y) return fail(PBG_ERR_INVALID, "pbg_comparator_prepare: null pointer");
  PBG_DISPATCH_NVH(nvh_for(dim), prepare_kernel, wave_grid(n), (hipStream_t)stream, cmp, dim, n, x, y, aux);
  return check_launch("pbg_comparator_prepare");
}

extern "C" int pbg_comparator_prepare_backward(int32_t cmp, int32_t dim, int64_t n, const float* dy, const float* y,
                                               const float* aux, float* dx, pbg_stream_t stream) {
  if (!valid_cmp(cmp)) return fail(PBG_ERR_INVALID, "pbg_comparator_prepare_backward: unknown comparator %d", cmp);
  if (dim <= 0 || dim > kMaxDim || n < 0) return fail(PBG_ERR_INVALID, "pbg_comparator_prepare_backward: bad sizes");
  if (n == 0) return PBG_OK;
  if (!dy || !y || !dx || (cmp == PBG_CMP_COS && !aux))
    return fail(PBG_ERR_INVALID, "pbg_comparator_prepare_backward: null pointer");
  PBG_DISPATCH_NVH(nvh_for(dim), prepare_backward_kernel, wave_grid(n), (hipStream_t)stream, cmp, dim, n, dy, y, aux,
                   dx);
  return check_launch("pbg_comparator_prepare_backward");
}

extern "C" size_t pbg_comparator_workspace_bytes(int32_t chunks, int32_t p, int32_t ln, int32_t rn) {
  return carve_cmp(nullptr, chunks, p, ln, rn).total;
}

extern "C" int pbg_comparator_forward(int32_t cmp, int32_t chunks, int32_t p, int32_t ln, int32_t rn, int32_t dim,
                                      const float* lhs_pos, const float* rhs_pos, const float* lhs_neg,
                                      const float* rhs_neg, float* pos, float* lhs_neg_scores, float* rhs_neg_scores,
                                      void* workspace, size_t workspace_bytes, pbg_stream_t stream) {
  if (!valid_cmp(cmp)) return fail(PBG_ERR_INVALID, "pbg_comparator_forward: unknown comparator %d", cmp);
  if (chunks < 0 || p < 0 || ln < 0 || rn < 0 || dim <= 0 || dim > kMaxDim)
    return fail(PBG_ERR_INVALID, "pbg_comparator_forward: bad sizes");
  if (chunks == 0 || p == 0) return PBG_OK;
  if (!lhs_pos || !rhs_pos || !pos || (ln > 0 && (!lhs_neg || !lhs_neg_scores)) ||
      (rn > 0 && (!rhs_neg || !rhs_neg_scores)))
    return fail(PBG_ERR_INVALID, "pbg_comparator_forward: null pointer");
  CmpWs ws = carve_cmp(workspace, chunks, p, ln, rn);
  if ((cmp == PBG_CMP_L2 || cmp == PBG_CMP_SQUARED_L2) && (!workspace || workspace_bytes < ws.total))
    return fail(PBG_ERR_WORKSPACE, "pbg_comparator_forward: workspace needs %zu bytes", ws.total);
  hipStream_t s = (hipStream_t)stream;
  const int64_t np = (int64_t)chunks * p;
  hipLaunchKernelGGL(pos_scores_kernel, wave_grid(np), dim3(kRowThreads), 0, s, cmp, dim, np, lhs_pos, rhs_pos, pos);
  const int nvh = nvh_for(dim);
  int rc;
  for (int side = 0; side < 2; ++side) {
    const int nn = side == 0 ? ln : rn;
    if (nn == 0) continue;
    const float* a = side == 0 ? rhs_pos : lhs_pos;  // R+ x L-  and  L+ x R-  (model.py:179-180)
    const float* b = side == 0 ? lhs_neg : rhs_neg;
    float* out = side == 0 ? lhs_neg_scores : rhs_neg_scores;
    GemmArgs g{};
    g.a = a; g.stride_a = (int64_t)p * dim; g.lda = dim; g.a_kmajor = 0;
    g.b = b; g.stride_b = (int64_t)nn * dim; g.ldb = dim; g.b_kmajor = 0;
    g.c = out; g.stride_c = (int64_t)p * nn; g.ldc = nn;
    g.m = p; g.n = nn; g.k = dim; g.batch = chunks; g.alpha = 1.f; g.beta = 0.f;
    if ((rc = gemm_f32(g, s)) != PBG_OK) return rc;
    if (cmp == PBG_CMP_L2 || cmp == PBG_CMP_SQUARED_L2) {
      float* a2 = side == 0 ? ws.a2_r : ws.a2_l;
      float* b2 = side == 0 ? ws.b2_l : ws.b2_r;
      PBG_DISPATCH_NVH(nvh, prepare_kernel, wave_grid(np), s, cmp, dim, np, a, (float*)nullptr, a2);
      PBG_DISPATCH_NVH(nvh, prepare_kernel, wave_grid((int64_t)chunks * nn), s, cmp, dim, (int64_t)chunks * nn, b,
                       (float*)nullptr, b2);
      const int64_t total = np * nn;
      hipLaunchKernelGGL(l2_epilogue_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, s, cmp, out, a2, b2,
                         (int64_t)chunks, p, nn);
    }
  }
  return check_launch("pbg_comparator_forward");
}

extern "C" int pbg_comparator_backward(int32_t cmp, int32_t chunks, int32_t p, int32_t ln, int32_t rn, int32_t dim,
                                       const float* lhs_pos, const float* rhs_pos, const float* lhs_neg,
                                       const float* rhs_neg, const float* pos, const float* lhs_neg_scores,
                                       const float* rhs_neg_scores, const float* dpos, const float* dlhs_neg_scores,
                                       const float* drhs_neg_scores, float* dlhs_pos, float* drhs_pos, float* dlhs_neg,
                                       float* drhs_neg, void* workspace, size_t workspace_bytes, pbg_stream_t stream) {
  if (!valid_cmp(cmp)) return fail(PBG_ERR_INVALID, "pbg_comparator_backward: unknown comparator %d", cmp);
  if (chunks < 0 || p < 0 || ln < 0 || rn < 0 || dim <= 0 || dim > kMaxDim)
    return fail(PBG_ERR_INVALID, "pbg_comparator_backward: bad sizes");
  if (chunks == 0) return PBG_OK;
  if (!lhs_pos || !rhs_pos || !pos || !dpos || !dlhs_pos || !drhs_pos)
    return fail(PBG_ERR_INVALID, "pbg_comparator_backward: null pointer");
  if ((ln > 0 && (!lhs_neg || !lhs_neg_scores || !dlhs_neg_scores || !dlhs_neg)) ||
      (rn > 0 && (!rhs_neg || !rhs_neg_scores || !drhs_neg_scores || !drhs_neg)))
    return fail(PBG_ERR_INVALID, "pbg_comparator_backward: null pointer");
  const bool l2 = cmp == PBG_CMP_L2 || cmp == PBG_CMP_SQUARED_L2;
  CmpWs ws = carve_cmp(workspace, chunks, p, ln, rn);
  if (l2 && (!workspace || workspace_bytes < ws.total))
    return fail(PBG_ERR_WORKSPACE, "pbg_comparator_backward: workspace needs %zu bytes", ws.total);
  hipStream_t s = (hipStream_t)stream;
  const int64_t np = (int64_t)chunks * p;
  const int nvh = nvh_for(dim);
  int rc;
  for (int side = 0; side < 2; ++side) {
    const int nn = side == 0 ? ln : rn;
    // the positives that were scored against this side's negatives: R+ for L-, L+ for R-
    const float* a = side == 0 ? rhs_pos : lhs_pos;
    float* da = side == 0 ? drhs_pos : dlhs_pos;
    if (nn == 0 || p == 0) {
      if (np > 0)
        hipLaunchKernelGGL(fill_kernel, dim3((unsigned)ceil_div(np * dim, 256)), dim3(256), 0, s, da, np * dim, 0.f);
      continue;
    }
    const float* b = side == 0 ? lhs_neg : rhs_neg;
    float* db = side == 0 ? dlhs_neg : drhs_neg;
    const float* g = side == 0 ? dlhs_neg_scores : drhs_neg_scores;
    const float* sc = side == 0 ? lhs_neg_scores : rhs_neg_scores;
    const float* gg = g;
    float* dq = side == 0 ? ws.dq_l : ws.dq_r;
    float* rs = side == 0 ? ws.rs_l : ws.rs_r;
    if (l2) {
      hipLaunchKernelGGL(l2_grad_kernel, wave_grid(np), dim3(kRowThreads), 0, s, cmp, g, sc, np, nn, dq, rs);
      gg = dq;
    }
    GemmArgs ga{};  // dA = G * B
    ga.a = gg; ga.stride_a = (int64_t)p * nn; ga.lda = nn; ga.a_kmajor = 0;
    ga.b = b; ga.stride_b = (int64_t)nn * dim; ga.ldb = dim; ga.b_kmajor = 1;
    ga.c = da; ga.stride_c = (int64_t)p * dim; ga.ldc = dim;
    ga.m = p; ga.n = dim; ga.k = nn; ga.batch = chunks; ga.alpha = 1.f; ga.beta = 0.f;
    if ((rc = gemm_f32(ga, s)) != PBG_OK) return rc;
    GemmArgs gb{};  // dB = G^T * A
    gb.a = gg; gb.stride_a = (int64_t)p * nn; gb.lda = nn; gb.a_kmajor = 1;
    gb.b = a; gb.stride_b = (int64_t)p * dim; gb.ldb = dim; gb.b_kmajor = 1;
    gb.c = db; gb.stride_c = (int64_t)nn * dim; gb.ldc = dim;
    gb.m = nn; gb.n = dim; gb.k = p; gb.batch = chunks; gb.alpha = 1.f; gb.beta = 0.f;
    if ((rc = gemm_f32(gb, s)) != PBG_OK) return rc;
    if (l2) {
      PBG_DISPATCH_NVH(nvh, comparator_terms_kernel, wave_grid((int64_t)chunks * nn), s, cmp, 1, dim,
                       (int64_t)chunks * nn, p, nn, b, (const float*)nullptr, (const float*)nullptr,
                       (const float*)nullptr, (const float*)nullptr, (const float*)dq, db);
    }
  }
  if (np > 0) {
    // positive-pair terms; rowsum of the side whose negatives a row was scored against
    PBG_DISPATCH_NVH(nvh, comparator_terms_kernel, wave_grid(np), s, cmp, 0, dim, np, p, 0, lhs_pos, rhs_pos, dpos, pos,
                     (const float*)((l2 && rn > 0) ? ws.rs_r : nullptr), (const float*)nullptr, dlhs_pos);
    PBG_DISPATCH_NVH(nvh, comparator_terms_kernel, wave_grid(np), s, cmp, 0, dim, np, p, 0, rhs_pos, lhs_pos, dpos, pos,
                     (const float*)((l2 && ln > 0) ? ws.rs_l : nullptr), (const float*)nullptr, drhs_pos);
  }
  return check_launch("pbg_comparator_backward");
}

extern "C" int pbg_loss_forward(int32_t loss, float margin, int64_t num_pos, int32_t num_neg, const float* pos,
                                const float* neg, const float* weight, float* out, float* row_workspace,
                                pbg_stream_t stream) {
  if (loss < PBG_LOSS_RANKING || loss > PBG_LOSS_SOFTMAX) return fail(PBG_ERR_INVALID, "pbg_loss_forward: unknown loss %d", loss);
  if (num_pos < 0 || num_neg < 0) return fail(PBG_ERR_INVALID, "pbg_loss_forward: bad sizes");
  if (!out) return fail(PBG_ERR_INVALID, "pbg_loss_forward: null output");
  hipStream_t s = (hipStream_t)stream;
  if (num_pos == 0) {
    hipLaunchKernelGGL(fill_kernel, dim3(1), dim3(64), 0, s, out, (int64_t)1, 0.f);
    return check_launch("pbg_loss_forward");
  }
  if (!pos || (num_neg > 0 && !neg) || !row_workspace) return fail(PBG_ERR_INVALID, "pbg_loss_forward: null pointer");
  hipLaunchKernelGGL(loss_rows_kernel, wave_grid(num_pos), dim3(kRowThreads), 0, s, loss, margin, num_pos, num_neg, pos,
                     neg, weight, 0, (const float*)nullptr, row_workspace, (float*)nullptr, (float*)nullptr);
  hipLaunchKernelGGL(sum_rows_kernel, dim3(1), dim3(256), 0, s, row_workspace, num_pos, out);
  return check_launch("pbg_loss_forward");
}

extern "C" int pbg_loss_backward(int32_t loss, float margin, int64_t num_pos, int32_t num_neg, const float* pos,
                                 const float* neg, const float* weight, const float* upstream, float* dpos,
                                 float* dneg, pbg_stream_t stream) {
  if (loss < PBG_LOSS_RANKING || loss > PBG_LOSS_SOFTMAX) return fail(PBG_ERR_INVALID, "pbg_loss_backward: unknown loss %d", loss);
  if (num_pos < 0 || num_neg < 0) return fail(PBG_ERR_INVALID, "pbg_loss_backward: bad sizes");
  if (num_pos == 0) return PBG_OK;
  if (!pos || !upstream || !dpos || (num_neg > 0 && (!neg || !dneg)))
    return fail(PBG_ERR_INVALID, "pbg_loss_backward: null pointer");
  hipLaunchKernelGGL(loss_rows_kernel, wave_grid(num_pos), dim3(kRowThreads), 0, (hipStream_t)stream, loss, margin,
                     num_pos, num_neg, pos, neg, weight, 1, upstream, (float*)nullptr, dpos, dneg);
  return check_launch("pbg_loss_backward");
}
