// The per-batch training step of PyTorch-BigGraph on one MI355X.
//
// One call handles K batches ("workers") that all read the tables as they are
// on entry; their updates are then applied in worker order.  Stages, each one
// kernel (or one batched GEMM) over all K batches:
//
//   prep      gather rows, apply the relation operator and comparator.prepare,
//             lay the results out as per-chunk operand matrices; emit the
//             (row, worker) sort keys of every gradient row        [HBM bound]
//   scores    S = A * N^T per chunk and side                        [MFMA]
//   loss      mask, comparator epilogue (l2), loss, dLoss/dS in place, positive
//             scores and their gradients, violator counts           [L2 bound]
//   backward  dA = dS * N, dN = dS^T * A per chunk and side          [MFMA]
//   rowback   chain rule through prepare and the operator back to raw rows,
//             one gradient row per gathered row                      [HBM bound]
//   params    operator-parameter gradients and their Adagrad step
//   update    radix sort of the keys, then a segmented RowAdagrad    [HBM bound]
//
// Layout of a row inside a wave: lane l owns elements {h, H + h} for
// h = l, l + 64, ... < H with H = ceil(D / 2), i.e. both halves of a complex
// pair sit in the same lane.
#include <cstdlib>
#include <cstring>

#include "pbg_internal.h"
#include "row_ops.h"
#include "step_ctx.h"
#include "mfma_tiles.h"
#include "fused.h"
#include "stream.h"

#include <atomic>
#include <mutex>

namespace pbg {
namespace {

constexpr int kRowThreads = 256;
constexpr int kWavesPerBlock = kRowThreads / kWave;

// x + the global embedding of the side's entity type (model.py:486-492)
template <int NVH>
__device__ __forceinline__ RowV<NVH> gathered_row(const SideCtx& sd, int64_t id, int D, int H, int lane) {
  RowV<NVH> x = row_load<NVH>(sd.w + id * D, D, H, lane);
  if (sd.glob) row_axpy<NVH>(x, 1.0f, row_load<NVH>(sd.glob, D, H, lane));
  return x;
}

// BiasedComparator.prepare (model.py:311-314) keeps a row's first coordinate, its
// bias, out of the comparator.  Here the bias is set aside and the row carries 0
// in its place, so every product, norm and distance that follows runs over the
// other coordinates only; the scores get the two biases of a pair added where
// they are read (ScoreRow::at, positive_scores).  Element 0 of a row is lane 0's.
template <int NVH>
__device__ __forceinline__ float take_bias(RowV<NVH>& y, int lane) {
  const float b = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(y.a[0][0])));
  if (lane == 0) y.a[0][0] = 0.f;
  return b;
}
template <int NVH>
__device__ __forceinline__ void add_to_first(RowV<NVH>& y, float v, int lane) {
  if (lane == 0) y.a[0][0] += v;
}

// ---------------------------------------------------------------------------
// max_norm
// ---------------------------------------------------------------------------
// The reference looks rows up with F.embedding(max_norm=...) (model.py:61,90-96):
// before they are read, the rows a batch names are renormalised in the table
// itself -- a row whose 2-norm exceeds max_norm is scaled by max_norm / (norm +
// 1e-7).  Two kernels, so that no wave reads a row that another is rewriting:
// `scan` only reads the table and keeps, per gathered slot, a too-long row and
// its scale; `apply` writes row * scale back for those slots.  Slots that name
// the same row hold the same row and the same scale, so their writes carry the
// same bytes.  The K batches of a call are renormalised together, then read.
__device__ __forceinline__ const SideCtx& slot_row(const StepCtx& c, int k, int slot, int64_t* id) {
  const int s = slot >= c.side[1].slot_pos;
  const SideCtx& sd = c.side[s];
  const int r = slot - sd.slot_pos;
  if (r < c.B) {
    *id = clamp_index(sd.idx[(int64_t)k * c.B + r], sd.num_rows);
  } else {
    const int r2 = r - c.B;
    *id = clamp_index(uniform_negative(sd, s, ((int64_t)k * c.C + r2 / sd.u) * sd.u + r2 % sd.u), sd.num_rows);
  }
  return sd;
}

template <int NVH>
__global__ __launch_bounds__(kRowThreads) void renorm_scan_kernel(StepCtx c, float max_norm, float* __restrict__ scale) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (job >= (int64_t)c.K * c.rk) return;
  const int D = c.D, H = (D + 1) / 2;
  int64_t id;
  const SideCtx& sd = slot_row(c, (int)(job / c.rk), (int)(job % c.rk), &id);
  const RowV<NVH> x = row_load<NVH>(sd.w + id * D, D, H, lane);
  const float norm = sqrtf(wave_sum(row_dot(x, x)));
  const bool renorm = norm > max_norm;
  if (renorm) row_store<NVH>(c.gr + job * D, x, D, H, lane);
  if (lane == 0) scale[job] = renorm ? max_norm / (norm + 1e-7f) : 0.f;
}

template <int NVH>
__global__ __launch_bounds__(kRowThreads) void renorm_apply_kernel(StepCtx c, const float* __restrict__ scale,
                                                                    float* w_lhs, float* w_rhs) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (job >= (int64_t)c.K * c.rk) return;
  const float sc = scale[job];
  if (sc == 0.f) return;
  const int D = c.D, H = (D + 1) / 2;
  int64_t id;
  const int slot = (int)(job % c.rk);
  slot_row(c, (int)(job / c.rk), slot, &id);
  RowV<NVH> x = row_load<NVH>(c.gr + job * D, D, H, lane);
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    x.a[0][v] *= sc;
    x.a[1][v] *= sc;
  }
  row_store<NVH>((slot >= c.side[1].slot_pos ? w_rhs : w_lhs) + id * D, x, D, H, lane);
}

// ---------------------------------------------------------------------------
// prep
// ---------------------------------------------------------------------------
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void prep_kernel(StepCtx c) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int CP = c.C * c.P;
  const int J0 = CP + c.C * c.side[0].u;
  const int J = J0 + CP + c.C * c.side[1].u;
  if (job >= (int64_t)c.K * J) return;
  const int k = (int)(job / J);
  int r = (int)(job % J);
  const int s = r >= J0;
  if (s) r -= J0;
  const SideCtx& sd = c.side[s];
  const int D = c.D, H = (D + 1) / 2;

  if (r < CP) {
    const int cc = r / c.P, i = r % c.P;
    const int64_t kc = (int64_t)k * c.C + cc;
    float* xp_row = sd.xp + (kc * sd.stride_p + i) * D;
    float* ap = sd.ap ? sd.ap + kc * sd.stride_p + i : nullptr;
    float* xa_row = c.dynamic ? sd.xa + (kc * c.P + i) * D : nullptr;
    float* aa = (c.dynamic && sd.aa) ? sd.aa + kc * c.P + i : nullptr;
    float* bp = c.bias ? sd.bp + kc * sd.stride_p + i : nullptr;
    float* ba = (c.bias && c.dynamic) ? sd.ba + kc * c.P + i : nullptr;
    if (r >= c.B) {  // padding of an incomplete last chunk (model.py:790-798)
      const RowV<NVH> zero = row_zero<NVH>();
      row_store<NVH>(xp_row, zero, D, H, lane);
      if (ap && lane == 0) *ap = 0.f;
      if (bp && lane == 0) *bp = 0.f;
      if (xa_row) row_store<NVH>(xa_row, zero, D, H, lane);
      if (aa && lane == 0) *aa = 0.f;
      if (ba && lane == 0) *ba = 0.f;
      return;
    }
    const int64_t e = (int64_t)k * c.B + r;
    const int64_t id = clamp_index(sd.idx[e], sd.num_rows);
    const int64_t rel = clamp_index(c.dynamic ? c.rel[e] : c.rel[k], c.num_relations);
    const RowV<NVH> x = gathered_row<NVH>(sd, id, D, H, lane);
    if (lane == 0) {
      const int64_t slot = (int64_t)k * c.rk + sd.slot_pos + r;
      c.keys[slot] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
      c.vals[slot] = (uint32_t)slot;
    }
    if (c.dynamic || !sd.has_op) {
      RowV<NVH> y = x;
      const float b = c.bias ? take_bias<NVH>(y, lane) : 0.f;
      const float aux = prepare_row<NVH>(c.cmp, y);
      if (c.half) row_round_half<NVH>(y);
      row_store<NVH>(xp_row, y, D, H, lane);
      if (ap && lane == 0) *ap = aux;
      if (bp && lane == 0) *bp = b;
    }
    if (sd.has_op) {
      if (c.op == PBG_OP_LINEAR) {
        row_store<NVH>(sd.xraw + ((int64_t)k * sd.op_rows + r) * D, x, D, H, lane);
      } else {
        RowV<NVH> y = op_forward<NVH>(c.op, x, sd.p0, sd.p1, rel, D, H, lane);
        const float b = c.bias ? take_bias<NVH>(y, lane) : 0.f;
        const float aux = prepare_row<NVH>(c.cmp, y);
        if (c.half) row_round_half<NVH>(y);
        row_store<NVH>(c.dynamic ? xa_row : xp_row, y, D, H, lane);
        float* auxdst = c.dynamic ? aa : ap;
        if (auxdst && lane == 0) *auxdst = aux;
        float* bdst = c.dynamic ? ba : bp;
        if (bdst && lane == 0) *bdst = b;
      }
    }
  } else {
    const int r2 = r - CP;
    const int cc = r2 / sd.u, uu = r2 % sd.u;
    const int64_t kc = (int64_t)k * c.C + cc;
    const int64_t id = clamp_index(uniform_negative(sd, s, kc * sd.u + uu), sd.num_rows);
    const RowV<NVH> x = gathered_row<NVH>(sd, id, D, H, lane);
    if (lane == 0) {
      const int64_t slot = (int64_t)k * c.rk + sd.slot_uni + r2;
      c.keys[slot] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
      c.vals[slot] = sd.uni_direct ? (uint32_t)(sd.uni_row0 + kc * sd.nn + sd.nb + uu) : (uint32_t)slot;
    }
    if (sd.op_uniform && c.op == PBG_OP_LINEAR) {
      row_store<NVH>(sd.xraw + ((int64_t)k * sd.op_rows + c.B + r2) * D, x, D, H, lane);
      return;
    }
    RowV<NVH> y = x;
    if (sd.op_uniform) {
      const int64_t rel = clamp_index(c.rel[k], c.num_relations);
      y = op_forward<NVH>(c.op, x, sd.p0, sd.p1, rel, D, H, lane);
    }
    const float b = c.bias ? take_bias<NVH>(y, lane) : 0.f;
    const float aux = prepare_row<NVH>(c.cmp, y);
    if (c.half) row_round_half<NVH>(y);
    row_store<NVH>(sd.xn + (kc * sd.nn + sd.nb + uu) * D, y, D, H, lane);
    if (sd.an && lane == 0) sd.an[kc * sd.nn + sd.nb + uu] = aux;
    if (c.bias && lane == 0) sd.bn[kc * sd.nn + sd.nb + uu] = b;
  }
}

// comparator.prepare on the rows a `linear` operator produced (staging z), moved
// to their operand positions.
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void prepare_staged_kernel(StepCtx c, int s) {
  const int lane = threadIdx.x & 63;
  const SideCtx& sd = c.side[s];
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (job >= (int64_t)c.K * sd.op_rows) return;
  const int k = (int)(job / sd.op_rows), r = (int)(job % sd.op_rows);
  const int D = c.D, H = (D + 1) / 2;
  RowV<NVH> y = row_load<NVH>(sd.z + job * D, D, H, lane);
  if (c.affine) {
    const int64_t rel = clamp_index((c.dynamic && r < c.B) ? c.rel[(int64_t)k * c.B + r] : c.rel[k], c.num_relations);
    y = op_forward<NVH>(PBG_OP_TRANSLATION, y, sd.p1, nullptr, rel, D, H, lane);
  }
  const float b = c.bias ? take_bias<NVH>(y, lane) : 0.f;
  const float aux = prepare_row<NVH>(c.cmp, y);
  if (c.half) row_round_half<NVH>(y);
  if (r < c.B) {
    const int cc = r / c.P, i = r % c.P;
    const int64_t kc = (int64_t)k * c.C + cc;
    if (c.dynamic) {
      row_store<NVH>(sd.xa + (kc * c.P + i) * D, y, D, H, lane);
      if (sd.aa && lane == 0) sd.aa[kc * c.P + i] = aux;
      if (c.bias && lane == 0) sd.ba[kc * c.P + i] = b;
    } else {
      row_store<NVH>(sd.xp + (kc * sd.stride_p + i) * D, y, D, H, lane);
      if (sd.ap && lane == 0) sd.ap[kc * sd.stride_p + i] = aux;
      if (c.bias && lane == 0) sd.bp[kc * sd.stride_p + i] = b;
    }
  } else {
    const int r2 = r - c.B;
    const int cc = r2 / sd.u, uu = r2 % sd.u;
    const int64_t kc = (int64_t)k * c.C + cc;
    row_store<NVH>(sd.xn + (kc * sd.nn + sd.nb + uu) * D, y, D, H, lane);
    if (sd.an && lane == 0) sd.an[kc * sd.nn + sd.nb + uu] = aux;
    if (c.bias && lane == 0) sd.bn[kc * sd.nn + sd.nb + uu] = b;
  }
}

// ---------------------------------------------------------------------------
// loss
// ---------------------------------------------------------------------------
// l2 and squared_l2 score a pair by ||a||^2 - 2ab + ||b||^2 (model.py:215-236)
__host__ __device__ __forceinline__ bool is_distance(int cmp) { return cmp == PBG_CMP_L2 || cmp == PBG_CMP_SQUARED_L2; }

// comparator on a matched pair (model.py:177,207,267-274,300)
__device__ __forceinline__ float kappa(int cmp, const float* __restrict__ a, const float* __restrict__ b, int D,
                                       int lane) {
  float acc = 0.f;
  if (is_distance(cmp)) {
    for (int d = lane; d < D; d += kWave) {
      const float t = a[d] - b[d];
      acc += t * t;
    }
    const float q = wave_sum(acc);
    return cmp == PBG_CMP_L2 ? -sqrtf(fmaxf(q, 1e-30f)) : -q;
  }
  for (int d = lane; d < D; d += kWave) acc += a[d] * b[d];
  return wave_sum(acc);
}

struct ScoreRow {
  const float* raw;  // chunk score row, a.b for every comparator
  const float* bn;   // squared norms of the negatives (l2)
  float a2;          // squared norm of the positive operand (l2)
  const float* cb;   // biases of the negatives (config.bias), or null
  float rb;          // bias of the positive operand
  int64_t own;       // all_negs: the column of the edge's own entity on this side (masked, model.py:596-618); else -1
  int cmp, nb, i, masked_from;  // batch-negative columns; own column; first padded column
  int half;  // config.half_precision: dLoss/dscore is stored as the float16 number the cast's backward makes of it (model.py:827-829)

  // score of column j as the model returns it (model.py:234-246,836-839); `live`
  // is false where the value is a constant with no gradient
  __device__ __forceinline__ float at(int j, bool* live) const {
    float t = raw[j];
    bool ok = true;
    if (cmp == PBG_CMP_L2) {
      const float qd = fmaf(-2.0f, t, bn[j]) + a2;
      ok = qd >= 1e-30f;
      t = -sqrtf(fmaxf(qd, 1e-30f));
    } else if (cmp == PBG_CMP_SQUARED_L2) {
      t = -(fmaf(-2.0f, t, bn[j]) + a2);
    }
    if (cb) t += rb + cb[j];  // model.py:338-342
    if ((j < nb && (j == i || j >= masked_from)) || j == own) {
      t = -1e9f;
      ok = false;
    }
    *live = ok;
    return t;
  }
  // the comparator's own part of a live column's score t: without the pair's biases
  __device__ __forceinline__ float without_bias(int j, float t) const { return cb ? t - (rb + cb[j]) : t; }
};

__device__ __forceinline__ void positive_scores(const StepCtx& c, int64_t kc, int i, int lane, float* posv) {
  const int D = c.D;
  const float* lp = c.side[0].xp + (kc * c.side[0].stride_p + i) * D;
  const float* rp = c.side[1].xp + (kc * c.side[1].stride_p + i) * D;
  if (!c.dynamic) {
    // With batch negatives the score block already holds the pair: column i of row i
    // is (rhs positive i) . (lhs positive i), before masking.  (Distances are
    // recomputed from the rows: the block's ||a||^2 - 2ab + ||b||^2 cancels for a close pair.)
    // (Nor with half_precision: the block then holds float16 numbers, the positive score is an fp32 sum, model.py:177.)
    if (!is_distance(c.cmp) && !c.half && c.side[0].nb > 0)
      posv[0] = posv[1] = c.side[0].s[(kc * c.P + i) * c.side[0].nn + i];
    else if (!is_distance(c.cmp) && !c.half && c.side[1].nb > 0)
      posv[0] = posv[1] = c.side[1].s[(kc * c.P + i) * c.side[1].nn + i];
    else
      posv[0] = posv[1] = kappa(c.cmp, lp, rp, D, lane);
  } else {
    posv[0] = kappa(c.cmp, lp, c.side[1].xa + (kc * c.P + i) * D, D, lane);
    posv[1] = kappa(c.cmp, rp, c.side[0].xa + (kc * c.P + i) * D, D, lane);
  }
  if (c.bias) {  // model.py:332-336: both rows' biases
    const float bl = c.side[0].bp[kc * c.side[0].stride_p + i], br = c.side[1].bp[kc * c.side[1].stride_p + i];
    if (!c.dynamic) {
      posv[0] += bl + br;
      posv[1] = posv[0];
    } else {
      posv[0] += bl + c.side[1].ba[kc * c.P + i];
      posv[1] += br + c.side[0].ba[kc * c.P + i];
    }
  }
}

__device__ __forceinline__ ScoreRow score_row(const StepCtx& c, int s, int64_t kc, int cc, int i) {
  const SideCtx& sd = c.side[s];
  const SideCtx& so = c.side[1 - s];
  ScoreRow sr;
  sr.raw = sd.s + (kc * c.P + i) * sd.nn;
  sr.cmp = c.cmp;
  sr.half = c.half;
  sr.bn = nullptr;
  sr.a2 = 0.f;
  if (is_distance(c.cmp)) {
    sr.bn = sd.an + kc * sd.nn;
    sr.a2 = c.dynamic ? so.aa[kc * c.P + i] : so.ap[kc * so.stride_p + i];
  }
  sr.own = -1;
  if (sd.all) {
    const int64_t e = (kc / c.C) * c.B + (int64_t)cc * c.P + i;
    sr.own = clamp_index(sd.idx[e], sd.num_rows);
  }
  sr.cb = nullptr;
  sr.rb = 0.f;
  if (c.bias) {
    sr.cb = sd.bn + kc * sd.nn;
    sr.rb = c.dynamic ? so.ba[kc * c.P + i] : so.bp[kc * so.stride_p + i];
  }
  sr.nb = sd.nb;
  sr.i = i;
  sr.masked_from = (cc == c.C - 1) ? c.last : c.P;
  return sr;
}

// Loss of one positive against one side's nn negatives, computed by one wave
// (lane `first` owns columns first, first + 64, ...).  Adds the unweighted per-lane
// loss partial to *loss_acc, overwrites the score row with dLoss/dscore (l2: -2
// dLoss/d squared distance) and returns the wave-reduced dLoss/dpos, violator count,
// (l2) row sum of dLoss/d squared distance and row sum of dLoss/dscore.
//
// Rows of up to 64 * DEPTH columns are read ONCE, with all of a lane's loads in
// flight together: the loads are issued from straight-line code at clamped
// (always valid) columns and what lies past the row is dropped afterwards -- a load
// inside a branch would make the code after the branch wait for it, one load
// after the other.  Every pass of the loss then runs over registers.
template <int DEPTH, bool DIST>  // DIST: a distance comparator (l2, squared_l2)
__device__ __forceinline__ void side_loss_held(int loss, float margin, int cmp, const ScoreRow& sr, float* out, int nn,
                                               float pos, float w, int first, float* loss_acc, float* dpos_out,
                                               int* viol_out, float* rowsum_out, float* gsum_out, float* gout) {
  float t[DEPTH];
  float half_inv[DIST ? DEPTH : 1];  // l2: 0.5 / (the distance score without the pair's biases), the slope of -sqrt
  unsigned live_bits = 0u;
  {
    float raw[DEPTH];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) raw[u] = sr.raw[min(first + u * kWave, nn - 1)];
    if (DIST) {
      float bn[DEPTH];
#pragma unroll
      for (int u = 0; u < DEPTH; ++u) bn[u] = sr.bn[min(first + u * kWave, nn - 1)];
#pragma unroll
      for (int u = 0; u < DEPTH; ++u) {
        const float qd = fmaf(-2.0f, raw[u], bn[u]) + sr.a2;
        if (cmp == PBG_CMP_L2) {
          if (qd >= 1e-30f) live_bits |= 1u << u;
          raw[u] = -sqrtf(fmaxf(qd, 1e-30f));
          half_inv[DIST ? u : 0] = 0.5f / raw[u];
        } else {
          live_bits |= 1u << u;
          raw[u] = -qd;
        }
      }
    } else {
      live_bits = 0xffffffffu;
    }
    if (sr.cb) {  // model.py:338-342
      float cb[DEPTH];
#pragma unroll
      for (int u = 0; u < DEPTH; ++u) cb[u] = sr.cb[min(first + u * kWave, nn - 1)];
#pragma unroll
      for (int u = 0; u < DEPTH; ++u) raw[u] += sr.rb + cb[u];
    }
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int j = first + u * kWave;
      t[u] = raw[u];
      if ((j < sr.nb && (j == sr.i || j >= sr.masked_from)) || j == sr.own) {
        t[u] = -1e9f;
        live_bits &= ~(1u << u);
      }
      if (j >= nn) {  // past the row: a score of -inf adds nothing to any loss
        t[u] = -INFINITY;
        live_bits &= ~(1u << u);
      }
    }
  }
  float dpos_part = 0.f, rowsum = 0.f, gsum = 0.f, mx = pos, inv_z = 0.f;
  int viol = 0;
  const float inv_nn = 1.0f / (float)nn;
  if (loss == PBG_LOSS_SOFTMAX) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) mx = fmaxf(mx, t[u]);
    mx = wave_max(mx);
    float z = 0.f;
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) z += exp_below(t[u], mx);
    z = wave_sum(z) + exp_below(pos, mx);
    inv_z = 1.0f / z;
    if (first == 0) {
      *loss_acc += (mx + logf(z)) - pos;
      dpos_part += (exp_below(pos, mx) * inv_z - 1.0f) * w;
    }
  } else if (loss == PBG_LOSS_LOGISTIC) {
    if (first == 0) {
      *loss_acc += softplusf(-pos);
      dpos_part += (sigmoidf(pos) - 1.0f) * w;
    }
  }
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) {
    const int j = first + u * kWave;
    const float tu = t[u];
    const bool live = (live_bits >> u) & 1u;
    float g;
    if (loss == PBG_LOSS_RANKING) {
      // F.margin_ranking_loss(neg, pos, target=-1): max(0, (t - pos) + margin); the
      // clamp lets the gradient through at exactly 0
      const float x = (tu - pos) + margin;
      if (x > 0.f) *loss_acc += x;
      g = (x >= 0.f) ? w : 0.f;
      dpos_part -= g;
    } else if (loss == PBG_LOSS_LOGISTIC) {
      float sg;
      *loss_acc += softplus_sigmoid(tu, &sg) * inv_nn;
      g = sg * inv_nn * w;
    } else {
      g = exp_below(tu, mx) * inv_z * w;
    }
    if (tu > pos) ++viol;
    if (!live) g = 0.f;
    gsum += g;
    float stored = g;
    if (DIST) {
      // t = -sqrt(q): dLoss/dq = g * 0.5 / t (squared_l2, t = -q: -g); stored as
      // -2 dLoss/dq so that the backward GEMMs produce the cross terms of
      // ||a||^2 - 2ab + ||b||^2
      const float dq = !live ? 0.f : (cmp == PBG_CMP_L2 ? g * half_inv[DIST ? u : 0] : -g);
      rowsum += dq;
      stored = -2.0f * dq;
    }
    if (j < nn) {
      out[j] = sr.half ? half_round(stored) : stored;
      if (gout) gout[j] = g;
    }
  }
  *dpos_out = wave_sum(dpos_part);
  *rowsum_out = wave_sum(rowsum);
  *gsum_out = wave_sum(gsum);
  *viol_out = wave_sum_int(viol);
}

// The same for rows of any length: the row is read once per pass of the loss.
__device__ __forceinline__ void side_loss_long(int loss, float margin, int cmp, const ScoreRow& sr, float* out, int nn,
                                               float pos, float w, int first, float* loss_acc, float* dpos_out,
                                               int* viol_out, float* rowsum_out, float* gsum_out, float* gout) {
  float dpos_part = 0.f, rowsum = 0.f, gsum = 0.f, mx = pos, inv_z = 0.f;
  int viol = 0;
  const float inv_nn = 1.0f / (float)nn;
  bool live;
  if (loss == PBG_LOSS_SOFTMAX) {
    for (int j = first; j < nn; j += kWave) mx = fmaxf(mx, sr.at(j, &live));
    mx = wave_max(mx);
    float z = 0.f;
    for (int j = first; j < nn; j += kWave) z += exp_below(sr.at(j, &live), mx);
    z = wave_sum(z) + exp_below(pos, mx);
    inv_z = 1.0f / z;
    if (first == 0) {
      *loss_acc += (mx + logf(z)) - pos;
      dpos_part += (exp_below(pos, mx) * inv_z - 1.0f) * w;
    }
  } else if (loss == PBG_LOSS_LOGISTIC) {
    if (first == 0) {
      *loss_acc += softplusf(-pos);
      dpos_part += (sigmoidf(pos) - 1.0f) * w;
    }
  }
  for (int j = first; j < nn; j += kWave) {
    const float t = sr.at(j, &live);
    float g;
    if (loss == PBG_LOSS_RANKING) {
      const float x = (t - pos) + margin;
      if (x > 0.f) *loss_acc += x;
      g = (x >= 0.f) ? w : 0.f;
      dpos_part -= g;
    } else if (loss == PBG_LOSS_LOGISTIC) {
      float sg;
      *loss_acc += softplus_sigmoid(t, &sg) * inv_nn;
      g = sg * inv_nn * w;
    } else {
      g = exp_below(t, mx) * inv_z * w;
    }
    if (t > pos) ++viol;
    if (!live) g = 0.f;
    gsum += g;
    if (gout) gout[j] = g;
    if (is_distance(cmp)) {
      const float dq = !live ? 0.f : (cmp == PBG_CMP_L2 ? g * 0.5f / sr.without_bias(j, t) : -g);
      rowsum += dq;
      out[j] = -2.0f * dq;
    } else {
      out[j] = sr.half ? half_round(g) : g;
    }
  }
  *dpos_out = wave_sum(dpos_part);
  *rowsum_out = wave_sum(rowsum);
  *gsum_out = wave_sum(gsum);
  *viol_out = wave_sum_int(viol);
}

// DEPTH: 0 = rows of any length, else rows of at most 64 * DEPTH columns
template <int DEPTH, bool DIST>
__device__ __forceinline__ void side_loss(int loss, float margin, int cmp, const ScoreRow& sr, float* out, int nn, float pos,
                                          float w, int first, float* loss_acc, float* dpos_out, int* viol_out,
                                          float* rowsum_out, float* gsum_out, float* gout) {
  if (DEPTH > 0)
    side_loss_held<(DEPTH > 0 ? DEPTH : 1), DIST>(loss, margin, cmp, sr, out, nn, pos, w, first, loss_acc, dpos_out, viol_out,
                                                  rowsum_out, gsum_out, gout);
  else
    side_loss_long(loss, margin, cmp, sr, out, nn, pos, w, first, loss_acc, dpos_out, viol_out, rowsum_out, gsum_out, gout);
}

// One kernel per row length class and comparator class: a lane's registers (and with
// them the number of waves a compute unit keeps in flight to hide the memory latency
// of the per-edge reads) follow the longest row the kernel accepts.
template <int DEPTH, bool DIST>
__global__ __launch_bounds__(kRowThreads) void loss_kernel(StepCtx c) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int CP = c.C * c.P;
  if (job >= (int64_t)c.K * CP) return;
  const int k = (int)(job / CP), q = (int)(job % CP);
  const int cc = q / c.P, i = q % c.P;
  const int64_t kc = (int64_t)k * c.C + cc;
  if (q >= c.B) {  // padded positive: its rows of dLoss/dS are zero
    for (int s = 0; s < 2; ++s) {
      const SideCtx& sd = c.side[s];
      float* row = sd.s + (kc * c.P + i) * sd.nn;
      for (int j = lane; j < sd.nn; j += kWave) row[j] = 0.f;
      if (sd.gs)
        for (int j = lane; j < sd.nn; j += kWave) sd.gs[(kc * c.P + i) * sd.nn + j] = 0.f;
      if (sd.rs && lane == 0) sd.rs[kc * c.P + i] = 0.f;
      if (sd.bs && lane == 0) sd.bs[kc * c.P + i] = 0.f;
    }
    if (lane == 0) {
      c.lossrow[job] = 0.f;
      c.violrow[job * 2] = 0;
      c.violrow[job * 2 + 1] = 0;
      c.dpos[0][job] = 0.f;
      if (c.dynamic) c.dpos[1][job] = 0.f;
      c.pos[0][job] = 0.f;
      if (c.dynamic) c.pos[1][job] = 0.f;
    }
    return;
  }
  float posv[2];
  positive_scores(c, kc, i, lane, posv);
  const int64_t e = (int64_t)k * c.B + q;
  float w = c.rel_weights[c.dynamic ? 0 : clamp_index(c.rel[k], c.num_relations)];
  if (c.edge_weight) w *= c.edge_weight[e];

  float loss_acc = 0.f;  // per-lane partial, unweighted
  float dposv[2] = {0.f, 0.f};
  int violv[2] = {0, 0};
  for (int s = 0; s < 2; ++s) {
    const SideCtx& sd = c.side[s];
    const int nn = sd.nn;
    const float pos = posv[s];
    if (nn == 0) {
      // losses.py:63,101-102,140-141: only the logistic loss keeps its positive term
      if (c.loss == PBG_LOSS_LOGISTIC) {
        if (lane == 0) loss_acc += softplusf(-pos);
        dposv[s] = (sigmoidf(pos) - 1.0f) * w;
      }
      continue;
    }
    ScoreRow sr = score_row(c, s, kc, cc, i);
    float* out = sd.s + (kc * c.P + i) * nn;
    float rowsum, gsum;
    side_loss<DEPTH, DIST>(c.loss, c.margin, c.cmp, sr, out, nn, pos, w, lane, &loss_acc, &dposv[s], &violv[s], &rowsum,
                          &gsum, sd.gs ? sd.gs + (kc * c.P + i) * nn : nullptr);
    if (sd.rs && lane == 0) sd.rs[kc * c.P + i] = rowsum;
    if (sd.bs && lane == 0) sd.bs[kc * c.P + i] = gsum;
  }
  const float loss_row = wave_sum(loss_acc) * w;
  if (lane == 0) {
    c.lossrow[job] = loss_row;
    c.violrow[job * 2] = violv[0];
    c.violrow[job * 2 + 1] = violv[1];
    c.pos[0][job] = posv[0];
    if (c.dynamic) {
      c.pos[1][job] = posv[1];
      c.dpos[0][job] = dposv[0];
      c.dpos[1][job] = dposv[1];
    } else {
      c.dpos[0][job] = dposv[0] + dposv[1];
    }
  }
}

// forward-only output: de-chunked, masked scores (model.py:842-844)
__global__ __launch_bounds__(kRowThreads) void scores_out_kernel(StepCtx c, float* __restrict__ lhs_pos,
                                                                 float* __restrict__ rhs_pos,
                                                                 float* __restrict__ lhs_neg,
                                                                 float* __restrict__ rhs_neg) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (job >= (int64_t)c.K * c.B) return;
  const int k = (int)(job / c.B), q = (int)(job % c.B);
  const int cc = q / c.P, i = q % c.P;
  const int64_t kc = (int64_t)k * c.C + cc;
  float posv[2];
  positive_scores(c, kc, i, lane, posv);
  if (lane == 0) {
    lhs_pos[job] = posv[0];
    rhs_pos[job] = posv[1];
  }
  for (int s = 0; s < 2; ++s) {
    const int nn = c.side[s].nn;
    if (nn == 0) continue;
    ScoreRow sr = score_row(c, s, kc, cc, i);
    float* out = (s == 0 ? lhs_neg : rhs_neg) + job * nn;
    bool live;
    for (int j = lane; j < nn; j += kWave) out[j] = sr.at(j, &live);
  }
}

// Ranking evaluation without the [B, N] score matrices (eval.py:57-81, batching.py:139-150): per edge
// the two positive scores, per side the rank of the positive among its negatives -- one more than the
// number of negatives scoring at least as high, masked entries (-1e9) included as they are in the
// reference's matrices -- and the edge's loss.  One wave per edge reads the chunk's score rows where the
// score GEMMs left them.
__device__ __forceinline__ void row_rank_and_loss(int loss, float margin, const ScoreRow& sr, int nn, float pos, int lane,
                                                  float* loss_acc, int* at_least) {
  bool live;
  int ge = 0;
  float mx = pos;
  for (int j = lane; j < nn; j += kWave) {
    const float t = sr.at(j, &live);
    if (t >= pos) ++ge;
    if (loss == PBG_LOSS_RANKING) {
      const float x = (t - pos) + margin;
      if (x > 0.f) *loss_acc += x;
    } else if (loss == PBG_LOSS_LOGISTIC) {
      float sg;
      *loss_acc += softplus_sigmoid(t, &sg) / (float)nn;
    } else {
      mx = fmaxf(mx, t);
    }
  }
  if (loss == PBG_LOSS_SOFTMAX) {
    mx = wave_max(mx);
    float z = 0.f;
    for (int j = lane; j < nn; j += kWave) z += exp_below(sr.at(j, &live), mx);
    z = wave_sum(z) + exp_below(pos, mx);
    if (lane == 0) *loss_acc += (mx + logf(z)) - pos;
  } else if (loss == PBG_LOSS_LOGISTIC) {
    if (lane == 0) *loss_acc += softplusf(-pos);
  }
  *at_least = wave_sum_int(ge);
}

__global__ __launch_bounds__(kRowThreads) void ranks_out_kernel(StepCtx c, float* __restrict__ lhs_pos,
                                                                float* __restrict__ rhs_pos,
                                                                int64_t* __restrict__ lhs_rank,
                                                                int64_t* __restrict__ rhs_rank,
                                                                float* __restrict__ loss_edge) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (job >= (int64_t)c.K * c.B) return;
  const int k = (int)(job / c.B), q = (int)(job % c.B);
  const int cc = q / c.P, i = q % c.P;
  const int64_t kc = (int64_t)k * c.C + cc;
  float posv[2];
  positive_scores(c, kc, i, lane, posv);
  float w = c.rel_weights[c.dynamic ? 0 : clamp_index(c.rel[k], c.num_relations)];
  if (c.edge_weight) w *= c.edge_weight[job];
  float loss_acc = 0.f;
  int64_t rank[2] = {0, 0};  // 0: the side has no negatives (the evaluator skips it, eval.py:61-62)
  for (int s = 0; s < 2; ++s) {
    const int nn = c.side[s].nn;
    if (nn == 0) {
      if (c.loss == PBG_LOSS_LOGISTIC && lane == 0) loss_acc += softplusf(-posv[s]);  // losses.py:63
      continue;
    }
    ScoreRow sr = score_row(c, s, kc, cc, i);
    int ge;
    row_rank_and_loss(c.loss, c.margin, sr, nn, posv[s], lane, &loss_acc, &ge);
    rank[s] = (int64_t)ge + 1;
  }
  const float loss_row = wave_sum(loss_acc) * w;
  if (lane == 0) {
    lhs_pos[job] = posv[0];
    rhs_pos[job] = posv[1];
    lhs_rank[job] = rank[0];
    rhs_rank[job] = rank[1];
    loss_edge[job] = loss_row;
  }
}

// util.py:420-428 over the call's edges: sample (a positive, an entry of the side's negatives), count
// "positive > negative".  One thread per sample and side; pos = the scores ranks_out_kernel wrote.
__global__ __launch_bounds__(256) void auc_sample_kernel(StepCtx c, const float* __restrict__ lhs_pos,
                                                         const float* __restrict__ rhs_pos, int64_t samples,
                                                         uint64_t seed, unsigned long long* __restrict__ hits) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int s = blockIdx.y;
  const int nn = c.side[s].nn;
  bool hit = false;
  if (n < samples && nn > 0) {
    const int64_t edges = (int64_t)c.K * c.B;
    const uint64_t r0 = philox_u64(seed, (uint64_t)n, (uint32_t)(2 * s)), r1 = philox_u64(seed, (uint64_t)n, (uint32_t)(2 * s + 1));
    const int64_t ep = (int64_t)(r0 % (uint64_t)edges);
    const uint64_t flat = r1 % ((uint64_t)edges * (uint64_t)nn);
    const int64_t en = (int64_t)(flat / (uint64_t)nn);
    const int j = (int)(flat % (uint64_t)nn);
    const int k = (int)(en / c.B), q = (int)(en % c.B);
    const int cc = q / c.P, i = q % c.P;
    ScoreRow sr = score_row(c, s, (int64_t)k * c.C + cc, cc, i);
    bool live;
    hit = (s == 0 ? lhs_pos : rhs_pos)[ep] > sr.at(j, &live);
  }
  const uint64_t m = __ballot(hit);
  if ((threadIdx.x & 63) == 0 && m != 0ull) atomicAdd(&hits[s], (unsigned long long)__popcll(m));
}

__global__ void zero_u64_kernel(unsigned long long* p, int n) {
  if ((int)threadIdx.x < n) p[threadIdx.x] = 0ull;
}

// ---------------------------------------------------------------------------
// rowback
// ---------------------------------------------------------------------------
// sum over the P rows of a chunk of column `col` of the stored -2 dLoss/dq
__device__ __forceinline__ float column_sum(const float* __restrict__ s, int64_t kc, int P, int nn, int col, int lane) {
  const float* base = s + kc * P * nn + col;
  float acc = 0.f;
  for (int r = lane; r < P; r += kWave) acc += base[(int64_t)r * nn];
  return wave_sum(acc);
}

// dy += dpos * d kappa(self, other) / d self
// (`half`: the term and the sum are float16 numbers, as the gradient of a Half tensor that autograd adds up is)
template <int NVH>
__device__ __forceinline__ void add_pos_term(int cmp, RowV<NVH>& dy, float dpos, const RowV<NVH>& self,
                                             const RowV<NVH>& other, float pos, bool half = false) {
  if (is_distance(cmp)) {
    // kappa = -sqrt(max(sum (a-b)^2, 1e-30)); no gradient where the clamp is active.
    // squared_l2: kappa = -sum (a-b)^2
    if (cmp == PBG_CMP_L2 && pos * pos <= 1e-30f) return;
    const float coef = cmp == PBG_CMP_L2 ? dpos / pos : -2.0f * dpos;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      dy.a[0][v] += coef * (self.a[0][v] - other.a[0][v]);
      dy.a[1][v] += coef * (self.a[1][v] - other.a[1][v]);
    }
  } else if (half) {
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      dy.a[0][v] = half_round(dy.a[0][v] + half_round(dpos * other.a[0][v]));
      dy.a[1][v] = half_round(dy.a[1][v] + half_round(dpos * other.a[1][v]));
    }
  } else {
    row_axpy<NVH>(dy, dpos, other);
  }
}

// config.bias: sum over a chunk's rows of dLoss/dscore in column `col` of side sd's score matrix
// (squared_l2 stores 2 dLoss/dscore in the matrix, l2 keeps dLoss/dscore in a matrix of its own)
__device__ __forceinline__ float bias_column_sum(const StepCtx& c, const SideCtx& sd, int64_t kc, int col, int lane) {
  if (sd.gs) return column_sum(sd.gs, kc, c.P, sd.nn, col, lane);
  return (c.cmp == PBG_CMP_SQUARED_L2 ? 0.5f : 1.0f) * column_sum(sd.s, kc, c.P, sd.nn, col, lane);
}

template <int NVH>
__global__ __launch_bounds__(kRowThreads) void rowback_kernel(StepCtx c) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int CP = c.C * c.P;
  const int J0 = c.B + c.C * c.side[0].u;
  const int J = J0 + c.B + c.C * c.side[1].u;
  if (job >= (int64_t)c.K * J) return;
  const int k = (int)(job / J);
  int r = (int)(job % J);
  const int s = r >= J0;
  if (s) r -= J0;
  const SideCtx& sd = c.side[s];
  const SideCtx& so = c.side[1 - s];
  const int D = c.D, H = (D + 1) / 2;
  const bool l2 = is_distance(c.cmp);
  const bool keep_dz = sd.dz != nullptr;
  // config.bias: a row's bias enters every score of the row (model.py:332-342), so its gradient is
  // the sum of dLoss/dscore over them: a row sum where the row is the positive operand, a column sum
  // where it is a negative, plus the positive pair's.  It joins the gradient after comparator.prepare,
  // which passes the first coordinate through.  With a regularizer the bias is a coordinate of the
  // regularized row like the others (BiasedComparator.prepare keeps it in the row, model.py:311-314):
  // it is put back for the N3 term, whose gradient at that coordinate joins the bias's.

  if (r < c.B) {
    const int cc = r / c.P, i = r % c.P;
    const int64_t kc = (int64_t)k * c.C + cc;
    const int64_t pq = (int64_t)k * CP + r;
    const int64_t e = (int64_t)k * c.B + r;
    const int64_t rel = clamp_index(c.dynamic ? c.rel[e] : c.rel[k], c.num_relations);
    float* out = c.gr + ((int64_t)k * c.rk + sd.slot_pos + r) * D;
    const RowV<NVH> y1 = row_load<NVH>(sd.xp + (kc * sd.stride_p + i) * D, D, H, lane);
    const float aux1 = sd.ap ? sd.ap[kc * sd.stride_p + i] : 0.f;
    if (!c.dynamic) {
      RowV<NVH> dy = sd.plain_written ? row_load<NVH>(sd.dxp + (kc * sd.stride_p + i) * D, D, H, lane)
                                      : row_zero<NVH>();
      if (l2) {
        float coef = 0.f;
        if (sd.nb > 0) coef -= column_sum(sd.s, kc, c.P, sd.nn, i, lane);
        if (so.nn > 0) coef += 2.0f * so.rs[kc * c.P + i];
        row_axpy<NVH>(dy, coef, y1);
      }
      const RowV<NVH> other = row_load<NVH>(so.xp + (kc * so.stride_p + i) * D, D, H, lane);
      // (the positive score carries the pair's two biases; the distance's gradient needs the distance)
      const float pair_bias = c.bias ? sd.bp[kc * sd.stride_p + i] + so.bp[kc * so.stride_p + i] : 0.f;
      add_pos_term<NVH>(c.cmp, dy, c.dpos[0][pq], y1, other, c.pos[0][pq] - pair_bias, c.half);
      float breg = 0.f;
      if (c.reg_coef != 0.f) {  // src_pos / dst_pos of the regularizer are these prepared rows (model.py:784-785,854)
        RowV<NVH> yb = y1;
        if (c.bias) add_to_first<NVH>(yb, sd.bp[kc * sd.stride_p + i], lane);
        const float cubes = wave_sum(n3_term<NVH>(c.op, c.reg_coef, dy, yb));
        if (c.bias) breg = take_bias<NVH>(dy, lane);  // (dy carried 0 there: the operand rows do)
        if (lane == 0) c.regrow[((int64_t)k * 2 + s) * c.B + r] = cubes;
      }
      RowV<NVH> dz = prepare_backward<NVH>(c.cmp, dy, y1, aux1);
      if (c.bias) {
        float db = c.dpos[0][pq] + breg;
        if (sd.nb > 0) db += bias_column_sum(c, sd, kc, i, lane);
        if (so.nn > 0) db += so.bs[kc * c.P + i];
        add_to_first<NVH>(dz, db, lane);
      }
      if (sd.has_op) {
        if (keep_dz) row_store<NVH>(sd.dz + ((int64_t)k * sd.op_rows + r) * D, dz, D, H, lane);
        if (c.op != PBG_OP_LINEAR)
          row_store<NVH>(out, op_backward<NVH>(c.op, dz, sd.p0, sd.p1, rel, D, H, lane), D, H, lane);
      } else {
        row_store<NVH>(out, dz, D, H, lane);
      }
    } else {
      // role 1: the plain row f(x), a batch negative of its own side and the
      // partner of the other side's operated positive
      RowV<NVH> dy = row_zero<NVH>();
      if (sd.alias) {
        dy = row_load<NVH>(sd.dxp + (kc * sd.stride_p + i) * D, D, H, lane);
        if (l2) row_axpy<NVH>(dy, -column_sum(sd.s, kc, c.P, sd.nn, i, lane), y1);
      }
      const RowV<NVH> other = row_load<NVH>(so.xa + (kc * c.P + i) * D, D, H, lane);
      const float pair_bias = c.bias ? sd.bp[kc * sd.stride_p + i] + so.ba[kc * c.P + i] : 0.f;
      add_pos_term<NVH>(c.cmp, dy, c.dpos[s][pq], y1, other, c.pos[s][pq] - pair_bias, c.half);
      // the plain row is src_pos of one direction's regularizer, the operated row
      // dst_pos of the other's (model.py:722-754)
      float cubes = 0.f, breg = 0.f, breg2 = 0.f;
      if (c.reg_coef != 0.f) {
        RowV<NVH> yb = y1;
        if (c.bias) add_to_first<NVH>(yb, sd.bp[kc * sd.stride_p + i], lane);
        cubes = n3_term<NVH>(c.op, c.reg_coef, dy, yb);
        if (c.bias) breg = take_bias<NVH>(dy, lane);
      }
      RowV<NVH> dx = prepare_backward<NVH>(c.cmp, dy, y1, aux1);
      if (c.bias) {
        float db = c.dpos[s][pq] + breg;
        if (sd.alias) db += bias_column_sum(c, sd, kc, i, lane);
        add_to_first<NVH>(dx, db, lane);
      }
      // role 2: the operated row f(op(x)), scored against the other side's negatives
      const RowV<NVH> y2 = row_load<NVH>(sd.xa + (kc * c.P + i) * D, D, H, lane);
      const float aux2 = sd.aa ? sd.aa[kc * c.P + i] : 0.f;
      RowV<NVH> dy2 = row_zero<NVH>();
      if (sd.opd_written) {
        dy2 = row_load<NVH>(sd.dxa + (kc * c.P + i) * D, D, H, lane);
        if (l2) row_axpy<NVH>(dy2, 2.0f * so.rs[kc * c.P + i], y2);
      }
      const RowV<NVH> other2 = row_load<NVH>(so.xp + (kc * so.stride_p + i) * D, D, H, lane);
      const float pair_bias2 = c.bias ? sd.ba[kc * c.P + i] + so.bp[kc * so.stride_p + i] : 0.f;
      add_pos_term<NVH>(c.cmp, dy2, c.dpos[1 - s][pq], y2, other2, c.pos[1 - s][pq] - pair_bias2, c.half);
      if (c.reg_coef != 0.f) {
        RowV<NVH> yb2 = y2;
        if (c.bias) add_to_first<NVH>(yb2, sd.ba[kc * c.P + i], lane);
        cubes = wave_sum(cubes + n3_term<NVH>(c.op, c.reg_coef, dy2, yb2));
        if (c.bias) breg2 = take_bias<NVH>(dy2, lane);
        if (lane == 0) c.regrow[((int64_t)k * 2 + s) * c.B + r] = cubes;
      }
      RowV<NVH> dz2 = prepare_backward<NVH>(c.cmp, dy2, y2, aux2);
      if (c.bias)
        add_to_first<NVH>(dz2, c.dpos[1 - s][pq] + breg2 + (sd.opd_written ? so.bs[kc * c.P + i] : 0.f), lane);
      if (keep_dz) row_store<NVH>(sd.dz + ((int64_t)k * sd.op_rows + r) * D, dz2, D, H, lane);
      if (c.op != PBG_OP_LINEAR) {
        const RowV<NVH> dx2 = op_backward<NVH>(c.op, dz2, sd.p0, sd.p1, rel, D, H, lane);
        row_axpy<NVH>(dx, 1.0f, dx2);
      }
      row_store<NVH>(out, dx, D, H, lane);
    }
  } else {
    if (sd.uni_direct) return;  // the GEMM's row is the gradient row
    const int r2 = r - c.B;
    const int cc = r2 / sd.u, uu = r2 % sd.u;
    const int64_t kc = (int64_t)k * c.C + cc;
    const int col = sd.nb + uu;
    float* out = c.gr + ((int64_t)k * c.rk + sd.slot_uni + r2) * D;
    // the prepared row itself only enters through the norm terms (l2, squared_l2) and cos's normalisation
    const RowV<NVH> y = c.cmp != PBG_CMP_DOT ? row_load<NVH>(sd.xn + (kc * sd.nn + col) * D, D, H, lane) : row_zero<NVH>();
    RowV<NVH> dy = row_load<NVH>(sd.dxn + (kc * sd.nn + col) * D, D, H, lane);
    if (l2) row_axpy<NVH>(dy, -column_sum(sd.s, kc, c.P, sd.nn, col, lane), y);
    RowV<NVH> dz = prepare_backward<NVH>(c.cmp, dy, y, sd.an ? sd.an[kc * sd.nn + col] : 0.f);
    if (c.bias) add_to_first<NVH>(dz, bias_column_sum(c, sd, kc, col, lane), lane);
    if (sd.op_uniform) {
      const int64_t rel = clamp_index(c.rel[k], c.num_relations);
      if (keep_dz && !sd.uni_dz_direct) row_store<NVH>(sd.dz + ((int64_t)k * sd.op_rows + c.B + r2) * D, dz, D, H, lane);
      if (c.op != PBG_OP_LINEAR)
        row_store<NVH>(out, op_backward<NVH>(c.op, dz, sd.p0, sd.p1, rel, D, H, lane), D, H, lane);
    } else {
      row_store<NVH>(out, dz, D, H, lane);
    }
  }
}

// ---------------------------------------------------------------------------
// operator parameters (standard mode: one relation per batch)
// ---------------------------------------------------------------------------
// dth[k, slice, e] = sum over the operator rows r = slice (mod slices) of batch k
// of the parameter gradient of element e: diagonal x.dz, translation dz,
// complex_diagonal (real | imag).  Fixed summation order, no atomics.
constexpr int kParamGroups = 16;
// `reg_op`: the operator whose parameters the N3 term is taken over (c.op, except where the caller
// has set c.op to translation to get plain column sums of rows that hold finished gradient terms).
__global__ __launch_bounds__(kParamGroups * 64) void param_grad_kernel(StepCtx c, int s, float* __restrict__ dth,
                                                                        int slices, int reg_op) {
  __shared__ float sh[kParamGroups][64];
  const SideCtx& sd = c.side[s];
  const int lane = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int k = blockIdx.y, slice = blockIdx.z;
  const int e = blockIdx.x * 64 + lane;
  const int D = c.D, H = D / 2;
  float acc = 0.f;
  if (e < D) {
    // chunk and column of the uniform negative the loop is at, kept without a division per row
    const int step = slices * kParamGroups;
    int cc = 0, uu = 0;
    bool in_uniform = false;
    for (int r = slice * kParamGroups + rg; r < sd.op_rows; r += step) {
      const float* dz = sd.dz + ((int64_t)k * sd.op_rows + r) * D;
      if (sd.uni_dz_direct && r >= c.B) {
        if (!in_uniform) {
          in_uniform = true;
          cc = (r - c.B) / sd.u;
          uu = (r - c.B) % sd.u;
        }
        dz = sd.dxn + (((int64_t)k * c.C + cc) * sd.nn + sd.nb + uu) * D;
        uu += step;
        while (uu >= sd.u) {
          uu -= sd.u;
          ++cc;
        }
      }
      if (c.op == PBG_OP_TRANSLATION) {
        acc += dz[e];
        continue;
      }
      int64_t id;
      if (r < c.B) {
        id = sd.idx[(int64_t)k * c.B + r];
      } else {
        id = uniform_negative(sd, s, (int64_t)k * c.C * sd.u + (r - c.B));  // = (k C + chunk) u + column
      }
      const float* x = sd.w + clamp_index(id, sd.num_rows) * D;
      const float* gl = sd.glob;  // the operator's input is the row plus the global embedding
      if (c.op == PBG_OP_DIAGONAL) {
        acc += (x[e] + (gl ? gl[e] : 0.f)) * dz[e];
      } else if (e < H) {  // d/d real
        acc += (x[e] + (gl ? gl[e] : 0.f)) * dz[e] + (x[e + H] + (gl ? gl[e + H] : 0.f)) * dz[e + H];
      } else {             // d/d imag
        const int h = e - H;
        acc += (x[h] + (gl ? gl[h] : 0.f)) * dz[h + H] - (x[h + H] + (gl ? gl[h + H] : 0.f)) * dz[h];
      }
    }
  }
  sh[rg][lane] = acc;
  __syncthreads();
  if (rg == 0 && e < D) {
    float total = 0.f;
#pragma unroll
    for (int g = 0; g < kParamGroups; ++g) total += sh[g][lane];
    if (slice == 0 && c.reg_coef != 0.f) {
      // N3 on the operator's parameters (regularizers.py:90-93): coef * C * sum m^3, with
      // m = |p| (operators.py:69-70,83-84) or the modulus of (real, imag) (operators.py:151-152)
      const int64_t r = clamp_index(c.rel[k], c.num_relations);
      const float c3 = 3.0f * c.reg_coef * (float)c.C;
      if (reg_op == PBG_OP_COMPLEX_DIAGONAL) {
        const int h = e < H ? e : e - H;
        const float re = sd.p0[r * H + h], im = sd.p1[r * H + h];
        total += c3 * sqrtf(re * re + im * im) * (e < H ? re : im);
      } else {
        const float pv = sd.p0[r * D + e];
        total += c3 * fabsf(pv) * pv;
      }
    }
    dth[((int64_t)k * slices + slice) * D + e] = total;
  }
}

// The same sums for rows whose length is a multiple of 4 (of 8 with complex_diagonal): four columns per lane --
// with complex_diagonal four (real, imaginary) pairs -- as 128-bit loads, four rows in flight.  The rows a group
// takes, their order and the order of the groups are param_grad_kernel's, and so is every sum.  On the fused
// route the rows' ids are the ones its id kernel has left behind (c.fused_rowid), not drawn again.
template <int OP>
__global__ __launch_bounds__(kParamGroups * 64) void param_grad_quad_kernel(StepCtx c, int s, float* __restrict__ dth,
                                                                             int slices, int reg_op) {
  constexpr bool cplx = OP == PBG_OP_COMPLEX_DIAGONAL;
  constexpr int NA = cplx ? 2 : 1;
  constexpr int kFusedSide = kFusedIds / 2;
  __shared__ float4 sh[NA][kParamGroups][64];
  const SideCtx& sd = c.side[s];
  const int lane = threadIdx.x & 63, rg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int k = blockIdx.y, slice = blockIdx.z;
  const int D = c.D, H = D / 2;
  const int quads = (cplx ? H : D) >> 2;
  const int q = blockIdx.x * 64 + lane;
  const int e = 4 * min(q, quads - 1);  // (lanes past the last quad read the last one and store nothing)
  const int step = slices * kParamGroups;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 acc[NA];
#pragma unroll
  for (int a = 0; a < NA; ++a) acc[a] = zero;
  float4 gl[NA];
#pragma unroll
  for (int a = 0; a < NA; ++a) gl[a] = (OP != PBG_OP_TRANSLATION && sd.glob) ? *reinterpret_cast<const float4*>(sd.glob + e + a * H) : zero;
  auto dz_of = [&](int r) -> const float* {
    if (sd.uni_dz_direct && r >= c.B) {
      const int cc = (r - c.B) / sd.u, uu = (r - c.B) - cc * sd.u;
      return sd.dxn + (((int64_t)k * c.C + cc) * sd.nn + sd.nb + uu) * D;
    }
    return sd.dz + ((int64_t)k * sd.op_rows + r) * D;
  };
  auto x_of = [&](int r) -> const float* {  // the operator's input row (without the global embedding)
    int64_t id;
    if (c.fused_rowid) {
      const bool uni = r >= c.B;
      const int cc = uni ? (r - c.B) / c.U : r / c.P;
      const int j = uni ? c.P + (r - c.B) - cc * c.U : r - cc * c.P;
      id = c.fused_rowid[((int64_t)k * c.C + cc) * kFusedIds + s * kFusedSide + j];
      if (id < 0) id = 0;
    } else if (r < c.B) {
      id = clamp_index(sd.idx[(int64_t)k * c.B + r], sd.num_rows);
    } else {
      id = clamp_index(uniform_negative(sd, s, (int64_t)k * c.C * sd.u + (r - c.B)), sd.num_rows);
    }
    return sd.w + id * D;
  };
  for (int r0 = slice * kParamGroups + rg; r0 < sd.op_rows; r0 += 4 * step) {
    float4 g[4][NA], x[4][NA];
    bool live[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = r0 + j * step;
      live[j] = r < sd.op_rows;
      const int rr = live[j] ? r : r0;
      const float* dz = dz_of(rr);
      const float* xr = OP == PBG_OP_TRANSLATION ? dz : x_of(rr);
#pragma unroll
      for (int a = 0; a < NA; ++a) {
        g[j][a] = *reinterpret_cast<const float4*>(dz + e + a * H);
        x[j][a] = OP == PBG_OP_TRANSLATION ? zero : *reinterpret_cast<const float4*>(xr + e + a * H);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!live[j]) break;
      if constexpr (OP == PBG_OP_TRANSLATION) {
        acc[0].x += g[j][0].x; acc[0].y += g[j][0].y; acc[0].z += g[j][0].z; acc[0].w += g[j][0].w;
      } else if constexpr (!cplx) {
        acc[0].x += (x[j][0].x + gl[0].x) * g[j][0].x; acc[0].y += (x[j][0].y + gl[0].y) * g[j][0].y;
        acc[0].z += (x[j][0].z + gl[0].z) * g[j][0].z; acc[0].w += (x[j][0].w + gl[0].w) * g[j][0].w;
      } else {
        const float4 xr = make_float4(x[j][0].x + gl[0].x, x[j][0].y + gl[0].y, x[j][0].z + gl[0].z, x[j][0].w + gl[0].w);
        const float4 xi = make_float4(x[j][1].x + gl[1].x, x[j][1].y + gl[1].y, x[j][1].z + gl[1].z, x[j][1].w + gl[1].w);
        const float4 gr = g[j][0], gi = g[j][1];
        acc[0].x += xr.x * gr.x + xi.x * gi.x; acc[0].y += xr.y * gr.y + xi.y * gi.y;
        acc[0].z += xr.z * gr.z + xi.z * gi.z; acc[0].w += xr.w * gr.w + xi.w * gi.w;
        acc[1].x += xr.x * gi.x - xi.x * gr.x; acc[1].y += xr.y * gi.y - xi.y * gr.y;
        acc[1].z += xr.z * gi.z - xi.z * gr.z; acc[1].w += xr.w * gi.w - xi.w * gr.w;
      }
    }
  }
#pragma unroll
  for (int a = 0; a < NA; ++a) sh[a][rg][lane] = acc[a];
  __syncthreads();
  if (rg == 0 && q < quads) {
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < kParamGroups; ++g) {
        const float4 v = sh[a][g][lane];
        t[0] += v.x; t[1] += v.y; t[2] += v.z; t[3] += v.w;
      }
      if (slice == 0 && c.reg_coef != 0.f) {  // N3 on the operator's parameters, as in param_grad_kernel
        const int64_t r = clamp_index(c.rel[k], c.num_relations);
        const float c3 = 3.0f * c.reg_coef * (float)c.C;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (reg_op == PBG_OP_COMPLEX_DIAGONAL) {
            const int col = e + a * H + i, h = col < H ? col : col - H;
            const float re = sd.p0[r * H + h], im = sd.p1[r * H + h];
            t[i] += c3 * sqrtf(re * re + im * im) * (col < H ? re : im);
          } else {
            const float pv = sd.p0[r * D + e + a * H + i];
            t[i] += c3 * fabsf(pv) * pv;
          }
        }
      }
      *reinterpret_cast<float4*>(dth + ((int64_t)k * slices + slice) * D + e + a * H) = make_float4(t[0], t[1], t[2], t[3]);
    }
  }
}

// param_grad_kernel, or its 128-bit form where the rows' length allows it
void launch_param_grad(const StepCtx& c, int s, float* dth, int slices, int reg_op, hipStream_t stream) {
  const int D = c.D, K = c.K;
  const dim3 block(kParamGroups * 64);
  if (c.op == PBG_OP_COMPLEX_DIAGONAL && D % 8 == 0) {
    hipLaunchKernelGGL((param_grad_quad_kernel<PBG_OP_COMPLEX_DIAGONAL>), dim3((unsigned)ceil_div(D / 8, 64), (unsigned)K, (unsigned)slices),
                       block, 0, stream, c, s, dth, slices, reg_op);
  } else if (c.op == PBG_OP_DIAGONAL && D % 4 == 0) {
    hipLaunchKernelGGL((param_grad_quad_kernel<PBG_OP_DIAGONAL>), dim3((unsigned)ceil_div(D / 4, 64), (unsigned)K, (unsigned)slices),
                       block, 0, stream, c, s, dth, slices, reg_op);
  } else if (c.op == PBG_OP_TRANSLATION && D % 4 == 0) {
    hipLaunchKernelGGL((param_grad_quad_kernel<PBG_OP_TRANSLATION>), dim3((unsigned)ceil_div(D / 4, 64), (unsigned)K, (unsigned)slices),
                       block, 0, stream, c, s, dth, slices, reg_op);
  } else {
    hipLaunchKernelGGL(param_grad_kernel, dim3((unsigned)ceil_div(D, 64), (unsigned)K, (unsigned)slices), block, 0, stream, c, s,
                       dth, slices, reg_op);
  }
}

// AsyncAdagrad (async_adagrad.py:75-85), the K batches' gradients applied in order.
__global__ void param_update_kernel(StepCtx c, int s, const float* __restrict__ dth, int slices, int64_t psize,
                                    float* p0, float* p1, float* s0, float* s1, float lr) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= psize) return;
  const int H = c.D / 2;
  for (int k = 0; k < c.K; ++k) {
    const int64_t r = clamp_index(c.rel[k], c.num_relations);
    float* p;
    float* st;
    if (c.op == PBG_OP_COMPLEX_DIAGONAL) {
      if (e < H) {
        p = p0 + r * H + e;
        st = s0 + r * H + e;
      } else {
        p = p1 + r * H + (e - H);
        st = s1 + r * H + (e - H);
      }
    } else {
      p = p0 + r * psize + e;
      st = s0 + r * psize + e;
    }
    float g = 0.f;
    for (int sl = 0; sl < slices; ++sl) g += dth[((int64_t)k * slices + sl) * psize + e];
    const float sum = *st + g * g;
    *st = sum;
    *p += -lr * (g / (sqrtf(sum) + 1e-10f));
  }
}

// The same for K <= 64 with one wave per parameter element: lane k sums batch k's
// slices and fetches the parameter and its Adagrad sum of batch k's relation, all
// lanes at once; the K updates then run in order on registers, an updated value
// handed on to the later batches of the same relation, and the last batch of
// every relation stores.  The chain of K dependent global read-modify-writes of
// the kernel above becomes one round trip.
__global__ __launch_bounds__(kRowThreads) void param_update_wave_kernel(StepCtx c, int s, const float* __restrict__ dth,
                                                                        int slices, int64_t psize, float* p0,
                                                                        float* p1, float* s0, float* s1, float lr) {
  const int lane = threadIdx.x & 63;
  const int64_t e = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (e >= psize) return;
  const int H = c.D / 2, K = c.K;
  const bool on = lane < K;
  const int64_t r = on ? clamp_index(c.rel[lane], c.num_relations) : -1 - lane;  // idle lanes match nobody
  float* p = nullptr;
  float* st = nullptr;
  if (on) {
    if (c.op == PBG_OP_COMPLEX_DIAGONAL) {
      p = e < H ? p0 + r * H + e : p1 + r * H + (e - H);
      st = e < H ? s0 + r * H + e : s1 + r * H + (e - H);
    } else {
      p = p0 + r * psize + e;
      st = s0 + r * psize + e;
    }
  }
  float g = 0.f;
  if (on)
    for (int sl = 0; sl < slices; ++sl) g += dth[((int64_t)lane * slices + sl) * psize + e];
  float pv = on ? *p : 0.f, sv = on ? *st : 0.f;
  const int rlo = (int)(uint32_t)r, rhi = (int)(uint32_t)((uint64_t)r >> 32);
  bool last = on;
  for (int k = 0; k < K; ++k) {
    const bool same = __builtin_amdgcn_readlane(rlo, k) == rlo && __builtin_amdgcn_readlane(rhi, k) == rhi;
    // batch k's step, computed by every lane from lane k's registers
    const float gk = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(g), k));
    const float sum = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sv), k)) + gk * gk;
    const float pn = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pv), k)) + -lr * (gk / (sqrtf(sum) + 1e-10f));
    if (same && lane >= k) {  // lane k itself and the later batches of the same relation
      sv = sum;
      pv = pn;
    }
    if (same && lane < k) last = false;
  }
  if (last) {
    *st = sv;
    *p = pv;
  }
}

// ---------------------------------------------------------------------------
// operator parameters, dynamic relations (one relation per edge)
// ---------------------------------------------------------------------------
// sort keys (relation << kbits | batch) of every positive, value = k * B + q
__global__ void rel_keys_kernel(StepCtx c, uint64_t* __restrict__ keys, uint32_t* __restrict__ vals) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)c.K * c.B) return;
  const int64_t r = clamp_index(c.rel[e], c.num_relations);
  keys[e] = ((uint64_t)r << c.kbits) | (uint64_t)(e / c.B);
  vals[e] = (uint32_t)e;
}

// First position after `start` whose key >> shift differs from `want` (block-wide, 256 threads).
__device__ __forceinline__ int64_t block_scan_end(const uint64_t* __restrict__ keys, int64_t start, int64_t n,
                                                  uint64_t want, int shift, int64_t* sh_end) {
  int64_t base = start + 1;
  while (true) {
    if (threadIdx.x == 0) *sh_end = -1;
    __syncthreads();
    const int64_t j = base + threadIdx.x;
    const bool same = (j < n) && ((keys[j] >> shift) == want);
    const bool prev_same = (j == base) || ((j - 1 < n) && ((keys[j - 1] >> shift) == want));
    if (!same && prev_same && j <= n) *sh_end = j;  // exactly one thread sees the first mismatch
    __syncthreads();
    const int64_t found = *sh_end;
    __syncthreads();
    if (found >= 0) return found;
    base += blockDim.x;
  }
}

// Element-wise operators, in two kernels.  A relation's runs (its edges of one batch each,
// ascending) update its parameters one after the other (AsyncAdagrad,
// async_adagrad.py:75-85: the K batches' updates in order), but a run's gradient depends
// on nothing but the tables as they were on entry:
//   grad    one workgroup per (run, 64-element slice) sums the run's parameter gradient over
//           its edges in a fixed order and leaves it at the run's first sorted position;
//   apply   one wave per (relation present in the call, 64-element slice) walks the
//           relation's runs and applies their gradients in order.
// With relation frequencies following a power law the busiest relation owns a tenth of a
// call's edges: walking its runs AND their edges in one chain of dependent loads would take
// longer than everything else in the call together.
__device__ __forceinline__ float dyn_param_term(const StepCtx& c, const SideCtx& sd, int64_t edge, int e, int H) {
  const int D = c.D;
  const float* dz = sd.dz + edge * D;
  if (c.op == PBG_OP_TRANSLATION) return dz[e];
  const float* x = sd.w + clamp_index(sd.idx[edge], sd.num_rows) * D;
  if (c.op == PBG_OP_DIAGONAL) return x[e] * dz[e];
  if (e < H) return x[e] * dz[e] + x[e + H] * dz[e + H];
  const int h = e - H;
  return x[h] * dz[h + H] - x[h + H] * dz[h];
}

__global__ __launch_bounds__(256) void dyn_param_grad_kernel(StepCtx c, int s, const uint64_t* __restrict__ keys,
                                                             const uint32_t* __restrict__ vals, float* __restrict__ grun) {
  __shared__ float sh[4][64];
  __shared__ int64_t sh_end;
  const SideCtx& sd = c.side[s];
  const int64_t n = (int64_t)c.K * c.B;
  const int64_t i = blockIdx.x;
  const uint64_t key = keys[i];
  if (i > 0 && keys[i - 1] == key) return;  // not the first position of a run
  const int lane = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int e = blockIdx.y * 64 + lane;
  const int D = c.D, H = D / 2;
  const int64_t end = block_scan_end(keys, i, n, key, 0, &sh_end);
  float acc = 0.f;
  if (e < D) {
    int64_t r = i + rg;
    for (; r + 4 < end; r += 8) {  // two edges' chains of loads (value -> index -> rows) in flight
      const int64_t e0 = vals[r], e1 = vals[r + 4];
      const float t0 = dyn_param_term(c, sd, e0, e, H), t1 = dyn_param_term(c, sd, e1, e, H);
      acc += t0;
      acc += t1;
    }
    if (r < end) acc += dyn_param_term(c, sd, vals[r], e, H);
  }
  sh[rg][lane] = acc;
  __syncthreads();
  if (rg == 0 && e < D) {
    float g = (sh[0][lane] + sh[1][lane]) + (sh[2][lane] + sh[3][lane]);
    // N3 on the parameters of the run's edges (regularizers.py:73-76), from the values before this call
    if (c.reg_coef != 0.f) g += (float)(end - i) * sd.reg_pgrad[(key >> c.kbits) * D + e];
    grun[i * D + e] = g;
  }
}

__global__ __launch_bounds__(64) void dyn_param_apply_kernel(StepCtx c, const uint64_t* __restrict__ keys,
                                                             const float* __restrict__ grun, float* p0, float* p1, float* s0,
                                                             float* s1, float lr) {
  const int64_t n = (int64_t)c.K * c.B;
  const int64_t i = blockIdx.x;
  const uint64_t rel = keys[i] >> c.kbits;
  if (i > 0 && (keys[i - 1] >> c.kbits) == rel) return;  // not the first position of a relation
  const int lane = threadIdx.x;
  const int e = blockIdx.y * 64 + lane;
  const int D = c.D, H = D / 2;
  const bool on = e < D;
  float* p = nullptr;
  float* st = nullptr;
  if (on) {
    if (c.op == PBG_OP_COMPLEX_DIAGONAL) {
      p = (e < H) ? p0 + rel * H + e : p1 + rel * H + (e - H);
      st = (e < H) ? s0 + rel * H + e : s1 + rel * H + (e - H);
    } else {
      p = p0 + rel * D + e;
      st = s0 + rel * D + e;
    }
  }
  float pv = on ? *p : 0.f, sum = on ? *st : 0.f;
  int64_t j = i;
  while (true) {
    const float g = on ? grun[j * D + e] : 0.f;
    // the next run: the first later position with another key (all lanes scan together)
    const uint64_t key = keys[j];
    int64_t base = j + 1, next;
    while (true) {
      const int64_t q = base + lane;
      const uint64_t m = __ballot(q < n && keys[q] == key);
      if (m != ~0ull) {
        next = base + (__ffsll((unsigned long long)~m) - 1);
        break;
      }
      base += 64;
    }
    sum += g * g;
    pv += -lr * (g / (sqrtf(sum) + 1e-10f));
    if (next >= n || (keys[next] >> c.kbits) != rel) break;
    j = next;
  }
  if (on) {
    *st = sum;
    *p = pv;
  }
}

// The same two kernels for rows whose length is a multiple of 4 (of 8 with complex_diagonal): four columns -- four
// (real, imaginary) pairs -- per lane as 128-bit loads, so one workgroup per run instead of one per 64 elements,
// every sum in dyn_param_grad_kernel's order.  The grad kernel also leaves at a run's first position where the
// relation's next run starts (-1: none), so that the apply kernel's walk is one dependent load per run instead
// of a scan of the run's keys.
template <int OP>
__global__ __launch_bounds__(256) void dyn_param_grad_quad_kernel(StepCtx c, int s, const uint64_t* __restrict__ keys,
                                                                  const uint32_t* __restrict__ vals, float* __restrict__ grun,
                                                                  int64_t* __restrict__ run_next) {
  constexpr bool cplx = OP == PBG_OP_COMPLEX_DIAGONAL;
  constexpr int NA = cplx ? 2 : 1;
  __shared__ float4 sh[NA][4][64];
  __shared__ int64_t sh_end;
  const SideCtx& sd = c.side[s];
  const int64_t n = (int64_t)c.K * c.B;
  const int64_t i = blockIdx.x;
  const uint64_t key = keys[i];
  if (i > 0 && keys[i - 1] == key) return;  // not the first position of a run
  const int lane = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int D = c.D, H = D / 2;
  const int quads = (cplx ? H : D) >> 2;
  const int q = blockIdx.y * 64 + lane;
  const int e = 4 * min(q, quads - 1);  // (lanes past the last quad read the last one and store nothing)
  const int64_t end = block_scan_end(keys, i, n, key, 0, &sh_end);
  if (blockIdx.y == 0 && threadIdx.x == 0)
    run_next[i] = (end < n && (keys[end] >> c.kbits) == (key >> c.kbits)) ? end : -1;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 acc[NA];
#pragma unroll
  for (int a = 0; a < NA; ++a) acc[a] = zero;
  auto add_term = [&](const float4 (&g)[NA], const float4 (&x)[NA]) {
    if constexpr (OP == PBG_OP_TRANSLATION) {
      acc[0].x += g[0].x; acc[0].y += g[0].y; acc[0].z += g[0].z; acc[0].w += g[0].w;
    } else if constexpr (!cplx) {
      acc[0].x += x[0].x * g[0].x; acc[0].y += x[0].y * g[0].y; acc[0].z += x[0].z * g[0].z; acc[0].w += x[0].w * g[0].w;
    } else {
      acc[0].x += x[0].x * g[0].x + x[1].x * g[1].x; acc[0].y += x[0].y * g[0].y + x[1].y * g[1].y;
      acc[0].z += x[0].z * g[0].z + x[1].z * g[1].z; acc[0].w += x[0].w * g[0].w + x[1].w * g[1].w;
      acc[1].x += x[0].x * g[1].x - x[1].x * g[0].x; acc[1].y += x[0].y * g[1].y - x[1].y * g[0].y;
      acc[1].z += x[0].z * g[1].z - x[1].z * g[0].z; acc[1].w += x[0].w * g[1].w - x[1].w * g[0].w;
    }
  };
  auto load_edge = [&](int64_t edge, float4 (&g)[NA], float4 (&x)[NA]) {
    const float* dz = sd.dz + edge * D + e;
    const float* xr = OP == PBG_OP_TRANSLATION ? dz : sd.w + clamp_index(sd.idx[edge], sd.num_rows) * D + e;
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      g[a] = *reinterpret_cast<const float4*>(dz + a * H);
      x[a] = OP == PBG_OP_TRANSLATION ? zero : *reinterpret_cast<const float4*>(xr + a * H);
    }
  };
  int64_t r = i + rg;
  for (; r + 4 < end; r += 8) {  // two edges' chains of loads (value -> index -> rows) in flight
    const int64_t e0 = vals[r], e1 = vals[r + 4];
    float4 g0[NA], x0[NA], g1[NA], x1[NA];
    load_edge(e0, g0, x0);
    load_edge(e1, g1, x1);
    add_term(g0, x0);
    add_term(g1, x1);
  }
  if (r < end) {
    float4 g0[NA], x0[NA];
    load_edge(vals[r], g0, x0);
    add_term(g0, x0);
  }
#pragma unroll
  for (int a = 0; a < NA; ++a) sh[a][rg][lane] = acc[a];
  __syncthreads();
  if (rg == 0 && q < quads) {
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      const float4 v0 = sh[a][0][lane], v1 = sh[a][1][lane], v2 = sh[a][2][lane], v3 = sh[a][3][lane];
      float4 g = make_float4((v0.x + v1.x) + (v2.x + v3.x), (v0.y + v1.y) + (v2.y + v3.y), (v0.z + v1.z) + (v2.z + v3.z),
                             (v0.w + v1.w) + (v2.w + v3.w));
      // N3 on the parameters of the run's edges (regularizers.py:73-76), from the values before this call
      if (c.reg_coef != 0.f) {
        const float4 rp = *reinterpret_cast<const float4*>(sd.reg_pgrad + (key >> c.kbits) * D + e + a * H);
        const float cnt = (float)(end - i);
        g.x += cnt * rp.x; g.y += cnt * rp.y; g.z += cnt * rp.z; g.w += cnt * rp.w;
      }
      *reinterpret_cast<float4*>(grun + i * D + e + a * H) = g;
    }
  }
}

__global__ __launch_bounds__(64) void dyn_param_apply_quad_kernel(StepCtx c, const uint64_t* __restrict__ keys,
                                                                  const float* __restrict__ grun,
                                                                  const int64_t* __restrict__ run_next, float* p0, float* p1,
                                                                  float* s0, float* s1, float lr) {
  const int64_t i = blockIdx.x;
  const uint64_t rel = keys[i] >> c.kbits;
  if (i > 0 && (keys[i - 1] >> c.kbits) == rel) return;  // not the first position of a relation
  const int lane = threadIdx.x;
  const int D = c.D, H = D / 2;
  const int q = blockIdx.y * 64 + lane;
  const bool on = q < (D >> 2);
  const int e = 4 * min(q, (D >> 2) - 1);
  float* p;
  float* st;
  if (c.op == PBG_OP_COMPLEX_DIAGONAL) {  // (H is a multiple of 4 here: a quad lies in one half)
    p = (e < H) ? p0 + rel * H + e : p1 + rel * H + (e - H);
    st = (e < H) ? s0 + rel * H + e : s1 + rel * H + (e - H);
  } else {
    p = p0 + rel * D + e;
    st = s0 + rel * D + e;
  }
  float4 pv = *reinterpret_cast<const float4*>(p), sum = *reinterpret_cast<const float4*>(st);
  int64_t j = i;
  while (j >= 0) {
    const float4 g = *reinterpret_cast<const float4*>(grun + j * D + e);
    const int64_t next = run_next[j];
    sum.x += g.x * g.x; sum.y += g.y * g.y; sum.z += g.z * g.z; sum.w += g.w * g.w;
    pv.x += -lr * (g.x / (sqrtf(sum.x) + 1e-10f)); pv.y += -lr * (g.y / (sqrtf(sum.y) + 1e-10f));
    pv.z += -lr * (g.z / (sqrtf(sum.z) + 1e-10f)); pv.w += -lr * (g.w / (sqrtf(sum.w) + 1e-10f));
    j = next;
  }
  if (on) {
    *reinterpret_cast<float4*>(st) = sum;
    *reinterpret_cast<float4*>(p) = pv;
  }
}

// The two kernels of an element-wise operator's parameters with one relation per edge, in their 128-bit form where
// the rows' length allows it.
void launch_dyn_params(const StepCtx& c, int s, int64_t ne, const uint64_t* rkeys, const uint32_t* rvals, float* grun,
                       int64_t* run_next, float* p0, float* p1, float* s0, float* s1, float lr, hipStream_t stream) {
  const int D = c.D;
  const bool cplx = c.op == PBG_OP_COMPLEX_DIAGONAL;
  if (D % (cplx ? 8 : 4) != 0 || (c.op != PBG_OP_TRANSLATION && c.op != PBG_OP_DIAGONAL && !cplx)) {
    hipLaunchKernelGGL(dyn_param_grad_kernel, dim3((unsigned)ne, (unsigned)ceil_div(D, 64)), dim3(256), 0, stream, c, s,
                       rkeys, rvals, grun);
    hipLaunchKernelGGL(dyn_param_apply_kernel, dim3((unsigned)ne, (unsigned)ceil_div(D, 64)), dim3(64), 0, stream, c, rkeys,
                       grun, p0, p1, s0, s1, lr);
    return;
  }
  const dim3 grid((unsigned)ne, (unsigned)ceil_div((cplx ? D / 2 : D) / 4, 64));
  if (cplx)
    hipLaunchKernelGGL((dyn_param_grad_quad_kernel<PBG_OP_COMPLEX_DIAGONAL>), grid, dim3(256), 0, stream, c, s, rkeys, rvals, grun, run_next);
  else if (c.op == PBG_OP_DIAGONAL)
    hipLaunchKernelGGL((dyn_param_grad_quad_kernel<PBG_OP_DIAGONAL>), grid, dim3(256), 0, stream, c, s, rkeys, rvals, grun, run_next);
  else
    hipLaunchKernelGGL((dyn_param_grad_quad_kernel<PBG_OP_TRANSLATION>), grid, dim3(256), 0, stream, c, s, rkeys, rvals, grun, run_next);
  hipLaunchKernelGGL(dyn_param_apply_quad_kernel, dim3((unsigned)ne, (unsigned)ceil_div(D / 4, 64)), dim3(64), 0, stream, c,
                     rkeys, grun, run_next, p0, p1, s0, s1, lr);
}

// ---------------------------------------------------------------------------
// N3 regularizer: parameter terms and the per-batch value
// ---------------------------------------------------------------------------
// Dynamic relations, one wave per relation: reg_pgrad[rel, e] = d (coef * sum m^3) / d p[rel, e]
// for one edge of the relation, reg_pcube[rel] = sum m^3 (regularizers.py:73-76;
// operators.py:225-228,246-249,332-333).
__global__ __launch_bounds__(kRowThreads) void reg_factor_kernel(StepCtx c, int s) {
  const SideCtx& sd = c.side[s];
  const int lane = threadIdx.x & 63;
  const int64_t rel = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (rel >= c.num_relations) return;
  const int D = c.D, H = D / 2;
  const float c3 = 3.0f * c.reg_coef;
  float cubes = 0.f;
  for (int e = lane; e < D; e += kWave) {
    float m, pv;
    if (c.op == PBG_OP_COMPLEX_DIAGONAL) {
      const int h = e < H ? e : e - H;
      const float re = sd.p0[rel * H + h], im = sd.p1[rel * H + h];
      m = sqrtf(re * re + im * im);
      pv = e < H ? re : im;
      if (e < H) cubes += m * m * m;  // one modulus per complex coordinate
    } else {
      pv = sd.p0[rel * D + e];
      m = fabsf(pv);
      cubes += m * m * m;
    }
    sd.reg_pgrad[rel * D + e] = c3 * m * pv;
  }
  cubes = wave_sum(cubes);
  if (lane == 0) sd.reg_pcube[rel] = cubes;
}

// One workgroup per batch: reg_out[k] = coef * (sum over the positives' prepared rows
// of m^3 (written by rowback_kernel) + the parameter term), summed in a fixed order.
__global__ __launch_bounds__(256) void reg_reduce_kernel(StepCtx c) {
  __shared__ float sh[256];
  const int k = blockIdx.x, t = threadIdx.x;
  const int D = c.D, H = D / 2;
  float acc = 0.f;
  const float* rows = c.regrow + (int64_t)k * 2 * c.B;
  for (int i = t; i < 2 * c.B; i += 256) acc += rows[i];
  if (c.op != PBG_OP_NONE) {
    if (c.dynamic) {  // once per edge and direction (regularizers.py:73-76, model.py:755-758)
      for (int i = t; i < c.B; i += 256) {
        const int64_t r = clamp_index(c.rel[(int64_t)k * c.B + i], c.num_relations);
        acc += c.side[0].reg_pcube[r] + c.side[1].reg_pcube[r];
      }
    } else {  // once per chunk (regularizers.py:91-93)
      const SideCtx& sd = c.side[1];
      const int64_t r = clamp_index(c.rel[k], c.num_relations);
      const int count = c.op == PBG_OP_COMPLEX_DIAGONAL ? H : D;
      for (int e = t; e < count; e += 256) {
        float m;
        if (c.op == PBG_OP_COMPLEX_DIAGONAL) {
          const float re = sd.p0[r * H + e], im = sd.p1[r * H + e];
          m = sqrtf(re * re + im * im);
        } else {
          m = fabsf(sd.p0[r * D + e]);
        }
        acc += (float)c.C * m * m * m;
      }
    }
  }
  sh[t] = acc;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (t < w) sh[t] += sh[t + w];
    __syncthreads();
  }
  if (t == 0 && c.reg_out) c.reg_out[k] = c.reg_coef * sh[0];
}

// ---------------------------------------------------------------------------
// global embeddings (model.py:433-441,486-492): gradient and AsyncAdagrad step
// ---------------------------------------------------------------------------
// The gradient of a side's global embedding is the sum of the raw-row gradients
// of the side's gathered rows: gth[s, k, slice, :] = sum over the rows
// r = slice (mod slices) of side s in batch k of gr[k, r, :].  Half a wave per
// row, 128-bit loads; fixed order, no atomics.
constexpr int kGlobalHalves = 8;  // half-waves per workgroup
// `direct`: gradient row r of batch k is row k * rk + r (the fused route; its value array may already be sorted)
__global__ __launch_bounds__(kGlobalHalves * 32) void global_grad_kernel(StepCtx c, float* __restrict__ gth, int slices,
                                                                          int direct) {
  __shared__ float4 sh[kGlobalHalves][32];
  const int lane = threadIdx.x & 31, hw = threadIdx.x >> 5;
  const int k = blockIdx.x, s = blockIdx.y / slices, slice = blockIdx.y % slices;
  const int D = c.D;
  const int begin = c.side[s].slot_pos;
  const int end = s == 0 ? c.side[1].slot_pos : c.rk;  // a side's positives and uniform negatives are contiguous
  const bool vec = (D & 3) == 0;
  for (int c0 = 0; c0 < D; c0 += 128) {
    const int col = c0 + lane * 4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int r = begin + slice * kGlobalHalves + hw; r < end; r += slices * kGlobalHalves) {
      const int64_t slot = (int64_t)k * c.rk + r;
      const float* row = c.gr + (direct ? slot : (int64_t)c.vals[slot]) * D;  // (a uniform negative's row may be the GEMM's)
      if (vec) {
        if (col < D) {
          const float4 v = *reinterpret_cast<const float4*>(row + col);
          acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
      } else {
        if (col < D) acc.x += row[col];
        if (col + 1 < D) acc.y += row[col + 1];
        if (col + 2 < D) acc.z += row[col + 2];
        if (col + 3 < D) acc.w += row[col + 3];
      }
    }
    sh[hw][lane] = acc;
    __syncthreads();
    if (hw == 0) {
      float4 t = sh[0][lane];
#pragma unroll
      for (int h = 1; h < kGlobalHalves; ++h) {
        t.x += sh[h][lane].x; t.y += sh[h][lane].y; t.z += sh[h][lane].z; t.w += sh[h][lane].w;
      }
      float* out = gth + (((int64_t)s * c.K + k) * slices + slice) * D;
      if (col < D) out[col] = t.x;
      if (col + 1 < D) out[col + 1] = t.y;
      if (col + 2 < D) out[col + 2] = t.z;
      if (col + 3 < D) out[col + 3] = t.w;
    }
    __syncthreads();
  }
}

// AsyncAdagrad (async_adagrad.py:75-85) on the global embeddings, the K batches'
// gradients applied in order.  `shared`: both sides have one entity type and one
// vector, whose gradient is the sum of the two sides'.  One wave per element:
// lane j sums the partial sums of batches j, j + 64, ...; the steps then run in
// batch order on registers.
__global__ __launch_bounds__(kRowThreads) void global_update_kernel(StepCtx c, const float* __restrict__ gth, int slices,
                                                                    int shared, float* p_l, float* s_l, float* p_r,
                                                                    float* s_r, float lr) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (e >= c.D) return;
  const int D = c.D;
  float p[2] = {p_l[e], shared ? 0.f : p_r[e]};
  float st[2] = {s_l[e], shared ? 0.f : s_r[e]};
  for (int k0 = 0; k0 < c.K; k0 += kWave) {
    const int k = k0 + lane;
    float g[2] = {0.f, 0.f};
    if (k < c.K)
      for (int s = 0; s < 2; ++s)
        for (int sl = 0; sl < slices; ++sl) g[s] += gth[(((int64_t)s * c.K + k) * slices + sl) * D + e];
    if (shared) {
      g[0] += g[1];
      g[1] = 0.f;
    }
    const int count = c.K - k0 < kWave ? c.K - k0 : kWave;
    for (int j = 0; j < count; ++j) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        if (s == 1 && shared) continue;
        const float gj = __shfl(g[s], j, 64);
        st[s] += gj * gj;
        p[s] += -lr * (gj / (sqrtf(st[s]) + 1e-10f));
      }
    }
  }
  if (lane == 0) {
    p_l[e] = p[0];
    s_l[e] = st[0];
    if (!shared) {
      p_r[e] = p[1];
      s_r[e] = st[1];
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct Plan {
  StepCtx c;
  size_t bytes;
  // buffers that only the host-side orchestration touches
  float* dth[2];
  float max_norm;      // 0: rows are read as they are
  float* renorm_scale; // [K * rk]
  float* dth_t[2];   // `affine`: the translations' gradients, [K, pslices_t, D]
  int pslices_t[2];
  uint64_t* keys_b;
  uint32_t* vals_b;
  void* sort_temp;
  int64_t psize;  // floats of parameter gradient per batch
  int pslices[2]; // partial sums per batch of the element-wise parameter gradients
  bool fused;          // the chunk fits the LDS-resident kernel
  int* fused_rowid;    // ... and this is where fused_ids_kernel leaves its row ids [K*C, kFusedIds]
  FusedLayout fl;
  bool stream;         // the chunk's positives fit LDS and its negatives are streamed past them
  StreamPlan sp;
  // cos on the streaming route: the route's dot kernels score on a normalised copy of the tables (cos(a, b) is the
  // dot product of the normalised rows, model.py:185-212), and the update takes every summed gradient back
  // through the normalisation (CosBack)
  bool stream_cos;
  float* ynorm[2];  // the copy of the lhs / rhs table (one copy when the sides share a table)
  float* yinv[2];   // 1 / |row|
  // dynamic relations: (relation, batch) keys of the positives and their sort buffers
  uint64_t *rkeys_a, *rkeys_b;
  uint32_t *rvals_a, *rvals_b;
  void* rsort_temp;
  void* rel_start;  // first sorted position of every relation (`linear` only)
  int64_t* dyn_next;  // ... and at the same position where the relation's next run starts (-1: none) [K * B]
  float* dyn_grun;  // element-wise operators: the parameter gradient of every (relation, batch) run, at the run's first sorted position [K * B, D]
  int nvh;
  float* gth;   // partial sums of the global embeddings' gradients [2, K, gslices, D]
  int gslices;
};

int validate(const pbg_step_desc* d, bool training) {
  if (!d) return fail(PBG_ERR_INVALID, "step: null descriptor");
  if (d->dim <= 0 || d->dim > kMaxDim)
    return fail(PBG_ERR_UNSUPPORTED, "step: dim must be in [1, %d], got %d", kMaxDim, d->dim);
  if (d->num_workers < 1 || d->num_workers > 256) return fail(PBG_ERR_INVALID, "step: num_workers must be in [1, 256]");
  if (d->batch_size < 1) return fail(PBG_ERR_INVALID, "step: batch_size must be positive");
  if (d->num_batch_negs < 0 || d->num_uniform_negs < 0) return fail(PBG_ERR_INVALID, "step: negative negatives count");
  if (d->num_batch_negs == 0 && d->num_uniform_negs == 0 && !d->all_negs)
    return fail(PBG_ERR_INVALID, "step: num_batch_negs and num_uniform_negs cannot both be 0");
  if (d->all_negs && (d->num_lhs_rows > (1 << 24) || d->num_rhs_rows > (1 << 24) ||
                      (int64_t)d->batch_size * (d->num_lhs_rows > d->num_rhs_rows ? d->num_lhs_rows : d->num_rhs_rows) > ((int64_t)1 << 31)))
    return fail(PBG_ERR_UNSUPPORTED, "step: all_negs needs batch_size x entities of a type within 2^31 scores");
  if (d->op < PBG_OP_NONE || d->op > PBG_OP_AFFINE) return fail(PBG_ERR_INVALID, "step: unknown operator %d", d->op);
  if (d->comparator < PBG_CMP_DOT || d->comparator > PBG_CMP_SQUARED_L2) return fail(PBG_ERR_INVALID, "step: unknown comparator %d", d->comparator);
  if (d->loss < PBG_LOSS_RANKING || d->loss > PBG_LOSS_SOFTMAX) return fail(PBG_ERR_INVALID, "step: unknown loss %d", d->loss);
  if (d->op == PBG_OP_COMPLEX_DIAGONAL && d->dim % 2 != 0)
    return fail(PBG_ERR_INVALID,
                "Need even dimension as 1st half is real and 2nd half is imaginary coordinates");  // operators.py:132-136
  if (d->num_relations < 1) return fail(PBG_ERR_INVALID, "step: num_relations must be positive");
  if (d->regularization_coef != 0.f && (d->op == PBG_OP_LINEAR || d->op == PBG_OP_AFFINE))
    return fail(PBG_ERR_UNSUPPORTED, "Regularizer not implemented for this operator");  // operators.py:40,188
  if (d->num_lhs_rows < 1 || d->num_rhs_rows < 1) return fail(PBG_ERR_INVALID, "step: empty table");
  if (d->bias) {
    if (d->dim < 2) return fail(PBG_ERR_INVALID, "step: bias needs at least two coordinates");
  }
  if (d->half_precision) {
    // The distance comparators clamp at 1e-30 before the square root (model.py:244), which is 0 as a
    // float16: every batch negative that is its own positive's row then has a NaN gradient in the
    // reference; bias and the regularizer would do their sums in float16.
    if (d->comparator == PBG_CMP_L2 || d->comparator == PBG_CMP_SQUARED_L2)
      return fail(PBG_ERR_UNSUPPORTED, "step: half_precision is built for the dot and cos comparators");
    if (d->bias || d->regularization_coef != 0.f)
      return fail(PBG_ERR_UNSUPPORTED, "step: half_precision is not built with bias or a regularizer");
  }
  return PBG_OK;
}

// Carves the workspace.  With base == nullptr only the size is computed.
int make_plan(const pbg_step_desc* d, const pbg_step_buffers* b, Plan* plan) {
  StepCtx& c = plan->c;
  memset(plan, 0, sizeof(*plan));
  char* base = b ? (char*)b->workspace : nullptr;
  size_t off = 0;
  auto take = [&](size_t count, size_t elem) -> void* {
    const size_t o = off;
    off += align_up(count * elem, 256);
    return base ? (void*)(base + o) : nullptr;
  };
  auto takef = [&](size_t count) -> float* { return (float*)take(count, sizeof(float)); };

  c.D = d->dim;
  c.K = d->num_workers;
  c.B = d->batch_size;
  c.U = d->num_uniform_negs;
  // all_negs (model.py:648-650,582-618): one chunk of all the positives, every entity of a side's type as negative
  const bool all_negs = d->all_negs != 0;
  const bool batch_mode = d->num_batch_negs > 0 && !all_negs;
  c.P = batch_mode ? (d->num_batch_negs < c.B ? d->num_batch_negs : c.B) : (c.U < c.B ? c.U : c.B);
  if (all_negs) c.P = c.B;
  c.C = (c.B - 1) / c.P + 1;
  c.last = c.B - (c.C - 1) * c.P;
  c.dynamic = d->dynamic;
  c.op = d->op == PBG_OP_AFFINE ? PBG_OP_LINEAR : d->op;
  c.affine = d->op == PBG_OP_AFFINE;
  c.bias = d->bias != 0;
  c.half = d->half_precision != 0;
  c.cmp = d->comparator;
  c.loss = d->loss;
  c.margin = d->margin;
  c.num_relations = d->num_relations;
  const int D = c.D, K = c.K, C = c.C, P = c.P;
  const int64_t KC = (int64_t)K * C;
  const bool need_aux = c.cmp != PBG_CMP_DOT;

  int slot = 0;
  for (int s = 0; s < 2; ++s) {
    SideCtx& sd = c.side[s];
    const bool enabled = s == 0 ? !d->disable_lhs_negs : !d->disable_rhs_negs;
    sd.nb = (enabled && batch_mode) ? P : 0;
    sd.num_rows = s == 0 ? d->num_lhs_rows : d->num_rhs_rows;
    sd.all = all_negs;
    sd.u = enabled ? (all_negs ? (int)sd.num_rows : c.U) : 0;
    sd.nn = sd.nb + sd.u;
    sd.alias = sd.nb > 0;
    sd.stride_p = sd.alias ? sd.nn : P;
    sd.key_base = (s == 1 && !d->shared_table) ? d->num_lhs_rows : 0;
    sd.slot_pos = slot;
    slot += c.B;
    sd.slot_uni = slot;
    slot += C * sd.u;
    if (c.dynamic) {
      sd.has_op = 1;
      sd.op_uniform = 0;
    } else {
      sd.has_op = (s == 1 && c.op != PBG_OP_NONE) ? 1 : 0;
      sd.op_uniform = sd.has_op;
    }
    sd.op_rows = sd.has_op ? c.B + (sd.op_uniform ? C * sd.u : 0) : 0;
  }
  c.rk = slot;
  c.kbits = bits_for((uint64_t)(K - 1));

  // gradient rows, and behind them (so that one 32-bit row number reaches both) the negatives' gradient
  // matrices of the sides whose uniform rows need no work after the GEMM
  const int64_t npairs = (int64_t)K * c.rk;
  int64_t block_rows = npairs;
  for (int s = 0; s < 2; ++s) {
    SideCtx& sd = c.side[s];
    sd.uni_direct = sd.u > 0 && c.cmp == PBG_CMP_DOT && !sd.op_uniform && !c.bias &&
                    block_rows + KC * sd.nn < ((int64_t)1 << 32);
    sd.uni_dz_direct = sd.u > 0 && c.cmp == PBG_CMP_DOT && sd.op_uniform && !c.bias && c.op != PBG_OP_LINEAR;
    if (sd.uni_direct) {
      sd.uni_row0 = block_rows;
      block_rows += KC * sd.nn;
    }
  }
  c.gr = takef((size_t)block_rows * D);

  for (int s = 0; s < 2; ++s) {
    SideCtx& sd = c.side[s];
    const SideCtx& so = c.side[1 - s];
    // prepared operands and their gradients
    if (sd.nn > 0) {
      sd.xn = takef(KC * sd.nn * D);
      sd.dxn = sd.uni_direct ? (c.gr ? c.gr + sd.uni_row0 * D : nullptr) : takef(KC * sd.nn * D);
      if (need_aux) sd.an = takef(KC * sd.nn);
      sd.s = takef(KC * P * sd.nn);
      if (is_distance(c.cmp)) sd.rs = takef(KC * P);
      if (c.bias) {
        sd.bn = takef(KC * sd.nn);
        sd.bs = takef(KC * P);
        if (c.cmp == PBG_CMP_L2) sd.gs = takef(KC * P * sd.nn);
      }
    }
    if (sd.alias) {
      sd.xp = sd.xn;
      sd.dxp = sd.dxn;
      sd.ap = sd.an;
      sd.bp = sd.bn;
    } else {
      sd.xp = takef(KC * P * D);
      sd.dxp = takef(KC * P * D);
      if (need_aux) sd.ap = takef(KC * P);
      if (c.bias) sd.bp = takef(KC * P);
    }
    if (c.dynamic) {
      sd.xa = takef(KC * P * D);
      sd.dxa = takef(KC * P * D);
      if (need_aux) sd.aa = takef(KC * P);
      if (c.bias) sd.ba = takef(KC * P);
    }
    // which gradient buffers a GEMM fills (see run_backward)
    sd.plain_written = sd.alias || (!c.dynamic && (s == 0 ? (d->disable_rhs_negs == 0) : (d->disable_lhs_negs == 0)));
    sd.opd_written = c.dynamic && (s == 0 ? (d->disable_rhs_negs == 0) : (d->disable_lhs_negs == 0));
    (void)so;
    if (sd.has_op && c.op != PBG_OP_NONE) {
      sd.dz = takef((size_t)K * sd.op_rows * D);
      if (c.op == PBG_OP_LINEAR) {
        sd.xraw = takef((size_t)K * sd.op_rows * D);
        sd.z = takef((size_t)K * sd.op_rows * D);
      }
    }
  }
  const int64_t CP = (int64_t)C * P;
  c.pos[0] = takef(K * CP);
  c.dpos[0] = takef(K * CP);
  if (c.dynamic) {
    c.pos[1] = takef(K * CP);
    c.dpos[1] = takef(K * CP);
  } else {
    c.pos[1] = c.pos[0];
    c.dpos[1] = c.dpos[0];
  }
  c.lossrow = takef(K * CP);
  c.violrow = (int*)take(K * CP * 2, sizeof(int));
  if (!c.dynamic) {  // room for the global embeddings' gradient (whether a call uses it is in its buffers)
    int sl = (int)ceil_div(c.rk, 2 * 16 * kGlobalHalves);  // about 16 rows per half-wave
    plan->gslices = sl < 1 ? 1 : (sl > 16 ? 16 : sl);
    plan->gth = takef((size_t)2 * K * plan->gslices * D);
  }
  c.reg_coef = d->regularization_coef;
  if (c.reg_coef != 0.f) {
    c.regrow = takef((size_t)K * 2 * c.B);
    if (c.dynamic && c.op != PBG_OP_NONE)
      for (int s = 0; s < 2; ++s) {
        c.side[s].reg_pgrad = takef((size_t)c.num_relations * D);
        c.side[s].reg_pcube = takef((size_t)c.num_relations);
      }
  }

  plan->psize = 0;
  if (c.op == PBG_OP_LINEAR) plan->psize = (int64_t)D * D;
  else if (c.op != PBG_OP_NONE) plan->psize = D;
  if (c.dynamic && plan->psize > 0) {
    const int64_t ne = (int64_t)K * c.B;
    plan->rkeys_a = (uint64_t*)take(ne, 8);
    plan->rkeys_b = (uint64_t*)take(ne, 8);
    plan->rvals_a = (uint32_t*)take(ne, 4);
    plan->rvals_b = (uint32_t*)take(ne, 4);
    plan->rsort_temp = take(sort_temp_bytes(ne), 1);
    if (c.op == PBG_OP_LINEAR) plan->rel_start = take(seg_linear_update_temp_bytes(c.num_relations, ne, D, K), 1);
    if (c.op != PBG_OP_LINEAR || c.affine) {
      plan->dyn_grun = takef((size_t)ne * D);
      plan->dyn_next = (int64_t*)take(ne, 8);
    }
  }
  for (int s = 0; s < 2; ++s) {
    plan->pslices[s] = 1;
    if (!c.side[s].has_op || plan->psize == 0 || c.dynamic) continue;
    if (c.op != PBG_OP_LINEAR) {
      int sl = (int)ceil_div(c.side[s].op_rows, 32 * kParamGroups);
      plan->pslices[s] = sl < 1 ? 1 : (sl > 16 ? 16 : sl);
    }
    plan->dth[s] = takef((size_t)K * plan->pslices[s] * plan->psize);
    if (c.affine) {
      int sl = (int)ceil_div(c.side[s].op_rows, 32 * kParamGroups);
      plan->pslices_t[s] = sl < 1 ? 1 : (sl > 16 ? 16 : sl);
      plan->dth_t[s] = takef((size_t)K * plan->pslices_t[s] * D);
    }
  }

  plan->max_norm = d->max_norm > 0.f ? d->max_norm : 0.f;
  if (plan->max_norm > 0.f) plan->renorm_scale = takef((size_t)npairs);
  c.keys = (uint64_t*)take(npairs, 8);
  plan->keys_b = (uint64_t*)take(npairs, 8);
  c.vals = (uint32_t*)take(npairs, 4);
  plan->vals_b = (uint32_t*)take(npairs, 4);
  plan->sort_temp = take(sort_temp_bytes(npairs), 1);
  plan->nvh = (int)ceil_div((D + 1) / 2, kWave);
  // (the regularizer's terms live in the staged kernels only)
  // (half_precision: the fused and the staged route, whose products then run on the fp16 matrix instructions)
  plan->fused = fused_layout(c, &plan->fl) && c.reg_coef == 0.f && !c.bias && getenv("PBG_DISABLE_FUSED") == nullptr;
  if (plan->fused) {  // the fused kernel writes every gradient row and every dz itself
    c.side[0].uni_direct = c.side[1].uni_direct = 0;
    c.side[0].uni_dz_direct = c.side[1].uni_dz_direct = 0;
    plan->fused_rowid = (int*)take((size_t)KC * kFusedIds, sizeof(int));
  }
  // The streaming route's own buffers lie behind the staged ones: a call with global
  // embeddings (known only from its buffers) takes the staged route on the same workspace.
  // cos takes it as dot on a normalised copy of the tables: without an operator (prepare follows the operator,
  // model.py:478-506, and a normalised copy per relation is not kept), when the copy is modest (2 GiB) and has no more
  // rows than the call gathers anyway
  StepCtx as_dot = c;
  bool cos_copy = false;
  {
    const int64_t table_rows = d->num_lhs_rows + (d->shared_table ? 0 : d->num_rhs_rows);
    if (c.cmp == PBG_CMP_COS && c.op == PBG_OP_NONE && c.reg_coef == 0.f && !c.bias && D % 4 == 0 &&
        table_rows <= (int64_t)npairs && (size_t)table_rows * D * sizeof(float) <= ((size_t)2 << 30)) {
      as_dot.cmp = PBG_CMP_DOT;
      cos_copy = true;
    }
  }
  plan->stream = !plan->fused && !c.half && stream_geometry(as_dot, &plan->sp) && getenv("PBG_DISABLE_STREAM") == nullptr;
  plan->stream_cos = plan->stream && cos_copy;
  plan->ynorm[0] = plan->ynorm[1] = plan->yinv[0] = plan->yinv[1] = nullptr;
  if (plan->stream_cos) {
    plan->ynorm[0] = takef((size_t)d->num_lhs_rows * D);
    plan->yinv[0] = takef((size_t)d->num_lhs_rows);
    if (!d->shared_table) {
      plan->ynorm[1] = takef((size_t)d->num_rhs_rows * D);
      plan->yinv[1] = takef((size_t)d->num_rhs_rows);
    }
  }
  if (plan->stream) {
    StreamPlan& sp = plan->sp;
    const size_t ne = (size_t)K * c.B;
    for (int s = 0; s < 2; ++s) {
      sp.sa[s] = takef(ne * D);
      sp.sdb[s] = takef(ne * D);
      sp.spos[s] = takef(ne);
      sp.sloss[s] = takef((size_t)K * CP);
      sp.colid[s] = (int*)take((size_t)KC * (c.P + c.side[s].u), sizeof(int));
      // dynamic relations: the operand's gradient IS the operator-output gradient of the side the operand came from
      float* dz = c.side[1 - s].dz;
      sp.sda[s] = (c.dynamic && c.op != PBG_OP_NONE) ? dz : takef(ne * D);
    }
    sp.scratch = takef(stream_scratch_floats(sp));
  }
  plan->bytes = off;

  if (b) {
    c.side[0].w = b->w_lhs;
    c.side[1].w = b->w_rhs;
    c.side[0].idx = b->lhs;
    c.side[1].idx = b->rhs;
    c.side[0].uidx = b->uniform_lhs;
    c.side[1].uidx = b->uniform_rhs;
    c.side[0].useed = c.side[1].useed = b->uniform_seed;
    c.side[0].glob = b->lhs_global;
    c.side[1].glob = b->rhs_global;
    c.side[0].p0 = b->lhs_op_p0;
    c.side[0].p1 = b->lhs_op_p1;
    c.side[1].p0 = b->rhs_op_p0;
    c.side[1].p1 = b->rhs_op_p1;
    c.rel = b->rel;
    c.edge_weight = b->edge_weight;
    c.rel_weights = b->relation_weights;
    c.violators = (unsigned long long*)b->violators_out;
    c.loss_out = b->loss_out;
    c.reg_out = b->reg_out;
  }
  return PBG_OK;
}

int check_buffers(const pbg_step_desc* d, const pbg_step_buffers* b, const Plan& plan, bool training) {
  if (!b) return fail(PBG_ERR_INVALID, "step: null buffers");
  if (!b->w_lhs || !b->w_rhs || !b->lhs || !b->rhs || !b->rel || !b->relation_weights)
    return fail(PBG_ERR_INVALID, "step: null table / edge / relation pointer");
  if (training && (!b->g_lhs || !b->g_rhs || !b->loss_out || !b->violators_out))
    return fail(PBG_ERR_INVALID, "step: null optimizer state or statistics pointer");
  if (d->shared_table && (b->w_lhs != b->w_rhs || d->num_lhs_rows != d->num_rhs_rows))
    return fail(PBG_ERR_INVALID, "step: shared_table needs w_lhs == w_rhs");
  if (!d->shared_table && b->w_lhs == b->w_rhs)
    return fail(PBG_ERR_INVALID, "step: w_lhs == w_rhs needs shared_table = 1");
  if ((uintptr_t)b->w_lhs % 16 != 0 || (uintptr_t)b->w_rhs % 16 != 0)
    return fail(PBG_ERR_INVALID, "step: tables must be 16-byte aligned");
  if (d->all_negs) {
    // the negatives are the tables' rows in order: nothing to pass and nothing to draw
  } else if (!b->sample_uniform) {
    if (plan.c.side[0].u > 0 && !b->uniform_lhs) return fail(PBG_ERR_INVALID, "step: uniform_lhs is null");
    if (plan.c.side[1].u > 0 && !b->uniform_rhs) return fail(PBG_ERR_INVALID, "step: uniform_rhs is null");
  } else if (b->uniform_lhs || b->uniform_rhs) {
    return fail(PBG_ERR_INVALID, "step: sample_uniform is set but uniform negatives were passed");
  }
  for (int s = 0; s < 2; ++s) {
    if (!plan.c.side[s].has_op || d->op == PBG_OP_NONE) continue;
    const float* p0 = s == 0 ? b->lhs_op_p0 : b->rhs_op_p0;
    const float* p1 = s == 0 ? b->lhs_op_p1 : b->rhs_op_p1;
    const float* s0 = s == 0 ? b->lhs_op_s0 : b->rhs_op_s0;
    const float* s1 = s == 0 ? b->lhs_op_s1 : b->rhs_op_s1;
    const bool two = d->op == PBG_OP_COMPLEX_DIAGONAL || d->op == PBG_OP_AFFINE;
    if (!p0 || (two && !p1)) return fail(PBG_ERR_INVALID, "step: null operator parameter");
    if (training && (!s0 || (two && !s1))) return fail(PBG_ERR_INVALID, "step: null operator optimizer state");
  }
  if ((b->lhs_global == nullptr) != (b->rhs_global == nullptr))
    return fail(PBG_ERR_INVALID, "step: global embeddings need both sides' vectors (the same pointer for one entity type)");
  if (b->lhs_global) {
    if (d->dynamic) return fail(PBG_ERR_INVALID, "Cannot have global embs with dynamic rels");  // model.py:488-489
    if ((uintptr_t)b->lhs_global % 16 != 0 || (uintptr_t)b->rhs_global % 16 != 0)
      return fail(PBG_ERR_INVALID, "step: global embeddings must be 16-byte aligned");
    if (training && (!b->lhs_global_sum || !b->rhs_global_sum))
      return fail(PBG_ERR_INVALID, "step: null optimizer state of the global embeddings");
    if (training && (b->lhs_global == b->rhs_global) != (b->lhs_global_sum == b->rhs_global_sum))
      return fail(PBG_ERR_INVALID, "step: one global embedding needs one optimizer state");
  }
  if (!b->workspace || b->workspace_bytes < plan.bytes)
    return fail(PBG_ERR_WORKSPACE, "step: workspace needs %zu bytes, got %zu", plan.bytes, b->workspace_bytes);
  if ((uintptr_t)b->workspace % 256 != 0) return fail(PBG_ERR_WORKSPACE, "step: workspace must be 256-byte aligned");
  const uint64_t rows = (uint64_t)d->num_lhs_rows + (d->shared_table ? 0 : (uint64_t)d->num_rhs_rows);
  if (bits_for(rows) + plan.c.kbits > 62) return fail(PBG_ERR_UNSUPPORTED, "step: tables too large for the sort key");
  if ((int64_t)plan.c.K * plan.c.rk >= ((int64_t)1 << 32))
    return fail(PBG_ERR_UNSUPPORTED, "step: too many gradient rows per call");
  return PBG_OK;
}

#define PBG_DISPATCH_NVH(nvh, KERNEL, grid, stream, ...)                                                      \
  do {                                                                                                       \
    if ((nvh) <= 1) hipLaunchKernelGGL((KERNEL<1>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);          \
    else if ((nvh) <= 2) hipLaunchKernelGGL((KERNEL<2>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);     \
    else if ((nvh) <= 4) hipLaunchKernelGGL((KERNEL<4>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);     \
    else if ((nvh) <= 8) hipLaunchKernelGGL((KERNEL<8>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);     \
    else if ((nvh) <= 16) hipLaunchKernelGGL((KERNEL<16>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);   \
    else hipLaunchKernelGGL((KERNEL<32>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);                    \
  } while (0)

dim3 wave_grid(int64_t jobs) { return dim3((unsigned)ceil_div(jobs > 0 ? jobs : 1, kWavesPerBlock)); }

// comparator.prepare of the cos comparator on every row of a table (model.py:187-192): out[r] = table[r] * (1 / |table[r]|),
// inv[r] = 1 / |table[r]|.  One wave per row.  (A zero row gives NaN, as it does in the reference.)
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void normalize_rows_kernel(const float* __restrict__ table, int64_t num_rows, int D,
                                                                     float* __restrict__ out, float* __restrict__ inv) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (r >= num_rows) return;
  const int H = (D + 1) / 2;
  RowV<NVH> x = row_load<NVH>(table + r * D, D, H, lane);
  const float rn = prepare_row<NVH>(PBG_CMP_COS, x);
  row_store<NVH>(out + r * D, x, D, H, lane);
  if (lane == 0) inv[r] = rn;
}

int run_renorm(const Plan& plan, const pbg_step_buffers* b, hipStream_t stream) {
  if (plan.max_norm <= 0.f) return PBG_OK;
  const StepCtx& c = plan.c;
  const dim3 grid = wave_grid((int64_t)c.K * c.rk);
  PBG_DISPATCH_NVH(plan.nvh, renorm_scan_kernel, grid, stream, c, plan.max_norm, plan.renorm_scale);
  PBG_DISPATCH_NVH(plan.nvh, renorm_apply_kernel, grid, stream, c, plan.renorm_scale, b->w_lhs,
                   b->w_rhs ? b->w_rhs : b->w_lhs);
  return check_launch("step max_norm");
}

int run_prep(const Plan& plan, hipStream_t stream) {
  const StepCtx& c = plan.c;
  const int64_t jobs = (int64_t)c.K * (2 * c.C * c.P + c.C * c.side[0].u + c.C * c.side[1].u);
  PBG_DISPATCH_NVH(plan.nvh, prep_kernel, wave_grid(jobs), stream, c);
  return check_launch("step prep");
}

// Dynamic relations: the call's edges ordered by (relation, batch).  Built once
// per call, by the first stage that needs it.
struct RelOrder {
  uint64_t* keys = nullptr;
  uint32_t* vals = nullptr;
};

int ensure_rel_order(const Plan& plan, hipStream_t stream, RelOrder* ro) {
  if (ro->keys) return PBG_OK;
  const StepCtx& c = plan.c;
  const int64_t ne = (int64_t)c.K * c.B;
  hipLaunchKernelGGL(rel_keys_kernel, dim3((unsigned)ceil_div(ne, 256)), dim3(256), 0, stream, c, plan.rkeys_a,
                     plan.rvals_a);
  // the edges arrive in batch order, so sorting on the relation bits orders by (relation, batch)
  return sort_pairs(plan.rkeys_a, plan.rvals_a, plan.rkeys_b, plan.rvals_b, ne, c.kbits,
                    bits_for((uint64_t)(c.num_relations - 1)) + c.kbits, plan.rsort_temp, stream, &ro->keys, &ro->vals);
}

// the `linear` operator: one GEMM per side that has it, then comparator.prepare
int run_operator_forward(const Plan& plan, hipStream_t stream, RelOrder* ro) {
  const StepCtx& c = plan.c;
  const int D = c.D, K = c.K;
  int rc;
  if (c.op == PBG_OP_LINEAR && c.dynamic) {
    if ((rc = ensure_rel_order(plan, stream, ro)) != PBG_OK) return rc;
    const int64_t ne = (int64_t)K * c.B;
    for (int s = 0; s < 2; ++s) {
      const SideCtx& sd = c.side[s];  // z_e = W[rel_e] x_e (operators.py:259-269)
      if ((rc = seg_linear_apply(ro->keys, ro->vals, ne, c.kbits, c.B, sd.xraw, sd.op_rows, sd.p0, D, false, sd.z,
                                 sd.op_rows, false, stream)) != PBG_OK)
        return rc;
      PBG_DISPATCH_NVH(plan.nvh, prepare_staged_kernel, wave_grid(ne), stream, c, s);
    }
    return check_launch("step operator");
  }
  if (c.op == PBG_OP_LINEAR) {
    for (int s = 0; s < 2; ++s) {
      const SideCtx& sd = c.side[s];
      if (!sd.has_op) continue;
      GemmArgs g{};  // z[k] = xraw[k] * W[rel[k]]^T   (operators.py:94-99)
      g.a = sd.xraw; g.stride_a = (int64_t)sd.op_rows * D; g.lda = D; g.a_kmajor = 0;
      g.b = sd.p0; g.stride_b = 0; g.ldb = D; g.b_kmajor = 0;
      g.b_index = c.rel; g.b_index_stride = (int64_t)D * D;
      g.c = sd.z; g.stride_c = (int64_t)sd.op_rows * D; g.ldc = D;
      g.m = sd.op_rows; g.n = D; g.k = D; g.batch = K; g.alpha = 1.f; g.beta = 0.f;
      if ((rc = gemm_f32(g, stream)) != PBG_OK) return rc;
      PBG_DISPATCH_NVH(plan.nvh, prepare_staged_kernel, wave_grid((int64_t)K * sd.op_rows), stream, c, s);
    }
  }
  return check_launch("step operator");
}

// score GEMMs
int run_scores(const Plan& plan, hipStream_t stream) {
  const StepCtx& c = plan.c;
  const int D = c.D, K = c.K, C = c.C, P = c.P;
  int rc;
  for (int s = 0; s < 2; ++s) {
    const SideCtx& sd = c.side[s];
    const SideCtx& so = c.side[1 - s];
    if (sd.nn == 0) continue;
    GemmArgs g{};  // S = A * N^T   (model.py:179-180, 234)
    g.a = c.dynamic ? so.xa : so.xp;
    g.stride_a = (int64_t)(c.dynamic ? P : so.stride_p) * D; g.lda = D; g.a_kmajor = 0;
    g.b = sd.xn; g.stride_b = (int64_t)sd.nn * D; g.ldb = D; g.b_kmajor = 0;
    g.c = sd.s; g.stride_c = (int64_t)P * sd.nn; g.ldc = sd.nn;
    g.m = P; g.n = sd.nn; g.k = D; g.batch = K * C; g.alpha = 1.f; g.beta = 0.f;
    g.half = c.half;
    if ((rc = gemm_f32(g, stream)) != PBG_OK) return rc;
  }
  return check_launch("step forward");
}

int run_backward_dn(const Plan& plan, hipStream_t stream) {
  const StepCtx& c = plan.c;
  const int D = c.D, K = c.K, C = c.C, P = c.P;
  int rc;
  for (int s = 0; s < 2; ++s) {  // dN = dS^T * A  -> dxn (all nn rows, first writer)
    const SideCtx& sd = c.side[s];
    const SideCtx& so = c.side[1 - s];
    if (sd.nn == 0) continue;
    GemmArgs g{};
    g.a = sd.s; g.stride_a = (int64_t)P * sd.nn; g.lda = sd.nn; g.a_kmajor = 1;  // A(m = col, k = row)
    g.b = c.dynamic ? so.xa : so.xp;
    g.stride_b = (int64_t)(c.dynamic ? P : so.stride_p) * D; g.ldb = D; g.b_kmajor = 1;
    g.c = sd.dxn; g.stride_c = (int64_t)sd.nn * D; g.ldc = D;
    g.m = sd.nn; g.n = D; g.k = P; g.batch = K * C; g.alpha = 1.f; g.beta = 0.f;
    g.half = c.half;
    if ((rc = gemm_f32(g, stream)) != PBG_OK) return rc;
  }
  return check_launch("step backward dN");
}

int run_backward_da(const Plan& plan, hipStream_t stream) {
  const StepCtx& c = plan.c;
  const int D = c.D, K = c.K, C = c.C, P = c.P;
  int rc;
  for (int s = 0; s < 2; ++s) {  // dA = dS * N -> the other side's positives (operated ones in dynamic mode)
    const SideCtx& sd = c.side[s];
    const SideCtx& so = c.side[1 - s];
    if (sd.nn == 0) continue;
    GemmArgs g{};
    g.a = sd.s; g.stride_a = (int64_t)P * sd.nn; g.lda = sd.nn; g.a_kmajor = 0;
    g.b = sd.xn; g.stride_b = (int64_t)sd.nn * D; g.ldb = D; g.b_kmajor = 1;
    if (c.dynamic) {
      g.c = so.dxa; g.stride_c = (int64_t)P * D; g.beta = 0.f;
    } else {
      g.c = so.dxp; g.stride_c = (int64_t)so.stride_p * D; g.beta = so.alias ? 1.f : 0.f;
    }
    g.ldc = D;
    g.m = P; g.n = D; g.k = sd.nn; g.batch = K * C; g.alpha = 1.f;
    g.half = c.half;
    if ((rc = gemm_f32(g, stream)) != PBG_OK) return rc;
  }
  return check_launch("step backward");
}

int run_rowback(const Plan& plan, hipStream_t stream) {
  const StepCtx& c = plan.c;
  const int64_t jobs = (int64_t)c.K * (2 * c.B + c.C * c.side[0].u + c.C * c.side[1].u);
  PBG_DISPATCH_NVH(plan.nvh, rowback_kernel, wave_grid(jobs), stream, c);
  return check_launch("step rowback");
}

// `edge_terms`: (streaming route, standard mode) dz holds every edge's term of the parameter
// gradient itself, so the gradient is a column sum
int run_params(const pbg_step_desc* d, const pbg_step_buffers* b, const Plan& plan, hipStream_t stream,
               RelOrder* ro, bool edge_terms) {
  const StepCtx& c = plan.c;
  if (c.op == PBG_OP_NONE) return PBG_OK;
  const int D = c.D, K = c.K;
  int rc;
  if (c.dynamic) {
    const int64_t ne = (int64_t)K * c.B;
    if ((rc = ensure_rel_order(plan, stream, ro)) != PBG_OK) return rc;
    uint64_t* rkeys = ro->keys;
    uint32_t* rvals = ro->vals;
    for (int s = 0; s < 2; ++s) {
      const SideCtx& sd = c.side[s];
      float* p0 = s == 0 ? b->lhs_op_p0 : b->rhs_op_p0;
      float* p1 = s == 0 ? b->lhs_op_p1 : b->rhs_op_p1;
      float* s0 = s == 0 ? b->lhs_op_s0 : b->rhs_op_s0;
      float* s1 = s == 0 ? b->lhs_op_s1 : b->rhs_op_s1;
      if (c.op == PBG_OP_LINEAR) {
        // gr[row of e] += W[rel_e]^T dz_e, then the relation matrices' own step
        if ((rc = seg_linear_apply(rkeys, rvals, ne, c.kbits, c.B, sd.dz, sd.op_rows, sd.p0, D, true,
                                   c.gr + (int64_t)sd.slot_pos * D, c.rk, true, stream)) != PBG_OK)
          return rc;
        if ((rc = seg_linear_update(rkeys, rvals, ne, c.kbits, c.K, sd.dz, sd.xraw, D, c.num_relations, p0, s0,
                                    d->relation_lr, plan.rel_start, stream)) != PBG_OK)
          return rc;
        if (c.affine) {  // the translations: the element-wise kernel on dz, parameters in the second slot
          StepCtx ct = c;
          ct.op = PBG_OP_TRANSLATION;
          launch_dyn_params(ct, s, ne, rkeys, rvals, plan.dyn_grun, plan.dyn_next, p1, nullptr, s1, nullptr, d->relation_lr, stream);
        }
      } else {
        launch_dyn_params(c, s, ne, rkeys, rvals, plan.dyn_grun, plan.dyn_next, p0, p1, s0, s1, d->relation_lr, stream);
      }
    }
    return check_launch("step params (dynamic)");
  }
  for (int s = 0; s < 2; ++s) {
    const SideCtx& sd = c.side[s];
    if (!sd.has_op) continue;
    float* p0 = s == 0 ? b->lhs_op_p0 : b->rhs_op_p0;
    float* p1 = s == 0 ? b->lhs_op_p1 : b->rhs_op_p1;
    float* s0 = s == 0 ? b->lhs_op_s0 : b->rhs_op_s0;
    float* s1 = s == 0 ? b->lhs_op_s1 : b->rhs_op_s1;
    if (c.op == PBG_OP_LINEAR) {
      GemmArgs g{};  // dx = dz * W  -> gradient rows of this side (positives, then uniform negatives)
      g.a = sd.dz; g.stride_a = (int64_t)sd.op_rows * D; g.lda = D; g.a_kmajor = 0;
      g.b = sd.p0; g.stride_b = 0; g.ldb = D; g.b_kmajor = 1;
      g.b_index = c.rel; g.b_index_stride = (int64_t)D * D;
      g.c = c.gr + (int64_t)sd.slot_pos * D; g.stride_c = (int64_t)c.rk * D; g.ldc = D;
      g.m = sd.op_rows; g.n = D; g.k = D; g.batch = K; g.alpha = 1.f; g.beta = 0.f;
      if ((rc = gemm_f32(g, stream)) != PBG_OK) return rc;
      GemmArgs h{};  // dW = dz^T * x
      h.a = sd.dz; h.stride_a = (int64_t)sd.op_rows * D; h.lda = D; h.a_kmajor = 1;
      h.b = sd.xraw; h.stride_b = (int64_t)sd.op_rows * D; h.ldb = D; h.b_kmajor = 1;
      h.c = plan.dth[s]; h.stride_c = (int64_t)D * D; h.ldc = D;
      h.m = D; h.n = D; h.k = sd.op_rows; h.batch = K; h.alpha = 1.f; h.beta = 0.f;
      if ((rc = gemm_f32(h, stream)) != PBG_OK) return rc;
    } else {
      StepCtx cg = c;
      if (edge_terms) cg.op = PBG_OP_TRANSLATION;  // (whose gradient is the column sum of dz)
      launch_param_grad(cg, s, plan.dth[s], plan.pslices[s], c.op, stream);
    }
    if (c.affine) {  // the translation: column sums of dz, then its own Adagrad steps (parameters in the second slot)
      StepCtx ct = c;
      ct.op = PBG_OP_TRANSLATION;
      const int sl = plan.pslices_t[s];
      launch_param_grad(ct, s, plan.dth_t[s], sl, PBG_OP_TRANSLATION, stream);
      if (K <= kWave) {
        hipLaunchKernelGGL(param_update_wave_kernel, dim3((unsigned)ceil_div(D, kWavesPerBlock)), dim3(kRowThreads), 0,
                           stream, ct, s, plan.dth_t[s], sl, (int64_t)D, p1, nullptr, s1, nullptr, d->relation_lr);
      } else {
        hipLaunchKernelGGL(param_update_kernel, dim3((unsigned)ceil_div(D, 256)), dim3(256), 0, stream, ct, s,
                           plan.dth_t[s], sl, (int64_t)D, p1, nullptr, s1, nullptr, d->relation_lr);
      }
    }
    if (K <= kWave && c.op != PBG_OP_LINEAR) {  // (a matrix's elements are better served one per thread)
      hipLaunchKernelGGL(param_update_wave_kernel, dim3((unsigned)ceil_div(plan.psize, kWavesPerBlock)), dim3(kRowThreads),
                         0, stream, c, s, plan.dth[s], plan.pslices[s], plan.psize, p0, p1, s0, s1, d->relation_lr);
    } else {
      hipLaunchKernelGGL(param_update_kernel, dim3((unsigned)ceil_div(plan.psize, 256)), dim3(256), 0, stream, c, s,
                         plan.dth[s], plan.pslices[s], plan.psize, p0, p1, s0, s1, d->relation_lr);
    }
  }
  return check_launch("step params");
}

}  // namespace
}  // namespace pbg

using namespace pbg;

namespace {
__global__ void sample_uniform_kernel(uint64_t seed, uint32_t side, int64_t num_rows, int64_t count,
                                      int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) out[i] = sampled_row(seed, (uint64_t)i, side, num_rows);
}
}  // namespace

extern "C" size_t pbg_sizeof_step_desc(void) { return sizeof(pbg_step_desc); }
extern "C" size_t pbg_sizeof_step_buffers(void) { return sizeof(pbg_step_buffers); }

extern "C" int pbg_sample_uniform_negatives(uint64_t seed, int32_t side, int64_t num_rows, int64_t count, int64_t* out,
                                            pbg_stream_t stream) {
  if (count < 0 || num_rows < 1 || (side != 0 && side != 1))
    return fail(PBG_ERR_INVALID, "pbg_sample_uniform_negatives: bad arguments");
  if (count == 0) return PBG_OK;
  if (!out) return fail(PBG_ERR_INVALID, "pbg_sample_uniform_negatives: null output");
  hipLaunchKernelGGL(sample_uniform_kernel, dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, (hipStream_t)stream, seed,
                     (uint32_t)side, num_rows, count, out);
  return check_launch("pbg_sample_uniform_negatives");
}

extern "C" size_t pbg_train_step_workspace_bytes(const pbg_step_desc* desc) {
  if (validate(desc, false) != PBG_OK) return 0;
  Plan plan;
  make_plan(desc, nullptr, &plan);
  return plan.bytes;
}

namespace {
// prep | operator forward | score GEMMs | loss | dN GEMMs | dA GEMMs | rowback | params | sort | update
constexpr int kStages = 10;

// The library's own second stream per device, on which the sort of a call's keys runs beside the
// chunk kernel (the keys do not depend on the embeddings).  A call forks it from the caller's stream
// with one event and joins it back with another before the update reads the sorted keys; a ring of
// event pairs, so that consecutive calls do not share one.  Default priority, like every stream here.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork[8], join[8], mid[8], tail[8];
  std::atomic<unsigned> next{0};
  bool ok = false;
};
SideStream* side_stream() {
  static SideStream tab[kMaxDevices];
  static bool tried[kMaxDevices];
  static std::mutex mu;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  SideStream& ss = tab[dev];
  if (!tried[dev]) {
    tried[dev] = true;
    bool ok = hipStreamCreateWithFlags(&ss.stream, hipStreamNonBlocking) == hipSuccess;
    for (int i = 0; ok && i < 8; ++i)
      ok = hipEventCreateWithFlags(&ss.fork[i], hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&ss.join[i], hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&ss.mid[i], hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&ss.tail[i], hipEventDisableTiming) == hipSuccess;
    ss.ok = ok;
    if (!ok) (void)hipGetLastError();
  }
  return ss.ok ? &ss : nullptr;
}

template <int DEPTH>
void launch_loss_depth(const StepCtx& c, hipStream_t s) {
  const dim3 grid = wave_grid((int64_t)c.K * c.C * c.P);
  if (is_distance(c.cmp)) hipLaunchKernelGGL((loss_kernel<DEPTH, true>), grid, dim3(kRowThreads), 0, s, c);
  else hipLaunchKernelGGL((loss_kernel<DEPTH, false>), grid, dim3(kRowThreads), 0, s, c);
}

void launch_loss(const StepCtx& c, hipStream_t s) {
  const int nn = c.side[0].nn > c.side[1].nn ? c.side[0].nn : c.side[1].nn;
  if (nn <= 4 * kWave) launch_loss_depth<4>(c, s);
  else if (nn <= 8 * kWave) launch_loss_depth<8>(c, s);
  else if (nn <= 20 * kWave) launch_loss_depth<20>(c, s);
  else launch_loss_depth<0>(c, s);
}

// The regularizer's parameter terms and per-batch value, once the positives' cubes are written.
// Reads the operator parameters: before run_params updates them.
void launch_reg(const StepCtx& c, hipStream_t s) {
  if (c.reg_coef == 0.f) return;
  if (c.dynamic && c.op != PBG_OP_NONE)
    for (int side = 0; side < 2; ++side)
      hipLaunchKernelGGL(reg_factor_kernel, wave_grid(c.num_relations), dim3(kRowThreads), 0, s, c, side);
  hipLaunchKernelGGL(reg_reduce_kernel, dim3((unsigned)c.K), dim3(256), 0, s, c);
}

int run_step(const pbg_step_desc* desc, const pbg_step_buffers* bufs, hipStream_t s, hipEvent_t* ev) {
  int rc = validate(desc, true);
  if (rc != PBG_OK) return rc;
  Plan plan;
  make_plan(desc, bufs, &plan);
  if ((rc = check_buffers(desc, bufs, plan, true)) != PBG_OK) return rc;
  const bool stream = plan.stream && !bufs->lhs_global;
  if (stream) {  // every gradient row is written in its final form; the operator-output gradients cover the positives only
    for (int side = 0; side < 2; ++side) {
      plan.c.side[side].uni_direct = plan.c.side[side].uni_dz_direct = 0;
      if (plan.c.side[side].has_op) plan.c.side[side].op_rows = plan.c.B;
    }
  }
  const StepCtx& c = plan.c;
  RelOrder rel_order;
  auto mark = [&](int i) {
    if (ev) (void)hipEventRecord(ev[i], s);
  };
  const int64_t npairs = (int64_t)c.K * c.rk;
  const uint64_t rows = (uint64_t)desc->num_lhs_rows + (desc->shared_table ? 0 : (uint64_t)desc->num_rhs_rows);
  // gradient rows are numbered batch by batch, so a stable sort on the row bits alone orders them by (row, batch)
  const int sort_bits = bits_for(rows - 1) + c.kbits;
  uint64_t* skeys = nullptr;
  uint32_t* svals = nullptr;
  const uint32_t* long_runs = nullptr;  // the sort's word on runs of equal keys (read by a single-worker update)
  hipEvent_t sort_done = nullptr;  // set: the sort was queued on the side stream and ends with this event
  // Once the side stream has been forked from `s` it must be joined back on EVERY way out of this function:
  // under a HIP graph capture an unjoined fork leaves the library's stream inside the caller's capture.
  struct JoinOnExit {
    hipStream_t into;
    hipEvent_t ev = nullptr, ev2 = nullptr;
    ~JoinOnExit() {
      if (ev) (void)hipStreamWaitEvent(into, ev, 0);
      if (ev2) (void)hipStreamWaitEvent(into, ev2, 0);
    }
  } join_guard{s};
  hipEvent_t params_done = nullptr;  // set: the operator parameters' kernels were queued on the side stream
  mark(0);
  if ((rc = run_renorm(plan, bufs, s)) != PBG_OK) return rc;
  CosBack cos_back{nullptr, nullptr, nullptr, nullptr};
  const CosBack* cos_back_p = nullptr;
  if (stream) {
    StepCtx cs = c;  // what the streaming kernels see
    if (plan.stream_cos) {
      // cos as dot on normalised rows: the tables' normalised copy (as they are now, after max_norm), the route's
      // dot kernels on it, and the normalisation's backward where the update has summed a row's gradients
      const int tables = desc->shared_table ? 1 : 2;
      for (int t = 0; t < tables; ++t) {
        const int64_t nrows = t ? desc->num_rhs_rows : desc->num_lhs_rows;
        PBG_DISPATCH_NVH(plan.nvh, normalize_rows_kernel, wave_grid(nrows), s, t ? bufs->w_rhs : bufs->w_lhs, nrows, c.D,
                         plan.ynorm[t], plan.yinv[t]);
      }
      cs.cmp = PBG_CMP_DOT;
      cs.side[0].w = plan.ynorm[0];
      cs.side[1].w = plan.ynorm[tables - 1];
      cos_back = CosBack{plan.ynorm[0], plan.yinv[0], plan.ynorm[1], plan.yinv[1]};
      cos_back_p = &cos_back;
    }
    if ((rc = stream_prep(cs, plan.sp, plan.nvh, s)) != PBG_OK) return rc;
    mark(1);
    mark(2);
    if ((rc = stream_chunks(cs, plan.sp, s)) != PBG_OK) return rc;
    // The sort needs the keys alone (made before the chunk kernel): on the side stream it runs beside the per-edge
    // finish and the parameter kernels instead of behind them.  (Beside the chunk kernel itself there is no room:
    // its workgroups hold every compute unit's LDS.)
    if (2 * c.K * c.C >= 128 && getenv("PBG_DISABLE_SIDE_STREAM") == nullptr) {
      if (SideStream* ss = side_stream()) {
        const unsigned slot = ss->next.fetch_add(1) & 7u;
        if (hipEventRecord(ss->fork[slot], s) != hipSuccess || hipStreamWaitEvent(ss->stream, ss->fork[slot], 0) != hipSuccess)
          return fail(PBG_ERR_LAUNCH, "step: cannot fork the side stream");
        const int sort_rc = sort_pairs(c.keys, c.vals, plan.keys_b, plan.vals_b, npairs, c.kbits, sort_bits, plan.sort_temp,
                                       ss->stream, &skeys, &svals, c.kbits == 0 ? &long_runs : nullptr);
        if (hipEventRecord(ss->join[slot], ss->stream) != hipSuccess)
          return fail(PBG_ERR_LAUNCH, "step: cannot record the side stream's join");
        join_guard.ev = sort_done = ss->join[slot];
        if (sort_rc != PBG_OK) return sort_rc;
      }
    }
    mark(3);
    mark(4);
    mark(5);
    mark(6);
    if ((rc = stream_finish(cs, plan.sp, plan.nvh, s)) != PBG_OK) return rc;
    launch_reg(c, s);
    mark(7);
  } else if (plan.fused) {
    // gather -> operator -> scores -> loss -> backward -> raw-row gradients in one kernel per chunk
    // One persistent workgroup per compute unit (the LDS footprint allows no more); workgroup b takes chunks
    // b, b + grid, ...: `rounds` of them at most.
    const int cus = compute_units(), chunks = c.K * c.C;
    const int rounds = (int)ceil_div(chunks, cus);
    int blocks = chunks < cus ? chunks : cus;
    // The sort keys do not depend on the embeddings: made by a kernel of their own first, they can be sorted
    // on the side stream while the chunk kernel runs -- on the compute units that it leaves alone (its
    // workgroups would otherwise hold every one of them until the last chunk is done).  That is free when
    // fewer workgroups finish in the same number of rounds, and pays for a round more when the sort is a
    // long one (two or more passes inside the buckets: tables beyond 2^17 rows, where hot rows make them long).
    // A small call keeps everything on one stream: two events cost more there than its sort.
    SideStream* ss = nullptr;
    if (chunks >= 128 && cus > 1 && getenv("PBG_DISABLE_SIDE_STREAM") == nullptr) {
      const int rounds_beside = (int)ceil_div(chunks, cus - 1);
      // (the sliced chunk kernel's rounds are far longer than any sort: beside it only when that is free)
      if (rounds_beside == rounds || (sort_bits - c.kbits > 17 && !plan.fl.sliced)) {
        ss = side_stream();
        if (ss) blocks = (int)ceil_div(chunks, rounds_beside);
      }
    }
    unsigned slot = 0;
    if (ss || plan.fl.sliced) {
      plan.c.fused_rowid = plan.fused_rowid;
      if ((rc = fused_ids(c, s)) != PBG_OK) return rc;
    }
    if (ss) {
      slot = ss->next.fetch_add(1) & 7u;
      if (hipEventRecord(ss->fork[slot], s) != hipSuccess) return fail(PBG_ERR_LAUNCH, "step: cannot fork the side stream");
    }
    if ((rc = fused_chunks(c, plan.fl, blocks, s)) != PBG_OK) return rc;  // (queued first: it is to find the machine empty)
    if (ss) {
      if (hipStreamWaitEvent(ss->stream, ss->fork[slot], 0) != hipSuccess)
        return fail(PBG_ERR_LAUNCH, "step: cannot fork the side stream");
      const int sort_rc = sort_pairs(c.keys, c.vals, plan.keys_b, plan.vals_b, npairs, c.kbits, sort_bits, plan.sort_temp,
                                     ss->stream, &skeys, &svals, c.kbits == 0 ? &long_runs : nullptr);
      if (hipEventRecord(ss->join[slot], ss->stream) != hipSuccess)
        return fail(PBG_ERR_LAUNCH, "step: cannot record the side stream's join");
      join_guard.ev = sort_done = ss->join[slot];
      if (sort_rc != PBG_OK) return sort_rc;
      // A translation's gradient and Adagrad steps read the operator-output gradients the chunk kernel left and
      // write the operator's parameters: nothing the table update touches (a diagonal's gradient reads table rows).
      // Two short launches with a handful of waves each: behind the sort on the side stream they run beside the
      // update instead of in front of it.
      if (c.op == PBG_OP_TRANSLATION && !bufs->lhs_global && getenv("PBG_DISABLE_SIDE_PARAMS") == nullptr) {
        if (hipEventRecord(ss->mid[slot], s) != hipSuccess || hipStreamWaitEvent(ss->stream, ss->mid[slot], 0) != hipSuccess)
          return fail(PBG_ERR_LAUNCH, "step: cannot order the side stream behind the chunk kernel");
        const int params_rc = run_params(desc, bufs, plan, ss->stream, &rel_order, false);
        if (hipEventRecord(ss->tail[slot], ss->stream) != hipSuccess)
          return fail(PBG_ERR_LAUNCH, "step: cannot record the side stream's second join");
        join_guard.ev2 = params_done = ss->tail[slot];
        if (params_rc != PBG_OK) return params_rc;
      }
    }
    mark(1);
    mark(2);
    mark(3);
    mark(4);
    mark(5);
    mark(6);
    mark(7);
  } else {
    if ((rc = run_prep(plan, s)) != PBG_OK) return rc;
    // The keys exist from here on and nothing before the update looks at them again (the global embeddings'
    // gradient kernel does: not with those): a large call sorts them on the side stream beside the products.
    if ((int64_t)c.K * c.C * c.P >= 16384 && !bufs->lhs_global && getenv("PBG_DISABLE_SIDE_STREAM") == nullptr) {
      if (SideStream* ss = side_stream()) {
        const unsigned slot = ss->next.fetch_add(1) & 7u;
        if (hipEventRecord(ss->fork[slot], s) != hipSuccess || hipStreamWaitEvent(ss->stream, ss->fork[slot], 0) != hipSuccess)
          return fail(PBG_ERR_LAUNCH, "step: cannot fork the side stream");
        const int sort_rc = sort_pairs(c.keys, c.vals, plan.keys_b, plan.vals_b, npairs, c.kbits, sort_bits, plan.sort_temp,
                                       ss->stream, &skeys, &svals, c.kbits == 0 ? &long_runs : nullptr);
        if (hipEventRecord(ss->join[slot], ss->stream) != hipSuccess)
          return fail(PBG_ERR_LAUNCH, "step: cannot record the side stream's join");
        join_guard.ev = sort_done = ss->join[slot];
        if (sort_rc != PBG_OK) return sort_rc;
      }
    }
    mark(1);
    if ((rc = run_operator_forward(plan, s, &rel_order)) != PBG_OK) return rc;
    mark(2);
    if ((rc = run_scores(plan, s)) != PBG_OK) return rc;
    mark(3);
    launch_loss(c, s);
    mark(4);
    if ((rc = run_backward_dn(plan, s)) != PBG_OK) return rc;
    mark(5);
    if ((rc = run_backward_da(plan, s)) != PBG_OK) return rc;
    mark(6);
    if ((rc = run_rowback(plan, s)) != PBG_OK) return rc;
    launch_reg(c, s);
    mark(7);
  }
  if (!params_done && (rc = run_params(desc, bufs, plan, s, &rel_order, stream)) != PBG_OK) return rc;
  if (bufs->lhs_global) {  // the raw-row gradients are complete and still one per gathered row
    hipLaunchKernelGGL(global_grad_kernel, dim3((unsigned)c.K, (unsigned)(2 * plan.gslices)), dim3(kGlobalHalves * 32), 0,
                       s, c, plan.gth, plan.gslices, plan.fused ? 1 : 0);
    hipLaunchKernelGGL(global_update_kernel, wave_grid(c.D), dim3(kRowThreads), 0, s, c, plan.gth, plan.gslices,
                       bufs->lhs_global == bufs->rhs_global ? 1 : 0, bufs->lhs_global, bufs->lhs_global_sum,
                       bufs->rhs_global, bufs->rhs_global_sum, desc->relation_lr);
    if ((rc = check_launch("step global embeddings")) != PBG_OK) return rc;
  }
  mark(8);
  if (sort_done) {
    join_guard.ev = nullptr;
    if (hipStreamWaitEvent(s, sort_done, 0) != hipSuccess) return fail(PBG_ERR_LAUNCH, "step: cannot join the side stream");
  } else {
    rc = sort_pairs(c.keys, c.vals, plan.keys_b, plan.vals_b, npairs, c.kbits, sort_bits, plan.sort_temp, s, &skeys, &svals,
                    c.kbits == 0 ? &long_runs : nullptr);
    if (rc != PBG_OK) return rc;
  }
  mark(9);
  if (c.kbits != 0) long_runs = nullptr;  // the word counts positions per ROW; only with one batch per call is that a run
  // loss_out[k] and violators[k]: the batches' sums of the per-edge values, with the update's first launch
  const BatchSums sums{c.lossrow, c.violrow, c.C * c.P, c.K, c.loss_out, c.violators};
  if (desc->shared_table) {
    rc = row_adagrad_sorted(skeys, svals, npairs, c.kbits, c.gr, c.D, bufs->w_lhs, bufs->g_lhs,
                            desc->num_lhs_rows, nullptr, nullptr, 0, desc->lr, s, long_runs, cos_back_p, &sums);
  } else {
    rc = row_adagrad_sorted(skeys, svals, npairs, c.kbits, c.gr, c.D, bufs->w_lhs, bufs->g_lhs,
                            desc->num_lhs_rows, bufs->w_rhs, bufs->g_rhs, desc->num_rhs_rows, desc->lr, s, long_runs,
                            cos_back_p, &sums);
  }
  if (params_done) {
    join_guard.ev2 = nullptr;
    if (hipStreamWaitEvent(s, params_done, 0) != hipSuccess) return fail(PBG_ERR_LAUNCH, "step: cannot join the side stream");
  }
  mark(10);
  return rc;
}
}  // namespace

extern "C" int pbg_train_step(const pbg_step_desc* desc, const pbg_step_buffers* bufs, pbg_stream_t stream) {
  return run_step(desc, bufs, (hipStream_t)stream, nullptr);
}

extern "C" int pbg_train_step_num_stages(void) { return kStages; }

extern "C" int pbg_train_step_is_fused(const pbg_step_desc* desc) {
  if (validate(desc, true) != PBG_OK) return 0;
  Plan plan;
  make_plan(desc, nullptr, &plan);
  return plan.fused ? 1 : 0;
}

extern "C" int pbg_train_step_route(const pbg_step_desc* desc) {
  if (validate(desc, true) != PBG_OK) return -1;
  Plan plan;
  make_plan(desc, nullptr, &plan);
  return plan.fused ? PBG_ROUTE_FUSED : (plan.stream ? PBG_ROUTE_STREAM : PBG_ROUTE_STAGED);
}

extern "C" int pbg_train_step_profile(const pbg_step_desc* desc, const pbg_step_buffers* bufs, pbg_stream_t stream,
                                      float* stage_ms) {
  if (!stage_ms) return fail(PBG_ERR_INVALID, "pbg_train_step_profile: null output");
  hipEvent_t ev[kStages + 1];
  for (int i = 0; i <= kStages; ++i) {
    if (hipEventCreate(&ev[i]) != hipSuccess) return fail(PBG_ERR_LAUNCH, "pbg_train_step_profile: hipEventCreate failed");
  }
  int rc = run_step(desc, bufs, (hipStream_t)stream, ev);
  if (rc == PBG_OK) {
    if (hipEventSynchronize(ev[kStages]) != hipSuccess) rc = fail(PBG_ERR_LAUNCH, "pbg_train_step_profile: sync failed");
  }
  for (int i = 0; i < kStages && rc == PBG_OK; ++i) {
    if (hipEventElapsedTime(&stage_ms[i], ev[i], ev[i + 1]) != hipSuccess)
      rc = fail(PBG_ERR_LAUNCH, "pbg_train_step_profile: elapsed time failed");
  }
  for (int i = 0; i <= kStages; ++i) hipEventDestroy(ev[i]);
  return rc;
}

extern "C" int pbg_model_ranks(const pbg_step_desc* desc, const pbg_step_buffers* bufs, float* lhs_pos, float* rhs_pos,
                               int64_t* lhs_rank, int64_t* rhs_rank, float* loss_edge, int64_t auc_samples,
                               uint64_t auc_seed, int64_t* auc_hits, pbg_stream_t stream) {
  int rc = validate(desc, false);
  if (rc != PBG_OK) return rc;
  Plan plan;
  make_plan(desc, bufs, &plan);
  if ((rc = check_buffers(desc, bufs, plan, false)) != PBG_OK) return rc;
  const StepCtx& c = plan.c;
  if (!lhs_pos || !rhs_pos || !lhs_rank || !rhs_rank || !loss_edge || (auc_samples > 0 && !auc_hits) || auc_samples < 0)
    return fail(PBG_ERR_INVALID, "pbg_model_ranks: null output");
  hipStream_t s = (hipStream_t)stream;
  RelOrder rel_order;
  if ((rc = run_renorm(plan, bufs, s)) != PBG_OK) return rc;
  if ((rc = run_prep(plan, s)) != PBG_OK) return rc;
  if ((rc = run_operator_forward(plan, s, &rel_order)) != PBG_OK) return rc;
  if ((rc = run_scores(plan, s)) != PBG_OK) return rc;
  hipLaunchKernelGGL(ranks_out_kernel, wave_grid((int64_t)c.K * c.B), dim3(kRowThreads), 0, s, c, lhs_pos, rhs_pos, lhs_rank,
                     rhs_rank, loss_edge);
  if (auc_samples > 0) {
    static_assert(sizeof(unsigned long long) == sizeof(int64_t), "auc_hits is written as two 64-bit counters");
    hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(64), 0, s, (unsigned long long*)auc_hits, 2);
    hipLaunchKernelGGL(auc_sample_kernel, dim3((unsigned)ceil_div(auc_samples, 256), 2), dim3(256), 0, s, c, lhs_pos, rhs_pos,
                       auc_samples, auc_seed, (unsigned long long*)auc_hits);
  }
  return check_launch("pbg_model_ranks");
}

extern "C" int pbg_model_forward(const pbg_step_desc* desc, const pbg_step_buffers* bufs, float* lhs_pos,
                                 float* rhs_pos, float* lhs_neg, float* rhs_neg, pbg_stream_t stream) {
  int rc = validate(desc, false);
  if (rc != PBG_OK) return rc;
  Plan plan;
  make_plan(desc, bufs, &plan);
  if ((rc = check_buffers(desc, bufs, plan, false)) != PBG_OK) return rc;
  const StepCtx& c = plan.c;
  if (!lhs_pos || !rhs_pos || (c.side[0].nn > 0 && !lhs_neg) || (c.side[1].nn > 0 && !rhs_neg))
    return fail(PBG_ERR_INVALID, "pbg_model_forward: null output");
  hipStream_t s = (hipStream_t)stream;
  RelOrder rel_order;
  if ((rc = run_renorm(plan, bufs, s)) != PBG_OK) return rc;
  if ((rc = run_prep(plan, s)) != PBG_OK) return rc;
  if ((rc = run_operator_forward(plan, s, &rel_order)) != PBG_OK) return rc;
  if ((rc = run_scores(plan, s)) != PBG_OK) return rc;
  hipLaunchKernelGGL(scores_out_kernel, wave_grid((int64_t)c.K * c.B), dim3(kRowThreads), 0, s, c, lhs_pos, rhs_pos,
                     lhs_neg, rhs_neg);
  return check_launch("pbg_model_forward");
}
