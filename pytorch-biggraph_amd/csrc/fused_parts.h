// Pieces shared by the two chunk kernels of the fused route (fused.hip: a chunk's rows whole in LDS;
// sliced.hip: in slices of 128 columns): the loss of a score row held in LDS and the chunk's geometry.
#pragma once

#include "fused.h"
#include "mfma_tiles.h"
#include "row_ops.h"

namespace pbg {
namespace {

constexpr int kFusedThreads = 512;
constexpr int kFusedSide = kFusedIds / 2;  // ... per side

// Loss of one positive against one side's negatives for a score row held in LDS
// and spread over 8 adjacent lanes: lane qd owns columns qd, qd + 8, ..., `ne` of
// them (the same for every lane: the row is read up to the next multiple of 8).
// Masked and pad columns hold their final score in LDS already (-1e9 resp. -inf;
// l2: -inf as a raw product, which turns into a distance score of -inf): such
// scores add nothing to any loss and get a zero gradient without a test per
// column.  Overwrites the row with dLoss/dscore (l2: -2 dLoss/d squared distance);
// the outputs are reduced over the group.  Every VALU instruction here competes
// with the matrix instructions of the compute waves for the same issue slots (the
// fp32 matrix products run on the vector ALUs), so the per-column work is kept
// to the loss's own arithmetic.
// HALF (config.half_precision): dLoss/dscore goes back through the scores' cast to fp32 (model.py:827-829)
// and is written as the float16 number that makes of it.
template <int CMP, int LOSS, int kCols, bool HALF>
__device__ __forceinline__ void fused_row_loss(float* lds, int row_at, int bn_at, float a2, float margin, float inv_nn, int ne,
                                               float pos, float w, int qd, float* loss_w, float* dpos_out, int* viol_out,
                                               float* rowsum_out) {
  constexpr bool l2 = CMP == PBG_CMP_L2;
  const int at = row_at + qd, bat = bn_at + qd;
  float loss_acc = 0.f, rowsum = 0.f, dpos = 0.f;
  int viol = 0;
  if (LOSS != PBG_LOSS_SOFTMAX) {
    float gsum = 0.f;
    if (LOSS == PBG_LOSS_LOGISTIC && qd == 0) {
      loss_acc += softplusf(-pos);
      dpos += (sigmoidf(pos) - 1.0f) * w;
    }
#pragma unroll
    for (int e = 0; e < kCols; ++e) {
      if (e >= ne) break;  // the same for all lanes
      float te = lds[at + 8 * e];
      bool lv = true;
      if (l2) {
        // v_sqrt_f32 and v_rcp_f32 (1 ulp) stand in for the correctly rounded sequences: the
        // expansion ||a||^2 - 2ab + ||b||^2 itself carries 1e-7 * ||a||^2 of rounding noise
        const float q = fmaf(-2.0f, te, lds[bat + 8 * e]) + a2;
        lv = q >= 1e-30f;  // clamped distances are constants (model.py:236)
        te = -__builtin_amdgcn_sqrtf(fmaxf(q, 1e-30f));
      }
      float g;
      if (LOSS == PBG_LOSS_RANKING) {
        // F.margin_ranking_loss(neg, pos, target=-1): max(0, (t - pos) + margin); the
        // clamp lets the gradient through at exactly 0
        const float x = (te - pos) + margin;
        loss_acc += fmaxf(x, 0.f);
        g = (x >= 0.f) ? w : 0.f;
        gsum += g;
      } else {
        float sg;
        loss_acc += softplus_sigmoid(te, &sg) * inv_nn;
        g = sg * inv_nn * w;
      }
      if (te > pos) ++viol;
      if (l2) {
        // t = -sqrt(q): dLoss/dq = g * 0.5 / t; stored as -2 dLoss/dq so that the
        // backward products give the cross terms of ||a||^2 - 2ab + ||b||^2
        const float dq = lv ? g * 0.5f * __builtin_amdgcn_rcpf(te) : 0.f;
        rowsum += dq;
        g = -2.0f * dq;
      }
      lds[at + 8 * e] = HALF ? half_round(g) : g;
    }
    if (LOSS == PBG_LOSS_RANKING) dpos -= gsum;
  } else {
    float t[kCols], ex[kCols];
    uint32_t live = 0xffffffffu;  // bit e clear: the distance of column e was clamped, a constant without gradient
    float mx = pos;
#pragma unroll
    for (int e = 0; e < kCols; ++e) {
      t[e] = -INFINITY;
      if (e < ne) {
        float te = lds[at + 8 * e];
        if (l2) {
          const float q = fmaf(-2.0f, te, lds[bat + 8 * e]) + a2;
          if (!(q >= 1e-30f)) live &= ~(1u << e);
          te = -sqrtf(fmaxf(q, 1e-30f));
        }
        t[e] = te;
        mx = fmaxf(mx, te);
        if (te > pos) ++viol;
      }
    }
    mx = oct_max(mx);
    float z = 0.f;
#pragma unroll
    for (int e = 0; e < kCols; ++e) {
      ex[e] = expf(t[e] - mx);
      z += ex[e];
    }
    const float epos = expf(pos - mx);
    z = oct_sum(z) + epos;
    const float inv_z = 1.0f / z;
    if (qd == 0) {
      loss_acc += (mx + logf(z)) - pos;
      dpos += (epos * inv_z - 1.0f) * w;
    }
    const float scale = inv_z * w;
#pragma unroll
    for (int e = 0; e < kCols; ++e) {
      if (e >= ne) break;
      float g = ex[e] * scale;
      if (l2) {
        const float dq = ((live >> e) & 1u) ? g * 0.5f / t[e] : 0.f;
        rowsum += dq;
        g = -2.0f * dq;
      }
      lds[at + 8 * e] = HALF ? half_round(g) : g;
    }
  }
  *loss_w = oct_sum(loss_acc) * w;
  *dpos_out = oct_sum(dpos);
  *rowsum_out = oct_sum(rowsum);
  *viol_out = oct_sum_int(viol);
}

// Geometry of one chunk, the same for both roles.
struct FusedGeom {
  int D, P, U, N, ldx, lds, xn0, xn1, sc0, sc1, sq0, sq1, rs0, rs1, cs0, cs1;
};

}  // namespace
}  // namespace pbg
