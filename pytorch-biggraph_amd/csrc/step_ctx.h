// What one call of the training step works on: the two sides' tables, index
// arrays and staging buffers, and the geometry of its batches and chunks.
#pragma once

#include "pbg_internal.h"
#include "row_ops.h"

namespace pbg {

struct SideCtx {
  const float* w;       // embedding table of this side
  const float* glob;    // global embedding of this side's entity type [D], or null
  const int64_t* idx;   // [K, B] positive entities
  const int64_t* uidx;  // [K, C, U] uniform negatives (null if u == 0, or if they are drawn in the step)
  uint64_t useed;       // seed of the in-step draw (uidx == null)
  int64_t key_base;     // offset of this table in the sort-key row space
  int64_t num_rows;
  int all;              // RelationSchema.all_negs: the negatives are the table's rows 0 .. num_rows - 1 (u == num_rows)
  int nb, u, nn;        // batch-negative / uniform / total negative columns of this side
  int stride_p;         // rows per chunk of the buffer that holds the positives
  int alias;            // positives are the first P rows of the negatives matrix
  float *xn, *xp, *xa;  // prepared negatives matrix, positives, operated positives (dynamic)
  float *an, *ap, *aa;  // per-row aux of the above: 1/norm (cos) or squared norm (l2)
  float *bn, *bp, *ba;  // with config.bias: the rows' biases (their first coordinates; the rows hold 0 there)
  float* bs;            // with config.bias: [K*C*P] row sums of dLoss/dscore of this side's score matrix
  float* gs;            // with config.bias and l2: [K*C, P, nn] dLoss/dscore itself (s then holds -2 dLoss/d squared distance, from which it cannot be read back)
  float *dxn, *dxp, *dxa;
  float* s;             // [K*C, P, nn] scores against this side's negatives, then dLoss/dS
  float* rs;            // [K*C*P] row sums of dLoss/d(squared distance) (l2)
  int slot_pos, slot_uni;
  // The gradient rows of this side's uniform negatives are read where the backward GEMM wrote them
  // (dxn, which then lies behind gr in one block; uni_row0 = row number of dxn's first row counted from gr):
  // with the dot comparator and no operator on them the raw-row gradient IS that row.
  int uni_direct;
  int64_t uni_row0;
  // (operator side, element-wise operator, dot comparator:) the gradient at the operator's output of a uniform
  // negative IS its row of dxn; it is not copied to dz, the parameter gradient reads it there
  int uni_dz_direct;
  int has_op;           // an operator acts on this side's positives
  int op_uniform;       // ... and on its uniform negatives (standard mode)
  const float *p0, *p1; // operator parameters
  float *xraw, *z, *dz; // [K, op_rows, D] staging of operator inputs / outputs / output grads
  int op_rows;
  // N3 regularizer, dynamic relations: per relation, the gradient of the parameter
  // term per edge [num_relations, D] and the term itself [num_relations], both
  // from the parameters as they are before the call's updates
  float *reg_pgrad, *reg_pcube;
  int plain_written, opd_written;  // dxp / dxa were produced by a GEMM
};

struct StepCtx {
  int D, K, B, P, C, U, last, dynamic, op, cmp, loss, num_relations;
  int bias;    // config.bias: BiasedComparator around the comparator (model.py:306-344,902-903)
  int half;    // config.half_precision: prepared rows, negative scores and their gradients are float16 numbers (model.py:504-505,827-829)
  int affine;  // op == PBG_OP_LINEAR with a translation added to the product (operators.py:103-115, 272-293)
  float margin;
  SideCtx side[2];
  const int64_t* rel;
  const float* edge_weight;
  const float* rel_weights;
  float* pos[2];   // [K*C*P] positive score paired with lhs negatives / rhs negatives
  float* dpos[2];  // gradients of the above (standard mode: only [0], already summed)
  float* lossrow;  // [K*C*P]
  int* violrow;    // [K*C*P, 2] violators of each edge (lhs, rhs)
  int rk;          // gradient rows per batch
  int kbits;
  float* gr;       // [K*rk, D] gradient rows
  uint64_t* keys;
  uint32_t* vals;
  unsigned long long* violators;  // [K, 2]
  float* loss_out;                // [K]
  float reg_coef;  // N3 regularizer weight (0: none)
  float* regrow;   // [K, 2, B] sum of cubed moduli of each positive's prepared row(s), per side
  float* reg_out;  // [K] or null
  int* fused_rowid;  // fused route: [K*C, 256] row id of every operand-row slot of a chunk (-1: none), see fused_ids_kernel
};

// Uniform negative number flat = (k * C + chunk) * U + u of side s: given by the
// caller or drawn here (model.py:70-75).
__device__ __forceinline__ int64_t uniform_negative(const SideCtx& sd, int s, int64_t flat) {
  if (sd.all) return flat % sd.u;  // (one chunk: flat = batch * u + entity)
  if (sd.uidx) return sd.uidx[flat];
  return sampled_row(sd.useed, (uint64_t)flat, (uint32_t)s, sd.num_rows);
}

}  // namespace pbg
