// The fused route of the training step: a chunk's operand rows and score
// matrices stay in LDS from the gather to the raw-row gradients (see fused.hip).
#pragma once

#include "step_ctx.h"

namespace pbg {

constexpr int kFusedIds = 256;  // slots of a chunk's row id array: 8 waves x 16 rounds x 2 half-waves

struct FusedLayout {
  int ldx, lds;                  // row strides (floats) of the operand rows and of the score rows
  int xn[2], sc[2], sq[2], rs[2], cs[2], pos, dpos;  // offsets in floats
  int part;                      // [2 sides][dLoss/dpos, weighted loss, violators][P] per-side results of the loss phase
  int xch;                       // cos: [2 column groups][64 rows] partial <row, gradient row> of the product being written out
  int ids;                       // int32 row ids of the 2N operand rows (-1: padding), kFusedIds slots; last block
  int total;                     // floats
  int sliced;                    // rows wider than 128 floats: they pass through LDS in slices of 128 columns (ldx is a slice's stride)
};

// Whether the route takes this configuration; fills the LDS layout.  (f->sliced: the chunk kernel then needs
// fused_ids to have run.)
bool fused_layout(const StepCtx& c, FusedLayout* f);

// Row ids and sort keys of every chunk, ahead of the chunk kernel (c.fused_rowid set): the keys can
// then be sorted while the chunks run.  Without this call (c.fused_rowid null) the chunk kernel
// makes both itself.
int fused_ids(const StepCtx& c, hipStream_t stream);

// Width of a slice of the sliced chunk kernel (sliced.hip), in columns.
constexpr int kSliceCols = 128;
// (fused_chunks hands a layout with `sliced` set on to this one)
int sliced_chunks(const StepCtx& c, const FusedLayout& fl, int blocks, hipStream_t stream);

// The chunk kernel on `blocks` workgroups, each of which takes chunks blockIdx, blockIdx + blocks, ...
int fused_chunks(const StepCtx& c, const FusedLayout& fl, int blocks, hipStream_t stream);

}  // namespace pbg
