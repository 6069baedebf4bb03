// The streaming route of the training step: a chunk's positives stay in LDS
// while its negatives pass through in tiles (see stream.hip).
#pragma once

#include "step_ctx.h"

namespace pbg {

struct StreamPlan {
  int lda;     // LDS row stride (floats) of the operand rows
  int pr;      // rows kept of the positives' operand block: P rounded up to 4
  int ntiles;  // tiles of 32 negatives per (chunk, side)
  int grid;    // workgroups
  int n_at, a_at, g_at, total;  // LDS offsets and size, in floats
  // Per side s, indexed by edge (k * B + position): the operand row that edge's OTHER
  // side contributes to the scores against side s's negatives, that row's gradient,
  // and the gradient of the edge's own side-s row as a batch negative of its chunk.
  float* sa[2];
  float* sda[2];
  float* sdb[2];
  float* spos[2];   // [K * B] positive score paired with side s's negatives
  float* sloss[2];  // [K * C * P] weighted loss against side s's negatives
  float* scratch;   // [grid, ntiles, 2048] score tiles between the two sweeps
  int* colid[2];    // [K * C, P + U] row id of every column of side s's negatives (-1: padded position)
};

// Whether the route takes this configuration; fills the geometry (not the pointers).
bool stream_geometry(const StepCtx& c, StreamPlan* sp);
inline size_t stream_scratch_floats(const StreamPlan& sp) { return (size_t)sp.grid * sp.ntiles * 2048; }

// prep -> chunks -> finish leaves every gradient row of the call in c.gr with its sort
// key, the per-edge losses and violator counts, and the operator-output gradients
// the parameter stage reads.
int stream_prep(const StepCtx& c, const StreamPlan& sp, int nvh, hipStream_t stream);
int stream_chunks(const StepCtx& c, const StreamPlan& sp, hipStream_t stream);
int stream_finish(const StepCtx& c, const StreamPlan& sp, int nvh, hipStream_t stream);

}  // namespace pbg
