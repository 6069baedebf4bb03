// The fused route of the training step: the whole chain from gather to raw-row
// gradients for one chunk in one workgroup, operands resident in LDS.
//
// Eligible shapes (standard mode, operator none / translation / diagonal,
// comparator dot / cos / l2, batch + uniform negatives on both sides, D <= 128,
// P <= 64, U <= 64) keep a chunk's 2(P+U) prepared rows and its two score
// matrices in LDS (132 KB at P = U = 50, D = 100).  Eight waves: phase 0 gathers
// and applies the operator; phase 1 forms S = A N^T with fp32 MFMA (one row tile
// per wave, all column tiles in registers); phase 2 is the per-edge loss, in
// place in LDS; phase 3 forms the four gradient matrices
//   dL = dS_R N_R + dS_L[:, :P]^T R      dU_L = dS_L[:, P:]^T R     (and L <-> R)
// with MFMA straight from LDS and writes the raw-row gradients to HBM.
//
// The kernel is instantiated per comparator and loss and keeps its straight-line
// parts short: a workgroup runs every instruction once, so code that does not
// fit the instruction cache is paid for in fetch stalls by every workgroup.
#include "fused.h"

#include <cstdlib>

#include "fused_parts.h"

namespace pbg {
namespace {


// ---- helper role: waves 8..15 ----
// The helpers' global loads are all issued from straight-line code at addresses
// that are valid whatever the slot is (clamped), and what does not apply is
// dropped by a select afterwards: a load inside a branch makes the code that
// follows the branch wait for it, which would put the latency of every load on
// the step's critical path one after the other.
//
// Row ids and sort keys of chunk kc = (k, cc).  The id array has kFusedSide slots
// per side (slot s * kFusedSide + j = row j of side s's operand rows, -1 from row N
// on), so that the side is the same for a whole wave and everything chosen by it
// stays in scalar registers; thread t < kFusedIds owns slot t.  When the call's keys
// are sorted beside this kernel, fused_ids_kernel has made ids and keys beforehand
// (c.fused_rowid) and the ids are only fetched here.
__device__ __forceinline__ void fused_load_ids(const StepCtx& c, const FusedGeom& g, int kc, int k, int cc, int t, int* ids) {
  if (t >= kFusedIds) return;
  if (c.fused_rowid) {
    ids[t] = c.fused_rowid[(int64_t)kc * kFusedIds + t];
    return;
  }
  const int s = __builtin_amdgcn_readfirstlane(t >> 7), j = t & (kFusedSide - 1);
  const SideCtx& sd = c.side[s];
  const bool is_pos = j < g.P;
  const int q = cc * g.P + j, u = min(max(j - g.P, 0), g.U - 1);
  const bool real = j < g.N && (!is_pos || q < c.B);  // false: a slot past the operand rows or a padded position of the last chunk
  const int64_t flat = (int64_t)kc * g.U + u;
  const int64_t* src = sd.idx + (int64_t)k * c.B + min(q, c.B - 1);
  if (!is_pos && sd.uidx) src = sd.uidx + flat;
  int64_t id = *src;
  if (!is_pos && !sd.uidx)  // the fused route's tables have fewer than 2^31 rows: the draw's 32-bit form (sampled_row)
    id = (int64_t)(((philox_u64(sd.useed, (uint64_t)flat, (uint32_t)s) & 0xffffffffull) * (uint64_t)sd.num_rows) >> 32);
  id = clamp_index(id, sd.num_rows);
  const int64_t pair = (int64_t)k * c.rk + (is_pos ? sd.slot_pos + q : sd.slot_uni + cc * g.U + u);
  if (real) {
    c.keys[pair] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
    c.vals[pair] = (uint32_t)pair;
  }
  ids[t] = real ? (int)id : -1;
}

constexpr int kFusedRounds = kFusedIds / 16;  // rows per half-wave of the 8 helper waves

// What a chunk's rows need besides themselves: the relation's operator parameters
// and the two global embeddings at this lane's four columns.
struct FusedRowExtras {
  float4 par, glob0, glob1;
};

// Half a wave per row, 128-bit loads, all of a wave's rows in flight: half-wave h of
// helper wave w takes rows h * 8 + w + 16 u of side 0 (u < 8) and of side 1 (u >= 8).
// Padding slots read row 0 (dropped when the rows are written).  `active` false:
// the ids are not read.
__device__ __forceinline__ void fused_issue_rows(const StepCtx& c, const FusedGeom& g, const int* ids, int64_t rel, int lwave,
                                                 int lane, float4* v, int* idv, FusedRowExtras* x, bool active) {
  const int half = lane >> 5, c4 = min((lane & 31) << 2, g.D - 4);
  const int slot0 = half * 8 + lwave;
#pragma unroll
  for (int u = 0; u < kFusedRounds; ++u) {
    const int id = ids[slot0 + 16 * u];
    idv[u] = active ? id : -1;
  }
  // row address = (table + this lane's column) + id * row bytes: one 32 x 32 -> 64-bit multiply-add per row
  const char* w0 = reinterpret_cast<const char*>(c.side[0].w + c4);
  const char* w1 = reinterpret_cast<const char*>(c.side[1].w + c4);
  const uint32_t row_bytes = (uint32_t)g.D * 4u;
#pragma unroll
  for (int u = 0; u < kFusedRounds; ++u) {
    const char* w = u >= kFusedRounds / 2 ? w1 : w0;
    v[u] = *reinterpret_cast<const float4*>(w + (uint64_t)(uint32_t)max(idv[u], 0) * row_bytes);
  }
  // What is absent is read from the table's first row instead and dropped: a load
  // from "this pointer or nothing" would become a flat load, whose completion the
  // next LDS barrier waits for, behind every row load above.
  const bool has_par = c.op != PBG_OP_NONE, has_g0 = c.side[0].glob != nullptr, has_g1 = c.side[1].glob != nullptr;
  const float* fallback = c.side[0].w;
  const float4 par = *reinterpret_cast<const float4*>((has_par ? c.side[1].p0 + rel * g.D : fallback) + c4);
  const float4 g0 = *reinterpret_cast<const float4*>((has_g0 ? c.side[0].glob : fallback) + c4);
  const float4 g1 = *reinterpret_cast<const float4*>((has_g1 ? c.side[1].glob : fallback) + c4);
  x->par = keep_if(par, has_par);
  x->glob0 = keep_if(g0, has_g0);
  x->glob1 = keep_if(g1, has_g1);
}

// Operator (rhs side) and, for l2, the squared norms (cos: the normalisation and the
// reciprocal norms); the rows of side S land in LDS.
// Only columns below D are written (the pad columns behind them were zeroed once,
// when the kernel started).  `pads`: the chunk has padded positives (a partial last
// chunk), whose rows are zeros.
template <int CMP, int S, bool HALF>
__device__ __forceinline__ void fused_store_side(const StepCtx& c, const FusedGeom& g, float* lds, int lwave, int lane,
                                                 const float4* v, const int* idv, const FusedRowExtras& x, bool pads) {
  const int half = lane >> 5, c4 = (lane & 31) << 2;
  const bool col_ok = c4 < g.D;
  const int j0 = half * 8 + lwave;
  const bool has_glob = (S ? c.side[1].glob : c.side[0].glob) != nullptr;
  const float4 gv = S ? x.glob1 : x.glob0;  // the global embedding of the side's entity type (model.py:486-492)
  int at = (S ? g.xn1 : g.xn0) + j0 * g.ldx + c4;
#pragma unroll
  for (int u = 0; u < kFusedRounds / 2; ++u, at += 16 * g.ldx) {
    const int j = j0 + 16 * u;
    if (j >= g.N) break;  // uniform per half-wave; the reduction below stays inside a half
    float4 y = v[S * (kFusedRounds / 2) + u];
    if (has_glob) {
      y.x += gv.x; y.y += gv.y; y.z += gv.z; y.w += gv.w;
    }
    if (S == 1) {
      if (c.op == PBG_OP_DIAGONAL) {
        y.x *= x.par.x; y.y *= x.par.y; y.z *= x.par.z; y.w *= x.par.w;
      } else if (c.op == PBG_OP_TRANSLATION) {
        y.x += x.par.x; y.y += x.par.y; y.z += x.par.z; y.w += x.par.w;
      }
    }
    if (CMP == PBG_CMP_COS) {  // comparator.prepare: the row times the reciprocal of its norm (model.py:187-192)
      const float sq = col_ok ? y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w : 0.f;
      const float part = half_sum_at_31(sq);  // complete in lanes 31 and 63
      const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(part), 31));
      const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(part), 63));
      const float inv = 1.0f / sqrtf(half ? hi : lo);
      y.x *= inv; y.y *= inv; y.z *= inv; y.w *= inv;
      if ((lane & 31) == 31) lds[(S ? g.sq1 : g.sq0) + j] = inv;
    }
    if (HALF) {  // embs.half() (model.py:504-505)
      y.x = half_round(y.x); y.y = half_round(y.y); y.z = half_round(y.z); y.w = half_round(y.w);
    }
    if (pads && idv[S * (kFusedRounds / 2) + u] < 0) y = make_float4(0.f, 0.f, 0.f, 0.f);
    if (col_ok) *reinterpret_cast<float4*>(&lds[at]) = y;
    if (CMP == PBG_CMP_L2) {
      const float sq = col_ok ? y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w : 0.f;
      const float nrm = sqrtf(half_sum_at_31(sq));
      if ((lane & 31) == 31) lds[(S ? g.sq1 : g.sq0) + j] = nrm * nrm;
    }
  }
}

// Results of one gradient product of the fused kernel on their way to HBM.
struct FusedOut {
  float* out;        // gradient row of the lane's row, at the wave's first column
  float* dz;         // the same place in the operator-output gradients, or null
  const float* par;  // diagonal operator: its parameters at the wave's first column, or null
  int self_at, other_at;  // l2: LDS offsets of the row's own operand row and of its partner's, at the wave's first column
  float coef, pcoef;      // l2: v += coef * self + pcoef * (self - other)
                          // cos: v = pcoef * (v - coef * self), the gradient through the normalisation
                          // (pcoef = 1 / norm, coef = <self, v over the whole row>)
};

// This lane's share of <own operand row, gradient row> over the columns it holds.
template <bool HALF>
__device__ __forceinline__ void fused_self_dot(const float* lds, int self_at, int col, int cols_left, float4 v, float* acc) {
  if (col >= cols_left) return;
  if (HALF) v = make_float4(half_round(v.x), half_round(v.y), half_round(v.z), half_round(v.w));
  const float4 self = *reinterpret_cast<const float4*>(&lds[self_at + col]);
  *acc += (self.x * v.x + self.y * v.y) + (self.z * v.z + self.w * v.w);
}

// HALF: the product is the gradient of a Half tensor, a float16 number; what follows (the cast's backward,
// prepare's, the operator's) is fp32.
template <int CMP, bool HALF>
__device__ __forceinline__ void fused_emit(const float* lds, const FusedOut& o, int col, int cols_left, float4 v) {
  if (col >= cols_left) return;  // past D (a multiple of 4)
  if (HALF) v = make_float4(half_round(v.x), half_round(v.y), half_round(v.z), half_round(v.w));
  constexpr bool L2 = CMP == PBG_CMP_L2;
  if (CMP == PBG_CMP_COS) {
    const float4 self = *reinterpret_cast<const float4*>(&lds[o.self_at + col]);
    v.x = o.pcoef * (v.x - o.coef * self.x);
    v.y = o.pcoef * (v.y - o.coef * self.y);
    v.z = o.pcoef * (v.z - o.coef * self.z);
    v.w = o.pcoef * (v.w - o.coef * self.w);
  }
  if (L2) {
    const float4 self = *reinterpret_cast<const float4*>(&lds[o.self_at + col]);
    float4 other = make_float4(0.f, 0.f, 0.f, 0.f);
    if (o.pcoef != 0.f) other = *reinterpret_cast<const float4*>(&lds[o.other_at + col]);
    v.x += o.coef * self.x + o.pcoef * (self.x - other.x);
    v.y += o.coef * self.y + o.pcoef * (self.y - other.y);
    v.z += o.coef * self.z + o.pcoef * (self.z - other.z);
    v.w += o.coef * self.w + o.pcoef * (self.w - other.w);
  }
  if (o.dz) *reinterpret_cast<float4*>(o.dz + col) = v;
  if (o.par) {
    const float4 p = *reinterpret_cast<const float4*>(o.par + col);
    v.x *= p.x; v.y *= p.y; v.z *= p.z; v.w *= p.w;
  }
  *reinterpret_cast<float4*>(o.out + col) = v;
}

// Score block of side s: S_s = A_(1-s) N_s^T, rows = the chunk's positives of the
// other side, columns = side s's negatives; this wave's row tile rt and NCT column
// tiles from ct0 on.  dot: the positive score is the diagonal (the i-th batch
// negative is the i-th positive's own partner row, model.py:177).
template <int NCT, bool L2, bool HALF>
__device__ __forceinline__ void fused_scores(float* lds, const FusedGeom& g, int s, int rt, int ct0, int lane, int pos_at,
                                             bool write_pos) {
  if (rt * 16 >= g.P || ct0 * 16 >= g.N) return;
  float4v acc[NCT];
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) acc[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
  // Row / column indices past the matrix are clamped or left to run into the
  // storage behind it instead of guarded: they only feed output rows / columns
  // that are never stored, and the loop body stays free of branches.
  const int ar = min(rt * 16 + (lane & 15), g.P - 1);
  const int a_at = (s ? g.xn0 : g.xn1) + ar * g.ldx;
  const int b_at = (s ? g.xn1 : g.xn0) + (ct0 * 16 + (lane & 15)) * g.ldx;  // column tile ct: 16 rows further down
  const int ksteps = (g.D + 3) >> 2;
  mfma_sweep_k16<NCT, HALF>(lds, a_at, b_at, 16 * g.ldx, ksteps >> 2, ksteps & 3, lane >> 4, acc);
  const int row = rt * 16 + (lane & 15);
  if (row >= g.P) return;
  const int at = (s ? g.sc1 : g.sc0) + row * g.lds + ct0 * 16 + 4 * (lane >> 4);
  const int n8 = (g.N + 7) & ~7;  // the loss reads whole groups of 8 columns: the pad columns among them score -inf
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) {
    const int col = (ct0 + ct) * 16 + 4 * (lane >> 4);
    // (HALF: a score is the float16 rounding of the fp32 sum, torch.bmm on Half tensors; the positive
    // score below is the fp32 sum itself, model.py:177)
    const float s0 = HALF ? half_round(acc[ct][0]) : acc[ct][0], s1 = HALF ? half_round(acc[ct][1]) : acc[ct][1];
    const float s2 = HALF ? half_round(acc[ct][2]) : acc[ct][2], s3 = HALF ? half_round(acc[ct][3]) : acc[ct][3];
    if (col < n8)  // columns from n8 on stay zero
      *reinterpret_cast<float4*>(&lds[at + ct * 16]) =
          make_float4(col < g.N ? s0 : -INFINITY, col + 1 < g.N ? s1 : -INFINITY, col + 2 < g.N ? s2 : -INFINITY,
                      col + 3 < g.N ? s3 : -INFINITY);
    if (!L2 && write_pos && row >= col && row < col + 4) {
      const int r = row - col;
      lds[pos_at + row] = r == 0 ? acc[ct][0] : (r == 1 ? acc[ct][1] : (r == 2 ? acc[ct][2] : acc[ct][3]));
    }
  }
}

// Persistent kernel: workgroup b takes chunks b, b + gridDim.x, ...  Waves 0..7
// ("compute") issue the matrix products; waves 8..15 ("helpers") do everything else
// -- row ids and sort keys, the gather, the loss, the fold -- while the products of
// another block run, between the same sequence of barriers:
//
//   step  compute waves (MFMA)                         helper waves
//   1     S_0 = X1pos X0^T                             ids + sort keys of the next chunk; l2: positive scores
//   2     S_1 = X0pos X1^T                             loss of side 0: S_0 -> dS_0 in place
//   3     uniform negatives of side 0: dS_0[:,P:]^T X1pos -> HBM      loss of side 1; l2: column sums of dS_0[:, :P]
//   4     uniform negatives of side 1: dS_1[:,P:]^T X0pos -> HBM      statistics; l2: column sums of dS_1[:, :P]; fold
//   5     positives of side 0: [G | dS_1[:,P:]] X1 -> HBM             issue the next chunk's row loads
//   6     positives of side 1: [G^T | dS_0[:,P:]] X0 -> HBM           dot: write the next chunk's side-1 rows (free now)
//   7     -                                            write the rest of the next chunk's rows
//
// A step's 4 row tiles x T column tiles are split over the 8 compute waves as
// (row tile, first ceil(T/2) or last floor(T/2) column tiles), two waves per SIMD,
// so every SIMD carries T tiles per step.

//
// LD != 0: both LDS row strides (operand rows, score rows) equal LD, known at compile
// time, so that the products' LDS addresses are one register plus immediates.
template <int T, int CMP, int LOSS, int LD, bool HALF>
__global__ __launch_bounds__(2 * kFusedThreads) void fused_chunk_kernel(StepCtx c, FusedLayout f, int num_chunks) {
  // All LDS accesses index `lds` directly (no pointer tables), so that they
  // compile to ds_read / ds_write rather than flat accesses.  Everything indexed
  // by the wave number or by a side reaches the kernel arguments through scalar
  // registers (readfirstlane) or selects: a per-lane index into an argument
  // array turns into a global load.
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr bool l2 = CMP == PBG_CMP_L2;
  // cos: a gradient row goes back through the normalisation, dz = (dy - y <y, dy>) / norm, and the
  // row is spread over the two waves that share its row tile: they exchange their shares of
  // <y, dy> through LDS, one more barrier per product, which the helpers keep as well.
  constexpr bool cosn = CMP == PBG_CMP_COS;
  constexpr int T0 = (T + 1) / 2, T1 = T - T0;
  constexpr int kLossCols = 2 * T;  // score columns per lane of the 8 lanes that share a row
  const int lane = threadIdx.x & 63;
  const int wave16 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave = wave16 & 7, tid = threadIdx.x & (kFusedThreads - 1);
  FusedGeom g;
  g.D = c.D; g.P = c.P; g.U = c.U; g.N = c.P + c.U; g.ldx = LD ? LD : f.ldx; g.lds = LD ? LD : f.lds;
  g.xn0 = f.xn[0]; g.xn1 = f.xn[1];  // operand rows of side 0 / 1: [N][ldx]
  g.sc0 = f.sc[0]; g.sc1 = f.sc[1];  // score rows against side 0 / 1's negatives: [P][lds]
  g.sq0 = f.sq[0]; g.sq1 = f.sq[1]; g.rs0 = f.rs[0]; g.rs1 = f.rs[1]; g.cs0 = f.cs[0]; g.cs1 = f.cs[1];
  const int D = g.D, P = g.P, U = g.U, N = g.N, ldx = g.ldx, lds_ = g.lds, CP = c.C * c.P;
  const int xn0 = g.xn0, xn1 = g.xn1, sc0 = g.sc0, sc1 = g.sc1;
  int* ids = reinterpret_cast<int*>(lds + f.ids);

  if (wave16 >= 8) {
    // ================= helper role =================
    // The helpers' few instructions go first wherever a SIMD has to choose: behind
    // the compute waves' back-to-back matrix instructions they would wait for most
    // of a step, and every step ends when its slower role does.
    __builtin_amdgcn_s_setprio(3);
    float4 v[kFusedRounds];
    int idv[kFusedRounds];
    FusedRowExtras extras;
    const int C = c.C;
    {
      const int k0 = (int)blockIdx.x / C;
      fused_load_ids(c, g, blockIdx.x, k0, (int)blockIdx.x - k0 * C, tid, ids);
      lds_barrier();  // ids visible; the compute waves have cleared the storage behind the operand rows
      fused_issue_rows(c, g, ids, clamp_index(c.rel[k0], c.num_relations), wave, lane, v, idv, &extras, true);
    }
    bool side1_stored = false;  // the side-1 rows of chunk kc are in LDS already
    bool pads = c.last < P && (int)blockIdx.x % C == C - 1;  // the chunk whose rows are in the registers has padded positives
    for (int kc = blockIdx.x; kc < num_chunks; kc += gridDim.x) {
      // The thread-to-cell mapping is the same for every chunk; hiding the thread's
      // indices from the optimiser once per chunk keeps it from hoisting every
      // address of the loop body into registers that stay live (and spill).
      int ln = lane, t = tid;
      asm volatile("" : "+v"(ln), "+v"(t));
      // ---- step 7 of the previous chunk ----
      fused_store_side<CMP, 0, HALF>(c, g, lds, wave, ln, v, idv, extras, pads);
      if (!side1_stored) fused_store_side<CMP, 1, HALF>(c, g, lds, wave, ln, v, idv, extras, pads);
      lds_barrier();  // (a) operand rows of chunk kc in LDS

      const int kn = kc + gridDim.x;
      const bool more = kn < num_chunks;
      const int k = kc / C, cc = kc - k * C;
      const int k_next = more ? kn / C : k, cc_next = more ? kn - k_next * C : cc;
      const int valid = (cc == C - 1) ? c.last : P;
      const int64_t rel = clamp_index(c.rel[k], c.num_relations);
      const int64_t rel_next = clamp_index(c.rel[k_next], c.num_relations);
      // the loss weight of this thread's edge (eight lanes per edge): asked for now, used in steps 2 and 3
      float w_edge = c.rel_weights[rel];
      if (c.edge_weight) w_edge *= c.edge_weight[(int64_t)k * c.B + min(cc * P + (t >> 3), c.B - 1)];

      // ---- step 1 ----
      if (more) fused_load_ids(c, g, kn, k_next, cc_next, t, ids);
      if (l2 && t < 4 * P) {  // positive scores in the direct form (model.py:267-274)
        const int i = t >> 2, qd = t & 3;
        float acc = 0.f;
        for (int d0 = qd; d0 < D; d0 += 32) {  // eight columns of both rows in flight
          float a[8], b[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int d = min(d0 + 4 * u, D - 1);
            a[u] = lds[xn0 + i * ldx + d];
            b[u] = lds[xn1 + i * ldx + d];
          }
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (d0 + 4 * u < D) acc += (a[u] - b[u]) * (a[u] - b[u]);
        }
        acc = quad_sum(acc);
        if (qd == 0) lds[f.pos + i] = -sqrtf(fmaxf(acc, 1e-30f));
      }
      lds_barrier();  // (b) S_0 and the positive scores are there

      // ---- steps 2 and 3: loss of side 0, then of side 1; eight lanes per edge, columns interleaved ----
      for (int s = 0; s < 2; ++s) {
        if (t < 8 * P) {
          const int i = t >> 3, qd = t & 7;
          const int row_at = (s ? sc1 : sc0) + i * lds_;
          float loss_w = 0.f, dpos_s = 0.f, rowsum = 0.f;
          int viol = 0;
          if (i >= valid) {  // padded positive: no loss, zero gradient rows
            for (int j = qd; j < lds_; j += 8) lds[row_at + j] = 0.f;
          } else {
            // The masks (model.py:566-580,836-839) go into the row before it is read: the i-th batch
            // negative is the positive's own entity, and in a partial last chunk the batch
            // negatives from `valid` on are padding.  A lane only ever reads its own columns,
            // so its own writes are all it has to wait for.
            const float masked = l2 ? -INFINITY : -1e9f;
            if (qd == (i & 7)) lds[row_at + i] = masked;
            if (valid < P)
              for (int j = valid + ((qd - valid) & 7); j < P; j += 8) lds[row_at + j] = masked;
            fused_row_loss<CMP, LOSS, kLossCols, HALF>(lds, row_at, s ? g.sq1 : g.sq0, l2 ? lds[(s ? g.sq0 : g.sq1) + i] : 0.f,
                                                   c.margin, 1.0f / (float)N, (N + 7) >> 3, lds[f.pos + i], w_edge, qd, &loss_w,
                                                   &dpos_s, &viol, &rowsum);
          }
          if (qd == 0) {
            lds[(s ? g.rs1 : g.rs0) + i] = rowsum;
            lds[f.part + (s * 3 + 0) * P + i] = dpos_s;
            lds[f.part + (s * 3 + 1) * P + i] = loss_w;
            lds[f.part + (s * 3 + 2) * P + i] = __int_as_float(viol);
          }
        }
        if (l2 && s == 1) {  // column sums of dS_0[:, :P] (stored as -2 dLoss/dq), complete since barrier (c)
          for (int j = t; j < P; j += kFusedThreads) {
            float acc = 0.f;
            for (int i = 0; i < P; ++i) acc += lds[sc0 + i * lds_ + j];
            lds[g.cs0 + j] = acc;
          }
        }
        if (cosn && s == 1) lds_barrier();  // the exchange of step 3
        lds_barrier();  // (c) after side 0, (d) after side 1
      }

      // ---- step 4: statistics out, fold ----
      if (t < P) {  // both sides of an edge together
        const int64_t job = (int64_t)k * CP + cc * P + t;
        const float dpos = lds[f.part + 0 * P + t] + lds[f.part + 3 * P + t];
        c.lossrow[job] = lds[f.part + 1 * P + t] + lds[f.part + 4 * P + t];
        c.violrow[job * 2] = __float_as_int(lds[f.part + 2 * P + t]);
        c.violrow[job * 2 + 1] = __float_as_int(lds[f.part + 5 * P + t]);
        if (l2) lds[f.dpos + t] = dpos;
      }
      if (l2) {
        for (int j = t; j < P; j += kFusedThreads) {
          float acc = 0.f;
          for (int i = 0; i < P; ++i) acc += lds[sc1 + i * lds_ + j];
          lds[g.cs1 + j] = acc;
        }
        lds_barrier();  // (e') the column sums read the blocks that the fold below rewrites
      }
      // Both score blocks carry a P x P part against the batch negatives, and the
      // batch negatives of one side are the positives of that side: the gradient of
      // positive row i of the lhs is  sum_j dS_R[i][j] rhs_j + sum_j dS_L[j][i] rhs_j,
      // so the two parts fold into G = dS_R[:, :P] + dS_L[:, :P]^T (and G^T for the
      // rhs rows), kept in place, and steps 5 and 6 need one product per row block.
      {
        int i = t / P, j = t - i * P;  // element t, t + 512, ... of the P x P block, walked without further divisions
        const int di = kFusedThreads / P, dj = kFusedThreads - di * P;
        for (int e = t; e < P * P; e += kFusedThreads) {
          float sum = lds[sc1 + i * lds_ + j] + lds[sc0 + j * lds_ + i];
          // dot: dLoss/dpos_i goes onto the (masked, so far zero) diagonal: the i-th batch
          // negative of the rhs side is the i-th positive's own rhs row, so the products
          // of steps 5 and 6 then carry dpos_i * rhs_i into the lhs gradient and
          // dpos_i * lhs_i into the rhs one.
          if (!l2 && i == j) sum += lds[f.part + 0 * P + i] + lds[f.part + 3 * P + i];
          // (HALF: the folded block is an operand of the fp16 products; the sum of its two or three terms is
          // rounded here, one rounding where autograd's float16 additions make two)
          if (HALF) sum = half_round(sum);
          lds[sc1 + i * lds_ + j] = sum;
          lds[sc0 + j * lds_ + i] = sum;
          i += di;
          j += dj;
          if (j >= P) {
            j -= P;
            ++i;
          }
        }
      }
      if (cosn) lds_barrier();  // the exchange of step 4
      lds_barrier();  // (e)

      // ---- step 5: the next chunk's rows into registers; they have two products' time to arrive ----
      fused_issue_rows(c, g, ids, rel_next, wave, ln, v, idv, &extras, more);
      if (cosn) lds_barrier();  // the exchange of step 5
      lds_barrier();  // (f) the products no longer read the side-1 rows (dot)

      // ---- step 6 ----
      side1_stored = CMP == PBG_CMP_DOT && more;  // (l2 and cos still read the rows' own values while writing gradients out)
      pads = c.last < P && cc_next == C - 1;  // of the chunk whose rows are in the registers now
      if (side1_stored) fused_store_side<CMP, 1, HALF>(c, g, lds, wave, ln, v, idv, extras, pads);
      if (cosn) lds_barrier();  // the exchange of step 6
      lds_barrier();  // (g) the products have let go of all operand rows
    }
    return;
  }

  // ================= compute role =================
  for (int t = tid * 4; t < f.ids; t += kFusedThreads * 4)  // operand rows (their pad columns and slack rows stay zero), score blocks, small arrays
    *reinterpret_cast<float4*>(&lds[t]) = make_float4(0.f, 0.f, 0.f, 0.f);
  lds_barrier();
  // Pad rows and pad columns of the score blocks are never written again, and
  // every other cell is rewritten by each chunk before it is read.

  const int rt = wave & 3;                     // row tile of this wave in every product
  const int grp = wave >> 2;                   // 0: column tiles [0, T0), 1: [T0, T)
  const int ct0 = grp ? T0 : 0;
  for (int kc = blockIdx.x; kc < num_chunks; kc += gridDim.x) {
    const int k = kc / c.C, cc = kc - k * c.C;
    const int valid = (cc == c.C - 1) ? c.last : P;
    const int64_t rel = clamp_index(c.rel[k], c.num_relations);
    int lane_ = threadIdx.x & 63;  // opaque per chunk, see the helper loop
    asm volatile("" : "+v"(lane_));
    const int m16 = lane_ & 15, kq = lane_ >> 4;
    lds_barrier();  // (a)

    // ---- steps 1 and 2: the score blocks ----
    for (int s = 0; s < 2; ++s) {
      if (grp == 0) fused_scores<T0, l2, HALF>(lds, g, s, rt, 0, lane_, f.pos, s == 0);
      else if (T1 > 0) fused_scores<(T1 > 0 ? T1 : 1), l2, HALF>(lds, g, s, rt, T0, lane_, f.pos, s == 0);
      lds_barrier();  // (b), (c)
    }

    // ---- steps 3 and 4: uniform negatives of side m: (dS_m[:, P:])^T (U x P) times the other side's positives ----
    for (int m = 0; m < 2; ++m) {
      const SideCtx& sd = c.side[m];
      const int dsn = m ? sc1 : sc0, bx = m ? xn0 : xn1, xs = m ? xn1 : xn0;
      const bool has_op = m == 1 && c.op != PBG_OP_NONE;
      const bool live = rt * 16 < U && ct0 * 16 < D;
      float4v acc[T0];
#pragma unroll
      for (int ct = 0; ct < T0; ++ct) acc[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
      float asum = 0.f;
      if (live) {
        const int au = min(rt * 16 + m16, U - 1);
        const int a_at = dsn + P + au, b_at = bx + ct0 * 16, pk = (P + 3) >> 2;
        if (grp == 0) asum = sweep_a_cols<T0, HALF>(lds, a_at, lds_, b_at, ldx, kq, m16, pk, acc);
        else if (T1 > 0) asum = sweep_a_cols<(T1 > 0 ? T1 : 1), HALF>(lds, a_at, lds_, b_at, ldx, kq, m16, pk, acc);
      }
      if (l2 && m == 1) lds_barrier();  // (e') of the helpers
      const int u = rt * 16 + m16;
      float row_dot_ = 0.f;
      if (cosn) {
        const int self_at = xs + (P + min(u, U - 1)) * ldx + ct0 * 16, left = D - ct0 * 16;
        float part = 0.f;
        if (live) {
          if (grp == 0) for_each_out<T0>(acc, kq, [&](int col, float4 v4) { fused_self_dot<HALF>(lds, self_at, col, left, v4, &part); });
          else if (T1 > 0) for_each_out<(T1 > 0 ? T1 : 1)>(acc, kq, [&](int col, float4 v4) { fused_self_dot<HALF>(lds, self_at, col, left, v4, &part); });
        }
        part += __shfl_xor(part, 16);
        part += __shfl_xor(part, 32);
        if (kq == 0) lds[f.xch + grp * 64 + rt * 16 + m16] = part;
        lds_barrier();
        row_dot_ = part + lds[f.xch + (1 - grp) * 64 + rt * 16 + m16];
      }
      if (live && u < U) {
        const int r2 = cc * U + u;
        FusedOut o;
        o.out = c.gr + ((int64_t)k * c.rk + sd.slot_uni + r2) * D + ct0 * 16;
        o.dz = (has_op && sd.dz) ? sd.dz + ((int64_t)k * sd.op_rows + c.B + r2) * D + ct0 * 16 : nullptr;
        o.par = (has_op && c.op == PBG_OP_DIAGONAL) ? sd.p0 + rel * D + ct0 * 16 : nullptr;
        o.self_at = xs + (P + u) * ldx + ct0 * 16;
        o.other_at = o.self_at;
        o.pcoef = 0.f;
        o.coef = 0.f;
        if (l2) {  // minus the column sum of the stored -2 dLoss/dq: the lane's share, then the other three k slots'
          asum += __shfl_xor(asum, 16);
          asum += __shfl_xor(asum, 32);
          o.coef = -asum;
        }
        if (cosn) {
          o.coef = row_dot_;
          o.pcoef = lds[(m ? g.sq1 : g.sq0) + P + u];
        }
        const int left = D - ct0 * 16;
        if (grp == 0) for_each_out<T0>(acc, kq, [&](int col, float4 v4) { fused_emit<CMP, HALF>(lds, o, col, left, v4); });
        else if (T1 > 0) for_each_out<(T1 > 0 ? T1 : 1)>(acc, kq, [&](int col, float4 v4) { fused_emit<CMP, HALF>(lds, o, col, left, v4); });
      }
      lds_barrier();  // (d), (e)
    }

    // ---- steps 5 and 6: positives of side m: [G | dS_a[:, P:]] (P x N) times the other side's N rows ----
    for (int m = 0; m < 2; ++m) {
      const SideCtx& sd = c.side[m];
      const int dsa = m ? sc0 : sc1;  // scores in which this side's positives were the A operand
      const int bx = m ? xn0 : xn1, xs = m ? xn1 : xn0;
      const int rs_o = m ? g.rs0 : g.rs1, cs_m = m ? g.cs1 : g.cs0;
      const bool has_op = m == 1 && c.op != PBG_OP_NONE;
      const bool live = rt * 16 < P && ct0 * 16 < D;
      float4v acc[T0];
#pragma unroll
      for (int ct = 0; ct < T0; ++ct) acc[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
      if (live) {
        // The k index runs past N up to the next multiple of 4: the score blocks keep
        // zero pad columns there, so those terms vanish.
        const int ar = min(rt * 16 + m16, P - 1);
        const int ksteps = (N + 3) >> 2;
        const int a_at = dsa + ar * lds_, b_at = bx + ct0 * 16;
        if (grp == 0) sweep_a_rows<T0, HALF>(lds, a_at, b_at, ldx, kq, m16, ksteps >> 2, ksteps & 3, acc);
        else if (T1 > 0) sweep_a_rows<(T1 > 0 ? T1 : 1), HALF>(lds, a_at, b_at, ldx, kq, m16, ksteps >> 2, ksteps & 3, acc);
      }
      float row_dot_ = 0.f;
      if (cosn) {
        const int self_at = xs + min(rt * 16 + m16, P - 1) * ldx + ct0 * 16, left = D - ct0 * 16;
        float part = 0.f;
        if (live) {
          if (grp == 0) for_each_out<T0>(acc, kq, [&](int col, float4 v4) { fused_self_dot<HALF>(lds, self_at, col, left, v4, &part); });
          else if (T1 > 0) for_each_out<(T1 > 0 ? T1 : 1)>(acc, kq, [&](int col, float4 v4) { fused_self_dot<HALF>(lds, self_at, col, left, v4, &part); });
        }
        part += __shfl_xor(part, 16);
        part += __shfl_xor(part, 32);
        if (kq == 0) lds[f.xch + grp * 64 + rt * 16 + m16] = part;
        lds_barrier();
        row_dot_ = part + lds[f.xch + (1 - grp) * 64 + rt * 16 + m16];
      }
      if (live) {
        const int i = rt * 16 + m16;
        if (i < valid) {
          const int q = cc * P + i;
          FusedOut o;
          o.out = c.gr + ((int64_t)k * c.rk + sd.slot_pos + q) * D + ct0 * 16;
          o.dz = (has_op && sd.dz) ? sd.dz + ((int64_t)k * sd.op_rows + q) * D + ct0 * 16 : nullptr;
          o.par = (has_op && c.op == PBG_OP_DIAGONAL) ? sd.p0 + rel * D + ct0 * 16 : nullptr;
          o.self_at = xs + i * ldx + ct0 * 16;
          o.other_at = bx + i * ldx + ct0 * 16;
          o.coef = 0.f;
          o.pcoef = 0.f;
          if (l2) {
            const float dpz = lds[f.dpos + i], pz = lds[f.pos + i];
            o.coef = 2.0f * lds[rs_o + i] - lds[cs_m + i];
            o.pcoef = pz * pz > 2e-30f ? dpz / pz : 0.f;
          }
          if (cosn) {
            o.coef = row_dot_;
            o.pcoef = lds[(m ? g.sq1 : g.sq0) + i];
          }
          const int left = D - ct0 * 16;
          if (grp == 0) for_each_out<T0>(acc, kq, [&](int col, float4 v4) { fused_emit<CMP, HALF>(lds, o, col, left, v4); });
          else if (T1 > 0) for_each_out<(T1 > 0 ? T1 : 1)>(acc, kq, [&](int col, float4 v4) { fused_emit<CMP, HALF>(lds, o, col, left, v4); });
        }
      }
      lds_barrier();  // (f), (g)
    }
  }
}

// One thread per operand-row slot of every chunk (kFusedIds per chunk, see fused_load_ids): the slot's
// row id (-1: a slot past the operand rows or a padded position of the last chunk) and, for real
// slots, the sort key and value of the slot's gradient row.  Nothing here depends on the
// embeddings, so the sort of the keys can run beside the chunk kernel.
__global__ __launch_bounds__(kFusedIds) void fused_ids_kernel(StepCtx c) {
  const int kc = blockIdx.x, t = threadIdx.x;
  const int P = c.P, U = c.U, N = P + U;
  const int k = kc / c.C, cc = kc - k * c.C;
  const int s = t >> 7, j = t & (kFusedSide - 1);
  const SideCtx& sd = c.side[s];
  const bool is_pos = j < P;
  const int q = cc * P + j, u = min(max(j - P, 0), U - 1);
  const bool real = j < N && (!is_pos || q < c.B);
  const int64_t flat = (int64_t)kc * U + u;
  int64_t id = is_pos ? sd.idx[(int64_t)k * c.B + min(q, c.B - 1)] : uniform_negative(sd, s, flat);
  id = clamp_index(id, sd.num_rows);
  if (real) {
    const int64_t pair = (int64_t)k * c.rk + (is_pos ? sd.slot_pos + q : sd.slot_uni + cc * U + u);
    c.keys[pair] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
    c.vals[pair] = (uint32_t)pair;
  }
  c.fused_rowid[(int64_t)kc * kFusedIds + t] = real ? (int)id : -1;
}

// One instantiation of the fused kernel per (tile count, comparator, loss, half precision); each
// raises its dynamic LDS limit the first time it needs more than it was given.
template <int T, int CMP, int LOSS, int LD, bool HALF>
int launch_fused_as(const StepCtx& c, const FusedLayout& fl, size_t lds_bytes, hipStream_t s, int blocks) {
  static LdsLimit limit;
  const int rc = reserve_lds((const void*)fused_chunk_kernel<T, CMP, LOSS, LD, HALF>, &limit, lds_bytes);
  if (rc != PBG_OK) return rc;
  const int chunks = c.K * c.C;
  hipLaunchKernelGGL((fused_chunk_kernel<T, CMP, LOSS, LD, HALF>), dim3((unsigned)blocks), dim3(2 * kFusedThreads), lds_bytes,
                     s, c, fl, chunks);
  return PBG_OK;
}

template <int T, int CMP, int LD, bool HALF>
int launch_fused_loss(const StepCtx& c, const FusedLayout& fl, size_t lds_bytes, hipStream_t s, int blocks) {
  switch (c.loss) {
    case PBG_LOSS_RANKING: return launch_fused_as<T, CMP, PBG_LOSS_RANKING, LD, HALF>(c, fl, lds_bytes, s, blocks);
    case PBG_LOSS_LOGISTIC: return launch_fused_as<T, CMP, PBG_LOSS_LOGISTIC, LD, HALF>(c, fl, lds_bytes, s, blocks);
    default: return launch_fused_as<T, CMP, PBG_LOSS_SOFTMAX, LD, HALF>(c, fl, lds_bytes, s, blocks);
  }
}

template <int T, int LD>
int launch_fused_cmp(const StepCtx& c, const FusedLayout& fl, size_t lds_bytes, hipStream_t s, int blocks) {
  if (c.half) {  // (dot and cos only: the step's validation has refused the rest)
    if (c.cmp == PBG_CMP_COS) return launch_fused_loss<T, PBG_CMP_COS, LD, true>(c, fl, lds_bytes, s, blocks);
    if (c.cmp == PBG_CMP_DOT) return launch_fused_loss<T, PBG_CMP_DOT, LD, true>(c, fl, lds_bytes, s, blocks);
    return fail(PBG_ERR_UNSUPPORTED, "step: half_precision on the fused route is built for dot and cos");
  }
  switch (c.cmp) {
    case PBG_CMP_L2: return launch_fused_loss<T, PBG_CMP_L2, LD, false>(c, fl, lds_bytes, s, blocks);
    case PBG_CMP_COS: return launch_fused_loss<T, PBG_CMP_COS, LD, false>(c, fl, lds_bytes, s, blocks);
    default: return launch_fused_loss<T, PBG_CMP_DOT, LD, false>(c, fl, lds_bytes, s, blocks);
  }
}

}  // namespace

bool fused_layout(const StepCtx& c, FusedLayout* f) {
  f->sliced = 0;
  if (c.dynamic) return false;
  // complex_diagonal: on slices only (pairs of coordinates, see sliced_chunk_kernel; a single slice up to dim 128), with dot
  const bool cplx = c.op == PBG_OP_COMPLEX_DIAGONAL;
  if (cplx && (c.D % 8 != 0 || c.cmp != PBG_CMP_DOT)) return false;
  if (c.op != PBG_OP_NONE && c.op != PBG_OP_TRANSLATION && c.op != PBG_OP_DIAGONAL && !cplx) return false;
  if (c.cmp != PBG_CMP_DOT && c.cmp != PBG_CMP_L2 && c.cmp != PBG_CMP_COS) return false;
  if (c.D % 4 != 0 || c.P > 64 || c.U > 64) return false;
  // rows wider than 128 floats pass through LDS in slices (sliced_chunk_kernel): fp32
  const bool sliced = c.D > 128 || cplx;
  if (sliced && getenv("PBG_DISABLE_SLICED") != nullptr)
    return false;
  if (c.side[0].num_rows >= ((int64_t)1 << 31) || c.side[1].num_rows >= ((int64_t)1 << 31)) return false;
  for (int s = 0; s < 2; ++s)
    if (c.side[s].nb != c.P || c.side[s].u != c.U) return false;
  const int N = c.P + c.U;
  f->sliced = sliced;
  f->ldx = lds_stride(sliced ? kSliceCols : c.D);
  f->lds = lds_stride((N + 7) / 8 * 8);  // the loss reads whole groups of 8 columns
  int off = 0;
  auto take = [&](int count) { int o = off; off += (count + 3) / 4 * 4; return o; };
  const int p4 = (c.P + 3) / 4 * 4;
  f->xn[0] = take(N * f->ldx);
  f->xn[1] = take(N * f->ldx + 4 * f->ldx);  // slack: k-steps and column tiles may read past the last row
  f->sc[0] = take(p4 * f->lds);              // pad rows and pad columns stay zero
  f->sc[1] = take(p4 * f->lds + 4 * f->lds);
  for (int s = 0; s < 2; ++s) f->sq[s] = take(N);
  for (int s = 0; s < 2; ++s) f->rs[s] = take(c.P);
  for (int s = 0; s < 2; ++s) f->cs[s] = take(N);
  f->pos = take(c.P);
  f->dpos = take(c.P);
  f->part = take(6 * c.P);
  f->xch = take(c.cmp == PBG_CMP_COS && !sliced ? 128 : 0);
  f->ids = take(kFusedIds);
  f->total = off;
  return (size_t)off * sizeof(float) <= 160 * 1024 - 512;
}

int fused_ids(const StepCtx& c, hipStream_t s) {
  if (!c.fused_rowid) return fail(PBG_ERR_INVALID, "step: the fused route's row ids have no place to go");
  hipLaunchKernelGGL(fused_ids_kernel, dim3((unsigned)(c.K * c.C)), dim3(kFusedIds), 0, s, c);
  return PBG_OK;
}

int fused_chunks(const StepCtx& c, const FusedLayout& fl, int blocks, hipStream_t s) {
  const size_t lds_bytes = (size_t)fl.total * sizeof(float);
  if (fl.sliced) return sliced_chunks(c, fl, blocks, s);
  const bool small_tiles = c.P + c.U <= 112 && c.D <= 112;
  // dim 100 with 50 + 50 negatives (and everything else whose two row strides come out as 104 floats)
  if (small_tiles && fl.ldx == 104 && fl.lds == 104) return launch_fused_cmp<7, 104>(c, fl, lds_bytes, s, blocks);
  if (small_tiles) return launch_fused_cmp<7, 0>(c, fl, lds_bytes, s, blocks);
  return launch_fused_cmp<8, 0>(c, fl, lds_bytes, s, blocks);
}

}  // namespace pbg
