// The streaming route of the training step, for chunks whose negatives do not fit
// LDS next to their positives (hundreds or thousands of uniform negatives per
// chunk, model.py:508-622 with num_uniform_negs large): dot comparator, operator
// none / diagonal / complex_diagonal, every loss.  (The cos comparator without an
// operator takes these kernels too: the caller hands them a normalised copy of the
// tables and undoes the normalisation where it applies the gradients.)
//
// A work item is (chunk, side s): the chunk's P positives against side s's
// P + U negatives (the chunk's own side-s rows, then its uniform draws).  The
// positives' operand rows A (P x D, prepared once per edge by stream_prep_kernel)
// stay in LDS for the whole item; the negatives pass through LDS in tiles of 32
// RAW table rows, gathered by id, twice:
//
//   sweep 1   S_t = A N_t^T per tile; masks, the loss's row statistics (running
//             maximum and sum of exponentials, hinge sums, violators), S_t parked in
//             a scratch area that each thread reads back itself
//   sweep 2   G_t = dLoss/dS_t from the parked scores and the finished statistics;
//             dA += G_t N_t (kept in registers over the whole sweep) and
//             dN_t = G_t^T A, written straight to the gradient rows
//
// so neither the operated negatives nor the score matrix nor dLoss/dS ever exist in
// HBM, and a negative's gradient row is written once, in its final form.
//
// The negatives stay raw because the operator is moved to the other operand:
// <a, op(x)> = <op^T(a), x> for the linear operators handled here (diagonal: the
// same scaling; complex_diagonal: multiplication by the conjugate).  The item of
// the operator's own side therefore scores op^T(other side's positive) against raw
// rows, the gradient of a raw negative is G^T A as it stands, and the operator's
// parameter gradient comes from the positives' rows alone (stream_finish_kernel).
// The positive pair's score is computed per edge beforehand, as the model does
// (model.py:177); its gradient rides on the diagonal of the batch-negative block
// (column i of row i is the edge's own partner row), so the two products of sweep 2
// carry it into both rows of the pair.
//
// Roles inside the workgroup, between the same LDS-only barriers: waves 0..7 issue
// the matrix products, waves 8..15 gather the next tile into registers, compute
// ids and sort keys, and do the loss arithmetic of the neighbouring tile.
#include "stream.h"

#include <cstring>

#include "mfma_tiles.h"

namespace pbg {
namespace {

constexpr int kTile = 32;                    // negatives per tile
// LDS timing on this chip, measured with the SQ_LDS_* counters on one access pattern at a time:
//   ds_read_b128 runs in 4 passes of 16 lanes -- lanes {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and
//   the same sets + 32 -- and a pass costs one cycle per distinct address in its busiest group of
//   banks, 16 groups of 16 bytes (address / 16 mod 16): 4 cycles at best;
//   ds_read_b32 runs in 2 passes (lanes 0-31, 32-63) over 32 banks of 4 bytes: 2 cycles at best.
// For the MFMA operand reads below (lane = 16 kq + m):
//   "16 rows x one 128-bit word at 4 kq" (k along the row) is conflict-free iff the row stride is
//   8 mod 16 floats; "row kq, word at 4 m" iff the rows of kq and kq + 1 are a multiple of 64 floats
//   apart; "row kq, float at m" iff they are 16 mod 32 floats apart.  The row strides and the
//   assignment of k values to the four k slots of a matrix instruction (any assignment is right as
//   long as both operands use the same one) are chosen to meet these.
constexpr int kLdg = 40;                     // row stride of a 64 x 32 score tile in LDS
// Column k of a tile of dLoss/dS sits at float swap23(k) of its LDS row (bits 2 and 3 of k exchanged): the
// word a lane of the dA product needs -- k = 8 kq + 4 h + (0..3), see stream_da_part -- then lies at
// 16 (kq >> 1) + 4 (kq & 1) + 8 h, an odd number of words from its pass partner's.
__device__ __forceinline__ int swap23(int k) { return (k & ~12) | ((k & 4) << 1) | ((k & 8) >> 1); }
constexpr int kTileFloats = 64 * kLdg;
constexpr int kHelpers = 512;                // threads of the helper role
constexpr int kSlack = 8 * kLdg;             // the products' operand reads run a few rows past their blocks
constexpr int kRowThreads = 256;
constexpr int kWavesPerBlock = kRowThreads / kWave;

// ---------------------------------------------------------------------------
// per-edge preparation
// ---------------------------------------------------------------------------
// One wave per (batch, side, position): the row's sort key, the operand row it
// contributes to the OTHER side's item, and the positive score.
//   standard mode, side 1 (rhs): op(x) -> item 0;   side 0 (lhs): op^T(x) -> item 1
//   dynamic relations: this side's own operator of the edge's relation (model.py:722-754)
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void stream_prep_kernel(StepCtx c, StreamPlan a) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (job >= (int64_t)c.K * 2 * c.B) return;
  const int k = (int)(job / (2 * c.B));
  int r = (int)(job % (2 * c.B));
  const int s = r >= c.B;
  if (s) r -= c.B;
  const SideCtx& sd = c.side[s];
  const SideCtx& so = c.side[1 - s];
  const int D = c.D, H = (D + 1) / 2;
  const int64_t e = (int64_t)k * c.B + r;
  const int64_t id = clamp_index(sd.idx[e], sd.num_rows);
  const int64_t rel = clamp_index(c.dynamic ? c.rel[e] : c.rel[k], c.num_relations);
  const RowV<NVH> x = row_load<NVH>(sd.w + id * D, D, H, lane);
  if (lane == 0) {
    const int64_t slot = (int64_t)k * c.rk + sd.slot_pos + r;
    c.keys[slot] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
    c.vals[slot] = (uint32_t)slot;
  }
  RowV<NVH> y = x;
  if (c.op != PBG_OP_NONE) {
    if (c.dynamic || s == 1) y = op_forward<NVH>(c.op, x, sd.p0, sd.p1, rel, D, H, lane);
    else y = op_backward<NVH>(c.op, x, so.p0, so.p1, rel, D, H, lane);
  }
  row_store<NVH>((s ? a.sa[0] : a.sa[1]) + e * D, y, D, H, lane);
  if (c.dynamic || s == 1) {
    const int64_t oid = clamp_index(so.idx[e], so.num_rows);
    const RowV<NVH> other = row_load<NVH>(so.w + oid * D, D, H, lane);
    const float pos = wave_sum(row_dot(other, y));
    if (lane == 0) (s ? a.spos[0] : a.spos[1])[e] = pos;
  }
}

// ---------------------------------------------------------------------------
// the chunk kernel
// ---------------------------------------------------------------------------
// One thread per (chunk, side, column): the row id of that column of the item's negatives
// (-1: a padded position of a partial last chunk), as 32 bits in the order the chunk kernel
// walks them, and the sort key of a uniform negative's gradient row.  Drawing the ids here
// (Philox, 40 quarter-rate multiplies per id) keeps that arithmetic out of the chunk kernel,
// whose helper waves share their vector ALUs with the matrix instructions.
__global__ __launch_bounds__(256) void stream_ids_kernel(StepCtx c, StreamPlan a) {
  const int P = c.P, U = c.side[0].u, ncols = P + U;
  const int64_t per_side = (int64_t)c.K * c.C * ncols;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= 2 * per_side) return;
  const int s = t >= per_side;
  const int64_t r = t - (s ? per_side : 0);
  const int kc = (int)(r / ncols), j = (int)(r - (int64_t)kc * ncols);
  const int k = kc / c.C, cc = kc - k * c.C;
  const int valid = (cc == c.C - 1) ? c.last : P;
  const SideCtx& sd = c.side[s];
  int64_t id;
  bool real;
  if (j < P) {
    real = j < valid;
    id = sd.idx[(int64_t)k * c.B + min(cc * P + j, c.B - 1)];
  } else {
    real = true;
    id = uniform_negative(sd, s, (int64_t)kc * U + (j - P));
  }
  id = clamp_index(id, sd.num_rows);
  if (j >= P) {
    const int64_t pair = (int64_t)k * c.rk + sd.slot_uni + (int64_t)cc * U + (j - P);
    c.keys[pair] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
    c.vals[pair] = (uint32_t)pair;
  }
  (s ? a.colid[1] : a.colid[0])[r] = real ? (int)id : -1;
}

// Half a wave per 128 columns of a row, 128-bit loads, the whole tile in flight:
// half-wave h of the 16 takes rows h and h + 16.  Absent rows read row 0 (zeroed
// when stored); all loads are issued from straight-line code.
template <int NSEG>
struct TileRows {
  float4 v[2 * NSEG];
  int id0, id1;
  // the two ids of this thread's rows of the tile that starts at column j0 (-1 past the last column)
  static __device__ __forceinline__ void fetch_ids(const int* colid, int j0, int ncols, int ht, int* a0, int* a1) {
    const int hw = ht >> 5;
    const int x0 = colid[min(j0 + hw, ncols - 1)], x1 = colid[min(j0 + hw + 16, ncols - 1)];
    *a0 = j0 + hw < ncols ? x0 : -1;
    *a1 = j0 + hw + 16 < ncols ? x1 : -1;
  }
  __device__ __forceinline__ void issue(const float* w, int D, int row0, int row1, int ht) {
    const int c4 = (ht & 31) << 2;
    id0 = row0;
    id1 = row1;
    const uint32_t row_bytes = (uint32_t)D * 4u;
    const char* base = reinterpret_cast<const char*>(w);
    const char* r0 = base + (uint64_t)(uint32_t)max(id0, 0) * row_bytes;
    const char* r1 = base + (uint64_t)(uint32_t)max(id1, 0) * row_bytes;
#pragma unroll
    for (int seg = 0; seg < NSEG; ++seg) {
      const int col = min(seg * 128 + c4, D - 4);
      v[2 * seg] = *reinterpret_cast<const float4*>(r0 + col * 4);
      v[2 * seg + 1] = *reinterpret_cast<const float4*>(r1 + col * 4);
    }
  }
  // `absent`: the tile may hold absent rows (the same for the whole workgroup).  `paced`: the writes are
  // spread out in time -- a burst of LDS writes holds up every read that arrives behind it, and in the
  // second sweep those are the operand reads of a running product while the helpers have time to spare.
  __device__ __forceinline__ void store(float* lds, int n_at, int lda, int D, int ht, bool absent, bool paced = false) const {
    const int hw = ht >> 5, c4 = (ht & 31) << 2;
#pragma unroll
    for (int seg = 0; seg < NSEG; ++seg) {
      if (paced && seg > 0) __builtin_amdgcn_s_sleep(6);
      const int col = seg * 128 + c4;
      if (col < D) {
        float4 v0 = v[2 * seg], v1 = v[2 * seg + 1];
        if (absent) {
          v0 = keep_if(v0, id0 >= 0);
          v1 = keep_if(v1, id1 >= 0);
        }
        *reinterpret_cast<float4*>(&lds[n_at + hw * lda + col]) = v0;
        if (paced) __builtin_amdgcn_s_sleep(6);
        *reinterpret_cast<float4*>(&lds[n_at + (hw + 16) * lda + col]) = v1;
      }
    }
  }
};

// B operand of one k-step for NCT column tiles (k along the LDS rows, columns = embedding
// coordinates), with the 16 columns of a tile chosen so that the reads are free of bank
// conflicts: lane m = lane & 15 reads NCT consecutive floats at column NCT * m (eight lanes
// of a 128-bit read cover 32 consecutive banks), tile t taking the t-th of them.  The
// instruction's row index i = m comes back as i = 4 q + r in lane group q, register r, so
//   4 tiles: register r of tile t holds column 16 q + 4 r + t -> four 128-bit words per lane, one 64-byte run
//   2 tiles: register r of tile t holds column 8 q + 2 r + t
//   1 tile:  register r holds column 4 q + r
// NCT = 3 is a 2-tile part followed by a 1-tile part 32 columns on.
template <int NCT>
__device__ __forceinline__ void tile_b(const float* lds, int at, int m, float* b) {
  if constexpr (NCT == 4) {
    const float4 v = *reinterpret_cast<const float4*>(&lds[at + 4 * m]);
    b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
  } else if constexpr (NCT >= 2) {
    const float2 v = *reinterpret_cast<const float2*>(&lds[at + 2 * m]);
    b[0] = v.x; b[1] = v.y;
    if constexpr (NCT == 3) b[2] = lds[at + 32 + m];
  } else {
    b[0] = lds[at + m];
  }
}
// fn(column offset from the first tile's first column, four consecutive values of the lane's row)
template <int NCT, class F>
__device__ __forceinline__ void tile_out(const float4v* acc, int q, F&& fn) {
  if constexpr (NCT == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) fn(16 * q + 4 * r, make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]));
  } else if constexpr (NCT >= 2) {
    fn(8 * q, make_float4(acc[0][0], acc[1][0], acc[0][1], acc[1][1]));
    fn(8 * q + 4, make_float4(acc[0][2], acc[1][2], acc[0][3], acc[1][3]));
    if constexpr (NCT == 3) fn(32 + 4 * q, make_float4(acc[2][0], acc[2][1], acc[2][2], acc[2][3]));
  } else {
    fn(4 * q, make_float4(acc[0][0], acc[0][1], acc[0][2], acc[0][3]));
  }
}

// dA[N column tiles] += G_t N_t for the lane's row of the score tile.  The k slots of step r
// (0..7) hold k = 8 kq + r in both operands: the four rows of the tile that the lanes of a step
// read are 8 rows = a multiple of 64 floats apart, which keeps the 128-bit reads of tile_b free
// of bank conflicts.  a_at = the row's word for (kq, h = 0) (see swap23), b_at = the tile's row
// 8 kq at the wave's first column.  The work is cut into units of (up to 4 column tiles) x (2 k
// steps): two of the tile's rows feed 8 matrix instructions, the score row's four values for
// steps 4 h .. 4 h + 3 come with one 128-bit read per two units.
// Two operand sets take turns, the reads of the next unit pinned above the matrix
// instructions of the current one; LDA is known at compile time, so every address is one
// register plus an immediate.
// The operands of one unit: two of the tile's rows for up to 4 column tiles.
struct DaOperands {
  float b[2][4];
  template <int NCT, int LDA>
  __device__ __forceinline__ void load(const float* lds, int b_at, int m16) {
    tile_b<NCT>(lds, b_at, m16, b[0]);
    tile_b<NCT>(lds, b_at + LDA, m16, b[1]);
  }
  template <int NCT>
  __device__ __forceinline__ void mma(float a0, float a1, float4v* acc) const {
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[0][t], a0, acc[t], 0, 0, 0);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[1][t], a1, acc[t], 0, 0, 0);
  }
};
// All N column tiles as one pipeline of units: part p = column tiles 4 p .. 4 p + 3 (the last
// part may hold fewer), unit u of a part = steps 4 (u / 2) + 2 (u % 2) and the next.  The reads
// of the next unit -- of the next part after a part's last unit -- are pinned above the matrix
// instructions of the current one, so the wave never waits for a read that it has only just issued.
template <int N, int LDA>
__device__ __forceinline__ void stream_da_product(const float* lds, int a_at, int b_at, int m16, float4v* acc) {
  constexpr int full = N / 4, rem = N % 4, parts = full + (rem > 0 ? 1 : 0);
  constexpr int upp = 2 * (kTile / 16);  // units per part
  constexpr int units = parts * upp;
  DaOperands x, y;
  auto load_unit = [&](DaOperands& ops, int idx) {
    const int part = idx / upp, u = idx % upp;
    const int at = b_at + 64 * part + (4 * (u / 2) + 2 * (u & 1)) * LDA;
    if (part < full) ops.template load<4, LDA>(lds, at, m16);
    else ops.template load<(rem > 0 ? rem : 1), LDA>(lds, at, m16);
  };
  float4 a = *reinterpret_cast<const float4*>(&lds[a_at]), an = a;
  load_unit(x, 0);
#pragma unroll
  for (int idx = 0; idx < units; ++idx) {
    DaOperands& cur = (idx & 1) ? y : x;
    DaOperands& nxt = (idx & 1) ? x : y;
    if (idx + 1 < units) {
      load_unit(nxt, idx + 1);
      if (((idx + 1) & 1) == 0) an = *reinterpret_cast<const float4*>(&lds[a_at + 8 * (((idx + 1) % upp) / 2)]);
    }
    __builtin_amdgcn_sched_barrier(0);
    const float a0 = (idx & 1) ? a.z : a.x, a1 = (idx & 1) ? a.w : a.y;
    if (idx / upp < full) cur.template mma<4>(a0, a1, acc + 4 * (idx / upp));
    else cur.template mma<(rem > 0 ? rem : 1)>(a0, a1, acc + 4 * full);
    __builtin_amdgcn_sched_barrier(0);
    if (idx & 1) a = an;
  }
}
// `cols`: the row's columns from dst on (ALL: every column the tiles cover exists)
template <int N, bool ALL>
__device__ __forceinline__ void stream_da_store(const float4v* acc, int kq, float* dst, int cols) {
  constexpr int full = N / 4, rem = N % 4;
#pragma unroll
  for (int p = 0; p < full; ++p)
    tile_out<4>(acc + 4 * p, kq, [&](int col, float4 v) {
      if (ALL || 64 * p + col < cols) *reinterpret_cast<float4*>(dst + 64 * p + col) = v;
    });
  if constexpr (rem > 0)
    tile_out<rem>(acc + 4 * full, kq, [&](int col, float4 v) {
      if (ALL || 64 * full + col < cols) *reinterpret_cast<float4*>(dst + 64 * full + col) = v;
    });
}

// NCT column tiles from `ct` on of dN_t = G_t^T A for the lane's negative, stored at dst (or
// dropped).  The k slots of step r hold k = 4 r + 2 (kq & 1) + (kq >> 1): the rows that the two
// halves of a 32-lane pass read are 2 rows = 16 banks apart in both operands.  g_at = the
// negative's column of G_t in row k(0, kq), a_at = row k(0, kq) of A at column 0.
// One k step = one element of G_t's column and, per tile, one float of A's row per lane;
// two operand sets take turns as above.  Here a tile is 16 ADJACENT columns (lane m reads
// column m of each tile: 32-bit reads without bank conflicts), so that a lane's four results
// of a tile are one 128-bit word and the four lanes of a row write 64 bytes in one piece:
// these rows are the bulk of what the kernel writes to HBM, and a store instruction
// whose 16-byte pieces lie 64 bytes apart costs four times the requests.
// Reads one step past the last (the rows behind both blocks exist).
template <int NCT, int LDA, bool ALL>
__device__ __forceinline__ void stream_dn_part(const float* lds, int g_at, int a_at, int ct, int ksteps, int kq, int m16,
                                               float* dst, int cols) {
  float4v acc[NCT];
#pragma unroll
  for (int t = 0; t < NCT; ++t) acc[t] = (float4v){0.f, 0.f, 0.f, 0.f};
  a_at += ct * 16 + m16;
  float gx = lds[g_at], gy;
  float bx[NCT], by[NCT];
#pragma unroll
  for (int t = 0; t < NCT; ++t) bx[t] = lds[a_at + 16 * t];
  int ks = 0;
  for (; ks + 2 <= ksteps; ks += 2) {
    gy = lds[g_at + 4 * kLdg];
#pragma unroll
    for (int t = 0; t < NCT; ++t) by[t] = lds[a_at + 4 * LDA + 16 * t];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(bx[t], gx, acc[t], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    g_at += 8 * kLdg;
    a_at += 8 * LDA;
    gx = lds[g_at];
#pragma unroll
    for (int t = 0; t < NCT; ++t) bx[t] = lds[a_at + 16 * t];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(by[t], gy, acc[t], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (ks < ksteps) {
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(bx[t], gx, acc[t], 0, 0, 0);
  }
  if (dst) {
#pragma unroll
    for (int t = 0; t < NCT; ++t)
      if (ALL || (ct + t) * 16 + 4 * kq < cols)
        *reinterpret_cast<float4*>(dst + (ct + t) * 16 + 4 * kq) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
  }
}

// The helpers' arithmetic competes with the compute waves' matrix instructions for the
// same issue slots (fp32 matrix products run on the vector ALUs, and a wave that wants one
// vector instruction waits for a gap between another wave's matrix instructions), so the
// per-element work uses the hardware's exp2 / log2 / rcp (1 ulp) with one multiply or fma
// around them instead of the library's correctly rounded sequences.  e^(x - m) is formed as
// 2^((x - m) log2 e) with the subtraction FIRST: its relative error is then about 1e-7 |x - m|,
// nothing for the scores near the maximum that carry the sum.  (Folding the subtraction into
// one fma with -m log2 e rounds that constant to 1e-7 |m| instead, and an edge whose own
// entity is also drawn as its negative has two score-sized terms, e^(t - m) / Z and the
// positive's 1 - e^(pos - m) / Z, that must cancel to the last bits.)
constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
__device__ __forceinline__ float exp_of_difference(float x, float m) {
  return __builtin_amdgcn_exp2f((x - m) * kLog2e);
}
// sigmoid(z) and (through *softplus) softplus(z) from one exponential
__device__ __forceinline__ float fast_sigmoid(float z, float* softplus) {
  const float e = __builtin_amdgcn_exp2f(-fabsf(z) * kLog2e);
  const float r = __builtin_amdgcn_rcpf(1.0f + e);
  if (softplus) *softplus = fmaxf(z, 0.f) + __builtin_amdgcn_logf(1.0f + e) * kLn2;
  return (z >= 0.f ? 1.0f : e) * r;
}

// Statistics of one row of the score matrix, spread over the 8 threads that own the row.
template <int LOSS>
struct RowLoss {
  float m, z;     // softmax: running maximum (starts at the positive score) and sum of exp(score - m)
  float acc;      // ranking: sum of hinges; logistic: sum of softplus(score)
  float gsum;     // ranking: sum of dLoss/dscore
  __device__ __forceinline__ void start(float pos) {
    m = pos;
    z = 0.f;
    acc = 0.f;
    gsum = 0.f;
  }
  __device__ __forceinline__ void add(const float* t, float pos, float w, float margin) {
    if (LOSS == PBG_LOSS_SOFTMAX) {
      const float mn = fmaxf(fmaxf(m, t[0]), fmaxf(fmaxf(t[1], t[2]), t[3]));
      z = z * exp_of_difference(m, mn) + ((exp_of_difference(t[0], mn) + exp_of_difference(t[1], mn)) +
                                          (exp_of_difference(t[2], mn) + exp_of_difference(t[3], mn)));
      m = mn;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (LOSS == PBG_LOSS_RANKING) {
        // F.margin_ranking_loss(neg, pos, target=-1): max(0, (t - pos) + margin); the clamp
        // lets the gradient through at exactly 0
        const float x = (t[e] - pos) + margin;
        acc += fmaxf(x, 0.f);
        gsum += (x >= 0.f) ? w : 0.f;
      } else if (LOSS == PBG_LOSS_LOGISTIC) {
        float sp;
        fast_sigmoid(t[e], &sp);
        acc += sp;
      }
    }
  }
};

// Persistent kernel: workgroup b takes items b, b + gridDim.x, ...; item = 2 * chunk + side.
template <int NT, int LOSS>
__global__ __launch_bounds__(2 * kHelpers) void stream_chunk_kernel(StepCtx c, StreamPlan a, int num_items) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // The rows are NT tiles of 16 columns wide in LDS; kExact: that is the embedding dimension itself (and a
  // compile-time constant), else the last tile is partly padding that stays zero from the start of the kernel.
  constexpr int DP = NT * 16, NSEG = (DP + 127) / 128;
  constexpr bool kExact = NT == 8 || NT == 16 || NT == 25;
  constexpr int lda = lds_stride(DP);           // (= a.lda)
  const int D = kExact ? DP : c.D, D4 = D >> 2;
  // column tiles of dA per wave group: [0, T0) and [NT - T0, NT) -- with NT odd the middle tile is formed by
  // both groups (bit-identical values, one code path for the two groups)
  constexpr int T0 = (NT + 1) / 2;
  const int wave16 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave = wave16 & 7, ht = threadIdx.x & (kHelpers - 1);
  const int P = c.P, C = c.C, U = c.side[0].u, ncols = P + U, nt = a.ntiles, pr = a.pr;
  const int CP = C * P;
  float* scr = a.scratch + (size_t)blockIdx.x * nt * (kHelpers * 4) + ht * 4;
  const bool helper = wave16 >= 8;
  if (!kExact) {
    for (int i = threadIdx.x * 4; i < a.total; i += 2 * kHelpers * 4)
      *reinterpret_cast<float4*>(&lds[i]) = make_float4(0.f, 0.f, 0.f, 0.f);
    lds_barrier();
  }
  if (helper) __builtin_amdgcn_s_setprio(3);

  for (int item = blockIdx.x; item < num_items; item += gridDim.x) {
    const int kc = item >> 1, s = item & 1;
    const int k = kc / C, cc = kc - k * C;
    const int valid = (cc == C - 1) ? c.last : P;
    const SideCtx& sd = c.side[s];
    const int64_t e0 = (int64_t)k * c.B + (int64_t)cc * P;  // first edge of the chunk

    // ---- prologue, all waves: the positives' operand rows (zeros from `valid` on), ids of the first two tiles ----
    {
      const float* src = (s ? a.sa[1] : a.sa[0]) + e0 * D;
      for (int idx = threadIdx.x; idx < pr * D4; idx += 2 * kHelpers) {
        const int row = idx / D4, c4 = (idx - row * D4) * 4;
        const float4 v = *reinterpret_cast<const float4*>(src + (int64_t)min(row, valid - 1) * D + c4);
        *reinterpret_cast<float4*>(&lds[a.a_at + row * lda + c4]) = keep_if(v, row < valid);
      }
    }
    lds_barrier();  // (p1)

    if (helper) {
      // ================= helper role =================
      const int hrow = ht >> 3, hc = (ht & 7) * 4;  // this thread's row and first column inside every score tile
      const bool row_live = hrow < valid;
      const int64_t my_edge = e0 + min(hrow, valid - 1);
      const float pos = (c.dynamic && s ? a.spos[1] : a.spos[0])[my_edge];
      float w = c.rel_weights[c.dynamic ? 0 : clamp_index(c.rel[k], c.num_relations)];
      if (c.edge_weight) w *= c.edge_weight[my_edge];
      if (!row_live) w = 0.f;
      const bool has_nb = sd.nb > 0;
      const float inv_nn = 1.0f / (float)sd.nn;

      // a tile with columns that are masked or absent: the chunk's own rows, and the columns past the last negative
      auto edge_tile = [&](int tile) { return tile * kTile < P || (tile + 1) * kTile > ncols; };
      // The ids of a tile's rows are fetched one step before the rows themselves, so that
      // neither load waits for the other inside a step.
      const int* colid = (s ? a.colid[1] : a.colid[0]) + (int64_t)kc * ncols;
      TileRows<NSEG> rows;
      int nid0, nid1;
      TileRows<NSEG>::fetch_ids(colid, 0, ncols, ht, &nid0, &nid1);
      rows.issue(sd.w, D, nid0, nid1, ht);
      TileRows<NSEG>::fetch_ids(colid, nt > 1 ? kTile : 0, ncols, ht, &nid0, &nid1);
      rows.store(lds, a.n_at, lda, D, ht, true);
      lds_barrier();  // (p2) tile 0 in LDS

      RowLoss<LOSS> st;
      st.start(pos);
      // masks (model.py:566-580,836-839), then the statistics; the masked tile goes to the scratch area
      auto absorb = [&](int tile, int gbuf) {
        const float4 sv = *reinterpret_cast<const float4*>(&lds[gbuf + hrow * kLdg + hc]);
        float t[4] = {sv.x, sv.y, sv.z, sv.w};
        if (edge_tile(tile)) {
          const int j0 = tile * kTile + hc;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = j0 + e;
            if (j < P && (!has_nb || j == hrow || j >= valid)) t[e] = -1e9f;
            if (j >= ncols) t[e] = -INFINITY;
          }
        }
        *reinterpret_cast<float4*>(scr + (size_t)tile * (kHelpers * 4)) = make_float4(t[0], t[1], t[2], t[3]);
        st.add(t, pos, w, c.margin);
      };

      // ---- sweep 1 ----
      for (int q = 0; q < nt; ++q) {
        const int tn = q + 1 == nt ? 0 : q + 1, t2 = tn + 1 == nt ? 0 : tn + 1;
        rows.issue(sd.w, D, nid0, nid1, ht);  // tile tn
        TileRows<NSEG>::fetch_ids(colid, t2 * kTile, ncols, ht, &nid0, &nid1);
        if (q >= 1) absorb(q - 1, a.g_at + ((q - 1) & 1) * kTileFloats);
        lds_barrier();  // (A) S_q complete, tile q no longer read
        rows.store(lds, a.n_at, lda, D, ht, edge_tile(tn));
        lds_barrier();  // (B) tile tn in LDS
      }
      absorb(nt - 1, a.g_at + ((nt - 1) & 1) * kTileFloats);

      // ---- the row's loss and the coefficients of its gradient ----
      float scale = 0.f, mx = 0.f, dpos, loss_w;
      if (LOSS == PBG_LOSS_SOFTMAX) {
        mx = oct_max(st.m);
        const float epos = expf(pos - mx);
        const float z = oct_sum(st.z * expf(st.m - mx)) + epos;
        const float inv_z = 1.0f / z;
        loss_w = ((mx + logf(z)) - pos) * w;
        dpos = (epos * inv_z - 1.0f) * w;
        scale = inv_z * w;
      } else if (LOSS == PBG_LOSS_RANKING) {
        loss_w = oct_sum(st.acc) * w;
        dpos = -oct_sum(st.gsum);
      } else {
        loss_w = (oct_sum(st.acc) * inv_nn + softplusf(-pos)) * w;
        dpos = (sigmoidf(pos) - 1.0f) * w;
        scale = inv_nn * w;
      }
      // dLoss/dS of this thread's four columns of a tile, the positive's gradient on the diagonal;
      // the violators are counted on the way (masked and absent columns score -1e9 / -inf)
      int viol = 0;
      auto parked = [&](int tile) { return *reinterpret_cast<const float4*>(scr + (size_t)tile * (kHelpers * 4)); };
      auto grad_tile = [&](int tile, int gbuf, float4 sv) {
        const float t[4] = {sv.x, sv.y, sv.z, sv.w};
        float g[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (LOSS == PBG_LOSS_SOFTMAX) g[e] = exp_of_difference(t[e], mx) * scale;
          else if (LOSS == PBG_LOSS_RANKING) g[e] = ((t[e] - pos) + c.margin >= 0.f) ? w : 0.f;
          else g[e] = fast_sigmoid(t[e], nullptr) * scale;
          viol += t[e] > pos ? 1 : 0;
        }
        if (tile * kTile < P) {
          const int j0 = tile * kTile + hc;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (j0 + e == hrow && hrow < P) g[e] = dpos;
        }
        *reinterpret_cast<float4*>(&lds[gbuf + hrow * kLdg + swap23(hc)]) = make_float4(g[0], g[1], g[2], g[3]);
      };
      grad_tile(0, a.g_at + (nt & 1) * kTileFloats, parked(0));
      // The parked scores come back from beyond the L2 (a workgroup parks 270 KB per item): those of
      // tile t + 1 are asked for a whole tile ahead, or the round trip would sit between the
      // helpers and barrier (A) in every tile.
      float4 sv = parked(min(1, nt - 1));
      lds_barrier();  // (T) G_0 in LDS

      // ---- sweep 2 ----
      for (int q = nt; q < 2 * nt; ++q) {
        const int t = q - nt;
        const bool more = t + 1 < nt;
        const float4 sv_next = parked(min(t + 2, nt - 1));
        rows.issue(sd.w, D, nid0, nid1, ht);  // tile t + 1 (with `more`; else rows that are not stored)
        TileRows<NSEG>::fetch_ids(colid, min(t + 2, nt - 1) * kTile, ncols, ht, &nid0, &nid1);
        lds_barrier();  // (A) dA has taken tile t
        if (more) rows.store(lds, a.n_at, lda, D, ht, edge_tile(t + 1), true);
        // G_(t+1) goes into the buffer that dN_(t-1) was the last to read.  It is formed on this side of (A):
        // every vector instruction of a helper waits for a gap between matrix instructions, and up to (A) the
        // helpers' loads above are all that stands between them and the barrier.
        if (more) grad_tile(t + 1, a.g_at + ((q + 1) & 1) * kTileFloats, sv);
        sv = sv_next;
        lds_barrier();  // (B) tile t + 1 and G_(t+1) in LDS, G_t no longer read
      }
      viol = oct_sum_int(viol);
      if ((ht & 7) == 0 && hrow < P) {
        const int64_t job = (int64_t)k * CP + cc * P + hrow;
        (s ? a.sloss[1] : a.sloss[0])[job] = row_live ? loss_w : 0.f;
        c.violrow[job * 2 + s] = row_live ? viol : 0;
      }
    } else {
      // ================= compute role =================
      // The lane's indices are hidden from the optimiser once per tile: the addresses derived from
      // them are then recomputed (a few instructions) instead of all being hoisted out of the loops
      // into registers that stay live next to the accumulators.
      int lane_ = threadIdx.x & 63;
      const int rt = wave & 3, grp = wave >> 2;
      float4v dA[T0];
#pragma unroll
      for (int t = 0; t < T0; ++t) dA[t] = (float4v){0.f, 0.f, 0.f, 0.f};
      lds_barrier();  // (p2)

      // ---- sweep 1: S_q = A N_q^T, one 16 x 16 block per wave ----
      for (int q = 0; q < nt; ++q) {
        asm volatile("" : "+v"(lane_));
        const int m16 = lane_ & 15, kq = lane_ >> 4;
        float4v acc = (float4v){0.f, 0.f, 0.f, 0.f};
        const int ar = min(rt * 16 + m16, pr - 1);
        mfma_sweep_k16<1>(lds, a.a_at + ar * lda, a.n_at + (grp * 16 + m16) * lda, 0, NT, 0, kq, &acc);
        *reinterpret_cast<float4*>(&lds[a.g_at + (q & 1) * kTileFloats + (rt * 16 + m16) * kLdg + grp * 16 + 4 * kq]) =
            make_float4(acc[0], acc[1], acc[2], acc[3]);
        lds_barrier();  // (A)
        lds_barrier();  // (B)
      }
      lds_barrier();  // (T)

      // ---- sweep 2 ----
      const int rt2 = wave & 1, qtr = wave >> 1;
      const int dn_base = NT / 4, dn_rem = NT % 4;
      const int dn_cnt = dn_base + (qtr < dn_rem ? 1 : 0), dn_ct0 = qtr * dn_base + min(qtr, dn_rem);
      float* const sdb = (s ? a.sdb[1] : a.sdb[0]) + e0 * D;
      float* const uni = c.gr + ((int64_t)k * c.rk + sd.slot_uni + (int64_t)cc * U) * D;
      for (int q = nt; q < 2 * nt; ++q) {
        const int t = q - nt;
        const int gbuf = a.g_at + (q & 1) * kTileFloats;
        asm volatile("" : "+v"(lane_));
        const int m16 = lane_ & 15, kq = lane_ >> 4;
        {  // dA += G_t N_t: this wave's row tile, its half of the column tiles
          const int a_at = gbuf + (rt * 16 + m16) * kLdg + 16 * (kq >> 1) + 4 * (kq & 1), b_at = a.n_at + 8 * kq * lda;
          stream_da_product<T0, lda>(lds, a_at, b_at + (grp ? (NT - T0) * 16 : 0), m16, dA);
        }
        // (where dN_t goes: worked out on this side of the barrier, while other waves still multiply)
        const int j = t * kTile + rt2 * 16 + m16;
        float* dst = nullptr;
        if (j < P) {
          if (j < valid) dst = sdb + (int64_t)j * D;
        } else if (j < ncols) {
          dst = uni + (int64_t)(j - P) * D;
        }
        const int k0 = 2 * (kq & 1) + (kq >> 1);
        const int g_at = gbuf + k0 * kLdg + rt2 * 16 + swap23(m16), a_at = a.a_at + k0 * lda;
        lds_barrier();  // (A)
        {  // dN_t = G_t^T A: 16 negatives x this wave's quarter of the column tiles
          // The two compute waves of a SIMD (wave and wave + 4) take their parts in opposite orders, so that
          // one is in the middle of a part while the other drains its accumulators and refills its operands.
          int ct = dn_ct0, left = dn_cnt;
          const int small = left & 3;
          if (qtr >= 2 && small) {
            if (small == 3) stream_dn_part<3, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
            else if (small == 2) stream_dn_part<2, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
            else stream_dn_part<1, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
            ct += small;
            left -= small;
          }
          for (; left >= 4; left -= 4, ct += 4) stream_dn_part<4, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
          if (left == 3) stream_dn_part<3, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
          else if (left == 2) stream_dn_part<2, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
          else if (left == 1) stream_dn_part<1, lda, kExact>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst, D);
        }
        lds_barrier();  // (B)
      }
      // ---- the positives' operand gradients ----
      const int m16 = lane_ & 15, kq = lane_ >> 4;
      const int i = rt * 16 + m16;
      if (i < valid) {
        const int first = grp ? (NT - T0) * 16 : 0;
        stream_da_store<T0, kExact>(dA, kq, (s ? a.sda[1] : a.sda[0]) + (e0 + i) * D + first, D - first);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// per-edge finish
// ---------------------------------------------------------------------------
// One wave per edge: the two raw-row gradients of the pair from the four partial
// rows the items left (the row as the other item's operand, mapped back through
// the operator, plus the row as a batch negative of its own side), the edge's loss,
// the N3 regularizer's terms of the edge's rows, and (standard mode) the edge's term
// of the operator's parameter gradient.
template <int NVH>
__global__ __launch_bounds__(kRowThreads) void stream_finish_kernel(StepCtx c, StreamPlan a) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int CP = c.C * c.P;
  if (job >= (int64_t)c.K * CP) return;
  const int k = (int)(job / CP), q = (int)(job % CP);
  if (q >= c.B) {  // padded position of the last chunk
    if (lane == 0) c.lossrow[job] = 0.f;
    return;
  }
  if (lane == 0) c.lossrow[job] = a.sloss[0][job] + a.sloss[1][job];
  const int D = c.D, H = (D + 1) / 2;
  const int64_t e = (int64_t)k * c.B + q;
  const SideCtx& s0 = c.side[0];
  const SideCtx& s1 = c.side[1];
  RowV<NVH> a0 = row_load<NVH>(a.sda[0] + e * D, D, H, lane);  // gradient at the operand derived from the rhs row
  RowV<NVH> a1 = row_load<NVH>(a.sda[1] + e * D, D, H, lane);  // ... from the lhs row
  RowV<NVH> gl = row_load<NVH>(a.sdb[0] + e * D, D, H, lane);
  RowV<NVH> gr = row_load<NVH>(a.sdb[1] + e * D, D, H, lane);
  const bool reg = c.reg_coef != 0.f;
  RowV<NVH> xl, xr;
  if (reg || (c.op != PBG_OP_NONE && !c.dynamic)) {
    xl = row_load<NVH>(s0.w + clamp_index(s0.idx[e], s0.num_rows) * D, D, H, lane);
    xr = row_load<NVH>(s1.w + clamp_index(s1.idx[e], s1.num_rows) * D, D, H, lane);
  }
  if (reg) {
    // N3 over the rows the model hands the regularizer (model.py:784-785,845-854): the lhs row
    // and op(rhs row); with one relation per edge each side's row in one direction and its
    // operated row in the other (model.py:722-758).  The term of an operated row joins the
    // gradient at that row, which then flows through the operator like the scores' part.
    float cubes0 = n3_term<NVH>(c.op, c.reg_coef, gl, xl), cubes1;
    const RowV<NVH> zr = row_load<NVH>(a.sa[0] + e * D, D, H, lane);  // op(rhs row)
    if (c.dynamic) {
      const RowV<NVH> zl = row_load<NVH>(a.sa[1] + e * D, D, H, lane);  // the lhs operator's op(lhs row)
      cubes0 += n3_term<NVH>(c.op, c.reg_coef, a1, zl);
      cubes1 = n3_term<NVH>(c.op, c.reg_coef, gr, xr) + n3_term<NVH>(c.op, c.reg_coef, a0, zr);
      if (c.op != PBG_OP_NONE) {  // these rows are the operator-output gradients the parameter stage reads
        row_store<NVH>(a.sda[0] + e * D, a0, D, H, lane);
        row_store<NVH>(a.sda[1] + e * D, a1, D, H, lane);
      }
    } else {
      cubes1 = n3_term<NVH>(c.op, c.reg_coef, a0, zr);
    }
    cubes0 = wave_sum(cubes0);
    cubes1 = wave_sum(cubes1);
    if (lane == 0) {
      c.regrow[((int64_t)k * 2 + 0) * c.B + q] = cubes0;
      c.regrow[((int64_t)k * 2 + 1) * c.B + q] = cubes1;
    }
  }
  if (c.op == PBG_OP_NONE) {
    row_axpy<NVH>(gl, 1.0f, a1);
    row_axpy<NVH>(gr, 1.0f, a0);
  } else if (c.dynamic) {
    const int64_t rel = clamp_index(c.rel[e], c.num_relations);
    row_axpy<NVH>(gl, 1.0f, op_backward<NVH>(c.op, a1, s0.p0, s0.p1, rel, D, H, lane));
    row_axpy<NVH>(gr, 1.0f, op_backward<NVH>(c.op, a0, s1.p0, s1.p1, rel, D, H, lane));
  } else {
    const int64_t rel = clamp_index(c.rel[k], c.num_relations);
    row_axpy<NVH>(gl, 1.0f, op_forward<NVH>(c.op, a1, s1.p0, s1.p1, rel, D, H, lane));  // the lhs operand was op^T(lhs)
    row_axpy<NVH>(gr, 1.0f, op_backward<NVH>(c.op, a0, s1.p0, s1.p1, rel, D, H, lane));
    // d/d parameter of <lhs, op(rhs)>-shaped scores: through op(rhs) with gradient a0, and through
    // op^T(lhs) with gradient a1 (operators.py:59-84,128-157)
    RowV<NVH> t;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      if (c.op == PBG_OP_DIAGONAL) {
        t.a[0][v] = xr.a[0][v] * a0.a[0][v] + xl.a[0][v] * a1.a[0][v];
        t.a[1][v] = xr.a[1][v] * a0.a[1][v] + xl.a[1][v] * a1.a[1][v];
      } else {  // (real | imaginary) halves
        t.a[0][v] = (xr.a[0][v] * a0.a[0][v] + xr.a[1][v] * a0.a[1][v]) + (xl.a[0][v] * a1.a[0][v] + xl.a[1][v] * a1.a[1][v]);
        t.a[1][v] = (xr.a[0][v] * a0.a[1][v] - xr.a[1][v] * a0.a[0][v]) + (xl.a[1][v] * a1.a[0][v] - xl.a[0][v] * a1.a[1][v]);
      }
    }
    row_store<NVH>(s1.dz + e * D, t, D, H, lane);
  }
  row_store<NVH>(c.gr + ((int64_t)k * c.rk + s0.slot_pos + q) * D, gl, D, H, lane);
  row_store<NVH>(c.gr + ((int64_t)k * c.rk + s1.slot_pos + q) * D, gr, D, H, lane);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
template <int NT, int LOSS>
int launch_chunk_as(const StepCtx& c, const StreamPlan& sp, hipStream_t s) {
  const size_t lds_bytes = (size_t)sp.total * sizeof(float);
  static LdsLimit limit;
  const int rc = reserve_lds((const void*)stream_chunk_kernel<NT, LOSS>, &limit, lds_bytes);
  if (rc != PBG_OK) return rc;
  const int items = 2 * c.K * c.C;
  hipLaunchKernelGGL((stream_chunk_kernel<NT, LOSS>), dim3((unsigned)(items < sp.grid ? items : sp.grid)),
                     dim3(2 * kHelpers), lds_bytes, s, c, sp, items);
  return PBG_OK;
}

template <int NT>
int launch_chunk_loss(const StepCtx& c, const StreamPlan& sp, hipStream_t s) {
  switch (c.loss) {
    case PBG_LOSS_RANKING: return launch_chunk_as<NT, PBG_LOSS_RANKING>(c, sp, s);
    case PBG_LOSS_LOGISTIC: return launch_chunk_as<NT, PBG_LOSS_LOGISTIC>(c, sp, s);
    default: return launch_chunk_as<NT, PBG_LOSS_SOFTMAX>(c, sp, s);
  }
}

// Column tiles of 16 per row for which the chunk kernel is built: the exact dims 128, 256, 400, and
// 13 / 19 tiles for any dim (a multiple of 4) in (192, 208] / (288, 304]; 0: not built.
int stream_tiles(int D) {
  if (D == 128 || D == 256 || D == 400) return D / 16;
  const int nt = (D + 15) / 16;
  return (D % 4 == 0 && (nt == 13 || nt == 19)) ? nt : 0;
}

#define PBG_STREAM_ROWS(nvh, KERNEL, jobs, stream, ...)                                                                  \
  do {                                                                                                                   \
    const dim3 grid((unsigned)ceil_div((jobs) > 0 ? (jobs) : 1, kWavesPerBlock));                                        \
    if ((nvh) <= 1) hipLaunchKernelGGL((KERNEL<1>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);                    \
    else if ((nvh) <= 2) hipLaunchKernelGGL((KERNEL<2>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);               \
    else hipLaunchKernelGGL((KERNEL<4>), grid, dim3(kRowThreads), 0, stream, __VA_ARGS__);                               \
  } while (0)

}  // namespace

bool stream_geometry(const StepCtx& c, StreamPlan* sp) {
  memset(sp, 0, sizeof(*sp));
  if (c.cmp != PBG_CMP_DOT || c.bias || c.affine) return false;
  if (c.op != PBG_OP_NONE && c.op != PBG_OP_DIAGONAL && c.op != PBG_OP_COMPLEX_DIAGONAL) return false;
  if (stream_tiles(c.D) == 0 || c.P > 64) return false;
  for (int s = 0; s < 2; ++s) {
    const SideCtx& sd = c.side[s];
    // (measured at dim 400 with 50 + 50 negatives: 50.8 M edges/s here against 34.5 M on the staged kernels)
    if (sd.all || sd.u < 8 || sd.u != c.side[0].u || sd.num_rows >= ((int64_t)1 << 31)) return false;
    if (sd.nb != 0 && sd.nb != c.P) return false;
  }
  sp->pr = (c.P + 3) / 4 * 4;
  sp->lda = lds_stride(stream_tiles(c.D) * 16);
  sp->ntiles = (int)ceil_div(c.P + c.side[0].u, kTile);
  // the tile first: the products' reads past its last row then land in the rows behind it
  sp->n_at = 0;
  sp->a_at = kTile * sp->lda;
  sp->g_at = sp->a_at + sp->pr * sp->lda;
  sp->total = sp->g_at + 2 * kTileFloats + kSlack;
  if ((size_t)sp->total * sizeof(float) > 160 * 1024 - 512) return false;
  const int cus = compute_units();  // (of the current device)
  const int items = 2 * c.K * c.C;
  sp->grid = items < cus ? items : cus;
  return true;
}

int stream_prep(const StepCtx& c, const StreamPlan& sp, int nvh, hipStream_t stream) {
  if (nvh > 4) return fail(PBG_ERR_UNSUPPORTED, "step: streaming route needs dim <= 512");
  PBG_STREAM_ROWS(nvh, stream_prep_kernel, (int64_t)c.K * 2 * c.B, stream, c, sp);
  const int64_t columns = 2 * (int64_t)c.K * c.C * (c.P + c.side[0].u);
  hipLaunchKernelGGL(stream_ids_kernel, dim3((unsigned)ceil_div(columns, 256)), dim3(256), 0, stream, c, sp);
  return check_launch("step streaming prep");
}

int stream_chunks(const StepCtx& c, const StreamPlan& sp, hipStream_t stream) {
  int rc;
  switch (stream_tiles(c.D)) {
    case 8: rc = launch_chunk_loss<8>(c, sp, stream); break;
    case 13: rc = launch_chunk_loss<13>(c, sp, stream); break;
    case 16: rc = launch_chunk_loss<16>(c, sp, stream); break;
    case 19: rc = launch_chunk_loss<19>(c, sp, stream); break;
    case 25: rc = launch_chunk_loss<25>(c, sp, stream); break;
    default: return fail(PBG_ERR_UNSUPPORTED, "step: streaming route not built for dim %d", c.D);
  }
  if (rc != PBG_OK) return rc;
  return check_launch("step streaming chunks");
}

int stream_finish(const StepCtx& c, const StreamPlan& sp, int nvh, hipStream_t stream) {
  PBG_STREAM_ROWS(nvh, stream_finish_kernel, (int64_t)c.K * c.C * c.P, stream, c, sp);
  return check_launch("step streaming finish");
}

}  // namespace pbg
