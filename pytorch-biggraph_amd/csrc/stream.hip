// The streaming route of the training step, for chunks whose negatives do not fit
// LDS next to their positives (hundreds or thousands of uniform negatives per
// chunk, model.py:508-622 with num_uniform_negs large): dot comparator, operator
// none / diagonal / complex_diagonal, every loss.
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
constexpr int kLdg = 44;                     // row stride of a 64 x 32 score tile in LDS (44 % 32 == 12)
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
// Row id of column j of an item's negatives (-1: a padded position of a partial
// last chunk, or a column past the last negative), and the sort key of a uniform
// negative's gradient row.
__device__ __forceinline__ int stream_column_id(const StepCtx& c, const SideCtx& sd, int s, int k, int cc, int kc, int valid,
                                                int j, bool write_key) {
  const int P = c.P, U = sd.u;
  const bool is_pos = j < P;
  const int q = cc * P + j, u = min(max(j - P, 0), U - 1);
  const bool real = is_pos ? j < valid : j < P + U;
  int64_t id;
  if (is_pos) id = sd.idx[(int64_t)k * c.B + min(q, c.B - 1)];
  else id = uniform_negative(sd, s, (int64_t)kc * U + u);
  id = clamp_index(id, sd.num_rows);
  if (write_key && real && !is_pos) {
    const int64_t pair = (int64_t)k * c.rk + sd.slot_uni + (int64_t)cc * U + u;
    c.keys[pair] = ((uint64_t)(sd.key_base + id) << c.kbits) | (uint64_t)k;
    c.vals[pair] = (uint32_t)pair;
  }
  return real ? (int)id : -1;
}

// Half a wave per 128 columns of a row, 128-bit loads, the whole tile in flight:
// half-wave h of the 16 takes rows h and h + 16.  Absent rows read row 0 (zeroed
// when stored); all loads are issued from straight-line code.
template <int NSEG>
struct TileRows {
  float4 v[2 * NSEG];
  int id0, id1;
  __device__ __forceinline__ void issue(const float* w, int D, const int* ids, int ht, bool active) {
    const int hw = ht >> 5, c4 = (ht & 31) << 2;
    id0 = active ? ids[hw] : -1;
    id1 = active ? ids[hw + 16] : -1;
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
  __device__ __forceinline__ void store(float* lds, int n_at, int lda, int D, int ht) const {
    const int hw = ht >> 5, c4 = (ht & 31) << 2;
#pragma unroll
    for (int seg = 0; seg < NSEG; ++seg) {
      const int col = seg * 128 + c4;
      if (col < D) {
        *reinterpret_cast<float4*>(&lds[n_at + hw * lda + col]) = keep_if(v[2 * seg], id0 >= 0);
        *reinterpret_cast<float4*>(&lds[n_at + (hw + 16) * lda + col]) = keep_if(v[2 * seg + 1], id1 >= 0);
      }
    }
  }
};

// NCT column tiles of dA += G_t N_t for the lane's row of the score tile: a_at = that row's first
// element + 4 kq, b_at = the tile's row 4 kq at the part's first column.  The k slots of
// step r of group g hold k = 16 g + 4 kq + r in both operands; LDA is known at compile
// time, so every address below is one register plus an immediate.  The other compute wave
// of the SIMD issues its matrix instructions while this one waits for its operands.
template <int NCT, int LDA>
__device__ __forceinline__ void stream_da_part(const float* lds, int a_at, int b_at, int m16, float4v* acc) {
#pragma unroll
  for (int g = 0; g < kTile / 16; ++g) {
    const float4 av4 = *reinterpret_cast<const float4*>(&lds[a_at + 16 * g]);
    const float av[4] = {av4.x, av4.y, av4.z, av4.w};
    float b[4][NCT];
#pragma unroll
    for (int r = 0; r < 4; ++r) load_b<NCT>(lds, b_at + (16 * g + r) * LDA, m16, b[r]);
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[r][t], av[r], acc[t], 0, 0, 0);
  }
}
template <int N, int LDA>
__device__ __forceinline__ void stream_da_product(const float* lds, int a_at, int b_at, int m16, float4v* acc) {
  constexpr int full = N / 4, rem = N % 4;
#pragma unroll
  for (int p = 0; p < full; ++p) stream_da_part<4, LDA>(lds, a_at, b_at + 64 * p, m16, acc + 4 * p);
  if constexpr (rem > 0) stream_da_part<rem, LDA>(lds, a_at, b_at + 64 * full, m16, acc + 4 * full);
}
template <int N>
__device__ __forceinline__ void stream_da_store(const float4v* acc, int kq, float* dst) {
  constexpr int full = N / 4, rem = N % 4;
#pragma unroll
  for (int p = 0; p < full; ++p)
    for_each_out<4>(acc + 4 * p, kq, [&](int col, float4 v) { *reinterpret_cast<float4*>(dst + 64 * p + col) = v; });
  if constexpr (rem > 0)
    for_each_out<rem>(acc + 4 * full, kq, [&](int col, float4 v) { *reinterpret_cast<float4*>(dst + 64 * full + col) = v; });
}

// NCT column tiles from `ct` on of dN_t = G_t^T A for the lane's negative, stored at dst (or
// dropped): g_at = the negative's column of G_t in row kq, a_at = row kq of A at column 0.
template <int NCT, int LDA>
__device__ __forceinline__ void stream_dn_part(const float* lds, int g_at, int a_at, int ct, int ksteps, int kq, int m16,
                                               float* dst) {
  float4v acc[NCT];
#pragma unroll
  for (int t = 0; t < NCT; ++t) acc[t] = (float4v){0.f, 0.f, 0.f, 0.f};
  a_at += ct * 16;
#pragma unroll 2
  for (int ks = 0; ks < ksteps; ++ks) {
    const float g = lds[g_at];
    float b[NCT];
    load_b<NCT>(lds, a_at, m16, b);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[t], g, acc[t], 0, 0, 0);
    g_at += 4 * kLdg;
    a_at += 4 * LDA;
  }
  if (dst) for_each_out<NCT>(acc, kq, [&](int col, float4 v) { *reinterpret_cast<float4*>(dst + ct * 16 + col) = v; });
}

// Statistics of one row of the score matrix, spread over the 8 threads that own the row.
template <int LOSS>
struct RowLoss {
  float m, z;     // softmax: running maximum (starts at the positive score) and sum of exp(score - m)
  float acc;      // ranking: sum of hinges; logistic: sum of softplus(score)
  float gsum;     // ranking: sum of dLoss/dscore
  int viol;
  __device__ __forceinline__ void start(float pos) {
    m = pos;
    z = 0.f;
    acc = 0.f;
    gsum = 0.f;
    viol = 0;
  }
  __device__ __forceinline__ void add(const float* t, float pos, float w, float margin) {
    if (LOSS == PBG_LOSS_SOFTMAX) {
      const float mt = fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3]));
      const float mn = fmaxf(m, mt);
      z = z * expf(m - mn) + ((expf(t[0] - mn) + expf(t[1] - mn)) + (expf(t[2] - mn) + expf(t[3] - mn)));
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
        acc += softplusf(t[e]);
      }
      if (t[e] > pos) ++viol;
    }
  }
};

// Persistent kernel: workgroup b takes items b, b + gridDim.x, ...; item = 2 * chunk + side.
template <int NT, int LOSS>
__global__ __launch_bounds__(2 * kHelpers) void stream_chunk_kernel(StepCtx c, StreamPlan a, int num_items) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int D = NT * 16, D4 = D / 4, NSEG = (D + 127) / 128;
  constexpr int lda = lds_stride(D);               // (= a.lda)
  constexpr int T0 = (NT + 1) / 2, T1 = NT - T0;  // column tiles of dA per wave group
  const int wave16 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave = wave16 & 7, ht = threadIdx.x & (kHelpers - 1);
  const int P = c.P, C = c.C, U = c.side[0].u, ncols = P + U, nt = a.ntiles, pr = a.pr;
  const int CP = C * P;
  int* idbuf = reinterpret_cast<int*>(lds + a.id_at);
  float* scr = a.scratch + (size_t)blockIdx.x * nt * (kHelpers * 4) + ht * 4;
  const bool helper = wave16 >= 8;
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
      if (threadIdx.x < 64) {
        const int b = threadIdx.x >> 5, tile = b < nt ? b : 0;
        idbuf[threadIdx.x] = stream_column_id(c, sd, s, k, cc, kc, valid, tile * kTile + (threadIdx.x & 31), b < nt);
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

      TileRows<NSEG> rows;
      rows.issue(sd.w, D, idbuf, ht, true);
      rows.store(lds, a.n_at, lda, D, ht);
      lds_barrier();  // (p2) tile 0 in LDS

      RowLoss<LOSS> st;
      st.start(pos);
      // masks (model.py:566-580,836-839), then the statistics; the masked tile goes to the scratch area
      auto absorb = [&](int tile, int gbuf) {
        const float4 sv = *reinterpret_cast<const float4*>(&lds[gbuf + hrow * kLdg + hc]);
        float t[4] = {sv.x, sv.y, sv.z, sv.w};
        const int j0 = tile * kTile + hc;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = j0 + e;
          if (j < P && (!has_nb || j == hrow || j >= valid)) t[e] = -1e9f;
          if (j >= ncols) t[e] = -INFINITY;
        }
        *reinterpret_cast<float4*>(scr + (size_t)tile * (kHelpers * 4)) = make_float4(t[0], t[1], t[2], t[3]);
        st.add(t, pos, w, c.margin);
      };

      // ---- sweep 1 ----
      for (int q = 0; q < nt; ++q) {
        const int tn = q + 1 == nt ? 0 : q + 1, t2 = tn + 1 == nt ? 0 : tn + 1;
        rows.issue(sd.w, D, idbuf + ((q + 1) & 1) * kTile, ht, true);
        if (ht < kTile) idbuf[(q & 1) * kTile + ht] = stream_column_id(c, sd, s, k, cc, kc, valid, t2 * kTile + ht, q + 2 < nt);
        if (q >= 1) absorb(q - 1, a.g_at + ((q - 1) & 1) * kTileFloats);
        lds_barrier();  // (A) S_q complete, tile q no longer read
        rows.store(lds, a.n_at, lda, D, ht);
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
      const int viol = oct_sum_int(st.viol);
      if ((ht & 7) == 0 && hrow < P) {
        const int64_t job = (int64_t)k * CP + cc * P + hrow;
        (s ? a.sloss[1] : a.sloss[0])[job] = row_live ? loss_w : 0.f;
        c.violrow[job * 2 + s] = row_live ? viol : 0;
      }
      // dLoss/dS of this thread's four columns of a tile; the positive's gradient on the diagonal
      auto grad_tile = [&](int tile, int gbuf) {
        const float4 sv = *reinterpret_cast<const float4*>(scr + (size_t)tile * (kHelpers * 4));
        const float t[4] = {sv.x, sv.y, sv.z, sv.w};
        float g[4];
        const int j0 = tile * kTile + hc;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (LOSS == PBG_LOSS_SOFTMAX) g[e] = expf(t[e] - mx) * scale;
          else if (LOSS == PBG_LOSS_RANKING) g[e] = ((t[e] - pos) + c.margin >= 0.f) ? w : 0.f;
          else g[e] = sigmoidf(t[e]) * scale;
          if (j0 + e == hrow && hrow < P) g[e] = dpos;
        }
        *reinterpret_cast<float4*>(&lds[gbuf + hrow * kLdg + hc]) = make_float4(g[0], g[1], g[2], g[3]);
      };
      grad_tile(0, a.g_at + (nt & 1) * kTileFloats);
      lds_barrier();  // (T) G_0 in LDS

      // ---- sweep 2 ----
      for (int q = nt; q < 2 * nt; ++q) {
        const int t = q - nt;
        const bool more = t + 1 < nt;
        rows.issue(sd.w, D, idbuf + ((q + 1) & 1) * kTile, ht, more);
        if (ht < kTile && t + 2 < nt)
          idbuf[(q & 1) * kTile + ht] = stream_column_id(c, sd, s, k, cc, kc, valid, (t + 2) * kTile + ht, false);
        if (more) grad_tile(t + 1, a.g_at + ((q + 1) & 1) * kTileFloats);
        lds_barrier();  // (A) dA has taken tile t
        if (more) rows.store(lds, a.n_at, lda, D, ht);
        lds_barrier();  // (B) tile t + 1 and G_(t+1) in LDS, G_t no longer read
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
          const int a_at = gbuf + (rt * 16 + m16) * kLdg + 4 * kq, b_at = a.n_at + 4 * kq * lda;
          if (grp == 0) stream_da_product<T0, lda>(lds, a_at, b_at, m16, dA);
          else if (T1 > 0) stream_da_product<(T1 > 0 ? T1 : 1), lda>(lds, a_at, b_at + T0 * 16, m16, dA);
        }
        lds_barrier();  // (A)
        {  // dN_t = G_t^T A: 16 negatives x this wave's quarter of the column tiles
          const int j = t * kTile + rt2 * 16 + m16;
          float* dst = nullptr;
          if (j < P) {
            if (j < valid) dst = sdb + (int64_t)j * D;
          } else if (j < ncols) {
            dst = uni + (int64_t)(j - P) * D;
          }
          const int g_at = gbuf + kq * kLdg + rt2 * 16 + m16, a_at = a.a_at + kq * lda;
          int ct = dn_ct0, left = dn_cnt;
          for (; left >= 4; left -= 4, ct += 4) stream_dn_part<4, lda>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst);
          if (left == 3) stream_dn_part<3, lda>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst);
          else if (left == 2) stream_dn_part<2, lda>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst);
          else if (left == 1) stream_dn_part<1, lda>(lds, g_at, a_at, ct, pr >> 2, kq, m16, dst);
        }
        lds_barrier();  // (B)
      }
      // ---- the positives' operand gradients ----
      const int m16 = lane_ & 15, kq = lane_ >> 4;
      const int i = rt * 16 + m16;
      if (i < valid) {
        float* dst = (s ? a.sda[1] : a.sda[0]) + (e0 + i) * D + (grp ? T0 * 16 : 0);
        if (grp == 0) stream_da_store<T0>(dA, kq, dst);
        else if (T1 > 0) stream_da_store<(T1 > 0 ? T1 : 1)>(dA, kq, dst);
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
// and (standard mode) the edge's term of the operator's parameter gradient.
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
  const RowV<NVH> a0 = row_load<NVH>(a.sda[0] + e * D, D, H, lane);  // gradient at the operand derived from the rhs row
  const RowV<NVH> a1 = row_load<NVH>(a.sda[1] + e * D, D, H, lane);  // ... from the lhs row
  RowV<NVH> gl = row_load<NVH>(a.sdb[0] + e * D, D, H, lane);
  RowV<NVH> gr = row_load<NVH>(a.sdb[1] + e * D, D, H, lane);
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
    const RowV<NVH> xl = row_load<NVH>(s0.w + clamp_index(s0.idx[e], s0.num_rows) * D, D, H, lane);
    const RowV<NVH> xr = row_load<NVH>(s1.w + clamp_index(s1.idx[e], s1.num_rows) * D, D, H, lane);
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
  static size_t lds_allowed = 0;
  if (lds_bytes > lds_allowed) {
    if (hipFuncSetAttribute((const void*)stream_chunk_kernel<NT, LOSS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess)
      return fail(PBG_ERR_LAUNCH, "step: cannot reserve %zu bytes of LDS", lds_bytes);
    lds_allowed = lds_bytes;
  }
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

bool stream_dim_built(int D) { return D == 128 || D == 256 || D == 400; }

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
  if (c.cmp != PBG_CMP_DOT || c.bias || c.affine || c.reg_coef != 0.f) return false;
  if (c.op != PBG_OP_NONE && c.op != PBG_OP_DIAGONAL && c.op != PBG_OP_COMPLEX_DIAGONAL) return false;
  if (!stream_dim_built(c.D) || c.P > 64) return false;
  for (int s = 0; s < 2; ++s) {
    const SideCtx& sd = c.side[s];
    if (sd.all || sd.u < 64 || sd.u != c.side[0].u || sd.num_rows >= ((int64_t)1 << 31)) return false;
    if (sd.nb != 0 && sd.nb != c.P) return false;
  }
  sp->pr = (c.P + 3) / 4 * 4;
  sp->lda = lds_stride(c.D);
  sp->ntiles = (int)ceil_div(c.P + c.side[0].u, kTile);
  // the tile first: the products' reads past its last row then land in the rows behind it
  sp->n_at = 0;
  sp->a_at = kTile * sp->lda;
  sp->g_at = sp->a_at + sp->pr * sp->lda;
  sp->id_at = sp->g_at + 2 * kTileFloats;
  sp->total = sp->id_at + 2 * kTile + kSlack;
  if ((size_t)sp->total * sizeof(float) > 160 * 1024 - 512) return false;
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
  }
  const int items = 2 * c.K * c.C;
  sp->grid = items < cus ? items : cus;
  return true;
}

int stream_prep(const StepCtx& c, const StreamPlan& sp, int nvh, hipStream_t stream) {
  if (nvh > 4) return fail(PBG_ERR_UNSUPPORTED, "step: streaming route needs dim <= 512");
  PBG_STREAM_ROWS(nvh, stream_prep_kernel, (int64_t)c.K * 2 * c.B, stream, c, sp);
  return check_launch("step streaming prep");
}

int stream_chunks(const StepCtx& c, const StreamPlan& sp, hipStream_t stream) {
  int rc;
  switch (c.D) {
    case 128: rc = launch_chunk_loss<8>(c, sp, stream); break;
    case 256: rc = launch_chunk_loss<16>(c, sp, stream); break;
    case 400: rc = launch_chunk_loss<25>(c, sp, stream); break;
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
