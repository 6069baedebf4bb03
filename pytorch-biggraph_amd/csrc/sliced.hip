// The chunk kernel of the fused route for rows wider than LDS: slices of 128 columns.
#include "fused.h"

#include "fused_parts.h"

namespace pbg {
namespace {

// ---------------------------------------------------------------------------
// The same chain for rows too wide for LDS (dim 132 ... 4096 in multiples of 4,
// at most 64 batch + 64 uniform negatives, operator none / translation / diagonal, dot / cos / l2): the chunk's
// 2 (P + U) rows pass through LDS in SLICES of 128 columns, twice.
//
//   sweep 1   per slice: rows -> LDS (raw; cos: the squared norms add up in
//             registers), both score blocks accumulate S += A_slice N_slice^T in
//             the matrix accumulators across all slices
//   between   cos: scores times the two reciprocal norms; scores -> LDS; masks, loss,
//             dLoss/dS in place, the fold G = dS_R + dS_L^T (+ dLoss/dpos on the
//             diagonal), exactly as in the one-piece kernel; cos: <y, dLoss/dy> of every
//             row from the scores and their gradients, t = sum_j dS_ij S_ij (the row is
//             never in LDS as a whole, its gradient neither)
//   sweep 2   per slice: rows -> LDS again (cos: normalised), the four gradient
//             products of the one-piece kernel on the slice, results through
//             (dy - t y) / ||x|| (cos) to the slice's columns of the gradient rows
//
// A row is read twice and its gradient written once; scores and their gradients never
// leave LDS.  Eight waves, no split into roles: the next slice's rows are on their way
// from HBM into registers while the products of the current one issue.
// Row ids and sort keys come from fused_ids_kernel (c.fused_rowid).
constexpr int kSliceThreads = 512;

// LDS != 0: the score rows' stride, known at compile time like the slice rows' (136 floats), so that the
// products' LDS addresses are one register plus immediates.
// HALF (config.half_precision, dot / cos): the rounding points of fused_chunk_kernel<..., HALF>.  The prepared row
// is what gets rounded, so with cos the norms must be known before the first product: one more pass over the rows
// ("sweep 0", nothing stored) adds up the squared norms, and both sweeps then store normalised, rounded rows.
template <int CMP, int LOSS, int LDS, bool HALF, bool CPLX>
__global__ __launch_bounds__(kSliceThreads) void sliced_chunk_kernel(StepCtx c, FusedLayout f, int num_chunks) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr bool cosn = CMP == PBG_CMP_COS;
  constexpr bool l2 = CMP == PBG_CMP_L2;  // as in fused_chunk_kernel: squared norms, positive scores in the direct form,
                                          // dS stored as -2 dLoss/dq, the rows' own terms added as the gradients leave
  constexpr int T0 = 4;         // column tiles per wave: of the score columns, and of a slice's 128 columns
  constexpr int kLossCols = 16; // score columns per lane of the 8 lanes that share a row (N <= 128)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  FusedGeom g;
  constexpr int kSliceLd = lds_stride(kSliceCols);
  g.D = kSliceCols; g.P = c.P; g.U = c.U; g.N = c.P + c.U; g.ldx = kSliceLd; g.lds = LDS ? LDS : f.lds;
  g.xn0 = f.xn[0]; g.xn1 = f.xn[1]; g.sc0 = f.sc[0]; g.sc1 = f.sc[1];
  g.sq0 = f.sq[0]; g.sq1 = f.sq[1]; g.rs0 = f.rs[0]; g.rs1 = f.rs[1]; g.cs0 = f.cs[0]; g.cs1 = f.cs[1];
  const int D = c.D, P = g.P, U = g.U, N = g.N, CP = c.C * c.P;
  constexpr int ldx = kSliceLd;
  const int lds_ = LDS ? LDS : f.lds;
  const int xn0 = g.xn0, xn1 = g.xn1, sc0 = g.sc0, sc1 = g.sc1;
  // CPLX (complex_diagonal, operators.py:118-152): the operator pairs coordinate h with h + D/2, so a slice holds 64 such
  // pairs instead of 128 consecutive coordinates -- LDS columns [0, 32) and [64, 96) are the real parts of the slice's
  // pairs 0..31 and 32..63, [32, 64) and [96, 128) their imaginary parts -- and a product that sums over all
  // coordinates does not care.  The partner of LDS column p is p ^ 32: in the stores, lane ^ 8; in the results of
  // the gradient products, register r ^ 2 of the same lane (for_each_out's columns are 16 r + 4 q).
  const int H = D >> 1;
  const int slices = CPLX ? (H + 63) / 64 : (D + kSliceCols - 1) / kSliceCols;  // (the last slice may be a partial one)
  const int rounds = (N + 15) >> 4;
  // LDS column p (a multiple of 4) of slice sl: its first coordinate (the last whole quad of the row, or of the
  // row's half, when the slice ends before p) and whether the column exists
  auto coord = [&](int sl, int p, bool* ok) -> int {
    if constexpr (CPLX) {
      const int h = sl * 64 + ((p >> 6) << 5) + (p & 31);
      *ok = h < H;
      return ((p >> 5) & 1) * H + min(h, H - 4);
    } else {
      const int col = sl * kSliceCols + p;
      *ok = col < D;
      return min(col, D - 4);
    }
  };
  const int p4 = (P + 3) & ~3;
  const int cp0 = xn0, cp1 = xn0 + p4 * lds_;  // cos: copies of the score blocks, in the operand rows' place between the sweeps
  int* ids = reinterpret_cast<int*>(lds + f.ids);
  const int rt = wave & 3, grp = wave >> 2, ct0 = grp * T0;

  for (int t = (int)threadIdx.x * 4; t < f.ids; t += kSliceThreads * 4)
    *reinterpret_cast<float4*>(&lds[t]) = make_float4(0.f, 0.f, 0.f, 0.f);
  lds_barrier();

  for (int kc = blockIdx.x; kc < num_chunks; kc += gridDim.x) {
    // The thread-to-cell mapping is the same for every chunk; hidden from the optimiser once per chunk, so
    // that it does not hoist every address of the loop body into registers that stay live (and spill).
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int m16 = lane & 15, kq = lane >> 4;
    const int hw = lane >> 5, c4 = (lane & 31) << 2;  // half a wave per row, four columns per lane
    const int k = kc / c.C, cc = kc - k * c.C;
    const int valid = (cc == c.C - 1) ? c.last : P;
    const int64_t rel = clamp_index(c.rel[k], c.num_relations);
    float w_edge = c.rel_weights[rel];
    if (c.edge_weight) w_edge *= c.edge_weight[(int64_t)k * c.B + min(cc * P + (tid >> 3), c.B - 1)];

    if (tid < kFusedIds) ids[tid] = c.fused_rowid[(int64_t)kc * kFusedIds + tid];
    lds_barrier();
    // this thread's rows: row j = 16 u + 2 wave + hw of side s, u < rounds (their ids are read from LDS where
    // they are needed: sixteen registers less)
    const int id_at = 2 * wave + hw;
    float4 v[2][8];
    float sqp[2][8];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int u = 0; u < 8; ++u) sqp[s][u] = 0.f;
    const uint32_t row_bytes = (uint32_t)D * 4u;
    auto load_slice = [&](int sl) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        // (columns past D: read from the row's last four instead and dropped when the slice is stored)
        bool ok;
        const char* w = reinterpret_cast<const char*>(c.side[s].w + coord(sl, c4, &ok));
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (u >= rounds) break;
          v[s][u] = *reinterpret_cast<const float4*>(w + (uint64_t)(uint32_t)max(ids[s * kFusedSide + 16 * u + id_at], 0) * row_bytes);
        }
      }
    };
    // The slice's rows (plus the type's global embedding, through the operator) into LDS.  kRaw: as they are, the
    // squared norms adding up; kNorms: the squared norms only, nothing stored; kPrepared: times the reciprocal norm
    // (cos), rounded to float16 numbers (HALF).
    constexpr int kRaw = 0, kPrepared = 1, kNorms = 2;
    auto store_slice = [&](int sl, int mode) {
      const bool raw = mode != kPrepared;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const float* glob = c.side[s].glob;
        bool col_ok;
        const int col = coord(sl, c4, &col_ok);
        float4 gv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (glob) gv = *reinterpret_cast<const float4*>(glob + col);
        // the relation's operator acts on side 1's rows (model.py:666-703); both kinds are local to a slice
        const bool has_op = s == 1 && c.op != PBG_OP_NONE;
        float4 par = make_float4(0.f, 0.f, 0.f, 0.f);
        const bool imag = CPLX && (c4 & 32) != 0;
        float4 par_o = par;  // CPLX: the partner's share of the parameter (imaginary for a real lane and the reverse)
        if (has_op) {
          if constexpr (CPLX) {
            par = *reinterpret_cast<const float4*>(imag ? c.side[1].p1 + (rel * H + col - H) : c.side[1].p0 + (rel * H + col));
            par_o = make_float4(__shfl_xor(par.x, 8), __shfl_xor(par.y, 8), __shfl_xor(par.z, 8), __shfl_xor(par.w, 8));
          } else {
            par = *reinterpret_cast<const float4*>(c.side[1].p0 + rel * D + col);
          }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (u >= rounds) break;
          const int j = 16 * u + 2 * wave + hw;
          float4 x = v[s][u];
          x.x += gv.x; x.y += gv.y; x.z += gv.z; x.w += gv.w;
          if (has_op) {
            if constexpr (CPLX) {
              // real: x_re a_re - x_im a_im; imaginary: x_im a_re + x_re a_im (operators.py:143-148)
              const float4 o = make_float4(__shfl_xor(x.x, 8), __shfl_xor(x.y, 8), __shfl_xor(x.z, 8), __shfl_xor(x.w, 8));
              if (imag) {
                x.x = x.x * par_o.x + o.x * par.x; x.y = x.y * par_o.y + o.y * par.y;
                x.z = x.z * par_o.z + o.z * par.z; x.w = x.w * par_o.w + o.w * par.w;
              } else {
                x.x = x.x * par.x - o.x * par_o.x; x.y = x.y * par.y - o.y * par_o.y;
                x.z = x.z * par.z - o.z * par_o.z; x.w = x.w * par.w - o.w * par_o.w;
              }
            } else if (c.op == PBG_OP_DIAGONAL) {
              x.x *= par.x; x.y *= par.y; x.z *= par.z; x.w *= par.w;
            } else {
              x.x += par.x; x.y += par.y; x.z += par.z; x.w += par.w;
            }
          }
          if (ids[s * kFusedSide + 16 * u + id_at] < 0 || !col_ok) x = make_float4(0.f, 0.f, 0.f, 0.f);
          if (cosn || l2) {
            if (raw) {
              sqp[s][u] += (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
            } else if (cosn) {
              const float inv = lds[(s ? g.sq1 : g.sq0) + min(j, N - 1)];
              x.x *= inv; x.y *= inv; x.z *= inv; x.w *= inv;
            }
          }
          if (HALF && !raw) {  // embs.half() (model.py:504-505)
            x.x = half_round(x.x); x.y = half_round(x.y); x.z = half_round(x.z); x.w = half_round(x.w);
          }
          if (j < N && mode != kNorms) *reinterpret_cast<float4*>(&lds[(s ? xn1 : xn0) + j * ldx + c4]) = x;
        }
      }
    };
    // cos: reciprocal norms (0 for a padded position: its row is zero); l2: squared norms as norm().pow(2)
    auto finish_norms = [&]() {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (u >= rounds) break;
          const float tot = half_sum_at_31(sqp[s][u]);  // complete in lanes 31 and 63
          const int j = 16 * u + 2 * wave + hw;
          const float nrm = sqrtf(tot);
          if ((lane & 31) == 31 && j < N)
            lds[(s ? g.sq1 : g.sq0) + j] = l2 ? nrm * nrm : (ids[s * kFusedSide + j] < 0 ? 0.f : 1.0f / nrm);
        }
    };
    constexpr bool pre_norms = HALF && cosn;  // the norms before the first product
    if (pre_norms) {
      load_slice(0);
      for (int sl = 0; sl < slices; ++sl) {
        store_slice(sl, kNorms);
        if (sl + 1 < slices) load_slice(sl + 1);
      }
      finish_norms();
      // (the first barrier of sweep 1 orders the norms before the stores that read them)
    }

    // ---- sweep 1: the score blocks ----
    float4v acc0[T0], acc1[T0];
#pragma unroll
    for (int ct = 0; ct < T0; ++ct) {
      acc0[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
      acc1[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
    }
    const bool score_live = rt * 16 < P && ct0 * 16 < N;
    const int ar = min(rt * 16 + m16, P - 1);
    float pos_part = 0.f;
    load_slice(0);
    for (int sl = 0; sl < slices; ++sl) {
      lds_barrier();  // the products of the previous slice (or of the previous chunk) have let go of the rows
      store_slice(sl, pre_norms || (HALF && !cosn) ? kPrepared : kRaw);
      lds_barrier();
      if (sl + 1 < slices) load_slice(sl + 1);
      if (l2 && tid < 4 * P) {  // positive scores in the direct form (model.py:267-274): this slice's share
        const int i = tid >> 2, qd = tid & 3;
        for (int d0 = qd; d0 < kSliceCols; d0 += 32) {
          float a[8], bb[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            a[u] = lds[xn0 + i * ldx + d0 + 4 * u];
            bb[u] = lds[xn1 + i * ldx + d0 + 4 * u];
          }
#pragma unroll
          for (int u = 0; u < 8; ++u) pos_part += (a[u] - bb[u]) * (a[u] - bb[u]);
        }
      }
      if (score_live) {
        // block b: rows = the positives of side 1 - b, columns = side b's negatives
        mfma_sweep_k16<T0, HALF>(lds, xn1 + ar * ldx, xn0 + (ct0 * 16 + m16) * ldx, 16 * ldx, kSliceCols / 16, 0, kq, acc0);
        mfma_sweep_k16<T0, HALF>(lds, xn0 + ar * ldx, xn1 + (ct0 * 16 + m16) * ldx, 16 * ldx, kSliceCols / 16, 0, kq, acc1);
      }
    }
    if ((cosn || l2) && !pre_norms) finish_norms();
    if (l2) {
      pos_part = quad_sum(pos_part);
      if (tid < 4 * P && (tid & 3) == 0) lds[f.pos + (tid >> 2)] = -sqrtf(fmaxf(pos_part, 1e-30f));
    }
    lds_barrier();  // every product has read its rows; the norms are there
    {
      const int row = rt * 16 + m16;
      const int n8 = (N + 7) & ~7;
      if (score_live && row < P) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const float4v* acc = b ? acc1 : acc0;
          constexpr bool scale = cosn && !pre_norms;  // (with the norms known beforehand the rows were normalised as they were stored)
          const float ia = scale ? lds[(b ? g.sq0 : g.sq1) + row] : 1.0f;
          const int at = (b ? sc1 : sc0) + row * lds_ + ct0 * 16 + 4 * kq;
          const int cat = (b ? cp1 : cp0) + row * lds_ + ct0 * 16 + 4 * kq;
#pragma unroll
          for (int ct = 0; ct < T0; ++ct) {
            const int col = (ct0 + ct) * 16 + 4 * kq;
            float sv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float x = acc[ct][r];
              if (scale) x *= ia * lds[(b ? g.sq1 : g.sq0) + min(col + r, N - 1)];
              sv[r] = col + r < N ? x : -INFINITY;
            }
            // (HALF: the positive score is the fp32 sum itself, model.py:177; the block holds float16 numbers)
            if (!l2 && b == 0 && row >= col && row < col + 4) {
              const int r = row - col;
              lds[f.pos + row] = r == 0 ? sv[0] : (r == 1 ? sv[1] : (r == 2 ? sv[2] : sv[3]));
            }
            if (HALF) {
#pragma unroll
              for (int r = 0; r < 4; ++r) sv[r] = half_round(sv[r]);
            }
            if (col < n8) {
              *reinterpret_cast<float4*>(&lds[at + ct * 16]) = make_float4(sv[0], sv[1], sv[2], sv[3]);
              if (cosn) *reinterpret_cast<float4*>(&lds[cat + ct * 16]) = make_float4(sv[0], sv[1], sv[2], sv[3]);
            }
          }
        }
      }
    }
    lds_barrier();

    // ---- the loss: side 0, then side 1; eight lanes per edge, columns interleaved ----
    for (int s = 0; s < 2; ++s) {
      if (tid < 8 * P) {
        const int i = tid >> 3, qd = tid & 7;
        const int row_at = (s ? sc1 : sc0) + i * lds_;
        float loss_w = 0.f, dpos_s = 0.f, rowsum = 0.f;
        int viol = 0;
        if (i >= valid) {
          for (int j = qd; j < lds_; j += 8) lds[row_at + j] = 0.f;
        } else {
          const float masked = l2 ? -INFINITY : -1e9f;  // model.py:566-580,836-839
          if (qd == (i & 7)) lds[row_at + i] = masked;
          if (valid < P)
            for (int j = valid + ((qd - valid) & 7); j < P; j += 8) lds[row_at + j] = masked;
          fused_row_loss<CMP, LOSS, kLossCols, HALF>(lds, row_at, s ? g.sq1 : g.sq0, l2 ? lds[(s ? g.sq0 : g.sq1) + i] : 0.f,
                                                        c.margin, 1.0f / (float)N, (N + 7) >> 3, lds[f.pos + i], w_edge, qd, &loss_w,
                                                        &dpos_s, &viol, &rowsum);
        }
        if (qd == 0) {
          if (l2) lds[(s ? g.rs1 : g.rs0) + i] = rowsum;
          lds[f.part + (s * 3 + 0) * P + i] = dpos_s;
          lds[f.part + (s * 3 + 1) * P + i] = loss_w;
          lds[f.part + (s * 3 + 2) * P + i] = __int_as_float(viol);
        }
      }
    }
    lds_barrier();
    // statistics out
    if (tid < P) {
      const int64_t job = (int64_t)k * CP + cc * P + tid;
      c.lossrow[job] = lds[f.part + 1 * P + tid] + lds[f.part + 4 * P + tid];
      c.violrow[job * 2] = __float_as_int(lds[f.part + 2 * P + tid]);
      c.violrow[job * 2 + 1] = __float_as_int(lds[f.part + 5 * P + tid]);
    }
    if (l2) {
      // column sums of the stored -2 dLoss/dq over the batch-negative columns of both blocks (before the fold
      // rewrites them), and dLoss/dpos of both sides together
      if (tid < 2 * P) {
        const int b = tid >= P, j = tid - b * P;
        float acc = 0.f;
        for (int i = 0; i < P; ++i) acc += lds[(b ? sc1 : sc0) + i * lds_ + j];
        lds[(b ? g.cs1 : g.cs0) + j] = acc;
      } else if (tid >= 256 && tid < 256 + P) {
        const int i = tid - 256;
        lds[f.dpos + i] = lds[f.part + 0 * P + i] + lds[f.part + 3 * P + i];
      }
      lds_barrier();
    }
    if (cosn) {
      // <y, dLoss/dy> of a row = sum over the scores it takes part in of dLoss/dscore * score:
      // per block the sums along its rows (the positives as left operands) and along its
      // columns (the negatives); masked and padded entries have a zero gradient
      if (tid < 2 * N) {
        const int b = tid >= N, j = tid - b * N;
        const int da = (b ? sc1 : sc0) + j, ca = (b ? cp1 : cp0) + j;
        float acc = 0.f;
        for (int i = 0; i < P; ++i) acc += lds[da + i * lds_] * lds[ca + i * lds_];
        lds[(b ? g.cs1 : g.cs0) + j] = acc;
      } else if (tid >= 256 && tid < 256 + 2 * P) {
        const int b = tid - 256 >= P, i = tid - 256 - b * P;
        const int da = (b ? sc1 : sc0) + i * lds_, ca = (b ? cp1 : cp0) + i * lds_;
        float acc = 0.f;
        for (int j = 0; j < N; ++j) acc += lds[da + j] * lds[ca + j];
        lds[(b ? g.rs1 : g.rs0) + i] = acc;
      }
      lds_barrier();
    }
    // the fold (see fused_chunk_kernel): G = dS_R[:, :P] + dS_L[:, :P]^T, dLoss/dpos on its diagonal
    {
      int i = tid / P, j = tid - i * P;
      const int di = kSliceThreads / P, dj = kSliceThreads - di * P;
      for (int e = tid; e < P * P; e += kSliceThreads) {
        float sum = lds[sc1 + i * lds_ + j] + lds[sc0 + j * lds_ + i];
        if (!l2 && i == j) sum += lds[f.part + 0 * P + i] + lds[f.part + 3 * P + i];
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
    // (the barrier at the head of sweep 2 orders the fold before the products)

    // ---- sweep 2: the gradient rows, slice by slice ----
    load_slice(0);
    for (int sl = 0; sl < slices; ++sl) {
      lds_barrier();
      store_slice(sl, kPrepared);
      lds_barrier();
      if (sl + 1 < slices) load_slice(sl + 1);
      // Where a finished quad of a gradient row goes: the row's place in the gradient array, at the operator's output
      // (dz, for the parameter stage) and, through the operator's transpose, at the raw row.  `lc`: the quad's LDS column.
      auto put = [&](float* out, float* dz, int lc, float4 r4, bool diag) {
        bool ok;
        const int col = coord(sl, ct0 * 16 + lc, &ok);
        if (!ok) return;
        if (dz) *reinterpret_cast<float4*>(dz + col) = r4;
        if (diag) {
          const float4 pv = *reinterpret_cast<const float4*>(c.side[1].p0 + rel * D + col);
          r4.x *= pv.x; r4.y *= pv.y; r4.z *= pv.z; r4.w *= pv.w;
        }
        *reinterpret_cast<float4*>(out + col) = r4;
      };
      // CPLX, a row the operator acted on: the real quad at LDS column lc and the imaginary one at lc + 32;
      // d/dx_re = a_re g_re + a_im g_im, d/dx_im = a_re g_im - a_im g_re
      auto put_pair = [&](float* out, float* dz, int lc, float4 gre, float4 gim) {
        bool ok;
        const int col = coord(sl, ct0 * 16 + lc, &ok);
        if (!ok) return;
        if (dz) {
          *reinterpret_cast<float4*>(dz + col) = gre;
          *reinterpret_cast<float4*>(dz + col + H) = gim;
        }
        const float4 are = *reinterpret_cast<const float4*>(c.side[1].p0 + (rel * H + col));
        const float4 aim = *reinterpret_cast<const float4*>(c.side[1].p1 + (rel * H + col));
        *reinterpret_cast<float4*>(out + col) = make_float4(are.x * gre.x + aim.x * gim.x, are.y * gre.y + aim.y * gim.y,
                                                            are.z * gre.z + aim.z * gim.z, are.w * gre.w + aim.w * gim.w);
        *reinterpret_cast<float4*>(out + col + H) = make_float4(are.x * gim.x - aim.x * gre.x, are.y * gim.y - aim.y * gre.y,
                                                                are.z * gim.z - aim.z * gre.z, are.w * gim.w - aim.w * gre.w);
      };
      // all quads of the lane's row: each through `adjust`, then to their places
      auto emit = [&](const float4v* acc, float* out, float* dz, bool has_op, auto&& adjust) {
        if constexpr (CPLX) {
          if (has_op) {
            float4 q4[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) q4[r] = adjust(16 * r + 4 * kq, make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]));
            put_pair(out, dz, 4 * kq, q4[0], q4[2]);
            put_pair(out, dz, 16 + 4 * kq, q4[1], q4[3]);
            return;
          }
        }
        const bool diag = has_op && c.op == PBG_OP_DIAGONAL;
        for_each_out<T0>(acc, kq, [&](int lc, float4 r4) { put(out, dz, lc, adjust(lc, r4), diag); });
      };
      // uniform negatives of side m: (dS_m[:, P:])^T (U x P) times the other side's positives
      for (int m = 0; m < 2; ++m) {
        const SideCtx& sd = c.side[m];
        const int dsn = m ? sc1 : sc0, bx = m ? xn0 : xn1, xs = m ? xn1 : xn0;
        if (rt * 16 >= U) continue;
        float4v acc[T0];
#pragma unroll
        for (int ct = 0; ct < T0; ++ct) acc[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
        const int au = min(rt * 16 + m16, U - 1);
        float asum = sweep_a_cols<T0, HALF>(lds, dsn + P + au, lds_, bx + ct0 * 16, ldx, kq, m16, (P + 3) >> 2, acc);
        if (l2) {  // the column sum of the stored -2 dLoss/dq: the lane's share, then the other three k slots'
          asum += __shfl_xor(asum, 16);
          asum += __shfl_xor(asum, 32);
        }
        const int u = rt * 16 + m16;
        if (u < U) {
          float* out = c.gr + ((int64_t)k * c.rk + sd.slot_uni + cc * U + u) * D;
          const int self_at = xs + (P + u) * ldx + ct0 * 16;
          const float inv = cosn ? lds[(m ? g.sq1 : g.sq0) + P + u] : 1.0f;
          const float tt = cosn ? lds[(m ? g.cs1 : g.cs0) + P + u] : 0.f;
          const bool has_op = m == 1 && c.op != PBG_OP_NONE;
          float* dz = (has_op && sd.dz) ? sd.dz + ((int64_t)k * sd.op_rows + c.B + cc * U + u) * D : nullptr;
          emit(acc, out, dz, has_op, [&](int col, float4 r4) {
            if (HALF) r4 = make_float4(half_round(r4.x), half_round(r4.y), half_round(r4.z), half_round(r4.w));
            if (cosn) {
              const float4 y = *reinterpret_cast<const float4*>(&lds[self_at + col]);
              r4.x = inv * (r4.x - tt * y.x); r4.y = inv * (r4.y - tt * y.y);
              r4.z = inv * (r4.z - tt * y.z); r4.w = inv * (r4.w - tt * y.w);
            }
            if (l2) {  // ||b||^2's share: minus the column sum times the row itself
              const float4 y = *reinterpret_cast<const float4*>(&lds[self_at + col]);
              r4.x -= asum * y.x; r4.y -= asum * y.y; r4.z -= asum * y.z; r4.w -= asum * y.w;
            }
            return r4;
          });
        }
      }
      // positives of side m: [G | dS_a[:, P:]] (P x N) times the other side's N rows
      for (int m = 0; m < 2; ++m) {
        const SideCtx& sd = c.side[m];
        const int dsa = m ? sc0 : sc1, bx = m ? xn0 : xn1, xs = m ? xn1 : xn0;
        if (rt * 16 >= P) continue;
        float4v acc[T0];
#pragma unroll
        for (int ct = 0; ct < T0; ++ct) acc[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
        const int ksteps = (N + 3) >> 2;
        sweep_a_rows<T0, HALF>(lds, dsa + ar * lds_, bx + ct0 * 16, ldx, kq, m16, ksteps >> 2, ksteps & 3, acc);
        const int i = rt * 16 + m16;
        if (i < valid) {
          float* out = c.gr + ((int64_t)k * c.rk + sd.slot_pos + cc * P + i) * D;
          const int self_at = xs + i * ldx + ct0 * 16;
          const float inv = cosn ? lds[(m ? g.sq1 : g.sq0) + i] : 1.0f;
          // the row was the left operand of block 1 - m, a batch negative (column i) of block m, and one of the positive pair
          float tt = 0.f;
          if (cosn)
            tt = lds[(m ? g.rs0 : g.rs1) + i] + lds[(m ? g.cs1 : g.cs0) + i] +
                 (lds[f.part + 0 * P + i] + lds[f.part + 3 * P + i]) * lds[f.pos + i];
          float l2_coef = 0.f, l2_pcoef = 0.f;
          const int other_at = bx + i * ldx + ct0 * 16;
          if (l2) {
            const float dpz = lds[f.dpos + i], pz = lds[f.pos + i];
            l2_coef = 2.0f * lds[(m ? g.rs0 : g.rs1) + i] - lds[(m ? g.cs1 : g.cs0) + i];
            l2_pcoef = pz * pz > 2e-30f ? dpz / pz : 0.f;
          }
          const bool has_op = m == 1 && c.op != PBG_OP_NONE;
          float* dz = (has_op && sd.dz) ? sd.dz + ((int64_t)k * sd.op_rows + cc * P + i) * D : nullptr;
          emit(acc, out, dz, has_op, [&](int col, float4 r4) {
            if (HALF) r4 = make_float4(half_round(r4.x), half_round(r4.y), half_round(r4.z), half_round(r4.w));
            if (cosn) {
              const float4 y = *reinterpret_cast<const float4*>(&lds[self_at + col]);
              r4.x = inv * (r4.x - tt * y.x); r4.y = inv * (r4.y - tt * y.y);
              r4.z = inv * (r4.z - tt * y.z); r4.w = inv * (r4.w - tt * y.w);
            }
            if (l2) {  // the row's own terms of ||a||^2 - 2ab + ||b||^2, and the positive pair's (see fused_emit)
              const float4 y = *reinterpret_cast<const float4*>(&lds[self_at + col]);
              const float4 o4 = *reinterpret_cast<const float4*>(&lds[other_at + col]);
              r4.x += l2_coef * y.x + l2_pcoef * (y.x - o4.x); r4.y += l2_coef * y.y + l2_pcoef * (y.y - o4.y);
              r4.z += l2_coef * y.z + l2_pcoef * (y.z - o4.z); r4.w += l2_coef * y.w + l2_pcoef * (y.w - o4.w);
            }
            return r4;
          });
        }
      }
    }
    lds_barrier();  // the last slice's products are done before the next chunk's ids and rows arrive
  }
}

template <int CMP, int LOSS, int LDS, bool HALF, bool CPLX>
int launch_sliced_as(const StepCtx& c, const FusedLayout& fl, size_t lds_bytes, hipStream_t s, int blocks) {
  static LdsLimit limit;
  const int rc = reserve_lds((const void*)sliced_chunk_kernel<CMP, LOSS, LDS, HALF, CPLX>, &limit, lds_bytes);
  if (rc != PBG_OK) return rc;
  hipLaunchKernelGGL((sliced_chunk_kernel<CMP, LOSS, LDS, HALF, CPLX>), dim3((unsigned)blocks), dim3(kSliceThreads), lds_bytes, s, c,
                     fl, c.K * c.C);
  return PBG_OK;
}

template <int CMP, int LDS, bool HALF, bool CPLX>
int launch_sliced_loss(const StepCtx& c, const FusedLayout& fl, size_t lds_bytes, hipStream_t s, int blocks) {
  switch (c.loss) {
    case PBG_LOSS_RANKING: return launch_sliced_as<CMP, PBG_LOSS_RANKING, LDS, HALF, CPLX>(c, fl, lds_bytes, s, blocks);
    case PBG_LOSS_LOGISTIC: return launch_sliced_as<CMP, PBG_LOSS_LOGISTIC, LDS, HALF, CPLX>(c, fl, lds_bytes, s, blocks);
    default: return launch_sliced_as<CMP, PBG_LOSS_SOFTMAX, LDS, HALF, CPLX>(c, fl, lds_bytes, s, blocks);
  }
}

template <int CMP, bool HALF, bool CPLX = false>
int launch_sliced_cmp(const StepCtx& c, const FusedLayout& fl, size_t lds_bytes, hipStream_t s, int blocks) {
  // 50 + 50 negatives (and everything else whose score rows come out at 104 floats)
  if (fl.lds == 104) return launch_sliced_loss<CMP, 104, HALF, CPLX>(c, fl, lds_bytes, s, blocks);
  return launch_sliced_loss<CMP, 0, HALF, CPLX>(c, fl, lds_bytes, s, blocks);
}

}  // namespace

int sliced_chunks(const StepCtx& c, const FusedLayout& fl, int blocks, hipStream_t s) {
  const size_t lds_bytes = (size_t)fl.total * sizeof(float);
  if (!c.fused_rowid) return fail(PBG_ERR_INVALID, "step: the sliced chunk kernel reads its row ids from fused_ids");
  // (complex_diagonal: with dot -- what fused_layout lets through)
  if (c.op == PBG_OP_COMPLEX_DIAGONAL) {
    if (c.half) return launch_sliced_cmp<PBG_CMP_DOT, true, true>(c, fl, lds_bytes, s, blocks);
    return launch_sliced_cmp<PBG_CMP_DOT, false, true>(c, fl, lds_bytes, s, blocks);
  }
  if (c.half) {  // (dot and cos only: the step's validation has refused the rest)
    if (c.cmp == PBG_CMP_COS) return launch_sliced_cmp<PBG_CMP_COS, true>(c, fl, lds_bytes, s, blocks);
    if (c.cmp == PBG_CMP_DOT) return launch_sliced_cmp<PBG_CMP_DOT, true>(c, fl, lds_bytes, s, blocks);
    return fail(PBG_ERR_UNSUPPORTED, "step: half_precision on the fused route is built for dot and cos");
  }
  if (c.cmp == PBG_CMP_COS) return launch_sliced_cmp<PBG_CMP_COS, false>(c, fl, lds_bytes, s, blocks);
  if (c.cmp == PBG_CMP_L2) return launch_sliced_cmp<PBG_CMP_L2, false>(c, fl, lds_bytes, s, blocks);
  return launch_sliced_cmp<PBG_CMP_DOT, false>(c, fl, lds_bytes, s, blocks);
}

}  // namespace pbg
