// fp32 matrix products of 16 x 16 tiles out of LDS (v_mfma_f32_16x16x4_f32), the
// reductions over 8 adjacent lanes and the LDS-only workgroup barrier shared by
// the kernels that keep a chunk in LDS.
//
// HALF variants of the products (config.half_precision: every operand value is a
// float16 number held as fp32): the four values of k that a lane feeds to four
// fp32 steps go, packed to fp16 (exactly), into ONE v_mfma_f32_16x16x16_f16 --
// lane group q holds four of the instruction's 16 k in both operands, and which k
// a slot stands for is free as long as both operands agree.  Sums stay fp32.
#pragma once

#include "pbg_internal.h"
#include "row_ops.h"

namespace pbg {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x2v __attribute__((ext_vector_type(2)));

// Four float16 numbers held as fp32, packed (the conversion is exact for such values).
__device__ __forceinline__ half4v pack_half4(float x, float y, float z, float w) {
  union {
    struct { fp16x2v lo, hi; } p;
    half4v h;
  } u;
  u.p.lo = __builtin_amdgcn_cvt_pkrtz(x, y);
  u.p.hi = __builtin_amdgcn_cvt_pkrtz(z, w);
  return u.h;
}
// One k per lane group (a single fp32 step's operands) as an fp16 instruction: the other three slots are zero.
__device__ __forceinline__ float4v mfma_step(float b, float a, float4v acc, bool half) {
  if (half) return __builtin_amdgcn_mfma_f32_16x16x16f16(pack_half4(b, 0.f, 0.f, 0.f), pack_half4(a, 0.f, 0.f, 0.f), acc, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x4f32(b, a, acc, 0, 0, 0);
}

// reductions over 8 adjacent lanes, result in every lane of the group
__device__ __forceinline__ float oct_sum(float v) {
  v = quad_sum(v);
  return v + dpp_f<kDppRowHalfMirror>(0.f, v);  // lane i of a half-row takes lane 7 - i: the other quad
}
__device__ __forceinline__ float oct_max(float v) {
  v = quad_max(v);
  return fmaxf(v, dpp_f<kDppRowHalfMirror>(v, v));
}
__device__ __forceinline__ int oct_sum_int(int v) {
  v = quad_sum_int(v);
  return v + dpp_i<kDppRowHalfMirror, 0xf, 0xf>(0, v);
}

// v, or zeros: by a bit mask (a select between a loaded value and a constant makes
// the compiler index a two-entry stack array).
__device__ __forceinline__ float4 keep_if(float4 v, bool keep) {
  const int m = keep ? -1 : 0;
  return make_float4(__int_as_float(__float_as_int(v.x) & m), __int_as_float(__float_as_int(v.y) & m),
                     __int_as_float(__float_as_int(v.z) & m), __int_as_float(__float_as_int(v.w) & m));
}

// Workgroup barrier of the LDS-resident kernels.  Only LDS traffic has to be ordered across
// it: the waves exchange data through LDS alone, rows on their way from HBM into
// registers and results on their way to HBM belong to one wave each.
// __syncthreads() would also wait for those (its fences drain the vector memory
// counter), which puts the latency of the gather on every step's critical path.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- MFMA products of the LDS-resident kernels ----
// Every product is formed as (B^T A^T): the instruction's first operand comes
// from B, so a lane ends up with four consecutive values of ONE row of A B.
//
// B operand of one k-step when k runs along B's LDS rows (the gradient products:
// B = a side's operand rows, columns = embedding coordinates).  A wave covers NCT
// column tiles starting at a multiple of 16.  Which 16 columns form a tile is
// free as long as the results are read back the same way, so lane m = lane & 15
// reads NCT consecutive floats with ONE wide load, at a place chosen so that the
// results leave the wave in 64-byte runs: the instruction's row index i = m ends
// up as i = 4q + r in lane group q, result register r, and a lane stores four
// results of four registers as one 128-bit word.
//   4-tile part: lane m reads columns 16 (m & 3) + 4 (m >> 2) + t, t = 0..3 (tile t)
//                -> register r of tile t holds column 16 r + 4 q + t
//   2-tile part: lane m reads columns 16 ((m & 3) >> 1) + 4 (m >> 2) + 2 (m & 1) + t
//                -> register r of tile t holds column 16 (r >> 1) + 4 q + 2 (r & 1) + t
//   1-tile part: lane m reads column m -> register r holds column 4 q + r
// NCT = 3 is a 2-tile part followed by a 1-tile part 32 columns on.
template <int NCT>
__device__ __forceinline__ void load_b(const float* lds, int at, int m, float* b) {
  if constexpr (NCT == 4) {
    const float4 v = *reinterpret_cast<const float4*>(&lds[at + 16 * (m & 3) + 4 * (m >> 2)]);
    b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
  } else if constexpr (NCT >= 2) {
    const float2 v = *reinterpret_cast<const float2*>(&lds[at + 16 * ((m & 3) >> 1) + 4 * (m >> 2) + 2 * (m & 1)]);
    b[0] = v.x; b[1] = v.y;
    if constexpr (NCT == 3) b[2] = lds[at + 32 + m];
  } else {
    b[0] = lds[at + m];
  }
}

// The results of such a product: fn(column offset from the wave's first column,
// four consecutive values of the lane's row), q = lane >> 4.
template <int NCT, class F>
__device__ __forceinline__ void for_each_out(const float4v* acc, int q, F&& fn) {
  if constexpr (NCT == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) fn(16 * r + 4 * q, make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]));
  } else if constexpr (NCT >= 2) {
    fn(4 * q, make_float4(acc[0][0], acc[1][0], acc[0][1], acc[1][1]));
    fn(16 + 4 * q, make_float4(acc[0][2], acc[1][2], acc[0][3], acc[1][3]));
    if constexpr (NCT == 3) fn(32 + 4 * q, make_float4(acc[2][0], acc[2][1], acc[2][2], acc[2][3]));
  } else {
    fn(4 * q, make_float4(acc[0][0], acc[0][1], acc[0][2], acc[0][3]));
  }
}

// acc += A B with A's k along its LDS row (a_at = element (row, 0) of the lane's A
// row): a lane reads four consecutive k as one 128-bit word, so the k slots of
// step r of group g hold k = 16 g + 4 kq + r, kq = lane >> 4; B's rows k start at
// b_at + k * ldb.  `groups` groups of 16 k, then `rest` single steps (slot kq
// holds k = 16 groups + 4 step + kq).  The operands of the next group are in
// flight while the MFMAs of the current one issue; reads run up to 16 k past the
// end (the caller's buffers keep finite values there).
template <int NCT>
struct RowOperands {
  float4 a;
  float b[4][NCT];
  __device__ __forceinline__ void load(const float* lds, int a_at, int b_at, int ldb, int m) {
    a = *reinterpret_cast<const float4*>(&lds[a_at]);
#pragma unroll
    for (int r = 0; r < 4; ++r) load_b<NCT>(lds, b_at + r * ldb, m, b[r]);
  }
  template <bool HALF>
  __device__ __forceinline__ void mma(float4v* acc) const {
    if constexpr (HALF) {
      const half4v ha = pack_half4(a.x, a.y, a.z, a.w);
#pragma unroll
      for (int t = 0; t < NCT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(pack_half4(b[0][t], b[1][t], b[2][t], b[3][t]), ha, acc[t], 0, 0, 0);
    } else {
      const float av[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[r][t], av[r], acc[t], 0, 0, 0);
    }
  }
};

template <int NCT, bool HALF = false>
__device__ __forceinline__ void sweep_a_rows(const float* lds, int a_at, int b_at, int ldb, int kq, int m, int groups,
                                             int rest, float4v* acc) {
  a_at += 4 * kq;
  b_at += 4 * kq * ldb;
  RowOperands<NCT> x, y;  // two operand sets taking turns, see mfma_sweep_k16
  x.load(lds, a_at, b_at, ldb, m);
  int gk = 0;
  for (; gk + 2 <= groups; gk += 2) {
    y.load(lds, a_at + 16, b_at + 16 * ldb, ldb, m);
    __builtin_amdgcn_sched_barrier(0);
    x.template mma<HALF>(acc);
    __builtin_amdgcn_sched_barrier(0);
    a_at += 32;
    b_at += 32 * ldb;
    x.load(lds, a_at, b_at, ldb, m);
    __builtin_amdgcn_sched_barrier(0);
    y.template mma<HALF>(acc);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (gk < groups) {
    x.template mma<HALF>(acc);
    a_at += 16;
    b_at += 16 * ldb;
  }
  a_at -= 3 * kq;
  b_at -= 3 * kq * ldb;
  for (int ks = 0; ks < rest; ++ks) {
    const float a1 = lds[a_at];
    float b1[NCT];
    load_b<NCT>(lds, b_at, m, b1);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = mfma_step(b1[t], a1, acc[t], HALF);
    a_at += 4;
    b_at += 4 * ldb;
  }
}

// acc += A B with A's k along LDS rows too (the transposed score block of the
// uniform negatives' gradient): the lane's A element of step ks is at a_at +
// (4 ks + kq) * lda.  Returns the sum of the A elements the lane has fed (its
// share of a column sum of the score block).  Reads up to two steps past the end.
template <int NCT, bool HALF = false>
__device__ __forceinline__ float sweep_a_cols(const float* lds, int a_at, int lda, int b_at, int ldb, int kq, int m,
                                              int ksteps, float4v* acc) {
  a_at += kq * lda;
  b_at += kq * ldb;
  if constexpr (HALF) {  // four steps' operands per instruction; nothing is read past the end
    float asum = 0.f;
    int ks = 0;
    for (; ks + 4 <= ksteps; ks += 4) {
      float a[4], b[4][NCT];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        a[r] = lds[a_at + 4 * r * lda];
        load_b<NCT>(lds, b_at + 4 * r * ldb, m, b[r]);
      }
      const half4v ha = pack_half4(a[0], a[1], a[2], a[3]);
#pragma unroll
      for (int t = 0; t < NCT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(pack_half4(b[0][t], b[1][t], b[2][t], b[3][t]), ha, acc[t], 0, 0, 0);
      asum += (a[0] + a[1]) + (a[2] + a[3]);
      a_at += 16 * lda;
      b_at += 16 * ldb;
    }
    for (; ks < ksteps; ++ks) {
      const float a1 = lds[a_at];
      float b1[NCT];
      load_b<NCT>(lds, b_at, m, b1);
#pragma unroll
      for (int t = 0; t < NCT; ++t) acc[t] = mfma_step(b1[t], a1, acc[t], true);
      asum += a1;
      a_at += 4 * lda;
      b_at += 4 * ldb;
    }
    return asum;
  }
  float ax = lds[a_at], ay, asum = 0.f;
  float bx[NCT], by[NCT];
  load_b<NCT>(lds, b_at, m, bx);
  int ks = 0;
  for (; ks + 2 <= ksteps; ks += 2) {
    ay = lds[a_at + 4 * lda];
    load_b<NCT>(lds, b_at + 4 * ldb, m, by);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(bx[t], ax, acc[t], 0, 0, 0);
    asum += ax;
    __builtin_amdgcn_sched_barrier(0);
    a_at += 8 * lda;
    b_at += 8 * ldb;
    ax = lds[a_at];
    load_b<NCT>(lds, b_at, m, bx);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(by[t], ay, acc[t], 0, 0, 0);
    asum += ay;
    __builtin_amdgcn_sched_barrier(0);
  }
  if (ks < ksteps) {
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(bx[t], ax, acc[t], 0, 0, 0);
    asum += ax;
  }
  return asum;
}

// The same product for operands whose k runs along the LDS rows (both operands
// of the score products): a lane reads FOUR consecutive k of its row as one
// 128-bit word and feeds them to four MFMAs, so the k slots of step r hold
// k = 16 g + 4 (lane >> 4) + r for group g -- any assignment of k to slots is
// right as long as both operands use the same one.  A quarter of the LDS
// instructions of mfma_sweep; `groups` groups of 16 k, then `rest` single steps.
// a_at / b_at address element (row, 0).  Reads up to 15 floats past the last k of
// a row (never used: the groups cover whole multiples of 16 only).
template <int T>
struct K16Operands {
  float4 a, b[T];
  __device__ __forceinline__ void load(const float* lds, int a_at, int b_at, int b_tile) {
    a = *reinterpret_cast<const float4*>(&lds[a_at]);
#pragma unroll
    for (int ct = 0; ct < T; ++ct) b[ct] = *reinterpret_cast<const float4*>(&lds[b_at + ct * b_tile]);
  }
  template <bool HALF>
  __device__ __forceinline__ void mma(float4v* acc) const {
    if constexpr (HALF) {
      const half4v ha = pack_half4(a.x, a.y, a.z, a.w);
#pragma unroll
      for (int ct = 0; ct < T; ++ct)
        acc[ct] = __builtin_amdgcn_mfma_f32_16x16x16f16(pack_half4(b[ct].x, b[ct].y, b[ct].z, b[ct].w), ha, acc[ct], 0, 0, 0);
    } else {
#pragma unroll
      for (int ct = 0; ct < T; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[ct].x, a.x, acc[ct], 0, 0, 0);
#pragma unroll
      for (int ct = 0; ct < T; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[ct].y, a.y, acc[ct], 0, 0, 0);
#pragma unroll
      for (int ct = 0; ct < T; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[ct].z, a.z, acc[ct], 0, 0, 0);
#pragma unroll
      for (int ct = 0; ct < T; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[ct].w, a.w, acc[ct], 0, 0, 0);
    }
  }
};

template <int T, bool HALF = false>
__device__ __forceinline__ void mfma_sweep_k16(const float* lds, int a_at, int b_at, int b_tile, int groups, int rest,
                                               int kq, float4v* acc) {
  a_at += 4 * kq;
  b_at += 4 * kq;
  // Two operand sets take turns: the operands of group g + 1 are requested before the
  // matrix instructions of group g issue, and nothing is copied between the sets.  The
  // scheduling barriers keep the compiler from sinking the loads down to their first
  // use, which would expose the LDS latency once per group.
  K16Operands<T> x, y;
  x.load(lds, a_at, b_at, b_tile);
  int gk = 0;
  for (; gk + 2 <= groups; gk += 2) {
    y.load(lds, a_at + 16, b_at + 16, b_tile);
    __builtin_amdgcn_sched_barrier(0);
    x.template mma<HALF>(acc);
    __builtin_amdgcn_sched_barrier(0);
    a_at += 32;
    b_at += 32;
    x.load(lds, a_at, b_at, b_tile);
    __builtin_amdgcn_sched_barrier(0);
    y.template mma<HALF>(acc);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (gk < groups) {
    x.template mma<HALF>(acc);
    a_at += 16;
    b_at += 16;
  }
  a_at -= 3 * kq;  // single steps: slot kq holds k = 16 groups + 4 step + kq
  b_at -= 3 * kq;
  for (int ks = 0; ks < rest; ++ks) {
    const float a1 = lds[a_at];
    float b1[T];
#pragma unroll
    for (int ct = 0; ct < T; ++ct) b1[ct] = lds[b_at + ct * b_tile];
#pragma unroll
    for (int ct = 0; ct < T; ++ct) acc[ct] = mfma_step(b1[ct], a1, acc[ct], HALF);
    a_at += 4;
    b_at += 4;
  }
}

// Row stride >= n that is 8 mod 16 floats: 128-bit reads of "16 rows, one word at 4 (lane >> 4)"
// -- an MFMA operand with k along the LDS row -- are then free of bank conflicts (ds_read_b128
// runs in 4 passes over lanes {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same + 32, each
// pass over 16 groups of 16 bytes; measured), and so are 32-bit reads of 4 rows x 8 columns.
constexpr int lds_stride(int n) {
  int ld = (n + 3) / 4 * 4;
  while (ld % 16 != 8) ld += 4;
  return ld;
}

}  // namespace pbg
