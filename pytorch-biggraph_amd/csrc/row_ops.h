// Wave-level row helpers shared by the step pipeline and the stand-alone
// operator / comparator / loss entry points.
//
// Layout of a row inside a wave: lane l owns elements {h, H + h} for
// h = l, l + 64, ... < H with H = ceil(D / 2), i.e. both halves of a complex
// pair sit in the same lane.
#pragma once

#include "pbg_internal.h"

namespace pbg {

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"):
// 64 random bits for (seed, counter, stream).  The uniform negatives of a step
// are drawn with it, one counter per negative, so a draw depends on nothing but
// its position and can be repeated anywhere (SimpleEmbedding.sample_entities,
// model.py:70-75, only fixes the distribution: uniform over the table's rows).
__host__ __device__ __forceinline__ uint64_t philox_u64(uint64_t seed, uint64_t counter, uint32_t stream) {
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = stream, c3 = 0u;
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return ((uint64_t)c1 << 32) | c0;
}
// id of uniform negative number `flat` of side `side`, in [0, num_rows): the high
// word of (32 random bits x num_rows) for tables below 2^32 rows (no division;
// the same 2^-32 * num_rows departure from uniformity as a 32-bit draw modulo
// num_rows), a 64-bit remainder beyond.
__host__ __device__ __forceinline__ int64_t sampled_row(uint64_t seed, uint64_t flat, uint32_t side, int64_t num_rows) {
  const uint64_t r = philox_u64(seed, flat, side);
  if ((uint64_t)num_rows <= 0xffffffffull) return (int64_t)(((r & 0xffffffffull) * (uint64_t)num_rows) >> 32);
  return (int64_t)(r % (uint64_t)num_rows);
}

// Cross-lane reductions with DPP moves (ALU-rate) instead of LDS permutes: four
// steps fold a row of 16 lanes onto itself (quad swaps, half-row mirror, row
// mirror), two row broadcasts carry the row sums into lane 63, which is then
// read back as a scalar.  Every lane returns the total.
template <int CTRL, int ROW_MASK, int BANK_MASK>
__device__ __forceinline__ int dpp_i(int old, int v) {
  return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, BANK_MASK, false);
}
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float old, float v) {
  return __int_as_float(dpp_i<CTRL, ROW_MASK, BANK_MASK>(__float_as_int(old), __float_as_int(v)));
}
constexpr int kDppQuadSwap1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kDppRowBcast15 = 0x142;   // lane 15 of each row -> the next row
constexpr int kDppRowBcast31 = 0x143;   // lane 31 -> rows 2 and 3

// sum over each row of 16 lanes, left in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f<kDppQuadSwap1>(0.f, v);
  v += dpp_f<kDppQuadSwap2>(0.f, v);
  v += dpp_f<kDppRowHalfMirror>(0.f, v);
  v += dpp_f<kDppRowMirror>(0.f, v);
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  v += dpp_f<kDppRowBcast15, 0xa>(0.f, v);
  v += dpp_f<kDppRowBcast31, 0xc>(0.f, v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
// sums of lanes 0..31 and of lanes 32..63: valid in lane 31 and lane 63 respectively
__device__ __forceinline__ float half_sum_at_31(float v) {
  v = row16_sum(v);
  v += dpp_f<kDppRowBcast15, 0xa>(0.f, v);
  return v;
}
__device__ __forceinline__ int wave_sum_int(int v) {
  v += dpp_i<kDppQuadSwap1, 0xf, 0xf>(0, v);
  v += dpp_i<kDppQuadSwap2, 0xf, 0xf>(0, v);
  v += dpp_i<kDppRowHalfMirror, 0xf, 0xf>(0, v);
  v += dpp_i<kDppRowMirror, 0xf, 0xf>(0, v);
  v += dpp_i<kDppRowBcast15, 0xa, 0xf>(0, v);
  v += dpp_i<kDppRowBcast31, 0xc, 0xf>(0, v);
  return __builtin_amdgcn_readlane(v, 63);
}
// reductions over the 4 lanes of a quad, result in all 4
__device__ __forceinline__ float quad_sum(float v) {
  v += dpp_f<kDppQuadSwap1>(0.f, v);
  v += dpp_f<kDppQuadSwap2>(0.f, v);
  return v;
}
__device__ __forceinline__ float quad_max(float v) {
  v = fmaxf(v, dpp_f<kDppQuadSwap1>(v, v));
  v = fmaxf(v, dpp_f<kDppQuadSwap2>(v, v));
  return v;
}
__device__ __forceinline__ int quad_sum_int(int v) {
  v += dpp_i<kDppQuadSwap1, 0xf, 0xf>(0, v);
  v += dpp_i<kDppQuadSwap2, 0xf, 0xf>(0, v);
  return v;
}
struct WaveReduce {  // a row spread over the 64 lanes of a wave
  static constexpr int kStep = 64;
  static __device__ __forceinline__ float sum(float v);
  static __device__ __forceinline__ float max(float v);
  static __device__ __forceinline__ int sum_int(int v);
};
struct QuadReduce {  // a row spread over the 4 lanes of a quad
  static constexpr int kStep = 4;
  static __device__ __forceinline__ float sum(float v) { return quad_sum(v); }
  static __device__ __forceinline__ float max(float v) { return quad_max(v); }
  static __device__ __forceinline__ int sum_int(int v) { return quad_sum_int(v); }
};
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<kDppQuadSwap1>(v, v));
  v = fmaxf(v, dpp_f<kDppQuadSwap2>(v, v));
  v = fmaxf(v, dpp_f<kDppRowHalfMirror>(v, v));
  v = fmaxf(v, dpp_f<kDppRowMirror>(v, v));
  v = fmaxf(v, dpp_f<kDppRowBcast15, 0xa>(v, v));
  v = fmaxf(v, dpp_f<kDppRowBcast31, 0xc>(v, v));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float WaveReduce::sum(float v) { return wave_sum(v); }
__device__ __forceinline__ float WaveReduce::max(float v) { return wave_max(v); }
__device__ __forceinline__ int WaveReduce::sum_int(int v) { return wave_sum_int(v); }

template <int NVH>
struct RowV {
  float a[2][NVH];
};

template <int NVH>
__device__ __forceinline__ RowV<NVH> row_zero() {
  RowV<NVH> r;
#pragma unroll
  for (int v = 0; v < NVH; ++v) r.a[0][v] = r.a[1][v] = 0.f;
  return r;
}
template <int NVH>
__device__ __forceinline__ RowV<NVH> row_load(const float* __restrict__ p, int D, int H, int lane) {
  RowV<NVH> r;
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    const int h = v * kWave + lane;
    r.a[0][v] = (h < H) ? p[h] : 0.f;
    r.a[1][v] = (h < H && H + h < D) ? p[H + h] : 0.f;
  }
  return r;
}
template <int NVH>
__device__ __forceinline__ void row_store(float* __restrict__ p, const RowV<NVH>& r, int D, int H, int lane) {
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    const int h = v * kWave + lane;
    if (h < H) p[h] = r.a[0][v];
    if (h < H && H + h < D) p[H + h] = r.a[1][v];
  }
}
// The value a float16 tensor would hold for x (round to nearest even; beyond 65504: infinity), as fp32.
__device__ __forceinline__ float half_round(float x) { return (float)(_Float16)x; }
// config.half_precision: the prepared row as `embs.half()` leaves it (model.py:504-505)
template <int NVH>
__device__ __forceinline__ void row_round_half(RowV<NVH>& y) {
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    y.a[0][v] = half_round(y.a[0][v]);
    y.a[1][v] = half_round(y.a[1][v]);
  }
}
template <int NVH>
__device__ __forceinline__ float row_dot(const RowV<NVH>& x, const RowV<NVH>& y) {  // per-lane partial
  float acc = 0.f;
#pragma unroll
  for (int v = 0; v < NVH; ++v) acc += x.a[0][v] * y.a[0][v] + x.a[1][v] * y.a[1][v];
  return acc;
}
template <int NVH>
__device__ __forceinline__ void row_axpy(RowV<NVH>& y, float alpha, const RowV<NVH>& x) {
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    y.a[0][v] += alpha * x.a[0][v];
    y.a[1][v] += alpha * x.a[1][v];
  }
}

// y = op_r(x) for the element-wise operators (operators.py:59-84,128-157 and
// their dynamic twins :212-249,306-338).  `linear` is a GEMM and not handled here.
template <int NVH>
__device__ __forceinline__ RowV<NVH> op_forward(int op, const RowV<NVH>& x, const float* __restrict__ p0,
                                                const float* __restrict__ p1, int64_t r, int D, int H, int lane) {
  RowV<NVH> y = x;
  if (op == PBG_OP_DIAGONAL || op == PBG_OP_TRANSLATION) {
    const float* p = p0 + r * D;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      const int h = v * kWave + lane;
      const float q0 = (h < H) ? p[h] : 0.f;
      const float q1 = (h < H && H + h < D) ? p[H + h] : 0.f;
      if (op == PBG_OP_DIAGONAL) {
        y.a[0][v] = q0 * x.a[0][v];
        y.a[1][v] = q1 * x.a[1][v];
      } else {
        y.a[0][v] = x.a[0][v] + q0;
        y.a[1][v] = x.a[1][v] + q1;
      }
    }
  } else if (op == PBG_OP_COMPLEX_DIAGONAL) {
    const float* re = p0 + r * H;
    const float* im = p1 + r * H;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      const int h = v * kWave + lane;
      const float br = (h < H) ? re[h] : 0.f;
      const float bi = (h < H) ? im[h] : 0.f;
      y.a[0][v] = x.a[0][v] * br - x.a[1][v] * bi;
      y.a[1][v] = x.a[0][v] * bi + x.a[1][v] * br;
    }
  }
  return y;
}

// dx = (d op_r / dx)^T dz for the element-wise operators.
template <int NVH>
__device__ __forceinline__ RowV<NVH> op_backward(int op, const RowV<NVH>& dz, const float* __restrict__ p0,
                                                 const float* __restrict__ p1, int64_t r, int D, int H, int lane) {
  RowV<NVH> dx = dz;
  if (op == PBG_OP_DIAGONAL) {
    const float* p = p0 + r * D;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      const int h = v * kWave + lane;
      dx.a[0][v] = ((h < H) ? p[h] : 0.f) * dz.a[0][v];
      dx.a[1][v] = ((h < H && H + h < D) ? p[H + h] : 0.f) * dz.a[1][v];
    }
  } else if (op == PBG_OP_COMPLEX_DIAGONAL) {
    const float* re = p0 + r * H;
    const float* im = p1 + r * H;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      const int h = v * kWave + lane;
      const float br = (h < H) ? re[h] : 0.f;
      const float bi = (h < H) ? im[h] : 0.f;
      dx.a[0][v] = br * dz.a[0][v] + bi * dz.a[1][v];
      dx.a[1][v] = br * dz.a[1][v] - bi * dz.a[0][v];
    }
  }
  return dx;
}

// N3 regularizer (regularizers.py:51-97) on one prepared row y: adds
// d (coef * sum m^3) / dy = 3 coef m y to dy and returns this lane's share of
// sum m^3, where m is the modulus of a complex coordinate (y[e], y[e + D/2]) for
// complex_diagonal (operators.py:154-157) and |y[e]| otherwise (operators.py:42-43).
template <int NVH>
__device__ __forceinline__ float n3_term(int op, float coef, RowV<NVH>& dy, const RowV<NVH>& y) {
  float cubes = 0.f;
  const float c3 = 3.0f * coef;
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    if (op == PBG_OP_COMPLEX_DIAGONAL) {
      const float m = sqrtf(y.a[0][v] * y.a[0][v] + y.a[1][v] * y.a[1][v]);
      dy.a[0][v] += c3 * m * y.a[0][v];
      dy.a[1][v] += c3 * m * y.a[1][v];
      cubes += m * m * m;
    } else {
      const float m0 = fabsf(y.a[0][v]), m1 = fabsf(y.a[1][v]);
      dy.a[0][v] += c3 * m0 * y.a[0][v];
      dy.a[1][v] += c3 * m1 * y.a[1][v];
      cubes += m0 * m0 * m0 + m1 * m1 * m1;
    }
  }
  return cubes;
}

// comparator.prepare (model.py:161-162,187-192,251-252), in place; returns the
// per-row aux value: 1/norm for cos, norm^2 for l2 (model.py:228-229).
template <int NVH>
__device__ __forceinline__ float prepare_row(int cmp, RowV<NVH>& y) {
  if (cmp == PBG_CMP_DOT) return 0.f;
  const float nrm = sqrtf(wave_sum(row_dot(y, y)));
  if (cmp == PBG_CMP_COS) {
    const float inv = 1.0f / nrm;
#pragma unroll
    for (int v = 0; v < NVH; ++v) {
      y.a[0][v] *= inv;
      y.a[1][v] *= inv;
    }
    return inv;
  }
  return nrm * nrm;
}

// gradient through comparator.prepare: cos: dz = (dy - y (y . dy)) / norm.
template <int NVH>
__device__ __forceinline__ RowV<NVH> prepare_backward(int cmp, const RowV<NVH>& dy, const RowV<NVH>& y, float aux) {
  if (cmp != PBG_CMP_COS) return dy;
  const float dot = wave_sum(row_dot(y, dy));
  RowV<NVH> dz;
#pragma unroll
  for (int v = 0; v < NVH; ++v) {
    dz.a[0][v] = aux * (dy.a[0][v] - y.a[0][v] * dot);
    dz.a[1][v] = aux * (dy.a[1][v] - y.a[1][v] * dot);
  }
  return dz;
}

__device__ __forceinline__ int64_t clamp_index(int64_t v, int64_t n) { return v < 0 ? 0 : (v >= n ? n - 1 : v); }

__device__ __forceinline__ float softplusf(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float sigmoidf(float z) {
  if (z >= 0.f) return 1.0f / (1.0f + expf(-z));
  const float e = expf(z);
  return e / (1.0f + e);
}
// e^(x - m) for the softmax's terms (x <= m): the hardware's 2^y (1 ulp) on (x - m) log2 e, the subtraction first --
// the correctly rounded expf costs a dozen instructions, twice per score of a row of a thousand, which made the
// loss kernel arithmetic-bound; the same form as the streaming route's, and every term of a row (the positive's
// included) goes through it, so that terms that must cancel still do.
__device__ __forceinline__ float exp_below(float x, float m) { return __builtin_amdgcn_exp2f((x - m) * 1.4426950408889634f); }

// softplus(z) and sigmoid(z) from one exponential (the same values as the two functions above)
__device__ __forceinline__ float softplus_sigmoid(float z, float* sigmoid) {
  const float e = expf(-fabsf(z));
  *sigmoid = (z >= 0.f ? 1.0f : e) / (1.0f + e);
  return fmaxf(z, 0.f) + log1pf(e);
}

}  // namespace pbg
