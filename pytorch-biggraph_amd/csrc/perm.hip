// GPU versions of the reference's native helpers (torchbiggraph/util.cpp):
// reverse_permutation, shuffle, randperm and sub_bucket.  All are HBM-bound
// integer / byte movers.
#include "pbg_internal.h"

namespace pbg {
namespace {

__global__ void reverse_permutation_kernel(const int64_t* __restrict__ perm, int64_t n, int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t p = perm[i];
  if (p >= 0 && p < n) out[p] = i;
}

// scratch[perm[i]] = rows[i]; one wave per row, WORD-sized elements.
template <typename WORD>
__global__ __launch_bounds__(256) void scatter_rows_kernel(const WORD* __restrict__ rows, int64_t n, int64_t row_words,
                                                           const int64_t* __restrict__ perm, WORD* __restrict__ scratch,
                                                           int32_t* __restrict__ oob_flag) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= n) return;
  const int64_t p = perm[i];
  if (p < 0 || p >= n) {
    if (lane == 0 && oob_flag) *oob_flag = 1;
    return;
  }
  const WORD* src = rows + i * row_words;
  WORD* dst = scratch + p * row_words;
  for (int64_t w = lane; w < row_words; w += kWave) dst[w] = src[w];
}

// Rows of at most 16 * LPR bytes (a multiple of 16): LPR lanes per row, one 128-bit word per
// lane, U rows per lane group in flight.  The reads are consecutive rows (coalesced), the writes
// land at perm's rows; a 400-byte row alone would leave 39 of a wave's 64 lanes idle.
template <int LPR, int U>
__global__ __launch_bounds__(256) void scatter_rows_multi_kernel(const uint4* __restrict__ rows, int64_t n,
                                                                 int row_words, const int64_t* __restrict__ perm,
                                                                 uint4* __restrict__ out,
                                                                 int32_t* __restrict__ oob_flag) {
  constexpr int kGroups = kWave / LPR;
  const int lane = threadIdx.x & 63;
  const int q = lane / LPR, v = lane % LPR;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t base = wave * (kGroups * U) + q;
  const bool col_ok = v < row_words;
  int64_t p[U];
  uint4 x[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kGroups;
    p[u] = i < n ? perm[i] : -1;
    x[u] = make_uint4(0u, 0u, 0u, 0u);
    if (i < n && col_ok) x[u] = rows[i * row_words + v];
  }
  bool bad = false;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kGroups;
    if (i >= n) continue;
    if (p[u] < 0 || p[u] >= n) {
      bad = true;
      continue;
    }
    if (col_ok) out[p[u] * row_words + v] = x[u];
  }
  if (bad && v == 0 && oob_flag) *oob_flag = 1;
}

// scalar rows (row = one 4- or 8-byte word): one thread per row
template <typename WORD>
__global__ void scatter_words_kernel(const WORD* __restrict__ rows, int64_t n, const int64_t* __restrict__ perm,
                                     WORD* __restrict__ scratch, int32_t* __restrict__ oob_flag) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t p = perm[i];
  if (p < 0 || p >= n) {
    if (oob_flag) *oob_flag = 1;
    return;
  }
  scratch[p] = rows[i];
}

// ---- randperm ------------------------------------------------------------------------------
// out[i] = P(i) for a keyed bijection P of [0, n): an alternating (unbalanced) Feistel network
// on the k = bits(n - 1) bits of i, walked along its cycle until the value falls below n (fewer
// than two steps on average, since 2^k < 2n).  Each of the kPermRounds rounds replaces
// (L, R) by (R, L xor F(R + key_r)) with F a 32-bit integer hash, so every round -- and the
// whole map -- is invertible whatever F is.  No sort, no workspace, 8 bytes written per entry.
constexpr int kPermRounds = 8;
struct PermKeys {
  uint32_t k[kPermRounds];
};

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

__global__ void randperm_kernel(int64_t n, int wl, int wr, PermKeys keys, int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t ml = wl >= 32 ? 0xffffffffu : ((1u << wl) - 1u);
  const uint32_t mr = wr >= 32 ? 0xffffffffu : ((1u << wr) - 1u);
  uint64_t x = (uint64_t)i;
  do {
    uint32_t l = (uint32_t)(x >> wr) & ml, r = (uint32_t)x & mr;
    // the halves change places every round and the widths with them; kPermRounds is even,
    // so the layout at the end is the one at the start
#pragma unroll
    for (int t = 0; t < kPermRounds; t += 2) {
      const uint32_t a = l ^ (mix32(r + keys.k[t]) & ml);      // (l, r) -> (r, a): widths (wr, wl)
      const uint32_t b = r ^ (mix32(a + keys.k[t + 1]) & mr);  // (r, a) -> (a, b): widths (wl, wr)
      l = a;
      r = b;
    }
    x = ((uint64_t)l << wr) | r;
  } while (x >= (uint64_t)n);
  out[i] = (int64_t)x;
}

uint64_t host_splitmix64(uint64_t x) {
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}

struct SubBucketArgs {
  const int64_t* lhs_in; const int64_t* rhs_in; const int64_t* rel_in;
  const int64_t* const* lhs_perms; const int64_t* const* rhs_perms;
  const int64_t* lhs_sizes; const int64_t* rhs_sizes;
  int64_t n; int num_relations; int parts_l; int parts_r; int dynamic;
};

__device__ __forceinline__ bool sub_bucket_locate(const SubBucketArgs& a, int64_t e, int64_t* lo, int64_t* ro,
                                                  int64_t* lsize, int64_t* rsize) {
  const int64_t r = a.dynamic ? 0 : a.rel_in[e];
  if (r < 0 || r >= a.num_relations) return false;
  *lo = a.lhs_perms[r][a.lhs_in[e]];
  *ro = a.rhs_perms[r][a.rhs_in[e]];
  *lsize = a.lhs_sizes[r];
  *rsize = a.rhs_sizes[r];
  return true;
}

__global__ void sub_bucket_keys_kernel(SubBucketArgs a, uint64_t* __restrict__ keys, uint32_t* __restrict__ vals,
                                       int32_t* __restrict__ error_flag) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= a.n) return;
  int64_t lo, ro, ls, rs;
  uint64_t key = 0;
  if (sub_bucket_locate(a, e, &lo, &ro, &ls, &rs)) {
    const int64_t lp = lo / ls, rp = ro / rs;
    if (lp < 0 || lp >= a.parts_l || rp < 0 || rp >= a.parts_r) {
      if (error_flag) *error_flag = 2;
    } else {
      key = (uint64_t)(lp * a.parts_r + rp);
    }
  } else if (error_flag) {
    *error_flag = 1;  // "rel > numRelations" (util.cpp:343-345)
  }
  keys[e] = key;
  vals[e] = (uint32_t)e;
}

__global__ void sub_bucket_emit_kernel(SubBucketArgs a, const uint64_t* __restrict__ keys,
                                       const uint32_t* __restrict__ vals, int64_t* __restrict__ lhs_out,
                                       int64_t* __restrict__ rhs_out, int64_t* __restrict__ rel_out,
                                       int64_t* __restrict__ offsets) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= a.n) return;
  const int64_t e = vals[p];
  int64_t lo = 0, ro = 0, ls = 1, rs = 1;
  sub_bucket_locate(a, e, &lo, &ro, &ls, &rs);
  lhs_out[p] = lo % ls;
  rhs_out[p] = ro % rs;
  rel_out[p] = a.rel_in[e];
  // offsets[b] = first sorted position whose sub-bucket id is >= b
  const int64_t nb = (int64_t)a.parts_l * a.parts_r;
  const int64_t key = (int64_t)keys[p];
  const int64_t prev = (p == 0) ? -1 : (int64_t)keys[p - 1];
  for (int64_t b = prev + 1; b <= key; ++b) offsets[b] = p;
  if (p == a.n - 1) {
    for (int64_t b = key + 1; b <= nb; ++b) offsets[b] = a.n;
  }
}

// ---- sub_bucket with at most kSbMaxBins sub-buckets: one histogram, one stable scatter -----------
// locate   per edge: the two permutation look-ups (the only random accesses of the whole call), the
//          sub-bucket number and the two output ids, kept in input order; per tile of kSbTile edges
//          the number of edges of every sub-bucket, laid out [sub-bucket][tile];
// scan     exclusive prefix sums over that array as it lies: the first output position of every
//          (sub-bucket, tile) pair, and with them the offsets of the sub-buckets;
// scatter  per tile: every edge's rank among the tile's earlier edges of its sub-bucket (a wave owns
//          consecutive edges, so (wave, round, lane) is the input order and the partition is stable),
//          then the three ids go to first position + rank -- read in order, written in runs.
constexpr int kSbMaxBins = 512;
constexpr int kSbThreads = 1024;
constexpr int kSbKpt = 4;
constexpr int kSbTile = kSbThreads * kSbKpt;
constexpr int kScanChunk = 4096;  // cells per block of the scan kernels (1024 threads x 4)

__global__ __launch_bounds__(kSbThreads) void sub_bucket_locate_kernel(SubBucketArgs a, int nb, int64_t tiles,
                                                                       uint16_t* __restrict__ bins,
                                                                       int64_t* __restrict__ lo_mod,
                                                                       int64_t* __restrict__ ro_mod,
                                                                       uint32_t* __restrict__ counts,
                                                                       int32_t* __restrict__ error_flag) {
  __shared__ uint32_t hist[kSbMaxBins];
  const int t = threadIdx.x;
  for (int d = t; d < nb; d += kSbThreads) hist[d] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSbTile;
  int64_t lo[kSbKpt], ro[kSbKpt], ls[kSbKpt], rs[kSbKpt];
  bool ok[kSbKpt];
#pragma unroll
  for (int q = 0; q < kSbKpt; ++q) {  // all look-ups of the thread are issued before the first is used
    const int64_t e = base + q * kSbThreads + t;
    lo[q] = ro[q] = 0;
    ls[q] = rs[q] = 1;
    ok[q] = e < a.n ? sub_bucket_locate(a, e, &lo[q], &ro[q], &ls[q], &rs[q]) : true;
  }
#pragma unroll
  for (int q = 0; q < kSbKpt; ++q) {
    const int64_t e = base + q * kSbThreads + t;
    if (e >= a.n) continue;
    uint32_t bin = 0;
    if (!ok[q]) {
      if (error_flag) *error_flag = 1;  // "rel > numRelations" (util.cpp:343-345)
    } else {
      const int64_t lp = lo[q] / ls[q], rp = ro[q] / rs[q];
      if (lp < 0 || lp >= a.parts_l || rp < 0 || rp >= a.parts_r) {
        if (error_flag) *error_flag = 2;
      } else {
        bin = (uint32_t)(lp * a.parts_r + rp);
      }
    }
    bins[e] = (uint16_t)bin;
    lo_mod[e] = lo[q] % ls[q];
    ro_mod[e] = ro[q] % rs[q];
    atomicAdd(&hist[bin], 1u);
  }
  __syncthreads();
  for (int d = t; d < nb; d += kSbThreads) counts[(int64_t)d * tiles + blockIdx.x] = hist[d];
}

// sums[b] = sum of cells [b * kScanChunk, (b + 1) * kScanChunk)
__global__ __launch_bounds__(1024) void scan_chunk_sums_kernel(const uint32_t* __restrict__ cells, int64_t count,
                                                               uint32_t* __restrict__ sums) {
  __shared__ uint32_t wave_total[16];
  const int t = threadIdx.x;
  const int64_t first = (int64_t)blockIdx.x * kScanChunk + (int64_t)t * 4;
  uint32_t v = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) v += first + q < count ? cells[first + q] : 0u;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  if ((t & 63) == 0) wave_total[t >> 6] = v;
  __syncthreads();
  if (t == 0) {
    uint32_t all = 0;
    for (int w = 0; w < 16; ++w) all += wave_total[w];
    sums[blockIdx.x] = all;
  }
}

// exclusive scan of sums[0, chunks) in place, by one block (any number of chunks)
__global__ __launch_bounds__(1024) void scan_sums_kernel(uint32_t* __restrict__ sums, int64_t chunks) {
  __shared__ uint32_t wave_total[16];
  __shared__ uint32_t carry_s;
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  if (t == 0) carry_s = 0;
  __syncthreads();
  for (int64_t base = 0; base < chunks; base += 1024) {
    const int64_t i = base + t;
    const uint32_t v = i < chunks ? sums[i] : 0u;
    uint32_t incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    uint32_t ahead = carry_s;
    for (int w = 0; w < wave; ++w) ahead += wave_total[w];
    if (i < chunks) sums[i] = ahead + incl - v;
    __syncthreads();
    if (t == 1023) carry_s = ahead + incl;
    __syncthreads();
  }
}

// cells -> their exclusive prefix sums (in place); a cell that starts a sub-bucket's row of tiles also
// gives that sub-bucket's offset
__global__ __launch_bounds__(1024) void scan_cells_kernel(uint32_t* __restrict__ cells, int64_t count,
                                                          const uint32_t* __restrict__ chunk_base, int64_t tiles,
                                                          int64_t* __restrict__ offsets) {
  __shared__ uint32_t wave_total[16];
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  const int64_t first = (int64_t)blockIdx.x * kScanChunk + (int64_t)t * 4;
  uint32_t c[4];
  uint32_t mine = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    c[q] = first + q < count ? cells[first + q] : 0u;
    mine += c[q];
  }
  uint32_t incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  uint32_t at = chunk_base[blockIdx.x] + incl - mine;
  for (int w = 0; w < wave; ++w) at += wave_total[w];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (first + q < count) {
      cells[first + q] = at;
      if ((first + q) % tiles == 0) offsets[(first + q) / tiles] = (int64_t)at;
    }
    at += c[q];
  }
}

__global__ __launch_bounds__(kSbThreads) void sub_bucket_scatter_kernel(
    const uint16_t* __restrict__ bins, const int64_t* __restrict__ lo_mod, const int64_t* __restrict__ ro_mod,
    const int64_t* __restrict__ rel_in, int64_t n, int nb, int bin_bits, int64_t tiles,
    const uint32_t* __restrict__ first_pos, int64_t* __restrict__ lhs_out, int64_t* __restrict__ rhs_out,
    int64_t* __restrict__ rel_out) {
  __shared__ uint16_t wave_count[kSbThreads / 64][kSbMaxBins];
  __shared__ uint32_t bin_first[kSbMaxBins];
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  for (int d = t; d < nb; d += kSbThreads) {
    bin_first[d] = first_pos[(int64_t)d * tiles + blockIdx.x];
    for (int w = 0; w < kSbThreads / 64; ++w) wave_count[w][d] = 0;
  }
  const int64_t base = (int64_t)blockIdx.x * kSbTile + (int64_t)wave * (64 * kSbKpt) + lane;
  uint32_t bin[kSbKpt];
  int64_t lo[kSbKpt], ro[kSbKpt], rel[kSbKpt];
#pragma unroll
  for (int q = 0; q < kSbKpt; ++q) {
    const int64_t e = base + q * 64;
    const bool in = e < n;
    bin[q] = in ? bins[e] : 0u;
    lo[q] = in ? lo_mod[e] : 0;
    ro[q] = in ? ro_mod[e] : 0;
    rel[q] = in ? rel_in[e] : 0;
  }
  __syncthreads();
  const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  uint32_t rank[kSbKpt];
#pragma unroll
  for (int q = 0; q < kSbKpt; ++q) {
    const bool valid = base + q * 64 < n;
    uint64_t peers = __ballot(valid);  // the lanes of this round with the same sub-bucket
    for (int b = 0; b < bin_bits; ++b) {
      const bool bit = (bin[q] >> b) & 1u;
      const uint64_t m = __ballot(valid && bit);
      peers &= bit ? m : ~m;
    }
    const int rank_in_round = __popcll(peers & below);
    const uint32_t prior = valid ? wave_count[wave][bin[q]] : 0u;  // this wave's earlier rounds (no other wave writes the row)
    rank[q] = prior + (uint32_t)rank_in_round;
    if (valid && rank_in_round == 0) wave_count[wave][bin[q]] = (uint16_t)(prior + __popcll(peers));
  }
  __syncthreads();
  for (int d = t; d < nb; d += kSbThreads) {  // the waves' counts become the waves' offsets inside the tile's run
    uint32_t at = 0;
    for (int w = 0; w < kSbThreads / 64; ++w) {
      const uint32_t cnt = wave_count[w][d];
      wave_count[w][d] = (uint16_t)at;
      at += cnt;
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < kSbKpt; ++q) {
    if (base + q * 64 >= n) continue;
    const int64_t pos = (int64_t)bin_first[bin[q]] + wave_count[wave][bin[q]] + rank[q];
    lhs_out[pos] = lo[q];
    rhs_out[pos] = ro[q];
    rel_out[pos] = rel[q];
  }
}

struct CountWs {
  uint16_t* bins; int64_t* lo_mod; int64_t* ro_mod; uint32_t* cells; uint32_t* sums;
  int64_t tiles, count, chunks;
  size_t total;
};
CountWs carve_count(void* base, int64_t n, int nb) {
  CountWs w;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return (char*)base + o; };
  const size_t nn = (size_t)(n > 0 ? n : 1);
  w.tiles = ceil_div((int64_t)nn, kSbTile);
  w.count = w.tiles * nb;
  w.chunks = ceil_div(w.count, kScanChunk);
  w.lo_mod = (int64_t*)take(nn * 8);
  w.ro_mod = (int64_t*)take(nn * 8);
  w.bins = (uint16_t*)take(nn * 2);
  w.cells = (uint32_t*)take((size_t)w.count * 4);
  w.sums = (uint32_t*)take((size_t)w.chunks * 4);
  w.total = off;
  return w;
}

__global__ void fill_i64_kernel(int64_t* out, int64_t count, int64_t value) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) out[i] = value;
}

struct PairWs {
  uint64_t* keys_a; uint64_t* keys_b; uint32_t* vals_a; uint32_t* vals_b; void* temp;
  size_t total;
};
PairWs carve_pairs(void* base, int64_t n) {
  PairWs w;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return (char*)base + o; };
  const size_t nn = (size_t)(n > 0 ? n : 1);
  w.keys_a = (uint64_t*)take(nn * 8);
  w.keys_b = (uint64_t*)take(nn * 8);
  w.vals_a = (uint32_t*)take(nn * 4);
  w.vals_b = (uint32_t*)take(nn * 4);
  w.temp = take(sort_temp_bytes(n));
  w.total = off;
  return w;
}

}  // namespace
}  // namespace pbg

using namespace pbg;

extern "C" int pbg_reverse_permutation(const int64_t* perm, int64_t n, int64_t* out, pbg_stream_t stream) {
  if (n < 0) return fail(PBG_ERR_INVALID, "pbg_reverse_permutation: negative size");
  if (n == 0) return PBG_OK;
  if (!perm || !out) return fail(PBG_ERR_INVALID, "pbg_reverse_permutation: null pointer");
  hipLaunchKernelGGL(reverse_permutation_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream,
                     perm, n, out);
  return check_launch("pbg_reverse_permutation");
}

namespace {
// dst[perm[i]] = src[i] for rows of row_bytes bytes (a multiple of 4); src and dst do not overlap
int scatter_rows(const void* rows, int64_t n, int64_t row_bytes, const int64_t* perm, void* out, int32_t* oob_flag,
                 hipStream_t s) {
  const bool a16 = row_bytes % 16 == 0 && (uintptr_t)rows % 16 == 0 && (uintptr_t)out % 16 == 0;
  const bool a8 = row_bytes % 8 == 0 && (uintptr_t)rows % 8 == 0 && (uintptr_t)out % 8 == 0;
  if (row_bytes == 4) {
    hipLaunchKernelGGL(scatter_words_kernel<uint32_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                       (const uint32_t*)rows, n, perm, (uint32_t*)out, oob_flag);
  } else if (row_bytes == 8 && a8) {
    hipLaunchKernelGGL(scatter_words_kernel<uint64_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                       (const uint64_t*)rows, n, perm, (uint64_t*)out, oob_flag);
  } else if (a16 && row_bytes <= 1024) {
    constexpr int kU = 8;
    const int words = (int)(row_bytes / 16);
    const uint4* src = (const uint4*)rows;
    uint4* dst = (uint4*)out;
    if (words <= 8) {
      hipLaunchKernelGGL((scatter_rows_multi_kernel<8, kU>), dim3((unsigned)ceil_div(n, 4 * 8 * kU)), dim3(256), 0, s, src,
                         n, words, perm, dst, oob_flag);
    } else if (words <= 16) {
      hipLaunchKernelGGL((scatter_rows_multi_kernel<16, kU>), dim3((unsigned)ceil_div(n, 4 * 4 * kU)), dim3(256), 0, s,
                         src, n, words, perm, dst, oob_flag);
    } else if (words <= 32) {
      hipLaunchKernelGGL((scatter_rows_multi_kernel<32, kU>), dim3((unsigned)ceil_div(n, 4 * 2 * kU)), dim3(256), 0, s,
                         src, n, words, perm, dst, oob_flag);
    } else {
      hipLaunchKernelGGL((scatter_rows_multi_kernel<64, kU>), dim3((unsigned)ceil_div(n, 4 * kU)), dim3(256), 0, s, src, n,
                         words, perm, dst, oob_flag);
    }
  } else if (a16) {
    hipLaunchKernelGGL(scatter_rows_kernel<uint4>, dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, s, (const uint4*)rows,
                       n, row_bytes / 16, perm, (uint4*)out, oob_flag);
  } else {
    hipLaunchKernelGGL(scatter_rows_kernel<uint32_t>, dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, s,
                       (const uint32_t*)rows, n, row_bytes / 4, perm, (uint32_t*)out, oob_flag);
  }
  return check_launch("pbg_shuffle_rows");
}
}  // namespace

extern "C" int pbg_shuffle_rows(void* rows, int64_t n, int64_t row_bytes, const int64_t* perm, void* scratch,
                                int32_t* oob_flag, pbg_stream_t stream) {
  if (n < 0 || row_bytes < 0) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows: negative size");
  if (n == 0 || row_bytes == 0) return PBG_OK;  // util.cpp:146-152
  if (!rows || !perm || !scratch) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows: null pointer");
  if (row_bytes % 4 != 0) return fail(PBG_ERR_UNSUPPORTED, "pbg_shuffle_rows: row_bytes must be a multiple of 4");
  hipStream_t s = (hipStream_t)stream;
  // A valid permutation writes every scratch row; with an invalid one the flag
  // is raised and the contents of `rows` are unspecified (the reference throws
  // mid-way, util.cpp:200-202, leaving a partly shuffled tensor too).
  const int rc = scatter_rows(rows, n, row_bytes, perm, scratch, oob_flag, s);
  if (rc != PBG_OK) return rc;
  const hipError_t err = hipMemcpyAsync(rows, scratch, (size_t)n * row_bytes, hipMemcpyDeviceToDevice, s);
  if (err != hipSuccess) return fail(PBG_ERR_LAUNCH, "pbg_shuffle_rows: %s", hipGetErrorString(err));
  return check_launch("pbg_shuffle_rows");
}

extern "C" int pbg_shuffle_rows_out(const void* rows, int64_t n, int64_t row_bytes, const int64_t* perm, void* out,
                                    int32_t* oob_flag, pbg_stream_t stream) {
  if (n < 0 || row_bytes < 0) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows_out: negative size");
  if (n == 0 || row_bytes == 0) return PBG_OK;
  if (!rows || !perm || !out) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows_out: null pointer");
  if (row_bytes % 4 != 0) return fail(PBG_ERR_UNSUPPORTED, "pbg_shuffle_rows_out: row_bytes must be a multiple of 4");
  const char* lo = (const char*)rows;
  const char* ol = (const char*)out;
  const size_t bytes = (size_t)n * (size_t)row_bytes;
  if (lo < ol + bytes && ol < lo + bytes) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows_out: rows and out overlap");
  return scatter_rows(rows, n, row_bytes, perm, out, oob_flag, (hipStream_t)stream);
}

extern "C" size_t pbg_randperm_workspace_bytes(int64_t) { return 0; }

extern "C" int pbg_randperm(int64_t n, uint64_t seed, int64_t* out, void*, size_t, pbg_stream_t stream) {
  if (n < 0) return fail(PBG_ERR_INVALID, "pbg_randperm: negative size");
  if (n == 0) return PBG_OK;
  if (!out) return fail(PBG_ERR_INVALID, "pbg_randperm: null pointer");
  int bits = bits_for((uint64_t)(n - 1));
  if (bits < 2) bits = 2;
  const int wl = bits / 2, wr = bits - wl;  // both at most 32: n is below 2^63
  PermKeys keys;
  for (int r = 0; r < kPermRounds; ++r)
    keys.k[r] = (uint32_t)(host_splitmix64(seed + 0x632be59bd9b4e019ull * (uint64_t)(r + 1)) >> 32);
  hipLaunchKernelGGL(randperm_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, n, wl, wr,
                     keys, out);
  return check_launch("pbg_randperm");
}

extern "C" size_t pbg_sub_bucket_workspace_bytes(int64_t n) {
  const size_t sorted = carve_pairs(nullptr, n).total, counted = carve_count(nullptr, n, kSbMaxBins).total;
  return sorted > counted ? sorted : counted;
}

extern "C" int pbg_sub_bucket(const int64_t* lhs_in, const int64_t* rhs_in, const int64_t* rel_in, int64_t n,
                              int32_t num_relations, const int64_t* const* lhs_perm_ptrs,
                              const int64_t* const* rhs_perm_ptrs, const int64_t* lhs_part_sizes,
                              const int64_t* rhs_part_sizes, int32_t num_lhs_parts, int32_t num_rhs_parts,
                              int32_t dynamic_relations, int64_t* lhs_out, int64_t* rhs_out, int64_t* rel_out,
                              int64_t* offsets_out, int32_t* error_flag, void* workspace, size_t workspace_bytes,
                              pbg_stream_t stream) {
  if (n < 0 || num_relations <= 0) return fail(PBG_ERR_INVALID, "pbg_sub_bucket: bad sizes");
  if (num_lhs_parts <= 0 || num_rhs_parts <= 0 || num_lhs_parts > 127 || num_rhs_parts > 127)
    return fail(PBG_ERR_INVALID, "pbg_sub_bucket: sub-part counts must be in [1, 127]");  // int8 in util.cpp:272-273
  if (!offsets_out) return fail(PBG_ERR_INVALID, "pbg_sub_bucket: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const int64_t nb = (int64_t)num_lhs_parts * num_rhs_parts;
  if (n == 0) {
    hipLaunchKernelGGL(fill_i64_kernel, dim3((unsigned)ceil_div(nb + 1, 256)), dim3(256), 0, s, offsets_out, nb + 1,
                       (int64_t)0);
    return check_launch("pbg_sub_bucket");
  }
  if (n >= (int64_t)1 << 32) return fail(PBG_ERR_UNSUPPORTED, "pbg_sub_bucket: n must be below 2^32");
  if (!lhs_in || !rhs_in || !rel_in || !lhs_perm_ptrs || !rhs_perm_ptrs || !lhs_part_sizes || !rhs_part_sizes ||
      !lhs_out || !rhs_out || !rel_out)
    return fail(PBG_ERR_INVALID, "pbg_sub_bucket: null pointer");
  if (!workspace || workspace_bytes < pbg_sub_bucket_workspace_bytes(n))
    return fail(PBG_ERR_WORKSPACE, "pbg_sub_bucket: workspace needs %zu bytes", pbg_sub_bucket_workspace_bytes(n));
  SubBucketArgs a{lhs_in, rhs_in, rel_in, lhs_perm_ptrs, rhs_perm_ptrs, lhs_part_sizes, rhs_part_sizes,
                  n, num_relations, num_lhs_parts, num_rhs_parts, dynamic_relations};
  if (nb <= kSbMaxBins) {  // a histogram and one stable scatter; every edge's ids are looked up once
    CountWs cw = carve_count(workspace, n, (int)nb);
    const int inb = (int)nb;
    hipLaunchKernelGGL(sub_bucket_locate_kernel, dim3((unsigned)cw.tiles), dim3(kSbThreads), 0, s, a, inb, cw.tiles,
                       cw.bins, cw.lo_mod, cw.ro_mod, cw.cells, error_flag);
    hipLaunchKernelGGL(scan_chunk_sums_kernel, dim3((unsigned)cw.chunks), dim3(1024), 0, s, cw.cells, cw.count, cw.sums);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(1024), 0, s, cw.sums, cw.chunks);
    hipLaunchKernelGGL(scan_cells_kernel, dim3((unsigned)cw.chunks), dim3(1024), 0, s, cw.cells, cw.count, cw.sums,
                       cw.tiles, offsets_out);
    hipLaunchKernelGGL(fill_i64_kernel, dim3(1), dim3(64), 0, s, offsets_out + nb, (int64_t)1, n);
    hipLaunchKernelGGL(sub_bucket_scatter_kernel, dim3((unsigned)cw.tiles), dim3(kSbThreads), 0, s, cw.bins, cw.lo_mod,
                       cw.ro_mod, rel_in, n, inb, bits_for((uint64_t)(nb - 1)), cw.tiles, cw.cells, lhs_out, rhs_out,
                       rel_out);
    return check_launch("pbg_sub_bucket");
  }
  PairWs ws = carve_pairs(workspace, n);
  const dim3 grid((unsigned)ceil_div(n, 256)), block(256);
  hipLaunchKernelGGL(sub_bucket_keys_kernel, grid, block, 0, s, a, ws.keys_a, ws.vals_a, error_flag);
  uint64_t* skeys;
  uint32_t* svals;
  int rc = sort_pairs(ws.keys_a, ws.vals_a, ws.keys_b, ws.vals_b, n, 0, bits_for((uint64_t)(nb - 1)), ws.temp, s,
                      &skeys, &svals);
  if (rc != PBG_OK) return rc;
  hipLaunchKernelGGL(sub_bucket_emit_kernel, grid, block, 0, s, a, skeys, svals, lhs_out, rhs_out, rel_out,
                     offsets_out);
  return check_launch("pbg_sub_bucket");
}
