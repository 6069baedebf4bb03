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

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}

constexpr int kRandKeyBits = 40;

__global__ void random_keys_kernel(int64_t n, uint64_t seed, uint64_t* __restrict__ keys, uint32_t* __restrict__ vals) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  keys[i] = splitmix64(splitmix64(seed) ^ (uint64_t)i) >> (64 - kRandKeyBits);
  vals[i] = (uint32_t)i;
}

__global__ void widen_kernel(const uint32_t* __restrict__ vals, int64_t n, int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (int64_t)vals[i];
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

extern "C" int pbg_shuffle_rows(void* rows, int64_t n, int64_t row_bytes, const int64_t* perm, void* scratch,
                                int32_t* oob_flag, pbg_stream_t stream) {
  if (n < 0 || row_bytes < 0) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows: negative size");
  if (n == 0 || row_bytes == 0) return PBG_OK;  // util.cpp:146-152
  if (!rows || !perm || !scratch) return fail(PBG_ERR_INVALID, "pbg_shuffle_rows: null pointer");
  if (row_bytes % 4 != 0) return fail(PBG_ERR_UNSUPPORTED, "pbg_shuffle_rows: row_bytes must be a multiple of 4");
  hipStream_t s = (hipStream_t)stream;
  const bool a16 = row_bytes % 16 == 0 && (uintptr_t)rows % 16 == 0 && (uintptr_t)scratch % 16 == 0;
  const bool a8 = row_bytes % 8 == 0 && (uintptr_t)rows % 8 == 0 && (uintptr_t)scratch % 8 == 0;
  // A valid permutation writes every scratch row; with an invalid one the flag
  // is raised and the contents of `rows` are unspecified (the reference throws
  // mid-way, util.cpp:200-202, leaving a partly shuffled tensor too).
  hipError_t err;
  if (row_bytes == 4) {
    hipLaunchKernelGGL(scatter_words_kernel<uint32_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                       (const uint32_t*)rows, n, perm, (uint32_t*)scratch, oob_flag);
  } else if (row_bytes == 8 && a8) {
    hipLaunchKernelGGL(scatter_words_kernel<uint64_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                       (const uint64_t*)rows, n, perm, (uint64_t*)scratch, oob_flag);
  } else if (a16) {
    hipLaunchKernelGGL(scatter_rows_kernel<uint4>, dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, s, (const uint4*)rows,
                       n, row_bytes / 16, perm, (uint4*)scratch, oob_flag);
  } else {
    hipLaunchKernelGGL(scatter_rows_kernel<uint32_t>, dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, s,
                       (const uint32_t*)rows, n, row_bytes / 4, perm, (uint32_t*)scratch, oob_flag);
  }
  err = hipMemcpyAsync(rows, scratch, (size_t)n * row_bytes, hipMemcpyDeviceToDevice, s);
  if (err != hipSuccess) return fail(PBG_ERR_LAUNCH, "pbg_shuffle_rows: %s", hipGetErrorString(err));
  return check_launch("pbg_shuffle_rows");
}

extern "C" size_t pbg_randperm_workspace_bytes(int64_t n) { return carve_pairs(nullptr, n).total; }

extern "C" int pbg_randperm(int64_t n, uint64_t seed, int64_t* out, void* workspace, size_t workspace_bytes,
                            pbg_stream_t stream) {
  if (n < 0) return fail(PBG_ERR_INVALID, "pbg_randperm: negative size");
  if (n == 0) return PBG_OK;
  if (n >= (int64_t)1 << 32) return fail(PBG_ERR_UNSUPPORTED, "pbg_randperm: n must be below 2^32");
  if (!out) return fail(PBG_ERR_INVALID, "pbg_randperm: null pointer");
  PairWs ws = carve_pairs(workspace, n);
  if (!workspace || workspace_bytes < ws.total)
    return fail(PBG_ERR_WORKSPACE, "pbg_randperm: workspace needs %zu bytes", ws.total);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(random_keys_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s, n, seed, ws.keys_a,
                     ws.vals_a);
  uint64_t* skeys;
  uint32_t* svals;
  int rc = sort_pairs(ws.keys_a, ws.vals_a, ws.keys_b, ws.vals_b, n, 0, kRandKeyBits, ws.temp, s, &skeys, &svals);
  if (rc != PBG_OK) return rc;
  hipLaunchKernelGGL(widen_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s, svals, n, out);
  return check_launch("pbg_randperm");
}

extern "C" size_t pbg_sub_bucket_workspace_bytes(int64_t n) { return carve_pairs(nullptr, n).total; }

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
  PairWs ws = carve_pairs(workspace, n);
  if (!workspace || workspace_bytes < ws.total)
    return fail(PBG_ERR_WORKSPACE, "pbg_sub_bucket: workspace needs %zu bytes", ws.total);
  SubBucketArgs a{lhs_in, rhs_in, rel_in, lhs_perm_ptrs, rhs_perm_ptrs, lhs_part_sizes, rhs_part_sizes,
                  n, num_relations, num_lhs_parts, num_rhs_parts, dynamic_relations};
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
