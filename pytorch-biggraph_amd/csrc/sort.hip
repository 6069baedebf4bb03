// Stable LSD radix sort of (uint64 key, uint32 value) pairs, 8 bits per pass.
//
// Every block owns a contiguous power-of-two tile of positions.  One histogram
// kernel counts the first digit per tile; after that each pass is ONE kernel:
// a block derives its digit offsets from the per-tile counts of all tiles (at
// most 256 of them), ranks its keys slice by slice (ballot matching inside a
// wave, LDS counts across the 4 waves, a running per-digit cursor across
// slices), scatters them, and counts the next pass's digit of every key into the
// tile the key lands in, so the next pass needs no histogram kernel of its own.
// Stability makes the order of equal keys the order of the input, which keeps
// segmented gradient sums deterministic.
#include "pbg_internal.h"

namespace pbg {
namespace {

constexpr int kSortThreads = 256;
constexpr int kRadix = 256;
constexpr int kMaxSortBlocks = 256;
constexpr int kMaxPasses = 9;

struct SortPlan {
  int tile_shift;  // keys per block = 1 << tile_shift
  int blocks;
};

SortPlan plan_sort(int64_t n) {
  SortPlan p;
  p.tile_shift = 9;
  while (ceil_div(n, (int64_t)1 << p.tile_shift) > kMaxSortBlocks) ++p.tile_shift;
  p.blocks = (int)ceil_div(n > 0 ? n : 1, (int64_t)1 << p.tile_shift);
  return p;
}

// counts[pass][block][digit]; this kernel fills pass 0 and clears the others
__global__ __launch_bounds__(kSortThreads) void sort_hist_kernel(const uint64_t* __restrict__ keys, int64_t n,
                                                                 int tile_shift, int passes,
                                                                 uint32_t* __restrict__ counts) {
  __shared__ uint32_t hist[kRadix];
  const int nblocks = gridDim.x;
  hist[threadIdx.x] = 0;
  for (int p = 1; p < passes; ++p) counts[((int64_t)p * nblocks + blockIdx.x) * kRadix + threadIdx.x] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x << tile_shift;
  int64_t end = begin + ((int64_t)1 << tile_shift);
  if (end > n) end = n;
  for (int64_t i = begin + threadIdx.x; i < end; i += kSortThreads) atomicAdd(&hist[keys[i] & 0xff], 1u);
  __syncthreads();
  counts[(int64_t)blockIdx.x * kRadix + threadIdx.x] = hist[threadIdx.x];
}

__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int64_t n, int tile_shift, int shift, const uint32_t* __restrict__ counts,
    uint32_t* __restrict__ next_counts) {
  __shared__ uint32_t cursor[kRadix];         // next output slot of each digit for this block
  __shared__ uint32_t wave_count[4][kRadix];  // per-wave digit counts of the current slice
  __shared__ uint32_t scan[kRadix];
  const int t = threadIdx.x;
  const int wave = t >> 6;
  const int lane = t & 63;
  const int nblocks = gridDim.x;
  // offset of digit t for this block = keys with a smaller digit anywhere
  //                                  + keys with digit t in earlier blocks
  uint32_t total = 0, before = 0;
  for (int b0 = 0; b0 < nblocks; b0 += 8) {  // eight independent loads in flight
    uint32_t cnt[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) cnt[u] = (b0 + u < nblocks) ? counts[(int64_t)(b0 + u) * kRadix + t] : 0u;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      total += cnt[u];
      if (b0 + u < (int)blockIdx.x) before += cnt[u];
    }
  }
  scan[t] = total;
  __syncthreads();
  for (int off = 1; off < kRadix; off <<= 1) {  // inclusive scan over the 256 digit totals
    const uint32_t v = (t >= off) ? scan[t - off] : 0;
    __syncthreads();
    scan[t] += v;
    __syncthreads();
  }
  cursor[t] = scan[t] - total + before;
  for (int w = 0; w < 4; ++w) wave_count[w][t] = 0;
  __syncthreads();

  const int64_t begin = (int64_t)blockIdx.x << tile_shift;
  int64_t end = begin + ((int64_t)1 << tile_shift);
  if (end > n) end = n;
  // the next slice's loads are issued before the current slice is ranked
  uint64_t key_next = 0;
  uint32_t val_next = 0;
  if (begin + t < end) {
    key_next = keys_in[begin + t];
    val_next = vals_in[begin + t];
  }
  for (int64_t base = begin; base < end; base += kSortThreads) {
    const int64_t i = base + t;
    const bool valid = i < end;
    const uint64_t key = key_next;
    const uint32_t val = val_next;
    if (i + kSortThreads < end) {
      key_next = keys_in[i + kSortThreads];
      val_next = vals_in[i + kSortThreads];
    }
    const uint32_t digit = shift < 64 ? (uint32_t)((key >> shift) & 0xff) : 0u;
    // lanes of this wave holding the same digit
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const bool bit = (digit >> b) & 1u;
      const uint64_t m = __ballot(valid && bit);
      peers &= bit ? m : ~m;
    }
    const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const int rank_in_wave = __popcll(peers & below);
    if (valid && rank_in_wave == 0) wave_count[wave][digit] = (uint32_t)__popcll(peers);
    __syncthreads();
    if (valid) {
      uint32_t ahead = 0;
      for (int w = 0; w < wave; ++w) ahead += wave_count[w][digit];
      const uint32_t pos = cursor[digit] + ahead + (uint32_t)rank_in_wave;
      keys_out[pos] = key;
      vals_out[pos] = val;
      if (next_counts) {
        const uint32_t next_digit = shift + 8 < 64 ? (uint32_t)((key >> (shift + 8)) & 0xff) : 0u;
        atomicAdd(&next_counts[(int64_t)(pos >> tile_shift) * kRadix + next_digit], 1u);
      }
    }
    __syncthreads();
    uint32_t slice_total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      slice_total += wave_count[w][t];
      wave_count[w][t] = 0;
    }
    cursor[t] += slice_total;
    __syncthreads();
  }
}

}  // namespace

size_t sort_temp_bytes(int64_t n) {
  SortPlan p = plan_sort(n);
  return align_up((size_t)kMaxPasses * p.blocks * kRadix * sizeof(uint32_t), 256);
}

int sort_pairs(uint64_t* keys_in, uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out, int64_t n,
               int key_bits, void* temp, hipStream_t stream) {
  if (n <= 0) return PBG_OK;
  if (n >= (int64_t)1 << 32)
    return fail(PBG_ERR_UNSUPPORTED, "sort_pairs: n=%lld does not fit 32-bit offsets", (long long)n);
  SortPlan p = plan_sort(n);
  uint32_t* counts = (uint32_t*)temp;
  int passes = (key_bits + 7) / 8;
  if (passes < 1) passes = 1;
  // an odd number of ping-pong passes ends in the "out" buffers; pad an even
  // count with one more pass over a zero digit
  if (passes % 2 == 0) passes += 1;
  if (passes > kMaxPasses) return fail(PBG_ERR_INVALID, "sort_pairs: too many key bits");
  hipLaunchKernelGGL(sort_hist_kernel, dim3(p.blocks), dim3(kSortThreads), 0, stream, keys_in, n, p.tile_shift, passes,
                     counts);
  uint64_t* ksrc = keys_in;
  uint32_t* vsrc = vals_in;
  uint64_t* kdst = keys_out;
  uint32_t* vdst = vals_out;
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = pass * 8;
    uint32_t* cur = counts + (size_t)pass * p.blocks * kRadix;
    uint32_t* next = (pass + 1 < passes) ? counts + (size_t)(pass + 1) * p.blocks * kRadix : nullptr;
    hipLaunchKernelGGL(sort_scatter_kernel, dim3(p.blocks), dim3(kSortThreads), 0, stream, ksrc, vsrc, kdst, vdst, n,
                       p.tile_shift, shift, cur, next);
    uint64_t* tk = ksrc; ksrc = kdst; kdst = tk;
    uint32_t* tv = vsrc; vsrc = vdst; vdst = tv;
  }
  return check_launch("sort_pairs");
}

}  // namespace pbg
