// Stable LSD radix sort of (uint64 key, uint32 value) pairs, 8 bits per pass.
//
// Per pass: (1) every block histograms its contiguous tile of keys into
// counts[digit][block]; (2) one block turns the digit-major counts into
// exclusive offsets; (3) every block re-reads its tile in 256-key slices, ranks
// each key among the equal digits before it (ballot matching inside a wave,
// LDS counts across the 4 waves, a running per-digit cursor across slices) and
// scatters.  Stability makes the order of equal keys the order of the input,
// which is what keeps segmented gradient sums deterministic.
#include "pbg_internal.h"

namespace pbg {
namespace {

constexpr int kSortThreads = 256;
constexpr int kRadix = 256;
constexpr int kMaxSortBlocks = 1024;

struct SortPlan {
  int64_t tile;  // keys per block (multiple of 256)
  int blocks;
};

SortPlan plan_sort(int64_t n) {
  SortPlan p;
  int64_t tile = 2048;
  while (ceil_div(n, tile) > kMaxSortBlocks) tile *= 2;
  p.tile = tile;
  p.blocks = (int)ceil_div(n > 0 ? n : 1, tile);
  return p;
}

__global__ __launch_bounds__(kSortThreads) void sort_hist_kernel(const uint64_t* __restrict__ keys, int64_t n,
                                                                 int64_t tile, int shift, int nblocks,
                                                                 uint32_t* __restrict__ counts) {
  __shared__ uint32_t hist[kRadix];
  hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x * tile;
  int64_t end = begin + tile;
  if (end > n) end = n;
  for (int64_t i = begin + threadIdx.x; i < end; i += kSortThreads) {
    atomicAdd(&hist[(keys[i] >> shift) & 0xff], 1u);
  }
  __syncthreads();
  counts[(int64_t)threadIdx.x * nblocks + blockIdx.x] = hist[threadIdx.x];
}

// Exclusive scan of `total` counters (digit-major) by one block of 1024 threads.
__global__ __launch_bounds__(1024) void sort_scan_kernel(uint32_t* __restrict__ counts, int total) {
  __shared__ uint32_t partial[1024];
  const int t = threadIdx.x;
  const int per = (total + 1023) / 1024;
  const int begin = t * per;
  int end = begin + per;
  if (end > total) end = total;
  uint32_t sum = 0;
  for (int i = begin; i < end; ++i) sum += counts[i];
  partial[t] = sum;
  __syncthreads();
  // Hillis-Steele inclusive scan over the 1024 partial sums.
  for (int off = 1; off < 1024; off <<= 1) {
    uint32_t v = (t >= off) ? partial[t - off] : 0;
    __syncthreads();
    partial[t] += v;
    __syncthreads();
  }
  uint32_t run = partial[t] - sum;
  for (int i = begin; i < end; ++i) {
    uint32_t c = counts[i];
    counts[i] = run;
    run += c;
  }
}

__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int64_t n, int64_t tile, int shift, int nblocks,
    const uint32_t* __restrict__ offsets) {
  __shared__ uint32_t cursor[kRadix];         // next output slot of each digit for this block
  __shared__ uint32_t wave_count[4][kRadix];  // per-wave digit counts of the current slice
  const int t = threadIdx.x;
  const int wave = t >> 6;
  const int lane = t & 63;
  cursor[t] = offsets[(int64_t)t * nblocks + blockIdx.x];
  for (int w = 0; w < 4; ++w) wave_count[w][t] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x * tile;
  int64_t end = begin + tile;
  if (end > n) end = n;
  for (int64_t base = begin; base < end; base += kSortThreads) {
    const int64_t i = base + t;
    const bool valid = i < end;
    uint64_t key = 0;
    uint32_t val = 0;
    if (valid) {
      key = keys_in[i];
      val = vals_in[i];
    }
    const uint32_t digit = (uint32_t)((key >> shift) & 0xff);
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
      uint32_t before = 0;
      for (int w = 0; w < wave; ++w) before += wave_count[w][digit];
      const uint32_t pos = cursor[digit] + before + (uint32_t)rank_in_wave;
      keys_out[pos] = key;
      vals_out[pos] = val;
    }
    __syncthreads();
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      total += wave_count[w][t];
      wave_count[w][t] = 0;
    }
    cursor[t] += total;
    __syncthreads();
  }
}

}  // namespace

size_t sort_temp_bytes(int64_t n) {
  SortPlan p = plan_sort(n);
  return align_up((size_t)p.blocks * kRadix * sizeof(uint32_t), 256);
}

int sort_pairs(uint64_t* keys_in, uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out, int64_t n,
               int key_bits, void* temp, hipStream_t stream) {
  if (n <= 0) return PBG_OK;
  if (n >= (int64_t)1 << 32) return fail(PBG_ERR_UNSUPPORTED, "sort_pairs: n=%lld does not fit 32-bit offsets", (long long)n);
  SortPlan p = plan_sort(n);
  uint32_t* counts = (uint32_t*)temp;
  int passes = (key_bits + 7) / 8;
  if (passes < 1) passes = 1;
  if (passes % 2 == 1) {
    // an odd number of ping-pong passes ends in the "out" buffers; an even
    // number would end in "in", so pad even counts with one more (zero) digit
  } else {
    passes += 1;
  }
  uint64_t* ksrc = keys_in;
  uint32_t* vsrc = vals_in;
  uint64_t* kdst = keys_out;
  uint32_t* vdst = vals_out;
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = pass * 8;
    if (shift >= 64) return fail(PBG_ERR_INVALID, "sort_pairs: too many key bits");
    hipLaunchKernelGGL(sort_hist_kernel, dim3(p.blocks), dim3(kSortThreads), 0, stream, ksrc, n, p.tile, shift,
                       p.blocks, counts);
    hipLaunchKernelGGL(sort_scan_kernel, dim3(1), dim3(1024), 0, stream, counts, p.blocks * kRadix);
    hipLaunchKernelGGL(sort_scatter_kernel, dim3(p.blocks), dim3(kSortThreads), 0, stream, ksrc, vsrc, kdst, vdst,
                       n, p.tile, shift, p.blocks, counts);
    uint64_t* tk = ksrc; ksrc = kdst; kdst = tk;
    uint32_t* tv = vsrc; vsrc = vdst; vdst = tv;
  }
  return check_launch("sort_pairs");
}

}  // namespace pbg
