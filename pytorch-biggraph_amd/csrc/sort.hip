// Stable radix sort of (uint64 key, uint32 value) pairs on a bit range of the key.
//
// The top (up to 9) bits of the range are sorted by ONE global pass: every block
// owns a contiguous power-of-two tile of positions, a histogram kernel counts the
// digit per tile, and the scatter kernel derives its digit offsets from the
// per-tile counts of all tiles (at most 256 of them, stored digit-major so that a
// thread reads its digit's counts with a few independent 128-bit loads), ranks
// its keys slice by slice (ballot matching inside a wave, LDS counts across the
// 4 waves, a running per-digit cursor across slices) and scatters them.  That
// leaves one bucket per digit value, contiguous in memory; the remaining low bits
// are sorted inside each bucket, one block per bucket, 8 bits per launch from the
// lowest up: no counts to exchange between blocks, no atomics on global memory.
// Every step is stable, so equal keys keep the order of the input, which keeps
// segmented gradient sums deterministic and lets a caller whose input is already
// ordered by the low bits leave those bits out.
#include "pbg_internal.h"

namespace pbg {
namespace {

constexpr int kSortThreads = 256;
constexpr int kMaxDigitBits = 9;
constexpr int kMaxSortBlocks = 256;

struct SortPlan {
  int tile_shift;  // keys per block = 1 << tile_shift
  int blocks;
  int stride;      // blocks rounded up to a multiple of 4: row length of the digit-major counts
};

SortPlan plan_sort(int64_t n) {
  SortPlan p;
  p.tile_shift = 9;
  while (ceil_div(n, (int64_t)1 << p.tile_shift) > kMaxSortBlocks) ++p.tile_shift;
  p.blocks = (int)ceil_div(n > 0 ? n : 1, (int64_t)1 << p.tile_shift);
  p.stride = (p.blocks + 3) / 4 * 4;
  return p;
}

// counts[digit][stride] of the global pass (padding columns cleared)
__global__ __launch_bounds__(kSortThreads) void sort_hist_kernel(const uint64_t* __restrict__ keys, int64_t n,
                                                                 int tile_shift, int shift, int digit_bits, int stride,
                                                                 uint32_t* __restrict__ counts) {
  __shared__ uint32_t hist[1 << kMaxDigitBits];
  const int digits = 1 << digit_bits;
  const uint32_t mask = (uint32_t)digits - 1u;
  for (int d = threadIdx.x; d < digits; d += kSortThreads) hist[d] = 0;
  if (blockIdx.x == 0)
    for (int d = threadIdx.x; d < digits; d += kSortThreads)
      for (int b = gridDim.x; b < stride; ++b) counts[(int64_t)d * stride + b] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x << tile_shift;
  int64_t end = begin + ((int64_t)1 << tile_shift);
  if (end > n) end = n;
  for (int64_t i = begin + threadIdx.x; i < end; i += kSortThreads)
    atomicAdd(&hist[(uint32_t)(keys[i] >> shift) & mask], 1u);
  __syncthreads();
  for (int d = threadIdx.x; d < digits; d += kSortThreads) counts[(int64_t)d * stride + blockIdx.x] = hist[d];
}

// One slice of up to 256 keys: rank every key among the keys of the slice with
// the same digit (earlier positions first), scatter it to cursor[digit] + rank,
// advance the cursors.  wave_count must be zero on entry and is zero on exit.
template <int DPT>
__device__ __forceinline__ void scatter_slice(bool valid, uint64_t key, uint32_t val, uint32_t digit,
                                              uint32_t* cursor, uint32_t (*wave_count)[DPT * kSortThreads],
                                              uint64_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out) {
  constexpr int kBits = DPT == 1 ? 8 : 9;
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  // lanes of this wave holding the same digit
  uint64_t peers = __ballot(valid);
#pragma unroll
  for (int b = 0; b < kBits; ++b) {
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
  }
  __syncthreads();
#pragma unroll
  for (int d = 0; d < DPT; ++d) {
    uint32_t slice_total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      slice_total += wave_count[w][t + d * kSortThreads];
      wave_count[w][t + d * kSortThreads] = 0;
    }
    cursor[t + d * kSortThreads] += slice_total;
  }
  __syncthreads();
}

// Exclusive scan over the 256 * DPT digit totals (digit = t + d * 256), in place.
template <int DPT>
__device__ __forceinline__ void scan_digits(uint32_t* total, uint32_t* wave_total, uint32_t* grand) {
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  uint32_t carry = 0;
#pragma unroll
  for (int d = 0; d < DPT; ++d) {
    uint32_t incl = total[d];
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    uint32_t ahead = carry;
    for (int w = 0; w < wave; ++w) ahead += wave_total[w];
    carry += wave_total[0] + wave_total[1] + wave_total[2] + wave_total[3];
    total[d] = ahead + incl - total[d];
    __syncthreads();
  }
  *grand = carry;
}

// The global pass.  DPT digits per thread: 1 (up to 8 digit bits) or 2 (9 digit
// bits); digit d belongs to thread d % 256.  Block 0 also writes the bucket
// offsets (digit d's keys end up in [bucket_off[d], bucket_off[d + 1])).
template <int DPT>
__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int64_t n, int tile_shift, int shift, int digit_bits, int stride,
    const uint32_t* __restrict__ counts, uint32_t* __restrict__ bucket_off) {
  constexpr int kDigits = DPT * kSortThreads;
  __shared__ uint32_t cursor[kDigits];         // next output slot of each digit for this block
  __shared__ uint32_t wave_count[4][kDigits];  // per-wave digit counts of the current slice
  __shared__ uint32_t wave_total[4];
  const int t = threadIdx.x;
  const int me = blockIdx.x;
  // offset of digit d for this block = keys with a smaller digit anywhere
  //                                  + keys with digit d in earlier blocks
  uint32_t total[DPT], before[DPT];
#pragma unroll
  for (int d = 0; d < DPT; ++d) total[d] = before[d] = 0;
  const int quads = stride >> 2;
  for (int q0 = 0; q0 < quads; q0 += 16) {  // 16 x DPT independent 128-bit loads in flight
    uint4 cnt[DPT][16];
#pragma unroll
    for (int d = 0; d < DPT; ++d) {
      const uint4* row = reinterpret_cast<const uint4*>(counts + (int64_t)(t + d * kSortThreads) * stride);
      const bool has = ((t + d * kSortThreads) >> digit_bits) == 0;  // digits past the pass's width hold no keys
#pragma unroll
      for (int u = 0; u < 16; ++u) cnt[d][u] = (has && q0 + u < quads) ? row[q0 + u] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int d = 0; d < DPT; ++d) {
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int b = (q0 + u) * 4;
        const uint4 c4 = cnt[d][u];
        total[d] += c4.x + c4.y + c4.z + c4.w;
        before[d] += (b < me ? c4.x : 0u) + (b + 1 < me ? c4.y : 0u) + (b + 2 < me ? c4.z : 0u) +
                     (b + 3 < me ? c4.w : 0u);
      }
    }
  }
  uint32_t grand;
  scan_digits<DPT>(total, wave_total, &grand);
#pragma unroll
  for (int d = 0; d < DPT; ++d) {
    const int digit = t + d * kSortThreads;
    cursor[digit] = total[d] + before[d];
    if (me == 0 && (digit >> digit_bits) == 0) bucket_off[digit] = total[d];
    for (int w = 0; w < 4; ++w) wave_count[w][digit] = 0;
  }
  if (me == 0 && t == 0) bucket_off[1 << digit_bits] = grand;
  __syncthreads();

  const uint32_t mask = (1u << digit_bits) - 1u;
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
    const uint64_t key = key_next;
    const uint32_t val = val_next;
    if (i + kSortThreads < end) {
      key_next = keys_in[i + kSortThreads];
      val_next = vals_in[i + kSortThreads];
    }
    scatter_slice<DPT>(i < end, key, val, (uint32_t)(key >> shift) & mask, cursor, wave_count, keys_out, vals_out);
  }
}

// A local pass: block b sorts bucket b (positions [bucket_off[b], bucket_off[b + 1]))
// by one digit of up to 8 bits, reading from the "in" pair and writing the same
// positions of the "out" pair.
__global__ __launch_bounds__(kSortThreads) void sort_bucket_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, const uint32_t* __restrict__ bucket_off, int shift, int digit_bits) {
  __shared__ uint32_t cursor[kSortThreads];
  __shared__ uint32_t wave_count[4][kSortThreads];
  __shared__ uint32_t wave_total[4];
  const int t = threadIdx.x;
  const int64_t begin = bucket_off[blockIdx.x], end = bucket_off[blockIdx.x + 1];
  if (begin >= end) return;
  const uint32_t mask = (1u << digit_bits) - 1u;
  uint64_t key_next = 0;
  uint32_t val_next = 0;
  if (begin + t < end) {
    key_next = keys_in[begin + t];
    val_next = vals_in[begin + t];
  }
  cursor[t] = 0;
  for (int w = 0; w < 4; ++w) wave_count[w][t] = 0;
  __syncthreads();
  if (begin + t < end) atomicAdd(&cursor[(uint32_t)(key_next >> shift) & mask], 1u);
  for (int64_t i = begin + kSortThreads + t; i < end; i += kSortThreads)
    atomicAdd(&cursor[(uint32_t)(keys_in[i] >> shift) & mask], 1u);
  __syncthreads();
  uint32_t total[1] = {cursor[t]};
  uint32_t grand;
  scan_digits<1>(total, wave_total, &grand);
  cursor[t] = (uint32_t)begin + total[0];
  __syncthreads();
  for (int64_t base = begin; base < end; base += kSortThreads) {
    const int64_t i = base + t;
    const uint64_t key = key_next;
    const uint32_t val = val_next;
    if (i + kSortThreads < end) {
      key_next = keys_in[i + kSortThreads];
      val_next = vals_in[i + kSortThreads];
    }
    scatter_slice<1>(i < end, key, val, (uint32_t)(key >> shift) & mask, cursor, wave_count, keys_out, vals_out);
  }
}

}  // namespace

size_t sort_temp_bytes(int64_t n) {
  SortPlan p = plan_sort(n);
  return align_up(((size_t)(1 << kMaxDigitBits) * p.stride + (1 << kMaxDigitBits) + 1) * sizeof(uint32_t), 256);
}

int sort_pairs(uint64_t* keys_in, uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out, int64_t n, int low_bit,
               int key_bits, void* temp, hipStream_t stream, uint64_t** keys_sorted, uint32_t** vals_sorted) {
  *keys_sorted = keys_in;
  *vals_sorted = vals_in;
  if (n <= 0) return PBG_OK;
  if (n >= (int64_t)1 << 32)
    return fail(PBG_ERR_UNSUPPORTED, "sort_pairs: n=%lld does not fit 32-bit offsets", (long long)n);
  if (low_bit < 0 || key_bits > 64 || low_bit > key_bits) return fail(PBG_ERR_INVALID, "sort_pairs: bad bit range");
  SortPlan p = plan_sort(n);
  uint32_t* counts = (uint32_t*)temp;
  uint32_t* bucket_off = counts + (size_t)(1 << kMaxDigitBits) * p.stride;
  int bits = key_bits - low_bit;
  if (bits < 1) bits = 1;
  const int top = bits < kMaxDigitBits ? bits : kMaxDigitBits;  // width of the global pass
  const int rest = bits - top;                                  // bits left for the bucket passes
  const int local = (rest + 7) / 8;
  const int top_shift = low_bit + rest;
  hipLaunchKernelGGL(sort_hist_kernel, dim3(p.blocks), dim3(kSortThreads), 0, stream, keys_in, n, p.tile_shift,
                     top_shift, top, p.stride, counts);
  if (top <= 8) {
    hipLaunchKernelGGL(sort_scatter_kernel<1>, dim3(p.blocks), dim3(kSortThreads), 0, stream, keys_in, vals_in,
                       keys_out, vals_out, n, p.tile_shift, top_shift, top, p.stride, counts, bucket_off);
  } else {
    hipLaunchKernelGGL(sort_scatter_kernel<2>, dim3(p.blocks), dim3(kSortThreads), 0, stream, keys_in, vals_in,
                       keys_out, vals_out, n, p.tile_shift, top_shift, top, p.stride, counts, bucket_off);
  }
  uint64_t* ksrc = keys_out;
  uint32_t* vsrc = vals_out;
  uint64_t* kdst = keys_in;
  uint32_t* vdst = vals_in;
  int shift = low_bit;
  for (int pass = 0; pass < local; ++pass) {  // lowest digit first; digits of (almost) equal width
    const int width = (rest - (shift - low_bit) + (local - pass) - 1) / (local - pass);
    hipLaunchKernelGGL(sort_bucket_kernel, dim3(1u << top), dim3(kSortThreads), 0, stream, ksrc, vsrc, kdst, vdst,
                       bucket_off, shift, width);
    shift += width;
    uint64_t* tk = ksrc; ksrc = kdst; kdst = tk;
    uint32_t* tv = vsrc; vsrc = vdst; vdst = tv;
  }
  *keys_sorted = ksrc;
  *vals_sorted = vsrc;
  return check_launch("sort_pairs");
}

}  // namespace pbg
