// Stable radix sort of (uint64 key, uint32 value) pairs on a bit range of the key.
//
// The top (up to 9) bits of the range are sorted by ONE global pass: every block
// owns a contiguous power-of-two tile of at least 4096 positions, a histogram
// kernel counts the digit per tile, and the scatter kernel derives its digit
// offsets from the per-tile counts of all tiles (at most 256 tiles, and few for
// the sizes of a training step, so the table that every block reads stays
// small), ranks its keys slice by slice (ballot matching inside a wave, LDS
// counts across the 16 waves, a running per-digit cursor across slices) and
// scatters them.  That leaves one bucket per digit value, contiguous in memory;
// the remaining low bits are sorted inside each bucket, one block per bucket, in
// ONE launch: no counts to exchange between blocks, no atomics on global memory.
// A bucket of up to `cap` keys (the common case: a few times the mean bucket) is
// sorted inside LDS -- its remaining bits and its positions packed into 32-bit
// words that go through all the digit passes there, then one gather of the
// bucket's pairs in sorted order -- so its keys cross HBM once more instead of
// once per digit; a larger bucket (swollen by a hot key) walks its digit passes
// through global memory, 8 bits per pass from the lowest up, with block barriers
// between them.  Every step is stable, so equal keys keep the order of the
// input, which keeps segmented gradient sums deterministic and lets a caller
// whose input is already ordered by the low bits leave those bits out.
#include <cstdlib>

#include "pbg_internal.h"

namespace pbg {
namespace {

constexpr int kGlobalWaves = 16;  // global pass: 1024 threads per block
constexpr int kBucketWaves = 16;  // bucket passes: 1024 threads per block, for the sake of buckets swollen by hot keys
constexpr int kMaxDigitBits = 9;
constexpr int kMaxDigits = 1 << kMaxDigitBits;
constexpr int kMaxSortBlocks = 256;
constexpr int kMinTileShift = 12;

struct SortPlan {
  int tile_shift;  // keys per block = 1 << tile_shift
  int blocks;
};

SortPlan plan_sort(int64_t n) {
  SortPlan p;
  p.tile_shift = kMinTileShift;
  while (ceil_div(n, (int64_t)1 << p.tile_shift) > kMaxSortBlocks) ++p.tile_shift;
  p.blocks = (int)ceil_div(n > 0 ? n : 1, (int64_t)1 << p.tile_shift);
  return p;
}

// counts[block][kMaxDigits] of the global pass.  With `idx` the pairs are made on the way: key = idx[i]
// (an index outside [0, park) is parked at `park`), value = i -- the stand-alone RowAdagrad step's keys
// need no pass of their own then.
__global__ __launch_bounds__(kGlobalWaves * 64) void sort_hist_kernel(uint64_t* __restrict__ keys, int64_t n,
                                                                      int tile_shift, int shift, int digit_bits,
                                                                      uint32_t* __restrict__ counts,
                                                                      uint32_t* __restrict__ long_flag,
                                                                      uint32_t long_init,
                                                                      const int64_t* __restrict__ idx, int64_t park,
                                                                      uint32_t* __restrict__ vals) {
  __shared__ uint32_t hist[kMaxDigits];
  if (blockIdx.x == 0 && threadIdx.x < kLongWords) long_flag[threadIdx.x] = threadIdx.x == 0 ? long_init : 0u;
  const uint32_t mask = (1u << digit_bits) - 1u;
  if (threadIdx.x < kMaxDigits) hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x << tile_shift;
  int64_t end = begin + ((int64_t)1 << tile_shift);
  if (end > n) end = n;
  if (idx) {
    for (int64_t i = begin + threadIdx.x; i < end; i += kGlobalWaves * 64) {
      int64_t r = idx[i];
      if (r < 0 || r >= park) r = park;
      keys[i] = (uint64_t)r;
      vals[i] = (uint32_t)i;
      atomicAdd(&hist[(uint32_t)((uint64_t)r >> shift) & mask], 1u);
    }
  } else {
    for (int64_t i = begin + threadIdx.x; i < end; i += kGlobalWaves * 64)
      atomicAdd(&hist[(uint32_t)(keys[i] >> shift) & mask], 1u);
  }
  __syncthreads();
  if (threadIdx.x < kMaxDigits) counts[(int64_t)blockIdx.x * kMaxDigits + threadIdx.x] = hist[threadIdx.x];
}

// Exclusive scan over one value per thread of the first `waves` waves of the
// block (all threads of the block must call it); *grand gets the sum.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t value, int waves, uint32_t* wave_total,
                                                         uint32_t* grand) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint32_t incl = value;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63 && wave < waves) wave_total[wave] = incl;
  __syncthreads();
  uint32_t ahead = 0, all = 0;
  for (int w = 0; w < waves; ++w) {
    const uint32_t wt = wave_total[w];
    if (w < wave) ahead += wt;
    all += wt;
  }
  __syncthreads();
  *grand = all;
  return ahead + incl - value;
}

// Rank-and-scatter state of one block: NW waves, digits of up to BITS bits.
template <int NW, int BITS>
struct SliceState {
  uint32_t cursor[1 << BITS];             // next output slot of each digit
  uint32_t slot[1 << BITS];               // first output slot of each digit in the current slice
  uint16_t wave_count[2][NW][1 << BITS];  // per-wave digit counts, one buffer per slice parity
  uint32_t wave_total[NW];
};

// One slice of up to NW * 64 keys: rank every key among the keys of the slice
// with the same digit (earlier positions first), scatter it to cursor[digit] +
// rank, advance the cursors.  Both count buffers must be zero before the first
// slice; each slice clears the buffer the previous one used.
template <int NW, int BITS>
__device__ __forceinline__ void scatter_slice(SliceState<NW, BITS>& st, int parity, bool valid, uint64_t key,
                                              uint32_t val, uint32_t digit, uint64_t* __restrict__ keys_out,
                                              uint32_t* __restrict__ vals_out) {
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  // lanes of this wave holding the same digit
  uint64_t peers = __ballot(valid);
#pragma unroll
  for (int b = 0; b < BITS; ++b) {
    const bool bit = (digit >> b) & 1u;
    const uint64_t m = __ballot(valid && bit);
    peers &= bit ? m : ~m;
  }
  const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  const int rank_in_wave = __popcll(peers & below);
  if (valid && rank_in_wave == 0) st.wave_count[parity][wave][digit] = (uint16_t)__popcll(peers);
  __syncthreads();
  // per digit: the waves' counts become the waves' offsets from the digit's first slot
  for (int d = t; d < (1 << BITS); d += NW * 64) {
    uint32_t at = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const uint32_t c = st.wave_count[parity][w][d];
      st.wave_count[parity][w][d] = (uint16_t)at;
      at += c;
      st.wave_count[parity ^ 1][w][d] = 0;
    }
    const uint32_t first = st.cursor[d];
    st.slot[d] = first;
    st.cursor[d] = first + at;
  }
  __syncthreads();
  if (valid) {
    const uint32_t pos = st.slot[digit] + st.wave_count[parity][wave][digit] + (uint32_t)rank_in_wave;
    keys_out[pos] = key;
    vals_out[pos] = val;
  }
}

template <int NW, int BITS>
__device__ __forceinline__ void scatter_range(SliceState<NW, BITS>& st, const uint64_t* __restrict__ keys_in,
                                              const uint32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
                                              uint32_t* __restrict__ vals_out, int64_t begin, int64_t end, int shift,
                                              uint32_t mask, uint64_t key_next, uint32_t val_next) {
  const int t = threadIdx.x;
  int parity = 0;
  // the next slice's loads are issued before the current slice is ranked
  for (int64_t base = begin; base < end; base += NW * 64) {
    const int64_t i = base + t;
    const uint64_t key = key_next;
    const uint32_t val = val_next;
    if (i + NW * 64 < end) {
      key_next = keys_in[i + NW * 64];
      val_next = vals_in[i + NW * 64];
    }
    scatter_slice<NW, BITS>(st, parity, i < end, key, val, (uint32_t)(key >> shift) & mask, keys_out, vals_out);
    parity ^= 1;
  }
}

// The same for a bucket swollen by hot keys (a power-law graph puts tens of
// thousands of equal row numbers into one bucket, which one block walks slice by
// slice): KPT keys per thread and slice.  A wave owns KPT * 64 CONSECUTIVE
// positions of the slice, 64 at a time, so that (wave, round, lane) is the order
// of the positions and the ranks stay stable; its digit counts accumulate over
// the rounds in its own row of wave_count (no other wave touches it, so the
// rounds need no barrier), and the two barriers and the walk over the waves'
// counts are paid once per KPT * NW * 64 keys instead of once per NW * 64.
// The lanes of the wave whose key has the same digit as this lane's (valid lanes only).  A bucket
// is swollen by ONE hot key, so most rounds of 64 consecutive keys carry a single digit value: that
// case costs two ballots instead of one per bit.
template <int BITS>
__device__ __forceinline__ uint64_t digit_peers(uint32_t digit, bool valid) {
  const uint64_t all = __ballot(valid);
  const uint32_t first = (uint32_t)__builtin_amdgcn_readfirstlane((int)digit);
  if ((all & 1ull) && __ballot(valid && digit == first) == all) return all;
  uint64_t peers = all;
#pragma unroll
  for (int b = 0; b < BITS; ++b) {
    const bool bit = (digit >> b) & 1u;
    const uint64_t m = __ballot(valid && bit);
    peers &= bit ? m : ~m;
  }
  return peers;
}

template <int NW, int BITS, int KPT>
__device__ __forceinline__ void scatter_range_wide(SliceState<NW, BITS>& st, const uint64_t* __restrict__ keys_in,
                                                   const uint32_t* __restrict__ vals_in,
                                                   uint64_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out,
                                                   int64_t begin, int64_t end, int shift, uint32_t mask,
                                                   const uint64_t* first_keys = nullptr,
                                                   const uint32_t* first_vals = nullptr) {
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  constexpr int kSlice = NW * 64 * KPT;
  const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  int parity = 0;
  uint64_t key[KPT], key_next[KPT];
  uint32_t val[KPT], val_next[KPT];
  auto fetch = [&](int64_t base) {
#pragma unroll
    for (int q = 0; q < KPT; ++q) {
      const int64_t i = base + (int64_t)wave * (64 * KPT) + q * 64 + lane;
      key_next[q] = i < end ? keys_in[i] : 0ull;
      val_next[q] = i < end ? vals_in[i] : 0u;
    }
  };
  if (first_keys) {  // the caller fetched the first slice already (wide_fetch)
#pragma unroll
    for (int q = 0; q < KPT; ++q) {
      key_next[q] = first_keys[q];
      val_next[q] = first_vals[q];
    }
  } else {
    fetch(begin);
  }
  for (int64_t base = begin; base < end; base += kSlice) {
#pragma unroll
    for (int q = 0; q < KPT; ++q) {
      key[q] = key_next[q];
      val[q] = val_next[q];
    }
    if (base + kSlice < end) fetch(base + kSlice);  // the next slice's loads are issued before this one is ranked
    uint32_t rank[KPT], digit[KPT];
    bool valid[KPT];
#pragma unroll
    for (int q = 0; q < KPT; ++q) {
      const int64_t i = base + (int64_t)wave * (64 * KPT) + q * 64 + lane;
      valid[q] = i < end;
      digit[q] = (uint32_t)(key[q] >> shift) & mask;
      const uint64_t peers = digit_peers<BITS>(digit[q], valid[q]);
      const int rank_in_round = __popcll(peers & below);
      const uint32_t prior = valid[q] ? st.wave_count[parity][wave][digit[q]] : 0u;  // this wave's earlier rounds
      rank[q] = prior + (uint32_t)rank_in_round;
      if (valid[q] && rank_in_round == 0) st.wave_count[parity][wave][digit[q]] = (uint16_t)(prior + __popcll(peers));
    }
    __syncthreads();
    for (int d = t; d < (1 << BITS); d += NW * 64) {
      uint32_t at = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const uint32_t c = st.wave_count[parity][w][d];
        st.wave_count[parity][w][d] = (uint16_t)at;
        at += c;
        st.wave_count[parity ^ 1][w][d] = 0;
      }
      const uint32_t first = st.cursor[d];
      st.slot[d] = first;
      st.cursor[d] = first + at;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < KPT; ++q) {
      if (valid[q]) {
        const uint32_t pos = st.slot[digit[q]] + st.wave_count[parity][wave][digit[q]] + rank[q];
        keys_out[pos] = key[q];
        vals_out[pos] = val[q];
      }
    }
    parity ^= 1;
  }
}

// This thread's keys of the slice that starts at `base`, in scatter_range_wide's layout.
template <int KPT>
__device__ __forceinline__ void wide_fetch(const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in,
                                           int64_t base, int64_t end, uint64_t* k, uint32_t* v) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int q = 0; q < KPT; ++q) {
    const int64_t i = base + (int64_t)wave * (64 * KPT) + q * 64 + lane;
    k[q] = i < end ? keys_in[i] : 0ull;
    v[q] = i < end ? vals_in[i] : 0u;
  }
}

// The global pass.  Block 0 also writes the bucket offsets (digit d's keys end up
// in [bucket_off[d], bucket_off[d + 1])).
__global__ __launch_bounds__(kGlobalWaves * 64) void sort_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int64_t n, int tile_shift, int shift, int digit_bits,
    const uint32_t* __restrict__ counts, uint32_t* __restrict__ bucket_off, uint32_t* __restrict__ bucket_order) {
  __shared__ SliceState<kGlobalWaves, kMaxDigitBits> st;
  __shared__ uint32_t part[2][2][kMaxDigits];  // [half][total, before][digit]
  const int t = threadIdx.x;
  const int me = blockIdx.x, blocks = gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x << tile_shift;
  int64_t end = begin + ((int64_t)1 << tile_shift);
  if (end > n) end = n;
  constexpr int kGlobalKpt = 4;  // a tile is at least 4096 keys: one slice of 4 keys per thread
  uint64_t first_keys[kGlobalKpt];
  uint32_t first_vals[kGlobalKpt];
  wide_fetch<kGlobalKpt>(keys_in, vals_in, begin, end, first_keys, first_vals);
  // offset of digit d for this block = keys with a smaller digit anywhere
  //                                  + keys with digit d in earlier blocks;
  // two threads per digit, each over every other block, 16 loads in flight
  {
    const int d = t & (kMaxDigits - 1), half = t >> kMaxDigitBits;
    uint32_t total = 0, before = 0;
    for (int b0 = half; b0 < blocks; b0 += 32) {
      uint32_t c[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) c[u] = (b0 + 2 * u < blocks) ? counts[(int64_t)(b0 + 2 * u) * kMaxDigits + d] : 0u;
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        total += c[u];
        if (b0 + 2 * u < me) before += c[u];
      }
    }
    part[half][0][d] = total;
    part[half][1][d] = before;
    for (int w = 0; w < kGlobalWaves; ++w) st.wave_count[half][w][d] = 0;
  }
  __syncthreads();
  uint32_t total = 0, before = 0;
  if (t < kMaxDigits) {
    total = part[0][0][t] + part[1][0][t];
    before = part[0][1][t] + part[1][1][t];
  }
  uint32_t grand;
  const uint32_t excl = block_exclusive_scan(total, kMaxDigits / 64, st.wave_total, &grand);
  if (t < kMaxDigits) {
    st.cursor[t] = excl + before;
    if (me == 0) bucket_off[t] = excl;  // digits past the pass's width hold no keys: their offset is n
  }
  if (me == 0 && t == 0) bucket_off[kMaxDigits] = grand;
  // The order in which the bucket passes' launch takes the buckets: those swollen by a hot key first (more than four
  // times the mean), the others behind them, each group by digit.  A swollen bucket is one workgroup's long chain of
  // slices, and it should be the first to start, not wait behind hundreds of ordinary ones.  The last block writes
  // the order (its tile is the one that may be short).
  if (bucket_order && me == blocks - 1) {
    const uint32_t limit = 4u * (grand >> digit_bits) + 1024u;
    const uint32_t big = (t < kMaxDigits && total > limit) ? 1u : 0u;
    uint32_t num_big;
    const uint32_t big_before = block_exclusive_scan(big, kMaxDigits / 64, st.wave_total, &num_big);
    if (t < kMaxDigits) bucket_order[big ? big_before : num_big + ((uint32_t)t - big_before)] = (uint32_t)t;
  }
  __syncthreads();
  scatter_range_wide<kGlobalWaves, kMaxDigitBits, kGlobalKpt>(st, keys_in, vals_in, keys_out, vals_out, begin, end,
                                                              shift, (1u << digit_bits) - 1u, first_keys, first_vals);
}

// One digit pass of a bucket through global memory.
__device__ __forceinline__ void bucket_pass_global(SliceState<kBucketWaves, 8>& st, const uint64_t* keys_in,
                                                   const uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out,
                                                   int64_t begin, int64_t end, int shift, int digit_bits) {
  const int t = threadIdx.x;
  const uint32_t mask = (1u << digit_bits) - 1u;
  const bool wide = end - begin > 2 * kBucketWaves * 64;  // a swollen bucket
  uint64_t key_next = 0;
  uint32_t val_next = 0;
  if (begin + t < end) {
    key_next = keys_in[begin + t];
    val_next = vals_in[begin + t];
  }
  if (t < 256) {
    st.cursor[t] = 0;
    for (int w = 0; w < kBucketWaves; ++w) st.wave_count[0][w][t] = st.wave_count[1][w][t] = 0;
  }
  __syncthreads();
  if (!wide) {
    if (begin + t < end) atomicAdd(&st.cursor[(uint32_t)(key_next >> shift) & mask], 1u);
    for (int64_t i = begin + kBucketWaves * 64 + t; i < end; i += kBucketWaves * 64)
      atomicAdd(&st.cursor[(uint32_t)(keys_in[i] >> shift) & mask], 1u);
  } else {
    // equal keys would queue up on one counter: one addition per wave and digit value present.
    // Eight loads per thread in flight (the ballots would otherwise wait for each load in turn).
    const int lane = t & 63;
    const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    constexpr int kInFlight = 8;
    for (int64_t base = begin; base < end; base += (int64_t)kInFlight * kBucketWaves * 64) {
      uint64_t kq[kInFlight];
#pragma unroll
      for (int q = 0; q < kInFlight; ++q) {
        const int64_t i = base + (int64_t)q * kBucketWaves * 64 + t;
        kq[q] = i < end ? keys_in[i] : 0ull;
      }
#pragma unroll
      for (int q = 0; q < kInFlight; ++q) {
        const bool valid = base + (int64_t)q * kBucketWaves * 64 + t < end;
        const uint32_t digit = (uint32_t)(kq[q] >> shift) & mask;
        const uint64_t peers = digit_peers<8>(digit, valid);
        if (valid && (peers & below) == 0ull) atomicAdd(&st.cursor[digit], (uint32_t)__popcll(peers));
      }
    }
  }
  __syncthreads();
  uint32_t grand;
  const uint32_t excl = block_exclusive_scan(t < 256 ? st.cursor[t] : 0u, 4, st.wave_total, &grand);
  if (t < 256) st.cursor[t] = (uint32_t)begin + excl;
  __syncthreads();
  if (wide)
    scatter_range_wide<kBucketWaves, 8, 4>(st, keys_in, vals_in, keys_out, vals_out, begin, end, shift, mask);
  else
    scatter_range<kBucketWaves, 8>(st, keys_in, vals_in, keys_out, vals_out, begin, end, shift, mask, key_next,
                                   val_next);
}

// One digit pass of a bucket's packed words inside LDS: `from` -> `to`, m words, digit = bits
// [shift, shift + digit_bits) of a word.  Same ranking as the global passes (a wave owns 4 x 64
// consecutive words of a slice of 4096, so (wave, round, lane) is the order of the positions).
__device__ __forceinline__ void bucket_pass_lds(SliceState<kBucketWaves, 8>& st, const uint32_t* from, uint32_t* to,
                                                int m, int shift, int digit_bits) {
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  const uint32_t mask = (1u << digit_bits) - 1u;
  constexpr int kKpt = 4, kSlice = kBucketWaves * 64 * kKpt;
  if (t < 256) {
    st.cursor[t] = 0;
    for (int w = 0; w < kBucketWaves; ++w) st.wave_count[0][w][t] = st.wave_count[1][w][t] = 0;
  }
  __syncthreads();
  for (int i = t; i < m; i += kBucketWaves * 64) atomicAdd(&st.cursor[(from[i] >> shift) & mask], 1u);
  __syncthreads();
  uint32_t grand;
  const uint32_t excl = block_exclusive_scan(t < 256 ? st.cursor[t] : 0u, 4, st.wave_total, &grand);
  if (t < 256) st.cursor[t] = excl;
  __syncthreads();
  const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  int parity = 0;
  for (int base = 0; base < m; base += kSlice) {
    uint32_t word[kKpt], digit[kKpt], rank[kKpt];
    bool valid[kKpt];
#pragma unroll
    for (int q = 0; q < kKpt; ++q) {
      const int i = base + wave * (64 * kKpt) + q * 64 + lane;
      valid[q] = i < m;
      word[q] = valid[q] ? from[i] : 0u;
      digit[q] = (word[q] >> shift) & mask;
      const uint64_t peers = digit_peers<8>(digit[q], valid[q]);
      const int rank_in_round = __popcll(peers & below);
      const uint32_t prior = valid[q] ? st.wave_count[parity][wave][digit[q]] : 0u;  // this wave's earlier rounds
      rank[q] = prior + (uint32_t)rank_in_round;
      if (valid[q] && rank_in_round == 0) st.wave_count[parity][wave][digit[q]] = (uint16_t)(prior + __popcll(peers));
    }
    __syncthreads();
    if (t < 256) {
      uint32_t at = 0;
#pragma unroll
      for (int w = 0; w < kBucketWaves; ++w) {
        const uint32_t c = st.wave_count[parity][w][t];
        st.wave_count[parity][w][t] = (uint16_t)at;
        at += c;
        st.wave_count[parity ^ 1][w][t] = 0;
      }
      const uint32_t first = st.cursor[t];
      st.slot[t] = first;
      st.cursor[t] = first + at;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kKpt; ++q)
      if (valid[q]) to[st.slot[digit[q]] + st.wave_count[parity][wave][digit[q]] + rank[q]] = word[q];
    parity ^= 1;
  }
  __syncthreads();
}

constexpr int kLdsIndexBits = 14;              // a bucket sorted inside LDS holds at most 2^14 keys ...
constexpr int kLdsMaxRestBits = 32 - kLdsIndexBits;  // ... and its remaining bits share a 32-bit word with the position

// All the bucket passes of one sort.  Block b sorts bucket b (positions [bucket_off[b],
// bucket_off[b + 1]) of the pair (ka, va), where the global pass left it) by bits
// [low_bit, low_bit + rest) of the key; the result goes to the same positions of (kfin, vfin), which
// is (ka, va) or (kb, vb) depending on the parity of `passes` (the number of digit passes a bucket too
// large for LDS takes through global memory).  `long_flag`, if given, is raised when some value of the
// sorted bits occurs more than kFoldMax times in a bucket sorted here (or the bucket was not looked at).
__global__ __launch_bounds__(kBucketWaves * 64) void sort_bucket_kernel(uint64_t* ka, uint32_t* va, uint64_t* kb,
                                                                        uint32_t* vb, uint64_t* kfin, uint32_t* vfin,
                                                                        const uint32_t* __restrict__ bucket_off,
                                                                        const uint32_t* __restrict__ bucket_order,
                                                                        int low_bit, int rest, int passes, int cap,
                                                                        uint32_t* __restrict__ long_flag) {
  __shared__ SliceState<kBucketWaves, 8> st;
  extern __shared__ uint32_t lds_words[];  // 2 * cap packed words
  const int t = threadIdx.x;
  const uint32_t bucket = bucket_order[blockIdx.x];  // largest first
  const int64_t begin = bucket_off[bucket], end = bucket_off[bucket + 1];
  if (begin >= end) return;
  const int64_t m64 = end - begin;
  // (a single digit pass gains nothing from the detour through LDS: one read and one write either way)
  if (passes >= 2 && m64 <= cap && rest <= kLdsMaxRestBits) {
    const int m = (int)m64;
    uint32_t* from = lds_words;
    uint32_t* to = lds_words + cap;
    const uint32_t rest_mask = rest >= 32 ? 0xffffffffu : ((1u << rest) - 1u);
    for (int i = t; i < m; i += kBucketWaves * 64)
      from[i] = (((uint32_t)(ka[begin + i] >> low_bit) & rest_mask) << kLdsIndexBits) | (uint32_t)i;
    // (bucket_pass_lds starts with a barrier)
    const int lds_passes = (rest + 7) / 8;
    int shift = kLdsIndexBits;
    for (int pass = 0; pass < lds_passes; ++pass) {  // lowest digit first; digits of (almost) equal width
      const int width = (rest - (shift - kLdsIndexBits) + (lds_passes - pass) - 1) / (lds_passes - pass);
      bucket_pass_lds(st, from, to, m, shift, width);
      shift += width;
      uint32_t* tmp = from; from = to; to = tmp;
    }
    if (long_flag) {
      bool found = false;
      for (int i = t; i + kFoldMax < m; i += kBucketWaves * 64)
        found |= (from[i] >> kLdsIndexBits) == (from[i + kFoldMax] >> kLdsIndexBits);
      if (found) *long_flag = 1u;
    }
    // The pairs in sorted order.  All of a thread's reads come before its first write, and a barrier
    // in between: the result may go where the bucket was read from.
    constexpr int kMaxPerThread = (1 << kLdsIndexBits) / (kBucketWaves * 64);
    uint64_t k[kMaxPerThread];
    uint32_t v[kMaxPerThread];
#pragma unroll
    for (int r = 0; r < kMaxPerThread; ++r) {
      const int j = r * kBucketWaves * 64 + t;
      if (j < m) {
        const int64_t src = begin + (from[j] & ((1u << kLdsIndexBits) - 1u));
        k[r] = ka[src];
        v[r] = va[src];
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kMaxPerThread; ++r) {
      const int j = r * kBucketWaves * 64 + t;
      if (j < m) {
        kfin[begin + j] = k[r];
        vfin[begin + j] = v[r];
      }
    }
    return;
  }
  uint64_t* ksrc = ka;
  uint32_t* vsrc = va;
  uint64_t* kdst = kb;
  uint32_t* vdst = vb;
  int shift = low_bit;
  for (int pass = 0; pass < passes; ++pass) {
    const int width = (rest - (shift - low_bit) + (passes - pass) - 1) / (passes - pass);
    bucket_pass_global(st, ksrc, vsrc, kdst, vdst, begin, end, shift, width);
    shift += width;
    uint64_t* tk = ksrc; ksrc = kdst; kdst = tk;
    uint32_t* tv = vsrc; vsrc = vdst; vdst = tv;
    __syncthreads();  // the next pass reads what this one wrote (same block, workgroup scope)
  }
  if (long_flag) {  // the bucket as it lies now: is some value of the sorted bits there more than kFoldMax times?
    bool found = false;
    for (int64_t i = begin + t; i + kFoldMax < end; i += kBucketWaves * 64)
      found |= (ksrc[i] >> low_bit) == (ksrc[i + kFoldMax] >> low_bit);
    if (found) *long_flag = 1u;
  }
}

// ---- a small input in ONE launch ------------------------------------------------------------------
// Up to kRankMax pairs: three dependent launches of the radix sort cost more than their work there (a
// single-batch training step has a few thousand keys).  The place of pair i in the stable order is the
// number of pairs j whose field is smaller, plus the number of j < i whose field is equal.  A workgroup
// owns kRankKeys consecutive pairs and copies ALL fields into LDS; the fields are cut into 64 shares, and
// lane (share % 4) * 16 + p of wave share / 4 counts pair p against that share (the 16 lanes of a group read
// the same words).  The 64 counts of a pair meet in LDS and the pair goes to its place.  n^2 comparisons in
// all, spread over n / 16 workgroups: 16 M for the 4000 keys of a single batch.
constexpr int kRankMax = 1 << 13;
constexpr int kRankWaves = 16;
constexpr int kRankKeys = 16;
constexpr int kRankShares = kRankWaves * 4;

template <bool FLAG>
__global__ __launch_bounds__(kRankWaves * 64) void sort_rank_kernel(
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ vals, uint64_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int n, int low_bit, uint32_t mask, uint32_t* __restrict__ long_flag,
    const int64_t* __restrict__ idx, int64_t park) {
  extern __shared__ uint32_t rank_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n4 = (n + 3) & ~3;
  uint32_t* field = rank_lds;      // [n4]
  uint32_t* part = rank_lds + n4;  // [3][kRankShares][kRankKeys]: smaller; equal and earlier; equal
  auto key_of = [&](int j) -> uint64_t {
    if (!idx) return keys[j];
    const int64_t r = idx[j];
    return (uint64_t)((r < 0 || r >= park) ? park : r);
  };
  for (int j = tid; j < n; j += kRankWaves * 64) field[j] = (uint32_t)(key_of(j) >> low_bit) & mask;
  __syncthreads();

  const int p = lane & (kRankKeys - 1), share = wave * 4 + (lane >> 4);
  const int i = blockIdx.x * kRankKeys + p;
  const uint32_t mine = field[i < n ? i : n - 1];
  const int len = ((n4 / 4 + kRankShares - 1) / kRankShares) * 4;  // whole quads, except at the end of the input
  const int s0 = min(share * len, n), s1 = min(s0 + len, n);
  uint32_t lt = 0, eq = 0, eqb = 0;
  int j = s0;
  for (; j + 4 <= s1; j += 4) {
    const uint4 f = *reinterpret_cast<const uint4*>(&field[j]);
    lt += (uint32_t)(f.x < mine) + (uint32_t)(f.y < mine) + (uint32_t)(f.z < mine) + (uint32_t)(f.w < mine);
    const uint32_t e0 = f.x == mine, e1 = f.y == mine, e2 = f.z == mine, e3 = f.w == mine;
    if (FLAG) eq += e0 + e1 + e2 + e3;
    eqb += (e0 & (uint32_t)(j < i)) + (e1 & (uint32_t)(j + 1 < i)) + (e2 & (uint32_t)(j + 2 < i)) + (e3 & (uint32_t)(j + 3 < i));
  }
  for (; j < s1; ++j) {
    const uint32_t f = field[j];
    lt += (uint32_t)(f < mine);
    if (FLAG) eq += (uint32_t)(f == mine);
    eqb += (uint32_t)(f == mine) & (uint32_t)(j < i);
  }
  part[(0 * kRankShares + share) * kRankKeys + p] = lt + eqb;
  if (FLAG) part[(1 * kRankShares + share) * kRankKeys + p] = eq;
  __syncthreads();
  if (wave != 0) return;
  // lane (q, p) adds the shares q, q + 4, ... of pair p; the four q meet through the lanes' exchange
  uint32_t place = 0, same = 0;
  const int q = lane >> 4;
#pragma unroll
  for (int w = 0; w < kRankWaves; ++w) {
    place += part[(0 * kRankShares + w * 4 + q) * kRankKeys + p];
    if (FLAG) same += part[(1 * kRankShares + w * 4 + q) * kRankKeys + p];
  }
  place += __shfl_xor(place, 16, 64);
  place += __shfl_xor(place, 32, 64);
  if (FLAG) {
    same += __shfl_xor(same, 16, 64);
    same += __shfl_xor(same, 32, 64);
  }
  const bool owner = lane < kRankKeys && i < n;
  if (owner) {
    keys_out[place] = key_of(i);
    vals_out[place] = idx ? (uint32_t)i : vals[i];
  }
  if (FLAG) {
    // every workgroup leaves its own word, and the first one clears the words no workgroup owns
    const bool found = __ballot(owner && same > (uint32_t)kFoldMax) != 0ull;
    if (lane == 0) long_flag[blockIdx.x] = found ? 1u : 0u;
    if (blockIdx.x == 0)
      for (int w = (int)gridDim.x + lane; w < kLongWords; w += 64) long_flag[w] = 0u;
  }
}

}  // namespace

size_t sort_temp_bytes(int64_t n) {
  SortPlan p = plan_sort(n);
  return align_up(((size_t)kMaxDigits * p.blocks + kMaxDigits + 1 + kLongWords + kMaxDigits) * sizeof(uint32_t), 256);
}

namespace {
LdsLimit g_bucket_lds, g_rank_lds[2];
}

int sort_pairs(uint64_t* keys_in, uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out, int64_t n, int low_bit,
               int key_bits, void* temp, hipStream_t stream, uint64_t** keys_sorted, uint32_t** vals_sorted,
               const uint32_t** long_runs, const int64_t* indices, int64_t park) {
  *keys_sorted = keys_in;
  *vals_sorted = vals_in;
  if (long_runs) *long_runs = nullptr;
  if (n <= 0) return PBG_OK;
  if (n >= (int64_t)1 << 32)
    return fail(PBG_ERR_UNSUPPORTED, "sort_pairs: n=%lld does not fit 32-bit offsets", (long long)n);
  if (low_bit < 0 || key_bits > 64 || low_bit > key_bits) return fail(PBG_ERR_INVALID, "sort_pairs: bad bit range");
  SortPlan p = plan_sort(n);
  uint32_t* counts = (uint32_t*)temp;
  uint32_t* bucket_off = counts + (size_t)kMaxDigits * p.blocks;
  uint32_t* long_flag = bucket_off + kMaxDigits + 1;
  uint32_t* bucket_order = long_flag + kLongWords;  // [kMaxDigits]
  int bits = key_bits - low_bit;
  if (bits < 1) bits = 1;
  if (n <= kRankMax && bits <= 32 && getenv("PBG_DISABLE_RANK_SORT") == nullptr) {  // one launch, see sort_rank_kernel
    static_assert(kRankMax / kRankKeys <= kLongWords, "one word per workgroup");
    const size_t lds_bytes = ((size_t)((n + 3) & ~(int64_t)3) + 2 * kRankShares * kRankKeys) * sizeof(uint32_t);
    const uint32_t mask = bits == 32 ? 0xffffffffu : ((1u << bits) - 1u);
    const dim3 grid((unsigned)ceil_div(n, kRankKeys)), block(kRankWaves * 64);
    int rc;
    if (long_runs) {
      if ((rc = reserve_lds((const void*)sort_rank_kernel<true>, &g_rank_lds[1], lds_bytes)) != PBG_OK) return rc;
      hipLaunchKernelGGL(sort_rank_kernel<true>, grid, block, lds_bytes, stream, keys_in, vals_in, keys_out, vals_out, (int)n,
                         low_bit, mask, long_flag, indices, park);
      *long_runs = long_flag;
    } else {
      if ((rc = reserve_lds((const void*)sort_rank_kernel<false>, &g_rank_lds[0], lds_bytes)) != PBG_OK) return rc;
      hipLaunchKernelGGL(sort_rank_kernel<false>, grid, block, lds_bytes, stream, keys_in, vals_in, keys_out, vals_out, (int)n,
                         low_bit, mask, long_flag, indices, park);
    }
    *keys_sorted = keys_out;
    *vals_sorted = vals_out;
    return check_launch("sort_pairs");
  }
  const int top = bits < kMaxDigitBits ? bits : kMaxDigitBits;  // width of the global pass
  const int rest = bits - top;                                  // bits left for the bucket passes
  const int local = (rest + 7) / 8;
  const int top_shift = low_bit + rest;
  // without bucket passes nobody looks at the lengths of the runs: the flag then says "there may be long ones"
  hipLaunchKernelGGL(sort_hist_kernel, dim3(p.blocks), dim3(kGlobalWaves * 64), 0, stream, keys_in, n, p.tile_shift,
                     top_shift, top, counts, long_flag, local == 0 ? 1u : 0u, indices, park, vals_in);
  hipLaunchKernelGGL(sort_scatter_kernel, dim3(p.blocks), dim3(kGlobalWaves * 64), 0, stream, keys_in, vals_in,
                     keys_out, vals_out, n, p.tile_shift, top_shift, top, counts, bucket_off, local > 0 ? bucket_order : nullptr);
  if (long_runs) *long_runs = long_flag;
  if (local == 0) {
    *keys_sorted = keys_out;
    *vals_sorted = vals_out;
    return check_launch("sort_pairs");
  }
  // buckets of up to `cap` keys are sorted inside LDS: four times the mean bucket, between 2048 and 2^14 keys
  int64_t cap = 4 * ceil_div(n, (int64_t)1 << top);
  cap = cap < 2048 ? 2048 : (cap > (1 << kLdsIndexBits) ? (1 << kLdsIndexBits) : cap);
  cap = (cap + 1023) / 1024 * 1024;
  const size_t lds_bytes = (size_t)cap * 2 * sizeof(uint32_t);
  const int rc = reserve_lds((const void*)sort_bucket_kernel, &g_bucket_lds, lds_bytes);
  if (rc != PBG_OK) return rc;
  uint64_t* kfin = (local & 1) ? keys_in : keys_out;
  uint32_t* vfin = (local & 1) ? vals_in : vals_out;
  hipLaunchKernelGGL(sort_bucket_kernel, dim3(1u << top), dim3(kBucketWaves * 64), lds_bytes, stream, keys_out, vals_out,
                     keys_in, vals_in, kfin, vfin, bucket_off, bucket_order, low_bit, rest, local, (int)cap,
                     long_runs ? long_flag : nullptr);
  *keys_sorted = kfin;
  *vals_sorted = vfin;
  return check_launch("sort_pairs");
}

}  // namespace pbg
