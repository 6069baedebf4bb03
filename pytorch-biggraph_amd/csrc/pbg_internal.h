// Internal declarations shared by the HIP translation units of libpbg_hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "../../include/pbg_hip.h"

namespace pbg {

constexpr int kWave = 64;
// Largest embedding dimension: the per-row kernels keep a row in the registers of one wave,
// 64 floats per lane at this width.
constexpr int kMaxDim = 4096;

// Records `msg` for pbg_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);
// Turns the pending HIP launch error (if any) into a pbg_status.
int check_launch(const char* what);

// Per-device state of the library is kept for devices 0 .. kMaxDevices - 1.
constexpr int kMaxDevices = 16;
// The dynamic LDS limit a kernel has been given so far, per device.
struct LdsLimit {
  std::atomic<size_t> allowed[kMaxDevices];
};
// Raises `kernel`'s dynamic LDS limit on the current device to `bytes` unless it is that high already.
int reserve_lds(const void* kernel, LdsLimit* limit, size_t bytes);
// Compute units of the current device.
int compute_units();

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int bits_for(uint64_t max_value) {  // number of bits needed to hold max_value
  int b = 0;
  while (b < 64 && (max_value >> b) != 0) ++b;
  return b;
}

// ---- device radix sort of (uint64 key, uint32 value) pairs ----------------
// LSD radix sort, up to 9 bits per pass, stable.  Sorts on key bits
// [low_bit, key_bits): an input already ordered by the bits below low_bit comes
// out ordered by all bits below key_bits.  Both buffer pairs are clobbered; the
// result is in whichever pair *keys_sorted / *vals_sorted name on return.
// `temp` holds sort_temp_bytes(n) bytes.
// With `indices` the input pairs are made by the sort's first kernel instead of being read: key i = indices[i]
// (an index outside [0, park) becomes `park`), value i = i; keys_in / vals_in are then only written.
// If `long_runs` is given it receives a device pointer (into `temp`) to kLongWords words that are all zero after
// the sort only if no value of the sorted bits occurs more than kFoldMax times -- what lets a single-worker
// RowAdagrad step skip its duplicate-summation kernels.  (Several words: the kernel that sorts a small input
// in one launch has every workgroup leave its own finding, and nobody has to clear a shared word first.)
constexpr int kFoldMax = 8;
constexpr int kLongWords = 512;
size_t sort_temp_bytes(int64_t n);
int sort_pairs(uint64_t* keys_in, uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out, int64_t n, int low_bit,
               int key_bits, void* temp, hipStream_t stream, uint64_t** keys_sorted, uint32_t** vals_sorted,
               const uint32_t** long_runs = nullptr, const int64_t* indices = nullptr, int64_t park = 0);

// ---- segmented RowAdagrad over sorted (row << kbits | worker) keys ---------
// keys are sorted ascending; vals[i] indexes a row of grad_rows[*, dim], which is
// clobbered (duplicate sums are formed in place).  A key's row field addresses table 0 for row < rows0, table 1 (row - rows0) for
// row < rows0 + rows1, and is ignored beyond.
// `long_runs` (single-worker calls, kbits == 0): the kLongWords words sort_pairs leaves behind; where all are zero the
// duplicate-summation kernels return at once (no key occurs more than kFoldMax times, and the update
// kernel sums such runs itself).  nullptr: not known.
// `cos_back`: the gradient rows are gradients at the NORMALISED rows y = x / |x| of the tables (a step with the
// cos comparator that scored on a normalised copy of the tables): y0 / y1 are that copy of table 0 / 1 and
// inv0 / inv1 the rows' 1 / |x|, all as they were when the call began.  Every run's summed gradient then goes back
// through the normalisation, g <- (g - y <y, g>) / |x| (model.py:187-192 under autograd), before its Adagrad step.
struct CosBack {
  const float* y0; const float* inv0; const float* y1; const float* inv1;
};
// `sums`: per-batch totals that ride along with the first of the update's launches (a launch of their own costs more
// than their work: five microseconds per training step): loss_out[b] = sum of lossrow[b * per_batch ... + per_batch) and
// violators[b][0 / 1] = sums of violrow[..][0 / 1], each in a fixed order.
struct BatchSums {
  const float* lossrow; const int* violrow; int per_batch; int batches; float* loss_out; unsigned long long* violators;
};
int row_adagrad_sorted(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits,
                       float* grad_rows, int dim, float* w0, float* g0, int64_t rows0, float* w1,
                       float* g1, int64_t rows1, float lr, hipStream_t stream, const uint32_t* long_runs = nullptr,
                       const CosBack* cos_back = nullptr, const BatchSums* sums = nullptr);

// ---- plain fp32 batched GEMM on MFMA ----------------------------------------
// C[b] (M x N, row-major, ldc) = alpha * A[b] * B[b] + beta * C[b], for b in [0, batch).
// a_kmajor = 0: A(m,k) = A[m * lda + k];  1: A(m,k) = A[k * lda + m].
// b_kmajor = 0: B(k,n) = B[n * ldb + k];  1: B(k,n) = B[k * ldb + n].
struct GemmArgs {
  const float* a; const float* b; float* c;
  int64_t stride_a, stride_b, stride_c;  // per-batch strides in floats
  int lda, ldb, ldc;
  int m, n, k;
  int batch;
  int a_kmajor, b_kmajor;
  float alpha, beta;
  // optional gather of the B operand: B[b] starts b_index[b] * b_index_stride
  // floats further (one operator matrix per relation)
  const int64_t* b_index = nullptr;
  int64_t b_index_stride = 0;
  // 1: every value of A and B is a float16 number (held as fp32): the products run on the fp16 matrix
  // instructions, still summed in fp32, and C is rounded to float16 numbers (torch.bmm on Half tensors)
  int half = 0;
};
int gemm_f32(const GemmArgs& args, hipStream_t stream);

// ---- `linear` operator with one relation per edge, over edges sorted by relation ----
// keys[n] = (relation << kbits | batch), sorted ascending; vals[n] = edge number
// e = batch * edges_per_batch + position.  Row of edge e in an array laid out
// [batches, batch_stride rows, dim]: (e / edges_per_batch) * batch_stride + e % edges_per_batch.
//   out[e] (+)= W[rel_e] in[e]     (transpose_w = false)
//   out[e] (+)= W[rel_e]^T in[e]   (transpose_w = true)
int seg_linear_apply(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, int edges_per_batch,
                     const float* in, int64_t in_batch_stride, const float* w, int dim, bool transpose_w, float* out,
                     int64_t out_batch_stride, bool accumulate, hipStream_t stream);
// For every relation and batch present: dW = sum over the run's edges of dz[e] (x) x[e]
// (dz, x: [n, dim] by edge number), then wsum += dW^2, w -= lr * dW / (sqrt(wsum) + 1e-10),
// batch after batch in ascending order.
// `num_batches`: batch numbers in the keys are below it.
// `temp` holds seg_linear_update_temp_bytes(num_relations, n, dim, num_batches) bytes.
size_t seg_linear_update_temp_bytes(int num_relations, int64_t n, int dim, int num_batches);
int seg_linear_update(const uint64_t* keys, const uint32_t* vals, int64_t n, int kbits, int num_batches,
                      const float* dz, const float* x, int dim, int num_relations, float* w, float* wsum, float lr,
                      void* temp, hipStream_t stream);

}  // namespace pbg
