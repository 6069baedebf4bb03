/*
 * pbg_hip.h -- C ABI of the MI355X (gfx950) implementation of the
 * PyTorch-BigGraph per-bucket training step.
 *
 * The reference has no C ABI of its own: the path is Python over PyTorch ops,
 * plus one pybind11 module (`_C`, torchbiggraph/util.cpp:425-460).  Each entry
 * point below names the reference interface it replaces.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its comment says "host";
 *   - all floats are fp32, all indices int64, tensors are row-major contiguous;
 *   - the caller owns every buffer, including workspaces (query the *_bytes
 *     function, allocate, pass in); the library never allocates device memory;
 *   - work is enqueued on `stream` (a hipStream_t) and the call returns without
 *     synchronising.  pbg_train_step may also run its key sort (and behind it
 *     the parameter kernels of a translation operator) on one more stream that
 *     the library creates per device on first use (default priority): it is
 *     forked from `stream` and joined back into it with events inside the
 *     call, so the caller sees the step's work as if it were all on `stream`
 *     (a HIP graph capture records the forks and the joins);
 *   - return value: PBG_OK or a negative pbg_status; pbg_last_error() gives the
 *     message of the last failure on the calling thread.
 */
#ifndef PBG_HIP_H
#define PBG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pbg_stream_t; /* hipStream_t */

typedef enum pbg_status {
  PBG_OK = 0,
  PBG_ERR_INVALID = -1,     /* bad argument (shape, enum, null pointer) */
  PBG_ERR_WORKSPACE = -2,   /* workspace missing or too small */
  PBG_ERR_LAUNCH = -3,      /* HIP reported an error at launch */
  PBG_ERR_UNSUPPORTED = -4  /* a combination this build does not implement */
} pbg_status;

/* Names follow the reference's registries: OPERATORS / DYNAMIC_OPERATORS
 * (operators.py:46,194), COMPARATORS (model.py:156), LOSS_FUNCTIONS
 * (losses.py:50). */
typedef enum pbg_operator {
  PBG_OP_NONE = 0,
  PBG_OP_DIAGONAL = 1,
  PBG_OP_TRANSLATION = 2,
  PBG_OP_LINEAR = 3,
  PBG_OP_COMPLEX_DIAGONAL = 4,
  PBG_OP_AFFINE = 5 /* linear_transformation, then translation (operators.py:102-115, 272-293) */
} pbg_operator;
typedef enum pbg_comparator { PBG_CMP_DOT = 0, PBG_CMP_COS = 1, PBG_CMP_L2 = 2, PBG_CMP_SQUARED_L2 = 3 } pbg_comparator;
typedef enum pbg_loss { PBG_LOSS_RANKING = 0, PBG_LOSS_LOGISTIC = 1, PBG_LOSS_SOFTMAX = 2 } pbg_loss;

int pbg_version(void);
const char* pbg_last_error(void);

/* ------------------------------------------------------------------------
 * Row gather.  Replaces SimpleEmbedding.get = F.embedding(idx, W, sparse=True)
 * (model.py:60-61) and the gather half of sample_entities (model.py:70-75).
 * out[i, :] = table[idx[i], :], bit-exact.  An index outside [0, num_rows)
 * writes a zero row and sets *oob_flag (if not null) to 1.
 * ---------------------------------------------------------------------- */
int pbg_gather_rows(const float* table, int64_t num_rows, int32_t dim, const int64_t* idx, int64_t n,
                    float* out, int32_t* oob_flag, pbg_stream_t stream);

/* What F.embedding(max_norm=...) does to the table before it reads it
 * (SimpleEmbedding with max_norm, model.py:52-61; torch.embedding_renorm_): every
 * row named in idx whose 2-norm exceeds max_norm is scaled, in the table, by
 * max_norm / (norm + 1e-7).  Indices outside [0, num_rows) are skipped.  The
 * workspace holds pbg_embedding_renorm_workspace_bytes(n, dim) bytes. */
size_t pbg_embedding_renorm_workspace_bytes(int64_t n, int32_t dim);
int pbg_embedding_renorm(float* table, int64_t num_rows, int32_t dim, const int64_t* idx, int64_t n,
                         float max_norm, void* workspace, size_t workspace_bytes, pbg_stream_t stream);

/* ------------------------------------------------------------------------
 * RowAdagrad.  Replaces RowAdagrad.step (row_adagrad.py:48-109).
 * Sparse branch (:80-96): `idx[n]` / `grad_rows[n, dim]` are the uncoalesced
 * COO gradient; duplicates are summed (sort by index, segmented sum, formed in
 * place: grad_rows is CLOBBERED) before
 *   delta = mean_d(g^2); G[r] += delta; W[r] -= lr * g / (sqrt(G_old + delta) + 1e-10).
 * Dense branch (:97-107): `grad[num_rows, dim]`.
 * ---------------------------------------------------------------------- */
size_t pbg_row_adagrad_sparse_workspace_bytes(int64_t n);
int pbg_row_adagrad_sparse(float* weight, float* state_sum, int64_t num_rows, int32_t dim,
                           const int64_t* idx, float* grad_rows, int64_t n, float lr,
                           void* workspace, size_t workspace_bytes, pbg_stream_t stream);
/* pbg_row_adagrad_sparse without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid it).  It has no counterpart in the reference.  The
 * sort's keys, values and counters live in a device array built into the library
 * (32 MiB per GPU, held until the process ends): n is limited to
 * pbg_row_adagrad_sparse_static_max_indices() = 2^20 indices and a larger n
 * returns PBG_ERR_WORKSPACE.  The call allocates nothing; the first call on a
 * device looks the array's address up (make it outside a graph capture).  All
 * calls on one GPU share the array: calls that overlap on one GPU (two streams,
 * two threads) race.  Results are bit-identical to pbg_row_adagrad_sparse. */
int64_t pbg_row_adagrad_sparse_static_max_indices(void);
int pbg_row_adagrad_sparse_static(float* weight, float* state_sum, int64_t num_rows, int32_t dim,
                                  const int64_t* idx, float* grad_rows, int64_t n, float lr,
                                  pbg_stream_t stream);
int pbg_row_adagrad_dense(float* weight, float* state_sum, int64_t num_rows, int32_t dim,
                          const float* grad, float lr, pbg_stream_t stream);

/* AsyncAdagrad dense step for operator parameters (async_adagrad.py:75-85,
 * lr_decay = 0): G += g^2; p -= lr * g / (sqrt(G) + eps). */
int pbg_async_adagrad_dense(float* param, float* state_sum, const float* grad, int64_t numel,
                            float lr, float eps, pbg_stream_t stream);

/* ------------------------------------------------------------------------
 * Batched fp32 matrix product on the matrix cores.  Replaces the torch.bmm /
 * torch.baddbmm call sites of the comparators (model.py:179-180,209-210,234)
 * and the matmul of the linear operator (operators.py:94-99).
 *   C[i] (m x n, row-major, ldc) = alpha * A[i] * B[i] + beta * C[i],  i < batch
 *   a_kmajor = 0: A(r, x) = a[r * lda + x];  1: A(r, x) = a[x * lda + r]
 *   b_kmajor = 0: B(x, j) = b[j * ldb + x];  1: B(x, j) = b[x * ldb + j]
 * stride_* are the distances between consecutive matrices, in floats.
 * ---------------------------------------------------------------------- */
int pbg_gemm_f32(const float* a, const float* b, float* c, int32_t batch, int32_t m, int32_t n, int32_t k,
                 int32_t lda, int32_t ldb, int32_t ldc, int64_t stride_a, int64_t stride_b,
                 int64_t stride_c, int32_t a_kmajor, int32_t b_kmajor, float alpha, float beta,
                 pbg_stream_t stream);
/* The same product for operands whose every value is a float16 number (held as fp32), as torch.bmm
 * computes it on Half tensors: the comparators' call sites under config.half_precision
 * (model.py:504-505 then :179-180,209-210).  Runs on the fp16 matrix instructions, sums in fp32,
 * and stores C rounded to float16 numbers (still as fp32). */
int pbg_gemm_f16(const float* a, const float* b, float* c, int32_t batch, int32_t m, int32_t n, int32_t k,
                 int32_t lda, int32_t ldb, int32_t ldc, int64_t stride_a, int64_t stride_b,
                 int64_t stride_c, int32_t a_kmajor, int32_t b_kmajor, float alpha, float beta,
                 pbg_stream_t stream);

/* ------------------------------------------------------------------------
 * The training step.  Replaces Trainer._process_one_batch (train_cpu.py:86-112):
 * MultiRelationEmbedder.forward (model.py:624-856), calc_loss
 * (batching.py:139-150), the Stats counters, autograd backward, AsyncAdagrad on
 * the operator parameters and RowAdagrad on the embedding tables.
 *
 * One call processes `num_workers` batches of `batch_size` edges each in
 * lock-step: every batch reads the tables as they are on entry, then the
 * updates of batch 0, 1, ... are applied in that order.  num_workers = 1 is the
 * reference's single-process sequence; num_workers = K is K HOGWILD workers
 * (train_cpu.py:849-884) in the one interleaving that is deterministic.
 * ---------------------------------------------------------------------- */
typedef struct pbg_step_desc {
  int32_t dim;              /* D, 1 .. 4096 (config.py:142-150 sets no limit; the per-row kernels keep a row in one wave's registers) */
  int32_t num_workers;      /* K >= 1 */
  int32_t batch_size;       /* B >= 1, edges per batch */
  int32_t num_batch_negs;   /* config.num_batch_negs; 0 selects uniform-only negatives (model.py:651-656) */
  int32_t num_uniform_negs; /* config.num_uniform_negs (U) */
  int32_t disable_lhs_negs; /* config.disable_lhs_negs */
  int32_t disable_rhs_negs; /* config.disable_rhs_negs */
  int32_t op;               /* pbg_operator */
  int32_t dynamic;          /* 0: one relation per batch, operator on rhs (model.py:666-703);
                               1: relation per edge, operators on both sides (model.py:705-758) */
  int32_t num_relations;    /* leading axis of the operator parameters and of relation_weights */
  int32_t comparator;       /* pbg_comparator */
  int32_t loss;             /* pbg_loss */
  float margin;             /* ranking loss margin (config.margin) */
  float lr;                 /* config.lr, RowAdagrad */
  float relation_lr;        /* config.relation_lr or config.lr, AsyncAdagrad (train_cpu.py:224-228) */
  int32_t shared_table;     /* 1: lhs and rhs index the same table (w_rhs == w_lhs, g_rhs == g_lhs) */
  int64_t num_lhs_rows;     /* rows of w_lhs */
  int64_t num_rhs_rows;     /* rows of w_rhs */
  /* config.regularization_coef with config.regularizer = "N3" (the one registered,
   * regularizers.py:51-97, model.py:845-854): the step minimises loss + reg
   * (train_cpu.py:102-103).  0 = no regularizer.  Not defined for `linear`
   * (operators.py:40). */
  float regularization_coef;
  float max_norm;           /* > 0: F.embedding(max_norm=...) (model.py:61,90-96): the rows a call looks up are
                             * first renormalised IN THE TABLE to at most this 2-norm (pbg_model_forward
                             * included, as in the reference); 0 = off */
  int32_t bias;             /* config.bias: BiasedComparator around `comparator` (model.py:306-344,902-903): a
                             * row's first coordinate stays out of the comparator and is added to its scores */
  int32_t all_negs;         /* RelationSchema.all_negs (config.py:123-131; model.py:648-650,582-618): one chunk of all
                             * B positives, negatives = EVERY entity of the side's type in table order (lhs_neg
                             * is [K, B, num_lhs_rows]), the edge's own entity masked; num_batch_negs,
                             * num_uniform_negs and the uniform index arrays are ignored */
  int32_t half_precision;   /* config.half_precision (config.py:496-498; model.py:504-505,827-829): every embedding
                             * is cast to float16 once it is prepared for the comparator, so the negatives' scores
                             * are float16 products and the prepared embeddings' gradients float16 tensors; positive
                             * scores, losses, operators and both optimizers stay fp32.  Tables, scores and gradients
                             * are still fp32 arrays here (holding float16 numbers where the reference holds Half
                             * tensors); the products run on the fp16 matrix instructions (fused and staged route).  dot and cos comparators,
                             * without bias and regularizer (anything else: PBG_ERR_UNSUPPORTED) */
} pbg_step_desc;

typedef struct pbg_step_buffers {
  float* w_lhs;               /* [num_lhs_rows, D] */
  float* g_lhs;               /* [num_lhs_rows]  RowAdagrad state["sum"] */
  float* w_rhs;               /* [num_rhs_rows, D] */
  float* g_rhs;               /* [num_rhs_rows] */
  /* Entity and relation ids are NOT validated on the device: an id outside
   * [0, num_*_rows) (or [0, num_relations)) is clamped to the nearest valid one, so the
   * step reads and updates row 0 or the last row instead, where the reference's
   * F.embedding raises IndexError (model.py:60-61).  A caller that cannot vouch for
   * its ids checks them first (pytorch_biggraph_amd.native.StepRunner.train(check_ids=True)
   * does, with one device reduction per array). */
  const int64_t* lhs;         /* [K, B] */
  const int64_t* rhs;         /* [K, B] */
  const int64_t* rel;         /* standard: [K]; dynamic: [K, B] */
  const int64_t* uniform_lhs; /* [K, C, U] entity indices (model.py:70-75), null if unused or sample_uniform */
  const int64_t* uniform_rhs; /* [K, C, U] */
  const float* edge_weight;   /* [K, B] or null (EdgeList.weight, edgelist.py:51-95) */
  const float* relation_weights; /* [num_relations] (batching.py:144-148) */
  /* Operator parameters, leading axis [num_relations]; p0 = diagonal |
   * translation | linear_transformation | real, p1 = imag | translation of
   * `affine`; s0/s1 = AsyncAdagrad
   * state["sum"] of the same shape.  lhs_* only in dynamic mode. */
  float* rhs_op_p0; float* rhs_op_p1; float* rhs_op_s0; float* rhs_op_s1;
  float* lhs_op_p0; float* lhs_op_p1; float* lhs_op_s0; float* lhs_op_s1;
  float* loss_out;            /* [K] loss of each batch (Stats.loss) */
  int64_t* violators_out;     /* [K, 2] violators_lhs, violators_rhs */
  void* workspace;
  size_t workspace_bytes;
  /* sample_uniform != 0: uniform_lhs / uniform_rhs are null and the step draws the
   * uniform negatives itself (SimpleEmbedding.sample_entities, model.py:70-75):
   * negative (k, chunk, u) of side s is row
   * pbg_sample_uniform_negatives(uniform_seed, s, num_rows)[(k * C + chunk) * U + u].
   * Pass a fresh seed per call. */
  int32_t sample_uniform;
  uint64_t uniform_seed;
  float* reg_out;             /* [K] regularizer value of each batch (Stats.reg, train_cpu.py:97), or null */
  /* config.global_emb (model.py:433-441,486-492): the learned vector [D] of each side's
   * entity type, added to every gathered row of that side before the operator, and
   * its AsyncAdagrad state["sum"] [D] (step size relation_lr: it is a parameter of the
   * model optimizer).  Null = disabled.  When both sides have the same entity type
   * pass the same pointers twice: the two sides' gradients are summed into one step.
   * Standard relations only (model.py:488-489). */
  float* lhs_global; float* rhs_global; float* lhs_global_sum; float* rhs_global_sum;
} pbg_step_buffers;

/* sizeof(pbg_step_desc) / sizeof(pbg_step_buffers) as this library was compiled:
 * a binding checks its own struct layout against them. */
size_t pbg_sizeof_step_desc(void);
size_t pbg_sizeof_step_buffers(void);

/* The rows the step draws for side `side` (0 lhs, 1 rhs) under `seed`:
 * out[i] = Philox4x32-10(key = seed, counter = i, stream = side) mod num_rows, i < count.
 * Replaces the torch.randint of sample_entities (model.py:72); lets a caller (or a
 * test) see the negatives of a call that drew them itself. */
int pbg_sample_uniform_negatives(uint64_t seed, int32_t side, int64_t num_rows, int64_t count, int64_t* out,
                                 pbg_stream_t stream);

size_t pbg_train_step_workspace_bytes(const pbg_step_desc* desc);
int pbg_train_step(const pbg_step_desc* desc, const pbg_step_buffers* bufs, pbg_stream_t stream);

/* The same step with HIP events recorded on `stream` between its stages; waits
 * for the step to finish and writes the pbg_train_step_num_stages() stage
 * durations in milliseconds to stage_ms (HOST memory).  Stages: 0 gather +
 * element-wise operator + prepare, 1 linear operator, 2 score GEMMs, 3 loss,
 * 4 dN GEMMs, 5 dA GEMMs, 6 chain rule to raw rows, 7 operator parameters,
 * 8 key sort, 9 RowAdagrad update (whose first launch also sums the batches'
 * losses and violator counts into loss_out / violators_out).  When the step runs its key sort on the
 * library's own stream beside the chunk kernel (see Conventions), that time
 * is hidden inside stage 0 and stage 8 reads as about zero.  No counterpart in
 * the reference (it logs wall-clock per bucket, train_cpu.py:696-703). */
int pbg_train_step_num_stages(void);
/* 1 when pbg_train_step runs this configuration's chain from the gather to the
 * raw-row gradients as ONE kernel with a chunk's operands resident in LDS (then
 * stage 0 is that kernel and stages 1-6 are empty), 0 when it runs the staged
 * kernels.  No counterpart in the reference. */
int pbg_train_step_is_fused(const pbg_step_desc* desc);
/* Which kernels pbg_train_step runs for this configuration (-1: the descriptor
 * is invalid): the staged chain, the one fused kernel above, or the streaming
 * route -- a chunk's positives resident in LDS, its negatives gathered raw from
 * the table and streamed past them in tiles, twice (scores and loss statistics,
 * then both gradient products), with stage 0 the per-edge preparation, stage 2
 * that kernel and stage 6 the per-edge finish.  A call whose buffers carry global
 * embeddings runs the staged chain where this says streaming.  No counterpart in
 * the reference. */
#define PBG_ROUTE_STAGED 0
#define PBG_ROUTE_FUSED 1
#define PBG_ROUTE_STREAM 2
int pbg_train_step_route(const pbg_step_desc* desc);
int pbg_train_step_profile(const pbg_step_desc* desc, const pbg_step_buffers* bufs, pbg_stream_t stream,
                           float* stage_ms);

/* MultiRelationEmbedder.forward alone (model.py:624-762): scores only, tables
 * untouched.  lhs_pos/rhs_pos: [K, B]; lhs_neg: [K, B, Nl]; rhs_neg: [K, B, Nr]
 * with N = (num_batch_negs ? min(num_batch_negs, B) : 0) + U, or 0 when that
 * side is disabled; masked entries hold -1e9. */
int pbg_model_forward(const pbg_step_desc* desc, const pbg_step_buffers* bufs, float* lhs_pos,
                      float* rhs_pos, float* lhs_neg, float* rhs_neg, pbg_stream_t stream);

/* RankingEvaluator._process_one_batch (eval.py:43-81) without the [B, N] score
 * matrices: the same forward as pbg_model_forward, then per edge e of the call
 * (K * batch_size of them) lhs_pos[e], rhs_pos[e], the ranks lhs_rank[e] /
 * rhs_rank[e] = 1 + the number of that side's negatives scoring at least as
 * high as the positive (entries the model masks to -1e9 take part with that
 * value, as they do in the reference's matrices; 0 for a side without
 * negatives, which the evaluator skips), and loss_edge[e] = relation weight x
 * edge weight x (lhs loss + rhs loss) of the edge under desc->loss / margin
 * (batching.py:139-150; sum over the edges = the batch's loss).  With
 * auc_samples > 0 also compute_randomized_auc's count (util.py:420-428):
 * auc_hits[side] (device, two int64) = how many of auc_samples random
 * (positive, negative-entry) pairs of the call have positive > negative, drawn
 * with Philox4x32-10 from auc_seed. */
int pbg_model_ranks(const pbg_step_desc* desc, const pbg_step_buffers* bufs, float* lhs_pos, float* rhs_pos,
                    int64_t* lhs_rank, int64_t* rhs_rank, float* loss_edge, int64_t auc_samples, uint64_t auc_seed,
                    int64_t* auc_hits, pbg_stream_t stream);

/* ------------------------------------------------------------------------
 * Plugin-level entry points: one operator / comparator / loss at a time, forward
 * and backward, for code that calls the plugin classes directly (the reference's
 * unit tests do).  The training step above does not go through these.
 * ---------------------------------------------------------------------- */
/* AbstractOperator.forward / AbstractDynamicOperator.forward (operators.py:49-157,
 * 197-338): y[i] = op(x[i]).  rel == NULL: one operator, parameters p0 (diagonal
 * | translation | linear_transformation | real) and p1 (imag | translation of
 * `affine`).  rel != NULL:
 * rel[n_rows] selects one of num_ops parameter rows per input row. */
int pbg_operator_forward(int32_t op, int32_t dim, int64_t n_rows, const float* x, const float* p0,
                         const float* p1, const int64_t* rel, int64_t num_ops, float* y, pbg_stream_t stream);
/* Its gradient: dx is written; dp0 / dp1 are ACCUMULATED into (zero them first). */
int pbg_operator_backward(int32_t op, int32_t dim, int64_t n_rows, const float* x, const float* dy,
                          const float* p0, const float* p1, const int64_t* rel, int64_t num_ops, float* dx,
                          float* dp0, float* dp1, pbg_stream_t stream);

/* AbstractComparator.prepare (model.py:161-162,187-192,251-252): y = x for dot
 * and l2, x / ||x|| for cos.  aux[n] (optional) receives 1/||x|| (cos) or
 * ||x||^2 (l2). */
int pbg_comparator_prepare(int32_t cmp, int32_t dim, int64_t n, const float* x, float* y, float* aux,
                           pbg_stream_t stream);
int pbg_comparator_prepare_backward(int32_t cmp, int32_t dim, int64_t n, const float* dy, const float* y,
                                    const float* aux, float* dx, pbg_stream_t stream);

/* AbstractComparator.forward (model.py:164-182,194-212,254-278):
 * lhs_pos, rhs_pos [chunks, p, dim]; lhs_neg [chunks, ln, dim]; rhs_neg [chunks, rn, dim]
 * -> pos [chunks, p], lhs_neg_scores [chunks, p, ln] = rhs_pos x lhs_neg,
 *    rhs_neg_scores [chunks, p, rn] = lhs_pos x rhs_neg.
 * The workspace is only needed by l2. */
size_t pbg_comparator_workspace_bytes(int32_t chunks, int32_t p, int32_t ln, int32_t rn);
int pbg_comparator_forward(int32_t cmp, int32_t chunks, int32_t p, int32_t ln, int32_t rn, int32_t dim,
                           const float* lhs_pos, const float* rhs_pos, const float* lhs_neg,
                           const float* rhs_neg, float* pos, float* lhs_neg_scores, float* rhs_neg_scores,
                           void* workspace, size_t workspace_bytes, pbg_stream_t stream);
int pbg_comparator_backward(int32_t cmp, int32_t chunks, int32_t p, int32_t ln, int32_t rn, int32_t dim,
                            const float* lhs_pos, const float* rhs_pos, const float* lhs_neg,
                            const float* rhs_neg, const float* pos, const float* lhs_neg_scores,
                            const float* rhs_neg_scores, const float* dpos, const float* dlhs_neg_scores,
                            const float* drhs_neg_scores, float* dlhs_pos, float* drhs_pos, float* dlhs_neg,
                            float* drhs_neg, void* workspace, size_t workspace_bytes, pbg_stream_t stream);

/* AbstractLossFunction.forward (losses.py:53-161): pos [num_pos], neg [num_pos,
 * num_neg], weight [num_pos] or NULL -> *out (device scalar).  row_workspace
 * holds num_pos floats. */
int pbg_loss_forward(int32_t loss, float margin, int64_t num_pos, int32_t num_neg, const float* pos,
                     const float* neg, const float* weight, float* out, float* row_workspace,
                     pbg_stream_t stream);
/* Its gradient, scaled by *upstream (device scalar). */
int pbg_loss_backward(int32_t loss, float margin, int64_t num_pos, int32_t num_neg, const float* pos,
                      const float* neg, const float* weight, const float* upstream, float* dpos,
                      float* dneg, pbg_stream_t stream);

/* ------------------------------------------------------------------------
 * Permutation helpers.  Replace the `_C` module (util.cpp:425-460).
 * ---------------------------------------------------------------------- */
/* _C.reverse_permutation (util.cpp:104-125): out[perm[i]] = i. */
int pbg_reverse_permutation(const int64_t* perm, int64_t n, int64_t* out, pbg_stream_t stream);

/* _C.shuffle (util.cpp:127-220): rows[perm[i]] <- rows[i], result left in
 * `rows`.  `scratch` holds n * row_bytes bytes.  row_bytes must be a multiple
 * of 4.  An out-of-range perm entry sets *oob_flag and drops that row. */
int pbg_shuffle_rows(void* rows, int64_t n, int64_t row_bytes, const int64_t* perm, void* scratch,
                     int32_t* oob_flag, pbg_stream_t stream);

/* The same move out of place: out[perm[i]] <- rows[i], `rows` untouched, `out`
 * (n * row_bytes bytes) not overlapping it.  For a caller that holds two
 * buffers and swaps them, so that the copy back of the in-place form (half of
 * its traffic) is not paid.  The reference only has the in-place form
 * (util.cpp:127-220, whose cycle-following needs no second buffer on a CPU). */
int pbg_shuffle_rows_out(const void* rows, int64_t n, int64_t row_bytes, const int64_t* perm, void* out,
                         int32_t* oob_flag, pbg_stream_t stream);

/* _C.randperm (util.cpp:14-102): a random permutation of [0, n).  The
 * reference's bit pattern depends on its thread count; only the contract is
 * kept.  Deterministic in (n, seed).  out[i] is a keyed bijection of i (a
 * Feistel network on the bits of n - 1, cycle-walked into [0, n)): no sort and
 * no workspace -- pbg_randperm_workspace_bytes returns 0 and the workspace
 * arguments are ignored (kept so that existing callers link). */
size_t pbg_randperm_workspace_bytes(int64_t n);
int pbg_randperm(int64_t n, uint64_t seed, int64_t* out, void* workspace, size_t workspace_bytes,
                 pbg_stream_t stream);

/* _C.sub_bucket (util.cpp:260-423): stable partition of a bucket's edges into
 * num_lhs_parts x num_rhs_parts sub-buckets.  lhs_perm_ptrs / rhs_perm_ptrs:
 * device arrays of num_relations device pointers to the per-relation entity
 * permutations; *_part_sizes: device arrays [num_relations] of
 * ceil(entity_count / parts).  offsets_out[parts_l * parts_r + 1] (device)
 * receives the start of every sub-bucket in the outputs. */
size_t pbg_sub_bucket_workspace_bytes(int64_t n);
int pbg_sub_bucket(const int64_t* lhs_in, const int64_t* rhs_in, const int64_t* rel_in, int64_t n,
                   int32_t num_relations, const int64_t* const* lhs_perm_ptrs,
                   const int64_t* const* rhs_perm_ptrs, const int64_t* lhs_part_sizes,
                   const int64_t* rhs_part_sizes, int32_t num_lhs_parts, int32_t num_rhs_parts,
                   int32_t dynamic_relations, int64_t* lhs_out, int64_t* rhs_out, int64_t* rel_out,
                   int64_t* offsets_out, int32_t* error_flag, void* workspace, size_t workspace_bytes,
                   pbg_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PBG_HIP_H */
