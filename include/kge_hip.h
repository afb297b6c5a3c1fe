/*
 * kge_hip.h - C ABI of the MI355X (gfx950) KvsAll scoring / link-prediction kernels.
 *
 * The reference (dicee 0.3.2) is pure Python on torch and has no FFI of its own; the seam this
 * library sits behind is the tensor-level protocol of its models and evaluator.  Every entry
 * point below names the reference code whose arithmetic it replaces.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer owned by the caller unless stated otherwise.
 *   - `stream` is a hipStream_t passed as void*; work is enqueued on it and, unless noted, the
 *     call returns without waiting for it.
 *   - Return value: KGE_OK (0) or an error code; kge_last_error() gives the thread-local text.
 *     Arguments are validated on the host before anything is launched.
 *   - Entity/relation ids are int64 (what torch.LongTensor holds).  Kernels never dereference an
 *     id outside [0,N) / [0,R): such a row yields NaN scores instead of a memory fault.
 *   - Tables are row-major [rows, d].  All three storages compute on the bf16 MFMA with fp32 accumulation:
 *     KGE_F32 splits every operand into three bf16 parts and sums the six leading part products (any d);
 *     KGE_BF16 needs d % 8 == 0; KGE_I8 (per-row symmetric int8 with a float scale per row) needs d % 16 == 0.
 *     Range of the KGE_F32 split: scores are within 1e-5 of an fp64 product (relative to max(|s|, row RMS)) while
 *     the products q*e that make up a score are at least 2^-100 in magnitude and every value rounds to a finite
 *     bf16 (|x| < 3.39e38).  Below that the low-order parts underflow one after the other and the result
 *     degrades towards a bf16-grade score (2e-2); products that underflow fp32 altogether give exact zeros.  A
 *     value whose bf16 rounding is infinite gives an infinite or NaN score.
 *   - A score is `dot(Q[b], E[e]) (* scale[e]) (+ bias[b])`.  The fp32 value of the dot product
 *     is the same bit pattern in every entry point (fixed reduction order), so a rank computed
 *     by kge_rank_filtered equals the rank counted on kge_scores output exactly.
 */
#ifndef KGE_HIP_H
#define KGE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KGE_ABI_VERSION 1

enum kge_status {
  KGE_OK = 0,
  KGE_ERR_INVALID = 1,      /* bad argument (null pointer, size, model/d mismatch, k > N ...) */
  KGE_ERR_UNSUPPORTED = 2,  /* valid request this build has no kernel for */
  KGE_ERR_WORKSPACE = 3,    /* workspace missing or too small */
  KGE_ERR_HIP = 4,          /* a HIP runtime call failed */
  KGE_ERR_OVERFLOW = 5      /* top-k candidate buffers overflowed beyond recovery */
};

enum kge_model { KGE_DISTMULT = 0, KGE_COMPLEX = 1, KGE_QMULT = 2, KGE_KECI = 3, KGE_OMULT = 4, KGE_DECAL = 5 };
enum kge_dtype { KGE_F32 = 0, KGE_BF16 = 1, KGE_I8 = 2 };
enum kge_norm_kind { KGE_NORM_NONE = 0, KGE_NORM_LAYERNORM = 1, KGE_NORM_BATCHNORM1D = 2 };

/* Optional input normalisation of the gathered head / relation rows
 * (dicee/models/base_model.py:283-294, applied at :381-383).
 * LayerNorm: a = weight[d], b = bias[d].  BatchNorm1d(affine=False), eval: a = running_mean[d],
 * b = running_var[d]. */
typedef struct kge_norm_params {
  int32_t kind; /* enum kge_norm_kind */
  float eps;
  const float* h_a;
  const float* h_b;
  const float* r_a;
  const float* r_b;
} kge_norm_params;

/* Where kge_build_query_backward_norm ADDS the gradients of LayerNorm's parameters (each [d] fp32, caller
 * initialised, may be NULL): h_a / h_b = weight / bias of the head normaliser, r_a / r_b of the relation
 * normaliser.  BatchNorm1d(affine=False) has no parameters: all four NULL (or the struct itself NULL). */
typedef struct kge_norm_grads {
  float* h_a;
  float* h_b;
  float* r_a;
  float* r_b;
} kge_norm_grads;

/* torch.nn.Dropout in training mode on the looked-up rows (dicee/models/base_model.py:149-151 applied at :381-383,
 * before the normalisation layer) and, for DistMult, on h * r (dicee/models/real.py:32), with the masks given by
 * the caller: keep_* [B,d] bytes, 1 = the element is kept (and multiplied by the scale), 0 = it is zeroed; a NULL
 * mask means no dropout at that place.  scale_in = 1 / (1 - input_dropout_rate); scale_hidden the same for the rate
 * of the module behind real.py:32 (base_model.py:151 builds it with input_dropout_rate as well).  The backward
 * calls take the masks of their forward. */
typedef struct kge_dropout_params {
  const uint8_t* keep_h;
  const uint8_t* keep_r;
  const uint8_t* keep_q; /* DistMult only */
  float scale_in;
  float scale_hidden;
} kge_dropout_params;

/* Text of the last error raised on the calling thread ("" if none). */
const char* kge_last_error(void);

/* KGE_ABI_VERSION the library was built with. */
int kge_abi_version(void);

/*
 * Gather + model interaction: one query vector per (head, relation) pair so that
 * forward_k_vs_all(x) == Q @ E^T + bias[:, None].
 * Replaces BaseKGE.get_head_relation_representation (dicee/models/base_model.py:377-384) and the
 * elementwise part of k_vs_all_score of DistMult (dicee/models/real.py:32), ComplEx
 * (dicee/models/complex.py:254-263), QMult (dicee/models/quaternion.py:138-144 with
 * quaternion_normalizer :74-100 and quaternion_mul dicee/models/static_funcs.py:4-18) and Keci
 * (dicee/models/clifford.py:260-304 with apply_coefficients :105-113), and of OMult
 * (dicee/models/octonion.py:112-152 with octonion_normalizer :57-70 and octonion_mul :5-19).
 *   ent [N,d] (ent_dtype; ent_scale [N] for KGE_I8 else NULL), rel [R,d] (KGE_F32 or KGE_BF16)
 *   p,q,coeff_p[p],coeff_q[q]: Keci only.  normalize_relation: QMult only (1 when the model's
 *   relation normaliser is the identity, quaternion.py:138; the same switch for OMult's octonion
 *   normaliser, octonion.py:121, which has no epsilon: a zero relation octonion gives NaN).  norm:
 *   NULL or see above.
 *   hr [B,2] int64.  Q [B,d] fp32 out.  bias [B] fp32 out (all zero except Keci with p>=2 or q>=2).
 */
int kge_build_query(int model, int p, int q, const void* ent, int ent_dtype, const float* ent_scale,
                    const void* rel, int rel_dtype, const float* coeff_p, const float* coeff_q,
                    int normalize_relation, const kge_norm_params* norm, const int64_t* hr,
                    int64_t B, int64_t d, int64_t N, int64_t R, float* Q, float* bias, void* stream);

/*
 * The same for the head direction: one query vector per (relation, tail) pair so that
 * score(x, r, t) == dot(Q[b], E[x]) for every entity x (bias is written as zero: every term of every
 * model's triple score holds the head).  With kge_rank_filtered / kge_topk / kge_scores this replaces
 * the head half of evaluate_lp (dicee/evaluation/link_prediction.py:421-429 scores every
 * (x, r, t) triple through forward_triples: DistMult.score dicee/models/real.py:48-49, ComplEx.score
 * dicee/models/complex.py:229-238, QMult.score dicee/models/quaternion.py:102-122, Keci.score
 * dicee/models/clifford.py:448-499).  For Keci with p > 0 the per-triple value is the one the
 * model's own KvsAll path gives, forward_k_vs_all((x, r))[t]; the reference's forward_triples sums
 * two of its einsums over the batch as well (clifford.py:528-529).
 *   rt [B,2] int64 = (relation id, tail id).  norm must be NULL or KGE_NORM_NONE (a normalised head
 *   row is not a row of the table): KGE_ERR_UNSUPPORTED otherwise.  Other arguments as above.
 */
int kge_build_query_head(int model, int p, int q, const void* ent, int ent_dtype, const float* ent_scale,
                         const void* rel, int rel_dtype, const float* coeff_p, const float* coeff_q,
                         int normalize_relation, const kge_norm_params* norm, const int64_t* rt,
                         int64_t B, int64_t d, int64_t N, int64_t R, float* Q, float* bias, void* stream);

/*
 * The same two builders for DeCaL, the Clifford model with degenerate bases Cl(p, q, r): a row is
 * 1 + p + q + r parts of d / (1 + p + q + r) values, laid out [scalar | p-block | q-block | r-block] with
 * element (rho, i) of a block at rho * count + i.  Follows DeCaL.forward_k_vs_all
 * (dicee/models/clifford.py:808-899): head and relation parts are scaled by coeff_p[p] / coeff_q[q] /
 * coeff_r[r] (apply_coefficients :901-912), Q holds h0*r0 + sum hp*rp - sum hq*rq against the tails'
 * scalar part and h0*r_x + h_x*r0 against every base part, bias the six sigma sums (:859-886, each
 * only when both of its base counts are >= 2, as there).  head != 0: pairs are (relation, tail) and Q
 * is the coefficient vector of the head row, as kge_build_query_head (norm must then be none).
 * With r = 0 this is Keci.
 */
int kge_build_query_decal(int head, int p, int q, int r, const void* ent, int ent_dtype, const float* ent_scale,
                          const void* rel, int rel_dtype, const float* coeff_p, const float* coeff_q,
                          const float* coeff_r, const kge_norm_params* norm, const int64_t* pairs, int64_t B,
                          int64_t d, int64_t N, int64_t R, float* Q, float* bias, void* stream);

/*
 * kge_build_query (any of the six models: r is DeCaL's third base count, ignored otherwise) with dropout in
 * training mode; dropout NULL: the plain call.  Tail direction only.
 */
int kge_build_query_dropout(int model, int p, int q, int r, const void* ent, int ent_dtype, const float* ent_scale,
                            const void* rel, int rel_dtype, const float* coeff_p, const float* coeff_q,
                            const float* coeff_r, int normalize_relation, const kge_norm_params* norm,
                            const kge_dropout_params* dropout, const int64_t* hr, int64_t B, int64_t d, int64_t N,
                            int64_t R, float* Q, float* bias, void* stream);

/*
 * Backward of kge_build_query (tail direction, fp32 tables, no normalisation layer; with one:
 * kge_build_query_backward_norm below): given dL/dQ [B,d] and
 * dL/dbias [B] (may be NULL), ADDS dL/d(head row) into d_ent[hr[b,0], :], dL/d(relation row) into
 * d_rel[hr[b,1], :] and, for Keci / DeCaL, dL/d(coefficients) into d_coeff_p/q/r (each may be NULL).  The
 * caller zeroes the outputs or passes gradients to accumulate onto (d_ent may be the dE of
 * kge_bce_multihot_backward: the entity table receives both).  Rows shared by several pairs are combined
 * with floating-point atomics.  This is the part of `loss_batch.backward()` that autograd runs through
 * get_head_relation_representation (dicee/models/base_model.py:377-384; the embedding lookups' scatter)
 * and the models' elementwise interaction (real.py:32, complex.py:252-264, quaternion.py:136-156 incl.
 * quaternion_normalizer :74-100, octonion.py:119-144 incl. octonion_normalizer, clifford.py:105-113 and
 * :269-305, DeCaL clifford.py:808-912).  r is ignored unless model == KGE_DECAL.
 */
int kge_build_query_backward(int model, int p, int q, int r, const float* ent, const float* rel,
                             const float* coeff_p, const float* coeff_q, const float* coeff_r,
                             int normalize_relation, const int64_t* hr, int64_t B, int64_t d, int64_t N, int64_t R,
                             const float* dQ, const float* dbias, float* d_ent, float* d_rel, float* d_coeff_p,
                             float* d_coeff_q, float* d_coeff_r, void* stream);

/*
 * The same with the normalisation layer of kge_build_query between the lookups and the interaction
 * (dicee/models/base_model.py:283-294 applied at :381-383; norm as there, NULL or KGE_NORM_NONE: exactly
 * kge_build_query_backward).  LayerNorm: the gradient passes through
 * y = (x - mean(x)) / sqrt(var(x) + eps) * weight + bias per row, and dL/dweight, dL/dbias of both normalisers are
 * ADDED into dnorm's arrays (what autograd leaves in normalize_head_entity_embeddings.weight.grad etc.).
 * BatchNorm1d(affine=False) with its running statistics (eval mode): the elementwise map
 * dx = dy / sqrt(running_var + eps); batch statistics (training mode) are not part of this call.  d <= 4096.
 * dropout: NULL, or the masks of the forward (kge_build_query_dropout); with norm NULL this is the plain backward
 * through dropout alone.
 */
int kge_build_query_backward_norm(int model, int p, int q, int r, const float* ent, const float* rel,
                                  const float* coeff_p, const float* coeff_q, const float* coeff_r,
                                  int normalize_relation, const kge_norm_params* norm, const kge_norm_grads* dnorm,
                                  const kge_dropout_params* dropout, const int64_t* hr, int64_t B, int64_t d,
                                  int64_t N, int64_t R, const float* dQ, const float* dbias, float* d_ent,
                                  float* d_rel, float* d_coeff_p, float* d_coeff_q, float* d_coeff_r, void* stream);

/*
 * BatchNorm1d(affine=False) in TRAINING mode (dicee/models/base_model.py:289-294 applied at :381-383 while
 * `self.training`): the layer normalises with the statistics of the batch it is given.
 *
 * kge_batchnorm_stats: per feature, mean and biased variance over the B looked-up head rows -> h_mean / h_var [d]
 * and over the B relation rows -> r_mean / r_var [d]; pass them to kge_build_query as a KGE_NORM_BATCHNORM1D
 * layer (a = mean, b = variance) for this batch's forward.  run_* (each may be NULL): the module's running
 * statistics, updated in place as torch does in training mode, running <- (1 - momentum) * running + momentum *
 * (mean | variance * B / (B - 1)).  A pair with an id outside its table makes every statistic NaN.  B >= 2 (torch
 * raises for one value per channel).  workspace: 32 * d bytes, 8-byte aligned.  The sums over the batch are taken
 * in double precision and met with floating-point atomics: the statistics can differ in their last bit from call
 * to call (and so can everything formed with them).
 *
 * kge_build_query_backward_batchnorm: kge_build_query_backward through that layer, the statistics being functions
 * of the batch: dx = (dy - mean_B(dy) - xh * mean_B(dy * xh)) / sqrt(var + eps) with xh the normalised row.  norm
 * holds the SAME statistics the forward used.  workspace: kge_batchnorm_workspace_bytes(B, d) = 32 * d +
 * 8 * B * d bytes (the gradients at the normalised rows make a round trip: their sums over the batch are needed
 * before any gradient at a raw row can be formed), 16-byte aligned.  d <= 4096.
 * dropout (both calls): NULL, or the masks of this batch's forward; the statistics are those of the rows after
 * dropout, which is what the layer is given (base_model.py:381-383).
 */
size_t kge_batchnorm_workspace_bytes(int64_t B, int64_t d);
int kge_batchnorm_stats(const float* ent, const float* rel, const int64_t* hr, int64_t B, int64_t d, int64_t N,
                        int64_t R, const kge_dropout_params* dropout, float momentum, float* h_mean, float* h_var,
                        float* r_mean, float* r_var, float* run_h_mean, float* run_h_var, float* run_r_mean,
                        float* run_r_var, void* workspace, size_t workspace_bytes, void* stream);
int kge_build_query_backward_batchnorm(int model, int p, int q, int r, const float* ent, const float* rel,
                                       const float* coeff_p, const float* coeff_q, const float* coeff_r,
                                       int normalize_relation, const kge_norm_params* norm,
                                       const kge_dropout_params* dropout, const int64_t* hr, int64_t B, int64_t d,
                                       int64_t N, int64_t R, const float* dQ, const float* dbias,
                                       float* d_ent, float* d_rel, float* d_coeff_p, float* d_coeff_q,
                                       float* d_coeff_r, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Materialised scores S[b, e] = dot(Q[b], E[e]) (* scale[e]) (+ bias[b]); S has row stride ldS.
 * Replaces the torch.mm / einsum calls and B x N adds of real.py:32, complex.py:260-264,
 * quaternion.py:152-156, clifford.py:269-305.  For callers that need the whole matrix
 * (KGE.predict, dicee/knowledge_graph_embeddings.py:404-408; model(x) itself).
 */
int kge_scores(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
               int64_t B, int64_t d, int64_t N, float* S, int64_t ldS, void* stream);

/*
 * Score of ONE given entity per query: out[b] = dot(Q[b], E[entity[b]]) (* scale) (+ bias[b]), formed
 * with the reduction order of the contraction kernels (the same bits as S[b, entity[b]] of kge_scores).
 * With kge_build_query on the (head, relation) columns and the tails as `entity` this is
 * forward_triples for the four models (BaseKGE.forward_triples dicee/models/base_model.py:346-362
 * with DistMult.score dicee/models/real.py:48-49, ComplEx.score dicee/models/complex.py:229-238,
 * QMult.score dicee/models/quaternion.py:102-122, Keci.forward_triples dicee/models/clifford.py:501-561;
 * for Keci with p > 0 see kge_build_query_head).  entity ids outside [0, N) give NaN.
 */
int kge_triple_scores(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                      int64_t B, int64_t d, int64_t N, const int64_t* entity, float* out, void* stream);

/*
 * Scores of k given entities per query: out[b, j] = dot(Q[b], E[entity[b, j]]) (* scale) (+ bias[b]), entity
 * int64 [B,k], out fp32 [B,k]; the same bits as S[b, entity[b,j]] of kge_scores.  With kge_build_query this
 * is forward_k_vs_sample (DistMult dicee/models/real.py:38-45, ComplEx complex.py:271-289, QMult
 * quaternion.py:173-215, Keci clifford.py:363-430), the branch BaseKGE.forward takes for a tuple input
 * (base_model.py:324-326).  The reference's Keci raises NotImplementedError for p > 0 there; here every
 * model gives the column of its own KvsAll scores.  ids outside [0, N) give NaN.
 */
int kge_sample_scores(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                      int64_t B, int64_t d, int64_t N, const int64_t* entity, int64_t k, float* out, void* stream);

/*
 * Filter row of every (head, relation) pair: csr_row[b] = index of key hr[b,0]*num_relations + hr[b,1]
 * in `keys` (sorted, unique, int64 [n_rows]: the CSR's row order), or -1 if the pair has no known
 * tails.  Replaces the dict lookup `self.er_vocab[(id_e, id_r)]` of
 * dicee/evaluation/evaluator.py:493 (vocabulary built at
 * dicee/read_preprocess_save_load_kg/util.py:355-363).
 */
int kge_csr_lookup(const int64_t* hr, int64_t B, const int64_t* keys, int64_t n_rows,
                   int64_t num_relations, int64_t* csr_row, void* stream);

/*
 * Known-answer vocabulary as a CSR, built on the GPU from id triples.  For every distinct pair
 * (a, b) = (triple[col_a], triple[col_b]) the sorted, de-duplicated values triple[col_v]:
 *   keys    int64 [n_rows]     a * range_b + b, ascending (the row order kge_csr_lookup searches)
 *   row_ptr int64 [n_rows + 1]
 *   col     int32 [nnz]
 *   counts  int64 [3]          n_rows, nnz, number of triples dropped for an id outside its range
 * all device memory; keys and col need room for n entries, row_ptr for n + 1.  Columns (0, 1, 2)
 * give the (head, relation) -> tails vocabulary of get_er_vocab
 * (dicee/read_preprocess_save_load_kg/util.py:355-363; the evaluator's filter, built over
 * train + valid + test at dicee/read_preprocess_save_load_kg/preprocess.py:51-60); (1, 2, 0) gives
 * get_re_vocab (:366-374) and (0, 2, 1) get_ee_vocab (:377-385).  The reference keeps insertion
 * order and duplicates; both are irrelevant to masking, which is all these lists are used for.
 * n < 2^31; the three id ranges must fit a 62-bit packed key (KGE_ERR_UNSUPPORTED otherwise).
 */
size_t kge_csr_build_workspace_bytes(int64_t n);
int kge_csr_build(const int64_t* triples, int64_t n, int col_a, int col_b, int col_v, int64_t range_a,
                  int64_t range_b, int64_t range_v, int64_t* keys, int64_t* row_ptr, int32_t* col,
                  int64_t* counts, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Fused filtered rank: the per-row mask loop, full torch.sort and torch.where of
 * Evaluator._evaluate_entity_prediction (dicee/evaluation/evaluator.py:484-508; same loop in
 * dicee/evaluation/link_prediction.py:144-171) without writing the B x N scores.
 *   target [B]: id of the true tail.  csr_row [B]: row of the filter CSR for (h,r), or -1.
 *   row_ptr [n_rows+1] int64, col [nnz] int32: known tails per (h,r), each row sorted and
 *   without duplicates (the target may be listed; it is never filtered, evaluator.py:494-501).
 *   csr_row/row_ptr/col may be NULL together (no filter).
 * Outputs, over entities not removed by the filter:
 *   n_greater[b]     = #{e : s_e >  s_target}
 *   n_equal[b]       = #{e != target : s_e == s_target}
 *   n_equal_lower[b] = #{e <  target : s_e == s_target}
 *   target_score[b]  = s_target (+ bias[b] if bias != NULL; bias does not change ranks)
 * so the reference's rank lies in [1+n_greater, 1+n_greater+n_equal] and a stable descending
 * sort gives 1+n_greater+n_equal_lower.
 * workspace: kge_rank_workspace_bytes(B) bytes of device memory.
 */
size_t kge_rank_workspace_bytes(int64_t B);
int kge_rank_filtered(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                      int64_t B, int64_t d, int64_t N, const int64_t* target, const int64_t* csr_row,
                      const int64_t* row_ptr, const int32_t* col, int64_t n_rows,
                      int32_t* n_greater, int32_t* n_equal, int32_t* n_equal_lower,
                      float* target_score, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same evaluation with the thresholds of MANY batches formed by one launch (evaluator.py:484-508 runs batch
 * after batch; the threshold of a query, the raw score of its target, depends on nothing but its own row of Q):
 *   kge_rank_thresholds   thr[b] = raw score of target[b] for b < B (any B: a whole evaluation), target_score[b]
 *                         (+ bias), and the three counters initialised as kge_rank_filtered initialises them.
 *   kge_rank_filtered_with_thresholds   kge_rank_filtered for a batch whose slices of thr and of the counters were
 *                         prepared by that call: plan of the filter correction, main loop, correction.
 *                         one_vector_per_row != 0: the caller guarantees that queries sharing a filter row hold the
 *                         same query vector bit for bit (queries built from (head, relation) pairs and filter rows
 *                         looked up from the same pairs do), which spares the launch that checks it.
 * Results are those of kge_rank_filtered on the same batch, bit for bit.
 */
int kge_rank_thresholds(const float* Q, const float* bias, const void* E, int dtype, const float* scale, int64_t B,
                        int64_t d, int64_t N, const int64_t* target, float* thr, int32_t* n_greater, int32_t* n_equal,
                        int32_t* n_equal_lower, float* target_score, void* stream);
int kge_rank_filtered_with_thresholds(const float* Q, const void* E, int dtype, const float* scale, int64_t B, int64_t d,
                                      int64_t N, const int64_t* target, const float* thr, const int64_t* csr_row,
                                      const int64_t* row_ptr, const int32_t* col, int64_t n_rows, int one_vector_per_row,
                                      int32_t* n_greater, int32_t* n_equal, int32_t* n_equal_lower, void* workspace,
                                      size_t workspace_bytes, void* stream);

/*
 * kge_rank_filtered without a workspace argument and without any allocation.  No counterpart in the reference:
 * it exists for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  The thresholds and the plan of the filter correction live in a
 * static device array inside the library (2.1 MB per GPU, held until the process ends), so
 *   - B <= KGE_RANK_STATIC_MAX_B, KGE_ERR_WORKSPACE otherwise (split the batch, or use kge_rank_filtered);
 *   - all calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads) race;
 *   - the current device must be the one the pointers and the stream belong to (checked for Q where the runtime
 *     answers the question: KGE_ERR_INVALID on a mismatch);
 *   - the first call on a device looks the array's address up (hipGetSymbolAddress, once per device): call
 *     kge_rank_static_init() on that device, or make one ordinary call, BEFORE a stream capture begins, so
 *     that nothing but kernel launches happens inside the capture.
 * Arguments, outputs and results are those of kge_rank_filtered, bit for bit.
 * kge_rank_static_init: resolves and keeps the scratch address for the current device; allocates nothing.
 */
#define KGE_RANK_STATIC_MAX_B 65536
#define KGE_RANK_STATIC_SCRATCH_BYTES (12 * KGE_RANK_STATIC_MAX_B + 8 * (20 * 8192 + 1024) + 1024) /* 2.1 MB */
int kge_rank_static_init(void);
int kge_rank_filtered_static(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                             int64_t B, int64_t d, int64_t N, const int64_t* target, const int64_t* csr_row,
                             const int64_t* row_ptr, const int32_t* col, int64_t n_rows,
                             int32_t* n_greater, int32_t* n_equal, int32_t* n_equal_lower,
                             float* target_score, void* stream);

/*
 * Fused top-k over all entities: torch.topk(model(batch_hr), k, dim=1) of
 * KGE.predict_missing_tail_entity (dicee/knowledge_graph_embeddings.py:397-401) and, with
 * apply_sigmoid, the torch.sigmoid of KGE.predict_topk (:568), without writing B x N scores.
 *   out_scores [B,k] fp32 descending, out_idx [B,k] int64; equal scores are ordered by
 *   ascending entity id.  Requires 1 <= k <= min(N, 1024).
 *   The order is that of the scores before the per-query bias is added (and before the sigmoid): two
 *   entities whose scores become equal only through the rounding of score + bias, or of the sigmoid, keep
 *   the order of their unbiased scores.
 * This call (and kge_topk_prepared) synchronises `stream`: once before returning to read back one overflow
 * counter, and once more per repair scan when a candidate buffer overflowed (at most 16 scans; still overflowing
 * after those: KGE_ERR_OVERFLOW).  Neither can be captured into a HIP graph.
 */
size_t kge_topk_workspace_bytes(int64_t B, int64_t N, int64_t k);
int kge_topk(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
             int64_t B, int64_t d, int64_t N, int64_t k, float* out_scores, int64_t* out_idx,
             int apply_sigmoid, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same top-k over a table whose derived form for the scan is made once and kept by the caller, the way the
 * int8 table itself is made once from the model's parameters (dicee keeps its tables as nn.Embedding weights and has
 * no quantised storage: there is no reference line for this; the results are those of kge_topk, bit for bit).
 * Per-row int8 tables with d = 128 have such a form (the rows written again with one scale per 32-row tile plus a
 * 32-byte record per 64 rows: kge_topk derives it in its workspace on every call, 2.6 GB of traffic at N = 10M);
 * kge_topk_prepared_bytes returns 0 for every other storage and kge_topk_prepare / kge_topk_prepared then return
 * KGE_ERR_UNSUPPORTED.  The prepared buffer must be rebuilt whenever E or scale change; it is only read by
 * kge_topk_prepared, so calls on several streams may share it.
 */
size_t kge_topk_prepared_bytes(int dtype, int64_t d, int64_t N);
int kge_topk_prepare(const void* E, int dtype, const float* scale, int64_t d, int64_t N, void* prepared,
                     size_t prepared_bytes, void* stream);
size_t kge_topk_prepared_workspace_bytes(int64_t B, int64_t N, int64_t k);
int kge_topk_prepared(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                      int64_t B, int64_t d, int64_t N, int64_t k, float* out_scores, int64_t* out_idx,
                      int apply_sigmoid, const void* prepared, size_t prepared_bytes, void* workspace,
                      size_t workspace_bytes, void* stream);

/*
 * Smallest and largest score of every query over all N entities: out_min[b] = min_e S[b, e],
 * out_max[b] = max_e S[b, e] (bias included), without writing S.  Replaces the `preds_raw.min(dim=1)` /
 * `.max(dim=1)` pair of the per-sample min-max normalisation in
 * evaluate_ensemble_link_prediction_performance (dicee/evaluation/ensemble.py:93-96); with the
 * per-model factors w_m / (max_m - min_m + 1e-8) folded into the query vectors the weighted average of
 * the normalised scores of M models is ONE contraction against the column-wise concatenation of their
 * entity tables, ranked by kge_rank_filtered.
 */
int kge_row_minmax(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                   int64_t B, int64_t d, int64_t N, float* out_min, float* out_max, void* stream);

/*
 * Fused KvsAll BCE: mean over B*N of BCEWithLogits(s, y) with y the multi-hot of the CSR row
 * (KvsAll.__getitem__, dicee/dataset_classes.py:354-361, incl. its label smoothing
 * y*(1-eps) + 1/N when eps != 0) and the default loss of dicee/models/base_model.py:138, as
 * used by training_step (:25-46).  Neither the dense target nor the logits are materialised.
 *   csr_row [B] (-1 = no positives), row_ptr, col as in kge_rank_filtered.  loss [1] fp32 out.
 * workspace: kge_bce_workspace_bytes() bytes.
 */
size_t kge_bce_workspace_bytes(void);
int kge_bce_multihot(const float* Q, const float* bias, const void* E, int dtype, const float* scale,
                     int64_t B, int64_t d, int64_t N, const int64_t* csr_row, const int64_t* row_ptr,
                     const int32_t* col, int64_t n_rows, float label_smoothing, float* loss,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward of the same step: with S = Q E^T + bias and the mean BCE loss L of kge_bce_multihot,
 *   g    = grad_out * (sigmoid(S) - y') / (B * N)          (y' the smoothed multi-hot target)
 *   dQ   [B,d] = g E          dE [N,d] = g^T Q          dbias [B] = row sums of g (may be NULL)
 * which is what autograd computes behind `loss_batch.backward()` for the KvsAll training step
 * (dicee/models/base_model.py:25-46 with the torch.nn.BCEWithLogitsLoss of :138; the two products are
 * the backward of the torch.mm / einsum of the model's k_vs_all_score).  `loss` may be NULL; otherwise
 * it receives L as kge_bce_multihot gives it.  dQ, dbias and dE are overwritten.  fp32 tables only
 * (KGE_ERR_UNSUPPORTED otherwise), N <= 2^24.  g is formed once by the fused contraction and kept in
 * the workspace as [B,N] for the two gradient contractions, which run on the same three-part bf16 MFMA
 * kernel as the scores and read g, E and Q where they lie (K-major operands); the workspace is about
 * 4 * B * N bytes.  When d is not a multiple of 4, g is kept in both layouts and E and Q are transposed
 * into the workspace as well (about 8 * B * N bytes).  dQ and dE are
 * reproducible bit for bit from call to call; dbias is summed with floating-point atomics (order varies).
 */
size_t kge_bce_backward_workspace_bytes(int64_t B, int64_t d, int64_t N);
int kge_bce_multihot_backward(const float* Q, const float* bias, const void* E, int dtype, int64_t B, int64_t d,
                              int64_t N, const int64_t* csr_row, const int64_t* row_ptr, const int32_t* col,
                              int64_t n_rows, float label_smoothing, float grad_out, float* loss, float* dQ,
                              float* dbias, float* dE, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Measurement aid; no counterpart in the reference.  Between kge_profile_begin() and
 * kge_profile_end(), every launch of a contraction main loop (the MFMA kernel inside kge_scores,
 * kge_rank_filtered, kge_topk and kge_bce_multihot) is bracketed by two HIP events recorded on the
 * stream it is launched on.  kge_profile_end waits for those events and returns the summed
 * kernel time in milliseconds and the number of launches.  Process-wide; not for concurrent use.
 */
int kge_profile_begin(void);
int kge_profile_end(double* total_ms, int64_t* launches);
/* Name (kernel and template arguments) of the main loop most recently bracketed while profiling was on, as the
 * library itself dispatched it; "" before the first.  The pointer stays valid until the next call. */
const char* kge_profile_kernel(void);

/*
 * Measurement aids; no counterpart in the reference and no part of any product path.  They time stripped-down
 * forms of the filtered-rank main loop of bf16 tables with d == 128 for about `seconds` (at most 30) on `stream`
 * and return the rate of the second half of the launches in TFLOP/s (2 * 32 * 32 * 16 flop per MFMA issued) and
 * the average launch duration, so that a benchmark run can show from one box and one process what the MFMA unit
 * sustains alone and what each part of the main loop costs:
 *   kge_probe_mfma   256 workgroups of 8 waves (two waves per SIMD) issue the main loop's tile statement on random
 *                    bf16 operands held in registers: count = 1 adds the rank count between the MFMAs (5 VALU
 *                    instructions per MFMA), reads = 1 re-reads the entity fragments from LDS under every tile as
 *                    the main loop does; no global memory traffic, no barriers.
 *   kge_probe_walk   the main loop itself over the caller's bf16 table E [N,128] and queries Q [B,128] (fp32):
 *                    global -> LDS stages, barriers, fragment reads and MFMAs, without the count.
 *   kge_probe_i8_scan  the top-k scan of per-row int8 tables with d == 128 (the integer filter) over a table's prepared
 *                    form (kge_topk_prepare; 256-byte aligned, as Q [B,128]) with every threshold at +inf: no tile
 *                    passes the bound, so the launch is the scan's hot loop alone (int8 MFMAs, the test of every tile,
 *                    the walk) without the parking and collecting of candidates; rate in tera-operations per second
 *                    (2 * 128 per entity score).
 * All three allocate (and free) a little device memory (kge_probe_i8_scan: 212 bytes per query) and synchronise the
 * stream.
 */
int kge_probe_mfma(int count, int reads, double seconds, double* tflops, double* ms_per_launch, void* stream);
int kge_probe_walk(const float* Q, const void* E, int64_t B, int64_t N, double seconds, double* tflops,
                   double* ms_per_launch, void* stream);
int kge_probe_i8_scan(const float* Q, const void* prepared, int64_t B, int64_t N, double seconds, double* tops,
                      double* ms_per_launch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KGE_HIP_H */
