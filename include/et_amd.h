/*
 * et_amd.h — C ABI of the MI355X (gfx950) implementation of the E.T. encoder
 * hot path.  Plain pointers and sizes only; every entry point returns 0 on
 * success or a negative ET_ERR_* code (never exits, never throws).  All
 * activation / weight pointers are DEVICE pointers to IEEE binary16 unless a
 * parameter is documented as host memory.  `stream` is a hipStream_t passed
 * as void* (NULL = the default stream); launches are asynchronous on it.
 *
 * Each launcher names the reference interface it replaces
 * (paths relative to the reference tree).
 */
#ifndef ET_AMD_H
#define ET_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ET_OK 0
#define ET_ERR_INVALID_ARG (-1) /* null pointer, non-positive or inconsistent size */
#define ET_ERR_ALIGNMENT (-2)   /* pointer or leading dimension not 16-byte aligned */
#define ET_ERR_UNSUPPORTED (-3) /* shape outside what the kernels cover */
#define ET_ERR_HIP (-4)         /* a HIP runtime call failed; see et_last_error() */
#define ET_ERR_FORMAT (-5)      /* malformed tile_mat / row_mat index arrays or container file */
#define ET_ERR_IO (-6)          /* a file could not be opened, read or written */

/* Human-readable text for a code; message of the last failure on this thread. */
const char *et_strerror(int code);
const char *et_last_error(void);
/* Version of this ABI (bumped on incompatible change). */
int et_abi_version(void);

/* ------------------------------------------------------------------------
 * L0 launchers — one per prototype of kernels/kernels.h:3-34.
 * ---------------------------------------------------------------------- */

/* Replaces skip_layernorm_kernelLauncher (kernels/kernels.h:3-5,
 * kernels/skip_layernorm.cu:101-112).  in_out[num x size] =
 * LayerNorm(in_out + skip) * gamma + beta, eps 1e-6, biased variance, fp32
 * statistics.  size must be even. */
int et_skip_layernorm(void *in_out, const void *skip, const void *gamma,
                      const void *beta, int num, int size, void *stream);

/* Replaces tile_spmm_add_bias_kernelLauncher (kernels/kernels.h:13-15,
 * kernels/linear.cu:152-158).  Y[M x N] = X[M x K] * W^T + bias with W[N x K]
 * held as tile_mat: W_row_ptr[N/16+1], W_row_offset[ntile] (element column
 * offsets, multiples of 16, any order inside a block-row),
 * W_data[ntile*256] with W_data[i*256+n*16+k] = W[bn*16+n][W_row_offset[i]+k].
 * K (= in_feat, the leading dimension of X) is an added argument: the
 * reference launcher omits it and uses M in its place.  M is any positive
 * row count; N and K are multiples of 16. */
int et_tile_spmm_add_bias(void *Y, const void *X, const int *W_row_ptr,
                          const int *W_row_offset, const void *W_data, int M,
                          int N, int K, const void *bias, void *stream);

/* Replaces tile_spmm_add_bias_gelu_kernelLauncher (kernels/kernels.h:17-20,
 * kernels/linear.cu:160-167): as above followed by the tanh-form GELU of
 * kernels/linear.cu:36-48 on the half-rounded sum. */
int et_tile_spmm_add_bias_gelu(void *Y, const void *X, const int *W_row_ptr,
                               const int *W_row_offset, const void *W_data,
                               int M, int N, int K, const void *bias,
                               void *stream);

/* Replaces row_spmm_add_bias_kernelLauncher (kernels/kernels.h:7-11,
 * kernels/linear.cu:18-34): out[M x N] = in[M x K] * weight^T + bias with
 * weight[N x K] row-major (the compacted surviving rows, N padded to a
 * multiple of 16).  The cuBLAS handle/algo pair becomes a stream. */
int et_row_spmm_add_bias(void *out, const void *in, const void *weight,
                         const void *bias, int M, int N, int K, void *stream);
/* the same followed by the tanh-form GELU of kernels/linear.cu:36-48 (the
 * reference's row linear has no GELU form; a row-pruned FFN1 needs it) */
int et_row_spmm_add_bias_gelu(void *out, const void *in, const void *weight,
                              const void *bias, int M, int N, int K,
                              void *stream);
/* n <= 3 such linears over the same input in one launch (Q and K of the
 * attention-aware pruned layer): outs[i][M x Ns[i]] = in * weights[i]^T +
 * biases[i].  No counterpart in the reference. */
int et_row_spmm_add_bias_multi(void *const *outs, const void *in,
                               const void *const *weights,
                               const void *const *biases, const int *Ns, int n,
                               int M, int K, void *stream);
/* 1 where the two functions above run the register-blocked dense GEMM kernel
 * for these sizes (from 1024 rows, K a multiple of 32) and 0 where they run
 * the tile kernels on W taken as is: a caller that also holds the weights as
 * a planned tile_mat (Linear_row does) runs the plan in the second case. */
int et_row_spmm_prefers_gemm(int M, int N, int K);

/* Replaces OTF_attention_kernelLauncher (kernels/kernels.h:22-24,
 * kernels/attention.cu:122-134).  out, Q, K, V are [batch*seq_len x d_model];
 * head h owns columns h*hd..(h+1)*hd-1, hd = d_model/nhead a multiple of 16
 * up to 128 (the reference walks the head in steps of 16,
 * kernels/attention.cu:86-90); 32, 64 and 128 have kernels of their own, the
 * other widths run as ragged heads on the register-staged kernel of the next
 * of these (padded batches only: not through et_OTF_attention_varlen).
 * Z = softmax((Q*scale) K^T + mask) V per head without writing the score
 * matrix to memory; scale = half(sqrt(1/hd)) applied to Q in half; mask is
 * one additive [seq_len x seq_len] half matrix shared by heads and batch, or
 * NULL.  p = 2^(log2_scale*(s-max)): log2_scale 1.0f is the reference's
 * base-2 softmax (kernels/attention.cu:33), 1.44269504f (log2 e) the textbook
 * one.  Added: batch (>=1) and seq_lens (NULL, or batch ints in
 * [0,seq_len]: keys at or beyond seq_lens[b] are ignored and query rows at or
 * beyond it are written as zero). */
int et_OTF_attention(void *out, const void *Q, const void *K, const void *V,
                     const void *mask, int seq_len, int d_model, int nhead,
                     int batch, const int *seq_lens, float log2_scale,
                     void *stream);

/* Optional accelerator for masks with all-zero regions (the usual padding
 * mask): a summary holds one bit per (16 query rows, 64 keys) of the mask,
 * set when any element there is not +-0.  A launcher that is handed a mask
 * pointer with an attached summary skips the mask loads and additions for
 * all-zero tiles; s + 0 == s, so no result bit changes.  The caller computes
 * the summary once (device buffer of et_attention_mask_summary_bytes), attaches
 * it to the mask pointer, and detaches it (summary = NULL) before the mask
 * changes or is freed.  No counterpart in the reference, which adds the mask
 * unconditionally (kernels/attention.cu:79-84). */
size_t et_attention_mask_summary_bytes(int seq_len);
int et_attention_mask_summary(const void *mask, int seq_len, void *summary, void *stream);
int et_attention_mask_summary_attach(const void *mask, int seq_len, const void *summary);
/* et_OTF_attention with the mask's summary passed along (a device buffer filled
 * by et_attention_mask_summary for this mask and seq_len; NULL: the mask is
 * added everywhere): nothing is attached to, or looked up by, the mask's
 * address, so the summary's lifetime is the caller's own business and a freed
 * mask leaves nothing behind.  Same bits as the other forms. */
int et_OTF_attention_summary(void *out, const void *Q, const void *K, const void *V,
                             const void *mask, const void *mask_summary, int seq_len,
                             int d_model, int nhead, int batch, const int *seq_lens,
                             float log2_scale, void *stream);

/* et_OTF_attention for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  Same arguments and the same result,
 * bit for bit, as et_OTF_attention; what differs is where the mask summary
 * lives: this call computes it from `mask` on `stream` into a 2 KiB array
 * that is part of the library's device image (one copy per GPU, held until the
 * process ends) and hands it to the attention kernel, so all-zero mask tiles
 * are skipped without any buffer of the caller's and without the attach
 * registry.  It calls no hipMalloc, hipFree or other allocating routine.
 * Limit: with a mask, seq_len <= 4096 (ET_ERR_UNSUPPORTED beyond).  All calls
 * on one GPU share that array: calls that overlap on one GPU (different
 * streams or host threads) race; calls in stream order do not, and every word
 * a call reads it has written itself, so nothing needs clearing in between.
 * The array's address is looked up on the first call on a device: make that
 * call outside a graph capture. */
int et_OTF_attention_noalloc(void *out, const void *Q, const void *K,
                             const void *V, const void *mask, int seq_len,
                             int d_model, int nhead, int batch,
                             const int *seq_lens, float log2_scale,
                             void *stream);

/* et_OTF_attention with Q and K holding qk_width < head_dim columns per head,
 * the same number in every head (attention-aware pruning that keeps the heads
 * balanced): Q, K are [batch*seq_len x nhead*qk_width], head h at columns
 * h*qk_width, the scores contract over qk_width and are scaled by
 * half(1/sqrt(head_dim)) as before; V and out keep d_model columns.  Same
 * result as et_Prune_attention with qk_head_ptr[h] = h*qk_width, through the
 * on-the-fly kernel: the DMA-staged one for qk_width 32 with head_dim 64, the
 * register-staged one for any other multiple of 16 below head_dim.  No
 * counterpart in the reference, whose
 * Prune_attention (kernels/kernels.h:26-30) prunes V only. */
int et_OTF_attention_qk_width(void *out, const void *Q, const void *K,
                              const void *V, const void *mask, int qk_width,
                              int seq_len, int d_model, int nhead, int batch,
                              const int *seq_lens, float log2_scale,
                              void *stream);

/* Variable-length (packed) form of et_OTF_attention for the
 * sequence-length-aware path: rows of sequence b are
 * cu_seqlens[b]..cu_seqlens[b+1]-1 of out/Q/K/V (no padding rows exist);
 * mask, if given, is [max_seq_len x max_seq_len].  No reference counterpart
 * (the reference has no batch dimension). */
int et_OTF_attention_varlen(void *out, const void *Q, const void *K,
                            const void *V, const void *mask,
                            const int *cu_seqlens, int max_seq_len,
                            int d_model, int nhead, int batch,
                            float log2_scale, void *stream);

/* Replaces Prune_attention_kernelLauncher (kernels/kernels.h:26-30,
 * kernels/attention.cu:252-271).  V is compact [rows x ldv]; head h owns
 * compact columns v_head_ptr[h]..v_head_ptr[h+1]-1 whose results are written
 * to out[:, v_col_id[j]] (v_col_id sorted, inside the head's slice); every
 * other column of out is written as zero.  The reference's nnz_col_v is ldv.
 * Added: qk_head_ptr/ldqk — when non-NULL, Q and K are compact [rows x ldqk]
 * and head h contracts over columns qk_head_ptr[h]..qk_head_ptr[h+1]-1 (at
 * most hd of them); NULL keeps the reference's dense Q/K. batch, seq_lens,
 * log2_scale as for et_OTF_attention. */
int et_Prune_attention(void *out, const void *Q, const void *K, const void *V,
                       const int *qk_head_ptr, int ldqk, const int *v_col_id,
                       const int *v_head_ptr, int ldv, const void *mask,
                       int seq_len, int d_model, int nhead, int batch,
                       const int *seq_lens, float log2_scale, void *stream);

/* Replaces sharedQK_attention_kernelLauncher (kernels/kernels.h:32-34,
 * kernels/attention.cu:342-350): scores are read from
 * QK[(b*nhead+h)][seq_len][seq_len] (halves, already scaled). */
int et_sharedQK_attention(void *out, const void *QK, const void *V,
                          const void *mask, int seq_len, int d_model,
                          int nhead, int batch, const int *seq_lens,
                          float log2_scale, void *stream);

/* Replaces the cublasHgemmStridedBatched call of Encoder_length::run
 * (encoder/encoder.cu:126-130): QK[(b*nhead+h)][q][k] =
 * half(scale * sum_d Q[q][h*hd+d] K[k][h*hd+d]) from row-major
 * [batch*seq_len x d_model] Q and K. */
int et_qk_scores(void *QK, const void *Q, const void *K, int seq_len,
                 int d_model, int nhead, int batch, void *stream);

/* ------------------------------------------------------------------------
 * Planned tile linear — what Linear_tile (encoder/Linear.h:4-46) owns.
 * The plan keeps device copies of the weight in a kernel-friendly order
 * (tiles of a block-row sorted by column so K can be walked in LDS-sized
 * chunks); results equal et_tile_spmm_add_bias on the same tile_mat up to
 * fp32 summation order.
 * ---------------------------------------------------------------------- */
typedef struct et_tile_plan et_tile_plan;

/* All pointers are HOST memory, as in the Linear_tile constructor
 * (encoder/Linear.h:18-24). */
int et_tile_plan_create(et_tile_plan **plan, int in_feat, int out_feat,
                        int ntile, const void *data, const int *row_ptr,
                        const int *row_offset, const void *bias);
void et_tile_plan_destroy(et_tile_plan *plan);
/* Linear_tile::run (encoder/Linear.h:36-45); gelu selects the GELU variant. */
int et_tile_plan_run(const et_tile_plan *plan, void *Y, const void *X, int M,
                     int gelu, void *stream);
/* Linear_tile::run followed by skip_layernorm_kernelLauncher on its output
 * (encoder/encoder.cu:33-35 and 41-44; kernels/kernels.h:3-5) in ONE launch:
 *   Y = LayerNorm(half(X W^T + bias) + skip) * gamma + beta,
 * the sum rounded to half once, as the reference does.  One workgroup holds
 * whole rows, so this needs out_feat <= 1536 (et_tile_plan_ln_fusable); wider
 * plans run the two kernels one after the other, and then Y must not alias
 * skip.  With the fused kernel Y may be the same buffer as skip. */
int et_tile_plan_run_ln(const et_tile_plan *plan, void *Y, const void *X,
                        const void *skip, const void *gamma, const void *beta,
                        int M, void *stream);
int et_tile_plan_ln_fusable(const et_tile_plan *plan);
/* The feed-forward block of a layer, encoder/encoder.cu:36-44 (MLP1_linear
 * with GELU, MLP2_linear, skip_layernorm_kernelLauncher), in ONE launch:
 *   Y = LayerNorm(half(gelu(X W1^T + b1) W2^T + b2) + skip) * gamma + beta.
 * The hidden activations are rounded to half exactly as the reference stores
 * them, but stay in LDS: a workgroup walks the hidden dimension in chunks and
 * feeds every chunk straight into the second linear.  Needs
 * et_tile_plan_ffn_fusable(first, second): in_feat of the first <= 992, hidden
 * chunks and out_feat of the second <= 768 columns.  `hidden` is a device
 * buffer of M x hidden-width halves for the cases where the fused kernel does
 * not apply or does not pay (few rows): then the launches run one after the
 * other through it.  It may be NULL, which forces the fused kernel and fails
 * with ET_ERR_UNSUPPORTED where that does not apply.  Y may alias skip (and
 * skip may be X, the usual residual) only when the fused kernel runs. */
int et_tile_plan_run_ffn_ln(const et_tile_plan *first, const et_tile_plan *second,
                            void *Y, const void *X, void *hidden, const void *skip,
                            const void *gamma, const void *beta, int M, void *stream);
int et_tile_plan_ffn_fusable(const et_tile_plan *first, const et_tile_plan *second);
/* Steps 6-10 of a layer, encoder/encoder.cu:33-44 (O_linear, skip + LayerNorm
 * with the layer input, MLP1 with GELU, MLP2, skip + LayerNorm), in ONE launch:
 *   mid = LayerNorm(half(attn Wo^T + bo) + input) * gamma1 + beta1
 *   Y   = LayerNorm(half(gelu(mid W1^T + b1) W2^T + b2) + mid) * gamma2 + beta2.
 * The workgroup that owns a 32-row panel runs the projection first and keeps
 * its normalised rows (rounded to half, as the reference stores them) in LDS
 * as the feed-forward input and the second skip operand; mid never reaches
 * memory.  Needs et_tile_plan_tail_fusable(out, first, second): a square
 * projection of the model width on top of et_tile_plan_ffn_fusable.  `mid`
 * (M x model width halves) and `hidden` (M x hidden width) are device buffers
 * for the cases where the fused kernel does not apply or does not pay; with
 * mid == NULL the fused kernel is forced (ET_ERR_UNSUPPORTED where it does not
 * apply).  Y may alias attn or input when the fused kernel runs. */
int et_tile_plan_run_tail(const et_tile_plan *out, const et_tile_plan *first,
                          const et_tile_plan *second, void *Y, const void *attn,
                          const void *input, void *mid, void *hidden,
                          const void *gamma1, const void *beta1, const void *gamma2,
                          const void *beta2, int M, void *stream);
int et_tile_plan_tail_fusable(const et_tile_plan *out, const et_tile_plan *first,
                              const et_tile_plan *second);
/* The same five steps with device scratch from the caller, which opens a second
 * form of the launch: PAIRS of workgroups over 64-row or 32-row panels.  Both
 * workgroups of a pair run the projection and the first LayerNorm on the panel,
 * each takes one half of the hidden columns of the feed-forward block, and
 * their fp32 partial sums meet in `ws` (whoever arrives second at a row-half's
 * counter finishes it: no workgroup waits for another).  With 64-row panels a
 * CU streams half the weights per row; with 32-row panels two workgroups share
 * a CU.  Taken only when switched on (et_tuning_set
 * "tile_tail_pair"), where it applies (model width 256, 512 or 768, hidden
 * width a multiple of 16 and at least 384), ws_bytes >=
 * et_tile_plan_tail_ws_bytes(out, first, second, M) and there are enough row
 * panels to fill the device; otherwise this is et_tile_plan_run_tail.  ws must
 * not overlap any operand; its contents are scratch.  The per-plan program is
 * built by et_tile_plan_tail_prepare (device allocations; called implicitly by
 * the first run, so call it beforehand where a run must not allocate).  The
 * `second` plan carries the program and the per-panel counters: runs that
 * share it must not overlap in time.  Results differ from et_tile_plan_run_tail
 * in fp32 summation order only. */
int et_tile_plan_run_tail_ws(const et_tile_plan *out, const et_tile_plan *first,
                             const et_tile_plan *second, void *Y, const void *attn,
                             const void *input, void *mid, void *hidden, const void *gamma1,
                             const void *beta1, const void *gamma2, const void *beta2, int M,
                             void *ws, size_t ws_bytes, void *stream);
int et_tile_plan_tail_prepare(const et_tile_plan *out, const et_tile_plan *first,
                              const et_tile_plan *second);
/* bytes of scratch the paired form needs for M rows (0 where it does not apply) */
size_t et_tile_plan_tail_ws_bytes(const et_tile_plan *out, const et_tile_plan *first,
                                  const et_tile_plan *second, int M);
/* the same figure from the shapes alone (what an encoder adds to its workspace);
 * 0 while the paired form is switched off (et_tuning_set "tile_tail_pair" 0, the
 * default), so that Encoder_*::buffer_size is then the reference's five units */
size_t et_tail_ws_bytes_for(int d_model, int rows);
/* n (<= 4) planned linears with the same in_feat applied to the same X in ONE
 * launch (the Q/K/V projections, encoder/encoder.cu:22-26, which the
 * reference spreads over three streams). */
int et_tile_plan_run_multi(const et_tile_plan *const *plans, void *const *Ys,
                           int n, const void *X, int M, void *stream);
/* device pointers of the plan's buffers, for tests (sorted order) */
int et_tile_plan_query(const et_tile_plan *plan, int *in_feat, int *out_feat,
                       int *ntile, int *nchunk, int *chunk_cols);

/* ------------------------------------------------------------------------
 * Pruned-weight formats (host side; all pointers HOST memory).
 * ---------------------------------------------------------------------- */

/* Seeded form of gen_sparse_tile_mat (test/tile_mat.cu:5-34): ntile =
 * int(total*(1.0-sparsity)) tiles chosen by a splitmix64-driven Fisher-Yates
 * shuffle of the row-major tile grid; block-rows list their tiles in shuffle
 * order; row_offset = tile column * 16.  row_ptr: nrow/16+1 ints; row_offset:
 * capacity (nrow/16)*(ncol/16) ints.  Returns ntile (>= 0) or an error. */
int et_gen_sparse_tile_mat(int nrow, int ncol, float sparsity, uint64_t seed,
                           int *row_ptr, int *row_offset);
/* Seeded form of gen_sparse_row_mat (test/row_mat.cu:5-14): returns nn_row and
 * fills row_id (capacity nrow) with the sorted surviving row ids. */
int et_gen_sparse_row_mat(int nrow, float sparsity, uint64_t seed,
                          int *row_id);
/* keep `keep` of every head's head_dim rows (seeded, sorted); row_id capacity
 * nhead*keep.  Balanced variant used for per-head Q/K pruning. */
int et_gen_head_balanced_rows(int nhead, int head_dim, int keep, uint64_t seed,
                              int *row_id);
/* Magnitude-based selection in place of the random one: from dense row-major
 * W[N x K] (halves) keep the int(total*(1.0-sparsity)) 16x16 tiles (resp.
 * int(N*(1.0-sparsity)) rows) with the largest sum of squares (accumulated in
 * double, row-major; ties keep the lower index; NaN counts as 0).  Tiles are
 * listed by ascending column inside a block-row, row_id ascending.  Counts
 * follow test/tile_mat.cu:10-11 and test/row_mat.cu:7; the reference itself
 * only selects at random (test/tile_mat.cu:16, test/row_mat.cu:11).  Returns
 * the number kept; follow with et_tile_pack / a row gather for the values. */
int et_prune_tile_mat(const void *W, int N, int K, float sparsity, int *row_ptr,
                      int *row_offset);
int et_prune_row_mat(const void *W, int N, int K, float sparsity, int *row_id);

/* On-disk container of a pruned linear (the reference keeps none): 64-byte
 * little-endian header (magic, version 1, in_feat, out_feat, count, payload
 * bytes, FNV-1a 64 of the payload) followed by
 *   tile_mat: row_ptr[out_feat/16+1], row_offset[ntile], data[ntile*256], bias[out_feat]
 *   row_mat : row_id[nrow], weight[nrow x in_feat] (compact rows), bias[out_feat]
 * _peek reads the sizes so that the caller can allocate; _load is told the
 * sizes that the arrays were allocated for, refuses a file whose header says
 * otherwise before it writes anything (the file may have changed since the
 * peek), verifies size, checksum and the format's invariants (ET_ERR_FORMAT)
 * and fills the arrays. */
int et_tile_mat_save(const char *path, int in_feat, int out_feat, int ntile,
                     const int *row_ptr, const int *row_offset, const void *data,
                     const void *bias);
int et_tile_mat_peek(const char *path, int *in_feat, int *out_feat, int *ntile);
int et_tile_mat_load(const char *path, int in_feat, int out_feat, int ntile,
                     int *row_ptr, int *row_offset, void *data, void *bias);
int et_row_mat_save(const char *path, int in_feat, int out_feat, int nrow,
                    const int *row_id, const void *weight, const void *bias);
int et_row_mat_peek(const char *path, int *in_feat, int *out_feat, int *nrow);
int et_row_mat_load(const char *path, int in_feat, int out_feat, int nrow,
                    int *row_id, void *weight, void *bias);

/* 0 if (row_ptr,row_offset) is a well-formed tile_mat of W[N x K]
 * (the asserts of test/tile_mat.cu:31-33 plus range/alignment/duplicates). */
int et_tile_mat_validate(int N, int K, int ntile, const int *row_ptr,
                         const int *row_offset);
/* data[i*256+n*16+k] = W[bn*16+n][row_offset[i]+k] from dense row-major W. */
int et_tile_pack(const void *W, int N, int K, const int *row_ptr,
                 const int *row_offset, void *data);
/* CSR of a sorted row_id over heads: head_ptr[h] = #ids < h*head_dim,
 * head_ptr[nhead] = n (intent of encoder/Linear.cu:74-88). */
int et_head_ptr(const int *row_id, int n, int nhead, int head_dim,
                int *head_ptr);

/* ------------------------------------------------------------------------
 * Sequence-length-aware path helpers (no reference counterpart).
 * ---------------------------------------------------------------------- */
/* packed[cu_seqlens[b]+t][:] = padded[b*seq_len+t][:] for t < len_b */
int et_pack_rows(void *packed, const void *padded, const int *cu_seqlens,
                 int batch, int seq_len, int width, void *stream);
/* inverse; padding rows of `padded` are written as zero */
int et_unpack_rows(void *padded, const void *packed, const int *cu_seqlens,
                   int batch, int seq_len, int width, void *stream);
/* The same with the packed sequences in another order: packed sequence i
 * (rows cu_seqlens[i] .. cu_seqlens[i+1]) is padded sequence order[i]; order
 * is a device array holding a permutation of 0..batch-1, NULL = identity.
 * Packing longest first makes the attention kernel, which dispatches packed
 * sequences in index order, start the longest ones first. */
int et_pack_rows_ordered(void *packed, const void *padded,
                         const int *cu_seqlens, const int *order, int batch,
                         int seq_len, int width, void *stream);
int et_unpack_rows_ordered(void *padded, const void *packed,
                           const int *cu_seqlens, const int *order, int batch,
                           int seq_len, int width, void *stream);
/* out[r][col_id[j]] = in[r][j] for j < n, every other column of out[rows x
 * width] zero: expands a row_mat linear's compact output
 * (kernels/linear.cu:30-32) back to model width. */
int et_scatter_cols(void *out, const void *in, const int *col_id, int rows,
                    int n, int ld_in, int width, void *stream);
/* et_scatter_cols followed by et_skip_layernorm (kernels/kernels.h:3-5) in
 * one launch: out[num x size] = LayerNorm(expand(compact) + skip), the
 * expanded rows never written to memory.  out may alias skip, not compact. */
int et_scatter_skip_layernorm(void *out, const void *compact,
                              const int *col_id, int n, int ld_in,
                              const void *skip, const void *gamma,
                              const void *beta, int num, int size,
                              void *stream);

/* ------------------------------------------------------------------------
 * Device memory / stream plumbing so that host code above this ABI needs no
 * HIP headers (Weight<T>, encoder/utils.h:14-43; streams,
 * encoder/encoder.h:36-39).
 * ---------------------------------------------------------------------- */
int et_malloc(void **ptr, size_t bytes);
int et_free(void *ptr);
int et_memcpy_h2d(void *dst, const void *src, size_t bytes);
int et_memcpy_d2h(void *dst, const void *src, size_t bytes);
int et_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream);
int et_fill_zero(void *dst, size_t bytes, void *stream);
/* plain device-to-device copy KERNEL (16-byte granularity); unlike a runtime
 * memcpy it always shows up as a kernel dispatch, which makes it the
 * known-size reference for scaling hardware traffic counters */
int et_copy(void *dst, const void *src, size_t bytes, void *stream);
int et_stream_create(void **stream);
int et_stream_destroy(void *stream);
int et_stream_synchronize(void *stream);
int et_device_synchronize(void);
/* Launch-heuristic overrides for benchmarking sweeps; value 0 restores the
 * automatic choice unless noted.  Keys:
 *   "tile_nb"         block-rows of W per wave in the tile linear (1, 2, 3; the
 *                     raw launchers also take 4 and 6)
 *   "tile_min_wgs"    workgroups the automatic choices aim for (default 512)
 *   "tile_ipw"        work items per persistent workgroup of a planned linear
 *   "tile_fuse_ln"    0: et_tile_plan_run_ln runs the linear and the LayerNorm
 *                     as two launches; 1 (default): fused where the rows fit
 *   "tile_ln_min_panels" fewest 32-row panels for which et_tile_plan_run_ln
 *                     fuses (default 96; below, two launches are faster); a
 *                     value > 0 also replaces the 72 panels from which
 *                     et_tile_plan_run_tail runs as one launch
 *   "tile_bm64"       0: planned linears always use 32-row panels; 1 (default):
 *                     64-row panels where two such items per CU exist; 2: also
 *                     with fewer items; 4: as 1 with eight waves per workgroup
 *                     only (no twelve-wave form)
 *   "tile_splitk_rows" most rows for which a planned linear with K > 992 runs
 *                     the few-rows kernel (16-row panels, a block-row's tile
 *                     pairs split over several waves); -1 (default): 128, or
 *                     256 where at least 3/4 of the tiles survive; 0: never
 *   "tile_splitk_k1"  1: the few-rows kernel also for K <= 992 (default 0)
 *   "row_gemm_min_rows" rows from which et_row_spmm_add_bias runs the dense
 *                     GEMM kernel (default 1024; 0: never)
 *   "tile_fuse_ffn"   0: et_tile_plan_ffn_fusable answers no (the feed-forward
 *                     block runs as separate launches); 1: the block is fused
 *                     but et_tile_plan_tail_fusable answers no; 2 (default)
 *   "tile_ln_chunked" 0: fused LayerNorm with K > 992 uses the single-buffer
 *                     kernel; 1 (default): the double-buffered one
 *   "ln_rows"         rows per wave of et_skip_layernorm (1, 2, 4)
 *   "attn_variant"    0: 4 waves x 32 query rows, 1: 8 waves x 16 rows,
 *                     2: 4 waves x 16 rows; -1 automatic
 *   "attn_vwin"       0: et_Prune_attention always stages K and V through
 *                     registers; 1 (default): dense Q/K with a compact V whose
 *                     pitch is a multiple of 8 take the DMA-staged kernel
 *   "attn_packed"     0: et_OTF_attention_varlen launches one workgroup per
 *                     possible query block; 1 (default): workgroups walk the
 *                     blocks that exist (up to 256 sequences)
 *   "tile_tail_pair"  0 (default): et_tile_plan_run_tail_ws never takes the paired
 *                     form (measured slower than the one-workgroup form on the
 *                     BERT-base shapes); 1: where it applies and there are
 *                     enough row panels (32-row panels); 2: wherever it applies,
 *                     64-row panels; 3: wherever it applies, 32-row panels
 *   "tile_tail_pair_min_wgs" fewest workgroups (two per 64-row panel) for the
 *                     paired form (default: three quarters of the CUs)
 *   "tile_wait_spin"  polls after which a bounded wait inside a workgroup gives
 *                     up (default 2^22; negative restores it).  A wave that gives
 *                     up sets a status word, the launch's result is wrong, and
 *                     the next launch of that kind returns ET_ERR_HIP once.  0
 *                     makes every wait give up at once (for testing the report)
 *   "tile_tail_min_panels"  row panels below which the layer tail runs step
 *                     by step when the caller gave it buffers (default 72)
 * Not thread-safe; results never depend on these beyond fp32 summation
 * order. */
int et_tuning_set(const char *key, int value);
/* The fused layer-tail kernels order their waves with bounded waits on LDS
 * counters.  A wave that gives up (it never should) sets one status word per
 * process and goes on, so the kernel ends - with a wrong result - instead of
 * hanging the GPU; the next launch of such a kernel returns ET_ERR_HIP once and
 * clears the word.  et_wait_status_take does the same check on demand (ET_OK or
 * ET_ERR_HIP); et_wait_status_raise_for_test sets the word from the host, which
 * is how the report is tested without a wave ever missing a signal.  No
 * counterpart in the reference, which has no kernel that waits. */
int et_wait_status_take(void);
void et_wait_status_raise_for_test(void);
/* number of compute units of the current device (0 if none) */
int et_device_cu_count(void);

#ifdef __cplusplus
}
#endif
#endif /* ET_AMD_H */
