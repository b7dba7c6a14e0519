/*
 * et_encoder.h — C ABI over the encoder-layer objects (the C++ classes in
 * et_amd/encoder/{Linear.h,encoder.h}, which carry the reference's names and
 * signatures).  This is what a non-C++ host (the Python binding, a cgo/JNI
 * stub) binds; C++ callers include the class headers directly.
 *
 * Conventions as in et_amd.h: 0 / negative ET_ERR_* return codes, device
 * pointers for activations and workspace, HOST pointers for everything a
 * constructor copies (weights, index arrays, LayerNorm parameters, mask).
 */
#ifndef ET_ENCODER_H
#define ET_ENCODER_H

#include "et_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct et_linear_tile et_linear_tile;
typedef struct et_linear_row et_linear_row;
typedef struct et_encoder et_encoder;
typedef struct et_encoder_stack et_encoder_stack;

/* Linear_tile(in_feat, out_feat, size, ntile, data, row_ptr, row_offset, bias,
 * is_gelu) — encoder/Linear.h:18-24.  Host pointers. */
int et_linear_tile_create(et_linear_tile **h, int in_feat, int out_feat, int size, int ntile,
                          const void *data, const int *row_ptr, const int *row_offset,
                          const void *bias, int is_gelu);
void et_linear_tile_destroy(et_linear_tile *h);
/* Linear_tile::run(out, in, stream) — encoder/Linear.h:36-45 */
int et_linear_tile_run(const et_linear_tile *h, void *out, const void *in, void *stream);
/* same on `rows` rows instead of the constructor's size */
int et_linear_tile_run_rows(const et_linear_tile *h, void *out, const void *in, int rows, void *stream);
/* the linear, the skip connection and LayerNorm in one launch
 * (et_tile_plan_run_ln): out = LayerNorm(half(linear(in)) + skip) */
int et_linear_tile_run_rows_ln(const et_linear_tile *h, void *out, const void *in, const void *skip,
                               const void *gamma, const void *beta, int rows, void *stream);
/* the feed-forward block (encoder/encoder.cu:36-44: MLP1 with GELU, MLP2,
 * skip + LayerNorm) in one launch (et_tile_plan_run_ffn_ln); `hidden`
 * ([rows x first.out_feat] halves, may be NULL to insist on the fused kernel)
 * is used only where that kernel does not apply */
int et_linear_tile_run_rows_ffn_ln(const et_linear_tile *first, const et_linear_tile *second, void *out,
                                   const void *in, void *hidden, const void *skip, const void *gamma,
                                   const void *beta, int rows, void *stream);
int et_linear_tile_ffn_fusable(const et_linear_tile *first, const et_linear_tile *second);
/* steps 6-10 of a layer (encoder/encoder.cu:33-44: O_linear, skip + LayerNorm,
 * MLP1 with GELU, MLP2, skip + LayerNorm) in one launch (et_tile_plan_run_tail);
 * `mid` ([rows x model width]) and `hidden` ([rows x first.out_feat]) are used
 * only where the fused kernel does not apply; mid == NULL insists on it */
int et_linear_tile_run_rows_tail(const et_linear_tile *out_proj, const et_linear_tile *first,
                                 const et_linear_tile *second, void *out, const void *attn, const void *input,
                                 void *mid, void *hidden, const void *gamma1, const void *beta1,
                                 const void *gamma2, const void *beta2, int rows, void *stream);
/* the same with device scratch `ws` (et_linear_tile_tail_ws_bytes for these rows),
 * which lets the launch take the form of pairs of workgroups over 64-row panels
 * (et_tile_plan_run_tail_ws); et_linear_tile_tail_prepare builds what that form
 * needs ahead of the first run */
int et_linear_tile_run_rows_tail_ws(const et_linear_tile *out_proj, const et_linear_tile *first,
                                    const et_linear_tile *second, void *out, const void *attn, const void *input,
                                    void *mid, void *hidden, const void *gamma1, const void *beta1,
                                    const void *gamma2, const void *beta2, int rows, void *ws, size_t ws_bytes,
                                    void *stream);
int et_linear_tile_tail_prepare(const et_linear_tile *out_proj, const et_linear_tile *first,
                                const et_linear_tile *second);
size_t et_linear_tile_tail_ws_bytes(const et_linear_tile *out_proj, const et_linear_tile *first,
                                    const et_linear_tile *second, int rows);
int et_linear_tile_tail_fusable(const et_linear_tile *out_proj, const et_linear_tile *first,
                                const et_linear_tile *second);
/* n <= 4 linears over one input in one launch (Q/K/V, encoder/encoder.cu:22-26) */
int et_linear_tile_run_multi(const et_linear_tile *const *hs, void *const *outs, int n,
                             const void *in, int rows, void *stream);

/* Linear_row(in_feat, out_feat, size, weight, row_id, nrow, bias, nhead) —
 * encoder/Linear.h:66-67, encoder/Linear.cu:60-91.  Host pointers; row_id
 * ascending. */
int et_linear_row_create(et_linear_row **h, int in_feat, int out_feat, int size, const void *weight,
                         const int *row_id, int row_id_size, const void *bias, int nhead);
/* added: apply the tanh-form GELU to the compact output (a row-pruned FFN1) */
int et_linear_row_set_gelu(et_linear_row *h, int on);
void et_linear_row_destroy(et_linear_row *h);
/* Linear_row::run(out, in, handle) — encoder/Linear.h:68-71; out is compact
 * [size x nrow]. */
int et_linear_row_run(const et_linear_row *h, void *out, const void *in, void *stream);
/* public members of Linear_row that Encoder_prune::run reads
 * (encoder/encoder.cu:77-78): padded row count, surviving row count, device
 * pointers of row_id and head_ptr. */
int et_linear_row_query(const et_linear_row *h, int *nrow, int *row_id_size, const int **row_id_dev,
                        const int **head_ptr_dev);

enum { ET_ENCODER_TILE = 0, ET_ENCODER_PRUNE = 1, ET_ENCODER_LENGTH = 2, ET_ENCODER_ATTNAWARE = 3 };

/* Encoder_tile / Encoder_prune / Encoder_length constructors
 * (encoder/encoder.h:70-75, 93-98, 122-127) with the added trailing `batch`.
 * q,k,o,mlp1,mlp2 are et_linear_tile handles; v is an et_linear_tile for
 * TILE/LENGTH and an et_linear_row for PRUNE.  The encoder takes ownership of
 * the six linears (the reference moves them in): the handles are consumed and
 * must not be used or destroyed afterwards.  buffer: device workspace of
 * et_encoder_buffer_size() bytes, caller-owned.  mask may be NULL. */
int et_encoder_create(et_encoder **h, int kind, int d_model, int seq_len, int nheads, int batch,
                      void *buffer, et_linear_tile *q, et_linear_tile *k, void *v, et_linear_tile *o,
                      et_linear_tile *mlp1, et_linear_tile *mlp2, const void *ln_gamma_1,
                      const void *ln_beta_1, const void *ln_gamma_2, const void *ln_beta_2,
                      const void *mask);
/* Encoder_attnaware: attention-aware pruning through the whole layer (no
 * counterpart in the reference, which row-prunes only V).  q and k keep the
 * same columns per head; o, mlp1 (GELU set) and mlp2 are row-pruned, with
 * mlp2's in_feat equal to mlp1's padded row count.  Ownership as for
 * et_encoder_create; kind of the result is ET_ENCODER_ATTNAWARE. */
int et_encoder_attnaware_create(et_encoder **h, int d_model, int seq_len, int nheads, int batch,
                                void *buffer, et_linear_row *q, et_linear_row *k, et_linear_tile *v,
                                et_linear_row *o, et_linear_row *mlp1, et_linear_row *mlp2,
                                const void *ln_gamma_1, const void *ln_beta_1, const void *ln_gamma_2,
                                const void *ln_beta_2, const void *mask);
void et_encoder_destroy(et_encoder *h);
/* Encoder_base::buffer_size / Encoder_length::buffer_size
 * (encoder/encoder.h:51-53,129-133), times batch. */
size_t et_encoder_buffer_size(int kind, int d_model, int seq_len, int nheads, int batch);
/* Encoder_*::run(out, in) — encoder/encoder.cu:20,65,116; out may alias in. */
int et_encoder_run(et_encoder *h, void *out, const void *in);
int et_encoder_set_stream(et_encoder *h, void *stream);
int et_encoder_set_log2_scale(et_encoder *h, float log2_scale);
/* host array of `batch` lengths, or NULL to clear */
int et_encoder_set_seq_lens(et_encoder *h, const int *lens);
/* ET_ENCODER_LENGTH only: route attention through scores in memory
 * (the reference's Encoder_length::run, encoder/encoder.cu:126-137) */
int et_encoder_set_shared_qk(et_encoder *h, int on);

/* N ET_ENCODER_LENGTH layers run as one stack on packed rows (layers are
 * borrowed, not owned). act: device scratch of batch*seq_len*d_model halves. */
int et_encoder_stack_create(et_encoder_stack **h, et_encoder *const *layers, int n, int d_model,
                            int seq_len, int batch);
void et_encoder_stack_destroy(et_encoder_stack *h);
int et_encoder_stack_run(et_encoder_stack *h, void *out, const void *in, void *act, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ET_ENCODER_H */
