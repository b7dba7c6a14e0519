// Encoder layer orchestration.  Same class names, constructor arguments and
// run() meaning as encoder/encoder.h of the reference.  Differences, all
// additive: an optional trailing `batch` (the reference binds one sequence per
// encoder), a caller-settable stream, an exponent-base switch for the softmax,
// optional per-sequence lengths.  One stream, no host synchronisation inside
// run() (the reference blocks the host three times per layer,
// encoder/encoder.cu:27-29), Q/K/V projected by one launch.
#pragma once
#include <algorithm>
#include <vector>

#include "Linear.h"
#include "utils.h"

class Encoder_base {
  public:
    static constexpr int buffer_num = 5; // encoder/encoder.h:9

  protected:
    int d_model;
    int seq_len;
    int nheads;
    int batch;
    half *buffer;              // caller-owned device workspace
    half *buffers[buffer_num]; // units of batch*seq_len*d_model halves
    Weight<half> ln_gamma[2];
    Weight<half> ln_beta[2];
    Weight<half> mask;  // [seq_len x seq_len] additive, shared by heads and batch
    bool has_mask;
    unsigned *mask_summary; // which 16x64 regions of the mask are non-zero (et_attention_mask_summary)
    void *stream;       // hipStream_t; NULL = default stream
    float log2_scale;   // 1 = base-2 softmax of the reference, log2(e) = textbook
    // per-sequence lengths (optional)
    std::vector<int> lens;
    Weight<int> d_lens;
    Weight<int> d_cu;    // row offsets of the packed sequences
    Weight<int> d_order; // packed position -> batch index
    int total_rows; // sum of lengths when set, else batch*seq_len
    // scratch of the layer tail's paired form (et_tile_plan_run_tail_ws), behind the
    // activation units (and behind the score buffer of Encoder_length)
    void *tail_ws;
    size_t tail_ws_bytes;

    int rows() const { return batch * seq_len; }
    static size_t align256(size_t v) { return (v + 255) / 256 * 256; }
    static size_t units_bytes(int d_model_, int seq_len_, int batch_) {
        return (size_t)buffer_num * d_model_ * seq_len_ * batch_ * sizeof(half);
    }
    void place_tail_ws(size_t byte_offset) {
        tail_ws = reinterpret_cast<char *>(buffer) + align256(byte_offset);
        tail_ws_bytes = et_tail_ws_bytes_for(d_model, batch * seq_len);
    }

  public:
    // ln_* and mask_ are HOST pointers (d_model halves; seq_len*seq_len halves).
    // mask_ == nullptr means no mask.
    Encoder_base(int d_model_, int seq_len_, int nheads_, half *buffer_, half *ln_gamma_1,
                 half *ln_beta_1, half *ln_gamma_2, half *ln_beta_2, half *mask_, int batch_ = 1)
        : d_model(d_model_), seq_len(seq_len_), nheads(nheads_), batch(batch_), buffer(buffer_),
          ln_gamma{Weight<half>(ln_gamma_1, d_model_), Weight<half>(ln_gamma_2, d_model_)},
          ln_beta{Weight<half>(ln_beta_1, d_model_), Weight<half>(ln_beta_2, d_model_)},
          has_mask(mask_ != nullptr), mask_summary(nullptr), stream(nullptr), log2_scale(1.0f),
          total_rows(batch_ * seq_len_), tail_ws(nullptr), tail_ws_bytes(0) {
        if (mask_) {
            mask = Weight<half>(mask_, seq_len_ * seq_len_);
            // the mask never changes after construction: let the attention
            // launchers skip its all-zero tiles
            etChk(et_malloc((void **)&mask_summary, et_attention_mask_summary_bytes(seq_len_)));
            etChk(et_attention_mask_summary(mask.get(), seq_len_, mask_summary, nullptr));
            etChk(et_device_synchronize());
            etChk(et_attention_mask_summary_attach(mask.get(), seq_len_, mask_summary));
        }
        for (int i = 0; i < buffer_num; i++)
            buffers[i] = buffer + (size_t)i * batch * seq_len * d_model;
        place_tail_ws(units_bytes(d_model, seq_len, batch));
    }
    virtual ~Encoder_base() {
        if (mask_summary) {
            et_attention_mask_summary_attach(mask.get(), seq_len, nullptr);
            et_free(mask_summary);
        }
    }
    Encoder_base(const Encoder_base &) = delete;
    Encoder_base &operator=(const Encoder_base &) = delete;
    virtual void run(half *out, half *in) = 0; // device pointers; out may alias in
    // the reference's five activation units (encoder/encoder.h:51-53) plus the
    // layer tail's scratch
    static size_t buffer_size(int d_model_, int seq_len_, int /*nheads_*/, int batch_ = 1) {
        return align256(units_bytes(d_model_, seq_len_, batch_)) + et_tail_ws_bytes_for(d_model_, batch_ * seq_len_);
    }

    void set_stream(void *s) { stream = s; }
    void set_log2_scale(float v) { log2_scale = v; }
    // HOST array of `batch` lengths in [0, seq_len]; nullptr clears them.
    void set_seq_lens(const int *host_lens) {
        // a length outside [0, seq_len] would push the packed row offsets past
        // the workspace units: refuse before anything changes or reaches the device
        for (int b = 0; host_lens && b < batch; b++)
            etRequire(host_lens[b] >= 0 && host_lens[b] <= seq_len,
                      "set_seq_lens: every length must lie in [0, seq_len]");
        lens.clear();
        total_rows = batch * seq_len;
        if (!host_lens)
            return;
        lens.assign(host_lens, host_lens + batch);
        // packed layout: longest sequence first (ties in batch order), so the
        // attention kernel, which starts workgroups in packed order, ends with
        // the short ones
        std::vector<int> order(batch);
        for (int b = 0; b < batch; b++)
            order[b] = b;
        std::stable_sort(order.begin(), order.end(), [this](int x, int y) { return lens[x] > lens[y]; });
        std::vector<int> cu(batch + 1, 0);
        for (int i = 0; i < batch; i++)
            cu[i + 1] = cu[i] + lens[order[i]];
        total_rows = cu[batch];
        d_lens = Weight<int>(lens.data(), batch);
        d_cu = Weight<int>(cu.data(), batch + 1);
        d_order = Weight<int>(order.data(), batch);
    }
    int valid_rows() const { return total_rows; }
    // packed sequence i is rows cu[i]..cu[i+1]-1 and is batch entry order[i]
    const int *device_cu_seqlens() const { return lens.empty() ? nullptr : d_cu.get(); }
    const int *device_pack_order() const { return lens.empty() ? nullptr : d_order.get(); }

  protected:
    half *mask_ptr() const { return has_mask ? mask.get() : nullptr; }
    const int *lens_ptr() const { return lens.empty() ? nullptr : d_lens.get(); }

    // steps 6-10 of encoder/encoder.cu:33-44, shared by every encoder kind:
    // O projection, skip-LN with the layer input, FFN1+GELU, FFN2, skip-LN.
    void tail(half *out, half *in, half *attn, const Linear_tile &O, const Linear_tile &M1,
              const Linear_tile &M2, int nrows) {
        // (all five steps are one launch; unit 0 for the first LayerNorm's rows
        // and units 1..4 for the hidden activations are only touched where the
        // fused kernel does not apply)
        Linear_tile::run_rows_tail(O, M1, M2, out, attn, in, buffers[0], buffers[1], ln_gamma[0].get(),
                                   ln_beta[0].get(), ln_gamma[1].get(), ln_beta[1].get(), nrows, stream, tail_ws,
                                   tail_ws_bytes);
    }
};

// On-the-fly attention + tensor-tile pruned linears (encoder/encoder.h:56-77,
// encoder/encoder.cu:20-45).
class Encoder_tile : public Encoder_base {
  private:
    Linear_tile Q_linear, K_linear, V_linear, O_linear, MLP1_linear, MLP2_linear;

  public:
    Encoder_tile(int d_model_, int seq_len_, int nheads_, half *buffer_, Linear_tile &&Q_linear_,
                 Linear_tile &&K_linear_, Linear_tile &&V_linear_, Linear_tile &&O_linear_,
                 Linear_tile &&MLP1_linear_, Linear_tile &&MLP2_linear_, half *ln_gamma_1,
                 half *ln_beta_1, half *ln_gamma_2, half *ln_beta_2, half *mask_, int batch_ = 1)
        : Encoder_base(d_model_, seq_len_, nheads_, buffer_, ln_gamma_1, ln_beta_1, ln_gamma_2,
                       ln_beta_2, mask_, batch_),
          Q_linear(std::move(Q_linear_)), K_linear(std::move(K_linear_)),
          V_linear(std::move(V_linear_)), O_linear(std::move(O_linear_)),
          MLP1_linear(std::move(MLP1_linear_)), MLP2_linear(std::move(MLP2_linear_)) {
        // the reference asserts this (encoder/encoder.cu:17)
        etRequire(MLP1_linear.is_gelu, "Encoder_tile: MLP1_linear must be the GELU variant");
        Linear_tile::tail_prepare(O_linear, MLP1_linear, MLP2_linear);
    }
    void run(half *out, half *in) override {
        const Linear_tile *qkv[3] = {&Q_linear, &K_linear, &V_linear};
        half *outs[3] = {buffers[0], buffers[1], buffers[2]};
        Linear_tile::run_multi(qkv, outs, 3, in, rows(), stream);
        etChk(et_OTF_attention(buffers[3], buffers[0], buffers[1], buffers[2], mask_ptr(), seq_len,
                               d_model, nheads, batch, lens_ptr(), log2_scale, stream));
        tail(out, in, buffers[3], O_linear, MLP1_linear, MLP2_linear, rows());
    }
};

// Attention-aware pruning: V projected by a row-pruned linear into a compact
// [rows x nrow] matrix, attention over the surviving V columns
// (encoder/encoder.h:79-100, encoder/encoder.cu:65-92).
class Encoder_prune : public Encoder_base {
  private:
    Linear_tile Q_linear, K_linear;
    Linear_row V_linear;
    Linear_tile O_linear, MLP1_linear, MLP2_linear;

  public:
    Encoder_prune(int d_model_, int seq_len_, int nheads_, half *buffer_, Linear_tile &&Q_linear_,
                  Linear_tile &&K_linear_, Linear_row &&V_linear_, Linear_tile &&O_linear_,
                  Linear_tile &&MLP1_linear_, Linear_tile &&MLP2_linear_, half *ln_gamma_1,
                  half *ln_beta_1, half *ln_gamma_2, half *ln_beta_2, half *mask_, int batch_ = 1)
        : Encoder_base(d_model_, seq_len_, nheads_, buffer_, ln_gamma_1, ln_beta_1, ln_gamma_2,
                       ln_beta_2, mask_, batch_),
          Q_linear(std::move(Q_linear_)), K_linear(std::move(K_linear_)),
          V_linear(std::move(V_linear_)), O_linear(std::move(O_linear_)),
          MLP1_linear(std::move(MLP1_linear_)), MLP2_linear(std::move(MLP2_linear_)) {
        etRequire(MLP1_linear.is_gelu, "Encoder_prune: MLP1_linear must be the GELU variant");
        Linear_tile::tail_prepare(O_linear, MLP1_linear, MLP2_linear);
    }
    void run(half *out, half *in) override {
        if (V_linear.plan && V_linear.in_feat == Q_linear.in_features() &&
            K_linear.in_features() == Q_linear.in_features()) {
            // the three projections in one launch (V compact, [rows x nrow])
            const et_tile_plan *plans[3] = {Q_linear.tile_plan(), K_linear.tile_plan(), V_linear.plan};
            void *ys[3] = {buffers[0], buffers[1], buffers[2]};
            etChk(et_tile_plan_run_multi(plans, ys, 3, in, rows(), stream));
        } else {
            const Linear_tile *qk[2] = {&Q_linear, &K_linear};
            half *outs[2] = {buffers[0], buffers[1]};
            Linear_tile::run_multi(qk, outs, 2, in, rows(), stream);
            V_linear.run_rows(buffers[2], in, rows(), stream);
        }
        // compact V has leading dimension nrow (what the GEMM wrote); the
        // reference passes row_id_size here (encoder/encoder.cu:78) and reads
        // the wrong rows whenever that is not a multiple of 16
        etChk(et_Prune_attention(buffers[3], buffers[0], buffers[1], buffers[2], nullptr, 0,
                                 V_linear.row_id.get(), V_linear.head_ptr.get(), V_linear.nrow,
                                 mask_ptr(), seq_len, d_model, nheads, batch, lens_ptr(), log2_scale,
                                 stream));
        tail(out, in, buffers[3], O_linear, MLP1_linear, MLP2_linear, rows());
    }
};

// Attention-aware pruning carried through the whole layer (no counterpart in
// the reference, which row-prunes only V, encoder/encoder.h:84): Q and K are
// row-pruned to the SAME column set per head, so the scores contract over the
// kept columns only; O, FFN1 and FFN2 are row-pruned too.  A row linear emits
// a compact [rows x nrow] result (kernels/linear.cu:30-32): O's and FFN2's
// are expanded back to model width (pruned columns zero) before the skip
// connection, FFN1's compact hidden feeds an FFN2 whose input columns were
// gathered to match (MLP2.in_feat == MLP1.nrow).
class Encoder_attnaware : public Encoder_base {
  private:
    Linear_row Q_linear, K_linear;
    Linear_tile V_linear;
    Linear_row O_linear, MLP1_linear, MLP2_linear;

  public:
    Encoder_attnaware(int d_model_, int seq_len_, int nheads_, half *buffer_, Linear_row &&Q_linear_,
                      Linear_row &&K_linear_, Linear_tile &&V_linear_, Linear_row &&O_linear_,
                      Linear_row &&MLP1_linear_, Linear_row &&MLP2_linear_, half *ln_gamma_1,
                      half *ln_beta_1, half *ln_gamma_2, half *ln_beta_2, half *mask_, int batch_ = 1)
        : Encoder_base(d_model_, seq_len_, nheads_, buffer_, ln_gamma_1, ln_beta_1, ln_gamma_2,
                       ln_beta_2, mask_, batch_),
          Q_linear(std::move(Q_linear_)), K_linear(std::move(K_linear_)),
          V_linear(std::move(V_linear_)), O_linear(std::move(O_linear_)),
          MLP1_linear(std::move(MLP1_linear_)), MLP2_linear(std::move(MLP2_linear_)) {
        etRequire(Q_linear.row_id_size == K_linear.row_id_size && Q_linear.nrow <= d_model,
                  "Encoder_attnaware: Q and K must keep the same columns");
        etRequire(MLP1_linear.is_gelu, "Encoder_attnaware: MLP1_linear must be the GELU variant");
        etRequire(MLP2_linear.in_feat == MLP1_linear.nrow,
                  "Encoder_attnaware: MLP2 must take MLP1's compact hidden as input");
        etRequire(MLP1_linear.nrow <= 3 * d_model && O_linear.out_feat == d_model && MLP2_linear.out_feat == d_model,
                  "Encoder_attnaware: widths do not fit the workspace");
    }
    void run(half *out, half *in) override {
        const int n = rows();
        if (Q_linear.plan && K_linear.plan && Q_linear.in_feat == V_linear.in_features() &&
            K_linear.in_feat == V_linear.in_features()) {
            // one launch for the three projections (Q and K compact [n x nrow])
            const et_tile_plan *plans[3] = {Q_linear.plan, K_linear.plan, V_linear.tile_plan()};
            void *ys[3] = {buffers[0], buffers[1], buffers[2]};
            etChk(et_tile_plan_run_multi(plans, ys, 3, in, n, stream));
        } else {
            Q_linear.run_rows(buffers[0], in, n, stream); // compact [n x nrow]
            K_linear.run_rows(buffers[1], in, n, stream);
            V_linear.run_rows(buffers[2], in, n, stream);
        }
        if (Q_linear.uniform_head_width == 32 && K_linear.uniform_head_width == 32 && d_model == 64 * nheads)
            // every head keeps 32 of its 64 columns: the on-the-fly kernel with narrow Q/K heads
            etChk(et_OTF_attention_qk_width(buffers[3], buffers[0], buffers[1], buffers[2], mask_ptr(), 32,
                                            seq_len, d_model, nheads, batch, lens_ptr(), log2_scale, stream));
        else
            etChk(et_Prune_attention(buffers[3], buffers[0], buffers[1], buffers[2], Q_linear.head_ptr.get(),
                                     Q_linear.nrow, nullptr, nullptr, d_model, mask_ptr(), seq_len, d_model,
                                     nheads, batch, lens_ptr(), log2_scale, stream));
        O_linear.run_rows(buffers[0], buffers[3], n, stream);
        // expansion to model width, skip connection and LayerNorm in one launch
        O_linear.scatter_skip_layernorm(buffers[1], buffers[0], in, ln_gamma[0].get(), ln_beta[0].get(), n, stream);
        MLP1_linear.run_rows(buffers[2], buffers[1], n, stream); // compact hidden, spans units 2..4
        MLP2_linear.run_rows(buffers[0], buffers[2], n, stream);
        MLP2_linear.scatter_skip_layernorm(out, buffers[0], buffers[1], ln_gamma[1].get(), ln_beta[1].get(), n,
                                           stream);
    }
};

// Sequence-aware encoder (encoder/encoder.h:102-134, encoder/encoder.cu:116-149).
// The reference's version writes scaled Q K^T for all heads to memory and runs
// a second attention kernel on it; that path is kept behind use_shared_qk.
// By default attention is the key-tiled on-the-fly kernel (no seq_len limit),
// and when per-sequence lengths are set the layer runs on the PACKED valid
// rows only: linears and LayerNorms see sum(len) rows, attention walks each
// sequence's own rows, padding rows of `out` are written as zero.
class Encoder_length : public Encoder_base {
  private:
    Linear_tile Q_linear, K_linear, V_linear, O_linear, MLP1_linear, MLP2_linear;
    half *QK_buf;

  public:
    bool use_shared_qk;
    Encoder_length(int d_model_, int seq_len_, int nheads_, half *buffer_, Linear_tile &&Q_linear_,
                   Linear_tile &&K_linear_, Linear_tile &&V_linear_, Linear_tile &&O_linear_,
                   Linear_tile &&MLP1_linear_, Linear_tile &&MLP2_linear_, half *ln_gamma_1,
                   half *ln_beta_1, half *ln_gamma_2, half *ln_beta_2, half *mask_, int batch_ = 1)
        : Encoder_base(d_model_, seq_len_, nheads_, buffer_, ln_gamma_1, ln_beta_1, ln_gamma_2,
                       ln_beta_2, mask_, batch_),
          Q_linear(std::move(Q_linear_)), K_linear(std::move(K_linear_)),
          V_linear(std::move(V_linear_)), O_linear(std::move(O_linear_)),
          MLP1_linear(std::move(MLP1_linear_)), MLP2_linear(std::move(MLP2_linear_)),
          use_shared_qk(false) {
        // after the five activation units (the reference offsets by
        // d_model*nheads*buffer_num, which lands inside them)
        QK_buf = buffer + (size_t)buffer_num * d_model * seq_len * batch;
        etRequire(MLP1_linear.is_gelu, "Encoder_length: MLP1_linear must be the GELU variant");
        place_tail_ws(units_and_scores_bytes(d_model, seq_len, nheads, batch));
        Linear_tile::tail_prepare(O_linear, MLP1_linear, MLP2_linear);
    }
    static size_t units_and_scores_bytes(int d_model_, int seq_len_, int nheads_, int batch_) {
        return ((size_t)buffer_num * d_model_ * seq_len_ + (size_t)nheads_ * seq_len_ * seq_len_) *
               batch_ * sizeof(half);
    }
    static size_t buffer_size(int d_model_, int seq_len_, int nheads_, int batch_ = 1) {
        return align256(units_and_scores_bytes(d_model_, seq_len_, nheads_, batch_)) +
               et_tail_ws_bytes_for(d_model_, batch_ * seq_len_);
    }

    // One layer on packed rows: in_p/out_p are [valid_rows() x d_model] with
    // packed sequence i (batch entry device_pack_order()[i]) at rows
    // cu[i]..cu[i+1]-1; out_p may alias in_p.
    void run_packed(half *out_p, half *in_p) {
        const int n = total_rows;
        const Linear_tile *qkv[3] = {&Q_linear, &K_linear, &V_linear};
        half *outs[3] = {buffers[0], buffers[1], buffers[2]};
        Linear_tile::run_multi(qkv, outs, 3, in_p, n, stream);
        etChk(et_OTF_attention_varlen(buffers[3], buffers[0], buffers[1], buffers[2], mask_ptr(),
                                      d_cu.get(), seq_len, d_model, nheads, batch, log2_scale, stream));
        tail(out_p, in_p, buffers[3], O_linear, MLP1_linear, MLP2_linear, n);
    }

    void run(half *out, half *in) override {
        if (!lens.empty()) {
            // packed input parks in unit 4 (free until FFN1); FFN2 writes its
            // packed result into the front of `out`, the second LayerNorm runs
            // with the operands swapped (a+b == b+a) so its result lands in
            // unit 0, from where it is expanded into `out`.
            const int n = total_rows;
            half *in_p = buffers[4];
            etChk(et_pack_rows_ordered(in_p, in, d_cu.get(), d_order.get(), batch, seq_len, d_model, stream));
            const Linear_tile *qkv[3] = {&Q_linear, &K_linear, &V_linear};
            half *outs[3] = {buffers[0], buffers[1], buffers[2]};
            Linear_tile::run_multi(qkv, outs, 3, in_p, n, stream);
            etChk(et_OTF_attention_varlen(buffers[3], buffers[0], buffers[1], buffers[2], mask_ptr(),
                                          d_cu.get(), seq_len, d_model, nheads, batch, log2_scale, stream));
            if (Linear_tile::tail_fusable(O_linear, MLP1_linear, MLP2_linear)) {
                // steps 6-10 in one launch, straight into unit 0.  (With few rows
                // they run one after the other, in place in unit 0 with the hidden
                // activations in units 1..4: the attention output and the packed
                // input are no longer needed by then.)
                Linear_tile::run_rows_tail(O_linear, MLP1_linear, MLP2_linear, buffers[0], buffers[3], in_p,
                                           buffers[0], buffers[1], ln_gamma[0].get(), ln_beta[0].get(),
                                           ln_gamma[1].get(), ln_beta[1].get(), n, stream, tail_ws, tail_ws_bytes);
                etChk(et_unpack_rows_ordered(out, buffers[0], d_cu.get(), d_order.get(), batch, seq_len, d_model, stream));
                return;
            }
            O_linear.run_rows_ln(buffers[0], buffers[3], in_p, ln_gamma[0].get(), ln_beta[0].get(), n, stream);
            if (Linear_tile::ffn_fusable(MLP1_linear, MLP2_linear) && MLP2_linear.ln_fusable()) {
                // in place over the skip operand: a workgroup reads its rows of
                // unit 0 before it writes them (fused or not, see run_rows_ln)
                Linear_tile::run_rows_ffn_ln(MLP1_linear, MLP2_linear, buffers[0], buffers[0], buffers[1],
                                             buffers[0], ln_gamma[1].get(), ln_beta[1].get(), n, stream);
            } else if (MLP2_linear.ln_fusable()) {
                MLP1_linear.run_rows(buffers[1], buffers[0], n, stream);
                MLP2_linear.run_rows_ln(buffers[0], buffers[1], buffers[0], ln_gamma[1].get(),
                                        ln_beta[1].get(), n, stream);
            } else {
                MLP1_linear.run_rows(buffers[1], buffers[0], n, stream);
                MLP2_linear.run_rows(out, buffers[1], n, stream);
                etChk(et_skip_layernorm(buffers[0], out, ln_gamma[1].get(), ln_beta[1].get(), n, d_model, stream));
            }
            etChk(et_unpack_rows_ordered(out, buffers[0], d_cu.get(), d_order.get(), batch, seq_len, d_model, stream));
            return;
        }
        const Linear_tile *qkv[3] = {&Q_linear, &K_linear, &V_linear};
        half *outs[3] = {buffers[0], buffers[1], buffers[2]};
        Linear_tile::run_multi(qkv, outs, 3, in, rows(), stream);
        if (use_shared_qk) {
            etChk(et_qk_scores(QK_buf, buffers[0], buffers[1], seq_len, d_model, nheads, batch, stream));
            etChk(et_sharedQK_attention(buffers[3], QK_buf, buffers[2], mask_ptr(), seq_len, d_model,
                                        nheads, batch, nullptr, log2_scale, stream));
        } else {
            etChk(et_OTF_attention(buffers[3], buffers[0], buffers[1], buffers[2], mask_ptr(), seq_len,
                                   d_model, nheads, batch, nullptr, log2_scale, stream));
        }
        tail(out, in, buffers[3], O_linear, MLP1_linear, MLP2_linear, rows());
    }
};

// N Encoder_length layers over one workspace for variable-length batches: the
// batch is packed once, every layer runs in place on the packed rows, the
// result is expanded once.  No reference counterpart (it has no batch).
class Encoder_stack {
    std::vector<Encoder_length *> layers;
    int d_model, seq_len, batch;

  public:
    Encoder_stack(std::vector<Encoder_length *> layers_, int d_model_, int seq_len_, int batch_)
        : layers(std::move(layers_)), d_model(d_model_), seq_len(seq_len_), batch(batch_) {}
    // act: device scratch of batch*seq_len*d_model halves (packed activations)
    void run(half *out, half *in, half *act, void *stream) {
        if (layers.empty())
            return;
        for (Encoder_length *l : layers)
            l->set_stream(stream);
        const int *cu = layers[0]->device_cu_seqlens();
        if (!cu) { // full-length batch: layers chain through `act`
            half *cur = in;
            for (size_t i = 0; i < layers.size(); i++) {
                half *dst = (i + 1 == layers.size()) ? out : act;
                layers[i]->run(dst, cur);
                cur = dst;
            }
            return;
        }
        const int *order = layers[0]->device_pack_order();
        etChk(et_pack_rows_ordered(act, in, cu, order, batch, seq_len, d_model, stream));
        for (Encoder_length *l : layers)
            l->run_packed(act, act);
        etChk(et_unpack_rows_ordered(out, act, cu, order, batch, seq_len, d_model, stream));
    }
};
