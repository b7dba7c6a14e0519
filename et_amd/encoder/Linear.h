// Pruned-weight linear operators.  Same names, constructor arguments and run()
// meaning as encoder/Linear.h of the reference; the device work goes through
// the C ABI (et_amd.h).
#pragma once
#include <algorithm>
#include <utility>
#include <vector>

#include "utils.h"

// Tensor-tile pruned linear: Y = X W^T + b with W as tile_mat
// (encoder/Linear.h:4-46).  All constructor pointers are HOST memory.
class Linear_tile {
  private:
    int in_feat;
    int out_feat;
    int size; // rows of X this operator is applied to (batch * seq_len)
    et_tile_plan *plan;

  public:
    const bool is_gelu;
    Linear_tile(int in_feat_, int out_feat_, int size_, int ntile, half *data_, int *row_ptr_,
                int *row_offset_, half *bias_, bool is_gelu_ = false)
        : in_feat(in_feat_), out_feat(out_feat_), size(size_), plan(nullptr), is_gelu(is_gelu_) {
        etChk(et_tile_plan_create(&plan, in_feat_, out_feat_, ntile, data_, row_ptr_, row_offset_, bias_));
    }
    Linear_tile(const Linear_tile &) = delete;
    Linear_tile &operator=(const Linear_tile &) = delete;
    Linear_tile(Linear_tile &&other) noexcept
        : in_feat(other.in_feat), out_feat(other.out_feat), size(other.size), plan(other.plan),
          is_gelu(other.is_gelu) {
        other.plan = nullptr;
    }
    ~Linear_tile() { et_tile_plan_destroy(plan); }

    // encoder/Linear.h:36-45; `stream` is a hipStream_t (NULL = default stream)
    void run(half *out, half *in, void *stream) const {
        etChk(et_tile_plan_run(plan, out, in, size, is_gelu ? 1 : 0, stream));
    }
    // same operator on a different row count (variable-length batches)
    void run_rows(half *out, half *in, int rows, void *stream) const {
        etChk(et_tile_plan_run(plan, out, in, rows, is_gelu ? 1 : 0, stream));
    }
    // several linears over the same input in one launch (Q, K, V)
    // this linear, the skip connection and LayerNorm in one launch:
    // out = LayerNorm(half(linear(in)) + skip); see et_tile_plan_run_ln
    void run_rows_ln(half *out, half *in, const half *skip, const half *gamma, const half *beta,
                     int rows, void *stream) const {
        etRequire(!is_gelu, "Linear_tile::run_rows_ln: not available for the GELU linear");
        etChk(et_tile_plan_run_ln(plan, out, in, skip, gamma, beta, rows, stream));
    }
    bool ln_fusable() const { return et_tile_plan_ln_fusable(plan) != 0; }

    // the feed-forward block in one launch: out = LayerNorm(half(second(gelu(first(in)))) + skip);
    // `hidden` ([rows x first.out_feat]) is used only where the fused kernel does
    // not apply or does not pay; see et_tile_plan_run_ffn_ln
    static void run_rows_ffn_ln(const Linear_tile &first, const Linear_tile &second, half *out, half *in,
                                half *hidden, const half *skip, const half *gamma, const half *beta,
                                int rows, void *stream) {
        etRequire(first.is_gelu && !second.is_gelu,
                  "Linear_tile::run_rows_ffn_ln: the first linear must be the GELU variant, the second not");
        etChk(et_tile_plan_run_ffn_ln(first.plan, second.plan, out, in, hidden, skip, gamma, beta, rows,
                                      stream));
    }
    static bool ffn_fusable(const Linear_tile &first, const Linear_tile &second) {
        return et_tile_plan_ffn_fusable(first.plan, second.plan) != 0;
    }

    // steps 6-10 of a layer (encoder/encoder.cu:33-44) in one launch; `mid`
    // ([rows x model width]) and `hidden` are used only where the fused kernel
    // does not apply or does not pay; see et_tile_plan_run_tail
    static void run_rows_tail(const Linear_tile &out_proj, const Linear_tile &first, const Linear_tile &second,
                              half *out, half *attn, const half *input, half *mid, half *hidden,
                              const half *gamma1, const half *beta1, const half *gamma2, const half *beta2,
                              int rows, void *stream, void *ws = nullptr, size_t ws_bytes = 0) {
        etRequire(!out_proj.is_gelu && first.is_gelu && !second.is_gelu,
                  "Linear_tile::run_rows_tail: only the first feed-forward linear is the GELU variant");
        // with scratch (`ws`, tail_ws_bytes()) the launch may take the form of pairs of
        // workgroups over 64-row panels; see et_tile_plan_run_tail_ws
        etChk(et_tile_plan_run_tail_ws(out_proj.plan, first.plan, second.plan, out, attn, input, mid, hidden,
                                       gamma1, beta1, gamma2, beta2, rows, ws, ws_bytes, stream));
    }
    // builds what run_rows_tail with scratch needs (device allocations: not inside a run)
    static void tail_prepare(const Linear_tile &out_proj, const Linear_tile &first, const Linear_tile &second) {
        etChk(et_tile_plan_tail_prepare(out_proj.plan, first.plan, second.plan));
    }
    static size_t tail_ws_bytes(const Linear_tile &out_proj, const Linear_tile &first, const Linear_tile &second,
                                int rows) {
        return et_tile_plan_tail_ws_bytes(out_proj.plan, first.plan, second.plan, rows);
    }
    static bool tail_fusable(const Linear_tile &out_proj, const Linear_tile &first, const Linear_tile &second) {
        return et_tile_plan_tail_fusable(out_proj.plan, first.plan, second.plan) != 0;
    }

    static void run_multi(const Linear_tile *const *lin, half *const *outs, int n, half *in, int rows,
                          void *stream) {
        const et_tile_plan *plans[4];
        void *ys[4];
        for (int i = 0; i < n && i < 4; i++) {
            plans[i] = lin[i]->plan;
            ys[i] = outs[i];
        }
        etChk(et_tile_plan_run_multi(plans, ys, n, in, rows, stream));
    }
    const et_tile_plan *tile_plan() const { return plan; } // for et_tile_plan_run_multi with other plans
    int rows() const { return size; }
    int in_features() const { return in_feat; }
    int out_features() const { return out_feat; }
};

// Row-pruned linear on compacted rows (encoder/Linear.h:48-72,
// encoder/Linear.cu:60-91).  Output is compact: [size x nrow].
class Linear_row {
  public:
    int in_feat;
    int out_feat;
    int size;
    int nhead;
    Weight<half> weight; // [nrow x in_feat], rows beyond row_id_size are zero
    Weight<int> row_id;  // sorted outside
    Weight<int> head_ptr;
    int nrow;        // row_id_size rounded up to a multiple of 16
    int row_id_size; // surviving rows
    Weight<half> bias;
    bool is_gelu;    // added: GELU on the compact output (a row-pruned FFN1)
    // the compact rows as a fully populated tile_mat: the planned tile kernels
    // (panel in LDS, pipelined weight stream) then serve the dense product too;
    // null when in_feat is not a multiple of 16
    et_tile_plan *plan;
    // kept rows per head where every head keeps the same number and no padding
    // row exists (head h is then columns h*w .. of the compact output), else 0
    int uniform_head_width;

    static int multiple_16(int x) { return ((x + 15) / 16) * 16; }

    // weight_: HOST [row_id_size_ x in_feat_]; row_id_: HOST, ascending; bias_: HOST [row_id_size_]
    Linear_row(int in_feat_, int out_feat_, int size_, half *weight_, int *row_id_, int row_id_size_,
               half *bias_, int nhead_, bool is_gelu_ = false)
        : in_feat(in_feat_), out_feat(out_feat_), size(size_), nhead(nhead_),
          weight(in_feat_ * multiple_16(row_id_size_)), row_id(row_id_, row_id_size_ > 0 ? row_id_size_ : 1),
          head_ptr(nhead_ + 1), nrow(multiple_16(row_id_size_)), row_id_size(row_id_size_),
          bias(multiple_16(row_id_size_)), is_gelu(is_gelu_), plan(nullptr), uniform_head_width(0) {
        // padded rows must contribute nothing: zero the buffers first
        etChk(et_fill_zero(weight.get(), sizeof(half) * (size_t)in_feat * nrow, nullptr));
        etChk(et_fill_zero(bias.get(), sizeof(half) * (size_t)nrow, nullptr));
        etChk(et_device_synchronize());
        etChk(et_memcpy_h2d(weight.get(), weight_, sizeof(half) * (size_t)in_feat * row_id_size));
        etChk(et_memcpy_h2d(bias.get(), bias_, sizeof(half) * (size_t)row_id_size));
        std::vector<int> h_head_ptr(nhead + 1);
        etChk(et_head_ptr(row_id_, row_id_size, nhead, out_feat / nhead, h_head_ptr.data()));
        head_ptr.set(h_head_ptr.data());
        if (nhead > 0 && row_id_size == nrow && row_id_size % nhead == 0) {
            uniform_head_width = row_id_size / nhead;
            for (int h = 0; h <= nhead; h++)
                if (h_head_ptr[h] != h * uniform_head_width)
                    uniform_head_width = 0;
        }
        if (in_feat % 16 == 0) {
            const int bcols = in_feat / 16, brows = nrow / 16;
            std::vector<half> wpad((size_t)nrow * in_feat), bpad(nrow); // (value-initialised: zero)
            std::copy(weight_, weight_ + (size_t)row_id_size * in_feat, wpad.begin());
            std::copy(bias_, bias_ + row_id_size, bpad.begin());
            std::vector<int> rp(brows + 1), ro((size_t)brows * bcols);
            for (int y = 0; y <= brows; y++)
                rp[y] = y * bcols;
            for (int y = 0; y < brows; y++)
                for (int x = 0; x < bcols; x++)
                    ro[(size_t)y * bcols + x] = x * 16;
            std::vector<half> data((size_t)brows * bcols * 256);
            etChk(et_tile_pack(wpad.data(), nrow, in_feat, rp.data(), ro.data(), data.data()));
            etChk(et_tile_plan_create(&plan, in_feat, nrow, brows * bcols, data.data(), rp.data(), ro.data(),
                                      bpad.data()));
        }
    }
    Linear_row(Linear_row &&o) noexcept
        : in_feat(o.in_feat), out_feat(o.out_feat), size(o.size), nhead(o.nhead), weight(std::move(o.weight)),
          row_id(std::move(o.row_id)), head_ptr(std::move(o.head_ptr)), nrow(o.nrow),
          row_id_size(o.row_id_size), bias(std::move(o.bias)), is_gelu(o.is_gelu), plan(o.plan),
          uniform_head_width(o.uniform_head_width) {
        o.plan = nullptr;
    }
    Linear_row(const Linear_row &) = delete;
    ~Linear_row() { et_tile_plan_destroy(plan); }

    // encoder/Linear.h:68-71; the cuBLAS handle becomes a stream
    void run(half *out, half *in, void *stream) const { run_rows(out, in, size, stream); }
    void run_rows(half *out, half *in, int rows, void *stream) const {
        if (plan)
            etChk(et_tile_plan_run(plan, out, in, rows, is_gelu ? 1 : 0, stream));
        else if (is_gelu)
            etChk(et_row_spmm_add_bias_gelu(out, in, weight.get(), bias.get(), rows, nrow, in_feat, stream));
        else
            etChk(et_row_spmm_add_bias(out, in, weight.get(), bias.get(), rows, nrow, in_feat, stream));
    }
    // out[rows x out_feat] = the compact result expanded to model width, pruned columns zero
    void scatter(half *out, const half *compact, int rows, void *stream) const {
        etChk(et_scatter_cols(out, compact, row_id.get(), rows, row_id_size, nrow, out_feat, stream));
    }
    // out = LayerNorm(scatter(compact) + skip) in one launch; out may alias skip
    void scatter_skip_layernorm(half *out, const half *compact, const half *skip, const half *gamma,
                                const half *beta, int rows, void *stream) const {
        etChk(et_scatter_skip_layernorm(out, compact, row_id.get(), row_id_size, nrow, skip, gamma, beta, rows,
                                        out_feat, stream));
    }
};
