// C wrappers over the encoder-layer classes (declared in et_encoder.h).
// Exceptions thrown by the classes' error policy are turned into error codes.
#include <memory>
#include <new>

#include "../../include/et_encoder.h"
#include "../encoder/encoder.h"

namespace et {
void set_error(const char *fmt, ...);
}

struct et_linear_tile {
    Linear_tile impl;
};
struct et_linear_row {
    Linear_row impl;
};
struct et_encoder {
    int kind;
    std::unique_ptr<Encoder_base> impl;
};
struct et_encoder_stack {
    std::unique_ptr<Encoder_stack> impl;
};

namespace {
struct ThrowScope { // class errors become exceptions while a C wrapper runs
    bool prev;
    ThrowScope() : prev(et_throw_on_error()) { et_throw_on_error() = true; }
    ~ThrowScope() { et_throw_on_error() = prev; }
};

template <typename F> int guarded(F &&f) {
    ThrowScope scope;
    try {
        f();
        return ET_OK;
    } catch (const std::bad_alloc &) {
        et::set_error("out of host memory");
        return ET_ERR_INVALID_ARG;
    } catch (const std::exception &e) {
        // the class layer already formatted the failing call's message
        et::set_error("%s", e.what());
        return ET_ERR_INVALID_ARG;
    }
}
half *H(const void *p) { return static_cast<half *>(const_cast<void *>(p)); }
int *I(const int *p) { return const_cast<int *>(p); }
} // namespace

extern "C" {

int et_linear_tile_create(et_linear_tile **h, int in_feat, int out_feat, int size, int ntile,
                          const void *data, const int *row_ptr, const int *row_offset,
                          const void *bias, int is_gelu) {
    if (!h) {
        et::set_error("et_linear_tile_create: null out pointer");
        return ET_ERR_INVALID_ARG;
    }
    *h = nullptr;
    return guarded([&] {
        *h = new et_linear_tile{Linear_tile(in_feat, out_feat, size, ntile, H(data), I(row_ptr),
                                            I(row_offset), H(bias), is_gelu != 0)};
    });
}
void et_linear_tile_destroy(et_linear_tile *h) { delete h; }

int et_linear_tile_run(const et_linear_tile *h, void *out, const void *in, void *stream) {
    if (!h) {
        et::set_error("et_linear_tile_run: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] { h->impl.run(H(out), H(in), stream); });
}
int et_linear_tile_run_rows(const et_linear_tile *h, void *out, const void *in, int rows, void *stream) {
    if (!h) {
        et::set_error("et_linear_tile_run_rows: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] { h->impl.run_rows(H(out), H(in), rows, stream); });
}
int et_linear_tile_run_rows_ln(const et_linear_tile *h, void *out, const void *in, const void *skip,
                               const void *gamma, const void *beta, int rows, void *stream) {
    if (!h) {
        et::set_error("et_linear_tile_run_rows_ln: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] {
        h->impl.run_rows_ln(H(out), H(in), static_cast<const half *>(skip), static_cast<const half *>(gamma),
                            static_cast<const half *>(beta), rows, stream);
    });
}
int et_linear_tile_run_rows_ffn_ln(const et_linear_tile *first, const et_linear_tile *second, void *out,
                                   const void *in, void *hidden, const void *skip, const void *gamma,
                                   const void *beta, int rows, void *stream) {
    if (!first || !second) {
        et::set_error("et_linear_tile_run_rows_ffn_ln: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] {
        Linear_tile::run_rows_ffn_ln(first->impl, second->impl, H(out), H(in), H(hidden),
                                     static_cast<const half *>(skip), static_cast<const half *>(gamma),
                                     static_cast<const half *>(beta), rows, stream);
    });
}
int et_linear_tile_run_rows_tail(const et_linear_tile *out_proj, const et_linear_tile *first,
                                 const et_linear_tile *second, void *out, const void *attn, const void *input,
                                 void *mid, void *hidden, const void *gamma1, const void *beta1,
                                 const void *gamma2, const void *beta2, int rows, void *stream) {
    if (!out_proj || !first || !second) {
        et::set_error("et_linear_tile_run_rows_tail: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] {
        Linear_tile::run_rows_tail(out_proj->impl, first->impl, second->impl, H(out), H(attn),
                                   static_cast<const half *>(input), H(mid), H(hidden),
                                   static_cast<const half *>(gamma1), static_cast<const half *>(beta1),
                                   static_cast<const half *>(gamma2), static_cast<const half *>(beta2), rows,
                                   stream);
    });
}
int et_linear_tile_run_rows_tail_ws(const et_linear_tile *out_proj, const et_linear_tile *first,
                                    const et_linear_tile *second, void *out, const void *attn, const void *input,
                                    void *mid, void *hidden, const void *gamma1, const void *beta1,
                                    const void *gamma2, const void *beta2, int rows, void *ws, size_t ws_bytes,
                                    void *stream) {
    if (!out_proj || !first || !second) {
        et::set_error("et_linear_tile_run_rows_tail_ws: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] {
        Linear_tile::run_rows_tail(out_proj->impl, first->impl, second->impl, H(out), H(attn),
                                   static_cast<const half *>(input), H(mid), H(hidden),
                                   static_cast<const half *>(gamma1), static_cast<const half *>(beta1),
                                   static_cast<const half *>(gamma2), static_cast<const half *>(beta2), rows,
                                   stream, ws, ws_bytes);
    });
}
int et_linear_tile_tail_prepare(const et_linear_tile *out_proj, const et_linear_tile *first,
                                const et_linear_tile *second) {
    if (!out_proj || !first || !second) {
        et::set_error("et_linear_tile_tail_prepare: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] { Linear_tile::tail_prepare(out_proj->impl, first->impl, second->impl); });
}
size_t et_linear_tile_tail_ws_bytes(const et_linear_tile *out_proj, const et_linear_tile *first,
                                    const et_linear_tile *second, int rows) {
    return out_proj && first && second ? Linear_tile::tail_ws_bytes(out_proj->impl, first->impl, second->impl, rows)
                                       : 0;
}
int et_linear_tile_tail_fusable(const et_linear_tile *out_proj, const et_linear_tile *first,
                                const et_linear_tile *second) {
    return out_proj && first && second && Linear_tile::tail_fusable(out_proj->impl, first->impl, second->impl)
               ? 1
               : 0;
}
int et_linear_tile_ffn_fusable(const et_linear_tile *first, const et_linear_tile *second) {
    return first && second && Linear_tile::ffn_fusable(first->impl, second->impl) ? 1 : 0;
}
int et_linear_tile_run_multi(const et_linear_tile *const *hs, void *const *outs, int n, const void *in,
                             int rows, void *stream) {
    if (!hs || !outs || n < 1 || n > 4) {
        et::set_error("et_linear_tile_run_multi: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    const Linear_tile *lin[4];
    half *ys[4];
    for (int i = 0; i < n; i++) {
        if (!hs[i]) {
            et::set_error("et_linear_tile_run_multi: null handle %d", i);
            return ET_ERR_INVALID_ARG;
        }
        lin[i] = &hs[i]->impl;
        ys[i] = H(outs[i]);
    }
    return guarded([&] { Linear_tile::run_multi(lin, ys, n, H(in), rows, stream); });
}

int et_linear_row_create(et_linear_row **h, int in_feat, int out_feat, int size, const void *weight,
                         const int *row_id, int row_id_size, const void *bias, int nhead) {
    if (!h || !weight || !row_id || !bias || in_feat <= 0 || out_feat <= 0 || row_id_size <= 0 ||
        nhead <= 0 || out_feat % nhead) {
        et::set_error("et_linear_row_create: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    *h = nullptr;
    for (int i = 0; i < row_id_size; i++)
        if (row_id[i] < 0 || row_id[i] >= out_feat || (i && row_id[i] <= row_id[i - 1])) {
            et::set_error("et_linear_row_create: row_id must be ascending and inside [0,out_feat)");
            return ET_ERR_FORMAT;
        }
    return guarded([&] {
        *h = new et_linear_row{Linear_row(in_feat, out_feat, size, H(weight), I(row_id), row_id_size,
                                          H(bias), nhead)};
    });
}
int et_linear_row_set_gelu(et_linear_row *h, int on) {
    if (!h) {
        et::set_error("et_linear_row_set_gelu: null handle");
        return ET_ERR_INVALID_ARG;
    }
    h->impl.is_gelu = on != 0;
    return ET_OK;
}
void et_linear_row_destroy(et_linear_row *h) { delete h; }
int et_linear_row_run(const et_linear_row *h, void *out, const void *in, void *stream) {
    if (!h) {
        et::set_error("et_linear_row_run: null handle");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] { h->impl.run(H(out), H(in), stream); });
}
int et_linear_row_query(const et_linear_row *h, int *nrow, int *row_id_size, const int **row_id_dev,
                        const int **head_ptr_dev) {
    if (!h) {
        et::set_error("et_linear_row_query: null handle");
        return ET_ERR_INVALID_ARG;
    }
    if (nrow) *nrow = h->impl.nrow;
    if (row_id_size) *row_id_size = h->impl.row_id_size;
    if (row_id_dev) *row_id_dev = h->impl.row_id.get();
    if (head_ptr_dev) *head_ptr_dev = h->impl.head_ptr.get();
    return ET_OK;
}

size_t et_encoder_buffer_size(int kind, int d_model, int seq_len, int nheads, int batch) {
    if (kind == ET_ENCODER_LENGTH)
        return Encoder_length::buffer_size(d_model, seq_len, nheads, batch);
    return Encoder_base::buffer_size(d_model, seq_len, nheads, batch);
}

int et_encoder_create(et_encoder **h, int kind, int d_model, int seq_len, int nheads, int batch,
                      void *buffer, et_linear_tile *q, et_linear_tile *k, void *v, et_linear_tile *o,
                      et_linear_tile *mlp1, et_linear_tile *mlp2, const void *g1, const void *b1,
                      const void *g2, const void *b2, const void *mask) {
    if (!h || !buffer || !q || !k || !v || !o || !mlp1 || !mlp2 || !g1 || !b1 || !g2 || !b2) {
        et::set_error("et_encoder_create: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    if (kind < ET_ENCODER_TILE || kind > ET_ENCODER_LENGTH || d_model <= 0 || seq_len <= 0 ||
        nheads <= 0 || batch <= 0 || d_model % nheads) {
        et::set_error("et_encoder_create: kind=%d d_model=%d seq_len=%d nheads=%d batch=%d", kind,
                      d_model, seq_len, nheads, batch);
        return ET_ERR_INVALID_ARG;
    }
    *h = nullptr;
    const int rc = guarded([&] {
        std::unique_ptr<Encoder_base> e;
        half *buf = static_cast<half *>(buffer);
        if (kind == ET_ENCODER_TILE) {
            auto *vt = static_cast<et_linear_tile *>(v);
            e.reset(new Encoder_tile(d_model, seq_len, nheads, buf, std::move(q->impl), std::move(k->impl),
                                     std::move(vt->impl), std::move(o->impl), std::move(mlp1->impl),
                                     std::move(mlp2->impl), H(g1), H(b1), H(g2), H(b2), H(mask), batch));
        } else if (kind == ET_ENCODER_PRUNE) {
            auto *vr = static_cast<et_linear_row *>(v);
            e.reset(new Encoder_prune(d_model, seq_len, nheads, buf, std::move(q->impl), std::move(k->impl),
                                      std::move(vr->impl), std::move(o->impl), std::move(mlp1->impl),
                                      std::move(mlp2->impl), H(g1), H(b1), H(g2), H(b2), H(mask), batch));
        } else {
            auto *vt = static_cast<et_linear_tile *>(v);
            e.reset(new Encoder_length(d_model, seq_len, nheads, buf, std::move(q->impl), std::move(k->impl),
                                       std::move(vt->impl), std::move(o->impl), std::move(mlp1->impl),
                                       std::move(mlp2->impl), H(g1), H(b1), H(g2), H(b2), H(mask), batch));
        }
        *h = new et_encoder{kind, std::move(e)};
    });
    if (rc == ET_OK) { // the linears were moved in: release the emptied shells
        delete q;
        delete k;
        if (kind == ET_ENCODER_PRUNE)
            delete static_cast<et_linear_row *>(v);
        else
            delete static_cast<et_linear_tile *>(v);
        delete o;
        delete mlp1;
        delete mlp2;
    }
    return rc;
}
int et_encoder_attnaware_create(et_encoder **h, int d_model, int seq_len, int nheads, int batch,
                                void *buffer, et_linear_row *q, et_linear_row *k, et_linear_tile *v,
                                et_linear_row *o, et_linear_row *mlp1, et_linear_row *mlp2, const void *g1,
                                const void *b1, const void *g2, const void *b2, const void *mask) {
    if (!h || !buffer || !q || !k || !v || !o || !mlp1 || !mlp2 || !g1 || !b1 || !g2 || !b2) {
        et::set_error("et_encoder_attnaware_create: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    if (d_model <= 0 || seq_len <= 0 || nheads <= 0 || batch <= 0 || d_model % nheads) {
        et::set_error("et_encoder_attnaware_create: d_model=%d seq_len=%d nheads=%d batch=%d", d_model,
                      seq_len, nheads, batch);
        return ET_ERR_INVALID_ARG;
    }
    *h = nullptr;
    const int rc = guarded([&] {
        std::unique_ptr<Encoder_base> e(new Encoder_attnaware(
            d_model, seq_len, nheads, static_cast<half *>(buffer), std::move(q->impl), std::move(k->impl),
            std::move(v->impl), std::move(o->impl), std::move(mlp1->impl), std::move(mlp2->impl), H(g1), H(b1),
            H(g2), H(b2), H(mask), batch));
        *h = new et_encoder{ET_ENCODER_ATTNAWARE, std::move(e)};
    });
    if (rc == ET_OK) { // the linears were moved in: release the emptied shells
        delete q;
        delete k;
        delete v;
        delete o;
        delete mlp1;
        delete mlp2;
    }
    return rc;
}
void et_encoder_destroy(et_encoder *h) { delete h; }

int et_encoder_run(et_encoder *h, void *out, const void *in) {
    if (!h || !out || !in) {
        et::set_error("et_encoder_run: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] { h->impl->run(H(out), H(in)); });
}
int et_encoder_set_stream(et_encoder *h, void *stream) {
    if (!h)
        return ET_ERR_INVALID_ARG;
    h->impl->set_stream(stream);
    return ET_OK;
}
int et_encoder_set_log2_scale(et_encoder *h, float v) {
    if (!h || !(v > 0.f)) {
        et::set_error("et_encoder_set_log2_scale: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    h->impl->set_log2_scale(v);
    return ET_OK;
}
int et_encoder_set_seq_lens(et_encoder *h, const int *lens) {
    if (!h)
        return ET_ERR_INVALID_ARG;
    return guarded([&] { h->impl->set_seq_lens(lens); });
}
int et_encoder_set_shared_qk(et_encoder *h, int on) {
    if (!h || h->kind != ET_ENCODER_LENGTH) {
        et::set_error("et_encoder_set_shared_qk: needs an ET_ENCODER_LENGTH handle");
        return ET_ERR_INVALID_ARG;
    }
    static_cast<Encoder_length *>(h->impl.get())->use_shared_qk = on != 0;
    return ET_OK;
}

int et_encoder_stack_create(et_encoder_stack **h, et_encoder *const *layers, int n, int d_model,
                            int seq_len, int batch) {
    if (!h || !layers || n <= 0) {
        et::set_error("et_encoder_stack_create: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    *h = nullptr;
    std::vector<Encoder_length *> ls;
    for (int i = 0; i < n; i++) {
        if (!layers[i] || layers[i]->kind != ET_ENCODER_LENGTH) {
            et::set_error("et_encoder_stack_create: layer %d is not an ET_ENCODER_LENGTH encoder", i);
            return ET_ERR_INVALID_ARG;
        }
        ls.push_back(static_cast<Encoder_length *>(layers[i]->impl.get()));
    }
    return guarded([&] {
        *h = new et_encoder_stack{std::unique_ptr<Encoder_stack>(new Encoder_stack(ls, d_model, seq_len, batch))};
    });
}
void et_encoder_stack_destroy(et_encoder_stack *h) { delete h; }
int et_encoder_stack_run(et_encoder_stack *h, void *out, const void *in, void *act, void *stream) {
    if (!h || !out || !in || !act) {
        et::set_error("et_encoder_stack_run: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    return guarded([&] { h->impl->run(H(out), H(in), H(act), stream); });
}

} // extern "C"
