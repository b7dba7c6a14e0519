// The reference's test/length_test.cu against this library (see tile_test.cpp),
// followed by what the reference's sequence-aware encoder does not have: the
// same batch with per-sequence lengths (sequence b keeps seq_len - 7 b rows),
// run on the packed valid rows.  Both outputs go to the file, one after the other.
//
//   length_test <out.bin> [seq_len = 128] [batch = 1] [sparsity = 0.8]
#include "gen_linear.h"

int main(int argc, char **argv) {
    const ExampleArgs a = example_args(argc, argv);
    const int d_model = 768, nhead = 12, rows = a.seq_len * a.batch;
    Linear_tile Q = gen_tile_linear(d_model, d_model, rows, a.sparsity, 1);
    Linear_tile K = gen_tile_linear(d_model, d_model, rows, a.sparsity, 2);
    Linear_tile V = gen_tile_linear(d_model, d_model, rows, a.sparsity, 3);
    Linear_tile O = gen_tile_linear(d_model, d_model, rows, a.sparsity, 4);
    Linear_tile MLP1 = gen_tile_linear(d_model, d_model * 4, rows, a.sparsity, 5, true);
    Linear_tile MLP2 = gen_tile_linear(d_model * 4, d_model, rows, a.sparsity, 6);
    std::vector<half> gamma(d_model, (half)1.0f), beta(d_model, (half)0.0f);
    std::vector<half> mask((size_t)a.seq_len * a.seq_len, (half)0.0f);

    half *buffer, *out;
    etChk(et_malloc((void **)&buffer, Encoder_length::buffer_size(d_model, a.seq_len, nhead, a.batch)));
    etChk(et_malloc((void **)&out, sizeof(half) * (size_t)2 * rows * d_model));
    half *in = example_input((size_t)rows * d_model);
    Encoder_length encoder(d_model, a.seq_len, nhead, buffer, std::move(Q), std::move(K), std::move(V), std::move(O),
                           std::move(MLP1), std::move(MLP2), gamma.data(), beta.data(), gamma.data(), beta.data(),
                           mask.data(), a.batch);
    encoder.run(out, in); // test/length_test.cu:38 (there in place)
    std::vector<int> lens(a.batch);
    for (int b = 0; b < a.batch; b++)
        lens[b] = a.seq_len - 7 * b > 1 ? a.seq_len - 7 * b : 1;
    encoder.set_seq_lens(lens.data());
    encoder.run(out + (size_t)rows * d_model, in);
    const int rc = example_dump("length_test", a.out_path, out, (size_t)2 * rows * d_model);
    et_free(in);
    et_free(out);
    et_free(buffer);
    return rc;
}
