// The reference's smoke program test/tile_test.cu against this library: the
// same calls on the same classes, built with a plain C++ compiler (no HIP
// headers) and linked with -let_amd.  Where the reference leaves its input
// uninitialised and prints nothing, this one fills the input from a seeded
// generator and writes the layer's output to a file, so that a test can
// compare it with the same layer run through another binding.
//
//   tile_test <out.bin> [seq_len = 128] [batch = 1] [sparsity = 0.8]
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

    half *buffer;
    etChk(et_malloc((void **)&buffer, Encoder_tile::buffer_size(d_model, a.seq_len, nhead, a.batch)));
    half *in = example_input((size_t)rows * d_model);
    Encoder_tile encoder(d_model, a.seq_len, nhead, buffer, std::move(Q), std::move(K), std::move(V), std::move(O),
                         std::move(MLP1), std::move(MLP2), gamma.data(), beta.data(), gamma.data(), beta.data(),
                         mask.data(), a.batch);
    encoder.run(in, in); // as test/tile_test.cu:41
    const int rc = example_dump("tile_test", a.out_path, in, (size_t)rows * d_model);
    et_free(in);
    et_free(buffer);
    return rc;
}
