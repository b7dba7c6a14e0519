// The reference's smoke program test/tile_test.cu (with test/gen_linear.cu)
// against this library: the same calls on the same classes, built with a plain
// C++ compiler (no HIP headers) and linked with -let_amd.  Where the reference
// leaves its input uninitialised and prints nothing, this one fills the input
// from a seeded generator and writes the layer's output to a file, so that a
// test can compare it with the same layer run through another binding.
//
//   tile_test <out.bin> [seq_len = 128] [batch = 1] [sparsity = 0.8]
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../encoder/encoder.h"

static const int d_model = 768, nhead = 12, d_ff = 3072;

// test/gen_linear.cu:3-13: every surviving weight 0.1, every bias 0.1 (here
// scaled down so that the activations stay well inside half range)
static Linear_tile gen_tile_linear(int in_feat, int out_feat, int size, float sparsity, uint64_t seed, float wval,
                                   bool is_gelu = false) {
    std::vector<int> row_ptr(out_feat / 16 + 1), row_offset((size_t)(out_feat / 16) * (in_feat / 16));
    const int ntile = et_gen_sparse_tile_mat(out_feat, in_feat, sparsity, seed, row_ptr.data(), row_offset.data());
    if (ntile < 0) {
        fprintf(stderr, "et_gen_sparse_tile_mat: %s\n", et_last_error());
        exit(1);
    }
    std::vector<half> data((size_t)ntile * 256, (half)wval), bias(out_feat, (half)0.1f);
    return Linear_tile(in_feat, out_feat, size, ntile, data.data(), row_ptr.data(), row_offset.data(), bias.data(),
                       is_gelu);
}

int main(int argc, char **argv) {
    if (argc < 2) {
        fprintf(stderr, "usage: %s <out.bin> [seq_len] [batch] [sparsity]\n", argv[0]);
        return 2;
    }
    const int seq_len = argc > 2 ? atoi(argv[2]) : 128;
    const int batch = argc > 3 ? atoi(argv[3]) : 1;
    const float sparsity = argc > 4 ? (float)atof(argv[4]) : 0.8f;
    const int rows = seq_len * batch;

    Linear_tile Q = gen_tile_linear(d_model, d_model, rows, sparsity, 1, 0.01f);
    Linear_tile K = gen_tile_linear(d_model, d_model, rows, sparsity, 2, 0.01f);
    Linear_tile V = gen_tile_linear(d_model, d_model, rows, sparsity, 3, 0.01f);
    Linear_tile O = gen_tile_linear(d_model, d_model, rows, sparsity, 4, 0.01f);
    Linear_tile MLP1 = gen_tile_linear(d_model, d_ff, rows, sparsity, 5, 0.01f, true);
    Linear_tile MLP2 = gen_tile_linear(d_ff, d_model, rows, sparsity, 6, 0.01f);

    std::vector<half> gamma(d_model, (half)1.0f), beta(d_model, (half)0.0f);
    std::vector<half> mask((size_t)seq_len * seq_len, (half)0.0f);

    half *buffer, *in;
    etChk(et_malloc((void **)&buffer, Encoder_tile::buffer_size(d_model, seq_len, nhead, batch)));
    etChk(et_malloc((void **)&in, sizeof(half) * (size_t)rows * d_model));
    // input: a 64-bit LCG, top bits mapped to [-1, 1)
    std::vector<half> h_in((size_t)rows * d_model);
    uint64_t s = 12345;
    for (size_t i = 0; i < h_in.size(); i++) {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        h_in[i] = (half)((float)(s >> 40) * (1.0f / 8388608.0f) - 1.0f);
    }
    etChk(et_memcpy_h2d(in, h_in.data(), sizeof(half) * h_in.size()));

    Encoder_tile encoder(d_model, seq_len, nhead, buffer, std::move(Q), std::move(K), std::move(V), std::move(O),
                         std::move(MLP1), std::move(MLP2), gamma.data(), beta.data(), gamma.data(), beta.data(),
                         mask.data(), batch);
    encoder.run(in, in); // as test/tile_test.cu:41
    etChk(et_device_synchronize());

    std::vector<half> h_out(h_in.size());
    etChk(et_memcpy_d2h(h_out.data(), in, sizeof(half) * h_out.size()));
    FILE *f = fopen(argv[1], "wb");
    if (!f || fwrite(h_out.data(), sizeof(half), h_out.size(), f) != h_out.size()) {
        fprintf(stderr, "cannot write %s\n", argv[1]);
        return 1;
    }
    fclose(f);
    double sum = 0.0;
    for (half v : h_out)
        sum += (double)(float)v;
    printf("tile_test: %d rows x %d, sparsity %.2f, output checksum %.6f\n", rows, d_model, sparsity, sum);
    et_free(in);
    et_free(buffer);
    return 0;
}
