// What the reference's test/gen_linear.cu and the three test mains share, on
// this library: constant-valued pruned linears from the seeded format
// generators, a seeded input, and the output written to a file.
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../encoder/encoder.h"

// test/gen_linear.cu:5-13: every surviving weight and every bias one constant
// (the weights scaled down here so that activations stay well inside half range)
inline Linear_tile gen_tile_linear(int in_feat, int out_feat, int size, float sparsity, uint64_t seed,
                                   bool is_gelu = false, float wval = 0.01f) {
    std::vector<int> row_ptr(out_feat / 16 + 1), row_offset((size_t)(out_feat / 16) * (in_feat / 16));
    const int ntile = et_gen_sparse_tile_mat(out_feat, in_feat, sparsity, seed, row_ptr.data(), row_offset.data());
    etChk(ntile);
    std::vector<half> data((size_t)ntile * 256, (half)wval), bias(out_feat, (half)0.1f);
    return Linear_tile(in_feat, out_feat, size, ntile, data.data(), row_ptr.data(), row_offset.data(), bias.data(),
                       is_gelu);
}

// test/gen_linear.cu:15-24
inline Linear_row gen_row_linear(int in_feat, int out_feat, int size, float sparsity, int nhead, uint64_t seed,
                                 float wval = 0.01f) {
    std::vector<int> row_id(out_feat);
    const int n = et_gen_sparse_row_mat(out_feat, sparsity, seed, row_id.data());
    etChk(n);
    std::vector<half> rows((size_t)n * in_feat, (half)wval), bias(n, (half)0.1f);
    return Linear_row(in_feat, out_feat, size, rows.data(), row_id.data(), n, bias.data(), nhead);
}

struct ExampleArgs {
    const char *out_path;
    int seq_len, batch;
    float sparsity;
};

inline ExampleArgs example_args(int argc, char **argv) {
    if (argc < 2) {
        fprintf(stderr, "usage: %s <out.bin> [seq_len = 128] [batch = 1] [sparsity = 0.8]\n", argv[0]);
        exit(2);
    }
    ExampleArgs a;
    a.out_path = argv[1];
    a.seq_len = argc > 2 ? atoi(argv[2]) : 128;
    a.batch = argc > 3 ? atoi(argv[3]) : 1;
    a.sparsity = argc > 4 ? (float)atof(argv[4]) : 0.8f;
    return a;
}

// device input [rows x width] from a 64-bit LCG, top bits mapped to [-1, 1)
inline half *example_input(size_t n) {
    std::vector<half> h(n);
    uint64_t s = 12345;
    for (size_t i = 0; i < n; i++) {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        h[i] = (half)((float)(s >> 40) * (1.0f / 8388608.0f) - 1.0f);
    }
    half *d;
    etChk(et_malloc((void **)&d, sizeof(half) * n));
    etChk(et_memcpy_h2d(d, h.data(), sizeof(half) * n));
    return d;
}

inline int example_dump(const char *what, const char *path, const half *dev, size_t n) {
    etChk(et_device_synchronize());
    std::vector<half> h(n);
    etChk(et_memcpy_d2h(h.data(), dev, sizeof(half) * n));
    FILE *f = fopen(path, "wb");
    if (!f || fwrite(h.data(), sizeof(half), n, f) != n) {
        fprintf(stderr, "cannot write %s\n", path);
        return 1;
    }
    fclose(f);
    double sum = 0.0;
    for (half v : h)
        sum += (double)(float)v;
    printf("%s: %zu values, checksum %.6f\n", what, n, sum);
    return 0;
}
