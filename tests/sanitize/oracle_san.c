/* Host AddressSanitizer / UBSan driver for the CPU oracle (oracle/et_oracle.c): one small pass through
 * every exported function with arrays of exactly the documented sizes.  Built by `make -C oracle asan`,
 * run by tests/test_sanitize.py.  CPU only. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef uint16_t h16;
int orc_gen_sparse_tile_mat(int, int, float, uint64_t, int *, int *);
int orc_gen_sparse_row_mat(int, float, uint64_t, int *);
void orc_gen_head_balanced_rows(int, int, int, uint64_t, int *);
void orc_head_ptr(const int *, int, int, int, int *);
void orc_tile_pack(const h16 *, int, int, const int *, const int *, h16 *);
void orc_tile_unpack(h16 *, int, int, const int *, const int *, const h16 *);
int orc_tile_mat_validate(int, int, int, const int *, const int *);
void orc_gelu(const h16 *, h16 *, long);
int orc_prune_tile_mat(const h16 *, int, int, float, int *, int *);
int orc_prune_row_mat(const h16 *, int, int, float, int *);
void orc_f2h(const float *, h16 *, long);
void orc_h2f(const h16 *, float *, long);
void orc_tile_linear_f32(h16 *, const h16 *, const int *, const int *, const h16 *, const h16 *, int, int, int, int);
void orc_row_linear_f64(h16 *, const h16 *, const h16 *, const h16 *, int, int, int);
void orc_skip_layernorm_f32(h16 *, const h16 *, const h16 *, const h16 *, int, int);
void orc_otf_attention_f32(h16 *, const h16 *, const h16 *, const h16 *, const h16 *, int, int, int, int, const int *,
                           float);
void orc_encoder_tile_layer_f32(h16 *, const h16 *, h16 *, const int *const *, const int *const *,
                                const h16 *const *, const h16 *const *, const h16 *, const h16 *, const h16 *,
                                const h16 *, const h16 *, int, int, int, int, int, const int *, float);

static h16 *halves(long n, unsigned seed, float scale) {
    float *f = (float *)malloc(sizeof(float) * (size_t)n);
    h16 *h = (h16 *)malloc(sizeof(h16) * (size_t)n);
    for (long i = 0; i < n; i++) {
        seed = seed * 1664525u + 1013904223u;
        f[i] = ((int)(seed >> 9) % 2001 - 1000) * 0.001f * scale;
    }
    orc_f2h(f, h, n);
    free(f);
    return h;
}

int main(void) {
    const int d = 64, dff = 128, S = 32, H = 2, B = 2, rows = S * B;
    int fail = 0;
    /* six linears of a small layer at 50 % */
    const int shapes[6][2] = {{d, d}, {d, d}, {d, d}, {d, d}, {dff, d}, {d, dff}};
    int *rp[6], *ro[6];
    h16 *data[6], *bias[6];
    for (int j = 0; j < 6; j++) {
        const int N = shapes[j][0], K = shapes[j][1];
        rp[j] = (int *)malloc(sizeof(int) * (size_t)(N / 16 + 1));
        int *cap = (int *)malloc(sizeof(int) * (size_t)((N / 16) * (K / 16)));
        const int nt = orc_gen_sparse_tile_mat(N, K, 0.5f, 10 + j, rp[j], cap);
        ro[j] = (int *)malloc(sizeof(int) * (size_t)nt); /* exactly ntile entries */
        memcpy(ro[j], cap, sizeof(int) * (size_t)nt);
        free(cap);
        fail += orc_tile_mat_validate(N, K, nt, rp[j], ro[j]) != 0;
        h16 *W = halves((long)N * K, 3 + j, 0.05f);
        data[j] = (h16 *)malloc(sizeof(h16) * (size_t)nt * 256);
        orc_tile_pack(W, N, K, rp[j], ro[j], data[j]);
        h16 *back = (h16 *)malloc(sizeof(h16) * (size_t)N * K);
        orc_tile_unpack(back, N, K, rp[j], ro[j], data[j]);
        free(back);
        free(W);
        bias[j] = halves(N, 40 + j, 0.1f);
    }
    h16 *x = halves((long)rows * d, 99, 1.0f), *mask = halves((long)S * S, 98, 0.5f);
    h16 *g1 = halves(d, 1, 1.0f), *b1 = halves(d, 2, 0.1f), *g2 = halves(d, 3, 1.0f), *b2 = halves(d, 4, 0.1f);
    h16 *out = (h16 *)malloc(sizeof(h16) * (size_t)rows * d);
    h16 *ws = (h16 *)malloc(sizeof(h16) * ((size_t)4 * rows * d + (size_t)rows * dff));
    const int lens[2] = {32, 9};
    orc_encoder_tile_layer_f32(out, x, ws, (const int *const *)rp, (const int *const *)ro, (const h16 *const *)data,
                               (const h16 *const *)bias, g1, b1, g2, b2, mask, S, d, H, dff, B, lens, 1.0f);
    float *of = (float *)malloc(sizeof(float) * (size_t)rows * d);
    orc_h2f(out, of, (long)rows * d);
    for (int b = 0; b < B; b++)
        for (int t = 0; t < lens[b]; t++)
            for (int c = 0; c < d; c++)
                fail += !isfinite(of[((size_t)b * S + t) * d + c]);
    /* the remaining entry points on their own */
    h16 *y = (h16 *)malloc(sizeof(h16) * (size_t)rows * dff);
    orc_tile_linear_f32(y, x, rp[4], ro[4], data[4], bias[4], rows, dff, d, 1);
    h16 *Wd = halves((long)48 * d, 7, 0.05f), *bd = halves(48, 8, 0.1f);
    orc_row_linear_f64(y, x, Wd, bd, rows, 48, d);
    orc_skip_layernorm_f32(out, x, g1, b1, rows, d);
    orc_otf_attention_f32(out, x, x, x, NULL, S, d, H, B, NULL, 1.44269504f);
    orc_gelu(x, out, (long)rows * d);
    int ids[64], hp[3], bal[2 * 8], prp[64 / 16 + 1], pro[16];
    const int nr = orc_gen_sparse_row_mat(d, 0.7f, 5, ids);
    orc_head_ptr(ids, nr, H, d / H, hp);
    fail += hp[H] != nr;
    orc_gen_head_balanced_rows(H, d / H, 8, 6, bal);
    h16 *Wp = halves((long)d * d, 11, 0.1f);
    fail += orc_prune_tile_mat(Wp, d, d, 0.5f, prp, pro) != 8;
    fail += orc_prune_row_mat(Wp, d, d, 0.75f, ids) != 16;
    if (fail) {
        fprintf(stderr, "oracle_san: %d checks failed\n", fail);
        return 1;
    }
    puts("oracle_san: ok");
    return 0;
}
