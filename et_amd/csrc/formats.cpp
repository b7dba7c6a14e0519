// Host-side pruned-weight formats: seeded tile_mat / row_mat index generation,
// validation and packing.  Independent of the device code (plain C++).
//
// The reference generates the index arrays with the unseeded
// std::random_shuffle (test/tile_mat.cu:16, test/row_mat.cu:11).  Here the
// selection is driven by splitmix64 + a descending Fisher-Yates pass so that a
// (shape, sparsity, seed) triple always names the same pruning mask; everything
// else — how many tiles survive, how a block-row lists them, what row_offset
// means — is the reference's.
#include <algorithm>
#include <cstring>
#include <vector>

#include "../../include/et_amd.h"

namespace et {
void set_error(const char *fmt, ...);
}

namespace {

struct SplitMix64 {
    uint64_t s;
    uint64_t next() {
        uint64_t z = (s += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
};

void fisher_yates(std::vector<int> &v, uint64_t seed) {
    SplitMix64 g{seed};
    for (size_t i = v.size(); i-- > 1;) {
        const size_t j = (size_t)(g.next() % (uint64_t)(i + 1));
        std::swap(v[i], v[j]);
    }
}

} // namespace

extern "C" int et_gen_sparse_tile_mat(int nrow, int ncol, float sparsity, uint64_t seed,
                                      int *row_ptr, int *row_offset) {
    if (!row_ptr || nrow <= 0 || ncol <= 0 || nrow % 16 || ncol % 16 || !(sparsity >= 0.f) ||
        !(sparsity <= 1.f)) {
        et::set_error("et_gen_sparse_tile_mat: nrow=%d ncol=%d sparsity=%f", nrow, ncol, (double)sparsity);
        return ET_ERR_INVALID_ARG;
    }
    const int brows = nrow / 16, bcols = ncol / 16;
    const int total = brows * bcols;
    // truncation of a double product, as test/tile_mat.cu:10-11
    const int ntile = (int)(total * (1.0 - (double)sparsity));
    if (ntile > 0 && !row_offset) {
        et::set_error("et_gen_sparse_tile_mat: null row_offset");
        return ET_ERR_INVALID_ARG;
    }
    std::vector<int> tiles(total);
    for (int t = 0; t < total; t++)
        tiles[t] = t; // row-major over the tile grid: t = y*bcols + x
    fisher_yates(tiles, seed);
    // bucket the kept tiles by block-row, preserving shuffle order
    std::vector<int> count(brows + 1, 0);
    for (int i = 0; i < ntile; i++)
        count[tiles[i] / bcols + 1]++;
    for (int r = 0; r < brows; r++)
        count[r + 1] += count[r];
    for (int r = 0; r <= brows; r++)
        row_ptr[r] = count[r];
    std::vector<int> cursor(count.begin(), count.end() - 1);
    for (int i = 0; i < ntile; i++) {
        const int y = tiles[i] / bcols, x = tiles[i] % bcols;
        row_offset[cursor[y]++] = x * 16;
    }
    return ntile;
}

extern "C" int et_gen_sparse_row_mat(int nrow, float sparsity, uint64_t seed, int *row_id) {
    if (!row_id || nrow <= 0 || !(sparsity >= 0.f) || !(sparsity <= 1.f)) {
        et::set_error("et_gen_sparse_row_mat: nrow=%d sparsity=%f", nrow, (double)sparsity);
        return ET_ERR_INVALID_ARG;
    }
    const int keep = (int)(nrow * (1.0 - (double)sparsity)); // test/row_mat.cu:7
    std::vector<int> ids(nrow);
    for (int i = 0; i < nrow; i++)
        ids[i] = i;
    fisher_yates(ids, seed);
    std::sort(ids.begin(), ids.begin() + keep);
    std::copy(ids.begin(), ids.begin() + keep, row_id);
    return keep;
}

extern "C" int et_gen_head_balanced_rows(int nhead, int head_dim, int keep, uint64_t seed,
                                         int *row_id) {
    if (!row_id || nhead <= 0 || head_dim <= 0 || keep < 0 || keep > head_dim) {
        et::set_error("et_gen_head_balanced_rows: nhead=%d head_dim=%d keep=%d", nhead, head_dim, keep);
        return ET_ERR_INVALID_ARG;
    }
    std::vector<int> ids(head_dim);
    for (int h = 0; h < nhead; h++) {
        for (int i = 0; i < head_dim; i++)
            ids[i] = i;
        fisher_yates(ids, seed + 0x1000003ull * (uint64_t)(h + 1));
        std::sort(ids.begin(), ids.begin() + keep);
        for (int i = 0; i < keep; i++)
            row_id[h * keep + i] = h * head_dim + ids[i];
    }
    return ET_OK;
}

extern "C" int et_tile_mat_validate(int N, int K, int ntile, const int *row_ptr,
                                    const int *row_offset) {
    if (N <= 0 || K <= 0 || N % 16 || K % 16 || !row_ptr || ntile < 0 || (ntile > 0 && !row_offset))
        return -1;
    const int nbr = N / 16;
    if (row_ptr[0] != 0)
        return -2;
    for (int r = 0; r < nbr; r++)
        if (row_ptr[r + 1] < row_ptr[r])
            return -3;
    if (row_ptr[nbr] != ntile)
        return -4;
    std::vector<char> seen(K / 16);
    for (int r = 0; r < nbr; r++) {
        std::fill(seen.begin(), seen.end(), 0);
        for (int i = row_ptr[r]; i < row_ptr[r + 1]; i++) {
            const int o = row_offset[i];
            if (o < 0 || o + 16 > K || o % 16)
                return -5;
            if (seen[o / 16])
                return -6;
            seen[o / 16] = 1;
        }
    }
    return 0;
}

extern "C" int et_tile_pack(const void *W, int N, int K, const int *row_ptr, const int *row_offset,
                            void *data) {
    if (!W || !row_ptr || N <= 0 || K <= 0 || N % 16 || K % 16) {
        et::set_error("et_tile_pack: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    const uint16_t *w = static_cast<const uint16_t *>(W);
    uint16_t *d = static_cast<uint16_t *>(data);
    for (int bn = 0; bn < N / 16; bn++)
        for (int i = row_ptr[bn]; i < row_ptr[bn + 1]; i++)
            for (int n = 0; n < 16; n++)
                memcpy(d + (size_t)i * 256 + n * 16, w + (size_t)(bn * 16 + n) * K + row_offset[i], 32);
    return ET_OK;
}

extern "C" int et_head_ptr(const int *row_id, int n, int nhead, int head_dim, int *head_ptr) {
    if (!head_ptr || nhead <= 0 || head_dim <= 0 || n < 0 || (n > 0 && !row_id)) {
        et::set_error("et_head_ptr: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    for (int h = 0; h <= nhead; h++)
        head_ptr[h] = (int)(std::lower_bound(row_id, row_id + n, h * head_dim) - row_id);
    head_ptr[nhead] = n;
    return ET_OK;
}
