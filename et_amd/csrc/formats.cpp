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
#include <cstdio>
#include <cstring>
#include <string>
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

// ---------------------------------------------------------------------------
// Magnitude-based pruning: keep the tiles / rows of a dense W with the largest
// L2 norm.  (The reference only selects at random, test/tile_mat.cu:16,
// test/row_mat.cu:11; how many survive and how they are listed is unchanged.)
// ---------------------------------------------------------------------------
namespace {

// IEEE binary16 -> double, exact
double half_to_double(uint16_t h) {
    const int sign = h >> 15, e = (h >> 10) & 31, m = h & 1023;
    double v;
    if (e == 0)
        v = m * (1.0 / 16777216.0); // subnormal: m * 2^-24
    else if (e == 31)
        v = m ? 0.0 : 65536.0 * 65536.0; // NaN counts as 0, Inf as huge
    else {
        v = (double)(1024 + m);
        int sh = e - 25;
        while (sh > 0) { v *= 2.0; sh--; }
        while (sh < 0) { v *= 0.5; sh++; }
    }
    return sign ? -v : v;
}

// indices 0..n-1 ordered by (key descending, index ascending), first `keep`
std::vector<int> top_by_key(const std::vector<double> &key, int keep) {
    std::vector<int> idx(key.size());
    for (size_t i = 0; i < idx.size(); i++)
        idx[i] = (int)i;
    auto before = [&](int a, int b) { return key[a] > key[b] || (key[a] == key[b] && a < b); };
    if (keep < (int)idx.size())
        std::nth_element(idx.begin(), idx.begin() + keep, idx.end(), before);
    idx.resize(keep);
    return idx;
}

} // namespace

extern "C" int et_prune_tile_mat(const void *W, int N, int K, float sparsity, int *row_ptr,
                                 int *row_offset) {
    if (!W || !row_ptr || N <= 0 || K <= 0 || N % 16 || K % 16 || !(sparsity >= 0.f) || !(sparsity <= 1.f)) {
        et::set_error("et_prune_tile_mat: N=%d K=%d sparsity=%f", N, K, (double)sparsity);
        return ET_ERR_INVALID_ARG;
    }
    const int brows = N / 16, bcols = K / 16, total = brows * bcols;
    const int ntile = (int)(total * (1.0 - (double)sparsity)); // as test/tile_mat.cu:10-11
    if (ntile > 0 && !row_offset) {
        et::set_error("et_prune_tile_mat: null row_offset");
        return ET_ERR_INVALID_ARG;
    }
    const uint16_t *w = static_cast<const uint16_t *>(W);
    std::vector<double> norm2(total);
    for (int t = 0; t < total; t++) {
        const int y = t / bcols, x = t % bcols;
        double acc = 0.0; // row-major over the tile, in double
        for (int n = 0; n < 16; n++)
            for (int k = 0; k < 16; k++) {
                const double v = half_to_double(w[(size_t)(y * 16 + n) * K + x * 16 + k]);
                acc += v * v;
            }
        norm2[t] = acc;
    }
    std::vector<int> kept = top_by_key(norm2, ntile);
    std::sort(kept.begin(), kept.end()); // row-major: block-row, then column
    int pos = 0;
    for (int y = 0; y < brows; y++) {
        row_ptr[y] = pos;
        while (pos < ntile && kept[pos] / bcols == y) {
            row_offset[pos] = (kept[pos] % bcols) * 16;
            pos++;
        }
    }
    row_ptr[brows] = ntile;
    return ntile;
}

extern "C" int et_prune_row_mat(const void *W, int N, int K, float sparsity, int *row_id) {
    if (!W || N <= 0 || K <= 0 || !(sparsity >= 0.f) || !(sparsity <= 1.f)) {
        et::set_error("et_prune_row_mat: N=%d K=%d sparsity=%f", N, K, (double)sparsity);
        return ET_ERR_INVALID_ARG;
    }
    const int keep = (int)(N * (1.0 - (double)sparsity)); // as test/row_mat.cu:7
    if (keep > 0 && !row_id) {
        et::set_error("et_prune_row_mat: null row_id");
        return ET_ERR_INVALID_ARG;
    }
    const uint16_t *w = static_cast<const uint16_t *>(W);
    std::vector<double> norm2(N);
    for (int n = 0; n < N; n++) {
        double acc = 0.0;
        for (int k = 0; k < K; k++) {
            const double v = half_to_double(w[(size_t)n * K + k]);
            acc += v * v;
        }
        norm2[n] = acc;
    }
    std::vector<int> kept = top_by_key(norm2, keep);
    std::sort(kept.begin(), kept.end());
    for (int i = 0; i < keep; i++)
        row_id[i] = kept[i];
    return keep;
}

// ---------------------------------------------------------------------------
// On-disk container for the two formats (the reference has none).  Little
// endian.  64-byte header, then the arrays back to back:
//   tile_mat: row_ptr[out/16+1] i32, row_offset[count] i32, data[count*256] f16, bias[out] f16
//   row_mat : row_id[count] i32, weight[count*in] f16 (compact rows), bias[out] f16
// The header carries the payload size and its FNV-1a 64 checksum.
// ---------------------------------------------------------------------------
namespace {

struct ContainerHeader {
    char magic[8];
    int32_t version, in_feat, out_feat, count;
    uint64_t payload_bytes, checksum;
    char reserved[24];
};
static_assert(sizeof(ContainerHeader) == 64, "container header is 64 bytes");

const char TILE_MAGIC[8] = {'E', 'T', 'T', 'I', 'L', 'E', 'M', 0};
const char ROW_MAGIC[8] = {'E', 'T', 'R', 'O', 'W', 'M', 'A', 0};

uint64_t fnv1a(const unsigned char *p, size_t n, uint64_t h = 0xcbf29ce484222325ull) {
    for (size_t i = 0; i < n; i++) {
        h ^= p[i];
        h *= 0x100000001b3ull;
    }
    return h;
}

struct Part {
    const void *src;
    void *dst;
    size_t bytes;
};

int save_container(const char *path, const char *magic, int in_feat, int out_feat, int count,
                   const std::vector<Part> &parts, const char *who) {
    ContainerHeader h;
    memset(&h, 0, sizeof(h));
    memcpy(h.magic, magic, 8);
    h.version = 1;
    h.in_feat = in_feat;
    h.out_feat = out_feat;
    h.count = count;
    h.checksum = 0xcbf29ce484222325ull;
    for (const Part &p : parts) {
        h.payload_bytes += p.bytes;
        h.checksum = fnv1a(static_cast<const unsigned char *>(p.src), p.bytes, h.checksum);
    }
    FILE *f = fopen(path, "wb");
    if (!f) {
        et::set_error("%s: cannot create %s", who, path);
        return ET_ERR_IO;
    }
    bool ok = fwrite(&h, sizeof(h), 1, f) == 1;
    for (const Part &p : parts)
        ok = ok && (p.bytes == 0 || fwrite(p.src, p.bytes, 1, f) == 1);
    ok = (fclose(f) == 0) && ok;
    if (!ok) {
        et::set_error("%s: write to %s failed", who, path);
        return ET_ERR_IO;
    }
    return ET_OK;
}

int read_header(FILE *f, const char *magic, ContainerHeader *h, const char *path, const char *who) {
    if (fread(h, sizeof(*h), 1, f) != 1 || memcmp(h->magic, magic, 8) != 0 || h->version != 1 ||
        h->in_feat <= 0 || h->out_feat <= 0 || h->count < 0) {
        et::set_error("%s: %s is not a version-1 container of this kind", who, path);
        return ET_ERR_FORMAT;
    }
    for (char c : h->reserved) // written as zero; anything else is damage (the checksum covers the payload only)
        if (c != 0) {
            et::set_error("%s: %s has a damaged header", who, path);
            return ET_ERR_FORMAT;
        }
    return ET_OK;
}

int peek_container(const char *path, const char *magic, int *in_feat, int *out_feat, int *count,
                   const char *who) {
    if (!path) {
        et::set_error("%s: null path", who);
        return ET_ERR_INVALID_ARG;
    }
    FILE *f = fopen(path, "rb");
    if (!f) {
        et::set_error("%s: cannot open %s", who, path);
        return ET_ERR_IO;
    }
    ContainerHeader h;
    const int rc = read_header(f, magic, &h, path, who);
    fclose(f);
    if (rc != ET_OK)
        return rc;
    if (in_feat) *in_feat = h.in_feat;
    if (out_feat) *out_feat = h.out_feat;
    if (count) *count = h.count;
    return ET_OK;
}

// parts(h) lists the destination arrays once the header is known
template <class PartsFn>
int load_container(const char *path, const char *magic, PartsFn parts_of, const char *who) {
    if (!path) {
        et::set_error("%s: null path", who);
        return ET_ERR_INVALID_ARG;
    }
    FILE *f = fopen(path, "rb");
    if (!f) {
        et::set_error("%s: cannot open %s", who, path);
        return ET_ERR_IO;
    }
    ContainerHeader h;
    int rc = read_header(f, magic, &h, path, who);
    if (rc == ET_OK) {
        const std::vector<Part> parts = parts_of(h);
        uint64_t total = 0, sum = 0xcbf29ce484222325ull;
        for (const Part &p : parts)
            total += p.bytes;
        if (parts.empty()) {
            et::set_error("%s: %s holds in_feat=%d out_feat=%d count=%d, not what the caller sized its arrays for", who,
                          path, h.in_feat, h.out_feat, h.count);
            rc = ET_ERR_FORMAT;
        } else if (total != h.payload_bytes) {
            et::set_error("%s: %s: payload size does not match its header", who, path);
            rc = ET_ERR_FORMAT;
        }
        for (size_t i = 0; rc == ET_OK && i < parts.size(); i++) {
            if (parts[i].bytes && fread(parts[i].dst, parts[i].bytes, 1, f) != 1) {
                et::set_error("%s: %s is truncated", who, path);
                rc = ET_ERR_FORMAT;
            } else {
                sum = fnv1a(static_cast<const unsigned char *>(parts[i].dst), parts[i].bytes, sum);
            }
        }
        if (rc == ET_OK && (sum != h.checksum || fgetc(f) != EOF)) {
            et::set_error("%s: %s: checksum mismatch or trailing bytes", who, path);
            rc = ET_ERR_FORMAT;
        }
    }
    fclose(f);
    return rc;
}

} // namespace

extern "C" int et_tile_mat_save(const char *path, int in_feat, int out_feat, int ntile,
                                const int *row_ptr, const int *row_offset, const void *data,
                                const void *bias) {
    if (!path || !row_ptr || !bias || (ntile > 0 && (!row_offset || !data))) {
        et::set_error("et_tile_mat_save: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    const int v = et_tile_mat_validate(out_feat, in_feat, ntile, row_ptr, row_offset);
    if (v != 0) {
        et::set_error("et_tile_mat_save: malformed tile_mat (check %d)", v);
        return ET_ERR_FORMAT;
    }
    return save_container(path, TILE_MAGIC, in_feat, out_feat, ntile,
                          {{row_ptr, nullptr, sizeof(int) * (size_t)(out_feat / 16 + 1)},
                           {row_offset, nullptr, sizeof(int) * (size_t)ntile},
                           {data, nullptr, 512 * (size_t)ntile},
                           {bias, nullptr, 2 * (size_t)out_feat}},
                          "et_tile_mat_save");
}

extern "C" int et_tile_mat_peek(const char *path, int *in_feat, int *out_feat, int *ntile) {
    return peek_container(path, TILE_MAGIC, in_feat, out_feat, ntile, "et_tile_mat_peek");
}

extern "C" int et_tile_mat_load(const char *path, int expect_in_feat, int expect_out_feat, int expect_ntile,
                                int *row_ptr, int *row_offset, void *data, void *bias) {
    if (!row_ptr || !row_offset || !data || !bias) {
        et::set_error("et_tile_mat_load: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    int in_feat = 0, out_feat = 0, ntile = 0;
    const int rc = load_container(
        path, TILE_MAGIC,
        [&](const ContainerHeader &h) {
            in_feat = h.in_feat, out_feat = h.out_feat, ntile = h.count;
            // the caller sized its arrays from an earlier peek: a file that has changed since, or
            // arrays meant for another file, must not be written past
            if (h.in_feat != expect_in_feat || h.out_feat != expect_out_feat || h.count != expect_ntile)
                return std::vector<Part>{};
            return std::vector<Part>{{nullptr, row_ptr, sizeof(int) * (size_t)(h.out_feat / 16 + 1)},
                                     {nullptr, row_offset, sizeof(int) * (size_t)h.count},
                                     {nullptr, data, 512 * (size_t)h.count},
                                     {nullptr, bias, 2 * (size_t)h.out_feat}};
        },
        "et_tile_mat_load");
    if (rc != ET_OK)
        return rc;
    if (out_feat % 16 || in_feat % 16 ||
        et_tile_mat_validate(out_feat, in_feat, ntile, row_ptr, row_offset) != 0) {
        et::set_error("et_tile_mat_load: %s holds a malformed tile_mat", path);
        return ET_ERR_FORMAT;
    }
    return ET_OK;
}

extern "C" int et_row_mat_save(const char *path, int in_feat, int out_feat, int nrow, const int *row_id,
                               const void *weight, const void *bias) {
    if (!path || !bias || in_feat <= 0 || out_feat <= 0 || nrow < 0 || nrow > out_feat ||
        (nrow > 0 && (!row_id || !weight))) {
        et::set_error("et_row_mat_save: bad arguments");
        return ET_ERR_INVALID_ARG;
    }
    for (int i = 0; i < nrow; i++)
        if (row_id[i] < 0 || row_id[i] >= out_feat || (i && row_id[i] <= row_id[i - 1])) {
            et::set_error("et_row_mat_save: row_id must be strictly ascending inside [0, out_feat)");
            return ET_ERR_FORMAT;
        }
    return save_container(path, ROW_MAGIC, in_feat, out_feat, nrow,
                          {{row_id, nullptr, sizeof(int) * (size_t)nrow},
                           {weight, nullptr, 2 * (size_t)nrow * in_feat},
                           {bias, nullptr, 2 * (size_t)out_feat}},
                          "et_row_mat_save");
}

extern "C" int et_row_mat_peek(const char *path, int *in_feat, int *out_feat, int *nrow) {
    return peek_container(path, ROW_MAGIC, in_feat, out_feat, nrow, "et_row_mat_peek");
}

extern "C" int et_row_mat_load(const char *path, int expect_in_feat, int expect_out_feat, int expect_nrow,
                               int *row_id, void *weight, void *bias) {
    if (!row_id || !weight || !bias) {
        et::set_error("et_row_mat_load: null pointer");
        return ET_ERR_INVALID_ARG;
    }
    int out_feat = 0, nrow = 0;
    const int rc = load_container(
        path, ROW_MAGIC,
        [&](const ContainerHeader &h) {
            out_feat = h.out_feat, nrow = h.count;
            if (h.in_feat != expect_in_feat || h.out_feat != expect_out_feat || h.count != expect_nrow)
                return std::vector<Part>{};
            return std::vector<Part>{{nullptr, row_id, sizeof(int) * (size_t)h.count},
                                     {nullptr, weight, 2 * (size_t)h.count * h.in_feat},
                                     {nullptr, bias, 2 * (size_t)h.out_feat}};
        },
        "et_row_mat_load");
    if (rc != ET_OK)
        return rc;
    for (int i = 0; i < nrow; i++)
        if (row_id[i] < 0 || row_id[i] >= out_feat || (i && row_id[i] <= row_id[i - 1])) {
            et::set_error("et_row_mat_load: %s holds an unsorted or out-of-range row_id", path);
            return ET_ERR_FORMAT;
        }
    return ET_OK;
}
