// Host AddressSanitizer / UBSan driver for et_amd/csrc/formats.cpp (the pruned-weight formats and the
// on-disk container parser).  CPU only: `make -C oracle asan` builds it with -fsanitize=address,undefined
// and tests/test_sanitize.py runs it.  Exit status 0 = every call behaved as stated and the sanitizers
// saw nothing.
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/et_amd.h"

namespace et {
void set_error(const char *, ...) {} // formats.cpp reports through the library's error slot; not needed here
} // namespace et

static int failures = 0;
#define EXPECT(cond)                                                                              \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            fprintf(stderr, "formats_san: line %d: %s\n", __LINE__, #cond);                       \
            failures++;                                                                           \
        }                                                                                         \
    } while (0)

static std::vector<unsigned char> slurp(const std::string &p) {
    std::vector<unsigned char> b;
    if (FILE *f = fopen(p.c_str(), "rb")) {
        unsigned char buf[4096];
        size_t n;
        while ((n = fread(buf, 1, sizeof buf, f)) > 0)
            b.insert(b.end(), buf, buf + n);
        fclose(f);
    }
    return b;
}
static void spit(const std::string &p, const std::vector<unsigned char> &b, size_t n) {
    FILE *f = fopen(p.c_str(), "wb");
    if (n)
        fwrite(b.data(), 1, n, f);
    fclose(f);
}

int main(int argc, char **argv) {
    const std::string dir = argc > 1 ? argv[1] : "/tmp";
    const int N = 96, K = 64;
    // ---- generators, validator, packer, pruner, head_ptr
    std::vector<int> rp(N / 16 + 1), ro((N / 16) * (K / 16));
    const int nt = et_gen_sparse_tile_mat(N, K, 0.5f, 7, rp.data(), ro.data());
    EXPECT(nt == 12 && rp.back() == nt);
    EXPECT(et_tile_mat_validate(N, K, nt, rp.data(), ro.data()) == 0);
    EXPECT(et_gen_sparse_tile_mat(N, K + 1, 0.5f, 7, rp.data(), ro.data()) < 0);
    std::vector<uint16_t> W((size_t)N * K), data((size_t)nt * 256), bias(N, 0x3c00);
    for (size_t i = 0; i < W.size(); i++)
        W[i] = (uint16_t)(0x2000 + (i * 37) % 0x1c00); // finite halves
    EXPECT(et_tile_pack(W.data(), N, K, rp.data(), ro.data(), data.data()) == 0);
    std::vector<int> rp2(N / 16 + 1), ro2((N / 16) * (K / 16)), ids(N), hp(4 + 1);
    const int ntp = et_prune_tile_mat(W.data(), N, K, 0.75f, rp2.data(), ro2.data());
    EXPECT(ntp == 6 && et_tile_mat_validate(N, K, ntp, rp2.data(), ro2.data()) == 0);
    const int nr = et_prune_row_mat(W.data(), N, K, 0.7f, ids.data());
    EXPECT(nr == 28);
    EXPECT(et_gen_sparse_row_mat(N, 0.7f, 3, ids.data()) == 28);
    EXPECT(et_head_ptr(ids.data(), 28, 4, 24, hp.data()) == 0 && hp[4] == 28);
    std::vector<int> bal(4 * 8);
    EXPECT(et_gen_head_balanced_rows(4, 24, 8, 5, bal.data()) >= 0 && bal[31] >= 3 * 24 && bal[31] < 96);
    { // malformed index arrays: each is refused
        std::vector<int> bad = ro;
        bad[0] = K; // column beyond the matrix
        EXPECT(et_tile_mat_validate(N, K, nt, rp.data(), bad.data()) != 0);
        bad = ro;
        bad[0] += 3; // not a multiple of 16
        EXPECT(et_tile_mat_validate(N, K, nt, rp.data(), bad.data()) != 0);
        std::vector<int> badp = rp;
        badp[1] = nt + 5;
        EXPECT(et_tile_mat_validate(N, K, nt, badp.data(), ro.data()) != 0);
    }
    // ---- container round trips
    const std::string pt = dir + "/san.ettile", pr = dir + "/san.etrow", pb = dir + "/san.bad";
    EXPECT(et_tile_mat_save(pt.c_str(), K, N, nt, rp.data(), ro.data(), data.data(), bias.data()) == 0);
    int a = 0, b = 0, c = 0;
    EXPECT(et_tile_mat_peek(pt.c_str(), &a, &b, &c) == 0 && a == K && b == N && c == nt);
    std::vector<int> rpl(N / 16 + 1), rol(nt);
    std::vector<uint16_t> dl((size_t)nt * 256), bl(N);
    EXPECT(et_tile_mat_load(pt.c_str(), K, N, nt, rpl.data(), rol.data(), dl.data(), bl.data()) == 0);
    EXPECT(rpl == rp && memcmp(dl.data(), data.data(), dl.size() * 2) == 0);
    std::vector<uint16_t> rows((size_t)28 * K, 0x3800);
    EXPECT(et_row_mat_save(pr.c_str(), K, N, 28, ids.data(), rows.data(), bias.data()) == 0);
    std::vector<int> idl(28);
    std::vector<uint16_t> rl((size_t)28 * K);
    EXPECT(et_row_mat_load(pr.c_str(), K, N, 28, idl.data(), rl.data(), bl.data()) == 0);
    // ---- damage: the loader must refuse without reading or writing out of bounds.  The arrays handed
    // to it are exactly as large as the caller's expectation says (the sanitizer watches their ends).
    const std::vector<unsigned char> raw = slurp(pt);
    EXPECT(raw.size() > 64);
    auto load_bad = [&](int eK, int eN, int ent) {
        std::vector<int> p1((size_t)eN / 16 + 1), p2((size_t)(ent > 0 ? ent : 1));
        std::vector<uint16_t> p3((size_t)(ent > 0 ? ent : 1) * 256), p4((size_t)eN);
        return et_tile_mat_load(pb.c_str(), eK, eN, ent, p1.data(), p2.data(), p3.data(), p4.data());
    };
    for (size_t n = 0; n < raw.size(); n += (n < 80 ? 1 : 97)) { // every truncation of the header, then strides
        spit(pb, raw, n);
        EXPECT(load_bad(K, N, nt) < 0);
        EXPECT(et_tile_mat_peek(pb.c_str(), &a, &b, &c) < 0 || n >= 64);
    }
    for (size_t at = 0; at < raw.size(); at += (at < 64 ? 1 : 53)) { // one flipped bit anywhere
        std::vector<unsigned char> d = raw;
        d[at] ^= 0x10;
        spit(pb, d, d.size());
        EXPECT(load_bad(K, N, nt) < 0);
    }
    { // trailing bytes, the other kind's file, sizes other than the caller's
        std::vector<unsigned char> d = raw;
        d.push_back(0);
        spit(pb, d, d.size());
        EXPECT(load_bad(K, N, nt) < 0);
        const std::vector<unsigned char> other = slurp(pr);
        spit(pb, other, other.size());
        EXPECT(load_bad(K, N, nt) < 0);
        spit(pb, raw, raw.size());
        EXPECT(load_bad(K, N, nt - 1) < 0);
        EXPECT(load_bad(K, N - 16, nt) < 0);
        EXPECT(load_bad(K, N, nt) == 0);
    }
    { // a header whose counts are absurd (and whose other fields still look right)
        std::vector<unsigned char> d = raw;
        for (size_t off = 8; off + 4 <= 40; off += 4) { // every 32-bit field after the magic, one at a time
            std::vector<unsigned char> e = d;
            e[off] = 0xff, e[off + 1] = 0xff, e[off + 2] = 0xff, e[off + 3] = 0x7f;
            spit(pb, e, e.size());
            EXPECT(load_bad(K, N, nt) < 0);
            EXPECT(load_bad(K, N, 0x7fffffff / 1024) < 0);
        }
    }
    EXPECT(et_tile_mat_load((dir + "/san.missing").c_str(), K, N, nt, rpl.data(), rol.data(), dl.data(), bl.data()) ==
           ET_ERR_IO);
    remove(pt.c_str());
    remove(pr.c_str());
    remove(pb.c_str());
    if (failures)
        return 1;
    puts("formats_san: ok");
    return 0;
}
