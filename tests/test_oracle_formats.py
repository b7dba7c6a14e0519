"""Pins for the oracle's number formats and pruned-weight formats (CPU only).

The reference holds no golden vectors (its tests assert nothing on data); the
only reference-held invariants are the three asserts of test/tile_mat.cu:31-33.
Everything else here is pinned by IEEE-754 (numpy's float16 as an independent
implementation), by counting rules worked out by hand, and by round trips.
"""
import numpy as np
import pytest

import oracle.et_oracle as orc
from helpers import rng, randn_h


def test_h2f_all_patterns_match_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.h2f(bits.view(np.float16))
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_f2h_matches_numpy_rne():
    r = rng(1)
    x = np.concatenate([
        r.standard_normal(200000).astype(np.float32),
        (r.standard_normal(100000) * 1e-5).astype(np.float32),      # subnormal halves
        (r.standard_normal(100000) * 3e4).astype(np.float32),       # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e30, -1e30, np.inf, -np.inf,
                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 6.1e-5, 6.103515625e-05], np.float32),
    ])
    # exact ties: halfway between adjacent halves must go to even
    h = np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float32)
    ties = (h[:-1] + h[1:]) / 2
    x = np.concatenate([x, ties, -ties])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = orc.f2h(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_d2h_matches_numpy_rne():
    r = rng(2)
    x = np.concatenate([r.standard_normal(100000), r.standard_normal(50000) * 1e-5, r.standard_normal(50000) * 4e4,
                        np.array([0.0, 65504.0, 65519.999, 65520.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -14, 1e300])])
    h = np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
    x = np.concatenate([x, (h[:-1] + h[1:]) / 2])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = orc.d2h(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


# ntile = int(total * (1.0 - double(float(sparsity)))): worked by hand for the
# BERT-base shapes (2304 and 9216 tiles) at the ratios the benchmark sweeps.
@pytest.mark.parametrize("N,K,sp,ntile", [
    (768, 768, 0.0, 2304), (768, 768, 0.5, 1152), (768, 768, 0.7, 691), (768, 768, 0.8, 460), (768, 768, 0.9, 230),
    (3072, 768, 0.0, 9216), (3072, 768, 0.5, 4608), (3072, 768, 0.7, 2764), (3072, 768, 0.8, 1843),
    (768, 3072, 0.9, 921), (64, 64, 0.5, 8), (16, 16, 0.0, 1), (16, 16, 1.0, 0),
])
def test_tile_mat_counts_and_invariants(N, K, sp, ntile):
    row_ptr, row_offset = orc.gen_sparse_tile_mat(N, K, sp, seed=7)
    # the reference's own asserts (test/tile_mat.cu:31-33)
    assert row_ptr.size == N // 16 + 1
    assert row_ptr[-1] == ntile
    assert row_offset.size == ntile
    assert orc.tile_mat_validate(N, K, row_ptr, row_offset) == 0
    assert row_ptr[0] == 0 and (np.diff(row_ptr) >= 0).all()
    assert (row_offset % 16 == 0).all() and (row_offset >= 0).all() and (row_offset < K).all()
    for bn in range(N // 16):  # no duplicate tile in a block-row
        seg = row_offset[row_ptr[bn]:row_ptr[bn + 1]]
        assert np.unique(seg).size == seg.size
    if sp == 0.0:
        assert (np.diff(row_ptr) == K // 16).all()


def test_tile_mat_seed_determinism_and_shuffle_order():
    a = orc.gen_sparse_tile_mat(768, 768, 0.8, seed=11)
    b = orc.gen_sparse_tile_mat(768, 768, 0.8, seed=11)
    c = orc.gen_sparse_tile_mat(768, 768, 0.8, seed=12)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    assert not np.array_equal(a[1], c[1])
    # within a block-row the order is shuffle order, not sorted (test/tile_mat.cu:22-29)
    rp, ro = a
    assert any((np.diff(ro[rp[i]:rp[i + 1]]) < 0).any() for i in range(48))
    # selection is uniform over tiles: block-row counts vary around the mean 9.58
    cnt = np.diff(rp)
    assert cnt.min() < cnt.mean() < cnt.max() and abs(cnt.mean() - 460 / 48) < 1e-9


def test_splitmix_fisher_yates_independent_restatement():
    """the seeded selection restated in pure Python must give the same index lists"""
    def splitmix(state):
        state = (state + 0x9e3779b97f4a7c15) & (2 ** 64 - 1)
        z = state
        z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & (2 ** 64 - 1)
        z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & (2 ** 64 - 1)
        return state, z ^ (z >> 31)

    N, K, sp, seed = 64, 96, 0.5, 1234
    bc = K // 16
    total = (N // 16) * bc
    ids = list(range(total))
    s = seed
    for i in range(total - 1, 0, -1):
        s, z = splitmix(s)
        j = z % (i + 1)
        ids[i], ids[j] = ids[j], ids[i]
    nt = int(total * (1.0 - float(np.float32(sp))))
    kept = ids[:nt]
    rp, ro = [0], []
    for r in range(N // 16):
        for t in kept:
            if t // bc == r:
                ro.append((t % bc) * 16)
        rp.append(len(ro))
    grp, gro = orc.gen_sparse_tile_mat(N, K, sp, seed)
    assert rp == grp.tolist() and ro == gro.tolist()


def test_tile_pack_roundtrip():
    r = rng(3)
    N, K = 96, 160
    W = randn_h(r, (N, K))
    rp, ro = orc.gen_sparse_tile_mat(N, K, 0.6, seed=5)
    data = orc.tile_pack(W, rp, ro)
    # layout: data[i*256 + n*16 + k] = W[bn*16+n][off+k]   (kernels/linear.cu:76)
    for bn in range(N // 16):
        for i in range(rp[bn], rp[bn + 1]):
            blk = data[i * 256:(i + 1) * 256].reshape(16, 16)
            assert np.array_equal(blk, W[bn * 16:bn * 16 + 16, ro[i]:ro[i] + 16])
    Wd = orc.tile_unpack(N, K, rp, ro, data)
    keep = np.zeros((N // 16, K // 16), bool)
    for bn in range(N // 16):
        keep[bn, ro[rp[bn]:rp[bn + 1]] // 16] = True
    mask = np.kron(keep, np.ones((16, 16), bool))
    assert np.array_equal(Wd[mask], W[mask]) and (Wd[~mask] == 0).all()
    # 0 % sparsity: every tile present, dense -> tile_mat -> dense is the identity
    rp0, ro0 = orc.gen_sparse_tile_mat(N, K, 0.0, seed=5)
    assert np.array_equal(orc.tile_unpack(N, K, rp0, ro0, orc.tile_pack(W, rp0, ro0)), W)


def test_tile_mat_validate_rejects_malformed():
    rp, ro = orc.gen_sparse_tile_mat(64, 64, 0.5, seed=1)
    assert orc.tile_mat_validate(64, 64, rp, ro) == 0
    bad = ro.copy(); bad[0] += 8
    assert orc.tile_mat_validate(64, 64, rp, bad) == -5
    bad = ro.copy(); bad[0] = 64
    assert orc.tile_mat_validate(64, 64, rp, bad) == -5
    bad = rp.copy(); bad[-1] += 1
    assert orc.tile_mat_validate(64, 64, bad, ro) == -4
    bad = rp.copy(); bad[0] = 1
    assert orc.tile_mat_validate(64, 64, bad, ro) == -2
    assert orc.tile_mat_validate(60, 64, rp, ro) == -1
    full_rp, full_ro = orc.gen_sparse_tile_mat(16, 64, 0.0, seed=1)
    dup = full_ro.copy(); dup[1] = dup[0]
    assert orc.tile_mat_validate(16, 64, full_rp, dup) == -6


@pytest.mark.parametrize("nrow,sp,nn", [(768, 0.5, 384), (768, 0.7, 230), (3072, 0.5, 1536), (3072, 0.7, 921), (768, 0.0, 768)])
def test_row_mat_counts_sorted(nrow, sp, nn):
    rid = orc.gen_sparse_row_mat(nrow, sp, seed=9)
    assert rid.size == nn  # int(nrow*(1.0-sparsity)), test/row_mat.cu:7
    assert (np.diff(rid) > 0).all() and rid.min() >= 0 and rid.max() < nrow  # sorted, unique (:13)


def test_head_ptr_csr():
    rid = np.array([0, 3, 63, 64, 130, 131, 700], np.int32)
    hp = orc.head_ptr(rid, 12, 64)
    # brute force: head_ptr[h] = #ids below h*64
    want = [int((rid < h * 64).sum()) for h in range(12)] + [rid.size]
    assert hp.tolist() == want
    # empty heads are legal (the reference's scan breaks on them, encoder/Linear.cu:79-87)
    assert hp[2] == hp[1] + 1 and hp[4] == hp[3] and hp[12] == 7
    bal = orc.gen_head_balanced_rows(12, 64, 32, seed=4)
    assert orc.head_ptr(bal, 12, 64).tolist() == [32 * h for h in range(13)]
    assert (np.diff(bal) > 0).all()


# ------------------------------------------------------------------ magnitude pruning
def test_prune_tile_mat_keeps_the_largest_tiles():
    """norms made distinct and well separated, so any correct ranking gives the same set"""
    r = rng(71)
    N, K = 96, 128
    nb = (N // 16) * (K // 16)
    scale = r.permutation(nb).astype(np.float64) + 1.0           # tile t gets magnitude ~ scale[t]
    W = np.zeros((N, K), np.float16)
    for t in range(nb):
        y, x = divmod(t, K // 16)
        W[y * 16:(y + 1) * 16, x * 16:(x + 1) * 16] = (scale[t] * (0.9 + 0.01 * r.random((16, 16)))).astype(np.float16)
    for sp in (0.0, 0.25, 0.5, 0.8, 0.97, 1.0):
        rp, ro = orc.prune_tile_mat(W, sp)
        keep = int(nb * (1.0 - float(np.float32(sp))))
        assert ro.size == keep and rp[-1] == keep and rp[0] == 0
        assert orc.tile_mat_validate(N, K, rp, ro) == 0
        want = np.sort(np.argsort(-scale, kind="stable")[:keep])      # the `keep` largest tiles, row-major
        got = np.concatenate([[bn * (K // 16) + o // 16 for o in ro[rp[bn]:rp[bn + 1]]] for bn in range(N // 16)]).astype(int) if keep else np.array([], int)
        assert np.array_equal(got, want)
        for bn in range(N // 16):                                    # ascending columns inside a block-row
            assert (np.diff(ro[rp[bn]:rp[bn + 1]]) > 0).all()


def test_prune_ties_keep_the_lower_index_and_rows():
    W = np.ones((64, 64), np.float16)                               # every tile / row has the same norm
    rp, ro = orc.prune_tile_mat(W, 0.5)
    assert np.array_equal(rp, [0, 4, 8, 8, 8]) and np.array_equal(ro, list(range(0, 64, 16)) * 2)
    assert np.array_equal(orc.prune_row_mat(W, 0.75), np.arange(16))
    r = rng(72)
    W = (r.standard_normal((200, 48)) * (1 + np.arange(200)[:, None] % 7)).astype(np.float16)
    ids = orc.prune_row_mat(W, 0.7)
    n2 = (W.astype(np.float64) ** 2).sum(1)
    assert ids.size == int(200 * (1.0 - float(np.float32(0.7)))) and (np.diff(ids) > 0).all()
    assert n2[ids].min() >= np.delete(n2, ids).max()                # nothing dropped outranks anything kept
    W[3, 5] = np.float16(np.nan)                                     # NaN contributes nothing; Inf dominates
    W[7, 0] = np.float16(np.inf)
    ids = orc.prune_row_mat(W, 0.99)                                  # int(200*(1-float(0.99f))) = 1 row
    assert ids.tolist() == [7]
