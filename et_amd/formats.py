"""tile_mat / row_mat pruned-weight formats, host side (numpy in, numpy out).

Thin wrappers over the library's own C++ generators; semantics follow
test/tile_mat.cu:5-34 and test/row_mat.cu:5-14 of the reference with an
explicit seed.
"""
from __future__ import annotations

import numpy as np

from ._lib import check, lib


def _ptr(a):
    return None if a is None else a.ctypes.data


def gen_sparse_tile_mat(nrow: int, ncol: int, sparsity: float, seed: int):
    """-> (row_ptr[nrow/16+1], row_offset[ntile]) as int32 arrays"""
    total = max((nrow // 16) * (ncol // 16), 1)
    row_ptr = np.zeros(nrow // 16 + 1, np.int32)
    row_offset = np.zeros(total, np.int32)
    nt = check(lib().et_gen_sparse_tile_mat(nrow, ncol, sparsity, seed, _ptr(row_ptr), _ptr(row_offset)))
    return row_ptr, row_offset[:nt].copy()


def gen_sparse_row_mat(nrow: int, sparsity: float, seed: int):
    """-> sorted surviving row ids (int32)"""
    row_id = np.zeros(max(nrow, 1), np.int32)
    n = check(lib().et_gen_sparse_row_mat(nrow, sparsity, seed, _ptr(row_id)))
    return row_id[:n].copy()


def gen_head_balanced_rows(nhead: int, head_dim: int, keep: int, seed: int):
    row_id = np.zeros(max(nhead * keep, 1), np.int32)
    check(lib().et_gen_head_balanced_rows(nhead, head_dim, keep, seed, _ptr(row_id)))
    return row_id[:nhead * keep].copy()


def tile_mat_validate(N: int, K: int, row_ptr, row_offset) -> int:
    row_ptr = np.ascontiguousarray(row_ptr, np.int32)
    row_offset = np.ascontiguousarray(row_offset, np.int32)
    return lib().et_tile_mat_validate(N, K, int(row_offset.size), _ptr(row_ptr), _ptr(row_offset))


def tile_pack(W, row_ptr, row_offset):
    """dense half W[N x K] -> tile_mat data[ntile*256]"""
    W = np.ascontiguousarray(W)
    assert W.dtype == np.float16 and W.ndim == 2
    row_ptr = np.ascontiguousarray(row_ptr, np.int32)
    row_offset = np.ascontiguousarray(row_offset, np.int32)
    data = np.zeros(row_offset.size * 256, np.float16)
    check(lib().et_tile_pack(_ptr(W), W.shape[0], W.shape[1], _ptr(row_ptr), _ptr(row_offset), _ptr(data)))
    return data


def head_ptr(row_id, nhead: int, head_dim: int):
    row_id = np.ascontiguousarray(row_id, np.int32)
    hp = np.zeros(nhead + 1, np.int32)
    check(lib().et_head_ptr(_ptr(row_id), int(row_id.size), nhead, head_dim, _ptr(hp)))
    return hp


def prune_tile_mat(W, sparsity: float):
    """magnitude pruning of dense half W[N x K] -> (row_ptr, row_offset): the tiles with the largest L2 norm"""
    W = np.ascontiguousarray(W)
    assert W.dtype == np.float16 and W.ndim == 2
    N, K = W.shape
    row_ptr = np.zeros(N // 16 + 1, np.int32)
    row_offset = np.zeros(max((N // 16) * (K // 16), 1), np.int32)
    nt = check(lib().et_prune_tile_mat(_ptr(W), N, K, sparsity, _ptr(row_ptr), _ptr(row_offset)))
    return row_ptr, row_offset[:nt].copy()


def prune_row_mat(W, sparsity: float):
    """magnitude pruning of dense half W[N x K] -> sorted ids of the rows with the largest L2 norm"""
    W = np.ascontiguousarray(W)
    assert W.dtype == np.float16 and W.ndim == 2
    row_id = np.zeros(max(W.shape[0], 1), np.int32)
    n = check(lib().et_prune_row_mat(_ptr(W), W.shape[0], W.shape[1], sparsity, _ptr(row_id)))
    return row_id[:n].copy()


def tile_mat_save(path, in_feat, out_feat, row_ptr, row_offset, data, bias):
    row_ptr = np.ascontiguousarray(row_ptr, np.int32)
    row_offset = np.ascontiguousarray(row_offset, np.int32)
    data = np.ascontiguousarray(data, np.float16)
    bias = np.ascontiguousarray(bias, np.float16)
    check(lib().et_tile_mat_save(str(path).encode(), in_feat, out_feat, int(row_offset.size), _ptr(row_ptr),
                                 _ptr(row_offset), _ptr(data), _ptr(bias)))


def tile_mat_load(path):
    """-> dict(in_feat, out_feat, row_ptr, row_offset, data, bias)"""
    import ctypes as C
    a, b, c = C.c_int(), C.c_int(), C.c_int()
    check(lib().et_tile_mat_peek(str(path).encode(), C.byref(a), C.byref(b), C.byref(c)))
    in_feat, out_feat, nt = a.value, b.value, c.value
    row_ptr = np.zeros(out_feat // 16 + 1, np.int32)
    row_offset = np.zeros(max(nt, 1), np.int32)
    data = np.zeros(max(nt, 1) * 256, np.float16)
    bias = np.zeros(out_feat, np.float16)
    check(lib().et_tile_mat_load(str(path).encode(), in_feat, out_feat, nt, _ptr(row_ptr), _ptr(row_offset), _ptr(data),
                                 _ptr(bias)))
    return dict(in_feat=in_feat, out_feat=out_feat, row_ptr=row_ptr, row_offset=row_offset[:nt].copy(),
                data=data[:nt * 256].copy(), bias=bias)


def row_mat_save(path, in_feat, out_feat, row_id, weight, bias):
    row_id = np.ascontiguousarray(row_id, np.int32)
    weight = np.ascontiguousarray(weight, np.float16)
    bias = np.ascontiguousarray(bias, np.float16)
    assert weight.size == row_id.size * in_feat
    check(lib().et_row_mat_save(str(path).encode(), in_feat, out_feat, int(row_id.size), _ptr(row_id),
                                _ptr(weight), _ptr(bias)))


def row_mat_load(path):
    """-> dict(in_feat, out_feat, row_id, weight[nrow x in_feat], bias)"""
    import ctypes as C
    a, b, c = C.c_int(), C.c_int(), C.c_int()
    check(lib().et_row_mat_peek(str(path).encode(), C.byref(a), C.byref(b), C.byref(c)))
    in_feat, out_feat, n = a.value, b.value, c.value
    row_id = np.zeros(max(n, 1), np.int32)
    weight = np.zeros((max(n, 1), in_feat), np.float16)
    bias = np.zeros(out_feat, np.float16)
    check(lib().et_row_mat_load(str(path).encode(), in_feat, out_feat, n, _ptr(row_id), _ptr(weight), _ptr(bias)))
    return dict(in_feat=in_feat, out_feat=out_feat, row_id=row_id[:n].copy(), weight=weight[:n].copy(), bias=bias)
