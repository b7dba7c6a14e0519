"""numpy front-end of the CPU oracle (oracle/et_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg — never by the et_amd package.  All tensors are
numpy arrays; halves are np.float16 (viewed as uint16 for the C side).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.orc_gen_sparse_tile_mat.restype = C.c_int
        _lib.orc_gen_sparse_tile_mat.argtypes = [C.c_int, C.c_int, C.c_float, C.c_uint64, C.c_void_p, C.c_void_p]
        _lib.orc_gen_sparse_row_mat.restype = C.c_int
        _lib.orc_gen_sparse_row_mat.argtypes = [C.c_int, C.c_float, C.c_uint64, C.c_void_p]
        _lib.orc_gen_head_balanced_rows.restype = None
        _lib.orc_gen_head_balanced_rows.argtypes = [C.c_int, C.c_int, C.c_int, C.c_uint64, C.c_void_p]
        _lib.orc_tile_mat_validate.restype = C.c_int
        _lib.orc_tile_mat_validate.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    return _lib


def _p(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def _h(a):
    """contiguous float16 array (no copy when already so)"""
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


def _i(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


def _suf(name, f64):
    return getattr(lib(), name + ("_f64" if f64 else "_f32"))


# ---------------------------------------------------------------- conversions
def f2h(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f2h(_p(x), _p(out), C.c_long(x.size))
    return out.view(np.float16)


def d2h(x):
    x = np.ascontiguousarray(x, dtype=np.float64)
    out = np.empty(x.shape, np.uint16)
    lib().orc_d2h(_p(x), _p(out), C.c_long(x.size))
    return out.view(np.float16)


def h2f(x):
    x = _h(x)
    out = np.empty(x.shape, np.float32)
    lib().orc_h2f(_p(x), _p(out), C.c_long(x.size))
    return out


# ------------------------------------------------------------------- formats
def gen_sparse_tile_mat(nrow, ncol, sparsity, seed):
    """-> (row_ptr[nrow/16+1], row_offset[ntile]) int32; test/tile_mat.cu:5-34"""
    total = (nrow // 16) * (ncol // 16)
    row_ptr = np.zeros(nrow // 16 + 1, np.int32)
    row_offset = np.zeros(max(total, 1), np.int32)
    nt = lib().orc_gen_sparse_tile_mat(nrow, ncol, C.c_float(sparsity), C.c_uint64(seed), _p(row_ptr), _p(row_offset))
    return row_ptr, row_offset[:nt].copy()


def prune_tile_mat(W, sparsity):
    """magnitude pruning: the tiles of dense half W[N x K] with the largest L2 norm -> (row_ptr, row_offset)"""
    W = _h(W)
    N, K = W.shape
    row_ptr = np.zeros(N // 16 + 1, np.int32)
    row_offset = np.zeros(max((N // 16) * (K // 16), 1), np.int32)
    nt = lib().orc_prune_tile_mat(_p(W), N, K, C.c_float(sparsity), _p(row_ptr), _p(row_offset))
    return row_ptr, row_offset[:nt].copy()


def prune_row_mat(W, sparsity):
    """magnitude pruning: sorted ids of the rows of dense half W[N x K] with the largest L2 norm"""
    W = _h(W)
    row_id = np.zeros(max(W.shape[0], 1), np.int32)
    n = lib().orc_prune_row_mat(_p(W), W.shape[0], W.shape[1], C.c_float(sparsity), _p(row_id))
    return row_id[:n].copy()


def gen_sparse_row_mat(nrow, sparsity, seed):
    """-> sorted row_id[nn_row] int32; test/row_mat.cu:5-14"""
    row_id = np.zeros(max(nrow, 1), np.int32)
    nn = lib().orc_gen_sparse_row_mat(nrow, C.c_float(sparsity), C.c_uint64(seed), _p(row_id))
    return row_id[:nn].copy()


def gen_head_balanced_rows(nhead, head_dim, keep, seed):
    row_id = np.zeros(nhead * keep, np.int32)
    lib().orc_gen_head_balanced_rows(nhead, head_dim, keep, C.c_uint64(seed), _p(row_id))
    return row_id


def head_ptr(row_id, nhead, head_dim):
    row_id = _i(row_id)
    hp = np.zeros(nhead + 1, np.int32)
    lib().orc_head_ptr(_p(row_id), C.c_int(row_id.size), C.c_int(nhead), C.c_int(head_dim), _p(hp))
    return hp


def tile_mat_validate(N, K, row_ptr, row_offset):
    row_ptr, row_offset = _i(row_ptr), _i(row_offset)
    return lib().orc_tile_mat_validate(N, K, int(row_offset.size), _p(row_ptr), _p(row_offset))


def tile_pack(W, row_ptr, row_offset):
    W = _h(W)
    N, K = W.shape
    row_ptr, row_offset = _i(row_ptr), _i(row_offset)
    data = np.zeros(row_offset.size * 256, np.float16)
    lib().orc_tile_pack(_p(W), C.c_int(N), C.c_int(K), _p(row_ptr), _p(row_offset), _p(data))
    return data


def tile_unpack(N, K, row_ptr, row_offset, data):
    row_ptr, row_offset, data = _i(row_ptr), _i(row_offset), _h(data)
    W = np.zeros((N, K), np.float16)
    lib().orc_tile_unpack(_p(W), C.c_int(N), C.c_int(K), _p(row_ptr), _p(row_offset), _p(data))
    return W


# ----------------------------------------------------------------------- ops
def gelu(x):
    x = _h(x)
    out = np.empty_like(x)
    lib().orc_gelu(_p(x), _p(out), C.c_long(x.size))
    return out


def tile_linear(X, row_ptr, row_offset, data, bias, N, gelu=False, f64=False):
    X = _h(X)
    M, K = X.shape
    row_ptr, row_offset, data, bias = _i(row_ptr), _i(row_offset), _h(data), _h(bias)
    Y = np.empty((M, N), np.float16)
    _suf("orc_tile_linear", f64)(_p(Y), _p(X), _p(row_ptr), _p(row_offset), _p(data), _p(bias),
                                 C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(int(gelu)))
    return Y


def row_linear(X, W, bias, f64=False):
    X, W, bias = _h(X), _h(W), _h(bias)
    M, K = X.shape
    N = W.shape[0]
    out = np.empty((M, N), np.float16)
    _suf("orc_row_linear", f64)(_p(out), _p(X), _p(W), _p(bias), C.c_int(M), C.c_int(N), C.c_int(K))
    return out


def skip_layernorm(a, skip, gamma, beta, f64=False):
    a = _h(a).copy()
    skip, gamma, beta = _h(skip), _h(gamma), _h(beta)
    num, size = a.shape
    _suf("orc_skip_layernorm", f64)(_p(a), _p(skip), _p(gamma), _p(beta), C.c_int(num), C.c_int(size))
    return a


def _lens(seq_lens):
    return None if seq_lens is None else _i(seq_lens)


def otf_attention(Q, K, V, mask, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, f64=False):
    Q, K, V = _h(Q), _h(K), _h(V)
    d_model = Q.shape[1]
    mask = None if mask is None else _h(mask)
    sl = _lens(seq_lens)
    out = np.empty((batch * seq_len, d_model), np.float16)
    _suf("orc_otf_attention", f64)(_p(out), _p(Q), _p(K), _p(V), _p(mask), C.c_int(seq_len), C.c_int(d_model),
                                   C.c_int(nhead), C.c_int(batch), _p(sl), C.c_float(log2_scale))
    return out


def prune_attention(Q, K, V, qk_head_ptr, v_col_id, v_head_ptr, mask, seq_len, d_model, nhead,
                    batch=1, seq_lens=None, log2_scale=1.0, f64=False):
    Q, K, V = _h(Q), _h(K), _h(V)
    mask = None if mask is None else _h(mask)
    qk = None if qk_head_ptr is None else _i(qk_head_ptr)
    vc = None if v_col_id is None else _i(v_col_id)
    vh = None if v_head_ptr is None else _i(v_head_ptr)
    sl = _lens(seq_lens)
    out = np.empty((batch * seq_len, d_model), np.float16)
    _suf("orc_prune_attention", f64)(_p(out), _p(Q), _p(K), _p(V), _p(qk), C.c_int(Q.shape[1]), _p(vc), _p(vh),
                                     C.c_int(V.shape[1]), _p(mask), C.c_int(seq_len), C.c_int(d_model),
                                     C.c_int(nhead), C.c_int(batch), _p(sl), C.c_float(log2_scale))
    return out


def qk_scores(Q, K, seq_len, nhead, batch=1, f64=False):
    Q, K = _h(Q), _h(K)
    d_model = Q.shape[1]
    QK = np.empty((batch * nhead, seq_len, seq_len), np.float16)
    _suf("orc_qk_scores", f64)(_p(QK), _p(Q), _p(K), C.c_int(seq_len), C.c_int(d_model), C.c_int(nhead), C.c_int(batch))
    return QK


def sharedqk_attention(QK, V, mask, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, f64=False):
    QK, V = _h(QK), _h(V)
    d_model = V.shape[1]
    mask = None if mask is None else _h(mask)
    sl = _lens(seq_lens)
    out = np.empty((batch * seq_len, d_model), np.float16)
    _suf("orc_sharedqk_attention", f64)(_p(out), _p(QK), _p(V), _p(mask), C.c_int(seq_len), C.c_int(d_model),
                                        C.c_int(nhead), C.c_int(batch), _p(sl), C.c_float(log2_scale))
    return out


def encoder_tile_layer(x, linears, ln, mask, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, f64=False):
    """linears: six dicts (Q,K,V,O,FFN1,FFN2) with row_ptr,row_offset,data,bias;
    ln: (gamma1, beta1, gamma2, beta2).  Follows encoder/encoder.cu:20-45."""
    x = _h(x)
    rows, d_model = x.shape
    d_ff = linears[4]["bias"].size
    keep = []
    arrs = {}
    for key, ct in (("row_ptr", np.int32), ("row_offset", np.int32), ("data", np.float16), ("bias", np.float16)):
        ptrs = (C.c_void_p * 6)()
        for j, l in enumerate(linears):
            a = np.ascontiguousarray(l[key], dtype=ct)
            keep.append(a)
            ptrs[j] = a.ctypes.data
        arrs[key] = ptrs
    g1, b1, g2, b2 = (_h(t) for t in ln)
    mask = None if mask is None else _h(mask)
    sl = _lens(seq_lens)
    ws = np.zeros(8 * rows * d_model + rows * d_ff, np.float16)
    out = np.empty_like(x)
    _suf("orc_encoder_tile_layer", f64)(_p(out), _p(x), _p(ws), arrs["row_ptr"], arrs["row_offset"], arrs["data"],
                                        arrs["bias"], _p(g1), _p(b1), _p(g2), _p(b2), _p(mask), C.c_int(seq_len),
                                        C.c_int(d_model), C.c_int(nhead), C.c_int(d_ff), C.c_int(batch), _p(sl),
                                        C.c_float(log2_scale))
    return out
