"""The launchers of the reference's kernels/kernels.h over torch device tensors.

Each function forwards raw device pointers to the C ABI (include/et_amd.h) on
torch's current stream.  Names follow the reference launchers.
"""
from __future__ import annotations

import weakref

import torch

from ._lib import check, lib

LOG2E = 1.4426950408889634


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device, contiguous tensors only"
    return t.data_ptr()


def _h(t):
    assert t is None or t.dtype == torch.float16
    return _p(t)


def _i32(t):
    assert t is None or t.dtype == torch.int32
    return _p(t)


def _want(t, what, *shape):
    """The C ABI takes bare pointers and cannot know a buffer's extent: the extents that the other
    arguments imply are checked here, before a kernel reads or writes past a tensor.  A single number
    is an element count, several are the exact shape; None tensors (optional operands) pass."""
    if t is None:
        return
    ok = t.numel() == shape[0] if len(shape) == 1 else tuple(t.shape) == tuple(shape)
    if not ok:
        raise ValueError(f"{what}: expected {shape[0] if len(shape) == 1 else tuple(shape)} "
                         f"{'elements' if len(shape) == 1 else ''}, got {tuple(t.shape)}")


def skip_layernorm(in_out, skip, gamma, beta):
    """in place on in_out[num x size]; kernels/kernels.h:3-5"""
    num, size = in_out.shape
    _want(skip, "skip_layernorm skip", num, size)
    _want(gamma, "skip_layernorm gamma", size)
    _want(beta, "skip_layernorm beta", size)
    check(lib().et_skip_layernorm(_h(in_out), _h(skip), _h(gamma), _h(beta), num, size, _stream()))
    return in_out


def tile_spmm_add_bias(X, row_ptr, row_offset, data, bias, N, gelu=False, out=None):
    """Y = X W^T + bias with W as tile_mat; kernels/kernels.h:13-20"""
    M, K = X.shape
    Y = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=X.device)
    _want(Y, "tile_spmm_add_bias out", M, N)
    _want(bias, "tile_spmm_add_bias bias", N)
    _want(data, "tile_spmm_add_bias data", (0 if row_offset is None else row_offset.numel()) * 256)
    if N % 16 == 0:  # (other widths are the C ABI's to refuse)
        _want(row_ptr, "tile_spmm_add_bias row_ptr", N // 16 + 1)
    fn = lib().et_tile_spmm_add_bias_gelu if gelu else lib().et_tile_spmm_add_bias
    check(fn(_h(Y), _h(X), _i32(row_ptr), _i32(row_offset), _h(data), M, N, K, _h(bias), _stream()))
    return Y


def row_spmm_add_bias(X, weight, bias, out=None, gelu=False):
    """out = X weight^T + bias, weight[N x K] row-major; kernels/kernels.h:7-11"""
    M, K = X.shape
    N = weight.shape[0]
    Y = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=X.device)
    _want(Y, "row_spmm_add_bias out", M, N)
    _want(weight, "row_spmm_add_bias weight", N, K)
    _want(bias, "row_spmm_add_bias bias", N)
    fn = lib().et_row_spmm_add_bias_gelu if gelu else lib().et_row_spmm_add_bias
    check(fn(_h(Y), _h(X), _h(weight), _h(bias), M, N, K, _stream()))
    return Y


def row_spmm_add_bias_multi(X, weights, biases):
    """several row linears over the same input in one launch"""
    import ctypes as C
    M, K = X.shape
    n = len(weights)
    if len(biases) != n:
        raise ValueError(f"row_spmm_add_bias_multi: {n} weights but {len(biases)} biases")
    for i, (w, b) in enumerate(zip(weights, biases)):
        if w.dim() != 2 or w.shape[1] != K:
            raise ValueError(f"row_spmm_add_bias_multi weights[{i}]: expected [N x {K}], got {tuple(w.shape)}")
        _want(b, f"row_spmm_add_bias_multi biases[{i}]", w.shape[0])
    outs = [torch.empty((M, w.shape[0]), dtype=torch.float16, device=X.device) for w in weights]
    arr = lambda ts: (C.c_void_p * n)(*[_h(t) for t in ts])
    ns = (C.c_int * n)(*[w.shape[0] for w in weights])
    check(lib().et_row_spmm_add_bias_multi(arr(outs), _h(X), arr(weights), arr(biases), ns, n, M, K, _stream()))
    return outs


def OTF_attention(Q, K, V, mask, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, out=None):
    """kernels/kernels.h:22-24 (+ batch, seq_lens, exponent base)"""
    d_model = Q.shape[1]
    Z = out if out is not None else torch.empty_like(Q)
    for t, name in ((Q, "Q"), (K, "K"), (V, "V"), (Z, "out")):
        _want(t, "OTF_attention " + name, batch * seq_len, d_model)
    _want(mask, "OTF_attention mask", seq_len * seq_len)
    _want(seq_lens, "OTF_attention seq_lens", batch)
    check(lib().et_OTF_attention(_h(Z), _h(Q), _h(K), _h(V), _h(mask), seq_len, d_model, nhead, batch,
                                 _i32(seq_lens), log2_scale, _stream()))
    return Z


def OTF_attention_summary(Q, K, V, mask, summary, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, out=None):
    """OTF_attention with the mask's summary (attention_mask_summary(mask, seq_len), or None) passed along
    instead of looked up by the mask's address"""
    d_model = Q.shape[1]
    Z = out if out is not None else torch.empty_like(Q)
    for t, name in ((Q, "Q"), (K, "K"), (V, "V"), (Z, "out")):
        _want(t, "OTF_attention_summary " + name, batch * seq_len, d_model)
    _want(mask, "OTF_attention_summary mask", seq_len * seq_len)
    _want(seq_lens, "OTF_attention_summary seq_lens", batch)
    if summary is not None and summary.numel() * summary.element_size() < lib().et_attention_mask_summary_bytes(seq_len):
        raise ValueError("OTF_attention_summary: the summary is smaller than et_attention_mask_summary_bytes(seq_len)")
    check(lib().et_OTF_attention_summary(_h(Z), _h(Q), _h(K), _h(V), _h(mask), None if summary is None else summary.data_ptr(),
                                         seq_len, d_model, nhead, batch, _i32(seq_lens), log2_scale, _stream()))
    return Z


def OTF_attention_noalloc(Q, K, V, mask, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, out=None):
    """OTF_attention through the entry point that allocates nothing: the mask summary is computed into a
    static device array of the library (seq_len <= 4096 with a mask).  `out` is required: this wrapper
    allocates nothing either."""
    if out is None:
        raise ValueError("OTF_attention_noalloc: pass the output tensor")
    d_model = Q.shape[1]
    for t, name in ((Q, "Q"), (K, "K"), (V, "V"), (out, "out")):
        _want(t, "OTF_attention_noalloc " + name, batch * seq_len, d_model)
    _want(mask, "OTF_attention_noalloc mask", seq_len * seq_len)
    _want(seq_lens, "OTF_attention_noalloc seq_lens", batch)
    check(lib().et_OTF_attention_noalloc(_h(out), _h(Q), _h(K), _h(V), _h(mask), seq_len, d_model, nhead, batch,
                                         _i32(seq_lens), log2_scale, _stream()))
    return out


def OTF_attention_qk_width(Q, K, V, mask, qk_width, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, out=None):
    """Q, K compact [rows x nhead*qk_width] (the same number of kept columns in every head); V full width"""
    d_model = V.shape[1]
    Z = out if out is not None else torch.empty_like(V)
    for t, name in ((Q, "Q"), (K, "K")):
        _want(t, "OTF_attention_qk_width " + name, batch * seq_len, nhead * qk_width)
    for t, name in ((V, "V"), (Z, "out")):
        _want(t, "OTF_attention_qk_width " + name, batch * seq_len, d_model)
    _want(mask, "OTF_attention_qk_width mask", seq_len * seq_len)
    _want(seq_lens, "OTF_attention_qk_width seq_lens", batch)
    check(lib().et_OTF_attention_qk_width(_h(Z), _h(Q), _h(K), _h(V), _h(mask), qk_width, seq_len, d_model, nhead,
                                          batch, _i32(seq_lens), log2_scale, _stream()))
    return Z


def OTF_attention_varlen(Q, K, V, mask, cu_seqlens, max_seq_len, nhead, log2_scale=1.0, out=None):
    d_model = Q.shape[1]
    batch = cu_seqlens.numel() - 1
    _check_cu(cu_seqlens, max_seq_len, Q.shape[0], "OTF_attention_varlen")
    Z = out if out is not None else torch.empty_like(Q)
    for t, name in ((K, "K"), (V, "V"), (Z, "out")):
        _want(t, "OTF_attention_varlen " + name, *Q.shape)
    _want(mask, "OTF_attention_varlen mask", max_seq_len * max_seq_len)
    check(lib().et_OTF_attention_varlen(_h(Z), _h(Q), _h(K), _h(V), _h(mask), _i32(cu_seqlens), max_seq_len,
                                        d_model, nhead, batch, log2_scale, _stream()))
    return Z


def Prune_attention(Q, K, V, qk_head_ptr, v_col_id, v_head_ptr, mask, seq_len, d_model, nhead, batch=1,
                    seq_lens=None, log2_scale=1.0, out=None):
    """kernels/kernels.h:26-30 (+ compact Q/K, batch, seq_lens, exponent base)"""
    rows = Q.shape[0]
    Z = out if out is not None else torch.empty((rows, d_model), dtype=torch.float16, device=Q.device)
    _want(Z, "Prune_attention out", batch * seq_len, d_model)
    for t, name in ((Q, "Q"), (K, "K"), (V, "V")):
        if t.dim() != 2 or t.shape[0] != batch * seq_len:
            raise ValueError(f"Prune_attention {name}: expected {batch * seq_len} rows, got {tuple(t.shape)}")
    _want(K, "Prune_attention K", *Q.shape)
    _want(mask, "Prune_attention mask", seq_len * seq_len)
    _want(seq_lens, "Prune_attention seq_lens", batch)
    check(lib().et_Prune_attention(_h(Z), _h(Q), _h(K), _h(V), _i32(qk_head_ptr), Q.shape[1], _i32(v_col_id),
                                   _i32(v_head_ptr), V.shape[1], _h(mask), seq_len, d_model, nhead, batch,
                                   _i32(seq_lens), log2_scale, _stream()))
    return Z


def qk_scores(Q, K, seq_len, nhead, batch=1):
    """scaled Q K^T per head into [(b*nhead+h), S, S]; encoder/encoder.cu:126-130"""
    d_model = Q.shape[1]
    _want(Q, "qk_scores Q", batch * seq_len, d_model)
    _want(K, "qk_scores K", batch * seq_len, d_model)
    QK = torch.empty((batch * nhead, seq_len, seq_len), dtype=torch.float16, device=Q.device)
    check(lib().et_qk_scores(_h(QK), _h(Q), _h(K), seq_len, d_model, nhead, batch, _stream()))
    return QK


def sharedQK_attention(QK, V, mask, seq_len, nhead, batch=1, seq_lens=None, log2_scale=1.0, out=None):
    """kernels/kernels.h:32-34"""
    d_model = V.shape[1]
    Z = out if out is not None else torch.empty_like(V)
    _want(QK, "sharedQK_attention QK", batch * nhead * seq_len * seq_len)
    for t, name in ((V, "V"), (Z, "out")):
        _want(t, "sharedQK_attention " + name, batch * seq_len, d_model)
    _want(mask, "sharedQK_attention mask", seq_len * seq_len)
    _want(seq_lens, "sharedQK_attention seq_lens", batch)
    check(lib().et_sharedQK_attention(_h(Z), _h(QK), _h(V), _h(mask), seq_len, d_model, nhead, batch,
                                      _i32(seq_lens), log2_scale, _stream()))
    return Z


_checked_cu = {}   # (address, elements, seq_len, rows) -> (weak reference to the tensor object, version that passed)


def _check_cu(cu_seqlens, seq_len, total_rows, what):
    """the packed row offsets must start at 0, rise by at most seq_len per sequence and end at the packed
    tensor's row count: the kernels trust them for every address.  Checking costs one small device-to-host copy,
    which waits for the stream; a tensor that passed is remembered by address and version counter, so only its
    first use (and the first one after it was written to in place) synchronises.  (The very tensor object: another
    tensor that the allocator later puts at the same address is checked again.)"""
    key = (cu_seqlens.data_ptr(), cu_seqlens.numel(), seq_len, total_rows)
    hit = _checked_cu.get(key)
    if hit is not None and hit[0]() is cu_seqlens and hit[1] == cu_seqlens._version:
        return
    cu = cu_seqlens.detach().cpu().numpy().astype("int64")
    if cu.size < 1 or cu[0] != 0 or cu[-1] != total_rows:
        raise ValueError(f"{what}: cu_seqlens must run from 0 to the {total_rows} packed rows, got "
                         f"{cu[0] if cu.size else None}..{cu[-1] if cu.size else None}")
    step = cu[1:] - cu[:-1]
    if step.size and (step.min() < 0 or step.max() > seq_len):
        raise ValueError(f"{what}: every sequence must hold 0..{seq_len} rows")
    if len(_checked_cu) > 64:
        _checked_cu.clear()
    _checked_cu[key] = (weakref.ref(cu_seqlens), cu_seqlens._version)


def pack_rows(padded, cu_seqlens, seq_len, total_rows, order=None):
    """order (int32 device tensor, optional): packed sequence i is padded sequence order[i]."""
    width = padded.shape[1]
    batch = cu_seqlens.numel() - 1
    _want(padded, "pack_rows padded", batch * seq_len, width)
    _want(order, "pack_rows order", batch)
    _check_cu(cu_seqlens, seq_len, total_rows, "pack_rows")
    packed = torch.empty((total_rows, width), dtype=torch.float16, device=padded.device)
    check(lib().et_pack_rows_ordered(_h(packed), _h(padded), _i32(cu_seqlens), _i32(order), batch, seq_len,
                                     width, _stream()))
    return packed


def unpack_rows(packed, cu_seqlens, seq_len, order=None):
    width = packed.shape[1]
    batch = cu_seqlens.numel() - 1
    _want(order, "unpack_rows order", batch)
    _check_cu(cu_seqlens, seq_len, packed.shape[0], "unpack_rows")
    padded = torch.empty((batch * seq_len, width), dtype=torch.float16, device=packed.device)
    check(lib().et_unpack_rows_ordered(_h(padded), _h(packed), _i32(cu_seqlens), _i32(order), batch, seq_len,
                                       width, _stream()))
    return padded


def scatter_cols(x, col_id, width):
    rows, ld = x.shape
    if col_id.numel() > ld or col_id.numel() > width:
        raise ValueError(f"scatter_cols: {col_id.numel()} column ids for a [{rows} x {ld}] input and width {width}")
    out = torch.empty((rows, width), dtype=torch.float16, device=x.device)
    check(lib().et_scatter_cols(_h(out), _h(x), _i32(col_id), rows, col_id.numel(), ld, width, _stream()))
    return out


def scatter_skip_layernorm(compact, col_id, skip, gamma, beta, out=None):
    """LayerNorm(expand(compact) + skip): compact[rows x ld] holds columns col_id of a [rows x width] matrix"""
    rows, ld = compact.shape
    width = skip.shape[1]
    out = torch.empty_like(skip) if out is None else out
    _want(skip, "scatter_skip_layernorm skip", rows, width)
    _want(out, "scatter_skip_layernorm out", rows, width)
    _want(gamma, "scatter_skip_layernorm gamma", width)
    _want(beta, "scatter_skip_layernorm beta", width)
    if col_id.numel() > ld or col_id.numel() > width:
        raise ValueError(f"scatter_skip_layernorm: {col_id.numel()} column ids for a [{rows} x {ld}] input and width {width}")
    check(lib().et_scatter_skip_layernorm(_h(out), _h(compact), _i32(col_id), col_id.numel(), ld, _h(skip),
                                          _h(gamma), _h(beta), rows, width, _stream()))
    return out


def attention_mask_summary(mask, seq_len):
    """Per-(16 rows x 64 keys) non-zero bits of an additive mask; attach() lets the
    attention launchers skip the all-zero tiles of that mask tensor."""
    nbytes = lib().et_attention_mask_summary_bytes(seq_len)
    out = torch.empty((nbytes // 4,), dtype=torch.int32, device=mask.device)
    check(lib().et_attention_mask_summary(_h(mask), seq_len, _p(out), _stream()))
    return out


def attention_mask_summary_attach(mask, seq_len, summary):
    """Raw form of the registry call (entries are keyed on the mask's device address): prefer MaskSummary,
    which ties the entry to the tensors' lifetime."""
    check(lib().et_attention_mask_summary_attach(_h(mask), seq_len, None if summary is None else _p(summary)))


class MaskSummary:
    """Owns the summary of an additive mask tensor and its registration with the attention launchers.

    The registry is keyed on the mask's device address, so an entry must not outlive the mask it was
    computed from: this object keeps the mask tensor alive while it is attached (its address cannot be
    handed to another tensor meanwhile) and detaches when it is closed or collected.  After writing
    into the mask in place, call refresh(): a stale summary would skip tiles that are no longer zero."""

    def __init__(self, mask, seq_len):
        _want(mask, "MaskSummary mask", seq_len * seq_len)
        self.mask, self.seq_len = mask, seq_len
        self.summary = None
        self.refresh()

    def refresh(self):
        self.summary = attention_mask_summary(self.mask, self.seq_len)
        attention_mask_summary_attach(self.mask, self.seq_len, self.summary)

    def close(self):
        if getattr(self, "summary", None) is not None:
            attention_mask_summary_attach(self.mask, self.seq_len, None)
            self.summary = None
            self.mask = None

    __del__ = close

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
