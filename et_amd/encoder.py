"""Linear_tile / Linear_row / Encoder_* — the reference's encoder objects
(encoder/Linear.h, encoder/encoder.h) over the C ABI in include/et_encoder.h.

Constructor arguments keep the reference's order and meaning: weights, index
arrays, LayerNorm parameters and the mask are HOST arrays (numpy) copied at
construction; activations and the workspace are DEVICE tensors (torch).
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from ._lib import check, lib

ENCODER_TILE, ENCODER_PRUNE, ENCODER_LENGTH = 0, 1, 2


def _np(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def _hp(a):
    return None if a is None else a.ctypes.data


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _dp(t):
    assert t.is_cuda and t.is_contiguous() and t.dtype == torch.float16
    return t.data_ptr()


def _chk2(t, rows, cols, what):
    if t.dim() != 2 or t.shape[0] < rows or t.shape[1] != cols:
        raise ValueError(f"{what}: expected at least {rows} rows of {cols} columns, got {tuple(t.shape)}")


def _dp2(t, rows, cols, what):
    """device pointer of a [>= rows x cols] half tensor.  The C ABI takes bare pointers and cannot know a
    buffer's extent: an operand of the wrong shape is refused here, before a kernel reads or writes past it."""
    _chk2(t, rows, cols, what)
    return _dp(t)


def _dpn(t, n, what):
    """device pointer of a half vector of exactly n elements (LayerNorm parameters)"""
    if t.numel() != n:
        raise ValueError(f"{what}: expected {n} elements, got {tuple(t.shape)}")
    return _dp(t)


class Linear_tile:
    """encoder/Linear.h:4-46"""

    def __init__(self, in_feat, out_feat, size, ntile, data, row_ptr, row_offset, bias, is_gelu=False):
        self.in_feat, self.out_feat, self.size, self.is_gelu = in_feat, out_feat, size, bool(is_gelu)
        data = _np(data, np.float16)
        row_ptr, row_offset, bias = _np(row_ptr, np.int32), _np(row_offset, np.int32), _np(bias, np.float16)
        assert data.size == ntile * 256 and row_offset.size == ntile and bias.size == out_feat
        h = C.c_void_p()
        check(lib().et_linear_tile_create(C.byref(h), in_feat, out_feat, size, ntile, _hp(data), _hp(row_ptr),
                                          _hp(row_offset), _hp(bias), int(is_gelu)))
        self._h = h

    def run(self, x, out=None, rows=None):
        rows = x.shape[0] if rows is None else rows
        out = out if out is not None else torch.empty((x.shape[0], self.out_feat), dtype=torch.float16, device=x.device)
        check(lib().et_linear_tile_run_rows(self._h, _dp2(out, rows, self.out_feat, "Linear_tile.run out"),
                                            _dp2(x, rows, self.in_feat, "Linear_tile.run x"), rows, _stream()))
        return out

    def run_ln(self, x, skip, gamma, beta, out=None, rows=None):
        """LayerNorm(half(linear(x)) + skip) * gamma + beta in one launch"""
        rows = x.shape[0] if rows is None else rows
        out = out if out is not None else torch.empty((x.shape[0], self.out_feat), dtype=torch.float16, device=x.device)
        check(lib().et_linear_tile_run_rows_ln(self._h, _dp2(out, rows, self.out_feat, "Linear_tile.run_ln out"),
                                               _dp2(x, rows, self.in_feat, "Linear_tile.run_ln x"),
                                               _dp2(skip, rows, self.out_feat, "Linear_tile.run_ln skip"),
                                               _dpn(gamma, self.out_feat, "Linear_tile.run_ln gamma"),
                                               _dpn(beta, self.out_feat, "Linear_tile.run_ln beta"), rows, _stream()))
        return out

    @staticmethod
    def run_ffn_ln(first, second, x, skip, gamma, beta, out=None, hidden=None, rows=None):
        """LayerNorm(half(second(gelu(first(x)))) + skip) * gamma + beta: the feed-forward block in one
        launch.  `hidden` ([rows, first.out_feat]) is only used where the fused kernel does not apply;
        None insists on the fused kernel."""
        rows = x.shape[0] if rows is None else rows
        out = out if out is not None else torch.empty((x.shape[0], second.out_feat), dtype=torch.float16, device=x.device)
        what = "Linear_tile.run_ffn_ln"
        check(lib().et_linear_tile_run_rows_ffn_ln(first._h, second._h, _dp2(out, rows, second.out_feat, what + " out"),
                                                   _dp2(x, rows, first.in_feat, what + " x"),
                                                   _dp2(hidden, rows, first.out_feat, what + " hidden") if hidden is not None else None,
                                                   _dp2(skip, rows, second.out_feat, what + " skip"),
                                                   _dpn(gamma, second.out_feat, what + " gamma"),
                                                   _dpn(beta, second.out_feat, what + " beta"), rows, _stream()))
        return out

    @staticmethod
    def ffn_fusable(first, second):
        return bool(lib().et_linear_tile_ffn_fusable(first._h, second._h))

    @staticmethod
    def run_tail(out_proj, first, second, attn, inp, gamma1, beta1, gamma2, beta2, out=None, mid=None,
                 hidden=None, rows=None, ws=None):
        """Steps 6-10 of a layer in one launch: out projection + skip + LayerNorm, feed-forward block + skip +
        LayerNorm.  `mid` / `hidden` are only used where the fused kernel does not apply; mid=None insists on it.
        `ws` (a uint8 device tensor of at least tail_ws_bytes(...) bytes that overlaps no operand) lets the launch
        take the form of pairs of workgroups over 64-row panels."""
        rows = attn.shape[0] if rows is None else rows
        out = out if out is not None else torch.empty((attn.shape[0], second.out_feat), dtype=torch.float16, device=attn.device)
        what = "Linear_tile.run_tail"
        opt = lambda t, cols, name: _dp2(t, rows, cols, what + name) if t is not None else None
        ws_ptr, ws_bytes = None, 0
        if ws is not None:
            if ws.dtype != torch.uint8 or not ws.is_cuda or not ws.is_contiguous():
                raise ValueError(what + " ws: a contiguous uint8 device tensor is required")
            ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
        check(lib().et_linear_tile_run_rows_tail_ws(out_proj._h, first._h, second._h,
                                                    _dp2(out, rows, second.out_feat, what + " out"),
                                                    _dp2(attn, rows, out_proj.in_feat, what + " attn"),
                                                    _dp2(inp, rows, out_proj.out_feat, what + " inp"),
                                                    opt(mid, out_proj.out_feat, " mid"), opt(hidden, first.out_feat, " hidden"),
                                                    _dpn(gamma1, out_proj.out_feat, what + " gamma1"),
                                                    _dpn(beta1, out_proj.out_feat, what + " beta1"),
                                                    _dpn(gamma2, second.out_feat, what + " gamma2"),
                                                    _dpn(beta2, second.out_feat, what + " beta2"), rows,
                                                    ws_ptr, ws_bytes, _stream()))
        return out

    @staticmethod
    def tail_ws_bytes(out_proj, first, second, rows):
        """bytes of scratch the paired form of run_tail needs for `rows` rows (0 where it does not apply)"""
        return int(lib().et_linear_tile_tail_ws_bytes(out_proj._h, first._h, second._h, rows))

    @staticmethod
    def tail_prepare(out_proj, first, second):
        check(lib().et_linear_tile_tail_prepare(out_proj._h, first._h, second._h))

    @staticmethod
    def tail_fusable(out_proj, first, second):
        return bool(lib().et_linear_tile_tail_fusable(out_proj._h, first._h, second._h))

    def _release(self):  # ownership moved into an encoder
        self._h = None

    def __del__(self):
        if getattr(self, "_h", None):
            lib().et_linear_tile_destroy(self._h)
            self._h = None


def run_multi(linears, x, outs=None):
    """several Linear_tile over the same input in one launch"""
    n = len(linears)
    if x.dim() != 2:
        raise ValueError(f"run_multi x: expected a matrix, got {tuple(x.shape)}")
    rows = x.shape[0]
    outs = outs or [torch.empty((rows, l.out_feat), dtype=torch.float16, device=x.device) for l in linears]
    if len(outs) != n:
        raise ValueError(f"run_multi: {n} linears but {len(outs)} outputs")
    _chk2(x, rows, linears[0].in_feat, "run_multi x")
    for i, (o, l) in enumerate(zip(outs, linears)):
        if l.in_feat != linears[0].in_feat:
            raise ValueError("run_multi: the linears must share in_feat")
        _chk2(o, rows, l.out_feat, f"run_multi outs[{i}]")
    hs = (C.c_void_p * n)(*[l._h for l in linears])
    ys = (C.c_void_p * n)(*[_dp(o) for o in outs])
    check(lib().et_linear_tile_run_multi(hs, ys, n, _dp(x), rows, _stream()))
    return outs


class Linear_row:
    """encoder/Linear.h:48-72"""

    def __init__(self, in_feat, out_feat, size, weight, row_id, nrow, bias, nhead, is_gelu=False):
        weight, row_id, bias = _np(weight, np.float16), _np(row_id, np.int32), _np(bias, np.float16)
        assert weight.size == nrow * in_feat and row_id.size == nrow and bias.size == nrow
        self.in_feat, self.out_feat, self.size, self.nhead = in_feat, out_feat, size, nhead
        h = C.c_void_p()
        check(lib().et_linear_row_create(C.byref(h), in_feat, out_feat, size, _hp(weight), _hp(row_id), nrow,
                                         _hp(bias), nhead))
        self._h = h
        if is_gelu:
            check(lib().et_linear_row_set_gelu(h, 1))
        a, b = C.c_int(), C.c_int()
        check(lib().et_linear_row_query(h, C.byref(a), C.byref(b), None, None))
        self.nrow, self.row_id_size = a.value, b.value

    def run(self, x, out=None):
        out = out if out is not None else torch.empty((x.shape[0], self.nrow), dtype=torch.float16, device=x.device)
        _chk2(out, self.size, self.nrow, "Linear_row.run out")
        _chk2(x, self.size, self.in_feat, "Linear_row.run x")
        check(lib().et_linear_row_run(self._h, _dp(out), _dp(x), _stream()))
        return out

    def _release(self):
        self._h = None

    def __del__(self):
        if getattr(self, "_h", None):
            lib().et_linear_row_destroy(self._h)
            self._h = None


class _Encoder:
    kind = None

    def __init__(self, d_model, seq_len, nheads, buffer, Q_linear, K_linear, V_linear, O_linear, MLP1_linear,
                 MLP2_linear, ln_gamma_1, ln_beta_1, ln_gamma_2, ln_beta_2, mask, batch=1):
        self.d_model, self.seq_len, self.nheads, self.batch = d_model, seq_len, nheads, batch
        need = self.buffer_size(d_model, seq_len, nheads, batch)
        assert buffer.is_cuda and buffer.numel() * buffer.element_size() >= need, "workspace too small"
        self.buffer = buffer
        ln = [_np(t, np.float16) for t in (ln_gamma_1, ln_beta_1, ln_gamma_2, ln_beta_2)]
        assert all(t.size == d_model for t in ln)
        mask = None if mask is None else _np(mask, np.float16)
        assert mask is None or mask.size == seq_len * seq_len
        lin = [Q_linear, K_linear, V_linear, O_linear, MLP1_linear, MLP2_linear]
        h = C.c_void_p()
        self._create(h, d_model, seq_len, nheads, batch, buffer, lin, ln, mask)
        for l in lin:
            l._release()
        self._h = h

    def _create(self, h, d_model, seq_len, nheads, batch, buffer, lin, ln, mask):
        check(lib().et_encoder_create(C.byref(h), self.kind, d_model, seq_len, nheads, batch, buffer.data_ptr(),
                                      *[l._h for l in lin], *[_hp(t) for t in ln], _hp(mask)))

    @classmethod
    def buffer_size(cls, d_model, seq_len, nheads, batch=1):
        return lib().et_encoder_buffer_size(cls.kind, d_model, seq_len, nheads, batch)

    def run(self, out, inp):
        """out, inp: [batch*seq_len, d_model] device tensors; out may be inp"""
        check(lib().et_encoder_set_stream(self._h, _stream()))
        rows = self.batch * self.seq_len
        check(lib().et_encoder_run(self._h, _dp2(out, rows, self.d_model, "Encoder.run out"),
                                   _dp2(inp, rows, self.d_model, "Encoder.run inp")))
        return out

    def set_log2_scale(self, v):
        check(lib().et_encoder_set_log2_scale(self._h, float(v)))

    def set_seq_lens(self, lens):
        if lens is None:
            check(lib().et_encoder_set_seq_lens(self._h, None))
        else:
            lens = _np(lens, np.int64)
            if lens.size != self.batch:
                raise ValueError(f"set_seq_lens: expected {self.batch} lengths, got {lens.size}")
            if lens.size and (lens.min() < 0 or lens.max() > self.seq_len):
                raise ValueError(f"set_seq_lens: lengths must lie in [0, {self.seq_len}], got "
                                 f"[{lens.min()}, {lens.max()}]")
            lens = _np(lens, np.int32)
            check(lib().et_encoder_set_seq_lens(self._h, _hp(lens)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().et_encoder_destroy(self._h)
            self._h = None


class Encoder_tile(_Encoder):
    """encoder/encoder.h:56-77"""
    kind = ENCODER_TILE


class Encoder_prune(_Encoder):
    """encoder/encoder.h:79-100; V_linear is a Linear_row"""
    kind = ENCODER_PRUNE


class Encoder_attnaware(_Encoder):
    """Attention-aware pruning through the whole layer: Q/K row-pruned to the same columns per head, V a tile
    linear, O/FFN1(GELU)/FFN2 row-pruned (no counterpart in the reference)"""
    kind = ENCODER_TILE  # same workspace as the tile encoder

    def _create(self, h, d_model, seq_len, nheads, batch, buffer, lin, ln, mask):
        check(lib().et_encoder_attnaware_create(C.byref(h), d_model, seq_len, nheads, batch, buffer.data_ptr(),
                                                *[l._h for l in lin], *[_hp(t) for t in ln], _hp(mask)))


class Encoder_length(_Encoder):
    """encoder/encoder.h:102-134"""
    kind = ENCODER_LENGTH

    def set_shared_qk(self, on):
        check(lib().et_encoder_set_shared_qk(self._h, int(bool(on))))


class Encoder_stack:
    """N Encoder_length layers run on packed rows (variable-length batches)."""

    def __init__(self, layers, d_model, seq_len, batch):
        self.layers = list(layers)
        n = len(self.layers)
        hs = (C.c_void_p * n)(*[l._h for l in self.layers])
        h = C.c_void_p()
        check(lib().et_encoder_stack_create(C.byref(h), hs, n, d_model, seq_len, batch))
        self._h = h
        self.act = None
        self.shape = (batch * seq_len, d_model)

    def set_seq_lens(self, lens):
        for l in self.layers:
            l.set_seq_lens(lens)

    def run(self, out, inp):
        if self.act is None or self.act.device != inp.device:
            self.act = torch.empty(self.shape, dtype=torch.float16, device=inp.device)
        check(lib().et_encoder_stack_run(self._h, _dp2(out, *self.shape, "Encoder_stack.run out"),
                                         _dp2(inp, *self.shape, "Encoder_stack.run inp"), _dp(self.act), _stream()))
        return out

    def __del__(self):
        if getattr(self, "_h", None):
            lib().et_encoder_stack_destroy(self._h)
            self._h = None
