"""Pins for the oracle's arithmetic (CPU only).

No reference golden vectors exist for this path, so each op is pinned against
what the mathematics fixes: numpy/torch textbook routines in float64, closed
forms, brute force on tiny inputs and invariants — chosen so that a dropped
term, a transposed operand or a wrong index fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch

import oracle.et_oracle as orc
from helpers import rng, randn_h, make_tile_linear, dense_masked, check_close

HALF_EPS = 2.0 ** -11  # relative rounding error of one fp16 rounding


# ------------------------------------------------------------------ tile GEMM
@pytest.mark.parametrize("sp", [0.0, 0.5, 0.8, 0.9])
def test_tile_linear_equals_dense_with_zeroed_tiles(sp):
    r = rng(10)
    M, N, K = 48, 96, 160
    lin = make_tile_linear(r, N, K, sp, seed=3, std=0.1, bias_std=0.5)
    X = randn_h(r, (M, K))
    want = X.astype(np.float64) @ dense_masked(lin).T + lin["bias"].astype(np.float64)
    for f64 in (False, True):
        got = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, f64=f64)
        # one fp16 rounding of the exact result (+ fp32 accumulation noise)
        assert np.abs(got.astype(np.float64) - want).max() <= np.abs(want).max() * HALF_EPS * 1.01 + 1e-6
    # f64 oracle is the correctly rounded exact result
    got64 = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, f64=True)
    assert np.array_equal(got64, want.astype(np.float16))


def test_tile_linear_bruteforce_32():
    r = rng(11)
    M = N = K = 32
    lin = make_tile_linear(r, N, K, 0.5, seed=8, std=1.0, bias_std=1.0)
    X = randn_h(r, (M, K))
    rp, ro, data = lin["row_ptr"], lin["row_offset"], lin["data"].astype(np.float64)
    want = np.zeros((M, N))
    for m in range(M):
        for bn in range(N // 16):
            for n in range(16):
                s = 0.0
                for i in range(rp[bn], rp[bn + 1]):
                    for k in range(16):
                        s += float(X[m, ro[i] + k]) * data[i * 256 + n * 16 + k]
                want[m, bn * 16 + n] = s + float(lin["bias"][bn * 16 + n])
    got = orc.tile_linear(X, rp, ro, lin["data"], lin["bias"], N, f64=True)
    assert np.array_equal(got, want.astype(np.float16))


def test_tile_linear_reference_smoke_closed_form():
    """weights = bias = 0.1 (test/gen_linear.cu:8,10): Y = 0.1*sum_{kept k} X + 0.1"""
    r = rng(12)
    M, N, K = 16, 64, 128
    rp, ro = orc.gen_sparse_tile_mat(N, K, 0.5, seed=2)
    data = np.full(ro.size * 256, 0.1, np.float16)
    bias = np.full(N, 0.1, np.float16)
    X = randn_h(r, (M, K))
    got = orc.tile_linear(X, rp, ro, data, bias, N, f64=True)
    c = float(np.float16(0.1))
    for bn in range(N // 16):
        cols = np.concatenate([np.arange(o, o + 16) for o in ro[rp[bn]:rp[bn + 1]]]) if rp[bn + 1] > rp[bn] else np.array([], int)
        want = (c * X[:, cols].astype(np.float64).sum(1) + c).astype(np.float16)
        assert np.array_equal(got[:, bn * 16:(bn + 1) * 16], np.repeat(want[:, None], 16, 1))


def test_tile_linear_empty_block_row_gives_bias():
    r = rng(13)
    N, K, M = 32, 32, 16
    rp = np.array([0, 0, 2], np.int32)
    ro = np.array([16, 0], np.int32)
    data = randn_h(r, (2 * 256,))
    bias = randn_h(r, (N,))
    X = randn_h(r, (M, K))
    got = orc.tile_linear(X, rp, ro, data, bias, N)
    assert np.array_equal(got[:, :16], np.repeat(bias[None, :16], M, 0))
    assert not np.array_equal(got[:, 16:], np.repeat(bias[None, 16:], M, 0))


def test_row_linear_equals_numpy():
    r = rng(14)
    M, N, K = 40, 48, 96
    X, W, b = randn_h(r, (M, K)), randn_h(r, (N, K), 0.1), randn_h(r, (N,))
    want = X.astype(np.float64) @ W.astype(np.float64).T + b.astype(np.float64)
    assert np.array_equal(orc.row_linear(X, W, b, f64=True), want.astype(np.float16))
    check_close(orc.row_linear(X, W, b), want, max_abs=np.abs(want).max() * HALF_EPS * 1.01 + 1e-6, what="row_linear f32")


# ----------------------------------------------------------------------- GELU
def test_gelu_closed_forms_and_fp64():
    x = np.array([0.0, -0.0, 10.0, -10.0, 1.0, -1.0, 0.5, 3.0, -3.0, 60000.0, -60000.0], np.float16)
    g = orc.gelu(x).astype(np.float64)
    assert g[0] == 0 and g[1] == 0
    assert g[2] == 10.0 and g[3] == 0.0          # tanh saturates: x*1, x*0
    assert abs(g[4] - 0.8411919906) < 1e-3 and abs(g[5] + 0.1588080094) < 1e-3   # tanh-form GELU(+-1)
    assert g[9] == 60000.0 and g[10] == 0.0      # x^3 overflows to inf in half; tanh(+-inf)=+-1 (kernels/linear.cu:37)
    xs = np.linspace(-8, 8, 4001).astype(np.float16)
    xd = xs.astype(np.float64)
    want = 0.5 * xd * (1 + np.tanh(math.sqrt(2 / math.pi) * (xd + 0.044715 * xd ** 3)))
    got = orc.gelu(xs).astype(np.float64)
    # three half roundings (x^3, 0.5(1+tanh), product): a few half ulps
    assert np.abs(got - want).max() <= 4 * HALF_EPS * np.abs(want).max() + 2e-3
    assert (np.abs(got - want) / np.maximum(np.abs(want), 1e-2)).mean() < 1e-3


def test_gelu_fused_in_tile_linear():
    r = rng(15)
    M, N, K = 16, 32, 64
    lin = make_tile_linear(r, N, K, 0.0, seed=1, std=0.3, bias_std=0.3)
    X = randn_h(r, (M, K))
    plain = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N)
    fused = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, gelu=True)
    assert np.array_equal(fused, orc.gelu(plain))   # gelu acts on the half-rounded sum (kernels/linear.cu:146-149)


# -------------------------------------------------------------------- skip-LN
def test_skip_layernorm_vs_fp64_and_invariants():
    r = rng(16)
    rows, d = 33, 768
    a, s = randn_h(r, (rows, d)), randn_h(r, (rows, d))
    g, b = randn_h(r, (d,), 0.5) + np.float16(1), randn_h(r, (d,), 0.5)
    x = (a.astype(np.float64) + s.astype(np.float64)).astype(np.float16).astype(np.float64)  # half(a+skip), :20
    mu = x.mean(1, keepdims=True)
    var = ((x - mu) ** 2).mean(1, keepdims=True)     # biased, :29-33
    want = (x - mu) / np.sqrt(var + 1e-6) * g.astype(np.float64) + b.astype(np.float64)
    got64 = orc.skip_layernorm(a, s, g, b, f64=True)
    # eps is 1e-6f (a float literal) in the reference; allow that last-bit difference
    assert np.abs(got64.astype(np.float64) - want).max() <= HALF_EPS * np.abs(want).max()
    assert (got64 != want.astype(np.float16)).mean() < 1e-3
    got32 = orc.skip_layernorm(a, s, g, b)
    assert (got32 != got64).mean() < 5e-3 and np.abs(got32.astype(np.float64) - want).max() <= 2 * HALF_EPS * np.abs(want).max()
    one, zero = np.ones(d, np.float16), np.zeros(d, np.float16)
    y = orc.skip_layernorm(a, s, one, zero).astype(np.float64)
    assert np.abs(y.mean(1)).max() < 2e-3 and np.abs(y.var(1) - 1).max() < 5e-3
    # constant row: x - mean == 0 -> output is beta exactly
    const = np.full((2, d), 0.75, np.float16)
    assert np.array_equal(orc.skip_layernorm(const, const, g, b), np.repeat(b[None], 2, 0))
    # torch's layer_norm as a library cross-check
    tw = torch.nn.functional.layer_norm(torch.from_numpy(x), (d,), torch.from_numpy(g.astype(np.float64)),
                                        torch.from_numpy(b.astype(np.float64)), eps=1e-6).numpy()
    assert np.abs(got64.astype(np.float64) - tw).max() <= HALF_EPS * np.abs(tw).max()


# ------------------------------------------------------------------ attention
def _np_attention(Q, K, V, mask, S, H, batch, lens, log2_scale):
    d = Q.shape[1]
    hd = d // H
    scale = float(np.float16(np.sqrt(np.float32(1.0) / np.float32(hd))))
    Qs = (Q.astype(np.float32) * np.float32(scale)).astype(np.float16).astype(np.float64)
    Kd, Vd = K.astype(np.float64), V.astype(np.float64)
    out = np.zeros((batch * S, d))
    for b in range(batch):
        L = S if lens is None else int(lens[b])
        for h in range(H):
            sl = slice(h * hd, (h + 1) * hd)
            q, k, v = Qs[b * S:b * S + L, sl], Kd[b * S:b * S + L, sl], Vd[b * S:b * S + L, sl]
            s = q @ k.T
            if mask is not None:
                s = s + mask.astype(np.float64)[:L, :L]
            p = np.exp2((s - s.max(1, keepdims=True)) * log2_scale)
            out[b * S:b * S + L, sl] = (p / p.sum(1, keepdims=True)) @ v
    return out


@pytest.mark.parametrize("log2_scale", [1.0, math.log2(math.e)])
def test_otf_attention_vs_numpy_fp64(log2_scale):
    r = rng(20)
    S, H, d, B = 48, 3, 96, 2
    Q, K, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S))
    lens = np.array([48, 29], np.int32)
    want = _np_attention(Q, K, V, mask, S, H, B, lens, log2_scale)
    got = orc.otf_attention(Q, K, V, mask, S, H, B, lens, log2_scale, f64=True)
    assert np.array_equal(got, want.astype(np.float16)) or np.abs(got.astype(np.float64) - want).max() < 1e-3
    assert (got[S + 29:] == 0).all()                 # padded query rows are +0
    got32 = orc.otf_attention(Q, K, V, mask, S, H, B, lens, log2_scale)
    check_close(got32, want, max_abs=2e-3, mean_rel=1e-3, what="otf f32")


def test_attention_textbook_mode_equals_torch_softmax_and_base2_identity():
    r = rng(21)
    S, H, d = 32, 2, 64
    Q, K, V = (randn_h(r, (S, d)) for _ in range(3))
    hd = d // H
    scale = float(np.float16(1 / math.sqrt(hd)))
    for mode, mult in ((math.log2(math.e), 1.0), (1.0, math.log(2.0))):
        got = orc.otf_attention(Q, K, V, None, S, H, log2_scale=mode, f64=True).astype(np.float64)
        for h in range(H):
            sl = slice(h * hd, (h + 1) * hd)
            qs = (Q[:, sl].astype(np.float32) * np.float32(scale)).astype(np.float16)
            s = torch.from_numpy(qs.astype(np.float64)) @ torch.from_numpy(K[:, sl].astype(np.float64)).T
            # base-2 softmax == softmax(ln2 * s)  (kernels/attention.cu:33)
            want = (torch.softmax(s * mult, -1) @ torch.from_numpy(V[:, sl].astype(np.float64))).numpy()
            assert np.abs(got[:, sl] - want).max() <= HALF_EPS * max(1.0, np.abs(want).max())


def test_attention_closed_forms():
    r = rng(22)
    S, H, d = 32, 4, 64
    V = randn_h(r, (S, d))
    K = randn_h(r, (S, d))
    zeroQ = np.zeros((S, d), np.float16)
    # uniform scores -> every output row is the column mean of V
    got = orc.otf_attention(zeroQ, K, V, None, S, H, f64=True).astype(np.float64)
    want = np.repeat(V.astype(np.float64).mean(0, keepdims=True), S, 0)
    assert np.abs(got - want).max() <= HALF_EPS * 2
    # one-hot additive mask: row q attends only to key (q*7)%S -> Z[q] = V[that key]
    mask = np.full((S, S), -60000.0, np.float16)
    tgt = (np.arange(S) * 7) % S
    mask[np.arange(S), tgt] = 0
    got = orc.otf_attention(randn_h(r, (S, d)), K, V, mask, S, H, f64=True)
    assert np.array_equal(got, V[tgt])
    # rows of P sum to 1: with V = ones the output is exactly 1
    ones = np.ones((S, d), np.float16)
    got = orc.otf_attention(randn_h(r, (S, d)), K, ones, randn_h(r, (S, S)), S, H)
    assert np.abs(got.astype(np.float64) - 1).max() <= HALF_EPS
    # shift invariance: adding a per-row constant to the mask changes nothing
    Q = randn_h(r, (S, d))
    m0 = randn_h(r, (S, S), 0.5).astype(np.float64)
    shift = np.arange(S)[:, None] * 0.25
    a = orc.otf_attention(Q, K, V, m0.astype(np.float16), S, H, f64=True)
    b = orc.otf_attention(Q, K, V, (m0 + shift).astype(np.float16), S, H, f64=True)
    assert np.abs(a.astype(np.float64) - b.astype(np.float64)).max() < 2e-2   # mask rounding only


def test_attention_bruteforce_16():
    r = rng(23)
    S, H, d = 16, 1, 16
    Q, K, V = (randn_h(r, (S, d)) for _ in range(3))
    mask = randn_h(r, (S, S))
    scale = float(np.float16(0.25))
    want = np.zeros((S, d))
    for q in range(S):
        s = [sum(float(np.float16(np.float32(Q[q, e]) * np.float32(scale))) * float(K[k, e]) for e in range(d)) + float(mask[q, k]) for k in range(S)]
        m = max(s)
        p = [2.0 ** (v - m) for v in s]
        for e in range(d):
            want[q, e] = sum(p[k] * float(V[k, e]) for k in range(S)) / sum(p)
    got = orc.otf_attention(Q, K, V, mask, S, H, f64=True)
    assert np.abs(got.astype(np.float64) - want).max() <= HALF_EPS * max(1, np.abs(want).max())


def test_prune_attention_equals_dense_with_zeroed_columns():
    r = rng(24)
    S, H, d, B = 32, 4, 64, 2
    hd = d // H
    Q, K, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.3)
    qk_id = orc.gen_head_balanced_rows(H, hd, 8, seed=1)       # same kept set for Q and K
    v_id = np.sort(rng(5).choice(d, 37, replace=False)).astype(np.int32)
    qk_hp, v_hp = orc.head_ptr(qk_id, H, hd), orc.head_ptr(v_id, H, hd)
    Qc, Kc, Vc = Q[:, qk_id], K[:, qk_id], V[:, v_id]
    got = orc.prune_attention(Qc, Kc, Vc, qk_hp, v_id, v_hp, mask, S, d, H, B, f64=True)
    Qz, Kz, Vz = np.zeros_like(Q), np.zeros_like(K), np.zeros_like(V)
    Qz[:, qk_id], Kz[:, qk_id], Vz[:, v_id] = Qc, Kc, Vc
    want = orc.otf_attention(Qz, Kz, Vz, mask, S, H, B, f64=True)
    assert np.array_equal(got, want)
    other = np.setdiff1d(np.arange(d), v_id)
    assert (got[:, other] == 0).all()
    # reference wiring (encoder/encoder.cu:76-79): dense Q,K, compact V only
    got2 = orc.prune_attention(Q, K, Vc, None, v_id, v_hp, mask, S, d, H, B, f64=True)
    assert np.array_equal(got2, orc.otf_attention(Q, K, Vz, mask, S, H, B, f64=True))


def test_sharedqk_attention_equals_otf_up_to_score_rounding():
    r = rng(25)
    S, H, d = 32, 2, 64
    Q, K, V = (randn_h(r, (S, d), 0.5) for _ in range(3))
    mask = randn_h(r, (S, S), 0.3)
    QK = orc.qk_scores(Q, K, S, H)
    hd = d // H
    for h in range(H):  # textbook scaled QK^T
        want = Q[:, h * hd:(h + 1) * hd].astype(np.float64) @ K[:, h * hd:(h + 1) * hd].astype(np.float64).T * float(np.float16(1 / math.sqrt(hd)))
        assert np.abs(QK[h].astype(np.float64) - want).max() <= HALF_EPS * np.abs(want).max() * 1.01
    a = orc.sharedqk_attention(QK, V, mask, S, H, f64=True)
    b = orc.otf_attention(Q, K, V, mask, S, H, f64=True)
    check_close(a, b, max_abs=5e-3, mean_rel=2e-3, what="sharedQK vs OTF")
    # and exactly: softmax2(QK+mask) V in numpy
    p = np.exp2(QK.astype(np.float64) + mask.astype(np.float64)[None])
    p = p / p.sum(-1, keepdims=True)
    for h in range(H):
        want = p[h] @ V[:, h * hd:(h + 1) * hd].astype(np.float64)
        assert np.abs(a[:, h * hd:(h + 1) * hd].astype(np.float64) - want).max() <= HALF_EPS * max(1, np.abs(want).max())


# ---------------------------------------------------------------- whole layer
def test_encoder_layer_is_the_composition_of_its_steps():
    r = rng(30)
    S, H, d, dff, B = 32, 2, 64, 256, 2
    shapes = [(d, d)] * 4 + [(dff, d), (d, dff)]
    lins = [make_tile_linear(r, n, k, 0.5, seed=40 + j, std=0.1, bias_std=0.1) for j, (n, k) in enumerate(shapes)]
    ln = [randn_h(r, (d,), 0.2) + np.float16(1), randn_h(r, (d,), 0.2), randn_h(r, (d,), 0.2) + np.float16(1), randn_h(r, (d,), 0.2)]
    x = randn_h(r, (B * S, d))
    mask = randn_h(r, (S, S), 0.2)
    lens = np.array([32, 20], np.int32)
    got = orc.encoder_tile_layer(x, lins, ln, mask, S, H, B, lens)
    tl = lambda j, inp, g=False: orc.tile_linear(inp, lins[j]["row_ptr"], lins[j]["row_offset"], lins[j]["data"], lins[j]["bias"], lins[j]["N"], gelu=g)
    q, k, v = tl(0, x), tl(1, x), tl(2, x)                        # encoder/encoder.cu:22-26
    z = orc.otf_attention(q, k, v, mask, S, H, B, lens)           # :31-32
    h1 = orc.skip_layernorm(tl(3, z), x, ln[0], ln[1])            # :34-37
    y = orc.skip_layernorm(tl(5, tl(4, h1, True)), h1, ln[2], ln[3])  # :39-44
    assert np.array_equal(got, y)
    # fp32 vs fp64 host loops stay well inside the activation tolerance
    got64 = orc.encoder_tile_layer(x, lins, ln, mask, S, H, B, lens, f64=True)
    check_close(got, got64, what="layer f32 vs f64")
