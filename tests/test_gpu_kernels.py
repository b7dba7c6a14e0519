"""Parity of the HIP kernels (through the C ABI) against the CPU oracle.

Integer/index data must match bit for bit; fp16 activations within
max-abs 2e-2 / mean-rel 1e-3 (helpers.MAX_ABS / MEAN_REL), usually far tighter.
"""
import math

import numpy as np
import pytest
import torch

import oracle.et_oracle as orc
from helpers import rng, randn_h, make_tile_linear, check_close

pytestmark = pytest.mark.gpu

LOG2E = math.log2(math.e)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


@pytest.fixture(scope="module")
def K():
    from et_amd import kernels
    return kernels


# ------------------------------------------------------------------ skip-LN
@pytest.mark.parametrize("rows,size", [(128, 768), (1000, 768), (33, 1024), (5, 2048), (7, 4096), (9, 64), (6, 100), (3, 8200)])
def test_skip_layernorm(K, rows, size):
    r = rng(100 + rows)
    a, s = randn_h(r, (rows, size)), randn_h(r, (rows, size))
    g, b = randn_h(r, (size,), 0.3) + np.float16(1), randn_h(r, (size,), 0.3)
    want = orc.skip_layernorm(a, s, g, b)
    got = host(K.skip_layernorm(dev(a), dev(s), dev(g), dev(b)))
    check_close(got, want, max_abs=4e-3, mean_rel=2e-4, what=f"skip_ln {rows}x{size}")
    assert (got != want).mean() < 0.02   # fp32 reduction order only


def test_skip_layernorm_streaming_form(K):
    """operands beyond the last-level cache take non-temporal loads: same bits as the ordinary form"""
    from et_amd import lib
    rows, size = 90000, 768          # 2 x 138 MB of operands
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randn((rows, size), device="cuda", generator=g).to(torch.float16)
    s = torch.randn((rows, size), device="cuda", generator=g).to(torch.float16)
    gam = (torch.randn(size, device="cuda", generator=g) * 0.3 + 1).to(torch.float16)
    bet = (torch.randn(size, device="cuda", generator=g) * 0.3).to(torch.float16)
    got = a.clone()
    K.skip_layernorm(got, s, gam, bet)
    try:
        lib().et_tuning_set(b"ln_rows", 2)   # a fixed row count per wave also keeps the ordinary loads
        ref = a.clone()
        K.skip_layernorm(ref, s, gam, bet)
    finally:
        lib().et_tuning_set(b"ln_rows", 0)
    assert torch.equal(got, ref)
    sel = np.r_[0:40, rows - 40:rows]
    want = orc.skip_layernorm(host(a[sel]), host(s[sel]), host(gam), host(bet), f64=True)
    check_close(host(got[sel]), want, what="skip + LayerNorm, streaming form")


def test_skip_layernorm_constant_row_and_unit_stats(K):
    d = 768
    g, b = np.ones(d, np.float16), np.zeros(d, np.float16)
    r = rng(7)
    beta = randn_h(r, (d,))
    const = np.full((4, d), 0.75, np.float16)
    assert np.array_equal(host(K.skip_layernorm(dev(const), dev(const), dev(g), dev(beta))), np.repeat(beta[None], 4, 0))
    a, s = randn_h(r, (64, d)), randn_h(r, (64, d))
    y = host(K.skip_layernorm(dev(a), dev(s), dev(g), dev(b))).astype(np.float64)
    assert np.abs(y.mean(1)).max() < 2e-3 and np.abs(y.var(1) - 1).max() < 5e-3


# --------------------------------------------------------------- tile linear
TILE_CASES = [
    # M, N, K, sparsity, gelu
    (128, 768, 768, 0.0, False),      # dense BERT projection (config 1 shape)
    (100, 768, 768, 0.8, False),      # M not a multiple of the row panel
    (64, 3072, 768, 0.5, True),       # FFN1 with GELU
    (64, 768, 3072, 0.8, False),      # FFN2: K walked in chunks
    (16, 16, 16, 0.0, False),         # one tile
    (48, 64, 96, 0.95, False),        # mostly empty block-rows
    (32, 32, 32, 1.0, True),          # no tile at all: Y = gelu(bias)
    (1, 128, 1024, 0.3, False),       # single row, odd tile counts
    (257, 1040, 1008, 0.6, True),     # ragged everything, largest single-panel K
    (40, 48, 1024, 0.5, False),       # smallest K that needs two chunks
]


@pytest.mark.parametrize("M,N,Kd,sp,gelu", TILE_CASES)
def test_tile_linear_raw_and_planned(K, M, N, Kd, sp, gelu):
    from et_amd.encoder import Linear_tile
    r = rng(200 + M + N)
    lin = make_tile_linear(r, N, Kd, sp, seed=M + N + Kd, std=0.05, bias_std=0.2)
    X = randn_h(r, (M, Kd))
    want = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, gelu=gelu)
    want64 = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, gelu=gelu, f64=True)
    Xd = dev(X)
    got = host(K.tile_spmm_add_bias(Xd, dev(lin["row_ptr"]), dev(lin["row_offset"]) if lin["row_offset"].size else None,
                                    dev(lin["data"]) if lin["data"].size else None, dev(lin["bias"]), N, gelu=gelu))
    tol = max(np.abs(want64.astype(np.float64)).max() * 2.0 ** -10, 1e-3)
    check_close(got, want64, max_abs=tol, mean_rel=5e-4, what="tile raw vs f64")
    check_close(got, want, max_abs=tol, mean_rel=5e-4, what="tile raw vs f32")
    lt = Linear_tile(Kd, N, M, lin["row_offset"].size, lin["data"], lin["row_ptr"], lin["row_offset"], lin["bias"], gelu)
    got2 = host(lt.run(Xd))
    check_close(got2, want64, max_abs=tol, mean_rel=5e-4, what="tile planned vs f64")


def test_magnitude_pruned_linear_through_container(K, tmp_path):
    """dense W -> et_prune_tile_mat -> et_tile_pack -> container file -> Linear_tile == oracle on the same tile_mat,
    and == the dense product with the dropped tiles zeroed"""
    from et_amd import formats
    from et_amd.encoder import Linear_tile
    r = rng(77)
    M, N, Kd = 200, 768, 768
    W = (r.standard_normal((N, Kd)) * 0.05 * (1 + (np.arange(N)[:, None] // 16 + np.arange(Kd)[None, :] // 16) % 5)).astype(np.float16)
    bias = randn_h(r, (N,), 0.2)
    rp, ro = formats.prune_tile_mat(W, 0.8)
    assert ro.size == 460
    formats.tile_mat_save(tmp_path / "o.ettile", Kd, N, rp, ro, formats.tile_pack(W, rp, ro), bias)
    t = formats.tile_mat_load(tmp_path / "o.ettile")
    X = randn_h(r, (M, Kd))
    lt = Linear_tile(Kd, N, M, t["row_offset"].size, t["data"], t["row_ptr"], t["row_offset"], t["bias"], False)
    got = host(lt.run(dev(X)))
    want = orc.tile_linear(X, t["row_ptr"], t["row_offset"], t["data"], t["bias"], N, f64=True)
    tol = max(np.abs(want.astype(np.float64)).max() * 2.0 ** -10, 1e-3)
    check_close(got, want, max_abs=tol, mean_rel=5e-4, what="magnitude-pruned linear")
    Wz = np.zeros_like(W)
    for bn in range(N // 16):
        for o in t["row_offset"][t["row_ptr"][bn]:t["row_ptr"][bn + 1]]:
            Wz[bn * 16:(bn + 1) * 16, o:o + 16] = W[bn * 16:(bn + 1) * 16, o:o + 16]
    dense = X.astype(np.float64) @ Wz.astype(np.float64).T + bias.astype(np.float64)
    check_close(got, dense.astype(np.float16), max_abs=tol, mean_rel=5e-4, what="vs dense with zeroed tiles")


LN_CASES = [
    # M, N, K, sparsity
    (128, 768, 768, 0.8),     # O projection + LayerNorm (resident panel, 3 block-rows per wave)
    (100, 768, 3072, 0.8),    # FFN2 + LayerNorm, K in chunks, ragged M
    (64, 256, 256, 0.5),      # one block-row per wave
    (40, 512, 1024, 0.6),     # two block-rows per wave, chunked K
    (33, 1024, 512, 0.7),     # four
    (70, 1536, 768, 0.9),     # six: the widest fused row
    (20, 48, 64, 0.0),        # most waves own nothing
    (50, 2048, 256, 0.8),     # too wide for one workgroup: two launches
]


@pytest.mark.parametrize("M,N,Kd,sp", LN_CASES)
def test_tile_linear_fused_skip_layernorm(K, M, N, Kd, sp):
    """Linear_tile.run_ln == skip_layernorm(tile_linear(x), skip) of the oracle"""
    from et_amd.encoder import Linear_tile
    r = rng(900 + M + N)
    lin = make_tile_linear(r, N, Kd, sp, seed=3 * M + N + Kd, std=0.05, bias_std=0.2)
    X, skip = randn_h(r, (M, Kd)), randn_h(r, (M, N))
    g, b = randn_h(r, (N,), 0.3) + np.float16(1), randn_h(r, (N,), 0.3)
    y = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N)
    want = orc.skip_layernorm(y, skip, g, b)
    want64 = orc.skip_layernorm(y, skip, g, b, f64=True)
    lt = Linear_tile(Kd, N, M, lin["row_offset"].size, lin["data"], lin["row_ptr"], lin["row_offset"], lin["bias"], False)
    got = host(lt.run_ln(dev(X), dev(skip), dev(g), dev(b)))
    check_close(got, want64, what="fused linear+LN vs f64")
    check_close(got, want, what="fused linear+LN vs f32")
    # against the two separate launches of this library: same linear, same
    # LayerNorm arithmetic, only the summation order of the row statistics differs
    two = lt.run(dev(X))
    K.skip_layernorm(two, dev(skip), dev(g), dev(b))
    two = host(two)
    assert np.abs(got.astype(np.float32) - two.astype(np.float32)).max() <= 2.0 ** -7
    assert (got != two).mean() < 0.02
    if N <= 1536:  # fused: the output may overwrite the skip operand
        sk = dev(skip)
        lt.run_ln(dev(X), sk, dev(g), dev(b), out=sk)
        inplace = host(sk)
        if M > 256:
            assert np.array_equal(inplace, got)
        else:
            # few rows: the call above ran the few-rows linear (a block-row's products summed in four
            # parts) and the LayerNorm kernel, the in-place call the fused kernel - other summation order
            assert np.abs(inplace.astype(np.float32) - got.astype(np.float32)).max() <= 2.0 ** -7
            assert (inplace != got).mean() < 0.02


FFN_CASES = [
    # M, d (in = out), hidden, sparsity, fused kernel expected
    (128, 768, 3072, 0.8, True),    # BERT-base block: four hidden chunks of 768
    (100, 768, 3072, 0.5, True),    # ragged M, denser
    (70, 256, 1024, 0.6, True),     # two chunks, narrow rows: most waves own nothing in the second linear
    (33, 512, 768, 0.7, True),      # hidden width in ONE chunk
    (40, 768, 1536 + 256, 0.8, True),  # last hidden chunk partial (256 of 768 columns)
    (64, 64, 3072, 0.9, True),      # tiny model width, many empty block-rows
    (45, 80, 400, 0.5, True),       # widths that are multiples of 16 but not of 32 (unpadded LDS rows)
    (32, 768, 768 * 17, 0.95, False),  # more hidden chunks than the kernel's event counters: step by step
    (50, 768, 896, 0.8, False),     # one hidden chunk of 896 columns: too wide for the fused kernel
    (36, 1024, 2048, 0.8, False),   # model width beyond one LDS panel
]


@pytest.mark.parametrize("M,d,F,sp,fused", FFN_CASES)
def test_tile_ffn_fused_gelu_linear_layernorm(K, M, d, F, sp, fused):
    """Linear_tile.run_ffn_ln == skip_layernorm(tile_linear(gelu(tile_linear(x))), skip) of the oracle"""
    from et_amd.encoder import Linear_tile
    r = rng(1700 + M + d)
    l1 = make_tile_linear(r, F, d, sp, seed=5 * M + F, std=0.05, bias_std=0.2)
    l2 = make_tile_linear(r, d, F, sp, seed=7 * M + d, std=0.05, bias_std=0.2)
    X = randn_h(r, (M, d))
    g, b = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    h = orc.tile_linear(X, l1["row_ptr"], l1["row_offset"], l1["data"], l1["bias"], F, gelu=True)
    y = orc.tile_linear(h, l2["row_ptr"], l2["row_offset"], l2["data"], l2["bias"], d)
    want = orc.skip_layernorm(y, X, g, b)
    t1 = Linear_tile(d, F, M, l1["row_offset"].size, l1["data"], l1["row_ptr"], l1["row_offset"], l1["bias"], True)
    t2 = Linear_tile(F, d, M, l2["row_offset"].size, l2["data"], l2["row_ptr"], l2["row_offset"], l2["bias"], False)
    assert Linear_tile.ffn_fusable(t1, t2) == fused
    xd = dev(X)
    if fused:
        got = host(Linear_tile.run_ffn_ln(t1, t2, xd, xd, dev(g), dev(b)))  # no hidden buffer: fused or error
    else:
        with pytest.raises(Exception):
            Linear_tile.run_ffn_ln(t1, t2, xd, xd, dev(g), dev(b))
        hid = torch.empty((M, F), dtype=torch.float16, device="cuda")
        got = host(Linear_tile.run_ffn_ln(t1, t2, xd, xd, dev(g), dev(b), hidden=hid))
    check_close(got, want, what="fused feed-forward vs oracle chain")
    # against the separate launches of this library: the hidden activations are
    # rounded to half at the same point, so only fp32 summation order differs
    hid = t1.run(xd)
    sep = host(t2.run_ln(hid, xd, dev(g), dev(b)))
    assert np.abs(got.astype(np.float32) - sep.astype(np.float32)).max() <= 2.0 ** -6
    assert (got != sep).mean() < 0.03
    if fused:  # in place over the input, which is also the skip operand
        xd2 = dev(X)
        Linear_tile.run_ffn_ln(t1, t2, xd2, xd2, dev(g), dev(b), out=xd2)
        assert np.array_equal(host(xd2), got)


TAIL_CASES = [
    # M, d, hidden, sparsity, fused kernel expected
    (128, 768, 3072, 0.8, True),   # BERT-base layer tail
    (77, 768, 3072, 0.5, True),    # ragged M
    (40, 256, 1024, 0.7, True),    # narrow rows: most waves own nothing in the projections
    (64, 64, 1536, 0.9, True),     # many empty block-rows
    (45, 80, 400, 0.5, True),      # widths that are multiples of 16 but not of 32 (unpadded LDS rows)
    (1, 768, 3072, 0.8, True),     # a single row
    (50, 768, 896, 0.8, False),    # hidden chunk too wide: step by step
]


@pytest.mark.parametrize("M,d,F,sp,fused", TAIL_CASES)
def test_tile_layer_tail_fused(K, M, d, F, sp, fused):
    """Linear_tile.run_tail == the oracle's O projection, skip+LN, FFN1+GELU, FFN2, skip+LN one after the other"""
    from et_amd.encoder import Linear_tile
    r = rng(2300 + M + d)
    lo = make_tile_linear(r, d, d, sp, seed=3 * M + d, std=0.05, bias_std=0.2)
    l1 = make_tile_linear(r, F, d, sp, seed=5 * M + F, std=0.05, bias_std=0.2)
    l2 = make_tile_linear(r, d, F, sp, seed=7 * M + d, std=0.05, bias_std=0.2)
    attn, inp = randn_h(r, (M, d)), randn_h(r, (M, d))
    g1, b1 = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    g2, b2 = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    o = orc.tile_linear(attn, lo["row_ptr"], lo["row_offset"], lo["data"], lo["bias"], d)
    mid = orc.skip_layernorm(o, inp, g1, b1)
    h = orc.tile_linear(mid, l1["row_ptr"], l1["row_offset"], l1["data"], l1["bias"], F, gelu=True)
    y = orc.tile_linear(h, l2["row_ptr"], l2["row_offset"], l2["data"], l2["bias"], d)
    want = orc.skip_layernorm(y, mid, g2, b2)
    mk = lambda l, K_, N_, gelu: Linear_tile(K_, N_, M, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], gelu)
    to, t1, t2 = mk(lo, d, d, False), mk(l1, d, F, True), mk(l2, F, d, False)
    assert Linear_tile.tail_fusable(to, t1, t2) == fused
    ln = [dev(t) for t in (g1, b1, g2, b2)]
    if fused:
        got = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln))  # no buffers: fused or error
    else:
        with pytest.raises(Exception):
            Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln)
        midb = torch.empty((M, d), dtype=torch.float16, device="cuda")
        hid = torch.empty((M, F), dtype=torch.float16, device="cuda")
        got = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln, mid=midb, hidden=hid))
    # two LayerNorms amplify half-ulp differences of the first one's output
    check_close(got, want, max_abs=3e-2, mean_rel=2e-3, what="fused layer tail vs oracle chain")
    # against this library's separate launches
    midg = to.run_ln(dev(attn), dev(inp), ln[0], ln[1])
    sep = host(t2.run_ln(t1.run(midg), midg, ln[2], ln[3]))
    assert np.abs(got.astype(np.float32) - sep.astype(np.float32)).max() <= 3e-2
    assert (got != sep).mean() < 0.05
    if fused:  # the output may overwrite the attention buffer
        ad = dev(attn)
        Linear_tile.run_tail(to, t1, t2, ad, dev(inp), *ln, out=ad)
        assert np.array_equal(host(ad), got)


PAIR_CASES = [
    (640, 768, 3072, 0.8),     # BERT-base widths, ten 64-row panels
    (200, 256, 1024, 0.5),     # a ragged last panel (8 rows), two block-rows per wave
    (130, 512, 2048, 0.7),     # four block-rows per wave
    (64, 768, 1008, 0.8),      # hidden width that ends inside a 192-column phase
    (96, 256, 384, 0.0),       # dense, one phase per half
    (128, 768, 3072, 0.95),    # block-rows without any tile
]


@pytest.mark.parametrize("mode", [2, 3])
@pytest.mark.parametrize("M,d,F,sp", PAIR_CASES)
def test_tile_layer_tail_pairs(K, M, d, F, sp, mode):
    """the layer tail as pairs of workgroups over 64-row (mode 2) or 32-row (mode 3) panels (scratch given, mid=None insists on it) == the
    oracle's chain of five steps; a second run on the same plans (the per-panel counters reset themselves) and a
    run whose output overwrites the attention buffer give the same bits; close to the one-workgroup form"""
    from et_amd.encoder import Linear_tile
    r = rng(7100 + M + d + F)
    lo = make_tile_linear(r, d, d, sp, seed=3 * M + d, std=0.05, bias_std=0.2)
    l1 = make_tile_linear(r, F, d, sp, seed=5 * M + F, std=0.05, bias_std=0.2)
    l2 = make_tile_linear(r, d, F, sp, seed=7 * M + d, std=0.05, bias_std=0.2)
    attn, inp = randn_h(r, (M, d)), randn_h(r, (M, d))
    g1, b1 = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    g2, b2 = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    o = orc.tile_linear(attn, lo["row_ptr"], lo["row_offset"], lo["data"], lo["bias"], d)
    mid = orc.skip_layernorm(o, inp, g1, b1)
    h = orc.tile_linear(mid, l1["row_ptr"], l1["row_offset"], l1["data"], l1["bias"], F, gelu=True)
    y = orc.tile_linear(h, l2["row_ptr"], l2["row_offset"], l2["data"], l2["bias"], d)
    want = orc.skip_layernorm(y, mid, g2, b2)
    mk = lambda l, K_, N_, gelu: Linear_tile(K_, N_, M, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], gelu)
    to, t1, t2 = mk(lo, d, d, False), mk(l1, d, F, True), mk(l2, F, d, False)
    from et_amd import lib
    ln = [dev(t) for t in (g1, b1, g2, b2)]
    assert Linear_tile.tail_ws_bytes(to, t1, t2, M) == 0          # the paired form is off by default
    lib().et_tuning_set(b"tile_tail_pair", mode)
    try:
        need = Linear_tile.tail_ws_bytes(to, t1, t2, M)
        assert need == ((M + 63) // 64) * 64 * (-(-d // 128) * 128) * 4 * 2   # eight waves x block-rows per wave x 16 columns
        Linear_tile.tail_prepare(to, t1, t2)
        ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")   # NaN patterns: nothing may be read before written
        print(f"pair tail: M={M} d={d} F={F} sp={sp} mode={mode}", flush=True)
        got = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln, ws=ws))
        check_close(got, want, max_abs=3e-2, mean_rel=2e-3, what="paired layer tail vs oracle chain")
        again = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln, ws=ws))
        assert np.array_equal(got, again)
        ad = dev(attn)
        Linear_tile.run_tail(to, t1, t2, ad, dev(inp), *ln, out=ad, ws=ws)
        assert np.array_equal(host(ad), got)
    finally:
        lib().et_tuning_set(b"tile_tail_pair", 0)
    if Linear_tile.tail_fusable(to, t1, t2):
        one = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln))
        assert np.abs(got.astype(np.float32) - one.astype(np.float32)).max() <= 3e-2
        assert (got != one).mean() < 0.05


@pytest.mark.parametrize("paired", [False, True])
def test_fused_tail_reports_a_wait_that_gave_up(K, paired):
    """with a poll limit of zero every bounded LDS wait of the fused layer-tail kernels gives up at once (no wave
    ever misses a signal: the kernels run to their normal end, only without waiting), the status word is set, and
    the NEXT launch of such a kernel returns ET_ERR_HIP once; afterwards the kernels work as before"""
    from et_amd import lib
    from et_amd._lib import EtError
    from et_amd.encoder import Linear_tile
    M, d, F, sp = 256, 768, 3072, 0.8
    r = rng(8800 + paired)
    lo = make_tile_linear(r, d, d, sp, seed=31, std=0.05, bias_std=0.2)
    l1 = make_tile_linear(r, F, d, sp, seed=32, std=0.05, bias_std=0.2)
    l2 = make_tile_linear(r, d, F, sp, seed=33, std=0.05, bias_std=0.2)
    attn, inp = randn_h(r, (M, d)), randn_h(r, (M, d))
    ln = [dev(np.ones(d, np.float16)), dev(np.zeros(d, np.float16))] * 2
    mk = lambda l, K_, N_, gelu: Linear_tile(K_, N_, M, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], gelu)
    to, t1, t2 = mk(lo, d, d, False), mk(l1, d, F, True), mk(l2, F, d, False)
    lib().et_tuning_set(b"tile_tail_pair", 2 if paired else 0)
    ws = None
    try:
        if paired:
            Linear_tile.tail_prepare(to, t1, t2)
            ws = torch.zeros(Linear_tile.tail_ws_bytes(to, t1, t2, M), dtype=torch.uint8, device="cuda")
        run = lambda: host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln, ws=ws))
        good = run()
        assert lib().et_wait_status_take() == 0
        lib().et_tuning_set(b"tile_wait_spin", 0)
        print(f"zero-poll launch, paired={paired}", flush=True)
        run()                                   # ends normally; its waves did not wait for each other
        lib().et_tuning_set(b"tile_wait_spin", -1)
        with pytest.raises(EtError) as e:
            run()
        assert "gave up a bounded wait" in str(e.value)
        assert np.array_equal(run(), good)      # reported once; the kernels are fine
    finally:
        lib().et_tuning_set(b"tile_wait_spin", -1)
        lib().et_tuning_set(b"tile_tail_pair", 0)
        lib().et_wait_status_take()


def test_tile_layer_tail_splits_off_a_small_last_round(K):
    """one workgroup per CU and 32-row panel: a last round of few panels runs step by step behind the fused launch"""
    from et_amd import lib
    from et_amd.encoder import Linear_tile
    cus = lib().et_device_cu_count()
    assert cus > 0
    d, F, sp = 256, 1024, 0.7
    M = cus * 32 + 1607
    r = rng(2900)
    lo = make_tile_linear(r, d, d, sp, seed=11, std=0.05, bias_std=0.2)
    l1 = make_tile_linear(r, F, d, sp, seed=12, std=0.05, bias_std=0.2)
    l2 = make_tile_linear(r, d, F, sp, seed=13, std=0.05, bias_std=0.2)
    attn, inp = randn_h(r, (M, d)), randn_h(r, (M, d))
    g1, b1 = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    g2, b2 = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    mk = lambda l, K_, N_, gelu: Linear_tile(K_, N_, M, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], gelu)
    to, t1, t2 = mk(lo, d, d, False), mk(l1, d, F, True), mk(l2, F, d, False)
    ln = [dev(t) for t in (g1, b1, g2, b2)]
    mid = torch.full((M, d), float("nan"), dtype=torch.float16, device="cuda")
    hid = torch.empty((M, F), dtype=torch.float16, device="cuda")
    got = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln, mid=mid, hidden=hid))
    # the fused launch never writes mid; the rows of the last round go through it
    midh = host(mid)
    assert np.isnan(midh[:cus * 32].astype(np.float32)).all() and np.isfinite(midh[cus * 32:].astype(np.float32)).all()
    rows = np.r_[0:64, cus * 32 - 64:cus * 32 + 64, M - 64:M]
    o = orc.tile_linear(attn[rows], lo["row_ptr"], lo["row_offset"], lo["data"], lo["bias"], d)
    m = orc.skip_layernorm(o, inp[rows], g1, b1)
    h = orc.tile_linear(m, l1["row_ptr"], l1["row_offset"], l1["data"], l1["bias"], F, gelu=True)
    y = orc.tile_linear(h, l2["row_ptr"], l2["row_offset"], l2["data"], l2["bias"], d)
    want = orc.skip_layernorm(y, m, g2, b2)
    check_close(got[rows], want, max_abs=3e-2, mean_rel=2e-3, what="layer tail with a split-off last round")
    # all rows: equal to the fused kernel forced on everything, up to fp32 summation order in the last round
    allf = host(Linear_tile.run_tail(to, t1, t2, dev(attn), dev(inp), *ln))
    assert np.array_equal(allf[:cus * 32], got[:cus * 32])
    assert np.abs(allf.astype(np.float32) - got.astype(np.float32)).max() <= 3e-2


def test_tile_linear_closed_form_reference_smoke_inputs(K):
    """weights = bias = 0.1 (test/gen_linear.cu:8,10): Y = 0.1*sum_{kept k} X + 0.1"""
    r = rng(12)
    M, N, Kd = 64, 768, 768
    rp, ro = orc.gen_sparse_tile_mat(N, Kd, 0.8, seed=2)
    data = np.full(ro.size * 256, 0.1, np.float16)
    bias = np.full(N, 0.1, np.float16)
    X = randn_h(r, (M, Kd))
    got = host(K.tile_spmm_add_bias(dev(X), dev(rp), dev(ro), dev(data), dev(bias), N)).astype(np.float64)
    c = float(np.float16(0.1))
    for bn in range(N // 16):
        cols = np.concatenate([np.arange(o, o + 16) for o in ro[rp[bn]:rp[bn + 1]]]) if rp[bn + 1] > rp[bn] else np.array([], int)
        want = c * X[:, cols].astype(np.float64).sum(1) + c
        assert np.abs(got[:, bn * 16:(bn + 1) * 16] - want[:, None]).max() <= np.abs(want).max() * 2.0 ** -10 + 1e-3


def test_tile_linear_multi_qkv_one_launch(K):
    from et_amd.encoder import Linear_tile, run_multi
    r = rng(31)
    M, d = 200, 768
    lins = [make_tile_linear(r, d, d, 0.8, seed=50 + j, std=0.05, bias_std=0.1) for j in range(3)]
    X = randn_h(r, (M, d))
    lts = [Linear_tile(d, d, M, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"]) for l in lins]
    outs = run_multi(lts, dev(X))
    for l, o in zip(lins, outs):
        want = orc.tile_linear(X, l["row_ptr"], l["row_offset"], l["data"], l["bias"], d, f64=True)
        check_close(host(o), want, max_abs=2e-3, mean_rel=5e-4, what="qkv multi")


@pytest.mark.parametrize("M", [200, 5700])
def test_tile_linear_multi_unequal_widths(K, M):
    """Q and K narrower than V (attention-aware pruning): linears of different widths in one launch,
    with column groups that exist for the widest one only (M = 5700 takes the 64-row kernel)"""
    from et_amd.encoder import Linear_tile, run_multi
    r = rng(33 + M)
    d = 768
    widths = (384, 384, 768)
    lins = [make_tile_linear(r, n, d, sp, seed=60 + j, std=0.05, bias_std=0.1) for j, (n, sp) in enumerate(zip(widths, (0.0, 0.5, 0.5)))]
    X = randn_h(r, (M, d))
    lts = [Linear_tile(d, l["N"], M, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"]) for l in lins]
    outs = [host(o) for o in run_multi(lts, dev(X))]
    rows = np.unique(np.concatenate([np.arange(0, 70), r.integers(0, M, 130), np.arange(M - 70, M)]))
    for l, lt, o in zip(lins, lts, outs):
        assert o.shape == (M, l["N"])
        want = orc.tile_linear(X[rows], l["row_ptr"], l["row_offset"], l["data"], l["bias"], l["N"], f64=True)
        check_close(o[rows], want, max_abs=2e-3, mean_rel=5e-4, what="multi, unequal widths")
        assert np.array_equal(o, host(lt.run(dev(X))))   # the same linear launched alone


@pytest.mark.parametrize("M,N,Kd,sp,gelu", [
    (128, 768, 3072, 0.0, False),   # BERT-base FFN2 on one sequence of 128, dense: four chunks, eight waves per block-row
    (128, 768, 3072, 0.8, False),
    (1, 768, 3072, 0.5, False), (17, 768, 3072, 0.8, True), (100, 256, 1536, 0.5, True),   # two chunks
    (200, 768, 3072, 0.0, True),    # above 128 rows: dense plans only
    (256, 768, 3072, 0.0, False), (64, 768, 6144, 0.8, False),   # eight chunks
    (120, 48, 1040, 0.3, False),    # ragged second chunk (272 columns), three block-rows
])
def test_tile_linear_few_rows_kernel(K, M, N, Kd, sp, gelu):
    """K in several chunks and few rows: 16-row panels, a block-row's pairs split over several waves.
    Against the oracle and against the kernels that take over from 257 rows (forced by the tuning key)."""
    from et_amd import lib
    from et_amd.encoder import Linear_tile
    r = rng(34 + M + Kd)
    lin = make_tile_linear(r, N, Kd, sp, seed=70 + M, std=0.03, bias_std=0.1)
    X = randn_h(r, (M, Kd))
    lt = Linear_tile(Kd, N, M, lin["row_offset"].size, lin["data"], lin["row_ptr"], lin["row_offset"], lin["bias"], gelu)
    want = orc.tile_linear(X, lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, f64=True)
    if gelu:
        want = orc.gelu(want)
    got = host(lt.run(dev(X)))
    try:
        lib().et_tuning_set(b"tile_splitk_rows", 0)
        other = host(lt.run(dev(X)))
    finally:
        lib().et_tuning_set(b"tile_splitk_rows", -1)
    check_close(got, want, max_abs=4e-3, mean_rel=5e-4, what="few-rows kernel")
    check_close(other, want, max_abs=4e-3, mean_rel=5e-4, what="general kernel, few rows")
    assert np.abs(got.astype(np.float32) - other.astype(np.float32)).max() <= 2.0 ** -7


@pytest.mark.parametrize("M,N,Kd,gelu", [
    (1024, 384, 768, False),    # Q / K of the attention-aware pruned layer
    (1100, 240, 768, False),    # ragged rows, columns not a multiple of the 128-wide block
    (2048, 928, 768, True),     # row-pruned FFN1
    (1024, 240, 928, False),    # K = 14.5 steps of 64
    (1500, 16, 32, False),      # the smallest shapes
    (4096, 768, 3072, False),
])
def test_row_linear_dense_gemm(K, M, N, Kd, gelu):
    """from 1024 rows the row-pruned linear runs the register-blocked GEMM kernel: against a float64
    product on a row sample and, everywhere, against the tile kernels on the same operands"""
    from et_amd import lib
    r = rng(35 + N + Kd)
    X, W, b = randn_h(r, (M, Kd)), randn_h(r, (N, Kd), 0.05), randn_h(r, (N,), 0.2)
    assert lib().et_row_spmm_prefers_gemm(M, N, Kd) == 1 and lib().et_row_spmm_prefers_gemm(512, N, Kd) == 0
    got = host(K.row_spmm_add_bias(dev(X), dev(W), dev(b), gelu=gelu))
    try:
        lib().et_tuning_set(b"row_gemm_min_rows", 0)
        other = host(K.row_spmm_add_bias(dev(X), dev(W), dev(b), gelu=gelu))
    finally:
        lib().et_tuning_set(b"row_gemm_min_rows", 1024)
    rows = np.unique(np.concatenate([np.arange(0, 130), r.integers(0, M, 100), np.arange(M - 130, M)]))
    want = (X[rows].astype(np.float64) @ W.astype(np.float64).T + b.astype(np.float64)).astype(np.float16)
    if gelu:
        want = orc.gelu(want)
    check_close(got[rows], want, max_abs=8e-3, mean_rel=5e-4, what="dense GEMM")
    assert np.abs(got.astype(np.float32) - other.astype(np.float32)).max() <= 2.0 ** -6
    assert (got != other).mean() < 0.02


def test_row_linear_multi_one_launch(K):
    r = rng(36)
    M, Kd = 1300, 768
    Ws = [randn_h(r, (n, Kd), 0.05) for n in (384, 384, 240)]
    bs = [randn_h(r, (w.shape[0],), 0.2) for w in Ws]
    X = randn_h(r, (M, Kd))
    outs = K.row_spmm_add_bias_multi(dev(X), [dev(w) for w in Ws], [dev(b) for b in bs])
    for w, b, o in zip(Ws, bs, outs):
        assert np.array_equal(host(o), host(K.row_spmm_add_bias(dev(X), dev(w), dev(b))))
    few = K.row_spmm_add_bias_multi(dev(X[:100]), [dev(w) for w in Ws], [dev(b) for b in bs])   # tile kernels
    for w, b, o in zip(Ws, bs, few):
        want = (X[:100].astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64)).astype(np.float16)
        check_close(host(o), want, max_abs=8e-3, mean_rel=5e-4, what="row linears, few rows")


@pytest.mark.parametrize("sp,ntile", [(0.8, 1843), (0.0, 9216), (0.5, 4608), (0.9, 921)])
def test_tile_linear_full_size_config2_rows_sample(K, sp, ntile):
    """config-2 shape (4096x768 -> 3072) at each sparsity of its sweep: rows are independent, so a row
    sample pins the full-size launch"""
    r = rng(32)
    M, N, Kd = 4096, 3072, 768
    lin = make_tile_linear(r, N, Kd, sp, seed=2024, std=0.02)
    assert lin["row_offset"].size == ntile
    X = randn_h(r, (M, Kd))
    got = host(K.tile_spmm_add_bias(dev(X), dev(lin["row_ptr"]), dev(lin["row_offset"]), dev(lin["data"]), dev(lin["bias"]), N))
    rows = np.sort(r.choice(M, 192, replace=False))
    rows[:3] = [0, 31, 4095]
    want = orc.tile_linear(X[rows], lin["row_ptr"], lin["row_offset"], lin["data"], lin["bias"], N, f64=True)
    check_close(got[rows], want, max_abs=2e-3, mean_rel=5e-4, what="config-2 sample")
    # linearity in X where it is exact in fp16: doubling X doubles Y (bias is 0),
    # except for results in the subnormal range, whose grid does not scale
    got2 = host(K.tile_spmm_add_bias(dev(X * np.float16(2)), dev(lin["row_ptr"]), dev(lin["row_offset"]), dev(lin["data"]), dev(lin["bias"]), N))
    normal = np.abs(got) >= 2.0 ** -13
    assert np.array_equal(got2[normal], (got * np.float16(2))[normal])
    assert np.abs(got2.astype(np.float64) - 2 * got.astype(np.float64))[~normal].max() <= 2.0 ** -23
    # the planned form of the same linear (Linear_tile::run: the 64-row resident kernel that the encoders
    # and the benchmark run at this size), its index arrays from the product's own generator and packer
    from et_amd import formats
    from et_amd.encoder import Linear_tile
    rp, ro = formats.gen_sparse_tile_mat(N, Kd, sp, 2024)
    assert np.array_equal(rp, lin["row_ptr"]) and np.array_equal(ro, lin["row_offset"])
    data = formats.tile_pack(lin["W"], rp, ro)
    assert np.array_equal(data, lin["data"])
    bias = randn_h(r, (N,), 0.1)
    want_b = orc.tile_linear(X[rows], rp, ro, data, bias, N, f64=True)
    planned = host(Linear_tile(Kd, N, M, ro.size, data, rp, ro, bias).run(dev(X)))
    check_close(planned[rows], want_b, max_abs=2e-3, mean_rel=5e-4, what="config-2 sample, planned")
    if sp in (0.8, 0.0):
        want_g = orc.tile_linear(X[rows], rp, ro, data, bias, N, gelu=True, f64=True)
        planned_g = host(Linear_tile(Kd, N, M, ro.size, data, rp, ro, bias, True).run(dev(X)))
        check_close(planned_g[rows], want_g, max_abs=2e-3, mean_rel=5e-4, what="config-2 sample, planned + GELU")


def test_tile_linear_argument_errors(K):
    from et_amd import EtError
    r = rng(33)
    lin = make_tile_linear(r, 32, 32, 0.0, seed=1)
    X = dev(randn_h(r, (16, 32)))
    with pytest.raises(EtError):   # N not a multiple of 16
        K.tile_spmm_add_bias(X, dev(lin["row_ptr"]), dev(lin["row_offset"]), dev(lin["data"]), dev(lin["bias"][:24]), 24)
    with pytest.raises(EtError):   # misaligned X
        K.tile_spmm_add_bias(dev(randn_h(r, (17, 32))).view(-1)[1:1 + 16 * 32].view(16, 32), dev(lin["row_ptr"]),
                             dev(lin["row_offset"]), dev(lin["data"]), dev(lin["bias"]), 32)


# ---------------------------------------------------------------- row linear
@pytest.mark.parametrize("M,N,Kd", [(64, 240, 768), (100, 928, 768), (33, 240, 928), (16, 16, 16), (70, 384, 2048)])
def test_row_linear(K, M, N, Kd):
    r = rng(300 + N)
    X, W, b = randn_h(r, (M, Kd)), randn_h(r, (N, Kd), 0.05), randn_h(r, (N,), 0.2)
    want = orc.row_linear(X, W, b, f64=True)
    got = host(K.row_spmm_add_bias(dev(X), dev(W), dev(b)))
    check_close(got, want, max_abs=max(np.abs(want.astype(np.float64)).max() * 2.0 ** -10, 1e-3), mean_rel=5e-4, what="row linear")


# ------------------------------------------------------------------ attention
ATT_CASES = [
    # S, H, d_model, batch, lens, mask, log2_scale
    (128, 12, 768, 1, None, True, 1.0),            # config-1 shape, reference exponent
    (128, 12, 768, 1, None, False, LOG2E),         # no mask, textbook exponent
    (512, 12, 768, 2, None, True, 1.0),            # config-3 shape (batch cut to 2)
    (512, 12, 768, 3, [512, 77, 300], True, LOG2E),  # per-sequence lengths
    (100, 4, 256, 2, [100, 37], True, 1.0),        # S not a multiple of any tile
    (64, 2, 64, 1, None, True, 1.0),               # head_dim 32
    (96, 2, 256, 2, [96, 50], True, LOG2E),        # head_dim 128
    (16, 1, 64, 1, None, True, 1.0),               # the reference's minimum block
    (200, 12, 768, 1, [0], False, 1.0),            # empty sequence -> zeros
]


@pytest.mark.parametrize("S,H,d,B,lens,use_mask,ls", ATT_CASES)
def test_otf_attention(K, S, H, d, B, lens, use_mask, ls):
    r = rng(400 + S + H)
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S)) if use_mask else None
    lens_np = None if lens is None else np.array(lens, np.int32)
    want = orc.otf_attention(Q, Kk, V, mask, S, H, B, lens_np, ls, f64=True)
    got = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), None if mask is None else dev(mask), S, H, B,
                               None if lens is None else dev(lens_np), ls))
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="OTF attention")
    if lens is not None:
        for b, L in enumerate(lens):
            assert (got[b * S + L:(b + 1) * S] == 0).all()


@pytest.mark.parametrize("S,H,d,B,lens,use_mask,ls", [
    (256, 8, 768, 2, None, False, 1.0),          # head_dim 96, the reference's `tile_test 8 768` shape
    (200, 8, 768, 2, [200, 77], True, LOG2E),
    (128, 8, 384, 1, None, True, 1.0),           # head_dim 48
    (96, 3, 240, 3, [96, 1, 50], True, 1.0),     # head_dim 80
    (64, 2, 224, 1, None, False, 1.0),           # head_dim 112
    (80, 4, 64, 2, [80, 33], True, 1.0),         # head_dim 16
])
def test_otf_attention_other_head_widths(K, S, H, d, B, lens, use_mask, ls):
    """head widths that are multiples of 16 but none of 32 / 64 / 128 (the reference loops over head_dim in steps
    of 16, kernels/attention.cu:86-90) == the oracle; the neighbouring heads' output columns are not touched"""
    r = rng(4400 + S + H + d)
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S)) if use_mask else None
    lens_np = None if lens is None else np.array(lens, np.int32)
    want = orc.otf_attention(Q, Kk, V, mask, S, H, B, lens_np, ls, f64=True)
    print(f"attention head_dim {d // H}: S={S} H={H} B={B}", flush=True)
    got = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), None if mask is None else dev(mask), S, H, B,
                               None if lens is None else dev(lens_np), ls))
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="OTF attention, other head widths")
    if lens is not None:
        for b, L in enumerate(lens):
            assert (got[b * S + L:(b + 1) * S] == 0).all()


def test_otf_attention_closed_forms(K):
    r = rng(41)
    S, H, d = 128, 12, 768
    V, Kk = randn_h(r, (S, d)), randn_h(r, (S, d))
    zeroQ = np.zeros((S, d), np.float16)
    got = host(K.OTF_attention(dev(zeroQ), dev(Kk), dev(V), None, S, H)).astype(np.float64)
    want = np.repeat(V.astype(np.float64).mean(0, keepdims=True), S, 0)
    assert np.abs(got - want).max() < 2e-3            # uniform scores -> column mean of V (P rounded to half)
    mask = np.full((S, S), -60000.0, np.float16)
    tgt = (np.arange(S) * 7) % S
    mask[np.arange(S), tgt] = 0
    got = host(K.OTF_attention(dev(randn_h(r, (S, d))), dev(Kk), dev(V), dev(mask), S, H))
    assert np.array_equal(got, V[tgt])                # one-hot mask -> that V row exactly
    ones = np.ones((S, d), np.float16)
    got = host(K.OTF_attention(dev(randn_h(r, (S, d))), dev(Kk), dev(ones), dev(randn_h(r, (S, S))), S, H))
    assert np.abs(got.astype(np.float64) - 1).max() <= 2.0 ** -10   # rows of P sum to 1


@pytest.mark.parametrize("S", [512, 200, 2100])
def test_attention_mask_summary(K, S):
    """summary bits == any non-zero element per (16 rows, 64 keys); attention with an attached
    summary is bit-identical to attention without, for zero, block-structured and dense masks"""
    r = rng(45 + S)
    H, d, B = 4, 256, 1
    nt, ng = (S + 63) // 64, (S + 15) // 16
    words = (nt + 31) // 32
    mask = np.zeros((S, S), np.float16)
    mask[:, S - S // 3:] = -30000.0               # padding-style: the last third of the keys
    mask[37, 5] = 0.25                            # one stray element
    mask[S - 1, 0] = np.float16(-0.0)             # -0 counts as zero
    md = dev(mask)
    summ = K.attention_mask_summary(md, S)
    got_bits = host(summ).view(np.uint32).reshape(ng, words)
    want_bits = np.zeros((ng, words), np.uint32)
    nz = (mask.view(np.uint16) & 0x7FFF) != 0
    for g in range(ng):
        for t in range(nt):
            if nz[g * 16:(g + 1) * 16, t * 64:(t + 1) * 64].any():
                want_bits[g, t // 32] |= np.uint32(1) << np.uint32(t % 32)
    assert np.array_equal(got_bits, want_bits)
    if S > 1024:
        return
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    for m in (mask, np.zeros((S, S), np.float16), randn_h(r, (S, S))):
        md = dev(m)
        plain = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H, B, None, 1.0))
        summ = K.attention_mask_summary(md, S)
        K.attention_mask_summary_attach(md, S, summ)
        try:
            fast = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H, B, None, 1.0))
        finally:
            K.attention_mask_summary_attach(md, S, None)
        assert np.array_equal(plain, fast)
        # the summary handed over with the call (nothing attached to the mask's address): the same bits
        assert np.array_equal(host(K.OTF_attention_summary(dev(Q), dev(Kk), dev(V), md, summ, S, H, B, None, 1.0)), plain)
        assert np.array_equal(host(K.OTF_attention_summary(dev(Q), dev(Kk), dev(V), md, None, S, H, B, None, 1.0)), plain)
        want = orc.otf_attention(Q, Kk, V, m, S, H, B, None, 1.0, f64=True)
        check_close(fast, want, max_abs=5e-3, mean_rel=1e-3, what="attention with mask summary")


def test_mask_summary_object_does_not_outlive_its_mask(K):
    """the summary registry is keyed on the mask's address: a MaskSummary holds its mask while attached
    and detaches when it goes, so another mask that the allocator puts at the same address is not
    treated with the old summary"""
    r = rng(46)
    S, H, d = 256, 4, 256
    Q, Kk, V = (randn_h(r, (S, d)) for _ in range(3))
    zeros = torch.zeros((S, S), dtype=torch.float16, device="cuda")
    addr = zeros.data_ptr()
    ms = K.MaskSummary(zeros, S)           # all-zero: the launchers take the no-mask kernel for this address
    no_mask = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), zeros, S, H))
    del zeros                              # the object still holds the tensor: the address stays taken
    other = torch.empty((S, S), dtype=torch.float16, device="cuda")
    assert other.data_ptr() != addr
    del ms, other                          # detaches, then frees
    mask = randn_h(r, (S, S), 2.0)
    md = torch.empty((S, S), dtype=torch.float16, device="cuda")
    md.copy_(torch.from_numpy(mask))
    if md.data_ptr() != addr:
        pytest.skip("the allocator did not hand the address out again")
    got = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H))
    want = orc.otf_attention(Q, Kk, V, mask, S, H, 1, None, 1.0, f64=True)
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="attention with a mask at a reused address")
    assert not np.array_equal(got, no_mask)
    # in-place update of an attached mask: refresh() brings the summary up to date
    with K.MaskSummary(md, S) as ms2:
        md.zero_()
        md[5, 200] = -4.0
        ms2.refresh()
        got2 = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H))
    m2 = np.zeros((S, S), np.float16)
    m2[5, 200] = -4.0
    check_close(got2, orc.otf_attention(Q, Kk, V, m2, S, H, 1, None, 1.0, f64=True), max_abs=5e-3, mean_rel=1e-3,
                what="attention after an in-place mask update")


@pytest.mark.parametrize("S,H,d,B,lens", [(2048, 12, 768, 1, [1500]), (4160, 2, 128, 2, [4160, 4097])])
def test_otf_attention_long_sequences(K, S, H, d, B, lens):
    """key tiles are walked with running statistics: no limit on seq_len (4160 = 65 tiles is past the
    64 tiles whose mask summary a workgroup keeps in registers)"""
    r = rng(48 + S)
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.5)
    mask[:, S // 2:S // 2 + 300] = 0          # some all-zero mask tiles
    lens = np.array(lens, np.int32)
    md = dev(mask)
    want = orc.otf_attention(Q, Kk, V, mask, S, H, B, lens, 1.0, f64=True)
    got = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H, B, dev(lens), 1.0))
    summ = K.attention_mask_summary(md, S)
    K.attention_mask_summary_attach(md, S, summ)
    try:
        fast = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H, B, dev(lens), 1.0))
    finally:
        K.attention_mask_summary_attach(md, S, None)
    assert np.array_equal(got, fast)
    valid = np.concatenate([np.arange(S) < n for n in lens])
    check_close(got[valid], want[valid], max_abs=5e-3, mean_rel=1e-3, what="attention, long sequence")
    assert (got[~valid] == 0).all()


def test_otf_attention_varlen_equals_padded(K):
    r = rng(42)
    S, H, d, B = 256, 12, 768, 4
    lens = np.array([256, 31, 130, 64], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.5)
    padded = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), dev(mask), S, H, B, dev(lens), 1.0))
    sel = np.concatenate([np.arange(b * S, b * S + lens[b]) for b in range(B)])
    packed = host(K.OTF_attention_varlen(dev(Q[sel]), dev(Kk[sel]), dev(V[sel]), dev(mask), dev(cu), S, H, 1.0))
    assert np.array_equal(packed, padded[sel])        # same kernel, same arithmetic order
    want = orc.otf_attention(Q, Kk, V, mask, S, H, B, lens, 1.0, f64=True)
    check_close(packed, want[sel], max_abs=5e-3, mean_rel=1e-3, what="varlen attention")


@pytest.mark.parametrize("S,H,d,lens", [
    (256, 12, 768, [256, 31, 130, 64, 0, 200, 1]),                  # one sequence without rows
    (128, 2, 128, [128, 5, 0, 0, 77, 64, 65, 128, 3, 90]),          # fewer heads than XCDs: sequences without a
                                                                    # head on some XCD
    (96, 4, 256, list(range(96, 96 - 70, -1))),                     # more than 64 sequences (two count registers)
    (64, 2, 128, [64 - (i % 50) for i in range(300)]),              # more than the walked form takes: one
                                                                    # workgroup per possible block
])
def test_otf_attention_varlen_walks_existing_blocks(K, S, H, d, lens):
    """packed sequences: workgroups that walk the existing query blocks == one workgroup per possible block (the
    same block code, bit for bit) == the oracle on the padded batch"""
    from et_amd._lib import lib
    r = rng(50 + S + H)
    lens = np.array(lens, np.int32)
    B = lens.size
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    Q, Kk, V = (randn_h(r, (T, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.5)
    args = (dev(Q), dev(Kk), dev(V), dev(mask), dev(cu), S, H, 1.0)
    walked = host(K.OTF_attention_varlen(*args))
    try:
        lib().et_tuning_set(b"attn_packed", 0)
        grid = host(K.OTF_attention_varlen(*args))
    finally:
        lib().et_tuning_set(b"attn_packed", 1)
    assert np.array_equal(walked, grid)
    Qp, Kp, Vp = (np.zeros((B * S, d), np.float16) for _ in range(3))
    sel = np.concatenate([np.arange(b * S, b * S + lens[b]) for b in range(B)]).astype(np.int64)
    Qp[sel], Kp[sel], Vp[sel] = Q, Kk, V
    want = orc.otf_attention(Qp, Kp, Vp, mask, S, H, B, lens, 1.0, f64=True)
    check_close(walked, want[sel], max_abs=5e-3, mean_rel=1e-3, what="varlen attention, walked blocks")


@pytest.mark.parametrize("S,keep,value", [(512, 300, -30000.0), (512, 64, -65504.0), (256, 200, -1000.0), (192, 1, -30000.0)])
def test_otf_attention_padding_mask_with_dead_tiles(K, S, keep, value):
    """a padding mask that blanks the keys from `keep` on: key tiles that lie wholly behind it add nothing (every
    exp2 is exactly zero) and the kernel passes over them; == the oracle, with and without a mask summary, and the
    blanked keys' V rows have no influence at all"""
    r = rng(60 + S + keep)
    H, d, B = 12, 768, 2
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = np.zeros((S, S), np.float16)
    mask[:, keep:] = value
    want = orc.otf_attention(Q, Kk, V, mask, S, H, B, None, 1.0, f64=True)
    md = dev(mask)
    got = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H, B, None, 1.0))
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="attention, padding mask")
    summ = K.attention_mask_summary(md, S)
    K.attention_mask_summary_attach(md, S, summ)
    try:
        fast = host(K.OTF_attention(dev(Q), dev(Kk), dev(V), md, S, H, B, None, 1.0))
    finally:
        K.attention_mask_summary_attach(md, S, None)
    assert np.array_equal(got, fast)
    if value <= -30000.0:
        V2 = V.copy()
        V2.reshape(B, S, d)[:, keep:] = randn_h(r, (B, S - keep, d), 7.0)
        assert np.array_equal(host(K.OTF_attention(dev(Q), dev(Kk), dev(V2), md, S, H, B, None, 1.0)), got)


def test_prune_attention(K):
    r = rng(43)
    S, H, d, B = 160, 12, 768, 2
    hd = d // H
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.3)
    lens = np.array([160, 99], np.int32)
    qk_id = orc.gen_head_balanced_rows(H, hd, 32, seed=1)
    v_id = orc.gen_sparse_row_mat(d, 0.7, seed=3)                 # 230 kept columns, ragged over heads
    qk_hp, v_hp = orc.head_ptr(qk_id, H, hd), orc.head_ptr(v_id, H, hd)
    Qc, Kc, Vc = (np.ascontiguousarray(t) for t in (Q[:, qk_id], Kk[:, qk_id], V[:, v_id]))
    want = orc.prune_attention(Qc, Kc, Vc, qk_hp, v_id, v_hp, mask, S, d, H, B, lens, f64=True)
    got = host(K.Prune_attention(dev(Qc), dev(Kc), dev(Vc), dev(qk_hp), dev(v_id), dev(v_hp), dev(mask), S, d, H, B, dev(lens)))
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="pruned attention")
    other = np.setdiff1d(np.arange(d), v_id)
    assert (got[:, other] == 0).all()
    # the reference's wiring: dense Q/K, compact V (encoder/encoder.cu:76-79)
    want2 = orc.prune_attention(Q, Kk, Vc, None, v_id, v_hp, mask, S, d, H, B, lens, f64=True)
    got2 = host(K.Prune_attention(dev(Q), dev(Kk), dev(Vc), None, dev(v_id), dev(v_hp), dev(mask), S, d, H, B, dev(lens)))
    check_close(got2, want2, max_abs=5e-3, mean_rel=1e-3, what="pruned attention, dense QK")


@pytest.mark.parametrize("S,B,with_mask,with_lens", [(160, 2, True, True), (256, 3, False, False),
                                                     (128, 20, False, False), (77, 1, False, True),
                                                     (512, 11, False, False), (512, 11, True, True)])
def test_prune_attention_value_windows(K, S, B, with_mask, with_lens):
    """dense Q/K with compact V whose row pitch is a multiple of 8 (the reference's wiring, encoder/encoder.cu:76-79):
    V is staged by DMA as aligned 80-column windows.  Heads that start at any column mod 8, a head that keeps all
    64 columns behind an odd start (5 subtiles), a head that keeps none; == the oracle, and bit for bit == the
    register-staged kernel (same products in the same order)"""
    from et_amd._lib import lib
    r = rng(49 + S)
    H, d = 12, 768
    hd = d // H
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.3) if with_mask else None
    lens = r.integers(1, S + 1, size=B).astype(np.int32) if with_lens else None
    keep = [3, 64, 0, 17, 8, 1, 64, 33, 64, 5, 21, 64]       # columns kept per head
    v_id = np.concatenate([h * hd + np.sort(r.choice(hd, k, replace=False)) for h, k in enumerate(keep)]).astype(np.int32)
    v_hp = orc.head_ptr(v_id, H, hd)
    ld = (v_id.size + 7) // 8 * 8
    Vc = np.zeros((B * S, ld), np.float16)
    Vc[:, :v_id.size] = V[:, v_id]
    md, lensd = (None if mask is None else dev(mask)), (None if lens is None else dev(lens))
    want = orc.prune_attention(Q, Kk, np.ascontiguousarray(Vc[:, :v_id.size]), None, v_id, v_hp, mask, S, d, H, B, lens, f64=True)
    got = host(K.Prune_attention(dev(Q), dev(Kk), dev(Vc), None, dev(v_id), dev(v_hp), md, S, d, H, B, lensd))
    try:
        lib().et_tuning_set(b"attn_vwin", 0)
        regs = host(K.Prune_attention(dev(Q), dev(Kk), dev(Vc), None, dev(v_id), dev(v_hp), md, S, d, H, B, lensd))
    finally:
        lib().et_tuning_set(b"attn_vwin", 1)
    assert np.array_equal(got, regs)
    valid = np.ones(B * S, bool) if lens is None else np.concatenate([np.arange(S) < n for n in lens])
    check_close(got[valid], want[valid], max_abs=5e-3, mean_rel=1e-3, what="pruned attention, value windows")
    assert (got[~valid] == 0).all()
    assert (got[:, np.setdiff1d(np.arange(d), v_id)] == 0).all()


def test_prune_attention_value_windows_trailing_empty_heads(K):
    """the last heads keep no value columns and the row pitch equals the kept total (a multiple of 8): their
    windows start at the end of the row and must be pulled back inside it"""
    r = rng(4242)
    H, d, S, B = 12, 768, 128, 2
    hd = d // H
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    keep = [64, 40, 16, 0, 0, 0, 0, 0, 0, 0, 0, 0]           # 120 kept columns, nothing behind head 2
    v_id = np.concatenate([h * hd + np.sort(r.choice(hd, k, replace=False)) for h, k in enumerate(keep)]).astype(np.int32)
    v_hp = orc.head_ptr(v_id, H, hd)
    assert v_id.size % 8 == 0 and v_hp[-1] == v_hp[3] == v_id.size
    Vc = np.ascontiguousarray(V[:, v_id])
    want = orc.prune_attention(Q, Kk, Vc, None, v_id, v_hp, None, S, d, H, B, None, f64=True)
    got = host(K.Prune_attention(dev(Q), dev(Kk), dev(Vc), None, dev(v_id), dev(v_hp), None, S, d, H, B, None))
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="pruned attention, trailing empty heads")
    assert (got[:, np.setdiff1d(np.arange(d), v_id)] == 0).all()


@pytest.mark.parametrize("S,B,with_mask,with_lens", [(160, 2, True, True), (256, 3, False, False),
                                                     (512, 2, True, False), (77, 1, False, True)])
def test_otf_attention_narrow_qk_heads(K, S, B, with_mask, with_lens):
    """every head keeps 32 of its 64 Q/K columns: the on-the-fly kernel on compact Q/K
    == the pruned-attention oracle == et_Prune_attention with the matching head_ptr"""
    r = rng(47 + S)
    H, d = 12, 768
    hd = d // H
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    mask = randn_h(r, (S, S), 0.3) if with_mask else None
    lens = r.integers(1, S + 1, size=B).astype(np.int32) if with_lens else None
    qk_id = orc.gen_head_balanced_rows(H, hd, 32, seed=2)
    qk_hp = orc.head_ptr(qk_id, H, hd)
    assert np.array_equal(qk_hp, 32 * np.arange(H + 1))
    Qc, Kc = np.ascontiguousarray(Q[:, qk_id]), np.ascontiguousarray(Kk[:, qk_id])
    md, ld = (None if mask is None else dev(mask)), (None if lens is None else dev(lens))
    want = orc.prune_attention(Qc, Kc, V, qk_hp, None, None, mask, S, d, H, B, lens, f64=True)
    got = host(K.OTF_attention_qk_width(dev(Qc), dev(Kc), dev(V), md, 32, S, H, B, ld))
    other = host(K.Prune_attention(dev(Qc), dev(Kc), dev(V), dev(qk_hp), None, None, md, S, d, H, B, ld))
    valid = np.ones(B * S, bool) if lens is None else np.concatenate([np.arange(S) < n for n in lens])
    check_close(got[valid], want[valid], max_abs=5e-3, mean_rel=1e-3, what="narrow Q/K heads")
    check_close(got[valid], other[valid], max_abs=2e-3, mean_rel=1e-3, what="narrow Q/K heads vs pruned kernel")
    assert (got[~valid] == 0).all()
    # another width (16 of 64) runs on the register-staged kernel: == the oracle on the narrower column set
    qk16 = orc.gen_head_balanced_rows(H, hd, 16, seed=3)
    Q16, K16 = np.ascontiguousarray(Q[:, qk16]), np.ascontiguousarray(Kk[:, qk16])
    want16 = orc.prune_attention(Q16, K16, V, orc.head_ptr(qk16, H, hd), None, None, mask, S, d, H, B, lens, f64=True)
    got16 = host(K.OTF_attention_qk_width(dev(Q16), dev(K16), dev(V), md, 16, S, H, B, ld))
    check_close(got16[valid], want16[valid], max_abs=5e-3, mean_rel=1e-3, what="narrow Q/K heads, 16 of 64")
    with pytest.raises(Exception):   # not a multiple of 16
        K.OTF_attention_qk_width(dev(Qc[:, :96]), dev(Kc[:, :96]), dev(V), md, 8, S, H, B, ld)


def test_sharedqk_attention_and_scores(K):
    r = rng(44)
    S, H, d, B = 200, 12, 768, 2
    Q, Kk, V = (randn_h(r, (B * S, d), 0.7) for _ in range(3))
    mask = randn_h(r, (S, S), 0.3)
    QK = host(K.qk_scores(dev(Q), dev(Kk), S, H, B))
    want_qk = orc.qk_scores(Q, Kk, S, H, B, f64=True)
    check_close(QK, want_qk, max_abs=2e-2, mean_rel=5e-4, what="qk scores")
    want = orc.sharedqk_attention(QK, V, mask, S, H, B, f64=True)
    got = host(K.sharedQK_attention(dev(QK), dev(V), dev(mask), S, H, B))
    check_close(got, want, max_abs=5e-3, mean_rel=1e-3, what="sharedQK attention")


# -------------------------------------------------------------- data movement
def test_pack_unpack_scatter(K):
    r = rng(45)
    S, B, d = 64, 5, 768
    lens = np.array([64, 1, 17, 0, 40], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    x = randn_h(r, (B * S, d))
    sel = np.concatenate([np.arange(b * S, b * S + lens[b]) for b in range(B)]).astype(np.int64)
    packed = host(K.pack_rows(dev(x), dev(cu), S, int(cu[-1])))
    assert np.array_equal(packed, x[sel])
    back = host(K.unpack_rows(dev(packed), dev(cu), S))
    want = np.zeros_like(x)
    want[sel] = x[sel]
    assert np.array_equal(back, want)
    # longest first: packed sequence i is padded sequence order[i]
    order = np.argsort(-lens, kind="stable").astype(np.int32)
    cu_o = np.concatenate([[0], np.cumsum(lens[order])]).astype(np.int32)
    sel_o = np.concatenate([np.arange(b * S, b * S + lens[b]) for b in order]).astype(np.int64)
    packed_o = host(K.pack_rows(dev(x), dev(cu_o), S, int(cu_o[-1]), order=dev(order)))
    assert np.array_equal(packed_o, x[sel_o])
    back_o = host(K.unpack_rows(dev(packed_o), dev(cu_o), S, order=dev(order)))
    assert np.array_equal(back_o, want)
    ids = np.sort(r.choice(d, 230, replace=False)).astype(np.int32)
    comp = randn_h(r, (50, 240))
    sc = host(K.scatter_cols(dev(comp), dev(ids), d))
    want = np.zeros((50, d), np.float16)
    want[:, ids] = comp[:, :230]
    assert np.array_equal(sc, want)


@pytest.mark.parametrize("rows,d,n,ld", [(50, 768, 230, 240), (131, 768, 768, 768), (7, 256, 1, 16),
                                          (33, 1536, 921, 928), (20, 1000, 300, 304), (9, 772, 100, 100)])
def test_scatter_skip_layernorm_one_launch(K, rows, d, n, ld):
    """LayerNorm(expand(compact) + skip) == et_scatter_cols then et_skip_layernorm, bit for bit, and the oracle"""
    r = rng(46 + d + n)
    ids = np.sort(r.choice(d, n, replace=False)).astype(np.int32)
    comp, skip = randn_h(r, (rows, ld)), randn_h(r, (rows, d))
    g, b = randn_h(r, (d,), 0.3) + np.float16(1), randn_h(r, (d,), 0.3)
    expanded = np.zeros((rows, d), np.float16)
    expanded[:, ids] = comp[:, :n]
    got = host(K.scatter_skip_layernorm(dev(comp), dev(ids), dev(skip), dev(g), dev(b)))
    check_close(got, orc.skip_layernorm(expanded, skip, g, b, f64=True), what="scatter + skip + LayerNorm")
    two = K.scatter_cols(dev(comp), dev(ids), d)
    K.skip_layernorm(two, dev(skip), dev(g), dev(b))
    assert np.array_equal(got, host(two))
    if d % 8 == 0 and ld % 8 == 0:   # the one-launch form may overwrite the skip operand
        sk = dev(skip)
        K.scatter_skip_layernorm(dev(comp), dev(ids), sk, dev(g), dev(b), out=sk)
        assert np.array_equal(host(sk), got)


# ------------------------------------------------------- empty inputs, bad arguments
def test_launchers_with_no_rows_touch_nothing_and_bad_arguments_fail_cleanly(K):
    """row count 0 is a valid call that does nothing; null pointers, misaligned operands and unsupported
    sizes come back as error codes with a message (nothing is launched, nothing exits)"""
    import ctypes as C
    from et_amd import lib
    from et_amd._lib import EtError, check
    L = lib()
    d = 768
    sentinel = torch.full((64, d), 7.0, dtype=torch.float16, device="cuda")
    x = torch.zeros((64, d), dtype=torch.float16, device="cuda")
    g = torch.ones(d, dtype=torch.float16, device="cuda")
    ids = torch.arange(16, dtype=torch.int32, device="cuda")
    p = lambda t: t.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    # zero rows
    check(L.et_skip_layernorm(p(sentinel), p(x), p(g), p(g), 0, d, st))
    check(L.et_scatter_skip_layernorm(p(sentinel), p(x), p(ids), 16, 16, p(x), p(g), p(g), 0, d, st))
    check(L.et_row_spmm_add_bias(p(sentinel), p(x), p(x), p(g), 0, 16, d, st))
    outs, ws, bs = (C.c_void_p * 1)(p(sentinel)), (C.c_void_p * 1)(p(x)), (C.c_void_p * 1)(p(g))
    check(L.et_row_spmm_add_bias_multi(outs, p(x), ws, bs, (C.c_int * 1)(16), 1, 0, d, st))
    lin = make_tile_linear(rng(1), d, d, 0.8, seed=2)
    from et_amd.encoder import Linear_tile
    lt = Linear_tile(d, d, 64, lin["row_offset"].size, lin["data"], lin["row_ptr"], lin["row_offset"], lin["bias"])
    lt.run(x, out=sentinel, rows=0)
    torch.cuda.synchronize()
    assert (sentinel == 7).all()
    # bad arguments
    for call in (
        lambda: check(L.et_skip_layernorm(None, p(x), p(g), p(g), 4, d, st)),
        lambda: check(L.et_skip_layernorm(p(sentinel), p(x), p(g), p(g), -1, d, st)),
        lambda: check(L.et_scatter_skip_layernorm(p(sentinel), p(sentinel), p(ids), 16, 16, p(x), p(g), p(g), 4, d, st)),
        lambda: check(L.et_scatter_skip_layernorm(p(sentinel), p(x), p(ids), 32, 16, p(x), p(g), p(g), 4, d, st)),
        lambda: check(L.et_row_spmm_add_bias(p(sentinel), p(x), p(x), p(g), 4, 24, d, st)),          # N not a multiple of 16
        lambda: check(L.et_row_spmm_add_bias(p(sentinel) + 2, p(x), p(x), p(g), 4, 16, d, st)),      # misaligned
        lambda: check(L.et_OTF_attention(p(sentinel), p(x), p(x), p(x), None, 64, 770, 12, 1, None, 1.0, st)),   # d_model % nhead
        lambda: check(L.et_OTF_attention(p(sentinel), p(x), p(x), p(x), None, 64, 768, 32, 1, None, 1.0, st)),   # head_dim 24: not a multiple of 16
        lambda: check(L.et_OTF_attention_qk_width(p(sentinel), p(x), p(x), p(x), None, 0, 64, 768, 12, 1, None, 1.0, st)),
        lambda: check(L.et_pack_rows_ordered(p(sentinel), None, p(ids), p(ids), 2, 8, d, st)),
    ):
        with pytest.raises(EtError):
            call()
    torch.cuda.synchronize()
    assert (sentinel == 7).all()
    assert L.et_last_error().decode() != ""



# ------------------------------------------------------------ machine rates
def test_microbenchmarks_report_plausible_rates():
    """et_microbench runs its three kernels and returns rates of the right order (not a performance assertion:
    the bounds are a factor of several around what an MI355X measures)"""
    import ctypes as C
    from et_amd._lib import lib, check
    from et_amd.build import MICROBENCH_LIB
    lib()
    mbl = C.CDLL(MICROBENCH_LIB)     # a library of its own: the microbenchmarks are not part of the encoder's C ABI
    mbl.et_microbench.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    sec, units = C.c_double(), C.c_double()
    def rate(what, p0, p1):
        check(mbl.et_microbench(what, p0, p1, C.byref(sec), C.byref(units)))
        assert sec.value > 0 and units.value > 0
        return units.value / sec.value
    mfma_per_s = rate(2, 0, 4)                  # MFMAs per second and wave: 16 clk each
    clock = mfma_per_s * 16
    assert 0.8e9 < clock < 3.0e9
    lds = rate(0, 1568, 16) / clock             # bytes per clock and CU
    assert 100 < lds < 300
    assert rate(0, 1536, 16) / clock < 0.5 * lds    # a row stride of a multiple of 256 bytes conflicts
    stream = rate(1, 0, 16) / clock
    assert 20 < stream < 140
    with pytest.raises(Exception):
        check(mbl.et_microbench(7, 0, 0, C.byref(sec), C.byref(units)))
    with pytest.raises(Exception):               # a stride the 16-byte reads cannot take: refused before anything is allocated
        check(mbl.et_microbench(0, 1570, 16, C.byref(sec), C.byref(units)))
