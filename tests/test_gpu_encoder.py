"""Encoder layers (the reference's Encoder_* objects) against the CPU oracle."""
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


def make_layer(r, d, dff, sp, seed, std=0.02, bias_std=0.02):
    shapes = [(d, d)] * 4 + [(dff, d), (d, dff)]
    lins = [make_tile_linear(r, n, k, sp, seed=seed + j, std=std, bias_std=bias_std) for j, (n, k) in enumerate(shapes)]
    ln = [randn_h(r, (d,), 0.1) + np.float16(1), randn_h(r, (d,), 0.1), randn_h(r, (d,), 0.1) + np.float16(1), randn_h(r, (d,), 0.1)]
    return lins, ln


def build_linears(lins, rows):
    from et_amd.encoder import Linear_tile
    return [Linear_tile(l["K"], l["N"], rows, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
            for j, l in enumerate(lins)]


def workspace(cls, d, S, H, B):
    return torch.empty(cls.buffer_size(d, S, H, B) // 2, dtype=torch.float16, device="cuda")


@pytest.mark.parametrize("S,B,sp,ls,use_mask", [
    (128, 1, 0.0, 1.0, True),       # config 1: dense single sequence
    (128, 2, 0.8, LOG2E, False),
    (512, 2, 0.8, 1.0, True),       # config 3 shape, batch cut to 2
])
def test_encoder_tile_layer(S, B, sp, ls, use_mask):
    from et_amd.encoder import Encoder_tile
    r = rng(500 + S + B)
    d, H, dff = 768, 12, 3072
    lins, ln = make_layer(r, d, dff, sp, seed=900)
    x = randn_h(r, (B * S, d))
    mask = randn_h(r, (S, S), 0.5) if use_mask else None
    want = orc.encoder_tile_layer(x, lins, ln, mask, S, H, B, None, ls)
    enc = Encoder_tile(d, S, H, workspace(Encoder_tile, d, S, H, B), *build_linears(lins, B * S), *ln, mask, B)
    enc.set_log2_scale(ls)
    xd = dev(x)
    out = torch.empty_like(xd)
    got = host(enc.run(out, xd))
    check_close(got, want, what="Encoder_tile")
    # out may alias in (test/tile_test.cu:41 calls run(in, in))
    got2 = host(enc.run(xd, xd))
    assert np.array_equal(got2, got)


def test_encoder_prune_layer():
    from et_amd.encoder import Encoder_prune, Linear_row
    r = rng(600)
    d, H, dff, S, B = 768, 12, 3072, 128, 2
    lins, ln = make_layer(r, d, dff, 0.8, seed=910)
    x = randn_h(r, (B * S, d))
    mask = randn_h(r, (S, S), 0.5)
    v_id = orc.gen_sparse_row_mat(d, 0.7, seed=5)              # 230 surviving V rows
    Wv, bv = randn_h(r, (v_id.size, d), 0.02), randn_h(r, (v_id.size,), 0.02)
    # oracle: step by step (encoder/encoder.cu:65-92)
    tl = lambda j, inp, g=False: orc.tile_linear(inp, lins[j]["row_ptr"], lins[j]["row_offset"], lins[j]["data"], lins[j]["bias"], lins[j]["N"], gelu=g)
    q, k = tl(0, x), tl(1, x)
    vc = orc.row_linear(x, Wv, bv)
    z = orc.prune_attention(q, k, vc, None, v_id, orc.head_ptr(v_id, H, d // H), mask, S, d, H, B)
    h1 = orc.skip_layernorm(tl(3, z), x, ln[0], ln[1])
    want = orc.skip_layernorm(tl(5, tl(4, h1, True)), h1, ln[2], ln[3])
    L = build_linears(lins, B * S)
    L[2] = Linear_row(d, d, B * S, Wv, v_id, v_id.size, bv, H)
    assert L[2].nrow == 240 and L[2].row_id_size == 230
    enc = Encoder_prune(d, S, H, workspace(Encoder_prune, d, S, H, B), *L, *ln, mask, B)
    xd = dev(x)
    got = host(enc.run(torch.empty_like(xd), xd))
    check_close(got, want, what="Encoder_prune")


def test_encoder_length_paths():
    from et_amd.encoder import Encoder_length
    r = rng(700)
    d, H, dff, S, B = 768, 12, 3072, 256, 3
    lins, ln = make_layer(r, d, dff, 0.8, seed=920)
    x = randn_h(r, (B * S, d))
    mask = randn_h(r, (S, S), 0.5)
    enc = Encoder_length(d, S, H, workspace(Encoder_length, d, S, H, B), *build_linears(lins, B * S), *ln, mask, B)
    xd = dev(x)
    want = orc.encoder_tile_layer(x, lins, ln, mask, S, H, B, None, 1.0)
    got = host(enc.run(torch.empty_like(xd), xd))
    check_close(got, want, what="Encoder_length, on-the-fly")
    enc.set_shared_qk(True)       # the reference's own route: scores through memory (encoder/encoder.cu:126-137)
    got_s = host(enc.run(torch.empty_like(xd), xd))
    check_close(got_s, want, what="Encoder_length, shared QK")
    enc.set_shared_qk(False)
    lens = np.array([256, 40, 131], np.int32)
    enc.set_seq_lens(lens)
    want_l = orc.encoder_tile_layer(x, lins, ln, mask, S, H, B, lens, 1.0)
    got_l = host(enc.run(torch.empty_like(xd), xd))
    for b in range(B):   # valid positions equal the padded run; padding rows are zero
        sl = slice(b * S, b * S + lens[b])
        check_close(got_l[sl], want_l[sl], what=f"Encoder_length packed, seq {b}")
        assert (got_l[b * S + lens[b]:(b + 1) * S] == 0).all()
    got_alias = host(enc.run(xd, xd))
    assert np.array_equal(got_alias, got_l)


def test_encoder_stack_variable_length():
    from et_amd.encoder import Encoder_length, Encoder_stack
    r = rng(800)
    d, H, dff, S, B, NL = 256, 4, 1024, 128, 4, 3
    layers, params = [], []
    for i in range(NL):
        lins, ln = make_layer(r, d, dff, 0.5, seed=930 + 10 * i, std=0.05)
        params.append((lins, ln))
        layers.append(Encoder_length(d, S, H, workspace(Encoder_length, d, S, H, B), *build_linears(lins, B * S), *ln, None, B))
    x = randn_h(r, (B * S, d))
    lens = np.array([128, 9, 77, 50], np.int32)
    stack = Encoder_stack(layers, d, S, B)
    stack.set_seq_lens(lens)
    xd = dev(x)
    got = host(stack.run(torch.empty_like(xd), xd))
    cur = x
    for lins, ln in params:
        cur = orc.encoder_tile_layer(cur, lins, ln, None, S, H, B, lens, 1.0)
    for b in range(B):
        sl = slice(b * S, b * S + lens[b])
        check_close(got[sl], cur[sl], what=f"stack seq {b}")
        assert (got[b * S + lens[b]:(b + 1) * S] == 0).all()
    stack.set_seq_lens(None)    # full-length batch through the same stack
    got_full = host(stack.run(torch.empty_like(xd), xd))
    cur = x
    for lins, ln in params:
        cur = orc.encoder_tile_layer(cur, lins, ln, None, S, H, B, None, 1.0)
    check_close(got_full, cur, what="stack full length")
