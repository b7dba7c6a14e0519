"""CPU-only checks of the shipped library: the C ABI loads and exports every
symbol the headers declare, the host-side format code is bit-identical to the
oracle's independent restatement, and argument validation fails cleanly
(negative codes, no exit) before anything touches a device."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle.et_oracle as orc
from et_amd import _lib, formats
from helpers import rng

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for hdr in ("et_amd.h", "et_encoder.h"):
        text = open(os.path.join(ROOT, "include", hdr)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(et_[A-Za-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(_lib.LIB_PATH)
    syms = declared_symbols()
    assert len(syms) >= 50
    missing = [s for s in syms if not hasattr(lib, s)]
    assert not missing, missing
    # and the Python binding covers the same set
    assert set(_lib.PROTOTYPES) == set(syms)
    assert _lib.lib().et_abi_version() == 2


@pytest.mark.parametrize("N,K,sp", [(768, 768, 0.8), (3072, 768, 0.5), (768, 3072, 0.9), (64, 96, 0.33), (16, 16, 0.0), (32, 32, 1.0)])
def test_tile_mat_generator_bit_exact_vs_oracle(N, K, sp):
    for seed in (0, 1, 12345678901234567):
        a = formats.gen_sparse_tile_mat(N, K, sp, seed)
        b = orc.gen_sparse_tile_mat(N, K, sp, seed)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        assert formats.tile_mat_validate(N, K, a[0], a[1]) == 0


def test_row_mat_and_head_ptr_bit_exact_vs_oracle():
    for nrow, sp in ((768, 0.7), (3072, 0.5), (768, 0.0), (100, 0.99)):
        assert np.array_equal(formats.gen_sparse_row_mat(nrow, sp, 9), orc.gen_sparse_row_mat(nrow, sp, 9))
    ids = formats.gen_sparse_row_mat(768, 0.7, 3)
    assert np.array_equal(formats.head_ptr(ids, 12, 64), orc.head_ptr(ids, 12, 64))
    assert np.array_equal(formats.gen_head_balanced_rows(12, 64, 32, 5), orc.gen_head_balanced_rows(12, 64, 32, 5))


def test_tile_pack_byte_identical_vs_oracle():
    r = np.random.default_rng(4)
    W = r.standard_normal((96, 160)).astype(np.float16)
    rp, ro = formats.gen_sparse_tile_mat(96, 160, 0.6, 8)
    assert np.array_equal(formats.tile_pack(W, rp, ro).view(np.uint16), orc.tile_pack(W, rp, ro).view(np.uint16))


def test_validate_codes_match_oracle():
    rp, ro = formats.gen_sparse_tile_mat(64, 64, 0.5, 1)
    cases = []
    bad = ro.copy(); bad[0] += 8; cases.append((64, 64, rp, bad))
    bad = ro.copy(); bad[0] = 64; cases.append((64, 64, rp, bad))
    bad = rp.copy(); bad[-1] += 1; cases.append((64, 64, bad, ro))
    bad = rp.copy(); bad[0] = 1; cases.append((64, 64, bad, ro))
    cases.append((60, 64, rp, ro))
    for N, K, p, o in cases:
        got, want = formats.tile_mat_validate(N, K, p, o), orc.tile_mat_validate(N, K, p, o)
        assert got == want and got < 0


def test_argument_errors_return_codes_without_a_device():
    l = _lib.lib()
    # null pointers / bad sizes are rejected before any HIP call
    assert l.et_skip_layernorm(None, None, None, None, 4, 768, None) == -1
    assert l.et_tile_spmm_add_bias(None, None, None, None, None, 16, 16, 16, None, None) == -1
    assert l.et_OTF_attention(None, None, None, None, None, 128, 768, 12, 1, None, 1.0, None) == -1
    assert l.et_row_spmm_add_bias(None, None, None, None, 16, 16, 16, None) == -1
    buf = (C.c_uint16 * 64)()
    p = C.addressof(buf)
    assert l.et_tile_spmm_add_bias(p, p, p, p, p, 16, 24, 16, p, None) == -3          # N not a multiple of 16
    assert l.et_OTF_attention(p, p, p, p, None, 128, 768, 7, 1, None, 1.0, None) == -1  # d_model % nhead
    assert l.et_OTF_attention(p, p, p, p, None, 128, 80, 2, 1, None, 1.0, None) == -3   # head_dim 40: not a multiple of 16
    assert b"head_dim" in l.et_last_error()
    assert l.et_strerror(-3) == b"unsupported shape"
    with pytest.raises(_lib.EtError):
        formats.gen_sparse_tile_mat(100, 64, 0.5, 1)     # nrow not a multiple of 16
    with pytest.raises(_lib.EtError):
        formats.gen_sparse_row_mat(64, 1.5, 1)
    # malformed tile_mat is refused at plan construction (ET_ERR_FORMAT), no device needed
    rp, ro = formats.gen_sparse_tile_mat(32, 32, 0.0, 1)
    bad = ro.copy(); bad[0] = 5
    data = np.zeros(ro.size * 256, np.float16); bias = np.zeros(32, np.float16)
    h = C.c_void_p()
    rc = l.et_tile_plan_create(C.byref(h), 32, 32, int(ro.size), data.ctypes.data, rp.ctypes.data, bad.ctypes.data, bias.ctypes.data)
    assert rc == -5 and not h.value


def test_magnitude_pruner_matches_the_oracle_bit_for_bit():
    from et_amd import formats
    r = rng(81)
    for N, K, sp in [(96, 128, 0.5), (768, 768, 0.8), (64, 64, 0.0), (64, 64, 1.0), (3072, 768, 0.9)]:
        W = (r.standard_normal((N, K)) * 0.05).astype(np.float16)
        W[::7] *= np.float16(3)
        rp, ro = formats.prune_tile_mat(W, sp)
        rp2, ro2 = orc.prune_tile_mat(W, sp)
        assert np.array_equal(rp, rp2) and np.array_equal(ro, ro2)
        assert np.array_equal(formats.prune_row_mat(W, sp), orc.prune_row_mat(W, sp))
    W = np.ones((64, 64), np.float16)
    W[5, 5] = np.float16(np.nan)
    W[40, 40] = np.float16(np.inf)
    for a, b in zip(formats.prune_tile_mat(W, 0.75), orc.prune_tile_mat(W, 0.75)):
        assert np.array_equal(a, b)
    assert np.array_equal(formats.prune_row_mat(W, 0.9), orc.prune_row_mat(W, 0.9))


def test_pruned_weight_containers_round_trip_and_reject_damage(tmp_path):
    from et_amd import formats
    from et_amd._lib import EtError
    r = rng(82)
    N, K = 96, 64
    W = (r.standard_normal((N, K)) * 0.1).astype(np.float16)
    bias = (r.standard_normal(N) * 0.1).astype(np.float16)
    rp, ro = formats.prune_tile_mat(W, 0.6)
    data = formats.tile_pack(W, rp, ro)
    p = tmp_path / "w.ettile"
    formats.tile_mat_save(p, K, N, rp, ro, data, bias)
    back = formats.tile_mat_load(p)
    assert (back["in_feat"], back["out_feat"]) == (K, N)
    for k, v in (("row_ptr", rp), ("row_offset", ro), ("data", data), ("bias", bias)):
        assert np.array_equal(back[k].view(np.uint8), np.ascontiguousarray(v).view(np.uint8)), k
    ids = formats.prune_row_mat(W, 0.7)
    q = tmp_path / "w.etrow"
    formats.row_mat_save(q, K, N, ids, W[ids], bias)
    back = formats.row_mat_load(q)
    assert np.array_equal(back["row_id"], ids) and np.array_equal(back["weight"], W[ids]) and np.array_equal(back["bias"], bias)
    # damage: one flipped payload byte, truncation, trailing bytes, the other kind's file, no file
    raw = p.read_bytes()
    for bad in (raw[:100] + bytes([raw[100] ^ 1]) + raw[101:], raw[:-3], raw + b"x", q.read_bytes()):
        (tmp_path / "bad").write_bytes(bad)
        with pytest.raises(EtError) as e:
            formats.tile_mat_load(tmp_path / "bad")
        assert e.value.code == -5
    with pytest.raises(EtError) as e:
        formats.tile_mat_load(tmp_path / "missing")
    assert e.value.code == -6
    # arrays sized for another file (or a file that changed after the peek): refused before anything is written
    from et_amd._lib import lib
    guard = np.full(8, 7, np.int32)
    rc = lib().et_tile_mat_load(str(p).encode(), K, N - 16, 3, guard.ctypes.data, guard.ctypes.data, guard.ctypes.data,
                                guard.ctypes.data)
    assert rc == -5 and (guard == 7).all()
    rc = lib().et_row_mat_load(str(q).encode(), K, N, ids.size - 1, guard.ctypes.data, guard.ctypes.data, guard.ctypes.data)
    assert rc == -5 and (guard == 7).all()
    with pytest.raises(EtError):                                      # unsorted row ids are refused on save
        formats.row_mat_save(tmp_path / "x", K, N, ids[::-1], W[ids], bias)


def test_class_headers_compile_with_a_plain_host_compiler(tmp_path):
    """et_amd/encoder/*.h (the reference's class surface) need no HIP headers: g++ takes them as is"""
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++ here")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    tu = tmp_path / "tu.cpp"
    tu.write_text('#include "et_amd/encoder/encoder.h"\n'
                  'size_t f() { return Encoder_tile::buffer_size(768, 128, 12, 2) + Encoder_length::buffer_size(768, 128, 12); }\n')
    res = subprocess.run([gxx, "-std=c++17", "-Wall", "-fsyntax-only", "-I", root, str(tu)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr



def test_python_binding_refuses_operands_of_the_wrong_shape():
    """the C ABI takes bare pointers; the Python classes check every operand's shape before a launch, so a
    swapped (x, out) pair or a short buffer is an error here and not a kernel writing past a buffer"""
    import torch
    from et_amd import encoder
    ok = torch.empty((8, 16), dtype=torch.float16)
    for rows, cols in ((8, 32), (9, 16)):                # wrong width, too few rows
        with pytest.raises(ValueError):
            encoder._dp2(ok, rows, cols, "operand")
    with pytest.raises(ValueError):
        encoder._dp2(ok.reshape(-1), 8, 16, "operand")   # not two-dimensional


def test_kernel_wrappers_refuse_operands_of_the_wrong_extent():
    """the same for the per-kernel wrappers: an extent that the other arguments imply is checked before
    anything is launched (here on host tensors, which the check meets before it would ask for a device)"""
    import torch
    from et_amd import kernels
    h = lambda *shape: torch.zeros(shape, dtype=torch.float16)
    with pytest.raises(ValueError):     # out narrower than N
        kernels.row_spmm_add_bias(h(8, 32), h(16, 32), h(16), out=h(8, 8))
    with pytest.raises(ValueError):     # skip with fewer rows
        kernels.skip_layernorm(h(8, 64), h(4, 64), h(64), h(64))
    with pytest.raises(ValueError):     # K of another sequence length
        kernels.OTF_attention(h(32, 64), h(16, 64), h(32, 64), None, 32, 1)
    with pytest.raises(ValueError):     # mask of another sequence length
        kernels.OTF_attention(h(32, 64), h(32, 64), h(32, 64), h(16, 16), 32, 1)


def test_more_wrappers_refuse_operands_of_the_wrong_extent():
    """run_multi, the packed-row copies, the multi row linear and the raw tile launcher on host tensors: the
    ValueError comes before any device pointer is asked for"""
    import torch
    from et_amd import encoder, kernels
    h = lambda *shape: torch.zeros(shape, dtype=torch.float16)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)

    class Stub:                         # stands in for a Linear_tile / Linear_row handle: never reached
        _h = None
        in_feat, out_feat, size, nrow = 32, 48, 8, 48

    with pytest.raises(ValueError):     # x of another width than in_feat
        encoder.run_multi([Stub(), Stub()], h(8, 64), [h(8, 48), h(8, 48)])
    with pytest.raises(ValueError):     # second output too narrow
        encoder.run_multi([Stub(), Stub()], h(8, 32), [h(8, 48), h(8, 16)])
    with pytest.raises(ValueError):     # fewer output rows than x has
        encoder.run_multi([Stub()], h(8, 32), [h(4, 48)])
    # the swap that once wrote 48-wide rows into a 32-wide tensor: Linear_row.run(x, out) with the two exchanged
    lr = encoder.Linear_row.__new__(encoder.Linear_row)
    lr.__dict__.update(_h=None, in_feat=32, out_feat=64, size=8, nrow=48)
    with pytest.raises(ValueError):
        encoder.Linear_row.run(lr, h(8, 48), out=h(8, 32))
    with pytest.raises(ValueError):     # gamma of the wrong length
        encoder._dpn(h(16), 48, "gamma")
    with pytest.raises(ValueError):     # cu_seqlens ends beyond the packed rows
        kernels.pack_rows(h(2 * 16, 8), i32([0, 10, 30]), 16, 26)
    with pytest.raises(ValueError):     # a sequence longer than seq_len
        kernels.pack_rows(h(2 * 16, 8), i32([0, 20, 26]), 16, 26)
    with pytest.raises(ValueError):     # order of the wrong length
        kernels.pack_rows(h(2 * 16, 8), i32([0, 10, 26]), 16, 26, order=i32([0, 1, 2]))
    with pytest.raises(ValueError):     # packed tensor shorter than cu_seqlens says
        kernels.unpack_rows(h(20, 8), i32([0, 10, 26]), 16)
    with pytest.raises(ValueError):     # bias shorter than the weight's rows
        kernels.row_spmm_add_bias_multi(h(8, 32), [h(16, 32), h(16, 32)], [h(16), h(8)])
    with pytest.raises(ValueError):     # weight with another K
        kernels.row_spmm_add_bias_multi(h(8, 32), [h(16, 64)], [h(16)])
    with pytest.raises(ValueError):     # row_ptr must hold N/16 + 1 entries
        kernels.tile_spmm_add_bias(h(8, 32), i32([0, 1]), i32([0]), h(256), h(32), 32)


def test_seq_lens_outside_the_sequence_are_refused():
    """a length above seq_len or below 0 would push the packed row offsets past the workspace: the Python
    class refuses it before the call (the C++ class's own check needs an encoder object, hence a device:
    tests/test_gpu_encoder.py covers its error code)"""
    import numpy as np
    from et_amd import encoder
    enc = encoder.Encoder_length.__new__(encoder.Encoder_length)
    enc.__dict__.update(_h=None, batch=3, seq_len=64)
    for bad in ([64, 65, 1], [3, -1, 2], [1, 2]):
        with pytest.raises(ValueError):
            encoder._Encoder.set_seq_lens(enc, np.array(bad))


def vwin_window_model(v_head_ptr, ldv, hd=64, rows=64):
    """Host restatement of the value-window staging addresses of attention.hip (window start, per-piece column
    clamp): yields (head, row, first column) of every 16-byte piece a tile fetches."""
    rowb = (hd + 16) * 2           # LDS bytes per staged window row: 80 columns, all of them data
    for h in range(len(v_head_ptr) - 1):
        vc0 = min(int(v_head_ptr[h]) & ~7, ldv - 8)
        for p in range(0, rows * rowb, 16):
            row, cb = divmod(p, rowb)
            yield h, row, vc0 + min(cb >> 1, ldv - 8 - vc0)


@pytest.mark.parametrize("keep", [[3, 64, 0, 17, 8, 1, 64, 33, 64, 5, 21, 64], [64, 40, 16, 0, 0, 0, 0, 0, 0, 0, 0, 0],
                                  [8] + [0] * 11, [0] * 11 + [8]])
def test_value_window_pieces_stay_inside_their_row(keep):
    """every staged piece of a value window lies inside its own row of compact V, also for heads that keep no
    columns and sit at the very end of the row (v_head_ptr[h] == ldv)"""
    hp = np.concatenate([[0], np.cumsum(keep)])
    ldv = (int(hp[-1]) + 7) // 8 * 8
    for h, row, col in vwin_window_model(hp, ldv):
        assert 0 <= col and col + 8 <= ldv, (h, row, col, ldv)


def test_wait_status_word_is_reported_once_and_cleared():
    """the status word that a fused kernel's bounded wait sets: raised from the host here (no device needed),
    the next check returns ET_ERR_HIP with a message, the one after that is clean again"""
    l = _lib.lib()
    assert l.et_wait_status_take() == 0
    l.et_wait_status_raise_for_test()
    rc = l.et_wait_status_take()
    assert rc < 0 and l.et_strerror(rc) == b"HIP runtime error"
    assert b"gave up a bounded wait" in l.et_last_error()
    assert l.et_wait_status_take() == 0


def test_encoder_workspace_grows_only_while_the_paired_tail_is_switched_on():
    """Encoder_*::buffer_size is the reference's five units (encoder/encoder.h:51-53; Encoder_length adds its
    scores) unless the paired layer tail is switched on, whose fp32 exchange area then follows them"""
    from et_amd.encoder import Encoder_length, Encoder_tile
    lib = _lib.lib()
    d, S, H, B = 768, 512, 12, 16
    units = 5 * B * S * d * 2
    assert lib.et_tail_ws_bytes_for(d, B * S) == 0
    assert Encoder_tile.buffer_size(d, S, H, B) == (units + 255) // 256 * 256
    base_len = Encoder_length.buffer_size(d, S, H, B)
    assert base_len >= units + B * H * S * S * 2
    try:
        for mode in (1, 2, 3):
            assert lib.et_tuning_set(b"tile_tail_pair", mode) == 0
            extra = lib.et_tail_ws_bytes_for(d, B * S)
            assert extra == (B * S) * 768 * 8                      # rows (a multiple of 64) x width x two floats
            assert Encoder_tile.buffer_size(d, S, H, B) == (units + 255) // 256 * 256 + extra
            assert Encoder_length.buffer_size(d, S, H, B) == base_len + extra
        assert lib.et_tail_ws_bytes_for(100, 64) == 0              # a width the paired kernel is not built for
    finally:
        lib.et_tuning_set(b"tile_tail_pair", 0)
    assert Encoder_tile.buffer_size(d, S, H, B) == (units + 255) // 256 * 256

