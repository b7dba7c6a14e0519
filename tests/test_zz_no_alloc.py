"""The entry point that allocates nothing: et_OTF_attention_noalloc keeps its mask summary in a static
device array of the library.  Its output must equal et_OTF_attention's bit for bit (skipping an
all-zero mask tile changes no bit: s + 0 == s) on two calls in a row, the second one smaller, so that
whatever the first call left in the shared array is seen not to leak into the second."""
import numpy as np
import pytest
import torch

import oracle.et_oracle as orc
from helpers import rng, randn_h, check_close

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def _case(r, S, H, d, B, lens, kind):
    Q, Kk, V = (randn_h(r, (B * S, d)) for _ in range(3))
    if kind == "padding":      # all-zero tiles in front, large negative values on the last third of the keys
        mask = np.zeros((S, S), np.float16)
        mask[:, S - S // 3:] = -30000.0
        mask[min(37, S - 1), 5] = 0.25
    elif kind == "dense":
        mask = randn_h(r, (S, S), 0.5)
    else:                      # banded: non-zero tiles the first case left zero, and the other way round
        mask = np.zeros((S, S), np.float16)
        mask[: S // 2, : S // 4] = -3.0
    return Q, Kk, V, mask, None if lens is None else np.array(lens, np.int32)


def test_no_alloc_attention_two_calls_in_a_row():
    from et_amd import kernels as K
    r = rng(77)
    # the second call is smaller (shorter sequences, fewer row groups and key tiles than the first)
    calls = [(640, 4, 256, 2, [640, 411], "padding"), (200, 4, 256, 1, None, "banded"),
             (128, 12, 768, 2, [128, 5], "dense")]
    for n, (S, H, d, B, lens, kind) in enumerate(calls):
        Q, Kk, V, mask, lens_np = _case(r, S, H, d, B, lens, kind)
        args = (dev(Q), dev(Kk), dev(V), dev(mask), S, H, B, None if lens_np is None else dev(lens_np), 1.0)
        want_dev = K.OTF_attention(*args)
        out = torch.full_like(want_dev, float("nan"))
        free_before = torch.cuda.mem_get_info()[0]
        got_dev = K.OTF_attention_noalloc(*args, out=out)
        torch.cuda.synchronize()
        if n > 0:       # (the first call may still load kernels)
            assert torch.cuda.mem_get_info()[0] == free_before  # no device allocation behind the call
        got, want = host(got_dev), host(want_dev)
        assert np.array_equal(got, want), f"S={S} {kind}: differs from et_OTF_attention"
        ref = orc.otf_attention(Q, Kk, V, mask, S, H, B, lens_np, 1.0, f64=True)
        valid = np.ones(B * S, bool) if lens_np is None else np.concatenate([np.arange(S) < n for n in lens_np])
        check_close(got[valid], ref[valid], max_abs=5e-3, mean_rel=1e-3, what=f"no-alloc attention S={S} {kind}")


def test_no_alloc_attention_limits():
    from et_amd import kernels as K
    from et_amd._lib import EtError
    r = rng(78)
    S, H, d = 4112, 1, 64
    Q, Kk, V = (dev(randn_h(r, (S, d))) for _ in range(3))
    out = torch.empty_like(Q)
    with pytest.raises(EtError) as e:      # beyond what the static array covers: refused, nothing launched
        K.OTF_attention_noalloc(Q, Kk, V, torch.zeros((S, S), dtype=torch.float16, device="cuda"), S, H, out=out)
    assert e.value.code == -3 and "4096" in str(e.value)
    want = host(K.OTF_attention(Q, Kk, V, None, S, H))
    got = host(K.OTF_attention_noalloc(Q, Kk, V, None, S, H, out=out))   # without a mask no scratch is needed
    assert np.array_equal(got, want)
