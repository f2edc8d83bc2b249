"""wol_quantize_static, the entry point that allocates nothing: its scratch is
a static device array inside the library.  Checked bit for bit against
wol_quantize (caller's workspace) on two calls in a row, the second smaller
than the first, so that what the first call left in the shared array would
show."""
import numpy as np
import pytest
import torch

import helpers as H
from paddle_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(w_bits, dt, bits, g):
    w = H.bits_to_torch(w_bits, dt, DEV)
    K, N = w.shape
    sshape = (N,) if g == -1 else ((K + g - 1) // g, N)
    res = []
    for static in (False, True):
        codes = torch.full((K * N * bits // 8,), 0x55, dtype=torch.uint8, device=DEV)
        scale = torch.zeros(sshape, dtype=w.dtype, device=DEV)
        if static:
            _lib.check(_lib.lib.wol_quantize_static(w.data_ptr(), dt, K, N, bits, g, _lib.ROUND_RNE,
                                                    _lib.LAYOUT_GFX950, codes.data_ptr(), scale.data_ptr(), None))
        else:
            wsb = _lib.lib.wol_quantize_workspace(K, N, bits, g)
            ws = torch.zeros(max(wsb, 16), dtype=torch.uint8, device=DEV)
            _lib.check(_lib.lib.wol_quantize(w.data_ptr(), dt, K, N, bits, g, _lib.ROUND_RNE, _lib.LAYOUT_GFX950,
                                             codes.data_ptr(), scale.data_ptr(), ws.data_ptr(), wsb, None))
        torch.cuda.synchronize()
        res.append((codes.cpu().numpy(), H.torch_to_bits(scale)))
    return res


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("bits", [8, 4])
def test_two_calls_second_smaller(dt, bits):
    # first call: large values in every column, so that stale maxima would
    # raise the scales of the second, smaller and weaker, weight
    big = H.make_weight(512, 1024, dt, seed=11, std=3.0)
    small = H.make_weight(256, 320, dt, seed=12, std=0.02)
    for wb in (big, small):
        (c0, s0), (c1, s1) = _both(wb, dt, bits, -1)
        assert np.array_equal(s0, s1)
        assert np.array_equal(c0, c1)


def test_group_wise_needs_no_scratch():
    wb = H.make_weight(256, 128, H.BF16, seed=13)
    (c0, s0), (c1, s1) = _both(wb, H.BF16, 4, 128)
    assert np.array_equal(s0, s1) and np.array_equal(c0, c1)


def test_rejects_sizes_beyond_the_static_array():
    # argument validation happens before any device work
    w = torch.zeros(16, dtype=torch.uint8, device=DEV)
    rc = _lib.lib.wol_quantize_static(w.data_ptr(), H.BF16, 64, 65536 + 16, 8, -1, _lib.ROUND_RNE,
                                      _lib.LAYOUT_GFX950, w.data_ptr(), w.data_ptr(), None)
    assert rc == 5  # WOL_ERR_BAD_SHAPE
    assert b"shape" in _lib.lib.wol_status_str(rc)
