"""The tile order the tiled kernel walks (psg_tile_order, evaluated on the device for every workgroup id) against
the oracle's restatement of the reference's xcd_remap_bx_by (kernels/common/mma/mfma_preshuffle_pipeline.py:685-729),
bit-exact, including ragged grids."""

import numpy as np
import pytest
import torch

from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tiles_m,tiles_n,group_m", [(32, 16, 8), (64, 112, 8), (7, 5, 3), (3, 4, 2), (1, 13, 8), (13, 1, 4),
                                                      (17, 9, 16), (5, 5, 1), (41, 28, 8)])
def test_device_tile_order_equals_oracle(tiles_m, tiles_n, group_m):
    from flydsl_amd import _lib

    handle = _lib.lib()
    out = torch.full((tiles_m * tiles_n, 2), -1, dtype=torch.int32, device="cuda")
    rc = handle.psg_debug_tile_order(tiles_m, tiles_n, group_m, out.data_ptr(), _lib.stream_handle(None))
    assert rc == 0, handle.psg_last_error()
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = np.array([O.xcd_remap_bx_by(i // tiles_n, i % tiles_n, tiles_m * 128, tile_m=128, tile_n=256, n=tiles_n * 256,
                                       xcd_swizzle=group_m) for i in range(tiles_m * tiles_n)], dtype=np.int32)
    assert np.array_equal(got, want)
    assert len({(int(a), int(b)) for a, b in got}) == tiles_m * tiles_n
