"""mg_forward_index_static: the forward pass with the library's fixed device scratch array (for
callers that cannot allocate) gives the grid of mg_forward_index_ws bit for bit, on two calls in a
row, the second with a smaller input; sizes beyond the array are refused."""
import numpy as np
import pytest
import torch

import synth
from util import dev

pytestmark = pytest.mark.gpu


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    import libmolgrid_amd as mg
    from libmolgrid_amd import _capi
    lib = _capi.lib
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(11)
    # a ragged batch of three, then a smaller single example
    for sizes in ((700, 1200, 40), (90,)):
        nbatch = len(sizes)
        offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
        coords, types, radii = synth.small_index_case(rng, int(offsets[-1]), 28, 13.0)
        centers = rng.uniform(-1, 1, (nbatch, 3)).astype(np.float32)
        d_off, d_cen = torch.as_tensor(offsets).cuda(), dev(centers)
        dc, dt, dr = dev(coords), dev(types), dev(radii)
        for binary in (False, True):
            gm = mg.GridMaker(0.5, 23.5, binary)
            shape = (nbatch,) + gm.grid_dimensions(28)
            ref = torch.full(shape, 3.0, device="cuda")
            got = torch.full(shape, 5.0, device="cuda")
            largest = max(sizes)
            need = lib.mg_forward_index_workspace_size(gm._p, nbatch, largest, 28)
            assert 0 < need <= _capi.MG_STATIC_SCRATCH_BYTES
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            z3 = _capi.f3((0, 0, 0))
            assert lib.mg_forward_index_ws(gm._p, nbatch, d_off.data_ptr(), largest, d_cen.data_ptr(),
                                           z3, dc.data_ptr(), dt.data_ptr(), dr.data_ptr(), 28,
                                           ref.data_ptr(), ws.data_ptr(), need, stream) == 0
            assert lib.mg_forward_index_static(gm._p, nbatch, d_off.data_ptr(), largest,
                                               d_cen.data_ptr(), z3, dc.data_ptr(), dt.data_ptr(),
                                               dr.data_ptr(), 28, got.data_ptr(), stream) == 0
            torch.cuda.synchronize()
            assert float(ref.max()) > 0.5
            assert torch.equal(got, ref)
    # more atoms than the fixed array holds records for: refused, nothing launched
    gm = mg.GridMaker(0.5, 23.5)
    too_many = _capi.MG_STATIC_SCRATCH_BYTES // 16 + 1
    assert lib.mg_forward_index_workspace_size(gm._p, 1, too_many, 28) > _capi.MG_STATIC_SCRATCH_BYTES
    one = dev(np.zeros(4, np.float32))
    assert lib.mg_forward_index_static(gm._p, 1, None, too_many, None, _capi.f3((0, 0, 0)),
                                       one.data_ptr(), one.data_ptr(), one.data_ptr(), 28,
                                       one.data_ptr(), stream) == _capi.MG_ERR_OUT_OF_RANGE
