"""tl_spmm_noalloc, the entry point that allocates nothing (its scratch is an array inside the library's
device code): called through the C ABI and compared bit for bit with tl_spmm on the same inputs, two
calls in a row on the same GPU, the second with a smaller input, so that what the first call left in
the shared scratch would show."""
import ctypes

import numpy as np
import pytest
import torch

from tests.util import activations, ternary_weight

pytestmark = pytest.mark.gpu


def _call(fn_name, dw, x, scale, ws=None):
    from ternaryllm_amd import _lib
    L = _lib.lib()
    M, K = x.shape
    y = torch.full((M, dw.columns), float("nan"), dtype=x.dtype, device=x.device)
    code = _lib.TL_F16 if x.dtype == torch.float16 else _lib.TL_F32
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    head = (ctypes.byref(dw.header), dw.blob.data_ptr(), x.data_ptr(), code, _lib.TL_X_ROW_MAJOR, x.stride(0), M, y.data_ptr(), code,
            y.stride(0), scale.data_ptr(), code)
    if fn_name == "tl_spmm_noalloc":
        rc = L.tl_spmm_noalloc(*head, stream)
    else:
        rc = L.tl_spmm(*head, ws.data_ptr(), ws.numel(), stream)
    _lib.check(rc)
    return y


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_noalloc_entry_point_equals_tl_spmm(cuda, oracle, dtype):
    from ternaryllm_amd import _lib, ops
    from ternaryllm_amd.packing import PackedWeight
    K, N = 2100, 300
    w = ternary_weight(K, N, 0.7, 131)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    scale = (0.5 + torch.rand(N, generator=torch.Generator().manual_seed(5))).to(dtype).to(cuda)
    ws = torch.empty(40 << 20, dtype=torch.uint8, device=cuda)   # no room for partial sums: whole output tiles, as in the other entry point
    # row counts of every kernel: 1 (no scratch), 16 and 40 (K-major image of a few rows), 700 and 130 (row kernel);
    # each pair runs larger first, then smaller, back to back on one stream
    for sizes in ((700, 130), (40, 16), (300, 1), (16, 700)):
        for M in sizes:
            x = activations(M, K, 200 + M, dtype).to(cuda)
            print(f"case noalloc dtype={dtype} M={M}", flush=True)
            got = _call("tl_spmm_noalloc", dw, x, scale)
            want = _call("tl_spmm", dw, x, scale, ws)
            assert torch.equal(got, want), (dtype, M)
    # and the product itself, on exact inputs, against the oracle
    xi = activations(70, K, 9, dtype, integer=True)
    ones = torch.ones(N, dtype=dtype, device=cuda)
    y = _call("tl_spmm_noalloc", dw, xi.to(cuda), ones)
    assert np.array_equal(y.double().cpu().numpy(), oracle.fast_product(xi.double().numpy(), w))
    # an input whose image does not fit the scratch is refused, nothing is launched
    big = ops.DeviceWeight(PackedWeight.from_dense(ternary_weight(11008, 16, 0.9, 3)), cuda)
    xb = torch.zeros((1024, 11008), dtype=torch.float32, device=cuda)
    if dtype == torch.float32:
        with pytest.raises(ValueError, match="scratch"):
            _call("tl_spmm_noalloc", big, xb, torch.ones(16, dtype=torch.float32, device=cuda))
    else:
        _call("tl_spmm_noalloc", big, xb.half(), torch.ones(16, dtype=torch.float16, device=cuda))   # 22.5 MB: fits
