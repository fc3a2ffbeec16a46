"""amos_conv2d_noalloc (the library's own scratch array instead of a workspace argument) against
amos_conv2d with a caller-owned workspace, through the C ABI: bit for bit, on two calls in a row,
the second on a smaller input, plus the refusal of a convolution the array cannot hold."""
import ctypes

import numpy as np
import pytest

from conftest import make_operand, to_device
from oracle import cpu_oracle as co

pytestmark = pytest.mark.gpu


def _both(lib, ops, _lib, torch, dtype, xs, ws, pad, pipeline, split_k=1, tile=(128, 64), kernel=None):
    rng = np.random.default_rng(sum(xs) + sum(ws))
    x, w = make_operand(rng, xs, dtype), make_operand(rng, ws, dtype)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    d = ops.conv_desc((xs[0], xs[1], 1, xs[2], xs[3]), (ws[0], ws[1], 1, ws[2], ws[3]), dx.dtype, (1, 1, 1),
                      (0, pad, pad), (1, 1, 1))
    # (pipeline None: no configuration at all, the library's own choice)
    cfg = None if pipeline is None else ops.make_config(dict(tile_i=tile[0], tile_j=tile[1], split_k=split_k, pipeline=pipeline))
    cref = None if cfg is None else ctypes.byref(cfg)
    need = int(lib.amos_workspace_bytes(_lib.AMOS_OP_CONV2D, ctypes.byref(d), cref))
    assert 0 < need <= _lib.AMOS_NOALLOC_SCRATCH_BYTES
    if kernel:
        name = lib.amos_kernel_name(_lib.AMOS_OP_CONV2D, ctypes.byref(d), cref)
        assert name is not None and kernel in name.decode(), name
    oshape = (xs[0], ws[0], xs[2] + 2 * pad - ws[2] + 1, xs[3] + 2 * pad - ws[3] + 1)
    odt = torch.int32 if dtype == "int8" else torch.float32
    ws_t = torch.empty(need + 256, dtype=torch.uint8, device="cuda")
    ws_ptr = (ws_t.data_ptr() + 255) // 256 * 256
    want = torch.full(oshape, -7, dtype=odt, device="cuda")
    _lib.check(lib.amos_conv2d(ctypes.byref(d), cref, dx.data_ptr(), dw.data_ptr(), want.data_ptr(),
                               ws_ptr, need, None))
    got = torch.full(oshape, -9, dtype=odt, device="cuda")
    _lib.check(lib.amos_conv2d_noalloc(ctypes.byref(d), cref, dx.data_ptr(), dw.data_ptr(),
                                       got.data_ptr(), None))
    torch.cuda.synchronize()
    assert torch.equal(got, want), "no-alloc entry point differs from amos_conv2d for %s %s" % (xs, ws)
    ref = co.lib_conv2d(x, w, dtype, 1, pad, 1)
    if dtype == "int8":
        assert np.array_equal(got.cpu().numpy(), ref)
    else:
        mx, mean = co.rel_errors(got.cpu().numpy(), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (mx, mean)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_conv2d_noalloc_two_calls(gpu, dtype):
    import torch
    from amos_amd import _lib, ops
    lib = _lib.load()
    c = 128 if dtype == "int8" else 64
    # the patch-staged pipeline (relaid operands in the scratch array), named explicitly
    _both(lib, ops, _lib, torch, dtype, (6, 2 * c, 14, 14), (96, 2 * c, 3, 3), 1, _lib.AMOS_PIPE_PATCH8)
    # a smaller input right after it: what the first call left in the array must not show
    _both(lib, ops, _lib, torch, dtype, (2, c, 9, 11), (40, c, 3, 3), 1, _lib.AMOS_PIPE_PATCH8)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_conv2d_noalloc_default_choice_and_splits(gpu, dtype):
    """the other things the array holds: the packed weights of the NCDHW-direct kernel, which a call
    without a configuration chooses for these shapes, and the slices of a split's partial sums
    behind the pipeline's own share"""
    import torch
    from amos_amd import _lib, ops
    lib = _lib.load()
    c = 256 if dtype == "int8" else 128
    # (the benchmark's fp16 convolution: its default is the NCDHW-direct kernel)
    _both(lib, ops, _lib, torch, dtype, (32, 256, 14, 14), (256, 256, 3, 3), 1, None,
          kernel="amos_conv_nchw" if dtype == "float16" else None)
    _both(lib, ops, _lib, torch, dtype, (2, c, 12, 12), (64, c, 3, 3), 1, _lib.AMOS_PIPE_PATCH8, split_k=2, kernel="amos_conv_fprop")
    _both(lib, ops, _lib, torch, dtype, (2, c, 12, 12), (64, c, 3, 3), 1, _lib.AMOS_PIPE_NCHW, split_k=2, tile=(64, 128),
          kernel="amos_conv_nchw")


def test_conv2d_noalloc_refuses_what_the_array_cannot_hold(gpu):
    import torch
    from amos_amd import _lib, ops
    lib = _lib.load()
    d = ops.conv_desc((64, 256, 1, 56, 56), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    cfg = ops.make_config(dict(tile_i=128, tile_j=64, split_k=1, pipeline=_lib.AMOS_PIPE_PATCH8))
    assert ops.workspace_bytes(_lib.AMOS_OP_CONV2D, d, cfg) > _lib.AMOS_NOALLOC_SCRATCH_BYTES
    x = torch.zeros(16, dtype=torch.float16, device="cuda")   # never read: the call is refused before any launch
    rc = lib.amos_conv2d_noalloc(ctypes.byref(d), ctypes.byref(cfg), x.data_ptr(), x.data_ptr(), x.data_ptr(), None)
    assert rc == _lib.AMOS_ERR_WORKSPACE
    assert b"scratch" in lib.amos_last_error()
    # ... and one whose pipeline share fits but whose split slices do not
    d2 = ops.conv_desc((16, 256, 1, 28, 28), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    one = ops.make_config(dict(tile_i=64, tile_j=128, split_k=1, pipeline=_lib.AMOS_PIPE_NCHW))
    two = ops.make_config(dict(tile_i=64, tile_j=128, split_k=2, pipeline=_lib.AMOS_PIPE_NCHW))
    assert ops.workspace_bytes(_lib.AMOS_OP_CONV2D, d2, one) <= _lib.AMOS_NOALLOC_SCRATCH_BYTES
    assert ops.workspace_bytes(_lib.AMOS_OP_CONV2D, d2, two) > _lib.AMOS_NOALLOC_SCRATCH_BYTES
    rc = lib.amos_conv2d_noalloc(ctypes.byref(d2), ctypes.byref(two), x.data_ptr(), x.data_ptr(), x.data_ptr(), None)
    assert rc == _lib.AMOS_ERR_WORKSPACE and b"scratch" in lib.amos_last_error()
