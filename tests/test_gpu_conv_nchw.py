"""The convolution kernel that reads NCDHW activations and KCTRS weights as they are
(AMOS_PIPE_NCHW: one launch, no workspace) against the CPU oracle on the same seeded inputs,
through the C ABI.  Bars as everywhere: int8 bit-exact, fp16 / bf16 max-rel 1e-2 and mean-rel 1e-3
against the fp64-accumulated exact-product result."""
import ctypes

import numpy as np
import pytest

from conftest import make_operand, to_device
from oracle import cpu_oracle as co

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_REL = 1e-2, 1e-3


def _check(got, ref, dtype, what):
    if dtype == "int8":
        bad = int((got != ref).sum())
        assert got.dtype == np.int32 and bad == 0, "%s: %d of %d int32 outputs differ" % (what, bad, got.size)
    else:
        mx, mean = co.rel_errors(got, ref)
        assert mx <= MAX_REL and mean <= MEAN_REL, "%s: max_rel=%.3e mean_rel=%.3e" % (what, mx, mean)


def _cfg(_lib, tj):
    return dict(tile_i=64, tile_j=tj, split_k=1, pipeline=_lib.AMOS_PIPE_NCHW)


# N, C, H, W, K, stride, pad, dil
CASES_2D = [
    (2, 64, 14, 14, 64, 1, 1, 1),
    (3, 128, 7, 8, 40, 1, 1, 1),       # several images per tile, ragged output channels
    (1, 64, 20, 18, 72, 1, 1, 1),      # ragged last tile of positions, two tiles of channels
    (2, 64, 9, 12, 96, 1, 0, 1),       # no padding
    (2, 64, 10, 12, 64, 2, 1, 1),      # stride
    (2, 64, 12, 12, 64, 1, 2, 2),      # dilation
    (1, 192, 16, 16, 130, (1, 2), (1, 2), 1),
    (5, 64, 6, 6, 64, 1, 1, 1),
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("tj", [128, 256])
@pytest.mark.parametrize("case", CASES_2D)
def test_conv2d_nchw_direct(gpu, dtype, tj, case):
    from amos_amd import _lib, ops
    N, C, H, W, K, st, pd, dl = case
    if dtype == "int8" and (H * W) % 8:
        pytest.skip("int8 needs channel planes of whole 8-byte loads")
    rng = np.random.default_rng(N * 1000 + C + H * 7 + K)
    x, w = make_operand(rng, (N, C, H, W), dtype), make_operand(rng, (K, C, 3, 3), dtype)
    print("conv2d nchw", dtype, tj, case, flush=True)
    oshape = ops.conv_out_shape((N, C, 1, H, W), (K, C, 1, 3, 3), (1,) + ops._tup(st, 2), (0,) + ops._tup(pd, 2), (1,) + ops._tup(dl, 2))
    opq, J = oshape[3] * oshape[4], N * oshape[3] * oshape[4]
    if max((min(j0 + tj, J) - 1) // opq - j0 // opq + 1 for j0 in range(0, J, tj)) > 4:
        # a tile would touch more than four images: the pipeline says so instead of running
        with pytest.raises(_lib.AmosError, match="more than four images"):
            ops.conv2d(to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj))
        return
    got = ops.conv2d(to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj)).cpu().numpy()
    ref = co.lib_conv2d(x, w, dtype, st, pd, dl, acc="float64") if dtype != "int8" else co.lib_conv2d(x, w, dtype, st, pd, dl)
    _check(got, ref, dtype, "conv2d %s tile 64x%d %s" % (dtype, tj, case))


# N, C, D, H, W, K, stride, pad, dil
CASES_3D = [
    (1, 64, 5, 12, 12, 64, 1, 1, 1),
    (2, 64, 3, 6, 8, 40, (2, 1, 2), (1, 1, 0), 1),
    (1, 128, 4, 10, 10, 80, 1, (0, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("tj", [128, 256])
@pytest.mark.parametrize("case", CASES_3D)
def test_conv3d_nchw_direct(gpu, dtype, tj, case):
    from amos_amd import _lib, ops
    N, C, D, H, W, K, st, pd, dl = case
    if dtype == "int8" and (H * W) % 8:
        pytest.skip("int8 needs channel planes of whole 8-byte loads")
    rng = np.random.default_rng(N * 1000 + C + D * 31 + H * 7 + K)
    x, w = make_operand(rng, (N, C, D, H, W), dtype), make_operand(rng, (K, C, 3, 3, 3), dtype)
    print("conv3d nchw", dtype, tj, case, flush=True)
    got = ops.conv3d(to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj)).cpu().numpy()
    ref = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64") if dtype != "int8" else co.lib_conv3d(x, w, dtype, st, pd, dl)
    _check(got, ref, dtype, "conv3d %s tile 64x%d %s" % (dtype, tj, case))


def test_conv2d_nchw_unaligned_weights_and_fused_tail(gpu):
    """weights that do not start on a 16-byte boundary take the per-channel loader; D is added"""
    import torch
    from amos_amd import _lib, ops
    rng = np.random.default_rng(77)
    x, w = make_operand(rng, (2, 64, 10, 10), "float16"), make_operand(rng, (48, 64, 3, 3), "float16")
    dx = to_device(x, "float16")
    wbuf = torch.zeros(w.size + 8, dtype=torch.float16, device="cuda")
    dw = wbuf[1:1 + w.size].view(48, 64, 3, 3)
    dw.copy_(torch.from_numpy(w))
    assert dw.data_ptr() % 16 == 2
    d = ops.conv_desc((2, 64, 1, 10, 10), (48, 64, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    cfg = ops.make_config(_cfg(_lib, 128))
    out = torch.empty((2, 48, 10, 10), dtype=torch.float32, device="cuda")
    _lib.check(_lib.load().amos_conv2d(ctypes.byref(d), ctypes.byref(cfg), dx.data_ptr(), dw.data_ptr(), out.data_ptr(),
                                       None, 0, None))
    torch.cuda.synchronize()
    ref = co.lib_conv2d(x, w, "float16", 1, 1, 1, acc="float64")
    _check(out.cpu().numpy(), ref, "float16", "unaligned weights")
    add = torch.randn((2, 48, 10, 10), device="cuda")
    got = ops.conv2d(dx, to_device(w, "float16"), 1, 1, 1, config=_cfg(_lib, 128), add=add)
    _check((got - add).cpu().numpy(), ref, "float16", "fused tail")


def test_conv_nchw_refusals(gpu):
    import torch
    from amos_amd import _lib, ops
    x = torch.zeros((1, 64, 8, 8), dtype=torch.float16, device="cuda")
    for ws, why in (((64, 64, 5, 5), "3x3"), ((64, 64, 3, 3), None)):
        w = torch.zeros(ws, dtype=torch.float16, device="cuda")
        if why is None:
            ops.conv2d(x, w, 1, 1, 1, config=_cfg(_lib, 128))
            continue
        with pytest.raises(_lib.AmosError) as e:
            ops.conv2d(x, w, 1, ws[2] // 2, 1, config=_cfg(_lib, 128))
        assert e.value.code == _lib.AMOS_ERR_INFEASIBLE and why in str(e.value)
    x24 = torch.zeros((1, 24, 8, 8), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.AmosError, match="64-byte"):
        ops.conv2d(x24, torch.zeros((64, 24, 3, 3), dtype=torch.float16, device="cuda"), 1, 1, 1, config=_cfg(_lib, 128))


def test_conv_nchw_benchmark_shapes(gpu):
    """the three benchmark convolutions at their full sizes: fp16 conv2d and int8 conv2d whole
    tensor, conv3d two images against the oracle"""
    import torch
    from amos_amd import _lib, ops
    rng = np.random.default_rng(0)
    x = rng.uniform(0, 1, (32, 256, 14, 14)).astype(np.float32).astype(np.float16)
    w = (rng.standard_normal((256, 256, 3, 3)) * 0.05).astype(np.float32).astype(np.float16)
    for tj in (128, 256):
        got = ops.conv2d(to_device(x, "float16"), to_device(w, "float16"), 1, 1, 1, config=_cfg(_lib, tj)).cpu().numpy()
        _check(got, co.lib_conv2d(x, w, "float16", 1, 1, 1, acc="float32"), "float16", "fp16 conv2d 64x%d" % tj)
    xi = rng.integers(-128, 128, (64, 128, 28, 28)).astype(np.int8)
    wi = rng.integers(-64, 64, (128, 128, 3, 3)).astype(np.int8)
    for tj in (128, 256):
        got = ops.conv2d(to_device(xi, "int8"), to_device(wi, "int8"), 1, 1, 1, config=_cfg(_lib, tj)).cpu().numpy()
        _check(got, co.lib_conv2d(xi, wi, "int8", 1, 1, 1), "int8", "int8 conv2d 64x%d" % tj)
    x3 = rng.standard_normal((2, 64, 16, 56, 56)).astype(np.float32).astype(np.float16)
    w3 = rng.standard_normal((64, 64, 3, 3, 3)).astype(np.float32).astype(np.float16)
    for tj in (128, 256):
        got = ops.conv3d(to_device(x3, "float16"), to_device(w3, "float16"), 1, 1, 1, config=_cfg(_lib, tj)).cpu().numpy()
        _check(got, co.lib_conv3d(x3, w3, "float16", 1, 1, 1, acc="float32"), "float16", "conv3d 64x%d" % tj)
