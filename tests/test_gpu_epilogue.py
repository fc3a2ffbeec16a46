"""Fused tail operation (out = acc + cast(D)) on every kernel family, through the C ABI.

The reference spells it as an element-wise stage behind the main op ("E = C + D",
tests/python/auto_tensorize/test_compute_transform_gemm.py:7-23) and checks the transformed
compute against its llvm build; here the oracle is the exact-product result plus D in float64
(int32 for the integer path, bit-exact), under the same bars as the un-fused kernels.
"""
import numpy as np
import pytest
import torch

from conftest import make_operand, to_device
from oracle import cpu_oracle as co
from test_gpu_parity import check

pytestmark = pytest.mark.gpu


def make_d(rng, shape, dtype, d_dtype):
    """D operand on the host (as float64 / int64 for the reference) and on the device"""
    if dtype == "int8":
        d = rng.integers(-(1 << 20), 1 << 20, size=shape).astype(np.int32)
        return d.astype(np.int64), torch.from_numpy(d).cuda()
    d = (rng.standard_normal(size=shape) * 4).astype(np.float32)
    t = torch.from_numpy(d).cuda().to({"float32": torch.float32, "float16": torch.float16,
                                       "bfloat16": torch.bfloat16}[d_dtype])
    return t.double().cpu().numpy(), t


def d_types(dtype):
    return ["int32"] if dtype == "int8" else ["float32", "float16", "bfloat16"]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", [
    # M, N, K, trans_a, trans_b, config
    (200, 136, 72, 0, 0, None),                                           # register-staged kernel, ragged
    (130, 264, 520, 1, 1, dict(tile_i=64, tile_j=128, split_k=3)),        # split-K: D is added once
    (512, 768, 256, 0, 1, dict(tile_i=256, tile_j=256, split_k=1, pipeline=3)),   # direct-to-LDS kernel
    (300, 520, 384, 0, 1, dict(tile_i=128, tile_j=128, split_k=1, pipeline=3)),
])
def test_gemm_add(gpu, dtype, case):
    from amos_amd import ops
    M, N, K, ta, tb, cfg = case
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    ref0 = co.lib_gemm(a, b, dtype, ta, tb, acc="float64")
    for dd in d_types(dtype):
        d_host, d_dev = make_d(rng, (M, N), dtype, dd)
        got = ops.gemm(to_device(a, dtype), to_device(b, dtype), ta, tb, config=cfg, add=d_dev).cpu().numpy()
        ref = (ref0.astype(np.int64) + d_host).astype(np.int32) if dtype == "int8" else ref0 + d_host
        check(got, ref, dtype, "gemm + D(%s) %s %s" % (dd, dtype, case))


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("cfg", [None, dict(tile_i=256, tile_j=256, split_k=1, pipeline=3)])
def test_bgemm_add(gpu, dtype, cfg):
    from amos_amd import ops
    B, M, N, K = 3, 256, 264, 128
    rng = np.random.default_rng(5)
    a = make_operand(rng, (B, M, K), dtype)
    b = make_operand(rng, (B, N, K), dtype)
    ref0 = co.lib_gemm(a, b, dtype, False, True, acc="float64")
    d_host, d_dev = make_d(rng, (B, M, N), dtype, d_types(dtype)[-1])
    got = ops.bgemm(to_device(a, dtype), to_device(b, dtype), False, True, config=cfg, add=d_dev).cpu().numpy()
    ref = (ref0.astype(np.int64) + d_host).astype(np.int32) if dtype == "int8" else ref0 + d_host
    check(got, ref, dtype, "bgemm + D %s %s" % (dtype, cfg))


CONV_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil, config
    (2, 128, 1, 14, 14, 96, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), None),                   # patch-staged
    (2, 256, 1, 9, 11, 64, 1, 3, 2, (1, 2, 1), (0, 1, 0), (1, 1, 2),
     dict(tile_i=64, tile_j=128, split_k=2, pipeline=4)),                                      # split-K, 4 waves
    (2, 128, 4, 6, 6, 24, 3, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1),
     dict(tile_i=128, tile_j=64, split_k=1, pipeline=5)),                                      # conv3d, 8 waves
    (2, 24, 1, 10, 10, 40, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), None),                    # register-staged
    (1, 24, 3, 5, 6, 8, 2, 2, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), dict(tile_i=64, tile_j=64, split_k=2)),
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_add(gpu, dtype, case):
    from amos_amd import ops
    N, C, D, H, W, K, T, R, S, st, pd, dl, cfg = case
    rng = np.random.default_rng(hash(case[:9]) % 2**32)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, T, R, S), dtype, "normal")
    ref0 = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64")
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    for dd in d_types(dtype):
        d_host, d_dev = make_d(rng, ref0.shape, dtype, dd)
        if D == 1 and T == 1:
            got = ops.conv2d(dx[:, :, 0], dw[:, :, 0], st[1:], pd[1:], dl[1:], config=cfg,
                             add=d_dev[:, :, 0].contiguous())[:, :, None]
        else:
            got = ops.conv3d(dx, dw, st, pd, dl, config=cfg, add=d_dev)
        ref = (ref0.astype(np.int64) + d_host).astype(np.int32) if dtype == "int8" else ref0 + d_host
        check(got.cpu().numpy(), ref, dtype, "conv + D(%s) %s %s" % (dd, dtype, case))


def test_epilogue_errors(gpu):
    import ctypes
    from amos_amd import _lib, ops
    a = torch.zeros(64, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        ops.gemm(a, a, add=torch.zeros(64, 32, device="cuda"))
    with pytest.raises(ValueError):
        ops.gemm(a, a, add=torch.zeros(64, 64, dtype=torch.int32, device="cuda"))
    lib = _lib.load()
    d = ops.gemm_desc(64, 64, 64, torch.float16)
    out = torch.zeros(64, 64, device="cuda")
    e = _lib.Epilogue(_lib.AMOS_EPI_ADD, _lib.AMOS_F32, None, 0, 0)
    rc = lib.amos_run_fused(_lib.AMOS_OP_GEMM, ctypes.byref(d), None, ctypes.byref(e), a.data_ptr(), a.data_ptr(),
                            out.data_ptr(), None, 0, None)
    assert rc == _lib.AMOS_ERR_BAD_ARG and b"operand is null" in lib.amos_last_error()
    e = _lib.Epilogue(7, _lib.AMOS_F32, out.data_ptr(), 0, 0)
    rc = lib.amos_run_fused(_lib.AMOS_OP_GEMM, ctypes.byref(d), None, ctypes.byref(e), a.data_ptr(), a.data_ptr(),
                            out.data_ptr(), None, 0, None)
    assert rc == _lib.AMOS_ERR_UNSUPPORTED
    e = _lib.Epilogue(_lib.AMOS_EPI_ADD, _lib.AMOS_F32, out.data_ptr(), 32, 0)
    rc = lib.amos_run_fused(_lib.AMOS_OP_GEMM, ctypes.byref(d), None, ctypes.byref(e), a.data_ptr(), a.data_ptr(),
                            out.data_ptr(), None, 0, None)
    assert rc == _lib.AMOS_ERR_BAD_ARG and b"below N" in lib.amos_last_error()


GROUPED_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil, groups
    (2, 64, 1, 12, 12, 96, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), 4),
    (3, 24, 1, 9, 7, 24, 1, 3, 3, (1, 2, 1), (0, 1, 1), (1, 1, 1), 24),     # depthwise
    (2, 16, 1, 8, 8, 48, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), 16),     # depthwise, 3 outputs per channel
    (1, 32, 3, 6, 6, 16, 2, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1), 2),      # grouped conv3d
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", GROUPED_CASES)
def test_grouped_conv(gpu, dtype, case):
    """grouped and depthwise convolution (reference computes:
    benchmark/amos/mapping_groupedconv2d_tensorcore.py:7-60, mapping_depthwiseconv2d_tensorcore.py:7-48)
    against the oracle run once per group, with and without split-K and a fused addition"""
    from amos_amd import _lib, ops
    N, C, D, H, W, K, T, R, S, st, pd, dl, G = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C // G, T, R, S), dtype, "normal")
    cg, kg = C // G, K // G
    ref = np.concatenate([co.lib_conv3d(np.ascontiguousarray(x[:, g * cg:(g + 1) * cg]),
                                        np.ascontiguousarray(w[g * kg:(g + 1) * kg]), dtype, st, pd, dl,
                                        acc="float64") for g in range(G)], axis=1)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    # (pipeline 1, the register-staged implicit GEMM, also for the depthwise cases, whose default is
    # the vector-ALU kernel)
    for cfg in (None, dict(tile_i=64, tile_j=64, split_k=2, pipeline=1)):
        if D == 1 and T == 1:
            got = ops.conv2d(dx[:, :, 0], dw[:, :, 0], st[1:], pd[1:], dl[1:], config=cfg, groups=G)[:, :, None]
        else:
            got = ops.conv3d(dx, dw, st, pd, dl, config=cfg, groups=G)
        check(got.cpu().numpy(), ref, dtype, "grouped conv %s %s cfg %s" % (dtype, case, cfg))
    d_host, d_dev = make_d(rng, ref.shape, dtype, d_types(dtype)[0])
    got = ops.conv3d(dx, dw, st, pd, dl, groups=G, add=d_dev).cpu().numpy()
    want = (ref.astype(np.int64) + d_host).astype(np.int32) if dtype == "int8" else ref + d_host
    check(got, want, dtype, "grouped conv + D %s %s" % (dtype, case))
    with pytest.raises(_lib.AmosError, match="not applicable"):
        ops.conv3d(dx, dw, st, pd, dl, groups=G, config=dict(tile_i=64, tile_j=64, split_k=1, pipeline=4))
