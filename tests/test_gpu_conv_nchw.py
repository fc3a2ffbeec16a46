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


def _cfg(_lib, tj, ti=64):
    return dict(tile_i=ti, tile_j=tj, split_k=1, pipeline=_lib.AMOS_PIPE_NCHW)


TILES = [(64, 128), (64, 256), (32, 128), (32, 256), (128, 128), (128, 256)]


def _run(fn, *args, **kw):
    """the call, or a skip where the planner says that this tile does not suit the shape (a tile
    whose input patch is more than its threads load in one round, or more than LDS holds)"""
    from amos_amd import _lib
    try:
        return fn(*args, **kw)
    except _lib.AmosError as e:
        if e.code == _lib.AMOS_ERR_INFEASIBLE and ("load budget" in str(e) or "fit LDS" in str(e)):
            pytest.skip(str(e))
        raise


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
@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("case", CASES_2D)
def test_conv2d_nchw_direct(gpu, dtype, tile, case):
    from amos_amd import _lib, ops
    ti, tj = tile
    N, C, H, W, K, st, pd, dl = case
    if dtype == "int8" and (H * W) % 8:
        pytest.skip("int8 needs channel planes of whole 8-byte loads")
    rng = np.random.default_rng(N * 1000 + C + H * 7 + K)
    x, w = make_operand(rng, (N, C, H, W), dtype), make_operand(rng, (K, C, 3, 3), dtype)
    print("conv2d nchw", dtype, tile, case, flush=True)
    oshape = ops.conv_out_shape((N, C, 1, H, W), (K, C, 1, 3, 3), (1,) + ops._tup(st, 2), (0,) + ops._tup(pd, 2), (1,) + ops._tup(dl, 2))
    opq, J = oshape[3] * oshape[4], N * oshape[3] * oshape[4]
    if max((min(j0 + tj, J) - 1) // opq - j0 // opq + 1 for j0 in range(0, J, tj)) > 4:
        # a tile would touch more than four images: the pipeline says so instead of running
        with pytest.raises(_lib.AmosError, match="more than four images"):
            ops.conv2d(to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj, ti))
        return
    got = _run(ops.conv2d, to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj, ti)).cpu().numpy()
    ref = co.lib_conv2d(x, w, dtype, st, pd, dl, acc="float64") if dtype != "int8" else co.lib_conv2d(x, w, dtype, st, pd, dl)
    _check(got, ref, dtype, "conv2d %s tile %dx%d %s" % (dtype, ti, tj, case))


# N, C, D, H, W, K, stride, pad, dil
CASES_3D = [
    (1, 64, 5, 12, 12, 64, 1, 1, 1),
    (2, 64, 3, 6, 8, 40, (2, 1, 2), (1, 1, 0), 1),
    (1, 128, 4, 10, 10, 80, 1, (0, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("case", CASES_3D)
def test_conv3d_nchw_direct(gpu, dtype, tile, case):
    from amos_amd import _lib, ops
    ti, tj = tile
    N, C, D, H, W, K, st, pd, dl = case
    if dtype == "int8" and (H * W) % 8:
        pytest.skip("int8 needs channel planes of whole 8-byte loads")
    rng = np.random.default_rng(N * 1000 + C + D * 31 + H * 7 + K)
    x, w = make_operand(rng, (N, C, D, H, W), dtype), make_operand(rng, (K, C, 3, 3, 3), dtype)
    print("conv3d nchw", dtype, tile, case, flush=True)
    got = _run(ops.conv3d, to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj, ti)).cpu().numpy()
    ref = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64") if dtype != "int8" else co.lib_conv3d(x, w, dtype, st, pd, dl)
    _check(got, ref, dtype, "conv3d %s tile %dx%d %s" % (dtype, ti, tj, case))


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


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("tile", TILES)
def test_conv_nchw_weight_modes_agree(gpu, dtype, tile):
    """the three ways the weights reach LDS -- packed into the workspace by the call, packed once by
    their owner (AMOS_FLAG_WEIGHTS_PACKED), transposed by every workgroup (no workspace) -- give the
    same bits (the accumulation order does not depend on them), 2-d and 3-d"""
    import torch
    from amos_amd import _lib, ops
    lib = _lib.load()
    ti, tj = tile
    for xs, ws, op in (((2, 128, 1, 12, 12), (72, 128, 1, 3, 3), _lib.AMOS_OP_CONV2D),
                       ((1, 64, 3, 8, 8), (40, 64, 3, 3, 3), _lib.AMOS_OP_CONV3D)):
        rng = np.random.default_rng(ti + tj + len(dtype))
        x, w = make_operand(rng, xs, dtype), make_operand(rng, ws, dtype)
        dx, dw = to_device(x, dtype), to_device(w, dtype)
        pad = (0, 1, 1) if op == _lib.AMOS_OP_CONV2D else (1, 1, 1)
        d = ops.conv_desc(xs, ws, dx.dtype, (1, 1, 1), pad, (1, 1, 1))
        oshape = ops.conv_out_shape(xs, ws, (1, 1, 1), pad, (1, 1, 1))
        fn = lib.amos_conv2d if op == _lib.AMOS_OP_CONV2D else lib.amos_conv3d
        outs = []
        cfg = ops.make_config(_cfg(_lib, tj, ti))
        need = ops.workspace_bytes(op, d, cfg)
        assert need == x.itemsize * w.size == lib.amos_conv_packed_weights_bytes(op, ctypes.byref(d))
        wsb = torch.empty(need + 256, dtype=torch.uint8, device="cuda")
        ws_ptr = (wsb.data_ptr() + 255) // 256 * 256
        for mode in ("workspace", "none", "owner"):
            out = torch.full(oshape, -3, dtype=torch.int32 if dtype == "int8" else torch.float32, device="cuda")
            c = ops.make_config(_cfg(_lib, tj, ti))
            if mode == "workspace":
                rc = fn(ctypes.byref(d), ctypes.byref(c), dx.data_ptr(), dw.data_ptr(), out.data_ptr(), ws_ptr, need, None)
            elif mode == "none":
                rc = fn(ctypes.byref(d), ctypes.byref(c), dx.data_ptr(), dw.data_ptr(), out.data_ptr(), None, 0, None)
            else:
                packed = torch.empty(need, dtype=torch.uint8, device="cuda")
                _lib.check(lib.amos_conv_pack_weights(op, ctypes.byref(d), dw.data_ptr(), packed.data_ptr(), None))
                # [K][T*9][C]: the caller can check the layout itself
                want = dw.reshape(ws[0], ws[1], -1).permute(0, 2, 1).contiguous()
                assert torch.equal(packed.view(dw.dtype).view(want.shape), want)
                c.reserved[0] = _lib.AMOS_FLAG_WEIGHTS_PACKED
                assert ops.workspace_bytes(op, d, c) == 0
                rc = fn(ctypes.byref(d), ctypes.byref(c), dx.data_ptr(), packed.data_ptr(), out.data_ptr(), None, 0, None)
            if rc == _lib.AMOS_ERR_INFEASIBLE and b"load budget" in lib.amos_last_error():
                pytest.skip(lib.amos_last_error().decode())
            _lib.check(rc)
            torch.cuda.synchronize()
            # (a conv2d with aligned weights may leave the workspace unused: the mapper's model decides)
            assert mode != "workspace" or op == _lib.AMOS_OP_CONV2D or "packed" in ops.kernel_name(op, d, c)
            outs.append(out)
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
        ref = (co.lib_conv2d if op == _lib.AMOS_OP_CONV2D else co.lib_conv3d)(
            x if op == _lib.AMOS_OP_CONV3D else x[:, :, 0], w if op == _lib.AMOS_OP_CONV3D else w[:, :, 0], dtype, 1,
            1, 1, **({} if dtype == "int8" else {"acc": "float64"}))
        got = outs[0].cpu().numpy()
        _check(got if op == _lib.AMOS_OP_CONV3D else got[:, :, 0], ref, dtype, "weight modes %s %s" % (dtype, tile))


@pytest.mark.parametrize("tile", TILES)
def test_conv_nchw_load_widths_agree(gpu, tile):
    """16-bit activations whose channel planes are whole 16-byte runs are fetched with 16-byte loads
    where the tensor is 16-byte aligned and with 8-byte loads where it is not: same bits either
    way (the accumulation order does not depend on it), 2-d with groups that straddle image rows,
    and 3-d"""
    import torch
    from amos_amd import _lib, ops
    ti, tj = tile
    for xs, ws, st, pd in (((3, 64, 1, 6, 12), (72, 64, 1, 3, 3), (1, 1, 1), (0, 1, 1)),
                           ((2, 64, 3, 10, 12), (40, 64, 3, 3, 3), (1, 1, 1), (1, 1, 1))):
        op = _lib.AMOS_OP_CONV2D if xs[2] == 1 else _lib.AMOS_OP_CONV3D
        rng = np.random.default_rng(ti + tj + xs[3])
        x, w = make_operand(rng, xs, "float16"), make_operand(rng, ws, "float16")
        dw = to_device(w, "float16")
        n = int(np.prod(xs))
        big = torch.zeros(n + 16, dtype=torch.float16, device="cuda")
        assert big.data_ptr() % 16 == 0
        outs = []
        for shift in (8, 4):   # halves: 16 and 8 bytes past an aligned address
            dx = big[shift:shift + n].view(xs)
            dx.copy_(to_device(x, "float16"))
            assert dx.data_ptr() % 16 == (0 if shift == 8 else 8)
            print("load widths", tile, xs, "shift", shift, flush=True)
            if op == _lib.AMOS_OP_CONV2D:
                out = _run(ops.conv2d, dx[:, :, 0], dw[:, :, 0], st[1:], pd[1:], 1, config=_cfg(_lib, tj, ti))
            else:
                out = _run(ops.conv3d, dx, dw, st, pd, 1, config=_cfg(_lib, tj, ti))
            outs.append(out)
        assert torch.equal(outs[0], outs[1])
        d = ops.conv_desc(xs, ws, torch.float16, st, pd, (1, 1, 1))
        c = ops.make_config(_cfg(_lib, tj, ti))
        assert "ld16" in ops.kernel_name(op, d, c)
        ref = (co.lib_conv2d(x[:, :, 0], w[:, :, 0], "float16", st[1:], pd[1:], 1, acc="float64") if op == _lib.AMOS_OP_CONV2D
               else co.lib_conv3d(x, w, "float16", st, pd, 1, acc="float64"))
        _check(outs[0].cpu().numpy(), ref, "float16", "load widths %s %s" % (tile, xs))


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("tile", TILES)
def test_conv_nchw_macro_step_counts(gpu, dtype, tile):
    """one to five macro steps (64 bytes of channels each) per tile, with packed weights (two
    staging sets, loads two steps ahead) and without a workspace (one set), 8- and 16-byte patch
    loads: every path through the loaders' prologue, loop and tail of every instance"""
    import torch
    from amos_amd import _lib, ops
    lib = _lib.load()
    ti, tj = tile
    es = 1 if dtype == "int8" else 2
    for hw in ((8, 8), (6, 6)):      # channel planes of 128 / 72 bytes (16-bit): 16- and 8-byte loads
        if dtype == "int8" and (hw[0] * hw[1]) % 8:
            continue
        for steps in (1, 2, 3, 4, 5):
            C = steps * 64 // es
            xs, ws = (3, C, 1) + hw, (48, C, 1, 3, 3)
            rng = np.random.default_rng(steps * 100 + hw[0] + ti + tj)
            x, w = make_operand(rng, xs, dtype), make_operand(rng, ws, dtype)
            dx, dw = to_device(x, dtype), to_device(w, dtype)
            d = ops.conv_desc(xs, ws, dx.dtype, (1, 1, 1), (0, 1, 1), (1, 1, 1))
            oshape = ops.conv_out_shape(xs, ws, (1, 1, 1), (0, 1, 1), (1, 1, 1))
            cfg = ops.make_config(_cfg(_lib, tj, ti))
            need = ops.workspace_bytes(_lib.AMOS_OP_CONV2D, d, cfg)
            wsb = torch.empty(need + 256, dtype=torch.uint8, device="cuda")
            ws_ptr = (wsb.data_ptr() + 255) // 256 * 256
            ref = co.lib_conv2d(x[:, :, 0], w[:, :, 0], dtype, 1, 1, 1, **({} if dtype == "int8" else {"acc": "float64"}))
            outs = []
            for mode in ("workspace", "none"):
                print("macro steps", dtype, tile, hw, steps, mode, flush=True)
                out = torch.full(oshape, -3, dtype=torch.int32 if dtype == "int8" else torch.float32, device="cuda")
                c = ops.make_config(_cfg(_lib, tj, ti))
                rc = lib.amos_conv2d(ctypes.byref(d), ctypes.byref(c), dx.data_ptr(), dw.data_ptr(), out.data_ptr(),
                                     ws_ptr if mode == "workspace" else None, need if mode == "workspace" else 0, None)
                _lib.check(rc)
                torch.cuda.synchronize()
                _check(out.cpu().numpy()[:, :, 0], ref, dtype, "macro steps %s %s %s %d %s" % (dtype, tile, hw, steps, mode))
                outs.append(out)
            assert torch.equal(outs[0], outs[1])


def test_conv_nchw_random_shapes(gpu):
    """seeded random 3x3 convolutions (2-d and 3-d, strides, paddings, dilations, ragged channel
    counts, every tile) through AMOS_PIPE_NCHW against the oracle; shapes the planner refuses
    (a tile over more than four images, a patch above the loaders' budget or LDS) are skipped"""
    from amos_amd import _lib, ops
    rng = np.random.default_rng(20240607)
    ran = 0
    for it in range(220):
        dtype = ("float16", "float16", "bfloat16", "int8")[int(rng.integers(0, 4))]
        es = 1 if dtype == "int8" else 2
        three_d = rng.integers(0, 3) == 0
        N, K = int(rng.integers(1, 4)), int(rng.integers(8, 80))
        C = int(rng.integers(1, 4)) * 64 // es
        D = int(rng.integers(1, 4)) if three_d else 1
        H, W = int(rng.integers(3, 21)), int(rng.integers(3, 21))
        if (H * W * es) % 8:
            continue
        st = tuple(int(v) for v in rng.integers(1, 3, 3))
        pd = tuple(int(v) for v in rng.integers(0, 3, 3))
        dl = (1,) + tuple(int(v) for v in rng.integers(1, 3, 2))
        if not three_d:
            st, pd = (1,) + st[1:], (0,) + pd[1:]
        ti, tj = TILES[int(rng.integers(0, len(TILES)))]
        xs, ws = (N, C, D, H, W), (K, C, 3 if three_d else 1, 3, 3)
        if min(ops.conv_out_shape(xs, ws, st, pd, dl)) <= 0:
            continue
        x, w = make_operand(rng, xs, dtype), make_operand(rng, ws, dtype)
        print("random nchw", it, dtype, (ti, tj), xs, K, st, pd, dl, flush=True)
        try:
            if three_d:
                got = ops.conv3d(to_device(x, dtype), to_device(w, dtype), st, pd, dl, config=_cfg(_lib, tj, ti))
            else:
                got = ops.conv2d(to_device(x[:, :, 0], dtype), to_device(w[:, :, 0], dtype), st[1:], pd[1:], dl[1:],
                                 config=_cfg(_lib, tj, ti))
        except _lib.AmosError as e:
            assert e.code == _lib.AMOS_ERR_INFEASIBLE, str(e)
            continue
        kw = {} if dtype == "int8" else {"acc": "float64"}
        ref = (co.lib_conv3d(x, w, dtype, st, pd, dl, **kw) if three_d
               else co.lib_conv2d(x[:, :, 0], w[:, :, 0], dtype, st[1:], pd[1:], dl[1:], **kw))
        _check(got.cpu().numpy(), ref, dtype, "random %d %s %s %s" % (it, dtype, (ti, tj), xs))
        ran += 1
    assert ran >= 60, ran


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_conv_nchw_two_rounds_with_packed_weights(gpu, dtype):
    """a patch of more than 64 load groups (two rounds of the loaders, `pt2`) together with weights
    packed by their owner: against the oracle, and the same bits as with the weights read as they are"""
    import torch
    from amos_amd import _lib, ops
    lib = _lib.load()
    xs, ws = (4, 64, 1, 14, 14), (72, 64, 1, 3, 3)
    rng = np.random.default_rng(11)
    x, w = make_operand(rng, xs, dtype), make_operand(rng, ws, dtype)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    d = ops.conv_desc(xs, ws, dx.dtype, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    oshape = ops.conv_out_shape(xs, ws, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    need = lib.amos_conv_packed_weights_bytes(_lib.AMOS_OP_CONV2D, ctypes.byref(d))
    packed = torch.empty(need, dtype=torch.uint8, device="cuda")
    _lib.check(lib.amos_conv_pack_weights(_lib.AMOS_OP_CONV2D, ctypes.byref(d), dw.data_ptr(), packed.data_ptr(), None))
    outs = []
    for flags, wptr in ((_lib.AMOS_FLAG_WEIGHTS_PACKED, packed.data_ptr()), (0, dw.data_ptr())):
        c = ops.make_config(_cfg(_lib, 256, 64))
        c.reserved[0] = flags
        name = ops.kernel_name(_lib.AMOS_OP_CONV2D, d, c)
        assert name.endswith(",pt2>") and (",packed" in name) == bool(flags), name
        print("two rounds", dtype, name, flush=True)
        out = torch.full(oshape, -3, dtype=torch.float32, device="cuda")
        _lib.check(lib.amos_conv2d(ctypes.byref(d), ctypes.byref(c), dx.data_ptr(), wptr, out.data_ptr(), None, 0, None))
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    ref = co.lib_conv2d(x[:, :, 0], w[:, :, 0], dtype, 1, 1, 1, acc="float64")
    _check(outs[0].cpu().numpy()[:, :, 0], ref, dtype, "two rounds, packed weights, %s" % dtype)


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
    for ti, tj in [(64, 128), (64, 256), (32, 128)]:   # (32 x 256: the patch of a tile is above 256 threads' load budget)
        got = ops.conv2d(to_device(x, "float16"), to_device(w, "float16"), 1, 1, 1, config=_cfg(_lib, tj, ti)).cpu().numpy()
        _check(got, co.lib_conv2d(x, w, "float16", 1, 1, 1, acc="float32"), "float16", "fp16 conv2d %dx%d" % (ti, tj))
    xi = rng.integers(-128, 128, (64, 128, 28, 28)).astype(np.int8)
    wi = rng.integers(-64, 64, (128, 128, 3, 3)).astype(np.int8)
    for ti, tj in TILES:
        got = ops.conv2d(to_device(xi, "int8"), to_device(wi, "int8"), 1, 1, 1, config=_cfg(_lib, tj, ti)).cpu().numpy()
        _check(got, co.lib_conv2d(xi, wi, "int8", 1, 1, 1), "int8", "int8 conv2d %dx%d" % (ti, tj))
    x3 = rng.standard_normal((2, 64, 16, 56, 56)).astype(np.float32).astype(np.float16)
    w3 = rng.standard_normal((64, 64, 3, 3, 3)).astype(np.float32).astype(np.float16)
    for ti, tj in [(64, 128), (64, 256), (32, 128)]:   # (32 x 256: the patch of a tile is above 256 threads' load budget)
        got = ops.conv3d(to_device(x3, "float16"), to_device(w3, "float16"), 1, 1, 1, config=_cfg(_lib, tj, ti)).cpu().numpy()
        _check(got, co.lib_conv3d(x3, w3, "float16", 1, 1, 1, acc="float32"), "float16", "conv3d %dx%d" % (ti, tj))
