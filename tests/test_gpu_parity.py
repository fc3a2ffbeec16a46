"""HIP path vs the CPU oracle on the same seeded inputs, through the C ABI.

Bars: int8 -> int32 bit-exact against exact integer arithmetic; fp16 / bf16 within
max-rel-err 1e-2 and mean-rel-err 1e-3 of the fp32-accumulated CPU result (relative
error with the denominator floored at 1e-2 * rms(ref), oracle.cpu_oracle.rel_errors).
The te_literal loop nest rounds every product to the input dtype, as the reference's llvm
build does, so it sits 2^-11 (fp16) or 2^-8 (bf16) per product away from any matrix-core
result; it is compared with the reference's own tolerances: allclose(atol=rtol=1e-2) for
fp16 (reference: README.md:334), atol=rtol=1e-1 for bf16 (reference:
tests/python/auto_tensorize/manual_mapping_conv2d_fp16fp32_tensorcore.py:114), both scaled
by max(1, rms) of the output, and mean-rel-err <= 1e-3 for fp16 on the config-sized cases.
"""
import ctypes

import numpy as np
import pytest

from conftest import make_operand, to_device
from oracle import cpu_oracle as co

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_REL = 1e-2, 1e-3


def check_float(got, ref, what):
    mx, mean = co.rel_errors(got, ref)
    assert mx <= MAX_REL and mean <= MEAN_REL, "%s: max_rel=%.3e mean_rel=%.3e" % (what, mx, mean)


def check_literal(got, lit, dtype, what, mean_bar=None):
    if dtype == "int8":
        assert np.array_equal(got, lit), what
        return
    tol = 1e-2 if dtype == "float16" else 1e-1
    scale = max(1.0, float(np.sqrt(np.mean(lit.astype(np.float64) ** 2))))
    assert np.allclose(got, lit, atol=tol * scale, rtol=tol), "%s: max abs diff %.3e (scale %.2f)" % (
        what, float(np.abs(got - lit).max()), scale)
    if mean_bar is not None:
        assert co.rel_errors(got, lit)[1] <= mean_bar, what


def check(got, ref, dtype, what):
    if dtype == "int8":
        assert got.dtype == np.int32
        bad = int((got != ref).sum())
        assert bad == 0, "%s: %d of %d int32 outputs differ" % (what, bad, got.size)
    else:
        check_float(got, ref, what)


GEMM_SHAPES = [(64, 64, 64), (128, 256, 192), (200, 136, 72), (33, 17, 19), (1, 1, 1), (300, 70, 520)]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("trans", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("shape", GEMM_SHAPES)
def test_gemm_small(gpu, dtype, trans, shape):
    from amos_amd import ops
    M, N, K = shape
    ta, tb = trans
    rng = np.random.default_rng(hash((M, N, K, ta, tb)) % 2**32)
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    got = ops.gemm(to_device(a, dtype), to_device(b, dtype), ta, tb).cpu().numpy()
    ref = co.lib_gemm(a, b, dtype, ta, tb, acc="float64")
    check(got, ref, dtype, "gemm %s %s %s vs exact" % (dtype, trans, shape))
    lit = co.te_literal_gemm(a, b, dtype, ta, tb, mode="exact" if dtype == "int8" else "te_literal")
    check_literal(got, lit, dtype, "gemm %s %s %s vs te_literal" % (dtype, trans, shape))


TILES = [(64, 64), (128, 128), (256, 256), (128, 64), (64, 128), (256, 128), (128, 256), (256, 64), (64, 256)]


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("split", [1, 3])
def test_gemm_every_tile(gpu, dtype, tile, split):
    from amos_amd import ops
    M, N, K = 520, 392, 1096
    rng = np.random.default_rng(7)
    a = make_operand(rng, (M, K), dtype)
    b = make_operand(rng, (N, K), dtype)
    cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=split)
    got = ops.gemm(to_device(a, dtype), to_device(b, dtype), False, True, config=cfg).cpu().numpy()
    ref = co.lib_gemm(a, b, dtype, False, True, acc="float64")
    check(got, ref, dtype, "gemm tile %s split %d" % (tile, split))


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
# direct-to-LDS copies: 256x256 and the smaller tiles (two and three LDS stages), eight waves
@pytest.mark.parametrize("pipeline,tile", [(3, (256, 256)), (3, (128, 128)), (3, (128, 256)),
                                           (3, (256, 128)), (0, (128, 128))])
@pytest.mark.parametrize("shape", [(256, 256, 128), (512, 768, 1024), (300, 520, 384), (1, 257, 128)])
def test_gemm_direct_pipeline(gpu, dtype, pipeline, tile, shape):
    from amos_amd import _lib, ops
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a = make_operand(rng, (M, K), dtype)
    b = make_operand(rng, (N, K), dtype)
    cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=1, pipeline=pipeline)
    d = ops.gemm_desc(M, N, K, to_device(a, dtype).dtype, False, True)
    name = ops.kernel_name(_lib.AMOS_OP_GEMM, d, cfg)
    if pipeline == 0 and M == 1:     # one row under the mapper's own pipeline: the vector-ALU kernel
        assert name.startswith("amos_skinny_gemm<")
    else:
        assert "amos_gemm_tn<%s,%dx%d" % ({"float16": "f16", "bfloat16": "bf16", "int8": "i8"}[dtype], tile[0], tile[1]) in name
    got = ops.gemm(to_device(a, dtype), to_device(b, dtype), False, True, config=cfg).cpu().numpy()
    check(got, co.lib_gemm(a, b, dtype, False, True, acc="float64"), dtype,
          "direct gemm %s pipe %d tile %s %s" % (dtype, pipeline, tile, shape))
    # batched through the same kernel
    ab = make_operand(rng, (3, M, K), dtype)
    bb = make_operand(rng, (3, N, K), dtype)
    gb = ops.bgemm(to_device(ab, dtype), to_device(bb, dtype), False, True, config=cfg).cpu().numpy()
    check(gb, co.lib_gemm(ab, bb, dtype, False, True, acc="float64"), dtype, "direct bgemm")


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("trans", [(0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("tile", TILES)
def test_gemm_row_contiguous_operands(gpu, dtype, trans, tile):
    """operands whose ROWS are contiguous (row-major B, transposed A) take vector loads along the
    rows and are transposed in registers; ragged K, row extents that are multiples of 8 but not
    of the tile, split-K, batches"""
    from amos_amd import _lib, ops
    M, N, K = 520, 392, 1104      # K: whole 16-byte chunks, not whole 64-element steps
    ta, tb = trans
    rng = np.random.default_rng(11)
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    da, db = to_device(a, dtype), to_device(b, dtype)
    d = ops.gemm_desc(M, N, K, da.dtype, ta, tb)
    cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=1)
    name = ops.kernel_name(_lib.AMOS_OP_GEMM, d, cfg)
    assert name.startswith("amos_igemm<") and "tvec" in name, name
    ref = co.lib_gemm(a, b, dtype, ta, tb, acc="float64")
    for split in (1, 3):
        got = ops.gemm(da, db, ta, tb, config=dict(cfg, split_k=split)).cpu().numpy()
        check(got, ref, dtype, "%s %s tile %s split %d" % (name, trans, tile, split))
    if tile == (128, 128):
        ab = make_operand(rng, (3, K, M) if ta else (3, M, K), dtype)
        bb = make_operand(rng, (3, N, K) if tb else (3, K, N), dtype)
        gb = ops.bgemm(to_device(ab, dtype), to_device(bb, dtype), ta, tb, config=cfg).cpu().numpy()
        check(gb, co.lib_gemm(ab, bb, dtype, ta, tb, acc="float64"), dtype, "batched %s" % name)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("trans", [(0, 0), (1, 1), (1, 0)])
def test_gemm_row_contiguous_operands_through_transposed_copies(gpu, dtype, trans):
    """large GEMMs with a transposed A / a row-major B and a workspace: the operands are copied
    K-contiguous and the direct-to-LDS kernel runs; without workspace (or with the register-staged
    pipeline asked for) the register-staged kernel does, and both agree with the oracle"""
    import torch
    from amos_amd import _lib, ops
    ta, tb = trans
    M, N, K = 2056, 1992, 1024      # ragged M and N, whole K steps
    rng = np.random.default_rng(31)
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    da, db = to_device(a, dtype), to_device(b, dtype)
    d = ops.gemm_desc(M, N, K, da.dtype, ta, tb)
    assert ops.workspace_bytes(_lib.AMOS_OP_GEMM, d) > 0
    assert "amos_gemm_tn" in ops.kernel_name(_lib.AMOS_OP_GEMM, d, None)
    assert "amos_igemm" in ops.kernel_name(_lib.AMOS_OP_GEMM, d, dict(tile_i=128, tile_j=128, split_k=1,
                                                                      pipeline=_lib.AMOS_PIPE_STAGED))
    ref = co.lib_gemm(a, b, dtype, bool(ta), bool(tb), acc="float64")
    got = ops.gemm(da, db, bool(ta), bool(tb))
    check(got.cpu().numpy(), ref, dtype, "transposed-copy gemm %s %s" % (dtype, trans))
    staged = ops.gemm(da, db, bool(ta), bool(tb), config=dict(tile_i=128, tile_j=128, split_k=1,
                                                              pipeline=_lib.AMOS_PIPE_STAGED))
    check(staged.cpu().numpy(), ref, dtype, "staged gemm %s %s" % (dtype, trans))
    # no workspace: the same call still works (register-staged kernel)
    out = torch.empty_like(got)
    _lib.check(_lib.load().amos_gemm(ctypes.byref(d), None, da.data_ptr(), db.data_ptr(), out.data_ptr(), None, 0, None))
    torch.cuda.synchronize()
    check(out.cpu().numpy(), ref, dtype, "gemm without workspace %s %s" % (dtype, trans))
    # batched, with the fused tail
    Bn, m, n, k = 5, 1000, 1096, 1024
    ab = make_operand(rng, (Bn, k, m) if ta else (Bn, m, k), dtype)
    bb = make_operand(rng, (Bn, n, k) if tb else (Bn, k, n), dtype)
    dd = torch.randn((Bn, m, n), device="cuda").to(torch.int32 if dtype == "int8" else torch.float32)
    bd = ops.bgemm_desc(Bn, m, n, k, da.dtype, ta, tb)
    assert "amos_gemm_tn" in ops.kernel_name(_lib.AMOS_OP_BGEMM, bd, None)
    gb = ops.bgemm(to_device(ab, dtype), to_device(bb, dtype), bool(ta), bool(tb), add=dd)
    check((gb - dd).cpu().numpy(), co.lib_gemm(ab, bb, dtype, bool(ta), bool(tb), acc="float64"), dtype,
          "transposed-copy bgemm %s %s" % (dtype, trans))


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("trans", [(0, 1), (0, 0), (1, 1), (1, 0)])
@pytest.mark.parametrize("K", [1000, 1027])
def test_gemm_ragged_k_through_padded_copies(gpu, dtype, trans, K):
    """K that is not a whole number of K steps (or not even of 16-byte vectors): with a workspace
    both operands are copied with zero-filled K steps and the direct-to-LDS kernel runs"""
    import torch
    from amos_amd import _lib, ops
    ta, tb = trans
    M, N = 1032, 1544
    rng = np.random.default_rng(41 + K)
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    da, db = to_device(a, dtype), to_device(b, dtype)
    d = ops.gemm_desc(M, N, K, da.dtype, ta, tb)
    es = 1 if dtype == "int8" else 2
    kp = -(-K // (128 // es)) * (128 // es)
    # (fp16 with K a multiple of 8 keeps its vector loaders in the register-staged kernel: copies
    # only pay for larger problems than this one)
    copies = dtype == "int8" or K % 8 != 0
    assert (ops.workspace_bytes(_lib.AMOS_OP_GEMM, d) >= (M + N) * kp * es) == copies
    # on copies both operands are K-contiguous vectors: the direct-to-LDS kernel or, where the
    # mapper's model prefers a small tile, the register-staged one with its vector loaders
    name = ops.kernel_name(_lib.AMOS_OP_GEMM, d, None)
    assert ("amos_gemm_tn" in name or ",vec,vec," in name) if copies else name.startswith("amos_igemm<"), name
    ref = co.lib_gemm(a, b, dtype, bool(ta), bool(tb), acc="float64")
    got = ops.gemm(da, db, bool(ta), bool(tb))
    check(got.cpu().numpy(), ref, dtype, "padded-copy gemm %s %s K=%d" % (dtype, trans, K))
    if copies:
        direct = dict(tile_i=128, tile_j=128, split_k=1, pipeline=_lib.AMOS_PIPE_DIRECT8)
        assert "amos_gemm_tn" in ops.kernel_name(_lib.AMOS_OP_GEMM, d, direct)
        got = ops.gemm(da, db, bool(ta), bool(tb), config=direct)
        check(got.cpu().numpy(), ref, dtype, "padded-copy gemm, direct tile %s %s K=%d" % (dtype, trans, K))
    staged = ops.gemm(da, db, bool(ta), bool(tb), config=dict(tile_i=64, tile_j=64, split_k=1,
                                                              pipeline=_lib.AMOS_PIPE_STAGED))
    check(staged.cpu().numpy(), ref, dtype, "staged gemm %s %s K=%d" % (dtype, trans, K))


SKINNY_CASES = [
    # M, N, K, trans_a, trans_b
    (1, 1000, 2048, 0, 1), (8, 1031, 1000, 0, 1), (5, 333, 1000, 0, 1), (3000, 1, 520, 0, 0), (777, 8, 264, 0, 1),
    (7, 7, 72, 0, 1), (1, 4099, 8192, 0, 1), (2050, 3, 16, 0, 1),
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", SKINNY_CASES)
def test_gemm_skinny(gpu, dtype, case):
    """GEMV and dense layers on a small batch (at most 8 rows on one side within 16 KB, K-contiguous
    operands) on the vector-ALU kernel: against the oracle, bit for bit in int8 against the register-staged
    kernel, with the fused addition"""
    import torch
    from amos_amd import _lib, ops
    M, N, K, ta, tb = case
    if dtype == "int8" and K % 16:
        K += 16 - K % 16           # whole 16-byte chunks of int8
    rng = np.random.default_rng(hash(case) % 2**32)
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    da, db = to_device(a, dtype), to_device(b, dtype)
    d = ops.gemm_desc(M, N, K, da.dtype, ta, tb)
    assert ops.kernel_name(_lib.AMOS_OP_GEMM, d, None).startswith("amos_skinny_gemm<")
    cfg = ops.default_config(_lib.AMOS_OP_GEMM, d)
    assert ops.kernel_name(_lib.AMOS_OP_GEMM, d, cfg).startswith("amos_skinny_gemm<")
    ref = co.lib_gemm(a, b, dtype, bool(ta), bool(tb), acc="float64")
    got = ops.gemm(da, db, bool(ta), bool(tb)).cpu().numpy()
    check(got, ref, dtype, "skinny gemm %s %s" % (dtype, case))
    staged = dict(tile_i=64, tile_j=64, split_k=1, pipeline=_lib.AMOS_PIPE_STAGED)
    assert ops.kernel_name(_lib.AMOS_OP_GEMM, d, staged).startswith("amos_igemm<")
    other = ops.gemm(da, db, bool(ta), bool(tb), config=staged).cpu().numpy()
    if dtype == "int8":
        assert np.array_equal(got, other)
    d_host = rng.integers(-1000, 1000, got.shape).astype(got.dtype)
    with_d = ops.gemm(da, db, bool(ta), bool(tb), add=torch.from_numpy(d_host).cuda()).cpu().numpy()
    want = (ref.astype(np.int64) + d_host).astype(np.int32) if dtype == "int8" else ref + d_host
    check(with_d, want, dtype, "skinny gemm + D %s %s" % (dtype, case))


def test_gemm_skinny_limits(gpu):
    """past the limits of the vector-ALU kernel (rows, LDS bytes, K-contiguous operands, a single
    GEMM) the matrix-core kernels run, with the same results"""
    import torch
    from amos_amd import _lib, ops
    rng = np.random.default_rng(5)
    for (M, N, K, ta, tb) in ((9, 500, 512, 0, 1), (4, 500, 4096, 0, 1), (4, 504, 512, 0, 0), (4, 500, 516, 0, 1)):
        a = make_operand(rng, (K, M) if ta else (M, K), "float16")
        b = make_operand(rng, (N, K) if tb else (K, N), "float16")
        d = ops.gemm_desc(M, N, K, torch.float16, ta, tb)
        assert ops.kernel_name(_lib.AMOS_OP_GEMM, d, None).startswith("amos_igemm<"), (M, N, K)
        got = ops.gemm(to_device(a, "float16"), to_device(b, "float16"), bool(ta), bool(tb)).cpu().numpy()
        check(got, co.lib_gemm(a, b, "float16", bool(ta), bool(tb), acc="float64"), "float16", "gemm %s" % ((M, N, K),))
    bd = ops.bgemm_desc(3, 4, 500, 512, torch.float16, False, True)
    assert not ops.kernel_name(_lib.AMOS_OP_BGEMM, bd, None).startswith("amos_skinny")


def test_gemm_direct_pipeline_rejects_ragged_k(gpu):
    import torch
    from amos_amd import _lib, ops
    a = torch.zeros((256, 72), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.AmosError) as e:
        ops.gemm(a, a, False, True, config=dict(tile_i=256, tile_j=256, split_k=1, pipeline=3))
    assert e.value.code == _lib.AMOS_ERR_INFEASIBLE


def test_gemm_four_wave_pipeline_withdrawn(gpu):
    """AMOS_PIPE_DIRECT4 (the four-wave direct-to-LDS instance) is refused: nothing is launched"""
    import torch
    from amos_amd import _lib, ops
    a = torch.zeros((256, 128), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.AmosError) as e:
        ops.gemm(a, a, False, True, config=dict(tile_i=256, tile_j=256, split_k=1, pipeline=_lib.AMOS_PIPE_DIRECT4))
    assert e.value.code == _lib.AMOS_ERR_INFEASIBLE and "withdrawn" in str(e.value)


@pytest.mark.skip(reason="the four-wave direct-to-LDS instance is withdrawn: a launch of it at 8192^3 ended in a "
                         "GPU memory fault whose cause is not found; the library refuses AMOS_PIPE_DIRECT4")
def test_gemm_four_wave_pipeline(gpu):
    from amos_amd import ops
    rng = np.random.default_rng(3)
    a = make_operand(rng, (300, 384), "float16")
    b = make_operand(rng, (520, 384), "float16")
    cfg = dict(tile_i=256, tile_j=256, split_k=1, pipeline=2)
    got = ops.gemm(to_device(a, "float16"), to_device(b, "float16"), False, True, config=cfg).cpu().numpy()
    check(got, co.lib_gemm(a, b, "float16", False, True, acc="float64"), "float16", "four-wave direct gemm")


def test_gemm_config1_512(gpu):
    """fp16 GEMM 512^3, inputs U[-1,1], against the full te_literal loop nest"""
    from amos_amd import ops
    rng = np.random.default_rng(0)
    a = make_operand(rng, (512, 512), "float16")
    b = make_operand(rng, (512, 512), "float16")
    got = ops.gemm(to_device(a, "float16"), to_device(b, "float16")).cpu().numpy()
    check_float(got, co.lib_gemm(a, b, "float16", acc="float32"), "C1 vs fp32 matmul")
    check_literal(got, co.te_literal_gemm(a, b, "float16", threads=8), "float16", "C1 vs te_literal", MEAN_REL)


def test_gemm_config2_8192(gpu):
    """fp16 GEMM 8192^3, row-major A, column-major B: slabs of rows against the oracle,
    plus linearity C(A, B) + C(A2, B) == C(A + A2, B) on exactly representable operands."""
    import torch
    from amos_amd import ops
    n = 8192
    rng = np.random.default_rng(0)
    a = make_operand(rng, (n, n), "float16")
    b = make_operand(rng, (n, n), "float16")
    da, db = to_device(a, "float16"), to_device(b, "float16")
    got = ops.gemm(da, db, False, True)
    g = got.cpu().numpy()
    rows = np.r_[0:4, 4093:4099, 8188:8192]
    ref = co.lib_gemm(a[rows], b, "float16", False, True, acc="float64")
    check_float(g[rows], ref, "C2 rows vs fp64")
    lit = co.te_literal_gemm(np.ascontiguousarray(a[rows[:4]]), b, "float16", False, True, threads=8)
    check_literal(g[rows[:4]], lit, "float16", "C2 rows vs te_literal", MEAN_REL)
    # column sums: sum_m C[m, n] == (sum_m A[m, :]) . B[n, :]  -- touches every output once
    colsum = got.double().sum(dim=0).cpu().numpy()
    want = (a.astype(np.float64).sum(axis=0))[None, :] @ b.astype(np.float64).T
    mx, mean = co.rel_errors(colsum, want[0])
    assert mx < 1e-2 and mean < 1e-3, (mx, mean)
    # small integers: every product and partial sum is exact in fp16 x fp16 -> fp32
    ai = rng.integers(-2, 3, size=(n, n)).astype(np.float16)
    bi = rng.integers(-2, 3, size=(n, n)).astype(np.float16)
    gi = ops.gemm(to_device(ai, "float16"), to_device(bi, "float16"), False, True)
    wi = torch.from_numpy(ai).cuda().float() @ torch.from_numpy(bi).cuda().float().T
    assert torch.equal(gi, wi)


def test_bgemm_small(gpu):
    from amos_amd import ops
    rng = np.random.default_rng(3)
    for dtype in ["float16", "bfloat16", "int8"]:
        for (B, M, N, K, ta, tb) in [(3, 70, 50, 40, 0, 1), (2, 64, 64, 64, 0, 0), (5, 17, 9, 33, 1, 1)]:
            a = make_operand(rng, (B, K, M) if ta else (B, M, K), dtype, "normal")
            b = make_operand(rng, (B, N, K) if tb else (B, K, N), dtype, "normal")
            got = ops.bgemm(to_device(a, dtype), to_device(b, dtype), ta, tb).cpu().numpy()
            check(got, co.lib_gemm(a, b, dtype, ta, tb, acc="float64"), dtype, "bgemm %s" % dtype)
            lit = co.te_literal_bgemm(a, b, dtype, ta, tb, mode="exact" if dtype == "int8" else "te_literal")
            check_literal(got, lit, dtype, "bgemm te_literal %s" % dtype)


def test_bgemm_config5a(gpu):
    """fp16 batched GEMM 192 x (512x512x64), scores = Q K^T, N(0,1) inputs: full check"""
    from amos_amd import ops
    rng = np.random.default_rng(0)
    q = make_operand(rng, (192, 512, 64), "float16", "normal")
    k = make_operand(rng, (192, 512, 64), "float16", "normal")
    got = ops.bgemm(to_device(q, "float16"), to_device(k, "float16"), False, True).cpu().numpy()
    check_float(got, co.lib_gemm(q, k, "float16", False, True, acc="float32"), "C5a vs fp32")
    lit = co.te_literal_bgemm(q, k, "float16", False, True, batches=(0, 4), threads=8)
    check_literal(got[:4], lit[:4], "float16", "C5a vs te_literal (4 batches)", MEAN_REL)


CONV2D_CASES = [
    # N, C, H, W, K, R, S, stride, pad, dil
    (1, 16, 8, 8, 16, 3, 3, 1, 1, 1),
    (2, 24, 14, 14, 40, 3, 3, 1, 1, 1),
    (3, 7, 9, 11, 5, 3, 2, 2, 1, 1),
    (2, 16, 15, 15, 32, 3, 3, 1, 2, 2),
    (1, 3, 32, 32, 8, 7, 7, 2, 3, 1),
    (2, 64, 7, 7, 64, 1, 1, 1, 0, 1),
    (2, 32, 10, 10, 16, 1, 1, 2, 0, 1),
    (1, 8, 5, 5, 4, 5, 5, 1, 0, 1),
    (1, 4, 12, 12, 4, 9, 9, 1, 4, 1),   # 81 taps: compare path instead of the tap bitmask
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", CONV2D_CASES)
def test_conv2d_small(gpu, dtype, case):
    from amos_amd import ops
    N, C, H, W, K, R, S, st, pd, dl = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, H, W), dtype)
    w = make_operand(rng, (K, C, R, S), dtype)
    got = ops.conv2d(to_device(x, dtype), to_device(w, dtype), st, pd, dl).cpu().numpy()
    ref = co.lib_conv2d(x, w, dtype, st, pd, dl, acc="float64")
    check(got, ref, dtype, "conv2d %s %s" % (dtype, case))
    lit = co.te_literal_conv2d(x, w, dtype, st, pd, dl, mode="exact" if dtype == "int8" else "te_literal")
    check_literal(got, lit, dtype, "conv2d te_literal %s %s" % (dtype, case))


@pytest.mark.parametrize("tile", TILES)
def test_conv2d_every_tile(gpu, tile):
    from amos_amd import ops
    rng = np.random.default_rng(11)
    x = make_operand(rng, (3, 40, 13, 13), "int8")
    w = make_operand(rng, (72, 40, 3, 3), "int8")
    for split in (1, 2):
        cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=split)
        got = ops.conv2d(to_device(x, "int8"), to_device(w, "int8"), 1, 1, 1, config=cfg).cpu().numpy()
        check(got, co.lib_conv2d(x, w, "int8", 1, 1, 1), "int8", "conv2d tile %s split %d" % (tile, split))


PATCH_CONV_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil   (C * element size is a multiple of 128 bytes)
    (2, 128, 1, 14, 14, 96, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1)),
    (5, 128, 1, 7, 7, 40, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1)),     # tiles straddle images
    (2, 256, 1, 9, 11, 64, 1, 3, 2, (1, 2, 1), (0, 1, 0), (1, 1, 2)),    # stride, dilation
    (3, 128, 1, 8, 8, 130, 1, 1, 1, (1, 1, 1), (0, 0, 0), (1, 1, 1)),    # 1x1, ragged K tile
    (1, 128, 1, 20, 20, 32, 1, 5, 5, (1, 1, 1), (0, 2, 2), (1, 1, 1)),
    (1, 128, 1, 13, 13, 16, 1, 3, 3, (1, 2, 2), (0, 0, 0), (1, 1, 1)),   # valid conv, stride 2
    (2, 128, 4, 6, 6, 24, 3, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1)),     # conv3d
    (1, 128, 5, 5, 7, 48, 2, 3, 2, (2, 1, 1), (1, 0, 1), (2, 1, 1)),     # conv3d stride / dilation in depth
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", PATCH_CONV_CASES)
def test_conv_patch_pipeline(gpu, dtype, case):
    """patch-staged convolution (4 and 8 waves): every tile shape, with and without split-K"""
    from amos_amd import _lib, ops
    N, C, D, H, W, K, T, R, S, st, pd, dl = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, T, R, S), dtype, "normal")
    ref = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64")
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    tiles = [(64, 64), (128, 64), (64, 128), (128, 128), (256, 64), (256, 128), (128, 256), (64, 256)]
    # (pipeline, flags): 4 waves; 8 waves with the 3x3 taps unrolled where that applies; 8 waves table-driven
    variants = [(_lib.AMOS_PIPE_PATCH, 0), (_lib.AMOS_PIPE_PATCH8, 0), (_lib.AMOS_PIPE_PATCH8, 1)]
    for tile, split, (pipe, flags) in [(t, s, v) for t in tiles for s in (1, 2) for v in variants]:
        if True:
            cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=split, pipeline=pipe, flags=flags)
            try:
                if D == 1 and T == 1:
                    got = ops.conv2d(dx[:, :, 0], dw[:, :, 0], st[1:], pd[1:], dl[1:], config=cfg)[:, :, None]
                else:
                    got = ops.conv3d(dx, dw, st, pd, dl, config=cfg)
            except _lib.AmosError as e:
                # a tile that spans too many slices or a patch too large: reported, never silent
                assert e.code == _lib.AMOS_ERR_INFEASIBLE and "not applicable" in str(e)
                continue
            check(got.cpu().numpy(), ref, dtype,
                  "patch conv %s %s tile %s split %d pipeline %d flags %d" % (dtype, case, tile, split, pipe, flags))


WALK_CASES = [
    # more tiles than compute units, 3x3 windows, at least two macro steps per tile
    ("float16", (16, 128, 1, 41, 41, 72, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1))),    # ragged K-out and J
    ("int8", (24, 256, 1, 40, 40, 64, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1))),
    ("float16", (4, 64, 9, 32, 32, 64, 3, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1))),      # three macro steps per tile
    ("bfloat16", (5, 64, 10, 34, 30, 40, 3, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1))),
]


@pytest.mark.parametrize("dtype,case", WALK_CASES)
def test_conv_tile_walk(gpu, dtype, case):
    """workgroups that walk several tiles: against the oracle, and bit for bit against the same
    kernel with one tile per workgroup (same accumulation order)"""
    import torch
    from amos_amd import _lib, ops
    N, C, D, H, W, K, T, R, S, st, pd, dl = case
    rng = np.random.default_rng(11)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, T, R, S), dtype, "normal")
    ref = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64")
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    is2d = D == 1 and T == 1
    xs5, ws5 = (N, C, D, H, W), (K, C, T, R, S)
    op = _lib.AMOS_OP_CONV2D if is2d else _lib.AMOS_OP_CONV3D
    desc = ops.conv_desc(xs5, ws5, getattr(torch, dtype), st, pd, dl)
    d_add = torch.randn(ref.shape, device="cuda").to(torch.int32 if dtype == "int8" else torch.float32)
    walked = 0
    for tile in [(64, 128), (128, 64)]:
        outs = {}
        for flags in (0, _lib.AMOS_FLAG_NO_TILE_WALK):
            cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=1, pipeline=_lib.AMOS_PIPE_PATCH8, flags=flags)
            name = ops.kernel_name(op, desc, cfg)
            assert name is not None and "9taps" in name and (("walk" in name) == (flags == 0)), name
            for add in (None, d_add):
                if is2d:
                    got = ops.conv2d(dx[:, :, 0], dw[:, :, 0], st[1:], pd[1:], dl[1:], config=cfg,
                                     add=None if add is None else add[:, :, 0])[:, :, None]
                else:
                    got = ops.conv3d(dx, dw, st, pd, dl, config=cfg, add=add)
                outs[(flags, add is None)] = got
        walked += 1
        assert torch.equal(outs[(0, True)], outs[(_lib.AMOS_FLAG_NO_TILE_WALK, True)]), "tile %s" % (tile,)
        assert torch.equal(outs[(0, False)], outs[(_lib.AMOS_FLAG_NO_TILE_WALK, False)]), "tile %s + D" % (tile,)
        check(outs[(0, True)].cpu().numpy(), ref, dtype, "walk %s %s tile %s" % (dtype, case, tile))
        check((outs[(0, False)] - d_add).cpu().numpy(), ref, dtype, "walk + D %s %s tile %s" % (dtype, case, tile))
    assert walked == 2


@pytest.mark.parametrize("layout", ["nhwc", "hwnc"])
def test_conv_tile_walk_channel_innermost(gpu, layout):
    """walking workgroups with vector stores of four output channels"""
    import torch
    from amos_amd import _lib, ops
    N, C, H, W, K, R, S = 16, 128, 41, 41, 72, 3, 3
    rng = np.random.default_rng(12)
    x = make_operand(rng, (N, C, 1, H, W), "float16", "normal")
    w = make_operand(rng, (K, C, 1, R, S), "float16", "normal")
    ref = co.lib_conv3d(x, w, "float16", (1, 1, 1), (0, 1, 1), (1, 1, 1), acc="float64")[:, :, 0]
    to_x = (0, 2, 3, 1) if layout == "nhwc" else (2, 3, 0, 1)
    dx = to_device(np.ascontiguousarray(np.transpose(x[:, :, 0], to_x)), "float16")
    dw = to_device(np.ascontiguousarray(np.transpose(w[:, :, 0], (2, 3, 1, 0))), "float16")
    refs = np.transpose(ref, to_x)
    d_add = torch.randn(refs.shape, device="cuda")
    desc = ops.conv_desc((N, C, 1, H, W), (K, C, 1, R, S), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1), 1, layout)
    for tile in [(64, 128), (128, 64)]:
        outs = {}
        for flags in (0, _lib.AMOS_FLAG_NO_TILE_WALK):
            cfg = dict(tile_i=tile[0], tile_j=tile[1], split_k=1, pipeline=_lib.AMOS_PIPE_PATCH8, flags=flags)
            assert ("walk" in ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, cfg)) == (flags == 0)
            for add in (None, d_add):
                outs[(flags, add is None)] = ops.conv2d(dx, dw, 1, 1, 1, config=cfg, add=add, layout=layout)
        assert torch.equal(outs[(0, True)], outs[(_lib.AMOS_FLAG_NO_TILE_WALK, True)])
        assert torch.equal(outs[(0, False)], outs[(_lib.AMOS_FLAG_NO_TILE_WALK, False)])
        check(outs[(0, True)].cpu().numpy(), refs, "float16", "walk %s tile %s" % (layout, tile))
        check((outs[(0, False)] - d_add).cpu().numpy(), refs, "float16", "walk + D %s tile %s" % (layout, tile))


@pytest.mark.parametrize("layout", ["nchw", "nhwc", "hwnc"])
@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("case", [(3, 64, 1, 9, 8, 40), (2, 24, 1, 7, 5, 33), (2, 128, 3, 6, 4, 72)])
def test_pointwise_conv_runs_as_gemm(gpu, layout, dtype, case):
    """1x1(x1) windows, unit stride, no padding: the (batched) GEMM kernels, no im2col gather"""
    import torch
    from amos_amd import _lib, ops
    N, C, D, H, W, K = case
    rng = np.random.default_rng(21)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, 1, 1, 1), dtype, "normal")
    ref = co.lib_conv3d(x, w, dtype, (1, 1, 1), (0, 0, 0), (1, 1, 1), acc="float64")
    to_x = {"nchw": (0, 1, 2, 3, 4), "nhwc": (0, 2, 3, 4, 1), "hwnc": (2, 3, 4, 0, 1)}[layout]
    xs = np.ascontiguousarray(np.transpose(x, to_x))
    ws_ = np.ascontiguousarray(w if layout == "nchw" else np.transpose(w, (2, 3, 4, 1, 0)))
    refs = np.ascontiguousarray(np.transpose(ref, to_x))
    lay3 = {"nchw": "ncdhw", "nhwc": "ndhwc", "hwnc": "dhwnc"}[layout]
    desc = ops.conv_desc((N, C, D, H, W), (K, C, 1, 1, 1), to_device(xs, dtype).dtype, (1, 1, 1), (0, 0, 0), (1, 1, 1),
                         1, lay3)
    name = ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, None)
    assert "im2col" not in name and "conv_fprop" not in name, name
    d_add = torch.randn(refs.shape, device="cuda").to(torch.int32 if dtype == "int8" else torch.float32)
    dx, dw = to_device(xs, dtype), to_device(ws_, dtype)
    for cfg in (None, dict(tile_i=64, tile_j=64, split_k=2), dict(tile_i=128, tile_j=128, split_k=1)):
        for add in (None, d_add):
            got = ops.conv3d(dx, dw, 1, 0, 1, config=cfg, add=add, layout=lay3)
            assert tuple(got.shape) == refs.shape
            check((got if add is None else got - add).cpu().numpy(), refs, dtype,
                  "pointwise %s %s %s cfg %s add %s" % (layout, dtype, case, cfg, add is not None))


# (channel-innermost operands are padded in whole 16-byte chunks only: no int8 C=104 in nhwc)
@pytest.mark.parametrize("dtype,C,layout", [(d, c, l) for d, c in [("float16", 96), ("float16", 40), ("bfloat16", 72),
                                                                    ("int8", 64), ("int8", 104)]
                                            for l in ("nchw", "nhwc") if not (l == "nhwc" and c == 104)])
def test_conv_padded_channels(gpu, dtype, C, layout):
    """channel counts that do not fill whole 128-byte K steps: the relayout launch zero-fills the
    rest, the patch-staged kernels run on the padded operands"""
    import torch
    from amos_amd import _lib, ops
    N, H, W, K, R, S = 3, 13, 11, 72, 3, 3
    rng = np.random.default_rng(51 + C)
    x = make_operand(rng, (N, C, 1, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, 1, R, S), dtype, "normal")
    ref = co.lib_conv3d(x, w, dtype, (1, 1, 1), (0, 1, 1), (1, 1, 1), acc="float64")[:, :, 0]
    if layout == "nhwc":
        xs, ws_, refs = np.transpose(x[:, :, 0], (0, 2, 3, 1)), np.transpose(w[:, :, 0], (2, 3, 1, 0)), np.transpose(ref, (0, 2, 3, 1))
    else:
        xs, ws_, refs = x[:, :, 0], w[:, :, 0], ref
    dx, dw = to_device(np.ascontiguousarray(xs), dtype), to_device(np.ascontiguousarray(ws_), dtype)
    desc = ops.conv_desc((N, C, 1, H, W), (K, C, 1, R, S), dx.dtype, (1, 1, 1), (0, 1, 1), (1, 1, 1), 1, layout)
    assert "amos_conv_fprop" in ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, None)
    ran = 0
    for pipe in (None, _lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8, _lib.AMOS_PIPE_STAGED):
        for tile, split in [((128, 128), 1), ((128, 64), 1), ((64, 128), 2)]:
            cfg = None if pipe is None else dict(tile_i=tile[0], tile_j=tile[1], split_k=split, pipeline=pipe)
            got = ops.conv2d(dx, dw, 1, 1, 1, config=cfg, layout=layout)
            check(got.cpu().numpy(), np.ascontiguousarray(refs), dtype,
                  "padded channels %s C=%d %s pipeline %s tile %s split %d" % (dtype, C, layout, pipe, tile, split))
            ran += 1
            if pipe is None:
                break
    assert ran == 10


LAYOUT_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil
    (3, 24, 1, 9, 7, 40, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1)),      # register-staged kernel only
    (2, 128, 1, 12, 10, 72, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1)),   # patch-staged applies
    (2, 128, 1, 9, 11, 64, 1, 3, 2, (1, 2, 1), (0, 1, 0), (1, 1, 2)),    # stride, dilation
    (2, 128, 4, 6, 6, 24, 3, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1)),     # conv3d
]


@pytest.mark.parametrize("layout", ["nhwc", "hwnc"])
@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("case", LAYOUT_CASES)
def test_conv_layouts(gpu, layout, dtype, case):
    """channel-innermost layouts (NHWC / RSCK / NPQK and HWNC / RSCK / PQNK, their 3-d forms):
    every pipeline against the oracle evaluated on the same tensors in NCDHW order"""
    import torch
    from amos_amd import _lib, ops
    N, C, D, H, W, K, T, R, S, st, pd, dl = case
    rng = np.random.default_rng(3)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, T, R, S), dtype, "normal")
    ref = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64")            # N K OD OP OQ
    is2d = D == 1 and T == 1
    to_x = (0, 2, 3, 4, 1) if layout == "nhwc" else (2, 3, 4, 0, 1)
    xs = np.ascontiguousarray(np.transpose(x, to_x))
    ws_ = np.ascontiguousarray(np.transpose(w, (2, 3, 4, 1, 0)))          # T R S C K
    refs = np.ascontiguousarray(np.transpose(ref, to_x))
    if is2d:
        xs, ws_, refs = (xs[:, 0], ws_[0], refs[:, 0]) if layout == "nhwc" else (xs[0], ws_[0], refs[0])
    dx, dw = to_device(np.ascontiguousarray(xs), dtype), to_device(np.ascontiguousarray(ws_), dtype)
    d_add = torch.randn(refs.shape, device="cuda").to(torch.int32 if dtype == "int8" else torch.float32)
    ran = set()
    for pipe in (None, _lib.AMOS_PIPE_STAGED, _lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8):
        for tile, split in [((64, 64), 1), ((128, 64), 2), ((64, 128), 1)]:
            cfg = None if pipe is None else dict(tile_i=tile[0], tile_j=tile[1], split_k=split, pipeline=pipe)
            for add in (None, d_add):
                try:
                    if is2d:
                        got = ops.conv2d(dx, dw, st[1:], pd[1:], dl[1:], config=cfg, add=add, layout=layout)
                    else:
                        got = ops.conv3d(dx, dw, st, pd, dl, config=cfg, add=add,
                                         layout="ndhwc" if layout == "nhwc" else "dhwnc")
                except _lib.AmosError as e:
                    assert pipe in (_lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8) and "not applicable" in str(e)
                    continue
                ran.add(pipe)
                assert tuple(got.shape) == refs.shape
                if add is not None:
                    got = got - add
                check(got.cpu().numpy(), refs, dtype, "%s %s %s pipeline %s tile %s split %d add %s"
                      % (layout, dtype, case, pipe, tile, split, add is not None))
            if pipe is None:
                break
    assert None in ran and _lib.AMOS_PIPE_STAGED in ran
    if C * (1 if dtype == "int8" else 2) % 128 == 0:
        assert _lib.AMOS_PIPE_PATCH in ran or _lib.AMOS_PIPE_PATCH8 in ran


def test_conv_defaults_when_applicable(gpu):
    """the kernel that reads the activations as they are for the 3x3 benchmark shapes (the int8 one
    with 128-row workgroups: one round of the compute units, as measured and as the planner's model
    says), the register-staged one where neither it nor the patch-staged kernel applies"""
    import torch
    from amos_amd import _lib, ops
    d = ops.conv_desc((32, 256, 1, 14, 14), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, d).startswith("amos_conv_nchw<f16,64x128,")
    d = ops.conv_desc((8, 64, 16, 56, 56), (64, 64, 3, 3, 3), torch.float16, (1, 1, 1), (1, 1, 1), (1, 1, 1))
    assert ops.kernel_name(_lib.AMOS_OP_CONV3D, d).startswith("amos_conv_nchw<f16,64x256,")
    d = ops.conv_desc((64, 128, 1, 28, 28), (128, 128, 1, 3, 3), torch.int8, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, d) == "amos_conv_nchw<i8,2x64x256,8+4w,kcrs>"
    d = ops.conv_desc((2, 24, 1, 14, 14), (40, 24, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, d).startswith("amos_igemm<f16,")


def test_conv_default_with_odd_addresses(gpu):
    """tensors that start 2 bytes past an aligned address (views into larger buffers): the default
    config must pick a kernel that takes them, not the one whose loads want 8-byte alignment"""
    import torch
    from amos_amd import ops
    rng = np.random.default_rng(5)
    xs, ws = (4, 64, 14, 14), (64, 64, 3, 3)
    x, w = make_operand(rng, xs, "float16"), make_operand(rng, ws, "float16")
    ref = co.lib_conv2d(x, w, "float16", 1, 1, 1, acc="float64")
    bx = torch.zeros(x.size + 8, dtype=torch.float16, device="cuda")
    bw = torch.zeros(w.size + 8, dtype=torch.float16, device="cuda")
    for sx, sw in ((1, 0), (0, 1), (1, 1), (4, 4)):
        dx = bx[sx:sx + x.size].view(xs)
        dw = bw[sw:sw + w.size].view(ws)
        dx.copy_(to_device(x, "float16"))
        dw.copy_(to_device(w, "float16"))
        print("odd addresses", sx, sw, flush=True)
        got = ops.conv2d(dx, dw, 1, 1, 1).cpu().numpy()
        check_float(got, ref, "default conv2d, x + %d B, w + %d B" % (2 * sx, 2 * sw))


def test_conv2d_config3(gpu):
    """fp16 conv2d N32 C256 14x14 K256 3x3 s1 p1; X ~ U[0,1], W ~ N(0, 0.05)"""
    from amos_amd import ops
    rng = np.random.default_rng(0)
    x = rng.uniform(0, 1, size=(32, 256, 14, 14)).astype(np.float32).astype(np.float16)
    w = (rng.standard_normal(size=(256, 256, 3, 3)) * 0.05).astype(np.float32).astype(np.float16)
    got = ops.conv2d(to_device(x, "float16"), to_device(w, "float16"), 1, 1, 1).cpu().numpy()
    check_float(got, co.lib_conv2d(x, w, "float16", 1, 1, 1, acc="float32"), "C3 vs fp32")
    lit = co.te_literal_conv2d(x, w, "float16", 1, 1, 1, images=(0, 2), threads=8)
    check_literal(got[:2], lit[:2], "float16", "C3 vs te_literal (2 images)", MEAN_REL)


def test_conv2d_config4_int8(gpu):
    """int8 conv2d N64 C128 28x28 K128 3x3 s1 p1: bit-exact on the whole tensor"""
    from amos_amd import ops
    rng = np.random.default_rng(0)
    x = rng.integers(-128, 128, size=(64, 128, 28, 28)).astype(np.int8)
    w = rng.integers(-64, 64, size=(128, 128, 3, 3)).astype(np.int8)
    got = ops.conv2d(to_device(x, "int8"), to_device(w, "int8"), 1, 1, 1).cpu().numpy()
    ref = co.lib_conv2d(x, w, "int8", 1, 1, 1)
    assert got.dtype == np.int32 and np.array_equal(got, ref)
    lit = co.te_literal_conv2d(x, w, "int8", 1, 1, 1, mode="exact", images=(0, 1), threads=8)
    assert np.array_equal(got[:1], lit[:1])


CONV3D_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil
    (1, 8, 4, 6, 6, 8, 3, 3, 3, 1, 1, 1),
    (2, 5, 5, 7, 9, 12, 3, 2, 3, (1, 2, 1), (1, 0, 2), (1, 1, 2)),
    (1, 16, 6, 6, 6, 16, 1, 1, 1, 1, 0, 1),
    (1, 4, 8, 8, 8, 8, 2, 2, 2, 2, 0, 1),
]


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("case", CONV3D_CASES)
def test_conv3d_small(gpu, dtype, case):
    from amos_amd import ops
    N, C, D, H, W, K, T, R, S, st, pd, dl = case
    rng = np.random.default_rng(5)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, C, T, R, S), dtype, "normal")
    got = ops.conv3d(to_device(x, dtype), to_device(w, dtype), st, pd, dl).cpu().numpy()
    check(got, co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64"), dtype, "conv3d %s" % (case,))
    lit = co.te_literal_conv3d(x, w, dtype, st, pd, dl, mode="exact" if dtype == "int8" else "te_literal")
    check_literal(got, lit, dtype, "conv3d te_literal %s" % (case,))


def test_conv3d_config5b(gpu):
    """fp16 conv3d N8 C64 D16 56x56 K64 3x3x3 s1 p1, N(0,1): one image against the library
    form, plus the batch-shift property (image n of the batched call == the same image alone)."""
    import torch
    from amos_amd import ops
    rng = np.random.default_rng(0)
    x = make_operand(rng, (8, 64, 16, 56, 56), "float16", "normal")
    w = make_operand(rng, (64, 64, 3, 3, 3), "float16", "normal")
    dx, dw = to_device(x, "float16"), to_device(w, "float16")
    got = ops.conv3d(dx, dw, 1, 1, 1)
    ref0 = co.lib_conv3d(x[5:6], w, "float16", 1, 1, 1, acc="float32")
    check_float(got[5:6].cpu().numpy(), ref0, "C5b image 5 vs fp32")
    # same tiling and no split-K => the same accumulation order => bitwise equal
    cfg = dict(tile_i=64, tile_j=128, split_k=1)
    full = ops.conv3d(dx, dw, 1, 1, 1, config=cfg)
    alone = ops.conv3d(dx[2:3].contiguous(), dw, 1, 1, 1, config=cfg)
    assert torch.equal(alone[0], full[2])
    check_float(full[5:6].cpu().numpy(), ref0, "C5b image 5 vs fp32 (64x128)")


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("case", [(20, 256, 30, 30, 512, (2, 2)), (24, 200, 41, 37, 520, (2, 3)), (24, 512, 14, 27, 256, (1, 2))])
def test_strided_pointwise_conv_runs_as_gemm(gpu, dtype, case):
    """a 1x1 window with a stride (ResNet's down-sampling shortcuts): the copy that makes the
    activations K-contiguous picks every stride-th pixel, the direct-to-LDS GEMM does the rest;
    against the oracle, against the implicit GEMM of the same op (bit for bit for int8), and
    without a workspace (the implicit GEMM again)"""
    import torch
    from amos_amd import _lib, ops
    N, C, H, W, K, st = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, H, W), dtype)
    w = make_operand(rng, (K, C, 1, 1), dtype)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    desc = ops.conv_desc((N, C, 1, H, W), (K, C, 1, 1, 1), dx.dtype, (1,) + st, (0, 0, 0), (1, 1, 1))
    name = ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, None)
    assert name.startswith("amos_gemm_tn<") or ",vec,vec," in name, name     # a GEMM on K-contiguous copies
    assert ops.workspace_bytes(_lib.AMOS_OP_CONV2D, desc) > 0
    cfg = ops.default_config(_lib.AMOS_OP_CONV2D, desc)
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, cfg) == ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, None)
    got = ops.conv2d(dx, dw, st, 0, 1).cpu().numpy()
    ref = co.lib_conv2d(x, w, dtype, st, 0, 1, acc="float64")
    check(got, ref, dtype, "strided pointwise %s %s" % (dtype, case))
    staged = dict(tile_i=64, tile_j=64, split_k=1, pipeline=1)
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, staged).startswith("amos_igemm<")
    other = ops.conv2d(dx, dw, st, 0, 1, config=staged).cpu().numpy()
    check(other, ref, dtype, "strided pointwise, implicit GEMM %s %s" % (dtype, case))
    if dtype == "int8":
        assert np.array_equal(got, other)
    # no workspace: the same call through the C ABI falls back to the implicit GEMM
    out = torch.empty(got.shape, dtype=torch.from_numpy(got).dtype, device="cuda")
    rc = _lib.load().amos_conv2d(ctypes.byref(desc), None, dx.data_ptr(), dw.data_ptr(), out.data_ptr(), None, 0, None)
    assert rc == 0
    check(out.cpu().numpy(), ref, dtype, "strided pointwise, no workspace %s %s" % (dtype, case))


IM2COL_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil
    (2, 17, 1, 64, 60, 256, 1, 7, 7, (1, 2, 2), (0, 3, 3), (1, 1, 1)),    # a wide 7x7 on 17 channels
    (3, 24, 1, 113, 97, 264, 1, 3, 3, (1, 2, 2), (0, 1, 1), (1, 1, 1)),   # 3x3 on 24 channels, ragged everything
    (4, 20, 1, 30, 31, 300, 1, 5, 3, (1, 1, 2), (0, 2, 0), (1, 2, 1)),    # 20 channels, dilated, uneven
    (4, 5, 6, 20, 18, 256, 3, 3, 3, (1, 2, 1), (1, 0, 1), (1, 1, 1)),     # 3-D
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", IM2COL_CASES)
def test_conv_through_im2col_copy(gpu, dtype, case):
    """a convolution on few channels: im2col copy + zero-padded weights in the workspace, then the
    GEMM kernels; against the oracle, against the on-the-fly im2col of the same op (bit for bit
    for int8), and without a workspace"""
    import torch
    from amos_amd import _lib, ops
    N, C, D, H, W, K, T, R, S, st, pd, dl = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, D, H, W), dtype)
    w = make_operand(rng, (K, C, T, R, S), dtype)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    desc = ops.conv_desc((N, C, D, H, W), (K, C, T, R, S), dx.dtype, st, pd, dl)
    assert ops.workspace_bytes(_lib.AMOS_OP_CONV3D, desc) > 0
    name = ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, None)
    assert name.startswith("amos_gemm_tn<") or ",vec,vec," in name, name
    cfg = ops.default_config(_lib.AMOS_OP_CONV3D, desc)
    assert ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, cfg) == name
    ref = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64")
    got = ops.conv3d(dx, dw, st, pd, dl).cpu().numpy()
    check(got, ref, dtype, "im2col copy %s %s" % (dtype, case))
    # a staged tile on the copies, split-K
    got2 = ops.conv3d(dx, dw, st, pd, dl, config=dict(tile_i=64, tile_j=64, split_k=2, pipeline=0)).cpu().numpy()
    check(got2, ref, dtype, "im2col copy, 64x64 split 2 %s %s" % (dtype, case))
    staged = dict(tile_i=64, tile_j=64, split_k=1, pipeline=1)
    assert ",im2col," in ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, staged)
    other = ops.conv3d(dx, dw, st, pd, dl, config=staged).cpu().numpy()
    check(other, ref, dtype, "on-the-fly im2col %s %s" % (dtype, case))
    if dtype == "int8":
        assert np.array_equal(got, other) and np.array_equal(got2, other)
    out = torch.empty(got.shape, dtype=torch.from_numpy(got).dtype, device="cuda")
    rc = _lib.load().amos_conv3d(ctypes.byref(desc), None, dx.data_ptr(), dw.data_ptr(), out.data_ptr(), None, 0, None)
    assert rc == 0
    check(out.cpu().numpy(), ref, dtype, "few channels, no workspace %s %s" % (dtype, case))


FEW_CHANNEL_CASES = [
    # N, C, H, W, K, R, S, stride, pad, dil
    (6, 3, 64, 60, 64, 7, 7, (2, 2), (3, 3), (1, 1)),       # ResNet's stem, small
    (8, 3, 113, 97, 100, 3, 3, (2, 2), (1, 1), (1, 1)),     # MobileNet's, ragged output channels
    (16, 8, 30, 31, 72, 5, 3, (1, 2), (2, 0), (2, 1)),      # a full pixel of channels, dilated, uneven
    (3, 1, 50, 300, 130, 3, 3, (1, 1), (1, 1), (1, 1)),     # one channel, wide rows
    (60, 4, 40, 37, 65, 2, 4, (3, 1), (0, 2), (1, 2)),      # even taps, 65 output channels
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", FEW_CHANNEL_CASES)
def test_conv_few_channels(gpu, dtype, case):
    """convolutions whose input channels fit one 16-byte pixel (the networks' stems) on
    amos_conv_few_channels: against the oracle, against the implicit GEMM of the same op (bit for
    bit for int8), with a fused addition, and without a workspace"""
    import torch
    from amos_amd import _lib, ops
    N, C, H, W, K, R, S, st, pd, dl = case
    if dtype == "int8":
        C = C * 2          # sixteen int8 channels fill a pixel
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, H, W), dtype)
    w = make_operand(rng, (K, C, R, S), dtype)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    desc = ops.conv_desc((N, C, 1, H, W), (K, C, 1, R, S), dx.dtype, (1,) + st, (0,) + pd, (1,) + dl)
    name = ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, None)
    assert name.startswith("amos_conv_few_channels<"), name
    cfg = ops.default_config(_lib.AMOS_OP_CONV2D, desc)
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, cfg) == name and ops.workspace_bytes(_lib.AMOS_OP_CONV2D, desc) > 0
    ref = co.lib_conv2d(x, w, dtype, st, pd, dl, acc="float64")
    got = ops.conv2d(dx, dw, st, pd, dl).cpu().numpy()
    check(got, ref, dtype, "few channels %s %s" % (dtype, case))
    staged = dict(tile_i=64, tile_j=64, split_k=1, pipeline=1)
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, staged).startswith("amos_igemm<")
    other = ops.conv2d(dx, dw, st, pd, dl, config=staged).cpu().numpy()
    if dtype == "int8":
        assert np.array_equal(got, other)
    else:
        check_float(got, other, "few channels vs implicit GEMM %s %s" % (dtype, case))
    # fused addition of a tensor of the output's shape
    d_host = rng.integers(-1000, 1000, got.shape).astype(got.dtype)
    with_d = ops.conv2d(dx, dw, st, pd, dl, add=torch.from_numpy(d_host).cuda()).cpu().numpy()
    want = (ref.astype(np.int64) + d_host).astype(np.int32) if dtype == "int8" else ref + d_host
    check(with_d, want, dtype, "few channels + D %s %s" % (dtype, case))
    out = torch.empty(got.shape, dtype=torch.from_numpy(got).dtype, device="cuda")
    rc = _lib.load().amos_conv2d(ctypes.byref(desc), None, dx.data_ptr(), dw.data_ptr(), out.data_ptr(), None, 0, None)
    assert rc == 0
    check(out.cpu().numpy(), ref, dtype, "few channels, no workspace %s %s" % (dtype, case))


def _random_route_cases():
    """seeded random int8 convolutions aimed at the routes beside the patch-staged and the
    register-staged kernels: few input channels, strided 1x1, depthwise, im2col copy"""
    rng = np.random.default_rng(20240607)
    cases = []
    for _ in range(10):     # few channels
        R, S = int(rng.integers(1, 8)), int(rng.integers(2, 8))
        cases.append(("few", int(rng.integers(3, 12)), int(rng.integers(1, 17)), int(rng.integers(24, 90)),
                      int(rng.integers(24, 130)), int(rng.integers(33, 140)), R, S,
                      (int(rng.integers(1, 4)), int(rng.integers(1, 4))), (int(rng.integers(0, R)), int(rng.integers(0, S))),
                      (int(rng.integers(1, 3)), int(rng.integers(1, 3))), 1))
    for _ in range(8):      # strided 1x1
        cases.append(("sub", int(rng.integers(6, 20)), int(rng.integers(40, 300)), int(rng.integers(14, 40)),
                      int(rng.integers(14, 40)), int(rng.integers(100, 400)), 1, 1,
                      (int(rng.integers(1, 4)), int(rng.integers(2, 4))), (0, 0), (1, 1), 1))
    for _ in range(10):     # depthwise, with and without a channel multiplier
        C = int(rng.integers(3, 70))
        R, S = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        cases.append(("dw", int(rng.integers(1, 5)), C, int(rng.integers(5, 60)), int(rng.integers(5, 60)),
                      C * int(rng.integers(1, 4)), R, S, (int(rng.integers(1, 4)), int(rng.integers(1, 4))),
                      (int(rng.integers(0, R + 1)), int(rng.integers(0, S + 1))),
                      (int(rng.integers(1, 3)), int(rng.integers(1, 3))), C))
    for _ in range(6):      # more than a pixel of channels, no 128-byte chunk, wide output
        cases.append(("col", int(rng.integers(2, 6)), int(rng.integers(17, 60)), int(rng.integers(12, 40)),
                      int(rng.integers(12, 40)), int(rng.integers(256, 400)), int(rng.integers(1, 5)), int(rng.integers(2, 5)),
                      (int(rng.integers(1, 3)), int(rng.integers(1, 3))), (int(rng.integers(0, 2)), int(rng.integers(0, 2))),
                      (1, 1), 1))
    return cases


@pytest.mark.parametrize("case", _random_route_cases())
def test_conv_routes_random_int8(gpu, case):
    """whatever kernel the default picks against the register-staged implicit GEMM of the same
    convolution: int8, so the two must agree bit for bit; a quarter of the cases also against the
    oracle"""
    from amos_amd import _lib, ops
    kind, N, C, H, W, K, R, S, st, pd, dl, G = case
    if (H + 2 * pd[0] - ((R - 1) * dl[0] + 1)) < 0 or (W + 2 * pd[1] - ((S - 1) * dl[1] + 1)) < 0:
        pytest.skip("window larger than the padded input")
    rng = np.random.default_rng(hash(case) % 2**32)
    x = make_operand(rng, (N, C, H, W), "int8")
    w = make_operand(rng, (K, C // G, R, S), "int8")
    dx, dw = to_device(x, "int8"), to_device(w, "int8")
    got = ops.conv2d(dx, dw, st, pd, dl, groups=G).cpu().numpy()
    other = ops.conv2d(dx, dw, st, pd, dl, groups=G, config=dict(tile_i=64, tile_j=64, split_k=1, pipeline=1)).cpu().numpy()
    desc = ops.conv_desc((N, C, 1, H, W), (K, C // G, 1, R, S), dx.dtype, (1,) + st, (0,) + pd, (1,) + dl, G)
    name = ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, None)
    assert np.array_equal(got, other), (name, case)
    if hash(case) % 4 == 0 and G == 1:
        assert np.array_equal(got, co.lib_conv2d(x, w, "int8", st, pd, dl)), (name, case)


def test_conv_few_channels_single_patch_buffer(gpu):
    """rows so wide that two patch buffers do not fit LDS: the kernel refills its one buffer
    between tiles"""
    from amos_amd import _lib, ops
    N, C, H, W, K = 2, 3, 20, 1198, 64
    rng = np.random.default_rng(5)
    x = make_operand(rng, (N, C, H, W), "int8")
    w = make_operand(rng, (K, C, 3, 3), "int8")
    dx, dw = to_device(x, "int8"), to_device(w, "int8")
    desc = ops.conv_desc((N, C, 1, H, W), (K, C, 1, 3, 3), dx.dtype, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    assert ops.kernel_name(_lib.AMOS_OP_CONV2D, desc, None) == "amos_conv_few_channels<i8>"
    got = ops.conv2d(dx, dw, 1, 1, 1).cpu().numpy()
    assert np.array_equal(got, co.lib_conv2d(x, w, "int8", 1, 1, 1))


DEPTHWISE_CASES = [
    # N, C, D, H, W, mult, T, R, S, stride, pad, dil, kernel-name suffix
    (2, 32, 1, 28, 28, 1, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), ",3x3>"),       # MobileNet's 3x3
    (3, 24, 1, 29, 31, 1, 1, 3, 3, (1, 2, 2), (0, 1, 1), (1, 1, 1), ",3x3/2>"),     # strided, ragged rows
    (1, 16, 1, 7, 7, 2, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), ",3x3>"),         # two outputs per channel
    (2, 8, 1, 20, 18, 1, 1, 5, 5, (1, 2, 1), (0, 2, 2), (1, 1, 1), ">"),            # 5x5
    (2, 8, 1, 17, 19, 3, 1, 3, 3, (1, 1, 1), (0, 2, 2), (1, 2, 2), ">"),            # dilated
    (2, 6, 5, 9, 12, 1, 3, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1), ",3x3>"),         # 3-D
    (1, 5, 4, 6, 10, 2, 2, 2, 3, (2, 1, 2), (1, 0, 1), (1, 2, 1), ">"),             # 3-D, uneven everything
    (1, 4, 1, 1, 3, 1, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1), ",3x3>"),          # one output row of 3
]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", DEPTHWISE_CASES)
def test_depthwise_conv(gpu, dtype, case):
    """depthwise convolution (reference compute: benchmark/amos/mapping_depthwiseconv2d_tensorcore.py:7-48)
    on the vector-ALU kernel: against the oracle run once per channel, and against the
    register-staged implicit GEMM of the same op (bit for bit for int8)"""
    from amos_amd import _lib, ops
    N, C, D, H, W, mult, T, R, S, st, pd, dl, suffix = case
    K = C * mult
    rng = np.random.default_rng(hash(case[:-1]) % 2**32)
    x = make_operand(rng, (N, C, D, H, W), dtype, "normal")
    w = make_operand(rng, (K, 1, T, R, S), dtype, "normal")
    ref = np.concatenate([co.lib_conv3d(np.ascontiguousarray(x[:, c:c + 1]),
                                        np.ascontiguousarray(w[c * mult:(c + 1) * mult]), dtype, st, pd, dl,
                                        acc="float64") for c in range(C)], axis=1)
    dx, dw = to_device(x, dtype), to_device(w, dtype)
    desc = ops.conv_desc((N, C, D, H, W), (K, 1, T, R, S), dx.dtype, st, pd, dl, C)
    name = ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, None)
    assert name.startswith("amos_depthwise_conv<") and name.endswith(suffix), name
    got = ops.conv3d(dx, dw, st, pd, dl, groups=C).cpu().numpy()
    check(got, ref, dtype, "depthwise %s %s" % (dtype, case))
    staged = dict(tile_i=64, tile_j=64, split_k=1, pipeline=1)
    assert ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, staged).startswith("amos_igemm<")
    other = ops.conv3d(dx, dw, st, pd, dl, groups=C, config=staged).cpu().numpy()
    if dtype == "int8":
        assert np.array_equal(got, other)
    else:
        check_float(got, other, "depthwise vs implicit GEMM %s %s" % (dtype, case))
    # the default configuration named explicitly is the same launch
    cfg = ops.default_config(_lib.AMOS_OP_CONV3D, desc)
    assert cfg.pipeline == 0 and ops.kernel_name(_lib.AMOS_OP_CONV3D, desc, cfg) == name
    # a misaligned output takes element stores
    flat = np.zeros(got.size + 1, dtype=got.dtype)
    import torch
    buf = torch.from_numpy(flat).cuda()
    out = buf[1:].view(got.shape)
    ops.conv3d(dx, dw, st, pd, dl, groups=C, out=out)
    assert np.array_equal(out.cpu().numpy(), got) and int(buf[0]) == 0


def test_errors(gpu):
    import torch
    from amos_amd import _lib, ops
    a = torch.zeros((8, 8), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.AmosError) as e:
        ops.gemm(a, a, config=dict(tile_i=96, tile_j=64, split_k=1))
    assert e.value.code == _lib.AMOS_ERR_INFEASIBLE
    with pytest.raises(RuntimeError):
        ops.gemm(a.cpu(), a.cpu())


def test_time_evaluator(gpu):
    import torch
    from amos_amd import _lib, ops
    a = torch.randn((512, 512), device="cuda").half()
    out = torch.empty((512, 512), device="cuda")
    d = ops.gemm_desc(512, 512, 512, torch.float16)
    res = ops.time_op(_lib.AMOS_OP_GEMM, d, a, a, out, number=10, repeat=3, min_repeat_ms=5)
    assert len(res) == 3 and all(0 < r < 1e-2 for r in res)
