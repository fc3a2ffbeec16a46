"""The C-ABI library loads and exports what include/amos_mi355x.h declares; host-side
validation, resource check and mapper defaults (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from amos_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "amos_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(amos_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    lib = _lib.load()
    names = header_functions()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), "libamos_mi355x.so does not export %s" % n
    assert sorted(_lib.EXPORTS) == names
    assert lib.amos_version() == 2


def test_struct_sizes_match_header():
    assert ctypes.sizeof(_lib.GemmDesc) == 3 * 8 + 4 * 4 + 3 * 8
    assert ctypes.sizeof(_lib.BGemmDesc) == 8 + ctypes.sizeof(_lib.GemmDesc) + 3 * 8
    assert ctypes.sizeof(_lib.ConvDesc) == 9 * 8 + 13 * 4 + 4 and _lib.ConvDesc.groups.offset == 9 * 8 + 11 * 4
    assert ctypes.sizeof(_lib.Epilogue) == 32 and _lib.Epilogue.operand.offset == 8
    assert ctypes.sizeof(_lib.KernelConfig) == 32
    assert _lib.KernelConfig.pipeline.offset == 12


def gemm_desc(M, N, K, ind=_lib.AMOS_F16, outd=_lib.AMOS_F32, ta=0, tb=0):
    d = _lib.GemmDesc()
    d.M, d.N, d.K, d.in_dtype, d.out_dtype, d.trans_a, d.trans_b = M, N, K, ind, outd, ta, tb
    d.lda, d.ldb, d.ldc = (M if ta else K), (K if tb else N), N
    return d


def test_bad_arguments_are_reported():
    lib = _lib.load()
    d = gemm_desc(16, 16, 16)
    buf = ctypes.create_string_buffer(64)
    rc = lib.amos_gemm(ctypes.byref(d), None, None, buf, buf, None, 0, None)
    assert rc == _lib.AMOS_ERR_BAD_ARG and b"null" in lib.amos_last_error()
    d2 = gemm_desc(0, 16, 16)
    assert lib.amos_gemm(ctypes.byref(d2), None, buf, buf, buf, None, 0, None) == _lib.AMOS_ERR_BAD_ARG
    d3 = gemm_desc(16, 16, 16, _lib.AMOS_F16, _lib.AMOS_I32)
    assert lib.amos_gemm(ctypes.byref(d3), None, buf, buf, buf, None, 0, None) == _lib.AMOS_ERR_UNSUPPORTED
    d4 = gemm_desc(16, 16, 16)
    d4.lda = 8
    assert lib.amos_gemm(ctypes.byref(d4), None, buf, buf, buf, None, 0, None) == _lib.AMOS_ERR_BAD_ARG
    with pytest.raises(_lib.AmosError):
        _lib.check(rc)


def test_check_config_budget():
    lib = _lib.load()
    d = gemm_desc(1024, 1024, 1024)
    lds, regs = ctypes.c_int64(), ctypes.c_int64()
    cfg = _lib.KernelConfig(256, 256, 1)
    assert lib.amos_check_config(0, ctypes.byref(d), ctypes.byref(cfg), ctypes.byref(lds), ctypes.byref(regs)) == 0
    assert lds.value == 2 * (256 + 256) * 128 + 2048 and lds.value <= 160 * 1024 and regs.value == 256
    bad = _lib.KernelConfig(96, 64, 1)
    assert lib.amos_check_config(0, ctypes.byref(d), ctypes.byref(bad), None, None) == _lib.AMOS_ERR_INFEASIBLE


def test_check_config_and_estimate_know_the_ncdhw_direct_tiles():
    """every tile the NCDHW-direct convolution is built for passes amos_check_config and gets an
    estimate (the sweep skips what has none), the default of the benchmark's convolutions among
    them; a tile it is not built for and a shape it does not take are refused with a reason"""
    from amos_amd import ops
    import torch
    lib = _lib.load()
    c3 = ops.conv_desc((32, 256, 1, 14, 14), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    c4 = ops.conv_desc((64, 128, 1, 28, 28), (128, 128, 1, 3, 3), torch.int8, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    lds, regs, est = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_double()
    for d in (c3, c4):
        for ti, tj in [(32, 128), (32, 256), (64, 128), (64, 256), (128, 128), (128, 256)]:
            cfg = _lib.KernelConfig(ti, tj, 1, _lib.AMOS_PIPE_NCHW)
            rc = lib.amos_check_config(_lib.AMOS_OP_CONV2D, ctypes.byref(d), ctypes.byref(cfg), ctypes.byref(lds), ctypes.byref(regs))
            if rc != 0:   # (a tile whose patch does not fit: said so, not "no kernel instance")
                assert b"NCDHW-direct" in lib.amos_last_error(), lib.amos_last_error()
                continue
            rows = 64 if ti == 128 else ti
            assert lds.value == 2 * 9 * rows * 64 + 2 * (32 if tj <= 128 else 40) * 1024 and regs.value > 0
            assert lib.amos_estimate_seconds(_lib.AMOS_OP_CONV2D, ctypes.byref(d), ctypes.byref(cfg), ctypes.byref(est)) == 0
            assert 1e-6 < est.value < 1e-3
        dflt = _lib.KernelConfig()
        assert lib.amos_default_config(_lib.AMOS_OP_CONV2D, ctypes.byref(d), ctypes.byref(dflt)) == 0
        assert dflt.pipeline == _lib.AMOS_PIPE_NCHW
        assert lib.amos_check_config(_lib.AMOS_OP_CONV2D, ctypes.byref(d), ctypes.byref(dflt), None, None) == 0
    bad = _lib.KernelConfig(96, 128, 1, _lib.AMOS_PIPE_NCHW)
    assert lib.amos_check_config(_lib.AMOS_OP_CONV2D, ctypes.byref(c3), ctypes.byref(bad), None, None) == _lib.AMOS_ERR_INFEASIBLE
    five = ops.conv_desc((32, 256, 1, 14, 14), (256, 256, 1, 5, 5), torch.float16, (1, 1, 1), (0, 2, 2), (1, 1, 1))
    ok = _lib.KernelConfig(64, 128, 1, _lib.AMOS_PIPE_NCHW)
    assert lib.amos_check_config(_lib.AMOS_OP_CONV2D, ctypes.byref(five), ctypes.byref(ok), None, None) == _lib.AMOS_ERR_INFEASIBLE
    assert b"3x3" in lib.amos_last_error()
    # a pointwise convolution asked to run on this pipeline is refused too, not run as a matrix product
    one = ops.conv_desc((4, 64, 1, 14, 14), (64, 64, 1, 1, 1), torch.float16, (1, 1, 1), (0, 0, 0), (1, 1, 1))
    assert lib.amos_kernel_name(_lib.AMOS_OP_CONV2D, ctypes.byref(one), ctypes.byref(ok)) is None
    assert b"3x3" in lib.amos_last_error()


def test_default_config_is_a_compiled_instance():
    lib = _lib.load()
    cfg = _lib.KernelConfig()
    for (M, N, K) in [(8192, 8192, 8192), (512, 512, 512), (64, 64, 4096), (33, 17, 19), (100000, 64, 64)]:
        d = gemm_desc(M, N, K, tb=1)
        assert lib.amos_default_config(0, ctypes.byref(d), ctypes.byref(cfg)) == 0
        assert lib.amos_check_config(0, ctypes.byref(d), ctypes.byref(cfg), None, None) == 0
        name = lib.amos_kernel_name(0, ctypes.byref(d), ctypes.byref(cfg))
        assert name is not None and (name.startswith(b"amos_igemm<f16,") or name.startswith(b"amos_gemm_tn<f16,"))
    d = gemm_desc(8192, 8192, 8192, tb=1)
    lib.amos_default_config(0, ctypes.byref(d), ctypes.byref(cfg))
    assert (cfg.tile_i, cfg.tile_j, cfg.split_k) == (256, 256, 1)
    # aligned K-contiguous operands at 256x256 take the direct-to-LDS pipeline
    assert lib.amos_kernel_name(0, ctypes.byref(d), ctypes.byref(cfg)) == b"amos_gemm_tn<f16,256x256,8w>"
    staged = _lib.KernelConfig(256, 256, 1, _lib.AMOS_PIPE_STAGED)
    assert lib.amos_kernel_name(0, ctypes.byref(d), ctypes.byref(staged)) == b"amos_igemm<f16,vec,vec,256x256>"


def test_kernel_name_reflects_layout():
    lib = _lib.load()
    cfg = _lib.KernelConfig(128, 128, 1)
    # aligned K-contiguous operands: the direct-to-LDS kernel where it has the tile, else (or on
    # request) the register-staged one
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 256, tb=1)), ctypes.byref(cfg)) == \
        b"amos_gemm_tn<f16,128x128,8w>"
    staged = _lib.KernelConfig(128, 128, 1, _lib.AMOS_PIPE_STAGED)
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 256, tb=1)), ctypes.byref(staged)) == \
        b"amos_igemm<f16,vec,vec,128x128>"
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 256, tb=1)),
                                ctypes.byref(_lib.KernelConfig(128, 64, 1))) == b"amos_igemm<f16,vec,vec,128x64>"
    # row-major B: rows (n) contiguous, vector loads transposed in registers ...
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 256)), ctypes.byref(cfg)) == \
        b"amos_igemm<f16,vec,tvec,128x128>"
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 256, ta=1)), ctypes.byref(cfg)) == \
        b"amos_igemm<f16,tvec,tvec,128x128>"
    # ... unless N is not a multiple of 8, or the type is 8-bit: element loads
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 252, 256)), ctypes.byref(cfg)) == \
        b"amos_igemm<f16,vec,strided,128x128>"
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 256, _lib.AMOS_I8, _lib.AMOS_I32)),
                                ctypes.byref(cfg)) == b"amos_igemm<i8,vec,strided,128x128>"
    assert lib.amos_kernel_name(0, ctypes.byref(gemm_desc(256, 256, 255, tb=1)), ctypes.byref(cfg)) == \
        b"amos_igemm<f16,strided,strided,128x128>"
    c = _lib.ConvDesc()
    c.N, c.C, c.D, c.H, c.W, c.K, c.T, c.R, c.S = 2, 16, 1, 8, 8, 16, 1, 3, 3
    c.stride_d = c.stride_h = c.stride_w = 1
    c.dil_d = c.dil_h = c.dil_w = 1
    c.pad_h = c.pad_w = 1
    c.in_dtype, c.out_dtype = _lib.AMOS_I8, _lib.AMOS_I32
    assert lib.amos_kernel_name(2, ctypes.byref(c), ctypes.byref(cfg)) == b"amos_igemm<i8,vec,im2col,128x128>"
    c.R = 20   # window larger than the padded input
    assert lib.amos_kernel_name(2, ctypes.byref(c), ctypes.byref(cfg)) is None


def test_wrong_arrays_are_refused_before_any_launch():
    """The kernels take raw pointers; an `out` (or an input) of the wrong extent or element type
    must never reach them.  These checks run on host tensors: nothing is launched."""
    import torch
    from amos_amd import ops
    like = torch.empty(4, 8, dtype=torch.float16)
    ops._check_out(torch.empty(4, 6), (4, 6), torch.float32, like)
    with pytest.raises(ValueError, match="shape"):
        ops._check_out(torch.empty(4, 5), (4, 6), torch.float32, like)
    with pytest.raises(ValueError, match="float32"):
        ops._check_out(torch.empty(4, 6, dtype=torch.float16), (4, 6), torch.float32, like)
    d = ops.gemm_desc(4, 6, 8, torch.float16, False, True)
    a, b = torch.empty(4, 8, dtype=torch.float16), torch.empty(6, 8, dtype=torch.float16)
    ops.check_operands(_lib.AMOS_OP_GEMM, d, a, b, torch.empty(4, 6))
    with pytest.raises(ValueError, match="output holds 20 elements"):
        ops.check_operands(_lib.AMOS_OP_GEMM, d, a, b, torch.empty(4, 5))
    with pytest.raises(ValueError, match="output is torch.float16"):
        ops.check_operands(_lib.AMOS_OP_GEMM, d, a, b, torch.empty(4, 6, dtype=torch.float16))
    with pytest.raises(ValueError, match="second input holds"):
        ops.check_operands(_lib.AMOS_OP_GEMM, d, a, b[:5], torch.empty(4, 6))
    # leading dimensions and batch strides count
    bd = ops.bgemm_desc(3, 4, 6, 8, torch.float16, False, True)
    bd.stride_c = 100
    assert ops.operand_spans(_lib.AMOS_OP_BGEMM, bd)[0] == (3 * 32, 3 * 48, 2 * 100 + 24)
    cd = ops.conv_desc((2, 8, 1, 5, 5), (4, 8, 1, 3, 3), torch.int8, (1, 1, 1), (0, 1, 1), (1, 1, 1))
    spans, in_dt, out_dt = ops.operand_spans(_lib.AMOS_OP_CONV2D, cd)
    assert spans == (2 * 8 * 25, 4 * 8 * 9, 2 * 4 * 25) and in_dt == torch.int8 and out_dt == torch.int32
    with pytest.raises(ValueError, match="output is torch.float32"):
        ops.check_operands(_lib.AMOS_OP_CONV2D, cd, torch.empty(400, dtype=torch.int8),
                           torch.empty(288, dtype=torch.int8), torch.empty(200))


def test_module_refuses_arrays_that_are_not_the_declared_tensors():
    import torch
    from amos_amd import te
    from amos_amd.auto_tensorize import runtime
    from amos_amd.auto_tensorize.hw_abstraction import compute_dag_from_tensors
    from amos_amd.auto_tensorize.lowering import lower_main_op
    A = te.placeholder([32, 64], dtype="float16", name="A")
    B = te.placeholder([64, 48], dtype="float16", name="B")
    k = te.reduce_axis([0, 64], name="k")
    C = te.compute([32, 48], lambda i, j: te.sum((A[i, k] * B[k, j]).astype("float32"), axis=k), name="C")
    dag = compute_dag_from_tensors([C])
    lowered = lower_main_op([op for op in dag.op_lst if op.reduce_axis][0], dag)
    mod = runtime.Module(lowered, None, [A, B, C])
    a, b = torch.empty(32, 64, dtype=torch.float16), torch.empty(64, 48, dtype=torch.float16)
    with pytest.raises(ValueError, match="declared float32"):
        mod(a, b, torch.empty(32, 40))                              # short output
    with pytest.raises(ValueError, match="declared float32"):
        mod(a, b, torch.empty(32, 48, dtype=torch.float16))        # fp16 output
    with pytest.raises(ValueError, match="declared float16"):
        mod(a.float(), b, torch.empty(32, 48))                      # float32 input wrapped by array()
    with pytest.raises(ValueError, match="device array"):
        mod(a, b, torch.empty(32, 48))                              # right shapes, but host memory


@pytest.mark.parametrize("waves", [4, 8])
@pytest.mark.parametrize("I,J,K", [(8192, 8192, 8192), (8000, 8100, 4096)])
def test_gemm_tn_copy_addresses_stay_inside_operands(waves, I, J, K):
    """The direct-to-LDS GEMM's address arithmetic (gemm_tn_kernel.h: a wave copies 1 KB chunks
    q = wave + NW * u of a stage, lane l the 16 bytes (row 8 * q' + l / 8, swizzled chunk)),
    evaluated on the host for the four- and the eight-wave grid of the 256x256 tile: every byte a
    lane fetches lies inside its operand, every LDS byte it lands on inside the stage.  (The
    four-wave instance faulted on the GPU at 8192^3 and is withdrawn; its addresses are the same
    set as the eight-wave instance's, so the fault is not an index error of the source.  What
    differs: its 128x128 wave tile leaves the 256 accumulator registers in scratch memory --
    1040 bytes per lane -- and the kernel's launch code refuses instances with scratch.)"""
    ES, BI, BJ, NS = 2, 256, 256, 2
    NW, QA, CH = waves, BI // 8, (BI + BJ) // 8 // waves
    lda = ldb = K
    stage_bytes = (BI + BJ) * 128
    a_bytes, b_bytes = I * lda * ES, J * ldb * ES
    tiles_i, tiles_j = -(-I // BI), -(-J // BJ)
    seen = set()
    for tile_i, tile_j in {(0, 0), (tiles_i - 1, tiles_j - 1), (tiles_i - 1, 0), (0, tiles_j - 1)}:
        bi0, bj0 = tile_i * BI, tile_j * BJ
        for wave in range(NW):
            for u in range(CH):
                q = wave + NW * u
                assert 0 <= q * 1024 and (q + 1) * 1024 <= stage_bytes
                seen.add(q)
                for lane in range(64):
                    qq = q if q < QA else q - QA
                    row = qq * 8 + (lane >> 3)
                    chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7)
                    for kt in (0, K * ES // 128 - 1):
                        if q < QA:
                            r = row if bi0 + row < I else I - 1 - bi0
                            off = bi0 * lda * ES + r * lda * ES + chunk * 16 + kt * 128
                            assert 0 <= off and off + 16 <= a_bytes
                        else:
                            r = row if bj0 + row < J else J - 1 - bj0
                            off = bj0 * ldb * ES + r * ldb * ES + chunk * 16 + kt * 128
                            assert 0 <= off and off + 16 <= b_bytes
    assert seen == set(range((BI + BJ) // 8))


@pytest.mark.parametrize("WI,WJ", [(2, 2), (4, 2)])
def test_gemm_tn_fragment_and_strip_offsets_stay_inside_lds(WI, WJ):
    """the same kernel's LDS side on the host, for the withdrawn four-wave grid (2 x 2 waves, wave
    tile 128x128: TI = TJ = 8) and the shipped eight-wave one: every 16-byte fragment read
    (lds_chunk_offset of the block's row plus whole 64-row strides for blocks beyond the fourth)
    lies inside its operand's half of a stage, every fragment row of the tile is read by exactly
    one (wave, block, lane row), and the epilogue's output strips lie inside the stages"""
    BI = BJ = 256
    NS, NW = 2, WI * WJ
    TI, TJ = BI // (16 * WI), BJ // (16 * WJ)
    OPER, STAGE = BI * 128, (BI + BJ) * 128

    def lds_chunk_offset(row, chunk):
        return row * 128 + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4)

    rows_a, rows_b = set(), set()
    for wave in range(NW):
        wi, wj = wave // WJ, wave % WJ
        for lane in range(64):
            frag_row, frag_q = lane & 15, lane >> 4
            frag_chunk = (frag_q >> 1) | ((frag_q & 1) << 1)
            for ks in range(2):
                for ab in range(TI):
                    off = lds_chunk_offset(wi * TI * 16 + (ab & 3) * 16 + frag_row, ks * 4 + frag_chunk) + (ab >> 2) * 64 * 128
                    assert 0 <= off and off + 16 <= OPER
                    assert off // 128 == wi * TI * 16 + ab * 16 + frag_row
                    rows_a.add((off // 128, wj))
                for b in range(TJ):
                    off = OPER + lds_chunk_offset(wj * TJ * 16 + (b & 3) * 16 + frag_row, ks * 4 + frag_chunk) + (b >> 2) * 64 * 128
                    assert OPER <= off and off + 16 <= STAGE
                    assert (off - OPER) // 128 == wj * TJ * 16 + b * 16 + frag_row
                    rows_b.add(((off - OPER) // 128, wi))
        SP = TJ * 16 + 4
        assert (wave + 1) * 16 * SP * 4 <= NS * STAGE
    assert rows_a == {(r, wj) for r in range(BI) for wj in range(WJ)}
    assert rows_b == {(r, wi) for r in range(BJ) for wi in range(WI)}


@pytest.mark.parametrize("WI,WJ,BI,BJ,NS", [(4, 2, 256, 256, 2), (2, 4, 128, 128, 2), (2, 4, 128, 256, 3), (4, 2, 256, 128, 3)])
def test_gemm_tn_output_strips_cover_every_element_once(WI, WJ, BI, BJ, NS):
    """the epilogue of every shipped direct-to-LDS instance on the host (gemm_tn_kernel.h): a wave
    writes a 16-row block of accumulators into its LDS strip in the matrix core's layout (lane l:
    column l % 16, rows 4 * (l / 16) + r) and reads it back as 16-byte pieces (TJ instructions of
    64 / (4 TJ) rows x the wave tile's width).  Every element of the block tile must leave in
    exactly one piece, from the strip slot it was written to, and the strips of the eight waves
    must fit the LDS stages they reuse"""
    NW = WI * WJ
    TI, TJ = BI // (16 * WI), BJ // (16 * WJ)
    assert TJ >= 2 and TJ & (TJ - 1) == 0
    SP, CPR = TJ * 16 + 4, TJ * 4
    RPI = 64 // CPR
    assert NW * 16 * SP * 4 <= NS * (BI + BJ) * 128
    stored = {}
    for wave in range(NW):
        wi, wj = wave // WJ, wave % WJ
        for a in range(TI):
            slot_of = {}                        # strip slot -> (row, column) of the tile written there
            for lane in range(64):
                frag_row, frag_q = lane & 15, lane >> 4
                for b in range(TJ):
                    for r in range(4):
                        slot = (4 * frag_q + r) * SP + b * 16 + frag_row
                        assert slot not in slot_of and slot < 16 * SP
                        slot_of[slot] = ((wi * TI + a) * 16 + 4 * frag_q + r, (wj * TJ + b) * 16 + frag_row)
            for lane in range(64):
                for n in range(TJ):
                    base = (n * RPI + lane // CPR) * SP + (lane % CPR) * 4
                    i = (wi * TI + a) * 16 + n * RPI + lane // CPR
                    j = wj * TJ * 16 + (lane % CPR) * 4
                    for e in range(4):
                        assert slot_of[base + e] == (i, j + e)
                        assert (i, j + e) not in stored
                        stored[(i, j + e)] = wave
    assert len(stored) == BI * BJ


@pytest.mark.parametrize("tiles_i,tiles_j,batches", [(4, 4, 192), (1, 1, 8), (9, 3, 16), (8, 5, 24), (17, 2, 8), (3, 7, 40)])
def test_gemm_tn_batches_go_to_xcds_whole(tiles_i, tiles_j, batches):
    """the workgroup renumbering of a batched launch (gemm_tn_kernel.h; gridDim = (T, 1, batches),
    batches a multiple of 8) on the host: workgroups reach the 8 XCDs round-robin in launch order
    L = x + T * z; XCD L % 8 takes tile (L / 8) % T of batch L % 8 + 8 * ((L / 8) / T).  Every
    (batch, tile) must be computed exactly once, every tile index must lie inside the tile grid,
    and all tiles of a batch must run on one XCD"""
    T = tiles_i * tiles_j
    seen, xcd_of_batch = set(), {}
    for z in range(batches):
        for x in range(T):
            L = x + T * z
            xcd, sq = L & 7, L >> 3
            tile, batch = sq % T, xcd + 8 * (sq // T)
            per_group = 8 * tiles_j
            gidx = tile // per_group
            first_i = gidx * 8
            rows_here = min(tiles_i - first_i, 8)
            in_group = tile - gidx * per_group
            ti, tj = first_i + in_group % rows_here, in_group // rows_here
            assert 0 <= batch < batches and 0 <= ti < tiles_i and 0 <= tj < tiles_j
            assert (batch, ti, tj) not in seen
            seen.add((batch, ti, tj))
            assert xcd_of_batch.setdefault(batch, xcd) == xcd
    assert len(seen) == batches * T


def test_mfma_ceiling_refuses_bad_arguments_before_any_launch():
    """amos_mfma_ceiling checks its arguments on the host: an instruction shape it does not have,
    null buffers, buffers too small for the variant asked for (8 MiB per operand without the
    copies, a whole 8192 x 8192 fp16 matrix with them), a misaligned buffer"""
    import ctypes
    lib = _lib.load()
    sec, flop = ctypes.c_double(), ctypes.c_double()
    buf = ctypes.create_string_buffer(64)          # (never dereferenced: every call below is refused)
    a = ctypes.addressof(buf) & ~15
    big = 8192 * 8192 * 2
    cases = [(8, 0, 0, 0, a, a, big, a, 1), (16, 0, 0, 0, None, a, big, a, 1), (16, 0, 0, 0, a, a, big, None, 1),
             (16, 0, 0, 0, a, a, big, a, 0), (16, 1, 0, 0, a, a, (8 << 20) - 1, a, 1), (32, 1, 1, 0, a, a, big - 1, a, 1),
             (32, 1, 0, 0, a + 2, a, big, a, 1)]
    for shape, rnd, copies, reads, pa, pb, nbytes, sink, launches in cases:
        rc = lib.amos_mfma_ceiling(shape, rnd, copies, reads, pa, pb, nbytes, sink, launches, None,
                                   ctypes.byref(sec), ctypes.byref(flop))
        assert rc == _lib.AMOS_ERR_BAD_ARG and b"amos_mfma_ceiling" in lib.amos_last_error(), (shape, rnd, copies, nbytes)


def test_default_config_is_kept_per_descriptor():
    """amos_default_config keeps its last choices keyed by the descriptor: the same answer on every
    call (a call that names no configuration asks for it every time), each descriptor its own, and
    repeated calls at a cost far below the ~150 model evaluations of a first call"""
    import ctypes
    import time
    import torch
    from amos_amd import ops
    lib = _lib.load()
    descs = [(_lib.AMOS_OP_GEMM, ops.gemm_desc(m, 512, 1024, torch.float16, False, True)) for m in (64, 512, 4096, 8192)]
    descs += [(_lib.AMOS_OP_CONV2D, ops.conv_desc((n, 128, 1, 28, 28), (128, 128, 1, 3, 3), dt, (1, 1, 1), (0, 1, 1), (1, 1, 1)))
              for n in (1, 16, 64) for dt in (torch.float16, torch.int8)]
    descs.append((_lib.AMOS_OP_BGEMM, ops.bgemm_desc(192, 512, 512, 64, torch.float16, False, True)))
    first = []
    for op, d in descs:
        c = _lib.KernelConfig()
        assert lib.amos_default_config(op, ctypes.byref(d), ctypes.byref(c)) == 0
        first.append((c.tile_i, c.tile_j, c.split_k, c.pipeline))
    assert len(set(first)) > 3                      # (the shapes do not all get one answer)
    t0 = time.perf_counter()
    for _ in range(50):
        for (op, d), want in zip(descs, first):
            c = _lib.KernelConfig()
            assert lib.amos_default_config(op, ctypes.byref(d), ctypes.byref(c)) == 0
            assert (c.tile_i, c.tile_j, c.split_k, c.pipeline) == want
    per_call = (time.perf_counter() - t0) / (50 * len(descs))
    assert per_call < 20e-6, per_call
    # an invalid descriptor is refused every time (errors are not kept)
    bad = ops.gemm_desc(64, 64, 64, torch.float16, False, True)
    bad.M = -1
    for _ in range(2):
        assert lib.amos_default_config(_lib.AMOS_OP_GEMM, ctypes.byref(bad), ctypes.byref(_lib.KernelConfig())) != 0


def test_planner_is_consistent_with_itself_on_random_shapes():
    """seeded random GEMMs, batched GEMMs and convolutions (2-d, 3-d, grouped, depthwise; windows
    1 to 7, strides, paddings): amos_default_config's choice passes amos_check_config, has a kernel
    instance (as does a null configuration), an estimate and a sane workspace size"""
    import ctypes
    import torch
    from amos_amd import ops
    lib = _lib.load()
    import numpy as np
    rng = np.random.default_rng(7)
    checked = 0
    for _ in range(500):
        kind = int(rng.integers(0, 4))
        dt = [torch.float16, torch.bfloat16, torch.int8][int(rng.integers(0, 3))]
        if kind == 0:
            M, N, K = [int(x) for x in rng.choice([1, 3, 8, 17, 64, 96, 128, 200, 512, 1000, 2048, 4096, 8192], 3)]
            op, d = _lib.AMOS_OP_GEMM, ops.gemm_desc(M, N, K, dt, bool(rng.integers(0, 2)), bool(rng.integers(0, 2)))
            what = ("gemm", M, N, K, dt)
        elif kind == 1:
            B = int(rng.choice([1, 2, 8, 16, 24, 192]))
            M, N, K = [int(x) for x in rng.choice([8, 64, 128, 512, 1024], 3)]
            op, d = _lib.AMOS_OP_BGEMM, ops.bgemm_desc(B, M, N, K, dt, bool(rng.integers(0, 2)), bool(rng.integers(0, 2)))
            what = ("bgemm", B, M, N, K, dt)
        else:
            three = kind == 3
            n, C = int(rng.choice([1, 2, 8, 16, 32, 64])), int(rng.choice([3, 16, 24, 32, 64, 96, 128, 256, 512]))
            K = int(rng.choice([8, 32, 64, 72, 128, 256, 512]))
            H = int(rng.choice([7, 14, 28, 56, 112]))
            W = H if rng.integers(0, 2) else int(rng.choice([7, 9, 14, 30]))
            D = int(rng.choice([1, 4, 16])) if three else 1
            R = int(rng.choice([1, 3, 5, 7]))
            T = int(rng.choice([1, 3])) if three else 1
            st, pd = int(rng.choice([1, 2])), int(rng.choice([0, 1, R // 2]))
            groups = 1
            if rng.integers(0, 6) == 0 and C % 4 == 0 and K % 4 == 0:
                groups = 4
            if rng.integers(0, 8) == 0:
                groups, K = C, C
            xs, ws = (n, C, D, H, W), (K, C // groups, T, R, R)
            stride, pad = (st if three else 1, st, st), (pd if three else 0, pd, pd)
            if min(ops.conv_out_shape(xs, ws, stride, pad, (1, 1, 1))) <= 0:
                continue
            op = _lib.AMOS_OP_CONV3D if three else _lib.AMOS_OP_CONV2D
            d = ops.conv_desc(xs, ws, dt, stride, pad, (1, 1, 1), groups)
            what = ("conv", xs, ws, st, pd, groups, dt)
        c = _lib.KernelConfig()
        assert lib.amos_default_config(op, ctypes.byref(d), ctypes.byref(c)) == 0, (what, lib.amos_last_error())
        cfg = (c.tile_i, c.tile_j, c.split_k, c.pipeline)
        assert lib.amos_kernel_name(op, ctypes.byref(d), ctypes.byref(c)) is not None, (what, cfg, lib.amos_last_error())
        assert lib.amos_kernel_name(op, ctypes.byref(d), None) is not None, (what, lib.amos_last_error())
        assert lib.amos_check_config(op, ctypes.byref(d), ctypes.byref(c), None, None) >= 0, (what, cfg, lib.amos_last_error())
        est = ctypes.c_double()
        assert lib.amos_estimate_seconds(op, ctypes.byref(d), ctypes.byref(c), ctypes.byref(est)) == 0 and 0 < est.value < 10, (what, cfg)
        assert 0 <= lib.amos_workspace_bytes(op, ctypes.byref(d), ctypes.byref(c)) < (64 << 30), (what, cfg)
        assert 0 <= lib.amos_workspace_bytes(op, ctypes.byref(d), None) < (64 << 30), what
        checked += 1
    assert checked > 400


@pytest.mark.parametrize("BI,BJ,WI,WJ,HV", [(64, 128, 2, 4, 1), (64, 256, 1, 8, 1), (32, 128, 1, 4, 1), (32, 256, 1, 4, 1),
                                            (64, 128, 2, 4, 2), (64, 256, 1, 8, 2)])
def test_conv_nchw_output_strips_cover_every_element_once(BI, BJ, WI, WJ, HV):
    """the strip epilogue of every NCDHW-direct instance on the host (conv_nchw_kernel.h): per
    16-row block and half of the output channels a matrix-core wave writes its accumulators into
    its LDS strip in the matrix core's layout and reads them back as 16-byte pieces of whole rows.
    Every element of the (HV * BI) x BJ tile leaves exactly once, from the slot it was written to;
    the eight (four) strips fit the two weight buffers they reuse"""
    NWM = WI * WJ
    TI, TJ = BI // (16 * WI), BJ // (16 * WJ)
    assert TJ & (TJ - 1) == 0 and TJ <= 16
    SP, CPR = TJ * 16 + 4, TJ * 4
    RPI = 64 // CPR
    assert NWM * 16 * SP * 4 <= 2 * 9 * BI * 64
    stored = set()
    for wave in range(NWM):
        wi, wj = wave // WJ, wave % WJ
        for ha in range(HV * TI):
            h, a = ha // TI, ha % TI
            slot_of = {}
            for lane in range(64):
                frag_row, frag_q = lane & 15, lane >> 4
                for b in range(TJ):
                    for r in range(4):
                        slot = (4 * frag_q + r) * SP + b * 16 + frag_row
                        assert slot not in slot_of and slot < 16 * SP
                        slot_of[slot] = (h * BI + (wi * TI + a) * 16 + 4 * frag_q + r, (wj * TJ + b) * 16 + frag_row)
            for lane in range(64):
                for x in range(TJ):
                    base = (x * RPI + lane // CPR) * SP + (lane % CPR) * 4
                    i = h * BI + (wi * TI + a) * 16 + x * RPI + lane // CPR
                    j4 = wj * TJ * 16 + (lane % CPR) * 4
                    for e in range(4):
                        assert slot_of[base + e] == (i, j4 + e)
                        assert (i, j4 + e) not in stored
                        stored.add((i, j4 + e))
    assert len(stored) == HV * BI * BJ
