"""The reference's script flow on the GPU: TE compute -> auto_tensorize -> schedule ->
build -> func(A, B, C), checked against the CPU oracle (reference flow: README.md:174-340,
benchmark/amos/mapping_gemm_tensorcore.py:18-85)."""
import json

import numpy as np
import pytest

import amos_amd.tvm as tvm
from amos_amd.tvm import auto_tensorize as at
from oracle import cpu_oracle as co
from test_mapper import (batch_conv2d, batched_fc, capsule_conv2d, conv1d, conv2d, conv2d_layout, depthwise_conv2d, from_nkpq, gemm, gemv,
                         grouped_conv2d, grouped_conv_reference, mean, scan, to_nchw, transposed_conv2d, variance)

pytestmark = pytest.mark.gpu


def test_conv2d_tutorial_flow(gpu, tmp_path, capsys):
    N, C, H, W, K, R, S, stride, padding, dilation = 2, 128, 14, 14, 64, 3, 3, 1, 1, 1
    A, B, Conv = conv2d(N, C, H, W, K, R, S, stride, padding, dilation)
    target_dag = at.compute_dag_from_tensors([Conv])
    target = "hip"
    measure_opt = at.MeasureOptions(target=target, timeout=10, number=5, min_repeat_ms=5)
    log = str(tmp_path / "conv2d_tutorial.log")
    result = at.auto_tensorize(target_dag, target, log, measure_opt, trials=6)
    assert result.defined()
    lines = [json.loads(l) for l in open(log)]
    assert len(lines) == 6 and all(set(l) == {"record", "value"} for l in lines)
    assert 1 / result.perf == pytest.approx(max(l["value"] for l in lines))
    # reload from the log, as the reference's scripts do
    result.sch_gen.load_from_file(log, clear=True)
    entry = result.sch_gen.get_best_entry()
    params, value = entry.record, 1 / entry.value
    cost = at.evaluate_params(result.sch_app, params, measure_opt, dump=False)
    assert 0 < cost < 1e3 and value > 0
    # retrieve schedule from the record, build, run
    schedule_app = result.sch_app
    inputs = schedule_app.target_dag.get_inputs()
    args = inputs + list(schedule_app.target_dag.tensors)
    sch = tvm.te.create_schedule([x.op for x in schedule_app.target_dag.tensors])
    sch = schedule_app.apply(sch, params)
    func = tvm.build(sch, args, target)
    rng = np.random.default_rng(0)
    A_np = rng.uniform(-10, 10, [int(x) for x in A.shape]).astype(A.dtype)
    B_np = rng.uniform(-10, 10, [int(x) for x in B.shape]).astype(B.dtype)
    Conv_np = np.zeros([int(x) for x in Conv.shape], dtype=Conv.dtype)
    ctx = tvm.context(target, 0)
    A_tvm, B_tvm, Conv_tvm = tvm.nd.array(A_np, ctx), tvm.nd.array(B_np, ctx), tvm.nd.array(Conv_np, ctx)
    func(A_tvm, B_tvm, Conv_tvm)
    ctx.sync()
    golden = co.lib_conv2d(A_np, B_np, "float16", stride, padding, dilation, acc="float32")
    tvm.testing.assert_allclose(golden, Conv_tvm.asnumpy(), atol=1e-2 * float(golden.std()), rtol=1e-2)
    mx, mean = co.rel_errors(Conv_tvm.asnumpy(), golden)
    assert mx <= 1e-2 and mean <= 1e-3
    assert "amos_" in func.imported_modules[0].get_source()
    t = func.time_evaluator(func.entry_name, ctx, number=5, min_repeat_ms=5)(A_tvm, B_tvm, Conv_tvm).mean
    assert 0 < t < 1e-2


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 1)])
def test_gemm_script_flow(gpu, tmp_path, ta, tb):
    M, N, K = 384, 256, 320
    A, B, C = gemm(M, N, K, ta=ta, tb=tb)
    dag = at.compute_dag_from_tensors([C])
    opt = at.MeasureOptions(target="hip", timeout=100, number=5, min_repeat_ms=5)
    result = at.auto_tensorize(dag, "hip", str(tmp_path / "gemm.log"), opt, trials=4)
    assert result.defined()
    sch, args = at.get_schedule(result.sch_app, result.params)
    func = tvm.build(sch, args, "hip")
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, [int(s) for s in A.shape]).astype(np.float16)
    b = rng.uniform(-1, 1, [int(s) for s in B.shape]).astype(np.float16)
    ctx = tvm.context("hip", 0)
    c = tvm.nd.array(np.zeros((M, N), dtype=np.float32), ctx)
    func(tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), c)
    mx, mean = co.rel_errors(c.asnumpy(), co.lib_gemm(a, b, "float16", ta, tb, acc="float32"))
    assert mx <= 1e-2 and mean <= 1e-3


def test_v4_explores_the_realised_mappings(gpu, tmp_path, capsys):
    A, B, Conv = conv2d(4, 128, 14, 14, 128, 3, 3, 1, 1, 1, dtype="int8", out_dtype="int32", exact_int=True)
    opt = at.MeasureOptions(target="hip", number=3, min_repeat_ms=2)
    res = at.auto_tensorize_v4(at.compute_dag_from_tensors([Conv]), "hip", "conv.log", opt,
                               schedule_log_dir=str(tmp_path / "logs"), trials=40, repeat_rounds=1,
                               search_group_size=1)
    out = capsys.readouterr().out
    assert res.defined() and "Round 1, Match 1, Mapping" in out and "New weights" in out
    assert "No kernel instance realises this mapping; skipped." in out
    sch, args = at.get_schedule(res.sch_app, res.params)
    func = tvm.build(sch, args, "hip")
    rng = np.random.default_rng(2)
    a = rng.integers(-128, 128, [int(s) for s in A.shape]).astype(np.int8)
    b = rng.integers(-64, 64, [int(s) for s in B.shape]).astype(np.int8)
    ctx = tvm.context("hip", 0)
    y = tvm.nd.array(np.zeros([int(s) for s in Conv.shape], dtype=np.int32), ctx)
    func(tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), y)
    assert np.array_equal(y.asnumpy(), co.lib_conv2d(a, b, "int8", 1, 1, 1))


def test_gemm_with_elementwise_tail(gpu, tmp_path):
    """E = C + D behind the GEMM, the compute of the reference's
    tests/python/auto_tensorize/test_compute_transform_gemm.py:7-23, through the script flow:
    the tail is fused into the kernel and D becomes the module's third input"""
    M, N, K = 256, 192, 320
    A = tvm.te.placeholder([M, K], dtype="float16", name="A")
    B = tvm.te.placeholder([K, N], dtype="float16", name="B")
    tk = tvm.te.reduce_axis([0, K], name="tk")
    C = tvm.te.compute([M, N], lambda ti, tj: tvm.te.sum((A[ti, tk] * B[tk, tj]).astype("float32"), axis=tk),
                       name="C")
    D = tvm.te.placeholder([M, N], dtype="float32", name="D")
    E = tvm.te.compute([M, N], lambda si, sj: C[si, sj] + D[si, sj], name="E")
    dag = at.compute_dag_from_tensors([E])
    opt = at.MeasureOptions(target="hip", timeout=100, number=5, min_repeat_ms=5)
    result = at.auto_tensorize(dag, "hip", str(tmp_path / "gemm_tail.log"), opt, trials=4)
    assert result.defined()
    assert result.sch_app.lowered.add_input is D
    sch, args = at.get_schedule(result.sch_app, result.params)
    assert [t.name for t in args] == ["A", "B", "D", "E"]
    func = tvm.build(sch, args, "hip")
    rng = np.random.default_rng(2)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float16)
    d = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    ctx = tvm.context("hip", 0)
    e = tvm.nd.array(np.zeros((M, N), dtype=np.float32), ctx)
    func(tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), tvm.nd.array(d, ctx), e)
    ctx.sync()
    ref = co.lib_gemm(a, b, "float16", 0, 0, acc="float64") + d
    mx, mean = co.rel_errors(e.asnumpy(), ref)
    assert mx <= 1e-2 and mean <= 1e-3
    t = func.time_evaluator(func.entry_name, ctx, number=5, min_repeat_ms=5)(
        tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), tvm.nd.array(d, ctx), e).mean
    assert 0 < t < 1e-2


def _run_script_flow(tensors, feeds, tmp_path, name, **kwargs):
    """auto_tensorize -> get_schedule -> build -> func(*arrays); returns the output array"""
    dag = at.compute_dag_from_tensors([tensors[-1]])
    opt = at.MeasureOptions(target="hip", timeout=100, number=5, min_repeat_ms=5)
    result = at.auto_tensorize(dag, "hip", str(tmp_path / (name + ".log")), opt, trials=4, **kwargs)
    assert result.defined()
    sch, args = at.get_schedule(result.sch_app, result.params)
    func = tvm.build(sch, args, "hip")
    ctx = tvm.context("hip", 0)
    arrays = [tvm.nd.array(feeds[t.name], ctx) for t in args[:-1]]
    out = tvm.nd.array(np.zeros([int(s) for s in args[-1].shape], dtype=args[-1].dtype), ctx)
    func(*arrays, out)
    ctx.sync()
    return out.asnumpy(), result


def test_gemv_script_flow(gpu, tmp_path):
    """reference compute: benchmark/amos/mapping_gemv_tensorcore.py:7-16 (GEMM with N = 1 and a
    reshaping stage behind it)"""
    M, K = 1000, 520
    A, B, D = gemv(M, K)
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    b = rng.uniform(-1, 1, (K, 1)).astype(np.float16)
    with pytest.raises(RuntimeError, match="infeasible"):   # N = 1 < 16: the strict rule of the reference
        _run_script_flow([A, B, D], {"A": a, "B": b}, tmp_path, "gemv_strict")
    got, result = _run_script_flow([A, B, D], {"A": a, "B": b}, tmp_path, "gemv", transform_strict=False)
    assert got.shape == (M,) and result.sch_app.lowered.kind == "gemm"
    ref = (a.astype(np.float64) @ b.astype(np.float64))[:, 0]
    mx, mean = co.rel_errors(got, ref)
    assert mx <= 1e-2 and mean <= 1e-3


def test_batched_fc_script_flow(gpu, tmp_path):
    """reference compute: benchmark/amos/mapping_batchedfc_tensorcore.py:7-37 (channel groups
    read through reshaping stages: a batched GEMM with strided batches)"""
    N, I, O, groups = 96, 512, 384, 4
    A, B, F = batched_fc(N, I, O, groups)
    rng = np.random.default_rng(6)
    a = rng.uniform(-1, 1, (N, I)).astype(np.float16)
    b = rng.uniform(-1, 1, (O, I // groups)).astype(np.float16)
    got, result = _run_script_flow([A, B, F], {"A": a, "B": b}, tmp_path, "bfc")
    assert result.sch_app.lowered.kind == "bgemm"
    a64 = a.astype(np.float64).reshape(N, groups, I // groups)
    b64 = b.astype(np.float64).reshape(groups, O // groups, I // groups)
    ref = np.einsum("ngc,gkc->ngk", a64, b64)
    mx, mean = co.rel_errors(got, ref)
    assert got.shape == (N, groups, O // groups) and mx <= 1e-2 and mean <= 1e-3


@pytest.mark.parametrize("C", [64, 24])    # patch-staged and register-staged kernels
def test_conv1d_script_flow(gpu, tmp_path, C):
    """reference compute: benchmark/amos/mapping_conv1d_tensorcore.py:7-42"""
    N, L, K, KL, stride, padding, dilation = 4, 200, 48, 5, 2, 2, 1
    A, B, Out = conv1d(N, C, L, K, KL, stride, padding, dilation)
    rng = np.random.default_rng(7)
    a = rng.uniform(-1, 1, (N, C, L)).astype(np.float16)
    b = rng.uniform(-1, 1, (K, C, KL)).astype(np.float16)
    got, result = _run_script_flow([A, B, Out], {"A": a, "B": b}, tmp_path, "conv1d")
    assert result.sch_app.lowered.kind == "conv2d"
    ref = co.lib_conv2d(a[:, :, None, :], b[:, :, None, :], "float16", (1, stride), (0, padding), (1, dilation),
                        acc="float64")[:, :, 0, :]
    mx, mean = co.rel_errors(got, ref)
    assert got.shape == ref.shape and mx <= 1e-2 and mean <= 1e-3


@pytest.mark.parametrize("layout", ["nhwc", "hwnc"])
@pytest.mark.parametrize("C", [64, 24])    # patch-staged and register-staged kernels
def test_conv2d_layout_script_flow(gpu, tmp_path, layout, C):
    """reference computes: benchmark/amos/mapping_conv2d_tensorcore.py:43-104"""
    N, H, W, K, R, S, stride, padding, dilation = 3, 20, 18, 40, 3, 3, 1, 1, 1
    A, B, Conv = conv2d_layout(N, C, H, W, K, R, S, stride, padding, dilation, layout)
    rng = np.random.default_rng(9)
    a = rng.uniform(-1, 1, [int(e) for e in A.shape]).astype(np.float16)
    b = rng.uniform(-1, 1, (R, S, C, K)).astype(np.float16)
    got, result = _run_script_flow([A, B, Conv], {"A": a, "B": b}, tmp_path, "conv2d_" + layout)
    low = result.sch_app.lowered
    assert low.kind == "conv2d" and low.attrs["layout"] == layout
    an, bn = to_nchw(a, b, layout)
    ref = from_nkpq(co.lib_conv2d(np.ascontiguousarray(an), np.ascontiguousarray(bn), "float16", stride, padding,
                                  dilation, acc="float64"), layout)
    mx, mean = co.rel_errors(got, ref)
    assert got.shape == ref.shape and mx <= 1e-2 and mean <= 1e-3


@pytest.mark.parametrize("dtype", ["float16", "int8", "float32"])
def test_gather_entry_point(gpu, dtype):
    """amos_gather against numpy: a padded, zero-expanded, flipped and transposed view"""
    import torch
    from amos_amd import ops
    from amos_amd.auto_tensorize.measure import _TORCH_DTYPE
    rng = np.random.default_rng(5)
    src = (rng.integers(-100, 100, (3, 5, 6, 7))).astype(dtype)
    # out[a, b, c, d] = src[b, a, 5 - (c - 2) / 2, d - 1] where c - 2 is even and in range, 0 <= d - 1 < 7
    strides = [5 * 6 * 7, 6 * 7, 7, 1]
    tables = [[i * strides[1] for i in range(5)], [i * strides[0] for i in range(3)],
              [(5 - (c - 2) // 2) * strides[2] if (c - 2) % 2 == 0 and 0 <= (c - 2) // 2 < 6 else -1 for c in range(15)],
              [(d - 1) * strides[3] if 0 <= d - 1 < 7 else -1 for d in range(10)]]
    want = np.zeros((5, 3, 15, 10), dtype=src.dtype)
    for c in range(15):
        for d in range(10):
            if tables[2][c] >= 0 and tables[3][d] >= 0:
                want[:, :, c, d] = src[:, :, 5 - (c - 2) // 2, d - 1].T
    g = ops.Gather([5, 3, 15, 10], tables, _TORCH_DTYPE[dtype], src.size, torch.device("cuda", 0))
    got = g(torch.from_numpy(src).cuda())
    assert np.array_equal(got.cpu().numpy(), want)
    secs = g.time(torch.from_numpy(src).cuda(), got, number=3, repeat=2, min_repeat_ms=1)
    assert len(secs) == 2 and all(0 < t < 1e-2 for t in secs)


@pytest.mark.parametrize("case", [(2, 48, 14, 14, 64, 4, 2, 1, 0, 1), (1, 24, 9, 11, 40, 3, 2, 1, 1, 1),
                                  (3, 64, 8, 8, 64, 3, 1, 1, 0, 2)])
def test_transposed_conv_script_flow(gpu, tmp_path, case):
    """reference compute: benchmark/amos/mapping_transposedconv2d_tensorcore.py:55-102; against the
    scatter definition of a transposed convolution in double precision"""
    import torch
    N, C, H, W, K, ks, stride, padding, output_padding, dilation = case
    A, B, Out = transposed_conv2d(N, C, H, W, K, ks, stride, padding, output_padding, dilation)
    rng = np.random.default_rng(8)
    a = rng.uniform(-1, 1, (N, K, H, W)).astype(np.float16)
    b = rng.uniform(-1, 1, (K, C, ks, ks)).astype(np.float16)
    got, result = _run_script_flow([A, B, Out], {"A": a, "B": b}, tmp_path, "tconv")
    low = result.sch_app.lowered
    assert low.kind == "conv2d" and sorted(low.gathers) == [0, 1]
    ref = torch.nn.functional.conv_transpose2d(torch.from_numpy(a).double(), torch.from_numpy(b).double(),
                                               stride=stride, padding=padding, output_padding=output_padding,
                                               dilation=dilation).numpy()
    mx, mean = co.rel_errors(got, ref)
    assert got.shape == ref.shape and mx <= 1e-2 and mean <= 1e-3
    # the module's timing covers the materialised stages as well
    sch, args = at.get_schedule(result.sch_app, result.params)
    func = tvm.build(sch, args, "hip")
    ctx = tvm.context("hip", 0)
    arrs = [tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), tvm.nd.array(np.zeros(ref.shape, dtype=np.float32), ctx)]
    t = func.time_evaluator(func.entry_name, ctx, number=3, min_repeat_ms=2)(*arrs).mean
    mx2, _ = co.rel_errors(arrs[2].asnumpy(), ref)     # (a split-K configuration sums in any order)
    assert 0 < t < 1e-2 and mx2 <= 1e-2


def test_mean_and_scan_script_flows(gpu, tmp_path):
    """reference computes: benchmark/amos/mapping_mean_tensorcore.py:7-25 (a GEMM whose left
    operand is a gathered view and whose right operand is a constant vector; like the GEMV its
    N = 1 needs transform_strict=False) and mapping_scan_tensorcore.py:7-21 (prefix sums as a
    GEMM with a constant triangle of ones)"""
    rng = np.random.default_rng(10)
    N, C, H, W = 8, 96, 14, 14
    A, B, E = mean(N, C, H, W)
    a = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float16)
    got, result = _run_script_flow([A, B, E], {"A": a}, tmp_path, "mean", transform_strict=False)
    low = result.sch_app.lowered
    assert low.kind == "gemm" and list(low.gathers) == [0] and list(low.constants) == [1]
    ref = (a.astype(np.float64) * float(np.float16(1.0 / (N * H * W)))).sum(axis=(0, 2, 3))
    assert got.shape == (C,) and np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max() + 1e-4
    M, Nn, K = 300, 256, 256
    A, B, Cc = scan(M, Nn, K)
    a = rng.integers(-3, 4, (M, K)).astype(np.float16)
    got, result = _run_script_flow([A, B, Cc], {"A": a}, tmp_path, "scan")
    assert list(result.sch_app.lowered.constants) == [1]
    assert np.array_equal(got, np.cumsum(a.astype(np.float32), axis=1))     # small integers: exact


@pytest.mark.parametrize("kind", ["grouped", "depthwise", "batch"])
def test_grouped_conv_script_flow(gpu, tmp_path, kind):
    """reference computes: benchmark/amos/mapping_groupedconv2d_tensorcore.py:7-60,
    mapping_depthwiseconv2d_tensorcore.py:7-48, mapping_batchconv2d_tensorcore.py:7-40 (a filter
    bank per image: the images are the groups of a one-image convolution)"""
    if kind == "batch":
        N, C, H, W, K, R, S, stride, padding = 6, 32, 14, 14, 48, 3, 3, 1, 1
        A, B, Out = batch_conv2d(N, C, H, W, K, R, S, stride, padding)
        rng = np.random.default_rng(10)
        a = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float16)
        b = rng.uniform(-1, 1, (N, K, C, R, S)).astype(np.float16)
        got, result = _run_script_flow([A, B, Out], {"A": a, "B": b}, tmp_path, kind, transform_strict=False)
        low = result.sch_app.lowered
        assert low.kind == "conv2d" and low.desc.groups == N and low.desc.N == 1
        ref = np.stack([co.lib_conv2d(a[n:n + 1], b[n], "float16", stride, padding, 1, acc="float64")[0]
                        for n in range(N)])
        mx, mean = co.rel_errors(got, ref)
        assert got.shape == ref.shape and mx <= 1e-2 and mean <= 1e-3
        return
    if kind == "grouped":
        N, C, H, W, K, R, S, stride, padding, groups = 4, 64, 14, 14, 128, 3, 3, 1, 1, 4
        A, B, Out = grouped_conv2d(N, C, H, W, K, R, S, stride, padding, groups)
    else:
        N, C, H, W, K, R, S, stride, padding = 2, 32, 14, 14, 64, 3, 3, 2, 1
        groups = C
        A, B, Out = depthwise_conv2d(N, C, H, W, K, R, S, stride, padding)
    rng = np.random.default_rng(9)
    a = rng.uniform(-1, 1, [int(s) for s in A.shape]).astype(np.float16)
    b = rng.uniform(-1, 1, [int(s) for s in B.shape]).astype(np.float16)
    got, result = _run_script_flow([A, B, Out], {"A": a, "B": b}, tmp_path, kind, transform_strict=False)
    low = result.sch_app.lowered
    assert low.kind == "conv2d" and low.desc.groups == groups
    ref = grouped_conv_reference(a, b, stride, padding, groups)
    mx, mean = co.rel_errors(got, ref)
    assert got.shape == ref.shape and mx <= 1e-2 and mean <= 1e-3


def test_capsule_conv_script_flow(gpu, tmp_path):
    """reference compute: benchmark/amos/mapping_capsuleconv2d_tensorcore.py:7-72 (filters with a
    trailing capsule axis: gathered in front of an ordinary convolution, the result reordered
    behind it); the module's time_evaluator counts both gathers"""
    N, C, H, W, K, R, S, caps, stride, padding, dilation = 4, 32, 14, 14, 16, 3, 3, 8, 1, 1, 1
    A, B, Out = capsule_conv2d(N, C, H, W, K, R, S, caps, stride, padding, dilation)
    rng = np.random.default_rng(12)
    a = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float16)
    b = rng.uniform(-1, 1, (K, C, R, S, caps)).astype(np.float16)
    got, result = _run_script_flow([A, B, Out], {"A": a, "B": b}, tmp_path, "capsule", transform_strict=False)
    low = result.sch_app.lowered
    assert low.kind == "conv2d" and low.desc.K == K * caps and low.out_view is not None and list(low.gathers) == [1]
    wk = np.ascontiguousarray(b.transpose(0, 4, 1, 2, 3).reshape(K * caps, C, R, S))
    ref = co.lib_conv2d(a, wk, "float16", stride, padding, dilation, acc="float64")
    ref = ref.reshape(N, K, caps, H, W).transpose(0, 1, 3, 4, 2)
    mx, mean = co.rel_errors(got, ref)
    assert got.shape == ref.shape == (N, K, H, W, caps) and mx <= 1e-2 and mean <= 1e-3
    # a second call reuses the module's buffers; timing includes the two gathers
    sch, args = at.get_schedule(result.sch_app, result.params)
    func = tvm.build(sch, args, "hip")
    ctx = tvm.context("hip", 0)
    arrays = [tvm.nd.array(x, ctx) for x in (a, b)] + [tvm.nd.array(np.zeros(got.shape, dtype=np.float32), ctx)]
    func(*arrays)
    func(*arrays)
    ctx.sync()
    # (a tuned split-K config accumulates with atomics: equal up to the order of additions)
    assert np.allclose(arrays[-1].asnumpy(), got, rtol=1e-5, atol=1e-5)
    t = func.time_evaluator(func.entry_name, ctx, number=5, min_repeat_ms=5)(*arrays).mean
    assert 0 < t < 1e-3


def test_variance_script_flow(gpu, tmp_path):
    """reference compute: benchmark/amos/mapping_variance_tensorcore.py:7-31 (squared differences
    computed element-wise in front of the mean's GEMM)"""
    N, C, H, W = 8, 96, 14, 14
    A, Mean, E = variance(N, C, H, W)
    rng = np.random.default_rng(14)
    a = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float16)
    m = rng.uniform(-0.2, 0.2, (N, C, H, W)).astype(np.float16)
    got, result = _run_script_flow([A, Mean, E], {"A": a, "Mean": m}, tmp_path, "variance", transform_strict=False)
    low = result.sch_app.lowered
    assert low.kind == "gemm" and list(low.computed) == [0]
    # as the compute's own fp16 arithmetic rounds: difference, then square, both to fp16
    diff = (a - m).astype(np.float16)
    sq = (diff * diff).astype(np.float16).astype(np.float64)
    ref = sq.transpose(1, 0, 2, 3).reshape(C, -1).sum(axis=1) * float(np.float16(1.0 / (N * H * W)))
    assert got.shape == (C,) and np.allclose(got, ref, rtol=2e-3, atol=1e-4)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
def test_eltwise_entry_point(gpu, dtype):
    """amos_eltwise: every operation rounds to the element type (int8 wraps)"""
    import torch
    from amos_amd import ops
    rng = np.random.default_rng(15)
    n = 100003
    if dtype == "int8":
        x = rng.integers(-128, 128, n).astype(np.int8)
        y = rng.integers(-128, 128, n).astype(np.int8)
        tx, ty = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
        d = (x - y).astype(np.int8)                     # numpy wraps like the compute's int8 arithmetic
        want = ((d * d).astype(np.int8) + np.int8(3)).astype(np.int8)
    else:
        tdt = torch.float16 if dtype == "float16" else torch.bfloat16
        tx = torch.from_numpy(rng.uniform(-4, 4, n).astype(np.float32)).cuda().to(tdt)
        ty = torch.from_numpy(rng.uniform(-4, 4, n).astype(np.float32)).cuda().to(tdt)
        d = (tx.float() - ty.float()).to(tdt)
        want = ((d.float() * d.float()).to(tdt).float() + 3.0).to(tdt)
    prog = [("load", 0), ("load", 1), "sub", ("load", 0), ("load", 1), "sub", "mul", ("const", 3.0), "add"]
    e = ops.Eltwise(prog, 2, tx.dtype, n)
    got = e([tx, ty])
    if dtype == "int8":
        assert np.array_equal(got.cpu().numpy(), want)
    else:
        assert torch.equal(got, want)
    with pytest.raises(Exception, match="stack|program"):
        ops.Eltwise(["add"], 1, tx.dtype, n)([tx])



@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("rows", ["npq", "nq", "np", "n", "npq+s", "nq+s", "npq+r", "np+r"])
def test_conv2d_mapping_classes_run_and_agree(gpu, rows, dtype):
    """Mappings that fuse only some of the output loops into the rows of the implicit GEMM (p and / or
    q stay time loops), with the reduce side on channels only (patch-staged kernels, window taps as
    time loops), on channels and one window loop ("+s" / "+r": that loop's taps become channels of
    the image the kernel sees) or on channels and both window loops (register-staged kernel): every
    class against the oracle (the reference builds a kernel per mapping:
    tensorization_phases/compute_transform.py:343-499; its A100 log for this shape family picks
    i <- {n, q}, rk <- {rc, rs}, here "nq+s")"""
    from amos_amd import _lib
    from amos_amd.auto_tensorize.lowering import lower_main_op, remap_conv2d_rows
    from amos_amd.auto_tensorize.runtime import Module
    from amos_amd.auto_tensorize.schedule import KernelParams
    N, C, H, W, K, stride, pad, dil = 4, 64, 10, 12, 40, 1, 1, 1
    if dtype == "int8":
        A, B, Conv = conv2d(N, C, H, W, K, 3, 3, stride, pad, dil, dtype="int8", out_dtype="int32", exact_int=True)
    else:
        A, B, Conv = conv2d(N, C, H, W, K, 3, 3, stride, pad, dil)
    dag = at.compute_dag_from_tensors([Conv])
    main_op = [op for op in dag.op_lst if op.reduce_axis][0]
    low = remap_conv2d_rows(lower_main_op(main_op, dag), rows)
    rng = np.random.default_rng(3)
    if dtype == "int8":
        a = rng.integers(-128, 128, [int(s) for s in A.shape]).astype(np.int8)
        b = rng.integers(-64, 64, [int(s) for s in B.shape]).astype(np.int8)
        ref = co.lib_conv2d(a, b, "int8", stride, pad, dil)
    else:
        a = rng.uniform(-1, 1, [int(s) for s in A.shape]).astype(np.float16)
        b = rng.uniform(-1, 1, [int(s) for s in B.shape]).astype(np.float16)
        ref = co.lib_conv2d(a, b, "float16", stride, pad, dil, acc="float64")
    ctx = tvm.context("hip", 0)
    ran = []
    # (the patch-staged kernel prefetches a tile's next patch behind its window taps: with the three
    # taps of a folded window a 128-wide tile's patch is too much for that, a 64-wide one is not)
    for pipe, tile_i, tile_j in ((_lib.AMOS_PIPE_PATCH8, 64, 128), (_lib.AMOS_PIPE_PATCH8, 128, 64), (_lib.AMOS_PIPE_STAGED, 64, 128)):
        if pipe in ran:
            continue
        params = KernelParams(tile_i, tile_j, 1, pipe)
        func = Module(low, params, [A, B, Conv])
        y = tvm.nd.array(np.zeros([int(s) for s in Conv.shape], dtype=ref.dtype if dtype == "int8" else np.float32), ctx)
        try:
            func(tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), y)
        except _lib.AmosError as e:
            assert pipe == _lib.AMOS_PIPE_PATCH8 and "not applicable" in str(e), str(e)
            continue
        ctx.sync()
        name = func.imported_modules[0].get_source()
        assert ("amos_conv_fprop" if pipe == _lib.AMOS_PIPE_PATCH8 else "amos_igemm") in name, name
        if dtype == "int8":
            assert np.array_equal(y.asnumpy(), ref), (rows, pipe)
        else:
            mx, mean = co.rel_errors(y.asnumpy(), ref)
            assert mx <= 1e-2 and mean <= 1e-3, (rows, pipe, mx, mean)
        ran.append(pipe)
    # the register-staged kernel runs every class; the patch-staged one all but "rows n" at most
    assert _lib.AMOS_PIPE_STAGED in ran and (rows == "n" or _lib.AMOS_PIPE_PATCH8 in ran)


def test_v4_times_every_runnable_mapping_class(gpu, tmp_path, capsys):
    # the convolution of the reference's tutorial (README.md:174-261): 20 feasible mappings
    A, B, Conv = conv2d(16, 64, 14, 14, 64, 3, 3, 1, 1, 1)
    opt = at.MeasureOptions(target="hip", number=3, min_repeat_ms=2)
    res = at.auto_tensorize_v4(at.compute_dag_from_tensors([Conv]), "hip", "conv.log", opt,
                               schedule_log_dir=str(tmp_path / "logs"), trials=60, repeat_rounds=1,
                               search_group_size=1)
    out = capsys.readouterr().out
    assert res.defined()
    assert "Num mapping: 20" in out and "Num runnable mapping: 11" in out
    assert (res.num_runnable_mappings, res.num_feasible_mappings) == (11, 20)
    timed = set()
    for line in out.splitlines():
        if line.startswith("Round 1, Match 1, Mapping"):
            value = float(line.split(": ")[1].split("/")[0])
            if value > 1.0:   # (1 / seconds of the mapping's best schedule; 1e-10 = nothing ran)
                timed.add(line.split('"vmap": ')[1].split("]")[0])
    assert len(timed) == 11, out[-3000:]
    # the winner runs and is right
    sch, args = at.get_schedule(res.sch_app, res.params)
    func = tvm.build(sch, args, "hip")
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, [int(s) for s in A.shape]).astype(np.float16)
    b = rng.uniform(-1, 1, [int(s) for s in B.shape]).astype(np.float16)
    ctx = tvm.context("hip", 0)
    y = tvm.nd.array(np.zeros([int(s) for s in Conv.shape], dtype=np.float32), ctx)
    func(tvm.nd.array(a, ctx), tvm.nd.array(b, ctx), y)
    mx, mean = co.rel_errors(y.asnumpy(), co.lib_conv2d(a, b, "float16", 1, 1, 1, acc="float64"))
    assert mx <= 1e-2 and mean <= 1e-3
