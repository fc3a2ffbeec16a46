"""Matcher, mapping enumeration, policies, lowering and the log format, pinned against what the
reference's README prints for its conv2d tutorial (tests/golden/readme_conv2d_mappings.json),
a tuning log it ships, and brute-force evaluation of the TE computes.  No GPU needed."""
import json
import os

import numpy as np
import pytest

from amos_amd import _lib, te
import amos_amd.tvm as tvm
from amos_amd.te import tir
from amos_amd import auto_tensorize as at
from amos_amd.auto_tensorize import hw_abs_dag as dagmod
from amos_amd.auto_tensorize.hw_abstraction import MFMABase, register_abstraction
from oracle import cpu_oracle as co
from oracle import te_interp

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def conv2d(N, C, H, W, K, R, S, stride, padding, dilation, dtype="float16", out_dtype="float32", exact_int=False):
    """the tutorial's compute (reference: README.md:131-165)"""
    kH, kW = (R - 1) * dilation + 1, (S - 1) * dilation + 1
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=dtype, name="A")
    B = te.placeholder([K, C, R, S], dtype=dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    rc = te.reduce_axis([0, C], name="rc")
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - kH) // stride + 1, (pW - kW) // stride + 1

    def body(n, k, p, q):
        a = Pad[n, rc, p * stride + rr * dilation, q * stride + rs * dilation]
        b = B[k, rc, rr, rs]
        prod = a.astype(out_dtype) * b.astype(out_dtype) if exact_int else (a * b).astype(out_dtype)
        return te.sum(prod, axis=[rc, rr, rs])

    Conv = te.compute([N, K, P, Q], body, name="Conv")
    return A, B, Conv


def gemm(M, N, K, dtype="float16", out="float32", ta=False, tb=False, batch=None):
    pre = [batch] if batch else []
    A = te.placeholder(pre + ([K, M] if ta else [M, K]), dtype=dtype, name="A")
    B = te.placeholder(pre + ([N, K] if tb else [K, N]), dtype=dtype, name="B")
    rk = te.reduce_axis([0, K], name="k")

    def la(b, i): return A[tuple(b) + ((rk, i) if ta else (i, rk))]
    def lb(b, j): return B[tuple(b) + ((j, rk) if tb else (rk, j))]
    if batch:
        C = te.compute([batch, M, N], lambda b, i, j: te.sum((la([b], i) * lb([b], j)).astype(out), axis=rk), name="C")
    else:
        C = te.compute([M, N], lambda i, j: te.sum((la([], i) * lb([], j)).astype(out), axis=rk), name="C")
    return A, B, C


# ---- a test-only intrinsic with the reference's Tensor Core shapes, to replay the README ----------
@pytest.fixture(scope="module")
def wmma_like_target():
    @register_abstraction("readme_test", "wmma_fp16_fp32::mma", override=True)
    class Mma(MFMABase):
        in_dtype, out_dtype = "float16", "float32"

    class WmmaLike(dagmod.MFMADag):
        mnemonic = "wmma_fp16_fp32"
        mma_mnemonic = "wmma_fp16_fp32::mma"
        shape_keys = ("16x16x16", "32x8x16", "8x32x16")

        def __init__(self):
            self.mma = Mma()

    dagmod.register_hw_abs_dag("readme_test", "wmma_fp16_fp32", override=True)(WmmaLike)
    yield "readme_test"
    dagmod.HW_ABS_DAG_REGISTER_POOL.remove("readme_test", "wmma_fp16_fp32")


def names(axis_map):
    return {k.var.name: [t.var.name for t in v] for k, v in axis_map.items()}


def test_readme_conv2d_matchings_and_mappings(wmma_like_target, capsys):
    gold = json.load(open(os.path.join(GOLDEN, "readme_conv2d_mappings.json")))
    L = gold["layer"]
    A, B, Conv = conv2d(L["N"], L["C"], L["H"], L["W"], L["K"], L["R"], L["S"], L["stride"], L["padding"], L["dilation"])
    dag = at.compute_dag_from_tensors([Conv])
    assert [op.name for op in dag.op_lst] == ["Pad", "Conv"]
    assert [t.name for t in dag.get_inputs()] == ["A", "B"]
    matches = at.get_match_results(dag, wmma_like_target)
    assert [str(m) for m in matches] == gold["matchings"]
    for m in matches:
        assert names(m.axis_map) == gold["axis_map"]
        assert list(m.main_op_map.values())[0].name == "Conv"
    chosen, record = at.all_fit(matches)
    assert str(chosen) == gold["selected"]
    assert record.vmap_choice[0] == [1] * 7
    mappings = at.MappingGenerator(chosen).get_all()
    assert len(mappings) == gold["num_mappings"]
    assert "Totally 35 different mappings for this matching" in capsys.readouterr().out
    app = at.MappingApplier(chosen, strict=True)
    infeasible, feasible = [], []
    for r in mappings:
        try:
            app.apply(r)
            feasible.append(list(r.vmap_choice[0]))
        except RuntimeError:
            infeasible.append(list(r.vmap_choice[0]))
    assert infeasible == gold["infeasible"]
    assert len(feasible) == gold["num_feasible"]
    assert feasible[0] == gold["first_explored_mapping"]
    assert str(mappings[0]) == '{"vmap": [[0, 0, 0, 0, 0, 0, 1], -1]}' and mappings[1].as_key() == "(0,0,0,0,0,1,0)"
    # non-strict mode accepts every mapping and flags padding instead
    lax = at.MappingApplier(chosen, strict=False)
    assert all(lax.apply(r).need_padding == (list(r.vmap_choice[0]) in infeasible) for r in mappings)
    # trial budget of the tutorial run: 1200 trials, 10 rounds, 1 matching, 20 equal weights
    t = gold["trials"]
    assert t["total"] // t["rounds"] // 1 == t["per_matching"]
    assert int(np.ceil(t["per_matching"] * (1.0 / gold["num_feasible"]))) == t["per_mapping"]


def test_mfma_registry_and_matches():
    keys = [c().get_name() for c in at.query_hw_abs_dag("hip")]
    assert keys == ["mfma_f16_f32", "mfma_bf16_f32", "mfma_i8_i32", "mfma_i8_i32_wrapped_spelling"]
    assert [c().get_name() for c in at.query_hw_abs_dag("rocm")] == keys
    assert at.query_hw_abs_dag("cuda") == []
    A, B, C = gemm(64, 48, 32)
    ms = at.get_match_results(at.compute_dag_from_tensors([C]), "hip")
    assert [str(m) for m in ms] == ["MatchResult(hw_abs_dag:mfma_f16_f32, compute:%s, shape:%s)" % (c, s)
                                    for c in ("nnn", "ntn", "tnn", "ttn") for s in ("32x32x16", "16x16x32")]
    assert names(ms[0].axis_map) == {"i": ["i"], "j": ["j"], "rk": ["k"]}
    # bf16 and int8 computes reach their own DAGs only
    _, _, Cb = gemm(64, 48, 32, dtype="bfloat16")
    assert {m.hw_abs_dag.get_name() for m in at.get_match_results(at.compute_dag_from_tensors([Cb]), "hip")} == {"mfma_bf16_f32"}
    _, _, Ci = gemm(64, 48, 32, dtype="int8", out="int32")
    assert {m.hw_abs_dag.get_name() for m in at.get_match_results(at.compute_dag_from_tensors([Ci]), "hip")} == \
        {"mfma_i8_i32_wrapped_spelling"}
    _, _, Conv = conv2d(2, 16, 8, 8, 16, 3, 3, 1, 1, 1, dtype="int8", out_dtype="int32", exact_int=True)
    assert {m.hw_abs_dag.get_name() for m in at.get_match_results(at.compute_dag_from_tensors([Conv]), "hip")} == {"mfma_i8_i32"}


def test_batched_gemm_batch_axis_is_a_time_loop():
    A, B, C = gemm(32, 32, 64, tb=True, batch=6)
    ms = at.get_match_results(at.compute_dag_from_tensors([C]), "hip")
    assert names(ms[0].axis_map) == {"i": ["i"], "j": ["j"], "rk": ["k"]}
    state = at.MappingApplier(ms[0]).apply(at.MappingGenerator(ms[0], verbose_init=False).get_all()[0])
    assert [a.var.name for a in state.time_loops] == ["b"]


def test_conv3d_has_13_match_points():
    N, C, D, H, W, K, T, R, S = 2, 16, 6, 8, 8, 16, 3, 3, 3
    A = te.placeholder([N, C, D, H, W], dtype="float16", name="A")
    Wt = te.placeholder([K, C, T, R, S], dtype="float16", name="W")
    rc, rd, rr, rs = (te.reduce_axis([0, e], name=n) for e, n in ((C, "rc"), (T, "rd"), (R, "rr"), (S, "rs")))
    Y = te.compute([N, K, D - 2, H - 2, W - 2], lambda n, k, d, p, q: te.sum(
        (A[n, rc, d + rd, p + rr, q + rs] * Wt[k, rc, rd, rr, rs]).astype("float32"), axis=[rc, rd, rr, rs]), name="Y")
    m = at.get_match_results(at.compute_dag_from_tensors([Y]), "hip")[0]
    nm = names(m.axis_map)
    pts = set(zip(nm["i"], nm["j"], nm["rk"]))
    want = {(i, "k", r) for i in "ndpq" for r in ("rc", "rd", "rr", "rs")} - {("d", "k", "rd"), ("p", "k", "rr"), ("q", "k", "rs")}
    assert len(nm["i"]) == 13 and pts == want
    low = at.lower_main_op(Y.op)
    assert low.kind == "conv3d" and low.attrs["stride"] == [1, 1, 1] and low.attrs["pad"] == [0, 0, 0]


def test_enumeration_rule_above_15_points():
    """more than 15 points: single points whose extents equal the intrinsic's, plus all ones"""
    import ctypes
    n_points, n_axes = 16, 3
    pts = []
    for p in range(n_points):
        pts += [p, 16, 17]                 # i differs per point, j and rk shared
    ext = [32 if p in (3, 9) else 8 for p in range(16)] + [32, 16]
    flat = (ctypes.c_int32 * len(pts))(*pts)
    text = (ctypes.c_int64 * len(ext))(*ext)
    iext = (ctypes.c_int64 * 3)(32, 32, 16)
    bits = (ctypes.c_uint8 * (32 * n_points))()
    feas = (ctypes.c_uint8 * 32)()
    n = _lib.load().amos_enumerate_mappings(n_points, n_axes, flat, text, iext, bits, feas, 32)
    rows = [[bits[m * n_points + i] for i in range(n_points)] for m in range(n)]
    assert n == 3 and rows[0] == [int(i == 3) for i in range(16)] and rows[1] == [int(i == 9) for i in range(16)]
    assert rows[2] == [1] * 16 and list(feas[:3]) == [1, 1, 1]


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_lowered_gemm_means_what_the_compute_says(ta, tb, dtype):
    M, N, K = 5, 4, 6
    A, B, C = gemm(M, N, K, dtype=dtype, out="int32" if dtype == "int8" else "float32", ta=ta, tb=tb)
    low = at.lower_main_op(C.op)
    assert low.kind == "gemm" and (low.attrs["trans_a"], low.attrs["trans_b"]) == (ta, tb)
    assert (low.desc.M, low.desc.N, low.desc.K, low.desc.lda, low.desc.ldb, low.desc.ldc) == \
        (M, N, K, M if ta else K, K if tb else N, N)
    rng = np.random.default_rng(1)
    a = rng.integers(-5, 6, [int(s) for s in A.shape]).astype(np.int8 if dtype == "int8" else np.float16)
    b = rng.integers(-5, 6, [int(s) for s in B.shape]).astype(a.dtype)
    want = te_interp.evaluate(C, {"A": a, "B": b})
    feeds = {low.inputs[0].name: a if low.inputs[0] is A else b, low.inputs[1].name: b if low.inputs[1] is B else a}
    got = co.te_literal_gemm(feeds[low.inputs[0].name], feeds[low.inputs[1].name], dtype,
                             bool(low.attrs["trans_a"]), bool(low.attrs["trans_b"]), mode="exact")
    assert np.array_equal(got, want)


def test_lowered_gemm_with_swapped_operands():
    """C[i, j] = sum_k B[k, j] * A[i, k]: the row operand is the second factor"""
    M, N, K = 4, 3, 5
    A = te.placeholder([M, K], dtype="float16", name="A")
    B = te.placeholder([K, N], dtype="float16", name="B")
    rk = te.reduce_axis([0, K], name="k")
    C = te.compute([M, N], lambda i, j: te.sum((B[rk, j] * A[i, rk]).astype("float32"), axis=rk), name="C")
    low = at.lower_main_op(C.op)
    assert [t.name for t in low.inputs] == ["A", "B"] and (low.attrs["trans_a"], low.attrs["trans_b"]) == (0, 0)


CONV_LOWER_CASES = [(2, 3, 7, 6, 4, 3, 3, 1, 1, 1), (1, 2, 9, 9, 3, 3, 3, 2, 1, 1), (1, 2, 9, 8, 2, 3, 3, 1, 2, 2),
                    (1, 3, 6, 6, 2, 1, 1, 1, 0, 1), (1, 2, 8, 8, 2, 3, 3, 2, 0, 1)]


@pytest.mark.parametrize("case", CONV_LOWER_CASES)
def test_lowered_conv2d_means_what_the_compute_says(case):
    N, C, H, W, K, R, S, st, pd, dl = case
    A, B, Conv = conv2d(N, C, H, W, K, R, S, st, pd, dl, dtype="int8", out_dtype="int32", exact_int=True)
    low = at.lower_main_op(Conv.op)
    assert low.kind == "conv2d" and low.attrs["stride"] == [st, st] and low.attrs["pad"] == [pd, pd] and low.attrs["dil"] == [dl, dl]
    assert [t.name for t in low.inputs] == ["A", "B"]
    rng = np.random.default_rng(2)
    a = rng.integers(-9, 10, (N, C, H, W)).astype(np.int8)
    b = rng.integers(-9, 10, (K, C, R, S)).astype(np.int8)
    want = te_interp.evaluate(Conv, {"A": a, "B": b})
    got = co.te_literal_conv2d(a, b, "int8", low.attrs["stride"], low.attrs["pad"], low.attrs["dil"], mode="exact")
    assert np.array_equal(got, want)


def conv2d_layout(N, C, H, W, K, R, S, stride, padding, dilation, layout, dtype="float16", out_dtype="float32",
                  exact_int=False):
    """the reference's conv2d in its nhwc and hwnc spellings (benchmark/amos/mapping_conv2d_tensorcore.py:43-104)"""
    kH, kW = (R - 1) * dilation + 1, (S - 1) * dilation + 1
    pH, pW = H + 2 * padding, W + 2 * padding
    P, Q = (pH - kH) // stride + 1, (pW - kW) // stride + 1
    rc = te.reduce_axis([0, C], name="rc")
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    B = te.placeholder([R, S, C, K], dtype=dtype, name="B")

    def mul(a, b):
        return a.astype(out_dtype) * b.astype(out_dtype) if exact_int else (a * b).astype(out_dtype)

    inside = lambda h, w: tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W)
    if layout == "nhwc":
        A = te.placeholder([N, H, W, C], dtype=dtype, name="A")
        Pad = te.compute([N, pH, pW, C], lambda n, h, w, c: tir.if_then_else(
            inside(h, w), A[n, h - padding, w - padding, c], tir.const(0.0, A.dtype)), name="Pad")
        Conv = te.compute([N, P, Q, K], lambda n, p, q, k: te.sum(
            mul(Pad[n, p * stride + rr * dilation, q * stride + rs * dilation, rc], B[rr, rs, rc, k]),
            axis=[rr, rs, rc]), name="Conv")
    else:
        A = te.placeholder([H, W, N, C], dtype=dtype, name="A")
        Pad = te.compute([pH, pW, N, C], lambda h, w, n, c: tir.if_then_else(
            inside(h, w), A[h - padding, w - padding, n, c], tir.const(0.0, A.dtype)), name="Pad")
        Conv = te.compute([P, Q, N, K], lambda p, q, n, k: te.sum(
            mul(Pad[p * stride + rr * dilation, q * stride + rs * dilation, n, rc], B[rr, rs, rc, k]),
            axis=[rr, rs, rc]), name="Conv")
    return A, B, Conv


def to_nchw(a, b, layout):
    """operands stored in `layout` -> NCHW activations, KCRS weights"""
    return (np.transpose(a, (0, 3, 1, 2) if layout == "nhwc" else (2, 3, 0, 1)), np.transpose(b, (3, 2, 0, 1)))


def from_nkpq(y, layout):
    return np.transpose(y, (0, 2, 3, 1) if layout == "nhwc" else (2, 3, 0, 1))


@pytest.mark.parametrize("layout", ["nhwc", "hwnc"])
@pytest.mark.parametrize("case", CONV_LOWER_CASES)
def test_lowered_conv2d_layouts_mean_what_the_compute_says(case, layout):
    N, C, H, W, K, R, S, st, pd, dl = case
    A, B, Conv = conv2d_layout(N, C, H, W, K, R, S, st, pd, dl, layout, dtype="int8", out_dtype="int32",
                               exact_int=True)
    assert len(at.get_match_results(at.compute_dag_from_tensors([Conv]), "hip")) > 0
    low = at.lower_main_op(Conv.op)
    assert low.kind == "conv2d" and low.attrs["layout"] == layout and low.desc.layout == _lib.LAYOUT_CODE[layout]
    assert low.attrs["stride"] == [st, st] and low.attrs["pad"] == [pd, pd] and low.attrs["dil"] == [dl, dl]
    assert (low.desc.N, low.desc.C, low.desc.H, low.desc.W, low.desc.K, low.desc.R, low.desc.S) == (N, C, H, W, K, R, S)
    assert [t.name for t in low.inputs] == ["A", "B"]
    rng = np.random.default_rng(2)
    a = rng.integers(-9, 10, [int(e) for e in A.shape]).astype(np.int8)
    b = rng.integers(-9, 10, (R, S, C, K)).astype(np.int8)
    want = te_interp.evaluate(Conv, {"A": a, "B": b})
    an, bn = to_nchw(a, b, layout)
    got = co.te_literal_conv2d(np.ascontiguousarray(an), np.ascontiguousarray(bn), "int8", low.attrs["stride"],
                               low.attrs["pad"], low.attrs["dil"], mode="exact")
    assert np.array_equal(from_nkpq(got, layout), want)


def transposed_conv2d(N, C, H, W, K, kernel_size, stride, padding, output_padding, dilation,
                      in_dtype="float16", out_dtype="float32", exact_int=False):
    """the reference's transposed convolution: zero expansion, one-sided padding, a stride-1
    convolution with the window flipped (benchmark/amos/mapping_transposedconv2d_tensorcore.py:7-102)"""
    A = te.placeholder([N, K, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, C, kernel_size, kernel_size], dtype=in_dtype, name="B")
    k_h = k_w = kernel_size
    He, We = (H - 1) * stride + 1, (W - 1) * stride + 1
    expanded = te.compute([N, K, He, We], lambda b, c, h, w: te.if_then_else(
        te.all(h % stride == 0, w % stride == 0), A[b, c, h // stride, w // stride], tir.const(0, in_dtype)),
        name="expanded")
    kernel_h, kernel_w = (k_h - 1) * dilation + 1, (k_w - 1) * dilation + 1
    p0, p1 = kernel_h - 1 - padding, kernel_h - 1 - padding + output_padding
    q0, q1 = kernel_w - 1 - padding, kernel_w - 1 - padding + output_padding
    padded = te.compute([N, K, He + p0 + p1, We + q0 + q1], lambda b, c, h, w: te.if_then_else(
        te.all(h >= p0, h < He + p0, w >= q0, w < We + q0), expanded[b, c, h - p0, w - q0], tir.const(0, in_dtype)),
        name="Padding")
    out_h = (H - 1) * stride - 2 * padding + kernel_h + output_padding
    out_w = (W - 1) * stride - 2 * padding + kernel_w + output_padding
    rc = te.reduce_axis((0, K), name="rc")
    rh = te.reduce_axis((0, k_h), name="rh")
    rw = te.reduce_axis((0, k_w), name="rw")

    def body(b, c, h, w):
        x, wt = padded[b, rc, h + rh * dilation, w + rw * dilation], B[rc, c, k_h - rh - 1, k_w - rw - 1]
        prod = x.astype(out_dtype) * wt.astype(out_dtype) if exact_int else (x * wt).astype(out_dtype)
        return te.sum(prod, axis=[rc, rw, rh])

    output = te.compute((N, C, out_h, out_w), body, name="output")
    return [A, B, output]


def apply_view(view, src):
    """numpy meaning of a lowering.OperandView"""
    off = np.zeros(view.shape, dtype=np.int64)
    ok = np.ones(view.shape, dtype=bool)
    for d, table in enumerate(view.tables):
        t = np.asarray(table, dtype=np.int64).reshape([-1 if k == d else 1 for k in range(len(view.shape))])
        ok &= t >= 0
        off += np.maximum(t, 0)
    return np.where(ok, src.reshape(-1)[off], 0).astype(src.dtype)


TRANSPOSED_CASES = [(2, 3, 5, 4, 6, 3, 2, 1, 1, 1), (1, 4, 6, 6, 2, 4, 2, 1, 0, 1), (1, 2, 4, 5, 3, 3, 1, 0, 0, 2),
                    (2, 2, 3, 3, 2, 2, 3, 0, 2, 1)]


@pytest.mark.parametrize("case", TRANSPOSED_CASES)
def test_transposed_conv_lowers_to_gathers_and_a_convolution(case):
    N, C, H, W, K, ks, st, pd, opd, dl = case
    A, B, Out = transposed_conv2d(N, C, H, W, K, ks, st, pd, opd, dl, "int8", "int32", exact_int=True)
    assert len(at.get_match_results(at.compute_dag_from_tensors([Out]), "hip")) > 0
    low = at.lower_main_op(Out.op)
    assert low.kind == "conv2d" and sorted(low.gathers) == [0, 1] and [t.name for t in low.inputs] == ["A", "B"]
    assert low.attrs["stride"] == [1, 1] and low.attrs["pad"] == [0, 0] and low.attrs["dil"] == [dl, dl]
    rng = np.random.default_rng(4)
    a = rng.integers(-9, 10, (N, K, H, W)).astype(np.int8)
    b = rng.integers(-9, 10, (K, C, ks, ks)).astype(np.int8)
    want = te_interp.evaluate(Out, {"A": a, "B": b})
    x, w = apply_view(low.gathers[0], a), apply_view(low.gathers[1], b)
    assert w.shape == (C, K, ks, ks) and np.array_equal(w, np.transpose(b, (1, 0, 2, 3))[:, :, ::-1, ::-1])
    got = co.te_literal_conv2d(x, w, "int8", [1, 1], [0, 0], [dl, dl], mode="exact")
    assert np.array_equal(got, want)
    # and the textbook definition: scatter every input element times the window into the output
    ref = np.zeros(want.shape, dtype=np.int64)
    for n in range(N):
        for k in range(K):
            for h in range(H):
                for ww in range(W):
                    for r in range(ks):
                        for s_ in range(ks):
                            oh, ow = h * st - pd + r * dl, ww * st - pd + s_ * dl
                            if 0 <= oh < ref.shape[2] and 0 <= ow < ref.shape[3]:
                                ref[n, :, oh, ow] += int(a[n, k, h, ww]) * b[k, :, r, s_].astype(np.int64)
    assert np.array_equal(ref, want)


def mean(N, C, H, W, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_mean_tensorcore.py:7-25"""
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.compute([C, N * H * W], lambda i, j: A[j // (H * W), i, j % (H * W) // W, j % W], name="B")
    C_ = te.compute([N * H * W, 1], lambda i, j: tir.const(1.0 / (N * H * W), in_dtype), name="C")
    rk = te.reduce_axis([0, N * H * W], name="k")
    D = te.compute([C, 1], lambda i, j: te.sum((B[i, rk] * C_[rk, j]).astype(out_dtype), axis=rk), name="D")
    E = te.compute([C], lambda i: D[i, 0], name="E")
    return [A, B, E]


def scan(M, N, K, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_scan_tensorcore.py:7-21"""
    A = te.placeholder([M, K], dtype=in_dtype, name="A")
    B = te.compute([K, N], lambda i, j: tir.if_then_else(i > j, tir.const(0.0, in_dtype), tir.const(1.0, "float16")),
                   name="B")
    rk = te.reduce_axis([0, K], name="k")
    C = te.compute([M, N], lambda i, j: te.sum((A[i, rk] * B[rk, j]).astype(out_dtype), axis=rk), name="C")
    return [A, B, C]


def test_mean_and_scan_lower_to_gemm_with_computed_operands():
    rng = np.random.default_rng(6)
    # mean: the [C, N*H*W] view of A is gathered, the vector of 1/n is a constant
    N, C, H, W = 2, 5, 3, 4
    A, B, E = mean(N, C, H, W)
    dag = at.compute_dag_from_tensors([E])
    low = at.lower_main_op([op for op in dag.op_lst if op.reduce_axis][0], dag)
    assert low.kind == "gemm" and (low.attrs["M"], low.attrs["N"], low.attrs["K"]) == (C, 1, N * H * W)
    assert list(low.gathers) == [0] and list(low.constants) == [1] and low.output is E
    a = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float16)
    b = apply_view(low.gathers[0], a)
    assert np.array_equal(b, np.transpose(a, (1, 0, 2, 3)).reshape(C, -1))
    assert np.array_equal(low.constants[1], np.full((N * H * W, 1), np.float16(1.0 / (N * H * W))))
    want = te_interp.evaluate(E, {"A": a})
    got = co.te_literal_gemm(b, low.constants[1], "float16").reshape(-1)
    # (the loop nest rounds every product to fp16, the interpreter does not)
    assert np.allclose(got, want, atol=1e-3) and np.allclose(want, a.astype(np.float64).mean(axis=(0, 2, 3)), atol=2e-3)
    # scan: the triangle of ones is a constant; row i of the result = prefix sums of row i of A
    M, Nn, K = 6, 7, 7
    A, B, Cc = scan(M, Nn, K)
    low = at.lower_main_op(Cc.op)
    assert low.kind == "gemm" and not low.gathers and list(low.constants) == [1]
    assert np.array_equal(low.constants[1], np.triu(np.ones((K, Nn), dtype=np.float16)))
    a = rng.integers(-4, 5, (M, K)).astype(np.float16)
    want = te_interp.evaluate(Cc, {"A": a})
    assert np.array_equal(want, np.cumsum(a.astype(np.float32), axis=1))


def test_no_kernel_for_other_layouts():
    # NHWC activations match the intrinsic but have no kernel
    N, H, W, C, K = 2, 6, 6, 8, 8
    A = te.placeholder([N, H, W, C], dtype="float16", name="A")
    B = te.placeholder([K, C, 3, 3], dtype="float16", name="B")
    rc, rr, rs = te.reduce_axis([0, C], "rc"), te.reduce_axis([0, 3], "rr"), te.reduce_axis([0, 3], "rs")
    Y = te.compute([N, K, H - 2, W - 2], lambda n, k, p, q: te.sum(
        (A[n, p + rr, q + rs, rc] * B[k, rc, rr, rs]).astype("float32"), axis=[rc, rr, rs]), name="Y")
    assert at.get_match_results(at.compute_dag_from_tensors([Y]), "hip")
    with pytest.raises(at.NoKernelError):
        at.lower_main_op(Y.op)
    # fp16 accumulate has no instruction
    _, _, C16 = gemm(32, 32, 32, out="float16")
    assert at.get_match_results(at.compute_dag_from_tensors([C16]), "hip") == []


def test_auto_tensorize_plumbing_config1_on_cpu(tmp_path, capsys):
    """fp16 GEMM 512^3: TE compute -> match -> mapping -> schedule object -> descriptor, no GPU;
    the CPU result of the same compute comes from the oracle"""
    A, B, C = gemm(512, 512, 512)
    dag = at.compute_dag_from_tensors([C])
    opt = at.MeasureOptions(target="hip", timeout=100, number=200, min_repeat_ms=500)
    res = at.auto_tensorize(dag, "hip", str(tmp_path / "gemm.log"), opt, trials=0)
    out = capsys.readouterr().out
    assert "Possible matchings:" in out and "Selected matching:" in out and "Axis mapping:" in out
    assert res.defined() and res.perf > 0 and opt.target == "hip"
    sch, args = at.get_schedule(res.sch_app, res.params)
    assert [t.name for t in args] == ["A", "B", "C"] and sch.lowered.kind == "gemm"
    cfg = res.params.to_config()
    assert _lib.load().amos_check_config(0, __import__("ctypes").byref(sch.lowered.desc), __import__("ctypes").byref(cfg), None, None) == 0
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, (512, 512)).astype(np.float16)
    b = rng.uniform(-1, 1, (512, 512)).astype(np.float16)
    lit = co.te_literal_gemm(a, b, "float16", threads=8)
    mx, mean = co.rel_errors(lit, co.lib_gemm(a, b, "float16", acc="float64"))
    assert mean < 1e-3
    with pytest.raises(RuntimeError):
        at.auto_tensorize(dag, "cuda", "", opt, trials=0)


def test_v4_pure_test_mode_lists_infeasible_mappings(tmp_path, capsys):
    A, B, Conv = conv2d(1, 128, 28, 28, 128, 3, 3, 1, 1, 1)
    opt = at.MeasureOptions(target="hip")
    res = at.auto_tensorize_v4(at.compute_dag_from_tensors([Conv]), "hip", "conv.log", opt,
                               schedule_log_dir=str(tmp_path / "logs"), trials=0)
    out = capsys.readouterr().out
    assert "Catch an infeasible mapping:" in out and "Pure testing mode..." in out and "Num mapping:" in out
    assert res.defined() and res.mapping is not None
    # the two mappings the kernel family realises: channels only on rk (patch staging), or all
    # reduce loops fused on rk (im2col staging); both put n, p, q on i
    # (the enumeration keeps the first bit vector of each distinct set of fused loops)
    m = at.all_fit(at.get_match_results(at.compute_dag_from_tensors([Conv]), "hip"))[0]
    fused = {k: set(v) for k, v in at.MappingApplier(m, strict=False).apply(res.mapping).fused_names().items()}
    assert fused["i"] == {"n", "p", "q"} and fused["j"] == {"k"}
    assert fused["rk"] in ({"rc"}, {"rc", "rr", "rs"})


@pytest.mark.parametrize("rows", ["nq", "np", "n", "npq+s", "nq+s", "npq+r", "np+r"])
@pytest.mark.parametrize("case", [(3, 4, 7, 9, 5, 1, 1, 1), (2, 3, 8, 6, 4, 2, 1, 1), (2, 2, 9, 9, 3, 1, 2, 2), (1, 5, 6, 7, 2, 2, 2, 1), (2, 3, 5, 8, 6, 1, 0, 1)])
def test_remapped_convolutions_mean_the_same(rows, case):
    """lowering.remap_conv2d_rows on the CPU: the gathered activations and weights, convolved as the
    sub-convolution's descriptor says (NHWC, its window, strides and paddings) and gathered back
    through out_view, are the original convolution -- for every class of rows and folded window
    loop, with strides, padding and dilation (int8: exact)"""
    from amos_amd.auto_tensorize.lowering import lower_main_op, remap_conv2d_rows
    N, C, H, W, K, st, pd, dl = case
    A, B, Conv = conv2d(N, C, H, W, K, 3, 3, st, pd, dl, dtype="int8", out_dtype="int32", exact_int=True)
    dag = at.compute_dag_from_tensors([Conv])
    main_op = [op for op in dag.op_lst if op.reduce_axis][0]
    low = remap_conv2d_rows(lower_main_op(main_op, dag), rows)
    rng = np.random.default_rng(7)
    a = rng.integers(-9, 10, (N, C, H, W)).astype(np.int8)
    b = rng.integers(-9, 10, (K, C, 3, 3)).astype(np.int8)
    want = co.lib_conv2d(a, b, "int8", st, pd, dl)
    d = low.desc
    assert d.layout == _lib.LAYOUT_CODE["nhwc"]
    # the kernel's operands: activations [N][H][W][C], weights [R][S][C][K] of the sub-convolution
    x = apply_view(low.gathers[0], a).reshape(d.N, d.H, d.W, d.C)
    w = apply_view(low.gathers[1], b).reshape(d.R, d.S, d.C, d.K)
    y = co.lib_conv2d(np.transpose(x, (0, 3, 1, 2)), np.transpose(w, (3, 2, 0, 1)), "int8", (d.stride_h, d.stride_w),
                      (d.pad_h, d.pad_w), (d.dil_h, d.dil_w))
    kernel_out = np.ascontiguousarray(np.transpose(y, (0, 2, 3, 1)))      # what the kernel writes: NHWC
    assert kernel_out.size == want.size
    got = apply_view(low.out_view, kernel_out)
    assert got.shape == want.shape and np.array_equal(got, want)


def test_v4_keeps_the_kernels_without_a_pipeline_value(tmp_path):
    """the network dispatcher tunes every layer through auto_tensorize_v4: the mapping the kernels
    implement as it is must keep the mapper's own choice among its candidates -- the depthwise,
    few-channel and skinny kernels and the direct-to-LDS GEMM are reached through it alone"""
    import contextlib
    import io
    from amos_amd import ops
    from amos_amd.auto_tensorize import network as net
    want = {"depthwise 3x3/1 32 @112": "amos_depthwise_conv", "conv 3x3/2 3->32 @224": "amos_conv_few_channels"}
    seen = {}
    for sg in list(net.mobilenet_v1(16))[:2] + list(net.mi_lstm(1))[:1] + list(net.bert_base(16))[:1]:
        with contextlib.redirect_stdout(io.StringIO()):
            res = at.auto_tensorize_v4(sg.dag, "hip", "x.log", at.MeasureOptions(target="hip"),
                                       schedule_log_dir=str(tmp_path / "logs"), trials=0, transform_strict=False)
        assert res.defined(), sg.note
        low = res.sch_gen.lowered
        seen[sg.note] = ops.kernel_name(low.op_code, low.desc, res.params.to_config())
    for note, kernel in want.items():
        assert kernel in seen[note], seen
    assert any("amos_skinny_gemm" in k for k in seen.values()) and any("amos_gemm_tn" in k for k in seen.values()), seen


def test_default_convolution_kernels():
    """what the mapper's model picks for the benchmark convolutions and a few network layers (the
    plan is host code: no GPU needed): the NCDHW-direct kernel with the weights read as they are
    where the packing launch would cost more than the transposes, packed where it would not, 16-byte
    patch loads where a channel plane is whole 16-byte runs; for the int8 benchmark shape the
    128-row workgroups (two halves of 64 output channels on one patch: its tiles in one round of
    the compute units)"""
    import torch
    from amos_amd import _lib, ops

    def name(xs, ws, dt=torch.float16, op=_lib.AMOS_OP_CONV2D, pad=(0, 1, 1)):
        return ops.kernel_name(op, ops.conv_desc(xs, ws, dt, (1, 1, 1), pad, (1, 1, 1)))

    assert name((32, 256, 1, 14, 14), (256, 256, 1, 3, 3)) == "amos_conv_nchw<f16,64x128,8+4w,kcrs>"
    assert name((8, 64, 16, 56, 56), (64, 64, 3, 3, 3), op=_lib.AMOS_OP_CONV3D, pad=(1, 1, 1)) == \
        "amos_conv_nchw<f16,64x256,8+4w,packed,ld16>"
    assert name((64, 128, 1, 28, 28), (128, 128, 1, 3, 3), torch.int8) == "amos_conv_nchw<i8,2x64x256,8+4w,kcrs>"
    assert name((16, 64, 1, 56, 56), (64, 64, 1, 3, 3)) == "amos_conv_nchw<f16,64x256,8+4w,kcrs,ld16>"
    assert name((64, 512, 1, 14, 14), (512, 512, 1, 3, 3)) == "amos_conv_nchw<f16,2x64x256,8+4w,packed,pt2>"
    # a channel count that does not fill 64-byte chunks, a 5x5 window: not this kernel's
    assert not name((2, 24, 1, 14, 14), (40, 24, 1, 3, 3)).startswith("amos_conv_nchw")
    assert not name((4, 64, 1, 30, 30), (96, 64, 1, 5, 5), pad=(0, 2, 2)).startswith("amos_conv_nchw")


def test_log_format_and_reference_fixture(tmp_path):
    from amos_amd.auto_tensorize.schedule import KernelParams, read_log
    rows = read_log(os.path.join(GOLDEN, "a100_conv2d_1_256_14_14_256_3_3_mapping_0010010.log"))
    assert len(rows) == 13 and set(rows[0][0].keys()) >= {"inline", "vectorize", "spatial_factors", "reduce_factors"}
    best = max(v for _, v in rows)
    assert abs(1 / best * 1e3 - 0.049993) < 1e-5      # ms, the figure quoted for this layer
    A, B, C = gemm(256, 256, 256, tb=True)
    m = at.get_match_results(at.compute_dag_from_tensors([C]), "hip")[0]
    log = str(tmp_path / "t.log")
    gen = at.MI355XScheduleGenerator(m, None, log_file=log, verbose_init=False)
    gen.feedback(KernelParams(128, 128, 1, 0), 1 / 20e-6)
    gen.feedback(KernelParams(256, 256, 1, 0), 1 / 10e-6)
    gen.feedback(KernelParams(64, 64, 2, 1), 1 / 30e-6)
    lines = [json.loads(l) for l in open(log)]
    assert lines[1] == {"record": {"tile_i": 256, "tile_j": 256, "split_k": 1, "pipeline": 0}, "value": 1 / 10e-6}
    gen2 = at.MI355XScheduleGenerator(m, None, log_file=str(tmp_path / "u.log"), verbose_init=False)
    gen2.load_from_file(log)
    e = gen2.get_best_entry()
    assert e.record.to_json() == lines[1]["record"] and gen2.num_entries() == 3 and 1 / e.value == pytest.approx(10e-6)
    # every candidate the sweep proposes resolves to a compiled kernel instance
    cands = gen.candidates()
    assert len(cands) > 8 and str(cands[0]) == str(KernelParams(256, 256, 1, 0)) or len(cands) > 8


def test_measure_options_defaults():
    o = at.MeasureOptions()
    assert (o.target, o.timeout, o.number, o.repeat, o.min_repeat_ms, o.dev_id) == ("llvm", 10, 100, 1, 150, 0)


def test_fragment_layout_is_a_bijection():
    from amos_amd.auto_tensorize.hw_abstraction import mfma_fragment_layout
    for key in ("32x32x16", "16x16x32", "32x32x32", "16x16x64"):
        m, n, k = (int(x) for x in key.split("x"))
        lay = mfma_fragment_layout(key)
        a = {lay["a"](l, e) for l in range(64) for e in range(lay["k_per_lane"])}
        d = {lay["d"](l, r) for l in range(64) for r in range(lay["acc_regs"])}
        assert a == {(i, kk) for i in range(m) for kk in range(k)}
        assert d == {(i, j) for i in range(m) for j in range(n)}


# ---- element-wise tail behind the main op (reference: tests/python/auto_tensorize/
# test_compute_transform_gemm.py:7-23, hw_abs_dag/cuda/wmma_fp16_bias.py) ---------------------
def _gemm_with_tail(M, N, K, d_dtype="float32", tail="add"):
    A = tvm.te.placeholder([M, K], dtype="float16", name="A")
    B = tvm.te.placeholder([K, N], dtype="float16", name="B")
    tk = tvm.te.reduce_axis([0, K], name="tk")
    C = tvm.te.compute([M, N], lambda ti, tj: tvm.te.sum((A[ti, tk] * B[tk, tj]).astype("float32"), axis=tk),
                       name="C")
    D = tvm.te.placeholder([M, N], dtype=d_dtype, name="D")

    def body(si, sj):
        d = D[si, sj] if d_dtype == "float32" else D[si, sj].astype("float32")
        return C[si, sj] + d if tail == "add" else C[si, sj] * d
    E = tvm.te.compute([M, N], body, name="E")
    return A, B, D, E


def test_tail_addition_is_fused_at_lowering():
    from amos_amd.auto_tensorize.lowering import NoKernelError, lower_main_op
    for d_dtype in ("float32", "float16", "bfloat16"):
        A, B, D, E = _gemm_with_tail(128, 128, 128, d_dtype)
        dag = at.compute_dag_from_tensors([E])
        assert [op.name for op in dag.op_lst] == ["C", "E"]
        # the tail does not change what matches: the main op alone, as for the plain GEMM
        results = at.get_match_results(dag, "hip")
        assert len(results) == 8 and all(list(r.main_op_map.values())[0] is dag.op_lst[0] for r in results)
        low = lower_main_op(dag.op_lst[0], dag)
        assert low.kind == "gemm" and low.add_input is D and low.output is E
        assert [t.name for t in dag.get_inputs()] == ["A", "B", "D"]
    A, B, D, E = _gemm_with_tail(128, 128, 128, tail="mul")
    dag = at.compute_dag_from_tensors([E])
    with pytest.raises(NoKernelError, match="not an element-wise addition"):
        lower_main_op(dag.op_lst[0], dag)
    A, B, D, E = _gemm_with_tail(128, 128, 128, "int32")
    with pytest.raises(NoKernelError, match="cannot add"):
        dag = at.compute_dag_from_tensors([E])
        lower_main_op(dag.op_lst[0], dag)


def test_bias_dag_is_unregistered_and_has_two_ops():
    dag_cls = at.MFMAFp16Fp32Bias
    assert dag_cls not in at.query_hw_abs_dag("hip")
    hw = dag_cls()
    assert hw.get_name() == "mfma_f16_f32_bias" and hw.anchor_point == "bias"
    assert hw.edges["bias"] == ["mma", "load_bias"] and hw.edges["store"] == ["bias"]
    intrin_dag, main = hw.get_effective_compute_dag("nnn", "32x32x16")
    assert len(intrin_dag.op_lst) == 2 and intrin_dag.op_lst[0] is main[0].op
    # the mapping the reference's test4 states by hand: main op <-> C, element-wise op <-> E
    A, B, D, E = _gemm_with_tail(128, 128, 128, "float16")
    target = at.compute_dag_from_tensors([E])
    main_op_map = {intrin_dag.op_lst[0]: target.op_lst[0]}
    elem_op_map = {intrin_dag.op_lst[1]: target.op_lst[1]}
    assert at.intrinsic_match(target.op_lst[0], intrin_dag.op_lst[0])
    assert len(main_op_map) == 1 and len(elem_op_map) == 1


# ---- more operators through the same lowering (reference: benchmark/amos/mapping_gemv_tensorcore.py:7-16,
# mapping_batchedfc_tensorcore.py:7-37, mapping_conv1d_tensorcore.py:7-42) --------------------------
def gemv(M, K, in_dtype="float16", out_dtype="float32"):
    A = te.placeholder([M, K], dtype=in_dtype, name="A")
    B = te.placeholder([K, 1], dtype=in_dtype, name="B")
    rk = te.reduce_axis([0, K], name="k")
    C = te.compute([M, 1], lambda i, j: te.sum((A[i, rk] * B[rk, j]).astype(out_dtype), axis=rk), name="C")
    D = te.compute([M], lambda i: C[i, 0], name="D")
    return A, B, D


def batched_fc(N, I, O, groups, in_dtype="float16", out_dtype="float32"):
    cpg, ocpg = I // groups, O // groups
    A = te.placeholder([N, I], dtype=in_dtype, name="A")
    B = te.placeholder([O, cpg], dtype=in_dtype, name="B")
    A_reshaped = te.compute([N, groups, cpg], lambda n, c_o, c_i: A[n, c_o * cpg + c_i])
    B_reshaped = te.compute([groups, ocpg, cpg], lambda k_o, k_i, c: B[k_o * ocpg + k_i, c])
    rc = te.reduce_axis([0, cpg], name="rc")
    BFC = te.compute([N, groups, ocpg], lambda n, k_o, k_i: te.sum(
        (A_reshaped[n, k_o, rc] * B_reshaped[k_o, k_i, rc]).astype(out_dtype), axis=[rc]), name="BatchedFC")
    return A, B, BFC


def conv1d(N, C, L, K, KL, stride, padding, dilation, in_dtype="float16", out_dtype="float32"):
    A = te.placeholder([N, C, L], dtype=in_dtype, name="A")
    B = te.placeholder([K, C, KL], dtype=in_dtype, name="B")
    out_len = (L + 2 * padding - dilation * (KL - 1) - 1) // stride + 1
    rc = te.reduce_axis((0, C), name="rc")
    rl = te.reduce_axis((0, KL), name="rl")
    padded = te.compute((N, C, L + 2 * padding), lambda b, c, l: tir.if_then_else(
        tir.all(l >= padding, l < L + padding), A[b, c, l - padding], tir.const(0, A.dtype)))
    conved = te.compute((N, K, out_len), lambda b, k, l: te.sum(
        (padded[b, rc, l * stride + rl * dilation] * B[k, rc, rl]).astype(out_dtype), axis=[rc, rl]))
    return A, B, conved


def gemm_from_desc(low, a, b):
    """what the C descriptor of a lowered GEMM / batched GEMM says, evaluated with numpy on the
    flat operand buffers (float64)"""
    d = low.desc.g if low.kind == "bgemm" else low.desc
    batch, sa, sb, sc = (low.desc.batch, low.desc.stride_a, low.desc.stride_b, low.desc.stride_c) \
        if low.kind == "bgemm" else (1, 0, 0, 0)
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    out = np.zeros(max(1, (batch - 1) * sc + (d.M - 1) * d.ldc + d.N))
    for g in range(batch):
        for i in range(d.M):
            for j in range(d.N):
                ai = [g * sa + (k * d.lda + i if d.trans_a else i * d.lda + k) for k in range(d.K)]
                bi = [g * sb + (j * d.ldb + k if d.trans_b else k * d.ldb + j) for k in range(d.K)]
                out[g * sc + i * d.ldc + j] = float(np.dot(a[ai], b[bi]))
    return out


@pytest.mark.parametrize("build", [lambda: gemv(24, 40), lambda: batched_fc(6, 32, 24, 4),
                                   lambda: gemm(20, 12, 16, ta=True, tb=True, batch=3)])
def test_strided_gemm_lowering_keeps_the_meaning(build):
    from amos_amd.auto_tensorize.lowering import lower_main_op
    A, B, Out = build()
    dag = at.compute_dag_from_tensors([Out])
    main = [op for op in dag.op_lst if op.reduce_axis][0]
    low = lower_main_op(main, dag)
    assert low.kind in ("gemm", "bgemm") and [t.name for t in low.inputs] == ["A", "B"] and low.output is Out
    rng = np.random.default_rng(3)
    a = rng.integers(-4, 5, [int(s) for s in A.shape]).astype(np.float64)
    b = rng.integers(-4, 5, [int(s) for s in B.shape]).astype(np.float64)
    want = te_interp.evaluate(Out, {"A": a, "B": b})
    got = gemm_from_desc(low, a, b)
    assert got.size == want.size and np.array_equal(got, want.ravel())


def test_gemv_and_batched_fc_descriptors():
    from amos_amd.auto_tensorize.lowering import lower_main_op
    A, B, D = gemv(256, 512)
    dag = at.compute_dag_from_tensors([D])
    low = lower_main_op(dag.op_lst[0], dag)
    g = low.desc
    assert (low.kind, g.M, g.N, g.K, g.trans_a, g.trans_b, g.lda, g.ldc) == ("gemm", 256, 1, 512, 0, 1, 512, 1)
    A, B, F = batched_fc(64, 512, 256, 4)
    dag = at.compute_dag_from_tensors([F])
    low = lower_main_op([op for op in dag.op_lst if op.reduce_axis][0], dag)
    d = low.desc
    assert (low.kind, d.batch, d.g.M, d.g.N, d.g.K) == ("bgemm", 4, 64, 64, 128)
    assert (d.g.trans_a, d.g.trans_b, d.g.lda, d.g.ldb, d.g.ldc) == (0, 1, 512, 128, 256)
    assert (d.stride_a, d.stride_b, d.stride_c) == (128, 64 * 128, 64)


def test_conv1d_lowers_to_conv2d_with_unit_height():
    from amos_amd.auto_tensorize.lowering import lower_main_op
    A, B, Out = conv1d(2, 16, 30, 8, 3, 2, 1, 2)
    dag = at.compute_dag_from_tensors([Out])
    low = lower_main_op([op for op in dag.op_lst if op.reduce_axis][0], dag)
    c = low.desc
    assert low.kind == "conv2d" and (c.N, c.C, c.D, c.H, c.W, c.K, c.T, c.R, c.S) == (2, 16, 1, 1, 30, 8, 1, 1, 3)
    assert (c.stride_h, c.stride_w, c.pad_h, c.pad_w, c.dil_h, c.dil_w) == (1, 2, 0, 1, 1, 2)
    rng = np.random.default_rng(4)
    a = rng.integers(-3, 4, (2, 16, 30)).astype(np.float64)
    b = rng.integers(-3, 4, (8, 16, 3)).astype(np.float64)
    want = te_interp.evaluate(Out, {"A": a, "B": b})
    ref = co.lib_conv2d(a[:, :, None, :].astype(np.float16), b[:, :, None, :].astype(np.float16), "float16",
                        (1, 2), (0, 1), (1, 2), acc="float64")
    assert np.array_equal(ref[:, :, 0, :], want)


def grouped_conv2d(N, C, H, W, K, R, S, stride, padding, groups, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_groupedconv2d_tensorcore.py:7-60"""
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, C // groups, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    A_reshaped = te.compute([N, groups, C // groups, pH, pW],
                            lambda n, c_o, c_i, r, s: Pad[n, c_o * (C // groups) + c_i, r, s])
    B_reshaped = te.compute([groups, K // groups, C // groups, R, S],
                            lambda k_o, k_i, c, r, s: B[k_o * (K // groups) + k_i, c, r, s])
    rc = te.reduce_axis([0, C // groups], name="rc")
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - R) // stride + 1, (pW - S) // stride + 1
    Conv = te.compute([N, groups, K // groups, P, Q], lambda n, k_o, k_i, p, q: te.sum(
        (A_reshaped[n, k_o, rc, p * stride + rr, q * stride + rs] * B_reshaped[k_o, k_i, rc, rr, rs]).astype(out_dtype),
        axis=[rc, rr, rs]), name="Conv")
    Reshaped = te.compute([N, K, P, Q], lambda n, k, p, q: Conv[n, k // (K // groups), k % (K // groups), p, q],
                          name="Reshaped")
    return A, B, Reshaped


def depthwise_conv2d(N, C, H, W, K, R, S, stride, padding, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_depthwiseconv2d_tensorcore.py:7-48"""
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    B_reshaped = te.compute([C, K // C, R, S], lambda k_o, k_i, r, s: B[k_o * (K // C) + k_i, r, s])
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - R) // stride + 1, (pW - S) // stride + 1
    Conv = te.compute([N, C, K // C, P, Q], lambda n, k_o, k_i, p, q: te.sum(
        (Pad[n, k_o, p * stride + rr, q * stride + rs] * B_reshaped[k_o, k_i, rr, rs]).astype(out_dtype),
        axis=[rr, rs]), name="Conv")
    Reshaped = te.compute([N, K, P, Q], lambda n, k, p, q: Conv[n, k // (K // C), k % (K // C), p, q],
                          name="Reshaped")
    return A, B, Reshaped


def grouped_conv_reference(a, b, stride, padding, groups):
    cg, kg = a.shape[1] // groups, b.shape[0] // groups
    b4 = b.reshape(b.shape[0], cg, b.shape[-2], b.shape[-1])
    return np.concatenate([co.lib_conv2d(np.ascontiguousarray(a[:, g * cg:(g + 1) * cg]).astype(np.float16),
                                         np.ascontiguousarray(b4[g * kg:(g + 1) * kg]).astype(np.float16),
                                         "float16", stride, padding, 1, acc="float64") for g in range(groups)], axis=1)


@pytest.mark.parametrize("build,groups", [(lambda: grouped_conv2d(2, 8, 6, 7, 12, 3, 3, 2, 1, 4), 4),
                                          (lambda: depthwise_conv2d(2, 6, 7, 6, 12, 3, 2, 1, 1), 6)])
def test_grouped_and_depthwise_conv_lowering(build, groups):
    from amos_amd.auto_tensorize.lowering import lower_main_op
    A, B, Out = build()
    dag = at.compute_dag_from_tensors([Out])
    main = [op for op in dag.op_lst if op.reduce_axis][0]
    assert at.get_match_results(dag, "hip")          # the 5-d main op matches the MFMA intrinsic
    low = lower_main_op(main, dag)
    assert low.kind == "conv2d" and low.desc.groups == groups and low.output is Out
    assert [t.name for t in low.inputs] == ["A", "B"]
    rng = np.random.default_rng(8)
    a = rng.integers(-3, 4, [int(s) for s in A.shape]).astype(np.float64)
    b = rng.integers(-3, 4, [int(s) for s in B.shape]).astype(np.float64)
    want = te_interp.evaluate(Out, {"A": a, "B": b})
    c = low.desc
    assert (c.N, c.C, c.H, c.W, c.K, c.R, c.S) == (a.shape[0], a.shape[1], a.shape[2], a.shape[3], b.shape[0],
                                                   b.shape[-2], b.shape[-1])
    got = grouped_conv_reference(a, b, (c.stride_h, c.stride_w), (c.pad_h, c.pad_w), groups)
    assert np.array_equal(got, want)


def test_other_networks_layer_lists():
    """layer counts and multiply-accumulate totals of the other networks the reference maps
    (benchmark/amos/mapping_{resnet50,mobilenetv1,bertbase}_tensorcore.py) against the published
    figures of the architectures: ResNet-50 4.09 G, MobileNet-V1 0.57 G multiply-accumulates at
    224x224; BERT-base at 512 tokens 12 x (4 x 512 x 768^2 + 2 x 512 x 768 x 3072 + 2 x 12 x 512^2 x 64)"""
    from amos_amd import auto_tensorize as _at

    def macs(mg):
        total = 0
        for sg in mg:
            main = [op for op in sg.dag.op_lst if op.reduce_axis][0]
            total += _at.lower_main_op(main, sg.dag).flops() // 2 * sg.count
        return total
    r50 = _at.resnet50(1)
    assert sum(sg.count for sg in r50) == 54 and abs(macs(r50) / 4.09e9 - 1) < 0.01    # 53 convolutions + fc
    mb = _at.mobilenet_v1(1)
    assert sum(sg.count for sg in mb) == 28 and abs(macs(mb) / 0.569e9 - 1) < 0.01    # 1 + 13 x 2 + fc
    bert = _at.bert_base(1)
    assert sum(sg.count for sg in bert) == 96
    assert macs(bert) == 12 * (4 * 512 * 768 ** 2 + 2 * 512 * 768 * 3072 + 2 * 12 * 512 ** 2 * 64)
    assert set(_at.NETWORKS) == {"resnet18", "resnet50", "mobilenet_v1", "bertbase", "shufflenet", "milstm"}
    # ShuffleNet (groups 3) as the reference's model builds it: 1 + 3 x (3 + 3 x repeats) + 1 layers;
    # multiply-accumulates from its channel arithmetic (shufflenet.py:68-185)
    sh = _at.shufflenet(1)
    assert sum(sg.count for sg in sh) == 1 + 3 * 3 + 3 * (3 + 7 + 3) + 1
    want, cin, hw = 112 * 112 * 24 * 27, 24, 56
    for cout, rep in ((240, 3), (480, 7), (960, 3)):
        mid = (cout - cin) // 4
        want += hw * hw * mid * cin // 3 + (hw // 2) ** 2 * mid * 9 + (hw // 2) ** 2 * (cout - cin) * mid // 3
        hw //= 2
        mid = cout // 4
        want += rep * (hw * hw * mid * cout // 3 + hw * hw * mid * 9 + hw * hw * cout * mid // 3)
        cin = cout
    assert macs(sh) == want + 960 * 1000
    lstm = _at.mi_lstm(8)
    assert sum(sg.count for sg in lstm) == 9 and macs(lstm) == 8 * (4 * 1024 * 1024 + 4 * 512 * 1024 + 10 * 1024)


def batch_conv2d(N, C, H, W, K, R, S, stride, padding, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_batchconv2d_tensorcore.py:7-40 (a filter bank per image)"""
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([N, K, C, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    rc = te.reduce_axis([0, C], name="rc")
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - R) // stride + 1, (pW - S) // stride + 1
    Conv = te.compute([N, K, P, Q], lambda n, k, p, q: te.sum(
        (Pad[n, rc, p * stride + rr, q * stride + rs] * B[n, k, rc, rr, rs]).astype(out_dtype),
        axis=[rc, rr, rs]), name="Conv")
    return A, B, Conv


def test_batch_conv_lowering():
    """per-image filters lower to a grouped convolution of one image with the images as groups;
    checked against the brute-force evaluation of the compute as written"""
    from amos_amd.auto_tensorize.lowering import lower_main_op
    A, B, Out = batch_conv2d(3, 4, 6, 5, 6, 3, 2, 2, 1)
    dag = at.compute_dag_from_tensors([Out])
    main = [op for op in dag.op_lst if op.reduce_axis][0]
    assert at.get_match_results(dag, "hip")
    low = lower_main_op(main, dag)
    c = low.desc
    assert low.kind == "conv2d" and (c.N, c.C, c.K, c.groups, c.R, c.S) == (1, 12, 18, 3, 3, 2)
    assert (c.stride_h, c.stride_w, c.pad_h, c.pad_w) == (2, 2, 1, 1) and [t.name for t in low.inputs] == ["A", "B"]
    rng = np.random.default_rng(21)
    a = rng.integers(-3, 4, (3, 4, 6, 5)).astype(np.float64)
    b = rng.integers(-3, 4, (3, 6, 4, 3, 2)).astype(np.float64)
    want = te_interp.evaluate(Out, {"A": a, "B": b})
    got = grouped_conv_reference(a.reshape(1, 12, 6, 5), b.reshape(18, 4, 3, 2), (2, 2), (1, 1), 3)
    assert np.array_equal(got.reshape(want.shape), want)


def capsule_conv2d(N, C, H, W, K, R, S, caps, stride, padding, dilation, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_capsuleconv2d_tensorcore.py:7-72"""
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, C, R, S, caps], dtype=in_dtype, name="B")
    P = (H + 2 * padding - dilation * (R - 1) - 1) // stride + 1
    Q = (W + 2 * padding - dilation * (S - 1) - 1) // stride + 1
    padded = te.compute([N, C, H + 2 * padding, W + 2 * padding], lambda b, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h < H + padding, w >= padding, w < W + padding),
        A[b, c, h - padding, w - padding], tir.const(0, A.dtype)), name="Padding")
    rc = te.reduce_axis((0, C), name="rc")
    rw = te.reduce_axis((0, S), name="rw")
    rh = te.reduce_axis((0, R), name="rh")
    Out = te.compute((N, K, P, Q, caps), lambda b, k, h, w, s: te.sum(
        (padded[b, rc, h * stride + rh * dilation, w * stride + rw * dilation] * B[k, rc, rh, rw, s]).astype(out_dtype),
        axis=[rc, rw, rh]), name="conv2d_capsule")
    return A, B, Out


def apply_out_view(view, flat):
    """what the module gathers from the kernel's output buffer"""
    out = np.zeros(view.shape, dtype=flat.dtype)
    for idx in np.ndindex(*view.shape):
        out[idx] = flat[sum(view.tables[d][i] for d, i in enumerate(idx))]
    return out


def test_capsule_conv_lowering():
    """a capsule axis on the filters: an ordinary convolution with K * caps filters between a
    gather of the filters and one of the result; checked against the compute as written"""
    from amos_amd.auto_tensorize.lowering import lower_main_op
    N, C, H, W, K, R, S, caps, stride, padding, dilation = 2, 3, 7, 6, 4, 3, 2, 5, 2, 1, 1
    A, B, Out = capsule_conv2d(N, C, H, W, K, R, S, caps, stride, padding, dilation)
    dag = at.compute_dag_from_tensors([Out])
    main = [op for op in dag.op_lst if op.reduce_axis][0]
    assert at.get_match_results(dag, "hip")
    low = lower_main_op(main, dag)
    c = low.desc
    assert low.kind == "conv2d" and (c.N, c.C, c.K, c.R, c.S, c.groups) == (N, C, K * caps, R, S, 0)
    assert (c.stride_h, c.pad_h, c.dil_w) == (stride, padding, dilation) and list(low.gathers) == [1]
    rng = np.random.default_rng(33)
    a = rng.integers(-3, 4, (N, C, H, W)).astype(np.float64)
    b = rng.integers(-3, 4, (K, C, R, S, caps)).astype(np.float64)
    want = te_interp.evaluate(Out, {"A": a, "B": b})
    w_kernel = apply_view(low.gathers[1], b)
    assert w_kernel.shape == (K * caps, C, R, S) and np.array_equal(w_kernel, b.transpose(0, 4, 1, 2, 3).reshape(K * caps, C, R, S))
    y_kernel = co.lib_conv2d(a.astype(np.int8), w_kernel.astype(np.int8), "int8", stride, padding, dilation).astype(np.float64)
    got = apply_out_view(low.out_view, y_kernel.reshape(-1))
    assert got.shape == want.shape and np.array_equal(got, want)


def variance(N, C, H, W, in_dtype="float16", out_dtype="float32"):
    """reference: benchmark/amos/mapping_variance_tensorcore.py:7-31"""
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    Mean = te.placeholder([N, C, H, W], dtype=in_dtype, name="Mean")
    Diff = te.compute([N, C, H, W], lambda n, c, h, w: (A[n, c, h, w] - Mean[n, c, h, w]) * (A[n, c, h, w] - Mean[n, c, h, w]),
                      name="Diff")
    B = te.compute([C, N * H * W], lambda i, j: Diff[j // (H * W), i, j % (H * W) // W, j % W], name="B")
    C_ = te.compute([N * H * W, 1], lambda i, j: tir.const(1.0 / (N * H * W), in_dtype), name="C")
    rk = te.reduce_axis([0, N * H * W], name="k")
    D = te.compute([C, 1], lambda i, j: te.sum((B[i, rk] * C_[rk, j]).astype(out_dtype), axis=rk), name="D")
    E = te.compute([C], lambda i: D[i, 0], name="E")
    return A, Mean, E


def test_variance_lowering():
    """squared differences in front of the mean's GEMM: an element-wise stage (computed per call),
    a gather on top of it, a constant second operand; checked against the compute as written"""
    from amos_amd.auto_tensorize.lowering import lower_main_op
    N, C, H, W = 2, 5, 3, 4
    A, Mean, E = variance(N, C, H, W)
    dag = at.compute_dag_from_tensors([E])
    main = [op for op in dag.op_lst if op.reduce_axis][0]
    assert at.get_match_results(dag, "hip")
    low = lower_main_op(main, dag)
    assert low.kind == "gemm" and list(low.computed) == [0] and list(low.gathers) == [0] and list(low.constants) == [1]
    stage = low.computed[0]
    assert [t.name for t in stage.inputs] == ["A", "Mean"]
    assert stage.program == [("load", 0), ("load", 1), "sub", ("load", 0), ("load", 1), "sub", "mul"]
    rng = np.random.default_rng(41)
    a = rng.integers(-3, 4, (N, C, H, W)).astype(np.float64)
    m = rng.integers(-2, 3, (N, C, H, W)).astype(np.float64)
    want = te_interp.evaluate(E, {"A": a, "Mean": m})
    # the program on numpy arrays, then the gather, then the product with the constant
    stack = []
    for step in stage.program:
        if isinstance(step, tuple):
            stack.append((a, m)[step[1]] if step[0] == "load" else step[1])
        else:
            y, x = stack.pop(), stack.pop()
            stack.append({"add": x + y, "sub": x - y, "mul": x * y}[step])
    lhs = apply_view(low.gathers[0], stack[0])
    got = (lhs @ low.constants[1].astype(np.float64)).reshape(-1)
    assert lhs.shape == (C, N * H * W) and np.allclose(got, want, rtol=1e-3)



def dilated_conv2d_as_scripted(N, C, H, W, K, R, S, stride, padding, dilation, in_dtype="float16", out_dtype="float32"):
    """the compute of benchmark/amos/mapping_dilatedconv2d_tensorcore.py:7-44 as it is spelled there:
    the reduce axes rr, rs run over the DILATED window's extents kH, kW (the tutorial's conv2d runs
    them over R, S) and index the filter B[k, rc, rr, rs] with them"""
    kH, kW = (R - 1) * dilation + 1, (S - 1) * dilation + 1
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, C, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    rc, rr, rs = te.reduce_axis([0, C], name="rc"), te.reduce_axis([0, kH], name="rr"), te.reduce_axis([0, kW], name="rs")
    P, Q = (pH - kH) // stride + 1, (pW - kW) // stride + 1
    Conv = te.compute([N, K, P, Q], lambda n, k, p, q: te.sum(
        (Pad[n, rc, p * stride + rr * dilation, q * stride + rs * dilation] * B[k, rc, rr, rs]).astype(out_dtype),
        axis=[rc, rr, rs]), name="Conv")
    return A, B, Conv


def test_dilated_conv_script_lowers_at_its_own_shapes():
    """every shape mapping_dilatedconv2d_tensorcore.py:122-129 runs has a 1x1 window (dilation 2 of
    one tap: kH = kW = 1 = R = S), where the script's spelling IS a convolution -- a pointwise one,
    whatever the dilation; with a wider window the same spelling indexes the filter past its
    extent (rr up to (R - 1) * dilation), which no convolution descriptor means: refused"""
    from amos_amd.auto_tensorize.lowering import NoKernelError, lower_main_op
    shapes_b1 = [(256, 56, 56, 512), (256, 56, 56, 128), (512, 28, 28, 1024), (512, 28, 28, 256), (1024, 14, 14, 2048),
                 (1024, 14, 14, 512)]
    for C, H, W, K in shapes_b1:
        A, B, Conv = dilated_conv2d_as_scripted(1, C, H, W, K, 1, 1, 1, 0, 2)
        low = lower_main_op(Conv.op, at.compute_dag_from_tensors([Conv]))
        d = low.desc
        assert low.kind == "conv2d" and (d.N, d.C, d.H, d.W, d.K, d.R, d.S) == (1, C, H, W, K, 1, 1)
        assert [int(x) for x in Conv.shape] == [1, K, H, W]
        name = _lib.load().amos_kernel_name(low.op_code, __import__("ctypes").byref(d), None)
        assert name is not None and (b"amos_gemm_tn" in name or b"amos_igemm" in name), name   # a matrix product
    # the interpreter agrees with the oracle's convolution on a small instance of the same spelling
    from oracle import cpu_oracle as co, te_interp
    rng = np.random.default_rng(3)
    A, B, Conv = dilated_conv2d_as_scripted(2, 8, 5, 6, 4, 1, 1, 1, 0, 2)
    a = rng.uniform(-1, 1, (2, 8, 5, 6)).astype(np.float16)
    b = rng.uniform(-1, 1, (4, 8, 1, 1)).astype(np.float16)
    got = te_interp.evaluate(Conv, {"A": a, "B": b})
    ref = co.te_literal_conv2d(a, b, "float16", 1, 0, 1)
    assert np.allclose(got, ref, atol=1e-3, rtol=1e-3)
    A, B, Conv = dilated_conv2d_as_scripted(1, 64, 14, 14, 64, 3, 3, 1, 2, 2)
    with pytest.raises(NoKernelError, match="reduce extent 5 differs from the kernel window 3"):
        lower_main_op(Conv.op, at.compute_dag_from_tensors([Conv]))
