"""Pins the CPU oracle (oracle/te_literal.c + oracle/cpu_oracle.py) without a GPU.

The reference holds no numeric vectors for this path (its tests compare two llvm builds
or print), so every oracle function is pinned by what the arithmetic fixes: numpy's own
fp16 conversions, exact integer closed forms, torch-CPU fp64 convolution, brute-force
Python loops on tiny inputs, and structured inputs (one-hot operands, all-ones images)
chosen so that a swapped index, a dropped tap or a wrong transposition changes the answer.
"""
import itertools

import numpy as np
import pytest

from conftest import make_operand
from oracle import cpu_oracle as co


def test_half_conversions_match_numpy():
    lib = co.load()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_half_to_float(int(b)) for b in bits], dtype=np.float32)
    ok = (got == want) | (np.isnan(got) & np.isnan(want))
    assert ok.all()
    rng = np.random.default_rng(1)
    # values across the whole fp16 range incl. subnormals, ties and overflow
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.9604645e-8, 2.9802322e-8, 2.98023224e-8 * 1.0001,
                  6.1035156e-5, 6.0975552e-5, np.inf, -np.inf], dtype=np.float32),
        (np.arange(2048, dtype=np.float32) + 0.5) * np.float32(2.0 ** -14),   # exact ties
        (np.arange(4096, dtype=np.float32) * 0.5) * np.float32(2.0 ** -24),   # subnormal ties
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want16 = xs.astype(np.float16).view(np.uint16)
    got16 = np.array([lib.oracle_float_to_half(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got16, want16)


def test_bf16_conversions():
    import torch
    lib = co.load()
    rng = np.random.default_rng(2)
    xs = (rng.standard_normal(5000) * 10.0 ** rng.integers(-20, 20, 5000)).astype(np.float32)
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([lib.oracle_float_to_bf16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(co.float_to_bf16_bits(xs), want)
    back = np.array([lib.oracle_bf16_to_float(int(b)) for b in want[:500]], dtype=np.float32)
    assert np.array_equal(back, torch.from_numpy(xs).to(torch.bfloat16).float().numpy()[:500])


def brute_gemm(a, b, dtype, ta, tb, literal):
    """pure-Python statement of the loop nest; numpy scalar types do the dtype rounding"""
    M, K = (a.shape[1], a.shape[0]) if ta else a.shape
    N = b.shape[0] if tb else b.shape[1]
    out = np.zeros((M, N), dtype=np.int32 if dtype == "int8" else np.float32)
    for m in range(M):
        for n in range(N):
            acc = np.int32(0) if dtype == "int8" else np.float32(0)
            for k in range(K):
                x = a[k, m] if ta else a[m, k]
                y = b[n, k] if tb else b[k, n]
                if dtype == "int8":
                    p = np.int32(np.int8((int(x) * int(y) + 128) % 256 - 128)) if literal else np.int32(int(x) * int(y))
                elif dtype == "float16":
                    p = np.float32(np.float16(np.float32(x) * np.float32(y))) if literal else np.float32(x) * np.float32(y)
                acc = acc + p
            out[m, n] = acc
    return out


@pytest.mark.parametrize("dtype", ["float16", "int8"])
@pytest.mark.parametrize("ta,tb", list(itertools.product([0, 1], [0, 1])))
def test_gemm_loop_nest_bit_exact_vs_brute_force(dtype, ta, tb):
    rng = np.random.default_rng(3)
    M, N, K = 5, 4, 7
    a = make_operand(rng, (K, M) if ta else (M, K), dtype)
    b = make_operand(rng, (N, K) if tb else (K, N), dtype)
    for mode, literal in (("te_literal", True), ("exact", False)):
        got = co.te_literal_gemm(a, b, dtype, ta, tb, mode=mode)
        assert np.array_equal(got, brute_gemm(a, b, dtype, ta, tb, literal)), (mode, ta, tb)


def _bf16_round(x):
    """float32 -> nearest bfloat16 (ties to even), returned as float32: torch-CPU's conversion"""
    import torch
    return torch.tensor([float(x)], dtype=torch.float32).to(torch.bfloat16).float().numpy()[0]


@pytest.mark.parametrize("ta,tb", list(itertools.product([0, 1], [0, 1])))
def test_bf16_gemm_loop_nest_bit_exact_vs_brute_force(ta, tb):
    """te_literal mode multiplies in bf16 (the product rounded to bf16 by torch-CPU here), widens,
    accumulates sequentially in fp32; exact mode keeps the fp32 product"""
    rng = np.random.default_rng(31)
    M, N, K = 4, 5, 9
    a = make_operand(rng, (K, M) if ta else (M, K), "bfloat16")
    b = make_operand(rng, (N, K) if tb else (K, N), "bfloat16")
    fa, fb = co.bf16_bits_to_float(a), co.bf16_bits_to_float(b)
    rounded_somewhere = False
    for mode in ("te_literal", "exact"):
        want = np.zeros((M, N), dtype=np.float32)
        for m in range(M):
            for n in range(N):
                acc = np.float32(0)
                for k in range(K):
                    x = fa[k, m] if ta else fa[m, k]
                    y = fb[n, k] if tb else fb[k, n]
                    p = np.float32(x) * np.float32(y)          # exact in fp32: 8-bit significands
                    if mode == "te_literal":
                        rounded_somewhere |= bool(_bf16_round(p) != p)
                        p = np.float32(_bf16_round(p))
                    acc = np.float32(acc + p)
                want[m, n] = acc
        assert np.array_equal(co.te_literal_gemm(a, b, "bfloat16", ta, tb, mode=mode), want), (mode, ta, tb)
    assert rounded_somewhere   # the two modes were told apart by this data


def brute_conv(x, w, dtype, stride, pad, dil, literal):
    """pure-Python statement of the conv loop nest: padded tensor materialised first, reduction
    rc outermost then rd, rr, rs, product in the input type (te_literal) or exact"""
    N, C, D, H, W = x.shape
    K, _, T, R, S = w.shape
    (sd, sh, sw), (pd, ph, pw), (dd, dh, dw) = stride, pad, dil
    if dtype == "bfloat16":
        x, w = co.bf16_bits_to_float(x), co.bf16_bits_to_float(w)
    xp = np.zeros((N, C, D + 2 * pd, H + 2 * ph, W + 2 * pw), dtype=x.dtype)
    xp[:, :, pd:pd + D, ph:ph + H, pw:pw + W] = x
    OD = (D + 2 * pd - (T - 1) * dd - 1) // sd + 1
    OP = (H + 2 * ph - (R - 1) * dh - 1) // sh + 1
    OQ = (W + 2 * pw - (S - 1) * dw - 1) // sw + 1
    out = np.zeros((N, K, OD, OP, OQ), dtype=np.int32 if dtype == "int8" else np.float32)
    for n, k, od, op, oq in itertools.product(range(N), range(K), range(OD), range(OP), range(OQ)):
        acc = np.int32(0) if dtype == "int8" else np.float32(0)
        for c, t, r, s_ in itertools.product(range(C), range(T), range(R), range(S)):
            a = xp[n, c, od * sd + t * dd, op * sh + r * dh, oq * sw + s_ * dw]
            b = w[k, c, t, r, s_]
            if dtype == "int8":
                p = np.int32(np.int8((int(a) * int(b) + 128) % 256 - 128)) if literal else np.int32(int(a) * int(b))
            elif dtype == "float16":
                p = np.float32(np.float16(np.float32(a) * np.float32(b))) if literal else np.float32(a) * np.float32(b)
            else:
                p = np.float32(a) * np.float32(b)
                p = np.float32(_bf16_round(p)) if literal else p
            acc = acc + p if dtype == "int8" else np.float32(acc + p)
        out[n, k, od, op, oq] = acc
    return out


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
@pytest.mark.parametrize("case", [((1, 2, 1, 4, 5), (2, 2, 1, 3, 3), (1, 1, 1), (0, 1, 1), (1, 1, 1)),
                                  ((1, 2, 3, 4, 4), (2, 2, 2, 3, 2), (1, 2, 1), (1, 1, 0), (1, 1, 2))])
def test_conv_loop_nest_bit_exact_vs_brute_force_in_both_modes(dtype, case):
    """the conv oracle in te_literal mode (and in exact mode) against a Python loop nest on shapes
    small enough for one: the same padding, the same reduce order, the same rounding of products"""
    xs, ws, stride, pad, dil = case
    rng = np.random.default_rng(32)
    x, w = make_operand(rng, xs, dtype), make_operand(rng, ws, dtype)
    lit = co.te_literal_conv3d(x, w, dtype, stride, pad, dil, mode="te_literal")
    exact = co.te_literal_conv3d(x, w, dtype, stride, pad, dil, mode="exact")
    assert np.array_equal(lit, brute_conv(x, w, dtype, stride, pad, dil, True))
    assert np.array_equal(exact, brute_conv(x, w, dtype, stride, pad, dil, False))
    assert not np.array_equal(lit, exact)   # the data tells the two modes apart


def test_int8_wraparound_mode_differs_and_matches_closed_form():
    """(a*b).astype(int32) on int8 wraps before widening in the reference's llvm build"""
    a = np.array([[127, -128, 100, 3]], dtype=np.int8)
    b = np.array([[127], [-128], [2], [5]], dtype=np.int8)
    exact = co.te_literal_gemm(a, b, "int8", mode="exact")
    lit = co.te_literal_gemm(a, b, "int8", mode="te_literal")
    assert exact[0, 0] == 127 * 127 + 128 * 128 + 200 + 15
    wrap = lambda v: (v + 128) % 256 - 128
    assert lit[0, 0] == wrap(127 * 127) + wrap(128 * 128) + wrap(200) + 15
    assert lit[0, 0] != exact[0, 0]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
def test_gemm_exact_mode_vs_float64_matmul(dtype):
    rng = np.random.default_rng(4)
    for (M, N, K, ta, tb) in [(33, 17, 65, 0, 0), (8, 40, 129, 0, 1), (21, 9, 30, 1, 0), (16, 16, 16, 1, 1)]:
        a = make_operand(rng, (K, M) if ta else (M, K), dtype)
        b = make_operand(rng, (N, K) if tb else (K, N), dtype)
        got = co.te_literal_gemm(a, b, dtype, ta, tb, mode="exact")
        ref = co.lib_gemm(a, b, dtype, ta, tb, acc="float64")
        if dtype == "int8":
            assert np.array_equal(got, ref)
        else:
            # exact products, fp32 sequential accumulation: |err| <= K * 2^-24 * sum|a b|
            bound = K * 2.0 ** -24 * np.abs(co.lib_gemm(np.abs(co.upcast(a, dtype)).astype(np.float16) if dtype == "float16" else a,
                                                        np.abs(co.upcast(b, dtype)).astype(np.float16) if dtype == "float16" else b,
                                                        dtype, ta, tb, acc="float64")).max() + 1e-30
            assert np.abs(got - ref).max() <= bound if dtype == "float16" else np.allclose(got, ref, rtol=1e-5, atol=1e-4)


def test_gemm_transposition_is_not_symmetric():
    """one-hot operands: C = A B with A = e_{1,2}, B = e_{2,3} has a single 1 at (1,3)"""
    a = np.zeros((4, 5), dtype=np.float16); a[1, 2] = 1
    b = np.zeros((5, 6), dtype=np.float16); b[2, 3] = 1
    c = co.te_literal_gemm(a, b, "float16")
    want = np.zeros((4, 6), dtype=np.float32); want[1, 3] = 1
    assert np.array_equal(c, want)
    assert np.array_equal(co.te_literal_gemm(a.T.copy(), b, "float16", trans_a=True), want)
    assert np.array_equal(co.te_literal_gemm(a, b.T.copy(), "float16", trans_b=True), want)
    assert np.array_equal(co.lib_gemm(a, b.T.copy(), "float16", False, True), want)


def test_gemm_rows_slab_and_threads():
    rng = np.random.default_rng(5)
    a, b = make_operand(rng, (40, 33), "float16"), make_operand(rng, (33, 20), "float16")
    full = co.te_literal_gemm(a, b, "float16")
    slab = co.te_literal_gemm(a, b, "float16", rows=(7, 19), threads=4)
    assert np.array_equal(slab[7:19], full[7:19]) and not slab[:7].any() and not slab[19:].any()


def test_bgemm_is_gemm_per_batch():
    rng = np.random.default_rng(6)
    for dtype in ("float16", "int8"):
        a, b = make_operand(rng, (3, 9, 14), dtype), make_operand(rng, (3, 6, 14), dtype)
        got = co.te_literal_bgemm(a, b, dtype, False, True)
        for i in range(3):
            assert np.array_equal(got[i], co.te_literal_gemm(a[i], b[i], dtype, False, True))
        mode_ref = co.lib_gemm(a, b, dtype, False, True, acc="float64")
        assert mode_ref.shape == got.shape


CONV_CASES = [
    # N, C, D, H, W, K, T, R, S, stride, pad, dil
    (2, 3, 1, 7, 6, 4, 1, 3, 3, (1, 1, 1), (0, 1, 1), (1, 1, 1)),
    (1, 2, 1, 9, 9, 3, 1, 3, 2, (1, 2, 1), (0, 1, 0), (1, 1, 2)),
    (1, 3, 5, 6, 7, 2, 3, 3, 3, (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    (2, 2, 6, 5, 8, 3, 2, 3, 2, (2, 1, 2), (1, 0, 2), (1, 2, 1)),
    (1, 4, 1, 5, 5, 2, 1, 1, 1, (1, 2, 2), (0, 0, 0), (1, 1, 1)),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "int8"])
def test_conv_vs_torch_cpu_float64(case, dtype):
    """padding / stride / dilation index math against torch.nn.functional.conv3d on the CPU"""
    import torch
    N, C, D, H, W, K, T, R, S, st, pd, dl = case
    rng = np.random.default_rng(7)
    x, w = make_operand(rng, (N, C, D, H, W), dtype), make_operand(rng, (K, C, T, R, S), dtype)
    ref = torch.nn.functional.conv3d(torch.from_numpy(co.upcast(x, dtype)), torch.from_numpy(co.upcast(w, dtype)),
                                     stride=st, padding=pd, dilation=dl).numpy()
    got = co.te_literal_conv3d(x, w, dtype, st, pd, dl, mode="exact")
    lib = co.lib_conv3d(x, w, dtype, st, pd, dl, acc="float64")
    assert got.shape == ref.shape == lib.shape
    if dtype == "int8":
        assert np.array_equal(got, ref.astype(np.int64)) and np.array_equal(lib, got)
    else:
        assert np.allclose(got, ref, rtol=1e-5, atol=1e-4) and np.allclose(lib, ref, rtol=1e-12, atol=1e-10)
    if D == 1 and T == 1:
        got2 = co.te_literal_conv2d(x[:, :, 0], w[:, :, 0], dtype, st[1:], pd[1:], dl[1:], mode="exact")
        assert np.array_equal(got2, got[:, :, 0])


def test_conv_all_ones_counts_in_bounds_taps():
    x = np.ones((1, 2, 5, 5), dtype=np.int8)
    w = np.ones((1, 2, 3, 3), dtype=np.int8)
    y = co.te_literal_conv2d(x, w, "int8", 1, 1, 1)
    assert y[0, 0, 0, 0] == 2 * 4 and y[0, 0, 0, 2] == 2 * 6 and y[0, 0, 2, 2] == 2 * 9
    assert y.shape == (1, 1, 5, 5)


def test_conv_reduce_order_is_rc_outermost():
    """fp32 sequential accumulation is order dependent: 2^24 + 1 - 2^24 differs by order.
    Channel 0 carries +2^12 * 2^12, the later taps carry 1 and -2^24."""
    x = np.zeros((1, 2, 1, 2), dtype=np.float16)
    w = np.zeros((1, 2, 1, 2), dtype=np.float16)
    # channel 0, s=0: 4096 * 4096 = 2^24 ; channel 0, s=1: 1 * 1 ; channel 1, s=0: -4096 * 4096
    x[0, 0, 0, 0], w[0, 0, 0, 0] = 4096, 4096
    x[0, 0, 0, 1], w[0, 0, 0, 1] = 1, 1
    x[0, 1, 0, 0], w[0, 1, 0, 0] = -4096, 4096
    y = co.te_literal_conv2d(x, w, "float16", 1, 0, 1, mode="exact")
    # rc outermost: ((2^24 + 1) - 2^24) = 0 in fp32 (the +1 is lost); any other order gives 1
    assert y.shape == (1, 1, 1, 1) and y[0, 0, 0, 0] == 0.0


def test_conv_images_slab():
    rng = np.random.default_rng(8)
    x, w = make_operand(rng, (4, 3, 6, 6), "float16"), make_operand(rng, (5, 3, 3, 3), "float16")
    full = co.te_literal_conv2d(x, w, "float16", 1, 1, 1)
    slab = co.te_literal_conv2d(x, w, "float16", 1, 1, 1, images=(1, 3), threads=3)
    assert np.array_equal(slab[1:3], full[1:3]) and not slab[0].any() and not slab[3].any()


def test_rel_errors_floor():
    ref = np.array([0.0, 1.0, -1.0, 2.0])
    got = ref + np.array([1e-3, 0, 0, 0])
    mx, mean = co.rel_errors(got, ref)
    rms = np.sqrt(np.mean(ref ** 2))
    assert abs(mx - 1e-3 / (1e-2 * rms)) < 1e-12 and mean == pytest.approx(mx / 4)
