"""Headline benchmark: fp16 GEMM M=N=K=8192, fp32 accumulate, row-major A, column-major B,
on one MI355X, next to the CPU restatement of the reference's llvm path timed in the same run.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--report FILE] [--model-check FILE]
  python bench.py --mfma-ceiling     (what the matrix cores sustain with nothing else in their way)

A step is one launch of the GEMM over device-resident operands.  Prints ONE JSON line; its
`per_op` holds the other configurations of the path (fp16 / int8 conv2d, batched GEMM,
conv3d), each timed in the same run next to the CPU loop nest on a slab of the same workload.
`--report FILE` additionally times every configuration of the path (GEMM, batched GEMM,
conv2d fp16 / int8, conv3d) and writes a per-config table as JSON to FILE.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "TFLOP/s + % of MFMA peak per op (fp16 conv2d/GEMM, int8 TOP/s), 1 MI355X"
# MI355X's published dense fp16 / int8 MFMA peaks and HBM3E bandwidth
from amos_amd.auto_tensorize.target import PEAK_F16_TFLOPS, PEAK_HBM_GBS, PEAK_I8_TOPS  # noqa: E402
# untimed launches of the workload before the warm-up steps (see main())
CLOCK_RAMP_LAUNCHES = 60


def kernel_source_hash(files):
    """first 12 hex digits of the sha256 over the named kernel sources (relative to the repository)"""
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:12]


def stale_summaries():
    """{configuration: record} of the `stale_json:` lines under profiles/: configurations whose
    default kernel has changed since its counters were read and has not been profiled again (the
    record names the kernel that ships now and why there is no reading of it)"""
    out = {}
    pdir = os.path.join(ROOT, "profiles")
    for fn in sorted(os.listdir(pdir)) if os.path.isdir(pdir) else []:
        if fn.endswith(".md"):
            for line in open(os.path.join(pdir, fn)):
                if line.startswith("stale_json:"):
                    try:
                        rec = json.loads(line[len("stale_json:"):])
                        out[rec["config"]] = rec
                    except (ValueError, KeyError):
                        continue
    return out


def measured_traffic(kernel_name):
    """HBM bytes per launch of `kernel_name` from the counter summaries under profiles/: a summary
    carries a line `traffic_json: {...}` with the kernel's name, the two counter readings (KiB per
    dispatch), the factors a plain copy of known size gave for them, and the hash of the kernel's
    sources at the time of the run.  Returns None when no summary names this kernel or its sources
    have changed since (the figure would describe a kernel that no longer ships).  A summary may
    carry its figure over to ONE later state of the sources (`carried_to`: that state's hash and
    the reason why the change cannot have moved the kernel's memory traffic), for changes that
    leave the measured instance's loop and addresses as they were."""
    pdir = os.path.join(ROOT, "profiles")
    if not os.path.isdir(pdir):
        return None
    for fn in sorted(os.listdir(pdir)):
        if not fn.endswith(".md"):
            continue
        for line in open(os.path.join(pdir, fn)):
            if not line.startswith("traffic_json:"):
                continue
            try:
                rec = json.loads(line[len("traffic_json:"):])
                if rec["kernel"] != kernel_name:
                    continue
                now = kernel_source_hash(rec["sources"])
                if now != rec["source_hash"] and now != rec.get("carried_to", {}).get("source_hash"):
                    continue
                return (rec["fetch_kib"] * rec["fetch_scale"] + rec["write_kib"] * rec["write_scale"]) * 1024.0
            except (ValueError, KeyError, OSError):
                continue
    return None


def mfma_ceiling(da, db, variants=None, launches=10, repeats=3):
    """amos_mfma_ceiling over the named variants (shape, random operands, copies, reads): the
    matrix-core instruction stream of the 8192^3 product with no wait anywhere.  da, db: device
    fp16 [8192][8192] operands.  Returns rows with the best of `repeats` means of `launches`."""
    import torch
    from amos_amd import _lib
    lib = _lib.load()
    sink = torch.zeros(256, device="cuda")
    variants = variants or [(16, 1, 0, 0)]
    rows = []
    for shape, rnd, copies, reads in variants:
        best, flop = None, ctypes.c_double()
        for _ in range(repeats):
            sec = ctypes.c_double()
            _lib.check(lib.amos_mfma_ceiling(shape, rnd, copies, reads, da.data_ptr(), db.data_ptr(),
                                             da.numel() * da.element_size(), sink.data_ptr(), launches, None,
                                             ctypes.byref(sec), ctypes.byref(flop)))
            best = sec.value if best is None else min(best, sec.value)
        rows.append({"instruction": "v_mfma_f32_16x16x32_f16" if shape == 16 else "v_mfma_f32_32x32x16_f16",
                     "operands": "random fp16 U[-1,1]" if rnd else "small constants",
                     "extra_traffic": " + ".join(n for n, on in (("global->LDS copies", copies), ("LDS fragment reads", reads)) if on) or "none",
                     "us_per_launch": best * 1e6, "tflops": flop.value / best / 1e12,
                     "frac_of_published_peak": flop.value / best / 1e12 / PEAK_F16_TFLOPS})
    return rows


def cpu_baseline_gemm(a, b, seconds_budget=12.0):
    """te_literal loop nest (single thread, as TVM's default schedule) on a slab of rows of the
    same 8192^3 workload, scaled linearly; plus an all-core OpenMP run of a larger slab."""
    from oracle import cpu_oracle as co
    n = a.shape[0]
    flop_row = 2.0 * n * n
    t0 = time.perf_counter()
    co.te_literal_gemm(a, b, "float16", False, True, rows=(0, 1), threads=1)
    t_row = time.perf_counter() - t0
    rows1 = int(max(2, min(64, seconds_budget / max(t_row, 1e-6))))
    t0 = time.perf_counter()
    co.te_literal_gemm(a, b, "float16", False, True, rows=(0, rows1), threads=1)
    t1 = time.perf_counter() - t0
    cores = min(co.load().oracle_max_threads(), int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
    rowsn = rows1 * cores
    t0 = time.perf_counter()
    co.te_literal_gemm(a, b, "float16", False, True, rows=(0, rowsn), threads=cores)
    tn = time.perf_counter() - t0
    return {
        "value": rows1 * flop_row / t1 / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": "rows [0,%d) of the 8192^3 GEMM, te_literal loop nest (fp16 product rounded to "
                  "fp16, fp32 sequential accumulate), gcc -O3, %.1f s; extrapolated_from=%.5f"
                  % (rows1, t1, rows1 / n),
        "all_cores": {"value": rowsn * flop_row / tn / 1e12, "unit": "TFLOP/s", "cores": cores,
                      "sample": "rows [0,%d), OpenMP over rows, %.1f s" % (rowsn, tn)},
    }


def _timed(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def run_all_configs(cpu=True, only=None, launches=None):
    """Every configuration of the path: GPU ms, TFLOP/s (TOP/s), % of the MFMA peak, % of the
    HBM roof for the algorithmic bytes, which roof binds, and the te_literal CPU loop nest
    (1 thread and all cores) on a slab of the same workload, linearly scaled."""
    import numpy as np
    import torch
    from amos_amd import _lib, ops
    from oracle import cpu_oracle as co
    cores = min(co.load().oracle_max_threads(), int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
    rng = np.random.default_rng(0)
    f16 = lambda x: x.astype(np.float32).astype(np.float16)
    rows = []

    def gpu_time(op, desc, i0, i1, out, fused=None):
        cfg = ops.default_config(op, desc)
        if launches:   # (a fixed, small number of launches: runs under a profiler)
            t = ops.time_op(op, desc, i0, i1, out, config=cfg, number=launches, repeat=1, min_repeat_ms=0, add=fused)
        else:
            t = ops.time_op(op, desc, i0, i1, out, config=cfg, number=20, repeat=3, min_repeat_ms=100, add=fused)
        return sum(t) / len(t), cfg   # mean seconds per call over all repeats

    def add(name, op, desc, hin, dtype, flop, nbytes, out_shape, cpu_fn, frac, fused_tail=False):
        if only and not any(o in name for o in ([only] if isinstance(only, str) else only)):
            return
        tin = [(torch.from_numpy(h) if isinstance(h, np.ndarray) else h).cuda() for h in hin]
        out = torch.empty(out_shape, dtype=torch.int32 if dtype == "int8" else torch.float32,
                          device="cuda")
        # fused tail out = acc + D: D has the output's shape and type, read once more
        fused = torch.ones_like(out) if fused_tail else None
        if fused_tail:
            nbytes += out.numel() * 4
        sec, cfg = gpu_time(op, desc, tin[0], tin[1], out, fused)
        peak = PEAK_I8_TOPS if dtype == "int8" else PEAK_F16_TFLOPS
        t_mfma, t_hbm = flop / (peak * 1e12), nbytes / (PEAK_HBM_GBS * 1e9)
        row = {"config": name, "kernel": ops.kernel_name(op, desc, cfg), "split_k": cfg.split_k,
               "gpu_us": sec * 1e6, "tflops": flop / sec / 1e12,
               "pct_mfma_peak": 100 * t_mfma / sec, "pct_hbm_roof": 100 * t_hbm / sec,
               "bound": "mfma" if t_mfma >= t_hbm else "hbm", "frac": max(t_mfma, t_hbm) / sec,
               "flop": flop, "bytes": nbytes}
        row["traffic_bytes"] = measured_traffic(row["kernel"])
        if cfg.pipeline == _lib.AMOS_PIPE_NCHW and not fused_tail and not launches:
            # the same convolution where the owner of the weights has packed them once
            # (amos_conv_pack_weights + AMOS_FLAG_WEIGHTS_PACKED): no packing launch in the call
            lib = _lib.load()
            packed = torch.empty(lib.amos_conv_packed_weights_bytes(op, ctypes.byref(desc)), dtype=torch.uint8,
                                 device="cuda")
            try:
                _lib.check(lib.amos_conv_pack_weights(op, ctypes.byref(desc), tin[1].data_ptr(), packed.data_ptr(), None))
                c2 = _lib.KernelConfig.from_buffer_copy(cfg)
                c2.reserved[0] |= _lib.AMOS_FLAG_WEIGHTS_PACKED
                res = (ctypes.c_double * 3)()
                _lib.check(lib.amos_time(op, ctypes.byref(desc), ctypes.byref(c2), tin[0].data_ptr(), packed.data_ptr(),
                                         out.data_ptr(), None, 0, None, 20, 3, 100, res))
                row["gpu_us_weights_packed_once"] = sum(res) / len(res) * 1e6
            except _lib.AmosError as e:      # (a side figure: the row stands without it)
                row["gpu_us_weights_packed_once_error"] = str(e)
            del packed
        if cpu and cpu_fn is not None:
            t1 = _timed(lambda: cpu_fn(1, False))
            tn = _timed(lambda: cpu_fn(cores, True))
            row["cpu"] = {"kind": "port (te_literal loop nest, gcc -O3)",
                          "threads1_tflops": flop * frac[0] / t1 / 1e12,
                          "threadsN_tflops": flop * frac[1] / tn / 1e12, "cores": cores,
                          "extrapolated_from": list(frac)}
        rows.append(row)
        del tin, out
        torch.cuda.empty_cache()

    # C2 fp16 GEMM 8192^3
    n = 8192
    a, b = f16(rng.uniform(-1, 1, (n, n))), f16(rng.uniform(-1, 1, (n, n)))
    add("C2 fp16 GEMM 8192^3 (ntn)", _lib.AMOS_OP_GEMM, ops.gemm_desc(n, n, n, torch.float16, False, True),
        [a, b], "float16", 2.0 * n ** 3, 2 * n * n * 2 + n * n * 4, (n, n),
        lambda th, big: co.te_literal_gemm(a, b, "float16", False, True, rows=(0, 8 * th), threads=th),
        (8 / n, 8 * cores / n))
    add("C2 + D: fp16 GEMM 8192^3 with the fused tail E = C + D (D fp32)", _lib.AMOS_OP_GEMM,
        ops.gemm_desc(n, n, n, torch.float16, False, True), [a, b], "float16", 2.0 * n ** 3,
        2 * n * n * 2 + n * n * 4, (n, n), None, None, fused_tail=True)
    # C3 fp16 conv2d
    x = f16(rng.uniform(0, 1, (32, 256, 14, 14)))
    w = f16(rng.standard_normal((256, 256, 3, 3)) * 0.05)
    add("C3 fp16 conv2d N32 C256 14x14 K256 3x3", _lib.AMOS_OP_CONV2D,
        ops.conv_desc((32, 256, 1, 14, 14), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1)),
        [x, w], "float16", 2.0 * 6272 * 256 * 2304, 10813440, (32, 256, 14, 14),
        lambda th, big: co.te_literal_conv2d(x, w, "float16", 1, 1, 1, images=(0, 2 * th), threads=th),
        (2 / 32, min(32, 2 * cores) / 32))
    add("C3 + D: fp16 conv2d with the fused tail (D fp32, NKPQ)", _lib.AMOS_OP_CONV2D,
        ops.conv_desc((32, 256, 1, 14, 14), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1)),
        [x, w], "float16", 2.0 * 6272 * 256 * 2304, 10813440, (32, 256, 14, 14), None, None, fused_tail=True)
    # C4 int8 conv2d
    xi = rng.integers(-128, 128, (64, 128, 28, 28)).astype(np.int8)
    wi = rng.integers(-64, 64, (128, 128, 3, 3)).astype(np.int8)
    add("C4 int8 conv2d N64 C128 28x28 K128 3x3", _lib.AMOS_OP_CONV2D,
        ops.conv_desc((64, 128, 1, 28, 28), (128, 128, 1, 3, 3), torch.int8, (1, 1, 1), (0, 1, 1), (1, 1, 1)),
        [xi, wi], "int8", 2.0 * 50176 * 128 * 1152, 32260096, (64, 128, 28, 28),
        lambda th, big: co.te_literal_conv2d(xi, wi, "int8", 1, 1, 1, mode="exact", images=(0, th), threads=th),
        (1 / 64, cores / 64))
    # C5a fp16 batched GEMM
    q, k = f16(rng.standard_normal((192, 512, 64))), f16(rng.standard_normal((192, 512, 64)))
    add("C5a fp16 bGEMM 192x(512x512x64) (ntn)", _lib.AMOS_OP_BGEMM,
        ops.bgemm_desc(192, 512, 512, 64, torch.float16, False, True), [q, k], "float16",
        2.0 * 192 * 512 * 512 * 64, 226492416, (192, 512, 512),
        lambda th, big: co.te_literal_bgemm(q, k, "float16", False, True, batches=(0, 4 * th), threads=th),
        (4 / 192, 4 * cores / 192))
    # C5b fp16 conv3d
    x3, w3 = f16(rng.standard_normal((8, 64, 16, 56, 56))), f16(rng.standard_normal((64, 64, 3, 3, 3)))
    x3s = np.ascontiguousarray(x3[:1, :, :4])   # CPU slab: one image, 4 of 16 depth slices
    add("C5b fp16 conv3d N8 C64 D16 56x56 K64 3x3x3", _lib.AMOS_OP_CONV3D,
        ops.conv_desc((8, 64, 16, 56, 56), (64, 64, 3, 3, 3), torch.float16, (1, 1, 1), (1, 1, 1), (1, 1, 1)),
        [x3, w3], "float16", 2.0 * 401408 * 64 * 1728, 154361856, (8, 64, 16, 56, 56),
        lambda th, big: co.te_literal_conv3d(x3s, w3, "float16", 1, 1, 1, threads=th),
        (1 / 32, 1 / 32))
    # beyond the headline configurations: MobileNet-V1's first depthwise layer at batch 16 (the
    # reference's benchmark/amos/mapping_depthwiseconv2d_tensorcore.py op), a byte mover
    xd, wd = f16(rng.standard_normal((16, 32, 112, 112))), f16(rng.standard_normal((32, 1, 3, 3)))
    add("depthwise fp16 conv2d N16 C32 112x112 3x3 (groups 32)", _lib.AMOS_OP_CONV2D,
        ops.conv_desc((16, 32, 1, 112, 112), (32, 1, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1), 32),
        [xd, wd], "float16", 2.0 * 16 * 32 * 112 * 112 * 9, 16 * 32 * 112 * 112 * 6 + 32 * 9 * 2,
        (16, 32, 112, 112), None, None)
    # ResNet's stem at batch 16 (three input channels: the kernel whose reduction unit is the pixel)
    xs, ws = f16(rng.standard_normal((16, 3, 224, 224))), f16(rng.standard_normal((64, 3, 7, 7)) * 0.1)
    add("stem fp16 conv2d N16 C3 224x224 K64 7x7/2", _lib.AMOS_OP_CONV2D,
        ops.conv_desc((16, 3, 1, 224, 224), (64, 3, 1, 7, 7), torch.float16, (1, 2, 2), (0, 3, 3), (1, 1, 1)),
        [xs, ws], "float16", 2.0 * 16 * 112 * 112 * 64 * 147, 16 * 3 * 224 * 224 * 2 + 64 * 147 * 2 + 16 * 64 * 112 * 112 * 4,
        (16, 64, 112, 112), None, None)
    # the 8192^3 product in the path's other two operand types (bf16 -> fp32, int8 -> int32)
    add("GEMM bf16 8192^3 (ntn)", _lib.AMOS_OP_GEMM, ops.gemm_desc(n, n, n, torch.bfloat16, False, True),
        [torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16), torch.from_numpy(b.astype(np.float32)).to(torch.bfloat16)],
        "bfloat16", 2.0 * n ** 3, 2 * n * n * 2 + n * n * 4, (n, n), None, None)
    a8, b8 = rng.integers(-128, 128, (n, n), dtype=np.int8), rng.integers(-128, 128, (n, n), dtype=np.int8)
    add("GEMM int8 8192^3 (ntn)", _lib.AMOS_OP_GEMM, ops.gemm_desc(n, n, n, torch.int8, False, True),
        [a8, b8], "int8", 2.0 * n ** 3, 2 * n * n + n * n * 4, (n, n), None, None)
    # a GEMV as benchmark/amos/mapping_gemv_tensorcore.py spells it (A [M, K], B [K, 1]), at a size
    # where it is the pass over A that is timed (the reference's own shapes, up to 1024 x 1024, are
    # launch-bound): one pass over 268 MB on the vector-ALU kernel
    mv, kv = 16384, 8192
    av, bv = f16(rng.uniform(-1, 1, (mv, kv))), f16(rng.uniform(-1, 1, (kv, 1)))
    add("GEMV fp16 M=16384 K=8192 (B [K, 1])", _lib.AMOS_OP_GEMM, ops.gemm_desc(mv, 1, kv, torch.float16, False, False),
        [av, bv], "float16", 2.0 * mv * kv, mv * kv * 2 + kv * 2 + mv * 4, (mv, 1), None, None)
    return rows


def model_check():
    """The mapper's analytical model against measurement: for a set of shapes (the benchmark
    configurations the constants were fitted on, and shapes they were not), every kernel
    configuration is timed and ranked both ways."""
    import ctypes
    import torch
    from scipy.stats import spearmanr
    from amos_amd import _lib, ops
    lib = _lib.load()
    tiles = [(256, 256), (256, 128), (128, 256), (128, 128), (256, 64), (128, 64), (64, 128), (64, 64), (64, 256)]

    def sweep(name, fitted, op, d, a, b, out, pipes, splits):
        rows = []
        for pipe in pipes:
            for ti, tj in tiles:
                for sp in splits:
                    cfg = dict(tile_i=ti, tile_j=tj, split_k=sp, pipeline=pipe)
                    c = ops.make_config(cfg)
                    est = ctypes.c_double()
                    if lib.amos_check_config(op, ctypes.byref(d), ctypes.byref(c), None, None) < 0 or \
                            lib.amos_kernel_name(op, ctypes.byref(d), ctypes.byref(c)) is None or \
                            lib.amos_estimate_seconds(op, ctypes.byref(d), ctypes.byref(c), ctypes.byref(est)) != 0:
                        continue
                    try:
                        t = ops.time_op(op, d, a, b, out, config=cfg, number=5, repeat=1, min_repeat_ms=20)[0]
                    except _lib.AmosError:
                        continue
                    rows.append((t, est.value, ops.kernel_name(op, d, cfg), sp))
        rows.sort(key=lambda r: r[0])
        by_est = sorted(rows, key=lambda r: r[1])
        dflt = ops.default_config(op, d)
        t_default = ops.time_op(op, d, a, b, out, config=dflt, number=5, repeat=1, min_repeat_ms=20)[0]
        return {"shape": name, "fitted_on": fitted, "configs": len(rows),
                "spearman": float(spearmanr([r[0] for r in rows], [r[1] for r in rows]).correlation),
                "best_us": rows[0][0] * 1e6, "best_kernel": "%s split %d" % (rows[0][2], rows[0][3]),
                "model_first_us": by_est[0][0] * 1e6, "model_first_est_us": by_est[0][1] * 1e6,
                "model_first_kernel": "%s split %d" % (by_est[0][2], by_est[0][3]),
                "rank_of_best_in_model_order": [i for i, r in enumerate(by_est) if r is rows[0]][0],
                "default_config_us": t_default * 1e6,
                "default_kernel": "%s split %d" % (ops.kernel_name(op, d, dflt), dflt.split_k)}

    out = []
    GEMM, BGEMM, CONV2D, CONV3D = _lib.AMOS_OP_GEMM, _lib.AMOS_OP_BGEMM, _lib.AMOS_OP_CONV2D, _lib.AMOS_OP_CONV3D
    f16, i8 = torch.float16, torch.int8

    def gemm_case(M, N, K, ta, tb, dt, fitted):
        if dt == i8:
            a = torch.randint(-8, 8, (K, M) if ta else (M, K), device="cuda", dtype=dt)
            b = torch.randint(-8, 8, (N, K) if tb else (K, N), device="cuda", dtype=dt)
            c = torch.empty(M, N, device="cuda", dtype=torch.int32)
        else:
            a = torch.randn((K, M) if ta else (M, K), device="cuda").to(dt)
            b = torch.randn((N, K) if tb else (K, N), device="cuda").to(dt)
            c = torch.empty(M, N, device="cuda")
        name = "GEMM %dx%dx%d %s%s %s" % (M, N, K, "t" if ta else "n", "t" if tb else "n", str(dt).split(".")[1])
        out.append(sweep(name, fitted, GEMM, ops.gemm_desc(M, N, K, dt, ta, tb), a, b, c, (0, 1), (1, 2, 4, 8)))

    def conv_case(name, fitted, xs, ws, st, pd, dt=f16, op=CONV2D):
        if dt == i8:
            x = torch.randint(-128, 127, xs, device="cuda", dtype=dt)
            w = torch.randint(-64, 63, ws, device="cuda", dtype=dt)
        else:
            x, w = torch.rand(xs, device="cuda").to(dt), (torch.randn(ws, device="cuda") * 0.05).to(dt)
        xs5 = tuple(xs) if op == CONV3D else (xs[0], xs[1], 1, xs[2], xs[3])
        ws5 = tuple(ws) if op == CONV3D else (ws[0], ws[1], 1, ws[2], ws[3])
        d = ops.conv_desc(xs5, ws5, dt, st, pd, (1, 1, 1))
        oshape = ops.conv_out_shape(xs5, ws5, st, pd, (1, 1, 1))
        y = torch.empty(oshape if op == CONV3D else (oshape[0], oshape[1], oshape[3], oshape[4]),
                        device="cuda", dtype=torch.int32 if dt == i8 else torch.float32)
        out.append(sweep(name, fitted, op, d, x, w, y, (_lib.AMOS_PIPE_NCHW, _lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8, _lib.AMOS_PIPE_STAGED),
                         (1, 2, 4) if op == CONV2D else (1,)))

    for M, N, K in [(8192, 8192, 8192), (2048, 2048, 2048), (512, 512, 4096), (4096, 256, 1024)]:
        gemm_case(M, N, K, 0, 1, f16, True)
    conv_case("C3 conv2d N32 C256 14x14 K256 3x3 f16", True, (32, 256, 14, 14), (256, 256, 3, 3), (1, 1, 1), (0, 1, 1))
    conv_case("C4 conv2d N64 C128 28x28 K128 3x3 i8", True, (64, 128, 28, 28), (128, 128, 3, 3), (1, 1, 1), (0, 1, 1), i8)
    conv_case("C5b conv3d N8 C64 D16 56x56 K64 3x3x3 f16", True, (8, 64, 16, 56, 56), (64, 64, 3, 3, 3), (1, 1, 1),
              (1, 1, 1), f16, CONV3D)
    for M, N, K, ta, tb, dt in [(3000, 1000, 2000, 0, 1, f16), (1024, 8192, 512, 0, 1, f16), (2048, 2048, 2048, 0, 0, f16),
                                (6144, 768, 3072, 1, 0, f16), (2048, 2048, 2048, 0, 1, i8), (200, 120, 5000, 0, 1, f16)]:
        gemm_case(M, N, K, ta, tb, dt, False)
    a = torch.randn(16, 512, 256, device="cuda").half()
    b = torch.randn(16, 512, 256, device="cuda").half()
    c = torch.empty(16, 512, 512, device="cuda")
    out.append(sweep("bGEMM 16x(512x512x256) nt f16", False, BGEMM, ops.bgemm_desc(16, 512, 512, 256, f16, False, True),
                     a, b, c, (0, 1), (1,)))
    conv_case("conv2d N8 C128 28x28 K256 3x3 f16", False, (8, 128, 28, 28), (256, 128, 3, 3), (1, 1, 1), (0, 1, 1))
    conv_case("conv2d N16 C64 56x56 K64 1x1 f16", False, (16, 64, 56, 56), (64, 64, 1, 1), (1, 1, 1), (0, 0, 0))
    conv_case("conv2d N4 C48 30x30 K96 5x5 f16", False, (4, 48, 30, 30), (96, 48, 5, 5), (1, 1, 1), (0, 2, 2))
    conv_case("conv2d N16 C64 56x56 K64 3x3 f16", False, (16, 64, 56, 56), (64, 64, 3, 3), (1, 1, 1), (0, 1, 1))
    conv_case("conv2d N64 C512 14x14 K512 3x3 f16", False, (64, 512, 14, 14), (512, 512, 3, 3), (1, 1, 1), (0, 1, 1))
    return out


def network_report(trials=200, networks=("resnet18", "resnet50", "mobilenet_v1", "bertbase", "shufflenet", "milstm"),
                   batches=(1, 16)):
    """The tensorisable layers of whole networks through the network dispatcher (the flow of the
    reference's benchmark/amos/mapping_{resnet18,resnet50,mobilenetv1,bertbase,shufflenet,milstm}_tensorcore.py): per
    distinct layer the tuned kernel and its time, and the sum over the network's layers"""
    import contextlib
    import io
    import tempfile
    from amos_amd import auto_tensorize as at
    out = []
    for name in networks:
        for batch in batches:
            multi_graph = at.NETWORKS[name](batch)
            opt = at.MeasureOptions(target="hip", timeout=100, number=5, min_repeat_ms=10)
            with tempfile.TemporaryDirectory() as log_dir:
                dispatch = at.AutoScheduleMultiGraphDispatch
                with contextlib.redirect_stdout(io.StringIO()):
                    tid = dispatch.add_graph_task(name, multi_graph, opt, trials=trials, log_dir=log_dir,
                                                  transform_strict=False)
                    dispatch.auto_schedule(tid)
                    sch_tensors = dispatch.get_schedules(tid)
                    total = at.evaluate_graph(multi_graph, sch_tensors, "hip", 0, 20, False, min_repeat_ms=50)
                rows = at.evaluate_graph.last_rows
            flop = sum(r[4] * r[2] for r in rows)
            out.append({"network": name, "batch": batch, "layers_ms": total, "flop": flop,
                        "tflops": flop / (total * 1e-3) / 1e12,
                        "layers": [{"name": r[0], "layer": r[1], "count": r[2], "ms": r[3], "flop": r[4],
                                    "kernel": r[5]} for r in rows]})
            print("network %s batch %d: %.3f ms over %d layers" % (name, batch, total, sum(r[2] for r in rows)),
                  file=sys.stderr, flush=True)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--no-per-op", action="store_true",
                    help="skip the per-configuration table (conv2d fp16 / int8, batched GEMM, conv3d)")
    ap.add_argument("--report", default=None, help="also time every config, write JSON here")
    ap.add_argument("--report-only", default=None,
                    help="restrict --report to the configurations whose name contains this text")
    ap.add_argument("--model-check", default=None,
                    help="also rank every kernel configuration of a set of shapes by the mapper's model "
                         "and by measurement, write JSON here")
    ap.add_argument("--network", default=None,
                    help="also tune and time the tensorisable layers of ResNet-18, ResNet-50, MobileNet-V1, "
                         "BERT-base, ShuffleNet and an MI-LSTM cell at batch 1 and 16 through the network "
                         "dispatcher, write JSON here")
    ap.add_argument("--networks", default="resnet18,resnet50,mobilenet_v1,bertbase,shufflenet,milstm",
                    help="the networks --network covers, comma-separated")
    ap.add_argument("--config", default=None,
                    help="run only the configuration whose name contains this text (C2, C3 fp16, C4 int8, C5a, "
                         "C5b), --steps launches of it, print its row and exit: the command that the counter "
                         "summaries under profiles/ were made with")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="only measure what the matrix cores sustain (amos_mfma_ceiling: both instruction shapes, "
                         "constant and random operands, with and without the data movement of a 256x256x64 "
                         "tiling), print the rows as JSON and exit")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 256 MiB device copy, the known-size kernel that rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures the one-GPU kernel path; --gpus %d is not supported "
                 "(this build has no multi-GPU path)" % args.gpus)

    import numpy as np
    import torch
    from amos_amd import _lib, ops
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    if args.mfma_ceiling:
        g = torch.Generator(device="cuda").manual_seed(0)
        da = (torch.rand((8192, 8192), device="cuda", generator=g) * 2 - 1).half()
        db = (torch.rand((8192, 8192), device="cuda", generator=g) * 2 - 1).half()
        # (the clock settles under load: two passes, the second one is reported)
        variants = [(32, 0, 0, 0), (32, 1, 0, 0), (16, 0, 0, 0), (16, 1, 0, 0), (32, 1, 1, 0), (32, 1, 0, 1),
                    (32, 1, 1, 1), (16, 1, 1, 1), (32, 0, 1, 1)]
        mfma_ceiling(da, db, variants, launches=20, repeats=1)
        print(json.dumps(mfma_ceiling(da, db, variants, launches=20, repeats=3), indent=1))
        return
    if args.config:
        if args.calibrate_copy:
            src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst
        rows = run_all_configs(cpu=False, only=(args.config,), launches=max(1, args.steps))
        rows = [r for r in rows if " + D" not in r["config"]]
        print(json.dumps(rows))
        return
    n = 8192
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, (n, n)).astype(np.float32).astype(np.float16)
    b = rng.uniform(-1, 1, (n, n)).astype(np.float32).astype(np.float16)   # stored [N, K]
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    dc = torch.empty((n, n), dtype=torch.float32, device="cuda")
    desc = ops.gemm_desc(n, n, n, torch.float16, False, True)
    cfg = ops.default_config(_lib.AMOS_OP_GEMM, desc)
    flop = 2.0 * n ** 3

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # The chip needs ~50 launches (~50 ms) of this load after an idle spell before it runs at the clock it
    # then sustains: launches 3-6 after idle take 1.07-1.17 ms, the 50th and every later one 0.83 ms.
    # The metric is sustained throughput, so the device is brought there first, with launches that are
    # neither warm-up steps nor timed steps (their count is reported in config.clock_ramp_launches).
    for _ in range(CLOCK_RAMP_LAUNCHES):
        ops.gemm(da, db, False, True, out=dc, config=cfg)
    for _ in range(args.warmup):
        ops.gemm(da, db, False, True, out=dc, config=cfg)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ops.gemm(da, db, False, True, out=dc, config=cfg)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = flop / (elapsed / args.steps) / 1e12

    # dominant (only) kernel: mean launch duration from HIP events on the launch stream
    per_launch = ops.time_op(_lib.AMOS_OP_GEMM, desc, da, db, dc, config=cfg, number=args.steps,
                             repeat=1, min_repeat_ms=0)[0]
    achieved = flop / per_launch / 1e12
    # what the matrix cores sustain on this box with the benchmark's operand values and nothing in
    # their way (amos_mfma_ceiling, the kernel's own instruction shape), right behind the timed
    # steps so that the chip is at the same clock
    # (an error of that side measurement must not cost the line: it is then reported as null)
    try:
        sustained = mfma_ceiling(da, db, [(16, 1, 0, 0)], launches=20, repeats=2)[0]["tflops"]
        sustained_note = ("amos_mfma_ceiling: v_mfma_f32_16x16x32_f16 on random fp16 U[-1,1] operands, no memory "
                          "traffic, same run (python bench.py --mfma-ceiling)")
    except _lib.AmosError as e:
        sustained, sustained_note = None, "amos_mfma_ceiling failed: %s" % e
    line = {
        "metric": METRIC, "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "fp16 GEMM M=N=K=8192, fp32 accumulate, row-major A, column-major B "
                               "(BASELINE configs[1])",
                   "kernel": ops.kernel_name(_lib.AMOS_OP_GEMM, desc, cfg),
                   "tile": "%dx%d" % (cfg.tile_i, cfg.tile_j), "split_k": cfg.split_k,
                   "clock_ramp_launches": CLOCK_RAMP_LAUNCHES,
                   "pct_of_mfma_peak": 100.0 * value / PEAK_F16_TFLOPS},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_F16_TFLOPS,
                     "traffic": measured_traffic(ops.kernel_name(_lib.AMOS_OP_GEMM, desc, cfg)),
                     "kernel_us": per_launch * 1e6,
                     "sustained_peak": sustained,
                     "frac_of_sustained_peak": achieved / sustained if sustained else None,
                     "sustained_peak_note": sustained_note},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_gemm(a, b)
    if not args.no_per_op:
        # every configuration of the path in the same run, each next to the CPU loop nest on a slab
        # of the same workload: the 8192^3 product from the measurement above, the others timed here
        del da, db, dc
        torch.cuda.empty_cache()
        per_op = [{"config": "C2 fp16 GEMM 8192^3 (ntn)", "kernel": line["config"]["kernel"],
                   "gpu_us": per_launch * 1e6, "tflops": achieved,
                   "pct_mfma_peak": 100 * achieved / PEAK_F16_TFLOPS,
                   "pct_hbm_roof": 100 * (2 * n * n * 2 + n * n * 4) / (PEAK_HBM_GBS * 1e9) / per_launch,
                   "bound": "mfma", "frac": achieved / PEAK_F16_TFLOPS}]
        if "cpu_baseline" in line:
            cb = line["cpu_baseline"]
            per_op[0]["cpu"] = {"threads1_tflops": cb["value"], "threadsN_tflops": cb["all_cores"]["value"],
                                "cores": cb["all_cores"]["cores"], "extrapolated_from": cb["sample"].split("=")[-1]}
        for r in run_all_configs(cpu=not args.no_cpu, only=("C3 fp16", "C4 int8", "C5a fp16", "C5b fp16")):
            row = {k: r[k] for k in ("config", "kernel", "split_k", "gpu_us", "tflops", "pct_mfma_peak",
                                     "pct_hbm_roof", "bound", "frac")}
            for k in ("traffic_bytes", "gpu_us_weights_packed_once"):
                if r.get(k) is not None:
                    row[k] = r[k]
            if "cpu" in r:
                row["cpu"] = {k: r["cpu"][k] for k in ("threads1_tflops", "threadsN_tflops", "cores",
                                                       "extrapolated_from")}
            per_op.append(row)
        per_op[0]["traffic_bytes"] = line["roofline"]["traffic"]
        line["per_op"] = per_op
        line["per_op_note"] = ("gpu_us: mean seconds per call by HIP events (time_evaluator loop, mean over "
                                         "its repeats), every launch of a call included; frac: fraction of the roof "
                                         "that binds (bound); tflops: TFLOP/s (int8: TOP/s); cpu: the "
                                         "te_literal loop nest (gcc -O3) on a slab, scaled linearly; traffic_bytes: HBM-side "
                                         "bytes per launch of the main kernel from the counter summaries under profiles/; "
                                         "gpu_us_weights_packed_once: the same convolution where the owner of the weights "
                                         "packed them once (no packing launch in the call)")
    if args.report:
        with open(args.report, "w") as f:
            json.dump(run_all_configs(cpu=not args.no_cpu, only=args.report_only), f, indent=1)
    if args.model_check:
        with open(args.model_check, "w") as f:
            json.dump(model_check(), f, indent=1)
    if args.network:
        with open(args.network, "w") as f:
            json.dump(network_report(networks=tuple(args.networks.split(","))), f, indent=1)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
