"""Tensor-level entry points over the C ABI.

PyTorch-ROCm only supplies device memory and the current stream here; every
computation goes through libamos_mi355x.so.  There is no CPU or eager fallback:
tensors that are not on a HIP device are rejected.
"""
import ctypes

import torch

from . import _lib
from ._lib import (AMOS_OP_BGEMM, AMOS_OP_CONV2D, AMOS_OP_CONV3D, AMOS_OP_GEMM, BGemmDesc, ConvDesc,
                   GemmDesc, KernelConfig, check)

_IN_CODE = {torch.float16: _lib.AMOS_F16, torch.bfloat16: _lib.AMOS_BF16, torch.int8: _lib.AMOS_I8}
_OUT_OF = {torch.float16: torch.float32, torch.bfloat16: torch.float32, torch.int8: torch.int32}
_OUT_CODE = {torch.float32: _lib.AMOS_F32, torch.int32: _lib.AMOS_I32}


def _need_device(*tensors):
    for t in tensors:
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise RuntimeError("amos_amd runs on the GPU only: got a tensor on %s"
                               % (getattr(t, "device", type(t)),))
        if not t.is_contiguous():
            raise ValueError("operands must be contiguous")


def _stream_ptr(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


_CODE_DTYPE = {_lib.AMOS_F16: torch.float16, _lib.AMOS_BF16: torch.bfloat16, _lib.AMOS_I8: torch.int8,
               _lib.AMOS_F32: torch.float32, _lib.AMOS_I32: torch.int32}


def _gemm_spans(g, batch=1, sa=0, sb=0, sc=0):
    """elements the three operands of a (batched) GEMM descriptor reach"""
    a = (g.K - 1) * g.lda + g.M if g.trans_a else (g.M - 1) * g.lda + g.K
    b = (g.N - 1) * g.ldb + g.K if g.trans_b else (g.K - 1) * g.ldb + g.N
    c = (g.M - 1) * g.ldc + g.N
    return (batch - 1) * sa + a, (batch - 1) * sb + b, (batch - 1) * sc + c


def operand_spans(op, desc):
    """(elements of in0, in1, out the kernels may touch, input dtype, output dtype) of a descriptor"""
    if op == AMOS_OP_GEMM:
        g, spans = desc, _gemm_spans(desc)
    elif op == AMOS_OP_BGEMM:
        g, spans = desc.g, _gemm_spans(desc.g, desc.batch, desc.stride_a, desc.stride_b, desc.stride_c)
    else:
        g = desc
        groups = max(1, desc.groups)
        xs = (desc.N, desc.C, desc.D, desc.H, desc.W)
        ws = (desc.K, desc.C // groups, desc.T, desc.R, desc.S)
        o = conv_out_shape(xs, ws, (desc.stride_d, desc.stride_h, desc.stride_w),
                           (desc.pad_d, desc.pad_h, desc.pad_w), (desc.dil_d, desc.dil_h, desc.dil_w))
        prod = lambda t: int(torch.Size(t).numel())
        spans = (prod(xs), prod(ws), prod(o))
    return spans, _CODE_DTYPE.get(g.in_dtype), _CODE_DTYPE.get(g.out_dtype)


def check_operands(op, desc, in0, in1, out):
    """Refuse, before any launch, arrays that do not hold what the descriptor says: the kernels
    take raw pointers, so a short or wrongly typed array would be read or written out of bounds.
    (The reference's argument binder asserts shape and dtype at call time the same way.)"""
    (n0, n1, nout), in_dt, out_dt = operand_spans(op, desc)
    for what, t, need, dt in (("first input", in0, n0, in_dt), ("second input", in1, n1, in_dt),
                              ("output", out, nout, out_dt)):
        if t.dtype != dt:
            raise ValueError("%s is %s, the descriptor says %s" % (what, t.dtype, dt))
        if t.numel() < need:
            raise ValueError("%s holds %d elements, the descriptor reaches %d" % (what, t.numel(), need))
        if t.device != in0.device:
            raise ValueError("%s is on %s, the first input on %s" % (what, t.device, in0.device))


def _check_out(out, shape, dtype, like):
    """a caller-supplied output: exactly the result's shape and type, on the operands' device"""
    if tuple(out.shape) != tuple(shape) or out.dtype != dtype or out.device != like.device:
        raise ValueError("out must be a %s tensor of shape %s on %s: got %s %s on %s"
                         % (dtype, tuple(shape), like.device, out.dtype, tuple(out.shape), out.device))


def make_config(config):
    """None | KernelConfig | dict(tile_i=, tile_j=, split_k=) -> KernelConfig or None"""
    if config is None or isinstance(config, KernelConfig):
        return config
    c = KernelConfig()
    c.tile_i = int(config.get("tile_i", 0))
    c.tile_j = int(config.get("tile_j", 0))
    c.split_k = int(config.get("split_k", 0))
    c.pipeline = int(config.get("pipeline", 0))
    c.reserved[0] = int(config.get("flags", 0))
    return c


def _cfg_ref(cfg):
    return ctypes.byref(cfg) if cfg is not None else None


def make_epilogue(add, out_shape, out_dtype):
    """None | tensor of the output's shape -> Epilogue (out = acc + add) or None.  `add` is fp32,
    fp16 or bf16 for fp32 outputs, int32 for int32 outputs."""
    if add is None:
        return None
    _need_device(add)
    if tuple(add.shape) != tuple(out_shape):
        raise ValueError("the added operand has shape %s, the output %s" % (tuple(add.shape), tuple(out_shape)))
    codes = {torch.float32: _lib.AMOS_F32, torch.float16: _lib.AMOS_F16, torch.bfloat16: _lib.AMOS_BF16,
             torch.int32: _lib.AMOS_I32}
    ok = (torch.int32,) if out_dtype == torch.int32 else (torch.float32, torch.float16, torch.bfloat16)
    if add.dtype not in ok:
        raise ValueError("cannot add a %s operand to a %s output" % (add.dtype, out_dtype))
    e = _lib.Epilogue()
    e.kind, e.dtype, e.operand, e.ld, e.stride = _lib.AMOS_EPI_ADD, codes[add.dtype], add.data_ptr(), 0, 0
    return e


def _epi_ref(e):
    return ctypes.byref(e) if e is not None else None


def gemm_desc(M, N, K, in_dtype, trans_a=False, trans_b=False, lda=None, ldb=None, ldc=None):
    d = GemmDesc()
    d.M, d.N, d.K = M, N, K
    d.in_dtype = _IN_CODE[in_dtype]
    d.out_dtype = _OUT_CODE[_OUT_OF[in_dtype]]
    d.trans_a, d.trans_b = int(trans_a), int(trans_b)
    d.lda = lda if lda is not None else (M if trans_a else K)
    d.ldb = ldb if ldb is not None else (K if trans_b else N)
    d.ldc = ldc if ldc is not None else N
    return d


def conv_desc(x_shape, w_shape, in_dtype, stride, pad, dil, groups=1, layout="nchw"):
    """x_shape NCDHW, w_shape K,(C/groups),T,R,S (the logical extents, whatever the layout in
    memory); stride / pad / dil are 3-tuples"""
    d = ConvDesc()
    d.layout = _lib.LAYOUT_CODE[layout] if isinstance(layout, str) else int(layout)
    d.N, d.C, d.D, d.H, d.W = x_shape
    d.K, cg, d.T, d.R, d.S = w_shape
    if cg * groups != d.C:
        raise ValueError("weights have %d channels per group, activations %d channels in %d groups"
                         % (cg, d.C, groups))
    d.groups = groups
    d.stride_d, d.stride_h, d.stride_w = stride
    d.pad_d, d.pad_h, d.pad_w = pad
    d.dil_d, d.dil_h, d.dil_w = dil
    d.in_dtype = _IN_CODE[in_dtype]
    d.out_dtype = _OUT_CODE[_OUT_OF[in_dtype]]
    return d


def _tup(v, n, unit=None):
    if isinstance(v, (tuple, list)):
        assert len(v) == n
        return tuple(int(t) for t in v)
    return (int(v),) * n


def conv_out_shape(x_shape, w_shape, stride, pad, dil):
    out = []
    for ext, k, s, p, d in zip(x_shape[2:], w_shape[2:], stride, pad, dil):
        out.append((ext + 2 * p - ((k - 1) * d + 1)) // s + 1)
    return (x_shape[0], w_shape[0]) + tuple(out)


def gemm(a, b, trans_a=False, trans_b=False, out=None, config=None, stream=None, add=None):
    """C[M,N] = A(m,k) B(k,n) (+ add[M,N]); a is [M,K] ([K,M] if trans_a), b is [K,N] ([N,K] if trans_b)."""
    _need_device(a, b)
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    if (b.shape[1] if trans_b else b.shape[0]) != K or a.dtype != b.dtype:
        raise ValueError("operand shapes / dtypes do not agree")
    if out is None:
        out = torch.empty((M, N), dtype=_OUT_OF[a.dtype], device=a.device)
    _need_device(out)
    _check_out(out, (M, N), _OUT_OF[a.dtype], a)
    d = gemm_desc(M, N, K, a.dtype, trans_a, trans_b)
    cfg = make_config(config)
    epi = make_epilogue(add, (M, N), out.dtype)
    ws, ws_ptr, ws_bytes = _workspace(AMOS_OP_GEMM, d, cfg, a.device, stream)
    check(_lib.load().amos_run_fused(AMOS_OP_GEMM, ctypes.byref(d), _cfg_ref(cfg), _epi_ref(epi), a.data_ptr(),
                                     b.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes, _stream_ptr(stream)))
    return out


def bgemm_desc(batch, M, N, K, in_dtype, trans_a=False, trans_b=False):
    d = BGemmDesc()
    d.batch = batch
    d.g = gemm_desc(M, N, K, in_dtype, trans_a, trans_b)
    d.stride_a, d.stride_b, d.stride_c = M * K, K * N, M * N
    return d


def bgemm(a, b, trans_a=False, trans_b=False, out=None, config=None, stream=None, add=None):
    """batched GEMM; a is [B,M,K] ([B,K,M] if trans_a), b is [B,K,N] ([B,N,K] if trans_b)."""
    _need_device(a, b)
    B = a.shape[0]
    M, K = (a.shape[2], a.shape[1]) if trans_a else a.shape[1:]
    N = b.shape[1] if trans_b else b.shape[2]
    if b.shape[0] != B or (b.shape[2] if trans_b else b.shape[1]) != K or a.dtype != b.dtype:
        raise ValueError("operand shapes / dtypes do not agree")
    if out is None:
        out = torch.empty((B, M, N), dtype=_OUT_OF[a.dtype], device=a.device)
    _need_device(out)
    _check_out(out, (B, M, N), _OUT_OF[a.dtype], a)
    d = bgemm_desc(B, M, N, K, a.dtype, trans_a, trans_b)
    cfg = make_config(config)
    epi = make_epilogue(add, (B, M, N), out.dtype)
    ws, ws_ptr, ws_bytes = _workspace(AMOS_OP_BGEMM, d, cfg, a.device, stream)
    check(_lib.load().amos_run_fused(AMOS_OP_BGEMM, ctypes.byref(d), _cfg_ref(cfg), _epi_ref(epi), a.data_ptr(),
                                     b.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes, _stream_ptr(stream)))
    return out


def workspace_bytes(op, desc, config=None):
    cfg = make_config(config)
    return int(_lib.load().amos_workspace_bytes(op, ctypes.byref(desc), _cfg_ref(cfg)))


def _workspace(op, desc, cfg, device, stream=None):
    """device scratch of amos_workspace_bytes() (conv: repacked weights); (tensor, ptr, bytes).
    The tensor is dropped as soon as the asynchronous launch returns, so it is allocated on the
    launch stream: the caching allocator then hands the block to later work of that stream only,
    which runs behind the kernel that still reads it."""
    need = _lib.load().amos_workspace_bytes(op, ctypes.byref(desc), _cfg_ref(cfg))
    if need == 0:
        return None, None, 0
    if stream is None:
        ws = torch.empty(need + 256, dtype=torch.uint8, device=device)
    else:
        with torch.cuda.stream(stream):
            ws = torch.empty(need + 256, dtype=torch.uint8, device=device)
    ptr = (ws.data_ptr() + 255) // 256 * 256
    return ws, ptr, need


def logical_conv_shapes(x_shape, w_shape, layout):
    """(N,C,D,H,W), (K,C/groups,T,R,S) of operands stored in `layout` (4-d operands: D = T = 1)"""
    code = _lib.LAYOUT_CODE[layout]
    x_shape, w_shape = tuple(int(e) for e in x_shape), tuple(int(e) for e in w_shape)
    if len(x_shape) == 4:
        x_shape = {0: x_shape[:2] + (1,) + x_shape[2:], 1: x_shape[:1] + (1,) + x_shape[1:],
                   2: (1,) + x_shape}[code]
        w_shape = w_shape[:2] + (1,) + w_shape[2:] if code == 0 else (1,) + w_shape
    if code == 0:
        return x_shape, w_shape
    t, r, s, c, k = w_shape
    if code == 1:
        n, d, h, w_, cx = x_shape
    else:
        d, h, w_, n, cx = x_shape
    return (n, cx, d, h, w_), (k, c, t, r, s)


def stored_conv_out_shape(oshape, layout, ndim):
    """NKDPQ extents -> the output's shape as stored in `layout` (ndim 4: without the depth)"""
    code = _lib.LAYOUT_CODE[layout]
    n, k, od, op, oq = oshape
    sp = (op, oq) if ndim == 4 else (od, op, oq)
    return {0: (n, k) + sp, 1: (n,) + sp + (k,), 2: sp + (n, k)}[code]


def conv2d(x, w, stride=1, pad=0, dil=1, out=None, config=None, stream=None, add=None, groups=1,
           layout="nchw"):
    """layout nchw: x NCHW, w K,(C/groups),R,S -> NKPQ; nhwc: x NHWC, w RSCK -> NPQK; hwnc:
    x HWNC, w RSCK -> PQNK (+ add of the output's shape)"""
    _need_device(x, w)
    st, pd, dl = (1,) + _tup(stride, 2), (0,) + _tup(pad, 2), (1,) + _tup(dil, 2)
    xs, ws = logical_conv_shapes(x.shape, w.shape, layout)
    if xs[1] != ws[1] * groups or x.dtype != w.dtype:
        raise ValueError("operand shapes / dtypes do not agree")
    oshape = conv_out_shape(xs, ws, st, pd, dl)
    if out is None:
        out = torch.empty(stored_conv_out_shape(oshape, layout, 4), dtype=_OUT_OF[x.dtype], device=x.device)
    _need_device(out)
    _check_out(out, stored_conv_out_shape(oshape, layout, 4), _OUT_OF[x.dtype], x)
    d = conv_desc(xs, ws, x.dtype, st, pd, dl, groups, layout)
    cfg = make_config(config)
    ws, ws_ptr, ws_bytes = _workspace(AMOS_OP_CONV2D, d, cfg, x.device, stream)
    epi = make_epilogue(add, tuple(out.shape), out.dtype)
    check(_lib.load().amos_run_fused(AMOS_OP_CONV2D, ctypes.byref(d), _cfg_ref(cfg), _epi_ref(epi), x.data_ptr(),
                                     w.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes, _stream_ptr(stream)))
    return out


def conv3d(x, w, stride=1, pad=0, dil=1, out=None, config=None, stream=None, add=None, groups=1,
           layout="ncdhw"):
    """layout ncdhw: x NCDHW, w K,(C/groups),T,R,S -> NKDPQ; ndhwc: x NDHWC, w TRSCK -> NDPQK;
    dhwnc: x DHWNC, w TRSCK -> DPQNK (+ add of the output's shape)"""
    _need_device(x, w)
    st, pd, dl = _tup(stride, 3), _tup(pad, 3), _tup(dil, 3)
    xs, ws = logical_conv_shapes(x.shape, w.shape, layout)
    if xs[1] != ws[1] * groups or x.dtype != w.dtype:
        raise ValueError("operand shapes / dtypes do not agree")
    oshape = conv_out_shape(xs, ws, st, pd, dl)
    if out is None:
        out = torch.empty(stored_conv_out_shape(oshape, layout, 5), dtype=_OUT_OF[x.dtype], device=x.device)
    _need_device(out)
    _check_out(out, stored_conv_out_shape(oshape, layout, 5), _OUT_OF[x.dtype], x)
    d = conv_desc(xs, ws, x.dtype, st, pd, dl, groups, layout)
    cfg = make_config(config)
    ws, ws_ptr, ws_bytes = _workspace(AMOS_OP_CONV3D, d, cfg, x.device, stream)
    epi = make_epilogue(add, tuple(out.shape), out.dtype)
    check(_lib.load().amos_run_fused(AMOS_OP_CONV3D, ctypes.byref(d), _cfg_ref(cfg), _epi_ref(epi), x.data_ptr(),
                                     w.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes, _stream_ptr(stream)))
    return out


class Gather(object):
    """device side of a dimension-separable gather (amos_gather): `tables[d][o]` = source element
    offset contributed by index o of output dimension d, or -1 where the result is zero"""

    def __init__(self, out_shape, tables, dtype, in_elems, device):
        self.out_shape = [int(e) for e in out_shape]
        self.dtype = dtype
        if not 1 <= len(self.out_shape) <= 5 or [len(t) for t in tables] != self.out_shape:
            raise ValueError("gather needs one table per output dimension, at most five")
        flat, offsets = [], []
        for t in tables:
            offsets.append(len(flat))
            flat.extend(int(e) for e in t)
        self.tables = torch.tensor(flat, dtype=torch.int32, device=device)
        d = _lib.GatherDesc()
        d.ndim, d.elem_bytes, d.in_elems = len(self.out_shape), torch.empty(0, dtype=dtype).element_size(), int(in_elems)
        for k, (ext, off) in enumerate(zip(self.out_shape, offsets)):
            d.out_shape[k], d.table_offset[k] = ext, off
        self.desc = d

    def _check(self, src, out):
        _need_device(src, out)
        if src.numel() != self.desc.in_elems or src.dtype != self.dtype or not src.is_contiguous():
            raise ValueError("gather source must be a dense %s tensor of %d elements" % (self.dtype, self.desc.in_elems))
        if list(out.shape) != self.out_shape or out.dtype != self.dtype or not out.is_contiguous():
            raise ValueError("gather output must be a dense %s tensor of shape %s" % (self.dtype, self.out_shape))

    def __call__(self, src, out=None, stream=None):
        if out is None:
            out = torch.empty(self.out_shape, dtype=self.dtype, device=src.device)
        self._check(src, out)
        check(_lib.load().amos_gather(ctypes.byref(self.desc), src.data_ptr(), self.tables.data_ptr(),
                                      out.data_ptr(), _stream_ptr(stream)))
        return out

    def time(self, src, out, number=100, repeat=1, min_repeat_ms=150, stream=None):
        self._check(src, out)
        res = (ctypes.c_double * repeat)()
        check(_lib.load().amos_time_gather(ctypes.byref(self.desc), src.data_ptr(), self.tables.data_ptr(),
                                           out.data_ptr(), _stream_ptr(stream), number, repeat, min_repeat_ms, res))
        return list(res)


class Eltwise(object):
    """device side of an element-wise stage in front of an operand (amos_eltwise): `program` is a
    list of ("load", k) / ("const", value) / "add" / "sub" / "mul" in postfix order"""

    _DT = {torch.float16: _lib.AMOS_F16, torch.bfloat16: _lib.AMOS_BF16, torch.int8: _lib.AMOS_I8}

    def __init__(self, program, n_inputs, dtype, elems):
        d = _lib.EltwiseDesc()
        d.dtype, d.n_inputs, d.elems = self._DT[dtype], int(n_inputs), int(elems)
        consts = []
        code = {"add": _lib.AMOS_ELT_ADD, "sub": _lib.AMOS_ELT_SUB, "mul": _lib.AMOS_ELT_MUL}
        if len(program) > 16:
            raise ValueError("element-wise stage of %d operations (16 at most)" % len(program))
        for k, step in enumerate(program):
            if isinstance(step, tuple) and step[0] == "load":
                d.program[k] = _lib.AMOS_ELT_LOAD | (int(step[1]) << 8)
            elif isinstance(step, tuple) and step[0] == "const":
                if len(consts) == 4:
                    raise ValueError("element-wise stage with more than four constants")
                d.program[k] = _lib.AMOS_ELT_CONST | (len(consts) << 8)
                consts.append(float(step[1]))
            else:
                d.program[k] = code[step]
        d.n_ops = len(program)
        for k, c in enumerate(consts):
            d.consts[k] = c
        self.desc, self.dtype, self.n_inputs = d, dtype, int(n_inputs)

    def _args(self, inputs, out):
        _need_device(out, *inputs)
        if len(inputs) != self.n_inputs or any(t.numel() != self.desc.elems or t.dtype != self.dtype or
                                               not t.is_contiguous() for t in list(inputs) + [out]):
            raise ValueError("element-wise stage wants %d dense %s tensors of %d elements" %
                             (self.n_inputs, self.dtype, self.desc.elems))
        return (ctypes.c_void_p * self.n_inputs)(*[t.data_ptr() for t in inputs])

    def __call__(self, inputs, out=None, stream=None):
        if out is None:
            out = torch.empty_like(inputs[0])
        ptrs = self._args(inputs, out)
        check(_lib.load().amos_eltwise(ctypes.byref(self.desc), ptrs, out.data_ptr(), _stream_ptr(stream)))
        return out

    def time(self, inputs, out, number=100, repeat=1, min_repeat_ms=150, stream=None):
        ptrs = self._args(inputs, out)
        res = (ctypes.c_double * repeat)()
        check(_lib.load().amos_time_eltwise(ctypes.byref(self.desc), ptrs, out.data_ptr(), _stream_ptr(stream),
                                            number, repeat, min_repeat_ms, res))
        return list(res)


def _epilogue_for(op, desc, add, out):
    """Epilogue for an operand laid out like the output the descriptor describes"""
    if add is None:
        return None
    if add.numel() != out.numel():
        raise ValueError("the added operand has %d elements, the output %d" % (add.numel(), out.numel()))
    epi = make_epilogue(add, tuple(add.shape), out.dtype)
    if op == AMOS_OP_GEMM:
        epi.ld = desc.ldc
    elif op == AMOS_OP_BGEMM:
        epi.ld, epi.stride = desc.g.ldc, desc.stride_c
    return epi


def run_desc(op, desc, in0, in1, out, config=None, stream=None, add=None):
    """launch an op from its C descriptor (leading dimensions and batch strides as the descriptor
    says; the tensors only supply the device memory)"""
    _need_device(in0, in1, out)
    check_operands(op, desc, in0, in1, out)
    cfg = make_config(config)
    ws, ws_ptr, ws_bytes = _workspace(op, desc, cfg, in0.device, stream)
    epi = _epilogue_for(op, desc, add, out)
    check(_lib.load().amos_run_fused(op, ctypes.byref(desc), _cfg_ref(cfg), _epi_ref(epi), in0.data_ptr(),
                                     in1.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes, _stream_ptr(stream)))
    return out


def time_op(op, desc, in0, in1, out, config=None, number=100, repeat=1, min_repeat_ms=150, stream=None,
            add=None):
    """mean seconds per launch, `repeat` values (time_evaluator semantics)"""
    _need_device(in0, in1, out)
    check_operands(op, desc, in0, in1, out)
    cfg = make_config(config)
    res = (ctypes.c_double * repeat)()
    ws, ws_ptr, ws_bytes = _workspace(op, desc, cfg, in0.device, stream)
    epi = _epilogue_for(op, desc, add, out)
    check(_lib.load().amos_time_fused(op, ctypes.byref(desc), _cfg_ref(cfg), _epi_ref(epi), in0.data_ptr(),
                                      in1.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes, _stream_ptr(stream),
                                      number, repeat, min_repeat_ms, res))
    return list(res)


def default_config(op, desc):
    cfg = KernelConfig()
    check(_lib.load().amos_default_config(op, ctypes.byref(desc), ctypes.byref(cfg)))
    return cfg


def kernel_name(op, desc, config=None):
    cfg = make_config(config)
    name = _lib.load().amos_kernel_name(op, ctypes.byref(desc), _cfg_ref(cfg))
    if name is None:
        raise _lib.AmosError(-3, _lib.load().amos_last_error().decode())
    return name.decode()


def device_info():
    info = _lib.DeviceInfo()
    check(_lib.load().amos_device_info(ctypes.byref(info)))
    return info
