"""Whole-network driver: every tensorisable layer of a network is mapped and tuned as a
subgraph of its own, the best (mapping, kernel configuration) of each is kept on disk, and the
network's cost is the sum over its layers.

Stands where the reference's tensor_graph dispatch stands for this path
(benchmark/amos/mapping_resnet18_tensorcore.py:20-60;
python/tvm/tensor_graph/core/auto_schedule/auto_schedule.py:1090-1160 `get_best_schedule`):
`AutoScheduleMultiGraphDispatch.add_graph_task / auto_schedule / get_schedules / ready` and
`evaluate_graph` keep their call shapes; a subgraph's log directory is
`<log_dir>/<network>/at-<network>:subgraph<i>/` and holds `best_mappings_<name>.txt` with the
reference's line `{"mapping": key, "params": {...}, "cost": seconds}`.  Layers without a
reduction on the matrix cores (batch norm, ReLU, pooling, the residual additions) are the part
the reference hands to its fallback scheduler; they are not run here and are listed as skipped.
"""
import json
import os

from .. import te
from ..te import tir
from .auto_tensorize import auto_tensorize_v4, get_schedule
from .compute_transform import MappingApplier, MappingGenerator
from .hw_abstraction import compute_dag_from_tensors
from .intrin_match import get_match_results
from .policy import all_fit
from .schedule import KernelParams, MI355XScheduleApplier, MI355XScheduleGenerator

MAX_FLOAT = 1e10


class SubGraph(object):
    """one tensorisable layer: `tensors` = its TE inputs + output, `count` = how often the
    network runs a layer of exactly this shape"""

    def __init__(self, name, tensors, count=1, note=""):
        self.name, self.tensors, self.count, self.note = name, list(tensors), int(count), note

    @property
    def dag(self):
        return compute_dag_from_tensors([self.tensors[-1]])


# ---- layer builders (the reference's spellings: benchmark/amos/mapping_conv2d_tensorcore.py:7-42,
# mapping_gemm_tensorcore.py:7-15) ------------------------------------------------------------------
def conv2d_nchw(N, C, H, W, K, R, S, stride, padding, in_dtype="float16", out_dtype="float32"):
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, C, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    rc = te.reduce_axis([0, C], name="rc")
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - R) // stride + 1, (pW - S) // stride + 1
    Conv = te.compute([N, K, P, Q], lambda n, k, p, q: te.sum(
        (Pad[n, rc, p * stride + rr, q * stride + rs] * B[k, rc, rr, rs]).astype(out_dtype),
        axis=[rc, rr, rs]), name="Conv")
    return [A, B, Conv]


def dense(M, N, K, in_dtype="float16", out_dtype="float32"):
    """activations [M, K] times weights stored [N, K] (torch's Linear)"""
    A = te.placeholder([M, K], dtype=in_dtype, name="A")
    B = te.placeholder([N, K], dtype=in_dtype, name="B")
    rk = te.reduce_axis([0, K], name="k")
    C = te.compute([M, N], lambda i, j: te.sum((A[i, rk] * B[j, rk]).astype(out_dtype), axis=rk), name="C")
    return [A, B, C]


def resnet18(batch=1, in_dtype="float16", out_dtype="float32", num_classes=1000):
    """the convolutions and the classifier of ResNet-18 at 224x224
    (python/tvm/tensor_graph/testing/models/resnet.py:122-215), equal shapes merged"""
    b = batch
    layers = [
        ("conv1 7x7/2 3->64 @224", conv2d_nchw(b, 3, 224, 224, 64, 7, 7, 2, 3, in_dtype, out_dtype), 1),
        ("layer1 3x3 64->64 @56", conv2d_nchw(b, 64, 56, 56, 64, 3, 3, 1, 1, in_dtype, out_dtype), 4),
        ("layer2 3x3/2 64->128 @56", conv2d_nchw(b, 64, 56, 56, 128, 3, 3, 2, 1, in_dtype, out_dtype), 1),
        ("layer2 1x1/2 64->128 @56", conv2d_nchw(b, 64, 56, 56, 128, 1, 1, 2, 0, in_dtype, out_dtype), 1),
        ("layer2 3x3 128->128 @28", conv2d_nchw(b, 128, 28, 28, 128, 3, 3, 1, 1, in_dtype, out_dtype), 3),
        ("layer3 3x3/2 128->256 @28", conv2d_nchw(b, 128, 28, 28, 256, 3, 3, 2, 1, in_dtype, out_dtype), 1),
        ("layer3 1x1/2 128->256 @28", conv2d_nchw(b, 128, 28, 28, 256, 1, 1, 2, 0, in_dtype, out_dtype), 1),
        ("layer3 3x3 256->256 @14", conv2d_nchw(b, 256, 14, 14, 256, 3, 3, 1, 1, in_dtype, out_dtype), 3),
        ("layer4 3x3/2 256->512 @14", conv2d_nchw(b, 256, 14, 14, 512, 3, 3, 2, 1, in_dtype, out_dtype), 1),
        ("layer4 1x1/2 256->512 @14", conv2d_nchw(b, 256, 14, 14, 512, 1, 1, 2, 0, in_dtype, out_dtype), 1),
        ("layer4 3x3 512->512 @7", conv2d_nchw(b, 512, 7, 7, 512, 3, 3, 1, 1, in_dtype, out_dtype), 3),
        ("fc 512->%d" % num_classes, dense(b, num_classes, 512, in_dtype, out_dtype), 1),
    ]
    return _subgraphs("resnet18", layers)


def batched_matmul(B, M, N, K, trans_b, in_dtype="float16", out_dtype="float32"):
    """B independent products A[b] (M x K) times B[b] (stored N x K if trans_b, else K x N)"""
    A = te.placeholder([B, M, K], dtype=in_dtype, name="A")
    Bt = te.placeholder([B, N, K] if trans_b else [B, K, N], dtype=in_dtype, name="B")
    rk = te.reduce_axis([0, K], name="k")
    C = te.compute([B, M, N], lambda b, i, j: te.sum(
        (A[b, i, rk] * (Bt[b, j, rk] if trans_b else Bt[b, rk, j])).astype(out_dtype), axis=rk), name="C")
    return [A, Bt, C]


def depthwise_conv2d_nchw(N, C, H, W, R, S, stride, padding, in_dtype="float16", out_dtype="float32"):
    """one 3x3 filter per channel (benchmark/amos/mapping_depthwiseconv2d_tensorcore.py:7-48, K = C)"""
    pH, pW = H + 2 * padding, W + 2 * padding
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([C, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    B_reshaped = te.compute([C, 1, R, S], lambda k_o, k_i, r, s: B[k_o + k_i, r, s])
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - R) // stride + 1, (pW - S) // stride + 1
    Conv = te.compute([N, C, 1, P, Q], lambda n, k_o, k_i, p, q: te.sum(
        (Pad[n, k_o, p * stride + rr, q * stride + rs] * B_reshaped[k_o, k_i, rr, rs]).astype(out_dtype),
        axis=[rr, rs]), name="Conv")
    Reshaped = te.compute([N, C, P, Q], lambda n, k, p, q: Conv[n, k, 0, p, q], name="Reshaped")
    return [A, B, Reshaped]


def grouped_conv2d_nchw(N, C, H, W, K, R, S, stride, padding, groups, in_dtype="float16", out_dtype="float32"):
    """convolution in channel groups (benchmark/amos/mapping_groupedconv2d_tensorcore.py:7-60)"""
    pH, pW = H + 2 * padding, W + 2 * padding
    cg, kg = C // groups, K // groups
    A = te.placeholder([N, C, H, W], dtype=in_dtype, name="A")
    B = te.placeholder([K, cg, R, S], dtype=in_dtype, name="B")
    Pad = te.compute([N, C, pH, pW], lambda n, c, h, w: tir.if_then_else(
        tir.all(h >= padding, h - padding < H, w >= padding, w - padding < W),
        A[n, c, h - padding, w - padding], tir.const(0.0, A.dtype)), name="Pad")
    A_reshaped = te.compute([N, groups, cg, pH, pW], lambda n, c_o, c_i, r, s: Pad[n, c_o * cg + c_i, r, s])
    B_reshaped = te.compute([groups, kg, cg, R, S], lambda k_o, k_i, c, r, s: B[k_o * kg + k_i, c, r, s])
    rc = te.reduce_axis([0, cg], name="rc")
    rr = te.reduce_axis([0, R], name="rr")
    rs = te.reduce_axis([0, S], name="rs")
    P, Q = (pH - R) // stride + 1, (pW - S) // stride + 1
    Conv = te.compute([N, groups, kg, P, Q], lambda n, k_o, k_i, p, q: te.sum(
        (A_reshaped[n, k_o, rc, p * stride + rr, q * stride + rs] * B_reshaped[k_o, k_i, rc, rr, rs]).astype(out_dtype),
        axis=[rc, rr, rs]), name="Conv")
    Reshaped = te.compute([N, K, P, Q], lambda n, k, p, q: Conv[n, k // kg, k % kg, p, q], name="Reshaped")
    return [A, B, Reshaped]


def _subgraphs(net, layers):
    return [SubGraph("%s:subgraph%d" % (net, i), ts, cnt, note) for i, (note, ts, cnt) in enumerate(layers)]


def resnet50(batch=1, in_dtype="float16", out_dtype="float32", num_classes=1000):
    """the convolutions and the classifier of ResNet-50 at 224x224 (the stride of a down-sampling
    bottleneck on its 3x3, python/tvm/tensor_graph/testing/models/resnet.py:60-215), equal shapes merged"""
    b, d = batch, (in_dtype, out_dtype)
    layers = [("conv1 7x7/2 3->64 @224", conv2d_nchw(b, 3, 224, 224, 64, 7, 7, 2, 3, *d), 1)]
    cin, hw = 64, 56
    for stage, (mid, blocks) in enumerate([(64, 3), (128, 4), (256, 6), (512, 3)]):
        cout, stride = 4 * mid, (1 if stage == 0 else 2)
        layers += [
            ("stage%d 1x1 %d->%d @%d" % (stage + 1, cin, mid, hw), conv2d_nchw(b, cin, hw, hw, mid, 1, 1, 1, 0, *d), 1),
            ("stage%d 3x3/%d %d->%d @%d" % (stage + 1, stride, mid, mid, hw), conv2d_nchw(b, mid, hw, hw, mid, 3, 3, stride, 1, *d), 1),
            ("stage%d 1x1/%d %d->%d @%d (shortcut)" % (stage + 1, stride, cin, cout, hw), conv2d_nchw(b, cin, hw, hw, cout, 1, 1, stride, 0, *d), 1),
        ]
        hw //= stride
        layers += [
            ("stage%d 1x1 %d->%d @%d" % (stage + 1, mid, cout, hw), conv2d_nchw(b, mid, hw, hw, cout, 1, 1, 1, 0, *d), blocks),
            ("stage%d 1x1 %d->%d @%d" % (stage + 1, cout, mid, hw), conv2d_nchw(b, cout, hw, hw, mid, 1, 1, 1, 0, *d), blocks - 1),
            ("stage%d 3x3 %d->%d @%d" % (stage + 1, mid, mid, hw), conv2d_nchw(b, mid, hw, hw, mid, 3, 3, 1, 1, *d), blocks - 1),
        ]
        cin = cout
    layers.append(("fc 2048->%d" % num_classes, dense(b, num_classes, 2048, *d), 1))
    return _subgraphs("resnet50", layers)


def mobilenet_v1(batch=1, in_dtype="float16", out_dtype="float32", num_classes=1000):
    """MobileNet-V1 at 224x224 (python/tvm/tensor_graph/testing/models/mobilenet_v1.py): the first
    convolution, thirteen depthwise 3x3 + pointwise 1x1 pairs, the classifier"""
    b, d = batch, (in_dtype, out_dtype)
    layers = [("conv 3x3/2 3->32 @224", conv2d_nchw(b, 3, 224, 224, 32, 3, 3, 2, 1, *d), 1)]
    cfg = [(32, 64, 1), (64, 128, 2), (128, 128, 1), (128, 256, 2), (256, 256, 1), (256, 512, 2)] + \
          [(512, 512, 1)] * 5 + [(512, 1024, 2), (1024, 1024, 1)]
    hw, seen = 112, {}
    for cin, cout, stride in cfg:
        key = (cin, cout, stride, hw)
        if key in seen:
            for i in seen[key]:
                layers[i] = (layers[i][0], layers[i][1], layers[i][2] + 1)
        else:
            seen[key] = [len(layers), len(layers) + 1]
            layers.append(("depthwise 3x3/%d %d @%d" % (stride, cin, hw),
                           depthwise_conv2d_nchw(b, cin, hw, hw, 3, 3, stride, 1, *d), 1))
            layers.append(("pointwise %d->%d @%d" % (cin, cout, hw // stride),
                           conv2d_nchw(b, cin, hw // stride, hw // stride, cout, 1, 1, 1, 0, *d), 1))
        hw //= stride
    layers.append(("fc 1024->%d" % num_classes, dense(b, num_classes, 1024, *d), 1))
    return _subgraphs("mobilenet_v1", layers)


def bert_base(batch=1, seq=512, in_dtype="float16", out_dtype="float32", blocks=12, heads=12, d_model=768, d_ff=3072):
    """the matrix products of BERT-base (benchmark/amos/mapping_bertbase_tensorcore.py:19-46;
    python/tvm/tensor_graph/testing/models/transformer.py:290-303): per block four d_model x d_model
    projections, the attention scores and context (batched over batch x heads), two feed-forward
    layers"""
    rows, d = batch * seq, (in_dtype, out_dtype)
    layers = [
        ("projection %d->%d (Q, K, V, O)" % (d_model, d_model), dense(rows, d_model, d_model, *d), 4 * blocks),
        ("scores Q K^T, %d x (%d x %d x %d)" % (batch * heads, seq, seq, d_model // heads),
         batched_matmul(batch * heads, seq, seq, d_model // heads, True, *d), blocks),
        ("context P V, %d x (%d x %d x %d)" % (batch * heads, seq, d_model // heads, seq),
         batched_matmul(batch * heads, seq, d_model // heads, seq, False, *d), blocks),
        ("feed-forward %d->%d" % (d_model, d_ff), dense(rows, d_ff, d_model, *d), blocks),
        ("feed-forward %d->%d" % (d_ff, d_model), dense(rows, d_model, d_ff, *d), blocks),
    ]
    return _subgraphs("bertbase", layers)


def shufflenet(batch=1, in_dtype="float16", out_dtype="float32", num_classes=1000, groups=3):
    """ShuffleNet (groups = 3) at 224x224 (python/tvm/tensor_graph/testing/models/shufflenet.py:68-185):
    the first convolution; per unit a grouped 1x1, a depthwise 3x3 (strided in the first unit of a
    stage, whose output channels are the stage's minus its input's: the rest is a pooled copy) and
    a grouped 1x1; the classifier.  Channel shuffles, pooling and concatenation have no reduction."""
    b, d = batch, (in_dtype, out_dtype)
    layers = [("conv 3x3/2 3->24 @224", conv2d_nchw(b, 3, 224, 224, 24, 3, 3, 2, 1, *d), 1)]
    cin, hw = 24, 56
    for stage, (cout, repeats) in enumerate([(240, 3), (480, 7), (960, 3)]):
        tag = "stage%d" % (stage + 2)
        grown, mid = cout - cin, (cout - cin) // 4
        layers += [
            ("%s grouped 1x1 %d->%d @%d" % (tag, cin, mid, hw), grouped_conv2d_nchw(b, cin, hw, hw, mid, 1, 1, 1, 0, groups, *d), 1),
            ("%s depthwise 3x3/2 %d @%d" % (tag, mid, hw), depthwise_conv2d_nchw(b, mid, hw, hw, 3, 3, 2, 1, *d), 1),
            ("%s grouped 1x1 %d->%d @%d" % (tag, mid, grown, hw // 2), grouped_conv2d_nchw(b, mid, hw // 2, hw // 2, grown, 1, 1, 1, 0, groups, *d), 1),
        ]
        hw //= 2
        mid = cout // 4
        layers += [
            ("%s grouped 1x1 %d->%d @%d" % (tag, cout, mid, hw), grouped_conv2d_nchw(b, cout, hw, hw, mid, 1, 1, 1, 0, groups, *d), repeats),
            ("%s depthwise 3x3 %d @%d" % (tag, mid, hw), depthwise_conv2d_nchw(b, mid, hw, hw, 3, 3, 1, 1, *d), repeats),
            ("%s grouped 1x1 %d->%d @%d" % (tag, mid, cout, hw), grouped_conv2d_nchw(b, mid, hw, hw, cout, 1, 1, 1, 0, groups, *d), repeats),
        ]
        cin = cout
    layers.append(("fc 960->%d" % num_classes, dense(b, num_classes, 960, *d), 1))
    return _subgraphs("shufflenet", layers)


def mi_lstm(batch=1, in_dtype="float16", out_dtype="float32", input_size=512, hidden=1024):
    """one step of the MI-LSTM cell (python/tvm/tensor_graph/testing/models/MI_LSTM.py:71-124;
    benchmark/amos/mapping_milstm_tensorcore.py:19-26): four gate projections of the hidden state,
    four of the input, the classifier; the gates' element-wise arithmetic has no reduction"""
    d = (in_dtype, out_dtype)
    layers = [
        ("gate projection of h %d->%d (f, i, z, o)" % (hidden, hidden), dense(batch, hidden, hidden, *d), 4),
        ("gate projection of x %d->%d (f, i, z, o)" % (input_size, hidden), dense(batch, hidden, input_size, *d), 4),
        ("classifier %d->10" % hidden, dense(batch, 10, hidden, *d), 1),
    ]
    return _subgraphs("milstm", layers)


NETWORKS = {"resnet18": None, "resnet50": resnet50, "mobilenet_v1": mobilenet_v1, "bertbase": bert_base,
            "shufflenet": shufflenet, "milstm": mi_lstm}


SKIPPED_RESNET18 = ("batch norm x20, ReLU x17, max pool, global average pool, residual additions x8: "
                    "no reduction that maps to the matrix cores (the reference's fallback scheduler)")


# ---- one subgraph -------------------------------------------------------------------------------------
class AutoTensorizeContext(object):
    def __init__(self, name, top_log_dir, subgraph, measure_option, transform_strict=True):
        self.name, self.subgraph, self.measure_option = name, subgraph, measure_option
        self.log_dir = os.path.join(top_log_dir, "at-" + name)
        os.makedirs(self.log_dir, exist_ok=True)
        self.best_file = os.path.join(self.log_dir, "best_mappings_%s.txt" % name)
        self.transform_strict = transform_strict
        self.result = None

    @staticmethod
    def can_use(subgraph, target="hip"):
        return len(get_match_results(subgraph.dag, target)) > 0

    def auto_schedule(self, trials):
        """one round of mapping exploration + kernel-configuration tuning; keeps the best on disk"""
        res = auto_tensorize_v4(self.subgraph.dag, "hip", self.name.replace(":", "_") + ".log",
                                self.measure_option, schedule_log_dir=self.log_dir, trials=trials,
                                repeat_rounds=1, transform_strict=self.transform_strict, search_group_size=1)
        if not res.defined():
            return
        known = self._read_best()
        if known is None or res.perf < known["cost"]:
            with open(self.best_file, "w") as fout:
                fout.write(json.dumps({"mapping": res.mapping.as_key(), "params": res.params.to_json(),
                                       "cost": res.perf}))
        self.result = res

    def _read_best(self):
        if os.path.isfile(self.best_file):
            with open(self.best_file, "r") as fin:
                for line in fin:
                    if line.strip():
                        return json.loads(line)
        return None

    def get_best_schedule(self):
        """(sch, args, cost in seconds) from the best-mappings file, or (None, None, MAX_FLOAT)"""
        best = self._read_best()
        if best is None:
            return None, None, MAX_FLOAT
        match_result, _ = all_fit(get_match_results(self.subgraph.dag, "hip"))
        app = MappingApplier(match_result, strict=self.transform_strict)
        for record in MappingGenerator(match_result).get_all():
            if record.as_key() == best["mapping"]:
                state = app.apply(record)
                gen = MI355XScheduleGenerator(match_result, state, log_file=None, verbose_init=False)
                sch_app = MI355XScheduleApplier(match_result, gen.lowered)
                sch, args = get_schedule(sch_app, KernelParams.from_json(best["params"]))
                return sch, args, best["cost"]
        return None, None, MAX_FLOAT


# ---- the network ---------------------------------------------------------------------------------------
class AutoScheduleMultiGraphDispatch(object):
    working_set = {}

    @classmethod
    def add_graph_task(cls, name, multi_graph, measure_option, scheduler_option="auto_tensorize", trials=20,
                       log_dir="network_logs", transform_strict=True):
        if scheduler_option != "auto_tensorize":
            raise ValueError("only scheduler_option='auto_tensorize' exists here")
        top = os.path.join(log_dir, name)
        os.makedirs(top, exist_ok=True)
        ctxs, skipped = [], []
        for sg in multi_graph:
            if AutoTensorizeContext.can_use(sg):
                ctxs.append(AutoTensorizeContext(sg.name, top, sg, measure_option, transform_strict))
            else:
                print("Fallback to TG: no kernel family for", sg.name, flush=True)
                skipped.append(sg)
        tid = len(cls.working_set)
        cls.working_set[tid] = dict(name=name, contexts=ctxs, skipped=skipped, trials=trials)
        return tid

    @classmethod
    def auto_schedule(cls, tid):
        task = cls.working_set[tid]
        for ctx in task["contexts"]:
            print("Tuning", ctx.name, "(%s)" % ctx.subgraph.note, flush=True)
            ctx.auto_schedule(task["trials"])

    @classmethod
    def get_schedules(cls, tid):
        """{subgraph name: (sch, args, cost seconds)}"""
        return {ctx.name: ctx.get_best_schedule() for ctx in cls.working_set[tid]["contexts"]}

    @classmethod
    def ready(cls, tid):
        return all(sch is not None for sch, _, _ in cls.get_schedules(tid).values())


def evaluate_graph(multi_graph, sch_tensors, target="hip", dev_id=0, number=100, verbose=False, min_repeat_ms=50):
    """milliseconds of one pass over the network's tensorisable layers: every layer's module is
    built and timed on the device (time_evaluator), times multiplied by how often the layer occurs
    (reference: auto_tensorize.evaluate_graph as called in mapping_resnet18_tensorcore.py:58)"""
    from . import runtime
    from .measure import random_device_arrays
    total, rows = 0.0, []
    ctx = runtime.context(target, dev_id)
    for sg in multi_graph:
        if sg.name not in sch_tensors or sch_tensors[sg.name][0] is None:
            continue
        sch, args, _ = sch_tensors[sg.name]
        func = runtime.build(sch, args, target)
        in0, in1, out = random_device_arrays(func.lowered, dev_id)
        arrays = [None] * len(args)
        for k, i in enumerate(func.arg_index[:3]):
            if i is not None:
                arrays[i] = (in0, in1, out)[k]
        ms = func.time_evaluator(func.entry_name, ctx, number=number, min_repeat_ms=min_repeat_ms)(*arrays).mean * 1e3
        rows.append((sg.name, sg.note, sg.count, ms, func.lowered.flops(), func.get_source().split("\n")[0][3:]))
        total += ms * sg.count
        if verbose:
            print("%s (%s) x%d: %.4f ms, %s" % (sg.name, sg.note, sg.count, ms, rows[-1][-1]), flush=True)
    evaluate_graph.last_rows = rows
    return total


NETWORKS["resnet18"] = resnet18
