"""Whole-network flow on the GPU: ResNet-18's tensorisable layers through the dispatcher
(reference flow: benchmark/amos/mapping_resnet18_tensorcore.py:20-60)."""
import json
import os

import numpy as np
import pytest

import amos_amd.tvm as tvm
from amos_amd.tvm import auto_tensorize as at
from oracle import cpu_oracle as co

pytestmark = pytest.mark.gpu


def test_resnet18_dispatch(gpu, tmp_path, capsys):
    multi_graph = at.resnet18(batch=2)
    assert len(multi_graph) == 12 and sum(sg.count for sg in multi_graph) == 21     # 20 convolutions + fc
    opt = at.MeasureOptions(target="hip", timeout=100, number=3, min_repeat_ms=2)
    dispatch = at.AutoScheduleMultiGraphDispatch
    tid = dispatch.add_graph_task("resnet18", multi_graph, opt, scheduler_option="auto_tensorize", trials=1,
                                  log_dir=str(tmp_path), transform_strict=False)
    assert not dispatch.ready(tid)
    dispatch.auto_schedule(tid)
    assert dispatch.ready(tid)
    sch_tensors = dispatch.get_schedules(tid)
    # the reference's on-disk format: one JSON line per subgraph
    for sg in multi_graph:
        path = os.path.join(str(tmp_path), "resnet18", "at-" + sg.name, "best_mappings_%s.txt" % sg.name)
        obj = json.loads(open(path).read())
        assert set(obj) == {"mapping", "params", "cost"} and obj["mapping"].startswith("(") and 0 < obj["cost"] < 1
        assert set(obj["params"]) == {"tile_i", "tile_j", "split_k", "pipeline"}
    cost = at.evaluate_graph(multi_graph, sch_tensors, "hip", 0, 10, False, min_repeat_ms=5)
    rows = at.evaluate_graph.last_rows
    assert len(rows) == 12 and 0 < cost < 50 and abs(cost - sum(r[3] * r[2] for r in rows)) < 1e-9
    capsys.readouterr()
    # a second dispatcher over the same directory is ready without tuning, and its modules compute
    # what the layers say
    tid2 = dispatch.add_graph_task("resnet18", multi_graph, opt, trials=1, log_dir=str(tmp_path),
                                   transform_strict=False)
    assert dispatch.ready(tid2)
    again = dispatch.get_schedules(tid2)
    rng = np.random.default_rng(13)
    ctx = tvm.context("hip", 0)
    for idx in (2, 7, 11):       # a strided 3x3, a 14x14 3x3, the classifier
        sg = multi_graph[idx]
        sch, args, _ = again[sg.name]
        func = tvm.build(sch, args, "hip")
        feeds = [rng.uniform(-1, 1, [int(e) for e in t.shape]).astype(np.float16) for t in args[:-1]]
        out = tvm.nd.array(np.zeros([int(e) for e in args[-1].shape], dtype=np.float32), ctx)
        func(*[tvm.nd.array(f, ctx) for f in feeds], out)
        ctx.sync()
        if idx == 11:
            ref = feeds[0].astype(np.float64) @ feeds[1].astype(np.float64).T
        else:
            stride = 2 if idx == 2 else 1
            ref = co.lib_conv2d(feeds[0], feeds[1], "float16", stride, 1, 1, acc="float64")
        mx, mean = co.rel_errors(out.asnumpy(), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (sg.name, mx, mean)


def _by_note(multi_graph, text):
    found = [sg for sg in multi_graph if text in sg.note]
    assert found, text
    return found[0]


def test_other_networks_dispatch(gpu, tmp_path, capsys):
    """layers of ResNet-50, MobileNet-V1 and BERT-base that ResNet-18 has no like of, through the
    dispatcher: the 7x7 stem, a strided pointwise shortcut, depthwise 3x3 with and without a
    stride, the attention products"""
    r50, mb, bert = at.resnet50(2), at.mobilenet_v1(2), at.bert_base(1, seq=128)
    picked = [_by_note(r50, "conv1 7x7/2"), _by_note(r50, "stage2 1x1/2 256->512 @56 (shortcut)"),
              _by_note(r50, "stage4 1x1 2048->512 @7"),
              _by_note(mb, "depthwise 3x3/2 64 @112"), _by_note(mb, "depthwise 3x3/1 512 @14"),
              _by_note(mb, "pointwise 512->1024 @7"),
              _by_note(bert, "scores"), _by_note(bert, "context"), _by_note(bert, "feed-forward 3072->768")]
    opt = at.MeasureOptions(target="hip", timeout=100, number=3, min_repeat_ms=2)
    dispatch = at.AutoScheduleMultiGraphDispatch
    tid = dispatch.add_graph_task("mixed", picked, opt, trials=2, log_dir=str(tmp_path), transform_strict=False)
    dispatch.auto_schedule(tid)
    assert dispatch.ready(tid)
    sch_tensors = dispatch.get_schedules(tid)
    capsys.readouterr()
    rng = np.random.default_rng(29)
    ctx = tvm.context("hip", 0)
    for sg in picked:
        sch, args, _ = sch_tensors[sg.name]
        func = tvm.build(sch, args, "hip")
        feeds = [rng.uniform(-1, 1, [int(e) for e in t.shape]).astype(np.float16) for t in args[:-1]]
        out = tvm.nd.array(np.zeros([int(e) for e in args[-1].shape], dtype=np.float32), ctx)
        func(*[tvm.nd.array(f, ctx) for f in feeds], out)
        ctx.sync()
        a, b = [f.astype(np.float64) for f in feeds]
        if "depthwise" in sg.note:
            stride = 2 if "/2" in sg.note else 1
            ap = np.pad(a, ((0, 0), (0, 0), (1, 1), (1, 1)))
            p, q = out.shape[2], out.shape[3]
            ref = sum(ap[:, :, r:r + stride * (p - 1) + 1:stride, s:s + stride * (q - 1) + 1:stride] *
                      b[None, :, r, s, None, None] for r in range(3) for s in range(3))
        elif "scores" in sg.note:
            ref = np.einsum("bik,bjk->bij", a, b)
        elif "context" in sg.note:
            ref = np.einsum("bik,bkj->bij", a, b)
        elif "feed-forward" in sg.note:
            ref = a @ b.T
        else:
            stride = 2 if "/2" in sg.note else 1
            ref = co.lib_conv2d(feeds[0], feeds[1], "float16", stride, 3 if "7x7" in sg.note else 0, 1, acc="float64")
        mx, mean = co.rel_errors(out.asnumpy(), ref)
        assert mx <= 1e-2 and mean <= 1e-3, (sg.note, mx, mean)
    cost = at.evaluate_graph(picked, sch_tensors, "hip", 0, 5, False, min_repeat_ms=2)
    assert len(at.evaluate_graph.last_rows) == len(picked) and 0 < cost < 50
