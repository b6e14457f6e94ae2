"""Externally authored plan files run as they are: the reference's tutorial plans
(examples/tutorial/plan_1_larger_tile.json, plan_2_split_k.json, plan_3_overwrite.json; written
for 108 processors, split-K through strided views on disjoint processor ranges, buffer reuse)
go into the Executor with one field added (they predate the "Architecture" field that the
reference's own plan check requires, ark/model/model_json.cpp:259-266), and every buffer they write is compared with a numpy/oracle
interpretation of the same plan, op by op in plan order.  ARK_ENFORCE_PLAN_PATH substitutes a
plan file for the plan the caller passes (ark/api/executor.cpp:892-895)."""
import collections
import json
import os

import numpy as np
import pytest

from helpers import make

pytestmark = pytest.mark.gpu
PLANS = os.path.join(os.path.dirname(__file__), "golden", "plans")
View = collections.namedtuple("View", "buffer_id dtype shape strides offsets")
_DT = {"FP16": "fp16", "BF16": "bf16", "FP32": "fp32"}


def _view(tj):
    return View(tj["Buffer"]["Id"], _DT[tj["DataType"]], list(tj["Shape"]), list(tj["Strides"]), list(tj["Offsets"]))


def _whole(v):
    """The view that spans the whole buffer a view lives in."""
    return View(v.buffer_id, v.dtype, list(v.strides), list(v.strides), [0] * len(v.strides))


def _window(buf, v):
    """numpy window of a view into its buffer's dense array (shape = the view's strides)."""
    return buf[tuple(slice(o, o + s) for o, s in zip(v.offsets, v.shape))]


def _interpret(oracle, plan, buffers):
    for ti in plan["TaskInfos"]:
        for op in ti["Ops"]:
            ins = [_window(buffers[_view(t).buffer_id], _view(t)) for t in op["ReadTensors"]]
            out_v = _view(op["WriteTensors"][0])
            dt = out_v.dtype
            kind = op["Type"]
            if kind == "Matmul":
                a, b = ins
                res = oracle.matmul(a.reshape(-1, a.shape[-1]), b, dt,
                                    trans_a=op["Args"]["TransposeInput"]["BOOL"],
                                    trans_b=op["Args"]["TransposeOther"]["BOOL"]).reshape(out_v.shape)
            elif kind in ("Add", "Mul", "Sub", "Div"):
                res = oracle.binary(ins[0], ins[1], kind.lower(), dt)
            elif kind in ("Sigmoid", "Relu", "Exp", "Gelu", "Sqrt", "Rsqrt"):
                res = oracle.unary(ins[0], kind.lower(), dt)
            else:
                raise AssertionError(f"plan interpreter: op {kind} not covered")
            _window(buffers[out_v.buffer_id], out_v)[...] = res.reshape(out_v.shape)


def _buffers_of(plan):
    """buffer id -> (whole-buffer view, written?, read before written?)"""
    info, written = {}, set()
    for ti in plan["TaskInfos"]:
        for op in ti["Ops"]:
            for t in op["ReadTensors"]:
                v = _view(t)
                info.setdefault(v.buffer_id, [_whole(v), False, False])
                if v.buffer_id not in written:
                    info[v.buffer_id][2] = True
            for t in op["WriteTensors"]:
                v = _view(t)
                info.setdefault(v.buffer_id, [_whole(v), False, False])
                info[v.buffer_id][1] = True
                written.add(v.buffer_id)
    return info


def _run_plan_file(oracle, name, monkeypatch=None, enforce=False, tmp_path=None):
    import ark_amd
    from ark_amd import Executor
    plan = json.loads(open(os.path.join(PLANS, name)).read())
    plan.setdefault("Architecture", "ROCM_950")
    text = json.dumps(plan)
    info = _buffers_of(plan)
    host = {}
    for i, (bid, (whole, _, is_input)) in enumerate(sorted(info.items())):
        if is_input:
            scale = 1.0 if i == 0 else 0.02
            host[bid] = make(oracle, tuple(whole.shape), whole.dtype, 900 + i, "uniform", -scale, scale)
        else:
            host[bid] = np.zeros(whole.shape, np.float16 if whole.dtype == "fp16" else np.uint16)
    if enforce:
        path = tmp_path / name
        path.write_text(text)
        monkeypatch.setenv("ARK_ENFORCE_PLAN_PATH", str(path))
        ark_amd.init()  # the environment is read once per process: read it again
        given = json.dumps({"Rank": 0, "WorldSize": 1, "Architecture": "ROCM_950", "NumProcessors": 1,
                            "NumWarpsPerProcessor": 8, "TaskInfos": [], "ProcessorGroups": []})
    else:
        given = text
    try:
        ex = Executor(given, device_id=0).compile()
    finally:
        if enforce:
            monkeypatch.delenv("ARK_ENFORCE_PLAN_PATH")
            ark_amd.init()
    for bid, (whole, _, is_input) in info.items():
        if is_input:
            ex.tensor_write(whole, host[bid])
    ex.launch()
    ex.run(2)
    ex.wait()
    got = {bid: ex.tensor_read(whole) for bid, (whole, was_written, _) in info.items() if was_written}
    einfo = ex.info()
    ex.stop()
    _interpret(oracle, plan, host)
    return got, host, einfo


def _compare(oracle, got, want):
    import llama_ref as R
    assert got
    for bid, a in got.items():
        # fp16 chains of up to three matmuls (K up to 11008) whose intermediates round to fp16:
        # judged like the composed Llama blocks, by the largest and the rms difference relative
        # to the output's scale, 1e-2 (cf. examples/llama/model_test.py:231-233)
        mx, rms = R.composite_error(oracle, want[bid], a, "fp16")
        assert mx <= 1e-2 and rms <= 1e-2, (bid, mx, rms)


@pytest.mark.parametrize("name", ["plan_1_larger_tile.json", "plan_2_split_k.json", "plan_3_overwrite.json"])
def test_tutorial_plan_runs_as_written(oracle, name):
    got, want, info = _run_plan_file(oracle, name)
    assert info["num_processors"] == 108
    _compare(oracle, got, want)


def test_enforced_plan_path_replaces_the_given_plan(oracle, monkeypatch, tmp_path):
    got, want, info = _run_plan_file(oracle, "plan_2_split_k.json", monkeypatch, enforce=True, tmp_path=tmp_path)
    assert info["num_processors"] == 108  # the file's plan, not the empty one that was passed
    _compare(oracle, got, want)
