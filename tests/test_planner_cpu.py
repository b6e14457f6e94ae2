"""CPU tests of the host side: model graph, planner, plan format, schedule.

Golden files under tests/golden/plans/ are the reference's own tutorial
fixtures (examples/tutorial/*.json, data files).  The planner must reproduce
default_plan.json and model.json byte for byte (the older fixtures carry no
"Architecture" key, model_json.cpp:259-271 added it later).
"""
import json
import os

import pytest

import ark_amd
from ark_amd import Model, reset_ids, ArkmiError, plan_schedule, schedule_tasks
from oracle import plan_oracle as P

GOLD = os.path.join(os.path.dirname(__file__), "golden", "plans")


def gold(name):
    with open(os.path.join(GOLD, name)) as f:
        return f.read()


def ffn_model():
    """The SwiGLU FFN of examples/tutorial/plan_tutorial.py (b1, s512, 4096 -> 11008 -> 4096, fp16)."""
    reset_ids()
    m = Model()
    x = m.tensor([1, 512, 4096], "fp16")
    w1 = m.tensor([11008, 4096], "fp16")
    w2 = m.tensor([4096, 11008], "fp16")
    w3 = m.tensor([11008, 4096], "fp16")
    x1 = m.matmul(x, w1, trans_other=True)
    sig = m.sigmoid(x1, m.tensor(x1.shape, "fp16"))
    x1s = m.mul(x1, sig)
    x2 = m.matmul(x, w3, trans_other=True)
    x3 = m.mul(x1s, x2)
    m.matmul(x3, w2, trans_other=True)
    return m


def strip_arch(plan_text):
    return plan_text.replace('  "Architecture": "CUDA_80",\n', "")


# ---------------------------------------------------------------- golden files
def test_default_plan_golden_byte_for_byte():
    m = ffn_model()
    plan = m.plan(arch="CUDA_80", num_processors=108)
    assert strip_arch(plan) == gold("default_plan.json")
    j = json.loads(plan)
    assert [ti["Ops"][0]["Config"]["NumTasks"] for ti in j["TaskInfos"]] == [172, 88064, 88064, 172, 88064, 64]
    assert [pg["ProcessorRange"] for pg in j["ProcessorGroups"]] == [[0, 108]] * 5 + [[0, 64]]


def test_model_json_golden_byte_for_byte():
    m = ffn_model()
    assert m.verify()
    m.compress()
    assert m.serialize() == gold("model.json")
    names = [n["Op"]["Name"] for n in json.loads(m.serialize())["Nodes"]]
    assert names == ["matmul", "sigmoid", "mul", "matmul_1", "mul_1", "matmul_2"]


def test_model_file_round_trip_plans_like_the_model_that_wrote_it():
    """The reference's model file is the hand-over format at the boundary: model.json (written by
    ark::Model::serialize, examples/tutorial/model.json) read back through arkmi_model_from_json
    serializes to the same bytes and plans to default_plan.json byte for byte."""
    from ark_amd import Model, ArkmiError
    m = Model.from_json(gold("model.json"))
    assert m.serialize() == gold("model.json")
    assert strip_arch(m.plan(arch="CUDA_80", num_processors=108)) == gold("default_plan.json")
    # tensors of the file are addressable by id, and new ops do not reuse ids of the file
    j = json.loads(gold("model.json"))
    ids = {t["Id"] for n in j["Nodes"] for k in ("ReadTensors", "WriteTensors", "ResultTensors") for t in n["Op"][k]}
    last = m.tensor_by_id(max(ids))
    assert last.shape == [1, 512, 4096] and last.dtype == "fp16"
    extra = m.relu(last)
    assert extra.id not in ids and extra.buffer_id not in {
        t["Buffer"]["Id"] for n in j["Nodes"] for k in ("ReadTensors", "WriteTensors", "ResultTensors") for t in n["Op"][k]}
    # the same file planned for this backend's architecture: the gfx950 rules apply
    m2 = Model.from_json(gold("model.json"))
    p950 = json.loads(m2.plan(arch="ROCM_950", num_processors=256))
    assert p950["Architecture"] == "ROCM_950" and p950["NumWarpsPerProcessor"] == 8
    # malformed files are model errors
    for bad in ("{", "{}", json.dumps({"Rank": 0, "WorldSize": 1, "Nodes": [{"Id": 0}]})):
        with pytest.raises(ArkmiError) as e:
            Model.from_json(bad)
        assert e.value.kind == "ModelError", bad


def test_plan_oracle_reproduces_golden():
    m = ffn_model()
    model = m.dump(compressed=True, with_context=True)
    ours = P.plan(model, "CUDA_80", 108)
    ref = json.loads(gold("default_plan.json"))
    ref["Architecture"] = "CUDA_80"
    assert ours == ref
    # and the product planner agrees with the oracle on another target
    assert json.loads(m.plan(arch="ROCM_942", num_processors=304)) == P.plan(model, "ROCM_942", 304)


def test_config_rule_reproduces_larger_tile_plan():
    """plan_1_larger_tile.json was made with the rule of plan_tutorial.py:285-300
    (Sigmoid/Mul get 128x256 tiles and 8 warps); restated here."""
    def rule(op_json, arch):
        op = json.loads(op_json)
        if op["Type"] in ("Sigmoid", "Mul"):
            ps = op["ResultTensors"][0]["PaddedShape"]
            if len(ps) < 2 or ps[-2] % 128 or ps[-1] % 256:
                return ""
            return json.dumps({"NumWarps": 8, "SramBytes": 0, "Tile": [128, 256],
                               "NumTasks": ps[-2] // 128 * ps[-1] // 256})
        return ""

    m = ffn_model()
    ours = json.loads(m.plan(arch="CUDA_80", num_processors=108, config_rules=[rule]))
    ref = json.loads(gold("plan_1_larger_tile.json"))
    del ours["Architecture"]
    # This older fixture names its last op "matmul_1" a second time (it predates
    # the current naming counter) and orders tensor keys differently; apart
    # from op names the content is equal.
    for plan in (ours, ref):
        for ti in plan["TaskInfos"]:
            for op in ti["Ops"]:
                del op["Name"]
    assert ours == ref


def test_rule_exceptions_are_swallowed():
    def bad(op_json, arch):
        raise RuntimeError("boom")
    m = ffn_model()
    # a Python exception cannot cross the C boundary; the wrapper turns it into "decline"
    def guarded(op_json, arch):
        try:
            return bad(op_json, arch)
        except RuntimeError:
            return ""
    assert strip_arch(m.plan(arch="CUDA_80", num_processors=108, config_rules=[guarded])) == gold("default_plan.json")


# ---------------------------------------------------------------- schedule (codegen rules)
def schedule_of(plan_text):
    """Normalises the product's schedule JSON to the oracle's tuple form."""
    out = []
    for st in plan_schedule(plan_text)["Steps"]:
        if st["Kind"] == "Barrier":
            out.append(("barrier", *st["ProcessorRange"]))
        else:
            out.append(("tasks", *st["Args"]))
    return out


@pytest.mark.parametrize("name", ["default_plan.json", "plan_1_larger_tile.json", "plan_2_split_k.json",
                                  "plan_3_overwrite.json"])
def test_schedule_matches_oracle_on_tutorial_plans(name):
    plan = json.loads(gold(name))
    plan.setdefault("Architecture", "CUDA_80")
    text = json.dumps(plan)
    ours = schedule_of(text)
    want = P.schedule(plan)
    assert ours == want
    grid = plan["NumProcessors"]
    for i, st in enumerate(want):
        if st[0] != "tasks":
            continue
        seen = []
        for block in range(grid):
            for k in range(st[9]):
                ids = schedule_tasks(text, i, block, k)
                assert ids == P.task_ids(st, block, grid, k)
                seen += ids
        assert sorted(seen) == list(range(st[5], st[6]))  # every task exactly once


def test_schedule_default_plan_barriers_by_hand():
    """Six groups: five on [0,108) then one on [0,64): the rule emits one
    barrier over [0,108) before groups 2-5 and — because [0,108) sticks out of
    [0,64) — a barrier over [0,108) followed by none over [0,64) before the last."""
    plan = json.loads(gold("default_plan.json"))
    plan["Architecture"] = "CUDA_80"
    kinds = [(s[0], s[1], s[2]) for s in P.schedule(plan)]
    assert kinds == [("tasks", 0, 108), ("barrier", 0, 108), ("tasks", 0, 108), ("barrier", 0, 108),
                     ("tasks", 0, 108), ("barrier", 0, 108), ("tasks", 0, 108), ("barrier", 0, 108),
                     ("tasks", 0, 108), ("barrier", 0, 108), ("tasks", 0, 64)]


def test_schedule_split_k_runs_disjoint_ranges_concurrently():
    plan = json.loads(gold("plan_2_split_k.json"))
    plan["Architecture"] = "CUDA_80"
    sch = P.schedule(plan)
    ranges = [(s[1], s[2]) for s in sch if s[0] == "tasks"]
    assert (0, 64) in ranges and (64, 108) in ranges
    i = ranges.index((0, 64))
    # the two K-halves sit next to each other in the schedule with no barrier between them
    flat = [(s[0], s[1], s[2]) for s in sch]
    a = flat.index(("tasks", 0, 64))
    assert flat[a + 1] == ("tasks", 64, 108)


def test_slots_and_not_enough_resources():
    plan = json.loads(gold("default_plan.json"))
    plan["Architecture"] = "CUDA_80"
    # elementwise groups: WarpRange [0,1], 1 warp per task -> 1 slot
    st = [s for s in P.schedule(plan) if s[0] == "tasks"][1]
    assert st[9] == 1 and st[10] == 1
    plan["ProcessorGroups"][0]["ResourceGroups"][0]["SramRange"] = [0, 1000]
    with pytest.raises(ArkmiError) as e:
        plan_schedule(json.dumps(plan))
    assert e.value.kind == "PlanError" and "not enough resources" in str(e.value)


def test_plan_format_verification():
    plan = json.loads(gold("default_plan.json"))
    with pytest.raises(ArkmiError) as e:
        plan_schedule(json.dumps(plan))       # no Architecture key
    assert e.value.kind == "PlanError" and "Architecture" in str(e.value)
    plan["Architecture"] = "CUDA_80"
    del plan["TaskInfos"][0]["Ops"][0]["Config"]
    with pytest.raises(ArkmiError) as e:
        plan_schedule(json.dumps(plan))
    assert e.value.kind == "PlanError"


# ---------------------------------------------------------------- planner contexts (planner_test.cpp)
def _ctx_model():
    m = Model()
    t0 = m.tensor([1], "fp32")
    t1 = m.tensor([1], "fp32")
    return m, m.add(t0, t1)


@pytest.mark.parametrize("member,key", [("processor_range", "ProcessorRange"), ("warp_range", "WarpRange"),
                                        ("sram_range", "SramRange")])
def test_planner_context_ranges(member, key):
    m, t2 = _ctx_model()
    with m.planner_context(**{member: [0, 4]}) as ctx:
        t3 = m.relu(t2)
        assert ctx.get(key) == "[0,4]"
        ctx.call(member, [2, 4])
        m.sqrt(t3)
        assert ctx.get(key) == "[2,4]"
        with pytest.raises(ArkmiError) as e:
            ctx.call(member, [0, 4])   # not a subset of [2,4]
        assert e.value.kind == "PlanError"
    with m.planner_context(**{member: [2, 6, 2]}) as ctx:
        m.exp(t2)
        assert ctx.get(key) == "[2,6,2]"
    assert m.verify()
    nodes = m.dump(compressed=True, with_context=True)["Nodes"]
    assert len(nodes) == 4
    assert nodes[0]["Context"] == {}
    assert nodes[1]["Context"][key] == [0, 4]
    assert nodes[2]["Context"][key] == [2, 4]
    assert nodes[3]["Context"][key] == [2, 6, 2]


def test_planner_context_sync_and_config():
    m, t2 = _ctx_model()
    with m.planner_context(sync=False) as ctx:
        t3 = m.relu(t2)
        ctx.call("sync", True)          # ignored with a warning
        m.sqrt(t3)
        assert ctx.get("Sync") == "false"
    with m.planner_context(sync=True) as ctx:
        m.exp(t2)
        assert ctx.get("Sync") == "true"
    with m.planner_context(config={"key0": "val1"}) as ctx:
        m.relu(t2)
        ctx.call("config", {"key1": "val2"})
        m.relu(t2)
        assert json.loads(ctx.get("Config")) == {"key0": "val1", "key1": "val2"}
    nodes = m.dump(compressed=True, with_context=True)["Nodes"]
    assert [n["Context"].get("Sync") for n in nodes[:4]] == [None, False, False, True]
    assert nodes[4]["Context"]["Config"] == {"key0": "val1"}
    assert nodes[5]["Context"]["Config"] == {"key0": "val1", "key1": "val2"}


def test_planner_context_plan():
    """planner_test.cpp:285-319."""
    m = Model()
    cfg = {"NumWarps": 1, "SramBytes": 0, "NumTasks": 1, "Tile": [1, 64]}
    with m.planner_context(processor_range=[0, 2], warp_range=[0, 4], sram_range=[0, 0], sync=False,
                           config=cfg):
        t0 = m.tensor([1024], "fp32")
        t1 = m.mul(t0, 0.5)
        m.add(t0, t1)
    for arch, n in (("ROCM_950", 256), ("CUDA_80", 108)):
        plan = json.loads(m.plan(arch=arch, num_processors=n, pretty=False))
        assert plan["NumProcessors"] == 2 and plan["NumWarpsPerProcessor"] == 4
        assert len(plan["TaskInfos"]) == 1
        ti = plan["TaskInfos"][0]
        assert ti["NumWarps"] == 1 and ti["SramBytes"] == 0
        assert [o["Type"] for o in ti["Ops"]] == ["ScalarMul", "Add"]
        assert ti["Ops"][0]["Config"] == cfg and ti["Ops"][1]["Config"] == cfg
        assert ti["Ops"][0]["Args"] == {"Factor": {"FLOAT": 0.5}}
        assert P.plan(m.dump(compressed=True, with_context=True), arch, n) == plan


def test_float_args_round_trip_in_plan_text():
    m = Model()
    t = m.tensor([64], "fp32")
    m.mul(t, 0.7)
    m.div(t, 0.7)
    text = m.plan(arch="ROCM_950", num_processors=256, pretty=False)
    assert '"Factor":{"FLOAT":0.699999988079071}' in text          # double(float(0.7)), shortest form
    assert '"Factor":{"FLOAT":1.4285714626312256}' in text         # float(1 / 0.7f)


# ---------------------------------------------------------------- gfx950 defaults (this backend's design)
def test_rocm950_default_configs():
    m = Model()
    a = m.tensor([4096, 4096], "fp16")
    b = m.tensor([4096, 4096], "fp16")
    m.matmul(a, b)
    x = m.tensor([16384, 4096], "fp16")
    m.reduce_sum(x, -1)
    m.softmax(x)
    w = m.tensor([4096], "fp32")
    m.rmsnorm(x, w, 1e-6)
    m.add(x, x)
    plan = json.loads(m.plan(arch="ROCM_950", num_processors=256))
    assert plan["NumProcessors"] == 256 and plan["NumWarpsPerProcessor"] == 8
    cfgs = [ti["Ops"][0]["Config"] for ti in plan["TaskInfos"]]
    assert cfgs[0] == {"NumWarps": 8, "SramBytes": 131072, "TileShapeMNK": [256, 256, 64], "NumTasks": 256}
    # 16384 rows on 256 CUs x 8 waves: 8 rows per wave, one task per CU
    assert cfgs[1] == {"NumWarps": 8, "ImplType": "WarpWise", "SramBytes": 0, "RowsPerWave": 8, "NumTasks": 256}
    for c in cfgs[2:4]:
        assert c["RowsPerWave"] == 8 and c["NumTasks"] == 256
    # few rows: one per wave, so that every CU still gets a task
    m2 = Model()
    m2.rmsnorm(m2.tensor([1, 2048, 4096], "bf16"), m2.tensor([1, 1, 4096], "fp32"), 1e-6)
    c2 = json.loads(m2.plan(arch="ROCM_950", num_processors=256))["TaskInfos"][0]["Ops"][0]["Config"]
    assert c2["RowsPerWave"] == 1 and c2["NumTasks"] == 256
    assert cfgs[4] == {"NumWarps": 8, "SramBytes": 0, "Tile": [8, 4096], "NumTasks": 2048}
    # one resident slot per CU: every task sequence has exactly one 8-wave slot
    for st in plan_schedule(json.dumps(plan))["Steps"]:
        if st["Kind"] == "TaskSeq":
            assert st["Args"][8] == 1 and st["Args"][9] == 8


def test_rocm950_matmul_tile_choice():
    def tile(mm, nn, kk, batch=()):
        m = Model()
        a = m.tensor(list(batch) + [mm, kk], "bf16")
        b = m.tensor([nn, kk], "bf16")
        m.matmul(a, b, trans_other=True)
        c = json.loads(m.plan(arch="ROCM_950", num_processors=256))["TaskInfos"][0]["Ops"][0]["Config"]
        return c["TileShapeMNK"][:2], c["NumTasks"]
    assert tile(8192, 11008, 4096) == ([256, 256], 32 * 43)
    assert tile(2048, 4096, 2048) == ([256, 128], 8 * 32)         # 256x256 would leave CUs idle
    assert tile(4096, 2048, 2048) == ([256, 128], 16 * 16)        # (of the half-size tiles the 256-row one first)
    assert tile(2048, 4096, 4096) == ([256, 256], 2 * 8 * 16)     # K of 4096 or more: large tiles, K split in two
    assert tile(128 * 33, 4096, 4096) == ([128, 256], 33 * 16)    # 33 tile rows of 128: no 256-row tile divides
    assert tile(2048, 4096, 11008 // 128 * 128) == ([256, 256], 2 * 8 * 16)  # long K: large tiles, K split in two
    assert tile(2048, 2048, 128, batch=(1, 32)) == ([256, 256], 32 * 64)
    assert tile(512, 512, 64) == ([128, 128], 16)
    with pytest.raises(ArkmiError) as e:
        tile(100, 512, 64)
    assert e.value.kind == "PlanError"


def test_follower_takes_producer_tiles_through_a_reshape():
    """An elementwise op fused (sync=False) behind a GEMM whose output it sees through a
    reshape takes the GEMM's tiles and says so with "ViewAs"; an operand that cannot be
    addressed over the GEMM's [rows, cols] keeps the op on its own tiling."""
    m = Model()
    x, w = m.tensor([1, 256, 512], "bf16"), m.tensor([1024, 512], "bf16")
    f = m.tensor([1, 256, 1, 128], "bf16")
    with m.planner_context(sync=False):
        y = m.reshape(m.matmul(x, w, trans_other=True), [1, 256, 8, 128])
        m.rope(y, f)
    plan = json.loads(m.plan(arch="ROCM_950", num_processors=256))
    assert len(plan["TaskInfos"]) == 1
    mm, rope = plan["TaskInfos"][0]["Ops"]
    assert rope["Config"]["ViewAs"] == [1, 1, 256, 1024]
    assert rope["Config"]["Tile"] == mm["Config"]["TileShapeMNK"][:2]
    assert rope["Config"]["NumTasks"] == mm["Config"]["NumTasks"]

    m = Model()
    x, w = m.tensor([1, 256, 512], "bf16"), m.tensor([1024, 512], "bf16")
    g = m.tensor([1, 1, 8, 1], "bf16")  # per-head factor: neither dense nor periodic over 1024 columns
    with m.planner_context(sync=False):
        y = m.reshape(m.matmul(x, w, trans_other=True), [1, 256, 8, 128])
        m.mul(y, g)
    plan = json.loads(m.plan(arch="ROCM_950", num_processors=256))
    assert "ViewAs" not in plan["TaskInfos"][0]["Ops"][1]["Config"]


def test_rocm950_matmul_tiles_and_split_k():
    """The gfx950 default rule: the largest tile that still gives every CU a task; an output that
    gives 256x256 tiles to between half and all of the CUs keeps them and splits K in two."""
    def cfg(M, N, K, ncu=256, trans_other=False):
        m = Model()
        a, b = m.tensor([M, K], "bf16"), m.tensor([N, K] if trans_other else [K, N], "bf16")
        m.matmul(a, b, trans_other=trans_other)
        return json.loads(m.plan(arch="ROCM_950", num_processors=ncu))["TaskInfos"][0]["Ops"][0]["Config"]
    c = cfg(4096, 4096, 4096)
    assert c["TileShapeMNK"][:2] == [256, 256] and c["NumTasks"] == 256 and "SplitK" not in c
    c = cfg(2048, 4096, 8192, trans_other=True)
    assert c["TileShapeMNK"][:2] == [256, 256] and c["SplitK"] == 2 and c["NumTasks"] == 256
    c = cfg(2048, 4096, 11008, trans_other=True)
    assert c["SplitK"] == 2 and c["NumTasks"] == 256
    c = cfg(2048, 4096, 4096)                       # from K = 4096 on the split beats smaller tiles
    assert c["TileShapeMNK"][:2] == [256, 256] and c["SplitK"] == 2 and c["NumTasks"] == 256
    c = cfg(2048, 4096, 2048)                       # below, the exchange of partial sums costs what the tile gains
    assert "SplitK" not in c and c["TileShapeMNK"][:2] == [256, 128] and c["NumTasks"] == 256
    c = cfg(2048, 2048, 4096)                       # 64 large tiles: smaller tiles fill the chip instead
    assert "SplitK" not in c and c["TileShapeMNK"][:2] == [128, 128]
    c = cfg(2048, 4096, 8192, ncu=128)              # a plan for 128 processors has a tile for each already
    assert "SplitK" not in c and c["TileShapeMNK"][:2] == [256, 256] and c["NumTasks"] == 128
