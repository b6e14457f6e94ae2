"""The host side of the dependency counters without a GPU (arkmi_plan_analysis): which barriers
compile() replaces by counters, and the wait spans / signal maps it builds, recomputed here from
first principles (task -> rows by the ops' own tiling rules) for every task of the plans.
The reference places one sync_gpu between consecutive ops instead (ark/codegen.cpp:109-158)."""
import json

import pytest

from ark_amd import Model, llama, plan_analysis


def _plan(m):
    return m.plan(arch="ROCM_950", num_processors=256)


def _tasks_steps(a):
    return [s for s in a["Steps"] if s["Kind"] == "Tasks"]


def _cfg(plan, task_info, op=0):
    return json.loads(plan)["TaskInfos"][task_info]["Ops"][op]["Config"]


def test_rows_feeding_matmuls_spans_by_first_principles():
    m = Model()
    x, w1, w2 = m.tensor([4096, 2048], "fp16"), m.tensor([2048, 4096], "fp16"), m.tensor([4096, 2048], "fp16")
    m.matmul(m.matmul(m.rmsnorm(x), w1), w2)
    plan = _plan(m)
    off = plan_analysis(plan, 0)
    assert off["BarriersCounted"] == 0 and off["NumCounters"] == 0
    assert [s["Kind"] for s in off["Steps"]] == ["Tasks", "Barrier", "Tasks", "Barrier", "Tasks"]
    a = plan_analysis(plan, 1)
    assert a["BarriersCounted"] == 2 and a["IterationSync"] == 2
    assert [s["Kind"] for s in a["Steps"]] == ["Tasks", "LocalSync", "Tasks", "LocalSync", "Tasks"]
    norm, mm1, mm2 = _tasks_steps(a)
    # producer 0: RMSNorm, a task covers NumWarps x RowsPerWave rows and signals its own block
    c0 = _cfg(plan, 0)
    rows_per_task = c0["NumWarps"] * c0["RowsPerWave"]
    assert norm["NumTasks"] == 4096 // rows_per_task and norm["SignalMap"] == list(range(norm["NumTasks"]))
    assert norm["Waits"] == []
    # consumer 1: tile t reads the rows of its tile row (tile index row-major, N fastest)
    c1 = _cfg(plan, 1)
    bm, bn = c1["TileShapeMNK"][:2]
    tiles_n = 4096 // bn
    (w,) = mm1["Waits"]
    assert w["ProducerGroup"] == norm["Group"] and w["Expect"] == 1
    for t, (lo, hi) in enumerate(w["Spans"]):
        r0, r1 = (t // tiles_n) * bm, (t // tiles_n + 1) * bm
        assert (lo, hi) == (r0 // rows_per_task, (r1 - 1) // rows_per_task), t
    # producer 1 signals the block of its tile row; every block collects one signal per tile column
    assert mm1["SignalMap"] == [t // tiles_n for t in range(mm1["NumTasks"])]
    # consumer 2 waits for the tile rows of the first matmul that cover its own rows
    # (4096 x 2048 x 4096 gives 256x256 tiles to half of the CUs: K is split, two tasks per tile)
    c2 = _cfg(plan, 2)
    bm2, bn2 = c2["TileShapeMNK"][:2]
    tiles_n2 = 2048 // bn2
    tiles2 = mm2["NumTasks"] // c2.get("SplitK", 1)
    assert c2.get("SplitK") == 2 and tiles2 == 128
    (w,) = mm2["Waits"]
    assert w["ProducerGroup"] == mm1["Group"] and w["Expect"] == tiles_n
    for t, (lo, hi) in enumerate(w["Spans"]):
        tile = t % tiles2
        r0, r1 = (tile // tiles_n2) * bm2, (tile // tiles_n2 + 1) * bm2
        assert (lo, hi) == (r0 // bm, (r1 - 1) // bm), t
    assert "SignalMap" not in mm2  # nobody waits for the last group
    assert a["NumCounters"] == norm["NumTasks"] + 4096 // bm


def test_write_after_read_keeps_the_last_barrier():
    """x <- x + 0.01 * (rmsnorm(x) @ w): the final add overwrites what the RMSNorm read, a hazard no
    counter expresses, so the barrier ahead of the add stays and the groups behind it start a new
    window; the barriers ahead of it are counted."""
    m = Model()
    x, w = m.tensor([16384, 2048], "fp16"), m.tensor([2048, 2048], "fp16")
    h = m.matmul(m.rmsnorm(x), w)
    m.add(x, m.mul(h, 0.01), output=x)
    a = plan_analysis(_plan(m), 1)
    kinds = [s["Kind"] for s in a["Steps"]]
    assert kinds.count("Tasks") == 4
    # RMSNorm -> matmul is counted; the barrier ahead of the scalar multiply stays (it is the last
    # full barrier between the reader of x and its writer: the multiply and the add share tiles, so
    # the barrier between those two was a workgroup sync already)
    assert kinds == ["Tasks", "LocalSync", "Tasks", "Barrier", "Tasks", "LocalSync", "Tasks"]
    assert a["Steps"][3]["Count"] == 256 and a["BarriersCounted"] == 1
    norm, mm, mul, add = _tasks_steps(a)
    assert [w["ProducerGroup"] for w in mm["Waits"]] == [norm["Group"]]
    assert mul["Waits"] == [] and add["Waits"] == []  # ordered by the barrier, not by counters
    assert "SignalMap" not in mm


def test_sub_grid_barriers_are_never_replaced():
    m = Model()
    """RMSNorm on 64 processors, then two matmuls of 16 tiles: the barrier between the matmuls spans
    16 of the plan's 64 processors.  A plan with such a barrier keeps all of them (the argument for
    reading without a cache invalidate needs every workgroup at every barrier that stays)."""
    x, w = m.tensor([512, 512], "fp16"), m.tensor([512, 512], "fp16")
    m.matmul(m.matmul(m.rmsnorm(x), w), w)
    a = plan_analysis(_plan(m), 1)
    assert a["NumProcessors"] == 64
    assert a["BarriersCounted"] == 0 and a["NumCounters"] == 0
    assert sorted(s["Count"] for s in a["Steps"] if s["Kind"] == "Barrier") == [16, 64]


def test_decoder_layer_replaces_every_barrier():
    m = Model()
    blk = llama.TransformerBlock(m, 4096, 32, 11008, "bf16")
    tx = m.tensor([1, 2048, 4096], "bf16")
    tf = m.tensor([1, 2048, 1, 128], "bf16")
    tm = m.tensor([1, 1, 2048, 2048], "bf16")
    blk.forward(tx, tf, tm, fused=True, causal=True)
    plan = _plan(m)
    off, on = plan_analysis(plan, 0), plan_analysis(plan, 1)
    assert off["BarriersCounted"] == 0 and [s["Kind"] for s in off["Steps"]].count("Barrier") == 6
    assert on["BarriersCounted"] == 6 and "Barrier" not in [s["Kind"] for s in on["Steps"]]
    # rows + matmul + split of K + attention: the rotation and the residual adds are folded into the
    # projections' stores and need no elementwise body in the kernel
    assert on["KernelFamilies"] == off["KernelFamilies"] == 85
    groups = _tasks_steps(on)
    names = ["norm1", "q", "k", "v", "attn", "wo", "norm2", "swiglu", "down"]
    g = dict(zip(names, groups))
    # the three projections wait for the first RMSNorm only, and not for each other
    for p in ("q", "k", "v"):
        assert [w["ProducerGroup"] for w in g[p]["Waits"]] == [g["norm1"]["Group"]]
    # attention: the query block's rows of Q, and K / V up to the causal diagonal (128-row blocks)
    waits = {w["ProducerGroup"]: w for w in g["attn"]["Waits"]}
    assert sorted(waits) == [g["q"]["Group"], g["k"]["Group"], g["v"]["Group"]]
    qb_count = 2048 // 128
    # (a projection's row blocks are its tile rows: bm rows each, one signal per tile column)
    bm, bn = _cfg(plan, g["q"]["Group"])["TileShapeMNK"][:2]
    for t in range(g["attn"]["NumTasks"]):
        bh, qb = divmod(t, qb_count)
        if bh >= 16:  # the upper half of the heads runs its query blocks backwards
            qb = qb_count - 1 - qb
        first, last = qb * 128 // bm, (qb * 128 + 127) // bm
        assert tuple(waits[g["q"]["Group"]]["Spans"][t]) == (first, last), t
        assert tuple(waits[g["k"]["Group"]]["Spans"][t]) == (0, last), t
        assert tuple(waits[g["v"]["Group"]]["Spans"][t]) == (0, last), t
    assert all(w["Expect"] == 4096 // bn for w in waits.values())
    # the output projection reads all heads of its rows: 128 query rows = 32 attention tasks per
    # attention row block, and a tile row of bm_o rows spans bm_o / 128 of them
    (w,) = g["wo"]["Waits"]
    assert w["ProducerGroup"] == g["attn"]["Group"] and w["Expect"] == 32
    c_o = _cfg(plan, g["wo"]["Group"])
    bm_o = c_o["TileShapeMNK"][0]
    tiles_n_o = 4096 // c_o["TileShapeMNK"][1]
    tiles_o = g["wo"]["NumTasks"] // c_o.get("SplitK", 1)  # K split in two: both tasks of a tile wait alike
    for t, (lo, hi) in enumerate(w["Spans"]):
        r0 = ((t % tiles_o) // tiles_n_o) * bm_o
        assert (lo, hi) == (r0 // 128, (r0 + bm_o - 1) // 128), t
    # the down projection needs the SwiGLU rows of its tile and the residual it adds
    assert sorted(w["ProducerGroup"] for w in g["down"]["Waits"]) == sorted([g["wo"]["Group"], g["swiglu"]["Group"]])
    assert "SignalMap" not in g["down"]


def test_analysis_rejects_what_compile_rejects():
    from ark_amd import ArkmiError
    with pytest.raises(ArkmiError) as e:
        plan_analysis("{not json", 1)
    assert e.value.kind == "PlanError"


def test_consecutive_skinny_matmuls_form_one_stream():
    """Skinny matmuls that follow one another with no barrier or sync between them are marked as one
    run (the first group carries the length, the others -1); anything in between, a dependency, or
    another element type breaks the run.  A run (or a matmul by itself) whose column blocks all have
    at least three units is cut into stretches that the workgroups claim at run time."""
    m = Model()
    for k, n in [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]:
        m.matmul(m.tensor([1, k], "bf16"), m.tensor([k, n], "bf16"))
    plan = _plan(m)
    a = plan_analysis(plan, 0)
    assert a["GemvChains"] == 1 and a["GemvClaimed"] == 1
    assert [s["Kind"] for s in a["Steps"]] == ["Tasks"] * 4
    assert [(s["Chain"], s["Claimed"]) for s in a["Steps"]] == [(4, True), (-1, False), (-1, False), (-1, False)]

    # y2 depends on y1: the barrier between them stays, nothing is chained, each claims by itself
    m = Model()
    y1 = m.matmul(m.tensor([1, 4096], "bf16"), m.tensor([4096, 4096], "bf16"))
    m.matmul(y1, m.tensor([4096, 4096], "bf16"))
    a = plan_analysis(_plan(m), 0)
    assert a["GemvChains"] == 0 and [s["Kind"] for s in a["Steps"]] == ["Tasks", "Barrier", "Tasks"]
    assert [(s["Chain"], s["Claimed"]) for s in _tasks_steps(a)] == [(0, True), (0, True)]
    assert a["GemvClaimed"] == 2 and a["IterationSync"] == 2

    # two runs separated by an elementwise op of its own
    m = Model()
    for _ in range(2):
        m.matmul(m.tensor([2, 1024], "fp16"), m.tensor([1024, 512], "fp16"))
    m.relu(m.tensor([64, 64], "fp16"))
    for _ in range(3):
        m.matmul(m.tensor([2, 1024], "fp16"), m.tensor([1024, 512], "fp16"))
    # a different element type does not join the run before it; K = 256 is two units: too few to
    # cut into claimable stretches
    m.matmul(m.tensor([2, 256], "bf16"), m.tensor([256, 512], "bf16"))
    a = plan_analysis(_plan(m), 0)
    assert a["GemvChains"] == 2 and a["GemvClaimed"] == 2
    assert [(s["Chain"], s["Claimed"]) for s in _tasks_steps(a)] == [
        (2, True), (-1, False), (0, False), (3, True), (-1, False), (-1, False), (0, False)]


def _tile_of(t2, tiles_m, tiles_n, xcd_round, band):
    """The tile that task index t2 computes in the XCD-aware order, restated from the rule: tiles
    ordered in bands of `band` rows, column by column; a task of a full round of `xcd_round` tasks
    takes position ((round * 8 + xcd) * xcd_round / 8 + number within the XCD), xcd = t2 mod 8."""
    p = t2
    if t2 < (tiles_m * tiles_n // xcd_round) * xcd_round:
        r, q = divmod(t2, xcd_round)
        p = (r * 8 + q % 8) * (xcd_round // 8) + q // 8
    b, w = divmod(p, band * tiles_n)
    return b * band + w % band, w // band


def test_matmul_tiles_in_xcd_aware_order():
    """compile() orders the tiles of the decoder layer's matmuls so that the tiles one XCD (task
    index mod 8) works on at a time form a compact block: every tile is still computed exactly once,
    and the 32 (or 16) concurrent tiles of an XCD span band x (n / band) tiles instead of being
    strewn over all tile rows."""
    m = Model()
    blk = llama.TransformerBlock(m, 4096, 32, 11008, "bf16")
    x, f, mask = m.tensor([1, 2048, 4096], "bf16"), m.tensor([1, 2048, 1, 128], "bf16"), m.tensor([1, 1, 2048, 2048], "bf16")
    blk.forward(x, f, mask, fused=True, causal=True)
    plan = _plan(m)
    a = plan_analysis(plan, 0)
    gemms = [s for s in _tasks_steps(a) if "XcdRound" in s]
    assert a["GemmXcdOrdered"] == len(gemms) == 6  # q, k, v, wo, the gate/up pair, w2
    infos = json.loads(plan)["TaskInfos"]
    for s in gemms:
        assert s["XcdRound"] > 0 and s["XcdRound"] % 8 == 0
        cfg = infos[s["Group"]]["Ops"][0]["Config"]
        tm_, tn_ = cfg["TileShapeMNK"][:2]
        tiles = s["NumTasks"] // cfg.get("SplitK", 1)
        out_n = 4096 if tiles in (128, 256) else 2 * 11008
        tiles_n = out_n // tn_
        tiles_m = tiles // tiles_n
        assert tiles_m * tiles_n == tiles and tiles_m % s["XcdBand"] == 0
        where = [_tile_of(t, tiles_m, tiles_n, s["XcdRound"], s["XcdBand"]) for t in range(tiles)]
        assert sorted(where) == [(i, j) for i in range(tiles_m) for j in range(tiles_n)]
        per = s["XcdRound"] // 8
        for xcd in range(8):
            mine = where[xcd:s["XcdRound"]:8]
            assert len(mine) == per
            assert len({i for i, _ in mine}) == s["XcdBand"] and len({j for _, j in mine}) == per // s["XcdBand"]
    # (waits and signals go by task index: a matmul that takes part in the dependency counters keeps
    # the plain order)
    assert plan_analysis(plan, 1)["GemmXcdOrdered"] < len(gemms)


def test_row_ops_whose_input_is_read_again():
    """A row op whose input another op of the plan reads afterwards fetches it through the caches
    (the later reader then finds it there); the last reader, and an op whose input is overwritten
    before anybody reads it again, stream it."""
    m = Model()
    x, y = m.tensor([16384, 4096], "fp16"), m.tensor([16384, 4096], "fp16")
    w = m.tensor([4096], "fp32")
    m.reduce_sum(x, -1)
    m.softmax(x)
    m.rmsnorm(x, w, 1e-6)          # the last reader of x
    m.reduce_sum(y, -1)            # y is overwritten next, before anybody reads it
    m.softmax(x, output=y)
    m.rmsnorm(y, w, 1e-6)          # reads the new y; nobody after it
    a = plan_analysis(_plan(m), 0)
    assert [s["InputReadAgain"] for s in _tasks_steps(a)] == [[1], [1], [1], [0], [0], [0]]
    # (x is read once more by the fifth op, so the third is not its last reader)
    m = Model()
    x = m.tensor([16384, 4096], "fp16")
    m.reduce_sum(x, -1)
    m.softmax(x)
    m.rmsnorm(x, m.tensor([4096], "fp32"), 1e-6)
    a = plan_analysis(_plan(m), 0)
    assert [s["InputReadAgain"] for s in _tasks_steps(a)] == [[1], [1], [0]]


def test_counted_barrier_with_a_local_hazard_keeps_the_plain_tile_order():
    """rmsnorm(x); y = a @ w; y + rmsnorm(x) with the add cut into the matmul's 256x256 tiles: with
    counters on, the barrier ahead of the add goes because its hazard with the RMSNorm is counted
    and its hazard with the matmul is local to a workgroup (task t of both covers tile t).  That
    second half rests on the matmul computing tile t in task t, so the XCD-aware permutation of
    its tiles must stay off; without counters the barrier stays and the permutation is on."""
    m = Model()
    x, a, w = (m.tensor([4096, 4096], "fp16") for _ in range(3))
    n = m.rmsnorm(x)
    m.add(m.matmul(a, w), n)
    plan = json.loads(_plan(m))
    add_cfg = plan["TaskInfos"][2]["Ops"][0]["Config"]
    add_cfg["Tile"], add_cfg["NumTasks"] = [256, 256], 256
    plan["ProcessorGroups"][2]["ResourceGroups"][0]["TaskGroups"][0]["TaskRange"] = [0, 256]
    plan = json.dumps(plan)
    on = plan_analysis(plan, 1)
    assert [s["Kind"] for s in on["Steps"]] == ["Tasks", "Tasks", "LocalSync", "Tasks"]
    assert on["BarriersCounted"] == 1 and on["BarriersLocal"] == 0
    norm, mm, add = _tasks_steps(on)
    assert [w_["ProducerGroup"] for w_ in add["Waits"]] == [norm["Group"]]   # nothing waits for the matmul
    assert mm["XcdRound"] == 0 and on["GemmXcdOrdered"] == 0
    off = plan_analysis(plan, 0)
    assert [s["Kind"] for s in off["Steps"]] == ["Tasks", "Tasks", "Barrier", "Tasks"]
    assert _tasks_steps(off)[1]["XcdRound"] == 256


def test_split_matmuls_give_the_sender_the_shorter_part(monkeypatch):
    """A matmul that splits K in two gives the sender the shorter part: its partial sums are on their
    way while the finisher still multiplies.  The split point is reported by the analysis."""
    m = Model()
    blk = llama.TransformerBlock(m, 4096, 32, 11008, "bf16")
    blk.forward(m.tensor([1, 2048, 4096], "bf16"), m.tensor([1, 2048, 1, 128], "bf16"),
                m.tensor([1, 1, 2048, 2048], "bf16"), fused=True, causal=True)
    plan = _plan(m)
    names = ["norm1", "q", "k", "v", "attn", "wo", "norm2", "swiglu", "down"]

    def split_points():
        g = dict(zip(names, _tasks_steps(plan_analysis(plan, 0))))
        assert all("SplitAt" not in g[n] for n in ("norm1", "attn", "norm2", "swiglu"))
        return [g[n]["SplitAt"] for n in ("q", "k", "v", "wo", "down")]

    assert split_points() == [2240] * 4 + [5696]
    monkeypatch.setenv("ARKMI_SPLITK_SKEW", "0")
    assert split_points() == [2048] * 4 + [5504]
    monkeypatch.setenv("ARKMI_SPLITK_SKEW", "1000000")  # a part of K keeps at least four K tiles
    assert split_points() == [4096 - 256] * 4 + [11008 - 256]


def test_row_ops_touch_the_first_rows_of_the_row_op_that_follows(monkeypatch):
    """Row ops that follow one another on the same workgroups with the same dealing of rows, and no grid
    barrier between them, are linked: each touches its waves' first rows of the next while it finishes
    (a hint that costs a load per wave).  A matmul in between, another row count or a kept barrier
    breaks the link."""
    def flags(m):
        a = plan_analysis(_plan(m), 0)
        return [s.get("TouchesNextRows") for s in _tasks_steps(a)], a["IterationSync"]

    m = Model()
    x, w = m.tensor([16384, 4096], "fp16"), m.tensor([1, 4096], "fp32")
    m.reduce_sum(x, axis=1)
    m.softmax(x)
    m.rmsnorm(x, w, 1e-5)
    got, it_sync = flags(m)
    # reduce_sum and softmax leave X in the caches for the op behind them (InputReadAgain): nothing to
    # touch there, and nothing ahead of a reader that fetches through the caches (the first op of the
    # next iteration)
    assert got == [False, False, False]
    monkeypatch.setenv("ARKMI_ROW_CACHED_INPUT", "0")   # every op streams: each touches the next one's rows
    assert flags(m)[0] == [True, True, it_sync != 2]
    monkeypatch.delenv("ARKMI_ROW_CACHED_INPUT")
    m2 = Model()
    xs = [m2.tensor([16384, 4096], "fp16") for _ in range(3)]
    for x in xs:
        m2.softmax(x)
    got2, it_sync2 = flags(m2)
    assert got2 == [True, True, it_sync2 != 2]  # different inputs, streamed: each touches the next one's rows
    monkeypatch.setenv("ARKMI_ROW_PREFETCH", "0")
    assert flags(m)[0] == [False, False, False]
    monkeypatch.delenv("ARKMI_ROW_PREFETCH")

    m = Model()
    x, y = m.tensor([16384, 4096], "fp16"), m.tensor([8192, 4096], "fp16")
    m.softmax(x)
    m.softmax(y)            # half the rows: another dealing
    m.matmul(m.tensor([4096, 4096], "fp16"), m.tensor([4096, 4096], "fp16"))
    got, _ = flags(m)
    assert got[0] is False and got[1] is False and got[2] is None

    m = Model()
    x = m.tensor([16384, 4096], "fp16")
    m.softmax(m.softmax(x))  # linked exactly when no grid barrier stays between the two
    a = plan_analysis(_plan(m), 0)
    kinds = [s["Kind"] for s in a["Steps"]]
    assert _tasks_steps(a)[0]["TouchesNextRows"] == ("Barrier" not in kinds[:kinds.index("Tasks", 1)])
