"""The cache's bookkeeping and the generation loop's decisions (no GPU)."""
import os
import random

import pytest
import torch

from llm_infer_amd.cache import Cache, CacheError, KVSpec, PagePool, SlotAllocator, StateSpec
from llm_infer_amd.config.spec import ConfigError, ModelSpec, PartSpec, ScheduleEntry
from llm_infer_amd.engine.generate import BatchTracker, RequestError, plan_batches
from llm_infer_amd.engine.step import decode_splits, split_bucket
from llm_infer_amd.cli import parse_args
from llm_infer_amd.tokenizer import Tokenizer


def test_slots_are_neither_lost_nor_held_twice_nor_freed_twice():
    a = SlotAllocator(4)
    got = [a.alloc() for _ in range(4)]
    assert sorted(got) == [0, 1, 2, 3] and a.n_free == 0
    with pytest.raises(CacheError, match="in use"):
        a.alloc()
    a.free(2)
    with pytest.raises(CacheError, match="not held"):
        a.free(2)
    with pytest.raises(CacheError, match="not held"):
        a.free(7)
    assert a.alloc() == 2
    rng = random.Random(0)
    held = set(got)
    for _ in range(2000):
        if held and (rng.random() < 0.5 or a.n_free == 0):
            s = rng.choice(sorted(held))
            a.free(s)
            held.remove(s)
        else:
            s = a.alloc()
            assert s not in held
            held.add(s)
        assert a.held() == held and a.n_free + len(held) == 4


def test_a_following_batch_uses_the_same_slots_again():
    a = SlotAllocator(8)
    first = [a.alloc() for _ in range(3)]
    for s in first:
        a.free(s)
    assert [a.alloc() for _ in range(3)] == first


def test_pages():
    p = PagePool(6, first=1)
    x = p.alloc(3)
    assert len(set(x)) == 3 and 0 not in x and p.n_free == 2
    with pytest.raises(CacheError, match="cache is full"):
        p.alloc(3)
    p.free(x[:1])
    with pytest.raises(CacheError, match="not held"):
        p.free(x[:1])
    assert p.n_free == 3 and p.held() == set(x[1:])


def _cache(specs, max_tokens=640, max_pos=512, slots=4):
    return Cache(specs, max_tokens, max_pos, torch.bfloat16, None, slots)


def test_cache_groups_lengths_and_page_accounting():
    full, win = KVSpec(2, 16), KVSpec(2, 16, window=100)
    c = _cache([full, win, None, full, StateSpec((3, 4))])
    assert len(c.groups) == 3
    kv_full = next(g for g in c.groups if getattr(g, "spec", None) == full)
    kv_win = next(g for g in c.groups if getattr(g, "spec", None) == win)
    assert kv_full.entries == [0, 3] and kv_win.entries == [1] and c.view(2) is None
    assert kv_full.page_elems == 2 * (2 * 64 * 16 + 2 * 64 * 32)       # values padded to 32 dims
    s0, s1 = c.alloc_slot(), c.alloc_slot()
    c.grow([s0, s1], [130, 1])
    assert c.lens[s0] == 130 and c.lens[s1] == 1
    assert len(kv_full.pages_of[s0]) == 3 and len(kv_full.pages_of[s1]) == 1
    assert kv_full.table_host[s0, :3].tolist() == [kv_full.pages_of[s0][i] for i in range(3)]
    assert c.tokens_free() == 640 - 4 * 64
    # a window group gives back pages that no later token can read
    c.grow([s0], [300])
    c.trim_windows([s0])
    assert sorted(kv_win.pages_of[s0]) == [3, 4] and kv_win.table_host[s0, 0] == 0
    assert sorted(kv_full.pages_of[s0]) == [0, 1, 2, 3, 4]
    with pytest.raises(CacheError, match="exceeds the model's 512 positions"):
        c.grow([s0], [513])
    with pytest.raises(CacheError, match="cache is full"):
        c.grow([s1], [500])
    c.free_slot(s0)
    assert kv_full.pool.n_free == 10 - 1 and kv_win.pool.n_free == 10 - 1 and c.lens[s0] == 0
    with pytest.raises(CacheError, match="not held"):
        c.free_slot(s0)
    with pytest.raises(CacheError, match="not held"):
        c.grow([s0], [5])
    c.free_slot(s1)
    assert kv_full.pool.n_free == 10 and not kv_full.pool.held() and c.slots.n_free == 4


def test_a_failed_step_gives_its_pages_back():
    """``truncate`` undoes ``grow``: lengths as before, the pages beyond them free again (and so cleared or
    wholly filled when they are next handed out), the page a sequence still reaches kept."""
    c = _cache([KVSpec(2, 16), KVSpec(2, 16, window=100)])
    full = c.groups[0]
    s0, s1 = c.alloc_slot(), c.alloc_slot()
    c.grow([s0, s1], [70, 64])
    free_before, pages_before = full.pool.n_free, dict(full.pages_of[s0])
    c.grow([s0, s1], [200, 65], filled=True)
    c.truncate([s0, s1], [70, 64])
    assert c.lens[s0] == 70 and c.lens[s1] == 64
    assert full.pool.n_free == free_before and full.pages_of[s0] == pages_before
    assert sorted(full.pages_of[s1]) == [0] and full.table_host[s1, 1] == 0 and full.table_host[s0, 2] == 0
    held = [p for s in (s0, s1) for p in full.pages_of[s].values()]
    assert set(held) == full.pool.held()
    c.grow([s0], [200])                                   # and the sequence grows again as if nothing had been
    assert len(full.pages_of[s0]) == 4


def test_random_sequences_never_share_a_page():
    c = _cache([KVSpec(1, 16)], max_tokens=64 * 40, max_pos=64 * 12, slots=6)
    g = c.groups[0]
    rng = random.Random(1)
    live = {}
    for _ in range(600):
        if live and rng.random() < 0.3:
            s = rng.choice(sorted(live))
            c.free_slot(s)
            del live[s]
        elif len(live) < 6 and rng.random() < 0.5:
            live[c.alloc_slot()] = 0
        elif live:
            s = rng.choice(sorted(live))
            n = min(64 * 12, live[s] + rng.randint(1, 90))
            try:
                c.grow([s], [n])
                live[s] = n
            except CacheError:
                pass
        pages = [p for s in live for p in g.pages_of[s].values()]
        assert len(pages) == len(set(pages)) and 0 not in pages
        assert set(pages) == g.pool.held()
        for s, n in live.items():
            assert len(g.pages_of[s]) == -(-n // 64) and c.lens[s] == n


def test_schedule_validation():
    def spec(schedule, n_layers=2):
        ps = PartSpec("x")
        from llm_infer_amd.config.spec import LayerSpec
        layer = LayerSpec.mixer_then_feed_forward("pre_norm", ps, ps, ps, ps)
        return ModelSpec(8, 8, 8, ps, tuple([layer] * n_layers), tuple(schedule), ps, ps)
    spec([ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_from=1)]).validate()
    with pytest.raises(ConfigError, match="names layer 5"):
        spec([ScheduleEntry(5)]).validate()
    with pytest.raises(ConfigError, match="does not run before"):
        spec([ScheduleEntry(0, cache_from=1), ScheduleEntry(1)]).validate()
    with pytest.raises(ConfigError, match="keeps none of its own"):
        spec([ScheduleEntry(0), ScheduleEntry(1, cache_from=0), ScheduleEntry(0, cache_from=1)]).validate()
    # a layer is a list of sub-layers, each a mixer or a feed-forward
    from llm_infer_amd.config.spec import LayerSpec, SubLayerSpec
    ps = PartSpec("x")
    layer = LayerSpec("pre_norm", (SubLayerSpec("mixer", ps, ps), SubLayerSpec("mixer", ps, ps, ps), SubLayerSpec("feed_forward", ps)))
    ModelSpec(8, 8, 8, ps, (layer,), (ScheduleEntry(0),), ps, ps).validate()
    with pytest.raises(ConfigError, match="no sub-layer"):
        ModelSpec(8, 8, 8, ps, (LayerSpec("pre_norm", ()),), (ScheduleEntry(0),), ps, ps).validate()
    with pytest.raises(ConfigError, match="'mixer' or a 'feed_forward'"):
        ModelSpec(8, 8, 8, ps, (LayerSpec("pre_norm", (SubLayerSpec("norm", ps),)),), (ScheduleEntry(0),), ps, ps).validate()


def test_plan_batches():
    assert plan_batches([5, 6, 7, 8, 9], 10, 2, 10_000, 100) == [[0, 1], [2, 3], [4]]
    assert plan_batches([60, 60, 60], 10, 8, 256, 1000) == [[0, 1], [2]]         # 128 tokens each
    assert plan_batches([10, 10], 1000, 8, 128, 64) == [[0, 1]]                  # capped by the context
    with pytest.raises(RequestError, match="Prompt too long: 100 tokens \\(max: 100\\)"):
        plan_batches([100], 1, 1, 10_000, 100)
    with pytest.raises(RequestError, match="empty prompt"):
        plan_batches([3, 0], 1, 1, 10_000, 100)
    with pytest.raises(RequestError, match="needs room"):
        plan_batches([200], 100, 1, 256, 1000)


def test_the_loop_decisions():
    t = BatchTracker([3, 5, 2], max_new_tokens=3, stop_token_ids={9}, max_positions=6)
    assert t.live() == [0, 1, 2]
    go = t.accept([0, 1, 2], [4, 9, 7])           # request 1 samples the stop token at once
    assert go == [0, 2] and t.outputs == [[4], [], [7]] and t.reason[1] == "stop"
    go = t.accept([0, 2], [5, 8])
    assert go == [0, 2]
    go = t.accept([0, 2], [6, 9])                 # request 0 reaches its budget: no forward after the last
    assert go == [] and t.outputs == [[4, 5, 6], [], [7, 8]] and t.reason == ["length", "stop", "stop"]
    with pytest.raises(RuntimeError):
        t.accept([0], [1])
    t = BatchTracker([5], 10, (), max_positions=6)
    assert t.accept([0], [1]) == [0]              # the token fits at position 5
    assert t.accept([0], [2]) == [] and t.reason == ["context"] and t.outputs == [[1, 2]]
    t = BatchTracker([5], 0, (), 100)
    assert t.live() == [] and t.reason == ["length"]


def test_a_budget_for_each_request_and_the_rows_of_a_recorded_step():
    from llm_infer_amd.engine.decode import batch_bucket
    from llm_infer_amd.engine.generate import per_request
    t = BatchTracker([3, 3, 3], max_new_tokens=[1, 3, 0], stop_token_ids=(), max_positions=100)
    assert t.live() == [0, 1] and t.reason[2] == "length"
    assert not t.will_go_on([0, 1]) and t.will_go_on([1])
    assert t.accept([0, 1], [4, 5]) == [1] and t.reason[0] == "length"
    assert t.accept([1], [6]) == [1] and t.accept([1], [7]) == [] and t.outputs == [[4], [5, 6, 7], []]
    assert plan_batches([60, 60, 60], [10, 200, 4], 8, 448, 1000) == [[0, 1], [2]]      # 128 + 320, then 64
    with pytest.raises(RequestError, match="2 values for 3 requests"):
        per_request([1, 2], 3)
    # a shrinking batch meets few sizes: every size at least the live sequences, at most the slots, and at
    # most a third of its rows idle
    sizes = [batch_bucket(n, 4096) for n in range(1, 300)]
    assert sizes[:17] == [1, 2, 4, 4, 8, 8, 8, 8, 12, 12, 12, 12, 16, 16, 16, 16, 24]
    assert len(set(sizes[:64])) == 10 and all(b >= n for n, b in zip(range(1, 300), sizes))
    assert all(b - n <= b // 3 + 1 for n, b in zip(range(1, 300), sizes))
    assert batch_bucket(5, 6) == 6 and batch_bucket(7, 7) == 7 and batch_bucket(64, 64) == 64


def test_the_loop_knows_beforehand_whether_all_go_on():
    """will_go_on is what lets a step be enqueued before the tokens of the step before are read:
    it must say exactly whether tokens that are no stop tokens keep every live request going."""
    for lens, budget, limit in (([3, 5, 2], 4, 8), ([5], 10, 6), ([1, 1], 1, 100), ([2, 9], 7, 12)):
        t = BatchTracker(lens, budget, {9}, limit)
        live = t.live()
        while live:
            said = t.will_go_on(live)
            go = t.accept(live, [1] * len(live))
            assert said == (go == live)
            live = go


def test_decode_splits_fill_the_chip_and_are_powers_of_two():
    def splits(n, k, h, ctx):
        return decode_splits(n, k, h, split_bucket(ctx))
    assert splits(1, 8, 32, 8192) == 64
    assert splits(8, 8, 32, 8192) == 16
    assert splits(64, 8, 32, 8192) == 2 and splits(32, 8, 32, 8192) == 4 and splits(128, 8, 32, 8192) == 1
    assert splits(64, 32, 32, 4096) == 1
    assert splits(1, 8, 32, 100) == 1 and splits(1, 1, 64, 640) == 4
    # the bucket is all that the count knows of the lengths: at least two pages a split, at most 64 splits
    assert [split_bucket(c) for c in (1, 64, 128, 192, 193, 256, 4096, 8192, 100_000)] == [1, 1, 1, 1, 2, 2, 32, 64, 64]
    for ctx in range(1, 9000, 37):
        pages = (ctx + 63) // 64
        for n, k, h in ((1, 8, 32), (3, 1, 4), (8, 2, 2)):
            s = splits(n, k, h, ctx)
            assert s & (s - 1) == 0 and 1 <= s <= max(1, pages // 2)


def test_the_prefill_product_plan():
    """What the planner of the prefill product hands the kernel: a tile it has, K split only where a split
    keeps at least 1,024 of K, few rows of X split (the chip has 256 CUs to fill), many rows not."""
    import random as _r

    from llm_infer_amd.kernels.ops import _WREG_TILES, _wreg_cost, _wreg_plan
    rng = _r.Random(0)
    shapes = [(2048, 28672, 4096), (33186, 2048, 8192), (3000, 6144, 4096), (97, 4096, 14336), (130, 128256, 4096)]
    shapes += [(rng.randint(17, 40000), 16 * rng.randint(1, 2000), 32 * rng.randint(1, 500)) for _ in range(300)]
    for m, n, k in shapes:
        tile, splits = _wreg_plan(m, n, k)
        assert tile in _WREG_TILES and splits >= 1 and (splits == 1 or k // splits >= 1024)
        assert _wreg_cost(tile, splits, m, n, k) <= min(_wreg_cost(t, 1, m, n, k) for t in _WREG_TILES)
    assert _wreg_plan(64, 4096, 4096)[1] > 1 and _wreg_plan(8192, 4096, 4096) == (0, 1)
    assert _wreg_plan(2048, 6144, 4096)[0] == 1           # 512 tiles of 192 x 128: two on every CU


def test_the_plan_for_products_of_a_few_dozen_rows():
    """17 to 128 rows: all of K in one workgroup (gemm_rows, no second kernel) where its estimate beats the tiled
    GEMM's; it fetches the rows of X once per workgroup, so it wins against the small matrices and loses against
    the wide ones, and two tiles of W a workgroup are for matrices with tiles enough for 256 CUs."""
    from llm_infer_amd.kernels import ops
    for m in (17, 32, 64, 128):
        assert ops._rows_plan(m, 4096, 4096, True) in (1, 2)            # attention output, 34 MB
        assert ops._rows_plan(m, 6144, 4096) in (1, 2)                  # q/k/v, 50 MB
        assert ops._rows_plan(m, 28672, 4096) == 0                      # gate and up, 235 MB: the tiled GEMM
    assert ops._rows_plan(64, 6144, 4096) == 2 and ops._rows_plan(64, 4096, 4096, True) == 1
    assert ops._rows_plan(96, 4096, 14336, True) == 0                   # down: K split and the norm taken along
    # more rows of X cost more, more tiles a workgroup cost fewer fetches of X
    assert ops._rows_cost(1, 128, 4096, 4096) > ops._rows_cost(1, 64, 4096, 4096) > ops._rows_cost(1, 32, 4096, 4096)
    assert ops._rows_cost(2, 64, 28672, 4096) < ops._rows_cost(1, 64, 28672, 4096)
    # the norm that would have ridden on the tiled GEMM's second kernel counts against gemm_rows
    assert any(ops._rows_plan(m, n, k, False) and not ops._rows_plan(m, n, k, True)
               for m in (24, 48, 96) for n, k in ((2048, 8192), (4096, 11008), (4096, 14336)))


def test_blocks_of_w_a_workgroup_for_products_whose_tiles_leave_cus_idle():
    """Up to 64 rows of X, K whole, the narrowest tile: a workgroup takes as few of its tile's eight blocks of 16 rows
    of W as make (rounds of 256 workgroups) x (blocks) least; everything else takes the whole tile."""
    from llm_infer_amd.kernels import ops
    assert ops._wreg_blocks(2, 1, 64, 28672) == 7            # 1,792 blocks: 224 workgroups of 8, 256 of 7
    assert ops._wreg_blocks(2, 1, 64, 22016) == 6            # 1,376 blocks: 172 of 8, 230 of 6
    assert ops._wreg_blocks(2, 1, 64, 4096 * 8) == 8         # 2,048 blocks: 256 of 8 already
    assert ops._wreg_blocks(2, 8, 64, 4096) == 8             # K split: the splits fill the CUs
    assert ops._wreg_blocks(2, 1, 128, 28672) == 8 and ops._wreg_blocks(0, 1, 64, 28672) == 16
    for n in range(16, 40000, 1008):
        b = ops._wreg_blocks(2, 1, 33, n)
        groups = lambda blocks: -(-(-(-n // 16)) // blocks)
        assert 5 <= b <= 8 and -(-groups(b) // 256) * b <= -(-groups(8) // 256) * 8


def test_the_index_arrays_of_a_recorded_prefill_step():
    """A recorded prefill step reads its step from one buffer of fixed layout; what the step does not fill is
    padding that belongs to no sequence: tokens on the scratch slot, sequences without tokens, tiles that begin
    beyond their sequence, wanted places that repeat row 0."""
    from llm_infer_amd.engine.prefill import PrefillRecorder
    from llm_infer_amd.engine.step import StepContext
    ctx = StepContext(None, [3, 1], [[5, 6, 7], [8] * 130], [10, 0], [[2], [0, 129]], upload=False)
    layout, total = PrefillRecorder._layout(192, 2, 4)
    assert [layout[k][1] for k in ("token_ids", "seq_slot", "want_rows", "tile_seq")] == [192, 2, 4, 4]
    packed = PrefillRecorder._fill(ctx, layout, total, scratch=9)
    get = lambda name: packed[layout[name][0]:layout[name][0] + layout[name][1]].tolist()
    assert get("token_ids")[:4] == [5, 6, 7, 8] and get("token_ids")[133:] == [0] * 59
    assert get("pos")[:5] == [10, 11, 12, 0, 1] and get("pos")[132] == 129
    assert get("tok_slot")[:4] == [3, 3, 3, 1] and set(get("tok_slot")[133:]) == {9}
    assert get("seq_slot") == [3, 1] and get("seq_qstart") == [0, 3] and get("seq_qlen") == [3, 130] and get("seq_ctx") == [13, 130]
    assert get("want_rows") == [2, 3, 132, 0]
    assert get("tile_seq") == [0, 1, 1, 0] and get("tile_q0") == [0, 0, 128, 1 << 30]
    # every array starts at a multiple of four elements (16 bytes)
    assert all(at % 4 == 0 for at, _ in layout.values()) and total % 4 == 0


def test_cache_rounding_option_is_for_a_float32_cache():
    with pytest.raises(CacheError, match="kv_round"):
        Cache([KVSpec(1, 16)], 256, 128, torch.bfloat16, None, 2, kv_round=torch.float16)
    with pytest.raises(CacheError, match="kv_round"):
        Cache([KVSpec(1, 16)], 256, 128, torch.float32, None, 2, kv_round=torch.float32)
    c = Cache([KVSpec(1, 16)], 256, 128, torch.float32, None, 2, kv_round=torch.float16)
    assert c.groups[0].round_to == torch.float16


def test_a_build_whose_hand_counted_kernel_spills_is_refused():
    """gemm_wreg places its own waits by counting its loads; a spill would be a load it does not count."""
    from llm_infer_amd.kernels import build
    ok = ("x.hip:1:1: remark: Function Name: _Z16gemm_wreg_kernelIDF16_Li4ELin1EEv [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:9:1: remark: Function Name: _Z15gemm_big_kernelIDF16_E [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:9:1: remark:     ScratchSize [bytes/lane]: 48 [-Rpass-analysis=kernel-resource-usage]\n")
    build._check_no_scratch(ok, "gemm_wreg_kernel", "x.hip")            # another kernel's scratch is its own business
    with pytest.raises(build.BuildError, match="16 bytes of scratch"):
        build._check_no_scratch(ok.replace("lane]: 0", "lane]: 16"), "gemm_wreg_kernel", "x.hip")
    with pytest.raises(build.BuildError, match="no resource usage"):
        build._check_no_scratch("", "gemm_wreg_kernel", "x.hip")
    assert build.NO_SCRATCH == {"gemm_prefill.hip": "gemm_wreg_kernel", "attention.hip": "attn_prefill_kernel"}


def test_build_folder_is_the_same_for_builds_that_run_side_by_side(tmp_path, monkeypatch):
    """Every library of one build lands in one folder: the probe for a writable folder must not
    collide between threads (a collision once sent some libraries to the temporary folder)."""
    from concurrent.futures import ThreadPoolExecutor
    from llm_infer_amd.kernels import build
    want = str(tmp_path / "libs")
    monkeypatch.setenv("LLM_INFER_AMD_BUILD_DIR", want)
    with ThreadPoolExecutor(max_workers=16) as pool:
        got = set(pool.map(lambda _: build.build_dir(), range(800)))
    assert got == {want} and os.listdir(want) == []


def test_a_current_library_is_taken_from_a_folder_that_cannot_be_written(tmp_path, monkeypatch):
    from llm_infer_amd.kernels import build
    kept, other = tmp_path / "kept", tmp_path / "other"
    kept.mkdir(); other.mkdir()
    monkeypatch.setenv("LLM_INFER_AMD_BUILD_DIR", str(kept))
    monkeypatch.setattr(build, "build_dir", lambda: str(other))            # as if `kept` were read-only
    def no_compiler():
        raise AssertionError("nothing has to be compiled")
    monkeypatch.setattr(build, "_hipcc", no_compiler)
    (kept / "libx.so").write_bytes(b"x")
    (kept / "libx.so.stamp").write_text(build._stamp((build.ATTN_SOURCE,), ("-DHEAD_DIM=16",)))
    assert build._build_library("libx.so", (build.ATTN_SOURCE,), ("-DHEAD_DIM=16",)) == str(kept / "libx.so")
    (kept / "libx.so.stamp").write_text("built from other sources")
    with pytest.raises(AssertionError, match="compiled"):
        build._build_library("libx.so", (build.ATTN_SOURCE,), ("-DHEAD_DIM=16",))


def test_command_line_follows_the_reference():
    c = parse_args(["m", "-i", "hi", "-n", "5", "-t", "0.5", "--seed", "7", "-T", "99"])
    assert (c["model"], c["prompt"], c["max_tokens"], c["temperature"], c["seed"], c["context"]) == \
        ("m", "hi", 5, 0.5, 7, 99)
    c = parse_args(["m", "--tokens", "1,2,3", "--tokens", "4 5"])
    assert c["tokens"] == [[1, 2, 3], [4, 5]] and c["max_tokens"] == 256 and c["temperature"] == 1.0
    assert parse_args(["m"]) is None and parse_args([]) is None
    assert parse_args(["m", "-i", "a", "-f", "b"]) is None and parse_args(["m", "-i", "a", "--bogus"]) is None
    assert parse_args(["m", "-i", "a", "-d", "cuda"]) is None and parse_args(["-h"])["help"]
    c = parse_args(["-", "--tokens", "1", "--random-weights", "--config", "c.json", "--slots", "2", "--dtype", "float16"])
    assert (c["random"], c["config"], c["slots"], c["dtype"]) == (True, "c.json", 2, "float16")
    assert parse_args(["m", "--tokens", "1", "--slots", "two"]) is None
    c = parse_args(["m", "--tokens", "1", "--dtype", "float32", "--kv-round", "float16"])
    assert (c["dtype"], c["kv_round"]) == ("float32", "float16") and parse_args(["m", "--tokens", "1"])["kv_round"] is None


def test_tokenizer_longest_match_and_bytes():
    vocab = {"<s>": 0, "</s>": 1, "a": 2, "ab": 3, "abc": 4, "▁b": 5, "c": 6, "<|eot_id|>": 300}
    vocab.update({f"<0x{i:02X}>": 10 + i for i in range(256)})
    t = Tokenizer(vocab, bos_id=0, eos_id=1)
    assert t.encode("abcab b", True) == [0, 4, 3, 5] and t.encode("abd", False) == [3, 10 + ord("d")]
    assert t.eot_id == 300 and t.decode([0, 5, 4, 10 + ord("!")]) == "<s>babc!"    # no blank after BOS
    assert t.decode(t.encode("cab é", False)) == "cab é"
