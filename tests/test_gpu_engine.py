"""The step function's own machinery against the plain implementation: batches that overlap in
time (a later batch starts while sequences of an earlier one are live and takes what their
leavers gave back), a batch of more than 256 rows (the largest graph buckets and the four-way
split of decode attention), graphs captured ahead of time and dropped again, and engines that
share one model."""
import numpy as np
import pytest
import torch

import helpers
import schedules
import tiny_configs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("engine_models")
    return {name: helpers.make_folder(tmp, name, cfg, seed=8) for name, cfg in tiny_configs.ALL.items()}


def make_engine(folders, name, dtype, **kw):
    from yalm_amd.engine import Engine, Model
    model = Model.from_folder(folders[name], dtype=helpers.torch_dtype(dtype), device="cuda:0")
    return Engine(model, **kw)


def poison_free_pages(engine):
    """Before every step, every page that no live sequence holds is filled with NaN: a kernel
    that reads behind a sequence's end, or a page that was given back, shows at once."""
    def before(step):
        for g in engine.cache.kv_groups:
            free = torch.tensor(sorted(g.pool._free), dtype=torch.long, device=g.k_pages.device)
            if free.numel():
                g.k_pages[:, free] = float("nan")
                g.v_pages[:, free] = float("nan")
    return before


OVERLAPPING = {
    # name: (lengths, groups of request indices, first-step lengths, first step of each group)
    "tiny_llama": ([40, 9, 128, 70, 5, 66, 100], [[0, 1, 2], [3, 4], [5, 6, 1]],
                   [[30, 2, 64], [65, 1], [3, 64, 9]], [0, 4, 30]),
    "tiny_mistral": ([30, 64, 12, 50, 41, 64], [[0, 1], [2, 3, 4], [5]], [[17, 40], [1, 33, 16], [2]], [0, 3, 45]),
    "small_windowed": ([300, 90, 200, 130, 64], [[0, 1], [2, 3], [4, 1]], [[260, 64], [97, 100], [1, 80]], [0, 5, 70]),
    # sinks beside the window: a slot that is taken again still holds its last sequence's sinks
    "tiny_sinks": ([150, 60, 200, 130, 64], [[0, 1], [2, 3], [4, 1]], [[120, 2], [97, 100], [1, 50]], [0, 5, 70]),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(OVERLAPPING))
def test_batches_that_overlap_in_time(folders, name, dtype):
    lengths, groups, firsts, start_at = OVERLAPPING[name]
    cfg = tiny_configs.ALL[name]
    base = helpers.random_requests(cfg, lengths, seed=9)
    requests, group_ids, first = {}, [], {}
    for gi, (idx, fl) in enumerate(zip(groups, firsts)):
        ids = []
        for i, f in zip(idx, fl):
            rid = "g%d_r%d" % (gi, i)
            requests[rid] = base["r%d" % i]
            first[rid] = f
            ids.append(rid)
        group_ids.append(ids)
    steps = schedules.interleaved(requests, group_ids, first, start_at)
    # the schedule does what it is for: some step starts a batch while another batch is live
    live, overlapped, most_live = set(), False, 0
    for s in steps:
        ids = {e["id"] for e in s["entries"]}
        if not ids & live and live:
            overlapped = True
        live |= ids
        most_live = max(most_live, len(live))
        live -= set(s["end"])
    assert overlapped and most_live < len(requests)
    # a cache with no room to spare: newcomers must take the slots and pages the leavers gave back
    engine = make_engine(folders, name, dtype, max_tokens=schedules.max_tokens_needed(steps), max_batch=most_live)
    out = schedules.replay_in_process(engine, steps, before_step=poison_free_pages(engine))
    got = schedules.per_request(steps, out, requests)
    for rid, toks in requests.items():
        want = helpers.plain_logits(folders[name], tuple(toks), dtype)
        helpers.check_logits(got[rid], want, dtype, "%s %s overlapping batches, request %s" % (name, dtype, rid))
    assert not engine.cache.slots.held
    for g in engine.cache.kv_groups:
        assert g.pool.n_free == g.n_pages


# head size 64 and two KV heads: the matrix-core decode attention, and 2 x 260 > 512 workgroups
MANY_ROWS = dict(tiny_configs.TINY_LONG, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
                 hidden_size=128, max_position_embeddings=1024)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_more_than_256_rows(tmp_path_factory, dtype):
    """260 sequences of 520 to 600 tokens start together and decode up to four tokens each: graph
    buckets 512 and 256, decode attention split in four because its workgroups outnumber what the
    chip holds at once.  Every 13th request is compared with the plain implementation."""
    from yalm_amd.engine import Engine, Model
    folder = helpers.make_folder(tmp_path_factory.mktemp("many_rows"), "many_rows", MANY_ROWS, seed=10)
    rng = np.random.default_rng(11)
    n = 260
    lengths = [int(x) for x in rng.integers(520, 601, size=n)]
    requests = helpers.random_requests(MANY_ROWS, lengths, seed=12)
    first = {rid: len(t) - 1 - (i % 4) for i, (rid, t) in enumerate(requests.items())}
    steps = schedules.batches(requests, [list(requests)], first)
    for s in steps:                                   # logits only where they are compared
        for e in s["entries"]:
            if int(e["id"][1:]) % 13 and len(e["tokens"]) > 1:
                e["want"] = []
    model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=schedules.max_tokens_needed(steps), max_batch=n)
    mixer = model.blocks[0].mixer
    if dtype == "bfloat16":
        assert mixer.decode_splits(n, 16) == 4 and mixer.decode_splits(64, 16) == 2      # the four-way branch
    out = schedules.replay_in_process(engine, steps)
    assert {k[0] for k in engine._graphs} >= {512, 256}
    rows = {rid: {} for rid in requests}
    pos = {rid: 0 for rid in requests}
    for s in steps:
        r = 0
        for e in s["entries"]:
            for j in e["want"]:
                rows[e["id"]][pos[e["id"]] + j] = out[s["step"]][r]
                r += 1
            pos[e["id"]] += len(e["tokens"])
    checked = 0
    for i, (rid, toks) in enumerate(requests.items()):
        whole = i % 13 == 0
        if not whole and i % 26 != 1:
            continue
        places = sorted(rows[rid])
        assert places == list(range(0 if whole else first[rid], len(toks)))
        want = helpers.plain_logits(folder, tuple(toks), dtype)
        helpers.check_logits(np.stack([rows[rid][p] for p in places]), want[places], dtype,
                             "260 rows %s request %s" % (dtype, rid))
        checked += 1
    assert checked >= 25


def test_warmup_captures_ahead_and_leaves_live_sequences_alone(folders):
    """Graphs are captured on padding rows: in the middle of a request, for the bucket the request
    is in, and nothing the request holds changes; afterwards no live step captures."""
    name, dtype = "tiny_llama", "float32"
    engine = make_engine(folders, name, dtype, max_tokens=1024, max_batch=4, max_graphs=6)
    requests = helpers.random_requests(tiny_configs.ALL[name], [100, 37], seed=13)
    first = {"r0": 60, "r1": 5}
    steps = schedules.batches(requests, [["r0", "r1"]], first)
    seen = []

    def before(step):
        if step["step"] == 3:
            free = [g.pool.n_free for g in engine.cache.kv_groups]
            held = engine.cache.slots.held
            assert engine.warmup(batch_sizes=[1, 2], max_len=128, min_len=1) >= 2
            assert [g.pool.n_free for g in engine.cache.kv_groups] == free and engine.cache.slots.held == held
        seen.append(engine.graphs_captured)
    out = schedules.replay_in_process(engine, steps, before_step=before)
    assert seen[3] > seen[2] and seen[-1] == seen[3]          # none captured by a live step after the warm-up
    got = schedules.per_request(steps, out, requests)
    for rid, toks in requests.items():
        helpers.check_logits(got[rid], helpers.plain_logits(folders[name], tuple(toks), dtype), dtype, "warmup " + rid)
    with pytest.raises(ValueError):
        engine.warmup(batch_sizes=list(range(1, 65)), max_len=128)      # more graphs than the engine keeps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_least_recently_used_graphs_are_dropped(folders, dtype):
    name = "tiny_long"
    engine = make_engine(folders, name, dtype, max_tokens=4096, max_graphs=2)
    requests = helpers.random_requests(tiny_configs.ALL[name], [300, 64, 129, 70], seed=14)
    # buckets (4, 1) .. (4, 8), then smaller batches as the short requests end
    steps = schedules.batches(requests, [["r0", "r1", "r2", "r3"]], {"r0": 40, "r1": 1, "r2": 60, "r3": 2})
    out = schedules.replay_in_process(engine, steps)
    assert len(engine._graphs) <= 2 and engine.graphs_captured > 2
    got = schedules.per_request(steps, out, requests)
    for rid, toks in requests.items():
        helpers.check_logits(got[rid], helpers.plain_logits(folders[name], tuple(toks), dtype), dtype, "lru " + rid)
    before = engine.graph_bytes()
    engine.drop_graphs()
    assert engine.graph_bytes() <= before and not engine._graphs


def test_engines_that_share_a_model(folders):
    """A second engine with a longer context makes the model's rotation table grow while the first
    engine's graphs still point at the old one: the first engine notices and captures again."""
    from yalm_amd.engine import Engine, Model
    name, dtype = "tiny_long", "float32"
    model = Model.from_folder(folders[name], dtype=torch.float32, device="cuda:0")
    small = Engine(model, max_tokens=128)
    table = model.blocks[0].mixer.position.table
    assert table.shape[0] == 128
    requests = helpers.random_requests(tiny_configs.ALL[name], [100, 90], seed=15)
    want = {rid: helpers.plain_logits(folders[name], tuple(t), dtype) for rid, t in requests.items()}
    slot = small.start(1)
    logits = [small.step(slot, [requests["r0"][:60]], [list(range(60))]).cpu().numpy()]
    for t in requests["r0"][60:80]:
        logits.append(small.step(slot, [[t]]).cpu().numpy())
    captured = small.graphs_captured
    assert captured > 0
    big = Engine(model, max_tokens=2048)                         # the table grows to 1,024 positions
    assert model.blocks[0].mixer.position.table.shape[0] == 1024
    same = Engine(model, max_tokens=256)                          # a sufficient table is left alone
    assert model.blocks[0].mixer.position.table.shape[0] == 1024 and same.n_positions == 256
    del table
    junk = torch.full((1 << 20,), float("nan"), device="cuda:0")  # whatever now lies where the old table was
    for t in requests["r0"][80:]:
        logits.append(small.step(slot, [[t]]).cpu().numpy())
    small.release(slot)
    assert small.graphs_captured > captured
    helpers.check_logits(np.concatenate(logits), want["r0"], dtype, "the small engine across the table's growth")
    steps = schedules.tail_one_by_one({"r1": requests["r1"]}, 30)
    got = schedules.per_request(steps, schedules.replay_in_process(big, steps), {"r1": requests["r1"]})
    helpers.check_logits(got["r1"], want["r1"], dtype, "the big engine")
    slot = small.start(1)
    with pytest.raises(ValueError):
        small.step(slot, [list(range(129))])                     # beyond the small engine's own positions
    small.release(slot)
    del junk


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_token_probabilities_in_blocks_of_rows(folders, dtype):
    """A step asked for the probability of given tokens makes its logits a few rows at a time;
    the result is softmax(plain logits)[target] at every wanted place, for whole prompts of
    unequal lengths and for the single tokens behind them."""
    name = "tiny_llama3"
    engine = make_engine(folders, name, dtype, max_tokens=1024)
    engine.HEAD_ROWS = 7                                   # several blocks, the last one short
    requests = helpers.random_requests(tiny_configs.ALL[name], [60, 23], seed=16)
    toks = list(requests.values())
    slots = engine.start(2)
    first = [50, 20]
    want_places = [list(range(f - 1)) for f in first]
    got = engine.step(slots, [t[:f] for t, f in zip(toks, first)], want_places,
                      targets=[t[1:f] for t, f in zip(toks, first)]).cpu().numpy()
    after = engine.step(slots, [[t[f]] for t, f in zip(toks, first)], targets=[[t[f + 1]] for t, f in zip(toks, first)])
    engine.release(slots)
    want, want_after, scale = [], [], 1.0
    for t, f in zip(toks, first):
        logits = torch.from_numpy(helpers.plain_logits(folders[name], tuple(t), dtype)).double()
        scale = max(scale, float(logits.abs().max()))
        p = torch.log_softmax(logits, dim=-1)
        want += [float(p[i, t[i + 1]]) for i in range(f - 1)]
        want_after.append(float(p[f, t[f + 1]]))
    # log p = logit - log sum exp: twice the bound on a logit's error
    tol = 2 * (helpers.F32_TOL if dtype == "float32" else helpers.BF16_MAX_TOL) * scale
    assert got.shape == (len(want),) and (got > 0).all()
    assert np.abs(np.log(got.astype(np.float64)) - np.asarray(want)).max() <= tol
    assert np.abs(np.log(after.cpu().numpy().astype(np.float64)) - np.asarray(want_after)).max() <= tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_in_the_largest_graph_bucket(tmp_path_factory, dtype):
    """520 sequences of 3 to 90 tokens decode together: the graph bucket of 1,024 rows, half of them
    padding.  Every 40th request is compared with the plain implementation at every place."""
    from yalm_amd.engine import Engine, Model
    folder = helpers.make_folder(tmp_path_factory.mktemp("bucket_1024"), "many_rows", MANY_ROWS, seed=10)
    rng = np.random.default_rng(21)
    n = 520
    lengths = [int(x) for x in rng.integers(3, 91, size=n)]
    requests = helpers.random_requests(MANY_ROWS, lengths, seed=22)
    first = {rid: len(t) - 2 for rid, t in requests.items()}
    steps = schedules.batches(requests, [list(requests)], first)
    for s in steps:
        for e in s["entries"]:
            if int(e["id"][1:]) % 40:
                e["want"] = []
    model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=schedules.max_tokens_needed(steps), max_batch=n)
    out = schedules.replay_in_process(engine, steps)
    assert 1024 in {k[0] for k in engine._graphs}
    got = {rid: [] for rid in requests if int(rid[1:]) % 40 == 0}
    for s in steps:
        r = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got[e["id"]].append(out[s["step"]][r])
                r += 1
    assert len(got) == 13
    for rid, rows in got.items():
        want = helpers.plain_logits(folder, tuple(requests[rid]), dtype)
        helpers.check_logits(np.stack(rows), want, dtype, "bucket 1024 %s request %s" % (dtype, rid))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["tiny_llama", "tiny_mistral"])
def test_a_sequence_at_its_first_token_beside_sequences_that_go_on(folders, name, dtype):
    """A step of one token each in which one sequence has nothing in the cache yet: the step function
    takes it as a decode step (position 0 beside later positions); that sequence's first page is
    new, the others' pages are old."""
    engine = make_engine(folders, name, dtype, max_tokens=1024)
    requests = helpers.random_requests(tiny_configs.ALL[name], [40, 12, 9], seed=23)
    a, b, c = (requests[r] for r in ("r0", "r1", "r2"))
    sa, sb = engine.start(2)
    rows = {"a": [], "b": [], "c": []}
    first = engine.step([sa, sb], [a[:30], b[:5]], [list(range(30)), list(range(5))]).cpu().numpy()
    rows["a"] += list(first[:30])
    rows["b"] += list(first[30:])
    (sc,) = engine.start(1)
    for k in range(7):                                     # c joins at its position 0, then all go on
        out = engine.step([sa, sc, sb], [[a[30 + k]], [c[k]], [b[5 + k]]]).cpu().numpy()
        rows["a"].append(out[0])
        rows["c"].append(out[1])
        rows["b"].append(out[2])
    engine.release([sa, sb, sc])
    for key, toks in (("a", a), ("b", b), ("c", c)):
        want = helpers.plain_logits(folders[name], tuple(toks), dtype)[:len(rows[key])]
        helpers.check_logits(np.stack(rows[key]), want, dtype, "%s %s joined at position 0, sequence %s" % (name, dtype, key))


def test_a_step_whose_widest_buffer_would_pass_the_checked_size_is_refused(folders):
    from yalm_amd.engine.engine import StepError
    engine = make_engine(folders, "tiny_llama", "float32", max_tokens=1024)
    assert engine.MAX_ELEMENTS == 1 << 31 and engine._widest_row == 176       # the feed-forward's hidden width
    engine.MAX_ELEMENTS = 176 * 20
    slots = engine.start(1)
    with pytest.raises(StepError, match="2\\^31"):
        engine.step(slots, [list(range(20))])
    assert engine.length(slots[0]) == 0                    # refused before anything was taken
    engine.step(slots, [list(range(13))])                  # 13 x 176 and one row of 256 logits fit
    with pytest.raises(StepError, match="2\\^31"):         # the logits alone: 14 rows x 256 reach 176 x 20
        s2 = engine.start(1)
        engine.step(s2, [list(range(15))], [list(range(14))])
    engine.release(slots + s2)


# widths that let every product of a decode step of 17..128 rows take the kernels that split K and chain the norms
# (K a multiple of 64 beyond 64 rows), and one that does not (hidden 144: beyond 64 rows its down projection goes
# another way)
MID_ROWS = dict(MANY_ROWS, intermediate_size=192)
MID_ROWS_ODD = dict(MANY_ROWS, intermediate_size=144, hidden_size=136, num_attention_heads=2, num_key_value_heads=1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,which", [(40, "even"), (100, "even"), (23, "odd"), (90, "odd")])
def test_decode_batches_of_17_to_128_rows(tmp_path_factory, n, which, dtype):
    """Decode steps of 17..128 sequences: the products whose K is split over workgroups, the kernel that adds the
    slices to the residual stream and prepares the next norm, and the consumers that scale their sums row by row.
    Sequences of unequal lengths, the shorter ones end earlier (the batch shrinks through the buckets); every fifth
    request is compared with the plain implementation at every place."""
    from yalm_amd.engine import Engine, Model
    cfg = MID_ROWS if which == "even" else MID_ROWS_ODD
    folder = helpers.make_folder(tmp_path_factory.mktemp("mid_rows"), "mid_rows_" + which, cfg, seed=30)
    rng = np.random.default_rng(31 + n)
    lengths = [int(x) for x in rng.integers(6, 80, size=n)]
    requests = helpers.random_requests(cfg, lengths, seed=32)
    first = {rid: max(1, len(t) - 5 - (i % 7)) for i, (rid, t) in enumerate(requests.items())}
    steps = schedules.batches(requests, [list(requests)], first)
    for s in steps:
        for e in s["entries"]:
            if int(e["id"][1:]) % 5:
                e["want"] = []
    model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=schedules.max_tokens_needed(steps), max_batch=n)
    out = schedules.replay_in_process(engine, steps)
    got = {rid: [] for rid in requests if int(rid[1:]) % 5 == 0}
    for s in steps:
        r = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got[e["id"]].append(out[s["step"]][r])
                r += 1
    for rid, rows in got.items():
        want = helpers.plain_logits(folder, tuple(requests[rid]), dtype)
        helpers.check_logits(np.stack(rows), want, dtype, "%d rows (%s) %s request %s" % (n, which, dtype, rid))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_decode_batch_of_very_unequal_lengths(tmp_path_factory, dtype):
    """Sequences of 30 to 900 tokens decode together: the step counts as ragged (its own captured graphs), the
    attention cuts every sequence into splits of the longest one's split size, and the short ones end early."""
    from yalm_amd.engine import Engine, Model
    folder = helpers.make_folder(tmp_path_factory.mktemp("ragged"), "many_rows", MANY_ROWS, seed=10)
    lengths = [900, 30, 410, 64, 65, 700, 129, 33, 512, 250, 31, 880]
    requests = helpers.random_requests(MANY_ROWS, lengths, seed=41)
    first = {rid: len(t) - 3 - (i % 5) for i, (rid, t) in enumerate(requests.items())}
    steps = schedules.batches(requests, [list(requests)], first)
    model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=schedules.max_tokens_needed(steps), max_batch=len(lengths))
    assert engine._is_ragged(lengths) and not engine._is_ragged([900, 880, 860]) and not engine._is_ragged([5])
    out = schedules.replay_in_process(engine, steps)
    assert any(key[2] for key in engine._graphs)                  # graphs of the ragged kind were captured and used
    if dtype == "bfloat16":
        mixer = model.blocks[0].mixer
        assert mixer.decode_splits(64, 16, ragged=True) == 4 and mixer.decode_splits(64, 16) == 2
    got = schedules.per_request(steps, out, requests)
    for rid, toks in requests.items():
        want = helpers.plain_logits(folder, tuple(toks), dtype)
        helpers.check_logits(got[rid][first[rid] - 1:], want[first[rid] - 1:], dtype, "ragged batch %s request %s" % (dtype, rid))
