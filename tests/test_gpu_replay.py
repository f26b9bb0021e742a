"""The engine against the plain implementation under every way of cutting the
requests into steps: each request alone and whole; with the last 32 tokens one
by one; in batches of unequal lengths whose shorter requests end earlier, one
batch after another so that slots and pages are used again (the cache is
poisoned with NaN between batches).  float32 and bfloat16, eight tiny
configurations."""
import numpy as np
import pytest
import torch

import helpers
import schedules
import tiny_configs

pytestmark = pytest.mark.gpu

LENGTHS = {
    "tiny_llama": [5, 17, 1, 40, 100, 128],
    "tiny_mistral": [2, 30, 9, 23, 64, 50],
    "tiny_llama3": [3, 70, 200, 33],
    "tiny_wide_heads": [150, 33, 260, 64, 65],
    "tiny_long": [700, 64, 129],
    "small_windowed": [300, 97, 64, 200, 31],
    "small_sinks": [300, 97, 130, 200, 31],
    "tiny_sinks": [150, 33, 260, 64, 41, 3],
}
# batches: (request indices, first-step lengths)
GROUPS = {
    "tiny_llama": [([0, 1, 2], [5, 17, 1]), ([3, 4, 5], [8, 64, 65]), ([1, 0], [1, 2])],
    "tiny_mistral": [([0, 1, 2, 3], [2, 30, 9, 23]), ([4, 5], [40, 17]), ([3, 2, 1], [1, 3, 16])],
    "tiny_llama3": [([0, 1], [1, 33]), ([2, 3], [130, 20]), ([1], [64])],
    "tiny_wide_heads": [([0, 1, 2], [120, 3, 101]), ([3, 4], [63, 64]), ([1, 0], [32, 100])],
    "tiny_long": [([0, 1, 2], [500, 1, 100]), ([2, 1], [128, 63])],
    "small_windowed": [([0, 1, 2], [250, 96, 1]), ([3, 4, 1], [97, 30, 60])],
    # a request that starts with one token writes its sinks in decode steps and passes the window later
    "small_sinks": [([0, 1, 2], [250, 96, 1]), ([3, 4, 1], [97, 30, 60])],
    "tiny_sinks": [([0, 1, 2], [120, 3, 101]), ([3, 4, 5], [1, 40, 2]), ([1, 0], [32, 100])],
}

_engines = {}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    return {name: helpers.make_folder(tmp, name, cfg, seed=3) for name, cfg in tiny_configs.ALL.items()}


def engine_for(folders, name, dtype, max_tokens=4096):
    from yalm_amd.engine import Engine, Model
    key = (name, dtype, max_tokens)
    if key not in _engines:
        model = Model.from_folder(folders[name], dtype=helpers.torch_dtype(dtype), device="cuda:0")
        _engines[key] = Engine(model, max_tokens=max_tokens)
    return _engines[key]


def poison_when_idle(engine):
    def before(step):
        if not engine.cache.slots.held:
            for g in engine.cache.kv_groups:
                g.k_pages.fill_(float("nan"))
                g.v_pages.fill_(float("nan"))
    return before


def compare(folders, name, dtype, steps, requests, engine, what):
    out = schedules.replay_in_process(engine, steps, before_step=poison_when_idle(engine))
    got = schedules.per_request(steps, out, requests)
    for rid, toks in requests.items():
        want = helpers.plain_logits(folders[name], tuple(toks), dtype)
        helpers.check_logits(got[rid], want, dtype, "%s %s %s request %s (%d tokens)" % (name, dtype, what, rid, len(toks)))
    assert not engine.cache.slots.held
    for g in engine.cache.kv_groups:
        assert g.pool.n_free == g.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_each_request_alone_and_whole(folders, name, dtype):
    cfg = tiny_configs.ALL[name]
    requests = helpers.random_requests(cfg, LENGTHS[name], seed=5)
    compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_last_32_tokens_one_by_one(folders, name, dtype):
    cfg = tiny_configs.ALL[name]
    requests = helpers.random_requests(cfg, LENGTHS[name], seed=5)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, 32), requests,
            engine_for(folders, name, dtype), "last 32 one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_unequal_batches_with_reuse(folders, name, dtype):
    cfg = tiny_configs.ALL[name]
    base = helpers.random_requests(cfg, LENGTHS[name], seed=5)
    requests, groups, prompt_lens = {}, [], {}
    for gi, (idx, firsts) in enumerate(GROUPS[name]):
        ids = []
        for i, p in zip(idx, firsts):
            rid = "g%d_r%d" % (gi, i)
            requests[rid] = base["r%d" % i]
            prompt_lens[rid] = min(p, len(requests[rid]))
            ids.append(rid)
        groups.append(ids)
    steps = schedules.batches(requests, groups, prompt_lens)
    compare(folders, name, dtype, steps, requests, engine_for(folders, name, dtype), "batches")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("min_tokens", [0, 1 << 30])
@pytest.mark.parametrize("name", ["tiny_sinks", "tiny_wide_heads", "tiny_long", "small_sinks"])
def test_prompt_steps_with_either_rotation_kernel(folders, name, min_tokens, dtype, monkeypatch):
    """A prompt step rotates and stores a page-shaped tile at a time from a number of tokens on and token by
    token below it: the same logits with the choice forced either way."""
    from yalm_amd.parts import attention
    monkeypatch.setattr(attention, "ROPE_TILES_MIN_TOKENS", min_tokens)
    cfg = tiny_configs.ALL[name]
    requests = helpers.random_requests(cfg, LENGTHS[name], seed=5)
    compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n_requests", [("tiny_llama", 20), ("tiny_mistral", 40), ("tiny_wide_heads", 70),
                                             ("tiny_llama", 130), ("small_windowed", 24), ("small_windowed", 66)])
def test_batches_of_many_requests(folders, name, n_requests, dtype):
    """Decode batches beyond 16, 64 and 128 rows take other GEMM kernels (split-K, tiled), norm and
    rotation kernels of their own and other graph buckets than the small batches; the requests have
    unequal lengths and end one after another, so the batch passes through the smaller buckets too."""
    cfg = tiny_configs.ALL[name]
    rng = np.random.default_rng(n_requests)
    lengths = [int(x) for x in rng.integers(2, 15, size=n_requests)]
    lengths[0], lengths[1] = 40, 33                      # two that outlive the others
    requests = helpers.random_requests(cfg, lengths, seed=11)
    first = {rid: int(rng.integers(1, len(t) + 1)) for rid, t in requests.items()}
    first["r1"] = 1
    steps = schedules.batches(requests, [list(requests)], first)
    compare(folders, name, dtype, steps, requests, engine_for(folders, name, dtype, max_tokens=16384), "many requests")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_eager_equals_graph(folders, dtype):
    """The same steps with and without HIP graphs give the same bits."""
    from yalm_amd.engine import Engine, Model
    name = "tiny_mistral"
    cfg = tiny_configs.ALL[name]
    requests = helpers.random_requests(cfg, [20, 45, 7], seed=8)
    steps = schedules.batches(requests, [list(requests)], {"r0": 3, "r1": 20, "r2": 1})
    model = Model.from_folder(folders[name], dtype=helpers.torch_dtype(dtype), device="cuda:0")
    a = schedules.replay_in_process(Engine(model, max_tokens=1024, use_graphs=True), steps)
    b = schedules.replay_in_process(Engine(model, max_tokens=1024, use_graphs=False), steps)
    for k in a:
        assert np.array_equal(a[k], b[k]), "step %s differs between graph and eager decode" % k


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_padding_and_company_change_nothing(folders, dtype):
    """A request's logits are the same alone, in a batch of 3 (padded to a bucket of 4),
    and in another slot, up to rounding; in float32 the decode bits are equal."""
    name = "tiny_llama"
    cfg = tiny_configs.ALL[name]
    engine = engine_for(folders, name, dtype)
    requests = helpers.random_requests(cfg, [30, 12, 50], seed=9)
    alone = schedules.batches({"r0": requests["r0"]}, [["r0"]], {"r0": 10})
    a = schedules.per_request(alone, schedules.replay_in_process(engine, alone), {"r0": requests["r0"]})["r0"]
    # occupy a slot first, so that r0 lands elsewhere, then run it in company
    dummy = engine.start(1)
    both = schedules.batches(requests, [["r2", "r0", "r1"]], {"r0": 10, "r1": 12, "r2": 31})
    b = schedules.per_request(both, schedules.replay_in_process(engine, both), requests)["r0"]
    engine.release(dummy)
    want = helpers.plain_logits(folders[name], tuple(requests["r0"]), dtype)
    helpers.check_logits(a, want, dtype, "alone")
    helpers.check_logits(b, want, dtype, "in company")
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert np.abs(a - b).max() <= tol * max(1.0, np.abs(want).max())


def test_trace_run_program(folders, tmp_path):
    """bin/trace_run itself, as a user runs it: unequal batches in both dtypes."""
    name = "tiny_mistral"
    cfg = tiny_configs.ALL[name]
    requests = helpers.random_requests(cfg, [33, 12, 40], seed=10)
    steps = schedules.batches(requests, [["r0", "r1"], ["r2"]], {"r0": 7, "r1": 12, "r2": 1})
    # a step that wants nothing writes no file
    steps[1]["entries"][0]["want"] = []
    for dtype in ("float32", "bfloat16"):
        out = schedules.replay_trace_run(folders[name], dtype, steps, str(tmp_path / dtype),
                                         schedules.max_tokens_needed(steps))
        vocab = cfg["vocab_size"]
        got = {rid: np.full((len(t), vocab), np.nan, np.float32) for rid, t in requests.items()}
        pos = {rid: 0 for rid in requests}
        for s in steps:
            row = 0
            for e in s["entries"]:
                for j in e["want"]:
                    got[e["id"]][pos[e["id"]] + j] = out[s["step"]][row]
                    row += 1
                pos[e["id"]] += len(e["tokens"])
        for rid, toks in requests.items():
            want = helpers.plain_logits(folders[name], tuple(toks), dtype)
            keep = ~np.isnan(got[rid]).any(axis=1)
            assert keep.sum() >= len(toks) - 1
            helpers.check_logits(got[rid][keep], want[keep], dtype, "trace_run %s %s" % (dtype, rid))


FULL_WIDTH = {"architectures": ["MistralForCausalLM"], "hidden_size": 4096, "intermediate_size": 14336,
              "num_hidden_layers": 1, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
              "vocab_size": 4096, "max_position_embeddings": 4096, "rope_theta": 1e6, "rms_norm_eps": 1e-5,
              "hidden_act": "silu", "tie_word_embeddings": False, "bos_token_id": 1, "eos_token_id": 2}


# the widths of Llama-3.2-3B: 24 heads in groups of 3, outputs of 3,072 (192 workgroups of 16 rows), llama3
# rope scaling, and the head shared with the embedding at a vocabulary that is no power of two
WIDTH_3B = {"architectures": ["LlamaForCausalLM"], "hidden_size": 3072, "intermediate_size": 8192,
            "num_hidden_layers": 1, "num_attention_heads": 24, "num_key_value_heads": 8, "head_dim": 128,
            "vocab_size": 5003, "max_position_embeddings": 4096, "rope_theta": 500000.0, "rms_norm_eps": 1e-5,
            "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                             "original_max_position_embeddings": 64},
            "hidden_act": "silu", "tie_word_embeddings": True, "bos_token_id": 1, "eos_token_id": 2}


@pytest.mark.parametrize("name,FULL_WIDTH", [("mistral_7b", FULL_WIDTH), ("llama_3b", WIDTH_3B)])
def test_one_layer_at_the_width_of_the_big_models(tmp_path_factory, name, FULL_WIDTH):
    """One layer with the sizes of Mistral-7B or Llama-3.2-3B (a small vocabulary): the kernels take their
    big-shape paths (256x256 and 128x128 GEMM tiles in the prompt step, 256 parts in the norm chain, split-K
    for 20 rows, matrix-core attention with 4 or 3 heads a group), and the logits still follow the plain
    implementation."""
    from yalm_amd.engine import Engine, Model
    folder = helpers.make_folder(tmp_path_factory.mktemp("wide"), "full_width_" + name, FULL_WIDTH, seed=1,
                                 stored=torch.bfloat16)
    model = Model.from_folder(folder, dtype=torch.bfloat16, device="cuda:0")
    engine = Engine(model, max_tokens=4096)
    requests = helpers.random_requests(FULL_WIDTH, [200, 70, 33] + [6 + (i % 5) for i in range(17)], seed=12)
    ids = list(requests)
    three = {rid: requests[rid] for rid in ids[:3]}
    first = {rid: max(1, len(requests[rid]) - 3) for rid in ids}
    first[ids[0]] = 180
    for reqs, steps in ((three, schedules.batches(three, [ids[:3]], {ids[0]: 200 - 32, ids[1]: 70, ids[2]: 1})),
                        (requests, schedules.batches(requests, [ids], first))):               # 3 rows, then 20 rows
        got = schedules.per_request(steps, schedules.replay_in_process(engine, steps), reqs)
        for rid, toks in reqs.items():
            want = helpers.plain_logits(folder, tuple(toks), "bfloat16")
            helpers.check_logits(got[rid], want, "bfloat16", "full width, request %s (%d tokens)" % (rid, len(toks)))
    assert not engine.cache.slots.held


# the Mistral-7B-v0.2 shape at its real layer sizes and vocabulary, all 32 layers
WHOLE_7B = dict(FULL_WIDTH, vocab_size=32000, num_hidden_layers=32, max_position_embeddings=32768)


@pytest.fixture(scope="module")
def folder_7b(tmp_path_factory):
    folder = helpers.make_folder(tmp_path_factory.mktemp("layers_7b"), "layers_7b", WHOLE_7B, seed=21,
                                 stored=torch.bfloat16, device="cuda:0")
    yield folder
    helpers.forget_plain_results()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_whole_mistral_7b_shape(folder_7b, dtype):
    """All 32 layers of 4096 x 14336 with 32/8 heads of 128 and the head of 32000 x 4096: three requests of at
    most 48 tokens, each alone and whole, with its last 32 tokens one by one, and as a batch of unequal
    lengths, in the true 32-bit path and in bfloat16, against the plain implementation on the same
    (bfloat16-stored) weights."""
    from yalm_amd.engine import Engine, Model
    model = Model.from_folder(folder_7b, dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=1024)
    requests = helpers.random_requests(WHOLE_7B, [48, 33, 17], seed=22)
    first = {"r0": 20, "r1": 33 - 5, "r2": 1}
    for what, steps in (("whole", schedules.whole(requests)),
                        ("last 32 one by one", schedules.tail_one_by_one(requests, 32)),
                        ("a batch of unequal lengths", schedules.batches(requests, [list(requests)], first))):
        got = schedules.per_request(steps, schedules.replay_in_process(engine, steps), requests)
        for rid, toks in requests.items():
            want = helpers.plain_logits(folder_7b, tuple(toks), dtype)
            helpers.check_logits(got[rid], want, dtype, "7B sizes, 32 layers, %s, %s, request %s" % (dtype, what, rid))
    assert not engine.cache.slots.held
    del engine, model
    torch.cuda.empty_cache()
