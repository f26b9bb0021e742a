"""The engine against the plain implementation for configurations drawn at random (seeded):
head sizes in steps of 16, group sizes that are no power of two, widths with and without the
factors that choose a kernel's path (8, 64), windows with and without attention sinks, heads rotated whole
or by half, tied and untied heads.  Each is replayed
whole, with its last tokens one by one and as a batch of unequal lengths, in both dtypes."""
import numpy as np
import pytest

import helpers
import schedules

pytestmark = pytest.mark.gpu


def random_config(seed):
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    n_kv = pick([1, 2, 3, 4])
    group = pick([1, 2, 3, 4, 5, 8])
    window = pick([0, 0, 24, 70])
    cfg = {
        "architectures": [pick(["LlamaForCausalLM", "MistralForCausalLM"])],
        "hidden_size": pick([64, 72, 104, 128, 136, 192, 200]),
        "intermediate_size": pick([136, 176, 200, 256, 320]),
        "num_hidden_layers": pick([1, 2, 3]),
        "num_attention_heads": n_kv * group,
        "num_key_value_heads": n_kv,
        "head_dim": pick([16, 32, 48, 64, 80, 96, 112, 128]),
        "vocab_size": int(rng.integers(200, 400)),
        "max_position_embeddings": 256,
        "rope_theta": float(pick([500.0, 10000.0, 1000000.0])),
        "rms_norm_eps": float(pick([1e-5, 1e-6, 3e-6])),
        "hidden_act": "silu",
        "tie_word_embeddings": bool(pick([True, False])),
        "bos_token_id": 1,
        "eos_token_id": 2,
    }
    if window:
        cfg["sliding_window"] = window
    # drawn after everything else, so that the seeds keep the sizes they had before these options existed
    sinks = pick([0, 1, 2, 4])
    if window and sinks:
        cfg["attention_sinks"] = sinks
    rotary = pick([1.0, 1.0, 0.5])
    if rotary != 1.0:
        cfg["partial_rotary_factor"] = rotary
    cfg["hidden_act"] = pick(["silu", "gelu"])
    return cfg


LENGTHS = [40, 1, 130, 67, 18]
SEEDS = [101, 102, 103, 104, 105, 106, 107, 127, 135, 185]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("random_models")
    return {seed: helpers.make_folder(tmp, "random%d" % seed, random_config(seed), seed=seed) for seed in SEEDS}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", SEEDS)
def test_random_configuration(folders, seed, dtype):
    from yalm_amd.engine import Engine, Model
    cfg = random_config(seed)
    model = Model.from_folder(folders[seed], dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=2048)
    requests = helpers.random_requests(cfg, LENGTHS, seed=seed)
    groups = [["r0", "r1", "r2"], ["r3", "r4", "r1"]]
    batch_requests = {"g%d_%s" % (gi, rid): requests[rid] for gi, ids in enumerate(groups) for rid in ids}
    batch_groups = [["g%d_%s" % (gi, rid) for rid in ids] for gi, ids in enumerate(groups)]
    first = {rid: max(1, len(t) // 2) for rid, t in batch_requests.items()}
    want = {rid: helpers.plain_logits(folders[seed], tuple(toks), dtype) for rid, toks in requests.items()}
    for what, reqs, steps in (("whole", requests, schedules.whole(requests)),
                              ("last 32 one by one", requests, schedules.tail_one_by_one(requests, 32)),
                              ("batches", batch_requests, schedules.batches(batch_requests, batch_groups, first))):
        out = schedules.replay_in_process(engine, steps)
        got = schedules.per_request(steps, out, reqs)
        for rid, toks in reqs.items():
            helpers.check_logits(got[rid], want[rid.split("_")[-1]], dtype,
                                 "seed %d %s %s %s request %s: %r" % (seed, cfg["architectures"][0], dtype, what, rid, cfg))
        assert not engine.cache.slots.held


def wide_random_config(seed):
    """Bigger sizes than random_config: widths up to 1,024 that are and are not multiples of 64 (the kernels' paths
    part there), more groups, longer windows, the other activation."""
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    n_kv = pick([1, 2, 3, 4, 8])
    group = pick([1, 2, 3, 4, 5, 8, 17])
    window = pick([0, 0, 24, 70, 200])
    cfg = {
        "architectures": [pick(["LlamaForCausalLM", "MistralForCausalLM"])],
        "hidden_size": pick([64, 72, 128, 192, 200, 256, 320, 512, 520, 1024]),
        "intermediate_size": pick([136, 176, 256, 320, 1000, 1024, 2048]),
        "num_hidden_layers": pick([1, 2, 3]),
        "num_attention_heads": n_kv * group,
        "num_key_value_heads": n_kv,
        "head_dim": pick([16, 32, 48, 64, 80, 96, 112, 128]),
        "vocab_size": int(rng.integers(200, 1200)),
        "max_position_embeddings": 512,
        "rope_theta": float(pick([500.0, 10000.0, 1000000.0])),
        "rms_norm_eps": float(pick([1e-5, 1e-6, 3e-6])),
        "hidden_act": pick(["silu", "gelu"]),
        "tie_word_embeddings": bool(pick([True, False])),
        "bos_token_id": 1,
        "eos_token_id": 2,
    }
    if window:
        cfg["sliding_window"] = window
        sinks = pick([0, 0, 1, 2, 4])
        if sinks:
            cfg["attention_sinks"] = sinks
    if pick([0, 0, 1]):
        cfg["partial_rotary_factor"] = 0.5
    return cfg


@pytest.mark.parametrize("seed", [1001, 1002, 1007, 1013, 1018, 1034, 1039, 1044])
def test_random_configuration_in_a_wide_batch(tmp_path, seed):
    """A configuration drawn at random, whole, with its last tokens one by one, and as ONE batch of 17 to 129 copies of
    its requests that start together, are cut at random places and end at different steps: the decode steps of 17 to
    128 rows (other GEMM kernels, the norm chain of the wide batches) with sequences of very unequal lengths."""
    from yalm_amd.engine import Engine, Model
    cfg = wide_random_config(seed)
    dtype = "bfloat16" if seed % 3 else "float32"
    folder = helpers.make_folder(tmp_path, "wide%d" % seed, cfg, seed=seed)
    rng = np.random.default_rng(seed + 7)
    lengths = [int(x) for x in rng.integers(1, 400, size=5)] + [1, 64, 65]
    model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=65536)
    requests = helpers.random_requests(cfg, lengths, seed=seed)
    want = {rid: helpers.plain_logits(folder, tuple(toks), dtype) for rid, toks in requests.items()}
    n = int(rng.integers(17, 130))
    ids = ["r%d" % int(rng.integers(len(lengths))) for _ in range(n)]
    wide = {"w%d_%s" % (i, rid): requests[rid] for i, rid in enumerate(ids)}
    first = {rid: int(rng.integers(1, max(2, len(t)))) for rid, t in wide.items()}
    for what, reqs, steps in (("whole", requests, schedules.whole(requests)),
                              ("last 32 one by one", requests, schedules.tail_one_by_one(requests, 32)),
                              ("wide batch", wide, schedules.batches(wide, [list(wide)], first))):
        out = schedules.replay_in_process(engine, steps)
        got = schedules.per_request(steps, out, reqs)
        for rid in reqs:
            helpers.check_logits(got[rid], want[rid.split("_")[-1]], dtype,
                                 "seed %d %s %s request %s: %r" % (seed, dtype, what, rid, cfg))
        assert not engine.cache.slots.held
