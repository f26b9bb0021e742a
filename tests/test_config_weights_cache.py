"""CPU tests: configuration and registry, the safetensors container and weight
errors, the cache's bookkeeping (no slot or page lost, held twice or freed
twice), the generation loop's decisions (with a scripted step function), the
sampler's random numbers, and the tokenizer."""
import json
import os
import struct

import numpy as np
import pytest
import torch

import tiny_configs
from yalm_amd.cache import CacheError, CacheFull, CacheManager, KVRequest, PagePool, SlotAllocator, StateRequest
from yalm_amd.config import (ConfigError, LlamaConfig, ModelSpec, PartSpec, ScheduleEntry, config_from_dict,
                             register_architecture, registered_architectures, unregister_architecture)
from yalm_amd.generate import generate, plan_batches
from yalm_amd.weights import SafetensorsError, SafetensorsFile, TensorSource, WeightsError, write_file, \
    write_random_model
from yalm_amd.weights.loader import device_dtype
from yalm_amd.weights.random_init import random_values


# ------------------------------------------------------------------ configuration

def test_config_reads_the_architectures_own_keys():
    c = config_from_dict(tiny_configs.TINY_MISTRAL)
    assert isinstance(c, LlamaConfig)
    assert (c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (96, 256, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 1, 32)
    assert c.sliding_window == 16 and c.rope_theta == 1e6 and c.rms_norm_eps == 1e-6
    assert c.tie_word_embeddings is False and c.eos_token_ids == [2]
    # defaults of convert.py:34-44
    d = {k: v for k, v in tiny_configs.TINY_LLAMA.items() if k not in ("head_dim", "num_key_value_heads", "rope_theta",
                                                                       "tie_word_embeddings")}
    c = config_from_dict(d)
    assert c.head_dim == 16 and c.num_key_value_heads == 4 and c.rope_theta == 10000.0
    assert c.tie_word_embeddings is True                      # absent -> tied (convert.py:241)
    assert config_from_dict(dict(d, sliding_window=None)).sliding_window == 0
    assert config_from_dict(dict(d, eos_token_id=[2, 7])).eos_token_ids == [2, 7]
    # round trip
    assert config_from_dict(c.to_dict()) == c
    c3 = config_from_dict(tiny_configs.TINY_LLAMA3)
    assert c3.rope_scaling.factor == 8.0 and config_from_dict(c3.to_dict()) == c3


def test_a_context_is_two_sinks_and_a_window():
    """The reference's -T n (src/infer.cpp:484-488, src/model.h:12): 2 sinks beside the last n - 2."""
    c = config_from_dict(tiny_configs.TINY_LLAMA)
    assert c.with_context(0) is c and c.attention_sinks == 0
    t = c.with_context(40)
    assert (t.sliding_window, t.attention_sinks) == (38, 2)
    assert all(l.mixer.params["window"] == 38 and l.mixer.params["sinks"] == 2 for l in t.to_spec().layers)
    assert config_from_dict(t.to_dict()) == t                  # the folder of such a model keeps both
    assert c.with_window(16).attention_sinks == 0 and c.with_window(16, 3).attention_sinks == 3
    for n in (1, 2, 3):
        with pytest.raises(ConfigError, match="sinks"):
            c.with_context(n)
    with pytest.raises(ConfigError, match="attention_sinks"):
        config_from_dict(dict(tiny_configs.TINY_LLAMA, attention_sinks=2))        # sinks without a window
    s = config_from_dict(tiny_configs.TINY_SINKS)
    assert (s.sliding_window, s.attention_sinks, s.rotary_dim) == (37, 3, 24)


def test_the_activation_comes_from_the_configuration():
    """hidden_act (silu or gelu, convert.py:51-52) reaches the feed-forward part as a parameter."""
    for act in ("silu", "gelu"):
        spec = config_from_dict(dict(tiny_configs.TINY_LLAMA, hidden_act=act)).to_spec()
        assert all(layer.part("feed_forward").params["activation"] == act for layer in spec.layers)
    assert config_from_dict(tiny_configs.TINY_WIDE_HEADS).hidden_act == "gelu"


@pytest.mark.parametrize("change,text", [
    ({"architectures": ["GPT2LMHeadModel"]}, "not supported"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_act": "relu"}, "hidden_act"),
    ({"attention_bias": True}, "bias"),
    ({"head_dim": 15}, "even"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_scaling"),
    ({"hidden_size": None}, "hidden_size"),
    ({"partial_rotary_factor": 0.2}, "rotary"),
])
def test_config_errors(change, text):
    with pytest.raises(ConfigError, match=text):
        config_from_dict(dict(tiny_configs.TINY_LLAMA, **change))


def test_unknown_architecture_lists_the_registered_ones():
    with pytest.raises(ConfigError) as e:
        config_from_dict({"architectures": ["Nope"]})
    assert "LlamaForCausalLM" in str(e.value) and "MistralForCausalLM" in str(e.value)


def test_registry_takes_another_architecture():
    class Other:
        @classmethod
        def from_dict(cls, d):
            return "made"
    register_architecture("OtherForCausalLM", Other)
    try:
        assert "OtherForCausalLM" in registered_architectures()
        assert config_from_dict({"architectures": ["OtherForCausalLM"]}) == "made"
        with pytest.raises(ValueError):
            register_architecture("OtherForCausalLM", LlamaConfig)
    finally:
        unregister_architecture("OtherForCausalLM")


def test_spec_is_data_layer_by_layer():
    spec = config_from_dict(tiny_configs.TINY_MISTRAL).to_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    m = spec.layers[1].mixer
    assert m.kind == "gqa_attention" and m.params["window"] == 16 and m.params["position"].kind == "rope"
    assert spec.layers[2].feed_forward.params == {"hidden": 256, "activation": "silu"}
    # the order of the layers is data: a layer twice, a layer that reads another's cache
    s2 = ModelSpec(spec.architecture, spec.dim, spec.vocab_size, spec.max_positions, spec.embedding, spec.layers,
                   spec.final_norm, spec.head,
                   schedule=[ScheduleEntry(0, 0), ScheduleEntry(0, 1), ScheduleEntry(2, 0, writes_cache=False)])
    assert len(s2.schedule) == 3
    with pytest.raises(ValueError, match="written by"):
        ModelSpec(spec.architecture, spec.dim, spec.vocab_size, spec.max_positions, spec.embedding, spec.layers,
                  spec.final_norm, spec.head, schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 0)])
    with pytest.raises(ValueError, match="before any"):
        ModelSpec(spec.architecture, spec.dim, spec.vocab_size, spec.max_positions, spec.embedding, spec.layers,
                  spec.final_norm, spec.head, schedule=[ScheduleEntry(0, 1, writes_cache=False)])


def test_a_layer_names_its_members_and_parts_that_follow_from_their_spec_are_shared():
    from yalm_amd.config import LayerSpec, PartSpec
    from yalm_amd.engine.model import Model
    norm = PartSpec("rmsnorm", {"eps": 1e-5}, prefix="n.")
    ff = PartSpec("swiglu", {"hidden": 32}, prefix="ff.")
    layer = LayerSpec("some_block", {"norm": norm}, prefix="l.", feed_forward=ff)
    assert layer.norm is norm and layer.part("feed_forward") is ff and layer.part("mixer") is None
    assert sorted(layer.parts) == ["feed_forward", "norm"] and layer.prefix == "l." and layer.block == "some_block"
    with pytest.raises(AttributeError, match="no member 'mixer'"):
        layer.mixer
    with pytest.raises(AttributeError):
        layer.block = "other"
    with pytest.raises(TypeError, match="PartSpec"):
        LayerSpec("some_block", mixer="attention")
    assert layer == LayerSpec("some_block", prefix="l.", norm=norm, feed_forward=ff)
    # the reference's block keeps its four names
    spec = config_from_dict(tiny_configs.TINY_MISTRAL).to_spec()
    assert sorted(spec.layers[0].parts) == ["feed_forward", "feed_forward_norm", "mixer", "mixer_norm"]
    # one position part for the layers that name the same spec; parts with tensors stay one each
    model = Model(spec)
    positions = {id(b.mixer.position) for b in model.blocks}
    assert len(positions) == 1 and len({id(b.mixer_norm) for b in model.blocks}) == 3
    assert sum(1 for p in model.all_parts() if p is model.blocks[0].mixer.position) == 1
    other = Model(spec)                                    # another model has its own
    assert other.blocks[0].mixer.position is not model.blocks[0].mixer.position
    assert [m.name for m in model.prompt_tables()] == ["kv_tiles"]
    tables = model.prompt_tables()[0]([130, 1, 64])
    assert list(tables["seq_tile0"]) == [0, 3, 4, 5] and tables["n_tiles"] == 5 and sorted(tables["tile_order"]) == [0, 2, 3, 4]


# ------------------------------------------------------------------ weights

def test_random_model_folder_round_trip(tmp_path):
    from plain import reference_model as R
    folder = write_random_model(str(tmp_path / "m"), tiny_configs.TINY_MISTRAL, seed=4)
    cfg, w = R.read_folder(folder)                     # the plain reader, not the package's
    assert cfg["sliding_window"] == 16 and "lm_head.weight" in w
    src = TensorSource(folder)
    for name, t in w.items():
        assert torch.equal(src.get(name), t)
    # distributions: embeddings N(0,1), linear U(+-1/sqrt(in)), norms 1 + U(+-0.1)
    e = w["model.embed_tokens.weight"]
    assert abs(e.mean()) < 0.02 and abs(e.std() - 1) < 0.02
    q = w["model.layers.1.self_attn.q_proj.weight"]
    assert q.abs().max() <= 1 / 96 ** 0.5 and q.abs().max() > 0.99 / 96 ** 0.5 and abs(q.mean()) < 0.005
    d = w["model.layers.0.mlp.down_proj.weight"]
    assert d.abs().max() <= 1 / 256 ** 0.5
    n = w["model.layers.2.input_layernorm.weight"]
    assert n.min() >= 0.9 and n.max() <= 1.1 and n.std() > 0.03
    # a function of (seed, name, index) alone
    again = write_random_model(str(tmp_path / "m2"), tiny_configs.TINY_MISTRAL, seed=4)
    assert all(torch.equal(R.read_folder(again)[1][k], v) for k, v in w.items())
    other = write_random_model(str(tmp_path / "m3"), tiny_configs.TINY_MISTRAL, seed=5)
    assert not torch.equal(R.read_folder(other)[1]["model.norm.weight"], w["model.norm.weight"])
    a = random_values("x", (1000,), "linear", 16, 1)
    assert torch.equal(random_values("x", (1000,), "linear", 16, 1)[10:20], a[10:20])
    # tied: no head in the folder
    tied = write_random_model(str(tmp_path / "t"), tiny_configs.TINY_LLAMA, seed=4, dtype=torch.bfloat16)
    _, wt = R.read_folder(tied)
    assert "lm_head.weight" not in wt and wt["model.norm.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    from yalm_amd.engine.model import Model
    folder = write_random_model(str(tmp_path / "m"), tiny_configs.TINY_LLAMA, seed=1)
    src = TensorSource(folder)
    t = {n: src.get(n).clone() for n in src.names()}
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    t["model.layers.7.extra.weight"] = torch.zeros(3)
    t["model.layers.0.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    write_file(os.path.join(bad, "model.safetensors"), t)
    with open(os.path.join(bad, "config.json"), "w") as f:
        json.dump(tiny_configs.TINY_LLAMA, f)
    with pytest.raises(WeightsError) as e:
        Model.from_folder(bad, dtype=torch.float32, device="cpu")
    msg = str(e.value)
    assert "missing (2)" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected (1)" in msg and "model.layers.7.extra.weight" in msg
    assert "model.layers.0.self_attn.k_proj.weight: expected [32, 64], found [16, 64]" in msg
    assert "input_layernorm.weight: expected a floating-point tensor" in msg


def test_tensors_the_model_does_not_use_are_passed_over(tmp_path, capsys):
    """What convert.py:127-207 does with a real folder's extras: rotary_emb.inv_freq buffers of older
    exports and an lm_head.weight stored next to a tied embedding are read past, not refused."""
    from yalm_amd.engine.model import Model
    folder = write_random_model(str(tmp_path / "m"), tiny_configs.TINY_LLAMA, seed=1)          # tied
    src = TensorSource(folder)
    t = {n: src.get(n).clone() for n in src.names()}
    assert "lm_head.weight" not in t
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    for l in range(tiny_configs.TINY_LLAMA["num_hidden_layers"]):
        t["model.layers.%d.self_attn.rotary_emb.inv_freq" % l] = torch.ones(8)
    extra = str(tmp_path / "extra")
    os.makedirs(extra)
    write_file(os.path.join(extra, "model.safetensors"), t)
    with open(os.path.join(extra, "config.json"), "w") as f:
        json.dump(tiny_configs.TINY_LLAMA, f)
    model = Model.from_folder(extra, dtype=torch.float32, device="cpu")
    assert model.head.weight is model.embedding.table
    warned = capsys.readouterr().err
    assert "3 tensors" in warned and "lm_head.weight" in warned and "rotary_emb.inv_freq" in warned
    with pytest.raises(WeightsError) as e:
        Model.from_folder(extra, dtype=torch.float32, device="cpu", strict=True)
    assert "unexpected (3)" in str(e.value) and "missing" not in str(e.value)


def test_container_errors(tmp_path):
    def write(header, data=b"", name="x.safetensors"):
        blob = json.dumps(header).encode()
        p = str(tmp_path / name)
        with open(p, "wb") as f:
            f.write(struct.pack("<Q", len(blob)) + blob + data)
        return p

    ok = {"a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 16]}}
    assert SafetensorsFile(write(ok, b"\0" * 16)).tensor("a").shape == (2, 2)
    for header, data, text in [
        ({"a": {"dtype": "F8_E5M2", "shape": [1], "data_offsets": [0, 1]}}, b"\0", "dtype"),
        ({"a": {"dtype": "F32", "shape": [1, 1, 1, 1, 1], "data_offsets": [0, 4]}}, b"\0" * 4, "at most 4"),
        ({"a": {"dtype": "F32", "shape": [1.5], "data_offsets": [0, 4]}}, b"\0" * 4, "integer"),
        ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0]}}, b"\0" * 4, "two integers"),
        ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [4, 0]}}, b"\0" * 4, "inside"),
        ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 8]}}, b"\0" * 4, "inside"),
        ({"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8, "need 12 bytes"),
    ]:
        with pytest.raises(SafetensorsError, match=text):
            SafetensorsFile(write(header, data))
    p = str(tmp_path / "short.safetensors")
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40))
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    # the same tensor in two files of a folder
    d = tmp_path / "dup"
    d.mkdir()
    write_file(str(d / "a.safetensors"), {"w": torch.zeros(2)})
    write_file(str(d / "b.safetensors"), {"w": torch.zeros(2)})
    with pytest.raises(WeightsError, match="occurs in both"):
        TensorSource(str(d))
    e = tmp_path / "empty"
    e.mkdir()
    with pytest.raises(WeightsError, match="no .safetensors"):
        TensorSource(str(e))


def test_shards_and_dtypes(tmp_path):
    d = tmp_path / "sh"
    d.mkdir()
    a = torch.arange(6, dtype=torch.float32).reshape(2, 3)
    write_file(str(d / "model-00001.safetensors"), {"a": a.to(torch.bfloat16), "i": torch.arange(4, dtype=torch.int64)})
    write_file(str(d / "model-00002.safetensors"), {"b": a.to(torch.float16), "c": a})
    src = TensorSource(str(d))
    assert src.get("a").dtype == torch.bfloat16 and torch.equal(src.get("a").float(), a)
    assert src.get("b").dtype == torch.float16 and torch.equal(src.get("c"), a)
    assert src.get("i").tolist() == [0, 1, 2, 3]
    # precision on the device: matrices in bfloat16, 32-bit vectors stay, integer tables int32
    bf, f32 = torch.bfloat16, torch.float32
    assert device_dtype(f32, 2, bf) == bf and device_dtype(bf, 2, bf) == bf and device_dtype(torch.float16, 2, bf) == bf
    assert device_dtype(f32, 1, bf) == f32 and device_dtype(bf, 1, bf) == bf
    assert device_dtype(bf, 2, f32) == f32 and device_dtype(bf, 1, f32) == f32
    assert device_dtype(torch.int64, 1, bf) == torch.int32


# ------------------------------------------------------------------ the cache

def test_slots_and_pages_are_never_lost_or_doubled():
    s = SlotAllocator(3)
    a, b, c = s.acquire(), s.acquire(), s.acquire()
    assert sorted([a, b, c]) == [0, 1, 2]
    with pytest.raises(CacheFull):
        s.acquire()
    s.release(b)
    with pytest.raises(CacheError):
        s.release(b)                                  # freed twice
    assert s.acquire() == b                           # used again
    with pytest.raises(CacheError):
        s.release(17)
    p = PagePool(2)
    x, y = p.take(), p.take()
    assert x != y
    with pytest.raises(CacheFull):
        p.take()
    p.give_back(x)
    with pytest.raises(CacheError):
        p.give_back(x)


def make_cache(max_tokens=64 * 10, n_slots=4, max_seq_len=64 * 8):
    reqs = {0: KVRequest(2, 16, 0), 1: KVRequest(2, 16, 0), 2: KVRequest(2, 16, 100), 3: StateRequest((5,)), 4: None}
    return CacheManager(reqs, max_tokens, max_seq_len, torch.float32, "cpu", n_slots=n_slots)


def test_cache_groups_and_page_accounting():
    c = make_cache()
    assert len(c.kv_groups) == 2 and len(c.state_groups) == 1
    full = c.group_of(0)
    ring = c.group_of(2)
    assert c.group_of(1) is full and full.lines == [0, 1] and ring.lines == [2]
    assert full.ring_pages == 8 and ring.ring_pages == 3            # ceil(100/64) + 1
    assert full.k_pages.shape == (2, 10, 2, 64, 16) and full.v_pages.shape == (2, 10, 2, 16, 64)
    assert full.sinks == 0 and full.sink_k is None and ring.sinks == 0
    # lines that keep sinks beside the window are a group of their own, with a place for them per slot
    reqs = {0: KVRequest(2, 16, 100), 1: KVRequest(2, 16, 100, 3), 2: KVRequest(2, 16, 100, 3)}
    s = CacheManager(reqs, 640, 512, torch.float32, "cpu", n_slots=4)
    assert len(s.kv_groups) == 2 and s.group_of(1) is s.group_of(2) and s.group_of(0).sinks == 0
    k, v = s.group_of(2).line_sinks(2)
    assert k.shape == v.shape == (4, 2, 3, 16) and k.is_contiguous() and s.group_of(1).ring_pages == 3
    s = c.acquire(2)
    assert c.extend(s, [70, 1]) == [70, 1]
    assert full.pool.n_free == 10 - 3 and ring.pool.n_free == 10 - 3
    assert (full.table_host[s[0], :2] >= 0).all() and full.table_host[s[0], 2] == -1
    assert torch.equal(full.table.cpu(), torch.from_numpy(full.table_host))
    # growth inside a page takes nothing; crossing takes one; the ring stops at its size
    c.extend(s, [58, 63])
    assert full.pool.n_free == 7 and c.seq_len[s[0]] == 128 and c.seq_len[s[1]] == 64
    c.extend(s, [1, 1])
    assert full.pool.n_free == 5 and ring.pool.n_free == 5
    c.extend([s[0]], [64 * 3])
    assert full.pool.n_free == 2 and ring.pool.n_free == 5           # the ring of slot 0 is complete (3 pages)
    # too much: nothing changes
    before = (full.pool.n_free, ring.pool.n_free, list(c.seq_len))
    with pytest.raises(CacheFull):
        c.extend(s, [64 * 2, 64 * 2])
    assert before == (full.pool.n_free, ring.pool.n_free, list(c.seq_len))
    with pytest.raises(CacheFull):
        c.extend([s[0]], [64 * 8])                                   # beyond the longest sequence
    c.release([s[0]])
    assert full.pool.n_free == 8 and c.seq_len[s[0]] == 0 and (full.table_host[s[0]] == -1).all()
    with pytest.raises(CacheError):
        c.release([s[0]])
    with pytest.raises(CacheError):
        c.extend([s[0]], [1])                                        # not held
    c.release([s[1]])
    assert full.pool.n_free == 10 and ring.pool.n_free == 10 and c.slots.n_free == 4
    assert c.tokens_held() == 0


def test_a_batch_takes_its_pages_in_turn():
    """Sequences that start together take their pages a page each in turn: page p of all of them lies
    together, not every sequence's pages in a run of its own."""
    c = make_cache()
    full = c.group_of(0)
    s = c.acquire(3)
    c.extend(s, [130, 64, 70])                                       # 3, 1 and 2 pages
    t = full.table_host
    assert [int(t[x, 0]) for x in s] == [0, 1, 2]
    assert [int(t[s[0], 1]), int(t[s[2], 1])] == [3, 4] and int(t[s[1], 1]) == -1
    assert int(t[s[0], 2]) == 5 and full.pool.n_free == 10 - 6
    c.extend(s, [1, 1, 58])                                          # only the second crosses into a new page
    assert int(t[s[1], 1]) == 6 and int(t[s[2], 2]) == -1
    c.release(s)
    assert full.pool.n_free == 10


def test_cache_state_is_cleared_on_acquire_and_random_use_keeps_the_books():
    c = make_cache(max_tokens=64 * 40, n_slots=6)
    st = c.state_groups[0]
    assert st.data.shape == (1, 6, 5)
    s = c.acquire(1)
    st.line_state(3)[s[0]] = 7.0
    c.release(s)
    s2 = c.acquire(1)
    assert s2 == s and (st.line_state(3)[s2[0]] == 0).all()
    c.release(s2)
    rng = np.random.default_rng(0)
    live = {}
    for _ in range(300):
        if live and rng.random() < 0.3:
            slot = list(live)[rng.integers(len(live))]
            c.release([slot])
            del live[slot]
        elif c.slots.n_free and rng.random() < 0.5:
            slot = c.acquire(1)[0]
            assert slot not in live
            live[slot] = 0
        elif live:
            slot = list(live)[rng.integers(len(live))]
            n = int(rng.integers(1, 100))
            try:
                c.extend([slot], [n])
                live[slot] += n
            except CacheFull:
                pass
        for g in c.kv_groups:
            held = [int(p) for slot in live for p in g.table_host[slot] if p >= 0]
            assert len(held) == len(set(held)) == g.n_pages - g.pool.n_free        # no page twice, none lost
            for slot, n in live.items():
                assert (g.table_host[slot] >= 0).sum() == min((n + 63) // 64, g.ring_pages)
    c.release(list(live))
    assert all(g.pool.n_free == g.n_pages for g in c.kv_groups)


# ------------------------------------------------------------------ generation loop

class ScriptedEngine:
    """Stands in for the engine: logits say 'next token = (last token + 1) % V'."""

    class _Spec:
        eos_token_ids = [9]

    class _Model:
        pass

    def __init__(self, vocab=12, n_slots=3, n_pages=64, n_positions=40):
        self.V = vocab
        self.model = self._Model()
        self.model.spec = self._Spec()
        self.cache = type("C", (), {"n_pages": n_pages, "n_slots": n_slots})()
        self.n_positions = n_positions
        self.free = list(range(n_slots))
        self.lens = {}
        self.log = []

    def start(self, n):
        out = [self.free.pop(0) for _ in range(n)]
        for s in out:
            assert s not in self.lens
            self.lens[s] = 0
        return out

    def release(self, slots):
        for s in slots:
            del self.lens[s]
            self.free.append(s)

    def step(self, slots, tokens, want=None):
        self.log.append((list(slots), [len(t) for t in tokens]))
        logits = torch.zeros(len(slots), self.V)
        for r, (s, t) in enumerate(zip(slots, tokens)):
            assert (self.lens[s] == 0) or len(t) == 1
            self.lens[s] += len(t)
            assert self.lens[s] <= self.n_positions
            logits[r, (t[-1] + 1) % self.V] = 5.0
        return logits


class ArgmaxSampler:
    def sample(self, logits, temperature, request_ids, steps):
        self.last = (list(request_ids), list(steps))
        return logits.argmax(dim=1).tolist()


def test_generation_loop_decisions():
    e = ScriptedEngine()
    prompts = [[1, 2, 3], [7], [4, 5], [0], [8]]
    out = generate(e, prompts, max_new_tokens=4, sampler=ArgmaxSampler(), batch_size=3)
    # stop token 9 is kept and ends its request; others stop at 4 new tokens
    assert out == [[4, 5, 6, 7], [8, 9], [6, 7, 8, 9], [1, 2, 3, 4], [9]]
    # first batch: 3 prompts whole, then one token each, the one that stopped leaves at once
    assert e.log[0] == ([0, 1, 2], [3, 1, 2])
    assert e.log[1] == ([0, 1, 2], [1, 1, 1])
    assert e.log[2] == ([0, 2], [1, 1]) and e.log[3] == ([0, 2], [1, 1])
    # second batch reuses the slots that were given back
    assert e.log[4][1] == [1, 1] and set(e.log[4][0]) <= {0, 1, 2}
    assert not e.lens and sorted(e.free) == [0, 1, 2]
    # no stop tokens at all; the context ends a request (prompt + new = n_positions)
    e2 = ScriptedEngine(n_positions=6)
    out = generate(e2, [[1, 2, 3]], max_new_tokens=50, sampler=ArgmaxSampler(), stop_ids=[])
    assert out == [[4, 5, 6]] and not e2.lens
    assert generate(e2, [[1]], max_new_tokens=0, sampler=ArgmaxSampler()) == [[]]


class ScriptedAheadEngine(ScriptedEngine):
    """Takes a step's tokens from the tensor of the draw before, as the engine's step_from does."""

    def step_from(self, slots, source, rows=None):
        rows = list(range(len(slots))) if rows is None else list(rows)
        assert len(rows) == len(slots) and all(self.lens[s] > 0 for s in slots)
        return self.step(slots, [[int(source[r])] for r in rows])


class DrawingSampler(ArgmaxSampler):
    """draw() as the sampler's: the tokens as a tensor at once, as a list on demand."""

    class _Drawn:
        def __init__(self, tokens, reads):
            self.tokens, self._reads = tokens, reads

        def tolist(self):
            self._reads.append(len(self.tokens))
            return self.tokens.tolist()

    def __init__(self):
        self.reads = []
        self.draws = []

    def draw(self, logits, temperature, request_ids, steps):
        self.draws.append((list(request_ids), list(steps)))
        return self._Drawn(logits.argmax(dim=1).to(torch.int32), self.reads)


def test_generation_loop_a_step_ahead():
    """The same tokens as the loop that reads every token first; a stop token is seen one step
    late (its sequence is in one more step), an end by count is known beforehand."""
    prompts = [[1, 2, 3], [7], [4, 5], [0], [8]]
    e = ScriptedAheadEngine()
    sampler = DrawingSampler()
    out = generate(e, prompts, max_new_tokens=4, sampler=sampler, batch_size=3)
    assert out == [[4, 5, 6, 7], [8, 9], [6, 7, 8, 9], [1, 2, 3, 4], [9]]
    assert e.log[0] == ([0, 1, 2], [3, 1, 2])
    assert e.log[1] == ([0, 1, 2], [1, 1, 1])
    assert e.log[2] == ([0, 1, 2], [1, 1, 1])            # the 9 of request 1 is read while this step runs
    assert e.log[3] == ([0, 2], [1, 1])
    assert e.log[4][1] == [1, 1] and len(e.log) == 8     # no step for a fourth token's successor
    assert not e.lens and sorted(e.free) == [0, 1, 2]
    # every draw is read once, after the step behind it was queued; the draw numbers count a request's tokens
    assert sampler.reads == [3, 3, 3, 2, 2, 2, 1, 1]
    assert sampler.draws[:4] == [([0, 1, 2], [0, 0, 0]), ([0, 1, 2], [1, 1, 1]), ([0, 1, 2], [2, 2, 2]), ([0, 2], [3, 3])]
    behind = generate(ScriptedAheadEngine(), prompts, max_new_tokens=4, sampler=DrawingSampler(), batch_size=3,
                      ahead=False)
    assert behind == out
    # the context ends a request by its count: no step beyond the last position
    e2 = ScriptedAheadEngine(n_positions=6)
    assert generate(e2, [[1, 2, 3]], max_new_tokens=50, sampler=DrawingSampler(), stop_ids=[]) == [[4, 5, 6]]
    assert not e2.lens and [n for _, n in e2.log] == [[3], [1], [1]]
    with pytest.raises(ValueError, match="step_from"):
        generate(ScriptedEngine(), prompts, max_new_tokens=4, sampler=DrawingSampler(), ahead=True)
    # a callback sees the tokens in the same order
    seen_a, seen_b = [], []
    generate(ScriptedAheadEngine(), prompts, max_new_tokens=4, sampler=DrawingSampler(), batch_size=3,
             on_token=lambda i, t: seen_a.append((i, t)))
    generate(ScriptedEngine(), prompts, max_new_tokens=4, sampler=ArgmaxSampler(), batch_size=3,
             on_token=lambda i, t: seen_b.append((i, t)))
    assert seen_a == seen_b


def test_the_prompt_clock_covers_the_prompt_step_when_the_loop_runs_ahead():
    """A draw does not wait for the device; the prompt step is over only when its tokens have landed.
    Here every landing takes 30 ms: the prompt's share of it must be in prefill_seconds, not in decode_seconds."""
    import time
    from yalm_amd.generate import GenerationStats

    class SlowLanding(DrawingSampler):
        class _Drawn(DrawingSampler._Drawn):
            def tolist(self):
                time.sleep(0.03)
                return super().tolist()

    stats = GenerationStats()
    out = generate(ScriptedAheadEngine(), [[1, 2, 3]], max_new_tokens=3, sampler=SlowLanding(), stats=stats, stop_ids=[])
    assert out == [[4, 5, 6]]
    assert stats.prefill_seconds >= 0.03
    assert stats.decode_seconds >= 0.06                      # the two later draws


@pytest.mark.parametrize("base, sampler", [(ScriptedEngine, ArgmaxSampler), (ScriptedAheadEngine, DrawingSampler)])
def test_a_failed_step_gives_the_slots_back(base, sampler):
    class Failing(base):
        def step(self, slots, tokens, want=None):
            if len(self.log) == 3:
                raise RuntimeError("step failed")
            return super().step(slots, tokens, want)
    eng = Failing()
    with pytest.raises(RuntimeError, match="step failed"):
        generate(eng, [[1], [7, 8], [3]], max_new_tokens=6, sampler=sampler())
    assert sorted(eng.free) == [0, 1, 2] and not eng.lens          # also the one that had ended before


def test_plan_batches():
    assert plan_batches([5, 17, 1, 300, 64], 8, 2, 1024, 8, 512) == [[0, 1], [2, 3], [4]]
    # the cache bounds a batch: 3 requests of 100 + 28 tokens = 2 pages each, 4 pages in all
    assert plan_batches([100, 100, 100], 28, None, 256, 8, 512) == [[0, 1], [2]]
    with pytest.raises(ValueError, match="context"):
        plan_batches([600], 8, None, 4096, 8, 512)
    with pytest.raises(ValueError, match="empty"):
        plan_batches([0], 8, None, 4096, 8, 512)
    with pytest.raises(ValueError, match="cache"):
        plan_batches([200], 8, None, 128, 8, 512)


def test_sampler_numbers_depend_on_seed_request_and_step_only():
    from yalm_amd.sampling import uniform
    u = [uniform(3, r, s) for r in range(50) for s in range(50)]
    assert all(0 <= x < 1 for x in u) and len(set(u)) > 2400
    assert abs(np.mean(u) - 0.5) < 0.02
    assert uniform(3, 7, 2) == uniform(3, 7, 2) != uniform(4, 7, 2)
    assert uniform(3, 7, 2) != uniform(3, 2, 7)


def test_tokenizer(tmp_path):
    from yalm_amd.tokenizer import Tokenizer
    vocab = {"<unk>": 0, "<s>": 1, "</s>": 2}
    for i in range(256):
        vocab["<0x%02X>" % i] = 3 + i
    for i, t in enumerate(["▁hello", "▁wor", "ld", "▁", "he", "▁w"]):
        vocab[t] = 259 + i
    with open(tmp_path / "tokenizer.json", "w") as f:
        json.dump({"model": {"vocab": vocab, "byte_fallback": True},
                   "added_tokens": [{"id": 265, "content": "<|eot_id|>"}]}, f)
    t = Tokenizer.from_folder(str(tmp_path), 266, 1, 2)
    assert t.eot_id == 265 and t.byte_fallback_start == 3
    e = t.encode(" hello world!", True)
    assert e == [1, 259, 260, 261, 3 + ord("!")]                   # longest match, byte fallback
    text = b"".join(t.decode_one(p, q) for p, q in zip(e[:-1], e[1:]))
    assert text == b"hello world!"                                 # the space after BOS is dropped
    assert t.encode("hé", False) == [3 + ord("h"), 3 + 0xC3, 3 + 0xA9]     # "he" does not match
    assert t.encode("he", False) == [263]


def test_command_line_options_have_the_references_meanings():
    """src/main.cpp:334-467: every option takes a value, -m and -d match by prefix,
    -n sets the step count and the number of junk lines, one prompt source only."""
    from yalm_amd.cli import parse_args
    a = parse_args(["folder", "-m", "c", "-i", "hello", "-n", "12", "-t", "0.5", "-T", "64"])
    assert (a["checkpoint"], a["mode"], a["prompt"], a["num_steps"], a["n_junk"], a["temperature"], a["context"]) == \
        ("folder", "completion", "hello", 12, 12, 0.5, 64)
    d = parse_args(["folder", "--tokens", "1,2"])
    assert (d["mode"], d["num_steps"], d["n_junk"], d["temperature"], d["passkey_pos"], d["device"]) == \
        ("completion", 256, 250, 1.0, -1, "hip")
    assert parse_args(["folder", "-m", "perp", "-f", "x.txt"])["mode"] == "perplexity"
    assert parse_args(["folder", "-m", "pass", "-n", "10", "-l", "9"])["passkey_pos"] == 9
    r = parse_args(["--random", "cfg.json", "--weight-seed", "3", "--tokens", "1 2 3", "-d", "cuda"])
    assert (r["checkpoint"], r["random"], r["weight_seed"], r["device"]) == ("", "cfg.json", 3, "cuda")
    for bad in (["folder"],                                            # no prompt
                ["folder", "-i", "a", "-f", "b"],                      # two prompts
                ["folder", "-m", "x", "-i", "a"],                      # unknown mode
                ["folder", "-d", "cpu", "-i", "a"],                    # no CPU path
                ["folder", "-i"],                                      # option without value
                ["folder", "-z", "1", "-i", "a"],                      # unknown option
                ["folder", "-m", "pass", "-n", "10", "-l", "10"],      # passkey line out of range (main.cpp:455-458)
                ["folder", "--random", "cfg.json", "-i", "a"],         # folder and --random
                ["folder", "--dtype", "float16", "-i", "a"],
                []):
        with pytest.raises(SystemExit) as e:
            parse_args(bad)
        assert e.value.code == 1


def test_prefill_tile_order_names_every_second_tile_once_the_longest_first():
    from yalm_amd.ops import kernels
    PAGE = kernels.PAGE

    def check(lens):
        order = kernels.prefill_tile_order(lens)
        assert order.dtype == np.int32
        tiles = [(n + PAGE - 1) // PAGE for n in lens]
        first = np.concatenate([[0], np.cumsum(tiles)])
        want = sorted(int(first[b]) + t for b, n in enumerate(tiles) for t in range(0, n, 2))
        assert sorted(order.tolist()) == want
        seqs = [int(np.searchsorted(first, g, side="right")) - 1 for g in order.tolist()]
        work = [min(g - int(first[b]) + 2, tiles[b]) for g, b in zip(order.tolist(), seqs)]
        return seqs, work, tiles

    seqs, work, tiles = check([130, 1, 64, 700, 65])              # short: by the keys a tile sees
    assert work == sorted(work, reverse=True)
    seqs, work, tiles = check([130, 1, 3000, 64, 2500, 65])        # long: sequence by sequence
    runs = [b for i, b in enumerate(seqs) if i == 0 or seqs[i - 1] != b]
    assert len(runs) == len(set(runs)) and [tiles[b] for b in runs] == sorted(tiles, reverse=True)
    for b in runs:
        w = [x for x, s in zip(work, seqs) if s == b]
        assert w == sorted(w, reverse=True)


def test_a_library_built_from_other_sources_is_built_again(tmp_path, monkeypatch):
    """The digest of the kernel sources is kept beside the built library; a library whose digest is another
    (or that has none) is not loaded but built again."""
    from yalm_amd.csrc import build

    class Reached(Exception):
        pass

    def no_compiler():
        raise Reached()
    lib = tmp_path / build.LIB_NAME
    lib.write_bytes(b"not a library")
    monkeypatch.setattr(build, "_candidates", lambda: [str(lib)])
    monkeypatch.setattr(build, "_hipcc", no_compiler)
    with pytest.raises(Reached):                          # no digest beside it: stale
        build.build(force=False)
    (tmp_path / (build.LIB_NAME + ".sources")).write_text("0" * 64 + "\n")
    with pytest.raises(Reached):                          # another digest: stale
        build.build(force=False)
    (tmp_path / (build.LIB_NAME + ".sources")).write_text(build.sources_digest() + "\n")
    assert build.build(force=False) == str(lib)           # built from these sources: taken as it is
    with pytest.raises(Reached):
        build.build(force=True)
    assert len(build.sources_digest()) == 64


def test_decode_metadata_orders_a_ragged_batch_by_length():
    """The step's metadata: tokens, rows, positions, slots, lengths, offsets, then the longest length and an order
    of the rows, which is a permutation whatever the lengths are: the longest rows first, the second half from the
    shortest up, padding rows in the middle."""
    import numpy as np
    from yalm_amd.engine.engine import Engine
    Bk = 8
    host = np.full(7 * Bk + 2, -7, dtype=np.int32)
    lens = [900, 30, 410, 64, 700]
    Engine._fill_decode_meta(host, Bk, [5, 6, 7, 8, 9], [n - 1 for n in lens], [3, 0, 4, 1, 2], lens, ragged=True)
    assert list(host[0:Bk]) == [5, 6, 7, 8, 9, -1, -1, -1] and list(host[3 * Bk:4 * Bk]) == [3, 0, 4, 1, 2, -1, -1, -1]
    assert list(host[4 * Bk:5 * Bk]) == lens + [0, 0, 0] and host[6 * Bk + 1] == 900
    order = list(host[6 * Bk + 2:7 * Bk + 2])
    assert sorted(order) == list(range(Bk))
    assert order[:4] == [0, 4, 2, 3] and order[4:] == [7, 6, 5, 1]        # 900, 700, 410, 64 | padding ..., then 30
    Engine._fill_decode_meta(host, Bk, [5, 6, 7, 8, 9], [n - 1 for n in lens], [3, 0, 4, 1, 2], lens)
    assert list(host[6 * Bk + 2:7 * Bk + 2]) == list(range(Bk))
    Engine._fill_decode_meta(host, Bk, [], [], [], [], ragged=True)        # a capture's rows of padding
    assert host[6 * Bk + 1] == 0 and list(host[6 * Bk + 2:]) == list(range(Bk))
    assert Engine._is_ragged(lens) and not Engine._is_ragged([900, 880]) and not Engine._is_ragged([100, 20, 60])
    for trial in range(50):
        rng = np.random.default_rng(trial)
        B = int(rng.integers(1, Bk + 1))
        ls = [int(x) for x in rng.integers(1, 5000, size=B)]
        Engine._fill_decode_meta(host, Bk, [0] * B, [n - 1 for n in ls], list(range(B)), ls, ragged=True)
        assert sorted(host[6 * Bk + 2:7 * Bk + 2]) == list(range(Bk))
