"""Each part of a layer alone against the plain implementation's function for it,
and the proof that parts are exchangeable: a toy mixer with state of its own
and a toy architecture, both defined here, are registered, built and stepped
without a change to the package's files."""
import math

import numpy as np
import pytest
import torch

import helpers
import schedules
from plain import reference_model as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_ctx(cache, lens, dtype, mode="prefill", starts=None):
    """A StepContext as Engine.step builds it, for parts driven by hand."""
    from yalm_amd.engine.context import StepContext, Workspace
    B = len(lens)
    if mode == "prefill":
        slots = cache.acquire(B)
        starts = [0] * B
    else:
        slots = starts[0]
        starts = starts[1]
    new_lens = cache.extend(slots, lens)
    ctx = StepContext(mode, cache, Workspace(DEV), dtype)
    i32 = lambda x: torch.tensor(np.asarray(x), dtype=torch.int32, device=DEV)
    ctx.tok_seq = i32(np.repeat(np.arange(B), lens))
    ctx.tok_pos = i32(np.concatenate([np.arange(s, s + n) for s, n in zip(starts, lens)]))
    ctx.seq_slot = i32(slots)
    ctx.seq_len = i32(new_lens)
    ctx.cu_seqlens = i32(np.concatenate([[0], np.cumsum(lens)]))
    tile0 = np.concatenate([[0], np.cumsum([(n + 63) // 64 for n in lens])])
    ctx.tables["kv_tiles"] = {"seq_tile0": i32(tile0), "n_tiles": int(tile0[-1])}
    ctx.max_position = max(new_lens) - 1
    ctx.host_slots, ctx.host_n_tokens, ctx.host_start = list(slots), list(lens), list(starts)
    return ctx, slots


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float64).float() * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from yalm_amd.config import PartSpec
    from yalm_amd.parts import build_part
    D = 72
    p = build_part("norm", PartSpec("rmsnorm", {"eps": 2e-4}, prefix="n."), D, "layer.")
    assert [s.name for s in p.param_specs()] == ["layer.n.weight"] and p.param_specs()[0].shape == (D,)
    w = 1 + 0.1 * rnd((D,), 1)
    p.load({"layer.n.weight": w}.__getitem__, dtype, DEV)
    assert p.weight.dtype == torch.float32            # a vector stored in 32-bit stays so
    x = rnd((5, D), 2, 4.0)
    out = torch.empty((5, D), dtype=dtype, device=DEV)
    p.forward(x.to(DEV), out, None)
    want = R.rmsnorm(x, w, 2e-4)
    lim = 1e-5 if dtype == torch.float32 else 1e-2
    assert (out.cpu().double() - want).abs().max() <= lim * want.abs().max()


def test_rope_part_table_and_row_order():
    from yalm_amd.config import PartSpec
    from yalm_amd.parts import build_part
    from yalm_amd.parts.rope import interleave_rows, inverse_frequencies
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 32}
    for hd, rd, theta, sc in [(16, 16, 1e4, None), (32, 32, 500.0, scaling), (48, 24, 1e6, None)]:
        p = build_part("position", PartSpec("rope", {"head_dim": hd, "rotary_dim": rd, "theta": theta, "scaling": sc,
                                                      "weight_rows": "half_split"}), 64, "")
        p.prepare(100, DEV)
        f = R.rope_inv_freq(hd, rd, theta)[: rd // 2]
        if sc:
            f = R.llama3_scaled_inv_freq(f, 8.0, 1.0, 4.0, 32)
        assert torch.allclose(inverse_frequencies(hd, rd, theta, sc), f, rtol=1e-14, atol=0)
        ang = torch.arange(100, dtype=torch.float64)[:, None] * f[None]
        assert p.table.shape == (100, rd // 2, 2)
        assert torch.allclose(p.table[..., 0].cpu().double(), torch.cos(ang), atol=1e-7)
        assert torch.allclose(p.table[..., 1].cpu().double(), torch.sin(ang), atol=1e-7)
        w = rnd((3 * hd, 10), 3)
        assert torch.equal(p.arrange_projection_rows(w, 3), R.hf_rows_to_interleaved(w, 3, rd))
        assert torch.equal(interleave_rows(w, 3, hd, rd), R.hf_rows_to_interleaved(w, 3, rd))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_heads,n_kv,hd,window,D", [(4, 2, 16, 0, 64), (3, 1, 32, 16, 80), (6, 6, 48, 0, 72)])
def test_attention_part_prefill_then_decode(n_heads, n_kv, hd, window, D, dtype):
    """The mixer alone: whole prompts of unequal lengths, then one more token each,
    against the plain rope + attention + projections."""
    from yalm_amd.cache import CacheManager
    from yalm_amd.config import PartSpec
    from yalm_amd.parts import build_part
    pos_spec = PartSpec("rope", {"head_dim": hd, "rotary_dim": hd, "theta": 1e4, "scaling": None,
                                 "weight_rows": "half_split"})
    spec = PartSpec("gqa_attention", {"n_heads": n_heads, "n_kv_heads": n_kv, "head_dim": hd, "window": window,
                                      "position": pos_spec}, prefix="attn.")
    part = build_part("mixer", spec, D, "l.")
    Q, KV = n_heads * hd, n_kv * hd
    names = {s.name: s.shape for s in part.param_specs()}
    assert names == {"l.attn.q_proj.weight": (Q, D), "l.attn.k_proj.weight": (KV, D),
                     "l.attn.v_proj.weight": (KV, D), "l.attn.o_proj.weight": (D, Q)}
    w = {n: rnd(s, 10 + i, 1 / math.sqrt(s[1])) for i, (n, s) in enumerate(sorted(names.items()))}
    if dtype == torch.bfloat16:
        w = {n: t.bfloat16().float() for n, t in w.items()}
    part.load(w.__getitem__, dtype, DEV)
    part.position.prepare(256, DEV)
    cache = CacheManager({0: part.cache_request()}, 64 * 16, 256, dtype, DEV, n_slots=4)
    lens = [70, 5, 33]
    T = sum(lens)
    h_all = [rnd((n + 1, D), 20 + i).to(dtype).float() for i, n in enumerate(lens)]     # one more token for decode

    def plain(h):
        n = h.shape[0]
        f = R.rope_inv_freq(hd, hd, 1e4)
        pos = torch.arange(n)
        q = (h.double() @ R.hf_rows_to_interleaved(w["l.attn.q_proj.weight"].double(), n_heads, hd).T)
        k = (h.double() @ R.hf_rows_to_interleaved(w["l.attn.k_proj.weight"].double(), n_kv, hd).T)
        v = h.double() @ w["l.attn.v_proj.weight"].double().T
        a = R.attention(R.rope_interleaved(q.reshape(n, n_heads, hd), pos, f),
                        R.rope_interleaved(k.reshape(n, n_kv, hd), pos, f), v.reshape(n, n_kv, hd), window)
        return a.reshape(n, Q) @ w["l.attn.o_proj.weight"].double().T

    want = [plain(h) for h in h_all]
    ctx, slots = make_ctx(cache, lens, dtype)
    h = torch.cat([x[:-1] for x in h_all]).to(DEV, dtype)
    x = torch.zeros((T, D), device=DEV)
    part.forward(h, x, ctx, 0, True)
    lim = 2e-5 if dtype == torch.float32 else 3e-2
    got = x.cpu().double()
    o = 0
    for i, n in enumerate(lens):
        assert (got[o:o + n] - want[i][:n]).abs().max() <= lim * max(1, want[i].abs().max()), ("prefill", i)
        o += n
    ctx, _ = make_ctx(cache, [1, 1, 1], dtype, "decode", (slots, lens))
    h = torch.stack([x[-1] for x in h_all]).to(DEV, dtype)
    x = torch.ones((3, D), device=DEV)                               # the mixer adds to the residual stream
    part.forward(h, x, ctx, 0, True)
    got = x.cpu().double() - 1
    for i in range(3):
        assert (got[i] - want[i][-1]).abs().max() <= lim * max(1, want[i].abs().max()), ("decode", i)


@pytest.mark.parametrize("act", ["silu", "gelu", None])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype, act):
    from yalm_amd.config import PartSpec
    from yalm_amd.engine.context import StepContext, Workspace
    from yalm_amd.parts import build_part
    D, H = 72, 200
    params = {"hidden": H} if act is None else {"hidden": H, "activation": act}      # silu unless said otherwise
    part = build_part("feed_forward", PartSpec("swiglu", params, prefix="mlp."), D, "l.")
    w = {"l.mlp.gate_proj.weight": rnd((H, D), 1, D ** -0.5), "l.mlp.up_proj.weight": rnd((H, D), 2, D ** -0.5),
         "l.mlp.down_proj.weight": rnd((D, H), 3, H ** -0.5)}
    if dtype == torch.bfloat16:
        w = {n: t.bfloat16().float() for n, t in w.items()}
    assert {s.name: s.shape for s in part.param_specs()} == {n: tuple(t.shape) for n, t in w.items()}
    part.load(w.__getitem__, dtype, DEV)
    h = rnd((9, D), 4).to(dtype)
    x0 = rnd((9, D), 5)
    x = x0.to(DEV).clone()
    part.forward(h.to(DEV), x, StepContext("prefill", None, Workspace(DEV), dtype))
    want = x0.double() + R.swiglu_ffn(h.float(), w["l.mlp.gate_proj.weight"], w["l.mlp.down_proj.weight"],
                                      w["l.mlp.up_proj.weight"], act or "silu")
    lim = 2e-5 if dtype == torch.float32 else 2e-2
    assert (x.cpu().double() - want).abs().max() <= lim * want.abs().max()


def test_embedding_and_tied_head():
    from yalm_amd.config import PartSpec
    from yalm_amd.parts import build_part
    V, D = 50, 24
    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": V}, prefix="emb."), D, "")
    head = build_part("head", PartSpec("lm_head", {"vocab_size": V, "tied": True}, prefix="head."), D, "",
                      embedding=emb)
    assert head.param_specs() == []
    table = rnd((V, D), 1)
    emb.load({"emb.weight": table}.__getitem__, torch.float32, DEV)
    head.load(None, torch.float32, DEV)
    assert head.weight.data_ptr() == emb.table.data_ptr()            # one copy on the device
    x = torch.empty((3, D), device=DEV)
    emb.forward(torch.tensor([4, 0, 49], dtype=torch.int32, device=DEV), x, None)
    assert torch.equal(x.cpu(), table[[4, 0, 49]])
    logits = torch.empty((3, V), device=DEV)
    head.forward(x, logits, None)
    assert torch.allclose(logits.cpu().double(), table[[4, 0, 49]].double() @ table.double().T, atol=1e-4)


# ---------------------------------------------------------------------------
# a toy mixer with state of its own, and a toy architecture that uses it
# ---------------------------------------------------------------------------

def toy_mixer_plain(h, w):
    """out[t] = W mean(h[0..t]) for one whole sequence, float64."""
    h = h.double()
    mean = torch.cumsum(h, 0) / torch.arange(1, h.shape[0] + 1, dtype=torch.float64)[:, None]
    return mean @ w.double().T


def define_toy_parts():
    from yalm_amd.cache import StateRequest
    from yalm_amd.parts import Part, register_part
    from yalm_amd.weights import ParamSpec

    class RunningMeanMixer(Part):
        """x += W * (mean of all inputs of the sequence so far).  Its state is the
        running sum, one vector per sequence, kept in the cache's state store."""
        graph_safe = False                    # its launches depend on host values

        def param_specs(self):
            return [ParamSpec(self.prefix + "w.weight", (self.dim, self.dim), fan_in=self.dim)]

        def load(self, get, compute_dtype, device):
            self.w = get(self.prefix + "w.weight").to(device, torch.float32)

        def cache_request(self):
            return StateRequest((self.dim,), torch.float32)

        def forward(self, h, x, ctx, line, writes_cache=True):
            state = ctx.cache.group_of(line).line_state(line)          # [n_slots, dim]
            o = 0
            for slot, n, start in zip(ctx.host_slots, ctx.host_n_tokens, ctx.host_start):
                hs = h[o:o + n].float()
                sums = state[slot][None, :] + torch.cumsum(hs, 0)
                counts = torch.arange(start + 1, start + n + 1, device=h.device, dtype=torch.float32)[:, None]
                x[o:o + n] += (sums / counts) @ self.w.T
                state[slot] = sums[-1]
                o += n

    class RunningMeanMixerOnDevice(RunningMeanMixer):
        """The same mixer with a decode step that a graph can hold: the rows' slots and positions are
        read on the device, the state is advanced by device operations, and padding rows (slot -1)
        change nothing.  Whole prompts (never captured) take the host-driven way."""
        graph_safe = True

        def forward(self, h, x, ctx, line, writes_cache=True):
            if ctx.mode != "decode":
                return super().forward(h, x, ctx, line, writes_cache)
            from yalm_amd.ops import kernels
            state = ctx.cache.group_of(line).line_state(line)          # [n_slots, dim]
            slot = ctx.seq_slot.long()
            live = (slot >= 0)[:, None]
            index = slot.clamp(min=0)
            state.index_add_(0, index, h.float() * live)               # a padding row adds zeros
            counts = (ctx.tok_pos + 1).float()[:, None]
            mean = (state.index_select(0, index) / counts * live).contiguous()
            kernels.gemm(mean, self.w, x, kernels.EPI_ADD_F32)

    register_part("mixer", "toy_running_mean", RunningMeanMixer, replace=True)
    register_part("mixer", "toy_running_mean_on_device", RunningMeanMixerOnDevice, replace=True)
    return RunningMeanMixer


class ToyConfig:
    """A toy architecture: layer 0 mixes with the running mean, layer 1 with
    attention; the schedule runs layer 1 twice (two cache lines) and then a third
    time as a reader of the first run's line: its queries are the present ones, its
    keys and values those that the first run stored.  `window` / `sinks` (optional)
    give the attention a window with attention sinks beside it."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def to_spec(self):
        from yalm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
        d = self.d
        D = d["width"]
        norm = {"eps": d["eps"]}
        pos = PartSpec("rope", {"head_dim": 16, "rotary_dim": 16, "theta": 100.0, "scaling": None,
                                "weight_rows": "interleaved"})
        mixers = [PartSpec(d.get("mean_mixer", "toy_running_mean"), {}, prefix="mean."),
                  PartSpec("gqa_attention", {"n_heads": 2, "n_kv_heads": 1, "head_dim": 16,
                                             "window": d.get("window", 0), "sinks": d.get("sinks", 0),
                                             "position": pos}, prefix="attn.")]
        layers = [LayerSpec("prenorm_residual", prefix="toy.%d." % i, mixer=m,
                            feed_forward=PartSpec("swiglu", {"hidden": d["hidden"]}, prefix="ff."),
                            mixer_norm=PartSpec("rmsnorm", norm, prefix="n1."),
                            feed_forward_norm=PartSpec("rmsnorm", norm, prefix="n2."))
                  for i, m in enumerate(mixers)]
        return ModelSpec("ToyForCausalLM", D, d["vocab"], d["positions"],
                         PartSpec("token_embedding", {"vocab_size": d["vocab"]}, prefix="toy.emb."), layers,
                         PartSpec("rmsnorm", norm, prefix="toy.norm."),
                         PartSpec("lm_head", {"vocab_size": d["vocab"], "tied": True}),
                         schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(1, 2),
                                   ScheduleEntry(1, 1, writes_cache=False)])


def toy_plain_forward(w, d, tokens):
    """The toy model written out with the plain implementation's functions."""
    T = len(tokens)
    x = R.embedding(w["toy.emb.weight"], torch.tensor(tokens))
    f = R.rope_inv_freq(16, 16, 100.0)
    pos = torch.arange(T)

    def ffn(x, p):
        return R.swiglu_ffn(R.rmsnorm(x, w[p + "n2.weight"], d["eps"]), w[p + "ff.gate_proj.weight"],
                            w[p + "ff.down_proj.weight"], w[p + "ff.up_proj.weight"])

    x = x + toy_mixer_plain(R.rmsnorm(x, w["toy.0.n1.weight"], d["eps"]), w["toy.0.mean.w.weight"])
    x = x + ffn(x, "toy.0.")
    first_kv = None
    for run in range(3):
        h = R.rmsnorm(x, w["toy.1.n1.weight"], d["eps"])
        q = (h @ w["toy.1.attn.q_proj.weight"].double().T).reshape(T, 2, 16)
        k = R.rope_interleaved((h @ w["toy.1.attn.k_proj.weight"].double().T).reshape(T, 1, 16), pos, f)
        v = (h @ w["toy.1.attn.v_proj.weight"].double().T).reshape(T, 1, 16)
        if run == 0:
            first_kv = (k, v)
        if run == 2:                       # the reader: keys and values as the first run stored them
            k, v = first_kv
        a = R.attention(R.rope_interleaved(q, pos, f), k, v, d.get("window", 0), d.get("sinks", 0), f)
        x = x + a.reshape(T, 32) @ w["toy.1.attn.o_proj.weight"].double().T
        x = x + ffn(x, "toy.1.")
    return R.rmsnorm(x, w["toy.norm.weight"], d["eps"]) @ w["toy.emb.weight"].double().T


@pytest.mark.parametrize("window,sinks", [(0, 0), (9, 2)])
@pytest.mark.parametrize("mixer", ["toy_running_mean", "toy_running_mean_on_device"])
def test_toy_mixer_and_architecture_from_outside(tmp_path, mixer, window, sinks):
    """Layer 0 carries state of its own.  With the host-driven mixer only that layer runs kernel by
    kernel in a decode step and the layers around it are replayed from graphs; with the device-driven
    one the whole step is one graph and the state is advanced inside it, once a step."""
    from yalm_amd import Engine, Model, register_architecture, write_random_model
    from yalm_amd.cache import StateGroup
    from yalm_amd.config import unregister_architecture
    from yalm_amd.parts import unregister_part
    define_toy_parts()
    register_architecture("ToyForCausalLM", ToyConfig, replace=True)
    try:
        d = {"architectures": ["ToyForCausalLM"], "width": 40, "hidden": 48, "vocab": 61, "positions": 200,
             "eps": 1e-5, "mean_mixer": mixer, "window": window, "sinks": sinks}
        folder = write_random_model(str(tmp_path / "toy"), d, seed=2)
        model = Model.from_folder(folder, dtype=torch.float32, device=DEV)
        engine = Engine(model, max_tokens=1024)
        if mixer == "toy_running_mean":
            assert not model.graph_safe()
            assert engine._segments == [(True, 0, 1), (False, 1, 2), (True, 2, 6)]
        else:
            assert model.graph_safe() and engine._segments == [(True, 0, 6)]
        assert len(engine.cache.state_groups) == 1 and isinstance(engine.cache.group_of(0), StateGroup)
        assert engine.cache.group_of(1) is engine.cache.group_of(2)          # the layer that runs twice: two lines
        assert engine.cache.group_of(1).lines == [1, 2]                      # the reader has no line of its own
        cfg, w = R.read_folder(folder)
        requests = {"a": [5, 9, 60, 3, 3, 17, 44, 8, 0, 31], "b": [7, 7, 2], "c": list(range(40, 61)) + list(range(30)),
                    "d": [60, 0, 1, 59, 2, 58]}
        for steps in (schedules.whole(requests), schedules.tail_one_by_one(requests, 4),
                      schedules.batches(requests, [["a", "b"], ["c", "d"]], {"a": 4, "b": 1, "c": 33, "d": 2}),
                      schedules.interleaved(requests, [["a", "b"], ["c", "d"]], {"a": 4, "b": 1, "c": 33, "d": 2},
                                            [0, 2])):
            out = schedules.replay_in_process(engine, steps)
            got = schedules.per_request(steps, out, requests)
            for rid, toks in requests.items():
                want = toy_plain_forward(w, d, toks).float().numpy()
                helpers.check_logits(got[rid], want, "float32", "toy %s" % rid)
        assert engine.graphs_captured > 0 and engine._graphs        # the decode steps above were replayed
    finally:
        unregister_architecture("ToyForCausalLM")
        unregister_part("mixer", "toy_running_mean")
        unregister_part("mixer", "toy_running_mean_on_device")


# ---------------------------------------------------------------------------
# a toy feed-forward with routing and a toy position encoding, in a second toy architecture
# ---------------------------------------------------------------------------

def define_routed_and_linear_parts():
    from yalm_amd.ops import kernels
    from yalm_amd.parts import Part, register_part
    from yalm_amd.weights import ParamSpec

    class Top1Experts(Part):
        """x += p_e * W2_e silu(W1_e h) with e = argmax of the router's logits and p_e its softmax
        probability (float32).  Rows are gathered per expert in front of the framework's GEMM and
        scattered back behind it."""
        graph_safe = False

        def __init__(self, spec, dim, prefix):
            super().__init__(spec, dim, prefix)
            self.n_experts, self.hidden = int(spec.params["n_experts"]), int(spec.params["hidden"])

        def param_specs(self):
            out = [ParamSpec(self.prefix + "router.weight", (self.n_experts, self.dim), fan_in=self.dim)]
            for e in range(self.n_experts):
                out.append(ParamSpec("%sexperts.%d.w1.weight" % (self.prefix, e), (self.hidden, self.dim), fan_in=self.dim))
                out.append(ParamSpec("%sexperts.%d.w2.weight" % (self.prefix, e), (self.dim, self.hidden),
                                     fan_in=self.hidden))
            return out

        def load(self, get, compute_dtype, device):
            self.router = get(self.prefix + "router.weight").to(device, torch.float32)
            self.w1 = [get("%sexperts.%d.w1.weight" % (self.prefix, e)).to(device, compute_dtype)
                       for e in range(self.n_experts)]
            self.w2 = [get("%sexperts.%d.w2.weight" % (self.prefix, e)).to(device, compute_dtype)
                       for e in range(self.n_experts)]

        def forward(self, h, x, ctx):
            logits = torch.empty((h.shape[0], self.n_experts), dtype=torch.float32, device=h.device)
            kernels.gemm(h.float().contiguous(), self.router, logits, kernels.EPI_STORE_F32)     # router in 32-bit
            prob, chosen = torch.softmax(logits, dim=-1).max(dim=-1)
            for e in range(self.n_experts):
                rows = (chosen == e).nonzero()[:, 0]
                if rows.numel() == 0:
                    continue
                he = h.index_select(0, rows).contiguous()
                mid = torch.empty((rows.numel(), self.hidden), dtype=torch.float32, device=h.device)
                self._gemm(ctx, he, self.w1[e], mid, kernels.EPI_STORE_F32)
                act = torch.nn.functional.silu(mid).to(h.dtype)
                y = torch.zeros((rows.numel(), self.dim), dtype=torch.float32, device=h.device)
                self._gemm(ctx, act, self.w2[e], y, kernels.EPI_ADD_F32)
                x.index_add_(0, rows, y * prob[rows][:, None])

    class LinearFrequencies(Part):
        """Rotation whose pair p turns by pos * step * (p + 1): the same table interface as the
        framework's rotary encoding, another law of frequencies."""

        def __init__(self, spec, dim, prefix):
            super().__init__(spec, dim, prefix)
            self.head_dim = int(spec.params["head_dim"])
            self.rotary_dim = int(spec.params["rotary_dim"])
            self.step = float(spec.params["step"])
            self.table = None

        def prepare(self, n_positions, device):
            f = self.step * torch.arange(1, self.rotary_dim // 2 + 1, dtype=torch.float64)
            ang = torch.arange(n_positions, dtype=torch.float64)[:, None] * f[None, :]
            self.table = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).float().contiguous().to(device)

        @property
        def n_positions(self):
            return 0 if self.table is None else self.table.shape[0]

        def arrange_projection_rows(self, w, n_heads):
            return w

    register_part("feed_forward", "toy_top1_experts", Top1Experts, replace=True)
    register_part("position", "toy_linear_frequencies", LinearFrequencies, replace=True)


class RoutedToyConfig:
    """Layer 0: attention with the linear-frequency rotation (half of each head rotated) and a dense
    feed-forward; layer 1: the same attention kind with a window and the routed feed-forward."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def to_spec(self):
        from yalm_amd.config import LayerSpec, ModelSpec, PartSpec
        d = self.d
        norm = {"eps": d["eps"]}
        pos = PartSpec("toy_linear_frequencies", {"head_dim": 32, "rotary_dim": 16, "step": d["step"]})

        def attn(window):
            return PartSpec("gqa_attention", {"n_heads": 3, "n_kv_heads": 3, "head_dim": 32, "window": window,
                                              "position": pos}, prefix="attn.")
        ffs = [PartSpec("swiglu", {"hidden": d["hidden"]}, prefix="ff."),
               PartSpec("toy_top1_experts", {"n_experts": d["experts"], "hidden": d["hidden"]}, prefix="moe.")]
        layers = [LayerSpec("prenorm_residual", prefix="toy.%d." % i, mixer=attn(w), feed_forward=ff,
                            mixer_norm=PartSpec("rmsnorm", norm, prefix="n1."),
                            feed_forward_norm=PartSpec("rmsnorm", norm, prefix="n2."))
                  for i, (w, ff) in enumerate(zip((0, 9), ffs))]
        return ModelSpec("RoutedToyForCausalLM", d["width"], d["vocab"], d["positions"],
                         PartSpec("token_embedding", {"vocab_size": d["vocab"]}, prefix="toy.emb."), layers,
                         PartSpec("rmsnorm", norm, prefix="toy.norm."),
                         PartSpec("lm_head", {"vocab_size": d["vocab"], "tied": False}, prefix="toy.head."))


def routed_toy_plain_forward(w, d, tokens):
    T = len(tokens)
    x = R.embedding(w["toy.emb.weight"], torch.tensor(tokens))
    f = torch.cat([d["step"] * torch.arange(1, 9, dtype=torch.float64), torch.zeros(8, dtype=torch.float64)])
    pos = torch.arange(T)
    for i, window in enumerate((0, 9)):
        p = "toy.%d." % i
        h = R.rmsnorm(x, w[p + "n1.weight"], d["eps"])
        q = (h @ w[p + "attn.q_proj.weight"].double().T).reshape(T, 3, 32)
        k = (h @ w[p + "attn.k_proj.weight"].double().T).reshape(T, 3, 32)
        v = (h @ w[p + "attn.v_proj.weight"].double().T).reshape(T, 3, 32)
        a = R.attention(R.rope_interleaved(q, pos, f), R.rope_interleaved(k, pos, f), v, window)
        x = x + a.reshape(T, 96) @ w[p + "attn.o_proj.weight"].double().T
        h = R.rmsnorm(x, w[p + "n2.weight"], d["eps"])
        if i == 0:
            x = x + R.swiglu_ffn(h, w[p + "ff.gate_proj.weight"], w[p + "ff.down_proj.weight"], w[p + "ff.up_proj.weight"])
        else:
            probs = torch.softmax(h @ w[p + "moe.router.weight"].double().T, dim=-1)
            for t in range(T):
                e = int(torch.argmax(probs[t]))
                mid = R.silu(w["%smoe.experts.%d.w1.weight" % (p, e)].double() @ h[t])
                x[t] = x[t] + probs[t, e] * (w["%smoe.experts.%d.w2.weight" % (p, e)].double() @ mid)
    return R.rmsnorm(x, w["toy.norm.weight"], d["eps"]) @ w["toy.head.weight"].double().T


def test_toy_routed_feed_forward_and_position_encoding_from_outside(tmp_path):
    """A feed-forward that routes rows to experts and a position encoding with its own law of angles,
    both defined above, take their places in a layer by configuration alone; every way of cutting the
    requests agrees with the toy written out in float64."""
    from yalm_amd import Engine, Model, register_architecture, write_random_model
    from yalm_amd.config import unregister_architecture
    from yalm_amd.parts import unregister_part
    define_routed_and_linear_parts()
    register_architecture("RoutedToyForCausalLM", RoutedToyConfig, replace=True)
    try:
        d = {"architectures": ["RoutedToyForCausalLM"], "width": 56, "hidden": 72, "vocab": 83, "positions": 128,
             "eps": 1e-6, "experts": 3, "step": 0.37}
        folder = write_random_model(str(tmp_path / "routed_toy"), d, seed=4)
        model = Model.from_folder(folder, dtype=torch.float32, device=DEV)
        assert not model.graph_safe()
        engine = Engine(model, max_tokens=1024)
        assert len(engine.cache.kv_groups) == 2                # all keys for layer 0, a window's ring for layer 1
        cfg, w = R.read_folder(folder)
        rng = np.random.default_rng(3)
        requests = {rid: [int(t) for t in rng.integers(0, d["vocab"], size=n)]
                    for rid, n in (("a", 30), ("b", 3), ("c", 70), ("d", 12))}
        used = set()
        probs = torch.softmax(R.rmsnorm(R.embedding(w["toy.emb.weight"], torch.tensor(requests["c"])),
                                        w["toy.1.n2.weight"], d["eps"]) @ w["toy.1.moe.router.weight"].double().T, -1)
        used.update(int(e) for e in probs.argmax(-1))
        assert len(used) > 1                                    # the routing has something to decide
        for steps in (schedules.whole(requests), schedules.tail_one_by_one(requests, 6),
                      schedules.batches(requests, [["a", "b"], ["c", "d"]], {"a": 11, "b": 1, "c": 64, "d": 2})):
            out = schedules.replay_in_process(engine, steps)
            got = schedules.per_request(steps, out, requests)
            for rid, toks in requests.items():
                want = routed_toy_plain_forward(w, d, toks).float().numpy()
                helpers.check_logits(got[rid], want, "float32", "routed toy %s" % rid)
    finally:
        unregister_architecture("RoutedToyForCausalLM")
        unregister_part("feed_forward", "toy_top1_experts")
        unregister_part("position", "toy_linear_frequencies")


# ---------------------------------------------------------------------------
# a toy position encoding that is no rotation: a term added to the scores by the distance of query and key
# ---------------------------------------------------------------------------

def define_distance_slopes():
    from yalm_amd.parts import Part, register_part

    class DistanceSlopes(Part):
        """No rotation.  Head h's score of a key `d` positions behind the query gets -slope * 2^(-h) * min(d, far)
        added: the framework's attention asks its position part for `score_bias` and hands it to the kernels."""
        rotary_dim = 0
        table = None
        n_positions = 0

        def __init__(self, spec, dim, prefix):
            super().__init__(spec, dim, prefix)
            self.n_heads, self.far, self.slope = int(spec.params["n_heads"]), int(spec.params["far"]), float(spec.params["slope"])
            self.score_bias = None

        def prepare(self, n_positions, device):
            if self.score_bias is None:                          # made once: captured graphs keep its address
                self.score_bias = distance_slopes_table(self.n_heads, self.far, self.slope).float().to(device)

        def arrange_projection_rows(self, w, n_heads):
            return w

    register_part("position", "toy_distance_slopes", DistanceSlopes, replace=True)


def distance_slopes_table(n_heads, far, slope):
    return -slope * (2.0 ** -torch.arange(n_heads, dtype=torch.float64))[:, None] * torch.arange(far + 1, dtype=torch.float64)[None, :]


class SlopesToyConfig:
    """Two layers of the framework's attention with the toy position part, the second with a window."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def to_spec(self):
        from yalm_amd.config import LayerSpec, ModelSpec, PartSpec
        d = self.d
        norm = {"eps": d["eps"]}
        pos = PartSpec("toy_distance_slopes", {"n_heads": d["heads"], "far": d["far"], "slope": d["slope"]})

        def attn(window):
            return PartSpec("gqa_attention", {"n_heads": d["heads"], "n_kv_heads": d["groups"], "head_dim": d["head"],
                                              "window": window, "position": pos}, prefix="attn.")
        layers = [LayerSpec("prenorm_residual", prefix="toy.%d." % i, mixer=attn(w),
                            feed_forward=PartSpec("swiglu", {"hidden": d["hidden"], "activation": "gelu"}, prefix="ff."),
                            mixer_norm=PartSpec("rmsnorm", norm, prefix="n1."),
                            feed_forward_norm=PartSpec("rmsnorm", norm, prefix="n2."))
                  for i, w in enumerate((0, d["window"]))]
        return ModelSpec("SlopesToyForCausalLM", d["width"], d["vocab"], d["positions"],
                         PartSpec("token_embedding", {"vocab_size": d["vocab"]}, prefix="toy.emb."), layers,
                         PartSpec("rmsnorm", norm, prefix="toy.norm."),
                         PartSpec("lm_head", {"vocab_size": d["vocab"], "tied": True}, prefix="toy.emb."))


def slopes_toy_plain_forward(w, d, tokens):
    T, H, G, hd = len(tokens), d["heads"], d["groups"], d["head"]
    x = R.embedding(w["toy.emb.weight"], torch.tensor(tokens))
    bias = distance_slopes_table(H, d["far"], d["slope"])
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    for l, window in enumerate((0, d["window"])):
        p = "toy.%d." % l
        h = R.rmsnorm(x, w[p + "n1.weight"], d["eps"])
        q = (h @ w[p + "attn.q_proj.weight"].double().T).reshape(T, H, hd)
        k = (h @ w[p + "attn.k_proj.weight"].double().T).reshape(T, G, hd)
        v = (h @ w[p + "attn.v_proj.weight"].double().T).reshape(T, G, hd)
        visible = (j <= i) & ((i - j < window) if window else torch.ones((T, T), dtype=torch.bool))
        a = torch.empty((T, H, hd), dtype=torch.float64)
        for hh in range(H):
            sc = q[:, hh] @ k[:, hh // (H // G)].T / hd ** 0.5 + bias[hh][(i - j).clamp(0, d["far"])]
            a[:, hh] = torch.softmax(sc.masked_fill(~visible, float("-inf")), dim=-1) @ v[:, hh // (H // G)]
        x = x + a.reshape(T, H * hd) @ w[p + "attn.o_proj.weight"].double().T
        h = R.rmsnorm(x, w[p + "n2.weight"], d["eps"])
        x = x + R.swiglu_ffn(h, w[p + "ff.gate_proj.weight"], w[p + "ff.down_proj.weight"], w[p + "ff.up_proj.weight"], "gelu")
    return R.rmsnorm(x, w["toy.norm.weight"], d["eps"]) @ w["toy.emb.weight"].double().T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encoding_that_is_no_rotation_from_outside(tmp_path, dtype):
    """A position part without any rotation, which instead has a term for every score by the distance of query and
    key, takes its place by configuration alone; prompts, single tokens and batches agree with the toy written out in
    float64 (and differ from the same model without the term, so the term is not lost on the way)."""
    from yalm_amd import Engine, Model, register_architecture, write_random_model
    from yalm_amd.config import unregister_architecture
    from yalm_amd.parts import unregister_part
    define_distance_slopes()
    register_architecture("SlopesToyForCausalLM", SlopesToyConfig, replace=True)
    try:
        d = {"architectures": ["SlopesToyForCausalLM"], "width": 72, "hidden": 104, "vocab": 91, "positions": 256,
             "eps": 1e-5, "heads": 6, "groups": 2, "head": 64, "window": 40, "far": 50, "slope": 0.8}
        folder = write_random_model(str(tmp_path / "slopes_toy"), d, seed=6)
        model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device=DEV)
        engine = Engine(model, max_tokens=2048)
        assert not model.describe()[1]                          # the matrix-core kernels take the term too
        cfg, w = R.read_folder(folder)
        if dtype == "bfloat16":
            w = {n: (t.bfloat16().float() if t.dim() > 1 else t) for n, t in w.items()}
        rng = np.random.default_rng(5)
        requests = {rid: [int(t) for t in rng.integers(0, d["vocab"], size=n)]
                    for rid, n in (("a", 30), ("b", 3), ("c", 150), ("d", 70))}
        want = {rid: slopes_toy_plain_forward(w, d, toks).float().numpy() for rid, toks in requests.items()}
        flat = slopes_toy_plain_forward(w, dict(d, slope=0.0), requests["c"]).float().numpy()
        assert np.abs(flat - want["c"]).max() > 0.05 * np.abs(want["c"]).max()
        for steps in (schedules.whole(requests), schedules.tail_one_by_one(requests, 32),
                      schedules.batches(requests, [["a", "b"], ["c", "d"]], {"a": 11, "b": 1, "c": 64, "d": 2})):
            out = schedules.replay_in_process(engine, steps)
            got = schedules.per_request(steps, out, requests)
            for rid in requests:
                helpers.check_logits(got[rid], want[rid], dtype, "slopes toy %s" % rid)
    finally:
        unregister_architecture("SlopesToyForCausalLM")
        unregister_part("position", "toy_distance_slopes")


# ---------------------------------------------------------------------------
# toy arrangements of a layer with other members than the reference's block has
# ---------------------------------------------------------------------------

def define_toy_blocks():
    from yalm_amd.parts import Part, build_part, register_part

    class ParallelBlock(Part):
        """x += mixer(norm(x)) + feed_forward(norm(x)): ONE norm, and both branches read its output.
        Members: norm, mixer, feed_forward."""

        def __init__(self, layer_spec, dim, prefix=""):
            super().__init__(None, dim, layer_spec.prefix)
            p = layer_spec.prefix
            self.norm = build_part("norm", layer_spec.norm, dim, p)
            self.mixer = build_part("mixer", layer_spec.mixer, dim, p)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, dim, p)

        def children(self):
            return [self.norm, self.mixer, self.feed_forward]

        def forward(self, x, ctx, line, writes_cache=True):
            h = ctx.ws.get("toy.parallel.h", (x.shape[0], self.dim), ctx.act_dtype)
            self.norm.forward(x, h, ctx)
            self.mixer.forward(h, x, ctx, line, writes_cache)
            self.feed_forward.forward(h, x, ctx)

    class FeedForwardOnlyBlock(Part):
        """x += feed_forward(norm(x)): no mixer, so the layer keeps nothing in the cache.
        Members: norm, feed_forward."""

        def __init__(self, layer_spec, dim, prefix=""):
            super().__init__(None, dim, layer_spec.prefix)
            self.norm = build_part("norm", layer_spec.norm, dim, layer_spec.prefix)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, dim, layer_spec.prefix)

        def children(self):
            return [self.norm, self.feed_forward]

        def forward(self, x, ctx, line, writes_cache=True):
            h = ctx.ws.get("toy.ffonly.h", (x.shape[0], self.dim), ctx.act_dtype)
            self.norm.forward(x, h, ctx)
            self.feed_forward.forward(h, x, ctx)

    register_part("block", "toy_parallel", ParallelBlock, replace=True)
    register_part("block", "toy_feed_forward_only", FeedForwardOnlyBlock, replace=True)


class BlocksToyConfig:
    """Three layers, three arrangements: the parallel block, the block without a mixer, and the
    reference's own.  Both attentions name the same position encoding."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def to_spec(self):
        from yalm_amd.config import LayerSpec, ModelSpec, PartSpec
        d = self.d
        norm = {"eps": d["eps"]}
        pos = PartSpec("rope", {"head_dim": 16, "rotary_dim": 8, "theta": 50.0, "scaling": None,
                                "weight_rows": "interleaved"})
        attn = PartSpec("gqa_attention", {"n_heads": 4, "n_kv_heads": 2, "head_dim": 16, "window": 0, "position": pos},
                        prefix="attn.")
        ff = PartSpec("swiglu", {"hidden": d["hidden"]}, prefix="ff.")
        layers = [LayerSpec("toy_parallel", prefix="toy.0.", norm=PartSpec("rmsnorm", norm, prefix="n."),
                            mixer=attn, feed_forward=ff),
                  LayerSpec("toy_feed_forward_only", {"norm": PartSpec("rmsnorm", norm, prefix="n."), "feed_forward": ff},
                            prefix="toy.1."),
                  LayerSpec("prenorm_residual", prefix="toy.2.", mixer=attn, feed_forward=ff,
                            mixer_norm=PartSpec("rmsnorm", norm, prefix="n1."),
                            feed_forward_norm=PartSpec("rmsnorm", norm, prefix="n2."))]
        return ModelSpec("BlocksToyForCausalLM", d["width"], d["vocab"], d["positions"],
                         PartSpec("token_embedding", {"vocab_size": d["vocab"]}, prefix="toy.emb."), layers,
                         PartSpec("rmsnorm", norm, prefix="toy.norm."),
                         PartSpec("lm_head", {"vocab_size": d["vocab"], "tied": True}))


def blocks_toy_plain_forward(w, d, tokens):
    T = len(tokens)
    x = R.embedding(w["toy.emb.weight"], torch.tensor(tokens))
    f = R.rope_inv_freq(16, 8, 50.0)
    pos = torch.arange(T)

    def attention(h, p):
        q = (h @ w[p + "attn.q_proj.weight"].double().T).reshape(T, 4, 16)
        k = (h @ w[p + "attn.k_proj.weight"].double().T).reshape(T, 2, 16)
        v = (h @ w[p + "attn.v_proj.weight"].double().T).reshape(T, 2, 16)
        a = R.attention(R.rope_interleaved(q, pos, f), R.rope_interleaved(k, pos, f), v, 0)
        return a.reshape(T, 64) @ w[p + "attn.o_proj.weight"].double().T

    def ffn(h, p):
        return R.swiglu_ffn(h, w[p + "ff.gate_proj.weight"], w[p + "ff.down_proj.weight"], w[p + "ff.up_proj.weight"])

    h = R.rmsnorm(x, w["toy.0.n.weight"], d["eps"])
    x = x + attention(h, "toy.0.") + ffn(h, "toy.0.")              # both branches from the one norm
    x = x + ffn(R.rmsnorm(x, w["toy.1.n.weight"], d["eps"]), "toy.1.")
    x = x + attention(R.rmsnorm(x, w["toy.2.n1.weight"], d["eps"]), "toy.2.")
    x = x + ffn(R.rmsnorm(x, w["toy.2.n2.weight"], d["eps"]), "toy.2.")
    return R.rmsnorm(x, w["toy.norm.weight"], d["eps"]) @ w["toy.emb.weight"].double().T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_blocks_with_other_members_from_outside(tmp_path, dtype):
    """Arrangements whose members are not the reference's four (one norm for two parallel branches; no mixer
    at all) are registered here, named by a configuration layer by layer, and stepped under every schedule.
    The two attentions share one table of angles, and the step's index tables are made once."""
    from yalm_amd import Engine, Model, register_architecture, write_random_model
    from yalm_amd.config import unregister_architecture
    from yalm_amd.parts import unregister_part
    define_toy_blocks()
    register_architecture("BlocksToyForCausalLM", BlocksToyConfig, replace=True)
    try:
        d = {"architectures": ["BlocksToyForCausalLM"], "width": 48, "hidden": 80, "vocab": 97, "positions": 160,
             "eps": 3e-6}
        folder = write_random_model(str(tmp_path / "blocks_toy"), d, seed=6)
        model = Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device=DEV)
        assert model.graph_safe()
        engine = Engine(model, max_tokens=1024)
        assert engine.cache.group_of(1) is None and engine.cache.group_of(0) is engine.cache.group_of(2)
        assert model.blocks[0].mixer.position is model.blocks[2].mixer.position          # one table for both
        assert model.blocks[0].mixer.position.table.shape[0] == 160
        assert [m.name for m in engine._prompt_tables] == ["kv_tiles"]                   # asked twice, made once
        cfg, w = R.read_folder(folder)
        if dtype == "bfloat16":
            w = {k: v if v.dim() <= 1 else v.to(torch.bfloat16) for k, v in w.items()}
        rng = np.random.default_rng(5)
        requests = {rid: [int(t) for t in rng.integers(0, d["vocab"], size=n)]
                    for rid, n in (("a", 40), ("b", 2), ("c", 130), ("d", 65))}
        for steps in (schedules.whole(requests), schedules.tail_one_by_one(requests, 32),
                      schedules.batches(requests, [["a", "b"], ["c", "d"]], {"a": 9, "b": 1, "c": 100, "d": 64}),
                      schedules.interleaved(requests, [["a", "b"], ["c", "d"]], {"a": 9, "b": 1, "c": 100, "d": 64},
                                            [0, 3])):
            out = schedules.replay_in_process(engine, steps)
            got = schedules.per_request(steps, out, requests)
            for rid, toks in requests.items():
                want = blocks_toy_plain_forward(w, d, toks).float().numpy()
                helpers.check_logits(got[rid], want, dtype, "blocks toy %s %s" % (dtype, rid))
        assert engine.graphs_captured > 0
    finally:
        unregister_architecture("BlocksToyForCausalLM")
        unregister_part("block", "toy_parallel")
        unregister_part("block", "toy_feed_forward_only")
