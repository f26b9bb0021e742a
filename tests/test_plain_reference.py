"""Pins the plain implementation (tests/plain/reference_model.py) by what fixes
it beside the reference's text: the vectors of the reference's own tests,
special cases that reduce to a library routine, and invariants.  Each check is
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the
wrong place, a scale applied twice) fails it."""
import math

import pytest
import torch

from plain import reference_model as R
import tiny_configs

F64 = torch.float64


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Seeded weights under Hugging Face names, made here (not by the package)."""
    c = R.read_config(cfg)
    g = torch.Generator().manual_seed(seed)
    D, H, Q, KV, V = c["dim"], c["hidden_dim"], c["n_heads"] * c["head_dim"], c["n_kv_heads"] * c["head_dim"], c["vocab_size"]

    def lin(o, i):
        return ((torch.rand(o, i, generator=g, dtype=F64) * 2 - 1) / math.sqrt(i)).to(dtype)

    def norm(n):
        return (1 + (torch.rand(n, generator=g, dtype=F64) * 2 - 1) * 0.1).to(dtype)

    w = {"model.embed_tokens.weight": torch.randn(V, D, generator=g, dtype=F64).to(dtype)}
    for l in range(c["n_layers"]):
        p = f"model.layers.{l}."
        w[p + "input_layernorm.weight"] = norm(D)
        w[p + "self_attn.q_proj.weight"] = lin(Q, D)
        w[p + "self_attn.k_proj.weight"] = lin(KV, D)
        w[p + "self_attn.v_proj.weight"] = lin(KV, D)
        w[p + "self_attn.o_proj.weight"] = lin(D, Q)
        w[p + "post_attention_layernorm.weight"] = norm(D)
        w[p + "mlp.gate_proj.weight"] = lin(H, D)
        w[p + "mlp.up_proj.weight"] = lin(H, D)
        w[p + "mlp.down_proj.weight"] = lin(D, H)
    w["model.norm.weight"] = norm(D)
    if not c["tied"]:
        w["lm_head.weight"] = lin(V, D)
    return w


# ---------------------------------------------------------------- attention

def test_attention_vector_of_the_reference():
    """src/test.cpp:67-126: 2 heads, 1 KV head, head_dim 3, 4 keys."""
    q = torch.tensor([[0., 1e4, 0.], [0., 0., 1e4]], dtype=F64)
    K = torch.tensor([[1., 0, 0], [0, 1., 0], [0, 0, 1.], [-1., 0, 0]], dtype=F64)
    V = K.clone()
    p0 = R.attention_probs_one_query(q[0], K, 3)
    p1 = R.attention_probs_one_query(q[1], K, 3)
    assert torch.allclose(p0, torch.tensor([0., 1, 0, 0], dtype=F64), atol=1e-4)
    assert torch.allclose(p1, torch.tensor([0., 0, 1, 0], dtype=F64), atol=1e-4)
    # the same through the whole-sequence function: the last query sees all 4 keys
    T = 4
    qq = torch.zeros(T, 2, 3, dtype=F64)
    qq[3] = q
    out = R.attention(qq, K.reshape(T, 1, 3), V.reshape(T, 1, 3))
    assert torch.allclose(out[3], torch.tensor([[0., 1, 0], [0, 0, 1.]], dtype=F64), atol=1e-4)


def test_attention_reduces_to_library_sdpa():
    """Causal attention == torch's scaled_dot_product_attention with an explicit
    boolean mask, with grouped heads written out by repetition."""
    g = torch.Generator().manual_seed(1)
    T, H, KV, hd = 9, 4, 2, 8
    q = torch.randn(T, H, hd, generator=g, dtype=F64)
    k = torch.randn(T, KV, hd, generator=g, dtype=F64)
    v = torch.randn(T, KV, hd, generator=g, dtype=F64)
    for window in (0, 3, 1, 100):
        i = torch.arange(T)[:, None]
        j = torch.arange(T)[None, :]
        mask = (j <= i) & ((i - j < window) if window else torch.ones_like(j <= i))
        kk = k.repeat_interleave(H // KV, dim=1)
        vv = v.repeat_interleave(H // KV, dim=1)
        lib = torch.nn.functional.scaled_dot_product_attention(
            q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), attn_mask=mask).transpose(0, 1)
        assert torch.allclose(R.attention(q, k, v, window), lib, atol=1e-12), window


def test_attention_invariants():
    g = torch.Generator().manual_seed(2)
    T, H, KV, hd = 7, 6, 3, 4
    q = torch.randn(T, H, hd, generator=g, dtype=F64)
    k = torch.randn(T, KV, hd, generator=g, dtype=F64)
    v = torch.randn(T, KV, hd, generator=g, dtype=F64)
    out = R.attention(q, k, v)
    # the first query sees one key: the output is its value
    for h in range(H):
        assert torch.allclose(out[0, h], v[0, h // 2])
    # window 1: every query sees only itself
    w1 = R.attention(q, k, v, window=1)
    assert torch.allclose(w1, v.repeat_interleave(2, dim=1))
    # q = 0: the mean of the visible values
    z = R.attention(torch.zeros_like(q), k, v)
    assert torch.allclose(z[4, 0], v[:5, 0].mean(dim=0))
    # causality: changing later keys does not change earlier outputs
    k2, v2 = k.clone(), v.clone()
    k2[5:] += 1.0
    v2[5:] -= 2.0
    assert torch.allclose(R.attention(q, k2, v2)[:5], out[:5])
    # the scale is 1/sqrt(head_dim), applied once
    s = R.attention_probs_one_query(q[0, 0], k[:3, 0], hd)
    lib = torch.softmax((k[:3, 0] @ q[0, 0]) / math.sqrt(hd), dim=0)
    assert torch.allclose(s, lib)


# ---------------------------------------------------------------- rope

def test_rope_is_complex_multiplication():
    g = torch.Generator().manual_seed(3)
    T, H, hd, theta = 5, 2, 8, 10000.0
    x = torch.randn(T, H, hd, generator=g, dtype=F64)
    pos = torch.tensor([0, 1, 7, 100, 4095])
    f = R.rope_inv_freq(hd, hd, theta)
    # frequencies: theta^(-2p/hd)
    assert torch.allclose(f, torch.tensor([theta ** (-2 * p / hd) for p in range(hd // 2)], dtype=F64))
    y = R.rope_interleaved(x, pos, f)
    z = torch.view_as_complex(x.reshape(T, H, hd // 2, 2).contiguous())
    rot = torch.polar(torch.ones(T, hd // 2, dtype=F64), pos.to(F64)[:, None] * f[None, :])
    lib = torch.view_as_real(z * rot[:, None, :]).reshape(T, H, hd)
    assert torch.allclose(y, lib, atol=1e-12)
    # position 0 is the identity; pair norms are kept
    assert torch.allclose(y[0], x[0])
    assert torch.allclose(y.reshape(T, H, -1, 2).norm(dim=-1), x.reshape(T, H, -1, 2).norm(dim=-1))


def test_rope_scores_depend_on_distance_only_and_compose():
    g = torch.Generator().manual_seed(4)
    hd = 16
    f = R.rope_inv_freq(hd, hd, 1e6)
    q = torch.randn(1, 1, hd, generator=g, dtype=F64)
    k = torch.randn(1, 1, hd, generator=g, dtype=F64)

    def score(m, n):
        return (R.rope_interleaved(q, torch.tensor([m]), f) * R.rope_interleaved(k, torch.tensor([n]), f)).sum()

    assert torch.allclose(score(10, 3), score(107, 100), atol=1e-9)
    assert not torch.allclose(score(10, 3), score(3, 10), atol=1e-6)       # direction matters
    a = R.rope_interleaved(R.rope_interleaved(q, torch.tensor([5]), f), torch.tensor([9]), f)
    assert torch.allclose(a, R.rope_interleaved(q, torch.tensor([14]), f), atol=1e-12)


def test_partial_rotary_leaves_the_rest():
    hd, rd = 16, 8
    f = R.rope_inv_freq(hd, rd, 10000.0)
    assert (f[rd // 2:] == 0).all() and (f[:rd // 2] > 0).all()
    x = torch.arange(hd, dtype=F64).reshape(1, 1, hd) + 1
    y = R.rope_interleaved(x, torch.tensor([11]), f)
    assert torch.equal(y[..., rd:], x[..., rd:]) and not torch.allclose(y[..., :rd], x[..., :rd])


def test_interleaved_with_permuted_rows_equals_half_split_with_hf_rows():
    """What convert.py:145-158 is for: scores agree between the two orderings."""
    g = torch.Generator().manual_seed(5)
    D, H, hd = 24, 3, 8
    for rd in (8, 4):
        wq = torch.randn(H * hd, D, generator=g, dtype=F64)
        wk = torch.randn(H * hd, D, generator=g, dtype=F64)
        x = torch.randn(2, D, generator=g, dtype=F64)
        pos = torch.tensor([3, 12])
        f = R.rope_inv_freq(hd, rd, 10000.0)
        q_hf = R.rope_half_split((x @ wq.T).reshape(2, H, hd), pos, f, rd)
        k_hf = R.rope_half_split((x @ wk.T).reshape(2, H, hd), pos, f, rd)
        q_il = R.rope_interleaved((x @ R.hf_rows_to_interleaved(wq, H, rd).T).reshape(2, H, hd), pos, f)
        k_il = R.rope_interleaved((x @ R.hf_rows_to_interleaved(wk, H, rd).T).reshape(2, H, hd), pos, f)
        s_hf = torch.einsum("ihd,jhd->hij", q_hf, k_hf)
        s_il = torch.einsum("ihd,jhd->hij", q_il, k_il)
        assert torch.allclose(s_hf, s_il, atol=1e-10)
    # the permutation itself, on a row index ramp: head_dim 8, rotary 8 -> 0,4,1,5,2,6,3,7
    ramp = torch.arange(8, dtype=F64).reshape(8, 1)
    assert R.hf_rows_to_interleaved(ramp, 1, 8).flatten().tolist() == [0, 4, 1, 5, 2, 6, 3, 7]
    assert R.hf_rows_to_interleaved(ramp, 1, 4).flatten().tolist() == [0, 2, 1, 3, 4, 5, 6, 7]


def test_llama3_scaling():
    f = R.rope_inv_freq(32, 32, 500.0)
    same = R.llama3_scaled_inv_freq(f, 1.0, 1.0, 4.0, 32)
    assert torch.allclose(same, f)
    s = R.llama3_scaled_inv_freq(f, 8.0, 1.0, 4.0, 32)
    lam = 2 * math.pi / f
    hi, lo = lam < 32 / 4.0, lam > 32 / 1.0
    assert hi.any() and lo.any() and (~hi & ~lo).any()           # all three regimes occur
    assert torch.equal(s[hi], f[hi])
    assert torch.allclose(s[lo], f[lo] / 8.0)
    mid = ~hi & ~lo
    assert ((s[mid] < f[mid]) & (s[mid] > f[mid] / 8.0)).all()
    assert (s[1:] <= s[:-1]).all()                               # still monotone in the pair index
    # continuity at both thresholds
    for lam0, want in ((32 / 4.0, 1.0), (32 / 1.0, 1 / 8.0)):
        f0 = torch.tensor([2 * math.pi / (lam0 * (1 - 1e-9)), 2 * math.pi / (lam0 * (1 + 1e-9))], dtype=F64)
        r = R.llama3_scaled_inv_freq(f0, 8.0, 1.0, 4.0, 32) / f0
        assert abs(r[0] - want) < 1e-6 and abs(r[1] - want) < 1e-6


# ---------------------------------------------------------------- norm, ffn, head

def test_rmsnorm():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(3, 10, generator=g, dtype=F64)
    w = torch.rand(10, generator=g, dtype=F64) + 0.5
    lib = x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(R.rmsnorm(x, w, 1e-5), lib, atol=1e-12)
    y = R.rmsnorm(x, torch.ones(10, dtype=F64), 0.0)
    assert torch.allclose((y * y).mean(dim=-1), torch.ones(3, dtype=F64))
    assert torch.allclose(R.rmsnorm(7.0 * x, w, 0.0), R.rmsnorm(x, w, 0.0))
    assert torch.equal(R.rmsnorm(torch.zeros(1, 10, dtype=F64), w, 1e-6), torch.zeros(1, 10, dtype=F64))
    # eps is added to the mean of squares, not to the sum and not outside the root
    one = torch.ones(1, 4, dtype=F64)
    assert torch.allclose(R.rmsnorm(one, torch.ones(4, dtype=F64), 3.0), one / 2.0)


def test_swiglu():
    g = torch.Generator().manual_seed(7)
    D, H = 6, 10
    x = torch.randn(4, D, generator=g, dtype=F64)
    w1, w3, w2 = (torch.randn(H, D, generator=g, dtype=F64), torch.randn(H, D, generator=g, dtype=F64),
                  torch.randn(D, H, generator=g, dtype=F64))
    lib = (torch.nn.functional.silu(x @ w1.T) * (x @ w3.T)) @ w2.T
    assert torch.allclose(R.swiglu_ffn(x, w1, w2, w3), lib, atol=1e-12)
    assert torch.equal(R.swiglu_ffn(x, w1, w2, torch.zeros_like(w3)), torch.zeros(4, D, dtype=F64))
    t = torch.tensor([0.0, 30.0, -30.0], dtype=F64)
    assert torch.allclose(R.silu(t), torch.tensor([0.0, 30.0, 0.0], dtype=F64), atol=1e-10)
    # gate and up are not interchangeable
    assert not torch.allclose(R.swiglu_ffn(x, w3, w2, w1), lib)


def test_gelu_gate():
    """The reference's other activation (src/infer.cpp:189-191): the tanh form with constants rounded to six
    figures, so the library's tanh form agrees to about 1e-6 and no closer; its ends (0 far left, the identity far
    right), the place of its minimum, and a gated feed-forward that differs from the silu one."""
    t = torch.linspace(-6, 6, 241, dtype=F64)
    lib = torch.nn.functional.gelu(t, approximate="tanh")
    assert (R.gelu(t) - lib).abs().max() < 3e-6
    assert (R.gelu(t) - torch.nn.functional.gelu(t)).abs().max() < 1e-3          # and the erf form to three figures
    ends = R.gelu(torch.tensor([0.0, 30.0, -30.0, 1.0], dtype=F64))
    assert torch.allclose(ends, torch.tensor([0.0, 30.0, 0.0, 0.841192], dtype=F64), atol=1e-6)
    assert abs(float(t[R.gelu(t).argmin()]) + 0.75) <= 0.05                       # silu's minimum lies at -1.28
    g = torch.Generator().manual_seed(8)
    D, H = 6, 10
    x = torch.randn(4, D, generator=g, dtype=F64)
    w1, w3, w2 = (torch.randn(H, D, generator=g, dtype=F64), torch.randn(H, D, generator=g, dtype=F64),
                  torch.randn(D, H, generator=g, dtype=F64))
    lib = (torch.nn.functional.gelu(x @ w1.T, approximate="tanh") * (x @ w3.T)) @ w2.T
    assert torch.allclose(R.swiglu_ffn(x, w1, w2, w3, "gelu"), lib, atol=1e-4)
    assert not torch.allclose(R.swiglu_ffn(x, w1, w2, w3, "gelu"), R.swiglu_ffn(x, w1, w2, w3), atol=1e-2)


# ---------------------------------------------------------------- whole model

@pytest.mark.parametrize("name", ["tiny_llama", "tiny_mistral", "tiny_llama3", "tiny_wide_heads"])
def test_whole_model_invariants(name):
    cfg = tiny_configs.ALL[name]
    w = random_weights(cfg, seed=11)
    g = torch.Generator().manual_seed(12)
    T = 24
    tokens = torch.randint(0, cfg["vocab_size"], (T,), generator=g).tolist()
    logits = R.forward(w, cfg, tokens)
    assert logits.shape == (T, cfg["vocab_size"]) and torch.isfinite(logits).all()
    # causality: a change of later tokens leaves earlier logits alone
    t2 = list(tokens)
    t2[15] = (t2[15] + 1) % cfg["vocab_size"]
    l2 = R.forward(w, cfg, t2)
    assert torch.equal(l2[:15], logits[:15]) and not torch.allclose(l2[15:], logits[15:])
    # a prefix gives the same logits as the whole
    assert torch.allclose(R.forward(w, cfg, tokens[:10]), logits[:10], atol=1e-10)
    # only distances count: a shift of all positions changes nothing
    # (llama3 scaling keeps this: it only changes the frequencies)
    shifted = R.forward(w, cfg, tokens, position_offset=37)
    assert torch.allclose(shifted, logits, atol=1e-8)
    # the window matters where it is shorter than the sequence, and only there
    W = cfg.get("sliding_window") or 0
    nowin = R.forward(w, cfg, tokens, window_override=0)
    if W and W < T:
        assert torch.allclose(nowin[:W], logits[:W], atol=1e-10)
        assert not torch.allclose(nowin[W:], logits[W:], atol=1e-6)
    else:
        assert torch.allclose(nowin, logits, atol=1e-10)


def test_tied_head_uses_the_embedding():
    cfg = dict(tiny_configs.TINY_LLAMA)
    w = random_weights(cfg, seed=13)
    tokens = [3, 9, 200, 17]
    tied = R.forward(w, cfg, tokens)
    cfg2 = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    assert torch.equal(R.forward(w2, cfg2, tokens), tied)
    # absent key means tied (convert.py:241: exported only when exactly False)
    cfg3 = {k: v for k, v in cfg.items() if k != "tie_word_embeddings"}
    assert torch.equal(R.forward(w, cfg3, tokens), tied)


def test_one_head_one_layer_by_hand():
    """One layer, one head, no rotation (theta-independent at position 0 only,
    so rotary_dim = 0): the whole model written out with library calls."""
    cfg = {"architectures": ["LlamaForCausalLM"], "hidden_size": 8, "intermediate_size": 12, "num_hidden_layers": 1,
           "num_attention_heads": 1, "num_key_value_heads": 1, "head_dim": 8, "vocab_size": 20,
           "max_position_embeddings": 16, "rms_norm_eps": 1e-5, "hidden_act": "silu", "partial_rotary_factor": 0,
           "tie_word_embeddings": False}
    w = random_weights(cfg, seed=14, dtype=F64)
    tokens = [1, 5, 7, 7, 19]
    x = w["model.embed_tokens.weight"][tokens]

    def n(x, wt):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5) * wt

    p = "model.layers.0."
    h = n(x, w[p + "input_layernorm.weight"])
    q, k, v = (h @ w[p + f"self_attn.{s}_proj.weight"].T for s in "qkv")
    a = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    x = x + a @ w[p + "self_attn.o_proj.weight"].T
    h = n(x, w[p + "post_attention_layernorm.weight"])
    x = x + (torch.nn.functional.silu(h @ w[p + "mlp.gate_proj.weight"].T) * (h @ w[p + "mlp.up_proj.weight"].T)) \
        @ w[p + "mlp.down_proj.weight"].T
    lib = n(x, w["model.norm.weight"]) @ w["lm_head.weight"].T
    assert torch.allclose(R.forward(w, cfg, tokens), lib, atol=1e-10)


# ---------------------------------------------------------------- sampler

def test_sampler():
    l = torch.tensor([1.0, 3.0, 3.0, -2.0])
    assert R.sample_argmax(l) == 1                                   # lowest index wins ties
    assert R.sample_temperature(l, 0.0, 0.99) == 1
    p = torch.softmax(l.to(F64), 0)
    assert abs(R.sample_prob(l, 2) - float(p[2])) < 1e-12
    c = torch.cumsum(p, 0)
    assert R.sample_temperature(l, 1.0, float(c[0]) - 1e-9) == 0
    assert R.sample_temperature(l, 1.0, float(c[0]) + 1e-9) == 1
    assert R.sample_temperature(l, 1.0, 0.0) == 0
    assert R.sample_temperature(l, 1.0, 1.0 + 1e-9) == 3             # fallback: V - 1
    # temperature divides the logits
    p2 = torch.softmax(l.to(F64) / 0.5, 0)
    assert R.sample_temperature(l, 0.5, float(p2[0]) + 1e-9) == 1


def test_perplexity_of_uniform_logits_is_the_vocabulary():
    V = 17
    ppl, err = R.perplexity(torch.zeros(5, V), [1, 2, 3, 4, 5])
    assert abs(ppl - V) < 1e-9 and err < 1e-6


# ---------------------------------------------------------------- attention sinks

def _rotated_qkv(seed, T, H, KV, hd, rotary_dim, theta):
    g = torch.Generator().manual_seed(seed)
    inv = R.rope_inv_freq(hd, rotary_dim, theta)
    pos = torch.arange(T)
    q = R.rope_interleaved(torch.randn(T, H, hd, generator=g, dtype=F64), pos, inv)
    k = R.rope_interleaved(torch.randn(T, KV, hd, generator=g, dtype=F64), pos, inv)
    v = torch.randn(T, KV, hd, generator=g, dtype=F64)
    return q, k, v, inv


@pytest.mark.parametrize("context,T,rotary_dim", [(5, 23, 8), (9, 30, 4), (3, 11, 8), (16, 16, 8)])
def test_sinks_in_closed_form_equal_the_reference_ring_step_by_step(context, T, rotary_dim):
    """`attention` with a window of context - 2 and 2 sinks against the reference's cache of
    `context` rows filled and turned a token at a time (src/infer.cpp:484-488, 298-330)."""
    q, k, v, inv = _rotated_qkv(context, T, 4, 2, 8, rotary_dim, 50.0)
    ring = R.attention_context_ring(q, k, v, context, inv)
    closed = R.attention(q, k, v, window=context - R.KV_SINKS, sinks=R.KV_SINKS, inv_freq=inv)
    assert torch.allclose(ring, closed, rtol=0, atol=1e-12)
    # what plausible mistakes give is different: sinks left as they were stored, sinks turned by one
    # position too few, and no sinks at all
    if T > context + 1:
        still = R.attention(q, k, v, window=context - 2, sinks=2, inv_freq=torch.zeros_like(inv))
        assert (still - ring).abs().max() > 1e-3
        assert (R.attention(q, k, v, window=context - 2) - ring).abs().max() > 1e-3


def test_sinks_reduce_to_the_window_and_to_all_keys():
    q, k, v, inv = _rotated_qkv(7, 40, 6, 3, 8, 8, 100.0)
    # no sinks: the window alone; a window that covers everything: all keys, whatever the sinks
    assert torch.equal(R.attention(q, k, v, window=9, sinks=0, inv_freq=inv), R.attention(q, k, v, window=9))
    assert torch.allclose(R.attention(q, k, v, window=40, sinks=3, inv_freq=inv), R.attention(q, k, v))
    # up to position window + sinks - 1 every key is visible and none is turned
    some = R.attention(q, k, v, window=9, sinks=3, inv_freq=inv)
    assert torch.allclose(some[:12], R.attention(q, k, v)[:12])
    assert (some[12] - R.attention(q, k, v)[12]).abs().max() > 1e-6
    # a sink behind the window lies window + sinks - 1 - j behind the query wherever the query is: with keys
    # and queries that are the same vector at every position (before rotation) and values that name
    # their position, the weights of the sinks are the same at every position past the context
    T, hd = 40, 8
    base_q, base_k = torch.randn(1, 1, hd, dtype=F64), torch.randn(1, 1, hd, dtype=F64)
    pos = torch.arange(T)
    qq = R.rope_interleaved(base_q.expand(T, 1, hd).clone(), pos, inv)
    kk = R.rope_interleaved(base_k.expand(T, 1, hd).clone(), pos, inv)
    vv = torch.zeros(T, 1, hd, dtype=F64)
    vv[0, 0, 0] = 1.0                       # element 0 of the output = weight of sink 0
    vv[1, 0, 1] = 1.0                       # element 1 = weight of sink 1
    out = R.attention(qq, kk, vv, window=6, sinks=2, inv_freq=inv)
    assert torch.allclose(out[8:, 0, :2], out[8, 0, :2].expand(T - 8, 2), rtol=0, atol=1e-12)
    assert out[8, 0, 0] > 0 and out[8, 0, 1] > 0
