"""Plain, slow implementation of the Llama / Mistral dense decoder.

Whole sequences, no cache, one function per part, float64 throughout.  It is
written from the formulas of andrewkchan/yalm (each function cites the file
and lines it follows) and shares no code with the `yalm_amd` package: it reads
the raw `config.json` dictionary and a dictionary of tensors under their
Hugging Face names.

The engine is compared with this file; this file itself is pinned by
`tests/test_plain_reference.py` (vectors of the reference's own tests, special
cases that reduce to library routines, invariants).
"""
import json
import math
import os
import struct

import torch

F64 = torch.float64


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------

def rmsnorm(x, weight, eps):
    """src/infer.cpp:136-146.  ss = sum(x^2); rms = sqrt(ss/size + eps);
    out = x * (1/rms) * weight.  eps sits inside the root, added to the mean;
    the weight multiplies last; no bias, no `1 + w`."""
    x = x.to(F64)
    ss = (x * x).sum(dim=-1, keepdim=True)
    rms = torch.sqrt(ss / x.shape[-1] + eps)
    return x * (1.0 / rms) * weight.to(F64)


def rope_inv_freq(head_dim, rotary_dim, theta):
    """src/infer.cpp:203-205.  For the even index j inside a head:
    freq = 1 / theta^(j / rotary_dim) if j < rotary_dim else 0.
    Returned per pair p = j / 2: theta^(-2p / rotary_dim)."""
    out = torch.zeros(head_dim // 2, dtype=F64)
    for p in range(head_dim // 2):
        j = 2 * p
        out[p] = 0.0 if j >= rotary_dim else 1.0 / (float(theta) ** (j / rotary_dim))
    return out


def llama3_scaled_inv_freq(inv_freq, factor, low_freq_factor, high_freq_factor, original_max_position):
    """The reference has no rope scaling (convert.py:42-43 reads only
    rope_theta and partial_rotary_factor).  Definition used here, per pair with
    frequency f and wavelength lam = 2 pi / f, L = original_max_position:
      lam < L / high_freq_factor  -> f
      lam > L / low_freq_factor   -> f / factor
      else s = (L / lam - low) / (high - low);  f' = (1 - s) f / factor + s f."""
    out = inv_freq.clone()
    for p in range(inv_freq.numel()):
        f = float(inv_freq[p])
        if f == 0.0:
            continue
        lam = 2.0 * math.pi / f
        if lam < original_max_position / high_freq_factor:
            out[p] = f
        elif lam > original_max_position / low_freq_factor:
            out[p] = f / factor
        else:
            s = (original_max_position / lam - low_freq_factor) / (high_freq_factor - low_freq_factor)
            out[p] = (1.0 - s) * f / factor + s * f
    return out


def rope_interleaved(x, positions, inv_freq):
    """src/infer.cpp:202-215.  x: [T, n_heads, head_dim], positions: [T].
    Adjacent pairs (x[2p], x[2p+1]) are rotated by the angle pos * freq_p:
      y0 = x0 cos - x1 sin ;  y1 = x0 sin + x1 cos."""
    x = x.to(F64)
    T, H, hd = x.shape
    ang = positions.to(F64)[:, None] * inv_freq[None, :]          # [T, hd/2]
    c = torch.cos(ang)[:, None, :]
    s = torch.sin(ang)[:, None, :]
    x0 = x[..., 0::2]
    x1 = x[..., 1::2]
    y = torch.empty_like(x)
    y[..., 0::2] = x0 * c - x1 * s
    y[..., 1::2] = x0 * s + x1 * c
    return y


def rope_half_split(x, positions, inv_freq, rotary_dim):
    """The Hugging Face ordering of the same rotation: inside the first
    rotary_dim elements of a head, element p pairs with element
    p + rotary_dim/2.  Only used to pin `hf_rows_to_interleaved`
    (convert.py:145-158 exists because of this ordering)."""
    x = x.to(F64)
    half = rotary_dim // 2
    ang = positions.to(F64)[:, None] * inv_freq[None, :half]
    c = torch.cos(ang)[:, None, :]
    s = torch.sin(ang)[:, None, :]
    a = x[..., :half]
    b = x[..., half:rotary_dim]
    y = x.clone()
    y[..., :half] = a * c - b * s
    y[..., half:rotary_dim] = a * s + b * c
    return y


def hf_rows_to_interleaved(w, n_heads, rotary_dim):
    """convert.py:145-158 (`permute_reverse`).  Rows of a q/k projection are
    re-ordered inside each head so that the half-split pairs (p, p + r/2)
    become the adjacent pairs (2p, 2p+1); rows >= rotary_dim stay."""
    out_rows = w.shape[0]
    head_dim = out_rows // n_heads
    assert rotary_dim <= head_dim
    w = w.reshape(n_heads, head_dim, *w.shape[1:])
    wr = w[:, :rotary_dim]
    wk = w[:, rotary_dim:]
    half = rotary_dim // 2
    new = torch.empty_like(wr)
    for p in range(half):
        new[:, 2 * p] = wr[:, p]
        new[:, 2 * p + 1] = wr[:, half + p]
    w = torch.cat([new, wk], dim=1)
    return w.reshape(out_rows, *w.shape[2:])


def attention_probs_one_query(qh, K, head_dim):
    """src/infer.cpp:229-240.  Scores of one query head against kv_len keys:
    dot first, then divide by sqrt(head_dim); softmax with the maximum
    subtracted (src/infer.cpp:172-187)."""
    scores = (K.to(F64) @ qh.to(F64)) / math.sqrt(head_dim)
    m = scores.max()
    e = torch.exp(scores - m)
    return e / e.sum()


def attention(q, k, v, window=0, sinks=0, inv_freq=None):
    """src/infer.cpp:218-250 and 321-330 for every query position of a whole
    sequence.  q: [T, n_heads, hd]; k, v: [T, n_kv_heads, hd].  Query head h
    reads KV head h // (n_heads // n_kv_heads).  The reference sees only the
    cache rows [0, kv_len); for a whole sequence that is: key j is visible to
    query i iff j <= i and (window == 0 or i - j < window), the last
    `window` positions including the current one (src/infer.cpp:486-488).

    sinks (src/infer.cpp:305-319, 484-488 in closed form; `attention_context_ring`
    below is the same a step at a time): the first `sinks` positions stay
    visible behind the window.  The reference's cache of n = window + sinks rows
    keeps them from position n on and turns their keys one position further at
    every such step, i - n + 1 times up to query i; rotations add up, so the
    sink keys are the rotated keys turned by max(0, i - n + 1) positions more."""
    T, n_heads, hd = q.shape
    n_kv = k.shape[1]
    group = n_heads // n_kv
    out = torch.zeros(T, n_heads, hd, dtype=F64)
    k = k.to(F64)
    v = v.to(F64)
    for i in range(T):
        lo = 0 if window == 0 else max(0, i - window + 1)
        K, V = k[lo:i + 1], v[lo:i + 1]
        n_behind = min(sinks, lo)                       # sinks the window no longer covers
        if n_behind > 0:
            turn = max(0, i - (window + sinks) + 1)
            ks = k[:n_behind]
            if turn > 0:
                ks = rope_interleaved(ks, torch.full((n_behind,), turn), inv_freq)
            K = torch.cat([ks, K], dim=0)
            V = torch.cat([v[:n_behind], V], dim=0)
        for h in range(n_heads):
            g = h // group
            p = attention_probs_one_query(q[i, h], K[:, g], hd)
            out[i, h] = p @ V[:, g]
    return out


KV_SINKS = 2                                            # src/model.h:12


def attention_context_ring(q, k, v, context, inv_freq):
    """The reference's cache of `context` rows a token at a time, as written
    (src/infer.cpp:484-488: kv_sink, kv_pos, kv_len; 298-303: the new key and
    value go to row kv_pos; 305-319: each kept sink key is turned by one
    position; 321-330: attention over rows [0, kv_len)).  q, k: rotated at
    their positions.  Pins the closed form of `attention` with
    window = context - KV_SINKS and sinks = KV_SINKS."""
    T, n_heads, hd = q.shape
    n_kv = k.shape[1]
    group = n_heads // n_kv
    kb = torch.zeros(context, n_kv, hd, dtype=F64)
    vb = torch.zeros(context, n_kv, hd, dtype=F64)
    out = torch.zeros(T, n_heads, hd, dtype=F64)
    one = torch.ones(1)
    for pos in range(T):
        kv_sink = KV_SINKS if pos >= context else 0
        kv_pos = kv_sink + (pos - kv_sink) % (context - kv_sink)
        kv_len = context if pos >= context else pos + 1
        kb[kv_pos] = k[pos].to(F64)
        vb[kv_pos] = v[pos].to(F64)
        for r in range(kv_sink):
            kb[r] = rope_interleaved(kb[r:r + 1], one, inv_freq)[0]
        for h in range(n_heads):
            g = h // group
            p = attention_probs_one_query(q[pos, h], kb[:kv_len, g], hd)
            out[pos, h] = p @ vb[:kv_len, g]
    return out


def silu(x):
    """src/infer.cpp:193-195."""
    return x / (1.0 + torch.exp(-x))


def gelu(x):
    """src/infer.cpp:189-191: the tanh form, with the reference's rounded constants."""
    return 0.5 * x * (1.0 + torch.tanh(0.797885 * (x + 0.044715 * x * x * x)))


def swiglu_ffn(x, w_gate, w_down, w_up, act="silu"):
    """src/infer.cpp:356-385 with one expert of weight 1:
    down( act(gate x) * (up x) ), act silu or gelu (src/infer.cpp:364-372).  w1 = gate_proj, w3 = up_proj,
    w2 = down_proj (convert.py:195-197)."""
    x = x.to(F64)
    g = x @ w_gate.to(F64).T
    u = x @ w_up.to(F64).T
    return ({"silu": silu, "gelu": gelu}[act](g) * u) @ w_down.to(F64).T


def embedding(table, tokens):
    """src/infer.cpp:454-475: the row of the table, widened; no scaling."""
    return table.to(F64)[tokens]


# ----------------------------------------------------------------------------
# configuration as the plain model reads it (raw config.json keys)
# ----------------------------------------------------------------------------

def read_config(cfg):
    """convert.py:22-54 with the additions `rope_scaling`, `sliding_window` and `attention_sinks`."""
    arch = cfg["architectures"][0]
    assert arch in ("LlamaForCausalLM", "MistralForCausalLM"), arch
    c = {}
    c["dim"] = cfg["hidden_size"]
    c["hidden_dim"] = cfg["intermediate_size"]
    c["n_heads"] = cfg["num_attention_heads"]
    c["head_dim"] = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    c["n_layers"] = cfg["num_hidden_layers"]
    c["n_kv_heads"] = cfg.get("num_key_value_heads") or cfg["num_attention_heads"]
    c["vocab_size"] = cfg["vocab_size"]
    c["rope_theta"] = cfg.get("rope_theta", 10000.0)
    c["rotary_dim"] = int(c["head_dim"] * cfg.get("partial_rotary_factor", 1))
    c["norm_eps"] = cfg["rms_norm_eps"]
    c["window"] = cfg.get("sliding_window") or 0
    c["sinks"] = cfg.get("attention_sinks") or 0
    c["tied"] = cfg.get("tie_word_embeddings", None) is not False   # convert.py:200-204, 241
    c["rope_scaling"] = cfg.get("rope_scaling")
    c["act"] = cfg.get("hidden_act", "silu")               # convert.py:51-52
    assert c["act"] in ("gelu", "silu")
    return c


def model_inv_freq(c):
    f = rope_inv_freq(c["head_dim"], c["rotary_dim"], c["rope_theta"])
    rs = c["rope_scaling"]
    if rs:
        kind = rs.get("rope_type", rs.get("type"))
        assert kind == "llama3", kind
        f = llama3_scaled_inv_freq(f, rs["factor"], rs["low_freq_factor"], rs["high_freq_factor"],
                                   rs["original_max_position_embeddings"])
    return f


# ----------------------------------------------------------------------------
# whole model
# ----------------------------------------------------------------------------

def forward(weights, cfg, tokens, window_override=None, position_offset=0, sinks_override=None):
    """src/infer.cpp:477-521 and 256-386 for every position of one sequence.

    weights: tensors under Hugging Face names; cfg: the config.json dict;
    tokens: list of ints.  Returns float64 logits [T, vocab].
    Order per layer: norm -> q,k,v -> rope(q), rope(k) -> attention ->
    o-projection added to x -> norm -> SwiGLU added to x; then the final norm
    and the classifier (the embedding table when tied, model.cpp:389-398)."""
    c = read_config(cfg)
    window = c["window"] if window_override is None else window_override
    sinks = c["sinks"] if sinks_override is None else sinks_override
    T = len(tokens)
    tok = torch.tensor(tokens, dtype=torch.long)
    pos = torch.arange(T) + position_offset
    inv_freq = model_inv_freq(c)
    H, KV, hd, rd = c["n_heads"], c["n_kv_heads"], c["head_dim"], c["rotary_dim"]

    x = embedding(weights["model.embed_tokens.weight"], tok)
    for l in range(c["n_layers"]):
        p = f"model.layers.{l}."
        xb = rmsnorm(x, weights[p + "input_layernorm.weight"], c["norm_eps"])
        wq = hf_rows_to_interleaved(weights[p + "self_attn.q_proj.weight"].to(F64), H, rd)
        wk = hf_rows_to_interleaved(weights[p + "self_attn.k_proj.weight"].to(F64), KV, rd)
        wv = weights[p + "self_attn.v_proj.weight"].to(F64)
        q = (xb @ wq.T).reshape(T, H, hd)
        k = (xb @ wk.T).reshape(T, KV, hd)
        v = (xb @ wv.T).reshape(T, KV, hd)
        q = rope_interleaved(q, pos, inv_freq)
        k = rope_interleaved(k, pos, inv_freq)
        a = attention(q, k, v, window, sinks, inv_freq).reshape(T, H * hd)
        x = x + a @ weights[p + "self_attn.o_proj.weight"].to(F64).T
        xb = rmsnorm(x, weights[p + "post_attention_layernorm.weight"], c["norm_eps"])
        x = x + swiglu_ffn(xb, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.down_proj.weight"],
                           weights[p + "mlp.up_proj.weight"], c["act"])
    x = rmsnorm(x, weights["model.norm.weight"], c["norm_eps"])
    wcls = weights["model.embed_tokens.weight"] if c["tied"] else weights["lm_head.weight"]
    return x @ wcls.to(F64).T


# ----------------------------------------------------------------------------
# sampling (src/sampler.cpp)
# ----------------------------------------------------------------------------

def sample_argmax(logits):
    """src/sampler.cpp:27-38: strict '>' so the lowest index wins ties."""
    best, arg = -float("inf"), 0
    for i, l in enumerate(logits.tolist()):
        if l > best:
            best, arg = l, i
    return arg


def sample_prob(logits, index):
    """src/sampler.cpp:11-25: softmax probability of one index, temperature 1."""
    l = logits.to(F64)
    e = torch.exp(l - l.max())
    return float(e[index] / e.sum())


def sample_temperature(logits, temperature, r):
    """src/sampler.cpp:40-65 with the uniform number r given by the caller:
    first index whose running sum of exp((l - max)/T)/Z reaches r, else V-1."""
    if temperature == 0.0:
        return sample_argmax(logits)
    l = logits.to(F64)
    e = torch.exp((l - l.max()) / temperature)
    c = torch.cumsum(e / e.sum(), dim=0)
    hit = torch.nonzero(c >= r)
    return int(hit[0]) if hit.numel() else l.numel() - 1


def perplexity(logits, tokens):
    """src/main.cpp:200-218: N = len - 1; ppl = exp(-sum(logprob)/N);
    err = ppl * sqrt((ss - s^2/N) / N / N)."""
    N = len(tokens) - 1
    s = ss = 0.0
    for i in range(N):
        lp = math.log(sample_prob(logits[i], tokens[i + 1]))
        s += lp
        ss += lp * lp
    ppl = math.exp(-s / N)
    return ppl, ppl * math.sqrt(max(0.0, (ss - s * s / N)) / N / N)


# ----------------------------------------------------------------------------
# reading a model folder without the package's loader
# ----------------------------------------------------------------------------

_DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
           "I32": torch.int32, "I64": torch.int64}


def read_folder(path):
    """config.json and every *.safetensors of a folder (convert.py:216-231).
    The container is the one codec.cpp:97-155 parses: u64 header length, JSON
    header {name: {dtype, shape, data_offsets}}, raw little-endian data."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    for name in sorted(os.listdir(path)):
        if not name.endswith(".safetensors"):
            continue
        with open(os.path.join(path, name), "rb") as f:
            blob = f.read()
        (hlen,) = struct.unpack("<Q", blob[:8])
        header = json.loads(blob[8:8 + hlen])
        base = 8 + hlen
        for key, meta in header.items():
            if key == "__metadata__":
                continue
            assert key not in tensors
            lo, hi = meta["data_offsets"]
            t = torch.frombuffer(bytearray(blob[base + lo:base + hi]), dtype=_DTYPES[meta["dtype"]])
            tensors[key] = t.reshape(meta["shape"]).clone()
    return cfg, tensors
