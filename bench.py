#!/usr/bin/env python3
"""Measures the library on one MI355X: decode tokens/s at batch 8 (the value),
at batch 1 and 64 (points), and the prefill of a 2,048-token prompt, for a
Mistral-7B-shaped model with random weights and random token ids (--shape: the
Llama-3.2-3B shape with prompts of 512 tokens at context 8,192, or the Mistral-7B-v0.1
shape with its window of 4,096 positions and prompts of 6,000 tokens).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers N] [--dtype bf16|fp32] [--shape NAME]
                    [--prompt-len N] [--prefill-len N] [--batch B] [--points B,B] [--no-prefill]
                    [--kernels] [--ragged] [--sweep]

--kernels adds the time of every kernel of a decode step and of a prompt step, each taken alone at the
shape's sizes (src/test.cpp:340-405 times single kernels so), with its rate against the peak;
--ragged adds generate() over 64 requests of unequal lengths beside the same batch at equal lengths;
--sweep adds the shape's whole workload end to end (src/main.cpp:104-147 times a whole run).

A step is one decode step as generation does it: the step function for a batch
of sequences (one token each, from the cache), greedy sampling on the device
and the read-back of the tokens.  The shape's workload decodes over a range of
positions (2,048 to 4,096 for the default shape); a run of K steps takes the K
positions in the middle of that range, so that its mean context is the whole
range's (K = 2,048 is the range itself), by prefilling that many random tokens.
One JSON line is printed.  Peaks are MI355X's
published ones: HBM 8 TB/s; dense MFMA bf16/fp16 2.5 PFLOP/s, fp32 157.3 TFLOP/s; beside them the line
names what a kernel that only reads memory and a loop of matrix-core instructions reach in this run
(`peak_measured`)."""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Mistral-7B-v0.2 shape
MISTRAL_7B = {
    "architectures": ["MistralForCausalLM"], "hidden_size": 4096, "intermediate_size": 14336,
    "num_hidden_layers": 32, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "vocab_size": 32000, "max_position_embeddings": 32768, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "hidden_act": "silu", "tie_word_embeddings": False, "bos_token_id": 1, "eos_token_id": 2,
}
# Llama-3.2-3B shape (llama3 rope scaling, tied head, a vocabulary that is no power of two)
LLAMA_3B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 3072, "intermediate_size": 8192,
    "num_hidden_layers": 28, "num_attention_heads": 24, "num_key_value_heads": 8, "head_dim": 128,
    "vocab_size": 128256, "max_position_embeddings": 131072, "rope_theta": 500000.0, "rms_norm_eps": 1e-5,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "hidden_act": "silu", "tie_word_embeddings": True, "bos_token_id": 128000, "eos_token_id": 128001,
}
# Mistral-7B-v0.1 shape (a window of 4,096 positions: ring cache)
MISTRAL_7B_V01 = dict(MISTRAL_7B, rope_theta=10000.0, sliding_window=4096)
# shape -> (config, name, context, first and last position of the workload's decoding)
SHAPES = {
    "mistral-7b-v0.2": (MISTRAL_7B, "Mistral-7B-v0.2 shape", 4096, (2048, 4096)),
    "llama-3.2-3b": (LLAMA_3B, "Llama-3.2-3B shape", 8192, (512, 8192)),
    "mistral-7b-v0.1": (MISTRAL_7B_V01, "Mistral-7B-v0.1 shape", 8192, (6000, 7024)),
}
PREFILL = 2048                   # tokens of the timed prompt
HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
BASELINE_TOK_S = 63.8            # the reference's published batch-1 figure (RTX 4090), README.md:14


def prefill_flops(cfg, n_layers, T):
    """GEMM flops of a prompt of T tokens + causal attention + the head on one row."""
    D, H, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    Q = cfg["num_attention_heads"] * cfg["head_dim"]
    KV = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = 2 * T * D * (Q + 2 * KV) + 2 * T * Q * D + 3 * 2 * T * D * H
    attn = 4 * cfg["num_attention_heads"] * cfg["head_dim"] * (T * (T + 1) // 2)
    return n_layers * (per_layer + attn) + 2 * D * V


def measured_peaks(torch, dtype):
    """(GB/s of a kernel that only reads 2 GB once, TFLOP/s of the better matrix-core loop on registers)."""
    from yalm_amd.ops import kernels
    buf = torch.empty(1 << 31, dtype=torch.uint8, device="cuda:0")
    buf.zero_()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = 0.0
    for wg in (256, 512, 1024, 2048):      # the fewer workgroups, the closer together the addresses in flight lie: 256 read fastest
        for _ in range(3):
            e0.record()
            n = kernels.probe_read(buf, wg)
            e1.record()
            e1.synchronize()
            best_read = max(best_read, n / (e0.elapsed_time(e1) * 1e-3) / 1e9)
    del buf
    best_mfma = 0.0
    if dtype == "bf16":
        for shape in (32, 16):
            for _ in range(3):
                e0.record()
                fl = kernels.probe_mfma(shape, 16384, 1024)
                e1.record()
                e1.synchronize()
                best_mfma = max(best_mfma, fl / (e0.elapsed_time(e1) * 1e-3) / 1e12)
    return round(best_read, 1), round(best_mfma, 1)


KERNEL_FACES = ("embed", "rmsnorm", "gemm", "gemm_norm", "gemm_norm_qkv_rope", "gemm_add_norm", "gemm_add_emit", "gemm_partial",
                "gemm_chain", "gemm_chain_qkv_rope", "rope_kv_write", "rope_kv_write_tiles", "attn_prefill",
                "attn_decode", "sink_store", "attn_sink_mix", "argmax")


def record_kernel_calls(run):
    """Runs `run()` with every face of ops.kernels wrapped; returns the calls it made, in order, as
    (face name, function, args, kwargs)."""
    from yalm_amd.ops import kernels
    calls, saved = [], {n: getattr(kernels, n) for n in KERNEL_FACES}

    def wrap(name, fn):
        def face(*a, **kw):
            calls.append((name, fn, a, kw))
            return fn(*a, **kw)
        return face
    for n, fn in saved.items():
        setattr(kernels, n, wrap(n, fn))
    try:
        run()
    finally:
        for n, fn in saved.items():
            setattr(kernels, n, fn)
    return calls


def kernel_cost(name, a, kw, kv_tokens, torch):
    """(label, bytes the call has to move, flops it has to do) from the call's own operands.  kv_tokens: the keys
    a decode attention reads, summed over its sequences."""
    def nbytes(*ts):
        return sum(t.numel() * t.element_size() for t in ts if torch.is_tensor(t))
    gemm_w = {"gemm": 1, "gemm_chain": 1, "gemm_add_norm": 1, "gemm_add_emit": 1, "gemm_partial": 1, "gemm_norm": 3,
              "gemm_norm_qkv_rope": 3, "gemm_chain_qkv_rope": 2}
    if name in gemm_w:
        x, w = a[0], a[gemm_w[name]]
        M, K = x.shape
        N = w.shape[0]
        out_bytes = M * N * 4
        return "%s %dx%dx%d" % (name, M, N, K), nbytes(x, w) + out_bytes, 2.0 * M * N * K
    if name == "attn_decode":
        q, kp = a[0], a[1]
        n_kv, hd = kp.shape[1], kp.shape[3]
        return "attn_decode %d rows" % q.shape[0], 2 * kv_tokens * n_kv * hd * kp.element_size() + 2 * nbytes(q), \
            4.0 * q.shape[1] * kv_tokens
    if name == "attn_prefill":
        q, cu = a[0], a[4]
        lens = (cu[1:] - cu[:-1]).tolist()
        pairs = sum(n * (n + 1) // 2 for n in lens)
        window = a[11]
        if window:
            pairs = sum(sum(min(i + 1, window) for i in range(n)) for n in lens)
        return "attn_prefill %d tokens" % q.shape[0], nbytes(q, a[1], a[2], a[3]), 4.0 * q.shape[1] * pairs
    if name in ("rope_kv_write", "rope_kv_write_tiles"):
        q_out = a[1]
        T, Q = q_out.shape
        n_kv, hd = a[15 if name == "rope_kv_write" else 14], a[16 if name == "rope_kv_write" else 15]
        width = Q + 2 * n_kv * hd
        slices = kw.get("slices", 1)
        return "%s %d tokens, %d slices" % (name, T, slices), T * width * (4 * slices + 2 * q_out.element_size()), 0.0
    if name == "rmsnorm":
        return "rmsnorm %dx%d" % tuple(a[2].shape), nbytes(a[2]) + a[2].numel() * 4, 0.0
    if name == "embed":
        return "embed %d" % a[1].shape[0], 2 * nbytes(a[2]), 0.0
    if name == "argmax":
        return "argmax %dx%d" % tuple(a[0].shape), nbytes(a[0]), 0.0
    return name, nbytes(*a), 0.0


def time_kernel_groups(calls, kv_tokens, torch, dtype, reps=5):
    """Every kernel of a step alone: the calls with the same face and shapes (one a layer) are captured into one
    graph in the order of the step, so that each reads weights that no call just before it has read, and the
    graph is replayed between two events (the best of `reps` replays counts).  Returns {label: {calls, us, GB/s, TFLOP/s, frac, bound}}."""
    groups = {}
    for name, fn, a, kw in calls:
        label, nb, fl = kernel_cost(name, a, kw, kv_tokens, torch)
        g = groups.setdefault(label, {"calls": [], "bytes": nb, "flops": fl})
        g["calls"].append((fn, a, kw))
    flush = torch.empty(1 << 29, dtype=torch.uint8, device="cuda:0")        # 512 MB: more than the caches hold
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(graph):
        graph.replay()
        best = None
        for _ in range(reps):
            e0.record()
            graph.replay()
            e1.record()
            e1.synchronize()
            t = e0.elapsed_time(e1)
            best = t if best is None else min(best, t)
        return best

    # every graph begins by overwriting 512 MB, so that no kernel finds its operands in a cache; the time of a
    # graph that does only that is taken off (with it goes what starting a graph costs)
    empty = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(empty):
        flush.zero_()
    base = timed(empty)
    out = {}
    for label, g in groups.items():
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            flush.zero_()
            for fn, a, kw in g["calls"]:
                fn(*a, **kw)
        total = max(timed(graph) - base, 1e-4) * reps
        n = len(g["calls"])
        us = total / reps / n * 1e3
        gbs = g["bytes"] / us / 1e3
        tfs = g["flops"] / us / 1e6
        frac_hbm, frac_mfma = gbs * 1e9 / HBM_PEAK, tfs * 1e12 / FLOP_PEAK[dtype]
        bound = "hbm" if frac_hbm >= frac_mfma else "mfma"
        out[label] = {"calls": n, "us": round(us, 2), "GB/s": round(gbs, 1), "TFLOP/s": round(tfs, 2),
                      "bound": bound, "frac": round(max(frac_hbm, frac_mfma), 4)}
        del graph
    return out


def mean_of(values):
    return int(sum(values) / len(values))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="build only the first N layers (0 = all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--points", default="1,64", help="further batch sizes to measure")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prompt-len", type=int, default=0,
                    help="tokens every sequence holds before decoding (0: so that the run lies in the middle of the "
                         "shape's range of positions)")
    ap.add_argument("--prefill-len", type=int, default=PREFILL, help="tokens of the timed prompt")
    ap.add_argument("--shape", default="mistral-7b-v0.2", choices=sorted(SHAPES),
                    help="the layer sizes: the Mistral-7B-v0.2 shape (default), Llama-3.2-3B or Mistral-7B-v0.1")
    ap.add_argument("--kernels", action="store_true",
                    help="also time every kernel of a decode step (at --batch) and of the prompt step alone")
    ap.add_argument("--ragged", action="store_true",
                    help="also run generate() over 64 requests of 1,024 to 3,072 tokens beside the same batch at "
                         "equal lengths")
    ap.add_argument("--ragged-new", type=int, default=128, help="new tokens of each request of --ragged")
    ap.add_argument("--sweep", action="store_true",
                    help="also run the shape's whole workload end to end at --batch: the prompts, then every "
                         "decode step of its range of positions")
    ap.add_argument("--context", type=int, default=0,
                    help="the reference's -T: past this many positions two attention sinks and the last "
                         "<context> - 2 positions are attended to (0: the shape's own window, if any)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this library runs on one GPU; --gpus %d is not measured" % args.gpus, flush=True)
        return 2

    import torch
    from yalm_amd import Engine, Model, Sampler
    from yalm_amd.cache import PAGE

    dtype = {"bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    CFG, shape_name, CONTEXT, (first, last) = SHAPES[args.shape]
    if args.context:
        CFG = dict(CFG, sliding_window=args.context - 2, attention_sinks=2)
        shape_name += ", context %d (2 sinks)" % args.context
    # the timed steps' positions lie in the middle of the workload's range (all of it if they are as many)
    run = args.steps + args.warmup
    PROMPT = max(first, min((first + last - args.steps) // 2 - args.warmup, last - run))
    if args.prompt_len:
        PROMPT = args.prompt_len
    CONTEXT = max(CONTEXT, PROMPT + run + 64)
    PREFILL_LEN = args.prefill_len
    n_layers = args.layers or CFG["num_hidden_layers"]
    dev = "cuda:0"
    t0 = time.time()
    model = Model.random(CFG, seed=0, dtype=dtype, device=dev, n_layers=n_layers)
    torch.cuda.synchronize()
    sys.stderr.write("[bench] %d layers of random weights in %.1f s\n" % (n_layers, time.time() - t0))
    batches = sorted({args.batch} | {int(b) for b in args.points.split(",") if b})
    RAGGED_B, RAGGED_LENS = 64, (1024, 3072)
    if args.ragged:
        CONTEXT = max(CONTEXT, RAGGED_LENS[1] + args.ragged_new + 64)
    most = max(batches + ([RAGGED_B] if args.ragged else []))
    engine = Engine(model, max_tokens=most * CONTEXT, max_batch=most)
    read_peak, mfma_peak = measured_peaks(torch, args.dtype)
    sys.stderr.write("[bench] measured here: a kernel that only reads memory %.0f GB/s, a loop of matrix-core "
                     "instructions %.0f TFLOP/s\n" % (read_peak, mfma_peak))
    t0 = time.time()
    n_graphs = engine.warmup(batches, min_len=PROMPT + 1, max_len=PROMPT + args.steps + args.warmup + 1)
    torch.cuda.synchronize()
    sys.stderr.write("[bench] %d decode graphs captured ahead in %.2f s; their shared buffers hold %.1f MB\n"
                     % (n_graphs, time.time() - t0, engine.graph_bytes() / 1e6))
    sampler = Sampler(0)
    V = CFG["vocab_size"]
    gen = torch.Generator().manual_seed(1)

    def sync():
        torch.cuda.synchronize()

    # ---------------------------------------------------------------- prefill of one 2,048-token prompt
    prefill = None
    if not args.no_prefill:
        prompt = torch.randint(0, V, (PREFILL_LEN,), generator=gen).tolist()
        times = []
        for i in range(3):
            slots = engine.start(1)
            sync()
            t = time.perf_counter()
            logits = engine.step(slots, [prompt])
            sampler.sample(logits, 0.0, [0], [0])
            sync()
            times.append(time.perf_counter() - t)
            engine.release(slots)
        sec = min(times[1:])
        fl = prefill_flops(CFG, n_layers, PREFILL_LEN)
        prefill = {"value": round(PREFILL_LEN / sec, 1), "tokens": PREFILL_LEN, "ms": round(sec * 1e3, 3),
                   "frac": round(fl / sec / FLOP_PEAK[args.dtype], 4)}
        if mfma_peak:
            prefill["peak_measured"] = mfma_peak
            prefill["peak_measured_unit"] = "TFLOP/s"
        sys.stderr.write("[bench] prefill %s\n" % prefill)

    # ---------------------------------------------------------------- decode
    def decode(B, steps, warmup, prompt_len=None):
        PROMPT_B = prompt_len or PROMPT
        prompts = [torch.randint(0, V, (PROMPT_B,), generator=gen).tolist() for _ in range(B)]
        slots = engine.start(B)
        ids = list(range(B))
        # prompts in chunks of sequences, so that the prefill workspace stays small
        tokens = []
        n = max(1, min(8, 48000 // PROMPT_B))
        for i in range(0, B, n):
            logits = engine.step(slots[i:i + n], prompts[i:i + n])
            tokens += sampler.sample(logits, 0.0, ids[i:i + n], [0] * len(slots[i:i + n]))
        # decode steps as generate() runs them: each step takes its tokens from the draw before on the
        # device, and the host reads every draw while the step behind it runs
        def advance(n, drawn):
            for _ in range(n):
                logits = engine.step_from(slots, drawn.tokens)
                ahead = sampler.draw(logits, 0.0, ids, [0] * B)
                drawn.tolist()
                drawn = ahead
            return drawn

        drawn = sampler.draw(engine.step(slots, [[t] for t in tokens]), 0.0, ids, [0] * B)
        drawn = advance(warmup, drawn)
        sync()
        start_len = engine.length(slots[0])
        t = time.perf_counter()
        advance(steps, drawn)
        sync()
        sec = time.perf_counter() - t
        end_len = engine.length(slots[0])
        engine.release(slots)
        mean_ctx = (start_len + 1 + end_len) / 2.0
        kv_bytes = sum(g.bytes_per_token() * (min(mean_ctx, g.window) if g.window else mean_ctx)
                       for g in engine.cache.kv_groups) * B          # a windowed group reads its window only
        step_bytes = model.weight_bytes() + (B - 1) * model.embedding.weight_bytes() + kv_bytes
        return {"tok_s": B * steps / sec, "ms": sec / steps * 1e3, "bytes": step_bytes, "ctx": mean_ctx}

    results = {}
    for B in batches:
        results[B] = decode(B, args.steps, args.warmup)
        sys.stderr.write("[bench] decode B=%d: %.1f tok/s, %.3f ms/step, %.1f GB/step -> %.0f GB/s\n" % (
            B, results[B]["tok_s"], results[B]["ms"], results[B]["bytes"] / 1e9,
            results[B]["bytes"] / results[B]["ms"] / 1e6))

    sys.stderr.write("[bench] %d graphs captured in all; graph buffers %.1f MB, other step buffers %.1f MB\n"
                     % (engine.graphs_captured, engine.graph_bytes() / 1e6, engine.ws.bytes() / 1e6))
    main_r = results[args.batch]
    achieved = main_r["bytes"] / (main_r["ms"] * 1e-3) / 1e9
    line = {
        "metric": "decode tok/s @ batch %d, %s, context %d" % (args.batch, shape_name.replace("-v0.2", ""), CONTEXT),
        "value": round(main_r["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(main_r["ms"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(results[1]["tok_s"] / BASELINE_TOK_S, 2) if 1 in results else None,
        "dtype": args.dtype, "data": "synthetic: seeded random weights and token ids",
        "config": {
            "model": shape_name, "global_batch": args.batch, "seq_len": CONTEXT, "parallelism": "none",
            "layers": n_layers, "layers_of_config": CFG["num_hidden_layers"], "dim": CFG["hidden_size"],
            "hidden_dim": CFG["intermediate_size"], "n_heads": CFG["num_attention_heads"],
            "n_kv_heads": CFG["num_key_value_heads"], "head_dim": CFG["head_dim"], "vocab_size": V,
            "rope_theta": CFG["rope_theta"], "norm_eps": CFG["rms_norm_eps"], "tied": CFG["tie_word_embeddings"],
            "window": CFG.get("sliding_window") or 0, "prompt_len": PROMPT,
            "decode_mean_context": round(main_r["ctx"], 1), "kv_dtype": args.dtype, "page_tokens": PAGE,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 4), "peak_measured": read_peak},
        "points": {"decode_b%d" % B: round(r["tok_s"], 1) for B, r in results.items() if B != args.batch},
        "points_roofline_frac": {"decode_b%d" % B: round(r["bytes"] / (r["ms"] * 1e-3) / HBM_PEAK, 4)
                                 for B, r in results.items()},
        "vs_baseline_note": "batch-1 decode tok/s over the reference's published 63.8 tok/s (RTX 4090, fp16)",
    }
    if prefill is not None:
        line["prefill"] = prefill

    # ---------------------------------------------------------------- every kernel of a step alone
    if args.kernels:
        B = args.batch
        L = int(main_r["ctx"])
        slots = engine.start(B)
        n = max(1, min(8, 48000 // L))
        tokens = []
        for i in range(0, B, n):
            part = [torch.randint(0, V, (L - 1,), generator=gen).tolist() for _ in slots[i:i + n]]
            tokens += sampler.sample(engine.step(slots[i:i + n], part), 0.0, list(range(len(part))), [0] * len(part))
        graphs_on, engine.use_graphs = engine.use_graphs, False
        try:
            calls = record_kernel_calls(
                lambda: sampler.draw(engine.step(slots, [[t] for t in tokens]), 0.0, list(range(B)), [0] * B))
        finally:
            engine.use_graphs = graphs_on
        sync()
        per_kernel = time_kernel_groups(calls, B * L, torch, args.dtype)
        engine.release(slots)
        total = sum(k["us"] * k["calls"] for k in per_kernel.values())
        line["kernels"] = {"decode_b%d" % B: dict(per_kernel, sum_us=round(total, 1),
                                                    step_us=round(main_r["ms"] * 1e3, 1), context=L)}
        for label, k in per_kernel.items():
            sys.stderr.write("[bench] decode B=%d  %-44s x%-3d %8.2f us  %8.1f GB/s  %7.2f TFLOP/s  %.3f of %s\n"
                             % (B, label, k["calls"], k["us"], k["GB/s"], k["TFLOP/s"], k["frac"], k["bound"]))
        sys.stderr.write("[bench] decode B=%d: kernels alone %.0f us, the step %.0f us\n" % (B, total, main_r["ms"] * 1e3))
        if not args.no_prefill:
            slots = engine.start(1)
            prompt = torch.randint(0, V, (PREFILL_LEN,), generator=gen).tolist()
            calls = record_kernel_calls(lambda: sampler.draw(engine.step(slots, [prompt]), 0.0, [0], [0]))
            sync()
            per_kernel = time_kernel_groups(calls, 0, torch, args.dtype)
            engine.release(slots)
            total = sum(k["us"] * k["calls"] for k in per_kernel.values())
            line["kernels"]["prefill_%d" % PREFILL_LEN] = dict(per_kernel, sum_us=round(total, 1),
                                                               step_us=round(prefill["ms"] * 1e3, 1))
            for label, k in per_kernel.items():
                sys.stderr.write("[bench] prefill %d  %-44s x%-3d %8.2f us  %8.1f GB/s  %7.2f TFLOP/s  %.3f of %s\n"
                                 % (PREFILL_LEN, label, k["calls"], k["us"], k["GB/s"], k["TFLOP/s"], k["frac"],
                                    k["bound"]))
            sys.stderr.write("[bench] prefill %d: kernels alone %.0f us, the step %.0f us\n"
                             % (PREFILL_LEN, total, prefill["ms"] * 1e3))

    # ---------------------------------------------------------------- requests of unequal lengths through generate()
    if args.ragged:
        from yalm_amd.generate import GenerationStats, generate
        lens = torch.randint(RAGGED_LENS[0], RAGGED_LENS[1] + 1, (RAGGED_B,), generator=gen).tolist()
        prompts = [torch.randint(0, V, (n,), generator=gen).tolist() for n in lens]
        engine.warmup([RAGGED_B], min_len=max(lens), max_len=max(lens) + args.ragged_new + 1, ragged=True)
        engine.warmup([RAGGED_B], min_len=mean_of(lens), max_len=mean_of(lens) + args.ragged_new + 1)
        stats = GenerationStats()
        generate(engine, prompts, max_new_tokens=args.ragged_new, temperature=0.0, stop_ids=(), batch_size=RAGGED_B,
                 sampler=sampler, stats=stats)
        mean_len = mean_of(lens)
        equal = decode(RAGGED_B, args.ragged_new - 8, 8, prompt_len=mean_len)
        line["ragged"] = {
            "requests": RAGGED_B, "prompt_min": min(lens), "prompt_max": max(lens), "prompt_mean": mean_len,
            "new_tokens": args.ragged_new, "decode_tok_s": round(stats.decode_tokens_per_second, 1),
            "ms_per_step": round(stats.decode_seconds / max(1, stats.decode_steps) * 1e3, 4),
            "prefill_tok_s": round(stats.prefill_tokens_per_second, 1),
            "equal_length_decode_tok_s": round(equal["tok_s"], 1), "equal_length_ms_per_step": round(equal["ms"], 4),
            "roofline_frac": round(stats.bytes_read / max(1, stats.decode_steps + 1)
                                   / (stats.decode_seconds / max(1, stats.decode_steps)) / HBM_PEAK, 4)}
        sys.stderr.write("[bench] ragged %s\n" % line["ragged"])

    # ---------------------------------------------------------------- the shape's whole workload, end to end
    if args.sweep:
        from yalm_amd.generate import GenerationStats, generate
        B = args.batch
        prompts = [torch.randint(0, V, (first,), generator=gen).tolist() for _ in range(B)]
        engine.warmup([B], min_len=first, max_len=last + 1)
        stats = GenerationStats()
        t = time.perf_counter()
        generate(engine, prompts, max_new_tokens=last - first, temperature=0.0, stop_ids=(), batch_size=B,
                 sampler=sampler, stats=stats)
        sync()
        sec = time.perf_counter() - t
        line["sweep"] = {
            "batch": B, "prompt_tokens": first, "new_tokens": last - first, "seconds": round(sec, 3),
            "tok_s_prompt_and_new": round((stats.prompt_tokens + stats.new_tokens) / sec, 1),       # src/main.cpp:139
            "prefill_tok_s": round(stats.prefill_tokens_per_second, 1),
            "decode_tok_s": round(stats.decode_tokens_per_second, 1),
            "decode_ms_per_step": round(stats.decode_seconds / max(1, stats.decode_steps) * 1e3, 4),
            "GB_per_s": round(stats.bytes_read / sec / 1e9, 1)}
        sys.stderr.write("[bench] sweep %s\n" % line["sweep"])
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
