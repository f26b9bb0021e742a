"""Command line in the reference's manner (src/main.cpp:17-40, 334-470):

    python -m yalm_amd <model folder> [options]
    python -m yalm_amd --random <config.json> [--weight-seed <int>] [options]     (random weights, no folder)
      -h                 this text
      -d [hip,cuda]      device; there is no CPU path here (default - hip)
      -m [completion,passkey,perplexity]   mode, may be abbreviated (default - completion)
      -T <int>           sliding window context length (0 - max): past <int> positions every layer attends
                         to the first two positions (attention sinks, placed as if they lay just behind
                         the window) and to the last <int> - 2, so a text may be longer than <int>
      -i <string>        input prompt           } completion and perplexity:
      -f <filepath>      input file with prompt } exactly one of -i, -f, --tokens
      -t <float>         temperature (default - 1.0; 0 = greedy)
      -n <int>           completion: number of steps (default 256; 0 = max_seq_len, -1 = until the context is full)
                         passkey: number of junk lines (default 250)
      -l <int>           passkey position (-1 - random)
    Additions: --tokens 1,2,3 (prompt as token ids; with --batch-file one prompt a line),
      --batch-file <path>, --seed <int>, --dtype bfloat16|float32, --max-tokens <int>,
      --random <config.json> in place of the folder, --weight-seed <int> (default 0)

Every option takes a value, as in the reference."""
import math
import random
import sys
import time


USAGE = __doc__


def error_usage(msg=None):
    if msg:
        sys.stderr.write("Error: %s\n" % msg)
    sys.stderr.write(USAGE + "\n")
    raise SystemExit(1)


def _prefix_choice(value, choices):
    for c in choices:
        if c.startswith(value) and value:
            return c
    return None


def parse_args(argv):
    if len(argv) < 1 or argv[0] in ("-h", "--help"):
        error_usage()
    positional = not argv[0].startswith("--random")
    a = {"checkpoint": argv[0] if positional else "", "random": "", "weight_seed": 0, "device": "hip", "mode": "completion", "prompt": "", "prompt_path": "",
         "context": 0, "num_steps": 256, "temperature": 1.0, "n_junk": 250, "passkey_pos": -1, "tokens": "",
         "batch_file": "", "seed": None, "dtype": "bfloat16", "max_tokens": 0}
    i = 1 if positional else 0
    long_opts = {"--random": "random", "--weight-seed": "weight_seed", "--tokens": "tokens", "--batch-file": "batch_file", "--seed": "seed", "--dtype": "dtype",
                 "--max-tokens": "max_tokens"}
    while i < len(argv):
        flag = argv[i]
        if i + 1 >= len(argv):
            error_usage("option %s needs a value" % flag)
        val = argv[i + 1]
        if flag in long_opts:
            key = long_opts[flag]
            a[key] = int(val) if key in ("seed", "max_tokens", "weight_seed") else val
        elif len(flag) != 2 or flag[0] != "-":
            error_usage("unknown option %s" % flag)
        elif flag[1] == "h":
            error_usage()
        elif flag[1] == "m":
            a["mode"] = _prefix_choice(val, ["completion", "passkey", "perplexity"]) or error_usage("unknown mode")
        elif flag[1] == "d":
            d = _prefix_choice(val, ["hip", "cuda", "cpu"]) or error_usage("unknown device")
            if d == "cpu":
                error_usage("there is no CPU path in yalm_amd; use -d hip")
            a["device"] = d
        elif flag[1] == "i":
            a["prompt"] = val
        elif flag[1] == "t":
            a["temperature"] = float(val)
        elif flag[1] == "f":
            a["prompt_path"] = val
        elif flag[1] == "T":
            a["context"] = int(val)
        elif flag[1] == "l":
            a["passkey_pos"] = int(val)
        elif flag[1] == "n":
            a["num_steps"] = int(val)
            a["n_junk"] = int(val)
        else:
            error_usage("unknown option %s" % flag)
        i += 2
    if a["dtype"] not in ("bfloat16", "float32"):
        error_usage("--dtype must be bfloat16 or float32")
    if bool(a["random"]) == bool(a["checkpoint"]):
        error_usage("give a model folder or --random <config.json>, not both")
    if a["mode"] in ("completion", "perplexity"):
        given = sum(1 for k in ("prompt", "prompt_path", "tokens", "batch_file") if a[k])
        if a["batch_file"] and a["tokens"] and not a["prompt"] and not a["prompt_path"]:
            given = 1
        if given != 1:
            error_usage("give exactly one of -i, -f, --tokens, --batch-file")
    elif a["passkey_pos"] != -1 and not 0 <= a["passkey_pos"] < a["n_junk"]:
        sys.stderr.write("Error: passkey position must be between 0 and %d\n" % (a["n_junk"] - 1))
        raise SystemExit(1)
    return a


def _load(a):
    import torch
    from .engine import Engine, Model
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a["dtype"]]
    if a["random"]:
        import json
        from .config import config_from_dict
        with open(a["random"]) as f:
            cfg = config_from_dict(json.load(f))
        if a["context"]:
            cfg = cfg.with_context(a["context"])
        return Model.random(cfg, a["weight_seed"], dtype=dtype, device="cuda:0")
    model = Model.from_folder(a["checkpoint"], dtype=dtype, device="cuda:0", context=a["context"])
    return model


def _prompts(a, model):
    """Token-id prompts from -i / -f / --tokens / --batch-file, and the tokenizer if there is one."""
    from .tokenizer import Tokenizer
    cfg = model.spec
    tok = None

    def tokenizer():
        nonlocal tok
        if tok is None:
            if not a["checkpoint"]:
                error_usage("a model made with --random has no tokenizer: give the prompt with --tokens")
            eos = cfg.eos_token_ids[0] if cfg.eos_token_ids else -1
            tok = Tokenizer.from_folder(a["checkpoint"], cfg.vocab_size,
                                        cfg.bos_token_id if cfg.bos_token_id is not None else -1, eos)
        return tok

    def ids(text):
        return [int(t) for t in text.replace(",", " ").split()]

    if a["batch_file"]:
        with open(a["batch_file"]) as f:
            lines = [l.rstrip("\n") for l in f if l.strip()]
        if a["tokens"] in ("ids", "1", "true") or all(c.isdigit() or c in ", " for l in lines for c in l):
            return [ids(l) for l in lines], None
        return [tokenizer().encode(l, True) for l in lines], tokenizer()
    if a["tokens"]:
        return [ids(a["tokens"])], None
    text = a["prompt"]
    if a["prompt_path"]:
        try:
            with open(a["prompt_path"]) as f:
                text = f.read()
        except OSError:
            sys.stderr.write("Error: could not open file %s\n" % a["prompt_path"])
            raise SystemExit(1)
    return [tokenizer().encode(text, True)], tokenizer()


def _engine(a, model, need_tokens, positions=None):
    from .engine import Engine
    budget = a["max_tokens"] or need_tokens
    return Engine(model, max_tokens=max(64, budget), positions=positions if a["context"] else None)


def run_completion(a):
    """src/main.cpp:54-148."""
    from .generate import GenerationStats, generate
    model = _load(a)
    prompts, tok = _prompts(a, model)
    max_len = model.spec.max_positions
    steps = a["num_steps"]
    if steps == 0 or steps == -1:                                   # main.cpp:71-74; -1 ends when the context is full
        steps = max_len
    if a["context"]:                                                # under -T a text may run past the model's positions
        max_len = max(max_len, max(len(p) for p in prompts) + steps)
    held = (a["context"] // 64 + 2) * 64 if a["context"] else max_len      # a window's ring of pages holds no more
    need = sum(min(max_len, len(p) + steps, max(held, len(p))) + 64 for p in prompts)
    engine = _engine(a, model, need, positions=max_len)
    seed = a["seed"] if a["seed"] is not None else int(time.time() * 1000)          # main.cpp:66
    stats = GenerationStats()
    stop = list(model.spec.eos_token_ids)
    if tok is not None and tok.eot_id >= 0:
        stop.append(tok.eot_id)
    last = {i: p[-1] for i, p in enumerate(prompts)}
    single = len(prompts) == 1

    def on_token(i, t):
        if single:
            if tok is not None:
                sys.stdout.buffer.write(tok.decode_one(last[i], t))
            else:
                sys.stdout.write("%d " % t)
            sys.stdout.flush()
        last[i] = t

    print("Model active bytes with full context window: %d" % (
        model.weight_bytes() + sum(g.bytes_per_token() * (g.window or engine.n_positions) for g in engine.cache.kv_groups)))
    # graphs for the decode steps to come are captured before the clock starts (main.cpp:81-85 warms up too)
    shortest, longest = min(len(p) for p in prompts), min(max_len, max(len(p) for p in prompts) + steps)
    sizes = list(range(1, min(len(prompts), engine.cache.n_slots) + 1))
    from .engine import StepError
    try:
        engine.warmup(sizes, min_len=shortest + 1, max_len=longest)
    except StepError:                                   # more bucket pairs than the engine keeps: the full batch only
        engine.warmup(sizes[-1:], min_len=shortest + 1, max_len=min(longest, 2 * shortest + 64))
    t0 = time.perf_counter()
    out = generate(engine, prompts, max_new_tokens=steps, temperature=a["temperature"], seed=seed, stop_ids=stop,
                   on_token=on_token, stats=stats)
    elapsed = time.perf_counter() - t0
    if not single:
        for i, o in enumerate(out):
            text = b"".join(tok.decode_one(p, t) for p, t in zip([prompts[i][-1]] + o[:-1], o)).decode(
                "utf-8", "replace") if tok is not None else " ".join(map(str, o))
            print("[%d] %s" % (i, text))
    total = stats.prompt_tokens + stats.new_tokens
    print("\n\nGeneration stats:\n  %d tokens\n  throughput: %.5gtok/s\n  latency: %.5gs/tok\n  hydrate: %.5gs\n"
          "  bandwidth: %.5gGB/s\n  prefill: %.5gtok/s\n  decode: %.5gtok/s\n  total: %.5gs\n"
          % (total, total / elapsed, elapsed / max(total, 1), stats.prefill_seconds, stats.bytes_read / 1e9 / elapsed,
             stats.prefill_tokens_per_second, stats.decode_tokens_per_second, elapsed))
    return out


def run_perplexity(a):
    """src/main.cpp:150-235: logits at every position, log-probability of the next
    token; ppl = exp(-sum/N), error = ppl * sqrt((ss - sum^2/N)/N/N), N = len - 1."""
    model = _load(a)
    prompts, _ = _prompts(a, model)
    engine = _engine(a, model, max(len(p) + 64 for p in prompts), positions=max(len(p) for p in prompts) + 1)
    results = []
    for p in prompts:
        if len(p) < 2:
            error_usage("perplexity needs at least two tokens")
        if len(p) > engine.n_positions:
            error_usage("the text has %d tokens, the context holds %d: give a window with -T" % (len(p), engine.n_positions))
        t0 = time.perf_counter()
        slots = engine.start(1)
        # the probability of each next token; the logits are made a block of rows at a time
        probs = engine.step(slots, [p], [list(range(len(p) - 1))], targets=[p[1:]]).tolist()
        engine.release(slots)
        elapsed = time.perf_counter() - t0
        N = len(p) - 1
        lps = [math.log(max(q, 1e-45)) for q in probs]
        s, ss = sum(lps), sum(l * l for l in lps)
        ppl = math.exp(-s / N)
        err = ppl * math.sqrt(max(0.0, ss - s * s / N) / N / N)
        print("Stats:\n  %d tokens\n  perplexity: %.5g ± %.5g\n  throughput: %.5gtok/s\n  latency: %.5gs/tok\n"
              "  total: %.5gs\n" % (N, ppl, err, N / elapsed, elapsed / N, elapsed))
        results.append((ppl, err))
    return results


def run_passkey(a):
    """src/main.cpp:237-332: a pass key hidden in filler text, then 16 greedy steps."""
    from .generate import generate
    model = _load(a)
    a2 = dict(a, prompt="x")
    _, tok = _prompts(a2, model)
    rng = random.Random(a["seed"])
    passkey = rng.randrange(50000) + 1
    n_junk = a["n_junk"]
    pos = rng.randrange(n_junk) if a["passkey_pos"] == -1 else a["passkey_pos"]
    text = ("There is an important info hidden inside a lot of irrelevant text. "
            "Find it and memorize them. I will quiz you about the important information there.")
    for i in range(n_junk):
        if i == pos:
            text += " The pass key is %d. Remember it. %d is the pass key." % (passkey, passkey)
        text += " The grass is green. The sky is blue. The sun is yellow. Here we go. There and back again."
    suffix = " What is the pass key? The pass key is"
    text += suffix
    prompt = tok.encode(text, True)
    print("Passkey test:\n  prompt: %d tokens\n  passkey: %d\n  passkey token index: ~%d\n"
          % (len(prompt), passkey, int(pos / n_junk * len(prompt))))
    engine = _engine(a, model, len(prompt) + 64)
    stop = list(model.spec.eos_token_ids) + ([tok.eot_id] if tok.eot_id >= 0 else [])
    sys.stdout.write(suffix)
    last = [prompt[-1]]

    def on_token(i, t):
        sys.stdout.buffer.write(tok.decode_one(last[0], t))
        sys.stdout.flush()
        last[0] = t

    out = generate(engine, [prompt], max_new_tokens=16, temperature=0.0, stop_ids=stop, on_token=on_token)
    print()
    return passkey, out[0]


def main(argv=None):
    a = parse_args(list(sys.argv[1:] if argv is None else argv))
    if a["mode"] == "completion":
        run_completion(a)
    elif a["mode"] == "passkey":
        run_passkey(a)
    else:
        run_perplexity(a)
    return 0
