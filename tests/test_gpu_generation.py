"""Generation through the entry points: greedy tokens against the plain
implementation, temperature sampling with a fixed seed (independent of the
batch), stop tokens and early ends, many batches one after another, long
decoding across pages and past the window, the first tokens of a sequence, and
the command line."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import schedules
import tiny_configs
from plain import reference_model as R

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("gen_models")
    return {name: helpers.make_folder(tmp, name, cfg, seed=6) for name, cfg in tiny_configs.ALL.items()}


def plain_greedy(folder, prompt, n_new, stop=()):
    cfg, w = R.read_folder(folder)
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(R.sample_argmax(R.forward(w, cfg, seq)[-1]))
        if seq[-1] in stop:
            break
    return seq[len(prompt):]


@pytest.mark.parametrize("name", ["tiny_llama", "tiny_mistral", "tiny_wide_heads"])
def test_greedy_generation_matches_the_plain_implementation(folders, name):
    """The tiny Llama workload: prompts of 5, 17 and 1 tokens, then 8 greedy steps (float32); also
    with untied heads, where the next token is not simply the last one again."""
    from yalm_amd import Engine, Model, generate
    model = Model.from_folder(folders[name], dtype=torch.float32, device="cuda:0")
    engine = Engine(model, max_tokens=2048)
    prompts = list(helpers.random_requests(tiny_configs.ALL[name], [5, 17, 1], seed=1).values())
    out = generate(engine, prompts, max_new_tokens=8, temperature=0.0, stop_ids=[])
    for p, o in zip(prompts, out):
        assert o == plain_greedy(folders[name], p, 8)
    # one request at a time gives the same tokens as the batch
    for p, o in zip(prompts, out):
        assert generate(engine, [p], max_new_tokens=8, temperature=0.0, stop_ids=[])[0] == o
    assert not engine.cache.slots.held


def test_temperature_sampling_with_a_fixed_seed(folders):
    """The tiny Mistral workload: prompts of 2, 30, 9, 23 tokens, 20 steps past the window at
    temperature 0.8.  A request's tokens depend on the seed and its id, not on its batch,
    and equal the plain sampler's pick given the same uniform numbers."""
    from yalm_amd import Engine, Model, generate
    from yalm_amd.sampling import uniform
    name = "tiny_mistral"
    model = Model.from_folder(folders[name], dtype=torch.float32, device="cuda:0")
    engine = Engine(model, max_tokens=2048)
    prompts = list(helpers.random_requests(tiny_configs.ALL[name], [2, 30, 9, 23], seed=2).values())
    a = generate(engine, prompts, max_new_tokens=20, temperature=0.8, seed=77, stop_ids=[])
    b = generate(engine, prompts, max_new_tokens=20, temperature=0.8, seed=77, stop_ids=[], batch_size=1)
    assert a == b and all(len(o) == 20 for o in a)
    assert generate(engine, prompts, max_new_tokens=20, temperature=0.8, seed=78, stop_ids=[]) != a
    cfg, w = R.read_folder(folders[name])
    for rid in (0, 2):
        seq = list(prompts[rid])
        agree = 0
        for step in range(20):
            logits = R.forward(w, cfg, seq)[-1]
            u = uniform(77, rid, step)
            want = R.sample_temperature(logits.float(), 0.8, u)
            got = a[rid][step]
            p = torch.softmax(logits / 0.8, 0)
            c = torch.cumsum(p, 0)
            # equal, or u lies on the edge of the picked token's interval of the running sum
            assert got == want or float(c[got] - p[got]) - 1e-4 <= u <= float(c[got]) + 1e-4
            agree += got == want
            seq.append(got)
        assert agree >= 18


def test_stop_tokens_end_a_request_early_and_batches_follow_each_other(folders):
    from yalm_amd import Engine, GenerationStats, Model, generate
    name = "tiny_llama3"
    model = Model.from_folder(folders[name], dtype=torch.bfloat16, device="cuda:0")
    engine = Engine(model, max_tokens=64 * 6, max_batch=3)
    prompts = list(helpers.random_requests(tiny_configs.ALL[name], [3, 40, 9, 1, 22, 5, 64], seed=3).values())
    free = generate(engine, prompts, max_new_tokens=12, temperature=0.0, stop_ids=[])
    # choose as stop token one that request 1 emits at its 4th step
    stop = free[1][3]
    stats = GenerationStats()
    out = generate(engine, prompts, max_new_tokens=12, temperature=0.0, stop_ids=[stop], stats=stats)
    for f, o in zip(free, out):
        cut = f.index(stop) + 1 if stop in f else len(f)
        assert o == f[:cut]                       # the stop token is kept, nothing follows it
    assert len(out[1]) <= 4
    assert stats.batches >= 3 and sum(stats.batch_sizes) == len(prompts) and max(stats.batch_sizes) <= 3
    assert stats.prompt_tokens == sum(map(len, prompts)) and stats.new_tokens == sum(map(len, out))
    assert not engine.cache.slots.held and all(g.pool.n_free == g.n_pages for g in engine.cache.kv_groups)
    # the loop that reads every token before it queues the next step gives the same, in fewer rows of work
    behind = GenerationStats()
    assert generate(engine, prompts, max_new_tokens=12, temperature=0.0, stop_ids=[stop], stats=behind,
                    ahead=False) == out
    assert behind.new_tokens == stats.new_tokens and behind.bytes_read < stats.bytes_read
    assert not engine.cache.slots.held and all(g.pool.n_free == g.n_pages for g in engine.cache.kv_groups)


def test_a_draw_stays_on_the_device_and_is_read_in_time():
    """draw() gives what sample() gives, as a device vector at once and as a list on demand; its host
    buffer is one of four used in turn, and a draw read after four later ones says so."""
    from yalm_amd import Sampler
    gen = torch.Generator().manual_seed(11)
    logits = torch.randn((5, 300), generator=gen).to("cuda:0")
    ids, steps = [3, 1, 4, 1, 5], [0, 7, 2, 9, 9]
    sampler = Sampler(21)
    for temperature in (0.0, 0.7):
        want = Sampler(21).sample(logits, temperature, ids, steps)
        drawn = sampler.draw(logits, temperature, ids, steps)
        assert drawn.tokens.dtype == torch.int32 and drawn.tokens.is_cuda
        assert drawn.tolist() == want == drawn.tokens.tolist()
    first = sampler.draw(logits, 0.0, ids, steps)
    later = [sampler.draw(logits[:2], 0.0, ids[:2], steps[:2]) for _ in range(Sampler.HOST_BUFFERS)]
    with pytest.raises(RuntimeError, match="later draws"):
        first.tolist()
    assert later[-1].tolist() == logits[:2].argmax(1).tolist()
    wide = sampler.draw(torch.randn((200, 50), generator=gen).to("cuda:0"), 0.0, range(200), [0] * 200)
    assert len(wide.tolist()) == 200                  # more rows than a buffer held so far


@pytest.mark.parametrize("use_graphs", [True, False])
def test_a_step_from_the_tokens_on_the_device(folders, use_graphs):
    """step_from takes a step's tokens from the vector of a draw, whole or by rows, and gives the
    logits of the step that is handed the same tokens as a list."""
    from yalm_amd import Engine, Model, Sampler, StepError
    name = "tiny_mistral"
    model = Model.from_folder(folders[name], dtype=torch.bfloat16, device="cuda:0")
    by_list = Engine(model, max_tokens=1024, max_batch=4, use_graphs=use_graphs, positions=160)
    by_device = Engine(model, max_tokens=1024, max_batch=4, use_graphs=use_graphs, positions=160)
    prompts = list(helpers.random_requests(tiny_configs.ALL[name], [7, 61, 30, 2], seed=5).values())
    sampler = Sampler(0)
    a, b = by_list.start(4), by_device.start(4)
    tokens = sampler.argmax(by_list.step(a, prompts))
    drawn = sampler.draw(by_device.step(b, prompts), 0.0, [0, 1, 2, 3], [0] * 4)
    live = [0, 1, 2, 3]                               # the requests that still run
    for step in range(70):                            # past a page's end and the window
        rows = None
        if step in (20, 40):                          # a sequence leaves: the rows of the draw are no longer 0..n-1
            gone = live[1] if step == 20 else live[0]
            rows = [k for k, i in enumerate(live) if i != gone]
            tokens = [tokens[k] for k in rows]
            live = [i for i in live if i != gone]
            by_list.release([a[gone]])
            by_device.release([b[gone]])
        want = by_list.step([a[i] for i in live], [[t] for t in tokens])
        got = by_device.step_from([b[i] for i in live], drawn.tokens, rows)
        assert torch.equal(got, want), step
        tokens = sampler.argmax(want)
        drawn = sampler.draw(got, 0.0, live, [step + 1] * len(live))
        assert drawn.tolist() == tokens
    a, b = [a[i] for i in live], [b[i] for i in live]
    fresh = by_device.start(1)
    with pytest.raises(StepError, match="after its prompt"):
        by_device.step_from(fresh, drawn.tokens[:1])
    with pytest.raises(StepError, match="int32"):
        by_device.step_from(b, drawn.tokens.to(torch.int64))
    with pytest.raises(StepError, match="one row"):
        by_device.step_from(b, drawn.tokens, [0, 2])
    with pytest.raises(StepError, match="one row"):
        by_device.step_from(b, drawn.tokens[:1])
    lengths = [by_device.length(s) for s in b]
    assert lengths == [by_list.length(s) for s in a]                   # a refused step changes nothing


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,prompt_len,total", [("tiny_long", 3, 600), ("tiny_mistral", 2, 64),
                                                   ("tiny_wide_heads", 40, 400)])
def test_long_decoding(folders, name, prompt_len, total, dtype):
    """Hundreds of single-token steps: across many pages, past the window, up to the
    last position of the context."""
    from yalm_amd import Engine, Model
    cfg = tiny_configs.ALL[name]
    toks = helpers.random_requests(cfg, [total], seed=4)["r0"]
    model = Model.from_folder(folders[name], dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=1024)
    steps = schedules.tail_one_by_one({"r0": toks}, total - prompt_len)
    out = schedules.replay_in_process(engine, steps)
    got = schedules.per_request(steps, out, {"r0": toks})["r0"]
    want = helpers.plain_logits(folders[name], tuple(toks), dtype)
    tol = (helpers.F32_TOL if dtype == "float32" else helpers.BF16_MAX_TOL) * max(1.0, np.abs(want).max())
    bad = helpers.first_bad_row(got, want, tol)
    assert bad is None, "first wrong position %d of %d (page %d, row %d)" % (bad, total, bad // 64, bad % 64)
    helpers.check_logits(got, want, dtype, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folders, dtype):
    """Prompts of one and two tokens, and the first decoded tokens after them."""
    from yalm_amd import Engine, Model
    name = "tiny_wide_heads"
    cfg = tiny_configs.ALL[name]
    model = Model.from_folder(folders[name], dtype=helpers.torch_dtype(dtype), device="cuda:0")
    engine = Engine(model, max_tokens=1024)
    requests = helpers.random_requests(cfg, [1, 2, 3, 4], seed=5)
    for steps in (schedules.whole(requests), schedules.tail_one_by_one(requests, 32),
                  schedules.batches(requests, [list(requests)], {r: 1 for r in requests})):
        out = schedules.replay_in_process(engine, steps)
        got = schedules.per_request(steps, out, requests)
        for rid, toks in requests.items():
            helpers.check_logits(got[rid], helpers.plain_logits(folders[name], tuple(toks), dtype), dtype, rid)


def test_a_far_key_decides(folders, tmp_path):
    """Weights made so that the fault would show: the query/key projections of one head
    are scaled up, which makes attention nearly one-hot on single far keys; a kernel
    that loses a page or a position changes the logits visibly."""
    from yalm_amd import Engine, Model
    from yalm_amd.weights import TensorSource, write_file
    import json
    import shutil
    name = "tiny_long"
    src = TensorSource(folders[name])
    t = {n: src.get(n).clone() for n in src.names()}
    for l in range(2):
        t["model.layers.%d.self_attn.q_proj.weight" % l][:64] *= 6.0
        t["model.layers.%d.self_attn.k_proj.weight" % l] *= 6.0
    folder = str(tmp_path / "sharp")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"), t)
    shutil.copy(os.path.join(folders[name], "config.json"), folder)
    toks = helpers.random_requests(tiny_configs.ALL[name], [900], seed=6)["r0"]
    cfg, w = R.read_folder(folder)
    want = R.forward(w, cfg, toks).float().numpy()
    model = Model.from_folder(folder, dtype=torch.float32, device="cuda:0")
    engine = Engine(model, max_tokens=1024)
    for steps in (schedules.whole({"r0": toks}), schedules.tail_one_by_one({"r0": toks}, 40)):
        got = schedules.per_request(steps, schedules.replay_in_process(engine, steps), {"r0": toks})["r0"]
        helpers.check_logits(got, want, "float32", "sharp attention")


def test_step_refuses_what_it_cannot_do(folders):
    from yalm_amd import Engine, Model, StepError
    model = Model.from_folder(folders["tiny_llama"], dtype=torch.float32, device="cuda:0")
    engine = Engine(model, max_tokens=128, max_batch=2)
    s = engine.start(2)
    with pytest.raises(StepError, match="vocabulary"):
        engine.step(s, [[1, 999], [2]])
    engine.step(s, [[1, 2, 3], [4]])
    with pytest.raises(StepError, match="either all start"):
        engine.step(s, [[1, 2], [3]])                      # a continuation by more than one token
    # the cache holds 128 tokens = 2 pages and both are taken: growing into a third page is refused
    for _ in range(61):
        engine.step([s[0]], [[5]])
    assert engine.length(s[0]) == 64
    with pytest.raises(StepError, match="cache pages"):
        engine.step([s[0]], [[5]])
    assert engine.length(s[0]) == 64                       # nothing changed
    engine.release(s)
    with pytest.raises(StepError, match="not held"):
        engine.step(s, [[1], [2]])
    on_cpu = Model.from_folder(folders["tiny_llama"], dtype=torch.float32, device="cpu")
    with pytest.raises(RuntimeError, match="no CPU path"):
        Engine(on_cpu, max_tokens=64)


def generated(stdout):
    """The token ids a completion printed: what stands between the first line and the statistics."""
    return stdout.split("\n\n")[0].split("\n", 1)[1].split()


def test_command_line(folders):
    """python -m yalm_amd <folder> in the reference's manner: completion with token ids,
    greedy; and perplexity of a token sequence against the plain implementation."""
    folder = folders["tiny_llama"]
    prompt = [1, 17, 200, 33, 5]
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-m", "c", "--tokens", ",".join(map(str, prompt)),
                        "-n", "6", "-t", "0", "--dtype", "float32"], cwd=ROOT, stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    assert p.stdout.startswith("Model active bytes with full context window: ")
    first = generated(p.stdout)
    want = plain_greedy(folder, prompt, 6, stop=(2,))
    assert [int(t) for t in first] == want
    assert "Generation stats:" in p.stdout and "throughput:" in p.stdout and "bandwidth:" in p.stdout
    # the same model made from its configuration and seed alone, without a folder
    p = subprocess.run([sys.executable, "-m", "yalm_amd", "--random", os.path.join(folder, "config.json"),
                        "--weight-seed", "6", "--tokens", ",".join(map(str, prompt)), "-n", "6", "-t", "0", "--dtype",
                        "float32"], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    assert [int(t) for t in generated(p.stdout)] == want
    toks = helpers.random_requests(tiny_configs.TINY_LLAMA, [30], seed=7)["r0"]
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-m", "perp", "--tokens", " ".join(map(str, toks)),
                        "--dtype", "float32"], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                       timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    cfg, w = R.read_folder(folder)
    ppl, err = R.perplexity(R.forward(w, cfg, toks), toks)
    line = [l for l in p.stdout.splitlines() if "perplexity:" in l][0]
    got = float(line.split()[1])
    assert abs(got - ppl) <= 2e-3 * ppl
    bad = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-d", "cpu", "--tokens", "1"], cwd=ROOT,
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert bad.returncode == 1 and "no CPU path" in bad.stderr


def test_a_context_shorter_than_the_text(folders):
    """The reference's -T <n>: the first two positions stay as sinks beside the last n - 2.  Greedy
    generation far past a context of 24 through the Python entry point and through the command line,
    against the plain implementation with the same sinks and window."""
    from yalm_amd import Engine, Model, StepError, generate
    folder = folders["tiny_mistral"]             # an untied head: the next token is not simply the last one again;
    cfg, w = R.read_folder(folder)               # 64 positions of its own, which the text runs past
    prompt = [1, 17, 200, 33, 5]
    n_new, context = 90, 24

    def plain(seq):
        return R.forward(w, cfg, seq, window_override=context - 2, sinks_override=2)

    want = []
    seq = list(prompt)
    for _ in range(n_new):
        want.append(R.sample_argmax(plain(seq)[-1]))
        seq.append(want[-1])
    unlimited, seq = [], list(prompt)            # every key visible: the same up to the context's end, then another text
    for _ in range(60):
        unlimited.append(R.sample_argmax(R.forward(w, cfg, seq, window_override=0)[-1]))
        seq.append(unlimited[-1])
    assert want[:context - len(prompt)] == unlimited[:context - len(prompt)] and want[:60] != unlimited
    model = Model.from_folder(folder, dtype=torch.float32, device="cuda:0", context=context)
    with pytest.raises(StepError, match="window"):            # without a window on every attention: the model's positions
        Engine(Model.from_folder(folders["tiny_llama"], dtype=torch.float32, device="cuda:0"), max_tokens=512,
               positions=1000)
    engine = Engine(model, max_tokens=512, positions=len(prompt) + n_new + 1)
    assert engine.n_positions == len(prompt) + n_new + 1 > cfg["max_position_embeddings"]
    assert generate(engine, [prompt], max_new_tokens=n_new, temperature=0.0, stop_ids=[])[0] == want
    # a prompt that is itself longer than the context, with company
    long_prompt = prompt + want[:50]
    out = generate(engine, [long_prompt, prompt], max_new_tokens=n_new - 50, temperature=0.0, stop_ids=[])
    assert out[0] == want[50:] and out[1] == want[:n_new - 50]
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "--tokens", ",".join(map(str, prompt)), "-n",
                        str(n_new), "-t", "0", "-T", str(context), "--dtype", "float32"], cwd=ROOT,
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    stop_at = want.index(2) + 1 if 2 in want else len(want)          # the command line stops at the end token
    assert [int(t) for t in generated(p.stdout)] == want[:stop_at]


def test_command_line_with_a_tokenizer(folders, tmp_path):
    """Text prompts and the passkey mode (src/main.cpp:237-332) need tokenizer.json: a byte-level one with a
    few words is written next to the random model; what the program prints is the plain implementation's
    greedy continuation, decoded."""
    import json
    import shutil
    from yalm_amd.tokenizer import Tokenizer
    name = "tiny_wide_heads"
    cfg = tiny_configs.ALL[name]
    folder = str(tmp_path / "with_tokenizer")
    shutil.copytree(folders[name], folder)
    vocab = {"<unk>": 0, "<s>": 1, "</s>": 2}
    for i in range(256):
        vocab["<0x%02X>" % i] = 3 + i
    for i, t in enumerate(["\u2581The", "\u2581pass", "\u2581key", "\u2581is", "\u2581the", "\u2581green", "."]):
        vocab[t] = 259 + i
    assert max(vocab.values()) < cfg["vocab_size"]
    with open(os.path.join(folder, "tokenizer.json"), "w") as f:
        json.dump({"model": {"vocab": vocab, "byte_fallback": True}, "added_tokens": []}, f)
    tok = Tokenizer.from_folder(folder, cfg["vocab_size"], cfg["bos_token_id"], cfg["eos_token_id"])

    def printed(tokens, last):
        out = b""
        for t in tokens:
            out += tok.decode_one(last, t)
            last = t
        return out

    text = "The pass key is green."
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-i", text, "-n", "5", "-t", "0", "--dtype", "float32"],
                       cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    prompt = tok.encode(text, True)
    assert prompt[:6] == [1, 3 + ord("T"), 3 + ord("h"), 3 + ord("e"), 260, 261]     # no space is put before the text
    want = plain_greedy(folder, prompt, 5, stop=(cfg["eos_token_id"],))
    shown = p.stdout.split(b"\n", 1)[1]                    # behind the line about the model's active bytes
    assert shown.startswith(printed(want, prompt[-1])), (shown[:80], printed(want, prompt[-1]))

    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-m", "passkey", "-n", "2", "-l", "1", "--seed", "4",
                        "--dtype", "float32"], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    out = p.stdout.decode("utf-8", "replace")
    assert "Passkey test:" in out and "passkey:" in out and " What is the pass key? The pass key is" in out
