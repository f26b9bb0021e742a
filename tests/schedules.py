"""Ways of cutting the same requests into steps, in the record format that
bin/trace_run reads, and the means to replay them (in this process through the
engine, or through bin/trace_run) and to put the logits back together per
request and position."""
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def whole(requests):
    """Each request alone, all its tokens in one step."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(toks),
                                                       "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_one_by_one(requests, tail=32):
    """Each request alone: all but the last `tail` tokens in one step (at least one),
    the rest one by one."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        first = max(1, len(toks) - tail)
        rest = toks[first:]
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:first],
                                                       "want": list(range(first))}],
                      "end": [] if rest else [rid]})
        for i, t in enumerate(rest):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [t], "want": [0]}],
                          "end": [rid] if i == len(rest) - 1 else []})
    return steps


def batches(requests, groups, prompt_lens):
    """Batches of unequal lengths, one after another.  groups: lists of request ids;
    prompt_lens[rid]: tokens of the request's first step; the rest follows one
    token a step; a request that has no tokens left ends and leaves the batch."""
    steps = []
    for group in groups:
        pos = {}
        entries = []
        for rid in group:
            p = prompt_lens[rid]
            entries.append({"id": rid, "tokens": list(requests[rid][:p]), "want": list(range(p))})
            pos[rid] = p
        live = list(group)
        while True:
            done = [rid for rid in live if pos[rid] >= len(requests[rid])]
            steps.append({"step": len(steps), "entries": entries, "end": done})
            live = [rid for rid in live if rid not in done]
            if not live:
                break
            entries = []
            for rid in live:
                entries.append({"id": rid, "tokens": [requests[rid][pos[rid]]], "want": [0]})
                pos[rid] += 1
    return steps


def interleaved(requests, groups, prompt_lens, start_at):
    """Batches that overlap in time: group g's first step is step number start_at[g] of the merged
    trace at the earliest, and from then on the live groups take turns, a step each.  Every step
    still belongs to one batch (its requests all start or all go on by one token); a later batch
    starts while sequences of earlier ones are still live, and takes the slots and pages that
    their leavers gave back."""
    per_group = [batches(requests, [g], prompt_lens) for g in groups]
    cursor = [0] * len(groups)
    steps = []
    while any(c < len(p) for c, p in zip(cursor, per_group)):
        progressed = False
        for g, plan in enumerate(per_group):
            if cursor[g] < len(plan) and len(steps) >= start_at[g]:
                s = dict(plan[cursor[g]], step=len(steps))
                steps.append(s)
                cursor[g] += 1
                progressed = True
        if not progressed:                    # nothing live yet and the next group starts later: it starts now
            g = min((g for g in range(len(groups)) if cursor[g] < len(per_group[g])), key=lambda g: start_at[g])
            start_at = list(start_at)
            start_at[g] = len(steps)
    return steps


def max_tokens_needed(steps):
    """The most tokens live requests hold at any time, each rounded up to 64."""
    held, worst = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum((n + 63) // 64 * 64 for n in held.values()))
        for rid in s["end"]:
            del held[rid]
    return worst


def replay_in_process(engine, steps, before_step=None):
    """Drives Engine.step as bin/trace_run does; returns {step: float32 array [wanted, vocab]}."""
    out = {}
    slot_of = {}
    for s in steps:
        if before_step is not None:
            before_step(s)
        entries = s["entries"]
        new = [e["id"] for e in entries if e["id"] not in slot_of]
        if new:
            assert len(new) == len(entries)
            for rid, slot in zip(new, engine.start(len(new))):
                slot_of[rid] = slot
        logits = engine.step([slot_of[e["id"]] for e in entries], [e["tokens"] for e in entries],
                             [e["want"] for e in entries])
        if logits.shape[0]:
            out[s["step"]] = logits.float().cpu().numpy().copy()
        engine.release([slot_of.pop(rid) for rid in s["end"]])
    return out


def replay_trace_run(folder, dtype, steps, out_dir, max_tokens, extra_args=(), env=None):
    """Runs bin/trace_run as a user would; returns {step: array}."""
    os.makedirs(out_dir, exist_ok=True)
    text = "".join(json.dumps(s) + "\n" for s in steps)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out",
           out_dir, "--max-tokens", str(max_tokens)] + list(extra_args)
    p = subprocess.run(cmd, input=text, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600,
                       env=env)
    assert p.returncode == 0, "trace_run failed (%d):\n%s\n%s" % (p.returncode, p.stdout[-2000:], p.stderr[-4000:])
    done = [l for l in p.stdout.splitlines() if l.startswith("done ")]
    assert [l.split()[1] for l in done] == [str(s["step"]) for s in steps], p.stdout[-2000:]
    out = {}
    for s in steps:
        f = os.path.join(out_dir, "%s.f32" % s["step"])
        n = sum(len(e["want"]) for e in s["entries"])
        if n:
            out[s["step"]] = np.fromfile(f, dtype="<f4").reshape(n, -1)
        else:
            assert not os.path.exists(f)
    return out


def per_request(steps, outputs, requests):
    """{rid: array [len, vocab]} from the step outputs (every position must have been wanted once)."""
    vocab = next(iter(outputs.values())).shape[1]
    res = {rid: np.full((len(t), vocab), np.nan, dtype=np.float32) for rid, t in requests.items()}
    pos = {rid: 0 for rid in requests}
    for s in steps:
        row = 0
        for e in s["entries"]:
            for j in e["want"]:
                res[e["id"]][pos[e["id"]] + j] = outputs[s["step"]][row]
                row += 1
            pos[e["id"]] += len(e["tokens"])
    return res
