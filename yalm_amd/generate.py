"""The generation loop above the step function (src/main.cpp:104-129 for many
requests): batches of unequal prompts, whole prompts in the first step, then
one token a step for every sequence that still runs; a sequence ends when it
samples a stop token (which is kept, src/main.cpp:120-126), has its number of
new tokens, or fills the context; it leaves the batch and its slot and pages go
back to the cache; when a batch has drained the next one starts, as many as
there are requests.

The loop runs one step ahead of the host where the engine and the sampler allow
it: a step's tokens stay on the device and feed the next step from there, and
the host reads them while that step runs, so the device never waits for the
host between two steps.  A sequence that samples a stop token is then seen one
step late: it has taken part in one more step, whose token is dropped.  The one
place where the host does wait is the end of a batch's prompt step, so that the
time of the prompt and the time of decoding are told apart on the device's clock
(src/main.cpp:133-147 reports them so)."""
import time
from dataclasses import dataclass, field
from typing import List

from .cache.manager import PAGE, pages_for


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    new_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    decode_steps: int = 0
    batches: int = 0
    batch_sizes: List[int] = field(default_factory=list)
    batches_first_tokens: int = 0          # tokens sampled from prefill logits (not decode steps)
    bytes_read: int = 0                    # what the steps had to read: weights once a step, live keys and values

    @property
    def prefill_tokens_per_second(self):
        return self.prompt_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_tokens_per_second(self):
        n = self.new_tokens - self.batches_first_tokens
        return n / self.decode_seconds if self.decode_seconds > 0 else 0.0


def plan_batches(prompt_lens, max_new_tokens, batch_size, max_tokens, n_slots, max_seq_len):
    """Splits the requests (in order) into batches that fit the cache: at most
    batch_size and n_slots sequences, and pages for every sequence at its longest
    (prompt + new tokens, capped by the context).  Returns lists of indices."""
    limit = max(1, min(batch_size or n_slots, n_slots))
    budget = pages_for(max_tokens)
    out, cur, used = [], [], 0
    for i, n in enumerate(prompt_lens):
        if n < 1:
            raise ValueError("request %d has an empty prompt" % i)
        if n > max_seq_len:
            raise ValueError("request %d: a prompt of %d tokens does not fit the context of %d" % (i, n, max_seq_len))
        need = pages_for(min(n + max_new_tokens, max_seq_len))
        if need > budget:
            raise ValueError("request %d needs %d tokens of cache, the engine holds %d"
                             % (i, need * PAGE, budget * PAGE))
        if cur and (len(cur) >= limit or used + need > budget):
            out.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        out.append(cur)
    return out


def generate(engine, prompts, max_new_tokens=256, temperature=0.0, seed=0, stop_ids=None, batch_size=None,
             sampler=None, on_token=None, stats=None, request_ids=None, ahead=None):
    """Generates for every prompt (a list of token ids).  Returns the new tokens of
    each request, in the order of the prompts.  stop_ids None means the model's own
    (config eos); on_token(request index, token) is called for every new token.
    ahead: queue each step before the host has read the tokens of the step before
    (default: if the engine has step_from and the sampler has draw).  A request that has ended
    leaves the batch a step later then, so a step may run with another number of rows and take other
    kernels: in float32 the tokens are the same either way, in bfloat16 up to choices between logits
    that lie within rounding of each other."""
    from .sampling import Sampler
    sampler = sampler or Sampler(seed)
    stats = stats if stats is not None else GenerationStats()
    if stop_ids is None:
        stop_ids = list(getattr(engine.model.spec, "eos_token_ids", []) or [])
    stop = set(stop_ids)
    ids = list(request_ids) if request_ids is not None else list(range(len(prompts)))
    max_len = engine.n_positions
    step_bytes = getattr(engine, "step_bytes", lambda slots: 0)
    can_ahead = hasattr(engine, "step_from") and hasattr(sampler, "draw")
    if ahead is None:
        ahead = can_ahead
    elif ahead and not can_ahead:
        raise ValueError("running a step ahead needs an engine with step_from and a sampler with draw")
    results = [[] for _ in prompts]
    if max_new_tokens <= 0 or not prompts:
        return results
    plan = plan_batches([len(p) for p in prompts], max_new_tokens, batch_size, engine.cache.n_pages * PAGE,
                        engine.cache.n_slots, max_len)
    for batch in plan:
        stats.batches += 1
        stats.batch_sizes.append(len(batch))
        slots = engine.start(len(batch))
        live = list(zip(batch, slots))
        held = set(slots)
        try:
            t0 = time.perf_counter()
            logits = engine.step(slots, [prompts[i] for i in batch])
            stats.bytes_read += step_bytes(slots)
            landed = None
            if ahead:
                drawn = sampler.draw(logits, temperature, [ids[i] for i, _ in live], [0] * len(live))
                tokens = None
                landed = drawn.tolist()                   # waits for the prompt step: its clock stops on the device's time
            else:
                tokens = sampler.sample(logits, temperature, [ids[i] for i, _ in live], [0] * len(live))
            stats.prefill_seconds += time.perf_counter() - t0
            stats.prompt_tokens += sum(len(prompts[i]) for i in batch)
            stats.batches_first_tokens += len(batch)
            t0 = time.perf_counter()
            rows = list(range(len(live)))                 # where each live sequence's token lies in the last draw
            while live:
                # who goes on: by the counts alone when the tokens are not read yet
                going, going_rows = [], []
                for (i, slot), r in zip(live, rows):
                    n = len(results[i]) + 1               # with the token just sampled
                    if n < max_new_tokens and len(prompts[i]) + n < max_len and (ahead or tokens[r] not in stop):
                        going.append((i, slot))
                        going_rows.append(r)
                next_drawn = next_tokens = None
                if going:
                    going_slots = [s for _, s in going]
                    if ahead:
                        logits = engine.step_from(going_slots, drawn.tokens, going_rows)
                    else:
                        logits = engine.step(going_slots, [[tokens[r]] for r in going_rows])
                    stats.bytes_read += step_bytes(going_slots)
                    stats.decode_steps += 1
                    draw_ids = [ids[i] for i, _ in going]
                    draw_steps = [len(results[i]) + 1 for i, _ in going]
                    if ahead:
                        next_drawn = sampler.draw(logits, temperature, draw_ids, draw_steps)
                if ahead:                                 # lands while the step just queued runs (a batch's first
                    tokens = drawn.tolist() if landed is None else landed       # draw was read with the prompt step)
                    landed = None
                still, still_rows, ended = [], [], []
                k = 0                                     # walks `going`, which keeps the order of `live`
                for (i, slot), r in zip(live, rows):
                    tok = tokens[r]
                    results[i].append(tok)
                    stats.new_tokens += 1
                    if on_token is not None:
                        on_token(i, tok)
                    if k < len(going) and going[k][0] == i:
                        if tok in stop:                   # seen a step late: its row of the next draw is dropped
                            ended.append(slot)
                        else:
                            still.append((i, slot))
                            still_rows.append(k)
                        k += 1
                    else:
                        ended.append(slot)
                if ended:
                    engine.release(ended)
                    held.difference_update(ended)
                if going and not ahead:                   # sampled only now: the tokens just appended are not in it
                    next_tokens = sampler.sample(logits, temperature, draw_ids, draw_steps)
                live, rows, drawn, tokens = still, still_rows, next_drawn, next_tokens
        except BaseException:
            engine.release(sorted(held))                  # a failed batch gives back what it still holds
            raise
        stats.decode_seconds += time.perf_counter() - t0
    return results
