"""The generation loop above the step function (src/main.cpp:104-129 for many
requests): batches of unequal prompts, whole prompts in the first step, then
one token a step for every sequence that still runs; a sequence ends when it
samples a stop token (which is kept, src/main.cpp:120-126), has its number of
new tokens, or fills the context; it leaves the batch at once and its slot and
pages go back to the cache; when a batch has drained the next one starts, as
many as there are requests."""
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
             sampler=None, on_token=None, stats=None, request_ids=None):
    """Generates for every prompt (a list of token ids).  Returns the new tokens of
    each request, in the order of the prompts.  stop_ids None means the model's own
    (config eos); on_token(request index, token) is called for every new token."""
    from .sampling import Sampler
    sampler = sampler or Sampler(seed)
    stats = stats if stats is not None else GenerationStats()
    if stop_ids is None:
        stop_ids = list(getattr(engine.model.spec, "eos_token_ids", []) or [])
    stop = set(stop_ids)
    ids = list(request_ids) if request_ids is not None else list(range(len(prompts)))
    max_len = engine.n_positions
    step_bytes = getattr(engine, "step_bytes", lambda slots: 0)
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
            tokens = sampler.sample(logits, temperature, [ids[i] for i, _ in live], [0] * len(live))
            stats.prefill_seconds += time.perf_counter() - t0
            stats.prompt_tokens += sum(len(prompts[i]) for i in batch)
            stats.batches_first_tokens += len(batch)
            t0 = time.perf_counter()
            while True:
                still = []
                ended = []
                for (i, slot), tok in zip(live, tokens):
                    results[i].append(tok)
                    stats.new_tokens += 1
                    if on_token is not None:
                        on_token(i, tok)
                    full = len(prompts[i]) + len(results[i]) >= max_len        # no room for the token just sampled
                    if tok in stop or len(results[i]) >= max_new_tokens or full:
                        ended.append(slot)
                    else:
                        still.append((i, slot))
                if ended:
                    engine.release(ended)
                    held.difference_update(ended)
                live = still
                if not live:
                    break
                logits = engine.step([s for _, s in live], [[results[i][-1]] for i, _ in live])
                stats.bytes_read += step_bytes([s for _, s in live])
                tokens = sampler.sample(logits, temperature, [ids[i] for i, _ in live],
                                        [len(results[i]) for i, _ in live])
                stats.decode_steps += 1
        except BaseException:
            engine.release(sorted(held))                  # a failed batch gives back what it still holds
            raise
        stats.decode_seconds += time.perf_counter() - t0
    return results
