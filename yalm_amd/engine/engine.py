"""The step function and what it stands on.

`Engine.step` takes a batch of sequences that started together: in their first
step each brings its whole prompt (unequal lengths, packed, no padding), in
every later step each still-running sequence brings one token.  It runs only
the tokens it is given, as one batch, from the cache that earlier steps left,
and returns float32 logits at the wanted places.  The reference's
Model::forward(state, token, pos, mode) (src/model.cpp:417-428) is the case of
one sequence and one token.

Decode steps are replayed from a HIP graph per batch-size bucket: the kernels
read positions, lengths, slots and block tables from device memory, so the
graph needs no patching from step to step (the reference patches kernel nodes
every step, src/infer.cu:1225-1247).  Rows that pad a batch to its bucket
carry slot -1 and change no result."""
import numpy as np
import torch

from ..cache.manager import PAGE, CacheError, CacheManager
from ..ops import kernels, library
from .context import StepContext, Workspace

DECODE_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 96, 128, 192, 256, 512, 1024)


class StepError(ValueError):
    pass


class _DecodeGraph:
    """A captured decode step for one bucket size, with its own buffers."""

    def __init__(self, engine, bucket):
        self.bucket = bucket
        self.ws = Workspace(engine.device)
        n_meta = 6 * bucket + 1
        self.meta_host = torch.empty(n_meta, dtype=torch.int32, pin_memory=True)
        self.meta = torch.zeros(n_meta, dtype=torch.int32, device=engine.device)
        self.logits = torch.empty((bucket, engine.model.vocab_size), dtype=torch.float32, device=engine.device)
        self.graph = None
        self.ctx = engine._context("decode", self.ws, self.meta, bucket, bucket, 0)
        self.copied = None            # event after the last upload of meta_host


class Engine:
    def __init__(self, model, max_tokens, max_batch=None, use_graphs=True):
        if model.device is None:
            raise StepError("the model has no weights yet")
        if model.device.type != "cuda":
            raise RuntimeError("yalm_amd runs on the GPU only (device %s given); there is no CPU path" % model.device)
        library.lib()                                   # fails loudly here if the kernels are missing
        self.model = model
        self.device = model.device
        self.dtype = model.compute_dtype
        self.cache = CacheManager(model.cache_requests(), max_tokens, model.spec.max_positions, self.dtype,
                                  self.device, n_slots=max_batch)
        n_positions = model.spec.max_positions if self.cache.unbounded else \
            min(model.spec.max_positions, self.cache.max_seq_len)
        self.n_positions = n_positions
        model.prepare(n_positions)
        self.ws = Workspace(self.device)
        self.use_graphs = use_graphs
        self._graph_safe = model.graph_safe()          # the parts are fixed from here on: asked once, not every step
        self._graphs = {}
        self._meta_host = None

    # ------------------------------------------------------------------ sequences
    def start(self, n):
        """Slots for n sequences that start together."""
        return self.cache.acquire(n)

    def release(self, slots):
        """Gives back what finished sequences hold."""
        self.cache.release(list(slots))

    def length(self, slot):
        return self.cache.seq_len[slot]

    # ------------------------------------------------------------------ the step
    def _context(self, mode, ws, meta, T, B, max_position):
        ctx = StepContext(mode, self.cache, ws, self.dtype, self.model.shared_lines)
        ctx.tokens = meta[0:T]
        ctx.tok_seq = meta[T:2 * T]
        ctx.tok_pos = meta[2 * T:3 * T]
        o = 3 * T
        ctx.seq_slot = meta[o:o + B]
        ctx.seq_len = meta[o + B:o + 2 * B]
        ctx.cu_seqlens = meta[o + 2 * B:o + 3 * B + 1]
        ctx.max_position = max_position
        return ctx

    def step(self, slots, tokens, want=None):
        """slots: the sequences of the batch that take part in this step;
        tokens[i]: the next tokens of slots[i]; want[i]: indices into tokens[i] whose
        logits are asked for (default: the last).  Returns float32 [n_wanted, vocab]
        on the device, in the order of the slots and of want; the tensor is valid
        until the next step."""
        B = len(slots)
        if B == 0:
            raise StepError("a step needs at least one sequence")
        if len(tokens) != B or (want is not None and len(want) != B):
            raise StepError("slots, tokens and want must have the same length")
        if len(set(slots)) != B:
            raise StepError("a slot occurs twice in the step")
        n_tok = [len(t) for t in tokens]
        if min(n_tok) < 1:
            raise StepError("every sequence of a step brings at least one token")
        starts = []
        for s in slots:
            if not self.cache.slots.is_held(s):
                raise StepError("slot %r is not held by a live sequence" % (s,))
            starts.append(self.cache.seq_len[s])
        V = self.model.vocab_size
        if max(n_tok) == 1:                               # a decode step: one comparison pair for the batch
            firsts = [t[0] for t in tokens]
            if not (0 <= min(firsts) and max(firsts) < V):
                bad = [tok for tok in firsts if not 0 <= tok < V]
                raise StepError("token id %r is outside the vocabulary of %d" % (bad[0] if bad else firsts, V))
        else:
            for t in tokens:
                ids = np.asarray(t, dtype=np.int64)
                if ids.ndim != 1 or ids.min() < 0 or ids.max() >= V:
                    bad = [tok for tok in t if not 0 <= tok < V]
                    raise StepError("token id %r is outside the vocabulary of %d" % (bad[0] if bad else t, V))
        if want is None:
            want = [[n - 1] for n in n_tok]
        for w, n in zip(want, n_tok):
            for j in w:
                if not 0 <= j < n:
                    raise StepError("wanted place %r is outside the %d tokens of its sequence" % (j, n))
        if all(s == 0 for s in starts):
            mode = "prefill"
        elif all(n == 1 for n in n_tok):
            mode = "decode"
        else:
            raise StepError("the sequences of a step either all start at their first token or all go on by one "
                            "token (lengths so far %s, tokens brought %s)" % (starts, n_tok))
        max_pos = max(s + n for s, n in zip(starts, n_tok)) - 1
        if max_pos >= self.n_positions:
            raise StepError("position %d is beyond the %d positions of this engine (max_position_embeddings / "
                            "max_tokens)" % (max_pos, self.n_positions))
        try:
            new_lens = self.cache.extend(slots, n_tok)
        except CacheError as e:
            raise StepError(str(e)) from None
        if mode == "decode":
            return self._decode(slots, tokens, want, starts, new_lens)
        return self._prefill(slots, tokens, want, n_tok, new_lens)

    def _prefill(self, slots, tokens, want, n_tok, new_lens):
        B, T = len(slots), sum(n_tok)
        rows = []
        cu = np.zeros(B + 1, dtype=np.int32)
        np.cumsum(n_tok, out=cu[1:])
        for i, w in enumerate(want):
            rows.extend(int(cu[i]) + j for j in w)
        R = len(rows)
        tile0 = np.zeros(B + 1, dtype=np.int32)
        np.cumsum([(n + PAGE - 1) // PAGE for n in n_tok], out=tile0[1:])
        order = kernels.prefill_tile_order(n_tok)
        n_meta = 3 * T + 4 * B + 2 + R + len(order)
        host = np.empty(n_meta, dtype=np.int32)
        host[0:T] = np.concatenate([np.asarray(t, dtype=np.int32) for t in tokens])
        host[T:2 * T] = np.repeat(np.arange(B, dtype=np.int32), n_tok)
        host[2 * T:3 * T] = np.concatenate([np.arange(n, dtype=np.int32) for n in n_tok])
        o = 3 * T
        host[o:o + B] = slots
        host[o + B:o + 2 * B] = new_lens
        host[o + 2 * B:o + 3 * B + 1] = cu
        host[o + 3 * B + 1:o + 4 * B + 2] = tile0
        host[o + 4 * B + 2:o + 4 * B + 2 + R] = rows
        host[o + 4 * B + 2 + R:] = order
        meta = self.ws.get("meta", (n_meta,), torch.int32)
        meta.copy_(torch.from_numpy(host))
        ctx = self._context("prefill", self.ws, meta, T, B, max(n_tok) - 1)
        ctx.seq_tile0 = meta[o + 3 * B + 1:o + 4 * B + 2]
        ctx.tile_order = meta[o + 4 * B + 2 + R:]
        ctx.n_tiles = int(tile0[-1])
        ctx.host_slots, ctx.host_n_tokens, ctx.host_start = list(slots), list(n_tok), [0] * B
        logits = self.ws.get("logits", (R, self.model.vocab_size), torch.float32) if R else None
        self.model.forward(ctx, meta[o + 4 * B + 2:o + 4 * B + 2 + R] if R else None, logits)
        return logits if R else torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)

    def _bucket(self, B):
        for b in DECODE_BUCKETS:
            if b >= B:
                return b
        return B

    def _decode(self, slots, tokens, want, starts, new_lens):
        B = len(slots)
        use_graph = self.use_graphs and self._graph_safe
        Bk = self._bucket(B) if use_graph else B
        # launch shapes may depend on the longest sequence only through this bucket (a power of
        # two of pages), so that a captured graph stays valid until a sequence outgrows it
        pages_bucket = 1
        while pages_bucket * PAGE < max(new_lens):
            pages_bucket *= 2
        g = self._graphs.get((Bk, pages_bucket)) if use_graph else None
        if use_graph and g is None:
            g = _DecodeGraph(self, Bk)
            g.ctx.pages_bucket = pages_bucket
            self._graphs[(Bk, pages_bucket)] = g
        if g is not None:
            if g.copied is not None:
                g.copied.synchronize()                   # the last upload has read the pinned buffer
            host = g.meta_host.numpy()
        else:
            host = np.empty(6 * Bk + 1, dtype=np.int32)
        host[0:Bk] = -1
        host[0:B] = [t[0] for t in tokens]
        host[Bk:2 * Bk] = np.arange(Bk, dtype=np.int32)
        host[2 * Bk:3 * Bk] = 0
        host[2 * Bk:2 * Bk + B] = starts
        host[3 * Bk:4 * Bk] = -1
        host[3 * Bk:3 * Bk + B] = slots
        host[4 * Bk:5 * Bk] = 0
        host[4 * Bk:4 * Bk + B] = new_lens
        host[5 * Bk:6 * Bk + 1] = np.arange(Bk + 1, dtype=np.int32)
        rows = [i for i, w in enumerate(want) if len(w) > 0]
        if g is None:
            meta = self.ws.get("meta", (6 * Bk + 1,), torch.int32)
            meta.copy_(torch.from_numpy(host))
            ctx = self._context("decode", self.ws, meta, Bk, Bk, max(starts))
            ctx.pages_bucket = pages_bucket
            ctx.host_slots, ctx.host_n_tokens, ctx.host_start = list(slots), [1] * B, list(starts)
            logits = self.ws.get("logits", (Bk, self.model.vocab_size), torch.float32)
            self.model.forward(ctx, None, logits)                     # every row
        else:
            g.meta.copy_(g.meta_host, non_blocking=True)
            if g.copied is None:
                g.copied = torch.cuda.Event()
            g.copied.record()
            g.ctx.max_position = max(starts)
            if g.graph is None:
                self._capture(g)
            g.graph.replay()
            logits = g.logits
        if rows == list(range(B)):
            return logits[:B]
        if not rows:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return logits[torch.tensor(rows, device=self.device)]

    def _capture(self, g):
        """Runs the step once eagerly on the graph's buffers (every buffer gets its
        size), then captures it."""
        self.model.forward(g.ctx, None, g.logits)
        torch.cuda.synchronize(self.device)
        g.ws.frozen = True
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.model.forward(g.ctx, None, g.logits)
        g.graph = graph

    def synchronize(self):
        torch.cuda.synchronize(self.device)
