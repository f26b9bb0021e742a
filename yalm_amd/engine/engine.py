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
import sys
from collections import OrderedDict

import numpy as np
import torch

from ..cache.manager import PAGE, CacheError, CacheManager
from ..ops import kernels, library
from .context import StepContext, Workspace

DECODE_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 96, 128, 192, 256, 512, 1024)


class StepError(ValueError):
    pass


class _BucketBuffers:
    """The step metadata of one batch-size bucket: the device tensor that every graph of the bucket
    reads, and two pinned host copies that are filled in turn, so that the host can write a step's
    metadata while the upload of the step before is still queued."""

    def __init__(self, engine, bucket):
        self.bucket = bucket
        n_meta = 7 * bucket + 2
        self.meta_host = [torch.empty(n_meta, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.copied = [None, None]    # the event after the last upload of each host copy
        self.turn = 0
        self.meta = torch.zeros(n_meta, dtype=torch.int32, device=engine.device)

    def host(self):
        """The host copy to fill for the next upload."""
        if self.copied[self.turn] is not None:
            self.copied[self.turn].synchronize()         # its last upload has read the pinned buffer
        return self.meta_host[self.turn].numpy()

    def upload(self):
        self.meta.copy_(self.meta_host[self.turn], non_blocking=True)
        if self.copied[self.turn] is None:
            self.copied[self.turn] = torch.cuda.Event()
        self.copied[self.turn].record()
        self.turn ^= 1


class _DecodeGraph:
    """A decode step for one (batch bucket, pages bucket): the model's graph-safe runs of units as
    captured graphs, the others as (None, first, end) to be run kernel by kernel in between."""

    def __init__(self, engine, bufs, pages_bucket, ragged):
        B = bufs.bucket
        self.bufs = bufs
        self.ctx = engine._context("decode", engine.graph_ws, bufs.meta, B, B, 0)
        self.eager_ctx = engine._context("decode", engine.ws, bufs.meta, B, B, 0)
        for ctx in (self.ctx, self.eager_ctx):
            ctx.pages_bucket = pages_bucket
            ctx.ragged = ragged
            ctx.step_max_len = bufs.meta[6 * B + 1:6 * B + 2]
            ctx.seq_order = bufs.meta[6 * B + 2:7 * B + 2] if ragged else None
        self.segments = []
        self.x = None
        self.logits = None


class Engine:
    """max_tokens: the most tokens live sequences hold at any time (each rounded up to a page);
    max_batch: the most sequences alive at once; use_graphs: replay decode steps from captured
    graphs; max_graphs: the most (batch bucket, pages bucket) graphs kept (the least recently
    used one goes first); positions: how far a sequence may run (default: the model's
    max_position_embeddings) - more than the model's own only if every attention keeps a window,
    whose scores depend on distances alone (the reference's -T lets a text run on without end,
    src/infer.cpp:484-488)."""

    def __init__(self, model, max_tokens, max_batch=None, use_graphs=True, max_graphs=24, positions=None):
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
        if positions is not None and int(positions) > n_positions:
            if not self.cache.unbounded:
                raise StepError("%d positions asked for, the model has %d: more need a window on every attention "
                                "(a context shorter than the text)" % (int(positions), model.spec.max_positions))
            n_positions = int(positions)
        self.n_positions = n_positions
        model.prepare(n_positions)                      # tables only ever grow: other engines of the model keep theirs
        self._tables_version = model.tables_version
        self.ws = Workspace(self.device)                # steps that run kernel by kernel
        self.graph_ws = Workspace(self.device)          # shared by all captured graphs (they never run together)
        self.use_graphs = use_graphs
        self.max_graphs = max(1, int(max_graphs))
        self._widest_row = model.widest_row()
        self._prompt_tables = model.prompt_tables()     # index tables that parts want made for a step of whole prompts
        self._segments = model.decode_segments()        # the parts are fixed from here on: asked once, not every step
        self._any_graph = any(safe for safe, _, _ in self._segments)
        for text in model.describe()[1]:                # a slow fallback is said once, not hidden
            sys.stderr.write("[yalm_amd] %s\n" % text)
        self._graphs = OrderedDict()                    # (batch bucket, pages bucket, ragged) -> _DecodeGraph, least recently used first
        self._buckets = {}
        self.graphs_captured = 0

    # ------------------------------------------------------------------ sequences
    def start(self, n):
        """Slots for n sequences that start together."""
        return self.cache.acquire(n)

    def release(self, slots):
        """Gives back what finished sequences hold."""
        self.cache.release(list(slots))

    def length(self, slot):
        return self.cache.seq_len[slot]

    def step_bytes(self, slots):
        """Bytes a step over these sequences has to read: every weight once, an embedding row each,
        and the keys and values the sequences hold (a window's worth where a line keeps a window).
        The reference's Config::active_bytes (src/model.cpp:71-96) for a batch, with the head at
        its stored width."""
        total = self.model.weight_bytes() + (len(slots) - 1) * self.model.embedding.weight_bytes()
        for g in self.cache.kv_groups:
            per_token = g.bytes_per_token()
            for s in slots:
                n = self.cache.seq_len[s]
                total += per_token * (min(n, g.window) if g.window else n)
        return total

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

    def step(self, slots, tokens, want=None, targets=None):
        """slots: the sequences of the batch that take part in this step;
        tokens[i]: the next tokens of slots[i]; want[i]: indices into tokens[i] whose
        logits are asked for (default: the last).  Returns float32 [n_wanted, vocab]
        on the device, in the order of the slots and of want; the tensor is valid
        until the next step.

        targets[i][k] (optional): a token id for the k-th wanted place of slots[i].  The step then
        returns float32 [n_wanted], the probability softmax(logits)[target] at each wanted place
        (src/sampler.cpp:11-25), and the logits are made and used a block of rows at a time: what a
        text's perplexity needs, in memory that does not grow with the text."""
        B = len(slots)
        starts = self._starts(slots)
        if len(tokens) != B or (want is not None and len(want) != B):
            raise StepError("slots, tokens and want must have the same length")
        n_tok = [len(t) for t in tokens]
        if min(n_tok) < 1:
            raise StepError("every sequence of a step brings at least one token")
        V = self.model.vocab_size
        decode = max(n_tok) == 1
        if decode:                                        # one comparison pair for the batch
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
        if want is not None:
            for w, n in zip(want, n_tok):
                for j in w:
                    if not 0 <= j < n:
                        raise StepError("wanted place %r is outside the %d tokens of its sequence" % (j, n))
        if targets is not None:
            if want is None:
                want = [[n - 1] for n in n_tok]
            if len(targets) != B or any(len(t) != len(w) for t, w in zip(targets, want)):
                raise StepError("targets must name one token for every wanted place")
            if any(not 0 <= tok < V for t in targets for tok in t):
                raise StepError("a target token is outside the vocabulary of %d" % V)
        if max(starts) == 0:
            mode = "prefill"
        elif decode:
            mode = "decode"
        else:
            raise StepError("the sequences of a step either all start at their first token or all go on by one "
                            "token (lengths so far %s, tokens brought %s)" % (starts, n_tok))
        n_wanted = B if want is None else sum(len(w) for w in want)
        if sum(n_tok) * self._widest_row >= self.MAX_ELEMENTS or (targets is None and n_wanted * V >= self.MAX_ELEMENTS):
            raise StepError("a step of %d tokens with %d rows of logits is refused: its widest buffer (%d elements a "
                            "token, %d logits a row) would reach 2^31 elements, more than any step that was ever "
                            "checked; cut the batch, or ask for fewer logits"
                            % (sum(n_tok), n_wanted, self._widest_row, V))
        max_pos = max(starts) if decode else max(s + n for s, n in zip(starts, n_tok)) - 1
        new_lens = self._extend(slots, n_tok, max_pos)
        if mode == "decode":
            logits = self._decode(slots, firsts, want, starts, new_lens)
            if targets is None:
                return logits
            flat = torch.tensor([tok for t in targets for tok in t], dtype=torch.int32, device=self.device)
            return kernels.token_prob(logits, flat, torch.empty(flat.shape[0], dtype=torch.float32, device=self.device))
        if want is None:
            want = [[n - 1] for n in n_tok]
        return self._prefill(slots, tokens, want, n_tok, new_lens, targets)

    def step_from(self, slots, source, rows=None):
        """A decode step whose tokens lie on the device: slots[i] goes on by the token source[rows[i]]
        (rows None: source[i]).  source: int32 [n] on the engine's device, as a sampling kernel has
        written it; the host need not have seen the tokens, so the step can be queued while the step
        that made them still runs.  Returns the logits of every sequence, float32 [len(slots), vocab],
        valid until the next step.  A token outside the vocabulary (no sampling kernel makes one)
        is not reported: its embedding is a row of zeros."""
        B = len(slots)
        starts = self._starts(slots)
        if not (torch.is_tensor(source) and source.is_cuda and source.dtype == torch.int32 and source.dim() == 1
                and source.is_contiguous()):
            raise StepError("the tokens of step_from are a contiguous int32 vector on the device")
        n_src = source.shape[0]
        if rows is None:
            rows = range(B)
        if len(rows) != B or min(rows) < 0 or max(rows) >= n_src:
            raise StepError("step_from needs one row of its %d tokens for each of the %d sequences" % (n_src, B))
        if min(starts) < 1:
            raise StepError("a sequence goes on only after its prompt (lengths so far %s)" % (starts,))
        new_lens = self._extend(slots, [1] * B, max(starts))
        return self._decode(slots, None, None, starts, new_lens, source, rows)

    def _starts(self, slots):
        """The lengths so far of the sequences of a step, after the checks on its slots."""
        B = len(slots)
        if B == 0:
            raise StepError("a step needs at least one sequence")
        if len(set(slots)) != B:
            raise StepError("a slot occurs twice in the step")
        if not self.cache.slots.holds_all(slots):
            bad = [s for s in slots if not self.cache.slots.is_held(s)]
            raise StepError("slot %r is not held by a live sequence" % (bad[0],))
        seq_len = self.cache.seq_len
        return [seq_len[s] for s in slots]

    def _extend(self, slots, n_tok, max_pos):
        if max_pos >= self.n_positions:
            raise StepError("position %d is beyond the %d positions of this engine (max_position_embeddings / "
                            "max_tokens)" % (max_pos, self.n_positions))
        try:
            return self.cache.extend(slots, n_tok)
        except CacheError as e:
            raise StepError(str(e)) from None

    HEAD_ROWS = 1024        # rows of logits made at a time when only token probabilities are asked for
    MAX_ELEMENTS = 1 << 31  # a step whose widest buffer reaches this many elements is refused

    def _prefill(self, slots, tokens, want, n_tok, new_lens, targets=None):
        B, T = len(slots), sum(n_tok)
        rows = []
        cu = np.zeros(B + 1, dtype=np.int32)
        np.cumsum(n_tok, out=cu[1:])
        for i, w in enumerate(want):
            rows.extend(int(cu[i]) + j for j in w)
        R = len(rows)
        # what the parts asked for beside the common tables: made once a step, whoever and however many ask
        extra, host_values = [], {}
        for make in self._prompt_tables:
            values = host_values[make.name] = {}
            for key, v in make(n_tok).items():
                if isinstance(v, np.ndarray):
                    extra.append((make.name, key, np.ascontiguousarray(v, dtype=np.int32).ravel()))
                else:
                    values[key] = v
        n_meta = 3 * T + 3 * B + 1 + R + sum(len(a) for _, _, a in extra)
        host = np.empty(n_meta, dtype=np.int32)
        host[0:T] = np.concatenate([np.asarray(t, dtype=np.int32) for t in tokens])
        host[T:2 * T] = np.repeat(np.arange(B, dtype=np.int32), n_tok)
        host[2 * T:3 * T] = np.concatenate([np.arange(n, dtype=np.int32) for n in n_tok])
        o = 3 * T
        host[o:o + B] = slots
        host[o + B:o + 2 * B] = new_lens
        host[o + 2 * B:o + 3 * B + 1] = cu
        at = o + 3 * B + 1
        host[at:at + R] = rows
        at += R
        for _, _, a in extra:
            host[at:at + len(a)] = a
            at += len(a)
        meta = self.ws.get("meta", (n_meta,), torch.int32)
        meta.copy_(torch.from_numpy(host))
        ctx = self._context("prefill", self.ws, meta, T, B, max(n_tok) - 1)
        at = o + 3 * B + 1 + R
        ctx.tables = host_values
        for name, key, a in extra:
            ctx.tables[name][key] = meta[at:at + len(a)]
            at += len(a)
        ctx.host_slots, ctx.host_n_tokens, ctx.host_start = list(slots), list(n_tok), [0] * B
        V = self.model.vocab_size
        want_rows = meta[o + 3 * B + 1:o + 3 * B + 1 + R]
        if targets is not None:
            probs = torch.empty(R, dtype=torch.float32, device=self.device)
            flat = torch.tensor([tok for t in targets for tok in t], dtype=torch.int32, device=self.device)
            n_units = self.model.n_units()
            self.model.run_units(ctx, 0, n_units - 1)
            for r0 in range(0, R, self.HEAD_ROWS):
                r1 = min(R, r0 + self.HEAD_ROWS)
                block = self.ws.get("logits", (r1 - r0, V), torch.float32)
                self.model.run_units(ctx, n_units - 1, n_units, want_rows[r0:r1], block)
                kernels.token_prob(block, flat[r0:r1], probs[r0:r1])
            return probs
        logits = self.ws.get("logits", (R, V), torch.float32) if R else None
        self.model.forward(ctx, want_rows if R else None, logits)
        return logits if R else torch.empty((0, V), dtype=torch.float32, device=self.device)

    def _bucket(self, B):
        for b in DECODE_BUCKETS:
            if b >= B:
                return b
        return B

    @staticmethod
    def _fill_decode_meta(host, Bk, tokens, starts, slots, new_lens, ragged=False):
        """The metadata of a decode step of len(slots) sequences in Bk rows; the rows behind
        them are padding (token -1, slot -1, length 0).  Behind the tensors of the context: the longest
        sequence's length, and an order of the rows for kernels whose work grows with a row's length."""
        B = len(slots)
        host[0:Bk] = -1
        host[0:B] = tokens
        host[Bk:2 * Bk] = np.arange(Bk, dtype=np.int32)
        host[2 * Bk:3 * Bk] = 0
        host[2 * Bk:2 * Bk + B] = starts
        host[3 * Bk:4 * Bk] = -1
        host[3 * Bk:3 * Bk + B] = slots
        host[4 * Bk:5 * Bk] = 0
        host[4 * Bk:4 * Bk + B] = new_lens
        host[5 * Bk:6 * Bk + 1] = np.arange(Bk + 1, dtype=np.int32)
        host[6 * Bk + 1] = max(new_lens) if len(new_lens) else 0
        order = host[6 * Bk + 2:7 * Bk + 2]
        order[:] = np.arange(Bk, dtype=np.int32)
        if ragged and B > 1:
            # The rows by length, the longest first, and the second half turned round: where a kernel's workgroups
            # stand two to a compute unit, the one that follows the longest sequence's is the shortest one's.
            ranks = np.argsort(-np.asarray(new_lens, dtype=np.int64), kind="stable").astype(np.int32)
            half = (Bk + 1) // 2
            rows = np.concatenate([ranks, np.arange(B, Bk, dtype=np.int32)])
            order[:half] = rows[:half]
            order[half:] = rows[half:][::-1]

    @staticmethod
    def _is_ragged(new_lens):
        """True if the sequences of a decode step differ so much in length that cutting each into the same number
        of pieces would leave workgroups of very unequal work (the longest is a fifth and two pages above the mean)."""
        n = len(new_lens)
        if n < 2:
            return False
        longest, mean = max(new_lens), sum(new_lens) / n
        return longest - mean >= max(2 * PAGE, 0.2 * longest)

    @staticmethod
    def _pages_bucket(n_tokens):
        """Launch shapes may depend on the longest sequence only through this bucket (a power of
        two of pages), so that a captured graph stays valid until a sequence outgrows it."""
        pages_bucket = 1
        while pages_bucket * PAGE < n_tokens:
            pages_bucket *= 2
        return pages_bucket

    def _decode(self, slots, firsts, want, starts, new_lens, source=None, source_rows=None):
        """firsts: the sequences' tokens, or None: they are source[source_rows] on the device."""
        B = len(slots)
        use_graph = self.use_graphs and self._any_graph
        Bk = self._bucket(B) if use_graph else B
        pages_bucket = self._pages_bucket(max(new_lens))
        ragged = self._is_ragged(new_lens)
        if firsts is None:
            firsts = 0                                                # a place holder; fed below
        if not use_graph:
            host = np.empty(7 * Bk + 2, dtype=np.int32)
            self._fill_decode_meta(host, Bk, firsts, starts, slots, new_lens, ragged)
            meta = self.ws.get("meta", (7 * Bk + 2,), torch.int32)
            meta.copy_(torch.from_numpy(host))
            self._feed(meta, B, source, source_rows)
            ctx = self._context("decode", self.ws, meta, Bk, Bk, max(starts))
            ctx.pages_bucket = pages_bucket
            ctx.ragged = ragged
            ctx.step_max_len = meta[6 * Bk + 1:6 * Bk + 2]
            ctx.seq_order = meta[6 * Bk + 2:7 * Bk + 2] if ragged else None
            ctx.host_slots, ctx.host_n_tokens, ctx.host_start = list(slots), [1] * B, list(starts)
            logits = self.ws.get("logits", (Bk, self.model.vocab_size), torch.float32)
            self.model.forward(ctx, None, logits)                     # every row
        else:
            g = self._graph(Bk, pages_bucket, ragged)
            self._fill_decode_meta(g.bufs.host(), Bk, firsts, starts, slots, new_lens, ragged)
            g.bufs.upload()
            self._feed(g.bufs.meta, B, source, source_rows)
            for graph, lo, hi in g.segments:
                if graph is not None:
                    graph.replay()
                else:                                                 # a run of units that no graph can hold
                    ctx = g.eager_ctx
                    ctx.x = g.x
                    ctx.max_position = max(starts)
                    ctx.host_slots, ctx.host_n_tokens, ctx.host_start = list(slots), [1] * B, list(starts)
                    self.model.run_units(ctx, lo, hi, None, g.logits)
            logits = g.logits
        if want is None:
            return logits[:B]
        rows = [i for i, w in enumerate(want) if len(w) > 0]
        if len(rows) == B:
            return logits[:B]
        if not rows:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return logits[torch.tensor(rows, device=self.device)]

    def _feed(self, meta, B, source, source_rows):
        """Puts the tokens that lie on the device into the step's metadata."""
        if source is None:
            return
        if isinstance(source_rows, range) or list(source_rows) == list(range(B)):
            meta[0:B].copy_(source[0:B])
        else:
            index = torch.tensor(list(source_rows), dtype=torch.int64, device=self.device)
            torch.index_select(source, 0, index, out=meta[0:B])

    # ------------------------------------------------------------------ captured decode steps
    def _graph(self, Bk, pages_bucket, ragged=False):
        """The captured step for the bucket pair (and for sequences of much the same or of very unequal lengths),
        made now if there is none (most recently used last)."""
        if self.model.tables_version != self._tables_version:       # a table the graphs point to was replaced
            self.drop_graphs()
            self._tables_version = self.model.tables_version
        key = (Bk, pages_bucket, bool(ragged))
        g = self._graphs.get(key)
        if g is None:
            if len(self._graphs) >= self.max_graphs or not self._graphs:
                torch.cuda.synchronize(self.device)      # a graph's last replay may still be queued: the host runs ahead
            while len(self._graphs) >= self.max_graphs:
                self._graphs.popitem(last=False)
            if not self._graphs:
                self.graph_ws.drop_retired()
            g = self._capture(Bk, pages_bucket, bool(ragged))
            self._graphs[key] = g
        else:
            self._graphs.move_to_end(key)
        return g

    def _capture(self, Bk, pages_bucket, ragged=False):
        """Captures the decode step of a bucket pair on rows of padding only: nothing that a live
        sequence holds (cache pages, per-sequence state) is read or written, so capturing in the
        middle of a request changes nothing for it.  The step runs once kernel by kernel first
        (every buffer gets its size), then under capture."""
        bufs = self._buckets.get(Bk)
        if bufs is None:
            bufs = self._buckets[Bk] = _BucketBuffers(self, Bk)
        self._fill_decode_meta(bufs.host(), Bk, [], [], [], [])
        bufs.upload()
        g = _DecodeGraph(self, bufs, pages_bucket, ragged)
        ws, ctx = self.graph_ws, g.ctx
        ctx.max_position = 0
        ctx.x = g.x = ws.get("x", (Bk, self.model.dim), torch.float32)
        g.logits = ws.get("logits", (Bk, self.model.vocab_size), torch.float32)
        for safe, lo, hi in self._segments:
            if safe:
                self.model.run_units(ctx, lo, hi, None, g.logits)
        torch.cuda.synchronize(self.device)
        ws.frozen = True
        try:
            for safe, lo, hi in self._segments:
                graph = None
                if safe:
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        self.model.run_units(ctx, lo, hi, None, g.logits)
                g.segments.append((graph, lo, hi))
        finally:
            ws.frozen = False
        ws.pinned = True
        self.graphs_captured += 1
        return g

    def warmup(self, batch_sizes=(1,), max_len=None, min_len=1, ragged=False):
        """Captures the decode graphs for batches of the given sizes and for sequences of min_len to
        max_len tokens (default: the longest the engine holds; ragged: for batches whose sequences differ
        much in length) ahead of the first request, so that no
        live step pays for a capture.  It runs on padding rows: no slot or page is taken and live
        sequences are left alone (the reference runs one forward before it measures,
        src/main.cpp:81-85, which overwrites a cache row).  Returns the number of graphs captured."""
        if not (self.use_graphs and self._any_graph):
            return 0
        longest = self.n_positions if self.cache.unbounded else min(self.n_positions, self.cache.max_seq_len)
        max_len = longest if max_len is None else min(int(max_len), longest)
        min_len = max(1, min(int(min_len), max_len))
        pairs = []
        for Bk in sorted({self._bucket(int(b)) for b in batch_sizes if int(b) > 0}):
            pb = self._pages_bucket(min_len)
            while True:
                pairs.append((Bk, pb))
                if pb * PAGE >= max_len:
                    break
                pb *= 2
        if len(pairs) > self.max_graphs:
            raise StepError("warmup asks for %d graphs, the engine keeps %d (max_graphs)" % (len(pairs), self.max_graphs))
        before = self.graphs_captured
        for Bk, pb in pairs:
            self._graph(Bk, pb, ragged)
        return self.graphs_captured - before

    def drop_graphs(self):
        """Forgets every captured graph and the buffers only they used (after their last replays have ended)."""
        torch.cuda.synchronize(self.device)
        self._graphs.clear()
        self.graph_ws.drop_retired()

    def graph_bytes(self):
        """Device bytes of the buffers that the captured graphs share."""
        return self.graph_ws.bytes() + sum(b.meta.numel() * 4 for b in self._buckets.values())

    def synchronize(self):
        torch.cuda.synchronize(self.device)
