"""What a step hands to the parts: the step's tokens and their places as device
tensors, the cache, and a workspace of reusable buffers."""
import torch


class Workspace:
    """Named device buffers that are reused from step to step and grow on demand.
    A buffer is a flat allocation; `get` returns a view of the asked shape.

    While `frozen` a buffer may not grow (a graph is being captured).  Once `pinned`
    (captured graphs hold the buffers' addresses) a buffer that has to grow is
    replaced for later users, and the old one is kept for the graphs that still use
    it until `drop_retired`."""

    def __init__(self, device):
        self.device = device
        self._flat = {}
        self._views = {}              # (name, dtype, shape) -> the view that was handed out last time
        self._retired = []
        self.frozen = False           # set while a graph is captured on these buffers
        self.pinned = False           # set once a captured graph uses these buffers

    def _buffer(self, name, shape, dtype, zeroed):
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        buf = self._flat.get(key)
        if buf is None or buf.numel() < n:
            if self.frozen:
                raise RuntimeError("workspace buffer %r would have to grow inside a captured graph" % (name,))
            if buf is not None and self.pinned:
                self._retired.append(buf)
            make = torch.zeros if zeroed else torch.empty
            buf = make(max(n, 1), dtype=dtype, device=self.device)
            self._flat[key] = buf
            for k in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[k]                 # views of the buffer that was replaced
        if len(self._views) > 4096:                # many shapes (prompts of every length): start afresh
            self._views.clear()
        view = buf[:n].view(*shape)
        self._views[(name, dtype, shape)] = view
        return view

    def get(self, name, shape, dtype):
        return self._buffer(name, shape, dtype, False)

    def get_zeroed(self, name, shape, dtype):
        """Like get, but the buffer is zero when it is first made (users keep it so)."""
        return self._buffer(name, shape, dtype, True)

    def drop_retired(self):
        """Frees the replaced buffers; only when no graph that used them is left."""
        self._retired.clear()
        self.pinned = False

    def bytes(self):
        return sum(b.numel() * b.element_size() for b in list(self._flat.values()) + self._retired)


class StepContext:
    """mode: 'prefill' (sequences that start at position 0, whole prompts, packed)
    or 'decode' (one token per sequence).  Device tensors, all int32:
      tokens[T], tok_seq[T] (row of the batch), tok_pos[T] (position in its sequence),
      seq_slot[B] (-1: padding row), seq_len[B] (length after this step), cu_seqlens[B+1].
    tables: prefill only; {maker's name: {key: int32 device tensor or host value}}, the index tables that parts
    asked for through their `prompt_tables` (made once a step and uploaded with the tensors above; the
    attention's staging tiles and the order in which it takes them are such a table).
    max_position: the largest position in the step (host value, for table checks).
    host_slots, host_n_tokens, host_start: the step's real sequences as host lists (a decode step's
    padding rows, seq_slot -1, are not in them), for parts whose launches depend on host values.
    pages_bucket: decode only; an upper bound (a power of two) of the pages of the step's
    longest sequence; with `ragged` (decode only: the step's sequences differ much in length, so that work
    cut per sequence would be uneven) the only way launch shapes may depend on lengths.
    step_max_len: decode only; int32 [1] on the device, the length of the step's longest sequence.
    seq_order: ragged decode steps only; int32 [B] on the device, the rows in the order in which a kernel whose
    work grows with a row's length should take them (the longest first, the second half from the shortest up)."""

    def __init__(self, mode, cache, ws, act_dtype, shared_lines=()):
        self.mode = mode
        self.cache = cache
        self.ws = ws
        self.act_dtype = act_dtype
        self.shared_lines = set(shared_lines)
        self.tokens = self.tok_seq = self.tok_pos = self.seq_slot = self.seq_len = self.cu_seqlens = None
        self.tables = {}
        self.x = None                     # the residual stream of the step, float32 [T, dim]
        self.normed = {}                  # id(norm part) -> (xn, ss, eps): activations a producer emitted for it
        self.pages_bucket = 1 << 30       # decode: no sequence of the step has more pages than this
        self.ragged = False
        self.step_max_len = None
        self.seq_order = None
        self.max_position = 0
        self.host_slots = []
        self.host_n_tokens = []
        self.host_start = []

    def line_is_shared(self, line):
        return line in self.shared_lines
