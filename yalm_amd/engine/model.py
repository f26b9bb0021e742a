"""The model: parts built from a ModelSpec, weights loaded by name, and the
forward pass over a step's tokens (src/infer.cpp:477-521): embedding, the layers
in the order the schedule gives, then for the wanted rows the final norm and the
head."""
import torch

from ..config import config_from_dict, config_from_folder
from ..parts import base as parts_base
from ..parts import build_part
from ..weights import random_init
from ..weights.loader import TensorSource, WeightsError


def build_block(layer_spec, dim):
    try:
        cls = parts_base._REGISTRY["block"][layer_spec.block]
    except KeyError:
        raise ValueError("no block arrangement named %r is registered (known: %s)"
                         % (layer_spec.block, sorted(parts_base._REGISTRY["block"]))) from None
    return cls(layer_spec, dim)


def _walk(part):
    yield part
    for c in part.children():
        yield from _walk(c)


class Model:
    def __init__(self, spec, config=None):
        self.spec = spec
        self.config = config
        self.dim = spec.dim
        self.vocab_size = spec.vocab_size
        with parts_base.sharing():        # parts that follow from their spec alone are built once (position tables)
            self.embedding = build_part("embedding", spec.embedding, spec.dim, "")
            self.blocks = [build_block(ls, spec.dim) for ls in spec.layers]
            self.final_norm = build_part("norm", spec.final_norm, spec.dim, "")
            self.head = build_part("head", spec.head, spec.dim, "", embedding=self.embedding)
        self.schedule = list(spec.schedule)
        import inspect
        self._takes_next_norm = ["next_norm" in inspect.signature(b.forward).parameters for b in self.blocks]
        readers = {}
        for e in self.schedule:
            if not e.writes_cache:
                readers[e.cache] = True
        self.shared_lines = set(readers)
        self.compute_dtype = None
        self.device = None
        self.tables_version = 0

    # ------------------------------------------------------------------ weights
    def top_parts(self):
        return [self.embedding] + self.blocks + [self.final_norm, self.head]

    def all_parts(self):
        """Every part once (a part that several others share is named by each of them)."""
        seen = set()
        for top in self.top_parts():
            for p in _walk(top):
                if id(p) not in seen:
                    seen.add(id(p))
                    yield p

    def param_specs(self):
        seen, out = set(), []
        for p in self.all_parts():
            for s in p.param_specs():
                if s.name not in seen:
                    seen.add(s.name)
                    out.append(s)
        return out

    def load(self, get, compute_dtype, device):
        """`get(name)` gives each declared tensor; parts lay them out on the device."""
        self.compute_dtype = compute_dtype
        self.device = torch.device(device)
        for p in self.all_parts():
            p.load(get, compute_dtype, self.device)
        return self

    @classmethod
    def from_folder(cls, path, dtype=torch.bfloat16, device="cuda:0", window=None, strict=False, context=None):
        """The model of a folder with config.json and *.safetensors; the class of the
        configuration is chosen by config.json's architecture.  strict: tensors in the
        folder that the model does not use are an error (else a warning).  window: attend over
        the last `window` positions only; context: the reference's -T (attention sinks and a window
        that fill a context of that many positions)."""
        cfg = config_from_folder(path)
        if window:
            cfg = cfg.with_window(window)
        if context:
            cfg = cfg.with_context(context)
        model = cls(cfg.to_spec(), cfg)
        source = TensorSource(path)
        source.check(model.param_specs(), strict=strict)
        return model.load(source.get, dtype, device)

    @classmethod
    def random(cls, config, seed, dtype=torch.bfloat16, device="cuda:0", stored_dtype=None, n_layers=None):
        """Random weights made directly on the device (same values as a folder written
        by write_random_model with the same seed and stored dtype).  n_layers < the
        configuration's builds only the first layers."""
        cfg = config_from_dict(config) if isinstance(config, dict) else config
        spec = cfg.to_spec()
        if n_layers is not None and n_layers < len(spec.layers):
            spec.layers = spec.layers[:n_layers]
            spec.schedule = [e for e in spec.schedule if e.layer < n_layers]
        model = cls(spec, cfg)
        specs = {s.name: s for s in model.param_specs()}
        stored = stored_dtype or dtype

        def get(name):
            s = specs[name]
            return random_init.random_values(s.name, s.shape, s.init, s.fan_in, seed, device=device).to(stored)

        return model.load(get, dtype, device)

    # ------------------------------------------------------------------ the cache's needs
    def cache_requests(self):
        """{cache line: what its mixer asks of the cache}, for the lines that are written."""
        out = {}
        for e in self.schedule:
            if e.writes_cache:
                mixer = getattr(self.blocks[e.layer], "mixer", None)     # a block without a mixer keeps nothing
                out[e.cache] = mixer.cache_request() if mixer is not None else None
        return out

    def prepare(self, n_positions):
        """Lets position encodings build their tables for positions < n_positions.  A table that
        already reaches that far stays as it is (engines that share the model keep using it);
        `tables_version` counts the times a table was replaced, for whoever holds its address."""
        def held(p):          # addresses of what a captured graph may point to: the rotation table, a score bias
            return tuple(t.data_ptr() for t in (getattr(p, "table", None), getattr(p, "score_bias", None)) if t is not None)
        for p in self.all_parts():
            if hasattr(p, "prepare"):
                before = getattr(p, "table", None)
                if before is not None and getattr(p, "n_positions", 0) >= n_positions:
                    continue
                was = held(p)
                p.prepare(n_positions, self.device)
                if was and held(p) != was:
                    self.tables_version += 1

    # ------------------------------------------------------------------ the step as a row of units
    # unit 0 is the embedding, units 1..n the schedule's entries, unit n + 1 the final norm and the head
    def n_units(self):
        return len(self.schedule) + 2

    def unit_parts(self, u):
        if u == 0:
            return list(_walk(self.embedding))
        if u == len(self.schedule) + 1:
            return list(_walk(self.final_norm)) + list(_walk(self.head))
        return list(_walk(self.blocks[self.schedule[u - 1].layer]))

    def unit_graph_safe(self, u):
        """True if the unit launches only kernels whose arguments stay valid from step to step
        (a part that does not says so with `graph_safe = False`)."""
        return all(getattr(p, "graph_safe", True) for p in self.unit_parts(u))

    def graph_safe(self):
        return all(self.unit_graph_safe(u) for u in range(self.n_units()))

    def decode_segments(self):
        """The units of a decode step in runs of equal kind: [(graph_safe, first unit, end unit)].
        A run that is graph-safe can be captured and replayed; the others run kernel by kernel."""
        out = []
        for u in range(self.n_units()):
            safe = self.unit_graph_safe(u)
            if out and out[-1][0] == safe:
                out[-1] = (safe, out[-1][1], u + 1)
            else:
                out.append((safe, u, u + 1))
        return out

    def describe(self):
        """({line on the kernels that serve a part: the schedule entries it stands for}, the lines that
        name a slow fallback), at the model's compute dtype."""
        lines, slow = {}, []
        for i, e in enumerate(self.schedule):
            for p in _walk(self.blocks[e.layer]):
                text, is_slow = p.describe(self.compute_dtype)
                entries = lines.setdefault(text, [])
                if i not in entries:
                    entries.append(i)
                if is_slow and text not in slow:
                    slow.append(text)
        return lines, slow

    def prompt_tables(self):
        """The makers of index tables that parts ask for in a step of whole prompts (a part names them in
        `prompt_tables`), each once, by its name.  A maker is called with the step's token counts and gives
        {key: int32 array (uploaded with the step's metadata) or host value}; parts find the result in
        ctx.tables[maker.name]."""
        out = {}
        for p in self.all_parts():
            for make in getattr(p, "prompt_tables", ()):
                out.setdefault(make.name, make)
        return list(out.values())

    def widest_row(self):
        """The most elements any part keeps for one token of a step (a part says so with `row_elements()`;
        the residual stream's width stands for the others)."""
        return max([self.dim] + [int(p.row_elements()) for p in self.all_parts() if hasattr(p, "row_elements")])

    def weight_bytes(self):
        """Bytes of weights a step reads: every weight once, one embedding row."""
        total = self.embedding.weight_bytes() + self.final_norm.weight_bytes() + self.head.weight_bytes()
        for e in self.schedule:
            total += sum(p.weight_bytes() for p in _walk(self.blocks[e.layer]))
        return total

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, want_rows, logits):
        """Runs the step's tokens through the layers (the cache is read and written
        through ctx) and writes logits for the rows want_rows (int32 device tensor;
        None: every row, in order)."""
        return self.run_units(ctx, 0, self.n_units(), want_rows, logits)

    def run_units(self, ctx, lo, hi, want_rows=None, logits=None):
        """Units lo..hi-1 of the step.  The residual stream stays in ctx.x between calls; nothing
        else is handed from one call to the next (the last entry of a run prepares no norm for
        whoever comes after it)."""
        n = len(self.schedule)
        ctx.normed.clear()
        for u in range(lo, hi):
            if u == 0:
                T = ctx.tokens.shape[0]
                ctx.x = ctx.ws.get("x", (T, self.dim), torch.float32)
                self.embedding.forward(ctx.tokens, ctx.x, ctx)
            elif u <= n:
                e = self.schedule[u - 1]
                block = self.blocks[e.layer]
                if self._takes_next_norm[e.layer]:
                    next_norm = None
                    if u + 1 < hi:                    # the consumer runs in this call
                        nxt = self.blocks[self.schedule[u].layer] if u < n else None
                        next_norm = self.final_norm if nxt is None else getattr(nxt, "first_norm", lambda: None)()
                    block.forward(ctx.x, ctx, e.cache, e.writes_cache, next_norm=next_norm)
                else:
                    block.forward(ctx.x, ctx, e.cache, e.writes_cache)
            elif logits is not None and logits.shape[0] > 0:
                x = ctx.x
                R, T = logits.shape[0], x.shape[0]
                if want_rows is None and R == T and self.head.fuses_norm(self.final_norm, x, ctx):
                    self.head.forward_prenorm(x, self.final_norm, logits, ctx)
                else:
                    h = ctx.ws.get("head.h", (R, self.dim), ctx.act_dtype)
                    self.final_norm.forward(x, h, ctx, row_index=want_rows)
                    self.head.forward(h, logits, ctx)
        ctx.normed.clear()
        return logits


def param_specs_of(spec):
    """The tensors a model of this spec needs (no device memory is touched)."""
    return Model(spec).param_specs()
