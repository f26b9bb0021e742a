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

    # ------------------------------------------------------------------ weights
    def top_parts(self):
        return [self.embedding] + self.blocks + [self.final_norm, self.head]

    def all_parts(self):
        for p in self.top_parts():
            yield from _walk(p)

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
    def from_folder(cls, path, dtype=torch.bfloat16, device="cuda:0", window=None):
        """The model of a folder with config.json and *.safetensors; the class of the
        configuration is chosen by config.json's architecture."""
        cfg = config_from_folder(path)
        if window:
            cfg = cfg.with_window(window)
        model = cls(cfg.to_spec(), cfg)
        source = TensorSource(path)
        source.check(model.param_specs())
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
                out[e.cache] = self.blocks[e.layer].mixer.cache_request()
        return out

    def prepare(self, n_positions):
        """Lets position encodings build their tables for positions < n_positions."""
        for p in self.all_parts():
            if hasattr(p, "prepare"):
                p.prepare(n_positions, self.device)

    def graph_safe(self):
        """True if every part launches only kernels whose arguments stay valid from
        step to step (a part that is not says so with `graph_safe = False`)."""
        return all(getattr(p, "graph_safe", True) for p in self.all_parts())

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
        T = ctx.tokens.shape[0]
        x = ctx.ws.get("x", (T, self.dim), torch.float32)
        self.embedding.forward(ctx.tokens, x, ctx)
        ctx.normed.clear()
        n = len(self.schedule)
        for i, e in enumerate(self.schedule):
            block = self.blocks[e.layer]
            if self._takes_next_norm[e.layer]:
                nxt = self.blocks[self.schedule[i + 1].layer] if i + 1 < n else None
                next_norm = getattr(nxt, "mixer_norm", None) if nxt is not None else self.final_norm
                block.forward(x, ctx, e.cache, e.writes_cache, next_norm=next_norm)
            else:
                block.forward(x, ctx, e.cache, e.writes_cache)
        if logits is not None and logits.shape[0] > 0:
            R = logits.shape[0]
            if want_rows is None and R == T and self.head.fuses_norm(self.final_norm, x, ctx):
                self.head.forward_prenorm(x, self.final_norm, logits, ctx)
            else:
                h = ctx.ws.get("head.h", (R, self.dim), ctx.act_dtype)
                self.final_norm.forward(x, h, ctx, row_index=want_rows)
                self.head.forward(h, logits, ctx)
        return logits


def param_specs_of(spec):
    """The tensors a model of this spec needs (no device memory is touched)."""
    return Model(spec).param_specs()
