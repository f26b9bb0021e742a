"""Interfaces of the parts a model is put together from, and their registries.

A part is built from a PartSpec (its sizes and constants), the width of the
residual stream and the prefix of its tensor names.  No part knows which model
it is in.  Kinds of parts and the methods each must have:

  norm           forward(x_f32[R, dim], out[R, dim], ctx, row_index=None)
  position       prepare(n_positions, device); used by the mixers that name it (one instance per distinct
                 PartSpec of a model if the class says `share_by_spec = True`: it then has no tensors
                 of its own and its prefix means nothing)
  mixer          cache_request() -> KVRequest | StateRequest | None
                 forward(h[T, dim], x_f32[T, dim], ctx, line, writes_cache): adds its output to x
  feed_forward   forward(h[T, dim], x_f32[T, dim], ctx): adds its output to x
  block          forward(x_f32[T, dim], ctx, line, writes_cache): one layer on the residual stream;
                 optional: a `next_norm` argument (the norm that reads the stream after this layer, whose
                 activations the layer may prepare) and first_norm() (the norm it applies first)
  embedding      forward(tokens_i32[T], x_f32[T, dim], ctx)
  head           forward(h[R, dim], logits_f32[R, vocab], ctx)

A mixer, feed-forward or head may fold the norm in front of it into its first
product: fuses_norm(norm, x, ctx) says so for a step, and forward_prenorm(x, norm,
..., emit_for=next_norm) then replaces norm.forward + forward.  With emit_for it may
also leave, in ctx.normed[id(next_norm)], either (xn, ss, eps): the activations already
multiplied by that norm's weights and the partial sums of squares [rows, parts] (its residual-add GEMM,
or the kernel that adds that GEMM's K slices, writes them: decode steps of up to 128 rows), or
(h, None, None): the norm's finished output (more rows, and steps of whole prompts), which the next
consumer takes instead of reading the residual stream.

A part whose launches in a decode step depend on host values (it reads ctx.host_*, or sizes that
change from step to step) says so with the class attribute `graph_safe = False`; the layers around
it are still replayed from captured graphs.  A graph-safe part reads positions, lengths and slots
from the step's device tensors only, and leaves rows with seq_slot -1 (padding) without effect on
the cache or on per-sequence state.

All of them: param_specs() -> [ParamSpec], load(get, compute_dtype, device),
weight_bytes().  `h` is in the compute dtype (bfloat16 or float32); the
residual stream `x` is always float32."""
import threading
from typing import Callable, Dict, List

from ..config.spec import PartSpec
from ..weights.loader import ParamSpec

ROLES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_REGISTRY: Dict[str, Dict[str, type]] = {r: {} for r in ROLES}


def register_part(role, kind, cls, replace=False):
    """Registers class `cls` as the part `kind` of role `role`."""
    if role not in _REGISTRY:
        raise ValueError("unknown role %r (one of %s)" % (role, ROLES))
    if kind in _REGISTRY[role] and not replace and _REGISTRY[role][kind] is not cls:
        raise ValueError("%s part %r is already registered" % (role, kind))
    _REGISTRY[role][kind] = cls
    return cls


def unregister_part(role, kind):
    _REGISTRY[role].pop(kind, None)


def part(role, kind):
    """Decorator form of register_part."""
    def deco(cls):
        return register_part(role, kind, cls)
    return deco


_building = threading.local()        # .pools: the pools of the models this thread is building (innermost last)


def _pools():
    if not hasattr(_building, "pools"):
        _building.pools = []
    return _building.pools


class sharing:
    """While a model is built inside `with sharing():`, parts whose class says `share_by_spec = True`
    (parts without tensors of their own, whose state follows from their PartSpec alone: the position
    encodings) are built once per distinct (role, PartSpec, width) and handed to everyone who asks
    for that spec.  The thirty-two attentions of a model then read one table of angles."""

    def __enter__(self):
        _pools().append({})
        return _pools()[-1]

    def __exit__(self, *exc):
        _pools().pop()
        return False


def build_part(role, spec: PartSpec, dim: int, prefix: str, **extra):
    try:
        cls = _REGISTRY[role][spec.kind]
    except KeyError:
        raise ValueError("no %s part named %r is registered (known: %s)"
                         % (role, spec.kind, sorted(_REGISTRY[role]))) from None
    pools = _pools()
    if pools and getattr(cls, "share_by_spec", False) and not extra:
        key = (role, spec, dim)
        made = pools[-1].get(key)
        if made is None:
            made = pools[-1][key] = cls(spec, dim, prefix + spec.prefix)
        return made
    return cls(spec, dim, prefix + spec.prefix, **extra)


class Part:
    """Common ground of all parts."""

    def __init__(self, spec: PartSpec, dim: int, prefix: str):
        self.spec = spec
        self.dim = dim
        self.prefix = prefix

    def param_specs(self) -> List[ParamSpec]:
        return []

    def load(self, get: Callable, compute_dtype, device):
        """Takes its tensors (`get(name)` gives a CPU tensor) and lays them out on the device."""

    def weight_bytes(self) -> int:
        """Bytes of weights one step reads (every weight once)."""
        return 0

    def children(self):
        return []

    def describe(self, compute_dtype):
        """(one line on which kernels serve this part at the compute dtype, True if that is a slow
        fallback the user should know of)."""
        return type(self).__name__, False

    @staticmethod
    def _gemm(ctx, a, w, out, epilogue, hidden=0, scale_from=None):
        """kernels.gemm with the scratch that lets small batches split K."""
        from ..ops import kernels
        import torch
        ws = None
        n = kernels.gemm_workspace_floats(a.shape[0], w.shape[0], a.shape[1]) if a.dtype == torch.bfloat16 else 0
        if n and ctx is not None:
            ws = ctx.ws.get("gemm.partial", (n,), torch.float32)
        return kernels.gemm(a, w, out, epilogue, hidden=hidden, workspace=ws, scale_from=scale_from)

    def _emit_args(self, emit_for, ctx, T, width):
        """Operands for a residual-add GEMM that also prepares the activations of the norm
        `emit_for` (the next norm on the residual stream), or None if that cannot be done."""
        from ..ops import kernels
        if emit_for is None or not hasattr(emit_for, "fused") or width >= 16384:
            return None
        if ctx.mode != "decode" or not kernels.can_chain(T, width, ctx.act_dtype):
            return None
        import torch
        nw, eps = emit_for.fused()
        xn = ctx.ws.get("chain.xn", (T, width), torch.bfloat16)
        ss = ctx.ws.get("chain.ss", (T, kernels.gemm_chain_parts(width)), torch.float32)
        return nw, xn, ss, eps

    def _add_norm_args(self, emit_for, ctx, T, width, K):
        """Operands for a residual-add GEMM [T, K] x [width, K] of more than 16 rows that also does the norm
        `emit_for` (the next one on the residual stream) and leaves its activations ready, or None."""
        from ..ops import kernels
        if emit_for is None or not hasattr(emit_for, "fused") or ctx.mode not in ("decode", "prefill"):
            return None
        if not kernels.can_add_norm(T, K, ctx.act_dtype):
            return None
        import torch
        nw, eps = emit_for.fused()
        h = ctx.ws.get("chain.h", (T, width), torch.bfloat16)          # read by the consumer before the next is written
        ws = ctx.ws.get("gemm.partial", (kernels.fused_workspace_floats(T, width, K),), torch.float32)
        return nw, eps, h, ws

    def _add_emit_args(self, emit_for, ctx, T, width, K):
        """Operands for a residual-add GEMM [T, K] x [width, K] of a decode step of 17..128 rows that prepares the
        norm `emit_for` as the chain of the small batches does (activations times the norm's weights, partial sums of
        squares; the consumer scales its sums), or None."""
        from ..ops import kernels
        if emit_for is None or not hasattr(emit_for, "fused") or ctx.mode != "decode":
            return None
        if not (kernels.can_add_emit(T, K, ctx.act_dtype) and kernels.can_add_emit(T, width, ctx.act_dtype)):
            return None
        import torch
        nw, eps = emit_for.fused()
        xn = ctx.ws.get("chain.h", (T, width), torch.bfloat16)
        ss = ctx.ws.get("chain.ss", (T, kernels.gemm_add_emit_parts(width)), torch.float32)
        ws = ctx.ws.get("gemm.partial", (kernels.fused_workspace_floats(T, width, K),), torch.float32)
        return nw, eps, xn, ss, ws

    def fuses_norm(self, norm, x, ctx):
        """True if this part can take the float32 residual stream x and do `norm` itself
        (it then offers forward_prenorm in place of forward)."""
        return False
