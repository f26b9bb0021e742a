"""Gated feed-forward, dense: x += down( act(gate h) * (up h) )
(src/infer.cpp:356-385 with one expert of weight 1).  act is silu(z) = z / (1 + exp(-z)) (SwiGLU) or, with the
parameter `activation` = "gelu", gelu(z) = z/2 (1 + tanh(0.797885 (z + 0.044715 z^3))): the two the reference
knows (src/infer.cpp:189-195, convert.py:51-52).
Gate and up rows are interleaved in blocks of 16 at load so that one GEMM
produces both and its epilogue multiplies them (the reference fuses the two
products by pointer, src/infer.cu:610-634)."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part

GATE_BLOCK = 16
ACTIVATIONS = {"silu": kernels.EPI_GATED, "gelu": kernels.EPI_GATED_GELU}


def interleave_gate_up(gate, up):
    """[H, D] x 2 -> [32 * ceil(H/16), D]: 16 gate rows, 16 up rows, ...; zero rows pad the last block."""
    H, D = gate.shape
    nb = (H + GATE_BLOCK - 1) // GATE_BLOCK
    out = torch.zeros((nb, 2, GATE_BLOCK, D), dtype=gate.dtype, device=gate.device)
    pad = nb * GATE_BLOCK
    g = torch.zeros((pad, D), dtype=gate.dtype, device=gate.device)
    u = torch.zeros((pad, D), dtype=gate.dtype, device=gate.device)
    g[:H] = gate
    u[:H] = up
    out[:, 0] = g.reshape(nb, GATE_BLOCK, D)
    out[:, 1] = u.reshape(nb, GATE_BLOCK, D)
    return out.reshape(nb * 2 * GATE_BLOCK, D)


@part("feed_forward", "swiglu")
class SwiGLU(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.hidden = int(spec.params["hidden"])
        self.activation = str(spec.params.get("activation", "silu"))
        if self.activation not in ACTIVATIONS:
            raise ValueError("feed-forward activation %r is not offered (%s)" % (self.activation, ", ".join(ACTIVATIONS)))
        self.gated = ACTIVATIONS[self.activation]          # the GEMM epilogue that applies it
        self.w_gate_up = None
        self.w_down = None

    def param_specs(self):
        D, H = self.dim, self.hidden
        return [ParamSpec(self.prefix + "gate_proj.weight", (H, D), fan_in=D),
                ParamSpec(self.prefix + "up_proj.weight", (H, D), fan_in=D),
                ParamSpec(self.prefix + "down_proj.weight", (D, H), fan_in=H)]

    def load(self, get, compute_dtype, device):
        gu = interleave_gate_up(get(self.prefix + "gate_proj.weight"), get(self.prefix + "up_proj.weight"))
        self.w_gate_up = place(gu, compute_dtype, device)
        self.w_down = place(get(self.prefix + "down_proj.weight"), compute_dtype, device)

    def weight_bytes(self):
        return 3 * self.hidden * self.dim * self.w_down.element_size()

    def row_elements(self):
        return self.hidden

    def fuses_norm(self, norm, x, ctx):
        if not hasattr(norm, "fused") or ctx.mode not in ("decode", "prefill"):
            return False
        T = x.shape[0]
        if ctx.mode == "prefill":             # takes the norm's output where the product before has left it
            return kernels.can_add_norm(T, self.dim, self.w_down.dtype)
        return kernels.can_chain(T, self.dim, self.w_down.dtype) or kernels.can_add_norm(T, self.dim, self.w_down.dtype)

    def forward_prenorm(self, x, norm, ctx, emit_for=None):
        T = x.shape[0]
        mid = ctx.ws.get("ffn.hidden", (T, self.hidden), self.w_down.dtype)
        src = ctx.normed.pop(id(norm), None)
        if src is not None and src[1] is not None and kernels.can_chain(T, self.dim, self.w_down.dtype):
            xn, ss, eps = src
            kernels.gemm_chain(xn, self.w_gate_up, mid, self.gated, hidden=self.hidden, scale_from=(ss, eps))
        elif src is not None and src[1] is not None:          # 17..128 rows: prepared by the kernel that added the K slices
            xn, ss, eps = src
            self._gemm(ctx, xn, self.w_gate_up, mid, self.gated, hidden=self.hidden, scale_from=(ss, eps))
        elif src is not None:                     # the norm's output is ready
            self._gemm(ctx, src[0], self.w_gate_up, mid, self.gated, hidden=self.hidden)
        elif kernels.can_fuse_norm(T, self.dim, self.w_down.dtype):
            nw, eps = norm.fused()
            kernels.gemm_norm(x, nw, eps, self.w_gate_up, mid, self.gated, hidden=self.hidden)
        else:
            h = ctx.ws.get("block.h", (T, self.dim), ctx.act_dtype)
            norm.forward(x, h, ctx)
            self._gemm(ctx, h, self.w_gate_up, mid, self.gated, hidden=self.hidden)
        emit = self._emit_args(emit_for, ctx, T, self.dim)
        prepared = self._add_emit_args(emit_for, ctx, T, self.dim, self.hidden) if emit is None else None
        ready = self._add_norm_args(emit_for, ctx, T, self.dim, self.hidden) if emit is None and prepared is None else None
        if emit is not None and kernels.can_chain(T, self.hidden, mid.dtype):
            nw2, xn2, ss2, eps2 = emit
            kernels.gemm_chain(mid, self.w_down, x, kernels.EPI_ADD_F32, emit=(nw2, xn2, ss2))
            ctx.normed[id(emit_for)] = (xn2, ss2, eps2)
        elif prepared is not None:
            nw2, eps2, xn2, ss2, ws2 = prepared
            kernels.gemm_add_emit(mid, self.w_down, x, nw2, xn2, ss2, ws2)
            ctx.normed[id(emit_for)] = (xn2, ss2, eps2)
        elif ready is not None and kernels.can_add_norm(T, self.hidden, mid.dtype):
            nw2, eps2, h2, ws2 = ready
            kernels.gemm_add_norm(mid, self.w_down, x, nw2, eps2, h2, ws2)
            ctx.normed[id(emit_for)] = (h2, None, None)
        else:
            self._gemm(ctx, mid, self.w_down, x, kernels.EPI_ADD_F32)

    def forward(self, h, x, ctx):
        T = h.shape[0]
        mid = ctx.ws.get("ffn.hidden", (T, self.hidden), h.dtype)
        self._gemm(ctx, h, self.w_gate_up, mid, self.gated, hidden=self.hidden)
        self._gemm(ctx, mid, self.w_down, x, kernels.EPI_ADD_F32)
