"""Token embedding and the LM head.  The head is the embedding table itself
when tied (src/model.cpp:389-398); one copy on the device either way."""
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part


@part("embedding", "token_embedding")
class TokenEmbedding(Part):
    """x[t] = float(table[token[t]]), no scaling (src/infer.cpp:454-475)."""

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.vocab_size = int(spec.params["vocab_size"])
        self.table = None

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.vocab_size, self.dim), init="embedding")]

    def load(self, get, compute_dtype, device):
        self.table = place(get(self.prefix + "weight"), compute_dtype, device)

    def weight_bytes(self):
        return self.dim * self.table.element_size()          # one row per token

    def forward(self, tokens, x, ctx):
        return kernels.embed(self.table, tokens, x)


@part("head", "lm_head")
class LMHead(Part):
    """logits = W h in float32; W is the embedding table when tied (src/infer.cpp:508-521)."""

    def __init__(self, spec, dim, prefix, embedding=None):
        super().__init__(spec, dim, prefix)
        self.vocab_size = int(spec.params["vocab_size"])
        self.tied = bool(spec.params.get("tied", False))
        self.embedding = embedding
        self.weight = None
        if self.tied and embedding is None:
            raise ValueError("a tied head needs the embedding part")

    def param_specs(self):
        if self.tied:
            return []
        return [ParamSpec(self.prefix + "weight", (self.vocab_size, self.dim), init="linear", fan_in=self.dim)]

    def load(self, get, compute_dtype, device):
        self.weight = self.embedding.table if self.tied else place(get(self.prefix + "weight"), compute_dtype, device)

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()

    def fuses_norm(self, norm, x, ctx):
        if not hasattr(norm, "fused") or ctx.mode != "decode":
            return False
        if id(norm) in ctx.normed:
            return True                                   # whoever prepared it checked the shape
        return kernels.can_fuse_norm(x.shape[0], self.dim, self.weight.dtype)

    def forward_prenorm(self, x, norm, logits, ctx):
        """logits for every row of x (no row selection)."""
        src = ctx.normed.pop(id(norm), None)
        if src is not None and src[1] is None:            # the norm's output is ready
            return self._gemm(ctx, src[0], self.weight, logits, kernels.EPI_STORE_F32)
        if src is not None:
            xn, ss, eps = src
            if kernels.can_chain(xn.shape[0], self.dim, self.weight.dtype):
                return kernels.gemm_chain(xn, self.weight, logits, kernels.EPI_STORE_F32, scale_from=(ss, eps))
            return self._gemm(ctx, xn, self.weight, logits, kernels.EPI_STORE_F32, scale_from=(ss, eps))
        nw, eps = norm.fused()
        return kernels.gemm_norm(x, nw, eps, self.weight, logits, kernels.EPI_STORE_F32)

    def forward(self, h, logits, ctx):
        return self._gemm(ctx, h, self.weight, logits, kernels.EPI_STORE_F32)
