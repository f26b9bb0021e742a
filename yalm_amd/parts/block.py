"""The arrangement of a layer's parts.  `prenorm_residual` is the reference's
(src/infer.cpp:256-386): x += mixer(norm(x)); x += feed_forward(norm(x)), the
residual stream in float32 and no scaling of the residual adds.  next_norm is the
norm that reads the residual stream after this layer (the next layer's, or the final
one): a part that can prepares that norm's activations on the way."""
from .base import Part, build_part, part


@part("block", "prenorm_residual")
class PreNormResidualBlock(Part):
    def __init__(self, layer_spec, dim, prefix=""):
        super().__init__(None, dim, layer_spec.prefix)
        p = layer_spec.prefix
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm, dim, p)
        self.mixer = build_part("mixer", layer_spec.mixer, dim, p)
        self.feed_forward_norm = build_part("norm", layer_spec.feed_forward_norm, dim, p)
        self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, dim, p)

    def children(self):
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def first_norm(self):
        """The norm that reads the residual stream first when this layer runs (the layer before
        may prepare its activations), or None."""
        return self.mixer_norm

    def forward(self, x, ctx, line, writes_cache=True, next_norm=None):
        if self.mixer.fuses_norm(self.mixer_norm, x, ctx):
            self.mixer.forward_prenorm(x, self.mixer_norm, ctx, line, writes_cache,
                                       emit_for=self.feed_forward_norm)
        else:
            h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
            self.mixer_norm.forward(x, h, ctx)
            self.mixer.forward(h, x, ctx, line, writes_cache)
        if self.feed_forward.fuses_norm(self.feed_forward_norm, x, ctx):
            self.feed_forward.forward_prenorm(x, self.feed_forward_norm, ctx, emit_for=next_norm)
        else:
            h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
            self.feed_forward_norm.forward(x, h, ctx)
            self.feed_forward.forward(h, x, ctx)
