"""Grouped-query self-attention over the cache, with a position encoding that
it owns and an optional window.

Per token (src/infer.cpp:278-338): q, k, v = W h; q and k rotated at the token's
position; k and v stored in the cache; per query head h with KV head h // group:
scores q.k / sqrt(head_dim) over the visible keys, softmax in float32, mix of
the values; the output projection is added to the residual stream.  Key j is
visible to the query at position i iff j <= i and (window == 0 or i - j <
window or j < sinks) (the reference's kv_len rows, src/infer.cpp:486-488).

Sinks (src/infer.cpp:305-319: with a context of n the reference keeps positions
0 and 1 and the last n - 2, and turns the kept keys one position further every
step past n): a sink j that the window no longer covers is scored as if it lay
window + sinks - 1 - j positions behind the query, whatever the query's
position.  Its key is stored as it was rotated at j and turned by
i - (window + sinks - 1) when it is read.

The three projections are one matrix [q; k; v] (the reference fuses them by
pointer, src/infer.cu:290-337); q/k rows are re-ordered at load if the folder
keeps them half-split (convert.py:145-158)."""
import torch

from ..cache.manager import KVRequest
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, build_part, part

# decode attention is split over pages so that about this many workgroups run
TARGET_WORKGROUPS = 256
RESIDENT_WORKGROUPS = 512       # decode-attention workgroups that the chip holds at once (two a compute unit)
# A prompt step of fewer tokens rotates and stores token by token: the kernel that works a page-shaped tile at a
# time has a workgroup per (tile, head), too few to fill the chip below this (64 tokens: 4.78 against 4.46 ms a
# step, 128: 5.75 against 5.48, 256: 6.87 against 6.76, 384: the same)
ROPE_TILES_MIN_TOKENS = 320


def kv_tiles(n_tok):
    """The index tables a step of whole prompts needs for attention over its own keys and values, which are
    staged in page-shaped tiles of 64 positions: seq_tile0[B + 1], the first tile of each sequence (n_tiles in
    all), and tile_order, the order in which the attention kernel should take the tiles of queries."""
    import numpy as np
    tile0 = np.zeros(len(n_tok) + 1, dtype=np.int32)
    np.cumsum([(n + kernels.PAGE - 1) // kernels.PAGE for n in n_tok], out=tile0[1:])
    return {"seq_tile0": tile0, "tile_order": np.asarray(kernels.prefill_tile_order(n_tok), dtype=np.int32),
            "n_tiles": int(tile0[-1])}


kv_tiles.name = "kv_tiles"


@part("mixer", "gqa_attention")
class GQAttention(Part):
    prompt_tables = (kv_tiles,)

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.n_kv_heads = int(p["n_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.window = int(p.get("window", 0) or 0)
        self.sinks = int(p.get("sinks", 0) or 0)
        if self.sinks and self.window < self.sinks:
            raise ValueError("%d attention sinks need a window at least as wide (window %d)" % (self.sinks, self.window))
        if not 0 <= self.sinks <= kernels.MAX_SINKS:
            raise ValueError("%d attention sinks asked for, at most %d are supported" % (self.sinks, kernels.MAX_SINKS))
        if self.n_heads % self.n_kv_heads:
            raise ValueError("n_heads %d is no multiple of n_kv_heads %d" % (self.n_heads, self.n_kv_heads))
        if self.head_dim % 2 or self.head_dim > kernels.MAX_HEAD_DIM:
            raise ValueError("head_dim %d is not supported (even, at most %d)" % (self.head_dim, kernels.MAX_HEAD_DIM))
        self.q_dim = self.n_heads * self.head_dim
        self.kv_dim = self.n_kv_heads * self.head_dim
        self.position = build_part("position", p["position"], dim, prefix)
        self.wqkv = None
        self.wo = None

    def children(self):
        return [self.position]

    @property
    def score_bias(self):
        """The position part's term for every score by the distance of query and key (float32 [n_heads, distances]
        on the device), if it has one: a position encoding that is no rotation."""
        bias = getattr(self.position, "score_bias", None)
        if bias is not None and self.sinks:
            raise ValueError("attention sinks are scored without a score bias: the two do not go together")
        return bias

    def param_specs(self):
        D = self.dim
        return [ParamSpec(self.prefix + "q_proj.weight", (self.q_dim, D), fan_in=D),
                ParamSpec(self.prefix + "k_proj.weight", (self.kv_dim, D), fan_in=D),
                ParamSpec(self.prefix + "v_proj.weight", (self.kv_dim, D), fan_in=D),
                ParamSpec(self.prefix + "o_proj.weight", (D, self.q_dim), fan_in=self.q_dim)]

    def load(self, get, compute_dtype, device):
        wq = self.position.arrange_projection_rows(get(self.prefix + "q_proj.weight"), self.n_heads)
        wk = self.position.arrange_projection_rows(get(self.prefix + "k_proj.weight"), self.n_kv_heads)
        wv = get(self.prefix + "v_proj.weight")
        self.wqkv = place(torch.cat([wq, wk, wv], dim=0), compute_dtype, device)
        self.wo = place(get(self.prefix + "o_proj.weight"), compute_dtype, device)

    def weight_bytes(self):
        return (self.wqkv.numel() + self.wo.numel()) * self.wqkv.element_size()

    def cache_request(self):
        return KVRequest(self.n_kv_heads, self.head_dim, self.window, self.sinks)

    def row_elements(self):
        """The widest buffer a token has in this part: q, k and v side by side."""
        return self.q_dim + 2 * self.kv_dim

    def describe(self, compute_dtype):
        what = "attention, %d heads in %d groups of head size %d%s" % (
            self.n_heads, self.n_kv_heads, self.head_dim,
            (", window %d" % self.window if self.window else "") + (" + %d sinks" % self.sinks if self.sinks else ""))
        if compute_dtype != torch.bfloat16:
            return what + ": float32-arithmetic kernels", False
        if self.head_dim in kernels.MFMA_HEAD_DIMS:
            return what + ": matrix-core kernels", False
        return what + ": float32-arithmetic kernels on bfloat16 storage (the matrix-core kernels take head sizes " \
                      "of 16 to 128 in steps of 16, not %d): correct, several times slower" % self.head_dim, True

    def decode_splits(self, B, max_pages, ragged=False):
        mfma = self.head_dim in kernels.MFMA_HEAD_DIMS and not kernels.FORCE_SIMPLE
        if mfma:         # a workgroup of 4 waves per (split, KV head and up to 16 of its query heads, sequence), a page per wave at a time
            per = max(1, B * self.n_kv_heads * ((self.n_heads // self.n_kv_heads + 15) // 16))
            quarters = max(1, min((max_pages + 3) // 4, 4))
            if per > RESIDENT_WORKGROUPS:         # more than run at once: in quarters the last round is short
                return quarters
            even = max(1, min((max_pages + 3) // 4, TARGET_WORKGROUPS // per))
            # Sequences of very unequal lengths.  Where the workgroups stand two to a compute unit anyway, one split and
            # the rows in the order that pairs a long sequence with a short one; else splits of the longest sequence's
            # split size (the kernel cuts them so), enough of them that the long sequences' work spreads over the chip.
            if ragged and per <= TARGET_WORKGROUPS:
                return max(even, quarters)
            return even
        return max(1, min(max_pages, TARGET_WORKGROUPS // max(1, B * self.n_heads)))

    def fuses_norm(self, norm, x, ctx):
        if not hasattr(norm, "fused") or self.head_dim % 16:
            return False
        T = x.shape[0]
        if ctx.mode == "prefill":             # takes the norm's output where the product before has left it
            return kernels.can_add_norm(T, self.dim, self.wo.dtype)
        if ctx.mode != "decode":
            return False
        return kernels.can_chain(T, self.dim, self.wo.dtype) or kernels.can_add_norm(T, self.dim, self.wo.dtype)

    def forward_prenorm(self, x, norm, ctx, line, writes_cache=True, emit_for=None):
        """A decode step from the residual stream: norm, q/k/v, rotation and cache write in
        one kernel, attention over the cache, output projection added to x (which may
        prepare the activations of the next norm, emit_for)."""
        if ctx.mode == "prefill":                 # whole prompts: the norm, unless its output is ready, then the plain way
            src = ctx.normed.pop(id(norm), None)
            if src is not None and src[1] is None:
                h = src[0]
            else:
                h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
                norm.forward(x, h, ctx)
            return self.forward(h, x, ctx, line, writes_cache, emit_for=emit_for)
        if not writes_cache:                      # a reader of another entry's line: the plain way
            ctx.normed.pop(id(norm), None)
            h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
            norm.forward(x, h, ctx)
            return self.forward(h, x, ctx, line, writes_cache)
        T = x.shape[0]
        pos = self.position
        if pos.table is not None and ctx.max_position >= pos.n_positions:
            raise ValueError("position %d is beyond the %d positions the rotation table holds"
                             % (ctx.max_position, pos.n_positions))
        group = ctx.cache.group_of(line)
        k_pages, v_pages = group.line_pages(line)
        q = ctx.ws.get("attn.q", (T, self.q_dim), self.wo.dtype)
        src = ctx.normed.pop(id(norm), None)
        if src is not None and src[1] is not None and kernels.can_chain(T, self.dim, self.wo.dtype):
            xn, ss, eps = src
            kernels.gemm_chain_qkv_rope(xn, (ss, eps), self.wqkv, q, k_pages, v_pages, group.table, group.ring_pages,
                                        ctx.tok_pos, ctx.seq_slot, pos.table, self.n_heads, self.n_kv_heads,
                                        self.head_dim, pos.rotary_dim)
        elif src is None and kernels.can_fuse_norm(T, self.dim, self.wo.dtype):
            nw, eps = norm.fused()
            kernels.gemm_norm_qkv_rope(x, nw, eps, self.wqkv, q, k_pages, v_pages, group.table, group.ring_pages,
                                       ctx.tok_pos, ctx.seq_slot, pos.table, self.n_heads, self.n_kv_heads,
                                       self.head_dim, pos.rotary_dim)
        else:             # the norm's output is ready or prepared, or the rows are too many for one kernel
            scale = None
            if src is not None and src[1] is not None:        # prepared: the product's sums are scaled row by row
                h, scale = src[0], (src[1], src[2])
            elif src is not None:
                h = src[0]
            else:
                h = ctx.ws.get("block.h", (T, self.dim), ctx.act_dtype)
                norm.forward(x, h, ctx)
            n_qkv = self.q_dim + 2 * self.kv_dim
            if kernels.can_gemm_partial(T, self.dim, h.dtype):
                # the GEMM's K slices go to the rotation kernel as they are, which adds them: no kernel in between
                qkv = ctx.ws.get("gemm.partial", (kernels.fused_workspace_floats(T, n_qkv, self.dim),), torch.float32)
                slices = kernels.gemm_partial(h, self.wqkv, qkv, scale_from=scale)
            else:
                qkv = ctx.ws.get("attn.qkv", (T, n_qkv), torch.float32)
                self._gemm(ctx, h, self.wqkv, qkv, kernels.EPI_STORE_F32, scale_from=scale)
                slices = 1
            kernels.rope_kv_write(qkv, q, None, None, None, k_pages, v_pages, group.table, group.ring_pages,
                                  ctx.tok_seq, ctx.tok_pos, ctx.seq_slot, ctx.seq_len, pos.table, self.n_heads,
                                  self.n_kv_heads, self.head_dim, pos.rotary_dim, slices=slices)
        o = ctx.ws.get("attn.o", (T, self.q_dim), self.wo.dtype)
        self._decode_attention(q, o, ctx, group, line, k_pages, v_pages, True)
        emit = self._emit_args(emit_for, ctx, T, self.dim)
        prepared = self._add_emit_args(emit_for, ctx, T, self.dim, self.q_dim) if emit is None else None
        ready = self._add_norm_args(emit_for, ctx, T, self.dim, self.q_dim) if emit is None and prepared is None else None
        if emit is not None and kernels.can_chain(T, self.q_dim, o.dtype):
            nw2, xn2, ss2, eps2 = emit
            kernels.gemm_chain(o, self.wo, x, kernels.EPI_ADD_F32, emit=(nw2, xn2, ss2))
            ctx.normed[id(emit_for)] = (xn2, ss2, eps2)
        elif prepared is not None:                # 17..128 rows: the K slices are added and the next norm prepared at once
            nw2, eps2, xn2, ss2, ws2 = prepared
            kernels.gemm_add_emit(o, self.wo, x, nw2, xn2, ss2, ws2)
            ctx.normed[id(emit_for)] = (xn2, ss2, eps2)
        elif ready is not None and kernels.can_add_norm(T, self.q_dim, o.dtype):
            nw2, eps2, h2, ws2 = ready
            kernels.gemm_add_norm(o, self.wo, x, nw2, eps2, h2, ws2)
            ctx.normed[id(emit_for)] = (h2, None, None)
        else:
            self._gemm(ctx, o, self.wo, x, kernels.EPI_ADD_F32)

    def _decode_attention(self, q, o, ctx, group, line, k_pages, v_pages, writes_cache):
        T = q.shape[0]
        n_splits = self.decode_splits(T, min(group.ring_pages, ctx.pages_bucket), ctx.ragged)
        partial = ctx.ws.get("attn.partial",
                             (kernels.attn_decode_workspace_floats(T, self.n_heads, self.head_dim, n_splits),),
                             torch.float32)
        sinks = None
        if self.sinks:       # taken in where the splits are merged; a sequence still at its first positions
            sink_k, sink_v = group.line_sinks(line)        # has just written a sink, which is stored on the way
            sinks = (sink_k, sink_v, self.position.table, self.position.rotary_dim, writes_cache)
        kernels.attn_decode(q, k_pages, v_pages, group.table, group.ring_pages, ctx.seq_slot, ctx.seq_len, o, partial,
                            self.n_heads, self.n_kv_heads, self.head_dim, self.window, n_splits, sinks=sinks,
                            step_max_len=ctx.step_max_len, seq_order=ctx.seq_order, score_bias=self.score_bias)

    def forward(self, h, x, ctx, line, writes_cache=True, emit_for=None):
        T = h.shape[0]
        act = h.dtype
        ws = ctx.ws
        pos = self.position
        if pos.table is not None and ctx.max_position >= pos.n_positions:
            raise ValueError("position %d is beyond the %d positions the rotation table holds"
                             % (ctx.max_position, pos.n_positions))
        prefill = ctx.mode == "prefill"
        n_qkv = self.q_dim + 2 * self.kv_dim
        slices = 1
        if prefill and kernels.can_gemm_partial(T, self.dim, act):
            # the product's K slices (a short prompt's has some) go to the rotation kernel as they are, which adds them
            qkv = ws.get("gemm.partial", (kernels.fused_workspace_floats(T, n_qkv, self.dim),), torch.float32)
            slices = kernels.gemm_partial(h, self.wqkv, qkv)
        else:
            qkv = ws.get("attn.qkv", (T, n_qkv), torch.float32)
            self._gemm(ctx, h, self.wqkv, qkv, kernels.EPI_STORE_F32)
        q = ws.get("attn.q", (T, self.q_dim), act)
        group = ctx.cache.group_of(line)
        k_pages, v_pages = group.line_pages(line)
        if prefill:
            # the step's own keys and values in page format; a line that later entries read
            # keeps them for those entries
            tiles = ctx.tables["kv_tiles"]
            seq_tile0, n_tiles = tiles["seq_tile0"], tiles["n_tiles"]
            tag = "attn.stage%d" % line if ctx.line_is_shared(line) else "attn.stage"
            kst = ws.get(tag + ".k", (n_tiles, self.n_kv_heads, kernels.PAGE, self.head_dim), act)
            vst = ws.get(tag + ".v", (n_tiles, self.n_kv_heads, self.head_dim, kernels.PAGE), act)
        else:
            kst = vst = seq_tile0 = None
        if writes_cache:
            done = prefill and T >= ROPE_TILES_MIN_TOKENS and kernels.rope_kv_write_tiles(
                qkv, q, kst, vst, ctx.cu_seqlens, seq_tile0, k_pages, v_pages, group.table, group.ring_pages,
                ctx.seq_slot, ctx.seq_len, pos.table, self.n_heads, self.n_kv_heads, self.head_dim, pos.rotary_dim,
                slices=slices)
            if not done:
                kernels.rope_kv_write(qkv, q, kst, vst, seq_tile0, k_pages, v_pages, group.table,
                                      group.ring_pages, ctx.tok_seq, ctx.tok_pos, ctx.seq_slot, ctx.seq_len, pos.table,
                                      self.n_heads, self.n_kv_heads, self.head_dim, pos.rotary_dim, slices=slices)
        else:
            kernels.rope_kv_write(qkv, q, None, None, None, None, None, None, 0, ctx.tok_seq, ctx.tok_pos,
                                  ctx.seq_slot, ctx.seq_len, pos.table, self.n_heads, self.n_kv_heads, self.head_dim,
                                  pos.rotary_dim, slices=slices)
        o = ws.get("attn.o", (T, self.q_dim), act)
        if prefill:
            lse = ws.get("attn.lse", (T, self.n_heads), torch.float32) if self.sinks else None
            # with sinks the result is kept unrounded too, so that the row with the sinks mixed in is rounded once
            o32 = ws.get("attn.o32", (T, self.q_dim), torch.float32) if self.sinks and act != torch.float32 else None
            if self.sinks and writes_cache:
                sink_k, sink_v = group.line_sinks(line)
                kernels.sink_store(kst, vst, seq_tile0, ctx.seq_slot, ctx.seq_len, sink_k, sink_v)
            kernels.attn_prefill(q, kst, vst, o, ctx.cu_seqlens, seq_tile0, ctx.tok_seq, ctx.tok_pos,
                                 self.n_heads, self.n_kv_heads, self.head_dim, self.window, tiles.get("tile_order"),
                                 lse=lse, out_f32=o32, score_bias=self.score_bias)
            if self.sinks:
                sink_k, sink_v = group.line_sinks(line)
                kernels.attn_sink_mix(q, o, lse, sink_k, sink_v, ctx.tok_seq, ctx.tok_pos, ctx.seq_slot, pos.table,
                                      self.n_heads, pos.rotary_dim, self.window, src_f32=o32)
        else:
            self._decode_attention(q, o, ctx, group, line, k_pages, v_pages, writes_cache)
        ready = self._add_norm_args(emit_for, ctx, T, self.dim, self.q_dim) if prefill else None
        if ready is not None:                     # the product's K slices (or the product) are added with the next norm behind
            nw2, eps2, h2, ws2 = ready
            kernels.gemm_add_norm(o, self.wo, x, nw2, eps2, h2, ws2)
            ctx.normed[id(emit_for)] = (h2, None, None)
        else:
            self._gemm(ctx, o, self.wo, x, kernels.EPI_ADD_F32)
