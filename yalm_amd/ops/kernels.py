"""Python faces of the HIP kernels.  Each function checks on the host that the
operands have the shapes, dtypes and layout its kernel and grid assume (a
mismatch is an error here, never a wrong result or a fault on the device), then
launches on torch's current stream.  Tensors must live on the GPU; there is no
CPU path."""
import ctypes

import numpy as np

import torch

from . import library

PAGE = 64                       # tokens per cache page (csrc/common.h)
PREFILL_MIXED_TILES = 64        # prefill_tile_order mixes the sequences of a step up to this many tiles
MAX_HEAD_DIM = 256
MFMA_HEAD_DIMS = tuple(range(16, 129, 16))   # head sizes of the matrix-core attention kernels (others: float32 arithmetic)

_DT = {torch.float32: 0, torch.bfloat16: 1}

# set by tests to run the float32-arithmetic kernels also for bfloat16 storage
FORCE_SIMPLE = False


def dtype_code(dtype):
    try:
        return _DT[dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (float32 or bfloat16)" % dtype) from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream's handle (a launch asks for it: the short way, where torch has one)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(t, name, dtype=None, shape=None):
    """The address of a tensor after the checks every kernel argument gets; the first lines are the way of an
    argument that passes them (a step of a short prompt is a few hundred launches that the host has to keep up with)."""
    try:
        fine = t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype)
    except AttributeError:
        fine = False
    if fine:
        if shape is None:
            return t.data_ptr()
        have = t.shape
        if len(have) == len(shape):
            for s, d in zip(shape, have):
                if s is not None and s != d:
                    break
            else:
                return t.data_ptr()
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s: expected a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s: the HIP kernels need GPU tensors (got %s); there is no CPU path" % (name, t.device))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if dtype is not None and t.dtype != dtype:
        raise TypeError("%s: expected %s, got %s" % (name, dtype, t.dtype))
    if shape is not None:
        if t.dim() != len(shape) or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise ValueError("%s: expected shape %s, got %s" % (name, list(shape), list(t.shape)))
    return t.data_ptr()


def _opt(t, name, dtype=None, shape=None):
    return None if t is None else _need(t, name, dtype, shape)


def embed(table, tokens, out):
    """out[t] = float(table[tokens[t]]); a negative token gives zeros."""
    V, D = table.shape
    T = tokens.shape[0]
    p_table = _need(table, "table")
    code = dtype_code(table.dtype)
    p_tok = _need(tokens, "tokens", torch.int32, (T,))
    p_out = _need(out, "out", torch.float32, (T, D))
    library.check(library.lib().yalm_embed(p_table, code, p_tok, p_out, T, D, V, _stream()), "embed")
    return out


def rmsnorm(x, weight, out, eps, row_index=None):
    """out[r] = x[row_index[r] or r] * rsqrt(mean(x^2) + eps) * weight."""
    D = x.shape[-1]
    R = out.shape[0]
    p_x = _need(x, "x", torch.float32, (None, D))
    p_w = _need(weight, "weight", None, (D,))
    p_o = _need(out, "out", None, (R, D))
    p_i = _opt(row_index, "row_index", torch.int32, (R,))
    if row_index is None and x.shape[0] < R:
        raise ValueError("rmsnorm: %d rows wanted of %d" % (R, x.shape[0]))
    library.check(library.lib().yalm_rmsnorm(p_x, p_w, dtype_code(weight.dtype), p_o, dtype_code(out.dtype), p_i, R, D,
                                             float(eps), _stream()), "rmsnorm")
    return out


EPI_STORE_F32, EPI_STORE, EPI_ADD_F32, EPI_GATED = 0, 1, 2, 3
EPI_GATED_GELU = 5          # as EPI_GATED with the reference's gelu (tanh form) in silu's place (src/infer.cpp:189-195)
GATED = (EPI_GATED, EPI_GATED_GELU)


GEMM_SPLIT_MAX = 16          # most K slices a GEMM uses, given the workspace


def gemm_workspace_floats(M, N, K):
    """Floats of scratch with which a bfloat16 gemm splits K across workgroups: 17..64 rows (to 128 with K a multiple of 64), and
    more rows than that while the output's tiles alone would leave most of the chip idle."""
    if 16 < M <= 64 or (M <= 128 and K % 64 == 0):
        return GEMM_SPLIT_MAX * M * N
    if M > 64:
        return int(library.lib().yalm_gemm_bf16_dma_workspace(M, N, K))
    return 0


def gemm(a, w, out, epilogue, hidden=0, workspace=None, scale_from=None):
    """out = a[M,K] @ w[N,K]^T with float32 accumulation and one of four epilogues:
    EPI_STORE_F32 (float32 out), EPI_STORE (out in a's dtype), EPI_ADD_F32
    (float32 out += product), EPI_GATED (w = gate/up rows interleaved in blocks of
    16; out[M, hidden] = silu(gate) * up in a's dtype; EPI_GATED_GELU: gelu(gate) * up).  workspace: float32 scratch of
    gemm_workspace_floats(M, N, K) elements, with which small batches split K.
    scale_from = (ss float32 [M, parts], eps), 17..128 bfloat16 rows only (can_add_emit): a was emitted by
    gemm_add_emit, and the sums are scaled by rsqrt(sum(ss[m]) / K + eps) per row before the epilogue."""
    M, K = a.shape
    N = w.shape[0]
    dt = a.dtype
    p_a = _need(a, "a", dt, (M, K))
    p_w = _need(w, "w", dt, (N, K))
    if epilogue in GATED:
        if hidden <= 0 or N != 32 * ((hidden + 15) // 16):
            raise ValueError("gated gemm: weight rows %d do not match hidden %d" % (N, hidden))
        p_o = _need(out, "out", dt, (M, hidden))
    elif epilogue == EPI_STORE:
        p_o = _need(out, "out", dt, (M, N))
    elif epilogue in (EPI_STORE_F32, EPI_ADD_F32):
        p_o = _need(out, "out", torch.float32, (M, N))
    else:
        raise ValueError("unknown epilogue %r" % (epilogue,))
    p_ws, n_ws = None, 0
    if workspace is not None:
        p_ws, n_ws = _need(workspace, "workspace", torch.float32), workspace.numel()
    if scale_from is not None:
        ss, eps = scale_from
        if dt != torch.bfloat16:
            raise TypeError("gemm: a row scale goes with bfloat16 activations")
        p_ss = _need(ss, "ss", torch.float32, (M, None))
        library.check(library.lib().yalm_gemm_scaled(p_a, p_w, p_o, p_ws, n_ws, M, N, K, epilogue, hidden, p_ss,
                                                     ss.shape[1], float(eps), _stream()), "gemm with a row scale")
        return out
    library.check(library.lib().yalm_gemm(p_a, p_w, p_o, p_ws, n_ws, M, N, K, dtype_code(dt), epilogue, hidden,
                                          1 if FORCE_SIMPLE else 0, _stream()), "gemm")
    return out


FUSED_NORM_MAX_ROWS = 8


def can_fuse_norm(M, K, dtype):
    """Whether gemm_norm / gemm_norm_qkv_rope take this shape (else: rmsnorm, then gemm)."""
    return dtype == torch.bfloat16 and 1 <= M <= FUSED_NORM_MAX_ROWS and K % 8 == 0 and \
        M * (K + 8) * 2 <= 72 * 1024 and not FORCE_SIMPLE


def gemm_norm(x, norm_w, eps, w, out, epilogue, hidden=0):
    """out = epilogue(rmsnorm(x, norm_w, eps) @ w^T) for at most 16 rows of the float32
    residual stream x; w bfloat16 [N, K], norm_w float32 [K]; EPI_STORE_F32, EPI_GATED or EPI_GATED_GELU.
    (Shapes: see can_fuse_norm.)"""
    M, K = x.shape
    N = w.shape[0]
    p_x = _need(x, "x", torch.float32, (M, K))
    p_n = _need(norm_w, "norm_w", torch.float32, (K,))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    if epilogue in GATED:
        if hidden <= 0 or N != 32 * ((hidden + 15) // 16):
            raise ValueError("gated gemm: weight rows %d do not match hidden %d" % (N, hidden))
        p_o = _need(out, "out", torch.bfloat16, (M, hidden))
    elif epilogue == EPI_STORE_F32:
        p_o = _need(out, "out", torch.float32, (M, N))
    else:
        raise ValueError("gemm_norm: epilogue %r is not offered" % (epilogue,))
    library.check(library.lib().yalm_gemm_norm(p_x, p_n, float(eps), p_w, p_o, M, N, K, epilogue, hidden, _stream()),
                  "gemm_norm")
    return out


PAGE_ROWS, PAGE_BLOCKS = 0, 1


def page_layout(head_dim):
    """How keys and values lie inside a cache page of a head: PAGE_ROWS (keys [row][element], values
    [element][row]) or, for head sizes that are multiples of 32, PAGE_BLOCKS (keys [element // 32][place of the
    row in the order the matrix-core decode attention takes rows][element % 32], values [row // 32][element]
    [row % 32]), in which every load instruction of that kernel reads 1 KB of consecutive bytes.  The tensors'
    shapes stay [pages, heads, PAGE, head_dim] and [pages, heads, head_dim, PAGE] either way."""
    return PAGE_BLOCKS if head_dim % 32 == 0 else PAGE_ROWS


def _layout(layout, head_dim):
    layout = page_layout(head_dim) if layout is None else int(layout)
    if layout not in (PAGE_ROWS, PAGE_BLOCKS) or (layout == PAGE_BLOCKS and head_dim % 32):
        raise ValueError("page layout %r does not fit head_dim %d" % (layout, head_dim))
    return layout


def gemm_norm_qkv_rope(x, norm_w, eps, wqkv, q_out, k_pages, v_pages, block_table, ring_pages, tok_pos, seq_slot,
                       cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, layout=None):
    """A decode step's rmsnorm + q/k/v projection + rotation + cache write in one kernel
    (row m is sequence m; see rope_kv_write for the operands)."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    if head_dim % 16:
        raise ValueError("gemm_norm_qkv_rope needs a head_dim that is a multiple of 16")
    M, K = x.shape
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    p_x = _need(x, "x", torch.float32, (M, K))
    p_n = _need(norm_w, "norm_w", torch.float32, (K,))
    p_w = _need(wqkv, "wqkv", torch.bfloat16, (Q + 2 * KV, K))
    p_q = _need(q_out, "q_out", torch.bfloat16, (M, Q))
    n_pages = k_pages.shape[0]
    p_kp = _need(k_pages, "k_pages", torch.bfloat16, (n_pages, n_kv_heads, PAGE, head_dim))
    p_vp = _need(v_pages, "v_pages", torch.bfloat16, (n_pages, n_kv_heads, head_dim, PAGE))
    p_bt = _need(block_table, "block_table", torch.int32, (None, None))
    stride = block_table.shape[1]
    if ring_pages <= 0 or ring_pages > stride:
        raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (M,))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (M,))
    n_pos, p_cs = 0, None
    if cos_sin is not None:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_gemm_norm_qkv_rope(
        p_x, p_n, float(eps), p_w, p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_tp, p_ss, p_cs, n_pos, M, K, n_heads,
        n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), _stream()), "gemm_norm_qkv_rope")


CHAIN_MAX_ROWS = 16


def can_chain(M, K, dtype):
    """Whether gemm_chain / gemm_chain_qkv_rope take this shape."""
    return dtype == torch.bfloat16 and 1 <= M <= CHAIN_MAX_ROWS and K % 8 == 0 and not FORCE_SIMPLE


def can_add_norm(M, K, dtype):
    """Whether gemm_add_norm takes this shape (the batches that gemm_chain leaves out)."""
    if dtype != torch.bfloat16 or FORCE_SIMPLE or M <= CHAIN_MAX_ROWS:
        return False
    return K % 8 == 0 if M <= 64 else K % 64 == 0


def fused_workspace_floats(M, N, K):
    """Floats of scratch for gemm_add_norm and gemm_partial: what lets the GEMM split K as it likes,
    and room for one whole product at least."""
    return max(gemm_workspace_floats(M, N, K), M * N)


def gemm_add_norm(a, w, x, norm_w, eps, h_out, workspace):
    """x float32 [M, N] += a[M, K] @ w[N, K]^T for more than 16 bfloat16 rows (more than 64: K a multiple
    of 64), and h_out bfloat16 [M, N] = RMSNorm(x_new) with the weights norm_w (float32 [N]): the residual add and the next norm in one.
    workspace: float32 scratch of gemm_workspace_floats(M, N, K) elements."""
    M, K = a.shape
    N = w.shape[0]
    p_a = _need(a, "a", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    p_x = _need(x, "x", torch.float32, (M, N))
    p_nw = _need(norm_w, "norm_w", torch.float32, (N,))
    p_h = _need(h_out, "h_out", torch.bfloat16, (M, N))
    if workspace is None or workspace.numel() < M * N:
        raise ValueError("gemm_add_norm needs a workspace of at least M * N floats")
    p_ws = _need(workspace, "workspace", torch.float32, None)
    library.check(library.lib().yalm_gemm_add_norm(p_a, p_w, p_x, p_ws, workspace.numel(), M, N, K, p_nw, float(eps),
                                                   p_h, _stream()), "gemm_add_norm")
    return h_out


def can_add_emit(M, K, dtype):
    """Whether gemm_add_emit takes this shape, and gemm / gemm_partial a row scale for M rows: batches beyond the
    norm chain of gemm_chain (16 rows) up to 128 rows."""
    return can_add_norm(M, K, dtype) and M <= 128


def gemm_add_emit_parts(N):
    """Columns of the partial sums of squares that gemm_add_emit leaves for rows of N columns."""
    return library.lib().yalm_gemm_add_emit_parts(int(N))


def gemm_add_emit(a, w, x, norm_w, xn_out, ss_out, workspace):
    """x float32 [M, N] += a[M, K] @ w[N, K]^T (shapes as gemm_add_norm), xn_out bfloat16 [M, N] = x_new * norm_w and
    ss_out float32 [M, gemm_add_emit_parts(N)] = partial sums of squares of x_new: the next norm prepared but not
    finished; its consumer scales its own sums (gemm / gemm_partial with scale_from)."""
    M, K = a.shape
    N = w.shape[0]
    p_a = _need(a, "a", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    p_x = _need(x, "x", torch.float32, (M, N))
    p_nw = _need(norm_w, "norm_w", torch.float32, (N,))
    p_xn = _need(xn_out, "xn_out", torch.bfloat16, (M, N))
    p_ss = _need(ss_out, "ss_out", torch.float32, (M, gemm_add_emit_parts(N)))
    if workspace is None or workspace.numel() < M * N:
        raise ValueError("gemm_add_emit needs a workspace of at least M * N floats")
    p_ws = _need(workspace, "workspace", torch.float32, None)
    library.check(library.lib().yalm_gemm_add_emit(p_a, p_w, p_x, p_ws, workspace.numel(), M, N, K, p_nw, p_xn, p_ss,
                                                   _stream()), "gemm_add_emit")
    return xn_out


def can_gemm_partial(M, K, dtype):
    """True if gemm_partial takes the shape (more than 16 rows of bfloat16; more than 64: K a multiple of 64)."""
    return can_add_norm(M, K, dtype)


def gemm_partial(a, w, workspace, scale_from=None):
    """The K slices of a[M,K] @ w[N,K]^T, more than 16 rows of bfloat16 (more than 64: K a multiple of
    64), left unadded in `workspace`
    ([slices][M][N] float32, flat; gemm_workspace_floats(M, N, K) elements let it split as it likes).
    Returns the number of slices, for a consumer that adds them (rope_kv_write).  scale_from as in gemm
    (every slice is scaled)."""
    M, K = a.shape
    N = w.shape[0]
    p_a = _need(a, "a", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    p_ws = _need(workspace, "workspace", torch.float32, (None,))
    if workspace.numel() < M * N:
        raise ValueError("workspace holds %d floats, at least %d are needed" % (workspace.numel(), M * N))
    slices = ctypes.c_int(0)
    if scale_from is not None:
        ss, eps = scale_from
        p_ss = _need(ss, "ss", torch.float32, (M, None))
        library.check(library.lib().yalm_gemm_partial_scaled(p_a, p_w, p_ws, workspace.numel(), M, N, K,
                                                             ctypes.byref(slices), p_ss, ss.shape[1], float(eps),
                                                             _stream()), "gemm_partial with a row scale")
        return slices.value
    library.check(library.lib().yalm_gemm_partial(p_a, p_w, p_ws, workspace.numel(), M, N, K, ctypes.byref(slices),
                                                  _stream()), "gemm_partial")
    return slices.value


def gemm_chain_parts(N):
    """Columns of the partial sums of squares that a producer with N output columns emits."""
    return library.lib().yalm_gemm_chain_parts(int(N))


def gemm_chain(x, w, out, epilogue, hidden=0, scale_from=None, emit=None):
    """Decode GEMM (bfloat16; at most CHAIN_MAX_ROWS rows: beyond that the per-workgroup sum of the
    partial sums costs more than a norm kernel) that chains norms.
    scale_from = (ss float32 [M, parts], eps): x was emitted as bfloat16(residual * norm weight) and
    the product is scaled by rsqrt(sum(ss[m]) / K + eps) per row.
    emit = (norm_w float32 [N], xn bfloat16 [M, N], ss float32 [M, gemm_chain_parts(N)]), with
    EPI_ADD_F32 only: also writes xn = bfloat16(out_new * norm_w) and the partial sums of squares."""
    M, K = x.shape
    N = w.shape[0]
    p_x = _need(x, "x", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    if epilogue in GATED:
        if hidden <= 0 or N != 32 * ((hidden + 15) // 16):
            raise ValueError("gated gemm: weight rows %d do not match hidden %d" % (N, hidden))
        p_o = _need(out, "out", torch.bfloat16, (M, hidden))
    elif epilogue in (EPI_STORE_F32, EPI_ADD_F32):
        p_o = _need(out, "out", torch.float32, (M, N))
    else:
        raise ValueError("gemm_chain: epilogue %r is not offered" % (epilogue,))
    p_ss, n_parts, eps = None, 0, 0.0
    if scale_from is not None:
        ss, eps = scale_from
        n_parts = ss.shape[1]
        p_ss = _need(ss, "ss", torch.float32, (M, n_parts))
    p_nw = p_xn = p_es = None
    if emit is not None:
        if epilogue != EPI_ADD_F32:
            raise ValueError("gemm_chain: only the residual-add epilogue emits")
        nw, xn, es = emit
        p_nw = _need(nw, "emit norm_w", torch.float32, (N,))
        p_xn = _need(xn, "emit xn", torch.bfloat16, (M, N))
        p_es = _need(es, "emit ss", torch.float32, (M, gemm_chain_parts(N)))
    library.check(library.lib().yalm_gemm_chain(p_x, p_w, p_o, M, N, K, epilogue, hidden, p_ss, n_parts, float(eps),
                                                p_nw, p_xn, p_es, _stream()), "gemm_chain")
    return out


def gemm_chain_qkv_rope(xn, scale_from, wqkv, q_out, k_pages, v_pages, block_table, ring_pages, tok_pos, seq_slot,
                        cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, layout=None):
    """gemm_norm_qkv_rope for activations a producer emitted (see gemm_chain)."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    if head_dim % 16:
        raise ValueError("gemm_chain_qkv_rope needs a head_dim that is a multiple of 16")
    M, K = xn.shape
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    ss, eps = scale_from
    n_parts = ss.shape[1]
    p_x = _need(xn, "xn", torch.bfloat16, (M, K))
    p_ss = _need(ss, "ss", torch.float32, (M, n_parts))
    p_w = _need(wqkv, "wqkv", torch.bfloat16, (Q + 2 * KV, K))
    p_q = _need(q_out, "q_out", torch.bfloat16, (M, Q))
    n_pages = k_pages.shape[0]
    p_kp = _need(k_pages, "k_pages", torch.bfloat16, (n_pages, n_kv_heads, PAGE, head_dim))
    p_vp = _need(v_pages, "v_pages", torch.bfloat16, (n_pages, n_kv_heads, head_dim, PAGE))
    p_bt = _need(block_table, "block_table", torch.int32, (None, None))
    stride = block_table.shape[1]
    if ring_pages <= 0 or ring_pages > stride:
        raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (M,))
    p_sl = _need(seq_slot, "seq_slot", torch.int32, (M,))
    n_pos, p_cs = 0, None
    if cos_sin is not None:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_gemm_chain_qkv_rope(
        p_x, p_ss, n_parts, float(eps), p_w, p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_tp, p_sl, p_cs, n_pos, M, K,
        n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), _stream()),
        "gemm_chain_qkv_rope")


def _check_heads(n_heads, n_kv_heads, head_dim):
    if n_heads % n_kv_heads != 0:
        raise ValueError("n_heads %d is no multiple of n_kv_heads %d" % (n_heads, n_kv_heads))
    if head_dim % 2 != 0 or head_dim <= 0 or head_dim > MAX_HEAD_DIM:
        raise ValueError("head_dim %d is not supported (even, at most %d)" % (head_dim, MAX_HEAD_DIM))


def rope_kv_write(qkv, q_out, k_stage, v_stage, seq_tile0, k_pages, v_pages, block_table, ring_pages, tok_seq, tok_pos,
                  seq_slot, seq_len, cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, slices=1, layout=None):
    """Rotates q and k by the angles of `cos_sin` at each token's position, writes q in
    q_out's dtype, k and v into the staging area (page format, tile seq_tile0[sequence] +
    position // PAGE) if one is given, and into the pages of the cache if given.
    slices > 1: qkv is the flat scratch of gemm_partial, [slices][T][q + 2 kv] float32, and the
    slices are added while they are read."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q_out.shape[0]
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    dt = q_out.dtype
    if slices == 1 and qkv.dim() == 2:
        p_qkv = _need(qkv, "qkv", torch.float32, (T, Q + 2 * KV))
    else:
        p_qkv = _need(qkv, "qkv", torch.float32, (None,))
        if slices < 1 or qkv.numel() < slices * T * (Q + 2 * KV):
            raise ValueError("qkv holds %d floats, %d slices of %d rows need %d"
                             % (qkv.numel(), slices, T, slices * T * (Q + 2 * KV)))
    p_q = _need(q_out, "q_out", dt, (T, Q))
    B = seq_slot.shape[0]
    p_ks = p_vs = p_t0 = None
    if k_stage is not None:
        n_tiles = k_stage.shape[0]
        p_ks = _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim))
        p_vs = _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE))
        p_t0 = _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,))
    n_pages = 0
    p_kp = p_vp = p_bt = None
    stride = 0
    if k_pages is not None:
        n_pages = k_pages.shape[0]
        p_kp = _need(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, head_dim))
        p_vp = _need(v_pages, "v_pages", dt, (n_pages, n_kv_heads, head_dim, PAGE))
        p_bt = _need(block_table, "block_table", torch.int32, (None, None))
        stride = block_table.shape[1]
        if ring_pages <= 0 or ring_pages > stride:
            raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_ts = _need(tok_seq, "tok_seq", torch.int32, (T,))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (T,))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (B,))
    p_sl = _need(seq_len, "seq_len", torch.int32, (B,))
    n_pos = 0
    p_cs = None
    if cos_sin is not None:
        if rotary_dim % 2 != 0 or rotary_dim > head_dim or rotary_dim <= 0:
            raise ValueError("rotary_dim %d does not fit head_dim %d" % (rotary_dim, head_dim))
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_rope_kv_write(
        p_qkv, p_q, p_ks, p_vs, p_t0, p_kp, p_vp, p_bt, stride, max(ring_pages, 1), p_ts, p_tp, p_ss, p_sl, p_cs,
        n_pos, T, n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), int(slices),
        dtype_code(dt), _stream()), "rope_kv_write")


def rope_kv_write_tiles(qkv, q_out, k_stage, v_stage, cu_seqlens, seq_tile0, k_pages, v_pages, block_table, ring_pages,
                        seq_slot, seq_len, cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, slices=1, layout=None):
    """rope_kv_write for a step of whole prompts (every sequence from position 0), a page-shaped
    tile of 64 positions at a time.  False if the kernel refuses the head size (the caller then
    uses rope_kv_write).  slices as in rope_kv_write."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q_out.shape[0]
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    dt = q_out.dtype
    if head_dim * (PAGE + 8) * dt.itemsize > 64 * 1024:
        return False
    B = seq_slot.shape[0]
    n_tiles = k_stage.shape[0]
    if slices == 1 and qkv.dim() == 2:
        p_qkv = _need(qkv, "qkv", torch.float32, (T, Q + 2 * KV))
    else:
        p_qkv = _need(qkv, "qkv", torch.float32, (None,))
        if slices < 1 or qkv.numel() < slices * T * (Q + 2 * KV):
            raise ValueError("qkv holds %d floats, %d slices of %d rows need %d"
                             % (qkv.numel(), slices, T, slices * T * (Q + 2 * KV)))
    p_q = _need(q_out, "q_out", dt, (T, Q))
    p_ks = _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim))
    p_vs = _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE))
    p_cu = _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,))
    p_t0 = _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,))
    n_pages, stride = 0, 0
    p_kp = p_vp = p_bt = None
    if k_pages is not None:
        n_pages = k_pages.shape[0]
        p_kp = _need(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, head_dim))
        p_vp = _need(v_pages, "v_pages", dt, (n_pages, n_kv_heads, head_dim, PAGE))
        p_bt = _need(block_table, "block_table", torch.int32, (None, None))
        stride = block_table.shape[1]
        if ring_pages <= 0 or ring_pages > stride:
            raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (B,))
    p_sl = _need(seq_len, "seq_len", torch.int32, (B,))
    n_pos = 0
    p_cs = None
    if cos_sin is not None:
        if rotary_dim % 2 != 0 or rotary_dim > head_dim or rotary_dim <= 0:
            raise ValueError("rotary_dim %d does not fit head_dim %d" % (rotary_dim, head_dim))
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_rope_kv_write_tiles(
        p_qkv, p_q, p_ks, p_vs, p_cu, p_t0, p_kp, p_vp, p_bt, stride, max(ring_pages, 1), p_ss, p_sl, p_cs, n_pos, T, B,
        n_tiles, n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), int(slices),
        dtype_code(dt), _stream()), "rope_kv_write_tiles")
    return True


def prefill_tile_order(n_tokens):
    """The order in which attn_prefill should take the tiles of a step whose sequences bring
    n_tokens tokens each: every second 64-token tile of a sequence (its workgroup covers the
    next one too).  A short step (at most 4,096 tokens with their padding) has the tiles that
    see the most keys first, whatever their sequence; a longer one goes sequence by sequence,
    the longest first and each from its end, so that the workgroups running together read the
    same keys (measured: 8 prompts of 2,048 tokens lose 4 % when their tiles are mixed).  A numpy
    int32 array for the host side of the step's metadata."""
    n_tiles = [(n + PAGE - 1) // PAGE for n in n_tokens]
    first = np.concatenate([[0], np.cumsum(n_tiles)])
    tiles, work = [], []
    for b in sorted(range(len(n_tiles)), key=lambda b: -n_tiles[b]):
        for tq in range((n_tiles[b] - 1) // 2 * 2, -1, -2):
            tiles.append(int(first[b]) + tq)
            work.append(min(tq + 2, n_tiles[b]))
    tiles = np.asarray(tiles, dtype=np.int32)
    if int(first[-1]) <= PREFILL_MIXED_TILES:
        tiles = tiles[np.argsort(-np.asarray(work, dtype=np.int64), kind="stable")]
    return tiles


def _bias(score_bias, n_heads):
    """(address, distances) of a score bias: float32 [n_heads, n] on the device, added to every score (scaled by
    1/sqrt(head_dim) already) as score_bias[head, min(query position - key position, n - 1)]; None: no bias.  What a
    position encoding that is no rotation needs (a slope per head times the distance, a learned table)."""
    if score_bias is None:
        return None, 0
    n = score_bias.shape[-1]
    return _need(score_bias, "score_bias", torch.float32, (n_heads, n)), n


def attn_prefill(q, k_stage, v_stage, out, cu_seqlens, seq_tile0, tok_seq, tok_pos, n_heads, n_kv_heads, head_dim,
                 window, tile_order=None, lse=None, out_f32=None, score_bias=None):
    """Causal (and windowed) attention of packed sequences that start at position 0, over
    the keys and values that rope_kv_write staged for this step.  tile_order (device int32,
    from prefill_tile_order) only changes the order of the work.  lse (float32 [T, n_heads], optional)
    receives the logarithm of every query's sum of exp(score), for attn_sink_mix; out_f32 (float32 [T, n_heads *
    head_dim], optional) the result before it is rounded to out's dtype, for the same.  score_bias: see _bias."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q.shape[0]
    dt = q.dtype
    B = cu_seqlens.shape[0] - 1
    n_tiles = k_stage.shape[0]
    p_q = _need(q, "q", dt, (T, n_heads * head_dim))
    p_k = _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim))
    p_v = _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE))
    p_o = _need(out, "out", dt, (T, n_heads * head_dim))
    p_cu = _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,))
    p_t0 = _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,))
    p_ts = _need(tok_seq, "tok_seq", torch.int32, (T,))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (T,))
    p_or, n_order = None, 0
    if tile_order is not None:
        n_order = tile_order.shape[0]
        p_or = _need(tile_order, "tile_order", torch.int32, (n_order,))
    p_lse = None if lse is None else _need(lse, "lse", torch.float32, (T, n_heads))
    p_o32 = _opt(out_f32, "out_f32", torch.float32, (T, n_heads * head_dim))
    library.check(library.lib().yalm_attn_prefill_lse(p_q, p_k, p_v, p_o, p_o32, p_lse, p_cu, p_t0, p_ts, p_tp, p_or, n_order,
                                                      T, B, n_tiles, n_heads, n_kv_heads, head_dim, int(window),
                                                      dtype_code(dt), 1 if FORCE_SIMPLE else 0,
                                                      *_bias(score_bias, n_heads), _stream()),
                  "attn_prefill")
    return out


def attn_decode_workspace_floats(B, n_heads, head_dim, n_splits):
    return library.lib().yalm_attn_decode_workspace(B, n_heads, head_dim, n_splits) // 4


def attn_decode(q, k_pages, v_pages, block_table, ring_pages, seq_slot, seq_len, out, partial, n_heads, n_kv_heads,
                head_dim, window, n_splits, lse=None, sinks=None, layout=None, step_max_len=None, seq_order=None,
                score_bias=None):
    """One query per sequence over the cache pages (laid out as `layout` says, default page_layout(head_dim));
    seq_len counts the new key.  lse as in attn_prefill.  step_max_len (int32 [1] on the device, optional): the
    length of the step's longest sequence, with which sequences of unequal lengths are cut into splits of equal
    size; seq_order (int32 [B] on the device, a permutation of the rows, optional): the order in which the
    workgroups take the rows (both change the division of the work and no result).  score_bias: see _bias (not with
    sinks).
    sinks = (sink_k, sink_v [slots, n_kv_heads, n_sinks, head_dim], cos_sin or None, rotary_dim, store):
    the attention sinks that a query's window no longer covers are taken in where the splits are merged
    (their keys turned by max(0, position - window - n_sinks + 1) positions with the table cos_sin); with
    `store` a token at one of its sequence's first n_sinks positions stores its key and value there."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    B = q.shape[0]
    dt = q.dtype
    n_pages = k_pages.shape[0]
    p_q = _need(q, "q", dt, (B, n_heads * head_dim))
    p_kp = _need(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, head_dim))
    p_vp = _need(v_pages, "v_pages", dt, (n_pages, n_kv_heads, head_dim, PAGE))
    p_bt = _need(block_table, "block_table", torch.int32, (None, None))
    stride = block_table.shape[1]
    if ring_pages <= 0 or ring_pages > stride:
        raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (B,))
    p_sl = _need(seq_len, "seq_len", torch.int32, (B,))
    p_o = _need(out, "out", dt, (B, n_heads * head_dim))
    need = attn_decode_workspace_floats(B, n_heads, head_dim, n_splits)
    p_w = _need(partial, "partial", torch.float32)
    if partial.numel() < need:
        raise ValueError("attn_decode workspace too small: %d floats, %d needed" % (partial.numel(), need))
    force = 1 if FORCE_SIMPLE else 0
    p_max = _opt(step_max_len, "step_max_len", torch.int32, (1,))
    p_ord = _opt(seq_order, "seq_order", torch.int32, (B,))
    if sinks is None:
        p_lse = None if lse is None else _need(lse, "lse", torch.float32, (B, n_heads))
        library.check(library.lib().yalm_attn_decode_lse(
            p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_ss, p_sl, p_o, p_lse, p_w, B, n_heads, n_kv_heads, head_dim,
            int(window), int(n_splits), n_pages, _layout(layout, head_dim), dtype_code(dt), force, p_max, p_ord,
            *_bias(score_bias, n_heads), _stream()), "attn_decode")
        return out
    if lse is not None:
        raise ValueError("attn_decode leaves no lse when it takes the sinks in itself")
    if score_bias is not None:
        raise ValueError("attention sinks are scored without a score bias: the two do not go together")
    sink_k, sink_v, cos_sin, rotary_dim, store = sinks
    n_slots, _, n_sinks, _ = sink_k.shape
    if window < n_sinks:
        raise ValueError("a window of %d is narrower than the %d sinks beside it" % (window, n_sinks))
    if block_table.shape[0] < n_slots:
        raise ValueError("the block table has %d rows for %d slots" % (block_table.shape[0], n_slots))
    n_pos, p_cs = 0, None
    if cos_sin is not None and rotary_dim > 0:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    library.check(library.lib().yalm_attn_decode_sinks(
        p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_ss, p_sl, p_o, p_w,
        _need(sink_k, "sink_k", dt, (n_slots, n_kv_heads, n_sinks, head_dim)),
        _need(sink_v, "sink_v", dt, (n_slots, n_kv_heads, n_sinks, head_dim)), 1 if store else 0, p_cs, n_pos, n_slots,
        int(rotary_dim) if p_cs is not None else 0, n_sinks, B, n_heads, n_kv_heads, head_dim, int(window),
        int(n_splits), n_pages, _layout(layout, head_dim), dtype_code(dt), force, p_max, p_ord, _stream()),
        "attn_decode with sinks")
    return out


MAX_SINKS = 16


def sink_store(k_stage, v_stage, seq_tile0, seq_slot, seq_len, sink_k, sink_v):
    """A step of whole prompts: copies the keys and values of positions < min(n_sinks, seq_len) from the
    staging area (sequence b's first tile is seq_tile0[b]) into the per-slot store sink_k, sink_v
    [slots, n_kv_heads, n_sinks, head_dim]."""
    n_slots, n_kv_heads, n_sinks, head_dim = sink_k.shape
    dt = sink_k.dtype
    n_tiles = k_stage.shape[0]
    B = seq_slot.shape[0]
    library.check(library.lib().yalm_sink_store(
        _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim)),
        _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE)),
        _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,)), _need(seq_slot, "seq_slot", torch.int32, (B,)),
        _need(seq_len, "seq_len", torch.int32, (B,)), _need(sink_k, "sink_k", dt),
        _need(sink_v, "sink_v", dt, (n_slots, n_kv_heads, n_sinks, head_dim)), B, n_tiles, n_slots, n_kv_heads,
        head_dim, n_sinks, dtype_code(dt), _stream()), "sink_store")


def attn_sink_mix(q, out, lse, sink_k, sink_v, tok_seq, tok_pos, seq_slot, cos_sin, n_heads, rotary_dim, window,
                  src_f32=None):
    """A step of whole prompts: adds the attention sinks that the window no longer covers to the attention
    result `out` (in place): for the token at position p the sinks j < min(n_sinks, p - window + 1), their
    keys turned by max(0, p - window - n_sinks + 1) positions with the table cos_sin (None: not turned).
    lse is what attn_prefill left for these queries; src_f32 (optional) its out_f32: the unrounded result is then read
    from there and the mixed row rounded once."""
    n_slots, n_kv_heads, n_sinks, head_dim = sink_k.shape
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q.shape[0]
    dt = q.dtype
    B = seq_slot.shape[0]
    if window < n_sinks:
        raise ValueError("a window of %d is narrower than the %d sinks beside it" % (window, n_sinks))
    n_pos, p_cs = 0, None
    if cos_sin is not None and rotary_dim > 0:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    library.check(library.lib().yalm_attn_sink_mix(
        _need(q, "q", dt, (T, n_heads * head_dim)), _need(out, "out", dt, (T, n_heads * head_dim)),
        _opt(src_f32, "src_f32", torch.float32, (T, n_heads * head_dim)),
        _need(lse, "lse", torch.float32, (T, n_heads)), _need(sink_k, "sink_k", dt),
        _need(sink_v, "sink_v", dt, (n_slots, n_kv_heads, n_sinks, head_dim)),
        _need(tok_seq, "tok_seq", torch.int32, (T,)), _need(tok_pos, "tok_pos", torch.int32, (T,)),
        _need(seq_slot, "seq_slot", torch.int32, (B,)), p_cs, n_pos, T, n_slots, n_heads, n_kv_heads, head_dim,
        int(rotary_dim) if p_cs is not None else 0, int(window), n_sinks, dtype_code(dt), _stream()), "attn_sink_mix")
    return out


def argmax(logits, out):
    R, V = logits.shape
    library.check(library.lib().yalm_argmax(_need(logits, "logits", torch.float32), _need(out, "out", torch.int32, (R,)),
                                            R, V, _stream()), "argmax")
    return out


def sample(logits, u, temperature, out):
    R, V = logits.shape
    if not temperature > 0:
        raise ValueError("temperature must be positive here (0 is argmax)")
    library.check(library.lib().yalm_sample(_need(logits, "logits", torch.float32), _need(u, "u", torch.float32, (R,)),
                                            float(temperature), _need(out, "out", torch.int32, (R,)), R, V, _stream()),
                  "sample")
    return out


def token_prob(logits, index, out):
    R, V = logits.shape
    library.check(library.lib().yalm_token_prob(_need(logits, "logits", torch.float32),
                                                _need(index, "index", torch.int32, (R,)),
                                                _need(out, "out", torch.float32, (R,)), R, V, _stream()), "token_prob")
    return out


def probe_read(src, workgroups=2048):
    """Queues a kernel that reads the tensor `src` once and does nothing else (a yardstick for what the
    memory gives a kernel).  Returns the bytes it reads."""
    n = src.numel() * src.element_size()
    piece = 256 * 8 * 16
    if n < piece:
        raise ValueError("probe_read needs at least %d bytes" % piece)
    out = _probe_scratch(src.device)
    library.check(library.lib().yalm_probe_read(_need(src, "src"), n, out.data_ptr(), int(workgroups), _stream()),
                  "probe_read")
    return n // piece * piece


def probe_mfma(shape, iters, workgroups=2048):
    """Queues a loop of matrix-core instructions on registers (shape 32: 32x32x16, 16: 16x16x32, bfloat16).
    Returns the floating-point operations of the launch."""
    out = _probe_scratch(torch.device("cuda", torch.cuda.current_device()))
    flops = ctypes.c_double(0.0)
    library.check(library.lib().yalm_probe_mfma(int(shape), int(iters), int(workgroups), out.data_ptr(),
                                                ctypes.byref(flops), _stream()), "probe_mfma")
    return flops.value


_probe_out = {}


def _probe_scratch(device):
    key = str(device)
    if key not in _probe_out:
        _probe_out[key] = torch.zeros(1024, dtype=torch.int32, device=device)
    return _probe_out[key]
