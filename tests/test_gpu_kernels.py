"""Each HIP kernel alone against its plain reference (the functions of
tests/plain/reference_model.py, or float64 library routines), at sizes other
than the engine's tiny models use: widths and vocabularies that are no powers
of two, head sizes in steps of 16, odd head counts and groups."""
import math

import numpy as np
import pytest
import torch

from plain import reference_model as R

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def K():
    from yalm_amd.ops import kernels
    return kernels


def rnd(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float64) * scale).to(dtype)


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 1.2e-2


ACTS = ["silu", "gelu"]


def gate(act):
    """The plain activation and the epilogue code of a gated product."""
    k = K()
    return {"silu": (R.silu, k.EPI_GATED), "gelu": (R.gelu, k.EPI_GATED_GELU)}[act]


def close(got, want, dtype, what, factor=1.0):
    got = got.detach().to("cpu", torch.float64)
    want = want.to(torch.float64)
    assert torch.isfinite(got).all(), what
    err = (got - want).abs().max().item()
    lim = factor * tol(dtype) * max(1.0, want.abs().max().item())
    assert err <= lim, "%s: max error %.3e, allowed %.3e" % (what, err, lim)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


# The cache's pages as the kernels store them.  Head sizes that are multiples of 32 are kept in blocks:
# keys [element // 32][place(row)][element % 32], values [row // 32][element][row % 32], where place(row) is
# the row's place in the order in which the matrix-core decode attention takes the rows of a page
# (16 rows an instruction: rows 8 a + b (+ 4) (+ 32) for a, b < 4).  Other head sizes: keys [row][element],
# values [element][row], which is also how the tests fill and read pages.
def row_place(r):
    return 16 * (2 * (r >> 5) + ((r >> 2) & 1)) + 4 * ((r >> 3) & 3) + (r & 3)


def pages_as_stored(kp, vp):
    """[pages, heads, 64, hd] keys and [pages, heads, hd, 64] values in rows -> the same shapes in storage order."""
    P, H, R, hd = kp.shape
    if hd % 32:
        return kp, vp
    place = torch.tensor([row_place(r) for r in range(R)], device=kp.device)
    ks = torch.empty_like(kp).view(P, H, hd // 32, R, 32)
    ks[:, :, :, place, :] = kp.view(P, H, R, hd // 32, 32).permute(0, 1, 3, 2, 4)
    vs = vp.view(P, H, hd, R // 32, 32).permute(0, 1, 3, 2, 4).contiguous()
    return ks.view(P, H, R, hd), vs.view(P, H, hd, R)


def pages_as_rows(kp, vp):
    """The inverse of pages_as_stored."""
    P, H, R, hd = kp.shape
    if hd % 32:
        return kp, vp
    place = torch.tensor([row_place(r) for r in range(R)], device=kp.device)
    kr = kp.view(P, H, hd // 32, R, 32)[:, :, :, place, :].permute(0, 1, 3, 2, 4).contiguous().view(P, H, R, hd)
    vr = vp.view(P, H, R // 32, hd, 32).permute(0, 1, 3, 2, 4).contiguous().view(P, H, hd, R)
    return kr, vr


def test_page_layout_helpers_invert_each_other():
    assert sorted(row_place(r) for r in range(64)) == list(range(64))
    assert [row_place(r) for r in (0, 1, 4, 8, 32, 63)] == [0, 1, 16, 4, 32, 63]
    for hd in (16, 64, 128):
        kp, vp = rnd((3, 2, 64, hd), 1), rnd((3, 2, hd, 64), 2)
        ks, vs = pages_as_stored(kp, vp)
        assert (hd % 32 != 0) == torch.equal(ks, kp)
        a, b = pages_as_rows(ks, vs)
        assert torch.equal(a, kp) and torch.equal(b, vp)
        if hd % 32 == 0:        # the formula of the layout, element by element
            for (r, e) in ((0, 0), (5, 33), (63, hd - 1), (36, 31)):
                assert ks[1, 1].reshape(-1)[((e // 32) * 64 + row_place(r)) * 32 + e % 32] == kp[1, 1, r, e]
                assert vs[1, 1].reshape(-1)[((r // 32) * hd + e) * 32 + r % 32] == vp[1, 1, e, r]


# ------------------------------------------------------------------ embedding, norm

@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    V, D = 37, 50
    table = rnd((V, D), 1, dtype)
    tokens = [0, 36, 5, 5, -1, 12]
    out = torch.full((len(tokens), D), 7.0, device=DEV)
    K().embed(table.to(DEV), i32(tokens), out)
    want = R.embedding(table, torch.tensor([t if t >= 0 else 0 for t in tokens]))
    want[4] = 0
    assert torch.equal(out.cpu().double(), want)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("D", [50, 1000, 4100, 4096, 8192, 8196, 2050])
def test_rmsnorm(D, w_dtype, out_dtype):
    x = rnd((7, D), 2, scale=3.0)
    w = (1 + 0.1 * rnd((D,), 3)).to(w_dtype)
    out = torch.empty((7, D), dtype=out_dtype, device=DEV)
    K().rmsnorm(x.to(DEV), w.to(DEV), out, 1e-3)
    close(out, R.rmsnorm(x, w, 1e-3), out_dtype, "rmsnorm")
    # gathered rows, one of them padding
    idx = [6, 0, -1, 3]
    out = torch.empty((4, D), dtype=out_dtype, device=DEV)
    K().rmsnorm(x.to(DEV), w.to(DEV), out, 1e-3, i32(idx))
    want = R.rmsnorm(x[[6, 0, 0, 3]], w, 1e-3)
    want[2] = 0
    close(out, want, out_dtype, "rmsnorm rows")
    # eps inside the root, added to the mean: ones with eps 3 -> 1/2
    one = torch.ones((1, D), device=DEV)
    out = torch.empty((1, D), dtype=torch.float32, device=DEV)
    K().rmsnorm(one, torch.ones(D, device=DEV), out, 3.0)
    assert torch.allclose(out.cpu(), torch.full((1, D), 0.5))


# ------------------------------------------------------------------ GEMM

# more than 64 rows: K a multiple of 64 takes the kernels that load straight into LDS (128x128 tiles up to 159 rows,
# 256-row tiles in a ring of LDS slots from 160), any other K the register-staged one
GEMM_SHAPES = [(1, 16, 256), (3, 70, 96), (64, 130, 264), (65, 64, 80), (200, 333, 1000), (8, 4096 + 16, 136),
               (130, 100, 50), (65, 64, 64), (200, 333, 1024), (300, 20480 + 8, 128), (513, 130, 192),
               # K a multiple of 64 (operands staged in LDS by DMA): few and odd rows, every row count of a stage
               (5, 70, 192), (16, 4112, 128), (9, 100, 64), (12, 33, 320), (8, 26000, 64), (13, 13000, 128),
               (3, 4096, 1024), (20, 70, 192), (33, 4112, 128), (50, 100, 64), (64, 333, 320),
               # widths of the big models' projections and rows that end inside a tile
               (8, 3072, 128), (5, 6144, 64), (16, 5120, 192), (3, 2048, 64), (7, 1000, 64), (9, 6010, 128),
               (1, 3080, 256), (12, 4100, 64)]


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,Kd", GEMM_SHAPES)
def test_gemm_store_and_add(M, N, Kd, dtype, simple):
    k = K()
    a = rnd((M, Kd), 4, dtype)
    w = rnd((N, Kd), 5, dtype, scale=1 / math.sqrt(Kd))
    want = a.double() @ w.double().T
    k.FORCE_SIMPLE = simple
    try:
        out = torch.empty((M, N), dtype=torch.float32, device=DEV)
        k.gemm(a.to(DEV), w.to(DEV), out, k.EPI_STORE_F32)
        close(out, want, torch.float32, "gemm f32 out", factor=4 if dtype == torch.float32 else 1)
        out2 = torch.empty((M, N), dtype=dtype, device=DEV)
        k.gemm(a.to(DEV), w.to(DEV), out2, k.EPI_STORE)
        close(out2, want, dtype, "gemm store")
        res = rnd((M, N), 6)
        acc = res.to(DEV).clone()
        k.gemm(a.to(DEV), w.to(DEV), acc, k.EPI_ADD_F32)
        close(acc, want + res.double(), torch.float32, "gemm add", factor=4 if dtype == torch.float32 else 1)
    finally:
        k.FORCE_SIMPLE = False


# (rows, columns or hidden width, K, epilogue): prompt-step shapes, one for every way the launcher of the 256-row
# tiles goes: tiles of 256, 192 and 128 columns, whole rounds of 256x256 followed by 256x128 tiles for the remaining
# columns (28,672 columns at 2,048 rows), K split over workgroups (few tiles), one, two and three k tiles (the
# start and the end of the ring of LDS slots), rows and columns that end inside a tile, many row tiles.
PROMPT_GEMMS = [(2048, 6144, 192, "f32"), (2048, 4096, 256, "add"), (1000, 4100, 320, "bf16"),
                (2048, 14336, 128, "gated"), (2048, 28672, 128, "f32"), (512, 4096, 4096, "add"),
                (384, 1000, 2048, "gated"), (160, 4096, 2048, "f32"), (8192, 512, 64, "f32"), (300, 700, 128, "add"),
                (257, 513, 192, "bf16"), (161, 96, 704, "gated"), (4096, 8192, 64, "bf16"), (700, 24000, 256, "add")]


@pytest.mark.parametrize("with_workspace", [True, False])
@pytest.mark.parametrize("M,N,Kd,epi", PROMPT_GEMMS)
def test_gemm_of_prompt_steps(M, N, Kd, epi, with_workspace):
    k = K()
    from yalm_amd.parts.swiglu import interleave_gate_up
    a = rnd((M, Kd), 91, torch.bfloat16).to(DEV)
    if epi == "gated":
        H = N
        wg = rnd((H, Kd), 92, torch.bfloat16, scale=1 / math.sqrt(Kd))
        wu = rnd((H, Kd), 93, torch.bfloat16, scale=1 / math.sqrt(Kd))
        w = interleave_gate_up(wg, wu).to(DEV)
        rows = w.shape[0]
        ad = a.double()
        act_fn, epi_code = gate("gelu" if M == 384 else "silu")
        want = (act_fn(ad @ wg.to(DEV).double().T) * (ad @ wu.to(DEV).double().T)).cpu()
    else:
        w = rnd((N, Kd), 92, torch.bfloat16, scale=1 / math.sqrt(Kd)).to(DEV)
        rows = N
        want = (a.double() @ w.double().T).cpu()
    floats = k.gemm_workspace_floats(M, rows, Kd) if with_workspace else 0
    ws = torch.full((floats,), float("nan"), device=DEV) if floats else None
    if epi == "gated":
        out = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        k.gemm(a, w, out, epi_code, hidden=N, workspace=ws)
        close(out, want, torch.bfloat16, "gated", factor=2.0)
    elif epi == "f32":
        out = torch.full((M, N), float("nan"), device=DEV)
        k.gemm(a, w, out, k.EPI_STORE_F32, workspace=ws)
        close(out, want, torch.float32, "float32 out")
    elif epi == "bf16":
        out = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        k.gemm(a, w, out, k.EPI_STORE, workspace=ws)
        close(out, want, torch.bfloat16, "bfloat16 out")
    else:
        res = rnd((M, N), 94)
        out = res.to(DEV).clone()
        k.gemm(a, w, out, k.EPI_ADD_F32, workspace=ws)
        close(out, want + res.double(), torch.float32, "residual add")


def test_gemm_of_a_prompt_step_is_the_same_with_and_without_k_slices():
    """A product in K slices agrees with the whole one within float32 rounding, and a launch repeats itself bit
    for bit."""
    k = K()
    M, N, Kd = 512, 4096, 4096
    a = rnd((M, Kd), 95, torch.bfloat16).to(DEV)
    w = rnd((N, Kd), 96, torch.bfloat16, scale=1 / 64).to(DEV)
    floats = k.gemm_workspace_floats(M, N, Kd)
    assert floats >= 2 * M * N                                   # few tiles: the launcher would split K
    outs = []
    for ws in (torch.empty((floats,), device=DEV), None):
        out = torch.empty((M, N), device=DEV)
        k.gemm(a, w, out, k.EPI_STORE_F32, workspace=ws)
        outs.append(out)
    # slices are added in order, but ((a + b) + (c + d)) is another rounding than (((a + b) + c) + d)
    close(outs[0], outs[1].double().cpu(), torch.float32, "sliced against whole")
    out = torch.empty((M, N), device=DEV)
    k.gemm(a, w, out, k.EPI_STORE_F32, workspace=None)
    assert torch.equal(out, outs[1])                             # and a launch repeats itself bit for bit


def _random_gemm_shapes(n, seed):
    """Row counts on both sides of every kernel's limits (16, 64, 128, 256), widths from tiny to several
    workgroups' worth, K with and without the factors (8, 64) that choose the path."""
    rng = np.random.default_rng(seed)
    rows = [1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300]
    shapes = []
    for _ in range(n):
        M = int(rng.choice(rows))
        N = int(rng.choice([1, 15, 16, 17, 100, 255, 256, 300, 1000, 2050, 4096, 6200]))
        K = int(rng.choice([8, 24, 64, 72, 128, 192, 200, 320, 1024, 1032]))
        shapes.append((M, N, K))
    return shapes


@pytest.mark.parametrize("with_workspace", [False, True])
def test_gemm_random_shapes(with_workspace):
    """Every dispatch branch of the bfloat16 GEMM at shapes nobody tuned for, all epilogues."""
    from yalm_amd.parts.swiglu import interleave_gate_up
    k = K()
    for idx, (M, N, Kd) in enumerate(_random_gemm_shapes(40, 7 if with_workspace else 8)):
        a = rnd((M, Kd), 1000 + idx, torch.bfloat16)
        w = rnd((N, Kd), 2000 + idx, torch.bfloat16, scale=1 / math.sqrt(Kd))
        want = a.double() @ w.double().T
        ad, wd = a.to(DEV), w.to(DEV)
        ws = None
        if with_workspace:
            n = k.gemm_workspace_floats(M, max(N, 32 * ((N + 15) // 16)), Kd)
            ws = torch.full((n,), float("nan"), device=DEV) if n else None
        tag = "M %d N %d K %d" % (M, N, Kd)
        out = torch.empty((M, N), device=DEV)
        k.gemm(ad, wd, out, k.EPI_STORE_F32, workspace=ws)
        close(out, want, torch.float32, tag + " f32")
        out2 = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        k.gemm(ad, wd, out2, k.EPI_STORE, workspace=ws)
        close(out2, want, torch.bfloat16, tag + " bf16")
        res = rnd((M, N), 3000 + idx)
        acc = res.to(DEV).clone()
        k.gemm(ad, wd, acc, k.EPI_ADD_F32, workspace=ws)
        close(acc, want + res.double(), torch.float32, tag + " add")
        wu = rnd((N, Kd), 4000 + idx, torch.bfloat16, scale=1 / math.sqrt(Kd))
        gated = R.silu(want) * (a.double() @ wu.double().T)
        outg = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        k.gemm(ad, interleave_gate_up(w, wu).to(DEV), outg, k.EPI_GATED, hidden=N, workspace=ws)
        close(outg, gated, torch.bfloat16, tag + " gated", factor=2.0)


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,H,D", [(1, 16, 64), (5, 176, 64), (70, 100, 96), (64, 1000, 264), (3, 14336, 128),
                                   (70, 100, 128), (300, 10300, 64), (260, 1000, 256), (7, 100, 192), (13, 7000, 128),
                                   (16, 13000, 64), (9, 3300, 320), (24, 100, 192), (61, 1000, 128),
                                   (513, 12820, 64), (2048, 14336, 64)])   # whole rounds of 256x256 tiles + a launch of 256x128
@pytest.mark.parametrize("act", ACTS)
def test_gemm_gated(M, H, D, dtype, simple, act):
    from yalm_amd.parts.swiglu import interleave_gate_up
    k = K()
    x = rnd((M, D), 7, dtype)
    wg = rnd((H, D), 8, dtype, scale=1 / math.sqrt(D))
    wu = rnd((H, D), 9, dtype, scale=1 / math.sqrt(D))
    g = x.double() @ wg.double().T
    u = x.double() @ wu.double().T
    act_fn, epi_code = gate(act)
    want = act_fn(g) * u
    k.FORCE_SIMPLE = simple
    try:
        out = torch.empty((M, H), dtype=dtype, device=DEV)
        k.gemm(x.to(DEV), interleave_gate_up(wg, wu).to(DEV), out, epi_code, hidden=H)
        close(out, want, dtype, "gated gemm")
    finally:
        k.FORCE_SIMPLE = False


def test_gemm_vector_of_the_reference():
    """src/test.cpp:157-168: n = 256 inputs, d = 16 outputs, N(0,1), absolute 1e-4."""
    k = K()
    for seed in (0, 1):
        w = rnd((16, 256), seed)
        x = rnd((1, 256), seed + 10)
        out = torch.empty((1, 16), device=DEV)
        k.gemm(x.to(DEV), w.to(DEV), out, k.EPI_STORE_F32)
        assert (out.cpu().double() - x.double() @ w.double().T).abs().max() < 1e-4


# ------------------------------------------------------------------ rotation + cache write

def make_table(n_pos, hd, rd, theta):
    f = R.rope_inv_freq(hd, rd, theta)[: rd // 2]
    ang = torch.arange(n_pos, dtype=torch.float64)[:, None] * f[None, :]
    return torch.stack([torch.cos(ang), torch.sin(ang)], -1).float().contiguous()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,rd", [(4, 2, 16, 16), (3, 1, 48, 48), (6, 3, 32, 16), (2, 2, 128, 128)])
def test_rope_kv_write(n_heads, n_kv, hd, rd, dtype):
    k = K()
    PAGE = k.PAGE
    n_pages, n_slots, ring = 9, 4, 3
    # two sequences: slot 2 with positions 60..69 (crosses a page), slot 0 with positions 0..4
    pos = list(range(60, 70)) + list(range(5))
    seq = [0] * 10 + [1] * 5
    T = len(pos)
    Q, KV = n_heads * hd, n_kv * hd
    qkv = rnd((T, Q + 2 * KV), 11)
    table = make_table(80, hd, rd, 10000.0)
    bt = torch.full((n_slots, ring), -1, dtype=torch.int32)
    bt[2, 0], bt[2, 1], bt[0, 0] = 5, 7, 1
    page_of = {0: {0: 5, 1: 7}, 1: {0: 1}}
    tile_of = {0: {0: 0, 1: 1}, 1: {0: 2}}            # staging: sequence 0 has tiles 0, 1; sequence 1 tile 2
    kp = torch.zeros((n_pages, n_kv, PAGE, hd), dtype=dtype, device=DEV)
    vp = torch.zeros((n_pages, n_kv, hd, PAGE), dtype=dtype, device=DEV)
    ks = torch.zeros((3, n_kv, PAGE, hd), dtype=dtype, device=DEV)
    vs = torch.zeros((3, n_kv, hd, PAGE), dtype=dtype, device=DEV)
    q_out = torch.empty((T, Q), dtype=dtype, device=DEV)
    k.rope_kv_write(qkv.to(DEV), q_out, ks, vs, i32([0, 2, 3]), kp, vp, bt.to(DEV), ring, i32(seq), i32(pos),
                    i32([2, 0]), i32([70, 5]), table.to(DEV), n_heads, n_kv, hd, rd)
    f = R.rope_inv_freq(hd, rd, 10000.0)
    p = torch.tensor(pos)
    q_want = R.rope_interleaved(qkv[:, :Q].reshape(T, n_heads, hd), p, f).reshape(T, Q)
    k_want = R.rope_interleaved(qkv[:, Q:Q + KV].reshape(T, n_kv, hd), p, f)
    v_want = qkv[:, Q + KV:].double().reshape(T, n_kv, hd)
    close(q_out, q_want, dtype, "q")
    kp, vp, ks, vs = kp.cpu(), vp.cpu(), ks.cpu(), vs.cpu()
    kp, vp = pages_as_rows(kp, vp)
    for t in range(T):
        page, tile, r = page_of[seq[t]][pos[t] // PAGE], tile_of[seq[t]][pos[t] // PAGE], pos[t] % PAGE
        close(ks[tile, :, r, :], k_want[t], dtype, "staged k")
        close(vs[tile, :, :, r], v_want[t], dtype, "staged v")
        assert torch.equal(kp[page, :, r, :], ks[tile, :, r, :])
        assert torch.equal(vp[page, :, :, r], vs[tile, :, :, r])
    # nothing else was touched
    touched = torch.zeros((n_pages, PAGE), dtype=torch.bool)
    for t in range(T):
        touched[page_of[seq[t]][pos[t] // PAGE], pos[t] % PAGE] = True
    assert (kp.float().abs().sum(dim=(1, 3)) > 0).equal(touched)


@pytest.mark.parametrize("M,n_heads,n_kv,hd,D", [(17, 4, 2, 16, 4096), (40, 3, 1, 48, 1024), (64, 8, 2, 128, 264),
                                                 (33, 2, 2, 64, 64), (65, 8, 2, 128, 4096), (200, 3, 1, 48, 1024),
                                                 (130, 2, 2, 64, 64)])
def test_gemm_partial_and_rotation_that_adds_the_slices(M, n_heads, n_kv, hd, D):
    """q/k/v projection of 17..64 rows whose K slices stay unadded, and the rotation kernel that adds them
    while it reads: the same q and cache pages as the product, added first, gives."""
    k = K()
    PAGE = k.PAGE
    Q, KV = n_heads * hd, n_kv * hd
    N = Q + 2 * KV
    h = rnd((M, D), 90, torch.bfloat16)
    w = rnd((N, D), 91, torch.bfloat16, scale=1 / math.sqrt(D))
    ws = torch.full((k.fused_workspace_floats(M, N, D),), float("nan"), device=DEV)
    slices = k.gemm_partial(h.to(DEV), w.to(DEV), ws)
    assert 1 <= slices and slices * M * N <= ws.numel()
    if D >= 1024 and N < 4096:
        assert slices > 1                                      # the case this test is for
    qkv = ws[:slices * M * N].reshape(slices, M, N).sum(dim=0)
    close(qkv, h.double() @ w.double().T, torch.float32, "sum of the slices")
    # one sequence per row, at positions 61 + row (so that some cross a page)
    table = make_table(200, hd, hd, 10000.0).to(DEV)
    pos = [61 + m for m in range(M)]
    bt = torch.arange(2 * M, dtype=torch.int32).reshape(M, 2).to(DEV)
    outs = []
    for source, n in ((qkv.contiguous(), 1), (ws, slices)):
        kp = torch.zeros((2 * M, n_kv, PAGE, hd), dtype=torch.bfloat16, device=DEV)
        vp = torch.zeros((2 * M, n_kv, hd, PAGE), dtype=torch.bfloat16, device=DEV)
        q = torch.zeros((M, Q), dtype=torch.bfloat16, device=DEV)
        k.rope_kv_write(source, q, None, None, None, kp, vp, bt, 2, i32(list(range(M))), i32(pos),
                        i32(list(range(M))), i32([p + 1 for p in pos]), table, n_heads, n_kv, hd, hd, slices=n)
        outs.append((q, kp, vp))
    for a, b, what in zip(outs[0], outs[1], ("q", "k pages", "v pages")):
        assert a.abs().sum() > 0
        close(b, a.double().cpu(), torch.bfloat16, what)       # the slices are added in another order than torch's sum
    with pytest.raises(ValueError):
        k.rope_kv_write(ws[:M * N], outs[0][0], None, None, None, None, None, None, 0, i32(list(range(M))), i32(pos),
                        i32(list(range(M))), i32([p + 1 for p in pos]), table, n_heads, n_kv, hd, hd, slices=2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,rd,lens,ring", [(4, 2, 16, 16, [5, 130, 64], 3), (3, 1, 48, 24, [200, 1], 2),
                                                          (8, 2, 128, 128, [70, 257], 8), (2, 2, 64, 64, [300], 3),
                                                          (2, 1, 16, 6, [70, 5], 2), (3, 3, 18, 10, [130], 3)])
def test_rope_kv_write_tiles(n_heads, n_kv, hd, rd, lens, ring, dtype):
    """Whole prompts, a tile of 64 positions at a time: the same q, staging area and cache pages as the
    per-token kernel (which the tests above pin to the plain rotation), also where a prompt ends inside a
    tile and where a ring keeps the last pages only."""
    k = K()
    PAGE = k.PAGE
    B, T = len(lens), sum(lens)
    Q, KV = n_heads * hd, n_kv * hd
    qkv = rnd((T, Q + 2 * KV), 21).to(DEV)
    table = make_table(max(lens) + 3, hd, rd, 10000.0).to(DEV)
    tiles = [(n + PAGE - 1) // PAGE for n in lens]
    tile0 = np.concatenate([[0], np.cumsum(tiles)])
    cu = np.concatenate([[0], np.cumsum(lens)])
    n_tiles, n_pages = int(tile0[-1]), B * ring + 2
    order = np.random.default_rng(5).permutation(n_pages)
    bt = torch.full((B + 1, ring), -1, dtype=torch.int32)
    slots = [B - b for b in range(B)]                         # slots B, B-1, ..., 1
    nxt = 0
    for b in range(B):
        for c in range(min(ring, tiles[b])):
            bt[slots[b], c] = int(order[nxt])
            nxt += 1
    seq = np.repeat(np.arange(B), lens)
    pos = np.concatenate([np.arange(n) for n in lens])

    def buffers():
        return (torch.zeros((n_pages, n_kv, PAGE, hd), dtype=dtype, device=DEV),
                torch.zeros((n_pages, n_kv, hd, PAGE), dtype=dtype, device=DEV),
                torch.zeros((n_tiles, n_kv, PAGE, hd), dtype=dtype, device=DEV),
                torch.zeros((n_tiles, n_kv, hd, PAGE), dtype=dtype, device=DEV),
                torch.zeros((T, Q), dtype=dtype, device=DEV))
    kp0, vp0, ks0, vs0, q0 = buffers()
    k.rope_kv_write(qkv, q0, ks0, vs0, i32(tile0), kp0, vp0, bt.to(DEV), ring, i32(seq), i32(pos), i32(slots),
                    i32(lens), table, n_heads, n_kv, hd, rd)
    kp1, vp1, ks1, vs1, q1 = buffers()
    assert k.rope_kv_write_tiles(qkv, q1, ks1, vs1, i32(cu), i32(tile0), kp1, vp1, bt.to(DEV), ring, i32(slots),
                                 i32(lens), table, n_heads, n_kv, hd, rd)
    for a, b, what in ((q0, q1, "q"), (ks0, ks1, "staged k"), (vs0, vs1, "staged v"), (kp0, kp1, "k pages"),
                       (vp0, vp1, "v pages")):
        assert torch.equal(a, b), what
    assert q0.abs().sum() > 0 and kp0.abs().sum() > 0
    # the K slices of a product instead of the product: added in order, as the per-token kernel adds them
    parts = torch.stack([rnd((T, Q + 2 * KV), 30 + s).to(DEV) for s in range(3)]).reshape(-1)
    kp2, vp2, ks2, vs2, q2 = buffers()
    k.rope_kv_write(parts, q2, ks2, vs2, i32(tile0), kp2, vp2, bt.to(DEV), ring, i32(seq), i32(pos), i32(slots),
                    i32(lens), table, n_heads, n_kv, hd, rd, slices=3)
    kp3, vp3, ks3, vs3, q3 = buffers()
    assert k.rope_kv_write_tiles(parts, q3, ks3, vs3, i32(cu), i32(tile0), kp3, vp3, bt.to(DEV), ring, i32(slots),
                                 i32(lens), table, n_heads, n_kv, hd, rd, slices=3)
    for a, b, what in ((q2, q3, "q"), (ks2, ks3, "staged k"), (vs2, vs3, "staged v"), (kp2, kp3, "k pages"),
                       (vp2, vp3, "v pages")):
        assert torch.equal(a, b), what + " from slices"
    assert not torch.equal(q2, q0)
    with pytest.raises(ValueError):
        k.rope_kv_write_tiles(parts[:2 * T * (Q + 2 * KV)], q3, ks3, vs3, i32(cu), i32(tile0), kp3, vp3, bt.to(DEV),
                              ring, i32(slots), i32(lens), table, n_heads, n_kv, hd, rd, slices=3)


def test_rope_kv_write_ring_keeps_the_last_pages_only():
    k = K()
    PAGE = k.PAGE
    n_kv, hd, ring = 1, 16, 2
    L = 3 * PAGE + 5                         # pages 0..3 exist, the ring keeps pages 2 and 3
    qkv = rnd((L, 2 * hd + hd), 12)          # one query head
    bt = torch.tensor([[4, 6]], dtype=torch.int32)
    kp = torch.zeros((8, n_kv, PAGE, hd), device=DEV)
    vp = torch.zeros((8, n_kv, hd, PAGE), device=DEV)
    q_out = torch.empty((L, hd), device=DEV)
    k.rope_kv_write(qkv.to(DEV), q_out, None, None, None, kp, vp, bt.to(DEV), ring, i32([0] * L),
                    i32(list(range(L))), i32([0]), i32([L]), None, 1, n_kv, hd, 0)
    kp = pages_as_rows(kp.cpu(), vp.cpu())[0]
    # absolute page 2 -> column 0 (page 4), page 3 -> column 1 (page 6)
    assert torch.equal(kp[4, 0], qkv[2 * PAGE:3 * PAGE, hd:2 * hd])
    assert torch.equal(kp[6, 0, :5], qkv[3 * PAGE:, hd:2 * hd])
    assert kp[6, 0, 5:].abs().sum() == 0
    assert torch.equal(q_out.cpu(), qkv[:, :hd])           # no table: no rotation


# ------------------------------------------------------------------ attention

def packed_attention_reference(q, k, v, lens, n_heads, n_kv, hd, window):
    outs, o = [], 0
    for n in lens:
        outs.append(R.attention(q[o:o + n].reshape(n, n_heads, hd), k[o:o + n].reshape(n, n_kv, hd),
                                v[o:o + n].reshape(n, n_kv, hd), window).reshape(n, n_heads * hd))
        o += n
    return torch.cat(outs)


def stage(kk, v, lens, n_kv, hd, dtype, poison=True):
    """Keys and values of packed sequences in the staging format of a prefill step."""
    PAGE = K().PAGE
    tile0 = np.concatenate([[0], np.cumsum([(n + PAGE - 1) // PAGE for n in lens])])
    fill = float("nan") if poison else 0.0
    ks = torch.full((int(tile0[-1]), n_kv, PAGE, hd), fill, dtype=dtype)
    vs = torch.full((int(tile0[-1]), n_kv, hd, PAGE), fill, dtype=dtype)
    o = 0
    for b, n in enumerate(lens):
        for p in range(n):
            ks[tile0[b] + p // PAGE, :, p % PAGE, :] = kk[o + p].reshape(n_kv, hd)
            vs[tile0[b] + p // PAGE, :, :, p % PAGE] = v[o + p].reshape(n_kv, hd)
        o += n
    return ks, vs, tile0


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,window,lens", [
    (4, 2, 16, 0, [5, 17, 1]), (3, 1, 32, 16, [2, 30, 70]), (6, 3, 48, 100, [130, 64]), (8, 2, 128, 0, [200]),
    (2, 2, 80, 7, [65, 3]), (5, 5, 64, 0, [129]), (4, 1, 64, 70, [300, 64, 1]), (8, 2, 128, 100, [17, 257]),
    (6, 2, 96, 50, [150, 64, 333]), (9, 3, 32, 0, [257, 1]), (4, 2, 112, 30, [200, 64]), (5, 1, 16, 0, [131, 7])])
def test_attn_prefill(n_heads, n_kv, hd, window, lens, dtype, simple):
    k = K()
    T = sum(lens)
    q = rnd((T, n_heads * hd), 13, dtype)
    kk = rnd((T, n_kv * hd), 14, dtype)
    v = rnd((T, n_kv * hd), 15, dtype)
    cu = np.concatenate([[0], np.cumsum(lens)])
    seq = np.repeat(np.arange(len(lens)), lens)
    pos = np.concatenate([np.arange(n) for n in lens])
    ks, vs, tile0 = stage(kk, v, lens, n_kv, hd, dtype)
    out = torch.empty((T, n_heads * hd), dtype=dtype, device=DEV)
    k.FORCE_SIMPLE = simple
    try:
        k.attn_prefill(q.to(DEV), ks.to(DEV), vs.to(DEV), out, i32(cu), i32(tile0), i32(seq), i32(pos), n_heads, n_kv,
                       hd, window)
    finally:
        k.FORCE_SIMPLE = False
    close(out, packed_attention_reference(q, kk, v, lens, n_heads, n_kv, hd, window), dtype, "prefill attention")


def masked_attention_float64(q, k, v, n_heads, n_kv, hd, window, bias=None):
    """softmax(q k^T / sqrt(hd) + mask) v for one sequence, all positions at once (float64).  bias ([n_heads,
    distances], optional): bias[h, min(i - j, distances - 1)] is added to the score of query i and key j."""
    n = q.shape[0]
    qh = q.double().reshape(n, n_heads, hd).transpose(0, 1)
    kh = k.double().reshape(n, n_kv, hd).transpose(0, 1).repeat_interleave(n_heads // n_kv, dim=0)
    vh = v.double().reshape(n, n_kv, hd).transpose(0, 1).repeat_interleave(n_heads // n_kv, dim=0)
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    visible = (j <= i) & ((i - j < window) if window else torch.ones((n, n), dtype=torch.bool))
    out = torch.empty((n_heads, n, hd), dtype=torch.float64)
    for h in range(n_heads):                          # a head at a time: [n, n] scores
        s = (qh[h] @ kh[h].T) / math.sqrt(hd)
        if bias is not None:
            s = s + bias[h].double()[(i - j).clamp(0, bias.shape[1] - 1)]
        s = s.masked_fill(~visible, float("-inf"))
        out[h] = torch.softmax(s, dim=-1) @ vh[h]
    return out.transpose(0, 1).reshape(n, n_heads * hd)


@pytest.mark.parametrize("n_heads,n_kv,hd,window,lens", [(40, 8, 64, 0, [1700]), (40, 8, 128, 300, [1500, 260]),
                                                         (32, 8, 128, 0, [2048]), (40, 8, 96, 0, [1500]),
                                                         (40, 10, 32, 200, [2200, 70]), (12, 4, 96, 0, [1300]),
                                                         (40, 8, 80, 0, [1500]), (24, 8, 48, 100, [2300, 65]),
                                                         (12, 4, 16, 0, [1300]), (40, 8, 112, 0, [1700])])
def test_attn_prefill_with_many_and_with_few_workgroups(n_heads, n_kv, hd, window, lens):
    """The matrix-core prefill kernel has two forms: workgroups of eight waves that take a tile's keys in two
    halves (launches of at most two workgroups a compute unit, the third case) and of four waves (more, the
    first two).  Both against a float64 masked softmax, itself checked against the plain implementation."""
    k = K()
    dtype = torch.bfloat16
    small = [rnd((70, 2 * 16), 31), rnd((70, 16), 32), rnd((70, 16), 33)]
    assert torch.allclose(masked_attention_float64(*small, 2, 1, 16, 9),
                          R.attention(small[0].reshape(70, 2, 16), small[1].reshape(70, 1, 16),
                                      small[2].reshape(70, 1, 16), 9).reshape(70, 32), atol=1e-12)
    T = sum(lens)
    q = rnd((T, n_heads * hd), 13, dtype)
    kk = rnd((T, n_kv * hd), 14, dtype)
    v = rnd((T, n_kv * hd), 15, dtype)
    cu = np.concatenate([[0], np.cumsum(lens)])
    seq = np.repeat(np.arange(len(lens)), lens)
    pos = np.concatenate([np.arange(n) for n in lens])
    ks, vs, tile0 = stage(kk, v, lens, n_kv, hd, dtype)
    out = torch.empty((T, n_heads * hd), dtype=dtype, device=DEV)
    order = i32(k.prefill_tile_order(lens))
    k.attn_prefill(q.to(DEV), ks.to(DEV), vs.to(DEV), out, i32(cu), i32(tile0), i32(seq), i32(pos), n_heads, n_kv, hd,
                   window, order)
    want, o = [], 0
    for n in lens:
        want.append(masked_attention_float64(q[o:o + n], kk[o:o + n], v[o:o + n], n_heads, n_kv, hd, window))
        o += n
    close(out, torch.cat(want), dtype, "prefill attention")


@pytest.mark.parametrize("n_heads,n_kv,hd,window,lens", [
    (8, 2, 128, 0, [200]), (5, 5, 64, 0, [129, 1, 640]), (4, 1, 64, 70, [300, 64, 1]), (40, 8, 128, 0, [700]),
    (24, 8, 64, 100, [1100, 90]), (8, 2, 128, 0, [2200, 90, 2100])])
def test_attn_prefill_in_a_given_tile_order(n_heads, n_kv, hd, window, lens):
    """The order of the tiles (with more workgroups than compute units it is folded) changes no
    bit of the result, and every position is still written."""
    k = K()
    dtype = torch.bfloat16
    T = sum(lens)
    q = rnd((T, n_heads * hd), 23, dtype).to(DEV)
    kk = rnd((T, n_kv * hd), 24, dtype)
    v = rnd((T, n_kv * hd), 25, dtype)
    cu = np.concatenate([[0], np.cumsum(lens)])
    seq = np.repeat(np.arange(len(lens)), lens)
    pos = np.concatenate([np.arange(n) for n in lens])
    ks, vs, tile0 = stage(kk, v, lens, n_kv, hd, dtype, poison=False)
    ks, vs = ks.to(DEV), vs.to(DEV)
    outs = []
    for order in (None, i32(k.prefill_tile_order(lens))):
        out = torch.full((T, n_heads * hd), float("nan"), dtype=dtype, device=DEV)
        k.attn_prefill(q, ks, vs, out, i32(cu), i32(tile0), i32(seq), i32(pos), n_heads, n_kv, hd, window, order)
        outs.append(out.cpu())
    assert not torch.isnan(outs[1].float()).any()
    assert torch.equal(outs[0], outs[1])


def paged_case(lens, n_kv, hd, window, dtype, seed, poison=True, stored=True):
    """Random keys/values of sequences of the given lengths laid out in pages the way
    the cache does (ring for a window), the rest of the pool poisoned with NaN.  stored=False: the pages in
    rows, for a caller that changes them before pages_as_stored."""
    k = K()
    PAGE = k.PAGE
    B = len(lens)
    full = max((n + PAGE - 1) // PAGE for n in lens)
    ring = min(full, (window + PAGE - 1) // PAGE + 1) if window else full
    n_pages = B * ring + 3
    kp = torch.full((n_pages, n_kv, PAGE, hd), float("nan") if poison else 0.0, dtype=dtype)
    vp = torch.full((n_pages, n_kv, hd, PAGE), float("nan") if poison else 0.0, dtype=dtype)
    order = np.random.default_rng(seed).permutation(n_pages)
    bt = torch.full((B + 2, ring), -1, dtype=torch.int32)
    slots = list(np.random.default_rng(seed + 1).permutation(B + 2)[:B])
    keys, vals = [], []
    nxt = 0
    for b, n in enumerate(lens):
        kb = rnd((n, n_kv, hd), seed + 10 * b, dtype)
        vb = rnd((n, n_kv, hd), seed + 10 * b + 1, dtype)
        keys.append(kb)
        vals.append(vb)
        last_ap = (n - 1) // PAGE
        for ap in range(max(0, last_ap - ring + 1), last_ap + 1):
            page = int(order[nxt])
            nxt += 1
            bt[slots[b], ap % ring] = page
            rows = range(ap * PAGE, min(n, (ap + 1) * PAGE))
            for p in rows:
                kp[page, :, p % PAGE, :] = kb[p]
                vp[page, :, :, p % PAGE] = vb[p]
    if stored:
        kp, vp = pages_as_stored(kp, vp)
    return kp, vp, bt, [int(s) for s in slots], ring, keys, vals


def one_query_reference(q, keys, vals, window):
    """The last position's attention (src/infer.cpp:218-250 per head over the visible rows)."""
    n_heads, hd = q.shape
    n, n_kv = keys.shape[0], keys.shape[1]
    lo = max(0, n - window) if window else 0
    out = torch.zeros((n_heads, hd), dtype=torch.float64)
    for h in range(n_heads):
        g = h // (n_heads // n_kv)
        p = R.attention_probs_one_query(q[h], keys[lo:n, g], hd)
        out[h] = p @ vals[lo:n, g].double()
    return out


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,window,lens,splits", [
    (4, 2, 16, 0, [5, 64, 65, 1], 1), (3, 1, 32, 16, [2, 30, 200], 2), (6, 3, 48, 100, [130, 640, 99], 3),
    (8, 2, 128, 0, [1000, 3], 7), (2, 2, 80, 0, [129], 4), (32, 8, 128, 0, [300], 2), (5, 5, 64, 70, [700, 64], 16),
    (6, 2, 96, 0, [900, 65, 2], 5), (12, 3, 96, 130, [400, 129], 2), (16, 1, 32, 0, [2000, 7], 9),
    (10, 2, 112, 0, [777, 3], 4), (9, 3, 80, 64, [500, 64], 3), (4, 4, 16, 0, [129, 1000], 5),
    (34, 2, 64, 0, [300, 65], 3), (40, 1, 128, 100, [700], 4), (51, 3, 32, 0, [129, 2], 2)])   # more than 16 heads a group
def test_attn_decode(n_heads, n_kv, hd, window, lens, splits, dtype, simple):
    _attn_decode_case(n_heads, n_kv, hd, window, lens, splits, dtype, simple, None)


@pytest.mark.parametrize("said", ["longest", 1, 100000])
@pytest.mark.parametrize("n_heads,n_kv,hd,window,lens,splits", [
    (8, 2, 128, 0, [1000, 3, 517, 64, 65], 4), (4, 1, 64, 0, [40, 900], 7), (5, 5, 64, 150, [700, 64, 164, 150, 128], 3),
    (8, 2, 128, 100, [164, 150, 128, 100, 99], 2)])
def test_attn_decode_with_the_length_of_the_longest_sequence(n_heads, n_kv, hd, window, lens, splits, said):
    """Splits of the longest sequence's split size: the same results, whatever length the step says its longest
    sequence has (the truth, too little, too much), also where a window makes a shorter sequence span more pages
    than the longest does; and the workgroups take the rows in another order than the rows'."""
    _attn_decode_case(n_heads, n_kv, hd, window, lens, splits, torch.bfloat16, False, max(lens) if said == "longest" else said)


def _attn_decode_case(n_heads, n_kv, hd, window, lens, splits, dtype, simple, step_max_len):
    k = K()
    B = len(lens)
    kp, vp, bt, slots, ring, keys, vals = paged_case(lens, n_kv, hd, window, dtype, 20)
    q = rnd((B, n_heads * hd), 16, dtype)
    # one padding row at the end
    qd = torch.cat([q, torch.zeros((1, n_heads * hd), dtype=dtype)]).to(DEV)
    out = torch.full((B + 1, n_heads * hd), 5.0, dtype=dtype, device=DEV)
    partial = torch.empty(k.attn_decode_workspace_floats(B + 1, n_heads, hd, splits), device=DEV)
    k.FORCE_SIMPLE = simple
    try:
        k.attn_decode(qd, kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, i32(slots + [-1]), i32(lens + [0]), out, partial,
                      n_heads, n_kv, hd, window, splits, step_max_len=None if step_max_len is None else i32([step_max_len]),
                      seq_order=None if step_max_len is None else i32(list(np.random.default_rng(5).permutation(B + 1))))
    finally:
        k.FORCE_SIMPLE = False
    for b, n in enumerate(lens):
        want = one_query_reference(q[b].double().reshape(n_heads, hd), keys[b], vals[b], window).reshape(-1)
        close(out[b], want, dtype, "decode attention row %d" % b)
    assert (out[B] == 0).all()


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,window,lens,n_bias", [
    (4, 2, 16, 0, [5, 130, 64], 200), (6, 3, 64, 70, [300, 1], 40), (8, 2, 128, 0, [257], 300), (3, 1, 48, 20, [90, 65], 7),
    (40, 8, 128, 0, [1500], 900), (40, 8, 96, 200, [1100, 1200], 64), (12, 4, 32, 0, [1300], 2000), (16, 1, 64, 0, [70, 2], 3),
    (6, 2, 80, 0, [300, 65], 100), (10, 5, 112, 40, [200], 50), (36, 2, 64, 0, [150, 70], 90)])
def test_attn_with_a_score_bias(n_heads, n_kv, hd, window, lens, n_bias, dtype, simple):
    """A term added to every score by the distance of query and key (a table a head, the last entry for every
    distance beyond it): prompt and decode kernels against a float64 softmax with the same term.  The table is steep
    (a slope a head plus noise), so that dropping it, taking another head's row or counting the distance from the
    wrong end changes the result by far more than rounding.  Both kinds of kernels take it; the long prompts reach
    each launch shape of the matrix-core prompt kernel."""
    k = K()
    k.FORCE_SIMPLE = simple
    try:
        _score_bias_case(k, n_heads, n_kv, hd, window, lens, n_bias, dtype)
    finally:
        k.FORCE_SIMPLE = False


def _score_bias_case(k, n_heads, n_kv, hd, window, lens, n_bias, dtype):
    slopes = 2.0 ** -(torch.arange(n_heads, dtype=torch.float64) * 3.0 / n_heads)
    bias = (-slopes[:, None] * torch.arange(n_bias, dtype=torch.float64)[None, :] + rnd((n_heads, n_bias), 77).double()).float()
    T = sum(lens)
    q = rnd((T, n_heads * hd), 13, dtype)
    kk = rnd((T, n_kv * hd), 14, dtype)
    v = rnd((T, n_kv * hd), 15, dtype)
    cu = np.concatenate([[0], np.cumsum(lens)])
    seq = np.repeat(np.arange(len(lens)), lens)
    pos = np.concatenate([np.arange(n) for n in lens])
    ks, vs, tile0 = stage(kk, v, lens, n_kv, hd, dtype)
    out = torch.empty((T, n_heads * hd), dtype=dtype, device=DEV)
    k.attn_prefill(q.to(DEV), ks.to(DEV), vs.to(DEV), out, i32(cu), i32(tile0), i32(seq), i32(pos), n_heads, n_kv, hd,
                   window, score_bias=bias.to(DEV))
    want, plain, o = [], [], 0
    for n in lens:
        want.append(masked_attention_float64(q[o:o + n], kk[o:o + n], v[o:o + n], n_heads, n_kv, hd, window, bias))
        plain.append(masked_attention_float64(q[o:o + n], kk[o:o + n], v[o:o + n], n_heads, n_kv, hd, window))
        o += n
    want, plain = torch.cat(want), torch.cat(plain)
    assert (want - plain).abs().max() > 0.1                     # the bias matters here
    close(out, want, dtype, "prefill attention with a score bias")
    # decode: the last query of every sequence over the cache pages
    B = len(lens)
    kp, vp, bt, slots, ring, keys, vals = paged_case(lens, n_kv, hd, window, dtype, 20)
    qd = rnd((B, n_heads * hd), 16, dtype)
    outd = torch.empty((B, n_heads * hd), dtype=dtype, device=DEV)
    partial = torch.empty(k.attn_decode_workspace_floats(B, n_heads, hd, 3), device=DEV)
    k.attn_decode(qd.to(DEV), kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, i32(slots), i32(lens), outd, partial,
                  n_heads, n_kv, hd, window, 3, score_bias=bias.to(DEV))
    for b, n in enumerate(lens):
        lo = max(0, n - window) if window else 0
        got_want = torch.zeros((n_heads, hd), dtype=torch.float64)
        for h in range(n_heads):
            g = h // (n_heads // n_kv)
            sc = keys[b][lo:n, g].double() @ qd[b].double().reshape(n_heads, hd)[h] / math.sqrt(hd)
            sc = sc + bias[h].double()[(n - 1 - torch.arange(lo, n)).clamp(0, n_bias - 1)]
            got_want[h] = torch.softmax(sc, dim=0) @ vals[b][lo:n, g].double()
        close(outd[b], got_want.reshape(-1), dtype, "decode attention with a score bias, row %d" % b)
    with pytest.raises(Exception):                              # a table for another number of heads
        k.attn_decode(qd.to(DEV), kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, i32(slots), i32(lens), outd, partial,
                      n_heads, n_kv, hd, window, 3, score_bias=bias[:-1].contiguous().to(DEV))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_decode_finds_a_far_key(dtype):
    """One key among a thousand, in an early page, carries all the weight: the query
    is scaled along that key, so a kernel that skips or misplaces a page misses it."""
    k = K()
    n_heads, n_kv, hd, n = 4, 1, 64, 1000
    for far in (3, 64 * 7 + 63, 998):
        kp, vp, bt, slots, ring, keys, vals = paged_case([n], n_kv, hd, 0, dtype, 30)
        q = (keys[0][far, 0].double() * 40.0).to(dtype).repeat(n_heads)[None]
        out = torch.empty((1, n_heads * hd), dtype=dtype, device=DEV)
        partial = torch.empty(k.attn_decode_workspace_floats(1, n_heads, hd, 5), device=DEV)
        k.attn_decode(q.to(DEV), kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, i32(slots), i32([n]), out, partial, n_heads,
                      n_kv, hd, 0, 5)
        got = out.cpu().double().reshape(n_heads, hd)
        assert (got - vals[0][far, 0].double()).abs().max() < 0.05, far

@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,window,n", [(64, 70, 300), (128, 64, 200), (128, 100, 513), (32, 16, 90), (48, 33, 200), (112, 64, 150), (16, 8, 70)])
def test_attn_window_edge_decides(hd, window, n, dtype, simple):
    """The key just outside the window has by far the largest score and a value of 1000; the key
    just inside has the next largest and a value of 7.  A window off by one, in either kernel,
    gives 1000 or loses the 7: among a hundred random keys it would hide in the rounding."""
    k = K()
    n_heads, n_kv = 4, 2
    unit = torch.zeros(hd, dtype=torch.float64)
    unit[3] = 1.0
    k.FORCE_SIMPLE = simple
    try:
        # decode: the query at position n - 1 sees positions n - window ... n - 1
        kp, vp, bt, slots, ring, keys, vals = paged_case([n], n_kv, hd, window, dtype, 40, stored=False)
        inside, outside = n - window, n - window - 1
        PAGE = k.PAGE
        for pos, strength, value in ((inside, 30.0, 7.0), (outside, 60.0, 1000.0)):
            page = int(bt[slots[0], (pos // PAGE) % ring])
            if pos // PAGE > (n - 1) // PAGE - ring:          # the ring still holds this position's page
                kp[page, :, pos % PAGE, :] = (unit * strength).to(dtype)
                vp[page, :, :, pos % PAGE] = value
        kp, vp = pages_as_stored(kp, vp)
        q = (unit * 8.0).to(dtype).repeat(n_heads)[None]
        out = torch.empty((1, n_heads * hd), dtype=dtype, device=DEV)
        partial = torch.empty(k.attn_decode_workspace_floats(1, n_heads, hd, 3), device=DEV)
        k.attn_decode(q.to(DEV), kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, i32(slots), i32([n]), out, partial, n_heads,
                      n_kv, hd, window, 3)
        assert (out.cpu().double() - 7.0).abs().max() < 0.1, "decode"

        # prefill: keys grow stronger towards the past, so that for query i the strongest visible key is the
        # oldest one, i - window + 1, and the one before it would be stronger still.  The strength T - j is
        # split over two elements (16 a + b) so that bfloat16 holds it exactly; scores of neighbours differ by 16.
        T = n
        s_q = 16.0 * math.sqrt(hd)
        qrow = torch.zeros(hd, dtype=torch.float64)
        qrow[3], qrow[4] = 16.0 * s_q, s_q
        qq = qrow.to(dtype).repeat(T, n_heads)
        kk = torch.zeros((T, n_kv * hd), dtype=dtype)
        v = torch.zeros((T, n_kv * hd), dtype=dtype)
        for j in range(T):
            krow = torch.zeros(hd, dtype=torch.float64)
            krow[3], krow[4] = (T - j) // 16, (T - j) % 16
            kk[j] = krow.to(dtype).repeat(n_kv)
            v[j] = float(j % 50)
        ks, vs, tile0 = stage(kk, v, [T], n_kv, hd, dtype)
        out = torch.empty((T, n_heads * hd), dtype=dtype, device=DEV)
        k.attn_prefill(qq.to(DEV), ks.to(DEV), vs.to(DEV), out, i32([0, T]), i32(tile0), i32([0] * T),
                       i32(list(range(T))), n_heads, n_kv, hd, window)
        got = out.cpu().double()[:, 0]
        want = torch.tensor([float(max(0, i - window + 1) % 50) for i in range(T)], dtype=torch.float64)
        assert (got - want).abs().max() < 0.1, "prefill, first bad position %d" % int(((got - want).abs() >= 0.1).nonzero()[0])
    finally:
        k.FORCE_SIMPLE = False



def test_attn_vector_of_the_reference():
    """src/test.cpp:67-126 through both attention kernels (head size padded from 3 to 16 with zeros)."""
    k = K()
    hd = 16
    q = torch.zeros((4, 2 * hd))
    q[3, 1], q[3, hd + 2] = 1e4, 1e4
    kv = torch.zeros((4, hd))
    kv[0, 0], kv[1, 1], kv[2, 2], kv[3, 0] = 1, 1, 1, -1
    out = torch.empty((4, 2 * hd), device=DEV)
    ks, vs, tile0 = stage(kv, kv, [4], 1, hd, torch.float32, poison=False)
    # the reference divides by sqrt(3); here sqrt(16): the scores stay far apart, the result is the same
    k.attn_prefill(q.to(DEV), ks.to(DEV), vs.to(DEV), out, i32([0, 4]), i32(tile0), i32([0] * 4), i32([0, 1, 2, 3]), 2,
                   1, hd, 0)
    got = out.cpu()[3].reshape(2, hd)
    assert torch.allclose(got[0, :3], torch.tensor([0., 1, 0]), atol=1e-4)
    assert torch.allclose(got[1, :3], torch.tensor([0., 0, 1]), atol=1e-4)


# ------------------------------------------------------------------ attention sinks

def window_lse_float64(q, k, window):
    """Logarithm of the sum of exp(score) over the keys a window shows, [T, n_heads]."""
    T, n_heads, hd = q.shape
    group = n_heads // k.shape[1]
    out = torch.zeros((T, n_heads), dtype=torch.float64)
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        for h in range(n_heads):
            out[i, h] = torch.logsumexp((k[lo:i + 1, h // group].double() @ q[i, h].double()) / math.sqrt(hd), 0)
    return out


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,rd,window,sinks,lens", [
    (4, 2, 16, 16, 5, 2, [30, 3, 1, 8]), (6, 3, 48, 24, 37, 3, [150, 41]), (8, 2, 128, 128, 94, 2, [300, 96, 97]),
    (4, 1, 64, 32, 70, 4, [200, 64]), (2, 2, 32, 0, 9, 1, [40])])
def test_attn_prefill_with_sinks(n_heads, n_kv, hd, rd, window, sinks, lens, dtype, simple):
    """Sinks stored from the staging area, the attention kernel's log-sum-exp, and the sinks behind the
    window mixed in with their keys turned, against the plain implementation's closed form."""
    k = K()
    T, B = sum(lens), len(lens)
    q = rnd((T, n_heads * hd), 33, dtype)
    kk = rnd((T, n_kv * hd), 34, dtype)
    v = rnd((T, n_kv * hd), 35, dtype)
    cu = np.concatenate([[0], np.cumsum(lens)])
    seq = np.repeat(np.arange(B), lens)
    pos = np.concatenate([np.arange(n) for n in lens])
    ks, vs, tile0 = stage(kk, v, lens, n_kv, hd, dtype)
    n_slots = B + 3
    slots = [int(x) for x in np.random.default_rng(5).permutation(n_slots)[:B]]
    sink_k = torch.full((n_slots, n_kv, sinks, hd), 7.0, dtype=dtype, device=DEV)
    sink_v = torch.full((n_slots, n_kv, sinks, hd), 7.0, dtype=dtype, device=DEV)
    table = make_table(max(lens) + 1, hd, rd, 80.0).to(DEV) if rd else None
    out = torch.empty((T, n_heads * hd), dtype=dtype, device=DEV)
    lse = torch.empty((T, n_heads), dtype=torch.float32, device=DEV)
    qd, ksd, vsd = q.to(DEV), ks.to(DEV), vs.to(DEV)
    k.FORCE_SIMPLE = simple
    try:
        k.sink_store(ksd, vsd, i32(tile0), i32(slots), i32(lens), sink_k, sink_v)
        # the unrounded result beside the rounded one: the row with the sinks mixed in is then rounded once
        o32 = torch.full((T, n_heads * hd), float("nan"), device=DEV) if dtype == torch.bfloat16 else None
        k.attn_prefill(qd, ksd, vsd, out, i32(cu), i32(tile0), i32(seq), i32(pos), n_heads, n_kv, hd, window, lse=lse,
                       out_f32=o32)
        plain_window = out.clone()
        if o32 is not None:
            assert torch.equal(o32.to(dtype), out)
        k.attn_sink_mix(qd, out, lse, sink_k, sink_v, i32(seq), i32(pos), i32(slots), table, n_heads, rd, window,
                        src_f32=o32)
    finally:
        k.FORCE_SIMPLE = False
    inv = R.rope_inv_freq(hd, rd, 80.0)
    o = 0
    for b, n in enumerate(lens):
        qb, kb, vb = (t[o:o + n].reshape(n, -1, hd) for t in (q, kk, v))
        have = min(n, sinks)
        assert torch.equal(sink_k[slots[b], :, :have].cpu(), kb[:have].transpose(0, 1)), "stored sink keys"
        assert torch.equal(sink_v[slots[b], :, :have].cpu(), vb[:have].transpose(0, 1)), "stored sink values"
        assert (sink_k[slots[b], :, have:] == 7.0).all(), "sinks that the sequence does not have yet stay untouched"
        close(lse[o:o + n], window_lse_float64(qb, kb, window), torch.float32, "log-sum-exp of sequence %d" % b)
        want = R.attention(qb, kb, vb, window, sinks, inv).reshape(n, -1)
        close(out[o:o + n], want, dtype, "prefill attention with sinks, sequence %d" % b)
        if n > window + 1:         # the sinks matter: without them the result is another
            assert (plain_window[o:o + n].double().cpu() - want).abs().max() > 1e-2
        o += n
    unused = [s for s in range(n_slots) if s not in slots]
    assert (sink_k[unused] == 7.0).all() and (sink_v[unused] == 7.0).all()


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,rd,window,sinks,lens,splits", [
    (4, 2, 16, 16, 5, 2, [30, 7, 6, 1, 2], 1), (6, 3, 48, 24, 37, 3, [150, 41, 40, 39, 3], 2),
    (8, 2, 128, 128, 94, 2, [300, 96, 97, 95], 1), (32, 8, 128, 128, 94, 2, [700, 200], 3),
    (4, 1, 64, 32, 70, 4, [200, 73, 74, 2], 2), (2, 2, 32, 0, 9, 1, [40, 1], 70)])
def test_attn_decode_with_sinks(n_heads, n_kv, hd, rd, window, sinks, lens, splits, dtype, simple):
    """A decode step's sinks: the sequences still at their first positions store the key they just wrote;
    the others have theirs from before; the merge of the splits takes in the sinks that a query's window
    no longer covers."""
    k = K()
    B = len(lens)
    kp, vp, bt, slots, ring, keys, vals = paged_case(lens, n_kv, hd, window, dtype, 40)
    n_slots = bt.shape[0]
    q = rnd((B, n_heads * hd), 36, dtype)
    sink_k = torch.full((n_slots, n_kv, sinks, hd), float("nan"), dtype=dtype)
    sink_v = torch.full((n_slots, n_kv, sinks, hd), float("nan"), dtype=dtype)
    for b, n in enumerate(lens):          # what earlier steps stored; the newest position is this step's to store
        have = min(sinks, n - 1)
        sink_k[slots[b], :, :have] = keys[b][:have].transpose(0, 1)
        sink_v[slots[b], :, :have] = vals[b][:have].transpose(0, 1)
    sink_k, sink_v = sink_k.to(DEV), sink_v.to(DEV)
    table = make_table(max(lens) + 1, hd, rd, 80.0).to(DEV) if rd else None
    qd = torch.cat([q, torch.zeros((1, n_heads * hd), dtype=dtype)]).to(DEV)
    out = torch.full((B + 1, n_heads * hd), 5.0, dtype=dtype, device=DEV)
    partial = torch.empty(k.attn_decode_workspace_floats(B + 1, n_heads, hd, splits), device=DEV)
    seq_slot, seq_len = i32(slots + [-1]), i32(lens + [0])
    k.FORCE_SIMPLE = simple
    try:
        k.attn_decode(qd, kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, seq_slot, seq_len, out, partial, n_heads, n_kv, hd,
                      window, splits, sinks=(sink_k, sink_v, table, rd, True))
    finally:
        k.FORCE_SIMPLE = False
    inv = R.rope_inv_freq(hd, rd, 80.0)
    for b, n in enumerate(lens):
        have = min(sinks, n)
        assert torch.equal(sink_k[slots[b], :, :have].cpu(), keys[b][:have].transpose(0, 1)), "sink keys of row %d" % b
        assert torch.equal(sink_v[slots[b], :, :have].cpu(), vals[b][:have].transpose(0, 1)), "sink values of row %d" % b
        qf = torch.zeros((n, n_heads, hd), dtype=torch.float64)
        qf[-1] = q[b].double().reshape(n_heads, hd)
        want = R.attention(qf, keys[b], vals[b], window, sinks, inv)[-1].reshape(-1)
        close(out[b], want, dtype, "decode attention with sinks, row %d (%d keys)" % (b, n))
    assert (out[B] == 0).all()


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_decode_leaves_the_log_sum_exp(dtype, simple):
    k = K()
    n_heads, n_kv, hd, window = 8, 2, 128, 94
    for lens, splits in (([300, 5, 96], 1), ([300, 5, 96], 3)):
        B = len(lens)
        kp, vp, bt, slots, ring, keys, vals = paged_case(lens, n_kv, hd, window, dtype, 41)
        q = rnd((B, n_heads * hd), 37, dtype)
        out = torch.empty((B, n_heads * hd), dtype=dtype, device=DEV)
        lse = torch.empty((B, n_heads), dtype=torch.float32, device=DEV)
        partial = torch.empty(k.attn_decode_workspace_floats(B, n_heads, hd, splits), device=DEV)
        k.FORCE_SIMPLE = simple
        try:
            k.attn_decode(q.to(DEV), kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, i32(slots), i32(lens), out, partial,
                          n_heads, n_kv, hd, window, splits, lse=lse)
        finally:
            k.FORCE_SIMPLE = False
        for b, n in enumerate(lens):
            qf = torch.zeros((n, n_heads, hd), dtype=torch.float64)
            qf[-1] = q[b].double().reshape(n_heads, hd)
            close(lse[b], window_lse_float64(qf, keys[b], window)[-1], torch.float32, "log-sum-exp of row %d" % b)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_far_behind_the_window_decides(dtype):
    """One sink key is made so that, turned by the number of positions the sinks have been pushed on at
    this query (position - window - sinks + 1), it is the query itself, at a position many windows on:
    the result is that sink's value if and only if the key is turned by exactly that much."""
    k = K()
    hd, window, sinks, n = 64, 20, 2, 333
    table = make_table(n, hd, hd, 4.0)
    inv = R.rope_inv_freq(hd, hd, 4.0)
    base = torch.zeros(hd, dtype=torch.float64)
    base[0::2] = 6.0                                   # every pair along its first axis
    pos = n - 1
    turn = pos - window - sinks + 1
    qrot = R.rope_interleaved(base.reshape(1, 1, hd), torch.tensor([pos]), inv).reshape(1, hd)
    kj = R.rope_interleaved(base.reshape(1, 1, hd), torch.tensor([pos - turn]), inv).reshape(hd)
    sink_k = torch.zeros((1, 1, sinks, hd), dtype=dtype)
    sink_v = torch.zeros((1, 1, sinks, hd), dtype=dtype)
    sink_k[0, 0, 1] = kj.to(dtype)
    sink_v[0, 0, 0, 0] = 1.0
    sink_v[0, 0, 1, 1] = 1.0
    out = torch.zeros((1, hd), dtype=dtype, device=DEV)
    out[0, 2] = 1.0                                    # what the window gave
    lse = torch.full((1, 1), 100.0, dtype=torch.float32, device=DEV)
    k.attn_sink_mix(qrot.to(dtype).to(DEV), out, lse, sink_k.to(DEV), sink_v.to(DEV), i32([0]), i32([pos]), i32([0]),
                    table.to(DEV), 1, hd, window)
    got = out.cpu().double()[0]
    # turned right, the sink scores |base|^2 / sqrt(hd) = 144 against 100 for the window; one position off
    # it would score 120 (the plain rotation says so) and still win, hence the second run below
    assert got[1] > 0.999 and got[0] < 1e-3 and got[2] < 1e-3, got[:3]
    right = R.rope_interleaved(kj.reshape(1, 1, hd), torch.tensor([turn]), inv).reshape(hd)
    assert abs(float(right @ qrot[0]) / math.sqrt(hd) - 144.0) < 1e-6
    for wrong in (turn - 1, turn + 1, 0):
        off = R.rope_interleaved(kj.reshape(1, 1, hd), torch.tensor([wrong]), inv).reshape(hd)
        assert float(off @ qrot[0]) / math.sqrt(hd) < 121.0
    # with the window at 132 a sink turned one position off (120) would lose; the right one (144) wins
    out2 = torch.zeros((1, hd), dtype=dtype, device=DEV)
    out2[0, 2] = 1.0
    lse.fill_(132.0)
    k.attn_sink_mix(qrot.to(dtype).to(DEV), out2, lse, sink_k.to(DEV), sink_v.to(DEV), i32([0]), i32([pos]), i32([0]),
                    table.to(DEV), 1, hd, window)
    got2 = out2.cpu().double()[0]
    assert got2[1] > 0.999 and got2[2] < 1e-3, got2[:3]


# ------------------------------------------------------------------ sampling

def test_argmax_and_sample():
    k = K()
    V = 1000
    g = torch.Generator().manual_seed(40)
    logits = torch.randn((6, V), generator=g) * 3
    logits[0, 17] = logits[0, 900] = 50.0                # a tie: the lowest index wins
    logits[1, V - 1] = 60.0
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    k.argmax(logits.to(DEV), out)
    assert out.cpu().tolist() == [R.sample_argmax(l) for l in logits]
    assert out[0] == 17 and out[1] == V - 1
    for temp in (1.0, 0.8, 2.5):
        u = torch.tensor([0.0, 0.999999, 0.5, 0.25, 0.9, 0.1])
        k.sample(logits.to(DEV), u.to(DEV), temp, out)
        got = out.cpu().tolist()
        for r in range(6):
            p = torch.softmax(logits[r].double() / temp, 0)
            c = torch.cumsum(p, 0)
            want = R.sample_temperature(logits[r], temp, float(u[r]))
            # equal up to an edge of the running sum: the picked token's interval contains u within rounding
            lo = float(c[got[r]] - p[got[r]])
            assert got[r] == want or (lo - 1e-5 <= float(u[r]) <= float(c[got[r]]) + 1e-5), (temp, r, got[r], want)
    # the distribution on a toy of 4 logits: frequencies match softmax
    l4 = torch.tensor([[0.0, 1.0, 2.0, -1.0]]).repeat(4000, 1)
    u = torch.rand(4000, generator=g)
    out = torch.empty(4000, dtype=torch.int32, device=DEV)
    k.sample(l4.to(DEV), u.to(DEV), 1.0, out)
    freq = torch.bincount(out.cpu().long(), minlength=4).double() / 4000
    assert (freq - torch.softmax(l4[0].double(), 0)).abs().max() < 0.03
    prob = torch.empty(6, device=DEV)
    k.token_prob(logits.to(DEV), i32([0, 1, 2, 3, 4, 999]), prob)
    want = [R.sample_prob(logits[r], i) for r, i in enumerate([0, 1, 2, 3, 4, 999])]
    assert torch.allclose(prob.cpu().double(), torch.tensor(want, dtype=torch.float64), rtol=1e-4, atol=1e-9)


@pytest.mark.parametrize("V", [4, 7, 255, 1029, 32003, 128256])
def test_sampling_at_vocabularies_of_any_size(V):
    """Rows that do not start on a 16-byte boundary (odd V), fewer entries than a wave's tile, and
    vocabularies that give every wave several tiles: the first maximum, the walk of the running sum
    and the probability of a token against the plain functions."""
    k = K()
    g = torch.Generator().manual_seed(41 + V)
    n = 5
    logits = torch.randn((n, V), generator=g) * 3
    logits[0, 0] = logits[0, V - 1] = 40.0                   # ties at both ends: the first wins
    logits[1, V - 1] = 41.0                                  # the last entry (the scalar tail)
    logits[2, min(V - 1, 2)] = logits[2, V // 2] = 42.0
    dl = logits.to(DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    k.argmax(dl, out)
    assert out.cpu().tolist() == [R.sample_argmax(l) for l in logits]
    flat = torch.randn((n, V), generator=g)                  # flat rows: the walk ends deep inside the row
    for rows, temp in ((logits, 1.0), (flat, 0.7), (flat, 3.0)):
        d = rows.to(DEV)
        for us in ([0.0, 0.999999, 0.5, 0.25, 0.9], [0.1, 0.33, 0.66, 0.75, 1.0]):
            u = torch.tensor(us)
            k.sample(d, u.to(DEV), temp, out)
            got = out.cpu().tolist()
            for r in range(n):
                assert 0 <= got[r] < V
                p = torch.softmax(rows[r].double() / temp, 0)
                c = torch.cumsum(p, 0)
                want = R.sample_temperature(rows[r], temp, float(u[r]))
                lo = float(c[got[r]] - p[got[r]])
                assert got[r] == want or (lo - 1e-5 <= float(u[r]) <= float(c[got[r]]) + 1e-5), (V, temp, r, got[r], want)
    idx = [0, V - 1, V // 2, min(V - 1, 3), V // 3]
    prob = torch.empty(n, device=DEV)
    k.token_prob(dl, i32(idx), prob)
    want = [R.sample_prob(logits[r], i) for r, i in enumerate(idx)]
    assert torch.allclose(prob.cpu().double(), torch.tensor(want, dtype=torch.float64), rtol=1e-4, atol=1e-9)


# ------------------------------------------------------------------ fused decode GEMMs

@pytest.mark.parametrize("M,N,Kd", [(1, 64, 256), (8, 4096 + 32, 136), (7, 100, 96), (3, 17000, 64), (2, 4096, 4096), (8, 48, 4096)])
def test_gemm_norm(M, N, Kd):
    """rmsnorm folded into the product: against the plain rmsnorm followed by a float64 product."""
    k = K()
    x = rnd((M, Kd), 50, scale=3.0)
    nw = 1 + 0.1 * rnd((Kd,), 51)
    w = rnd((N, Kd), 52, torch.bfloat16, scale=1 / math.sqrt(Kd))
    want = R.rmsnorm(x, nw, 1e-5) @ w.double().T
    out = torch.empty((M, N), device=DEV)
    k.gemm_norm(x.to(DEV), nw.to(DEV), 1e-5, w.to(DEV), out, k.EPI_STORE_F32)
    close(out, want, torch.bfloat16, "gemm_norm")          # the activations are rounded to bfloat16 on the way


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,H,D", [(8, 14336, 4096), (1, 14336, 192), (16, 14336, 1024), (11, 13003, 64), (4, 12810, 320),
                                   (9, 20000, 128), (3, 28672, 256)])
def test_gemm_gated_wide_at_up_to_16_rows(M, H, D, act):
    """Up to 16 rows and a gated matrix wide enough for the workgroups of 128 weight rows: hidden widths that are no
    multiples of 8 or of 64, one and many stages of K, with and without the row scale of the norm chain; every hidden
    column is written, nothing beyond them."""
    from yalm_amd.parts.swiglu import interleave_gate_up
    k = K()
    act_fn, epi_code = gate(act)
    x = rnd((M, D), 53, torch.bfloat16, scale=2.0)
    wg = rnd((H, D), 55, torch.bfloat16, scale=1 / math.sqrt(D))
    wu = rnd((H, D), 56, torch.bfloat16, scale=1 / math.sqrt(D))
    w = interleave_gate_up(wg, wu).to(DEV)
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    out = torch.full((M + 1, H), 7.0, dtype=torch.bfloat16, device=DEV)
    k.gemm(x.to(DEV), w, out[:M], epi_code, hidden=H)
    close(out[:M], act_fn(g) * u, torch.bfloat16, "gated product")
    assert (out[M] == 7.0).all()
    # the same behind the norm chain: the sums are scaled row by row before the activation
    ss = (x.double() ** 2).sum(dim=1, keepdim=True).float() * torch.tensor([[0.25, 0.5, 0.25]])
    eps = 1e-5
    scale = 1.0 / torch.sqrt((x.double() ** 2).sum(dim=1, keepdim=True) / D + eps)
    out2 = torch.full((M + 1, H), 7.0, dtype=torch.bfloat16, device=DEV)
    k.gemm_chain(x.to(DEV), w, out2[:M], epi_code, hidden=H, scale_from=(ss.to(DEV).contiguous(), eps))
    close(out2[:M], act_fn(g * scale) * (u * scale), torch.bfloat16, "gated product with a row scale", factor=2.0)
    assert (out2[M] == 7.0).all()


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,H,D", [(1, 176, 64), (8, 1000, 264), (5, 14336, 128)])
def test_gemm_norm_gated(M, H, D, act):
    from yalm_amd.parts.swiglu import interleave_gate_up
    k = K()
    x = rnd((M, D), 53, scale=2.0)
    nw = 1 + 0.1 * rnd((D,), 54)
    wg = rnd((H, D), 55, torch.bfloat16, scale=1 / math.sqrt(D))
    wu = rnd((H, D), 56, torch.bfloat16, scale=1 / math.sqrt(D))
    h = R.rmsnorm(x, nw, 1e-6)
    act_fn, epi_code = gate(act)
    want = act_fn(h @ wg.double().T) * (h @ wu.double().T)
    out = torch.empty((M, H), dtype=torch.bfloat16, device=DEV)
    k.gemm_norm(x.to(DEV), nw.to(DEV), 1e-6, interleave_gate_up(wg, wu).to(DEV), out, epi_code, hidden=H)
    close(out, want, torch.bfloat16, "gemm_norm gated", factor=1.5)


@pytest.mark.parametrize("n_heads,n_kv,hd,rd,D", [(4, 2, 16, 16, 64), (3, 1, 48, 48, 80), (6, 3, 32, 16, 96),
                                                   (32, 8, 128, 128, 256)])
def test_gemm_norm_qkv_rope(n_heads, n_kv, hd, rd, D):
    """norm + q/k/v + rotation + cache write in one kernel against the plain parts."""
    k = K()
    PAGE = k.PAGE
    M = 5
    pos = [0, 63, 64, 130, 7]
    slots = [3, 0, -1, 2, 1]                       # row 2 is a padding row
    Q, KV = n_heads * hd, n_kv * hd
    x = rnd((M, D), 57, scale=2.0)
    nw = 1 + 0.1 * rnd((D,), 58)
    w = rnd((Q + 2 * KV, D), 59, torch.bfloat16, scale=1 / math.sqrt(D))
    table = make_table(200, hd, rd, 10000.0)
    ring, n_pages = 4, 12
    bt = torch.arange(4 * ring, dtype=torch.int32).reshape(4, ring) % n_pages
    kp = torch.zeros((n_pages, n_kv, PAGE, hd), dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros((n_pages, n_kv, hd, PAGE), dtype=torch.bfloat16, device=DEV)
    q_out = torch.zeros((M, Q), dtype=torch.bfloat16, device=DEV)
    k.gemm_norm_qkv_rope(x.to(DEV), nw.to(DEV), 1e-5, w.to(DEV), q_out, kp, vp, bt.to(DEV), ring, i32(pos), i32(slots),
                         table.to(DEV), n_heads, n_kv, hd, rd)
    qkv = R.rmsnorm(x, nw, 1e-5) @ w.double().T
    f = R.rope_inv_freq(hd, rd, 10000.0)
    p = torch.tensor(pos)
    q_want = R.rope_interleaved(qkv[:, :Q].reshape(M, n_heads, hd), p, f).reshape(M, Q)
    k_want = R.rope_interleaved(qkv[:, Q:Q + KV].reshape(M, n_kv, hd), p, f)
    v_want = qkv[:, Q + KV:].reshape(M, n_kv, hd)
    close(q_out, q_want, torch.bfloat16, "q", factor=1.5)
    kp, vp = pages_as_rows(kp.cpu(), vp.cpu())
    touched = torch.zeros((n_pages, PAGE), dtype=torch.bool)
    for m in range(M):
        if slots[m] < 0:
            continue
        page, r = int(bt[slots[m], (pos[m] // PAGE) % ring]), pos[m] % PAGE
        close(kp[page, :, r, :], k_want[m], torch.bfloat16, "k row %d" % m, factor=1.5)
        close(vp[page, :, :, r], v_want[m], torch.bfloat16, "v row %d" % m, factor=1.5)
        touched[page, r] = True
    assert (kp.float().abs().sum(dim=(1, 3)) > 0).equal(touched)
    assert (vp.float().abs().sum(dim=(1, 2)) > 0).equal(touched)


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("n_heads,n_kv,hd,rd,D", [(4, 2, 16, 16, 64), (3, 1, 48, 48, 80), (6, 3, 32, 16, 192),
                                                   (32, 8, 128, 128, 128), (24, 8, 128, 128, 64), (10, 5, 64, 64, 256)])
def test_gemm_chain_qkv_rope(n_heads, n_kv, hd, rd, D, M):
    """The q/k/v projection of a decode step from activations a producer emitted (already multiplied by the
    norm's weights, with partial sums of squares), with rotation and cache write in its epilogue; among the
    shapes the 6144 and 5120 weight rows of the big models' projections."""
    k = K()
    PAGE = k.PAGE
    rng = np.random.default_rng(M)
    pos = [int(p) for p in rng.integers(0, 190, size=M)]
    slots = [int(s) for s in rng.permutation(M + 2)[:M]]
    if M > 2:
        slots[2] = -1                                  # a padding row
    Q, KV = n_heads * hd, n_kv * hd
    x = rnd((M, D), 57, scale=2.0)
    nw = 1 + 0.1 * rnd((D,), 58)
    w = rnd((Q + 2 * KV, D), 59, torch.bfloat16, scale=1 / math.sqrt(D))
    xn = (x * nw).to(torch.bfloat16)
    parts = 3
    ss = torch.zeros((M, parts))
    for p_, cols in enumerate(np.array_split(np.arange(D), parts)):
        ss[:, p_] = (x[:, cols].double() ** 2).sum(dim=1).float()
    table = make_table(200, hd, rd, 10000.0)
    ring, n_pages = 3, 64
    bt = torch.tensor(rng.permutation(n_pages)[: (M + 2) * ring].reshape(M + 2, ring), dtype=torch.int32)
    kp = torch.zeros((n_pages, n_kv, PAGE, hd), dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros((n_pages, n_kv, hd, PAGE), dtype=torch.bfloat16, device=DEV)
    q_out = torch.zeros((M, Q), dtype=torch.bfloat16, device=DEV)
    k.gemm_chain_qkv_rope(xn.to(DEV), (ss.to(DEV), 1e-5), w.to(DEV), q_out, kp, vp, bt.to(DEV), ring, i32(pos),
                          i32(slots), table.to(DEV), n_heads, n_kv, hd, rd)
    scale = 1.0 / torch.sqrt((x.double() ** 2).mean(dim=1, keepdim=True) + 1e-5)
    qkv = (xn.double() @ w.double().T) * scale
    f = R.rope_inv_freq(hd, rd, 10000.0)
    p = torch.tensor(pos)
    q_want = R.rope_interleaved(qkv[:, :Q].reshape(M, n_heads, hd), p, f).reshape(M, Q)
    k_want = R.rope_interleaved(qkv[:, Q:Q + KV].reshape(M, n_kv, hd), p, f)
    v_want = qkv[:, Q + KV:].reshape(M, n_kv, hd)
    close(q_out, q_want, torch.bfloat16, "q", factor=1.5)
    kp, vp = pages_as_rows(kp.cpu(), vp.cpu())
    touched = torch.zeros((n_pages, PAGE), dtype=torch.bool)
    for m in range(M):
        if slots[m] < 0:
            continue
        page, r = int(bt[slots[m], (pos[m] // PAGE) % ring]), pos[m] % PAGE
        close(kp[page, :, r, :], k_want[m], torch.bfloat16, "k row %d" % m, factor=1.5)
        close(vp[page, :, :, r], v_want[m], torch.bfloat16, "v row %d" % m, factor=1.5)
        touched[page, r] = True
    assert (kp.float().abs().sum(dim=(1, 3)) > 0).equal(touched)
    assert (vp.float().abs().sum(dim=(1, 2)) > 0).equal(touched)


@pytest.mark.parametrize("M,N,Kd", [(1, 64, 256), (8, 4096, 1000), (33, 80, 96), (64, 4096, 264), (5, 16400, 64),
                                    (11, 192, 192), (16, 4096, 128), (9, 1024, 64), (8, 3072, 128), (3, 3000, 64),
                                    (20, 3072, 64)])
def test_gemm_chain_producer_and_consumer(M, N, Kd):
    """A residual-add GEMM that emits the next norm's activations and partial sums of squares,
    and a consumer that scales by them: together they equal rmsnorm(x_new) @ W2^T."""
    k = K()
    a = rnd((M, Kd), 60, torch.bfloat16)
    w = rnd((N, Kd), 61, torch.bfloat16, scale=1 / math.sqrt(Kd))
    res = rnd((M, N), 62, scale=2.0)
    nw = 1 + 0.1 * rnd((N,), 63)
    x = res.to(DEV).clone()
    if N >= 16384:                                      # too wide to emit: refused
        with pytest.raises(Exception):
            k.gemm_chain(a.to(DEV), w.to(DEV), x, k.EPI_ADD_F32,
                         emit=(nw.to(DEV), torch.empty((M, N), dtype=torch.bfloat16, device=DEV),
                               torch.empty((M, k.gemm_chain_parts(N)), device=DEV)))
        return
    xn = torch.zeros((M, N), dtype=torch.bfloat16, device=DEV)
    ss = torch.zeros((M, k.gemm_chain_parts(N)), device=DEV)
    k.gemm_chain(a.to(DEV), w.to(DEV), x, k.EPI_ADD_F32, emit=(nw.to(DEV), xn, ss))
    x_want = res.double() + a.double() @ w.double().T
    close(x, x_want, torch.float32, "residual")
    close(xn, x_want * nw.double(), torch.bfloat16, "emitted activations")
    assert torch.allclose(ss.sum(dim=1).cpu().double(), (x_want ** 2).sum(dim=1), rtol=1e-5)
    # consumers: float32 store and gated
    H = 48
    from yalm_amd.parts.swiglu import interleave_gate_up
    w2 = rnd((70, N), 64, torch.bfloat16, scale=1 / math.sqrt(N))
    out = torch.empty((M, 70), device=DEV)
    k.gemm_chain(xn, w2.to(DEV), out, k.EPI_STORE_F32, scale_from=(ss, 1e-5))
    want = R.rmsnorm(x_want, nw, 1e-5) @ w2.double().T
    close(out, want, torch.bfloat16, "chained consumer", factor=1.5)
    wg = rnd((H, N), 65, torch.bfloat16, scale=1 / math.sqrt(N))
    wu = rnd((H, N), 66, torch.bfloat16, scale=1 / math.sqrt(N))
    outg = torch.empty((M, H), dtype=torch.bfloat16, device=DEV)
    h = R.rmsnorm(x_want, nw, 1e-5)
    for act in ACTS:
        act_fn, epi_code = gate(act)
        k.gemm_chain(xn, interleave_gate_up(wg, wu).to(DEV), outg, epi_code, hidden=H, scale_from=(ss, 1e-5))
        close(outg, act_fn(h @ wg.double().T) * (h @ wu.double().T), torch.bfloat16, "chained gated " + act, factor=2.0)


@pytest.mark.parametrize("with_workspace", [True, False])
@pytest.mark.parametrize("M,N,Kd", [(17, 4096, 4096), (64, 100, 264), (48, 6144, 1000), (33, 4096, 14336)])
def test_gemm_batches_of_17_to_64_rows(M, N, Kd, with_workspace):
    """The kernel for 17..64 rows, with K split across workgroups (given scratch) and without."""
    k = K()
    a = rnd((M, Kd), 70, torch.bfloat16)
    w = rnd((N, Kd), 71, torch.bfloat16, scale=1 / math.sqrt(Kd))
    want = a.double() @ w.double().T
    ws = torch.empty(k.gemm_workspace_floats(M, N, Kd), device=DEV) if with_workspace else None
    out = torch.empty((M, N), device=DEV)
    k.gemm(a.to(DEV), w.to(DEV), out, k.EPI_STORE_F32, workspace=ws)
    close(out, want, torch.float32, "f32 out")
    out2 = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    k.gemm(a.to(DEV), w.to(DEV), out2, k.EPI_STORE, workspace=ws)
    close(out2, want, torch.bfloat16, "bf16 out")
    res = rnd((M, N), 72)
    acc = res.to(DEV).clone()
    k.gemm(a.to(DEV), w.to(DEV), acc, k.EPI_ADD_F32, workspace=ws)
    close(acc, want + res.double(), torch.float32, "add")


@pytest.mark.parametrize("with_workspace", [True, False])
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,H,D", [(64, 14336, 256), (20, 1000, 264), (40, 176, 4096)])
def test_gemm_gated_batches_of_17_to_64_rows(M, H, D, with_workspace, act):
    from yalm_amd.parts.swiglu import interleave_gate_up
    k = K()
    x = rnd((M, D), 73, torch.bfloat16)
    wg = rnd((H, D), 74, torch.bfloat16, scale=1 / math.sqrt(D))
    wu = rnd((H, D), 75, torch.bfloat16, scale=1 / math.sqrt(D))
    act_fn, epi_code = gate(act)
    want = act_fn(x.double() @ wg.double().T) * (x.double() @ wu.double().T)
    w = interleave_gate_up(wg, wu).to(DEV)
    ws = torch.empty(k.gemm_workspace_floats(M, w.shape[0], D), device=DEV) if with_workspace else None
    out = torch.empty((M, H), dtype=torch.bfloat16, device=DEV)
    k.gemm(x.to(DEV), w, out, epi_code, hidden=H, workspace=ws)
    close(out, want, torch.bfloat16, "gated")


@pytest.mark.parametrize("M,N,Kd", [(65, 4096, 4096), (128, 1000, 14336), (130, 333, 1024), (256, 4096, 2112),
                                    (70, 100, 4160)])
def test_gemm_of_more_than_64_rows_splits_k(M, N, Kd):
    """A batch of more than 64 rows whose output has few tiles: K in slices, given the scratch (whole, and
    too small for all the slices the kernel would like), and the same products without it."""
    k = K()
    a = rnd((M, Kd), 76, torch.bfloat16)
    w = rnd((N, Kd), 77, torch.bfloat16, scale=1 / math.sqrt(Kd))
    want = a.double() @ w.double().T
    res = rnd((M, N), 78)
    full = k.gemm_workspace_floats(M, N, Kd)
    assert full >= 2 * M * N and full % (M * N) == 0
    for floats in (full, 2 * M * N, 0):
        ws = torch.full((floats,), float("nan"), device=DEV) if floats else None
        out = torch.empty((M, N), device=DEV)
        k.gemm(a.to(DEV), w.to(DEV), out, k.EPI_STORE_F32, workspace=ws)
        close(out, want, torch.float32, "f32 out, %d floats" % floats)
        out2 = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        k.gemm(a.to(DEV), w.to(DEV), out2, k.EPI_STORE, workspace=ws)
        close(out2, want, torch.bfloat16, "bf16 out, %d floats" % floats)
        acc = res.to(DEV).clone()
        k.gemm(a.to(DEV), w.to(DEV), acc, k.EPI_ADD_F32, workspace=ws)
        close(acc, want + res.double(), torch.float32, "add, %d floats" % floats)
    assert k.gemm_workspace_floats(8192, 4096, 4096) == 0       # enough tiles: no slices


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,H,D", [(100, 1000, 4096), (128, 176, 2048), (65, 3000, 1024)])
def test_gemm_gated_of_more_than_64_rows_splits_k(M, H, D, act):
    from yalm_amd.parts.swiglu import interleave_gate_up
    k = K()
    x = rnd((M, D), 79, torch.bfloat16)
    wg = rnd((H, D), 84, torch.bfloat16, scale=1 / math.sqrt(D))
    wu = rnd((H, D), 85, torch.bfloat16, scale=1 / math.sqrt(D))
    act_fn, epi_code = gate(act)
    want = act_fn(x.double() @ wg.double().T) * (x.double() @ wu.double().T)
    w = interleave_gate_up(wg, wu).to(DEV)
    floats = k.gemm_workspace_floats(M, w.shape[0], D)
    assert floats >= 2 * M * w.shape[0]
    out = torch.empty((M, H), dtype=torch.bfloat16, device=DEV)
    k.gemm(x.to(DEV), w, out, epi_code, hidden=H, workspace=torch.full((floats,), float("nan"), device=DEV))
    close(out, want, torch.bfloat16, "gated")


@pytest.mark.parametrize("small_workspace", [False, True])
@pytest.mark.parametrize("M,N,Kd", [(17, 4096, 4096), (64, 100, 264), (40, 4096, 14336), (33, 96, 64),
                                    (65, 4096, 4096), (130, 333, 1024), (300, 20488, 128), (256, 96, 14336)])
def test_gemm_add_norm(M, N, Kd, small_workspace):
    """Residual add and the next RMSNorm in one, more than 16 rows: x += a W^T; h = rmsnorm(x) * w."""
    k = K()
    a = rnd((M, Kd), 80, torch.bfloat16)
    w = rnd((N, Kd), 81, torch.bfloat16, scale=1 / math.sqrt(Kd))
    x0 = rnd((M, N), 82, scale=2.0)
    nw = (1 + 0.1 * rnd((N,), 83)).float()
    eps = 1e-5
    x = x0.clone().to(DEV)
    h = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(M * N if small_workspace else k.fused_workspace_floats(M, N, Kd), device=DEV)
    k.gemm_add_norm(a.to(DEV), w.to(DEV), x, nw.to(DEV), eps, h, ws)
    want_x = x0.double() + a.double() @ w.double().T
    close(x, want_x, torch.float32, "residual", factor=4)
    close(h, R.rmsnorm(want_x, nw, eps), torch.bfloat16, "normed")
    with pytest.raises(ValueError):
        k.gemm_add_norm(a.to(DEV), w.to(DEV), x, nw.to(DEV), eps, h, torch.empty(M * N - 1, device=DEV))


@pytest.mark.parametrize("small_workspace", [False, True])
@pytest.mark.parametrize("M,N,Kd,N2", [(17, 4096, 4096, 6144), (64, 104, 264, 48), (40, 4096, 14336, 320),
                                       (33, 96, 64, 200), (65, 4096, 4096, 1000), (128, 1088, 1024, 96)])
def test_gemm_add_emit_and_its_consumers(M, N, Kd, N2, small_workspace):
    """The norm chain of 17..128 rows: x += a W^T with the next norm only prepared (activations times the norm's
    weights, partial sums of squares), and the consumers that scale their sums row by row: a plain product, a gated
    one, and K slices left for another kernel to add.  Together they must give what a finished norm in front of the
    same products gives."""
    k = K()
    a = rnd((M, Kd), 90, torch.bfloat16)
    w = rnd((N, Kd), 91, torch.bfloat16, scale=1 / math.sqrt(Kd))
    x0 = rnd((M, N), 92, scale=2.0)
    x0[M // 2] *= 37.0                                   # rows of very different sizes: every row has its own scale
    x0[0] *= 1e-3
    nw = (1 + 0.1 * rnd((N,), 93)).float()
    eps = 1e-5
    x = x0.clone().to(DEV)
    xn = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    parts = k.gemm_add_emit_parts(N)
    assert parts == (N + 1023) // 1024
    ss = torch.full((M, parts), float("nan"), device=DEV)
    ws = torch.empty(M * N if small_workspace else k.fused_workspace_floats(M, N, Kd), device=DEV)
    assert k.can_add_emit(M, Kd, torch.bfloat16) and not k.can_add_emit(16, Kd, torch.bfloat16)
    k.gemm_add_emit(a.to(DEV), w.to(DEV), x, nw.to(DEV), xn, ss, ws)
    want_x = x0.double() + a.double() @ w.double().T
    close(x, want_x, torch.float32, "residual", factor=4)
    close(xn, want_x * nw.double(), torch.bfloat16, "activations times the norm's weights")
    close(ss.sum(dim=1), (want_x ** 2).sum(dim=1), torch.float32, "sums of squares", factor=4)
    h = R.rmsnorm(want_x, nw, eps)                       # what the consumers' products must be products of
    # a plain consumer (the head's epilogue) and the K slices of one
    w2 = rnd((N2, N), 94, torch.bfloat16, scale=1 / math.sqrt(N))
    want = h @ w2.double().T
    out = torch.empty((M, N2), device=DEV)
    ws2 = torch.full((k.gemm_workspace_floats(M, N2, N),), float("nan"), device=DEV)
    k.gemm(xn, w2.to(DEV), out, k.EPI_STORE_F32, workspace=ws2, scale_from=(ss, eps))
    close(out, want, torch.bfloat16, "scaled product")
    if k.can_gemm_partial(M, N, torch.bfloat16):
        ws3 = torch.full((k.fused_workspace_floats(M, N2, N),), float("nan"), device=DEV)
        slices = k.gemm_partial(xn, w2.to(DEV), ws3, scale_from=(ss, eps))
        close(ws3[:slices * M * N2].view(slices, M, N2).sum(dim=0), want, torch.bfloat16, "scaled slices")
    # a gated consumer
    H = 72
    wg = rnd((H, N), 95, torch.bfloat16, scale=1 / math.sqrt(N))
    wu = rnd((H, N), 96, torch.bfloat16, scale=1 / math.sqrt(N))
    from yalm_amd.parts.swiglu import interleave_gate_up
    wgu = interleave_gate_up(wg, wu).to(DEV)
    mid = torch.empty((M, H), dtype=torch.bfloat16, device=DEV)
    ws4 = torch.full((k.gemm_workspace_floats(M, wgu.shape[0], N),), float("nan"), device=DEV)
    for act in ACTS:
        act_fn, epi_code = gate(act)
        k.gemm(xn, wgu, mid, epi_code, hidden=H, workspace=ws4, scale_from=(ss, eps))
        close(mid, act_fn(h @ wg.double().T) * (h @ wu.double().T), torch.bfloat16, "scaled gated product " + act, factor=2)
    with pytest.raises(Exception):                        # a row scale is for these batches only
        k.gemm(xn[:8].contiguous(), w2.to(DEV), out[:8].contiguous(), k.EPI_STORE_F32, scale_from=(ss[:8].contiguous(), eps))
