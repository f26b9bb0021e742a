"""Shared by the GPU tests: model folders with random weights (made in a
temporary folder), logits of the plain implementation, and the tolerances."""
import functools
import os

import numpy as np
import torch

from plain import reference_model as R

# float32: |engine - plain| <= 1e-4 * max(1, max|plain|) on every logit
F32_TOL = 1e-4
# bfloat16 (plain implementation on the bfloat16-rounded weights): activations are
# rounded to 8 bits of mantissa (relative step 2^-8) at about six places a layer,
# so errors of about a hundredth of the logits' scale are rounding; bounds fixed
# before the first run: largest error <= 6e-2 * max(1, max|plain|), and relative
# root-mean-square error <= 2e-2
BF16_MAX_TOL = 6e-2
BF16_RMS_TOL = 2e-2


def make_folder(tmp, name, cfg, seed=0, stored=torch.float32, device="cpu"):
    from yalm_amd.weights import write_random_model
    folder = os.path.join(str(tmp), "%s_%d_%s" % (name, seed, str(stored).split(".")[-1]))
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(folder, cfg, seed=seed, dtype=stored, device=device)
    return folder


@functools.lru_cache(maxsize=None)
def _folder_weights(folder, rounded):
    """The folder's tensors for the plain implementation, which widens each to float64 where it
    uses it (layer by layer: a model of billions of elements never stands in float64 as a whole).
    rounded: the values the engine's bfloat16 path stores: matrices rounded to bfloat16, while a vector
    that the folder keeps in 32-bit (the norm weights of the folders here) stays as it is."""
    if rounded:
        cfg, w = _folder_weights(folder, False)           # tensors stored in bfloat16 are shared, not read again
        return cfg, {k: v if v.dtype == torch.bfloat16 or (v.dim() <= 1 and v.dtype in (torch.float32, torch.float64))
                     else v.to(torch.bfloat16) for k, v in w.items()}
    return R.read_folder(folder)


def forget_plain_results():
    """Drops the cached weights and logits of the plain implementation (after a test with a big model)."""
    plain_logits.cache_clear()
    _folder_weights.cache_clear()


@functools.lru_cache(maxsize=None)
def plain_logits(folder, tokens, dtype="float32"):
    """float32 numpy [T, vocab] of the plain implementation; with dtype bfloat16
    the matrices are rounded to bfloat16 first, as the engine stores them (vectors
    that a folder keeps in 32-bit stay in 32-bit, there as here)."""
    cfg, w = _folder_weights(folder, dtype == "bfloat16")
    return R.forward(w, cfg, list(tokens)).to(torch.float32).numpy()


def check_logits(got, want, dtype, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all(), "%s: engine logits are not finite" % what
    err = np.abs(got - want)
    scale = max(1.0, np.abs(want).max())
    if dtype == "float32":
        bad = np.unravel_index(err.argmax(), err.shape)
        assert err.max() <= F32_TOL * scale, \
            "%s: max error %.3e at %s (row, token id) of %s, allowed %.3e" % (what, err.max(), bad, got.shape,
                                                                           F32_TOL * scale)
    else:
        bad = np.unravel_index(err.argmax(), err.shape)
        assert err.max() <= BF16_MAX_TOL * scale, \
            "%s: max error %.3e at %s of %s, allowed %.3e" % (what, err.max(), bad, got.shape, BF16_MAX_TOL * scale)
        rms = np.sqrt((err ** 2).mean()) / max(1e-12, np.sqrt((want ** 2).mean()))
        assert rms <= BF16_RMS_TOL, "%s: relative rms error %.3e, allowed %.3e" % (what, rms, BF16_RMS_TOL)


def first_bad_row(got, want, tol):
    err = np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)).max(axis=1)
    bad = np.nonzero(err > tol)[0]
    return int(bad[0]) if len(bad) else None


def random_requests(cfg, lengths, seed=0):
    g = np.random.default_rng(seed)
    return {"r%d" % i: g.integers(0, cfg["vocab_size"], size=n).tolist() for i, n in enumerate(lengths)}


def torch_dtype(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]
