"""Small Lomozen configurations of the test-suite and what the tests of that design share.

The configurations differ from one another in every size and constant: widths, head counts, key, value and
rotated sizes, ranks, windows (none, shorter than a page, no multiple of a page), rotated dimensions below
the rotated size, rescaled and plain frequencies, decays from 0 to 1, expert counts, choices per token,
layers with and without a feed-forward or a shared expert, and the order of the mixers.
"""
import numpy as np
import torch

from tests.plain import lomozen_plain as P


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window=None, scale=None, dims=None, base=10000.0, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot_dim:
        m["rot"] = {"base": base, "dims": dims if dims is not None else rot_dim}
        if scaling:
            m["rot"]["scaling"] = scaling
    return {"type": "latent_attention", "mixer": m}


def lightning(heads, dim, vdim, decay):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def moe(experts, top, ff, shared_ff=None):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff}
    return f


def layer(mixer, mlp=None):
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, eps=1e-5):
    return {"architecture": "Lomozen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}

# three layers, both mixers, windows of 20 (no multiple of the page), scores flat enough that every key in the window counts
SMALL_A = dict(name="A", seed=3, std=0.25, norm_std=0.1, page_size=8, config=config(48, 131, [
    layer(lightning(3, 8, 12, (0.5, 0.97, 0.999)), moe(6, 2, 40, 24)),
    layer(latent(3, 16, 8, 12, 24, 40, window=20, scale=0.4, scaling=YARN), moe(6, 2, 40, 24)),
    layer(latent(3, 16, 8, 12, 24, 40, window=20, scale=0.4, scaling=YARN), None),
]))
# odd sizes: a cached vector of 44 (no multiple of 16), rotated dimensions below the rotated size, plain
# frequencies, no window, one expert chosen of five without a shared one, decays 0 and 1
SMALL_B = dict(name="B", seed=4, std=0.2, norm_std=0.2, page_size=16, config=config(88, 300, [
    layer(latent(2, 24, 12, 20, 32, 56, window=None, dims=8, base=500.0), moe(5, 1, 72)),
    layer(lightning(2, 20, 36, (0.0, 1.0)), None),
    layer(latent(5, 8, 4, 6, 44, 16, window=7, scale=0.5, dims=4), moe(4, 4, 16, 50)),
], eps=1e-6))
# a window of one token, a window longer than every prompt, heads of 1, key size above a wave
SMALL_C = dict(name="C", seed=5, std=0.3, norm_std=0.05, page_size=32, config=config(64, 97, [
    layer(latent(1, 32, 16, 32, 48, 32, window=1, scaling=YARN), moe(3, 2, 96, 32)),
    layer(lightning(1, 72, 80, (0.9,)), moe(3, 2, 96, 32)),
    layer(latent(4, 32, 16, 16, 64, 64, window=1000, scale=0.7, base=1e6, scaling=dict(YARN, factor=1.5)), None),
], eps=1e-4))
ALL_SMALL = [SMALL_A, SMALL_B, SMALL_C]


def make_folder(small, tmp_path):
    from jax_vllm_amd import write_random_model

    return write_random_model(tmp_path, small["config"], seed=small["seed"], std=small["std"], norm_std=small["norm_std"])


def plain_of(folder, dtype=torch.float64):
    return P.read_config(folder), P.read_weights(folder, dtype)


def plain_logits(cfg, w, tokens):
    return P.forward(w, cfg, tokens).to(torch.float32).numpy()


def expected(cfg, w, tokens, dtype):
    """What ``check_rows`` compares with: the plain logits, and for bfloat16 also the plain logits with every
    matrix product rounded to bfloat16 (the model's own sensitivity to that rounding)."""
    want = plain_logits(cfg, w, tokens)
    if dtype in ("float32", "fp32"):
        return want
    with P.rounded_products(torch.bfloat16):
        return want, plain_logits(cfg, w, tokens)


def _row_rms(a, b):
    d = a - b
    d = d - d.mean(axis=-1, keepdims=True)
    return np.sqrt((d * d).mean(axis=-1))


def check_rows(dtype, got, want, what=""):
    """float32: every row agrees with the plain logits to the rounding of deep float sums.
    bfloat16: ``want`` is (plain logits, plain logits with products rounded to bfloat16).  The rows' errors
    (root mean square over the vocabulary) are compared with those that the rounding alone causes in the
    plain implementation.  Rounding turns close choices between experts, which changes a row altogether, in
    the engine and in the rounded plain run alike but not in the same rows; so the distributions are
    compared, not row by row: the median may be 3 times the rounded plain run's (plus a small floor), and
    the share of rows far off (6 times that median) twice its share plus 20 % (one row at least): the
    engine rounds more than the products (cached vectors, softmax weights), so it turns more choices.  A fault
    that touches few rows is the float32 tests' to find; they run the same code but for the matrix-core
    attention kernels."""
    if isinstance(want, tuple):
        want, rounded = want
    else:
        rounded = None
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shapes {got.shape} and {want.shape}"
    assert np.isfinite(got).all(), f"{what}: logits that are not finite"
    scale = max(float(np.abs(want).max()), 1.0)
    if dtype in ("float32", "fp32"):
        err = np.abs(got - want).max(axis=-1)
        assert err.max() <= 3e-5 * scale + 1e-5, f"{what}: max error {err.max()} at row {int(err.argmax())} (scale {scale})"
        return
    assert rounded is not None, "bfloat16 rows are compared with expected(..., dtype)"
    spread = float(np.sqrt(((want - want.mean(-1, keepdims=True)) ** 2).mean()))
    e, r = _row_rms(got, want), _row_rms(np.asarray(rounded, dtype=np.float64), want)
    floor = 0.01 * spread
    assert np.median(e) <= 3 * np.median(r) + floor, \
        f"{what}: median of the rows' errors {np.median(e):.4f}, rounding alone {np.median(r):.4f} (spread {spread:.3f})"
    far = 6 * np.median(r) + floor
    allowed = max(1, int(np.ceil((2 * (r > far).mean() + 0.2) * len(e))))
    assert (e > far).sum() <= allowed, \
        f"{what}: {int((e > far).sum())} of {len(e)} rows are off by more than {far:.4f}, {int((r > far).sum())} by rounding alone"
