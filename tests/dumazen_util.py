"""Small Dumazen configurations of the test-suite and what the tests of that design share.

The configurations differ from one another in every size and constant: widths, head counts and ratios, key, value
and state sizes, groups and norm groups, taps of the convolutions, windows (none, shorter than a page, no multiple of a
page), rotated dimensions below the head size, scaled and plain frequencies, decays from 0 to 1, the two scales of the
mixers side by side, the residual factor, layers with and without a feed-forward, and the order of the mixers.
"""
import numpy as np
import torch

from tests.lomozen_util import check_rows  # noqa: F401  (the same judgement of rows serves both designs)
from tests.plain import dumazen_plain as P


def rot(dims, base=10000.0, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = scaling
    return r


def retention(heads, dim, vdim, decay, rot_=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot_:
        m["rot"] = rot_
    return {"type": "retention", "mixer": m}


def mamba2(heads, vdim, state, groups=1, norm_groups=1, conv=4):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                        "norm_groups": norm_groups, "conv": conv}}


def window_attention(heads, kv_heads, dim, vdim, window=None, scale=None, rot_=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot_:
        m["rot"] = rot_
    return m


def gated_delta(heads, kv_heads, dim, vdim, conv=4):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def parallel(left, right, left_scale=1.0, right_scale=1.0):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def layer(mixer, ff=None):
    return dict(mixer, mlp={"kind": "dense", "ff": ff} if ff else None)


def config(width, vocab, layers, eps=1e-5, mult=1.0):
    return {"architecture": "Dumazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "layers": layers}


WAVES = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}      # wavelengths of 16..64 tokens are blended

# every mixer once; value heads in pairs over the q/k heads of the delta rule; two groups and two norm groups in the
# state-space mixer; a window of 20 (no multiple of the page); rotated dimensions below the head size
SMALL_A = dict(name="A", seed=3, std=0.25, norm_std=0.1, page_size=8, config=config(48, 131, [
    layer(retention(3, 8, 12, (0.5, 0.97, 0.999), rot(6, 100.0)), 40),
    layer(mamba2(4, 6, 10, groups=2, norm_groups=2, conv=3)),
    layer(parallel(window_attention(4, 2, 12, 20, window=20, scale=0.4, rot_=rot(8, 500.0, WAVES)), gated_delta(4, 2, 8, 12, conv=2),
                   0.7, 1.3), 56),
    layer(mamba2(2, 16, 8, conv=4), 24),
], mult=0.8))
# sizes that are no multiples of 4, no window, one kv head for three q heads, decays 0 and 1, five taps,
# a parallel layer first and without a feed-forward, a retention without rotation
SMALL_B = dict(name="B", seed=4, std=0.2, norm_std=0.2, page_size=16, config=config(90, 301, [
    layer(parallel(window_attention(3, 1, 10, 6, window=None, rot_=rot(10, 1e4)), gated_delta(2, 2, 18, 7, conv=5), 1.0, 0.5)),
    layer(retention(2, 20, 36, (0.0, 1.0)), 50),
    layer(mamba2(3, 10, 6, groups=3, norm_groups=3, conv=2), 34),
], eps=1e-6, mult=1.0))
# a window of one token, a window longer than every prompt, heads of 1, key and state sizes above a wave, a value
# size above the key size and below it
SMALL_C = dict(name="C", seed=5, std=0.3, norm_std=0.05, page_size=32, config=config(64, 97, [
    layer(parallel(window_attention(1, 1, 32, 16, window=1, rot_=rot(32, 1e6, dict(WAVES, factor=1.5))), gated_delta(1, 1, 72, 80), 0.3, 1.0), 96),
    layer(mamba2(1, 80, 72, conv=4)),
    layer(retention(1, 72, 40, (0.9,), rot(72, 250000.0)), 32),
    layer(parallel(window_attention(4, 4, 16, 48, window=1000, scale=0.7, rot_=rot(4)), gated_delta(2, 1, 16, 16, conv=3), 1.0, 1.0)),
], eps=1e-4, mult=0.5))
ALL_SMALL = [SMALL_A, SMALL_B, SMALL_C]


def make_folder(small, tmp_path, patch=None):
    """A model folder with random weights; ``patch`` {tensor name: value or function of the tensor} rewrites some."""
    from jax_vllm_amd import write_random_model

    folder = write_random_model(tmp_path, small["config"], seed=small["seed"], std=small["std"], norm_std=small["norm_std"])
    if patch:
        from safetensors.torch import load_file, save_file

        path = str(folder / "model.safetensors")
        tensors = load_file(path)
        for name, change in patch.items():
            t = tensors[name]
            new = change(t.float()) if callable(change) else torch.full_like(t.float(), float(change))
            tensors[name] = new.to(t.dtype).contiguous()
        save_file(tensors, path)
    return folder


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


def tokens_of(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=n).tolist()
