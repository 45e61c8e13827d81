"""Plain, slow, whole-sequence Lomozen in torch: the oracle of the test-suite for that design.

No cache, no batching, no kernels, one function per mechanism, nothing imported from the
product package.  A model is ``(config dict, {tensor name: tensor})``; every function works
in the type of the tensors it is given (float32, or float64 for a tighter oracle).

The design in this file's notation (n tokens, width w):

* layer:      x += N1b(mixer(N1(x)));  x += N2b(ff(N2(x)))   (the second line only with a feed-forward)
* N(x):       x / sqrt(mean(x^2) + eps) * weight
* latent attention: a low-rank query (down, norm, up), one normed latent c per token from which
  every head's unrotated key and its value are made, one rotated key part shared by the heads,
  a sliding window, softmax, a sigmoid gate on the concatenated heads;
* lightning:  per head a matrix state S <- decay * S + k v^T, output S^T q, with q, k, v = silu
  of projections; the heads' outputs normed together, gated, projected;
* feed-forward: routed experts chosen by the largest sigmoid scores, the score multiplying the
  expert's input, plus an expert that every token uses.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- files
def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def read_weights(folder, dtype=torch.float32) -> dict:
    from safetensors.torch import load_file

    out = {}
    for shard in sorted(Path(folder).glob("*.safetensors")):
        for k, v in load_file(str(shard)).items():
            out[k] = v.to(dtype) if v.is_floating_point() else v
    return out


# --------------------------------------------------------------------------- small pieces
def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


_ROUND_PRODUCTS_TO = None     # see ``rounded_products``


def linear(x, w):
    """w is stored [out, in]."""
    y = x @ w.T
    return y if _ROUND_PRODUCTS_TO is None else y.to(_ROUND_PRODUCTS_TO).to(y.dtype)


class rounded_products:
    """Within this context every matrix product's result is rounded to ``dtype`` (and widened again): what
    an implementation that keeps its activations in bfloat16 does to the numbers at the least.  The
    difference to the unrounded run says how much of such rounding the model at hand lets through to its
    logits, which is the measure for the bfloat16 tests' tolerances."""

    def __init__(self, dtype=torch.bfloat16):
        self.dtype = dtype

    def __enter__(self):
        global _ROUND_PRODUCTS_TO
        self.before, _ROUND_PRODUCTS_TO = _ROUND_PRODUCTS_TO, self.dtype

    def __exit__(self, *exc):
        global _ROUND_PRODUCTS_TO
        _ROUND_PRODUCTS_TO = self.before


# --------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict, dtype=torch.float64):
    """(frequencies [dims/2], amplitude of cos and sin).  Without ``scaling``: base^(-2i/dims)
    and 1.  With it (YaRN): dimensions that turn fast keep their frequency, slow ones are
    divided by ``factor``, a linear ramp between; amplitude 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    amp = 1.0
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(t):
            return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))

        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    return f.to(dtype), amp


def rotate(x, positions, rot: dict):
    """x [..., tokens, size]: the first rot['dims'] elements turn by position (element i paired
    with i + dims/2), the others pass."""
    dims = int(rot["dims"])
    f, amp = rotary_frequencies(rot, torch.float32)
    ang = positions.to(torch.float32)[:, None] * f[None, :]          # angles in 32-bit
    cos, sin = (torch.cos(ang) * amp).to(x.dtype), (torch.sin(ang) * amp).to(x.dtype)
    u, v, rest = x[..., : dims // 2], x[..., dims // 2: dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


# --------------------------------------------------------------------------- mixers
def latent_attention(w: dict, p: str, m: dict, h, eps: float):
    """h [tokens, width] of one sequence from position 0."""
    n = h.shape[0]
    H, d, r, dv, kr = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(n)
    cq = rms_norm(linear(h, w[p + "dq"]), w[p + "dq.norm"], eps)
    q = linear(cq, w[p + "uq"]).view(n, H, d + r)
    q_plain, q_rot = q[..., :d], q[..., d:]
    dkv = linear(h, w[p + "dkv"])
    c = rms_norm(dkv[:, :kr], w[p + "dkv.norm"], eps)
    k_rot = rotate(dkv[:, kr:], pos, m["rot"])                        # [n, r], one for all heads
    q_rot = rotate(q_rot.transpose(0, 1), pos, m["rot"]).transpose(0, 1)
    k_plain = linear(c, w[p + "uk"]).view(n, H, d)
    v = linear(c, w[p + "uv"]).view(n, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * float(m["scale"])
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i)
    size = (m.get("mask") or {}).get("size")
    if size:
        seen = seen & (i - j < int(size))
    scores = scores.masked_fill(~seen, float("-inf"))
    out = torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v).reshape(n, H * dv)
    out = out * torch.sigmoid(linear(h, w[p + "g"]))
    return linear(out, w[p + "o"])


def lightning(w: dict, p: str, m: dict, h, eps: float, state=None):
    """Token by token.  ``state`` [heads, dim, vdim] or None for zeros; returns (out, state)."""
    n = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(linear(h, w[p + "q"])).view(n, H, d)
    k = silu(linear(h, w[p + "k"])).view(n, H, d)
    v = silu(linear(h, w[p + "v"])).view(n, H, dv)
    decay = torch.tensor([float(x) for x in m["decay"]], dtype=h.dtype)
    S = torch.zeros(H, d, dv, dtype=h.dtype) if state is None else state.clone()
    outs = []
    for t in range(n):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        outs.append(torch.einsum("hde,hd->he", S, q[t]))
    o = torch.stack(outs).reshape(n, H * dv)
    o = rms_norm(o, w[p + "norm"], eps) * torch.sigmoid(linear(h, w[p + "g"]))
    return linear(o, w[p + "o"]), S


# --------------------------------------------------------------------------- feed-forward
def expert(w: dict, p: str, x):
    return linear(silu(linear(x, w[p + "gate"])) * linear(x, w[p + "up"]), w[p + "down"])


def routed_feed_forward(w: dict, p: str, f: dict, h):
    n_exp, top = int(f["router"]["experts"]), int(f["router"]["top"])
    s = torch.sigmoid(linear(h, w[p + "router"]))
    val, idx = torch.topk(s, top, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for kk in range(top):
            e = int(idx[t, kk])
            out[t] += expert(w, f"{p}e{e}.", val[t, kk] * h[t])
    if f.get("shared"):
        out = out + expert(w, p + "shared.", h)
    return out


# --------------------------------------------------------------------------- the model
def forward(w: dict, cfg: dict, tokens, residuals: list | None = None):
    """Logits [tokens, vocab] of one sequence; ``residuals`` receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        hin = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            a = latent_attention(w, p + "mix.", layer["mixer"], hin, eps)
        elif layer["type"] == "lightning":
            a, _ = lightning(w, p + "mix.", layer["mixer"], hin, eps)
        else:
            raise ValueError(f"unknown mixer {layer['type']!r}")
        x = x + rms_norm(a, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            f = routed_feed_forward(w, p + "mlp.", layer["mlp"], rms_norm(x, w[p + "norm2"], eps))
            x = x + rms_norm(f, w[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return linear(rms_norm(x, w["final.norm"], eps), w["head"])
