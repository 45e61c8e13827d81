"""Plain, slow, whole-sequence Dumazen in torch: the oracle of the test-suite for that design.

No cache, no batching, no kernels, one function per mechanism, nothing imported from the product
package.  A model is ``(config dict, {tensor name: tensor})``; every function works in the type of
the tensors it is given (float32, or float64 for a tighter oracle).  Recurrences run token by token.

The design in this file's notation (n tokens, width w, residual factor m):

* layer:      x += m * N1(mixer(x));  x += m * N2(ff(x))      (the sublayers read x itself; the second
              line only with a feed-forward);  N(y) = y / sqrt(mean(y^2) + eps) * (1 + weight)
* retention:  rotated q and k, k / sqrt(dim); per head S <- decay * S + k v^T, o = S^T q; every head's o by
              its own root mean square (no weight), times silu(gate), projected
* mamba2:     one input product cut into [z | x | B | C | dt]; x, B, C through a short causal convolution
              with bias and silu; dt = softplus(dt + bias); per head S <- exp(-exp(A) dt) S + dt B x^T,
              y = S^T C + D x; y * silu(z), normed in equal parts with a weight, projected
* parallel:   left_scale * (attention inside a sliding window: biases, a norm over the WHOLE q and the whole k
              projection, partial rotation with Llama-3.1-style frequency scaling, softmax) + right_scale *
              (gated delta rule: q, k, v through short convolutions without bias and silu, q and k unit
              vectors per head, q / sqrt(dim); S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
              per-head norm with a shared weight, times silu(gate), projected)
* feed-forward: down(gelu(up(x))) with biases, the exact (erf) gelu
* output:     N(x) with the final weight, logits = embed @ that
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
import torch.nn.functional as F


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
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


_ROUND_PRODUCTS_TO = None     # see ``rounded_products``


def linear(x, w, b=None):
    """w is stored [out, in]."""
    y = x @ w.T
    if b is not None:
        y = y + b
    return y if _ROUND_PRODUCTS_TO is None else y.to(_ROUND_PRODUCTS_TO).to(y.dtype)


class rounded_products:
    """Within this context every matrix product's result is rounded to ``dtype`` (and widened again): the
    least that an implementation with bfloat16 activations does to the numbers; the measure of the
    bfloat16 tests' tolerances."""

    def __init__(self, dtype=torch.bfloat16):
        self.dtype = dtype

    def __enter__(self):
        global _ROUND_PRODUCTS_TO
        self.before, _ROUND_PRODUCTS_TO = _ROUND_PRODUCTS_TO, self.dtype

    def __exit__(self, *exc):
        global _ROUND_PRODUCTS_TO
        _ROUND_PRODUCTS_TO = self.before


def short_conv(x, taps_w, bias=None):
    """x [n, channels]; taps_w [channels, taps], the last column weighs the current token, zeros stand
    before the first token."""
    n, c = x.shape
    taps = taps_w.shape[1]
    padded = torch.cat([x.new_zeros(taps - 1, c), x], dim=0)
    y = x.new_zeros(n, c)
    for j in range(taps):
        y = y + padded[j:j + n] * taps_w[:, j]
    return y if bias is None else y + bias


# --------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict):
    """Frequencies [dims/2] in double: base^(-2i/dims); with ``scaling`` = {factor, low, high, original}
    a pair whose wavelength is below original/high keeps its frequency, one above original/low is slowed
    down by ``factor``, and between the two they are blended by s = (original/wavelength - low)/(high - low)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for x in f:
            wave = 2 * math.pi / x
            if wave < orig / high:
                out.append(x)
            elif wave > orig / low:
                out.append(x / factor)
            else:
                s = (orig / wave - low) / (high - low)
                out.append((1 - s) * x / factor + s * x)
        f = out
    return torch.tensor(f, dtype=torch.float64)


def rotate(x, positions, rot: dict):
    """x [..., tokens, size]: the first rot['dims'] elements turn by position (element i paired with
    i + dims/2), the others pass.  Angles in 32-bit."""
    dims = int(rot["dims"])
    f = rotary_frequencies(rot).to(torch.float32)
    ang = positions.to(torch.float32)[:, None] * f[None, :]
    cos, sin = torch.cos(ang).to(x.dtype), torch.sin(ang).to(x.dtype)
    u, v, rest = x[..., : dims // 2], x[..., dims // 2: dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


# --------------------------------------------------------------------------- mixers
def retention(w: dict, p: str, m: dict, h, eps: float):
    n = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(n)
    q = linear(h, w[p + "q"]).view(n, H, d).transpose(0, 1)
    k = linear(h, w[p + "k"]).view(n, H, d).transpose(0, 1)
    v = linear(h, w[p + "v"]).view(n, H, dv).transpose(0, 1)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    k = k * d ** -0.5
    out = h.new_zeros(n, H, dv)
    for hd in range(H):
        S = h.new_zeros(d, dv)
        lam = float(m["decay"][hd])
        for t in range(n):
            S = lam * S + torch.outer(k[hd, t], v[hd, t])
            out[t, hd] = S.T @ q[hd, t]
    out = rms(out, eps).reshape(n, H * dv) * silu(linear(h, w[p + "g"]))
    return linear(out, w[p + "o"])


def mamba2(w: dict, p: str, m: dict, h, eps: float):
    n = h.shape[0]
    H, dv, N, G, NG = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["norm_groups"])
    inner = H * dv
    proj = linear(h, w[p + "in"])
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    if _ROUND_PRODUCTS_TO is not None:
        xbc = xbc.to(_ROUND_PRODUCTS_TO).to(h.dtype)
    x = xbc[:, :inner].view(n, H, dv)
    B = xbc[:, inner:inner + G * N].view(n, G, N)
    C = xbc[:, inner + G * N:].view(n, G, N)
    dt = F.softplus(dt + w[p + "dt_bias"], threshold=1e9)
    a = torch.exp(-torch.exp(w[p + "A_log"]) * dt)             # [n, H]
    y = h.new_zeros(n, H, dv)
    for hd in range(H):
        g = hd // (H // G)
        S = h.new_zeros(N, dv)
        for t in range(n):
            S = a[t, hd] * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + w[p + "D"][hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    y = rms(y.view(n, NG, inner // NG), eps).reshape(n, inner) * w[p + "norm"]
    return linear(y, w[p + "o"])


def window_attention(w: dict, p: str, m: dict, h, eps: float):
    n = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(n)
    q = linear(h, w[p + "q"], w[p + "q.b"])
    k = linear(h, w[p + "k"], w[p + "k.b"])
    v = linear(h, w[p + "v"], w[p + "v.b"]).view(n, G, dv).transpose(0, 1)
    q = (rms(q, eps) * w[p + "q.norm"]).view(n, H, d).transpose(0, 1)
    k = (rms(k, eps) * w[p + "k.norm"]).view(n, G, d).transpose(0, 1)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    k = k.repeat_interleave(H // G, dim=0)
    v = v.repeat_interleave(H // G, dim=0)
    s = (q @ k.transpose(1, 2)) * float(m["scale"])
    dist = pos[:, None] - pos[None, :]
    seen = dist >= 0
    size = (m.get("mask") or {}).get("size")
    if size:
        seen = seen & (dist < int(size))
    s = s.masked_fill(~seen, float("-inf"))
    o = torch.softmax(s, dim=-1) @ v
    return linear(o.transpose(0, 1).reshape(n, H * dv), w[p + "o"])


def gated_delta(w: dict, p: str, m: dict, h, eps: float):
    n = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])

    def conv_silu(name):
        y = silu(short_conv(linear(h, w[p + name]), w[p + name + ".conv"]))
        return y if _ROUND_PRODUCTS_TO is None else y.to(_ROUND_PRODUCTS_TO).to(h.dtype)

    q = conv_silu("q").view(n, G, d)
    k = conv_silu("k").view(n, G, d)
    v = conv_silu("v").view(n, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                      # [n, H]
    g = torch.exp(-torch.exp(w[p + "A_log"]) * F.softplus(h @ w[p + "a"].T + w[p + "dt_bias"], threshold=1e9))
    out = h.new_zeros(n, H, dv)
    for hd in range(H):
        kh = hd // (H // G)
        S = h.new_zeros(d, dv)
        for t in range(n):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hd] = S.T @ q[t, kh]
    out = rms(out, eps) * w[p + "norm"]
    out = out.reshape(n, H * dv) * silu(linear(h, w[p + "g"]))
    return linear(out, w[p + "o"])


def parallel(w: dict, p: str, m: dict, h, eps: float):
    left = window_attention(w, p + "left.", m["left"], h, eps)
    right = gated_delta(w, p + "right.", m["right"], h, eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


MIXERS = {"retention": retention, "mamba2": mamba2, "parallel": parallel}


# --------------------------------------------------------------------------- feed-forward
def dense_ff(w: dict, p: str, f: dict, h):
    a = linear(h, w[p + "up"], w[p + "up.b"])
    a = 0.5 * a * (1 + torch.erf(a / math.sqrt(2.0)))
    if _ROUND_PRODUCTS_TO is not None:
        a = a.to(_ROUND_PRODUCTS_TO).to(h.dtype)
    return linear(a, w[p + "down"], w[p + "down.b"])


# --------------------------------------------------------------------------- the model
def one_plus_norm(x, weight, eps):
    return rms(x, eps) * (1 + weight)


def forward(w: dict, cfg: dict, tokens, layers_out: list | None = None):
    """Logits [n, vocab] of one sequence from position 0; with ``layers_out`` the residual stream after
    every layer is appended to it."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](w, p + "mix.", layer["mixer"], x, eps)
        x = x + mult * one_plus_norm(y, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = dense_ff(w, p + "mlp.", layer["mlp"], x)
            x = x + mult * one_plus_norm(y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = one_plus_norm(x, w["final.norm"], eps)
    return linear(x, w["embed"])
