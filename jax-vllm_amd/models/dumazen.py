"""Dumazen: a decoder whose layers are listed one by one in ``config.json``, each with one of three mixers
(retention; a Mamba-2 state-space mixer; attention inside a sliding window side by side with a gated delta
rule), an optional dense feed-forward with biases, and a norm on every sublayer's OUTPUT only: the sublayers
read the residual stream itself, and their normed results join it times a constant.  The head is the embedding
table.  This file reads that configuration and turns it into a ``ModelSpec``; the mechanisms are parts of their
own (``parts/recurrent.py``, ``parts/attention.py``, ``parts/mlp.py: DenseMLP``, ``parts/block.py:
OutputNormBlock``, ``parts/rotary.py``).

``config.json``: ``architecture`` "Dumazen", ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, and ``layers``:
a list of ``{type, mixer: {...sizes and constants...}, mlp: {kind: "dense", ff} | null}``.  Tensor names: ``embed``,
``final.norm``, and per layer ``l<i>.norm1 | norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from ..config.errors import ConfigError
from ..config.model import config_value, read_config_json
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MIXERS = ("retention", "mamba2", "parallel")


def _positive(where: str, c: Mapping, key: str) -> int:
    v = config_value(c, key, int)
    if v <= 0:
        raise ConfigError(f"{where}.{key} must be positive, got {v}")
    return v


def _section(where: str, c: Mapping, key: str, required: bool = True) -> Optional[Mapping]:
    v = c.get(key)
    if v is None:
        if required:
            raise ConfigError(f"config.json lacks {where}.{key}")
        return None
    if not isinstance(v, Mapping):
        raise ConfigError(f"{where}.{key} must be an object")
    return v


def _check_rot(where: str, m: Mapping, dim: int) -> None:
    rot = _section(where, m, "rot", required=False)
    if rot is None:
        return
    dims = _positive(where + ".rot", rot, "dims")
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}.rot.dims must be even and at most dim = {dim}, got {dims}")
    if not config_value(rot, "base", float) > 1.0:
        raise ConfigError(f"{where}.rot.base must be above 1")
    sc = _section(where + ".rot", rot, "scaling", required=False)
    if sc is not None:
        for key in ("factor", "low", "high", "original"):
            if not config_value(sc, key, float) > 0:
                raise ConfigError(f"{where}.rot.scaling.{key} must be positive")
        if float(sc["high"]) == float(sc["low"]):
            raise ConfigError(f"{where}.rot.scaling: high and low must differ")


def _check_retention(where: str, m: Mapping) -> None:
    heads, dim = _positive(where, m, "heads"), _positive(where, m, "dim")
    _positive(where, m, "vdim")
    decay = m.get("decay")
    if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(d, (int, float)) and 0 <= d <= 1 for d in decay):
        raise ConfigError(f"{where}.decay must list one number in [0, 1] for each of the {heads} heads")
    _check_rot(where, m, dim)


def _check_mamba2(where: str, m: Mapping) -> None:
    heads, vdim = _positive(where, m, "heads"), _positive(where, m, "vdim")
    _positive(where, m, "state")
    groups, parts = _positive(where, m, "groups"), _positive(where, m, "norm_groups")
    if heads % groups:
        raise ConfigError(f"{where}: {heads} heads are not a multiple of {groups} groups")
    if (heads * vdim) % parts:
        raise ConfigError(f"{where}: heads * vdim = {heads * vdim} does not split into {parts} norm groups")
    _positive(where, m, "conv")


def _check_window_attention(where: str, m: Mapping) -> None:
    heads, kv = _positive(where, m, "heads"), _positive(where, m, "kv_heads")
    if heads % kv:
        raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv} kv_heads")
    dim = _positive(where, m, "dim")
    _positive(where, m, "vdim")
    if not config_value(m, "scale", float) > 0:
        raise ConfigError(f"{where}.scale must be positive")
    mask = _section(where, m, "mask", required=False)
    if mask is not None and mask.get("size") is not None:
        _positive(where + ".mask", mask, "size")
    _check_rot(where, m, dim)


def _check_gated_delta(where: str, m: Mapping) -> None:
    heads, kv = _positive(where, m, "heads"), _positive(where, m, "kv_heads")
    if heads % kv:
        raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv} kv_heads")
    for key in ("dim", "vdim", "conv"):
        _positive(where, m, key)


def _check_parallel(where: str, m: Mapping) -> None:
    _check_window_attention(where + ".left", _section(where, m, "left"))
    _check_gated_delta(where + ".right", _section(where, m, "right"))
    for key in ("left_scale", "right_scale"):
        config_value(m, key, float)


_CHECKS = {"retention": _check_retention, "mamba2": _check_mamba2, "parallel": _check_parallel}


def _check_mlp(where: str, f: Mapping) -> None:
    kind = f.get("kind", "dense")
    if kind != "dense":
        raise ConfigError(f"{where}.kind {kind!r}: this architecture's feed-forward is 'dense'")
    _positive(where, f, "ff")


@dataclass(frozen=True)
class DumazenLayer:
    kind: str                       # one of MIXERS
    mixer: Mapping[str, Any]        # the mixer's sizes and constants, checked
    mlp: Optional[Mapping[str, Any]]


@dataclass(frozen=True)
class DumazenConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    layers: tuple
    raw: Mapping[str, Any]

    @classmethod
    def from_dict(cls, c: Mapping[str, Any]) -> "DumazenConfig":
        vocab, width = _positive("config", c, "vocab"), _positive("config", c, "width")
        eps = config_value(_section("config", c, "norm"), "eps", float)
        if not eps >= 0.0:
            raise ConfigError("norm.eps must be non-negative")
        mult = config_value(c, "residual_mult", float)
        listed = c.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json needs a non-empty list 'layers'")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{where} must be an object")
            kind = config_value(entry, "type", str)
            if kind not in MIXERS:
                raise ConfigError(f"{where}.type {kind!r} is not one of {MIXERS}")
            m = _section(where, entry, "mixer")
            _CHECKS[kind](where + ".mixer", m)
            mlp = _section(where, entry, "mlp", required=False)
            if mlp is not None:
                _check_mlp(where + ".mlp", mlp)
            layers.append(DumazenLayer(kind, m, mlp))
        return cls(vocab, width, eps, mult, tuple(layers), dict(c))

    @classmethod
    def from_folder(cls, path) -> "DumazenConfig":
        return cls.from_dict(read_config_json(path))

    def to_dict(self) -> dict:
        return dict(self.raw)


def _rotary(m: Mapping) -> Optional[PartSpec]:
    rot = m.get("rot")
    if not rot:
        return None
    sc = rot.get("scaling")
    return PartSpec("rotary", {
        "head_dim": m["dim"], "theta": float(rot["base"]), "rotary_dim": rot["dims"],
        "by_wavelength": {k: float(sc[k]) for k in ("factor", "low", "high", "original")} if sc else None})


def _retention(cfg: DumazenConfig, m: Mapping):
    spec = PartSpec("retention", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "head_dim": m["dim"], "v_dim": m["vdim"],
        "decay": tuple(float(d) for d in m["decay"]), "norm_eps": cfg.eps, "position": _rotary(m)})
    return spec, {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate.weight": "g", "o_proj.weight": "o"}


def _mamba2(cfg: DumazenConfig, m: Mapping):
    spec = PartSpec("state_space", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "v_dim": m["vdim"], "state_size": m["state"],
        "groups": m["groups"], "conv_taps": m["conv"], "norm_groups": m["norm_groups"], "norm_eps": cfg.eps})
    return spec, {"in_proj.weight": "in", "conv.weight": "conv", "conv.bias": "conv.b", "norm.weight": "norm",
                  "o_proj.weight": "o"}


def _window_attention(cfg: DumazenConfig, m: Mapping):
    spec = PartSpec("gqa_attention", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
        "v_head_dim": m["vdim"], "qk_norm_eps": cfg.eps, "qk_norm": "whole", "position": _rotary(m),
        "window": (m.get("mask") or {}).get("size"), "scale": float(m["scale"]), "qkv_bias": True})
    names = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "q_proj.bias": "q.b", "k_proj.bias": "k.b",
             "v_proj.bias": "v.b", "q_norm.weight": "q.norm", "k_norm.weight": "k.norm", "o_proj.weight": "o"}
    return spec, names


def _gated_delta(cfg: DumazenConfig, m: Mapping):
    spec = PartSpec("gated_delta", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "num_qk_heads": m["kv_heads"], "head_dim": m["dim"],
        "v_dim": m["vdim"], "conv_taps": m["conv"], "norm_eps": cfg.eps})
    names = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "q_conv.weight": "q.conv",
             "k_conv.weight": "k.conv", "v_conv.weight": "v.conv", "beta_proj.weight": "b", "decay_proj.weight": "a",
             "gate.weight": "g", "norm.weight": "norm", "o_proj.weight": "o"}
    return spec, names


def _parallel(cfg: DumazenConfig, m: Mapping):
    left, left_names = _window_attention(cfg, m["left"])
    right, right_names = _gated_delta(cfg, m["right"])
    spec = PartSpec("parallel", {"left": left, "right": right, "left_scale": float(m["left_scale"]),
                                 "right_scale": float(m["right_scale"])})
    names = {"left." + k: "left." + v for k, v in left_names.items()}
    names.update({"right." + k: "right." + v for k, v in right_names.items()})
    return spec, names


_MIXER_SPECS = {"retention": _retention, "mamba2": _mamba2, "parallel": _parallel}


def build_spec(cfg: DumazenConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        mixer, mixer_names = _MIXER_SPECS[layer.kind](cfg, layer.mixer)
        rename = {"mix." + k: "mix." + v for k, v in mixer_names.items()}
        ffn = None
        norms = ("norm1", "norm2") if layer.mlp is not None else ("norm1",)
        if layer.mlp is not None:
            ffn = PartSpec("dense_mlp", {"hidden_size": cfg.width, "intermediate_size": layer.mlp["ff"],
                                         "activation": "gelu", "bias": True})
            rename.update({"mlp.up_proj.weight": "mlp.up", "mlp.up_proj.bias": "mlp.up.b",
                           "mlp.down_proj.weight": "mlp.down", "mlp.down_proj.bias": "mlp.down.b"})
        rename.update({f"{n}.weight": n for n in norms})
        # the constant on every sublayer's share of the stream is part of that sublayer's norm
        norm = PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps, "one_plus": True, "gain": cfg.residual_mult})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn,
                                block=PartSpec("output_norm", {"norm": norm, "has_feed_forward": ffn is not None}),
                                mixer_prefix="mix.", feed_forward_prefix="mlp.", rename=rename))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}),
        embedding_prefix="embed.",
        final_norm=PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps, "one_plus": True}), final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}), head_prefix="head.",
        layers=layers, schedule=[LayerRun(i) for i in range(len(layers))], tie_head_to_embedding=True,
        rename={"embed.weight": "embed", "final.norm.weight": "final.norm"},
    )


register_architecture("Dumazen", DumazenConfig.from_dict, build_spec)
