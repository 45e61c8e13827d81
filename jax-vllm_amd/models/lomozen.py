"""Lomozen: a decoder whose layers are listed one by one in ``config.json``, each with one of two
mixers (attention through a cached latent with a sliding window and rescaled rotary frequencies, or
linear attention with a decaying matrix state), an optional feed-forward of routed experts with a
shared expert, and a norm before AND after every sublayer.  This file reads that configuration and
turns it into a ``ModelSpec``; the mechanisms are parts of their own (``parts/latent_attention.py``,
``parts/lightning.py``, ``parts/moe.py``, ``parts/block.py: SandwichBlock``, ``parts/rotary.py``).

``config.json``: ``architecture`` "Lomozen", ``vocab``, ``width``, ``norm.eps``, and ``layers``: a list of
``{type, mixer: {...sizes and constants...}, mlp: {...} | null}``.  Tensor names: ``embed``, ``final.norm``,
``head``, and per layer ``l<i>.norm1 | norm1b | norm2 | norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from ..config.errors import ConfigError
from ..config.model import config_value, read_config_json
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MIXERS = ("latent_attention", "lightning")


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


@dataclass(frozen=True)
class LomozenLayer:
    kind: str                       # one of MIXERS
    mixer: Mapping[str, Any]        # the mixer's sizes and constants, checked
    mlp: Optional[Mapping[str, Any]]


@dataclass(frozen=True)
class LomozenConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    raw: Mapping[str, Any]

    @classmethod
    def from_dict(cls, c: Mapping[str, Any]) -> "LomozenConfig":
        vocab, width = _positive("config", c, "vocab"), _positive("config", c, "width")
        eps = config_value(_section("config", c, "norm"), "eps", float)
        if not eps >= 0.0:
            raise ConfigError("norm.eps must be non-negative")
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
            (_check_latent if kind == "latent_attention" else _check_lightning)(where + ".mixer", m)
            mlp = _section(where, entry, "mlp", required=False)
            if mlp is not None:
                _check_mlp(where + ".mlp", mlp)
            layers.append(LomozenLayer(kind, m, mlp))
        return cls(vocab, width, eps, tuple(layers), dict(c))

    @classmethod
    def from_folder(cls, path) -> "LomozenConfig":
        return cls.from_dict(read_config_json(path))

    def to_dict(self) -> dict:
        return dict(self.raw)


def _check_latent(where: str, m: Mapping) -> None:
    for key in ("heads", "dim", "vdim", "kv_rank", "q_rank"):
        _positive(where, m, key)
    rot_dim = config_value(m, "rot_dim", int)
    if rot_dim < 0:
        raise ConfigError(f"{where}.rot_dim must not be negative")
    if not config_value(m, "scale", float) > 0:
        raise ConfigError(f"{where}.scale must be positive")
    mask = _section(where, m, "mask", required=False)
    if mask is not None and mask.get("size") is not None:
        _positive(where + ".mask", mask, "size")
    if rot_dim:
        rot = _section(where, m, "rot")
        dims = _positive(where + ".rot", rot, "dims")
        if dims % 2 or dims > rot_dim:
            raise ConfigError(f"{where}.rot.dims must be even and at most rot_dim = {rot_dim}, got {dims}")
        if not config_value(rot, "base", float) > 1.0:
            raise ConfigError(f"{where}.rot.base must be above 1")
        sc = _section(where + ".rot", rot, "scaling", required=False)
        if sc is not None:
            for key in ("factor", "original", "fast", "slow"):
                if not config_value(sc, key, float) > 0:
                    raise ConfigError(f"{where}.rot.scaling.{key} must be positive")


def _check_lightning(where: str, m: Mapping) -> None:
    heads = _positive(where, m, "heads")
    _positive(where, m, "dim")
    _positive(where, m, "vdim")
    decay = m.get("decay")
    if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(d, (int, float)) and 0 <= d <= 1 for d in decay):
        raise ConfigError(f"{where}.decay must list one number in [0, 1] for each of the {heads} heads")


def _check_mlp(where: str, f: Mapping) -> None:
    kind = f.get("kind", "moe")
    if kind != "moe":
        raise ConfigError(f"{where}.kind {kind!r}: this architecture's feed-forward is 'moe'")
    router = _section(where, f, "router")
    experts, top = _positive(where + ".router", router, "experts"), _positive(where + ".router", router, "top")
    if top > experts:
        raise ConfigError(f"{where}.router.top = {top} exceeds its {experts} experts")
    _positive(where + ".expert", _section(where, f, "expert"), "ff")
    shared = _section(where, f, "shared", required=False)
    if shared is not None:
        _positive(where + ".shared", shared, "ff")


def _mixer_spec(cfg: LomozenConfig, layer: LomozenLayer):
    """(PartSpec of the mixer, local tensor name -> name below the layer's prefix)."""
    m = layer.mixer
    if layer.kind == "lightning":
        spec = PartSpec("lightning_attention", {
            "hidden_size": cfg.width, "num_heads": m["heads"], "head_dim": m["dim"], "v_dim": m["vdim"],
            "decay": tuple(float(d) for d in m["decay"]), "norm_eps": cfg.eps})
        names = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate.weight": "g",
                 "o_proj.weight": "o", "norm.weight": "norm"}
        return spec, names
    position = None
    if m["rot_dim"]:
        rot = m["rot"]
        sc = rot.get("scaling")
        position = PartSpec("rotary", {
            "head_dim": m["rot_dim"], "theta": float(rot["base"]), "rotary_dim": rot["dims"],
            "rescale": {k: float(sc[k]) for k in ("factor", "original", "fast", "slow")} if sc else None})
    mask = m.get("mask") or {}
    spec = PartSpec("latent_attention", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
        "v_dim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": float(m["scale"]),
        "norm_eps": cfg.eps, "position": position, "window": mask.get("size"), "output_gate": True})
    names = {"q_down.weight": "dq", "q_norm.weight": "dq.norm", "q_up.weight": "uq", "kv_down.weight": "dkv",
             "kv_norm.weight": "dkv.norm", "k_up.weight": "uk", "v_up.weight": "uv", "gate.weight": "g",
             "o_proj.weight": "o"}
    return spec, names


def _mlp_spec(cfg: LomozenConfig, f: Mapping):
    experts, top, ff = f["router"]["experts"], f["router"]["top"], f["expert"]["ff"]
    shared = f.get("shared")
    spec = PartSpec("routed_experts", {
        "hidden_size": cfg.width, "num_experts": experts, "top": top, "expert_size": ff, "activation": "silu",
        "weight_on_input": True,
        "shared": PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": shared["ff"],
                                         "activation": "silu"}) if shared else None})
    names = {"router.weight": "router"}
    for e in range(experts):
        for part in ("gate", "up", "down"):
            names[f"experts.{e}.{part}.weight"] = f"e{e}.{part}"
    if shared:
        names.update({"shared.gate_proj.weight": "shared.gate", "shared.up_proj.weight": "shared.up",
                      "shared.down_proj.weight": "shared.down"})
    return spec, names


def build_spec(cfg: LomozenConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps})
    layers = []
    for i, layer in enumerate(cfg.layers):
        mixer, mixer_names = _mixer_spec(cfg, layer)
        rename = {"mix." + k: "mix." + v for k, v in mixer_names.items()}
        ffn = None
        norms = ("norm1", "norm1b", "norm2", "norm2b") if layer.mlp is not None else ("norm1", "norm1b")
        if layer.mlp is not None:
            ffn, ffn_names = _mlp_spec(cfg, layer.mlp)
            rename.update({"mlp." + k: "mlp." + v for k, v in ffn_names.items()})
        rename.update({f"{n}.weight": n for n in norms})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn,
                                block=PartSpec("sandwich", {"norm": norm, "has_feed_forward": ffn is not None}),
                                mixer_prefix="mix.", feed_forward_prefix="mlp.", rename=rename))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}),
        embedding_prefix="embed.",
        final_norm=norm, final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}), head_prefix="head.",
        layers=layers, schedule=[LayerRun(i) for i in range(len(layers))],
        rename={"embed.weight": "embed", "final.norm.weight": "final.norm", "head.weight": "head"},
    )


register_architecture("Lomozen", LomozenConfig.from_dict, build_spec)
