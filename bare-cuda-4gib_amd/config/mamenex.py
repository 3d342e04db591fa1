"""Configuration of the Mamenex decoder: a stack of layers that each name their mixer -- latent attention or a
real-gated linear recurrent unit -- and, optionally, a dense feed-forward; every sublayer normed on both sides, a short
causal convolution in front of every mixer, the output head tied to the embedding table.

config.json keys: ``vocab``, ``width``, ``norm.eps``, ``canon.taps`` and ``layers``, a list of
``{"type": "latent_attention" | "rglru", "mixer": {...sizes...}, "mlp": {"kind": "dense", "ff": N} | null}``.
Tensor names: ``embed``, ``final.norm``, and for layer i ``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``,
``l<i>.norm2b``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List

from ..errors import ConfigError
from .base import ModelConfig, field_from_json
from .registry import Architecture, register_architecture

_MIXER_KEYS = {
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"),
    "rglru": ("width", "blocks", "conv"),
}


def _number(where: str, d: Dict[str, Any], key: str, integer: bool = True):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (integer and int(v) != v):
        raise ConfigError(f"config.json: {where}.{key} must be {'an integer' if integer else 'a number'}, got {v!r}")
    return int(v) if integer else float(v)


@dataclasses.dataclass
class MamenexConfig(ModelConfig):
    vocab_size: int = field_from_json("vocab")
    hidden_size: int = field_from_json("width")
    layers: List[Dict[str, Any]] = field_from_json("layers")
    norm: Dict[str, Any] = field_from_json("norm")
    canon: Dict[str, Any] = field_from_json("canon")
    max_seq_len: int = field_from_json("max_positions", 1 << 20)     # (nothing in the design bounds a position)

    def derive(self, raw: Dict[str, Any]) -> None:
        if not isinstance(self.norm, dict) or not isinstance(self.canon, dict):
            raise ConfigError("config.json: 'norm' and 'canon' must be objects")
        self.norm_eps = _number("norm", self.norm, "eps", integer=False)
        self.canon_taps = _number("canon", self.canon, "taps")

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or self.max_seq_len <= 0:
            raise ConfigError(f"config.json: vocab {self.vocab_size} and width {self.hidden_size} must be positive")
        if self.norm_eps < 0 or self.canon_taps < 1:
            raise ConfigError(f"config.json: norm.eps {self.norm_eps} must not be negative, canon.taps {self.canon_taps} at least 1")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        for n, layer in enumerate(self.layers):
            where = f"layers[{n}]"
            if not isinstance(layer, dict) or layer.get("type") not in _MIXER_KEYS:
                raise ConfigError(f"config.json: {where}.type must be one of {sorted(_MIXER_KEYS)}, got "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where}.mixer must be an object")
            missing = [k for k in _MIXER_KEYS[layer["type"]] if k not in m]
            if missing:
                raise ConfigError(f"config.json: {where}.mixer lacks {', '.join(missing)}")
            if layer["type"] == "latent_attention":
                for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
                    _number(where + ".mixer", m, k)
                _number(where + ".mixer", m, "scale", integer=False)
                if not isinstance(m["rot"], dict):
                    raise ConfigError(f"config.json: {where}.mixer.rot must be an object")
                _number(where + ".mixer.rot", m["rot"], "dims")
                _number(where + ".mixer.rot", m["rot"], "base", integer=False)
            else:
                for k in ("width", "blocks", "conv"):
                    _number(where + ".mixer", m, k)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp must be null or of kind 'dense', got {mlp!r}")
                _number(where + ".mlp", mlp, "ff")

    def to_dict(self) -> Dict[str, Any]:
        out = super().to_dict()
        out["architecture"] = "Mamenex"
        return out


def describe_mamenex(cfg: MamenexConfig):
    """The layer stack as data: every layer a ``sandwich`` block (norms before and after each sublayer, weights stored
    around zero) whose mixer reads its input plus a causal convolution of it."""
    from ..engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

    width = cfg.hidden_size

    def norm(prefix: str, name: str) -> "PartSpec":
        return PartSpec("rmsnorm", dict(size=width, eps=cfg.norm_eps, offset=1.0), prefix=prefix, rename={"weight": name})

    layers = []
    for n, layer in enumerate(cfg.layers):
        p, m = f"l{n}.", layer["mixer"]
        if layer["type"] == "latent_attention":
            mixer = PartSpec("latent_attention", dict(
                hidden_size=width, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                kv_rank=int(m["kv_rank"]), scale=float(m["scale"]), rot_dims=int(m["rot"]["dims"]),
                rot_base=float(m["rot"]["base"]), eps=cfg.norm_eps, sink=True), prefix=p + "mix.")
        else:
            mixer = PartSpec("rglru", dict(hidden_size=width, width=int(m["width"]), blocks=int(m["blocks"]),
                                           conv_taps=int(m["conv"])), prefix=p + "mix.")
        extras = {"mixer_post_norm": ("norm", norm(p, "norm1b")),
                  "mixer_conv": ("conv", PartSpec("causal", dict(channels=width, taps=cfg.canon_taps), prefix=p,
                                                  rename={"weight": "canon1"}))}
        ffn = ffn_norm = None
        if layer.get("mlp") is not None:
            ffn = PartSpec("dense_xielu", dict(hidden_size=width, intermediate_size=int(layer["mlp"]["ff"])), prefix=p + "mlp.")
            ffn_norm = norm(p, "norm2")
            extras["ffn_post_norm"] = ("norm", norm(p, "norm2b"))
        layers.append(LayerSpec(block="sandwich", mixer=mixer, ffn=ffn, mixer_norm=norm(p, "norm1"), ffn_norm=ffn_norm,
                                extras=extras))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=width, max_seq_len=cfg.max_seq_len,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=width), rename={"weight": "embed"}),
        layers=layers,
        schedule=[ScheduleEntry(layer=n, cache=n, writes=True) for n in range(len(layers))],
        final_norm=norm("final.", "norm"),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=width, tied_to="embed"), prefix="head."),
    )


MAMENEX = register_architecture(Architecture(name="Mamenex", model_type="mamenex", config_class=MamenexConfig,
                                             describe=describe_mamenex))
