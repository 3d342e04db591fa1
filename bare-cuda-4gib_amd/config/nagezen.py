"""Configuration of the Nagezen decoder: a stack of layers that each name their mixer -- differential attention with a
window, retention, or gated linear attention -- and, optionally, a dense gated feed-forward; the residual stream is kept
in several copies that every sublayer reads and writes through small learned vectors and a matrix (hyper-connections),
and every norm is a Dynamic Tanh.

config.json keys: ``vocab``, ``width``, ``streams``, ``logit_scale``, ``norm.eps`` and ``layers``, a list of
``{"type": "attention" | "retention" | "gla", "mixer": {...sizes and constants...},
"mlp": {"kind": "dense", "ff": N, "limit": L} | null}``.  The rank of a ``gla`` mixer's decay map is the shape of its
tensors ``a1`` and ``a2``; a configuration may name it (``rank``), and one that is to be filled with random weights must.
Tensor names: ``embed``, ``head``, ``final.norm`` (with ``.b`` and ``.alpha``), and for layer i ``l<i>.norm1``,
``l<i>.norm2`` (each with ``.b`` and ``.alpha``), ``l<i>.hc1.{in,out,mix}``, ``l<i>.hc2.{in,out,mix}``, ``l<i>.mix.*``,
``l<i>.mlp.{gate,up,down}``.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List

from ..errors import ConfigError
from .base import ModelConfig, field_from_json
from .registry import Architecture, register_architecture

_MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "diff"),
    "retention": ("heads", "dim", "vdim", "decay"),
    "gla": ("heads", "dim", "vdim", "tau"),
}


def _number(where: str, d: Dict[str, Any], key: str, integer: bool = True):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (integer and int(v) != v):
        raise ConfigError(f"config.json: {where}.{key} must be {'an integer' if integer else 'a number'}, got {v!r}")
    return int(v) if integer else float(v)


def _rotation(where: str, m: Dict[str, Any]):
    """The mixer's ``rot`` object as the parameters of a rotary part, or None where it has none (or rotates nothing)."""
    rot = m.get("rot")
    if rot is None:
        return None
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where}.rot must be an object")
    dims = _number(where + ".rot", rot, "dims")
    if dims == 0:
        return None
    scaling = rot.get("scaling")
    if scaling is not None:
        if not isinstance(scaling, dict):
            raise ConfigError(f"config.json: {where}.rot.scaling must be an object")
        scaling = {k: _number(where + ".rot.scaling", scaling, k, integer=False) for k in ("factor", "original", "fast", "slow")}
    return dict(theta=_number(where + ".rot", rot, "base", integer=False), dim=dims, scaling=scaling)


@dataclasses.dataclass
class NagezenConfig(ModelConfig):
    vocab_size: int = field_from_json("vocab")
    hidden_size: int = field_from_json("width")
    layers: List[Dict[str, Any]] = field_from_json("layers")
    norm: Dict[str, Any] = field_from_json("norm")
    streams: int = field_from_json("streams", 1)
    logit_scale: float = field_from_json("logit_scale", 1.0)
    max_seq_len: int = field_from_json("max_positions", 1 << 20)     # (nothing in the design bounds a position)

    def derive(self, raw: Dict[str, Any]) -> None:
        if not isinstance(self.norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        self.norm_eps = _number("norm", self.norm, "eps", integer=False)

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or self.max_seq_len <= 0 or self.streams <= 0:
            raise ConfigError(f"config.json: vocab {self.vocab_size}, width {self.hidden_size} and streams {self.streams} must be positive")
        if self.norm_eps < 0:
            raise ConfigError(f"config.json: norm.eps {self.norm_eps} must not be negative")
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
            for k in ("heads", "dim", "vdim"):
                _number(where + ".mixer", m, k)
            _rotation(where + ".mixer", m)
            if layer["type"] == "attention":
                _number(where + ".mixer", m, "kv_heads")
                _number(where + ".mixer", m, "scale", integer=False)
                _number(where + ".mixer", m, "diff", integer=False)
                mask = m.get("mask")
                if mask is not None:
                    if not isinstance(mask, dict):
                        raise ConfigError(f"config.json: {where}.mixer.mask must be an object")
                    _number(where + ".mixer.mask", mask, "size")
                    if "keep_first" in mask:
                        _number(where + ".mixer.mask", mask, "keep_first")
            elif layer["type"] == "retention":
                decay = m["decay"]
                if not isinstance(decay, list) or len(decay) != int(m["heads"]) or any(
                        isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
                    raise ConfigError(f"config.json: {where}.mixer.decay must list one number for each of the {m['heads']} heads")
            else:
                _number(where + ".mixer", m, "tau", integer=False)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp must be null or of kind 'dense', got {mlp!r}")
                _number(where + ".mlp", mlp, "ff")
                _number(where + ".mlp", mlp, "limit", integer=False)

    def to_dict(self) -> Dict[str, Any]:
        out = super().to_dict()
        out["architecture"] = "Nagezen"
        return out


def describe_nagezen(cfg: NagezenConfig):
    """The layer stack as data: every layer a ``hyper`` block (sublayers that read and write a stream kept in copies)."""
    from ..engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

    width, eps, n_streams = cfg.hidden_size, cfg.norm_eps, cfg.streams

    def norm(prefix: str, name: str, out_scale: float = 1.0) -> "PartSpec":
        return PartSpec("dynamic_tanh", dict(size=width, out_scale=out_scale), prefix=prefix,
                        rename={"weight": name, "b": name + ".b", "alpha": name + ".alpha"})

    def connection(prefix: str) -> "PartSpec":
        return PartSpec("hyper", dict(streams=n_streams), prefix=prefix)

    layers = []
    for n, layer in enumerate(cfg.layers):
        p, m, kind = f"l{n}.", layer["mixer"], layer["type"]
        rot = _rotation(f"layers[{n}].mixer", m)
        position = PartSpec("rotary", rot) if rot is not None else None
        sizes = dict(hidden_size=width, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), eps=eps)
        if kind == "attention":
            mask = m.get("mask") or {}
            mixer = PartSpec("diff_attention", dict(sizes, kv_heads=int(m["kv_heads"]), scale=float(m["scale"]), diff=float(m["diff"]),
                                                    window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)),
                                                    position=position), prefix=p + "mix.")
        elif kind == "retention":
            mixer = PartSpec("retention", dict(sizes, decay=[float(d) for d in m["decay"]], position=position), prefix=p + "mix.")
        else:
            mixer = PartSpec("gla", dict(sizes, tau=float(m["tau"]), gate_rank=int(m["rank"]) if "rank" in m else None), prefix=p + "mix.")
        extras = {"mixer_conn": ("connection", connection(p + "hc1."))}
        ffn = ffn_norm = None
        if layer.get("mlp") is not None:
            ffn = PartSpec("clamped_glu", dict(hidden_size=width, intermediate_size=int(layer["mlp"]["ff"]),
                                               limit=float(layer["mlp"]["limit"])), prefix=p + "mlp.")
            ffn_norm = norm(p, "norm2")
            extras["ffn_conn"] = ("connection", connection(p + "hc2."))
        layers.append(LayerSpec(block="hyper", mixer=mixer, ffn=ffn, mixer_norm=norm(p, "norm1"), ffn_norm=ffn_norm, extras=extras))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=width, max_seq_len=cfg.max_seq_len,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=width), rename={"weight": "embed"}),
        layers=layers,
        schedule=[ScheduleEntry(layer=n, cache=n, writes=True) for n in range(len(layers))],
        # (the factor on the logits rides on the last norm's output: one multiplication per element of a row)
        final_norm=norm("final.", "norm", out_scale=cfg.logit_scale),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=width), rename={"weight": "head"}),
        streams=n_streams,
    )


NAGEZEN = register_architecture(Architecture(name="Nagezen", model_type="nagezen", config_class=NagezenConfig,
                                             describe=describe_nagezen))
