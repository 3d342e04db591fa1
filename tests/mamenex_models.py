"""Small Mamenex configurations and model folders for the tests.

The folders are written here with draws of the tests' own (not by the framework's random-weights mode): matrices
N(0, 1/in) so that activations stay of order one through every layer, norm weights, biases and sinks spread
visibly around their neutral values, and query weights a few times larger, so that attention is peaked and a
wrong key, a missing sink or a scale at the wrong norm changes the logits.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import torch


def latent(heads, dim, rot_dim, vdim, kv_rank, dims, base=10000.0, scale=None, ff=None):
    mixer = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
                 scale=scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim), rot=dict(base=base, dims=dims))
    return dict(type="latent_attention", mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff))


def recurrent(width, blocks, conv, ff=None):
    return dict(type="rglru", mixer=dict(width=width, blocks=blocks, conv=conv),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


# Configurations that differ in every size and constant: rotated dimensions fewer than the rotated part (P) or all
# of it, one head (P) and several, one gate block (P, R) and several, convolutions of one tap (P: the recurrent
# layer's; R: the one in front of the mixers), a latent row longer than a wave (Q: 72 + 24, R: 130 + 6, no multiple
# of four), layers with and without a feed-forward after either mixer, an odd vocabulary; S has latent rows of whole
# matrix-core steps (48 + 16, 112 + 16) with four heads and with twenty (more than a tile's sixteen columns).
CONFIGS: Dict[str, dict] = {
    "P": dict(architecture="Mamenex", vocab=96, width=48, norm=dict(eps=1e-6), canon=dict(taps=2), layers=[
        recurrent(40, 5, 3, ff=80),
        latent(3, 8, 12, 10, 20, dims=8, base=100.0),
        latent(1, 16, 4, 6, 24, dims=4, scale=0.17, ff=64),
        recurrent(24, 1, 1)]),
    "Q": dict(architecture="Mamenex", vocab=131, width=64, norm=dict(eps=1e-5), canon=dict(taps=4), layers=[
        latent(5, 4, 8, 16, 72, dims=8, base=500.0, scale=0.4, ff=96),
        recurrent(64, 2, 4),
        latent(2, 24, 24, 8, 72, dims=24, ff=40)]),
    "R": dict(architecture="Mamenex", vocab=77, width=40, norm=dict(eps=1e-3), canon=dict(taps=1), layers=[
        recurrent(36, 1, 2, ff=44),
        latent(2, 10, 6, 12, 130, dims=2, base=50.0)]),
    "S": dict(architecture="Mamenex", vocab=200, width=64, norm=dict(eps=1e-5), canon=dict(taps=3), layers=[
        latent(4, 16, 16, 16, 48, dims=16, ff=64),
        recurrent(64, 4, 4),
        latent(20, 8, 16, 8, 112, dims=8, base=1000.0)]),
    "T": dict(architecture="Mamenex", vocab=64, width=32, norm=dict(eps=1e-5), canon=dict(taps=2), layers=[
        recurrent(32, 2, 3), recurrent(48, 3, 2, ff=40)]),                         # no attention: nothing is kept per token
    "U": dict(architecture="Mamenex", vocab=64, width=32, norm=dict(eps=1e-5), canon=dict(taps=5), layers=[
        latent(2, 8, 8, 8, 24, dims=8), latent(6, 4, 2, 4, 10, dims=2, ff=48)]),    # no recurrence
    "V": dict(architecture="Mamenex", vocab=53, width=50, norm=dict(eps=1e-4), canon=dict(taps=6), layers=[
        latent(3, 5, 6, 7, 9, dims=4, base=30.0, ff=35),                            # nothing a multiple of four
        recurrent(30, 3, 7, ff=22),
        latent(7, 3, 2, 5, 11, dims=2)]),
}
SEEDS = {"P": 11, "Q": 22, "R": 33, "S": 44, "T": 55, "U": 66, "V": 77}


def tensors_for(config: dict, seed: int, query_factor: float = 3.0, sink_mean: float = 0.0) -> Dict[str, torch.Tensor]:
    gen = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=gen) * std + mean

    def matrix(out, inn, factor=1.0):
        return normal(out, inn, std=factor / math.sqrt(inn))
    W = config["width"]
    t = {"embed": normal(config["vocab"], W), "final.norm": normal(W, std=0.2)}
    for n, layer in enumerate(config["layers"]):
        p, m = f"l{n}.", layer["mixer"]
        t[p + "norm1"], t[p + "norm1b"] = normal(W, std=0.2), normal(W, std=0.2)
        t[p + "canon1"] = normal(W, config["canon"]["taps"], std=0.4)
        if layer["type"] == "latent_attention":
            H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            t[p + "mix.q"] = matrix(H * (dn + dr), W, query_factor)
            t[p + "mix.dkv"] = matrix(r + dr, W)
            t[p + "mix.dkv.norm"] = normal(r, std=0.2, mean=1.0)
            t[p + "mix.uk"] = matrix(H * dn, r, query_factor)
            t[p + "mix.uv"] = matrix(H * dv, r)
            t[p + "mix.sink"] = normal(H, mean=sink_mean)
            t[p + "mix.o"] = matrix(W, H * dv)
        else:
            w, B = m["width"], m["blocks"]
            bs = w // B
            t[p + "mix.y"], t[p + "mix.y.b"] = matrix(w, W), normal(w, std=0.3)
            t[p + "mix.x"], t[p + "mix.x.b"] = matrix(w, W), normal(w, std=0.3)
            t[p + "mix.conv"], t[p + "mix.conv.b"] = normal(w, m["conv"], std=0.5), normal(w, std=0.3)
            t[p + "mix.ra"], t[p + "mix.ra.b"] = normal(B, bs, bs, std=1.0 / math.sqrt(bs)), normal(B, bs, std=0.5)
            t[p + "mix.ri"], t[p + "mix.ri.b"] = normal(B, bs, bs, std=1.0 / math.sqrt(bs)), normal(B, bs, std=0.5)
            t[p + "mix.lam"] = normal(w, std=1.0, mean=-1.0)
            t[p + "mix.o"] = matrix(W, w)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            t[p + "norm2"], t[p + "norm2b"] = normal(W, std=0.2), normal(W, std=0.2)
            t[p + "mlp.up"], t[p + "mlp.down"] = matrix(ff, W), matrix(W, ff)
            t[p + "mlp.act"] = normal(2, std=0.7)
    return t


def write_folder(root, name: str, dtype: str, config: Optional[dict] = None, seed: Optional[int] = None, tag: str = "",
                 **draw) -> str:
    """config.json and model.safetensors of configuration ``name`` (or of ``config``) under ``root``."""
    from safetensors.torch import save_file
    config = config or CONFIGS[name]
    out = os.path.join(str(root), f"mamenex_{name}_{dtype}{tag}")
    if not os.path.exists(os.path.join(out, "model.safetensors")):
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as fh:
            json.dump(config, fh)
        store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        tensors = tensors_for(config, SEEDS.get(name, 1) if seed is None else seed, **draw)
        save_file({k: v.to(store).contiguous() for k, v in tensors.items()}, os.path.join(out, "model.safetensors"))
    return out
