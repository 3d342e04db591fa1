"""Small Nagezen configurations and model folders for the tests.

The folders are written here with draws of the tests' own (not by the framework's random-weights mode): matrices
N(0, 1/in) so that activations stay of order one through every layer, the streams' matrices near the identity with
visible off-diagonal terms, read and write vectors, norm weights, biases and slopes spread visibly around their neutral
values, and query and key norm weights a few times larger, so that attention is peaked and a wrong key, a window one
token off or a factor at the wrong place changes the logits.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, vdim, window=None, keep_first=None, dims=None, base=10000.0, scaling=None, scale=None,
              diff=0.5, ff=None, limit=3.0):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, diff=diff, scale=scale if scale is not None else dim ** -0.5)
    if window is not None:
        mixer["mask"] = dict(size=window) if keep_first is None else dict(size=window, keep_first=keep_first)
    if dims is not None:
        mixer["rot"] = dict(base=base, dims=dims) if scaling is None else dict(base=base, dims=dims, scaling=scaling)
    return dict(type="attention", mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff, limit=limit))


def retention(heads, dim, vdim, decay, dims=None, base=10000.0, ff=None, limit=3.0):
    mixer = dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))
    if dims is not None:
        mixer["rot"] = dict(base=base, dims=dims)
    return dict(type="retention", mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff, limit=limit))


def gla(heads, dim, vdim, tau, rank, ff=None, limit=3.0):
    return dict(type="gla", mixer=dict(heads=heads, dim=dim, vdim=vdim, tau=tau, rank=rank),
                mlp=None if ff is None else dict(kind="dense", ff=ff, limit=limit))


YARN = dict(factor=8.0, original=64, fast=16.0, slow=2.0)

# Configurations that differ in every size and constant: one copy of the stream (B), two and five; one key/value head
# for all query heads, one for each, and groups; key and value sizes that are no multiple of four, larger than a wave
# (70, 130) and on both sides of the scan's register buckets (5, 40, 72, 130); rotation of a whole head, of a part of it,
# of none; scaled frequencies and plain ones; windows of 9 to 50 tokens with and without kept first tokens, more kept
# tokens than the window is wide, no window at all; layers with and without a feed-forward; a factor on the logits and none.
CONFIGS: Dict[str, dict] = {
    "A": dict(architecture="Nagezen", vocab=96, width=48, streams=2, logit_scale=1.5, norm=dict(eps=1e-5), layers=[
        retention(3, 8, 12, [0.9, 0.97, 0.995], dims=4, base=100.0, ff=80, limit=1.0),
        attention(4, 2, 12, 20, window=9, keep_first=3, dims=8, base=500.0, scaling=YARN, scale=0.5, diff=0.3, ff=56),
        gla(2, 16, 10, tau=4.0, rank=6),
        attention(3, 3, 10, 6, window=11, keep_first=0, dims=10, base=50.0, diff=0.7, ff=40, limit=0.7)]),
    "B": dict(architecture="Nagezen", vocab=131, width=64, streams=1, logit_scale=1.0, norm=dict(eps=1e-6), layers=[
        gla(5, 5, 70, tau=9.0, rank=3, ff=96),
        attention(6, 1, 24, 130, window=50, keep_first=7, dims=24, scale=0.3, diff=0.55),
        retention(2, 40, 24, [0.5, 0.999], ff=72, limit=5.0)]),
    "C": dict(architecture="Nagezen", vocab=77, width=42, streams=5, logit_scale=0.25, norm=dict(eps=1e-3), layers=[
        attention(2, 2, 6, 9, dims=2, base=30.0, diff=0.1, ff=44),                                   # no window: every key
        retention(1, 72, 7, [0.98], dims=72, base=1000.0),
        attention(5, 1, 7, 5, window=6, keep_first=10, dims=6, scaling=dict(factor=2.0, original=16, fast=4.0, slow=1.0), diff=0.8),
        gla(1, 130, 33, tau=32.0, rank=8, ff=30, limit=0.5)]),
    "D": dict(architecture="Nagezen", vocab=64, width=32, streams=3, logit_scale=3.0, norm=dict(eps=1e-5), layers=[
        gla(4, 8, 8, tau=1.0, rank=4), retention(4, 8, 8, [1.0, 0.0, 0.75, 0.9375], dims=8, ff=48)]),   # nothing kept per token
    "E": dict(architecture="Nagezen", vocab=64, width=32, streams=4, logit_scale=1.0, norm=dict(eps=1e-5), layers=[
        attention(2, 1, 16, 16, window=17, keep_first=1, dims=16, ff=48),
        attention(8, 4, 4, 3, window=33, keep_first=16, dims=2, base=7.0, scale=1.1, diff=0.45)]),    # no state slots
}
SEEDS = {"A": 12, "B": 23, "C": 34, "D": 45, "E": 56}


def tensors_for(config: dict, seed: int, query_factor: float = 2.5) -> Dict[str, torch.Tensor]:
    gen = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=gen) * std + mean

    def matrix(out, inn, factor=1.0):
        return normal(out, inn, std=factor / math.sqrt(inn))
    W, n = config["width"], config["streams"]
    t = {"embed": normal(config["vocab"], W), "head": matrix(config["vocab"], W)}

    def norm(name):
        t[name], t[name + ".b"], t[name + ".alpha"] = normal(W, std=0.2, mean=1.0), normal(W, std=0.1), normal(1, std=0.1, mean=0.7).reshape(())

    def connection(name):
        t[name + ".in"] = normal(n, std=0.15, mean=1.0 / n)
        t[name + ".out"] = normal(n, std=0.2, mean=1.0)
        t[name + ".mix"] = torch.eye(n) * 0.9 + normal(n, n, std=0.1)
    norm("final.norm")
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norm(p + "norm1")
        connection(p + "hc1")
        H, d, e = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            t[p + "mix.q"], t[p + "mix.q.b"] = matrix(H * 2 * d, W), normal(H * 2 * d, std=0.3)
            t[p + "mix.k"], t[p + "mix.k.b"] = matrix(G * 2 * d, W), normal(G * 2 * d, std=0.3)
            t[p + "mix.v"], t[p + "mix.v.b"] = matrix(G * e, W), normal(G * e, std=0.3)
            t[p + "mix.q.norm"] = normal(d, std=0.2, mean=1.0) * query_factor
            t[p + "mix.k.norm"] = normal(d, std=0.2, mean=1.0)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                t[p + "mix." + name] = normal(d, std=0.8 / math.sqrt(d))
        else:
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = matrix(H * d, W), matrix(H * d, W), matrix(H * e, W)
            if layer["type"] == "gla":
                r = m["rank"]
                t[p + "mix.a1"], t[p + "mix.a2"] = matrix(r, W), matrix(H * d, r, 2.0)
                t[p + "mix.a2.b"] = normal(H * d, std=2.0, mean=2.0)              # decays from near 0 to near 1
                t[p + "mix.norm"] = normal(e, std=0.2, mean=1.0)
        t[p + "mix.g"], t[p + "mix.o"] = matrix(H * e, W), matrix(W, H * e)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            norm(p + "norm2")
            connection(p + "hc2")
            t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = matrix(ff, W, 1.5), matrix(ff, W, 1.5), matrix(W, ff)
    return t


def write_folder(root, name: str, dtype: str, config: Optional[dict] = None, seed: Optional[int] = None, tag: str = "",
                 drop_rank: bool = False, **draw) -> str:
    """config.json and model.safetensors of configuration ``name`` (or of ``config``) under ``root``.  ``drop_rank``:
    the written config.json does not name the rank of a gla mixer's decay map (its tensors' shapes do)."""
    from safetensors.torch import save_file
    config = config or CONFIGS[name]
    out = os.path.join(str(root), f"nagezen_{name}_{dtype}{tag}")
    if not os.path.exists(os.path.join(out, "model.safetensors")):
        os.makedirs(out, exist_ok=True)
        written = json.loads(json.dumps(config))
        if drop_rank:
            for layer in written["layers"]:
                layer["mixer"].pop("rank", None)
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as fh:
            json.dump(written, fh)
        store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        tensors = tensors_for(config, SEEDS.get(name, 1) if seed is None else seed, **draw)
        save_file({k: v.to(store).contiguous() for k, v in tensors.items()}, os.path.join(out, "model.safetensors"))
    return out
