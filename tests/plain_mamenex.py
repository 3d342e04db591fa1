"""A plain, slow implementation of the Mamenex decoder for the tests.

Whole sequences, no cache, no state carried between calls, one function for each mechanism, written from
the design's equations and sharing no code with the engine: it reads config.json with ``json`` and the
weights with the ``safetensors`` package.  Arithmetic is float64 by default, so that what the engine's
float32 path is compared with has no rounding of its own worth mentioning.

The design, in this file's notation (x: the residual stream [T, width]; a linear weight is stored
[out, in] and applied as W x):

  layer      x <- x + N1b(mixer(h + canon(h))) with h = N1(x); then, if the layer has a feed-forward,
             x <- x + N2b(ff(N2(x)))
  N(v)       v / sqrt(mean(v^2) + eps) * (1 + w)                       (the weight is stored around zero)
  canon      a causal convolution over time on each channel, taps wide, zeros before the sequence
  mixers     latent attention (a low-rank latent per token shared by all heads, one rotated key part
             shared by all heads, a sink in the softmax) and the real-gated linear recurrent unit
  ff         W_down act(W_up v) with act(z) = softplus(p) z^2 + z/2 for z > 0 and
             (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 otherwise
  output     N(x) with the model's last norm, logits = E N(x) with the embedding table E
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --- mechanisms -----------------------------------------------------------------

def offset_rmsnorm(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) * (1 + w): eps under the root, the weight counted from one."""
    ms = (v * v).mean(dim=-1, keepdim=True)
    return v / torch.sqrt(ms + eps) * (1.0 + w)


def plain_rmsnorm(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) * w: the weight as it is stored."""
    ms = (v * v).mean(dim=-1, keepdim=True)
    return v / torch.sqrt(ms + eps) * w


def causal_conv(v: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, c] = bias[c] + sum_j w[c, j] * v[t - taps + 1 + j, c]; rows before the sequence are zero.
    The last column of w is the current token's."""
    T, C = v.shape
    taps = w.shape[1]
    out = torch.zeros_like(v)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * v[src]
    if bias is not None:
        out = out + bias
    return out


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (torch.expm1(z) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def interleaved_rotation(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, ..., d]: among the first ``dims`` elements, element 2i is paired with element 2i+1;
    the pair (a, b) at position p becomes (a cos t - b sin t, b cos t + a sin t), t = p * base^(-2i/dims).
    Elements from ``dims`` on pass unchanged."""
    out = v.clone()
    T = v.shape[0]
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        ang = positions.to(v.dtype) * f
        shape = [T] + [1] * (v.dim() - 2)
        c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
        a, b = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def sink_softmax(scores: torch.Tensor, sink: float) -> torch.Tensor:
    """Weights of one row: exp(s_j) / (sum_k exp(s_k) + exp(sink)).  The sink has no key and no value."""
    m = max(float(scores.max()), float(sink))
    e = torch.exp(scores - m)
    return e / (e.sum() + math.exp(float(sink) - m))


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """h [T, width] -> [T, width].  Keys and values are made explicitly for every head (nothing is absorbed)."""
    T = h.shape[0]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ w["q"].T).view(T, H, dn + dr)
    q_plain, q_rot = q[..., :dn], interleaved_rotation(q[..., dn:], pos, m["rot"]["base"], m["rot"]["dims"])
    dkv = h @ w["dkv"].T
    latent = plain_rmsnorm(dkv[:, :rank], w["dkv.norm"], eps)
    k_rot = interleaved_rotation(dkv[:, rank:], pos, m["rot"]["base"], m["rot"]["dims"])     # one for all heads
    k_plain = (latent @ w["uk"].T).view(T, H, dn)
    val = (latent @ w["uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        for t in range(T):
            s = (k_plain[:t + 1, head] @ q_plain[t, head] + k_rot[:t + 1] @ q_rot[t, head]) * m["scale"]
            out[t, head] = sink_softmax(s, w["sink"][head]) @ val[:t + 1, head]
    return out.reshape(T, H * dv) @ w["o"].T


def rglru(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """The recurrent block: a gated branch and a recurrent one, state from zero."""
    T = h.shape[0]
    W, B = m["width"], m["blocks"]
    gate = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = causal_conv(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    ub = u.view(T, B, W // B)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", w["ra"], ub) + w["ra.b"]).reshape(T, W)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", w["ri"], ub) + w["ri.b"]).reshape(T, W)
    log_a = -8.0 * r * softplus(w["lam"])
    a = torch.exp(log_a)
    state = torch.zeros(W, dtype=h.dtype)
    out = torch.zeros(T, W, dtype=h.dtype)
    for t in range(T):
        state = a[t] * state + torch.sqrt(1.0 - a[t] * a[t]) * i[t] * u[t]
        out[t] = state
    return (out * gate) @ w["o"].T


def dense_ff(v: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return xielu(v @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


# --- the model -------------------------------------------------------------------

def _sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int], dtype=torch.float64,
            layer_outputs: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``layer_outputs`` receives the stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    for n, layer in enumerate(config["layers"]):
        p = f"l{n}."
        h = offset_rmsnorm(x, w[p + "norm1"], eps)
        h = h + causal_conv(h, w[p + "canon1"])
        if layer["type"] == "latent_attention":
            y = latent_attention(h, _sub(w, p + "mix."), layer["mixer"], eps)
        elif layer["type"] == "rglru":
            y = rglru(h, _sub(w, p + "mix."), layer["mixer"])
        else:
            raise ValueError(f"layer {n}: no mixer '{layer['type']}'")
        x = x + offset_rmsnorm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {n}: no feed-forward '{layer['mlp']['kind']}'")
            y = dense_ff(offset_rmsnorm(x, w[p + "norm2"], eps), _sub(w, p + "mlp."))
            x = x + offset_rmsnorm(y, w[p + "norm2b"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return offset_rmsnorm(x, w["final.norm"], eps) @ w["embed"].T


def load_folder(folder: str):
    """(config dictionary, tensors by name) of a model folder."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as fh:
        config = json.load(fh)
    return config, load_file(os.path.join(folder, "model.safetensors"))
