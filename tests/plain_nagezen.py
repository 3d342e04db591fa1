"""A plain, slow implementation of the Nagezen decoder for the tests.

Whole sequences, no cache, no state carried between calls, one function for each mechanism, written from the
design's equations and sharing no code with the engine: it reads config.json with ``json`` and the weights with
the ``safetensors`` package.  Arithmetic is float64 by default, so that what the engine's float32 path is compared
with has no rounding of its own worth mentioning.

The design, in this file's notation (a linear weight is stored [out, in] and applied as W x):

  streams    n copies X[0..n-1] of the residual stream, all the embedding at the start.  A sublayer f with its
             vectors r (read), w (write) and its matrix M [from, to]:
                 u = sum_s r[s] X[s];  y = f(N(u));  X'[t] = sum_s M[s, t] X[s] + w[t] y   (all t from the old X)
             The model's output norm reads sum_s X[s].
  N(v)       tanh(a v) * g + b with one number a, vectors g and b: no mean, no variance
  mixers     ``attention``  two softmax maps per head over the same values, their difference normed and gated;
                            a window of the last keys plus the first few keys of the sequence
             ``retention``  S_t = c_h S_(t-1) + k_t v_t^T per head with a constant c_h, o_t = S_t^T q_t
             ``gla``        S_t = diag(a_t) S_(t-1) + k_t v_t^T with a decay per key channel made from the input
  ff         W_down (g sigmoid(1.702 g) (u + 1)) with g = min(W_gate v, L), u = clamp(W_up v, -L, L)
  output     logits = c * W_head N(sum_s X[s])
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --- mechanisms -----------------------------------------------------------------

def dynamic_tanh(v: torch.Tensor, a: torch.Tensor, g: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """tanh(a v) * g + b."""
    return torch.tanh(a * v) * g + b


def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last axis: eps under the root, no weight."""
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def half_rotation_angles(positions: torch.Tensor, dims: int, base: float, scaling: Optional[dict] = None):
    """(cos, sin) [T, dims/2] of the rotation of pair i (element i with element i + dims/2):
    angle = p * f_i, f_i = base^(-2i/dims).  With ``scaling`` (factor F, original L, fast, slow) the
    frequencies of the slow pairs are divided by F: with e(t) = dims ln(L / (2 pi t)) / (2 ln base),
    lo = max(floor(e(fast)), 0), hi = min(ceil(e(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    the frequency is f_i / F * r_i + f_i (1 - r_i), and cos and sin are multiplied by 0.1 ln F + 1."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    amp = 1.0
    if scaling is not None:
        F, L = float(scaling["factor"]), float(scaling["original"])
        e = lambda t: dims * math.log(L / (2.0 * math.pi * t)) / (2.0 * math.log(base))      # noqa: E731
        lo = max(math.floor(e(float(scaling["fast"]))), 0)
        hi = min(math.ceil(e(float(scaling["slow"]))), dims - 1)
        r = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / F * r + f * (1.0 - r)
        amp = 0.1 * math.log(F) + 1.0
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    return torch.cos(ang) * amp, torch.sin(ang) * amp


def half_rotation(v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """v [T, ..., d]: among the first 2 * cos.shape[1] elements, element i is paired with element i + half;
    the pair (a, b) becomes (a cos - b sin, b cos + a sin).  The other elements pass unchanged."""
    half = cos.shape[1]
    if half == 0:
        return v.clone()
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = cos.reshape(shape).to(v.dtype), sin.reshape(shape).to(v.dtype)
    a, b = v[..., :half], v[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., 2 * half:]], dim=-1)


def visible(i: int, j: int, window: int, keep_first: int) -> bool:
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    if window <= 0:
        return True
    return i - j < window or j < keep_first


def two_map_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int, keep_first: int,
                      lam: float, diff: float, eps: float) -> torch.Tensor:
    """q [T, H, 2, d], k [T, G, 2, d], v [T, G, e] -> [T, H, e].  Per head and map a softmax over the visible keys;
    o = a1 - lam * a2, divided by its root mean square over e, times (1 - diff)."""
    T, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        maps = []
        for m in range(2):
            s = (q[:, h, m] @ k[:, g, m].T) * scale
            mask = torch.tensor([[visible(i, j, window, keep_first) for j in range(T)] for i in range(T)])
            s = s.masked_fill(~mask, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        out[:, h] = unit_rms(maps[0] - lam * maps[1], eps) * (1.0 - diff)
    return out


def decayed_outer_products(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """One head: q, k [T, d], v [T, e], decay [T, d] (a row per token, a number per key channel).
    S_t = diag(decay_t) S_(t-1) + k_t v_t^T from S = 0; o_t = S_t^T q_t."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for t in range(T):
        S = decay[t][:, None] * S + k[t][:, None] * v[t][None, :]
        out[t] = S.T @ q[t]
    return out


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def clamped_glu(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


# --- the model --------------------------------------------------------------------

class PlainNagezen:
    def __init__(self, folder: str, dtype: torch.dtype = torch.float64):
        from safetensors import safe_open
        with open(os.path.join(folder, "config.json")) as fh:
            self.cfg = json.load(fh)
        self.w: Dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                self.w[name] = f.get_tensor(name).to(dtype)
        self.dtype = dtype
        self.eps = float(self.cfg["norm"]["eps"])

    def lin(self, name: str, x: torch.Tensor, bias: bool = False) -> torch.Tensor:
        y = x @ self.w[name].T
        return y + self.w[name + ".b"] if bias else y

    def norm(self, name: str, x: torch.Tensor) -> torch.Tensor:
        return dynamic_tanh(x, self.w[name + ".alpha"], self.w[name], self.w[name + ".b"])

    def attention(self, p: str, m: dict, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        T, H, G, d, e = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = self.lin(p + "q", h, bias=True).view(T, H, 2, d)
        k = self.lin(p + "k", h, bias=True).view(T, G, 2, d)
        v = self.lin(p + "v", h, bias=True).view(T, G, e)
        q = unit_rms(q, self.eps) * self.w[p + "q.norm"]
        k = unit_rms(k, self.eps) * self.w[p + "k.norm"]
        rot = m.get("rot")
        if rot is not None and rot.get("dims", 0) > 0:
            cos, sin = half_rotation_angles(positions, rot["dims"], rot["base"], rot.get("scaling"))
            q, k = half_rotation(q, cos, sin), half_rotation(k, cos, sin)
        w = self.w
        lam = (math.exp(float((w[p + "lq1"] * w[p + "lk1"]).sum())) - math.exp(float((w[p + "lq2"] * w[p + "lk2"]).sum()))
               + float(m["diff"]))
        mask = m.get("mask") or {}
        o = two_map_attention(q, k, v, float(m["scale"]), int(mask.get("size", 0)), int(mask.get("keep_first", 0)), lam,
                              float(m["diff"]), self.eps)
        o = o.reshape(T, H * e) * torch.sigmoid(self.lin(p + "g", h))
        return self.lin(p + "o", o)

    def retention(self, p: str, m: dict, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        T, H, d, e = h.shape[0], m["heads"], m["dim"], m["vdim"]
        q, k, v = self.lin(p + "q", h).view(T, H, d), self.lin(p + "k", h).view(T, H, d), self.lin(p + "v", h).view(T, H, e)
        rot = m.get("rot")
        if rot is not None and rot.get("dims", 0) > 0:
            cos, sin = half_rotation_angles(positions, rot["dims"], rot["base"], rot.get("scaling"))
            q, k = half_rotation(q, cos, sin), half_rotation(k, cos, sin)
        k = k * d ** -0.5
        o = torch.zeros(T, H, e, dtype=h.dtype)
        for a in range(H):
            decay = torch.full((T, d), float(m["decay"][a]), dtype=h.dtype)
            o[:, a] = unit_rms(decayed_outer_products(q[:, a], k[:, a], v[:, a], decay), self.eps)
        return self.lin(p + "o", o.reshape(T, H * e) * silu(self.lin(p + "g", h)))

    def gla(self, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
        T, H, d, e = h.shape[0], m["heads"], m["dim"], m["vdim"]
        q = (self.lin(p + "q", h) * d ** -0.5).view(T, H, d)
        k, v = self.lin(p + "k", h).view(T, H, d), self.lin(p + "v", h).view(T, H, e)
        z = self.lin(p + "a2", self.lin(p + "a1", h), bias=True)
        decay = (torch.sigmoid(z) ** (1.0 / float(m["tau"]))).view(T, H, d)
        o = torch.zeros(T, H, e, dtype=h.dtype)
        for a in range(H):
            o[:, a] = unit_rms(decayed_outer_products(q[:, a], k[:, a], v[:, a], decay[:, a]), self.eps) * self.w[p + "norm"]
        return self.lin(p + "o", o.reshape(T, H * e) * silu(self.lin(p + "g", h)))

    def feed_forward(self, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
        return self.lin(p + "down", clamped_glu(self.lin(p + "gate", h), self.lin(p + "up", h), float(m["limit"])))

    def sublayer(self, X: torch.Tensor, hc: str, norm: str, f) -> torch.Tensor:
        """X [n, T, width] -> the streams after the sublayer."""
        r, wv, M = self.w[hc + ".in"], self.w[hc + ".out"], self.w[hc + ".mix"]
        u = torch.einsum("s,std->td", r, X)
        y = f(self.norm(norm, u))
        return torch.einsum("st,snd->tnd", M, X) + wv[:, None, None] * y[None]

    def forward(self, tokens: Sequence[int], return_layers: bool = False):
        """float logits [T, vocab] of a whole sequence from position 0 (and the sum of the streams after every layer)."""
        cfg = self.cfg
        ids = torch.as_tensor(list(tokens), dtype=torch.long)
        positions = torch.arange(len(ids))
        x = self.w["embed"][ids]
        X = x[None].repeat(int(cfg["streams"]), 1, 1)
        after: List[torch.Tensor] = []
        for n, layer in enumerate(cfg["layers"]):
            p, m = f"l{n}.", layer["mixer"]
            if layer["type"] == "attention":
                mixer = lambda h: self.attention(p + "mix.", m, h, positions)      # noqa: E731
            elif layer["type"] == "retention":
                mixer = lambda h: self.retention(p + "mix.", m, h, positions)      # noqa: E731
            elif layer["type"] == "gla":
                mixer = lambda h: self.gla(p + "mix.", m, h)                        # noqa: E731
            else:
                raise ValueError(f"layer {n}: unknown type {layer['type']!r}")
            X = self.sublayer(X, p + "hc1", p + "norm1", mixer)
            if layer.get("mlp") is not None:
                X = self.sublayer(X, p + "hc2", p + "norm2", lambda h: self.feed_forward(p + "mlp.", layer["mlp"], h))
            after.append(X.sum(dim=0))
        logits = self.lin("head", self.norm("final.norm", X.sum(dim=0))) * float(cfg["logit_scale"])
        return (logits, after) if return_layers else logits
