"""Differential attention: two softmax maps per head over the same values, their difference normed and gated."""
from __future__ import annotations

import math
from typing import Dict

import torch

from ..cache.specs import PagedHeads
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, build_part, register_part
from .linear import linear


class DifferentialAttention(Part):
    """q = Wq h + bq has heads x 2 x dim rows and k = Wk h + bk kv_heads x 2 x dim, head by head as [map 1, map 2];
    v = Wv h + bv has kv_heads x vdim.  Every map of q and k is RMS-normed over dim with a weight (``q.norm``,
    ``k.norm``: one vector for all heads and maps) and then rotated by position (``position``: a rotary part).  Each map
    is a softmax attention of its own over the keys the row sees -- key j <= p with p - j < window or j < keep_first
    (window 0: all) -- with scores (q . k) * scale; query head a reads key/value head a // (heads / kv_heads).  With
    lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer: o = a1 - lam a2, divided by
    sqrt(mean(o^2) + eps) over the head's vdim values, times (1 - diff); the heads side by side are multiplied by
    sigmoid(Wg h) and projected by Wo.  Scores, weights and sums are float32; keys and values are cached rotated."""
    category = "mixer"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, diff: float, eps: float,
                 window: int = 0, keep_first: int = 0, position=None):
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads:
            raise ConfigError(f"differential attention: {heads} heads cannot share {kv_heads} key/value heads")
        if window < 0 or keep_first < 0:
            raise ConfigError(f"differential attention: window {window} and kept first tokens {keep_first} must not be negative")
        if not (0 < dim <= ops.HEADS_MAX_DIM and 0 < vdim <= ops.HEADS_MAX_DIM):
            raise ConfigError(f"differential attention: dim {dim} and vdim {vdim} must lie in 1..{ops.HEADS_MAX_DIM}")
        self.hidden_size, self.heads, self.kv_heads = int(hidden_size), int(heads), int(kv_heads)
        self.dim, self.vdim, self.scale, self.diff, self.eps = int(dim), int(vdim), float(scale), float(diff), float(eps)
        self.window, self.keep_first = int(window), int(keep_first)
        self.position = build_part("position", position) if position is not None else None
        if self.position is not None and getattr(self.position, "dim", 0) > self.dim:
            raise ConfigError(f"differential attention: {self.position.dim} rotated elements of a map of {self.dim}")

    def children(self):
        return [self.position] if self.position is not None else []

    def cache_spec(self):
        return PagedHeads(self.kv_heads * 2, self.dim, self.kv_heads, self.vdim, self.window, self.keep_first)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        H, G, d, e, h = self.heads, self.kv_heads, self.dim, self.vdim, self.hidden_size
        vec = lambda n, init="normal": WeightSpec((n,), kind="vector", init=init)      # noqa: E731
        return {"q": WeightSpec((H * 2 * d, h)), "q.b": vec(H * 2 * d), "k": WeightSpec((G * 2 * d, h)), "k.b": vec(G * 2 * d),
                "v": WeightSpec((G * e, h)), "v.b": vec(G * e), "q.norm": vec(d, "ones"), "k.norm": vec(d, "ones"),
                "lq1": vec(d), "lk1": vec(d), "lq2": vec(d), "lk2": vec(d), "g": WeightSpec((H * e, h)), "o": WeightSpec((h, H * e))}

    def bind(self, tensors, rt) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()      # noqa: E731
        self.w_in = ops.StreamedWeight(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0).contiguous())
        self.w_o = ops.StreamedWeight(tensors["o"])
        self.q_b, self.k_b, self.v_b = f32("q.b"), f32("k.b"), f32("v.b")
        self.q_norm, self.k_norm = f32("q.norm"), f32("k.norm")
        lam = [float((f32("lq" + i).double() * f32("lk" + i).double()).sum()) for i in ("1", "2")]
        self.lam = math.exp(lam[0]) - math.exp(lam[1]) + self.diff
        self.act_dtype = rt.act_dtype

    def step_work(self, batch, rows: int, elem: int):
        """The products' work, plus attention's own: per visible key, query head and map a product of dim and one of
        vdim, and every visible key and value read once per request."""
        flops, nbytes = super().step_work(batch, rows, elem)
        pairs = keys = 0
        span = self.window + self.keep_first
        for s in range(batch.n_seqs):
            cached, new = int(batch.seq_ctx[s]), int(batch.seq_start[s + 1] - batch.seq_start[s])
            if self.window > 0:
                pairs += sum(min(span, cached + i + 1) for i in range(new))
                keys += min(cached + new, span + new - 1)
            else:
                pairs += new * cached + new * (new + 1) // 2
                keys += cached + new
        return (flops + 4.0 * pairs * self.heads * (self.dim + self.vdim),
                nbytes + keys * self.kv_heads * (2 * self.dim + self.vdim) * elem)

    def working_bytes_per_row(self, elem: int) -> float:
        return super().working_bytes_per_row(elem) + self.heads * (8 * self.dim + self.vdim * elem)

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        H, G, d, e, t = self.heads, self.kv_heads, self.dim, self.vdim, h.shape[0]
        # float32 sums: the biases are added to them and the maps normed before anything is rounded
        x = linear(h, self.w_in, out_dtype=torch.float32)
        nq, nk, nv = H * 2 * d, G * 2 * d, G * e
        q, k, v, g = x[:, :nq], x[:, nq:nq + nk], x[:, nq + nk:nq + nk + nv], x[:, nq + nk + nv:]
        table = self.position.table(ctx) if self.position is not None and hasattr(self.position, "table") else None
        q_maps = torch.empty((t, H * 2, d), dtype=torch.float32, device=x.device)
        # queries dense in float32, keys and values straight into their pages: one launch for the three
        sections = [ops.heads_section(q, H * 2, d, q_maps, bias=self.q_b, norm_weight=self.q_norm, eps=self.eps, table=table)]
        if writes:
            slots = ctx.slot_maps[cache.group]
            sections.append(ops.heads_section(k, G * 2, d, cache.k, bias=self.k_b, norm_weight=self.k_norm, eps=self.eps, table=table,
                                              slot_map=slots, page_tokens=cache.page_tokens))
            sections.append(ops.heads_section(v, G, e, cache.v, bias=self.v_b, slot_map=slots, page_tokens=cache.page_tokens))
        ops.heads_prepare_many(sections)
        o = ops.attention_maps(q_maps.view(t, H, 2, d), cache.k, cache.v, ctx.block_tables[cache.group], ctx, self.act_dtype,
                               H, G, 2, d, e, self.window, self.keep_first, self.scale, lam=self.lam, normalize=True,
                               eps=self.eps, factor=1.0 - self.diff, gate=g, act=ops.ACT_SIGMOID)
        linear(o, self.w_o, accumulate_into=residual, ctx=ctx)


register_part("mixer", "diff_attention", DifferentialAttention)
