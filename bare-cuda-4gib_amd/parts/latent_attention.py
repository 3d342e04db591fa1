"""Attention over a low-rank latent that all heads share, with a sink in the softmax."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.specs import PagedLatent
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear


class LatentAttention(Part):
    """Every token keeps a latent c = rmsnorm(Wdkv h [:rank]) * g and one rotated key part kr = rotate(Wdkv h [rank:])
    for all heads; head a's key is [Wuk_a c | kr], its value Wuv_a c, its query [q_plain | rotate(q_rot)] of
    q = Wq h.  Scores (q . k) * scale over the keys at or before the row's position (within ``window`` if not 0); the
    softmax's denominator also holds exp(sink_a) (``sink``: a learned number per head without key or value).
    Rotation: elements 2i and 2i+1 of the first ``rot_dims`` of a rotated part turn by position * base^(-2i/rot_dims).

    Only c and kr are cached (cache.specs.PagedLatent).  The keys' up-projection is absorbed into the query
    (Wuk_a^T q_plain scores against c directly) and the values' up-projection is applied to the weighted sum of the
    latents, so no key or value is ever made per head and token; scores, weights and the sums are float32."""
    category = "mixer"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float,
                 rot_dims: int, rot_base: float, eps: float, sink: bool = True, window: int = 0):
        for name, v in (("heads", heads), ("dim", dim), ("vdim", vdim), ("kv_rank", kv_rank), ("hidden_size", hidden_size)):
            if int(v) <= 0:
                raise ConfigError(f"latent attention: {name} must be positive, got {v}")
        if rot_dim < 0 or rot_dims < 0 or rot_dims % 2 or rot_dims > rot_dim:
            raise ConfigError(f"latent attention: {rot_dims} rotated dimensions (even) of a rotated part of {rot_dim}")
        if rot_base <= 0 or window < 0:
            raise ConfigError(f"latent attention: rotation base {rot_base}, window {window}")
        if kv_rank + rot_dim > ops.LATENT_MAX_ROW:
            raise ConfigError(f"latent attention: kv_rank + rot_dim = {kv_rank + rot_dim} is beyond the kernel's {ops.LATENT_MAX_ROW}")
        self.hidden_size, self.heads, self.dim, self.rot_dim = int(hidden_size), int(heads), int(dim), int(rot_dim)
        self.vdim, self.kv_rank, self.scale, self.rot_dims = int(vdim), int(kv_rank), float(scale), int(rot_dims)
        self.rot_base, self.eps, self.sink, self.window = float(rot_base), float(eps), bool(sink), int(window)

    def cache_spec(self):
        return PagedLatent(self.kv_rank, self.rot_dim, self.window)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        H, w = self.heads, self.hidden_size
        out = {"q": WeightSpec((H * (self.dim + self.rot_dim), w)), "dkv": WeightSpec((self.kv_rank + self.rot_dim, w)),
               "dkv.norm": WeightSpec((self.kv_rank,), kind="vector", init="ones"),
               "uk": WeightSpec((H * self.dim, self.kv_rank)), "uv": WeightSpec((H * self.vdim, self.kv_rank)),
               "o": WeightSpec((w, H * self.vdim))}
        if self.sink:
            out["sink"] = WeightSpec((H,), kind="vector")
        return out

    def bind(self, tensors, rt) -> None:
        H = self.heads
        # one product for the queries and the latent: their rows one after the other
        self.w_qd = ops.StreamedWeight(torch.cat([tensors["q"], tensors["dkv"]], dim=0).contiguous())
        self.w_o = ops.StreamedWeight(tensors["o"])
        self.g = tensors["dkv.norm"].to(torch.float32).contiguous()
        # [heads, rank, dim]: the keys' up-projection as it is applied to the query
        self.uk_t = tensors["uk"].view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.uv = tensors["uv"].view(H, self.vdim, self.kv_rank).contiguous()
        self.sinks = tensors["sink"].to(torch.float32).contiguous() if self.sink else None
        self.act_dtype = rt.act_dtype

    def step_work(self, batch, rows: int, elem: int):
        flops, nbytes = super().step_work(batch, rows, elem)
        f, b = ops.attention_latent_work(batch, self.heads, self.kv_rank, self.rot_dim, self.window, elem)
        return flops + f, nbytes + b

    def working_bytes_per_row(self, elem: int) -> float:
        """The products' outputs, and in float32 the absorbed queries and the weighted sums of the latents."""
        return (super().working_bytes_per_row(elem) + 4 * self.heads * (2 * self.kv_rank + self.rot_dim)
                + self.heads * self.vdim * elem)

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        H, rank, rot, t = self.heads, self.kv_rank, self.rot_dim, h.shape[0]
        n_q = H * (self.dim + rot)
        qd = linear(h, self.w_qd, out_dtype=self.act_dtype)
        q, dkv = qd[:, :n_q], qd[:, n_q:]
        q_lat = torch.empty((t, H, rank + rot), dtype=torch.float32, device=q.device)
        angles = None
        if self.rot_dims:                 # the same in every layer that rotates alike: a table made once a step
            angles = ctx.shared(("latent_angles", self.rot_dims, self.rot_base),
                                lambda: ops.latent_angles(ctx.positions, self.rot_dims, self.rot_base))
        ops.latent_prepare(q, dkv, self.g, self.eps, angles, ctx.slot_maps[cache.group] if writes else None,
                           cache.latent if writes else None, q_lat, H, self.dim, rot, rank, self.rot_dims)
        ops.heads_gemm(q.unflatten(1, (H, self.dim + rot)), self.uk_t, q_lat, k=self.dim, n=rank)
        mixed = ops.attention_latent(q_lat, cache.latent, self.sinks, ctx.block_tables[cache.group], ctx, H, rank, rot,
                                     cache.page_tokens, self.window, self.scale)
        o = torch.empty((t, H, self.vdim), dtype=self.act_dtype, device=q.device)
        ops.heads_gemm(mixed, self.uv, o, k=rank, n=self.vdim)
        linear(o.view(t, H * self.vdim), self.w_o, accumulate_into=residual, ctx=ctx)


register_part("mixer", "latent_attention", LatentAttention)
