"""Linear attention with a decayed matrix state per head: retention (a constant decay per head, rotated queries and
keys) and gated linear attention (a decay per key channel and token, made from the input)."""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..cache.specs import FixedState
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, build_part, register_part
from .linear import linear


class _DecayedState(Part):
    """What both kinds share: per head a float32 state S [dim, vdim] per request (zero at admission),
    S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t -- no softmax and no denominator --, each head's o divided by its
    root mean square, the heads side by side multiplied by silu(Wg h) and projected by Wo.  Queries, keys, values and the
    gate are one product; everything that enters the recurrence after the projections is float32."""
    category = "mixer"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh
    step_signature = ("decay_scan",)      # every such mixer cuts a step's requests into the same chunks

    def _sizes(self, hidden_size: int, heads: int, dim: int, vdim: int, what: str) -> None:
        for name, v in (("hidden_size", hidden_size), ("heads", heads), ("dim", dim), ("vdim", vdim)):
            if int(v) <= 0:
                raise ConfigError(f"{what}: {name} must be positive, got {v}")
        if dim > ops.HEADS_MAX_DIM or vdim > ops.HEADS_MAX_DIM:
            raise ConfigError(f"{what}: heads of {dim} key channels and {vdim} values; the kernels take {ops.HEADS_MAX_DIM} of each")
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(heads), int(dim), int(vdim)

    def cache_spec(self):
        return FixedState((self.heads, self.dim, self.vdim), "float32")

    def prepare_step(self, batch):
        """Where every request's chunks of rows lie among all chunks of the step (for the scan's scratch memory)."""
        base, total = ops.decay_scan_chunks(batch)
        return {"chunk_base": base}, total

    def _chunks(self, ctx):
        arrays, total = ctx.step_data.get(self.step_signature, ({}, 0))
        return arrays.get("chunk_base"), int(total or 0)

    def step_work(self, batch, rows: int, elem: int):
        """The products' work, the state read and written once per request and head, and per row and head the update of
        the state and its product with the query."""
        flops, nbytes = super().step_work(batch, rows, elem)
        per_state = self.heads * self.dim * self.vdim
        return flops + 4.0 * rows * per_state, nbytes + 8.0 * batch.n_seqs * per_state

    def working_bytes_per_row(self, elem: int) -> float:
        return (super().working_bytes_per_row(elem) + self.heads * (8 * self.dim + 4 * self.vdim + elem * self.vdim)
                + 4.0 * self.heads * self.dim * (self.vdim + 1) / ops.DECAY_SCAN_CHUNK)


class Retention(_DecayedState):
    """q = Wq h, k = Wk h (heads x dim), v = Wv h (heads x vdim); q and k rotated by position (``position``: a rotary
    part; pairs i and i + dims/2 of the first dims elements of a head), k then multiplied by dim^(-1/2); the decay of
    head a is the constant ``decay[a]``; the head's output is divided by sqrt(mean(o^2) + eps), no weight."""

    def __init__(self, hidden_size: int, heads: int, dim: int, vdim: int, decay: Sequence[float], eps: float, position=None):
        self._sizes(hidden_size, heads, dim, vdim, "retention")
        if len(decay) != self.heads or any(not (0.0 <= float(d) <= 1.0) for d in decay):
            raise ConfigError(f"retention: {self.heads} heads need as many decays in [0, 1], got {list(decay)!r}")
        self.decay, self.eps = tuple(float(d) for d in decay), float(eps)
        self.position = build_part("position", position) if position is not None else None
        if self.position is not None and getattr(self.position, "dim", 0) > self.dim:
            raise ConfigError(f"retention: {self.position.dim} rotated elements of a head of {self.dim}")

    def children(self):
        return [self.position] if self.position is not None else []

    def weight_specs(self) -> Dict[str, WeightSpec]:
        qk, v, h = self.heads * self.dim, self.heads * self.vdim, self.hidden_size
        return {"q": WeightSpec((qk, h)), "k": WeightSpec((qk, h)), "v": WeightSpec((v, h)), "g": WeightSpec((v, h)),
                "o": WeightSpec((h, v))}

    def bind(self, tensors, rt) -> None:
        self.w_in = ops.StreamedWeight(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0).contiguous())
        self.w_o = ops.StreamedWeight(tensors["o"])
        self.head_decay = torch.tensor(self.decay, dtype=torch.float32, device=tensors["q"].device)
        self.act_dtype = rt.act_dtype

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        H, d, e, t = self.heads, self.dim, self.vdim, h.shape[0]
        x = linear(h, self.w_in, out_dtype=self.act_dtype)
        q, k, v, g = x[:, :H * d], x[:, H * d:2 * H * d], x[:, 2 * H * d:2 * H * d + H * e], x[:, 2 * H * d + H * e:]
        table = self.position.table(ctx) if self.position is not None and hasattr(self.position, "table") else None
        qk = torch.empty((2, t, H, d), dtype=torch.float32, device=x.device)
        ops.heads_prepare_many([ops.heads_section(q, H, d, qk[0], table=table),
                                ops.heads_section(k, H, d, qk[1], table=table, factor=d ** -0.5)])
        base, n_chunks = self._chunks(ctx)
        o = ops.decay_scan(qk[0].view(t, H * d), qk[1].view(t, H * d), v, cache.state, ctx, H, d, e, head_decay=self.head_decay,
                           chunk_base=base, n_chunks=n_chunks)
        linear(ops.heads_finish(o, self.act_dtype, eps=self.eps, gate=g, act=ops.ACT_SILU), self.w_o, accumulate_into=residual, ctx=ctx)


class GatedLinearAttention(_DecayedState):
    """q = Wq h dim^(-1/2), k = Wk h (heads x dim), v = Wv h (heads x vdim); the decay of key channel c at a token is
    sigmoid(z_c)^(1/tau) with z = Wa2 (Wa1 h) + a2.b (heads x dim), a low-rank map of the input; the head's output is
    RMS-normed with the weight ``norm`` [vdim] that all heads share."""

    def __init__(self, hidden_size: int, heads: int, dim: int, vdim: int, tau: float, eps: float, gate_rank: Optional[int] = None):
        self._sizes(hidden_size, heads, dim, vdim, "gated linear attention")
        if float(tau) <= 0 or (gate_rank is not None and int(gate_rank) <= 0):
            raise ConfigError(f"gated linear attention: tau {tau} and the decay's rank {gate_rank} must be positive")
        # (the rank of the decay's map is the tensors' to say where the configuration does not: known once they are bound)
        self.tau, self.eps, self.gate_rank = float(tau), float(eps), int(gate_rank) if gate_rank is not None else None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        qk, v, h = self.heads * self.dim, self.heads * self.vdim, self.hidden_size
        r = self.gate_rank if self.gate_rank is not None else -1
        return {"q": WeightSpec((qk, h)), "k": WeightSpec((qk, h)), "v": WeightSpec((v, h)), "g": WeightSpec((v, h)),
                "a1": WeightSpec((r, h)), "a2": WeightSpec((qk, r)), "a2.b": WeightSpec((qk,), kind="vector"),
                "norm": WeightSpec((self.vdim,), kind="vector", init="ones"), "o": WeightSpec((h, v))}

    def bind(self, tensors, rt) -> None:
        if tensors["a1"].shape[0] != tensors["a2"].shape[1]:
            raise ConfigError(f"gated linear attention: the decay's two maps disagree on their rank ({tensors['a1'].shape[0]} and "
                              f"{tensors['a2'].shape[1]})")
        self.gate_rank = int(tensors["a1"].shape[0])
        # one product for q, k, v, the gate and the decay's low-rank half
        self.w_in = ops.StreamedWeight(torch.cat([tensors[n] for n in ("q", "k", "v", "g", "a1")], dim=0).contiguous())
        self.w_a2 = ops.StreamedWeight(tensors["a2"])
        self.w_o = ops.StreamedWeight(tensors["o"])
        self.a2_b = tensors["a2.b"].to(torch.float32).contiguous()
        self.norm_w = tensors["norm"].to(torch.float32).contiguous()
        self.act_dtype = rt.act_dtype

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        H, d, e = self.heads, self.dim, self.vdim
        x = linear(h, self.w_in, out_dtype=self.act_dtype)
        at = [0, H * d, 2 * H * d, 2 * H * d + H * e, 2 * H * d + 2 * H * e]
        q, k, v, g, low = (x[:, at[0]:at[1]], x[:, at[1]:at[2]], x[:, at[2]:at[3]], x[:, at[3]:at[4]], x[:, at[4]:])
        z = linear(low.contiguous(), self.w_a2, out_dtype=torch.float32)          # the decays' logits stay float32
        base, n_chunks = self._chunks(ctx)
        o = ops.decay_scan(q, k, v, cache.state, ctx, H, d, e, z=z, z_bias=self.a2_b, inv_tau=1.0 / self.tau,
                           q_scale=d ** -0.5, chunk_base=base, n_chunks=n_chunks)
        linear(ops.heads_finish(o, self.act_dtype, weight=self.norm_w, eps=self.eps, gate=g, act=ops.ACT_SILU), self.w_o,
               accumulate_into=residual, ctx=ctx)


register_part("mixer", "retention", Retention)
register_part("mixer", "gla", GatedLinearAttention)
