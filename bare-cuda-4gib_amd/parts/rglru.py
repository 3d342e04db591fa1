"""The recurrent block with a real-gated linear recurrent unit."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.specs import States
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear


class RGLRU(Part):
    """Two branches of ``width`` channels: y = gelu_tanh(Wy h + by) and u = conv(Wx h + bx), a causal convolution over
    time on each channel with a bias.  u is cut into ``blocks`` equal parts; in part b, r = sigmoid(Ra[b] u_b + ra_b)
    and i = sigmoid(Ri[b] u_b + ri_b); a = exp(-8 r softplus(lam)); S_t = a S_(t-1) + sqrt(1 - a^2) i u from S = 0;
    the block adds Wo (S * y) to the stream.  Gates, decay and the state S are float32.  A request's state is S and
    the convolution's last taps - 1 inputs."""
    category = "mixer"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, width: int, blocks: int, conv_taps: int):
        if hidden_size <= 0 or width <= 0 or blocks <= 0 or width % blocks or conv_taps < 1:
            raise ConfigError(f"rglru: width {width} in {blocks} blocks, {conv_taps} taps, stream width {hidden_size}")
        self.hidden_size, self.width, self.blocks, self.conv_taps = int(hidden_size), int(width), int(blocks), int(conv_taps)

    def cache_spec(self):
        return States((("state", (self.width,), "float32"), ("tail", (self.conv_taps - 1, self.width), None)))

    def weight_specs(self) -> Dict[str, WeightSpec]:
        W, h, B = self.width, self.hidden_size, self.blocks
        bs = W // B
        vec = lambda *shape: WeightSpec(tuple(shape), kind="vector")      # noqa: E731
        return {"y": WeightSpec((W, h)), "y.b": vec(W), "x": WeightSpec((W, h)), "x.b": vec(W),
                "conv": vec(W, self.conv_taps), "conv.b": vec(W),
                "ra": WeightSpec((B, bs, bs)), "ra.b": vec(B, bs), "ri": WeightSpec((B, bs, bs)), "ri.b": vec(B, bs),
                "lam": vec(W), "o": WeightSpec((h, W))}

    def bind(self, tensors, rt) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).reshape(-1).contiguous()      # noqa: E731
        # one product for both branches: the gated branch's rows, then the recurrent one's
        self.w_yx = ops.StreamedWeight(torch.cat([tensors["y"], tensors["x"]], dim=0).contiguous())
        self.w_o = ops.StreamedWeight(tensors["o"])
        self.y_b, self.x_b, self.conv_b, self.lam = f32("y.b"), f32("x.b"), f32("conv.b"), f32("lam")
        self.ra_b, self.ri_b = f32("ra.b"), f32("ri.b")
        self.conv_w = tensors["conv"].to(torch.float32).t().contiguous()   # by taps
        # [block, 2 bs, bs]: both gates' matrices of a block in one product per block
        self.w_gates = torch.cat([tensors["ra"], tensors["ri"]], dim=1).contiguous()
        self.act_dtype = rt.act_dtype

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        yx = linear(h, self.w_yx, out_dtype=self.act_dtype)
        y, x = yx[:, :self.width], yx[:, self.width:]
        u = ops.causal_conv(x, self.conv_w, cache.tail if self.conv_taps > 1 else None, ctx, in_bias=self.x_b,
                            out_bias=self.conv_b)
        out = ops.rglru(u, y, self.w_gates, self.ra_b, self.ri_b, self.lam, self.y_b, cache.state, ctx)
        linear(out, self.w_o, accumulate_into=residual, ctx=ctx)


register_part("mixer", "rglru", RGLRU)
