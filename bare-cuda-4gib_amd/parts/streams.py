"""The residual stream in several copies, and the vectors and the matrix by which a sublayer reads and writes them."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part


class HyperConnection(Part):
    """A sublayer's connection to a residual stream kept in ``streams`` copies X [T, n, H] (float32):

        read    u = sum_s in[s] X[s]                              what the sublayer's norm gets
        write   X'[t] = sum_s mix[s, t] X[s] + out[t] y           all copies at once, from the old ones

    ``in`` and ``out`` are vectors [n], ``mix`` a matrix [n, n] indexed [from, to].  A norm that is applied element by
    element (``pointwise()``) rides along with the read; the read of the sublayer that follows rides along with the
    write (``then``), while the new copies are in registers."""
    category = "connection"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, streams: int):
        if not (1 <= int(streams) <= ops.MAX_STREAMS):
            raise ConfigError(f"hyper-connection: {streams} copies of the stream; the kernels take 1 to {ops.MAX_STREAMS}")
        self.streams = int(streams)
        self.read_w = self.write_w = self.mix = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        n = self.streams
        return {"in": WeightSpec((n,), kind="vector", init="ones"), "out": WeightSpec((n,), kind="vector", init="ones"),
                "mix": WeightSpec((n, n), kind="vector", init="ones")}

    def bind(self, tensors, rt) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()      # noqa: E731
        self.read_w, self.write_w, self.mix = f32("in"), f32("out"), f32("mix")
        self.act_dtype = rt.act_dtype

    def read(self, x: torch.Tensor, norm, ctx) -> torch.Tensor:
        """The sublayer's input: norm(sum_s in[s] X[s]) in the activations' type."""
        pointwise = norm.pointwise() if hasattr(norm, "pointwise") else None
        if pointwise is not None:
            return ops.streams_read(x, self.read_w, pointwise, self.act_dtype)
        return norm.forward(ops.streams_read(x, self.read_w, None, torch.float32), ctx)

    def write(self, x: torch.Tensor, y: torch.Tensor, then: Optional["StreamReader"] = None, ctx=None) -> Optional[torch.Tensor]:
        """Updates the copies in place with the sublayer's output y [T, H] (float32); with ``then`` returns the input of
        the sublayer that reads next."""
        if then is None:
            ops.streams_write(x, y, self.mix, self.write_w)
            return None
        pointwise = then.norm.pointwise() if hasattr(then.norm, "pointwise") else None
        if pointwise is not None:
            return ops.streams_write(x, y, self.mix, self.write_w, then.connection.read_w, pointwise, self.act_dtype)
        return then.norm.forward(ops.streams_write(x, y, self.mix, self.write_w, then.connection.read_w, None, torch.float32), ctx)


class StreamReader:
    """Who reads the copies next: a connection's read vector and the norm behind it.  (It is also what a block names as
    its first reader, so that the block before can prepare its input.)"""

    def __init__(self, connection: HyperConnection, norm):
        self.connection, self.norm = connection, norm


register_part("connection", "hyper", HyperConnection)
