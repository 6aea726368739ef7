"""Connectors: how a sublayer reads, and writes back into, a stream that is kept as several copies."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import CONNECTORS, Part


@CONNECTORS.register("stream_mixer")
class StreamMixer(Part):
    """The stream is n copies x_1 .. x_n [n, T, width], 32-bit.  A sublayer reads u = sum_s in[s] x_s (normed by the block's
    norm); with its result y every copy is made anew from the old ones: x_t <- sum_s mix[s, t] x_s + out[t] * y.
    Tensors: `in` [n], `out` [n], `mix` [n, n] (indexed [from, to])."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, n_streams: int, in_name: str, out_name: str, mix_name: str):
        if not 1 <= n_streams <= ops.STREAMS_MAX:
            raise ValueError(f"stream_mixer: {n_streams} copies of the stream; the kernels take 1 to {ops.STREAMS_MAX}")
        self.n, self.in_name, self.out_name, self.mix_name = n_streams, in_name, out_name, mix_name

    def param_specs(self):
        n = self.n
        return [ParamSpec(self.in_name, (n,), "vector", ("normal", 1.0 / n, 0.1)),
                ParamSpec(self.out_name, (n,), "vector", ("normal", 1.0, 0.2)),
                ParamSpec(self.mix_name, (n, n), "vector", ("normal", 1.0 / n, 0.15))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.w_in, self.w_out = tensors[self.in_name].contiguous(), tensors[self.out_name].contiguous()
        self.mix = tensors[self.mix_name].contiguous()

    def read(self, xs, norm, out_dtype):
        """norm(sum_s in[s] x_s) as rows of out_dtype; norm: a norm without a mean (`weight`, `eps`)."""
        out = torch.empty(xs.shape[1:], dtype=out_dtype, device=xs.device)
        return ops.streams_read(xs, self.w_in, norm.weight, norm.eps, out)

    def write(self, xs, y, then=None, norm=None, out_dtype=None, branches=None):
        """The copies anew, in place.  then: the connector of the sublayer that reads the stream next; its read (with `norm`)
        then happens in the same kernel and its rows come back.  branches: y is the first of two results whose normed mean
        is the sublayer's (ops.streams_write)."""
        if then is None:
            ops.streams_write(xs, y, self.mix, self.w_out, branches=branches)
            return None
        out = torch.empty(xs.shape[1:], dtype=out_dtype, device=xs.device)
        return ops.streams_write(xs, y, self.mix, self.w_out, next_in=then.w_in, weight=norm.weight, eps=norm.eps, out=out,
                                 branches=branches)
