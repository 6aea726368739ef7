"""Token inputs: what a layer adds to the stream from a table's rows that the step's own tokens pick (a second way in
for the token, behind the embedding).  The table belongs to the model (DecoderSpec.tables): several layers read their
own columns of one table."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import TOKEN_INPUTS, Part
from .linear import Linear

F32 = torch.float32


@TOKEN_INPUTS.register("gated_table_rows")
class GatedTableRows(Part):
    """e = table[token, offset : offset + dim];  g = act(W_gate x) * e;  y = W_proj g;  x += y / sqrt(mean(y^2) + eps) * w,
    with x the stream's rows as they stand (not normed).  act: "gelu_tanh".  Steps of many rows run it as two products with
    the activation in the first one's epilogue; steps of up to `ops.TOKEN_INPUT_ROWS_MAX` rows as one kernel."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, width: int, dim: int, table: str, offset: int, eps: float, gate: str, proj: str, norm: str,
                 activation: str = "gelu_tanh"):
        if activation != "gelu_tanh":
            raise ValueError(f"gated_table_rows: activation {activation!r}; known: ['gelu_tanh']")
        if dim < 1 or offset < 0:
            raise ValueError(f"gated_table_rows: {dim} columns from column {offset}")
        self.width, self.dim, self.table, self.offset, self.eps, self.norm_name = width, dim, table, offset, eps, norm
        self.activation = activation
        self.gate = Linear(width, dim, gate, None, init_std=width ** -0.5)
        self.proj = Linear(dim, width, proj, None, init_std=dim ** -0.5)

    def param_specs(self):
        return self.gate.param_specs() + self.proj.param_specs() + [
            ParamSpec(self.norm_name, (self.width,), "vector", ("normal", 1.0, 0.1))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.gate.bind(tensors), self.proj.bind(tensors)
        self.norm = tensors[self.norm_name]
        # the matrices in rows as well, for the kernel that makes a step of few rows in one launch
        wg, wp = tensors[self.gate.weight_name], tensors[self.proj.weight_name]
        fits = (2 * self.width + self.dim) * 4 <= 60000 and wg.dtype == wp.dtype
        self.gate_rows, self.proj_rows = (wg.contiguous(), wp.contiguous()) if runtime.act_dtype != F32 and fits else (None, None)
        rows = runtime.tables.get(self.table)
        if rows is None:
            raise KeyError(f"gated_table_rows: the model has no table {self.table!r}")
        if rows.shape[1] < self.offset + self.dim:
            raise ValueError(f"gated_table_rows: columns {self.offset} .. {self.offset + self.dim} of a table with {rows.shape[1]}")
        self.rows = rows

    def forward(self, x, ctx, then=None):
        """then: the norm that reads the stream next: where it is a plain `rmsnorm` its rows come out of the last kernel and
        are returned (else None)."""
        from .norms import following_norm
        act = self.runtime.act_dtype
        nxt = following_norm(then, x, act)
        if self.gate_rows is not None and x.shape[0] <= ops.TOKEN_INPUT_ROWS_MAX:
            # a step of few rows: one launch (the bfloat16 engine; the 32-bit engine keeps the products' one order of sums)
            ops.token_input(x, self.gate_rows, self.proj_rows, self.rows, ctx.tokens, self.offset, self.norm, self.eps, then=nxt)
        else:
            g = self.gate(x, out_dtype=act, epilogue=self.activation)
            ops.rows_times_table(g, self.rows, ctx.tokens, self.offset, g)
            ops.rmsnorm_add(self.proj(g, out_dtype=F32), self.norm, None, 1.0, self.eps, x, then=nxt)
        return nxt[2] if nxt is not None else None


@TOKEN_INPUTS.register("none")
class NoTokenInput(Part):
    graph_safe = True
    absent = True

    def __init__(self):
        pass

    def forward(self, x, ctx, then=None):
        return None
