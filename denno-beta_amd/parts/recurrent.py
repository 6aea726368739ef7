"""Mixers that keep a matrix per head instead of keys and values: S <- diag(w) S + a v^T, read with a query.
Both run the one scan kernel (kernels.ops.state_scan); what differs is how a token makes r, a, v and w."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import MIXERS, FixedState, Part
from .linear import Linear

F32 = torch.float32


@MIXERS.register("wkv")
class WKV(Part):
    """Every projection reads its own blend of the token's row and the row before it, h + (h' - h) mu.  r, k, v are
    plain projections, the gate silu(W_g .), the decay w = exp(-exp(W_2 tanh(W_1 .) + w0)) per head and key channel.
    o_t = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T; each head's o is divided by its root mean square,
    times a weight per column, times the gate, then the output projection.  State: S in 32-bit and the last row."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, head_dim: int, eps: float, lora: int, names: dict):
        """names: r, k, v, g, w1, w2, o (matrices); mu_r, mu_k, mu_v, mu_g, mu_w, w0, u, norm (vectors)."""
        self.width, self.n_heads, self.head_dim, self.eps, self.lora, self.names = width, n_heads, head_dim, eps, lora, dict(names)
        n = n_heads * head_dim
        self.inner = n
        self.r, self.k, self.v, self.g = (Linear(width, n, names[s], None) for s in "rkvg")
        self.w1, self.w2 = Linear(width, lora, names["w1"], None), Linear(lora, n, names["w2"], None)
        self.out = Linear(n, width, names["o"], None)

    def param_specs(self):
        n, W = self.inner, self.width
        specs = []
        for lin in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.out):
            specs += lin.param_specs()
        specs += [ParamSpec(self.names["mu_" + s], (W,), "vector", ("normal", 0.5, 0.15)) for s in "rkvgw"]
        specs += [ParamSpec(self.names["w0"], (n,), "vector", ("normal", -1.0, 0.7)),
                  ParamSpec(self.names["u"], (self.n_heads, self.head_dim), "vector", ("normal", 0.3, 0.3)),
                  ParamSpec(self.names["norm"], (n,), "vector", ("normal", 1.0, 0.1))]
        return specs

    def cache_spec(self):
        return FixedState((self.inner * self.head_dim + self.width,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        for lin in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.out):
            lin.bind(tensors)
        self.mu = torch.stack([tensors[self.names["mu_" + s]] for s in "rkvgw"]).contiguous()
        self.w0, self.norm = tensors[self.names["w0"]], tensors[self.names["norm"]]
        self.u = tensors[self.names["u"]].reshape(-1).contiguous()

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, n = self.runtime.act_dtype, h.shape[0], self.inner
        state, last = cache.state[:, :n * self.head_dim], cache.state[:, n * self.head_dim:]
        mixes = torch.empty((5, T, self.width), dtype=act, device=h.device)
        ops.shift_mix(h, last, self.mu, ctx.row_start, ctx.state_slots, mixes)
        if cache.writes:
            ops.history_update(h, last, ctx.row_start, ctx.state_slots)
        r, k, v, g = (lin(mixes[i], out_dtype=F32) for i, lin in enumerate((self.r, self.k, self.v, self.g)))
        low = ops.activate(self.w1(mixes[4], out_dtype=F32), "tanh", torch.empty((T, self.lora), dtype=act, device=h.device))
        w = self.w2(low, out_dtype=F32)
        ops.activate(w, "exp_neg_exp", w, bias=self.w0)
        o = torch.empty((T, n), dtype=F32, device=h.device)
        ops.state_scan(r, k, v, w, self.u, state, ctx.row_start, ctx.state_slots, self.n_heads, self.head_dim, self.head_dim, o)
        y = torch.empty((T, n), dtype=act, device=h.device)
        ops.head_norm(o, self.norm, self.eps, y, self.n_heads, gate=g, gate_kind="silu")
        self.out(y, residual=accumulate_into)


@MIXERS.register("hgrn2")
class HGRN2(Part):
    """The forget gate f = lower + (1 - lower) sigmoid(W_f h + b) per head and channel also decides what is written:
    S <- diag(f) S + (1 - f) v^T, o = S^T q with q = silu(W_q h); each head's o is normed over its value columns with
    one weight shared by the heads, then the output projection.  State: S in 32-bit."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, head_dim: int, value_dim: int, eps: float, names: dict):
        """names: q, f, v, o (matrices); f_bias, lower, norm (vectors)."""
        self.width, self.n_heads, self.head_dim, self.value_dim, self.eps = width, n_heads, head_dim, value_dim, eps
        self.names = dict(names)
        self.qk, self.vw = n_heads * head_dim, n_heads * value_dim
        self.proj = Linear(width, 2 * self.qk + self.vw, names["q"] + "+f+v", None,
                           weight_sources=((names["q"], self.qk), (names["f"], self.qk), (names["v"], self.vw)))
        self.out = Linear(self.vw, width, names["o"], None)

    def param_specs(self):
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(self.names["f_bias"], (self.qk,), "vector", ("normal", 0.0, 1.0)),
            ParamSpec(self.names["lower"], (self.qk,), "vector", ("uniform", 0.0, 0.9)),
            ParamSpec(self.names["norm"], (self.value_dim,), "vector", ("normal", 1.0, 0.1))]

    def cache_spec(self):
        return FixedState((self.qk * self.value_dim,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        self.f_bias, self.lower, self.norm = (tensors[self.names[s]] for s in ("f_bias", "lower", "norm"))

    def forward(self, h, ctx, cache, accumulate_into):
        act, T = self.runtime.act_dtype, h.shape[0]
        z = self.proj(h, out_dtype=F32)
        q, f, v = z[:, :self.qk], z[:, self.qk:2 * self.qk], z[:, 2 * self.qk:]
        ops.activate(q, "silu", q)
        ops.activate(f, "bounded_sigmoid", f, bias=self.f_bias, lower=self.lower)
        o = torch.empty((T, self.vw), dtype=F32, device=h.device)
        ops.state_scan(q, None, v, f, None, cache.state, ctx.row_start, ctx.state_slots, self.n_heads, self.head_dim,
                       self.value_dim, o, read_after=True, key_from_decay=True)
        y = torch.empty((T, self.vw), dtype=act, device=h.device)
        ops.head_norm(o, self.norm, self.eps, y, self.n_heads)
        self.out(y, residual=accumulate_into)


@MIXERS.register("lightning")
class Lightning(Part):
    """A matrix per head that fades by a constant of the head: q, k and v go through silu, S <- decay_h S + k v^T, o = S^T q
    (the token's own write is read).  All heads' o are normed together as one vector with a weight per column, times
    sigmoid(W_g h), then the output projection.  State: S in 32-bit."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, head_dim: int, value_dim: int, decay, eps: float, names: dict):
        """decay: a number per head; names: q, k, v, g, o (matrices); norm (vector)."""
        self.width, self.n_heads, self.head_dim, self.value_dim, self.eps = width, n_heads, head_dim, value_dim, eps
        self.decay = [float(d) for d in decay]
        if len(self.decay) != n_heads:
            raise ValueError(f"lightning: {len(self.decay)} decays for {n_heads} heads")
        self.names = dict(names)
        self.qk, self.vw = n_heads * head_dim, n_heads * value_dim
        self.proj = Linear(width, 2 * self.qk + 2 * self.vw, names["q"] + "+k+v+g", None, init_std=width ** -0.5,
                           weight_sources=((names["q"], self.qk), (names["k"], self.qk), (names["v"], self.vw), (names["g"], self.vw)))
        self.out = Linear(self.vw, width, names["o"], None)

    def param_specs(self):
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(self.names["norm"], (self.vw,), "vector", ("normal", 1.0, 0.1))]

    def cache_spec(self):
        return FixedState((self.qk * self.value_dim,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        self.norm = tensors[self.names["norm"]]
        self.decay_t = torch.tensor(self.decay, dtype=torch.float64).to(F32).to(runtime.device)

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, qk, vw = self.runtime.act_dtype, h.shape[0], self.qk, self.vw
        z = self.proj(h, out_dtype=F32)
        qkv = z[:, :2 * qk + vw]
        ops.activate(qkv, "silu", qkv)
        o = torch.empty((T, vw), dtype=F32, device=h.device)
        ops.state_scan(z[:, :qk], z[:, qk:2 * qk], z[:, 2 * qk:2 * qk + vw], None, None, cache.state, ctx.row_start, ctx.state_slots,
                       self.n_heads, self.head_dim, self.value_dim, o, read_after=True, w_head=self.decay_t)
        y = torch.empty((T, vw), dtype=act, device=h.device)
        ops.head_norm(o, self.norm, self.eps, y, 1, gate=z[:, 2 * qk + vw:], gate_kind="sigmoid")
        if accumulate_into is None:
            return self.out(y, out_dtype=F32)
        self.out(y, residual=accumulate_into)


@MIXERS.register("channel_delta")
class ChannelDelta(Part):
    """The delta rule with a decay per head and key channel.  q and k (n_qk_heads heads of head_dim) and v (n_heads of
    value_dim) each pass a short causal convolution over time on every channel and silu; q and k are made unit vectors per
    head (x / sqrt(sum x^2 + 1e-6)), q times head_dim^(-1/2); head h reads q and k of head h // (n_heads // n_qk_heads).
    beta = sigmoid(W_b h) per head; the decay g = exp(-exp(A_log_h) * softplus(W_a2 W_a1 h + dt_bias)) per head and key
    channel.  Per head: S <- diag(g) S; e = beta (v - S^T k); S <- S + k e^T; o = S^T q.  Each head's o is divided by its
    root mean square, times a weight per value column that the heads share, times sigmoid(W_g2 W_g1 h); then the output
    projection.  State: S in 32-bit and the convolutions' last taps - 1 inputs."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, n_qk_heads: int, head_dim: int, value_dim: int, taps: int, eps: float,
                 decay_rank: int, gate_rank: int, names: dict, unit_eps: float = 1e-6, query_scale=None):
        """names: q, k, v, b, a1, a2, g1, g2, o (matrices); q_conv, k_conv, v_conv ([channels, taps]); A_log, dt_bias, norm.
        unit_eps: what is added to the sum of squares under the unit vectors' root; query_scale: what the unit queries are
        multiplied by (None: head_dim^(-1/2))."""
        if n_heads % n_qk_heads != 0:
            raise ValueError(f"channel_delta: {n_heads} heads cannot share {n_qk_heads} heads of queries and keys")
        if taps < 1:
            raise ValueError(f"channel_delta: {taps} taps")
        self.width, self.n_heads, self.n_qk_heads, self.head_dim, self.value_dim = width, n_heads, n_qk_heads, head_dim, value_dim
        self.taps, self.eps, self.names = taps, eps, dict(names)
        self.unit_eps = float(unit_eps)
        self.query_scale = head_dim ** -0.5 if query_scale is None else float(query_scale)
        self.qk, self.vw, self.gw = n_qk_heads * head_dim, n_heads * value_dim, n_heads * head_dim
        self.channels = 2 * self.qk + self.vw
        self.decay_rank, self.gate_rank = decay_rank, gate_rank
        n = names
        # two products for everything that reads h: q | k | v | b, which stay 32-bit for the recurrence, and a1 | g1, whose
        # results are the next products' rows
        self.proj = Linear(width, self.channels + n_heads, n["q"] + "+k+v+b", None, init_std=width ** -0.5,
                           weight_sources=((n["q"], self.qk), (n["k"], self.qk), (n["v"], self.vw), (n["b"], n_heads)))
        self.low = Linear(width, decay_rank + gate_rank, n["a1"] + "+g1", None, init_std=width ** -0.5,
                          weight_sources=((n["a1"], decay_rank), (n["g1"], gate_rank)))
        self.a2 = Linear(decay_rank, self.gw, n["a2"], None, init_std=decay_rank ** -0.5)
        self.g2 = Linear(gate_rank, self.vw, n["g2"], None, init_std=gate_rank ** -0.5)
        self.out = Linear(self.vw, width, n["o"], None)

    def param_specs(self):
        n, taps = self.names, self.taps
        specs = []
        for lin in (self.proj, self.low, self.a2, self.g2, self.out):
            specs += lin.param_specs()
        return specs + [
            ParamSpec(n["q_conv"] + "+k+v", (self.channels, taps), "vector", ("normal", 0.0, 0.4),
                      sources=((n["q_conv"], self.qk), (n["k_conv"], self.qk), (n["v_conv"], self.vw))),
            ParamSpec(n["A_log"], (self.n_heads,), "vector", ("uniform", -2.0, 0.5)),
            ParamSpec(n["dt_bias"], (self.gw,), "vector", ("normal", -1.0, 1.0)),
            ParamSpec(n["norm"], (self.value_dim,), "vector", ("normal", 1.0, 0.1))]

    def cache_spec(self):
        return FixedState((self.gw * self.value_dim + (self.taps - 1) * self.channels,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        for lin in (self.proj, self.low, self.a2, self.g2, self.out):
            lin.bind(tensors)
        n = self.names
        self.conv = tensors[n["q_conv"] + "+k+v"]
        self.dt_bias, self.norm = tensors[n["dt_bias"]], tensors[n["norm"]]
        # the decay's rate per head, spread over the head's key channels
        self.rate = torch.exp(tensors[n["A_log"]].to(F32)).repeat_interleave(self.head_dim).contiguous()
        # the second halves of the small products read columns of the first halves' rows where those start at 16 bytes
        per = 16 // (2 if self.a2.weight.dtype == torch.bfloat16 else 4)
        self._views_fit = self.decay_rank % per == 0 and (self.decay_rank + self.gate_rank) % per == 0

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, dev = self.runtime.act_dtype, h.shape[0], h.device
        qk, vw, C, H = self.qk, self.vw, self.channels, self.n_heads
        n_state = self.gw * self.value_dim
        state, past = cache.state[:, :n_state], cache.state[:, n_state:]
        z = self.proj(h, out_dtype=F32)
        x = torch.empty((T, C), dtype=F32, device=dev)
        # the three convolutions, silu, and queries and keys made unit vectors (the queries times dim^(-1/2)): one kernel
        ops.conv_heads(z[:, :C], self.conv, past, ctx.row_start, ctx.state_slots, x, 2 * self.n_qk_heads, self.head_dim,
                       self.n_qk_heads, self.query_scale, 1.0, self.unit_eps, H, self.value_dim)
        if self.taps > 1 and cache.writes:
            ops.history_update(z[:, :C], past, ctx.row_start, ctx.state_slots)
        q, k, v = x[:, :qk], x[:, qk:2 * qk], x[:, 2 * qk:]
        low = self.low(h, out_dtype=self.a2.weight.dtype)
        a_in, g_in = low[:, :self.decay_rank], low[:, self.decay_rank:]
        if not self._views_fit:      # (rows that the products cannot read where they lie)
            a_in, g_in = a_in.contiguous(), g_in.contiguous()
        g = self.a2(a_in, out_dtype=F32)
        ops.activate(g, "exp_neg_softplus", g, bias=self.dt_bias, lower=self.rate)
        gate = self.g2(g_in, out_dtype=F32)
        o = torch.empty((T, vw), dtype=F32, device=dev)
        # (beta = sigmoid of the projection's columns behind the channels, taken inside the scan)
        ops.state_scan(q, k, v, g, None, state, ctx.row_start, ctx.state_slots, H, self.head_dim, self.value_dim, o, beta=z[:, C:C + H],
                       qk_heads=self.n_qk_heads, beta_logits=True)
        y = torch.empty((T, vw), dtype=act, device=dev)
        ops.head_norm(o, self.norm, self.eps, y, H, gate=gate, gate_kind="sigmoid")
        if accumulate_into is None:
            return self.out(y, out_dtype=F32)
        self.out(y, residual=accumulate_into)


@MIXERS.register("min_gru")
class MinGRU(Part):
    """A recurrence of single numbers whose gates read the token alone: z = sigmoid(W_z h + b_z); u = W_x h + b_x; the
    candidate is u + 1/2 where u >= 0 and sigmoid(u) below; S_t = (1 - z) S_(t-1) + z * candidate; the result is
    W_o (S_t * silu(W_g h)).  State: S, `inner` numbers in 32-bit."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, inner: int, names: dict):
        """names: z, x, g, o (matrices); z_bias, x_bias (vectors)."""
        self.width, self.inner, self.names = width, inner, dict(names)
        n = names
        # one product for everything that reads h; its 32-bit result feeds the recurrence (the biases are added there)
        self.proj = Linear(width, 3 * inner, n["z"] + "+x+g", None, init_std=width ** -0.5,
                           weight_sources=((n["z"], inner), (n["x"], inner), (n["g"], inner)))
        self.out = Linear(inner, width, n["o"], None, init_std=inner ** -0.5)

    def param_specs(self):
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(self.names["z_bias"], (self.inner,), "vector", ("normal", 0.0, 1.0)),
            ParamSpec(self.names["x_bias"], (self.inner,), "vector", ("normal", 0.0, 0.5))]

    def cache_spec(self):
        return FixedState((self.inner,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        self.z_bias, self.x_bias = tensors[self.names["z_bias"]], tensors[self.names["x_bias"]]

    def forward(self, h, ctx, cache, accumulate_into):
        n = self.inner
        z = self.proj(h, out_dtype=F32)
        y = torch.empty((h.shape[0], n), dtype=self.runtime.act_dtype, device=h.device)
        ops.gate_scan(z[:, :n], z[:, n:2 * n], z[:, 2 * n:], self.z_bias, self.x_bias, cache.state, ctx.row_start, ctx.state_slots, y)
        if accumulate_into is None:
            return self.out(y, out_dtype=F32)
        self.out(y, residual=accumulate_into)


@MIXERS.register("mamba2")
class Mamba2(Part):
    """A state-space mixer with one decay per head and token.  W_in h is laid out [z: inner | x: inner | B: groups * N |
    C: groups * N | dt: heads], inner = heads * value_dim.  x, B and C pass a short causal convolution per channel (with a
    bias) and silu; dt = log(1 + e^(dt + dt_bias)).  Per head (head a reads B and C of group a // (heads // groups)):
    S <- exp(-e^(A_log) dt) S + dt B x^T (S is N x value_dim), y = S^T C + D x.  y times silu(z) is normed without a mean in
    `norm_groups` equal parts, times a weight per column; then the output projection.  State: S in 32-bit and the
    convolution's last taps - 1 inputs."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, value_dim: int, state_dim: int, n_groups: int, taps: int, norm_groups: int,
                 eps: float, names: dict):
        """names: in, o (matrices); conv [channels, taps], conv_bias, dt_bias, A_log, D, norm."""
        if n_heads % n_groups != 0:
            raise ValueError(f"mamba2: {n_heads} heads cannot share {n_groups} groups of B and C")
        inner = n_heads * value_dim
        if norm_groups < 1 or inner % norm_groups != 0:
            raise ValueError(f"mamba2: {inner} columns cannot be normed in {norm_groups} equal parts")
        if taps < 1:
            raise ValueError(f"mamba2: {taps} taps")
        self.width, self.n_heads, self.value_dim, self.state_dim, self.n_groups = width, n_heads, value_dim, state_dim, n_groups
        self.taps, self.norm_groups, self.eps, self.names = taps, norm_groups, eps, dict(names)
        self.inner, self.bc = inner, n_groups * state_dim
        self.channels = inner + 2 * self.bc
        self.proj = Linear(width, 2 * inner + 2 * self.bc + n_heads, names["in"], None, init_std=width ** -0.5)
        self.out = Linear(inner, width, names["o"], None, init_std=inner ** -0.5)

    def param_specs(self):
        n = self.names
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(n["conv"], (self.channels, self.taps), "vector", ("normal", 0.0, 0.4)),
            ParamSpec(n["conv_bias"], (self.channels,), "vector", ("normal", 0.0, 0.1)),
            ParamSpec(n["dt_bias"], (self.n_heads,), "vector", ("normal", -1.0, 1.0)),
            ParamSpec(n["A_log"], (self.n_heads,), "vector", ("uniform", -2.0, 0.5)),
            ParamSpec(n["D"], (self.n_heads,), "vector", ("normal", 1.0, 0.3)),
            ParamSpec(n["norm"], (self.inner,), "vector", ("normal", 1.0, 0.1))]

    def cache_spec(self):
        return FixedState((self.inner * self.state_dim + (self.taps - 1) * self.channels,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        n = self.names
        self.conv, self.conv_bias = tensors[n["conv"]].contiguous(), tensors[n["conv_bias"]]
        self.dt_bias, self.skip, self.norm = tensors[n["dt_bias"]], tensors[n["D"]], tensors[n["norm"]]
        self.rate = torch.exp(tensors[n["A_log"]].to(F32)).contiguous()

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, dev = self.runtime.act_dtype, h.shape[0], h.device
        H, inner, bc, C = self.n_heads, self.inner, self.bc, self.channels
        n_state = inner * self.state_dim
        state, past = cache.state[:, :n_state], cache.state[:, n_state:]
        proj = self.proj(h, out_dtype=F32)
        gate, raw, dt = proj[:, :inner], proj[:, inner:inner + C], proj[:, inner + C:]
        xbc = torch.empty((T, C), dtype=F32, device=dev)
        ops.conv_rows(raw, self.conv, past, ctx.row_start, ctx.state_slots, xbc, identity=False, act="silu", bias=self.conv_bias)
        if self.taps > 1 and cache.writes:
            ops.history_update(raw, past, ctx.row_start, ctx.state_slots)
        x, B, Cm = xbc[:, :inner], xbc[:, inner:inner + bc], xbc[:, inner + bc:]
        decay = torch.empty((T, H), dtype=F32, device=dev)
        v = torch.empty((T, inner), dtype=F32, device=dev)
        ops.step_sizes(dt, self.dt_bias, self.rate, x, H, decay, v)
        o = torch.empty((T, inner), dtype=F32, device=dev)
        ops.state_scan(Cm, B, v, decay, None, state, ctx.row_start, ctx.state_slots, H, self.state_dim, self.value_dim, o,
                       read_after=True, qk_heads=self.n_groups, w_rows=True)
        y = torch.empty((T, inner), dtype=act, device=dev)
        ops.head_norm(o, self.norm, self.eps, y, self.norm_groups, gate=gate, gate_kind="silu", gate_first=True, skip=x,
                      skip_scale=self.skip)
        if accumulate_into is None:
            return self.out(y, out_dtype=F32)
        self.out(y, residual=accumulate_into)


@MIXERS.register("mamba1")
class Mamba1(Part):
    """The selective scan: a state per channel and state index whose decay the token chooses.  W_in h is laid out
    [x: inner | z: inner]; x passes a short causal convolution per channel (with a bias) and silu.  W_x x is [dt: dt_rank |
    B: N | C: N]; the step of a channel is dt_c = log(1 + e^(W_dt dt + bias)_c); A = -e^(A_log), [inner, N].  Per channel c and
    state index n: S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n; y_c = sum_n S[c, n] C_n + D_c x_c; y times silu(z);
    then the output projection.  State: S in 32-bit and the convolution's last taps - 1 inputs.  32-bit are the
    projections' results that enter the recurrence (dt, B, C, z; the convolution reads its input in 32-bit), the steps, the
    decays, the state and its sums; the products' operands, and x behind its convolution and silu, are the engine's."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, inner: int, state_dim: int, dt_rank: int, taps: int, names: dict):
        """names: in, x, dt, o (matrices); conv [inner, taps], conv_bias, dt_bias, A_log [inner, state_dim], D."""
        if taps < 1 or inner < 1 or dt_rank < 1 or not 1 <= state_dim <= 256:
            raise ValueError(f"mamba1: {inner} channels, {state_dim} states (up to 256), a step of rank {dt_rank}, {taps} taps")
        self.width, self.inner, self.state_dim, self.dt_rank, self.taps, self.names = width, inner, state_dim, dt_rank, taps, dict(names)
        n = names
        self.proj = Linear(width, 2 * inner, n["in"], None, init_std=width ** -0.5)
        self.low = Linear(inner, dt_rank + 2 * state_dim, n["x"], None, init_std=inner ** -0.5)
        self.step = Linear(dt_rank, inner, n["dt"], n["dt_bias"], init_std=dt_rank ** -0.5)
        self.out = Linear(inner, width, n["o"], None, init_std=inner ** -0.5)

    def param_specs(self):
        n = self.names
        specs = []
        for lin in (self.proj, self.low, self.step, self.out):
            specs += lin.param_specs()
        return specs + [
            ParamSpec(n["conv"], (self.inner, self.taps), "vector", ("normal", 0.0, 0.4)),
            ParamSpec(n["conv_bias"], (self.inner,), "vector", ("normal", 0.0, 0.1)),
            ParamSpec(n["A_log"], (self.inner, self.state_dim), "vector", ("uniform", -2.0, 1.0)),
            ParamSpec(n["D"], (self.inner,), "vector", ("normal", 1.0, 0.3))]

    def cache_spec(self):
        return FixedState((self.inner * self.state_dim + (self.taps - 1) * self.inner,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        for lin in (self.proj, self.low, self.step, self.out):
            lin.bind(tensors)
        n = self.names
        self.conv, self.conv_bias, self.skip = tensors[n["conv"]].contiguous(), tensors[n["conv_bias"]], tensors[n["D"]]
        self.rates = (-torch.exp(tensors[n["A_log"]].to(F32))).contiguous()       # A, once
        # the step's product reads the first columns of the rows that W_x left, where those start at 16 bytes
        per = 16 // (2 if self.step.weight.dtype == torch.bfloat16 else 4)
        self._view_fits = (self.dt_rank + 2 * self.state_dim) % per == 0

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, dev = self.runtime.act_dtype, h.shape[0], h.device
        inner, N, R = self.inner, self.state_dim, self.dt_rank
        state, past = cache.state[:, :inner * N], cache.state[:, inner * N:]
        xz = self.proj(h, out_dtype=F32)
        # (what the convolution and its silu leave is in the engine's precision: the next product's rows as they are)
        x = torch.empty((T, inner), dtype=act, device=dev)
        ops.conv_rows(xz, self.conv, past, ctx.row_start, ctx.state_slots, x, identity=False, act="silu", bias=self.conv_bias)
        if self.taps > 1 and cache.writes:
            ops.history_update(xz[:, :inner], past, ctx.row_start, ctx.state_slots)
        low = self.low(x, out_dtype=F32)                              # [dt | B | C], 32-bit: B and C enter the recurrence
        wdt = self.step.weight.dtype
        dt_in = low[:, :R]
        if wdt != F32:
            dt_in = ops.cast(low, torch.empty(low.shape, dtype=wdt, device=dev))[:, :R]
        if not self._view_fits:
            dt_in = dt_in.contiguous()
        dt = self.step(dt_in, out_dtype=F32)                          # (with its bias; the softplus is the scan's)
        y = torch.empty((T, inner), dtype=act, device=dev)
        # (the 32-bit engine walks a request's rows in order: its logits are the same bits however a prompt is cut)
        ops.selective_scan(x, dt, None, low[:, R:R + N], low[:, R + N:], self.rates, self.skip, xz[:, inner:], state,
                           ctx.row_start, ctx.state_slots, y, in_order=act == F32)
        if accumulate_into is None:
            return self.out(y, out_dtype=F32)
        self.out(y, residual=accumulate_into)
