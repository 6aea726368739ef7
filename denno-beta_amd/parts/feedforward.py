"""Feed-forwards: the parts that work on each token alone."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import FEED_FORWARDS, Part
from .linear import Linear

ACTIVATION_EPILOGUES = {"gelu_tanh": "gelu_tanh", "gelu_erf": "gelu_erf"}
# activations with numbers of their own in a tensor: a kernel between the two products, on the first one's 32-bit result
ACTIVATION_KERNELS = ("xielu",)
F32 = torch.float32


@FEED_FORWARDS.register("dense_mlp")
class DenseMLP(Part):
    """act(h W_up + b_up) W_down + b_down, added into the residual stream
    (crates/denno-engine/src/model/gpt2.rs:211-219).  The activation runs in the first
    product's epilogue, in 32-bit, before the rounding to the activation dtype.

    activation "xielu": z > 0: softplus(p) z^2 + z / 2; else (1/2 + softplus(q)) (e^z - 1 - z) + z / 2, with (p, q) the two
    numbers of the tensor `activation_params`; it runs as a kernel of its own on the first product's 32-bit result."""
    graph_safe = True
    returns_rows = True

    def __init__(self, width: int, inner: int, activation: str, up_weight: str, up_bias, down_weight: str,
                 down_bias, stored_in_out: bool = False, down_init_std: float = 0.02, activation_params=None):
        if activation not in ACTIVATION_EPILOGUES and activation not in ACTIVATION_KERNELS:
            raise ValueError(f"activation {activation!r}; known: {sorted(ACTIVATION_EPILOGUES) + list(ACTIVATION_KERNELS)}")
        if (activation in ACTIVATION_KERNELS) != (activation_params is not None):
            raise ValueError(f"activation {activation!r}: the tensor of its numbers is " +
                             ("missing" if activation_params is None else "not used"))
        self.width, self.inner, self.activation, self.activation_params = width, inner, activation, activation_params
        if activation in ACTIVATION_KERNELS:
            self.libraries = ("sequence",)
        self.up = Linear(width, inner, up_weight, up_bias, stored_in_out)
        self.down = Linear(inner, width, down_weight, down_bias, stored_in_out, down_init_std)

    def param_specs(self):
        own = [ParamSpec(self.activation_params, (2,), "vector", ("normal", 0.3, 0.3))] if self.activation_params else []
        return self.up.param_specs() + self.down.param_specs() + own

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.up.bind(tensors)
        self.down.bind(tensors)
        if self.activation_params:
            pq = tensors[self.activation_params].to(F32)
            sp = torch.nn.functional.softplus(pq)
            self.act_numbers = torch.stack([sp[0], 0.5 + sp[1]]).contiguous()      # (softplus(p), 1/2 + softplus(q)), once

    def packed_input(self, n_rows):
        return self.activation in ACTIVATION_EPILOGUES and self.up.packed_input(n_rows)

    def prepare_lazy_norm(self, norm):
        self.up.fold_norm(norm)

    def takes_lazy_norm(self, n_rows, norm):
        return self.up.takes_lazy_norm(n_rows, norm)

    def writes_norm_stats(self, n_rows):
        return self.down.writes_norm_stats(n_rows)

    def defers_sum(self, n_rows):
        return self.down.defers(n_rows)

    def forward(self, h, ctx, accumulate_into, stats=None, deferred=None):
        n = h.shape[0]
        if self.activation in ACTIVATION_KERNELS:
            z = self.up(h, out_dtype=F32)
            f = ops.activate(z, self.activation, torch.empty(z.shape, dtype=self.runtime.act_dtype, device=z.device),
                             lower=self.act_numbers)
        else:
            f = self.up(h, out_dtype=self.runtime.act_dtype, epilogue=ACTIVATION_EPILOGUES[self.activation],
                        packed_out=self.up.few_rows(n) and self.down.packed_input(n) and accumulate_into is not None)
        if accumulate_into is None:
            return self.down(f, out_dtype=F32)
        self.down(f, residual=accumulate_into, stats=stats, deferred=deferred)


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    """W_down (act(W_gate h) * (W_up h)), act "silu"; no biases.  Gate and up are one product whose 32-bit result the
    activation reads."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, inner: int, gate_weight: str, up_weight: str, down_weight: str, activation: str = "silu"):
        if activation != "silu":
            raise ValueError(f"gated_mlp: activation {activation!r}; known: ['silu']")
        self.width, self.inner, self.activation = width, inner, activation
        self.up = Linear(width, 2 * inner, gate_weight + "+up", None, init_std=width ** -0.5,
                         weight_sources=((gate_weight, inner), (up_weight, inner)))
        self.down = Linear(inner, width, down_weight, None, init_std=inner ** -0.5)

    def param_specs(self):
        return self.up.param_specs() + self.down.param_specs()

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.up.bind(tensors), self.down.bind(tensors)

    def forward(self, h, ctx, accumulate_into):
        n = self.inner
        gu = self.up(h, out_dtype=F32)
        f = ops.gated(gu[:, n:], gu[:, :n], self.activation, torch.empty((h.shape[0], n), dtype=self.runtime.act_dtype, device=h.device))
        if accumulate_into is None:
            return self.down(f, out_dtype=F32)
        self.down(f, residual=accumulate_into)


@FEED_FORWARDS.register("none")
class NoFeedForward(Part):
    """A block without a feed-forward: nothing is added to the stream (and the block does not run the norm before it)."""
    graph_safe = True
    absent = True

    def __init__(self):
        pass

    def forward(self, h, ctx, accumulate_into):
        return None


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(Part):
    """A mixture of small feed-forwards.  The router's scores are s = softmax(W_router h) over all experts, in 32-bit; a
    token's `top` experts are the ones with the largest s + correction, its weights their s divided by their sum
    (+ 1e-20).  An expert: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit), W_down (g sigmoid(alpha g) (u + 1)).
    The step's (token, expert) pairs are sorted by expert on the device, each expert's products run over tiles of its
    own rows, and the results are added into the stream per token in the order of its choices.

    What an architecture may choose otherwise: score "sigmoid" (each expert's own 1 / (1 + e^-z)); renorm False (the
    weights are the chosen scores as they are); weigh "input" (a weight multiplies what the expert reads, not what it
    returns); act "silu" (an expert is W_down (silu(W_gate h) * (W_up h)), nothing clamped; limit and alpha are then not
    used), act "relu2" (an expert without a gate, W_down max(W_up h, 0)^2; `gate` is then None, also the shared expert's);
    shared: an expert of the same form that every token uses, dict(inner, gate, up, down, token_gate): its result is
    added, times sigmoid(w . h) with w the vector `token_gate` (a name, or None: as it is); groups and keep: the experts are
    `groups` equal runs of neighbours, a group's score is the sum of its two largest s + correction, and only the experts
    of the `keep` best groups can be chosen; route_scale multiplies the weights."""
    graph_safe = True
    returns_rows = True
    libraries = ("grouped", "sequence")

    def __init__(self, width: int, inner: int, n_experts: int, top: int, router: str, correction, gate: str, up: str, down: str,
                 limit: float = 0.0, alpha: float = 1.0, score: str = "softmax", renorm: bool = True, weigh: str = "output",
                 act: str = "clamped", shared=None, groups: int = 1, keep: int = 1, route_scale: float = 1.0):
        """gate, up, down: tensor names with {e} for the expert's number; correction: a name or None."""
        if not 1 <= top <= n_experts:
            raise ValueError(f"routed_experts: {top} of {n_experts} experts")
        if score not in ("softmax", "sigmoid") or weigh not in ("output", "input") or act not in ("clamped", "silu", "relu2"):
            raise ValueError(f"routed_experts: score {score!r}, weigh {weigh!r}, act {act!r}")
        if weigh == "input" and act != "silu":
            raise ValueError("routed_experts: a weight on what the expert reads goes with act 'silu'")
        if (act == "relu2") != (gate is None):
            raise ValueError("routed_experts: act 'relu2' is an expert without a gate matrix, and only that one")
        if groups < 1 or n_experts % groups != 0 or not 1 <= keep <= groups or top > keep * (n_experts // groups):
            raise ValueError(f"routed_experts: {n_experts} experts in {groups} groups of which {keep} are kept, for {top} choices")
        self.groups, self.keep, self.route_scale = int(groups), int(keep), float(route_scale)
        self.gated = gate is not None
        self.width, self.inner, self.n_experts, self.top = width, inner, n_experts, top
        self.limit, self.alpha = float(limit), float(alpha)
        self.score, self.renorm, self.weigh, self.act = score, bool(renorm), weigh, act
        self.correction_name = correction
        self.templates = dict(gate=gate, up=up, down=down)
        self.shared = dict(shared) if shared else None
        self.token_gate = self.shared.get("token_gate") if self.shared else None
        # the router, and behind its rows the shared expert's gate: one product for both
        if self.token_gate:
            self.router = Linear(width, n_experts + 1, router + "+gate", None, init_std=width ** -0.5,
                                 weight_sources=((router, n_experts), (self.token_gate, 1)))
        else:
            self.router = Linear(width, n_experts, router, None)
        if self.shared:
            sh = self.shared
            if self.gated:
                self.shared_up = Linear(width, 2 * sh["inner"], sh["gate"] + "+up", None, init_std=width ** -0.5,
                                        weight_sources=((sh["gate"], sh["inner"]), (sh["up"], sh["inner"])))
            else:
                self.shared_up = Linear(width, sh["inner"], sh["up"], None, init_std=width ** -0.5)
            self.shared_down = Linear(sh["inner"], width, sh["down"], None)

    def _stacked(self, which):
        E = self.n_experts
        rows, cols = (self.width, self.inner) if which == "down" else (self.inner, self.width)
        t = self.templates[which]
        return ParamSpec(t.format(e="*"), (E * rows, cols), "matrix", ("normal", 0.0, cols ** -0.5),
                         sources=tuple((t.format(e=e), rows) for e in range(E)), concat_dim=0)

    def param_specs(self):
        specs = self.router.param_specs() + [self._stacked(w) for w in (("gate", "up", "down") if self.gated else ("up", "down"))]
        if self.correction_name:
            specs.append(ParamSpec(self.correction_name, (self.n_experts,), "vector", ("normal", 0.0, 0.02)))
        if self.shared:
            specs += self.shared_up.param_specs() + self.shared_down.param_specs()
        return specs

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.router.bind(tensors)
        if self.shared:
            self.shared_up.bind(tensors), self.shared_down.bind(tensors)
        E = self.n_experts
        self.w_gate = tensors[self.templates["gate"].format(e="*")].view(E, self.inner, self.width) if self.gated else None
        self.w_up = tensors[self.templates["up"].format(e="*")].view(E, self.inner, self.width)
        self.w_down = tensors[self.templates["down"].format(e="*")].view(E, self.width, self.inner)
        self.correction = tensors[self.correction_name] if self.correction_name else None
        # bfloat16 experts on the GPU are held packed for the matrix cores, the stack as one matrix, where an expert's
        # rows start at a block's border (the rows they came from are not kept)
        self.up_dims = self.down_dims = None
        if self.w_up.dtype == torch.bfloat16 and self.w_up.is_cuda:
            if ops.experts_packable(E, self.inner, self.width):
                if self.gated:
                    self.w_gate = ops.pack_matrix(self.w_gate.view(E * self.inner, self.width))
                self.w_up = ops.pack_matrix(self.w_up.view(E * self.inner, self.width))
                self.up_dims = (E, self.inner, self.width)
            if ops.experts_packable(E, self.width, self.inner):
                self.w_down = ops.pack_matrix(self.w_down.view(E * self.width, self.inner))
                self.down_dims = (E, self.width, self.inner)
        self.w_dtype = torch.bfloat16 if isinstance(self.w_up, ops.PackedMatrix) else self.w_up.dtype

    def forward(self, h, ctx, accumulate_into):
        T, top, dev = h.shape[0], self.top, h.device
        wdt = self.w_dtype
        if h.dtype != wdt:        # (experts stored in 32-bit in a bfloat16 engine: their products run on widened rows)
            h = ops.cast(h.contiguous(), torch.empty(h.shape, dtype=wdt, device=dev))
        returns = accumulate_into is None
        if returns:
            accumulate_into = torch.zeros((T, self.width), dtype=torch.float32, device=dev)
        z = self.router(h, out_dtype=torch.float32)
        ids = torch.empty((T, top), dtype=torch.int32, device=dev)
        wts = torch.empty((T, top), dtype=torch.float32, device=dev)
        ops.moe_route(z, self.correction, top, ids, wts, score=self.score, renorm=self.renorm, n_experts=self.n_experts,
                      groups=self.groups, keep=self.keep, scale=self.route_scale)
        offsets = torch.empty(self.n_experts + 1, dtype=torch.int32, device=dev)
        order = torch.empty(T * top, dtype=torch.int32, device=dev)
        ops.moe_plan(ids, self.n_experts, offsets, order)
        y = torch.empty((T * top, self.inner), dtype=wdt, device=dev)
        on_input = self.weigh == "input"
        ops.moe_up(h, order, offsets, top, self.w_gate, self.w_up, self.limit, self.alpha, y, dims=self.up_dims,
                   kind=self.act, in_scale=wts if on_input else None)
        out = torch.empty((T * top, self.width), dtype=torch.float32, device=dev)
        ops.moe_down(y, order, offsets, self.w_down, out, dims=self.down_dims)
        ops.moe_combine(out, None if on_input else wts, accumulate_into)
        if self.shared:
            n = self.shared["inner"]
            if not self.gated and not self.token_gate:
                # max(W_up h, 0)^2 in the first product's epilogue, the second product added where the experts' results are
                f = self.shared_up(h, out_dtype=self.shared_down.weight.dtype, epilogue="relu2")
                self.shared_down(f, residual=accumulate_into)
                return accumulate_into if returns else None
            gu = self.shared_up(h, out_dtype=torch.float32)
            f = torch.empty((T, n), dtype=self.shared_down.weight.dtype, device=dev)
            if self.gated:
                ops.gated(gu[:, n:], gu[:, :n], "silu", f)
            else:
                ops.activate(gu, "relu2", f)
            s = self.shared_down(f, out_dtype=torch.float32)
            if self.token_gate:
                E = self.n_experts
                ops.moe_combine(s, z[:, E:E + 1], accumulate_into, logits=True)      # (times sigmoid of the gate's column)
            else:
                ops.moe_combine(s, None, accumulate_into)
        if returns:
            return accumulate_into
