"""Mixers: the parts that let a token see other tokens."""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import MIXERS, POSITIONS, PagedKV, Part
from .linear import Linear


@MIXERS.register("causal_attention")
class CausalSelfAttention(Part):
    """One fused projection to q | k | v, keys and values to the cache, causal softmax
    attention over the cache, output projection added into the residual stream
    (crates/denno-engine/src/model/gpt2.rs:155-208).

    n_kv_heads < n_heads: query head h reads key head h // (n_heads // n_kv_heads).
    window > 0: a query at position p reads keys p - window + 1 .. p only.
    scale multiplies the scores before the softmax.
    position: a position encoding of this layer's own, as (kind name, arguments), of the kind that
    turns queries and keys; None: the model's.
    qkv_weight_sources, qkv_bias_sources: ((file name, columns), ...) where the checkpoint stores the three
    projections as tensors of their own; qkv_weight / qkv_bias then only name the joined tensors.
    value_dim: the width of a value where it is not the keys' (None: head_dim); the output projection then reads
    n_heads * value_dim columns.  exact_turn: the projection's result stays 32-bit until queries and keys are turned by
    their positions, so they are rounded once; it is also the way values of another width go (keys and values are then
    kept side by side in one width, the next multiple of 16 from the wider of the two, the narrower padded with zeros,
    which add nothing to a score or a result).  unit_eps: behind the turn every head's q and k are divided by their root
    mean square, x / sqrt(mean(x^2) + unit_eps) over the head's entries (None: they stay).  head_gate: the name of a matrix
    [n_heads, width]: head a's result is multiplied by sigmoid(W_g h)_a before the output projection (its rows ride behind
    the fused projection's; qkv_weight_sources then names the pieces of q, k and v).  Both go the 32-bit way of exact_turn."""
    graph_safe = True
    returns_rows = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 qkv_weight: str, qkv_bias, out_weight: str, out_bias, stored_in_out: bool = False,
                 window: int = 0, out_init_std: float = 0.02, position=None, qkv_weight_sources=None,
                 qkv_bias_sources=None, value_dim=None, exact_turn: bool = False, unit_eps=None, head_gate=None):
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        self.unit_eps = None if unit_eps is None else float(unit_eps)
        self.head_gate = head_gate
        self.split = bool(exact_turn) or self.value_dim != head_dim or self.unit_eps is not None or head_gate is not None
        if head_gate is not None and (qkv_bias is not None or not qkv_weight_sources or stored_in_out):
            raise ValueError("causal_attention: a gate per head rides behind a projection without a bias that is stored [out, in] "
                             "and whose pieces qkv_weight_sources names")
        # (the split way keeps keys and values in one width that every attention kernel takes)
        self.kept_dim = -(-max(head_dim, self.value_dim) // 16) * 16 if self.split else head_dim
        if not 1 <= self.kept_dim <= 256:
            raise ValueError(f"keys of {head_dim} and values of {self.value_dim}: the attention kernels take up to 256")
        self.scale, self.window = float(scale), int(window)
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} heads cannot share {n_kv_heads} key heads")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim}: the attention kernels take head sizes up to 256")
        self.q_width = n_heads * head_dim
        self.kv_width = n_kv_heads * head_dim
        self.v_width = n_kv_heads * self.value_dim
        # (a checkpoint that stores q, k and v apart names them in qkv_*_sources: joined at load, one product here)
        if head_gate is not None:
            qkv_weight_sources = tuple(qkv_weight_sources) + ((head_gate, n_heads),)
        self.gate_col = self.q_width + self.kv_width + self.v_width
        self.qkv = Linear(width, self.gate_col + (n_heads if head_gate is not None else 0), qkv_weight, qkv_bias, stored_in_out,
                          weight_sources=qkv_weight_sources, bias_sources=qkv_bias_sources)
        self.out = Linear(n_heads * self.value_dim, width, out_weight, out_bias, stored_in_out, out_init_std)
        self.position = POSITIONS.make(position) if position is not None else None
        if self.position is not None:
            self.graph_safe = getattr(self.position, "graph_safe", False)

    def param_specs(self):
        own = self.position.param_specs() if self.position is not None else []
        return self.qkv.param_specs() + self.out.param_specs() + own

    def cache_spec(self):
        return PagedKV(self.n_kv_heads, self.kept_dim, self.window)

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.qkv.bind(tensors)
        self.out.bind(tensors)
        if self.position is not None:
            self.position.bind(tensors, runtime)
        self.no_freq = torch.empty(0, dtype=torch.float32, device=runtime.device)

    def packed_input(self, n_rows):
        return self.qkv.packed_input(n_rows)

    def prepare_lazy_norm(self, norm):
        self.qkv.fold_norm(norm)

    def takes_lazy_norm(self, n_rows, norm):
        return self.qkv.takes_lazy_norm(n_rows, norm)

    def writes_norm_stats(self, n_rows):
        return self.out.writes_norm_stats(n_rows)

    def defers_sum(self, n_rows):
        return self.out.defers(n_rows)

    def _forward_split(self, h, ctx, cache, g, position, accumulate_into):
        """The projection's result in 32-bit; queries and keys turned (or copied) from there into rows of the kept width,
        values copied beside the keys; the cache write, the attention, and the heads' first value_dim columns on."""
        act, T, dev = self.runtime.act_dtype, h.shape[0], h.device
        H, G, dk, dv, hw = self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim, self.kept_dim
        z = self.qkv(h, out_dtype=torch.float32)
        turns = position is not None and getattr(position, "rotates", False)
        padded = hw != dk or hw != dv
        new = torch.zeros if padded else torch.empty
        q = new((T, H * hw), dtype=act, device=dev)
        kv = new((T, 2 * G * hw), dtype=act, device=dev)      # keys at column 0, values at G * hw

        if turns and not hasattr(position, "freq"):
            raise TypeError(f"{type(position).__name__}: the 32-bit turn needs an encoding with a table of frequencies (rotary_pairs)")
        dims = position.dims if turns else 0
        freq = position.freq if turns else self.no_freq
        # (one launch: queries and keys turned, values moved, each to its place in rows of the kept width)
        unit = self.unit_eps is not None
        ops.rotary_runs(z, ctx.positions, freq, [(q, 0, H, dk, dims, 0, hw), (kv, self.q_width, G, dk, dims, 0, hw),
                                                 (kv, self.q_width + self.kv_width, G, dv, 0, G * hw, hw)],
                        mag=getattr(position, "mag", 1.0) if turns else 1.0, unit=[unit, unit, False] if unit else None,
                        eps=self.unit_eps or 0.0)
        if cache.writes:
            ops.kv_write(kv, 0, G * hw, g.slot_map, cache.k, cache.v)
        o = torch.empty((T, H * hw), dtype=act, device=dev)
        ops.attention(q, o, cache.k, cache.v, g.block_tables, g.tiles, H, self.scale, self.window, tiles_wide=g.tiles_wide,
                      single_rows=g.single_rows, max_context=g.max_context)
        if self.head_gate is not None:      # (the gate per head, and the heads' first value_dim columns on, in one launch)
            o = ops.head_gate(o, z[:, self.gate_col:self.gate_col + H], H, dv, torch.empty((T, H * dv), dtype=act, device=dev),
                              head_stride=hw)
        elif hw != dv:
            narrow = torch.empty((T, H * dv), dtype=act, device=dev)
            ops.rotary(o, narrow, ctx.positions, self.no_freq, H, 0, dv, src_off=0, src_stride=hw, dst_off=0, dst_stride=dv)
            o = narrow
        if accumulate_into is None:
            return self.out(o, out_dtype=torch.float32)
        self.out(o, residual=accumulate_into)

    def forward(self, h, ctx, cache, accumulate_into, stats=None, deferred=None):
        act = self.runtime.act_dtype
        g = ctx.groups[cache.group]
        position = self.position if self.position is not None else self.runtime.position
        if self.split:
            return self._forward_split(h, ctx, cache, g, position, accumulate_into)
        if position is not None and getattr(position, "rotates", False):
            # queries and keys are turned by their positions before the keys go to the cache: the
            # product, the turn and the cache write are three steps here, not one kernel
            qkv = self.qkv(h, out_dtype=act)
            q = qkv[:, :self.q_width]
            position.rotate(q, qkv[:, self.q_width:self.q_width + self.kv_width], ctx)
            if cache.writes:
                ops.kv_write(qkv, self.q_width, self.q_width + self.kv_width, g.slot_map, cache.k, cache.v)
        elif cache.writes:
            q = self.qkv.project_qkv(h, act, g.slot_map, cache.k, cache.v, self.q_width)
        else:
            q = self.qkv(h, out_dtype=act)[:, :self.q_width]
        # the bfloat16 kernels hand their rows to the output projection packed, if it wants that
        if self.out.packed_input(h.shape[0]) and ops.attention_writes_packed(
                act, cache.k.shape[2], self.head_dim, g.single_rows, g.max_context, g.tiles_wide):
            o = ops.packed_rows(h.shape[0], self.q_width, h.device)
        else:
            o = torch.empty((h.shape[0], self.q_width), dtype=act, device=h.device)
        ops.attention(q, o, cache.k, cache.v, g.block_tables, g.tiles, self.n_heads,
                      self.scale, self.window, tiles_wide=g.tiles_wide, single_rows=g.single_rows,
                      max_context=g.max_context)
        if accumulate_into is None:
            return self.out(o, out_dtype=torch.float32)
        self.out(o, residual=accumulate_into, stats=stats, deferred=deferred)


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    """Causal softmax attention whose keys and values are made from one small vector per token.

    Per token: q = W_q h, per head [dim plain | rot_dim turned]; W_dkv h gives kv_rank numbers, normed without a mean to
    the latent c, and rot_dim numbers that, turned by the position, are a key part shared by all heads.  Head h's plain
    key is W_uk[h] c, its value W_uv[h] c; the score is (q_plain . k_plain + q_turned . k_turned) * scale.  The heads'
    results, times sigmoid(W_g h), go through the output projection.

    Only c and the turned key part are kept, as one key of kv_rank + rot_dim numbers per token that every head reads:
    q_plain . (W_uk c) = (W_uk^T q_plain) . c, so the query is carried to the latent's space once per token, the
    attention kernels run with one key head of that width (the same rows serve as values), and W_uv is applied to
    the weighted sum of latents.  position: the arguments of a "rotary_pairs" encoding for the turned parts."""
    graph_safe = True
    libraries = ("sequence", "grouped")

    def __init__(self, width: int, n_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int, scale: float,
                 eps: float, position: dict, names: dict, keep: str = None, window: int = 0):
        """names: q, dkv, g, uk, uv, o (matrices; without "g" the heads' results go on ungated); dkv_norm (vector).
        window > 0: a query at position p reads the keys p - window + 1 .. p only.
        keep: "latent" (the form above), "heads" (every head's own key [W_uk c | turned part] and value W_uv c are kept,
        as an ordinary attention does: more cache, and the way out where kv_rank + rot_dim is beyond the attention kernels'
        largest head), or None: "latent" where it fits."""
        self.width, self.n_heads, self.head_dim, self.rot_dim = width, n_heads, head_dim, rot_dim
        self.value_dim, self.kv_rank, self.scale, self.eps, self.names = value_dim, kv_rank, float(scale), eps, dict(names)
        self.key_dim = kv_rank + rot_dim
        self.head_width = max(head_dim + rot_dim, value_dim)      # "heads": keys and values padded with zeros to one width
        if keep not in (None, "latent", "heads"):
            raise ValueError(f"latent_attention: keep = {keep!r}")
        self.keep = keep or ("latent" if self.key_dim <= 256 else "heads")
        kept = self.key_dim if self.keep == "latent" else self.head_width
        if not 1 <= kept <= 256:
            raise ValueError(f"latent_attention: a kept key of {kept} numbers; the attention kernels take up to 256")
        self.q_width = n_heads * (head_dim + rot_dim)
        self.o_width = n_heads * value_dim
        self.window = int(window)
        self.gated = "g" in names
        # one product for everything that reads h: q | dkv | g
        if self.gated:
            self.proj = Linear(width, self.q_width + self.key_dim + self.o_width, names["q"] + "+dkv+g", None,
                               weight_sources=((names["q"], self.q_width), (names["dkv"], self.key_dim), (names["g"], self.o_width)))
        else:
            self.proj = Linear(width, self.q_width + self.key_dim, names["q"] + "+dkv", None,
                               weight_sources=((names["q"], self.q_width), (names["dkv"], self.key_dim)))
        self.out = Linear(self.o_width, width, names["o"], None)
        self.position = POSITIONS.make(("rotary_pairs", dict(position, head_dim=rot_dim)))

    def param_specs(self):
        H, r = self.n_heads, self.kv_rank
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(self.names["uk"], (H * self.head_dim, r), "matrix", ("normal", 0.0, r ** -0.5)),
            ParamSpec(self.names["uv"], (H * self.value_dim, r), "matrix", ("normal", 0.0, r ** -0.5)),
            ParamSpec(self.names["dkv_norm"], (r,), "vector", ("normal", 1.0, 0.1))]

    def cache_spec(self):
        return (PagedKV(1, self.key_dim, self.window) if self.keep == "latent"
                else PagedKV(self.n_heads, self.head_width, self.window))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        self.position.bind(tensors, runtime)
        self.no_freq = torch.empty(0, dtype=torch.float32, device=runtime.device)
        H, r = self.n_heads, self.kv_rank
        # W_uk per head, transposed once: [heads, kv_rank, dim], so that both per-head products are out = W[h] a
        self.uk_t = tensors[self.names["uk"]].view(H, self.head_dim, r).transpose(1, 2).contiguous()
        self.uk = tensors[self.names["uk"]].view(H, self.head_dim, r).contiguous()
        self.uv = tensors[self.names["uv"]].view(H, self.value_dim, r).contiguous()
        self.c_norm = tensors[self.names["dkv_norm"]]

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, H = self.runtime.act_dtype, h.shape[0], self.n_heads
        dn, dr, r, kd = self.head_dim, self.rot_dim, self.kv_rank, self.key_dim
        g = ctx.groups[cache.group]
        z = self.proj(h, out_dtype=torch.float32)
        low, gate = self.q_width, self.q_width + kd
        if self.keep == "heads":
            return self._forward_heads(z, ctx, cache, g, accumulate_into)
        # the token's key: [c | turned part]
        key = torch.empty((T, kd), dtype=act, device=h.device)
        ops.rmsnorm(z[:, low:low + r], self.c_norm, self.eps, key[:, :r])
        self.position.turn(z, key, ctx.positions, 1, dr, src_off=low + r, dst_off=r)
        if cache.writes:
            ops.kv_write(key, 0, 0, g.slot_map, cache.k, cache.v)
        # the queries in the latent's space: [W_uk^T q_plain | turned part] per head
        q = torch.empty((T, H * kd), dtype=act, device=h.device)
        ops.heads_linear(z, self.uk_t, q, a_off=0, a_stride=dn + dr, o_off=0, o_stride=kd)
        self.position.turn(z, q, ctx.positions, H, dr, src_off=dn, src_stride=dn + dr, dst_off=r, dst_stride=kd)
        o_lat = torch.empty((T, H * kd), dtype=act, device=h.device)
        ops.attention(q, o_lat, cache.k, cache.v, g.block_tables, g.tiles, H, self.scale, self.window, tiles_wide=g.tiles_wide,
                      single_rows=g.single_rows, max_context=g.max_context)
        if self.gated:
            o = torch.empty((T, self.o_width), dtype=torch.float32, device=h.device)
            ops.heads_linear(o_lat, self.uv, o, a_off=0, a_stride=kd)
            og = torch.empty((T, self.o_width), dtype=act, device=h.device)
            ops.gated(o, z[:, gate:], "sigmoid", og)
        else:
            og = torch.empty((T, self.o_width), dtype=act, device=h.device)
            ops.heads_linear(o_lat, self.uv, og, a_off=0, a_stride=kd)
        if accumulate_into is None:
            return self.out(og, out_dtype=torch.float32)
        self.out(og, residual=accumulate_into)

    def _forward_heads(self, z, ctx, cache, g, accumulate_into):
        """Every head's key [W_uk c | turned part | zeros] and value [W_uv c | zeros], `head_width` wide, go to the cache;
        the queries are [q_plain | turned part | zeros]: the zeros add nothing to a score or a result."""
        act, T, H, dev = self.runtime.act_dtype, z.shape[0], self.n_heads, z.device
        dn, dr, r, dv, hw = self.head_dim, self.rot_dim, self.kv_rank, self.value_dim, self.head_width
        low, gate = self.q_width, self.q_width + self.key_dim
        copy = lambda src, dst, width, **layout: ops.rotary(src, dst, ctx.positions, self.no_freq, H, 0, width, **layout)   # noqa: E731
        c = torch.empty((T, r), dtype=act, device=dev)
        ops.rmsnorm(z[:, low:low + r], self.c_norm, self.eps, c)
        kv = torch.zeros((T, 2 * H * hw), dtype=act, device=dev)      # keys at column 0, values at H * hw
        ops.heads_linear(c, self.uk, kv, a_off=0, a_stride=0, o_off=0, o_stride=hw)
        self.position.turn(z, kv, ctx.positions, H, dr, src_off=low + r, src_stride=0, dst_off=dn, dst_stride=hw)
        ops.heads_linear(c, self.uv, kv, a_off=0, a_stride=0, o_off=H * hw, o_stride=hw)
        if cache.writes:
            ops.kv_write(kv, 0, H * hw, g.slot_map, cache.k, cache.v)
        q = torch.zeros((T, H * hw), dtype=act, device=dev)
        copy(z, q, dn, src_off=0, src_stride=dn + dr, dst_off=0, dst_stride=hw)
        self.position.turn(z, q, ctx.positions, H, dr, src_off=dn, src_stride=dn + dr, dst_off=dn, dst_stride=hw)
        o = torch.empty((T, H * hw), dtype=act, device=dev)
        ops.attention(q, o, cache.k, cache.v, g.block_tables, g.tiles, H, self.scale, self.window, tiles_wide=g.tiles_wide,
                      single_rows=g.single_rows, max_context=g.max_context)
        if hw != dv:
            packed = torch.empty((T, self.o_width), dtype=act, device=dev)
            copy(o, packed, dv, src_off=0, src_stride=hw, dst_off=0, dst_stride=dv)
            o = packed
        og = o
        if self.gated:
            og = torch.empty((T, self.o_width), dtype=act, device=dev)
            ops.gated(o, z[:, gate:], "sigmoid", og)
        if accumulate_into is None:
            return self.out(og, out_dtype=torch.float32)
        self.out(og, residual=accumulate_into)


def distance_buckets(n_distances: int, n_buckets: int, far: float):
    """The bucket of every distance 0 .. n_distances - 1: a bucket each below half the buckets; from there on the buckets are
    spaced evenly in the logarithm of the distance up to `far`; the last bucket takes everything beyond."""
    half = n_buckets // 2
    out = []
    for n in range(n_distances):
        if n < half or half == 0:
            out.append(min(n, n_buckets - 1))
        else:
            out.append(min(n_buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (n_buckets - half)))))
    return out


@MIXERS.register("chunk_attention")
class ChunkAttention(Part):
    """Causal softmax attention inside chunks, without a rotation, whose values are the keys' projection.

    q = W_q h and k = W_k h are each normed as one vector over all heads (x / sqrt(mean(x^2) + eps) times a weight per
    entry); the values are k as projected, before that norm.  score(i, j) = q_i . k_j * scale * temp[head] + rel[bucket(i - j),
    head], with `distance_buckets` over the table's rows; position i reads j <= i of its own run of `chunk` positions
    (runs counted from the sequence's position 0); a sink (score 0, no value) stands under the softmax if `sink`.
    Query head a reads key head a // (n_heads // n_kv_heads).  Then the output projection.

    The temperature rides on the queries' norm weight; the bias is a table by distance, made once (a row sees distances
    below `chunk` only), that the attention kernels add to the scaled score."""
    graph_safe = True
    returns_rows = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: float, chunk: int, n_buckets: int,
                 bias_far: float, eps: float, names: dict, sink: bool = True):
        """names: q, k, o (matrices); q_norm, k_norm (vectors over all heads); rel [n_buckets, heads]; temp [heads]."""
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"chunk_attention: {n_heads} heads cannot share {n_kv_heads} key heads")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"chunk_attention: head size {head_dim}: the attention kernels take head sizes up to 256")
        if chunk < 1 or n_buckets < 1 or not bias_far > max(1, n_buckets // 2):
            raise ValueError(f"chunk_attention: chunk {chunk}, {n_buckets} buckets up to a distance of {bias_far}")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.scale, self.chunk, self.n_buckets, self.bias_far, self.eps = float(scale), int(chunk), int(n_buckets), float(bias_far), eps
        self.sink, self.names = bool(sink), dict(names)
        self.q_width, self.kv_width = n_heads * head_dim, n_kv_heads * head_dim
        self.proj = Linear(width, self.q_width + self.kv_width, names["q"] + "+k", None, init_std=width ** -0.5,
                           weight_sources=((names["q"], self.q_width), (names["k"], self.kv_width)))
        self.out = Linear(self.q_width, width, names["o"], None, init_std=self.q_width ** -0.5)

    def param_specs(self):
        n = self.names
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(n["q_norm"], (self.q_width,), "vector", ("normal", 1.0, 0.1)),
            ParamSpec(n["k_norm"], (self.kv_width,), "vector", ("normal", 1.0, 0.1)),
            ParamSpec(n["rel"], (self.n_buckets, self.n_heads), "vector", ("normal", 0.0, 0.5)),
            ParamSpec(n["temp"], (self.n_heads,), "vector", ("normal", 1.0, 0.2))]

    def cache_spec(self):
        return PagedKV(self.n_kv_heads, self.head_dim)

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        n = self.names
        temp = tensors[n["temp"]].to(torch.float32)
        self.q_norm = (tensors[n["q_norm"]].to(torch.float32) * temp.repeat_interleave(self.head_dim)).contiguous()
        self.k_norm = tensors[n["k_norm"]].contiguous()
        rows = torch.tensor(distance_buckets(self.chunk, self.n_buckets, self.bias_far), dtype=torch.long, device=temp.device)
        self.bias = tensors[n["rel"]].to(torch.float32)[rows].t().contiguous()      # [heads, chunk]
        self.no_freq = torch.empty(0, dtype=torch.float32, device=runtime.device)

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, dev = self.runtime.act_dtype, h.shape[0], h.device
        H, G, d, qw, kw = self.n_heads, self.n_kv_heads, self.head_dim, self.q_width, self.kv_width
        g = ctx.groups[cache.group]
        z = self.proj(h, out_dtype=torch.float32)
        # one kernel: both norms, the normed keys and the projection as values to their places in the cache
        q = ops.norm_pair_write(z, qw, self.q_norm, self.k_norm, self.eps, torch.empty((T, qw), dtype=act, device=dev), g.slot_map,
                                cache.k, cache.v, write=cache.writes)
        o = torch.empty((T, qw), dtype=act, device=dev)
        ops.attention(q, o, cache.k, cache.v, g.block_tables, g.tiles, H, self.scale, 0, tiles_wide=g.tiles_wide,
                      single_rows=g.single_rows, max_context=g.max_context, chunk=self.chunk, bias=self.bias, sink=self.sink)
        if accumulate_into is None:
            return self.out(o, out_dtype=torch.float32)
        self.out(o, residual=accumulate_into)


@MIXERS.register("parallel_mixers")
class ParallelMixers(Part):
    """Several mixers side by side that read the same rows; each result is normed over the width (without a mean, with a
    weight per column of its own) and the result is their mean.  branches: [(kind name, arguments)] of mixers that can
    return their result as rows (`returns_rows`); every branch keeps a cache or state of its own, so a LayerCall of a
    layer with this mixer lists one cache per branch."""
    returns_rows = True

    def __init__(self, width: int, eps: float, branches, norm_names):
        if len(branches) < 1 or len(branches) != len(norm_names):
            raise ValueError("parallel_mixers: a norm weight's name for every branch")
        self.width, self.eps, self.norm_names = width, eps, list(norm_names)
        self.branches = [MIXERS.make(tuple(b)) for b in branches]
        for b in self.branches:
            if not getattr(b, "returns_rows", False):
                raise TypeError(f"parallel_mixers: {type(b).__name__} cannot return its result as rows")
        self.graph_safe = all(getattr(b, "graph_safe", False) for b in self.branches)
        self.libraries = tuple(sorted({"sequence"} | {lib for b in self.branches for lib in getattr(b, "libraries", ())}))

    def cache_parts(self):
        return list(self.branches)

    def param_specs(self):
        specs = [ParamSpec(n, (self.width,), "vector", ("normal", 1.0, 0.1)) for n in self.norm_names]
        for b in self.branches:
            specs += b.param_specs()
        return specs

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        for b in self.branches:
            b.bind(tensors, runtime)
        self.norms = [tensors[n] for n in self.norm_names]

    def forward_pair(self, h, ctx, caches):
        """For two branches: -> (first result, (second result, first weight, second weight, eps)): whoever adds the
        result into the stream norms and halves both in its own kernel (ops.streams_write's `branches`); None otherwise."""
        if len(self.branches) != 2:
            return None
        a, b = (br.forward(h, ctx, cache, accumulate_into=None) for br, cache in zip(self.branches, caches))
        return a, (b, self.norms[0], self.norms[1], self.eps)

    def forward(self, h, ctx, caches, accumulate_into):
        if not isinstance(caches, (list, tuple)):
            caches = [caches]
        y = accumulate_into
        if y is None:
            y = torch.zeros((h.shape[0], self.width), dtype=torch.float32, device=h.device)
        share = 1.0 / len(self.branches)
        for b, w, cache in zip(self.branches, self.norms, caches):
            ops.rmsnorm_add(b.forward(h, ctx, cache, accumulate_into=None), w, None, share, self.eps, y)
        return y if accumulate_into is None else None
