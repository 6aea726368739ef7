"""A decoder described as data, and the model built from the description.

DecoderSpec names, layer by layer, the arrangement and the parts of each layer (for every slot
that the arrangement declares, a kind name and its arguments, looked up in the parts'
registries), and the order in which layers run: a list of LayerCall, which may name a layer
twice (its weights are shared; each call has caches of its own) or let a call read the cache
that another call writes.  What stands around the layers is described too: the token table
and a multiplier for its rows, the position encoding, the final norm, the head (tied to the token
table or a matrix of its own, with or without a bias) and what happens to its logits (a scale, a
soft cap).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import ARRANGEMENTS, KINDS, NORMS, POSITIONS, FixedState, PagedKV, Runtime
from .linear import Linear
from .positions import TokenEmbedding

PartSpec = Tuple[str, dict]   # (kind name in its registry, constructor arguments)


@dataclass
class LayerSpec:
    arrangement: str              # name in ARRANGEMENTS
    parts: Dict[str, PartSpec]    # a part for every slot that the arrangement declares (its SLOTS)


@dataclass
class LayerCall:
    layer: int                    # index into DecoderSpec.layers
    cache: Union[int, Tuple[int, ...]]   # the cache this call uses; a tuple: one for each mixer of the layer
    writes_cache: bool = True     # False: it only reads what another call wrote
    inject: Optional[str] = None  # a name in DecoderSpec.injections: done to the stream right before this call
    # the checkpoint name of a vector of i + 2 weights for call i of the run order: what goes on behind this call is the sum
    # of weight[j] * X_j, with X_0 the embedding stage's output and X_(j+1) the stream as call j left it (before its own average)
    average: Optional[str] = None

    def caches(self) -> Tuple[int, ...]:
        return (self.cache,) if isinstance(self.cache, int) else tuple(self.cache)


@dataclass
class EmbeddingTable:
    """A further table [rows, width] whose rows are added to the token and position rows in the embedding kernel.
    index: which per-row integers of the step pick its rows: "tokens" or "positions" (fields of StepContext), or "pairs":
    row (token before * pair[0] + token * pair[1]) mod pair[2], and row pair[2], the table's last, for a request's first
    token; the token before a step's first is then a state of the request (one int32), kept like a mixer's."""
    name: str                     # checkpoint name
    rows: int
    index: str = "tokens"
    scale: float = 1.0
    pair: Optional[Tuple[int, int, int]] = None     # index "pairs": (multiplier of the token before, of the token, buckets)


@dataclass
class DecoderSpec:
    vocab: int
    width: int
    max_positions: int
    token_table: str              # checkpoint name of the token table
    position: PartSpec
    layers: List[LayerSpec]
    run_order: List[LayerCall]
    final_norm: PartSpec
    head_weight: Optional[str] = None     # None: the head is the token table, transposed
    head_bias: Optional[str] = None       # a bias added to the logits
    logit_scale: float = 1.0              # the logits times this
    logit_softcap: float = 0.0            # > 0: then cap * tanh(logit / cap)
    embedding_scale: float = 1.0          # the token table's rows times this, before the position table's
    extra_embeddings: List[EmbeddingTable] = field(default_factory=list)   # added behind them, in this order
    # further tables that parts of any layer pick rows of: checkpoint name -> (rows, columns); bound into Runtime.tables
    tables: Dict[str, Tuple[int, int]] = field(default_factory=dict)
    embedding_norm: Optional[PartSpec] = None   # a norm of the embedded rows, before the first layer
    # > 0: the stream is kept as this many copies, all equal to the embedding stage's output at the start and added up
    # behind the last layer; every layer is then of an arrangement that works on copies ("multi_stream")
    streams: int = 0
    # name -> checkpoint name of a matrix [width, 2 width]: where a LayerCall names it, the stream becomes
    # W [x ; x0], x the stream as it stands and x0 the embedding stage's output (a loop's way back in)
    injections: Dict[str, str] = field(default_factory=dict)
    eos_token_ids: Tuple[int, ...] = ()
    # how checkpoints of this architecture name things
    name_prefixes: Tuple[str, ...] = ("",)
    ignore_tensors: Tuple[str, ...] = ()
    tied_tensors: Dict[str, str] = field(default_factory=dict)

    def instantiate(self) -> "DecoderModel":
        return DecoderModel(self)

    def param_specs(self) -> List[ParamSpec]:
        return self.instantiate().param_specs()


@dataclass
class CacheView:
    """What a mixer sees of the cache during one call."""
    group: int                    # index into ctx.groups
    writes: bool
    k: Optional[torch.Tensor] = None       # paged: [n_pages, Hkv, page_size, dh] of this call's cache
    v: Optional[torch.Tensor] = None       #        [n_pages, Hkv, dh, page_size]
    state: Optional[torch.Tensor] = None   # fixed state: [n_slots, *shape]


class DecoderModel:
    def __init__(self, spec: DecoderSpec):
        self.spec = spec
        self.embedding = TokenEmbedding(spec.vocab, spec.width, spec.token_table)
        self.position = POSITIONS.make(spec.position)
        for t in spec.extra_embeddings:
            if t.index not in ("tokens", "positions", "pairs"):
                raise ValueError(f"embedding table {t.name!r}: rows are picked by 'tokens', 'positions' or 'pairs', not {t.index!r}")
            if t.index == "pairs" and (t.pair is None or len(t.pair) != 3 or t.pair[2] < 1 or t.pair[2] + 1 != t.rows
                                       or min(t.pair[:2]) < 0):
                raise ValueError(f"embedding table {t.name!r}: pairs need (multiplier, multiplier, buckets) with buckets + 1 = rows")
        if len(spec.extra_embeddings) > ops.EMBED_TABLES_MAX - 2:
            raise ValueError(f"{len(spec.extra_embeddings)} further embedding tables; the kernel adds up {ops.EMBED_TABLES_MAX} in all")
        self.extra_tables = {}
        self.blocks = []
        for i, ls in enumerate(spec.layers):
            if ls.arrangement not in ARRANGEMENTS:
                raise KeyError(f"no block arrangement named {ls.arrangement!r}; known: {sorted(ARRANGEMENTS)}")
            cls = ARRANGEMENTS[ls.arrangement]
            if set(ls.parts) != set(cls.SLOTS):
                raise ValueError(f"layer {i}: arrangement {ls.arrangement!r} has the parts {sorted(cls.SLOTS)}, "
                                 f"the description gives {sorted(ls.parts)}")
            self.blocks.append(cls(**{slot: KINDS[kind].make(ls.parts[slot]) for slot, kind in cls.SLOTS.items()}))
        self.final_norm = NORMS.make(spec.final_norm)
        self.embedding_norm = NORMS.make(spec.embedding_norm) if spec.embedding_norm is not None else None
        self.injections = {name: Linear(2 * spec.width, spec.width, weight, None) for name, weight in spec.injections.items()}
        # the head: a matrix of its own, or the token table, transposed
        self.head = Linear(spec.width, spec.vocab, spec.head_weight or spec.token_table, spec.head_bias)
        self._check_run_order()
        # the states of the embedding stage (the token before, for tables picked by pairs) are caches behind the layers'
        self.pair_caches = {}
        for t in spec.extra_embeddings:
            if t.index == "pairs":
                self.pair_caches[t.name] = self.n_caches
                self.cache_specs.append(FixedState((1,), "int32"))
                self.n_caches += 1
        many = [bool(getattr(b, "multi_stream", False)) for b in self.blocks]
        if spec.streams < 0 or (spec.streams > 0) != all(many) or (spec.streams == 0 and any(many)):
            raise ValueError("DecoderSpec.streams > 0 goes with layers of a multi-stream arrangement, all of them, and only with those")
        if spec.streams > 0 and (spec.injections or spec.embedding_norm is not None or any(c.average or c.inject for c in spec.run_order)):
            raise ValueError("a stream kept as several copies has no injections, averages over depth or embedding norm")
        self.runtime = None
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.all_parts())

    # -- description ---------------------------------------------------------------------
    def _check_run_order(self):
        spec = self.spec
        if not spec.run_order:
            raise ValueError("run_order is empty")
        n_caches = max(max(c.caches()) for c in spec.run_order) + 1
        writer = [None] * n_caches        # cache -> (call, the cache's need) of the call that writes it
        for i, c in enumerate(spec.run_order):
            if not 0 <= c.layer < len(spec.layers):
                raise ValueError(f"run_order[{i}] names layer {c.layer}; there are {len(spec.layers)}")
            if c.inject is not None and c.inject not in spec.injections:
                raise ValueError(f"run_order[{i}] names the injection {c.inject!r}; known: {sorted(spec.injections)}")
            mixers = self.blocks[c.layer].mixers()
            if len(c.caches()) != len(mixers):
                raise ValueError(f"run_order[{i}] names {len(c.caches())} caches; layer {c.layer} has {len(mixers)} mixers")
            for cache, mixer in zip(c.caches(), mixers):
                cs = mixer.cache_spec()
                if cache < 0:
                    raise ValueError(f"run_order[{i}] names cache {cache}")
                if c.writes_cache:
                    if writer[cache] is not None:
                        raise ValueError(f"run_order[{i}] writes cache {cache}, which run_order[{writer[cache][0]}] writes")
                    writer[cache] = (i, cs)
                else:
                    if writer[cache] is None:
                        raise ValueError(f"run_order[{i}] reads cache {cache} before any call has written it")
                    if writer[cache][1] != cs:
                        raise ValueError(f"run_order[{i}] reads cache {cache}, whose writer keeps another kind of cache")
        if any(w is None for w in writer):
            raise ValueError("a cache index is never written")
        self.n_caches = n_caches
        self.cache_specs = [w[1] for w in writer]

    def all_parts(self):
        parts = [self.embedding, self.position]
        for b in self.blocks:
            parts += b.parts()
        parts.append(self.final_norm)
        if self.embedding_norm is not None:
            parts.append(self.embedding_norm)
        return parts

    def param_specs(self) -> List[ParamSpec]:
        specs, seen = [], set()
        for p in self.all_parts():
            for s in p.param_specs():
                if s.name in seen:
                    raise ValueError(f"two parts claim the tensor {s.name!r}")
                seen.add(s.name)
                specs.append(s)
        for t in self.spec.extra_embeddings:
            if t.name in seen:
                raise ValueError(f"two parts claim the tensor {t.name!r}")
            seen.add(t.name)
            specs.append(ParamSpec(t.name, (t.rows, self.spec.width), "table", ("normal", 0.0, 0.02)))
        for lin in self.injections.values():
            specs += lin.param_specs()
        for name, (rows, cols) in self.spec.tables.items():
            if name in seen:
                raise ValueError(f"two parts claim the tensor {name!r}")
            seen.add(name)
            specs.append(ParamSpec(name, (rows, cols), "table", ("normal", 0.0, 1.0)))
        for i, call in enumerate(self.spec.run_order):
            if call.average is not None:
                specs.append(ParamSpec(call.average, (i + 2,), "vector", ("normal", 1.0 / (i + 2), 0.1)))
        specs += [s for s in self.head.param_specs() if s.name not in seen]     # (a tied head's weight is the table's)
        return specs

    # -- binding -------------------------------------------------------------------------
    def bind(self, tensors: Dict[str, torch.Tensor], runtime: Runtime):
        self.runtime = runtime
        runtime.position = self.position          # mixers ask it to turn their queries and keys, if it does that
        runtime.tables = {name: tensors[name] for name in self.spec.tables}
        for p in self.all_parts():
            p.bind(tensors, runtime)
        self.head.bind(tensors)
        for lin in self.injections.values():
            lin.bind(tensors)
        self.extra_tables = {t.name: tensors[t.name] for t in self.spec.extra_embeddings}
        self.averages = {i: tensors[c.average] for i, c in enumerate(self.spec.run_order) if c.average is not None}
        self._one = torch.ones(1, dtype=torch.float32, device=runtime.device) if self.averages else None
        for b in self.blocks:
            after = getattr(b, "after_bind", None)     # an arrangement may make its parts ready for each other
            if after is not None:
                after()
        return self

    def weight_bytes(self, tensors=None):
        """Bytes of every weight a step reads once (the position table aside: a step reads T rows of it)."""
        total, seen = 0, set()
        def add(t):
            nonlocal total
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        for b in self.blocks:
            for p in b.parts():
                for v in vars(p).values():
                    if isinstance(v, Linear):
                        add(v.weight), add(v.bias)
                    elif isinstance(v, (torch.Tensor, ops.PackedMatrix)):
                        add(v)
        add(self.head.weight)
        add(getattr(self.final_norm, "weight", None)), add(getattr(self.final_norm, "bias", None))
        return total

    # -- the forward pass over one step's rows -------------------------------------------
    def forward(self, ctx, cache) -> torch.Tensor:
        """ctx: engine.batch.StepContext; cache: cache.storage.CacheStorage.
        -> 32-bit logits [R, vocab] at ctx.logit_rows."""
        rt = self.runtime
        order = self.spec.run_order
        kept = None
        xs = None
        if self.spec.streams:
            xs = torch.empty((self.spec.streams, ctx.T, self.spec.width), dtype=torch.float32, device=rt.device)
            x = xs[0]
        elif self.averages:
            # every call's result is kept, plane j + 1 for call j behind the embedding stage's in plane 0; a call works in
            # its own plane, which holds what went on from the call before
            kept = torch.empty((len(order) + 2, ctx.T, self.spec.width), dtype=torch.float32, device=rt.device)
            x = kept[0]
        else:
            x = torch.empty((ctx.T, self.spec.width), dtype=torch.float32, device=rt.device)
        if not self.spec.extra_embeddings:
            ops.embed(ctx.tokens, ctx.positions, self.embedding.weight, self.position.table(), x,
                      token_scale=self.spec.embedding_scale)
        else:
            parts = [(self.embedding.weight, ctx.tokens, self.spec.embedding_scale)]
            if self.position.table() is not None:
                parts.append((self.position.table(), ctx.positions, 1.0))
            for t in self.spec.extra_embeddings:
                if t.index == "pairs":
                    picked = ops.pair_rows(ctx.tokens, ctx.positions, ctx.row_start, ctx.state_slots,
                                           cache.view(self.pair_caches[t.name], True).state, t.pair[0], t.pair[1], t.pair[2],
                                           torch.empty_like(ctx.tokens))
                else:
                    picked = getattr(ctx, t.index)
                parts.append((self.extra_tables[t.name], picked, t.scale))
            ops.embed_sum(parts, x)
        rt.stream_stats = rt.stream_deferred = rt.normed_rows = None      # nobody has left anything for a norm of these rows yet
        if self.embedding_norm is not None:
            x = self.embedding_norm.forward(x, torch.float32)
        x0 = x.clone() if self.injections else None      # (the blocks add into x in place)
        if kept is not None:
            if x.data_ptr() != kept[0].data_ptr():
                kept[0].copy_(x)
            x = ops.depth_mix(kept, 1, self._one, kept[1])
        if xs is not None:
            xs[1:].copy_(x)      # (every copy starts as the embedding stage's output)
            rt.stream_rows = None
        for i, call in enumerate(order):
            if xs is not None:
                nxt = self.blocks[order[i + 1].layer] if i + 1 < len(order) else None
                rt.next_read = nxt.first_read() if nxt is not None else None
                self.blocks[call.layer].forward(xs, ctx, [cache.view(c, call.writes_cache) for c in call.caches()], rt)
                continue
            if call.inject is not None:
                if rt.stream_deferred is not None:
                    rt.stream_deferred.flush(x)
                rt.stream_stats = rt.stream_deferred = rt.normed_rows = None
                both = ops.concat_cast(x, x0, torch.empty((ctx.T, 2 * self.spec.width), dtype=rt.act_dtype, device=rt.device))
                x = self.injections[call.inject](both, out_dtype=torch.float32)
            nxt = self.blocks[order[i + 1].layer] if i + 1 < len(order) else None
            rt.next_norm = nxt.first_norm() if nxt is not None and hasattr(nxt, "first_norm") else None
            rt.next_takes_deferred = nxt is not None and getattr(nxt, "takes_deferred", False)
            block = self.blocks[call.layer]
            if rt.stream_deferred is not None and not getattr(block, "takes_deferred", False):
                rt.stream_deferred.flush(x)         # (an arrangement that knows nothing of sums left for its norm)
                rt.stream_deferred = None
            block.forward(x, ctx, [cache.view(c, call.writes_cache) for c in call.caches()], rt)
            if kept is not None:
                if rt.stream_deferred is not None:
                    rt.stream_deferred.flush(x)
                rt.stream_stats = rt.stream_deferred = rt.normed_rows = None
                if x.data_ptr() != kept[i + 1].data_ptr():      # (an injection made new rows)
                    kept[i + 1].copy_(x)
                w = self.averages.get(i)
                x = ops.depth_mix(kept, i + 2, w, kept[i + 2]) if w is not None else ops.depth_mix(kept[i + 1:], 1, self._one, kept[i + 2])
        if rt.stream_deferred is not None:
            rt.stream_deferred.flush(x)
        rt.stream_stats = rt.next_norm = rt.stream_deferred = rt.normed_rows = None
        rt.next_takes_deferred = False
        if ctx.R == 0:
            return torch.empty((0, self.spec.vocab), dtype=torch.float32, device=rt.device)
        if xs is not None:
            # the copies are added up; a norm without a mean runs in the same kernel, on the wanted rows alone
            fn = self.final_norm
            if getattr(fn, "kind_name", None) == "rmsnorm":
                h = ops.streams_read(xs, None, fn.weight, fn.eps, torch.empty((ctx.R, self.spec.width), dtype=rt.act_dtype, device=rt.device),
                                     rows=ctx.logit_rows)
            else:
                x = ops.streams_read(xs, None, None, None, torch.empty((ctx.T, self.spec.width), dtype=torch.float32, device=rt.device))
                h = fn.forward(x, rt.act_dtype, rows=ctx.logit_rows, packed=self.head.packed_input(ctx.R))
        else:
            h = self.final_norm.forward(x, rt.act_dtype, rows=ctx.logit_rows, packed=self.head.packed_input(ctx.R))
        logits = self.head(h, out_dtype=torch.float32)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap > 0:
            ops.logits_post(logits, self.spec.logit_scale, self.spec.logit_softcap)
        return logits
