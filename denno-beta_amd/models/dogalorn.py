"""Dogalorn: a decoder whose layers are either two mixers side by side (attention in chunks beside a gated recurrence of
single numbers) or a state-space mixer, on a stream that is kept as several copies, with token rows that the pair (token
before, token) adds to.

config.json: `vocab`, `width`, `norm.eps`, `layers` (each: `type`, `mixer` with the mixer's sizes and constants, `mlp` or
null, and optionally `weights_of`: the layer has no tensors of its own and runs with those of the layer named, on a cache
and state of its own).  Optional: `streams` (the number of copies of the stream; absent: one stream with plain residual
sums), `embedding.bigram` (`buckets`, `mul_prev`, `mul_cur`; absent: token rows alone), `logit_scale` (absent: 1),
`max_positions` (the engine's limit on a request's length; the architecture itself has none).  The number of rows of an
attention's table of distance biases is not in config.json: the tensor gives it by its shape (`with_shapes`); weights
made here take it from the mixer's entry `bias_buckets`, or 16.

The model: x = embed[token] + bigram[(token before * mul_prev + token * mul_cur) mod buckets], the table's last row for a
sequence's first token.  All norms are x / sqrt(mean(x^2) + eps) * g with g one number.  A layer: x += mixer(norm1(x)), then,
if it has a feed-forward, x += ff(norm2(x)); with `streams` copies x_1 .. x_n instead, for sublayer q with the layer's
tensors hc<q>.in / out / mix: u = sum_s in[s] x_s; y = sublayer(norm(u)); x_t <- sum_s mix[s, t] x_s + out[t] y for all t at
once, and behind the last layer x is the sum of the copies.  Then the model's norm, the head, and the logits times
`logit_scale`.

Mixers: "parallel" (parts.mixers.ParallelMixers over parts.mixers.ChunkAttention, tensors under `left`, and
parts.recurrent.MinGRU, tensors under `right`) and "mamba2" (parts.recurrent.Mamba2).  Feed-forward: "dense"
(parts.feedforward.DenseMLP with the erf GELU and biases).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from ..config.base import ConfigError, read_float, read_int, read_str
from ..config.registry import register_architecture
from ..parts.model import DecoderSpec, EmbeddingTable, LayerCall, LayerSpec

LAYER_TYPES = ("parallel", "mamba2")
DEFAULT_MAX_POSITIONS = 65536
DEFAULT_BIAS_BUCKETS = 16       # for weights made here; a checkpoint's own table says its rows


def _sub(d, key, where="config.json"):
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object")
    return v


def _check_layer(i, layer, layers):
    where = f"config.json: layers[{i}]"
    if not isinstance(layer, dict):
        raise ConfigError(f"{where} must be an object")
    kind = read_str(layer, "type", choices=LAYER_TYPES)
    m = _sub(layer, "mixer", where)
    if kind == "parallel":
        left, right = _sub(m, "left", where + ".mixer"), _sub(m, "right", where + ".mixer")
        heads, kv = read_int(left, "heads", minimum=1), read_int(left, "kv_heads", minimum=1)
        if heads % kv != 0:
            raise ConfigError(f"{where}.mixer.left: heads ({heads}) is no multiple of kv_heads ({kv})")
        dim = read_int(left, "dim", minimum=1)
        if read_int(left, "vdim", default=dim, minimum=1) != dim:
            raise ConfigError(f"{where}.mixer.left: the values are the keys' projection, so vdim ({left['vdim']}) must equal dim ({dim})")
        read_float(left, "scale"), read_float(left, "bias_max")
        read_int(_sub(left, "mask", where + ".mixer.left"), "size", minimum=1)
        read_int(left, "bias_buckets", default=None, minimum=1)
        read_int(right, "width", minimum=1)
    else:
        heads, groups = read_int(m, "heads", minimum=1), read_int(m, "groups", minimum=1)
        if heads % groups != 0:
            raise ConfigError(f"{where}.mixer: heads ({heads}) is no multiple of groups ({groups})")
        vdim = read_int(m, "vdim", minimum=1)
        read_int(m, "state", minimum=1), read_int(m, "conv", minimum=1)
        parts = read_int(m, "norm_groups", minimum=1)
        if (heads * vdim) % parts != 0:
            raise ConfigError(f"{where}.mixer: heads * vdim ({heads * vdim}) is no multiple of norm_groups ({parts})")
    mlp = layer.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict):
            raise ConfigError(f"{where}.mlp must be an object or null")
        read_str(mlp, "kind", choices=("dense",))
        read_int(mlp, "ff", minimum=1)
    src = read_int(layer, "weights_of", default=None, minimum=0)
    if src is not None:
        if src >= len(layers) or src == i or not isinstance(layers[src], dict) or layers[src].get("weights_of") is not None:
            raise ConfigError(f"{where}.weights_of = {src}: it must name another layer, one with tensors of its own")
        if layers[src].get("type") != kind or (layers[src].get("mlp") is None) != (mlp is None):
            raise ConfigError(f"{where}: a layer that runs with layer {src}'s tensors is of that layer's type, with or without a feed-forward as it")


@dataclass(frozen=True)
class DogalornConfig:
    raw: dict

    architecture = "Dogalorn"

    @property
    def vocab(self):
        return self.raw["vocab"]

    @property
    def width(self):
        return self.raw["width"]

    @property
    def eps(self):
        return float(self.raw["norm"]["eps"])

    @property
    def layers(self):
        return self.raw["layers"]

    @property
    def streams(self):
        return self.raw.get("streams") or 0

    @property
    def max_positions(self):
        return self.raw.get("max_positions") or DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "DogalornConfig":
        raw = copy.deepcopy({k: v for k, v in d.items() if k not in ("architectures", "torch_dtype")})
        read_int(raw, "vocab", minimum=1), read_int(raw, "width", minimum=1)
        read_float(_sub(raw, "norm"), "eps")
        read_int(raw, "streams", default=None, minimum=1)
        read_float(raw, "logit_scale", default=1.0)
        read_int(raw, "max_positions", default=None, minimum=1)
        emb = raw.get("embedding")
        if emb is not None:
            if not isinstance(emb, dict):
                raise ConfigError("config.json: key 'embedding' must be an object")
            if emb.get("bigram") is not None:
                bg = _sub(emb, "bigram", "config.json: embedding")
                read_int(bg, "buckets", minimum=1), read_int(bg, "mul_prev", minimum=0), read_int(bg, "mul_cur", minimum=0)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: key 'layers' must be a list of layers")
        for i, layer in enumerate(layers):
            _check_layer(i, layer, layers)
        return cls(raw)

    def with_shapes(self, shapes: dict) -> "DogalornConfig":
        """Sizes that config.json leaves to the tensors: the rows of an attention's table of distance biases."""
        raw = copy.deepcopy(self.raw)
        for i, layer in enumerate(raw["layers"]):
            if layer["type"] != "parallel":
                continue
            src = i if layer.get("weights_of") is None else layer["weights_of"]
            shape = shapes.get(f"l{src}.mix.left.rel")
            if shape is not None and len(shape) == 2:
                layer["mixer"]["left"]["bias_buckets"] = int(shape[0])
        return DogalornConfig(raw)

    def to_dict(self) -> dict:
        d = copy.deepcopy(self.raw)
        d["architecture"] = self.architecture
        return d


def _mixer(cfg: DogalornConfig, i: int, layer: dict):
    m, p, W = layer["mixer"], f"l{i}.mix.", cfg.width
    if layer["type"] == "mamba2":
        names = {s: p + s for s in ("in", "o", "conv", "dt_bias", "A_log", "D", "norm")}
        names["conv_bias"] = p + "conv.b"
        return ("mamba2", dict(width=W, n_heads=m["heads"], value_dim=m["vdim"], state_dim=m["state"], n_groups=m["groups"],
                               taps=m["conv"], norm_groups=m["norm_groups"], eps=cfg.eps, names=names))
    left, right = m["left"], m["right"]
    lp, rp = p + "left.", p + "right."
    attention = ("chunk_attention", dict(
        width=W, n_heads=left["heads"], n_kv_heads=left["kv_heads"], head_dim=left["dim"], scale=left["scale"],
        chunk=left["mask"]["size"], n_buckets=left.get("bias_buckets") or DEFAULT_BIAS_BUCKETS, bias_far=left["bias_max"],
        eps=cfg.eps, sink=True,
        names=dict(q=lp + "q", k=lp + "k", o=lp + "o", q_norm=lp + "q.norm", k_norm=lp + "k.norm", rel=lp + "rel", temp=lp + "temp")))
    gru = ("min_gru", dict(width=W, inner=right["width"],
                           names=dict(z=rp + "z", x=rp + "x", g=rp + "g", o=rp + "o", z_bias=rp + "z.b", x_bias=rp + "x.b")))
    return ("parallel_mixers", dict(width=W, eps=cfg.eps, branches=[attention, gru], norm_names=[lp + "out", rp + "out"]))


def _feed_forward(cfg: DogalornConfig, i: int, mlp):
    if mlp is None:
        return ("none", {})
    p = f"l{i}.mlp."
    return ("dense_mlp", dict(width=cfg.width, inner=mlp["ff"], activation="gelu_erf", up_weight=p + "up", up_bias=p + "up.b",
                              down_weight=p + "down", down_bias=p + "down.b"))


def build_dogalorn(cfg: DogalornConfig) -> DecoderSpec:
    W, n = cfg.width, cfg.streams

    def norm(name):
        return ("rmsnorm", dict(width=W, eps=cfg.eps, weight_name=name, one_weight=True))

    # layers with tensors of their own become the model's layers; a layer that names another's runs that one again
    own, layers, ignore = {}, [], []
    for i, layer in enumerate(cfg.layers):
        if layer.get("weights_of") is not None:
            continue
        p = f"l{i}."
        parts = dict(norm1=norm(p + "norm1"), mixer=_mixer(cfg, i, layer), norm2=norm(p + "norm2"),
                     ffn=_feed_forward(cfg, i, layer.get("mlp")))
        if n:
            parts.update(hc1=("stream_mixer", dict(n_streams=n, in_name=p + "hc1.in", out_name=p + "hc1.out", mix_name=p + "hc1.mix")),
                         hc2=("stream_mixer", dict(n_streams=n, in_name=p + "hc2.in", out_name=p + "hc2.out", mix_name=p + "hc2.mix")))
        if layer.get("mlp") is None:      # (no use for the second sublayer's tensors, whether or not a file holds them)
            ignore.append(rf"^l{i}\.(norm2|hc2\.(in|out|mix))$")
        own[i] = len(layers)
        layers.append(LayerSpec(arrangement="multi_stream" if n else "pre_norm_plain", parts=parts))
    order, caches = [], 0
    for i, layer in enumerate(cfg.layers):
        src = layer.get("weights_of")
        k = 2 if layer["type"] == "parallel" else 1
        order.append(LayerCall(layer=own[i if src is None else src], cache=tuple(range(caches, caches + k)) if k > 1 else caches))
        caches += k
    bg = (cfg.raw.get("embedding") or {}).get("bigram")
    tables = [EmbeddingTable("bigram", bg["buckets"] + 1, index="pairs", pair=(bg["mul_prev"], bg["mul_cur"], bg["buckets"]))] if bg else []
    return DecoderSpec(
        vocab=cfg.vocab, width=W, max_positions=cfg.max_positions, token_table="embed", position=("none", {}),
        layers=layers, run_order=order, final_norm=norm("final.norm"), head_weight="head",
        logit_scale=1.0 if cfg.raw.get("logit_scale") is None else float(cfg.raw["logit_scale"]), extra_embeddings=tables, streams=n, ignore_tensors=tuple(ignore))


register_architecture(["Dogalorn"], DogalornConfig, build_dogalorn)
