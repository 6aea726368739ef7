"""Nigilorn: a decoder whose layers choose among three mixers (a selective scan, attention in a window with grouped key
heads, latent attention in a window), with a norm on both sides of every sublayer, a gate on every sublayer's result and
a second way in for the token behind every layer.

config.json: `vocab`, `width`, `norm.eps`, `token_side.dim` (optional: without it no layer has a token input), `layers`
(each: `type`, `mixer` with the mixer's sizes and constants, `mlp` or null).  Optional: `max_positions` (the engine's limit
on a request's length; the architecture itself has none).

The model: x = embed[token].  Layer i, with h = norm1(x): x += norm1b(mixer(h) * sigmoid(rg1 h + b)); then, if it has a
feed-forward, with h = norm2(x): x += norm2b(ff(h) * sigmoid(rg2 h + b)); then e = side.embed[token][i * dim : (i + 1) * dim],
y = side.proj (gelu_tanh(side.gate x) * e), x += y / rms(y) * side.norm.  All norms are root-mean-square norms with a
weight.  Behind the last layer the final norm and the head, a matrix of its own.

Mixers: "mamba1" (parts.recurrent.Mamba1), "attention" (parts.mixers.CausalSelfAttention: grouped key heads, values of a
width of their own, pairs of the first rot.dims dimensions turned by the position with a scaled encoding, q and k divided
by their root mean square per head behind the turn, the score's scale from config.json, a window, a gate per head) and
"latent_attention" (parts.mixers.LatentAttention without its gate, with a window).  Feed-forwards: "dense"
(parts.feedforward.GatedMLP) and "moe" (parts.feedforward.RoutedExperts: sigmoid scores, groups of experts of which the
best are kept, the chosen scores divided by their sum and times router.scale, experts of max(W_up h, 0)^2 without biases,
a shared expert of the same form that every token uses).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from ..config.base import ConfigError, read_float, read_int, read_str
from ..config.registry import register_architecture
from ..parts.model import DecoderSpec, LayerCall, LayerSpec

MIXER_TYPES = ("mamba1", "attention", "latent_attention")
DEFAULT_MAX_POSITIONS = 65536


def _sub(d, key, where="config.json"):
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object")
    return v


def _read_rot(m, where, widest):
    """mixer.rot: base, dims, and optionally scaling (factor, original, fast, slow)."""
    rot = _sub(m, "rot", where)
    base = read_float(rot, "base")
    dims = read_int(rot, "dims", minimum=0)
    if dims % 2 or dims > widest:
        raise ConfigError(f"{where}.rot.dims = {dims}: an even number up to {widest}")
    if rot.get("scaling") is not None:
        sc = _sub(rot, "scaling", where + ".rot")
        factor, original = read_float(sc, "factor"), read_float(sc, "original")
        fast, slow = read_float(sc, "fast"), read_float(sc, "slow")
        if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and base > 1):
            raise ConfigError(f"{where}.rot.scaling: factor, original, fast and slow must be positive, and rot.base above 1")


def _read_window(m, where):
    if m.get("mask") is not None:
        read_int(_sub(m, "mask", where), "size", minimum=1)


@dataclass(frozen=True)
class NigilornConfig:
    raw: dict

    architecture = "Nigilorn"

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
    def side_dim(self):
        side = self.raw.get("token_side")
        return int(side["dim"]) if side else 0

    @property
    def max_positions(self):
        return self.raw.get("max_positions") or DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "NigilornConfig":
        raw = copy.deepcopy({k: v for k, v in d.items() if k not in ("architectures", "torch_dtype")})
        read_int(raw, "vocab", minimum=1), read_int(raw, "width", minimum=1)
        read_float(_sub(raw, "norm"), "eps")
        read_int(raw, "max_positions", default=None, minimum=1)
        if raw.get("token_side") is not None:
            read_int(_sub(raw, "token_side"), "dim", minimum=1)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: key 'layers' must be a list of layers")
        for i, layer in enumerate(layers):
            where = f"config.json: layers[{i}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"{where} must be an object")
            kind = read_str(layer, "type", choices=MIXER_TYPES)
            m = _sub(layer, "mixer", where)
            wm = where + ".mixer"
            if kind == "mamba1":
                read_int(m, "inner", minimum=1), read_int(m, "dt_rank", minimum=1), read_int(m, "conv", minimum=1)
                if read_int(m, "state", minimum=1) > 256:
                    raise ConfigError(f"{wm}.state = {m['state']}: the scan keeps up to 256 states a channel")
            else:
                heads = read_int(m, "heads", minimum=1)
                dim = read_int(m, "dim", minimum=1)
                read_int(m, "vdim", minimum=1), read_float(m, "scale")
                _read_window(m, wm)
                if kind == "attention":
                    kv = read_int(m, "kv_heads", minimum=1)
                    if heads % kv != 0:
                        raise ConfigError(f"{wm}: heads ({heads}) is no multiple of kv_heads ({kv})")
                    if m.get("rot") is not None:
                        _read_rot(m, wm, dim)
                else:
                    rot_dim = read_int(m, "rot_dim", minimum=2)
                    read_int(m, "kv_rank", minimum=1)
                    _read_rot(m, wm, rot_dim)
                    if rot_dim % 2:
                        raise ConfigError(f"{wm}.rot_dim = {rot_dim}: the turned part is made of pairs")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict):
                    raise ConfigError(f"{where}.mlp must be an object or null")
                if read_str(mlp, "kind", choices=("dense", "moe")) == "dense":
                    read_int(mlp, "ff", minimum=1)
                else:
                    read_int(_sub(mlp, "expert", where + ".mlp"), "ff", minimum=1)
                    ro = _sub(mlp, "router", where + ".mlp")
                    n, top = read_int(ro, "experts", minimum=1), read_int(ro, "top", minimum=1)
                    read_float(ro, "scale", default=1.0)
                    groups, keep = 1, 1
                    if ro.get("groups") is not None:
                        gr = _sub(ro, "groups", where + ".mlp.router")
                        groups, keep = read_int(gr, "count", minimum=1), read_int(gr, "keep", minimum=1)
                    if n % groups or keep > groups or top > keep * (n // groups):
                        raise ConfigError(f"{where}.mlp.router: {n} experts in {groups} groups of which {keep} are kept cannot "
                                          f"give {top} choices")
                    if mlp.get("shared") is not None:
                        read_int(_sub(mlp, "shared", where + ".mlp"), "ff", minimum=1)
        return cls(raw)

    def to_dict(self) -> dict:
        d = copy.deepcopy(self.raw)
        d["architecture"] = self.architecture
        return d


def _rotation(rot, dims, head_dim):
    return dict(dims=dims, base=rot["base"], head_dim=head_dim, scaling=rot.get("scaling"))


def _mixer(cfg: NigilornConfig, i: int, layer: dict):
    m, p, W = layer["mixer"], f"l{i}.mix.", cfg.width
    if layer["type"] == "mamba1":
        names = {s: p + s for s in ("in", "x", "dt", "o", "conv", "A_log", "D")}
        names.update(conv_bias=p + "conv.b", dt_bias=p + "dt.b")
        return ("mamba1", dict(width=W, inner=m["inner"], state_dim=m["state"], dt_rank=m["dt_rank"], taps=m["conv"], names=names))
    window = (m.get("mask") or {}).get("size", 0)
    if layer["type"] == "attention":
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        rot = m.get("rot")
        return ("causal_attention", dict(
            width=W, n_heads=H, n_kv_heads=G, head_dim=dk, value_dim=dv, scale=m["scale"], window=window, exact_turn=True,
            unit_eps=cfg.eps, head_gate=p + "g", qkv_weight=p + "q+k+v+g", qkv_bias=None, out_weight=p + "o", out_bias=None,
            qkv_weight_sources=((p + "q", H * dk), (p + "k", G * dk), (p + "v", G * dv)),
            position=("rotary_pairs", _rotation(rot, rot["dims"], dk)) if rot else None))
    names = {s: p + s for s in ("q", "dkv", "uk", "uv", "o")}
    names["dkv_norm"] = p + "dkv.norm"
    return ("latent_attention", dict(
        width=W, n_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], value_dim=m["vdim"], kv_rank=m["kv_rank"],
        scale=m["scale"], eps=cfg.eps, window=window, names=names,
        position={k: v for k, v in _rotation(m["rot"], m["rot_dim"], m["rot_dim"]).items() if k != "head_dim"}))


def _feed_forward(cfg: NigilornConfig, i: int, mlp):
    p, W = f"l{i}.mlp.", cfg.width
    if mlp is None:
        return ("none", {})
    if mlp["kind"] == "dense":
        return ("gated_mlp", dict(width=W, inner=mlp["ff"], gate_weight=p + "gate", up_weight=p + "up", down_weight=p + "down"))
    ro = mlp["router"]
    groups = ro.get("groups") or {"count": 1, "keep": 1}
    sh = mlp.get("shared")
    shared = dict(inner=sh["ff"], gate=None, up=p + "shared.up", down=p + "shared.down", token_gate=None) if sh else None
    return ("routed_experts", dict(
        width=W, inner=mlp["expert"]["ff"], n_experts=ro["experts"], top=ro["top"], router=p + "router", correction=None,
        gate=None, up=p + "e{e}.up", down=p + "e{e}.down", score="sigmoid", renorm=True, weigh="output", act="relu2",
        shared=shared, groups=groups["count"], keep=groups["keep"], route_scale=float(ro.get("scale", 1.0))))


def build_nigilorn(cfg: NigilornConfig) -> DecoderSpec:
    W, dim = cfg.width, cfg.side_dim
    n_layers = len(cfg.layers)

    def norm(name):
        return ("rmsnorm", dict(width=W, eps=cfg.eps, weight_name=name))

    def post(name):
        return ("rmsnorm_into_stream", dict(width=W, eps=cfg.eps, weight_name=name))

    def gate(name):
        return ("sigmoid_linear", dict(width=W, out_width=W, weight_name=name, bias_name=name + ".b"))
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        side = ("gated_table_rows", dict(width=W, dim=dim, table="side.embed", offset=i * dim, eps=cfg.eps, gate=p + "side.gate",
                                         proj=p + "side.proj", norm=p + "side.norm")) if dim else ("none", {})
        has_ff = layer.get("mlp") is not None
        layers.append(LayerSpec(arrangement="gated_sandwich", parts=dict(
            norm1=norm(p + "norm1"), mixer=_mixer(cfg, i, layer), gate1=gate(p + "rg1"), post1=post(p + "norm1b"),
            norm2=norm(p + "norm2"), ffn=_feed_forward(cfg, i, layer.get("mlp")), gate2=gate(p + "rg2") if has_ff else ("none", {}),
            post2=post(p + "norm2b"), side=side)))
    order = [LayerCall(layer=i, cache=i) for i in range(n_layers)]
    return DecoderSpec(
        vocab=cfg.vocab, width=W, max_positions=cfg.max_positions, token_table="embed", position=("none", {}),
        layers=layers, run_order=order, final_norm=norm("final.norm"), head_weight="head",
        tables={"side.embed": (cfg.vocab, n_layers * dim)} if dim else {},
        # (a layer without a feed-forward has no use for its second pair of norms and its second gate, whether or not a file holds them)
        ignore_tensors=tuple(rf"^l{i}\.(norm2|norm2b|rg2|rg2\.b)$" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None))


register_architecture(["Nigilorn"], NigilornConfig, build_nigilorn)
