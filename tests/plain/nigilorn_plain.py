"""A plain, slow Nigilorn: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Every function works on one sequence, [tokens, ...] torch tensors on
the CPU, in the precision of the tensors it is given (float32, or float64 to see how much of a
difference is rounding).  Weights come as a dict from tensor name to tensor; `cfg` is config.json as a
dict.

Notation: T tokens, W the model's width, H heads, G key heads; `p(name)` is a layer's tensor.
"""
from __future__ import annotations

import math

import torch


# ----------------------------------------------------------------------------
# small pieces
# ----------------------------------------------------------------------------

def rms_norm(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) [* weight], over the last dimension."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_taps(x, w, b):
    """x [T, C], w [C, taps], b [C]: y_t = b + sum_j w[:, j] x_(t - taps + 1 + j); the last column weighs the token
    itself; nothing before the first token."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x) + b
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def yarn_frequencies(dims, base, scaling):
    """-> (frequency per pair [dims / 2], the factor on cos and sin), in 64-bit.  Pair i turns by position * f_i with
    f_i = base^(-2i/dims); with scaling (factor, original, fast, slow) the pairs that turn slowly are slowed down by
    `factor`, the fast ones stay, and a ramp over the pair's index blends the two between."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):     # the (fractional) dimension whose pair makes `turns` turns over the original length
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_pairs(x, positions, rot):
    """x [T, n, d]: of each vector's first rot.dims entries, entry 2i and 2i+1 are turned by the angle
    position * frequency_i (cos and sin times the scaling's factor); the rest stay."""
    dims = int(rot["dims"])
    out = x.clone()
    if dims == 0:
        return out
    freq, mag = yarn_frequencies(dims, rot["base"], rot.get("scaling"))
    ang = positions.to(torch.float64)[:, None] * freq[None, :]
    cos, sin = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def window_softmax(scores, window):
    """scores [H, T, T] (query, key): a query at i sees keys j with 0 <= i - j < window (window 0 or None: all before it)."""
    T = scores.shape[-1]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) if not window else ((j <= i) & (i - j < window))
    return torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)


# ----------------------------------------------------------------------------
# mixers
# ----------------------------------------------------------------------------

def mamba1(h, p, m):
    """Selective scan.  W_in h = [x | z]; x through a causal convolution per channel with a bias and silu; W_x x =
    [dt_low | B | C]; dt = softplus(W_dt dt_low + b); A = -exp(A_log).  Per channel c and state n:
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;  y_c = sum_n S[c, n] C_n + D_c x_c;  then y * silu(z), W_o."""
    T = h.shape[0]
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ p("in").T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_taps(x, p("conv"), p("conv.b")))
    low = x @ p("x").T
    dt = softplus(low[:, :R] @ p("dt").T + p("dt.b"))
    B, C = low[:, R:R + N], low[:, R + N:R + 2 * N]
    A = -torch.exp(p("A_log"))
    S = torch.zeros(inner, N, dtype=h.dtype)
    y = torch.zeros(T, inner, dtype=h.dtype)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + p("D") * x[t]
    return (y * silu(z)) @ p("o").T


def attention(h, p, m, eps):
    """Grouped key heads, part of each head turned by the position, q and k divided by their root mean square per head
    behind the turn, a window, softmax, a gate per head, the output projection."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ p("q").T).view(T, H, d)
    k = (h @ p("k").T).view(T, G, d)
    v = (h @ p("v").T).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        q, k = turn_pairs(q, pos, rot), turn_pairs(k, pos, rot)
    q, k = rms_norm(q, None, eps), rms_norm(k, None, eps)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    w = window_softmax(scores, (m.get("mask") or {}).get("size"))
    o = torch.einsum("hij,jhd->ihd", w, v)
    gate = torch.sigmoid(h @ p("g").T)                  # [T, H]
    return (o * gate[:, :, None]).reshape(T, H * dv) @ p("o").T


def latent_attention(h, p, m, eps):
    """Keys and values from one small vector per token: c = norm(first kv_rank rows of W_dkv h); a turned key part shared
    by all heads; per head k = [W_uk c | shared part], v = W_uv c, q = [plain | turned]."""
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    rot = dict(m["rot"], dims=dr)
    q = (h @ p("q").T).view(T, H, d + dr)
    q_plain, q_turn = q[..., :d], turn_pairs(q[..., d:], pos, rot)
    low = h @ p("dkv").T
    c = rms_norm(low[:, :r], p("dkv.norm"), eps)
    k_turn = turn_pairs(low[:, None, r:], pos, rot)[:, 0]          # [T, dr], one for all heads
    k_plain = (c @ p("uk").T).view(T, H, d)
    v = (c @ p("uv").T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_turn, k_turn)) * m["scale"]
    w = window_softmax(scores, (m.get("mask") or {}).get("size"))
    o = torch.einsum("hij,jhd->ihd", w, v)
    return o.reshape(T, H * dv) @ p("o").T


# ----------------------------------------------------------------------------
# feed-forwards
# ----------------------------------------------------------------------------

def dense_ff(h, p):
    return (silu(h @ p("gate").T) * (h @ p("up").T)) @ p("down").T


def expert(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def choose_experts(s, top, n_groups, keep):
    """s [E] scores of one token -> the chosen experts, best first.  The experts are n_groups equal runs of neighbours; a
    group's score is the sum of its two largest; only experts of the `keep` best groups can be chosen."""
    E = s.shape[0]
    per = E // n_groups
    allowed = torch.ones(E, dtype=torch.bool)
    if n_groups > 1:
        gs = torch.stack([s[g * per:(g + 1) * per].topk(min(2, per)).values.sum() for g in range(n_groups)])
        allowed[:] = False
        for g in gs.topk(keep).indices.tolist():
            allowed[g * per:(g + 1) * per] = True
    masked = torch.where(allowed, s, torch.full_like(s, float("-inf")))
    return masked.topk(top).indices


def moe_ff(h, p, mlp):
    T = h.shape[0]
    ro = mlp["router"]
    groups = ro.get("groups") or {"count": 1, "keep": 1}
    s = torch.sigmoid((h @ p("router").T).float())
    y = torch.zeros_like(h)
    for t in range(T):
        ids = choose_experts(s[t], ro["top"], groups["count"], groups["keep"])
        w = s[t][ids]
        w = w / (w.sum() + 1e-20) * ro.get("scale", 1.0)
        for e, we in zip(ids.tolist(), w):
            y[t] += we.to(h.dtype) * expert(h[t], p(f"e{e}.up"), p(f"e{e}.down"))
    if mlp.get("shared"):
        y = y + expert(h, p("shared.up"), p("shared.down"))
    return y


# ----------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------

def layer_forward(x, tokens, i, layer, cfg, w):
    eps = cfg["norm"]["eps"]
    lp = lambda name: w[f"l{i}.{name}"]                      # noqa: E731
    mp = lambda name: w[f"l{i}.mix.{name}"]                  # noqa: E731
    fp = lambda name: w[f"l{i}.mlp.{name}"]                  # noqa: E731
    h = rms_norm(x, lp("norm1"), eps)
    kind, m = layer["type"], layer["mixer"]
    if kind == "mamba1":
        y = mamba1(h, mp, m)
    elif kind == "attention":
        y = attention(h, mp, m, eps)
    elif kind == "latent_attention":
        y = latent_attention(h, mp, m, eps)
    else:
        raise ValueError(kind)
    y = y * torch.sigmoid(h @ lp("rg1").T + lp("rg1.b"))
    x = x + rms_norm(y, lp("norm1b"), eps)
    mlp = layer.get("mlp")
    if mlp is not None:
        h = rms_norm(x, lp("norm2"), eps)
        y = dense_ff(h, fp) if mlp["kind"] == "dense" else moe_ff(h, fp, mlp)
        y = y * torch.sigmoid(h @ lp("rg2").T + lp("rg2.b"))
        x = x + rms_norm(y, lp("norm2b"), eps)
    side = cfg.get("token_side")
    if side:
        d = side["dim"]
        e = w["side.embed"][tokens][:, i * d:(i + 1) * d]
        g = gelu_tanh(x @ lp("side.gate").T) * e
        x = x + rms_norm(g @ lp("side.proj").T, lp("side.norm"), eps)
    return x


def forward(tokens, cfg, w, return_layers=False):
    """tokens: list of ints -> logits [T, vocab] (and the stream behind every layer)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tokens]
    layers = []
    for i, layer in enumerate(cfg["layers"]):
        x = layer_forward(x, tokens, i, layer, cfg, w)
        layers.append(x)
    logits = rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
    return (logits, layers) if return_layers else logits
