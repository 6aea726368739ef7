"""A plain, slow Dogalorn: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Every function works on one sequence, [tokens, ...] torch tensors on
the CPU, in the precision of the tensors it is given (float32, or float64 to see how much of a
difference is rounding).  Weights come as a dict from tensor name to tensor; `cfg` is config.json as a
dict.

Notation: T tokens, W the model's width, H query heads, G key heads, d a head's size, N a state's size.
"""
from __future__ import annotations

import math

import torch


# ----------------------------------------------------------------------------
# small pieces
# ----------------------------------------------------------------------------

def rms_norm(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) [* weight], over the last dimension; weight a vector or one number."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def causal_taps(x, w, b):
    """x [T, C], w [C, taps], b [C]: y_t = b + sum_j w[:, j] x_(t - taps + 1 + j); the last column weighs the token itself;
    nothing before the first token."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x) + b
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


# ----------------------------------------------------------------------------
# embedding: token rows plus rows picked by the pair (token before, token)
# ----------------------------------------------------------------------------

def pair_rows(tokens, mul_prev, mul_cur, buckets):
    """Row of the pair table for every token: (prev * mul_prev + cur * mul_cur) mod buckets; the first token has no
    token before it and takes the table's last row, number `buckets`."""
    rows = []
    for t, cur in enumerate(tokens):
        rows.append(buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(cur) * mul_cur) % buckets)
    return rows


def embed(cfg, w, tokens):
    x = w["embed"][torch.tensor(tokens)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + w["bigram"][torch.tensor(pair_rows(tokens, bg["mul_prev"], bg["mul_cur"], bg["buckets"]))]
    return x


# ----------------------------------------------------------------------------
# attention in chunks, with a bias by distance and a sink
# ----------------------------------------------------------------------------

def distance_bucket(n, n_buckets, far):
    """Distances below half the buckets have a bucket each; from there on the buckets are spaced evenly in the distance's
    logarithm up to `far`, and the last bucket takes everything beyond."""
    half = n_buckets // 2
    if n < half:
        return n
    return min(n_buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (n_buckets - half))))


def chunk_attention(h, p, m, eps):
    """h [T, W].  q = W_q h and k = W_k h are each normed as one vector over all heads (a weight per entry); the values are
    k as projected.  Head a of H reads key head a // (H // G).  score(i, j) = q_i . k_j * scale * temp[a] + rel[bucket(i - j), a]
    for j <= i in the same chunk of `mask.size` positions; the weights are exp(score) / (1 + sum exp(score))."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q_raw, k_raw = h @ p("left.q").T, h @ p("left.k").T
    q = rms_norm(q_raw, p("left.q.norm"), eps).view(T, H, d)
    k = rms_norm(k_raw, p("left.k.norm"), eps).view(T, G, d)
    v = k_raw.view(T, G, m["vdim"])
    rel, temp = p("left.rel"), p("left.temp")
    B = rel.shape[0]
    chunk = m["mask"]["size"]
    out = torch.zeros(T, H, m["vdim"], dtype=h.dtype)
    for i in range(T):
        lo = (i // chunk) * chunk
        js = list(range(lo, i + 1))
        bias = torch.stack([rel[distance_bucket(i - j, B, m["bias_max"])] for j in js])      # [keys, H]
        for a in range(H):
            g = a // (H // G)
            s = (k[js, g] @ q[i, a]) * m["scale"] * temp[a] + bias[:, a]
            top = torch.clamp(s.max(), min=0.0)
            e = torch.exp(s - top)
            wts = e / (torch.exp(-top) + e.sum())
            out[i, a] = wts @ v[js, g]
    return out.reshape(T, H * m["vdim"]) @ p("left.o").T


# ----------------------------------------------------------------------------
# a gated recurrence whose gates read the token alone
# ----------------------------------------------------------------------------

def min_gru(h, p):
    """z = sigmoid(W_z h + b_z); u = W_x h + b_x; c = u + 1/2 where u >= 0, sigmoid(u) below; S_t = (1 - z) S_(t-1) + z c;
    the result is W_o (S_t * silu(W_g h))."""
    z = torch.sigmoid(h @ p("right.z").T + p("right.z.b"))
    u = h @ p("right.x").T + p("right.x.b")
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = silu(h @ p("right.g").T)
    S = torch.zeros(z.shape[1], dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * c[t]
        rows.append(S * gate[t])
    return torch.stack(rows) @ p("right.o").T


def parallel_mixer(h, p, m, eps):
    """Both halves read h; each result is normed over the width with its own weight; half their sum."""
    left = rms_norm(chunk_attention(h, p, m["left"], eps), p("left.out"), eps)
    right = rms_norm(min_gru(h, p), p("right.out"), eps)
    return 0.5 * (left + right)


# ----------------------------------------------------------------------------
# a state-space mixer with one decay per head and token
# ----------------------------------------------------------------------------

def mamba2(h, p, m, eps):
    T = h.shape[0]
    H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * dv
    proj = h @ p("in").T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_taps(xbc, p("conv"), p("conv.b")))
    x = xbc[:, :inner].view(T, H, dv)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + p("dt_bias"))                       # [T, H]
    rate = torch.exp(p("A_log"))
    S = torch.zeros(H, N, dv, dtype=h.dtype)
    y = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        for a in range(H):
            g = a // (H // G)
            S[a] = torch.exp(-rate[a] * dt[t, a]) * S[a] + dt[t, a] * torch.outer(Bm[t, g], x[t, a])
            y[t, a] = S[a].T @ Cm[t, g] + p("D")[a] * x[t, a]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * p("norm")
    return y @ p("o").T


# ----------------------------------------------------------------------------
# feed-forward
# ----------------------------------------------------------------------------

def dense_ffn(h, p):
    return gelu_erf(h @ p("up").T + p("up.b")) @ p("down").T + p("down.b")


# ----------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------

def forward(cfg, w, tokens, layers_out=None):
    """-> logits [T, vocab].  layers_out: a list that receives the stream behind every layer (the sum of the copies
    where there are several)."""
    eps = cfg["norm"]["eps"]
    n_streams = cfg.get("streams")
    x = embed(cfg, w, tokens)
    xs = [x.clone() for _ in range(n_streams)] if n_streams else None
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        pre = f"l{src}."

        def mix(name):
            return w[pre + "mix." + name]

        def ff(name):
            return w[pre + "mlp." + name]

        def mixer(hh):
            if layer["type"] == "parallel":
                return parallel_mixer(hh, mix, layer["mixer"], eps)
            return mamba2(hh, mix, layer["mixer"], eps)
        subs = [(1, mixer)] + ([(2, lambda hh: dense_ffn(hh, ff))] if layer.get("mlp") else [])
        for q, f in subs:
            g = w[pre + f"norm{q}"]
            if xs is None:
                x = x + f(rms_norm(x, g, eps))
                continue
            a_in, a_out, a_mix = w[pre + f"hc{q}.in"], w[pre + f"hc{q}.out"], w[pre + f"hc{q}.mix"]
            u = sum(a_in[s] * xs[s] for s in range(n_streams))
            y = f(rms_norm(u, g, eps))
            xs = [sum(a_mix[s, t] * xs[s] for s in range(n_streams)) + a_out[t] * y for t in range(n_streams)]
        if layers_out is not None:
            layers_out.append(x.clone() if xs is None else sum(xs))
    if xs is not None:
        x = sum(xs)
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T * cfg.get("logit_scale", 1.0)
