"""Plain PyTorch references of the kernels, one function per entry of
`denno_beta_amd.kernels.ops`, with the same arguments.  Computation is 32-bit (inputs in
bfloat16 are widened first); outputs are rounded to the output tensor's dtype once.

They serve two ends: the GPU tests compare each HIP kernel with its reference here, and the
CPU tests put them in the kernels' place to run the engine's host logic (batching, cache,
scheduling) without a GPU.
"""
from __future__ import annotations

import math

import torch


def embed(tokens, positions, wte, wpe, out, token_scale=1.0):
    x = wte[tokens.long()].float()
    if token_scale != 1.0:
        x = x * torch.tensor(token_scale, dtype=torch.float32)
    if wpe is not None:
        x = x + wpe[positions.long()].float()
    out.copy_(x)
    return out


def embed_sum(parts, out):
    x = None
    for table, index, scale in parts:
        a = table[index.long()].float()
        if scale != 1.0:
            a = a * torch.tensor(scale, dtype=torch.float32)
        x = a if x is None else x + a
    out.copy_(x)
    return out


def logits_post(logits, scale=1.0, softcap=0.0):
    logits.mul_(torch.tensor(scale, dtype=torch.float32))
    if softcap > 0:
        logits.copy_(softcap * torch.tanh(logits / softcap))
    return logits


def layernorm(x, gamma, beta, eps, out, rows=None):
    src = x if rows is None else x[rows.long()]
    mean = src.mean(dim=-1, keepdim=True)
    d = src - mean
    var = (d * d).mean(dim=-1, keepdim=True)
    y = d / torch.sqrt(var + eps) * gamma
    if beta is not None:
        y = y + beta
    out.copy_(y)
    return out


def kv_write(src, k_col, v_col, slot_map, k_pool, v_pool):
    n_pages, hkv, ps, dh = k_pool.shape
    w = hkv * dh
    for t in range(src.shape[0]):
        slot = int(slot_map[t])
        if slot < 0:
            continue
        page, off = divmod(slot, ps)
        k_pool[page, :, off, :] = src[t, k_col:k_col + w].view(hkv, dh)
        v_pool[page, :, :, off] = src[t, v_col:v_col + w].view(hkv, dh)


def cast(x, out):
    out.copy_(x)
    return out


def linear(a, w, bias=None, out=None, epilogue="none", residual=None):
    wide = torch.float64 if a.dtype == torch.float64 else torch.float32
    y = a.to(wide) @ w.to(wide).t()
    if bias is not None:
        y = y + bias
    if residual is not None:
        residual += y
        return residual
    if epilogue == "gelu_tanh":
        y = torch.nn.functional.gelu(y, approximate="tanh")
    elif epilogue == "gelu_erf":
        y = torch.nn.functional.gelu(y)
    elif epilogue == "relu2":
        y = torch.relu(y) ** 2
    elif epilogue != "none":
        raise ValueError(epilogue)
    out.copy_(y)
    return out


def norm_folded(w_rows, bias, gamma, beta):
    w = w_rows.float()
    c1 = w @ gamma.float()
    c2 = torch.zeros_like(c1) if beta is None else w @ beta.float()
    return c1, (c2 if bias is None else c2 + bias.float())


def linear_norm_out(a, w, bias, residual, gamma, copy, stats):
    linear(a, w, bias, residual=residual)
    copy.copy_(residual * gamma)
    blocks = residual.view(residual.shape[0], -1, 16)
    mean = blocks.mean(dim=-1)
    stats[:, :, 0] = mean
    stats[:, :, 1] = ((blocks - mean[:, :, None]) ** 2).sum(dim=-1)
    return residual


def linear_norm_in(copy, stats, c1, c2, eps, w, out, epilogue="none", kv=None, no_mean=False):
    """The kernel's own formula: the product of the rows that are not normalised, then the row's mean
    and 1 / sqrt(var + eps), joined from the blocks' pairs, on the sums.  no_mean: the mean counts as 0."""
    mean = stats[:, :, 0].mean(dim=1, keepdim=True)
    if no_mean:
        mean = torch.zeros_like(mean)
    var = (stats[:, :, 1] + 16.0 * (stats[:, :, 0] - mean) ** 2).sum(dim=1, keepdim=True) / copy.shape[1]
    y = (copy.float() @ w.float().t() - mean * c1) / torch.sqrt(var + eps) + c2
    if epilogue == "gelu_tanh":
        y = torch.nn.functional.gelu(y, approximate="tanh")
    elif epilogue == "gelu_erf":
        y = torch.nn.functional.gelu(y)
    elif epilogue == "relu2":
        y = torch.relu(y) ** 2
    if kv is None:
        out.copy_(y)
        return out
    slot_map, k_pool, v_pool, q_width = kv
    hkv, dh = k_pool.shape[1], k_pool.shape[3]
    full = y.to(out.dtype)
    kv_write(full, q_width, q_width + hkv * dh, slot_map, k_pool, v_pool)
    out.copy_(full[:, :out.shape[1]])
    return out[:, :q_width]


def attention(q, out, k_pool, v_pool, block_tables, tiles, n_heads, scale, window=0, tiles_wide=None,
              single_rows=False, max_context=0, decode_waves=None, chunk=0, bias=None, sink=False):
    n_pages, hkv, ps, dh = k_pool.shape
    group = n_heads // hkv
    tl = tiles.cpu().tolist()
    bt = block_tables.cpu()
    kf, vf = k_pool.float(), v_pool.float()
    for seq, row0, nrows, pos0 in zip(*tl):
        if seq < 0:
            continue
        for i in range(nrows):
            pos = pos0 + i
            lo = max(0, pos - window + 1) if window > 0 else 0
            if chunk > 0:
                lo = max(lo, pos // chunk * chunk)
            keys = torch.arange(lo, pos + 1)
            pages = bt[seq][keys // ps].long()
            offs = keys % ps
            assert (pages >= 0).all(), "attention reads a page that was given back"
            for h in range(n_heads):
                k = kf[pages, h // group, offs, :]                  # [n, dh]
                v = vf[pages, h // group, :, offs]
                qv = q[row0 + i, h * dh:(h + 1) * dh].float()
                sc = (k @ qv) * scale
                if bias is not None:
                    sc = sc + bias[h][torch.clamp(pos - keys, max=bias.shape[1] - 1)]
                if sink:      # (a key with score 0 and no value)
                    p = torch.softmax(torch.cat([sc, sc.new_zeros(1)]), dim=0)[:-1]
                else:
                    p = torch.softmax(sc, dim=0)
                out[row0 + i, h * dh:(h + 1) * dh] = (p @ v).to(out.dtype)
    return out


def sample(logits, temperature, uniform, out):
    for r in range(logits.shape[0]):
        row = logits[r]
        t = float(temperature[r])
        if not t > 0:
            best, best_v = 0, float("-inf")
            for i, v in enumerate(row.tolist()):
                if v > best_v:
                    best, best_v = i, v
            out[r] = best
            continue
        z = row / t
        e = torch.exp(z - z.max())
        c = torch.cumsum(e.double(), 0)
        target = float(uniform[r]) * float(c[-1])
        idx = int(torch.searchsorted(c, torch.tensor(target, dtype=torch.float64)))
        out[r] = min(idx, row.shape[0] - 1)
    return out


def penalties(logits, ctx, begin, length, repetition, frequency, presence, ngram, bounds=None):
    from plain import sampler_plain as sp
    for r in range(logits.shape[0]):
        c = ctx[int(begin[r]):int(begin[r]) + int(length[r])].tolist()
        row = logits[r].tolist()
        row = sp.repetition_penalty(row, c, float(repetition[r]))
        row = sp.frequency_presence(row, c, float(frequency[r]), float(presence[r]))
        row = sp.no_repeat_ngram(row, c, int(ngram[r]))
        logits[r] = torch.tensor(row, dtype=torch.float32)
    return logits


def history_append(history, begin, length, rows, tokens, bounds=None):
    for b, n, r in zip(begin.tolist(), length.tolist(), rows.tolist()):
        history[b + n] = tokens[r]
    return history


def sample_top(logits, rows, temperature, uniform, top_k, top_p, out, undecided):
    from plain import sampler_plain as sp
    for j, r in enumerate(rows.tolist()):
        k, p = int(top_k[j]), float(top_p[j])
        if k > 0:
            out[r] = sp.top_k_top_p(logits[r].tolist(), float(temperature[r]), min(k, 2048),
                                    None if p >= 1.0 else p, float(uniform[r]))
            undecided[j] = 0
        else:
            tok, whole = sp.top_p_alone(logits[r].tolist(), float(temperature[r]), p, float(uniform[r]))
            out[r], undecided[j] = tok, int(whole)
    return out


def sample_full(logits, rows, temperature, uniform, top_p, out, only=None):
    from plain import sampler_plain as sp
    for j, r in enumerate(rows.tolist()):
        if only is not None and int(only[j]) == 0:
            continue
        p = float(top_p[j])
        out[r] = sp.top_k_top_p(logits[r].tolist(), float(temperature[r]), None, None if p >= 1.0 else p,
                                float(uniform[r]))
    return out


def linear_qkv(a, w, bias, out, slot_map, k_pool, v_pool, q_width):
    linear(a, w, bias, out=out)
    kvw = k_pool.shape[1] * k_pool.shape[3]
    kv_write(out, q_width, q_width + kvw, slot_map, k_pool, v_pool)
    return out[:, :q_width]


# -- layers that carry more than keys and values from token to token ---------------------------------------------------
def _act(kind, z, lower=None):
    if kind == "silu":
        return z * torch.sigmoid(z)
    if kind == "sigmoid":
        return torch.sigmoid(z)
    if kind == "tanh":
        return torch.tanh(z)
    if kind == "exp_neg_exp":
        return torch.exp(-torch.exp(z))
    if kind == "bounded_sigmoid":
        return lower + (1.0 - lower) * torch.sigmoid(z)
    if kind == "exp_neg_softplus":
        return torch.exp(-lower * torch.nn.functional.softplus(z))
    if kind == "xielu":
        neg = torch.clamp(z, max=0)
        return torch.where(z > 0, lower[0] * z * z + 0.5 * z, lower[1] * (torch.expm1(neg) - neg) + 0.5 * z)
    if kind == "relu2":
        return torch.relu(z) ** 2
    raise ValueError(kind)


def rmsnorm(x, weight, eps, out, rows=None):
    E = out.shape[1]
    src = (x if rows is None else x[rows.long()])[:, :E].float()
    y = src / torch.sqrt((src * src).mean(dim=-1, keepdim=True) + eps)
    out.copy_(y if weight is None else y * weight)
    return out


def _then(then, x):
    if then is not None:
        w, eps, out = then
        n = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
        out.copy_(n if w is None else n * w)


def rmsnorm_add(y, weight, scale, mult, eps, x, gate=None, then=None):
    src = y.float()
    if gate is not None:
        src = src * torch.sigmoid(gate.float())
    n = src / torch.sqrt((src * src).mean(dim=-1, keepdim=True) + eps)
    if weight is not None:
        n = n * weight
    if scale is not None:
        n = n * scale
    x += mult * n
    _then(then, x)
    return x


def depth_mix(hist, n, weights, out):
    acc = torch.zeros_like(hist[0])
    for j in range(n):
        acc = acc + weights[j] * hist[j]
    out.copy_(acc)
    return out


def unit_heads(x, n_heads, dim, eps, scale, out):
    T = x.shape[0]
    v = x[:, :n_heads * dim].reshape(T, n_heads, dim)
    y = v / torch.sqrt((v * v).sum(dim=-1, keepdim=True) + eps) * scale
    out[:, :n_heads * dim] = y.reshape(T, n_heads * dim)
    return out


def concat_cast(a, b, out):
    out.copy_(torch.cat([a, b], dim=1))
    return out


def _requests(row_start, slots):
    rs, sl = row_start.tolist(), slots.tolist()
    return [(sl[s], rs[s], rs[s + 1]) for s in range(len(sl)) if sl[s] >= 0]


def conv_rows(h, w, hist, row_start, slots, out, identity=True, act=None, bias=None):
    width, taps = w.shape
    h = h[:, :width]
    res = torch.zeros((h.shape[0], width), dtype=torch.float32)
    for slot, a, b in _requests(row_start, slots):
        rows = h[a:b] if taps == 1 else torch.cat([hist[slot].view(taps - 1, width), h[a:b]], dim=0)
        for t in range(b - a):
            acc = h[a + t].clone() if identity else torch.zeros(width)
            if bias is not None:
                acc = acc + bias
            for j in range(taps):
                acc += w[:, j] * rows[t + j]
            res[a + t] = acc
    out.copy_(res if act is None else _act(act, res))
    return out


def conv_heads(h, w, hist, row_start, slots, out, n_unit, unit_dim, n_first, scale_first, scale_rest, eps, n_rest, rest_dim):
    conv_rows(h, w, hist, row_start, slots, out, identity=False, act="silu")
    T = out.shape[0]
    if n_unit:
        v = out[:, :n_unit * unit_dim].reshape(T, n_unit, unit_dim)
        scale = torch.cat([torch.full((n_first,), float(scale_first)), torch.full((n_unit - n_first,), float(scale_rest))])
        y = v / torch.sqrt((v * v).sum(dim=-1, keepdim=True) + eps) * scale[None, :, None]
        out[:, :n_unit * unit_dim] = y.reshape(T, -1)
    return out


def rotary_runs(src, positions, freq, runs, mag=1.0, unit=None, eps=0.0):
    unit = [False] * len(runs) if unit is None else unit
    for (dst, src_off, n_vec, width, dims, dst_off, dst_stride), un in zip(runs, unit):
        rotary(src, dst, positions, freq[:dims // 2], n_vec, dims, width, src_off=src_off, src_stride=width, dst_off=dst_off,
               dst_stride=dst_stride, mag=mag, unit_eps=eps if un else None)


def history_update(h, hist, row_start, slots):
    width = h.shape[1]
    keep = hist.shape[1] // width
    for slot, a, b in _requests(row_start, slots):
        rows = torch.cat([hist[slot].view(keep, width), h[a:b].float()], dim=0)
        hist[slot] = rows[rows.shape[0] - keep:].reshape(-1)


def shift_mix(h, hist, mu, row_start, slots, out):
    hf = h.float()
    res = torch.zeros(out.shape, dtype=torch.float32)
    for slot, a, b in _requests(row_start, slots):
        prev = torch.cat([hist[slot].view(1, -1), hf[a:b - 1]], dim=0)
        for m in range(mu.shape[0]):
            res[m, a:b] = hf[a:b] + (prev - hf[a:b]) * mu[m]
    out.copy_(res)
    return out


def rotary(src, dst, positions, freq, n_vec, dims, width, src_off=0, src_stride=None, dst_off=0, dst_stride=None, mag=1.0,
           unit_eps=None):
    src_stride = width if src_stride is None else src_stride
    dst_stride = width if dst_stride is None else dst_stride
    ang = positions.float()[:, None] * freq[None, :]
    cos, sin = torch.cos(ang) * mag, torch.sin(ang) * mag
    for n in range(n_vec):
        vec = src[:, src_off + n * src_stride: src_off + n * src_stride + width].float().clone()
        a, b = vec[:, 0:dims:2].clone(), vec[:, 1:dims:2].clone()
        vec[:, 0:dims:2] = a * cos - b * sin
        vec[:, 1:dims:2] = b * cos + a * sin
        if unit_eps is not None:      # (rotary_runs' norm behind the turn)
            vec = vec / torch.sqrt((vec * vec).mean(dim=-1, keepdim=True) + unit_eps)
        dst[:, dst_off + n * dst_stride: dst_off + n * dst_stride + width] = vec.to(dst.dtype)
    return dst


def activate(x, kind, out, bias=None, lower=None):
    z = x if bias is None else x + bias
    out.copy_(_act(kind, z, lower))
    return out


def gated(x, g, kind, out):
    out.copy_(x.float() * _act(kind, g))
    return out


def state_scan(r, k, v, w, u, state, row_start, slots, n_heads, dk, dv, out, read_after=False, key_from_decay=False, beta=None,
               w_head=None, qk_heads=None, beta_logits=False, w_rows=False):
    H = n_heads
    if beta is not None and beta_logits:
        beta = torch.sigmoid(beta)
    G = H if qk_heads is None else qk_heads
    spread = lambda x: x.view(G, dk).repeat_interleave(H // G, dim=0)      # noqa: E731  (head h reads head h // (H // G))
    for slot, a, b in _requests(row_start, slots):
        S = state[slot].view(H, dv, dk).transpose(1, 2).clone()      # (held [head][value column][key channel])
        for t in range(a, b):
            rt, vt = spread(r[t]), v[t].view(H, dv)
            wt = (w[t].view(H, 1).expand(H, dk) if w_rows else w[t].view(H, dk)) if w is not None else w_head.view(H, 1).expand(H, dk)
            at = (1.0 - wt) if key_from_decay else spread(k[t])
            kv = at[:, :, None] * vt[:, None, :]
            if beta is not None:
                S = wt[:, :, None] * S
                e = beta[t].view(H, 1) * (vt - torch.einsum("hi,hij->hj", at, S))
                S = S + at[:, :, None] * e[:, None, :]
                out[t] = torch.einsum("hi,hij->hj", rt, S).reshape(-1)
            elif read_after:
                S = wt[:, :, None] * S + kv
                out[t] = torch.einsum("hi,hij->hj", rt, S).reshape(-1)
            else:
                bonus = kv * u.view(H, dk)[:, :, None] if u is not None else 0.0
                out[t] = torch.einsum("hi,hij->hj", rt, S + bonus).reshape(-1)
                S = wt[:, :, None] * S + kv
        state[slot] = S.transpose(1, 2).reshape(-1)
    return out


def head_norm(o, weight, eps, out, n_heads, gate=None, gate_kind="silu", gate_first=False, skip=None, skip_scale=None):
    T, n = o.shape
    dv = n // n_heads
    y = o
    if skip is not None:
        y = y + skip * skip_scale.repeat_interleave(n // skip_scale.numel())
    if gate is not None and gate_first:
        y = y * _act(gate_kind, gate)
    y = y.reshape(T, n_heads, dv)
    y = y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)
    if weight is not None:
        y = y * (weight.view(n_heads, dv) if weight.numel() == n else weight)
    y = y.reshape(T, n)
    if gate is not None and not gate_first:
        y = y * _act(gate_kind, gate)
    out.copy_(y)
    return out


def step_sizes(z, bias, rate, x, n_heads, decay, v):
    T, n = x.shape
    dt = torch.nn.functional.softplus(z.double() + (bias.double() if bias is not None else 0.0))
    decay.copy_(torch.exp(-rate.double() * dt))
    v.copy_((dt[:, :, None] * x.double().view(T, n_heads, n // n_heads)).reshape(T, n))
    return decay, v


def gate_scan(a, b, g, bias_a, bias_b, state, row_start, slots, out):
    z = torch.sigmoid(a.double() + (bias_a.double() if bias_a is not None else 0.0))
    u = b.double() + (bias_b.double() if bias_b is not None else 0.0)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = _act("silu", g.double())
    for slot, lo, hi in _requests(row_start, slots):
        S = state[slot].double().clone()
        for t in range(lo, hi):
            S = (1 - z[t]) * S + z[t] * cand[t]
            out[t] = (S * gate[t]).to(out.dtype)
        state[slot] = S.to(state.dtype)
    return out


def head_gate(o, gate, n_heads, dv, out, head_stride=None):
    hs = dv if head_stride is None else head_stride
    T = o.shape[0]
    for h in range(n_heads):
        out[:, h * dv:(h + 1) * dv] = (o[:, h * hs:h * hs + dv].float() * torch.sigmoid(gate[:, h:h + 1].float())).to(out.dtype)
    return out


def rows_times_table(a, table, ids, off, out):
    n = a.shape[1]
    out.copy_(a.float() * table[ids.long(), off:off + n].float())
    return out


def token_input(x, w_gate, w_proj, table, ids, off, weight, eps, then=None):
    dim = w_gate.shape[0]
    z = x @ w_gate.float().T
    g = torch.nn.functional.gelu(z, approximate="tanh") * table[ids.long(), off:off + dim].float()
    y = g @ w_proj.float().T
    n = y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)
    x += n if weight is None else n * weight
    _then(then, x)
    return x


def selective_scan(x, dt, dt_bias, B, C, A, D, z, state, row_start, slots, out, in_order=False):
    inner, N = A.shape
    step = torch.nn.functional.softplus(dt.double() + (dt_bias.double() if dt_bias is not None else 0.0))
    for slot, lo, hi in _requests(row_start, slots):
        S = state[slot].double().view(inner, N).clone()
        for t in range(lo, hi):
            S = torch.exp(step[t][:, None] * A.double()) * S + (step[t] * x[t].double())[:, None] * B[t].double()[None, :]
            y = S @ C[t].double()
            if D is not None:
                y = y + D.double() * x[t].double()
            if z is not None:
                y = y * _act("silu", z[t].double())
            out[t] = y.to(out.dtype)
        state[slot] = S.reshape(-1).to(state.dtype)
    return out


def streams_read(xs, w_in, weight, eps, out, rows=None):
    n = xs.shape[0]
    u = sum((w_in[s].double() if w_in is not None else 1.0) * xs[s].double() for s in range(n))
    if rows is not None:
        u = u[rows.long()]
    if eps is not None:
        u = u / torch.sqrt((u * u).mean(dim=-1, keepdim=True) + eps)
    if weight is not None:
        u = u * weight.double()
    out.copy_(u)
    return out


def streams_write(xs, y, mix, w_out, next_in=None, weight=None, eps=0.0, out=None, branches=None):
    n = xs.shape[0]
    old = xs.double().clone()
    if branches is not None:
        y2, w1, w2, beps = branches
        unit = lambda v: v.double() / torch.sqrt((v.double() ** 2).mean(dim=-1, keepdim=True) + beps)      # noqa: E731
        y = 0.5 * (unit(y) * w1.double() + unit(y2) * w2.double())
    m = mix.double().view(n, n)
    for t in range(n):
        xs[t] = (sum(m[s, t] * old[s] for s in range(n)) + w_out[t].double() * y.double()).to(xs.dtype)
    if next_in is not None:
        streams_read(xs, next_in, weight, eps, out)
    return out


def norm_pair_write(z, q_width, wq, wk, eps, q_out, slot_map, k_pool, v_pool, write=True):
    n_pages, hkv, ps, dh = k_pool.shape
    unit = lambda v: v.double() / torch.sqrt((v.double() ** 2).mean(dim=-1, keepdim=True) + eps)      # noqa: E731
    q_out.copy_(unit(z[:, :q_width]) * wq.double())
    if write:
        keys = (unit(z[:, q_width:]) * wk.double()).to(k_pool.dtype)
        for t, slot in enumerate(slot_map.tolist()):
            if slot >= 0:
                k_pool[slot // ps, :, slot % ps, :] = keys[t].view(hkv, dh)
                v_pool[slot // ps, :, :, slot % ps] = z[t, q_width:].view(hkv, dh).to(v_pool.dtype)
    return q_out


def pair_rows(tokens, positions, row_start, slots, last, mul_prev, mul_cur, buckets, out, write=True):
    tok = tokens.tolist()
    out.fill_(buckets)
    for slot, lo, hi in _requests(row_start, slots):
        for t in range(lo, hi):
            if int(positions[t]) == 0:
                continue
            prev = tok[t - 1] if t > lo else int(last[slot, 0])
            out[t] = (prev * mul_prev + tok[t] * mul_cur) % buckets
        if write:
            last[slot, 0] = tok[hi - 1]
    return out


def heads_linear(a, w, out, a_off=0, a_stride=None, o_off=0, o_stride=None):
    H, N, K = w.shape
    a_stride = K if a_stride is None else a_stride
    o_stride = N if o_stride is None else o_stride
    for h in range(H):
        y = a[:, a_off + h * a_stride: a_off + h * a_stride + K].float() @ w[h].float().t()
        out[:, o_off + h * o_stride: o_off + h * o_stride + N] = y.to(out.dtype)
    return out


def moe_route(z, correction, top, ids, wts, score="softmax", renorm=True, n_experts=None, groups=1, keep=1, scale=1.0):
    if n_experts is not None:
        z = z[:, :n_experts]
    E = z.shape[1]
    s = torch.softmax(z, dim=-1) if score == "softmax" else torch.sigmoid(z)
    choice = s if correction is None else s + correction
    for t in range(z.shape[0]):
        c = choice[t].clone()
        if keep < groups:
            per = E // groups
            gs = c.view(groups, per).topk(min(2, per), dim=-1).values.sum(dim=-1)
            closed = torch.ones(groups, dtype=torch.bool)
            for _ in range(keep):
                g = int(torch.argmax(torch.where(closed, gs, torch.full_like(gs, -float("inf")))))
                closed[g] = False
            c[closed.repeat_interleave(per)] = -float("inf")
        picked = []
        for _ in range(top):
            e = int(torch.argmax(c))           # (the first of equal values)
            picked.append(e)
            c[e] = -float("inf")
        ws = s[t, picked]
        ids[t] = torch.tensor(picked, dtype=torch.int32)
        wts[t] = (ws / (ws.sum() + 1e-20) if renorm else ws) * scale


def moe_plan(ids, n_experts, offsets, order):
    flat = ids.reshape(-1).long()
    idx = torch.sort(flat, stable=True).indices
    order.copy_(idx.to(torch.int32))
    counts = torch.bincount(flat, minlength=n_experts)
    offsets[0] = 0
    offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)


def moe_up(h, order, offsets, top, w_gate, w_up, limit, alpha, y, dims=None, kind="clamped", in_scale=None):
    assert dims is None, "packed experts are for the GPU's kernels"
    off = offsets.tolist()
    for e in range(w_up.shape[0]):
        for p in range(off[e], off[e + 1]):
            x = h[int(order[p]) // top].float()
            if kind == "relu2":
                sc = 1.0 if in_scale is None else in_scale.reshape(-1)[int(order[p])]
                y[p] = (torch.relu((w_up[e].float() @ x) * sc) ** 2).to(y.dtype)
                continue
            if kind == "silu":
                sc = 1.0 if in_scale is None else in_scale.reshape(-1)[int(order[p])]
                g, u = (w_gate[e].float() @ x) * sc, (w_up[e].float() @ x) * sc
                y[p] = (g * torch.sigmoid(g) * u).to(y.dtype)
                continue
            g = torch.clamp(w_gate[e].float() @ x, max=limit)
            u = torch.clamp(w_up[e].float() @ x, min=-limit, max=limit)
            y[p] = (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(y.dtype)


def moe_down(y, order, offsets, w_down, out, dims=None):
    assert dims is None, "packed experts are for the GPU's kernels"
    off = offsets.tolist()
    for e in range(w_down.shape[0]):
        for p in range(off[e], off[e + 1]):
            out[int(order[p])] = w_down[e].float() @ y[p].float()


def moe_combine(out, wts, x, logits=False):
    T = x.shape[0]
    if logits:
        wts = torch.sigmoid(wts)
    if wts is None:
        x += out.view(T, -1, x.shape[1]).sum(dim=1)
        return
    top = wts.shape[1]
    x += (out.view(T, top, -1) * wts[:, :, None]).sum(dim=1)
