"""Dogalorn through the engine against the plain implementation (tests/plain/dogalorn_plain.py): each mechanism alone,
every way of cutting the work, first tokens, far tokens, chunk edges, long decoding, slots and pages used again, other
sizes, generation through the scheduler.  Backend "host" runs the engine's own code on the CPU with the kernels' plain
references in their place; backend "gpu" runs the HIP kernels."""
import copy
import json
import math
import os

import pytest
import torch

import replay_util as U
from conftest import seeded_tokens
from plain import dogalorn_plain as plain


# ----------------------------------------------------------------------------------------------------------------
# configurations: each differs from the others in every size
# ----------------------------------------------------------------------------------------------------------------
def parallel(heads=4, kv_heads=2, dim=8, chunk=24, gru=20, scale=None, far=40, buckets=8):
    return dict(type="parallel", mixer=dict(
        left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5 if scale is None else scale, bias_max=far,
                  mask=dict(size=chunk), bias_buckets=buckets),
        right=dict(width=gru)))


def mamba(heads=4, vdim=8, state=16, groups=2, conv=3, norm_groups=2):
    return dict(type="mamba2", mixer=dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups))


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def with_mlp(layer, mlp):
    return dict(copy.deepcopy(layer), mlp=mlp)


def again(layers, i):
    """A layer that runs with layer i's tensors."""
    return dict(copy.deepcopy(layers[i]), weights_of=i)


def config(layers, width=32, vocab=97, eps=1e-5, streams=2, bigram=(53, 7, 11), logit_scale=1.5):
    c = dict(architecture="Dogalorn", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)
    if streams:
        c["streams"] = streams
    if bigram:
        c["embedding"] = dict(bigram=dict(buckets=bigram[0], mul_prev=bigram[1], mul_cur=bigram[2]))
    if logit_scale is not None:
        c["logit_scale"] = logit_scale
    return c


_p = [with_mlp(parallel(4, 2, 8, 24, 20), dense(40)), with_mlp(mamba(4, 8, 16, 2, 3, 2), dense(24)),
      with_mlp(parallel(2, 2, 16, 40, 12, far=70, buckets=12), None)]
# both mixers, grouped key heads, groups of B and C, a layer without a feed-forward, two layers run a second time
CFG_P = config(_p + [again(_p, 1), again(_p, 0)], width=32, vocab=97, streams=2)
# other sizes: four copies of the stream; one key head; a head size that no 16 divides; one tap and four; one norm group;
# chunks shorter than a page and no multiple of one; another order of layers; multipliers beyond the buckets
_q = [with_mlp(mamba(3, 12, 24, 1, 1, 1), None), with_mlp(parallel(3, 1, 24, 13, 36, scale=0.31, far=500, buckets=6), dense(20)),
      with_mlp(mamba(2, 20, 8, 2, 4, 4), dense(56))]
CFG_Q = config(_q + [again(_q, 1)], width=48, vocab=131, eps=1e-6, streams=4, bigram=(17, 1000, 999), logit_scale=0.5)
# sizes that are multiples of nothing (the kernels' paths for single numbers): a width of 36, heads of 6 and 10, five taps, one copy
# of the stream, a single bucket pair, a table of pairs with one bucket
CFG_R = config([with_mlp(parallel(2, 1, 6, 7, 9, far=9, buckets=2), dense(9)), with_mlp(mamba(2, 10, 6, 1, 5, 1), dense(11)),
                with_mlp(parallel(1, 1, 10, 100, 5, far=33, buckets=5), None)], width=36, vocab=61, streams=1, bigram=(1, 3, 2),
               logit_scale=None)
# the plain residual stream (no copies) and token rows alone (no table of pairs)
CFG_S = config([with_mlp(mamba(2, 8, 8, 1, 2, 1), dense(16)), with_mlp(parallel(2, 1, 8, 16, 8), None),
                with_mlp(parallel(2, 2, 8, 9, 16), dense(12))], width=24, vocab=71, streams=None, bigram=None, logit_scale=2.5)
CONFIGS = {"P": (CFG_P, 41), "Q": (CFG_Q, 42), "R": (CFG_R, 43), "S": (CFG_S, 44)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from denno_beta_amd.weights import write_model_folder
    made = {}

    def get(name, dtype="float32", cfg=None, seed=None, change=None):
        key = (name, dtype)
        if key not in made:
            c, s = CONFIGS[name] if cfg is None else (cfg, seed)
            d = str(tmp_path_factory.mktemp(f"dogalorn{name}_{dtype}"))
            write_model_folder(d, c, s, dtype)
            if change is not None:
                from safetensors.torch import load_file, save_file
                path = os.path.join(d, "model.safetensors")
                stored = load_file(path)
                tensors = {k: v.float() for k, v in stored.items()}
                change(tensors)
                save_file({k: v.to(stored[k].dtype).contiguous() for k, v in tensors.items()}, path)
            made[key] = d
        return made[key]
    return get


def runner_for(folder, dtype, device, cache_tokens, max_live=4, page_size=16, **more):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, device=device, page_size=page_size,
                                                         cache_tokens=cache_tokens, max_live=max_live, **more))


_plain = {}


def plain_logits(folder, seq, layers_out=None):
    key = (folder, tuple(seq))
    if key not in _plain or layers_out is not None:
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        w = {k: (v.double() if v.is_floating_point() else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
        _plain[key] = plain.forward(cfg, w, seq, layers_out)
    return _plain[key]


def row_errors(got, want):
    """Per position: the root mean square of the difference (its mean taken off) over the spread of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(dim=1, keepdim=True)
    return torch.sqrt((d * d).mean(dim=1)) / want.double().std(dim=1)


# bfloat16, in models 24 to 48 wide: a typical row is off by 0.01 of its spread and a row in a few hundred by several times
# that, so one row in fifty may pass the bound, none by more than two and a half times; a fault moves rows by 0.2 and more
BOUND = {"float32": 2e-5, "bfloat16": 0.06}
BF16_OVER, BF16_WORST = 0.02, 0.15


def assert_rows(got, want, dtype, what, bound=None, worst=BF16_WORST):
    e = row_errors(got, want)
    b = bound or BOUND[dtype]
    if dtype == "bfloat16" and bound is None:
        over = int((e > b).sum())
        assert over <= max(1, BF16_OVER * len(e)) and e.max() <= worst, (
            f"{what}: {over} of {len(e)} positions are off by more than {b} of their row's spread, the worst (position "
            f"{int(e.argmax())}) by {e.max().item():.3g}")
        return
    assert bool((e <= b).all()), f"{what}: position {int(e.argmax())} is off by {e.max().item():.3g} of its row's spread (bound {b})"


def seqs_for(cfg, lengths, seed=3):
    return [seeded_tokens(seed + i, n, cfg["vocab"]) for i, n in enumerate(lengths)]


# ----------------------------------------------------------------------------------------------------------------
# the plain implementation against itself: what its pieces must satisfy whatever the weights
# ----------------------------------------------------------------------------------------------------------------
def test_plain_pieces():
    # distances: a bucket each below half; never beyond the last; never falling; the last bucket from `far` on
    for B, far in ((8, 40), (16, 300), (2, 9), (6, 500)):
        got = [plain.distance_bucket(n, B, far) for n in range(2 * far)]
        assert got[:B // 2] == list(range(B // 2)) and max(got) == B - 1 and got == sorted(got)
        assert all(b == B - 1 for b in got[far:]) and got[B // 2] == B // 2
        # just below `far` the distance is still short of the last bucket's edge (unless the buckets are too few to tell)
        edge = B // 2 + math.floor(math.log((far - 1) / (B // 2)) / math.log(far / (B // 2)) * (B - B // 2))
        assert got[far - 1] == min(B - 1, edge)
    # the first token takes the table's last row; the others the pair's remainder, in whole numbers however large
    rows = plain.pair_rows([5, 9, 9, 2], 1000003, 999983, 17)
    assert rows[0] == 17 and rows[1] == (5 * 1000003 + 9 * 999983) % 17 and rows[2] == (9 * 1000003 + 9 * 999983) % 17
    # the candidate of the gated recurrence: both branches meet at 0 with the same value and slope
    g = torch.Generator().manual_seed(0)
    W = 6
    p = {"right.z": torch.zeros(W, W, dtype=torch.float64), "right.z.b": torch.full((W,), 50.0, dtype=torch.float64),
         "right.x": torch.eye(W, dtype=torch.float64), "right.x.b": torch.zeros(W, dtype=torch.float64),
         "right.g": torch.zeros(W, W, dtype=torch.float64), "right.o": torch.eye(W, dtype=torch.float64)}
    # (z = 1: the state is the candidate; a gate of silu(0) = 0 would hide it, so the gate's matrix is made to give 1.2785, silu = 1)
    p["right.g"] = torch.zeros(W, W, dtype=torch.float64)
    h = torch.tensor([[-1e-7] * W, [1e-7] * W, [2.0] * W, [-2.0] * W], dtype=torch.float64)
    z = torch.sigmoid(h @ p["right.z"].T + p["right.z.b"])
    u = h @ p["right.x"].T
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    assert abs(float(c[0, 0]) - 0.5) < 1e-6 and abs(float(c[1, 0]) - 0.5) < 1e-6 and float(c[2, 0]) == 2.5
    assert abs(float(c[3, 0]) - 1 / (1 + math.exp(2.0))) < 1e-12 and float(z.min()) > 0.999999
    # the convolution's last column weighs the token itself, and the bias is added once
    x = torch.randn(5, 2, generator=g, dtype=torch.float64)
    w = torch.zeros(2, 3, dtype=torch.float64)
    w[:, 2] = 1.0
    b = torch.tensor([0.25, -1.0], dtype=torch.float64)
    assert torch.allclose(plain.causal_taps(x, w, b), x + b)
    w = torch.zeros(2, 3, dtype=torch.float64)
    w[:, 0] = 1.0
    assert torch.allclose(plain.causal_taps(x, w, b)[2:], x[:3] + b) and torch.allclose(plain.causal_taps(x, w, b)[:2], b.expand(2, 2))


def test_the_sink_takes_its_share_and_chunks_hide_what_lies_before():
    """One head, queries and keys made so that every score is 0: with n keys in sight the weights are 1 / (n + 1) each, the
    sink taking the rest; the first position of a chunk sees itself alone."""
    W, d, chunk = 4, 4, 3
    m = dict(heads=1, kv_heads=1, dim=d, vdim=d, scale=1.0, bias_max=50, mask=dict(size=chunk))
    t = {"left.q": torch.zeros(d, W, dtype=torch.float64), "left.k": torch.eye(d, W, dtype=torch.float64),
         "left.q.norm": torch.ones(d, dtype=torch.float64), "left.k.norm": torch.ones(d, dtype=torch.float64),
         "left.rel": torch.zeros(4, 1, dtype=torch.float64), "left.temp": torch.ones(1, dtype=torch.float64),
         "left.o": torch.eye(W, d, dtype=torch.float64)}
    h = torch.randn(7, W, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    out = plain.chunk_attention(h, lambda n: t[n], m, 1e-6)
    for i in range(7):
        lo = i // chunk * chunk
        want = h[lo:i + 1].sum(dim=0) / (i - lo + 2)
        assert torch.allclose(out[i], want, atol=1e-12), i


# ----------------------------------------------------------------------------------------------------------------
# each mechanism alone
# ----------------------------------------------------------------------------------------------------------------
ALONE = {
    "parallel": dict(layers=[with_mlp(parallel(4, 2, 8, 11, 20), None)]),
    "parallel_one_key_head": dict(layers=[with_mlp(parallel(3, 1, 12, 64, 7, scale=0.9, far=20, buckets=4), None)]),
    "parallel_chunks_of_one": dict(layers=[with_mlp(parallel(2, 2, 8, 1, 8), None)]),
    "mamba": dict(layers=[with_mlp(mamba(4, 8, 16, 2, 3, 2), None)]),
    "mamba_one_tap_one_group": dict(layers=[with_mlp(mamba(1, 24, 12, 1, 1, 1), None)]),
    "mamba_head_per_group": dict(layers=[with_mlp(mamba(3, 4, 20, 3, 2, 3), None)]),
    "dense": dict(layers=[with_mlp(mamba(1, 8, 8, 1, 2, 1), dense(28))]),
    "three_copies": dict(layers=[with_mlp(mamba(2, 8, 8, 1, 2, 1), dense(12)), with_mlp(parallel(2, 2, 8, 9, 8), None)], streams=3),
    "one_copy": dict(layers=[with_mlp(parallel(2, 2, 8, 9, 8), dense(12))], streams=1),
    "no_copies": dict(layers=[with_mlp(parallel(2, 2, 8, 9, 8), dense(12)), with_mlp(mamba(2, 8, 8, 1, 2, 1), None)], streams=None),
    "no_pairs": dict(layers=[with_mlp(mamba(2, 8, 8, 1, 2, 1), None)], bigram=None),
    "a_layer_twice": dict(layers=[with_mlp(parallel(2, 1, 8, 6, 8), dense(12)), again([with_mlp(parallel(2, 1, 8, 6, 8), dense(12))], 0)]),
}


@pytest.mark.parametrize("what", sorted(ALONE))
def test_each_mechanism_alone(backend, folders, what):
    kw = dict(ALONE[what])
    cfg = config(kw.pop("layers"), width=24, vocab=53, **kw)
    folder = folders(f"alone_{what}", "float32", cfg, 5)
    seq = seqs_for(cfg, [29])[0]
    want = plain_logits(folder, seq)
    r = runner_for(folder, "float32", backend, 64)
    got = U.replay(r, U.whole_trace([seq]))["r0"]
    assert_rows(got, want, "float32", what)
    got = U.replay(runner_for(folder, "float32", backend, 64), U.chunk_trace([seq], sizes=(2, 5, 1, 7)))["r0"]
    assert_rows(got, want, "float32", what + " in portions")


def test_what_the_model_fixes_matters(folders):
    """The constants and orders that the plain model is built from change its logits: a test against it would see them."""
    from safetensors.torch import load_file
    cfg = CFG_P
    folder = folders("P", "float32")
    W = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    seq = seqs_for(cfg, [50])[0]
    want = plain_logits(folder, seq)
    for change in ("chunk", "far", "scale", "pairs", "temp", "rel", "hc_mix", "hc_in", "conv_b", "D", "left_out", "logit_scale"):
        other, weights = copy.deepcopy(cfg), dict(W)
        if change == "chunk":
            for i in (0, 4):
                other["layers"][i]["mixer"]["left"]["mask"]["size"] = 25
        elif change == "far":
            for i in (0, 4):
                other["layers"][i]["mixer"]["left"]["bias_max"] = 20
        elif change == "scale":
            for i in (0, 4):
                other["layers"][i]["mixer"]["left"]["scale"] *= 1.3
        elif change == "pairs":
            other["embedding"]["bigram"]["mul_prev"] += 1
        elif change == "temp":
            weights["l0.mix.left.temp"] = torch.ones_like(W["l0.mix.left.temp"])
        elif change == "rel":
            weights["l0.mix.left.rel"] = W["l0.mix.left.rel"].flip(0)
        elif change == "hc_mix":
            weights["l1.hc1.mix"] = W["l1.hc1.mix"].T.contiguous()
        elif change == "hc_in":
            weights["l2.hc1.in"] = W["l2.hc1.in"].flip(0)
        elif change == "conv_b":
            weights["l1.mix.conv.b"] = torch.zeros_like(W["l1.mix.conv.b"])
        elif change == "D":
            weights["l1.mix.D"] = torch.zeros_like(W["l1.mix.D"])
        elif change == "left_out":
            weights["l0.mix.left.out"], weights["l0.mix.right.out"] = W["l0.mix.right.out"], W["l0.mix.left.out"]
        else:
            other["logit_scale"] = 1.0
        assert row_errors(plain.forward(other, weights, seq), want).max() > 1e-3, change


# ----------------------------------------------------------------------------------------------------------------
# every way of cutting the work
# ----------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,dtype", [("P", "float32"), ("Q", "float32"), ("R", "float32"), ("S", "float32"), ("P", "bfloat16"),
                                        ("Q", "bfloat16"), ("R", "bfloat16"), ("S", "bfloat16")])
def test_every_cutting_matches_the_plain_implementation(backend, folders, name, dtype):
    cfg = CONFIGS[name][0]
    lengths = (1, 2, 37, 70, 23) if backend == "cpu" else (1, 2, 37, 150, 23, 301)
    folder = folders(name, dtype)
    seqs = seqs_for(cfg, lengths)
    want = [plain_logits(folder, s) for s in seqs]
    traces = {"whole": U.whole_trace(seqs), "tail": U.tail_decode_trace(seqs, 20),
              "chunks": U.chunk_trace(seqs, sizes=(2, 3, 5, 17, 2, 16, 7, 32, 2, 31)), "mixed": U.mixed_trace(seqs, seed=5, max_live=3)}
    results = {}
    for kind, steps in traces.items():
        tokens = U.max_live_tokens(steps)
        r = runner_for(folder, dtype, backend, cache_tokens=tokens, max_live=3)
        got = U.replay(r, steps)
        r.cache.manager.check()
        assert r.cache.manager.live() == 0
        if kind == "mixed":
            assert r.cache.manager.reuse_count(r.cache.paged_groups()[0]) > 0, "the pool was too large: no page was used again"
        for i in range(len(seqs)):
            assert_rows(got[f"r{i}"], want[i], dtype, f"{name} {dtype} {kind} request {i}")
        results[kind] = got
    for kind in ("tail", "chunks", "mixed"):
        for i in range(len(seqs)):
            a, b = results["whole"][f"r{i}"], results[kind][f"r{i}"]
            assert_rows(b, a, dtype, f"{name} {dtype} {kind} against whole, request {i}", 1e-5 if dtype == "float32" else None)


def test_the_stream_after_every_layer(backend, folders):
    """Layer by layer: the sum of the stream's copies behind each layer, read from the engine's own buffers."""
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    seq = seqs_for(cfg, [19], seed=11)[0]
    layers = []
    plain_logits(folder, seq, layers)
    from denno_beta_amd.kernels import ops
    r = runner_for(folder, "float32", backend, 64)
    seen = []
    real = ops.streams_write

    def spy(xs, *a, **k):
        res = real(xs, *a, **k)
        seen.append(xs.detach().sum(dim=0).cpu().clone())
        return res
    ops.streams_write = spy
    try:
        U.replay(r, U.whole_trace([seq]))
    finally:
        ops.streams_write = real
    ends, n = [], 0
    for layer in cfg["layers"]:      # (a layer writes once per sublayer)
        n += 2 if layer.get("mlp") else 1
        ends.append(n - 1)
    assert len(seen) == n
    for i, want in enumerate(layers):
        d = (seen[ends[i]].double() - want).abs().max() / want.abs().max()
        assert d < 2e-5, f"the stream behind layer {i} differs by {d:.3g} of its largest entry"


# ----------------------------------------------------------------------------------------------------------------
# far tokens and chunk edges: weights made so that losing one token shows
# ----------------------------------------------------------------------------------------------------------------
MARKER = 7      # the token that the crafted layers look for


def _directions(tensors, seed):
    """Every token's row becomes a random vector of length about 1 plus 0.7 along a common direction u; the marker's row
    alone has a part along m (at right angles to u and to every other row).  No table of pairs disturbs them."""
    g = torch.Generator().manual_seed(seed)
    V, W = tensors["embed"].shape
    unit = lambda n: torch.nn.functional.normalize(torch.randn(n, generator=g), dim=0)   # noqa: E731
    u, m = unit(W), unit(W)
    m = torch.nn.functional.normalize(m - (m @ u) * u, dim=0)
    e = torch.randn(V, W, generator=g) / W ** 0.5
    e = e - torch.outer(e @ m, m) - torch.outer(e @ u, u)
    tensors["embed"] = e + 0.7 * u
    tensors["embed"][MARKER] += 2.0 * m
    if "bigram" in tensors:
        tensors["bigram"] = tensors["bigram"] * 0.01
    return u, m, g


def needle(tensors):
    """An attention that looks for one token wherever it lies in the chunk: every query points along a direction d (made
    from the common direction u), the marker's key alone has a large part along d (made from m), the bias by distance is
    nothing and the temperature high.  A key that is lost, misplaced, read from a wrong page or hidden by a chunk's edge
    that is one position off changes the rows behind it as much as a head can."""
    u, m, g = _directions(tensors, 1)
    q, k = tensors["l0.mix.left.q"], tensors["l0.mix.left.k"]
    d = torch.nn.functional.normalize(torch.randn(k.shape[0], generator=g), dim=0)
    reps = q.shape[0] // k.shape[0]
    tensors["l0.mix.left.q"] = torch.outer(d.repeat(reps), u) * 4.0
    tensors["l0.mix.left.k"] = k * 0.3 + torch.outer(d, m) * 4.0
    tensors["l0.mix.left.q.norm"] = torch.ones_like(tensors["l0.mix.left.q.norm"])
    tensors["l0.mix.left.k.norm"] = torch.ones_like(tensors["l0.mix.left.k.norm"])
    tensors["l0.mix.left.temp"] = torch.full_like(tensors["l0.mix.left.temp"], 6.0)
    tensors["l0.mix.left.rel"] = torch.zeros_like(tensors["l0.mix.left.rel"])
    tensors["l0.mix.left.o"] = tensors["l0.mix.left.o"] * 6.0
    tensors["l0.mix.left.out"] = tensors["l0.mix.left.out"] * 3.0
    tensors["l0.mix.right.out"] = tensors["l0.mix.right.out"] * 0.2


def imprint(tensors):
    """Recurrences that keep what one token wrote.  The gated recurrence's gate z is nearly shut for ordinary tokens (a bias
    far below zero) and open for the marker, whose candidate is large; the state-space layer hardly decays (A_log far below
    zero), steps little for ordinary tokens and far for the marker.  A state that is lost, started anew or taken from
    another slot changes every later row."""
    u, m, g = _directions(tensors, 2)
    n = tensors["l0.mix.right.z"].shape[0]
    tensors["l0.mix.right.z"] = torch.outer(torch.ones(n), 6.0 * m)
    tensors["l0.mix.right.z.b"] = torch.full((n,), -7.0)
    tensors["l0.mix.right.x"] = tensors["l0.mix.right.x"] + torch.outer(torch.rand(n, generator=g) + 0.5, 3.0 * m)
    tensors["l0.mix.right.out"] = tensors["l0.mix.right.out"] * 3.0
    tensors["l0.mix.left.out"] = tensors["l0.mix.left.out"] * 0.2
    H = tensors["l1.mix.A_log"].shape[0]
    tensors["l1.mix.A_log"] = torch.full((H,), -8.0)
    tensors["l1.mix.dt_bias"] = torch.full((H,), -4.0)
    w = tensors["l1.mix.in"]
    w[-H:] = torch.outer(torch.ones(H), 5.0 * m)      # (the step's rows are the last of the projection)
    tensors["l1.mix.in"] = w


FAR = {"attention": (config([with_mlp(parallel(2, 1, 16, 64, 8, far=100, buckets=8), None), with_mlp(parallel(2, 2, 8, 300, 8), None)],
                            width=32, vocab=71, streams=2), needle),
       "states": (config([with_mlp(parallel(2, 1, 8, 16, 24), None), with_mlp(mamba(2, 16, 16, 1, 3, 1), None)], width=32, vocab=71,
                         streams=2), imprint)}


@pytest.mark.parametrize("what", sorted(FAR))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_tokens_count(backend, folders, what, dtype):
    cfg, change = FAR[what]
    n = 90 if backend == "cpu" else 420
    folder = folders(f"far_{what}", dtype, cfg, 9, change)
    ordinary = [t if t != MARKER else MARKER + 1 for t in seqs_for(cfg, [n], seed=40)[0]]
    if what == "attention":
        # the last rows lie in the chunk that starts at the last multiple of 64: the marker at that chunk's first place, at a
        # page's last and first place inside it, and at the last place before it (which no row behind may see)
        start = (n - 1) // 64 * 64
        places = (start, start + 15, start + 16, start - 1)
    else:
        places = (0, 15, 16, 37)
    without = plain_logits(folder, ordinary)
    for at in places:
        seq = list(ordinary)
        seq[at] = MARKER
        want = plain_logits(folder, seq)
        # the test's own check: with an ordinary token there the last rows differ by far more than the bound allows (and,
        # for the place just outside the chunk, the first layer's attention must not see it: the rows behind stay close)
        moved = row_errors(without[-4:], want[-4:]).min()
        if what == "attention" and at == places[-1]:
            inside = list(ordinary)
            inside[at + 1] = MARKER
            assert row_errors(without[-4:], plain_logits(folder, inside)[-4:]).min() > 0.4
        else:
            assert moved > (0.4 if what == "attention" else 0.15), f"the marked token at {at} does not reach the last rows ({moved:.3g})"
        for kind, steps in (("whole", U.whole_trace([seq])), ("tail", U.tail_decode_trace([seq], 20)),
                            ("chunks", U.chunk_trace([seq], sizes=(15, 2, 16, 33, 1, 17))),
                            ("pages", U.chunk_trace([seq], sizes=(16, 16, 32, 1, 15, 48)))):
            if at != places[0] and kind in ("chunks", "pages") and backend == "cpu":
                continue          # (the host backend is slow)
            r = runner_for(folder, dtype, backend, U.max_live_tokens(steps))
            # (these weights are large on purpose, and so are the rounding errors: 32-bit sums, and bfloat16 scores under a
            # high temperature, gates that open steeply: a single row may be off by more than elsewhere, but no more than one in
            # fifty by more than the bound; losing the marker moves every row behind it)
            assert_rows(U.replay(r, steps)["r0"], want, dtype, f"far {what} {dtype} {kind}, the marker at {at}",
                        1e-4 if dtype == "float32" else 0.15 if what == "attention" else None, worst=0.3)


def test_chunk_edges_in_prompts_and_in_decoding(backend, folders):
    """Chunks of 13 positions on pages of 16 (and of 4): every row just behind and just before a chunk's edge, as part of a
    prompt and decoded alone, with the portions cut at, before and behind the edges."""
    cfg = CONFIGS["Q"][0]
    folder = folders("Q", "float32")
    seq = seqs_for(cfg, [60], seed=21)[0]
    want = plain_logits(folder, seq)
    for sizes in ((13, 13, 1, 12, 1, 1, 1), (12, 2, 11, 3, 25, 1, 1, 1), (14, 1, 1, 1, 9, 1, 1, 1, 1)):
        for page in (16, 4):
            steps = U.chunk_trace([seq], sizes=sizes)
            r = runner_for(folder, "float32", backend, U.max_live_tokens(steps), page_size=page)
            assert_rows(U.replay(r, steps)["r0"], want, "float32", f"portions of {sizes}, pages of {page}")


# ----------------------------------------------------------------------------------------------------------------
# the first tokens; slots given out again; a request beside others
# ----------------------------------------------------------------------------------------------------------------
def test_first_tokens_one_by_one(backend, folders):
    """Every token alone from the first: the first has no token before it, the convolutions' histories are shorter than
    their taps, the states start at zero, the first chunk has one key."""
    for name in ("R", "Q"):
        cfg = CONFIGS[name][0]
        folder = folders(name, "float32")
        seq = seqs_for(cfg, [9], seed=77)[0]
        want = plain_logits(folder, seq)
        steps = U.tail_decode_trace([seq], 9)
        r = runner_for(folder, "float32", backend, 64)
        assert_rows(U.replay(r, steps)["r0"], want, "float32", f"{name} token by token from the first")


def test_a_slot_given_out_again_starts_from_nothing(backend, folders):
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    a, b, c = seqs_for(cfg, [33, 21, 18], seed=90)
    r = runner_for(folder, "float32", backend, 64, max_live=1)
    steps = U.whole_trace([a]) + [dict(s, step=1 + i) for i, s in enumerate(U.chunk_trace([b], sizes=(5, 2, 9)))]
    for i, s in enumerate(steps[1:]):      # (other names than the first request's)
        s["entries"][0]["id"], s["end"] = "second", (["second"] if s["end"] else [])
    got = U.replay(r, steps)
    assert_rows(got["second"], plain_logits(folder, b), "float32", "the second request in the first one's slot")
    got = U.replay(r, [dict(U.whole_trace([c])[0], step=99)])
    assert_rows(got["r0"], plain_logits(folder, c), "float32", "the third")
    r.cache.manager.check()


def test_unequal_requests_together_equal_each_alone(backend, folders):
    cfg = CONFIGS["Q"][0]
    folder = folders("Q", "float32")
    seqs = seqs_for(cfg, [5, 40, 1, 17], seed=123)
    r = runner_for(folder, "float32", backend, 4 * 64)
    together = U.replay(r, [{"step": 0, "entries": [{"id": f"r{i}", "tokens": s, "want": list(range(len(s)))} for i, s in enumerate(seqs)],
                             "end": [f"r{i}" for i in range(len(seqs))]}])
    alone = U.replay(runner_for(folder, "float32", backend, 64), U.whole_trace(seqs))
    for i in range(len(seqs)):
        if backend == "cpu":     # (the host's library products sum in an order that depends on the batch)
            assert_rows(together[f"r{i}"], alone[f"r{i}"], "float32", f"request {i} beside the others", 1e-5)
        else:                    # every kernel sums a row in one order whatever else the step holds
            assert torch.equal(together[f"r{i}"], alone[f"r{i}"]), f"request {i}: 32-bit logits depend on the batch"


# ----------------------------------------------------------------------------------------------------------------
# generation through the engine's own entry point and scheduler
# ----------------------------------------------------------------------------------------------------------------
def test_greedy_generation_through_the_scheduler(backend, folders):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, SamplingParams
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    prompts = seqs_for(cfg, [3, 19, 11], seed=300)
    n_new = 10
    eng = Engine.from_folder(folder, EngineOptions(dtype="float32", device=backend, cache_tokens=4 * 64, max_live=2,
                                                   prefill_chunk=7, max_batch_tokens=16))
    got = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
    for p, g in zip(prompts, got):
        seq = list(p)
        for n, tok in enumerate(g):
            row = plain_logits(folder, seq)[-1]
            top = row.topk(2)
            if tok != int(top.indices[0]):
                assert float(top.values[0] - top.values[1]) < 1e-4 * float(row.std()), f"token {n} of {g}: the plain model says {int(top.indices[0])}"
            seq.append(tok)
        assert len(g) == n_new


def test_generation_with_few_pages_recomputes_what_it_gave_back(backend, folders):
    """A pool too small for all requests at once: the youngest gives its pages and its slot back and is run again from its
    known tokens, with the token before its first portion and its states started anew."""
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, SamplingParams
    cfg = CONFIGS["S"][0]
    folder = folders("S", "float32")
    prompts = seqs_for(cfg, [30, 28, 17], seed=310)
    eng = Engine.from_folder(folder, EngineOptions(dtype="float32", device=backend, cache_tokens=96, max_live=3, prefill_chunk=16,
                                                   max_batch_tokens=32))
    got = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    for p, g in zip(prompts, got):
        seq = list(p)
        for n, tok in enumerate(g):
            row = plain_logits(folder, seq)[-1]
            top = row.topk(2)
            if tok != int(top.indices[0]):
                assert float(top.values[0] - top.values[1]) < 1e-4 * float(row.std()), f"token {n} of {g}: the plain model says {int(top.indices[0])}"
            seq.append(tok)


# ----------------------------------------------------------------------------------------------------------------
# configuration and weights
# ----------------------------------------------------------------------------------------------------------------
def test_config_is_read_with_errors_that_name_the_key(folders):
    from denno_beta_amd.config import ConfigError, load_config, resolve_architecture
    from denno_beta_amd.models.dogalorn import DogalornConfig
    assert resolve_architecture({"architecture": "Dogalorn"}).config_cls is DogalornConfig
    for path, match in ((("layers", 0, "mixer", "left", "kv_heads"), "kv_heads"), (("layers", 0, "mixer", "left", "mask"), "mask"),
                        (("layers", 0, "mixer", "right"), "right"), (("layers", 1, "mixer", "state"), "state"),
                        (("layers", 1, "mixer", "norm_groups"), "norm_groups"), (("norm",), "norm"),
                        (("embedding", "bigram", "mul_cur"), "mul_cur"), (("layers", 0, "mlp", "ff"), "ff")):
        bad = copy.deepcopy(CFG_P)
        d = bad
        for key in path[:-1]:
            d = d[key]
        del d[path[-1]]
        with pytest.raises(ConfigError, match=match):
            DogalornConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][0]["type"] = "something"
    with pytest.raises(ConfigError, match="type"):
        DogalornConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][3]["weights_of"] = 4
    with pytest.raises(ConfigError, match="weights_of"):
        DogalornConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][0]["mixer"]["left"]["vdim"] = 4
    with pytest.raises(ConfigError, match="vdim"):
        DogalornConfig.from_dict(bad)
    # a size that only the tensors give: the rows of the table of distance biases come from the file, whatever config.json holds
    folder = folders("P", "float32")
    with open(os.path.join(folder, "config.json")) as f:
        stored = json.load(f)
    for layer in stored["layers"]:
        if layer["type"] == "parallel":
            del layer["mixer"]["left"]["bias_buckets"]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stored, f)
    _, cfg = load_config(folder)
    assert [l["mixer"]["left"]["bias_buckets"] for l in cfg.layers if l["type"] == "parallel"] == [8, 12, 8]


def test_a_checkpoint_that_does_not_fit_is_reported_whole(folders, tmp_path):
    from safetensors.torch import load_file, save_file
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.weights import CheckpointError
    import shutil
    d = str(tmp_path / "m")
    shutil.copytree(folders("R", "float32"), d)
    tensors = load_file(os.path.join(d, "model.safetensors"))
    del tensors["l0.mix.right.x.b"]
    tensors["l1.hc1.mix"] = tensors["l1.hc1.mix"].reshape(-1).contiguous()
    tensors["stray"] = torch.zeros(3)
    save_file(tensors, os.path.join(d, "model.safetensors"))
    with pytest.raises(CheckpointError) as e:
        ModelRunner.from_folder(d, EngineOptions(dtype="float32", device="cpu", cache_tokens=64, max_live=1))
    assert "l0.mix.right.x.b" in e.value.missing and "stray" in e.value.unexpected and e.value.wrong_shape[0][0] == "l1.hc1.mix"


# ----------------------------------------------------------------------------------------------------------------
# the command line and the trace runner as child processes; a long run of decoded tokens
# ----------------------------------------------------------------------------------------------------------------
def plain_greedy(folder, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(plain_logits(folder, seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.gpu
def test_command_line_generates_what_the_plain_model_does(folders):
    import subprocess
    import sys
    from conftest import ROOT
    folder = folders("R", "float32")
    prompt = seqs_for(CONFIGS["R"][0], [7], seed=410)[0]
    want = plain_greedy(folder, prompt, 6)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "denno"), "generate", folder, "--prompt-ids",
                          ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0", "--quant", "fp32", "--raw",
                          "--cache-tokens", "128"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.strip().split(",")] == want


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_as_a_child_process(folders, tmp_path, dtype):
    """bin/trace_run on a mixed trace with four state slots: the files it writes against the plain implementation."""
    import subprocess
    from conftest import ROOT
    cfg = CONFIGS["P"][0]
    folder = folders("P", dtype)
    seqs = seqs_for(cfg, [90, 3, 41, 17, 64, 29, 5], seed=500)
    steps = U.mixed_trace(seqs, seed=3, max_live=4)
    out = str(tmp_path / "out")
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out, "--max-tokens",
                        str(U.max_live_tokens(steps))], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    got = U.collect_files(out, steps, cfg["vocab"])
    for i, s in enumerate(seqs):
        assert_rows(got[f"r{i}"], plain_logits(folder, s), dtype, f"trace_run {dtype} request {i}")


def test_two_hundred_decoded_tokens(backend, folders):
    """A short prompt, then token after token for long: pages fill and new ones are taken, chunks end and begin, the states
    run on."""
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    n = 60 if backend == "cpu" else 230
    seq = seqs_for(cfg, [n], seed=600)[0]
    steps = U.tail_decode_trace([seq], n - 4)
    r = runner_for(folder, "float32", backend, U.max_live_tokens(steps))
    assert_rows(U.replay(r, steps)["r0"], plain_logits(folder, seq), "float32", "long decoding")
