"""Nigilorn through the engine against the plain implementation (tests/plain/nigilorn_plain.py): each mechanism alone,
every way of cutting the work, windows' edges, first tokens, far tokens, long decoding, slots and pages used again, other
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
from plain import nigilorn_plain as plain


# ----------------------------------------------------------------------------------------------------------------
# configurations: each differs from the others in every size
# ----------------------------------------------------------------------------------------------------------------
def scan(inner=24, state=6, dt_rank=3, conv=3):
    return dict(type="mamba1", mixer=dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv))


def scaling(factor=4.0, original=64, fast=8.0, slow=1.0):
    return dict(factor=factor, original=original, fast=fast, slow=slow)


def attention(heads=4, kv_heads=2, dim=16, vdim=8, dims=8, base=10000.0, scale=None, window=20, scaled=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 0.9 * dim ** -0.5)
    if dims is not None:
        m["rot"] = dict(base=base, dims=dims)
        if scaled:
            m["rot"]["scaling"] = scaled
    if window:
        m["mask"] = dict(size=window)
    return dict(type="attention", mixer=m)


def latent(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=12, base=5000.0, scale=None, window=20, scaled=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale if scale is not None else (dim + rot_dim) ** -0.5,
             rot=dict(base=base, dims=rot_dim))
    if scaled:
        m["rot"]["scaling"] = scaled
    if window:
        m["mask"] = dict(size=window)
    return dict(type="latent_attention", mixer=m)


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def moe(ff=24, experts=6, top=2, groups=(3, 2), scale=1.5, shared=16):
    m = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale))
    if groups:
        m["router"]["groups"] = dict(count=groups[0], keep=groups[1])
    if shared:
        m["shared"] = dict(ff=shared)
    return m


def config(layers, width=32, vocab=97, eps=1e-5, side=6):
    c = dict(architecture="Nigilorn", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)
    if side:
        c["token_side"] = dict(dim=side)
    return c


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


# every mixer and both feed-forwards; grouped key heads; part of a head turned, with a stretched encoding; windows that are
# no multiple of a page; a layer without a feed-forward
CFG_P = config([with_mlp(scan(24, 6, 3, 3), dense(40)),
                with_mlp(attention(4, 2, 16, 8, dims=8, window=23, scaled=scaling(4.0, 64, 8.0, 1.0)), moe(24, 6, 2, (3, 2), 1.5, 16)),
                with_mlp(latent(3, 8, 4, 12, 12, window=37, scaled=scaling(2.0, 32, 4.0, 0.5)), dense(24)),
                with_mlp(scan(40, 17, 5, 2), None)], width=32, vocab=97, side=6)
# other sizes: one key head; values wider than keys; a head size that no 16 divides; one tap; a whole head turned without
# stretching; a window shorter than a page and one that never closes; one expert of four in all groups; no shared expert;
# no token input; another order of layers
CFG_Q = config([with_mlp(latent(2, 12, 6, 5, 20, base=300.0, window=5), moe(16, 4, 1, None, 1.0, None)),
                with_mlp(scan(16, 1, 1, 1), None),
                with_mlp(attention(3, 1, 24, 40, dims=24, base=300.0, scale=0.31, window=0), dense(20)),
                with_mlp(attention(2, 2, 8, 4, dims=None, window=16), moe(40, 6, 3, (2, 1), 2.5, 8)),
                with_mlp(scan(56, 33, 7, 5), dense(56))], width=48, vocab=131, eps=1e-6, side=0)
# sizes that are multiples of nothing: a width of 36, heads of 6 and 10, a token input of one column
CFG_R = config([with_mlp(attention(2, 1, 10, 6, dims=4, window=9, scaled=scaling(8.0, 16, 2.0, 1.0)), moe(12, 9, 3, (3, 1), 0.7, 20)),
                with_mlp(scan(21, 5, 2, 4), dense(9)),
                with_mlp(latent(5, 6, 2, 10, 7, window=50), moe(8, 2, 2, (2, 2), 1.0, None))], width=36, vocab=61, side=1)
# sizes nearer a small model's: heads of 32 and 48, a kept key of 96, windows of about a hundred, twelve experts in three groups
CFG_S = config([with_mlp(latent(4, 32, 16, 48, 80, base=20000.0, window=100, scaled=scaling(2.0, 256, 16.0, 2.0)), dense(320)),
                with_mlp(scan(320, 24, 12, 3), moe(48, 12, 4, (3, 2), 2.0, 96)),
                with_mlp(attention(6, 3, 48, 32, dims=24, base=100000.0, window=130, scaled=scaling(3.0, 128, 24.0, 1.0)), moe(48, 12, 4, (3, 2), 2.0, 96)),
                with_mlp(scan(320, 24, 12, 3), dense(160))], width=192, vocab=300, side=12)
CONFIGS = {"P": (CFG_P, 31), "Q": (CFG_Q, 32), "R": (CFG_R, 33), "S": (CFG_S, 34)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from denno_beta_amd.weights import write_model_folder
    made = {}

    def get(name, dtype="float32", cfg=None, seed=None, change=None):
        key = (name, dtype)
        if key not in made:
            c, s = CONFIGS[name] if cfg is None else (cfg, seed)
            d = str(tmp_path_factory.mktemp(f"nigilorn{name}_{dtype}"))
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


def runner_for(folder, dtype, device, cache_tokens, max_live=4, page_size=16, graphs=True):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, device=device, page_size=page_size,
                                                         cache_tokens=cache_tokens, max_live=max_live, use_graphs=graphs))


_plain = {}


def plain_model(folder):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {k: (v.double() if v.is_floating_point() else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def plain_logits(folder, seq, layers=None):
    key = (folder, tuple(seq))
    if key not in _plain or layers is not None:
        cfg, w = plain_model(folder)
        logits, streams = plain.forward(seq, cfg, w, return_layers=True)
        if layers is not None:
            layers.extend(streams)
        _plain[key] = logits
    return _plain[key]


def row_errors(got, want):
    """Per position: the root mean square of the difference (its mean taken off) over the spread of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(dim=1, keepdim=True)
    return torch.sqrt((d * d).mean(dim=1)) / want.double().std(dim=1)


# bfloat16, in models 32 to 48 wide: a typical row is off by 0.01 of its spread; a row in thirty by several times that (a
# sublayer's result passes a gate and a norm of its own on its way into the stream, and an expert squares what it made, which
# doubles a rounding error's share), so one row in twenty may pass the bound, none by more than two and a half times; a fault
# moves rows by 0.2 and more
BOUND = {"float32": 2e-5, "bfloat16": 0.06}
BF16_OVER, BF16_WORST = 0.05, 0.15
# bfloat16: a router's choice between two experts whose scores are close may fall the other way under rounding, which
# moves that row, and through states and keys later rows, by as much as a fault would.  The bfloat16 models of these
# tests therefore let every token use all its experts (`all_experts`): the same kernels run, no choice can turn, and
# every row keeps the bound.  The choice itself is tested in 32-bit.


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


def all_experts(cfg):
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer.get("mlp") and layer["mlp"]["kind"] == "moe":
            ro = layer["mlp"]["router"]
            ro["top"] = ro["experts"]
            if ro.get("groups"):
                ro["groups"]["keep"] = ro["groups"]["count"]
    return cfg


# ----------------------------------------------------------------------------------------------------------------
# the plain implementation against itself, and the engine's own constants against it
# ----------------------------------------------------------------------------------------------------------------
def test_plain_pieces():
    g = torch.Generator().manual_seed(0)
    # the convolution's last column weighs the token itself, its first the token taps - 1 before; the bias is added
    x = torch.randn(5, 2, generator=g, dtype=torch.float64)
    w = torch.zeros(2, 3, dtype=torch.float64)
    w[:, 2] = 1.0
    b = torch.tensor([0.5, -1.0], dtype=torch.float64)
    assert torch.allclose(plain.causal_taps(x, w, b), x + b)
    w = torch.zeros(2, 3, dtype=torch.float64)
    w[:, 0] = 1.0
    y = plain.causal_taps(x, w, torch.zeros(2, dtype=torch.float64))
    assert torch.equal(y[2:], x[:3]) and float(y[:2].abs().sum()) == 0.0
    # a window of n: the row itself and the n - 1 before it
    p = plain.window_softmax(torch.zeros(1, 6, 6, dtype=torch.float64), 3)[0]
    assert torch.allclose(p[5], torch.tensor([0, 0, 0, 1 / 3, 1 / 3, 1 / 3], dtype=torch.float64))
    assert torch.allclose(p[1], torch.tensor([0.5, 0.5, 0, 0, 0, 0], dtype=torch.float64))
    assert torch.allclose(plain.window_softmax(torch.zeros(1, 4, 4, dtype=torch.float64), None)[0][3], torch.full((4,), 0.25, dtype=torch.float64))
    # the stretched encoding: a factor of 1 changes nothing; fast pairs stay and slow ones are slowed down by the factor
    f0, m0 = plain.yarn_frequencies(16, 10000.0, None)
    f1, m1 = plain.yarn_frequencies(16, 10000.0, dict(factor=1.0, original=64, fast=8.0, slow=1.0))
    assert torch.allclose(f0, f1) and m0 == 1.0 and m1 == 1.0
    f4, m4 = plain.yarn_frequencies(16, 10000.0, dict(factor=4.0, original=64, fast=8.0, slow=1.0))
    assert abs(m4 - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    assert float(f4[0]) == float(f0[0]) and abs(float(f4[-1]) - float(f0[-1]) / 4) < 1e-18
    assert bool((f4 <= f0 + 1e-18).all()) and bool((f4 >= f0 / 4 - 1e-18).all())
    # a turn keeps a pair's length (times the factor) and turns nothing at position 0 but for the factor
    v = torch.randn(3, 2, 8, generator=g, dtype=torch.float64)
    rot = dict(base=100.0, dims=4, scaling=dict(factor=3.0, original=16, fast=4.0, slow=1.0))
    t = plain.turn_pairs(v, torch.tensor([0, 7, 1000]), rot)
    mag = 0.1 * math.log(3.0) + 1.0
    assert torch.allclose(t[..., 4:], v[..., 4:]) and torch.allclose(t[0, :, :4], v[0, :, :4] * mag)
    assert torch.allclose(t[..., :4].pow(2).sum(-1), v[..., :4].pow(2).sum(-1) * mag * mag)
    # the choice of experts: only the kept groups' experts; a group's score is the sum of its two largest
    s = torch.tensor([0.9, 0.1, 0.1, 0.6, 0.6, 0.1, 0.5, 0.5, 0.5], dtype=torch.float64)        # groups of 3: 1.0, 1.2, 1.0
    assert sorted(plain.choose_experts(s, 2, 3, 1).tolist()) == [3, 4]
    assert plain.choose_experts(s, 1, 1, 1).tolist() == [0]
    assert set(plain.choose_experts(s, 3, 3, 2).tolist()) <= {0, 1, 2, 3, 4}
    # the selective scan with a decay of one (A_log far below zero) adds up what the tokens write
    inner, N, T = 3, 2, 4
    pw = {"in": torch.randn(2 * inner, 5, generator=g, dtype=torch.float64), "conv": torch.ones(inner, 1, dtype=torch.float64),
          "conv.b": torch.zeros(inner, dtype=torch.float64), "x": torch.randn(1 + 2 * N, inner, generator=g, dtype=torch.float64),
          "dt": torch.randn(inner, 1, generator=g, dtype=torch.float64), "dt.b": torch.zeros(inner, dtype=torch.float64),
          "A_log": torch.full((inner, N), -40.0, dtype=torch.float64), "D": torch.zeros(inner, dtype=torch.float64),
          "o": torch.eye(inner, dtype=torch.float64)}
    h = torch.randn(T, 5, generator=g, dtype=torch.float64)
    y = plain.mamba1(h, pw.__getitem__, dict(inner=inner, state=N, dt_rank=1, conv=1))
    xz = h @ pw["in"].T
    xs, z = plain.silu(xz[:, :inner]), xz[:, inner:]
    low = xs @ pw["x"].T
    dt = plain.softplus(low[:, :1] @ pw["dt"].T)
    S = torch.zeros(inner, N, dtype=torch.float64)
    for t in range(T):
        S = S + (dt[t] * xs[t])[:, None] * low[t, 1:1 + N][None, :]
        assert torch.allclose(y[t], (S @ low[t, 1 + N:]) * plain.silu(z[t]), atol=1e-12)


@pytest.mark.parametrize("dims,base,sc", [(8, 10000.0, scaling(4.0, 64, 8.0, 1.0)), (4, 5000.0, scaling(2.0, 32, 4.0, 0.5)), (24, 300.0, None),
                                          (16, 250000.0, scaling(1.0, 128, 32.0, 1.0)), (2, 10.0, scaling(8.0, 16, 2.0, 1.0)),
                                          (64, 1e6, scaling(16.0, 4096, 32.0, 1.0))])
def test_frequencies_of_the_stretched_encoding(dims, base, sc):
    from denno_beta_amd.parts.positions import RotaryPairs
    part = RotaryPairs(dims=dims, base=base, head_dim=dims, scaling=sc)
    want, mag = plain.yarn_frequencies(dims, base, sc)
    assert torch.allclose(part.frequencies(), want, rtol=1e-14, atol=0) and abs(part.mag - mag) < 1e-15


# ----------------------------------------------------------------------------------------------------------------
# each mechanism alone
# ----------------------------------------------------------------------------------------------------------------
ALONE = {
    "scan": [with_mlp(scan(20, 4, 2, 3), None)],
    "scan_one_state_one_tap": [with_mlp(scan(9, 1, 1, 1), None)],
    "scan_many_states": [with_mlp(scan(7, 37, 4, 2), None)],
    "attention": [with_mlp(attention(4, 2, 8, 8, dims=8, window=0), None)],
    "attention_window": [with_mlp(attention(2, 2, 8, 8, dims=4, window=7), None)],
    "attention_stretched": [with_mlp(attention(2, 1, 12, 20, dims=6, window=0, scaled=scaling(4.0, 16, 3.0, 0.5)), None)],
    "attention_not_turned": [with_mlp(attention(3, 3, 16, 8, dims=None, window=11), None)],
    "latent": [with_mlp(latent(2, 8, 4, 8, 8, window=0), None)],
    "latent_window_stretched": [with_mlp(latent(3, 6, 6, 10, 5, window=6, scaled=scaling(3.0, 8, 2.0, 1.0)), None)],
    # a latent too wide for one key of the attention kernels: every head's own keys and values are kept instead
    "latent_kept_by_heads": [with_mlp(latent(2, 8, 4, 12, 262, window=9), None)],
    "dense": [with_mlp(scan(8, 2, 1, 2), dense(28))],
    "experts": [with_mlp(scan(8, 2, 1, 2), moe(12, 6, 3, None, 1.0, None))],
    "experts_in_groups": [with_mlp(scan(8, 2, 1, 2), moe(12, 8, 2, (4, 2), 2.0, None))],
    "experts_one_group_kept_with_shared": [with_mlp(scan(8, 2, 1, 2), moe(12, 6, 1, (3, 1), 0.5, 20))],
}


@pytest.mark.parametrize("side", [0, 5])
@pytest.mark.parametrize("what", sorted(ALONE))
def test_each_mechanism_alone(backend, folders, what, side):
    cfg = config(ALONE[what], width=24, vocab=53, side=side)
    folder = folders(f"alone_{what}_{side}", "float32", cfg, 5)
    seq = seqs_for(cfg, [29])[0]
    want = plain_logits(folder, seq)
    r = runner_for(folder, "float32", backend, 64)
    assert_rows(U.replay(r, U.whole_trace([seq]))["r0"], want, "float32", what)
    r = runner_for(folder, "float32", backend, 64)
    assert_rows(U.replay(r, U.chunk_trace([seq], sizes=(2, 5, 1, 9, 3)))["r0"], want, "float32", what + " in portions")


def test_what_the_model_fixes_matters(folders):
    """The constants and orders that the plain model is built from change its logits: a test against it would see them."""
    cfg0 = CFG_P
    folder = folders("P", "float32")
    _, W = plain_model(folder)
    seq = seqs_for(cfg0, [45])[0]
    want = plain_logits(folder, seq)
    for change in ("window", "scaling", "router_scale", "groups", "rg", "rg_bias", "side", "eps", "A", "D", "head_gate", "dkv_norm"):
        other, weights = copy.deepcopy(cfg0), dict(W)
        if change == "window":
            other["layers"][1]["mixer"]["mask"]["size"] += 1
        elif change == "scaling":
            del other["layers"][1]["mixer"]["rot"]["scaling"]
        elif change == "router_scale":
            other["layers"][1]["mlp"]["router"]["scale"] = 1.0
        elif change == "groups":
            other["layers"][1]["mlp"]["router"]["groups"] = dict(count=1, keep=1)
        elif change == "rg":
            weights["l0.rg1"] = torch.zeros_like(W["l0.rg1"])
        elif change == "rg_bias":
            weights["l2.rg2.b"] = torch.zeros_like(W["l2.rg2.b"])
        elif change == "side":
            del other["token_side"]
        elif change == "eps":
            other["norm"]["eps"] = 1e-2
        elif change == "A":
            weights["l0.mix.A_log"] = W["l0.mix.A_log"] + 1.0
        elif change == "D":
            weights["l3.mix.D"] = torch.zeros_like(W["l3.mix.D"])
        elif change == "head_gate":
            weights["l1.mix.g"] = torch.zeros_like(W["l1.mix.g"])
        else:
            weights["l2.mix.dkv.norm"] = torch.ones_like(W["l2.mix.dkv.norm"])
        assert row_errors(plain.forward(seq, other, weights), want).max() > 1e-3, change


# ----------------------------------------------------------------------------------------------------------------
# every way of cutting the work
# ----------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,dtype", [("P", "float32"), ("Q", "float32"), ("R", "float32"), ("S", "float32"), ("P", "bfloat16"),
                                        ("Q", "bfloat16"), ("R", "bfloat16"), ("S", "bfloat16")])
def test_every_cutting_matches_the_plain_implementation(backend, folders, name, dtype):
    cfg = CONFIGS[name][0]
    lengths = ((1, 2, 37, 70, 23) if name != "S" else (2, 40)) if backend == "cpu" else (1, 2, 37, 150, 23, 301)
    if dtype == "bfloat16":
        cfg = all_experts(cfg)
        if cfg.get("token_side", {}).get("dim") == 1:
            # (a token input of one column is a fixed vector times the sign of one number, which a rounding can turn; one of
            # a few columns is all rounding where all of them are nearly zero, since it is normed)
            cfg["token_side"]["dim"] = 8
    folder = folders(name, dtype, cfg, CONFIGS[name][1])
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
            assert max(r.cache.manager.reuse_count(g) for g in r.cache.paged_groups()) > 0, "the pool was too large: no page was used again"
        for i in range(len(seqs)):
            # (bfloat16: a sublayer's result is normed on its way into the stream, so a row where a result is small beside
            # the terms it is the sum of is rounding scaled up: in models this narrow it happens to a row in a few hundred,
            # which then is off by as much as its spread; the share of rows over the bound is what a fault would move, and
            # the 32-bit runs hold every row)
            assert_rows(got[f"r{i}"], want[i], dtype, f"{name} {dtype} {kind} request {i}", worst=1.0)
        results[kind] = got
    for kind in ("tail", "chunks", "mixed"):
        for i in range(len(seqs)):
            a, b = results["whole"][f"r{i}"], results[kind][f"r{i}"]
            assert_rows(b, a, dtype, f"{name} {dtype} {kind} against whole, request {i}", 1e-5 if dtype == "float32" else None, worst=1.0)


def test_the_stream_after_every_layer(backend, folders):
    """Layer by layer: the stream behind each layer (behind its token input), read from the engine's own rows."""
    from denno_beta_amd.parts.blocks import GatedSandwichBlock
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    seq = seqs_for(cfg, [19], seed=11)[0]
    streams = []
    plain_logits(folder, seq, streams)
    r = runner_for(folder, "float32", backend, 64)
    seen = []
    real = GatedSandwichBlock.forward

    def spy(self, x, ctx, caches, runtime):
        real(self, x, ctx, caches, runtime)
        seen.append(x.detach().cpu().clone())
    GatedSandwichBlock.forward = spy
    try:
        U.replay(r, U.whole_trace([seq]))
    finally:
        GatedSandwichBlock.forward = real
    assert len(seen) == len(cfg["layers"])
    for i, want in enumerate(streams):
        d = (seen[i].double() - want).abs().max() / want.abs().max()
        assert d < 2e-5, f"the stream behind layer {i} differs by {d:.3g} of its largest entry"


def test_norms_in_front_of_sublayers_come_out_of_the_kernels_before(backend, folders):
    """The norm in front of a sublayer is made by the kernel that takes the sublayer before it into the stream: a whole step
    launches the norm's own kernel for the first layer and for the head only, and the logits are those of the norms as
    kernels of their own (on the GPU the same bits)."""
    from denno_beta_amd.kernels import ops
    from denno_beta_amd.parts import norms, token_inputs
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    seqs = seqs_for(cfg, [21, 70], seed=15)
    steps = U.whole_trace(seqs) + [dict(s, step=10 + i) for i, s in enumerate(U.tail_decode_trace([seqs[0]], 5))]
    for i, s in enumerate(steps[2:]):
        s["entries"][0]["id"], s["end"] = "again", (["again"] if s["end"] else [])
    for dtype in ("float32", "bfloat16"):
        calls = []
        real, real_following = ops.rmsnorm, norms.following_norm

        def spy(x, weight, eps, out, rows=None):
            if out.shape[1] == cfg["width"]:
                calls.append(out.shape[0])
            return real(x, weight, eps, out, rows)
        ops.rmsnorm = spy
        try:
            fused = U.replay(runner_for(folder, dtype, backend, 256, graphs=False), steps)      # (every step kernel by kernel)
            per_step = len(calls) / len(steps)
            norms.following_norm = lambda norm, x, out_dtype: None
            apart = U.replay(runner_for(folder, dtype, backend, 256), steps)
        finally:
            ops.rmsnorm, norms.following_norm = real, real_following
        assert per_step == 2, f"{per_step} norm kernels a step; the first layer's and the head's are two"
        for rid in fused:
            if backend == "cpu":
                assert_rows(fused[rid], apart[rid], "float32", f"{dtype} {rid}", 1e-5 if dtype == "float32" else 0.02)
            elif dtype == "float32":
                assert torch.equal(fused[rid], apart[rid]), f"{rid}: the norm inside the kernel before gives other bits"
            else:       # (the token input of few rows sums a row over sixteen waves, the norm's own kernel over four)
                assert_rows(fused[rid], apart[rid], "float32", f"{dtype} {rid}", 0.02)


# ----------------------------------------------------------------------------------------------------------------
# far tokens and windows' edges: weights made so that losing one token, or seeing one too many, shows
# ----------------------------------------------------------------------------------------------------------------
MARKER = 7      # the token that the crafted layers look for
NEEDLE_DIM = 16             # the crafted attention's head size
LATENT_DIM, LATENT_ROT = 8, 8      # the crafted latent attention's plain and turned dimensions a head


def _directions(tensors, seed):
    """Every token's row becomes a random vector of length about 1 plus 0.7 along a common direction u; the marker's row
    alone has a part along m (at right angles to u and to every other row)."""
    g = torch.Generator().manual_seed(seed)
    V, W = tensors["embed"].shape
    unit = lambda n: torch.nn.functional.normalize(torch.randn(n, generator=g), dim=0)   # noqa: E731
    u, m = unit(W), unit(W)
    m = torch.nn.functional.normalize(m - (m @ u) * u, dim=0)
    e = torch.randn(V, W, generator=g) / W ** 0.5
    e = e - torch.outer(e @ m, m) - torch.outer(e @ u, u)
    tensors["embed"] = e + 0.7 * u
    tensors["embed"][MARKER] += 2.0 * m
    tensors["l0.norm1"] = torch.ones_like(tensors["l0.norm1"])
    return u, m, g


def needle(tensors):
    """An attention whose first head looks for one token wherever it lies in its window: every query points along d (made
    from the common direction u), the marker's key alone has a part along d (made from m), and every key of that key head
    has the same part along c, at right angles to d; d lies in the pair of dimensions that the position turns slowest, c
    in the fastest.  Behind the norm of q and k the marker's score is large, the others' zero.  A key that is lost, misplaced, read from a wrong page or seen from
    outside the window changes a row as much as one head can."""
    u, m, g = _directions(tensors, 1)
    q, k = tensors["l0.mix.q"], tensors["l0.mix.k"]
    dk = NEEDLE_DIM      # (the first query head and the only key head)
    d = torch.zeros(dk)
    d[-2:] = torch.tensor([0.6, 0.8])
    c = torch.zeros(dk)
    c[:2] = torch.tensor([0.8, -0.6])
    q[:dk] = 8.0 * torch.outer(d, u)
    k[:dk] = 4.0 * torch.outer(d, m) + 4.0 * torch.outer(c, u)
    tensors["l0.mix.v"] = tensors["l0.mix.v"] * 20.0
    tensors["l0.mix.g"] = torch.zeros_like(tensors["l0.mix.g"])       # (every head's gate at one half)
    tensors["l0.rg1"] = torch.zeros_like(tensors["l0.rg1"])
    tensors["l0.rg1.b"] = torch.full_like(tensors["l0.rg1.b"], 3.0)


def latent_needle(tensors):
    """The same in a latent attention: the first head's turned query part points along d, the marker's shared turned key
    part alone has a part along d."""
    u, m, g = _directions(tensors, 4)
    q, dkv = tensors["l0.mix.q"], tensors["l0.mix.dkv"]
    rot = LATENT_ROT
    plain_dims = LATENT_DIM
    d = torch.zeros(rot)
    d[-2:] = torch.tensor([0.6, 0.8])
    q[plain_dims:plain_dims + rot] = 3.0 * torch.outer(d, u)
    dkv[-rot:] = 2.0 * torch.outer(d, m)
    tensors["l0.mix.uv"] = tensors["l0.mix.uv"] * 10.0
    tensors["l0.rg1"] = torch.zeros_like(tensors["l0.rg1"])
    tensors["l0.rg1.b"] = torch.full_like(tensors["l0.rg1.b"], 3.0)


def imprint(tensors):
    """A selective scan that keeps what one token wrote: the decays are nearly one (A_log far below zero), and the marker's
    channels are several times an ordinary token's, so its product with B stays a large part of the state and is read by
    every later token (not so many times that the state is this one product alone: every channel would then read it
    through the same number, and a row where that number is small would be all rounding).  A state that is lost, started
    anew or taken from another slot changes every later row."""
    u, m, g = _directions(tensors, 2)
    inner = tensors["l0.mix.conv"].shape[0]
    tensors["l0.mix.in"][:inner] += 0.8 * torch.outer(torch.rand(inner, generator=g) + 0.5, m)
    tensors["l0.mix.A_log"] = torch.full_like(tensors["l0.mix.A_log"], -9.0)
    tensors["l0.mix.dt.b"] = torch.full_like(tensors["l0.mix.dt.b"], -2.0)
    tensors["l0.rg1"] = torch.zeros_like(tensors["l0.rg1"])
    tensors["l0.rg1.b"] = torch.full_like(tensors["l0.rg1.b"], 3.0)


WINDOW = 40
FAR = {"attention": (config([with_mlp(attention(2, 1, NEEDLE_DIM, 16, dims=16, base=1e6, scale=1.0, window=WINDOW), None)],
                            width=32, vocab=71, side=3), needle),
       "latent": (config([with_mlp(latent(2, LATENT_DIM, LATENT_ROT, 16, 24, base=1e6, scale=0.05, window=WINDOW), None)],
                         width=32, vocab=71, side=3), latent_needle),
       "states": (config([with_mlp(scan(32, 8, 4, 3), None), with_mlp(scan(16, 4, 2, 2), None)], width=32, vocab=71, side=0), imprint)}


@pytest.mark.parametrize("what", ["attention", "latent"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_edge_of_a_window(backend, folders, what, dtype):
    """One layer, so that a row sees the marked token through the attention alone: the row `window - 1` behind it must, the
    row `window` behind it must not, in a prompt, in portions cut at, before and behind the edge, and in decoded tokens."""
    cfg, change = FAR[what]
    folder = folders(f"far_{what}", dtype, cfg, 9, change)
    n = 100
    ordinary = [t if t != MARKER else MARKER + 1 for t in seqs_for(cfg, [n], seed=40)[0]]
    for at in (0, 15, 16, 29):       # the first place, a page's last and first place, the middle of one
        seq = list(ordinary)
        seq[at] = MARKER
        want, without = plain_logits(folder, seq), plain_logits(folder, ordinary)
        inside, outside = at + WINDOW - 1, at + WINDOW
        # the test's own check: the last row inside the window depends on the marker, the first outside does not at all
        e = row_errors(without, want)
        assert e[at + 1:inside + 1].min() > 0.15 and e[outside:].max() < 1e-9, "the crafted weights do not show the window's edge"
        cuts = {"whole": U.whole_trace([seq]), "tail": U.tail_decode_trace([seq], n - at - 3),
                "at_the_edge": U.chunk_trace([seq], sizes=(inside, 1, 1, 1000)),
                "around": U.chunk_trace([seq], sizes=(outside, 2, 1000) if at else (inside - 1, 3, 2, 1000)),
                "pages": U.chunk_trace([seq], sizes=(16, 16, 32, 1, 15, 48))}
        for kind, steps in cuts.items():
            if backend == "cpu" and at not in (0, 16) and kind in ("around", "pages"):
                continue          # (the host backend is slow)
            r = runner_for(folder, dtype, backend, U.max_live_tokens(steps))
            got = U.replay(r, steps)["r0"]
            assert_rows(got, want, dtype, f"window {what} {dtype} {kind}, the marker at {at}", 1e-4 if dtype == "float32" else None)
            # sharper at the two rows: each is far nearer to the model with the right window than to one that is off by one
            right = row_errors(got[[inside, outside]], want[[inside, outside]])
            assert right[0] < 0.05 and right[1] < 0.05, (kind, at, right)
            assert row_errors(got[[inside]], without[[inside]])[0] > 0.1, f"{kind}: the row at the window's edge lost the marked token"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_tokens_count(backend, folders, dtype):
    cfg, change = FAR["states"]
    n = 90 if backend == "cpu" else 400
    folder = folders("far_states", dtype, cfg, 9, change)
    ordinary = [t if t != MARKER else MARKER + 1 for t in seqs_for(cfg, [n], seed=40)[0]]
    for at in (0, 15, 16, 37):
        seq = list(ordinary)
        seq[at] = MARKER
        want = plain_logits(folder, seq)
        without = plain_logits(folder, ordinary)
        assert row_errors(without[-8:], want[-8:]).min() > 0.15, "the marked token does not reach the last rows"
        for kind, steps in (("whole", U.whole_trace([seq])), ("tail", U.tail_decode_trace([seq], 40)),
                            ("chunks", U.chunk_trace([seq], sizes=(15, 2, 16, 33, 1, 17))),
                            ("pages", U.chunk_trace([seq], sizes=(16, 16, 32, 1, 15, 48)))):
            if at not in (0, 16) and kind in ("chunks", "pages") and backend == "cpu":
                continue
            r = runner_for(folder, dtype, backend, U.max_live_tokens(steps))
            # (weights made large on purpose round coarsely: a single row may be off by a quarter of its spread; a lost state
            # moves every row behind it by more than the bound)
            assert_rows(U.replay(r, steps)["r0"], want, dtype, f"far states {dtype} {kind}, the marker at {at}",
                        1e-4 if dtype == "float32" else None, worst=0.25)


def test_pages_behind_a_window_are_given_back(backend, folders):
    """A request much longer than its windows runs in a pool that holds a few windows: pages that every window has passed
    are used again, by the request itself and by its neighbour."""
    # (a token input of few columns is all rounding where all of them are nearly zero: it is normed; hence five columns)
    cfg = config([with_mlp(attention(2, 1, 8, 8, dims=4, window=9), None), with_mlp(latent(2, 8, 4, 8, 8, window=20), dense(16))],
                 width=24, vocab=53, side=5)
    folder = folders("windows_only", "float32", cfg, 17)
    n = 150 if backend == "cpu" else 400
    seqs = seqs_for(cfg, [n, n // 2], seed=70)
    steps = U.mixed_trace(seqs, seed=2, max_live=2, sizes=(1, 1, 2, 7, 19))
    r = runner_for(folder, "float32", backend, cache_tokens=8 * 16, max_live=2)       # far fewer than the requests' tokens
    got = U.replay(r, steps)
    r.cache.manager.check()
    assert min(r.cache.manager.reuse_count(g) for g in r.cache.paged_groups()) > 0
    for i, s in enumerate(seqs):
        assert_rows(got[f"r{i}"], plain_logits(folder, s), "float32", f"request {i} in a pool of a few windows")


# ----------------------------------------------------------------------------------------------------------------
# the first tokens; slots given out again; a request beside others
# ----------------------------------------------------------------------------------------------------------------
def test_first_tokens_one_by_one(backend, folders):
    """Every token alone from the first: the convolutions' histories are shorter than their taps, the states start at
    zero, the windows are not full."""
    cfg = CONFIGS["R"][0]
    folder = folders("R", "float32")
    seq = seqs_for(cfg, [12], seed=77)[0]
    want = plain_logits(folder, seq)
    r = runner_for(folder, "float32", backend, 64)
    assert_rows(U.replay(r, U.tail_decode_trace([seq], 12))["r0"], want, "float32", "token by token from the first")
    cfg = CONFIGS["Q"][0]
    folder = folders("Q", "float32")
    seq = seqs_for(cfg, [10], seed=78)[0]
    r = runner_for(folder, "float32", backend, 64)
    assert_rows(U.replay(r, U.chunk_trace([seq], sizes=(1, 2, 1, 3, 2, 1)))["r0"], plain_logits(folder, seq), "float32", "the first tokens in portions")


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


# ----------------------------------------------------------------------------------------------------------------
# configuration and weights
# ----------------------------------------------------------------------------------------------------------------
def test_config_is_read_with_errors_that_name_the_key(folders):
    from denno_beta_amd.config import ConfigError, resolve_architecture
    from denno_beta_amd.models.nigilorn import NigilornConfig, build_nigilorn
    assert resolve_architecture({"architecture": "Nigilorn"}).config_cls is NigilornConfig
    for path, match in ((("layers", 1, "mixer", "kv_heads"), "kv_heads"), (("layers", 0, "mixer", "dt_rank"), "dt_rank"),
                        (("norm",), "norm"), (("layers", 2, "mixer", "rot_dim"), "rot_dim"), (("layers", 1, "mixer", "scale"), "scale"),
                        (("layers", 1, "mlp", "router"), "router"), (("layers", 2, "mixer", "rot"), "rot"),
                        (("layers", 1, "mixer", "rot", "scaling", "fast"), "fast"), (("layers", 3, "mixer", "state"), "state")):
        bad = copy.deepcopy(CFG_P)
        d = bad
        for key in path[:-1]:
            d = d[key]
        del d[path[-1]]
        with pytest.raises(ConfigError, match=match):
            NigilornConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][0]["type"] = "something"
    with pytest.raises(ConfigError, match="type"):
        NigilornConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][1]["mixer"]["rot"]["dims"] = 18
    with pytest.raises(ConfigError, match="rot.dims"):
        NigilornConfig.from_dict(bad)
    bad = copy.deepcopy(CFG_P)
    bad["layers"][1]["mlp"]["router"]["groups"]["count"] = 4
    with pytest.raises(ConfigError, match="groups"):
        NigilornConfig.from_dict(bad)
    # what config.json may leave out: no groups, no scale, no stretching, no window, no token input
    lean = copy.deepcopy(CFG_Q)
    spec = build_nigilorn(NigilornConfig.from_dict(lean))
    assert spec.tables == {} and spec.layers[0].parts["side"][0] == "none" and spec.layers[1].parts["gate2"][0] == "none"
    assert spec.layers[0].parts["ffn"][1]["groups"] == 1 and spec.layers[2].parts["mixer"][1]["window"] == 0
    spec = build_nigilorn(NigilornConfig.from_dict(CFG_P))
    assert spec.tables == {"side.embed": (97, 4 * 6)} and spec.layers[3].parts["side"][1]["offset"] == 18


def test_a_checkpoint_that_does_not_fit_is_reported_whole(folders, tmp_path):
    from safetensors.torch import load_file, save_file
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.weights import CheckpointError
    import shutil
    d = str(tmp_path / "m")
    shutil.copytree(folders("R", "float32"), d)
    tensors = load_file(os.path.join(d, "model.safetensors"))
    del tensors["l0.mlp.e1.up"]
    tensors["side.embed"] = tensors["side.embed"][:, :2].contiguous()
    tensors["stray"] = torch.zeros(3)
    save_file(tensors, os.path.join(d, "model.safetensors"))
    with pytest.raises(CheckpointError) as e:
        ModelRunner.from_folder(d, EngineOptions(dtype="float32", device="cpu", cache_tokens=64, max_live=1))
    assert "l0.mlp.e1.up" in e.value.missing and "stray" in e.value.unexpected and e.value.wrong_shape[0][0] == "side.embed"


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
    cfg = CONFIGS["P"][0] if dtype == "float32" else all_experts(CONFIGS["P"][0])
    folder = folders("P", dtype, cfg, CONFIGS["P"][1])
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
    """A short prompt, then token after token for long: pages fill, windows pass on, the states run on."""
    cfg = CONFIGS["P"][0]
    folder = folders("P", "float32")
    n = 60 if backend == "cpu" else 230
    seq = seqs_for(cfg, [n], seed=600)[0]
    steps = U.tail_decode_trace([seq], n - 4)
    r = runner_for(folder, "float32", backend, U.max_live_tokens(steps))
    assert_rows(U.replay(r, steps)["r0"], plain_logits(folder, seq), "float32", "long decoding")
