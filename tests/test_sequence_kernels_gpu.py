"""The kernels of csrc/kernels/sequence.hip and grouped.hip, each alone against its plain reference in
tests/kernel_refs.py, at sizes that are multiples of nothing, in both precisions of what they read and write."""
import pytest
import torch

import kernel_refs as ref
from denno_beta_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = [torch.float32, torch.bfloat16]


def close(got, want, dtype=torch.float32, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    bound = tol * (1.0 + want.abs())
    assert bool(((got - want).abs() <= bound).all()), f"{what}: worst {(got - want).abs().max().item():.3g}"


def tables(lengths, slots):
    starts = [0]
    for n in lengths:
        starts.append(starts[-1] + n)
    return (torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV), starts[-1])


def both(fn_name, make, outs, dtype=torch.float32):
    """Runs ops.<fn> on the device and kernel_refs.<fn> on copies on the host; compares the tensors named in `outs`."""
    args = make()
    cpu = lambda a: a.detach().cpu().clone() if isinstance(a, torch.Tensor) else a      # noqa: E731
    host = [tuple(cpu(x) for x in a) if isinstance(a, tuple) else cpu(a) for a in args]
    getattr(ops, fn_name)(*args)
    getattr(ref, fn_name)(*host)
    torch.cuda.synchronize()
    for i in outs:
        close(args[i], host[i], dtype, f"{fn_name} argument {i}")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("width", [7, 96, 1000])
def test_rmsnorm(dtype, width):
    x = torch.randn(13, width + 5, device=DEV) * 3
    w = torch.randn(width, device=DEV)
    rows = torch.tensor([12, 0, 5], dtype=torch.int32, device=DEV)
    both("rmsnorm", lambda: (x, w, 1e-5, torch.empty(13, width, dtype=dtype, device=DEV)), [3], dtype)
    both("rmsnorm", lambda: (x, None, 1e-3, torch.empty(3, width, dtype=dtype, device=DEV), rows), [3], dtype)
    # in place, 32-bit
    y = x[:, :width].contiguous()
    want = ref.rmsnorm(y.cpu(), w.cpu(), 1e-5, torch.empty(13, width))
    ops.rmsnorm(y, w, 1e-5, y)
    close(y, want)


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
@pytest.mark.parametrize("dtype", DT)
def test_conv_rows_and_history(taps, dtype):
    width = 37
    row_start, slots, T = tables([1, 7, 2, 3], [2, 0, -1, 3])
    h = torch.randn(T, width, device=DEV)
    w = torch.randn(width, taps, device=DEV)
    hist = torch.randn(5, max(taps - 1, 1) * width, device=DEV)[:, :(taps - 1) * width]
    both("conv_rows", lambda: (h, w, hist, row_start, slots, torch.zeros(T, width, dtype=dtype, device=DEV)), [5], dtype)
    if taps > 1:
        both("history_update", lambda: (h.to(dtype), hist.clone(), row_start, slots), [1])


@pytest.mark.parametrize("dtype", DT)
def test_shift_mix(dtype):
    width = 50
    row_start, slots, T = tables([4, 1, 1, 9], [1, 3, 0, -1])
    h = torch.randn(T, width, device=DEV).to(dtype)
    state = torch.randn(4, 100 + width, device=DEV)
    mu = torch.rand(5, width, device=DEV)
    both("shift_mix", lambda: (h, state[:, 100:], mu, row_start, slots, torch.zeros(5, T, width, dtype=dtype, device=DEV)), [5], dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("dims,width", [(8, 8), (6, 10), (0, 4), (64, 64)])
def test_rotary(dtype, dims, width):
    T, n_vec = 9, 3
    src = torch.randn(T, 5 + n_vec * (width + 2), device=DEV)
    pos = torch.tensor([0, 1, 2, 500, 17, 4095, 33, 100000, 7], dtype=torch.int32, device=DEV)
    freq = (10000.0 ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / max(dims, 1))).float().to(DEV)
    both("rotary", lambda: (src, torch.zeros(T, 3 + n_vec * (width + 7), dtype=dtype, device=DEV), pos, freq, n_vec, dims, width,
                             5, width + 2, 3, width + 7), [1], dtype)


@pytest.mark.parametrize("kind", sorted(ops.ACTIVATIONS))
def test_activate_and_gated(kind):
    x = torch.randn(6, 45, device=DEV) * 2
    bias, lower = torch.randn(45, device=DEV), torch.rand(45, device=DEV)
    if kind == "xielu":      # (two numbers for all columns)
        lower = (lower[:2] + 0.3).contiguous()
    both("activate", lambda: (x, kind, torch.empty(6, 45, device=DEV), bias, lower), [2])
    # the columns of wider rows, in place
    wide = torch.randn(6, 60, device=DEV)
    want = ref.activate(wide[:, 5:50].cpu(), kind, torch.empty(6, 45), bias.cpu(), lower.cpu())
    ops.activate(wide[:, 5:50], kind, wide[:, 5:50], bias, lower)
    close(wide[:, 5:50], want)
    if kind in ("silu", "sigmoid", "tanh"):
        g = torch.randn(6, 45, device=DEV)
        both("gated", lambda: (x.bfloat16(), g, kind, torch.empty(6, 45, dtype=torch.bfloat16, device=DEV)), [3], torch.bfloat16)


# (sizes that are multiples of 4 take the fetches of 16 bytes a lane, the others the fetches of single numbers)
@pytest.mark.parametrize("dk,dv,heads", [(16, 16, 2), (48, 32, 3), (5, 70, 1), (64, 64, 4), (100, 9, 2), (130, 20, 1), (32, 12, 2),
                                         (128, 36, 1), (252, 8, 1), (64, 128, 2)])
@pytest.mark.parametrize("mode", ["bonus", "gate"])
@pytest.mark.parametrize("lengths", [[1, 12, 40], [1, 2, 1]])      # portions; a step of single rows (another kernel variant)
def test_state_scan(dk, dv, heads, mode, lengths):
    row_start, slots, T = tables(lengths, [2, -1, 0])
    r, k = torch.randn(T, heads * dk, device=DEV), torch.randn(T, heads * dk, device=DEV)
    v = torch.randn(T, heads * dv, device=DEV)
    w = torch.rand(T, heads * dk, device=DEV) * 0.5 + 0.5
    u = torch.randn(heads * dk, device=DEV)
    state = torch.randn(3, heads * dk * dv + 11, device=DEV)

    def make():
        st = state.clone()
        out = torch.zeros(T, heads * dv, device=DEV)
        if mode == "bonus":
            return (r, k, v, w, u, st[:, :heads * dk * dv], row_start, slots, heads, dk, dv, out, False, False)
        return (r, None, v, w, None, st[:, :heads * dk * dv], row_start, slots, heads, dk, dv, out, True, True)
    both("state_scan", make, [5, 11])


@pytest.mark.parametrize("dk,dv,heads,qk_heads", [(16, 16, 2, 2), (48, 32, 4, 2), (5, 70, 1, 1), (64, 64, 4, 1), (100, 9, 2, 2), (130, 20, 3, 1),
                                                  (32, 12, 6, 3), (128, 36, 1, 1), (252, 8, 1, 1), (64, 128, 2, 2), (6, 10, 2, 1)])
@pytest.mark.parametrize("lengths", [[1, 12, 40], [1, 2, 1]])
def test_state_scan_delta_rule(dk, dv, heads, qk_heads, lengths):
    """S <- diag(w) S; e = beta (v - S^T k); S <- S + k e^T; o = S^T r, with fewer heads of r and k than of v."""
    row_start, slots, T = tables(lengths, [2, -1, 0])
    wide = torch.randn(T, 4 + 2 * qk_heads * dk, device=DEV)                  # r and k: columns of wider rows
    r, k = wide[:, :qk_heads * dk], wide[:, qk_heads * dk:2 * qk_heads * dk]
    k = torch.nn.functional.normalize(k.reshape(T, qk_heads, dk), dim=-1).reshape(T, -1).contiguous()
    v = torch.randn(T, heads * dv, device=DEV)
    w = torch.rand(T, heads * dk, device=DEV) * 0.5 + 0.5
    beta = torch.rand(T, heads, device=DEV)
    state = torch.randn(3, heads * dk * dv + 11, device=DEV)

    def make():
        st = state.clone()
        return (r, k, v, w, None, st[:, :heads * dk * dv], row_start, slots, heads, dk, dv, torch.zeros(T, heads * dv, device=DEV), False,
                False, beta, None, qk_heads)
    both("state_scan", make, [5, 11])


@pytest.mark.parametrize("dk,dv,heads", [(16, 8, 2), (40, 24, 1), (64, 64, 3), (7, 5, 2)])
@pytest.mark.parametrize("lengths", [[3, 1, 50], [1, 1, 1]])
def test_state_scan_with_one_decay_a_head(dk, dv, heads, lengths):
    row_start, slots, T = tables(lengths, [1, 0, -1])
    r, k, v = (torch.randn(T, heads * n, device=DEV) for n in (dk, dk, dv))
    decay = torch.rand(heads, device=DEV) * 0.6 + 0.4
    state = torch.randn(2, heads * dk * dv, device=DEV)
    both("state_scan", lambda: (r, k, v, None, None, state.clone(), row_start, slots, heads, dk, dv, torch.zeros(T, heads * dv, device=DEV),
                                True, False, None, decay), [5, 11])


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_without_the_row_itself_then_silu(taps):
    """The channels are the first columns of wider rows; the history is kept from the same columns."""
    width = 41
    row_start, slots, T = tables([1, 7, 2, 3], [2, 0, -1, 3])
    h = torch.randn(T, width + 9, device=DEV)
    w = torch.randn(width, taps, device=DEV)
    hist = torch.randn(5, max(taps - 1, 1) * width + 6, device=DEV)[:, 6:6 + (taps - 1) * width]
    both("conv_rows", lambda: (h[:, :width], w, hist, row_start, slots, torch.zeros(T, width, device=DEV), False, "silu"), [5])
    both("conv_rows", lambda: (h[:, :width], w, hist, row_start, slots, torch.zeros(T, width, device=DEV), False, None), [5])
    if taps > 1:
        mine, theirs = hist.clone(), hist.cpu().clone()
        ops.history_update(h[:, :width], mine, row_start, slots)
        ref.history_update(h[:, :width].cpu(), theirs, row_start.cpu(), slots.cpu())
        close(mine, theirs)


@pytest.mark.parametrize("taps", [1, 3, 4])
@pytest.mark.parametrize("n_unit,unit_dim,n_rest,rest_dim", [(4, 8, 3, 12), (2, 70, 1, 300), (6, 5, 0, 1), (0, 1, 2, 9)])
def test_conv_of_heads_with_unit_vectors(taps, n_unit, unit_dim, n_rest, rest_dim):
    width = n_unit * unit_dim + n_rest * rest_dim
    row_start, slots, T = tables([1, 7, 2, 3], [2, 0, -1, 3])
    h = torch.randn(T, width + 5, device=DEV)
    w = torch.randn(width, taps, device=DEV)
    hist = torch.randn(5, max(taps - 1, 1) * width + 2, device=DEV)[:, 2:2 + (taps - 1) * width]
    both("conv_heads", lambda: (h[:, :width], w, hist, row_start, slots, torch.zeros(T, width, device=DEV), n_unit, unit_dim, n_unit // 2,
                                unit_dim ** -0.5, 1.0, 1e-6, n_rest, rest_dim), [5])


@pytest.mark.parametrize("dtype", DT)
def test_three_runs_turned_in_one_launch(dtype):
    T, H, G, dk, dv, hw, dims = 9, 4, 2, 12, 20, 32, 8
    z = torch.randn(T, H * dk + G * dk + G * dv, device=DEV)
    positions = torch.randint(0, 500, (T,), dtype=torch.int32, device=DEV)
    freq = torch.rand(dims // 2, device=DEV)

    def make():
        q, kv = torch.zeros(T, H * hw, dtype=dtype, device=DEV), torch.zeros(T, 2 * G * hw, dtype=dtype, device=DEV)
        return (z, positions, freq, [(q, 0, H, dk, dims, 0, hw), (kv, H * dk, G, dk, dims, 0, hw), (kv, H * dk + G * dk, G, dv, 0, G * hw, hw)])
    args = make()
    host = [z.cpu(), positions.cpu(), freq.cpu(), [(torch.zeros_like(r[0]).cpu(),) + r[1:] for r in args[3]]]
    host[3][2] = (host[3][1][0],) + host[3][2][1:]          # (keys and values share their rows)
    ops.rotary_runs(*args)
    ref.rotary_runs(*host)
    close(args[3][0][0], host[3][0][0], dtype, "queries")
    close(args[3][1][0], host[3][1][0], dtype, "keys and values")


def test_delta_rule_with_beta_as_sigmoid_argument():
    row_start, slots, T = tables([5, 1], [1, 0])
    H, dk, dv = 2, 16, 8
    r, k, v, w = (torch.randn(T, H * n, device=DEV) for n in (dk, dk, dv, dk))
    w = torch.sigmoid(w)
    z = torch.randn(T, H + 3, device=DEV)
    state = torch.randn(2, H * dk * dv, device=DEV)
    a = ops.state_scan(r, k, v, w, None, state.clone(), row_start, slots, H, dk, dv, torch.zeros(T, H * dv, device=DEV), beta=z[:, 1:1 + H],
                       beta_logits=True)
    b = ops.state_scan(r, k, v, w, None, state.clone(), row_start, slots, H, dk, dv, torch.zeros(T, H * dv, device=DEV),
                       beta=torch.sigmoid(z[:, 1:1 + H]).contiguous())
    close(a, b)


def test_sum_of_results_weighted_by_sigmoid_of_a_column():
    T, width = 7, 40
    out, x = torch.randn(T, width, device=DEV), torch.randn(T, width, device=DEV)
    z = torch.randn(T, 6, device=DEV)
    hx = x.cpu().clone()
    ops.moe_combine(out, z[:, 5:6], x, logits=True)
    ref.moe_combine(out.cpu(), z[:, 5:6].cpu(), hx, logits=True)
    close(x, hx)


@pytest.mark.parametrize("width", [7, 96, 1000])
@pytest.mark.parametrize("dtype", DT)
def test_norm_added_into_the_stream(width, dtype):
    y = (torch.randn(11, width, device=DEV) * 3).to(dtype)
    w, scale = torch.randn(width, device=DEV), torch.randn(width, device=DEV)
    x = torch.randn(11, width + 3, device=DEV)
    both("rmsnorm_add", lambda: (y, w, scale, 0.37, 1e-5, x[:, :width].clone()), [5])
    both("rmsnorm_add", lambda: (y, None, None, 1.0, 1e-3, x[:, :width].clone()), [5])


@pytest.mark.parametrize("T,width", [(5, 32), (3, 7), (40, 100)])
def test_average_over_depth(T, width):
    planes = 6
    hist = torch.randn(planes, T, width, device=DEV)
    weights = torch.randn(planes, device=DEV)
    for n in (1, 2, 5):
        mine, theirs = hist.clone(), hist.cpu().clone()
        ops.depth_mix(mine, n, weights, mine[n])              # (into the next plane)
        ref.depth_mix(theirs, n, weights.cpu(), theirs[n])
        close(mine, theirs)
    both("depth_mix", lambda: (hist, planes, weights, torch.empty(T, width, device=DEV)), [3])


def test_unit_vectors_per_head():
    T, H, dim = 9, 3, 20
    x = torch.randn(T, H * dim + 5, device=DEV)
    both("unit_heads", lambda: (x[:, :H * dim], H, dim, 1e-6, dim ** -0.5, torch.zeros(T, H * dim, device=DEV)), [5])
    tiny = x * 1e-4                                              # (the eps counts where the vector is short)
    both("unit_heads", lambda: (tiny[:, :H * dim], H, dim, 1e-6, 1.0, torch.zeros(T, H * dim, device=DEV)), [5])
    mine = x.clone()
    ops.unit_heads(mine[:, :H * dim], H, dim, 1e-6, 1.0, mine[:, :H * dim])
    close(mine[:, :H * dim], ref.unit_heads(x[:, :H * dim].cpu(), H, dim, 1e-6, 1.0, torch.zeros(T, H * dim)))
    close(mine[:, H * dim:], x[:, H * dim:])


@pytest.mark.parametrize("T,E,top", [(1, 4, 2), (50, 16, 3), (33, 70, 1), (9, 5, 5)])
def test_route_by_sigmoid_scores_as_they_are(T, E, top):
    z = torch.randn(T, E + 2, device=DEV) * 2                   # (further columns behind the experts')
    ids, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
    ops.moe_route(z, None, top, ids, wts, score="sigmoid", renorm=False, n_experts=E)
    hi, hw = torch.zeros(T, top, dtype=torch.int32), torch.zeros(T, top)
    ref.moe_route(z.cpu(), None, top, hi, hw, score="sigmoid", renorm=False, n_experts=E)
    assert torch.equal(ids.cpu(), hi)
    close(wts, hw)
    close(wts, torch.sigmoid(z[:, :E]).cpu().gather(1, hi.long()))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,E,top,ff,width", [(1, 3, 2, 8, 24), (45, 6, 3, 70, 50), (200, 5, 2, 64, 128), (9, 8, 2, 96, 64), (3, 40, 1, 32, 160)])
def test_experts_that_read_weighted_rows(dtype, T, E, top, ff, width):
    """silu(W_gate s h) * (W_up s h) with a factor s per (token, choice); weights None in the sum of a token's results."""
    h = torch.randn(T, width, device=DEV).to(dtype)
    wg, wu = ((torch.randn(E, ff, width, device=DEV) / width ** 0.5).to(dtype) for _ in range(2))
    ids = torch.stack([torch.randperm(E, device=DEV)[:top] for _ in range(T)]).int()
    offsets, order = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
    ops.moe_plan(ids, E, offsets, order)
    s = torch.rand(T, top, device=DEV) + 0.2
    for scale in (s, None):
        y = torch.zeros(T * top, ff, dtype=dtype, device=DEV)
        ops.moe_up(h, order, offsets, top, wg, wu, 0.0, 1.0, y, kind="silu", in_scale=scale)
        hy = torch.zeros(T * top, ff, dtype=dtype)
        ref.moe_up(h.cpu(), order.cpu(), offsets.cpu(), top, wg.cpu(), wu.cpu(), 0.0, 1.0, hy, kind="silu",
                   in_scale=None if scale is None else scale.cpu())
        close(y, hy, dtype, "moe_up")
        if dtype == torch.bfloat16 and ops.experts_packable(E, ff, width):
            y2 = torch.zeros_like(y)
            ops.moe_up(h, order, offsets, top, ops.pack_matrix(wg.view(E * ff, width)), ops.pack_matrix(wu.view(E * ff, width)), 0.0, 1.0,
                       y2, dims=(E, ff, width), kind="silu", in_scale=scale)
            close(y2, hy, dtype, "moe_up, packed")
    out = torch.randn(T * top, width, device=DEV)
    x = torch.randn(T, width, device=DEV)
    hx = x.cpu().clone()
    ops.moe_combine(out, None, x)
    ref.moe_combine(out.cpu(), None, hx)
    close(x, hx)


@pytest.mark.parametrize("dtype", DT)
def test_head_norm(dtype):
    T, H, dv = 7, 3, 20
    o, gate = torch.randn(T, H * dv, device=DEV), torch.randn(T, H * dv, device=DEV)
    both("head_norm", lambda: (o, torch.randn(H * dv, device=DEV), 1e-5, torch.empty(T, H * dv, dtype=dtype, device=DEV), H, gate, "silu"), [3], dtype)
    both("head_norm", lambda: (o, torch.randn(dv, device=DEV), 1e-5, torch.empty(T, H * dv, dtype=dtype, device=DEV), H), [3], dtype)
    both("head_norm", lambda: (o, None, 1e-2, torch.empty(T, H * dv, dtype=dtype, device=DEV), H), [3], dtype)
    # all heads as one vector, and heads of many columns (a workgroup a head)
    both("head_norm", lambda: (o, torch.randn(H * dv, device=DEV), 1e-5, torch.empty(T, H * dv, dtype=dtype, device=DEV), 1, gate, "sigmoid"), [3], dtype)
    wide, wgate = torch.randn(T, 2 * 700, device=DEV), torch.randn(T, 2 * 700, device=DEV)
    both("head_norm", lambda: (wide, torch.randn(700, device=DEV), 1e-5, torch.empty(T, 1400, dtype=dtype, device=DEV), 2, wgate, "sigmoid"), [3], dtype)
    both("head_norm", lambda: (wide, torch.randn(1400, device=DEV), 1e-5, torch.empty(T, 1400, dtype=dtype, device=DEV), 1, wgate, "silu"), [3], dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,H,N,K", [(1, 2, 24, 16), (19, 3, 70, 33), (130, 1, 5, 100)])
def test_heads_linear(dtype, T, H, N, K):
    a = torch.randn(T, 4 + H * (K + 3), device=DEV).to(dtype)
    w = (torch.randn(H, N, K, device=DEV) / K ** 0.5).to(dtype)
    both("heads_linear", lambda: (a, w, torch.zeros(T, 2 + H * (N + 1), dtype=dtype, device=DEV), 4, K + 3, 2, N + 1), [2], dtype)


@pytest.mark.parametrize("T,E,top", [(1, 4, 2), (50, 16, 3), (700, 5, 5), (33, 70, 1), (20, 200, 64), (7, 130, 70), (5, 64, 64)])
def test_route_and_plan(T, E, top):
    z = torch.randn(T, E, device=DEV) * 2
    corr = torch.randn(E, device=DEV) * 0.1
    ids, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
    ops.moe_route(z, corr, top, ids, wts)
    hi, hw = torch.zeros(T, top, dtype=torch.int32), torch.zeros(T, top)
    ref.moe_route(z.cpu(), corr.cpu(), top, hi, hw)
    assert torch.equal(ids.cpu(), hi)
    close(wts, hw)
    offsets, order = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
    ops.moe_plan(ids, E, offsets, order)
    ho, hr = torch.zeros(E + 1, dtype=torch.int32), torch.zeros(T * top, dtype=torch.int32)
    ref.moe_plan(hi, E, ho, hr)
    assert torch.equal(offsets.cpu(), ho) and torch.equal(order.cpu(), hr)


@pytest.mark.parametrize("dtype", DT)
# (bfloat16 with a width and an inner size that are multiples of 32 takes the matrix-core kernels; tiles of 64 places with
# one row, with a last block that is not full, experts that nobody chose)
@pytest.mark.parametrize("T,E,top,ff,width", [(1, 3, 2, 8, 24), (45, 6, 3, 70, 50), (300, 4, 1, 33, 96), (200, 5, 2, 64, 128),
                                              (9, 8, 2, 96, 64), (77, 3, 3, 40, 32), (3, 40, 2, 32, 160), (150, 4, 2, 160, 192), (70, 2, 2, 16, 32)])
def test_experts(dtype, T, E, top, ff, width):
    h = torch.randn(T, width, device=DEV).to(dtype)
    wg, wu = ((torch.randn(E, ff, width, device=DEV) / width ** 0.5).to(dtype) for _ in range(2))
    wd = (torch.randn(E, width, ff, device=DEV) / ff ** 0.5).to(dtype)
    ids = torch.stack([torch.randperm(E, device=DEV)[:top] for _ in range(T)]).int()
    offsets, order = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
    ops.moe_plan(ids, E, offsets, order)
    y = torch.zeros(T * top, ff, dtype=dtype, device=DEV)
    ops.moe_up(h, order, offsets, top, wg, wu, 1.5, 1.702, y)
    hy = torch.zeros(T * top, ff, dtype=dtype)
    ref.moe_up(h.cpu(), order.cpu(), offsets.cpu(), top, wg.cpu(), wu.cpu(), 1.5, 1.702, hy)
    close(y, hy, dtype, "moe_up")
    out = torch.zeros(T * top, width, device=DEV)
    ops.moe_down(y, order, offsets, wd, out)
    ho = torch.zeros(T * top, width)
    ref.moe_down(y.cpu(), order.cpu(), offsets.cpu(), wd.cpu(), ho)
    close(out, ho, dtype, "moe_down")
    if dtype == torch.bfloat16 and ops.experts_packable(E, ff, width) and ops.experts_packable(E, width, ff):
        # the experts' matrices stacked and packed for the matrix cores: the same numbers
        pg, pu = ops.pack_matrix(wg.view(E * ff, width)), ops.pack_matrix(wu.view(E * ff, width))
        y2 = torch.zeros_like(y)
        ops.moe_up(h, order, offsets, top, pg, pu, 1.5, 1.702, y2, dims=(E, ff, width))
        close(y2, hy, dtype, "moe_up, packed")
        out2 = torch.zeros_like(out)
        ops.moe_down(y, order, offsets, ops.pack_matrix(wd.view(E * width, ff)), out2, dims=(E, width, ff))
        close(out2, ho, dtype, "moe_down, packed")
    wts = torch.rand(T, top, device=DEV)
    x = torch.randn(T, width, device=DEV)
    hx = x.cpu().clone()
    ops.moe_combine(out, wts, x)
    ref.moe_combine(out.cpu(), wts.cpu(), hx)
    close(x, hx)


@pytest.mark.parametrize("T,H,N,K", [(1, 2, 24, 32), (130, 3, 70, 64), (65, 1, 33, 96)])
def test_heads_linear_on_the_matrix_cores(T, H, N, K):
    """bfloat16 rows at offsets that are multiples of 8 numbers: the kernel of 16 x 16 x 32 blocks."""
    a = torch.randn(T, 8 + H * (K + 8), device=DEV).bfloat16()
    w = (torch.randn(H, N, K, device=DEV) / K ** 0.5).bfloat16()
    for dtype in DT:
        both("heads_linear", lambda: (a, w, torch.zeros(T, 2 + H * (N + 1), dtype=dtype, device=DEV), 8, K + 8, 2, N + 1), [2], dtype)
    # 32-bit rows into a bfloat16 result: rounded on their way into the matrix instruction
    both("heads_linear", lambda: (a.float(), w, torch.zeros(T, 2 + H * (N + 1), dtype=torch.bfloat16, device=DEV), 8, K + 8, 2, N + 1),
         [2], torch.bfloat16)
    one = ops.heads_linear(a[T // 2:T // 2 + 1].contiguous(), w, torch.zeros(1, 2 + H * (N + 1), device=DEV), 8, K + 8, 2, N + 1)
    many = ops.heads_linear(a, w, torch.zeros(T, 2 + H * (N + 1), device=DEV), 8, K + 8, 2, N + 1)
    assert torch.equal(many[T // 2:T // 2 + 1], one), "a row's sums depend on the rows beside it"


def test_a_row_does_not_depend_on_its_neighbours():
    """The same row alone and among others: the same bits from every kernel that works on tiles of rows."""
    H, N, K = 2, 40, 24
    a = torch.randn(50, H * K, device=DEV)
    w = torch.randn(H, N, K, device=DEV)
    many = ops.heads_linear(a, w, torch.zeros(50, H * N, device=DEV))
    one = ops.heads_linear(a[17:18].contiguous(), w, torch.zeros(1, H * N, device=DEV))
    assert torch.equal(many[17:18], one)


# ---- a convolution's bias, a decay per row and head, a gate before the norm, a recurrence of single numbers, a stream in copies ----
@pytest.mark.parametrize("taps", [1, 3, 4])
def test_conv_with_a_bias(taps):
    width = 29
    row_start, slots, T = tables([2, 9, 1, 4], [1, 3, -1, 0])
    h = torch.randn(T, width + 6, device=DEV)
    w = torch.randn(width, taps, device=DEV)
    b = torch.randn(width, device=DEV)
    hist = torch.randn(4, max(taps - 1, 1) * width, device=DEV)
    both("conv_rows", lambda: (h, w, hist, row_start, slots, torch.zeros(T, width, device=DEV), False, "silu", b), [5])


@pytest.mark.parametrize("dk,dv,heads,groups", [(16, 8, 4, 2), (48, 48, 6, 1), (24, 12, 3, 3), (128, 64, 2, 1), (6, 10, 2, 1),
                                                (128, 32, 64, 2), (64, 16, 128, 1), (100, 20, 64, 4)])
@pytest.mark.parametrize("lengths", [[1, 1, 1], [5, 40, 1, 17]])
def test_state_scan_with_a_decay_per_row_and_head(dk, dv, heads, groups, lengths):
    row_start, slots, T = tables(lengths, list(range(len(lengths)))[::-1])
    g = torch.Generator(device=DEV).manual_seed(dk * 7 + dv)
    rnd = lambda *s: torch.randn(*s, device=DEV, generator=g)      # noqa: E731
    r, k, v = rnd(T, groups * dk), rnd(T, groups * dk), rnd(T, heads * dv)
    w = torch.sigmoid(rnd(T, heads) + 2.0)
    state0 = rnd(len(lengths), heads * dk * dv) * 0.3

    def make():
        return (r, k, v, w, None, state0.clone(), row_start, slots, heads, dk, dv, torch.zeros(T, heads * dv, device=DEV), True, False, None,
                None, groups, False, True)
    both("state_scan", make, [5, 11])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("heads,dv", [(2, 24), (1, 300), (4, 16), (1, 3000), (1, 5000), (2, 2048)])
def test_head_norm_with_the_gate_first_and_a_second_summand(dtype, heads, dv):
    T, n = 9, heads * dv
    o, gate, skip = torch.randn(T, n, device=DEV), torch.randn(T, n, device=DEV), torch.randn(T, n, device=DEV)
    w = torch.randn(n, device=DEV)
    for parts in (1, 2, n // 4):
        scale = torch.randn(parts, device=DEV)
        both("head_norm", lambda: (o, w, 1e-5, torch.empty(T, n, dtype=dtype, device=DEV), heads, gate, "silu", True, skip, scale), [3], dtype)
    both("head_norm", lambda: (o, w, 1e-5, torch.empty(T, n, dtype=dtype, device=DEV), heads, gate, "sigmoid", False, skip, scale), [3], dtype)
    both("head_norm", lambda: (o, None, 1e-5, torch.empty(T, n, dtype=dtype, device=DEV), heads, gate, "silu", True), [3], dtype)


def test_step_sizes():
    T, H, dv = 11, 3, 10
    z = torch.randn(T, H + 4, device=DEV) * 4
    x = torch.randn(T, H * dv + 2, device=DEV)
    bias, rate = torch.randn(H, device=DEV), torch.rand(H, device=DEV) * 3
    both("step_sizes", lambda: (z[:, 2:2 + H], bias, rate, x[:, :H * dv], H, torch.empty(T, H, device=DEV), torch.empty(T, H * dv, device=DEV)),
         [5, 6])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("lengths", [[1, 1, 1, 1], [3, 70, 1, 9, 8]])
@pytest.mark.parametrize("width", [5, 64, 200])
def test_gate_scan(dtype, lengths, width):
    row_start, slots, T = tables(lengths, [3, 0, -1, 2, 1][:len(lengths)])
    z = torch.randn(T, 3 * width + 1, device=DEV) * 2
    ba, bb = torch.randn(width, device=DEV), torch.randn(width, device=DEV)
    state0 = torch.randn(4, width, device=DEV)

    def make():
        return (z[:, :width], z[:, width:2 * width], z[:, 2 * width:3 * width], ba, bb, state0.clone(), row_start, slots,
                torch.zeros(T, width, dtype=dtype, device=DEV))
    both("gate_scan", make, [5, 8], dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,width", [(1, 40), (3, 256), (4, 77), (8, 1030), (2, 2000), (4, 3000), (2, 5000), (5, 300)])
def test_a_stream_in_copies_read_and_written(dtype, n, width):
    T = 7
    xs = torch.randn(n, T, width, device=DEV)
    w_in, w_out, mix = torch.randn(n, device=DEV), torch.randn(n, device=DEV), torch.randn(n, n, device=DEV)
    g = torch.randn(width, device=DEV)
    y = torch.randn(T, width, device=DEV)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    both("streams_read", lambda: (xs, w_in, g, 1e-5, torch.empty(T, width, dtype=dtype, device=DEV)), [4], dtype)
    both("streams_read", lambda: (xs, None, g, 1e-5, torch.empty(3, width, dtype=dtype, device=DEV), rows), [4], dtype)
    both("streams_read", lambda: (xs, None, None, None, torch.empty(T, width, device=DEV)), [4])
    both("streams_write", lambda: (xs.clone(), y, mix, w_out), [0])
    both("streams_write", lambda: (xs.clone(), y, mix, w_out, w_in, g, 1e-6, torch.empty(T, width, dtype=dtype, device=DEV)), [0, 7], dtype)
    # the write that also reads gives what the two kernels give one after the other, bit for bit
    a, b = xs.clone(), xs.clone()
    one = ops.streams_write(a, y, mix, w_out, w_in, g, 1e-6, torch.empty(T, width, dtype=dtype, device=DEV))
    ops.streams_write(b, y, mix, w_out)
    two = ops.streams_read(b, w_in, g, 1e-6, torch.empty(T, width, dtype=dtype, device=DEV))
    assert torch.equal(a, b) and torch.equal(one, two)


def test_rows_picked_by_pairs_of_tokens():
    row_start, slots, T = tables([1, 6, 2, 3], [2, 0, -1, 1])
    tokens = torch.randint(0, 50000, (T,), dtype=torch.int32, device=DEV)
    positions = torch.tensor([0, 0, 1, 2, 3, 4, 5, 0, 0, 7, 8, 9], dtype=torch.int32, device=DEV)
    last0 = torch.randint(0, 50000, (3, 1), dtype=torch.int32, device=DEV)
    for write in (True, False):
        last_d, last_h = last0.clone(), last0.cpu().clone()
        got = ops.pair_rows(tokens, positions, row_start, slots, last_d, 1000003, 999983, 30011, torch.empty(T, dtype=torch.int32, device=DEV), write)
        want = ref.pair_rows(tokens.cpu(), positions.cpu(), row_start.cpu(), slots.cpu(), last_h, 1000003, 999983, 30011,
                             torch.empty(T, dtype=torch.int32), write)
        assert torch.equal(got.cpu()[:7], want[:7]) and torch.equal(got.cpu()[9:], want[9:]) and torch.equal(last_d.cpu(), last_h)
        assert got.cpu()[7:9].tolist() == [30011, 30011]      # (padding at position 0: the table's last row, no state touched)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,width", [(2, 96), (3, 1030)])
def test_a_write_that_norms_two_branches(dtype, n, width):
    T = 6
    xs = torch.randn(n, T, width, device=DEV)
    w_in, w_out, mix = torch.randn(n, device=DEV), torch.randn(n, device=DEV), torch.randn(n, n, device=DEV)
    g, w1, w2 = torch.randn(width, device=DEV), torch.randn(width, device=DEV), torch.randn(width, device=DEV)
    y1, y2 = torch.randn(T, width, device=DEV) * 3, torch.randn(T, width, device=DEV) * 0.2
    both("streams_write", lambda: (xs.clone(), y1, mix, w_out, None, None, 0.0, None, (y2, w1, w2, 1e-5)), [0])
    both("streams_write", lambda: (xs.clone(), y1, mix, w_out, w_in, g, 1e-6, torch.empty(T, width, dtype=dtype, device=DEV),
                                   (y2, w1, w2, 1e-5)), [0, 7], dtype)
    # the same bits as the norms as kernels of their own, added one after the other into zeros
    a, b = xs.clone(), xs.clone()
    ops.streams_write(a, y1, mix, w_out, branches=(y2, w1, w2, 1e-5))
    y = torch.zeros(T, width, device=DEV)
    ops.rmsnorm_add(y1, w1, None, 0.5, 1e-5, y), ops.rmsnorm_add(y2, w2, None, 0.5, 1e-5, y)
    ops.streams_write(b, y, mix, w_out)
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("H,Hkv,dh,ps", [(4, 2, 16, 16), (3, 1, 24, 8), (8, 8, 96, 16), (2, 2, 10, 4)])
def test_queries_and_keys_normed_whole_and_written_to_the_cache(dtype, H, Hkv, dh, ps):
    T, n_pages = 9, 5
    z = torch.randn(T, (H + Hkv) * dh, device=DEV) * 2
    wq, wk = torch.randn(H * dh, device=DEV), torch.randn(Hkv * dh, device=DEV)
    places = torch.randperm(n_pages * ps)[:T].to(torch.int32)
    places[3] = -1
    slot_map = places.to(DEV)

    def make():
        return (z, H * dh, wq, wk, 1e-5, torch.empty(T, H * dh, dtype=dtype, device=DEV), slot_map,
                torch.zeros(n_pages, Hkv, ps, dh, dtype=dtype, device=DEV), torch.zeros(n_pages, Hkv, dh, ps, dtype=dtype, device=DEV))
    both("norm_pair_write", make, [5, 7, 8], dtype)
    args = make() + (False,)
    ops.norm_pair_write(*args)
    assert float(args[7].float().abs().sum()) == 0.0 and float(args[8].float().abs().sum()) == 0.0


# ---- a state per channel and state index, gates on results, rows of a table, routing in groups, experts without a gate ----
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("inner,N,lengths", [(16, 16, [5]), (37, 1, [1, 9, 1]), (50, 5, [3, 1, 40]), (24, 24, [1, 1, 1, 1]), (19, 40, [33, 2]),
                                             (8, 100, [7, 12]), (5, 256, [6]), (130, 8, [70]), (22, 16, [300, 1, 77]), (9, 30, [150, 64]), (2100, 16, [1] * 20), (1100, 20, [1, 2, 1] * 11),
                                             (7, 50, [129]), (6, 70, [200])])
@pytest.mark.parametrize("in_order", [False, True])
def test_selective_scan(dtype, inner, N, lengths, in_order):
    """Portions, single rows and padding; long portions of few requests go the way of rows shared out among waves unless
    `in_order` (up to 64 states a channel), so both ways are held against the reference."""
    n_slots = max(5, len(lengths))
    slot_of = [3, -1, 0, 2, 1] if len(lengths) <= 5 else [(-1 if i % 7 == 1 else i) for i in range(len(lengths))]
    row_start, slots, T = tables(lengths, slot_of[:len(lengths)] if len(lengths) > 1 else [1])
    wide = torch.randn(T, 2 * inner + 3, device=DEV)                       # x and z as columns of wider rows
    low = torch.randn(T, 4 + 2 * N, device=DEV)
    dt = torch.randn(T, inner, device=DEV) * 2 - 1
    A = -torch.exp(torch.rand(inner, N, device=DEV) * 4 - 3)
    D, bias = torch.randn(inner, device=DEV), torch.randn(inner, device=DEV)

    def make(z, d, b):
        state = torch.randn(n_slots, inner * N + 7, device=DEV)[:, :inner * N]
        return (wide[:, :inner], dt, b, low[:, 4:4 + N], low[:, 4 + N:], A, d, z, state, row_start, slots,
                torch.zeros(T, inner, dtype=dtype, device=DEV))
    keep = torch.random.get_rng_state(), torch.cuda.get_rng_state()
    for z, d, b in ((wide[:, inner + 3:], D, bias), (None, None, None)):
        torch.random.set_rng_state(keep[0]), torch.cuda.set_rng_state(keep[1])
        args = make(z, d, b)
        host = [a.detach().cpu().clone() if isinstance(a, torch.Tensor) else a for a in args]
        ops.selective_scan(*args, in_order=in_order)
        ref.selective_scan(*host)
        live = [i for i, s in enumerate(slots.tolist()) if s >= 0]
        rows = torch.cat([torch.arange(row_start[i], row_start[i + 1]) for i in live])
        close(args[11][rows], host[11][rows], dtype, "selective_scan rows")
        close(args[8], host[8], torch.float32, "selective_scan state")
        assert float(args[11][[r for r in range(T) if r not in rows.tolist()]].abs().sum()) == 0.0      # (padding is left alone)


def test_selective_scan_cut_anywhere_gives_the_same_bits():
    inner, N, T = 21, 12, 147
    x, dt, z = (torch.randn(T, inner, device=DEV) for _ in range(3))
    B, C = torch.randn(T, N, device=DEV), torch.randn(T, N, device=DEV)
    A = -torch.exp(torch.rand(inner, N, device=DEV) * 3 - 2)
    D = torch.randn(inner, device=DEV)
    one = torch.tensor([0], dtype=torch.int32, device=DEV)

    def run(cuts):
        state, out = torch.zeros(1, inner * N, device=DEV), torch.zeros(T, inner, device=DEV)
        for a, b in zip(cuts[:-1], cuts[1:]):
            rs = torch.tensor([0, b - a], dtype=torch.int32, device=DEV)
            ops.selective_scan(x[a:b], dt[a:b], None, B[a:b], C[a:b], A, D, z[a:b], state, rs, one, out[a:b], in_order=True)
        return out, state
    whole = run([0, T])
    for cuts in ([0, 1, 2, 3, T], [0, 5, 7, 40, 41, T], list(range(T + 1))):
        got = run(cuts)
        assert torch.equal(got[0], whole[0]) and torch.equal(got[1], whole[1]), cuts
    # the rows shared out among waves: the same to rounding
    state, out = torch.zeros(1, inner * N, device=DEV), torch.zeros(T, inner, device=DEV)
    ops.selective_scan(x, dt, None, B, C, A, D, z, state, torch.tensor([0, T], dtype=torch.int32, device=DEV), one, out)
    close(out, whole[0]), close(state, whole[1])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("width", [9, 64, 700])
def test_norm_of_a_gated_result_added_into_the_stream(width, dtype):
    T = 11
    y = (torch.randn(T, width, device=DEV) * 2).to(dtype)
    gate = torch.randn(T, width + 3, device=DEV)[:, :width] * 2
    w = torch.randn(width, device=DEV)
    x = torch.randn(T, width, device=DEV)
    hx = x.cpu().clone()
    ops.rmsnorm_add(y, w, None, 1.0, 1e-5, x, gate=gate)
    ref.rmsnorm_add(y.cpu(), w.cpu(), None, 1.0, 1e-5, hx, gate=gate.cpu())
    close(x, hx)
    # with the norm that reads the stream next in the same launch: the same bits as that norm's own kernel behind it
    w2 = torch.randn(width, device=DEV)
    for nw in (w2, None):
        x1, x2 = x.clone(), x.clone()
        out = torch.zeros(T, width + 2, dtype=dtype, device=DEV)[:, :width]
        ops.rmsnorm_add(y, w, None, 0.5, 1e-5, x1, gate=gate, then=(nw, 1e-6, out))
        ops.rmsnorm_add(y, w, None, 0.5, 1e-5, x2, gate=gate)
        assert torch.equal(x1, x2)
        assert torch.equal(out, ops.rmsnorm(x2, nw, 1e-6, torch.zeros(T, width, dtype=dtype, device=DEV)))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("H,G,dk,dv,dims,hw", [(4, 2, 16, 8, 8, 16), (3, 1, 24, 40, 24, 48), (2, 2, 10, 6, 4, 16), (5, 5, 256, 32, 64, 256),
                                               (1, 1, 3, 2, 2, 16)])
def test_runs_turned_and_normed_in_one_launch(dtype, H, G, dk, dv, dims, hw):
    T = 9
    z = torch.randn(T, H * dk + G * dk + G * dv + 2, device=DEV) * 2
    pos = torch.randint(0, 5000, (T,), dtype=torch.int32, device=DEV)
    freq = (10000.0 ** (-torch.arange(dims // 2, dtype=torch.float64) * 2 / dims)).float().to(DEV)
    for mag, unit in ((1.0, [True, True, False]), (1.07, [True, False, False]), (0.9, None)):
        q, kv = torch.zeros(T, H * hw, dtype=dtype, device=DEV), torch.zeros(T, 2 * G * hw, dtype=dtype, device=DEV)
        hq, hkv = q.cpu().clone(), kv.cpu().clone()
        runs = lambda a, b: [(a, 0, H, dk, dims, 0, hw), (b, H * dk, G, dk, dims, 0, hw), (b, H * dk + G * dk, G, dv, 0, G * hw, hw)]  # noqa: E731
        ops.rotary_runs(z, pos, freq, runs(q, kv), mag=mag, unit=unit, eps=1e-5)
        ref.rotary_runs(z.cpu(), pos.cpu(), freq.cpu(), runs(hq, hkv), mag=mag, unit=unit, eps=1e-5)
        close(q, hq, dtype, "queries"), close(kv, hkv, dtype, "keys and values")
    if dk <= 64:
        # a normed vector has a root mean square of one whatever its position
        qf = torch.zeros(T, H * hw, device=DEV)
        ops.rotary_runs(z, pos, freq, [(qf, 0, H, dk, dims, 0, hw)], mag=1.3, unit=[True], eps=0.0)
        rms = qf.view(T, H, hw)[:, :, :dk].pow(2).mean(-1).sqrt()
        assert float((rms - 1).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", DT)
def test_a_gate_per_head_and_rows_times_a_table(dtype):
    T, H, dv, hs = 7, 3, 10, 16
    o = torch.randn(T, H * hs, device=DEV).to(dtype)
    g = torch.randn(T, H + 5, device=DEV)[:, 2:2 + H]
    both("head_gate", lambda: (o, g, H, dv, torch.zeros(T, H * dv, dtype=dtype, device=DEV), hs), [4], dtype)
    both("head_gate", lambda: (o[:, :H * dv], g, H, dv, torch.zeros(T, H * dv, dtype=dtype, device=DEV)), [4], dtype)
    table = torch.randn(23, 40, device=DEV).to(dtype)
    a = torch.randn(T, 12, device=DEV).to(dtype)
    ids = torch.randint(0, 23, (T,), dtype=torch.int32, device=DEV)
    both("rows_times_table", lambda: (a, table, ids, 17, torch.zeros(T, 12, dtype=dtype, device=DEV)), [4], dtype)
    want = a.float() * table.float()[ids.long(), 28:40]
    got = ops.rows_times_table(a, table, ids, 28, torch.zeros(T, 12, dtype=dtype, device=DEV))
    close(got, want, dtype)


@pytest.mark.parametrize("T,E,top,groups,keep", [(40, 8, 3, 2, 1), (17, 12, 2, 3, 2), (9, 6, 1, 6, 2), (33, 64, 4, 8, 3), (5, 192, 6, 4, 1),
                                                 (12, 10, 10, 5, 5), (7, 9, 2, 1, 1)])
def test_route_inside_the_best_groups(T, E, top, groups, keep):
    z = torch.randn(T, E, device=DEV) * 2
    corr = torch.randn(E, device=DEV) * 0.1
    for score, renorm, scale, c in (("sigmoid", True, 2.5, None), ("softmax", False, 1.0, corr), ("sigmoid", True, 1.0, corr)):
        ids, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
        ops.moe_route(z, c, top, ids, wts, score=score, renorm=renorm, groups=groups, keep=keep, scale=scale)
        hi, hw = torch.zeros(T, top, dtype=torch.int32), torch.zeros(T, top)
        ref.moe_route(z.cpu(), None if c is None else c.cpu(), top, hi, hw, score=score, renorm=renorm, groups=groups, keep=keep, scale=scale)
        assert torch.equal(ids.cpu(), hi), (score, ids.cpu()[:3], hi[:3])
        close(wts, hw)
        # every choice lies in one of at most `keep` groups
        assert int((ids.cpu() // (E // groups)).sort(dim=1).values.diff(dim=1).ne(0).sum(dim=1).max()) + 1 <= keep if top > 1 else True
        if renorm:
            close(wts.sum(dim=1), torch.full((T,), scale))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,E,top,ff,width", [(1, 3, 2, 8, 24), (45, 6, 3, 70, 50), (200, 5, 2, 64, 128), (9, 8, 2, 96, 64), (3, 40, 1, 32, 160)])
def test_experts_without_a_gate(dtype, T, E, top, ff, width):
    """max(W_up h, 0)^2 through the plain kernel, the matrix-core kernel and the one for packed weights."""
    h = torch.randn(T, width, device=DEV).to(dtype)
    wu = (torch.randn(E, ff, width, device=DEV) / width ** 0.5).to(dtype)
    ids = torch.stack([torch.randperm(E, device=DEV)[:top] for _ in range(T)]).int()
    offsets, order = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
    ops.moe_plan(ids, E, offsets, order)
    y = torch.zeros(T * top, ff, dtype=dtype, device=DEV)
    ops.moe_up(h, order, offsets, top, None, wu, 0.0, 1.0, y, kind="relu2")
    hy = torch.zeros(T * top, ff, dtype=dtype)
    ref.moe_up(h.cpu(), order.cpu(), offsets.cpu(), top, None, wu.cpu(), 0.0, 1.0, hy, kind="relu2")
    close(y, hy, dtype, "moe_up")
    if dtype == torch.bfloat16 and ops.experts_packable(E, ff, width):
        y2 = torch.zeros_like(y)
        ops.moe_up(h, order, offsets, top, None, ops.pack_matrix(wu.view(E * ff, width)), 0.0, 1.0, y2, dims=(E, ff, width), kind="relu2")
        close(y2, hy, dtype, "moe_up, packed")
    z = torch.randn(T, ff, device=DEV)
    close(ops.activate(z, "relu2", torch.zeros(T, ff, dtype=dtype, device=DEV)), torch.relu(z) ** 2, dtype)


@pytest.mark.parametrize("wdt", DT)
@pytest.mark.parametrize("T,width,dim", [(1, 24, 1), (8, 100, 5), (64, 1024, 64), (3, 36, 16), (5, 2048, 250), (2, 4096, 256), (7, 40, 8)])
def test_a_token_input_in_one_launch(wdt, T, width, dim):
    x = torch.randn(T, width + 3, device=DEV)[:, :width] * 2
    wg = (torch.randn(dim, width, device=DEV) / width ** 0.5).to(wdt)
    wp = (torch.randn(width, dim, device=DEV) / dim ** 0.5).to(wdt)
    table = torch.randn(31, 3 * dim + 2, device=DEV).to(wdt)
    ids = torch.randint(0, 31, (T,), dtype=torch.int32, device=DEV)
    w = torch.randn(width, device=DEV)
    for weight, off in ((w, 0), (None, 2 * dim + 2)):
        mine, host = x.clone(), x.cpu().clone()
        ops.token_input(mine, wg, wp, table, ids, off, weight, 1e-5)
        ref.token_input(host, wg.cpu(), wp.cpu(), table.cpu(), ids.cpu(), off, None if weight is None else weight.cpu(), 1e-5)
        close(mine, host, torch.float32, "token_input")
        again, nxt = x.clone(), torch.zeros(T, width, dtype=wdt, device=DEV)
        ops.token_input(again, wg, wp, table, ids, off, weight, 1e-5, then=(weight, 1e-6, nxt))
        assert torch.equal(again, mine)
        close(nxt, ref.rmsnorm(mine.cpu(), None if weight is None else weight.cpu(), 1e-6, torch.zeros(T, width)), wdt, "token_input, the next norm")


def test_selective_scan_reads_rounded_channels():
    inner, N = 20, 16
    row_start, slots, T = tables([90, 3], [1, 0])
    x = torch.randn(T, inner, device=DEV).to(torch.bfloat16)
    dt, z = torch.randn(T, inner, device=DEV), torch.randn(T, inner, device=DEV)
    B, C = torch.randn(T, N, device=DEV), torch.randn(T, N, device=DEV)
    A = -torch.exp(torch.rand(inner, N, device=DEV) * 3 - 2)
    for in_order in (True, False):
        both("selective_scan", lambda: (x, dt, None, B, C, A, None, z, torch.zeros(2, inner * N, device=DEV), row_start, slots,
                                        torch.zeros(T, inner, device=DEV), in_order), [8, 11])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("M,N,K", [(3, 40, 24), (70, 96, 64), (300, 128, 160)])
def test_a_product_that_ends_in_a_squared_relu(dtype, M, N, K):
    a = torch.randn(M, K, device=DEV).to(dtype)
    w = (torch.randn(N, K, device=DEV) / K ** 0.5).to(dtype)
    want = ref.linear(a.cpu(), w.cpu(), None, torch.zeros(M, N, dtype=dtype), epilogue="relu2")
    close(ops.linear(a, w, None, torch.zeros(M, N, dtype=dtype, device=DEV), epilogue="relu2"), want, dtype, "rows")
    if dtype == torch.bfloat16:
        close(ops.linear(a, ops.pack_matrix(w), None, torch.zeros(M, N, dtype=dtype, device=DEV), epilogue="relu2"), want, dtype, "packed")
