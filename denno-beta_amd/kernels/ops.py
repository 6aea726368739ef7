"""The kernels' Python face: one function per entry point of the HIP libraries.

Every function checks on the host what its kernel and launch assume (device, dtype,
shape, strides), then passes raw pointers and the current HIP stream.  There is no other
implementation behind these names: without a GPU or without the built library they raise.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from ..build import load_library

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}
EPILOGUES = {"none": 0, "gelu_tanh": 1, "gelu_erf": 2, "relu2": 3}

_libs = {}


class KernelError(RuntimeError):
    pass


_fail_after = None      # fail_after_launches
launches = 0            # kernel launches asked for through this module since import


def fail_after_launches(n):
    """Failure injection: the next n launches go through, the one after them raises KernelError on
    the host before anything is launched (so every kernel that did start ends normally); then
    launches go through again.  None: off.  The reference's tests wrap the model in one that fails
    after it has written the cache (crates/denno-engine/src/engine.rs:3354-3385)."""
    global _fail_after
    _fail_after = None if n is None else launches + int(n)


_timed = None           # time_launches: [(what, start event, end event)]
_started = None


def time_launches(on=True):
    """Per-kernel timers behind one switch: while on, every launch made through this module stands between
    two HIP events (steps must then run kernel by kernel, not from captured graphs).  `launch_times()`
    gives what they measured.  The reference has its profiler behind DENNO_PROF in the same way
    (crates/denno-engine/src/prof.rs)."""
    global _timed, _started
    _timed, _started = ([] if on else None), None


def launch_times():
    """-> {what: (launches, milliseconds in all)} of the launches since time_launches(True); waits for
    the device."""
    torch.cuda.synchronize()
    out = {}
    for what, a, b in _timed or []:
        n, ms = out.get(what, (0, 0.0))
        out[what] = (n + 1, ms + a.elapsed_time(b))
    return out


def _lib(name):
    global launches, _fail_after, _started
    if _fail_after is not None and launches >= _fail_after:
        _fail_after = None
        raise KernelError(f"injected failure: launch number {launches + 1} was refused")
    launches += 1
    if _timed is not None:
        _started = torch.cuda.Event(enable_timing=True)
        _started.record()
    lib = _libs.get(name)
    if lib is None:
        if not torch.cuda.is_available():
            raise KernelError("the HIP kernels need a GPU (torch.cuda.is_available() is False); "
                              "there is no CPU path")
        lib = load_library(name)
        _declare(name, lib)
        _libs[name] = lib
    return lib


def _lib_quiet(name):
    """The library for a call that launches nothing (not counted, not timed)."""
    lib = _libs.get(name)
    if lib is None:
        global launches
        lib = _lib(name)
        launches -= 1
    return lib


def _declare(name, lib):
    P, I, F = c_void_p, c_int, c_float
    sigs = {
        "elementwise": {
            "dn_embed": [P, P, P, P, P, I, I, I, I, I, F, P],
            "dn_embed_sum": [P, P, P, P, I, P, I, I, I, P],
            "dn_logits_post": [P, I, I, I, F, F, P],
            "dn_layernorm": [P, P, P, P, P, I, I, F, I, I, P],
            "dn_layernorm_join": [P, P, I, c_longlong, P, P, P, P, I, I, F, I, I, P],
            "dn_kv_write": [P, I, I, I, P, P, P, I, I, I, I, I, P],
            "dn_cast": [P, P, c_longlong, I, I, P],
            "dn_pair_rows": [P, P, P, P, I, P, c_longlong, c_longlong, c_longlong, I, I, P, I, P],
        },
        "gemm": {
            "dn_gemm": [P, I, P, P, P, I, P, I, I, I, I, I, I, I, I, P, c_longlong, P],
            "dn_gemm_plain_qkv_takes": [P, I, P, I, I, I, I],
            "dn_gemm_plain_qkv": [P, I, P, P, P, I, I, I, I, I, P, P, P, I, I, I, I, P, c_longlong, P],
            "dn_pack_matrix": [P, P, I, I, P],
            "dn_gemm_norm_out": [P, I, P, P, P, I, I, I, I, P, P, I, P, P],
            "dn_gemm_norm_in": [P, I, P, P, P, F, P, P, I, I, I, I, I, P, P, P, I, I, I, I, I, I, P],
            "dn_gemm_qkv": [P, I, P, P, P, I, I, I, I, P, P, P, I, I, I, I, I, I, P],
            "dn_gemm_deferred_shares": [I, I, I],
            "dn_gemm_deferred": [P, I, P, I, I, I, I, P, c_longlong, P],
            "dn_join": [P, I, P, P, I, I, I, P],
        },
        "attention": {
            "dn_attention": [P, I, P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, F, I, I, P],
            "dn_attention_rows": [P, I, P, I, P, P, P, I, P, P, I, P, I, I, I, I, I, F, I, I, P],
            "dn_attention_rows_tile": [I],
            "dn_attention_extras": [P, I, P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, F, I, I, P, I, I, I, P],
            "dn_attention_rows_extras": [P, I, P, I, P, P, P, I, P, P, I, P, I, I, I, I, I, F, I, I, P, I, I, I, P],
            "dn_attention_flash_extras": [P, I, P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, F, I, I, P, I, I, P],
            "dn_attention_decode_extras": [P, I, P, I, P, P, P, I, P, P, P, I, P, I, I, I, I, I, I, I, F, I, I, P, I, I, P],
            "dn_attention_flash": [P, I, P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, F, I, P],
            "dn_attention_decode": [P, I, P, I, P, P, P, I, P, P, P, I, P, I, I, I, I, I, I, I, F, I, P],
        },
        "sequence": {
            "dn_rmsnorm": [P, I, c_longlong, P, P, I, c_longlong, P, I, I, F, P],
            "dn_concat_cast": [P, c_longlong, I, P, c_longlong, I, P, I, I, P],
            "dn_rmsnorm_add": [P, I, c_longlong, P, P, F, P, c_longlong, I, I, F, P, c_longlong, P, F, P, I, c_longlong, P],
            "dn_depth_mix": [P, c_longlong, I, P, P, c_longlong, P],
            "dn_unit_heads": [P, c_longlong, P, c_longlong, I, I, I, F, F, P],
            "dn_conv_rows": [P, c_longlong, P, P, P, P, P, I, I, I, I, I, I, P, I, c_longlong, c_longlong, P],
            "dn_history_update": [P, I, c_longlong, P, P, P, I, I, I, c_longlong, P],
            "dn_conv_heads": [P, c_longlong, P, P, P, P, I, I, I, I, I, I, F, F, F, I, I, P, c_longlong, c_longlong, P],
            "dn_rotary_runs": [P, I, c_longlong, P, I, P, P, I, F, c_longlong, F, P],
            "dn_shift_mix": [P, I, P, P, I, P, P, I, I, I, P, I, c_longlong, P],
            "dn_rotary": [P, I, c_longlong, I, I, P, I, c_longlong, I, I, P, P, I, I, I, I, F, P],
            "dn_activate": [P, c_longlong, P, P, I, P, I, c_longlong, I, I, P],
            "dn_gated": [P, I, c_longlong, P, c_longlong, I, P, I, c_longlong, I, I, P],
            "dn_state_scan": [P, c_longlong, P, c_longlong, P, c_longlong, P, c_longlong, P, P, c_longlong, P, I, P, c_longlong, P, P,
                              I, I, I, I, I, I, I, I, I, P, c_longlong, P],
            "dn_head_norm": [P, c_longlong, P, I, F, P, c_longlong, I, I, P, c_longlong, P, I, P, I, c_longlong, I, I, I, P],
            "dn_step_sizes": [P, c_longlong, P, P, P, c_longlong, I, I, I, P, c_longlong, P, c_longlong, P],
            "dn_gate_scan": [P, c_longlong, P, c_longlong, P, c_longlong, P, P, P, c_longlong, P, P, I, I, I, P, I, c_longlong, P],
            "dn_streams_read": [P, c_longlong, I, P, P, F, P, I, c_longlong, P, I, I, P],
            "dn_streams_write": [P, c_longlong, I, P, P, P, c_longlong, P, c_longlong, P, P, F, P, P, F, P, I, c_longlong, I, I, P],
            "dn_norm_pair_write": [P, c_longlong, I, I, P, P, F, P, c_longlong, P, P, P, I, I, I, I, I, I, P],
            "dn_head_gate": [P, I, c_longlong, I, P, c_longlong, P, I, c_longlong, I, I, I, P],
            "dn_token_input": [P, c_longlong, P, P, I, P, I, c_longlong, I, P, I, P, I, I, I, F, P, F, P, I, c_longlong, P],
            "dn_rows_times_table": [P, I, c_longlong, P, I, c_longlong, I, P, I, P, I, c_longlong, I, I, P],
            "dn_selective_scan": [P, I, c_longlong, P, c_longlong, P, P, c_longlong, P, c_longlong, P, P, P, c_longlong, P, c_longlong,
                                  P, P, I, I, I, I, P, I, c_longlong, I, P],
        },
        "grouped": {
            "dn_heads_linear": [P, I, c_longlong, I, I, P, I, P, I, c_longlong, I, I, I, I, I, I, P],
            "dn_moe_route": [P, c_longlong, P, I, I, I, I, I, P, P, I, I, F, P],
            "dn_moe_plan": [P, I, I, P, P, P],
            "dn_moe_up": [P, I, c_longlong, P, P, I, I, I, P, P, I, I, I, F, F, I, P, P, I, I, P],
            "dn_moe_down": [P, I, P, P, I, I, P, I, I, I, P, I, P],
            "dn_moe_combine": [P, P, c_longlong, I, I, I, I, P, c_longlong, P],
        },
        "sampling": {
            "dn_sample": [P, I, I, I, P, P, P, P],
            "dn_penalties": [P, I, I, I, P, P, P, P, P, P, P, P],
            "dn_history_append": [P, P, P, P, P, I, P],
            "dn_sample_top": [P, I, I, I, P, P, P, P, P, P, P, P, P],
            "dn_sample_full": [P, I, I, I, I, P, P, P, P, P, P, P, P],
        },
    }[name]
    for fn, args in sigs.items():
        f = getattr(lib, fn)
        f.argtypes = args
        f.restype = c_int
    if name == "gemm":
        lib.dn_gemm_work_floats.argtypes = [I, I, I, I]
        lib.dn_gemm_work_floats.restype = c_longlong


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream's handle, asked for before every launch: through torch's own short way where it has
    one (building a Stream object costs several microseconds, as much as the launch itself)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ok(rc, what):
    global _started
    if _timed is not None and _started is not None:
        end = torch.cuda.Event(enable_timing=True)
        end.record()
        _timed.append((what, _started, end))
        _started = None
    if rc != 0:
        if rc == -1:
            raise KernelError(f"{what}: unsupported dtype combination")
        if rc == -2:
            raise KernelError(f"{what}: the kernel does not take these sizes")
        raise KernelError(f"{what}: HIP error {rc} at launch")


def _need(cond, msg):
    """msg: the text, or what makes it (a message that has to be put together is made only when it is needed:
    these checks stand in front of every launch)."""
    if not cond:
        raise KernelError(msg() if callable(msg) else msg)


def _dev(t, name, dtypes=None, dims=None):
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise KernelError(f"{name}: must be a tensor on the GPU")
    if dtypes is not None and t.dtype not in dtypes:
        raise KernelError(f"{name}: dtype {t.dtype}, wanted one of {dtypes}")
    if dims is not None and t.dim() != dims:
        raise KernelError(f"{name}: {t.dim()} dimensions, wanted {dims}")
    return t


def _rows(t, name):
    """A 2-D tensor whose rows are contiguous; returns its leading dimension."""
    _need(t.dim() == 2 and (t.shape[1] == 1 or t.stride(1) == 1), lambda: f"{name}: rows must be contiguous")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    _need(ld >= t.shape[1], lambda: f"{name}: rows overlap")
    return ld


def _ptr(t):
    return 0 if t is None else t.data_ptr()


_FLOATS = (torch.float32, torch.bfloat16)
_I32 = (torch.int32,)


def embed(tokens, positions, wte, wpe, out, token_scale=1.0):
    """out[t,:] = wte[tokens[t],:] * token_scale + wpe[positions[t],:]; wpe may be None.  out is 32-bit."""
    T = tokens.shape[0]
    _dev(tokens, "tokens", _I32, 1), _dev(positions, "positions", _I32, 1)
    _dev(wte, "wte", _FLOATS, 2), _dev(out, "out", (torch.float32,), 2)
    _need(tokens.is_contiguous() and positions.is_contiguous() and positions.shape[0] == T, "tokens/positions")
    E = wte.shape[1]
    _need(wte.is_contiguous() and out.is_contiguous() and tuple(out.shape) == (T, E), "embed: shapes")
    n_pos = 0
    if wpe is not None:
        _dev(wpe, "wpe", (wte.dtype,), 2)
        _need(wpe.is_contiguous() and wpe.shape[1] == E, "embed: wpe shape")
        n_pos = wpe.shape[0]
    _ok(_lib("elementwise").dn_embed(tokens.data_ptr(), positions.data_ptr(), wte.data_ptr(), _ptr(wpe),
                                     out.data_ptr(), T, E, wte.shape[0], n_pos, _CODE[wte.dtype], float(token_scale),
                                     _stream()), "embed")
    return out


EMBED_TABLES_MAX = 4


def embed_sum(parts, out):
    """out[t,:] = sum over parts, in their order, of table[index[t],:] * scale.  parts: up to four
    (table [rows, E], index int32 [T], scale); all tables of one dtype; out is 32-bit [T, E]."""
    _need(1 <= len(parts) <= EMBED_TABLES_MAX, lambda: f"embed_sum: 1 to {EMBED_TABLES_MAX} tables, not {len(parts)}")
    _dev(out, "out", (torch.float32,), 2)
    T, E = out.shape
    _need(out.is_contiguous(), "embed_sum: out")
    dtype = parts[0][0].dtype
    n = len(parts)
    tables, indices = (c_void_p * n)(), (c_void_p * n)()
    rows, scales = (c_int * n)(), (c_float * n)()
    for i, (table, index, scale) in enumerate(parts):
        _dev(table, "table", (dtype,), 2), _dev(index, "index", _I32, 1)
        _need(dtype in _FLOATS, "embed_sum: table dtype")
        _need(table.is_contiguous() and table.shape[1] == E, lambda: f"embed_sum: table {i} is {tuple(table.shape)}, rows are {E} wide")
        _need(index.is_contiguous() and index.shape[0] == T, lambda: f"embed_sum: index {i}")
        tables[i], indices[i], rows[i], scales[i] = table.data_ptr(), index.data_ptr(), table.shape[0], float(scale)
    _ok(_lib("elementwise").dn_embed_sum(tables, indices, rows, scales, n, out.data_ptr(), T, E, _CODE[dtype], _stream()),
        "embed")
    return out


def pair_rows(tokens, positions, row_start, slots, last, mul_prev, mul_cur, buckets, out, write=True):
    """out[t] = (token before * mul_prev + tokens[t] * mul_cur) mod buckets, in 64-bit: the row of a table that the pair (token
    before, token) picks; a request's first token (positions[t] == 0) takes row `buckets`.  The token before a request's
    first row of this step is last[slot] (int32 [slots, 1]); with `write` the request's last token of this step is left there."""
    _dev(tokens, "tokens", _I32, 1), _dev(positions, "positions", _I32, 1), _dev(out, "out", _I32, 1), _dev(last, "last", _I32, 2)
    T = tokens.shape[0]
    S = _request_tables(row_start, slots, "pair_rows")
    _need(tokens.is_contiguous() and positions.is_contiguous() and out.is_contiguous() and positions.shape[0] == T and out.shape[0] == T
          and last.shape[1] == 1 and buckets >= 1 and mul_prev >= 0 and mul_cur >= 0, "pair_rows: shapes")
    _ok(_lib("elementwise").dn_pair_rows(tokens.data_ptr(), positions.data_ptr(), row_start.data_ptr(), slots.data_ptr(), S,
                                         last.data_ptr(), last.stride(0), int(mul_prev), int(mul_cur), int(buckets), int(bool(write)),
                                         out.data_ptr(), T, _stream()), "pair_rows")
    return out


def logits_post(logits, scale=1.0, softcap=0.0):
    """In place on 32-bit logits [R, V]: times `scale`, then, if softcap > 0, softcap * tanh(l / softcap)."""
    _dev(logits, "logits", (torch.float32,), 2)
    R, V = logits.shape
    _ok(_lib("elementwise").dn_logits_post(logits.data_ptr(), _rows(logits, "logits"), R, V, float(scale),
                                           float(softcap), _stream()), "logits_post")
    return logits


class PackedMatrix:
    """A bfloat16 matrix [N, K] laid out for the matrix cores: blocks of 16 rows x 32 columns, 1 KB
    each and contiguous, block (n // 16, k // 32) at ((n // 16) * ceil(K / 32) + k // 32) * 512
    elements; inside it row n % 16, columns (k % 32) // 8 * 8 .. + 7 at (((k % 32) // 8) * 16 + n % 16) * 8.
    `linear` takes it for the MFMA kernels.  Every bfloat16 weight is held so (rows and columns
    beyond N and K are zeros), and so are the bfloat16 rows that one kernel hands to the next
    while a step has at most 256 of them (`packed_rows`; K a multiple of 32, rows beyond N are
    not written and never read into a result)."""
    __slots__ = ("data", "shape")
    dtype = torch.bfloat16

    def __init__(self, data, shape):
        self.data, self.shape = data, tuple(shape)

    @property
    def device(self):
        return self.data.device

    def data_ptr(self):
        return self.data.data_ptr()

    def numel(self):
        return self.shape[0] * self.shape[1]

    def element_size(self):
        return 2

    def rows(self):
        """The matrix [N, K] again (for tests and tools)."""
        N, K = self.shape
        nb, ks = -(-N // 16), -(-K // 32)
        return self.data.view(nb, ks, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nb * 16, ks * 32)[:N, :K].contiguous()


PACKED_ROWS_MAX = 256    # the few-rows product's limit
PACKED_ROWS_MIN = 17     # up to 16 rows the few-rows product turns ordinary rows round itself, as fast or faster


def packed_rows(n_rows, width, device) -> PackedMatrix:
    """An empty packed matrix for n_rows <= 256 rows of activations."""
    _need(n_rows <= PACKED_ROWS_MAX and width % 32 == 0,
          lambda: f"packed rows: at most {PACKED_ROWS_MAX} rows of a width that is a multiple of 32, not {n_rows} x {width}")
    data = torch.empty(-(-n_rows // 16) * (width // 32) * 512, dtype=torch.bfloat16, device=device)
    return PackedMatrix(data, (n_rows, width))


def pack_matrix(w) -> PackedMatrix:
    """w: bfloat16 [N, K], rows contiguous, K a multiple of 8."""
    _dev(w, "w", (torch.bfloat16,), 2)
    N, K = w.shape
    _need(w.is_contiguous(), "pack_matrix: w must be contiguous")
    _need(K % 8 == 0, lambda: f"pack_matrix: the inner size {K} must be a multiple of 8")
    data = torch.empty(-(-N // 16) * -(-K // 32) * 512, dtype=torch.bfloat16, device=w.device)
    _ok(_lib("gemm").dn_pack_matrix(w.data_ptr(), data.data_ptr(), N, K, _stream()), "pack_matrix")
    return PackedMatrix(data, (N, K))


def layernorm(x, gamma, beta, eps, out, rows=None):
    """out[r,:] = LayerNorm(x[rows[r],:]) (rows None: every row).  x, gamma, beta are 32-bit;
    out: a tensor [R, E], or packed rows."""
    packed = isinstance(out, PackedMatrix)
    _dev(x, "x", (torch.float32,), 2), _dev(gamma, "gamma", (torch.float32,), 1)
    if packed:
        _need(out.device == x.device, "layernorm: out on another device")
    else:
        _dev(out, "out", _FLOATS, 2)
    E = x.shape[1]
    _need(x.is_contiguous() and (packed or out.is_contiguous()) and gamma.is_contiguous() and gamma.shape[0] == E,
          "layernorm: shapes")
    if beta is not None:
        _dev(beta, "beta", (torch.float32,), 1)
        _need(beta.is_contiguous() and beta.shape[0] == E, "layernorm: beta")
    R = out.shape[0]
    if rows is not None:
        _dev(rows, "rows", _I32, 1)
        _need(rows.is_contiguous() and rows.shape[0] == R, "layernorm: rows")
    else:
        _need(R == x.shape[0], "layernorm: out rows")
    _need(out.shape[1] == E, "layernorm: out width")
    _ok(_lib("elementwise").dn_layernorm(x.data_ptr(), gamma.data_ptr(), _ptr(beta), out.data_ptr(), _ptr(rows),
                                         R, E, float(eps), _CODE[out.dtype], int(packed), _stream()), "layernorm")
    return out


def layernorm_join(x, part, bias, gamma, beta, eps, out):
    """x += (part[0] + part[1] + ...) + bias (in place: what `linear_deferred` left of a product into the stream),
    then out = LayerNorm(x), all rows, in one kernel.  part: 32-bit [shares, R, E]; out: a tensor [R, E] or packed rows."""
    packed = isinstance(out, PackedMatrix)
    _dev(x, "x", (torch.float32,), 2), _dev(gamma, "gamma", (torch.float32,), 1), _dev(part, "part", (torch.float32,), 3)
    if not packed:
        _dev(out, "out", _FLOATS, 2)
    R, E = x.shape
    _need(x.is_contiguous() and part.is_contiguous() and tuple(part.shape[1:]) == (R, E) and part.shape[0] >= 1,
          lambda: f"layernorm_join: shares of shape {tuple(part.shape)} for rows of shape {tuple(x.shape)}")
    _need((packed or out.is_contiguous()) and tuple(out.shape) == (R, E) and gamma.is_contiguous() and gamma.shape[0] == E
          and E <= 8192, "layernorm_join: shapes")
    for v, name in ((beta, "beta"), (bias, "bias")):
        if v is not None:
            _dev(v, name, (torch.float32,), 1)
            _need(v.is_contiguous() and v.shape[0] == E, lambda: f"layernorm_join: {name}")
    _ok(_lib("elementwise").dn_layernorm_join(x.data_ptr(), part.data_ptr(), part.shape[0], R * E, _ptr(bias), gamma.data_ptr(),
                                              _ptr(beta), out.data_ptr(), R, E, float(eps), _CODE[out.dtype], int(packed),
                                              _stream()), "layernorm (adds a product's shares first)")
    return out


def kv_write(src, k_col, v_col, slot_map, k_pool, v_pool):
    """Rows of src ([T, ld]; keys at columns k_col.., values at v_col..) go to the slots
    slot_map[t] = page * page_size + offset; k_pool is [n_pages, Hkv, page_size, dh], v_pool
    [n_pages, Hkv, dh, page_size]."""
    _dev(src, "src", _FLOATS, 2), _dev(slot_map, "slot_map", _I32, 1)
    _dev(k_pool, "k_pool", (src.dtype,), 4), _dev(v_pool, "v_pool", (src.dtype,), 4)
    ld = _rows(src, "src")
    T = src.shape[0]
    n_pages, Hkv, ps, dh = k_pool.shape
    _need(k_pool.is_contiguous() and v_pool.is_contiguous() and tuple(v_pool.shape) == (n_pages, Hkv, dh, ps),
          "kv_write: pools")
    _need(slot_map.is_contiguous() and slot_map.shape[0] == T, "kv_write: slot_map")
    w = Hkv * dh
    _need(0 <= k_col and k_col + w <= src.shape[1] and 0 <= v_col and v_col + w <= src.shape[1],
          "kv_write: columns outside src")
    _ok(_lib("elementwise").dn_kv_write(src.data_ptr(), ld, k_col, v_col, slot_map.data_ptr(), k_pool.data_ptr(),
                                        v_pool.data_ptr(), T, Hkv, dh, ps, _CODE[src.dtype], _stream()),
        "kv_write")


def cast(x, out):
    _dev(x, "x", _FLOATS), _dev(out, "out", _FLOATS)
    _need(x.is_contiguous() and out.is_contiguous() and x.numel() == out.numel() and x.dtype != out.dtype, "cast")
    _ok(_lib("elementwise").dn_cast(x.data_ptr(), out.data_ptr(), x.numel(), _CODE[x.dtype], _CODE[out.dtype],
                                    _stream()), "cast")
    return out


PACKED_W, PACKED_A, PACKED_C = 1, 2, 4


def _operands(a, w, what):
    """(leading dimension of a, N, packed flags) of the product a [M, K] . w [N, K]^T."""
    M, K = a.shape
    if isinstance(a, PackedMatrix):
        _need(isinstance(w, PackedMatrix), lambda: f"{what}: packed rows need a packed matrix")
        _need(M <= PACKED_ROWS_MAX and K % 32 == 0, lambda: f"{what}: packed rows {a.shape}")
        lda, flags = 0, PACKED_A
    else:
        _dev(a, "a", _FLOATS, 2)
        lda, flags = _rows(a, "a"), 0
    if isinstance(w, PackedMatrix):
        _need(a.dtype == torch.bfloat16, lambda: f"{what}: a packed matrix needs bfloat16 rows, not {a.dtype}")
        _need(w.device == a.device and w.shape[1] == K, lambda: f"{what}: w {w.shape} does not fit a {tuple(a.shape)}")
        _need(a.data_ptr() % 16 == 0 and lda % 8 == 0, lambda: f"{what}: the rows of a must be aligned to 16 bytes")
        return lda, w.shape[0], flags | PACKED_W
    _dev(w, "w", (a.dtype,), 2)
    _need(w.is_contiguous() and w.shape[1] == K, lambda: f"{what}: w {tuple(w.shape)} does not fit a {tuple(a.shape)}")
    return lda, w.shape[0], flags


def linear(a, w, bias=None, out=None, epilogue="none", residual=None):
    """out = epilogue(a @ w.T + bias), or residual += a @ w.T + bias (32-bit, in place).
    a: [M, K] rows contiguous; w: [N, K] held [out, in], in rows (the plain kernel: 32-bit, or a
    reference for bfloat16) or a PackedMatrix (the MFMA kernels); bias: 32-bit [N].  With a packed
    w and at most 256 rows, a and a bfloat16 out may be packed rows."""
    M, K = a.shape
    # (the plain kernels take any inner size; a packed matrix has one that is a multiple of 8: pack_matrix)
    lda, N, packed = _operands(a, w, "linear")
    wp = w.data_ptr()
    if bias is not None:
        _dev(bias, "bias", (torch.float32,), 1)
        _need(bias.is_contiguous() and bias.shape[0] == N, "linear: bias")
    epi = EPILOGUES[epilogue]
    if isinstance(out, PackedMatrix):
        packed |= PACKED_C
    work, work_floats = None, 0
    if M <= 64 if not packed & PACKED_W else (64 < M <= 512 and residual is not None):
        # products that share K out among workgroups leave the shares' sums in a workspace: the plain one
        # of few rows, and the MFMA one of a long K beside few rows and columns that adds into the stream
        work_floats = _lib_quiet("gemm").dn_gemm_work_floats(M, N, K, packed)
        if work_floats:
            work = torch.empty(work_floats, dtype=torch.float32, device=a.device)
    if residual is not None:
        _dev(residual, "residual", (torch.float32,), 2)
        _need(tuple(residual.shape) == (M, N) and epi == 0 and out is None, "linear: residual")
        ldr = _rows(residual, "residual")
        _ok(_lib("gemm").dn_gemm(a.data_ptr(), lda, wp, _ptr(bias), 0, 0, residual.data_ptr(), ldr,
                                 M, N, K, _CODE[a.dtype], F32, 0, packed, _ptr(work), work_floats, _stream()),
            "linear" if _timed is None else f"linear {K} -> {N}, added into the stream")
        return residual
    if isinstance(out, PackedMatrix):
        _need((packed & PACKED_W) and M <= PACKED_ROWS_MAX and N % 32 == 0 and out.device == a.device,
              lambda: f"linear: packed rows as out need a packed w, at most {PACKED_ROWS_MAX} rows and N a multiple of 32")
        ldc = 0
    else:
        _dev(out, "out", _FLOATS, 2)
        ldc = _rows(out, "out")
    _need(tuple(out.shape) == (M, N), "linear: out shape")
    _ok(_lib("gemm").dn_gemm(a.data_ptr(), lda, wp, _ptr(bias), out.data_ptr(), ldc, 0, 0, M, N, K,
                             _CODE[a.dtype], _CODE[out.dtype], epi, packed, _ptr(work), work_floats, _stream()),
        "linear" if _timed is None else f"linear {K} -> {N}" + (f", {epilogue}" if epi else ""))
    return out


def linear_deferred_shares(n_rows, w):
    """How many shares of K `linear_deferred` cuts the product of n_rows rows with w into; 0: it does not take it
    (the product then adds into the stream itself)."""
    if not isinstance(w, PackedMatrix):
        return 0
    return _lib_quiet("gemm").dn_gemm_deferred_shares(n_rows, w.shape[0], w.shape[1])


def linear_deferred(a, w):
    """-> part, 32-bit [shares, M, N]: the shares' parts of a @ w.T, for whoever adds them into the residual stream
    with the bias (`layernorm_join`, the norm that reads the stream next, or `join`).  a: bfloat16 rows or packed
    rows; w: a PackedMatrix."""
    M, K = a.shape
    lda, N, packed = _operands(a, w, "linear_deferred")
    shares = linear_deferred_shares(M, w)
    _need(shares > 0 and (packed & PACKED_W), lambda: f"linear_deferred: {M} rows x {tuple(w.shape)} is not deferred")
    part = torch.empty((shares, M, N), dtype=torch.float32, device=a.device)
    _ok(_lib("gemm").dn_gemm_deferred(a.data_ptr(), lda, w.data_ptr(), M, N, K, packed, part.data_ptr(), part.numel(), _stream()),
        "linear_deferred" if _timed is None else f"linear {K} -> {N}, its shares left for the next norm")
    return part


def join(part, bias, residual):
    """residual += (part[0] + part[1] + ...) + bias, in place: a deferred product's shares, where no norm adds them."""
    _dev(part, "part", (torch.float32,), 3), _dev(residual, "residual", (torch.float32,), 2)
    M, N = residual.shape
    _need(part.is_contiguous() and tuple(part.shape[1:]) == (M, N), "join: shares of another shape than the rows")
    if bias is not None:
        _dev(bias, "bias", (torch.float32,), 1)
        _need(bias.is_contiguous() and bias.shape[0] == N, "join: bias")
    _ok(_lib("gemm").dn_join(part.data_ptr(), part.shape[0], _ptr(bias), residual.data_ptr(), _rows(residual, "residual"), M, N,
                             _stream()), "join")
    return residual


def linear_qkv(a, w, bias, out, slot_map, k_pool, v_pool, q_width):
    """The fused projection q | k | v = a @ w.T + bias: the key columns (q_width ..) and the value
    columns after them go to the slots slot_map[t] of the pools, as kv_write does.  out: [M, N], or
    [M, q_width] for the queries alone (nothing reads keys and values from out).  Returns the
    queries [M, q_width] (a view of out).  One kernel with a PackedMatrix and bfloat16 all through
    (the cache write is in the product's epilogue), else two, and out must then be [M, N]."""
    n_pages, Hkv, ps, dh = k_pool.shape
    kvw = Hkv * dh
    M, K = a.shape
    N = w.shape[0]
    _need(N == q_width + 2 * kvw, "linear_qkv: columns are not q | k | v")
    _need(not isinstance(out, PackedMatrix) and out.dim() == 2 and out.shape[0] == M and out.shape[1] in (N, q_width),
          lambda: f"linear_qkv: out must be [{M}, {N}] or [{M}, {q_width}]")
    if isinstance(w, PackedMatrix) and out.dtype == torch.bfloat16:
        _dev(out, "out", None, 2)
        _dev(slot_map, "slot_map", _I32, 1), _dev(k_pool, "k_pool", (torch.bfloat16,), 4)
        _dev(v_pool, "v_pool", (torch.bfloat16,), 4)
        lda, N, packed = _operands(a, w, "linear_qkv")
        _need(k_pool.is_contiguous() and v_pool.is_contiguous() and tuple(v_pool.shape) == (n_pages, Hkv, dh, ps),
              "linear_qkv: pools")
        _need(slot_map.is_contiguous() and slot_map.shape[0] == M, "linear_qkv: slot_map")
        if bias is not None:
            _dev(bias, "bias", (torch.float32,), 1)
            _need(bias.is_contiguous() and bias.shape[0] == N, "linear_qkv: bias")
        _ok(_lib("gemm").dn_gemm_qkv(a.data_ptr(), lda, w.data_ptr(), _ptr(bias), out.data_ptr(),
                                     _rows(out, "out"), M, N, K, slot_map.data_ptr(), k_pool.data_ptr(),
                                     v_pool.data_ptr(), q_width, Hkv, dh, ps, int(bool(packed & PACKED_A)),
                                     out.shape[1], _stream()),
            "linear_qkv" if _timed is None else f"linear {K} -> {N}, cache write")
        return out[:, :q_width]
    _need(out.shape[1] == N, "linear_qkv: without the fused kernel out must hold all columns")
    if not isinstance(w, PackedMatrix) and not isinstance(a, PackedMatrix) and out.dtype == a.dtype and M <= 64:
        # few rows in the plain kernels: where K is shared out among workgroups, the kernel that adds their sums
        # writes the keys and values to the cache as well
        lda, _, _ = _operands(a, w, "linear_qkv")
        _dev(out, "out", (a.dtype,), 2)
        if _lib_quiet("gemm").dn_gemm_plain_qkv_takes(a.data_ptr(), lda, w.data_ptr(), M, N, K, _CODE[a.dtype]):
            _dev(slot_map, "slot_map", _I32, 1), _dev(k_pool, "k_pool", (a.dtype,), 4), _dev(v_pool, "v_pool", (a.dtype,), 4)
            _need(k_pool.is_contiguous() and v_pool.is_contiguous() and tuple(v_pool.shape) == (n_pages, Hkv, dh, ps),
                  "linear_qkv: pools")
            _need(slot_map.is_contiguous() and slot_map.shape[0] == M, "linear_qkv: slot_map")
            if bias is not None:
                _dev(bias, "bias", (torch.float32,), 1)
                _need(bias.is_contiguous() and bias.shape[0] == N, "linear_qkv: bias")
            work_floats = _lib_quiet("gemm").dn_gemm_work_floats(M, N, K, 0)
            work = torch.empty(work_floats, dtype=torch.float32, device=a.device)
            _ok(_lib("gemm").dn_gemm_plain_qkv(a.data_ptr(), lda, w.data_ptr(), _ptr(bias), out.data_ptr(), _rows(out, "out"),
                                               M, N, K, _CODE[a.dtype], slot_map.data_ptr(), k_pool.data_ptr(),
                                               v_pool.data_ptr(), q_width, Hkv, dh, ps, work.data_ptr(), work_floats,
                                               _stream()),
                "linear_qkv" if _timed is None else f"linear {K} -> {N}, cache write")
            return out[:, :q_width]
    linear(a, w, bias, out=out)
    kv_write(out, q_width, q_width + kvw, slot_map, k_pool, v_pool)
    return out[:, :q_width]


FLASH_HEAD_DIMS = tuple(range(16, 257, 16))
DECODE_HEAD_DIMS = tuple(range(16, 257, 16))
DECODE_SPLIT = 256     # the decode kernel's smallest chunk; captured decode steps round contexts up to it


def decode_attention_applies(dtype, page_size, head_dim, single_rows, max_context):
    """Whether `attention` takes the split kernel of pure decode steps."""
    return (dtype == torch.bfloat16 and page_size % 16 == 0 and bool(single_rows) and head_dim in DECODE_HEAD_DIMS
            and max_context > 0)


def attention_writes_packed(dtype, page_size, head_dim, single_rows, max_context, tiles_wide):
    """Whether `attention` with these arguments takes one of the two bfloat16 kernels, which can write
    packed rows (the plain kernel cannot)."""
    return decode_attention_applies(dtype, page_size, head_dim, single_rows, max_context) or (
        dtype == torch.bfloat16 and page_size % 16 == 0 and tiles_wide is not None and head_dim in FLASH_HEAD_DIMS)


def attention(q, out, k_pool, v_pool, block_tables, tiles, n_heads, scale, window=0, tiles_wide=None,
              single_rows=False, max_context=0, decode_waves=None, chunk=0, bias=None, sink=False):
    """Causal attention of the batch's rows over the paged cache.

    q: [T, >= H*dh] rows contiguous, head h at columns h*dh..; out: [T, H*dh];
    k_pool: [n_pages, Hkv, page_size, dh]; v_pool: [n_pages, Hkv, dh, page_size];
    block_tables: int32 [S, max_blocks];
    tiles: int32 [4, n_tiles] = (request, first row, rows <= 16, first position), request < 0: padding;
    tiles_wide: the same rows cut into tiles of up to 128 rows;
    single_rows: a pure decode step: request s brings row s and is tile s, (s or -1, s, 1, position);
    max_context: the longest context then.

    chunk > 0: the row at position p reads only the keys from p // chunk * chunk on (runs of `chunk` positions counted from
    the request's first); bias: 32-bit [H, span], bias[h, p - key] is added to the scaled score (distances from span on
    take the last entry); sink: one more summand exp(0) under the softmax (a key with score 0 and no value).

    Three kernels: 32-bit takes the plain one; bfloat16 takes the MFMA kernel over tiles_wide, or,
    for a pure decode step, the split kernel (with both, out may be packed rows); a head size that
    those do not take falls to the plain one."""
    out_packed = isinstance(out, PackedMatrix)
    _dev(q, "q", _FLOATS, 2)
    if not out_packed:
        _dev(out, "out", (q.dtype,), 2)
    _dev(k_pool, "k_pool", (q.dtype,), 4), _dev(v_pool, "v_pool", (q.dtype,), 4)
    _dev(block_tables, "block_tables", _I32, 2), _dev(tiles, "tiles", _I32, 2)
    n_pages, Hkv, ps, dh = k_pool.shape
    T = q.shape[0]
    _need(v_pool.shape[2] == dh, lambda: f"attention: values of width {v_pool.shape[2]} beside keys of width {dh}: "
                                         "these kernels take keys and values of one width")
    _need(k_pool.is_contiguous() and v_pool.is_contiguous() and tuple(v_pool.shape) == (n_pages, Hkv, dh, ps),
          "attention: pools")
    _need(q.shape[1] >= n_heads * dh and tuple(out.shape) == (T, n_heads * dh), "attention: q/out shapes")
    _need(block_tables.is_contiguous() and tiles.is_contiguous() and tiles.shape[0] == 4, "attention: tables")
    # (the plain kernel takes any head size up to 256; the bfloat16 kernels and the kernels for single rows take
    # multiples of 16, and a head size that is none goes the plain kernel's way)
    _need(1 <= dh <= 256, lambda: f"attention: head size {dh} must be at most 256")
    _need(n_heads % Hkv == 0, lambda: f"attention: {n_heads} heads over {Hkv} key heads")
    ldq, ldo = _rows(q, "q"), (0 if out_packed else _rows(out, "out"))
    extras = chunk > 0 or bias is not None or bool(sink)
    span = 0
    if bias is not None:
        _dev(bias, "bias", (torch.float32,), 2)
        _need(bias.is_contiguous() and bias.shape[0] == n_heads and bias.shape[1] >= 1, "attention: bias is [heads, span]")
        span = bias.shape[1]
    _need(chunk >= 0, "attention: chunk")
    lib = _lib("attention")
    # (the kernel for portions takes the largest score for the largest product: a scale that is not positive goes the plain way)
    # (with chunks, a bias or a sink the two bfloat16 kernels take pages of a power of two)
    fast = (q.dtype == torch.bfloat16 and ps % 16 == 0 and ldq % 8 == 0 and q.data_ptr() % 16 == 0 and scale > 0
            and (not extras or ps & (ps - 1) == 0))
    decode = fast and decode_attention_applies(q.dtype, ps, dh, single_rows, max_context)
    _need(not out_packed or (fast and attention_writes_packed(q.dtype, ps, dh, single_rows, max_context, tiles_wide)),
          "attention: packed rows as out are written by the bfloat16 kernels only")
    if decode:
        n_tiles = tiles.shape[1]
        # (the split kernel does not read the tiles' rows: tile s is row s)
        _need(n_tiles == T, "attention: a step of single rows has a tile for every row, tile s for row s")
        # a workgroup's waves take 64 keys each at a time: as many waves as make the context one
        # chunk (every load issued at once), within what the head size leaves registers for
        # (where the batch alone gives two workgroups or more per CU the chip is busy anyway, and
        # the smallest workgroups were measured fastest)
        groups = n_tiles * n_heads
        # (a head size that is no power of two leaves lanes empty and needs more registers: from a thousand
        # workgroups on its smallest ones are up to a third faster, where the others' sizes are level)
        many = 8 if dh & (dh - 1) == 0 else 4
        waves = (4 if max_context <= 256 else many if groups >= 1024 else 4 if groups >= 512 else
                 8 if groups >= 300 or max_context <= 512 else 16)
        waves = min(waves, 16 if dh <= 64 else 8 if dh <= 128 else 4)
        if decode_waves is not None:       # (for measurements and tests: 4, 8 or 16 as far as the head size allows)
            _need(decode_waves in (4, 8, 16) and decode_waves <= (16 if dh <= 64 else 8 if dh <= 128 else 4),
                  lambda: f"attention: {decode_waves} waves with a head size of {dh}")
            waves = decode_waves
        # the context is split over workgroups only where the batch alone does not give about one
        # workgroup per CU: a second kernel has to join the splits
        total_chunks = -(-max_context // (waves * 64))
        n_splits = max(1, min(total_chunks, 256 // max(1, n_tiles * n_heads)))
        chunks = -(-total_chunks // n_splits)
        n_splits = -(-total_chunks // chunks)
        _need(max_context <= block_tables.shape[1] * ps, "attention: max_context exceeds the block tables")
        part = torch.empty(n_tiles * n_heads * n_splits * (dh + 2) if n_splits > 1 else 1, dtype=torch.float32,
                           device=q.device)
        base = tiles.data_ptr()
        _ok(lib.dn_attention_decode_extras(
            q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], base, base + 4 * n_tiles, base + 12 * n_tiles, n_tiles, part.data_ptr(), n_splits,
            chunks, waves, n_heads, Hkv, dh, ps, float(scale), int(window), int(chunk), _ptr(bias), span, int(bool(sink)),
            _stream()), "attention (decode)")
        return out
    if fast and tiles_wide is not None and dh in FLASH_HEAD_DIMS:
        _dev(tiles_wide, "tiles_wide", _I32, 2)
        _need(tiles_wide.is_contiguous() and tiles_wide.shape[0] == 4, "attention: tiles_wide")
        n_tiles = tiles_wide.shape[1]
        base = tiles_wide.data_ptr()
        _ok(lib.dn_attention_flash_extras(
            q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], base, base + 4 * n_tiles, base + 8 * n_tiles, base + 12 * n_tiles, n_tiles,
            n_heads, Hkv, dh, ps, float(scale), int(window), int(chunk), _ptr(bias), span, int(bool(sink)), _stream()),
            "attention (flash)")
        return out
    n_tiles = tiles.shape[1]
    base = tiles.data_ptr()
    if single_rows and max_context > 0 and dh % 16 == 0:
        # a step of single rows in the plain kernels: every tile of keys a workgroup of its own, the
        # tiles' results joined in order by a second kernel; the same bits as the kernel below gives
        _need(max_context <= block_tables.shape[1] * ps, "attention: max_context exceeds the block tables")
        _need(n_tiles == T, "attention: a step of single rows has a tile for every row")
        key_tiles = -(-max_context // lib.dn_attention_rows_tile(dh))
        part = torch.empty(n_tiles * n_heads * key_tiles * (dh + 2), dtype=torch.float32, device=q.device)
        _ok(lib.dn_attention_rows_extras(
            q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], base, base + 12 * n_tiles, n_tiles, part.data_ptr(), int(max_context), n_heads, Hkv,
            dh, ps, float(scale), int(window), int(chunk), _ptr(bias), span, int(bool(sink)), _CODE[q.dtype], _stream()),
            "attention (single rows)")
        return out
    _ok(lib.dn_attention_extras(
        q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], base, base + 4 * n_tiles, base + 8 * n_tiles, base + 12 * n_tiles, n_tiles,
        n_heads, Hkv, dh, ps, float(scale), int(window), int(chunk), _ptr(bias), span, int(bool(sink)), _CODE[q.dtype],
        _stream()), "attention")
    return out


def sample(logits, temperature, uniform, out):
    """out[r] = token of row r: the first maximum if temperature[r] <= 0, else the walk with
    uniform[r] in [0,1)."""
    _dev(logits, "logits", (torch.float32,), 2), _dev(temperature, "temperature", (torch.float32,), 1)
    _dev(uniform, "uniform", (torch.float32,), 1), _dev(out, "out", _I32, 1)
    R, V = logits.shape
    ld = _rows(logits, "logits")
    _need(temperature.shape[0] == R and uniform.shape[0] == R and out.shape[0] == R, "sample: rows")
    _ok(_lib("sampling").dn_sample(logits.data_ptr(), ld, R, V, temperature.data_ptr(), uniform.data_ptr(),
                                   out.data_ptr(), _stream()), "sample")
    return out


def sample_top(logits, rows, temperature, uniform, top_k, top_p, out, undecided):
    """For the rows listed in `rows` (each with temperature > 0): top_k[j] largest candidates
    (0: no limit but the 2048 that the kernel keeps), cut at cumulative probability top_p[j]
    (1: no cut), then the walk with uniform[row].  temperature, uniform and out are indexed by
    row, top_k, top_p and undecided by the place in `rows`.  undecided[j] = 1: top-p alone did not
    find its cut before the last of the 2048 candidates; the row needs `sample_full`."""
    _dev(logits, "logits", (torch.float32,), 2), _dev(rows, "rows", _I32, 1)
    _dev(temperature, "temperature", (torch.float32,), 1), _dev(uniform, "uniform", (torch.float32,), 1)
    _dev(top_k, "top_k", _I32, 1), _dev(top_p, "top_p", (torch.float32,), 1), _dev(out, "out", _I32, 1)
    _dev(undecided, "undecided", _I32, 1)
    R, V = logits.shape
    ld = _rows(logits, "logits")
    n = rows.shape[0]
    _need(top_k.shape[0] == n and top_p.shape[0] == n and undecided.shape[0] == n,
          "sample_top: one top_k, top_p and undecided per listed row")
    _need(temperature.shape[0] == R and uniform.shape[0] == R and out.shape[0] == R, "sample_top: rows")
    work = torch.empty(max(1, n) * V, dtype=torch.int32, device=logits.device)      # every row's keys, made once
    _ok(_lib("sampling").dn_sample_top(logits.data_ptr(), ld, n, V, rows.data_ptr(), temperature.data_ptr(),
                                       uniform.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), out.data_ptr(),
                                       undecided.data_ptr(), work.data_ptr(), _stream()), "sample_top")
    return out


def sample_full(logits, rows, temperature, uniform, top_p, out, only=None):
    """top-p over the whole sorted vocabulary for the rows listed in `rows` (each with temperature
    > 0), then the walk with uniform[row]: what `sample_top` leaves undecided.  only: int32, a flag per listed
    row, on the device; a row whose flag is 0 keeps its token (`sample_top`'s `undecided`: launched behind it, the
    rows that it left undecided are done without the host reading which they are)."""
    _dev(logits, "logits", (torch.float32,), 2), _dev(rows, "rows", _I32, 1)
    _dev(temperature, "temperature", (torch.float32,), 1), _dev(uniform, "uniform", (torch.float32,), 1)
    _dev(top_p, "top_p", (torch.float32,), 1), _dev(out, "out", _I32, 1)
    R, V = logits.shape
    ld = _rows(logits, "logits")
    n = rows.shape[0]
    _need(top_p.shape[0] == n, "sample_full: one top_p per listed row")
    if only is not None:
        _dev(only, "only", _I32, 1)
        _need(only.shape[0] == n and only.is_contiguous(), "sample_full: one flag per listed row")
    _need(temperature.shape[0] == R and uniform.shape[0] == R and out.shape[0] == R, "sample_full: rows")
    n_pad = 2
    while n_pad < V:
        n_pad *= 2
    work = torch.empty(n * 3 * n_pad, dtype=torch.int32, device=logits.device)
    _ok(_lib("sampling").dn_sample_full(logits.data_ptr(), ld, n, V, n_pad, rows.data_ptr(), temperature.data_ptr(),
                                        uniform.data_ptr(), top_p.data_ptr(), _ptr(only), work.data_ptr(),
                                        out.data_ptr(), _stream()), "sample_full")
    return out


def penalties(logits, ctx, begin, length, repetition, frequency, presence, ngram, bounds=None):
    """In place on logits [R, V]: repetition, frequency, presence penalties and the n-gram ban,
    each row over its own context ctx[begin[r] : begin[r] + length[r]] (ctx: int32, one dimension: the
    contexts one after the other, or a table of histories seen as one run).  bounds: the largest
    begin + length, as the host knows it (the tables themselves are on the device)."""
    _dev(logits, "logits", (torch.float32,), 2)
    R, V = logits.shape
    ld = _rows(logits, "logits")
    _dev(ctx, "ctx", _I32, 1), _dev(begin, "begin", _I32, 1), _dev(length, "length", _I32, 1)
    _need(ctx.is_contiguous() and begin.shape[0] == R and length.shape[0] == R, "penalties: one begin and one length per row")
    _need(bounds is None or 0 <= bounds <= ctx.shape[0], "penalties: a context beyond the end of ctx")
    for t, n in ((repetition, "repetition"), (frequency, "frequency"), (presence, "presence")):
        _dev(t, n, (torch.float32,), 1)
        _need(t.shape[0] == R, lambda: f"penalties: {n}")
    _dev(ngram, "ngram", _I32, 1)
    _need(ngram.shape[0] == R, "penalties: ngram")
    _ok(_lib("sampling").dn_penalties(logits.data_ptr(), ld, R, V, ctx.data_ptr(), begin.data_ptr(), length.data_ptr(),
                                      repetition.data_ptr(), frequency.data_ptr(), presence.data_ptr(),
                                      ngram.data_ptr(), _stream()), "penalties")
    return logits


def history_append(history, begin, length, rows, tokens, bounds=None):
    """history[begin[j] + length[j]] = tokens[rows[j]] for every j: the tokens sampled for the listed rows, each
    into its request's history (int32, one dimension) at the history's next place.  bounds: (the largest
    begin + length, the largest row), as the host knows them."""
    for t, n in ((history, "history"), (begin, "begin"), (length, "length"), (rows, "rows"), (tokens, "tokens")):
        _dev(t, n, _I32, 1)
        _need(t.is_contiguous(), lambda: f"history_append: {n}")
    n = begin.shape[0]
    _need(length.shape[0] == n and rows.shape[0] == n, "history_append: one length and one row per begin")
    if bounds is not None:
        _need(0 <= bounds[0] < history.shape[0] and 0 <= bounds[1] < tokens.shape[0], "history_append: beyond the history or the tokens")
    _ok(_lib("sampling").dn_history_append(history.data_ptr(), begin.data_ptr(), length.data_ptr(), rows.data_ptr(),
                                           tokens.data_ptr(), n, _stream()), "history_append")
    return history


# ---------------------------------------------------------------------------------------
# A norm that runs inside the products before and after it (steps of at most 16 rows)
# ---------------------------------------------------------------------------------------
NORM_STREAM_ROWS_MAX = 64     # 0 switches it off: norms then run as kernels of their own
NORM_STREAM_WIDTH_MAX = 4096


def norm_stream_takes(n_rows, width, w):
    """Whether linear_norm_out can leave, and linear_norm_in can use, what a norm of n_rows rows of
    `width` columns needs, with the packed weight w [out, in] of the product in question.  Up to 16
    rows: widths that are multiples of 16, up to 4,096.  17 to 64 rows (the rows then travel
    packed): widths that are multiples of 32 from 1,024 to 2,048, and products of at least 1,024 inner
    columns."""
    if not isinstance(w, PackedMatrix) or not 1 <= n_rows <= NORM_STREAM_ROWS_MAX:
        return False
    if n_rows <= 16:
        return width % 16 == 0 and 16 <= width <= NORM_STREAM_WIDTH_MAX
    return n_rows <= 64 and width % 32 == 0 and 1024 <= width <= 2048 and w.shape[1] >= 1024


def norm_stream_buffers(n_rows, width, device):
    """(copy, stats): the residual stream's rows times the next norm's weight, in bfloat16 ([n_rows,
    width], from 17 rows on as packed rows), and, per row and block of 16 columns, the mean and
    the sum of squared distances from it [n_rows, width / 16, 2]."""
    copy = (packed_rows(n_rows, width, device) if n_rows >= PACKED_ROWS_MIN else
            torch.empty((n_rows, width), dtype=torch.bfloat16, device=device))
    return copy, torch.empty((n_rows, width // 16, 2), dtype=torch.float32, device=device)


def norm_folded(w_rows, bias, gamma, beta, no_mean=False):
    """(c1, c2) for linear_norm_in: with y = (x - mean) / sqrt(var + eps) * gamma + beta,
    y @ w.T + bias = ((x * gamma) @ w.T - mean * c1) / sqrt(var + eps) + c2, where
    c1 = w @ gamma and c2 = w @ beta + bias, in 32-bit from the weight as the kernel holds it.
    w_rows: [N, K] (any float dtype); made once per pair of norm and weight.  no_mean: a norm that takes no
    mean off (an RMS norm): c1 is zeros and is not used."""
    w = w_rows.float()
    c1 = torch.zeros(w.shape[0], dtype=torch.float32, device=w.device) if no_mean else w @ gamma.float()
    c2 = torch.zeros_like(c1) if beta is None else w @ beta.float()
    if bias is not None:
        c2 = c2 + bias.float()
    return c1.contiguous(), c2.contiguous()


def _rows_or_packed(t, name, M, width):
    """The leading dimension of a bfloat16 [M, width] tensor in rows, or 0 for packed rows."""
    if isinstance(t, PackedMatrix):
        _need(tuple(t.shape) == (M, width) and width % 32 == 0, lambda: f"{name}: packed rows of another shape")
        return 0
    _dev(t, name, (torch.bfloat16,), 2)
    _need(tuple(t.shape) == (M, width), lambda: f"{name}: shape")
    return _rows(t, name)


def linear_norm_out(a, w, bias, residual, gamma, copy, stats):
    """residual += a @ w.T + bias (32-bit, in place), and what a LayerNorm of the updated rows with
    weight gamma needs: copy = the rows times gamma in bfloat16 (a tensor, or packed rows), stats =
    each row's means and squared distances by blocks of 16 columns.  a: bfloat16 [M, K] in rows or
    packed rows; w: PackedMatrix [N, K], N a multiple of 16."""
    _dev(residual, "residual", (torch.float32,), 2)
    M, K = a.shape
    N = w.shape[0]
    _need(norm_stream_takes(M, N, w) and w.shape[1] == K and K % 8 == 0, "linear_norm_out: sizes it does not take")
    lda, ldcopy = _rows_or_packed(a, "a", M, K), _rows_or_packed(copy, "copy", M, N)
    _need(M > 16 or lda > 0, "linear_norm_out: up to 16 rows come in rows")
    _need(tuple(residual.shape) == (M, N) and tuple(stats.shape) == (M, N // 16, 2) and stats.dtype == torch.float32
          and stats.is_contiguous(), "linear_norm_out: residual or stats")
    for v, name in ((bias, "bias"), (gamma, "gamma")):
        if v is not None:
            _dev(v, name, (torch.float32,), 1)
            _need(v.is_contiguous() and v.shape[0] == N, lambda: f"linear_norm_out: {name}")
    _need(gamma is not None, "linear_norm_out: gamma")
    _ok(_lib("gemm").dn_gemm_norm_out(a.data_ptr(), lda, w.data_ptr(), _ptr(bias), residual.data_ptr(),
                                      _rows(residual, "residual"), M, N, K, gamma.data_ptr(), copy.data_ptr(),
                                      ldcopy, stats.data_ptr(), _stream()),
        "linear_norm_out" if _timed is None else f"linear {K} -> {N}, added into the stream, leaves the next norm's statistics")
    return residual


def linear_norm_in(copy, stats, c1, c2, eps, w, out, epilogue="none", kv=None, no_mean=False):
    """out = epilogue(LayerNorm(x) @ w.T + bias) where copy and stats are what linear_norm_out left
    of x (with this norm's gamma) and c1, c2 = norm_folded(w, bias, gamma, beta).  out: bfloat16
    [M, N]; kv = (slot_map, k_pool, v_pool, q_width): a fused projection whose key and value columns
    go to the cache (out may then hold the queries alone); returns out, or the queries.
    no_mean: the norm takes no mean off (x / sqrt(mean(x^2) + eps) * gamma); c1 is then not used."""
    M, K = copy.shape
    N = w.shape[0]
    _need(norm_stream_takes(M, K, w) and w.shape[1] == K, "linear_norm_in: sizes it does not take")
    if isinstance(out, PackedMatrix):
        _need(kv is None and M > 16 and N % 32 == 0, "linear_norm_in: packed rows as out need 17 rows or more, N a multiple of 32, no cache write")
        ldc = 0
    else:
        _dev(out, "out", (torch.bfloat16,), 2)
        ldc = _rows(out, "out")
    lda = _rows_or_packed(copy, "copy", M, K)
    _need(M > 16 or lda > 0, "linear_norm_in: up to 16 rows come in rows")
    _need(tuple(stats.shape) == (M, K // 16, 2) and stats.dtype == torch.float32 and stats.is_contiguous(),
          "linear_norm_in: stats")
    for v, name in ((c1, "c1"), (c2, "c2")):
        _dev(v, name, (torch.float32,), 1)
        _need(v.is_contiguous() and v.shape[0] == N, lambda: f"linear_norm_in: {name}")
    if kv is None:
        _need(tuple(out.shape) == (M, N), "linear_norm_in: out shape")
        args = (0, 0, 0, 0, 0, 0, 0, 0)
    else:
        slot_map, k_pool, v_pool, q_width = kv
        n_pages, Hkv, ps, dh = k_pool.shape
        _need(N == q_width + 2 * Hkv * dh and out.shape[0] == M and out.shape[1] in (N, q_width),
              "linear_norm_in: columns are not q | k | v, or out's shape")
        _dev(slot_map, "slot_map", _I32, 1), _dev(k_pool, "k_pool", (torch.bfloat16,), 4)
        _dev(v_pool, "v_pool", (torch.bfloat16,), 4)
        _need(k_pool.is_contiguous() and v_pool.is_contiguous() and tuple(v_pool.shape) == (n_pages, Hkv, dh, ps)
              and slot_map.is_contiguous() and slot_map.shape[0] == M and dh % 4 == 0, "linear_norm_in: pools or slot map")
        args = (slot_map.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), q_width, Hkv, dh, ps, out.shape[1])
    _ok(_lib("gemm").dn_gemm_norm_in(copy.data_ptr(), lda, stats.data_ptr(), c1.data_ptr(),
                                     c2.data_ptr(), float(eps), w.data_ptr(), out.data_ptr(), ldc,
                                     M, N, K, EPILOGUES[epilogue], *args, int(bool(no_mean)), _stream()),
        "linear_norm_in" if _timed is None else
        f"norm + linear {K} -> {N}" + (", cache write" if kv is not None else "") + (f", {epilogue}" if epilogue != "none" else ""))
    return out if kv is None else out[:, :kv[3]]


# -- layers that carry more than keys and values from token to token (csrc/kernels/sequence.hip) -----------------------
ACTIVATIONS = {"silu": 0, "sigmoid": 1, "tanh": 2, "exp_neg_exp": 3, "bounded_sigmoid": 4, "exp_neg_softplus": 5, "xielu": 6, "relu2": 7}


def _f32vec(t, name, n=None):
    if t is None:
        return None
    _dev(t, name, (torch.float32,))
    _need(t.is_contiguous() and (n is None or t.numel() == n), lambda: f"{name}: {tuple(t.shape)}, wanted {n} contiguous 32-bit numbers")
    return t


def _request_tables(row_start, slots, what):
    _dev(row_start, "row_start", _I32, 1), _dev(slots, "slots", _I32, 1)
    S = slots.shape[0]
    _need(row_start.is_contiguous() and slots.is_contiguous() and row_start.shape[0] == S + 1 and S >= 1, lambda: f"{what}: tables")
    return S


def _history(hist, n_floats, what):
    """A state tensor [slots, n_floats] whose rows are contiguous; -> a slot's stride in floats."""
    _dev(hist, "history", (torch.float32,), 2)
    _need(hist.shape[1] == n_floats and (hist.stride(1) == 1 or n_floats == 1), lambda: f"{what}: history {tuple(hist.shape)}, wanted [slots, {n_floats}]")
    return hist.stride(0)


def rmsnorm(x, weight, eps, out, rows=None):
    """out[r, :] = x[rows[r], :E] / sqrt(mean(x[.., :E]^2) + eps) * weight, E = out.shape[1] (the first E columns of x;
    rows None: every row; weight None: no weight).  32-bit statistics; x and out may be the same tensor."""
    _dev(x, "x", _FLOATS, 2), _dev(out, "out", _FLOATS, 2)
    E = out.shape[1]
    ldx, ldo = _rows(x, "x"), _rows(out, "out")
    _need(x.shape[1] >= E, "rmsnorm: x is narrower than out")
    _f32vec(weight, "weight", E)
    if rows is not None:
        _dev(rows, "rows", _I32, 1)
        _need(rows.is_contiguous() and rows.shape[0] == out.shape[0], "rmsnorm: rows")
    else:
        _need(out.shape[0] == x.shape[0], "rmsnorm: out rows")
    _ok(_lib("sequence").dn_rmsnorm(x.data_ptr(), _CODE[x.dtype], ldx, _ptr(weight), out.data_ptr(), _CODE[out.dtype], ldo,
                                    _ptr(rows), out.shape[0], E, float(eps), _stream()), "rmsnorm")
    return out


def _then(then, T, width, what):
    """then = (weight or None, eps, out): the norm that reads the stream next, made by the same kernel -> its five arguments."""
    if then is None:
        return 0, 0.0, 0, 0, 0
    w, eps, out = then
    _f32vec(w, "next weight", width), _dev(out, "next out", _FLOATS, 2)
    _need(tuple(out.shape) == (T, width), lambda: f"{what}: the next norm's rows")
    return _ptr(w), float(eps), out.data_ptr(), _CODE[out.dtype], _rows(out, "next out")


def rmsnorm_add(y, weight, scale, mult, eps, x, gate=None, then=None):
    """x[t, :] += mult * (y[t, :] / sqrt(mean(y[t, :]^2) + eps) * weight) * scale; weight and scale: 32-bit vectors or None;
    x: 32-bit rows (the stream), changed in place; statistics in 32-bit.  gate: 32-bit [T, width] (columns of wider rows):
    y is y * sigmoid(gate) first, under the norm too.  then = (weight or None, eps, out): out[t, :] = x[t, :] / sqrt(mean(x[t, :]^2)
    + eps) * weight on the rows as they then stand, the same bits as `rmsnorm` behind this call."""
    _dev(y, "y", _FLOATS, 2), _dev(x, "x", (torch.float32,), 2)
    T, width = y.shape
    _need(tuple(x.shape) == (T, width), "rmsnorm_add: shapes")
    _f32vec(weight, "weight", width), _f32vec(scale, "scale", width)
    if gate is not None:
        _dev(gate, "gate", (torch.float32,), 2)
        _need(tuple(gate.shape) == (T, width), "rmsnorm_add: gate")
    _ok(_lib("sequence").dn_rmsnorm_add(y.data_ptr(), _CODE[y.dtype], _rows(y, "y"), _ptr(weight), _ptr(scale), float(mult),
                                        x.data_ptr(), _rows(x, "x"), T, width, float(eps), _ptr(gate),
                                        _rows(gate, "gate") if gate is not None else 0, *_then(then, T, width, "rmsnorm_add"),
                                        _stream()), "rmsnorm_add")
    return x


def depth_mix(hist, n, weights, out):
    """out = sum over j < n of weights[j] * hist[j], j ascending; hist: 32-bit [planes, rows, width], contiguous; weights:
    at least n 32-bit numbers; out: 32-bit [rows, width], contiguous; it may be a plane of hist from n on."""
    _dev(hist, "hist", (torch.float32,), 3), _dev(out, "out", (torch.float32,), 2)
    _f32vec(weights, "weights")
    planes, T, width = hist.shape
    _need(hist.is_contiguous() and out.is_contiguous() and tuple(out.shape) == (T, width) and 1 <= n <= planes
          and weights.numel() >= n, "depth_mix: shapes")
    _ok(_lib("sequence").dn_depth_mix(hist.data_ptr(), T * width, n, weights.data_ptr(), out.data_ptr(), T * width, _stream()),
        "depth_mix")
    return out


def unit_heads(x, n_heads, dim, eps, scale, out):
    """out[t, h, :] = x[t, h, :] / sqrt(sum(x[t, h, :]^2) + eps) * scale for the n_heads vectors of `dim` numbers at the start
    of each row; x and out 32-bit (out may be x)."""
    _dev(x, "x", (torch.float32,), 2), _dev(out, "out", (torch.float32,), 2)
    T = x.shape[0]
    _need(out.shape[0] == T and x.shape[1] >= n_heads * dim and out.shape[1] >= n_heads * dim and n_heads >= 1 and dim >= 1,
          "unit_heads: shapes")
    _ok(_lib("sequence").dn_unit_heads(x.data_ptr(), _rows(x, "x"), out.data_ptr(), _rows(out, "out"), T, n_heads, dim, float(eps),
                                       float(scale), _stream()), "unit_heads")
    return out


def concat_cast(a, b, out):
    """out[t, :] = [a[t, :] | b[t, :]], a and b 32-bit, out contiguous in its own dtype."""
    _dev(a, "a", (torch.float32,), 2), _dev(b, "b", (torch.float32,), 2), _dev(out, "out", _FLOATS, 2)
    T = a.shape[0]
    _need(b.shape[0] == T and tuple(out.shape) == (T, a.shape[1] + b.shape[1]) and out.is_contiguous(), "concat_cast: shapes")
    _ok(_lib("sequence").dn_concat_cast(a.data_ptr(), _rows(a, "a"), a.shape[1], b.data_ptr(), _rows(b, "b"), b.shape[1],
                                        out.data_ptr(), _CODE[out.dtype], T, _stream()), "concat_cast")
    return out


def conv_rows(h, w, hist, row_start, slots, out, identity=True, act=None, bias=None):
    """out[t, c] = act((h[t, c] if identity else 0) + bias[c] + sum_j w[c, j] h[t - taps + 1 + j, c]) inside each request; the rows
    before a request's first row of this step come from hist [slots, (taps - 1) * width] (oldest first).  h: 32-bit rows whose
    first `width` columns are the channels (width = w.shape[0]); act: None or "silu"."""
    _dev(h, "h", (torch.float32,), 2), _dev(w, "w", (torch.float32,), 2), _dev(out, "out", _FLOATS, 2)
    T = h.shape[0]
    width, taps = w.shape
    S = _request_tables(row_start, slots, "conv_rows")
    _need(h.shape[1] >= width and w.is_contiguous() and tuple(out.shape) == (T, width) and act in (None, "silu"), "conv_rows: shapes")
    stride = _history(hist, (taps - 1) * width, "conv_rows") if taps > 1 else 0
    _f32vec(bias, "bias", width)
    _ok(_lib("sequence").dn_conv_rows(h.data_ptr(), _rows(h, "h"), w.data_ptr(), _ptr(bias), _ptr(hist) if taps > 1 else 0, row_start.data_ptr(),
                                      slots.data_ptr(), S, T, width, taps, int(bool(identity)), int(act == "silu"), out.data_ptr(),
                                      _CODE[out.dtype], _rows(out, "out"), stride, _stream()),
        "conv_rows")
    return out


def history_update(h, hist, row_start, slots):
    """hist [slots, keep * width]: the last `keep` rows of (a request's history ++ its rows of this step) become its history;
    width = h.shape[1] (h may be the first columns of wider rows)."""
    _dev(h, "h", _FLOATS, 2)
    T, width = h.shape
    S = _request_tables(row_start, slots, "history_update")
    _dev(hist, "history", (torch.float32,), 2)
    _need(hist.shape[1] % width == 0, "history_update: shapes")
    keep = hist.shape[1] // width
    stride = _history(hist, keep * width, "history_update")
    _ok(_lib("sequence").dn_history_update(h.data_ptr(), _CODE[h.dtype], _rows(h, "h"), hist.data_ptr(), row_start.data_ptr(),
                                           slots.data_ptr(), S, width, keep, stride, _stream()), "history_update")


def conv_heads(h, w, hist, row_start, slots, out, n_unit, unit_dim, n_first, scale_first, scale_rest, eps, n_rest, rest_dim):
    """conv_rows(identity=False, act="silu") over channels that are heads' vectors, and the first n_unit vectors (unit_dim
    channels each; n_rest more of rest_dim follow) made unit vectors on the way out: x / sqrt(sum(x^2) + eps), times
    scale_first for the first n_first of them and scale_rest for the others.  h: 32-bit rows whose first columns are the
    channels; out: 32-bit [T, channels]."""
    _dev(h, "h", (torch.float32,), 2), _dev(w, "w", (torch.float32,), 2), _dev(out, "out", (torch.float32,), 2)
    T = h.shape[0]
    width, taps = w.shape
    S = _request_tables(row_start, slots, "conv_heads")
    _need(width == n_unit * unit_dim + n_rest * rest_dim and h.shape[1] >= width and w.is_contiguous() and tuple(out.shape) == (T, width)
          and 0 <= n_first <= n_unit and n_unit + n_rest >= 1 and n_unit + n_rest <= 65535, "conv_heads: shapes")
    stride = _history(hist, (taps - 1) * width, "conv_heads") if taps > 1 else 0
    _ok(_lib("sequence").dn_conv_heads(h.data_ptr(), _rows(h, "h"), w.data_ptr(), _ptr(hist) if taps > 1 else 0, row_start.data_ptr(),
                                       slots.data_ptr(), S, T, taps, n_unit, unit_dim, n_first, float(scale_first), float(scale_rest),
                                       float(eps), n_rest, rest_dim, out.data_ptr(), _rows(out, "out"), stride, _stream()), "conv_heads")
    return out


def rotary_runs(src, positions, freq, runs, mag=1.0, unit=None, eps=0.0):
    """Up to three runs of vectors of src's rows in one launch.  runs: [(dst, src_off, n_vec, width, dims, dst_off, dst_stride)]:
    the n_vec vectors of `width` numbers that lie side by side from column src_off go to columns dst_off + n * dst_stride of
    dst, their first `dims` entries turned in pairs by positions[t] * freq[i] (dims 0: only moved); as `rotary` does.
    mag multiplies cos and sin.  unit: a flag per run: the run's vectors are divided by their root mean square behind the
    turn, x / sqrt(mean(x^2) + eps) over their `width` entries (vectors of up to 256 numbers then, in every run)."""
    _dev(src, "src", _FLOATS, 2), _dev(positions, "positions", _I32, 1)
    T = src.shape[0]
    _need(1 <= len(runs) <= 3 and positions.is_contiguous() and positions.shape[0] == T, "rotary_runs: runs or rows")
    unit = [False] * len(runs) if unit is None else [bool(u) for u in unit]
    _need(len(unit) == len(runs), "rotary_runs: a unit flag per run")
    table, most = [], 0
    for dst, src_off, n_vec, width, dims, dst_off, dst_stride in runs:
        _dev(dst, "dst", _FLOATS, 2)
        _need(dst.shape[0] == T and dims % 2 == 0 and 0 <= dims <= width and n_vec >= 0, "rotary_runs: a run's sizes")
        _need(not any(unit) or width <= 256, lambda: f"rotary_runs: vectors of {width} numbers; with a norm behind the turn up to 256")
        if n_vec:
            _need(src_off >= 0 and src_off + n_vec * width <= src.shape[1] and dst_off >= 0
                  and dst_off + (n_vec - 1) * dst_stride + width <= dst.shape[1], "rotary_runs: vectors outside their rows")
        table += [dst.data_ptr(), _CODE[dst.dtype], _rows(dst, "dst"), src_off, dst_off, dst_stride, n_vec, width, dims]
        most = max(most, dims)
    _f32vec(freq, "freq")
    _need(freq.numel() >= most // 2 and all(r[4] in (0, most) for r in runs), "rotary_runs: one table of frequencies for the turned runs")
    import ctypes
    arr = (ctypes.c_longlong * len(table))(*table)
    mask = sum(1 << i for i, u in enumerate(unit) if u)
    _ok(_lib("sequence").dn_rotary_runs(src.data_ptr(), _CODE[src.dtype], _rows(src, "src"), arr, len(runs), positions.data_ptr(),
                                        freq.data_ptr(), T, float(mag), mask, float(eps), _stream()), "rotary_runs")


def shift_mix(h, hist, mu, row_start, slots, out):
    """out[m, t, :] = h[t] + (h[t - 1] - h[t]) * mu[m]; the row before a request's first row of the step is hist[slot]."""
    _dev(h, "h", _FLOATS, 2), _dev(out, "out", _FLOATS, 3)
    T, width = h.shape
    n = mu.shape[0]
    S = _request_tables(row_start, slots, "shift_mix")
    _f32vec(mu, "mu", n * width)
    _need(h.is_contiguous() and out.is_contiguous() and tuple(out.shape) == (n, T, width), "shift_mix: shapes")
    stride = _history(hist, width, "shift_mix")
    _ok(_lib("sequence").dn_shift_mix(h.data_ptr(), _CODE[h.dtype], hist.data_ptr(), mu.data_ptr(), n, row_start.data_ptr(),
                                      slots.data_ptr(), S, T, width, out.data_ptr(), _CODE[out.dtype], stride, _stream()), "shift_mix")
    return out


def rotary(src, dst, positions, freq, n_vec, dims, width, src_off=0, src_stride=None, dst_off=0, dst_stride=None, mag=1.0):
    """Vector n (n < n_vec) of row t, `width` wide, starts at column src_off + n * src_stride of src; of its first `dims`
    entries, 2i and 2i + 1 are turned by positions[t] * freq[i] (32-bit angles; cos and sin times `mag`), the rest pass; it
    goes to column dst_off + n * dst_stride of dst (which may be src)."""
    _dev(src, "src", _FLOATS, 2), _dev(dst, "dst", _FLOATS, 2), _dev(positions, "positions", _I32, 1)
    T = src.shape[0]
    src_stride = width if src_stride is None else src_stride
    dst_stride = width if dst_stride is None else dst_stride
    _f32vec(freq, "freq", dims // 2)
    _need(dst.shape[0] == T and positions.is_contiguous() and positions.shape[0] == T, "rotary: rows")
    _need(dims % 2 == 0 and 0 <= dims <= width and n_vec >= 0, "rotary: dims")
    if n_vec:
        _need(src_off >= 0 and src_off + (n_vec - 1) * src_stride + width <= src.shape[1]
              and dst_off >= 0 and dst_off + (n_vec - 1) * dst_stride + width <= dst.shape[1], "rotary: vectors outside their rows")
    _ok(_lib("sequence").dn_rotary(src.data_ptr(), _CODE[src.dtype], _rows(src, "src"), src_off, src_stride, dst.data_ptr(),
                                   _CODE[dst.dtype], _rows(dst, "dst"), dst_off, dst_stride, positions.data_ptr(), freq.data_ptr(),
                                   T, n_vec, dims, width, float(mag), _stream()), "rotary")
    return dst


def activate(x, kind, out, bias=None, lower=None):
    """out = act(x + bias): "silu", "sigmoid", "tanh", "exp_neg_exp" (exp(-exp(z))), "bounded_sigmoid"
    (lower + (1 - lower) * sigmoid(z)), "exp_neg_softplus" (exp(-lower * log(1 + e^z)), lower a rate per column), "xielu"
    (z > 0: a z^2 + z / 2, else b (e^z - 1 - z) + z / 2, with lower = (a, b), two numbers), "relu2" (max(z, 0)^2).  x 32-bit; out
    may be x."""
    _dev(x, "x", (torch.float32,), 2), _dev(out, "out", _FLOATS, 2)
    T, n = x.shape
    _need(tuple(out.shape) == (T, n), "activate: shapes")
    _need(kind not in ("xielu", "exp_neg_softplus") or lower is not None, lambda: f"activate: {kind} needs its numbers in `lower`")
    _f32vec(bias, "bias", n), _f32vec(lower, "lower", 2 if kind == "xielu" else n)
    _ok(_lib("sequence").dn_activate(x.data_ptr(), _rows(x, "x"), _ptr(bias), _ptr(lower), ACTIVATIONS[kind], out.data_ptr(),
                                     _CODE[out.dtype], _rows(out, "out"), T, n, _stream()), "activate")
    return out


def gated(x, g, kind, out):
    """out = x * act(g), act "silu", "sigmoid" or "tanh"; g 32-bit."""
    _dev(x, "x", _FLOATS, 2), _dev(g, "g", (torch.float32,), 2), _dev(out, "out", _FLOATS, 2)
    T, n = x.shape
    _need(tuple(g.shape) == (T, n) and tuple(out.shape) == (T, n) and kind in ("silu", "sigmoid", "tanh"), "gated: shapes")
    _ok(_lib("sequence").dn_gated(x.data_ptr(), _CODE[x.dtype], _rows(x, "x"), g.data_ptr(), _rows(g, "g"), ACTIVATIONS[kind],
                                  out.data_ptr(), _CODE[out.dtype], _rows(out, "out"), T, n, _stream()), "gated")
    return out


def state_scan(r, k, v, w, u, state, row_start, slots, n_heads, dk, dv, out, read_after=False, key_from_decay=False, beta=None,
               w_head=None, qk_heads=None, beta_logits=False, w_rows=False):
    """The recurrence of a matrix state per head, S [dk, dv], over each request's rows of this step in order:
      a = 1 - w if key_from_decay else k
      read_after:  S <- diag(w) S + a v^T ;  o = S^T r
      beta given:  S <- diag(w) S ;  e = beta (v - S^T a) ;  S <- S + a e^T ;  o = S^T r        (the delta rule)
      else:        o = (S + diag(u) a v^T)^T r ;  S <- diag(w) S + a v^T        (u None: no bonus)
    r, k: 32-bit [T, qk_heads * dk] (qk_heads None: n_heads; fewer: head h reads head h // (n_heads // qk_heads));
    w: 32-bit [T, heads * dk], or (w_rows) [T, heads], one decay per row and head for all the head's channels, or None with
    w_head: 32-bit [heads], one decay per head for every row and channel;
    v, out: 32-bit [T, heads * dv]; beta: 32-bit [T, heads] (beta_logits: it holds z, and beta is 1 / (1 + e^-z)); state: 32-bit [slots, heads * dv * dk] (a head's state
    held [value column][key channel]), read and written at the requests' slots."""
    G = n_heads if qk_heads is None else qk_heads
    _need(G >= 1 and n_heads % G == 0, lambda: f"state_scan: {n_heads} heads over {G} heads of queries and keys")
    _need((w is None) != (w_head is None), "state_scan: a decay per row and channel (w) or one per head (w_head)")
    _need(not (key_from_decay and (w is None or w_rows)), "state_scan: keys from the decay need w per channel")
    _need(not w_rows or w is not None, "state_scan: w_rows needs w")
    given = ((r, "r", G * dk), (v, "v", n_heads * dv), (out, "out", n_heads * dv)) + (() if key_from_decay else ((k, "k", G * dk),)) \
        + (() if w is None else ((w, "w", n_heads if w_rows else n_heads * dk),)) + (() if beta is None else ((beta, "beta", n_heads),))
    for t, name, n in given:
        _dev(t, name, (torch.float32,), 2)
        _need(t.shape[1] == n, lambda: f"state_scan: {name} {tuple(t.shape)}")
    T = r.shape[0]
    S = _request_tables(row_start, slots, "state_scan")
    _need(all(t.shape[0] == T for t, _, _ in given), "state_scan: rows")
    _need(1 <= dk <= 256, lambda: f"state_scan: {dk} key channels a head; the kernel keeps up to 256 in registers")
    _need(beta is None or (not read_after and u is None), "state_scan: the delta rule reads after its write and has no bonus")
    _f32vec(u, "u", n_heads * dk), _f32vec(w_head, "w_head", n_heads)
    stride = _history(state, n_heads * dk * dv, "state_scan")
    mode = 2 if beta is not None else int(bool(read_after))
    _ok(_lib("sequence").dn_state_scan(r.data_ptr(), _rows(r, "r"), 0 if key_from_decay else k.data_ptr(),
                                       0 if key_from_decay else _rows(k, "k"), v.data_ptr(), _rows(v, "v"), _ptr(w),
                                       _rows(w, "w") if w is not None else 0, _ptr(u), _ptr(beta),
                                       _rows(beta, "beta") if beta is not None else 0, _ptr(w_head), G, state.data_ptr(), stride,
                                       row_start.data_ptr(), slots.data_ptr(), S, T, n_heads, dk, dv, mode, int(key_from_decay),
                                       int(bool(beta_logits)), int(bool(w_rows)), out.data_ptr(), _rows(out, "out"), _stream()),
        "state_scan" if beta is None else "state_scan (delta rule)")
    return out


def head_norm(o, weight, eps, out, n_heads, gate=None, gate_kind="silu", gate_first=False, skip=None, skip_scale=None):
    """y = o (+ skip * skip_scale, a second summand [T, n] with a number per run of n / len(skip_scale) columns); gate_first: y
    times act(gate) before the norm, else behind it; out[t, h, :] = y[t, h, :] / sqrt(mean(y[t, h, :]^2) + eps) * weight.
    weight: None, one per column of o, or one per column of a head (shared by the heads); o, gate and skip 32-bit."""
    _dev(o, "o", (torch.float32,), 2), _dev(out, "out", _FLOATS, 2)
    T, n = o.shape
    _need(n % n_heads == 0 and tuple(out.shape) == (T, n), "head_norm: shapes")
    dv = n // n_heads
    w_stride = 0
    if weight is not None:
        _f32vec(weight, "weight")
        _need(weight.numel() in (n, dv), "head_norm: weight")
        w_stride = dv if weight.numel() == n and n_heads > 1 else 0
    if gate is not None:
        _dev(gate, "gate", (torch.float32,), 2)
        _need(tuple(gate.shape) == (T, n) and gate_kind in ("silu", "sigmoid", "tanh"), "head_norm: gate")
    skip_dim = 0
    if skip is not None:
        _dev(skip, "skip", (torch.float32,), 2), _f32vec(skip_scale, "skip_scale")
        _need(tuple(skip.shape) == (T, n) and skip_scale is not None and skip_scale.numel() >= 1 and n % skip_scale.numel() == 0,
              "head_norm: skip")
        skip_dim = n // skip_scale.numel()
    _ok(_lib("sequence").dn_head_norm(o.data_ptr(), _rows(o, "o"), _ptr(weight), w_stride, float(eps), _ptr(gate),
                                      _rows(gate, "gate") if gate is not None else 0, ACTIVATIONS[gate_kind], int(bool(gate_first)),
                                      _ptr(skip), _rows(skip, "skip") if skip is not None else 0, _ptr(skip_scale), skip_dim,
                                      out.data_ptr(), _CODE[out.dtype], _rows(out, "out"), T, n_heads, dv, _stream()), "head_norm")
    return out


def step_sizes(z, bias, rate, x, n_heads, decay, v):
    """dt = log(1 + e^(z[t, h] + bias[h])); decay[t, h] = exp(-rate[h] * dt); v[t, h, :] = dt * x[t, h, :]: what a recurrence with
    one decay per head and token reads.  z [T, heads], x and v [T, heads * dv], decay [T, heads]; all 32-bit."""
    for t, name in ((z, "z"), (x, "x"), (decay, "decay"), (v, "v")):
        _dev(t, name, (torch.float32,), 2)
    T, n = x.shape
    _need(n % n_heads == 0 and z.shape == (T, n_heads) and decay.shape == (T, n_heads) and v.shape == (T, n), "step_sizes: shapes")
    _f32vec(bias, "bias", n_heads), _f32vec(rate, "rate", n_heads)
    _ok(_lib("sequence").dn_step_sizes(z.data_ptr(), _rows(z, "z"), _ptr(bias), rate.data_ptr(), x.data_ptr(), _rows(x, "x"), T, n_heads,
                                       n // n_heads, decay.data_ptr(), _rows(decay, "decay"), v.data_ptr(), _rows(v, "v"), _stream()),
        "step_sizes")
    return decay, v


def gate_scan(a, b, g, bias_a, bias_b, state, row_start, slots, out):
    """A recurrence of single numbers over each request's rows in order: z = sigmoid(a + bias_a); u = b + bias_b;
    c = u + 1/2 where u >= 0, sigmoid(u) below; S <- (1 - z) S + z c; out = S * silu(g).  a, b, g: 32-bit [T, width] (columns of
    wider rows); state: 32-bit [slots, width]; out [T, width]."""
    for t, name in ((a, "a"), (b, "b"), (g, "g")):
        _dev(t, name, (torch.float32,), 2)
    _dev(out, "out", _FLOATS, 2)
    T, width = a.shape
    S = _request_tables(row_start, slots, "gate_scan")
    _need(b.shape == (T, width) and g.shape == (T, width) and out.shape == (T, width), "gate_scan: shapes")
    _f32vec(bias_a, "bias_a", width), _f32vec(bias_b, "bias_b", width)
    stride = _history(state, width, "gate_scan")
    _ok(_lib("sequence").dn_gate_scan(a.data_ptr(), _rows(a, "a"), b.data_ptr(), _rows(b, "b"), g.data_ptr(), _rows(g, "g"), _ptr(bias_a),
                                      _ptr(bias_b), state.data_ptr(), stride, row_start.data_ptr(), slots.data_ptr(), S, T, width,
                                      out.data_ptr(), _CODE[out.dtype], _rows(out, "out"), _stream()), "gate_scan")
    return out


def head_gate(o, gate, n_heads, dv, out, head_stride=None):
    """out[t, h * dv + d] = o[t, h * head_stride + d] * sigmoid(gate[t, h]) for d < dv: a gate per head on heads that may be
    padded to head_stride columns (None: dv).  gate: 32-bit [T, n_heads] (columns of wider rows)."""
    _dev(o, "o", _FLOATS, 2), _dev(gate, "gate", (torch.float32,), 2), _dev(out, "out", _FLOATS, 2)
    T = o.shape[0]
    hs = dv if head_stride is None else head_stride
    _need(hs >= dv >= 1 and n_heads >= 1 and o.shape[1] >= (n_heads - 1) * hs + dv and tuple(gate.shape) == (T, n_heads)
          and tuple(out.shape) == (T, n_heads * dv), "head_gate: shapes")
    _ok(_lib("sequence").dn_head_gate(o.data_ptr(), _CODE[o.dtype], _rows(o, "o"), hs, gate.data_ptr(), _rows(gate, "gate"),
                                      out.data_ptr(), _CODE[out.dtype], _rows(out, "out"), T, n_heads, dv, _stream()), "head_gate")
    return out


def rows_times_table(a, table, ids, off, out):
    """out[t, c] = a[t, c] * table[ids[t], off + c] for the columns of a: rows of a table picked by an index per row."""
    _dev(a, "a", _FLOATS, 2), _dev(table, "table", _FLOATS, 2), _dev(ids, "ids", _I32, 1), _dev(out, "out", _FLOATS, 2)
    T, n = a.shape
    _need(tuple(out.shape) == (T, n) and ids.is_contiguous() and ids.shape[0] == T and off >= 0 and off + n <= table.shape[1],
          "rows_times_table: shapes")
    _ok(_lib("sequence").dn_rows_times_table(a.data_ptr(), _CODE[a.dtype], _rows(a, "a"), table.data_ptr(), _CODE[table.dtype],
                                             _rows(table, "table"), off, ids.data_ptr(), table.shape[0], out.data_ptr(),
                                             _CODE[out.dtype], _rows(out, "out"), T, n, _stream()), "rows_times_table")
    return out


TOKEN_INPUT_ROWS_MAX = 64      # steps of more rows make a token input from matrix products


def token_input(x, w_gate, w_proj, table, ids, off, weight, eps, then=None):
    """x[t, :] += y / sqrt(mean(y^2) + eps) * weight with y = w_proj (gelu_tanh(w_gate x[t, :]) * table[ids[t], off : off + dim]),
    one launch for steps of few rows.  x: 32-bit rows, changed in place; w_gate [dim, width] and w_proj [width, dim] in rows,
    both 32-bit or both bfloat16; weight: 32-bit [width] or None; sums in 32-bit.  then: as in `rmsnorm_add`: the norm that reads
    the stream next, in the same launch."""
    _dev(x, "x", (torch.float32,), 2), _dev(w_gate, "w_gate", _FLOATS, 2), _dev(w_proj, "w_proj", (w_gate.dtype,), 2)
    _dev(table, "table", _FLOATS, 2), _dev(ids, "ids", _I32, 1)
    T, width = x.shape
    dim = w_gate.shape[0]
    _need(tuple(w_gate.shape) == (dim, width) and tuple(w_proj.shape) == (width, dim) and w_gate.is_contiguous() and w_proj.is_contiguous()
          and ids.is_contiguous() and ids.shape[0] == T and off >= 0 and off + dim <= table.shape[1], "token_input: shapes")
    _need((2 * width + dim) * 4 <= 60000, lambda: f"token_input: a row of {width} and {dim} columns does not fit the workgroup's memory")
    _f32vec(weight, "weight", width)
    _ok(_lib("sequence").dn_token_input(x.data_ptr(), _rows(x, "x"), w_gate.data_ptr(), w_proj.data_ptr(), _CODE[w_gate.dtype], table.data_ptr(),
                                        _CODE[table.dtype], _rows(table, "table"), off, ids.data_ptr(), table.shape[0], _ptr(weight), T, width,
                                        dim, float(eps), *_then(then, T, width, "token_input"), _stream()), "token_input")
    return x


def selective_scan(x, dt, dt_bias, B, C, A, D, z, state, row_start, slots, out, in_order=False):
    """A state per channel c and state index n with a decay of its own, over each request's rows in order:
      step = log(1 + e^(dt[t, c] + dt_bias[c]));  S[c, n] <- exp(step * A[c, n]) S[c, n] + step * x[t, c] * B[t, n]
      y[t, c] = sum_n S[c, n] C[t, n] + D[c] x[t, c];  out[t, c] = y * silu(z[t, c])      (z None: y as it is)
    x [T, inner]: 32-bit or bfloat16 (what a convolution and its activation left); dt, z: 32-bit [T, inner]; B, C: 32-bit
    [T, N] (all may be columns of wider rows); A: 32-bit [inner, N]; dt_bias, D:
    32-bit [inner] or None; state: 32-bit [slots, inner * N], read and written at the requests' slots; out [T, inner].
    in_order: every request's rows are walked one after the other, which gives the same bits however a prompt is cut; else
    long portions of few requests are shared out among a workgroup's waves and joined, which changes a result by rounding."""
    _dev(x, "x", _FLOATS, 2)
    for t, name in ((dt, "dt"), (B, "B"), (C, "C")) + (((z, "z"),) if z is not None else ()):
        _dev(t, name, (torch.float32,), 2)
    _dev(out, "out", _FLOATS, 2), _dev(A, "A", (torch.float32,), 2)
    T, inner = x.shape
    N = B.shape[1]
    S = _request_tables(row_start, slots, "selective_scan")
    _need(tuple(dt.shape) == (T, inner) and tuple(B.shape) == (T, N) and tuple(C.shape) == (T, N) and tuple(out.shape) == (T, inner)
          and (z is None or tuple(z.shape) == (T, inner)) and tuple(A.shape) == (inner, N) and A.is_contiguous(), "selective_scan: shapes")
    _need(1 <= N <= 256, lambda: f"selective_scan: {N} states a channel; the kernel keeps up to 256 on a channel's lanes")
    _f32vec(dt_bias, "dt_bias", inner), _f32vec(D, "D", inner)
    stride = _history(state, inner * N, "selective_scan")
    _ok(_lib("sequence").dn_selective_scan(x.data_ptr(), _CODE[x.dtype], _rows(x, "x"), dt.data_ptr(), _rows(dt, "dt"), _ptr(dt_bias), B.data_ptr(),
                                           _rows(B, "B"), C.data_ptr(), _rows(C, "C"), A.data_ptr(), _ptr(D), _ptr(z),
                                           _rows(z, "z") if z is not None else 0, state.data_ptr(), stride, row_start.data_ptr(),
                                           slots.data_ptr(), S, T, inner, N, out.data_ptr(), _CODE[out.dtype], _rows(out, "out"),
                                           int(bool(in_order)), _stream()), "selective_scan")
    return out


STREAMS_MAX = 8


def _streams(xs, what):
    _dev(xs, "xs", (torch.float32,), 3)
    n, T, width = xs.shape
    _need(xs.is_contiguous() and 1 <= n <= STREAMS_MAX, lambda: f"{what}: 1 to {STREAMS_MAX} copies of the stream, contiguous")
    return n, T, width


def streams_read(xs, w_in, weight, eps, out, rows=None):
    """xs: the stream as n copies, 32-bit [n, T, width].  u = sum_s w_in[s] xs[s] (w_in None: the plain sum); out[r] =
    u[rows[r]] / sqrt(mean(u^2) + eps) * weight (weight: a number per column or None; eps None: no norm, u itself)."""
    n, T, width = _streams(xs, "streams_read")
    _dev(out, "out", _FLOATS, 2)
    _f32vec(w_in, "w_in", n), _f32vec(weight, "weight", width)
    R = out.shape[0]
    if rows is not None:
        _dev(rows, "rows", _I32, 1)
        _need(rows.is_contiguous() and rows.shape[0] == R, "streams_read: rows")
    else:
        _need(R == T, "streams_read: out rows")
    _need(out.shape[1] == width, "streams_read: out")
    _ok(_lib("sequence").dn_streams_read(xs.data_ptr(), T * width, n, _ptr(w_in), _ptr(weight), -1.0 if eps is None else float(eps),
                                         out.data_ptr(), _CODE[out.dtype], _rows(out, "out"), _ptr(rows), R, width, _stream()),
        "streams_read")
    return out


def streams_write(xs, y, mix, w_out, next_in=None, weight=None, eps=0.0, out=None, branches=None):
    """Every copy anew from the old ones and a sublayer's result: xs[t] <- sum_s mix[s, t] xs[s] + w_out[t] * y, in place.
    next_in given: the same kernel then reads the new copies as streams_read(xs, next_in, weight, eps, out) does.
    branches = (y2, w1, w2, eps): the result is the mean of two branches, each normed over the width first with a weight of its
    own: (y / rms(y) * w1 + y2 / rms(y2) * w2) / 2, as two calls of rmsnorm_add with mult 1/2 into zeros make it."""
    n, T, width = _streams(xs, "streams_write")
    _dev(y, "y", (torch.float32,), 2)
    _need(tuple(y.shape) == (T, width), "streams_write: y")
    _f32vec(mix, "mix", n * n), _f32vec(w_out, "w_out", n), _f32vec(next_in, "next_in", n), _f32vec(weight, "weight", width)
    y2 = w1 = w2 = None
    beps = 0.0
    if branches is not None:
        y2, w1, w2, beps = branches
        _dev(y2, "y2", (torch.float32,), 2)
        _need(tuple(y2.shape) == (T, width), "streams_write: the second branch")
        _f32vec(w1, "w1", width), _f32vec(w2, "w2", width)
    if next_in is not None:
        _dev(out, "out", _FLOATS, 2)
        _need(tuple(out.shape) == (T, width), "streams_write: out")
    _ok(_lib("sequence").dn_streams_write(xs.data_ptr(), T * width, n, mix.data_ptr(), w_out.data_ptr(), y.data_ptr(), _rows(y, "y"),
                                          _ptr(y2), _rows(y2, "y2") if y2 is not None else 0, _ptr(w1), _ptr(w2), float(beps),
                                          _ptr(next_in), _ptr(weight), float(eps), _ptr(out) if next_in is not None else 0,
                                          _CODE[out.dtype] if next_in is not None else 0,
                                          _rows(out, "out") if next_in is not None else 0, T, width, _stream()), "streams_write")
    return out


def norm_pair_write(z, q_width, wq, wk, eps, q_out, slot_map, k_pool, v_pool, write=True):
    """A row of z (32-bit) is [q: q_width | k: the rest].  q_out = q / sqrt(mean(q^2) + eps) * wq; the key that goes to the cache
    (k_pool [pages, Hkv, page, dh]) is k / sqrt(mean(k^2) + eps) * wk, each normed as one vector over all heads; the value
    (v_pool [pages, Hkv, dh, page]) is k as it is.  slot_map: int32 [T], page * page_size + offset, negative: not written."""
    _dev(z, "z", (torch.float32,), 2), _dev(q_out, "q_out", _FLOATS, 2), _dev(slot_map, "slot_map", _I32, 1)
    _dev(k_pool, "k_pool", (q_out.dtype,), 4), _dev(v_pool, "v_pool", (q_out.dtype,), 4)
    T = z.shape[0]
    n_pages, Hkv, ps, dh = k_pool.shape
    kw = z.shape[1] - q_width
    _need(kw == Hkv * dh and q_width >= 1 and tuple(q_out.shape) == (T, q_width) and slot_map.is_contiguous() and slot_map.shape[0] == T,
          "norm_pair_write: shapes")
    _need(k_pool.is_contiguous() and v_pool.is_contiguous() and tuple(v_pool.shape) == (n_pages, Hkv, dh, ps), "norm_pair_write: pools")
    _f32vec(wq, "wq", q_width), _f32vec(wk, "wk", kw)
    _ok(_lib("sequence").dn_norm_pair_write(z.data_ptr(), _rows(z, "z"), q_width, kw, wq.data_ptr(), wk.data_ptr(), float(eps),
                                            q_out.data_ptr(), _rows(q_out, "q_out"), slot_map.data_ptr(), k_pool.data_ptr(),
                                            v_pool.data_ptr(), T, Hkv, dh, ps, _CODE[q_out.dtype], int(bool(write)), _stream()),
        "norm_pair_write")
    return q_out


# -- a matrix per head, a matrix per expert (csrc/kernels/grouped.hip) -----------------------------------------------------
def heads_linear(a, w, out, a_off=0, a_stride=None, o_off=0, o_stride=None):
    """out[t, o_off + h * o_stride + n] = sum_k w[h, n, k] * a[t, a_off + h * a_stride + k]; w [heads, N, K]; 32-bit sums."""
    _dev(a, "a", _FLOATS, 2), _dev(w, "w", _FLOATS, 3), _dev(out, "out", _FLOATS, 2)
    H, N, K = w.shape
    T = a.shape[0]
    a_stride = K if a_stride is None else a_stride
    o_stride = N if o_stride is None else o_stride
    _need(w.is_contiguous() and out.shape[0] == T, "heads_linear: shapes")
    _need(a_off >= 0 and a_off + (H - 1) * a_stride + K <= a.shape[1] and o_off >= 0 and o_off + (H - 1) * o_stride + N <= out.shape[1],
          "heads_linear: heads outside their rows")
    _ok(_lib("grouped").dn_heads_linear(a.data_ptr(), _CODE[a.dtype], _rows(a, "a"), a_off, a_stride, w.data_ptr(), _CODE[w.dtype],
                                        out.data_ptr(), _CODE[out.dtype], _rows(out, "out"), o_off, o_stride, T, H, N, K, _stream()),
        "heads_linear")
    return out


def moe_route(z, correction, top, ids, wts, score="softmax", renorm=True, n_experts=None, groups=1, keep=1, scale=1.0):
    """Per row: s = softmax(z) over the experts, or (score "sigmoid") each expert's own 1 / (1 + e^-z); the `top` experts with
    the largest s + correction (the lower index wins a tie) go to ids [T, top]; wts [T, top] gets their s divided by the sum
    of the chosen s (+ 1e-20), or (renorm False) their s as it is, times `scale`.  n_experts: the first columns of z that are
    experts (None: all of them).  groups > 1: the experts are that many equal runs of neighbours, a group's score is the sum
    of its two largest s + correction, and only experts of the `keep` best groups can be chosen."""
    _dev(z, "z", (torch.float32,), 2), _dev(ids, "ids", _I32, 2), _dev(wts, "wts", (torch.float32,), 2)
    T = z.shape[0]
    E = z.shape[1] if n_experts is None else n_experts
    _need(ids.is_contiguous() and wts.is_contiguous() and tuple(ids.shape) == (T, top) and E <= z.shape[1]
          and tuple(wts.shape) == (T, top) and 1 <= top <= E and score in ("softmax", "sigmoid"), "moe_route: shapes")
    _need(groups >= 1 and E % groups == 0 and 1 <= keep <= groups and top <= keep * (E // groups),
          lambda: f"moe_route: {E} experts in {groups} groups of which {keep} are kept, for {top} choices")
    _f32vec(correction, "correction", E)
    _ok(_lib("grouped").dn_moe_route(z.data_ptr(), _rows(z, "z"), _ptr(correction), T, E, top, int(score == "sigmoid"),
                                     int(bool(renorm)), ids.data_ptr(), wts.data_ptr(), int(groups), int(keep), float(scale),
                                     _stream()), "moe_route")


def moe_plan(ids, n_experts, offsets, order):
    """The pairs (row, choice), pair i = row * top + choice, sorted by expert and then by i: order [T * top]; expert e has
    the places offsets[e] .. offsets[e + 1] - 1 (offsets [experts + 1])."""
    _dev(ids, "ids", _I32, 2), _dev(offsets, "offsets", _I32, 1), _dev(order, "order", _I32, 1)
    n = ids.numel()
    _need(ids.is_contiguous() and offsets.shape[0] == n_experts + 1 and order.shape[0] == n and offsets.is_contiguous()
          and order.is_contiguous(), "moe_plan: shapes")
    _ok(_lib("grouped").dn_moe_plan(ids.data_ptr(), n, n_experts, offsets.data_ptr(), order.data_ptr(), _stream()), "moe_plan")


def experts_packable(n_experts, rows, inner):
    """Whether stacked expert matrices [experts * rows, inner] can be held packed for the matrix cores (pack_matrix on
    the stack): an expert's rows start at a block of 16, the inner size is whole steps of 32."""
    return rows % 16 == 0 and inner % 32 == 0


def moe_up(h, order, offsets, top, w_gate, w_up, limit, alpha, y, dims=None, kind="clamped", in_scale=None):
    """For place p of expert e, the row t = order[p] // top: kind "clamped": g = min(w_gate[e] h[t], limit), u = clamp(w_up[e]
    h[t], -limit, limit), y[p] = g * sigmoid(alpha * g) * (u + 1); kind "silu": the expert reads s h[t] with s =
    in_scale[order[p]] (32-bit [T * top]; None: 1), y[p] = silu(w_gate[e] s h[t]) * (w_up[e] s h[t]), the factor applied to
    the 32-bit sums; kind "relu2": an expert without a gate (w_gate None), y[p] = max(w_up[e] s h[t], 0)^2.
    w_gate, w_up: [experts, ff, width]; y [T * top, ff].
    dims = (experts, ff, width): w_gate and w_up are PackedMatrix of the stacked [experts * ff, width] (experts_packable)."""
    _dev(h, "h", _FLOATS, 2), _dev(y, "y", _FLOATS, 2)
    n = order.shape[0]
    _need(kind in ("clamped", "silu", "relu2") and (w_gate is None) == (kind == "relu2"), "moe_up: kind, or a gate that it does not have")
    if dims is not None:
        E, ff, width = dims
        _need(all(w is None or (isinstance(w, PackedMatrix) and tuple(w.shape) == (E * ff, width)) for w in (w_gate, w_up))
              and experts_packable(E, ff, width), "moe_up: packed weights")
        wdt = torch.bfloat16
    else:
        _dev(w_up, "w_up", _FLOATS, 3)
        E, ff, width = w_up.shape
        _need(w_up.is_contiguous(), "moe_up: weights")
        if w_gate is not None:
            _dev(w_gate, "w_gate", (w_up.dtype,), 3)
            _need(w_gate.is_contiguous() and tuple(w_gate.shape) == (E, ff, width), "moe_up: weights")
        wdt = w_up.dtype
    _need(h.shape[1] == width and y.is_contiguous() and tuple(y.shape) == (n, ff) and offsets.shape[0] == E + 1
          and n == h.shape[0] * top, "moe_up: shapes")
    if in_scale is not None:
        _dev(in_scale, "in_scale", (torch.float32,))
        _need(in_scale.is_contiguous() and in_scale.numel() == n and kind != "clamped", "moe_up: in_scale")
    _ok(_lib("grouped").dn_moe_up(h.data_ptr(), _CODE[h.dtype], _rows(h, "h"), order.data_ptr(), offsets.data_ptr(), E, top, n,
                                  w_gate.data_ptr() if w_gate is not None else 0, w_up.data_ptr(), _CODE[wdt], ff, width, float(limit),
                                  float(alpha), {"clamped": 0, "silu": 1, "relu2": 2}[kind], _ptr(in_scale), y.data_ptr(),
                                  _CODE[y.dtype], int(dims is not None), _stream()), "moe_up")


def moe_down(y, order, offsets, w_down, out, dims=None):
    """out[order[p], :] = w_down[e] y[p, :] for the places p of expert e; w_down [experts, width, ff]; out 32-bit [T * top, width].
    dims = (experts, width, ff): w_down is a PackedMatrix of the stacked [experts * width, ff]."""
    _dev(y, "y", _FLOATS, 2), _dev(out, "out", (torch.float32,), 2)
    n = order.shape[0]
    if dims is not None:
        E, width, ff = dims
        _need(isinstance(w_down, PackedMatrix) and tuple(w_down.shape) == (E * width, ff) and experts_packable(E, width, ff),
              "moe_down: packed weights")
        wdt = torch.bfloat16
    else:
        _dev(w_down, "w_down", _FLOATS, 3)
        E, width, ff = w_down.shape
        _need(w_down.is_contiguous(), "moe_down: weights")
        wdt = w_down.dtype
    _need(y.is_contiguous() and tuple(y.shape) == (n, ff) and out.is_contiguous() and tuple(out.shape) == (n, width)
          and offsets.shape[0] == E + 1, "moe_down: shapes")
    _ok(_lib("grouped").dn_moe_down(y.data_ptr(), _CODE[y.dtype], order.data_ptr(), offsets.data_ptr(), E, n, w_down.data_ptr(),
                                    _CODE[wdt], width, ff, out.data_ptr(), int(dims is not None), _stream()), "moe_down")


def moe_combine(out, wts, x, logits=False):
    """x[t, :] += sum_c wts[t, c] * out[t * top + c, :], the choices in their order (wts None: every weight is 1; logits: a
    weight is 1 / (1 + e^-z) of what wts holds; wts may be columns of wider rows)."""
    _dev(out, "out", (torch.float32,), 2), _dev(x, "x", (torch.float32,), 2)
    T, width = x.shape
    top = out.shape[0] // max(T, 1) if wts is None else wts.shape[1]
    if wts is not None:
        _dev(wts, "wts", (torch.float32,), 2)
        _need(wts.shape[0] == T and not (logits and wts is None), "moe_combine: weights")
    _need(out.is_contiguous() and tuple(out.shape) == (T * top, width), "moe_combine: shapes")
    _ok(_lib("grouped").dn_moe_combine(out.data_ptr(), _ptr(wts), _rows(wts, "wts") if wts is not None else 0, int(bool(logits)), T, top,
                                       width, x.data_ptr(), _rows(x, "x"), _stream()),
        "moe_combine")
