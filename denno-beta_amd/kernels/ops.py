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
EPILOGUES = {"none": 0, "gelu_tanh": 1, "gelu_erf": 2}

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
            "dn_attention_flash": [P, I, P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, F, I, P],
            "dn_attention_decode": [P, I, P, I, P, P, P, I, P, P, P, I, P, I, I, I, I, I, I, I, F, I, P],
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
              single_rows=False, max_context=0, decode_waves=None):
    """Causal attention of the batch's rows over the paged cache.

    q: [T, >= H*dh] rows contiguous, head h at columns h*dh..; out: [T, H*dh];
    k_pool: [n_pages, Hkv, page_size, dh]; v_pool: [n_pages, Hkv, dh, page_size];
    block_tables: int32 [S, max_blocks];
    tiles: int32 [4, n_tiles] = (request, first row, rows <= 16, first position), request < 0: padding;
    tiles_wide: the same rows cut into tiles of up to 128 rows;
    single_rows: a pure decode step: request s brings row s and is tile s, (s or -1, s, 1, position);
    max_context: the longest context then.

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
    lib = _lib("attention")
    # (the kernel for portions takes the largest score for the largest product: a scale that is not positive goes the plain way)
    fast = q.dtype == torch.bfloat16 and ps % 16 == 0 and ldq % 8 == 0 and q.data_ptr() % 16 == 0 and scale > 0
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
        _ok(lib.dn_attention_decode(
            q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], base, base + 4 * n_tiles, base + 12 * n_tiles, n_tiles, part.data_ptr(), n_splits,
            chunks, waves, n_heads, Hkv, dh, ps, float(scale), int(window), _stream()), "attention (decode)")
        return out
    if fast and tiles_wide is not None and dh in FLASH_HEAD_DIMS:
        _dev(tiles_wide, "tiles_wide", _I32, 2)
        _need(tiles_wide.is_contiguous() and tiles_wide.shape[0] == 4, "attention: tiles_wide")
        n_tiles = tiles_wide.shape[1]
        base = tiles_wide.data_ptr()
        _ok(lib.dn_attention_flash(
            q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], base, base + 4 * n_tiles, base + 8 * n_tiles, base + 12 * n_tiles, n_tiles,
            n_heads, Hkv, dh, ps, float(scale), int(window), _stream()), "attention (flash)")
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
        _ok(lib.dn_attention_rows(
            q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], base, base + 12 * n_tiles, n_tiles, part.data_ptr(), int(max_context), n_heads, Hkv,
            dh, ps, float(scale), int(window), _CODE[q.dtype], _stream()), "attention (single rows)")
        return out
    _ok(lib.dn_attention(
        q.data_ptr(), ldq, out.data_ptr(), ldo, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], base, base + 4 * n_tiles, base + 8 * n_tiles, base + 12 * n_tiles, n_tiles,
        n_heads, Hkv, dh, ps, float(scale), int(window), _CODE[q.dtype], _stream()), "attention")
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
