"""The op table: every operation of the engine bound to exactly one HIP kernel.

Each function checks on the host that its operands have the device, element
type, contiguity and shape the kernel assumes (a kernel is never launched on
operands it cannot address), allocates the result with torch's allocator and
launches on torch's current stream.  There is no CPU path and no library
fallback: without the compiled library every call raises.

The reference binds ops to kernels by name in its FunctionFactory
(include/FunctionFactory.h:18-116, kernel/include/TFFOPCreatorBase.h:73-97)
with a device dispatch; here the table has one entry per op and no dispatch.
"""
from __future__ import annotations

import ctypes
import math

import numpy as np
import torch

from . import lib as _lib
from .key_runs import deal_key_runs
from . import staging as _staging

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise _lib.KernelError(f"element type {dt} is not supported (float32 or bfloat16)") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle.  Asked for at every launch (hundreds a step when a step is
    launched kernel by kernel): through torch's C binding where there is one, which costs a
    tenth of building a Stream object."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _req(t: torch.Tensor, name: str, dtype=None, ndim=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise _lib.KernelError(f"{name}: expected a tensor on the GPU")
    if not t.is_contiguous():
        raise _lib.KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise _lib.KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise _lib.KernelError(f"{name}: expected {ndim} dimensions, got shape {tuple(t.shape)}")
    return t


def _check_cache(k_cache, v_cache, nkv, d, what):
    """Keys [pages, nkv, page_size, d]; values transposed [pages, nkv, d, page_size]."""
    pages, h, ps, dd = k_cache.shape
    if h != nkv or dd != d or tuple(v_cache.shape) != (pages, nkv, d, ps) or v_cache.dtype != k_cache.dtype:
        raise _lib.KernelError(
            f"{what}: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} are not keys "
            f"[pages, {nkv}, page_size, {d}] and values [pages, {nkv}, {d}, page_size]")


def _ptr(t):
    return None if t is None else t.data_ptr()


class PackedWeight:
    """A bfloat16 matrix [N, K] in the fragment order of the matrix-core
    products: tiles of 16 rows by 32 k stored as the 1 KB operand a wave loads,
    rows and k padded with zeros to multiples of 16 and 32."""
    __slots__ = ("data", "N", "K", "glu_out", "k_in")

    def __init__(self, data: torch.Tensor, N: int, K: int, glu_out: int = 0, k_in: int | None = None):
        self.data, self.N, self.K = data, int(N), int(K)
        #: the inner size of the matrix it was packed from, where that was no multiple of 8 (K is
        #: the next one, the columns between are zeros; ``linear`` widens its rows to match)
        self.k_in = int(k_in) if k_in is not None else int(K)
        #: > 0: the 16-row groups alternate between a gate and an up projection and the
        #: product yields silu(gate) * up with this many columns
        self.glu_out = int(glu_out)

    @property
    def shape(self):
        return (self.N, self.K)

    @property
    def out_features(self) -> int:
        return self.glu_out or self.N

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def unpack(self) -> torch.Tensor:
        """Back to row-major [N, K] (for tests and inspection)."""
        NB, KB = -(-self.N // 16), -(-self.K // 32)
        t = self.data.view(NB, KB, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(NB * 16, KB * 32)
        return t[:self.N, :self.K].contiguous()


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """Row-major bfloat16 [N, K] on the GPU -> fragment order."""
    _req(w, "pack_weight", torch.bfloat16, 2)
    N, k_in = w.shape
    if k_in % 8:
        # (the products take inner sizes in units of 8: zero columns change no sum)
        w = torch.nn.functional.pad(w, (0, 8 - k_in % 8)).contiguous()
    N, K = w.shape
    NB, KB = -(-N // 16), -(-K // 32)
    out = torch.empty(NB * KB * 512, dtype=torch.bfloat16, device=w.device)
    L = _lib.load()
    _lib.check(L.tff_pack_weight(w.data_ptr(), out.data_ptr(), N, K, _stream()))
    return PackedWeight(out, N, K, k_in=k_in)


def pack_gate_up(gate: torch.Tensor, up: torch.Tensor) -> PackedWeight:
    """Gate and up projections [I, K] (bfloat16, on the GPU) as one weight whose
    16-row groups alternate gate, up, gate, up, ..., in fragment order.  A
    product with it yields silu(x gate^T) * (x up^T) directly: the activation
    runs in the product's epilogue, on the float32 accumulators."""
    _req(gate, "gate", torch.bfloat16, 2)
    _req(up, "up", torch.bfloat16, 2)
    if gate.shape != up.shape:
        raise _lib.KernelError(f"pack_gate_up: gate {tuple(gate.shape)} and up {tuple(up.shape)} differ")
    I, K = gate.shape
    groups = -(-I // 16)
    padded = torch.zeros(2, groups * 16, K, dtype=torch.bfloat16, device=gate.device)
    padded[0, :I] = gate
    padded[1, :I] = up
    both = padded.view(2, groups, 16, K).permute(1, 0, 2, 3).reshape(groups * 32, K).contiguous()
    pw = pack_weight(both)
    pw.glu_out = I
    return pw


def embed(table, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """Rows of ``table`` [V, H] (a row-major tensor or a PackedWeight) for
    int32 ``ids`` [T] as float32 [T, H]."""
    packed = isinstance(table, PackedWeight)
    if packed:
        _req(table.data, "embed table", torch.bfloat16, 1)
    else:
        _req(table, "embed table", ndim=2)
    _req(ids, "embed ids", torch.int32, 1)
    V, H = table.shape
    T = ids.numel()
    if packed and table.k_in != H:
        # (a table whose rows were widened to a multiple of 8: the rows come out as wide, and are cut)
        wide = torch.empty(T, H, dtype=torch.float32, device=table.device)
        _lib.check(_lib.load().tff_embed_packed(table.data_ptr(), ids.data_ptr(), wide.data_ptr(), T, H, V, _stream()))
        cut = wide[:, :table.k_in].contiguous()
        if out is not None:
            out.copy_(cut)
            return out
        return cut
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    else:
        _req(out, "embed out", torch.float32, 2)
        if tuple(out.shape) != (T, H):
            raise _lib.KernelError(f"embed out: shape {tuple(out.shape)} is not {(T, H)}")
    L = _lib.load()
    if packed:
        _lib.check(L.tff_embed_packed(table.data_ptr(), ids.data_ptr(), out.data_ptr(), T, H, V, _stream()))
    else:
        _lib.check(L.tff_embed(table.data_ptr(), ids.data_ptr(), out.data_ptr(), T, H, V,
                               dtype_code(table.dtype), _stream()))
    return out


class PendingProduct:
    """A product ``x . weight^T`` of up to 16 bfloat16 rows that ``linear`` was
    asked for with ``partials=True`` and has not run: ``add_rmsnorm`` runs it
    with the residual sum and the norm's weight in its epilogue when the norm's
    result goes to another such product, and plainly (:meth:`run`) otherwise."""

    def __init__(self, x: torch.Tensor, weight: "PackedWeight"):
        self.x, self.weight = x, weight
        self.shape = (x.shape[0], weight.shape[0])
        self.device = x.device

    def run(self) -> torch.Tensor:
        return linear(self.x, self.weight, out_dtype=torch.float32)


class ScaledRows:
    """The result of an RMS norm whose per-row factor has not been applied:
    ``x`` [M, H] bfloat16 = (residual stream) * (norm weight), and the sums of
    squares of every row's groups of 16 columns, ``ss`` [16, stride] float32
    (``count`` of them a row).  ``linear`` applies rsqrt(sum / H + eps) to its
    accumulators; :meth:`materialize` writes the normalised rows out, from the
    float32 residual stream ``resid`` (which must still hold the sum the norm
    was taken of) and the norm's ``weight``, so that they are rounded to
    bfloat16 once, as the norm's own kernel rounds them."""

    def __init__(self, x: torch.Tensor, ss: torch.Tensor, count: int, eps: float,
                 resid: torch.Tensor, weight: torch.Tensor):
        self.x, self.ss, self.count, self.eps = x, ss, int(count), float(eps)
        self.resid, self.weight = resid, weight
        self.shape, self.dtype, self.device = x.shape, x.dtype, x.device

    def materialize(self) -> torch.Tensor:
        return add_rmsnorm(self.resid, None, self.weight, self.eps, self.x.dtype)


def _as_tensor_terms(t) -> torch.Tensor:
    parts = [as_tensor(x) for x in t.terms]
    return parts[0] if len(parts) == 1 else parts[0] + parts[1]


def as_tensor(t) -> torch.Tensor:
    """Whatever ``linear`` or ``add_rmsnorm`` returned, as a plain tensor: a
    product that has not run is run, partial sums [S, T, H] are added up in
    order, rows that lack their norm's factor get it."""
    if isinstance(t, PendingProduct):
        return t.run()
    if isinstance(t, ScaledRows):
        return t.materialize()
    if isinstance(t, PendingTerms):
        return _as_tensor_terms(t)
    if isinstance(t, torch.Tensor) and t.dim() == 3:
        acc = t[0].clone()
        for part in t[1:]:
            acc += part
        return acc
    return t


def _fused_prenorm(p: PendingProduct, resid: torch.Tensor, weight: torch.Tensor, eps: float) -> ScaledRows:
    x = p.x
    M, K = x.shape
    N = p.weight.shape[0]
    lda = x.stride(0) if M > 1 else K
    groups = -(-N // 16)
    stride = -(-groups // 4) * 4
    xs = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    ss = torch.empty(16, stride, dtype=torch.float32, device=x.device)
    L = _lib.load()
    _lib.check(L.tff_gemm_residual_prenorm(x.data_ptr(), p.weight.data_ptr(), M, N, K, lda, resid.data_ptr(),
                                           weight.data_ptr(), xs.data_ptr(), ss.data_ptr(), stride, _stream()))
    return ScaledRows(xs, ss, groups, eps, resid, weight)


def add_rmsnorm(resid: torch.Tensor, delta, weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None,
                out: torch.Tensor | None = None, for_linear: bool = False):
    """``resid += delta`` (when given and ``rows`` is None) and the RMS norm of
    the sum; with ``rows`` the norm of those rows only, ``resid`` untouched.
    ``delta`` may be what ``linear`` returns with ``partials=True``: a stack
    [S, T, H] of partial sums, which are added up first, in order, or a
    product that has not run.  ``for_linear``: the result goes to ``linear``
    and nowhere else, so it may be a :class:`ScaledRows`."""
    if isinstance(delta, PendingTerms):
        if out is not None:
            raise _lib.KernelError("add_rmsnorm: several pending terms and a given result do not go together")
        return add_rmsnorm_pair(resid, delta, None, weight, None, eps, out_dtype, rows=rows)[0]
    _req(resid, "add_rmsnorm resid", torch.float32, 2)
    H = resid.shape[1]
    _req(weight, "add_rmsnorm weight", torch.float32, 1)
    if weight.numel() != H:
        raise _lib.KernelError(f"add_rmsnorm: weight has {weight.numel()} elements, rows have {H}")
    if isinstance(delta, PendingProduct):
        if tuple(delta.shape) != tuple(resid.shape):
            raise _lib.KernelError(
                f"add_rmsnorm: delta {tuple(delta.shape)} does not match resid {tuple(resid.shape)}")
        if for_linear and rows is None and out is None and out_dtype == torch.bfloat16:
            return _fused_prenorm(delta, resid, weight, eps)
        delta = delta.run()
    planes, plane = 1, 0
    if delta is not None:
        _req(delta, "add_rmsnorm delta", torch.float32, 3 if delta.dim() == 3 else 2)
        if tuple(delta.shape[-2:]) != tuple(resid.shape):
            raise _lib.KernelError(
                f"add_rmsnorm: delta {tuple(delta.shape)} does not match resid {tuple(resid.shape)}")
        if delta.dim() == 3:
            planes, plane = delta.shape[0], delta.stride(0)
    if rows is not None:
        _req(rows, "add_rmsnorm rows", torch.int32, 1)
        n = rows.numel()
    else:
        n = resid.shape[0]
    if out is None:
        out = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    else:
        _req(out, "add_rmsnorm out", out_dtype, 2)
        if tuple(out.shape) != (n, H):
            raise _lib.KernelError(f"add_rmsnorm out: shape {tuple(out.shape)} is not {(n, H)}")
    L = _lib.load()
    _lib.check(L.tff_add_rmsnorm(resid.data_ptr(), _ptr(delta), planes, plane, weight.data_ptr(), float(eps),
                                 out.data_ptr(), _ptr(rows), n, H, dtype_code(out_dtype), _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the last dimension of a dense tensor, float32 weight."""
    _req(x, "rmsnorm x")
    H = x.shape[-1]
    _req(weight, "rmsnorm weight", torch.float32, 1)
    if weight.numel() != H:
        raise _lib.KernelError(f"rmsnorm: weight has {weight.numel()} elements, rows have {H}")
    out = torch.empty_like(x)
    L = _lib.load()
    _lib.check(L.tff_rmsnorm(x.data_ptr(), weight.data_ptr(), float(eps), out.data_ptr(),
                             x.numel() // H, H, dtype_code(x.dtype), _stream()))
    return out


_plan_cache: dict = {}


def _plan_tile(L, M: int, N: int, K: int) -> int:
    """Rows of the tile the product's plan takes when partial sums are kept (0: the streaming kernel)."""
    key = (M, N, K)
    if key not in _plan_cache:
        r, c, s = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _lib.check(L.tff_gemm_plan(M, N, K, 0, 1, ctypes.byref(r), ctypes.byref(c), ctypes.byref(s)))
        _plan_cache[key] = r.value
    return _plan_cache[key]


def linear(x: torch.Tensor, weight, out_dtype: torch.dtype | None = None,
           out: torch.Tensor | None = None, partials: bool = False) -> torch.Tensor:
    """``x . weight^T`` for x [M, K] (rows may be strided) and weight [N, K]:
    a row-major float32 tensor, or a PackedWeight for bfloat16.

    ``partials=True`` (float32 result): where the product splits K over
    blocks, the partial sums are returned as they are, [S, M, N], for a
    consumer that adds them up anyway (``add_rmsnorm``); else the result is
    [M, N] as always."""
    packed = isinstance(weight, PackedWeight)
    if isinstance(x, ScaledRows):
        if packed and out is None and not partials and x.shape[1] == weight.shape[1]:
            return _linear_row_scaled(x, weight, out_dtype or x.dtype)
        x = x.materialize()
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise _lib.KernelError("linear x: expected a GPU matrix with unit inner stride")
    if packed:
        _req(weight.data, "linear weight", x.dtype, 1)
    else:
        _req(weight, "linear weight", x.dtype, 2)
        if weight.dtype == torch.bfloat16:
            raise _lib.KernelError("linear: a bfloat16 weight must be a PackedWeight (pack_weight)")
    M, K = x.shape
    N, K2 = weight.shape
    if packed and K != K2 and K == weight.k_in:
        x = torch.nn.functional.pad(x, (0, K2 - K))      # a weight whose inner size was rounded up to 8
        K = K2
    if K != K2:
        raise _lib.KernelError(f"linear: x has inner size {K}, weight [out, in] = {tuple(weight.shape)}")
    lda = x.stride(0) if M > 1 else K
    if lda < K:
        raise _lib.KernelError("linear x: rows overlap")
    out_dtype = out_dtype or x.dtype
    glu_out = weight.glu_out if packed else 0
    n_out = glu_out or N
    L = _lib.load()
    # some shapes (few columns for the rows) split K over blocks and need room for partial sums
    want = bool(partials and packed and out is None and out_dtype == torch.float32 and not glu_out)
    if want and M <= 16 and N % 8 == 0 and x.dtype == torch.bfloat16 and x.data_ptr() % 16 == 0 and lda % 8 == 0:
        if _plan_tile(L, M, N, K) == 0:
            return PendingProduct(x, weight)   # a few rows: the consumer runs it with its own work in the epilogue
        # (else the streaming kernel's blocks would go badly round the CUs: tiles that split K, partial sums kept)
    ws_bytes = (L.tff_gemm_workspace_bytes(M, N, K, dtype_code(x.dtype), 1 if glu_out else 0, 1 if want else 0)
                if packed else 0)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=x.device) if ws_bytes else None
    keep = want and ws is not None
    if keep:
        out = ws.view(-1, M, N)
    elif out is None:
        out = torch.empty(M, n_out, dtype=out_dtype, device=x.device)
    else:
        _req(out, "linear out", out_dtype, 2)
        if tuple(out.shape) != (M, n_out):
            raise _lib.KernelError(f"linear out: shape {tuple(out.shape)} is not {(M, n_out)}")
    _lib.check(L.tff_gemm(x.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K, lda,
                          dtype_code(x.dtype), dtype_code(out_dtype), 1 if packed else 0, glu_out,
                          _ptr(ws), ws_bytes, 1 if keep else 0, _stream()))
    return out


def _linear_row_scaled(x: ScaledRows, weight: "PackedWeight", out_dtype: torch.dtype) -> torch.Tensor:
    M, K = x.shape
    N = weight.shape[0]
    glu_out = weight.glu_out
    out = torch.empty(M, glu_out or N, dtype=out_dtype, device=x.device)
    L = _lib.load()
    _lib.check(L.tff_gemm_row_scaled(x.x.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K, K,
                                     dtype_code(out_dtype), glu_out, x.ss.data_ptr(), x.ss.stride(0), x.count, K,
                                     x.eps, _stream()))
    return out


def qk_norm_rope_kv(qkv: torch.Tensor, nq: int, nkv: int, d: int,
                    q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float,
                    cos_sin: torch.Tensor | None, pairing: int,
                    positions: torch.Tensor, slot_mapping: torch.Tensor,
                    k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """In place on the fused projection output ``qkv`` [T, (nq + 2 nkv) d]; see
    the entry point's comment.  ``cos_sin`` is [max_pos, rot/2, 2] float32."""
    _req(qkv, "qk_norm_rope_kv qkv", ndim=2)
    T = qkv.shape[0]
    if qkv.shape[1] != (nq + 2 * nkv) * d:
        raise _lib.KernelError(
            f"qk_norm_rope_kv: rows of {qkv.shape[1]} are not (nq + 2 nkv) d = {(nq + 2 * nkv) * d}")
    for w, nm in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if w is not None:
            _req(w, nm, torch.float32, 1)
            if w.numel() != d:
                raise _lib.KernelError(f"{nm}: {w.numel()} elements, head size {d}")
    rot, max_pos = 0, 0
    if cos_sin is not None:
        _req(cos_sin, "rotation table", torch.float32, 3)
        max_pos, half, two = cos_sin.shape
        if two != 2:
            raise _lib.KernelError("rotation table: last dimension must hold (cos, sin)")
        rot = 2 * half
    _req(positions, "positions", torch.int32, 1)
    _req(slot_mapping, "slot_mapping", torch.int32, 1)
    if positions.numel() != T or slot_mapping.numel() != T:
        raise _lib.KernelError("qk_norm_rope_kv: positions and slot_mapping need one entry per token")
    _req(k_cache, "k cache", ndim=4)
    _req(v_cache, "v cache", ndim=4)
    _check_cache(k_cache, v_cache, nkv, d, "qk_norm_rope_kv")
    L = _lib.load()
    _lib.check(L.tff_qk_norm_rope_kv(
        qkv.data_ptr(), T, nq, nkv, d, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin),
        rot, int(pairing), max_pos, positions.data_ptr(), slot_mapping.data_ptr(),
        k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[2], k_cache.shape[0],
        dtype_code(qkv.dtype), dtype_code(k_cache.dtype), _stream()))


def attention_generic(q: torch.Tensor, nq: int, nkv: int, d: int, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, block_tables: torch.Tensor, token_req: torch.Tensor,
                      positions: torch.Tensor, window: int = 0, scale: float | None = None,
                      out: torch.Tensor | None = None, sinks: torch.Tensor | None = None,
                      softcap: float = 0.0) -> torch.Tensor:
    """Attention of each token over its request's pages; q is [T, >= nq*d]
    with the query heads at the start of each row.  Returns [T, nq*d].
    ``sinks`` (float32 [nq]) and ``softcap``: see :func:`paged_attention`."""
    _req(q, "attention q", ndim=2)
    T = q.shape[0]
    if q.shape[1] < nq * d:
        raise _lib.KernelError(f"attention q: rows of {q.shape[1]} hold fewer than nq*d = {nq * d}")
    _req(k_cache, "k cache", q.dtype, 4)
    _req(v_cache, "v cache", q.dtype, 4)
    _check_cache(k_cache, v_cache, nkv, d, "attention")
    _req(block_tables, "block tables", torch.int32, 2)
    _req(token_req, "token_req", torch.int32, 1)
    _req(positions, "positions", torch.int32, 1)
    if token_req.numel() != T or positions.numel() != T:
        raise _lib.KernelError("attention: token_req and positions need one entry per token")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty(T, nq * d, dtype=q.dtype, device=q.device)
    _check_sinks(sinks, nq)
    L = _lib.load()
    _lib.check(L.tff_attention_generic(
        q.data_ptr(), q.stride(0), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        block_tables.data_ptr(), block_tables.stride(0), token_req.data_ptr(), positions.data_ptr(),
        T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale), _ptr(sinks), float(softcap or 0.0),
        dtype_code(q.dtype), dtype_code(k_cache.dtype), _stream()))
    return out


def _check_sinks(sinks, nq: int) -> None:
    if sinks is not None:
        _req(sinks, "attention sinks", torch.float32, 1)
        if sinks.numel() != nq:
            raise _lib.KernelError(f"attention sinks: {sinks.numel()} numbers for {nq} query heads")


def mfma_attention_supported(dtype: torch.dtype, d: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and bool(_lib.load().tff_attention_mfma_supported(int(d), int(page_size)))


def _entries(batch, which: str) -> list[int]:
    """Rows of the step's entries: all, those that bring one token, or the others."""
    cu = batch.host_cu_tokens
    rows = range(len(cu) - 1)
    if which == "all":
        return list(rows)
    one = which == "single"
    return [r for r in rows if (cu[r + 1] - cu[r] == 1) == one]


def _attention_work(batch, G: int, cols: int, device, which: str = "all") -> torch.Tensor:
    """(entry, first column) of every wave's tile for the step's entries; a
    column is a (token, q head of the group) pair numbered token * G + head."""
    cache = getattr(batch, "_attn_work", None)
    if cache is None:
        cache = batch._attn_work = {}
    key = (G, cols, which)
    if key not in cache:
        cu = batch.host_cu_tokens
        flat = []
        for r in _entries(batch, which):
            for c0 in range(0, (cu[r + 1] - cu[r]) * G, cols):
                flat.extend((r, c0))
        cache[key] = _staging.send(device, [np.asarray(flat, dtype=np.int32).reshape(-1, 2)])[0]
    return cache[key]


_cu_count = {}


def _num_cus(device) -> int:
    idx = torch.device(device).index or 0
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def _attention_block_work(batch, G: int, nkv: int, window: int, device, cols: int = 128,
                          bins: int | None = None, which: str = "all", key_groups: int | None = None,
                          head_dim: int = 128, num_cus: int | None = None):
    """Work table of the block kernel: items (entry, first column) of ``cols``
    columns, dealt to blocks so that every block goes through about the same
    number of 32-key slices (an item late in a long prompt sees many times the
    keys of an early one).  There are at most as many blocks as the device
    can hold at once, so none waits for another to end: with little work one
    block a CU whose two groups of waves share an item's slices, with plenty
    (some 96 slices a block and more) two blocks of one group a CU.  Returns
    (items [n, 2], block_items [blocks + 1], blocks, key groups)."""
    cache = getattr(batch, "_attn_work", None)
    if cache is None:
        cache = batch._attn_work = {}
    key = ("blocks", G, nkv, cols, window, bins, which, key_groups, head_dim, num_cus)
    if key not in cache:
        cu, P = batch.host_cu_tokens, batch.host_start_pos
        items = []                       # (slices, entry, first column)
        for r in _entries(batch, which):
            ncols = (cu[r + 1] - cu[r]) * G
            for c0 in range(0, ncols, cols):
                first = P[r] + c0 // G
                last = P[r] + (min(c0 + cols, ncols) - 1) // G
                lo = max(0, first - window + 1) if window > 0 else 0
                items.append((last // 32 - lo // 32 + 1, r, c0))
        if num_cus is None:
            num_cus = _num_cus(device) if torch.device(device).type == "cuda" else 256
        per_cu = max(1, num_cus // max(1, nkv))
        groups = key_groups
        if groups is None:
            groups = 2
            if head_dim <= 128 and sum(it[0] for it in items) >= 96 * 2 * per_cu:
                groups = 1
        if head_dim > 128:
            groups = 1                   # LDS holds one group's stages there
        nbins = bins if bins is not None else (per_cu if groups == 2 or head_dim > 128 else 2 * per_cu)
        if len(items) <= nbins:
            order = sorted(items, reverse=True)        # the longest start first
            starts = list(range(len(order) + 1))
        else:
            # longest first, each to the block with the least to do so far
            import heapq
            loads = [(0, b) for b in range(nbins)]
            heapq.heapify(loads)
            per_bin = [[] for _ in range(nbins)]
            for it in sorted(items, reverse=True):
                load, b = heapq.heappop(loads)
                per_bin[b].append(it)
                heapq.heappush(loads, (load + it[0], b))
            order, starts = [], [0]
            for lst in per_bin:
                order.extend(lst)
                starts.append(len(order))
        flat = [x for it in order for x in it[1:]]
        items_d, starts_d = _staging.send(device, [np.asarray(flat, dtype=np.int32).reshape(-1, 2),
                                                   np.asarray(starts, dtype=np.int32)])
        cache[key] = (items_d, starts_d, len(starts) - 1, groups)
    return cache[key]


def _pick_block_cols(batch, G: int, nkv: int, window: int, device, which: str, head_dim: int) -> int:
    """128 or 256 columns to a block of the prompt attention.  Blocks of 256 columns (two
    column tiles a wave) read half as much from LDS and fetch half as many keys per flop.
    Measured alone they are ahead from some 3,500 tokens on (a tenth at 32,768 tokens, a
    quarter on the slower boxes of the pool); inside a whole prefill, between products that
    hold the chip at its power limit, the two are within a percent or two of each other up to
    16,384 tokens.  They are taken for the longest prompts only, where they were never behind:
    4,096 slices of 32 keys a block and more (some 24,000 tokens at four query heads to a key
    head)."""
    if head_dim > 128:
        return 128
    cache = getattr(batch, "_attn_work", None)
    if cache is None:
        cache = batch._attn_work = {}
    key = ("block_cols", G, nkv, window, which, head_dim)
    if key not in cache:
        cu, P = batch.host_cu_tokens, batch.host_start_pos
        slices = 0
        for r in _entries(batch, which):
            ncols = (cu[r + 1] - cu[r]) * G
            for c0 in range(0, ncols, 256):
                first = P[r] + c0 // G
                last = P[r] + (min(c0 + 256, ncols) - 1) // G
                lo = max(0, first - window + 1) if window > 0 else 0
                slices += last // 32 - lo // 32 + 1
        num_cus = _num_cus(device) if torch.device(device).type == "cuda" else 256
        per_cu = max(1, num_cus // max(1, nkv))
        cache[key] = 256 if slices >= 4096 * per_cu else 128
    return cache[key]


#: (for a caller that brings no runs of keys, see ``kernels.key_runs``, which is how the engine's steps come)
#: entries x kv heads from which a decode step gives every pair a block of eight waves that
#: split its keys and merge in LDS, instead of splitting the keys over blocks of one wave and
#: merging in a second kernel.  A block a pair keeps only as many CUs busy as there are pairs, and
#: eight waves do not pull a CU's share of HBM alone: measured at the 8B shape (eight kv heads),
#: 128 pairs are 1 % (2,048 cached tokens) to 11 % (32,768) slower as blocks, 160 pairs and more
#: 3 to 7 % faster at every length.
BLOCK_DECODE_MIN_PAIRS = 160


def pick_splits(waves: int, max_context: int) -> int:
    """Into how many runs the keys of a decoding request are split so that
    the launch has enough waves to pull on all of HBM: about 512 waves (a wave
    alone on its SIMD streams some 30 GB/s), at least 128 keys per run."""
    return max(1, min(-(-512 // max(1, waves)), -(-max_context // 128), 256))


def attention_mfma(q: torch.Tensor, nq: int, nkv: int, d: int, kv, batch, window: int = 0,
                   scale: float | None = None, splits: int | None = None,
                   block_bins: int | None = None, key_groups: int | None = None,
                   block_cols: int | None = None, sinks: torch.Tensor | None = None,
                   softcap: float = 0.0) -> torch.Tensor:
    """bfloat16 attention of the step's tokens on the matrix cores; decode-only
    steps split each request's keys over several waves and merge them.
    ``splits``, ``block_bins`` (blocks per kv head that share the work of
    long portions) and ``key_groups`` (groups of waves in such a block)
    override the choices made from the step's sizes."""
    _req(q, "attention q", torch.bfloat16, 2)
    T = q.shape[0]
    if q.shape[1] < nq * d:
        raise _lib.KernelError(f"attention q: rows of {q.shape[1]} hold fewer than nq*d = {nq * d}")
    k_cache, v_cache = kv.k_cache, kv.v_cache
    _req(k_cache, "k cache", q.dtype, 4)
    _req(v_cache, "v cache", q.dtype, 4)
    _check_cache(k_cache, v_cache, nkv, d, "attention")
    bt = _req(kv.block_tables, "block tables", torch.int32, 2)
    _req(batch.cu_tokens, "cu_tokens", torch.int32, 1)
    _req(batch.start_pos, "start_pos", torch.int32, 1)
    R = batch.num_reqs
    if batch.cu_tokens.numel() != R + 1 or batch.start_pos.numel() != R or bt.shape[0] != R:
        raise _lib.KernelError("attention: the step's tables do not describe the same number of requests")
    if batch.num_tokens != T:
        raise _lib.KernelError(f"attention: {T} query rows for a step of {batch.num_tokens} tokens")
    G = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.empty(T, nq * d, dtype=q.dtype, device=q.device)
    _check_sinks(sinks, nq)
    softcap = float(softcap or 0.0)
    L = _lib.load()
    stream = _stream()

    def launch(work, num_work, block_items, num_blocks, tiles, cols, splits, rows=None, groups=2):
        # partial results of split keys are kept by entry (split entries bring one token each)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty(splits, R, nq, d, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(splits, R, nq, 2, dtype=torch.float32, device=q.device)
        _lib.check(L.tff_attention_mfma(
            q.data_ptr(), q.stride(0), out.data_ptr(), _ptr(part_o), _ptr(part_ml), k_cache.data_ptr(),
            v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(),
            batch.start_pos.data_ptr(), _ptr(work), num_work, _ptr(block_items), num_blocks, tiles, cols,
            groups, splits, R if splits > 1 else T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window),
            float(scale), _ptr(sinks), softcap, stream))
        if splits > 1:
            _lib.check(L.tff_attention_split_reduce(
                part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), splits, R, nq, d, _ptr(rows),
                0 if rows is None else rows.shape[0], _ptr(sinks), stream))

    if batch.max_new_tokens == 1:
        # decoding only: a wave per request, kv head and run of keys; sizes come from the tables
        tiles = -(-G // 16)
        runs = getattr(kv, "key_runs", None)
        if splits is None and runs is not None and kv.runs_window == int(window) and T == R:
            # (the keys dealt into runs by the step's tables; entry i's token is row i)
            part_o = torch.empty(runs.shape[0], nq, d, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(runs.shape[0], nq, 2, dtype=torch.float32, device=q.device)
            _lib.check(L.tff_attention_mfma_runs(
                q.data_ptr(), q.stride(0), out.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), k_cache.data_ptr(),
                v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
                runs.data_ptr(), kv.run_start.data_ptr(), batch.cu_tokens.data_ptr(), runs.shape[0], R,
                1 if kv.runs_merge else 0, T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale),
                _ptr(sinks), softcap, stream))
            return out
        if splits is None:
            splits = pick_splits(R * tiles * nkv, batch.max_context)
        launch(None, R * tiles, None, 0, tiles, 16, splits)
        return out
    # long portions: blocks that share their keys through LDS (128 columns); short ones: a wave
    # of its own per 16 columns
    cols = 128 if batch.max_new_tokens * G > 64 else 16
    which = "all"
    single = _entries(batch, "single")
    if single and batch.max_context >= 256:
        # Requests that decode beside the portions have one token each and possibly long
        # contexts: they get the split-key kernel of their own rather than one block, or one
        # wave, each for all their keys.
        which = "multi"
        cache = getattr(batch, "_attn_work", None)
        if cache is None:
            cache = batch._attn_work = {}
        if splits is None and getattr(batch, "host_start_pos", None) is not None:
            # their keys dealt into runs of similar length, whatever the requests' lengths
            key = ("single_runs", nkv, int(window))
            if key not in cache:
                cu = batch.host_cu_tokens
                dealt = deal_key_runs([batch.host_start_pos[r] for r in single], int(window), nkv, blocks=False)
                runs = dealt.runs.copy()
                used = int(dealt.run_start[-1])
                runs[:used, 0] = np.asarray(single, dtype=np.int32)[runs[:used, 0]]     # rows of the step's tables
                cache[key] = tuple(_staging.send(q.device, [runs, dealt.run_start.copy(),
                                                            np.asarray([cu[r] for r in single], dtype=np.int32)])) \
                    + (dealt.merge,)
            runs, run_start, tokens, merge = cache[key]
            part_o = torch.empty(runs.shape[0], nq, d, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(runs.shape[0], nq, 2, dtype=torch.float32, device=q.device)
            _lib.check(L.tff_attention_mfma_runs(
                q.data_ptr(), q.stride(0), out.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), k_cache.data_ptr(),
                v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
                runs.data_ptr(), run_start.data_ptr(), tokens.data_ptr(), runs.shape[0], len(single), 1 if merge else 0,
                T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale), _ptr(sinks), softcap, stream))
        else:
            work = _attention_work(batch, G, 16, q.device, "single")
            if "single_rows" not in cache:
                cu = batch.host_cu_tokens
                cache["single_rows"] = _staging.send(q.device, [np.asarray([(r, cu[r]) for r in single], dtype=np.int32)])[0]
            sp = splits if splits is not None else pick_splits(work.shape[0] * nkv, batch.max_context)
            launch(work, work.shape[0], None, 0, 1, 16, sp, cache["single_rows"])
    if cols == 128:
        bcols = block_cols or _pick_block_cols(batch, G, nkv, int(window), q.device, which, d)
        if bcols == 256:
            # long prompts: items of 256 columns for blocks whose waves take two column tiles
            # each (one block a CU, so one bin a CU and kv head)
            per_cu = max(1, _num_cus(q.device) // max(1, nkv))
            work, block_items, num_blocks, _ = _attention_block_work(
                batch, G, nkv, int(window), q.device, cols=256, bins=block_bins or per_cu, which=which,
                key_groups=1, head_dim=d)
            launch(work, work.shape[0], block_items, num_blocks, 1, 256, 1, groups=1)
            return out
        work, block_items, num_blocks, groups = _attention_block_work(
            batch, G, nkv, int(window), q.device, bins=block_bins, which=which, key_groups=key_groups, head_dim=d)
        launch(work, work.shape[0], block_items, num_blocks, 1, 128, 1, groups=groups)
    else:
        work = _attention_work(batch, G, cols, q.device, which)
        launch(work, work.shape[0], None, 0, 1, cols, 1)
    return out


def decode_fused_supported(qkv: torch.Tensor, d: int, page_size: int, cos_sin, pairing: int, batch) -> bool:
    """Whether :func:`attention_decode_fused` takes this step: bfloat16, a head
    size of the matrix-core kernel, every entry one token, the whole head
    rotated (or none of it) with a pairing the kernel has in one lane."""
    if batch.max_new_tokens != 1 or not mfma_attention_supported(qkv.dtype, d, page_size):
        return False
    if cos_sin is None:
        return True
    return 2 * cos_sin.shape[1] == d and (pairing == 1 or d % 64 == 0)


def attention_decode_fused(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight, k_weight, eps: float,
                           cos_sin, pairing: int, kv, batch, window: int = 0, scale: float | None = None,
                           slot_mapping: torch.Tensor | None = None, splits: int | None = None,
                           key_runs: torch.Tensor | None = None, run_start: torch.Tensor | None = None,
                           runs_for_blocks: bool = False, runs_merge: bool = True) -> torch.Tensor:
    """A decode-only step from the fused projection's output ``qkv`` [R, (nq +
    2 nkv) d]: q/k norm, rotation, the new keys and values into their pages and
    the attention over the pages, in one kernel (plus the merge of split keys).
    ``slot_mapping`` (int32 [R]) says which tokens' keys and values are written
    (entries >= 0; the place is the one the block table gives for the token's
    position); None: no token's, the pages hold them already.  ``key_runs``
    (int32 [runs, 4]: row, first key, end of keys, the row's position) and ``run_start`` (int32
    [R + 1]): the rows' keys dealt into runs by the host, a wave per run and
    kv head (``kernels.key_runs``), or a block of eight waves if they were
    dealt for that (``runs_for_blocks``) and the head size allows it;
    ``runs_merge`` False: the caller knows that every row is one run, and the
    kernel that merges partial results is left out.  Without runs every
    row's keys are split alike (``splits``)."""
    _req(qkv, "attention_decode_fused qkv", torch.bfloat16, 2)
    R = batch.num_reqs
    if qkv.shape[0] != R or batch.num_tokens != R or batch.max_new_tokens != 1:
        raise _lib.KernelError("attention_decode_fused: every entry of the step must bring one token")
    if qkv.shape[1] != (nq + 2 * nkv) * d:
        raise _lib.KernelError(
            f"attention_decode_fused: rows of {qkv.shape[1]} are not (nq + 2 nkv) d = {(nq + 2 * nkv) * d}")
    k_cache, v_cache = kv.k_cache, kv.v_cache
    _req(k_cache, "k cache", qkv.dtype, 4)
    _req(v_cache, "v cache", qkv.dtype, 4)
    _check_cache(k_cache, v_cache, nkv, d, "attention_decode_fused")
    bt = _req(kv.block_tables, "block tables", torch.int32, 2)
    _req(batch.cu_tokens, "cu_tokens", torch.int32, 1)
    _req(batch.start_pos, "start_pos", torch.int32, 1)
    if batch.cu_tokens.numel() != R + 1 or batch.start_pos.numel() != R or bt.shape[0] != R:
        raise _lib.KernelError("attention_decode_fused: the step's tables do not describe the same number of requests")
    for w, nm in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if w is not None:
            _req(w, nm, torch.float32, 1)
            if w.numel() != d:
                raise _lib.KernelError(f"{nm}: {w.numel()} elements, head size {d}")
    max_pos = 0
    if cos_sin is not None:
        _req(cos_sin, "rotation table", torch.float32, 3)
        max_pos = cos_sin.shape[0]
        if 2 * cos_sin.shape[1] != d or cos_sin.shape[2] != 2:
            raise _lib.KernelError(f"attention_decode_fused: a rotation table of shape {tuple(cos_sin.shape)} "
                                   f"does not rotate whole heads of {d}")
    if slot_mapping is not None:
        _req(slot_mapping, "slot_mapping", torch.int32, 1)
        if slot_mapping.numel() != R:
            raise _lib.KernelError("attention_decode_fused: slot_mapping needs one entry per token")
    G = nq // nkv
    tiles = -(-G // 16)
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if key_runs is not None and splits is None:
        _req(key_runs, "key_runs", torch.int32, 2)
        _req(run_start, "run_start", torch.int32, 1)
        if key_runs.shape[1] != 4 or run_start.numel() != R + 1:
            raise _lib.KernelError(f"attention_decode_fused: runs of shape {tuple(key_runs.shape)} and "
                                   f"{run_start.numel()} run starts for {R} rows")
        P = key_runs.shape[0]
        out = torch.empty(R, nq * d, dtype=qkv.dtype, device=qkv.device)
        part_o = torch.empty(P, nq, d, dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty(P, nq, 2, dtype=torch.float32, device=qkv.device)
        _lib.check(_lib.load().tff_attention_decode_runs(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), k_cache.data_ptr(),
            v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
            _ptr(slot_mapping), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin), max_pos, int(pairing),
            key_runs.data_ptr(), run_start.data_ptr(), P, 8 if (runs_for_blocks and d <= 128 and tiles == 1) else 1,
            1 if runs_merge else 0, R, nq, nkv, d, k_cache.shape[2], k_cache.shape[0],
            int(window), float(scale), _stream()))
        return out
    if splits is None:
        # entries x kv heads enough for a block each to saturate HBM between them: the keys of
        # an entry are split among the eight waves of its block and merged in LDS (splits 0)
        splits = 0 if (R * nkv >= BLOCK_DECODE_MIN_PAIRS and tiles == 1 and d <= 128) else \
            pick_splits(R * tiles * nkv, batch.max_context)
    out = torch.empty(R, nq * d, dtype=qkv.dtype, device=qkv.device)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(splits, R, nq, d, dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty(splits, R, nq, 2, dtype=torch.float32, device=qkv.device)
    L = _lib.load()
    stream = _stream()
    _lib.check(L.tff_attention_decode_fused(
        qkv.data_ptr(), qkv.stride(0), out.data_ptr(), _ptr(part_o), _ptr(part_ml), k_cache.data_ptr(),
        v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
        _ptr(slot_mapping), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin), max_pos, int(pairing),
        splits, R, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale), stream))
    if splits > 1:
        _lib.check(L.tff_attention_split_reduce(part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), splits, R,
                                                nq, d, None, 0, None, stream))
    return out


def qkv_attention(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight, k_weight, eps: float, cos_sin,
                  pairing: int, kv, batch, window: int = 0, scale: float | None = None) -> torch.Tensor:
    """From the fused projection's output to the attention's output [T, nq d]:
    q/k norm and rotation, the step's keys and values into the cache at
    ``kv.slot_mapping`` (negative entries: not written; the call reads a cache
    that another call fills, or the row is padding), attention over the cache.  Decode-only steps in bfloat16 are one kernel."""
    if decode_fused_supported(qkv, d, kv.k_cache.shape[2], cos_sin, pairing, batch):
        # (a call that only reads its cache, or a padding row, has negative slots)
        runs = getattr(kv, "key_runs", None)
        if runs is not None and kv.runs_window != int(window):
            runs = None       # dealt for another window than this call's
        return attention_decode_fused(qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, pairing, kv, batch,
                                      window, scale, slot_mapping=kv.slot_mapping, key_runs=runs,
                                      run_start=kv.run_start if runs is not None else None,
                                      runs_for_blocks=runs is not None and kv.runs_for_blocks,
                                      runs_merge=runs is None or kv.runs_merge)
    qk_norm_rope_kv(qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, pairing, batch.positions,
                    kv.slot_mapping, kv.k_cache, kv.v_cache)
    return paged_attention(qkv, nq, nkv, d, kv, batch, window, scale)


def paged_attention(q: torch.Tensor, nq: int, nkv: int, d: int, kv, batch, window: int = 0,
                    scale: float | None = None, sinks: torch.Tensor | None = None,
                    softcap: float = 0.0) -> torch.Tensor:
    """Attention of a step's tokens over the cache view ``kv`` (k_cache,
    v_cache, block_tables) with the step's ``batch``.  bfloat16 with a head
    size the matrix-core kernel takes runs there; everything else (float32,
    other head sizes) on the general kernel.  ``sinks`` (float32 [nq]): a
    number per query head whose exponential is one more term of the softmax's
    denominator, with no key and no value, not scaled.  ``softcap`` c > 0: the
    scaled scores are capped, s <- c tanh(s / c), before the mask."""
    # (the matrix-core kernels cap scores at head sizes up to 192)
    if mfma_attention_supported(q.dtype, d, kv.k_cache.shape[2]) and not (softcap and d > 192):
        return attention_mfma(q, nq, nkv, d, kv, batch, window, scale, sinks=sinks, softcap=softcap)
    return attention_generic(q, nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                             batch.token_req, batch.positions, window, scale, sinks=sinks, softcap=softcap)


MFMA_HEAD_SIZES = tuple(range(16, 129, 16)) + (192, 256)


def padded_head_size(d: int, dtype: torch.dtype) -> int:
    """The head size a cache is laid out for when the attention's own is ``d``: the next size
    the matrix-core kernels take (bfloat16; beyond their largest, and in float32, the next
    multiple of 8, which the general kernel takes)."""
    if dtype == torch.bfloat16:
        for s in MFMA_HEAD_SIZES:
            if s >= d:
                return s
    return -(-d // 8) * 8


def latent_kv_store(x: torch.Tensor | None, rank: int, rot: int, norm_w: torch.Tensor | None, eps: float,
                    cos_sin: torch.Tensor | None, positions: torch.Tensor, slot_mapping: torch.Tensor,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, pairing: int = 1,
                    q_latent: torch.Tensor | None = None, q_norm_w: torch.Tensor | None = None) -> torch.Tensor | None:
    """Rows x [T, >= rank + rot] (rows may be strided; float32 rows may go to a bfloat16 cache): the RMS norm of
    the first ``rank`` elements times ``norm_w`` and the next ``rot`` elements, rotated by ``cos_sin``
    [max_pos, dims / 2, 2] in pairs (2i, 2i+1) (``pairing`` 1) or (i, i + dims/2) (``pairing`` 0), go to the
    tokens' slots of a cache of one key head of the padded size (keys [pages, 1, page_size, Dp], values
    transposed).  ``q_latent`` [T, q_rank] (rows may be strided, x's type): the queries' latent vectors, whose
    RMS norm times ``q_norm_w`` is returned in the cache's type, from the same launch.  ``x`` None: only
    that (a layer that reads a cache another layer fills)."""
    _req(k_cache, "k cache", ndim=4)
    _req(v_cache, "v cache", k_cache.dtype, 4)
    Dp = k_cache.shape[3]
    _check_cache(k_cache, v_cache, 1, Dp, "latent_kv_store")
    src = x if x is not None else q_latent
    if src is None:
        raise _lib.KernelError("latent_kv_store: neither rows for the cache nor latent vectors of queries")
    T = src.shape[0]
    for t, nm in ((x, "x"), (q_latent, "q_latent")):
        if t is not None and (not isinstance(t, torch.Tensor) or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1
                              or t.dtype != src.dtype or t.shape[0] != T):
            raise _lib.KernelError(f"latent_kv_store {nm}: expected a GPU matrix with unit inner stride, one row a token")
    if src.dtype != k_cache.dtype and not (src.dtype == torch.float32 and k_cache.dtype == torch.bfloat16):
        raise _lib.KernelError(f"latent_kv_store: rows of {src.dtype} for a cache of {k_cache.dtype}")
    dims, max_pos = 0, 0
    if x is not None:
        if x.shape[1] < rank + rot:
            raise _lib.KernelError(f"latent_kv_store: rows of {x.shape[1]} hold fewer than {rank} + {rot}")
        _req(norm_w, "latent norm weight", torch.float32, 1)
        if norm_w.numel() != rank:
            raise _lib.KernelError(f"latent norm weight: {norm_w.numel()} elements for a rank of {rank}")
        if Dp < rank + rot:
            raise _lib.KernelError(f"latent_kv_store: a cache of head size {Dp} does not hold {rank} + {rot}")
        if cos_sin is not None:
            _req(cos_sin, "rotation table", torch.float32, 3)
            max_pos, dims = cos_sin.shape[0], 2 * cos_sin.shape[1]
            if cos_sin.shape[2] != 2 or dims > rot:
                raise _lib.KernelError(f"rotation table {tuple(cos_sin.shape)} does not fit a rotated part of {rot}")
        _req(positions, "positions", torch.int32, 1)
        _req(slot_mapping, "slot_mapping", torch.int32, 1)
        if positions.numel() != T or slot_mapping.numel() != T:
            raise _lib.KernelError("latent_kv_store: positions and slot_mapping need one entry per token")
    q_out, q_rank = None, 0
    if q_latent is not None:
        q_rank = q_latent.shape[1]
        _req(q_norm_w, "query latent norm weight", torch.float32, 1)
        if q_norm_w.numel() != q_rank:
            raise _lib.KernelError(f"query latent norm weight: {q_norm_w.numel()} elements for a rank of {q_rank}")
        q_out = torch.empty(T, q_rank, dtype=k_cache.dtype, device=src.device)

    def row(t):
        return t.stride(0) if T > 1 else t.shape[1]

    _lib.check(_lib.load().tff_latent_kv_store(
        _ptr(x), row(x) if x is not None else 0, T, int(rank), int(rot), dims, int(pairing), _ptr(norm_w), float(eps),
        _ptr(cos_sin) if x is not None else None, max_pos, _ptr(positions), _ptr(slot_mapping), k_cache.data_ptr(),
        v_cache.data_ptr(), k_cache.shape[2], k_cache.shape[0], Dp, _ptr(q_latent), row(q_latent) if q_latent is not None else 0,
        q_rank, _ptr(q_norm_w), _ptr(q_out), q_rank, dtype_code(src.dtype), dtype_code(k_cache.dtype), _stream()))
    return q_out


def head_linear(x: torch.Tensor, x_head: int, weight_t: torch.Tensor, out_head: int | None = None,
                gate: torch.Tensor | None = None, tail: int = 0, cos_sin: torch.Tensor | None = None,
                positions: torch.Tensor | None = None, pairing: int = 1) -> torch.Tensor:
    """Products per head: x [T, >= H * x_head] (head h starts at h * x_head; rows may be strided),
    ``weight_t`` [H, N, K]: out[t, h, :N] = weight_t[h] x[t, h, :K].  Returns [T, H * out_head]
    (``out_head`` >= N + tail, by default N + tail), zeros behind what is written.
    ``gate`` [T, >= H * N] (rows may be strided): the products are multiplied by its sigmoid.
    ``tail``: so many elements of the input head behind the K are copied behind the products, the
    first ``2 * cos_sin.shape[1]`` of them rotated by the tokens' positions, in pairs (2i, 2i+1)
    (``pairing`` 1) or (i, i + dims/2) (``pairing`` 0)."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise _lib.KernelError("head_linear x: expected a GPU matrix with unit inner stride")
    _req(weight_t, "head_linear weight", x.dtype, 3)
    H, N, K = weight_t.shape
    T = x.shape[0]
    if x_head < K + tail or x.shape[1] < (H - 1) * x_head + K + tail:
        raise _lib.KernelError(f"head_linear: rows of {x.shape[1]} do not hold {H} heads of {K} + {tail}, {x_head} apart")
    width = N + tail
    out_head = width if out_head is None else int(out_head)
    if out_head < width:
        raise _lib.KernelError(f"head_linear: an output head of {out_head} does not hold {N} + {tail}")
    gate_row = 0
    if gate is not None:
        if not gate.is_cuda or gate.dim() != 2 or gate.stride(1) != 1 or gate.dtype != x.dtype \
                or gate.shape[0] != T or gate.shape[1] < H * N:
            raise _lib.KernelError("head_linear gate: expected [T, >= H * N] of the input's type on the GPU")
        gate_row = gate.stride(0) if T > 1 else gate.shape[1]
    dims, max_pos = 0, 0
    if cos_sin is not None and tail > 0:
        _req(cos_sin, "rotation table", torch.float32, 3)
        _req(positions, "positions", torch.int32, 1)
        max_pos, dims = cos_sin.shape[0], 2 * cos_sin.shape[1]
        if cos_sin.shape[2] != 2 or dims > tail or positions.numel() != T:
            raise _lib.KernelError(f"head_linear: rotation table {tuple(cos_sin.shape)} or positions do not fit")
    out = torch.empty(T, H * out_head, dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().tff_head_linear(
        x.data_ptr(), x.stride(0) if T > 1 else x.shape[1], int(x_head), weight_t.data_ptr(), out.data_ptr(),
        H * out_head, out_head, T, H, K, N, _ptr(gate), gate_row, int(tail), dims, int(pairing), out_head if out_head > N else 0,
        _ptr(cos_sin) if dims else None, max_pos, _ptr(positions) if dims else None, dtype_code(x.dtype), _stream()))
    return out


def scale_add_rmsnorm(resid: torch.Tensor, delta, weight: torch.Tensor, eps: float, alpha: float,
                      out_dtype: torch.dtype | None = None) -> torch.Tensor | None:
    """``resid <- rmsnorm(alpha * resid + delta) * weight`` in place on the float32 residual
    stream (the norm of a block that norms after the sum); returns the same rows in
    ``out_dtype`` (None: no copy).  ``delta`` may be None or what ``linear`` returns with
    ``partials=True``."""
    _req(resid, "scale_add_rmsnorm resid", torch.float32, 2)
    n, H = resid.shape
    _req(weight, "scale_add_rmsnorm weight", torch.float32, 1)
    if weight.numel() != H:
        raise _lib.KernelError(f"scale_add_rmsnorm: weight has {weight.numel()} elements, rows have {H}")
    if isinstance(delta, PendingProduct):
        delta = delta.run()
    planes, plane = 1, 0
    if delta is not None:
        _req(delta, "scale_add_rmsnorm delta", torch.float32, 3 if delta.dim() == 3 else 2)
        if tuple(delta.shape[-2:]) != tuple(resid.shape):
            raise _lib.KernelError(
                f"scale_add_rmsnorm: delta {tuple(delta.shape)} does not match resid {tuple(resid.shape)}")
        if delta.dim() == 3:
            planes, plane = delta.shape[0], delta.stride(0)
    out = torch.empty(n, H, dtype=out_dtype, device=resid.device) if out_dtype is not None else None
    _lib.check(_lib.load().tff_scale_add_rmsnorm(
        resid.data_ptr(), _ptr(delta), planes, plane, float(alpha), weight.data_ptr(), float(eps), _ptr(out), n, H,
        dtype_code(out_dtype) if out_dtype is not None else 0, _stream()))
    return out


def gelu(x: torch.Tensor, tanh_form: bool = False) -> torch.Tensor:
    """0.5 z (1 + erf(z / sqrt 2)), or the tanh form, element by element, in float32."""
    _req(x, "gelu input")
    out = torch.empty_like(x)
    _lib.check(_lib.load().tff_gelu(x.data_ptr(), out.data_ptr(), x.numel(), 1 if tanh_form else 0,
                                    dtype_code(x.dtype), _stream()))
    return out


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    """max(z, 0)^2, element by element, in float32."""
    _req(x, "relu_squared input")
    out = torch.empty_like(x)
    _lib.check(_lib.load().tff_gelu(x.data_ptr(), out.data_ptr(), x.numel(), 2, dtype_code(x.dtype), _stream()))
    return out


def route_topk(h: torch.Tensor | None, router: torch.Tensor | None, bias: torch.Tensor | None, top: int,
               logits: torch.Tensor | None = None, softmax: bool = False, normalize: bool = True):
    """s = sigmoid(z) with z = h . router^T in float32 (router float32 [E, width]) or z = ``logits``
    (float32 [T, E], a product that ran before); the ``top`` experts with the largest s + bias;
    returns (int32 [T, top], float32 [T, top] = s / (sum of the chosen s + 1e-20)).  With
    ``softmax``, s = softmax(z) over all experts and the weights are the chosen s as they are; without
    ``normalize``, s = sigmoid(z) and the weights are the chosen s as they are."""
    if logits is not None:
        _req(logits, "router logits", torch.float32, 2)
        T, E = logits.shape
        width, dev, dt = 0, logits.device, torch.float32
    else:
        _req(h, "route_topk h", ndim=2)
        _req(router, "router", torch.float32, 2)
        T, width = h.shape
        E = router.shape[0]
        dev, dt = h.device, h.dtype
        if router.shape[1] != width:
            raise _lib.KernelError(f"route_topk: router {tuple(router.shape)} for rows of {width}")
    if bias is not None:
        _req(bias, "router bias", torch.float32, 1)
        if bias.numel() != E:
            raise _lib.KernelError(f"route_topk: {bias.numel()} bias terms for {E} experts")
    idx = torch.empty(T, top, dtype=torch.int32, device=dev)
    wts = torch.empty(T, top, dtype=torch.float32, device=dev)
    _lib.check(_lib.load().tff_route_topk(None if logits is not None else h.data_ptr(), width,
                                          None if logits is not None else router.data_ptr(), _ptr(logits), _ptr(bias),
                                          T, width, E, int(top), 1 if softmax else (0 if normalize else 2), idx.data_ptr(), wts.data_ptr(), dtype_code(dt), _stream()))
    return idx, wts


def pad_expert_rows(w: torch.Tensor) -> torch.Tensor:
    """Stacked expert matrices [E, out, in] with a little room behind every row where the rows
    would lie a multiple of 1 KB apart: such rows all come through the same few memory channels,
    and a tile of sixteen of them is fetched at a fraction of the speed."""
    k = w.shape[-1]
    if (k * w.element_size()) % 1024:
        return w.contiguous()
    return torch.nn.functional.pad(w, (0, 128 // w.element_size())).contiguous()


#: tokens from which a step's (token, expert) pairs are dealt to their experts and run on the matrix
#: cores; below, every pair streams its expert's rows itself, which is what few tokens are bound by
EXPERT_TILES_MIN_TOKENS = 32


def routed_experts(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                   idx: torch.Tensor, wts: torch.Tensor, limit: float, act_alpha: float,
                   by_tiles: bool | None = None, up_offset: float = 1.0, weight_input: bool = False) -> torch.Tensor:
    """The weighted sum of each token's chosen experts: y = g sigmoid(act_alpha g) (u + up_offset) with
    g = min(Wg h, limit), u = clamp(Wu h, -limit, limit); out = sum_k wts[:, k] Wd y.
    ``w_gate`` None: experts without a gate, y = max(Wu h, 0)^2.  ``weight_input``: a pair's weight multiplies
    what goes into its expert instead of what comes out, out = sum_k expert_k(wts[:, k] h); since W (w h) = w (W h)
    it is applied to both first products, before clamps and activation.
    ``w_gate``, ``w_up`` [E, ff, >= width], ``w_down`` [E, width, >= ff] of h's type (the last
    dimension may be wider than what is multiplied: see :func:`pad_expert_rows`).  float32
    [T, width], or (many tokens in bfloat16, ``by_tiles``) [top, T, width]: the terms of the sum
    over k, which ``scale_add_rmsnorm`` and ``as_tensor`` add up in order."""
    _req(h, "routed_experts h", ndim=2)
    T, width = h.shape
    for w, nm in ((w_gate, "gate"), (w_up, "up"), (w_down, "down")):
        if w is not None or nm != "gate":
            _req(w, f"experts {nm}", h.dtype, 3)
    E, ff, ld_in = w_up.shape
    ld_down = w_down.shape[2]
    if ld_in < width or (w_gate is not None and tuple(w_gate.shape) != (E, ff, ld_in)) \
            or tuple(w_down.shape[:2]) != (E, width) or ld_down < ff:
        raise _lib.KernelError(f"routed_experts: weights {w_gate is not None and tuple(w_gate.shape)}, {tuple(w_up.shape)}, "
                               f"{tuple(w_down.shape)} for rows of {width}")
    _req(idx, "experts idx", torch.int32, 2)
    _req(wts, "experts weights", torch.float32, 2)
    top = idx.shape[1]
    if tuple(idx.shape) != (T, top) or tuple(wts.shape) != (T, top):
        raise _lib.KernelError("routed_experts: idx and weights must be [T, top]")
    L = _lib.load()
    y = torch.empty(T * top, ff, dtype=h.dtype, device=h.device)
    if by_tiles is None:
        by_tiles = T >= EXPERT_TILES_MIN_TOKENS
    if by_tiles and h.dtype == torch.bfloat16 and L.tff_experts_tiles_supported(width, ff, width):
        # many tokens: the pairs dealt to their experts, the products on the matrix cores; the result
        # comes as one plane per chosen expert, for the norm that follows to add up in their order
        max_tiles = T * top // 64 + E
        tables = torch.empty(129 * max_tiles + 1, dtype=torch.int32, device=h.device)
        out = torch.empty(top, T, width, dtype=torch.float32, device=h.device)
        _lib.check(L.tff_experts_by_tiles(
            h.data_ptr(), width, _ptr(w_gate), w_up.data_ptr(), w_down.data_ptr(), idx.data_ptr(), wts.data_ptr(),
            T, top, E, width, ff, ld_in, ld_down, float(limit), float(act_alpha), float(up_offset), tables.data_ptr(), tables[max_tiles:].data_ptr(),
            tables[129 * max_tiles:].data_ptr(), max_tiles, y.data_ptr(), out.data_ptr(), 1 if weight_input else 0, _stream()))
        return out if top > 1 else out[0]
    _lib.check(L.tff_experts_gate_up(h.data_ptr(), width, _ptr(w_gate), w_up.data_ptr(), idx.data_ptr(), T, top, E,
                                     width, ff, ld_in, float(limit), float(act_alpha), float(up_offset),
                                     wts.data_ptr() if weight_input else None, y.data_ptr(), dtype_code(h.dtype), _stream()))
    out = torch.empty(T, width, dtype=torch.float32, device=h.device)
    _lib.check(L.tff_experts_down(y.data_ptr(), w_down.data_ptr(), idx.data_ptr(), None if weight_input else wts.data_ptr(), T, top, E, width, ff,
                                  ld_down, out.data_ptr(), dtype_code(h.dtype), _stream()))
    return out


def group_rmsnorm_add(resid: torch.Tensor | None, delta, weight: torch.Tensor, groups: int, eps: float,
                      out_dtype: torch.dtype | None = None, rows: torch.Tensor | None = None):
    """A norm on a sublayer's output: every row of ``delta`` is cut into ``groups`` equal parts, each
    divided by its own root mean square, the whole times ``weight``.  With ``resid`` the result is
    added into the float32 residual stream in place and the new rows are returned in ``out_dtype``
    (None: nothing is returned); without, the normed rows themselves are returned (of the rows
    ``rows`` only, where given).  ``delta`` may be what ``linear`` returns with ``partials=True``."""
    if isinstance(delta, PendingProduct):
        delta = delta.run()
    if isinstance(delta, ScaledRows):
        delta = delta.materialize()
    _req(delta, "group_rmsnorm_add delta", torch.float32, 3 if delta.dim() == 3 else 2)
    planes, plane = 1, 0
    if delta.dim() == 3:
        planes, plane = delta.shape[0], delta.stride(0)
    n_src, H = delta.shape[-2:]
    _req(weight, "group_rmsnorm_add weight", torch.float32, 1)
    if weight.numel() != H or groups <= 0 or H % groups:
        raise _lib.KernelError(f"group_rmsnorm_add: rows of {H}, weight of {weight.numel()}, {groups} groups")
    n = n_src
    if resid is not None:
        _req(resid, "group_rmsnorm_add resid", torch.float32, 2)
        if tuple(resid.shape) != (n_src, H) or rows is not None:
            raise _lib.KernelError(f"group_rmsnorm_add: resid {tuple(resid.shape)} for delta {tuple(delta.shape)}")
    elif rows is not None:
        _req(rows, "group_rmsnorm_add rows", torch.int32, 1)
        if planes != 1:
            raise _lib.KernelError("group_rmsnorm_add: chosen rows of partial sums")
        n = rows.numel()
    if resid is None and out_dtype is None:
        out_dtype = torch.float32
    out = torch.empty(n, H, dtype=out_dtype, device=delta.device) if out_dtype is not None else None
    _lib.check(_lib.load().tff_group_rmsnorm_add(
        _ptr(resid), delta.data_ptr(), planes, plane, _ptr(rows), weight.data_ptr(), int(groups), float(eps), _ptr(out),
        n, H, dtype_code(out_dtype) if out_dtype is not None else 0, _stream()))
    return out


def depth_average(hist: torch.Tensor, n: int, coef: torch.Tensor, x: torch.Tensor,
                  out_dtype: torch.dtype | None = None):
    """``hist[n - 1] <- x; x <- sum_{j < n} coef[j] * hist[j]`` on the float32 residual stream ``x``
    [T, W], with ``hist`` [depths, T, W] the stream as the embedding and every layer so far left it;
    returns the new x in ``out_dtype`` (None: nothing)."""
    _req(hist, "depth_average hist", torch.float32, 3)
    _req(x, "depth_average x", torch.float32, 2)
    _req(coef, "depth_average coef", torch.float32, 1)
    if tuple(hist.shape[1:]) != tuple(x.shape) or not 1 <= n <= hist.shape[0] or coef.numel() < n:
        raise _lib.KernelError(f"depth_average: {n} levels of {tuple(hist.shape)} for x {tuple(x.shape)}, "
                               f"{coef.numel()} coefficients")
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) if out_dtype is not None else None
    _lib.check(_lib.load().tff_depth_average(hist.data_ptr(), hist.stride(0), int(n), coef.data_ptr(), x.data_ptr(),
                                             _ptr(out), x.numel(), dtype_code(out_dtype) if out_dtype is not None else 0,
                                             _stream()))
    return out


def scale_rows(x: torch.Tensor, alpha: float) -> torch.Tensor:
    """``x <- alpha * x`` in place on float32 rows."""
    _req(x, "scale_rows x", torch.float32)
    _lib.check(_lib.load().tff_scale_rows(x.data_ptr(), float(alpha), x.numel(), _stream()))
    return x


def _state_rows(state: torch.Tensor, what: str) -> int:
    _req(state, what, torch.float32, 2)
    return state.stride(0)


def token_shift_mix(x: torch.Tensor, state: torch.Tensor, prev_off: int, mu: torch.Tensor, batch,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """out[m, t] = x[t] + (x'[t] - x[t]) * mu[m] with x' the row of the token before t in its request:
    the row above, or for the first token of a request's portion ``state[slot, prev_off:prev_off + W]``
    (float32 [slots, row])."""
    _req(x, "token_shift_mix x", torch.float32, 2)
    _req(mu, "token_shift_mix mu", torch.float32, 2)
    T, W = x.shape
    M = mu.shape[0]
    row = _state_rows(state, "token_shift_mix state")
    if mu.shape[1] != W or prev_off < 0 or prev_off + W > row:
        raise _lib.KernelError(f"token_shift_mix: rows of {W}, mu {tuple(mu.shape)}, state rows of {row}")
    out = torch.empty(M, T, W, dtype=out_dtype, device=x.device)
    _lib.check(_lib.load().tff_token_shift_mix(x.data_ptr(), state.data_ptr(), row, int(prev_off), mu.data_ptr(), M,
                                               batch.token_req.data_ptr(), batch.cu_tokens.data_ptr(),
                                               batch.state_slots.data_ptr(), out.data_ptr(), T, W, dtype_code(out_dtype),
                                               _stream()))
    return out


#: tokens of a step's longest entry from which the recurrence runs in its form for prompts
WKV_LONG_PORTION = 16


def wkv_recurrence(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, z: torch.Tensor, w0: torch.Tensor,
                   u: torch.Tensor, state: torch.Tensor, batch, H: int, D: int, x: torch.Tensor | None = None,
                   prev_off: int = 0) -> torch.Tensor:
    """The recurrence o_t = (S + diag(u) k_t v_t^T)^T r_t, S <- diag(w_t) S + k_t v_t^T with
    w_t = exp(-exp(z_t + w0)) over each request's tokens of this step, per head; S [D, D] float32 lies at
    the start of the request's row of ``state`` (float32 [slots, row]).  r, k, v, z float32 [T, H * D]
    (columns of wider rows are fine, all with the same stride).  ``x`` [T, W]: each request's last row
    of it is left at ``state[slot, prev_off:]``.  Returns o float32 [T, H * D]."""
    T = r.shape[0]
    HD = H * D
    for t, nm in ((r, "r"), (k, "k"), (v, "v"), (z, "z")):
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.float32 or t.dim() != 2 \
                or tuple(t.shape) != (T, HD) or t.stride(1) != 1 or t.stride(0) != r.stride(0):
            raise _lib.KernelError(f"wkv_recurrence {nm}: expected float32 [{T}, {HD}] with the rows' stride of r")
    _req(w0, "wkv_recurrence w0", torch.float32, 1)
    _req(u, "wkv_recurrence u", torch.float32, 1)
    if w0.numel() != HD or u.numel() != HD:
        raise _lib.KernelError(f"wkv_recurrence: w0 and u must hold {HD} elements")
    row = _state_rows(state, "wkv_recurrence state")
    W = 0
    if x is not None:
        _req(x, "wkv_recurrence x", torch.float32, 2)
        W = x.shape[1]
        if x.shape[0] != T or prev_off < HD * D or prev_off + W > row:
            raise _lib.KernelError("wkv_recurrence: the state's row does not hold x behind the heads' matrices")
    if HD * D > row:
        raise _lib.KernelError(f"wkv_recurrence: state rows of {row} for {H} heads of {D} x {D}")
    o = torch.empty(T, HD, dtype=torch.float32, device=r.device)
    if T == 0:
        return o
    _lib.check(_lib.load().tff_wkv_recurrence(r.data_ptr(), k.data_ptr(), v.data_ptr(), z.data_ptr(), r.stride(0),
                                              w0.data_ptr(), u.data_ptr(), state.data_ptr(), row,
                                              batch.cu_tokens.data_ptr(), batch.state_slots.data_ptr(), o.data_ptr(),
                                              batch.num_reqs, H, D, _ptr(x), W, int(prev_off),
                                              1 if getattr(batch, "max_new_tokens", 0) >= WKV_LONG_PORTION else 0, _stream()))
    return o


def head_norm_gate(o: torch.Tensor, g: torch.Tensor, weight: torch.Tensor, eps: float, H: int, D: int,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """``o / sqrt(mean over each head of o^2 + eps) * weight * silu(g)`` for o, g float32 [T, H * D]."""
    _req(o, "head_norm_gate o", torch.float32, 2)
    _req(weight, "head_norm_gate weight", torch.float32, 1)
    T = o.shape[0]
    if not isinstance(g, torch.Tensor) or g.dtype != torch.float32 or g.dim() != 2 or g.stride(1) != 1 \
            or tuple(g.shape) != (T, H * D) or o.shape[1] != H * D or weight.numel() != H * D:
        raise _lib.KernelError("head_norm_gate: o and g must be float32 [T, heads * dim]")
    out = torch.empty(T, H * D, dtype=out_dtype, device=o.device)
    _lib.check(_lib.load().tff_head_norm_gate(o.data_ptr(), g.data_ptr(), g.stride(0) if T > 1 else H * D,
                                              weight.data_ptr(), float(eps), out.data_ptr(), T, H, D,
                                              dtype_code(out_dtype), _stream()))
    return out


def tanh(x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    _req(x, "tanh input", torch.float32)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _lib.check(_lib.load().tff_tanh(x.data_ptr(), out.data_ptr(), x.numel(), dtype_code(out_dtype), _stream()))
    return out


def qk_bias_norm_store(qk: torch.Tensor, q_bias, k_bias, eps: float, H: int, G: int, D: int, kv) -> torch.Tensor:
    """q and k of one projection (float32 [T, (H + G) * D]) with their biases added; q divided by its root
    mean square per head and returned in the cache's type [T, H * D]; k written to the token's slot
    as projected (the value pages) and divided by its root mean square (the key pages)."""
    _req(qk, "qk_bias_norm_store qk", torch.float32, 2)
    T = qk.shape[0]
    if qk.shape[1] != (H + G) * D:
        raise _lib.KernelError(f"qk_bias_norm_store: rows of {qk.shape[1]} for {H} + {G} heads of {D}")
    for b, n, nm in ((q_bias, H * D, "q bias"), (k_bias, G * D, "k bias")):
        if b is not None:
            _req(b, nm, torch.float32, 1)
            if b.numel() != n:
                raise _lib.KernelError(f"qk_bias_norm_store: {nm} of {b.numel()} elements, expected {n}")
    _check_cache(kv.k_cache, kv.v_cache, G, D, "qk_bias_norm_store")
    dt = kv.k_cache.dtype
    q = torch.empty(T, H * D, dtype=dt, device=qk.device)
    _req(kv.slot_mapping, "slot_mapping", torch.int32, 1)
    if kv.slot_mapping.numel() < T:
        raise _lib.KernelError("qk_bias_norm_store: fewer slots than tokens")
    _lib.check(_lib.load().tff_qk_bias_norm_store(qk.data_ptr(), qk.stride(0), _ptr(q_bias), _ptr(k_bias), float(eps),
                                                  q.data_ptr(), kv.k_cache.data_ptr(), kv.v_cache.data_ptr(),
                                                  kv.slot_mapping.data_ptr(), kv.page_size, T, H, G, D, dtype_code(dt),
                                                  _stream()))
    return q


#: blocks a step of few tokens spreads its attention over (two a CU)
MIXED_ATTENTION_BLOCKS = 512
#: tokens of a step from which bfloat16 attention runs sixteen queries a block on the matrix cores
MIXED_ATTENTION_Q16_TOKENS = 64
#: blocks that kernel's items are spread over where they are fewer (a block a CU)
MIXED_ATTENTION_Q16_BLOCKS = 256


def mixed_attention(q: torch.Tensor, H: int, G: int, D: int, kv, batch, scale: float, softcap: float = 0.0,
                    bias: torch.Tensor | None = None, mix: torch.Tensor | None = None, window: int = 0,
                    keep_first: int = 0, sink: bool = False, splits: int | None = None) -> torch.Tensor:
    """Causal attention over the paged cache whose heads exchange their scores before the softmax:
    s_g = softcap * tanh(scale * q_g . k_g / softcap) (softcap 0: scale * q_g . k_g) + bias[min(i - j, rows - 1), g];
    s'_h = sum_g mix[h, g] s_g; key j is visible to query i if j <= i and (i - j < window or j < keep_first)
    (window 0: all j <= i); softmax over the visible keys, with one more term of 1 in the denominator
    if ``sink``; the values are the value pages.  q [T, H * D] in the cache's type; bias float32 [rows, H];
    mix float32 [H, H].  A step of few tokens deals each token's keys (tiles of 64) to several blocks
    (``splits``; by default so many that some 512 blocks run, from the longest context the step's tables
    can hold) and merges them in a second kernel."""
    dt = kv.k_cache.dtype
    _req(q, "mixed_attention q", dt, 2)
    T = q.shape[0]
    if q.shape[1] != H * D or H % G:
        raise _lib.KernelError(f"mixed_attention: q {tuple(q.shape)} for {H} heads of {D} on {G} kv heads")
    _check_cache(kv.k_cache, kv.v_cache, G, D, "mixed_attention")
    L = _lib.load()
    if not L.tff_mixed_attention_supported(H, D, 1 if mix is not None else 0):
        raise _lib.KernelError(f"mixed_attention: {H} heads of {D} are more than a block holds")
    rows = 0
    if bias is not None:
        _req(bias, "mixed_attention bias", torch.float32, 2)
        rows = bias.shape[0]
        if bias.shape[1] != H or rows < 1:
            raise _lib.KernelError(f"mixed_attention: bias {tuple(bias.shape)} for {H} heads")
    if mix is not None:
        _req(mix, "mixed_attention mix", torch.float32, 2)
        if tuple(mix.shape) != (H, H):
            raise _lib.KernelError(f"mixed_attention: mix {tuple(mix.shape)} for {H} heads")
    bt = _req(kv.block_tables, "block_tables", torch.int32, 2)
    if batch.token_req.numel() < T or batch.positions.numel() < T:
        raise _lib.KernelError("mixed_attention: the step's tables are shorter than q")
    out = torch.empty(T, H * D, dtype=dt, device=q.device)
    cu = getattr(batch, "host_cu_tokens", None)
    if (splits is None and dt == torch.bfloat16 and cu is not None and T >= MIXED_ATTENTION_Q16_TOKENS
            and getattr(batch, "max_new_tokens", 0) >= 16
            and L.tff_mixed_attention_q16_supported(H, D, kv.page_size, 1 if mix is not None else 0)):
        # a prompt's portions: sixteen queries a block, the products on the matrix cores
        cache = getattr(batch, "_q16_work", None)
        if cache is None:
            items = [(t, min(16, cu[r + 1] - t)) for r in range(len(cu) - 1) for t in range(cu[r], cu[r + 1], 16)]
            cache = batch._q16_work = _staging.send(q.device, [np.asarray(items, dtype=np.int32).reshape(-1, 2)])[0]
        # tiles of 16 keys an item can have at most; where the items are fewer than the CUs, their tiles are dealt
        # to several blocks
        reach = min(bt.shape[1] * kv.page_size, getattr(batch, "max_context", 1 << 30))
        tiles16 = -(-min(keep_first, reach) // 16) + (-(-min(window + 15, reach) // 16) + 1 if window > 0 else -(-reach // 16))
        parts = max(1, min(tiles16, 8, MIXED_ATTENTION_Q16_BLOCKS // cache.shape[0]))
        per = -(-tiles16 // parts)
        parts = -(-tiles16 // per) if parts > 1 else 1
        ws = None
        if parts > 1:
            ws = torch.empty(L.tff_mixed_attention_workspace_bytes(T, H, D, parts) // 4, dtype=torch.float32, device=q.device)
        _lib.check(L.tff_mixed_attention_q16(q.data_ptr(), kv.k_cache.data_ptr(), kv.v_cache.data_ptr(), bt.data_ptr(),
                                             bt.shape[1], batch.token_req.data_ptr(), batch.positions.data_ptr(),
                                             cache.data_ptr(), cache.shape[0], _ptr(bias), rows, _ptr(mix), float(scale),
                                             float(softcap), int(window), int(keep_first), 1 if sink else 0,
                                             out.data_ptr(), T, H, G, D, kv.page_size, parts, per, _ptr(ws), _stream()))
        return out
    # tiles of 64 keys that a token of this step can have at most (what the block tables can hold, or the window
    # and the kept tokens): a size the host knows without reading a position, so a captured step keeps it
    reach = bt.shape[1] * kv.page_size
    tiles = -(-min(keep_first, reach) // 64) + (-(-min(window, reach) // 64) + 1 if window > 0 else -(-reach // 64))
    if splits is None:
        splits = max(1, min(tiles, MIXED_ATTENTION_BLOCKS // max(T, 1)))
    per = -(-tiles // max(1, splits))
    splits = -(-tiles // per) if splits > 1 else 1
    ws = None
    if splits > 1:
        ws = torch.empty(L.tff_mixed_attention_workspace_bytes(T, H, D, splits) // 4, dtype=torch.float32, device=q.device)
    _lib.check(L.tff_mixed_attention(q.data_ptr(), kv.k_cache.data_ptr(), kv.v_cache.data_ptr(), bt.data_ptr(),
                                     bt.shape[1], batch.token_req.data_ptr(), batch.positions.data_ptr(), _ptr(bias),
                                     rows, _ptr(mix), float(scale), float(softcap), int(window), int(keep_first),
                                     1 if sink else 0, out.data_ptr(), T, H, G, D, kv.page_size, splits, per, _ptr(ws),
                                     dtype_code(dt), _stream()))
    return out


class PendingTerms:
    """Several terms that a block has not added to the residual stream yet (a layer whose mixer and
    feed-forward read the same rows leaves two); each is what a mixer or feed-forward may return:
    a tensor, a stack of partial sums or a product that has not run.  ``add_rmsnorm_pair`` and
    ``add_rmsnorm`` take them; ``as_tensor`` adds them up."""

    def __init__(self, terms):
        self.terms = [t for t in terms if t is not None]
        if len(self.terms) > 2:
            raise _lib.KernelError("pending terms: at most two")


def _planes_of(delta, shape, what: str):
    """(tensor or None, planes, plane stride) of a pending term for a kernel that adds planes up."""
    if delta is None:
        return None, 0, 0
    if isinstance(delta, PendingProduct):
        delta = delta.run()
    _req(delta, what, torch.float32, 3 if delta.dim() == 3 else 2)
    if tuple(delta.shape[-2:]) != tuple(shape):
        raise _lib.KernelError(f"{what}: {tuple(delta.shape)} does not match the stream {tuple(shape)}")
    if delta.dim() == 3:
        return delta, delta.shape[0], delta.stride(0)
    return delta, 1, 0


def add_rmsnorm_pair(resid: torch.Tensor, delta, bias: torch.Tensor | None, w1: torch.Tensor,
                     w2: torch.Tensor | None, eps: float, out_dtype: torch.dtype,
                     rows: torch.Tensor | None = None):
    """``resid += terms + bias`` (``delta``: None, one pending term or :class:`PendingTerms`; ``bias``
    float32 [H] or None) and two RMS norms of the sum, one with each weight (``w2`` None: one);
    with ``rows`` the norms of those rows only, ``resid`` untouched.  Returns (out1, out2 or None)."""
    _req(resid, "add_rmsnorm_pair resid", torch.float32, 2)
    H = resid.shape[1]
    for w, nm in ((w1, "first weight"), (w2, "second weight"), (bias, "bias")):
        if w is not None:
            _req(w, f"add_rmsnorm_pair {nm}", torch.float32, 1)
            if w.numel() != H:
                raise _lib.KernelError(f"add_rmsnorm_pair: {nm} has {w.numel()} elements, rows have {H}")
    terms = delta.terms if isinstance(delta, PendingTerms) else ([] if delta is None else [delta])
    d = [_planes_of(t, resid.shape, "add_rmsnorm_pair term") for t in terms] + [(None, 0, 0)] * 2
    if rows is not None:
        _req(rows, "add_rmsnorm_pair rows", torch.int32, 1)
        n = rows.numel()
    else:
        n = resid.shape[0]
    out1 = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    out2 = torch.empty(n, H, dtype=out_dtype, device=resid.device) if w2 is not None else None
    _lib.check(_lib.load().tff_add_rmsnorm_pair(
        resid.data_ptr(), _ptr(d[0][0]), d[0][1], d[0][2], _ptr(d[1][0]), d[1][1], d[1][2], _ptr(bias), w1.data_ptr(),
        _ptr(w2), float(eps), out1.data_ptr(), _ptr(out2), _ptr(rows), n, H, dtype_code(out_dtype), _stream()))
    return out1, out2


def softcap_(z: torch.Tensor, cap: float) -> torch.Tensor:
    """z <- cap * tanh(z / cap) in place on float32."""
    _req(z, "softcap", torch.float32)
    _lib.check(_lib.load().tff_softcap(z.data_ptr(), z.numel(), float(cap), _stream()))
    return z


def route_by_table(table: torch.Tensor, token_ids: torch.Tensor, num_experts: int):
    """Experts by a table over the token ids (int32 [vocab, top]): (int32 [T, top], float32 [T, top] = 1 / top)."""
    _req(table, "route_by_table table", torch.int32, 2)
    _req(token_ids, "route_by_table ids", torch.int32, 1)
    T, (V, top) = token_ids.numel(), table.shape
    idx = torch.empty(T, top, dtype=torch.int32, device=table.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=table.device)
    _lib.check(_lib.load().tff_route_by_table(table.data_ptr(), token_ids.data_ptr(), T, V, top, int(num_experts),
                                              idx.data_ptr(), wts.data_ptr(), _stream()))
    return idx, wts


def _rows2(t: torch.Tensor, name: str, dtype, cols: int):
    """A GPU matrix with unit inner stride (rows may be strided) of at least ``cols`` columns; its row stride."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.dtype != dtype \
            or t.shape[1] < cols:
        raise _lib.KernelError(f"{name}: expected a GPU matrix of {dtype} with unit inner stride and {cols} columns or more")
    return t.stride(0) if t.shape[0] > 1 else t.shape[1]


def gated_delta(proj: torch.Tensor, conv_w: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                state: torch.Tensor, batch, H: int, G: int, D: int, E: int) -> torch.Tensor:
    """The gated delta rule over the step's tokens.  ``proj`` float32 [T, >= C + 2 H]: the projections q [G, D],
    k [G, D], v [H, E] (C = 2 G D + H E channels), b [H], a [H]; ``conv_w`` float32 [C, taps]; ``state`` float32
    [slots, >= H E D + (taps - 1) C]: per request the heads' matrices and the convolution's last inputs.
    q, k, v pass the causal convolution and silu; q, k become unit vectors per head (q times D^(-1/2));
    beta = sigmoid(b); decay = exp(-exp(a_log) softplus(a + dt_bias)); per head (keys and queries of head
    h // (H / G)): S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns o float32 [T, H E]."""
    C = 2 * G * D + H * E
    T = proj.shape[0]
    ldp = _rows2(proj, "gated_delta proj", torch.float32, C + 2 * H)
    _req(conv_w, "gated_delta conv", torch.float32, 2)
    _req(a_log, "gated_delta a_log", torch.float32, 1)
    _req(dt_bias, "gated_delta dt_bias", torch.float32, 1)
    taps = conv_w.shape[1]
    if conv_w.shape[0] != C or a_log.numel() != H or dt_bias.numel() != H:
        raise _lib.KernelError(f"gated_delta: conv {tuple(conv_w.shape)}, {a_log.numel()} / {dt_bias.numel()} decay terms "
                               f"for {C} channels and {H} heads")
    row = _state_rows(state, "gated_delta state")
    tail = H * E * D
    if tail + (taps - 1) * C > row:
        raise _lib.KernelError(f"gated_delta: state rows of {row} do not hold {H} x {E} x {D} and {taps - 1} x {C}")
    if batch.num_tokens != T:
        raise _lib.KernelError(f"gated_delta: {T} rows for a step of {batch.num_tokens} tokens")
    pre = torch.empty(T, C + 2 * H, dtype=torch.float32, device=proj.device)
    o = torch.empty(T, H * E, dtype=torch.float32, device=proj.device)
    if T == 0:
        return o
    L = _lib.load()
    stream = _stream()
    _lib.check(L.tff_gdelta_prep(proj.data_ptr(), ldp, conv_w.data_ptr(), taps, a_log.data_ptr(), dt_bias.data_ptr(),
                                 state.data_ptr(), row, tail, batch.token_req.data_ptr(), batch.cu_tokens.data_ptr(),
                                 batch.state_slots.data_ptr(), pre.data_ptr(), T, H, G, D, E, stream))
    _lib.check(L.tff_gdelta_recurrence(pre.data_ptr(), proj.data_ptr(), ldp, state.data_ptr(), row, tail, taps,
                                       batch.cu_tokens.data_ptr(), batch.state_slots.data_ptr(), o.data_ptr(),
                                       batch.num_reqs, H, G, D, E, int(getattr(batch, "max_new_tokens", 0) or 0), stream))
    return o


def head_norm_silu_gate(o: torch.Tensor, g: torch.Tensor, weight: torch.Tensor, eps: float, H: int, E: int,
                        out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """``out[:, h E + e] = o[:, h, e] / sqrt(mean over the head of o^2 + eps) * weight[e] * silu(g) * scale`` for o
    float32 [T, H E], g float32 [T, >= H E] and out [T, >= H E] (rows of g and out may be strided)."""
    _req(o, "head_norm_silu_gate o", torch.float32, 2)
    _req(weight, "head_norm_silu_gate weight", torch.float32, 1)
    T = o.shape[0]
    if o.shape[1] != H * E or weight.numel() != E or g.shape[0] != T or out.shape[0] != T:
        raise _lib.KernelError("head_norm_silu_gate: o must be [T, heads * vdim], the weight [vdim]")
    g_row = _rows2(g, "head_norm_silu_gate g", torch.float32, H * E)
    out_row = _rows2(out, "head_norm_silu_gate out", out.dtype, H * E)
    _lib.check(_lib.load().tff_head_norm_silu_gate(o.data_ptr(), g.data_ptr(), g_row, weight.data_ptr(), float(eps),
                                                   float(scale), out.data_ptr(), out_row, T, H, E, dtype_code(out.dtype),
                                                   _stream()))
    return out


def sigmoid_gate_heads(o: torch.Tensor, o_head: int, g: torch.Tensor, H: int, E: int, out: torch.Tensor,
                       scale: float = 1.0) -> torch.Tensor:
    """``out[:, h E + e] = o[:, h o_head + e] * sigmoid(g[:, h E + e]) * scale``: the first E elements of every head
    of o (heads ``o_head`` apart) times a gate; rows of all three may be strided."""
    T = o.shape[0]
    o_row = _rows2(o, "sigmoid_gate_heads o", o.dtype, H * o_head)
    g_row = _rows2(g, "sigmoid_gate_heads g", o.dtype, H * E)
    out_row = _rows2(out, "sigmoid_gate_heads out", o.dtype, H * E)
    if g.shape[0] != T or out.shape[0] != T or o_head < E:
        raise _lib.KernelError("sigmoid_gate_heads: o, g and out must have one row per token")
    _lib.check(_lib.load().tff_sigmoid_gate_heads(o.data_ptr(), o_row, int(o_head), g.data_ptr(), g_row, float(scale),
                                                  out.data_ptr(), out_row, T, H, E, dtype_code(o.dtype), _stream()))
    return out


def add_dyt(resid: torch.Tensor, delta, alpha: float, weight: torch.Tensor, bias: torch.Tensor,
            out_dtype: torch.dtype, rows: torch.Tensor | None = None) -> torch.Tensor:
    """``resid += delta`` (``delta``: None, what a mixer or feed-forward returned, or :class:`PendingTerms`; not
    added when ``rows`` is given) and the norm without statistics of the sum, tanh(alpha v) * weight + bias element
    by element; with ``rows`` (int32) the norm of those rows only, ``resid`` untouched."""
    _req(resid, "add_dyt resid", torch.float32, 2)
    H = resid.shape[1]
    for w, nm in ((weight, "weight"), (bias, "bias")):
        _req(w, f"add_dyt {nm}", torch.float32, 1)
        if w.numel() != H:
            raise _lib.KernelError(f"add_dyt: {nm} has {w.numel()} elements, rows have {H}")
    if isinstance(delta, PendingProduct) and rows is None and out_dtype == torch.bfloat16 \
            and tuple(delta.shape) == tuple(resid.shape):
        # a product of a few rows that has not run: it runs with the sum and the norm in its epilogue
        p = delta
        M, K = p.x.shape
        out = torch.empty(M, H, dtype=torch.bfloat16, device=resid.device)
        _lib.check(_lib.load().tff_gemm_residual_dyt(p.x.data_ptr(), p.weight.data_ptr(), M, H, K,
                                                     p.x.stride(0) if M > 1 else K, resid.data_ptr(), float(alpha),
                                                     weight.data_ptr(), bias.data_ptr(), out.data_ptr(), _stream()))
        return out
    terms = delta.terms if isinstance(delta, PendingTerms) else ([] if delta is None else [delta])
    d = [_planes_of(t, resid.shape, "add_dyt term") for t in terms] + [(None, 0, 0)] * 2
    if rows is not None:
        _req(rows, "add_dyt rows", torch.int32, 1)
        n = rows.numel()
    else:
        n = resid.shape[0]
    out = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    _lib.check(_lib.load().tff_add_dyt(resid.data_ptr(), _ptr(d[0][0]), d[0][1], d[0][2], _ptr(d[1][0]), d[1][1], d[1][2],
                                       float(alpha), weight.data_ptr(), bias.data_ptr(), out.data_ptr(), _ptr(rows), n, H,
                                       dtype_code(out_dtype), _stream()))
    return out


def diff_qkv_store(proj: torch.Tensor, H: int, G: int, D: int, E: int, q_bias, k_bias, v_bias,
                   cos_sin: torch.Tensor | None, pairing: int, positions: torch.Tensor, kv) -> torch.Tensor:
    """The projections of a differential attention, ``proj`` float32 [T, >= 2 H D + 2 G D + G E] = q [H, 2, D],
    k [G, 2, D], v [G, E] (rows may be strided), with their biases (float32, or None) added and the first
    ``2 * cos_sin.shape[1]`` elements of every map of q and k rotated.  Returns the queries [T, 2 H P] in the
    cache's type, P the cache's head size: head 2 h + m holds map m at elements m D .. m D + D - 1 and zeros
    elsewhere.  The token's key row [k_g0 | k_g1 | 0 ..] and value row [v_g | 0 ..] go to its slot of ``kv``."""
    cols = 2 * H * D + 2 * G * D + G * E
    T = proj.shape[0]
    row = _rows2(proj, "diff_qkv_store proj", torch.float32, cols)
    k_cache, v_cache = kv.k_cache, kv.v_cache
    _req(k_cache, "k cache", ndim=4)
    _req(v_cache, "v cache", k_cache.dtype, 4)
    P = k_cache.shape[3]
    _check_cache(k_cache, v_cache, G, P, "diff_qkv_store")
    if P < 2 * D or P < E:
        raise _lib.KernelError(f"diff_qkv_store: a cache head of {P} does not hold two maps of {D} or values of {E}")
    for b, n, nm in ((q_bias, 2 * H * D, "q bias"), (k_bias, 2 * G * D, "k bias"), (v_bias, G * E, "v bias")):
        if b is not None:
            _req(b, nm, torch.float32, 1)
            if b.numel() != n:
                raise _lib.KernelError(f"diff_qkv_store: {nm} of {b.numel()} elements, expected {n}")
    dims, max_pos = 0, 0
    if cos_sin is not None:
        _req(cos_sin, "rotation table", torch.float32, 3)
        max_pos, dims = cos_sin.shape[0], 2 * cos_sin.shape[1]
        if cos_sin.shape[2] != 2 or dims > D:
            raise _lib.KernelError(f"rotation table {tuple(cos_sin.shape)} does not fit a map of {D}")
    _req(positions, "positions", torch.int32, 1)
    _req(kv.slot_mapping, "slot_mapping", torch.int32, 1)
    if positions.numel() < T or kv.slot_mapping.numel() < T:
        raise _lib.KernelError("diff_qkv_store: positions and slot_mapping need one entry per token")
    q = torch.empty(T, 2 * H * P, dtype=k_cache.dtype, device=proj.device)
    _lib.check(_lib.load().tff_diff_qkv_store(
        proj.data_ptr(), row, _ptr(q_bias), _ptr(k_bias), _ptr(v_bias), _ptr(cos_sin), dims, int(pairing), max_pos,
        positions.data_ptr(), kv.slot_mapping.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        k_cache.shape[2], k_cache.shape[0], T, H, G, D, E, P, dtype_code(k_cache.dtype), _stream()))
    return q


def diff_combine(a: torch.Tensor, P: int, gate: torch.Tensor | None, lam: float, eps: float, out_scale: float,
                 H: int, E: int) -> torch.Tensor:
    """``a`` [T, 2 H P]: the outputs of a head's two score maps side by side (E values each at the start of their
    P).  o = a_0 - lam a_1; returns o / sqrt(mean over the head of o^2 + eps) * out_scale * sigmoid(gate), [T, H E]
    in a's type.  ``gate`` float32 [T, >= H E] (rows may be strided) or None."""
    T = a.shape[0]
    a_row = _rows2(a, "diff_combine a", a.dtype, 2 * H * P)
    gate_row = _rows2(gate, "diff_combine gate", torch.float32, H * E) if gate is not None else 0
    if gate is not None and gate.shape[0] != T:
        raise _lib.KernelError("diff_combine: the gate needs one row per token")
    out = torch.empty(T, H * E, dtype=a.dtype, device=a.device)
    _lib.check(_lib.load().tff_diff_combine(a.data_ptr(), a_row, int(P), _ptr(gate), gate_row, float(lam), float(eps),
                                            float(out_scale), out.data_ptr(), H * E, T, H, E, dtype_code(a.dtype), _stream()))
    return out


def swiglu(gate_up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``silu(gate) * up`` for gate_up [T, 2I] = [gate | up]."""
    _req(gate_up, "swiglu input", ndim=2)
    T, two_i = gate_up.shape
    if two_i % 2:
        raise _lib.KernelError("swiglu: odd row width")
    I = two_i // 2
    if out is None:
        out = torch.empty(T, I, dtype=gate_up.dtype, device=gate_up.device)
    L = _lib.load()
    _lib.check(L.tff_swiglu(gate_up.data_ptr(), out.data_ptr(), T, I, dtype_code(gate_up.dtype), _stream()))
    return out


def cast(src: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _req(src, "cast src")
    out = torch.empty(src.shape, dtype=dtype, device=src.device)
    L = _lib.load()
    _lib.check(L.tff_cast(src.data_ptr(), dtype_code(src.dtype), out.data_ptr(), dtype_code(dtype),
                          src.numel(), _stream()))
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Lowest index among the maxima of each row of float32 logits [R, V]."""
    _req(logits, "argmax logits", torch.float32, 2)
    R, V = logits.shape
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    L = _lib.load()
    ws_bytes = L.tff_argmax_workspace_bytes(R, V)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=logits.device) if ws_bytes else None
    _lib.check(L.tff_argmax(logits.data_ptr(), out.data_ptr(), R, V, _ptr(ws), _stream()))
    return out


def repetition_penalty(logits: torch.Tensor, seen: torch.Tensor, cu_seen: torch.Tensor,
                       penalty: torch.Tensor) -> None:
    _req(logits, "repetition_penalty logits", torch.float32, 2)
    R, V = logits.shape
    _req(seen, "seen", torch.int32, 1)
    _req(cu_seen, "cu_seen", torch.int32, 1)
    _req(penalty, "penalty", torch.float32, 1)
    if cu_seen.numel() != R + 1 or penalty.numel() != R:
        raise _lib.KernelError("repetition_penalty: cu_seen needs rows + 1 entries, penalty one per row")
    L = _lib.load()
    _lib.check(L.tff_repetition_penalty(logits.data_ptr(), R, V, seen.data_ptr(), cu_seen.data_ptr(),
                                        penalty.data_ptr(), _stream()))


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           top_k: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
           min_p: torch.Tensor | None = None, return_probs: bool = False):
    """One token per row of float32 logits [R, V]; see the entry point."""
    _req(logits, "sample logits", torch.float32, 2)
    R, V = logits.shape
    _req(temperature, "temperature", torch.float32, 1)
    _req(uniform, "uniform", torch.float32, 1)
    for t, nm, dt in ((top_k, "top_k", torch.int32), (top_p, "top_p", torch.float32),
                      (min_p, "min_p", torch.float32)):
        if t is not None:
            _req(t, nm, dt, 1)
            if t.numel() != R:
                raise _lib.KernelError(f"sample: {nm} needs one entry per row")
    if temperature.numel() != R or uniform.numel() != R:
        raise _lib.KernelError("sample: temperature and uniform need one entry per row")
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    probs = torch.empty(R, V, dtype=torch.float32, device=logits.device) if return_probs else None
    L = _lib.load()
    _lib.check(L.tff_sample(logits.data_ptr(), out.data_ptr(), R, V, temperature.data_ptr(),
                            _ptr(top_k), _ptr(top_p), _ptr(min_p), uniform.data_ptr(), _ptr(probs),
                            _stream()))
    return (out, probs) if return_probs else out


def measure_ceilings(device="cuda:0", gib: float = 4.0, quick: bool = False) -> dict:
    """What this machine gives to kernels that do nothing else: streaming reads
    from HBM into registers (a buffer of ``gib`` GiB, far larger than the
    caches) and back-to-back bfloat16 MFMAs at 1, 2 and 4 waves per SIMD, with
    operands that never change and (``..._varied_operands``) with operands that
    change from one instruction to the next as a real product's do: the matrix
    cores then draw more power and the clock settles lower.  ``quick``: the
    streaming read and the four-wave MFMA figure only (some 50 ms)."""
    L = _lib.load()
    dev = torch.device(device)
    cus = _num_cus(dev)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    buf = torch.empty(int(gib * (1 << 30)) // 4, dtype=torch.int32, device=dev).fill_(1)
    nbytes = buf.numel() * 4

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize(dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize(dev)
        return e0.elapsed_time(e1) / 1e3 / reps

    out = {"compute_units": cus}
    with torch.cuda.device(dev):
        st = _stream()
        t = min(timed(lambda: _lib.check(L.tff_probe_stream_read(buf.data_ptr(), nbytes, sink.data_ptr(), cus * b, st)), 3)
                for b in (8, 16, 32))
        out["stream_read_GBps"] = round(nbytes / t / 1e9, 1)
        iters = 20000
        for waves in ((4,) if quick else (1, 2, 4)):
            t = timed(lambda: _lib.check(L.tff_probe_mfma(sink.data_ptr(), cus * waves, iters, 0, st)), 2)
            out[f"mfma_bf16_TFLOPs_{waves}_waves_per_simd"] = round(cus * waves * 4 * iters * 16 * 16384 / t / 1e12, 1)
        if quick:
            return out
        iters = 100000   # long enough for the clock to settle
        t = timed(lambda: _lib.check(L.tff_probe_mfma(sink.data_ptr(), cus * 4, iters, 1, st)), 2)
        out["mfma_bf16_TFLOPs_varied_operands"] = round(cus * 4 * 4 * iters * 16 * 16384 / t / 1e12, 1)
    return out


OP_TABLE = {
    "embed": embed,
    "add_rmsnorm": add_rmsnorm,
    "rmsnorm": rmsnorm,
    "linear": linear,
    "as_tensor": as_tensor,
    "pack_weight": pack_weight,
    "qk_norm_rope_kv": qk_norm_rope_kv,
    "attention": paged_attention,
    "attention_generic": attention_generic,
    "attention_mfma": attention_mfma,
    "attention_decode_fused": attention_decode_fused,
    "qkv_attention": qkv_attention,
    "swiglu": swiglu,
    "latent_kv_store": latent_kv_store,
    "head_linear": head_linear,
    "scale_add_rmsnorm": scale_add_rmsnorm,
    "gelu": gelu,
    "relu_squared": relu_squared,
    "add_dyt": add_dyt,
    "diff_qkv_store": diff_qkv_store,
    "diff_combine": diff_combine,
    "route_topk": route_topk,
    "routed_experts": routed_experts,
    "cast": cast,
    "argmax": argmax,
    "repetition_penalty": repetition_penalty,
    "sample": sample,
}
