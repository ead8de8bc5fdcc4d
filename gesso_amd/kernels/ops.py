"""Python faces of the HIP kernels: they check shapes and types on the host, then launch.

Every function takes torch tensors that live on the GPU, launches on torch's current stream
and returns its output tensor.  There is no other implementation behind these functions: a
missing library or a refused size raises :class:`~gesso_amd.errors.KernelError`.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long

import torch

from ..errors import KernelError
from . import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _build.load()
    return _lib


def _dt(t: torch.Tensor) -> int:
    d = t.dtype
    if d is torch.bfloat16:
        return BF16
    if d is torch.float32:
        return F32
    raise KernelError(f"kernels take float32 or bfloat16, got {d}")


def _p(t):
    """A tensor's address as the library's entry points take it (their argument types are declared when the library is
    loaded, so a plain integer or None is all a pointer argument needs)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream of the current device as a raw handle (a launch asks for it every time: the short way;
    ``torch.cuda.current_device`` alone costs a microsecond a call, and a step of prompt portions asks 150 times)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _check(rc: int):
    if rc != 0:
        raise KernelError(lib().gs_last_error().decode())


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*ts):
    # (the messages are made only when a check fails: these run before every launch)
    for t in ts:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise KernelError("kernel operands must live on the GPU" if not t.is_cuda else "kernel operands must be contiguous")


def _i32(t, n=None, what="index"):
    if t.dtype != torch.int32:
        raise KernelError(f"{what} must be int32, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what} holds {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------- tiled rows

class TiledRows:
    """Rows of bfloat16 that feed a weight-streaming product, kept in the order the matrix cores take them.

    ``(M, K)`` with K a multiple of 32; the buffer holds, for each step of 32 columns and each tile of 16 rows,
    64 lanes x 16 bytes: lane ``l`` has row ``l % 16``, columns ``8 (l / 16) ... + 7`` of the step.  A product reads
    such a tile with one contiguous kilobyte per wavefront instead of sixteen pieces of rows.  Kernels that write
    rows for a product (embedding, the SwiGLU, convolution and residual epilogues, decode attention) write this
    order when handed one of these; the products read it.  ``rows()`` gives the ordinary tensor.
    """

    __slots__ = ("buf", "shape", "dtype", "device")

    def __init__(self, M: int, K: int, device):
        _need(K % 32 == 0, f"tiled rows are a multiple of 32 wide, not {K}")
        self.buf = torch.empty(((M + 15) // 16) * 16 * K, dtype=torch.bfloat16, device=device)
        self.shape = (M, K)
        self.dtype = torch.bfloat16
        self.device = self.buf.device

    @staticmethod
    def fits(K: int) -> bool:
        return K % 32 == 0

    @classmethod
    def of(cls, x: torch.Tensor) -> "TiledRows":
        """The tiled copy of a bfloat16 tensor ``(M, K)``."""
        _need(x.dim() == 2 and x.dtype == torch.bfloat16 and x.stride(1) == 1, "tiled rows are made from bfloat16 (M, K)")
        M, K = x.shape
        t = cls(M, K, x.device)
        t.buf.zero_()
        _check(lib().gs_retile_rows(_p(x), _p(t.buf), c_int(M), c_int(K), c_int(x.stride(0) if M > 1 else K), c_int(1),
                                    _stream()))
        return t

    def rows(self) -> torch.Tensor:
        M, K = self.shape
        out = torch.empty((M, K), dtype=torch.bfloat16, device=self.device)
        _check(lib().gs_retile_rows(_p(self.buf), _p(out), c_int(M), c_int(K), c_int(K), c_int(0), _stream()))
        return out


def _rows_out(out, M, N, device, dtype=torch.bfloat16):
    """An output of rows ``(M, N)``: a tensor, or tiled rows when ``out`` is True (made here) or a TiledRows."""
    if out is True:
        out = TiledRows(M, N, device)
    if isinstance(out, TiledRows):
        _need(out.shape == (M, N), f"tiled rows of shape {out.shape}, expected {(M, N)}")
        return out, out.buf, 1
    if out is None or out is False:
        out = torch.empty((M, N), dtype=dtype, device=device)
    return out, out, 0


# ---------------------------------------------------------------------- elementwise

def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor = None, ssq: torch.Tensor = None,
          next_weight: torch.Tensor = None, xs: torch.Tensor = None, scale: float = 1.0) -> torch.Tensor:
    """``out[t] = table[ids[t]] * scale`` as float32 ``(T, H)``; with ``ssq (T, 1)`` also each row's sum of squares;
    with ``next_weight (H,)`` and ``xs (T, H)`` bfloat16 also ``xs = out * next_weight``."""
    _dev(ids, table, out, ssq, next_weight, None if isinstance(xs, TiledRows) else xs)
    _i32(ids, what="token ids")
    V, H = table.shape
    T = ids.numel()
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (T, H), "embed: out must be float32 (T, H)")
    _need(ssq is None or (ssq.dtype == torch.float32 and ssq.numel() == T), "embed: ssq must be float32 (T, 1)")
    _need((next_weight is None) == (xs is None), "embed: next_weight and xs come together")
    xs_buf, xs_tiled = xs, 0
    if xs is not None:
        if isinstance(xs, TiledRows):
            xs_buf, xs_tiled = xs.buf, 1
        _need(next_weight.dtype == torch.float32 and next_weight.shape == (H,) and xs.dtype == torch.bfloat16
              and tuple(xs.shape) == (T, H) and xs_buf.is_contiguous(), "embed: next_weight float32 (H,), xs bfloat16 (T, H)")
    _check(lib().gs_embed(_p(ids), _p(table), _dt(table), _p(out), _p(ssq), _p(next_weight), _p(xs_buf), c_int(xs_tiled),
                          c_int(T), c_int(H), c_int(V), c_float(scale), _stream()))
    return out


def add_rmsnorm(res: torch.Tensor, delta, weight: torch.Tensor, eps: float, out_dtype, rows=None,
                out: torch.Tensor = None) -> torch.Tensor:
    """``res += delta`` (when given and no ``rows``), then ``out = rmsnorm(res) * weight``.

    ``rows`` (int32) picks source rows; then ``res`` is not written.
    """
    f32 = torch.float32
    if not (res.is_cuda and res.is_contiguous() and res.dtype is f32 and res.dim() == 2):
        raise KernelError("add_rmsnorm: the residual stream is float32 (T, H), contiguous, on the GPU")
    T, H = res.shape
    if not (weight.is_cuda and weight.dtype is f32 and weight.shape == (H,) and weight.is_contiguous()):
        raise KernelError("add_rmsnorm: weight must be float32 (H,)")
    if delta is not None and not (delta.is_cuda and delta.is_contiguous() and delta.shape == res.shape):
        raise KernelError("add_rmsnorm: delta must have the stream's shape")
    n_out = T
    if rows is not None:
        _dev(rows)
        _i32(rows, what="rows")
        n_out = rows.numel()
    if out is None:
        out = torch.empty((n_out, H), dtype=out_dtype, device=res.device)
    elif not (out.is_cuda and out.is_contiguous() and out.shape == (n_out, H) and out.dtype == out_dtype):
        raise KernelError("add_rmsnorm: out has the wrong shape or type")
    rc = lib().gs_add_rmsnorm(res.data_ptr(), None if delta is None else delta.data_ptr(),
                              _dt(delta) if delta is not None else _dt(out), weight.data_ptr(), eps, out.data_ptr(),
                              _dt(out), None if rows is None else rows.data_ptr(), n_out, H, _stream())
    if rc != 0:
        _check(rc)
    return out


def residual_add(res: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _dev(res, delta)
    _need(res.dtype == torch.float32 and delta.shape == res.shape, "residual_add: shapes or types differ")
    _check(lib().gs_residual_add(_p(res), _p(delta), c_int(_dt(delta)), c_long(res.numel()), _stream()))
    return res


def swiglu(x: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """``x (T, 2F)`` = gate | up  ->  ``silu(gate) * up (T, F)``."""
    if not (x.is_cuda and x.is_contiguous() and x.dim() == 2):
        raise KernelError("swiglu: rows (T, 2F), contiguous, on the GPU")
    T, F2 = x.shape
    if F2 % 2:
        raise KernelError("swiglu: the input holds gate and up side by side")
    F = F2 // 2
    if out is None:
        out = torch.empty((T, F), dtype=x.dtype, device=x.device)
    elif not (out.is_cuda and out.is_contiguous() and out.shape == (T, F) and out.dtype == x.dtype):
        raise KernelError("swiglu: out has the wrong shape or type")
    rc = lib().gs_swiglu(x.data_ptr(), out.data_ptr(), _dt(x), T, F, _stream())
    if rc != 0:
        _check(rc)
    return out


def add_bias(y: torch.Tensor, bias: torch.Tensor, out_dtype=None, out: torch.Tensor = None) -> torch.Tensor:
    """``y + bias`` row by row: ``y`` float32 ``(M, N)`` contiguous (a product's sums), ``bias`` float32 ``(N,)``;
    the result in ``out_dtype``, rounded once."""
    _dev(y, bias)
    _need(out is None or out.is_cuda, "kernel operands must live on the GPU")
    _need(y.dtype == torch.float32 and y.dim() == 2 and y.is_contiguous(), "add_bias: y must be float32 (M, N), contiguous")
    M, N = y.shape
    _need(bias.dtype == torch.float32 and bias.shape == (N,) and bias.is_contiguous(), "add_bias: bias must be float32 (N,)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or torch.float32, device=y.device)
    _need(out.shape == (M, N) and out.stride(1) == 1 and out.dtype in (torch.float32, torch.bfloat16),
          "add_bias: out has the wrong shape or type")
    _check(lib().gs_add_bias(_p(y), _p(bias), _p(out), c_int(_dt(out)), c_int(M), c_int(N),
                             c_long(out.stride(0) if M > 1 else N), _stream()))
    return out


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """``cap * tanh(logits / cap)`` in place (float32)."""
    _dev(logits)
    _need(logits.dtype == torch.float32, "softcap takes float32 logits")
    _check(lib().gs_softcap(_p(logits), c_float(cap), c_long(logits.numel()), _stream()))
    return logits


def stream_read(buf: torch.Tensor, blocks: int = 2048, contiguous: bool = True, sink: torch.Tensor = None) -> None:
    """Read ``buf`` once from memory with a plain streaming kernel (a measurement, see ``bench.py``): each block its
    own contiguous share, or the grid sweeping the buffer together."""
    _dev(buf, sink)
    nbytes = buf.numel() * buf.element_size()
    if sink is None:
        sink = torch.zeros(blocks, dtype=torch.int32, device=buf.device)
    _need(sink.dtype == torch.int32 and sink.numel() >= blocks, "stream_read: sink holds an int32 per block")
    _check(lib().gs_stream_read(_p(buf), c_long(nbytes), _p(sink), c_int(blocks), c_int(1 if contiguous else 0), _stream()))


FILL_MAX = 65535


def fill_rows(pool: torch.Tensor, ids: torch.Tensor, value: float, planes: int = 1) -> None:
    """``pool[..., id, ...] = value`` for each id in ``ids`` (int32): ``pool`` is ``(planes..., rows, *row shape)`` with
    ``planes`` leading axes flattened into one (1: ``(rows, ...)``), float32 or bfloat16.  A fresh state slot gets its
    initial value this way; with poisoning on, so do the pages and slots a request gave back (NaN)."""
    _dev(pool, ids)
    _i32(ids, what="row ids")
    lead = pool.shape[:planes - 1] if planes > 1 else ()
    outer = 1
    for n in lead:
        outer *= n
    rows = pool.shape[len(lead)]
    row = pool[(0,) * (len(lead) + 1)].numel() if pool.numel() else 0
    _need(outer <= FILL_MAX, f"fill_rows: {outer} planes are more than a launch takes ({FILL_MAX})")
    for at in range(0, ids.numel(), FILL_MAX):            # a launch takes 65,535 ids: many freed pages go in turns
        part = ids[at:at + FILL_MAX]
        _check(lib().gs_fill_rows(_p(pool), c_int(_dt(pool)), _p(part), c_int(part.numel()), c_long(row), c_int(outer),
                                  c_long(rows), c_float(value), _stream()))


# ---------------------------------------------------------------------- short convolution

def short_conv(bcx, taps, bias, state, seq_of_token, q_start, slots, nseq: int, all_single: bool,
               out: torch.Tensor = None) -> torch.Tensor:
    """Gated short convolution over segments; ``state (num_slots, H, W-1)`` is read and advanced."""
    _dev(bcx, taps, bias, state, seq_of_token, q_start, slots, out)
    T, H3 = bcx.shape
    _need(H3 % 3 == 0, "short_conv: bcx holds B, C, X side by side")
    H = H3 // 3
    W = taps.shape[1]
    _need(taps.dtype == torch.float32 and taps.shape == (H, W), "short_conv: taps must be float32 (H, W)")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (H,)), "short_conv: bias must be float32 (H,)")
    _need(state.dtype == torch.float32 and state.dim() == 3 and state.shape[1:] == (H, W - 1),
          "short_conv: state must be float32 (slots, H, W-1)")
    _i32(seq_of_token, T, "seq_of_token")
    _i32(q_start, nseq + 1, "q_start")
    _i32(slots, nseq, "slots")
    if out is None:
        out = torch.empty((T, H), dtype=bcx.dtype, device=bcx.device)
    _need(out.shape == (T, H) and out.dtype == bcx.dtype, "short_conv: out has the wrong shape or type")
    _check(lib().gs_short_conv(_p(bcx), c_int(_dt(bcx)), _p(taps), _p(bias), _p(state), _p(seq_of_token),
                               _p(q_start), _p(slots), _p(out), c_int(T), c_int(nseq), c_int(H), c_int(W),
                               c_int(1 if all_single else 0), _stream()))
    return out


# ---------------------------------------------------------------------- attention

ROPE_LAYOUTS = ("half", "interleaved")


def qknorm_rope_kv(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, positions, seq_of_token, block_table,
                   page_size, kcache, vcache, nh, nkv, d, write_kv=True, layout: str = "half") -> None:
    """Head norm and rotation of q (in place) and k; k and v written into the pages.  ``layout``: which features
    form a rotation pair, ``"half"`` (i, i + rotary_dim/2) or ``"interleaved"`` (2i, 2i + 1)."""
    _need(layout in ROPE_LAYOUTS, f"qknorm_rope_kv: pairs are laid out 'half' or 'interleaved', not {layout!r}")
    _dev(qkv, q_weight, k_weight, cos, sin, positions, seq_of_token, block_table, kcache, vcache)
    T = qkv.shape[0]
    _need(qkv.shape == (T, (nh + 2 * nkv) * d), "qknorm_rope_kv: qkv must be (T, (nh + 2 nkv) d)")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.shape == (d,)), "qknorm_rope_kv: head norm weight must be float32 (d,)")
    max_pos = 0
    if rotary_dim:
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.dim() == 2 and cos.shape[1] == rotary_dim // 2, "qknorm_rope_kv: tables must be float32 (P, rotary_dim/2)")
        max_pos = cos.shape[0]
    _i32(positions, T, "positions")
    _i32(seq_of_token, T, "seq_of_token")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    _need(kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype, "cache and activations differ in type")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _check(lib().gs_qknorm_rope_kv(_p(qkv), c_int(_dt(qkv)), _p(q_weight), _p(k_weight), c_float(eps), _p(cos),
                                   _p(sin), c_int(rotary_dim), c_int(1 if layout == "interleaved" else 0), c_int(max_pos),
                                   _p(positions), _p(seq_of_token),
                                   _p(block_table), c_int(block_table.shape[1]), c_int(page_size), _p(kcache),
                                   _p(vcache), c_int(T), c_int(nh), c_int(nkv), c_int(d),
                                   c_int(1 if write_kv else 0), _stream()))


def attention_generic(q, q_stride, kcache, vcache, positions, seq_of_token, block_table, page_size, window, scale,
                      nh, nkv, d, ntok, out: torch.Tensor = None) -> torch.Tensor:
    """Causal GQA over the paged cache, any sizes; ``q`` rows are ``q_stride`` apart."""
    _dev(q, kcache, vcache, positions, seq_of_token, block_table, out)
    _need(q.numel() >= (ntok - 1) * q_stride + nh * d if ntok else True, "attention: q is too small")
    _need(kcache.dtype == q.dtype and vcache.dtype == q.dtype, "cache and activations differ in type")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, ntok, "positions")
    _i32(seq_of_token, ntok, "seq_of_token")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, nh * d), dtype=q.dtype, device=q.device)
    _need(out.shape == (ntok, nh * d) and out.dtype == q.dtype, "attention: out has the wrong shape or type")
    _check(lib().gs_attention_generic(_p(q), c_int(q_stride), _p(kcache), _p(vcache), c_int(_dt(q)), _p(positions),
                                      _p(seq_of_token), _p(block_table), c_int(block_table.shape[1]),
                                      c_int(page_size), c_int(window or 0), c_float(scale), _p(out), c_int(ntok),
                                      c_int(nh), c_int(nkv), c_int(d), _stream()))
    return out


# ---------------------------------------------------------------------- matrix products

def gemm_tiled(x: torch.Tensor, w: torch.Tensor, bias=None, out_dtype=None, out: torch.Tensor = None) -> torch.Tensor:
    """``y = x @ w.T (+ bias)`` by float32 FMAs; any sizes, any mix of float32/bfloat16 storage."""
    _dev(w, bias, out)
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1, "gemm: x must be (M, K) with unit column stride")
    M, K = x.shape
    N = w.shape[0]
    if w.shape != (N, K):
        raise KernelError(f"gemm: weight is {tuple(w.shape)}, expected ({N}, {K})")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (N,)), "gemm: bias must be float32 (N,)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "gemm: out has the wrong shape")
    ldx = x.stride(0) if M > 1 else K
    if (x.dtype == torch.float32 and w.dtype == torch.float32 and w.is_contiguous()
            and lib().gs_gemv_f32_supports(c_int(M), c_int(K), c_int(ldx), _p(x), _p(w))):
        # few rows: the weights are streamed once, each output summed in an order that depends on K alone
        _check(lib().gs_gemv_f32(_p(x), c_int(ldx), _p(w), _p(bias), _p(out), c_int(_dt(out)),
                                 c_int(out.stride(0) if M > 1 else N), c_int(M), c_int(N), c_int(K), _stream()))
        return out
    _check(lib().gs_gemm_tiled(_p(x), c_int(_dt(x)), c_int(x.stride(0) if M > 1 else K), _p(w), c_int(_dt(w)),
                               _p(bias), _p(out), c_int(_dt(out)), c_int(out.stride(0) if M > 1 else N), c_int(M),
                               c_int(N), c_int(K), _stream()))
    return out


def mfma_ok(x, w: torch.Tensor) -> bool:
    """Whether the matrix-core product for many rows takes these operands (bfloat16, K a multiple of 8, aligned)."""
    return (isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and x.shape[0] > 0 and x.shape[1] % 8 == 0 and x.stride(1) == 1
            and (x.shape[0] <= 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0 and w.is_contiguous()
            and w.data_ptr() % 16 == 0)


def gemm_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype=None, out: torch.Tensor = None, swiglu: bool = False):
    """``x @ w.T`` for many rows on the matrix cores (bfloat16 in, float32 sums, bfloat16 or float32 out); with
    ``swiglu`` the weight holds gate rows then up rows and the result is ``silu(gate) * up``, half as wide."""
    _dev(w, out)
    _need(mfma_ok(x, w), "gemm_mfma: operands must be bfloat16, K a multiple of 8, 16-byte aligned")
    M, K = x.shape
    N = w.shape[0]
    if w.shape != (N, K):
        raise KernelError(f"gemm_mfma: weight is {tuple(w.shape)}, expected ({N}, {K})")
    _need(not swiglu or N % 2 == 0, "gemm_mfma: SwiGLU needs gate and up rows")
    cols = N // 2 if swiglu else N
    if out is None:
        out = torch.empty((M, cols), dtype=out_dtype or torch.bfloat16, device=w.device)
    _need(out.shape == (M, cols) and out.stride(1) == 1, "gemm_mfma: out has the wrong shape")
    _need(not swiglu or out.dtype == torch.bfloat16, "gemm_mfma: the SwiGLU epilogue stores bfloat16")
    _check(lib().gs_gemm_mfma(_p(x), c_int(x.stride(0) if M > 1 else K), _p(w), _p(out), c_int(_dt(out)),
                              c_int(out.stride(0) if M > 1 else cols), c_int(M), c_int(N), c_int(K),
                              c_int(1 if swiglu else 0), _stream()))
    return out


def library_gemm(x: torch.Tensor, w: torch.Tensor, workspace: torch.Tensor, out: torch.Tensor = None, tune: bool = True,
                 checked: bool = False):
    """``x @ w.T`` for many rows by the vendor's library, called directly (bfloat16 in and out, float32 sums).  The
    first call of a shape makes its plan, with ``tune`` by measuring the library's two dozen best guesses on these
    operands (a few milliseconds), else by taking its first choice.
    ``workspace``: device bytes the library's kernels may use.  Not to be recorded into a graph.
    ``checked``: the caller has asked :func:`library_gemm_ok` about ``x`` and ``w`` (and ``out`` is None or fits): the
    operands are not looked at again here (a step of prompt portions makes 64 such calls; the entry point still
    refuses misaligned or missing operands)."""
    bf = torch.bfloat16
    M, K = x.shape
    N = w.shape[0]
    if not checked:
        if not (x.is_cuda and x.dim() == 2 and x.dtype is bf and w.dtype is bf and x.stride(1) == 1 and w.is_cuda
                and w.is_contiguous() and workspace.is_cuda):
            raise KernelError("library_gemm: bfloat16 (M, K) rows and a contiguous bfloat16 weight on the GPU")
        if w.shape != (N, K):
            raise KernelError(f"library_gemm: weight is {tuple(w.shape)}, expected ({N}, {K})")
        if out is not None and not (out.is_cuda and out.shape == (M, N) and out.dtype is bf and out.stride(1) == 1):
            raise KernelError("library_gemm: out is bfloat16 (M, N) on the GPU")
    if out is None:
        out = torch.empty((M, N), dtype=bf, device=w.device)
    rc = lib().gs_library_gemm(x.data_ptr(), x.stride(0) if M > 1 else K, w.data_ptr(), out.data_ptr(),
                               out.stride(0) if M > 1 else N, M, N, K, workspace.data_ptr(),
                               workspace.numel() * workspace.element_size(), 1 if tune else 0, _stream())
    if rc != 0:
        _check(rc)
    return out


def library_gemm_ok(x, w: torch.Tensor) -> bool:
    """Whether :func:`library_gemm` takes these operands (bfloat16 on the GPU, a weight ``(N, K)`` for rows of K, K and
    the row stride multiples of 8, aligned)."""
    bf = torch.bfloat16
    if not (isinstance(x, torch.Tensor) and x.dtype is bf and w.dtype is bf and x.dim() == 2 and w.dim() == 2):
        return False
    M, K = x.shape
    return (M > 0 and K % 8 == 0 and w.shape[1] == K and w.shape[0] % 8 == 0 and x.stride(1) == 1
            and (M <= 1 or x.stride(0) % 8 == 0) and x.is_cuda and w.is_cuda and w.is_contiguous()
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def library_gemm_plan(M: int, N: int, K: int):
    """``(plans kept in all, candidates measured for this shape, the best one's microseconds)``."""
    cand, best = c_int(0), c_float(0.0)
    n = lib().gs_library_gemm_plans(c_int(M), c_int(N), c_int(K), ctypes.byref(cand), ctypes.byref(best))
    return n, cand.value, best.value


# ---------------------------------------------------------------------- sampling

def argmax_rows(logits: torch.Tensor):
    """``(ids int32 (rows,), bad int32 (rows,))``: first maximum per row; bad = a non-finite logit."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: logits are float32 (rows, V)")
    rows, V = logits.shape
    ids = torch.empty(rows, dtype=torch.int32, device=logits.device)
    bad = torch.empty(rows, dtype=torch.int32, device=logits.device)
    _check(lib().gs_argmax_rows(_p(logits), c_int(rows), c_int(V), _p(ids), _p(bad), _stream()))
    return ids, bad


def sample_temperature(logits: torch.Tensor, temperature: torch.Tensor, u: torch.Tensor):
    """One id per row from ``softmax(logits / temperature)`` by inverse CDF at ``u`` (float64 each)."""
    return choose_rows(logits, temperature, torch.ones_like(temperature), u)


def sample_top_p(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, u: torch.Tensor):
    """Nucleus sampling: one id per row from the shortest descending-weight prefix whose mass reaches ``top_p``."""
    return choose_rows(logits, temperature, top_p, u)


def choose_rows(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, u: torch.Tensor):
    """One id per row, each row in its own manner: ``temperature <= 0`` greedy, else a draw at ``u`` from the whole row
    or (``top_p < 1``) from its nucleus; float64 ``(rows,)`` each.  ``(ids, bad)`` int32 as :func:`argmax_rows`.  The
    weights are made by many blocks a row (the kernels of the decode loop's choice)."""
    _dev(logits, temperature, top_p, u)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "choose: logits are float32 (rows, V)")
    rows, V = logits.shape
    for name, t in (("temperature", temperature), ("top_p", top_p), ("u", u)):
        _need(t.dtype == torch.float64 and t.numel() == rows, f"choose: {name} is float64 (rows,)")
    dev = logits.device
    zeros = torch.zeros((5, rows), dtype=torch.int32, device=dev)      # counter, next id, position, key count, live
    out = torch.empty((2, 1, rows), dtype=torch.int32, device=dev)
    nucleus = bool((top_p < 1).any())
    wide = (torch.empty(rows * choice_parts(V), dtype=torch.float64, device=dev), torch.empty(rows, dtype=torch.int32, device=dev),
            torch.empty(rows, dtype=torch.int32, device=dev), torch.empty(rows * choice_hist(), dtype=torch.int64, device=dev))
    decode_choose(logits, temperature, u.reshape(1, rows), zeros[0], zeros[1], out[0], out[1], zeros[2], zeros[3], zeros[4],
                  wide, top_p=top_p if nucleus else None,
                  wbuf=torch.empty(rows * V, dtype=torch.float64, device=dev) if nucleus else None)
    return out[0, 0], out[1, 0]


# ---------------------------------------------------------------------- decoding

SKINNY_MAX_ROWS = 64


def skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel takes this product (few rows, bfloat16, aligned rows)."""
    if isinstance(x, TiledRows):
        return (w.dtype == torch.bfloat16 and x.shape[0] <= SKINNY_MAX_ROWS and w.is_contiguous()
                and w.data_ptr() % 16 == 0)
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and x.shape[0] <= SKINNY_MAX_ROWS
            and x.shape[1] % 8 == 0 and x.stride(1) == 1 and (x.shape[0] <= 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0 and w.is_contiguous() and w.data_ptr() % 16 == 0)


class LazyNorm:
    """An RMSNorm not yet applied: the float32 stream, its rows' sums of squares as partial sums, weight and eps.

    The weight-streaming products take it in place of a tensor and norm on the fly; ``materialize``
    runs a light norm kernel for everything else.  ``xs``, when given, holds ``res * weight`` in bfloat16,
    written by whatever last added to the stream: then a product reads ``xs`` and multiplies its result by the
    row's inverse root mean square, and the norm costs nothing of its own.
    """

    __slots__ = ("res", "ssq", "weight", "eps", "dtype", "xs", "ready")

    def __init__(self, res, ssq, weight, eps, dtype, xs=None, ready=None):
        self.res, self.ssq, self.weight, self.eps, self.dtype, self.xs = res, ssq, weight, eps, dtype, xs
        self.ready = ready            # the normed rows themselves, where whatever wrote the stream last made them

    @property
    def shape(self):
        return self.res.shape

    def materialize(self) -> torch.Tensor:
        """The normed rows as a tensor; the sums of squares are at hand, so one light pass does it."""
        if self.ready is not None:
            return self.ready
        T, H = self.res.shape
        out = torch.empty((T, H), dtype=self.dtype, device=self.res.device)
        _check(lib().gs_norm_from_ssq(_p(self.res), _p(self.ssq), c_int(self.ssq.shape[1]), _p(self.weight),
                                      c_float(self.eps), _p(out), c_int(_dt(out)), c_int(T), c_int(H), _stream()))
        return out


def lazy_ok(x, w: torch.Tensor) -> bool:
    return (isinstance(x, LazyNorm) and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and x.res.shape[0] <= SKINNY_MAX_ROWS and x.res.shape[1] % 8 == 0 and x.res.is_contiguous()
            and w.is_contiguous() and w.data_ptr() % 16 == 0 and x.res.data_ptr() % 16 == 0)


def _lazy_args(x):
    if isinstance(x, LazyNorm):
        if x.xs is not None:
            return _x_args(x.xs) + (None, _p(x.ssq), c_int(x.ssq.shape[1]), None, c_float(x.eps))
        return (None, c_int(x.res.shape[1]), c_int(0), _p(x.res), _p(x.ssq), c_int(x.ssq.shape[1]), _p(x.weight),
                c_float(x.eps))
    return _x_args(x) + (None, None, c_int(0), None, c_float(0.0))


def _x_args(x):
    """Pointer, row stride and layout flag of a product's rows."""
    M, K = x.shape
    if isinstance(x, TiledRows):
        return (_p(x.buf), c_int(K), c_int(1))
    return (_p(x), c_int(x.stride(0) if M > 1 else K), c_int(0))


def tile_major(w: torch.Tensor) -> torch.Tensor:
    """The tile-major copy of a bfloat16 weight ``(N, K)``, N a multiple of 16 and K of 32, that the
    weight-streaming kernels read fastest: each 16 x 32 tile as 64 lanes x 16 bytes, in the MFMA operand's order."""
    _dev(w)
    N, K = w.shape
    _need(w.dtype == torch.bfloat16 and N % 16 == 0 and K % 32 == 0, "tile_major: bfloat16 (N, K), N % 16 == 0, K % 32 == 0")
    out = torch.empty_like(w)
    _check(lib().gs_tile_major(_p(w), _p(out), c_int(N), c_int(K), _stream()))
    return out


def gemm_skinny(x, w: torch.Tensor, out_dtype=None, out=None, swiglu: bool = False, wt=None):
    """``x @ w.T`` for at most 64 rows, streaming the weights once; optionally ``silu(gate) * up`` of the result.

    ``x`` is a bfloat16 tensor, :class:`TiledRows` or a :class:`LazyNorm`.  With ``swiglu`` the weight holds gate
    rows then up rows and the output is half as wide, and ``out`` may be True or a :class:`TiledRows` for tiled rows.
    """
    _dev(w, out if isinstance(out, torch.Tensor) else None)
    lazy = isinstance(x, LazyNorm)
    _need(lazy_ok(x, w) if lazy else skinny_ok(x, w),
          "gemm_skinny: operands must be bfloat16, at most 64 rows, K a multiple of 8, aligned")
    M, K = x.shape
    N = w.shape[0]
    if w.shape != (N, K):
        raise KernelError(f"gemm_skinny: weight is {tuple(w.shape)}, expected ({N}, {K})")
    cols = N // 2 if swiglu else N
    out, buf, tiled = _rows_out(out, M, cols, w.device, out_dtype or torch.bfloat16)
    _need(not tiled or swiglu, "gemm_skinny: only the SwiGLU epilogue writes tiled rows")
    _need(tiled or (out.shape == (M, cols) and out.stride(1) == 1), "gemm_skinny: out has the wrong shape")
    _check(lib().gs_gemm_skinny(*_lazy_args(x), _p(w), _p(wt), _p(buf), c_int(_dt(out)),
                                c_int(cols if tiled or M <= 1 else out.stride(0)), c_int(M), c_int(N), c_int(K),
                                c_int(1 if swiglu else 0), c_int(tiled), _stream()))
    return out


def gemm_skinny_residual(x: torch.Tensor, w: torch.Tensor, res: torch.Tensor, wt=None, next_weight=None,
                         xs: torch.Tensor = None) -> torch.Tensor:
    """``res += x @ w.T`` in place (float32); returns the new rows' sums of squares as partial sums ``(M, nb)``.
    With ``next_weight (N,)`` and ``xs (M, N)`` bfloat16 also ``xs = res * next_weight``."""
    _dev(w, res, next_weight, None if isinstance(xs, TiledRows) else xs)
    _need(skinny_ok(x, w), "gemm_skinny_residual: operands must be bfloat16, at most 64 rows, K a multiple of 8, aligned")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape == (N, K) and res.shape == (M, N) and res.dtype == torch.float32, "gemm_skinny_residual: shapes")
    nb = lib().gs_gemm_skinny_residual_blocks(c_int(N), c_int(0 if wt is None else 1))
    ssq = torch.empty((M, nb), dtype=torch.float32, device=res.device)
    _need((next_weight is None) == (xs is None), "gemm_skinny_residual: next_weight and xs come together")
    xs_buf, xs_tiled = xs, 0
    if xs is not None:
        if isinstance(xs, TiledRows):
            xs_buf, xs_tiled = xs.buf, 1
        _need(next_weight.dtype == torch.float32 and next_weight.shape == (N,) and xs.dtype == torch.bfloat16
              and tuple(xs.shape) == (M, N) and xs_buf.is_contiguous(), "gemm_skinny_residual: next_weight float32 (N,), xs bfloat16 (M, N)")
    _check(lib().gs_gemm_skinny_residual(*_x_args(x), _p(w), _p(wt), _p(res), _p(ssq), _p(next_weight), _p(xs_buf),
                                         c_int(xs_tiled), c_int(M), c_int(N), c_int(K), _stream()))
    return ssq


def gemm_skinny_residual_parts(x, w: torch.Tensor, res: torch.Tensor, parts: int, wt=None,
                               next_weight=None, eps: float = 0.0, out_dtype=None, tiled: bool = False):
    """``res += x @ w.T`` for up to 64 rows in two kernels: partial sums over ``parts`` parts of K from many blocks,
    then one pass that adds them to the stream.  Returns ``(ssq (M, 1), normed)``: the new rows' sums of squares and,
    with ``next_weight``, the rows normed with that weight and ``eps`` (else None; as :class:`TiledRows` with ``tiled``)."""
    _dev(w, res, next_weight)
    _need(skinny_ok(x, w), "gemm_skinny_residual_parts: operands must be bfloat16, at most 64 rows, K a multiple of 8, aligned")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape == (N, K) and res.shape == (M, N) and res.dtype == torch.float32 and res.is_contiguous(),
          "gemm_skinny_residual_parts: shapes")
    _need(1 <= parts <= 64, "gemm_skinny_residual_parts: 1 to 64 parts")
    part = torch.empty((parts, M, N), dtype=torch.float32, device=res.device)
    _check(lib().gs_gemm_skinny_parts(*_x_args(x), _p(w), _p(wt), _p(part), c_int(parts), c_int(M), c_int(N), c_int(K),
                                      _stream()))
    ssq = torch.empty((M, 1), dtype=torch.float32, device=res.device)
    normed = None
    if next_weight is not None:
        _need(next_weight.dtype == torch.float32 and next_weight.shape == (N,), "next_weight must be float32 (N,)")
        normed, nbuf, ntiled = _rows_out(bool(tiled), M, N, res.device, out_dtype or torch.bfloat16)
    else:
        nbuf, ntiled = None, 0
    _check(lib().gs_residual_from_parts(_p(part), c_int(parts), _p(res), _p(ssq), _p(next_weight), c_float(eps),
                                        _p(nbuf), c_int(_dt(normed) if normed is not None else 1), c_int(ntiled),
                                        c_int(M), c_int(N), _stream()))
    return ssq, normed


def gemm_skinny_conv(x, w_in, taps, bias, state, slots, wt=None, tiled: bool = False):
    """A decode step's gated short convolution fused into its input product; ``state`` is advanced.
    With ``tiled`` the mixed rows come as :class:`TiledRows`."""
    _dev(w_in, taps, bias, state, slots)
    _need(lazy_ok(x, w_in) if isinstance(x, LazyNorm) else skinny_ok(x, w_in),
          "gemm_skinny_conv: needs bfloat16 rows or a lazy norm, and a bfloat16 weight")
    M, K = x.shape
    H, W = taps.shape
    _need(w_in.shape == (3 * H, K), "gemm_skinny_conv: the input weight must be (3H, K)")
    _need(taps.dtype == torch.float32 and state.dtype == torch.float32 and state.shape[1:] == (H, W - 1),
          "gemm_skinny_conv: taps float32 (H, W), state float32 (slots, H, W-1)")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (H,)), "gemm_skinny_conv: bias float32 (H,)")
    _i32(slots, M, "slots")
    out, buf, otiled = _rows_out(bool(tiled), M, H, w_in.device)
    _check(lib().gs_gemm_skinny_conv(*_lazy_args(x), _p(w_in), _p(wt), _p(taps), _p(bias), _p(state), _p(slots), c_int(W),
                                     _p(buf), c_int(otiled), c_int(M), c_int(H), c_int(K), _stream()))
    return out


def choice_parts(V: int) -> int:
    """Partial sums a row of ``V`` logits has in the many-block form of the decode loop's choice."""
    return int(lib().gs_choice_parts(c_int(V)))


def choice_hist() -> int:
    """64-bit sums a row has in the ready-made histograms of the many-block choice."""
    return int(lib().gs_choice_hist())


def _choice_rows(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live):
    _dev(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "decode_choose: logits are float32 (rows, V)")
    rows, V = logits.shape
    for t in (counter, next_ids, positions, kv_len, live):
        _i32(t, rows)
    for t in (ring, bad_ring):
        _i32(t)
    _need(ring.dim() == 2 and ring.shape[1] == rows and bad_ring.shape == ring.shape, "decode_choose: rings are (steps, rows)")
    return rows, V


def decode_choose_greedy(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live) -> None:
    """The decode loop's choice while every row is greedy, one kernel: per row the first maximum into the loop's buffers
    (``ring[counter[row], row]``, the flag of a non-finite row beside it, the id fed back); then the row's counter counts
    up and a live row moves one position on.  A counter at or beyond the rings' step count writes into their last row
    and marks the step bad."""
    rows, V = _choice_rows(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live)
    _check(lib().gs_decode_choose(_p(logits), c_int(rows), c_int(V), _p(counter), _p(next_ids), _p(ring), _p(bad_ring),
                                  _p(positions), _p(kv_len), _p(live), c_int(ring.shape[0]), _stream()))


def decode_choose(logits, temperature, u, counter, next_ids, ring, bad_ring, positions, kv_len, live, wide, top_p=None,
                  wbuf=None) -> None:
    """The decode loop's choice when rows draw, three kernels (the rows' weights by many blocks: one block weighs a row
    of 65,536 logits in some 40 us).  Per row: greedy (temperature <= 0) or a draw with ``u[counter[row], row]``, from
    the whole row or, where ``top_p[row] < 1``, from its nucleus (``wbuf``: float64 scratch of at least ``rows * V``);
    results and the rows' advance as in :func:`decode_choose_greedy`.

    ``wide``: ``(part, amax, bad0, hist)``, float64 ``rows * choice_parts(V)``, int32 ``rows`` twice and int64
    ``rows * choice_hist()``: scratch."""
    rows, V = _choice_rows(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live)
    _dev(temperature, u, top_p, wbuf)
    _need(temperature.dtype == torch.float64 and temperature.numel() == rows, "decode_choose: temperature float64 (rows,)")
    _need(u.dtype == torch.float64 and u.shape == ring.shape, "decode_choose: u is float64 (steps, rows)")
    _need((top_p is None) == (wbuf is None), "decode_choose: top_p and its scratch come together")
    if top_p is not None:
        _need(top_p.dtype == torch.float64 and top_p.numel() == rows, "decode_choose: top_p float64 (rows,)")
        _need(wbuf.dtype == torch.float64 and wbuf.numel() >= rows * V, "decode_choose: wbuf float64, rows * V at least")
    part, amax, bad0, hist = wide
    _dev(part, amax, bad0, hist)
    _need(part.dtype == torch.float64 and part.numel() >= rows * choice_parts(V), "decode_choose: part float64, rows * choice_parts(V) at least")
    _need(hist.dtype == torch.int64 and hist.numel() >= rows * choice_hist(), "decode_choose: hist int64, rows * choice_hist() at least")
    _i32(amax, rows)
    _i32(bad0, rows)
    _check(lib().gs_decode_choose_wide(_p(logits), c_int(rows), c_int(V), _p(temperature), _p(top_p), _p(wbuf), _p(part),
                                       _p(amax), _p(bad0), _p(hist), _p(u), _p(counter), _p(next_ids), _p(ring), _p(bad_ring),
                                       _p(positions), _p(kv_len), _p(live), c_int(u.shape[0]), _stream()))


def attention_decode_supports(nh: int, nkv: int, d: int) -> bool:
    return bool(lib().gs_attention_decode_supports(c_int(nh), c_int(nkv), c_int(d)))


_decode_ws = {}


def _decode_workspace(device, nseq, nh, nkv, d, nsplit):
    key = (device, nseq, nh, nkv, d, nsplit)
    ws = _decode_ws.get(key)
    if ws is None:
        n = lib().gs_attention_decode_workspace
        n.restype = c_long
        floats = n(c_int(nseq), c_int(nh), c_int(nkv), c_int(d), c_int(nsplit))
        ws = _decode_ws[key] = torch.empty(max(1, floats), dtype=torch.float32, device=device)
    return ws


def attention_decode(q, q_stride, kcache, vcache, positions, block_table, page_size, window, scale, nh, nkv, d, nseq,
                     nsplit: int, out=None):
    """One query per sequence over its paged keys (bfloat16), keys split over ``nsplit`` blocks per key head.
    ``out``: a tensor, or True / a :class:`TiledRows` for tiled rows."""
    _dev(q, kcache, vcache, positions, block_table, out if isinstance(out, torch.Tensor) else None)
    _need(q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_decode takes bfloat16")
    _need(q.numel() >= (nseq - 1) * q_stride + nh * d if nseq else True, "attention_decode: q is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, nseq, "positions")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= nseq,
          "block_table must be int32 (nseq, max_blocks)")
    ws = _decode_workspace(q.device, nseq, nh, nkv, d, nsplit)
    out, buf, tiled = _rows_out(out, nseq, nh * d, q.device, q.dtype)
    _need(tuple(out.shape) == (nseq, nh * d) and out.dtype == q.dtype, "attention_decode: out has the wrong shape or type")
    _check(lib().gs_attention_decode(_p(q), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(block_table),
                                     c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0), c_float(scale),
                                     _p(buf), c_int(tiled), _p(ws), c_int(nseq), c_int(nh), c_int(nkv), c_int(d),
                                     c_int(nsplit), _stream()))
    return out


def attention_decode_raw_supports(nh: int, nkv: int, d: int, rotary_dim: int) -> bool:
    return bool(lib().gs_attention_decode_raw_supports(c_int(nh), c_int(nkv), c_int(d), c_int(rotary_dim)))


def attention_decode_raw(qkv, q_stride, kcache, vcache, positions, block_table, page_size, window, scale, q_weight,
                         k_weight, head_eps, cos, sin, nh, nkv, d, nseq, nsplit: int, write_kv: bool = True,
                         out=None):
    """Decode attention straight from the rows of q|k|v as their product left them: the kernel norms and rotates
    the queries and the new key, writes the new key and value into their pages, and attends."""
    _dev(qkv, kcache, vcache, positions, block_table, q_weight, k_weight, cos, sin,
         out if isinstance(out, torch.Tensor) else None)
    _need(qkv.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_decode_raw takes bfloat16")
    _need(qkv.numel() >= (nseq - 1) * q_stride + (nh + 2 * nkv) * d if nseq else True, "attention_decode_raw: qkv is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.shape == (d,)), "head norm weight float32 (d,)")
    _need(cos.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == d // 2
          and cos.is_contiguous() and sin.is_contiguous(), "rotation tables (positions, d/2) float32")
    _i32(positions, nseq, "positions")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= nseq,
          "block_table must be int32 (nseq, max_blocks)")
    ws = _decode_workspace(qkv.device, nseq, nh, nkv, d, nsplit)
    out, buf, tiled = _rows_out(out, nseq, nh * d, qkv.device, qkv.dtype)
    _need(tuple(out.shape) == (nseq, nh * d) and out.dtype == qkv.dtype, "attention_decode_raw: out has the wrong shape or type")
    _check(lib().gs_attention_decode_raw(_p(qkv), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(block_table),
                                         c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0),
                                         c_float(scale), _p(q_weight), _p(k_weight), c_float(head_eps), _p(cos), _p(sin),
                                         c_int(d), c_int(1 if write_kv else 0), _p(buf), c_int(tiled), _p(ws), c_int(nseq),
                                         c_int(nh), c_int(nkv), c_int(d), c_int(nsplit), _stream()))
    return out


def attention_prefill_supports(nh: int, nkv: int, d: int) -> bool:
    return bool(lib().gs_attention_prefill_supports(c_int(nh), c_int(nkv), c_int(d)))


def attention_prefill(q, q_stride, kcache, vcache, positions, tiles, block_table, page_size, window, scale, nh, nkv, d,
                      ntok, out: torch.Tensor = None, tile_rows: int = 16) -> torch.Tensor:
    """Causal GQA of many queries per sequence on the matrix cores (bfloat16).

    ``tiles``: int32 ``(3, ntiles)``: sequence, first row and number of rows (at most ``tile_rows``, 16 or
    32) of each tile of consecutive queries of one sequence.
    """
    _dev(q, kcache, vcache, positions, tiles, block_table, out)
    _need(q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_prefill takes bfloat16")
    _need(q.numel() >= (ntok - 1) * q_stride + nh * d if ntok else True, "attention_prefill: q is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, ntok, "positions")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[0] == 3, "tiles must be int32 (3, ntiles)")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, nh * d), dtype=q.dtype, device=q.device)
    _need(out.shape == (ntok, nh * d) and out.dtype == q.dtype, "attention_prefill: out has the wrong shape or type")
    nt = tiles.shape[1]
    _check(lib().gs_attention_prefill(_p(q), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(tiles[0]),
                                      _p(tiles[1]), _p(tiles[2]), c_int(nt), _p(block_table),
                                      c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0), c_float(scale),
                                      _p(out), c_int(nh), c_int(nkv), c_int(d), c_int(tile_rows), _stream()))
    return out


def attention_prefill_wide_supports(nh: int, nkv: int, d: int) -> bool:
    return bool(lib().gs_attention_prefill_wide_supports(c_int(nh), c_int(nkv), c_int(d)))


def attention_prefill_wide_rows(nh: int, nkv: int) -> int:
    """The most queries a block of :func:`attention_prefill_wide` holds for these head counts when it walks the keys
    whole (half as many with the keys in two halves)."""
    return int(lib().gs_attention_prefill_wide_rows(c_int(nh), c_int(nkv)))


def attention_prefill_wide(q, q_stride, kcache, vcache, positions, tiles, block_table, page_size, window, scale, nh, nkv,
                           d, ntok, out: torch.Tensor = None, key_splits: int = 1) -> torch.Tensor:
    """Causal GQA of long prompt portions (bfloat16, heads of 64): 32 queries a wavefront, keys and values shared by a
    block through LDS.  ``tiles``: int32 ``(3, blocks * wq)``, the sequence, first row and row count (at most 32; 0: none)
    of every sub-tile, ``wq = attention_prefill_wide_rows(nh, nkv) // 32 // key_splits`` of them a block, all of
    one sequence, neighbours or not (``BatchContext.query_subtiles`` pairs late ones with early ones).  With
    ``key_splits = 2`` (groups of up to four heads) a block holds half as many queries and two wavefronts walk half
    of the keys each: twice the blocks, half the longest walk."""
    _dev(q, kcache, vcache, positions, tiles, block_table, out)
    _need(q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_prefill_wide takes bfloat16")
    _need(q.numel() >= (ntok - 1) * q_stride + nh * d if ntok else True, "attention_prefill_wide: q is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, ntok, "positions")
    _need(key_splits in (1, 2) and (key_splits == 1 or attention_prefill_wide_rows(nh, nkv) >= 64),
          "attention_prefill_wide: the keys in two halves only for groups of up to four heads")
    rows = attention_prefill_wide_rows(nh, nkv) // key_splits
    wq = rows // 32
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[0] == 3 and wq > 0 and tiles.shape[1] % wq == 0,
          "tiles must be int32 (3, blocks * sub-tiles a block)")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, nh * d), dtype=q.dtype, device=q.device)
    _need(out.shape == (ntok, nh * d) and out.dtype == q.dtype, "attention_prefill_wide: out has the wrong shape or type")
    nt = tiles.shape[1] // wq
    _check(lib().gs_attention_prefill_wide(_p(q), q_stride, _p(kcache), _p(vcache), _p(positions), _p(tiles[0]),
                                           _p(tiles[1]), _p(tiles[2]), nt, _p(block_table),
                                           block_table.shape[1], page_size, kcache.shape[0],
                                           window or 0, scale, _p(out), nh, nkv, d, rows, key_splits, _stream()))
    return out
