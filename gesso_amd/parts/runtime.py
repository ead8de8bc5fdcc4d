"""What parts share at run time: device, activation type, kernels, matrix products.

``Runtime.linear`` is the one place where a matrix product is chosen:

* float32 anywhere (activations, weight or wanted output) -> the tiled FMA kernel, which is the
  true 32-bit product and also takes mixed storage (a weight stored in 32-bit stays so);
* bfloat16 x bfloat16: the hand-written weight-streaming kernel for up to 64 rows; for more rows the
  hand-written matrix-core kernel (``gemm_mfma``) or the vendor library through ``torch``, whichever
  ``Runtime.many_rows`` says (the reference hands every matrix product to the vendor library,
  ``ext/amdgpu_ops.jl:453-465``).
"""
from __future__ import annotations

import os

import torch

from ..errors import KernelError


class DeferredLinear:
    """A sub-layer's last product, not yet computed: ``x @ w.T`` to be added to the residual stream."""

    __slots__ = ("x", "w")

    def __init__(self, x, w):
        self.x, self.w = x, w


class RawQKV:
    """Rows of q|k|v as their product left them, with what the attention kernel needs to finish them itself
    (head norms, rotation, cache write).  Opaque to the mixer: it hands it from ``attention_in`` to ``attention``."""

    __slots__ = ("qkv", "q_norm", "k_norm", "eps", "position", "dtype")

    def __init__(self, qkv, q_norm, k_norm, eps, position):
        self.qkv, self.q_norm, self.k_norm, self.eps, self.position = qkv, q_norm, k_norm, eps, position
        self.dtype = qkv.dtype


class Runtime:
    def __init__(self, device, dtype: torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise KernelError(f"the engine runs in float32 or bfloat16, not {dtype}")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError("the engine runs on the GPU only; there is no CPU path")
        from ..kernels import ops
        ops.lib()                      # fail here, loudly, if the extension is missing
        self.ops = ops
        self.dtype = dtype
        self._shared = {}
        self.no_library = False        # set while a HIP graph is recorded: only our own kernels go into it
        self.fused = False             # set while a decode step is recorded: norms, adds and small ops fold into products
        self.tile_weights = dtype == torch.bfloat16   # keep a tile-major copy of weights for the streaming kernels
        self._tiles = {}
        # a lazy norm is folded into the product that follows for up to this many rows; for more, one
        # light kernel norms the rows first (the fold repeats the norm's arithmetic in every block)
        self.fold_norm_rows = int(os.environ.get("GESSO_FOLD_NORM_ROWS", "0"))
        # up to this many rows a deferred product also leaves the rows weighted for the next norm, whose consumer
        # then only scales its result; for more rows every block's reading of the partial sums costs more than
        # one light norm pass
        self.weighted_rows_max = int(os.environ.get("GESSO_WEIGHTED_ROWS_MAX", "32"))
        # q|k|v with head norm, rotation and cache write as the product's epilogue needs a whole head in one block:
        # 48 blocks for LFM2-1.2B, and a block streams weights no faster than about 45 GB/s.  The plain product over
        # the whole chip plus the small kernel for norm, rotation and cache write measured half a percent faster.
        self.fuse_qkv = os.environ.get("GESSO_FUSE_QKV", "0") != "0"
        # rows handed from one fused kernel to the next product travel in the order the matrix cores take them
        # (ops.TiledRows): a product then loads them a contiguous kilobyte at a time
        self.tiled_rows = dtype == torch.bfloat16 and os.environ.get("GESSO_TILED_ROWS", "1") != "0"
        # products of more than 64 rows: "own" = the hand-written matrix-core kernel everywhere (gate|up with SwiGLU in
        # one kernel), "library" = the vendor's wherever it can go, "auto" = the vendor's for bfloat16 results (measured
        # on random data at 2,048 rows: 109 us against our 161 for gate|up, 124 against 162 with the SwiGLU pass
        # counted in; 50 against 75 for 6144 x 2048), ours where the result is float32 and inside a recorded graph
        self.many_rows = os.environ.get("GESSO_GEMM", "auto")
        if self.many_rows not in ("auto", "own", "library"):
            raise KernelError(f"GESSO_GEMM is 'auto', 'own' or 'library', not {self.many_rows!r}")

    def shared(self, key, make):
        """One object per key for all parts (rotary tables and the like)."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]

    # ------------------------------------------------------------------ matrix products

    def prepare(self, w: torch.Tensor, unit: int = 16) -> torch.Tensor:
        """Called by a part for each weight of a matrix product, once, at bind time.

        Makes the tile-major copy that the weight-streaming kernels read (a layout choice, the values
        are the same); ``unit`` is the number of rows after which the part's epilogue starts a new
        group (half the rows for gate|up, a third for B|C|X), which must be whole tiles.  The weight
        as stored stays, for the products of many rows.  Returns ``w``.
        """
        if (self.tile_weights and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
                and w.shape[1] % 32 == 0 and unit % 16 == 0 and w.shape[0] % unit == 0):
            self._tiles[w.data_ptr()] = self.ops.tile_major(w)
        return w

    def _wt(self, w):
        return self._tiles.get(w.data_ptr())

    def rows_tiled(self, width: int) -> bool:
        """Whether rows of this width, written by one fused kernel for the next product, are kept as tiled rows."""
        return self.fused and self.tiled_rows and self.ops.TiledRows.fits(width)

    def new_rows(self, M: int, width: int):
        """Room for bfloat16 rows that a fused kernel writes for the product that follows."""
        if self.rows_tiled(width):
            return self.ops.TiledRows(M, width, self.device)
        return torch.empty((M, width), dtype=torch.bfloat16, device=self.device)

    def _dense(self, x):
        """``x`` as an ordinary tensor, whatever handle it came as."""
        if isinstance(x, self.ops.LazyNorm):
            x = x.materialize()
        return x.rows() if isinstance(x, self.ops.TiledRows) else x

    def linear(self, x, w: torch.Tensor, bias=None, out_dtype=None, out=None) -> torch.Tensor:
        """``x @ w.T (+ bias)``; ``w (out, in)``; ``x`` a tensor or a lazy norm."""
        ops = self.ops
        out_dtype = out_dtype or self.dtype
        if isinstance(x, ops.LazyNorm):
            if bias is None and self._keep_lazy(x) and ops.lazy_ok(x, w):
                return ops.gemm_skinny(x, w, out_dtype=out_dtype, out=out, wt=self._wt(w))
            x = x.materialize()
        if isinstance(x, ops.TiledRows) and not (bias is None and ops.skinny_ok(x, w)):
            x = x.rows()
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and bias is None:
            if ops.skinny_ok(x, w):
                return ops.gemm_skinny(x, w, out_dtype=out_dtype, out=out, wt=self._wt(w))
            library = out_dtype == torch.bfloat16 and not self.no_library and self.many_rows != "own"
            if library:
                return torch.mm(x, w.t(), out=out) if out is not None else torch.mm(x, w.t())
            if self.many_rows != "library" and ops.mfma_ok(x, w) and (out is None or out.is_contiguous()):
                return ops.gemm_mfma(x, w, out_dtype=out_dtype, out=out)
        return ops.gemm_tiled(x, w, bias, out_dtype=out_dtype, out=out)

    def linear_swiglu(self, x, w13: torch.Tensor) -> torch.Tensor:
        """``silu(x @ w1.T) * (x @ w3.T)`` with ``w13`` holding w1's rows, then w3's."""
        ops = self.ops
        tiled = self.rows_tiled(w13.shape[0] // 2)
        if isinstance(x, ops.LazyNorm):
            if self._keep_lazy(x) and ops.lazy_ok(x, w13):
                return ops.gemm_skinny(x, w13, swiglu=True, wt=self._wt(w13), out=tiled)
            x = x.materialize()
        if ops.skinny_ok(x, w13):
            return ops.gemm_skinny(x, w13, swiglu=True, wt=self._wt(w13), out=tiled)
        x = self._dense(x)
        if ((self.many_rows == "own" or (self.no_library and self.many_rows != "library"))
                and self.dtype == torch.bfloat16 and ops.mfma_ok(x, w13) and w13.shape[0] % 2 == 0):
            return ops.gemm_mfma(x, w13, swiglu=True)          # gate|up never goes to memory
        return ops.swiglu(self.linear(x, w13))

    def project(self, x: torch.Tensor, w: torch.Tensor, bias=None):
        """A sub-layer's last product.  While fused kernels are on it is deferred, so that the block can
        compute it straight into the residual stream; else it is computed here."""
        if self.fused and bias is None and self.ops.skinny_ok(x, w):
            return DeferredLinear(x, w)
        return self.linear(x, w, bias)

    # ------------------------------------------------------------------ mixers' inner steps

    def split_parts(self, w) -> int:
        """Into how many parts a deferred product of many rows shares K out: enough blocks to fill the chip
        (a block takes 32 weight rows), each part at least 512 wide (measured at 64 rows, 2048 x 2048: 12.1 us with
        4 parts, 13.1 with 8; 2048 x 8192: 19.2 us with 8 parts, 20.0 with 4, 21.0 with 16)."""
        blocks = max(1, w.shape[0] // 32)
        return max(1, min(16, 512 // blocks, w.shape[1] // 512))

    def _keep_lazy(self, x) -> bool:
        """Whether a lazy norm goes to the product as it is: always when its rows come pre-weighted (the product
        only scales its result), else for few rows (the fold repeats the norm's arithmetic in every block)."""
        return x.xs is not None or x.shape[0] <= self.fold_norm_rows

    def _rows(self, x):
        """A lazy norm as the kernels of this step should take it: kept, or normed by one light pass."""
        if isinstance(x, self.ops.LazyNorm) and not self._keep_lazy(x):
            return x.materialize()
        return x

    def conv_in(self, x, w_in, b_in, taps, b_conv, state, ctx) -> torch.Tensor:
        """Input product and gated short convolution: ``(T, H)`` mixed rows; ``state`` is advanced."""
        ops = self.ops
        if self.fused and b_in is None and ctx.all_single and taps.shape[1] <= 16:
            x = self._rows(x)
            if ops.lazy_ok(x, w_in) or (not isinstance(x, ops.LazyNorm) and ops.skinny_ok(x, w_in)):
                return ops.gemm_skinny_conv(x, w_in, taps, b_conv, state, ctx.slots, wt=self._wt(w_in),
                                            tiled=self.rows_tiled(taps.shape[0]))
        x = self._dense(x)
        bcx = self.linear(x, w_in, b_in)
        return ops.short_conv(bcx, taps, b_conv, state, ctx.seq_of_token, ctx.q_start, ctx.slots, ctx.nseq,
                              ctx.all_single)

    def attention_in(self, x, wqkv, bqkv, q_norm, k_norm, head_eps, position, ctx, cache, nh, nkv, d):
        """q, k, v products, head norms, position encoding, cache write.  Returns ``(q, q_stride)``:
        the queries as rows of a buffer, ``q_stride`` apart, head h at ``[h d, (h+1) d)``."""
        ops = self.ops
        if (self.fused and self.fuse_qkv and bqkv is None and ctx.all_single and cache.k.dtype == torch.bfloat16
                and ops.gemm_skinny_qkv_supports(d, position.rotary_dim)):
            x = self._rows(x)
            if ops.lazy_ok(x, wqkv) or (not isinstance(x, ops.LazyNorm) and ops.skinny_ok(x, wqkv)):
                q = ops.gemm_skinny_qkv(x, wqkv, q_norm, k_norm, head_eps, position.cos, position.sin, ctx.positions,
                                        cache.block_table, cache.page_size, cache.k, cache.v, nh, nkv, d,
                                        write_kv=cache.write, wt=self._wt(wqkv))
                return q, nh * d
        qkv = self.linear(x, wqkv, bqkv)          # a lazy norm goes through as it is where the product takes it
        if (self.fused and ctx.all_single and cache.k.dtype == torch.bfloat16 and qkv.dtype == torch.bfloat16
                and cache.page_size >= 2 and (q_norm is None) == (k_norm is None)
                and ops.attention_decode_raw_supports(nh, nkv, d, position.rotary_dim)):
            # a decode step: the attention kernel norms, rotates and writes the cache itself
            return RawQKV(qkv, q_norm, k_norm, head_eps, position), (nh + 2 * nkv) * d
        ops.qknorm_rope_kv(qkv, q_norm, k_norm, head_eps, position.cos, position.sin, position.rotary_dim,
                           ctx.positions, ctx.seq_of_token, cache.block_table, cache.page_size, cache.k, cache.v,
                           nh, nkv, d, write_kv=cache.write)
        return qkv, (nh + 2 * nkv) * d

    def _attention_single(self, q, q_stride, cache, ctx, window, scale, nh, nkv, d, nseq, out):
        """The first ``nseq`` sequences, one query each (their rows are the first ``nseq`` rows).  A block of eight
        wavefronts takes a tile of 64 keys per wavefront and pass; key streams are split over blocks (and a merge
        kernel) only when the batch alone does not fill the chip."""
        longest = ctx.max_kv_len if ctx.max_kv_len is not None else cache.block_table.shape[1] * cache.page_size
        if window:
            longest = min(longest, window)
        tiles = max(1, -(-longest // 64))
        # (sequence, key head) pairs fill the chip by themselves from about 256 on; fewer pairs share their keys out
        # over blocks, each split at least 1,024 keys long (measured at 8 sequences of 32,768 keys: 4 splits 107 us,
        # 32 splits 145 us; at 64 sequences any split is slower than none)
        nsplit = max(1, min(tiles // 16, 64, 256 // max(1, nseq * nkv)))
        if isinstance(q, RawQKV):
            return self.ops.attention_decode_raw(q.qkv, q_stride, cache.k, cache.v, ctx.positions, cache.block_table,
                                                 cache.page_size, window, scale, q.q_norm, q.k_norm, q.eps,
                                                 q.position.cos, q.position.sin, nh, nkv, d, nseq, nsplit,
                                                 write_kv=cache.write, out=out)
        return self.ops.attention_decode(q, q_stride, cache.k, cache.v, ctx.positions, cache.block_table,
                                         cache.page_size, window, scale, nh, nkv, d, nseq, nsplit, out=out)

    def attention(self, q, q_stride, cache, ctx, window, scale, nh, nkv, d) -> torch.Tensor:
        """Causal attention of this step's queries over the paged cache; ``(T, nh * d)``.

        The generic kernel takes every size; faster kernels take over for the sizes and batch
        shapes they are written for.
        """
        ops = self.ops
        out = True if self.rows_tiled(nh * d) else None
        if isinstance(q, RawQKV):
            return self._attention_single(q, q_stride, cache, ctx, window, scale, nh, nkv, d, ctx.nseq, out)
        fast = q.dtype == torch.bfloat16 and cache.page_size >= 2
        if ctx.all_single and fast and ops.attention_decode_supports(nh, nkv, d):
            return self._attention_single(q, q_stride, cache, ctx, window, scale, nh, nkv, d, ctx.nseq, out)
        if (not ctx.all_single and fast and q_stride % 8 == 0 and ops.attention_prefill_supports(nh, nkv, d)):
            # prompts: queries in tiles per sequence, both products on the matrix cores; tiles of 32 share
            # every key and value fragment between two products, which pays when portions are long
            # (groups of more than four heads have no registers for tiles of 32)
            rows = 32 if ctx.max_q_len >= 64 and nh // nkv <= 4 else 16
            # decoded tokens at the batch's head go to the kernel for single queries: as tiles of one query they
            # would each hold a whole block that walks all the keys alone
            lead = getattr(ctx, "lead_single", 0)
            if not ops.attention_decode_supports(nh, nkv, d):
                lead = 0
            out = torch.empty((ctx.T, nh * d), dtype=q.dtype, device=q.device)
            if lead:
                self._attention_single(q, q_stride, cache, ctx, window, scale, nh, nkv, d, lead, out[:lead])
            return ops.attention_prefill(q, q_stride, cache.k, cache.v, ctx.positions, ctx.query_tiles(rows, lead),
                                         cache.block_table, cache.page_size, window, scale, nh, nkv, d, ctx.T,
                                         out=out, tile_rows=rows)
        return ops.attention_generic(q, q_stride, cache.k, cache.v, ctx.positions, ctx.seq_of_token,
                                     cache.block_table, cache.page_size, window, scale, nh, nkv, d, ctx.T)
