"""What parts share at run time: device, activation type, kernels, matrix products.

``Runtime.linear`` is the one place where a matrix product is chosen:

* float32 anywhere (activations, weight or wanted output) -> the tiled FMA kernel, which is the
  true 32-bit product and also takes mixed storage (a weight stored in 32-bit stays so);
* bfloat16 x bfloat16: the hand-written weight-streaming kernel for up to 64 rows; for more rows the
  hand-written matrix-core kernel (``gemm_mfma``) or the vendor library through ``torch``, whichever
  ``RuntimeOptions.many_rows`` says (the reference hands every matrix product to the vendor library,
  ``ext/amdgpu_ops.jl:453-465``).

What a mixer or a feed-forward does between its products is its own business (its file chooses its kernels);
the runtime offers the products and the handles that travel between fused kernels while a decode step is
recorded: a norm not yet applied (``ops.LazyNorm``), rows in the matrix cores' operand order (``ops.TiledRows``),
a product deferred into the residual stream (:class:`DeferredLinear`).  ``dense`` turns any of them into a tensor.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..errors import KernelError


@dataclass(frozen=True)
class RuntimeOptions:
    """How kernels are chosen where more than one can do the work; given to the engine's constructor.

    ``many_rows``: products of more than 64 rows in bfloat16: ``"own"`` = the hand-written matrix-core kernel
    everywhere (gate|up with SwiGLU in one kernel), ``"library"`` = the vendor's wherever it can go, ``"auto"`` = the
    vendor's for bfloat16 results (measured on random data at 2,048 rows: 109 us against our 161 for gate|up, 124
    against 162 with the SwiGLU pass counted in; 50 against 75 for 6144 x 2048), ours where the result is float32 and
    inside the recording of the fused decode loop.
    ``tune_library``: where the vendor library computes a product of 128, 256, 512, 1024, ... rows (whole prompt portions, the decode loop for many rows),
    the first product of a shape measures the library's two dozen best guesses on the operands at hand, cold, and
    keeps the library's first choice unless another is clearly faster (some ten milliseconds a shape).  Other row
    counts, and all with this off, take the library's first choice.  Off unless asked for: which candidate a
    measurement prefers can differ between two processes, and with it the rounding of prompt logits, so that one seed
    would no longer give the same ids in every run; the benchmark switches it on.
    ``prompt_attention``: attention of prompt portions in bfloat16: ``"wide"`` = the kernel for long portions wherever it
    takes the sizes (heads of 64), ``"tiles"`` = the kernel with tiles of 16 or 32 queries always, ``"auto"`` = the
    first for steps with a portion of at least 64 tokens, else the second.
    ``tiled_rows``: rows handed from one fused kernel to the next product travel in the order the matrix cores
    take them (``ops.TiledRows``): a product then loads them a contiguous kilobyte at a time.
    ``tile_weights``: keep a tile-major copy of each bfloat16 weight for the streaming kernels.
    ``fold_norm_rows``: a lazy norm is folded into the product that follows for up to this many rows; for more,
    one light kernel norms the rows first (the fold repeats the norm's arithmetic in every block).
    ``weighted_rows_max``: up to this many rows a deferred product also leaves the rows weighted for the next norm,
    whose consumer then only scales its result; for more rows every block's reading of the partial sums costs
    more than one light norm pass.
    ``record_portions``: steps that hold prompt portions are recorded as HIP graphs once their kind (token count,
    room for keys, how attention walks) has come twice, and replayed from then on: a scheduler that fills its token
    budget repeats one kind step after step, and launching such a step's kernels one by one takes the host longer than
    the device needs for them on small models.  The logits are the same bit for bit.
    """

    many_rows: str = "auto"
    record_portions: bool = False
    tune_library: bool = False
    prompt_attention: str = "auto"
    tiled_rows: bool = True
    tile_weights: bool = True
    fold_norm_rows: int = 0
    weighted_rows_max: int = 32

    def __post_init__(self):
        if self.many_rows not in ("auto", "own", "library"):
            raise KernelError(f"many_rows is 'auto', 'own' or 'library', not {self.many_rows!r}")
        if self.prompt_attention not in ("auto", "wide", "tiles"):
            raise KernelError(f"prompt_attention is 'auto', 'wide' or 'tiles', not {self.prompt_attention!r}")
        if self.fold_norm_rows < 0 or self.weighted_rows_max < 0:
            raise KernelError("row limits are nonnegative")


class _NoStage:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_STAGE = _NoStage()


class DeferredLinear:
    """A sub-layer's last product, not yet computed: ``x @ w.T`` to be added to the residual stream."""

    __slots__ = ("x", "w")

    def __init__(self, x, w):
        self.x, self.w = x, w


class Runtime:
    def __init__(self, device, dtype: torch.dtype, options: RuntimeOptions = None):
        if dtype not in (torch.float32, torch.bfloat16):
            raise KernelError(f"the engine runs in float32 or bfloat16, not {dtype}")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError("the engine runs on the GPU only; there is no CPU path")
        from ..kernels import ops
        ops.lib()                      # fail here, loudly, if the extension is missing
        self.ops = ops
        self.dtype = dtype
        self.options = options = options or RuntimeOptions()
        self._shared = {}
        self.no_library = False        # set while a HIP graph is recorded: only our own kernels go into it
        self.fused = False             # set while a decode step is recorded: norms, adds and small ops fold into products
        self.tile_weights = dtype == torch.bfloat16 and options.tile_weights
        self._tiles = {}
        self.fold_norm_rows = options.fold_norm_rows
        self.weighted_rows_max = options.weighted_rows_max
        self.tiled_rows = dtype == torch.bfloat16 and options.tiled_rows
        self.many_rows = options.many_rows
        self.tune_library = options.tune_library
        self.compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        self.streaming_rows_max = ops.SKINNY_MAX_ROWS   # the most rows a weight-streaming product takes
        self._library_ws = None        # device bytes for the vendor library's kernels, made at the first such product
        self.profile = None            # a StageProfile while decode steps are profiled (engine/profile.py)

    def stage(self, name: str):
        """A context manager that brackets a named stage of the decode step when the profiler is on; else nothing."""
        return _NO_STAGE if self.profile is None else self.profile.bracket(name)

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

    def tiles_of(self, w):
        """The tile-major copy of a weight that went through :meth:`prepare`, or None."""
        return self._tiles.get(w.data_ptr())

    def rows_tiled(self, width: int) -> bool:
        """Whether rows of this width, written by one fused kernel for the next product, are kept as tiled rows."""
        return self.fused and self.tiled_rows and self.ops.TiledRows.fits(width)

    def new_rows(self, M: int, width: int):
        """Room for bfloat16 rows that a fused kernel writes for the product that follows."""
        if self.rows_tiled(width):
            return self.ops.TiledRows(M, width, self.device)
        return torch.empty((M, width), dtype=torch.bfloat16, device=self.device)

    def dense(self, x):
        """``x`` as an ordinary tensor, whatever handle it came as."""
        if isinstance(x, self.ops.LazyNorm):
            x = x.materialize()
        return x.rows() if isinstance(x, self.ops.TiledRows) else x

    def linear(self, x, w: torch.Tensor, bias=None, out_dtype=None, out=None) -> torch.Tensor:
        """``x @ w.T (+ bias)``; ``w (out, in)``; ``x`` a tensor or a lazy norm."""
        ops = self.ops
        out_dtype = out_dtype or self.dtype
        if isinstance(x, ops.LazyNorm):
            if bias is None and self.keep_lazy(x) and ops.lazy_ok(x, w):
                return ops.gemm_skinny(x, w, out_dtype=out_dtype, out=out, wt=self.tiles_of(w))
            x = x.materialize()
        if isinstance(x, ops.TiledRows) and not (bias is None and ops.skinny_ok(x, w)):
            x = x.rows()
        if (bias is not None and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and bias.dtype == torch.float32
                and (ops.skinny_ok(x, w) or (self.many_rows != "library" and ops.mfma_ok(x, w)))):
            # the matrix cores' float32 sums, then the bias and one rounding
            return ops.add_bias(self.linear(x, w, out_dtype=torch.float32), bias, out_dtype, out)
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and bias is None:
            if ops.skinny_ok(x, w):
                return ops.gemm_skinny(x, w, out_dtype=out_dtype, out=out, wt=self.tiles_of(w))
            library = out_dtype == torch.bfloat16 and not self.no_library and self.many_rows != "own"
            if library:
                return self._library_product(x, w, out)
            if self.many_rows != "library" and ops.mfma_ok(x, w) and (out is None or out.is_contiguous()):
                return ops.gemm_mfma(x, w, out_dtype=out_dtype, out=out)
        return ops.gemm_tiled(x, w, bias, out_dtype=out_dtype, out=out)

    LIBRARY_WORKSPACE = 64 << 20

    def _library_product(self, x, w, out):
        """``x @ w.T`` by the vendor library: called directly where it takes the operands (``ops.library_gemm``: a plan
        per shape, a few microseconds of host time a call), else through ``torch.mm``."""
        ops = self.ops
        if ops.library_gemm_ok(x, w) and (out is None or (out.dtype == torch.bfloat16 and out.is_cuda and out.stride(1) == 1
                                                          and out.shape == (x.shape[0], w.shape[0])
                                                          and out.data_ptr() % 16 == 0
                                                          and (out.shape[0] <= 1 or out.stride(0) % 8 == 0))):
            if self._library_ws is None:
                self._library_ws = torch.empty(self.LIBRARY_WORKSPACE, dtype=torch.uint8, device=self.device)
            # measured only for the row counts that come again and again (whole prompt portions: a power of two from
            # 512 on): a measurement takes some ten milliseconds a shape, and a server's steps bring ever new row counts
            M = x.shape[0]
            return ops.library_gemm(x, w, self._library_ws, out=out,
                                    tune=self.tune_library and M >= 128 and M & (M - 1) == 0, checked=True)
        return torch.mm(x, w.t(), out=out) if out is not None else torch.mm(x, w.t())

    def linear_swiglu(self, x, w13: torch.Tensor) -> torch.Tensor:
        """``silu(x @ w1.T) * (x @ w3.T)`` with ``w13`` holding w1's rows, then w3's."""
        ops = self.ops
        tiled = self.rows_tiled(w13.shape[0] // 2)
        if isinstance(x, ops.LazyNorm):
            if self.keep_lazy(x) and ops.lazy_ok(x, w13):
                return ops.gemm_skinny(x, w13, swiglu=True, wt=self.tiles_of(w13), out=tiled)
            x = x.materialize()
        if ops.skinny_ok(x, w13):
            return ops.gemm_skinny(x, w13, swiglu=True, wt=self.tiles_of(w13), out=tiled)
        x = self.dense(x)
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

    # ------------------------------------------------------------------ handles between fused kernels

    def split_parts(self, w) -> int:
        """Into how many parts a deferred product of many rows shares K out: enough blocks to fill the chip
        (a block takes 32 weight rows), each part at least 512 wide (measured at 64 rows, 2048 x 2048: 12.1 us with
        4 parts, 13.1 with 8; 2048 x 8192: 19.2 us with 8 parts, 20.0 with 4, 21.0 with 16)."""
        blocks = max(1, w.shape[0] // 32)
        return max(1, min(16, 512 // blocks, w.shape[1] // 512))

    def keep_lazy(self, x) -> bool:
        """Whether a lazy norm goes to the product as it is: always when its rows come pre-weighted (the product
        only scales its result), else for few rows (the fold repeats the norm's arithmetic in every block)."""
        return x.xs is not None or x.shape[0] <= self.fold_norm_rows

    def lazy_rows(self, x):
        """A lazy norm as the kernels of this step should take it: kept, or normed by one light pass."""
        if isinstance(x, self.ops.LazyNorm) and not self.keep_lazy(x):
            return x.materialize()
        return x

    def streams(self, x, w) -> bool:
        """Whether the weight-streaming kernels take ``x`` (rows, tiled rows or a lazy norm) against ``w``."""
        if isinstance(x, self.ops.LazyNorm):
            return self.ops.lazy_ok(x, w)
        return self.ops.skinny_ok(x, w)
