"""What parts share at run time: device, activation type, kernels, matrix products.

``Runtime.linear`` is the one place where a matrix product is chosen:

* float32 anywhere (activations, weight or wanted output) -> the tiled FMA kernel, which is the
  true 32-bit product and also takes mixed storage (a weight stored in 32-bit stays so);
* bfloat16 x bfloat16 -> bfloat16: the hand-written skinny kernel for few rows, the vendor
  library (through ``torch``) for many.  The reference hands every matrix product to the
  vendor library as well (``ext/amdgpu_ops.jl:453-465``).
"""
from __future__ import annotations

import torch

from ..errors import KernelError


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

    def shared(self, key, make):
        """One object per key for all parts (rotary tables and the like)."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]

    def linear(self, x: torch.Tensor, w: torch.Tensor, bias=None, out_dtype=None, out=None) -> torch.Tensor:
        """``x @ w.T (+ bias)``; ``w (out, in)``."""
        out_dtype = out_dtype or x.dtype
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and bias is None:
            if self.ops.skinny_ok(x, w):
                return self.ops.gemm_skinny(x, w, out_dtype=out_dtype, out=out)
            if out_dtype == torch.bfloat16 and not self.no_library:
                return torch.mm(x, w.t(), out=out) if out is not None else torch.mm(x, w.t())
        return self.ops.gemm_tiled(x, w, bias, out_dtype=out_dtype, out=out)

    def linear_swiglu(self, x: torch.Tensor, w13: torch.Tensor) -> torch.Tensor:
        """``silu(x @ w1.T) * (x @ w3.T)`` with ``w13`` holding w1's rows, then w3's."""
        if self.ops.skinny_ok(x, w13):
            return self.ops.gemm_skinny(x, w13, swiglu=True)
        return self.ops.swiglu(self.linear(x, w13))

    def attention(self, q, q_stride, cache, ctx, window, scale, nh, nkv, d) -> torch.Tensor:
        """Causal attention of this step's queries over the paged cache; ``(T, nh * d)``.

        The generic kernel takes every size; faster kernels take over for the sizes and batch
        shapes they are written for.
        """
        ops = self.ops
        if ctx.all_single and q.dtype == torch.bfloat16 and ops.attention_decode_supports(nh, nkv, d):
            # one query per sequence: the key stream is split so that the whole chip reads it
            nsplit = max(1, min(16, 512 // max(1, ctx.nseq * nkv)))
            return ops.attention_decode(q, q_stride, cache.k, cache.v, ctx.positions, cache.block_table,
                                        cache.page_size, window, scale, nh, nkv, d, ctx.nseq, nsplit)
        return ops.attention_generic(q, q_stride, cache.k, cache.v, ctx.positions, ctx.seq_of_token,
                                     cache.block_table, cache.page_size, window, scale, nh, nkv, d, ctx.T)
