"""Grouped-query causal attention over the paged cache.

``q, k, v = x Wq^T, x Wk^T, x Wv^T``; per-head RMSNorm of q and k (when the spec has one),
then the position encoding, both before the cache write; keys and values of this step go
into the request's pages and the queries read all keys they may see from there.
Reference: ``src/Inference/Inference.jl:296-357`` (order of norm and rotation ``:307-323``),
causal rule ``:1206-1207``, grouping ``:1852-1870``.  The cache holds post-norm, post-rotation
keys and raw values (``:2417-2422``).  Wq, Wk, Wv are laid side by side at load.
"""
from __future__ import annotations

import math

import torch

from ..errors import InvalidPlan
from .base import MATRIX, VECTOR, PagedKV, Part, TensorSpec
from .registry import build, register


class RawQKV:
    """Rows of q|k|v as their product left them, with what the decode kernel needs to finish them itself
    (head norms, rotation, cache write)."""

    __slots__ = ("qkv", "q_norm", "k_norm", "eps", "position", "dtype")

    def __init__(self, qkv, q_norm, k_norm, eps, position):
        self.qkv, self.q_norm, self.k_norm, self.eps, self.position = qkv, q_norm, k_norm, eps, position
        self.dtype = qkv.dtype


class Attention(Part):
    graph_safe = True
    portions_recordable = True
    stage, out_stage = "attn_mixer", "attn_outproj"   # the decode profiler's names
    HALVES_MAX_KEYS = 4096    # prompts whose sequences hold fewer keys may have their keys walked in two halves

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("query heads must be a multiple of key heads")
        self.position = build("position", spec.position, rt)
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(spec.head_dim)

    @staticmethod
    def tensor_specs(spec):
        H, nh, nkv, d = spec.hidden, spec.n_heads, spec.n_kv_heads, spec.head_dim
        out = {"q_proj.weight": TensorSpec((nh * d, H), MATRIX), "k_proj.weight": TensorSpec((nkv * d, H), MATRIX),
               "v_proj.weight": TensorSpec((nkv * d, H), MATRIX), "out_proj.weight": TensorSpec((H, nh * d), MATRIX)}
        if spec.bias:
            out.update({"q_proj.bias": TensorSpec((nh * d,), VECTOR), "k_proj.bias": TensorSpec((nkv * d,), VECTOR),
                        "v_proj.bias": TensorSpec((nkv * d,), VECTOR), "out_proj.bias": TensorSpec((H,), VECTOR)})
        if spec.qk_norm is not None:
            out.update({"q_norm.weight": TensorSpec((d,), VECTOR, "one_plus_normal"),
                        "k_norm.weight": TensorSpec((d,), VECTOR, "one_plus_normal")})
        return out

    @staticmethod
    def cache_need(spec):
        return PagedKV(spec.n_kv_heads, spec.head_dim, spec.window)

    def bind(self, tensors):
        ws = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.float() for w in ws]
        self.wqkv = self.rt.prepare(torch.cat(ws, 0).contiguous())
        self.wo = self.rt.prepare(tensors["out_proj.weight"])
        self.bqkv = self.bo = None
        if self.spec.bias:
            self.bqkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]], 0).contiguous()
            self.bo = tensors["out_proj.bias"]
        self.q_norm = tensors.get("q_norm.weight")
        self.k_norm = tensors.get("k_norm.weight")

    def forward(self, x, ctx, cache):
        q, q_stride = self.project_in(x, ctx, cache)
        with self.rt.stage("attn_core"):
            o = self.attend(q, q_stride, ctx, cache)
        return self.rt.project(o, self.wo, self.bo)

    # ------------------------------------------------------------------ the mixer's inner steps

    def project_in(self, x, ctx, cache):
        """q, k, v products, head norms, position encoding, cache write.  Returns ``(q, q_stride)``: the queries
        as rows of a buffer, ``q_stride`` apart, head h at ``[h d, (h+1) d)``; or a :class:`RawQKV` for the decode
        kernel that norms, rotates and writes the cache itself."""
        s, rt, ops, pos = self.spec, self.rt, self.rt.ops, self.position
        nh, nkv, d = s.n_heads, s.n_kv_heads, s.head_dim
        eps = s.qk_norm.eps if s.qk_norm is not None else 1.0
        layout = getattr(pos, "layout", "half")
        with rt.stage("attn_proj"):
            qkv = rt.linear(x, self.wqkv, self.bqkv)      # a lazy norm goes through as it is where the product takes it
        stride = (nh + 2 * nkv) * d
        if (rt.fused and ctx.all_single and cache.k.dtype == torch.bfloat16 and qkv.dtype == torch.bfloat16
                and cache.page_size >= 2 and (self.q_norm is None) == (self.k_norm is None) and layout == "half"
                and ops.attention_decode_raw_supports(nh, nkv, d, pos.rotary_dim)):
            return RawQKV(qkv, self.q_norm, self.k_norm, eps, pos), stride
        with rt.stage("attn_headnorm_rope"):
            ops.qknorm_rope_kv(qkv, self.q_norm, self.k_norm, eps, pos.cos, pos.sin, pos.rotary_dim, ctx.positions,
                               ctx.seq_of_token, cache.block_table, cache.page_size, cache.k, cache.v, nh, nkv, d,
                               write_kv=cache.write, layout=layout)
        return qkv, stride

    def _single(self, q, q_stride, cache, ctx, nseq, out):
        """The first ``nseq`` sequences, one query each (their rows are the first ``nseq`` rows).  A block of eight
        wavefronts takes a tile of 64 keys per wavefront and pass; key streams are split over blocks (and a merge
        kernel) only when the batch alone does not fill the chip."""
        s, ops = self.spec, self.rt.ops
        nh, nkv, d, window = s.n_heads, s.n_kv_heads, s.head_dim, s.window
        longest = ctx.max_kv_len if ctx.max_kv_len is not None else cache.block_table.shape[1] * cache.page_size
        if window:
            longest = min(longest, window)
        tiles = max(1, -(-longest // 64))
        # (sequence, key head) pairs fill the chip by themselves from about 256 on; fewer pairs share their keys out
        # over blocks, each split at least 1,024 keys long (measured at 8 sequences of 32,768 keys: 4 splits 107 us,
        # 32 splits 145 us; at 64 sequences any split is slower than none)
        nsplit = max(1, min(tiles // 16, 64, 256 // max(1, nseq * nkv)))
        if isinstance(q, RawQKV):
            return ops.attention_decode_raw(q.qkv, q_stride, cache.k, cache.v, ctx.positions, cache.block_table,
                                            cache.page_size, window, self.scale, q.q_norm, q.k_norm, q.eps,
                                            q.position.cos, q.position.sin, nh, nkv, d, nseq, nsplit,
                                            write_kv=cache.write, out=out)
        return ops.attention_decode(q, q_stride, cache.k, cache.v, ctx.positions, cache.block_table,
                                    cache.page_size, window, self.scale, nh, nkv, d, nseq, nsplit, out=out)

    def prompt_walk(self, q_lens, max_kv_len):
        """How the kernel for long portions takes sequences that bring ``q_lens`` tokens: ``(sub-tiles a block, key
        halves, late sub-tiles paired with early ones)``."""
        s, rt, ops = self.spec, self.rt, self.rt.ops
        nkv = s.n_kv_heads
        wq = ops.attention_prefill_wide_rows(s.n_heads, nkv) // 32
        blocks = sum(-(-(-(-n // 32)) // wq) for n in q_lens) * nkv
        few = blocks <= rt.compute_units
        halves = 2 if few and wq >= 2 and max_kv_len is not None and max_kv_len < self.HALVES_MAX_KEYS else 1
        wq //= halves
        return wq, halves, (not s.window and wq >= 2 and few)

    def replay_key(self, q_lens, max_kv_len):
        """A recorded step of prompt portions walks the keys as the step that replays it would: whole (1) or in halves
        (2); a step of single tokens: "single".  False: such a step does not go through the kernel for long portions
        (or, of single tokens, would split their keys over blocks by the longest sequence), and is not to be recorded."""
        s, rt, ops = self.spec, self.rt, self.rt.ops
        nh, nkv, d = s.n_heads, s.n_kv_heads, s.head_dim
        lead = 0
        while lead < len(q_lens) and q_lens[lead] == 1:
            lead += 1
        if lead == len(q_lens):
            # single tokens only: the kernel for single queries takes every sequence's keys in one block when the
            # (sequence, key head) pairs fill the chip by themselves, and its launch then depends on their number alone
            return "single" if (rt.dtype == torch.bfloat16 and ops.attention_decode_supports(nh, nkv, d)
                                and 256 // (lead * nkv) <= 1) else False
        choice = rt.options.prompt_attention
        stride = (nh + 2 * nkv) * d
        if not (rt.dtype == torch.bfloat16 and stride % 8 == 0
                and ops.attention_prefill_supports(nh, nkv, d) and ops.attention_decode_supports(nh, nkv, d)
                and choice != "tiles" and ops.attention_prefill_wide_supports(nh, nkv, d)
                and (choice == "wide" or max(q_lens) >= 64)):
            return False
        return self.prompt_walk(q_lens[lead:], max_kv_len)[1]

    def _attend_recorded(self, q, q_stride, ctx, cache) -> torch.Tensor:
        """The prompt part of :meth:`attend` while a step is recorded for replay: the tile lists lie in a buffer that
        every replay refills (as many blocks as the token count and the most sequences can make, the unused ones
        without queries), and the decoded tokens at the batch's head, whose number changes from step to step, are left
        to a call that every replay makes anew."""
        s, rt, ops, rec = self.spec, self.rt, self.rt.ops, ctx.recording
        nh, nkv, d, window = s.n_heads, s.n_kv_heads, s.head_dim, s.window
        halves = rec.key_of(self)
        if halves not in (1, 2) or isinstance(q, RawQKV) or q.dtype != torch.bfloat16 or cache.page_size < 2:
            raise InvalidPlan("this step's attention cannot be recorded (see replay_key)")
        wq = ops.attention_prefill_wide_rows(nh, nkv) // 32 // halves
        out = torch.empty((ctx.T, nh * d), dtype=q.dtype, device=q.device)

        def lists(c):
            lead = c.lead_single
            return c.subtile_lists(wq, lead, paired=self.prompt_walk(c.q_lens[lead:], c.max_kv_len)[2])

        def decoded(c):
            if c.lead_single:
                self._single(q, q_stride, cache, c, c.lead_single, out[:c.lead_single])

        # layers of one shape walk alike and share a list
        tiles = rec.subtiles(("attention", nh, nkv, bool(window), halves), wq, lists)
        rec.eager(decoded)
        return ops.attention_prefill_wide(q, q_stride, cache.k, cache.v, ctx.positions, tiles, cache.block_table,
                                          cache.page_size, window, self.scale, nh, nkv, d, ctx.T, out=out,
                                          key_splits=halves)

    def attend(self, q, q_stride, ctx, cache) -> torch.Tensor:
        """Causal attention of this step's queries over the paged cache; ``(T, nh * d)``.

        The generic kernel takes every size; faster kernels take over for the sizes and batch
        shapes they are written for.
        """
        s, rt, ops = self.spec, self.rt, self.rt.ops
        nh, nkv, d, window = s.n_heads, s.n_kv_heads, s.head_dim, s.window
        out = True if rt.rows_tiled(nh * d) else None
        if isinstance(q, RawQKV):
            return self._single(q, q_stride, cache, ctx, ctx.nseq, out)
        fast = q.dtype == torch.bfloat16 and cache.page_size >= 2
        if ctx.recording is not None and not ctx.all_single:
            return self._attend_recorded(q, q_stride, ctx, cache)
        if ctx.all_single and fast and ops.attention_decode_supports(nh, nkv, d):
            return self._single(q, q_stride, cache, ctx, ctx.nseq, out)
        if (not ctx.all_single and fast and q_stride % 8 == 0 and ops.attention_prefill_supports(nh, nkv, d)):
            # prompts: queries in tiles per sequence, both products on the matrix cores
            # decoded tokens at the batch's head go to the kernel for single queries: as tiles of one query they
            # would each hold a whole block that walks all the keys alone
            lead = ctx.lead_single if ops.attention_decode_supports(nh, nkv, d) else 0
            out = torch.empty((ctx.T, nh * d), dtype=q.dtype, device=q.device)
            if lead:
                self._single(q, q_stride, cache, ctx, lead, out[:lead])
            choice = rt.options.prompt_attention
            if (choice != "tiles" and ops.attention_prefill_wide_supports(nh, nkv, d)
                    and (choice == "wide" or ctx.max_q_len >= 64)):
                # long portions: 32 queries a wavefront, keys and values shared by the block through LDS
                # While the launch has at most a block a compute unit its time is the longest block's walk: then a
                # block pairs late queries with early ones and all walk alike (a prompt of 2,048 tokens, 32 query
                # heads on 8 key heads: 46.7 against 53.1 us; 2,048 over a prefix of 2,048: 97.8 against 104.7).  With
                # more blocks than units the chip balances by itself and paired blocks, which all walk to their late
                # queries' end, only add steps (4,096 tokens: 156 against 122 us); a window makes every walk as short.
                # Short walks at most a block a unit: two wavefronts a head walk half of the keys each and merge at the end,
                # so that the longest walk is half as long and twice the blocks spread evenly (the same prompt 40.4 us;
                # 1,024 tokens 18.9 against 25.4; 512 over a prefix of 1,024: 24.5 against 37.4; over a prefix of 30,720,
                # where every walk is long, staging two halves a step costs more than it saves: 897 against 834).
                lens = ctx.q_lens[lead:]
                wq, halves, paired = self.prompt_walk(lens, ctx.max_kv_len)
                return ops.attention_prefill_wide(q, q_stride, cache.k, cache.v, ctx.positions,
                                                  ctx.query_subtiles(wq, lead, paired=paired), cache.block_table,
                                                  cache.page_size, window, self.scale, nh, nkv, d, ctx.T, out=out,
                                                  key_splits=halves)
            # tiles of 32 share every key and value fragment between two products, which pays when portions are
            # long (groups of more than four heads have no registers for tiles of 32)
            rows = 32 if ctx.max_q_len >= 64 and nh // nkv <= 4 else 16
            return ops.attention_prefill(q, q_stride, cache.k, cache.v, ctx.positions, ctx.query_tiles(rows, lead),
                                         cache.block_table, cache.page_size, window, self.scale, nh, nkv, d, ctx.T,
                                         out=out, tile_rows=rows)
        return ops.attention_generic(q, q_stride, cache.k, cache.v, ctx.positions, ctx.seq_of_token,
                                     cache.block_table, cache.page_size, window, self.scale, nh, nkv, d, ctx.T)


register("mixer", "attention", Attention)
