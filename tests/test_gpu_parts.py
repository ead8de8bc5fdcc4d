"""Each part alone against the plain implementation, and parts that the framework has never seen.

A harness builds one part from its spec with random tensors, a cache for it and step contexts,
and runs it whole and in portions.  The toy parts at the end (a mixer with a running state of
its own, in float32 and in bfloat16, that starts from a value other than zero; a feed-forward with routing; a
position encoding with another table and interleaved pairs; a schedule that runs a block twice and lets a
layer read another layer's cache; a scaled embedding and capped logits) are defined here, registered here and
stepped through the unchanged engine.
"""
import dataclasses
import os
import math

import pytest
import torch

import plain_lfm2 as P

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(scope="module")
def fw():
    import gesso_amd
    from gesso_amd.kernels import ops
    ops.lib()
    return gesso_amd


def gen(seed):
    return torch.Generator().manual_seed(seed)


class Harness:
    """One mixer (or any part with tensors) with its own cache, stepped like the engine steps it."""

    def __init__(self, category, spec, dtype, seed=0, page_size=8, num_pages=32, std=0.2):
        from gesso_amd.cache.manager import CacheLayout, CacheManager
        from gesso_amd.cache.storage import CacheStorage
        from gesso_amd.parts import Runtime, build, part_class
        from gesso_amd.weights import random_tensors
        from gesso_amd.weights.loader import held_dtype

        self.rt = Runtime(DEV, dtype)
        self.part = build(category, spec, self.rt)
        cls = part_class(category, spec)
        table = cls.tensor_specs(spec)
        cpu = random_tensors(table, seed, dtype, std=std)
        self.tensors = {k: v.double() for k, v in cpu.items()}
        self.part.bind({k: v.to(DEV, held_dtype(v.dtype, table[k].role, dtype)) for k, v in cpu.items()})
        need = cls.cache_need(spec) if hasattr(cls, "cache_need") else None
        layout = CacheLayout.plan([need], [None])
        self.manager = CacheManager(layout, page_size, num_pages, 4, 4096)
        self.storage = CacheStorage(layout, page_size, num_pages, 4, dtype, DEV)
        self.dtype = dtype

    def ctx(self, entries):
        from gesso_amd.engine.batch import StepContext, StepEntry
        es = [StepEntry(rid, [0] * n, []) for rid, n in entries]
        for e in es:
            if e.rid not in self.manager.requests:
                self.manager.admit(e.rid)
        if self.manager.fresh_slots:
            self.storage.fill_slots(self.rt.ops, self.manager.fresh_slots, "initial")
            self.manager.fresh_slots.clear()
        self.manager.reserve_many([(e.rid, len(e.tokens)) for e in es])
        c = StepContext(es, self.manager, self.storage, 1, DEV)
        for e in es:
            self.manager.commit(e.rid, len(e.tokens))
        return c

    def mixer(self, x, entries):
        c = self.ctx(entries)
        return self.part.forward(x.to(DEV, self.dtype), c, c.cache_view(0)).double().cpu()


def tol(dtype, ref):
    # bfloat16: 1e-2 of the largest value (at 8e-3 the first sound part fails: a toy mixer with values 40 wide)
    return (2e-5 if dtype == torch.float32 else 1e-2) * max(1.0, float(ref.abs().max()))


# ------------------------------------------------------------------ norm, position, feed-forward

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(fw, dtype):
    from gesso_amd.config import RMSNormSpec
    from gesso_amd.parts import ResidualStream
    h = Harness("norm", RMSNormSpec(size=144, eps=1e-4), dtype)
    res = torch.randn(6, 144, generator=gen(0))
    delta = torch.randn(6, 144, generator=gen(1)).to(dtype)
    stream = ResidualStream(res.clone().to(DEV), delta.to(DEV))
    out = h.part.add_norm(stream).double().cpu()
    want = P.rmsnorm(res.double() + delta.double(), h.tensors["weight"], 1e-4)
    assert float((out - want).abs().max()) <= tol(dtype, want)
    assert stream.pending is None and torch.allclose(stream.res.cpu().double(), res.double() + delta.double(), atol=1e-6)


def test_rope_part_tables(fw):
    from gesso_amd.config import RopeSpec
    from gesso_amd.parts import Runtime, build
    rt = Runtime(DEV, torch.float32)
    r = build("position", RopeSpec(head_dim=48, rotary_dim=32, theta=5e5, max_position=300), rt)
    assert r.cos.shape == (300, 16) and r.rotary_dim == 32
    for pos, i in ((0, 0), (1, 0), (299, 15), (77, 9)):
        ang = pos * 5e5 ** (-2 * i / 32)
        assert float(r.cos[pos, i]) == pytest.approx(math.cos(ang), abs=1e-7)
        assert float(r.sin[pos, i]) == pytest.approx(math.sin(ang), abs=1e-7)
    assert build("position", RopeSpec(head_dim=48, rotary_dim=32, theta=5e5, max_position=300), rt).cos is r.cos
    with pytest.raises(ValueError):
        build("position", RopeSpec(head_dim=16, rotary_dim=18, theta=1e4, max_position=8), rt)


def test_library_products_of_many_rows_are_planned_once_per_shape_and_stay_right(fw):
    """A product of many rows goes to the vendor library directly; the first product of a shape measures the library's
    candidates (with tuning on) and keeps a plan; what it computes equals the plain product before and after."""
    from gesso_amd.kernels import ops
    from gesso_amd.parts import Runtime, RuntimeOptions
    g = gen(11)
    x = torch.randn(512, 384, generator=g).bfloat16()
    w = (torch.randn(320, 384, generator=g) / math.sqrt(384)).bfloat16()
    want = x.double() @ w.double().T
    rt = Runtime(DEV, torch.bfloat16, RuntimeOptions(tune_library=True))
    before = ops.library_gemm_plan(512, 320, 384)[0]
    for _ in range(3):
        got = rt.linear(x.to(DEV), w.to(DEV)).double().cpu()
        assert float((got - want).abs().max()) <= tol(torch.bfloat16, want)
    plans, candidates, best_us = ops.library_gemm_plan(512, 320, 384)
    assert plans == before + 1 and candidates >= 1 and best_us > 0
    # rows of another stride (a slice of a wider buffer), an output given, and tuning off
    wide = torch.randn(200, 768, generator=g).bfloat16().to(DEV)
    out = torch.full((200, 320), float("nan"), dtype=torch.bfloat16, device=DEV)
    plain = Runtime(DEV, torch.bfloat16, RuntimeOptions(tune_library=False))
    got = plain.linear(wide[:, :384], w.to(DEV), out=out)
    assert got is out
    ref = wide[:, :384].double().cpu() @ w.double().T
    assert float((out.double().cpu() - ref).abs().max()) <= tol(torch.bfloat16, ref)
    # a width the direct call does not take (no multiple of 8) still goes to the library, through torch
    w5 = (torch.randn(77, 384, generator=g) / math.sqrt(384)).bfloat16()
    y = rt.linear(x.to(DEV), w5.to(DEV)).double().cpu()
    assert float((y - x.double() @ w5.double().T).abs().max()) <= tol(torch.bfloat16, want)


@pytest.mark.parametrize("rows", [1, 9, 64, 65, 300])
@pytest.mark.parametrize("N,K", [(96, 64), (77, 40)])
def test_a_bfloat16_product_with_bias_sums_on_the_matrix_cores_and_rounds_once(fw, rows, N, K, monkeypatch):
    """A projection with a bias (``conv_bias: true``) takes the same matrix-core kernels as one without: float32 sums,
    then bias and one rounding.  The FMA kernel must not be what computes it where the fast kernels take the operands
    (K a multiple of 8), and the result is within half a bfloat16 step of the float64 one, which a product rounded
    before the bias would not always be."""
    from gesso_amd.kernels import ops
    from gesso_amd.parts import Runtime
    g = gen(rows + N)
    x = torch.randn(rows, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    bias = torch.randn(N, generator=g) * 3
    want = x.double() @ w.double().T + bias.double()
    rt = Runtime(DEV, torch.bfloat16)
    calls = []
    real = ops.gemm_tiled
    monkeypatch.setattr(ops, "gemm_tiled", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    out = torch.full((rows, N + 8), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = rt.linear(x.to(DEV), w.to(DEV), bias.to(DEV), out=out[:, :N])
    assert not calls
    assert torch.isnan(out[:, N:]).all()
    err = (got.double().cpu() - want).abs()
    step = 2.0 ** (torch.floor(torch.log2(want.abs().clamp_min(1e-30))) - 7)      # a bfloat16 step at each value
    assert bool((err <= 0.5 * step + 1e-4).all()), float((err / step).max())
    f32 = rt.linear(x.to(DEV), w.to(DEV), bias.to(DEV), out_dtype=torch.float32)
    assert f32.dtype == torch.float32 and float((f32.double().cpu() - want).abs().max()) <= 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part(fw, dtype):
    from gesso_amd.config import SwiGLUSpec
    h = Harness("ffn", SwiGLUSpec(hidden=80, intermediate=100), dtype)
    x = torch.randn(7, 80, generator=gen(2)).to(dtype)
    got = h.part.forward(x.to(DEV), None).double().cpu()
    w = h.tensors
    want = P.linear(P.swiglu(P.linear(x.double(), w["w1.weight"]), P.linear(x.double(), w["w3.weight"])), w["w2.weight"])
    assert float((got - want).abs().max()) <= tol(dtype, want)


# ------------------------------------------------------------------ mixers

@pytest.mark.parametrize("bias,W", [(False, 3), (True, 4), (False, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_short_conv_mixer_whole_and_in_portions(fw, dtype, bias, W):
    from gesso_amd.config import ShortConvSpec
    H = 48
    h = Harness("mixer", ShortConvSpec(hidden=H, width=W, bias=bias), dtype, seed=W)
    x = torch.randn(19, H, generator=gen(3)).to(dtype)
    w = h.tensors
    bcx = P.linear(x.double(), w["in_proj.weight"], w.get("in_proj.bias"))
    mixed, _ = P.short_conv(bcx, w["conv.weight"].reshape(H, W), w.get("conv.bias"))
    want = P.linear(mixed, w["out_proj.weight"], w.get("out_proj.bias"))
    whole = h.mixer(x, [("a", 19)])
    assert float((whole - want).abs().max()) <= tol(dtype, want)
    parts, at = [], 0
    for n in (5, 1, 1, 4, 2, 6):
        parts.append(h.mixer(x[at:at + n], [("b", n)]))
        at += n
    cut = torch.cat(parts)
    assert float((cut - want).abs().max()) <= tol(dtype, want)
    if dtype == torch.float32:
        assert torch.equal(cut, whole)             # the cut changes nothing at all


@pytest.mark.parametrize("nh,nkv,d,window,qk", [(4, 2, 16, None, True), (3, 1, 32, None, True), (3, 3, 48, 7, False),
                                                (8, 2, 64, None, True)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_mixer_whole_and_in_portions(fw, dtype, nh, nkv, d, window, qk):
    from gesso_amd.config import AttentionSpec, RMSNormSpec, RopeSpec
    H, eps, theta = nh * d, 1e-5, 1e4
    spec = AttentionSpec(hidden=H, n_heads=nh, n_kv_heads=nkv, head_dim=d, window=window,
                         position=RopeSpec(head_dim=d, rotary_dim=d, theta=theta, max_position=128),
                         qk_norm=RMSNormSpec(size=d, eps=eps) if qk else None)
    h = Harness("mixer", spec, dtype, seed=d, std=1.0 / math.sqrt(H))
    T = 29
    x = torch.randn(T, H, generator=gen(4)).to(dtype)
    w = h.tensors
    q = P.linear(x.double(), w["q_proj.weight"]).reshape(T, nh, d)
    k = P.linear(x.double(), w["k_proj.weight"]).reshape(T, nkv, d)
    v = P.linear(x.double(), w["v_proj.weight"]).reshape(T, nkv, d)
    if qk:
        q, k = P.rmsnorm(q, w["q_norm.weight"], eps), P.rmsnorm(k, w["k_norm.weight"], eps)
    q, k = P.rope(q, range(T), theta), P.rope(k, range(T), theta)
    want = P.linear(P.causal_attention(q, k, v, window or 0).reshape(T, H), w["out_proj.weight"])
    whole = h.mixer(x, [("a", T)])
    assert float((whole - want).abs().max()) <= tol(dtype, want)
    parts, at = [], 0
    for n in (7, 1, 9, 2, 1, 1, 8):
        parts.append(h.mixer(x[at:at + n], [("b", n)]))
        at += n
    cut = torch.cat(parts)
    assert float((cut - want).abs().max()) <= tol(dtype, want)
    if dtype == torch.float32:
        assert torch.equal(cut, whole)
    if window:
        # the windowed group gave pages back as it went: 29 tokens, window 7, pages of 8
        held = [p for p in h.manager.get("b").tables[0] if p >= 0]
        assert len(held) <= 2


@dataclasses.dataclass(frozen=True)
class LatentSpec:
    hidden: int
    latent: int
    value: int                      # 0: no value rows, values are the latent rows themselves
    kind: str = "toy_latent"


@pytest.mark.parametrize("value", [0, 40])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_toy_mixer_whose_cache_rows_are_not_keys_and_values_of_one_width(fw, dtype, value):
    """A mixer defined here that caches one latent row of 24 numbers per token and either no value rows at all
    (``value_dim=0``: it attends with the latent rows and sums them) or value rows of another width (40): the cache
    manager gives its layer pages, the storage a key pool of the one width and a value pool of the other (or an empty
    one), the block table addresses both; stepped whole and in portions against the arithmetic written out."""
    from gesso_amd.parts import MATRIX, PagedKV, Part, TensorSpec, register, unregister

    class LatentMixer(Part):
        @staticmethod
        def tensor_specs(spec):
            out = {"down.weight": TensorSpec((spec.latent, spec.hidden), MATRIX),
                   "query.weight": TensorSpec((spec.latent, spec.hidden), MATRIX),
                   "out.weight": TensorSpec((spec.hidden, spec.value or spec.latent), MATRIX)}
            if spec.value:
                out["value.weight"] = TensorSpec((spec.value, spec.hidden), MATRIX)
            return out

        @staticmethod
        def cache_need(spec):
            return PagedKV(1, spec.latent, None, value_dim=spec.value)

        def bind(self, tensors):
            self.w = tensors

        def forward(self, x, ctx, cache):
            s = self.spec
            assert cache.k.shape[1:] == (1, cache.page_size, s.latent) and cache.v.shape[1:] == (1, cache.page_size, s.value)
            c = self.rt.linear(x, self.w["down.weight"])
            q = self.rt.linear(x, self.w["query.weight"]).float()
            v = self.rt.linear(x, self.w["value.weight"]) if s.value else None
            pos, seq = ctx.positions.long(), ctx.seq_of_token.long()
            page = cache.block_table.long()[seq, pos // cache.page_size]
            cache.k[page, 0, pos % cache.page_size] = c
            if s.value:
                cache.v[page, 0, pos % cache.page_size] = v
            rows = []
            for t in range(x.shape[0]):
                u = torch.arange(int(pos[t]) + 1, device=x.device)
                pg = cache.block_table.long()[seq[t], u // cache.page_size]
                keys = cache.k[pg, 0, u % cache.page_size].float()
                vals = cache.v[pg, 0, u % cache.page_size].float() if s.value else keys
                p = torch.softmax(keys @ q[t] / math.sqrt(s.latent), dim=0)
                rows.append(p @ vals)
            return self.rt.linear(torch.stack(rows).to(x.dtype), self.w["out.weight"])

    register("mixer", "toy_latent", LatentMixer, replace=True)
    try:
        H, L = 48, 24
        h = Harness("mixer", LatentSpec(H, L, value), dtype, seed=3 + value, std=0.3)
        assert h.storage.keys[0].shape[-1] == L and h.storage.values[0].shape[-1] == value
        T = 21
        x = torch.randn(T, H, generator=gen(8)).to(dtype)
        w = h.tensors
        c = x.double() @ w["down.weight"].T
        q = x.double() @ w["query.weight"].T
        vals = x.double() @ w["value.weight"].T if value else c
        want = torch.stack([torch.softmax(c[:t + 1] @ q[t] / math.sqrt(L), dim=0) @ vals[:t + 1] for t in range(T)])
        want = want @ w["out.weight"].T
        whole = h.mixer(x, [("a", T)])
        assert float((whole - want).abs().max()) <= tol(dtype, want)
        parts, at = [], 0
        for n in (5, 1, 9, 2, 4):
            parts.append(h.mixer(x[at:at + n], [("b", n)]))
            at += n
        assert float((torch.cat(parts) - want).abs().max()) <= tol(dtype, want)
        h.manager.release("a")
        h.manager.release("b")
        h.manager.check()
        assert h.manager.stats()["pages_free"] == [32]
    finally:
        unregister("mixer", "toy_latent")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_alone(fw, dtype):
    from gesso_amd.config import BlockSpec, RMSNormSpec, ShortConvSpec, SwiGLUSpec
    from gesso_amd.parts import ResidualStream
    H = 32
    spec = BlockSpec(mixer=ShortConvSpec(hidden=H, width=3), mixer_norm=RMSNormSpec(H, 1e-5),
                     ffn=SwiGLUSpec(hidden=H, intermediate=40), ffn_norm=RMSNormSpec(H, 1e-5))
    h = Harness("block", spec, dtype, std=0.2)
    x = torch.randn(9, H, generator=gen(5))
    w = {"p." + {"mixer_norm.weight": "operator_norm.weight", "ffn_norm.weight": "ffn_norm.weight"}.get(k, k)
         .replace("mixer.", "conv.").replace("ffn.w", "feed_forward.w"): v for k, v in h.tensors.items()}
    hh, _ = P.conv_block(x.double(), w, "p.", 1e-5)
    want = P.feed_forward_block(hh, w, "p.", 1e-5)
    c = h.ctx([("a", 9)])
    stream = ResidualStream(x.clone().to(DEV))
    h.part.forward(stream, c, c.cache_view(0))
    got = stream.res.double().cpu() + stream.pending.double().cpu()
    assert float((got - want).abs().max()) <= tol(dtype, want)


# ------------------------------------------------------------------ parts the framework has never seen

@dataclasses.dataclass(frozen=True)
class DecaySpec:
    hidden: int
    decay: float
    kind: str = "toy_decay"


@dataclasses.dataclass(frozen=True)
class RoutedSpec:
    hidden: int
    experts: int
    inner: int
    kind: str = "toy_routed"


def register_toys():
    from gesso_amd.parts import MATRIX, Part, SlotState, TensorSpec, register

    class RoutedFFN(Part):
        """A feed-forward with routing: router logits in float32, the best expert per token, relu(x U^T) D^T of that
        expert alone, weighted by the softmax weight of the choice."""

        @staticmethod
        def tensor_specs(spec):
            out = {"router.weight": TensorSpec((spec.experts, spec.hidden), MATRIX)}
            for e in range(spec.experts):
                out[f"e{e}.up.weight"] = TensorSpec((spec.inner, spec.hidden), MATRIX)
                out[f"e{e}.down.weight"] = TensorSpec((spec.hidden, spec.inner), MATRIX)
            return out

        def bind(self, tensors):
            self.router = tensors["router.weight"]
            self.up = [tensors[f"e{e}.up.weight"] for e in range(self.spec.experts)]
            self.down = [tensors[f"e{e}.down.weight"] for e in range(self.spec.experts)]

        def forward(self, x, ctx):
            logits = self.rt.linear(x, self.router, out_dtype=torch.float32)
            gate, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            out = torch.zeros((x.shape[0], self.spec.hidden), dtype=torch.float32, device=x.device)
            for e in range(self.spec.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    h = torch.relu(self.rt.linear(x[rows].contiguous(), self.up[e]))
                    out[rows] = self.rt.linear(h, self.down[e]).float() * gate[rows, None]
            return out.to(x.dtype)

    class DecayMixer(Part):
        """s_t = decay * s_{t-1} + x_t W^T from s_{-1} = 0.25, output s_t (1 + t / 64): a running state per request in
        float32 that starts from a value other than zero, and a count of the tokens seen, kept in bfloat16 (whole
        numbers up to 256 are exact there)."""

        @staticmethod
        def tensor_specs(spec):
            return {"proj.weight": TensorSpec((spec.hidden, spec.hidden), MATRIX)}

        @staticmethod
        def cache_need(spec):
            return SlotState((("running", (spec.hidden,), "float32", 0.25), ("seen", (1,), "bfloat16")))

        def bind(self, tensors):
            self.w = tensors["proj.weight"]

        def forward(self, x, ctx, cache):
            y = self.rt.linear(x, self.w).float()
            state, seen = cache.state["running"], cache.state["seen"]
            assert state.dtype == torch.float32 and seen.dtype == torch.bfloat16
            out = torch.empty_like(y)
            slots = ctx.slots.tolist()
            at = 0
            for slot, n in zip(slots, ctx.q_lens):
                s, c = state[slot], float(seen[slot, 0])
                for t in range(at, at + n):
                    s = self.spec.decay * s + y[t]
                    out[t] = s * (1.0 + c / 64.0)
                    c += 1.0
                state[slot] = s
                seen[slot, 0] = c
                at += n
            return out.to(x.dtype)

    class ScaledRope(Part):
        """Another position encoding: position p rotates by the angle of 4 p, and the pairs are (2i, 2i + 1)."""

        layout = "interleaved"

        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            from gesso_amd.parts.rope import rope_tables
            cos, sin = rope_tables(spec.rotary_dim, spec.theta, spec.max_position * 4)
            self.rotary_dim = spec.rotary_dim
            self.cos = cos[::4].contiguous().to(rt.device)
            self.sin = sin[::4].contiguous().to(rt.device)

    register("mixer", "toy_decay", DecayMixer, replace=True)
    register("position", "toy_scaled_rope", ScaledRope, replace=True)
    register("ffn", "toy_routed", RoutedFFN, replace=True)


def toy_spec():
    from gesso_amd.config import AttentionSpec, BlockSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, SwiGLUSpec
    H, V = 32, 40
    norm = RMSNormSpec(H, 1e-5)
    pos = dataclasses.replace(RopeSpec(head_dim=16, rotary_dim=16, theta=1e4, max_position=64), kind="toy_scaled_rope")
    attn = AttentionSpec(hidden=H, n_heads=2, n_kv_heads=1, head_dim=16, position=pos, qk_norm=None)
    ffn = SwiGLUSpec(hidden=H, intermediate=24)
    routed = RoutedSpec(hidden=H, experts=3, inner=16)
    routed_names = ["router.weight"] + [f"e{e}.{k}.weight" for e in range(3) for k in ("up", "down")]

    def names(i, mixer_names):
        n = {"mixer_norm.weight": f"L{i}.n1", "ffn_norm.weight": f"L{i}.n2", "ffn.w1.weight": f"L{i}.w1",
             "ffn.w3.weight": f"L{i}.w3", "ffn.w2.weight": f"L{i}.w2"}
        n.update({f"mixer.{k}": f"L{i}.{k}" for k in mixer_names})
        return n

    attn_names = ["q_proj.weight", "k_proj.weight", "v_proj.weight", "out_proj.weight"]
    n1 = {k: v for k, v in names(1, attn_names).items() if not k.startswith("ffn.")}
    n1.update({f"ffn.{k}": f"L1.{k}" for k in routed_names})
    blocks = (BlockSpec(DecaySpec(H, 0.5), norm, ffn, norm, names(0, ["proj.weight"])),
              BlockSpec(attn, norm, routed, norm, n1),
              BlockSpec(attn, norm, None, None, {k: v for k, v in names(2, attn_names).items() if not k.startswith("ffn")}))
    # block 0 runs twice (two states of its own); the last call reads the cache that call 1 wrote
    schedule = (LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(2, cache=1))
    return ModelSpec(architecture="ToyForTests", hidden=H, vocab=V, blocks=blocks, schedule=schedule, final_norm=norm,
                     tie_embeddings=True, max_position=64, names={"embed": "emb", "final_norm.weight": "fn", "head": "head"},
                     embed_scale=1.5, logit_softcap=3.0)


def rope_interleaved(x, positions, theta):
    """Pairs ``(2i, 2i + 1)`` at angle ``pos * theta^(-2i/d)``: the reference's ``interleaved=true``
    (``src/Operators/cpu.jl:357-371``)."""
    T, _, d = x.shape
    out = x.clone()
    for t in range(T):
        for i in range(d // 2):
            ang = float(positions[t]) * float(theta) ** (-2.0 * i / d)
            c, s = math.cos(ang), math.sin(ang)
            a, b = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            out[t, :, 2 * i] = a * c - b * s
            out[t, :, 2 * i + 1] = a * s + b * c
    return out


def toy_plain(w, ids, margins=None):
    """The toy model by hand, whole sequence, float64.  ``margins`` collects, per routed layer, the least distance
    between a token's best and second-best expert (a choice that near a tie may fall either way in bfloat16)."""
    T = len(ids)
    margins = [] if margins is None else margins
    h = P.embedding(w["emb"], ids) * 1.5
    eps = 1e-5

    def decay_block(h, i):
        y = P.linear(P.rmsnorm(h, w[f"L{i}.n1"], eps), w[f"L{i}.proj.weight"])
        s, out = torch.full((h.shape[1],), 0.25, dtype=h.dtype), []
        for t in range(T):
            s = 0.5 * s + y[t]
            out.append(s * (1.0 + t / 64.0))
        return h + torch.stack(out)

    def ffn(h, i):
        n = P.rmsnorm(h, w[f"L{i}.n2"], eps)
        return h + P.linear(P.swiglu(P.linear(n, w[f"L{i}.w1"]), P.linear(n, w[f"L{i}.w3"])), w[f"L{i}.w2"])

    def routed_ffn(h, i, margins):
        n = P.rmsnorm(h, w[f"L{i}.n2"], eps)
        prob = torch.softmax(P.linear(n, w[f"L{i}.router.weight"]), dim=-1)
        top = prob.sort(dim=-1, descending=True).values
        margins.append(float((top[:, 0] - top[:, 1]).min()))
        gate, choice = prob.max(dim=-1)
        out = torch.zeros_like(h)
        for t in range(T):
            e = int(choice[t])
            out[t] = P.linear(torch.relu(P.linear(n[t:t + 1], w[f"L{i}.e{e}.up.weight"])), w[f"L{i}.e{e}.down.weight"])[0] * gate[t]
        return h + out

    def qkv(h, i):
        n = P.rmsnorm(h, w[f"L{i}.n1"], eps)
        q = P.linear(n, w[f"L{i}.q_proj.weight"]).reshape(T, 2, 16)
        k = P.linear(n, w[f"L{i}.k_proj.weight"]).reshape(T, 1, 16)
        v = P.linear(n, w[f"L{i}.v_proj.weight"]).reshape(T, 1, 16)
        pos = [4 * t for t in range(T)]                      # the scaled encoding: table row p is angle of 4 p
        return rope_interleaved(q, pos, 1e4), rope_interleaved(k, pos, 1e4), v

    h = ffn(decay_block(h, 0), 0)
    q1, k1, v1 = qkv(h, 1)
    h = routed_ffn(h + P.linear(P.causal_attention(q1, k1, v1).reshape(T, 32), w["L1.out_proj.weight"]), 1, margins)
    h = ffn(decay_block(h, 0), 0)
    q2, _, _ = qkv(h, 2)                                     # its own queries over layer 1's keys and values
    h = h + P.linear(P.causal_attention(q2, k1, v1).reshape(T, 32), w["L2.out_proj.weight"])
    return 3.0 * torch.tanh(P.linear(P.rmsnorm(h, w["fn"], eps), w["emb"]) / 3.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_parts_register_build_and_step(fw, dtype):
    from gesso_amd import Engine, StepEntry
    from gesso_amd.models.model import tensor_table
    from gesso_amd.parts import unregister
    from gesso_amd.weights import random_tensors
    from gesso_amd.weights.loader import held_dtype

    register_toys()
    try:
        spec = toy_spec()
        table = tensor_table(spec)
        assert "L0.proj.weight" in table and "L2.w1" not in table and "L1.e2.down.weight" in table and "L1.w1" not in table
        cpu = random_tensors(table, 17, dtype, std=0.2)          # a seed whose routing choices are clear of ties
        from gesso_amd.parts import RuntimeOptions
        eng = Engine(spec, {k: v.to(DEV, held_dtype(v.dtype, table[k].role, dtype)) for k, v in cpu.items()}, dtype,
                     DEV, page_size=4, num_pages=24, num_slots=3, options=RuntimeOptions(record_portions=True))
        # parts that say nothing about recorded steps are never recorded, whatever the options ask for
        assert eng.recorder is None and not eng.model.portions_recordable
        lay = eng.manager.layout
        assert len(lay.paged) == 1 and lay.paged[0].members == (1,) and [m.call for m in lay.slots] == [0, 2]
        assert lay.source_of_call[3] == 1
        ids = {"a": [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7], "b": [2, 7, 1, 8, 2, 8, 1, 8, 2, 8, 4]}
        w64 = {k: v.double() for k, v in cpu.items()}
        margins = []
        want = {k: toy_plain(w64, v, margins) for k, v in ids.items()}
        assert min(margins) > 0.02, "the fixed weights and ids keep every routing choice clear of a tie"

        t = (2e-5 if dtype == torch.float32 else 3e-2) * max(1.0, max(float(x.abs().max()) for x in want.values()))
        # whole
        for k, v in ids.items():
            eng.add_request(k)
            got = eng.step([StepEntry(k, v, list(range(len(v))))]).double().cpu()
            eng.finish_request(k)
            assert float((got - want[k]).abs().max()) <= t, k
        # mixed and cut: a in portions 5, 1, 1, 7 beside b in 3, 6, 1, 1
        eng.add_request("a"); eng.add_request("b")
        got = {"a": [], "b": []}
        cuts = {"a": [5, 1, 1, 7], "b": [3, 6, 1, 1]}
        at = {"a": 0, "b": 0}
        for s in range(4):
            entries = []
            for k in ("a", "b"):
                n = cuts[k][s]
                entries.append(StepEntry(k, ids[k][at[k]:at[k] + n], list(range(n))))
                at[k] += n
            lg = eng.step(entries).double().cpu()
            o = 0
            for e in entries:
                got[e.rid].append(lg[o:o + len(e.tokens)])
                o += len(e.tokens)
        for k in ids:
            assert float((torch.cat(got[k]) - want[k]).abs().max()) <= t, k
        eng.finish_request("a"); eng.finish_request("b")
        assert eng.manager.stats()["pages_free"] == [24] and eng.manager.stats()["slots_free"] == 3
    finally:
        unregister("mixer", "toy_decay")
        unregister("position", "toy_scaled_rope")
        unregister("ffn", "toy_routed")


def test_a_toy_architecture_goes_from_its_folder_to_tokens(fw, tmp_path):
    """Another architecture is a typed configuration, a function from it to a model spec and one call of
    `register_architecture`: here the toy model above gets a configuration of two keys, a folder is written for it with
    seeded weights, `Session` loads the folder by the name in its config.json and generates greedily (prompt in
    portions, recorded decode steps or not: the toy mixer decides), and the tokens are the plain toy model's."""
    from gesso_amd import Session
    from gesso_amd.config import register_architecture, unregister_architecture
    from gesso_amd.parts import unregister
    from gesso_amd.weights import write_model_folder
    from gesso_amd.weights.safetensors_io import SafetensorsFile

    @dataclasses.dataclass(frozen=True)
    class ToyConfig:
        decay: float = 0.5
        max_position_embeddings: int = 64

        def to_json(self):
            return {"architectures": ["ToyForTests"], "decay": self.decay, "max_position_embeddings": self.max_position_embeddings}

    def parse(raw):
        assert set(raw) == {"architectures", "decay", "max_position_embeddings"}
        return ToyConfig(float(raw["decay"]), int(raw["max_position_embeddings"]))

    register_toys()
    register_architecture("ToyForTests", parse, lambda c: toy_spec(), lambda c: c.to_json())
    try:
        folder = write_model_folder(str(tmp_path / "toy"), ToyConfig(), seed=30, dtype=torch.float32, std=0.2)
        stored = SafetensorsFile(os.path.join(folder, "model.safetensors"))
        w64 = {k: stored.tensor(k).double() for k in stored.names()}
        stored.close()
        prompt = [3, 1, 4, 1, 5, 9, 2, 6, 5]
        want, margins = list(prompt), []
        for _ in range(5):
            logits = toy_plain(w64, want, [])[-1]
            top = logits.topk(2).values
            margins.append(float(top[0] - top[1]))
            want.append(int(logits.argmax()))
        assert min(margins) > 1e-3, "the seed keeps the greedy choices clear of ties"
        sess = Session(folder, dtype="float32", context_length=64, page_size=4, chunk_size=4, max_num_seqs=2)
        assert sess.engine.spec.architecture == "ToyForTests"
        got = sess.generate([prompt], max_new_tokens=5)[0]
        assert got == want
        sess.close()
    finally:
        unregister_architecture("ToyForTests")
        unregister("mixer", "toy_decay")
        unregister("position", "toy_scaled_rope")
        unregister("ffn", "toy_routed")



@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_toy_norm_and_a_toy_block_arrangement_register_build_and_step(fw, dtype):
    """The two kinds of part that the other toy tests leave out.  A norm that centres its rows and has a bias (no
    ``row_weight``: nothing may pre-weight rows for it) serves as a block's norm, beside an RMSNorm in the same block,
    and as the model's last norm (with ``rows``).  A block arrangement that feeds one normed input to the mixer and to
    the feed-forward at once and adds both (no ``first_norm`` hint) runs before an ordinary block.  Registered from
    here, built by kind, stepped whole and in portions beside another request, against the arithmetic written out."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.config import AttentionSpec, BlockSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, ShortConvSpec, SwiGLUSpec
    from gesso_amd.models.model import tensor_table
    from gesso_amd.parts import VECTOR, Part, TensorSpec, register, unregister
    from gesso_amd.parts.registry import build, part_class
    from gesso_amd.weights import random_tensors
    from gesso_amd.weights.loader import held_dtype

    @dataclasses.dataclass(frozen=True)
    class CenteredSpec:
        size: int
        eps: float
        kind: str = "toy_centered"

    @dataclasses.dataclass(frozen=True)
    class ParallelSpec:
        mixer: object
        norm: object
        ffn: object
        names: dict = dataclasses.field(compare=False, hash=False, default_factory=dict)
        kind: str = "toy_parallel"

    class CenteredNorm(Part):
        @staticmethod
        def tensor_specs(spec):
            return {"weight": TensorSpec((spec.size,), VECTOR, "one_plus_normal"), "bias": TensorSpec((spec.size,), VECTOR)}

        def bind(self, tensors):
            self.weight, self.bias = tensors["weight"], tensors["bias"]

        def add_norm(self, stream, rows=None, out=None):
            stream.flush(self.rt)
            x = stream.res if rows is None else stream.res[rows.long()]
            x = x - x.mean(-1, keepdim=True)
            y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.spec.eps) * self.weight + self.bias
            return y.to(self.rt.dtype)

    class ParallelBlock(Part):
        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            self.norm, self.mixer, self.ffn = build("norm", spec.norm, rt), build("mixer", spec.mixer, rt), build("ffn", spec.ffn, rt)

        @staticmethod
        def tensor_specs(spec):
            return {f"{role}.{k}": ts for role, cat, sub in (("norm", "norm", spec.norm), ("mixer", "mixer", spec.mixer),
                                                             ("ffn", "ffn", spec.ffn))
                    for k, ts in part_class(cat, sub).tensor_specs(sub).items()}

        @staticmethod
        def cache_need(spec):
            return part_class("mixer", spec.mixer).cache_need(spec.mixer)

        def bind(self, tensors):
            from gesso_amd.parts.base import sub_tensors
            for role in ("norm", "mixer", "ffn"):
                getattr(self, role).bind(sub_tensors(tensors, role))

        def forward(self, stream, ctx, cache):
            x = self.norm.add_norm(stream)
            stream.push(self.mixer.forward(x, ctx, cache), self.rt)
            stream.push(self.ffn.forward(x, ctx), self.rt)

    H, V, eps = 48, 56, 1e-4
    centered = CenteredSpec(H, eps)
    attn = AttentionSpec(hidden=H, n_heads=3, n_kv_heads=1, head_dim=16, qk_norm=None,
                         position=RopeSpec(head_dim=16, rotary_dim=16, theta=1e4, max_position=64))
    b0 = ParallelSpec(attn, centered, SwiGLUSpec(hidden=H, intermediate=40),
                      {**{f"mixer.{k}_proj.weight": f"A.{k}" for k in ("q", "k", "v", "out")}, "norm.weight": "A.nw",
                       "norm.bias": "A.nb", "ffn.w1.weight": "A.w1", "ffn.w3.weight": "A.w3", "ffn.w2.weight": "A.w2"})
    b1 = BlockSpec(ShortConvSpec(hidden=H, width=3), centered, SwiGLUSpec(hidden=H, intermediate=24), RMSNormSpec(H, 1e-5),
                   {"mixer.in_proj.weight": "B.in", "mixer.conv.weight": "B.taps", "mixer.out_proj.weight": "B.out",
                    "mixer_norm.weight": "B.nw", "mixer_norm.bias": "B.nb", "ffn_norm.weight": "B.n2",
                    "ffn.w1.weight": "B.w1", "ffn.w3.weight": "B.w3", "ffn.w2.weight": "B.w2"})
    spec = ModelSpec(architecture="ToyNormsAndBlocks", hidden=H, vocab=V, blocks=(b0, b1), schedule=(LayerCall(0), LayerCall(1)),
                     final_norm=centered, tie_embeddings=False, max_position=64,
                     names={"embed": "emb", "head": "head", "final_norm.weight": "fw", "final_norm.bias": "fb"})

    def centered_norm(x, w, b):
        x = x - x.mean(-1, keepdim=True)
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w + b

    def plain(w, ids):
        T = len(ids)
        h = P.embedding(w["emb"], ids)
        n = centered_norm(h, w["A.nw"], w["A.nb"])
        pos = list(range(T))
        q = P.rope(P.linear(n, w["A.q"]).reshape(T, 3, 16), pos, 1e4)
        k = P.rope(P.linear(n, w["A.k"]).reshape(T, 1, 16), pos, 1e4)
        v = P.linear(n, w["A.v"]).reshape(T, 1, 16)
        mixed = P.linear(P.causal_attention(q, k, v).reshape(T, 48), w["A.out"])
        fed = P.linear(P.swiglu(P.linear(n, w["A.w1"]), P.linear(n, w["A.w3"])), w["A.w2"])
        h = h + mixed + fed
        n = centered_norm(h, w["B.nw"], w["B.nb"])
        u, _ = P.short_conv(P.linear(n, w["B.in"]), w["B.taps"].reshape(H, 3))
        h = h + P.linear(u, w["B.out"])
        n = P.rmsnorm(h, w["B.n2"], 1e-5)
        h = h + P.linear(P.swiglu(P.linear(n, w["B.w1"]), P.linear(n, w["B.w3"])), w["B.w2"])
        return P.linear(centered_norm(h, w["fw"], w["fb"]), w["head"])

    register("norm", "toy_centered", CenteredNorm, replace=True)
    register("block", "toy_parallel", ParallelBlock, replace=True)
    try:
        table = tensor_table(spec)
        assert {"A.nb", "B.nb", "fb", "A.q", "B.taps", "head"} <= set(table) and "A.n2" not in table
        cpu = random_tensors(table, 5, dtype, std=0.2)
        eng = Engine(spec, {k: v.to(DEV, held_dtype(v.dtype, table[k].role, dtype)) for k, v in cpu.items()}, dtype,
                     DEV, page_size=4, num_pages=16, num_slots=3)
        assert not eng.model.graph_safe          # the toy parts do not say that they may be recorded
        w64 = {k: v.double() for k, v in cpu.items()}
        ids = {"a": [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9], "b": [2, 7, 1, 8, 2, 8, 1, 8, 2]}
        want = {k: plain(w64, v) for k, v in ids.items()}
        # the bias and the centring matter: the same rows through an RMSNorm in their place are far off
        off = P.linear(P.rmsnorm(P.embedding(w64["emb"], ids["a"]), w64["fw"], eps), w64["head"])
        t = (2e-5 if dtype == torch.float32 else 3e-2) * max(1.0, max(float(x.abs().max()) for x in want.values()))
        assert float((off - want["a"]).abs().max()) > 20 * t
        eng.add_request("a")
        got = eng.step([StepEntry("a", ids["a"], list(range(13)))]).double().cpu()
        eng.finish_request("a")
        assert float((got - want["a"]).abs().max()) <= t
        # a in portions 6, 1, 6 beside b in 2, 6, 1; only some places wanted (the last norm gets ``rows``)
        eng.add_request("a"); eng.add_request("b")
        at = {"a": 0, "b": 0}
        for na, nb in ((6, 2), (1, 6), (6, 1)):
            ea = StepEntry("a", ids["a"][at["a"]:at["a"] + na], [na - 1])
            eb = StepEntry("b", ids["b"][at["b"]:at["b"] + nb], [0, nb - 1])
            lg = eng.step([ea, eb]).double().cpu()
            rows = torch.stack([want["a"][at["a"] + na - 1], want["b"][at["b"]], want["b"][at["b"] + nb - 1]])
            assert float((lg - rows).abs().max()) <= t, (na, nb)
            at["a"] += na; at["b"] += nb
        # decoding goes step by step where a part cannot be recorded, through the same entry point
        out, bad = eng.decode(["a", "b"], [7, 11], 2)
        assert not bad.any()
        lg = plain(w64, ids["a"] + [7])[-1]
        assert int(out[0, 0]) == int(lg.argmax()) or float(lg.topk(2).values.diff().abs()) < 2 * t
        eng.finish_request("a"); eng.finish_request("b")
        assert eng.manager.stats()["pages_free"] == [16] and eng.manager.stats()["slots_free"] == 3
    finally:
        unregister("norm", "toy_centered")
        unregister("block", "toy_parallel")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_model_with_a_full_and_a_windowed_attention_layer_runs_on_two_page_groups(fw, dtype):
    """Layers with different needs keep pages of their own: one attention layer sees all keys, one only the last 10,
    a short convolution keeps a slot.  With pages of 4 the windowed group gives pages back as the window passes them,
    to the other request among others; what is given back is filled with NaN (``poison``), so a kernel that read a key
    before the window, through a stale table entry or a page that now belongs to someone else, shows in the logits.
    Whole, in portions beside another request, and through the recorded decode loop (heads of 64: the fast kernels in
    bfloat16), against the arithmetic written out."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.config import AttentionSpec, BlockSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, ShortConvSpec, SwiGLUSpec
    from gesso_amd.models.model import tensor_table
    from gesso_amd.weights import random_tensors
    from gesso_amd.weights.loader import held_dtype

    H, V, eps, W = 128, 72, 1e-5, 10
    norm = RMSNormSpec(H, eps)
    rope = RopeSpec(head_dim=64, rotary_dim=64, theta=1e4, max_position=128)
    full = AttentionSpec(hidden=H, n_heads=2, n_kv_heads=1, head_dim=64, position=rope, qk_norm=RMSNormSpec(64, eps))
    near = AttentionSpec(hidden=H, n_heads=2, n_kv_heads=2, head_dim=64, position=rope, qk_norm=None, window=W)

    def names(i, mixer_names, ffn=True):
        n = {f"mixer.{k}": f"L{i}.{k}" for k in mixer_names}
        n["mixer_norm.weight"] = f"L{i}.n1"
        if ffn:
            n.update({"ffn_norm.weight": f"L{i}.n2", "ffn.w1.weight": f"L{i}.w1", "ffn.w3.weight": f"L{i}.w3", "ffn.w2.weight": f"L{i}.w2"})
        return n

    proj = ["q_proj.weight", "k_proj.weight", "v_proj.weight", "out_proj.weight"]
    blocks = (BlockSpec(full, norm, SwiGLUSpec(H, 96), norm, names(0, proj + ["q_norm.weight", "k_norm.weight"])),
              BlockSpec(near, norm, SwiGLUSpec(H, 64), norm, names(1, proj)),
              BlockSpec(ShortConvSpec(H, 3), norm, None, None, names(2, ["in_proj.weight", "conv.weight", "out_proj.weight"], False)))
    spec = ModelSpec(architecture="ToyTwoGroups", hidden=H, vocab=V, blocks=blocks,
                     schedule=(LayerCall(0), LayerCall(1), LayerCall(2)), final_norm=norm, tie_embeddings=True,
                     max_position=128, names={"embed": "emb", "final_norm.weight": "fn"})

    def attention(h, w, i, nkv, window, qk):
        T = h.shape[0]
        n = P.rmsnorm(h, w[f"L{i}.n1"], eps)
        q = P.linear(n, w[f"L{i}.q_proj.weight"]).reshape(T, 2, 64)
        k = P.linear(n, w[f"L{i}.k_proj.weight"]).reshape(T, nkv, 64)
        v = P.linear(n, w[f"L{i}.v_proj.weight"]).reshape(T, nkv, 64)
        if qk:
            q, k = P.rmsnorm(q, w[f"L{i}.q_norm.weight"], eps), P.rmsnorm(k, w[f"L{i}.k_norm.weight"], eps)
        q, k = P.rope(q, range(T), 1e4), P.rope(k, range(T), 1e4)
        h = h + P.linear(P.causal_attention(q, k, v, window).reshape(T, H), w[f"L{i}.out_proj.weight"])
        n = P.rmsnorm(h, w[f"L{i}.n2"], eps)
        return h + P.linear(P.swiglu(P.linear(n, w[f"L{i}.w1"]), P.linear(n, w[f"L{i}.w3"])), w[f"L{i}.w2"])

    def plain(w, ids):
        h = attention(attention(P.embedding(w["emb"], ids), w, 0, 1, 0, True), w, 1, 2, W, False)
        n = P.rmsnorm(h, w["L2.n1"], eps)
        u, _ = P.short_conv(P.linear(n, w["L2.in_proj.weight"]), w["L2.conv.weight"].reshape(H, 3))
        h = h + P.linear(u, w["L2.out_proj.weight"])
        return P.linear(P.rmsnorm(h, w["fn"], eps), w["emb"])

    table = tensor_table(spec)
    cpu = random_tensors(table, 23, dtype, std=0.15)
    w64 = {k: v.double() for k, v in cpu.items()}
    eng = Engine(spec, {k: v.to(DEV, held_dtype(v.dtype, table[k].role, dtype)) for k, v in cpu.items()}, dtype, DEV,
                 page_size=4, num_pages=32, num_slots=3, max_context=96, poison=True)
    lay = eng.manager.layout
    assert [g.need.window for g in lay.paged] == [None, W] and len(lay.slots) == 1
    g = gen(31)
    ids = {"a": torch.randint(0, V, (41,), generator=g).tolist(), "b": torch.randint(0, V, (30,), generator=g).tolist()}
    want = {k: plain(w64, v) for k, v in ids.items()}
    # the window matters: with all keys the last logits are far off
    t = (3e-5 if dtype == torch.float32 else 3e-2) * max(1.0, max(float(x.abs().max()) for x in want.values()))
    h_all = attention(attention(P.embedding(w64["emb"], ids["a"]), w64, 0, 1, 0, True), w64, 1, 2, 0, False)
    h_win = attention(attention(P.embedding(w64["emb"], ids["a"]), w64, 0, 1, 0, True), w64, 1, 2, W, False)
    assert float((h_all - h_win).abs().max()) > 1e-2

    eng.add_request("a")
    got = eng.step([StepEntry("a", ids["a"], list(range(41)))]).double().cpu()
    assert float((got - want["a"]).abs().max()) <= t
    held = [[p for p in tb if p >= 0] for tb in eng.manager.get("a").tables]
    assert len(held[0]) == 11 and len(held[1]) <= 4          # 41 tokens: all pages of group 0, the window's of group 1
    eng.finish_request("a")
    # portions beside each other: what a's window leaves behind, b takes, and the other way round
    eng.add_request("a"); eng.add_request("b")
    cuts = {"a": [9, 1, 13, 2, 8, 8], "b": [2, 7, 1, 11, 3, 6]}
    at = {"a": 0, "b": 0}
    out = {"a": [], "b": []}
    for s in range(6):
        entries = []
        for k in ("a", "b"):
            n = cuts[k][s]
            entries.append(StepEntry(k, ids[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
        lg = eng.step(entries).double().cpu()
        assert bool(torch.isfinite(lg).all()), s
        o = 0
        for e in entries:
            out[e.rid].append(lg[o:o + len(e.tokens)])
            o += len(e.tokens)
        eng.manager.check()
    for k in ids:
        assert float((torch.cat(out[k]) - want[k][:at[k]]).abs().max()) <= t, k
    assert at == {"a": 41, "b": 30}
    # the recorded loop: 20 steps from the greedy choice, past several more pages of the window
    first = [int(want["a"][-1].argmax()), int(want["b"][-1].argmax())]
    chosen, bad = eng.decode(["a", "b"], first, 20)
    assert not bad.any()
    eng.manager.check()
    for col, k in enumerate(("a", "b")):
        seq = ids[k] + [first[col]] + [int(x) for x in chosen[:-1, col]]
        ref = plain(w64, seq)[len(ids[k]):]
        for s in range(20):
            top = ref[s].topk(2).values
            assert int(chosen[s, col]) == int(ref[s].argmax()) or float(top[0] - top[1]) < 2 * t, (k, s)
        assert len([p for p in eng.manager.get(k).tables[1] if p >= 0]) <= 4
    eng.finish_request("a"); eng.finish_request("b")
    st = eng.manager.stats()
    assert st["pages_free"] == [32, 32] and st["slots_free"] == 3
