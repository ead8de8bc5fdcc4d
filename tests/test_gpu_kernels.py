"""Each HIP kernel alone against the plain implementation's function, at other sizes than the models'.

Sizes are chosen off the kernels' tiles: widths below a wavefront, no multiples of the tile,
one token, partially filled pages, head widths in steps of 16.  float32 results must agree to
rounding of float32 sums; bfloat16 results to the rounding of their stored outputs.
"""
import math

import pytest
import torch

import plain_lfm2 as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from gesso_amd.kernels import ops
    ops.lib()
    return ops


def gen(seed):
    return torch.Generator().manual_seed(seed)


def close(got, want, dtype, scale=1.0):
    """float32: 2e-6 of the largest value.  bfloat16: every element within an ulp of its own size (2^-7 of it: a
    stored value is off by half an ulp, what was rounded on the way to it by as much again) plus 2e-3 of the largest
    value (sums of rounded terms), so that a small element may not be off by what only a large one may.  (At half of
    both, 2^-8 and 1e-3, 55 of these tests fail on sound kernels: the bound stands within a factor of two of their
    rounding.)"""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    top = max(1.0, float(want.abs().max())) * scale
    if dtype == torch.float32:
        d = float((got - want).abs().max())
        assert d <= 2e-6 * top, f"max |diff| {d:.3e} above {2e-6 * top:.3e}"
        return
    over = (got - want).abs() - (want.abs() * 2.0 ** -7 * scale + 2e-3 * top)
    worst = float(over.max())
    assert worst <= 0 and not bool(torch.isnan(got).any()), \
        f"an element is {worst:.3e} beyond its bound (2^-7 of itself + {2e-3 * top:.3e}); max |diff| {float((got - want).abs().max()):.3e}"


# ------------------------------------------------------------------ elementwise

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(ops, dtype):
    table = torch.randn(37, 24, generator=gen(0)).to(dtype)
    ids = torch.tensor([36, 0, 5, 5, 36], dtype=torch.int32)
    out = ops.embed(ids.to(DEV), table.to(DEV))
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), P.embedding(table.float(), ids.tolist()))
    bad = ops.embed(torch.tensor([1, 37, -1], dtype=torch.int32, device=DEV), table.to(DEV)).cpu()
    assert torch.isfinite(bad[0]).all() and torch.isnan(bad[1]).all() and torch.isnan(bad[2]).all()


@pytest.mark.parametrize("H", [24, 80, 2048, 3000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm(ops, H, dtype):
    g = gen(H)
    T, eps = 5, 1e-4
    res = torch.randn(T, H, generator=g) * 3
    delta = torch.randn(T, H, generator=g).to(dtype)
    w = 1 + 0.1 * torch.randn(H, generator=g)
    r = res.clone().to(DEV)
    out = ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, dtype)
    summed = res.double() + delta.double()
    close(r, summed, torch.float32)                       # the stream moved on, in float32
    close(out, P.rmsnorm(summed, w.double(), eps), dtype)
    # no delta: the stream stays
    r2 = res.clone().to(DEV)
    close(ops.add_rmsnorm(r2, None, w.to(DEV), eps, dtype), P.rmsnorm(res.double(), w.double(), eps), dtype)
    assert torch.equal(r2.cpu(), res)
    # gathered rows (one of them twice): the stream is left alone
    rows = torch.tensor([4, 1, 4], dtype=torch.int32, device=DEV)
    r3 = res.clone().to(DEV)
    got = ops.add_rmsnorm(r3, delta.to(DEV), w.to(DEV), eps, dtype, rows=rows)
    close(got, P.rmsnorm(summed, w.double(), eps)[[4, 1, 4]], dtype)
    assert torch.equal(r3.cpu(), res)


def test_a_norm_whose_sum_of_squares_overflows_poisons_the_row(ops):
    """Values that are finite with a sum of squares that is not: dividing by an infinite root would quietly give a row
    of zeros; the row comes out NaN instead, so that the request fails where its next token is chosen (the reference
    raises at the norm, ``src/Operators/cpu.jl:260-266``).  Other rows are untouched."""
    res = torch.randn(3, 64, generator=gen(12))
    res[1] *= 1e30
    w = torch.ones(64)
    out = ops.add_rmsnorm(res.to(DEV), None, w.to(DEV), 1e-5, torch.float32).cpu()
    assert bool(torch.isnan(out[1]).all()) and bool(torch.isfinite(out[[0, 2]]).all())
    close(out[[0, 2]], P.rmsnorm(res[[0, 2]].double(), w.double(), 1e-5), torch.float32)


def test_rmsnorm_does_not_depend_on_the_batch(ops):
    g = gen(1)
    res = torch.randn(9, 200, generator=g)
    w = torch.randn(200, generator=g)
    whole = ops.add_rmsnorm(res.clone().to(DEV), None, w.to(DEV), 1e-5, torch.float32).cpu()
    one = ops.add_rmsnorm(res[4:5].clone().to(DEV), None, w.to(DEV), 1e-5, torch.float32).cpu()
    assert torch.equal(whole[4:5], one)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(ops, dtype):
    x = (torch.randn(7, 200, generator=gen(2)) * 3).to(dtype)
    got = ops.swiglu(x.to(DEV))
    close(got, P.swiglu(x[:, :100].double(), x[:, 100:].double()), dtype)


def test_residual_add_and_fill_rows(ops):
    res = torch.randn(3, 10, generator=gen(3))
    d = torch.randn(3, 10, generator=gen(4)).bfloat16()
    assert torch.equal(ops.residual_add(res.clone().to(DEV), d.to(DEV)).cpu(), res + d.float())
    ids = torch.tensor([3, 1, -1], dtype=torch.int32, device=DEV)     # a negative id is skipped
    state = torch.ones(5, 4, 2, device=DEV)
    ops.fill_rows(state, ids, 0.0)
    assert state.sum(dim=(1, 2)).tolist() == [8, 0, 8, 0, 8]
    half = torch.ones(5, 301, dtype=torch.bfloat16, device=DEV)       # a row that is no multiple of the block
    ops.fill_rows(half, ids, 0.25)
    assert half.float().sum(dim=1).tolist() == [301, 75.25, 301, 75.25, 301]
    # pages: rows 3 and 1 in every one of 2 x 2 planes of 5 rows, NaN, nothing else touched
    pool = torch.ones(2, 2, 5, 3, 4, 6, dtype=torch.bfloat16, device=DEV)
    ops.fill_rows(pool, ids, float("nan"), planes=3)
    bad = torch.isnan(pool.float()).flatten(3).all(dim=3)
    assert bad[:, :, [1, 3]].all() and not torch.isnan(pool[:, :, [0, 2, 4]].float()).any()


# ------------------------------------------------------------------ short convolution

@pytest.mark.parametrize("H,W,bias", [(13, 3, False), (200, 4, True), (64, 2, False), (1, 3, True), (72, 6, True),
                                      (520, 3, True)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_short_conv_segments_and_history(ops, H, W, bias, dtype):
    g = gen(10 * H + W)
    taps = torch.randn(H, W, generator=g)
    b = torch.randn(H, generator=g) if bias else None
    # three requests in slots 2, 0, 3 of a pool of 5; they advance in steps cut differently
    lens = {2: [5, 1, 1, 4], 0: [1, 1, 7, 2], 3: [11]}
    total = {s: sum(v) for s, v in lens.items()}
    data = {s: torch.randn(total[s], 3 * H, generator=g).to(dtype) for s in lens}
    want = {s: P.short_conv(data[s].double(), taps.double(), None if b is None else b.double()) for s in lens}
    state = torch.full((5, H, W - 1), 7.0, device=DEV)
    ops.fill_rows(state, torch.tensor(list(lens), dtype=torch.int32, device=DEV), 0.0)
    at = {s: 0 for s in lens}
    got = {s: [] for s in lens}
    for step in range(4):
        live = [s for s in lens if step < len(lens[s])]
        n = [lens[s][step] for s in live]
        bcx = torch.cat([data[s][at[s]:at[s] + k] for s, k in zip(live, n)]).to(DEV)
        q_start = torch.tensor([0] + list(torch.tensor(n).cumsum(0)), dtype=torch.int32, device=DEV)
        seq_of = torch.cat([torch.full((k,), i, dtype=torch.int32) for i, k in enumerate(n)]).to(DEV)
        slots = torch.tensor(live, dtype=torch.int32, device=DEV)
        out = ops.short_conv(bcx, taps.to(DEV), None if b is None else b.to(DEV), state, seq_of, q_start, slots,
                             len(live), all(k == 1 for k in n)).cpu()
        o = 0
        for s, k in zip(live, n):
            got[s].append(out[o:o + k])
            o += k
            at[s] += k
    for s in lens:
        close(torch.cat(got[s]), want[s][0], dtype)
        close(state[s], want[s][1], torch.float32)        # the history is float32 in both precisions
    assert torch.equal(state[1].cpu(), torch.full((H, W - 1), 7.0)) and torch.equal(state[4].cpu(), torch.full((H, W - 1), 7.0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("W", [2, 3, 4, 5])
@pytest.mark.parametrize("H", [8, 136, 2048])
def test_short_conv_of_single_tokens_step_after_step(ops, H, W, bias, dtype):
    """Every sequence brings one token a step (the kernel that asks for a thread's history, taps and values together, for
    widths up to 4; width 5 goes the general way): 70 sequences in slots of their own order, six steps from an empty
    history, against the convolution of the whole sequences; slots of no sequence stay as they were."""
    g = gen(100 * H + 10 * W + bias)
    nseq, steps = 70, 6
    taps = torch.randn(H, W, generator=g)
    b = torch.randn(H, generator=g) if bias else None
    data = torch.randn(nseq, steps, 3 * H, generator=g).to(dtype)
    want = [P.short_conv(data[i].double(), taps.double(), None if b is None else b.double()) for i in range(nseq)]
    slots_h = torch.randperm(nseq + 3, generator=g)[:nseq].to(torch.int32)
    state = torch.full((nseq + 3, H, W - 1), 7.0, device=DEV)
    ops.fill_rows(state, slots_h.to(DEV), 0.0)
    seq_of = torch.arange(nseq, dtype=torch.int32, device=DEV)
    q_start = torch.arange(nseq + 1, dtype=torch.int32, device=DEV)
    got = []
    for s in range(steps):
        got.append(ops.short_conv(data[:, s].contiguous().to(DEV), taps.to(DEV), None if b is None else b.to(DEV), state,
                                  seq_of, q_start, slots_h.to(DEV), nseq, True).cpu())
    got = torch.stack(got, 1)                                 # (nseq, steps, H)
    for i in range(nseq):
        close(got[i], want[i][0], dtype)
        close(state[int(slots_h[i])], want[i][1], torch.float32)
    idle = sorted(set(range(nseq + 3)) - set(slots_h.tolist()))
    assert all(torch.equal(state[j].cpu(), torch.full((H, W - 1), 7.0)) for j in idle)


@pytest.mark.parametrize("H,n", [(136, [37, 1, 2, 19, 8, 3]), (4096, [500, 1, 2, 333, 3, 190])])
@pytest.mark.parametrize("W", [2, 3, 4])
def test_short_conv_long_portions_beside_short_ones(ops, W, H, n):
    """Portions longer than a thread's run of tokens, beside ones of one and two tokens, each with its own history;
    few tokens of few channels (runs of two tokens a thread) and enough of both for runs of four."""
    g = gen(W)
    taps = torch.randn(H, W, generator=g)
    b = torch.randn(H, generator=g)
    state0 = torch.randn(len(n) + 1, H, W - 1, generator=g)
    slots = torch.tensor([4, 0, 6, 2, 1, 5], dtype=torch.int32)
    rows = [torch.randn(k, 3 * H, generator=g).bfloat16() for k in n]
    state = state0.clone().to(DEV)
    q_start = torch.tensor([0] + list(torch.tensor(n).cumsum(0)), dtype=torch.int32, device=DEV)
    seq_of = torch.cat([torch.full((k,), i, dtype=torch.int32) for i, k in enumerate(n)]).to(DEV)
    out = ops.short_conv(torch.cat(rows).to(DEV), taps.to(DEV), b.to(DEV), state, seq_of, q_start, slots.to(DEV),
                         len(n), False).cpu()
    o = 0
    for i, k in enumerate(n):
        want, hist = P.short_conv(rows[i].double(), taps.double(), b.double(), state0[slots[i]].double())
        close(out[o:o + k], want, torch.bfloat16)
        close(state[slots[i]], hist, torch.float32)
        o += k
    assert torch.equal(state[3].cpu(), state0[3])


def test_short_conv_refuses_a_width_it_cannot_take(ops):
    from gesso_amd.errors import KernelError
    H, W = 4, 17
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelError, match="width 17"):
        ops.short_conv(torch.zeros(1, 3 * H, device=DEV), torch.zeros(H, W, device=DEV), None,
                       torch.zeros(1, H, W - 1, device=DEV), z, torch.tensor([0, 1], dtype=torch.int32, device=DEV), z, 1, True)


# ------------------------------------------------------------------ head norm, rotation, cache write

def rope_tables(rd, theta, n):
    from gesso_amd.parts.rope import rope_tables as rt
    cos, sin = rt(rd, theta, n)
    return cos.to(DEV), sin.to(DEV)


@pytest.mark.parametrize("nh,nkv,d,rd,norm", [(4, 2, 16, 16, True), (3, 1, 48, 48, True), (2, 2, 128, 64, False),
                                               (5, 5, 80, 80, True), (8, 2, 256, 256, True), (32, 8, 64, 64, True),
                                               (3, 1, 32, 32, False), (2, 1, 128, 128, True)])
@pytest.mark.parametrize("layout", ["half", "interleaved"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_qknorm_rope_kv(ops, nh, nkv, d, rd, norm, dtype, layout):
    g = gen(nh * 100 + d)
    ps, theta, eps = 8, 1e4, 1e-5
    # two sequences: one continues at position 13 with 5 tokens (crossing a page edge at 16), one starts with 3
    pos = [13, 14, 15, 16, 17, 0, 1, 2]
    seq = [0] * 5 + [1] * 3
    T = len(pos)
    qkv = torch.randn(T, (nh + 2 * nkv) * d, generator=g).to(dtype)
    qw = (1 + 0.1 * torch.randn(d, generator=g)) if norm else None
    kw = (1 + 0.1 * torch.randn(d, generator=g)) if norm else None
    table = torch.tensor([[5, 2, 7], [4, 0, 0]], dtype=torch.int32)     # pages out of order
    kc = torch.zeros(9, nkv, ps, d, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    cos, sin = rope_tables(rd, theta, 64)
    x = qkv.clone().to(DEV)
    ops.qknorm_rope_kv(x, None if qw is None else qw.to(DEV), None if kw is None else kw.to(DEV), eps, cos, sin, rd,
                       torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(seq, dtype=torch.int32, device=DEV),
                       table.to(DEV), ps, kc, vc, nh, nkv, d, layout=layout)
    src = qkv.double()
    q = src[:, :nh * d].reshape(T, nh, d)
    k = src[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d)
    v = src[:, (nh + nkv) * d:].reshape(T, nkv, d)
    if norm:
        q, k = P.rmsnorm(q, qw.double(), eps), P.rmsnorm(k, kw.double(), eps)

    def rot(t):
        out = t.clone()
        if layout == "half":
            out[..., :rd] = P.rope(t[..., :rd], pos, theta)
        else:
            # pairs (2i, 2i + 1) (reference src/Operators/cpu.jl:357-371, interleaved): the half-split rotation of the
            # features put in the order evens, odds, and put back
            order = list(range(0, rd, 2)) + list(range(1, rd, 2))
            out[..., order] = P.rope(t[..., order], pos, theta)
        return out

    q, k = rot(q), rot(k)
    close(x[:, :nh * d].reshape(T, nh, d), q, dtype)
    for t in range(T):
        page = int(table[seq[t], pos[t] // ps])
        close(kc[page, :, pos[t] % ps, :], k[t], dtype)
        assert torch.equal(vc[page, :, pos[t] % ps, :].cpu(), qkv[t, (nh + nkv) * d:].reshape(nkv, d))
    # nothing else was written: 8 rows of the cache are filled
    assert int((kc.float().abs().sum(dim=(1, 3)) > 0).sum()) == T


# ------------------------------------------------------------------ attention over pages

def paged_case(ops, dtype, nh, nkv, d, ps, prefix, new, window, seed, boost=None):
    """One sequence with `prefix` cached tokens and `new` queries, another short one beside it."""
    g = gen(seed)
    K = prefix + new
    k = torch.randn(K, nkv, d, generator=g)
    v = torch.randn(K, nkv, d, generator=g)
    q = torch.randn(new, nh, d, generator=g)
    if boost is not None:                       # make one far key stand out for the last query
        far, amount = boost
        q[-1] *= amount
        k[far] = q[-1, ::nh // nkv][:nkv] / amount * 2.0
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    nblk = -(-K // ps)
    pages = torch.randperm(nblk + 3, generator=g)[:nblk] + 1
    kc = torch.randn(nblk + 5, nkv, ps, d, generator=g).to(dtype)      # garbage wherever nothing is written
    vc = torch.randn(nblk + 5, nkv, ps, d, generator=g).to(dtype)
    for u in range(K):
        kc[pages[u // ps], :, u % ps] = k[u]
        vc[pages[u // ps], :, u % ps] = v[u]
    # the second sequence: 3 tokens on page 0
    k2, v2, q2 = (torch.randn(3, n, d, generator=g).to(dtype) for n in (nkv, nkv, nh))
    kc[0, :, :3] = k2.transpose(0, 1)
    vc[0, :, :3] = v2.transpose(0, 1)
    table = torch.zeros(2, nblk, dtype=torch.int32)
    table[0] = pages.to(torch.int32)
    qall = torch.cat([q.reshape(new, -1), q2.reshape(3, -1)])
    positions = torch.tensor(list(range(prefix, K)) + [0, 1, 2], dtype=torch.int32)
    seq = torch.tensor([0] * new + [1] * 3, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    got = ops.attention_generic(qall.to(DEV), nh * d, kc.to(DEV), vc.to(DEV), positions.to(DEV), seq.to(DEV),
                                table.to(DEV), ps, window, scale, nh, nkv, d, new + 3)
    want = torch.cat([P.causal_attention(q.double(), k.double(), v.double(), window or 0).reshape(new, -1),
                      P.causal_attention(q2.double(), k2.double(), v2.double(), window or 0).reshape(3, -1)])
    return got, want


@pytest.mark.parametrize("nh,nkv,d,ps", [(4, 2, 16, 8), (3, 1, 32, 16), (5, 5, 80, 4), (8, 2, 64, 16), (2, 1, 256, 16),
                                         (6, 3, 48, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_generic_chunk_over_prefix(ops, nh, nkv, d, ps, dtype):
    got, want = paged_case(ops, dtype, nh, nkv, d, ps, prefix=37, new=9, window=None, seed=d + nh)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_generic_decode_far_key_among_hundreds(ops, dtype):
    # 700 cached keys, one query; key 3 (on the first page) carries most of the weight
    got, want = paged_case(ops, dtype, 4, 2, 64, 16, prefix=700, new=1, window=None, seed=5, boost=(3, 4.0))
    close(got, want, dtype)
    got2, want2 = paged_case(ops, dtype, 4, 2, 64, 16, prefix=700, new=1, window=None, seed=5)
    assert float((want - want2).abs().max()) > 0.1        # the far key did matter


@pytest.mark.parametrize("window", [1, 5, 16, 17, 64, 200])
def test_attention_generic_window_edge(ops, window):
    # a key just outside the window stands out: it must have no weight at all
    prefix, new = 90, 4
    far = prefix + new - 1 - window                        # first key the last query does not see
    boost = (far, 4.0) if far >= 0 else None
    got, want = paged_case(ops, torch.float32, 2, 1, 32, 16, prefix, new, window, seed=window, boost=boost)
    close(got, want, torch.float32)


def test_attention_refuses_what_it_cannot_take(ops):
    from gesso_amd.errors import KernelError
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    kc = torch.zeros(1, 1, 16, 272, device=DEV)
    with pytest.raises(KernelError, match="head width 272"):
        ops.attention_generic(torch.zeros(1, 272, device=DEV), 272, kc, kc, z, z, z.reshape(1, 1), 16, None, 1.0, 1, 1, 272, 1)
    kc = torch.zeros(1, 2, 16, 16, device=DEV)
    with pytest.raises(KernelError, match="no multiple"):
        ops.attention_generic(torch.zeros(1, 48, device=DEV), 48, kc, kc, z, z, z.reshape(1, 1), 16, None, 1.0, 3, 2, 16, 1)


# ------------------------------------------------------------------ matrix products

@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (70, 130, 100), (3, 301, 144), (64, 64, 16), (129, 65, 33)])
@pytest.mark.parametrize("xd,wd,yd", [(torch.float32,) * 3, (torch.bfloat16,) * 3, (torch.bfloat16, torch.bfloat16, torch.float32),
                                      (torch.bfloat16, torch.float32, torch.bfloat16)])
def test_gemm_tiled(ops, M, N, K, xd, wd, yd):
    g = gen(M + N + K)
    x = torch.randn(M, K, generator=g).to(xd)
    w = torch.randn(N, K, generator=g).to(wd)
    b = torch.randn(N, generator=g)
    want = x.double() @ w.double().T
    close(ops.gemm_tiled(x.to(DEV), w.to(DEV), out_dtype=yd), want, yd, scale=math.sqrt(K) / 4 if yd == torch.float32 else 1)
    close(ops.gemm_tiled(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=yd), want + b.double(), yd,
          scale=math.sqrt(K) / 4 if yd == torch.float32 else 1)


def test_gemm_rows_do_not_depend_on_the_batch(ops):
    g = gen(9)
    x = torch.randn(70, 100, generator=g).to(DEV)
    w = torch.randn(130, 100, generator=g).to(DEV)
    whole = ops.gemm_tiled(x, w)
    assert torch.equal(whole[69:70], ops.gemm_tiled(x[69:70].contiguous(), w))
    # a view with a row stride
    wide = torch.randn(6, 250, generator=g).to(DEV)
    assert torch.equal(ops.gemm_tiled(wide[:, 50:150], w), ops.gemm_tiled(wide[:, 50:150].contiguous(), w))


@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 301, 8192), (16, 96, 100), (5, 7, 64), (3, 130, 4)])
def test_float32_product_of_few_rows_streams_the_weights_and_adds_in_the_same_order(ops, M, N, K):
    g = gen(M * N + K)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(N, K, generator=g)
    b = torch.randn(N, generator=g)
    got = ops.gemm_tiled(x.to(DEV), w.to(DEV), b.to(DEV))                    # few aligned rows: the streaming kernel
    close(got, x.double() @ w.double().T + b.double(), torch.float32, scale=math.sqrt(K) / 4)
    # the same rows inside a launch of many rows go through the tiled kernel: equal to the bit
    many = torch.cat([x, torch.randn(40, K, generator=g)]).to(DEV)
    assert torch.equal(ops.gemm_tiled(many, w.to(DEV), b.to(DEV))[:M], got)
    close(ops.gemm_tiled(x.to(DEV), w.to(DEV), out_dtype=torch.bfloat16), x.double() @ w.double().T, torch.bfloat16)


# ------------------------------------------------------------------ choosing tokens

def test_argmax_rows(ops):
    x = torch.randn(6, 301, generator=gen(11))
    x[1, 17] = x[1, 200] = 50.0                     # a tie: the lowest id wins
    x[2, 300] = 60.0
    x[3, 5] = float("nan")
    x[4, 7] = float("inf")
    x[5] = -1e30
    ids, bad = ops.argmax_rows(x.to(DEV))
    ids, bad = ids.tolist(), bad.tolist()
    assert bad == [0, 0, 0, 1, 1, 0]
    assert ids[0] == int(x[0].argmax()) and ids[1] == 17 and ids[2] == 300 and ids[5] == 0
    big = torch.randn(3, 65536, generator=gen(12))
    ids, bad = ops.argmax_rows(big.to(DEV))
    assert ids.tolist() == big.argmax(1).tolist() and bad.tolist() == [0, 0, 0]


@pytest.mark.parametrize("V,temp", [(301, 0.8), (512, 1.5), (5000, 0.3)])
def test_sample_temperature_follows_the_plain_sampler(ops, V, temp):
    rows = 24
    logits = torch.randn(rows, V, generator=gen(V)) * 2
    states = list(range(100, 100 + rows))
    want, us = [], []
    for r in range(rows):
        i, _ = P.sample_id(logits[r].tolist(), temp, 1.0, states[r])
        want.append(i)
        us.append(P.splitmix64_unit(states[r])[1])
    ids, bad = ops.sample_temperature(logits.to(DEV), torch.full((rows,), temp, dtype=torch.float64, device=DEV),
                                      torch.tensor(us, dtype=torch.float64, device=DEV))
    assert ids.tolist() == want and not any(bad.tolist())


def test_sample_edges(ops):
    x = torch.tensor([[0.0, 1.0, 2.0, 1.0]])
    t = torch.tensor([1.0], dtype=torch.float64, device=DEV)
    w = torch.exp(x[0].double() - 2.0)
    cdf = (w.cumsum(0) / w.sum()).tolist()
    for u, want in ((0.0, 0), (cdf[0] - 1e-9, 0), (cdf[0] + 1e-9, 1), (cdf[2] + 1e-9, 3), (1 - 1e-12, 3)):
        ids, _ = ops.sample_temperature(x.to(DEV), t, torch.tensor([u], dtype=torch.float64, device=DEV))
        assert ids.tolist() == [want], u
    # a very low temperature is the argmax; a NaN row is flagged and emits nothing
    ids, _ = ops.sample_temperature(x.to(DEV), t * 1e-3, torch.tensor([0.999], dtype=torch.float64, device=DEV))
    assert ids.tolist() == [2]
    x[0, 1] = float("nan")
    _, bad = ops.sample_temperature(x.to(DEV), t, torch.tensor([0.5], dtype=torch.float64, device=DEV))
    assert bad.tolist() == [1]


@pytest.mark.parametrize("V,temp,top_p", [(301, 0.8, 0.9), (512, 1.0, 0.5), (5000, 1.2, 0.95), (64, 1.0, 0.1)])
def test_sample_top_p_follows_the_plain_sampler(ops, V, temp, top_p):
    rows = 24
    logits = torch.randn(rows, V, generator=gen(V + 1)) * 2
    logits[3, 10] = logits[3, 20] = logits[3, 5] = 6.0          # ties inside the nucleus keep id order
    logits[4] = 0.0                                             # all equal: the nucleus is a prefix of the ids
    want, us = [], []
    for r in range(rows):
        i, _ = P.sample_id(logits[r].tolist(), temp, top_p, 500 + r)
        want.append(i)
        us.append(P.splitmix64_unit(500 + r)[1])
    ids, bad = ops.sample_top_p(logits.to(DEV), torch.full((rows,), temp, dtype=torch.float64, device=DEV),
                                torch.full((rows,), top_p, dtype=torch.float64, device=DEV),
                                torch.tensor(us, dtype=torch.float64, device=DEV))
    assert ids.tolist() == want and not any(bad.tolist())


def test_sample_top_p_where_the_nucleus_edge_lies_among_weights_too_small_for_the_ready_histograms(ops):
    """One id carries nearly all the mass, tens of thousands of others a weight of about 2^-64 each, and top_p is so
    close to 1 that the nucleus' edge falls among those: the histograms that the many blocks make resolve weights from
    2^-63 up only, so the descent starts again and reads the row itself.  The draws land where the plain sampler's do."""
    V, rows, T = 65536, 4, 1.0
    logits = torch.full((rows, V), -64.06 * math.log(2.0))
    for r in range(rows):
        logits[r, V - 1 - 7 * r] = 0.0                   # the heavy id late in the row: the small weights add up before it
    top_p = 1.0 - 2.0 ** -50
    want, us = [], []
    for r in range(rows):
        want.append(P.sample_id(logits[r].tolist(), T, top_p, 77 + r)[0])
        us.append(P.splitmix64_unit(77 + r)[1])
    ids, bad = ops.sample_top_p(logits.to(DEV), torch.full((rows,), T, dtype=torch.float64, device=DEV),
                                torch.full((rows,), top_p, dtype=torch.float64, device=DEV),
                                torch.tensor(us, dtype=torch.float64, device=DEV))
    assert ids.tolist() == want and not any(bad.tolist())


def test_sample_top_p_gives_the_same_id_every_time_and_at_the_models_vocabulary(ops):
    """The histogram's masses are integer sums, so no order of the threads' additions can move an edge; a row of
    65,536 logits with thousands of weights that differ in their last bits, drawn many times with the same draw."""
    V, rows = 65536, 6
    logits = torch.randn(rows, V, generator=gen(91)) * 1.5
    logits[1] = (logits[1] * 4096).round() / 4096 * 1e-3          # near-ties everywhere
    logits[2, 1000:3000] = 5.0                                      # two thousand exact ties inside the nucleus
    t = torch.full((rows,), 0.9, dtype=torch.float64, device=DEV)
    p = torch.full((rows,), 0.73, dtype=torch.float64, device=DEV)
    us = [P.splitmix64_unit(40 + r)[1] for r in range(rows)]
    u = torch.tensor(us, dtype=torch.float64, device=DEV)
    x = logits.to(DEV)
    first, _ = ops.sample_top_p(x, t, p, u)
    for _ in range(30):
        again, bad = ops.sample_top_p(x, t, p, u)
        assert again.tolist() == first.tolist() and not any(bad.tolist())
    for r in (0, 2, 5):                                              # and they are the plain sampler's ids
        assert first[r].item() == P.sample_id(logits[r].tolist(), 0.9, 0.73, 40 + r)[0], r


@pytest.mark.parametrize("V", [777, 9000, 65536])
def test_the_decode_loops_choice_draws_greedy_plain_and_nucleus_rows_side_by_side(ops, V):
    """What the recorded decode step ends with when rows draw (three kernels, the weights by many blocks): rows that are
    greedy, rows that draw from the whole row and rows that draw from a nucleus, each with its own draw per step; ids
    against the plain sampler's, the rows' steps, positions and key counts advanced, a non-finite row marked.  And the
    one kernel for steps in which every row is greedy."""
    rows, steps = 6, 3
    logits = torch.randn(rows, V, generator=gen(5)) * 2
    logits[5, 13] = float("inf")
    temp = [0.0, 0.8, 0.8, 1.3, 0.0, 0.9]
    top_p = [1.0, 1.0, 0.6, 0.2, 0.5, 0.7]              # a greedy row ignores its top_p
    states = [[900 + r] for r in range(rows)]                # the plain sampler's generator, one step a draw
    u = torch.zeros(steps, rows, dtype=torch.float64)
    for r in range(rows):
        for step in range(steps):
            nxt_state, u[step, r] = P.splitmix64_unit(states[r][-1])
            states[r].append(nxt_state)
    dev = lambda t: t.to(DEV)
    i32 = lambda *a: torch.tensor(*a, dtype=torch.int32, device=DEV)
    counter, nxt = i32([0] * rows), i32([0] * rows)
    ring, bad = torch.full((steps, rows), -1, dtype=torch.int32, device=DEV), torch.full((steps, rows), -1, dtype=torch.int32, device=DEV)
    pos, kv, live = i32([10, 11, 12, 13, 14, 15]), i32([11, 12, 13, 14, 15, 16]), i32([1, 1, 1, 0, 1, 1])
    wbuf = torch.full((rows * V,), float("nan"), dtype=torch.float64, device=DEV)
    scratch = (torch.full((rows * ops.choice_parts(V),), float("nan"), dtype=torch.float64, device=DEV), i32([7] * rows),
               i32([7] * rows), torch.full((rows * ops.choice_hist(),), 12345, dtype=torch.int64, device=DEV))
    for step in range(steps):
        ops.decode_choose(dev(logits), dev(torch.tensor(temp, dtype=torch.float64)), dev(u), counter, nxt, ring, bad, pos, kv,
                          live, scratch, top_p=dev(torch.tensor(top_p, dtype=torch.float64)), wbuf=wbuf)
    assert counter.tolist() == [steps] * rows
    assert pos.tolist() == [13, 14, 15, 13, 17, 18] and kv.tolist() == [14, 15, 16, 14, 18, 19]     # row 3 is not live
    assert bad[:, :5].sum().item() == 0 and bad[:, 5].tolist() == [1] * steps
    got = ring.cpu()
    for step in range(steps):
        for r in range(5):
            if temp[r] <= 0:
                want = int(logits[r].argmax())
            else:
                want = P.sample_id(logits[r].tolist(), temp[r], top_p[r], states[r][step])[0]
            assert int(got[step, r]) == want, (step, r)
    assert nxt.tolist()[:5] == got[steps - 1].tolist()[:5]
    # all greedy, in one kernel
    counter, pos, kv = i32([0, 1, 2, 0, 1, 2]), i32([10] * rows), i32([11] * rows)
    ring.fill_(-1); bad.fill_(-1)
    ops.decode_choose_greedy(dev(logits), counter, nxt, ring, bad, pos, kv, live)
    assert counter.tolist() == [1, 2, 3, 1, 2, 3] and pos.tolist() == [11, 11, 11, 10, 11, 11]
    for r in range(rows):
        step = [0, 1, 2, 0, 1, 2][r]
        assert int(bad[step, r]) == (1 if r == 5 else 0)
        if r < 5:
            assert int(ring[step, r]) == int(logits[r].argmax()) == int(nxt[r])


# ------------------------------------------------------------------ the weight-streaming product

@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(48, 64), (100, 200), (2048, 2048), (6144, 2048), (2048, 8192), (301, 144)])
def test_gemm_skinny(ops, M, N, K):
    g = gen(M * 7 + N + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    want = x.double() @ w.double().T
    got32 = ops.gemm_skinny(x.to(DEV), w.to(DEV), out_dtype=torch.float32)
    assert float((got32.double().cpu() - want).abs().max()) <= 2e-5 * max(1.0, float(want.abs().max())) * math.sqrt(K)
    close(ops.gemm_skinny(x.to(DEV), w.to(DEV)), want, torch.bfloat16)
    # a view with a row stride, as the attention output and portions of a buffer are
    wide = torch.randn(M, K + 16, generator=g).bfloat16().to(DEV)
    close(ops.gemm_skinny(wide[:, 8:8 + K], w.to(DEV)), wide[:, 8:8 + K].double().cpu() @ w.double().T, torch.bfloat16) \
        if ops.skinny_ok(wide[:, 8:8 + K], w.to(DEV)) else None


@pytest.mark.parametrize("M,F,K", [(1, 24, 64), (8, 100, 96), (40, 8192, 2048), (64, 50, 144)])
def test_gemm_skinny_swiglu(ops, M, F, K):
    g = gen(M + F + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(2 * F, K, generator=g) / math.sqrt(K) * 2).bfloat16()
    y = x.double() @ w.double().T
    want = P.swiglu(y[:, :F], y[:, F:])
    got = ops.gemm_skinny(x.to(DEV), w.to(DEV), swiglu=True)
    assert got.shape == (M, F)
    close(got, want, torch.bfloat16)


def test_gemm_skinny_refuses(ops):
    from gesso_amd.errors import KernelError
    x = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(16, 64, dtype=torch.bfloat16, device=DEV)
    assert not ops.skinny_ok(x, w) and not ops.skinny_ok(x[:4, :60], w[:, :60])
    with pytest.raises(KernelError):
        ops.gemm_skinny(x, w)


# ------------------------------------------------------------------ decode attention (one query per sequence)

@pytest.mark.parametrize("nh,nkv,d,ps", [(4, 2, 16, 8), (3, 1, 32, 16), (32, 8, 64, 16), (8, 1, 128, 16), (5, 5, 64, 4)])
@pytest.mark.parametrize("nsplit", [1, 3, 16])
@pytest.mark.parametrize("window", [None, 70])
def test_attention_decode(ops, nh, nkv, d, ps, nsplit, window):
    g = gen(nh + d + nsplit)
    lens = [1, 2, 63, 64, 65, 300, 700, 129, 1500]      # keys per sequence, the query's own included; the last
                                                          # takes a block of eight wavefronts three passes
    nseq = len(lens)
    nblk = [-(-n // ps) for n in lens]
    total = sum(nblk)
    perm = torch.randperm(total + 2, generator=g)[:total] + 1
    kc = torch.randn(total + 3, nkv, ps, d, generator=g).bfloat16()
    vc = torch.randn(total + 3, nkv, ps, d, generator=g).bfloat16()
    table = torch.zeros(nseq, max(nblk), dtype=torch.int32)
    q = torch.randn(nseq, nh * d, generator=g)
    q[5] *= 3.0                                           # sharper weights on one sequence
    q = q.bfloat16()
    want, at = [], 0
    for i, n in enumerate(lens):
        pages = perm[at:at + nblk[i]]
        at += nblk[i]
        table[i, :nblk[i]] = pages.to(torch.int32)
        k = kc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:n]
        v = vc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:n]
        want.append(P.causal_attention(q[i].double().reshape(1, nh, d), k.double(), v.double(), window or 0).reshape(-1))
    want = torch.stack(want)
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    for _ in range(2):                                    # twice: the counters must be back at zero
        got = ops.attention_decode(q.to(DEV), nh * d, kc.to(DEV), vc.to(DEV), positions.to(DEV), table.to(DEV), ps,
                                   window, scale, nh, nkv, d, nseq, nsplit)
        close(got, want, torch.bfloat16)
    same = ops.attention_generic(q.to(DEV), nh * d, kc.to(DEV), vc.to(DEV), positions.to(DEV),
                                 torch.arange(nseq, dtype=torch.int32, device=DEV), table.to(DEV), ps, window, scale,
                                 nh, nkv, d, nseq)
    close(got, same.double().cpu(), torch.bfloat16)


@pytest.mark.parametrize("nsplit", [1, 3])
@pytest.mark.parametrize("window", [None, 70])
def test_attention_decode_sees_the_far_key_and_not_the_keys_outside(ops, nsplit, window):
    """A key far back that carries most of the weight must count in full; a key one place past the sequence's end (on
    the last page) and, with a window, the key one place before the window's start are made to stand out ten times
    more and must count for nothing: a mask off by one moves the result by far more than the tolerance."""
    g = gen(31 + nsplit)
    nh, nkv, d, ps = 8, 2, 64, 16
    lens = [17, 63, 64, 65, 300, 700, 129, 1030]
    nseq = len(lens)
    nblk = [-(-(n + 1) // ps) for n in lens]                 # room for the key past the end
    total = sum(nblk)
    perm = torch.randperm(total + 2, generator=g)[:total] + 1
    kc = torch.randn(total + 3, nkv, ps, d, generator=g)
    vc = torch.randn(total + 3, nkv, ps, d, generator=g)
    table = torch.zeros(nseq, max(nblk), dtype=torch.int32)
    q = torch.randn(nseq, nh, d, generator=g)
    want, moved, at = [], [], 0
    G = nh // nkv
    for i, n in enumerate(lens):
        pages = perm[at:at + nblk[i]]
        at += nblk[i]
        table[i, :nblk[i]] = pages.to(torch.int32)

        def put(u, row):                                     # key u of this sequence, for every key head
            kc[pages[u // ps], :, u % ps] = row

        lo = max(0, n - window) if window else 0
        far = lo + min(3, n - 1 - lo)                        # a visible key near the far end of what is seen
        qdir = q[i, ::G]                                     # one query per key head: (nkv, d)
        put(far, qdir * 2.0)
        put(n, qdir * 20.0)                                  # one past the end: must not be seen
        if window and lo > 0:
            put(lo - 1, qdir * 20.0)                         # one before the window: must not be seen
        k = kc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:n].bfloat16().double()
        v = vc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:n].bfloat16().double()
        qi = q[i].bfloat16().double().reshape(1, nh, d)
        want.append(P.causal_attention(qi, k, v, window or 0).reshape(-1))
        k2 = k.clone()
        k2[far] = 0.0                                        # without the far key the result is another one
        moved.append(float((P.causal_attention(qi, k2, v, window or 0).reshape(-1) - want[-1]).abs().max()))
    want = torch.stack(want)
    assert min(moved) > 0.1
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    got = ops.attention_decode(q.reshape(nseq, -1).bfloat16().to(DEV), nh * d, kc.bfloat16().to(DEV), vc.bfloat16().to(DEV),
                               positions.to(DEV), table.to(DEV), ps, window, 1.0 / math.sqrt(d), nh, nkv, d, nseq, nsplit)
    close(got, want, torch.bfloat16)


@pytest.mark.parametrize("nh,nkv,d,norm,nsplit,write,copies", [(32, 8, 64, True, 1, True, 1), (2, 1, 64, False, 3, True, 1),
                                                               (8, 1, 128, True, 2, True, 1), (5, 5, 64, True, 1, False, 1),
                                                               (32, 8, 64, True, 1, True, 12), (4, 2, 64, True, 2, True, 24)])
def test_attention_decode_from_raw_rows_equals_the_separate_kernels(ops, nh, nkv, d, norm, nsplit, write, copies):
    """Head norms, rotation and cache write inside the attention kernel against the kernel that does them alone.
    With many sequences (`copies` of the six lengths) the grid holds two blocks and more a compute unit, and the
    kernel runs in blocks of four wavefronts."""
    g = gen(nh * 7 + d + nsplit)
    ps, lens = 16, [1, 64, 65, 300, 17, 129] * copies
    nseq = len(lens)
    nblk = [-(-n // ps) for n in lens]
    total = sum(nblk)
    kc = torch.randn(total + 1, nkv, ps, d, generator=g).bfloat16()
    vc = torch.randn(total + 1, nkv, ps, d, generator=g).bfloat16()
    table = torch.zeros(nseq, max(nblk), dtype=torch.int32)
    at = 0
    for i in range(nseq):
        table[i, :nblk[i]] = torch.arange(at, at + nblk[i], dtype=torch.int32)
        at += nblk[i]
    qkv = torch.randn(nseq, (nh + 2 * nkv) * d, generator=g).bfloat16()
    qw = (1 + 0.2 * torch.randn(d, generator=g)).to(DEV) if norm else None
    kw = (1 + 0.2 * torch.randn(d, generator=g)).to(DEV) if norm else None
    cos, sin = rope_tables(d, 1e4, 512)
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32).to(DEV)
    seq_of = torch.arange(nseq, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(d)
    stride = (nh + 2 * nkv) * d
    # the separate kernels
    k1, v1, q1 = kc.clone().to(DEV), vc.clone().to(DEV), qkv.clone().to(DEV)
    ops.qknorm_rope_kv(q1, qw, kw, 1e-5, cos, sin, d, positions, seq_of, table.to(DEV), ps, k1, v1, nh, nkv, d, write_kv=write)
    want = ops.attention_decode(q1, stride, k1, v1, positions, table.to(DEV), ps, None, scale, nh, nkv, d, nseq, nsplit)
    # all in one; what the rows of the new keys and values held before (a page that was another request's, anything)
    # must not reach the result: the kernel loads those rows before it writes them, for the places past the end too
    k2, v2 = kc.clone().to(DEV), vc.clone().to(DEV)
    if write:
        for i, n in enumerate(lens):
            page, row = int(table[i, (n - 1) // ps]), (n - 1) % ps
            k2[page, :, row] = float("nan")
            v2[page, :, row] = float("nan")
    got = ops.attention_decode_raw(qkv.to(DEV), stride, k2, v2, positions, table.to(DEV), ps, None, scale, qw, kw, 1e-5,
                                   cos, sin, nh, nkv, d, nseq, nsplit, write_kv=write)
    assert float((got.float() - want.float()).abs().max()) <= 2e-2 * max(1.0, float(want.float().abs().max()))
    assert float((k2.float() - k1.float()).abs().max()) <= 2e-2 * max(1.0, float(k1.float().abs().max()))
    assert torch.equal(v2, v1)
    if not write:
        assert torch.equal(k2.cpu(), kc) and torch.equal(v2.cpu(), vc)


def test_attention_decode_supports(ops):
    assert ops.attention_decode_supports(32, 8, 64) and ops.attention_decode_supports(3, 1, 32)
    assert not ops.attention_decode_supports(3, 3, 48) and not ops.attention_decode_supports(18, 2, 64)


# ------------------------------------------------------------------ the decode step's fused products

def lazy_case(ops, M, K, seed, weighted=False):
    g = gen(seed)
    res = torch.randn(M, K, generator=g)
    nw = 1 + 0.1 * torch.randn(K, generator=g)
    nb = 5
    part = torch.rand(M, nb, generator=g)
    part = part / part.sum(1, keepdim=True) * (res * res).sum(1, keepdim=True)      # partial sums of the true sums
    xs = (res * nw).bfloat16().to(DEV) if weighted else None     # as a producer would have left them
    lazy = ops.LazyNorm(res.to(DEV), part.to(DEV), nw.to(DEV), 1e-5, torch.bfloat16, xs=xs)
    return res, nw, lazy


@pytest.mark.parametrize("M", [1, 8, 33, 64])
@pytest.mark.parametrize("N,K", [(2048, 2048), (100, 96), (6144, 2048)])
def test_gemm_skinny_with_lazy_norm(ops, M, N, K):
    res, nw, lazy = lazy_case(ops, M, K, M + N)
    w = (torch.randn(N, K, generator=gen(N)) / math.sqrt(K)).bfloat16()
    normed = ops.add_rmsnorm(res.clone().to(DEV), None, nw.to(DEV), 1e-5, torch.bfloat16)
    want = ops.gemm_skinny(normed, w.to(DEV), out_dtype=torch.float32).double().cpu()
    got = ops.gemm_skinny(lazy, w.to(DEV), out_dtype=torch.float32).double().cpu()
    # the same rounded inputs but for the last bit of the inverse root: float32 sums apart by rounding only
    assert float((got - want).abs().max()) <= 2e-3 * max(1.0, float(want.abs().max()))
    ref = P.rmsnorm(res.double(), nw.double(), 1e-5) @ w.double().T
    close(ops.gemm_skinny(lazy, w.to(DEV)), ref, torch.bfloat16)
    if N % 2 == 0:
        close(ops.gemm_skinny(lazy, w.to(DEV), swiglu=True), P.swiglu(ref[:, :N // 2], ref[:, N // 2:]), torch.bfloat16, scale=2)


@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 2048, 8192), (40, 96, 320), (64, 144, 104)])
def test_gemm_skinny_residual(ops, M, N, K):
    g = gen(M + N + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    res = torch.randn(M, N, generator=g)
    r = res.clone().to(DEV)
    ssq = ops.gemm_skinny_residual(x.to(DEV), w.to(DEV), r)
    want = res.double() + (x.double() @ w.double().T)
    close(r, want, torch.bfloat16)                       # the product is rounded to bfloat16 before the add
    assert ssq.shape[0] == M
    total = ssq.double().sum(1).cpu()
    assert torch.allclose(total, (r.double().cpu() ** 2).sum(1), rtol=1e-5)
    # and the partial sums feed a lazy norm that equals the norm kernel on the new stream
    nw = torch.ones(N)
    lazy = ops.LazyNorm(r, ssq, nw.to(DEV), 1e-5, torch.bfloat16)
    if N % 8 == 0:
        eye = torch.eye(N).bfloat16().to(DEV)
        a = ops.gemm_skinny(lazy, eye, out_dtype=torch.float32)
        b = ops.add_rmsnorm(r.clone(), None, nw.to(DEV), 1e-5, torch.bfloat16).float()
        assert float((a - b).abs().max()) <= 1e-2 * float(b.abs().max())


@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 2048, 8192), (40, 96, 320), (64, 144, 104)])
def test_gemm_skinny_residual_leaves_rows_weighted_for_the_next_norm(ops, M, N, K):
    g = gen(M + N + K + 1)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    res = torch.randn(M, N, generator=g)
    nw = 1 + 0.3 * torch.randn(N, generator=g)
    r1, r2 = res.clone().to(DEV), res.clone().to(DEV)
    xs = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ssq1 = ops.gemm_skinny_residual(x.to(DEV), w.to(DEV), r1, next_weight=nw.to(DEV), xs=xs)
    ssq2 = ops.gemm_skinny_residual(x.to(DEV), w.to(DEV), r2)
    assert torch.equal(r1, r2) and torch.equal(ssq1, ssq2)
    assert torch.equal(xs.cpu(), (r1.cpu() * nw).bfloat16())
    # a product that reads the weighted rows and scales its result equals the product of the normed rows
    N2 = 112
    w2 = (torch.randn(N2, N, generator=g) / math.sqrt(N)).bfloat16()
    lazy = ops.LazyNorm(r1, ssq1, nw.to(DEV), 1e-5, torch.bfloat16, xs=xs)
    if N % 8 == 0:
        ref = P.rmsnorm(r1.double().cpu(), nw.double(), 1e-5) @ w2.double().T
        close(ops.gemm_skinny(lazy, w2.to(DEV), out_dtype=torch.float32), ref, torch.bfloat16)
        close(ops.gemm_skinny(lazy, w2.to(DEV), swiglu=True), P.swiglu(ref[:, :N2 // 2], ref[:, N2 // 2:]), torch.bfloat16, scale=2)


@pytest.mark.parametrize("M,N,K,parts", [(64, 2048, 8192, 8), (40, 96, 320, 3), (33, 144, 104, 1), (17, 2048, 2048, 16),
                                          (5, 100, 64, 4), (33, 144, 128, 2)])   # the last: an odd number of weight tiles, tile-major
def test_gemm_skinny_residual_in_parts(ops, M, N, K, parts):
    g = gen(M + N + K + parts)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    res = torch.randn(M, N, generator=g)
    nw = 1 + 0.3 * torch.randn(N, generator=g)
    r = res.clone().to(DEV)
    wt = ops.tile_major(w.to(DEV)) if N % 16 == 0 and K % 32 == 0 else None
    ssq, normed = ops.gemm_skinny_residual_parts(x.to(DEV), w.to(DEV), r, parts, wt=wt, next_weight=nw.to(DEV), eps=1e-5)
    want = res.double() + (x.double() @ w.double().T)
    close(r, want, torch.bfloat16)                       # the product is rounded to bfloat16 before the add
    assert torch.allclose(ssq.double().cpu()[:, 0], (r.double().cpu() ** 2).sum(1), rtol=1e-5)
    close(normed, P.rmsnorm(r.double().cpu(), nw.double(), 1e-5), torch.bfloat16)
    # and without a norm to prepare for
    r2 = res.clone().to(DEV)
    ssq2, none = ops.gemm_skinny_residual_parts(x.to(DEV), w.to(DEV), r2, parts, wt=wt)
    assert none is None and torch.equal(r2, r) and torch.equal(ssq2, ssq)


@pytest.mark.parametrize("T,H,V", [(1, 2048, 1000), (9, 104, 301)])
def test_embed_leaves_rows_weighted_for_the_first_norm(ops, T, H, V):
    g = gen(T + H)
    table = torch.randn(V, H, generator=g).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    nw = 1 + 0.3 * torch.randn(H, generator=g)
    ssq = torch.empty(T, 1, device=DEV)
    xs = torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    out = ops.embed(ids.to(DEV), table.to(DEV), ssq=ssq, next_weight=nw.to(DEV), xs=xs)
    rows = table[ids.long()].float()
    assert torch.equal(out.cpu(), rows)
    assert torch.equal(xs.cpu(), (rows * nw).bfloat16())
    assert torch.allclose(ssq.cpu()[:, 0].double(), (rows.double() ** 2).sum(1), rtol=1e-5)


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("M,H,W,bias", [(1, 64, 3, False), (8, 2048, 3, False), (20, 96, 4, True), (64, 48, 2, False),
                                        (64, 2048, 3, False), (40, 1024, 3, False)])
def test_gemm_skinny_conv_equals_the_separate_kernels(ops, M, H, W, bias, weighted):
    res, nw, lazy = lazy_case(ops, M, H, M + H, weighted)
    g = gen(H + W)
    w_in = (torch.randn(3 * H, H, generator=g) / math.sqrt(H)).bfloat16().to(DEV)
    taps = torch.randn(H, W, generator=g).to(DEV)
    b = torch.randn(H, generator=g).to(DEV) if bias else None
    state0 = torch.randn(M + 2, H, W - 1, generator=g)
    slots = torch.randperm(M + 2, generator=g)[:M].to(torch.int32).to(DEV)
    s1, s2 = state0.clone().to(DEV), state0.clone().to(DEV)
    got = ops.gemm_skinny_conv(lazy, w_in, taps, b, s1, slots)
    bcx = ops.gemm_skinny(lazy, w_in)
    ar = torch.arange(M, dtype=torch.int32, device=DEV)
    want = ops.short_conv(bcx, taps, b, s2, ar, torch.arange(M + 1, dtype=torch.int32, device=DEV), slots, M, True)
    assert float((got.float() - want.float()).abs().max()) <= 1e-2 * max(1.0, float(want.float().abs().max()))
    assert float((s1 - s2).abs().max()) <= 1e-2 * max(1.0, float(s2.abs().max()))
    untouched = [i for i in range(M + 2) if i not in slots.tolist()]
    assert torch.equal(s1[untouched].cpu(), state0[untouched])


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("H", [64, 96, 256, 1280])
def test_gemm_skinny_conv_over_row_tiles_widths_and_shares_of_k(ops, H, W, bias, weighted):
    """The fused input product + convolution at one to four row tiles (3, 20, 40 and 64 rows), every width the
    epilogue holds in registers, with and without a bias, rows normed on the fly and pre-weighted, and hidden sizes that
    give a wavefront less than a batch of steps, exactly one, and several with a remainder: the same as the product
    followed by the convolution kernel, channel by channel (a value of one lane's four channels that went missing
    would show in every fourth column)."""
    for M in (3, 20, 40, 64):
        res, nw, lazy = lazy_case(ops, M, H, M + H + W, weighted)
        g = gen(H + W + M)
        w_in = (torch.randn(3 * H, H, generator=g) / math.sqrt(H)).bfloat16().to(DEV)
        taps = torch.randn(H, W, generator=g).to(DEV)
        b = torch.randn(H, generator=g).to(DEV) if bias else None
        state0 = torch.randn(M + 2, H, W - 1, generator=g)
        slots = torch.randperm(M + 2, generator=g)[:M].to(torch.int32).to(DEV)
        s1, s2 = state0.clone().to(DEV), state0.clone().to(DEV)
        for wt in ([None] if H % 16 else [None, ops.tile_major(w_in)]):
            s1.copy_(state0)
            s2.copy_(state0)
            got = ops.gemm_skinny_conv(lazy, w_in, taps, b, s1, slots, wt=wt)
            bcx = ops.gemm_skinny(lazy, w_in, wt=wt)
            ar = torch.arange(M, dtype=torch.int32, device=DEV)
            want = ops.short_conv(bcx, taps, b, s2, ar, torch.arange(M + 1, dtype=torch.int32, device=DEV), slots, M, True)
            d = (got.float() - want.float()).abs()
            tol = 1e-2 * max(1.0, float(want.float().abs().max()))
            assert float(d.max()) <= tol, f"M={M} tile-major={wt is not None}: columns {sorted(set((torch.nonzero(d > tol)[:, 1] % 4).tolist()))} (mod 4) differ"
            assert float((s1 - s2).abs().max()) <= 1e-2 * max(1.0, float(s2.abs().max())), f"M={M}: history"


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("M,H,W", [(1, 2048, 3), (8, 2048, 3), (64, 2048, 3), (48, 1024, 3), (33, 96, 4)])
def test_gemm_skinny_conv_against_the_plain_convolution(ops, M, H, W, weighted):
    """The input product with the short convolution as its epilogue, at the widths and row counts of the benchmarked
    decode steps (1, 8 and 64 rows of 2048; 48 of 1024), against the plain formulas: norm, product, ``B * x``, taps
    over the slot's history and the new row, ``C * y``, and the history shifted by one."""
    res, nw, lazy = lazy_case(ops, M, H, 3 * M + H, weighted)
    g = gen(H + W + M)
    w_in = (torch.randn(3 * H, H, generator=g) / math.sqrt(H)).bfloat16()
    taps = torch.randn(H, W, generator=g)
    state0 = torch.randn(M + 3, H, W - 1, generator=g)
    slots = torch.randperm(M + 3, generator=g)[:M].to(torch.int32)
    state = state0.clone().to(DEV)
    got = ops.gemm_skinny_conv(lazy, w_in.to(DEV), taps.to(DEV), None, state, slots.to(DEV))
    # plain: the product's inputs rounded to bfloat16 where the kernel holds them so, the rest in float64: the normed
    # rows, or (pre-weighted rows) the rows times the norm's weight, whose product is then scaled by the row's inverse
    # root mean square
    if weighted:
        inv = 1.0 / torch.sqrt((res.double() ** 2).mean(1, keepdim=True) + 1e-5)
        bcx = (P.to_bfloat16(res.double() * nw.double()) @ w_in.double().T) * inv
    else:
        bcx = P.to_bfloat16(P.rmsnorm(res.double(), nw.double(), 1e-5)) @ w_in.double().T
    want = torch.zeros(M, H, dtype=torch.float64)
    hist = state0.double().clone()
    for i in range(M):
        out, h = P.short_conv(bcx[i:i + 1], taps.double(), None, state0[slots[i]].double())
        want[i], hist[slots[i]] = out[0], h
    close(got, want, torch.bfloat16)
    assert float((state.double().cpu() - hist).abs().max()) <= 1e-2 * max(1.0, float(hist.abs().max()))
    untouched = [i for i in range(M + 3) if i not in slots.tolist()]
    assert torch.equal(state[untouched].cpu(), state0[untouched])


@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 16384, 2048), (24, 96, 64), (64, 2048, 8192)])
def test_tile_major_copy_gives_the_same_products(ops, M, N, K):
    g = gen(M + N + K)
    x = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    wt = ops.tile_major(w)
    # the copy holds the same values: tile (t, s), lane l, element j
    t, s, l, j = N // 16 - 1, K // 32 - 1, 37, 5
    assert wt.reshape(-1)[((t * (K // 32) + s) * 64 + l) * 8 + j] == w[16 * t + l % 16, 32 * s + 8 * (l // 16) + j]
    for kw in ({}, {"swiglu": True}, {"out_dtype": torch.float32}):
        assert torch.equal(ops.gemm_skinny(x, w, wt=wt, **kw), ops.gemm_skinny(x, w, **kw))
    if N <= 2048:
        r1, r2 = torch.ones(M, N, device=DEV), torch.ones(M, N, device=DEV)
        s1, s2 = ops.gemm_skinny_residual(x, w, r1, wt=wt), ops.gemm_skinny_residual(x, w, r2)
        # a weight of few rows is shared out in half tiles: twice the partial sums, and K split over other
        # numbers of wavefronts, so the float32 sums differ by rounding (and a bfloat16 rounding may flip)
        assert s1.shape == (M, N // 8) and s2.shape == (M, N // 16)
        assert float((r1 - r2).abs().max()) <= 2.0 ** -7 * float((r2 - 1).abs().max())
        assert torch.allclose(s1.sum(1), s2.sum(1), rtol=1e-3)
        assert torch.allclose(s1.double().sum(1), (r1.double() ** 2).sum(1), rtol=1e-5)


# ------------------------------------------------------------------ prompt attention on the matrix cores

@pytest.mark.parametrize("nh,nkv,d,ps", [(4, 2, 32, 8), (32, 8, 64, 16), (3, 1, 64, 16), (8, 1, 128, 16), (5, 5, 64, 4)])
@pytest.mark.parametrize("window", [None, 37])
@pytest.mark.parametrize("rows", [16, 32])
def test_attention_prefill(ops, nh, nkv, d, ps, window, rows):
    """Three sequences in one launch: a chunk over a cached prefix, a fresh prompt, a single token."""
    g = gen(nh + d + ps)
    prefix = [70, 0, 45]
    new = [41, 33, 1]
    nseq = 3
    K = [a + b for a, b in zip(prefix, new)]
    nblk = [-(-k // ps) for k in K]
    total = sum(nblk)
    perm = torch.randperm(total + 2, generator=g)[:total] + 1
    kc = torch.randn(total + 3, nkv, ps, d, generator=g).bfloat16()
    vc = torch.randn(total + 3, nkv, ps, d, generator=g).bfloat16()
    table = torch.zeros(nseq, max(nblk), dtype=torch.int32)
    qs, want, at = [], [], 0
    for i in range(nseq):
        pages = perm[at:at + nblk[i]]
        at += nblk[i]
        table[i, :nblk[i]] = pages.to(torch.int32)
        k = kc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:K[i]]
        v = vc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:K[i]]
        q = torch.randn(new[i], nh, d, generator=g)
        if i == 0:
            q[-1] *= 3.0
        q = q.bfloat16()
        qs.append(q.reshape(new[i], -1))
        want.append(P.causal_attention(q.double(), k.double(), v.double(), window or 0).reshape(new[i], -1))
    qall, want = torch.cat(qs), torch.cat(want)
    positions = torch.tensor([p + j for p, n in zip(prefix, new) for j in range(n)], dtype=torch.int32)
    seq_of = torch.tensor([i for i, n in enumerate(new) for _ in range(n)], dtype=torch.int32)
    tiles, row = [[], [], []], 0
    for i, n in enumerate(new):
        for a in range(0, n, rows):
            tiles[0].append(i); tiles[1].append(row + a); tiles[2].append(min(rows, n - a))
        row += n
    tiles = torch.tensor(tiles, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    # q as a strided view, as the attention mixer hands it over (q, k, v side by side)
    wide = torch.zeros(sum(new), (nh + 2 * nkv) * d, dtype=torch.bfloat16)
    wide[:, :nh * d] = qall
    got = ops.attention_prefill(wide.to(DEV), (nh + 2 * nkv) * d, kc.to(DEV), vc.to(DEV), positions.to(DEV),
                                tiles.to(DEV), table.to(DEV), ps, window, scale, nh, nkv, d, sum(new), tile_rows=rows)
    close(got, want, torch.bfloat16)
    same = ops.attention_generic(wide.to(DEV), (nh + 2 * nkv) * d, kc.to(DEV), vc.to(DEV), positions.to(DEV),
                                 seq_of.to(DEV), table.to(DEV), ps, window, scale, nh, nkv, d, sum(new))
    close(got, same.double().cpu(), torch.bfloat16)


@pytest.mark.parametrize("rows,window", [(32, None), (16, 3000)])
def test_attention_prefill_over_more_pages_than_the_kernel_keeps_at_hand(ops, rows, window):
    """4,700 keys in pages of two: the kernel keeps 2,048 page numbers in LDS and walks the rest window by window.
    One key far back, in the first window, carries weight for the last query."""
    g = gen(5)
    nh, nkv, d, ps, prefix, new = 2, 1, 64, 2, 4650, 50
    K = prefix + new
    k, v, q = torch.randn(K, nkv, d, generator=g), torch.randn(K, nkv, d, generator=g), torch.randn(new, nh, d, generator=g)
    far = 1999 if window is None else K - 2990
    k[far, 0] = q[-1, 0] * 1.5
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    nblk = -(-K // ps)
    perm = torch.randperm(nblk, generator=g)
    kc = torch.zeros(nblk, nkv, ps, d, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kc[perm] = k.reshape(nblk, ps, nkv, d).permute(0, 2, 1, 3)
    vc[perm] = v.reshape(nblk, ps, nkv, d).permute(0, 2, 1, 3)
    table = perm.to(torch.int32)[None].contiguous()
    tiles = torch.tensor([[0] * -(-new // rows), list(range(0, new, rows)),
                          [min(rows, new - a) for a in range(0, new, rows)]], dtype=torch.int32)
    got = ops.attention_prefill(q.reshape(new, -1).to(DEV), nh * d, kc.to(DEV), vc.to(DEV),
                                torch.arange(prefix, K, dtype=torch.int32, device=DEV), tiles.to(DEV), table.to(DEV), ps,
                                window, 1.0 / math.sqrt(d), nh, nkv, d, new, tile_rows=rows)
    want = P.causal_attention(q.double(), k.double(), v.double(), window or 0).reshape(new, -1)
    close(got, want, torch.bfloat16)


def test_attention_prefill_far_key_and_supports(ops):
    assert ops.attention_prefill_supports(32, 8, 64) and not ops.attention_prefill_supports(3, 3, 48)
    assert not ops.attention_prefill_supports(18, 2, 64)
    # 600 cached keys; key 5 carries most of the weight for the last query of a 20-token chunk
    g = gen(77)
    nh, nkv, d, ps, prefix, new = 4, 2, 64, 16, 600, 20
    K = prefix + new
    k, v, q = torch.randn(K, nkv, d, generator=g), torch.randn(K, nkv, d, generator=g), torch.randn(new, nh, d, generator=g)
    q[-1] *= 4.0
    k[5] = q[-1, ::2][:nkv] / 4.0 * 2.0
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    nblk = -(-K // ps)
    kc = torch.zeros(nblk, nkv, ps, d, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    for u in range(K):
        kc[u // ps, :, u % ps], vc[u // ps, :, u % ps] = k[u], v[u]
    table = torch.arange(nblk, dtype=torch.int32)[None]
    tiles = torch.tensor([[0, 0], [0, 16], [16, 4]], dtype=torch.int32)
    got = ops.attention_prefill(q.reshape(new, -1).to(DEV), nh * d, kc.to(DEV), vc.to(DEV),
                                torch.arange(prefix, K, dtype=torch.int32, device=DEV), tiles.to(DEV), table.to(DEV), ps,
                                None, 1.0 / math.sqrt(d), nh, nkv, d, new)
    close(got, P.causal_attention(q.double(), k.double(), v.double()).reshape(new, -1), torch.bfloat16)


def paged(k, v, ps, g):
    """Keys and values (K, nkv, d) laid into pages of ps in a random order; returns caches and the block table row."""
    K, nkv, d = k.shape
    nblk = -(-K // ps)
    pad = nblk * ps - K
    kp = torch.cat([k, torch.full((pad, nkv, d), float("nan"), dtype=k.dtype)])      # rows past the end: never read
    vp = torch.cat([v, torch.full((pad, nkv, d), float("nan"), dtype=v.dtype)])
    perm = torch.randperm(nblk + 2, generator=g)[:nblk]
    kc = torch.full((nblk + 2, nkv, ps, d), float("nan"), dtype=k.dtype)
    vc = torch.full_like(kc, float("nan"))
    kc[perm] = kp.reshape(nblk, ps, nkv, d).permute(0, 2, 1, 3)
    vc[perm] = vp.reshape(nblk, ps, nkv, d).permute(0, 2, 1, 3)
    return kc, vc, perm.to(torch.int32)


@pytest.mark.parametrize("nh,nkv,ps", [(32, 8, 16), (3, 1, 16), (5, 5, 4), (4, 2, 8), (16, 2, 16), (6, 2, 6)])
@pytest.mark.parametrize("window,paired,halves", [(None, True, 1), (None, False, 1), (37, False, 1), (200, False, 1), (200, True, 1),
                                                   (None, False, 2), (None, True, 2), (37, False, 2), (200, True, 2)])
def test_attention_prefill_wide(ops, nh, nkv, ps, window, paired, halves):
    """The kernel for long portions, heads of 64: four sequences in one launch (a long chunk over a cached prefix that
    ends inside a page, a fresh prompt of some hundred tokens, a single token, a chunk that starts at a step's edge).
    Rows of pages past a sequence's end hold NaN: a value read from there, even with weight zero, would show.
    A block's sub-tiles of 32 queries as neighbours, and paired from both ends of the sequence (late with early); the
    keys walked whole, and in two halves by two wavefronts that merge at the end."""
    from gesso_amd.engine.batch import subtile_lists
    d = 64
    assert ops.attention_prefill_wide_supports(nh, nkv, d) and not ops.attention_prefill_wide_supports(nh, nkv, 128)
    rows = ops.attention_prefill_wide_rows(nh, nkv)
    assert rows == {1: 256, 2: 128, 3: 64, 4: 64}.get(nh // nkv, 32)
    if halves == 2 and rows < 64:
        pytest.skip("groups of more than four heads hold one sub-tile a block: nothing to halve")
    rows //= halves
    g = gen(nh + ps + (window or 0))
    prefix, new = [75, 0, 45, 128], [141, 333, 1, 70]
    kcs, vcs, tables, qs, want = [], [], [], [], []
    base = 0
    for i, (p0, n) in enumerate(zip(prefix, new)):
        K = p0 + n
        k, v = torch.randn(K, nkv, d, generator=g).bfloat16(), torch.randn(K, nkv, d, generator=g).bfloat16()
        q = torch.randn(n, nh, d, generator=g)
        if i == 1:
            q[-1] *= 3.0                                   # sharper weights on one row
            k[7] = (q[-1, ::nh // nkv] * 0.5).bfloat16()   # and a far key that carries weight for it
        q = q.bfloat16()
        kc, vc, tab = paged(k, v, ps, g)
        kcs.append(kc); vcs.append(vc); tables.append(tab + base)
        base += kc.shape[0]
        qs.append(q.reshape(n, -1))
        want.append(P.causal_attention(q.double(), k.double(), v.double(), window or 0).reshape(n, -1))
    kc, vc = torch.cat(kcs), torch.cat(vcs)
    table = torch.zeros(len(new), max(t.numel() for t in tables), dtype=torch.int32)
    for i, t in enumerate(tables):
        table[i, :t.numel()] = t
    qall, want = torch.cat(qs), torch.cat(want)
    positions = torch.tensor([p + j for p, n in zip(prefix, new) for j in range(n)], dtype=torch.int32)
    tiles = torch.tensor(subtile_lists(new, rows // 32, 0, paired), dtype=torch.int32)
    assert tiles.shape[1] % (rows // 32) == 0 and int(tiles[2].sum()) == sum(new)
    stride = (nh + 2 * nkv) * d
    wide = torch.zeros(sum(new), stride, dtype=torch.bfloat16)
    wide[:, :nh * d] = qall
    got = ops.attention_prefill_wide(wide.to(DEV), stride, kc.to(DEV), vc.to(DEV), positions.to(DEV), tiles.to(DEV),
                                     table.to(DEV), ps, window, 1.0 / math.sqrt(d), nh, nkv, d, sum(new), key_splits=halves)
    close(got, want, torch.bfloat16)


@pytest.mark.parametrize("kernel", ["wide", "wide-halves", "tiles16", "tiles32"])
@pytest.mark.parametrize("window", [None, 50])
def test_prompt_attention_never_sees_the_next_key_nor_the_one_before_its_window(ops, kernel, window):
    """Every key stands out for the query one place before it (and, with a window, for the query `window` places after
    it): a causal mask or a window's edge that is off by one lets one such key in, and it then carries nearly all of
    that query's weight.  One chunk of 150 queries over a prefix of 83 keys, heads of 64 in groups of two."""
    g = gen(9 + (window or 0))
    nh, nkv, d, ps, prefix, new = 4, 2, 64, 16, 83, 150
    K = prefix + new
    G = nh // nkv
    v = torch.randn(K, nkv, d, generator=g)
    q = torch.randn(new, nh, d, generator=g)
    k = torch.randn(K, nkv, d, generator=g) * 0.3
    for u in range(prefix + 1, K):                        # key u: for query u - 1 (the next key: never visible)
        k[u] += q[u - 1 - prefix, ::G] * 6.0
    if window:
        for u in range(prefix - window, K - window):      # key u: also for query u + window (just outside its window)
            if u >= 0:
                k[u] += q[u + window - prefix, ::G] * 6.0
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    want = P.causal_attention(q.double(), k.double(), v.double(), window or 0).reshape(new, -1)
    # the control: with the mask one place too wide the result is another one altogether
    if not window:
        loose = P.causal_attention(torch.cat([q.double()[1:], q.double()[-1:]]), k.double(), v.double(), 0).reshape(new, -1)
        assert float((loose - want).abs().max()) > 0.5
    kc, vc, tab = paged(k, v, ps, g)
    positions = torch.arange(prefix, K, dtype=torch.int32)
    halves = 2 if kernel == "wide-halves" else 1
    rows = ops.attention_prefill_wide_rows(nh, nkv) // halves if kernel.startswith("wide") else int(kernel[5:])
    if kernel.startswith("wide"):
        from gesso_amd.engine.batch import subtile_lists
        tiles = torch.tensor(subtile_lists([new], rows // 32, 0, paired=not window), dtype=torch.int32)
    else:
        tiles = torch.tensor([[0] * -(-new // rows), list(range(0, new, rows)), [min(rows, new - a) for a in range(0, new, rows)]],
                             dtype=torch.int32)
    args = (q.reshape(new, -1).to(DEV), nh * d, kc.to(DEV), vc.to(DEV), positions.to(DEV), tiles.to(DEV), tab[None].to(DEV), ps,
            window, 1.0 / math.sqrt(d), nh, nkv, d, new)
    got = ops.attention_prefill_wide(*args, key_splits=halves) if kernel.startswith("wide") else ops.attention_prefill(*args, tile_rows=rows)
    close(got, want, torch.bfloat16)


def test_attention_prefill_wide_over_thousands_of_keys(ops):
    """A chunk of 200 queries over a prefix of 5,000 keys in pages of two (the most pages a step can touch), with and
    without a window; one key far back carries weight for the last query."""
    g = gen(6)
    nh, nkv, d, ps, prefix, new = 8, 2, 64, 2, 5000, 200
    K = prefix + new
    for window in (None, 3000):
        k, v, q = torch.randn(K, nkv, d, generator=g), torch.randn(K, nkv, d, generator=g), torch.randn(new, nh, d, generator=g)
        far = 1999 if window is None else K - 2990
        k[far, 0] = q[-1, 0] * 1.5
        q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
        kc, vc, tab = paged(k, v, ps, g)
        from gesso_amd.engine.batch import subtile_lists
        want = P.causal_attention(q.double(), k.double(), v.double(), window or 0).reshape(new, -1)
        for halves in (1, 2):          # the far key lies in the first half of the walk, the queries' own keys in the second
            rows = ops.attention_prefill_wide_rows(nh, nkv) // halves
            tiles = torch.tensor(subtile_lists([new], rows // 32, 0, paired=not window), dtype=torch.int32)
            got = ops.attention_prefill_wide(q.reshape(new, -1).to(DEV), nh * d, kc.to(DEV), vc.to(DEV),
                                             torch.arange(prefix, K, dtype=torch.int32, device=DEV), tiles.to(DEV),
                                             tab[None].contiguous().to(DEV), ps, window, 1.0 / math.sqrt(d), nh, nkv, d, new,
                                             key_splits=halves)
            close(got, want, torch.bfloat16)


# ------------------------------------------------------------------ rows in the matrix cores' order (tiled rows)



@pytest.mark.parametrize("M,K", [(1, 32), (5, 96), (16, 2048), (33, 64), (64, 8192)])
def test_tiled_rows_hold_the_same_values(ops, M, K):
    x = torch.randn(M, K, generator=gen(M + K)).bfloat16().to(DEV)
    t = ops.TiledRows.of(x)
    assert t.shape == (M, K) and t.buf.numel() == -(-M // 16) * 16 * K
    # element (m, k): step k // 32, row tile m // 16, lane 16 ((k % 32) // 8) + m % 16, element k % 8
    for m, k in ((0, 0), (M - 1, K - 1), (M // 2, K // 3), (M - 1, 17)):
        at = (((k // 32) * (-(-M // 16)) + m // 16) * 64 + ((k % 32) // 8) * 16 + m % 16) * 8 + k % 8
        assert t.buf[at] == x[m, k]
    assert torch.equal(t.rows(), x)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(2048, 2048), (128, 64), (6144, 2048), (192, 8192)])
def test_products_of_tiled_rows_equal_those_of_rows_bit_for_bit(ops, M, N, K):
    g = gen(M + N + K)
    x = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    xt = ops.TiledRows.of(x)
    for wt in (None, ops.tile_major(w)):
        for kw in ({}, {"out_dtype": torch.float32}, {"swiglu": True}):
            assert torch.equal(ops.gemm_skinny(xt, w, wt=wt, **kw), ops.gemm_skinny(x, w, wt=wt, **kw))
        # the SwiGLU epilogue writing tiled rows
        a = ops.gemm_skinny(xt, w, wt=wt, swiglu=True, out=True)
        assert isinstance(a, ops.TiledRows) and torch.equal(a.rows(), ops.gemm_skinny(x, w, wt=wt, swiglu=True))
        # into the residual stream, the rows for the next norm tiled as well
        res = torch.randn(M, N, generator=g)
        nw = (1 + 0.3 * torch.randn(N, generator=g)).to(DEV)
        r1, r2 = res.clone().to(DEV), res.clone().to(DEV)
        xs1, xs2 = ops.TiledRows(M, N, DEV), torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        s1 = ops.gemm_skinny_residual(xt, w, r1, wt=wt, next_weight=nw, xs=xs1)
        s2 = ops.gemm_skinny_residual(x, w, r2, wt=wt, next_weight=nw, xs=xs2)
        assert torch.equal(r1, r2) and torch.equal(s1, s2) and torch.equal(xs1.rows(), xs2)
        # a product of the pre-weighted tiled rows, scaled by the rows' inverse root mean squares
        w2 = (torch.randn(64, N, generator=g) / math.sqrt(N)).bfloat16().to(DEV)
        l1 = ops.LazyNorm(r1, s1, nw, 1e-5, torch.bfloat16, xs=xs1)
        l2 = ops.LazyNorm(r2, s2, nw, 1e-5, torch.bfloat16, xs=xs2)
        assert torch.equal(ops.gemm_skinny(l1, w2), ops.gemm_skinny(l2, w2))
        # in parts, the normed rows tiled
        for parts in (1, 4):
            r1, r2 = res.clone().to(DEV), res.clone().to(DEV)
            q1, n1 = ops.gemm_skinny_residual_parts(xt, w, r1, parts, wt=wt, next_weight=nw, eps=1e-5, tiled=True)
            q2, n2 = ops.gemm_skinny_residual_parts(x, w, r2, parts, wt=wt, next_weight=nw, eps=1e-5)
            assert isinstance(n1, ops.TiledRows)
            assert torch.equal(r1, r2) and torch.equal(q1, q2) and torch.equal(n1.rows(), n2)


@pytest.mark.parametrize("M,H,W,bias", [(1, 64, 3, False), (8, 2048, 3, False), (20, 96, 4, True), (64, 160, 2, False),
                                         (40, 2048, 3, False)])
def test_convolution_product_of_tiled_rows(ops, M, H, W, bias):
    g = gen(M + H + W)
    x = torch.randn(M, H, generator=g).bfloat16().to(DEV)
    w_in = (torch.randn(3 * H, H, generator=g) / math.sqrt(H)).bfloat16().to(DEV)
    taps = torch.randn(H, W, generator=g).to(DEV)
    b = torch.randn(H, generator=g).to(DEV) if bias else None
    state0 = torch.randn(M + 2, H, W - 1, generator=g)
    slots = torch.randperm(M + 2, generator=g)[:M].to(torch.int32).to(DEV)
    for wt in (None, ops.tile_major(w_in)):
        s1, s2 = state0.clone().to(DEV), state0.clone().to(DEV)
        got = ops.gemm_skinny_conv(ops.TiledRows.of(x), w_in, taps, b, s1, slots, wt=wt, tiled=True)
        want = ops.gemm_skinny_conv(x, w_in, taps, b, s2, slots, wt=wt)
        assert isinstance(got, ops.TiledRows) and torch.equal(got.rows(), want) and torch.equal(s1, s2)


@pytest.mark.parametrize("T,H,V", [(1, 2048, 1000), (9, 96, 301), (40, 64, 50)])
def test_embed_writes_tiled_rows(ops, T, H, V):
    g = gen(T + H)
    table = torch.randn(V, H, generator=g).bfloat16().to(DEV)
    ids = torch.randint(0, V, (T,), generator=g).to(torch.int32).to(DEV)
    nw = (1 + 0.3 * torch.randn(H, generator=g)).to(DEV)
    xs1, xs2 = ops.TiledRows(T, H, DEV), torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    o1 = ops.embed(ids, table, next_weight=nw, xs=xs1)
    o2 = ops.embed(ids, table, next_weight=nw, xs=xs2)
    assert torch.equal(o1, o2) and torch.equal(xs1.rows(), xs2)


@pytest.mark.parametrize("nh,nkv,d,nsplit,raw", [(32, 8, 64, 1, True), (32, 8, 64, 4, True), (4, 2, 16, 1, False),
                                                 (3, 1, 32, 3, False), (8, 1, 128, 2, True)])
def test_attention_decode_writes_tiled_rows(ops, nh, nkv, d, nsplit, raw):
    g = gen(nh + d + nsplit)
    ps, lens = 16, [1, 64, 65, 300, 17, 129] * 4          # 24 sequences: two row tiles
    nseq = len(lens)
    nblk = [-(-n // ps) for n in lens]
    kc = torch.randn(sum(nblk) + 1, nkv, ps, d, generator=g).bfloat16().to(DEV)
    vc = torch.randn(sum(nblk) + 1, nkv, ps, d, generator=g).bfloat16().to(DEV)
    table = torch.zeros(nseq, max(nblk), dtype=torch.int32)
    at = 0
    for i in range(nseq):
        table[i, :nblk[i]] = torch.arange(at, at + nblk[i], dtype=torch.int32)
        at += nblk[i]
    table = table.to(DEV)
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32).to(DEV)
    scale = 1.0 / math.sqrt(d)
    if raw:
        stride = (nh + 2 * nkv) * d
        qkv = torch.randn(nseq, stride, generator=g).bfloat16().to(DEV)
        qw = (1 + 0.2 * torch.randn(d, generator=g)).to(DEV)
        kw = (1 + 0.2 * torch.randn(d, generator=g)).to(DEV)
        cos, sin = rope_tables(d, 1e4, 512)
        run = lambda out: ops.attention_decode_raw(qkv, stride, kc.clone(), vc.clone(), positions, table, ps, None, scale,
                                                   qw, kw, 1e-5, cos, sin, nh, nkv, d, nseq, nsplit, out=out)
    else:
        q = torch.randn(nseq, nh * d, generator=g).bfloat16().to(DEV)
        run = lambda out: ops.attention_decode(q, nh * d, kc, vc, positions, table, ps, None, scale, nh, nkv, d, nseq,
                                               nsplit, out=out)
    got, want = run(True), run(None)
    assert isinstance(got, ops.TiledRows) and torch.equal(got.rows(), want)


def test_tiled_rows_refuse_widths_that_are_no_multiple_of_32(ops):
    from gesso_amd.errors import KernelError
    with pytest.raises(KernelError):
        ops.TiledRows(4, 40, DEV)
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(80, 64, dtype=torch.bfloat16, device=DEV)      # SwiGLU output 40 wide
    with pytest.raises(KernelError):
        ops.gemm_skinny(x, w, swiglu=True, out=True)


# ------------------------------------------------------------------ the matrix-core product for many rows

@pytest.mark.parametrize("M,N,K", [(65, 96, 72), (200, 320, 192), (513, 1000, 264), (129, 64, 8), (2048, 6144, 2048),
                                    (300, 16384, 512), (1, 40, 64), (256, 256, 64)])
def test_gemm_mfma(ops, M, N, K):
    g = gen(M + N + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    want = x.double() @ w.double().T
    close(ops.gemm_mfma(x.to(DEV), w.to(DEV)), want, torch.bfloat16)
    got32 = ops.gemm_mfma(x.to(DEV), w.to(DEV), out_dtype=torch.float32)
    assert got32.dtype == torch.float32
    # float32 sums of exact products: only the order of the sums differs from the float64 reference
    assert float((got32.double().cpu() - want).abs().max()) <= 2e-5 * math.sqrt(K) * max(1.0, float(want.abs().max()))
    # rows of a wider buffer (a row stride beyond K)
    wide = torch.zeros(M, K + 16, dtype=torch.bfloat16)
    wide[:, :K] = x
    assert torch.equal(ops.gemm_mfma(wide.to(DEV)[:, :K], w.to(DEV)), ops.gemm_mfma(x.to(DEV), w.to(DEV)))


@pytest.mark.parametrize("M,F,K", [(65, 24, 64), (200, 100, 96), (130, 8192, 256), (700, 1000, 136), (2048, 4608, 1024)])
def test_gemm_mfma_swiglu(ops, M, F, K):
    g = gen(M + F + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(2 * F, K, generator=g) / math.sqrt(K) * 2).bfloat16()
    got = ops.gemm_mfma(x.to(DEV), w.to(DEV), swiglu=True)
    assert got.shape == (M, F)
    y = x.double() @ w.double().T
    close(got, P.swiglu(y[:, :F], y[:, F:]), torch.bfloat16, scale=2)
    # and it is the plain product followed by the SwiGLU kernel, value for value (both round gate and up to bfloat16)
    two = ops.swiglu(ops.gemm_mfma(x.to(DEV), w.to(DEV)))
    assert float((got.float() - two.float()).abs().max()) <= 1e-2 * max(1.0, float(two.float().abs().max()))


def test_gemm_mfma_stands_out_where_one_weight_row_matters(ops):
    """A product whose every output is zero but one: a wrong pairing of rows and columns anywhere shows."""
    M, N, K = 300, 520, 200
    x = torch.zeros(M, K, dtype=torch.bfloat16)
    w = torch.zeros(N, K, dtype=torch.bfloat16)
    for (m, n, k) in ((0, 0, 0), (299, 519, 199), (37, 301, 65), (256, 255, 64), (128, 256, 127)):
        x[m, k] = 2.0
        w[n, k] = 3.0
    got = ops.gemm_mfma(x.to(DEV), w.to(DEV), out_dtype=torch.float32).cpu()
    want = x.float() @ w.float().T
    assert torch.equal(got, want) and int((want != 0).sum()) == 5


def test_gemm_mfma_refuses(ops):
    from gesso_amd.errors import KernelError
    x = torch.zeros(70, 60, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(16, 60, dtype=torch.bfloat16, device=DEV)
    assert not ops.mfma_ok(x, w)                           # K no multiple of 8
    with pytest.raises(KernelError):
        ops.gemm_mfma(x, w)
