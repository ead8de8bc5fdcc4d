"""What fixes the plain implementation beside the reference's text.

Vectors that the reference's own tests hold, special cases that reduce to a library routine,
and invariants; each chosen so that a plausible mistake (a wrong sign or pairing, a norm in
the wrong place, a tap order reversed) fails it.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_lfm2 as P
from tiny import CONFIGS, random_ids, write_tiny



@pytest.fixture(autouse=True)
def float64_by_default():
    """The plain implementation is exercised in float64; the default is put back after each test."""
    before = torch.get_default_dtype()
    torch.set_default_dtype(torch.float64)
    yield
    torch.set_default_dtype(before)


# ------------------------------------------------------------------ vectors of the reference's tests

def test_embedding_zero_based_ids():
    # test/test_cpu_ops.jl:14-24
    table = torch.tensor([[10., 11, 12], [20, 21, 22], [30, 31, 32], [40, 41, 42]])
    got = P.embedding(table, [2, 0])
    assert torch.equal(got, torch.tensor([[30., 31, 32], [10, 11, 12]]))
    with pytest.raises(ValueError):
        P.embedding(table, [4])


def test_rmsnorm_vector_and_last_axis():
    # test/test_cpu_ops.jl:26-51, eps 1e-6
    x = torch.tensor([[1., 2], [3, 4]])
    w = torch.tensor([10., 20])
    eps = 1e-6
    want = torch.stack([x[i] / math.sqrt((x[i, 0] ** 2 + x[i, 1] ** 2) / 2 + eps) * w for i in range(2)])
    assert torch.allclose(P.rmsnorm(x, w, eps), want, atol=1e-12)
    x3 = torch.arange(1., 13.).reshape(2, 2, 3)
    got = P.rmsnorm(x3, torch.ones(3), eps)
    for t in range(2):
        for h in range(2):
            row = x3[t, h]
            assert torch.allclose(got[t, h], row / math.sqrt(float((row * row).sum()) / 3 + eps), atol=1e-12)


def test_rmsnorm_ones_and_scale_invariance():
    w = torch.tensor([0.5, 2.0, -1.0, 3.0])
    eps = 1e-5
    assert torch.allclose(P.rmsnorm(torch.ones(1, 4), w, eps), (w / math.sqrt(1 + eps))[None], atol=1e-15)
    x = torch.randn(3, 4, generator=torch.Generator().manual_seed(0))
    assert torch.allclose(P.rmsnorm(1e6 * x, w, eps), P.rmsnorm(1e3 * x, w, eps), atol=1e-9)
    # eps sits inside the root: for a zero row the result is 0 / sqrt(eps), not a division by zero
    assert torch.equal(P.rmsnorm(torch.zeros(1, 4), w, eps), torch.zeros(1, 4))


def _julia_cube(start, t, h, d):
    """reshape(start:..., t, h, d) of a column-major language: element [a, b, c] = start + a + t*b + t*h*c."""
    out = torch.empty(t, h, d)
    for a in range(t):
        for b in range(h):
            for c in range(d):
                out[a, b, c] = start + a + t * b + t * h * c
    return out


def test_rope_half_split_vector():
    # test/test_rope_layout.jl:3-24: positions [0, 3], theta 10000, pairs (i, i + d/2); K over its own single head
    q0, k0 = _julia_cube(1, 2, 2, 8), _julia_cube(33, 2, 1, 8)
    for src in (q0, k0):
        got = P.rope(src, [0, 3], 10000.0)
        assert torch.equal(got[0], src[0])          # position 0 is the identity, bit for bit
        for h in range(src.shape[1]):
            for i in range(4):
                ang = 3 * 10000.0 ** (-2 * i / 8)
                a, b = float(src[1, h, i]), float(src[1, h, i + 4])
                assert got[1, h, i] == pytest.approx(a * math.cos(ang) - b * math.sin(ang), abs=1e-12)
                assert got[1, h, i + 4] == pytest.approx(b * math.cos(ang) + a * math.sin(ang), abs=1e-12)


def test_rope_is_a_rotation_and_relative():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 16, generator=g), torch.randn(1, 1, 16, generator=g)
    rq = P.rope(q, [7], 1e4)
    for i in range(8):   # each pair keeps its length
        assert rq[0, 0, i] ** 2 + rq[0, 0, i + 8] ** 2 == pytest.approx(float(q[0, 0, i] ** 2 + q[0, 0, i + 8] ** 2))
    dots = [float((P.rope(q, [m], 1e4) * P.rope(k, [n], 1e4)).sum()) for m, n in ((5, 2), (13, 10), (103, 100))]
    assert dots[0] == pytest.approx(dots[1], abs=1e-10) and dots[0] == pytest.approx(dots[2], abs=1e-10)
    assert abs(dots[0] - float((P.rope(q, [5], 1e4) * P.rope(k, [3], 1e4)).sum())) > 1e-3


def test_conv_hand_vector():
    # test/test_lfm25.jl:79-90: h = ones(4,1), norm weight 1, W_in = ones(3,1), taps [2,-1,3], W_out = 1, eps 1e-5
    w = {"p.operator_norm.weight": torch.ones(1), "p.conv.in_proj.weight": torch.ones(3, 1),
         "p.conv.conv.weight": torch.tensor([[[2., -1, 3]]]), "p.conv.out_proj.weight": torch.ones(1, 1)}
    h = torch.ones(4, 1)
    out, _ = P.conv_block(h, w, "p.", 1e-5)
    want = torch.tensor([3., 2, 4, 4]) / (1 + 1e-5) ** 1.5
    assert torch.allclose((out - h)[:, 0], want, atol=1e-12)


def test_softmax_vectors_through_attention():
    # test/test_cpu_ops.jl:87-132: with q = sqrt(d) * I and k_u = column u of S the scores are S; v = I shows the weights
    S = torch.tensor([[3., 1, .5], [2, 4, 1], [.1, .2, .3]])
    q = (math.sqrt(3) * torch.eye(3))[:, None, :]
    k = S.t().contiguous()[:, None, :]
    v = torch.eye(3)[:, None, :]
    p = P.causal_attention(q, k, v)[:, 0, :]
    assert p[0, 0] == 1.0 and p[0, 1] == 0.0 and p[0, 2] == 0.0 and p[1, 2] == 0.0
    e = math.exp(2.0) / (math.exp(2.0) + math.exp(4.0))
    assert torch.allclose(p[1, :2], torch.tensor([e, 1 - e]), atol=1e-12)
    r = torch.exp(torch.tensor([.1, .2, .3]))
    assert torch.allclose(p[2], r / r.sum(), atol=1e-12)
    assert torch.allclose(p.sum(1), torch.ones(3), atol=1e-12)
    # a decode row (one query, three keys) sees the whole cache
    p1 = P.causal_attention(q[2:3] * 0 + torch.tensor([[[math.sqrt(3), 0, 0]]]),
                            torch.tensor([[1., 0, 0], [2, 0, 0], [3, 0, 0]])[:, None, :], v)[0, 0]
    r = torch.exp(torch.tensor([1., 2, 3]))
    assert torch.allclose(p1, r / r.sum(), atol=1e-12)
    # huge scores do not overflow
    big = P.causal_attention(1e6 * q, 1e6 * torch.ones(3, 1, 3), v)
    assert torch.isfinite(big).all()


def test_swiglu_vector():
    # test/test_cpu_ops.jl:134-141
    g, u = torch.tensor([-1., .5, 2.]), torch.tensor([3., -.25, 1.])
    assert torch.allclose(P.swiglu(g, u), g / (1 + torch.exp(-g)) * u, atol=1e-15)
    assert torch.allclose(P.swiglu(g, u), F.silu(g) * u, atol=1e-12)


def test_linear_is_x_times_w_transposed():
    # test/test_cpu_ops.jl:77-85: W is (out, in)
    x = torch.tensor([[1., 2, 3], [4, 5, 6]])
    w = torch.tensor([[1., 0, 1], [0, 1, 0]])
    assert torch.equal(P.linear(x, w), torch.tensor([[4., 2], [10, 5]]))


# ------------------------------------------------------------------ special cases that are library routines

def test_conv_with_unit_gates_is_conv1d():
    g = torch.Generator().manual_seed(2)
    T, H, W = 11, 5, 4
    x = torch.randn(T, H, generator=g)
    taps = torch.randn(H, W, generator=g)
    bcx = torch.cat([torch.ones(T, H), torch.ones(T, H), x], 1)
    got, hist = P.short_conv(bcx, taps)
    want = F.conv1d(F.pad(x.t()[None], (W - 1, 0)), taps[:, None, :], groups=H)[0].t()
    assert torch.allclose(got, want, atol=1e-12)
    assert torch.allclose(hist, x[-(W - 1):].t(), atol=0)
    # reversed taps are another convolution (test/test_lfm25.jl:189-194)
    assert (P.short_conv(bcx, taps.flip(1))[0] - got).abs().max() > 1e-2


def test_conv_gate_placement_and_bias():
    g = torch.Generator().manual_seed(3)
    T, H, W = 6, 3, 3
    bcx = torch.randn(T, 3 * H, generator=g)
    taps, bias = torch.randn(H, W, generator=g), torch.randn(H, generator=g)
    B, C, X = bcx[:, :H], bcx[:, H:2 * H], bcx[:, 2 * H:]
    u = F.pad((B * X).t()[None], (W - 1, 0))
    y = F.conv1d(u, taps[:, None, :], groups=H)[0].t()
    assert torch.allclose(P.short_conv(bcx, taps)[0], C * y, atol=1e-12)
    assert torch.allclose(P.short_conv(bcx, taps, bias)[0], C * (y + bias), atol=1e-12)


def test_conv_chunks_carry_the_history():
    # test/test_amdgpu_lfm2.jl:66-73: seq in (5, 1, 1, 4) with the history carried equals the whole
    g = torch.Generator().manual_seed(4)
    H, W = 7, 4
    bcx = torch.randn(11, 3 * H, generator=g)
    taps = torch.randn(H, W, generator=g)
    whole, hist_whole = P.short_conv(bcx, taps)
    hist, at, outs = None, 0, []
    for n in (5, 1, 1, 4):
        o, hist = P.short_conv(bcx[at:at + n], taps, hist=hist)
        outs.append(o)
        at += n
    assert torch.equal(torch.cat(outs), whole) and torch.equal(hist, hist_whole)
    # a history that lags one token behind gives another result (test/test_lfm25.jl:206-235)
    _, lag = P.short_conv(bcx[:9], taps)
    _, good = P.short_conv(bcx[:10], taps)
    assert (P.short_conv(bcx[10:], taps, hist=lag)[0] - whole[10:]).abs().max() > 1e-3
    assert torch.equal(P.short_conv(bcx[10:], taps, hist=good)[0], whole[10:])


def test_conv_nan_stays_in_its_channel():
    # test/test_amdgpu_lfm2.jl:95-101
    g = torch.Generator().manual_seed(5)
    bcx = torch.randn(4, 9, generator=g)
    bcx[1, 1] = float("nan")
    out, _ = P.short_conv(bcx, torch.randn(3, 3, generator=g))
    assert torch.isnan(out[:, 1]).any() and torch.isfinite(out[:, [0, 2]]).all()


@pytest.mark.parametrize("nh,nkv", [(4, 4), (4, 2), (3, 1), (1, 1)])
def test_attention_is_sdpa_with_repeated_heads(nh, nkv):
    g = torch.Generator().manual_seed(6)
    T, d = 9, 8
    q, k, v = (torch.randn(T, n, d, generator=g) for n in (nh, nkv, nkv))
    got = P.causal_attention(q, k, v)
    rep = nh // nkv
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(rep, 1).transpose(0, 1)[None],
                                          v.repeat_interleave(rep, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-12)


def test_attention_offset_window_and_zero_weight():
    g = torch.Generator().manual_seed(7)
    K, L, d = 10, 3, 4
    q = torch.randn(L, 2, d, generator=g)
    k, v = torch.randn(K, 1, d, generator=g), torch.randn(K, 1, d, generator=g)
    got = P.causal_attention(q, k, v)
    # query t of the last L rows sees keys 0 .. K-L+t: changing a later key or value changes nothing
    k2, v2 = k.clone(), v.clone()
    k2[K - L + 1:] += 100.0
    v2[K - L + 1:] -= 50.0
    assert torch.equal(P.causal_attention(q, k2, v2)[0], got[0])
    assert not torch.equal(P.causal_attention(q, k2, v2)[1], got[1])
    # a window of 4: key K-L+t-4 has no weight, key K-L+t-3 has
    w = P.causal_attention(q, k, v, window=4)
    k3 = k.clone()
    k3[K - L - 4] += 100.0
    assert torch.equal(P.causal_attention(q, k3, v, window=4)[0], w[0])
    k3 = k.clone()
    k3[K - L - 3] += 100.0
    assert not torch.equal(P.causal_attention(q, k3, v, window=4)[0], w[0])
    # a window as long as the sequence is no window
    assert torch.equal(P.causal_attention(q, k, v, window=K), got)


def test_each_head_has_its_own_softmax():
    # test/test_attention_heads.jl:4: scaling one head's queries changes only that head's output
    g = torch.Generator().manual_seed(8)
    q, k, v = torch.randn(5, 2, 4, generator=g), torch.randn(5, 2, 4, generator=g), torch.randn(5, 2, 4, generator=g)
    a = P.causal_attention(q, k, v)
    q2 = q.clone()
    q2[:, 0] *= 3.0
    b = P.causal_attention(q2, k, v)
    assert torch.equal(a[:, 1], b[:, 1]) and not torch.equal(a[:, 0], b[:, 0])


# ------------------------------------------------------------------ the whole model

@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("plain"))
    out = {}
    for name in CONFIGS:
        d = write_tiny(root, name, torch.float32)
        out[name] = (P.read_config(d), P.read_weights(d))
    return out


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_shift_of_all_positions_changes_nothing(tiny, name):
    cfg, w = tiny[name]
    ids = random_ids(12, cfg["V"], 3)
    a = P.forward(cfg, w, ids)
    b = P.forward(cfg, w, ids, start_pos=37)
    assert torch.allclose(a, b, atol=1e-9)
    # and a change of distances does change it: rotating q and k by different amounts
    assert (P.forward(dict(cfg, theta=cfg["theta"] * 3), w, ids) - a).abs().max() > 1e-4


def test_controls_that_must_move_the_logits(tiny):
    cfg, w = tiny["A"]
    ids = random_ids(10, cfg["V"], 4)
    ref = P.forward(cfg, w, ids)

    def moved(w2):
        return float((P.forward(cfg, w2, ids) - ref).abs().max())

    swapped = dict(w)
    swapped["model.layers.0.feed_forward.w1.weight"], swapped["model.layers.0.feed_forward.w3.weight"] = \
        w["model.layers.0.feed_forward.w3.weight"], w["model.layers.0.feed_forward.w1.weight"]
    assert moved(swapped) > 1e-3
    rev = dict(w)
    rev["model.layers.0.conv.conv.weight"] = w["model.layers.0.conv.conv.weight"].flip(-1)
    assert moved(rev) > 1e-3
    qn = dict(w)
    qn["model.layers.1.self_attn.q_layernorm.weight"] = w["model.layers.1.self_attn.q_layernorm.weight"].flip(0)
    assert moved(qn) > 1e-4        # the head norm's weight is indexed by feature, before the rotation


def test_head_norm_stands_before_the_rotation(tiny):
    cfg, w = tiny["A"]
    g = torch.Generator().manual_seed(9)
    x = torch.randn(3, cfg["nh"], cfg["d"], generator=g)
    wn = w["model.layers.1.self_attn.q_layernorm.weight"]
    a = P.rope(P.rmsnorm(x, wn, cfg["eps"]), [0, 5, 9], cfg["theta"])
    b = P.rmsnorm(P.rope(x, [0, 5, 9], cfg["theta"]), wn, cfg["eps"])
    assert (a - b).abs().max() > 1e-3
    # the block does it in the first order: recompute one attention block by hand
    h = torch.randn(4, cfg["H"], generator=g)
    p = "model.layers.1."
    n = P.rmsnorm(h, w[p + "operator_norm.weight"], cfg["eps"])
    q = P.rope(P.rmsnorm((n @ w[p + "self_attn.q_proj.weight"].T).reshape(4, cfg["nh"], cfg["d"]), wn, cfg["eps"]),
               range(4), cfg["theta"])
    k = P.rope(P.rmsnorm((n @ w[p + "self_attn.k_proj.weight"].T).reshape(4, cfg["nkv"], cfg["d"]),
                         w[p + "self_attn.k_layernorm.weight"], cfg["eps"]), range(4), cfg["theta"])
    v = (n @ w[p + "self_attn.v_proj.weight"].T).reshape(4, cfg["nkv"], cfg["d"])
    o = P.causal_attention(q, k, v).reshape(4, -1) @ w[p + "self_attn.out_proj.weight"].T
    assert torch.allclose(P.attention_block(h, w, p, cfg, list(range(4))), h + o, atol=1e-12)


def test_tied_and_untied_heads(tiny):
    cfg, w = tiny["A"]
    assert cfg["tied"] and "lm_head.weight" not in w
    cfg_b, w_b = tiny["B"]
    assert not cfg_b["tied"] and "lm_head.weight" in w_b
    ids = random_ids(6, cfg_b["V"], 5)
    a = P.forward(cfg_b, w_b, ids)
    w2 = dict(w_b)
    w2["lm_head.weight"] = w_b["lm_head.weight"].flip(0)
    assert torch.allclose(P.forward(cfg_b, w2, ids), a.flip(1), atol=1e-12)


def test_prefix_logits_do_not_depend_on_what_follows(tiny):
    cfg, w = tiny["B"]
    ids = random_ids(14, cfg["V"], 6)
    a = P.forward(cfg, w, ids)
    b = P.forward(cfg, w, ids[:9])
    assert torch.allclose(a[:9], b, atol=1e-10)


def test_greedy_is_argmax_of_the_last_row(tiny):
    cfg, w = tiny["B"]
    prompt = random_ids(5, cfg["V"], 7)
    ids = P.greedy(cfg, w, prompt, 3)
    assert P.greedy(cfg, w, prompt, 0) == prompt
    for k in range(3):
        assert ids[5 + k] == int(torch.argmax(P.forward(cfg, w, ids[:5 + k])[-1]))


# ------------------------------------------------------------------ sampling

def test_splitmix64_stream():
    # the generator's published first outputs for seed 0
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    state = 0
    for z in want:
        state, u = P.splitmix64_unit(state)
        assert u == float(z >> 11) * 2.0 ** -53 and 0.0 <= u < 1.0


def test_sampling_rules():
    logits = [0.1, 2.0, -1.0, 2.0, 0.5]
    # low temperature picks the first maximum, whatever the draw (test/test_sampling.jl)
    for seed in range(5):
        assert P.sample_id(logits, 1e-3, 1.0, seed)[0] in (1, 3)
    # same seed, same id; the state advances by exactly one draw
    a, s1 = P.sample_id(logits, 0.8, 1.0, 7)
    b, s2 = P.sample_id(logits, 0.8, 1.0, 7)
    assert a == b and s1 == s2 == P.splitmix64_unit(7)[0]
    # nucleus: probabilities 0.5, 0.3, 0.2 with top_p 0.5 keep only the first id
    lg = [math.log(0.5), math.log(0.3), math.log(0.2)]
    assert {P.sample_id(lg, 1.0, 0.5, s)[0] for s in range(50)} == {0}
    assert {P.sample_id(lg, 1.0, 0.75, s)[0] for s in range(200)} == {0, 1}
    # frequencies follow the distribution
    n, state, hits = 4000, 11, [0, 0, 0]
    for _ in range(n):
        i, state = P.sample_id(lg, 1.0, 1.0, state)
        hits[i] += 1
    assert abs(hits[0] / n - 0.5) < 0.03 and abs(hits[2] / n - 0.2) < 0.03
