"""Plain LFM2: a slow, whole-sequence, cache-free implementation used as the oracle.

Every function here is written from the formulas of the reference (Orcein-Labs/Gesso)
and cites where they stand.  Nothing is imported from ``gesso_amd``: the model folder
is read with ``json`` and the ``safetensors`` package, the math is explicit loops over
torch CPU tensors in float64 (or float32 on request).  One function per part:

    embedding   rmsnorm   rope   causal_attention   short_conv   swiglu
    conv_block  attention_block  feed_forward_block  forward

Activations are ``(T, features)`` rows, linear weights are ``(out, in)`` and apply as
``y = x @ W.T`` (reference ``src/Operators/cpu.jl:622-632``).
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- parts

def embedding(table: torch.Tensor, ids) -> torch.Tensor:
    """``h[t, :] = E[id_t, :]`` with 0-based ids and no scale.

    Reference: ``src/Operators/cpu.jl:85-90`` (ids are 0-based, one row per token).
    """
    rows = []
    for tok in ids:
        tok = int(tok)
        if not 0 <= tok < table.shape[0]:
            raise ValueError(f"token id {tok} outside the vocabulary of {table.shape[0]}")
        rows.append(table[tok])
    return torch.stack(rows, 0)


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``y = x / sqrt(mean(x^2) + eps) * w`` over the last axis; eps inside the root, no +1.

    Reference: ``src/Operators/cpu.jl:293-312`` (sum of squares / d + eps, sqrt, divide,
    multiply by the scale).
    """
    d = x.shape[-1]
    acc = (x * x).sum(dim=-1, keepdim=True)
    r = torch.sqrt(acc / d + eps)
    return (x / r) * weight


def rope(x: torch.Tensor, positions, theta: float) -> torch.Tensor:
    """Half-split rotary encoding of ``x (T, heads, d)`` at absolute 0-based positions.

    Pair ``(i, i + d/2)``, angle ``pos * theta^(-2i/d)``;
    ``x_i' = x_i cos - x_{i+d/2} sin``, ``x_{i+d/2}' = x_i sin + x_{i+d/2} cos``.
    Reference: ``src/Operators/cpu.jl:357-371`` with ``interleaved=false``
    (``src/Inference/architecture_spec.jl:66``); pinned by ``test/test_rope_layout.jl:3-24``.
    """
    T, _, d = x.shape
    half = d // 2
    out = x.clone()
    for t in range(T):
        m = float(positions[t])
        for i in range(half):
            ang = m * float(theta) ** (-2.0 * i / d)
            c, s = math.cos(ang), math.sin(ang)
            a = x[t, :, i]
            b = x[t, :, i + half]
            out[t, :, i] = a * c - b * s
            out[t, :, i + half] = a * s + b * c
    return out


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0) -> torch.Tensor:
    """Grouped-query causal attention; ``q (L, nh, d)``, ``k, v (K, nkv, d)`` -> ``(L, nh, d)``.

    Query row ``t`` of ``L`` new rows over ``K`` keys sees keys ``u <= K - L + t`` and, with a
    window, ``u >= K - L + t - window + 1`` (reference ``src/Inference/Inference.jl:1206-1207``).
    Scores are ``q.k / sqrt(d)``; the key head of query head ``h`` is ``h // (nh/nkv)``
    (``src/Inference/Inference.jl:1852-1870``, ``ext/amdgpu_attention.jl:231``); each
    (row, head) has its own softmax: subtract the maximum, ``exp``, divide by the sum
    (``src/Inference/Inference.jl:1414-1430``).
    """
    L, nh, d = q.shape
    K, nkv, _ = k.shape
    g = nh // nkv
    out = torch.zeros_like(q)
    for h in range(nh):
        kh = h // g
        for t in range(L):
            last = K - L + t
            first = max(0, last - window + 1) if window > 0 else 0
            s = (k[first:last + 1, kh, :] @ q[t, h, :]) / math.sqrt(d)
            p = torch.exp(s - s.max())
            p = p / p.sum()
            out[t, h, :] = p @ v[first:last + 1, kh, :]
    return out


def short_conv(bcx: torch.Tensor, taps: torch.Tensor, bias=None, hist=None):
    """Gated causal depthwise convolution between the two projections.

    ``bcx (T, 3H)`` holds B, C, X side by side (in that order); per channel
    ``u = B*X``; ``y[t] = sum_{p<W-1} hist[p] * w[p] + u[t] * w[W-1]`` with taps oldest to
    newest and the current input on the last tap; ``out = C * y``; the history is shifted
    after every token.  Returns ``(out (T, H), hist (H, W-1))``.
    Reference: ``src/Inference/lfm2.jl:253-271``; history zero at a sequence's start
    (``src/Inference/lfm2.jl:195``).  A bias (not bound by the reference) is added to
    ``y`` after the tap sum and before the C gate.
    """
    T, three_h = bcx.shape
    H = three_h // 3
    W = taps.shape[1]
    hist = torch.zeros(H, W - 1, dtype=bcx.dtype) if hist is None else hist.clone()
    out = torch.zeros(T, H, dtype=bcx.dtype)
    for t in range(T):
        bx = bcx[t, 0:H] * bcx[t, 2 * H:3 * H]
        y = torch.zeros(H, dtype=bcx.dtype)
        for p in range(W - 1):
            y = y + hist[:, p] * taps[:, p]
        y = y + bx * taps[:, W - 1]
        if bias is not None:
            y = y + bias
        out[t] = bcx[t, H:2 * H] * y
        for p in range(W - 2):
            hist[:, p] = hist[:, p + 1]
        hist[:, W - 2] = bx
    return out, hist


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(g) * u`` with ``silu(g) = g / (1 + exp(-g))``.  Reference: ``src/Operators/cpu.jl:482-488``."""
    return (gate / (1.0 + torch.exp(-gate))) * up


def linear(x: torch.Tensor, w: torch.Tensor, b=None) -> torch.Tensor:
    """``y = x @ W.T (+ b)`` with ``W (out, in)``.  Reference: ``src/Operators/cpu.jl:622-632``."""
    y = x @ w.T
    return y if b is None else y + b


# --------------------------------------------------------------------------- blocks
#
# ``store`` (default: nothing) is applied wherever an implementation that keeps activations in a narrower type than it
# computes in would store one: the rows a norm hands to a product, a product's result, the mixed rows of the
# convolution, rotated queries and keys, attention's output, the SwiGLU's output.  The residual stream and everything
# inside a function above stay in the type of the inputs.  With ``store = to_bfloat16`` the model shows how far any
# pipeline with bfloat16 activations must stand from the plain one; the reference has no such mode (its device path
# is float32, ``ext/GessoAMDGPUExt.jl:25``).

def _keep(x):
    return x


def to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 (nearest, ties to even) and widen again."""
    return x.to(torch.bfloat16).to(x.dtype)


def conv_block(h, w, prefix, eps, hist=None, store=_keep):
    """norm -> in_proj -> gated conv -> out_proj, added to the stream.

    Reference: ``src/Inference/lfm2.jl:192-204`` and the add at ``src/Inference/Inference.jl:282``.
    """
    n = store(rmsnorm(h, w[prefix + "operator_norm.weight"], eps))
    bcx = store(linear(n, w[prefix + "conv.in_proj.weight"], w.get(prefix + "conv.in_proj.bias")))
    taps = w[prefix + "conv.conv.weight"]
    taps = taps.reshape(taps.shape[0], taps.shape[-1])
    mixed, hist = short_conv(bcx, taps, w.get(prefix + "conv.conv.bias"), hist)
    sub = store(linear(store(mixed), w[prefix + "conv.out_proj.weight"], w.get(prefix + "conv.out_proj.bias")))
    return h + sub, hist


def attention_block(h, w, prefix, cfg, positions, store=_keep):
    """norm -> q,k,v -> per-head q/k norm -> rope -> causal GQA -> out_proj, added to the stream.

    Reference: ``src/Inference/Inference.jl:296-357`` (head norm before the rotation at
    ``:307-323``; heads are feature-major ``f = head*d + j``, ``:302-306``).
    """
    T = h.shape[0]
    nh, nkv, d, eps = cfg["nh"], cfg["nkv"], cfg["d"], cfg["eps"]
    n = store(rmsnorm(h, w[prefix + "operator_norm.weight"], eps))
    q = store(linear(n, w[prefix + "self_attn.q_proj.weight"])).reshape(T, nh, d)
    k = store(linear(n, w[prefix + "self_attn.k_proj.weight"])).reshape(T, nkv, d)
    v = store(linear(n, w[prefix + "self_attn.v_proj.weight"])).reshape(T, nkv, d)
    q = rmsnorm(q, w[prefix + "self_attn.q_layernorm.weight"], eps)
    k = rmsnorm(k, w[prefix + "self_attn.k_layernorm.weight"], eps)
    q = store(rope(q, positions, cfg["theta"]))
    k = store(rope(k, positions, cfg["theta"]))
    o = store(causal_attention(q, k, v).reshape(T, nh * d))
    return h + store(linear(o, w[prefix + "self_attn.out_proj.weight"]))


def feed_forward_block(h, w, prefix, eps, store=_keep):
    """norm -> w1 (gate), w3 (up) -> swiglu -> w2 (down), added to the stream.

    Reference: ``src/Inference/Inference.jl:360-363`` and ``:843-884``.
    """
    n = store(rmsnorm(h, w[prefix + "ffn_norm.weight"], eps))
    gate = store(linear(n, w[prefix + "feed_forward.w1.weight"]))
    up = store(linear(n, w[prefix + "feed_forward.w3.weight"]))
    a = store(swiglu(gate, up))
    return h + store(linear(a, w[prefix + "feed_forward.w2.weight"]))


# --------------------------------------------------------------------------- model

def read_config(model_dir: str) -> dict:
    """The sizes the plain model needs, from the folder's config.json (same keys as the engine)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        c = json.load(f)
    n = c["num_hidden_layers"]
    if "layer_types" in c:
        kinds = ["attn" if t == "full_attention" else "conv" for t in c["layer_types"]]
    else:
        kinds = ["attn" if i in c["full_attn_idxs"] else "conv" for i in range(n)]
    return {
        "layers": kinds,
        "H": c["hidden_size"],
        "nh": c["num_attention_heads"],
        "nkv": c["num_key_value_heads"],
        "d": c["hidden_size"] // c["num_attention_heads"],
        "V": c["vocab_size"],
        "eps": c.get("norm_eps", 1e-5),
        "theta": c.get("rope_theta", 1e6),
        "tied": c.get("tie_word_embeddings", True),
    }


def read_weights(model_dir: str, dtype=torch.float64) -> dict:
    from safetensors import safe_open

    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name).to(dtype)
    return out


def forward(cfg: dict, w: dict, ids, start_pos: int = 0, store=_keep) -> torch.Tensor:
    """Logits ``(T, V)`` of a whole sequence, positions ``start_pos .. start_pos+T-1``.

    Reference: ``reference_prefill``, ``src/Inference/Inference.jl:179-391`` (embedding,
    blocks, final norm ``embedding_norm``, head; tied head is the embedding table itself,
    ``:368-386``).
    """
    h = embedding(w["model.embed_tokens.weight"], ids)
    positions = [start_pos + t for t in range(len(ids))]
    for i, kind in enumerate(cfg["layers"]):
        prefix = f"model.layers.{i}."
        if kind == "conv":
            h, _ = conv_block(h, w, prefix, cfg["eps"], store=store)
        else:
            h = attention_block(h, w, prefix, cfg, positions, store=store)
        h = feed_forward_block(h, w, prefix, cfg["eps"], store=store)
    n = store(rmsnorm(h, w["model.embedding_norm.weight"], cfg["eps"]))
    head = w["model.embed_tokens.weight"] if cfg["tied"] else w["lm_head.weight"]
    return linear(n, head)


def greedy(cfg: dict, w: dict, prompt, max_new_tokens: int):
    """Greedy continuation by whole re-forwards; ties go to the lowest id
    (``test/test_numeric_failures.jl:1-12``)."""
    ids = list(prompt)
    for _ in range(max_new_tokens):
        row = forward(cfg, w, ids)[-1]
        ids.append(int(torch.argmax(row)))  # torch.argmax returns the first maximum
    return ids


# --------------------------------------------------------------------------- sampling

_M64 = (1 << 64) - 1


def splitmix64_unit(state: int):
    """One splitmix64 step -> ``(new_state, u in [0,1))`` from the top 53 bits.

    Reference: ``src/Inference/sampling.jl:32-39``.
    """
    state = (state + 0x9E3779B97F4A7C15) & _M64
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    z = z ^ (z >> 31)
    return state, float(z >> 11) * 2.0 ** -53


def sample_id(logits, temperature: float, top_p: float, state: int):
    """One draw from ``softmax(logits / temperature)`` cut to the nucleus ``top_p``.

    Weights ``exp((x - max)/T)`` in float64; inverse-CDF walk in id order when
    ``top_p >= 1``, else in descending-weight stable order over the smallest prefix whose
    mass reaches ``top_p * total``.  Reference: ``src/Inference/sampling.jl:43-74`` and the
    full-sort form of the nucleus at ``:128-134``.  Returns ``(id, new_state)``.
    """
    x = [float(v) for v in logits]
    hi = max(x)
    w = [math.exp((v - hi) / temperature) for v in x]
    total = 0.0
    for v in w:
        total += v
    state, u = splitmix64_unit(state)
    n = len(w)
    if top_p >= 1:
        r = u * total
        acc = 0.0
        for i in range(n):
            acc += w[i]
            if r < acc:
                return i, state
        return n - 1, state
    order = sorted(range(n), key=lambda i: -w[i])  # stable: ties keep id order
    target = top_p * total
    acc, keep = 0.0, n
    for j, i in enumerate(order):
        acc += w[i]
        if acc >= target:
            keep = j + 1
            break
    cut = 0.0
    for i in order[:keep]:
        cut += w[i]
    r = u * cut
    acc = 0.0
    for i in order[:keep]:
        acc += w[i]
        if r < acc:
            return i, state
    return order[keep - 1], state
