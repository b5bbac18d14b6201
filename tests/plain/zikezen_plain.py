"""A plain, slow Zikezen decoder: whole sequences, no cache, one function per mechanism.

This module is the oracle the engine's Zikezen model is compared with.  It shares no code with the
product package: it does not import it, keeps no pages or state slots, uses no kernels, and walks
every sequence from its first token.  Everything takes a dict of tensors keyed by checkpoint name and
the plain dict of config.json, so the same functions serve any size.  `dtype` is the working
precision (float64 or float32).

The design in this module's own notation (x: residual stream [T, width]; N_w(x) = x / sqrt(mean(x^2) + eps) * w):

    x0 = s E[tok_t] + P[t]                                   (P: a learned row per position)
    layers run in order, the layers a .. b-1 `times` times over (same weights); before every pass over them
    but the first, x <- x + x0
    per layer:   x <- x + N_norm1b(mixer(N_norm1(x)));   x <- x + N_norm2b(ff(N_norm2(x)))  (if it has a feed-forward);
                 x <- x + N_side.norm(W_proj (gelu_tanh(W_gate x) * Z_i[tok_t]))            (Z_i: layer i's columns
                                                                                            of a second token table)
    logits = c tanh(W_head N_final(x) / c)

The mixer is two mixers on the same input, cl * left + cr * right: left, softmax attention inside a sliding
window with per-head norms of q and k, a rotation of neighbouring pairs with stretched frequencies, and a
denominator that is one larger than the sum of exponentials; right, linear attention whose state decays by
a learned factor per key channel and token.  The feed-forward is dense and gated, or routes every token to
a few small gated experts.
"""

from __future__ import annotations

import math

import torch

# See tests/plain/danonex_plain.py: with STORAGE set, products read and write values rounded to it;
# with JITTER = (generator, size) their sums are moved at random by that relative size first.
STORAGE = None
JITTER = None


def stored(x: torch.Tensor) -> torch.Tensor:
    return x if STORAGE is None else x.to(STORAGE).to(x.dtype)


def product(h: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    y = stored(h) @ weight.T
    if bias is not None:
        y = y + bias
    if JITTER is not None:
        y = y * (1.0 + JITTER[1] * torch.randn(y.shape, generator=JITTER[0], dtype=y.dtype))
    return stored(y)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * sigmoid(z)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# --------------------------------------------------------------------------- embedding


def embed(W: dict, cfg: dict, tokens, dtype) -> torch.Tensor:
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = W["embed"].to(dtype)[ids] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    return x + W["pos"].to(dtype)[: len(ids)]


def layer_order(cfg: dict):
    """[(layer index, does the embedding's output join the stream before it?)] for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(a)]
    for turn in range(times):
        order += [(i, turn > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


# --------------------------------------------------------------------------- the left mixer


def stretched_frequencies(rot: dict) -> torch.Tensor:
    """Frequency of each rotated pair, float64: base^(-2i/dims), divided by `factor` where the wavelength exceeds
    original / low, kept where it is below original / high, and blended linearly in original / wavelength between."""
    dims = int(rot["dims"])
    f = float(rot["base"]) ** (-torch.arange(0, dims, 2, dtype=torch.float64) / dims)
    scaling = rot.get("scaling")
    if not scaling:
        return f
    factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
    original = float(scaling["original"])
    out = f.clone()
    for i in range(f.numel()):
        wavelength = 2.0 * math.pi / float(f[i])
        if wavelength > original / low:
            out[i] = f[i] / factor
        elif wavelength >= original / high:
            share = (original / wavelength - low) / (high - low)
            out[i] = (1.0 - share) * f[i] / factor + share * f[i]
    return out


def rotate_pairs(x: torch.Tensor, freq: torch.Tensor, angle_dtype=None) -> torch.Tensor:
    """x [T, heads, dim]: features (2i, 2i + 1), i < len(freq), of the token at place t turn by t * freq_i."""
    T, dims = x.shape[0], 2 * freq.numel()
    if angle_dtype is not None:  # the angle as a product of two numbers of that type
        angle = (torch.arange(T, dtype=angle_dtype)[:, None] * freq.to(angle_dtype)[None, :]).to(torch.float64)
    else:
        angle = torch.arange(T, dtype=torch.float64)[:, None] * freq[None, :]
    c, s = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def window_softmax_one_more(q, k, v, scale: float, window) -> torch.Tensor:
    """q [T, D], k [T, D], v [T, V] of one head pair, key by key: the query at i sees the keys j with
    0 <= i - j < window (all j <= i without a window); weights exp(s_j) / (1 + sum_j exp(s_j))."""
    T = q.shape[0]
    out = torch.zeros((T, v.shape[1]), dtype=q.dtype)
    for i in range(T):
        first = 0 if not window else max(0, i - int(window) + 1)
        s = (k[first:i + 1] @ q[i]) * scale
        m = torch.clamp(s.max(), min=0.0)
        e = torch.exp(s - m)
        out[i] = (e[:, None] * v[first:i + 1]).sum(0) / (torch.exp(-m) + e.sum())
    return out


def left_mixer(W: dict, prefix: str, m: dict, h: torch.Tensor, eps: float, dtype, angle_dtype=None) -> torch.Tensor:
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    w = lambda name: W[prefix + name].to(dtype)
    q = product(h, w("q"), w("q.b")).view(T, H, D)
    k = product(h, w("k"), w("k.b")).view(T, G, D)
    v = product(h, w("v"), w("v.b")).view(T, G, V)
    q, k = rms_norm(q, w("q.norm"), eps), rms_norm(k, w("k.norm"), eps)
    rot = m.get("rot")
    if rot and int(rot.get("dims", 0)):
        freq = stretched_frequencies(rot)
        q, k = rotate_pairs(q, freq, angle_dtype), rotate_pairs(k, freq, angle_dtype)
    q, k = stored(q), stored(k)
    window = (m.get("mask") or {}).get("size")
    heads = [window_softmax_one_more(q[:, j], k[:, j // (H // G)], v[:, j // (H // G)], float(m["scale"]), window)
             for j in range(H)]
    return product(stored(torch.cat(heads, dim=-1)), w("o"))


# --------------------------------------------------------------------------- the right mixer


def channel_decays(W: dict, prefix: str, m: dict, h: torch.Tensor, dtype) -> torch.Tensor:
    """[T, heads, dim]: sigmoid(z)^(1 / tau), z through two narrow products and a bias."""
    z = product(product(h, W[prefix + "a1"].to(dtype)), W[prefix + "a2"].to(dtype)) + W[prefix + "a2.b"].to(dtype)
    return torch.exp(torch.log(sigmoid(z)) / float(m["tau"])).view(h.shape[0], int(m["heads"]), int(m["dim"]))


def decaying_state_readout(q, k, v, decay) -> torch.Tensor:
    """One head, token by token from an empty state S [D, V]: S <- decay_t (row by row) * S + k_t v_t^T; o_t = S^T q_t."""
    T, D = q.shape
    S = torch.zeros((D, v.shape[1]), dtype=q.dtype)
    out = torch.zeros((T, v.shape[1]), dtype=q.dtype)
    for t in range(T):
        S = decay[t][:, None] * S + k[t][:, None] * v[t][None, :]
        out[t] = S.T @ q[t]
    return out


def right_mixer(W: dict, prefix: str, m: dict, h: torch.Tensor, eps: float, dtype) -> torch.Tensor:
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    w = lambda name: W[prefix + name].to(dtype)
    q = product(h, w("q")).view(T, H, D) * D ** -0.5
    k = product(h, w("k")).view(T, H, D)
    v = product(h, w("v")).view(T, H, V)
    decay = channel_decays(W, prefix, m, h, dtype)
    o = torch.stack([decaying_state_readout(q[:, j], k[:, j], v[:, j], decay[:, j]) for j in range(H)], dim=1)
    o = rms_norm(o, w("norm"), eps).reshape(T, H * V) * silu(product(h, w("g")))
    return product(stored(o), w("o"))


def mixer(W: dict, prefix: str, m: dict, h: torch.Tensor, eps: float, dtype, angle_dtype=None) -> torch.Tensor:
    return (float(m["left_scale"]) * left_mixer(W, prefix + "left.", m["left"], h, eps, dtype, angle_dtype)
            + float(m["right_scale"]) * right_mixer(W, prefix + "right.", m["right"], h, eps, dtype))


# --------------------------------------------------------------------------- feed-forwards


def gated(W: dict, prefix: str, h: torch.Tensor, dtype) -> torch.Tensor:
    act = stored(silu(product(h, W[prefix + "gate"].to(dtype))) * product(h, W[prefix + "up"].to(dtype)))
    return product(act, W[prefix + "down"].to(dtype))


def route(W: dict, prefix: str, mlp: dict, h: torch.Tensor, dtype, margins=None):
    """(experts [T, top], their weights [T, top]): scores are the softmax of the router's logits over all experts;
    the `top` largest of score + correction are chosen (the lower index wins a tie); the weights are the scores
    themselves.  `margins`, a list, receives the gap between the last chosen and the first dropped, per token."""
    top = int(mlp["router"]["top"])
    s = torch.softmax(stored(h) @ W[prefix + "router"].to(dtype).T, dim=-1)
    ranked = (s + W[prefix + "correction"].to(dtype)).sort(dim=-1, descending=True, stable=True)
    chosen = ranked.indices[:, :top]
    if margins is not None and top < s.shape[1]:
        margins.append(ranked.values[:, top - 1] - ranked.values[:, top])
    return chosen, s.gather(1, chosen)


def mixture(W: dict, prefix: str, mlp: dict, h: torch.Tensor, dtype, margins=None, forced=None) -> torch.Tensor:
    """`forced` [T, top]: experts to use instead of the ones `route` chooses (weighted by this function's own
    scores), for comparing with an implementation in reduced precision whose close calls may fall the other way."""
    chosen, weights = route(W, prefix, mlp, h, dtype, margins)
    if forced is not None:
        chosen = torch.as_tensor(forced, dtype=torch.long)
        weights = torch.softmax(stored(h) @ W[prefix + "router"].to(dtype).T, dim=-1).gather(1, chosen)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, weight in zip(chosen[t].tolist(), weights[t]):
            out[t] = out[t] + weight * gated(W, f"{prefix}e{e}.", h[t:t + 1], dtype)[0]
    return out


def feed_forward(W: dict, prefix: str, mlp: dict, h: torch.Tensor, dtype, margins=None, forced=None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return gated(W, prefix, h, dtype)
    if mlp["kind"] == "moe":
        return mixture(W, prefix, mlp, h, dtype, margins, forced)
    raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")


# --------------------------------------------------------------------------- the token's own input to a layer


def token_side(W: dict, cfg: dict, index: int, x: torch.Tensor, tokens, eps: float, dtype) -> torch.Tensor:
    """What layer `index` adds from the second token table: its columns [index * dim, (index + 1) * dim)."""
    dim = int(cfg["token_side"]["dim"])
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    rows = W["side.embed"].to(dtype)[ids, index * dim:(index + 1) * dim]
    at = f"l{index}.side."
    g = stored(gelu_tanh(product(x, W[at + "gate"].to(dtype))) * rows)
    return rms_norm(product(g, W[at + "proj"].to(dtype)), W[at + "norm"].to(dtype), eps)


# --------------------------------------------------------------------------- the model


def forward(W: dict, cfg: dict, tokens, dtype=torch.float64, taps=None, margins=None, routing=None,
            angle_dtype=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `taps`, a list, receives the stream after every layer run; `margins`,
    a list, every routed feed-forward's margins [T]; `routing` {layer run: experts [T, top]} forces those runs' choices."""
    eps = float(cfg["norm"]["eps"])
    x0 = embed(W, cfg, tokens, dtype)
    x = x0.clone()
    for run, (i, joins) in enumerate(layer_order(cfg)):
        layer, at = cfg["layers"][i], f"l{i}."
        if layer["type"] != "parallel":
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if joins:
            x = x + x0
        h = rms_norm(x, W[at + "norm1"].to(dtype), eps)
        x = x + rms_norm(mixer(W, at + "mix.", layer["mixer"], h, eps, dtype, angle_dtype), W[at + "norm1b"].to(dtype), eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, W[at + "norm2"].to(dtype), eps)
            y = feed_forward(W, at + "mlp.", layer["mlp"], h, dtype, margins, None if routing is None else routing.get(run))
            x = x + rms_norm(y, W[at + "norm2b"].to(dtype), eps)
        if cfg.get("token_side"):
            x = x + token_side(W, cfg, i, x, tokens, eps, dtype)
        if taps is not None:
            taps.append(x.clone())
    logits = product(rms_norm(x, W["final.norm"].to(dtype), eps), W["head"].to(dtype))
    cap = cfg.get("logit_softcap")
    return float(cap) * torch.tanh(logits / float(cap)) if cap else logits


def greedy_generate(W: dict, cfg: dict, prompt, count: int, dtype=torch.float64):
    """(the `count` tokens that follow `prompt` greedily, the logits each was chosen from [count, vocab])."""
    tokens, rows = list(prompt), []
    for _ in range(count):
        rows.append(forward(W, cfg, tokens, dtype)[-1])
        tokens.append(int(rows[-1].argmax()))
    return tokens[len(prompt):], torch.stack(rows)
