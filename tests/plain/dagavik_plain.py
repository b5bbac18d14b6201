"""A plain, slow Dagavik decoder: whole sequences, no cache, one function per mechanism.

This module is the oracle the engine's Dagavik model is compared with.  It shares no code with the
product package: it does not import it, keeps no pages or state slots, uses no kernels, and walks
every sequence from its first token.  Everything takes a dict of tensors keyed by checkpoint name and
the plain dict of config.json, so the same functions serve any size.  `dtype` is the working
precision (float64 or float32).

The design in this module's own notation (x: residual stream [T, width]; N_w: RMS norm with an
offset weight, x / sqrt(mean(x^2) + eps) * (1 + w)):

    x <- E[tok_t] + B[hash(tok_(t-1), tok_t)]         (B's last row for a sequence's first token)
    per layer:   x <- x + mixer(N_norm1(x)) + moe(N_norm2(x))     (both branches read the same x)
    logits = W_head N_final(x)

Mixers: "parallel" (windowed softmax attention with a partial half-split rotation beside a matrix
memory with exponential gates, added with two constants), "latent_attention" (all heads' keys and values
from one latent row per token, a sink in the softmax, optionally the latent rows of an earlier layer)
and "channel_delta" (the gated delta rule with a decay per key channel).  The feed-forward routes
every token to a few small gated experts chosen among the best groups of experts.
"""

from __future__ import annotations

import math

import torch

UNIT_EPS = 1e-6        # inside the root when the delta rule's q and k are made unit vectors
READOUT_FLOOR = 1e-6   # added to the matrix memory's denominator

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


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * (1.0 + weight)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


def log_sigmoid(z: torch.Tensor) -> torch.Tensor:
    return -softplus(-z)


# --------------------------------------------------------------------------- embedding


def bigram_rows(tokens, table: dict) -> list:
    """Row of the bigram table for every token of one sequence."""
    buckets, a, b = int(table["buckets"]), int(table["mul_prev"]), int(table["mul_cur"])
    return [buckets if t == 0 else (int(tokens[t - 1]) * a + int(tokens[t]) * b) % buckets for t in range(len(tokens))]


def embed(W: dict, cfg: dict, tokens, dtype) -> torch.Tensor:
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = W["embed"].to(dtype)[ids]
    table = (cfg.get("embedding") or {}).get("bigram")
    if table:
        x = x + W["bigram"].to(dtype)[torch.as_tensor(bigram_rows(tokens, table), dtype=torch.long)]
    return x


# --------------------------------------------------------------------------- windowed attention


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, dim]: feature i < dims/2 of every head turns with feature i + dims/2."""
    if not dims:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def softmax_attend(q, k, v, scale: float, window: int | None, sinks=None) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, V] of one sequence -> [T, H, V], key by key."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[-1]), dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            first = 0 if window is None else max(0, i - window + 1)
            s = (k[first:i + 1, g] @ q[i, h]) * scale
            top = s.max() if sinks is None else torch.maximum(s.max(), sinks[h])
            w = torch.exp(s - top)
            denom = w.sum() + (torch.exp(sinks[h] - top) if sinks is not None else 0.0)
            out[i, h] = (w / denom) @ v[first:i + 1, g]
    return out


def window_attention(W: dict, prefix: str, m: dict, h: torch.Tensor, dtype) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    get = lambda name: W[prefix + name].to(dtype)
    q = product(h, get("q"), get("q.b")).view(T, H, D)
    k = product(h, get("k"), get("k.b")).view(T, G, D)
    v = product(h, get("v"), get("v.b")).view(T, G, V)
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    q = stored(rotate_halves(q, pos, int(rot.get("dims", 0)), float(rot.get("base", 1.0))))
    k = stored(rotate_halves(k, pos, int(rot.get("dims", 0)), float(rot.get("base", 1.0))))
    size = (m.get("mask") or {}).get("size")
    o = softmax_attend(q, k, v, float(m["scale"]), int(size) if size else None)
    return product(o.reshape(T, H * V), get("o"))


# --------------------------------------------------------------------------- matrix memory


def soft_cap(z: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(z / cap)


def matrix_memory_recurrence(q, k, v, log_in, log_keep):
    """q, k [T, H, D], v [T, H, V], log_in and log_keep [T, H] -> read-outs [T, H, V].  The memory C [D, V],
    the key sum n [D] and the running maximum m all start at zero."""
    T, H, D = q.shape
    V = v.shape[-1]
    out = torch.zeros((T, H, V), dtype=q.dtype)
    for h in range(H):
        C = torch.zeros((D, V), dtype=q.dtype)
        n = torch.zeros(D, dtype=q.dtype)
        m = torch.zeros((), dtype=q.dtype)
        for t in range(T):
            m_new = torch.maximum(log_keep[t, h] + m, log_in[t, h])
            keep, take = torch.exp(log_keep[t, h] + m - m_new), torch.exp(log_in[t, h] - m_new)
            C = keep * C + take * torch.outer(k[t, h], v[t, h])
            n = keep * n + take * k[t, h]
            m = m_new
            denom = torch.maximum(torch.abs(n @ q[t, h]), torch.exp(-m)) + READOUT_FLOOR
            out[t, h] = (C.T @ q[t, h]) / denom
    return out


def matrix_memory(W: dict, prefix: str, m: dict, h: torch.Tensor, eps: float, dtype) -> torch.Tensor:
    T = h.shape[0]
    H, D, V, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    get = lambda name: W[prefix + name].to(dtype)
    q = product(h, get("q")).view(T, H, D) * D ** -0.5
    k = product(h, get("k")).view(T, H, D)
    v = product(h, get("v")).view(T, H, V)
    # the gates' logarithms add up over a sequence: their sums do not pass the storage type
    log_in = soft_cap(stored(h) @ get("i").T + get("i.b"), cap)
    log_keep = log_sigmoid(soft_cap(stored(h) @ get("f").T + get("f.b"), cap))
    o = matrix_memory_recurrence(q, k, v, log_in, log_keep)
    o = rms(o, eps).reshape(T, H * V) * get("norm") * sigmoid(product(h, get("g")))
    return product(o, get("o"))


def parallel_mixer(W: dict, prefix: str, m: dict, h: torch.Tensor, eps: float, dtype) -> torch.Tensor:
    left = window_attention(W, prefix + "left.", m["left"], h, dtype)
    right = matrix_memory(W, prefix + "right.", m["right"], h, eps, dtype)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# --------------------------------------------------------------------------- latent attention


def latent_rows(W: dict, prefix: str, h: torch.Tensor, eps: float, dtype) -> torch.Tensor:
    c = product(h, W[prefix + "dkv"].to(dtype))
    return stored(rms(c, eps) * W[prefix + "dkv.norm"].to(dtype))


def latent_attention(W: dict, prefix: str, m: dict, h: torch.Tensor, c: torch.Tensor, dtype) -> torch.Tensor:
    """`c`: the latent rows [T, kv_rank] this layer reads (its own or an earlier layer's)."""
    T = h.shape[0]
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    get = lambda name: W[prefix + name].to(dtype)
    q = product(h, get("q")).view(T, H, D)
    k = product(c, get("uk")).view(T, H, D)
    v = product(c, get("uv")).view(T, H, V)
    o = softmax_attend(q, k, v, float(m["scale"]), None, get("sink"))
    return product(o.reshape(T, H * V), get("o"))


# --------------------------------------------------------------------------- delta rule


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K] (the last column meets the current token), zeros before the start."""
    T, K = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros((K - 1, x.shape[1]), dtype=x.dtype), x], dim=0)
    y = sum(padded[j:j + T] * taps[:, j] for j in range(K))
    return silu(y)


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + UNIT_EPS)


def channel_delta_recurrence(q, k, v, beta, decay):
    """q, k [T, G, D], v [T, H, V], beta [T, H], decay [T, H, D] -> [T, H, V]; head h reads q/k head h // (H / G)."""
    T, G, D = q.shape
    H, V = v.shape[1], v.shape[2]
    out = torch.zeros((T, H, V), dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros((D, V), dtype=q.dtype)
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, h] = S.T @ q[t, g]
    return out


def channel_delta(W: dict, prefix: str, m: dict, h: torch.Tensor, eps: float, dtype) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    get = lambda name: W[prefix + name].to(dtype)
    q = causal_conv_silu(product(h, get("q")), get("q.conv")).view(T, G, D)
    k = causal_conv_silu(product(h, get("k")), get("k.conv")).view(T, G, D)
    v = causal_conv_silu(product(h, get("v")), get("v.conv")).view(T, H, V)
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = sigmoid(product(h, get("b")))
    rate = torch.exp(get("A_log"))[None, :, None]
    step = softplus(product(product(h, get("a1")), get("a2")) + get("dt_bias")).view(T, H, D)
    decay = torch.exp(-rate * step)
    o = channel_delta_recurrence(q, k, v, beta, decay)
    gate = sigmoid(product(product(h, get("g1")), get("g2"))).view(T, H, V)
    o = rms(o, eps) * get("norm") * gate
    return product(o.reshape(T, H * V), get("o"))


# --------------------------------------------------------------------------- feed-forward


def route(z: torch.Tensor, router: dict, margins=None):
    """z [T, E] router logits -> (chosen experts [T, top], their weights [T, top]).  `margins`, a list,
    receives [T]: how far, in units of the logits, each token's choice is from another one (the
    smaller of the gaps between the last group kept and the first one dropped, and between the last
    expert chosen and the first one passed over)."""
    E, top = z.shape[1], int(router["top"])
    groups = router.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(groups["count"]), int(groups["keep"])
    s = torch.softmax(z, dim=-1)
    best = s.view(-1, count, E // count).max(dim=-1).values
    kept = best.topk(keep, dim=-1).indices
    allowed = torch.zeros((z.shape[0], count), dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed.repeat_interleave(E // count, dim=1), s, torch.full_like(s, -1.0))
    chosen = masked.topk(top, dim=-1).indices
    if margins is not None:
        gap = torch.full((z.shape[0],), float("inf"), dtype=z.dtype)
        if keep < count:
            ranked = torch.log(best).sort(dim=-1, descending=True).values
            gap = ranked[:, keep - 1] - ranked[:, keep]
        if top < keep * (E // count):
            ranked = torch.log(masked.clamp_min(1e-300)).sort(dim=-1, descending=True).values
            gap = torch.minimum(gap, ranked[:, top - 1] - ranked[:, top])
        margins.append(gap)
    return chosen, s.gather(1, chosen) * float(router["scale"])


def expert(W: dict, prefix: str, h: torch.Tensor, dtype) -> torch.Tensor:
    act = stored(silu(product(h, W[prefix + "gate"].to(dtype))) * product(h, W[prefix + "up"].to(dtype)))
    return product(act, W[prefix + "down"].to(dtype))


def mixture(W: dict, prefix: str, mlp: dict, h: torch.Tensor, dtype, margins=None, forced=None) -> torch.Tensor:
    """`forced` [T, top]: experts to use instead of the ones `route` chooses (their weights are still this
    function's own scores), for comparing with an implementation in reduced precision, where a choice
    between two nearly equal scores may fall the other way."""
    z = stored(h) @ W[prefix + "router"].to(dtype).T
    chosen, weights = route(z, mlp["router"], margins)
    if forced is not None:
        chosen = torch.as_tensor(forced, dtype=torch.long)
        weights = torch.softmax(z, dim=-1).gather(1, chosen) * float(mlp["router"]["scale"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            out[t] = out[t] + w * expert(W, f"{prefix}e{e}.", h[t:t + 1], dtype)[0]
    return out


# --------------------------------------------------------------------------- the model


def forward(W: dict, cfg: dict, tokens, dtype=torch.float64, taps=None, margins=None, routing=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `taps`, a list, receives the stream after every layer;
    `margins`, a list, every feed-forward's routing margins [T] (see `route`); `routing` {layer: experts
    [T, top]} forces those layers' choices (see `mixture`)."""
    eps = float(cfg["norm"]["eps"])
    x = embed(W, cfg, tokens, dtype)
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        at, m = f"l{i}.", layer["mixer"]
        h = offset_norm(x, W[at + "norm1"].to(dtype), eps)
        if layer["type"] == "parallel":
            y = parallel_mixer(W, at + "mix.", m, h, eps, dtype)
        elif layer["type"] == "latent_attention":
            source = m.get("kv_from")
            if source is None:
                latents[i] = latent_rows(W, at + "mix.", h, eps, dtype)
            y = latent_attention(W, at + "mix.", m, h, latents[i if source is None else int(source)], dtype)
        elif layer["type"] == "channel_delta":
            y = channel_delta(W, at + "mix.", m, h, eps, dtype)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            y = y + mixture(W, at + "mlp.", layer["mlp"], offset_norm(x, W[at + "norm2"].to(dtype), eps), dtype, margins,
                            None if routing is None else routing.get(i))
        x = x + y
        if taps is not None:
            taps.append(x.clone())
    return product(offset_norm(x, W["final.norm"].to(dtype), eps), W["head"].to(dtype))


def greedy_generate(W: dict, cfg: dict, prompt, count: int, dtype=torch.float64):
    """(the `count` tokens that follow `prompt` greedily, the logits each was chosen from [count, vocab])."""
    tokens, rows = list(prompt), []
    for _ in range(count):
        rows.append(forward(W, cfg, tokens, dtype)[-1])
        tokens.append(int(rows[-1].argmax()))
    return tokens[len(prompt):], torch.stack(rows)
