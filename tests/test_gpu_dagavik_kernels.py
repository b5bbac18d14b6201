"""Each Dagavik mechanism's kernels alone against the plain function of that mechanism
(tests/plain/dagavik_plain.py), at sizes of their own, with inputs made so that a fault shows: one
key scaled to stand out just inside and just outside a window, far back among hundreds, on both sides of
a page border; a sink that takes most of a softmax; gates at their caps; experts with hundreds of tokens
and with none."""

import math

import pytest
import torch

from tests.plain import dagavik_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def K():
    from paged_attention_engine_amd.kernels import lib
    return lib


def runs_of(lengths, pasts):
    rows, start = [], 0
    for n, past in zip(lengths, pasts):
        rows += [start, n, past, 0]
        start += n
    return torch.tensor(rows, dtype=torch.int32, device=DEV).view(-1, 4)


def close(got, want, rel, what):
    got, want = got.double().cpu(), want.double().cpu()
    worst, top = float((got - want).abs().max()), float(want.abs().max())
    assert worst <= rel * top, f"{what}: {worst:.3e} > {rel:.1e} * {top:.3e}"


# ----------------------------------------------------------------------------- embedding


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pair_embedding_over_steps_and_slots(dtype):
    """Three sequences in steps of unequal portions: the pair row of a step's first token comes from the slot's last
    token, a sequence's first token takes the last row, and a slot that is taken again starts anew."""
    gen = torch.Generator().manual_seed(3)
    vocab, H, buckets = 50, 24, 13
    table = torch.randn((vocab, H), generator=gen).to(dtype)
    pairs = torch.randn((buckets + 1, H), generator=gen).to(dtype)
    seqs = [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in (9, 1, 6)]
    cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": 100003, "mul_cur": 7}}}
    want = [plain.embed({"embed": table, "bigram": pairs}, cfg, s, torch.float64) for s in seqs]
    last = torch.full((4,), 12345, dtype=torch.int32, device=DEV)  # what another request left behind: never read at position 0
    slots = torch.tensor([2, 0, 3], dtype=torch.int32, device=DEV)
    got = [[] for _ in seqs]
    at = [0, 0, 0]
    for cut in ((4, 1, 2), (1, 0, 1), (4, 0, 3)):
        ids, pos, tok_seq, live = [], [], [], []
        for s, n in enumerate(cut):
            if n:
                live.append((s, len(ids), n))
                ids += seqs[s][at[s]:at[s] + n]
                pos += range(at[s], at[s] + n)
                tok_seq += [s] * n
                at[s] += n
        out = torch.empty((len(ids), H), dtype=torch.float32, device=DEV)
        t = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        K().embedding_pairs(out, table.to(DEV), pairs.to(DEV), t(ids), t(pos), t(tok_seq), slots, last, 1.0, buckets, 100003, 7)
        for s, first, n in live:
            got[s].append(out[first:first + n].cpu())
    for s in range(3):
        close(torch.cat(got[s]), want[s], 1e-6, f"sequence {s}")
    assert last.cpu().tolist()[2] == seqs[0][-1] and last.cpu().tolist()[3] == seqs[2][-1]


# ----------------------------------------------------------------------------- two norms of one stream


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [48, 100, 1536])
def test_terms_join_the_stream_and_both_norms_read_it(dtype, H):
    gen = torch.Generator().manual_seed(H)
    T = 7
    x = torch.randn((T, H), generator=gen)
    a = torch.randn((T, H), generator=gen).to(dtype)
    b = torch.randn((3, T, H), generator=gen)
    w1, w2 = torch.randn(H, generator=gen) * 0.2, torch.randn(H, generator=gen) * 0.2
    new = x.double() + 0.6 * a.double() + 0.9 * b.double().sum(0)
    residual = x.to(DEV)
    out1, out2 = (torch.empty((T, H), dtype=dtype, device=DEV) for _ in range(2))
    K().sum_norm2(residual, [(a.to(DEV), 0.6), (b.to(DEV), 0.9)], (1 + w1).to(DEV), (1 + w2).to(DEV), 1e-5, out1, out2)
    rel = 1e-5 if dtype == torch.float32 else 1e-2
    close(residual, new, 1e-6, "the new stream")
    close(out1, plain.offset_norm(new, w1.double(), 1e-5), rel, "first norm")
    close(out2, plain.offset_norm(new, w2.double(), 1e-5), rel, "second norm")
    # some rows only: nothing is written back, and the terms still count
    rows = torch.tensor([5, 0], dtype=torch.int32, device=DEV)
    residual = x.to(DEV)
    some = torch.empty((2, H), dtype=dtype, device=DEV)
    K().sum_norm2(residual, [(a.to(DEV), 0.6), (b.to(DEV), 0.9)], (1 + w1).to(DEV), None, 1e-5, some, None, rows)
    assert torch.equal(residual.cpu(), x)
    close(some, plain.offset_norm(new, w1.double(), 1e-5)[[5, 0]], rel, "gathered rows")


# ----------------------------------------------------------------------------- matrix memory


def memory_inputs(gen, T, H, D, V, dtype, cap):
    proj = (torch.randn((T, 2 * H * D + 2 * H * V), generator=gen) * 0.7).to(dtype)
    logits = torch.randn((T, 2 * H), generator=gen) * 3.0
    logits[T // 3] = 40.0 * cap        # both gates far beyond the cap
    logits[T // 2, :H] = -40.0 * cap   # an input gate at the cap's other end
    norm = 1.0 + 0.2 * torch.randn(H * V, generator=gen)
    return proj, logits, norm


def memory_plain(proj, logits, norm, H, D, V, cap, eps):
    T = proj.shape[0]
    p = proj.double()
    q = p[:, :H * D].view(T, H, D) * D ** -0.5
    k = p[:, H * D:2 * H * D].view(T, H, D)
    v = p[:, 2 * H * D:2 * H * D + H * V].view(T, H, V)
    gate = p[:, 2 * H * D + H * V:]
    z = logits.double()
    o = plain.matrix_memory_recurrence(q, k, v, plain.soft_cap(z[:, :H], cap), plain.log_sigmoid(plain.soft_cap(z[:, H:], cap)))
    return plain.rms(o, eps).reshape(T, H * V) * norm.double() * plain.sigmoid(gate)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 16, 24), (3, 48, 7), (1, 72, 40), (2, 130, 33)])
def test_matrix_memory_whole_and_in_steps_in_used_slots(dtype, shape):
    H, D, V = shape
    cap, eps, T = 6.0, 1e-5, 150
    gen = torch.Generator().manual_seed(D)
    proj, logits, norm = memory_inputs(gen, T, H, D, V, dtype, cap)
    want = memory_plain(proj, logits, norm, H, D, V, cap, eps)
    rel = 2e-5 if dtype == torch.float32 else 1e-2
    for cuts in ((T,), (1,), (7, 2, 5, 3, 2, 11, 64, 1, 70)):
        state = torch.randn((3, H, V + 1, D), device=DEV)  # what other requests left in the slots
        top = torch.randn((3, H), device=DEV)
        state[1].zero_()
        top[1].zero_()  # the slot is zeroed when it is taken
        slots = torch.tensor([1], dtype=torch.int32, device=DEV)
        rows, p, i = [], 0, 0
        while p < T:
            n = min(cuts[i % len(cuts)], T - p)
            i += 1
            out = torch.empty((n, H * V), dtype=dtype, device=DEV)
            piece = proj[p:p + n].to(DEV)
            K().matrix_memory_step(piece, piece[:, 2 * H * D + H * V:], logits[p:p + n].contiguous().to(DEV), out,
                                   runs_of([n], [p]), slots, state, top, norm.to(DEV), H, D, V, cap, eps, 1e-6)
            rows.append(out)
            p += n
        close(torch.cat(rows), want, rel, f"memory {shape} cut {cuts[:2]}")


def test_matrix_memory_keeps_what_it_was_told_to():
    """A forget gate wide open and one input gate far above the others: the read-out long afterwards is that token's value."""
    H, D, V, T, cap = 1, 32, 16, 300, 20.0
    gen = torch.Generator().manual_seed(1)
    proj = torch.randn((T, 2 * D + 2 * V), generator=gen) * 0.5
    logits = torch.zeros((T, 2))
    logits[:, 0] = -15.0
    logits[:, 1] = 15.0
    logits[40, 0] = 15.0
    proj[-1, :D] = proj[40, D:2 * D] * 4  # the last query asks for token 40's key
    want = memory_plain(proj, logits, torch.ones(V), H, D, V, cap, 1e-6)
    state, top = torch.zeros((1, 1, V + 1, D), device=DEV), torch.zeros((1, 1), device=DEV)
    out = torch.empty((T, V), device=DEV)
    piece = proj.to(DEV)
    K().matrix_memory_step(piece, piece[:, 2 * D + V:], logits.to(DEV), out, runs_of([T], [0]),
                           torch.zeros(1, dtype=torch.int32, device=DEV), state, top, torch.ones(V, device=DEV), H, D, V, cap, 1e-6, 1e-6)
    close(out, want, 2e-5, "recall")
    v40 = proj[40, 2 * D:2 * D + V].double()
    direction = plain.rms(v40[None], 1e-6)[0] * plain.sigmoid(proj[-1, 2 * D + V:].double())
    assert float((out[-1].cpu().double() - direction).abs().max()) < 0.05 * float(direction.abs().max())


# ----------------------------------------------------------------------------- delta rule with channel decays


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 3), (3, 3, 20, 36, 4), (2, 1, 72, 16, 1), (2, 2, 132, 8, 2)])
def test_channel_delta_whole_and_in_steps(dtype, shape):
    H, G, D, V, taps = shape
    T, eps = 120, 1e-5
    gen = torch.Generator().manual_seed(D + taps)
    C = 2 * G * D + H * V
    proj = (torch.randn((T, C), generator=gen) * 0.8).to(dtype)
    gate = torch.randn((T, H * V), generator=gen).to(dtype)
    beta = torch.randn((T, H), generator=gen).to(dtype)
    decay_in = torch.randn((T, H * D), generator=gen).to(dtype)
    conv = torch.randn((C, taps), generator=gen) * 0.5
    a_log, dt_bias = torch.randn(H, generator=gen) * 0.7, torch.randn(H * D, generator=gen)
    norm = 1.0 + 0.2 * torch.randn(V, generator=gen)
    # the plain mechanism from the same rows
    p = proj.double()
    conv_d = conv.double()
    q = plain.causal_conv_silu(p[:, :G * D], conv_d[:G * D]).view(T, G, D)
    k = plain.causal_conv_silu(p[:, G * D:2 * G * D], conv_d[G * D:2 * G * D]).view(T, G, D)
    v = plain.causal_conv_silu(p[:, 2 * G * D:], conv_d[2 * G * D:]).view(T, H, V)
    q, k = plain.unit(q) * D ** -0.5, plain.unit(k)
    decay = torch.exp(-torch.exp(a_log.double())[None, :, None] * plain.softplus(decay_in.double() + dt_bias.double()).view(T, H, D))
    o = plain.channel_delta_recurrence(q, k, v, plain.sigmoid(beta.double()), decay)
    want = (plain.rms(o, eps) * norm.double() * plain.sigmoid(gate.double()).view(T, H, V)).reshape(T, H * V)
    rel = 5e-5 if dtype == torch.float32 else 1.5e-2
    for cuts in ((T,), (1,), (7, 2, 5, 3, 2, 11, 33)):
        tail = torch.randn((2, max(taps - 1, 0), C), device=DEV)
        state = torch.randn((2, H, V, D), device=DEV)
        tail[0].zero_()
        state[0].zero_()
        slots = torch.zeros(1, dtype=torch.int32, device=DEV)
        rows, at, i = [], 0, 0
        while at < T:
            n = min(cuts[i % len(cuts)], T - at)
            i += 1
            out = torch.empty((n, H * V), dtype=dtype, device=DEV)
            seq = torch.zeros(n, dtype=torch.int32, device=DEV)
            pos = torch.arange(at, at + n, dtype=torch.int32, device=DEV)
            K().delta_rule_step(proj[at:at + n].to(DEV), out, seq, pos, runs_of([n], [at]), slots, conv.to(DEV), tail, state,
                                a_log.to(DEV), dt_bias.to(DEV), norm.to(DEV), G, H, D, V, taps, 1e-6, eps,
                                gate=gate[at:at + n].to(DEV), beta=beta[at:at + n].to(DEV), decay_in=decay_in[at:at + n].to(DEV),
                                channel_decay=True, gate_activation="sigmoid")
            rows.append(out)
            at += n
        close(torch.cat(rows), want, rel, f"channel delta {shape} cut {cuts[:2]}")


# ----------------------------------------------------------------------------- latent attention with sinks


def latent_case(gen, T, H, C, dtype, bs, scale, mark=None, sink_scale=1.0):
    """One sequence's folded queries and latent rows in pages handed out in a scrambled order; `mark` = (query, key)
    makes that key stand out for that query."""
    q = torch.randn((T, H, C), generator=gen) * 0.5
    rows = torch.randn((T, C), generator=gen) * 0.5
    if mark is not None:
        i, j = mark
        rows[j] = q[i, 0] * 4.0 / (q[i, 0].norm() ** 2 * scale) * 6.0  # score 24 where the others are of order one
    sinks = torch.randn(H, generator=gen) * sink_scale
    pages = -(-T // bs)
    table = torch.randperm(pages, generator=gen).to(torch.int32)
    pool = torch.zeros((pages + 1, bs, C), dtype=dtype)
    pool_t = torch.zeros((pages + 1, C, bs), dtype=dtype)
    for t in range(T):
        pool[table[t // bs], t % bs] = rows[t].to(dtype)
        pool_t[table[t // bs], :, t % bs] = rows[t].to(dtype)
    return q.to(dtype), rows.to(dtype), sinks, table, pool, pool_t


def latent_plain(q, rows, sinks, scale):
    T, H, C = q.shape
    keys = rows.double()[:, None, :]
    return plain.softmax_attend(q.double(), keys, keys, scale, None, sinks.double()).reshape(T, H * C)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [dict(H=3, C=40, bs=8), dict(H=4, C=64, bs=16), dict(H=12, C=128, bs=16), dict(H=20, C=96, bs=32)])
def test_latent_attention_with_sinks_any_shape_and_on_the_matrix_cores(dtype, case):
    """A prompt of 300 and single tokens at its end: a far key made to stand out for the last query, sinks about a
    unit wide; by the kernel for any shape and, where it takes the shape, by the matrix-core kernel."""
    H, C, bs = case["H"], case["C"], case["bs"]
    T, scale = 300, 0.3
    gen = torch.Generator().manual_seed(C)
    q, rows, sinks, table, pool, pool_t = latent_case(gen, T, H, C, dtype, bs, scale, mark=(T - 1, 5))
    want = latent_plain(q, rows, sinks, scale)
    rel = 2e-5 if dtype == torch.float32 else 2e-2
    dev = lambda t: t.to(DEV)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    tab = dev(table)[None, :].contiguous()
    out = torch.empty((T, H * C), dtype=dtype, device=DEV)
    K().paged_attention_masked(out, dev(q).view(T, H * C), dev(pool), None, pos, seq, tab, H, 1, C, C, scale, 0, False, sinks=dev(sinks))
    close(out, want, rel, f"any shape {case}")
    # the marked key takes nearly all of the last query's first head
    assert float((out[-1, :C].cpu().double() - rows[5].double()).abs().max()) < 0.1 * float(rows[5].abs().max())
    if dtype == torch.bfloat16 and K().latent_attn_supported(dtype, C, C, bs):
        from paged_attention_engine_amd.parts.base import StepShape
        from paged_attention_engine_amd.parts.latent import latent_tiles
        for lens in ((T,), (T - 3, 1, 1, 1), (100, 57, 143)):
            got, past = [], 0
            for n in lens:
                lists = latent_tiles(StepShape((0,), (0,), (n,), (past,), bs), K().latent_attn_tokens(H, 1), K().latent_attn_tokens(H, 2))
                o = torch.zeros((n, H * C), dtype=dtype, device=DEV)
                for name, ct in (("single", 1), ("runs", 2)):
                    flat = lists[name][0]
                    if flat:
                        tiles = torch.tensor(flat, dtype=torch.int32, device=DEV).view(-1, 4)
                        K().latent_attn(o, dev(q[past:past + n]).reshape(n, H * C), dev(pool), dev(pool_t), tiles, ct, pos[past:past + n].contiguous(),
                                        tab, H, C, scale, 0, False, dev(sinks))
                got.append(o)
                past += n
            close(torch.cat(got), want, rel, f"matrix cores {case} {lens}")


def test_a_sink_takes_its_share_of_a_flat_softmax():
    """All scores zero and a sink of ln 3: after n keys the values' mean is scaled by n / (n + 3)."""
    H, C, bs, T = 2, 64, 16, 40
    q = torch.zeros((T, H * C), dtype=torch.bfloat16, device=DEV)
    rows = torch.ones((T, C))
    pool = torch.zeros((4, bs, C), dtype=torch.bfloat16)
    for t in range(T):
        pool[t // bs, t % bs] = rows[t]
    sinks = torch.full((H,), math.log(3.0), device=DEV)
    out = torch.empty((T, H * C), dtype=torch.bfloat16, device=DEV)
    K().paged_attention_masked(out, q, pool.to(DEV), None, torch.arange(T, dtype=torch.int32, device=DEV),
                               torch.zeros(T, dtype=torch.int32, device=DEV), torch.arange(3, dtype=torch.int32, device=DEV)[None, :].contiguous(),
                               H, 1, C, C, 0.5, 0, False, sinks=sinks)
    want = torch.tensor([(t + 1) / (t + 4) for t in range(T)])
    assert float((out[:, 0].float().cpu() - want).abs().max()) < 1e-2


# ----------------------------------------------------------------------------- the window's edges through the mixer's kernels


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [dict(H=4, G=2, D=16, V=24, window=11, bs=8), dict(H=8, G=2, D=64, V=64, window=32, bs=16),
                                  dict(H=2, G=2, D=32, V=32, window=16, bs=16), dict(H=3, G=1, D=48, V=80, window=37, bs=16)])
def test_a_key_just_inside_and_just_outside_the_window(dtype, case):
    """For the last query of a prompt and for a token decoded alone: the key at distance window - 1 made to stand out takes
    the softmax; the key at distance window made to stand out changes nothing."""
    H, G, D, V, W, bs = (case[k] for k in ("H", "G", "D", "V", "window", "bs"))
    T, scale = 3 * W + 5, 0.25
    lib = K()
    mfma = dtype == torch.bfloat16 and V == D and lib.mfma_attention_supported(dtype, H, G, D, bs)
    for distance in (W - 1, W):
        gen = torch.Generator().manual_seed(W + distance)
        q = torch.randn((T, H, D), generator=gen) * 0.5
        k = torch.randn((T, G, D), generator=gen) * 0.5
        v = torch.randn((T, G, V), generator=gen)
        j = T - 1 - distance
        k[j, 0] = q[T - 1, 0] * 30.0 / (q[T - 1, 0].norm() ** 2 * scale)
        want = plain.softmax_attend(q.to(dtype).double(), k.to(dtype).double(), v.to(dtype).double(), scale, W).reshape(T, H * V)
        inside = float((want[-1, :V] - v[j, 0].to(dtype).double()).abs().max()) < 0.05 * float(v[j, 0].abs().max())
        assert inside == (distance == W - 1)
        pages = -(-T // bs)
        table = torch.randperm(pages, generator=gen).to(torch.int32)
        kc = torch.zeros((pages + 1, G, bs, D), dtype=dtype)
        vc = torch.zeros((pages + 1, G, V, bs), dtype=dtype)
        for t in range(T):
            kc[table[t // bs], :, t % bs] = k[t].to(dtype)
            vc[table[t // bs], :, :, t % bs] = v[t].to(dtype)
        pos = torch.arange(T, dtype=torch.int32, device=DEV)
        seq = torch.zeros(T, dtype=torch.int32, device=DEV)
        tab = table.to(DEV)[None, :].contiguous()
        qd = q.to(dtype).to(DEV).view(T, H * D)
        rel = 2e-5 if dtype == torch.float32 else 2e-2
        out = torch.empty((T, H * V), dtype=dtype, device=DEV)
        lib.paged_attention_capped(out, qd, kc.to(DEV), vc.to(DEV), pos, seq, tab, H, G, D, V, scale, W, 0.0, None)
        close(out, want, rel, f"any shape {case} distance {distance}")
        if mfma:
            from paged_attention_engine_amd.parts.attention import attention_work_lists
            from paged_attention_engine_amd.parts.base import StepShape
            for lens in ((T,), (T - 1, 1)):
                got, past = [], 0
                for n in lens:
                    lists = attention_work_lists(StepShape((0,), (0,), (n,), (past,), bs))
                    work = {name: torch.tensor(flat, dtype=torch.int32, device=DEV).view(-1, width) for name, (flat, width) in lists.items()}
                    o = torch.zeros((n, H * V), dtype=dtype, device=DEV)
                    if work["decode_work"].numel():
                        lib.attn_decode(o, qd[past:past + n], kc.to(DEV), vc.to(DEV), work["decode_work"], tab, H, G, D, scale, W)
                    if work["prefill_tiles"].numel():
                        lib.attn_prefill(o, qd[past:past + n], kc.to(DEV), vc.to(DEV), work["prefill_tiles"], pos[past:past + n].contiguous(), tab, H, G, D, scale, W)
                    got.append(o)
                    past += n
                close(torch.cat(got), want, rel, f"matrix cores {case} distance {distance} {lens}")


# ----------------------------------------------------------------------------- routing and experts


@pytest.mark.parametrize("case", [dict(E=12, groups=2, keep=1, top=2), dict(E=9, groups=3, keep=2, top=3), dict(E=5, groups=1, keep=1, top=5),
                                  dict(E=64, groups=8, keep=3, top=6), dict(E=200, groups=4, keep=1, top=1)])
def test_routing_chooses_among_the_best_groups(case):
    gen = torch.Generator().manual_seed(case["E"])
    z = torch.randn((300, case["E"]), generator=gen) * 2.0
    router = {"top": case["top"], "scale": 1.7, "groups": {"count": case["groups"], "keep": case["keep"]}}
    want_chosen, want_weights = plain.route(z.double(), router)
    chosen, weights = K().moe_route(z.to(DEV), case["groups"], case["keep"], case["top"], 1.7)
    assert torch.equal(chosen.cpu().long(), want_chosen)  # in order of falling score
    close(weights, want_weights, 1e-5, "weights")


def test_routing_passes_over_a_better_expert_of_a_dropped_group():
    """Two groups, one kept: the second-best expert overall sits in the losing group and is not chosen."""
    z = torch.tensor([[5.0, 0.0, 1.0, 4.5, 4.4, 0.0]])
    chosen, weights = K().moe_route(z.to(DEV), 2, 1, 2, 1.0)
    assert chosen.cpu().tolist() == [[0, 2]]
    s = torch.softmax(z, -1)[0]
    close(weights, torch.stack([s[0], s[2]])[None], 1e-6, "weights are not renormalised")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [dict(T=5, E=6, top=2, H=64, F=32), dict(T=70, E=4, top=1, H=96, F=64), dict(T=700, E=7, top=3, H=64, F=96),
                                  dict(T=9, E=5, top=2, H=40, F=24), dict(T=1500, E=6, top=3, H=96, F=160),
                                  dict(T=2100, E=3, top=2, H=288, F=64)])
def test_experts_by_pairs_and_by_sorted_tiles(dtype, case):
    """Few tokens (tiles of 16 rows), hundreds (tiles of 64), thousands (tiles of 128 staged through LDS, widths that
    end inside a workgroup's features), experts with many tiles and one with no token at all, and widths the matrix-core
    kernels do not take."""
    T, E, top, H, F = (case[k] for k in ("T", "E", "top", "H", "F"))
    gen = torch.Generator().manual_seed(T)
    x = (torch.randn((T, H), generator=gen)).to(dtype)
    W = {}
    for e in range(E):
        W[f"e{e}.gate"] = (torch.randn((F, H), generator=gen) * 0.2).to(dtype)
        W[f"e{e}.up"] = (torch.randn((F, H), generator=gen) * 0.2).to(dtype)
        W[f"e{e}.down"] = (torch.randn((H, F), generator=gen) * 0.2).to(dtype)
    chosen = torch.stack([torch.randperm(E - 1, generator=gen)[:top] for _ in range(T)])  # the last expert gets no token
    weights = torch.rand((T, top), generator=gen) + 0.5
    want = torch.zeros((T, H), dtype=torch.float64)
    plain.STORAGE = None if dtype == torch.float32 else torch.bfloat16
    try:
        for t in range(T):
            for e, w in zip(chosen[t].tolist(), weights[t].double()):
                want[t] += w * plain.expert(W, f"e{e}.", x[t:t + 1].double(), torch.float64)[0]
    finally:
        plain.STORAGE = None
    stack = lambda name: torch.stack([W[f"e{e}.{name}"] for e in range(E)]).to(DEV)
    got = K().moe_experts(x.to(DEV), stack("gate"), stack("up"), stack("down"), chosen.to(torch.int32).to(DEV), weights.to(DEV))
    tiles = dtype == torch.bfloat16 and H % 32 == 0 and F % 32 == 0
    assert (got.dim() == 3) == tiles
    close(got.sum(0) if got.dim() == 3 else got, want, 1e-5 if dtype == torch.float32 else 1.5e-2, f"experts {case}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_few_features_summed_in_float32(dtype):
    gen = torch.Generator().manual_seed(8)
    a = torch.randn((9, 100), generator=gen).to(dtype)
    w = torch.randn((7, 100), generator=gen).to(dtype)
    bias = torch.randn(7, generator=gen)
    got = K().project_f32(a.to(DEV), w.to(DEV), bias.to(DEV))
    close(got, a.double() @ w.double().T + bias.double(), 1e-5, "float32 sums")
