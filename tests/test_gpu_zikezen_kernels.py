"""Each Zikezen mechanism's kernels alone against the plain function of that mechanism
(tests/plain/zikezen_plain.py), at sizes of their own, with inputs made so that a fault shows: one key
scaled to stand out just inside and just outside a window, far back among hundreds, on both sides of a
page border; a softmax whose only other term is the sink; a value written once and read hundreds of tokens
later through decays close to one; a correction that changes which experts are chosen."""

import math

import pytest
import torch

from tests.plain import zikezen_plain as plain

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


# ----------------------------------------------------------------------------- embedding with positions, the token's gate


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_rows_scaled_and_position_rows_as_they_are(dtype):
    gen = torch.Generator().manual_seed(1)
    table = torch.randn((50, 36), generator=gen).to(dtype)
    rows = torch.randn((70, 36), generator=gen).to(dtype)
    ids = torch.randint(0, 50, (23,), generator=gen, dtype=torch.int32)
    positions = torch.tensor([0, 1, 2, 69, 68, 5] + list(range(10, 27)), dtype=torch.int32)
    out = torch.empty((23, 36), dtype=torch.float32, device=DEV)
    K().embedding_positions(out, table.to(DEV), ids.to(DEV), rows.to(DEV), positions.to(DEV), 0.7)
    want = 0.7 * table.double()[ids.long()] + rows.double()[positions.long()]
    close(out, want, 1e-6, "embedding with positions")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim", [8, 24, 40])
def test_the_tokens_columns_gate_a_narrow_product(dtype, dim):
    gen = torch.Generator().manual_seed(dim)
    wide = (torch.randn((19, dim + 16), generator=gen) * 2.0).to(dtype)
    columns = torch.randn((30, dim), generator=gen).to(dtype)
    ids = torch.randint(0, 30, (19,), generator=gen, dtype=torch.int32)
    gate = wide.to(DEV)[:, 8:8 + dim]  # a view of wider rows
    got = K().token_gate(gate, columns.to(DEV), ids.to(DEV), "gelu_tanh")
    want = plain.gelu_tanh(wide.double()[:, 8:8 + dim]) * columns.double()[ids.long()]
    close(got, want, 1e-6 if dtype == torch.float32 else 5e-3, f"token gate {dim}")


# ----------------------------------------------------------------------------- a sublayer's output joins through its norm


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [48, 90, 1536])
def test_terms_join_through_the_norm_after_and_the_next_reader_gets_its_form(dtype, H):
    """Two terms with factors (one as float32 partial sums), the norm after, the stream; then the norm before the next
    sublayer and the stream itself in the activation type; without a norm after (a plain add); with nothing asked for."""
    lib = K()
    gen = torch.Generator().manual_seed(H)
    T, eps, eps_next = 7, 1e-5, 3e-6
    x = torch.randn((T, H), generator=gen) * 3.0
    a = torch.randn((T, H), generator=gen).to(dtype)
    parts = torch.randn((3, T, H), generator=gen)
    w_out = 1.0 + 0.2 * torch.randn((H,), generator=gen)
    w_next = 1.0 + 0.2 * torch.randn((H,), generator=gen)
    y = 0.7 * a.double() + 1.3 * parts.double().sum(0)
    want_x = x.double() + plain.rms_norm(y, w_out.double(), eps)
    want_normed = plain.rms_norm(want_x, w_next.double(), eps_next)
    rel = 1e-6 if dtype == torch.float32 else 5e-3
    terms = [(a.to(DEV), 0.7), (parts.to(DEV), 1.3)]
    res = x.to(DEV)
    normed = torch.empty((T, H), dtype=dtype, device=DEV)
    rows = torch.empty((T, H), dtype=dtype, device=DEV)
    lib.norm_join(res, terms, w_out.to(DEV), eps, w_next.to(DEV), eps_next, normed, rows)
    close(res, want_x, 1e-6, f"stream {H}")
    close(normed, want_normed, rel, f"next norm {H}")
    close(rows, want_x, rel, f"rows {H}")
    res = x.to(DEV)
    lib.norm_join(res, terms, w_out.to(dtype).to(DEV), eps)  # nothing handed on; the weight in the activation type
    close(res, x.double() + plain.rms_norm(y, w_out.to(dtype).double(), eps), 1e-6, f"stream alone {H}")
    res = x.to(DEV)
    lib.norm_join(res, [(a.to(DEV), 1.0)], None, 0.0, w_next.to(DEV), eps_next, normed)
    close(res, x.double() + a.double(), 1e-6, f"plain add {H}")
    close(normed, plain.rms_norm(x.double() + a.double(), w_next.double(), eps_next), rel, f"norm after a plain add {H}")


# ----------------------------------------------------------------------------- per-head norms, the rotation, the cache write


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [dict(H=4, G=2, D=16, V=24, rot=8, bs=8), dict(H=6, G=2, D=64, V=16, rot=48, bs=16),
                                  dict(H=3, G=3, D=22, V=22, rot=10, bs=16), dict(H=5, G=1, D=18, V=10, rot=0, bs=8),
                                  dict(H=2, G=2, D=32, V=32, rot=32, bs=16)])
def test_every_head_normed_by_itself_then_rotated_and_stored(dtype, case):
    """Query and key heads divided by their own root mean square with one weight for all heads, pairs (2i, 2i + 1) of
    the first `rot` features turned, queries in place, keys and values in pages; positions start anywhere in a page."""
    H, G, D, V, rot, bs = (case[k] for k in ("H", "G", "D", "V", "rot", "bs"))
    lib = K()
    gen = torch.Generator().manual_seed(D + rot)
    T, past, eps = 21, 13, 1e-5
    qkv = (torch.randn((T, (H + G) * D + G * V), generator=gen) * 2.0).to(dtype)
    qw = (1.0 + 0.3 * torch.randn((D,), generator=gen)).to(dtype)
    kw = (1.0 + 0.3 * torch.randn((D,), generator=gen)).to(dtype)
    scaling = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16}
    rot_cfg = {"dims": rot, "base": 300.0, "scaling": scaling}
    x = qkv.double()
    q = plain.rms_norm(x[:, :H * D].view(T, H, D), qw.double(), eps)
    k = plain.rms_norm(x[:, H * D:(H + G) * D].view(T, G, D), kw.double(), eps)
    v = x[:, (H + G) * D:].view(T, G, V)
    positions = torch.arange(past, past + T, dtype=torch.int32)
    cos_sin = None
    if rot:
        freq = plain.stretched_frequencies(rot_cfg)
        # the plain rotation counts positions from 0: rotate a sequence that is `past` tokens longer and cut
        pad = lambda t: torch.cat([torch.zeros((past, *t.shape[1:]), dtype=t.dtype), t])
        q = plain.rotate_pairs(pad(q), freq, torch.float32)[past:]
        k = plain.rotate_pairs(pad(k), freq, torch.float32)[past:]
        from paged_attention_engine_amd.config.model_config import WavelengthRamp
        from paged_attention_engine_amd.parts.rope import ramped_frequencies
        mine, _ = ramped_frequencies(rot, 300.0, WavelengthRamp(factor=4.0, original=16.0, low=1.0, high=4.0))
        cos_sin = lib.rope_table(positions.to(DEV), mine.to(DEV))
    pages = -(-(past + T) // bs)
    table = torch.randperm(pages, generator=gen).to(torch.int32)
    kc = torch.zeros((pages + 1, G, bs, D), dtype=dtype, device=DEV)
    vc = torch.zeros((pages + 1, G, V, bs), dtype=dtype, device=DEV)
    dev = qkv.to(DEV)
    lib.qk_norm_rotate_store(dev, H, G, D, V, qw.to(DEV), kw.to(DEV), eps, rot, True, cos_sin, 1.0, positions.to(DEV),
                             torch.zeros(T, dtype=torch.int32, device=DEV), table.to(DEV)[None, :].contiguous(), bs, kc, vc,
                             per_head=True)
    rel = 2e-6 if dtype == torch.float32 else 8e-3
    close(dev[:, :H * D], q.reshape(T, H * D), rel, f"queries {case}")
    for t in range(T):
        p = past + t
        close(kc[table[p // bs], :, p % bs], k[t], rel, f"key {t} {case}")
        close(vc[table[p // bs], :, :, p % bs], v[t], rel, f"value {t} {case}")


# ----------------------------------------------------------------------------- the window's edges and the sink through the attention kernels


def attend(lib, dtype, q, k, v, H, G, D, V, scale, W, bs, lens, gen, mfma):
    """The step's queries over pages in a shuffled order, the portions `lens` one after the other: [T, H * V]."""
    T = q.shape[0]
    pages = -(-T // bs)
    table = torch.randperm(pages, generator=gen).to(torch.int32)
    kc = torch.zeros((pages + 1, G, bs, D), dtype=dtype)
    vc = torch.zeros((pages + 1, G, V, bs), dtype=dtype)
    for t in range(T):
        kc[table[t // bs], :, t % bs] = k[t].to(dtype)
        vc[table[t // bs], :, :, t % bs] = v[t].to(dtype)
    kc, vc = kc.to(DEV), vc.to(DEV)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    tab = table.to(DEV)[None, :].contiguous()
    qd = q.to(dtype).to(DEV).view(T, H * D)
    sinks = torch.zeros(H, dtype=torch.float32, device=DEV)  # every head's sink has the score 0
    if not mfma:
        out = torch.empty((T, H * V), dtype=dtype, device=DEV)
        lib.paged_attention_capped(out, qd, kc, vc, pos, seq, tab, H, G, D, V, scale, W, 0.0, sinks)
        return out
    from paged_attention_engine_amd.parts.attention import attention_work_lists
    from paged_attention_engine_amd.parts.base import StepShape
    got, past = [], 0
    for n in lens:
        lists = attention_work_lists(StepShape((0,), (0,), (n,), (past,), bs))
        work = {name: torch.tensor(flat, dtype=torch.int32, device=DEV).view(-1, width) for name, (flat, width) in lists.items()}
        o = torch.zeros((n, H * V), dtype=dtype, device=DEV)
        if work["decode_work"].numel():
            lib.attn_decode(o, qd[past:past + n], kc, vc, work["decode_work"], tab, H, G, D, scale, W, 0.0, sinks)
        if work["prefill_tiles"].numel():
            lib.attn_prefill(o, qd[past:past + n], kc, vc, work["prefill_tiles"], pos[past:past + n].contiguous(), tab, H, G, D,
                             scale, W, 0.0, sinks)
        got.append(o)
        past += n
    return torch.cat(got)


def plain_heads(q, k, v, H, G, scale, W, dtype):
    q, k, v = (t.to(dtype).double() for t in (q, k, v))
    return torch.cat([plain.window_softmax_one_more(q[:, j], k[:, j // (H // G)], v[:, j // (H // G)], scale, W)
                      for j in range(H)], dim=-1)


CASES = [dict(H=4, G=2, D=16, V=24, window=11, bs=8), dict(H=8, G=2, D=64, V=64, window=32, bs=16),
         dict(H=2, G=2, D=32, V=32, window=16, bs=16), dict(H=3, G=1, D=48, V=80, window=37, bs=16),
         dict(H=10, G=5, D=64, V=48, window=70, bs=16)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_a_key_just_inside_and_just_outside_the_window(dtype, case):
    """For the last query of a prompt and for a token decoded alone: the key at distance window - 1 made to stand out takes
    the softmax (the sink's one in the denominator is then small beside it); at distance window it changes nothing."""
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
        want = plain_heads(q, k, v, H, G, scale, W, dtype)
        inside = float((want[-1, :V] - v[j, 0].to(dtype).double()).abs().max()) < 0.05 * float(v[j, 0].abs().max())
        assert inside == (distance == W - 1)
        rel = 2e-5 if dtype == torch.float32 else 2e-2
        close(attend(lib, dtype, q, k, v, H, G, D, V, scale, W, bs, (T,), gen, False), want, rel, f"any shape {case} {distance}")
        if mfma:
            for lens in ((T,), (T - 1, 1), (T - W - 2, W + 1, 1)):
                close(attend(lib, dtype, q, k, v, H, G, D, V, scale, W, bs, lens, gen, True), want, rel,
                      f"matrix cores {case} {distance} {lens}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [CASES[0], CASES[1], CASES[3]])
def test_the_sink_takes_its_share(dtype, case):
    """Scores far below zero: the sink's one is nearly the whole denominator and the heads' outputs nearly vanish; scores of
    zero: n keys weigh 1 / (n + 1) each, also for the first tokens of a sequence, whose windows are not yet full."""
    H, G, D, V, W, bs = (case[k] for k in ("H", "G", "D", "V", "window", "bs"))
    lib = K()
    mfma = dtype == torch.bfloat16 and V == D and lib.mfma_attention_supported(dtype, H, G, D, bs)
    gen = torch.Generator().manual_seed(7)
    T, scale = W + 9, 0.5
    v = torch.randn((T, G, V), generator=gen)
    flat_q = torch.zeros((T, H, D))
    k = torch.randn((T, G, D), generator=gen)
    want = plain_heads(flat_q, k, v, H, G, scale, W, dtype)
    for i in (0, 1, W - 1, W, T - 1):
        seen = list(range(max(0, i - W + 1), i + 1))
        mean = v[seen, 0].to(dtype).double().sum(0) / (len(seen) + 1.0)
        assert float((want[i, :V] - mean).abs().max()) < 1e-9
    rel = 2e-5 if dtype == torch.float32 else 2e-2
    for use in ((False, True) if mfma else (False,)):
        close(attend(lib, dtype, flat_q, k, v, H, G, D, V, scale, W, bs, (T - 1, 1), gen, use), want, rel, f"flat scores {case} {use}")
    # every score about -25: exp(-25) against the sink's one
    unit = torch.ones((D,)) / math.sqrt(D)
    q = unit.expand(T, H, D).clone() * 10.0
    k = -unit.expand(T, G, D).clone() * 5.0
    want = plain_heads(q, k, v, H, G, scale, W, dtype)
    assert float(want.abs().max()) < 1e-8 * W
    for use in ((False, True) if mfma else (False,)):
        got = attend(lib, dtype, q, k, v, H, G, D, V, scale, W, bs, (T - 1, 1), gen, use)
        assert float(got.double().abs().max()) < 1e-6, f"scores far below the sink's {case} {use}"


# ----------------------------------------------------------------------------- gated linear attention


def gla_inputs(gen, T, H, D, V, dtype, z_mean=2.0):
    proj = (torch.randn((T, 2 * H * D + 2 * H * V + 8), generator=gen) * 0.7).to(dtype)  # [q | k | v | gate | unused]
    z = (torch.randn((T, H * D), generator=gen) * 1.5 + z_mean).to(dtype)
    bias = torch.randn((H * D,), generator=gen)
    norm = (1.0 + 0.2 * torch.randn((V,), generator=gen)).to(dtype)
    return proj, z, bias, norm


def gla_plain(proj, z, bias, norm, H, D, V, tau, eps):
    T = proj.shape[0]
    x = proj.double()
    q = x[:, :H * D].view(T, H, D) * D ** -0.5
    k = x[:, H * D:2 * H * D].view(T, H, D)
    v = x[:, 2 * H * D:2 * H * D + H * V].view(T, H, V)
    gate = x[:, 2 * H * D + H * V:2 * H * D + 2 * H * V]
    decay = torch.exp(torch.log(plain.sigmoid(z.double() + bias.double())) / tau).view(T, H, D)
    o = torch.stack([plain.decaying_state_readout(q[:, j], k[:, j], v[:, j], decay[:, j]) for j in range(H)], dim=1)
    return plain.rms_norm(o, norm.double(), eps).reshape(T, H * V) * plain.silu(gate)


def gla_step(lib, proj, z, bias, norm, H, D, V, tau, eps, lens, pasts, slots, state, first_row=0):
    n = sum(lens)
    rows = slice(first_row, first_row + n)
    p = proj[rows].to(DEV)
    out = torch.empty((n, H * V), dtype=proj.dtype, device=DEV)
    lib.linear_attention_step(p, z[rows].to(DEV), bias.to(DEV), tau, p[:, 2 * H * D + H * V:2 * H * D + 2 * H * V], out,
                              runs_of(lens, pasts), torch.tensor(slots, dtype=torch.int32, device=DEV), state, norm.to(DEV),
                              H, D, V, eps)
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 16, 24), (3, 8, 40), (4, 48, 32), (1, 24, 16), (2, 72, 16), (1, 128, 32), (2, 130, 6),
                                   (1, 200, 12), (1, 260, 9), (3, 10, 14)])
def test_linear_attention_whole_and_in_steps_in_used_slots(dtype, shape):
    """Every lane grouping of the recurrence (key widths up to 16, 32, 64, 128, 256 and beyond), widths that are no
    multiples of four; a sequence whole, token by token and in portions, beside another sequence, in slots that held
    other state."""
    H, D, V = shape
    lib = K()
    gen = torch.Generator().manual_seed(D * 7 + V)
    T, tau, eps = 45, 4.0, 1e-5
    proj, z, bias, norm = gla_inputs(gen, T, H, D, V, dtype)
    want = gla_plain(proj, z, bias, norm, H, D, V, tau, eps)
    rel = 3e-5 if dtype == torch.float32 else 1.5e-2
    state = torch.randn((4, H, V, D), device=DEV)  # what other requests left
    state[1].zero_()  # a slot is zeroed when a request takes it
    got = gla_step(lib, proj, z, bias, norm, H, D, V, tau, eps, (T,), (0,), [1], state)
    close(got, want, rel, f"whole {shape}")
    whole_state = state[1].clone()
    for cuts in ((1,) * T, (7, 2, 5, 1, 1, 13, 2, 14)):
        state[2].zero_()
        parts, at = [], 0
        for n in cuts:
            parts.append(gla_step(lib, proj, z, bias, norm, H, D, V, tau, eps, (n,), (at,), [2], state, first_row=at))
            at += n
        close(torch.cat(parts), want, rel, f"steps {cuts[:3]} {shape}")
        close(state[2], whole_state, 3e-5, f"state after steps {shape}")
    # two sequences in one step: the second is the same tokens from another start, and the slots are not in order
    state[3].zero_()
    state[0].zero_()
    both = torch.cat([proj[:20], proj[:T]]), torch.cat([z[:20], z[:T]])
    got = gla_step(lib, both[0], both[1], bias, norm, H, D, V, tau, eps, (20, T), (0, 0), [3, 0], state)
    close(got[20:], want, rel, f"beside another {shape}")
    close(got[:20], want[:20], rel, f"the other {shape}")


def test_linear_attention_keeps_what_it_was_told_to():
    """A value written once is read back 400 tokens later through decays close to one (a large temperature), and is gone
    when the decays are small (a temperature of one and inputs below zero)."""
    lib = K()
    H, D, V, T, eps = 1, 32, 16, 420, 1e-6
    gen = torch.Generator().manual_seed(3)
    key = torch.randn((D,), generator=gen)
    key = key / key.norm()
    for tau, z_mean, kept in ((4000.0, 3.0, True), (1.0, -2.0, False)):
        proj = torch.zeros((T, 2 * H * D + 2 * H * V))
        proj[:, 2 * H * D + H * V:] = 5.0                      # the gate wide open
        proj[10, H * D:2 * H * D] = key * 4.0                   # written at token 10 ...
        value = torch.randn((V,), generator=gen)
        proj[10, 2 * H * D:2 * H * D + V] = value
        proj[T - 1, :H * D] = key * 4.0                         # ... and asked for by the last token
        z = torch.full((T, H * D), z_mean)
        bias, norm = torch.zeros((H * D,)), torch.ones((V,))
        want = gla_plain(proj, z, bias, norm, H, D, V, tau, eps)
        state = torch.zeros((1, H, V, D), device=DEV)
        got = gla_step(lib, proj, z, bias, norm, H, D, V, tau, eps, (300,), (0,), [0], state)
        got = torch.cat([got, gla_step(lib, proj, z, bias, norm, H, D, V, tau, eps, (T - 300,), (300,), [0], state, first_row=300)])
        close(got, want, 1e-4, f"recall tau {tau}")
        direction = float(torch.nn.functional.cosine_similarity(got[-1].double().cpu(), value.double(), dim=0))
        if kept:
            assert direction > 0.999 and float(got[-1].abs().max()) > 0.5
        else:
            assert float(state.abs().max()) < 1e-30


# ----------------------------------------------------------------------------- routing with a correction


@pytest.mark.parametrize("case", [dict(E=16, top=3), dict(E=6, top=2), dict(E=5, top=5), dict(E=70, top=4), dict(E=4, top=1)])
def test_routing_chooses_by_score_plus_correction_and_weighs_by_score(case):
    E, top = case["E"], case["top"]
    gen = torch.Generator().manual_seed(E)
    T = 200
    logits = torch.randn((T, E), generator=gen) * 1.5
    correction = torch.randn((E,), generator=gen) * 0.2
    W = {"r.router": torch.eye(E, dtype=torch.float64), "r.correction": correction.double()}
    margins = []
    want_chosen, want_weights = plain.route(W, "r.", {"router": {"experts": E, "top": top}}, logits.double(), torch.float64, margins)
    chosen, weights = K().moe_route(logits.to(DEV), 1, 1, top, 1.0, correction.to(DEV))
    clear = margins[0] > 1e-5 if margins else torch.ones(T, dtype=torch.bool)
    assert clear.float().mean() > 0.95
    assert torch.equal(chosen.cpu().long()[clear], want_chosen[clear])
    close(weights.cpu()[clear], want_weights[clear], 1e-5, f"weights {case}")
    if top < E:  # the correction matters: without it other experts are chosen for many tokens
        plainly, _ = K().moe_route(logits.to(DEV), 1, 1, top, 1.0)
        assert (plainly.cpu().long().sort(-1).values != want_chosen.sort(-1).values).any(-1).float().mean() > 0.1
