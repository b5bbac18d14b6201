"""The Zikezen model through the engine's step function, cache and kernels against the plain
implementation (tests/plain/zikezen_plain.py, float64 on the same weights).

Per model and precision one replayer runs the same requests whole, decoded token by token from the
first token on, in portions of several sizes down to two tokens, and mixed: unequal requests side by
side in a pool and in state slots so small that pages and slots are given back and used again.  Every
logit is compared with the plain one.  Greedy generation goes through the engine's own entry point and
scheduler, and through `bin/trace_run` as a program.

Routing is a choice between numbers: where two experts' scores are within a rounding of each other,
reduced precision may choose the other one, and everything after differs.  In float32 the engine must
choose as the plain implementation does.  In bfloat16 the engine's choices are read out (a tap on the
feed-forward, once per run of a layer); the plain implementation is run on those choices, which gives the
logits the engine is compared with and, run by run, what the plain implementation would have chosen itself
on the same stream: wherever its margin is clear, the engine's choice must be that one.
"""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests import zikezen_models as M
from tests.plain import zikezen_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = (150, 37, 90, 1)
PORTIONS = (7, 2, 5, 3, 2, 11, 4, 2, 9, 17, 33)
CLEAR_MARGIN = 0.1    # of a score plus its correction (scores add up to 1): a choice this far from the next falls the same way in bfloat16


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("zikezen")
    return {name: M.make_folder(tmp, name) for name in M.CONFIGS}


_PLAIN, _WEIGHTS = {}, {}


def weights_of(folders, name):
    if name not in _WEIGHTS:
        _WEIGHTS[name] = M.read_folder(folders[name])
    return _WEIGHTS[name]


def plain_logits(folders, name, length):
    key = (name, length)
    if key not in _PLAIN:
        cfg, weights = weights_of(folders, name)
        _PLAIN[key] = plain.forward(weights, cfg, M.tokens_for(name, length), torch.float64, angle_dtype=torch.float32)
    return _PLAIN[key]


def routed_runs(cfg):
    """Indices of the layer runs that route (a layer that runs twice routes twice, on different streams)."""
    return [run for run, (i, _) in enumerate(plain.layer_order(cfg)) if (cfg["layers"][i].get("mlp") or {}).get("kind") == "moe"]


def rounding_alone(folders, name, tokens, want, routing):
    """(largest, root-mean-square) error of the plain implementation when its products' operands and
    results are rounded to bfloat16 and nothing else changes (the routing held fixed)."""
    cfg, weights = weights_of(folders, name)
    worst = rms = 0.0
    plain.STORAGE = torch.bfloat16
    try:
        for trial in range(3):  # the products' sums as they are, and in two other orders of adding
            plain.JITTER = (torch.Generator().manual_seed(trial), 3e-4) if trial else None
            diff = plain.forward(weights, cfg, tokens, torch.float64, routing=routing, angle_dtype=torch.float32) - want
            worst, rms = max(worst, float(diff.abs().max())), max(rms, float(diff.pow(2).mean().sqrt()))
    finally:
        plain.STORAGE = plain.JITTER = None
    return worst, rms


def check(got, want, dtype, what, rounding=None):
    """float32: a few hundred roundings relative to the largest logit.  bfloat16: the engine may be off by
    three times what rounding alone does to the plain implementation on the same tokens, plus a unit in
    the last place of the largest logit."""
    got, want = torch.as_tensor(got).double(), torch.as_tensor(want).double()
    top = float(want.abs().max())
    worst = float((got - want).abs().max())
    if dtype == "float32":
        assert worst <= 1e-4 * top, f"{what}: worst logit error {worst:.3e} > {1e-4 * top:.3e}"
        return worst
    bound = 3.0 * rounding[0] + helpers.bf16_ulp(want)
    assert worst <= bound, f"{what}: worst logit error {worst:.3e} > {bound:.3e} (rounding alone {rounding[0]:.3e})"
    return worst


class Replay:
    """A replayer and, in bfloat16, what its feed-forwards chose in every step (read on the host, so
    those steps are launched kernel by kernel)."""

    def __init__(self, folders, name, dtype, max_tokens, max_live=4, block_size=16):
        from paged_attention_engine_amd.engine.step import StepRunner
        from paged_attention_engine_amd.engine.trace import TraceReplayer

        self.name, self.dtype, self.folders = name, dtype, folders
        self.rp = TraceReplayer(folders[name], dtype, max_tokens, block_size, max_live)
        self.cfg = weights_of(folders, name)[0]
        self.runs = routed_runs(self.cfg)
        self.step_choices = []
        if dtype == "bfloat16":
            self.rp.runner = StepRunner(self.rp.model, self.rp.cache, use_graphs=False)
            for block in self.rp.model.blocks:
                if hasattr(block.feed_forward, "routing_tap"):
                    block.feed_forward.routing_tap = lambda chosen, weights: self.step_choices.append(chosen.cpu().long())

    def step(self, record):
        """(logits, {routed run: chosen experts [rows of the step, top]}): the taps fire in the order of the runs"""
        self.step_choices = []
        out = self.rp.step(record)
        return torch.from_numpy(out.copy()), dict(zip(self.runs, self.step_choices))

    def alone(self, rid, tokens, cuts):
        """Feed `tokens` as one request in portions of the sizes `cuts` (cycled): ([T, vocab], routing)."""
        rows, routing, p, i = [], {}, 0, 0
        while p < len(tokens):
            n = min(cuts[i % len(cuts)], len(tokens) - p)
            i += 1
            out, chosen = self.step({"step": 0, "entries": [{"id": rid, "tokens": tokens[p:p + n], "want": list(range(n))}],
                                     "end": [rid] if p + n == len(tokens) else []})
            rows.append(out)
            for run, c in chosen.items():
                routing.setdefault(run, []).append(c)
            p += n
        return torch.cat(rows), {run: torch.cat(parts) for run, parts in routing.items()}

    def compare(self, got, routing, tokens, want, what):
        """`got` against the plain logits: in float32 `want` itself; in bfloat16 the plain logits under the
        engine's own routing, which must be the plain one wherever that is clear."""
        if self.dtype == "float32":
            return check(got, want, "float32", what)
        cfg, weights = weights_of(self.folders, self.name)
        free, own_margins = [], []
        original = plain.route

        def spy(*args, **kwargs):
            chosen, w = original(*args, **kwargs)
            free.append(chosen)
            return chosen, w

        plain.route = spy
        try:
            own = plain.forward(weights, cfg, tokens, torch.float64, margins=own_margins, routing=routing,
                                angle_dtype=torch.float32)
        finally:
            plain.route = original
        margins = iter(own_margins)
        for run, chosen in zip(self.runs, free):
            router = cfg["layers"][plain.layer_order(cfg)[run][0]]["mlp"]["router"]
            if int(router["top"]) == int(router["experts"]):
                continue  # every expert is chosen: there is no margin
            clear = next(margins) >= CLEAR_MARGIN
            assert torch.equal(routing[run][clear].sort(-1).values, chosen[clear].sort(-1).values), \
                f"{what}: run {run} routes a token with a clear margin otherwise than the plain implementation"
        return check(got, own, "bfloat16", what, rounding_alone(self.folders, self.name, tokens, own, routing))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.CONFIGS))
def test_whole_decoded_and_in_portions(folders, name, dtype):
    """A prompt whole, token by token from its first token on (which is prefill against decoding, and a
    long decode), and in portions of changing sizes: all against the plain logits, and in float32 the
    three against each other to a few roundings."""
    replay = Replay(folders, name, dtype, 256)
    for length in LENGTHS[:3]:
        tokens = M.tokens_for(name, length)
        want = plain_logits(folders, name, length)
        whole, routing = replay.alone("w", tokens, (length,))
        replay.compare(whole, routing, tokens, want, f"{name} {dtype} whole {length}")
        single, routing = replay.alone("d", tokens, (1,))
        replay.compare(single, routing, tokens, want, f"{name} {dtype} token by token {length}")
        for first in (0, 4):
            cut, routing = replay.alone("c", tokens, PORTIONS[first:] + PORTIONS[:first])
            replay.compare(cut, routing, tokens, want, f"{name} {dtype} portions {length}")
        cut, routing = replay.alone("c2", tokens, (2,))
        replay.compare(cut, routing, tokens, want, f"{name} {dtype} portions of two {length}")
        if dtype == "float32":
            top = float(want.abs().max())
            assert float((whole - single).abs().max()) <= 2e-5 * top
            assert float((whole - cut).abs().max()) <= 2e-5 * top
    cache = replay.rp.cache
    assert cache.slots.num_free == 4 and all(g.allocator.num_free == g.allocator.num_blocks for g in cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "S"])
def test_the_first_tokens_of_a_sequence(folders, name, dtype):
    """One token to five, each as a request of its own: the first positions' rows, the state's zeros, a window
    that is not yet full, a softmax of one key and the sink."""
    replay = Replay(folders, name, dtype, 64)
    for length in (1, 2, 3, 4, 5):
        cfg, weights = weights_of(folders, name)
        tokens = M.tokens_for(name, length, salt=7)
        want = plain.forward(weights, cfg, tokens, torch.float64, angle_dtype=torch.float32)
        got, routing = replay.alone("f", tokens, (length,))
        replay.compare(got, routing, tokens, want, f"{name} first {length} whole")
        got, routing = replay.alone("g", tokens, (1,))
        replay.compare(got, routing, tokens, want, f"{name} first {length} one by one")


def mixed_schedule(lengths):
    """Steps of (request index, count): requests arrive staggered, run a portion a step and then single
    tokens beside the others' portions; at most four are live; every request runs twice."""
    order = [i for _ in range(2) for i in range(len(lengths))]
    steps, live, arrivals = [], {}, list(enumerate(order))
    tick = 0
    while arrivals or live:
        if arrivals and len(live) < 4 and tick % 2 == 0:
            rid, which = arrivals.pop(0)
            live[rid] = [which, 0]
        step = []
        for rid, (which, at) in list(live.items()):
            remaining = lengths[which] - at
            tail = min(12, lengths[which] // 2)
            n = 1 if remaining <= tail else min(PORTIONS[(tick + rid) % len(PORTIONS)], remaining - tail)
            if (tick + rid) % 5 == 4 and remaining > 1:
                continue  # a request is left out of a step and goes on later
            step.append((rid, which, at, n))
            live[rid][1] = at + n
            if at + n == lengths[which]:
                del live[rid]
        if step:
            steps.append(step)
        tick += 1
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.CONFIGS))
def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(folders, name, dtype):
    lengths = LENGTHS
    tokens = [M.tokens_for(name, n) for n in lengths]
    plains = [plain_logits(folders, name, n) for n in lengths]
    steps = mixed_schedule(lengths)
    # the pool holds what the four longest live requests need and no more, so pages are used again
    replay = Replay(folders, name, dtype, sum(-(-n // 64) * 64 for n in lengths))
    rows_of, routing_of = {}, {}
    for step in steps:
        record = {"step": 0, "entries": [], "end": []}
        for rid, which, at, n in step:
            record["entries"].append({"id": f"r{rid}", "tokens": tokens[which][at:at + n], "want": list(range(n))})
            if at + n == lengths[which]:
                record["end"].append(f"r{rid}")
        out, chosen = replay.step(record)
        row = 0
        for rid, which, at, n in step:
            rows_of.setdefault((rid, which), []).append(out[row:row + n])
            for run, c in chosen.items():
                routing_of.setdefault((rid, which), {}).setdefault(run, []).append(c[row:row + n])
            row += n
    assert len(steps) > 30 and max(len(s) for s in steps) == 4
    for (rid, which), rows in rows_of.items():
        routing = {run: torch.cat(parts) for run, parts in routing_of.get((rid, which), {}).items()}
        replay.compare(torch.cat(rows), routing, tokens[which], plains[which], f"{name} {dtype} request {rid}")
    assert replay.rp.cache.slots.num_free == 4
    if dtype == "float32" and replay.rp.runner.use_graphs:
        assert replay.rp.runner.graph_replays > 0  # steps of single tokens ran as recorded graphs


def test_a_slot_that_held_another_request_starts_from_zero(folders):
    """One state slot: every request takes the slot the one before gave back (every pass's state matrices), and
    must not see any of it."""
    replay = Replay(folders, "P", "float32", 128, max_live=1)
    for length in (37, 90, 37):
        tokens = M.tokens_for("P", length)
        got, routing = replay.alone("s", tokens, (5, 1, 1, 9))
        replay.compare(got, routing, tokens, plain_logits(folders, "P", length), f"P in a used slot, {length}")


def test_the_stream_after_every_layer_run(folders):
    """The float32 stream after each run of a layer against the plain one: a layer that runs twice is seen twice."""
    from paged_attention_engine_amd.engine.step import StepRunner

    for name in ("P", "Q"):
        replay = Replay(folders, name, "float32", 64)
        replay.rp.runner = StepRunner(replay.rp.model, replay.rp.cache, use_graphs=False)
        seen = []
        replay.rp.model.residual_tap = lambda index, stream: seen.append(stream.residual.clone().cpu().double())
        tokens = M.tokens_for(name, 37)
        replay.alone("t", tokens, (37,))
        cfg, weights = weights_of(folders, name)
        taps = []
        plain.forward(weights, cfg, tokens, torch.float64, taps=taps, angle_dtype=torch.float32)
        assert len(seen) == len(taps) == len(plain.layer_order(cfg))
        for i, (got, want) in enumerate(zip(seen, taps)):
            assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max()), f"{name} run {i}"


def test_recorded_steps_give_the_eager_steps_logits(folders):
    """Steps of single tokens replay as HIP graphs; the same steps launched kernel by kernel give the same bits."""
    from paged_attention_engine_amd.engine.step import StepRunner

    tokens = M.tokens_for("P", 60)
    outs = []
    for graphs in (True, False):
        replay = Replay(folders, "P", "float32", 128)
        replay.rp.runner = StepRunner(replay.rp.model, replay.rp.cache, use_graphs=graphs)
        outs.append(replay.alone("a", tokens, (20,) + (1,) * 40)[0])
        if graphs:
            assert replay.rp.runner.graph_replays >= 39
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("name", ["P", "R"])
def test_greedy_generation_through_the_entry_point(folders, name):
    import paged_attention_engine_amd as pae

    cfg, weights = weights_of(folders, name)
    prompt = M.tokens_for(name, 21, salt=3)
    want_tokens, want_logits = plain.greedy_generate(weights, cfg, prompt, 12, torch.float64)
    engine = pae.Engine(folders[name], dtype="float32", block_size=16, num_blocks=8, max_num_seqs=2)
    got = engine.generate(prompt, 12)
    assert list(got.token_ids) == want_tokens
    check(got.step_logits.cpu(), want_logits, "float32", f"{name} generation")
    # bfloat16: the same entry point runs; its tokens agree until two plain logits nearly tie or a routing falls otherwise
    engine = pae.Engine(folders[name], dtype="bfloat16", block_size=16, num_blocks=8, max_num_seqs=2)
    assert len(engine.generate(prompt, 12).token_ids) == 12


def test_requests_through_the_scheduler_with_few_pages(folders):
    """Several requests through the scheduler in a pool that forces waiting and portions; every request's
    tokens are those it generates alone."""
    import paged_attention_engine_amd as pae

    prompts = [M.tokens_for("P", n, salt=9) for n in (33, 5, 70, 18, 41)]
    alone = []
    for prompt in prompts:
        engine = pae.Engine(folders["P"], dtype="float32", block_size=16, num_blocks=16, max_num_seqs=1)
        alone.append(list(engine.generate(prompt, 10).token_ids))
    engine = pae.Engine(folders["P"], dtype="float32", block_size=16, num_blocks=14, max_num_seqs=3,
                        max_num_batched_tokens=24)
    for i, prompt in enumerate(prompts):
        assert engine.add_request(pae.Request(f"r{i}", tuple(prompt), max_new_tokens=10))
    done = engine.run_to_completion()
    assert [list(done[f"r{i}"]) for i in range(len(prompts))] == alone


def test_a_request_that_would_pass_the_last_position_is_refused(folders):
    """The model has a row for every position up to max_positions and none beyond: the admission guard says no."""
    import paged_attention_engine_amd as pae

    engine = pae.Engine(folders["S"], dtype="float32", block_size=16, num_blocks=32, max_num_seqs=2)
    limit = M.S["max_positions"]
    assert not engine.add_request(pae.Request("long", tuple(M.tokens_for("S", limit - 3)), max_new_tokens=10))
    assert engine.add_request(pae.Request("fits", tuple(M.tokens_for("S", limit - 12)), max_new_tokens=10))


def test_the_program_replays_a_trace(folders, tmp_path):
    """bin/trace_run as a program: steps on standard input, logits in files, `done` lines."""
    tokens = M.tokens_for("Q", 37)
    want = plain_logits(folders, "Q", 37)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[20:22], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": tokens[22:], "want": [14]}], "end": ["a"]}]
    out = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["Q"], "--dtype",
                           "float32", "--out", str(out), "--max-tokens", "64"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    first = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    last = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    check(first, want[[0, 19]], "float32", "trace_run step 0")
    check(last, want[[36]], "float32", "trace_run step 2")


def test_the_command_line_generates_and_samples(folders, tmp_path):
    """`python -m paged_attention_engine_amd` on a model folder: greedy tokens of two prompts are the plain ones; with a
    temperature the same seed gives the same tokens twice and another seed gives others."""
    cfg, weights = weights_of(folders, "Q")
    prompts = [M.tokens_for("Q", 19, salt=5), M.tokens_for("Q", 7, salt=6)]
    want = [plain.greedy_generate(weights, cfg, p, 6, torch.float64)[0] for p in prompts]

    def run(*extra):
        cmd = [sys.executable, "-m", "paged_attention_engine_amd", "--model", folders["Q"], "--dtype", "float32", "--max-new-tokens", "6",
               "--num-blocks", "16", "--max-num-seqs", "2"]
        for p in prompts:
            cmd += ["--prompt-ids", ",".join(map(str, p))]
        proc = subprocess.run(cmd + list(extra), capture_output=True, text=True, timeout=600, cwd=ROOT)
        assert proc.returncode == 0, proc.stderr[-2000:]
        lines = [json.loads(line) for line in proc.stdout.splitlines() if line.startswith("{")]
        return [line["token_ids"] for line in lines]

    assert run() == want
    first = run("--temperature", "0.9", "--sample-seed", "3")
    assert first == run("--temperature", "0.9", "--sample-seed", "3")
    assert first != run("--temperature", "0.9", "--sample-seed", "4") and first != want
