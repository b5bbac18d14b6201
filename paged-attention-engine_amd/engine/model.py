"""A model built from a plan: embedding, the scheduled blocks, final norm, head.

One body serves every way of calling it, as `_run_layers` does in the reference
(engine/model.py:322-351): embedding gather (:401,448), each scheduled block,
final norm (:351), selection of the wanted rows and the head product without
bias (:406,453-455).  The reference norms every row and then selects; the norm
is row-wise, so selecting first gives the same rows.  Logits are float32 in both
precisions.  `forward_pass_count` counts traversals of the schedule, the
reference's proof that a step is one pass (:180-186,338).
"""

from __future__ import annotations

from typing import Dict, List, Mapping, Optional, Tuple

import torch

from .. import models as _models  # noqa: F401  (registers the architectures)
from ..cache.manager import CacheManager, StateSpec, bytes_of_one_page_everywhere
from ..config.model_config import ModelPlan
from ..config.registry import read_config, read_config_dict
from ..kernels import lib as K
from ..parts import OwedRows, ResidualStream, StepContext, build_block, build_part
from ..parts.base import NORMS
from ..parts.linear import Linear
from ..weights.loader import load_weights
from ..weights.random_init import RandomWeights

TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}
NAME_OF_DTYPE = {v: k for k, v in TORCH_DTYPE.items()}


def default_dtype(config) -> str:
    """The precision a model computes in when the caller names none: what its config.json says
    under `torch_dtype`, if that is one of the two the engine computes in; checkpoints stored in any
    other type (float16, say) are served in bfloat16."""
    stored = str(getattr(config, "torch_dtype", "") or "").replace("torch.", "")
    return stored if stored in TORCH_DTYPE else "bfloat16"


def plan_has_stops(plan: ModelPlan) -> bool:
    return len(plan.schedule) > 0


def _blocks_of(plan: ModelPlan, dtype, device):
    return [build_block(spec, dtype, device) for spec in plan.layers]


def expected_tensors(plan: ModelPlan) -> Dict[str, Tuple[int, ...]]:
    """Every checkpoint tensor the plan's parts declare, name -> shape."""
    out: Dict[str, Tuple[int, ...]] = {plan.embedding_name: (plan.vocab_size, plan.hidden_size)}
    for block in _blocks_of(plan, torch.float32, "meta"):
        out.update(block.tensors())
    out.update(build_part(NORMS, "norm", plan.final_norm, torch.float32, "meta").tensors(plan.final_norm_prefix))
    if plan.head_name is not None:
        out[plan.head_name] = (plan.vocab_size, plan.hidden_size)
    if plan.pair_embedding is not None:
        out[plan.pair_embedding.name] = (plan.pair_embedding.buckets + 1, plan.hidden_size)
    if plan.position_table_name is not None:
        out[plan.position_table_name] = (plan.max_positions, plan.hidden_size)
    return out


class Model:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device: str = "cuda:0") -> None:
        self.plan = plan
        self.dtype = dtype
        self.device = torch.device(device)
        self.blocks = _blocks_of(plan, dtype, self.device)
        self.final_norm = build_part(NORMS, "norm", plan.final_norm, dtype, self.device)
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[Linear] = None
        self.forward_pass_count = 0
        # for debugging a model against another implementation: called after every stop with (index,
        # stream); the stream's residual is complete there only for blocks that leave nothing pending
        self.residual_tap = None

    # ------------------------------------------------------------------ weights
    def expected_tensors(self) -> Dict[str, Tuple[int, ...]]:
        return expected_tensors(self.plan)

    def optional_tensors(self) -> Tuple[str, ...]:
        return tuple(self.plan.optional_names)

    def bind(self, weights: Mapping[str, torch.Tensor]) -> None:
        plan = self.plan
        embedding = weights[plan.embedding_name]
        self.embedding = embedding.to(device=self.device, dtype=self.dtype).contiguous()
        self.pair_table = None
        if plan.pair_embedding is not None:
            self.pair_table = weights[plan.pair_embedding.name].to(device=self.device, dtype=self.dtype).contiguous()
        self.position_table = None
        if plan.position_table_name is not None:
            self.position_table = weights[plan.position_table_name].to(device=self.device, dtype=self.dtype).contiguous()
        self._embedding_joins_again = any(entry.add_embedding for entry in plan.schedule)
        for block in self.blocks:
            block.bind(weights)
        self.final_norm.bind(plan.final_norm_prefix, weights)
        self._sum_weights = torch.ones(plan.streams, dtype=torch.float32, device=self.device)
        if self.dtype == torch.bfloat16:
            K.skinny_tickets(self.device)  # made before any step is recorded as a graph
        if plan.head_name is None:
            self.head = Linear(self.embedding)  # tied: the same buffer, no second copy
        else:
            self.head = Linear(weights[plan.head_name].to(device=self.device, dtype=self.dtype).contiguous())

    @property
    def graph_max_rows(self) -> Optional[int]:
        """Most rows a step may hold and still be recorded as a HIP graph (None: any number), as the
        parts and the head's product say."""
        limits = [block.graph_max_rows for block in self.blocks if block.graph_max_rows is not None]
        if self.head is not None and self.head.graph_max_rows is not None:
            limits.append(self.head.graph_max_rows)
        return min(limits) if limits else None

    @property
    def graph_safe(self) -> bool:
        """Can a step of this model be recorded as a HIP graph?  Every part must launch device
        work from device-side data only, for some number of rows."""
        if not (all(block.graph_safe for block in self.blocks) and self.final_norm.graph_safe):
            return False
        return self.graph_max_rows is None or self.graph_max_rows > 0

    def step_list_parts(self, block_size: int) -> Dict[object, object]:
        """key -> the first part that asks for index lists under that key (see `Part.step_lists`)."""
        out: Dict[object, object] = {}
        for block in self.blocks:
            listed = list(getattr(block, "parts", lambda: [])())
            for part in listed:  # a part made of parts (mixers side by side) names them
                listed.extend(getattr(part, "inner_parts", lambda: [])())
            for part in listed:
                key = part.step_lists_key(block_size) if hasattr(part, "step_lists_key") else None
                if key is not None and key not in out:
                    out[key] = part
        return out

    # ------------------------------------------------------------------ cache needs
    def cache_specs(self):
        """(paged, states): per schedule stop, what it keeps per token / per request."""
        paged, states = [], []
        for entry in self.plan.schedule:
            mixer = self.blocks[entry.layer].mixer
            borrowed = entry.cache_from is not None
            paged.append(None if borrowed else mixer.paged_spec())
            # a mixer that says so keeps state of its own at a stop that borrows its pages (the inputs of
            # convolutions on its queries, say)
            states.append(mixer.state_spec() if not borrowed or getattr(mixer, "state_when_borrowing", False) else None)
        if self.plan.pair_embedding is not None:
            # what the embedding keeps per request (the token before the next one) lives behind the last stop
            paged.append(None)
            states.append(StateSpec((), torch.int32, "last_token"))
        return paged, states

    @property
    def embedding_state_entry(self) -> int:
        return len(self.plan.schedule)

    def page_bytes(self, block_size: int) -> int:
        """Bytes of one page in every cache group of this model (all stops)."""
        return bytes_of_one_page_everywhere(self.cache_specs()[0], block_size, self.dtype)

    def new_cache(self, block_size: int, num_blocks, num_slots: int) -> CacheManager:
        paged, states = self.cache_specs()
        return CacheManager(paged, states, block_size, num_blocks, num_slots, self.dtype, str(self.device))

    def decode_fusable(self, ctx: StepContext) -> bool:
        """Whether this step's blocks can run as one decode program: every sequence brings one token,
        and every scheduled block, and the final norm that takes over from the last, says it launches
        recordable kernels only at this many rows."""
        rows, bs = ctx.num_tokens, ctx.cache.block_size
        if rows != ctx.num_seqs or not plan_has_stops(self.plan):
            return False
        blocks = {entry.layer for entry in self.plan.schedule}
        return (all(getattr(self.blocks[i], "decode_fusable", lambda *_: False)(rows, bs) for i in blocks)
                and getattr(self.final_norm, "folded_for", lambda _: None)(rows) is not None)

    def max_program_phases(self) -> int:
        return 8 * len(self.plan.schedule) + 8

    def _run_blocks(self, ctx: StepContext, stream: ResidualStream, first_norms, embedded=None) -> None:
        schedule = self.plan.schedule
        for index, entry in enumerate(schedule):
            ctx.entry = index
            ctx.cache_entry = index if entry.cache_from is None else entry.cache_from
            ctx.writes_cache = entry.cache_from is None
            if entry.add_embedding:
                # the embedding's output joins the stream once more before this stop (a pass over shared layers)
                if stream.pending is not None or stream.owed is not None or stream.copies != 1 or stream.prepared is not None:
                    raise ValueError(f"stop {index}: the embedding's output can only join a plain stream with nothing pending")
                K.residual_add(stream.residual, embedded)
                stream.rows = None
            stream.next_norm = first_norms[index + 1]
            after = schedule[index + 1].layer if index + 1 < len(schedule) else None
            stream.rows_wanted_next = (after is not None and getattr(self.blocks[after], "reads_stream_rows", False)
                                       and not schedule[index + 1].add_embedding)
            stream.prepared_wanted_next = (after is not None and getattr(self.blocks[after], "takes_prepared_norm", False)
                                           and not schedule[index + 1].add_embedding)
            self.blocks[entry.layer].forward(ctx, stream)
            if self.residual_tap is not None:
                self.residual_tap(index, stream)

    # ------------------------------------------------------------------ forward
    def forward(self, ctx: StepContext, token_ids: torch.Tensor, logit_rows: torch.Tensor) -> torch.Tensor:
        """Run `token_ids` (int32 [T]) through the schedule once; float32 logits
        [len(logit_rows), vocab] at the flat rows `logit_rows` (int32)."""
        self.forward_pass_count += 1
        plan = self.plan
        T, H = ctx.num_tokens, plan.hidden_size
        copies = plan.streams
        residual = torch.empty((T, H), dtype=torch.float32, device=self.device)
        stream = ResidualStream(residual)
        if copies > 1:
            # the stream is kept in several copies, all equal to the embedding's output at the start
            stream = ResidualStream(torch.empty((T, copies * H), dtype=torch.float32, device=self.device))
            stream.copies = copies
        stream.sum_weights = self._sum_weights
        ctx.token_ids = token_ids
        # the norm that reads the stream first at every stop (and the final norm after the last)
        first_norms = [getattr(self.blocks[entry.layer], "mixer_norm", None) for entry in plan.schedule] + [self.final_norm]
        entry_fold = getattr(self.blocks[plan.schedule[0].layer], "entry_fold", None) if plan.schedule and T else None
        own_kernel = plan.pair_embedding is not None or self.position_table is not None
        fold = entry_fold(T) if entry_fold is not None and not own_kernel else None
        if self.position_table is not None:
            if plan.pair_embedding is not None or copies > 1:
                raise ValueError("a table of learned positions goes with a plain embedding and one copy of the stream")
            if ctx.q_lens and max(p + n for p, n in zip(ctx.past_lens, ctx.q_lens)) > plan.max_positions:
                raise ValueError(f"a sequence passes the {plan.max_positions} positions the model has rows for")
            K.embedding_positions(residual, self.embedding, token_ids, self.position_table, ctx.positions, plan.embedding_scale)
        elif fold is not None:
            # the first block's norm lets the embedding prepare its rows (see parts.OwedRows)
            norm, weight, eps = fold
            rows = torch.empty((T, H), dtype=torch.bfloat16, device=self.device)
            stats = torch.empty((T, K.stat_tiles(H)), dtype=torch.float32, device=self.device)
            K.embedding_rows(residual, self.embedding, token_ids, plan.embedding_scale, rows, weight, stats)
            stream.owed, stream.owed_to = OwedRows(rows, stats, eps), norm
        elif plan.pair_embedding is not None:
            pairs = plan.pair_embedding
            K.embedding_pairs(residual, self.embedding, self.pair_table, token_ids, ctx.positions, ctx.tok_seq, ctx.slots,
                              ctx.cache.state_of(self.embedding_state_entry), plan.embedding_scale, pairs.buckets,
                              pairs.mul_prev, pairs.mul_cur)
            if copies > 1:
                K.hyper_spread(stream.residual, residual, copies)
        else:
            K.embedding(residual, self.embedding, token_ids, plan.embedding_scale)
            if copies > 1:
                K.hyper_spread(stream.residual, residual, copies)
        embedded = None
        if self._embedding_joins_again:
            if copies > 1:
                raise ValueError("the embedding's output joins a plain stream, not one kept in copies")
            embedded = residual.clone()  # the stream as it was before the first stop
        program = ctx.program if fold is not None and self.decode_fusable(ctx) else None
        if program is not None:
            # every block's kernels become phases of one resident kernel, which runs when all are recorded
            with K.recording(program):
                self._run_blocks(ctx, stream, first_norms, embedded)
            program.launch()
        else:
            self._run_blocks(ctx, stream, first_norms, embedded)
        rows = logit_rows.numel()
        if rows == 0:
            return torch.empty((0, plan.vocab_size), dtype=torch.float32, device=self.device)
        last = self.final_norm.forward(stream, logit_rows)
        logits = self.head.float32(last)
        if plan.logit_scale != 1.0 or plan.logit_softcap:
            K.logits_finish(logits, plan.logit_scale, plan.logit_softcap or 0.0)
        return logits


def load_model(model_dir: str, dtype: Optional[str] = None, device: str = "cuda:0") -> Model:
    """The model of a folder with config.json and safetensors weights; the class
    of model is chosen by config.json's `architectures`, and so is the precision if `dtype` is None
    (`default_dtype`)."""
    config = read_config(model_dir)
    if dtype is None:
        dtype = default_dtype(config)
    if dtype not in TORCH_DTYPE:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    model = Model(config.plan(), TORCH_DTYPE[dtype], device)
    model.config = config
    weights = load_weights(model_dir, model.expected_tensors(), model.optional_tensors())
    model.bind(weights)
    return model


def random_model(config, seed: int = 0, dtype: Optional[str] = None, device: str = "cuda:0", std: float = 0.02,
                 norm_std: float = 0.0) -> Model:
    """A model of `config` (a config.json dict, or a registered architecture's typed config) with
    random weights drawn on the device, tensor by tensor as the parts bind them: nothing is written
    to disk and no tensor exists twice, so the 72B shape's 145 GB fit one GPU.  The reference draws
    random weights only for its tiny test model (tests/tiny_model.py:21-50)."""
    if isinstance(config, Mapping):
        config = read_config_dict(config)
    if dtype is None:
        dtype = default_dtype(config)
    if dtype not in TORCH_DTYPE:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    model = Model(config.plan(), TORCH_DTYPE[dtype], device)
    model.config = config
    model.bind(RandomWeights(model.expected_tensors(), seed, std, norm_std, device))
    return model
